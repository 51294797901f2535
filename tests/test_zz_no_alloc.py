"""bpt_attention_forward_noalloc (the entry point that allocates nothing: its workspace is a static device array
inside libbptattn) against bpt_attention_forward, both called through the C ABI with the same plan and tensors.

Two calls in a row, the second on a smaller graph, so that the second call finds the first one's partial rows in
the shared array; outputs must be bit-identical to the allocating entry point's (same kernels, same order of
sums), and within the stated float32 tolerance of the CPU oracle."""
import ctypes

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _graph(L, step):
    from bpt_amd import graphbuilder as gb
    g = gb.BinaryPartition(L, True, step, 10)
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    csr = gb.get_csrs(src, dst, n, as_torch=False)
    _, in_csr, _, _, COL, IC = csr
    args = tuple(torch.from_numpy(a).to(DEV) for a in (COL, IC, in_csr[2], in_csr[1]))
    return n, csr, args


def _both_entries(n, args, h, d, dtype, seed):
    """(o, lse) of the allocating entry point and of the allocation-free one, same plan, same inputs."""
    from bpt_amd import graphop
    from bpt_amd._lib import attn_lib
    from bpt_amd.plan import plan_cache
    lib = attn_lib()
    gen = torch.Generator().manual_seed(seed)
    q, k, v = ((torch.randn(n, h, d, generator=gen) / 8).to(dtype).to(DEV) for _ in range(3))
    plan = plan_cache.get(*args, n, n)
    if graphop._attention_groups(plan, 0.0, None, q, k):
        ref = ctypes.byref(plan.ensure_groups(graphop._forward_rows(q, h, d, plan))["struct"])
    else:
        ref = plan.ref
    dt = graphop._dtype(q)
    need = lib.bpt_workspace_bytes(graphop.OP_ATTN_FWD, ref, None, h, d, dt)
    assert 0 < need <= 16 * 1024 * 1024, "the case must use the scratch and fit it"
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    scale = 1.0 / 8.0
    o0, lse0 = torch.empty_like(q), torch.empty(n, h, dtype=torch.float32, device=DEV)
    st = lib.bpt_attention_forward(ref, p(q), p(k), p(v), None, p(o0), p(lse0), p(ws), need, scale, 0.0, 0, h, d, dt, stream)
    assert st == 0, st
    # poison the outputs of the second entry so that an entry that does nothing cannot pass
    o1, lse1 = torch.full_like(q, float("nan")), torch.full((n, h), float("nan"), dtype=torch.float32, device=DEV)
    st = lib.bpt_attention_forward_noalloc(ref, p(q), p(k), p(v), None, p(o1), p(lse1), scale, 0.0, 0, h, d, dt, stream)
    assert st == 0, st
    torch.cuda.synchronize()
    return (q, k, v), (o0, lse0), (o1, lse1)


def test_noalloc_forward_equals_the_allocating_entry_on_two_calls_in_a_row():
    # first call: L = 2048 (row groups, matrix-core kernel, 500+ partial rows); second, smaller: L = 300 (one wavefront per row)
    for L, step, seed in ((2048, 4, 11), (300, 2, 12)):
        n, csr, args = _graph(L, step)
        (q, k, v), (o0, lse0), (o1, lse1) = _both_entries(n, args, 8, 64, torch.float32, seed)
        assert torch.equal(o0, o1), f"L={L}: o differs"
        assert torch.equal(lse0, lse1), f"L={L}: lse differs"
        f64 = lambda t: t.detach().cpu().double().numpy()
        want, _ = oracle.attention_forward(csr, f64(q), f64(k), f64(v))
        assert np.allclose(f64(o1), want, rtol=1e-5, atol=1e-5), f"L={L}: o against the oracle"


def test_noalloc_forward_bf16_and_a_plan_that_does_not_fit():
    n, csr, args = _graph(1024, 4)
    _, (o0, lse0), (o1, lse1) = _both_entries(n, args, 8, 64, torch.bfloat16, 13)
    assert torch.equal(o0, o1) and torch.equal(lse0, lse1)
    # a plan whose partial rows need more than the static array is refused before anything is launched
    from bpt_amd._lib import PlanStruct, attn_lib
    big = PlanStruct(None, None, None, None, None, 0, 0, 0, 0, 10 ** 6)
    assert attn_lib().bpt_attention_forward_noalloc(ctypes.byref(big), None, None, None, None, None, None, 0.125, 0.0, 0, 8, 64, 0, None) == -8
