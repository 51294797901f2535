"""The transformer block (bpt_amd/block.py, reference modules/attention.py:22-81) on the GPU against a float64
CPU restatement built from torch modules and the oracle's attention (oracle/torch_ops.py)."""
import copy

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def ref_block_forward(blk, h, src, dst, etype):
    """modules/attention.py:54-81 in float64 on the CPU, attention by gather / index_add."""
    from oracle import torch_ops
    q = blk.proj_q(h).view(-1, blk.h, blk.d_k)
    k = blk.proj_k(h).view(-1, blk.h, blk.d_k)
    v = blk.proj_v(h).view(-1, blk.h, blk.d_k)
    ak = blk.embed_ak(etype) if blk.rel_pos else None
    a = torch_ops.attention(src, dst, q, k, v, ak).reshape(-1, blk.h * blk.d_k)
    h = blk.norm_in(h + blk.proj_o(a))
    return blk.norm_inter(h + blk.ffn(h))


@pytest.mark.parametrize("rel_pos", [False, True])
@pytest.mark.parametrize("dims", [(512, 8, 256), (96, 3, 64)])       # (dim_model, heads, dim_ff): fused shape / generic shape
def test_block_matches_cpu_restatement(rel_pos, dims):
    from bpt_amd import graphbuilder as gb
    from bpt_amd.block import BPTBlock
    dim_model, heads, dim_ff = dims
    g = gb.BinaryPartition(300, True, 2, 10)
    src, dst, etype = g.get_edges()
    n = g.number_of_nodes
    csr = gb.get_csrs(src, dst, n)                         # torch int64 tensors, the reference's 6-tuple
    csr_dev = tuple(tuple(t.to(DEV) for t in c) if isinstance(c, (tuple, list)) else c.to(DEV) for c in csr)
    torch.manual_seed(7)
    blk = BPTBlock(dim_model, heads, dim_ff, rel_pos=rel_pos, drop_h=0.0, drop_a=0.0)
    blk.reset_parameters()
    ref = copy.deepcopy(blk).double()
    blk = blk.to(DEV)
    h0 = torch.randn(n, dim_model, generator=torch.Generator().manual_seed(1))
    gout = torch.randn(n, dim_model, generator=torch.Generator().manual_seed(2))
    et = torch.from_numpy(etype.astype(np.int64))

    h_dev = h0.to(DEV).requires_grad_(True)
    out = blk(h_dev, csr_dev, et.to(DEV) if rel_pos else None)
    out.backward(gout.to(DEV))

    h_ref = h0.double().requires_grad_(True)
    out_ref = ref_block_forward(ref, h_ref, torch.from_numpy(src), torch.from_numpy(dst), et)
    out_ref.backward(gout.double())

    def close(a, b, what, rtol=2e-4, atol=2e-5):
        a = a.detach().cpu().double().numpy(); b = b.detach().numpy()
        err = np.abs(a - b); bound = atol + rtol * np.abs(b)
        assert np.all(err <= bound), f"{what}: max err {err.max():.3e}, worst excess {(err - bound).max():.3e}"

    close(out, out_ref, "block output")
    close(h_dev.grad, h_ref.grad, "d input", rtol=1e-3, atol=1e-4)
    for (name, p), (_, pr) in zip(blk.named_parameters(), ref.named_parameters()):
        close(p.grad, pr.grad, f"d {name}", rtol=1e-3, atol=1e-4)


def test_block_loads_reference_state_dict_names():
    from bpt_amd.block import BPTBlock
    names = set(BPTBlock(64, 2, 32, rel_pos=True).state_dict().keys())
    # parameter names of modules/attention.py:24-47
    assert names == {"norm_in.weight", "norm_in.bias", "norm_inter.weight", "norm_inter.bias", "proj_q.weight",
                     "proj_k.weight", "proj_v.weight", "proj_o.weight", "embed_ak.weight", "ffn.0.w_1.weight",
                     "ffn.0.w_1.bias", "ffn.0.w_2.weight", "ffn.0.w_2.bias"}
