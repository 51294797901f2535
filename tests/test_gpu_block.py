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


def ref_mem_block_forward(blk, h, mem, src, dst, etype, isrc, idst):
    """modules/attention.py:116-172 in float64 on the CPU (attention by gather / index_add, no padding needed)."""
    from oracle import torch_ops
    heads = lambda proj, x: proj(x).view(-1, blk.h, blk.d_k)
    ak = blk.embed_ak(etype) if blk.rel_pos else None
    a = torch_ops.attention(src, dst, heads(blk.proj_q[0], h), heads(blk.proj_k[0], h), heads(blk.proj_v[0], h), ak)
    h = blk.norm_in[0](h + blk.proj_o[0](a.reshape(-1, blk.h * blk.d_k)))
    a = torch_ops.attention(isrc, idst, heads(blk.proj_q[1], h), heads(blk.proj_k[1], mem), heads(blk.proj_v[1], mem))
    h = blk.norm_in[1](h + blk.proj_o[1](a.reshape(-1, blk.h * blk.d_k)))
    return blk.norm_inter(h + blk.ffn(h))


MEM_LONGER = ((40, 70, 25), (30, 20, 45))      # memory longer than the decoder side: the case the reference runs
DEC_LONGER = ((20, 15), (60, 33))              # decoder side longer: the reference's square form cannot express it (attention.py:148-149)


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("form,lengths", [("square", MEM_LONGER), ("bipartite", MEM_LONGER), ("bipartite", DEC_LONGER)])
def test_mem_block_matches_cpu_restatement(form, fused, lengths):
    """BPTMemBlock (self-attention + attention to memory over the inter graph of graph/mt.py:286-321 + FFN) against
    the float64 restatement, all parameter gradients included; the attention to memory has n_q != n_k rows."""
    from bpt_amd import graphbuilder as gb
    from bpt_amd.block import BPTMemBlock
    enc_len, dec_len = lengths
    enc = [gb.BinaryPartition(L, False, 2, 10) for L in enc_len]
    dec = [gb.BinaryPartition(L, True, 2, 10) for L in dec_len]
    src, dst, etype, _, n_dec = gb.merge_graphs(dec)
    n_enc = sum(g.number_of_nodes for g in enc)
    isrc, idst, ne, nd = gb.inter_graph_edges(enc, dec)
    assert (ne, nd) == (n_enc, n_dec) and n_enc != n_dec
    to_dev = lambda csr: tuple(tuple(t.to(DEV) for t in c) if isinstance(c, (tuple, list)) else c.to(DEV) for c in csr)
    csr = to_dev(gb.get_csrs(src, dst, n_dec))
    csr_inter = to_dev(gb.get_csrs(isrc, idst, max(n_enc, n_dec)) if form == "square" else gb.get_csrs_bipartite(isrc, idst, n_enc, n_dec))
    torch.manual_seed(5)
    blk = BPTMemBlock(512, 8, 256, rel_pos=True, drop_h=0.0, drop_a=0.0, fused=fused)
    blk.reset_parameters()
    ref = copy.deepcopy(blk).double()
    blk = blk.to(DEV)
    h0 = torch.randn(n_dec, 512, generator=torch.Generator().manual_seed(1))
    mem0 = torch.randn(n_enc, 512, generator=torch.Generator().manual_seed(2))
    gout = torch.randn(n_dec, 512, generator=torch.Generator().manual_seed(3))
    et = torch.from_numpy(etype.astype(np.int64))

    h_dev, mem_dev = h0.to(DEV).requires_grad_(True), mem0.to(DEV).requires_grad_(True)
    out = blk(h_dev, csr, mem_dev, csr_inter, et.to(DEV))
    assert out.shape == (n_dec, 512)
    out.backward(gout.to(DEV))

    h_ref, mem_ref = h0.double().requires_grad_(True), mem0.double().requires_grad_(True)
    t = torch.from_numpy
    out_ref = ref_mem_block_forward(ref, h_ref, mem_ref, t(src), t(dst), et, t(isrc), t(idst))
    out_ref.backward(gout.double())

    def close(a, b, what, rtol=2e-4, atol=2e-5):
        a = a.detach().cpu().double().numpy(); b = b.detach().numpy()
        err = np.abs(a - b); bound = atol + rtol * np.abs(b)
        assert np.all(err <= bound), f"{what}: max err {err.max():.3e}, worst excess {(err - bound).max():.3e}"

    close(out, out_ref, "block output")
    close(h_dev.grad, h_ref.grad, "d input", rtol=1e-3, atol=1e-4)
    close(mem_dev.grad, mem_ref.grad, "d memory", rtol=1e-3, atol=1e-4)
    for (name, p), (_, pr) in zip(blk.named_parameters(), ref.named_parameters()):
        close(p.grad, pr.grad, f"d {name}", rtol=1e-3, atol=1e-4)


def test_mem_block_loads_reference_state_dict_names():
    from bpt_amd.block import BPTMemBlock
    names = set(BPTMemBlock(64, 2, 32, rel_pos=True).state_dict().keys())
    # parameter names of modules/attention.py:86-110
    want = {"norm_inter.weight", "norm_inter.bias", "embed_ak.weight", "ffn.0.w_1.weight", "ffn.0.w_1.bias", "ffn.0.w_2.weight",
            "ffn.0.w_2.bias"}
    for i in (0, 1):
        want |= {f"norm_in.{i}.weight", f"norm_in.{i}.bias", f"proj_q.{i}.weight", f"proj_k.{i}.weight", f"proj_v.{i}.weight",
                 f"proj_o.{i}.weight"}
    assert names == want


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_q,n_k", [(900, 2100), (2100, 900)])
def test_fused_attention_with_different_row_counts_on_the_two_sides(dtype, n_q, n_k):
    """Fused kernels on a bipartite graph whose query side and key side have different node counts (large enough for
    the row-group kernels), against the float64 gather / index_add restatement."""
    import oracle  # noqa: F401
    from oracle import torch_ops
    from bpt_amd import graphbuilder as gb
    from bpt_amd import graphop, op
    rng = np.random.default_rng(3)
    deg = rng.integers(0, 40, n_q)
    idst = np.repeat(np.arange(n_q), deg).astype(np.int64)
    start = rng.integers(0, n_k - 64, n_q)
    isrc = (np.repeat(start, deg) + rng.integers(0, 64, len(idst))).astype(np.int64)          # neighbours in a window: rows share them
    csr = gb.get_csrs_bipartite(isrc, idst, n_k, n_q)
    out_csr, in_csr, ROW, IR, COL, IC = csr
    args = tuple(x.to(DEV) for x in (ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1]))
    gen = torch.Generator().manual_seed(9)
    q, do = ((torch.randn(n_q, 8, 64, generator=gen) / 8).to(dtype) for _ in range(2))
    k, v = ((torch.randn(n_k, 8, 64, generator=gen) / 8).to(dtype) for _ in range(2))
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    old = graphop.set_group_rows(8)
    try:
        o = op.bpt_attention(*args, qd, kd, vd, fused=True)
        o.backward(do.to(DEV))
    finally:
        graphop.set_group_rows(old)
    t64 = lambda x: x.detach().cpu().double()
    ro, rdq, rdk, rdv = torch_ops.attention_fwd_bwd(torch.from_numpy(isrc), torch.from_numpy(idst), t64(q), t64(k), t64(v), t64(do))
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    gtol = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    for got, want, tl, nm in ((o, ro, tol, "o"), (qd.grad, rdq, gtol, "dq"), (kd.grad, rdk, gtol, "dk"), (vd.grad, rdv, gtol, "dv")):
        err = (t64(got) - want).abs().numpy(); bound = tl["atol"] + tl["rtol"] * want.abs().numpy()
        assert got.shape == want.shape and np.all(err <= bound), f"{nm}: max err {err.max():.3e}"
