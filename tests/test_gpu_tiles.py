"""The dense-tile kernels of the fused attention (groups of 16 rows, one wavefront per head, every block of 16 entries a
16 x 16 matrix-core product with the missing pairs masked) against the float64 CPU oracle, forward and backward, with
the stated float32 tolerances as they stand (outputs rtol 1e-5 / atol 1e-5, gradients rtol 1e-4 / atol 1e-5).

The library picks tiles by graph size and density; here they are forced (graphop.TILE_BACKWARD, _MIN_GROUP_ITEMS) so that
small graphs with the awkward cases run through them: parallel edges, rows without edges, rows longer than a work item
on both sides (partial rows + combine), entry lists longer than one staged piece, different node counts on the two
sides, every compiled head count, both walks (with and without read-ahead)."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = dict(rtol=1e-5, atol=1e-5)
GTOL = dict(rtol=1e-4, atol=1e-5)


def f64(t):
    return t.detach().cpu().to(torch.float64)


def check(got, want, tol, what):
    err = (f64(got) - want).abs().numpy()
    bound = tol["atol"] + tol["rtol"] * want.abs().numpy()
    assert got.shape == want.shape and np.all(err <= bound), f"{what}: max err {err.max():.3e}, worst excess {(err - bound).max():.3e}"


class forced_tiles:
    """Tiles for every graph size, forward and backward, work items of `seg` edges."""
    def __init__(self, seg=None):
        self.seg = seg

    def __enter__(self):
        from bpt_amd import graphop, plan
        self.old = (graphop._MIN_GROUP_ITEMS, graphop.TILE_BACKWARD, graphop.TILE_SEG_LEN)
        graphop._MIN_GROUP_ITEMS, graphop.TILE_BACKWARD, graphop.TILE_SEG_LEN = 0, True, self.seg
        plan.plan_cache.clear()

    def __exit__(self, *exc):
        from bpt_amd import graphop, plan
        graphop._MIN_GROUP_ITEMS, graphop.TILE_BACKWARD, graphop.TILE_SEG_LEN = self.old
        plan.plan_cache.clear()


def graphs(name):
    from bpt_amd import graphbuilder as gb
    rng = np.random.default_rng(5)
    if name == "multigraph":                       # parallel edges, a node without edges, rows of 500+ edges on both sides
        n, E = 97, 3000
        src = rng.integers(0, n, E); dst = rng.integers(0, n, E)
        dst[: E // 3] = 1; src[E // 3: E // 2] = 2
        src[src == 0] = 3; dst[dst == 0] = 3
        src[-1], dst[-1] = src[-2], dst[-2]
        return src.astype(np.int64), dst.astype(np.int64), n, n
    if name == "bipartite":                        # 700 query nodes, 1500 key nodes, neighbours in windows
        n_q, n_k = 700, 1500
        deg = rng.integers(0, 40, n_q)
        dst = np.repeat(np.arange(n_q), deg)
        src = np.repeat(rng.integers(0, n_k - 64, n_q), deg) + rng.integers(0, 64, len(dst))
        return src.astype(np.int64), dst.astype(np.int64), n_k, n_q
    g = {"bpt512_k4": lambda: gb.BinaryPartition(512, False, 4, 10),            # non-causal: duplicate edges, a row of 512
         "bpt2048_causal": lambda: gb.BinaryPartition(2048, True, 4, 10),         # partial rows on both sides
         "bpt256_k24": lambda: gb.BinaryPartition(256, False, 24, 10),            # rows of 100-300 edges
         "window100": lambda: gb.FullyConnected(260, False, 100),                 # dense band, tall tiles (read-ahead walk)
         "window128_causal": lambda: gb.FullyConnected(700, True, 128)}[name]()
    src, dst, _ = g.get_edges()
    return src, dst, g.number_of_nodes, g.number_of_nodes


CASES = [("multigraph", 64), ("bipartite", None), ("bpt512_k4", None), ("bpt2048_causal", 64), ("bpt2048_causal", 256),
         ("bpt256_k24", 128), ("window100", 256), ("window128_causal", None)]
OTHER_HEADS = [("multigraph", 64), ("bpt2048_causal", 64), ("window100", 256)]          # 4 and 16 heads on three of the graphs


@pytest.mark.parametrize("gname,seg,heads", [(g, s, 8) for g, s in CASES] + [(g, s, h) for h in (4, 16) for g, s in OTHER_HEADS])
def test_tile_kernels_match_the_oracle(gname, seg, heads):
    from oracle import torch_ops
    from bpt_amd import graphbuilder as gb
    from bpt_amd import op, graphop
    src, dst, n_k, n_q = graphs(gname)
    csr = gb.get_csrs_bipartite(src, dst, n_k, n_q)
    out_csr, in_csr, ROW, IR, COL, IC = csr
    args = tuple(x.to(DEV) for x in (ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1]))
    gen = torch.Generator().manual_seed(17)
    q, do = (torch.randn(n_q, heads, 64, generator=gen) / 8 for _ in range(2))
    k, v = (torch.randn(n_k, heads, 64, generator=gen) / 8 for _ in range(2))
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    with forced_tiles(seg):
        o = op.bpt_attention(*args, qd, kd, vd, fused=True)
        o.backward(do.to(DEV))
        o2 = op.bpt_attention(*args, qd.detach(), kd.detach(), vd.detach(), fused=True)
        # the forward really ran on tiles: the plan it used carries groups of 16 rows
        from bpt_amd.plan import plan_cache
        tiled = [p for p, _ in plan_cache._d.values() if any(key[0] == 16 for key in p._groups)]
        assert tiled, "no plan with groups of 16 rows: the tile kernels did not run"
    assert torch.equal(o.detach(), o2)                                            # run-to-run bit identical
    ro, rdq, rdk, rdv = torch_ops.attention_fwd_bwd(torch.from_numpy(src), torch.from_numpy(dst), f64(q), f64(k), f64(v), f64(do))
    check(o, ro, TOL, "o")
    check(qd.grad, rdq, GTOL, "dq"); check(kd.grad, rdk, GTOL, "dk"); check(vd.grad, rdv, GTOL, "dv")
    if gname == "multigraph":
        assert not o[0].any() and not qd.grad[0].any()                            # the node without edges


BF16_TOL = dict(rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("gname,seg,heads", [(g, s, 8) for g, s in CASES] + [(g, s, 16) for g, s in OTHER_HEADS])
def test_tile_kernels_in_bfloat16_match_the_oracle(gname, seg, heads):
    """bfloat16 rows on the tile kernels (operands as loaded on the bfloat16 matrix instructions, float32 accumulation,
    (p, ds) handed from the destination to the source side as bfloat16 pairs): rtol 2e-2 / atol 2e-2 against the float64
    oracle on the same (bfloat16-rounded) inputs; 8 heads and 16 (the two sizes the fused bfloat16 path is compiled for)."""
    from oracle import torch_ops
    from bpt_amd import graphbuilder as gb
    from bpt_amd import op
    src, dst, n_k, n_q = graphs(gname)
    csr = gb.get_csrs_bipartite(src, dst, n_k, n_q)
    out_csr, in_csr, ROW, IR, COL, IC = csr
    args = tuple(x.to(DEV) for x in (ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1]))
    gen = torch.Generator().manual_seed(19)
    q, do = (torch.randn(n_q, heads, 64, generator=gen).to(torch.bfloat16) for _ in range(2))
    k, v = (torch.randn(n_k, heads, 64, generator=gen).to(torch.bfloat16) for _ in range(2))
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    with forced_tiles(seg):
        o = op.bpt_attention(*args, qd, kd, vd, fused=True)
        o.backward(do.to(DEV))
        o2 = op.bpt_attention(*args, qd.detach(), kd.detach(), vd.detach(), fused=True)
        from bpt_amd.plan import plan_cache
        assert [p for p, _ in plan_cache._d.values() if any(key[0] == 16 for key in p._groups)], "the tile kernels did not run"
    assert o.dtype == torch.bfloat16 and torch.equal(o.detach(), o2)
    ro, rdq, rdk, rdv = torch_ops.attention_fwd_bwd(torch.from_numpy(src), torch.from_numpy(dst), f64(q), f64(k), f64(v), f64(do))
    check(o, ro, BF16_TOL, "o")
    check(qd.grad, rdq, BF16_TOL, "dq"); check(kd.grad, rdk, BF16_TOL, "dk"); check(vd.grad, rdv, BF16_TOL, "dv")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gname,seg", [("multigraph", 64), ("bpt2048_causal", 64), ("window100", 256)])
def test_tile_kernels_with_dropout_and_score_term(gname, seg, dtype):
    """The DROP / BIAS variants of the tile kernels (forward and destination-side backward read the edge id of every pair):
    dropout 0.25 with the mask attention_dropout_mask reproduces, and a rel_pos table of 23 types, together, against the
    float64 oracle given the same mask; float32 rtol 1e-5 / atol 1e-5 (gradients rtol 1e-4), bfloat16 rtol 2e-2 / atol 2e-2."""
    from oracle import torch_ops
    from bpt_amd import graphbuilder as gb
    from bpt_amd import op, graphop
    src, dst, n_k, n_q = graphs(gname)
    csr = gb.get_csrs_bipartite(src, dst, n_k, n_q)
    out_csr, in_csr, ROW, IR, COL, IC = csr
    args = tuple(x.to(DEV) for x in (ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1]))
    h, n_types, p, seed = 8, 23, 0.25, 424242
    gen = torch.Generator().manual_seed(23)
    q, do = ((torch.randn(n_q, h, 64, generator=gen) / 8).to(dtype) for _ in range(2))
    k, v = ((torch.randn(n_k, h, 64, generator=gen) / 8).to(dtype) for _ in range(2))
    table = (torch.randn(n_types, 64, generator=gen) / 8).to(dtype)
    etype = torch.from_numpy(np.random.default_rng(24).integers(0, n_types, len(src))).to(DEV)
    qd, kd, vd, td = (x.to(DEV).requires_grad_(True) for x in (q, k, v, table))
    with forced_tiles(seg):
        mask = graphop.attention_dropout_mask(*args[4:], qd, kd, p, seed)
        o = op.bpt_attention(*args, qd, kd, vd, fused=True, dropout_p=p, seed=seed, rel_table=td, etype=etype)
        o.backward(do.to(DEV))
        from bpt_amd.plan import plan_cache
        assert [pl for pl, _ in plan_cache._d.values() if any(key[0] == 16 for key in pl._groups)], "the tile kernels did not run"
    et = etype.cpu()
    ro, rdq, rdk, rdv, rdak = torch_ops.attention_fwd_bwd(torch.from_numpy(src), torch.from_numpy(dst), f64(q), f64(k), f64(v), f64(do),
                                                          ak=f64(table)[et], drop=mask.double())
    rdt = torch.zeros(n_types, 64, dtype=torch.float64).index_add_(0, et, rdak)
    tol, gtol = (TOL, GTOL) if dtype == torch.float32 else (BF16_TOL, BF16_TOL)
    check(o, ro, tol, "o")
    check(qd.grad, rdq, gtol, "dq"); check(kd.grad, rdk, gtol, "dk"); check(vd.grad, rdv, gtol, "dv")
    # a table row is a raw sum over all edges of its type and all heads (h * E / n_types products): atol grows with
    # its length as in tests/test_gpu_parity.py::close
    terms = h * len(src) / n_types
    err = (f64(td.grad) - rdt).abs().numpy()
    assert np.all(err <= gtol["atol"] * max(1.0, terms / 64.0) + gtol["rtol"] * rdt.abs().numpy()), err.max()


def test_tiles_agree_with_the_row_group_kernels_on_the_headline_graph():
    """L = 8192, k = 4, causal, 8 x 64: tile forward + tile backward against the row-group kernels (themselves checked
    against the oracle in test_headline_graph_full_parity) and against the oracle's forward."""
    from bpt_amd import graphbuilder as gb
    from bpt_amd import graphop
    g = gb.BinaryPartition(8192, True, 4, 10)
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    csr = gb.get_csrs(src, dst, n, as_torch=False)
    out_csr, in_csr, ROW, IR, COL, IC = csr
    t = lambda a: torch.from_numpy(a).to(DEV)
    args = (t(ROW), t(IR), t(out_csr[2]), t(out_csr[1]), t(COL), t(IC), t(in_csr[2]), t(in_csr[1]))
    gen = torch.Generator().manual_seed(2345)
    q, k, v, do = ((torch.randn(n, 8, 64, generator=gen) / 8).to(DEV) for _ in range(4))

    def step():
        o, lse = graphop.attention_forward(*args[4:], q, k, v)
        return (o,) + tuple(graphop.attention_backward(*args, q, k, v, o, lse, do))

    old = graphop.set_tiles(False)
    try:
        ref = step()
    finally:
        graphop.set_tiles(old)
    with forced_tiles():
        got = step()
    ro, _ = oracle.attention_forward(csr, f64(q).numpy(), f64(k).numpy(), f64(v).numpy())
    check(got[0], torch.from_numpy(ro), TOL, "o")
    for a, b, nm in zip(got, ref, ("o", "dq", "dk", "dv")):
        check(a, f64(b), GTOL if nm != "o" else TOL, nm + " (tiles against row groups)")
