"""GPU parity: every op of the HIP library against the CPU oracle on the same seeded inputs.

Tolerances (stated by the task): fp32 outputs rtol 1e-5 / atol 1e-5, fp32 gradients rtol 1e-4,
bf16 rtol 2e-2; fp64 (generic kernels only) 1e-12.  The oracle runs in float64 on the float32 /
bf16 input values, so the comparison measures the kernel's own rounding.  Index tensors are
bit-exact by construction (tests/test_graphbuilder.py).
"""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from bpt_amd import graphop, op
    return graphop, op


# --------------------------------------------------------------------------------------------
# graphs
# --------------------------------------------------------------------------------------------
def block_graph(batch, l):
    x = np.repeat(np.arange(batch * l), l)
    y = (np.arange(batch * l * l) % l) + (np.arange(batch * l * l) // (l * l)) * l
    return x.astype(np.int64), y.astype(np.int64), batch * l


def bpt_graph(L, triu, step):
    from bpt_amd import graphbuilder as gb
    g = gb.BinaryPartition(L, triu, step, 10)
    src, dst, _ = g.get_edges()
    return src, dst, g.number_of_nodes


def fc_graph(L, window):
    from bpt_amd import graphbuilder as gb
    g = gb.FullyConnected(L, False, window)
    src, dst, _ = g.get_edges()
    return src, dst, g.number_of_nodes


def random_multigraph(n, E, seed=1):
    rng = np.random.default_rng(seed)
    src = rng.integers(0, n, E); dst = rng.integers(0, n, E)
    dst[: E // 3] = 1; src[E // 3: E // 2] = 2
    src[src == 0] = 3; dst[dst == 0] = 3
    src[-1], dst[-1] = src[-2], dst[-2]
    return src.astype(np.int64), dst.astype(np.int64), n


GRAPHS = {
    "blocks8x30": lambda: block_graph(8, 30),
    "bpt512_k4": lambda: bpt_graph(512, False, 4),          # benchmark configuration 1 (non-causal: duplicate edges, deg 512 row)
    "bpt300_causal_k2": lambda: bpt_graph(300, True, 2),
    "multigraph": lambda: random_multigraph(97, 3000),      # zero-degree node, heavy rows both sides, duplicates
    "fc_w100": lambda: fc_graph(260, 100),                  # every row longer than 64 edges
    "bpt256_k24": lambda: bpt_graph(256, False, 24),        # rows of 100-300 edges
}
LONG_ITEMS = {"fc_w100": 256, "bpt256_k24": 128}            # run these with work items of that many edges


class long_items:
    """Plans built inside the block cut rows into segments of LONG_ITEMS[gname] edges (the length large graphs
    with long rows get automatically) instead of 64."""
    def __init__(self, gname):
        self.seg = LONG_ITEMS.get(gname)

    def __enter__(self):
        from bpt_amd import plan
        if self.seg:
            plan.plan_cache.clear()
            plan.FORCE_SEG_LEN = self.seg

    def __exit__(self, *exc):
        from bpt_amd import plan
        if self.seg:
            plan.FORCE_SEG_LEN = None
            plan.plan_cache.clear()


class Case:
    def __init__(self, name, chunk=32):
        from bpt_amd import graphbuilder as gb
        self.src, self.dst, self.n = GRAPHS[name]()
        self.E = len(self.src)
        self.csr = gb.get_csrs(self.src, self.dst, self.n, chunk_size=chunk, as_torch=False)
        out_csr, in_csr, ROW, IR, COL, IC = self.csr
        t = lambda a: torch.from_numpy(a).to(DEV)
        # argument tuples in the reference's order
        self.out = (t(ROW), t(IR), t(out_csr[2]), t(out_csr[1]))
        self.inn = (t(COL), t(IC), t(in_csr[2]), t(in_csr[1]))
        self.np_out = (ROW, IR, out_csr[2], out_csr[1])
        self.np_in = (COL, IC, in_csr[2], in_csr[1])
        self.max_deg = int(max(np.bincount(self.src, minlength=self.n).max(), np.bincount(self.dst, minlength=self.n).max()))


_cases = {}


def case(name, chunk=32):
    key = (name, chunk)
    if key not in _cases:
        _cases[key] = Case(name, chunk)
    return _cases[key]


def rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * scale).to(dtype)


def f64(t):
    return t.detach().cpu().to(torch.float64).numpy()


TOL = {torch.float32: dict(rtol=1e-5, atol=1e-5), torch.float64: dict(rtol=1e-12, atol=1e-12),
       torch.bfloat16: dict(rtol=2e-2, atol=2e-2)}
GTOL = {torch.float32: dict(rtol=1e-4, atol=1e-5), torch.float64: dict(rtol=1e-11, atol=1e-12),
        torch.bfloat16: dict(rtol=2e-2, atol=2e-2)}


def close(got, want, tol, what, terms=1):
    """|got - want| <= atol * max(1, terms / 64) + rtol * |want|.  The stated tolerances are applied literally
    (terms = 1) to every output of the attention layer, normalised or not: o, dq, dk, dv, the softmax and the SpMM
    of softmax weights.  `terms` is passed only where a test feeds an op UNNORMALISED N(0,1) edge weights, so that
    an element is a raw sum of up to `terms` products of size ~1 whose float32 rounding floor grows with its length
    (the stated atol is for attention-like sums); every such call says so."""
    got = f64(got)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    err = np.abs(got - want)
    bound = tol["atol"] * max(1.0, terms / 64.0) + tol["rtol"] * np.abs(want)
    assert np.all(err <= bound), f"{what}: max err {err.max():.3e}, worst excess {(err - bound).max():.3e}"


# --------------------------------------------------------------------------------------------
# the eight ops
# --------------------------------------------------------------------------------------------
SHAPES = [(8, 64), (1, 40), (3, 20), (4, 64), (16, 64), (8, 32)]   # (1,40) and (3,20) only have the generic kernels
FAST = {torch.float32: {(8, 64), (4, 64), (16, 64), (8, 32)}, torch.bfloat16: {(8, 64), (16, 64)}, torch.float64: set()}


def _ops_cases():
    """(graph, chunk, shape, dtype, kernel family): every family a shape and dtype have, the wide (16x64) and the
    narrow (8x32) shape on three of the graphs."""
    out = []
    for gname, chunk in (("blocks8x30", 32), ("blocks8x30", 7), ("bpt512_k4", 32), ("multigraph", 8), ("fc_w100", 32), ("bpt256_k24", 32)):
        for hd in SHAPES:
            if hd in ((16, 64), (8, 32)) and gname not in ("bpt512_k4", "multigraph", "bpt256_k24"):
                continue
            for dtype in (torch.float32, torch.float64, torch.bfloat16):
                families = ["groups-4", "groups-8", "rows", "generic"] if hd in FAST[dtype] else ["groups-4"]
                out += [pytest.param(gname, chunk, hd, dtype, f, id=f"{gname}-{chunk}-{hd[0]}x{hd[1]}-{str(dtype)[6:]}-{f}") for f in families]
    return out


@pytest.mark.parametrize("gname,chunk,hd,dtype,kernels", _ops_cases())
def test_ops_match_oracle(ops, gname, chunk, hd, dtype, kernels):
    """kernels: which family the SpMM / SDDMM ops run in: row groups of 4 or 8 rows, one wavefront per row
    (specialised shapes), or the shape-generic kernels (the only family of the other shapes and of float64)."""
    graphop, _ = ops
    h, d = hd
    force_generic = kernels == "generic"
    c = case(gname, chunk)
    n, E = c.n, c.E
    A = rand((n, h, d), dtype, 1, 0.5).to(DEV)
    B = rand((n, h, d), dtype, 2, 0.5).to(DEV)
    w = rand((E, h), dtype, 3).to(DEV)
    gy = rand((n, h, d), dtype, 4).to(DEV)
    Be = rand((E, d), dtype, 5, 0.5).to(DEV)
    tol, gtol = TOL[dtype], GTOL[dtype]
    graphop.set_force_generic(force_generic)
    old_grouped = graphop.set_grouped_ops(kernels.startswith("groups"))
    old_rows = graphop.set_group_rows(8 if kernels == "groups-8" else 4)
    ctx = long_items(gname)
    ctx.__enter__()
    try:
        # SDDMM as attention.py:66-67 calls it: out-CSR, A = k, B = q
        y = graphop.maskedmm_csr_forward(*c.out, A, B)
        close(y, oracle.maskedmm_csr_forward(*c.np_out, f64(A), f64(B)), tol, "maskedmm fwd")
        dA, dB = graphop.maskedmm_csr_backward(*c.out, *c.inn, A, B, w)
        rA, rB = oracle.maskedmm_csr_backward(*c.np_out, *c.np_in, f64(A), f64(B), f64(w))
        # dy = unnormalised N(0,1) per edge: dA / dB are raw sums of up to max_deg such products (terms)
        close(dA, rA, gtol, "maskedmm dA", c.max_deg); close(dB, rB, gtol, "maskedmm dB", c.max_deg)
        # edge softmax over in-edges
        a = graphop.sparse_softmax_forward(*c.inn[:3], w)
        ra = oracle.sparse_softmax_forward(*c.np_in[:3], f64(w), n_nodes=n)
        close(a, ra, tol, "softmax fwd")
        dx = graphop.sparse_softmax_backward(*c.inn[:3], a, w)
        close(dx, oracle.sparse_softmax_backward(*c.np_in[:3], f64(a), f64(w), n_nodes=n), gtol, "softmax bwd")
        # SpMM over the in-CSR, as the layer calls it: the edge weights are the softmax output (rows sum to 1), so
        # the forward is held to the stated output tolerance as it stands
        o = graphop.vector_spmm_forward(*c.inn, a, A)
        close(o, oracle.vector_spmm_forward(*c.np_in, f64(a), f64(A)), tol, "spmm fwd")
        dw, dxx = graphop.vector_spmm_backward(*c.inn, *c.out, w, gy, A)
        rdw, rdx = oracle.vector_spmm_backward(*c.np_in, *c.np_out, f64(w), f64(gy), f64(A))
        # dedata is one dot product per edge; dx sums up to max_deg products of unnormalised N(0,1) weights: terms
        close(dw, rdw, gtol, "spmm dedata"); close(dxx, rdx, gtol, "spmm dx", c.max_deg)
        # node . edge (rel-pos term), in-CSR, A = q
        yn = graphop.node_mul_edge_forward(*c.inn[:3], A, Be)
        close(yn, oracle.node_mul_edge_forward(*c.np_in[:3], f64(A), f64(Be)), tol, "node_mul_edge fwd")
        dAn, dBe = graphop.node_mul_edge_backward(*c.inn[:3], A, Be, w)
        rAn, rBe = oracle.node_mul_edge_backward(*c.np_in[:3], f64(A), f64(Be), f64(w))
        # dA: raw sum of up to max_deg products of unnormalised N(0,1) edge gradients (terms); dB: h products
        close(dAn, rAn, gtol, "node_mul_edge dA", c.max_deg); close(dBe, rBe, gtol, "node_mul_edge dB")
    finally:
        graphop.set_force_generic(False)
        graphop.set_grouped_ops(old_grouped)
        graphop.set_group_rows(old_rows)
        ctx.__exit__()


def test_single_head_2d_inputs(ops):
    """(n, d) node tensors and (e,) edge tensors, graph_kernel/test.py:148-301 (dim 1024)."""
    graphop, _ = ops
    c = case("blocks8x30")
    A = rand((c.n, 1024), torch.float32, 1, 0.1).to(DEV)
    B = rand((c.n, 1024), torch.float32, 2, 0.1).to(DEV)
    w = rand((c.E,), torch.float32, 3).to(DEV)
    y = graphop.maskedmm_csr_forward(*c.out, A, B)
    assert y.shape == (c.E,)
    close(y, oracle.maskedmm_csr_forward(*c.np_out, f64(A), f64(B)), TOL[torch.float32], "2-D maskedmm")
    a = graphop.sparse_softmax_forward(*c.out[:3], w)
    assert a.shape == (c.E,)
    close(a, oracle.sparse_softmax_forward(*c.np_out[:3], f64(w), n_nodes=c.n), TOL[torch.float32], "2-D softmax")
    o = graphop.vector_spmm_forward(*c.out, a, A)
    close(o, oracle.vector_spmm_forward(*c.np_out, f64(a), f64(A)), TOL[torch.float32], "2-D spmm")


# --------------------------------------------------------------------------------------------
# the attention layer: fused kernels and the unfused op chain, forward + backward
# --------------------------------------------------------------------------------------------
def _layer_cases():
    """(graph, dtype, shape, path): the fused kernels over groups of 4 / 8 rows and per row, and the op chain; (2, 24)
    has no fused instantiation and runs the op chain only."""
    shapes = [(torch.float32, (8, 64)), (torch.float32, (16, 64)), (torch.float32, (8, 32)),
              (torch.bfloat16, (8, 64)), (torch.bfloat16, (16, 64)), (torch.float32, (2, 24))]
    return [pytest.param(g, dt, hd, f, id=f"{g}-{str(dt)[6:]}-{hd[0]}x{hd[1]}-{f or 'chain'}")
            for g in ("bpt512_k4", "bpt300_causal_k2", "multigraph", "fc_w100", "bpt256_k24") for dt, hd in shapes
            for f in (("groups-4", "groups-8", "rows", False) if hd != (2, 24) else (False,))]


@pytest.mark.parametrize("gname,dtype,hd,fused", _layer_cases())
def test_attention_layer(ops, gname, dtype, hd, fused):
    graphop, op = ops
    h, d = hd
    c = case(gname)
    q, k, v, do = (rand((c.n, h, d), dtype, s, 1.0 / 8).to(DEV) for s in (11, 12, 13, 14))   # N(0,1)/sqrt(64)
    q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)
    # fused kernels: one wavefront per group of rows that share neighbours, or one wavefront per row
    old = graphop.set_row_groups(fused != "rows")
    old_r = graphop.set_group_rows({"groups-4": 4, "groups-8": 8}.get(fused))      # None: chosen from dtype and graph
    ctx = long_items(gname)
    ctx.__enter__()
    try:
        o = op.bpt_attention(*c.out, *c.inn, q, k, v, fused=bool(fused))
        o.backward(do)
    finally:
        ctx.__exit__()
        graphop.set_row_groups(old)
        graphop.set_group_rows(old_r)
    ro, ra = oracle.attention_forward(c.csr, f64(q), f64(k), f64(v))
    rdq, rdk, rdv = oracle.attention_backward(c.csr, f64(q), f64(k), f64(v), ra, f64(do))
    close(o, ro, TOL[dtype], "o")
    close(q.grad, rdq, GTOL[dtype], "dq"); close(k.grad, rdk, GTOL[dtype], "dk"); close(v.grad, rdv, GTOL[dtype], "dv")


def test_attention_with_rel_pos_chain(ops):
    """modules/attention.py:66-77 with rel_pos: masked_mm + node_mul_edge -> softmax -> spmm, through autograd."""
    _, op = ops
    c = case("bpt300_causal_k2")
    h, d = 8, 64
    q, k, v, do = (rand((c.n, h, d), torch.float32, s, 1.0 / 8).to(DEV).requires_grad_(s < 14) for s in (11, 12, 13, 14))
    ak = rand((c.E, d), torch.float32, 15, 1.0 / 8).to(DEV).requires_grad_(True)
    e = op.masked_mm(*c.out, *c.inn, k, q)
    e_rel = op.node_mul_edge(*c.inn[:3], q, ak)
    a = op.sparse_softmax(*c.inn[:3], (e_rel + e) / np.sqrt(d))
    o = op.vec_spmm(*c.inn, *c.out, a, v)
    o.backward(do)
    ro, ra = oracle.attention_forward(c.csr, f64(q), f64(k), f64(v), f64(ak))
    rdq, rdk, rdv, rdak = oracle.attention_backward(c.csr, f64(q), f64(k), f64(v), ra, f64(do), f64(ak))
    close(o, ro, TOL[torch.float32], "o")
    for got, want, nm in ((q.grad, rdq, "dq"), (k.grad, rdk, "dk"), (v.grad, rdv, "dv"), (ak.grad, rdak, "dak")):
        close(got, want, GTOL[torch.float32], nm)


def test_headline_graph_full_parity(ops):
    """benchmark configuration 3 at full size (L=8192, k=4, causal, 8x64 fp32) directly against the oracle."""
    _, op = ops
    from bpt_amd import graphbuilder as gb
    g = gb.BinaryPartition(8192, True, 4, 10)
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    csr = gb.get_csrs(src, dst, n, as_torch=False)
    out_csr, in_csr, ROW, IR, COL, IC = csr
    t = lambda a: torch.from_numpy(a).to(DEV)
    args = (t(ROW), t(IR), t(out_csr[2]), t(out_csr[1]), t(COL), t(IC), t(in_csr[2]), t(in_csr[1]))
    gen = torch.Generator().manual_seed(2345)
    q, k, v, do = (torch.randn(n, 8, 64, generator=gen) / 8 for _ in range(4))
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    o = op.bpt_attention(*args, qd, kd, vd)
    o.backward(do.to(DEV))
    ro, ra = oracle.attention_forward(csr, f64(q), f64(k), f64(v))
    rdq, rdk, rdv = oracle.attention_backward(csr, f64(q), f64(k), f64(v), ra, f64(do))
    close(o, ro, TOL[torch.float32], "o")
    close(qd.grad, rdq, GTOL[torch.float32], "dq"); close(kd.grad, rdk, GTOL[torch.float32], "dk")
    close(vd.grad, rdv, GTOL[torch.float32], "dv")
    # unfused chain agrees with the fused kernels
    o2 = op.bpt_attention(*args, qd.detach(), kd.detach(), vd.detach(), fused=False)
    assert torch.allclose(o2, o.detach(), rtol=1e-5, atol=1e-5)


def test_stress_graph_properties(ops):
    """benchmark configuration 5 (L=32768, k=8, causal, 16x64, bf16): size-independent properties."""
    _, op = ops
    from bpt_amd import graphbuilder as gb
    g = gb.BinaryPartition(32768, True, 8, 10)
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    assert (n, len(src)) == (65535, 3293955)
    csr = gb.get_csrs(src, dst, n)
    out_csr, in_csr, ROW, IR, COL, IC = csr
    args = tuple(x.to(DEV) for x in (ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1]))
    gen = torch.Generator().manual_seed(2345)
    q, k, do = (((torch.randn(n, 16, 64, generator=gen) / 8).to(torch.bfloat16)).to(DEV) for _ in range(3))
    # 1. v == 1  =>  o == 1 wherever a node has in-edges (softmax rows sum to one); every node has one here
    ones = torch.ones(n, 16, 64, dtype=torch.bfloat16, device=DEV)
    o = op.bpt_attention(*args, q, k, ones)
    assert torch.allclose(o.float(), torch.ones_like(o, dtype=torch.float32), rtol=1e-2, atol=1e-2)
    # 2. column sums of dV equal column sums of dO (sum_e p_e = 1 per destination)
    v = ones.clone().requires_grad_(True)
    qg = q.clone().requires_grad_(True)
    op.bpt_attention(*args, qg, k, v).backward(do)
    assert torch.allclose(v.grad.float().sum(0), do.float().sum(0), rtol=2e-2, atol=0.5)
    # 3. with constant v the output does not depend on q: dq == 0 (dp == delta for every edge)
    assert qg.grad.float().abs().max().item() < 2e-2
    # 4. run-to-run bit reproducibility (no atomics)
    o2 = op.bpt_attention(*args, q, k, ones)
    assert torch.equal(o, o2)
    # 5. the op chain (row-group SDDMM / SpMM, segmented softmax) agrees with the fused kernels on random v
    vr = ((torch.randn(n, 16, 64, generator=gen) / 8).to(torch.bfloat16)).to(DEV)
    of = op.bpt_attention(*args, q, k, vr)
    oc = op.bpt_attention(*args, q, k, vr, fused=False)
    assert torch.allclose(of.float(), oc.float(), rtol=2e-2, atol=2e-2)
    # 6. plans built on the host and on the GPU (this size takes the GPU by default) give the same result up to rounding
    from bpt_amd import plan
    assert isinstance(plan.plan_cache.get(*args[4:], n, n), plan.DevicePlan)
    old = plan.set_device_build(False)
    plan.plan_cache.clear()
    try:
        oh = op.bpt_attention(*args, q, k, vr)
        assert isinstance(plan.plan_cache.get(*args[4:], n, n), plan.Plan)
    finally:
        plan.set_device_build(old)
        plan.plan_cache.clear()
    assert torch.allclose(of.float(), oh.float(), rtol=2e-2, atol=2e-2)


def test_determinism_and_cache(ops):
    graphop, op = ops
    from bpt_amd.plan import plan_cache
    c = case("bpt512_k4")
    q, k, v, do = (rand((c.n, 8, 64), torch.float32, s, 1.0 / 8).to(DEV) for s in (1, 2, 3, 4))
    outs = []
    for _ in range(2):
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (q, k, v))
        o = op.bpt_attention(*c.out, *c.inn, qq, kk, vv)
        o.backward(do)
        outs.append((o.detach(), qq.grad, kk.grad, vv.grad))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    h0 = plan_cache.hits
    graphop.sparse_softmax_forward(*c.inn[:3], rand((c.E, 8), torch.float32, 5).to(DEV))
    graphop.sparse_softmax_forward(*c.inn[:3], rand((c.E, 8), torch.float32, 6).to(DEV))
    assert plan_cache.hits >= h0 + 1


def test_input_checks(ops):
    graphop, _ = ops
    c = case("blocks8x30")
    A = rand((c.n, 8, 64), torch.float32, 1).to(DEV)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):          # graphop.cpp:4
        graphop.maskedmm_csr_forward(*c.out, A.cpu(), A)
    with pytest.raises(RuntimeError, match="must be contiguous"):             # graphop.cpp:5
        graphop.maskedmm_csr_forward(*c.out, A.transpose(0, 1).contiguous().transpose(0, 1), A)
    with pytest.raises(RuntimeError, match="dtype"):
        graphop.maskedmm_csr_forward(*c.out, A.half(), A.half())
    bad_idx = c.out[3].clone(); bad_idx[0] = c.n + 5
    with pytest.raises(ValueError, match="out of range"):
        graphop.maskedmm_csr_forward(c.out[0], c.out[1], c.out[2], bad_idx, A, A)


def test_zero_degree_rows_are_zero(ops):
    graphop, _ = ops
    c = case("multigraph")
    x = rand((c.n, 8, 64), torch.float32, 1).to(DEV)
    w = rand((c.E, 8), torch.float32, 2).to(DEV)
    y = graphop.vector_spmm_forward(*c.inn, w, x)
    assert torch.all(y[0] == 0)
    o, lse = graphop.attention_forward(*c.inn, x, x, x)
    assert torch.all(o[0] == 0)


# --------------------------------------------------------------------------------------------
# dropout on the attention probabilities inside the fused kernels (modules/attention.py:73)
# --------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,hd", [(torch.float32, (8, 64)), (torch.float32, (16, 64)), (torch.bfloat16, (8, 64))])
@pytest.mark.parametrize("gname,rows", [("bpt512_k4", 4), ("bpt512_k4", 8), ("multigraph", 4), ("fc_w100", 8),
                                        ("bpt512_k4", None), ("multigraph", None)])          # None: the library's choice (tiles of 16 rows)
def test_fused_attention_dropout_matches_oracle_with_the_same_mask(ops, gname, rows, dtype, hd):
    from oracle import torch_ops
    graphop, op = ops
    h, d = hd
    p, seed = 0.25, 1234567890123
    c = case(gname)
    q, k, v, do = (rand((c.n, h, d), dtype, s, 1.0 / 8).to(DEV) for s in (21, 22, 23, 24))
    q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)
    old_r = graphop.set_group_rows(rows)
    ctx = long_items(gname)
    ctx.__enter__()
    try:
        mask = graphop.attention_dropout_mask(*c.inn, q, k, p, seed)          # (E, h): 0 or 1 / (1 - p)
        o = op.bpt_attention(*c.out, *c.inn, q, k, v, dropout_p=p, seed=seed)
        o.backward(do)
        o2 = op.bpt_attention(*c.out, *c.inn, q, k, v, dropout_p=p, seed=seed)
        o3 = op.bpt_attention(*c.out, *c.inn, q, k, v, dropout_p=p, seed=seed + 1)
    finally:
        ctx.__exit__()
        graphop.set_group_rows(old_r)
    vals = mask.numpy()
    assert np.all((vals == 0) | (np.abs(vals - 1 / (1 - p)) < 1e-6))
    kept = float((mask > 0).float().mean())
    assert abs(kept - (1 - p)) < 4 * np.sqrt(p * (1 - p) / mask.numel()) + 1e-3, kept      # Bernoulli(1 - p) per (edge, head)
    assert torch.equal(o, o2) and not torch.equal(o, o3)                                  # a function of the seed
    t64 = lambda x: x.detach().cpu().double()
    src, dst = torch.from_numpy(c.src), torch.from_numpy(c.dst)
    ro, rdq, rdk, rdv = torch_ops.attention_fwd_bwd(src, dst, t64(q), t64(k), t64(v), t64(do), drop=mask.double())
    close(o, ro.numpy(), TOL[dtype], "o")
    close(q.grad, rdq.numpy(), GTOL[dtype], "dq")
    close(k.grad, rdk.numpy(), GTOL[dtype], "dk")
    close(v.grad, rdv.numpy(), GTOL[dtype], "dv")


# --------------------------------------------------------------------------------------------
# the rel_pos score term inside the fused kernels (modules/attention.py:69-71), with and without dropout
# --------------------------------------------------------------------------------------------
@pytest.mark.parametrize("p", [0.0, 0.25])
@pytest.mark.parametrize("dtype,hd", [(torch.float32, (8, 64)), (torch.float32, (16, 64)), (torch.float32, (4, 64)), (torch.bfloat16, (8, 64))])
@pytest.mark.parametrize("gname,rows", [("bpt512_k4", 4), ("bpt512_k4", 8), ("bpt300_causal_k2", None), ("multigraph", 4), ("fc_w100", 8),
                                        ("bpt256_k24", 8), ("multigraph", None), ("fc_w100", None)])    # None: the library's choice (tiles of 16 rows)
def test_fused_attention_with_rel_pos_matches_oracle(ops, gname, rows, dtype, hd, p):
    from oracle import torch_ops
    graphop, op = ops
    h, d = hd
    n_types, seed = 37, 987654321
    c = case(gname)
    q, k, v, do = (rand((c.n, h, d), dtype, s, 1.0 / 8).to(DEV) for s in (31, 32, 33, 34))
    table = rand((n_types, d), dtype, 35, 1.0 / 8).to(DEV)
    etype = torch.from_numpy(np.random.default_rng(36).integers(0, n_types, c.E)).to(DEV)
    for t in (q, k, v, table):
        t.requires_grad_(True)
    old_r = graphop.set_group_rows(rows)
    ctx = long_items(gname)
    ctx.__enter__()
    try:
        mask = graphop.attention_dropout_mask(*c.inn, q, k, p, seed) if p > 0 else None
        o = op.bpt_attention(*c.out, *c.inn, q, k, v, dropout_p=p, seed=seed, rel_table=table, etype=etype)
        o.backward(do)
    finally:
        ctx.__exit__()
        graphop.set_group_rows(old_r)
    t64 = lambda x: x.detach().cpu().double()
    src, dst, et = torch.from_numpy(c.src), torch.from_numpy(c.dst), etype.cpu()
    ro, rdq, rdk, rdv, rdak = torch_ops.attention_fwd_bwd(src, dst, t64(q), t64(k), t64(v), t64(do), ak=t64(table)[et],
                                                          drop=mask.double() if mask is not None else None)
    rdt = torch.zeros(n_types, d, dtype=torch.float64).index_add_(0, et, rdak)
    close(o, ro.numpy(), TOL[dtype], "o")
    close(q.grad, rdq.numpy(), GTOL[dtype], "dq")
    close(k.grad, rdk.numpy(), GTOL[dtype], "dk")
    close(v.grad, rdv.numpy(), GTOL[dtype], "dv")
    # a table row is a raw sum over all edges of its type and all heads (h * E / n_types products): terms
    close(table.grad, rdt.numpy(), GTOL[dtype], "dtable", h * c.E / n_types)


def test_rel_pos_without_row_groups_takes_the_op_chain_and_the_raw_call_refuses(ops):
    graphop, op = ops
    c = case("bpt300_causal_k2")
    h, d, n_types = 8, 64, 11
    q, k, v = (rand((c.n, h, d), torch.float32, s, 1.0 / 8).to(DEV) for s in (41, 42, 43))
    table = rand((n_types, d), torch.float32, 44, 1.0 / 8).to(DEV)
    etype = torch.from_numpy(np.random.default_rng(45).integers(0, n_types, c.E)).to(DEV)
    want = op.bpt_attention(*c.out, *c.inn, q, k, v, rel_table=table, etype=etype)
    old = graphop.set_row_groups(False)
    try:
        got = op.bpt_attention(*c.out, *c.inn, q, k, v, rel_table=table, etype=etype)          # op chain
        bias = torch.zeros((c.E + 1, h), dtype=torch.float32, device=DEV)
        with pytest.raises(RuntimeError):
            graphop.attention_forward(*c.inn, q, k, v, bias=bias)
    finally:
        graphop.set_row_groups(old)
    close(got, f64(want), TOL[torch.float32], "chain vs fused")
    with pytest.raises(ValueError):
        graphop.attention_forward(*c.inn, q, k, v, bias=torch.zeros((c.E, h), dtype=torch.float32, device=DEV))   # no spare row
    with pytest.raises(ValueError):
        op.bpt_attention(*c.out, *c.inn, q, k, v, rel_table=table)                                                  # etype missing


@pytest.mark.parametrize("rows", [4, 8])
def test_fused_attention_with_large_scores(ops, rows):
    """Scores of +-60 (q, k four times the usual size): nearly one-hot softmax rows, exponent references that move by
    large steps.  Errors are measured against the largest element (rounding of a score of 60 moves its exponential
    by 4e-6 relative in float32)."""
    from oracle import torch_ops
    graphop, op = ops
    c = case("bpt512_k4")
    h, d = 8, 64
    q, k = (rand((c.n, h, d), torch.float32, s, 4.0).to(DEV).requires_grad_(True) for s in (51, 52))
    v = rand((c.n, h, d), torch.float32, 53).to(DEV).requires_grad_(True)
    do = rand((c.n, h, d), torch.float32, 54).to(DEV)
    old_r = graphop.set_group_rows(rows)
    try:
        o = op.bpt_attention(*c.out, *c.inn, q, k, v)
        o.backward(do)
    finally:
        graphop.set_group_rows(old_r)
    t64 = lambda x: x.detach().cpu().double()
    ro, rdq, rdk, rdv = torch_ops.attention_fwd_bwd(torch.from_numpy(c.src), torch.from_numpy(c.dst), t64(q), t64(k), t64(v), t64(do))
    assert torch.isfinite(o).all()
    for got, want, nm in ((o, ro, "o"), (q.grad, rdq, "dq"), (k.grad, rdk, "dk"), (v.grad, rdv, "dv")):
        err = float((t64(got) - want).abs().max() / want.abs().max())
        assert err < 5e-5, (nm, err)


def test_block_uses_fused_dropout_in_training(ops):
    from bpt_amd.block import BPTBlock
    from bpt_amd import graphbuilder as gb
    c = case("bpt300_causal_k2")
    csr = gb.get_csrs(c.src, c.dst, c.n)
    csr_dev = tuple(tuple(t.to(DEV) for t in x) if isinstance(x, (tuple, list)) else x.to(DEV) for x in csr)
    torch.manual_seed(3)
    blk = BPTBlock(512, 8, 128, rel_pos=False, drop_h=0.0, drop_a=0.3).to(DEV)
    h0 = torch.randn(c.n, 512, device=DEV)
    blk.train()
    torch.manual_seed(11); a = blk(h0, csr_dev)
    torch.manual_seed(11); b = blk(h0, csr_dev)
    torch.manual_seed(12); d_ = blk(h0, csr_dev)
    blk.eval()
    e = blk(h0, csr_dev)
    assert torch.equal(a, b) and not torch.equal(a, d_) and not torch.equal(a, e)
    assert torch.isfinite(a).all()


# --------------------------------------------------------------------------------------------
# attention to memory over an inter graph (modules/attention.py:144-168, graph/mt.py:318-347): bipartite blocks
# from encoder nodes to decoder nodes in one index space of max(n_enc, n_dec) nodes, most rows without edges
# --------------------------------------------------------------------------------------------
def inter_graph(n_enc, n_dec, seg_enc, seg_dec):
    rows, cols = [], []
    e0 = d0 = 0
    for le, ld in zip(seg_enc, seg_dec):
        src = np.arange(e0, e0 + le); dst = np.arange(d0, d0 + ld)
        rows.append(np.repeat(src, ld)); cols.append(np.tile(dst, le))     # graph/mt.py:318-321
        e0 += le + 3; d0 += ld + 2                                          # internal (span) nodes in between have no inter edges
    assert e0 <= n_enc + 3 and d0 <= n_dec + 2
    return np.concatenate(rows).astype(np.int64), np.concatenate(cols).astype(np.int64), max(n_enc, n_dec)


@pytest.mark.parametrize("n_enc,n_dec", [(200, 120), (150, 150)])     # the reference needs n_dec <= n_enc: y = zeros_like(v)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_to_memory_over_an_inter_graph(ops, n_enc, n_dec, dtype):
    from bpt_amd import graphbuilder as gb
    from oracle import torch_ops
    graphop, op = ops
    h, d = 8, 64
    src, dst, n = inter_graph(n_enc, n_dec, [40, 70, 25], [30, 20, 45])
    out_csr, in_csr, ROW, IR, COL, IC = gb.get_csrs(src, dst, n)
    t = lambda a: a.to(DEV)
    graph = (t(ROW), t(IR), t(out_csr[2]), t(out_csr[1]), t(COL), t(IC), t(in_csr[2]), t(in_csr[1]))
    # queries: decoder states padded to the memory's length when shorter (attention.py:148-149); keys/values: the memory
    nq = max(n_dec, n_enc)
    q = rand((nq, h, d), dtype, 31, 1.0 / 8).to(DEV).requires_grad_(True)
    k = rand((n_enc, h, d), dtype, 32, 1.0 / 8).to(DEV).requires_grad_(True)
    v = rand((n_enc, h, d), dtype, 33, 1.0 / 8).to(DEV).requires_grad_(True)
    do = rand((nq, h, d), dtype, 34, 1.0 / 8).to(DEV)
    o = op.bpt_attention(*graph, q, k, v)          # fused when q and k have the same number of rows, else the op chain
    o.backward(do)
    t64 = lambda x: x.detach().cpu().double()
    ro, rdq, rdk, rdv = torch_ops.attention_fwd_bwd(torch.from_numpy(src), torch.from_numpy(dst), t64(q), t64(k), t64(v), t64(do))
    close(o, ro.numpy(), TOL[dtype], "o")
    close(q.grad, rdq.numpy(), GTOL[dtype], "dq")
    close(k.grad, rdk.numpy(), GTOL[dtype], "dk")
    close(v.grad, rdv.numpy(), GTOL[dtype], "dv")
    assert not o[min(n_dec, 101):].any()             # rows without in-edges (span nodes, padding) stay zero


@pytest.mark.parametrize("grouped", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_vector_spmm_accumulates_into_out(ops, dtype, grouped):
    """vector_spmm_forward(out=y0) returns y0 + the product: in the row-group kernel's store, or by a separate addition
    where there is none (one wavefront per row; 2-D inputs)."""
    graphop, _ = ops
    c = case("bpt512_k4")
    w = rand((c.E, 8), dtype, 1).to(DEV)
    x = rand((c.n, 8, 64), dtype, 2, 0.5).to(DEV)
    y0 = rand((c.n, 8, 64), dtype, 3).to(DEV)
    old = graphop.set_grouped_ops(grouped)
    try:
        want = oracle.vector_spmm_forward(*c.np_in, f64(w), f64(x)) + f64(y0)
        out = y0.clone()
        got = graphop.vector_spmm_forward(*c.inn, w, x, out=out)
        assert got is out
        # unnormalised N(0,1) edge weights: an element is a raw sum of up to max_deg products (terms)
        close(got, want, GTOL[dtype] if dtype == torch.float32 else TOL[dtype], "spmm accumulate", c.max_deg)
        with pytest.raises(ValueError):
            graphop.vector_spmm_forward(*c.inn, w, x, out=y0[:-1])
    finally:
        graphop.set_grouped_ops(old)
