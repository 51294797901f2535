"""The one degree of freedom of the graph layouts that nothing in the reference pins: the order of the slots INSIDE a
CSR row (the reference takes both CSRs from DGL 0.4's adjacency_matrix_scipy, graph/base.py:72,79).  Every op and the
fused layer are run on three layouts of the same graph:

  (a) the default (ascending edge id in both CSRs),
  (b) in-CSR rows in (source, edge id) order (get_csrs(..., in_order="src_eid")),
  (c) a seeded random permutation inside every row of BOTH CSRs,

and must give: bit-identical results wherever an element is computed from one edge alone (SDDMM scores, the
node-times-edge scores and its per-edge gradient, the per-edge gradient of the SpMM), and results within the
stated tolerances of the float64 oracle wherever a row is reduced (softmax, SpMM, all node gradients, the fused
layer), whose rounding depends on the order of the sum."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = dict(rtol=1e-5, atol=1e-5)
GTOL = dict(rtol=1e-4, atol=1e-5)


def f64(t):
    return t.detach().cpu().to(torch.float64).numpy()


def check(got, want, tol, what):
    err = np.abs(f64(got) - want)
    bound = tol["atol"] + tol["rtol"] * np.abs(want)
    assert np.all(err <= bound), f"{what}: max err {err.max():.3e}, worst excess {(err - bound).max():.3e}"


def permute_rows(csr, seed):
    indptr, indices, eid = (np.array(a) for a in csr)
    rng = np.random.default_rng(seed)
    for r in range(len(indptr) - 1):
        p = rng.permutation(indptr[r + 1] - indptr[r]) + indptr[r]
        indices[indptr[r]:indptr[r + 1]] = indices[p]
        eid[indptr[r]:indptr[r + 1]] = eid[p]
    return indptr, indices, eid


def layouts(L, triu, step):
    from bpt_amd import graphbuilder as gb
    g = gb.BinaryPartition(L, triu, step, 10)
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    base = gb.get_csrs(src, dst, n, as_torch=False)
    alt = gb.get_csrs(src, dst, n, as_torch=False, in_order="src_eid")
    perm = (permute_rows(base[0], 1), permute_rows(base[1], 2)) + tuple(base[2:])
    assert not np.array_equal(perm[1][2], base[1][2]) and not np.array_equal(perm[0][2], base[0][2])
    return n, len(src), {"eid": base, "src_eid": alt, "permuted": perm}


def dev_args(csr):
    out_csr, in_csr, ROW, IR, COL, IC = csr
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    return (t(ROW), t(IR), t(out_csr[2]), t(out_csr[1])), (t(COL), t(IC), t(in_csr[2]), t(in_csr[1]))


@pytest.mark.parametrize("L,triu,step", [(512, False, 4), (300, True, 2), (2048, True, 4)])
def test_results_do_not_depend_on_the_order_inside_csr_rows(L, triu, step):
    from bpt_amd import graphop, op
    n, E, lay = layouts(L, triu, step)
    h, d = 8, 64
    gen = torch.Generator().manual_seed(7)
    q, k, v, do = ((torch.randn(n, h, d, generator=gen) / 8).to(DEV) for _ in range(4))
    w = torch.randn(E, h, generator=gen).to(DEV)
    be = (torch.randn(E, d, generator=gen) / 8).to(DEV)
    base = lay["eid"]
    np_out = (base[2], base[3], base[0][2], base[0][1])
    np_in = (base[4], base[5], base[1][2], base[1][1])
    ro, ra = oracle.attention_forward(base, f64(q), f64(k), f64(v))
    rdq, rdk, rdv = oracle.attention_backward(base, f64(q), f64(k), f64(v), ra, f64(do))
    r_soft = oracle.sparse_softmax_forward(*np_in[:3], f64(w), n_nodes=n)
    results = {}
    for name, csr in lay.items():
        out, inn = dev_args(csr)
        res = {}
        # one edge per element: must not depend on the layout at all
        res["sddmm"] = graphop.maskedmm_csr_forward(*out, k, q)
        res["nme"] = graphop.node_mul_edge_forward(*inn[:3], q, be)
        res["nme_dB"] = graphop.node_mul_edge_backward(*inn[:3], q, be, w)[1]
        a = graphop.sparse_softmax_forward(*inn[:3], w)
        res["spmm_dedata"] = graphop.vector_spmm_backward(*inn, *out, a, do, v)[0]
        # row reductions: within tolerance of the oracle for every layout
        check(a, r_soft, TOL, f"{name}: softmax")
        check(graphop.vector_spmm_forward(*inn, a, v), oracle.vector_spmm_forward(*np_in, f64(a), f64(v)), TOL, f"{name}: spmm")
        qd, kd, vd = (x.clone().requires_grad_(True) for x in (q, k, v))
        for fused in (True, False):
            o = op.bpt_attention(*out, *inn, qd, kd, vd, fused=fused)
            check(o, ro, TOL, f"{name}: o (fused={fused})")
        o.backward(do)                                       # the op chain's backward
        for got, want, nm in ((qd.grad, rdq, "dq"), (kd.grad, rdk, "dk"), (vd.grad, rdv, "dv")):
            check(got, want, GTOL, f"{name}: chain {nm}")
        qd, kd, vd = (x.clone().requires_grad_(True) for x in (q, k, v))
        op.bpt_attention(*out, *inn, qd, kd, vd, fused=True).backward(do)
        for got, want, nm in ((qd.grad, rdq, "dq"), (kd.grad, rdk, "dk"), (vd.grad, rdv, "dv")):
            check(got, want, GTOL, f"{name}: fused {nm}")
        results[name] = res
    for name in ("src_eid", "permuted"):
        for key, t in results[name].items():
            assert torch.equal(t, results["eid"][key]), f"{key} differs between the default layout and {name}"
