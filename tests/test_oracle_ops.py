"""Pins the oracle's operator semantics without retyping its formulas: dense closed forms on
block-diagonal fully-connected graphs (the method of graph_kernel/test.py:185,218,245,274,314,364),
dense-adjacency matmuls on random multigraphs, autograd of an independent gather/index_add
restatement, and invariants."""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ops


def block_graph(batch, l):
    """graph_kernel/test.py:79-112: `batch` fully connected blocks of l nodes; edge x->y has id
    cnt in row-major (x, y) order.  Returns src(=x), dst(=y)."""
    x = np.repeat(np.arange(batch * l), l)
    y = (np.arange(batch * l * l) % l) + (np.arange(batch * l * l) // (l * l)) * l
    return x.astype(np.int64), y.astype(np.int64)


def rand(rng, *shape, dtype=np.float64):
    return rng.standard_normal(shape).astype(dtype)


@pytest.mark.parametrize("chunk", [32, 7])       # chunk 7 splits every 10-edge row over 2 units
@pytest.mark.parametrize("multi_head", [True, False])
def test_block_dense_closed_forms(chunk, multi_head):
    rng = np.random.default_rng(0)
    batch, l, h, d = 5, 10, (4 if multi_head else 1), 6
    src, dst = block_graph(batch, l)
    n, E = batch * l, len(src)
    out_csr, in_csr, ROW, IR, COL, IC = oracle.get_csrs(src, dst, n, chunk)
    # closed form of the CSC edge ids, graph_kernel/test.py:104-112
    b_, y_, x_ = np.meshgrid(np.arange(batch), np.arange(l), np.arange(l), indexing="ij")
    assert np.array_equal(in_csr[2], (b_ * l * l + x_ * l + y_).ravel())
    assert np.array_equal(out_csr[2], np.arange(E))

    shp = (n, h, d) if multi_head else (n, d)
    A, B = rand(rng, *shp), rand(rng, *shp)
    A4, B4 = A.reshape(batch, l, h, d), B.reshape(batch, l, h, d)
    # --- SDDMM vs bmm (test.py:185, 364): y[(b,x,y),h] = A[b,x,h].B[b,y,h]
    y = oracle.maskedmm_csr_forward(ROW, IR, out_csr[2], out_csr[1], A, B)
    y_dense = np.einsum("bxhd,byhd->bxyh", A4, B4)
    assert np.allclose(y.reshape(batch, l, l, h), y_dense, rtol=1e-12, atol=1e-12)
    assert y.shape == ((E, h) if multi_head else (E,))
    g = rand(rng, *y.shape)
    dA, dB = oracle.maskedmm_csr_backward(ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1], A, B, g)
    g4 = g.reshape(batch, l, l, h)
    assert np.allclose(dA.reshape(A4.shape), np.einsum("bxyh,byhd->bxhd", g4, B4))
    assert np.allclose(dB.reshape(B4.shape), np.einsum("bxyh,bxhd->byhd", g4, A4))

    # --- softmax "scatter" (rows, test.py:218,395) and "gather" (columns, test.py:245,422)
    x = rand(rng, *y.shape)
    xs = torch.tensor(x.reshape(batch, l, l, h), requires_grad=True)
    for (units, ip, eid, dim) in ((ROW, IR, out_csr[2], 2), (COL, IC, in_csr[2], 1)):
        ys = torch.softmax(xs, dim)
        got = oracle.sparse_softmax_forward(units, ip, eid, x, n_nodes=n)
        assert np.allclose(got.reshape(batch, l, l, h), ys.detach().numpy(), rtol=1e-12, atol=1e-14)
        (gx,) = torch.autograd.grad(ys, xs, torch.tensor(g4))
        got_dx = oracle.sparse_softmax_backward(units, ip, eid, got, g, n_nodes=n)
        assert np.allclose(got_dx.reshape(batch, l, l, h), gx.numpy(), rtol=1e-10, atol=1e-13)

    # --- SpMM vs dense adjacency matmul per head (test.py:274-299, 465-481): y[b,x] = sum_y w[b,x,y] A[b,y]
    w = rand(rng, *y.shape)
    w4 = w.reshape(batch, l, l, h)
    ysp = oracle.vector_spmm_forward(ROW, IR, out_csr[2], out_csr[1], w, A)
    assert np.allclose(ysp.reshape(A4.shape), np.einsum("bxyh,byhd->bxhd", w4, A4))
    gy = rand(rng, *shp)
    dw, dx = oracle.vector_spmm_backward(ROW, IR, out_csr[2], out_csr[1], COL, IC, in_csr[2], in_csr[1], w, gy, A)
    gy4 = gy.reshape(A4.shape)
    assert np.allclose(dw.reshape(w4.shape), np.einsum("bxhd,byhd->bxyh", gy4, A4))
    assert np.allclose(dx.reshape(A4.shape), np.einsum("bxyh,bxhd->byhd", w4, gy4))

    # --- node_mul_edge vs gather-to-edge formulation (test.py:314-337)
    Be = rand(rng, E, d)
    A3 = A.reshape(n, h, d)
    yn = oracle.node_mul_edge_forward(ROW, IR, out_csr[2], A, Be)
    assert np.allclose(yn.reshape(E, h), np.einsum("ehd,ed->eh", A3[src], Be))
    dAn, dBe = oracle.node_mul_edge_backward(ROW, IR, out_csr[2], A, Be, g)
    g2 = g.reshape(E, h)
    ref_dA = np.zeros_like(A3)
    np.add.at(ref_dA, src, g2[:, :, None] * Be[:, None, :])
    assert np.allclose(dAn.reshape(n, h, d), ref_dA)
    assert np.allclose(dBe, np.einsum("eh,ehd->ed", g2, A3[src]))


def random_multigraph(rng, n, E):
    """random edges with duplicates, zero-degree nodes and one heavy row."""
    src = rng.integers(0, n, E)
    dst = rng.integers(0, n, E)
    dst[: E // 3] = 1                      # heavy destination
    src[E // 3: E // 2] = 2                # heavy source
    src[src == 0] = 3; dst[dst == 0] = 3   # node 0 isolated
    src[-1], dst[-1] = src[-2], dst[-2]    # guaranteed duplicate edge
    return src.astype(np.int64), dst.astype(np.int64)


def test_multigraph_vs_dense_adjacency():
    rng = np.random.default_rng(1)
    n, E, h, d = 23, 400, 3, 5
    src, dst = random_multigraph(rng, n, E)
    out_csr, in_csr, ROW, IR, COL, IC = oracle.get_csrs(src, dst, n, chunk_size=8)
    assert len(ROW) != len(COL)             # exercises the dx grid of vector_spmm_backward
    q, k, v = rand(rng, n, h, d), rand(rng, n, h, d), rand(rng, n, h, d)
    w = rand(rng, E, h)
    # dense: W[dst, src, h] accumulates duplicates
    W = np.zeros((n, n, h))
    np.add.at(W, (dst, src), w)
    o = oracle.vector_spmm_forward(COL, IC, in_csr[2], in_csr[1], w, v)
    assert np.allclose(o, np.einsum("rsh,shd->rhd", W, v))
    assert np.all(o[0] == 0)                # zero-degree row stays zero
    gy = rand(rng, n, h, d)
    dw, dv = oracle.vector_spmm_backward(COL, IC, in_csr[2], in_csr[1], ROW, IR, out_csr[2], out_csr[1], w, gy, v)
    assert np.allclose(dv, np.einsum("rsh,rhd->shd", W, gy))
    assert np.allclose(dw, np.einsum("ehd,ehd->eh", gy[dst], v[src]))
    # the reference's launch (row-side grid for the dx kernel) drops units when U_out > U_in
    _, dv_ref = oracle.vector_spmm_backward(COL, IC, in_csr[2], in_csr[1], ROW, IR, out_csr[2], out_csr[1], w, gy, v,
                                            reference_grid=True)
    if len(ROW) > len(COL):
        assert not np.allclose(dv_ref, dv)
    # SDDMM over the out-CSR as attention.py:66-67 calls it (A=k, B=q): e = k[src].q[dst]
    e = oracle.maskedmm_csr_forward(ROW, IR, out_csr[2], out_csr[1], k, q)
    assert np.allclose(e, np.einsum("ehd,ehd->eh", k[src], q[dst]))
    # softmax rows sum to one per destination with in-edges; sum_row dx = 0
    a = oracle.sparse_softmax_forward(COL, IC, in_csr[2], e, n_nodes=n)
    sums = np.zeros((n, h)); np.add.at(sums, dst, a)
    has = np.bincount(dst, minlength=n) > 0
    assert np.allclose(sums[has], 1.0) and np.all(sums[~has] == 0)
    dx = oracle.sparse_softmax_backward(COL, IC, in_csr[2], a, w, n_nodes=n)
    tot = np.zeros((n, h)); np.add.at(tot, dst, dx)
    assert np.allclose(tot, 0, atol=1e-12)


@pytest.mark.parametrize("cfg", [(33, False, 2), (64, True, 4), (100, False, 1)])
@pytest.mark.parametrize("rel", [False, True])
def test_attention_vs_autograd(cfg, rel):
    """C-oracle layer (op sequence + hand-derived backward ops) vs autograd of the torch restatement."""
    L, triu, step = cfg
    rng = np.random.default_rng(2)
    g = oracle.BinaryPartition(L, triu, step, 10)
    src, dst, _ = g.get_edges()
    n, E, h, d = g.number_of_nodes, g.number_of_edges, 2, 8
    csr = oracle.get_csrs(src, dst, n)
    q, k, v, do = (rand(rng, n, h, d) for _ in range(4))
    ak = rand(rng, E, d) if rel else None
    o, a = oracle.attention_forward(csr, q, k, v, ak)
    grads = oracle.attention_backward(csr, q, k, v, a, do, ak)
    t = lambda z: None if z is None else torch.tensor(z)
    ref = torch_ops.attention_fwd_bwd(t(src), t(dst), t(q), t(k), t(v), t(do), t(ak))
    assert np.allclose(o, ref[0].numpy(), rtol=1e-11, atol=1e-12)
    for got, want in zip(grads, ref[1:]):
        assert np.allclose(got, want.numpy(), rtol=1e-10, atol=1e-12)


def test_torch_restatement_gradcheck():
    g = oracle.BinaryPartition(9, False, 1, 10)
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    gen = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(n, 2, 3, dtype=torch.float64, generator=gen, requires_grad=True) for _ in range(3))
    s, d_ = torch.tensor(src), torch.tensor(dst)
    assert torch.autograd.gradcheck(lambda a, b, c: torch_ops.attention(s, d_, a, b, c), (q, k, v), atol=1e-7)


def test_tiny_brute_force():
    """3 nodes, edges 0->2, 1->2, 2->2, 0->1: softmax/attention by hand in Python floats."""
    import math
    src = np.array([0, 1, 2, 0]); dst = np.array([2, 2, 2, 1])
    q = np.array([[[1.0, 2.0]], [[0.5, -1.0]], [[-1.0, 0.25]]])
    k = np.array([[[0.3, 0.1]], [[-0.2, 0.4]], [[1.0, 1.0]]])
    v = np.array([[[1.0, 0.0]], [[0.0, 1.0]], [[2.0, 2.0]]])
    csr = oracle.get_csrs(src, dst, 3)
    o, a = oracle.attention_forward(csr, q, k, v)
    s = [sum(k[src[e], 0, i] * q[dst[e], 0, i] for i in range(2)) / math.sqrt(2) for e in range(4)]
    z2 = sum(math.exp(s[e]) for e in (0, 1, 2))
    want_a = [math.exp(s[0]) / z2, math.exp(s[1]) / z2, math.exp(s[2]) / z2, 1.0]
    assert np.allclose(a[:, 0], want_a)
    assert np.allclose(o[2, 0], sum(want_a[e] * v[src[e], 0] for e in (0, 1, 2)))
    assert np.allclose(o[1, 0], v[0, 0]) and np.all(o[0] == 0)


def test_f32_matches_f64():
    rng = np.random.default_rng(3)
    g = oracle.BinaryPartition(64, True, 4, 10)
    src, dst, _ = g.get_edges()
    n = g.number_of_nodes
    csr = oracle.get_csrs(src, dst, n)
    q, k, v, do = (rand(rng, n, 2, 16) / 4 for _ in range(4))
    o64, a64 = oracle.attention_forward(csr, q, k, v)
    f = lambda z: z.astype(np.float32)
    o32, a32 = oracle.attention_forward(csr, f(q), f(k), f(v))
    assert o32.dtype == np.float32 and np.allclose(o32, o64, rtol=1e-5, atol=1e-5)
    g64 = oracle.attention_backward(csr, q, k, v, a64, do)
    g32 = oracle.attention_backward(csr, f(q), f(k), f(v), a32, f(do))
    for x32, x64 in zip(g32, g64):
        assert np.allclose(x32, x64, rtol=1e-4, atol=1e-5)
