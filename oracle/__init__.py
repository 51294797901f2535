"""TEST INFRASTRUCTURE — CPU oracle of the BPT graph-attention path (not the product).

Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import
this package, and only as the checker.  The product (``bpt_amd``) never imports it.

Contents
  * ctypes bindings of ``liboracle.so`` (``bpt_oracle.c``: C restatement of
    graph_builder/builder.pyx:41-116,171-199,243-274,305-321 and of the 13 kernels of
    graph_kernel/graphop_kernel.cu:19-230), numpy in / numpy out;
  * ``get_csrs``: out-/in-CSR with edge ids + chunked units, the layout of graph/base.py:71-86
    (stable counting sort by row, ties in ascending edge id — DGL's intra-row order is not
    available offline: **parity unpinned** for the order inside a row; indptr and each row's
    multiset of (index, eid) are order independent);
  * ``merge_graphs``: block-diagonal batch merge of graph/lm.py:53-98;
  * ``attention_forward`` / ``attention_backward``: the op sequence of
    modules/attention.py:66-77 and its reverse through modules/op.py:10-58.

Pinned by tests/test_oracle_graph.py (golden vectors from the reference's own builder) and
tests/test_oracle_ops.py (dense closed forms, brute force, invariants).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_i64p = ctypes.POINTER(ctypes.c_int64)


def build(force=False):
    """Compile liboracle.so with gcc (make)."""
    so = os.path.join(_HERE, "liboracle.so")
    if force and os.path.exists(so):
        os.remove(so)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            build()
        L = ctypes.CDLL(so)
        for name in ("oracle_binary_partition", "oracle_fully_connected", "oracle_openai_sparse"):
            getattr(L, name).restype = ctypes.c_void_p
        L.oracle_binary_partition.argtypes = [ctypes.c_size_t, ctypes.c_int, ctypes.c_size_t, ctypes.c_size_t]
        L.oracle_fully_connected.argtypes = [ctypes.c_size_t, ctypes.c_int, ctypes.c_size_t]
        L.oracle_openai_sparse.argtypes = [ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t]
        L.oracle_graph_free.argtypes = [ctypes.c_void_p]
        for name in ("oracle_graph_n_nodes", "oracle_graph_n_edges", "oracle_graph_n_levels"):
            getattr(L, name).restype = ctypes.c_size_t
            getattr(L, name).argtypes = [ctypes.c_void_p]
        L.oracle_graph_nodes_at_lvl.restype = ctypes.c_size_t
        L.oracle_graph_nodes_at_lvl.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
        L.oracle_graph_export.argtypes = [ctypes.c_void_p, ctypes.c_int64] + [ctypes.c_void_p] * 4
        L.oracle_partition_csr.restype = ctypes.c_int64
        L.oracle_partition_csr.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                           ctypes.c_void_p, ctypes.c_void_p]
        _LIB = L
    return _LIB


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _i64(a):
    return np.ascontiguousarray(np.asarray(a), dtype=np.int64)


# --------------------------------------------------------------------------------------------
# graphs
# --------------------------------------------------------------------------------------------
class _Graph:
    def __init__(self, handle):
        self._h = handle
        L = lib()
        self.number_of_nodes = L.oracle_graph_n_nodes(handle)
        self.number_of_edges = L.oracle_graph_n_edges(handle)
        self.number_of_levels = L.oracle_graph_n_levels(handle)

    def __del__(self):
        if getattr(self, "_h", None):
            lib().oracle_graph_free(self._h)
            self._h = None

    def get_edges(self, v_shift=0):
        E = self.number_of_edges
        src, dst, et = (np.empty(E, dtype=np.int64) for _ in range(3))
        lib().oracle_graph_export(self._h, v_shift, _p(src), _p(dst), _p(et), None)
        return src, dst, et

    def get_pos(self):
        pos = np.empty(self.number_of_nodes, dtype=np.int64)
        lib().oracle_graph_export(self._h, 0, None, None, None, _p(pos))
        return pos

    def number_of_nodes_at_lvl(self, i):
        return lib().oracle_graph_nodes_at_lvl(self._h, i)

    # builder.pyx:142-149
    def leaf_ids(self, v_shift=0, start=0):
        return np.arange(v_shift + start, v_shift + self.number_of_nodes_at_lvl(0))

    def internal_ids(self, v_shift=0):
        return np.arange(v_shift + self.number_of_nodes_at_lvl(0), v_shift + self.number_of_nodes)

    def root_id(self, v_shift=0):
        return v_shift + self.number_of_nodes - 1


class BinaryPartition(_Graph):
    def __init__(self, length, triu=False, step=1, clip_dist=10):
        super().__init__(lib().oracle_binary_partition(length, int(triu), step, clip_dist))


class FullyConnected(_Graph):
    def __init__(self, length, triu=False, window=8192):
        super().__init__(lib().oracle_fully_connected(length, int(triu), window))


class OpenAISparse(_Graph):
    def __init__(self, length, stride, c, triu=True):
        assert triu
        super().__init__(lib().oracle_openai_sparse(length, stride, c))


def partition_csr(indptr, chunk_size=32):
    indptr = _i64(indptr)
    n = lib().oracle_partition_csr(_p(indptr), len(indptr), chunk_size, None, None)
    row = np.empty(n, dtype=np.int64)
    ip = np.empty(n + 1, dtype=np.int64)
    lib().oracle_partition_csr(_p(indptr), len(indptr), chunk_size, _p(row), _p(ip))
    return row, ip


def merge_graphs(graphs):
    """graph/lm.py:53-98: concatenate (src+v_shift, dst+v_shift, etype, pos); edge id = position."""
    v_shift = 0
    src, dst, et, pos = [], [], [], []
    for g in graphs:
        s, d, e = g.get_edges(v_shift=v_shift)
        src.append(s); dst.append(d); et.append(e); pos.append(g.get_pos())
        v_shift += g.number_of_nodes
    return (np.concatenate(src), np.concatenate(dst), np.concatenate(et), np.concatenate(pos), v_shift)


def _csr(rows, cols, n):
    order = np.argsort(rows, kind="stable")          # ties keep ascending edge id
    indptr = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(np.bincount(rows, minlength=n), out=indptr[1:])
    return indptr, cols[order].astype(np.int64), order.astype(np.int64)


def get_csrs(src, dst, n, chunk_size=32):
    """graph/base.py:71-86: (out_csr, in_csr, ROW, INDPTR_R, COL, INDPTR_C); csr = (indptr, indices, eid)."""
    src, dst = _i64(src), _i64(dst)
    out_csr = _csr(src, dst, n)
    in_csr = _csr(dst, src, n)
    ROW, INDPTR_R = partition_csr(out_csr[0], chunk_size)
    COL, INDPTR_C = partition_csr(in_csr[0], chunk_size)
    return out_csr, in_csr, ROW, INDPTR_R, COL, INDPTR_C


# --------------------------------------------------------------------------------------------
# ops (numpy float32 / float64; names and argument orders of graph_kernel/graphop.cpp:216-225)
# --------------------------------------------------------------------------------------------
def _suf(a):
    if a.dtype == np.float32:
        return "f32"
    if a.dtype == np.float64:
        return "f64"
    raise TypeError(a.dtype)


def _c(a):
    return np.ascontiguousarray(a)


def _hd(A):
    return (1, A.shape[-1]) if A.ndim == 2 else (A.shape[1], A.shape[2])


def _call(name, *args):
    fn = getattr(lib(), name)
    conv = []
    for a in args:
        if isinstance(a, np.ndarray):
            conv.append(_p(a))
        else:
            conv.append(ctypes.c_int64(int(a)))
    fn.restype = None
    fn(*conv)


def maskedmm_csr_forward(row, indptr, eid, indices, A, B):
    A, B = _c(A), _c(B)
    h, d = _hd(A)
    y = np.zeros((len(eid),) if A.ndim == 2 else (len(eid), h), dtype=A.dtype)
    _call("oracle_maskedmm_csr_forward_" + _suf(A), _i64(row), _i64(indptr), _i64(eid), _i64(indices),
          A, B, y, len(row), d, h)
    return y


def maskedmm_csr_backward(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, A, B, dy):
    A, B, dy = _c(A), _c(B), _c(dy)
    h, d = _hd(A)
    dA, dB = np.zeros_like(A), np.zeros_like(B)
    s = _suf(A)
    _call("oracle_maskedmm_csr_backward_side_" + s, _i64(row), _i64(indptr_r), _i64(eid_r), _i64(indices_r),
          B, dy, dA, len(row), d, h)
    _call("oracle_maskedmm_csr_backward_side_" + s, _i64(col), _i64(indptr_c), _i64(eid_c), _i64(indices_c),
          A, dy, dB, len(col), d, h)
    return dA, dB


def node_mul_edge_forward(row, indptr, eid, A, B):
    A, B = _c(A), _c(B)
    h, d = _hd(A)
    y = np.zeros((len(eid),) if A.ndim == 2 else (len(eid), h), dtype=A.dtype)
    _call("oracle_node_mul_edge_forward_" + _suf(A), _i64(row), _i64(indptr), _i64(eid), A, B, y, len(row), d, h)
    return y


def node_mul_edge_backward(row, indptr, eid, A, B, dy):
    A, B, dy = _c(A), _c(B), _c(dy)
    h, d = _hd(A)
    dA, dB = np.zeros_like(A), np.zeros_like(B)
    _call("oracle_node_mul_edge_backward_" + _suf(A), _i64(row), _i64(indptr), _i64(eid), A, B, dy, dA, dB,
          len(row), d, h)
    return dA, dB


def sparse_softmax_forward(row, indptr, eid, x, n_nodes=None):
    x = _c(x)
    h = 1 if x.ndim == 1 else x.shape[1]
    n_nodes = int(max(row) + 1) if n_nodes is None and len(row) else (n_nodes or 1)
    y = np.zeros_like(x)
    scratch = np.empty(2 * n_nodes * h, dtype=x.dtype)
    _call("oracle_sparse_softmax_forward_" + _suf(x), _i64(row), _i64(indptr), _i64(eid), x, y, scratch,
          len(row), n_nodes, h)
    return y


def sparse_softmax_backward(row, indptr, eid, y, dy, n_nodes=None):
    y, dy = _c(y), _c(dy)
    h = 1 if y.ndim == 1 else y.shape[1]
    n_nodes = int(max(row) + 1) if n_nodes is None and len(row) else (n_nodes or 1)
    dx = np.zeros_like(dy)
    scratch = np.empty(n_nodes * h, dtype=y.dtype)
    _call("oracle_sparse_softmax_backward_" + _suf(y), _i64(row), _i64(indptr), _i64(eid), y, dy, dx, scratch,
          len(row), n_nodes, h)
    return dx


def vector_spmm_forward(row, indptr, eid, indices, edata, x):
    edata, x = _c(edata), _c(x)
    h, d = _hd(x)
    y = np.zeros_like(x)
    _call("oracle_vector_spmm_forward_" + _suf(x), _i64(row), _i64(indptr), _i64(eid), _i64(indices), edata, x, y,
          len(row), d, h)
    return y


def vector_spmm_backward(row, indptr, eid, indices, col, indptr_t, eid_t, indices_t, edata, dy, x,
                         reference_grid=False):
    """reference_grid=True reproduces the reference's launch of the dx kernel with the row-side
    grid (graphop_kernel.cu:566,588): only min(len(row), len(col)) units contribute to dx."""
    edata, dy, x = _c(edata), _c(dy), _c(x)
    h, d = _hd(x)
    dedata, dx = np.zeros_like(edata), np.zeros_like(x)
    n_dx = min(len(row), len(col)) if reference_grid else len(col)
    _call("oracle_vector_spmm_backward_" + _suf(x), _i64(row), _i64(indptr), _i64(eid), _i64(indices),
          _i64(col), _i64(indptr_t), _i64(eid_t), _i64(indices_t), edata, dy, x, dedata, dx,
          len(row), n_dx, d, h)
    return dedata, dx


# --------------------------------------------------------------------------------------------
# one attention layer = modules/attention.py:66-77 (dropout off), backward via modules/op.py
# --------------------------------------------------------------------------------------------
def attention_forward(csr, q, k, v, ak=None):
    """csr as returned by get_csrs.  ak: optional per-edge rel-pos rows (E, D).
    Returns (o, saved) with saved = (e_scaled, a) needed by attention_backward."""
    out_csr, in_csr, ROW, INDPTR_R, COL, INDPTR_C = csr
    d_k = q.shape[-1]
    e = maskedmm_csr_forward(ROW, INDPTR_R, out_csr[2], out_csr[1], k, q)
    if ak is not None:
        e = e + node_mul_edge_forward(COL, INDPTR_C, in_csr[2], q, ak)
    x = (e / np.sqrt(d_k)).astype(q.dtype)
    a = sparse_softmax_forward(COL, INDPTR_C, in_csr[2], x, n_nodes=q.shape[0])
    o = vector_spmm_forward(COL, INDPTR_C, in_csr[2], in_csr[1], a, v)
    return o, a


def attention_backward(csr, q, k, v, a, do, ak=None):
    """Returns (dq, dk, dv[, dak])."""
    out_csr, in_csr, ROW, INDPTR_R, COL, INDPTR_C = csr
    d_k = q.shape[-1]
    da, dv = vector_spmm_backward(COL, INDPTR_C, in_csr[2], in_csr[1], ROW, INDPTR_R, out_csr[2], out_csr[1],
                                  a, do, v)
    dx = sparse_softmax_backward(COL, INDPTR_C, in_csr[2], a, da, n_nodes=q.shape[0])
    de = (dx / np.sqrt(d_k)).astype(q.dtype)
    dk, dq = maskedmm_csr_backward(ROW, INDPTR_R, out_csr[2], out_csr[1], COL, INDPTR_C, in_csr[2], in_csr[1],
                                   k, q, de)
    if ak is not None:
        dq_rel, dak = node_mul_edge_backward(COL, INDPTR_C, in_csr[2], q, ak, de)
        return dq + dq_rel, dk, dv, dak
    return dq, dk, dv
