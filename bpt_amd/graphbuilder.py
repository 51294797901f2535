"""Host graph builder with the API of the reference's Cython module `graphbuilder`
(graph_builder/builder.pyx): `BinaryPartition`, `FullyConnected`, `OpenAISparse`, `partition_csr`,
backed by libbptgraph (C++).  Arrays are numpy int64 exactly as `np.asarray(vector) + v_shift`
yields there.  Also provides what graph/base.py:71-86 and graph/lm.py:53-98 obtain through DGL and
scipy: `build_csr`, `get_csrs`, `merge_graphs`.
"""
import ctypes

import numpy as np

from ._lib import check_graph, graph_lib

__all__ = ["BinaryPartition", "FullyConnected", "OpenAISparse", "partition_csr",
           "build_csr", "get_csrs", "merge_graphs", "get_csrs_device", "merge_graphs_device",
           "inter_graph_edges", "nli_inter_graph_edges", "get_csrs_bipartite"]


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


class _Graph:
    _kind = -1

    def _init(self, length, triu, a, b):
        lib = graph_lib()
        self._length, self._triu, self._a, self._b = int(length), bool(triu), int(a), int(b)
        n, e, lv = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
        check_graph(lib.bptg_graph_sizes(self._kind, self._length, int(self._triu), self._a, self._b,
                                         ctypes.byref(n), ctypes.byref(e), ctypes.byref(lv)))
        self._n_nodes, self._n_edges, self._n_lvl = n.value, e.value, lv.value
        self._lvl_sizes = np.empty(self._n_lvl, dtype=np.int64)
        check_graph(lib.bptg_graph_fill(self._kind, self._length, int(self._triu), self._a, self._b, 0,
                                        None, None, None, None, _ptr(self._lvl_sizes)))

    # builder.pyx:118-132
    @property
    def number_of_nodes(self):
        return self._n_nodes

    @property
    def number_of_edges(self):
        return self._n_edges

    @property
    def is_triu(self):
        return self._triu

    # builder.pyx:134
    def get_pos(self):
        pos = np.empty(self._n_nodes, dtype=np.int64)
        check_graph(graph_lib().bptg_graph_fill(self._kind, self._length, int(self._triu), self._a, self._b, 0,
                                                None, None, None, _ptr(pos), None))
        return pos

    # builder.pyx:137-140
    def get_edges(self, v_shift=0):
        src, dst, et = (np.empty(self._n_edges, dtype=np.int64) for _ in range(3))
        check_graph(graph_lib().bptg_graph_fill(self._kind, self._length, int(self._triu), self._a, self._b, int(v_shift),
                                                _ptr(src), _ptr(dst), _ptr(et), None, None))
        return src, dst, et

    def get_edges_device(self, device, v_shift=0):
        """get_edges built on the GPU (libbptplan: one thread per token, count / prefix sum / write): int64 device
        tensors (src, dst, etype), bit for bit the arrays of get_edges.  One synchronisation (the edge count)."""
        import torch
        from ._lib import plan_lib
        lib, device = plan_lib(), torch.device(device)
        L = self._length
        offsets = torch.empty(L + 1, dtype=torch.int32, device=device)
        ws = torch.empty(8 * (L + 1) + (1 << 20), dtype=torch.uint8, device=device)
        with torch.cuda.device(device):
            stream = torch.cuda.current_stream().cuda_stream
            st = lib.bpt_graph_count_device(self._kind, L, int(self._triu), self._a, self._b, offsets.data_ptr(),
                                            ws.data_ptr(), ws.numel(), stream)
            if st != 0:
                raise RuntimeError(f"bpt_graph_count_device: status {st}")
            n_edges = int(offsets[L])
            if n_edges != self._n_edges:
                raise RuntimeError("device and host edge counts differ")
            src, dst, et = (torch.empty(n_edges, dtype=torch.int64, device=device) for _ in range(3))
            st = lib.bpt_graph_fill_device(self._kind, L, int(self._triu), self._a, self._b, int(v_shift),
                                           offsets.data_ptr(), n_edges, src.data_ptr(), dst.data_ptr(), et.data_ptr(), stream)
            if st != 0:
                raise RuntimeError(f"bpt_graph_fill_device: status {st}")
        return src, dst, et

    # builder.pyx:142-149
    def leaf_ids(self, v_shift=0, start=0):
        return np.arange(v_shift + start, v_shift + self._length)

    def internal_ids(self, v_shift=0):
        return np.arange(v_shift + self._length, v_shift + self._n_nodes)

    def root_id(self, v_shift=0):
        return v_shift + self._n_nodes - 1


class BinaryPartition(_Graph):
    """builder.pyx:23-152."""
    _kind = 0

    def __init__(self, length, triu=False, step=1, clip_dist=10):
        self._init(length, triu, step, clip_dist)

    def __reduce__(self):
        return BinaryPartition, (self._length, self._triu, self._a, self._b)

    @property
    def number_of_levels(self):
        return self._n_lvl

    def number_of_nodes_at_lvl(self, i):
        return int(self._lvl_sizes[i])


class FullyConnected(_Graph):
    """builder.pyx:228-303."""
    _kind = 1

    def __init__(self, length, triu=False, window=8192):
        self._init(length, triu, window, 0)

    def __reduce__(self):
        return FullyConnected, (self._length, self._triu, self._a)


class OpenAISparse(_Graph):
    """builder.pyx:154-225."""
    _kind = 2

    def __init__(self, length, stride, c, triu=True):
        assert triu, "bidirectional model is not supported"
        self._init(length, triu, stride, c)

    def __reduce__(self):
        return OpenAISparse, (self._length, self._a, self._b, self._triu)


def partition_csr(indptr, chunk_size=32):
    """builder.pyx:305-321: (row, indptr_) of the chunked units, int64 numpy."""
    indptr = np.ascontiguousarray(indptr, dtype=np.int64)
    lib = graph_lib()
    n = ctypes.c_int64()
    check_graph(lib.bptg_partition_csr_count(_ptr(indptr), len(indptr), int(chunk_size), ctypes.byref(n)))
    row = np.empty(n.value, dtype=np.int64)
    units = np.empty(n.value + 1, dtype=np.int64)
    check_graph(lib.bptg_partition_csr_fill(_ptr(indptr), len(indptr), int(chunk_size), _ptr(row), _ptr(units)))
    return row, units


def build_csr(rows, cols, n_nodes):
    """(indptr, indices, eid) of the edge list grouped by `rows`; ascending edge id inside a row."""
    rows = np.ascontiguousarray(rows, dtype=np.int64)
    cols = np.ascontiguousarray(cols, dtype=np.int64)
    if rows.shape != cols.shape:
        raise ValueError("rows and cols must have the same length")
    indptr = np.empty(n_nodes + 1, dtype=np.int64)
    indices = np.empty(len(rows), dtype=np.int64)
    eid = np.empty(len(rows), dtype=np.int64)
    check_graph(graph_lib().bptg_build_csr(_ptr(rows), _ptr(cols), len(rows), int(n_nodes),
                                           _ptr(indptr), _ptr(indices), _ptr(eid)))
    return indptr, indices, eid


def get_csrs(src, dst, n_nodes, chunk_size=32, as_torch=True, in_order="eid"):
    """Replacement of graph/base.py:71-86 without DGL: returns
    (out_csr, in_csr, ROW, INDPTR_R, COL, INDPTR_C) with csr = (indptr, indices, eid), all int64
    (torch CPU tensors by default, numpy with as_torch=False).

    The reference takes both CSRs from DGL 0.4 (`adjacency_matrix_scipy`), which fixes `indptr` and the set of
    (index, edge id) pairs of every row but whose order INSIDE a row is not specified by anything in the reference.
    in_order picks it for the in-CSR: "eid" (default) = ascending edge id, the order of a stable counting sort of the
    edge list by destination; "src_eid" = ascending (source, edge id), the order a transpose of the out-CSR gives.
    The out-CSR is in ascending edge id either way.  Every op result is the same for both up to float rounding, and
    edge-addressed results do not depend on it at all."""
    if in_order not in ("eid", "src_eid"):
        raise ValueError('in_order must be "eid" or "src_eid"')
    out_csr = build_csr(src, dst, n_nodes)
    in_csr = build_csr(dst, src, n_nodes)
    if in_order == "src_eid":
        indptr, indices, eid = in_csr
        row_of_slot = np.repeat(np.arange(n_nodes, dtype=np.int64), np.diff(indptr))
        order = np.lexsort((eid, indices, row_of_slot))
        in_csr = (indptr, np.ascontiguousarray(indices[order]), np.ascontiguousarray(eid[order]))
    ROW, INDPTR_R = partition_csr(out_csr[0], chunk_size)
    COL, INDPTR_C = partition_csr(in_csr[0], chunk_size)
    res = (out_csr, in_csr, ROW, INDPTR_R, COL, INDPTR_C)
    if as_torch:
        import torch
        t = torch.from_numpy
        res = (tuple(map(t, out_csr)), tuple(map(t, in_csr)), t(ROW), t(INDPTR_R), t(COL), t(INDPTR_C))
    return res


def get_csrs_bipartite(src, dst, n_src, n_dst, chunk_size=32, as_torch=True):
    """get_csrs for a bipartite graph whose two sides have index spaces of their own (sources 0 .. n_src - 1, the
    keys / values of an attention to memory; destinations 0 .. n_dst - 1, its queries): the out-CSR has n_src rows,
    the in-CSR n_dst.  The reference stores such a graph in one square index space of max(n_src, n_dst) nodes
    (graph/mt.py:340-344) and pads the shorter node tensor (modules/attention.py:148-149); get_csrs(src, dst,
    max(n_src, n_dst)) gives that form, and the ops accept both."""
    src = np.ascontiguousarray(src, dtype=np.int64)
    dst = np.ascontiguousarray(dst, dtype=np.int64)
    if src.shape != dst.shape or src.ndim != 1:
        raise ValueError("src and dst must be 1-D arrays of the same length")
    if len(src) and (src.min() < 0 or dst.min() < 0 or src.max() >= n_src or dst.max() >= n_dst):
        raise ValueError("node id out of range")

    def side(rows, cols, n_rows):          # stable sort by row = ascending edge id inside a row, as build_csr
        eid = np.argsort(rows, kind="stable").astype(np.int64)
        indptr = np.zeros(n_rows + 1, dtype=np.int64)
        np.cumsum(np.bincount(rows, minlength=n_rows), out=indptr[1:])
        return indptr, np.ascontiguousarray(cols[eid]), eid

    out_csr = side(src, dst, int(n_src))
    in_csr = side(dst, src, int(n_dst))
    ROW, INDPTR_R = partition_csr(out_csr[0], chunk_size)
    COL, INDPTR_C = partition_csr(in_csr[0], chunk_size)
    res = (out_csr, in_csr, ROW, INDPTR_R, COL, INDPTR_C)
    if as_torch:
        import torch
        t = torch.from_numpy
        res = (tuple(map(t, out_csr)), tuple(map(t, in_csr)), t(ROW), t(INDPTR_R), t(COL), t(INDPTR_C))
    return res


def _segments(seg, length):
    seg = [0, length] if seg is None else [int(x) for x in seg]
    if len(seg) < 2 or seg[0] < 0 or seg[-1] > length or any(b < a for a, b in zip(seg, seg[1:])):
        raise ValueError("segment boundaries must be non-decreasing positions inside the sequence")
    return seg


def inter_graph_edges(enc_graphs, dec_graphs, enc_segments=None, dec_segments=None):
    """Edges of the encoder -> decoder graph of a batch of sequence pairs, graph/mt.py:286-321: for pair b and
    segment i, every token (leaf node) of the source sentence's segment i is connected to every token of the target
    sentence's segment i; node ids are those of the merged encoder graph (sources) and of the merged decoder graph
    (destinations), i.e. the sequences' leaf ids shifted by the node counts of the graphs before them.
    enc_segments / dec_segments: per pair a list of boundaries [s_0, s_1, ...] (segment i = tokens s_i .. s_{i+1} - 1),
    or None for one segment covering the whole sentence (mt.py:260-262).
    Returns (src, dst, n_enc, n_dec): int64 edge list in the reference's order and the two node counts; the
    reference's square form is get_csrs(src, dst, max(n_enc, n_dec)) (mt.py:340-344)."""
    if len(enc_graphs) != len(dec_graphs):
        raise ValueError("one encoder graph per decoder graph")
    enc_segments = enc_segments or [None] * len(enc_graphs)
    dec_segments = dec_segments or [None] * len(dec_graphs)
    rows, cols, ve, vd = [], [], 0, 0
    for ge, gd, se, sd in zip(enc_graphs, dec_graphs, enc_segments, dec_segments):
        se, sd = _segments(se, len(ge.leaf_ids())), _segments(sd, len(gd.leaf_ids()))
        if len(se) != len(sd):
            raise ValueError("source and target must have the same number of segments")
        for i in range(1, len(se)):
            a = np.arange(ve + se[i - 1], ve + se[i], dtype=np.int64)
            b = np.arange(vd + sd[i - 1], vd + sd[i], dtype=np.int64)
            rows.append(np.repeat(a, len(b)))
            cols.append(np.tile(b, len(a)))
        ve += ge.number_of_nodes
        vd += gd.number_of_nodes
    cat = lambda xs: np.concatenate(xs) if xs else np.empty(0, dtype=np.int64)
    return cat(rows), cat(cols), ve, vd


def nli_inter_graph_edges(premise_graphs, hypo_graphs):
    """Edges of the inter graph of graph/nli.py:60-99: premise and hypothesis of a pair are laid out one after the other
    in ONE node index space; every premise token is connected to every hypothesis token and back.
    Returns (src, dst, n_nodes)."""
    if len(premise_graphs) != len(hypo_graphs):
        raise ValueError("one premise graph per hypothesis graph")
    rows, cols, v = [], [], 0
    for gp, gh in zip(premise_graphs, hypo_graphs):
        a = gp.leaf_ids(v_shift=v).astype(np.int64)
        v += gp.number_of_nodes
        b = gh.leaf_ids(v_shift=v).astype(np.int64)
        v += gh.number_of_nodes
        rows += [np.repeat(a, len(b)), np.repeat(b, len(a))]
        cols += [np.tile(b, len(a)), np.tile(a, len(b))]
    cat = lambda xs: np.concatenate(xs) if xs else np.empty(0, dtype=np.int64)
    return cat(rows), cat(cols), v


def get_csrs_device(src, dst, n_nodes, chunk_size=32):
    """get_csrs for an edge list that already lives on the GPU (int64 CUDA tensors): the same 6-tuple, built there by
    libbptplan (bpt_csr_build_device: a stable radix sort by row, binary searches, a prefix sum) and bit for bit what
    get_csrs returns for the same edges.  One synchronisation (the number of units of each side comes back)."""
    import torch
    from ._lib import plan_lib
    if not (src.is_cuda and dst.is_cuda and src.dtype == torch.int64 and dst.dtype == torch.int64):
        raise ValueError("src and dst must be int64 CUDA tensors")
    if src.shape != dst.shape or src.dim() != 1:
        raise ValueError("src and dst must be 1-D tensors of the same length")
    src, dst = src.contiguous(), dst.contiguous()
    lib, E, n, dev = plan_lib(), int(src.numel()), int(n_nodes), src.device
    b = (ctypes.c_int64 * 2)()
    st = lib.bpt_csr_device_bounds(E, n, int(chunk_size), ctypes.byref(b))
    if st != 0:
        raise RuntimeError(f"bpt_csr_device_bounds: status {st}")
    i64 = lambda k: torch.empty(max(k, 1), dtype=torch.int64, device=dev)
    sides = []
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream().cuda_stream
        for rows, cols in ((src, dst), (dst, src)):
            indptr, indices, eid = i64(n + 1), i64(E), i64(E)
            unit_row, unit_ptr = i64(int(b[0])), i64(int(b[0]) + 1)
            info = torch.empty(16, dtype=torch.int32, device=dev)
            ws = torch.empty(int(b[1]), dtype=torch.uint8, device=dev)
            st = lib.bpt_csr_build_device(rows.data_ptr() if E else None, cols.data_ptr() if E else None, E, n,
                                          int(chunk_size), indptr.data_ptr(), indices.data_ptr(), eid.data_ptr(),
                                          unit_row.data_ptr(), unit_ptr.data_ptr(), info.data_ptr(), ws.data_ptr(),
                                          ws.numel(), stream)
            if st != 0:
                raise RuntimeError(f"bpt_csr_build_device: status {st}")
            sides.append((indptr, indices[:E], eid[:E], unit_row, unit_ptr, info))
    out = []
    for indptr, indices, eid, unit_row, unit_ptr, info in sides:
        err, n_units = info[:2].tolist()
        if err:
            raise ValueError("bptplan: row id, column id or edge id out of range")
        out.append(((indptr, indices, eid), unit_row[:n_units].clone(), unit_ptr[:n_units + 1].clone()))
    (out_csr, ROW, INDPTR_R), (in_csr, COL, INDPTR_C) = out
    return out_csr, in_csr, ROW, INDPTR_R, COL, INDPTR_C


def merge_graphs(graphs):
    """Block-diagonal batch merge of graph/lm.py:53-98 / graph/text_classification.py:30-67:
    returns (src, dst, etype, pos, n_nodes); the edge id of an edge is its position."""
    v_shift = 0
    src, dst, et, pos = [], [], [], []
    for g in graphs:
        s, d, e = g.get_edges(v_shift=v_shift)
        src.append(s); dst.append(d); et.append(e); pos.append(g.get_pos())
        v_shift += g.number_of_nodes
    cat = np.concatenate
    return cat(src), cat(dst), cat(et), cat(pos), v_shift


_DEVICE_EDGES = {}           # (graph class, constructor arguments, device) -> (src, dst, etype, pos) device tensors
_DEVICE_EDGES_MAX = 4096


def merge_graphs_device(graphs, device):
    """merge_graphs with the result on the GPU: the edge lists of the single graphs are kept on the device per
    (class, length, ...) the way the reference caches them on the host (graph/base.py:12-26), and a batch is their
    concatenation plus the node shifts (graph/lm.py:83-98), formed there; only the shifts and counts of the batch
    (one number per graph) cross the bus.  Returns int64 device tensors (src, dst, etype, pos) and n_nodes."""
    import torch
    device = torch.device(device)
    parts, shifts, v_shift = [], [], 0
    for g in graphs:
        key = (type(g).__name__,) + tuple(g.__reduce__()[1]) + (str(device),)
        hit = _DEVICE_EDGES.get(key)
        if hit is None:
            if len(_DEVICE_EDGES) >= _DEVICE_EDGES_MAX:
                _DEVICE_EDGES.clear()
            hit = (*g.get_edges_device(device), torch.from_numpy(g.get_pos()).to(device))
            _DEVICE_EDGES[key] = hit
        parts.append(hit)
        shifts.append(v_shift)
        v_shift += g.number_of_nodes
    if not parts:
        e = torch.empty(0, dtype=torch.int64, device=device)
        return e, e.clone(), e.clone(), e.clone(), 0
    counts = torch.tensor([p[0].numel() for p in parts], dtype=torch.int64)
    n_edges = int(counts.sum())
    shift = torch.repeat_interleave(torch.tensor(shifts, dtype=torch.int64).to(device), counts.to(device), output_size=n_edges)
    src = torch.cat([p[0] for p in parts]) + shift
    dst = torch.cat([p[1] for p in parts]) + shift
    return src, dst, torch.cat([p[2] for p in parts]), torch.cat([p[3] for p in parts]), v_shift
