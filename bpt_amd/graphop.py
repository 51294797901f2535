"""The `graphop` operator surface of the reference (graph_kernel/graphop.cpp:216-225) on MI355X.

Same eight names, positional argument orders and return arities as the pybind module that
modules/op.py imports with `from graphop import *`; each call validates its tensors like the
reference shim (graphop.cpp:4-6: CUDA + contiguous), looks up the launch plan of its index
tensors and enqueues HIP kernels from libbptattn on the current stream.  Nothing here computes on
the CPU; without the built HIP library the import fails.

Beyond the reference: bf16 tensors are accepted, `attention_forward/backward` expose the fused
SDDMM -> edge-softmax -> SpMM pass, and vector_spmm_backward returns the complete dx (the
reference's launch drops trailing units of the transposed side, graphop_kernel.cu:566,588).
"""
import collections
import contextlib
import ctypes
import math
import threading

import torch

from ._lib import BPT_ERR_UNSUPPORTED, BptStatusError, PlanStruct, attn_lib, check_attn
from . import plan as _plan
from .plan import GROUP_ORDER_SRC, TILE_GROUP_R, plan_cache

__all__ = ["maskedmm_csr_forward", "maskedmm_csr_backward", "node_mul_edge_forward", "node_mul_edge_backward",
           "sparse_softmax_forward", "sparse_softmax_backward", "vector_spmm_forward", "vector_spmm_backward"]

_LIB = attn_lib()          # fail at import time if the HIP library is missing


class _Settings(collections.namedtuple("_Settings", "use_groups grouped_ops group_rows use_tiles")):
    """Which kernel family the ops take: use_groups (fused attention: one wavefront per group of rows that share
    neighbours, or per row), grouped_ops (the same for the unfused SpMM / SDDMM ops), group_rows (None: chosen per call
    from dtype and shape; 4 or 8: forced), use_tiles (fused attention on dense 16 x 16 tiles where they exist).  Immutable: the set_* hooks below replace the whole tuple under a lock, and
    every op reads it ONCE on entry, so a call (forward on the Python thread, backward on autograd's) works with one
    consistent set even if another thread flips a hook meanwhile.  The hooks are process-wide testing / measurement
    aids, not per-thread state; every family computes the same results."""
    __slots__ = ()


_SETTINGS = _Settings(True, True, None, True)
_SETTINGS_LOCK = threading.Lock()


def _replace_setting(**kw):
    global _SETTINGS
    with _SETTINGS_LOCK:
        old = _SETTINGS
        _SETTINGS = old._replace(**kw)
    return old

_DTYPE = {torch.float32: 0, torch.float64: 1, torch.bfloat16: 2}
OP_MASKEDMM_BWD, OP_NME_BWD, OP_SPMM_FWD, OP_SPMM_BWD, OP_ATTN_FWD, OP_ATTN_BWD, OP_SOFTMAX_FWD, OP_SOFTMAX_BWD = 1, 2, 3, 4, 5, 6, 7, 8


def _check_input(t, name):
    # graphop.cpp:4-6
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _check_all(**tensors):
    for name, t in tensors.items():
        _check_input(t, name)


def _dtype(t):
    try:
        return _DTYPE[t.dtype]
    except KeyError:
        raise RuntimeError(f"unsupported dtype {t.dtype}: float32, float64 and bfloat16 are implemented") from None


def _hd(A):
    # graphop_kernel.cu:245-247: (n, d) means a single head
    if A.dim() == 2:
        return 1, A.size(1)
    if A.dim() == 3:
        return A.size(1), A.size(2)
    raise RuntimeError("node tensors must be (n, d) or (n, h, d)")


def _edge_h(x):
    return 1 if x.dim() == 1 else x.size(1)


def _same_dtype(*ts):
    for t in ts[1:]:
        if t.dtype != ts[0].dtype:
            raise RuntimeError("all floating point arguments must share one dtype")
        if t.device != ts[0].device:
            raise ValueError("all tensors of a call must be on one device")


# The kernels take raw pointers and trust the sizes of the plan, so every tensor's shape is checked here, before
# anything is launched: a mismatch raises ValueError instead of reading or writing out of bounds on the GPU.
def _expect_shape(t, shape, name):
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")


def _expect_edges(t, n_edges, h, name, two_d_node):
    """Edge tensors are (E,) next to (n, d) node tensors and (E, h) next to (n, h, d) ones (graphop_kernel.cu:247-248)."""
    if h == 1 and tuple(t.shape) in ((n_edges,), (n_edges, 1)):
        return                                   # one head: the two spellings are the same memory
    _expect_shape(t, (n_edges,) if two_d_node else (n_edges, h), name)


def _expect_index(eid, indices):
    if eid.dim() != 1 or (indices is not None and tuple(indices.shape) != tuple(eid.shape)):
        raise ValueError("eid and indices must be 1-D tensors of the same length")


# The per-call host work counts on small graphs, where a step's kernels take tens of microseconds: the current stream and
# device come from torch's raw accessors (a fraction of a microsecond; torch.cuda.current_stream() builds a Stream object,
# about 10 us a call), and the device guard is entered only when the tensors live on another device than the current one.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _current_device():
    return _raw_device() if _raw_device is not None else torch.cuda.current_device()


def _stream_handle(index=None):
    """The current stream of the device (default: the current device) as an integer handle."""
    if _raw_stream is not None:
        return _raw_stream(_current_device() if index is None else index)
    return torch.cuda.current_stream(index).cuda_stream


def _stream():
    return ctypes.c_void_p(_stream_handle())


_NO_GUARD = contextlib.nullcontext()


def _on_device_of(t):
    """Context in which t's device is the current one (what the kernels launch on and the raw stream accessor reads)."""
    return _NO_GUARD if t.device.index == _current_device() else torch.cuda.device_of(t)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None and t.numel() else None


def _workspace(op, plan, plan_t, h, d, dt, device, plan_ref=None, plan_t_ref=None):
    if plan_t_ref is None and plan_t is not None:
        plan_t_ref = plan_t.ref
    n = _LIB.bpt_workspace_bytes(op, plan.ref if plan_ref is None else plan_ref, plan_t_ref, h, d, dt)
    if n < 0:
        raise RuntimeError("bpt_workspace_bytes failed")
    if n == 0:
        return None, 0
    return _scratch(n, device), n


# Workspaces are kept per (device, stream) and grown on demand: calls on one stream are ordered, so the next call may
# overwrite what the previous one left there, and a step no longer asks the allocator for tens of MB per call (after
# torch.cuda.empty_cache() such requests were measured at 0.16 ms each, GPU idle).  Under stream capture the buffer comes
# from the capture's own pool as before.  release_workspaces() gives the memory back.
_SCRATCH = {}
_SCRATCH_LOCK = threading.Lock()
KEEP_WORKSPACES = True


def _scratch(n, device):
    if not KEEP_WORKSPACES or torch.cuda.is_current_stream_capturing():
        return torch.empty(n, dtype=torch.uint8, device=device)
    index = device.index if device.index is not None else _current_device()
    key = (index, _stream_handle(index))
    with _SCRATCH_LOCK:
        buf = _SCRATCH.get(key)
        if buf is None or buf.numel() < n:
            buf = None
            _SCRATCH.pop(key, None)
            buf = torch.empty(max(n, 1 << 20), dtype=torch.uint8, device=device)
            _SCRATCH[key] = buf
    return buf


def release_workspaces():
    """Frees the workspaces kept for reuse (one per device and stream that ran an op with split rows or a fused backward)."""
    with _SCRATCH_LOCK:
        _SCRATCH.clear()


def _spmm_ref(plan, x, h, d, cfg):
    """The plan to hand a SpMM- or SDDMM-shaped op: with row groups (one load of a neighbour row per group entry instead of one
    per edge) where the row-group kernels apply, else the plain plan."""
    if not (cfg.use_groups and cfg.grouped_ops and attention_supported(x) and plan.covers_all_edges and plan.has_indices
            and plan.n_edges > 0 and max(plan.n_rows, plan.n_index_nodes) * h * d * x.element_size() < 2 ** 32):
        return plan.ref
    return ctypes.byref(plan.ensure_groups(_group_rows(x, h, d, plan, cfg), GROUP_ORDER_SRC)["struct"])


def _edge_out(plan, shape, like):
    # kernels write every edge id the plan covers; zero-fill only when some edge is not covered
    return (torch.empty if plan.covers_all_edges else torch.zeros)(shape, dtype=like.dtype, device=like.device)


def maskedmm_csr_forward(row, indptr, eid, indices, A, B):
    """y[eid[p]] = <A[row], B[indices[p]]> per head (graphop.cpp:16-31, graphop_kernel.cu:269-304)."""
    cfg = _SETTINGS
    _check_all(row=row, indptr=indptr, eid=eid, indices=indices, A=A, B=B)
    _same_dtype(A, B)
    h, d = _hd(A)
    _expect_index(eid, indices)
    _expect_shape(B, (B.size(0),) + tuple(A.shape[1:]), "B")
    plan = plan_cache.get(row, indptr, eid, indices, A.size(0), B.size(0))
    e = eid.size(0)
    y = _edge_out(plan, (e,) if A.dim() == 2 else (e, h), A)
    with _on_device_of(A):
        check_attn(_LIB.bpt_maskedmm_csr_forward(_spmm_ref(plan, A, h, d, cfg), _ptr(A), _ptr(B), _ptr(y), h, d, _dtype(A), _stream()),
                   "maskedmm_csr_forward")
    return y


def maskedmm_csr_backward(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, A, B, dy):
    """[dA, dB] (graphop.cpp:108-139, graphop_kernel.cu:355-409)."""
    cfg = _SETTINGS
    _check_all(row=row, indptr_r=indptr_r, eid_r=eid_r, indices_r=indices_r, col=col, indptr_c=indptr_c,
               eid_c=eid_c, indices_c=indices_c, A=A, B=B)
    dy = dy.contiguous()
    _same_dtype(A, B, dy)
    h, d = _hd(A)
    _expect_index(eid_r, indices_r)
    _expect_index(eid_c, indices_c)
    _expect_shape(B, (B.size(0),) + tuple(A.shape[1:]), "B")
    _expect_shape(eid_c, eid_r.shape, "eid_c")
    _expect_edges(dy, eid_r.size(0), h, "dy", A.dim() == 2)
    plan_r = plan_cache.get(row, indptr_r, eid_r, indices_r, A.size(0), B.size(0))
    plan_c = plan_cache.get(col, indptr_c, eid_c, indices_c, B.size(0), A.size(0))
    dA, dB = torch.empty_like(A), torch.empty_like(B)
    dt = _dtype(A)
    ws, nws = _workspace(OP_MASKEDMM_BWD, plan_r, plan_c, h, d, dt, A.device)
    with _on_device_of(A):
        check_attn(_LIB.bpt_maskedmm_csr_backward(_spmm_ref(plan_r, A, h, d, cfg), _spmm_ref(plan_c, A, h, d, cfg), _ptr(A), _ptr(B), _ptr(dy), _ptr(dA), _ptr(dB),
                                                  _ptr(ws), nws, h, d, dt, _stream()), "maskedmm_csr_backward")
    return [dA, dB]


def node_mul_edge_forward(row, indptr, eid, A, B):
    """y[eid[p], h] = <A[row, h], B[eid[p]]> with B (e, d) (graphop.cpp:39-51, graphop_kernel.cu:235-266)."""
    _check_all(row=row, indptr=indptr, eid=eid, A=A, B=B)
    _same_dtype(A, B)
    h, d = _hd(A)
    _expect_index(eid, None)
    _expect_shape(B, (eid.size(0), d), "B")
    plan = plan_cache.get(row, indptr, eid, None, A.size(0), None)
    e = eid.size(0)
    y = _edge_out(plan, (e,) if A.dim() == 2 else (e, h), A)
    with _on_device_of(A):
        check_attn(_LIB.bpt_node_mul_edge_forward(plan.ref, _ptr(A), _ptr(B), _ptr(y), h, d, _dtype(A), _stream()),
                   "node_mul_edge_forward")
    return y


def node_mul_edge_backward(row, indptr, eid, A, B, dy):
    """[dA, dB] (graphop.cpp:141-155, graphop_kernel.cu:306-351)."""
    _check_all(row=row, indptr=indptr, eid=eid, A=A, B=B)
    dy = dy.contiguous()
    _same_dtype(A, B, dy)
    h, d = _hd(A)
    _expect_index(eid, None)
    _expect_shape(B, (eid.size(0), d), "B")
    _expect_edges(dy, eid.size(0), h, "dy", A.dim() == 2)
    plan = plan_cache.get(row, indptr, eid, None, A.size(0), None)
    dA = torch.empty_like(A)
    dB = (torch.empty_like if plan.covers_all_edges else torch.zeros_like)(B)
    dt = _dtype(A)
    ws, nws = _workspace(OP_NME_BWD, plan, None, h, d, dt, A.device)
    with _on_device_of(A):
        check_attn(_LIB.bpt_node_mul_edge_backward(plan.ref, _ptr(A), _ptr(B), _ptr(dy), _ptr(dA), _ptr(dB),
                                                   _ptr(ws), nws, h, d, dt, _stream()), "node_mul_edge_backward")
    return [dA, dB]


def sparse_softmax_forward(row, indptr, eid, x):
    """softmax of x over the slots of each row (graphop.cpp:59-71, graphop_kernel.cu:411-463)."""
    _check_all(row=row, indptr=indptr, eid=eid, x=x)
    _expect_index(eid, None)
    if x.dim() not in (1, 2) or x.size(0) != eid.size(0):
        raise ValueError(f"x must be ({eid.size(0)},) or ({eid.size(0)}, h), got {tuple(x.shape)}")
    plan = plan_cache.get(row, indptr, eid, None, None, None)
    y = (torch.empty_like if plan.covers_all_edges else torch.zeros_like)(x)
    ws, nws = _workspace(OP_SOFTMAX_FWD, plan, None, _edge_h(x), 1, _dtype(x), x.device)
    with _on_device_of(x):
        check_attn(_LIB.bpt_sparse_softmax_forward(plan.ref, _ptr(x), _ptr(y), _ptr(ws), nws, _edge_h(x), _dtype(x), _stream()),
                   "sparse_softmax_forward")
    return y


def sparse_softmax_backward(row, indptr, eid, y, dy):
    """dx = y * (dy - sum_row dy*y) (graphop.cpp:163-177, graphop_kernel.cu:465-507)."""
    _check_all(row=row, indptr=indptr, eid=eid, y=y, dy=dy)
    _same_dtype(y, dy)
    _expect_index(eid, None)
    if y.dim() not in (1, 2) or y.size(0) != eid.size(0):
        raise ValueError(f"y must be ({eid.size(0)},) or ({eid.size(0)}, h), got {tuple(y.shape)}")
    _expect_shape(dy, y.shape, "dy")
    plan = plan_cache.get(row, indptr, eid, None, None, None)
    dx = (torch.empty_like if plan.covers_all_edges else torch.zeros_like)(dy)
    ws, nws = _workspace(OP_SOFTMAX_BWD, plan, None, _edge_h(dy), 1, _dtype(y), y.device)
    with _on_device_of(y):
        check_attn(_LIB.bpt_sparse_softmax_backward(plan.ref, _ptr(y), _ptr(dy), _ptr(dx), _ptr(ws), nws, _edge_h(dy), _dtype(y),
                                                    _stream()),
                   "sparse_softmax_backward")
    return dx


def vector_spmm_forward(row, indptr, eid, indices, edata, x, *, n_rows=None, out=None):
    """y[row] = sum_p edata[eid[p]] * x[indices[p]] (graphop.cpp:79-95, graphop_kernel.cu:509-542).

    n_rows (keyword only, not in the reference): number of rows of y when it differs from x.size(0) — a
    rectangular operator, used for the segment sums of the relative-position table's gradient.
    out (keyword only, not in the reference): a contiguous tensor of y's shape that the sum is ADDED to and that is
    returned (in the kernel's store where the row-group kernels apply, else by a separate addition)."""
    cfg = _SETTINGS
    _check_all(row=row, indptr=indptr, eid=eid, indices=indices, edata=edata, x=x)
    _same_dtype(edata, x)
    h, d = _hd(x)
    _expect_index(eid, indices)
    _expect_edges(edata, eid.size(0), h, "edata", x.dim() == 2)
    n_out = x.size(0) if n_rows is None else int(n_rows)
    plan = plan_cache.get(row, indptr, eid, indices, n_out, x.size(0))
    y = torch.empty_like(x) if n_rows is None else torch.empty((n_out,) + tuple(x.shape[1:]), dtype=x.dtype, device=x.device)
    dt = _dtype(x)
    ws, nws = _workspace(OP_SPMM_FWD, plan, None, h, d, dt, x.device)
    if out is not None and (out.shape != y.shape or out.dtype != y.dtype or out.device != y.device or not out.is_contiguous()):
        raise ValueError("out must be a contiguous tensor of the result's shape, dtype and device")
    with _on_device_of(x):
        ref = _spmm_ref(plan, x, h, d, cfg)
        if out is not None:
            st = _LIB.bpt_vector_spmm_accumulate(ref, _ptr(edata), _ptr(x), _ptr(out), _ptr(ws), nws, h, d, dt, _stream())
            if st == 0:
                return out
            if st != BPT_ERR_UNSUPPORTED:     # no row-group kernel for this call
                check_attn(st, "vector_spmm_accumulate")
        check_attn(_LIB.bpt_vector_spmm_forward(ref, _ptr(edata), _ptr(x), _ptr(y), _ptr(ws), nws, h, d, dt, _stream()),
                   "vector_spmm_forward")
    return y if out is None else out.add_(y)


def vector_spmm_backward(row, indptr, eid, indices, col, indptr_t, eid_t, indices_t, edata, dy, x):
    """[dedata, dx] (graphop.cpp:190-214, graphop_kernel.cu:544-600; dx over all units of the transposed side)."""
    cfg = _SETTINGS
    _check_all(row=row, indptr=indptr, eid=eid, indices=indices, col=col, indptr_t=indptr_t, eid_t=eid_t,
               indices_t=indices_t, edata=edata, x=x)
    dy = dy.contiguous()
    _same_dtype(edata, dy, x)
    h, d = _hd(x)
    _expect_index(eid, indices)
    _expect_index(eid_t, indices_t)
    _expect_shape(eid_t, eid.shape, "eid_t")
    _expect_edges(edata, eid.size(0), h, "edata", x.dim() == 2)
    # y = dy may have another number of rows than x (a rectangular operator: attention to a memory of another length)
    _expect_shape(dy, (dy.size(0),) + tuple(x.shape[1:]), "dy")
    plan = plan_cache.get(row, indptr, eid, indices, dy.size(0), x.size(0))
    plan_t = plan_cache.get(col, indptr_t, eid_t, indices_t, x.size(0), dy.size(0))
    dedata = (torch.empty_like if plan.covers_all_edges else torch.zeros_like)(edata)
    dx = torch.empty_like(x)
    dt = _dtype(x)
    ws, nws = _workspace(OP_SPMM_BWD, plan, plan_t, h, d, dt, x.device)
    with _on_device_of(x):
        check_attn(_LIB.bpt_vector_spmm_backward(_spmm_ref(plan, x, h, d, cfg), _spmm_ref(plan_t, x, h, d, cfg), _ptr(edata), _ptr(dy), _ptr(x), _ptr(dedata), _ptr(dx),
                                                 _ptr(ws), nws, h, d, dt, _stream()), "vector_spmm_backward")
    return [dedata, dx]


# ---- fused attention (no counterpart in the reference's extension) ---------------------------
def attention_supported(q):
    """True if the fused kernels have an instantiation for q's (h, d, dtype)."""
    h, d = _hd(q)
    fast = {torch.float32: {(4, 64), (8, 64), (16, 64), (8, 32)}, torch.bfloat16: {(8, 64), (16, 64)}}
    return q.dim() == 3 and (h, d) in fast.get(q.dtype, ())


def attention_padded_shape(q):
    """(h', 64) if the fused kernels can run q's (h, d, dtype) after zero-padding every head to 64 columns and the heads to the next
    compiled count (the reference's kernels take any d, graphop_kernel.cu:269-304; its configs use 6 x 50 and 8 x 40 beside 8 x 64),
    else None.  Zero columns add nothing to q.k, and a zero head (q = k = v = 0) gives a zero output row and zero gradients."""
    if q.dim() != 3 or q.dtype not in (torch.float32, torch.bfloat16) or attention_supported(q):
        return None
    h, d = _hd(q)
    if d > 64:
        return None
    heads = sorted(hh for hh, dd in {torch.float32: {(4, 64), (8, 64), (16, 64)}, torch.bfloat16: {(8, 64), (16, 64)}}[q.dtype] if hh >= h)
    return (heads[0], 64) if heads else None


def _by_pair(plan_struct):
    """A copy of a `bpt_plan` with bias_by_pair set: the per-edge term it reads or writes is (h, E), head-major."""
    st = PlanStruct.from_buffer_copy(plan_struct)
    st.bias_by_pair = 1
    return st


def rel_bias_forward(col, indptr_c, eid_c, type_slot, q, table, used_types=None, by_pair=False):
    """The rel_pos score term of modules/attention.py:69-71 without the (E, d) embedding rows:
    bias[eid_c[p], head] = q[row(p), head, :] . table[type(p), :] for every slot p of the in-CSR.  Returns float32
    (E + 1, h); the last row is a zero spare row that the fused kernels read for absent pairs.
    used_types None: type_slot[p] is the type of the edge in slot p (etype[eid_c]).
    used_types (n_used,) int32, the types that occur: type_slot[p] is the NUMBER of the slot's type in that list; takes the
    kernel that keeps those table rows on chip (needs rel_rows_supported(q) and n_used <= REL_MAX_USED_TYPES).
    by_pair (with used_types only): returns float32 (h, E) instead, bias[head, eid_c[p]], the form attention_forward takes
    with bias_by_pair=True when eid_c[p] is the number attention_pair_rows() gives the slot's edge."""
    cfg = _SETTINGS
    _check_all(col=col, indptr_c=indptr_c, eid_c=eid_c, type_slot=type_slot, q=q, table=table)
    _same_dtype(q, table)
    h, d = _hd(q)
    if table.dim() != 2 or table.size(1) != d:
        raise ValueError(f"table must be (n_types, {d})")
    _expect_index(eid_c, type_slot)
    E = eid_c.size(0)
    if used_types is not None:
        _check_input(used_types, "used_types")
        if used_types.dtype != torch.int32 or used_types.dim() != 1 or used_types.numel() > table.size(0):
            raise ValueError("used_types must be a 1-D int32 tensor of at most table.size(0) elements")
        # (only work items are walked, no row groups: the GPU builder's plan, 0.2 ms instead of 2 ms for a new graph of 16 K rows)
        plan = plan_cache.get(col, indptr_c, eid_c, type_slot, q.size(0), max(used_types.numel(), 1), prefer_device=True)
        ref, n_used = (ctypes.byref(_by_pair(plan.struct)) if by_pair else plan.ref), used_types.numel()
    else:
        if by_pair:
            raise ValueError("by_pair needs used_types")
        plan = plan_cache.get(col, indptr_c, eid_c, type_slot, q.size(0), table.size(0))
        ref, n_used = _spmm_ref(plan, q, h, d, cfg), 0
    bias = (torch.empty if plan.covers_all_edges else torch.zeros)((h, E) if by_pair else (E + 1, h), dtype=torch.float32, device=q.device)
    if not by_pair and (used_types is None or not plan.n_items):
        bias[E].zero_()                     # (the kernel of the other form clears the spare row itself)
    with _on_device_of(q):
        check_attn(_LIB.bpt_rel_bias_forward(ref, _ptr(q), _ptr(table), _ptr(used_types) if used_types is not None else None, n_used,
                                             _ptr(bias), h, d, _dtype(q), _stream()), "rel_bias_forward")
    return bias


REL_MAX_USED_TYPES = 240      # edge types that may occur in one graph for the kernels that keep their table rows on chip


def rel_rows_supported(q):
    """True if the rel_pos term of q's (h, d, dtype) has the kernels that keep the table rows in use on chip."""
    h, d = _hd(q)
    return q.dim() == 3 and d == 64 and h in (4, 8, 16) and q.dtype in (torch.float32, torch.bfloat16)


def rel_bias_backward_supported(q, n_used):
    """True if rel_bias_backward has a kernel configuration for n_used types in use on q's device (asked before the forward,
    so that a step never finds out in its backward that the gradient kernel does not fit)."""
    if not (rel_rows_supported(q) and n_used <= REL_MAX_USED_TYPES):
        return False
    h, d = _hd(q)
    with _on_device_of(q):
        return _LIB.bpt_rel_bias_backward_supported(int(n_used), h, d, _dtype(q)) == 0


def rel_bias_backward(col, indptr_c, eid_c, number_slot, used, used_types, ds, q, table, dq, by_pair=False):
    """Gradients of the rel_pos score term (modules/attention.py:55-56,69-71: autograd of nn.Embedding and of
    node_mul_edge) from ds (E or more rows, h) float32 = dL/d(score before scaling) per edge and head:
    dq[row] += sum_p ds[eid_c[p]] * table[type(p)] in place, and returns dtable (n_types, d) with
    dtable[t] = sum over the slots of type t and the heads of ds * q[row].  used_types (n_used,) int32: the types that
    occur; number_slot[p]: the number of slot p's type in that list; used (n_types,) int32: the number of every type
    in the list, -1 for the others.  by_pair: ds is (h, E), ds[head, eid_c[p]], as attention_backward returns it with
    bias_by_pair=True.  Raises if rel_rows_supported(q) is False or n_used > REL_MAX_USED_TYPES."""
    _check_all(col=col, indptr_c=indptr_c, eid_c=eid_c, number_slot=number_slot, used=used, used_types=used_types, ds=ds, q=q, table=table, dq=dq)
    _same_dtype(q, table, dq)
    h, d = _hd(q)
    if table.dim() != 2 or table.size(1) != d:
        raise ValueError(f"table must be (n_types, {d})")
    if used.dtype != torch.int32 or used.numel() != table.size(0):
        raise ValueError("used must be int32 with one element per table row")
    if used_types.dtype != torch.int32 or used_types.dim() != 1 or used_types.numel() > table.size(0):
        raise ValueError("used_types must be a 1-D int32 tensor of at most table.size(0) elements")
    if by_pair:
        if ds.dtype != torch.float32 or tuple(ds.shape) != (h, eid_c.size(0)):
            raise ValueError(f"ds must be float32 ({h}, {eid_c.size(0)})")
    elif ds.dtype != torch.float32 or ds.dim() != 2 or ds.size(1) != h or ds.size(0) < eid_c.size(0):
        raise ValueError(f"ds must be float32 (>= {eid_c.size(0)}, {h})")
    if dq.shape != q.shape:
        raise ValueError("dq must have the shape of q")
    _expect_index(eid_c, number_slot)
    n_used = used_types.numel()
    plan = plan_cache.get(col, indptr_c, eid_c, number_slot, q.size(0), max(n_used, 1), prefer_device=True)       # (as in rel_bias_forward)
    dtable = torch.empty_like(table)
    ref = ctypes.byref(_by_pair(plan.struct)) if by_pair else plan.ref
    with _on_device_of(q):
        nws = int(_LIB.bpt_rel_bias_backward_workspace_bytes(ref, n_used, h))
        ws = _scratch(max(nws, 16), q.device)
        check_attn(_LIB.bpt_rel_bias_backward(ref, _ptr(ds), _ptr(q), _ptr(table), _ptr(used), _ptr(used_types), table.size(0), n_used,
                                              _ptr(dq), _ptr(dtable), _ptr(ws), nws, h, d, _dtype(q), _stream()), "rel_bias_backward")
    return dtable


def _check_bias(bias, n_edges, h, device, cfg, by_pair=False):
    if bias is None:
        return
    shape = (h, n_edges) if by_pair else (n_edges + 1, h)
    if bias.dtype != torch.float32 or tuple(bias.shape) != shape or not bias.is_contiguous() or bias.device != device:
        raise ValueError(f"bias must be a contiguous float32 {shape} tensor on {device}")
    if not cfg.use_groups:
        raise RuntimeError("the per-edge score term needs the row-group kernels")


def attention_forward(col, indptr_c, eid_c, indices_c, q, k, v, scale=None, dropout_p=0.0, seed=0, bias=None, bias_by_pair=False):
    """o[dst] = sum over in-edges drop(softmax((q[dst].k[src] + bias[e])*scale)) v[src]; returns (o, lse) with lse
    (n, h) float32 in base-2 units.  Arithmetic of modules/attention.py:66-77 in one pass.  dropout_p > 0
    drops attention probabilities as attention.py:73 does; the mask is a function of (seed, graph), see
    attention_dropout_mask.  bias: None or the float32 score term of rel_bias_forward: (E + 1, h) with its rows by edge
    id, or with bias_by_pair (h, E) with the edges in the order of the numbers attention_pair_rows() gives them (tile
    kernels only)."""
    cfg = _SETTINGS
    _check_all(col=col, indptr_c=indptr_c, eid_c=eid_c, indices_c=indices_c, q=q, k=k, v=v)
    _check_bias(bias, eid_c.size(0), _hd(q)[0], q.device, cfg, bias_by_pair)
    _same_dtype(q, k, v)
    h, d = _hd(q)
    _expect_index(eid_c, indices_c)
    _expect_shape(k, (k.size(0),) + tuple(q.shape[1:]), "k")
    _expect_shape(v, k.shape, "v")
    scale = 1.0 / math.sqrt(d) if scale is None else float(scale)
    seg = _tile_seg_without_plan(col, eid_c.size(0), q, k, h, d, dropout_p, bias, cfg)
    if seg is None:
        # the choices look at a plan of the graph (where the tile kernels may run it comes from the GPU builder too:
        # 0.2 ms instead of 1.5 ms for a new graph of 16 K rows)
        plan = plan_cache.get(col, indptr_c, eid_c, indices_c, q.size(0), k.size(0), prefer_device=_tiles(q, h, d, None, dropout_p, bias, cfg))
        if _attention_groups(plan, dropout_p, bias, q, k, cfg) and _tiles(q, h, d, plan, dropout_p, bias, cfg):
            seg = _tile_seg_len(plan)
    tiles = seg is not None
    if tiles:
        plan = plan_cache.get(col, indptr_c, eid_c, indices_c, q.size(0), k.size(0), seg_len=seg, prefer_device=True)
        ref = ctypes.byref(plan.bias_rows(TILE_ROWS)["struct"] if bias_by_pair else plan.ensure_groups(TILE_ROWS)["struct"])
    elif not _attention_groups(plan, dropout_p, bias, q, k, cfg):
        ref = plan.ref
    else:
        ref = ctypes.byref(plan.ensure_groups(_forward_rows(q, h, d, plan, cfg))["struct"])
    if bias_by_pair and not (tiles and bias is not None):
        raise RuntimeError("bias_by_pair: this call does not run on the tile kernels (ask attention_pair_rows() first)")
    o = torch.empty_like(q)
    lse = torch.empty((q.size(0), h), dtype=torch.float32, device=q.device)
    dt = _dtype(q)
    ws, nws = _workspace(OP_ATTN_FWD, plan, None, h, d, dt, q.device)
    with _on_device_of(q):
        check_attn(_LIB.bpt_attention_forward(ref, _ptr(q), _ptr(k), _ptr(v), _ptr(bias), _ptr(o), _ptr(lse), _ptr(ws), nws,
                                              scale, float(dropout_p), int(seed) & (2 ** 64 - 1), h, d, dt, _stream()),
                   "attention_forward")
    return o, lse


def attention_backward(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, v, o, lse, do, scale=None,
                       dropout_p=0.0, seed=0, bias=None, bias_by_pair=False):
    """(dq, dk, dv) of attention_forward (same dropout_p, seed, bias and bias_by_pair).  With bias a fourth result: ds,
    float32 (E, h), or (h, E) with bias_by_pair, the gradient with respect to q.k + bias of every edge and head (= the
    gradient of bias), laid out like bias."""
    cfg = _SETTINGS
    _check_all(row=row, indptr_r=indptr_r, eid_r=eid_r, indices_r=indices_r, col=col, indptr_c=indptr_c,
               eid_c=eid_c, indices_c=indices_c, q=q, k=k, v=v, o=o, lse=lse)
    do = do.contiguous()
    _same_dtype(q, k, v, o, do)
    h, d = _hd(q)
    _expect_index(eid_c, indices_c)
    _expect_index(eid_r, indices_r)
    _expect_shape(eid_r, eid_c.shape, "eid_r")
    _expect_shape(k, (k.size(0),) + tuple(q.shape[1:]), "k")
    _expect_shape(v, k.shape, "v")
    _expect_shape(o, q.shape, "o")
    _expect_shape(do, q.shape, "do")
    if lse.dtype != torch.float32 or lse.device != q.device:
        raise ValueError("lse must be the float32 tensor that attention_forward returned")
    _expect_shape(lse, (q.size(0), h), "lse")
    _check_bias(bias, eid_c.size(0), h, q.device, cfg, bias_by_pair)
    scale = 1.0 / math.sqrt(d) if scale is None else float(scale)
    on_gpu = _tiles(q, h, d, None, dropout_p, bias, cfg)        # (as in attention_forward)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    ds = torch.empty((h, eid_c.size(0)) if bias_by_pair else (eid_c.size(0) + 1, h), dtype=torch.float32, device=q.device) if bias is not None else None
    dt = _dtype(q)
    def tile_plans(seg):
        """The two tile plans and the structs the kernels take, or None where a side does not cover every edge."""
        pi = plan_cache.get(col, indptr_c, eid_c, indices_c, q.size(0), k.size(0), seg_len=seg, prefer_device=True)
        po = plan_cache.get(row, indptr_r, eid_r, indices_r, k.size(0), q.size(0), seg_len=seg, prefer_device=True)
        if not (pi.covers_all_edges and po.covers_all_edges):
            return None
        # the destination side writes (p, ds) by its own pair numbers; the source side finds them through its pair mapping
        return (pi, po, ctypes.byref(pi.bias_rows(TILE_ROWS)["struct"] if bias_by_pair else pi.ensure_groups(TILE_ROWS)["struct"]),
                ctypes.byref(po.linked_to(pi, TILE_ROWS, order=_plan.tile_order_src(po.n_rows, po.n_edges), partner_order=None, pair_numbers=True)))

    # as in attention_forward: the tile plans straight away where the tile kernels are certain
    seg = _tile_seg_without_plan(col, eid_c.size(0), q, k, h, d, dropout_p, bias, cfg) if _tiles_backward(None, q.dtype, bias) else None
    chosen = tile_plans(seg) if seg is not None else None
    if chosen is None:
        plan_in = plan_cache.get(col, indptr_c, eid_c, indices_c, q.size(0), k.size(0), prefer_device=on_gpu)
        plan_out = plan_cache.get(row, indptr_r, eid_r, indices_r, k.size(0), q.size(0), prefer_device=on_gpu)
        in_ref, out_ref = plan_in.ref, plan_out.ref
        if _attention_groups(plan_in, dropout_p, bias, q, k, cfg) and plan_in.covers_all_edges and plan_out.covers_all_edges:
            if _tiles(q, h, d, plan_in, dropout_p, bias, cfg) and _tiles_backward(plan_in, q.dtype, bias):
                chosen = tile_plans(_tile_seg_len(plan_in))
            else:
                R = _group_rows(q, h, d, plan_in, cfg)
                in_ref = ctypes.byref(plan_in.linked_to(plan_out, R))
                out_ref = ctypes.byref(plan_out.ensure_groups(R, GROUP_ORDER_SRC)["struct"])
    tiles = chosen is not None
    if tiles:
        plan_in, plan_out, in_ref, out_ref = chosen
    if bias_by_pair and not (tiles and bias is not None):
        raise RuntimeError("bias_by_pair: this call does not run on the tile kernels (ask attention_pair_rows() first)")
    ws, nws = _workspace(OP_ATTN_BWD, plan_in, plan_out, h, d, dt, q.device, plan_ref=in_ref, plan_t_ref=out_ref)
    with _on_device_of(q):
        check_attn(_LIB.bpt_attention_backward(in_ref, out_ref, _ptr(q), _ptr(k), _ptr(v), _ptr(bias), _ptr(o), _ptr(do),
                                               _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(ds), _ptr(ws), nws,
                                               scale, float(dropout_p), int(seed) & (2 ** 64 - 1), h, d, dt, _stream()),
                   "attention_backward")
    if bias is not None:
        return dq, dk, dv, ds if bias_by_pair else ds[:-1]
    return dq, dk, dv


def _pair_order(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, dropout_p):
    """The in-CSR's tile plan and its pair-order tables (DevicePlan.bias_rows) where attention_forward and
    attention_backward will both run on the tile kernels with a per-edge score term for these arguments, else None."""
    cfg = _SETTINGS
    if q.dim() != 3 or not q.is_cuda:
        return None
    h, d = _hd(q)
    marker = q                                             # (stands for "a score term is given" in the choices below)
    seg = _tile_seg_without_plan(col, eid_c.size(0), q, k, h, d, dropout_p, marker, cfg) if attention_supported(q) and \
        _tiles_backward(None, q.dtype, marker) else None
    if seg is not None:
        plan_in = plan_cache.get(col, indptr_c, eid_c, indices_c, q.size(0), k.size(0), seg_len=seg, prefer_device=True)
        plan_out = plan_cache.get(row, indptr_r, eid_r, indices_r, k.size(0), q.size(0), seg_len=seg, prefer_device=True)
        if plan_in.covers_all_edges and plan_out.covers_all_edges:
            return plan_in, plan_in.bias_rows(TILE_ROWS)
    on_gpu = _tiles(q, h, d, None, dropout_p, q, cfg)
    plan_in = plan_cache.get(col, indptr_c, eid_c, indices_c, q.size(0), k.size(0), prefer_device=on_gpu)
    plan_out = plan_cache.get(row, indptr_r, eid_r, indices_r, k.size(0), q.size(0), prefer_device=on_gpu)
    if not (attention_supported(q) and _attention_groups(plan_in, dropout_p, marker, q, k, cfg) and plan_in.covers_all_edges
            and plan_out.covers_all_edges and _tiles(q, h, d, plan_in, dropout_p, marker, cfg)
            and _tiles_backward(plan_in, q.dtype, marker)):
        return None
    plan_in = plan_cache.get(col, indptr_c, eid_c, indices_c, q.size(0), k.size(0), seg_len=_tile_seg_len(plan_in), prefer_device=True)
    return plan_in, plan_in.bias_rows(TILE_ROWS)


def attention_pair_rows(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, dropout_p=0.0):
    """For a step with a per-edge score term: None, or, where attention_forward and attention_backward will both run on
    the tile kernels for these arguments, the (E,) int64 tensor that numbers the edges the way the tiles meet them (the pair
    numbers of the in-CSR's tile plan).  A score term stored in that order, head-major ((h, E): the value of edge e and a
    head at [head, number[e]]), and passed with bias_by_pair=True is read, and its gradient written, in runs of
    neighbouring values per tile, with no index read on the way, instead of rows scattered by edge id."""
    hit = _pair_order(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, dropout_p)
    return None if hit is None else hit[1]["pair_of_eid"]


def attention_pair_members(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, dropout_p=0.0):
    """Where attention_pair_rows gives numbers: the (E,) int32 tensor with, for every pair number, which of its tile's
    16 rows the pair's destination is (what rel_bias_forward_tiles needs beside the pair's edge type); else None."""
    hit = _pair_order(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, dropout_p)
    return None if hit is None else hit[1]["member_of_pair"]


def rel_bias_forward_tiles(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, table, used_types, pair_types,
                           dropout_p=0.0):
    """The rel_pos score term of modules/attention.py:69-71 in the pair order of the tile kernels: float32 (h, E) with
    [head, t] = q[dst of pair t, head, :] . table[used_types[pair_types[t] & 255], :], the form attention_forward takes with
    bias_by_pair=True.  pair_types (E,) int32: per pair number (attention_pair_rows) the number of its edge's type in
    used_types, plus its attention_pair_members() value << 8.  Needs rel_rows_supported(q), at most
    REL_MAX_USED_TYPES types in use and arguments for which attention_pair_rows() gives numbers (RuntimeError else)."""
    _check_all(q=q, table=table, used_types=used_types, pair_types=pair_types)
    _same_dtype(q, table)
    h, d = _hd(q)
    if table.dim() != 2 or table.size(1) != d:
        raise ValueError(f"table must be (n_types, {d})")
    E = eid_c.size(0)
    if used_types.dtype != torch.int32 or used_types.dim() != 1 or used_types.numel() > table.size(0):
        raise ValueError("used_types must be a 1-D int32 tensor of at most table.size(0) elements")
    if pair_types.dtype != torch.int32 or tuple(pair_types.shape) != (E,):
        raise ValueError(f"pair_types must be int32 ({E},)")
    hit = _pair_order(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, dropout_p)
    if hit is None:
        raise RuntimeError("rel_bias_forward_tiles: these arguments do not run on the tile kernels (ask attention_pair_rows() first)")
    bias = torch.empty((h, E), dtype=torch.float32, device=q.device)
    with _on_device_of(q):
        check_attn(_LIB.bpt_rel_bias_forward_tiles(ctypes.byref(hit[1]["struct"]), _ptr(q), _ptr(table), _ptr(used_types), used_types.numel(),
                                                   _ptr(pair_types), _ptr(bias), h, d, _dtype(q), _stream()), "rel_bias_forward_tiles")
    return bias


def attention_dropout_mask(col, indptr_c, eid_c, indices_c, q, k, dropout_p, seed):
    """The (E, h) float32 multipliers (0 or 1 / (1 - p)) that attention_forward(..., dropout_p, seed) applies to the
    attention probabilities, computed on the host (testing and debugging aid).  The decision is a hash of
    (seed, edge id, head): it does not depend on the graph's plan."""
    import numpy as np
    h, d = _hd(q)
    E = eid_c.size(0)
    p = float(dropout_p)
    if not p > 0.0:
        return torch.ones((E, h), dtype=torch.float32)
    t = p * 4294967296.0
    thr = np.uint32(min(max(t, 1.0), 4294967295.0))
    seed = int(seed) & (2 ** 64 - 1)
    s32 = np.uint32((seed ^ (seed >> 32)) & 0xffffffff)
    key = (np.arange(E, dtype=np.uint64)[:, None] * np.uint64(h) + np.arange(h, dtype=np.uint64)[None, :]).astype(np.uint32)
    x = key ^ s32
    x ^= x >> np.uint32(16); x = (x.astype(np.uint64) * np.uint64(0x7feb352d)).astype(np.uint32)
    x ^= x >> np.uint32(15); x = (x.astype(np.uint64) * np.uint64(0x846ca68b)).astype(np.uint32)
    x ^= x >> np.uint32(16)
    keep = np.where(x >= thr, np.float32(1.0 / (1.0 - np.float32(p))), np.float32(0.0)).astype(np.float32)
    return torch.from_numpy(keep)


_MIN_GROUP_ITEMS = 1536     # graphs with fewer work items run one wavefront per row (unless set_group_rows forces groups)


def _attention_groups(plan, dropout_p, bias, q, k, cfg=None):
    """Whether the fused kernels take the row groups for this graph.  Very small graphs do not fill the GPU with one
    wavefront per group of rows and run faster with one per row (measured: L = 512, 0.055 against 0.070 ms per step;
    even at L = 1024); dropout and the score term exist in the row-group kernels only.  The row-group kernels address
    the rows of q AND of k / v with 32-bit byte offsets, so both node tensors have to stay below 4 GiB."""
    cfg = _SETTINGS if cfg is None else cfg
    if not cfg.use_groups:
        return False
    if max(q.size(0), k.size(0)) * q.size(1) * q.size(2) * q.element_size() >= 2 ** 32:
        if dropout_p > 0.0 or bias is not None:
            raise RuntimeError("dropout and the score term need the row-group kernels, which address node tensors below 4 GiB")
        return False
    return plan.n_items >= _MIN_GROUP_ITEMS or cfg.group_rows is not None or dropout_p > 0.0 or bias is not None


def _group_rows(q, h, d, plan, cfg=None):
    """Rows per group for the fused kernels.  Groups of 8 nearly halve the row fetches of groups of 4 but double
    the work of the longest wavefront, which measured as a gain only on graphs with enough groups to fill the
    GPU twice or with long rows (average degree >= 48: at L = 4096, k = 8 (37) groups of 4 win, at k = 16 (59) groups of 8),
    and not for bfloat16 rows of up to 512 columns."""
    cfg = _SETTINGS if cfg is None else cfg
    if cfg.group_rows is not None:
        return cfg.group_rows
    big = plan.n_items >= 16384 or plan.n_edges >= 48 * max(plan.n_rows, 1)
    return 8 if (big and (q.dtype == torch.float32 or h * d > 512)) else 4


def _forward_rows(q, h, d, plan, cfg=None):
    """Rows per group for the forward kernel.  Groups of 8 run on the matrix cores (two wavefronts per group; bfloat16
    rows go through the bfloat16 matrix instructions as loaded), which measured faster than the vector kernels at every
    size and both dtypes."""
    cfg = _SETTINGS if cfg is None else cfg
    if cfg.group_rows is not None:
        return cfg.group_rows
    return 8


TILE_ROWS = TILE_GROUP_R
TILE_BACKWARD = None       # testing / measurement hook: True / False force the backward on / off tiles (None: by graph size and density)
TILE_BF16 = True           # testing / measurement hook: bfloat16 rows on tiles too
TILE_SEG_LEN = None        # testing / measurement hook: edges per work item of the tile plans (None: by average degree)


def _tiles(q, h, d, plan, dropout_p, bias, cfg):
    """Whether the fused forward runs on dense tiles (groups of 16 rows, one wavefront per head, every block of 16
    entries a dense 16 x 16 matrix product with the missing pairs masked): float32 or bfloat16 rows of 64 columns per
    head (dropout and the score term included: their variants read the edge id of every pair), and the library's choice of
    rows per group not overridden."""
    return (cfg.use_tiles and cfg.group_rows is None and (q.dtype == torch.float32 or (TILE_BF16 and q.dtype == torch.bfloat16))
            and d == 64 and h <= 16)


def _tiles_backward(plan, dtype, bias=None):
    """The backward runs on tiles wherever the forward does.  float32 (8 x 64), step time on tiles against row groups:
    L = 8192, k = 4 0.175 against 0.187 ms, with attention dropout 0.178 against 0.203; the 32-graph batch 0.298 against
    0.307; L = 32768, k = 4 0.807 against 0.841; L = 4096, k = 1 ... 32 level to 27 % faster, window 128 1.9 x.  With the
    score term: L = 8192, k = 4 0.281 against 0.288 ms and the 32-graph batch 0.445 against 0.449 when the term is stored
    in the tiles' own order (attention_pair_rows), level with it stored by edge id.  bfloat16: a block costs six matrix
    instructions instead of 32 to 48 and every graph measured runs faster (L = 8192, k = 4: 0.112 against 0.135 ms;
    L = 32768, k = 8, 16 heads: 1.20 against 1.49; window 128: 0.081 against 0.188)."""
    if TILE_BACKWARD is not None:
        return TILE_BACKWARD
    return True


def _tile_seg_without_plan(units, n_edges, q, k, h, d, dropout_p, bias, cfg):
    """The work-item length of the tile plans where the tile kernels are certain for this call without a plan of the
    graph to look at, else None (the choices then look at one).  Certain: the shape has tile kernels, the node tensors
    fit 32-bit offsets, and the graph has at least _MIN_GROUP_ITEMS rows with edges (`units` lists them; a plan has at
    least one work item per such row) or the call carries dropout or a score term.  The length is _tile_seg_len's."""
    if not (cfg.use_groups and _tiles(q, h, d, None, dropout_p, bias, cfg)):
        return None
    if max(q.size(0), k.size(0)) * h * d * q.element_size() >= 2 ** 32:
        return None
    if not (units.numel() >= _MIN_GROUP_ITEMS or dropout_p > 0.0 or bias is not None):
        return None
    if TILE_SEG_LEN is not None:
        return TILE_SEG_LEN
    deg = n_edges / max(q.size(0), 1)
    return 64 if deg < 32 else (128 if deg < 80 else 256)


def _tile_seg_len(plan):
    """Edges per work item of the plans the tile kernels walk (TILE_SEG_LEN overrides when set)."""
    if TILE_SEG_LEN is not None:
        return TILE_SEG_LEN
    deg = plan.n_edges / max(plan.n_rows, 1)
    return 64 if deg < 32 else (128 if deg < 80 else 256)


def set_tiles(on):
    """Testing / measurement hook (process-wide): dense-tile kernels on (default) or off.  Returns the old setting."""
    return _replace_setting(use_tiles=bool(on)).use_tiles


def set_group_rows(R):
    """Testing / measurement hook (process-wide): force groups of R (4 or 8) rows, or None for the default choice.
    Returns the old value."""
    if R not in (None, 4, 8):
        raise ValueError("R must be None, 4 or 8")
    return _replace_setting(group_rows=R).group_rows


def row_groups_enabled():
    return _SETTINGS.use_groups


def set_row_groups(on):
    """Testing / measurement hook (process-wide): fused attention lets one wavefront own several rows that share
    neighbours (default) or one row each.  Returns the old setting."""
    return _replace_setting(use_groups=bool(on)).use_groups


def set_grouped_ops(on):
    """Testing / measurement hook (process-wide): let the unfused SpMM- and SDDMM-shaped ops (masked_mm and vector_spmm,
    forward and backward) use the row groups (default) or one wavefront per row.  Returns the old setting."""
    return _replace_setting(grouped_ops=bool(on)).grouped_ops


def set_force_generic(on):
    """Testing hook (process-wide, an atomic flag inside the library): route every op through the shape-generic kernels."""
    global _FORCE_GENERIC
    _FORCE_GENERIC = bool(on)
    return bool(_LIB.bpt_set_force_generic(1 if on else 0))


_FORCE_GENERIC = False


def force_generic_enabled():
    """What set_force_generic last set."""
    return _FORCE_GENERIC
