"""Autograd operators with the surface of the reference's modules/op.py:10-70 (same Function
names, argument orders, saved tensors and `None` gradient slots), running on the HIP kernels,
plus `bpt_attention`, the fused layer core.
"""
import math

import torch
from torch.autograd import Function

from . import graphop as _g
from .graphop import (maskedmm_csr_backward, maskedmm_csr_forward, node_mul_edge_backward, node_mul_edge_forward,
                      sparse_softmax_backward, sparse_softmax_forward, vector_spmm_backward, vector_spmm_forward)

__all__ = ["SparseSoftmax", "MaskedMMCSR", "NodeMulEdge", "VectorSPMM", "BPTAttention", "EdgeTypeEmbedding",
           "sparse_softmax", "masked_mm", "node_mul_edge", "vec_spmm", "bpt_attention", "edge_type_embedding"]


class SparseSoftmax(Function):
    # modules/op.py:10-20
    @staticmethod
    def forward(ctx, row, indptr, eid, x):
        y = sparse_softmax_forward(row, indptr, eid, x)
        ctx.save_for_backward(row, indptr, eid, y)
        return y

    @staticmethod
    def backward(ctx, dy):
        row, indptr, eid, y = ctx.saved_tensors
        return None, None, None, sparse_softmax_backward(row, indptr, eid, y, dy.contiguous())


class MaskedMMCSR(Function):
    # modules/op.py:23-33
    @staticmethod
    def forward(ctx, row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, A, B):
        ctx.save_for_backward(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, A, B)
        return maskedmm_csr_forward(row, indptr_r, eid_r, indices_r, A, B)

    @staticmethod
    def backward(ctx, grad):
        row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, A, B = ctx.saved_tensors
        dA, dB = maskedmm_csr_backward(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, A, B, grad)
        return None, None, None, None, None, None, None, None, dA, dB


class NodeMulEdge(Function):
    # modules/op.py:35-45
    @staticmethod
    def forward(ctx, row, indptr, eid, A, B):
        ctx.save_for_backward(row, indptr, eid, A, B)
        return node_mul_edge_forward(row, indptr, eid, A, B)

    @staticmethod
    def backward(ctx, grad):
        row, indptr, eid, A, B = ctx.saved_tensors
        dA, dB = node_mul_edge_backward(row, indptr, eid, A, B, grad)
        return None, None, None, dA, dB


class VectorSPMM(Function):
    # modules/op.py:47-58
    @staticmethod
    def forward(ctx, row, indptr, eid, indices, col, ptr_t, eid_t, indices_t, edata, x, n_rows=None):
        # n_rows (not in the reference): rows of y when the operator is rectangular (y = zeros_like(x) there, :527)
        y = vector_spmm_forward(row, indptr, eid, indices, edata, x, n_rows=n_rows)
        ctx.save_for_backward(row, indptr, eid, indices, col, ptr_t, eid_t, indices_t, edata, x)
        return y

    @staticmethod
    def backward(ctx, dy):
        row, indptr, eid, indices, col, ptr_t, eid_t, indices_t, edata, x = ctx.saved_tensors
        dedata, dx = vector_spmm_backward(row, indptr, eid, indices, col, ptr_t, eid_t, indices_t, edata, dy, x)
        return None, None, None, None, None, None, None, None, dedata, dx, None


class BPTAttention(Function):
    """Fused masked_mm -> scale -> sparse_softmax -> dropout -> vec_spmm (modules/attention.py:66-77 with
    rel_pos off).  Saves q, k, v, o and the per-(node, head) log-sum-exp instead of the (E, h) score and
    probability tensors; the dropout mask is regenerated in backward from (dropout_p, seed)."""

    @staticmethod
    def forward(ctx, row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, v, scale, dropout_p=0.0, seed=0):
        o, lse = _g.attention_forward(col, indptr_c, eid_c, indices_c, q, k, v, scale, dropout_p, seed)
        ctx.save_for_backward(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, v, o, lse)
        ctx.scale, ctx.dropout_p, ctx.seed = scale, dropout_p, seed
        return o

    @staticmethod
    def backward(ctx, do):
        row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, v, o, lse = ctx.saved_tensors
        dq, dk, dv = _g.attention_backward(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c,
                                           q, k, v, o, lse, do, ctx.scale, ctx.dropout_p, ctx.seed)
        return None, None, None, None, None, None, None, None, dq, dk, dv, None, None, None


class BPTRelAttention(Function):
    """BPTAttention with the rel_pos score term of modules/attention.py:69-71, s = (q.k + q.table[etype]) * scale,
    without the (E, d) rows of the embedding lookup: a small kernel writes the (E, h) term q[dst].table[etype], the
    fused kernels add it to the scores, and the backward kernel returns ds = dL/d(q.k + term) per edge and head,
    from which the term's gradients follow: dq += sum_e ds[e] table[etype[e]] over the in-CSR and
    dtable[t] = sum_h sum_{e of type t} ds[e, h] q[dst(e), h].  One kernel forms both where the shape has it
    (graphop.rel_bias_backward); otherwise two SpMMs do, the first over the in-CSR with the edge types as column indices,
    the second over a CSR whose rows are the edge types.  All sums are row-owned (no atomics)."""

    @staticmethod
    def forward(ctx, row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, v, scale, dropout_p, seed,
                table, etype):
        aux = _rel_aux(etype, col, indptr_c, eid_c, table.size(0))
        table = table.contiguous()
        # (the gradient kernel's configuration is asked for here: the SpMM form is then chosen for both passes up front)
        ctx.on_chip = (_g.rel_rows_supported(q) and aux["n_used"] <= _g.REL_MAX_USED_TYPES and not _g.force_generic_enabled()
                       and _g.rel_bias_backward_supported(q, aux["n_used"]))
        # where forward and backward both run on the tile kernels, the term and its gradient are stored head-major in the
        # order in which the tiles meet the edges (rows_slot: the place of every in-CSR slot) instead of by edge id
        graph = (row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k)
        pair = _g.attention_pair_rows(*graph, dropout_p) if ctx.on_chip else None
        ctx.rows_slot = None
        if pair is not None:
            held = aux.get("rows_slot")
            if held is None or held[0] is not pair:
                rows_slot = pair.index_select(0, eid_c).contiguous()
                # per pair number: the number of its edge's type and which row of its tile its destination is
                types = torch.empty_like(aux["number_slot"]).index_copy_(0, rows_slot, aux["number_slot"]).to(torch.int32)
                held = aux["rows_slot"] = (pair, rows_slot, (types | (_g.attention_pair_members(*graph, dropout_p) << 8)).contiguous())
            ctx.rows_slot = held[1]
            try:
                bias = _g.rel_bias_forward_tiles(*graph, table, aux["used_types"], held[2], dropout_p)
            except _g.BptStatusError as err:
                # (many types in use need more than 64 KB of LDS there, which a runtime may refuse: the kernel over the
                # in-CSR writes the same layout from within 64 KB)
                if err.status != _g.BPT_ERR_UNSUPPORTED:
                    raise
                bias = _g.rel_bias_forward(col, indptr_c, ctx.rows_slot, aux["number_slot"], q, table, used_types=aux["used_types"],
                                           by_pair=True)
        elif ctx.on_chip:
            bias = _g.rel_bias_forward(col, indptr_c, eid_c, aux["number_slot"], q, table, used_types=aux["used_types"])
        else:
            bias = _g.rel_bias_forward(col, indptr_c, eid_c, aux["etype_slot"], q, table)
        o, lse = _g.attention_forward(col, indptr_c, eid_c, indices_c, q, k, v, scale, dropout_p, seed, bias=bias,
                                      bias_by_pair=ctx.rows_slot is not None)
        ctx.save_for_backward(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, v, o, lse, bias, table)
        ctx.scale, ctx.dropout_p, ctx.seed, ctx.aux, ctx.etype = scale, dropout_p, seed, aux, etype
        return o

    @staticmethod
    def backward(ctx, do):
        row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, v, o, lse, bias, table = ctx.saved_tensors
        aux = ctx.aux
        dq, dk, dv, ds = _g.attention_backward(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c,
                                               q, k, v, o, lse, do, ctx.scale, ctx.dropout_p, ctx.seed, bias=bias,
                                               bias_by_pair=ctx.rows_slot is not None)
        if ctx.on_chip:
            dtable = _g.rel_bias_backward(col, indptr_c, eid_c if ctx.rows_slot is None else ctx.rows_slot, aux["number_slot"], aux["used"],
                                          aux["used_types"], ds, q, table, dq, by_pair=ctx.rows_slot is not None)
        else:
            t_row, t_indptr, t_order, t_dst = _rel_type_rows(aux, ctx.etype, col, indptr_c, eid_c, table.size(0))
            h = q.size(1)
            ds = ds.to(q.dtype)
            table_h = table.unsqueeze(1).expand(-1, h, -1).contiguous()
            dq = vector_spmm_forward(col, indptr_c, eid_c, aux["etype_slot"], ds, table_h, n_rows=q.size(0), out=dq)
            dtable = vector_spmm_forward(t_row, t_indptr, t_order, t_dst, ds, q, n_rows=table.size(0))
            dtable = dtable.float().sum(1).to(table.dtype)
        return None, None, None, None, None, None, None, None, dq, dk, dv, None, None, None, dtable, None


_rel_aux_cache = {}


def _rel_aux(etype, col, indptr_c, eid_c, n_types):
    """Index tensors of the rel_pos term, cached per (etype, in-CSR): etype_slot, the edge type of every in-CSR slot;
    used_types (n_used,) int32, the types that occur in a slot, ascending; used (n_types,) int32, the number of every
    type in that list (-1 for the others); number_slot, the number of every slot's type.  Built where etype lives;
    two scalars are read back (the range check and n_used)."""
    key = tuple((t.data_ptr(), t.numel(), t._version) for t in (etype, col, indptr_c, eid_c)) + (str(etype.device), n_types)
    hit = _rel_aux_cache.get(key)
    if hit is None:
        et = etype.detach()
        if et.dim() != 1 or et.dtype != torch.int64:
            raise ValueError("etype must be a 1-D int64 tensor")
        if et.numel() and (int(et.min()) < 0 or int(et.max()) >= n_types):
            raise ValueError("edge type out of range")
        etype_slot = et.index_select(0, eid_c).contiguous()
        present = torch.zeros(n_types, dtype=torch.bool, device=et.device).index_fill_(0, etype_slot, True)
        number = torch.cumsum(present, 0, dtype=torch.int32) - 1
        used = torch.where(present, number, torch.full_like(number, -1)).contiguous()
        used_types = torch.nonzero(present).flatten().to(torch.int32)           # (the read-back of n_used)
        hit = {"etype_slot": etype_slot, "used": used, "used_types": used_types, "n_used": used_types.numel(),
               "number_slot": used.index_select(0, etype_slot).to(torch.int64), "keep": (etype, col, indptr_c, eid_c)}
        if len(_rel_aux_cache) > 16:
            _rel_aux_cache.clear()
        _rel_aux_cache[key] = hit           # "keep" holds the tensors so that their data_ptrs are not reused while cached
    return hit


def _rel_type_rows(aux, etype, col, indptr_c, eid_c, n_types):
    """For the SpMM form of the table's gradient: the CSR whose row t lists the edges of type t (_type_csr) and the
    destination node of each of its slots; kept with the other index tensors of the graph."""
    if "type_rows" not in aux:
        t_row, t_indptr, t_order = _type_csr(etype, n_types)
        slot_dst = torch.repeat_interleave(col, indptr_c[1:] - indptr_c[:-1], output_size=eid_c.numel())   # destination of every in-CSR slot
        dst_of_eid = torch.empty_like(slot_dst)
        dst_of_eid[eid_c] = slot_dst
        aux["type_rows"] = (t_row, t_indptr, t_order, dst_of_eid.index_select(0, t_order).contiguous())
    return aux["type_rows"]


def sparse_softmax(row, indptr, eid, x):
    return SparseSoftmax.apply(row, indptr, eid, x)


def masked_mm(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, A, B):
    return MaskedMMCSR.apply(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, A, B)


def node_mul_edge(row, indptr, eid, A, B):
    return NodeMulEdge.apply(row, indptr, eid, A, B)


def vec_spmm(row, indptr, eid, indices, col, ptr_t, eid_t, indices_t, edata, x, n_rows=None):
    return VectorSPMM.apply(row, indptr, eid, indices, col, ptr_t, eid_t, indices_t, edata, x, n_rows)


class EdgeTypeEmbedding(Function):
    """table[etype] -> (E, d): what `self.embed_ak(g.edata['etype'])` computes (modules/attention.py:57), with a
    deterministic backward: the (E, d) gradient rows are summed per edge type by the SpMM kernels over a CSR whose
    rows are the edge types (torch's embedding backward scatters with atomics, about 1 ms at E = 430 k)."""

    @staticmethod
    def forward(ctx, table, etype, type_csr):
        ctx.type_csr = type_csr
        ctx.n_types = table.size(0)
        return table.index_select(0, etype)

    @staticmethod
    def backward(ctx, grad):
        row, indptr, order = ctx.type_csr
        grad = grad.contiguous()
        ones = torch.ones(grad.size(0), dtype=grad.dtype, device=grad.device)
        return vector_spmm_forward(row, indptr, order, order, ones, grad, n_rows=ctx.n_types), None, None


_type_csr_cache = {}


def _type_csr(etype, n_types, chunk_size=32):
    """(row, indptr, order) of the CSR whose row t lists the edges of type t (ascending edge id), chunked like the
    reference's other CSRs (builder.pyx:305-321); cached per etype tensor.  Built where etype lives: on the GPU a stable
    sort, a histogram and prefix sums, with two scalars read back (the range check and the number of units), so the
    edge types never travel to the host."""
    key = (etype.data_ptr(), etype.numel(), etype._version, str(etype.device), n_types)
    hit = _type_csr_cache.get(key)
    if hit is None:
        et = etype.detach()
        if et.dim() != 1 or et.dtype != torch.int64:
            raise ValueError("etype must be a 1-D int64 tensor")
        if et.numel() and (int(et.min()) < 0 or int(et.max()) >= n_types):
            raise ValueError("edge type out of range")
        order = torch.argsort(et, stable=True)
        counts = torch.bincount(et, minlength=n_types)
        indptr = torch.zeros(n_types + 1, dtype=torch.int64, device=et.device)
        torch.cumsum(counts, 0, out=indptr[1:])
        # partition_csr on the device: row t gives ceil(count_t / chunk) units; unit u of row t starts at indptr[t] + u * chunk
        units = (counts + (chunk_size - 1)) // chunk_size
        first = torch.cumsum(units, 0) - units                           # number of the first unit of every row
        n_units = int(units.sum())
        row = torch.repeat_interleave(torch.arange(n_types, device=et.device), units, output_size=n_units)
        rank = torch.arange(n_units, device=et.device) - first.index_select(0, row)
        indptr_units = torch.empty(n_units + 1, dtype=torch.int64, device=et.device)
        indptr_units[:n_units] = indptr.index_select(0, row) + rank * chunk_size
        indptr_units[n_units] = et.numel()
        hit = (row, indptr_units, order, etype)
        if len(_type_csr_cache) > 16:
            _type_csr_cache.clear()
        _type_csr_cache[key] = hit          # holds etype so that its data_ptr is not reused while cached
    return hit[:3]


def edge_type_embedding(table, etype):
    """Rows of `table` for every edge, differentiable w.r.t. `table` (deterministic segment-sum backward)."""
    return EdgeTypeEmbedding.apply(table, etype, _type_csr(etype, table.size(0)))


def bpt_attention(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, v, scale=None, fused=None,
                  dropout_p=0.0, seed=None, rel_table=None, etype=None):
    """Attention over the graph: (ROW, INDPTR_R, out_eid, out_idx) is the out-CSR side (rows =
    sources), (COL, INDPTR_C, in_eid, in_idx) the in-CSR side (rows = destinations), exactly the
    eight graph arguments modules/attention.py:66-67 passes to masked_mm.

    fused=None picks the fused kernels when they cover (h, d, dtype) and otherwise composes the
    unfused HIP ops in the reference's order; both run on the GPU.

    dropout_p > 0 applies dropout to the attention probabilities (attention.py:73).  The fused path hashes
    (seed, edge, head); seed=None draws one from torch's CPU generator (reproducible under torch.manual_seed).  The
    unfused path uses torch's dropout, so the two paths drop different elements.

    rel_table (n_types, d) and etype (E,) int64 add the rel_pos term q[dst] . rel_table[etype[e]] to the score of
    edge e (attention.py:69-71); the gradient of rel_table is returned like any other."""
    scale = 1.0 / math.sqrt(q.size(-1)) if scale is None else float(scale)
    if (rel_table is None) != (etype is None):
        raise ValueError("rel_table and etype go together")
    padded = None
    if fused is None:
        fused = _g.attention_supported(q)
        if not fused and not _g.force_generic_enabled():
            padded = _g.attention_padded_shape(q)
            fused = padded is not None
        if (dropout_p > 0 or rel_table is not None) and not _g.row_groups_enabled():
            fused = False                       # only the row-group kernels implement dropout and the rel_pos term
    elif fused and not _g.attention_supported(q):
        padded = _g.attention_padded_shape(q)
    if fused and padded is not None:
        # heads of fewer than 64 columns (6 x 50, 8 x 40 in the reference's configs): the fused kernels run on zero-padded copies
        # (h', 64) with the scale of the real d; the pads and the slices are ordinary differentiable torch ops
        h, d = q.size(1), q.size(2)
        hp, dp = padded
        grow = lambda x: torch.nn.functional.pad(x, (0, dp - d, 0, hp - h))
        o = bpt_attention(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, grow(q), grow(k), grow(v), scale=scale,
                          fused=True, dropout_p=dropout_p, seed=seed,
                          rel_table=None if rel_table is None else torch.nn.functional.pad(rel_table, (0, dp - d)), etype=etype)
        return o[:, :h, :d].contiguous()
    if fused:
        if dropout_p > 0 and seed is None:
            seed = int(torch.randint(0, 2 ** 62, (1,)).item())
        if rel_table is not None:
            return BPTRelAttention.apply(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, v, scale,
                                         float(dropout_p), int(seed or 0), rel_table, etype)
        return BPTAttention.apply(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, q, k, v, scale,
                                  float(dropout_p), int(seed or 0))
    e = masked_mm(row, indptr_r, eid_r, indices_r, col, indptr_c, eid_c, indices_c, k, q)
    if rel_table is not None:
        e = e + node_mul_edge(col, indptr_c, eid_c, q, edge_type_embedding(rel_table, etype))
    a = torch.nn.functional.dropout(sparse_softmax(col, indptr_c, eid_c, e * scale), p=float(dropout_p), training=dropout_p > 0)
    return vec_spmm(col, indptr_c, eid_c, indices_c, row, indptr_r, eid_r, indices_r, a, v,
                    n_rows=None if q.size(0) == v.size(0) else q.size(0))
