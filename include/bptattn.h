/*
 * libbptattn — gfx950 (MI355X) HIP kernels of the BPT graph-attention path, C ABI.
 *
 * Drop-in boundary for the reference's `graphop` extension (graph_kernel/graphop.cpp:216-225):
 * one entry point per pybind function, plus the fused attention pair.  Plain pointers and sizes
 * only; no torch types.  All data pointers are DEVICE pointers; outputs and the workspace are
 * allocated by the caller (the library never allocates or frees device memory and never
 * synchronises); kernels are enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 * default stream).  Every function returns 0 on success, a negative bpt_status for an argument
 * error (nothing was launched) or a positive hipError_t if a launch failed.  Nothing throws.
 *
 * Graph arguments.  The reference passes chunked units (row, indptr), eid and indices as int64
 * tensors.  Here they are passed as a `bpt_plan`: the int32 row-level form of exactly those four
 * arrays plus the wavefront work list, produced once per graph by bptg_plan_fill()
 * (include/bptgraph.h) and uploaded by the caller.  Row ownership replaces the reference's float
 * atomics: every output row is written by one wavefront (rows longer than the plan's segment
 * length by a fixed-order combine), so results are deterministic.
 *
 * Tensor layouts (row-major, contiguous): node tensors (n, h, d); edge tensors (n_edges, h)
 * addressed by edge id; the per-edge feature of node_mul_edge (n_edges, d).  A reference call
 * with 2-D node tensors (n, d) is h = 1.
 */
#ifndef BPTATTN_H
#define BPTATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { BPT_F32 = 0, BPT_F64 = 1, BPT_BF16 = 2 } bpt_dtype;

typedef enum {
    BPT_OK = 0,
    BPT_ERR_NULL = -1,        /* required pointer is NULL */
    BPT_ERR_SIZE = -2,        /* negative or inconsistent size */
    BPT_ERR_DTYPE = -3,       /* unknown dtype */
    BPT_ERR_SHAPE = -4,       /* h or d not positive / too large */
    BPT_ERR_WORKSPACE = -5,   /* workspace missing or smaller than bpt_workspace_bytes() */
    BPT_ERR_PLAN = -6,        /* plans do not describe the same graph (edge / node counts differ) */
    BPT_ERR_UNSUPPORTED = -7, /* combination not implemented (e.g. fused attention in f64) */
    BPT_ERR_SCRATCH = -8      /* the call needs more than BPT_NOALLOC_SCRATCH_BYTES of the library's static scratch */
} bpt_status;

/* Device-resident plan of one CSR side (see bptg_plan_fill / bptg_group_plan for the array contents).
 * The grp_* fields are optional (n_groups == 0: none); the fused attention entries use them to let one
 * wavefront own up to grp_R rows that share neighbours, loading each neighbour row once for all (grp_R = 4 or 8:
 * row-group kernels; grp_R = 16 with d = 64, f32 or bf16: the kernels that multiply 16 x 16 blocks of
 * (row, neighbour) pairs on the matrix cores, one wavefront per group and head), and so do the
 * SDDMM / SpMM-shaped ops (maskedmm_csr, vector_spmm, rel_bias) when the plan also carries grp_eids and the shape
 * has specialised kernels; without groups every row (segment) has a wavefront of its own. */
typedef struct {
    const int32_t *rowptr;   /* n_rows + 1 */
    const int32_t *idx;      /* n_edges : other endpoint of the edge in slot p */
    const int32_t *eid;      /* n_edges : edge id of slot p */
    const int32_t *items;    /* n_items * 4 : row, begin, end, slot */
    const int32_t *heavy;    /* n_heavy * 3 : row, first_slot, n_slots (may be NULL if n_heavy == 0) */
    int64_t n_rows, n_edges, n_items, n_heavy, n_slots;
    const int32_t *grp_members;  /* n_groups * grp_R * 2 : (row, slot), row = -1 unused */
    const int32_t *grp_ptr;      /* n_groups + 1 : entry range of each group */
    const int32_t *grp_entries;  /* n_grp_entries * 4 : neighbour id, member mask, first pair, 0 */
    const int32_t *grp_pairs;    /* (n_grp_entries + 8) * grp_R or NULL.  Links the two sides' plans for the
                                    fused backward, whose per-pair scratch one side writes and the other reads.
                                    grp_R = 4 or 8 (row groups): on the DESTINATION-side plan, for (entry u,
                                    member m) of this plan, at [u * grp_R + m], the position u' * grp_R + m' of
                                    the same edge in the source-side plan (the scratch is laid out in that
                                    order); where the entry's mask has no bit m, and in the 8 entries of
                                    padding, the spare position (n_grp_entries of the source side + 8) * grp_R - 1.
                                    grp_R = 16 (tiles): on the SOURCE-side plan, at [u * 16 + m], the pair number
                                    of the same edge in the destination-side plan, i.e. that side's
                                    grp_entries[u'].first_pair + (number of mask bits below m'), in 0 .. n_edges-1
                                    (the scratch is compact, one record per edge and head); 0 where the mask has
                                    no bit m and in the padding (never dereferenced) */
    const int32_t *grp_chunks;   /* 9 : groups grp_chunks[x] .. grp_chunks[x+1]-1 are walked by XCD x */
    int64_t n_groups, grp_R;
    int64_t grp_max_chunk;       /* largest chunk length; the row-group kernels launch 8 * grp_max_chunk workgroups */
    int64_t n_grp_entries;       /* grp_ptr[n_groups] */
    const int32_t *grp_eids;     /* (n_grp_entries + 8) * grp_R or NULL: edge id of (entry u, member m) at
                                    [u * grp_R + m]; n_edges where the entry's mask has no bit m and in the 8
                                    entries of padding.  Needed by the attention calls that take a per-edge score
                                    term or dropout and by the row-group kernels of the SDDMM / SpMM-shaped ops */
    int64_t bias_by_pair;        /* 0: the per-edge score term `bias` and its gradient `ds_out` are (n_edges + 1, h)
                                    arrays with one row per edge id.  Non-zero (grp_R = 16 only): they are (h, n_edges)
                                    arrays, head-major, and the value of (entry u, member m) sits at
                                    [head * n_edges + grp_entries[u].first_pair + (number of mask bits below m)], the
                                    plan's own pair number: a tile's values are neighbours in memory and no index is
                                    read on the way.  Forward and backward must be given the same setting, and whoever
                                    produces `bias` / consumes `ds_out` uses the same places: bpt_rel_bias_forward /
                                    _backward do when THEIR plan has the flag set and carries, as eid, the pair number
                                    of every slot's edge */
    int64_t n_index_nodes;       /* rows of the node tensor that idx points into (the other side's node count: attention to a
                                    memory of another length, modules/attention.py:144-168); 0 = the same as n_rows.  The
                                    row-group and tile kernels address rows of BOTH node tensors with 32-bit byte offsets and
                                    are taken only when max(n_rows, n_index_nodes) * h * d * sizeof(element) < 4 GiB; a
                                    caller whose neighbour tensor has more rows than n_rows must say so here */
} bpt_plan;

/* sizeof(bpt_plan) as this library was compiled: a binding checks its own mirror of the struct against it before the first call
 * (a shorter struct would make the library read past the caller's memory). */
int64_t bpt_plan_struct_bytes(void);

const char *bpt_strerror(int status);

/* Bytes of workspace the call needs (0 possible).  op: one of the BPT_OP_* below. */
enum {
    BPT_OP_MASKEDMM_BWD = 1, BPT_OP_NODE_MUL_EDGE_BWD = 2, BPT_OP_SPMM_FWD = 3, BPT_OP_SPMM_BWD = 4,
    BPT_OP_ATTN_FWD = 5, BPT_OP_ATTN_BWD = 6, BPT_OP_SOFTMAX_FWD = 7, BPT_OP_SOFTMAX_BWD = 8
};
int64_t bpt_workspace_bytes(int op, const bpt_plan *plan, const bpt_plan *plan_t, int h, int d, int dtype);

/* graphop.cpp:16  maskedmm_csr_forward(row, indptr, eid, indices, A, B) -> y
 * y[eid[p], :] = sum_d A[row, :, d] * B[indices[p], :, d]; y is (n_edges, h), fully written when
 * the plan's eid covers every edge, so the caller zero-fills it otherwise. */
int bpt_maskedmm_csr_forward(const bpt_plan *plan, const void *A, const void *B, void *y,
                             int h, int d, int dtype, void *stream);

/* graphop.cpp:108 maskedmm_csr_backward(row.., col.., A, B, dy) -> [dA, dB]
 * dA[r] = sum_{p in row r of plan_r} dy[eid[p]] * B[idx[p]];  dB likewise over plan_c with A. */
int bpt_maskedmm_csr_backward(const bpt_plan *plan_r, const bpt_plan *plan_c, const void *A, const void *B,
                              const void *dy, void *dA, void *dB, void *workspace, int64_t workspace_bytes,
                              int h, int d, int dtype, void *stream);

/* graphop.cpp:39  node_mul_edge_forward(row, indptr, eid, A, B) -> y;  B is (n_edges, d) */
int bpt_node_mul_edge_forward(const bpt_plan *plan, const void *A, const void *B, void *y,
                              int h, int d, int dtype, void *stream);

/* graphop.cpp:141 node_mul_edge_backward(row, indptr, eid, A, B, dy) -> [dA, dB] */
int bpt_node_mul_edge_backward(const bpt_plan *plan, const void *A, const void *B, const void *dy,
                               void *dA, void *dB, void *workspace, int64_t workspace_bytes,
                               int h, int d, int dtype, void *stream);

/* graphop.cpp:59  sparse_softmax_forward(row, indptr, eid, x) -> y   (softmax over each row's slots;
 * the running maximum starts at -1e9 as in graphop_kernel.cu:428).  The workspace (bpt_workspace_bytes with
 * BPT_OP_SOFTMAX_FWD, d = 1) holds the per-segment maxima and sums of the rows that the plan splits. */
int bpt_sparse_softmax_forward(const bpt_plan *plan, const void *x, void *y, void *workspace, int64_t workspace_bytes,
                               int h, int dtype, void *stream);

/* graphop.cpp:163 sparse_softmax_backward(row, indptr, eid, y, dy) -> dx   (workspace: BPT_OP_SOFTMAX_BWD) */
int bpt_sparse_softmax_backward(const bpt_plan *plan, const void *y, const void *dy, void *dx, void *workspace,
                                int64_t workspace_bytes, int h, int dtype, void *stream);

/* graphop.cpp:79  vector_spmm_forward(row, indptr, eid, indices, edata, x) -> y
 * y[r] = sum_p edata[eid[p]] * x[idx[p]];  every row of y is written (zero for empty rows). */
int bpt_vector_spmm_forward(const bpt_plan *plan, const void *edata, const void *x, void *y,
                            void *workspace, int64_t workspace_bytes, int h, int d, int dtype, void *stream);

/* y[r] += sum_p edata[eid[p]] * x[idx[p]]: bpt_vector_spmm_forward accumulating into y.  No counterpart in the reference
 * (it serves the q gradient of the fused rel_pos term).  Row-group kernels only: BPT_ERR_UNSUPPORTED unless the plan
 * carries row groups with grp_eids and the shape has specialised kernels; the caller then adds the plain result. */
int bpt_vector_spmm_accumulate(const bpt_plan *plan, const void *edata, const void *x, void *y,
                               void *workspace, int64_t workspace_bytes, int h, int d, int dtype, void *stream);

/* graphop.cpp:190 vector_spmm_backward(row.., col.., edata, dy, x) -> [dedata, dx]
 * dedata[eid[p]] = <dy[row], x[idx[p]]> over `plan`; dx[c] = sum over ALL rows c of `plan_t` of
 * edata[eid_t[p]] * dy[idx_t[p]].  (The reference launches the dx kernel with the grid of the
 * other side, graphop_kernel.cu:566,588, and drops trailing units when plan_t has more units;
 * this entry computes the complete gradient.) */
int bpt_vector_spmm_backward(const bpt_plan *plan, const bpt_plan *plan_t, const void *edata, const void *dy,
                             const void *x, void *dedata, void *dx, void *workspace, int64_t workspace_bytes,
                             int h, int d, int dtype, void *stream);

/* Score term of the relative positions, modules/attention.py:69-71 (embed_ak looked up per edge, then
 * node_mul_edge): bias[eid[p], head] = sum_d q[row, head, d] * table[type(p), d] over `plan`, whose rows are the
 * destinations (a plan built with the types as `indices`).  bias is float32 (n_edges, h) or larger; the (n_edges, d)
 * rows of the reference's nn.Embedding lookup are never materialised.
 * used_types == NULL: idx[p] is the edge TYPE of the edge in slot p (n_index_nodes = rows of table); compile-time
 * shapes only (BPT_ERR_UNSUPPORTED else).
 * used_types (n_used) int32: the edge types that occur, in any order without repeats, and idx[p] is the NUMBER of the
 * slot's type in that list (n_index_nodes = n_used).  The kernel keeps those rows of the table on chip and multiplies
 * on the matrix cores; h in {4, 8, 16}, d = 64, f32 or bf16, n_used <= 240 (BPT_ERR_UNSUPPORTED else).  In this form
 * bias must have n_edges + 1 rows: the kernel also clears row n_edges, the spare row of bpt_attention_forward.
 * With plan->bias_by_pair set (this form only) the result goes to bias[head * n_edges + eid[p]] instead, (h, n_edges)
 * floats, the layout bpt_attention_forward reads when its plan has the flag; eid[p] then has to be the attention
 * plan's pair number of the slot's edge. */
int bpt_rel_bias_forward(const bpt_plan *plan, const void *q, const void *table, const int32_t *used_types, int64_t n_used,
                         float *bias, int h, int d, int dtype, void *stream);

/* The same score term (modules/attention.py:69-71) for a term kept in the pair order of the attention kernels' tile plan:
 * `plan` is that plan (the destination side's, grp_R = 16), and the value of pair number t and a head goes to
 * bias[head * n_edges + t], (h, n_edges) floats, the layout bpt_attention_forward reads with plan->bias_by_pair.
 * pair_types (n_edges) int32: for pair number t, (number of its edge's type in used_types) | (its member index in the tile,
 * i.e. the position of its mask bit) << 8.  used_types (n_used) as for bpt_rel_bias_forward.  One wavefront per tile and
 * head multiplies the tile's 16 rows of q with all n_used table rows on the matrix cores, and every pair picks its value;
 * all per-pair reads and writes are contiguous.  h in {4, 8, 16}, d = 64, f32 or bf16, n_used <= 240, a plan with tiles
 * (BPT_ERR_UNSUPPORTED else). */
int bpt_rel_bias_forward_tiles(const bpt_plan *plan, const void *q, const void *table, const int32_t *used_types, int64_t n_used,
                               const int32_t *pair_types, float *bias, int h, int d, int dtype, void *stream);

/* Gradients of that score term, the backward of embed_ak + node_mul_edge in modules/attention.py:55-56,69-71 (autograd of
 * nn.Embedding and graphop.py's NodeMulEdgeFunction.backward), from ds (n_edges or more rows, h) float32 =
 * dL/d(score of the edge before scaling), which bpt_attention_backward returns in ds_out:
 *   dq[row, head, :] += sum over the slots p of the row of ds[eid[p], head] * table[type(p), :]      (added to dq)
 *   dtable[t, :]      = sum over the slots p of type t and the heads of ds[eid[p], head] * q[row(p), head, :]
 * without the (n_edges, d) gradient rows of the embedding lookup.  `plan` and used_types (n_used) as for
 * bpt_rel_bias_forward with used_types: idx[p] is the number of the slot's type.  used (n_types) int32 is the inverse:
 * for every type in used_types its number, -1 for the others, whose rows of dtable become zero.  dq and dtable have the
 * dtype of q and table.  workspace: bpt_rel_bias_backward_workspace_bytes(plan, n_used, h) bytes, 16-byte aligned.
 * With plan->bias_by_pair set, ds is read as (h, n_edges), ds[head * n_edges + eid[p]], the layout
 * bpt_attention_backward writes when its plan has the flag.
 * Row-owned sums in a fixed order, no atomics.  h in {4, 8, 16}, d = 64, f32 or bf16, n_used <= 240;
 * BPT_ERR_UNSUPPORTED otherwise (compose bpt_vector_spmm_forward calls instead). */
int64_t bpt_rel_bias_backward_workspace_bytes(const bpt_plan *plan, int64_t n_used, int h);
/* BPT_OK if bpt_rel_bias_backward has a kernel configuration for n_used types in use that the current device accepts (its
 * per-type sums live in LDS; many types with many heads need more than the 64 KB a runtime grants without asking), else
 * BPT_ERR_UNSUPPORTED.  Nothing is launched.  A caller asks BEFORE the forward, so that it can form the term's gradients with
 * bpt_vector_spmm_forward calls from the start instead of finding out in the backward. */
int bpt_rel_bias_backward_supported(int64_t n_used, int h, int d, int dtype);
int bpt_rel_bias_backward(const bpt_plan *plan, const float *ds, const void *q, const void *table, const int32_t *used,
                          const int32_t *used_types, int64_t n_types, int64_t n_used, void *dq, void *dtable, void *workspace,
                          int64_t workspace_bytes, int h, int d, int dtype, void *stream);

/* Fused attention layer core = modules/attention.py:66-77:
 *   o[dst] = sum_{e: src->dst} drop( softmax_dst( (q[dst].k[src] + bias[e]) * scale ) )[e] * v[src]
 * plan_in: rows = destinations (the reference's COL/INDPTR_C/in_csr), plan_out: rows = sources.
 * lse (n, h) float32 receives the base-2 log-sum-exp of the scaled scores, needed by backward.
 * f32 and bf16 only (accumulation in f32).
 * bias: NULL, or float32 (n_edges + 1, h): per edge and head, added to q.k before scaling (the rel_pos term,
 * bpt_rel_bias_forward); row n_edges is a spare row that is read for absent pairs and never used.  With
 * plan_in->bias_by_pair set: float32 (h, n_edges) in the plan's pair order (see bpt_plan; tile kernels only,
 * BPT_ERR_PLAN where they do not run).  Needs the row groups with grp_eids (BPT_ERR_UNSUPPORTED / BPT_ERR_PLAN
 * without them).
 * dropout_p in [0, 1): dropout on the attention probabilities (attention.py:73); 0 = none.  Each (edge, head) is
 * kept with probability 1 - p and scaled by 1 / (1 - p); the decision is a hash of (dropout_seed, edge id, head),
 * so it does not depend on the plan and backward only needs the same p and seed.  Needs the row groups with
 * grp_eids (BPT_ERR_UNSUPPORTED / BPT_ERR_PLAN without them). */
int bpt_attention_forward(const bpt_plan *plan_in, const void *q, const void *k, const void *v, const float *bias,
                          void *o, float *lse, void *workspace, int64_t workspace_bytes,
                          float scale, float dropout_p, uint64_t dropout_seed, int h, int d, int dtype, void *stream);

/* Backward of bpt_attention_forward.  With bias, ds_out (float32 (n_edges + 1, h), row n_edges spare; with
 * plan_in->bias_by_pair (h, n_edges), laid out like bias) receives
 * dL/d(q.k + bias) of every edge and head, from which the caller forms the gradients of what produced the bias
 * (for rel_pos: dq += sum_e ds[e] * table[type(e)], dtable[t] = sum_{e of type t} sum_h ds[e, h] * q[dst(e), h]);
 * bias and ds_out are both given or both NULL. */
int bpt_attention_backward(const bpt_plan *plan_in, const bpt_plan *plan_out, const void *q, const void *k,
                           const void *v, const float *bias, const void *o, const void *d_o, const float *lse,
                           void *dq, void *dk, void *dv, float *ds_out, void *workspace, int64_t workspace_bytes,
                           float scale, float dropout_p, uint64_t dropout_seed, int h, int d, int dtype, void *stream);

/* bpt_attention_forward for callers that cannot allocate device memory (code under HIP graph capture, serving
 * loops that forbid it, harnesses that fail on any hipMalloc).  No counterpart in the reference.  Same arguments,
 * kernels and results as bpt_attention_forward, except that the workspace (partial rows of the nodes that the
 * plan splits) is a static device array of BPT_NOALLOC_SCRATCH_BYTES inside the library instead of an argument;
 * the call allocates and frees nothing (inputs and outputs are still the caller's).  A plan that needs more
 * (bpt_workspace_bytes(BPT_OP_ATTN_FWD, ...) > BPT_NOALLOC_SCRATCH_BYTES) is refused with BPT_ERR_SCRATCH and
 * nothing is launched.  The first call on a device looks up that device's copy of the array (no allocation,
 * but not capturable: make one call before capturing).  Every call on a device uses that device's one array:
 * calls that overlap on one GPU (two streams, two threads) race on it; calls on one stream are ordered.
 * Nothing in the array has to start at zero: every slot that is read has been written by the same call. */
#define BPT_NOALLOC_SCRATCH_BYTES (16 * 1024 * 1024)
int bpt_attention_forward_noalloc(const bpt_plan *plan_in, const void *q, const void *k, const void *v,
                                  const float *bias, void *o, float *lse, float scale, float dropout_p,
                                  uint64_t dropout_seed, int h, int d, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BPTATTN_H */
