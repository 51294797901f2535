/*
 * libbptgraph — host-side (CPU) integer half of the BPT graph-attention path, C ABI.
 *
 * Replaces the reference's Cython module `graphbuilder` (graph_builder/builder.pyx) and the
 * DGL adjacency export used by graph/base.py:71-86.  Everything here is host code working on
 * caller-owned buffers: the library never allocates memory it hands out and never throws.
 * Every function returns 0 on success or a negative bptg_status.
 *
 * Calling pattern: `*_sizes` tells how large the output arrays must be, the caller allocates
 * them (numpy / torch / malloc), `*_fill` writes them.
 */
#ifndef BPTGRAPH_H
#define BPTGRAPH_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    BPTG_OK = 0,
    BPTG_ERR_NULL = -1,          /* a required pointer is NULL */
    BPTG_ERR_SIZE = -2,          /* negative / inconsistent size, or a count exceeding int32 */
    BPTG_ERR_ORDER = -3,         /* `row` not non-decreasing or `indptr` not non-decreasing */
    BPTG_ERR_RANGE = -4,         /* a row id, index or edge id outside its valid range */
    BPTG_ERR_ARG = -5            /* invalid scalar argument (e.g. chunk_size <= 0) */
} bptg_status;

const char *bptg_strerror(int status);

/* ---- graph construction --------------------------------------------------------------------
 * kind 0: BinaryPartition(length, triu, step=a, clip_dist=b)   builder.pyx:23-152
 * kind 1: FullyConnected(length, triu, window=a)               builder.pyx:228-303
 * kind 2: OpenAISparse(length, stride=a, c=b) (causal only)    builder.pyx:154-225
 * Edge e goes src[e] -> dst[e]; the order of edges is part of the contract (edge id = position,
 * graph/lm.py:96-98).  lvl_sizes receives n_levels entries (nodes per tree level). */
int bptg_graph_sizes(int kind, int64_t length, int triu, int64_t a, int64_t b,
                     int64_t *n_nodes, int64_t *n_edges, int64_t *n_levels);
int bptg_graph_fill(int kind, int64_t length, int triu, int64_t a, int64_t b, int64_t v_shift,
                    int64_t *src, int64_t *dst, int64_t *etype, int64_t *pos, int64_t *lvl_sizes);

/* ---- partition_csr (builder.pyx:305-321 == graph_kernel/part_csr.py:13-27) -----------------
 * Splits every row's slot range into chunks of at most chunk_size slots.  n_indptr = rows + 1. */
int bptg_partition_csr_count(const int64_t *indptr, int64_t n_indptr, int64_t chunk_size, int64_t *n_units);
int bptg_partition_csr_fill(const int64_t *indptr, int64_t n_indptr, int64_t chunk_size,
                            int64_t *row, int64_t *indptr_units);

/* ---- CSR with edge ids (what graph/base.py:72,79 obtains from DGL) -------------------------
 * Stable counting sort of the edge list by `rows`: indptr (n+1), indices[p] = cols[eid[p]],
 * eid[p] ascending inside each row.  For the out-CSR pass rows=src, cols=dst; in-CSR swapped. */
int bptg_build_csr(const int64_t *rows, const int64_t *cols, int64_t n_edges, int64_t n_nodes,
                   int64_t *indptr, int64_t *indices, int64_t *eid);

/* ---- launch plan ----------------------------------------------------------------------------
 * The reference kernels receive only chunked units (row[u], indptr[u..u+1]); a row spread over
 * several units is combined there with float atomics.  The HIP library instead gives every row
 * to one wavefront, and rows longer than seg_len edges to several wavefronts whose partial
 * results are combined in a fixed order.  The plan derives that work list from the reference's
 * arguments once per graph:
 *   rowptr  int32[n_nodes+1]   row-level slot ranges recovered from the units
 *   idx     int32[n_edges]     `indices` narrowed to 32 bit (zeros when indices == NULL)
 *   eid     int32[n_edges]
 *   items   int32[n_items*4]   (row, begin, end, slot); slot < 0: the item owns its whole row
 *                              and writes results directly; slot >= 0: partial result number
 *   heavy   int32[n_heavy*3]   (row, first_slot, n_slots) for every split row
 * Every node gets at least one item (empty rows too) so kernels can write all outputs.
 * When `indices` is given the items are ordered by the smallest neighbour id they touch (ties in row
 * order) so that consecutive items share neighbours; otherwise they are in row order.
 * flags bit0: eid is a permutation of 0..n_edges-1 (every edge output gets written). */
typedef struct {
    int64_t n_items, n_heavy, n_slots, max_degree, flags;
} bptg_plan_info;

int bptg_plan_sizes(const int64_t *row, const int64_t *indptr_units, int64_t n_units,
                    int64_t n_nodes, int64_t seg_len, bptg_plan_info *info);
int bptg_plan_fill(const int64_t *row, const int64_t *indptr_units, int64_t n_units,
                   const int64_t *eid, const int64_t *indices, int64_t n_edges,
                   int64_t n_nodes, int64_t n_index_nodes, int64_t seg_len,
                   int32_t *rowptr, int32_t *idx32, int32_t *eid32, int32_t *items, int32_t *heavy,
                   bptg_plan_info *info);

/* ---- row groups ------------------------------------------------------------------------------
 * Clusters the plan's items (rows / row segments) into groups of at most R (<= 16) members that read
 * mostly the same neighbour rows, so that one wavefront can load each neighbour row once for all of
 * them.  Inputs are the arrays bptg_plan_fill produced.  Outputs (caller allocates the upper bounds
 * given in brackets):
 *   members  int32[n_items*R*2]   per group R x (row, slot); row = -1 for an unused member
 *   grp_ptr  int32[n_items+1]     entry range of each group
 *   entries  int32[n_edges*4]     (neighbour id, member bit mask, first pair, 0)
 *   pair_eid int32[n_edges]       edge id of every pair; pairs are numbered entry by entry, members
 *                                 ascending, and every edge of the plan appears exactly once
 *   slot_eid int32[n_edges*R]     or NULL: edge id of (entry, member) at [entry*R + member], -1 where the
 *                                 entry's mask has no such member (the first n_entries*R elements are written)
 *   chunks   int32[9]             groups chunks[x] .. chunks[x+1]-1 go to XCD x (contiguous, about equal work)
 * order_mode: low two bits = order of the groups inside a chunk — 0 locality, 1 at-least-average work first
 * then the small ones, 2 decreasing work; + 4 = inside a group, entries with equal member masks are made
 * adjacent (larger masks first, neighbour order kept among equal masks) instead of plain neighbour order;
 * + 8 = aligned order (overrides + 4): going through the groups in locality order, a neighbour keeps the position
 * it had in the last group that read it whenever that position is free and the rest fill the gaps, so that
 * wavefronts running side by side ask for a shared row at about the same time.
 * max_pairs: no item joins a group whose edges would then number more than this (0 = no limit); it bounds
 * the work of the wavefront that walks the group.
 * A neighbour that a member reaches through several parallel edges gets one entry per multiplicity. */
int bptg_group_plan(const int32_t *items, int64_t n_items, const int32_t *idx32, const int32_t *eid32,
                    int64_t n_edges, int64_t n_index_nodes, int32_t R, int32_t window, int32_t order_mode,
                    int32_t max_pairs, int32_t *members, int32_t *grp_ptr, int32_t *entries, int32_t *pair_eid, int32_t *slot_eid,
                    int32_t *chunks, int64_t *n_groups, int64_t *n_entries);

/* For every (entry, member) of the destination-side groups (slot_eid_dst: n_entries_dst * R_dst edge ids, -1 = absent)
 * the position entry' * R_src + member' of the same edge in the source-side groups; where absent, and in the
 * pad_entries * R_dst elements of padding, the spare position (n_entries_src + pad_entries) * R_src - 1.
 * pairs: int32[(n_entries_dst + pad_entries) * R_dst].  BPTG_ERR_RANGE unless the source side holds every edge
 * 0 .. n_edges-1 exactly once. */
int bptg_link_groups(const int32_t *slot_eid_dst, int64_t n_entries_dst, int32_t R_dst, const int32_t *slot_eid_src,
                     int64_t n_entries_src, int32_t R_src, int64_t n_edges, int32_t pad_entries, int32_t *pairs);

#ifdef __cplusplus
}
#endif
#endif /* BPTGRAPH_H */
