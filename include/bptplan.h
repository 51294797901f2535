/* bptplan.h — C ABI of libbptplan.so: launch plans and row groups built on the GPU.
 *
 * The reference hands every op the int64 CSR arrays (row, indptr, eid, indices) of graph/base.py:71-86, which it
 * builds on the host for every batch and copies to the device (graph/base.py:84-86).  The kernels of bptattn.h
 * read a `bpt_plan` instead.  include/bptgraph.h derives that plan on the host (one device-to-host copy of the
 * index arrays per new graph plus tens of milliseconds of host work); the functions here derive an equivalent plan
 * from the same device arrays without leaving the GPU: sorts and prefix sums (rocPRIM) plus small kernels, all on
 * the caller's stream (a hipStream_t passed as void*, NULL = the default stream).  Nothing is allocated: outputs and the workspace are the caller's, sized by the bounds below.
 * The only host <-> device traffic is the caller's own read of the 16-int `info` blocks afterwards (they hold the
 * actual sizes and the validation result).  No counterpart in the reference.
 *
 * Every function returns 0, a negative bpt_status of bptattn.h (bad argument, nothing launched) or a positive
 * hipError_t.  Malformed graph arrays do not fault: the validation kernels record an error in info[BPT_PI_ERR]
 * and every later kernel of the call returns at once.
 */
#ifndef BPTPLAN_H
#define BPTPLAN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* indices into the int32[16] info block of bpt_plan_build_device */
enum { BPT_PI_ERR = 0,        /* 0 ok, 1 id out of range, 2 row / indptr not monotone, 3 sizes out of the int32 range */
       BPT_PI_N_ITEMS = 1, BPT_PI_N_HEAVY = 2, BPT_PI_N_SLOTS = 3, BPT_PI_MAX_DEGREE = 4,
       BPT_PI_FLAGS = 5 };    /* bit 0: the units cover every edge slot and eid is a permutation */
/* indices into the int32[16] info block of bpt_plan_group_device */
enum { BPT_GI_N_GROUPS = 0, BPT_GI_N_ENTRIES = 1, BPT_GI_MAX_CHUNK = 2 };

/* Edge lists of the reference's graph builder on the device, in the reference's order (kind 0: BinaryPartition,
 * builder.pyx:41-116, a = step, b = clip_dist; 1: FullyConnected, :243-274, a = window; 2: OpenAISparse, :171-199,
 * a = stride, b = c; same arguments as bptg_graph_fill, bptgraph.h).  Two calls: bpt_graph_count_device writes
 * offsets (length + 1 int32: offsets[i] = position of token i's first edge, offsets[length] = number of edges; the
 * caller reads that one number to size the lists; workspace: 8 * (length + 1) bytes + 1 MiB are enough), then
 * bpt_graph_fill_device writes src / dst (+ v_shift) and etype (n_edges int64 each; nothing is written unless n_edges
 * equals offsets[length]). */
int bpt_graph_count_device(int kind, int64_t length, int triu, int64_t a, int64_t b, int32_t *offsets, void *workspace,
                           int64_t workspace_bytes, void *stream);
int bpt_graph_fill_device(int kind, int64_t length, int triu, int64_t a, int64_t b, int64_t v_shift,
                          const int32_t *offsets, int64_t n_edges, int64_t *src, int64_t *dst, int64_t *etype,
                          void *stream);

/* One CSR side of graph/base.py:71-86 from an edge list on the device: the edges grouped by rows[e], ascending edge
 * id inside a row (the order of bptg_build_csr, bptgraph.h), in the reference's int64 layout: indptr (n_nodes + 1),
 * indices (n_edges: cols of the slots), eid (n_edges); and the chunked units of builder.pyx:305-321 (partition_csr):
 * unit_row (bounds[0]), unit_ptr (bounds[0] + 1), unit_ptr[n_units] = n_edges, no unit for an empty row.
 * bpt_csr_device_bounds: bounds[0] = most units there can be, bounds[1] = workspace bytes.
 * info: int32[16]; info[0] = 0, or 1 when a row / column id is outside [0, n_nodes) (then nothing else is valid);
 * info[1] = number of units. */
int bpt_csr_device_bounds(int64_t n_edges, int64_t n_nodes, int32_t chunk_size, int64_t bounds[2]);
int bpt_csr_build_device(const int64_t *rows, const int64_t *cols, int64_t n_edges, int64_t n_nodes, int32_t chunk_size,
                         int64_t *indptr, int64_t *indices, int64_t *eid, int64_t *unit_row, int64_t *unit_ptr,
                         int32_t *info, void *workspace, int64_t workspace_bytes, void *stream);

/* Upper bounds of the data-dependent sizes, for the caller's allocations:
 *   bounds[0] = items      (rows of 4 int32)      n_rows + n_edges / seg_len
 *   bounds[1] = heavy rows (rows of 3 int32)      n_edges / (seg_len + 1)
 *   bounds[2] = groups     (R > 0)                ceil(bounds[0] / R)
 *   bounds[3] = workspace bytes that any of the three calls below needs for these sizes. */
int bpt_plan_device_bounds(int64_t n_units, int64_t n_edges, int64_t n_rows, int32_t seg_len, int32_t R,
                           int64_t bounds[4]);

/* Base plan of one CSR side = what bptg_plan_fill (bptgraph.h) computes, bit for bit: the row-level rowptr
 * (n_rows + 1), idx32 / eid32 (n_edges), the work items (row, begin, end, slot) in locality order and the heavy
 * rows.  row / indptr_units (n_units, n_units + 1), eid and indices (n_edges; indices may be NULL) are the
 * reference's int64 device arrays.  items / heavy hold bounds[0] / bounds[1] rows; info: int32[16]. */
int bpt_plan_build_device(const int64_t *row, const int64_t *indptr_units, int64_t n_units, const int64_t *eid,
                          const int64_t *indices, int64_t n_edges, int64_t n_rows, int64_t n_index_nodes,
                          int32_t seg_len, int32_t *rowptr, int32_t *idx32, int32_t *eid32, int32_t *items,
                          int32_t *heavy, int32_t *info, void *workspace, int64_t workspace_bytes, void *stream);

/* Row groups of R rows over a base plan (the arrays bpt_plan's grp_* fields point at).  The items are taken in
 * the order of their largest neighbour id, R consecutive ones form a group; the groups are numbered by the smallest
 * neighbour id any member reads (groups that read the same rows end up on the same XCD at about the same time), cut
 * into 8 ranges of equal work (one per XCD) and ordered by decreasing work inside a range (work: the group's pairs plus a
 * fixed cost; for R = 16, the tile kernels' plans, its number of blocks of 16 entries plus one, which is what a tile costs the
 * matrix kernels whether a third or all of a block's pairs exist); the entries of a group
 * (its distinct neighbours) are in ascending neighbour order (by_mask = 0), sorted by member mask, larger first
 * (by_mask = 1), or by (neighbour mod 16, neighbour) (by_mask = 2: every group walks the id range in the same
 * interleaved way, so groups that run side by side ask for a shared row at about the same step).  by_mask + 4: the
 * groups of a range keep their locality order instead of the order by decreasing work (fewer bytes from HBM: the groups
 * that run at the same time read the same rows; longer tail: the last groups of a range are not the lightest).
 * plan_info is the info block bpt_plan_build_device wrote (device memory; groups are only built when its flags
 * say that the plan covers every edge, else n_groups = 0).  max_items = bounds[0].
 *   members   (bounds[2], R, 2)    grp_ptr (bounds[2] + 1)      entries (n_edges + 1, 4)
 *   pair_eid  (n_edges)            grp_eids ((n_edges + 8) * R)  chunks (9)        group_info: int32[16] */
int bpt_plan_group_device(const int32_t *items, const int32_t *idx32, const int32_t *eid32, const int32_t *plan_info,
                          int64_t max_items, int64_t n_edges, int64_t n_index_nodes, int32_t seg_len, int32_t R,
                          int32_t by_mask, int32_t *members, int32_t *grp_ptr, int32_t *entries, int32_t *pair_eid,
                          int32_t *grp_eids, int32_t *chunks, int32_t *group_info, void *workspace,
                          int64_t workspace_bytes, void *stream);

/* grp_pairs of the destination-side groups: for every (entry, member) the position entry' * R_src + member' of the
 * same edge in the source-side groups, the spare position (n_entries_src + pad_entries) * R_src - 1 where the
 * entry has no such member and in pad_entries entries of padding.  pairs: (n_edges + pad_entries) * R_dst int32. */
int bpt_plan_link_device(const int32_t *grp_eids_dst, const int32_t *group_info_dst, int32_t R_dst,
                         const int32_t *grp_eids_src, const int32_t *group_info_src, int32_t R_src, int64_t n_edges,
                         int32_t pad_entries, int32_t *pairs, void *workspace, int64_t workspace_bytes,
                         void *stream);

#ifdef __cplusplus
}
#endif
#endif
