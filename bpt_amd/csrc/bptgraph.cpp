// libbptgraph: host-side integer half of the BPT graph-attention path (see include/bptgraph.h).
//
// Graph generators reproduce the edge ORDER of the reference bit for bit because edge ids are
// positions in that order (graph/lm.py:96-98) and every (E, .) tensor on the device is addressed
// by edge id.  Generators are written against a sink so the same walk first counts and then
// writes straight into caller-owned int64 arrays (no intermediate vectors, no allocation).
#include "../../include/bptgraph.h"

#include <algorithm>
#include <climits>
#include <cstring>
#include <vector>

namespace {

struct CountSink {
    int64_t n = 0;
    inline void operator()(int64_t, int64_t, int64_t) { ++n; }
};

struct WriteSink {
    int64_t *src, *dst, *etype;
    int64_t shift;
    int64_t n = 0;
    inline void operator()(int64_t s, int64_t d, int64_t t) {
        if (src) src[n] = s + shift;
        if (dst) dst[n] = d + shift;
        if (etype) etype[n] = t;
        ++n;
    }
};

// Level table of the binary partition tree: level 0 = tokens, each next level halves (rounding
// up) until a single root remains (builder.pyx:43-57).
struct Levels {
    std::vector<int64_t> size, offset;
    int64_t n_nodes = 0;
    explicit Levels(int64_t length) {
        int64_t n = length;
        while (n >= 2) {
            size.push_back(n);
            offset.push_back(n_nodes);
            n_nodes += n;
            n = (n + 1) >> 1;
        }
        size.push_back(1);
        offset.push_back(n_nodes);
        n_nodes += 1;
    }
    int64_t count() const { return (int64_t)size.size(); }
};

// builder.pyx:64-116.  For token `tok` two cursors walk outwards, `step` nodes per side per
// level, then move one level up.  When a cursor stops on a node whose sibling was already
// taken, the parent would overlap it, so the first neighbour on the next level is that child
// itself (taken from the level below).  The right-hand bound is checked against the CURRENT
// level even in that case — for odd level sizes this yields the first node of the current level
// instead of a child; kept, since edge lists must match the reference exactly.
template <class Sink>
void walk_binary_partition(const Levels &lv, int64_t length, bool causal, int64_t step, int64_t clip, Sink &out) {
    const int64_t n_lvl = lv.count();
    for (int64_t tok = 0; tok < length; ++tok) {
        int64_t left = tok - 1, right = tok + 1, ancestor = tok;
        bool left_child = false, right_child = false;
        for (int64_t j = 0; j < n_lvl; ++j) {
            const int64_t type0 = (2 * step + 1) * std::min(j, clip);
            for (int64_t s = 0; s < step; ++s) {
                if (!causal && right < lv.size[j]) {
                    out(right_child ? lv.offset[j - 1] + 2 * right + 1 : lv.offset[j] + right, tok, type0 + 2 * (s + 1));
                    right_child = false;
                }
                ++right;
                if (left >= 0) {
                    out(left_child ? lv.offset[j - 1] + 2 * left : lv.offset[j] + left, tok, type0 + 2 * s + 1);
                    left_child = false;
                }
                --left;
            }
            if ((left & 1) == 0) left_child = true;
            if ((right & 1) == 1) right_child = true;
            right >>= 1;
            left >>= 1;                       // arithmetic shift: stays negative once it is
            out(tok, lv.offset[j] + ancestor, type0);   // self loop (j = 0) / token -> ancestor
            ancestor >>= 1;
        }
    }
}

// builder.pyx:243-274
template <class Sink>
void walk_fully_connected(int64_t length, bool causal, int64_t window, Sink &out) {
    const int64_t reach = std::min(length, window + 1);
    for (int64_t i = 0; i < length; ++i) {
        out(i, i, 0);
        for (int64_t j = 1; j < reach; ++j) {
            if (i >= j) out(i - j, i, 2 * j - 1);
            if (!causal && i + j < length) out(i + j, i, 2 * j);
        }
        out(i, length, 0);
    }
}

// builder.pyx:171-199
template <class Sink>
void walk_openai_sparse(int64_t length, int64_t stride, int64_t c, Sink &out) {
    for (int64_t i = 0; i < length; ++i) {
        for (int64_t j = (i / stride) * stride; j <= i; ++j) out(j, i, 0);
        for (int64_t blk = 1; blk <= i / stride; ++blk)
            for (int64_t k = stride * blk - c; k < stride * blk; ++k) out(k, i, 0);
        out(i, length, 0);
    }
}

bool graph_args_ok(int kind, int64_t length, int64_t a, int64_t b) {
    if (length < 1) return false;
    if (kind == 0) return a >= 1 && b >= 0;
    if (kind == 1) return a >= 0;
    if (kind == 2) return a >= 1 && b >= 0 && b <= a;
    return false;
}

template <class Sink>
void walk(int kind, int64_t length, int triu, int64_t a, int64_t b, Sink &sink) {
    if (kind == 0) {
        Levels lv(length);
        walk_binary_partition(lv, length, triu != 0, a, b, sink);
    } else if (kind == 1) {
        walk_fully_connected(length, triu != 0, a, sink);
    } else {
        walk_openai_sparse(length, a, b, sink);
    }
}

}  // namespace

extern "C" {

const char *bptg_strerror(int status) {
    switch (status) {
        case BPTG_OK: return "ok";
        case BPTG_ERR_NULL: return "required pointer is NULL";
        case BPTG_ERR_SIZE: return "negative, inconsistent or too large size";
        case BPTG_ERR_ORDER: return "units must be grouped by row: `row` and `indptr` non-decreasing";
        case BPTG_ERR_RANGE: return "row id, index or edge id out of range";
        case BPTG_ERR_ARG: return "invalid scalar argument";
        default: return "unknown bptgraph status";
    }
}

int bptg_graph_sizes(int kind, int64_t length, int triu, int64_t a, int64_t b,
                     int64_t *n_nodes, int64_t *n_edges, int64_t *n_levels) {
    if (!n_nodes || !n_edges || !n_levels) return BPTG_ERR_NULL;
    if (!graph_args_ok(kind, length, a, b)) return BPTG_ERR_ARG;
    if (kind == 0) {
        Levels lv(length);
        *n_nodes = lv.n_nodes;
        *n_levels = lv.count();
    } else {
        *n_nodes = length + 1;
        *n_levels = 2;
    }
    CountSink cnt;
    walk(kind, length, triu, a, b, cnt);
    *n_edges = cnt.n;
    return BPTG_OK;
}

int bptg_graph_fill(int kind, int64_t length, int triu, int64_t a, int64_t b, int64_t v_shift,
                    int64_t *src, int64_t *dst, int64_t *etype, int64_t *pos, int64_t *lvl_sizes) {
    if (!graph_args_ok(kind, length, a, b)) return BPTG_ERR_ARG;
    if (src || dst || etype) {
        WriteSink w{src, dst, etype, v_shift};
        walk(kind, length, triu, a, b, w);
    }
    if (kind == 0) {
        Levels lv(length);
        if (lvl_sizes)
            for (int64_t j = 0; j < lv.count(); ++j) lvl_sizes[j] = lv.size[j];
        if (pos) {
            // builder.pyx:46,57-62: last token covered by the node, clipped to the sequence
            int64_t p = 0;
            for (int64_t j = 0; j + 1 < lv.count(); ++j)
                for (int64_t i = 0; i < lv.size[j]; ++i) pos[p++] = std::min(((i + 1) << j) - 1, length - 1);
            pos[p] = length - 1;
        }
    } else {
        if (lvl_sizes) { lvl_sizes[0] = length; lvl_sizes[1] = 1; }
        if (pos) {
            for (int64_t i = 0; i < length; ++i) pos[i] = i;
            pos[length] = (kind == 1) ? length : length - 1;   // builder.pyx:274 / :199
        }
    }
    return BPTG_OK;
}

int bptg_partition_csr_count(const int64_t *indptr, int64_t n_indptr, int64_t chunk_size, int64_t *n_units) {
    if (!indptr || !n_units) return BPTG_ERR_NULL;
    if (n_indptr < 1) return BPTG_ERR_SIZE;
    if (chunk_size < 1) return BPTG_ERR_ARG;
    int64_t n = 0;
    for (int64_t r = 0; r + 1 < n_indptr; ++r) {
        const int64_t deg = indptr[r + 1] - indptr[r];
        if (deg < 0) return BPTG_ERR_ORDER;
        n += (deg + chunk_size - 1) / chunk_size;
    }
    *n_units = n;
    return BPTG_OK;
}

int bptg_partition_csr_fill(const int64_t *indptr, int64_t n_indptr, int64_t chunk_size,
                            int64_t *row, int64_t *indptr_units) {
    if (!indptr || !indptr_units) return BPTG_ERR_NULL;
    if (n_indptr < 1) return BPTG_ERR_SIZE;
    if (chunk_size < 1) return BPTG_ERR_ARG;
    int64_t u = 0;
    for (int64_t r = 0; r + 1 < n_indptr; ++r)
        for (int64_t p = indptr[r]; p < indptr[r + 1]; p += chunk_size) {
            if (!row) return BPTG_ERR_NULL;
            row[u] = r;
            indptr_units[u] = p;
            ++u;
        }
    indptr_units[u] = indptr[n_indptr - 1];
    return BPTG_OK;
}

int bptg_build_csr(const int64_t *rows, const int64_t *cols, int64_t n_edges, int64_t n_nodes,
                   int64_t *indptr, int64_t *indices, int64_t *eid) {
    if (!indptr || (n_edges > 0 && (!rows || !cols || !indices || !eid))) return BPTG_ERR_NULL;
    if (n_edges < 0 || n_nodes < 0) return BPTG_ERR_SIZE;
    std::memset(indptr, 0, sizeof(int64_t) * (size_t)(n_nodes + 1));
    for (int64_t e = 0; e < n_edges; ++e) {
        if (rows[e] < 0 || rows[e] >= n_nodes || cols[e] < 0 || cols[e] >= n_nodes) return BPTG_ERR_RANGE;
        ++indptr[rows[e] + 1];
    }
    for (int64_t r = 0; r < n_nodes; ++r) indptr[r + 1] += indptr[r];
    std::vector<int64_t> cursor(indptr, indptr + n_nodes);
    for (int64_t e = 0; e < n_edges; ++e) {          // ascending e => ascending eid inside a row
        const int64_t p = cursor[rows[e]]++;
        indices[p] = cols[e];
        eid[p] = e;
    }
    return BPTG_OK;
}

// ---- plan --------------------------------------------------------------------------------------

static int plan_scan(const int64_t *row, const int64_t *ip, int64_t n_units, int64_t n_nodes, int64_t seg_len,
                     int32_t *rowptr, int32_t *items, int32_t *heavy, bptg_plan_info *info) {
    if (!info || (n_units > 0 && (!row || !ip))) return BPTG_ERR_NULL;
    if (n_units < 0 || n_nodes < 0 || n_nodes >= INT32_MAX) return BPTG_ERR_SIZE;
    if (seg_len < 1) return BPTG_ERR_ARG;
    const int64_t first = n_units ? ip[0] : 0, last = n_units ? ip[n_units] : 0;
    if (first < 0 || last >= INT32_MAX) return BPTG_ERR_SIZE;
    for (int64_t u = 0; u < n_units; ++u) {
        if (row[u] < 0 || row[u] >= n_nodes) return BPTG_ERR_RANGE;
        if (u && row[u] < row[u - 1]) return BPTG_ERR_ORDER;
        if (ip[u + 1] < ip[u]) return BPTG_ERR_ORDER;
    }
    int64_t n_items = 0, n_heavy = 0, n_slots = 0, max_deg = 0;
    int64_t u = 0;
    for (int64_t r = 0; r < n_nodes; ++r) {
        const int64_t u0 = u;
        while (u < n_units && row[u] == r) ++u;
        const int64_t begin = (u0 < n_units) ? ip[u0] : last;
        const int64_t end = (u > u0) ? ip[u] : begin;
        const int64_t deg = end - begin;
        max_deg = std::max(max_deg, deg);
        if (rowptr) rowptr[r] = (int32_t)begin;
        if (deg <= seg_len) {
            if (items) {
                int32_t *it = items + 4 * n_items;
                it[0] = (int32_t)r; it[1] = (int32_t)begin; it[2] = (int32_t)end; it[3] = -1;
            }
            ++n_items;
        } else {
            const int64_t n_seg = (deg + seg_len - 1) / seg_len;
            if (heavy) {
                int32_t *hv = heavy + 3 * n_heavy;
                hv[0] = (int32_t)r; hv[1] = (int32_t)n_slots; hv[2] = (int32_t)n_seg;
            }
            for (int64_t s = 0; s < n_seg; ++s) {
                if (items) {
                    int32_t *it = items + 4 * n_items;
                    it[0] = (int32_t)r;
                    it[1] = (int32_t)(begin + s * seg_len);
                    it[2] = (int32_t)std::min(end, begin + (s + 1) * seg_len);
                    it[3] = (int32_t)(n_slots + s);
                }
                ++n_items;
            }
            ++n_heavy;
            n_slots += n_seg;
        }
    }
    if (rowptr) rowptr[n_nodes] = (int32_t)last;
    if (n_items >= INT32_MAX) return BPTG_ERR_SIZE;
    info->n_items = n_items;
    info->n_heavy = n_heavy;
    info->n_slots = n_slots;
    info->max_degree = max_deg;
    info->flags = 0;
    return BPTG_OK;
}

int bptg_plan_sizes(const int64_t *row, const int64_t *indptr_units, int64_t n_units,
                    int64_t n_nodes, int64_t seg_len, bptg_plan_info *info) {
    return plan_scan(row, indptr_units, n_units, n_nodes, seg_len, nullptr, nullptr, nullptr, info);
}

int bptg_plan_fill(const int64_t *row, const int64_t *indptr_units, int64_t n_units,
                   const int64_t *eid, const int64_t *indices, int64_t n_edges,
                   int64_t n_nodes, int64_t n_index_nodes, int64_t seg_len,
                   int32_t *rowptr, int32_t *idx32, int32_t *eid32, int32_t *items, int32_t *heavy,
                   bptg_plan_info *info) {
    if (!rowptr || !items || (n_edges > 0 && (!eid || !idx32 || !eid32))) return BPTG_ERR_NULL;
    if (n_edges < 0 || n_edges >= INT32_MAX || n_index_nodes < 0 || n_index_nodes >= INT32_MAX) return BPTG_ERR_SIZE;
    int st = plan_scan(row, indptr_units, n_units, n_nodes, seg_len, rowptr, items, heavy, info);
    if (st != BPTG_OK) return st;
    if (info->n_heavy > 0 && !heavy) return BPTG_ERR_NULL;
    // the units must address slots inside the eid / indices arrays
    if (n_units > 0 && indptr_units[n_units] > n_edges) return BPTG_ERR_RANGE;
    std::vector<uint8_t> seen((size_t)n_edges, 0);
    bool perm = (n_units > 0) ? (indptr_units[0] == 0 && indptr_units[n_units] == n_edges) : (n_edges == 0);
    for (int64_t p = 0; p < n_edges; ++p) {
        const int64_t e = eid[p];
        if (e < 0 || e >= n_edges) return BPTG_ERR_RANGE;
        if (seen[(size_t)e]) perm = false;
        seen[(size_t)e] = 1;
        eid32[p] = (int32_t)e;
        if (indices) {
            const int64_t c = indices[p];
            if (c < 0 || c >= n_index_nodes) return BPTG_ERR_RANGE;
            idx32[p] = (int32_t)c;
        } else {
            idx32[p] = 0;
        }
    }
    info->flags = perm ? 1 : 0;
    // Locality order: consecutive work items should touch the same neighbour rows, because the
    // kernels hand consecutive items to the same XCD (shared L2) at about the same time.  Key =
    // smallest neighbour id of the item.  For the binary-partition graphs this interleaves every
    // span node with the tokens it covers and spreads the long token rows evenly over the item
    // list (in plain row order all token rows come first and half of the XCDs get all of them).
    if (indices && info->n_items > 1) {
        const int64_t n_items = info->n_items;
        std::vector<int32_t> key((size_t)n_items), order((size_t)n_items);
        for (int64_t i = 0; i < n_items; ++i) {
            const int32_t *it = items + 4 * i;
            int32_t k = it[0] < n_index_nodes ? it[0] : (int32_t)n_index_nodes;   // empty row: its own id
            if (it[2] > it[1]) {
                k = idx32[it[1]];
                for (int32_t p = it[1] + 1; p < it[2]; ++p) k = std::min(k, idx32[p]);
            }
            key[(size_t)i] = k;
            order[(size_t)i] = (int32_t)i;
        }
        std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return key[(size_t)a] < key[(size_t)b]; });
        std::vector<int32_t> sorted((size_t)n_items * 4);
        for (int64_t i = 0; i < n_items; ++i) std::memcpy(&sorted[(size_t)i * 4], items + 4 * (int64_t)order[(size_t)i], 4 * sizeof(int32_t));
        std::memcpy(items, sorted.data(), sorted.size() * sizeof(int32_t));
    }
    return BPTG_OK;
}

// ---- row groups --------------------------------------------------------------------------------
// Greedy clustering of work items (rows / row segments) that read mostly the same neighbour rows.
// Items are visited in locality order; an item opens a group and the next `window` unused items
// join it while at least half of their neighbours are already in the group's union (at most R
// members, and at most max_pairs edges in total unless max_pairs is 0: a group is walked by one
// wavefront from start to end, so the largest group bounds the kernel's duration from below).  The groups are then cut into 8 contiguous chunks of about equal work (one per XCD) and
// ordered inside each chunk (order_mode 0: locality order; 1: groups with at least average work first,
// the small ones last, each part in locality order; 2: by decreasing work).  For every group the union
// of neighbour ids becomes a list of entries (idx, member mask, first pair); a pair = one original
// edge = (entry, member).  Pairs are numbered entry by entry, members ascending.  With order_mode + 4
// the entries of a group are sorted by member mask (stable, larger first), which lets a kernel that
// handles two consecutive entries per step find the same members in both most of the time.
constexpr int32_t MAX_GROUP_ROWS = 32;          // member masks are 32-bit

int bptg_group_plan(const int32_t *items, int64_t n_items, const int32_t *idx32, const int32_t *eid32,
                    int64_t n_edges, int64_t n_index_nodes, int32_t R, int32_t window, int32_t order_mode,
                    int32_t max_pairs, int32_t *members, int32_t *grp_ptr, int32_t *entries, int32_t *pair_eid, int32_t *slot_eid,
                    int32_t *chunks, int64_t *n_groups_out, int64_t *n_entries_out) {
    if (!items || !members || !grp_ptr || !chunks || !n_groups_out || !n_entries_out) return BPTG_ERR_NULL;
    if (n_edges > 0 && (!idx32 || !eid32 || !entries || !pair_eid)) return BPTG_ERR_NULL;
    if (n_items < 0 || n_edges < 0 || n_index_nodes < 0) return BPTG_ERR_SIZE;
    if (R < 1 || R > MAX_GROUP_ROWS || window < 0 || order_mode < 0 || order_mode > 15 || max_pairs < 0) return BPTG_ERR_ARG;
    const bool aligned = (order_mode & 8) != 0;
    const bool by_mask = (order_mode & 4) != 0 && !aligned;
    order_mode &= 3;
    for (int64_t i = 0; i < n_items; ++i) {
        const int32_t *it = items + 4 * i;
        if (it[1] < 0 || it[2] < it[1] || it[2] > n_edges) return BPTG_ERR_RANGE;
    }
    for (int64_t p = 0; p < n_edges; ++p)
        if (idx32[p] < 0 || idx32[p] >= n_index_nodes) return BPTG_ERR_RANGE;

    // locality order of the items
    std::vector<int32_t> key((size_t)n_items), order((size_t)n_items);
    for (int64_t i = 0; i < n_items; ++i) {
        const int32_t *it = items + 4 * i;
        int32_t k = INT32_MAX;
        for (int32_t p = it[1]; p < it[2]; ++p) k = std::min(k, idx32[p]);
        key[(size_t)i] = k;
        order[(size_t)i] = (int32_t)i;
    }
    std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return key[(size_t)a] < key[(size_t)b]; });

    // ---- phase 1: form the groups (member item lists) in locality order
    std::vector<uint8_t> used((size_t)n_items, 0);
    std::vector<int64_t> stamp((size_t)n_index_nodes, -1);     // stamp[node] == group id  <=>  node in the union
    std::vector<int32_t> grp_items;                            // R slots per group, -1 = unused
    std::vector<int64_t> work;                                 // pairs + fixed cost per group
    int64_t n_groups = 0;
    for (int64_t oi = 0; oi < n_items; ++oi) {
        const int32_t first = order[(size_t)oi];
        if (used[(size_t)first]) continue;
        used[(size_t)first] = 1;
        int32_t mem[MAX_GROUP_ROWS];
        for (int32_t m = 0; m < MAX_GROUP_ROWS; ++m) mem[m] = -1;
        int32_t n_mem = 1;
        mem[0] = first;
        int64_t w = 0;
        {
            const int32_t *it = items + 4 * (int64_t)first;
            w += it[2] - it[1];
            for (int32_t p = it[1]; p < it[2]; ++p) stamp[(size_t)idx32[p]] = n_groups;
        }
        int32_t seen = 0;
        for (int64_t oj = oi + 1; oj < n_items && n_mem < R && seen < window; ++oj) {
            const int32_t cand = order[(size_t)oj];
            if (used[(size_t)cand]) continue;
            ++seen;
            const int32_t *it = items + 4 * (int64_t)cand;
            const int32_t len = it[2] - it[1];
            if (len == 0) continue;
            int32_t hit = 0;
            for (int32_t p = it[1]; p < it[2]; ++p) hit += (stamp[(size_t)idx32[p]] == n_groups);
            if (2 * hit >= len && (max_pairs == 0 || w + len <= max_pairs)) {
                used[(size_t)cand] = 1;
                mem[n_mem++] = cand;
                w += len;
                for (int32_t p = it[1]; p < it[2]; ++p) stamp[(size_t)idx32[p]] = n_groups;
            }
        }
        std::sort(mem, mem + n_mem);          // members in ascending item order (independent of the join order)
        for (int32_t m = 0; m < R; ++m) grp_items.push_back(mem[m]);
        work.push_back(w + 24);               // fixed cost of a wavefront, in pair equivalents
        ++n_groups;
    }

    // ---- phase 2: 8 contiguous chunks of about equal work, then the order inside each chunk
    std::vector<int32_t> gorder((size_t)n_groups);
    for (int64_t g = 0; g < n_groups; ++g) gorder[(size_t)g] = (int32_t)g;
    int64_t total = 0;
    for (int64_t g = 0; g < n_groups; ++g) total += work[(size_t)g];
    {
        int64_t acc = 0, g = 0;
        chunks[0] = 0;
        for (int x = 1; x <= 8; ++x) {
            const int64_t target = total * x / 8;
            while (g < n_groups && (acc + work[(size_t)g] / 2 < target || x == 8)) acc += work[(size_t)g++];
            chunks[x] = (int32_t)g;
        }
    }
    if (order_mode != 0) {
        for (int x = 0; x < 8; ++x) {
            auto b = gorder.begin() + chunks[x], e = gorder.begin() + chunks[x + 1];
            if (order_mode == 2) {
                std::stable_sort(b, e, [&](int32_t a, int32_t c) { return work[(size_t)a] > work[(size_t)c]; });
            } else if (order_mode == 3) {
                // runs of four groups that are consecutive in locality order stay together; the runs go by decreasing work
                const int64_t n = e - b, nq = (n + 3) / 4;
                std::vector<int64_t> qwork((size_t)nq, 0);
                std::vector<int32_t> qorder((size_t)nq), tmp(b, e);
                for (int64_t i = 0; i < n; ++i) qwork[(size_t)(i / 4)] += work[(size_t)tmp[(size_t)i]];
                for (int64_t i = 0; i < nq; ++i) qorder[(size_t)i] = (int32_t)i;
                std::stable_sort(qorder.begin(), qorder.end(), [&](int32_t a, int32_t c) { return qwork[(size_t)a] > qwork[(size_t)c]; });
                auto out = b;
                for (int64_t i = 0; i < nq; ++i)
                    for (int64_t j = 4 * (int64_t)qorder[(size_t)i]; j < std::min<int64_t>(n, 4 * (int64_t)qorder[(size_t)i] + 4); ++j) *out++ = tmp[(size_t)j];
            } else {
                int64_t sum = 0;
                for (auto it = b; it != e; ++it) sum += work[(size_t)*it];
                const int64_t avg = (e > b) ? sum / (e - b) : 0;
                std::stable_partition(b, e, [&](int32_t a) { return work[(size_t)a] >= avg; });
            }
        }
    }

    // ---- phase 3: emit members, entries and pairs in the final group order
    struct Triple { int32_t idx, member, eid; };
    struct Entry { int32_t idx; uint32_t mask; int32_t eids[MAX_GROUP_ROWS]; };
    std::vector<Triple> tri;
    std::vector<Entry> ents, placed;
    // the entries of one group in neighbour order
    auto collect_sorted = [&](const int32_t *gmem) {        // general path: handles parallel edges
        tri.clear();
        ents.clear();
        for (int32_t m = 0; m < R; ++m)
            if (gmem[m] >= 0) {
                const int32_t *it = items + 4 * (int64_t)gmem[m];
                for (int32_t p = it[1]; p < it[2]; ++p) tri.push_back({idx32[p], m, eid32[p]});
            }
        std::stable_sort(tri.begin(), tri.end(), [](const Triple &a, const Triple &b) {
            return a.idx != b.idx ? a.idx < b.idx : a.member < b.member;
        });
        // one run of equal idx -> as many entries as the largest multiplicity among the members
        size_t a = 0;
        while (a < tri.size()) {
            size_t b = a;
            int32_t cnt[MAX_GROUP_ROWS] = {0};
            size_t start[MAX_GROUP_ROWS] = {0};
            while (b < tri.size() && tri[b].idx == tri[a].idx) {
                if (cnt[tri[b].member] == 0) start[tri[b].member] = b;
                ++cnt[tri[b].member];
                ++b;
            }
            int32_t mult = 0;
            for (int32_t m = 0; m < R; ++m) mult = std::max(mult, cnt[m]);
            for (int32_t t = 0; t < mult; ++t) {
                Entry en;
                en.idx = tri[a].idx;
                en.mask = 0;
                for (int32_t m = 0; m < R; ++m)
                    if (cnt[m] > t) {
                        en.mask |= 1u << m;
                        en.eids[m] = tri[start[m] + (size_t)t].eid;
                    }
                ents.push_back(en);
            }
            a = b;
        }
    };
    // Fast path (no member reaches a neighbour twice): the distinct neighbours are found through a stamped map and
    // only they are sorted, not every edge of the group.
    std::vector<int64_t> seen_in((size_t)n_index_nodes, -1);
    std::vector<int32_t> local_of((size_t)n_index_nodes, 0);
    std::vector<Entry> found;
    std::vector<int32_t> by_idx;
    int64_t collect_id = 0;
    auto collect = [&](const int32_t *gmem) {
        found.clear();
        ++collect_id;
        bool repeated = false;
        for (int32_t m = 0; m < R && !repeated; ++m)
            if (gmem[m] >= 0) {
                const int32_t *it = items + 4 * (int64_t)gmem[m];
                for (int32_t p = it[1]; p < it[2]; ++p) {
                    const int32_t v = idx32[p];
                    if (seen_in[(size_t)v] != collect_id) {
                        seen_in[(size_t)v] = collect_id;
                        local_of[(size_t)v] = (int32_t)found.size();
                        Entry en;
                        en.idx = v;
                        en.mask = 0;
                        found.push_back(en);
                    }
                    Entry &en = found[(size_t)local_of[(size_t)v]];
                    if (en.mask >> m & 1) { repeated = true; break; }
                    en.mask |= 1u << m;
                    en.eids[m] = eid32[p];
                }
            }
        if (repeated) { collect_sorted(gmem); return; }
        by_idx.resize(found.size());
        for (size_t i = 0; i < found.size(); ++i) by_idx[i] = (int32_t)i;
        std::sort(by_idx.begin(), by_idx.end(), [&](int32_t a, int32_t b) { return found[(size_t)a].idx < found[(size_t)b].idx; });
        ents.resize(found.size());
        for (size_t i = 0; i < found.size(); ++i) ents[i] = found[(size_t)by_idx[i]];
    };
    // Aligned order: walking the groups in locality order, a neighbour keeps the position (the time step) it had
    // in the last group that read it whenever that position is free, and the other entries fill the gaps.  Wavefronts
    // that run side by side at the same pace then ask for a shared row at about the same time.
    std::vector<int32_t> pos_of;                 // per group (locality order): position of each entry
    std::vector<int64_t> pos_ptr;
    if (aligned) {
        std::vector<int32_t> lastpos((size_t)n_index_nodes, -1);
        std::vector<uint8_t> taken;
        pos_ptr.assign((size_t)n_groups + 1, 0);
        for (int64_t g = 0; g < n_groups; ++g) {
            collect(&grp_items[(size_t)g * R]);
            const int32_t n = (int32_t)ents.size();
            const size_t base = pos_of.size();
            pos_of.resize(base + (size_t)n, -1);
            taken.assign((size_t)n, 0);
            for (int32_t e = 0; e < n; ++e) {
                if (e > 0 && ents[(size_t)e].idx == ents[(size_t)e - 1].idx) continue;      // repeats only fill gaps
                const int32_t lp = lastpos[(size_t)ents[(size_t)e].idx];
                if (lp >= 0 && lp < n && !taken[(size_t)lp]) {
                    pos_of[base + (size_t)e] = lp;
                    taken[(size_t)lp] = 1;
                }
            }
            int32_t f = 0;
            for (int32_t e = 0; e < n; ++e) {
                if (pos_of[base + (size_t)e] < 0) {
                    while (taken[(size_t)f]) ++f;
                    pos_of[base + (size_t)e] = f;
                    taken[(size_t)f] = 1;
                }
                lastpos[(size_t)ents[(size_t)e].idx] = pos_of[base + (size_t)e];
            }
            pos_ptr[(size_t)g + 1] = (int64_t)pos_of.size();
        }
    }
    int64_t n_entries = 0, n_pairs = 0;
    grp_ptr[0] = 0;
    for (int64_t gi = 0; gi < n_groups; ++gi) {
        const int32_t *gmem = &grp_items[(size_t)gorder[(size_t)gi] * R];
        for (int32_t m = 0; m < R; ++m) {
            int32_t *mem = members + ((int64_t)gi * R + m) * 2;
            if (gmem[m] >= 0) {
                const int32_t *it = items + 4 * (int64_t)gmem[m];
                mem[0] = it[0];
                mem[1] = it[3];
            } else {
                mem[0] = -1;
                mem[1] = -1;
            }
        }
        collect(gmem);
        if (aligned) {
            const int64_t base = pos_ptr[(size_t)gorder[(size_t)gi]];
            placed.resize(ents.size());
            for (size_t e = 0; e < ents.size(); ++e) placed[(size_t)pos_of[(size_t)base + e]] = ents[e];
            ents.swap(placed);
        }
        // equal masks next to each other (larger masks first), neighbour order kept inside a mask
        if (by_mask) std::stable_sort(ents.begin(), ents.end(), [](const Entry &x, const Entry &y) { return x.mask > y.mask; });
        for (const Entry &e : ents) {
            int32_t *en = entries + 4 * n_entries;
            en[0] = e.idx;
            en[1] = (int32_t)e.mask;
            en[2] = (int32_t)n_pairs;
            en[3] = 0;
            for (int32_t m = 0; m < R; ++m) {
                const bool has = e.mask >> m & 1;
                if (has) pair_eid[n_pairs++] = e.eids[m];
                if (slot_eid) slot_eid[n_entries * R + m] = has ? e.eids[m] : -1;
            }
            ++n_entries;
        }
        grp_ptr[gi + 1] = (int32_t)n_entries;
    }
    *n_groups_out = n_groups;
    *n_entries_out = n_entries;
    return BPTG_OK;
}

int bptg_link_groups(const int32_t *slot_eid_dst, int64_t n_entries_dst, int32_t R_dst, const int32_t *slot_eid_src,
                     int64_t n_entries_src, int32_t R_src, int64_t n_edges, int32_t pad_entries, int32_t *pairs) {
    if (!pairs || (n_entries_dst > 0 && !slot_eid_dst) || (n_entries_src > 0 && !slot_eid_src)) return BPTG_ERR_NULL;
    if (n_entries_dst < 0 || n_entries_src < 0 || n_edges < 0 || pad_entries < 0) return BPTG_ERR_SIZE;
    if (R_dst < 1 || R_dst > MAX_GROUP_ROWS || R_src < 1 || R_src > MAX_GROUP_ROWS) return BPTG_ERR_ARG;
    if ((n_entries_src + pad_entries) * R_src >= INT32_MAX) return BPTG_ERR_SIZE;
    std::vector<int32_t> pos_of((size_t)n_edges, -1);
    int64_t covered = 0;
    for (int64_t i = 0; i < n_entries_src * R_src; ++i) {
        const int32_t e = slot_eid_src[i];
        if (e < 0) continue;
        if (e >= n_edges || pos_of[(size_t)e] >= 0) return BPTG_ERR_RANGE;          // not an edge, or an edge twice
        pos_of[(size_t)e] = (int32_t)i;
        ++covered;
    }
    if (covered != n_edges) return BPTG_ERR_RANGE;
    const int32_t spare = (int32_t)((n_entries_src + pad_entries) * R_src - 1);
    const int64_t n_real = n_entries_dst * R_dst, n_all = (n_entries_dst + pad_entries) * R_dst;
    for (int64_t i = 0; i < n_real; ++i) {
        const int32_t e = slot_eid_dst[i];
        if (e >= n_edges) return BPTG_ERR_RANGE;
        pairs[i] = e >= 0 ? pos_of[(size_t)e] : spare;
    }
    for (int64_t i = n_real; i < n_all; ++i) pairs[i] = spare;
    return BPTG_OK;
}

}  // extern "C"
