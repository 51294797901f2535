// libbptplan — launch plans and row groups built on the GPU (gfx950), C ABI of include/bptplan.h.
//
// The host builder (bptgraph.cpp) needs the index arrays on the host and tens of milliseconds per new graph.  Here the
// same plan comes out of sorts and prefix sums over the device arrays: every step is a data-parallel kernel or a
// rocPRIM primitive on the caller's stream, sizes that depend on the data stay on the device (kernels are launched
// for the upper bounds and read the actual counts from the info blocks), and all integer results are independent of
// the execution order (the only atomics are integer max / or / add whose results do not depend on their order).
//
// The reference has no plans: its kernels take the chunked CSR arrays of graph/base.py:71-86 as they are.
#include <cstring>

#include <hip/hip_runtime.h>

#include <rocprim/rocprim.hpp>

#include <cstdint>

#include "../../include/bptattn.h"
#include "../../include/bptplan.h"

namespace {

constexpr int TPB = 256;
constexpr int FIXED_WORK = 24;        // cost of a group beyond its pairs, in pair equivalents (as the host builder)
constexpr uint32_t PAD32 = 0xFFFFFFFFu;
constexpr uint64_t PAD64 = ~uint64_t(0);

inline unsigned blocks_for(int64_t n) { return (unsigned)((n + TPB - 1) / TPB); }

inline unsigned bits_for(uint64_t max_value) {      // bits needed to hold values 0 .. max_value
    unsigned b = 1;
    while (b < 64 && (max_value >> b) != 0) ++b;
    return b;
}

// Carves 256-byte aligned arrays out of the caller's workspace; with a null base it only adds up the sizes.
struct Bump {
    char *base;
    size_t off;
    template <typename T> T *take(int64_t n) {
        off = (off + 255) & ~size_t(255);
        T *p = base ? reinterpret_cast<T *>(base + off) : nullptr;
        off += (size_t)(n > 0 ? n : 1) * sizeof(T);
        return p;
    }
};

// ---- rocPRIM wrappers (temporary storage = one shared region of the workspace) ------------------------------------
template <typename K>
hipError_t sort_pairs(void *tmp, size_t &bytes, const K *kin, K *kout, const int32_t *vin, int32_t *vout, int64_t n,
                      unsigned end_bit, hipStream_t s) {
    return rocprim::radix_sort_pairs(tmp, bytes, kin, kout, vin, vout, (size_t)n, 0u, end_bit, s, false);
}

hipError_t scan_i32(void *tmp, size_t &bytes, const int32_t *in, int32_t *out, int64_t n, hipStream_t s) {
    return rocprim::exclusive_scan(tmp, bytes, in, out, (int32_t)0, (size_t)n, rocprim::plus<int32_t>(), s, false);
}

// largest temporary storage any primitive of the three entry points asks for
hipError_t temp_bytes(int64_t max_items, int64_t max_groups, int64_t n_edges, int64_t n_rows, size_t *out) {
    size_t best = 0, b = 0;
    hipError_t e;
    if ((e = sort_pairs<uint32_t>(nullptr, b, nullptr, nullptr, nullptr, nullptr, max_items + 1, 32, nullptr)) != hipSuccess) return e;
    best = b > best ? b : best;
    if ((e = sort_pairs<uint32_t>(nullptr, b, nullptr, nullptr, nullptr, nullptr, max_groups + 1, 32, nullptr)) != hipSuccess) return e;
    best = b > best ? b : best;
    if ((e = sort_pairs<uint64_t>(nullptr, b, nullptr, nullptr, nullptr, nullptr, n_edges + 1, 64, nullptr)) != hipSuccess) return e;
    best = b > best ? b : best;
    int64_t ns = n_rows + 1;
    ns = ns > n_edges + 1 ? ns : n_edges + 1;
    ns = ns > max_groups + 1 ? ns : max_groups + 1;
    if ((e = scan_i32(nullptr, b, nullptr, nullptr, ns, nullptr)) != hipSuccess) return e;
    best = b > best ? b : best;
    *out = best + 256;
    return hipSuccess;
}

// ---- small helpers ---------------------------------------------------------------------------------------------------
__global__ void k_fill_i32(int32_t *p, int64_t n, int32_t v) {
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) p[i] = v;
}

__global__ void k_iota_i32(int32_t *p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n) p[i] = (int32_t)i;
}

// ---- base plan ---------------------------------------------------------------------------------------------------------
struct BaseWs {
    int32_t *c_items, *c_heavy, *c_slots, *b_items, *b_heavy, *b_slots, *seen, *items_tmp, *iota, *perm;
    uint32_t *key, *key_s;
    void *tmp;
};

BaseWs base_layout(Bump &b, int64_t n_rows, int64_t n_edges, int64_t max_items, size_t tmp_bytes) {
    BaseWs w;
    w.c_items = b.take<int32_t>(n_rows + 1);
    w.c_heavy = b.take<int32_t>(n_rows + 1);
    w.c_slots = b.take<int32_t>(n_rows + 1);
    w.b_items = b.take<int32_t>(n_rows + 1);
    w.b_heavy = b.take<int32_t>(n_rows + 1);
    w.b_slots = b.take<int32_t>(n_rows + 1);
    w.seen = b.take<int32_t>(n_edges);
    w.items_tmp = b.take<int32_t>(4 * max_items);
    w.iota = b.take<int32_t>(max_items);
    w.perm = b.take<int32_t>(max_items);
    w.key = b.take<uint32_t>(max_items);
    w.key_s = b.take<uint32_t>(max_items);
    w.tmp = b.take<char>((int64_t)tmp_bytes);
    return w;
}

__global__ void k_base_init(int32_t *info, const int64_t *ipu, int64_t n_units, int64_t n_edges) {
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    for (int i = 0; i < 16; ++i) info[i] = 0;
    int err = 0;
    bool covers = (n_edges == 0);
    if (n_units > 0) {
        const int64_t first = ipu[0], last = ipu[n_units];
        if (first < 0 || last >= INT32_MAX) err = 3;
        else if (last > n_edges) err = 1;
        covers = (first == 0 && last == n_edges);
    }
    info[BPT_PI_ERR] = err;
    info[BPT_PI_FLAGS] = covers ? 1 : 0;
}

__global__ void k_check_units(const int64_t *row, const int64_t *ipu, int64_t n_units, int64_t n_rows, int32_t *info) {
    const int64_t u = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (u >= n_units) return;
    int err = 0;
    if (row[u] < 0 || row[u] >= n_rows) err = 1;
    if (u > 0 && row[u] < row[u - 1]) err = err > 2 ? err : 2;
    if (ipu[u + 1] < ipu[u]) err = err > 2 ? err : 2;
    if (err) atomicMax(&info[BPT_PI_ERR], err);
}

// rowptr[r] = start of the first unit whose row is >= r (rows without a unit are empty)
__global__ void k_rowptr(const int64_t *row, const int64_t *ipu, int64_t n_units, int64_t n_rows, const int32_t *info,
                         int32_t *rowptr) {
    const int64_t r = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (r > n_rows || info[BPT_PI_ERR]) return;
    int64_t lo = 0, hi = n_units;
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (row[mid] < r) lo = mid + 1; else hi = mid;
    }
    rowptr[r] = n_units > 0 ? (int32_t)ipu[lo] : 0;
}

__global__ void k_row_counts(const int32_t *rowptr, int64_t n_rows, int32_t seg_len, int32_t *info, int32_t *c_items,
                             int32_t *c_heavy, int32_t *c_slots) {
    const int64_t r = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (r > n_rows || info[BPT_PI_ERR]) return;
    int32_t ni = 0, nh = 0, ns = 0;
    if (r < n_rows) {
        const int32_t deg = rowptr[r + 1] - rowptr[r];
        ni = 1;
        if (deg > seg_len) {
            nh = 1;
            ni = ns = (deg + seg_len - 1) / seg_len;
        }
        atomicMax(&info[BPT_PI_MAX_DEGREE], deg);
    }
    c_items[r] = ni;
    c_heavy[r] = nh;
    c_slots[r] = ns;
}

__global__ void k_emit_items(const int32_t *rowptr, int64_t n_rows, int32_t seg_len, const int32_t *b_items,
                             const int32_t *b_heavy, const int32_t *b_slots, int32_t *info, int32_t *items, int32_t *heavy) {
    const int64_t r = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (r > n_rows || info[BPT_PI_ERR]) return;
    if (r == n_rows) {
        info[BPT_PI_N_ITEMS] = b_items[n_rows];
        info[BPT_PI_N_HEAVY] = b_heavy[n_rows];
        info[BPT_PI_N_SLOTS] = b_slots[n_rows];
        return;
    }
    const int32_t begin = rowptr[r], end = rowptr[r + 1], deg = end - begin;
    int4 *out = reinterpret_cast<int4 *>(items) + b_items[r];
    if (deg <= seg_len) {
        *out = make_int4((int32_t)r, begin, end, -1);
        return;
    }
    const int32_t n_seg = (deg + seg_len - 1) / seg_len, s0 = b_slots[r];
    int32_t *hv = heavy + 3 * (int64_t)b_heavy[r];
    hv[0] = (int32_t)r;
    hv[1] = s0;
    hv[2] = n_seg;
    for (int32_t s = 0; s < n_seg; ++s) {
        const int32_t b = begin + s * seg_len;
        out[s] = make_int4((int32_t)r, b, min(end, b + seg_len), s0 + s);
    }
}

__global__ void k_narrow(const int64_t *eid, const int64_t *indices, int64_t n_edges, int64_t n_index_nodes, int32_t *info,
                         int32_t *idx32, int32_t *eid32, int32_t *seen) {
    const int64_t p = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (p >= n_edges) return;
    const int64_t e = eid[p], c = indices ? indices[p] : 0;
    if (e < 0 || e >= n_edges || c < 0 || (indices && c >= n_index_nodes)) {
        atomicMax(&info[BPT_PI_ERR], 1);
        eid32[p] = 0;
        idx32[p] = 0;
        return;
    }
    eid32[p] = (int32_t)e;
    idx32[p] = (int32_t)c;
    if (atomicAdd(&seen[e], 1) != 0) atomicAnd(&info[BPT_PI_FLAGS], ~1);
}

// Sort key of every item: smallest (LARGEST = false) or largest neighbour id; an empty item takes its own row id,
// clipped to n_index_nodes.  Positions past n_items get the padding key, which sorts behind every real one.
template <bool LARGEST>
__global__ void k_item_keys(const int32_t *items, const int32_t *idx32, const int32_t *info, int64_t max_items,
                            int64_t n_index_nodes, int64_t n_edges, uint32_t *key) {
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= max_items) return;
    if (info[BPT_PI_ERR] || i >= info[BPT_PI_N_ITEMS]) {
        key[i] = PAD32;
        return;
    }
    const int4 it = reinterpret_cast<const int4 *>(items)[i];
    int32_t k = (it.x >= 0 && it.x < n_index_nodes) ? it.x : (int32_t)n_index_nodes;
    if (it.z > it.y && it.y >= 0 && it.z <= n_edges) {          // (an item list from elsewhere is not trusted with addresses)
        k = idx32[it.y];
        for (int32_t p = it.y + 1; p < it.z; ++p) k = LARGEST ? max(k, idx32[p]) : min(k, idx32[p]);
    }
    key[i] = (uint32_t)k;
}

__global__ void k_gather_items(const int32_t *items_tmp, const int32_t *perm, const int32_t *info, int64_t max_items,
                               int32_t *items) {
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= max_items || info[BPT_PI_ERR] || i >= info[BPT_PI_N_ITEMS]) return;
    reinterpret_cast<int4 *>(items)[i] = reinterpret_cast<const int4 *>(items_tmp)[perm[i]];
}

// ---- row groups --------------------------------------------------------------------------------------------------------
struct GroupWs {
    uint32_t *key, *key_s;            // item keys, then group keys
    int32_t *iota, *jorder;           // items in the order of their largest neighbour
    int32_t *work0;                   // per group as formed
    int32_t *lorder, *lpos;           // locality numbering of the groups (by smallest neighbour) and its inverse
    int32_t *work, *prefix;           // per group in locality numbering, max_groups + 1
    int32_t *gorder, *inv;            // final group order (positions in locality numbering) and its inverse
    uint64_t *ekey, *ekey_s;          // one record per edge slot: (group, neighbour, member), unsorted and sorted
    uint64_t *mkey_s;                 // sorted (group, mask) keys of the entries (ekey is reused for the unsorted ones)
    int32_t *eval, *eval_s;           // the slot of a record; later the entry permutation
    int32_t *rank, *head, *run, *mult, *ebase, *ent_of;   // per record
    int32_t *ent_idx, *ent_g, *ent_mask, *newpos, *pop, *first;   // per entry
    void *tmp;
};

GroupWs group_layout(Bump &b, int64_t max_items, int64_t max_groups, int64_t n_edges, size_t tmp_bytes) {
    GroupWs w;
    const int64_t nk = max_items > max_groups ? max_items : max_groups;
    w.key = b.take<uint32_t>(nk);
    w.key_s = b.take<uint32_t>(nk);
    w.iota = b.take<int32_t>(nk > n_edges ? nk : n_edges);
    w.jorder = b.take<int32_t>(max_items);
    w.work0 = b.take<int32_t>(max_groups + 1);
    w.lorder = b.take<int32_t>(max_groups);
    w.lpos = b.take<int32_t>(max_groups);
    w.work = b.take<int32_t>(max_groups + 1);
    w.prefix = b.take<int32_t>(max_groups + 1);
    w.gorder = b.take<int32_t>(max_groups);
    w.inv = b.take<int32_t>(max_groups);
    w.ekey = b.take<uint64_t>(n_edges);
    w.ekey_s = b.take<uint64_t>(n_edges);
    w.mkey_s = b.take<uint64_t>(n_edges);
    w.eval = b.take<int32_t>(n_edges);
    w.eval_s = b.take<int32_t>(n_edges);
    w.rank = b.take<int32_t>(n_edges);
    w.head = b.take<int32_t>(n_edges + 1);
    w.run = b.take<int32_t>(n_edges + 1);
    w.mult = b.take<int32_t>(n_edges + 1);
    w.ebase = b.take<int32_t>(n_edges + 1);
    w.ent_of = b.take<int32_t>(n_edges);
    w.ent_idx = b.take<int32_t>(n_edges);
    w.ent_g = b.take<int32_t>(n_edges);
    w.ent_mask = b.take<int32_t>(n_edges);
    w.newpos = b.take<int32_t>(n_edges);
    w.pop = b.take<int32_t>(n_edges + 1);
    w.first = b.take<int32_t>(n_edges + 1);
    w.tmp = b.take<char>((int64_t)tmp_bytes);
    return w;
}

__device__ inline bool plan_usable(const int32_t *pinfo) { return pinfo[BPT_PI_ERR] == 0 && (pinfo[BPT_PI_FLAGS] & 1); }

__device__ inline int32_t n_groups_of(const int32_t *pinfo, int32_t R) {
    return plan_usable(pinfo) ? (pinfo[BPT_PI_N_ITEMS] + R - 1) / R : 0;
}

// work of every group as formed (its pairs plus a fixed cost) and its locality key: the smallest neighbour id any
// member reads
__global__ void k_group_work(const int32_t *items, const int32_t *jorder, const uint32_t *kmin, const int32_t *pinfo,
                             int64_t max_groups, int32_t R, int32_t *work0, uint32_t *lkey, int32_t *ginfo) {
    const int64_t g = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (g > max_groups) return;
    const int32_t ng = n_groups_of(pinfo, R), n_items = pinfo[BPT_PI_N_ITEMS];
    if (g == 0) {
        for (int i = 0; i < 16; ++i) ginfo[i] = 0;
        ginfo[BPT_GI_N_GROUPS] = ng;
    }
    int32_t w = 0;
    uint32_t key = PAD32;
    if (g < ng) {
        w = FIXED_WORK;
        for (int32_t m = 0; m < R; ++m) {
            const int64_t j = g * R + m;
            if (j < n_items) {
                const int32_t item = jorder[j];
                const int4 it = reinterpret_cast<const int4 *>(items)[item];
                w += it.z - it.y;
                key = min(key, kmin[item]);
            }
        }
    }
    work0[g] = w;
    if (g < max_groups) lkey[g] = key;
}

__global__ void k_gather_work(const int32_t *work0, const int32_t *lorder, const int32_t *ginfo, int64_t max_groups, int32_t *work) {
    const int64_t l = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (l > max_groups) return;
    work[l] = (l < ginfo[BPT_GI_N_GROUPS]) ? work0[lorder[l]] : 0;
}

// 8 contiguous ranges of about equal work: chunks[x] = number of groups whose midpoint lies before x/8 of the total
__global__ void k_chunks(const int32_t *work, const int32_t *prefix, const int32_t *pinfo, int32_t R, int32_t *chunks,
                         int32_t *ginfo) {
    __shared__ int32_t sh[9];
    const int x = threadIdx.x;
    const int32_t ng = n_groups_of(pinfo, R);
    if (x <= 8) {
        int32_t c = (x == 8) ? ng : 0;
        if (x >= 1 && x <= 7 && ng > 0) {
            const int64_t total = (int64_t)prefix[ng - 1] + work[ng - 1];
            const int64_t target = total * x / 8;
            int32_t lo = 0, hi = ng;                      // first group with prefix + work / 2 >= target
            while (lo < hi) {
                const int32_t mid = (lo + hi) >> 1;
                if ((int64_t)prefix[mid] + work[mid] / 2 < target) lo = mid + 1; else hi = mid;
            }
            c = lo;
        }
        sh[x] = c;
        chunks[x] = c;
    }
    __syncthreads();
    if (x == 0) {
        int32_t mx = 0;
        for (int i = 0; i < 8; ++i) mx = max(mx, sh[i + 1] - sh[i]);
        ginfo[BPT_GI_MAX_CHUNK] = mx;
    }
}

__global__ void k_group_keys(const int32_t *work, const int32_t *chunks, const int32_t *pinfo, int64_t max_groups, int32_t R,
                             int by_work, uint32_t *key) {
    const int64_t g = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (g >= max_groups) return;
    if (g >= n_groups_of(pinfo, R)) {
        key[g] = PAD32;
        return;
    }
    uint32_t c = 0;
    for (int x = 1; x <= 7; ++x) c += (chunks[x] <= g) ? 1u : 0u;
    key[g] = (c << 16) | (by_work ? 0xFFFFu - (uint32_t)work[g] : 0u);      // (the sort is stable: locality order otherwise)
}

__global__ void k_invert(const int32_t *order, const int32_t *count, int idx_of_count, int64_t max_n, int32_t *inv) {
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= max_n || i >= count[idx_of_count]) return;
    inv[order[i]] = (int32_t)i;
}

// members of the groups in their final order (members given), and one sort record per edge slot (ekey given).  inv == nullptr:
// the records carry the locality number of their group (the tile plans number their groups only once the entries are known).
__global__ void k_members_and_records(const int32_t *items, const int32_t *idx32, const int32_t *jorder, const int32_t *lpos,
                                      const int32_t *inv, const int32_t *pinfo, int64_t max_groups, int64_t n_edges, int32_t R,
                                      int32_t *members, uint64_t *ekey, int32_t *eval) {
    const int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (j >= max_groups * R) return;
    const int32_t ng = n_groups_of(pinfo, R), n_items = pinfo[BPT_PI_N_ITEMS];
    const int64_t g0 = j / R;
    const int32_t m = (int32_t)(j % R);
    if (g0 >= ng) return;
    const int32_t gi = inv ? inv[lpos[g0]] : lpos[g0];
    if (j >= n_items) {
        if (members) {
            members[((int64_t)gi * R + m) * 2] = -1;
            members[((int64_t)gi * R + m) * 2 + 1] = -1;
        }
        return;
    }
    const int4 it = reinterpret_cast<const int4 *>(items)[jorder[j]];
    if (members) {
        members[((int64_t)gi * R + m) * 2] = it.x;
        members[((int64_t)gi * R + m) * 2 + 1] = it.w;
    }
    if (!ekey) return;
    const int32_t p_end = it.z < n_edges ? it.z : (int32_t)n_edges;
    for (int32_t p = it.y > 0 ? it.y : 0; p < p_end; ++p) {
        ekey[p] = ((uint64_t)(uint32_t)gi << 35) | ((uint64_t)(uint32_t)idx32[p] << 4) | (uint64_t)m;
        eval[p] = p;
    }
}

// Tile plans: what a group costs the matrix kernels is its number of blocks of R entries (a block costs the same whether a
// third or all of its pairs exist), known once the entries are: work[l] = 4 * (blocks + 1) for the group with locality
// number l, from the entries' group numbers (ascending, ent_g[u] = l).
__global__ void k_block_work(const int32_t *ent_g, const int32_t *ginfo, int64_t max_groups, int32_t R, int32_t *work) {
    const int64_t l = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (l > max_groups) return;
    const int32_t ng = ginfo[BPT_GI_N_GROUPS], ne = ginfo[BPT_GI_N_ENTRIES];
    if (l >= ng) {
        work[l] = 0;
        return;
    }
    int32_t bound[2];
    for (int t = 0; t < 2; ++t) {                         // first entry whose group is >= l + t
        int32_t lo = 0, hi = ne;
        while (lo < hi) {
            const int32_t mid = (lo + hi) >> 1;
            if (ent_g[mid] < (int32_t)l + t) lo = mid + 1; else hi = mid;
        }
        bound[t] = lo;
    }
    work[l] = 4 * ((bound[1] - bound[0] + R - 1) / R + 1);
}

// the entries' groups from locality numbers to final numbers
__global__ void k_renumber(int32_t *ent_g, const int32_t *inv, int64_t n_edges, const int32_t *ginfo) {
    const int64_t u = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (u >= n_edges || u >= ginfo[BPT_GI_N_ENTRIES]) return;
    ent_g[u] = inv[ent_g[u]];
}

__global__ void k_pad_records(uint64_t *ekey, int32_t *eval, int64_t n_edges, const int32_t *pinfo) {
    const int64_t p = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (p >= n_edges) return;
    if (!plan_usable(pinfo)) {
        ekey[p] = PAD64;
        eval[p] = (int32_t)p;
    }
}

// rank of a record among the equal ones before it (an edge that a member holds several times), and the starts of the
// runs of equal (group, neighbour)
__global__ void k_rank(const uint64_t *skey, int64_t n_edges, const int32_t *pinfo, int32_t *rank, int32_t *head) {
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i > n_edges) return;
    if (i == n_edges || !plan_usable(pinfo)) {
        head[i] = 0;
        if (i < n_edges) rank[i] = 0;
        return;
    }
    const uint64_t k = skey[i];
    int32_t t = 0;
    for (int64_t b = i - 1; b >= 0 && skey[b] == k; --b) ++t;
    rank[i] = t;
    head[i] = (i == 0 || (skey[i - 1] >> 4) != (k >> 4)) ? 1 : 0;
}

__global__ void k_multiplicity(const int32_t *rank, const int32_t *head, const int32_t *run_excl, int64_t n_edges,
                               const int32_t *pinfo, int32_t *run, int32_t *mult) {
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n_edges || !plan_usable(pinfo)) return;
    const int32_t r = run_excl[i] + head[i] - 1;
    run[i] = r;
    atomicMax(&mult[r], rank[i] + 1);
}

__global__ void k_entry_fill(const uint64_t *skey, const int32_t *rank, const int32_t *run, const int32_t *ebase,
                             int64_t n_edges, const int32_t *pinfo, int32_t *ent_of, int32_t *ent_idx, int32_t *ent_g,
                             int32_t *ent_mask, int32_t *ginfo) {
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n_edges || !plan_usable(pinfo)) return;
    if (i == 0) ginfo[BPT_GI_N_ENTRIES] = ebase[n_edges];
    const uint64_t k = skey[i];
    const int32_t u = ebase[run[i]] + rank[i];
    ent_of[i] = u;
    ent_idx[u] = (int32_t)((k >> 4) & 0x7FFFFFFFu);
    ent_g[u] = (int32_t)(k >> 35);
    atomicOr(&ent_mask[u], 1 << (int)(k & 15));
}

// sort keys of the entries inside their groups.  mode 1: by member mask, larger first; mode 2: by (neighbour mod 16,
// neighbour), which spreads a group's walk over the id range the same way in every group, so that groups running
// side by side ask for a shared row at about the same step
__global__ void k_entry_keys(const int32_t *ent_g, const int32_t *ent_mask, const int32_t *ent_idx, int64_t n_edges,
                             const int32_t *ginfo, int mode, uint64_t *ekey) {
    const int64_t u = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (u >= n_edges) return;
    uint64_t k = PAD64;
    if (u < ginfo[BPT_GI_N_ENTRIES]) {
        const uint64_t g = (uint64_t)(uint32_t)ent_g[u], x = (uint64_t)(uint32_t)ent_idx[u];
        k = (mode == 1) ? ((g << 16) | (uint64_t)(0xFFFF ^ ent_mask[u])) : (mode == 2) ? ((g << 35) | ((x & 15) << 31) | x) : ((g << 31) | x);
    }
    ekey[u] = k;
}

__global__ void k_popcounts(const int32_t *ent_mask, const int32_t *perm, int64_t n_edges, const int32_t *ginfo, int32_t *pop) {
    const int64_t u = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (u > n_edges) return;
    pop[u] = (u < ginfo[BPT_GI_N_ENTRIES]) ? __popc((uint32_t)ent_mask[perm[u]]) : 0;
}

__global__ void k_entries_out(const int32_t *ent_idx, const int32_t *ent_mask, const int32_t *perm, const int32_t *first,
                              int64_t n_edges, const int32_t *ginfo, int32_t *entries) {
    const int64_t u = (int64_t)blockIdx.x * TPB + threadIdx.x;
    const int32_t ne = ginfo[BPT_GI_N_ENTRIES];
    if (u > n_edges || u > ne) return;
    int4 e = make_int4(0, 0, 0, 0);                   // the row behind the last entry is zero
    if (u < ne) e = make_int4(ent_idx[perm[u]], ent_mask[perm[u]], first[u], 0);
    reinterpret_cast<int4 *>(entries)[u] = e;
}

__global__ void k_group_ptr(const int32_t *ent_g, const int32_t *perm, int64_t max_groups, const int32_t *ginfo, int32_t *grp_ptr) {
    const int64_t g = (int64_t)blockIdx.x * TPB + threadIdx.x;
    const int32_t ng = ginfo[BPT_GI_N_GROUPS], ne = ginfo[BPT_GI_N_ENTRIES];
    if (g > max_groups || g > ng) return;
    int32_t lo = 0, hi = ne;                          // first entry whose group is >= g
    while (lo < hi) {
        const int32_t mid = (lo + hi) >> 1;
        if (ent_g[perm[mid]] < g) lo = mid + 1; else hi = mid;
    }
    grp_ptr[g] = lo;
}

__global__ void k_edge_ids(const uint64_t *skey, const int32_t *slot_of, const int32_t *ent_of, const int32_t *newpos,
                           const int32_t *ent_mask, const int32_t *first, const int32_t *eid32, int64_t n_edges,
                           const int32_t *pinfo, int32_t R, int32_t *grp_eids, int32_t *pair_eid) {
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n_edges || !plan_usable(pinfo)) return;
    const int32_t m = (int32_t)(skey[i] & 15), old = ent_of[i], u = newpos[old];
    if (m >= R) return;                                   // (only with an item list that does not cover the edge slots)
    const int32_t e = eid32[slot_of[i]];
    grp_eids[(int64_t)u * R + m] = e;
    pair_eid[first[u] + __popc((uint32_t)ent_mask[old] & ((1u << m) - 1u))] = e;
}

// ---- link -----------------------------------------------------------------------------------------------------------------
__global__ void k_positions(const int32_t *eids_src, const int32_t *ginfo_src, int32_t R_src, int64_t n_edges, int32_t *pos) {
    const int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (j >= (int64_t)ginfo_src[BPT_GI_N_ENTRIES] * R_src) return;
    const int32_t e = eids_src[j];
    if (e >= 0 && e < n_edges) pos[e] = (int32_t)j;
}

__global__ void k_pairs(const int32_t *eids_dst, const int32_t *ginfo_dst, int32_t R_dst, const int32_t *ginfo_src,
                        int32_t R_src, int64_t n_edges, int32_t pad, const int32_t *pos, int32_t *pairs) {
    const int64_t j = (int64_t)blockIdx.x * TPB + threadIdx.x;
    const int64_t n_real = (int64_t)ginfo_dst[BPT_GI_N_ENTRIES] * R_dst;
    if (j >= n_real + (int64_t)pad * R_dst) return;
    const int32_t spare = (ginfo_src[BPT_GI_N_ENTRIES] + pad) * R_src - 1;
    int32_t out = spare;
    if (j < n_real) {
        const int32_t e = eids_dst[j];
        if (e >= 0 && e < n_edges) out = pos[e];
    }
    pairs[j] = out;
}

// ---- edge lists of the reference's graph builder --------------------------------------------------------------------
// builder.pyx:41-116 (binary partition), :243-274 (fully connected), :171-199 (strided sparse) emit the edges token by
// token, so one thread walks one token: a first pass counts its edges, a prefix sum gives every token its place in
// the list, a second pass writes them there — the same list, in the same order, as the host walk (bptgraph.cpp).
constexpr int MAX_LEVELS = 48;
struct LevelTable {
    int64_t size[MAX_LEVELS], offset[MAX_LEVELS];
    int n;
};

struct EdgeCount {
    int64_t n = 0;
    __device__ void operator()(int64_t, int64_t, int64_t) { ++n; }
};
struct EdgeWrite {
    int64_t *src, *dst, *etype;
    int64_t shift, at;
    __device__ void operator()(int64_t s, int64_t d, int64_t t) {
        src[at] = s + shift;
        dst[at] = d + shift;
        etype[at] = t;
        ++at;
    }
};

// One token of builder.pyx:64-116: two cursors walk outwards, `step` nodes per side per level, then move one level
// up; a cursor that stops on a node whose sibling was taken continues with that child on the next level (the
// right-hand bound is checked against the current level even then, as the reference does).
template <class Sink>
__device__ void token_binary_partition(const LevelTable &lv, int64_t tok, bool causal, int64_t step, int64_t clip, Sink &out) {
    int64_t left = tok - 1, right = tok + 1, ancestor = tok;
    bool left_child = false, right_child = false;
    for (int j = 0; j < lv.n; ++j) {
        const int64_t type0 = (2 * step + 1) * (j < clip ? j : clip);
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
        left >>= 1;                           // arithmetic shift: stays negative once it is
        out(tok, lv.offset[j] + ancestor, type0);
        ancestor >>= 1;
    }
}

template <class Sink>
__device__ void token_edges(int kind, const LevelTable &lv, int64_t length, int64_t i, bool causal, int64_t a, int64_t b, Sink &out) {
    if (kind == 0) {
        token_binary_partition(lv, i, causal, a, b, out);
    } else if (kind == 1) {                   // builder.pyx:243-274: a = window
        const int64_t reach = length < a + 1 ? length : a + 1;
        out(i, i, 0);
        for (int64_t j = 1; j < reach; ++j) {
            if (i >= j) out(i - j, i, 2 * j - 1);
            if (!causal && i + j < length) out(i + j, i, 2 * j);
        }
        out(i, length, 0);
    } else {                                  // builder.pyx:171-199: a = stride, b = c
        for (int64_t j = (i / a) * a; j <= i; ++j) out(j, i, 0);
        for (int64_t blk = 1; blk <= i / a; ++blk)
            for (int64_t k = a * blk - b; k < a * blk; ++k) out(k, i, 0);
        out(i, length, 0);
    }
}

__global__ void k_graph_count(int kind, LevelTable lv, int64_t length, int causal, int64_t a, int64_t b, int32_t *counts) {
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i > length) return;
    EdgeCount c;
    if (i < length) token_edges(kind, lv, length, i, causal != 0, a, b, c);
    counts[i] = (int32_t)c.n;
}

__global__ void k_graph_fill(int kind, LevelTable lv, int64_t length, int causal, int64_t a, int64_t b, int64_t shift,
                             const int32_t *offsets, int64_t n_edges, int64_t *src, int64_t *dst, int64_t *etype) {
    const int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= length || offsets[length] != n_edges) return;     // the caller's edge count must be the list's
    EdgeWrite w{src, dst, etype, shift, offsets[i]};
    token_edges(kind, lv, length, i, causal != 0, a, b, w);
}

bool level_table(int kind, int64_t length, LevelTable &lv) {
    lv.n = 0;
    if (kind != 0) return true;
    int64_t n = length, nodes = 0;
    while (n >= 2) {
        if (lv.n >= MAX_LEVELS - 1) return false;
        lv.size[lv.n] = n;
        lv.offset[lv.n++] = nodes;
        nodes += n;
        n = (n + 1) >> 1;
    }
    lv.size[lv.n] = 1;
    lv.offset[lv.n++] = nodes;
    return true;
}

bool graph_args_ok(int kind, int64_t length, int64_t a, int64_t b) {
    if (length < 1 || length >= INT32_MAX) return false;
    if (kind == 0) return a >= 1 && b >= 0;
    if (kind == 1) return a >= 0;
    if (kind == 2) return a >= 1 && b >= 0 && b <= a;
    return false;
}

// ---- CSR of an edge list ------------------------------------------------------------------------------------------------
__global__ void k_csr_keys(const int64_t *rows, const int64_t *cols, int64_t n_edges, int64_t n_nodes, int32_t *info,
                           uint32_t *key, int32_t *val) {
    const int64_t e = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (e == 0) info[1] = 0;
    if (e >= n_edges) return;
    const int64_t r = rows[e], c = cols[e];
    const bool ok = r >= 0 && r < n_nodes && c >= 0 && c < n_nodes;
    if (!ok) atomicMax(&info[0], 1);
    key[e] = ok ? (uint32_t)r : PAD32;
    val[e] = (int32_t)e;
}

__global__ void k_csr_slots(const int64_t *cols, const int32_t *val_s, int64_t n_edges, const int32_t *info, int64_t *indices,
                            int64_t *eid) {
    const int64_t p = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (p >= n_edges || info[0]) return;
    const int32_t e = val_s[p];
    eid[p] = e;
    indices[p] = cols[e];
}

// indptr[r] = first slot whose row is >= r; number of chunked units of every row
__global__ void k_csr_indptr(const uint32_t *key_s, int64_t n_edges, int64_t n_nodes, int32_t chunk, const int32_t *info,
                             int64_t *indptr, int32_t *lo_of, int32_t *n_units_of) {
    const int64_t r = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (r > n_nodes || info[0]) return;
    int64_t lo = 0, hi = n_edges;
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (key_s[mid] < (uint32_t)r) lo = mid + 1; else hi = mid;
    }
    indptr[r] = lo;
    lo_of[r] = (int32_t)lo;
}

__global__ void k_csr_unit_counts(const int32_t *lo_of, int64_t n_nodes, int32_t chunk, const int32_t *info, int32_t *n_units_of) {
    const int64_t r = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (r > n_nodes || info[0]) return;
    n_units_of[r] = (r < n_nodes) ? (lo_of[r + 1] - lo_of[r] + chunk - 1) / chunk : 0;
}

// the units of builder.pyx:305-321: each row's slot range in chunks of at most `chunk` slots; empty rows give no unit
__global__ void k_csr_units(const int32_t *lo_of, const int32_t *unit_base, int64_t n_nodes, int64_t n_edges, int32_t chunk,
                            int32_t *info, int64_t *unit_row, int64_t *unit_ptr) {
    const int64_t r = (int64_t)blockIdx.x * TPB + threadIdx.x;
    if (r > n_nodes || info[0]) return;
    if (r == n_nodes) {
        info[1] = unit_base[n_nodes];
        unit_ptr[unit_base[n_nodes]] = n_edges;
        return;
    }
    const int32_t b = lo_of[r], e = lo_of[r + 1];
    int64_t u = unit_base[r];
    for (int32_t p = b; p < e; p += chunk, ++u) {
        unit_row[u] = r;
        unit_ptr[u] = p;
    }
}

struct CsrWs {
    uint32_t *key, *key_s;
    int32_t *val, *val_s, *lo_of, *n_units_of, *unit_base;
    void *tmp;
};

CsrWs csr_layout(Bump &b, int64_t n_edges, int64_t n_nodes, size_t tmp_bytes) {
    CsrWs w;
    w.key = b.take<uint32_t>(n_edges);
    w.key_s = b.take<uint32_t>(n_edges);
    w.val = b.take<int32_t>(n_edges);
    w.val_s = b.take<int32_t>(n_edges);
    w.lo_of = b.take<int32_t>(n_nodes + 1);
    w.n_units_of = b.take<int32_t>(n_nodes + 1);
    w.unit_base = b.take<int32_t>(n_nodes + 1);
    w.tmp = b.take<char>((int64_t)tmp_bytes);
    return w;
}

hipError_t csr_temp_bytes(int64_t n_edges, int64_t n_nodes, size_t *out) {
    size_t a = 0, b = 0;
    hipError_t e;
    if ((e = sort_pairs<uint32_t>(nullptr, a, nullptr, nullptr, nullptr, nullptr, n_edges + 1, 32, nullptr)) != hipSuccess) return e;
    if ((e = scan_i32(nullptr, b, nullptr, nullptr, n_nodes + 1, nullptr)) != hipSuccess) return e;
    *out = (a > b ? a : b) + 256;
    return hipSuccess;
}

int sizes_ok(int64_t n_units, int64_t n_edges, int64_t n_rows, int64_t n_index_nodes, int32_t seg_len) {
    if (n_units < 0 || n_edges < 0 || n_rows < 0 || n_index_nodes < 0) return BPT_ERR_SIZE;
    if (n_rows >= INT32_MAX || n_edges >= INT32_MAX || n_index_nodes >= INT32_MAX || n_units > n_edges + n_rows) return BPT_ERR_SIZE;
    if (seg_len < 1) return BPT_ERR_SHAPE;
    return BPT_OK;
}

#define HIP_TRY(expr)                                   \
    do {                                                \
        const hipError_t e_ = (expr);                   \
        if (e_ != hipSuccess) return (int)e_;           \
    } while (0)

#define LAUNCH(kernel, n, ...)                                                         \
    do {                                                                               \
        if ((n) > 0) {                                                                 \
            hipLaunchKernelGGL(kernel, dim3(blocks_for(n)), dim3(TPB), 0, s, __VA_ARGS__); \
            HIP_TRY(hipGetLastError());                                                \
        }                                                                              \
    } while (0)

}  // namespace

extern "C" {

int bpt_graph_count_device(int kind, int64_t length, int triu, int64_t a, int64_t b, int32_t *offsets, void *workspace,
                           int64_t workspace_bytes, void *stream) {
    if (!graph_args_ok(kind, length, a, b)) return BPT_ERR_SIZE;
    if (!offsets || !workspace) return BPT_ERR_NULL;
    LevelTable lv;
    if (!level_table(kind, length, lv)) return BPT_ERR_SIZE;
    size_t tmp = 0, tb = 0;
    HIP_TRY(scan_i32(nullptr, tmp, nullptr, nullptr, length + 1, nullptr));
    Bump bump{(char *)workspace, 0};
    int32_t *counts = bump.take<int32_t>(length + 1);
    void *scratch = bump.take<char>((int64_t)tmp + 256);
    if (workspace_bytes < (int64_t)bump.off) return BPT_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    LAUNCH(k_graph_count, length + 1, kind, lv, length, triu, a, b, counts);
    tb = tmp + 256;
    HIP_TRY(scan_i32(scratch, tb, counts, offsets, length + 1, s));
    return BPT_OK;
}

int bpt_graph_fill_device(int kind, int64_t length, int triu, int64_t a, int64_t b, int64_t v_shift, const int32_t *offsets,
                          int64_t n_edges, int64_t *src, int64_t *dst, int64_t *etype, void *stream) {
    if (!graph_args_ok(kind, length, a, b) || n_edges < 0) return BPT_ERR_SIZE;
    if (!offsets || (n_edges > 0 && (!src || !dst || !etype))) return BPT_ERR_NULL;
    LevelTable lv;
    if (!level_table(kind, length, lv)) return BPT_ERR_SIZE;
    hipStream_t s = (hipStream_t)stream;
    LAUNCH(k_graph_fill, length, kind, lv, length, triu, a, b, v_shift, offsets, n_edges, src, dst, etype);
    return BPT_OK;
}

int bpt_csr_device_bounds(int64_t n_edges, int64_t n_nodes, int32_t chunk_size, int64_t bounds[2]) {
    if (!bounds) return BPT_ERR_NULL;
    if (n_edges < 0 || n_nodes < 0 || n_edges >= INT32_MAX || n_nodes >= INT32_MAX) return BPT_ERR_SIZE;
    if (chunk_size < 1) return BPT_ERR_SHAPE;
    size_t tmp = 0;
    HIP_TRY(csr_temp_bytes(n_edges, n_nodes, &tmp));
    Bump dry{nullptr, 0};
    csr_layout(dry, n_edges, n_nodes, tmp);
    const int64_t by_rows = n_nodes + n_edges / chunk_size;
    bounds[0] = by_rows < n_edges ? by_rows : n_edges;
    bounds[1] = (int64_t)dry.off + 256;
    return BPT_OK;
}

int bpt_csr_build_device(const int64_t *rows, const int64_t *cols, int64_t n_edges, int64_t n_nodes, int32_t chunk_size,
                         int64_t *indptr, int64_t *indices, int64_t *eid, int64_t *unit_row, int64_t *unit_ptr, int32_t *info,
                         void *workspace, int64_t workspace_bytes, void *stream) {
    int64_t bounds[2];
    const int st = bpt_csr_device_bounds(n_edges, n_nodes, chunk_size, bounds);
    if (st != BPT_OK) return st;
    if (!indptr || !unit_ptr || !info || !workspace) return BPT_ERR_NULL;
    if (n_edges > 0 && (!rows || !cols || !indices || !eid || !unit_row)) return BPT_ERR_NULL;
    if (workspace_bytes < bounds[1]) return BPT_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    size_t tmp = 0;
    HIP_TRY(csr_temp_bytes(n_edges, n_nodes, &tmp));
    Bump bump{(char *)workspace, 0};
    CsrWs w = csr_layout(bump, n_edges, n_nodes, tmp);
    LAUNCH(k_fill_i32, 16, info, 16, 0);
    size_t tb;
    if (n_edges > 0) {
        LAUNCH(k_csr_keys, n_edges, rows, cols, n_edges, n_nodes, info, w.key, w.val);
        tb = tmp;
        HIP_TRY(sort_pairs<uint32_t>(w.tmp, tb, w.key, w.key_s, w.val, w.val_s, n_edges, 32, s));
        LAUNCH(k_csr_slots, n_edges, cols, w.val_s, n_edges, info, indices, eid);
    }
    LAUNCH(k_csr_indptr, n_nodes + 1, w.key_s, n_edges, n_nodes, chunk_size, info, indptr, w.lo_of, w.n_units_of);
    LAUNCH(k_csr_unit_counts, n_nodes + 1, w.lo_of, n_nodes, chunk_size, info, w.n_units_of);
    tb = tmp;
    HIP_TRY(scan_i32(w.tmp, tb, w.n_units_of, w.unit_base, n_nodes + 1, s));
    LAUNCH(k_csr_units, n_nodes + 1, w.lo_of, w.unit_base, n_nodes, n_edges, chunk_size, info, unit_row, unit_ptr);
    return BPT_OK;
}

int bpt_plan_device_bounds(int64_t n_units, int64_t n_edges, int64_t n_rows, int32_t seg_len, int32_t R, int64_t bounds[4]) {
    if (!bounds) return BPT_ERR_NULL;
    const int st = sizes_ok(n_units, n_edges, n_rows, 0, seg_len);
    if (st != BPT_OK) return st;
    if (R < 0 || R > 16) return BPT_ERR_SHAPE;
    const int64_t max_items = n_rows + n_edges / seg_len;
    const int64_t max_heavy = n_edges / ((int64_t)seg_len + 1);
    const int64_t max_groups = R > 0 ? (max_items + R - 1) / R : 0;
    if (max_items >= INT32_MAX || (R > 0 && (n_edges + 8) * R >= INT32_MAX)) return BPT_ERR_SIZE;
    size_t tmp = 0;
    HIP_TRY(temp_bytes(max_items, max_groups, n_edges, n_rows, &tmp));
    Bump a{nullptr, 0}, b{nullptr, 0}, c{nullptr, 0};
    base_layout(a, n_rows, n_edges, max_items, tmp);
    group_layout(b, max_items, max_groups, n_edges, tmp);
    c.take<int32_t>(n_edges);
    size_t ws = a.off > b.off ? a.off : b.off;
    ws = ws > c.off ? ws : c.off;
    bounds[0] = max_items;
    bounds[1] = max_heavy;
    bounds[2] = max_groups;
    bounds[3] = (int64_t)ws + 256;
    return BPT_OK;
}

int bpt_plan_build_device(const int64_t *row, const int64_t *indptr_units, int64_t n_units, const int64_t *eid,
                          const int64_t *indices, int64_t n_edges, int64_t n_rows, int64_t n_index_nodes, int32_t seg_len,
                          int32_t *rowptr, int32_t *idx32, int32_t *eid32, int32_t *items, int32_t *heavy, int32_t *info,
                          void *workspace, int64_t workspace_bytes, void *stream) {
    int64_t bounds[4];
    const int st = sizes_ok(n_units, n_edges, n_rows, n_index_nodes, seg_len);
    if (st != BPT_OK) return st;
    if (!rowptr || !items || !info || !workspace) return BPT_ERR_NULL;
    if (n_units > 0 && (!row || !indptr_units)) return BPT_ERR_NULL;
    if (n_edges > 0 && (!eid || !idx32 || !eid32)) return BPT_ERR_NULL;
    const int bs = bpt_plan_device_bounds(n_units, n_edges, n_rows, seg_len, 0, bounds);
    if (bs != BPT_OK) return bs;
    if (bounds[1] > 0 && !heavy) return BPT_ERR_NULL;
    if (workspace_bytes < bounds[3]) return BPT_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    const int64_t max_items = bounds[0];
    size_t tmp = 0;
    HIP_TRY(temp_bytes(max_items, 0, n_edges, n_rows, &tmp));
    Bump bump{(char *)workspace, 0};
    BaseWs w = base_layout(bump, n_rows, n_edges, max_items, tmp);

    hipLaunchKernelGGL(k_base_init, dim3(1), dim3(1), 0, s, info, indptr_units, n_units, n_edges);
    HIP_TRY(hipGetLastError());
    LAUNCH(k_check_units, n_units, row, indptr_units, n_units, n_rows, info);
    LAUNCH(k_fill_i32, n_edges, w.seen, n_edges, 0);
    LAUNCH(k_narrow, n_edges, eid, indices, n_edges, n_index_nodes, info, idx32, eid32, w.seen);
    LAUNCH(k_rowptr, n_rows + 1, row, indptr_units, n_units, n_rows, info, rowptr);
    LAUNCH(k_row_counts, n_rows + 1, rowptr, n_rows, seg_len, info, w.c_items, w.c_heavy, w.c_slots);
    size_t tb = tmp;
    HIP_TRY(scan_i32(w.tmp, tb, w.c_items, w.b_items, n_rows + 1, s));
    tb = tmp;
    HIP_TRY(scan_i32(w.tmp, tb, w.c_heavy, w.b_heavy, n_rows + 1, s));
    tb = tmp;
    HIP_TRY(scan_i32(w.tmp, tb, w.c_slots, w.b_slots, n_rows + 1, s));
    LAUNCH(k_emit_items, n_rows + 1, rowptr, n_rows, seg_len, w.b_items, w.b_heavy, w.b_slots, info, w.items_tmp, heavy);
    if (max_items > 0) {
        // locality order: by smallest neighbour id (without indices the items stay in row order, as on the host)
        LAUNCH(k_iota_i32, max_items, w.iota, max_items);
        const int32_t *perm = w.iota;
        if (indices) {
            LAUNCH(k_item_keys<false>, max_items, w.items_tmp, idx32, info, max_items, n_index_nodes, n_edges, w.key);
            tb = tmp;
            HIP_TRY(sort_pairs<uint32_t>(w.tmp, tb, w.key, w.key_s, w.iota, w.perm, max_items, 32, s));
            perm = w.perm;
        }
        LAUNCH(k_gather_items, max_items, w.items_tmp, perm, info, max_items, items);
    }
    return BPT_OK;
}

int bpt_plan_group_device(const int32_t *items, const int32_t *idx32, const int32_t *eid32, const int32_t *plan_info,
                          int64_t max_items, int64_t n_edges, int64_t n_index_nodes, int32_t seg_len, int32_t R,
                          int32_t by_mask, int32_t *members, int32_t *grp_ptr, int32_t *entries, int32_t *pair_eid,
                          int32_t *grp_eids, int32_t *chunks, int32_t *group_info, void *workspace,
                          int64_t workspace_bytes, void *stream) {
    if (max_items < 0 || n_edges < 0 || n_index_nodes < 0 || max_items >= INT32_MAX || n_edges >= INT32_MAX ||
        n_index_nodes >= INT32_MAX)
        return BPT_ERR_SIZE;
    if (R < 1 || R > 16 || seg_len < 1 || by_mask < 0 || (by_mask & 3) > 2 || by_mask > 6) return BPT_ERR_SHAPE;
    const int by_work = (by_mask & 4) ? 0 : 1;                   // + 4: the groups of a range keep their locality order
    by_mask &= 3;
    if ((int64_t)R * seg_len + FIXED_WORK > 0xFFFF) return BPT_ERR_UNSUPPORTED;       // the work of a group is a 16-bit sort key
    if ((n_edges + 8) * R >= INT32_MAX) return BPT_ERR_SIZE;
    if (!plan_info || !grp_ptr || !entries || !grp_eids || !chunks || !group_info || !workspace) return BPT_ERR_NULL;
    if (max_items > 0 && (!items || !members)) return BPT_ERR_NULL;
    if (n_edges > 0 && (!idx32 || !eid32 || !pair_eid)) return BPT_ERR_NULL;
    const int64_t max_groups = (max_items + R - 1) / R;
    if (max_groups >= (int64_t)1 << 28) return BPT_ERR_UNSUPPORTED;                    // group numbers are 28-bit sort keys
    size_t tmp = 0;
    HIP_TRY(temp_bytes(max_items, max_groups, n_edges, 0, &tmp));
    Bump dry{nullptr, 0};
    group_layout(dry, max_items, max_groups, n_edges, tmp);
    if (workspace_bytes < (int64_t)dry.off) return BPT_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    Bump bump{(char *)workspace, 0};
    GroupWs w = group_layout(bump, max_items, max_groups, n_edges, tmp);
    size_t tb;

    // the items in the order of their largest neighbour; R consecutive ones are a group
    if (max_items > 0) {
        LAUNCH(k_item_keys<true>, max_items, items, idx32, plan_info, max_items, n_index_nodes, n_edges, w.key);
        LAUNCH(k_iota_i32, max_items, w.iota, max_items);
        tb = tmp;
        HIP_TRY(sort_pairs<uint32_t>(w.tmp, tb, w.key, w.key_s, w.iota, w.jorder, max_items, 32, s));
    }
    // the groups numbered by locality (smallest neighbour id), cut into 8 ranges of equal work, by decreasing work
    // inside a range
    if (max_items > 0) LAUNCH(k_item_keys<false>, max_items, items, idx32, plan_info, max_items, n_index_nodes, n_edges, w.key);
    LAUNCH(k_group_work, max_groups + 1, items, w.jorder, w.key, plan_info, max_groups, R, w.work0, w.key_s, group_info);
    if (max_groups > 0) {
        LAUNCH(k_iota_i32, max_groups, w.iota, max_groups);
        tb = tmp;
        HIP_TRY(sort_pairs<uint32_t>(w.tmp, tb, w.key_s, w.key, w.iota, w.lorder, max_groups, 32, s));
        LAUNCH(k_invert, max_groups, w.lorder, group_info, (int)BPT_GI_N_GROUPS, max_groups, w.lpos);
    }
    // Tiles (R = 16) are cut into ranges and ordered by their blocks of entries, which are known only after the record sort
    // below: their records carry the locality numbers first.  The other groups are balanced by their pairs, as formed.
    const bool by_blocks = (R == 16);
    auto number_groups = [&]() -> int {                   // w.work (locality numbering) -> chunks, w.gorder, w.inv
        size_t tb2 = tmp;
        HIP_TRY(scan_i32(w.tmp, tb2, w.work, w.prefix, max_groups + 1, s));
        hipLaunchKernelGGL(k_chunks, dim3(1), dim3(64), 0, s, w.work, w.prefix, plan_info, R, chunks, group_info);
        HIP_TRY(hipGetLastError());
        if (max_groups > 0) {
            LAUNCH(k_group_keys, max_groups, w.work, chunks, plan_info, max_groups, R, by_work, w.key_s);
            LAUNCH(k_iota_i32, max_groups, w.iota, max_groups);
            tb2 = tmp;
            HIP_TRY(sort_pairs<uint32_t>(w.tmp, tb2, w.key_s, w.key, w.iota, w.gorder, max_groups, 32, s));
            LAUNCH(k_invert, max_groups, w.gorder, group_info, (int)BPT_GI_N_GROUPS, max_groups, w.inv);
        }
        return BPT_OK;
    };
    if (!by_blocks) {
        LAUNCH(k_gather_work, max_groups + 1, w.work0, w.lorder, group_info, max_groups, w.work);
        const int st = number_groups();
        if (st != BPT_OK) return st;
    }
    if (max_groups > 0)
        LAUNCH(k_members_and_records, max_groups * R, items, idx32, w.jorder, w.lpos, by_blocks ? (const int32_t *)nullptr : w.inv, plan_info,
               max_groups, n_edges, R, by_blocks ? (int32_t *)nullptr : members, w.ekey, w.eval);
    // entries: distinct (group, neighbour, multiplicity) of the records sorted by (group, neighbour, member)
    LAUNCH(k_fill_i32, (n_edges + 8) * R, grp_eids, (n_edges + 8) * R, (int32_t)n_edges);
    if (n_edges > 0) {
        LAUNCH(k_pad_records, n_edges, w.ekey, w.eval, n_edges, plan_info);
        tb = tmp;
        HIP_TRY(sort_pairs<uint64_t>(w.tmp, tb, w.ekey, w.ekey_s, w.eval, w.eval_s, n_edges, 35 + bits_for((uint64_t)max_groups), s));
    }
    LAUNCH(k_rank, n_edges + 1, w.ekey_s, n_edges, plan_info, w.rank, w.head);
    tb = tmp;
    HIP_TRY(scan_i32(w.tmp, tb, w.head, w.run, n_edges + 1, s));       // w.run = exclusive scan for now
    LAUNCH(k_fill_i32, n_edges + 1, w.mult, n_edges + 1, 0);
    LAUNCH(k_fill_i32, n_edges, w.ent_mask, n_edges, 0);
    LAUNCH(k_multiplicity, n_edges, w.rank, w.head, w.run, n_edges, plan_info, w.run, w.mult);
    tb = tmp;
    HIP_TRY(scan_i32(w.tmp, tb, w.mult, w.ebase, n_edges + 1, s));
    LAUNCH(k_entry_fill, n_edges, w.ekey_s, w.rank, w.run, w.ebase, n_edges, plan_info, w.ent_of, w.ent_idx, w.ent_g,
           w.ent_mask, group_info);
    if (by_blocks) {
        // the tiles' cost is known now: their ranges, their final numbers, their members; the entries take the final numbers
        LAUNCH(k_block_work, max_groups + 1, w.ent_g, group_info, max_groups, R, w.work);
        const int st = number_groups();
        if (st != BPT_OK) return st;
        if (max_groups > 0)
            LAUNCH(k_members_and_records, max_groups * R, items, idx32, w.jorder, w.lpos, w.inv, plan_info, max_groups, n_edges, R, members,
                   (uint64_t *)nullptr, (int32_t *)nullptr);
        if (n_edges > 0) LAUNCH(k_renumber, n_edges, w.ent_g, w.inv, n_edges, group_info);
    }
    // entry order inside a group: neighbour order, or by member mask (larger first, neighbour order inside a mask); the
    // entries of renumbered groups are sorted in every case
    int32_t *perm = w.iota;                               // new position -> entry as numbered above
    LAUNCH(k_iota_i32, n_edges, w.iota, n_edges);
    if ((by_mask != 0 || by_blocks) && n_edges > 0) {
        LAUNCH(k_entry_keys, n_edges, w.ent_g, w.ent_mask, w.ent_idx, n_edges, group_info, (int)by_mask, w.ekey);
        tb = tmp;
        HIP_TRY(sort_pairs<uint64_t>(w.tmp, tb, w.ekey, w.mkey_s, w.iota, w.eval, n_edges,
                                     (by_mask == 1 ? 16 : by_mask == 2 ? 35 : 31) + bits_for((uint64_t)max_groups), s));
        perm = w.eval;
    }
    LAUNCH(k_invert, n_edges, perm, group_info, (int)BPT_GI_N_ENTRIES, n_edges, w.newpos);
    LAUNCH(k_popcounts, n_edges + 1, w.ent_mask, perm, n_edges, group_info, w.pop);
    tb = tmp;
    HIP_TRY(scan_i32(w.tmp, tb, w.pop, w.first, n_edges + 1, s));
    LAUNCH(k_entries_out, n_edges + 1, w.ent_idx, w.ent_mask, perm, w.first, n_edges, group_info, entries);
    LAUNCH(k_group_ptr, max_groups + 1, w.ent_g, perm, max_groups, group_info, grp_ptr);
    LAUNCH(k_edge_ids, n_edges, w.ekey_s, w.eval_s, w.ent_of, w.newpos, w.ent_mask, w.first, eid32, n_edges, plan_info, R, grp_eids,
           pair_eid);
    return BPT_OK;
}

int bpt_plan_link_device(const int32_t *grp_eids_dst, const int32_t *group_info_dst, int32_t R_dst,
                         const int32_t *grp_eids_src, const int32_t *group_info_src, int32_t R_src, int64_t n_edges,
                         int32_t pad_entries, int32_t *pairs, void *workspace, int64_t workspace_bytes, void *stream) {
    if (n_edges < 0 || n_edges >= INT32_MAX || pad_entries < 0) return BPT_ERR_SIZE;
    if (R_dst < 1 || R_dst > 16 || R_src < 1 || R_src > 16) return BPT_ERR_SHAPE;
    if (((int64_t)n_edges + pad_entries) * (R_dst > R_src ? R_dst : R_src) >= INT32_MAX) return BPT_ERR_SIZE;
    if (!grp_eids_dst || !group_info_dst || !grp_eids_src || !group_info_src || !pairs || !workspace) return BPT_ERR_NULL;
    if (workspace_bytes < (int64_t)((n_edges > 0 ? n_edges : 1) * sizeof(int32_t) + 256)) return BPT_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    Bump bump{(char *)workspace, 0};
    int32_t *pos = bump.take<int32_t>(n_edges);
    LAUNCH(k_fill_i32, n_edges, pos, n_edges, 0);
    LAUNCH(k_positions, n_edges * R_src, grp_eids_src, group_info_src, R_src, n_edges, pos);
    LAUNCH(k_pairs, (n_edges + pad_entries) * R_dst, grp_eids_dst, group_info_dst, R_dst, group_info_src, R_src, n_edges,
           pad_entries, pos, pairs);
    return BPT_OK;
}

}  // extern "C"
