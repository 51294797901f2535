/*
 * TEST INFRASTRUCTURE — CPU oracle for the BPT graph-attention path.  Not part of the product:
 * only tests, the smoke check and the cpu_baseline leg of the benchmark may load this file's
 * library.  The shipped path is the HIP library and never calls into here.
 *
 * Plain-C restatement of the reference's algorithms, one function per reference routine:
 *
 *   graph construction   graph_builder/builder.pyx:41-116 (BinaryPartition.build_graph)
 *                        graph_builder/builder.pyx:243-274 (FullyConnected.build_graph)
 *                        graph_builder/builder.pyx:171-199 (OpenAISparse.build_graph)
 *                        graph_builder/builder.pyx:305-321 (partition_csr)
 *   operator semantics   graph_kernel/graphop_kernel.cu:19-230 (the 13 kernels), with the
 *                        launch shapes / zero fill / -1e9 initialiser of :235-600.
 *
 * Pinned by: tests/golden/builder_small.npz + builder_digests.json (written by the reference's
 * own Cython module, see tests/golden/make_builder_golden.py) for every graph routine; dense
 * closed forms (bmm, softmax over the dense block view, dense adjacency matmul — the method of
 * graph_kernel/test.py:185,218,245,274,314,364) and brute force on tiny graphs for every op.
 *
 * Every op exists as _f32 (accumulates in float, like scalar_t=float in the reference) and
 * _f64 (the truth used for tolerances).  A "unit" u is one entry of `row`: node row[u], edge
 * slots indptr[u] .. indptr[u+1]-1 (graphop_kernel.cu: `i = blockIdx.x`).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------
 * Graph construction
 * ---------------------------------------------------------------------------------------- */

typedef struct {
    uint32_t *a;
    size_t n, cap;
} vec_u32;

static int vpush(vec_u32 *v, uint32_t x) {
    if (v->n == v->cap) {
        size_t nc = v->cap ? v->cap * 2 : 1024;
        uint32_t *p = (uint32_t *)realloc(v->a, nc * sizeof(uint32_t));
        if (!p) return -1;
        v->a = p;
        v->cap = nc;
    }
    v->a[v->n++] = x;
    return 0;
}

typedef struct {
    vec_u32 src, dst, etype, pos, n_nodes_arr, shift;
    size_t n_nodes, n_lvl, n_edges;
} oracle_graph;

void oracle_graph_free(oracle_graph *g) {
    if (!g) return;
    free(g->src.a); free(g->dst.a); free(g->etype.a); free(g->pos.a);
    free(g->n_nodes_arr.a); free(g->shift.a);
    free(g);
}

size_t oracle_graph_n_nodes(const oracle_graph *g) { return g->n_nodes; }
size_t oracle_graph_n_edges(const oracle_graph *g) { return g->n_edges; }
size_t oracle_graph_n_levels(const oracle_graph *g) { return g->n_lvl; }
size_t oracle_graph_nodes_at_lvl(const oracle_graph *g, size_t i) { return g->n_nodes_arr.a[i]; }

/* builder.pyx:137-140 get_edges(v_shift) and :134 get_pos() — copies as int64 */
void oracle_graph_export(const oracle_graph *g, int64_t v_shift, int64_t *src, int64_t *dst,
                         int64_t *etype, int64_t *pos) {
    for (size_t e = 0; e < g->n_edges; ++e) {
        if (src) src[e] = (int64_t)g->src.a[e] + v_shift;
        if (dst) dst[e] = (int64_t)g->dst.a[e] + v_shift;
        if (etype) etype[e] = (int64_t)g->etype.a[e];
    }
    if (pos)
        for (size_t i = 0; i < g->pos.n; ++i) pos[i] = (int64_t)g->pos.a[i];
}

/* builder.pyx:41-116 */
oracle_graph *oracle_binary_partition(size_t length, int triu, size_t step, size_t clip_dist) {
    oracle_graph *g = (oracle_graph *)calloc(1, sizeof(oracle_graph));
    g->n_lvl = 1;
    /* :43-52 count nodes and the shift of each level */
    int n = (int)length, i;
    vpush(&g->shift, 0);
    while (n >= 2) {
        for (i = 0; i < n; ++i) vpush(&g->pos, (uint32_t)((i + 1) * (1 << (g->n_lvl - 1))));
        vpush(&g->n_nodes_arr, (uint32_t)n);
        g->n_nodes += (size_t)n;
        vpush(&g->shift, (uint32_t)g->n_nodes);
        g->n_lvl += 1;
        n = (n + 1) >> 1;
    }
    /* :54-57 root */
    vpush(&g->n_nodes_arr, 1);
    g->n_nodes += 1;
    vpush(&g->pos, (uint32_t)length);
    /* :59-62 pos = last covered token, clipped */
    for (size_t p = 0; p < g->pos.n; ++p) {
        g->pos.a[p] = g->pos.a[p] - 1;
        if (g->pos.a[p] >= length) g->pos.a[p] = (uint32_t)(length - 1);
    }
    /* :64-116 edges */
    int j, v, l_ptr, r_ptr;
    int l_overlap, r_overlap;
    for (i = 0; i < (int)length; ++i) {
        v = i;
        size_t shift = 0;
        l_ptr = v - 1; r_ptr = v + 1;
        l_overlap = 0; r_overlap = 0;
        for (j = 0; j < (int)g->n_lvl; ++j) {
            size_t clipped = (size_t)j < clip_dist ? (size_t)j : clip_dist;
            for (size_t k = 0; k < step; ++k) {
                /* :77-85 right connection; the bound is tested against level j even when the
                 * node pushed comes from level j-1 (reproduced as written) */
                if (!triu && (unsigned)r_ptr < g->n_nodes_arr.a[j]) {
                    if (r_overlap) vpush(&g->src, g->shift.a[j - 1] + (uint32_t)((r_ptr << 1) + 1));
                    else vpush(&g->src, g->shift.a[j] + (uint32_t)r_ptr);
                    vpush(&g->dst, (uint32_t)i);
                    vpush(&g->etype, (uint32_t)((2 * step + 1) * clipped + 2 * (k + 1)));
                    g->n_edges += 1;
                    r_overlap = 0;
                }
                r_ptr += 1;
                /* :90-98 left connection */
                if (l_ptr >= 0) {
                    if (l_overlap) vpush(&g->src, g->shift.a[j - 1] + (uint32_t)(l_ptr << 1));
                    else vpush(&g->src, g->shift.a[j] + (uint32_t)l_ptr);
                    vpush(&g->dst, (uint32_t)i);
                    vpush(&g->etype, (uint32_t)((2 * step + 1) * clipped + 2 * k + 1));
                    g->n_edges += 1;
                    l_overlap = 0;
                }
                l_ptr -= 1;
            }
            /* :102-107 */
            if ((l_ptr & 1) == 0) l_overlap = 1;
            if ((r_ptr & 1) == 1) r_overlap = 1;
            r_ptr >>= 1;
            l_ptr >>= 1;
            /* :109-113 self / bottom-up connection */
            vpush(&g->src, (uint32_t)i);
            vpush(&g->dst, (uint32_t)(shift + (size_t)v));
            vpush(&g->etype, (uint32_t)((2 * step + 1) * clipped));
            g->n_edges += 1;
            /* :115-116 */
            shift += g->n_nodes_arr.a[j];
            v >>= 1;
        }
    }
    return g;
}

/* builder.pyx:243-274 */
oracle_graph *oracle_fully_connected(size_t length, int triu, size_t window) {
    oracle_graph *g = (oracle_graph *)calloc(1, sizeof(oracle_graph));
    g->n_nodes = length + 1;
    g->n_lvl = 2;
    vpush(&g->n_nodes_arr, (uint32_t)length);
    vpush(&g->n_nodes_arr, 1);
    size_t lim = length < window + 1 ? length : window + 1;
    for (size_t i = 0; i < length; ++i) {
        vpush(&g->pos, (uint32_t)i);
        vpush(&g->src, (uint32_t)i); vpush(&g->dst, (uint32_t)i); vpush(&g->etype, 0);
        g->n_edges += 1;
        for (size_t j = 1; j < lim; ++j) {
            if (i >= j) {
                vpush(&g->src, (uint32_t)(i - j)); vpush(&g->dst, (uint32_t)i);
                vpush(&g->etype, (uint32_t)(2 * j - 1));
                g->n_edges += 1;
            }
            if (!triu && i + j < length) {
                vpush(&g->src, (uint32_t)(i + j)); vpush(&g->dst, (uint32_t)i);
                vpush(&g->etype, (uint32_t)(2 * j));
                g->n_edges += 1;
            }
        }
        vpush(&g->src, (uint32_t)i); vpush(&g->dst, (uint32_t)length); vpush(&g->etype, 0);
        g->n_edges += 1;
    }
    vpush(&g->pos, (uint32_t)length);
    return g;
}

/* builder.pyx:171-199 (strided baseline; causal only) */
oracle_graph *oracle_openai_sparse(size_t length, size_t stride, size_t c) {
    oracle_graph *g = (oracle_graph *)calloc(1, sizeof(oracle_graph));
    g->n_nodes = length + 1;
    g->n_lvl = 2;
    vpush(&g->n_nodes_arr, (uint32_t)length);
    vpush(&g->n_nodes_arr, 1);
    for (size_t i = 0; i < length; ++i) {
        vpush(&g->pos, (uint32_t)i);
        for (size_t j = (i / stride) * stride; j < i + 1; ++j) {
            vpush(&g->src, (uint32_t)j); vpush(&g->dst, (uint32_t)i); vpush(&g->etype, 0);
            g->n_edges += 1;
        }
        for (size_t j = 1; j < i / stride + 1; ++j)
            for (size_t k = stride * j - c; k < stride * j; ++k) {
                vpush(&g->src, (uint32_t)k); vpush(&g->dst, (uint32_t)i); vpush(&g->etype, 0);
                g->n_edges += 1;
            }
        vpush(&g->src, (uint32_t)i); vpush(&g->dst, (uint32_t)length); vpush(&g->etype, 0);
        g->n_edges += 1;
    }
    vpush(&g->pos, (uint32_t)(length - 1));
    return g;
}

/* builder.pyx:305-321.  Call with row==NULL to get the unit count. */
int64_t oracle_partition_csr(const int64_t *indptr, int64_t length, int64_t chunk_size,
                             int64_t *row, int64_t *indptr_) {
    int64_t n = 0;
    for (int64_t i = 0; i < length - 1; ++i)
        n += (indptr[i + 1] + chunk_size - 1 - indptr[i]) / chunk_size;
    if (!row) return n;
    int64_t cnt = 0;
    for (int64_t i = 0; i < length - 1; ++i)
        for (int64_t j = indptr[i]; j < indptr[i + 1]; j += chunk_size) {
            row[cnt] = i;
            indptr_[cnt] = j;
            cnt += 1;
        }
    indptr_[n] = indptr[length - 1];
    return n;
}

/* ------------------------------------------------------------------------------------------
 * Operator semantics (graphop_kernel.cu).  T = element type, generated twice below.
 * Layouts: node tensors (n, h, d) row-major; edge tensors (e, h); B of node_mul_edge (e, d).
 * Outputs must be zero-filled by the caller (the reference's at::zeros).
 * ---------------------------------------------------------------------------------------- */

#define DEFINE_OPS(T, SUF, EXP)                                                                   \
    /* kernel :40-55 (B is read through its (h,d,n) transpose there; same values) */             \
    void oracle_maskedmm_csr_forward_##SUF(const int64_t *row, const int64_t *indptr,             \
                                           const int64_t *eid, const int64_t *indices,            \
                                           const T *A, const T *B, T *y, int64_t n_row, int64_t d, \
                                           int64_t h) {                                           \
        for (int64_t i = 0; i < n_row; ++i)                                                       \
            for (int64_t j = indptr[i]; j < indptr[i + 1]; ++j)                                   \
                for (int64_t ko = 0; ko < h; ++ko) {                                              \
                    T sum = 0;                                                                    \
                    for (int64_t ki = 0; ki < d; ++ki)                                            \
                        sum += A[(row[i] * h + ko) * d + ki] * B[(indices[j] * h + ko) * d + ki]; \
                    y[eid[j] * h + ko] = sum;                                                     \
                }                                                                                 \
    }                                                                                             \
    /* kernel :100-112, one call per side (launcher :382-407 calls it for dA then dB) */        \
    void oracle_maskedmm_csr_backward_side_##SUF(const int64_t *row, const int64_t *indptr,       \
                                                 const int64_t *eid, const int64_t *indices,      \
                                                 const T *B, const T *dy, T *dA, int64_t n,       \
                                                 int64_t d, int64_t h) {                          \
        for (int64_t i = 0; i < n; ++i)                                                           \
            for (int64_t j = 0; j < d * h; ++j) {                                                 \
                T sum = 0;                                                                        \
                for (int64_t k = indptr[i]; k < indptr[i + 1]; ++k)                               \
                    sum += dy[eid[k] * h + j / d] * B[indices[k] * d * h + j];                    \
                dA[row[i] * d * h + j] += sum;                                                    \
            }                                                                                     \
    }                                                                                             \
    /* kernel :19-34 */                                                                           \
    void oracle_node_mul_edge_forward_##SUF(const int64_t *row, const int64_t *indptr,            \
                                            const int64_t *eid, const T *A, const T *B, T *y,     \
                                            int64_t n, int64_t d, int64_t h) {                    \
        for (int64_t i = 0; i < n; ++i)                                                           \
            for (int64_t j = indptr[i]; j < indptr[i + 1]; ++j)                                   \
                for (int64_t ko = 0; ko < h; ++ko) {                                              \
                    T sum = 0;                                                                    \
                    for (int64_t ki = 0; ki < d; ++ki)                                            \
                        sum += A[(row[i] * h + ko) * d + ki] * B[eid[j] * d + ki];                \
                    y[eid[j] * h + ko] = sum;                                                     \
                }                                                                                 \
    }                                                                                             \
    /* kernels :61-73 (dA) and :79-94 (dB) */                                                     \
    void oracle_node_mul_edge_backward_##SUF(const int64_t *row, const int64_t *indptr,           \
                                             const int64_t *eid, const T *A, const T *B,          \
                                             const T *dy, T *dA, T *dB, int64_t n, int64_t d,     \
                                             int64_t h) {                                         \
        for (int64_t i = 0; i < n; ++i)                                                           \
            for (int64_t j = 0; j < d * h; ++j) {                                                 \
                T sum = 0;                                                                        \
                for (int64_t k = indptr[i]; k < indptr[i + 1]; ++k)                               \
                    sum += dy[eid[k] * h + j / d] * B[eid[k] * d + j % d];                        \
                dA[row[i] * d * h + j] += sum;                                                    \
            }                                                                                     \
        for (int64_t i = 0; i < n; ++i)                                                           \
            for (int64_t j = 0; j < d; ++j)                                                       \
                for (int64_t k = indptr[i]; k < indptr[i + 1]; ++k) {                             \
                    T sum = 0;                                                                    \
                    for (int64_t ki = 0; ki < h; ++ki)                                            \
                        sum += dy[eid[k] * h + ki] * A[(row[i] * h + ki) * d + j];                \
                    dB[eid[k] * d + j] = sum;                                                     \
                }                                                                                 \
    }                                                                                             \
    /* kernel :118-130 */                                                                         \
    void oracle_vector_spmm_forward_##SUF(const int64_t *row, const int64_t *indptr,              \
                                          const int64_t *eid, const int64_t *indices,             \
                                          const T *edata, const T *x, T *y, int64_t n, int64_t d, \
                                          int64_t h) {                                            \
        for (int64_t i = 0; i < n; ++i)                                                           \
            for (int64_t j = 0; j < d * h; ++j) {                                                 \
                T sum = 0;                                                                        \
                for (int64_t k = indptr[i]; k < indptr[i + 1]; ++k)                               \
                    sum += edata[eid[k] * h + j / d] * x[indices[k] * d * h + j];                 \
                y[row[i] * d * h + j] += sum;                                                     \
            }                                                                                     \
    }                                                                                             \
    /* kernels :135-149 (dedata) and :151-163 (dx).  n_dx_units: how many units of the           \
     * transposed side are processed.  The reference launches the dx kernel with the row-side    \
     * grid (:566 reused at :588), i.e. min(n_row, n_col) units; pass n_col for the              \
     * mathematically complete gradient (what graph_kernel/test.py:299 asserts). */             \
    void oracle_vector_spmm_backward_##SUF(                                                       \
        const int64_t *row, const int64_t *indptr, const int64_t *eid, const int64_t *indices,    \
        const int64_t *col, const int64_t *indptr_t, const int64_t *eid_t,                        \
        const int64_t *indices_t, const T *edata, const T *dy, const T *x, T *dedata, T *dx,      \
        int64_t n_row, int64_t n_dx_units, int64_t d, int64_t h) {                                \
        for (int64_t i = 0; i < n_row; ++i)                                                       \
            for (int64_t j = indptr[i]; j < indptr[i + 1]; ++j)                                   \
                for (int64_t ko = 0; ko < h; ++ko) {                                              \
                    T sum = 0;                                                                    \
                    for (int64_t ki = 0; ki < d; ++ki)                                            \
                        sum += dy[(row[i] * h + ko) * d + ki] * x[(indices[j] * h + ko) * d + ki]; \
                    dedata[eid[j] * h + ko] = sum;                                                \
                }                                                                                 \
        for (int64_t i = 0; i < n_dx_units; ++i)                                                  \
            for (int64_t j = 0; j < d * h; ++j) {                                                 \
                T sum = 0;                                                                        \
                for (int64_t k = indptr_t[i]; k < indptr_t[i + 1]; ++k)                           \
                    sum += edata[eid_t[k] * h + j / d] * dy[indices_t[k] * d * h + j];            \
                dx[col[i] * d * h + j] += sum;                                                    \
            }                                                                                     \
    }                                                                                             \
    /* kernels :170-178, :180-192, :194-202; max_val starts at -1e9 (:428).  scratch: 2*n_nodes*h */ \
    void oracle_sparse_softmax_forward_##SUF(const int64_t *row, const int64_t *indptr,           \
                                             const int64_t *eid, const T *x, T *y, T *scratch,    \
                                             int64_t n_row, int64_t n_nodes, int64_t h) {         \
        T *max_val = scratch, *sum = scratch + n_nodes * h;                                       \
        for (int64_t q = 0; q < n_nodes * h; ++q) { max_val[q] = (T)-1e9; sum[q] = 0; }           \
        for (int64_t i = 0; i < n_row; ++i)                                                       \
            for (int64_t tx = 0; tx < h; ++tx)                                                    \
                for (int64_t k = indptr[i]; k < indptr[i + 1]; ++k) {                             \
                    T xv = x[eid[k] * h + tx];                                                    \
                    if (xv > max_val[row[i] * h + tx]) max_val[row[i] * h + tx] = xv;             \
                }                                                                                 \
        for (int64_t i = 0; i < n_row; ++i)                                                       \
            for (int64_t tx = 0; tx < h; ++tx) {                                                  \
                T max_v = max_val[row[i] * h + tx];                                               \
                for (int64_t k = indptr[i]; k < indptr[i + 1]; ++k) {                             \
                    T now = EXP(x[eid[k] * h + tx] - max_v);                                      \
                    y[eid[k] * h + tx] = now;                                                     \
                    sum[row[i] * h + tx] += now;                                                  \
                }                                                                                 \
            }                                                                                     \
        for (int64_t i = 0; i < n_row; ++i)                                                       \
            for (int64_t tx = 0; tx < h; ++tx)                                                    \
                for (int64_t k = indptr[i]; k < indptr[i + 1]; ++k)                               \
                    y[eid[k] * h + tx] /= sum[row[i] * h + tx];                                   \
    }                                                                                             \
    /* kernels :208-219, :221-230.  scratch: n_nodes*h */                                         \
    void oracle_sparse_softmax_backward_##SUF(const int64_t *row, const int64_t *indptr,          \
                                              const int64_t *eid, const T *y, const T *dy, T *dx, \
                                              T *scratch, int64_t n_row, int64_t n_nodes,         \
                                              int64_t h) {                                        \
        T *aggre = scratch;                                                                       \
        for (int64_t q = 0; q < n_nodes * h; ++q) aggre[q] = 0;                                   \
        for (int64_t i = 0; i < n_row; ++i)                                                       \
            for (int64_t tx = 0; tx < h; ++tx) {                                                  \
                T sum = 0;                                                                        \
                for (int64_t k = indptr[i]; k < indptr[i + 1]; ++k)                               \
                    sum += dy[eid[k] * h + tx] * y[eid[k] * h + tx];                              \
                aggre[row[i] * h + tx] += sum;                                                    \
            }                                                                                     \
        for (int64_t i = 0; i < n_row; ++i)                                                       \
            for (int64_t tx = 0; tx < h; ++tx)                                                    \
                for (int64_t k = indptr[i]; k < indptr[i + 1]; ++k)                               \
                    dx[eid[k] * h + tx] = dy[eid[k] * h + tx] * y[eid[k] * h + tx] -              \
                                          aggre[row[i] * h + tx] * y[eid[k] * h + tx];            \
    }

DEFINE_OPS(float, f32, expf)
DEFINE_OPS(double, f64, exp)
