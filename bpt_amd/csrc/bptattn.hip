// libbptattn: gfx950 HIP kernels of the BPT graph-attention path (C ABI in include/bptattn.h).
//
// Execution model.  One 64-lane wavefront owns one work item of the plan: a whole row of the
// CSR side it walks, or one segment of a row that is longer than the plan's segment length.
// Whole rows write their result directly; segments write a partial result into the workspace
// and a second kernel combines the partials of each split row in slot order.  No atomics
// anywhere, so every output is bit-reproducible run to run.
//
// Two kernel families:
//   * "generic": any h, d and f32 / f64 / bf16, lanes stride over the columns of a node row;
//   * "fast":    compile-time (h, d) for f32 / bf16.  A node row of C = h*d elements is spread
//                over the wavefront so that lane l holds C/64 elements of head l / (64/h) and
//                every 16-byte load instruction of the wavefront covers whole 128-byte lines.
//                A per-head dot product is then C/64 FMAs plus log2(64/h) DPP additions.
// Work items are dealt to workgroups so that each XCD (blocks are distributed round-robin over
// the 8 XCDs) walks a contiguous range of rows: neighbouring tokens share most of their
// neighbours, which keeps the gathered K/V rows in that XCD's L2.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdint>
#include <mutex>
#include <utility>
#include <vector>

#include "../../include/bptattn.h"
#include "../../include/bptattn_measure.h"

namespace {

constexpr int WAVE = 64;
constexpr int WAVES_PER_BLOCK = 4;
constexpr int BLOCK = WAVE * WAVES_PER_BLOCK;
constexpr float M_INIT_LOG2 = -1.4426950408889634e9f;   // -1e9 (graphop_kernel.cu:428) in base-2 units
constexpr float LOG2E = 1.4426950408889634f;

std::atomic<int> g_force_generic{0};

// optional measurement hook (bpt_profile_kernel): which main kernel to bracket with events
std::atomic<int> g_prof_which{0};
std::atomic<void *> g_prof_start{nullptr}, g_prof_stop{nullptr};

struct ProfScope {
    hipStream_t s;
    bool on;
    ProfScope(int which, hipStream_t stream) : s(stream), on(g_prof_which.load(std::memory_order_relaxed) == which) {
        if (on) (void)hipEventRecord((hipEvent_t)g_prof_start.load(), s);
    }
    ~ProfScope() {
        if (on) (void)hipEventRecord((hipEvent_t)g_prof_stop.load(), s);
    }
};

// ------------------------------------------------------------------------------------------
// element types
// ------------------------------------------------------------------------------------------
struct bf16_t { uint16_t bits; };
typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);   // NaN stays NaN
    u += 0x7fffu + ((u >> 16) & 1u);                                              // round to nearest even
    return (uint16_t)(u >> 16);
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    using acc_t = float;
    static __device__ __forceinline__ float ld(const float *p) { return *p; }
    static __device__ __forceinline__ void st(float *p, float v) { *p = v; }
};
template <> struct Elem<double> {
    using acc_t = double;
    static __device__ __forceinline__ double ld(const double *p) { return *p; }
    static __device__ __forceinline__ void st(double *p, double v) { *p = v; }
};
template <> struct Elem<bf16_t> {
    using acc_t = float;
    static __device__ __forceinline__ float ld(const bf16_t *p) { return bf16_to_f32(p->bits); }
    static __device__ __forceinline__ void st(bf16_t *p, float v) { p->bits = f32_to_bf16(v); }
};

__device__ __forceinline__ float exp_acc(float x) { return expf(x); }
__device__ __forceinline__ double exp_acc(double x) { return exp(x); }

// ------------------------------------------------------------------------------------------
// work distribution
// ------------------------------------------------------------------------------------------
struct Item { int row, begin, end, slot; };

// Blocks go round-robin to the 8 XCDs; remap so XCD x gets a contiguous run of block indices.
__device__ __forceinline__ int xcd_contiguous_block() {
    const int nb = gridDim.x, b = blockIdx.x;
    const int q = nb >> 3, rem = nb & 7, x = b & 7, k = b >> 3;
    return x * q + (x < rem ? x : rem) + k;
}

__device__ __forceinline__ bool fetch_item(const bpt_plan &P, Item &it) {
    const int w = xcd_contiguous_block() * WAVES_PER_BLOCK + (int)(threadIdx.x >> 6);
    if (w >= (int)P.n_items) return false;
    const int4 v = reinterpret_cast<const int4 *>(P.items)[w];
    // the item is the same for all lanes of the wavefront: keep it in scalar registers
    it.row = __builtin_amdgcn_readfirstlane(v.x);
    it.begin = __builtin_amdgcn_readfirstlane(v.y);
    it.end = __builtin_amdgcn_readfirstlane(v.z);
    it.slot = __builtin_amdgcn_readfirstlane(v.w);
    return true;
}

template <typename A> __device__ __forceinline__ A wave_sum(A x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
    return x;
}
template <typename A> __device__ __forceinline__ A wave_max(A x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        A y = __shfl_xor(x, o);
        x = x > y ? x : y;
    }
    return x;
}

// Reduction over NW wavefronts of a block (NW == 1: a single wavefront, no LDS, no barrier).
template <typename A, int NW, bool IS_MAX> __device__ __forceinline__ A group_reduce(A x, A *smem) {
    x = IS_MAX ? wave_max(x) : wave_sum(x);
    if (NW == 1) return x;
    const int w = threadIdx.x >> 6;
    __syncthreads();                       // smem may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) smem[w] = x;
    __syncthreads();
    A r = smem[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) r = IS_MAX ? (r > smem[i] ? r : smem[i]) : r + smem[i];
    return r;
}

// ------------------------------------------------------------------------------------------
// generic kernels
// ------------------------------------------------------------------------------------------
// y[eid[p], h] = sum_d A[row, h, d] * B[..]   MODE 0: B (n, H, D) row idx[p];  MODE 1: B (E, D) row eid[p]
template <typename T, int MODE>
__global__ __launch_bounds__(BLOCK) void k_sddmm_generic(bpt_plan P, const T *__restrict__ A, const T *__restrict__ B,
                                                         T *__restrict__ y, int H, int D) {
    using acc_t = typename Elem<T>::acc_t;
    Item it;
    if (!fetch_item(P, it)) return;
    const int lane = threadIdx.x & 63;
    const T *a = A + (size_t)it.row * H * D;
    for (int p = it.begin; p < it.end; ++p) {
        const int e = P.eid[p];
        const T *b = (MODE == 0) ? B + (size_t)P.idx[p] * H * D : B + (size_t)e * D;
        for (int h = 0; h < H; ++h) {
            acc_t s = 0;
            for (int dd = lane; dd < D; dd += WAVE)
                s += (acc_t)Elem<T>::ld(a + h * D + dd) * (acc_t)Elem<T>::ld(b + (MODE == 0 ? h * D : 0) + dd);
            s = wave_sum(s);
            if (lane == 0) Elem<T>::st(y + (size_t)e * H + h, s);
        }
    }
}

// Y[row, j] = sum_p W[eid[p], j / D] * X[..]   MODE 0: X (n, H, D) row idx[p];  MODE 1: X (E, D) row eid[p], column j % D
template <typename T, int MODE>
__global__ __launch_bounds__(BLOCK) void k_spmm_generic(bpt_plan P, const T *__restrict__ W, const T *__restrict__ X,
                                                        T *__restrict__ Y, typename Elem<T>::acc_t *__restrict__ ws,
                                                        int H, int D) {
    using acc_t = typename Elem<T>::acc_t;
    Item it;
    if (!fetch_item(P, it)) return;
    const int lane = threadIdx.x & 63;
    const int C = H * D;
    for (int j = lane; j < C; j += WAVE) {
        const int h = j / D;
        acc_t s = 0;
        for (int p = it.begin; p < it.end; ++p) {
            const int e = P.eid[p];
            const acc_t w = Elem<T>::ld(W + (size_t)e * H + h);
            const acc_t xv = (MODE == 0) ? Elem<T>::ld(X + (size_t)P.idx[p] * C + j) : Elem<T>::ld(X + (size_t)e * D + (j - h * D));
            s += w * xv;
        }
        if (it.slot < 0) Elem<T>::st(Y + (size_t)it.row * C + j, s);
        else ws[(size_t)it.slot * C + j] = s;
    }
}

// Y[row, :] = sum of the row's partial slots.  Grid (n_heavy, ceil(C / 64), n_out): one block per split
// row, 64-column strip and output tensor (output z reads its partials n_slots*C further into the
// workspace).  Wave w adds slots w, w+4, ... (eight independent loads per step); the four wave sums
// are then added in wave order, so the result is a fixed function of the plan.
template <typename T>
__device__ __forceinline__ void combine_sum_block(const int32_t *__restrict__ hv, const typename Elem<T>::acc_t *__restrict__ ws,
                                                  T *__restrict__ Y, int C, bool accumulate = false) {
    using acc_t = typename Elem<T>::acc_t;
    __shared__ acc_t part[WAVES_PER_BLOCK][WAVE];
    const int row = hv[0], s0 = hv[1], ns = hv[2];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int j = blockIdx.y * WAVE + lane;
    acc_t s = 0;
    if (j < C) {
        const acc_t *col = ws + (size_t)s0 * C + j;
        int k = w;
        for (; k + 7 * WAVES_PER_BLOCK < ns; k += 8 * WAVES_PER_BLOCK) {
            acc_t t[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) t[u] = col[(size_t)(k + u * WAVES_PER_BLOCK) * C];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += t[u];
        }
        for (; k < ns; k += WAVES_PER_BLOCK) s += col[(size_t)k * C];
    }
    part[w][lane] = s;
    __syncthreads();
    if (w == 0 && j < C) {
        acc_t r = part[0][lane];
#pragma unroll
        for (int i = 1; i < WAVES_PER_BLOCK; ++i) r += part[i][lane];
        if (accumulate) r += Elem<T>::ld(Y + (size_t)row * C + j);
        Elem<T>::st(Y + (size_t)row * C + j, r);
    }
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void k_combine_sum(const int32_t *__restrict__ heavy,
                                                       const typename Elem<T>::acc_t *__restrict__ ws, T *__restrict__ Y0,
                                                       T *__restrict__ Y1, int C, size_t ws_stride, int accumulate = 0) {
    combine_sum_block<T>(heavy + 3 * blockIdx.x, ws + (size_t)blockIdx.z * ws_stride, blockIdx.z == 0 ? Y0 : Y1, C, accumulate != 0);
}

// The three sums of the fused backward in one launch, four columns per lane (C a multiple of 256, float partials): grid
// (n_a + n_b, C / 256, 2); blocks x < n_a combine rows of list A into YA (z = 0 only), the others rows of list B into YB0
// (z = 0) and YB1 (z = 1).  Every column is added in the order combine_sum_block uses (wave w takes slots w, w + 4, ...;
// the four wave sums in wave order).
template <typename T> __device__ __forceinline__ void store4(T *p, float4 v);
template <> __device__ __forceinline__ void store4<float>(float *p, float4 v) { *reinterpret_cast<float4 *>(p) = v; }
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t *p, float4 v) {
    *reinterpret_cast<uint2 *>(p) = make_uint2((uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16),
                                               (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16));
}
template <typename T> __device__ __forceinline__ float4 load4(const T *p);
template <> __device__ __forceinline__ float4 load4<float>(const float *p) { return *reinterpret_cast<const float4 *>(p); }
template <> __device__ __forceinline__ float4 load4<bf16_t>(const bf16_t *p) {
    const uint2 x = *reinterpret_cast<const uint2 *>(p);
    return make_float4(__uint_as_float(x.x << 16), __uint_as_float(x.x & 0xffff0000u), __uint_as_float(x.y << 16), __uint_as_float(x.y & 0xffff0000u));
}
template <typename T>
__device__ __forceinline__ void combine_sum_block4(const int32_t *__restrict__ hv, const float *__restrict__ ws, T *__restrict__ Y, int C,
                                                   bool accumulate = false, int strip = -1) {
    __shared__ float4 part[WAVES_PER_BLOCK][WAVE];
    const int row = hv[0], s0 = hv[1], ns = hv[2];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int j = ((strip < 0 ? (int)blockIdx.y : strip) * WAVE + lane) * 4;     // strip of 256 columns: the grid's y unless given
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    const float *col = ws + (size_t)s0 * C + j;
    int k = w;
    for (; k + 7 * WAVES_PER_BLOCK < ns; k += 8 * WAVES_PER_BLOCK) {
        float4 t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) t[u] = *reinterpret_cast<const float4 *>(col + (size_t)(k + u * WAVES_PER_BLOCK) * C);
#pragma unroll
        for (int u = 0; u < 8; ++u) { s.x += t[u].x; s.y += t[u].y; s.z += t[u].z; s.w += t[u].w; }
    }
    for (; k < ns; k += WAVES_PER_BLOCK) {
        const float4 t = *reinterpret_cast<const float4 *>(col + (size_t)k * C);
        s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
    }
    part[w][lane] = s;
    __syncthreads();
    if (w == 0) {
        float4 r = part[0][lane];
#pragma unroll
        for (int i = 1; i < WAVES_PER_BLOCK; ++i) { r.x += part[i][lane].x; r.y += part[i][lane].y; r.z += part[i][lane].z; r.w += part[i][lane].w; }
        if (accumulate) {
            const float4 y = load4<T>(Y + (size_t)row * C + j);
            r.x += y.x; r.y += y.y; r.z += y.z; r.w += y.w;
        }
        store4<T>(Y + (size_t)row * C + j, r);
    }
}
template <typename T>
__global__ __launch_bounds__(BLOCK) void k_combine_sum3(const int32_t *__restrict__ heavy_a, int n_a, const float *__restrict__ ws_a,
                                                           T *__restrict__ YA, const int32_t *__restrict__ heavy_b,
                                                           const float *__restrict__ ws_b, T *__restrict__ YB0, T *__restrict__ YB1, int C,
                                                           size_t ws_stride_b) {
    if ((int)blockIdx.x < n_a) {
        if (blockIdx.z == 0) combine_sum_block4<T>(heavy_a + 3 * blockIdx.x, ws_a, YA, C);
    } else {
        combine_sum_block4<T>(heavy_b + 3 * (blockIdx.x - n_a), ws_b + (size_t)blockIdx.z * ws_stride_b, blockIdx.z == 0 ? YB0 : YB1, C);
    }
}

// k_combine_sum for the specialised shapes (float partials, C a multiple of 256): grid (n_heavy, C / 256, n_out)
template <typename T>
__global__ __launch_bounds__(BLOCK) void k_combine_sum_v4(const int32_t *__restrict__ heavy, const float *__restrict__ ws, T *__restrict__ Y0,
                                                          T *__restrict__ Y1, int C, size_t ws_stride, int accumulate = 0) {
    combine_sum_block4<T>(heavy + 3 * blockIdx.x, ws + (size_t)blockIdx.z * ws_stride, blockIdx.z == 0 ? Y0 : Y1, C, accumulate != 0);
}

// dB[eid[p], d] = sum_h dy[eid[p], h] * A[row, h, d]      (graphop_kernel.cu:79-94)
template <typename T>
__global__ __launch_bounds__(BLOCK) void k_nme_dB_generic(bpt_plan P, const T *__restrict__ A, const T *__restrict__ dy,
                                                          T *__restrict__ dB, int H, int D) {
    using acc_t = typename Elem<T>::acc_t;
    Item it;
    if (!fetch_item(P, it)) return;
    const int lane = threadIdx.x & 63;
    const T *a = A + (size_t)it.row * H * D;
    for (int p = it.begin; p < it.end; ++p) {
        const int e = P.eid[p];
        for (int dd = lane; dd < D; dd += WAVE) {
            acc_t s = 0;
            for (int h = 0; h < H; ++h) s += (acc_t)Elem<T>::ld(dy + (size_t)e * H + h) * (acc_t)Elem<T>::ld(a + h * D + dd);
            Elem<T>::st(dB + (size_t)e * D + dd, s);
        }
    }
}

// Row softmax.  NW == 1: one wavefront per whole-row item (segments of split rows exit);
// NW == WAVES_PER_BLOCK: one block per split row (grid = n_heavy).
template <typename T, int NW>
__global__ __launch_bounds__(BLOCK) void k_softmax_fwd(bpt_plan P, const T *__restrict__ x, T *__restrict__ y, int H) {
    using acc_t = typename Elem<T>::acc_t;
    __shared__ acc_t smem[WAVES_PER_BLOCK];
    int begin, end, tid;
    if (NW == 1) {
        Item it;
        if (!fetch_item(P, it) || it.slot >= 0) return;
        begin = it.begin; end = it.end; tid = threadIdx.x & 63;
    } else {
        const int row = P.heavy[3 * blockIdx.x];
        begin = P.rowptr[row]; end = P.rowptr[row + 1]; tid = threadIdx.x;
    }
    constexpr int NT = NW * WAVE;
    for (int h = 0; h < H; ++h) {
        acc_t m = (acc_t)-1e9;
        for (int p = begin + tid; p < end; p += NT) {
            const acc_t v = Elem<T>::ld(x + (size_t)P.eid[p] * H + h);
            m = v > m ? v : m;
        }
        m = group_reduce<acc_t, NW, true>(m, smem);
        acc_t s = 0;
        for (int p = begin + tid; p < end; p += NT) s += exp_acc((acc_t)Elem<T>::ld(x + (size_t)P.eid[p] * H + h) - m);
        s = group_reduce<acc_t, NW, false>(s, smem);
        for (int p = begin + tid; p < end; p += NT) {
            const size_t o = (size_t)P.eid[p] * H + h;
            Elem<T>::st(y + o, exp_acc((acc_t)Elem<T>::ld(x + o) - m) / s);
        }
    }
}

// dx = dy*y - (sum_row dy*y) * y      (graphop_kernel.cu:208-230)
template <typename T, int NW>
__global__ __launch_bounds__(BLOCK) void k_softmax_bwd(bpt_plan P, const T *__restrict__ y, const T *__restrict__ dy,
                                                       T *__restrict__ dx, int H) {
    using acc_t = typename Elem<T>::acc_t;
    __shared__ acc_t smem[WAVES_PER_BLOCK];
    int begin, end, tid;
    if (NW == 1) {
        Item it;
        if (!fetch_item(P, it) || it.slot >= 0) return;
        begin = it.begin; end = it.end; tid = threadIdx.x & 63;
    } else {
        const int row = P.heavy[3 * blockIdx.x];
        begin = P.rowptr[row]; end = P.rowptr[row + 1]; tid = threadIdx.x;
    }
    constexpr int NT = NW * WAVE;
    for (int h = 0; h < H; ++h) {
        acc_t s = 0;
        for (int p = begin + tid; p < end; p += NT) {
            const size_t o = (size_t)P.eid[p] * H + h;
            s += (acc_t)Elem<T>::ld(dy + o) * (acc_t)Elem<T>::ld(y + o);
        }
        s = group_reduce<acc_t, NW, false>(s, smem);
        for (int p = begin + tid; p < end; p += NT) {
            const size_t o = (size_t)P.eid[p] * H + h;
            const acc_t yv = Elem<T>::ld(y + o);
            Elem<T>::st(dx + o, (acc_t)Elem<T>::ld(dy + o) * yv - s * yv);
        }
    }
}

// Row softmax with the heads side by side: thread t handles head t % H of edge slot t / H, so a wavefront reads
// 64 / H whole (E, H) rows per step (H must divide 64).  NW == 1: one wavefront per whole-row item; NW > 1: one
// block of NW wavefronts per split row (grid = n_heavy).  Rows of up to SM_CACHE steps keep their values in
// registers and read memory once; longer rows re-read.  Loads are issued SM_CACHE at a time.
constexpr int SM_CACHE = 8;

// reduction over the threads of a block that share t % H (H divides 64): first inside each wavefront, then over LDS
template <typename A, int NW, bool IS_MAX> __device__ __forceinline__ A head_reduce(A x, int H, int h, A *smem) {
    for (int off = H; off < WAVE; off <<= 1) {
        const A o = __shfl_xor(x, off);
        x = IS_MAX ? (x > o ? x : o) : x + o;
    }
    if (NW == 1) return x;
    const int w = threadIdx.x >> 6;
    __syncthreads();                       // smem may still be read from the previous reduction
    if ((int)(threadIdx.x & 63) < H) smem[w * WAVE + h] = x;
    __syncthreads();
    A r = smem[h];
    for (int i = 1; i < NW; ++i) r = IS_MAX ? (r > smem[i * WAVE + h] ? r : smem[i * WAVE + h]) : r + smem[i * WAVE + h];
    return r;
}

// seg_slot: NULL = whole rows only (segments of split rows are skipped); else it receives the item's slot (-1 = whole row)
template <int NW> __device__ __forceinline__ bool softmax_range(const bpt_plan &P, int &begin, int &end, int *seg_slot = nullptr) {
    if (NW == 1) {
        Item it;
        if (!fetch_item(P, it) || (it.slot >= 0 && !seg_slot)) return false;
        begin = it.begin; end = it.end;
        if (seg_slot) *seg_slot = it.slot;
    } else {
        const int row = P.heavy[3 * blockIdx.x];
        begin = P.rowptr[row]; end = P.rowptr[row + 1];
    }
    return true;
}

template <typename T, int NW>
__global__ __launch_bounds__(NW == 1 ? BLOCK : NW * WAVE) void k_softmax_fwd_heads(bpt_plan P, const T *__restrict__ x, T *__restrict__ y, int H,
                                                                                   typename Elem<T>::acc_t *__restrict__ seg) {
    using acc_t = typename Elem<T>::acc_t;
    __shared__ acc_t smem[NW == 1 ? 1 : NW * WAVE];
    int begin, end, seg_slot = -1;
    if (!softmax_range<NW>(P, begin, end, seg ? &seg_slot : nullptr)) return;
    const int tid = NW == 1 ? (int)(threadIdx.x & 63) : (int)threadIdx.x;
    const int h = tid % H, slot = tid / H, nslots = NW * WAVE / H;
    const bool cached = end - begin <= SM_CACHE * nslots;
    acc_t vc[SM_CACHE];
    size_t oc[SM_CACHE];
#pragma unroll
    for (int u = 0; u < SM_CACHE; ++u) { vc[u] = (acc_t)-INFINITY; oc[u] = (size_t)-1; }    // threads past a short row's end
    acc_t m = (acc_t)-1e9;
    for (int p0 = begin + slot; p0 < end; p0 += SM_CACHE * nslots) {
        int e[SM_CACHE];
#pragma unroll
        for (int u = 0; u < SM_CACHE; ++u) { const int p = p0 + u * nslots; e[u] = p < end ? P.eid[p] : -1; }
#pragma unroll
        for (int u = 0; u < SM_CACHE; ++u) {
            oc[u] = (size_t)(e[u] < 0 ? 0 : e[u]) * H + h;
            vc[u] = e[u] < 0 ? (acc_t)-INFINITY : (acc_t)Elem<T>::ld(x + oc[u]);
            m = vc[u] > m ? vc[u] : m;
            if (e[u] < 0) oc[u] = (size_t)-1;
        }
    }
    m = head_reduce<acc_t, NW, true>(m, H, h, smem);
    acc_t s = 0;
    if (cached) {
#pragma unroll
        for (int u = 0; u < SM_CACHE; ++u) { vc[u] = exp_acc(vc[u] - m); s += vc[u]; }      // exp(-inf) = 0 for the empty slots
    } else {
        for (int p = begin + slot; p < end; p += nslots) s += exp_acc((acc_t)Elem<T>::ld(x + (size_t)P.eid[p] * H + h) - m);
    }
    s = head_reduce<acc_t, NW, false>(s, H, h, smem);
    if (seg_slot >= 0) {
        // a segment of a split row: y gets exp(x - m) of the segment; its (m, s) go to the workspace, from which
        // k_softmax_seg_rows forms the factor exp(m - M) / S that k_softmax_seg_scale applies
        if (slot == 0) { seg[((size_t)seg_slot * H + h) * 2] = m; seg[((size_t)seg_slot * H + h) * 2 + 1] = s; }
        s = 1;
    }
    if (cached) {
#pragma unroll
        for (int u = 0; u < SM_CACHE; ++u)
            if (oc[u] != (size_t)-1) Elem<T>::st(y + oc[u], vc[u] / s);
    } else {
        for (int p0 = begin + slot; p0 < end; p0 += SM_CACHE * nslots) {
            int e[SM_CACHE];
#pragma unroll
            for (int u = 0; u < SM_CACHE; ++u) { const int p = p0 + u * nslots; e[u] = p < end ? P.eid[p] : -1; }
            acc_t v[SM_CACHE];
#pragma unroll
            for (int u = 0; u < SM_CACHE; ++u) v[u] = e[u] < 0 ? (acc_t)0 : (acc_t)Elem<T>::ld(x + (size_t)e[u] * H + h);
#pragma unroll
            for (int u = 0; u < SM_CACHE; ++u)
                if (e[u] >= 0) Elem<T>::st(y + (size_t)e[u] * H + h, exp_acc(v[u] - m) / s);
        }
    }
}

template <typename T, int NW>
__global__ __launch_bounds__(NW == 1 ? BLOCK : NW * WAVE) void k_softmax_bwd_heads(bpt_plan P, const T *__restrict__ y, const T *__restrict__ dy,
                                                                                   T *__restrict__ dx, int H,
                                                                                   typename Elem<T>::acc_t *__restrict__ seg) {
    using acc_t = typename Elem<T>::acc_t;
    __shared__ acc_t smem[NW == 1 ? 1 : NW * WAVE];
    int begin, end, seg_slot = -1;
    if (!softmax_range<NW>(P, begin, end, seg ? &seg_slot : nullptr)) return;
    const int tid = NW == 1 ? (int)(threadIdx.x & 63) : (int)threadIdx.x;
    const int h = tid % H, slot = tid / H, nslots = NW * WAVE / H;
    const bool cached = end - begin <= SM_CACHE * nslots;
    acc_t yc[SM_CACHE], dc[SM_CACHE];
    size_t oc[SM_CACHE];
#pragma unroll
    for (int u = 0; u < SM_CACHE; ++u) { yc[u] = 0; dc[u] = 0; oc[u] = (size_t)-1; }
    acc_t s = 0;
    for (int p0 = begin + slot; p0 < end; p0 += SM_CACHE * nslots) {
        int e[SM_CACHE];
#pragma unroll
        for (int u = 0; u < SM_CACHE; ++u) { const int p = p0 + u * nslots; e[u] = p < end ? P.eid[p] : -1; }
#pragma unroll
        for (int u = 0; u < SM_CACHE; ++u) {
            oc[u] = (size_t)(e[u] < 0 ? 0 : e[u]) * H + h;
            yc[u] = e[u] < 0 ? (acc_t)0 : (acc_t)Elem<T>::ld(y + oc[u]);
            dc[u] = e[u] < 0 ? (acc_t)0 : (acc_t)Elem<T>::ld(dy + oc[u]);
            if (e[u] < 0) oc[u] = (size_t)-1;
        }
#pragma unroll
        for (int u = 0; u < SM_CACHE; ++u) s += dc[u] * yc[u];
    }
    s = head_reduce<acc_t, NW, false>(s, H, h, smem);
    if (seg_slot >= 0) {
        // a segment of a split row: only its part of sum(dy * y); k_softmax_seg_rows adds the parts up and
        // k_softmax_bwd_seg_finish writes dx
        if (slot == 0) seg[(size_t)seg_slot * H + h] = s;
        return;
    }
    if (cached) {
#pragma unroll
        for (int u = 0; u < SM_CACHE; ++u)
            if (oc[u] != (size_t)-1) Elem<T>::st(dx + oc[u], dc[u] * yc[u] - s * yc[u]);
    } else {
        for (int p0 = begin + slot; p0 < end; p0 += SM_CACHE * nslots) {
            int e[SM_CACHE];
#pragma unroll
            for (int u = 0; u < SM_CACHE; ++u) { const int p = p0 + u * nslots; e[u] = p < end ? P.eid[p] : -1; }
            acc_t yv[SM_CACHE], dv[SM_CACHE];
#pragma unroll
            for (int u = 0; u < SM_CACHE; ++u) {
                const size_t o = (size_t)(e[u] < 0 ? 0 : e[u]) * H + h;
                yv[u] = e[u] < 0 ? (acc_t)0 : (acc_t)Elem<T>::ld(y + o);
                dv[u] = e[u] < 0 ? (acc_t)0 : (acc_t)Elem<T>::ld(dy + o);
            }
#pragma unroll
            for (int u = 0; u < SM_CACHE; ++u)
                if (e[u] >= 0) Elem<T>::st(dx + (size_t)e[u] * H + h, dv[u] * yv[u] - s * yv[u]);
        }
    }
}

// Split rows of the softmax, second step: one block per split row.  Forward (PAIR): the segments' (m_i, s_i) become the
// factors exp(m_i - M) / S with M = max(-1e9, m_i), S = sum s_i exp(m_i - M) (stored over m_i); backward: the segments'
// partial sums are replaced by their total.  Thread t handles head t % H of slots t / H, t / H + n, ...
template <typename A, bool PAIR>
__global__ __launch_bounds__(BLOCK) void k_softmax_seg_rows(const int32_t *__restrict__ heavy, A *__restrict__ seg, int H) {
    __shared__ A smem[WAVES_PER_BLOCK * WAVE];
    const int s0 = heavy[3 * blockIdx.x + 1], ns = heavy[3 * blockIdx.x + 2];
    const int h = threadIdx.x % H, j0 = threadIdx.x / H, nj = BLOCK / H;
    constexpr int ST = PAIR ? 2 : 1;
    if constexpr (PAIR) {
        A m = (A)-1e9;
        for (int j = j0; j < ns; j += nj) { const A v = seg[((size_t)(s0 + j) * H + h) * ST]; m = v > m ? v : m; }
        m = head_reduce<A, WAVES_PER_BLOCK, true>(m, H, h, smem);
        A s = 0;
        for (int j = j0; j < ns; j += nj) s += seg[((size_t)(s0 + j) * H + h) * ST + 1] * exp_acc(seg[((size_t)(s0 + j) * H + h) * ST] - m);
        s = head_reduce<A, WAVES_PER_BLOCK, false>(s, H, h, smem);
        for (int j = j0; j < ns; j += nj) {
            A *q = seg + ((size_t)(s0 + j) * H + h) * ST;
            q[0] = exp_acc(q[0] - m) / s;
        }
    } else {
        A s = 0;
        for (int j = j0; j < ns; j += nj) s += seg[(size_t)(s0 + j) * H + h];
        s = head_reduce<A, WAVES_PER_BLOCK, false>(s, H, h, smem);
        for (int j = j0; j < ns; j += nj) seg[(size_t)(s0 + j) * H + h] = s;
    }
}

// third step, one wavefront per item, segments only.  Forward: y *= factor of the segment.
template <typename T>
__global__ __launch_bounds__(BLOCK) void k_softmax_seg_scale(bpt_plan P, T *__restrict__ y, int H, const typename Elem<T>::acc_t *__restrict__ seg) {
    using acc_t = typename Elem<T>::acc_t;
    Item it;
    if (!fetch_item(P, it) || it.slot < 0) return;
    const int tid = threadIdx.x & 63, h = tid % H, nslots = WAVE / H;
    const acc_t f = seg[((size_t)it.slot * H + h) * 2];
    for (int p = it.begin + tid / H; p < it.end; p += nslots) {
        const size_t o = (size_t)P.eid[p] * H + h;
        Elem<T>::st(y + o, (acc_t)Elem<T>::ld(y + o) * f);
    }
}

// Backward: dx = y * (dy - total) on the segments.
template <typename T>
__global__ __launch_bounds__(BLOCK) void k_softmax_bwd_seg_finish(bpt_plan P, const T *__restrict__ y, const T *__restrict__ dy, T *__restrict__ dx,
                                                                  int H, const typename Elem<T>::acc_t *__restrict__ seg) {
    using acc_t = typename Elem<T>::acc_t;
    Item it;
    if (!fetch_item(P, it) || it.slot < 0) return;
    const int tid = threadIdx.x & 63, h = tid % H, nslots = WAVE / H;
    const acc_t t = seg[(size_t)it.slot * H + h];
    for (int p = it.begin + tid / H; p < it.end; p += nslots) {
        const size_t o = (size_t)P.eid[p] * H + h;
        const acc_t yv = (acc_t)Elem<T>::ld(y + o);
        Elem<T>::st(dx + o, yv * ((acc_t)Elem<T>::ld(dy + o) - t));
    }
}

// ------------------------------------------------------------------------------------------
// fast family: compile-time (H, D), f32 / bf16
// ------------------------------------------------------------------------------------------
template <typename T, int H_, int D_> struct Lay {
    static constexpr int H = H_, D = D_, C = H_ * D_;
    static constexpr int LPH = 64 / H_;                 // lanes per head
    static constexpr int EPL = C / 64;                  // elements per lane (all of one head)
    static constexpr int VE = 16 / (int)sizeof(T);      // elements per 16-byte vector
    static constexpr int NV = EPL / VE;                 // 16-byte vectors per lane
    static_assert(64 % H_ == 0 && C % 64 == 0 && EPL % VE == 0 && NV >= 1, "unsupported fast shape");
    static_assert(LPH >= 4, "the row-group kernels broadcast per-member values inside quads of one head");
    static_assert(D_ == NV * LPH * VE, "layout does not tile the head");
    // element offset inside a node row of vector i of `lane`: LPH consecutive lanes cover
    // LPH*16 contiguous bytes of their head
    static __device__ __forceinline__ int off(int lane, int i) { return (lane / LPH) * D + (i * LPH + lane % LPH) * VE; }
};

template <typename T, int H, int D>
__device__ __forceinline__ void load_row(const T *__restrict__ row, int lane, float (&out)[Lay<T, H, D>::EPL]) {
    using L = Lay<T, H, D>;
#pragma unroll
    for (int i = 0; i < L::NV; ++i) {
        if constexpr (sizeof(T) == 4) {
            const float4 v = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(row) + L::off(lane, i));
            out[4 * i] = v.x; out[4 * i + 1] = v.y; out[4 * i + 2] = v.z; out[4 * i + 3] = v.w;
        } else {
            const uint4 v = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(row) + L::off(lane, i));
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                out[8 * i + 2 * c] = __uint_as_float(w[c] << 16);
                out[8 * i + 2 * c + 1] = __uint_as_float(w[c] & 0xffff0000u);
            }
        }
    }
}

template <typename T, int H, int D>
__device__ __forceinline__ void store_row(T *__restrict__ row, int lane, const float (&in)[Lay<T, H, D>::EPL]) {
    using L = Lay<T, H, D>;
#pragma unroll
    for (int i = 0; i < L::NV; ++i) {
        if constexpr (sizeof(T) == 4) {
            *reinterpret_cast<float4 *>(reinterpret_cast<float *>(row) + L::off(lane, i)) =
                make_float4(in[4 * i], in[4 * i + 1], in[4 * i + 2], in[4 * i + 3]);
        } else {
            uint32_t w[4];
#pragma unroll
            for (int c = 0; c < 4; ++c)
                w[c] = (uint32_t)f32_to_bf16(in[8 * i + 2 * c]) | ((uint32_t)f32_to_bf16(in[8 * i + 2 * c + 1]) << 16);
            *reinterpret_cast<uint4 *>(reinterpret_cast<uint16_t *>(row) + L::off(lane, i)) = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
}

// The D elements of an (E, D) edge-feature row that go with this lane's slice of a head (every head's lanes read
// the same D elements).
template <typename T, int H, int D>
__device__ __forceinline__ void load_head_row(const T *__restrict__ row, int lane, float (&out)[Lay<T, H, D>::EPL]) {
    using L = Lay<T, H, D>;
#pragma unroll
    for (int i = 0; i < L::NV; ++i) {
        const int off = (i * L::LPH + lane % L::LPH) * L::VE;
        if constexpr (sizeof(T) == 4) {
            const float4 v = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(row) + off);
            out[4 * i] = v.x; out[4 * i + 1] = v.y; out[4 * i + 2] = v.z; out[4 * i + 3] = v.w;
        } else {
            const uint4 v = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(row) + off);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                out[8 * i + 2 * c] = __uint_as_float(w[c] << 16);
                out[8 * i + 2 * c + 1] = __uint_as_float(w[c] & 0xffff0000u);
            }
        }
    }
}

// f32 partial rows in the workspace are stored in natural column order (the combine kernels
// index them by column), whatever the element type of the node tensors
template <typename T, int H, int D>
__device__ __forceinline__ void store_row_ws(float *__restrict__ row, int lane, const float (&in)[Lay<T, H, D>::EPL]) {
    using L = Lay<T, H, D>;
#pragma unroll
    for (int i = 0; i < L::NV; ++i)
#pragma unroll
        for (int c = 0; c < L::VE / 4; ++c)
            *reinterpret_cast<float4 *>(row + L::off(lane, i) + 4 * c) =
                make_float4(in[L::VE * i + 4 * c], in[L::VE * i + 4 * c + 1], in[L::VE * i + 4 * c + 2], in[L::VE * i + 4 * c + 3]);
}

template <int CTRL> __device__ __forceinline__ float dpp_mov(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true));
}

template <int I> __device__ __forceinline__ float quad_lane(float x) { return dpp_mov<I * 0x55>(x); }   // value of lane I of the quad
__device__ __forceinline__ float quad_bcast(float x, int i) {      // the same for an index that is constant after unrolling
    switch (i & 3) {
    case 0: return quad_lane<0>(x);
    case 1: return quad_lane<1>(x);
    case 2: return quad_lane<2>(x);
    default: return quad_lane<3>(x);
    }
}

// Sum over the LPH lanes that hold one head; the result is in all of them.
template <int LPH> __device__ __forceinline__ float head_sum(float x) {
    if constexpr (LPH >= 2) x += dpp_mov<0xB1>(x);    // quad_perm [1,0,3,2]
    if constexpr (LPH >= 4) x += dpp_mov<0x4E>(x);    // quad_perm [2,3,0,1]
    if constexpr (LPH >= 8) x += dpp_mov<0x141>(x);   // row_half_mirror
    if constexpr (LPH >= 16) x += dpp_mov<0x140>(x);  // row_mirror
    if constexpr (LPH >= 32) x += __shfl_xor(x, 16);
    if constexpr (LPH >= 64) x += __shfl_xor(x, 32);
    return x;
}

template <int N> __device__ __forceinline__ float dot_n(const float (&a)[N], const float (&b)[N]) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < N; ++i) s = fmaf(a[i], b[i], s);
    return s;
}

// The gathers are latency bound: all row loads of a batch must be in flight before the first
// one is consumed.  Without this fence the instruction scheduler interleaves loads and FMAs to
// save registers and waits for every load separately.
__device__ __forceinline__ void issue_loads_first() { __builtin_amdgcn_sched_barrier(0); }

// weight loads for the fast SpMM: the unfused API passes T-typed edge data, the fused backward f32
template <typename WT> __device__ __forceinline__ float ld_w(const WT *p) { return Elem<WT>::ld(p); }

// y[eid[p], head] = A[row, head, :] . B[idx[p], head, :]   (MODE 1: . B[eid[p], :], B an (E, D) edge feature;
// MODE 2: . B[idx[p], :], B a (n_index, D) table shared by the heads).  YT: element type of y.
template <typename T, int H, int D, int BATCH, int MODE = 0, typename YT = T>
__global__ __launch_bounds__(BLOCK) void k_sddmm_fast(bpt_plan P, const T *__restrict__ A, const T *__restrict__ B, YT *__restrict__ y) {
    using L = Lay<T, H, D>;
    Item it;
    if (!fetch_item(P, it)) return;
    const int lane = threadIdx.x & 63, head = lane / L::LPH;
    float a[L::EPL];
    load_row<T, H, D>(A + (size_t)it.row * L::C, lane, a);
    for (int p0 = it.begin; p0 < it.end; p0 += WAVE) {
        const int cnt = min(WAVE, it.end - p0);
        const int my_idx = (MODE != 1 && lane < cnt) ? P.idx[p0 + lane] : 0;
        const int my_eid = lane < cnt ? P.eid[p0 + lane] : 0;
        for (int b = 0; b < cnt; b += BATCH) {
            float bv[BATCH][L::EPL];
            int ee[BATCH];
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                const int j = (b + e < cnt) ? b + e : b;
                ee[e] = __builtin_amdgcn_readlane(my_eid, j);
                if constexpr (MODE == 0) load_row<T, H, D>(B + (size_t)__builtin_amdgcn_readlane(my_idx, j) * L::C, lane, bv[e]);
                else if constexpr (MODE == 1) load_head_row<T, H, D>(B + (size_t)ee[e] * D, lane, bv[e]);
                else load_head_row<T, H, D>(B + (size_t)__builtin_amdgcn_readlane(my_idx, j) * D, lane, bv[e]);
            }
            issue_loads_first();
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                const float s = head_sum<L::LPH>(dot_n<L::EPL>(a, bv[e]));
                if (b + e < cnt && lane % L::LPH == 0) Elem<YT>::st(y + (size_t)ee[e] * H + head, s);
            }
        }
    }
}

// Y0[row] = sum_p W0[eid[p], head] * X0[idx[p]]  (and the same with W1, X1 -> Y1 when NOUT == 2);
// MODE 1: * X0[eid[p], :], X0 an (E, D) edge feature shared by the heads
template <typename T, typename WT, int H, int D, int BATCH, int NOUT, int MODE = 0>
__global__ __launch_bounds__(BLOCK) void k_spmm_fast(bpt_plan P, const WT *__restrict__ W0, const T *__restrict__ X0, T *__restrict__ Y0,
                                                     const WT *__restrict__ W1, const T *__restrict__ X1, T *__restrict__ Y1,
                                                     float *__restrict__ ws0, float *__restrict__ ws1) {
    using L = Lay<T, H, D>;
    Item it;
    if (!fetch_item(P, it)) return;
    const int lane = threadIdx.x & 63, head = lane / L::LPH;
    float acc0[L::EPL], acc1[L::EPL];
#pragma unroll
    for (int i = 0; i < L::EPL; ++i) { acc0[i] = 0.f; acc1[i] = 0.f; }
    for (int p0 = it.begin; p0 < it.end; p0 += WAVE) {
        const int cnt = min(WAVE, it.end - p0);
        const int my_idx = (MODE == 0 && lane < cnt) ? P.idx[p0 + lane] : 0;
        const int my_eid = lane < cnt ? P.eid[p0 + lane] : 0;
        for (int b = 0; b < cnt; b += BATCH) {
            float x0[BATCH][L::EPL], x1[NOUT == 2 ? BATCH : 1][L::EPL];
            float w0[BATCH], w1[BATCH];
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                const bool ok = b + e < cnt;
                const int j = ok ? b + e : b;
                const int src = __builtin_amdgcn_readlane(my_idx, j);
                const int ed = __builtin_amdgcn_readlane(my_eid, j);
                if constexpr (MODE == 0) load_row<T, H, D>(X0 + (size_t)src * L::C, lane, x0[e]);
                else load_head_row<T, H, D>(X0 + (size_t)ed * D, lane, x0[e]);
                w0[e] = ok ? ld_w(W0 + (size_t)ed * H + head) : 0.f;
                if constexpr (NOUT == 2) {
                    load_row<T, H, D>(X1 + (size_t)src * L::C, lane, x1[e]);
                    w1[e] = ok ? ld_w(W1 + (size_t)ed * H + head) : 0.f;
                }
            }
            issue_loads_first();
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
#pragma unroll
                for (int i = 0; i < L::EPL; ++i) {
                    acc0[i] = fmaf(w0[e], x0[e][i], acc0[i]);
                    if constexpr (NOUT == 2) acc1[i] = fmaf(w1[e], x1[e][i], acc1[i]);
                }
            }
        }
    }
    if (it.slot < 0) {
        store_row<T, H, D>(Y0 + (size_t)it.row * L::C, lane, acc0);
        if constexpr (NOUT == 2) store_row<T, H, D>(Y1 + (size_t)it.row * L::C, lane, acc1);
    } else {
        store_row_ws<T, H, D>(ws0 + (size_t)it.slot * L::C, lane, acc0);
        if constexpr (NOUT == 2) store_row_ws<T, H, D>(ws1 + (size_t)it.slot * L::C, lane, acc1);
    }
}

// dB[eid[p], d] = sum_h dy[eid[p], h] * A[row, h, d]   (graphop_kernel.cu:79-94), lane = column d (D <= 64):
// the row's H head vectors stay in registers, each edge costs one 4*H-byte load, H FMAs and one D-element store.
template <typename T, int H, int D, int BATCH>
__global__ __launch_bounds__(BLOCK) void k_nme_dB_fast(bpt_plan P, const T *__restrict__ A, const T *__restrict__ dy, T *__restrict__ dB) {
    static_assert(D <= WAVE && H <= WAVE, "one lane per column");
    Item it;
    if (!fetch_item(P, it)) return;
    const int lane = threadIdx.x & 63;
    const int col = lane < D ? lane : 0;
    float a[H];
#pragma unroll
    for (int h = 0; h < H; ++h) a[h] = Elem<T>::ld(A + (size_t)it.row * H * D + h * D + col);
    for (int p0 = it.begin; p0 < it.end; p0 += WAVE) {
        const int cnt = min(WAVE, it.end - p0);
        const int my_eid = lane < cnt ? P.eid[p0 + lane] : 0;
        for (int b = 0; b < cnt; b += BATCH) {
            int ee[BATCH];
            float g[BATCH];
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                ee[e] = __builtin_amdgcn_readlane(my_eid, (b + e < cnt) ? b + e : b);
                g[e] = Elem<T>::ld(dy + (size_t)ee[e] * H + (lane < H ? lane : 0));     // lane h holds dy[e, h]
            }
            issue_loads_first();
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                float s = 0.f;
#pragma unroll
                for (int h = 0; h < H; ++h) s = fmaf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(g[e]), h)), a[h], s);
                if (b + e < cnt && lane < D) Elem<T>::st(dB + (size_t)ee[e] * D + lane, s);
            }
        }
    }
}

// Fused forward: per destination row, online softmax over the in-edges in batches of BATCH.
// Scores are kept in base-2 units (q is pre-multiplied by scale*log2(e)).
template <typename T, int H, int D, int BATCH>
__global__ __launch_bounds__(BLOCK) void k_attn_fwd(bpt_plan P, const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v,
                                                    T *__restrict__ o, float *__restrict__ lse, float *__restrict__ ws_acc,
                                                    float *__restrict__ ws_ml, float scale_log2e) {
    using L = Lay<T, H, D>;
    Item it;
    if (!fetch_item(P, it)) return;
    const int lane = threadIdx.x & 63, head = lane / L::LPH;
    float qv[L::EPL], acc[L::EPL];
    load_row<T, H, D>(q + (size_t)it.row * L::C, lane, qv);
#pragma unroll
    for (int i = 0; i < L::EPL; ++i) { qv[i] *= scale_log2e; acc[i] = 0.f; }
    float m = M_INIT_LOG2, l = 0.f;
    for (int p0 = it.begin; p0 < it.end; p0 += WAVE) {
        const int cnt = min(WAVE, it.end - p0);
        const int my_idx = lane < cnt ? P.idx[p0 + lane] : 0;
        for (int b = 0; b < cnt; b += BATCH) {
            float kv[BATCH][L::EPL], vv[BATCH][L::EPL], s[BATCH];
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                const int src = __builtin_amdgcn_readlane(my_idx, (b + e < cnt) ? b + e : b);
                load_row<T, H, D>(k + (size_t)src * L::C, lane, kv[e]);
                load_row<T, H, D>(v + (size_t)src * L::C, lane, vv[e]);
            }
            issue_loads_first();
            float mx = m;
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                const float t = head_sum<L::LPH>(dot_n<L::EPL>(qv, kv[e]));
                s[e] = (b + e < cnt) ? t : -INFINITY;
                mx = fmaxf(mx, s[e]);
            }
            const float alpha = __builtin_amdgcn_exp2f(m - mx);
            l *= alpha;
#pragma unroll
            for (int i = 0; i < L::EPL; ++i) acc[i] *= alpha;
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                const float pe = __builtin_amdgcn_exp2f(s[e] - mx);
                l += pe;
#pragma unroll
                for (int i = 0; i < L::EPL; ++i) acc[i] = fmaf(pe, vv[e][i], acc[i]);
            }
            m = mx;
        }
    }
    if (it.slot < 0) {
        const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
        for (int i = 0; i < L::EPL; ++i) acc[i] *= inv;
        store_row<T, H, D>(o + (size_t)it.row * L::C, lane, acc);
        if (lane % L::LPH == 0) lse[(size_t)it.row * H + head] = l > 0.f ? m + log2f(l) : 0.f;
    } else {
        store_row_ws<T, H, D>(ws_acc + (size_t)it.slot * L::C, lane, acc);
        if (lane % L::LPH == 0) {
            ws_ml[((size_t)it.slot * H + head) * 2] = m;
            ws_ml[((size_t)it.slot * H + head) * 2 + 1] = l;
        }
    }
}

// Combine the (m, l, acc) partials of each split row.  Grid (n_heavy, C / 64): one block per split row
// and 64-column strip; wave w folds slots w, w+4, ... with a running maximum (one pass, eight
// independent loads per step), then the four wave results are merged in wave order.
template <typename T, int H, int D>
__global__ __launch_bounds__(BLOCK) void k_attn_fwd_combine(const int32_t *__restrict__ heavy, const float *__restrict__ ws_acc,
                                                            const float *__restrict__ ws_ml, T *__restrict__ o, float *__restrict__ lse) {
    constexpr int C = H * D;
    static_assert(C % WAVE == 0, "strip width");
    __shared__ float pm[WAVES_PER_BLOCK][WAVE], pl[WAVES_PER_BLOCK][WAVE], pa[WAVES_PER_BLOCK][WAVE];
    const int row = heavy[3 * blockIdx.x], s0 = heavy[3 * blockIdx.x + 1], ns = heavy[3 * blockIdx.x + 2];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int j = blockIdx.y * WAVE + lane, head = j / D;
    const float *ml = ws_ml + ((size_t)s0 * H + head) * 2;      // slot stride 2*H
    const float *col = ws_acc + (size_t)s0 * C + j;              // slot stride C
    float M = M_INIT_LOG2, lsum = 0.f, a = 0.f;
    int kk = w;
    for (; kk + 7 * WAVES_PER_BLOCK < ns; kk += 8 * WAVES_PER_BLOCK) {
        float tm[8], tl[8], ta[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const size_t sl = (size_t)(kk + u * WAVES_PER_BLOCK);
            tm[u] = ml[sl * 2 * H];
            tl[u] = ml[sl * 2 * H + 1];
            ta[u] = col[sl * C];
        }
        float mx = M;
#pragma unroll
        for (int u = 0; u < 8; ++u) mx = fmaxf(mx, tm[u]);
        const float resc = __builtin_amdgcn_exp2f(M - mx);
        lsum *= resc;
        a *= resc;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float wgt = __builtin_amdgcn_exp2f(tm[u] - mx);
            lsum = fmaf(tl[u], wgt, lsum);
            a = fmaf(ta[u], wgt, a);
        }
        M = mx;
    }
    for (; kk < ns; kk += WAVES_PER_BLOCK) {
        const float tm = ml[(size_t)kk * 2 * H], mx = fmaxf(M, tm);
        const float resc = __builtin_amdgcn_exp2f(M - mx), wgt = __builtin_amdgcn_exp2f(tm - mx);
        lsum = fmaf(ml[(size_t)kk * 2 * H + 1], wgt, lsum * resc);
        a = fmaf(col[(size_t)kk * C], wgt, a * resc);
        M = mx;
    }
    pm[w][lane] = M; pl[w][lane] = lsum; pa[w][lane] = a;
    __syncthreads();
    if (w == 0) {
        float Mx = pm[0][lane];
#pragma unroll
        for (int i = 1; i < WAVES_PER_BLOCK; ++i) Mx = fmaxf(Mx, pm[i][lane]);
        float L = 0.f, A = 0.f;
#pragma unroll
        for (int i = 0; i < WAVES_PER_BLOCK; ++i) {
            const float wgt = __builtin_amdgcn_exp2f(pm[i][lane] - Mx);
            L = fmaf(pl[i][lane], wgt, L);
            A = fmaf(pa[i][lane], wgt, A);
        }
        Elem<T>::st(o + (size_t)row * C + j, L > 0.f ? A / L : 0.f);
        if (j % D == 0) lse[(size_t)row * H + head] = L > 0.f ? Mx + log2f(L) : 0.f;
    }
}

// Fused backward, destination side: recompute p from lse, delta = dO.O, ds = p*(dO.v - delta)*scale,
// dQ[row] = sum ds*k; p and ds go to (E, H) f32 buffers addressed by edge id for the source-side pass.
template <typename T, int H, int D, int BATCH>
__global__ __launch_bounds__(BLOCK) void k_attn_bwd_dst(bpt_plan P, const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v,
                                                        const T *__restrict__ o, const T *__restrict__ d_o, const float *__restrict__ lse,
                                                        T *__restrict__ dq, float *__restrict__ pbuf, float *__restrict__ dsbuf,
                                                        float *__restrict__ ws_dq, float scale, float scale_log2e) {
    using L = Lay<T, H, D>;
    Item it;
    if (!fetch_item(P, it)) return;
    const int lane = threadIdx.x & 63, head = lane / L::LPH;
    float qv[L::EPL], dov[L::EPL], dqa[L::EPL];
    float delta;
    {
        float ov[L::EPL];
        load_row<T, H, D>(o + (size_t)it.row * L::C, lane, ov);
        load_row<T, H, D>(d_o + (size_t)it.row * L::C, lane, dov);
        delta = head_sum<L::LPH>(dot_n<L::EPL>(dov, ov));
    }
    load_row<T, H, D>(q + (size_t)it.row * L::C, lane, qv);
#pragma unroll
    for (int i = 0; i < L::EPL; ++i) dqa[i] = 0.f;
    const float lse2 = lse[(size_t)it.row * H + head];
    for (int p0 = it.begin; p0 < it.end; p0 += WAVE) {
        const int cnt = min(WAVE, it.end - p0);
        const int my_idx = lane < cnt ? P.idx[p0 + lane] : 0;
        const int my_eid = lane < cnt ? P.eid[p0 + lane] : 0;
        for (int b = 0; b < cnt; b += BATCH) {
            float kv[BATCH][L::EPL], vv[BATCH][L::EPL];
            int ee[BATCH];
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                const int j = (b + e < cnt) ? b + e : b;
                const int src = __builtin_amdgcn_readlane(my_idx, j);
                ee[e] = __builtin_amdgcn_readlane(my_eid, j);
                load_row<T, H, D>(k + (size_t)src * L::C, lane, kv[e]);
                load_row<T, H, D>(v + (size_t)src * L::C, lane, vv[e]);
            }
            issue_loads_first();
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                const float s = head_sum<L::LPH>(dot_n<L::EPL>(qv, kv[e]));
                const float dp = head_sum<L::LPH>(dot_n<L::EPL>(dov, vv[e]));
                const bool ok = b + e < cnt;
                const float pe = ok ? __builtin_amdgcn_exp2f(fmaf(s, scale_log2e, -lse2)) : 0.f;
                const float ds = pe * (dp - delta) * scale;
#pragma unroll
                for (int i = 0; i < L::EPL; ++i) dqa[i] = fmaf(ds, kv[e][i], dqa[i]);
                if (ok && lane % L::LPH == 0) {
                    pbuf[(size_t)ee[e] * H + head] = pe;
                    dsbuf[(size_t)ee[e] * H + head] = ds;
                }
            }
        }
    }
    if (it.slot < 0) store_row<T, H, D>(dq + (size_t)it.row * L::C, lane, dqa);
    else store_row_ws<T, H, D>(ws_dq + (size_t)it.slot * L::C, lane, dqa);
}

// ------------------------------------------------------------------------------------------
// row-group kernels of the fused path: one wavefront (= one workgroup) owns a group of up to
// R (4 or 8) rows (or row segments) that share neighbours; every neighbour row of the group's union
// ("entry") is loaded once and used for all members that have an edge to it (entry mask).
//
// The kernels issue about one instruction per four cycles and SIMD, whatever its kind, so they are
// written for a low instruction count per (member, entry) pair: 32-bit byte offsets from uniform
// base pointers (no 64-bit vector address arithmetic), the entry list of up to GRP_CHUNK entries
// held one per lane and read with v_readlane, per-pair scratch addressed by entry * R + member
// (no popcounts), unmasked scratch stores.
// ------------------------------------------------------------------------------------------
// entries whose rows are loaded together (one where a row takes 16 registers per lane)
template <int EPL> constexpr int grp_batch() { return EPL >= 16 ? 1 : 2; }
constexpr int GRP_CHUNK = 56;                      // entries per lane-held list: a multiple of twice the batch, and
                                                   // GRP_CHUNK + 3 * batch <= 64 keeps every look-ahead index a lane id
constexpr int GRP_PAD_ENTRIES = 8;                 // the per-entry arrays are readable this far past the end

template <int R> struct GroupHead {
    int rows[R], slots[R], begin, end;
};

// wavefronts per SIMD the row-group kernels are compiled for: the members' state has to stay in registers
template <typename T, int EPL, int R> constexpr int grp_wpe() { return R * EPL <= 32 ? 3 : 2; }

// Workgroup b (one wavefront) runs on XCD b % 8 and takes head slice (b / 8) % HS of group number (b / 8) / HS of
// that XCD's chunk: HS wavefronts share a group, each handling H / HS of the heads of every row.  (Dispatching all
// first slices before the second ones, to halve the rows an XCD's L2 has to hold at a time, measured slower.)
template <int R, int HS> __device__ __forceinline__ int group_slice() { return (int)((blockIdx.x >> 3) % HS); }
template <int R, int HS> __device__ __forceinline__ bool fetch_group(const bpt_plan &P, GroupHead<R> &gh) {
    const int x = blockIdx.x & 7, w = (blockIdx.x >> 3) / HS;
    const int g = __builtin_amdgcn_readfirstlane(P.grp_chunks[x]) + w;
    if (g >= __builtin_amdgcn_readfirstlane(P.grp_chunks[x + 1])) return false;
    const int lane = threadIdx.x;
    const int mem = P.grp_members[(size_t)g * (2 * R) + (lane & (2 * R - 1))];
    const int ptr = P.grp_ptr[g + (lane & 1)];
#pragma unroll
    for (int m = 0; m < R; ++m) {
        gh.rows[m] = __builtin_amdgcn_readlane(mem, 2 * m);
        gh.slots[m] = __builtin_amdgcn_readlane(mem, 2 * m + 1);
    }
    gh.begin = __builtin_amdgcn_readlane(ptr, 0);
    gh.end = __builtin_amdgcn_readlane(ptr, 1);
    return true;
}

// Row `row` of a node tensor (PITCH elements per row; the layout may cover a slice of the row's heads) through a
// uniform base pointer, a uniform 32-bit row offset and this lane's constant byte offset `loff` (global_load with scalar base + 32-bit vector offset + immediate).
template <typename T, int H, int D, int PITCH = Lay<T, H, D>::C>
__device__ __forceinline__ void load_row32(const T *__restrict__ base, uint32_t row, uint32_t loff, float (&out)[Lay<T, H, D>::EPL]) {
    using L = Lay<T, H, D>;
    const char *p = reinterpret_cast<const char *>(base) + (size_t)(row * (uint32_t)(PITCH * sizeof(T)));
#pragma unroll
    for (int i = 0; i < L::NV; ++i) {
        const char *pi = p + (size_t)(loff + (uint32_t)(i * L::LPH * 16));
        if constexpr (sizeof(T) == 4) {
            const float4 v = *reinterpret_cast<const float4 *>(pi);
            out[4 * i] = v.x; out[4 * i + 1] = v.y; out[4 * i + 2] = v.z; out[4 * i + 3] = v.w;
        } else {
            const uint4 v = *reinterpret_cast<const uint4 *>(pi);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                out[8 * i + 2 * c] = __uint_as_float(w[c] << 16);
                out[8 * i + 2 * c + 1] = __uint_as_float(w[c] & 0xffff0000u);
            }
        }
    }
}

// The same row as loaded, not yet converted: the software pipeline keeps rows in flight in this form, and
// converts them where they are used, after the wait (bf16 to f32 costs a shift or a mask per element).
template <typename T, int H, int D> struct RawRow { uint32_t w[Lay<T, H, D>::EPL * sizeof(T) / 4]; };

template <typename T, int H, int D, int PITCH = Lay<T, H, D>::C>
__device__ __forceinline__ void load_row32_raw(const T *__restrict__ base, uint32_t row, uint32_t loff, RawRow<T, H, D> &out) {
    using L = Lay<T, H, D>;
    const char *p = reinterpret_cast<const char *>(base) + (size_t)(row * (uint32_t)(PITCH * sizeof(T)));
#pragma unroll
    for (int i = 0; i < L::NV; ++i) {
        const uint4 v = *reinterpret_cast<const uint4 *>(p + (size_t)(loff + (uint32_t)(i * L::LPH * 16)));
        out.w[4 * i] = v.x; out.w[4 * i + 1] = v.y; out.w[4 * i + 2] = v.z; out.w[4 * i + 3] = v.w;
    }
}

template <typename T, int H, int D>
__device__ __forceinline__ void unpack_row(const RawRow<T, H, D> &in, float (&out)[Lay<T, H, D>::EPL]) {
    using L = Lay<T, H, D>;
    if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int i = 0; i < L::EPL; ++i) out[i] = __uint_as_float(in.w[i]);
    } else {
#pragma unroll
        for (int j = 0; j < L::EPL / 2; ++j) {
            out[2 * j] = __uint_as_float(in.w[j] << 16);
            out[2 * j + 1] = __uint_as_float(in.w[j] & 0xffff0000u);
        }
    }
}

// A wavefront-private row in LDS, lane-major (float4 c of lane l at slot c * 64 + l: conflict free).
template <int EPL> __device__ __forceinline__ void lds_put_row(float4 *slot, int lane, const float (&r)[EPL]) {
#pragma unroll
    for (int c = 0; c < EPL / 4; ++c) slot[c * WAVE + lane] = make_float4(r[4 * c], r[4 * c + 1], r[4 * c + 2], r[4 * c + 3]);
}
template <int EPL> __device__ __forceinline__ void lds_get_row(const float4 *slot, int lane, float (&r)[EPL]) {
#pragma unroll
    for (int c = 0; c < EPL / 4; ++c) {
        const float4 t = slot[c * WAVE + lane];
        r[4 * c] = t.x; r[4 * c + 1] = t.y; r[4 * c + 2] = t.z; r[4 * c + 3] = t.w;
    }
}

// Dropout on the attention probabilities (modules/attention.py:73): the keep / drop decision of (pair n, head h) is
// a hash of n * H + h and the call's seed, so that forward and backward agree without storing a mask.  n is the
// pair's number in the destination-side groups (entry's first pair + rank of the member in the entry's mask).
// Returns the multiplier 1 / (1 - p) or 0.
__device__ __forceinline__ float dropout_keep(uint32_t key, uint32_t seed, uint32_t thr, float inv_keep) {
    uint32_t x = key ^ seed;
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x >= thr ? inv_keep : 0.f;
}

// two independent head sums, interleaved so that one hides the other's DPP wait states
template <int LPH> __device__ __forceinline__ void head_sum2(float &a, float &b) {
    if constexpr (LPH >= 2) { a += dpp_mov<0xB1>(a); b += dpp_mov<0xB1>(b); }
    if constexpr (LPH >= 4) { a += dpp_mov<0x4E>(a); b += dpp_mov<0x4E>(b); }
    if constexpr (LPH >= 8) { a += dpp_mov<0x141>(a); b += dpp_mov<0x141>(b); }
    if constexpr (LPH >= 16) { a += dpp_mov<0x140>(a); b += dpp_mov<0x140>(b); }
    if constexpr (LPH >= 32) { a += __shfl_xor(a, 16); b += __shfl_xor(b, 16); }
    if constexpr (LPH >= 64) { a += __shfl_xor(a, 32); b += __shfl_xor(b, 32); }
}

// max of three finite-or-minus-infinity values (no NaN canonicalisation of the operands)
__device__ __forceinline__ float max3f(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Forward: online softmax in base 2 over the group's entries, two entries per step.  The members' q rows
// (pre-scaled) live in LDS and are re-read for every use, which keeps the kernel at three wavefronts per SIMD.
template <typename T, int H, int D, int R, int HS, bool DROP, bool BIAS>
__global__ __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(grp_wpe<T, Lay<T, H / HS, D>::EPL, R>()))) void k_attn_fwd_grp(
    bpt_plan P, const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v, T *__restrict__ o,
    float *__restrict__ lse, float *__restrict__ ws_acc, float *__restrict__ ws_ml, float scale_log2e, uint32_t drop_thr,
    uint32_t drop_seed, float drop_inv, const float *__restrict__ bias) {
    constexpr int HL = H / HS, CF = H * D;                  // heads of this wavefront's slice; elements of a full row
    using L = Lay<T, HL, D>;
    constexpr int EPL = L::EPL, NQ = R / 4, GRP_BATCH = BIAS ? 1 : grp_batch<L::EPL>()   /* the score term's registers take the place of a second entry */;
    static_assert(H % HS == 0 && R % 4 == 0 && L::LPH >= 4, "members are handled in quads inside the lanes of one head");
    GroupHead<R> gh;
    if (!fetch_group<R, HS>(P, gh)) return;
    const int slice = group_slice<R, HS>(), coff = slice * HL * D;
    const int lane = threadIdx.x, head = slice * HL + lane / L::LPH;
    const uint32_t loff = (uint32_t)((coff + L::off(lane, 0)) * sizeof(T));
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
    struct Batch {
        RawRow<T, HL, D> kr[GRP_BATCH], vr[GRP_BATCH];
        int mk[GRP_BATCH], pz[GRP_BATCH];
        float bz[GRP_BATCH][BIAS ? R / 4 : 1];      // score term of (entry, member 4c + lane % 4), this lane's head
    };
    struct Rows {
        float kv[GRP_BATCH][EPL], vv[GRP_BATCH][EPL];
        int mk[GRP_BATCH], pz[GRP_BATCH];
    };
    const int4 *eids4 = reinterpret_cast<const int4 *>(P.grp_eids);
    __shared__ float4 q_lds[R * (EPL / 4) * WAVE];
    float acc[R][EPL], mrun[R], lrun[R];
#pragma unroll
    for (int m = 0; m < R; ++m) {
        float qr[EPL];
        load_row32<T, HL, D, CF>(q, (uint32_t)max(gh.rows[m], 0), loff, qr);
        mrun[m] = M_INIT_LOG2;
        lrun[m] = 0.f;
#pragma unroll
        for (int i = 0; i < EPL; ++i) { qr[i] *= scale_log2e; acc[m][i] = 0.f; }
        lds_put_row<EPL>(q_lds + m * (EPL / 4) * WAVE, lane, qr);
    }
    for (int p0 = gh.begin; p0 < gh.end; p0 += GRP_CHUNK) {
        const int cnt = min(GRP_CHUNK, gh.end - p0);
        // lanes past the end repeat the last entry with an empty mask
        int4 ent = entries[p0 + min(lane, cnt - 1)];
        ent.y = lane < cnt ? ent.y : 0;
        // edge ids of the lane's entry, four members per vector (the list is padded like the entries)
        int4 xe[R / 4];
        if constexpr (BIAS || DROP) {
#pragma unroll
            for (int c = 0; c < R / 4; ++c) xe[c] = eids4[(size_t)(p0 + min(lane, cnt - 1)) * (R / 4) + c];
        }
        auto load_batch = [&](Batch &B, int b) {
#pragma unroll
            for (int e = 0; e < GRP_BATCH; ++e) {
                const uint32_t src = (uint32_t)__builtin_amdgcn_readlane(ent.x, b + e);
                B.mk[e] = __builtin_amdgcn_readlane(ent.y, b + e);
                B.pz[e] = DROP ? b + e : 0;                  // position of the entry in the chunk: the lane that holds its edge ids
                if constexpr (BIAS) {
#pragma unroll
                    for (int c = 0; c < R / 4; ++c) {
                        // lane l fetches the term of member 4c + l % 4; the quad's lanes hand it round when it is used
                        const uint32_t e0 = (uint32_t)__builtin_amdgcn_readlane(xe[c].x, b + e), e1 = (uint32_t)__builtin_amdgcn_readlane(xe[c].y, b + e);
                        const uint32_t e2 = (uint32_t)__builtin_amdgcn_readlane(xe[c].z, b + e), e3 = (uint32_t)__builtin_amdgcn_readlane(xe[c].w, b + e);
                        const uint32_t el = (lane & 3) == 0 ? e0 : (lane & 3) == 1 ? e1 : (lane & 3) == 2 ? e2 : e3;
                        B.bz[e][c] = bias[(size_t)(el * (uint32_t)H) + head];
                    }
                }
                load_row32_raw<T, HL, D, CF>(k, src, loff, B.kr[e]);
                load_row32_raw<T, HL, D, CF>(v, src, loff, B.vr[e]);
            }
        };
        // multiplier of the pair (member m, entry at position pz of the chunk): 1 without dropout; keyed by the edge id
        auto keep = [&](int m, int mk, int pz) -> float {
            if constexpr (!DROP) return 1.f;
            const int4 &x = xe[m / 4];
            const int held = (m & 3) == 0 ? x.x : (m & 3) == 1 ? x.y : (m & 3) == 2 ? x.z : x.w;
            const uint32_t edge = (uint32_t)__builtin_amdgcn_readlane(held, pz);
            return dropout_keep(edge * (uint32_t)H + (uint32_t)head, drop_seed, drop_thr, drop_inv);
        };
        auto one = [&](int m, const float (&kr)[EPL], const float (&vr)[EPL], int mk, int pz, float bz) {
            float qm[EPL];
            lds_get_row<EPL>(q_lds + m * (EPL / 4) * WAVE, lane, qm);
            const float s = head_sum<L::LPH>(dot_n<EPL>(qm, kr)) + bz;
            const float mx = fmaxf(mrun[m], s);
            const float al = __builtin_amdgcn_exp2f(mrun[m] - mx), pe = __builtin_amdgcn_exp2f(s - mx);
            lrun[m] = fmaf(lrun[m], al, pe);                       // the softmax denominator ignores dropout
            const float pk = pe * keep(m, mk, pz);
#pragma unroll
            for (int i = 0; i < EPL; ++i) acc[m][i] = fmaf(pk, vr[i], acc[m][i] * al);
            mrun[m] = mx;
        };
        auto compute = [&](const Batch &raw) {
            Rows B;
#pragma unroll
            for (int e = 0; e < GRP_BATCH; ++e) {
                unpack_row<T, HL, D>(raw.kr[e], B.kv[e]);
                unpack_row<T, HL, D>(raw.vr[e], B.vv[e]);
                B.mk[e] = raw.mk[e];
                B.pz[e] = raw.pz[e];
            }
#pragma unroll
            for (int m = 0; m < R; ++m) {
                const bool h0 = (B.mk[0] >> m) & 1, h1 = (B.mk[GRP_BATCH - 1] >> m) & 1;
                // the score term in the units of the scaled scores
                const float z0 = BIAS ? quad_bcast(raw.bz[0][BIAS ? m / 4 : 0], m) * scale_log2e : 0.f;
                const float z1 = BIAS ? quad_bcast(raw.bz[GRP_BATCH - 1][BIAS ? m / 4 : 0], m) * scale_log2e : 0.f;
                if constexpr (GRP_BATCH == 1) {
                    if (h0) one(m, B.kv[0], B.vv[0], B.mk[0], B.pz[0], z0);
                } else if (h0 && h1) {
                    float qm[EPL];
                    lds_get_row<EPL>(q_lds + m * (EPL / 4) * WAVE, lane, qm);
                    float s0 = dot_n<EPL>(qm, B.kv[0]), s1 = dot_n<EPL>(qm, B.kv[GRP_BATCH - 1]);
                    head_sum2<L::LPH>(s0, s1);
                    s0 += z0;
                    s1 += z1;
                    const float mx = max3f(mrun[m], s0, s1);
                    const float al = __builtin_amdgcn_exp2f(mrun[m] - mx);
                    const float p0e = __builtin_amdgcn_exp2f(s0 - mx), p1e = __builtin_amdgcn_exp2f(s1 - mx);
                    lrun[m] = fmaf(lrun[m], al, p0e + p1e);
                    const float k0 = p0e * keep(m, B.mk[0], B.pz[0]), k1 = p1e * keep(m, B.mk[GRP_BATCH - 1], B.pz[GRP_BATCH - 1]);
#pragma unroll
                    for (int i = 0; i < EPL; ++i) acc[m][i] = fmaf(k1, B.vv[GRP_BATCH - 1][i], fmaf(k0, B.vv[0][i], acc[m][i] * al));
                    mrun[m] = mx;
                } else if (h0) {
                    one(m, B.kv[0], B.vv[0], B.mk[0], B.pz[0], z0);
                } else if (h1) {
                    one(m, B.kv[GRP_BATCH - 1], B.vv[GRP_BATCH - 1], B.mk[GRP_BATCH - 1], B.pz[GRP_BATCH - 1], z1);
                }
            }
        };
        // two-stage software pipeline: the rows of the next batch are in flight while one is used.  The loads
        // are unconditional (a branch around them would make the compiler drain the load queue at the join);
        // look-ahead past the end re-reads the chunk's last entry with an empty mask.
        Batch A, B;
        load_batch(A, 0);
        for (int b = 0; b < cnt; b += 2 * GRP_BATCH) {
            load_batch(B, b + GRP_BATCH);
            issue_loads_first();
            compute(A);
            issue_loads_first();
            load_batch(A, b + 2 * GRP_BATCH);
            issue_loads_first();
            compute(B);
            issue_loads_first();
        }
    }
#pragma unroll
    for (int m = 0; m < R; ++m) {
        if (gh.rows[m] < 0) continue;
        if (gh.slots[m] < 0) {
            const float inv = lrun[m] > 0.f ? 1.f / lrun[m] : 0.f;
#pragma unroll
            for (int i = 0; i < EPL; ++i) acc[m][i] *= inv;
            store_row<T, HL, D>(o + (size_t)gh.rows[m] * CF + coff, lane, acc[m]);
            if (lane % L::LPH == 0) lse[(size_t)gh.rows[m] * H + head] = lrun[m] > 0.f ? mrun[m] + log2f(lrun[m]) : 0.f;
        } else {
            store_row_ws<T, HL, D>(ws_acc + (size_t)gh.slots[m] * CF + coff, lane, acc[m]);
            if (lane % L::LPH == 0) {
                ws_ml[((size_t)gh.slots[m] * H + head) * 2] = mrun[m];
                ws_ml[((size_t)gh.slots[m] * H + head) * 2 + 1] = lrun[m];
            }
        }
    }
}

// ---- matrix-core forward for groups of 8 rows -------------------------------------------------------------------
// v_mfma_f32_4x4x1 works on 16 blocks of 4 lanes: D_b[i][j] += A_b[i] * B_b[j] with A_b[i] taken from lane 4b+i,
// B_b[j] from lane 4b+j and D_b[i][j] held in register i of lane 4b+j.  Block b owns the 4 * EPL columns that its
// four lanes hold in the row layout (all of one head).
//   scores   S^T = K Q^T: lane 4b+i supplies column c of the row of entry i (of a batch of four), lane 4b+j column c
//            of the q row of member j; after one instruction per column of the block and a sum over the blocks of a
//            head, register i of lane 4b+j holds (entry i, member j).  The rows reach this "one row per lane of a
//            block" arrangement through LDS: written as loaded, read back by (row, block).
//   output   O += P V: A = the lane's own probability (member j = lane % 4, entry e), B = register r of the V row
//            of entry e in the row layout; D is the accumulator of (member i, this lane's r-th column).
// A wavefront issues at most one instruction every eight cycles, so the time of a group is its instruction count:
// the matrix-core form needs about a third of the instructions per (entry, member) of the vector form.
// The exponent reference of a (member, head) is raised only when a score exceeds it by more than MFMA_TAU (base-2
// units), so the accumulators are rescaled rarely; probabilities stay below 2^MFMA_TAU times the usual ones, and
// o and lse come out the same up to rounding.
constexpr float MFMA_TAU = 8.f;
constexpr int MFMA_NB = 4;                          // entries per batch = rows of the A operand

// sum over the blocks (quads of lanes) that hold one head; the result is in all of them.  Every lane has to take
// part: a lane switched off by a branch would hand zero to its partners.
template <int BPH> __device__ __forceinline__ float block_sum(float x) {
    if constexpr (BPH >= 2) x += dpp_mov<0x1B>(dpp_mov<0x141>(x));     // lane ^ 4: row_half_mirror, then quad_perm [3,2,1,0]
    if constexpr (BPH >= 4) x += dpp_mov<0x141>(dpp_mov<0x140>(x));    // lane ^ 8: row_mirror, then row_half_mirror
    return x;
}

__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

typedef short bf16x4_t __attribute__((ext_vector_type(4)));
// two registers of bfloat16 pairs as the four-element operand of the bfloat16 matrix instructions
__device__ __forceinline__ bf16x4_t as_bf16x4(uint32_t a, uint32_t b) {
    const uint2 u = make_uint2(a, b);
    return __builtin_bit_cast(bf16x4_t, u);
}

// 16-byte vector as VE floats
template <typename T> __device__ __forceinline__ void unpack_vec(const uint4 &w, float *out) {
    const uint32_t x[4] = {w.x, w.y, w.z, w.w};
    if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int c = 0; c < 4; ++c) out[c] = __uint_as_float(x[c]);
    } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            out[2 * c] = __uint_as_float(x[c] << 16);
            out[2 * c + 1] = __uint_as_float(x[c] & 0xffff0000u);
        }
    }
}

// Two wavefronts per group of 8 rows: wavefront w owns members 4 w .. 4 w + 3 (one quad: the B operand of the
// score products), both share the staged rows.  Each wavefront loads and stages half of a batch.  With two staging
// buffers one workgroup barrier per batch orders the writes of batch b + 1 after the reads of batch b - 1; where V
// has a single buffer (W3 below) a second barrier separates the reads of batch b from the writes of batch b + 1.
template <typename T, int H, int D, int HS, bool DROP, bool BIAS>
__global__ __launch_bounds__(2 * WAVE) __attribute__((amdgpu_waves_per_eu(sizeof(T) == 4 && !BIAS && !DROP ? 3 : 2))) void k_attn_fwd_mfma(
    bpt_plan P, const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v, T *__restrict__ o,
    float *__restrict__ lse, float *__restrict__ ws_acc, float *__restrict__ ws_ml, float scale_log2e, uint32_t drop_thr,
    uint32_t drop_seed, float drop_inv, const float *__restrict__ bias) {
    constexpr int R = 8, NB = MFMA_NB, HL = H / HS, CF = H * D, NE = NB / 2;      // NE: entries a wavefront loads per batch
    // float32: one V area instead of two (a second barrier per batch) and no read-ahead registers, which fits three
    // wavefronts per SIMD and six workgroups per CU (measured 5 % faster); bfloat16 rows are half as large
    constexpr bool W3 = sizeof(T) == 4 && !BIAS && !DROP;  // (the edge ids and score terms would not fit)
    using L = Lay<T, HL, D>;
    constexpr int EPL = L::EPL, NV = L::NV, VE = L::VE, BPH = L::LPH / 4, CB = 4 * EPL, PITCH = NV * WAVE + 1;
    static_assert(EPL % VE == 0 && EPL <= 8 && (BPH == 1 || BPH == 2 || BPH == 4), "shape not covered by the matrix-core kernels");
    const int lane = threadIdx.x & (WAVE - 1), wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // the group of this workgroup (as fetch_group, for workgroups of two wavefronts)
    int rows[4], slots[4], g_begin, g_end;
    {
        const int x = blockIdx.x & 7, w = (blockIdx.x >> 3) / HS;
        const int g = __builtin_amdgcn_readfirstlane(P.grp_chunks[x]) + w;
        if (g >= __builtin_amdgcn_readfirstlane(P.grp_chunks[x + 1])) return;
        const int mem = P.grp_members[(size_t)g * (2 * R) + (lane & (2 * R - 1))];
        const int ptr = P.grp_ptr[g + (lane & 1)];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            rows[i] = __builtin_amdgcn_readlane(mem, 8 * wv + 2 * i);
            slots[i] = __builtin_amdgcn_readlane(mem, 8 * wv + 2 * i + 1);
        }
        g_begin = __builtin_amdgcn_readlane(ptr, 0);
        g_end = __builtin_amdgcn_readlane(ptr, 1);
    }
    const int slice = (int)((blockIdx.x >> 3) % HS), coff = slice * HL * D;
    const int head = slice * HL + lane / L::LPH, j = lane & 3, blk = lane >> 2;
    const uint32_t loff = (uint32_t)((coff + L::off(lane, 0)) * sizeof(T));
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
    const int eid_last = (int)P.n_grp_entries + GRP_PAD_ENTRIES - 1;      // last entry of grp_eids, padding included
    __shared__ uint4 kst[2][NB * PITCH];              // rows as loaded, one spare vector per row against bank conflicts
    __shared__ uint4 vst[W3 ? 1 : 2][NB * NV * WAVE];
    // q row of member 4 wv + j, the columns of this lane's block: float32 pre-scaled, or (bfloat16) as loaded, the
    // scale then being applied to the scores
    constexpr bool B16 = sizeof(T) == 2;
    float qb[B16 ? 1 : CB];
    uint4 qraw[B16 ? NV * 4 : 1];
    {
        // wavefront 0 stages its q rows through the K area, wavefront 1 through the V area
        uint4 *qst = wv == 0 ? &kst[0][0] : &vst[0][0];
        constexpr int QP = NV * WAVE;                  // unpadded: four rows fill either area exactly
        RawRow<T, HL, D> qr[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) load_row32_raw<T, HL, D, CF>(q, (uint32_t)max(rows[i], 0), loff, qr[i]);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int c = 0; c < NV; ++c) qst[i * QP + c * WAVE + lane] = make_uint4(qr[i].w[4 * c], qr[i].w[4 * c + 1], qr[i].w[4 * c + 2], qr[i].w[4 * c + 3]);
        wave_lds_fence();
        if constexpr (B16) {
#pragma unroll
            for (int t = 0; t < NV * 4; ++t) qraw[t] = qst[j * QP + (t / 4) * WAVE + 4 * blk + (t % 4)];
        } else {
#pragma unroll
            for (int t = 0; t < NV * 4; ++t) unpack_vec<T>(qst[j * QP + (t / 4) * WAVE + 4 * blk + (t % 4)], &qb[t * VE]);
#pragma unroll
            for (int c = 0; c < CB; ++c) qb[c] *= scale_log2e;
        }
    }
    floatx4 acc[EPL];                                  // [row register r][member 4 wv + i]
    float mref = M_INIT_LOG2, lrun = 0.f;
#pragma unroll
    for (int r = 0; r < EPL; ++r) acc[r] = floatx4{0.f, 0.f, 0.f, 0.f};
    struct Raw {
        RawRow<T, HL, D> kr[NE], vr[NE];
        int xe[(BIAS || DROP) ? NB : 1];               // edge ids of this lane's member with the batch's entries
    };
    for (int p0 = g_begin; p0 < g_end; p0 += GRP_CHUNK) {
        const int cnt = min(GRP_CHUNK, g_end - p0);
        int4 ent = entries[p0 + min(lane, cnt - 1)];    // lanes past the end repeat the last entry with an empty mask
        ent.y = lane < cnt ? ent.y : 0;
        auto load_half = [&](Raw &B, int b) {          // this wavefront's entries of batch b
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                const uint32_t src = (uint32_t)__builtin_amdgcn_readlane(ent.x, b + NE * wv + e);
                load_row32_raw<T, HL, D, CF>(k, src, loff, B.kr[e]);
                load_row32_raw<T, HL, D, CF>(v, src, loff, B.vr[e]);
            }
            if constexpr (BIAS || DROP) {
                // the look-ahead reaches up to 2 * NB + NB - 1 entries past the group's last one: clamped to the last
                // entry of the list's padding (all values there are the spare edge id)
#pragma unroll
                for (int e = 0; e < NB; ++e) B.xe[e] = P.grp_eids[(size_t)min(p0 + b + e, eid_last) * R + 4 * wv + j];
            }
        };
        // the score terms of a batch are fetched one batch ahead, with the edge ids that came in the batch before
        float bz[NB];
        int xd[NB];                                    // edge ids of the batch in use (dropout is keyed by them)
        auto load_bias = [&](const Raw &B) {
            if constexpr (BIAS) {
#pragma unroll
                for (int e = 0; e < NB; ++e) bz[e] = bias[(size_t)((uint32_t)B.xe[e] * (uint32_t)H) + head];
            }
            if constexpr (DROP) {
#pragma unroll
                for (int e = 0; e < NB; ++e) xd[e] = B.xe[e];
            }
        };
        auto stage_half = [&](const Raw &B, int buf) {
#pragma unroll
            for (int e = 0; e < NE; ++e)
#pragma unroll
                for (int c = 0; c < NV; ++c) {
                    kst[buf][(NE * wv + e) * PITCH + c * WAVE + lane] = make_uint4(B.kr[e].w[4 * c], B.kr[e].w[4 * c + 1], B.kr[e].w[4 * c + 2], B.kr[e].w[4 * c + 3]);
                    vst[W3 ? 0 : buf][((NE * wv + e) * NV + c) * WAVE + lane] = make_uint4(B.vr[e].w[4 * c], B.vr[e].w[4 * c + 1], B.vr[e].w[4 * c + 2], B.vr[e].w[4 * c + 3]);
                }
        };
        Raw raw;
        load_half(raw, 0);
        __syncthreads();                               // the staging area is free (q rows, the previous chunk's last batch)
        stage_half(raw, 0);
        load_bias(raw);
        load_half(raw, NB);
        __syncthreads();
        for (int b = 0, buf = 0; b < cnt; b += NB, buf ^= 1) {
            int mk[NB];
#pragma unroll
            for (int e = 0; e < NB; ++e) mk[e] = __builtin_amdgcn_readlane(ent.y, b + e);
            // all LDS reads of the batch go out first: the K rows of this lane's entry by block, the V rows as loaded
            uint4 kv[NV * 4], vv[NB][NV];
#pragma unroll
            for (int t = 0; t < NV * 4; ++t) kv[t] = kst[buf][j * PITCH + (t / 4) * WAVE + 4 * blk + (t % 4)];
#pragma unroll
            for (int e = 0; e < NB; ++e)
#pragma unroll
                for (int c = 0; c < NV; ++c) vv[e][c] = vst[W3 ? 0 : buf][(e * NV + c) * WAVE + lane];
            if constexpr (!W3) issue_loads_first();
            // scores: register e of lane 4 blk + j = (entry e, member 4 wv + j), head of the block
            floatx4 st[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) st[c] = floatx4{0.f, 0.f, 0.f, 0.f};
            if constexpr (B16) {
                // four columns per instruction, operands as loaded (v_mfma_f32_4x4x4 on bfloat16)
#pragma unroll
                for (int t = 0; t < NV * 4; ++t) {
                    st[0] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(as_bf16x4(kv[t].x, kv[t].y), as_bf16x4(qraw[t].x, qraw[t].y), st[0], 0, 0, 0);
                    st[1] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(as_bf16x4(kv[t].z, kv[t].w), as_bf16x4(qraw[t].z, qraw[t].w), st[1], 0, 0, 0);
                }
            } else {
#pragma unroll
                for (int t = 0; t < NV * 4; ++t) {
                    float kf[VE];
                    unpack_vec<T>(kv[t], kf);
#pragma unroll
                    for (int c = 0; c < VE; ++c) st[c & 3] = __builtin_amdgcn_mfma_f32_4x4x1f32(kf[c], qb[t * VE + c], st[c & 3], 0, 0, 0);
                }
            }
            float sc[NB];
#pragma unroll
            for (int e = 0; e < NB; ++e) sc[e] = block_sum<BPH>((st[0][e] + st[1][e]) + (st[2][e] + st[3][e])) * (B16 ? scale_log2e : 1.f);
#pragma unroll
            for (int e = 0; e < NB; ++e) sc[e] = ((mk[e] >> (4 * wv + j)) & 1) ? (BIAS ? fmaf(bz[e], scale_log2e, sc[e]) : sc[e]) : -INFINITY;
            const float mb = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
            if (__builtin_amdgcn_ballot_w64(mb > mref + MFMA_TAU) != 0) {
                const float mn = fmaxf(mref, mb);
                const float al = __builtin_amdgcn_exp2f(mref - mn);
                mref = mn;
                lrun *= al;
                const float a0 = quad_lane<0>(al), a1 = quad_lane<1>(al), a2 = quad_lane<2>(al), a3 = quad_lane<3>(al);
#pragma unroll
                for (int r = 0; r < EPL; ++r) {
                    acc[r][0] *= a0; acc[r][1] *= a1; acc[r][2] *= a2; acc[r][3] *= a3;
                }
            }
            float pk[NB];
#pragma unroll
            for (int e = 0; e < NB; ++e) {
                const float pe = __builtin_amdgcn_exp2f(sc[e] - mref);
                lrun += pe;                                          // the softmax denominator ignores dropout
                if constexpr (DROP) {
                    pk[e] = pe * dropout_keep((uint32_t)xd[e] * (uint32_t)H + (uint32_t)head, drop_seed, drop_thr, drop_inv);
                } else {
                    pk[e] = pe;
                }
            }
            if constexpr (B16) {
                // A = the lane's four probabilities (one per entry of the batch) rounded to bfloat16; B = column r of
                // the four V rows, gathered from the rows' registers by byte permutes
                const uint32_t p01 = (uint32_t)f32_to_bf16(pk[0]) | ((uint32_t)f32_to_bf16(pk[1]) << 16);
                const uint32_t p23 = (uint32_t)f32_to_bf16(pk[2]) | ((uint32_t)f32_to_bf16(pk[3]) << 16);
                static_assert(NV == 1 && NB == 4, "one 16-byte vector per row and lane");
                const uint32_t v0[4] = {vv[0][0].x, vv[0][0].y, vv[0][0].z, vv[0][0].w}, v1[4] = {vv[1][0].x, vv[1][0].y, vv[1][0].z, vv[1][0].w};
                const uint32_t v2[4] = {vv[2][0].x, vv[2][0].y, vv[2][0].z, vv[2][0].w}, v3[4] = {vv[3][0].x, vv[3][0].y, vv[3][0].z, vv[3][0].w};
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const uint32_t lo01 = __builtin_amdgcn_perm(v1[c], v0[c], 0x05040100u), lo23 = __builtin_amdgcn_perm(v3[c], v2[c], 0x05040100u);
                    const uint32_t hi01 = __builtin_amdgcn_perm(v1[c], v0[c], 0x07060302u), hi23 = __builtin_amdgcn_perm(v3[c], v2[c], 0x07060302u);
                    acc[2 * c] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(as_bf16x4(p01, p23), as_bf16x4(lo01, lo23), acc[2 * c], 0, 0, 0);
                    acc[2 * c + 1] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(as_bf16x4(p01, p23), as_bf16x4(hi01, hi23), acc[2 * c + 1], 0, 0, 0);
                }
            } else {
#pragma unroll
                for (int e = 0; e < NB; ++e) {
                    float vf[EPL];
#pragma unroll
                    for (int c = 0; c < NV; ++c) unpack_vec<T>(vv[e][c], &vf[c * VE]);
#pragma unroll
                    for (int r = 0; r < EPL; ++r) acc[r] = __builtin_amdgcn_mfma_f32_4x4x1f32(pk[e], vf[r], acc[r], 0, 0, 0);
                }
            }
            // the other buffer was last read one batch ago, before the previous barrier
            if constexpr (W3) __syncthreads();
            stage_half(raw, buf ^ 1);
            load_bias(raw);
            load_half(raw, b + 2 * NB);                // look-ahead (past the end: the last entry again, unused)
            __syncthreads();
        }
    }
    const float ls[4] = {quad_lane<0>(lrun), quad_lane<1>(lrun), quad_lane<2>(lrun), quad_lane<3>(lrun)};
    const float ms[4] = {quad_lane<0>(mref), quad_lane<1>(mref), quad_lane<2>(mref), quad_lane<3>(mref)};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (rows[i] < 0) continue;
        float out[EPL];
        if (slots[i] < 0) {
            const float inv = ls[i] > 0.f ? 1.f / ls[i] : 0.f;
#pragma unroll
            for (int r = 0; r < EPL; ++r) out[r] = acc[r][i] * inv;
            store_row<T, HL, D>(o + (size_t)rows[i] * CF + coff, lane, out);
            if (lane % L::LPH == 0) lse[(size_t)rows[i] * H + head] = ls[i] > 0.f ? ms[i] + log2f(ls[i]) : 0.f;
        } else {
#pragma unroll
            for (int r = 0; r < EPL; ++r) out[r] = acc[r][i];
            store_row_ws<T, HL, D>(ws_acc + (size_t)slots[i] * CF + coff, lane, out);
            if (lane % L::LPH == 0) {
                ws_ml[((size_t)slots[i] * H + head) * 2] = ms[i];
                ws_ml[((size_t)slots[i] * H + head) * 2 + 1] = ls[i];
            }
        }
    }
}

// ---- dense tiles: groups of 16 rows, one wavefront per head ---------------------------------------------------------
// A group of TILE_R = 16 rows (or row segments) and its entries (the union of the members' neighbours, each with a
// 16-bit member mask) is walked in blocks of 16 entries as a dense 16 x 16 problem on the matrix cores: the pairs a
// block does not have are computed and masked.  Adjacent rows of a BPT graph share most neighbours (35 % of a block's
// pairs exist at L = 8192, k = 4), and a dense block costs 4 cycles per pair and head in float32 against 25-35 issue
// slots of the gather form.  Workgroup = H wavefronts, wavefront = one head, so every lane keeps 1/64 of a
// 16 x 64 tile per operand and nothing is exchanged between wavefronts.
//
// v_mfma_f32_16x16x4f32: D[i][n] += sum_k A[i][k] B[k][n], lane (c = lane % 16, g = lane / 16) supplies A[c][g] and
// B[g][c] and holds D[4 g + r][c] in register r.  Which column of a row a (step, g) pair stands for is free as long as
// A and B agree, so operands are held as 16-byte vectors (the members' rows are loaded that way; the entries' rows
// reach the first layout below through LDS, see tile_rows_to_operand):
//   scores S^T = K Q^T : A = K[entry e(c)][16 t + 4 g + e], B = q[member c][16 t + 4 g + e] (steps t, e = 0..3), where
//                        row c of the product is entry e(c) = 4 (c % 4) + c / 4 of the block, so that
//                        register r of lane (c, g) = score of (entry 4 r + g, member c);
//   output O += P V    : A = register r of the probabilities as they stand (row = member c, k = g stands for entry
//                        4 r + g), B = V[entry 4 r + g][4 c + nb]; register r' of accumulator nb of lane (c, g) =
//                        O[member 4 g + r'][4 c + nb]: four consecutive columns per lane, 256 contiguous bytes per
//                        member and 16 lanes.  Step r of such a product covers the neighbouring entries 4 r .. 4 r + 3:
//                        past the end of a group's entry list (half of its last block on average) steps are left out.
//   (The bfloat16 kernels below keep entry 4 g + r in register r: their products over the entries are one instruction.)
// Softmax state is per lane for member c (the four lanes of a member hold partial denominators that are added at the
// end); the exponent reference is raised lazily as in the matrix-core forward above.
constexpr int TILE_R = 16;
constexpr int TILE_CHUNK = 128;                     // entries staged in LDS at a time = 8 blocks

typedef float floatx4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float lane_bcast(float x, int src_lane) {
    return __int_as_float(__builtin_amdgcn_ds_bpermute(src_lane << 2, __float_as_int(x)));
}
__device__ __forceinline__ int lane_bcast(int x, int src_lane) { return __builtin_amdgcn_ds_bpermute(src_lane << 2, x); }

// Common start of the tile kernels.  HW heads (= wavefronts) per workgroup: workgroup b handles head slice
// (b / 8) % (H / HW) of group (b / 8) / (H / HW) of XCD b % 8's range.
struct TileCtx {
    int lane, wv, c, g, head, p_begin, p_end;
    int2 member;                 // (row, slot) of member c
    uint32_t offa, offv;         // byte offsets of this lane inside a node row: its 16-column slice of the head (operands of the
                                 // products that contract over columns, + 64 t bytes per step), and its columns 4 c .. 4 c + 3
};

template <typename T, int H, int D, int HW>
__device__ __forceinline__ bool tile_begin(const bpt_plan &P, TileCtx &t) {
    static_assert(D == 64 && H % HW == 0 && (sizeof(T) == 4 || sizeof(T) == 2), "64 columns per head: one 16-column slice per lane group");
    constexpr int HS = H / HW;
    t.lane = threadIdx.x & (WAVE - 1);
    t.wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    t.c = t.lane & 15;
    t.g = t.lane >> 4;
    const int x = blockIdx.x & 7, w = (blockIdx.x >> 3) / HS;
    const int grp = __builtin_amdgcn_readfirstlane(P.grp_chunks[x]) + w;
    if (grp >= __builtin_amdgcn_readfirstlane(P.grp_chunks[x + 1])) return false;
    t.member = reinterpret_cast<const int2 *>(P.grp_members)[(size_t)grp * TILE_R + t.c];
    t.p_begin = __builtin_amdgcn_readfirstlane(P.grp_ptr[grp]);
    t.p_end = __builtin_amdgcn_readfirstlane(P.grp_ptr[grp + 1]);
    t.head = (int)((blockIdx.x >> 3) % HS) * HW + t.wv;
    t.offa = (uint32_t)((t.head * D + 4 * t.g) * sizeof(T));
    t.offv = (uint32_t)((t.head * D + 4 * t.c) * sizeof(T));
    return true;
}

// The entry list of a group is staged, TILE_CHUNK entries at a time, in a wavefront-private piece of LDS as (neighbour,
// mask) pairs: every lane needs five of them per block (its A-operand row and the four rows / masks of its lane
// group), which would otherwise be five dependent global loads in front of every block's row loads.
struct TileEntryRegs {
    int4 x[TILE_CHUNK / WAVE];
};
// first half: the loads.  A kernel asks for its first piece before it reads its members' rows, so that the two round trips
// run side by side; in source order the compiler puts the members' arithmetic (and its wait) in front of these loads.
__device__ __forceinline__ void tile_ask_entries(const bpt_plan &P, int p0, int cnt, int lane, TileEntryRegs &r) {
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
#pragma unroll
    for (int u = 0; u < TILE_CHUNK / WAVE; ++u) r.x[u] = entries[p0 + min(u * WAVE + lane, cnt - 1)];   // past the end: the last entry again
}
// second half: into the wavefront's piece of LDS
__device__ __forceinline__ void tile_put_entries(const TileEntryRegs &r, int2 *lds, int cnt, int lane, int *first = nullptr) {
#pragma unroll
    for (int u = 0; u < TILE_CHUNK / WAVE; ++u) {
        const int e = u * WAVE + lane;
        int nbr = r.x[u].x, mask = r.x[u].y;
        asm volatile("" : "+v"(nbr), "+v"(mask));                 // (the values are used from here on: nothing of this half moves up to the loads)
        lds[e] = make_int2(nbr, e < cnt ? mask : 0);              // past the end: an empty mask
        if (first) first[e] = r.x[u].z;                          // number of the entry's first pair (members follow in ascending order)
    }
    wave_lds_fence();
}
__device__ __forceinline__ void tile_stage_entries(const bpt_plan &P, int2 *lds, int p0, int cnt, int lane, int *first = nullptr) {
    TileEntryRegs r;
    tile_ask_entries(P, p0, cnt, lane, r);
    tile_put_entries(r, lds, cnt, lane, first);
}
// number of the pair (entry, member c) among the plan's pairs: the entry's first pair + the members before c in its mask
__device__ __forceinline__ int tile_pair_number(int first, int mask, int c) { return first + __popc((uint32_t)mask & ((1u << c) - 1u)); }

// this lane's 16 columns of a node row (bytes offa + 64 t), as the A or B operand of a product over columns
__device__ __forceinline__ void tile_load16(const char *row, float (&out)[16]) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const float4 x = *reinterpret_cast<const float4 *>(row + 64 * t);
        out[4 * t] = x.x; out[4 * t + 1] = x.y; out[4 * t + 2] = x.z; out[4 * t + 3] = x.w;
    }
}

// register r of the result of lane (c, g) = sum over the 64 columns of a[row 4 g + r] * b[member c], a[row c] = what lane c passes
__device__ __forceinline__ floatx4v tile_dot(const float (&a)[16], const float (&b)[16]) {
    floatx4v s0 = floatx4v{0.f, 0.f, 0.f, 0.f}, s1 = s0;
#pragma unroll
    for (int i = 0; i < 16; i += 2) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[i], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i + 1], b[i + 1], s1, 0, 0, 0);
    }
    return s0 + s1;
}

// acc[nb][r'] (member 4 g + r', column 4 c + nb) += sum over the block's entries of w[member][entry] * row[entry][column]:
// w = this lane's four weights (member c with entries 4 r + g), rows = columns 4 c .. 4 c + 3 of the rows of entries 4 r + g.
// Step r of the product stands for the four NEIGHBOURING entries 4 r .. 4 r + 3 (one per lane group), so a step whose
// entries lie past the end of the group's list (nv = the block's entries that exist) is left out.
__device__ __forceinline__ void tile_axpy_upto(const float (&w)[4], const float4 (&rows)[4], floatx4v (&acc)[4], int nv) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (4 * r < nv) {
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[r], rows[r].x, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[r], rows[r].y, acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[r], rows[r].z, acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[r], rows[r].w, acc[3], 0, 0, 0);
        } else {
            // (the step's rows are marked as read: left in flight, they would make the next block's loads wait for
            // everything that is outstanding, this block's stores included)
            asm volatile("" ::"v"(rows[r].x), "v"(rows[r].y), "v"(rows[r].z), "v"(rows[r].w));
        }
    }
}

// The members' result rows: whole rows go to `out` (scaled by inv[member] where given), segments of split rows to the
// workspace in natural column order.
template <int H, int D, bool SCALE, typename T>
__device__ __forceinline__ void tile_store_rows(const TileCtx &t, const floatx4v (&acc)[4], float inv_c, T *__restrict__ out,
                                                float *__restrict__ ws) {
    constexpr int C = H * D;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int m = 4 * t.g + r;                                // the member whose row this lane stores a piece of
        const int row = lane_bcast(t.member.x, m), slot = lane_bcast(t.member.y, m);
        const float inv = SCALE ? lane_bcast(inv_c, m) : 1.f;
        if (row < 0) continue;
        float4 x = make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]);
        if (slot < 0) {
            if (SCALE) { x.x *= inv; x.y *= inv; x.z *= inv; x.w *= inv; }
            if constexpr (sizeof(T) == 4) {
                *reinterpret_cast<float4 *>(out + (size_t)row * C + t.head * D + 4 * t.c) = x;
            } else {
                const uint2 y = make_uint2(((uint32_t)f32_to_bf16(x.x)) | ((uint32_t)f32_to_bf16(x.y) << 16),
                               ((uint32_t)f32_to_bf16(x.z)) | ((uint32_t)f32_to_bf16(x.w) << 16));
                *reinterpret_cast<uint2 *>(out + (size_t)row * C + t.head * D + 4 * t.c) = y;
            }
        } else {
            *reinterpret_cast<float4 *>(ws + (size_t)slot * C + t.head * D + 4 * t.c) = x;
        }
    }
}

// Edge ids of this lane's four pairs of a block, (entry first_entry + step * r, member c): what the dropout hash and the score term are
// indexed by (n_edges, the spare row, where the pair does not exist; past the group's end the last entry is read again).
__device__ __forceinline__ void tile_pair_eids(const bpt_plan &P, int first_entry, int p_end, int c, int (&xe)[4], int step = 1) {
#pragma unroll
    for (int r = 0; r < 4; ++r) xe[r] = P.grp_eids[(size_t)min(first_entry + step * r, p_end - 1) * TILE_R + c];
}
// Which entry of a block lane c loads as row c of the products over the columns, in the float32 tile kernels: the
// scores of entries 4 r + g have to come out in register r of lane group g (row 4 g + r of the product), so that step r
// of the products over the entries stands for four NEIGHBOURING entries and can be left out past the end of the list.
__device__ __forceinline__ int tile_entry_of_row(int c) { return 4 * (c & 3) + (c >> 2); }
// Where the score term of the pair (entry, member c) sits and its gradient goes.  BIAS == 1, stored by edge id: row eid
// of (n_edges + 1, H), the spare last row for a pair that does not exist.  BIAS == 2, stored in the plan's own order:
// head-major at the pair's number, x[head * n_edges + number]: the lanes of an entry touch one run of memory and no
// index is read on the way; a pair that does not exist gets a neighbour's place, which is read and not used.
template <int H, int BIAS>
__device__ __forceinline__ uint32_t tile_bias_at(const bpt_plan &P, int head, int eid, int number) {
    if constexpr (BIAS == 2) return (uint32_t)head * (uint32_t)P.n_edges + (uint32_t)min(number, (int)P.n_edges - 1);
    else return (uint32_t)eid * (uint32_t)H + (uint32_t)head;
}

// The rows of a block's entries come from memory in the layout of the products over the entries (lane (c, g): columns
// 4 c .. 4 c + 3 of the rows of entries 4 r + g: the sixteen lanes of a lane group read one row's 256 contiguous bytes).
// The products over the COLUMNS want lane c to hold sixteen columns of ONE row (entry tile_entry_of_row(c)); loaded that
// way, neighbouring lanes read different rows and the texture addresser spends four cycles on every group of four lanes
// instead of one.  So the rows are loaded once, in the first layout, and turned in a wavefront-private piece of LDS:
// rows of TILE_KT_STRIDE floats (64 + 4: the sixteen rows of a read fall on different banks).
constexpr int TILE_KT_STRIDE = 68;
__device__ __forceinline__ void tile_rows_to_operand(float *kt, const float4 (&rows)[4], int c, int g, float (&out)[16]) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
        *reinterpret_cast<floatx4v *>(kt + (4 * r + g) * TILE_KT_STRIDE + 4 * c) = floatx4v{rows[r].x, rows[r].y, rows[r].z, rows[r].w};
    wave_lds_fence();
    const float *src = kt + tile_entry_of_row(c) * TILE_KT_STRIDE + 4 * g;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const floatx4v x = *reinterpret_cast<const floatx4v *>(src + 16 * t);
        out[4 * t] = x[0]; out[4 * t + 1] = x[1]; out[4 * t + 2] = x[2]; out[4 * t + 3] = x[3];
    }
    wave_lds_fence();                                             // (read before the next block's rows are written)
}

// PIPE: the rows of the next block are loaded while one is used (two-stage register pipeline).  Pays on graphs with few,
// tall tiles (a dense window graph: 9 blocks per tile, two wavefronts per SIMD in all), costs a wavefront per SIMD:
// at L = 8192, k = 4 (1217 tiles of 4 blocks) the forward takes 47 us with it and 44 without.
// Other forms measured there and dropped: groups of 32 rows (two member blocks per wavefront sharing the K / V
// registers: a third fewer rows through the L1s, two or three wavefronts per SIMD, 56 us; two wavefronts per head in step
// on the same entries, one member block each, so that the L1 fetches a row once: 60 us: the time follows the number
// of 16 x 16 blocks, 4716 against 6324, not the bytes), five or six wavefronts per SIMD by spilling (53 / 85 us).
template <bool PIPE, typename Blk, typename Issue, typename Compute>
__device__ __forceinline__ void tile_walk(int nblk, Issue &&issue, Compute &&compute) {
    if constexpr (PIPE) {
        Blk A, B;
        issue(A, 0);
        for (int b = 0; b < nblk; b += 2) {
            issue(B, min(b + 1, nblk - 1));                       // past the end: the last block again, not used
            issue_loads_first();
            compute(A);
            issue_loads_first();
            issue(A, min(b + 2, nblk - 1));
            issue_loads_first();
            if (b + 1 < nblk) compute(B);
            issue_loads_first();
        }
    } else {
        for (int b = 0; b < nblk; ++b) {
            Blk A;
            issue(A, b);
            issue_loads_first();
            compute(A);
            issue_loads_first();
        }
    }
}

// The rows a block needs FIRST (the K rows of its scores) are asked for one block ahead, the others (V) when the block
// begins: sixteen more registers instead of the thirty-two of the two-stage pipeline, so four wavefronts per SIMD stay.
// once_loads_left(): called once the first loads have left, for work that waits for loads asked for before them.
template <typename Blk, typename IssueFirst, typename IssueRest, typename Compute, typename Hook>
__device__ __forceinline__ void tile_walk_first_ahead(int nblk, IssueFirst &&first, IssueRest &&rest, Compute &&compute, Hook &&once_loads_left) {
    Blk A, B;
    first(A, 0);
    issue_loads_first();
    once_loads_left();
    int b = 0;
    for (; b + 2 < nblk; b += 2) {
        rest(A, b);
        first(B, b + 1);
        issue_loads_first();
        compute(A);
        issue_loads_first();
        rest(B, b + 1);
        first(A, b + 2);
        issue_loads_first();
        compute(B);
        issue_loads_first();
    }
    rest(A, b);
    if (b + 1 < nblk) {
        first(B, b + 1);
        issue_loads_first();
        compute(A);
        issue_loads_first();
        rest(B, b + 1);
        issue_loads_first();
        compute(B);
    } else {
        issue_loads_first();
        compute(A);
    }
    issue_loads_first();
}

template <typename T, int H, int D, int HW, bool PIPE, bool DROP, int BIAS>
__global__ __launch_bounds__(HW * WAVE) __attribute__((amdgpu_waves_per_eu(PIPE ? 3 : 4))) void k_attn_fwd_tile(
    bpt_plan P, const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v, T *__restrict__ o, float *__restrict__ lse,
    float *__restrict__ ws_acc, float *__restrict__ ws_ml, float scale_log2e, uint32_t drop_thr, uint32_t drop_seed, float drop_inv,
    const float *__restrict__ bias) {
    constexpr int C = H * D;
    TileCtx t;
    if (!tile_begin<T, H, D, HW>(P, t)) return;
    __shared__ int2 ent_lds[HW][TILE_CHUNK];
    __shared__ int fst_lds[HW][BIAS == 2 ? TILE_CHUNK : 1];      // the entries' first pair numbers: where a term in pair order sits
    int2 *ent = ent_lds[t.wv];
    int *fst = BIAS == 2 ? fst_lds[t.wv] : nullptr;
    __shared__ float kt_lds[HW][TILE_R * TILE_KT_STRIDE];
    float *kt = kt_lds[t.wv];
    TileEntryRegs er;
    if (t.p_end > t.p_begin) tile_ask_entries(P, t.p_begin, min(TILE_CHUNK, t.p_end - t.p_begin), t.lane, er);
    issue_loads_first();
    const int c = t.c, g = t.g;
    const char *kb = reinterpret_cast<const char *>(k), *vb = reinterpret_cast<const char *>(v);
    float qb[16];
    // The members' q rows are asked for behind the first block's K rows: asked for here, ahead of the loop, they are waited
    // for before the entry list is (one more round trip in front of the K rows).  They stay as they are and the scores are
    // scaled instead, so nothing has to happen to them between their arrival and the first product.
    const char *const qrow = reinterpret_cast<const char *>(q) + (size_t)max(t.member.x, 0) * (C * sizeof(T)) + t.offa;
    constexpr bool AHEAD = !PIPE && !DROP && BIAS == 0;         // (with dropout or the score term the sixteen registers are not there)
    if constexpr (!AHEAD) tile_load16(qrow, qb);
    floatx4v acc[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) acc[nb] = floatx4v{0.f, 0.f, 0.f, 0.f};
    float mref = M_INIT_LOG2, lrun = 0.f;
    struct Blk {
        float4 kq[4];                                             // columns 4 c .. 4 c + 3 of the K rows of entries 4 r + g
        float4 vr[4];
        int has, nv;                                              // bit r of has: the pair (entry 4 r + g, member c) exists; nv: entries of the block that exist
        int xe[DROP || BIAS == 1 ? 4 : 1];
        float bz[BIAS ? 4 : 1];
    };
    for (int p0 = t.p_begin; p0 < t.p_end; p0 += TILE_CHUNK) {
        const int cnt = min(TILE_CHUNK, t.p_end - p0), nblk = (cnt + TILE_R - 1) / TILE_R;
        if (p0 != t.p_begin) tile_ask_entries(P, p0, cnt, t.lane, er);
        tile_put_entries(er, ent, cnt, t.lane, fst);
        auto issue_k = [&](Blk &B, int b) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                B.kq[r] = *reinterpret_cast<const float4 *>(kb + ((uint32_t)ent[TILE_R * b + 4 * r + g].x * (uint32_t)(C * sizeof(T)) + t.offv));
        };
        auto issue_rest = [&](Blk &B, int b) {
            if constexpr (DROP || BIAS == 1) tile_pair_eids(P, p0 + TILE_R * b + g, t.p_end, c, B.xe, 4);
            B.nv = min(TILE_R, cnt - TILE_R * b);
            int idxv[4], mk[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int2 en = ent[TILE_R * b + 4 * r + g];
                idxv[r] = en.x; mk[r] = en.y;
            }
            B.has = ((mk[0] >> c) & 1) | (((mk[1] >> c) & 1) << 1) | (((mk[2] >> c) & 1) << 2) | (((mk[3] >> c) & 1) << 3);
#pragma unroll
            for (int r = 0; r < 4; ++r)
                B.vr[r] = *reinterpret_cast<const float4 *>(vb + ((uint32_t)idxv[r] * (uint32_t)(C * sizeof(T)) + t.offv));
            if constexpr (BIAS == 1) {
#pragma unroll
                for (int r = 0; r < 4; ++r) B.bz[r] = bias[tile_bias_at<H, 1>(P, t.head, B.xe[BIAS == 1 ? r : 0], 0)];
            }
            if constexpr (BIAS == 2) {
#pragma unroll
                for (int r = 0; r < 4; ++r) B.bz[r] = bias[tile_bias_at<H, 2>(P, t.head, 0, tile_pair_number(fst[TILE_R * b + 4 * r + g], mk[r], c))];
            }
        };
        auto compute = [&](const Blk &B) {
            float kr[16];
            tile_rows_to_operand(kt, B.kq, c, g, kr);
            const floatx4v st = tile_dot(kr, qb);
            float sc[4];
#pragma unroll
            for (int r = 0; r < 4; ++r)
                sc[r] = ((B.has >> r) & 1) ? (BIAS ? fmaf(st[r], scale_log2e, B.bz[BIAS ? r : 0] * scale_log2e) : st[r] * scale_log2e) : -INFINITY;
            const float mb = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
            if (__builtin_amdgcn_ballot_w64(mb > mref + MFMA_TAU) != 0) {
                float gm = fmaxf(mb, __shfl_xor(mb, 16));
                gm = fmaxf(gm, __shfl_xor(gm, 32));              // over the four lanes of member c
                const float mn = fmaxf(mref, gm);
                const float al = __builtin_amdgcn_exp2f(mref - mn);
                mref = mn;
                lrun *= al;
                // register r' of the accumulators belongs to member 4 g + r': its factor sits in lane 4 g + r'
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float a = lane_bcast(al, 4 * g + r);
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) acc[nb][r] *= a;
                }
            }
            float pr[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                pr[r] = __builtin_amdgcn_exp2f(sc[r] - mref);
                lrun += pr[r];                                   // the softmax denominator ignores dropout
                if constexpr (DROP)
                    pr[r] *= dropout_keep((uint32_t)B.xe[DROP ? r : 0] * (uint32_t)H + (uint32_t)t.head, drop_seed, drop_thr, drop_inv);
            }
            tile_axpy_upto(pr, B.vr, acc, B.nv);
        };
        auto issue = [&](Blk &B, int b) { issue_k(B, b); issue_rest(B, b); };
        if constexpr (!AHEAD) tile_walk<PIPE, Blk>(nblk, issue, compute);
        else tile_walk_first_ahead<Blk>(nblk, issue_k, issue_rest, compute, [&]() { if (p0 == t.p_begin) tile_load16(qrow, qb); });
        wave_lds_fence();                                         // the piece is read to the end before the next one is staged
    }
    float lt = lrun + __shfl_xor(lrun, 16);
    lt += __shfl_xor(lt, 32);                                    // denominator of member c, in its four lanes
    tile_store_rows<H, D, true>(t, acc, lt > 0.f ? 1.f / lt : 0.f, o, ws_acc);
    if (g == 0 && t.member.x >= 0) {                              // lanes 0 .. 15: one member each
        if (t.member.y < 0) {
            lse[(size_t)t.member.x * H + t.head] = lt > 0.f ? mref + log2f(lt) : 0.f;
        } else {
            ws_ml[((size_t)t.member.y * H + t.head) * 2] = mref;
            ws_ml[((size_t)t.member.y * H + t.head) * 2 + 1] = lt;
        }
    }
}

// Backward on tiles, destination side: per block the scores and dO . v of all 16 x 16 pairs (two products over the
// columns, the K and V rows turned in LDS from the layout they are loaded in), p = 2^(s - lse),
// ds = p (dO . v - delta) scale, dq += ds K (third product, on the K rows as loaded).  With dropout or a score term the
// kernel is compiled for three wavefronts per SIMD: at four it keeps the members' q rows in scratch memory and reads
// them back for every block (83 against 58 us with dropout at L = 8192, k = 4).
// (p, ds) of the pairs that exist go to a scratch in THIS side's order, compact:
// pds[head * n_edges + t] for the pair number t of (entry, member) = the entry's first pair + the rank of the member in
// its mask, so the lanes of an entry write one contiguous run and the runs of consecutive entries follow each other.  The
// source side looks its pairs up there through its pair mapping (grp_pairs = this side's pair numbers).  Writing in the
// source side's layout instead (scattered 8-byte stores here, contiguous reads there) cost this kernel a third of its
// time (126 against 85 us at L = 4096, k = 32); letting the source side recompute p and ds (two more products there,
// delta (n, H) handed over) measured slower than either on every graph tried.
template <typename T, int H, int D, int HW, bool PIPE, bool DROP, int BIAS>
__global__ __launch_bounds__(HW * WAVE) __attribute__((amdgpu_waves_per_eu(PIPE ? 2 : DROP || BIAS ? 3 : 4))) void k_attn_bwd_dst_tile(
    bpt_plan P, const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v, const T *__restrict__ o,
    const T *__restrict__ d_o, const float *__restrict__ lse, T *__restrict__ dq, float2 *__restrict__ pds, float *__restrict__ ws_dq,
    float scale, float scale_log2e, uint32_t drop_thr, uint32_t drop_seed, float drop_inv, const float *__restrict__ bias,
    float *__restrict__ ds_out) {
    constexpr int C = H * D;
    TileCtx t;
    if (!tile_begin<T, H, D, HW>(P, t)) return;
    __shared__ int2 ent_lds[HW][TILE_CHUNK];
    __shared__ int fst_lds[HW][TILE_CHUNK];
    int2 *ent = ent_lds[t.wv];
    int *fst = fst_lds[t.wv];
    __shared__ float kt_lds[HW][TILE_R * TILE_KT_STRIDE];
    float *kt = kt_lds[t.wv];
    TileEntryRegs er;
    if (t.p_end > t.p_begin) tile_ask_entries(P, t.p_begin, min(TILE_CHUNK, t.p_end - t.p_begin), t.lane, er);
    issue_loads_first();
    const int c = t.c, g = t.g;
    const char *kb = reinterpret_cast<const char *>(k), *vb = reinterpret_cast<const char *>(v);
    const size_t mrow = (size_t)max(t.member.x, 0) * (C * sizeof(T)) + t.offa;
    float2 *const pds_h = pds + (size_t)t.head * (size_t)P.n_edges;     // this head's part of the scratch
    // the member's dO columns live in LDS (lane-major, read back before every product with them): with them in registers
    // the kernel needs 144 and a SIMD holds three wavefronts, without them 128 and four
    __shared__ float4 dob_lds[HW][4][WAVE];
    // (q stays as it is and the scores are scaled, as in the forward: the same roundings in both)
    float qb[16], delta, lse_c;
    {
        float ob[16], dob[16];
        tile_load16(reinterpret_cast<const char *>(q) + mrow, qb);
        tile_load16(reinterpret_cast<const char *>(d_o) + mrow, dob);
        tile_load16(reinterpret_cast<const char *>(o) + mrow, ob);
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) part = fmaf(dob[i], ob[i], part);
        part += __shfl_xor(part, 16);
        delta = part + __shfl_xor(part, 32);                      // dO . O of member c, this head
        lse_c = lse[(size_t)max(t.member.x, 0) * H + t.head];
#pragma unroll
        for (int i = 0; i < 4; ++i) dob_lds[t.wv][i][t.lane] = make_float4(dob[4 * i], dob[4 * i + 1], dob[4 * i + 2], dob[4 * i + 3]);
    }
    floatx4v acc[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) acc[nb] = floatx4v{0.f, 0.f, 0.f, 0.f};
    struct Blk {
        float4 kc[4], vc[4];                                      // columns 4 c .. 4 c + 3 of the K / V rows of entries 4 r + g
        int pos[4], has, nv;                                       // bit r of has: the pair (entry 4 r + g, member c) exists; nv: entries of the block that exist
        int xe[DROP || BIAS == 1 ? 4 : 1];
        float bz[BIAS ? 4 : 1];
    };
    for (int p0 = t.p_begin; p0 < t.p_end; p0 += TILE_CHUNK) {
        const int cnt = min(TILE_CHUNK, t.p_end - p0), nblk = (cnt + TILE_R - 1) / TILE_R;
        if (p0 != t.p_begin) tile_ask_entries(P, p0, cnt, t.lane, er);
        tile_put_entries(er, ent, cnt, t.lane, fst);
        auto issue = [&](Blk &B, int b) {
            if constexpr (DROP || BIAS == 1) tile_pair_eids(P, p0 + TILE_R * b + g, t.p_end, c, B.xe, 4);
            B.nv = min(TILE_R, cnt - TILE_R * b);
            int idxv[4];
            B.has = 0;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int2 en = ent[TILE_R * b + 4 * r + g];
                idxv[r] = en.x;
                B.has |= ((en.y >> c) & 1) << r;
                B.pos[r] = tile_pair_number(fst[TILE_R * b + 4 * r + g], en.y, c);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r)
                B.kc[r] = *reinterpret_cast<const float4 *>(kb + ((uint32_t)idxv[r] * (uint32_t)(C * sizeof(T)) + t.offv));
#pragma unroll
            for (int r = 0; r < 4; ++r)
                B.vc[r] = *reinterpret_cast<const float4 *>(vb + ((uint32_t)idxv[r] * (uint32_t)(C * sizeof(T)) + t.offv));
            if constexpr (BIAS) {
#pragma unroll
                for (int r = 0; r < 4; ++r) B.bz[r] = bias[tile_bias_at<H, BIAS>(P, t.head, B.xe[BIAS == 1 ? r : 0], B.pos[r])];
            }
        };
        auto compute = [&](const Blk &B) {
            floatx4v st;
            {
                float kr[16];
                tile_rows_to_operand(kt, B.kc, c, g, kr);
                st = tile_dot(kr, qb);
            }
            float va[16];
            tile_rows_to_operand(kt, B.vc, c, g, va);
            float dob[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 x = dob_lds[t.wv][i][t.lane];
                dob[4 * i] = x.x; dob[4 * i + 1] = x.y; dob[4 * i + 2] = x.z; dob[4 * i + 3] = x.w;
            }
            const floatx4v dp = tile_dot(va, dob);
            float ds[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const bool has = (B.has >> r) & 1;
                float pe = has ? __builtin_amdgcn_exp2f((BIAS ? fmaf(st[r], scale_log2e, B.bz[BIAS ? r : 0] * scale_log2e) : st[r] * scale_log2e) - lse_c) : 0.f;
                float mt = 1.f;                                   // dropout multiplier of this pair (as in the forward)
                if constexpr (DROP)
                    mt = dropout_keep((uint32_t)B.xe[DROP ? r : 0] * (uint32_t)H + (uint32_t)t.head, drop_seed, drop_thr, drop_inv);
                ds[r] = pe * (dp[r] * mt - delta) * scale;
                pe *= mt;                                         // what multiplies v (forward) and dO (dV)
                if (has) {
                    pds_h[B.pos[r]] = make_float2(pe, ds[r]);
                    if constexpr (BIAS) ds_out[tile_bias_at<H, BIAS>(P, t.head, B.xe[BIAS == 1 ? r : 0], B.pos[r])] = ds[r];   // dL/d(score before scaling)
                }
            }
            tile_axpy_upto(ds, B.kc, acc, B.nv);
        };
        tile_walk<PIPE, Blk>(nblk, issue, compute);
        wave_lds_fence();
    }
    tile_store_rows<H, D, false>(t, acc, 1.f, dq, ws_dq);
}

// Backward on tiles, source side (groups of the out-CSR plan: members = source rows, entries = destinations):
// dk += ds^T q, dv += p^T dO with (p, ds) of every pair fetched from the scratch the destination side filled, at the
// destination side's pair number that this plan's grp_pairs gives for (entry, member).
template <typename T, int H, int D, int HW, bool PIPE>
__global__ __launch_bounds__(HW * WAVE) __attribute__((amdgpu_waves_per_eu(PIPE ? 3 : 4))) void k_attn_bwd_src_tile(
    bpt_plan P, const T *__restrict__ q, const T *__restrict__ d_o, const float2 *__restrict__ pds, T *__restrict__ dk, T *__restrict__ dv,
    float *__restrict__ ws_dk, float *__restrict__ ws_dv) {
    constexpr int C = H * D;
    TileCtx t;
    if (!tile_begin<T, H, D, HW>(P, t)) return;
    __shared__ int2 ent_lds[HW][TILE_CHUNK];
    int2 *ent = ent_lds[t.wv];
    const int c = t.c, g = t.g;
    const char *qb = reinterpret_cast<const char *>(q), *db = reinterpret_cast<const char *>(d_o);
    const float2 *const pds_h = pds + (size_t)t.head * (size_t)P.n_edges;
    floatx4v ak[4], av[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) { ak[nb] = floatx4v{0.f, 0.f, 0.f, 0.f}; av[nb] = floatx4v{0.f, 0.f, 0.f, 0.f}; }
    // Both products contract over the block's entries, four per step; lane group g takes entries 4 r + g in step r, so that
    // the steps past the end of the group's list (half of a group's last block on average) can be left out.
    struct Blk {
        float4 qr[4], dr[4];
        float2 w[4];
        int has, nv;                                              // bit r of has: the pair (entry 4 r + g, member c) exists; nv: entries of the block that exist
    };
    for (int p0 = t.p_begin; p0 < t.p_end; p0 += TILE_CHUNK) {
        const int cnt = min(TILE_CHUNK, t.p_end - p0), nblk = (cnt + TILE_R - 1) / TILE_R;
        tile_stage_entries(P, ent, p0, cnt, t.lane);
        // Where this lane's four pairs of block b sit in the scratch (positions past the group's end are read at its last
        // entry: their masks are empty).  They are fetched one block ahead, so that the (p, ds) loads of a block leave
        // together with its row loads instead of one round trip later.
        auto positions = [&](int b, int (&pos)[4]) {
#pragma unroll
            for (int r = 0; r < 4; ++r) pos[r] = P.grp_pairs[(size_t)min(p0 + TILE_R * b + 4 * r + g, t.p_end - 1) * TILE_R + c];
        };
        int pos_ahead[4], ahead_of = -1;                          // the positions of block ahead_of
        auto issue = [&](Blk &B, int b) {
            B.nv = min(TILE_R, cnt - TILE_R * b);
            B.has = 0;
            int pos[4];
            if constexpr (PIPE) {                                 // (rows are read a block ahead there, and registers are short)
                positions(b, pos);
            } else {
                if (b == ahead_of) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) pos[r] = pos_ahead[r];
                } else {
                    positions(b, pos);
                }
                if (b + 1 < nblk) positions(b + 1, pos_ahead);
                ahead_of = b + 1;
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int2 en = ent[TILE_R * b + 4 * r + g];
                B.has |= ((en.y >> c) & 1) << r;
                const uint32_t off = (uint32_t)en.x * (uint32_t)(C * sizeof(T)) + t.offv;
                B.qr[r] = *reinterpret_cast<const float4 *>(qb + off);
                B.dr[r] = *reinterpret_cast<const float4 *>(db + off);
                B.w[r] = pds_h[pos[r]];
            }
        };
        auto compute = [&](const Blk &B) {
            float pe[4], ds[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const bool has = (B.has >> r) & 1;              // the scratch of pairs that do not exist is not initialised
                pe[r] = has ? B.w[r].x : 0.f;
                ds[r] = has ? B.w[r].y : 0.f;
            }
            tile_axpy_upto(ds, B.qr, ak, B.nv);
            tile_axpy_upto(pe, B.dr, av, B.nv);
        };
        tile_walk<PIPE, Blk>(nblk, issue, compute);
        wave_lds_fence();
    }
    tile_store_rows<H, D, false>(t, ak, 1.f, dk, ws_dk);
    tile_store_rows<H, D, false>(t, av, 1.f, dv, ws_dv);
}

// ---- Dense tiles for bfloat16 rows.  Same walk and the same lane roles as the float32 tile kernels above, on
// v_mfma_f32_16x16x32_bf16 (products over the 64 columns: two instructions) and v_mfma_f32_16x16x16_bf16 (products over
// the 16 entries of a block: one instruction per four output columns), float32 accumulation:
//   lane (c, g) holds columns 16 g .. 16 g + 15 of the row of entry c (32 contiguous bytes; slot j of step t of the product
//   stands for column 16 g + 8 t + j in both operands; the members' rows are loaded that way, the entries' rows turned in
//   LDS, see tile_rows_to_operand_bf16) and loads columns 4 c .. 4 c + 3 of the rows of entries 4 g + r (8 bytes; the B
//   operand of output columns {4 c + nb} takes element nb of each of the four, packed by byte permutes).
// Probabilities and ds are rounded to bfloat16 where they enter a product (the softmax denominator is summed unrounded);
// the scratch between the two backward kernels holds (p, ds) as two bfloat16 in 4 bytes, by head and destination-side pair number.
// The two-stage register pipeline of tile_walk does not pay here: at six wavefronts per SIMD it spills (2.4 x slower),
// at four it measured 5 to 10 % slower on the sparse graphs and level on the window graph.  Tiles of 32 rows (two member
// blocks per wavefront on the same loaded rows, three or four wavefronts per SIMD) did not pay either: the entry lists
// shrink by a third on the destination side but only by an eighth on the source side (L = 8192, k = 4: 67 k -> 46 k and
// 71 k -> 62 k entries), and the step went from 0.113 to 0.117 ms (32-graph batch 0.177 -> 0.205, window 128 level).
constexpr bool TILE_BF16_PIPE = false;
constexpr int TILE_BF16_WPE = 5, TILE_BF16_WPE_DST = 5, TILE_BF16_WPE_SRC = 5;     // wavefronts per SIMD the bfloat16 tile kernels are compiled for
typedef __bf16 bf16x8v __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
typedef float floatx2v __attribute__((ext_vector_type(2)));
typedef short shortx4v __attribute__((ext_vector_type(4)));
union Bf8 { bf16x8v v; uint4 q; };
union Bf4 { shortx4v v; uint32_t u[2]; };

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    union { bf16x2v v; uint32_t u; } r;
    r.v = __builtin_convertvector(floatx2v{lo, hi}, bf16x2v);      // round to nearest even
    return r.u;
}
__device__ __forceinline__ uint32_t pack_lo16(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x05040100u); }   // (a.lo, b.lo)
__device__ __forceinline__ uint32_t pack_hi16(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x07060302u); }   // (a.hi, b.hi)

// B operand of output columns {4 c + nb}: element nb of the 8-byte pieces of the rows of entries 4 g + r, r = 0 .. 3
template <int NB>
__device__ __forceinline__ Bf4 tile_cols_bf16(const uint2 (&rows)[4]) {
    Bf4 b;
    if constexpr (NB == 0) { b.u[0] = pack_lo16(rows[0].x, rows[1].x); b.u[1] = pack_lo16(rows[2].x, rows[3].x); }
    if constexpr (NB == 1) { b.u[0] = pack_hi16(rows[0].x, rows[1].x); b.u[1] = pack_hi16(rows[2].x, rows[3].x); }
    if constexpr (NB == 2) { b.u[0] = pack_lo16(rows[0].y, rows[1].y); b.u[1] = pack_lo16(rows[2].y, rows[3].y); }
    if constexpr (NB == 3) { b.u[0] = pack_hi16(rows[0].y, rows[1].y); b.u[1] = pack_hi16(rows[2].y, rows[3].y); }
    return b;
}
// acc[nb][r'] (member 4 g + r', column 4 c + nb) += sum over the block's entries of w[member c][entry 4 g + r] * row[entry][column]
__device__ __forceinline__ void tile_axpy_bf16(const Bf4 &w, const uint2 (&rows)[4], floatx4v (&acc)[4]) {
    acc[0] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(w.v, tile_cols_bf16<0>(rows).v, acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(w.v, tile_cols_bf16<1>(rows).v, acc[1], 0, 0, 0);
    acc[2] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(w.v, tile_cols_bf16<2>(rows).v, acc[2], 0, 0, 0);
    acc[3] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(w.v, tile_cols_bf16<3>(rows).v, acc[3], 0, 0, 0);
}
// register r of lane (c, g) = sum over the 64 columns of a[entry 4 g + r] * b[member c]
__device__ __forceinline__ floatx4v tile_dot_bf16(const Bf8 (&a)[2], const Bf8 (&b)[2]) {
    floatx4v s = floatx4v{0.f, 0.f, 0.f, 0.f};
    s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[0].v, b[0].v, s, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[1].v, b[1].v, s, 0, 0, 0);
}
__device__ __forceinline__ void tile_load_row_bf16(const char *p, Bf8 (&out)[2]) {
    out[0].q = *reinterpret_cast<const uint4 *>(p);
    out[1].q = *reinterpret_cast<const uint4 *>(p + 16);
}
// As tile_rows_to_operand: the rows of a block's entries, loaded as columns 4 c .. 4 c + 3 of the rows of entries 4 g + r
// (the sixteen lanes of a lane group read one row's 128 contiguous bytes), turned in a wavefront-private piece of LDS
// into the operand of the products over the columns (lane (c, g): columns 16 g .. 16 g + 15 of the row of entry c).
// Rows of TILE_KT_BYTES_BF16 = 128 + 16 bytes: the sixteen rows of a read fall on different banks.
constexpr int TILE_KT_BYTES_BF16 = 144;
typedef uint32_t uintx2v __attribute__((ext_vector_type(2)));
typedef uint32_t uintx4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void tile_rows_to_operand_bf16(char *kt, const uint2 (&rows)[4], int c, int g, Bf8 (&out)[2]) {
#pragma unroll
    for (int r = 0; r < 4; ++r) *reinterpret_cast<uintx2v *>(kt + (4 * g + r) * TILE_KT_BYTES_BF16 + 8 * c) = uintx2v{rows[r].x, rows[r].y};
    wave_lds_fence();
    const char *src = kt + c * TILE_KT_BYTES_BF16 + 32 * g;
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
        const uintx4v x = *reinterpret_cast<const uintx4v *>(src + 16 * h2);
        out[h2].q = make_uint4(x[0], x[1], x[2], x[3]);
    }
    wave_lds_fence();                                             // (read before the next block's rows are written)
}

template <int H, int D, int HW, int WPE, bool PIPE, bool DROP, int BIAS>
__global__ __launch_bounds__(HW * WAVE) __attribute__((amdgpu_waves_per_eu(WPE))) void k_attn_fwd_tile_bf16(
    bpt_plan P, const bf16_t *__restrict__ q, const bf16_t *__restrict__ k, const bf16_t *__restrict__ v, bf16_t *__restrict__ o,
    float *__restrict__ lse, float *__restrict__ ws_acc, float *__restrict__ ws_ml, float scale_log2e, uint32_t drop_thr,
    uint32_t drop_seed, float drop_inv, const float *__restrict__ bias) {
    constexpr int RB = H * D * 2;                                 // bytes of a node row
    TileCtx t;
    if (!tile_begin<bf16_t, H, D, HW>(P, t)) return;
    __shared__ int2 ent_lds[HW][TILE_CHUNK];
    __shared__ int fst_lds[HW][BIAS == 2 ? TILE_CHUNK : 1];      // the entries' first pair numbers: where a term in pair order sits
    int2 *ent = ent_lds[t.wv];
    int *fst = BIAS == 2 ? fst_lds[t.wv] : nullptr;
    __shared__ __attribute__((aligned(16))) char kt_lds[HW][TILE_R * TILE_KT_BYTES_BF16];
    char *kt = kt_lds[t.wv];
    TileEntryRegs er;
    if (t.p_end > t.p_begin) tile_ask_entries(P, t.p_begin, min(TILE_CHUNK, t.p_end - t.p_begin), t.lane, er);
    issue_loads_first();
    const int c = t.c, g = t.g;
    const uint32_t offr = (uint32_t)((t.head * D + 16 * g) * 2), offc = (uint32_t)((t.head * D + 4 * c) * 2);
    const char *kb = reinterpret_cast<const char *>(k), *vb = reinterpret_cast<const char *>(v);
    Bf8 qb[2];
    tile_load_row_bf16(reinterpret_cast<const char *>(q) + (size_t)max(t.member.x, 0) * RB + offr, qb);
    floatx4v acc[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) acc[nb] = floatx4v{0.f, 0.f, 0.f, 0.f};
    float mref = M_INIT_LOG2, lrun = 0.f;
    struct Blk {
        uint2 kq[4];                                              // columns 4 c .. 4 c + 3 of the K rows of entries 4 g + r
        uint2 vr[4];
        int has;                                                  // bit r: the pair (entry 4 g + r, member c) exists
        int xe[DROP || BIAS == 1 ? 4 : 1];
        float bz[BIAS ? 4 : 1];
    };
    for (int p0 = t.p_begin; p0 < t.p_end; p0 += TILE_CHUNK) {
        const int cnt = min(TILE_CHUNK, t.p_end - p0), nblk = (cnt + TILE_R - 1) / TILE_R;
        if (p0 != t.p_begin) tile_ask_entries(P, p0, cnt, t.lane, er);
        tile_put_entries(er, ent, cnt, t.lane, fst);
        auto issue_k = [&](Blk &B, int b) {
            const int4 e01 = *reinterpret_cast<const int4 *>(&ent[TILE_R * b + 4 * g]);
            const int4 e23 = *reinterpret_cast<const int4 *>(&ent[TILE_R * b + 4 * g + 2]);
            const int idxv[4] = {e01.x, e01.z, e23.x, e23.z};
#pragma unroll
            for (int r = 0; r < 4; ++r) B.kq[r] = *reinterpret_cast<const uint2 *>(kb + ((uint32_t)idxv[r] * (uint32_t)RB + offc));
        };
        auto issue_rest = [&](Blk &B, int b) {
            if constexpr (DROP || BIAS == 1) tile_pair_eids(P, p0 + TILE_R * b + 4 * g, t.p_end, c, B.xe);
            const int4 e01 = *reinterpret_cast<const int4 *>(&ent[TILE_R * b + 4 * g]);
            const int4 e23 = *reinterpret_cast<const int4 *>(&ent[TILE_R * b + 4 * g + 2]);
            const int idxv[4] = {e01.x, e01.z, e23.x, e23.z};
            const int mk[4] = {e01.y, e01.w, e23.y, e23.w};
            B.has = ((mk[0] >> c) & 1) | (((mk[1] >> c) & 1) << 1) | (((mk[2] >> c) & 1) << 2) | (((mk[3] >> c) & 1) << 3);
#pragma unroll
            for (int r = 0; r < 4; ++r) B.vr[r] = *reinterpret_cast<const uint2 *>(vb + ((uint32_t)idxv[r] * (uint32_t)RB + offc));
            if constexpr (BIAS == 1) {
#pragma unroll
                for (int r = 0; r < 4; ++r) B.bz[r] = bias[tile_bias_at<H, 1>(P, t.head, B.xe[BIAS == 1 ? r : 0], 0)];
            }
            if constexpr (BIAS == 2) {
                const int4 f4 = *reinterpret_cast<const int4 *>(&fst[TILE_R * b + 4 * g]);
                const int fv[4] = {f4.x, f4.y, f4.z, f4.w};
#pragma unroll
                for (int r = 0; r < 4; ++r) B.bz[r] = bias[tile_bias_at<H, 2>(P, t.head, 0, tile_pair_number(fv[r], mk[r], c))];
            }
        };
        auto compute = [&](const Blk &B) {
            Bf8 kr[2];
            tile_rows_to_operand_bf16(kt, B.kq, c, g, kr);
            const floatx4v st = tile_dot_bf16(kr, qb);
            float sc[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) sc[r] = ((B.has >> r) & 1) ? (BIAS ? st[r] + B.bz[BIAS ? r : 0] : st[r]) * scale_log2e : -INFINITY;
            const float mb = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
            if (__builtin_amdgcn_ballot_w64(mb > mref + MFMA_TAU) != 0) {
                float gm = fmaxf(mb, __shfl_xor(mb, 16));
                gm = fmaxf(gm, __shfl_xor(gm, 32));              // over the four lanes of member c
                const float mn = fmaxf(mref, gm);
                const float al = __builtin_amdgcn_exp2f(mref - mn);
                mref = mn;
                lrun *= al;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float a = lane_bcast(al, 4 * g + r);
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) acc[nb][r] *= a;
                }
            }
            float pr[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                pr[r] = __builtin_amdgcn_exp2f(sc[r] - mref);
                lrun += pr[r];                                   // the softmax denominator ignores dropout
                if constexpr (DROP)
                    pr[r] *= dropout_keep((uint32_t)B.xe[DROP ? r : 0] * (uint32_t)H + (uint32_t)t.head, drop_seed, drop_thr, drop_inv);
            }
            Bf4 pa;
            pa.u[0] = pack_bf16(pr[0], pr[1]);
            pa.u[1] = pack_bf16(pr[2], pr[3]);
            tile_axpy_bf16(pa, B.vr, acc);
        };
        auto issue = [&](Blk &B, int b) { issue_k(B, b); issue_rest(B, b); };
        if constexpr (PIPE || DROP || BIAS != 0) tile_walk<PIPE, Blk>(nblk, issue, compute);      // (the K rows ahead: eight registers more)
        else tile_walk_first_ahead<Blk>(nblk, issue_k, issue_rest, compute, []() {});
        wave_lds_fence();
    }
    float lt = lrun + __shfl_xor(lrun, 16);
    lt += __shfl_xor(lt, 32);
    tile_store_rows<H, D, true>(t, acc, lt > 0.f ? 1.f / lt : 0.f, o, ws_acc);
    if (g == 0 && t.member.x >= 0) {
        if (t.member.y < 0) {
            lse[(size_t)t.member.x * H + t.head] = lt > 0.f ? mref + log2f(lt) : 0.f;
        } else {
            ws_ml[((size_t)t.member.y * H + t.head) * 2] = mref;
            ws_ml[((size_t)t.member.y * H + t.head) * 2 + 1] = lt;
        }
    }
}

template <int H, int D, int HW, int WPE, bool PIPE, bool DROP, int BIAS>
__global__ __launch_bounds__(HW * WAVE) __attribute__((amdgpu_waves_per_eu(DROP || BIAS ? WPE - 1 : WPE))) void k_attn_bwd_dst_tile_bf16(
    bpt_plan P, const bf16_t *__restrict__ q, const bf16_t *__restrict__ k, const bf16_t *__restrict__ v, const bf16_t *__restrict__ o,
    const bf16_t *__restrict__ d_o, const float *__restrict__ lse, bf16_t *__restrict__ dq, uint32_t *__restrict__ pds,
    float *__restrict__ ws_dq, float scale, float scale_log2e, uint32_t drop_thr, uint32_t drop_seed, float drop_inv,
    const float *__restrict__ bias, float *__restrict__ ds_out) {
    constexpr int RB = H * D * 2;
    TileCtx t;
    if (!tile_begin<bf16_t, H, D, HW>(P, t)) return;
    __shared__ int2 ent_lds[HW][TILE_CHUNK];
    __shared__ int fst_lds[HW][TILE_CHUNK];
    int2 *ent = ent_lds[t.wv];
    int *fst = fst_lds[t.wv];
    __shared__ __attribute__((aligned(16))) char kt_lds[HW][TILE_R * TILE_KT_BYTES_BF16];
    char *kt = kt_lds[t.wv];
    TileEntryRegs er;
    if (t.p_end > t.p_begin) tile_ask_entries(P, t.p_begin, min(TILE_CHUNK, t.p_end - t.p_begin), t.lane, er);
    issue_loads_first();
    const int c = t.c, g = t.g;
    const uint32_t offr = (uint32_t)((t.head * D + 16 * g) * 2), offc = (uint32_t)((t.head * D + 4 * c) * 2);
    const char *kb = reinterpret_cast<const char *>(k), *vb = reinterpret_cast<const char *>(v);
    const size_t mrow = (size_t)max(t.member.x, 0) * RB + offr;
    uint32_t *const pds_h = pds + (size_t)t.head * (size_t)P.n_edges;     // this head's part of the scratch
    Bf8 qb[2], dob[2];
    float delta, lse_c;
    {
        Bf8 ob[2];
        tile_load_row_bf16(reinterpret_cast<const char *>(q) + mrow, qb);
        tile_load_row_bf16(reinterpret_cast<const char *>(d_o) + mrow, dob);
        tile_load_row_bf16(reinterpret_cast<const char *>(o) + mrow, ob);
        float part = 0.f;
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
            const uint32_t a[4] = {dob[h2].q.x, dob[h2].q.y, dob[h2].q.z, dob[h2].q.w}, b[4] = {ob[h2].q.x, ob[h2].q.y, ob[h2].q.z, ob[h2].q.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                part = fmaf(__uint_as_float(a[i] << 16), __uint_as_float(b[i] << 16), part);
                part = fmaf(__uint_as_float(a[i] & 0xffff0000u), __uint_as_float(b[i] & 0xffff0000u), part);
            }
        }
        part += __shfl_xor(part, 16);
        delta = part + __shfl_xor(part, 32);                      // dO . O of member c, this head
        lse_c = lse[(size_t)max(t.member.x, 0) * H + t.head];
    }
    floatx4v acc[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) acc[nb] = floatx4v{0.f, 0.f, 0.f, 0.f};
    struct Blk {
        uint2 kc[4], vc[4];                                       // columns 4 c .. 4 c + 3 of the K / V rows of entries 4 g + r
        int has, pos[4];                                           // bit r of has: the pair (entry 4 g + r, member c) exists
        int xe[DROP || BIAS == 1 ? 4 : 1];
        float bz[BIAS ? 4 : 1];
    };
    for (int p0 = t.p_begin; p0 < t.p_end; p0 += TILE_CHUNK) {
        const int cnt = min(TILE_CHUNK, t.p_end - p0), nblk = (cnt + TILE_R - 1) / TILE_R;
        if (p0 != t.p_begin) tile_ask_entries(P, p0, cnt, t.lane, er);
        tile_put_entries(er, ent, cnt, t.lane, fst);
        auto issue = [&](Blk &B, int b) {
            if constexpr (DROP || BIAS == 1) tile_pair_eids(P, p0 + TILE_R * b + 4 * g, t.p_end, c, B.xe);
            const int4 e01 = *reinterpret_cast<const int4 *>(&ent[TILE_R * b + 4 * g]);
            const int4 e23 = *reinterpret_cast<const int4 *>(&ent[TILE_R * b + 4 * g + 2]);
            const int4 f4 = *reinterpret_cast<const int4 *>(&fst[TILE_R * b + 4 * g]);
            const int idxv[4] = {e01.x, e01.z, e23.x, e23.z};
            B.has = ((e01.y >> c) & 1) | (((e01.w >> c) & 1) << 1) | (((e23.y >> c) & 1) << 2) | (((e23.w >> c) & 1) << 3);
            B.pos[0] = tile_pair_number(f4.x, e01.y, c); B.pos[1] = tile_pair_number(f4.y, e01.w, c);
            B.pos[2] = tile_pair_number(f4.z, e23.y, c); B.pos[3] = tile_pair_number(f4.w, e23.w, c);
#pragma unroll
            for (int r = 0; r < 4; ++r) B.kc[r] = *reinterpret_cast<const uint2 *>(kb + ((uint32_t)idxv[r] * (uint32_t)RB + offc));
#pragma unroll
            for (int r = 0; r < 4; ++r) B.vc[r] = *reinterpret_cast<const uint2 *>(vb + ((uint32_t)idxv[r] * (uint32_t)RB + offc));
            if constexpr (BIAS) {
#pragma unroll
                for (int r = 0; r < 4; ++r) B.bz[r] = bias[tile_bias_at<H, BIAS>(P, t.head, B.xe[BIAS == 1 ? r : 0], B.pos[r])];
            }
        };
        auto compute = [&](const Blk &B) {
            Bf8 kr[2];
            tile_rows_to_operand_bf16(kt, B.kc, c, g, kr);
            const floatx4v st = tile_dot_bf16(kr, qb);
            tile_rows_to_operand_bf16(kt, B.vc, c, g, kr);
            const floatx4v dp = tile_dot_bf16(kr, dob);
            float ds[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const bool has = (B.has >> r) & 1;
                float pe = has ? __builtin_amdgcn_exp2f((BIAS ? st[r] + B.bz[BIAS ? r : 0] : st[r]) * scale_log2e - lse_c) : 0.f;
                float mt = 1.f;                                   // dropout multiplier of this pair (as in the forward)
                if constexpr (DROP)
                    mt = dropout_keep((uint32_t)B.xe[DROP ? r : 0] * (uint32_t)H + (uint32_t)t.head, drop_seed, drop_thr, drop_inv);
                ds[r] = pe * (dp[r] * mt - delta) * scale;
                pe *= mt;                                         // what multiplies v (forward) and dO (dV)
                if (has) {
                    pds_h[B.pos[r]] = pack_bf16(pe, ds[r]);
                    if constexpr (BIAS) ds_out[tile_bias_at<H, BIAS>(P, t.head, B.xe[BIAS == 1 ? r : 0], B.pos[r])] = ds[r];   // dL/d(score before scaling)
                }
            }
            Bf4 da;
            da.u[0] = pack_bf16(ds[0], ds[1]);
            da.u[1] = pack_bf16(ds[2], ds[3]);
            tile_axpy_bf16(da, B.kc, acc);
        };
        tile_walk<PIPE, Blk>(nblk, issue, compute);
        wave_lds_fence();
    }
    tile_store_rows<H, D, false>(t, acc, 1.f, dq, ws_dq);
}

template <int H, int D, int HW, int WPE, bool PIPE>
__global__ __launch_bounds__(HW * WAVE) __attribute__((amdgpu_waves_per_eu(WPE))) void k_attn_bwd_src_tile_bf16(
    bpt_plan P, const bf16_t *__restrict__ q, const bf16_t *__restrict__ d_o, const uint32_t *__restrict__ pds, bf16_t *__restrict__ dk,
    bf16_t *__restrict__ dv, float *__restrict__ ws_dk, float *__restrict__ ws_dv) {
    constexpr int RB = H * D * 2;
    TileCtx t;
    if (!tile_begin<bf16_t, H, D, HW>(P, t)) return;
    __shared__ int2 ent_lds[HW][TILE_CHUNK];
    int2 *ent = ent_lds[t.wv];
    const int c = t.c, g = t.g;
    const uint32_t offc = (uint32_t)((t.head * D + 4 * c) * 2);
    const char *qb = reinterpret_cast<const char *>(q), *db = reinterpret_cast<const char *>(d_o);
    const uint32_t *const pds_h = pds + (size_t)t.head * (size_t)P.n_edges;
    floatx4v ak[4], av[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) { ak[nb] = floatx4v{0.f, 0.f, 0.f, 0.f}; av[nb] = floatx4v{0.f, 0.f, 0.f, 0.f}; }
    struct Blk {
        uint2 qr[4], dr[4];
        uint32_t w[4];
        int has;                                                  // bit r: the pair (entry 4 g + r, member c) exists
    };
    for (int p0 = t.p_begin; p0 < t.p_end; p0 += TILE_CHUNK) {
        const int cnt = min(TILE_CHUNK, t.p_end - p0), nblk = (cnt + TILE_R - 1) / TILE_R;
        tile_stage_entries(P, ent, p0, cnt, t.lane);
        // (the positions of a block's pairs in the scratch are fetched one block ahead, as in the float32 kernel, so that the
        // (p, ds) loads leave with the row loads; positions past the group's end are read at its last entry: their masks are
        // empty.  The four registers this takes are why the kernel is compiled for five wavefronts per SIMD, not six: with
        // six it spills and loses what the prefetch gains)
        auto positions = [&](int b, int (&pos)[4]) {
#pragma unroll
            for (int r = 0; r < 4; ++r) pos[r] = P.grp_pairs[(size_t)min(p0 + TILE_R * b + 4 * g + r, t.p_end - 1) * TILE_R + c];
        };
        int pos_ahead[4], ahead_of = -1;
        auto issue = [&](Blk &B, int b) {
            const int4 e01 = *reinterpret_cast<const int4 *>(&ent[TILE_R * b + 4 * g]);
            const int4 e23 = *reinterpret_cast<const int4 *>(&ent[TILE_R * b + 4 * g + 2]);
            const int idxv[4] = {e01.x, e01.z, e23.x, e23.z};
            B.has = ((e01.y >> c) & 1) | (((e01.w >> c) & 1) << 1) | (((e23.y >> c) & 1) << 2) | (((e23.w >> c) & 1) << 3);
            int pos[4];
            if (b == ahead_of) {
#pragma unroll
                for (int r = 0; r < 4; ++r) pos[r] = pos_ahead[r];
            } else {
                positions(b, pos);
            }
            if (b + 1 < nblk) positions(b + 1, pos_ahead);
            ahead_of = b + 1;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t off = (uint32_t)idxv[r] * (uint32_t)RB + offc;
                B.qr[r] = *reinterpret_cast<const uint2 *>(qb + off);
                B.dr[r] = *reinterpret_cast<const uint2 *>(db + off);
                B.w[r] = pds_h[pos[r]];
            }
        };
        auto compute = [&](const Blk &B) {
            uint32_t w[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) w[r] = ((B.has >> r) & 1) ? B.w[r] : 0u;     // the scratch of pairs that do not exist is not initialised
            Bf4 pa, da;
            pa.u[0] = pack_lo16(w[0], w[1]); pa.u[1] = pack_lo16(w[2], w[3]);
            da.u[0] = pack_hi16(w[0], w[1]); da.u[1] = pack_hi16(w[2], w[3]);
            tile_axpy_bf16(da, B.qr, ak);
            tile_axpy_bf16(pa, B.dr, av);
        };
        tile_walk<PIPE, Blk>(nblk, issue, compute);
        wave_lds_fence();
    }
    tile_store_rows<H, D, false>(t, ak, 1.f, dk, ws_dk);
    tile_store_rows<H, D, false>(t, av, 1.f, dv, ws_dv);
}

// Backward, destination side.  Writes (p, ds) of every pair to pds[(t * H + head)], t = the pair's
// position (entry * R + member) in the SOURCE-side plan, which P.grp_pairs gives for every
// (entry, member) of this plan (a spare position for members the entry does not have).  One store per
// entry and quad of members: lane l carries the pair of member 4c + l % 4; the same register of ds values is
// the A operand of the MFMA that accumulates dq.  The members' q rows live in LDS.
template <typename T, int H, int D, int R, int HS, bool DROP, bool BIAS>
__global__ __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(grp_wpe<T, Lay<T, H / HS, D>::EPL, R>()))) void k_attn_bwd_dst_grp(
    bpt_plan P, const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v, const T *__restrict__ o,
    const T *__restrict__ d_o, const float *__restrict__ lse, T *__restrict__ dq, float2 *__restrict__ pds,
    float *__restrict__ ws_dq, float scale, float scale_log2e, uint32_t drop_thr, uint32_t drop_seed, float drop_inv,
    const float *__restrict__ bias, float *__restrict__ ds_out) {
    constexpr int HL = H / HS, CF = H * D;                  // heads of this wavefront's slice; elements of a full row
    using L = Lay<T, HL, D>;
    constexpr int EPL = L::EPL, NQ = R / 4, GRP_BATCH = BIAS ? 1 : grp_batch<L::EPL>()   /* the score term's registers take the place of a second entry */;
    static_assert(H % HS == 0 && R % 4 == 0 && L::LPH >= 4, "members are handled in quads inside the lanes of one head");
    GroupHead<R> gh;
    if (!fetch_group<R, HS>(P, gh)) return;
    const int slice = group_slice<R, HS>(), coff = slice * HL * D;
    const int lane = threadIdx.x, head = slice * HL + lane / L::LPH;
    const uint32_t loff = (uint32_t)((coff + L::off(lane, 0)) * sizeof(T));
    const int mine = lane & 3;
    const uint32_t hoff = (uint32_t)head * 8u, poff = (uint32_t)mine * 4u;
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
    struct Batch {
        RawRow<T, HL, D> kr[GRP_BATCH], vr[GRP_BATCH];
        int mk[GRP_BATCH], pz[GRP_BATCH], xp[GRP_BATCH][NQ];
        int xl[GRP_BATCH][BIAS ? NQ : 1];           // edge id of (entry, member 4c + lane % 4): where ds_out gets this lane's ds
        float bz[GRP_BATCH][BIAS ? NQ : 1];         // score term of (entry, member 4c + lane % 4), this lane's head
    };
    const int4 *eids4 = reinterpret_cast<const int4 *>(P.grp_eids);
    __shared__ float4 q_lds[R * (EPL / 4) * WAVE];
    float dov[R][EPL], delta_s[R], lse2[R];
    floatx4 dqa[NQ][EPL];                       // [quad c][row register t][member 4c + i], as the source-side kernel's accumulators
#pragma unroll
    for (int m = 0; m < R; ++m) {
        const uint32_t row = (uint32_t)max(gh.rows[m], 0);
        float ov[EPL], qr[EPL];
        load_row32<T, HL, D, CF>(o, row, loff, ov);
        load_row32<T, HL, D, CF>(d_o, row, loff, dov[m]);
        load_row32<T, HL, D, CF>(q, row, loff, qr);
        lds_put_row<EPL>(q_lds + m * (EPL / 4) * WAVE, lane, qr);
        delta_s[m] = head_sum<L::LPH>(dot_n<EPL>(dov[m], ov)) * scale;
        lse2[m] = lse[(size_t)row * H + head];
    }
#pragma unroll
    for (int c = 0; c < NQ; ++c)
#pragma unroll
        for (int t = 0; t < EPL; ++t) dqa[c][t] = floatx4{0.f, 0.f, 0.f, 0.f};
    for (int p0 = gh.begin; p0 < gh.end; p0 += GRP_CHUNK) {
        const int cnt = min(GRP_CHUNK, gh.end - p0);
        // lanes past the end repeat the last entry with an empty mask
        int4 ent = entries[p0 + min(lane, cnt - 1)];
        ent.y = lane < cnt ? ent.y : 0;
        // edge ids of the lane's entry, four members per vector (the list is padded like the entries)
        int4 xe[R / 4];
        if constexpr (BIAS || DROP) {
#pragma unroll
            for (int c = 0; c < R / 4; ++c) xe[c] = eids4[(size_t)(p0 + min(lane, cnt - 1)) * (R / 4) + c];
        }
        auto load_batch = [&](Batch &B, int b) {
#pragma unroll
            for (int e = 0; e < GRP_BATCH; ++e) {
                const uint32_t src = (uint32_t)__builtin_amdgcn_readlane(ent.x, b + e);
                B.mk[e] = __builtin_amdgcn_readlane(ent.y, b + e);
                B.pz[e] = DROP ? b + e : 0;                  // position of the entry in the chunk: the lane that holds its edge ids
                if constexpr (BIAS) {
#pragma unroll
                    for (int c = 0; c < R / 4; ++c) {
                        const uint32_t e0 = (uint32_t)__builtin_amdgcn_readlane(xe[c].x, b + e), e1 = (uint32_t)__builtin_amdgcn_readlane(xe[c].y, b + e);
                        const uint32_t e2 = (uint32_t)__builtin_amdgcn_readlane(xe[c].z, b + e), e3 = (uint32_t)__builtin_amdgcn_readlane(xe[c].w, b + e);
                        // lane l fetches the term of member 4c + l % 4; the quad's lanes hand it round when it is used
                        B.xl[e][c] = (int)(mine == 0 ? e0 : mine == 1 ? e1 : mine == 2 ? e2 : e3);
                        B.bz[e][c] = bias[(size_t)((uint32_t)B.xl[e][c] * (uint32_t)H) + head];
                    }
                }
                // lane l fetches the scratch positions of the pairs of members l % 4, 4 + l % 4, ... with this entry
                const char *pp = reinterpret_cast<const char *>(P.grp_pairs) + (size_t)((uint32_t)(p0 + b + e) * (uint32_t)(R * 4));
#pragma unroll
                for (int c = 0; c < NQ; ++c) B.xp[e][c] = *reinterpret_cast<const int *>(pp + (size_t)(poff + (uint32_t)(c * 16)));
                load_row32_raw<T, HL, D, CF>(k, src, loff, B.kr[e]);
                load_row32_raw<T, HL, D, CF>(v, src, loff, B.vr[e]);
            }
        };
        auto compute = [&](const Batch &B) {
#pragma unroll
            for (int e = 0; e < GRP_BATCH; ++e) {
                float kv[EPL], vv[EPL];
                unpack_row<T, HL, D>(B.kr[e], kv);
                unpack_row<T, HL, D>(B.vr[e], vv);
                float wp[NQ], wd[NQ];
#pragma unroll
                for (int c = 0; c < NQ; ++c) { wp[c] = 0.f; wd[c] = 0.f; }
#pragma unroll
                for (int m = 0; m < R; ++m) {
                    if ((B.mk[e] >> m) & 1) {
                        float qm[EPL];
                        lds_get_row<EPL>(q_lds + m * (EPL / 4) * WAVE, lane, qm);
                        float s = dot_n<EPL>(qm, kv), dp = dot_n<EPL>(dov[m], vv);
                        head_sum2<L::LPH>(s, dp);
                        if constexpr (BIAS) s += quad_bcast(B.bz[e][BIAS ? m / 4 : 0], m);
                        float pe = __builtin_amdgcn_exp2f(fmaf(s, scale_log2e, -lse2[m]));
                        float mt = 1.f;                   // dropout multiplier of this pair (as in the forward kernel)
                        if constexpr (DROP) {
                            const int4 &x = xe[m / 4];
                            const int held = (m & 3) == 0 ? x.x : (m & 3) == 1 ? x.y : (m & 3) == 2 ? x.z : x.w;
                            const uint32_t edge = (uint32_t)__builtin_amdgcn_readlane(held, B.pz[e]);
                            mt = dropout_keep(edge * (uint32_t)H + (uint32_t)head, drop_seed, drop_thr, drop_inv);
                        }
                        const float ds = pe * fmaf(dp * mt, scale, -delta_s[m]);
                        pe *= mt;                         // what multiplies v (forward) and dO (dV)
                        wp[m / 4] = mine == (m & 3) ? pe : wp[m / 4];
                        wd[m / 4] = mine == (m & 3) ? ds : wd[m / 4];
                    }
                }
#pragma unroll
                for (int c = 0; c < NQ; ++c) {
                    if ((B.mk[e] >> (4 * c)) & 15) {      // (look-ahead batches past the group's end have empty masks)
                        char *w = reinterpret_cast<char *>(pds);
                        *reinterpret_cast<float2 *>(w + (size_t)((uint32_t)B.xp[e][c] * (uint32_t)(H * 8) + hoff)) = make_float2(wp[c], wd[c]);
                        // dL/d(score before scaling) in edge order (absent members write the spare row n_edges)
                        if constexpr (BIAS) ds_out[(size_t)((uint32_t)B.xl[e][c] * (uint32_t)H) + head] = wd[c];
                        // dq[member 4c + i] += ds[member] * k row: wd (0 for absent members) is the A operand
#pragma unroll
                        for (int t = 0; t < EPL; ++t) dqa[c][t] = __builtin_amdgcn_mfma_f32_4x4x1f32(wd[c], kv[t], dqa[c][t], 0, 0, 0);
                    }
                }
            }
        };
        // two-stage software pipeline: the rows of the next batch are in flight while one is used.  The loads
        // are unconditional (a branch around them would make the compiler drain the load queue at the join);
        // look-ahead past the end re-reads the chunk's last entry with an empty mask.
        Batch A, B;
        load_batch(A, 0);
        for (int b = 0; b < cnt; b += 2 * GRP_BATCH) {
            load_batch(B, b + GRP_BATCH);
            issue_loads_first();
            compute(A);
            issue_loads_first();
            load_batch(A, b + 2 * GRP_BATCH);
            issue_loads_first();
            compute(B);
            issue_loads_first();
        }
    }
#pragma unroll
    for (int m = 0; m < R; ++m) {
        if (gh.rows[m] < 0) continue;
        float rq[EPL];
#pragma unroll
        for (int t = 0; t < EPL; ++t) rq[t] = dqa[m / 4][t][m & 3];
        if (gh.slots[m] < 0) store_row<T, HL, D>(dq + (size_t)gh.rows[m] * CF + coff, lane, rq);
        else store_row_ws<T, HL, D>(ws_dq + (size_t)gh.slots[m] * CF + coff, lane, rq);
    }
}

// Backward, source side: dK[src] = sum ds * q[dst], dV[src] = sum p * dO[dst]; the (p, ds) of the pair
// (entry u, member m) of this plan sits at pds[(u * R + m) * H + head].  One load per entry and quad of
// members: lane l fetches the pair of member 4c + l % 4 for its head.  That is the A operand of
// v_mfma_f32_4x4x1 (16 blocks of 4 lanes: A_b[i] in lane 4b+i, B_b[j] in lane 4b+j, D_b[i][j] in register i
// of lane 4b+j): with a register of the entry's row as B, one instruction adds weight[member i] * row[..]
// to that register's slice of all four members' accumulators (register i of the result = member i).
template <typename T, int H, int D, int R, int HS>
__global__ __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(grp_wpe<T, Lay<T, H / HS, D>::EPL, R>()))) void k_attn_bwd_src_grp(
    bpt_plan P, const T *__restrict__ q, const T *__restrict__ d_o, const float2 *__restrict__ pds, T *__restrict__ dk,
    T *__restrict__ dv, float *__restrict__ ws_dk, float *__restrict__ ws_dv) {
    constexpr int HL = H / HS, CF = H * D;                  // heads of this wavefront's slice; elements of a full row
    using L = Lay<T, HL, D>;
    constexpr int EPL = L::EPL, NQ = R / 4, GRP_BATCH = grp_batch<L::EPL>();
    static_assert(H % HS == 0 && R % 4 == 0 && L::LPH >= 4, "members are handled in quads inside the lanes of one head");
    GroupHead<R> gh;
    if (!fetch_group<R, HS>(P, gh)) return;
    const int slice = group_slice<R, HS>(), coff = slice * HL * D;
    const int lane = threadIdx.x, head = slice * HL + lane / L::LPH;
    const uint32_t loff = (uint32_t)((coff + L::off(lane, 0)) * sizeof(T));
    const uint32_t woff = (uint32_t)(((lane & 3) * H + head) * 8);
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
    struct Batch {
        RawRow<T, HL, D> qr[GRP_BATCH], dr[GRP_BATCH];
        float2 w[GRP_BATCH][NQ];
        int mk[GRP_BATCH];
    };
    floatx4 ak[NQ][EPL], av[NQ][EPL];          // [quad c][row register t][member 4c + i]
#pragma unroll
    for (int c = 0; c < NQ; ++c)
#pragma unroll
        for (int t = 0; t < EPL; ++t) { ak[c][t] = floatx4{0.f, 0.f, 0.f, 0.f}; av[c][t] = floatx4{0.f, 0.f, 0.f, 0.f}; }
    for (int p0 = gh.begin; p0 < gh.end; p0 += GRP_CHUNK) {
        const int cnt = min(GRP_CHUNK, gh.end - p0);
        // lanes past the end repeat the last entry with an empty mask
        int4 ent = entries[p0 + min(lane, cnt - 1)];
        ent.y = lane < cnt ? ent.y : 0;
        auto load_batch = [&](Batch &B, int b) {
#pragma unroll
            for (int e = 0; e < GRP_BATCH; ++e) {
                const uint32_t dst = (uint32_t)__builtin_amdgcn_readlane(ent.x, b + e);
                B.mk[e] = __builtin_amdgcn_readlane(ent.y, b + e);
                load_row32_raw<T, HL, D, CF>(q, dst, loff, B.qr[e]);
                load_row32_raw<T, HL, D, CF>(d_o, dst, loff, B.dr[e]);
                // the entry's R pairs, present or not (absent ones are zeroed before use)
                const char *pw = reinterpret_cast<const char *>(pds) + (size_t)((uint32_t)(p0 + b + e) * (uint32_t)(R * H * 8));
#pragma unroll
                for (int c = 0; c < NQ; ++c) B.w[e][c] = *reinterpret_cast<const float2 *>(pw + (size_t)(woff + (uint32_t)(c * 4 * H * 8)));
            }
        };
        auto compute = [&](const Batch &B) {
#pragma unroll
            for (int e = 0; e < GRP_BATCH; ++e) {
                float qv[EPL], dv_[EPL];
                unpack_row<T, HL, D>(B.qr[e], qv);
                unpack_row<T, HL, D>(B.dr[e], dv_);
#pragma unroll
                for (int c = 0; c < NQ; ++c) {
                    if ((B.mk[e] >> (4 * c)) & 15) {
                        // all-ones where this lane's member has the edge: the scratch of absent pairs is not initialised
                        const int keep = __builtin_amdgcn_sbfe(B.mk[e], 4 * c + (lane & 3), 1);
                        const float pe = __int_as_float(__float_as_int(B.w[e][c].x) & keep);
                        const float ds = __int_as_float(__float_as_int(B.w[e][c].y) & keep);
#pragma unroll
                        for (int t = 0; t < EPL; ++t) {
                            ak[c][t] = __builtin_amdgcn_mfma_f32_4x4x1f32(ds, qv[t], ak[c][t], 0, 0, 0);
                            av[c][t] = __builtin_amdgcn_mfma_f32_4x4x1f32(pe, dv_[t], av[c][t], 0, 0, 0);
                        }
                    }
                }
            }
        };
        // two-stage software pipeline: the rows of the next batch are in flight while one is used.  The loads
        // are unconditional (a branch around them would make the compiler drain the load queue at the join);
        // look-ahead past the end re-reads the chunk's last entry with an empty mask.
        Batch A, B;
        load_batch(A, 0);
        for (int b = 0; b < cnt; b += 2 * GRP_BATCH) {
            load_batch(B, b + GRP_BATCH);
            issue_loads_first();
            compute(A);
            issue_loads_first();
            load_batch(A, b + 2 * GRP_BATCH);
            issue_loads_first();
            compute(B);
            issue_loads_first();
        }
    }
#pragma unroll
    for (int m = 0; m < R; ++m) {
        if (gh.rows[m] < 0) continue;
        float rk[EPL], rv[EPL];
#pragma unroll
        for (int t = 0; t < EPL; ++t) { rk[t] = ak[m / 4][t][m & 3]; rv[t] = av[m / 4][t][m & 3]; }
        if (gh.slots[m] < 0) {
            store_row<T, HL, D>(dk + (size_t)gh.rows[m] * CF + coff, lane, rk);
            store_row<T, HL, D>(dv + (size_t)gh.rows[m] * CF + coff, lane, rv);
        } else {
            store_row_ws<T, HL, D>(ws_dk + (size_t)gh.slots[m] * CF + coff, lane, rk);
            store_row_ws<T, HL, D>(ws_dv + (size_t)gh.slots[m] * CF + coff, lane, rv);
        }
    }
}

// Y[row] = sum over the row's edges of W[eid, head] * X[idx]: the row-group form of k_spmm_fast for the unfused ops.
// X[idx] is loaded once per entry for every member that has the edge; the weight of (entry, member 4c + lane % 4) is
// fetched by its edge id (grp_eids) and is the A operand of v_mfma_f32_4x4x1 exactly as in k_attn_bwd_src_grp.
template <typename T, int H, int D, int R, int HS>
__global__ __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(grp_wpe<T, Lay<T, H / HS, D>::EPL, R>()))) void k_spmm_grp(
    bpt_plan P, const T *__restrict__ W, const T *__restrict__ X, T *__restrict__ Y, float *__restrict__ ws, int accumulate) {
    constexpr int HL = H / HS, CF = H * D;                  // heads of this wavefront's slice; elements of a full row
    using L = Lay<T, HL, D>;
    constexpr int EPL = L::EPL, NQ = R / 4, GRP_BATCH = grp_batch<L::EPL>();
    static_assert(H % HS == 0 && R % 4 == 0 && L::LPH >= 4, "members are handled in quads inside the lanes of one head");
    GroupHead<R> gh;
    if (!fetch_group<R, HS>(P, gh)) return;
    const int slice = group_slice<R, HS>(), coff = slice * HL * D;
    const int lane = threadIdx.x, head = slice * HL + lane / L::LPH, mine = lane & 3;
    const uint32_t loff = (uint32_t)((coff + L::off(lane, 0)) * sizeof(T));
    const uint32_t last_edge = (uint32_t)max(P.n_edges, (int64_t)1) - 1u;
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
    const int4 *eids4 = reinterpret_cast<const int4 *>(P.grp_eids);
    struct Batch {
        RawRow<T, HL, D> xr[GRP_BATCH];
        float w[GRP_BATCH][NQ];
        int mk[GRP_BATCH];
    };
    floatx4 acc[NQ][EPL];                      // [quad c][row register t][member 4c + i]
#pragma unroll
    for (int c = 0; c < NQ; ++c)
#pragma unroll
        for (int t = 0; t < EPL; ++t) acc[c][t] = floatx4{0.f, 0.f, 0.f, 0.f};
    for (int p0 = gh.begin; p0 < gh.end; p0 += GRP_CHUNK) {
        const int cnt = min(GRP_CHUNK, gh.end - p0);
        // lanes past the end repeat the last entry with an empty mask
        int4 ent = entries[p0 + min(lane, cnt - 1)];
        ent.y = lane < cnt ? ent.y : 0;
        // edge ids of the lane's entry, four members per vector
        int4 xe[R / 4];
#pragma unroll
        for (int c = 0; c < R / 4; ++c) xe[c] = eids4[(size_t)(p0 + min(lane, cnt - 1)) * (R / 4) + c];
        auto load_batch = [&](Batch &B, int b) {
#pragma unroll
            for (int e = 0; e < GRP_BATCH; ++e) {
                const uint32_t src = (uint32_t)__builtin_amdgcn_readlane(ent.x, b + e);
                B.mk[e] = __builtin_amdgcn_readlane(ent.y, b + e);
#pragma unroll
                for (int c = 0; c < NQ; ++c) {
                    const uint32_t e0 = (uint32_t)__builtin_amdgcn_readlane(xe[c].x, b + e), e1 = (uint32_t)__builtin_amdgcn_readlane(xe[c].y, b + e);
                    const uint32_t e2 = (uint32_t)__builtin_amdgcn_readlane(xe[c].z, b + e), e3 = (uint32_t)__builtin_amdgcn_readlane(xe[c].w, b + e);
                    // absent members carry the id n_edges: read the last edge instead, the mask zeroes the weight
                    const uint32_t el = min(mine == 0 ? e0 : mine == 1 ? e1 : mine == 2 ? e2 : e3, last_edge);
                    B.w[e][c] = ld_w(W + (size_t)el * H + head);
                }
                load_row32_raw<T, HL, D, CF>(X, src, loff, B.xr[e]);
            }
        };
        auto compute = [&](const Batch &B) {
#pragma unroll
            for (int e = 0; e < GRP_BATCH; ++e) {
                float xv[EPL];
                unpack_row<T, HL, D>(B.xr[e], xv);
#pragma unroll
                for (int c = 0; c < NQ; ++c) {
                    if ((B.mk[e] >> (4 * c)) & 15) {
                        const int keep = __builtin_amdgcn_sbfe(B.mk[e], 4 * c + mine, 1);     // all-ones where the member has the edge
                        const float wt = __int_as_float(__float_as_int(B.w[e][c]) & keep);
#pragma unroll
                        for (int t = 0; t < EPL; ++t) acc[c][t] = __builtin_amdgcn_mfma_f32_4x4x1f32(wt, xv[t], acc[c][t], 0, 0, 0);
                    }
                }
            }
        };
        // two-stage software pipeline as in the fused kernels (unconditional loads; look-ahead past the end re-reads
        // the chunk's last entry with an empty mask)
        Batch A, B;
        load_batch(A, 0);
        for (int b = 0; b < cnt; b += 2 * GRP_BATCH) {
            load_batch(B, b + GRP_BATCH);
            issue_loads_first();
            compute(A);
            issue_loads_first();
            load_batch(A, b + 2 * GRP_BATCH);
            issue_loads_first();
            compute(B);
            issue_loads_first();
        }
    }
#pragma unroll
    for (int m = 0; m < R; ++m) {
        if (gh.rows[m] < 0) continue;
        float out[EPL];
#pragma unroll
        for (int t = 0; t < EPL; ++t) out[t] = acc[m / 4][t][m & 3];
        if (gh.slots[m] < 0) {
            if (accumulate) {                 // Y += the sum (rows in segments get theirs when the segments are combined)
                float old[EPL];
                load_row32<T, HL, D, CF>(Y, (uint32_t)gh.rows[m], loff, old);
#pragma unroll
                for (int t = 0; t < EPL; ++t) out[t] += old[t];
            }
            store_row<T, HL, D>(Y + (size_t)gh.rows[m] * CF + coff, lane, out);
        } else {
            store_row_ws<T, HL, D>(ws + (size_t)gh.slots[m] * CF + coff, lane, out);
        }
    }
}

// y[eid, head] = <A[row, head, :], B[idx, head, :]> for every edge: the row-group form of k_sddmm_fast.  The
// members' A rows stay in registers, B[idx] is loaded once per entry and every member that has the edge takes its
// dot products with it; the edge id of (entry, member) comes from grp_eids.  TABLE: B is a (n, D) table whose rows
// all heads share (the rel_pos score term q[row] . table[idx], written as float32).
template <typename T, int H, int D, int R, int HS, bool TABLE = false, typename YT = T>
__global__ __launch_bounds__(WAVE) void k_sddmm_grp(bpt_plan P, const T *__restrict__ A, const T *__restrict__ B, YT *__restrict__ y) {
    constexpr int HL = H / HS, CF = H * D;                  // heads of this wavefront's slice; elements of a full row
    using L = Lay<T, HL, D>;
    constexpr int EPL = L::EPL, GRP_BATCH = 2;
    static_assert(H % HS == 0 && R % 4 == 0, "edge ids come four members per vector");
    GroupHead<R> gh;
    if (!fetch_group<R, HS>(P, gh)) return;
    const int slice = group_slice<R, HS>(), coff = slice * HL * D;
    const int lane = threadIdx.x, head = slice * HL + lane / L::LPH;
    const uint32_t loff = (uint32_t)((coff + L::off(lane, 0)) * sizeof(T));
    const uint32_t toff = (uint32_t)((lane % L::LPH) * L::VE * sizeof(T));      // the lane's columns inside a table row
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
    const int4 *eids4 = reinterpret_cast<const int4 *>(P.grp_eids);
    float a[R][EPL];
#pragma unroll
    for (int m = 0; m < R; ++m) load_row32<T, HL, D, CF>(A, (uint32_t)max(gh.rows[m], 0), loff, a[m]);
    struct Batch {
        RawRow<T, HL, D> br[GRP_BATCH];
        int mk[GRP_BATCH], pz[GRP_BATCH];
    };
    for (int p0 = gh.begin; p0 < gh.end; p0 += GRP_CHUNK) {
        const int cnt = min(GRP_CHUNK, gh.end - p0);
        // lanes past the end repeat the last entry with an empty mask
        int4 ent = entries[p0 + min(lane, cnt - 1)];
        ent.y = lane < cnt ? ent.y : 0;
        int4 xe[R / 4];                                     // edge ids of the lane's entry, four members per vector
#pragma unroll
        for (int c = 0; c < R / 4; ++c) xe[c] = eids4[(size_t)(p0 + min(lane, cnt - 1)) * (R / 4) + c];
        auto load_batch = [&](Batch &Bt, int b) {
#pragma unroll
            for (int e = 0; e < GRP_BATCH; ++e) {
                const uint32_t src = (uint32_t)__builtin_amdgcn_readlane(ent.x, b + e);
                Bt.mk[e] = __builtin_amdgcn_readlane(ent.y, b + e);
                Bt.pz[e] = b + e;
                if constexpr (TABLE) load_row32_raw<T, HL, D, D>(B, src, toff, Bt.br[e]);
                else load_row32_raw<T, HL, D, CF>(B, src, loff, Bt.br[e]);
            }
        };
        auto compute = [&](const Batch &Bt) {
#pragma unroll
            for (int e = 0; e < GRP_BATCH; ++e) {
                float bv[EPL];
                unpack_row<T, HL, D>(Bt.br[e], bv);
#pragma unroll
                for (int m = 0; m < R; ++m) {
                    if ((Bt.mk[e] >> m) & 1) {
                        const float s = head_sum<L::LPH>(dot_n<EPL>(a[m], bv));
                        const int4 &x = xe[m / 4];
                        const int held = (m & 3) == 0 ? x.x : (m & 3) == 1 ? x.y : (m & 3) == 2 ? x.z : x.w;
                        const uint32_t edge = (uint32_t)__builtin_amdgcn_readlane(held, Bt.pz[e]);
                        if (lane % L::LPH == 0) Elem<YT>::st(y + (size_t)edge * H + head, s);
                    }
                }
            }
        };
        // two-stage software pipeline as in the fused kernels (unconditional loads; look-ahead past the end re-reads
        // the chunk's last entry with an empty mask)
        Batch X0, X1;
        load_batch(X0, 0);
        for (int b = 0; b < cnt; b += 2 * GRP_BATCH) {
            load_batch(X1, b + GRP_BATCH);
            issue_loads_first();
            compute(X0);
            issue_loads_first();
            load_batch(X0, b + 2 * GRP_BATCH);
            issue_loads_first();
            compute(X1);
            issue_loads_first();
        }
    }
}

// ------------------------------------------------------------------------------------------
// rel_pos score term (modules/attention.py:69-71) over the plan of the destinations with the edge types as indices: the
// table's rows are shared by all heads and few (at most 1000, 64 columns), so the products go to the matrix cores.
// ------------------------------------------------------------------------------------------
// 16 consecutive elements as floats
template <typename T> __device__ __forceinline__ void rel_load16(const T *p, float (&out)[16]);
template <> __device__ __forceinline__ void rel_load16<float>(const float *p, float (&out)[16]) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const float4 x = *reinterpret_cast<const float4 *>(p + 4 * t);
        out[4 * t] = x.x; out[4 * t + 1] = x.y; out[4 * t + 2] = x.z; out[4 * t + 3] = x.w;
    }
}
template <> __device__ __forceinline__ void rel_load16<bf16_t>(const bf16_t *p, float (&out)[16]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const uint4 x = *reinterpret_cast<const uint4 *>(reinterpret_cast<const char *>(p) + 16 * t);
        const uint32_t w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[8 * t + 2 * i] = __uint_as_float(w[i] << 16);
            out[8 * t + 2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
}

// A work item (a row or a segment of a long row) and the types and edge ids of its first 64 slots (lane l: slot b + l).
struct RelHead {
    int row, b, e, out_slot;
    int type, edge;
};
__device__ __forceinline__ void rel_head_load(const bpt_plan &P, const int4 item, int lane, RelHead &r) {
    // the item is the same for all lanes of the wavefront: keep it in scalar registers
    r.row = __builtin_amdgcn_readfirstlane(item.x); r.b = __builtin_amdgcn_readfirstlane(item.y);
    r.e = __builtin_amdgcn_readfirstlane(item.z); r.out_slot = __builtin_amdgcn_readfirstlane(item.w);
    const int slot = r.b + min(lane, max(min(WAVE, r.e - r.b), 1) - 1);        // lanes past the end repeat the last slot
    r.type = r.b < r.e ? P.idx[slot] : 0;
    r.edge = r.b < r.e ? P.eid[slot] : 0;
}

// The rows of the table that a graph uses, as floats in LDS: row u (`pitch` floats apart) = table[used_types[u]].  All
// threads of the workgroup.
template <typename T>
__device__ __forceinline__ void rel_table_to_lds(const T *__restrict__ table, const int32_t *__restrict__ used_types, int n_used, float *lds,
                                                 int pitch) {
    for (int x = threadIdx.x; x < n_used * 16; x += blockDim.x) {
        const int u = x >> 4, c4 = (x & 15) * 4;
        *reinterpret_cast<float4 *>(lds + u * pitch + c4) = load4<T>(table + (size_t)used_types[u] * 64 + c4);
    }
}

// bias[eid[p], head] = q[row(p), head, :] . table[used_types[idx[p]], :] for every slot p of the plan (idx = the number of
// the edge's type among the n_used types that occur).  The heads of an item's row are rows of the A operand of
// v_mfma_f32_16x16x4f32 (row number c of A = head c % H), 16 consecutive slots of the item the 16 columns of B; lane
// (g, c) holds columns 16 g .. 16 g + 15 of q for head c % H and of the table row of slot c, and receives the results of
// heads 4 g .. 4 g + 3 for slot c, which it stores as one vector where 4 g < H.  The table rows come from a copy in LDS
// (rows REL_LDS_PITCH floats apart, so that the 16 rows of an operand fall into different banks): fetched from memory
// block by block they would cost one round trip each, far longer than a block's products.  A wavefront takes
// REL_FWD_ITEMS work items and fetches for all of them at once first the items, then their q rows and the type numbers
// and edge ids of their first 64 slots.
constexpr int REL_FWD_ITEMS = 4, REL_LDS_PITCH = 68;
template <typename T, int H>
__global__ __launch_bounds__(BLOCK) void k_rel_bias_rows(bpt_plan P, const T *__restrict__ q, const T *__restrict__ table,
                                                         const int32_t *__restrict__ used_types, int n_used, float *__restrict__ bias) {
    constexpr int D = 64, K = REL_FWD_ITEMS;
    static_assert(H == 4 || H == 8 || H == 16, "four consecutive heads per lane");
    extern __shared__ float rel_lds[];
    const int lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;
    // wavefront gw of GW takes the items gw, gw + GW, ...: the segments of a long row, which are neighbours and all full, go to
    // different wavefronts
    const int GW = (int)gridDim.x * WAVES_PER_BLOCK, i0 = (int)blockIdx.x * WAVES_PER_BLOCK + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int n_items = (int)P.n_items;
    const int4 *items = reinterpret_cast<const int4 *>(P.items);
    int4 desc[K];
#pragma unroll
    for (int k = 0; k < K; ++k) desc[k] = items[min(i0 + k * GW, n_items - 1)];
    rel_table_to_lds<T>(table, used_types, n_used, rel_lds, REL_LDS_PITCH);
    const bool head_major = P.bias_by_pair != 0;                // results at bias[head * n_edges + eid] instead of bias[eid * H + head]
    if (blockIdx.x == 0 && threadIdx.x < H && !head_major) bias[(size_t)P.n_edges * H + threadIdx.x] = 0.f;     // the spare row the fused kernels read for absent pairs
    RelHead hd[K];
    float aq[K][16];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (i0 + k * GW >= n_items) desc[k].z = desc[k].y;  // (past the last item: nothing to do)
        rel_head_load(P, desc[k], lane, hd[k]);
        rel_load16<T>(q + ((size_t)hd[k].row * H + (c % H)) * D + 16 * g, aq[k]);
    }
    __syncthreads();
    auto table_rows = [&](int type, int first, float (&bt)[16]) {          // of the 16 slots from `first` of a chunk (lane l: slot l)
        const float *row = rel_lds + lane_bcast(type, first + c) * REL_LDS_PITCH + 16 * g;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float4 x = *reinterpret_cast<const float4 *>(row + 4 * t);
            bt[4 * t] = x.x; bt[4 * t + 1] = x.y; bt[4 * t + 2] = x.z; bt[4 * t + 3] = x.w;
        }
    };
#pragma unroll
    for (int k = 0; k < K; ++k) {
        for (int p0 = hd[k].b; p0 < hd[k].e; p0 += WAVE) {
            const int cnt = min(WAVE, hd[k].e - p0);
            int type = hd[k].type, edge = hd[k].edge;
            if (p0 != hd[k].b) {                             // (items longer than 64 slots: the rest, fetched on the spot)
                const int slot = p0 + min(lane, cnt - 1);
                type = P.idx[slot]; edge = P.eid[slot];
            }
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                if (16 * blk < cnt) {
                    float bt[16];
                    table_rows(type, 16 * blk, bt);
                    const floatx4v acc = tile_dot(aq[k], bt);
                    const int e = lane_bcast(edge, 16 * blk + c);
                    if (16 * blk + c < cnt && 4 * g < H) {
                        if (head_major) {
#pragma unroll
                            for (int r = 0; r < 4; ++r) bias[(size_t)(4 * g + r) * (size_t)P.n_edges + e] = acc[r];
                        } else {
                            *reinterpret_cast<float4 *>(bias + (size_t)e * H + 4 * g) = make_float4(acc[0], acc[1], acc[2], acc[3]);
                        }
                    }
                }
            }
        }
    }
}

// The same term over the TILE plan of the attention kernels, for a term kept in that plan's pair order (bias_by_pair:
// one value per pair and head at bias[head * n_edges + pair number]).  One wavefront per (tile, head), as in the attention
// kernels.  First the products of the tile's 16 member rows with every table row in use, QT[type number][member] (16
// type numbers per step: A = table rows, B = the members' q), which go to a wavefront-private piece of LDS; then the
// lanes walk the tile's pairs, which are consecutive numbers, and every pair picks its value by what pair_tm[number] =
// type number | member << 8 says.  The per-pair arrays are read and written in runs; the table rows in use are staged in
// LDS once per workgroup (fetched from memory step by step, each step waits for two dependent loads: 32 us against
// the products' 7).
template <typename T>
__device__ __forceinline__ void rel_cols16(const T *row, int g, float (&out)[16]) {     // columns 16 t + 4 g + e of a 64-column row
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const float4 x = load4<T>(row + 16 * t + 4 * g);
        out[4 * t] = x.x; out[4 * t + 1] = x.y; out[4 * t + 2] = x.z; out[4 * t + 3] = x.w;
    }
}
template <typename T, int H, int HW>
__global__ __launch_bounds__(HW * WAVE) void k_rel_bias_tiles(bpt_plan P, const T *__restrict__ q, const T *__restrict__ table,
                                                              const int32_t *__restrict__ used_types, int n_used,
                                                              const int32_t *__restrict__ pair_tm, float *__restrict__ bias) {
    constexpr int D = 64, C = H * D;
    extern __shared__ float rel_lds[];                        // the table rows in use, then QT of every wavefront
    const int n16 = (n_used + 15) & ~15;
    rel_table_to_lds<T>(table, used_types, n_used, rel_lds, REL_LDS_PITCH);
    TileCtx t;
    const bool mine = tile_begin<T, H, D, HW>(P, t) && t.p_begin < t.p_end;
    __syncthreads();
    if (!mine) return;
    float *qt = rel_lds + (size_t)n_used * REL_LDS_PITCH + (size_t)t.wv * n16 * TILE_R;
    auto table_rows = [&](int tb, float (&out)[16]) {           // of type numbers tb + c: this lane's columns
        const float *row = rel_lds + min(tb + t.c, n_used - 1) * REL_LDS_PITCH + 4 * t.g;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 x = *reinterpret_cast<const float4 *>(row + 16 * i);
            out[4 * i] = x.x; out[4 * i + 1] = x.y; out[4 * i + 2] = x.z; out[4 * i + 3] = x.w;
        }
    };
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
    const int4 last = entries[t.p_end - 1];
    const int first = __builtin_amdgcn_readfirstlane(entries[t.p_begin].z), end = __builtin_amdgcn_readfirstlane(last.z + __popc((uint32_t)last.y));
    if (end <= first) return;
    constexpr int AHEAD = 4;                                    // pairs per lane whose loads are in flight together
    int tm[AHEAD];
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) tm[k] = pair_tm[min(first + t.lane + k * WAVE, end - 1)];
    float qb[16];
    rel_cols16<T>(q + (size_t)max(t.member.x, 0) * C + t.head * D, t.g, qb);
    for (int tb = 0; tb < n16; tb += TILE_R) {
        float kr[16];
        table_rows(tb, kr);
        const floatx4v st = tile_dot(kr, qb);                   // register r: (type number tb + 4 g + r, member c)
#pragma unroll
        for (int r = 0; r < 4; ++r) qt[(tb + 4 * t.g + r) * TILE_R + t.c] = st[r];
    }
    wave_lds_fence();
    float *out = bias + (size_t)t.head * (size_t)P.n_edges;
    for (int x = first + t.lane; x < end; x += AHEAD * WAVE) {
        int nt[AHEAD];
#pragma unroll
        for (int k = 0; k < AHEAD; ++k) nt[k] = pair_tm[min(x + (AHEAD + k) * WAVE, end - 1)];
        float val[AHEAD];
#pragma unroll
        for (int k = 0; k < AHEAD; ++k) val[k] = qt[(tm[k] & 0xff) * TILE_R + (tm[k] >> 8)];
        // (the next round's loads are waited for before this round's stores: behind them the wait would include the stores)
#pragma unroll
        for (int k = 0; k < AHEAD; ++k) asm volatile("" ::"v"(nt[k]));
#pragma unroll
        for (int k = 0; k < AHEAD; ++k) {
            if (x + k * WAVE < end) out[x + k * WAVE] = val[k];
            tm[k] = nt[k];
        }
    }
}

// Gradients of that term from ds[e, head] = dL/d(score of edge e before scaling): dq[row] += sum over the row's slots of
// ds[eid] * table row of the slot's type (all heads), and the table's gradient, for type number u, the sum over the slots
// with idx = u and the heads of ds[eid, head] * q[row, head].  Lane l owns column l.  Each wavefront walks every GW-th of
// the plan's work items (rows and segments of long rows; a segment's part of dq goes to the workspace slot of the item,
// which k_combine_sum_v4 adds to dq) and keeps its own sums per type number in LDS, beside the workgroup's copy of the
// table rows in use; the wavefronts of a workgroup add theirs in a fixed order and the workgroup writes one partial
// table, part[(u * gridDim.x + block) * 64 + column], which k_rel_table_sum adds up.  Every sum has one owner and a fixed
// order.  The loads of an item run ahead of its use in three steps (descriptor; type numbers and edge ids of its first 64
// slots; their ds values and the item's q and dq rows), each one item further ahead than the one that needs its result.
template <int H>
struct RelBody {             // what the walk of those slots needs: per lane the ds values of its slot; the item's q row
    float dsv[H];            // and, for a whole row, the dq row it adds to (lane l: column l)
    float qh[H], old[H];
};
// the H values of ds that belong to `edge`: a row of (n_edges, H), or with head_major one of each head's n_edges values
template <int H>
__device__ __forceinline__ void rel_ds_load(const float *__restrict__ ds, int edge, bool head_major, size_t n_edges, float (&out)[H]) {
    if (head_major) {
#pragma unroll
        for (int h = 0; h < H; ++h) out[h] = ds[(size_t)h * n_edges + edge];
    } else {
#pragma unroll
        for (int h = 0; h < H; h += 4) {
            const float4 x = *reinterpret_cast<const float4 *>(ds + (size_t)edge * H + h);
            out[h] = x.x; out[h + 1] = x.y; out[h + 2] = x.z; out[h + 3] = x.w;
        }
    }
}
template <typename T, int H>
__device__ __forceinline__ void rel_body_load(const RelHead &r, const float *__restrict__ ds, bool head_major, size_t n_edges, const T *__restrict__ q,
                                              const T *__restrict__ dq, int lane, RelBody<H> &y) {
    constexpr int D = 64;
    rel_ds_load<H>(ds, r.edge, head_major, n_edges, y.dsv);
#pragma unroll
    for (int h = 0; h < H; ++h) {
        y.qh[h] = Elem<T>::ld(q + ((size_t)r.row * H + h) * D + lane);
        y.old[h] = r.out_slot < 0 ? Elem<T>::ld(dq + ((size_t)r.row * H + h) * D + lane) : 0.f;
    }
}
template <typename T, int H, int NW>
__global__ __launch_bounds__(NW * WAVE) void k_rel_bias_bwd(bpt_plan P, const float *__restrict__ ds, const T *__restrict__ q,
                                                            const T *__restrict__ table, const int32_t *__restrict__ used_types, int n_used,
                                                            T *__restrict__ dq, float *__restrict__ ws_dq, float *__restrict__ part) {
    constexpr int D = 64, C = H * D, AHEAD = H >= 16 ? 4 : 8;
    extern __shared__ float rel_lds[];                    // NW tables of n_used x 64 sums, the table rows in use, NW x 64 x H staged ds values
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const bool head_major = P.bias_by_pair != 0;                // ds[head * n_edges + eid] instead of ds[eid * H + head]
    float *acc = rel_lds + (size_t)w * n_used * D;
    const float *rows = rel_lds + (size_t)NW * n_used * D;
    float *stage = rel_lds + (size_t)(NW + 1) * n_used * D + (size_t)w * WAVE * H;
    for (int u = 0; u < n_used; ++u) acc[u * D + lane] = 0.f;
    rel_table_to_lds<T>(table, used_types, n_used, rel_lds + (size_t)NW * n_used * D, D);
    // wavefront gw of GW takes the items gw, gw + GW, ...: the segments of a long row, which are neighbours, go to different wavefronts
    const int GW = (int)gridDim.x * NW, i_begin = (int)blockIdx.x * NW + w, i_end = (int)P.n_items;
    const int4 *items = reinterpret_cast<const int4 *>(P.items);
    const int4 none = make_int4(0, 0, 0, -1);             // (an empty row: nothing to read, nothing to write)
    RelHead hd, hd_next;
    RelBody<H> bd, bd_next;
    rel_head_load(P, i_begin < i_end ? items[i_begin] : none, lane, hd_next);
    rel_body_load<T, H>(hd_next, ds, head_major, (size_t)P.n_edges, q, dq, lane, bd_next);
    hd = hd_next;
    rel_head_load(P, i_begin + GW < i_end ? items[i_begin + GW] : none, lane, hd_next);
    int4 desc = i_begin + 2 * GW < i_end ? items[i_begin + 2 * GW] : none;
    __syncthreads();
    // one chunk of at most 64 slots whose ds values are staged: lane j of u (type numbers) belongs to slot j of the chunk
    auto walk = [&](int cnt, int u, const float (&qh)[H], float (&dqa)[H]) {
        wave_lds_fence();
        for (int j0 = 0; j0 < cnt; j0 += AHEAD) {
            // the ds values of AHEAD slots first (zeros are staged for the slots past the chunk's end, which so add nothing),
            // then four slots at a time: the sums so far and the table rows, the products, the new sums.  The reads of
            // the sums come before the products so that their latency is covered; where slots of a four have the same
            // type, the later one's sum takes the earlier ones' terms in slot order, as if the four were added one
            // after the other.
            float4 dv[AHEAD][H / 4];
#pragma unroll
            for (int x = 0; x < AHEAD; ++x)
#pragma unroll
                for (int h = 0; h < H; h += 4) dv[x][h / 4] = *reinterpret_cast<const float4 *>(stage + min(j0 + x, WAVE - 1) * H + h);
#pragma unroll
            for (int x0 = 0; x0 < AHEAD; x0 += 4) {
                if (j0 + x0 < cnt) {
                    int un[4];
                    float before[4], gsum[4], tv[4];
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        un[x] = __builtin_amdgcn_readlane(u, min(j0 + x0 + x, cnt - 1));
                        before[x] = acc[un[x] * D + lane];
                        tv[x] = rows[un[x] * D + lane];
                    }
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        gsum[x] = 0.f;
#pragma unroll
                        for (int h = 0; h < H; h += 4) {
                            const float4 d4 = dv[x0 + x][h / 4];
                            gsum[x] = fmaf(d4.x, qh[h], gsum[x]); gsum[x] = fmaf(d4.y, qh[h + 1], gsum[x]);
                            gsum[x] = fmaf(d4.z, qh[h + 2], gsum[x]); gsum[x] = fmaf(d4.w, qh[h + 3], gsum[x]);
                            dqa[h] = fmaf(d4.x, tv[x], dqa[h]); dqa[h + 1] = fmaf(d4.y, tv[x], dqa[h + 1]);
                            dqa[h + 2] = fmaf(d4.z, tv[x], dqa[h + 2]); dqa[h + 3] = fmaf(d4.w, tv[x], dqa[h + 3]);
                        }
                    }
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        float v = before[x];
#pragma unroll
                        for (int y = 0; y < x; ++y) v += un[y] == un[x] ? gsum[y] : 0.f;
                        acc[un[x] * D + lane] = v + gsum[x];
                    }
                }
            }
        }
        wave_lds_fence();
    };
    for (int i = i_begin; i < i_end; i += GW) {
        bd = bd_next;
        rel_body_load<T, H>(hd_next, ds, head_major, (size_t)P.n_edges, q, dq, lane, bd_next);                // the item after this one
        const RelHead cur = hd;
        hd = hd_next;
        rel_head_load(P, desc, lane, hd_next);                                   // the second after
        desc = i + 3 * GW < i_end ? items[i + 3 * GW] : none;
        float dqa[H];
#pragma unroll
        for (int h = 0; h < H; ++h) dqa[h] = 0.f;
        if (cur.b < cur.e) {
#pragma unroll
            for (int h = 0; h < H; h += 4)
                *reinterpret_cast<float4 *>(stage + lane * H + h) =
                    lane < cur.e - cur.b ? make_float4(bd.dsv[h], bd.dsv[h + 1], bd.dsv[h + 2], bd.dsv[h + 3]) : make_float4(0.f, 0.f, 0.f, 0.f);
            walk(min(WAVE, cur.e - cur.b), cur.type, bd.qh, dqa);
        }
        for (int p0 = cur.b + WAVE; p0 < cur.e; p0 += WAVE) {                  // (items longer than 64 slots: the rest, fetched on the spot)
            const int cnt = min(WAVE, cur.e - p0);
            const int slot = p0 + min(lane, cnt - 1);
            const int u = P.idx[slot], edge = P.eid[slot];
            float rest[H];
            rel_ds_load<H>(ds, edge, head_major, (size_t)P.n_edges, rest);
#pragma unroll
            for (int h = 0; h < H; h += 4)
                *reinterpret_cast<float4 *>(stage + lane * H + h) =
                    lane < cnt ? make_float4(rest[h], rest[h + 1], rest[h + 2], rest[h + 3]) : make_float4(0.f, 0.f, 0.f, 0.f);
            walk(cnt, u, bd.qh, dqa);
        }
        if (cur.out_slot < 0) {
            if (cur.b < cur.e) {
#pragma unroll
                for (int h = 0; h < H; ++h) Elem<T>::st(dq + ((size_t)cur.row * H + h) * D + lane, bd.old[h] + dqa[h]);
            }
        } else {
#pragma unroll
            for (int h = 0; h < H; ++h) ws_dq[(size_t)cur.out_slot * C + h * D + lane] = dqa[h];
        }
    }
    __syncthreads();
    for (int u = w; u < n_used; u += NW) {
        float sum = rel_lds[(size_t)u * D + lane];
#pragma unroll
        for (int x = 1; x < NW; ++x) sum += rel_lds[((size_t)x * n_used + u) * D + lane];
        part[((size_t)u * gridDim.x + blockIdx.x) * D + lane] = sum;
    }
}

// dtable[type] = the sum of the n_parts partial rows of the type's number u = used[type] (zero for a type that does
// not occur).  One workgroup per type; 16 lanes cover a row (four columns each), so a wavefront reads four partial rows
// per load: lane group s of wave w adds the rows 4 w + s, 4 w + s + 16, ...; the 16 sums are then added in a fixed order.
template <typename T>
__device__ __forceinline__ void rel_table_sum_block(int type, const float *__restrict__ part, const int32_t *__restrict__ used, int n_parts,
                                                    T *__restrict__ dtable) {
    constexpr int D = 64, GROUPS = BLOCK / 16;
    __shared__ float4 sums[GROUPS][16];
    const int u = used[type], grp = threadIdx.x >> 4, c4 = (threadIdx.x & 15) * 4;
    if (u < 0) {
        if (threadIdx.x < 16) store4<T>(dtable + (size_t)type * D + c4, make_float4(0.f, 0.f, 0.f, 0.f));
        return;
    }
    const float *p = part + (size_t)u * n_parts * D + c4;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    int x = grp;
    for (; x + 7 * GROUPS < n_parts; x += 8 * GROUPS) {
        float4 t[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) t[k] = *reinterpret_cast<const float4 *>(p + (size_t)(x + k * GROUPS) * D);
#pragma unroll
        for (int k = 0; k < 8; ++k) { s.x += t[k].x; s.y += t[k].y; s.z += t[k].z; s.w += t[k].w; }
    }
    for (; x < n_parts; x += GROUPS) {
        const float4 t = *reinterpret_cast<const float4 *>(p + (size_t)x * D);
        s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
    }
    sums[grp][threadIdx.x & 15] = s;
    __syncthreads();
    if (threadIdx.x < 16) {
        float4 tot = sums[0][threadIdx.x];
#pragma unroll
        for (int k = 1; k < GROUPS; ++k) { const float4 t = sums[k][threadIdx.x]; tot.x += t.x; tot.y += t.y; tot.z += t.z; tot.w += t.w; }
        store4<T>(dtable + (size_t)type * D + c4, tot);
    }
}

// What is left after k_rel_bias_bwd, in one launch of n_types + n_heavy * C / 256 workgroups: the first n_types sum
// the partial tables (above), the others add the partial dq rows of the split rows to dq (one workgroup per split row
// and strip of 256 columns, in the order combine_sum_block uses).
template <typename T>
__global__ __launch_bounds__(BLOCK) void k_rel_finish(const float *__restrict__ part, const int32_t *__restrict__ used, int n_parts, int n_types,
                                                      T *__restrict__ dtable, const int32_t *__restrict__ heavy, const float *__restrict__ ws_dq,
                                                      T *__restrict__ dq, int C) {
    const int b = blockIdx.x;
    if (b < n_types) {
        rel_table_sum_block<T>(b, part, used, n_parts, dtable);
    } else {
        const int strips = C / 256, x = b - n_types;
        combine_sum_block4<T>(heavy + 3 * (x / strips), ws_dq, dq, C, true, x % strips);
    }
}

// Measurement aid: what the memory system delivers to row gathers.  Every wavefront reads `iters` batches of
// IN_FLIGHT pseudo-random 1 KB rows (16 bytes per lane, the access pattern of the attention kernels' neighbour rows)
// of a region and keeps a checksum, so that nothing but the loads is timed.
template <int IN_FLIGHT>
__global__ __launch_bounds__(BLOCK) void k_gather_probe(const float4 *__restrict__ base, uint32_t n_rows, int iters, float *__restrict__ sink) {
    const int lane = threadIdx.x & 63;
    uint32_t r = (uint32_t)((blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6)) * 2654435761u);
    float acc = 0.f;
    for (int i = 0; i < iters; ++i) {
        float4 x[IN_FLIGHT];
#pragma unroll
        for (int u = 0; u < IN_FLIGHT; ++u) {
            r = r * 1664525u + 1013904223u;                       // row = high word of r * n_rows: two instructions per address
            x[u] = base[(size_t)__umulhi(r, n_rows) * 64 + lane];
        }
#pragma unroll
        for (int u = 0; u < IN_FLIGHT; ++u) acc += x[u].x + x[u].w;
    }
    if (acc == 12345.678f) sink[0] = acc;                      // never true for the zero / random data of the probe
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
inline int grid_for(const bpt_plan *p) { return (int)((p->n_items + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK); }

inline int check_plan(const bpt_plan *p, bool need_idx) {
    if (!p) return BPT_ERR_NULL;
    if (p->n_rows < 0 || p->n_edges < 0 || p->n_items < 0 || p->n_heavy < 0 || p->n_slots < 0) return BPT_ERR_SIZE;
    if (p->n_items > 0 && (!p->items || !p->rowptr)) return BPT_ERR_NULL;
    if (p->n_edges > 0 && (!p->eid || (need_idx && !p->idx))) return BPT_ERR_NULL;
    if (p->n_heavy > 0 && !p->heavy) return BPT_ERR_NULL;
    if (p->n_items < p->n_rows) return BPT_ERR_SIZE;     // every row owns at least one item
    if (p->n_groups < 0 || p->grp_R < 0 || p->grp_R > 32 || p->n_grp_entries < 0) return BPT_ERR_SIZE;
    if (p->n_groups > 0 && (!p->grp_members || !p->grp_ptr || !p->grp_chunks || (p->n_edges > 0 && !p->grp_entries))) return BPT_ERR_NULL;
    if (p->n_groups > 0 && (p->grp_max_chunk < 1 || p->grp_max_chunk > p->n_groups)) return BPT_ERR_SIZE;
    if (p->n_index_nodes < 0) return BPT_ERR_SIZE;
    return BPT_OK;
}

inline int check_shape(int h, int d, int dtype) {
    if (dtype != BPT_F32 && dtype != BPT_F64 && dtype != BPT_BF16) return BPT_ERR_DTYPE;
    if (h < 1 || d < 1 || (int64_t)h * d > (1 << 20)) return BPT_ERR_SHAPE;
    return BPT_OK;
}

inline size_t acc_size(int dtype) { return dtype == BPT_F64 ? 8 : 4; }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int launch_status() {
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? BPT_OK : (int)e;
}

// (H, D) pairs with a fast instantiation.  bf16 needs C >= 512 (eight elements per 16-byte vector).
#define BPT_FAST_SHAPES_F32(X) X(4, 64) X(8, 64) X(16, 64) X(8, 32)
#define BPT_FAST_SHAPES_BF16(X) X(8, 64) X(16, 64)

inline bool fast_shape(int h, int d, int dtype) {
    if (g_force_generic.load(std::memory_order_relaxed)) return false;
#define X(HH, DD) if (h == HH && d == DD) return true;
    if (dtype == BPT_F32) { BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { BPT_FAST_SHAPES_BF16(X) }
#undef X
    return false;
}

constexpr int FAST_BATCH = 4;

// ---- generic launchers (dtype dispatch) ----
template <typename T, int MODE>
int run_sddmm_generic(const bpt_plan *P, const void *A, const void *B, void *y, int h, int d, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
    hipLaunchKernelGGL((k_sddmm_generic<T, MODE>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)A, (const T *)B, (T *)y, h, d);
    return launch_status();
}

template <typename T, int MODE>
int run_spmm_generic(const bpt_plan *P, const void *W, const void *X, void *Y, void *ws, int h, int d, hipStream_t s) {
    using acc_t = typename Elem<T>::acc_t;
    if (P->n_items == 0) return BPT_OK;
    hipLaunchKernelGGL((k_spmm_generic<T, MODE>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)W, (const T *)X, (T *)Y, (acc_t *)ws, h, d);
    int st = launch_status();
    if (st != BPT_OK || P->n_heavy == 0) return st;
    hipLaunchKernelGGL((k_combine_sum<T>), dim3((int)P->n_heavy, (h * d + WAVE - 1) / WAVE, 1), dim3(BLOCK), 0, s, P->heavy,
                       (const acc_t *)ws, (T *)Y, (T *)nullptr, h * d, (size_t)0);
    return launch_status();
}

template <typename T>
int run_softmax_fwd(const bpt_plan *P, const void *x, void *y, void *ws, int h, hipStream_t s) {
    using acc_t = typename Elem<T>::acc_t;
    if (P->n_items == 0) return BPT_OK;
    if (WAVE % h == 0) {       // heads side by side; split rows in three steps over their segments
        acc_t *seg = P->n_heavy > 0 ? (acc_t *)ws : nullptr;
        hipLaunchKernelGGL((k_softmax_fwd_heads<T, 1>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)x, (T *)y, h, seg);
        int st = launch_status();
        if (st != BPT_OK || P->n_heavy == 0) return st;
        hipLaunchKernelGGL((k_softmax_seg_rows<acc_t, true>), dim3((int)P->n_heavy), dim3(BLOCK), 0, s, P->heavy, seg, h);
        st = launch_status();
        if (st != BPT_OK) return st;
        hipLaunchKernelGGL((k_softmax_seg_scale<T>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (T *)y, h, (const acc_t *)seg);
        return launch_status();
    }
    hipLaunchKernelGGL((k_softmax_fwd<T, 1>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)x, (T *)y, h);
    int st = launch_status();
    if (st != BPT_OK || P->n_heavy == 0) return st;
    hipLaunchKernelGGL((k_softmax_fwd<T, WAVES_PER_BLOCK>), dim3((int)P->n_heavy), dim3(BLOCK), 0, s, *P, (const T *)x, (T *)y, h);
    return launch_status();
}

template <typename T>
int run_softmax_bwd(const bpt_plan *P, const void *y, const void *dy, void *dx, void *ws, int h, hipStream_t s) {
    using acc_t = typename Elem<T>::acc_t;
    if (P->n_items == 0) return BPT_OK;
    if (WAVE % h == 0) {       // heads side by side; split rows in three steps over their segments
        acc_t *seg = P->n_heavy > 0 ? (acc_t *)ws : nullptr;
        hipLaunchKernelGGL((k_softmax_bwd_heads<T, 1>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)y, (const T *)dy, (T *)dx, h, seg);
        int st = launch_status();
        if (st != BPT_OK || P->n_heavy == 0) return st;
        hipLaunchKernelGGL((k_softmax_seg_rows<acc_t, false>), dim3((int)P->n_heavy), dim3(BLOCK), 0, s, P->heavy, seg, h);
        st = launch_status();
        if (st != BPT_OK) return st;
        hipLaunchKernelGGL((k_softmax_bwd_seg_finish<T>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)y, (const T *)dy, (T *)dx, h,
                           (const acc_t *)seg);
        return launch_status();
    }
    hipLaunchKernelGGL((k_softmax_bwd<T, 1>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)y, (const T *)dy, (T *)dx, h);
    int st = launch_status();
    if (st != BPT_OK || P->n_heavy == 0) return st;
    hipLaunchKernelGGL((k_softmax_bwd<T, WAVES_PER_BLOCK>), dim3((int)P->n_heavy), dim3(BLOCK), 0, s, *P, (const T *)y, (const T *)dy, (T *)dx, h);
    return launch_status();
}

template <typename T>
int run_nme_dB(const bpt_plan *P, const void *A, const void *dy, void *dB, int h, int d, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
    hipLaunchKernelGGL((k_nme_dB_generic<T>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)A, (const T *)dy, (T *)dB, h, d);
    return launch_status();
}

#define DISPATCH_DTYPE(dtype, CALL)                     \
    switch (dtype) {                                    \
        case BPT_F32: { using T = float; return CALL; } \
        case BPT_F64: { using T = double; return CALL; }\
        case BPT_BF16: { using T = bf16_t; return CALL; }\
        default: return BPT_ERR_DTYPE;                  \
    }

int sddmm_generic(const bpt_plan *P, const void *A, const void *B, void *y, int h, int d, int dtype, hipStream_t s) {
    DISPATCH_DTYPE(dtype, (run_sddmm_generic<T, 0>(P, A, B, y, h, d, s)))
}
int sddmm_edge_generic(const bpt_plan *P, const void *A, const void *B, void *y, int h, int d, int dtype, hipStream_t s) {
    DISPATCH_DTYPE(dtype, (run_sddmm_generic<T, 1>(P, A, B, y, h, d, s)))
}
int spmm_generic(const bpt_plan *P, const void *W, const void *X, void *Y, void *ws, int h, int d, int dtype, hipStream_t s) {
    DISPATCH_DTYPE(dtype, (run_spmm_generic<T, 0>(P, W, X, Y, ws, h, d, s)))
}
int spmm_edge_generic(const bpt_plan *P, const void *W, const void *X, void *Y, void *ws, int h, int d, int dtype, hipStream_t s) {
    DISPATCH_DTYPE(dtype, (run_spmm_generic<T, 1>(P, W, X, Y, ws, h, d, s)))
}

// ---- fast launchers ----
template <typename T, int H, int D>
int run_sddmm_fast(const bpt_plan *P, const void *A, const void *B, void *y, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
    hipLaunchKernelGGL((k_sddmm_fast<T, H, D, FAST_BATCH>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)A, (const T *)B, (T *)y);
    return launch_status();
}

template <typename T, typename WT, int H, int D, int NOUT>
int run_spmm_fast(const bpt_plan *P, const void *W0, const void *X0, void *Y0, const void *W1, const void *X1, void *Y1,
                  float *ws, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
    float *ws1 = ws ? ws + (size_t)P->n_slots * H * D : nullptr;
    {
        ProfScope prof(NOUT == 2 ? BPT_KERNEL_ATTN_BWD_SRC : -1, s);
        hipLaunchKernelGGL((k_spmm_fast<T, WT, H, D, FAST_BATCH, NOUT>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const WT *)W0,
                           (const T *)X0, (T *)Y0, (const WT *)W1, (const T *)X1, (T *)Y1, ws, ws1);
    }
    int st = launch_status();
    if (st != BPT_OK || P->n_heavy == 0) return st;
    hipLaunchKernelGGL((k_combine_sum_v4<T>), dim3((int)P->n_heavy, H * D / (4 * WAVE), NOUT), dim3(BLOCK), 0, s, P->heavy, (const float *)ws,
                       (T *)Y0, (T *)Y1, H * D, (size_t)P->n_slots * H * D);
    return launch_status();
}

// score term of the relative positions: bias[eid[p], head] = A[row, head, :] . table[idx[p], :], float32
bool spmm_grp_ok(const bpt_plan *P, int h, int d, int dtype);
template <typename T, int H, int D> constexpr int head_slices();
inline int group_grid(const bpt_plan *P);

// shapes of the matrix-core kernel of the rel_pos term and of its gradient kernel
inline bool rel_rows_shape(int h, int d, int dtype) {
    return !g_force_generic.load(std::memory_order_relaxed) && d == 64 && (h == 4 || h == 8 || h == 16) && (dtype == BPT_F32 || dtype == BPT_BF16);
}

constexpr int REL_MAX_PARTS = 512;        // partial tables of the gradient kernel: two workgroups per compute unit
constexpr int REL_MAX_USED = 240;         // type numbers whose table rows fit the 64 KB of LDS of the score kernel

// LDS of k_rel_bias_bwd with nw wavefronts: their sums, the table rows, their staged ds values
inline size_t rel_bwd_lds(int nw, int64_t n_used, int h) { return ((size_t)(nw + 1) * n_used * 64 + (size_t)nw * WAVE * h) * 4; }
// wavefronts per workgroup of k_rel_bias_bwd for n_used types: the 4, 2 or 1 that put most wavefronts on a compute unit
// (workgroups that fit its 160 KB of LDS x wavefronts each; more per workgroup on a tie: fewer partial tables), a
// workgroup taking at most 144 KB (large_lds false: at most the 64 KB every kernel may take).  0: no configuration fits.
inline int rel_bwd_waves(int64_t n_used, int h, bool large_lds = true) {
    const size_t cap = (large_lds ? 144 : 64) * 1024;
    int best = 0, best_waves = 0;
    for (int nw = 4; nw >= 1; nw >>= 1) {
        const size_t lds = rel_bwd_lds(nw, n_used, h);
        if (lds > cap) continue;
        const int waves = nw * (int)((160 * 1024) / lds);
        if (waves > best_waves) { best = nw; best_waves = waves; }
    }
    return best;
}

// a kernel may take more than 64 KB of dynamic LDS only after it has been told so (once per kernel and device; kernels of
// one signature are different kernels, so what has been done is kept by kernel address)
inline int allow_large_lds_at(const void *kernel, size_t bytes) {
    static std::mutex lock;
    static std::vector<std::pair<const void *, int>> done;
    if (bytes <= 64 * 1024) return BPT_OK;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return BPT_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> hold(lock);
    for (const auto &x : done)
        if (x.first == kernel && x.second == dev) return BPT_OK;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return BPT_ERR_UNSUPPORTED;          // (the caller then takes a configuration inside 64 KB)
    }
    done.emplace_back(kernel, dev);
    return BPT_OK;
}
template <typename K>
int allow_large_lds(K kernel, size_t bytes) { return allow_large_lds_at(reinterpret_cast<const void *>(kernel), bytes); }

template <typename T, int H, int NW>
int launch_rel_bias_bwd(const bpt_plan *P, const float *ds, const void *q, const void *table, const int32_t *used_types, int64_t n_used,
                        void *dq, float *ws_dq, float *part, int n_parts, hipStream_t s) {
    const size_t lds = rel_bwd_lds(NW, n_used, H);
    const int st = allow_large_lds(k_rel_bias_bwd<T, H, NW>, lds);
    if (st != BPT_OK) return st;
    hipLaunchKernelGGL((k_rel_bias_bwd<T, H, NW>), dim3(n_parts), dim3(NW * WAVE), lds, s, *P, ds, (const T *)q, (const T *)table, used_types,
                       (int)n_used, (T *)dq, ws_dq, part);
    return launch_status();
}

template <typename T, int H>
int run_rel_bias_bwd(const bpt_plan *P, const float *ds, const void *q, const void *table, const int32_t *used, const int32_t *used_types,
                     int64_t n_types, int64_t n_used, void *dq, void *dtable, float *ws, hipStream_t s) {
    float *ws_dq = ws, *part = ws + (size_t)P->n_slots * H * 64;       // partial rows of dq of the split rows, then the partial tables
    int n_parts = 0;
    auto launch = [&](int nw) {
        n_parts = (int)std::min<int64_t>(REL_MAX_PARTS, std::max<int64_t>(1, (P->n_edges + nw * 128 - 1) / (nw * 128)));
        return nw == 4   ? launch_rel_bias_bwd<T, H, 4>(P, ds, q, table, used_types, n_used, dq, ws_dq, part, n_parts, s)
               : nw == 2 ? launch_rel_bias_bwd<T, H, 2>(P, ds, q, table, used_types, n_used, dq, ws_dq, part, n_parts, s)
                         : launch_rel_bias_bwd<T, H, 1>(P, ds, q, table, used_types, n_used, dq, ws_dq, part, n_parts, s);
    };
    if (P->n_edges > 0) {
        const int nw = rel_bwd_waves(n_used, H);
        int st = launch(nw);
        if (st == BPT_ERR_UNSUPPORTED && rel_bwd_lds(nw, n_used, H) > 64 * 1024) {      // more than 64 KB of LDS refused by the runtime
            const int small = rel_bwd_waves(n_used, H, false);
            if (small == 0) return BPT_ERR_UNSUPPORTED;
            st = launch(small);
        }
        if (st != BPT_OK) return st;
    }
    // (without edges there are no partial tables and no partial rows: every row of dtable becomes zero)
    const bool edges = P->n_edges > 0;
    const int n_split = edges ? (int)P->n_heavy : 0;
    hipLaunchKernelGGL((k_rel_finish<T>), dim3((unsigned)(n_types + (int64_t)n_split * (H * 64 / 256))), dim3(BLOCK), 0, s, part, used,
                       edges ? n_parts : 0, (int)n_types, (T *)dtable, P->heavy, ws_dq, (T *)dq, H * 64);
    return launch_status();
}

// whether run_rel_bias_bwd has a configuration that this device accepts for n_used types (nothing is launched)
template <typename T, int H>
int rel_bias_bwd_config(int64_t n_used) {
    const int nw = rel_bwd_waves(n_used, H);
    if (nw == 0) return BPT_ERR_UNSUPPORTED;
    const size_t lds = rel_bwd_lds(nw, n_used, H);
    const int st = nw == 4   ? allow_large_lds(k_rel_bias_bwd<T, H, 4>, lds)
                   : nw == 2 ? allow_large_lds(k_rel_bias_bwd<T, H, 2>, lds)
                             : allow_large_lds(k_rel_bias_bwd<T, H, 1>, lds);
    if (st == BPT_OK) return BPT_OK;
    return rel_bwd_waves(n_used, H, false) != 0 ? BPT_OK : BPT_ERR_UNSUPPORTED;      // inside the 64 KB every kernel may take
}

// the score term with the table rows in LDS: plan indices are type numbers
template <typename T, int H>
int run_rel_bias_rows(const bpt_plan *P, const void *q, const void *table, const int32_t *used_types, int64_t n_used, float *bias, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
    const int64_t waves = (P->n_items + REL_FWD_ITEMS - 1) / REL_FWD_ITEMS;
    hipLaunchKernelGGL((k_rel_bias_rows<T, H>), dim3((unsigned)((waves + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK)), dim3(BLOCK),
                       (size_t)n_used * REL_LDS_PITCH * 4, s, *P, (const T *)q, (const T *)table, used_types, (int)n_used, bias);
    return launch_status();
}

// the score term over the attention kernels' tile plan, in that plan's pair order
template <typename T, int H, int HW>
int launch_rel_bias_tiles(const bpt_plan *P, const void *q, const void *table, const int32_t *used_types, int64_t n_used, const int32_t *pair_tm,
                          float *bias, size_t lds, hipStream_t s) {
    const int st = allow_large_lds(k_rel_bias_tiles<T, H, HW>, lds);
    if (st != BPT_OK) return st;
    hipLaunchKernelGGL((k_rel_bias_tiles<T, H, HW>), dim3(group_grid(P) * (H / HW)), dim3(HW * WAVE), lds, s, *P, (const T *)q, (const T *)table,
                       used_types, (int)n_used, pair_tm, bias);
    return launch_status();
}
template <typename T, int H>
int run_rel_bias_tiles(const bpt_plan *P, const void *q, const void *table, const int32_t *used_types, int64_t n_used, const int32_t *pair_tm,
                       float *bias, hipStream_t s) {
    // the table rows once per workgroup, QT once per wavefront (= head); eight heads share the rows where that fits 64 KB
    auto lds = [&](int hw) { return ((size_t)n_used * REL_LDS_PITCH + (size_t)hw * (size_t)((n_used + 15) & ~(int64_t)15) * TILE_R) * 4; };
    if constexpr (H >= 8) {
        if (lds(8) <= 64 * 1024) return launch_rel_bias_tiles<T, H, 8>(P, q, table, used_types, n_used, pair_tm, bias, lds(8), s);
    }
    return launch_rel_bias_tiles<T, H, 4>(P, q, table, used_types, n_used, pair_tm, bias, lds(4), s);
}

template <typename T, int H, int D>
int run_rel_bias(const bpt_plan *P, const void *A, const void *table, float *bias, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
    if (spmm_grp_ok(P, H, D, sizeof(T) == 2 ? BPT_BF16 : BPT_F32)) {      // row groups: one load of a table row per group entry
        constexpr int HS = head_slices<T, H, D>();
        if (P->grp_R == 8)
            hipLaunchKernelGGL((k_sddmm_grp<T, H, D, 8, HS, true, float>), dim3(group_grid(P) * HS), dim3(WAVE), 0, s, *P, (const T *)A,
                               (const T *)table, bias);
        else
            hipLaunchKernelGGL((k_sddmm_grp<T, H, D, 4, HS, true, float>), dim3(group_grid(P) * HS), dim3(WAVE), 0, s, *P, (const T *)A,
                               (const T *)table, bias);
        return launch_status();
    }
    hipLaunchKernelGGL((k_sddmm_fast<T, H, D, FAST_BATCH, 2, float>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)A, (const T *)table,
                       bias);
    return launch_status();
}

// node_mul_edge with the specialised kernels: y = A . B[e] (forward), dA = sum dy * B[e], dB[e] = sum_h dy * A
template <typename T, int H, int D>
int run_nme_fwd_fast(const bpt_plan *P, const void *A, const void *B, void *y, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
    hipLaunchKernelGGL((k_sddmm_fast<T, H, D, FAST_BATCH, 1>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)A, (const T *)B, (T *)y);
    return launch_status();
}

template <typename T, int H, int D>
int run_nme_bwd_fast(const bpt_plan *P, const void *A, const void *B, const void *dy, void *dA, void *dB, float *ws, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
    hipLaunchKernelGGL((k_spmm_fast<T, T, H, D, FAST_BATCH, 1, 1>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)dy, (const T *)B,
                       (T *)dA, (const T *)nullptr, (const T *)nullptr, (T *)nullptr, ws, (float *)nullptr);
    int st = launch_status();
    if (st != BPT_OK) return st;
    if (P->n_heavy > 0) {
        hipLaunchKernelGGL((k_combine_sum_v4<T>), dim3((int)P->n_heavy, H * D / (4 * WAVE), 1), dim3(BLOCK), 0, s, P->heavy, (const float *)ws,
                           (T *)dA, (T *)nullptr, H * D, (size_t)0);
        st = launch_status();
        if (st != BPT_OK) return st;
    }
    hipLaunchKernelGGL((k_nme_dB_fast<T, H, D, FAST_BATCH>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)A, (const T *)dy, (T *)dB);
    return launch_status();
}

int nme_fwd_fast(const bpt_plan *P, const void *A, const void *B, void *y, int h, int d, int dtype, hipStream_t s) {
#define X(HH, DD) if (h == HH && d == DD) return run_nme_fwd_fast<T, HH, DD>(P, A, B, y, s);
    if (dtype == BPT_F32) { using T = float; BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { using T = bf16_t; BPT_FAST_SHAPES_BF16(X) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

int nme_bwd_fast(const bpt_plan *P, const void *A, const void *B, const void *dy, void *dA, void *dB, void *ws, int h, int d, int dtype,
                 hipStream_t s) {
#define X(HH, DD) if (h == HH && d == DD) return run_nme_bwd_fast<T, HH, DD>(P, A, B, dy, dA, dB, (float *)ws, s);
    if (dtype == BPT_F32) { using T = float; BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { using T = bf16_t; BPT_FAST_SHAPES_BF16(X) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

int sddmm_fast(const bpt_plan *P, const void *A, const void *B, void *y, int h, int d, int dtype, hipStream_t s) {
#define X(HH, DD) if (h == HH && d == DD) return run_sddmm_fast<T, HH, DD>(P, A, B, y, s);
    if (dtype == BPT_F32) { using T = float; BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { using T = bf16_t; BPT_FAST_SHAPES_BF16(X) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

int spmm_fast(const bpt_plan *P, const void *W, const void *Xp, void *Y, void *ws, int h, int d, int dtype, hipStream_t s) {
#define X(HH, DD) if (h == HH && d == DD) return run_spmm_fast<T, T, HH, DD, 1>(P, W, Xp, Y, nullptr, nullptr, nullptr, (float *)ws, s);
    if (dtype == BPT_F32) { using T = float; BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { using T = bf16_t; BPT_FAST_SHAPES_BF16(X) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

// SDDMM / SpMM with automatic family choice
bool spmm_grp_ok(const bpt_plan *P, int h, int d, int dtype);
int sddmm_grp(const bpt_plan *P, const void *A, const void *B, void *y, int h, int d, int dtype, hipStream_t s);
int sddmm(const bpt_plan *P, const void *A, const void *B, void *y, int h, int d, int dtype, hipStream_t s) {
    if (fast_shape(h, d, dtype) && aligned16(A) && aligned16(B)) {
        if (spmm_grp_ok(P, h, d, dtype)) return sddmm_grp(P, A, B, y, h, d, dtype, s);
        return sddmm_fast(P, A, B, y, h, d, dtype, s);
    }
    return sddmm_generic(P, A, B, y, h, d, dtype, s);
}
int spmm_grp(const bpt_plan *P, const void *W, const void *X, void *Y, void *ws, int h, int d, int dtype, hipStream_t s, int accumulate = 0);
int spmm(const bpt_plan *P, const void *W, const void *X, void *Y, void *ws, int h, int d, int dtype, hipStream_t s) {
    if (fast_shape(h, d, dtype) && aligned16(X) && aligned16(Y) && aligned16(ws)) {
        // a plan that carries row groups and their edge ids: one row load per entry instead of one per edge
        if (spmm_grp_ok(P, h, d, dtype)) return spmm_grp(P, W, X, Y, ws, h, d, dtype, s);
        return spmm_fast(P, W, X, Y, ws, h, d, dtype, s);
    }
    return spmm_generic(P, W, X, Y, ws, h, d, dtype, s);
}

inline int64_t round16(int64_t b) { return (b + 15) & ~(int64_t)15; }

// dropout of the fused path: threshold on the 32-bit hash (0 = off), seed, 1 / (1 - p)
struct Dropout {
    uint32_t thr, seed;
    float inv;
};
inline Dropout make_dropout(float p, uint64_t seed) {
    if (!(p > 0.f)) return Dropout{0u, 0u, 1.f};
    const double t = (double)p * 4294967296.0;
    return Dropout{(uint32_t)(t >= 4294967295.0 ? 4294967295.0 : (t < 1.0 ? 1.0 : t)), (uint32_t)(seed ^ (seed >> 32)), 1.f / (1.f - p)};
}

// The row-group kernels address node rows and the per-pair scratch with 32-bit byte offsets.
inline bool fits32(int64_t n, int64_t unit) { return n >= 0 && n <= (int64_t)0xffffffffu / unit; }

inline int group_grid(const bpt_plan *P) { return (int)(8 * P->grp_max_chunk); }

// The row-group kernels split a group's heads over wavefronts so that one wavefront handles at most 512 columns of
// every row (8 registers per lane and row: the members' state has to fit the register file).  Slices of 256
// float32 columns were also measured: faster on small graphs, slower at the benchmark sizes.
template <typename T, int H, int D> constexpr int head_slices() {
    constexpr int CS = 512, C = H * D;
    return (C > CS && C % CS == 0 && H % (C / CS) == 0) ? C / CS : 1;
}

// The matrix-core forward gives a wavefront at most 512 columns of every row.  0 slices = shape not covered.
template <typename T, int H, int D> constexpr int mfma_slices() {
    constexpr int CS = 512, C = H * D;
    if (C <= CS) return 1;
    return (C % CS == 0 && H % (C / CS) == 0) ? C / CS : 0;
}
template <typename T, int H, int D> constexpr bool mfma_ok() {
    constexpr int HS = mfma_slices<T, H, D>();
    if (HS == 0) return false;
    constexpr int HL = H / HS, CS = HL * D, VE = 16 / (int)sizeof(T);
    if (64 % HL != 0 || CS % 64 != 0) return false;
    constexpr int LPH = 64 / HL, EPL = CS / 64;
    return (LPH == 4 || LPH == 8 || LPH == 16) && EPL % VE == 0 && EPL <= 8;
}

// rows per group the row-group kernels exist for
inline bool group_rows_ok(int64_t R) { return R == 4 || R == 8; }

inline bool has_groups(const bpt_plan *P, int h, int d, size_t elem) {
    return P->n_groups > 0 && group_rows_ok(P->grp_R) && P->grp_members && P->grp_ptr && P->grp_entries && P->grp_chunks &&
           P->grp_max_chunk > 0 && 8 * P->grp_max_chunk >= P->n_groups && P->n_grp_entries >= 0 &&
           fits32(std::max(P->n_rows, P->n_index_nodes), (int64_t)h * d * (int64_t)elem) &&
           fits32((P->n_grp_entries + GRP_PAD_ENTRIES) * P->grp_R, (int64_t)h * 8);
}

// groups of 16 rows for the dense-tile kernels (one wavefront per head: h * 64 threads per workgroup)
inline bool has_tiles(const bpt_plan *P, int h, int d, size_t elem) {
    return P->n_groups > 0 && P->grp_R == TILE_R && P->grp_members && P->grp_ptr && P->grp_entries && P->grp_chunks &&
           P->grp_max_chunk > 0 && 8 * P->grp_max_chunk >= P->n_groups && P->n_grp_entries >= 0 && d == 64 && h <= 16 && (elem == 4 || elem == 2) &&
           fits32(std::max(P->n_rows, P->n_index_nodes), (int64_t)h * d * (int64_t)elem);
}

// Few and tall tiles (fewer wavefronts than three per SIMD, six or more blocks each on average): the kernels then read one
// block ahead in registers instead of counting on other wavefronts to cover the loads.
inline bool tall_tiles(const bpt_plan *P, int h) {
    return P->n_groups * h < 3 * 1024 && P->n_grp_entries >= 6 * TILE_R * P->n_groups;
}

bool spmm_grp_ok(const bpt_plan *P, int h, int d, int dtype) {
    return has_groups(P, h, d, dtype == BPT_BF16 ? 2 : 4) && P->grp_eids && P->n_edges > 0;
}

template <typename T, int H, int D>
int run_spmm_grp(const bpt_plan *P, const void *W, const void *X, void *Y, float *ws, hipStream_t s, int accumulate = 0) {
    constexpr int HS = head_slices<T, H, D>();
#define LAUNCH_SPMM(RR)                                                                                                     \
    hipLaunchKernelGGL((k_spmm_grp<T, H, D, RR, HS>), dim3(group_grid(P) * HS), dim3(WAVE), 0, s, *P, (const T *)W, (const T *)X, \
                       (T *)Y, ws, accumulate)
    if (P->grp_R == 8) LAUNCH_SPMM(8);
    else LAUNCH_SPMM(4);
#undef LAUNCH_SPMM
    int st = launch_status();
    if (st != BPT_OK || P->n_heavy == 0) return st;
    hipLaunchKernelGGL((k_combine_sum_v4<T>), dim3((int)P->n_heavy, H * D / (4 * WAVE), 1), dim3(BLOCK), 0, s, P->heavy, (const float *)ws,
                       (T *)Y, (T *)nullptr, H * D, (size_t)0, accumulate);
    return launch_status();
}

template <typename T, int H, int D>
int run_sddmm_grp(const bpt_plan *P, const void *A, const void *B, void *y, hipStream_t s) {
    constexpr int HS = head_slices<T, H, D>();
    if (P->grp_R == 8) hipLaunchKernelGGL((k_sddmm_grp<T, H, D, 8, HS>), dim3(group_grid(P) * HS), dim3(WAVE), 0, s, *P, (const T *)A, (const T *)B, (T *)y);
    else hipLaunchKernelGGL((k_sddmm_grp<T, H, D, 4, HS>), dim3(group_grid(P) * HS), dim3(WAVE), 0, s, *P, (const T *)A, (const T *)B, (T *)y);
    return launch_status();
}

int sddmm_grp(const bpt_plan *P, const void *A, const void *B, void *y, int h, int d, int dtype, hipStream_t s) {
#define X(HH, DD) if (h == HH && d == DD) return run_sddmm_grp<T, HH, DD>(P, A, B, y, s);
    if (dtype == BPT_F32) { using T = float; BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { using T = bf16_t; BPT_FAST_SHAPES_BF16(X) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

int spmm_grp(const bpt_plan *P, const void *W, const void *Xp, void *Y, void *ws, int h, int d, int dtype, hipStream_t s, int accumulate) {
#define X(HH, DD) if (h == HH && d == DD) return run_spmm_grp<T, HH, DD>(P, W, Xp, Y, (float *)ws, s, accumulate);
    if (dtype == BPT_F32) { using T = float; BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { using T = bf16_t; BPT_FAST_SHAPES_BF16(X) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

inline bool grouped_backward(const bpt_plan *Pin, const bpt_plan *Pout, int h, int d, size_t elem) {
    return has_groups(Pin, h, d, elem) && has_groups(Pout, h, d, elem) && Pin->grp_R == Pout->grp_R && Pin->grp_pairs;
}

// the tile kernels run the backward when both sides carry tiles and the source side the destination side's pair numbers
inline bool tiled_backward(const bpt_plan *Pin, const bpt_plan *Pout, int h, int d, size_t elem) {
    return has_tiles(Pin, h, d, elem) && has_tiles(Pout, h, d, elem) && Pout->grp_pairs;
}

// float2 (p, ds) scratch of the fused backward: one per (entry, member) of the source-side groups (plus the
// look-ahead padding) for the row-group kernels, one per edge for the per-row and the tile kernels
inline int64_t pds_bytes(const bpt_plan *Pin, const bpt_plan *Pout, int h, int d, size_t elem) {
    int64_t n = Pin->n_edges;
    if (Pout && grouped_backward(Pin, Pout, h, d, elem)) n = std::max(n, (Pout->n_grp_entries + GRP_PAD_ENTRIES) * Pout->grp_R);
    return 2 * round16(n * h * 4);
}

// how the tile kernels find the score term: 0 none, 1 by edge id, 2 in the plan's own pair order, head-major
inline int tile_bias_mode(const bpt_plan *P, const float *bias) { return !bias ? 0 : P->bias_by_pair ? 2 : 1; }

template <typename T, int H, int D>
int run_attn_fwd(const bpt_plan *P, const void *q, const void *k, const void *v, void *o, float *lse, void *ws, float scale, Dropout drop,
                 const float *bias, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
    float *ws_acc = (float *)ws;
    float *ws_ml = ws_acc ? ws_acc + (size_t)P->n_slots * H * D : nullptr;
    {
        ProfScope prof(BPT_KERNEL_ATTN_FWD, s);
        if constexpr (D == 64 && sizeof(T) == 4) {
            if (has_tiles(P, H, D, sizeof(T)) && ((drop.thr == 0 && !bias) || P->grp_eids)) {
                constexpr int HW = H >= 4 ? 4 : H;          // heads per workgroup
#define LAUNCH_FWD_TILE(PI, DR, BI)                                                                                                  \
    hipLaunchKernelGGL((k_attn_fwd_tile<T, H, D, HW, PI, DR, BI>), dim3(group_grid(P) * (H / HW)), dim3(HW * WAVE), 0, s, *P, (const T *)q, \
                       (const T *)k, (const T *)v, (T *)o, lse, ws_acc, ws_ml, scale * LOG2E, drop.thr, drop.seed, drop.inv, bias)
                switch ((drop.thr != 0 ? 1 : 0) + 2 * tile_bias_mode(P, bias)) {
                case 0: if (tall_tiles(P, H)) LAUNCH_FWD_TILE(true, false, 0); else LAUNCH_FWD_TILE(false, false, 0); break;
                case 1: LAUNCH_FWD_TILE(false, true, 0); break;
                case 2: LAUNCH_FWD_TILE(false, false, 1); break;
                case 3: LAUNCH_FWD_TILE(false, true, 1); break;
                case 4: LAUNCH_FWD_TILE(false, false, 2); break;
                default: LAUNCH_FWD_TILE(false, true, 2); break;
                }
#undef LAUNCH_FWD_TILE
                goto launched;
            }
        }
        if constexpr (D == 64 && sizeof(T) == 2) {
            if (has_tiles(P, H, D, sizeof(T)) && ((drop.thr == 0 && !bias) || P->grp_eids)) {
                constexpr int HW = H >= 4 ? 4 : H;
#define LAUNCH_FWD_TILE(DR, BI)                                                                                                          \
    hipLaunchKernelGGL((k_attn_fwd_tile_bf16<H, D, HW, TILE_BF16_WPE, TILE_BF16_PIPE, DR, BI>), dim3(group_grid(P) * (H / HW)), dim3(HW * WAVE), \
                       0, s, *P, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, (bf16_t *)o, lse, ws_acc, ws_ml, scale * LOG2E,   \
                       drop.thr, drop.seed, drop.inv, bias)
                switch ((drop.thr != 0 ? 1 : 0) + 2 * tile_bias_mode(P, bias)) {
                case 0: LAUNCH_FWD_TILE(false, 0); break;
                case 1: LAUNCH_FWD_TILE(true, 0); break;
                case 2: LAUNCH_FWD_TILE(false, 1); break;
                case 3: LAUNCH_FWD_TILE(true, 1); break;
                case 4: LAUNCH_FWD_TILE(false, 2); break;
                default: LAUNCH_FWD_TILE(true, 2); break;
                }
#undef LAUNCH_FWD_TILE
                goto launched;
            }
        }
        if (has_groups(P, H, D, sizeof(T))) {
#define LAUNCH_FWD(RR, DR, BI)                                                                                                   \
    hipLaunchKernelGGL((k_attn_fwd_grp<T, H, D, RR, HS, DR, BI>), dim3(group_grid(P) * HS), dim3(WAVE), 0, s, *P, (const T *)q, \
                       (const T *)k, (const T *)v, (T *)o, lse, ws_acc, ws_ml, scale * LOG2E, drop.thr, drop.seed, drop.inv, bias)
#define LAUNCH_FWD_MFMA(DR, BI)                                                                                                      \
    hipLaunchKernelGGL((k_attn_fwd_mfma<T, H, D, HSM, DR, BI>), dim3(group_grid(P) * HSM), dim3(2 * WAVE), 0, s, *P, (const T *)q, \
                       (const T *)k, (const T *)v, (T *)o, lse, ws_acc, ws_ml, scale * LOG2E, drop.thr, drop.seed, drop.inv, bias)
            constexpr int HS = head_slices<T, H, D>();
            const int variant = (drop.thr != 0 ? 1 : 0) + (bias ? 2 : 0);
            if (P->grp_R == 8) {
                // every compile-time shape has the matrix-core form for groups of 8
                static_assert(mfma_ok<T, H, D>(), "groups of 8 rows need the matrix-core forward");
                constexpr int HSM = mfma_slices<T, H, D>();
                switch (variant) {
                case 0: LAUNCH_FWD_MFMA(false, false); break;
                case 1: LAUNCH_FWD_MFMA(true, false); break;
                case 2: LAUNCH_FWD_MFMA(false, true); break;
                default: LAUNCH_FWD_MFMA(true, true); break;
                }
            } else {
                switch (variant) {
                case 0: LAUNCH_FWD(4, false, false); break;
                case 1: LAUNCH_FWD(4, true, false); break;
                case 2: LAUNCH_FWD(4, false, true); break;
                default: LAUNCH_FWD(4, true, true); break;
                }
            }
#undef LAUNCH_FWD
#undef LAUNCH_FWD_MFMA
        } else {
            hipLaunchKernelGGL((k_attn_fwd<T, H, D, FAST_BATCH>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)q, (const T *)k,
                               (const T *)v, (T *)o, lse, ws_acc, ws_ml, scale * LOG2E);
        }
    launched:;
    }
    int st = launch_status();
    if (st != BPT_OK || P->n_heavy == 0) return st;
    hipLaunchKernelGGL((k_attn_fwd_combine<T, H, D>), dim3((int)P->n_heavy, H * D / WAVE), dim3(BLOCK), 0, s, P->heavy,
                       (const float *)ws_acc, (const float *)ws_ml, (T *)o, lse);
    return launch_status();
}

template <typename T, int H, int D>
int run_attn_bwd(const bpt_plan *Pin, const bpt_plan *Pout, const void *q, const void *k, const void *v, const void *o,
                 const void *d_o, const float *lse, void *dq, void *dk, void *dv, void *ws, float scale, Dropout drop, const float *bias,
                 float *ds_out, hipStream_t s) {
    if (Pin->n_items == 0) return BPT_OK;
    const bool grouped = grouped_backward(Pin, Pout, H, D, sizeof(T));
    const int64_t pbytes = pds_bytes(Pin, Pout, H, D, sizeof(T));
    float *pbuf = (float *)ws;                                   // per-row kernels: p (E, H) then ds (E, H)
    float *dsbuf = pbuf + pbytes / 8;
    float2 *pds = (float2 *)ws;                                  // row-group kernels: interleaved (p, ds)
    float *ws_rows = (float *)ws + pbytes / 4;
    if constexpr (D == 64 && sizeof(T) == 4) {
        if (tiled_backward(Pin, Pout, H, D, sizeof(T)) && ((drop.thr == 0 && !bias) || Pin->grp_eids)) {
            constexpr int HW = H >= 4 ? 4 : H;
            float *ws_dk = ws_rows + (size_t)Pin->n_slots * H * D, *ws_dv = ws_dk + (size_t)Pout->n_slots * H * D;
            {
                ProfScope prof(BPT_KERNEL_ATTN_BWD_DST, s);
#define LAUNCH_DST_TILE(PI, DR, BI)                                                                                                    \
    hipLaunchKernelGGL((k_attn_bwd_dst_tile<T, H, D, HW, PI, DR, BI>), dim3(group_grid(Pin) * (H / HW)), dim3(HW * WAVE), 0, s, *Pin,     \
                       (const T *)q, (const T *)k, (const T *)v, (const T *)o, (const T *)d_o, lse, (T *)dq, pds, ws_rows, scale,         \
                       scale * LOG2E, drop.thr, drop.seed, drop.inv, bias, ds_out)
                switch ((drop.thr != 0 ? 1 : 0) + 2 * tile_bias_mode(Pin, bias)) {
                case 0: if (tall_tiles(Pin, H)) LAUNCH_DST_TILE(true, false, 0); else LAUNCH_DST_TILE(false, false, 0); break;
                case 1: LAUNCH_DST_TILE(false, true, 0); break;
                case 2: LAUNCH_DST_TILE(false, false, 1); break;
                case 3: LAUNCH_DST_TILE(false, true, 1); break;
                case 4: LAUNCH_DST_TILE(false, false, 2); break;
                default: LAUNCH_DST_TILE(false, true, 2); break;
                }
#undef LAUNCH_DST_TILE
            }
            int st = launch_status();
            if (st != BPT_OK) return st;
            {
                ProfScope prof(BPT_KERNEL_ATTN_BWD_SRC, s);
                if (tall_tiles(Pout, H))
                    hipLaunchKernelGGL((k_attn_bwd_src_tile<T, H, D, HW, true>), dim3(group_grid(Pout) * (H / HW)), dim3(HW * WAVE), 0, s, *Pout,
                                       (const T *)q, (const T *)d_o, (const float2 *)pds, (T *)dk, (T *)dv, ws_dk, ws_dv);
                else
                    hipLaunchKernelGGL((k_attn_bwd_src_tile<T, H, D, HW, false>), dim3(group_grid(Pout) * (H / HW)), dim3(HW * WAVE), 0, s, *Pout,
                                       (const T *)q, (const T *)d_o, (const float2 *)pds, (T *)dk, (T *)dv, ws_dk, ws_dv);
            }
            st = launch_status();
            if (st != BPT_OK || Pin->n_heavy + Pout->n_heavy == 0) return st;
            hipLaunchKernelGGL((k_combine_sum3<T>), dim3((int)(Pin->n_heavy + Pout->n_heavy), H * D / (4 * WAVE), 2), dim3(BLOCK), 0, s, Pin->heavy,
                               (int)Pin->n_heavy, (const float *)ws_rows, (T *)dq, Pout->heavy, (const float *)ws_dk, (T *)dk, (T *)dv, H * D,
                               (size_t)Pout->n_slots * H * D);
            return launch_status();
        }
    }
    if constexpr (D == 64 && sizeof(T) == 2) {
        if (tiled_backward(Pin, Pout, H, D, sizeof(T)) && ((drop.thr == 0 && !bias) || Pin->grp_eids)) {
            constexpr int HW = H >= 4 ? 4 : H;
            float *ws_dk = ws_rows + (size_t)Pin->n_slots * H * D, *ws_dv = ws_dk + (size_t)Pout->n_slots * H * D;
            {
                ProfScope prof(BPT_KERNEL_ATTN_BWD_DST, s);
#define LAUNCH_DST_TILE(DR, BI)                                                                                                          \
    hipLaunchKernelGGL((k_attn_bwd_dst_tile_bf16<H, D, HW, TILE_BF16_WPE_DST, TILE_BF16_PIPE, DR, BI>), dim3(group_grid(Pin) * (H / HW)),   \
                       dim3(HW * WAVE), 0, s, *Pin, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, (const bf16_t *)o,             \
                       (const bf16_t *)d_o, lse, (bf16_t *)dq, (uint32_t *)ws, ws_rows, scale, scale * LOG2E, drop.thr, drop.seed,          \
                       drop.inv, bias, ds_out)
                switch ((drop.thr != 0 ? 1 : 0) + 2 * tile_bias_mode(Pin, bias)) {
                case 0: LAUNCH_DST_TILE(false, 0); break;
                case 1: LAUNCH_DST_TILE(true, 0); break;
                case 2: LAUNCH_DST_TILE(false, 1); break;
                case 3: LAUNCH_DST_TILE(true, 1); break;
                case 4: LAUNCH_DST_TILE(false, 2); break;
                default: LAUNCH_DST_TILE(true, 2); break;
                }
#undef LAUNCH_DST_TILE
            }
            int st = launch_status();
            if (st != BPT_OK) return st;
            {
                ProfScope prof(BPT_KERNEL_ATTN_BWD_SRC, s);
                hipLaunchKernelGGL((k_attn_bwd_src_tile_bf16<H, D, HW, TILE_BF16_WPE_SRC, TILE_BF16_PIPE>), dim3(group_grid(Pout) * (H / HW)), dim3(HW * WAVE), 0, s,
                                   *Pout, (const bf16_t *)q, (const bf16_t *)d_o, (const uint32_t *)ws, (bf16_t *)dk, (bf16_t *)dv, ws_dk, ws_dv);
            }
            st = launch_status();
            if (st != BPT_OK || Pin->n_heavy + Pout->n_heavy == 0) return st;
            hipLaunchKernelGGL((k_combine_sum3<T>), dim3((int)(Pin->n_heavy + Pout->n_heavy), H * D / (4 * WAVE), 2), dim3(BLOCK), 0, s, Pin->heavy,
                               (int)Pin->n_heavy, (const float *)ws_rows, (T *)dq, Pout->heavy, (const float *)ws_dk, (T *)dk, (T *)dv, H * D,
                               (size_t)Pout->n_slots * H * D);
            return launch_status();
        }
    }
    {
        ProfScope prof(BPT_KERNEL_ATTN_BWD_DST, s);
        if (grouped) {
#define LAUNCH_DST(RR, DR, BI)                                                                                                           \
    hipLaunchKernelGGL((k_attn_bwd_dst_grp<T, H, D, RR, HS, DR, BI>), dim3(group_grid(Pin) * HS), dim3(WAVE), 0, s, *Pin, (const T *)q, \
                       (const T *)k, (const T *)v, (const T *)o, (const T *)d_o, lse, (T *)dq, pds, ws_rows, scale, scale * LOG2E,      \
                       drop.thr, drop.seed, drop.inv, bias, ds_out)
            constexpr int HS = head_slices<T, H, D>();
            const int variant = (drop.thr != 0 ? 1 : 0) + (bias ? 2 : 0) + (Pin->grp_R == 8 ? 4 : 0);
            switch (variant) {
            case 0: LAUNCH_DST(4, false, false); break;
            case 1: LAUNCH_DST(4, true, false); break;
            case 2: LAUNCH_DST(4, false, true); break;
            case 3: LAUNCH_DST(4, true, true); break;
            case 4: LAUNCH_DST(8, false, false); break;
            case 5: LAUNCH_DST(8, true, false); break;
            case 6: LAUNCH_DST(8, false, true); break;
            default: LAUNCH_DST(8, true, true); break;
            }
#undef LAUNCH_DST
        } else {
            hipLaunchKernelGGL((k_attn_bwd_dst<T, H, D, FAST_BATCH>), dim3(grid_for(Pin)), dim3(BLOCK), 0, s, *Pin, (const T *)q,
                               (const T *)k, (const T *)v, (const T *)o, (const T *)d_o, lse, (T *)dq, pbuf, dsbuf, ws_rows, scale,
                               scale * LOG2E);
        }
    }
    int st = launch_status();
    if (st != BPT_OK) return st;
    if (Pin->n_heavy > 0 && !grouped) {
        hipLaunchKernelGGL((k_combine_sum_v4<T>), dim3((int)Pin->n_heavy, H * D / (4 * WAVE), 1), dim3(BLOCK), 0, s, Pin->heavy,
                           (const float *)ws_rows, (T *)dq, (T *)nullptr, H * D, (size_t)0);
        st = launch_status();
        if (st != BPT_OK) return st;
    }
    // source side: dK[src] = sum ds * q[dst], dV[src] = sum p * dO[dst]
    if (!grouped) {
        ProfScope prof(BPT_KERNEL_ATTN_BWD_SRC, s);
        return run_spmm_fast<T, float, H, D, 2>(Pout, dsbuf, q, dk, pbuf, d_o, dv, ws_rows, s);
    }
    float *ws_dk = ws_rows + (size_t)Pin->n_slots * H * D, *ws_dv = ws_dk + (size_t)Pout->n_slots * H * D;
    {
        ProfScope prof(BPT_KERNEL_ATTN_BWD_SRC, s);
#define LAUNCH_SRC(RR)                                                                                                            \
    hipLaunchKernelGGL((k_attn_bwd_src_grp<T, H, D, RR, HS>), dim3(group_grid(Pout) * HS), dim3(WAVE), 0, s, *Pout, (const T *)q, \
                       (const T *)d_o, (const float2 *)pds, (T *)dk, (T *)dv, ws_dk, ws_dv)
        constexpr int HS = head_slices<T, H, D>();
        if (Pout->grp_R == 8) LAUNCH_SRC(8);
        else LAUNCH_SRC(4);
#undef LAUNCH_SRC
    }
    st = launch_status();
    if (st != BPT_OK || Pin->n_heavy + Pout->n_heavy == 0) return st;
    // partial rows of dq (destination side) and of dk, dv (source side) in one launch
    hipLaunchKernelGGL((k_combine_sum3<T>), dim3((int)(Pin->n_heavy + Pout->n_heavy), H * D / (4 * WAVE), 2), dim3(BLOCK), 0, s, Pin->heavy,
                       (int)Pin->n_heavy, (const float *)ws_rows, (T *)dq, Pout->heavy, (const float *)ws_dk, (T *)dk, (T *)dv, H * D,
                       (size_t)Pout->n_slots * H * D);
    return launch_status();
}

}  // namespace

// Workspace of bpt_attention_forward_noalloc: one copy per GPU, held until the process ends.  In host code this
// name is only a handle for hipGetSymbolAddress; kernels get the device address that call returns.
static __device__ __align__(256) unsigned char scratch[BPT_NOALLOC_SCRATCH_BYTES];

namespace {

constexpr int MAX_SCRATCH_DEVICES = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[MAX_SCRATCH_DEVICES] = {};

// device address of `scratch` on the current device (looked up once per device)
int scratch_of_current_device(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_SCRATCH_DEVICES) return BPT_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return BPT_ERR_NULL;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return BPT_OK;
}

}  // namespace

// ------------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------------
extern "C" {

const char *bpt_strerror(int status) {
    if (status > 0) return hipGetErrorString((hipError_t)status);
    switch (status) {
        case BPT_OK: return "ok";
        case BPT_ERR_NULL: return "required pointer is NULL";
        case BPT_ERR_SIZE: return "negative or inconsistent size";
        case BPT_ERR_DTYPE: return "unknown dtype";
        case BPT_ERR_SHAPE: return "h and d must be positive (h*d <= 2^20)";
        case BPT_ERR_WORKSPACE: return "workspace missing or too small";
        case BPT_ERR_PLAN: return "plans do not describe the same graph";
        case BPT_ERR_UNSUPPORTED: return "combination not implemented";
        case BPT_ERR_SCRATCH: return "the call needs more than the library's static scratch (BPT_NOALLOC_SCRATCH_BYTES)";
        default: return "unknown bptattn status";
    }
}

int64_t bpt_plan_struct_bytes(void) { return (int64_t)sizeof(bpt_plan); }

int bpt_set_force_generic(int on) { return g_force_generic.exchange(on ? 1 : 0); }

int bpt_gather_probe(const void *region, int64_t region_bytes, int waves_per_cu, int in_flight, int iters, float *sink, void *stream) {
    if (!region || !sink) return BPT_ERR_NULL;
    if (region_bytes < 1024 || region_bytes / 1024 > 0x7fffffff || waves_per_cu < WAVES_PER_BLOCK || waves_per_cu > 64 || iters < 1)
        return BPT_ERR_SIZE;
    if (!aligned16(region)) return BPT_ERR_UNSUPPORTED;
    const int grid = 256 * (waves_per_cu / WAVES_PER_BLOCK);      // 256 compute units
    const uint32_t n_rows = (uint32_t)(region_bytes / 1024);
    hipStream_t s = (hipStream_t)stream;
    switch (in_flight) {
    case 2: hipLaunchKernelGGL((k_gather_probe<2>), dim3(grid), dim3(BLOCK), 0, s, (const float4 *)region, n_rows, iters, sink); break;
    case 4: hipLaunchKernelGGL((k_gather_probe<4>), dim3(grid), dim3(BLOCK), 0, s, (const float4 *)region, n_rows, iters, sink); break;
    case 8: hipLaunchKernelGGL((k_gather_probe<8>), dim3(grid), dim3(BLOCK), 0, s, (const float4 *)region, n_rows, iters, sink); break;
    default: return BPT_ERR_SIZE;
    }
    return launch_status();
}

int bpt_profile_kernel(int which, void *start_event, void *stop_event) {
    if (which != 0 && (!start_event || !stop_event)) return BPT_ERR_NULL;
    g_prof_start.store(start_event);
    g_prof_stop.store(stop_event);
    g_prof_which.store(which);
    return BPT_OK;
}

int64_t bpt_workspace_bytes(int op, const bpt_plan *plan, const bpt_plan *plan_t, int h, int d, int dtype) {
    if (!plan || h < 1 || d < 1) return -1;
    const int64_t C = (int64_t)h * d, a = (int64_t)acc_size(dtype);
    const int64_t s0 = plan->n_slots, s1 = plan_t ? plan_t->n_slots : 0;
    switch (op) {
        case BPT_OP_MASKEDMM_BWD: return round16((s0 > s1 ? s0 : s1) * C * a);
        case BPT_OP_NODE_MUL_EDGE_BWD:
        case BPT_OP_SPMM_FWD: return round16(s0 * C * a);
        case BPT_OP_SPMM_BWD: return round16(s1 * C * a);
        case BPT_OP_ATTN_FWD: return round16(s0 * (C + 2 * h) * 4);
        case BPT_OP_SOFTMAX_FWD: return WAVE % h == 0 ? round16(s0 * h * 2 * a) : 0;      // (m, s) of every segment and head
        case BPT_OP_SOFTMAX_BWD: return WAVE % h == 0 ? round16(s0 * h * a) : 0;
        case BPT_OP_ATTN_BWD: {
            // partial rows of dq, then of dk and dv (the three are merged by one launch after the source-side kernel)
            return pds_bytes(plan, plan_t, h, d, dtype == BPT_BF16 ? 2 : 4) + round16((s0 + 2 * s1) * C * 4);
        }
        default: return -1;
    }
}

#define CHECK(expr) do { const int st_ = (expr); if (st_ != BPT_OK) return st_; } while (0)

int bpt_maskedmm_csr_forward(const bpt_plan *plan, const void *A, const void *B, void *y, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan, true));
    CHECK(check_shape(h, d, dtype));
    if (plan->n_edges > 0 && (!A || !B || !y)) return BPT_ERR_NULL;
    return sddmm(plan, A, B, y, h, d, dtype, (hipStream_t)stream);
}

int bpt_maskedmm_csr_backward(const bpt_plan *plan_r, const bpt_plan *plan_c, const void *A, const void *B, const void *dy,
                              void *dA, void *dB, void *workspace, int64_t workspace_bytes, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan_r, true));
    CHECK(check_plan(plan_c, true));
    CHECK(check_shape(h, d, dtype));
    if (plan_r->n_edges != plan_c->n_edges) return BPT_ERR_PLAN;
    if (!dA || !dB || (plan_r->n_edges > 0 && (!A || !B || !dy))) return BPT_ERR_NULL;
    const int64_t need = bpt_workspace_bytes(BPT_OP_MASKEDMM_BWD, plan_r, plan_c, h, d, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    CHECK(spmm(plan_r, dy, B, dA, workspace, h, d, dtype, (hipStream_t)stream));
    return spmm(plan_c, dy, A, dB, workspace, h, d, dtype, (hipStream_t)stream);
}

int bpt_rel_bias_forward(const bpt_plan *plan, const void *q, const void *table, const int32_t *used_types, int64_t n_used, float *bias, int h,
                         int d, int dtype, void *stream) {
    CHECK(check_plan(plan, true));
    CHECK(check_shape(h, d, dtype));
    if (plan->n_edges > 0 && (!q || !table || !bias)) return BPT_ERR_NULL;
    if (plan->bias_by_pair && !used_types) return BPT_ERR_UNSUPPORTED;      // only the kernel below writes the head-major form
    hipStream_t s = (hipStream_t)stream;
    if (used_types) {                       // plan indices are type numbers: the kernel with the table rows in LDS
        if (n_used < 0) return BPT_ERR_SIZE;
        if (!rel_rows_shape(h, d, dtype) || n_used > REL_MAX_USED || !aligned16(q) || !aligned16(table) || !aligned16(bias)) return BPT_ERR_UNSUPPORTED;
#define X(HH) if (h == HH) return run_rel_bias_rows<T, HH>(plan, q, table, used_types, n_used, bias, s);
        if (dtype == BPT_F32) { using T = float; X(4) X(8) X(16) }
        if (dtype == BPT_BF16) { using T = bf16_t; X(4) X(8) X(16) }
#undef X
        return BPT_ERR_UNSUPPORTED;
    }
    if (!fast_shape(h, d, dtype) || !aligned16(q) || !aligned16(table)) return BPT_ERR_UNSUPPORTED;
#define X(HH, DD) if (h == HH && d == DD) return run_rel_bias<T, HH, DD>(plan, q, table, bias, s);
    if (dtype == BPT_F32) { using T = float; BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { using T = bf16_t; BPT_FAST_SHAPES_BF16(X) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

int bpt_rel_bias_forward_tiles(const bpt_plan *plan, const void *q, const void *table, const int32_t *used_types, int64_t n_used,
                               const int32_t *pair_types, float *bias, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan, true));
    CHECK(check_shape(h, d, dtype));
    if (n_used < 0) return BPT_ERR_SIZE;
    if (!rel_rows_shape(h, d, dtype) || n_used > REL_MAX_USED || !has_tiles(plan, h, d, dtype == BPT_BF16 ? 2 : 4)) return BPT_ERR_UNSUPPORTED;
    if (plan->n_edges == 0) return BPT_OK;
    if (!q || !table || !used_types || !pair_types || !bias) return BPT_ERR_NULL;
    if (n_used == 0) return BPT_ERR_SIZE;                        // (edges without a type in use)
    if (!aligned16(q) || !aligned16(table)) return BPT_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
#define X(HH) if (h == HH) return run_rel_bias_tiles<T, HH>(plan, q, table, used_types, n_used, pair_types, bias, s);
    if (dtype == BPT_F32) { using T = float; X(4) X(8) X(16) }
    if (dtype == BPT_BF16) { using T = bf16_t; X(4) X(8) X(16) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

int64_t bpt_rel_bias_backward_workspace_bytes(const bpt_plan *plan, int64_t n_used, int h) {
    if (!plan || n_used < 0 || h < 1) return 0;
    return (plan->n_slots * h * 64 + n_used * REL_MAX_PARTS * 64) * 4;
}

int bpt_rel_bias_backward_supported(int64_t n_used, int h, int d, int dtype) {
    if (n_used < 0) return BPT_ERR_SIZE;
    if (!rel_rows_shape(h, d, dtype) || n_used > REL_MAX_USED) return BPT_ERR_UNSUPPORTED;
#define X(HH) if (h == HH) return rel_bias_bwd_config<T, HH>(n_used);
    if (dtype == BPT_F32) { using T = float; X(4) X(8) X(16) }
    if (dtype == BPT_BF16) { using T = bf16_t; X(4) X(8) X(16) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

int bpt_rel_bias_backward(const bpt_plan *plan, const float *ds, const void *q, const void *table, const int32_t *used,
                          const int32_t *used_types, int64_t n_types, int64_t n_used, void *dq, void *dtable, void *workspace,
                          int64_t workspace_bytes, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan, true));
    CHECK(check_shape(h, d, dtype));
    if (n_types < 0 || n_used < 0 || n_used > n_types) return BPT_ERR_SIZE;
    if (!rel_rows_shape(h, d, dtype) || n_used > REL_MAX_USED || rel_bwd_waves(n_used, h) == 0) return BPT_ERR_UNSUPPORTED;
    if (n_types == 0) return BPT_OK;
    if (!used || !dtable || (n_used > 0 && !used_types) || (plan->n_edges > 0 && (!ds || !q || !table || !dq))) return BPT_ERR_NULL;
    if (!aligned16(ds) || !aligned16(table)) return BPT_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < bpt_rel_bias_backward_workspace_bytes(plan, n_used, h) || !aligned16(workspace)) return BPT_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
#define X(HH) if (h == HH) return run_rel_bias_bwd<T, HH>(plan, ds, q, table, used, used_types, n_types, n_used, dq, dtable, (float *)workspace, s);
    if (dtype == BPT_F32) { using T = float; X(4) X(8) X(16) }
    if (dtype == BPT_BF16) { using T = bf16_t; X(4) X(8) X(16) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

int bpt_node_mul_edge_forward(const bpt_plan *plan, const void *A, const void *B, void *y, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan, false));
    CHECK(check_shape(h, d, dtype));
    if (plan->n_edges > 0 && (!A || !B || !y)) return BPT_ERR_NULL;
    if (fast_shape(h, d, dtype) && aligned16(A) && aligned16(B)) return nme_fwd_fast(plan, A, B, y, h, d, dtype, (hipStream_t)stream);
    return sddmm_edge_generic(plan, A, B, y, h, d, dtype, (hipStream_t)stream);
}

int bpt_node_mul_edge_backward(const bpt_plan *plan, const void *A, const void *B, const void *dy, void *dA, void *dB,
                               void *workspace, int64_t workspace_bytes, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan, false));
    CHECK(check_shape(h, d, dtype));
    if (!dA || (plan->n_edges > 0 && (!A || !B || !dy || !dB))) return BPT_ERR_NULL;
    const int64_t need = bpt_workspace_bytes(BPT_OP_NODE_MUL_EDGE_BWD, plan, nullptr, h, d, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    if (fast_shape(h, d, dtype) && aligned16(B) && aligned16(dA) && aligned16(workspace))
        return nme_bwd_fast(plan, A, B, dy, dA, dB, workspace, h, d, dtype, (hipStream_t)stream);
    CHECK(spmm_edge_generic(plan, dy, B, dA, workspace, h, d, dtype, (hipStream_t)stream));
    DISPATCH_DTYPE(dtype, (run_nme_dB<T>(plan, A, dy, dB, h, d, (hipStream_t)stream)))
}

int bpt_sparse_softmax_forward(const bpt_plan *plan, const void *x, void *y, void *workspace, int64_t workspace_bytes, int h,
                               int dtype, void *stream) {
    CHECK(check_plan(plan, false));
    CHECK(check_shape(h, 1, dtype));
    if (plan->n_edges > 0 && (!x || !y)) return BPT_ERR_NULL;
    const int64_t need = bpt_workspace_bytes(BPT_OP_SOFTMAX_FWD, plan, nullptr, h, 1, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    DISPATCH_DTYPE(dtype, (run_softmax_fwd<T>(plan, x, y, workspace, h, (hipStream_t)stream)))
}

int bpt_sparse_softmax_backward(const bpt_plan *plan, const void *y, const void *dy, void *dx, void *workspace,
                                int64_t workspace_bytes, int h, int dtype, void *stream) {
    CHECK(check_plan(plan, false));
    CHECK(check_shape(h, 1, dtype));
    if (plan->n_edges > 0 && (!y || !dy || !dx)) return BPT_ERR_NULL;
    const int64_t need = bpt_workspace_bytes(BPT_OP_SOFTMAX_BWD, plan, nullptr, h, 1, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    DISPATCH_DTYPE(dtype, (run_softmax_bwd<T>(plan, y, dy, dx, workspace, h, (hipStream_t)stream)))
}

int bpt_vector_spmm_forward(const bpt_plan *plan, const void *edata, const void *x, void *y, void *workspace,
                            int64_t workspace_bytes, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan, true));
    CHECK(check_shape(h, d, dtype));
    if (!y || (plan->n_edges > 0 && (!edata || !x))) return BPT_ERR_NULL;
    const int64_t need = bpt_workspace_bytes(BPT_OP_SPMM_FWD, plan, nullptr, h, d, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    return spmm(plan, edata, x, y, workspace, h, d, dtype, (hipStream_t)stream);
}

int bpt_vector_spmm_accumulate(const bpt_plan *plan, const void *edata, const void *x, void *y, void *workspace,
                               int64_t workspace_bytes, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan, true));
    CHECK(check_shape(h, d, dtype));
    if (!y || (plan->n_edges > 0 && (!edata || !x))) return BPT_ERR_NULL;
    if (plan->n_edges == 0) return BPT_OK;
    const int64_t need = bpt_workspace_bytes(BPT_OP_SPMM_FWD, plan, nullptr, h, d, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    // exists in the row-group kernels only
    if (!(fast_shape(h, d, dtype) && aligned16(x) && aligned16(y) && aligned16(workspace) && spmm_grp_ok(plan, h, d, dtype)))
        return BPT_ERR_UNSUPPORTED;
    return spmm_grp(plan, edata, x, y, workspace, h, d, dtype, (hipStream_t)stream, 1);
}

int bpt_vector_spmm_backward(const bpt_plan *plan, const bpt_plan *plan_t, const void *edata, const void *dy, const void *x,
                             void *dedata, void *dx, void *workspace, int64_t workspace_bytes, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan, true));
    CHECK(check_plan(plan_t, true));
    CHECK(check_shape(h, d, dtype));
    if (plan->n_edges != plan_t->n_edges) return BPT_ERR_PLAN;
    if (!dx || (plan->n_edges > 0 && (!edata || !dy || !x || !dedata))) return BPT_ERR_NULL;
    const int64_t need = bpt_workspace_bytes(BPT_OP_SPMM_BWD, plan, plan_t, h, d, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    CHECK(sddmm(plan, dy, x, dedata, h, d, dtype, (hipStream_t)stream));
    return spmm(plan_t, edata, dy, dx, workspace, h, d, dtype, (hipStream_t)stream);
}

int bpt_attention_forward(const bpt_plan *plan_in, const void *q, const void *k, const void *v, const float *bias, void *o,
                          float *lse, void *workspace, int64_t workspace_bytes, float scale, float dropout_p, uint64_t dropout_seed,
                          int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan_in, true));
    CHECK(check_shape(h, d, dtype));
    if (!q || !k || !v || !o || !lse) return BPT_ERR_NULL;
    if (!(dropout_p >= 0.f && dropout_p < 1.f)) return BPT_ERR_SIZE;
    const Dropout drop = make_dropout(dropout_p, dropout_seed);
    // dropout and the score term exist in the row-group and the tile kernels only
    if ((drop.thr != 0 || bias) && !has_groups(plan_in, h, d, dtype == BPT_BF16 ? 2 : 4) && !has_tiles(plan_in, h, d, dtype == BPT_BF16 ? 2 : 4))
        return BPT_ERR_UNSUPPORTED;
    if ((bias || drop.thr != 0) && !plan_in->grp_eids) return BPT_ERR_PLAN;
    // only the tile kernels look the rows of the score term up in a numbering of the plan's own
    if (bias && plan_in->bias_by_pair && !has_tiles(plan_in, h, d, dtype == BPT_BF16 ? 2 : 4)) return BPT_ERR_PLAN;
    if (!fast_shape(h, d, dtype) || !aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(workspace))
        return BPT_ERR_UNSUPPORTED;
    const int64_t need = bpt_workspace_bytes(BPT_OP_ATTN_FWD, plan_in, nullptr, h, d, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
#define X(HH, DD) if (h == HH && d == DD) return run_attn_fwd<T, HH, DD>(plan_in, q, k, v, o, lse, workspace, scale, drop, bias, s);
    if (dtype == BPT_F32) { using T = float; BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { using T = bf16_t; BPT_FAST_SHAPES_BF16(X) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

int bpt_attention_forward_noalloc(const bpt_plan *plan_in, const void *q, const void *k, const void *v, const float *bias, void *o,
                                  float *lse, float scale, float dropout_p, uint64_t dropout_seed, int h, int d, int dtype,
                                  void *stream) {
    CHECK(check_plan(plan_in, true));
    CHECK(check_shape(h, d, dtype));
    const int64_t need = bpt_workspace_bytes(BPT_OP_ATTN_FWD, plan_in, nullptr, h, d, dtype);
    if (need < 0) return BPT_ERR_SIZE;
    if (need > (int64_t)BPT_NOALLOC_SCRATCH_BYTES) return BPT_ERR_SCRATCH;
    void *ws = nullptr;
    CHECK(scratch_of_current_device(&ws));
    return bpt_attention_forward(plan_in, q, k, v, bias, o, lse, ws, (int64_t)BPT_NOALLOC_SCRATCH_BYTES, scale, dropout_p, dropout_seed,
                                 h, d, dtype, stream);
}

int bpt_attention_backward(const bpt_plan *plan_in, const bpt_plan *plan_out, const void *q, const void *k, const void *v,
                           const float *bias, const void *o, const void *d_o, const float *lse, void *dq, void *dk, void *dv,
                           float *ds_out, void *workspace, int64_t workspace_bytes, float scale, float dropout_p,
                           uint64_t dropout_seed, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan_in, true));
    CHECK(check_plan(plan_out, true));
    CHECK(check_shape(h, d, dtype));
    if (!(dropout_p >= 0.f && dropout_p < 1.f)) return BPT_ERR_SIZE;
    const Dropout drop = make_dropout(dropout_p, dropout_seed);
    if ((drop.thr != 0 || bias) && !grouped_backward(plan_in, plan_out, h, d, dtype == BPT_BF16 ? 2 : 4) &&
        !tiled_backward(plan_in, plan_out, h, d, dtype == BPT_BF16 ? 2 : 4))
        return BPT_ERR_UNSUPPORTED;
    if ((bias != nullptr) != (ds_out != nullptr)) return BPT_ERR_NULL;       // the score term and its gradient go together
    if ((bias || drop.thr != 0) && !plan_in->grp_eids) return BPT_ERR_PLAN;
    if (bias && plan_in->bias_by_pair && !tiled_backward(plan_in, plan_out, h, d, dtype == BPT_BF16 ? 2 : 4)) return BPT_ERR_PLAN;
    // (the two sides may have different row counts: attention to a memory of another length, attention.py:144-168)
    if (plan_in->n_edges != plan_out->n_edges) return BPT_ERR_PLAN;
    if (!q || !k || !v || !o || !d_o || !lse || !dq || !dk || !dv) return BPT_ERR_NULL;
    if (!fast_shape(h, d, dtype) || !aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(d_o) ||
        !aligned16(dq) || !aligned16(dk) || !aligned16(dv) || !aligned16(workspace))
        return BPT_ERR_UNSUPPORTED;
    const int64_t need = bpt_workspace_bytes(BPT_OP_ATTN_BWD, plan_in, plan_out, h, d, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
#define X(HH, DD) \
    if (h == HH && d == DD) return run_attn_bwd<T, HH, DD>(plan_in, plan_out, q, k, v, o, d_o, lse, dq, dk, dv, workspace, scale, drop, bias, ds_out, s);
    if (dtype == BPT_F32) { using T = float; BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { using T = bf16_t; BPT_FAST_SHAPES_BF16(X) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

}  // extern "C"
