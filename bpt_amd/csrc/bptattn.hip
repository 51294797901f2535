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

#include "../../include/bptattn.h"

namespace {

constexpr int WAVE = 64;
constexpr int WAVES_PER_BLOCK = 4;
constexpr int BLOCK = WAVE * WAVES_PER_BLOCK;
constexpr float M_INIT_LOG2 = -1.4426950408889634e9f;   // -1e9 (graphop_kernel.cu:428) in base-2 units
constexpr float LOG2E = 1.4426950408889634f;

std::atomic<int> g_force_generic{0};
// tuning of the row-group kernels, one value per kernel (fwd, bwd_dst, bwd_src): 4 = batches of four
// neighbour rows; 2 = batches of two; 3 = batches of two compiled for three waves per SIMD
std::atomic<int> g_group_variant[3] = {{2}, {2}, {2}};
// wavefronts per XCD that walk the groups of that XCD's chunk (0: one wavefront per group)
std::atomic<int> g_group_waves[3] = {{0}, {0}, {0}};

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
__global__ __launch_bounds__(BLOCK) void k_combine_sum(const int32_t *__restrict__ heavy,
                                                       const typename Elem<T>::acc_t *__restrict__ ws, T *__restrict__ Y0,
                                                       T *__restrict__ Y1, int C, size_t ws_stride) {
    using acc_t = typename Elem<T>::acc_t;
    __shared__ acc_t part[WAVES_PER_BLOCK][WAVE];
    const int row = heavy[3 * blockIdx.x], s0 = heavy[3 * blockIdx.x + 1], ns = heavy[3 * blockIdx.x + 2];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int j = blockIdx.y * WAVE + lane;
    T *Y = blockIdx.z == 0 ? Y0 : Y1;
    acc_t s = 0;
    if (j < C) {
        const acc_t *col = ws + (size_t)blockIdx.z * ws_stride + (size_t)s0 * C + j;
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
        Elem<T>::st(Y + (size_t)row * C + j, r);
    }
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

// y[eid[p], head] = A[row, head, :] . B[idx[p], head, :]
template <typename T, int H, int D, int BATCH>
__global__ __launch_bounds__(BLOCK) void k_sddmm_fast(bpt_plan P, const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ y) {
    using L = Lay<T, H, D>;
    Item it;
    if (!fetch_item(P, it)) return;
    const int lane = threadIdx.x & 63, head = lane / L::LPH;
    float a[L::EPL];
    load_row<T, H, D>(A + (size_t)it.row * L::C, lane, a);
    for (int p0 = it.begin; p0 < it.end; p0 += WAVE) {
        const int cnt = min(WAVE, it.end - p0);
        const int my_idx = lane < cnt ? P.idx[p0 + lane] : 0;
        const int my_eid = lane < cnt ? P.eid[p0 + lane] : 0;
        for (int b = 0; b < cnt; b += BATCH) {
            float bv[BATCH][L::EPL];
            int ee[BATCH];
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                const int j = (b + e < cnt) ? b + e : b;
                ee[e] = __builtin_amdgcn_readlane(my_eid, j);
                load_row<T, H, D>(B + (size_t)__builtin_amdgcn_readlane(my_idx, j) * L::C, lane, bv[e]);
            }
            issue_loads_first();
#pragma unroll
            for (int e = 0; e < BATCH; ++e) {
                const float s = head_sum<L::LPH>(dot_n<L::EPL>(a, bv[e]));
                if (b + e < cnt && lane % L::LPH == 0) Elem<T>::st(y + (size_t)ee[e] * H + head, s);
            }
        }
    }
}

// Y0[row] = sum_p W0[eid[p], head] * X0[idx[p]]  (and the same with W1, X1 -> Y1 when NOUT == 2)
template <typename T, typename WT, int H, int D, int BATCH, int NOUT>
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
        const int my_idx = lane < cnt ? P.idx[p0 + lane] : 0;
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
                load_row<T, H, D>(X0 + (size_t)src * L::C, lane, x0[e]);
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
// row-group kernels of the fused path: one wavefront owns up to R rows (or row segments) that
// share neighbours; every neighbour row of the group's union is loaded once and used for all
// members that have an edge to it (entry mask).  One wavefront per workgroup.
// ------------------------------------------------------------------------------------------
template <int R> struct GroupHead {
    int rows[R], slots[R], begin, end;
};

template <int R> __device__ __forceinline__ GroupHead<R> fetch_group(const bpt_plan &P, int g) {
    GroupHead<R> gh;
#pragma unroll
    for (int m = 0; m < R; ++m) {
        gh.rows[m] = __builtin_amdgcn_readfirstlane(P.grp_members[((size_t)g * R + m) * 2]);
        gh.slots[m] = __builtin_amdgcn_readfirstlane(P.grp_members[((size_t)g * R + m) * 2 + 1]);
    }
    gh.begin = __builtin_amdgcn_readfirstlane(P.grp_ptr[g]);
    gh.end = __builtin_amdgcn_readfirstlane(P.grp_ptr[g + 1]);
    return gh;
}

// Persistent walk over the groups of one XCD chunk.  Workgroup b (one wavefront) runs on XCD b % 8; it
// takes the groups first + b/8, + stride, + 2*stride, ... of that XCD's chunk, stride = gridDim.x / 8.
// A group costs a chain of dependent loads before its first FMA (header -> entries -> rows); the walk
// hides it by fetching the header two groups ahead and the first 64 entries one group ahead.  With
// gridDim.x = 8 * (largest chunk) every wavefront gets exactly one group.
template <int R, class Body>
__device__ __forceinline__ void walk_groups(const bpt_plan &P, Body &&body) {
    const int x = blockIdx.x & 7, w = blockIdx.x >> 3, stride = gridDim.x >> 3;
    const int first = __builtin_amdgcn_readfirstlane(P.grp_chunks[x]), last = __builtin_amdgcn_readfirstlane(P.grp_chunks[x + 1]);
    int g = first + w;
    if (g >= last) return;
    const int lane = threadIdx.x;
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
    GroupHead<R> cur = fetch_group<R>(P, g);
    GroupHead<R> nxt = fetch_group<R>(P, min(g + stride, last - 1));
    int4 ent_cur = lane < min(WAVE, cur.end - cur.begin) ? entries[cur.begin + lane] : make_int4(0, 0, 0, 0);
    for (; g < last; g += stride) {
        const GroupHead<R> nn = fetch_group<R>(P, min(g + 2 * stride, last - 1));
        const int ncnt = g + stride < last ? min(WAVE, nxt.end - nxt.begin) : 0;
        const int4 ent_nxt = lane < ncnt ? entries[nxt.begin + lane] : make_int4(0, 0, 0, 0);
        body(cur, ent_cur);
        cur = nxt;
        nxt = nn;
        ent_cur = ent_nxt;
    }
}

// All three kernels run the same two-stage software pipeline over a group's entries: while the rows
// of batch i are being used, the loads of batch i+1 are already in flight (two register buffers,
// unconditional loads: a batch past the end re-reads the chunk's first row with an empty mask).
template <typename T, int H, int D, int R, int BATCH, int WPE>
__global__ __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(WPE))) void k_attn_fwd_grp(
    bpt_plan P, const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v, T *__restrict__ o,
    float *__restrict__ lse, float *__restrict__ ws_acc, float *__restrict__ ws_ml, float scale_log2e) {
    using L = Lay<T, H, D>;
    const int lane = threadIdx.x, head = lane / L::LPH;
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
    struct Batch {
        float kv[BATCH][L::EPL], vv[BATCH][L::EPL];
        int mk[BATCH], any;
    };
    walk_groups<R>(P, [&](const GroupHead<R> &gh, const int4 &ent0) {
        float qv[R][L::EPL], acc[R][L::EPL], mrun[R], lrun[R];
#pragma unroll
        for (int m = 0; m < R; ++m) {
            load_row<T, H, D>(q + (size_t)max(gh.rows[m], 0) * L::C, lane, qv[m]);
            mrun[m] = M_INIT_LOG2;
            lrun[m] = 0.f;
#pragma unroll
            for (int i = 0; i < L::EPL; ++i) { qv[m][i] *= scale_log2e; acc[m][i] = 0.f; }
        }
        for (int p0 = gh.begin; p0 < gh.end; p0 += WAVE) {
            const int cnt = min(WAVE, gh.end - p0);
            int4 ent = ent0;
            if (p0 != gh.begin) ent = lane < cnt ? entries[p0 + lane] : make_int4(0, 0, 0, 0);
            auto load_batch = [&](Batch &B, int b) {
                B.any = 0;
#pragma unroll
                for (int e = 0; e < BATCH; ++e) {
                    const bool ok = b + e < cnt;
                    const int j = ok ? b + e : 0;
                    const int src = __builtin_amdgcn_readlane(ent.x, j);
                    B.mk[e] = ok ? __builtin_amdgcn_readlane(ent.y, j) : 0;
                    B.any |= B.mk[e];
#ifdef BPT_PROBE_NO_LOADS
#pragma unroll
                    for (int i = 0; i < L::EPL; ++i) { B.kv[e][i] = qv[0][i] + (float)src; B.vv[e][i] = qv[1][i] - (float)src; }
#else
                    load_row<T, H, D>(k + (size_t)src * L::C, lane, B.kv[e]);
                    load_row<T, H, D>(v + (size_t)src * L::C, lane, B.vv[e]);
#endif
                }
            };
            auto compute = [&](const Batch &B) {
#ifdef BPT_PROBE_NO_MATH
#pragma unroll
                for (int e = 0; e < BATCH; ++e) acc[0][0] += B.kv[e][0] + B.vv[e][0] + B.kv[e][L::EPL - 1] + B.vv[e][L::EPL - 1];
                return;
#endif
#pragma unroll
                for (int m = 0; m < R; ++m) {
                    const int bit = 1 << m;
                    if ((B.any & bit) == 0) continue;
                    float s[BATCH], mx = mrun[m];
#pragma unroll
                    for (int e = 0; e < BATCH; ++e) {
                        s[e] = -INFINITY;
                        if (B.mk[e] & bit) {
                            s[e] = head_sum<L::LPH>(dot_n<L::EPL>(qv[m], B.kv[e]));
                            mx = fmaxf(mx, s[e]);
                        }
                    }
                    const float alpha = __builtin_amdgcn_exp2f(mrun[m] - mx);
                    lrun[m] *= alpha;
#pragma unroll
                    for (int i = 0; i < L::EPL; ++i) acc[m][i] *= alpha;
#pragma unroll
                    for (int e = 0; e < BATCH; ++e) {
                        if (B.mk[e] & bit) {
                            const float pe = __builtin_amdgcn_exp2f(s[e] - mx);
                            lrun[m] += pe;
#pragma unroll
                            for (int i = 0; i < L::EPL; ++i) acc[m][i] = fmaf(pe, B.vv[e][i], acc[m][i]);
                        }
                    }
                    mrun[m] = mx;
                }
            };
            Batch A, B;
            load_batch(A, 0);
            for (int b = 0; b < cnt; b += 2 * BATCH) {
                load_batch(B, b + BATCH);
                issue_loads_first();
                compute(A);
                issue_loads_first();
                load_batch(A, b + 2 * BATCH);
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
                for (int i = 0; i < L::EPL; ++i) acc[m][i] *= inv;
                store_row<T, H, D>(o + (size_t)gh.rows[m] * L::C, lane, acc[m]);
                if (lane % L::LPH == 0) lse[(size_t)gh.rows[m] * H + head] = lrun[m] > 0.f ? mrun[m] + log2f(lrun[m]) : 0.f;
            } else {
                store_row_ws<T, H, D>(ws_acc + (size_t)gh.slots[m] * L::C, lane, acc[m]);
                if (lane % L::LPH == 0) {
                    ws_ml[((size_t)gh.slots[m] * H + head) * 2] = mrun[m];
                    ws_ml[((size_t)gh.slots[m] * H + head) * 2 + 1] = lrun[m];
                }
            }
        }
    });
}

// Backward, destination side, row groups.  pds[(pair, head)] = (p, ds) in the pair order of the
// source-side plan (P.grp_pairs maps this plan's pairs to it).
template <typename T, int H, int D, int R, int BATCH, int WPE>
__global__ __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(WPE))) void k_attn_bwd_dst_grp(
    bpt_plan P, const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v, const T *__restrict__ o,
    const T *__restrict__ d_o, const float *__restrict__ lse, T *__restrict__ dq, float2 *__restrict__ pds,
    float *__restrict__ ws_dq, float scale, float scale_log2e) {
    using L = Lay<T, H, D>;
    const int lane = threadIdx.x, head = lane / L::LPH;
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
    const int last_pair = (int)P.n_edges - 1;
    struct Batch {
        float kv[BATCH][L::EPL], vv[BATCH][L::EPL];
        int mk[BATCH], xp[BATCH], any;
    };
    walk_groups<R>(P, [&](const GroupHead<R> &gh, const int4 &ent0) {
        float qv[R][L::EPL], dov[R][L::EPL], dqa[R][L::EPL], delta[R], lse2[R];
#pragma unroll
        for (int m = 0; m < R; ++m) {
            const size_t row = (size_t)max(gh.rows[m], 0);
            float ov[L::EPL];
            load_row<T, H, D>(o + row * L::C, lane, ov);
            load_row<T, H, D>(d_o + row * L::C, lane, dov[m]);
            load_row<T, H, D>(q + row * L::C, lane, qv[m]);
            delta[m] = head_sum<L::LPH>(dot_n<L::EPL>(dov[m], ov));
            lse2[m] = lse[row * H + head];
#pragma unroll
            for (int i = 0; i < L::EPL; ++i) dqa[m][i] = 0.f;
        }
        for (int p0 = gh.begin; p0 < gh.end; p0 += WAVE) {
            const int cnt = min(WAVE, gh.end - p0);
            int4 ent = ent0;
            if (p0 != gh.begin) ent = lane < cnt ? entries[p0 + lane] : make_int4(0, 0, 0, 0);
            auto load_batch = [&](Batch &B, int b) {
                B.any = 0;
#pragma unroll
                for (int e = 0; e < BATCH; ++e) {
                    const bool ok = b + e < cnt;
                    const int j = ok ? b + e : 0;
                    const int src = __builtin_amdgcn_readlane(ent.x, j);
                    B.mk[e] = ok ? __builtin_amdgcn_readlane(ent.y, j) : 0;
                    B.any |= B.mk[e];
                    // lane r (< R) fetches the scratch position of this entry's r-th pair
                    B.xp[e] = P.grp_pairs[min(__builtin_amdgcn_readlane(ent.z, j) + (lane & (R - 1)), last_pair)];
                    load_row<T, H, D>(k + (size_t)src * L::C, lane, B.kv[e]);
                    load_row<T, H, D>(v + (size_t)src * L::C, lane, B.vv[e]);
                }
            };
            auto compute = [&](const Batch &B) {
#pragma unroll
                for (int m = 0; m < R; ++m) {
                    const int bit = 1 << m;
                    if ((B.any & bit) == 0) continue;
#pragma unroll
                    for (int e = 0; e < BATCH; ++e) {
                        if (B.mk[e] & bit) {
                            const int pos = __builtin_amdgcn_readlane(B.xp[e], __builtin_popcount(B.mk[e] & (bit - 1)));
                            const float s = head_sum<L::LPH>(dot_n<L::EPL>(qv[m], B.kv[e]));
                            const float dp = head_sum<L::LPH>(dot_n<L::EPL>(dov[m], B.vv[e]));
                            const float pe = __builtin_amdgcn_exp2f(fmaf(s, scale_log2e, -lse2[m]));
                            const float ds = pe * (dp - delta[m]) * scale;
#pragma unroll
                            for (int i = 0; i < L::EPL; ++i) dqa[m][i] = fmaf(ds, B.kv[e][i], dqa[m][i]);
                            if (lane % L::LPH == 0) pds[(size_t)pos * H + head] = make_float2(pe, ds);
                        }
                    }
                }
            };
            Batch A, B;
            load_batch(A, 0);
            for (int b = 0; b < cnt; b += 2 * BATCH) {
                load_batch(B, b + BATCH);
                issue_loads_first();
                compute(A);
                issue_loads_first();
                load_batch(A, b + 2 * BATCH);
                issue_loads_first();
                compute(B);
                issue_loads_first();
            }
        }
#pragma unroll
        for (int m = 0; m < R; ++m) {
            if (gh.rows[m] < 0) continue;
            if (gh.slots[m] < 0) store_row<T, H, D>(dq + (size_t)gh.rows[m] * L::C, lane, dqa[m]);
            else store_row_ws<T, H, D>(ws_dq + (size_t)gh.slots[m] * L::C, lane, dqa[m]);
        }
    });
}

// Backward, source side, row groups: dK[src] = sum ds * q[dst], dV[src] = sum p * dO[dst]; the (p, ds)
// of this plan's pair number n sits at pds[n].
template <typename T, int H, int D, int R, int BATCH, int WPE>
__global__ __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(WPE))) void k_attn_bwd_src_grp(
    bpt_plan P, const T *__restrict__ q, const T *__restrict__ d_o, const float2 *__restrict__ pds, T *__restrict__ dk,
    T *__restrict__ dv, float *__restrict__ ws_dk, float *__restrict__ ws_dv) {
    using L = Lay<T, H, D>;
    const int lane = threadIdx.x, head = lane / L::LPH;
    const int4 *entries = reinterpret_cast<const int4 *>(P.grp_entries);
    struct Batch {
        float qr[BATCH][L::EPL], dr[BATCH][L::EPL];
        float2 w[BATCH][R];
        int mk[BATCH];
    };
    walk_groups<R>(P, [&](const GroupHead<R> &gh, const int4 &ent0) {
        float ak[R][L::EPL], av[R][L::EPL];
#pragma unroll
        for (int m = 0; m < R; ++m)
#pragma unroll
            for (int i = 0; i < L::EPL; ++i) { ak[m][i] = 0.f; av[m][i] = 0.f; }
        for (int p0 = gh.begin; p0 < gh.end; p0 += WAVE) {
            const int cnt = min(WAVE, gh.end - p0);
            int4 ent = ent0;
            if (p0 != gh.begin) ent = lane < cnt ? entries[p0 + lane] : make_int4(0, 0, 0, 0);
            auto load_batch = [&](Batch &B, int b) {
#pragma unroll
                for (int e = 0; e < BATCH; ++e) {
                    const bool ok = b + e < cnt;
                    const int j = ok ? b + e : 0;
                    const int dst = __builtin_amdgcn_readlane(ent.x, j);
                    B.mk[e] = ok ? __builtin_amdgcn_readlane(ent.y, j) : 0;
                    const int pb = __builtin_amdgcn_readlane(ent.z, j);
                    load_row<T, H, D>(q + (size_t)dst * L::C, lane, B.qr[e]);
                    load_row<T, H, D>(d_o + (size_t)dst * L::C, lane, B.dr[e]);
#pragma unroll
                    for (int m = 0; m < R; ++m) {
                        B.w[e][m] = make_float2(0.f, 0.f);
                        if (B.mk[e] & (1 << m))
                            B.w[e][m] = pds[(size_t)(pb + __builtin_popcount(B.mk[e] & ((1 << m) - 1))) * H + head];
                    }
                }
            };
            auto compute = [&](const Batch &B) {
#pragma unroll
                for (int e = 0; e < BATCH; ++e) {
#pragma unroll
                    for (int m = 0; m < R; ++m) {
                        if (B.mk[e] & (1 << m)) {
#pragma unroll
                            for (int i = 0; i < L::EPL; ++i) {
                                ak[m][i] = fmaf(B.w[e][m].y, B.qr[e][i], ak[m][i]);
                                av[m][i] = fmaf(B.w[e][m].x, B.dr[e][i], av[m][i]);
                            }
                        }
                    }
                }
            };
            Batch A, B;
            load_batch(A, 0);
            for (int b = 0; b < cnt; b += 2 * BATCH) {
                load_batch(B, b + BATCH);
                issue_loads_first();
                compute(A);
                issue_loads_first();
                load_batch(A, b + 2 * BATCH);
                issue_loads_first();
                compute(B);
                issue_loads_first();
            }
        }
#pragma unroll
        for (int m = 0; m < R; ++m) {
            if (gh.rows[m] < 0) continue;
            if (gh.slots[m] < 0) {
                store_row<T, H, D>(dk + (size_t)gh.rows[m] * L::C, lane, ak[m]);
                store_row<T, H, D>(dv + (size_t)gh.rows[m] * L::C, lane, av[m]);
            } else {
                store_row_ws<T, H, D>(ws_dk + (size_t)gh.slots[m] * L::C, lane, ak[m]);
                store_row_ws<T, H, D>(ws_dv + (size_t)gh.slots[m] * L::C, lane, av[m]);
            }
        }
    });
}

// ------------------------------------------------------------------------------------------
// team kernels of the fused path.  A team = one group of up to 16 rows (grp_R == 16) handled by a
// workgroup of 4 wavefronts; wavefront w keeps the state of members 4w .. 4w+3 in registers.  The
// team's neighbour rows are fetched from global memory ONCE per team: at every stage of TEAM_S = 4
// entries wavefront w loads the two rows of entry 4*stage + w into registers (one stage ahead),
// writes them to LDS in lane-major order (float4 slot c*64 + lane, conflict free), and after one
// barrier every wavefront reads the rows its own members need (nibble w of the entry's 16-bit
// mask).  LDS is double buffered, so there is one barrier per stage.  This turns the L2->L1
// traffic of the single-wavefront row groups (each wavefront fetching its own union) into LDS reads.
// ------------------------------------------------------------------------------------------
constexpr int TEAM_WAVES = 4, TEAM_RW = 4, TEAM_R = TEAM_WAVES * TEAM_RW, TEAM_S = 4;

// Workgroup b runs on XCD b % 8 and takes the (b / 8)-th team of that XCD's chunk (-1: none).
__device__ __forceinline__ int team_index(const bpt_plan &P) {
    const int x = blockIdx.x & 7, kk = blockIdx.x >> 3;
    const int first = P.grp_chunks[x], last = P.grp_chunks[x + 1];
    return first + kk < last ? first + kk : -1;
}

template <int EPL> __device__ __forceinline__ void lds_put_row(float4 *slot, int lane, const float (&r)[EPL]) {
#pragma unroll
    for (int c = 0; c < EPL / 4; ++c) slot[c * WAVE + lane] = make_float4(r[4 * c], r[4 * c + 1], r[4 * c + 2], r[4 * c + 3]);
}
template <int EPL> __device__ __forceinline__ void lds_get_row(const float4 *slot, int lane, float (&r)[EPL]) {
#pragma unroll
    for (int c = 0; c < EPL / 4; ++c) {
        const float4 v = slot[c * WAVE + lane];
        r[4 * c] = v.x; r[4 * c + 1] = v.y; r[4 * c + 2] = v.z; r[4 * c + 3] = v.w;
    }
}

// Entry descriptors of up to 128 consecutive entries, two per lane (fetched with two vector loads per
// wavefront); field f of entry j is read with v_readlane, so no memory access sits between stages.
struct TeamDesc {
    int4 lo, hi;
    __device__ __forceinline__ void fetch(const int4 *ent, int count, int lane) {
        lo = lane < count ? ent[lane] : make_int4(0, 0, 0, 0);
        hi = lane + WAVE < count ? ent[lane + WAVE] : make_int4(0, 0, 0, 0);
    }
    __device__ __forceinline__ int idx(int j) const { return j < WAVE ? __builtin_amdgcn_readlane(lo.x, j) : __builtin_amdgcn_readlane(hi.x, j - WAVE); }
    __device__ __forceinline__ int mask(int j) const { return j < WAVE ? __builtin_amdgcn_readlane(lo.y, j) : __builtin_amdgcn_readlane(hi.y, j - WAVE); }
    __device__ __forceinline__ int pair0(int j) const { return j < WAVE ? __builtin_amdgcn_readlane(lo.z, j) : __builtin_amdgcn_readlane(hi.z, j - WAVE); }
};
constexpr int TEAM_SPAN = 2 * WAVE;      // entries per descriptor fetch

template <typename T, int H, int D>
__global__ __launch_bounds__(BLOCK) void k_attn_fwd_team(bpt_plan P, const T *__restrict__ q, const T *__restrict__ k,
                                                         const T *__restrict__ v, T *__restrict__ o, float *__restrict__ lse,
                                                         float *__restrict__ ws_acc, float *__restrict__ ws_ml, float scale_log2e) {
    using L = Lay<T, H, D>;
    constexpr int S = TEAM_S, RW = TEAM_RW, F4 = L::EPL / 4;
    __shared__ float4 lds[2][S][2][F4 * WAVE];
    const int t = team_index(P);
    if (t < 0) return;
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), head = lane / L::LPH;
    int rows[RW], slots[RW];
#pragma unroll
    for (int m = 0; m < RW; ++m) {
        rows[m] = __builtin_amdgcn_readfirstlane(P.grp_members[((size_t)t * TEAM_R + w * RW + m) * 2]);
        slots[m] = __builtin_amdgcn_readfirstlane(P.grp_members[((size_t)t * TEAM_R + w * RW + m) * 2 + 1]);
    }
    const int begin = __builtin_amdgcn_readfirstlane(P.grp_ptr[t]);
    const int n = __builtin_amdgcn_readfirstlane(P.grp_ptr[t + 1]) - begin;
    const int4 *ent = reinterpret_cast<const int4 *>(P.grp_entries) + begin;

    float qv[RW][L::EPL], acc[RW][L::EPL], mrun[RW], lrun[RW];
#pragma unroll
    for (int m = 0; m < RW; ++m) {
        load_row<T, H, D>(q + (size_t)max(rows[m], 0) * L::C, lane, qv[m]);
        mrun[m] = M_INIT_LOG2;
        lrun[m] = 0.f;
#pragma unroll
        for (int i = 0; i < L::EPL; ++i) { qv[m][i] *= scale_log2e; acc[m][i] = 0.f; }
    }
    // two stages of row loads are in flight per wavefront: register set A holds even stages, B odd ones
    struct StageRegs { float ra[L::EPL], rb[L::EPL]; };
    for (int c0 = 0; c0 < n; c0 += TEAM_SPAN) {
        const int cnt = min(TEAM_SPAN, n - c0);
        const int n_stage = (cnt + S - 1) / S;
        TeamDesc dsc;
        dsc.fetch(ent + c0, cnt, lane);
        auto stage_load = [&](StageRegs &R, int st) {
            const int j = st * S + w;
            const int idx = j < cnt ? dsc.idx(j) : 0;
            load_row<T, H, D>(k + (size_t)idx * L::C, lane, R.ra);
            load_row<T, H, D>(v + (size_t)idx * L::C, lane, R.rb);
        };
        auto stage_write = [&](const StageRegs &R, int buf) {
            lds_put_row<L::EPL>(lds[buf][w][0], lane, R.ra);
            lds_put_row<L::EPL>(lds[buf][w][1], lane, R.rb);
        };
        auto stage_compute = [&](int st, int buf) {
            int mk[S], any = 0;
#pragma unroll
            for (int e = 0; e < S; ++e) {
                const int j = st * S + e;
                mk[e] = j < cnt ? (dsc.mask(j) >> (w * RW)) & ((1 << RW) - 1) : 0;
                any |= mk[e];
            }
            if (any == 0) return;
            float sc[RW][S];
            // K phase: scores of this stage
#pragma unroll
            for (int e = 0; e < S; ++e) {
                if (mk[e] == 0) continue;
                float kr[L::EPL];
                lds_get_row<L::EPL>(lds[buf][e][0], lane, kr);
#pragma unroll
                for (int m = 0; m < RW; ++m)
                    if (mk[e] & (1 << m)) sc[m][e] = head_sum<L::LPH>(dot_n<L::EPL>(qv[m], kr));
            }
            // one running-maximum update (and accumulator rescale) per member and stage
#pragma unroll
            for (int m = 0; m < RW; ++m) {
                if ((any & (1 << m)) == 0) continue;
                float mx = mrun[m];
#pragma unroll
                for (int e = 0; e < S; ++e)
                    if (mk[e] & (1 << m)) mx = fmaxf(mx, sc[m][e]);
                const float alpha = __builtin_amdgcn_exp2f(mrun[m] - mx);
                lrun[m] *= alpha;
#pragma unroll
                for (int i = 0; i < L::EPL; ++i) acc[m][i] *= alpha;
                mrun[m] = mx;
            }
            // V phase
#pragma unroll
            for (int e = 0; e < S; ++e) {
                if (mk[e] == 0) continue;
                float vr[L::EPL];
                lds_get_row<L::EPL>(lds[buf][e][1], lane, vr);
#pragma unroll
                for (int m = 0; m < RW; ++m) {
                    if (mk[e] & (1 << m)) {
                        const float pe = __builtin_amdgcn_exp2f(sc[m][e] - mrun[m]);
                        lrun[m] += pe;
#pragma unroll
                        for (int i = 0; i < L::EPL; ++i) acc[m][i] = fmaf(pe, vr[i], acc[m][i]);
                    }
                }
            }
        };
        StageRegs A, B;
        stage_load(A, 0);
        stage_load(B, 1);
        stage_write(A, 0);
        stage_load(A, 2);
        __syncthreads();
        for (int st = 0; st < n_stage; st += 2) {
            stage_compute(st, 0);
            issue_loads_first();
            stage_write(B, 1);         // B holds stage st + 1
            stage_load(B, st + 3);
            __syncthreads();
            stage_compute(st + 1, 1);  // masks are empty past the last stage
            issue_loads_first();
            stage_write(A, 0);         // A holds stage st + 2
            stage_load(A, st + 4);
            __syncthreads();
        }
    }
#pragma unroll
    for (int m = 0; m < RW; ++m) {
        if (rows[m] < 0) continue;
        if (slots[m] < 0) {
            const float inv = lrun[m] > 0.f ? 1.f / lrun[m] : 0.f;
#pragma unroll
            for (int i = 0; i < L::EPL; ++i) acc[m][i] *= inv;
            store_row<T, H, D>(o + (size_t)rows[m] * L::C, lane, acc[m]);
            if (lane % L::LPH == 0) lse[(size_t)rows[m] * H + head] = lrun[m] > 0.f ? mrun[m] + log2f(lrun[m]) : 0.f;
        } else {
            store_row_ws<T, H, D>(ws_acc + (size_t)slots[m] * L::C, lane, acc[m]);
            if (lane % L::LPH == 0) {
                ws_ml[((size_t)slots[m] * H + head) * 2] = mrun[m];
                ws_ml[((size_t)slots[m] * H + head) * 2 + 1] = lrun[m];
            }
        }
    }
}

// Backward, destination side, teams.  pds[(pair, head)] = (p, ds) in the pair order of the source-side plan.
template <typename T, int H, int D>
__global__ __launch_bounds__(BLOCK) void k_attn_bwd_dst_team(bpt_plan P, const T *__restrict__ q, const T *__restrict__ k,
                                                             const T *__restrict__ v, const T *__restrict__ o, const T *__restrict__ d_o,
                                                             const float *__restrict__ lse, T *__restrict__ dq, float2 *__restrict__ pds,
                                                             float *__restrict__ ws_dq, float scale, float scale_log2e) {
    using L = Lay<T, H, D>;
    constexpr int S = TEAM_S, RW = TEAM_RW, F4 = L::EPL / 4;
    static_assert(S * TEAM_R == WAVE, "one lane per (entry of the stage, pair of the entry)");
    __shared__ float4 lds[2][S][2][F4 * WAVE];
    const int t = team_index(P);
    if (t < 0) return;
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), head = lane / L::LPH;
    int rows[RW], slots[RW];
#pragma unroll
    for (int m = 0; m < RW; ++m) {
        rows[m] = __builtin_amdgcn_readfirstlane(P.grp_members[((size_t)t * TEAM_R + w * RW + m) * 2]);
        slots[m] = __builtin_amdgcn_readfirstlane(P.grp_members[((size_t)t * TEAM_R + w * RW + m) * 2 + 1]);
    }
    const int begin = __builtin_amdgcn_readfirstlane(P.grp_ptr[t]);
    const int n = __builtin_amdgcn_readfirstlane(P.grp_ptr[t + 1]) - begin;
    const int4 *ent = reinterpret_cast<const int4 *>(P.grp_entries) + begin;
    const int last_pair = (int)P.n_edges - 1;

    float qv[RW][L::EPL], dov[RW][L::EPL], dqa[RW][L::EPL], delta[RW], lse2[RW];
#pragma unroll
    for (int m = 0; m < RW; ++m) {
        const size_t row = (size_t)max(rows[m], 0);
        float ov[L::EPL];
        load_row<T, H, D>(o + row * L::C, lane, ov);
        load_row<T, H, D>(d_o + row * L::C, lane, dov[m]);
        load_row<T, H, D>(q + row * L::C, lane, qv[m]);
        delta[m] = head_sum<L::LPH>(dot_n<L::EPL>(dov[m], ov));
        lse2[m] = lse[row * H + head];
#pragma unroll
        for (int i = 0; i < L::EPL; ++i) dqa[m][i] = 0.f;
    }
    // xp: lane e*16 + r holds the scratch position of pair r of entry e of the stage
    struct StageRegs { float ra[L::EPL], rb[L::EPL]; int xp; };
    for (int c0 = 0; c0 < n; c0 += TEAM_SPAN) {
        const int cnt = min(TEAM_SPAN, n - c0);
        const int n_stage = (cnt + S - 1) / S;
        TeamDesc dsc;
        dsc.fetch(ent + c0, cnt, lane);
        auto stage_load = [&](StageRegs &R, int st) {
            const int j = st * S + w;
            const int idx = j < cnt ? dsc.idx(j) : 0;
            // first pair of entry st*S + lane/16, fetched from the lane that holds that descriptor
            const int je = min(st * S + (lane >> 4), cnt - 1);
            const int pb = je < WAVE ? __shfl(dsc.lo.z, je) : __shfl(dsc.hi.z, je - WAVE);
            R.xp = P.grp_pairs[min(pb + (lane & 15), last_pair)];
            load_row<T, H, D>(k + (size_t)idx * L::C, lane, R.ra);
            load_row<T, H, D>(v + (size_t)idx * L::C, lane, R.rb);
        };
        auto stage_write = [&](const StageRegs &R, int buf) {
            lds_put_row<L::EPL>(lds[buf][w][0], lane, R.ra);
            lds_put_row<L::EPL>(lds[buf][w][1], lane, R.rb);
        };
        auto stage_compute = [&](int st, int buf, int xp) {
#pragma unroll
            for (int e = 0; e < S; ++e) {
                const int j = st * S + e;
                const int mask16 = j < cnt ? dsc.mask(j) : 0;
                const int mk = (mask16 >> (w * RW)) & ((1 << RW) - 1);
                if (mk == 0) continue;
                float kr[L::EPL], vr[L::EPL];
                lds_get_row<L::EPL>(lds[buf][e][0], lane, kr);
                lds_get_row<L::EPL>(lds[buf][e][1], lane, vr);
#pragma unroll
                for (int m = 0; m < RW; ++m) {
                    if (mk & (1 << m)) {
                        const int rank = __builtin_popcount(mask16 & ((1 << (w * RW + m)) - 1));
                        const unsigned pos = (unsigned)__builtin_amdgcn_readlane(xp, e * TEAM_R + rank);
                        const float sdot = head_sum<L::LPH>(dot_n<L::EPL>(qv[m], kr));
                        const float dp = head_sum<L::LPH>(dot_n<L::EPL>(dov[m], vr));
                        const float pe = __builtin_amdgcn_exp2f(fmaf(sdot, scale_log2e, -lse2[m]));
                        const float ds = pe * (dp - delta[m]) * scale;
#pragma unroll
                        for (int i = 0; i < L::EPL; ++i) dqa[m][i] = fmaf(ds, kr[i], dqa[m][i]);
                        pds[(size_t)pos * H + head] = make_float2(pe, ds);     // all lanes of a head write the same value
                    }
                }
            }
        };
        StageRegs A, B;
        stage_load(A, 0);
        stage_load(B, 1);
        stage_write(A, 0);
        int xp_even = A.xp, xp_odd = B.xp;
        stage_load(A, 2);
        __syncthreads();
        for (int st = 0; st < n_stage; st += 2) {
            stage_compute(st, 0, xp_even);
            issue_loads_first();
            stage_write(B, 1);         // B holds stage st + 1
            xp_odd = B.xp;
            stage_load(B, st + 3);
            __syncthreads();
            stage_compute(st + 1, 1, xp_odd);
            issue_loads_first();
            stage_write(A, 0);         // A holds stage st + 2
            xp_even = A.xp;
            stage_load(A, st + 4);
            __syncthreads();
        }
    }
#pragma unroll
    for (int m = 0; m < RW; ++m) {
        if (rows[m] < 0) continue;
        if (slots[m] < 0) store_row<T, H, D>(dq + (size_t)rows[m] * L::C, lane, dqa[m]);
        else store_row_ws<T, H, D>(ws_dq + (size_t)slots[m] * L::C, lane, dqa[m]);
    }
}

// Backward, source side, teams: dK[src] = sum ds * q[dst], dV[src] = sum p * dO[dst].  The (p, ds) of
// this plan's pairs are contiguous per stage; the workgroup copies them to LDS with one 16-byte
// load per thread.
template <typename T, int H, int D>
__global__ __launch_bounds__(BLOCK) void k_attn_bwd_src_team(bpt_plan P, const T *__restrict__ q, const T *__restrict__ d_o,
                                                             const float2 *__restrict__ pds, T *__restrict__ dk, T *__restrict__ dv,
                                                             float *__restrict__ ws_dk, float *__restrict__ ws_dv) {
    using L = Lay<T, H, D>;
    constexpr int S = TEAM_S, RW = TEAM_RW, F4 = L::EPL / 4;
    constexpr int WF4 = S * TEAM_R * H / 2;                 // float4 per stage of weights (at most S*16 pairs)
    constexpr int WPT = (WF4 + BLOCK - 1) / BLOCK;          // float4 per thread
    __shared__ float4 lds[2][S][2][F4 * WAVE];
    __shared__ float4 wts[2][WPT * BLOCK];
    const int t = team_index(P);
    if (t < 0) return;
    const int tid = threadIdx.x;
    const int lane = tid & 63, w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), head = lane / L::LPH;
    int rows[RW], slots[RW];
#pragma unroll
    for (int m = 0; m < RW; ++m) {
        rows[m] = __builtin_amdgcn_readfirstlane(P.grp_members[((size_t)t * TEAM_R + w * RW + m) * 2]);
        slots[m] = __builtin_amdgcn_readfirstlane(P.grp_members[((size_t)t * TEAM_R + w * RW + m) * 2 + 1]);
    }
    const int begin = __builtin_amdgcn_readfirstlane(P.grp_ptr[t]);
    const int n = __builtin_amdgcn_readfirstlane(P.grp_ptr[t + 1]) - begin;
    const int4 *ent = reinterpret_cast<const int4 *>(P.grp_entries) + begin;
    const float4 *pds4 = reinterpret_cast<const float4 *>(pds);
    const int n_f4 = (int)(P.n_edges * H / 2);              // float4 in the whole scratch

    float ak[RW][L::EPL], av[RW][L::EPL];
#pragma unroll
    for (int m = 0; m < RW; ++m)
#pragma unroll
        for (int i = 0; i < L::EPL; ++i) { ak[m][i] = 0.f; av[m][i] = 0.f; }
    struct StageRegs { float ra[L::EPL], rb[L::EPL]; float4 wreg[WPT]; };
    for (int c0 = 0; c0 < n; c0 += TEAM_SPAN) {
        const int cnt = min(TEAM_SPAN, n - c0);
        const int n_stage = (cnt + S - 1) / S;
        TeamDesc dsc;
        dsc.fetch(ent + c0, cnt, lane);
        auto stage_load = [&](StageRegs &R, int st) {
            const int j = st * S + w;
            const int idx = j < cnt ? dsc.idx(j) : 0;
            const int pb0 = dsc.pair0(min(st * S, cnt - 1));                     // first pair of the stage
#pragma unroll
            for (int u = 0; u < WPT; ++u) R.wreg[u] = pds4[min(pb0 * (H / 2) + u * BLOCK + tid, n_f4 - 1)];
            load_row<T, H, D>(q + (size_t)idx * L::C, lane, R.ra);
            load_row<T, H, D>(d_o + (size_t)idx * L::C, lane, R.rb);
        };
        auto stage_write = [&](const StageRegs &R, int buf) {
            lds_put_row<L::EPL>(lds[buf][w][0], lane, R.ra);
            lds_put_row<L::EPL>(lds[buf][w][1], lane, R.rb);
#pragma unroll
            for (int u = 0; u < WPT; ++u) wts[buf][u * BLOCK + tid] = R.wreg[u];
        };
        auto stage_compute = [&](int st, int buf) {
            if (st >= n_stage) return;
            const float2 *wbuf = reinterpret_cast<const float2 *>(wts[buf]);
            const int pb0 = dsc.pair0(st * S);
#pragma unroll
            for (int e = 0; e < S; ++e) {
                const int j = st * S + e;
                const int mask16 = j < cnt ? dsc.mask(j) : 0;
                const int mk = (mask16 >> (w * RW)) & ((1 << RW) - 1);
                if (mk == 0) continue;
                const int pbe = dsc.pair0(j) - pb0;       // first pair of the entry, relative to the stage
                float qr[L::EPL], dr[L::EPL];
                lds_get_row<L::EPL>(lds[buf][e][0], lane, qr);
                lds_get_row<L::EPL>(lds[buf][e][1], lane, dr);
#pragma unroll
                for (int m = 0; m < RW; ++m) {
                    if (mk & (1 << m)) {
                        const int lp = pbe + __builtin_popcount(mask16 & ((1 << (w * RW + m)) - 1));
                        const float2 wgt = wbuf[lp * H + head];
#pragma unroll
                        for (int i = 0; i < L::EPL; ++i) {
                            ak[m][i] = fmaf(wgt.y, qr[i], ak[m][i]);
                            av[m][i] = fmaf(wgt.x, dr[i], av[m][i]);
                        }
                    }
                }
            }
        };
        StageRegs A, B;
        stage_load(A, 0);
        stage_load(B, 1);
        stage_write(A, 0);
        stage_load(A, 2);
        __syncthreads();
        for (int st = 0; st < n_stage; st += 2) {
            stage_compute(st, 0);
            issue_loads_first();
            stage_write(B, 1);         // B holds stage st + 1
            stage_load(B, st + 3);
            __syncthreads();
            stage_compute(st + 1, 1);
            issue_loads_first();
            stage_write(A, 0);         // A holds stage st + 2
            stage_load(A, st + 4);
            __syncthreads();
        }
    }
#pragma unroll
    for (int m = 0; m < RW; ++m) {
        if (rows[m] < 0) continue;
        if (slots[m] < 0) {
            store_row<T, H, D>(dk + (size_t)rows[m] * L::C, lane, ak[m]);
            store_row<T, H, D>(dv + (size_t)rows[m] * L::C, lane, av[m]);
        } else {
            store_row_ws<T, H, D>(ws_dk + (size_t)slots[m] * L::C, lane, ak[m]);
            store_row_ws<T, H, D>(ws_dv + (size_t)slots[m] * L::C, lane, av[m]);
        }
    }
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
    if (p->n_groups < 0 || p->grp_R < 0 || p->grp_R > 16) return BPT_ERR_SIZE;
    if (p->n_groups > 0 && (!p->grp_members || !p->grp_ptr || !p->grp_chunks || (p->n_edges > 0 && !p->grp_entries))) return BPT_ERR_NULL;
    if (p->n_groups > 0 && (p->grp_max_chunk < 1 || p->grp_max_chunk > p->n_groups)) return BPT_ERR_SIZE;
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
int run_softmax_fwd(const bpt_plan *P, const void *x, void *y, int h, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
    hipLaunchKernelGGL((k_softmax_fwd<T, 1>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)x, (T *)y, h);
    int st = launch_status();
    if (st != BPT_OK || P->n_heavy == 0) return st;
    hipLaunchKernelGGL((k_softmax_fwd<T, WAVES_PER_BLOCK>), dim3((int)P->n_heavy), dim3(BLOCK), 0, s, *P, (const T *)x, (T *)y, h);
    return launch_status();
}

template <typename T>
int run_softmax_bwd(const bpt_plan *P, const void *y, const void *dy, void *dx, int h, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
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
    hipLaunchKernelGGL((k_combine_sum<T>), dim3((int)P->n_heavy, H * D / WAVE, NOUT), dim3(BLOCK), 0, s, P->heavy, (const float *)ws,
                       (T *)Y0, (T *)Y1, H * D, (size_t)P->n_slots * H * D);
    return launch_status();
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
int sddmm(const bpt_plan *P, const void *A, const void *B, void *y, int h, int d, int dtype, hipStream_t s) {
    if (fast_shape(h, d, dtype) && aligned16(A) && aligned16(B)) return sddmm_fast(P, A, B, y, h, d, dtype, s);
    return sddmm_generic(P, A, B, y, h, d, dtype, s);
}
int spmm(const bpt_plan *P, const void *W, const void *X, void *Y, void *ws, int h, int d, int dtype, hipStream_t s) {
    if (fast_shape(h, d, dtype) && aligned16(X) && aligned16(Y) && aligned16(ws)) return spmm_fast(P, W, X, Y, ws, h, d, dtype, s);
    return spmm_generic(P, W, X, Y, ws, h, d, dtype, s);
}

inline int64_t round16(int64_t b) { return (b + 15) & ~(int64_t)15; }

constexpr int GROUP_R = 4;

inline int group_grid(const bpt_plan *P, int kernel) {
    const int64_t per_xcd = g_group_waves[kernel].load(std::memory_order_relaxed);
    const int64_t n = (per_xcd > 0 && per_xcd < P->grp_max_chunk) ? per_xcd : P->grp_max_chunk;
    return (int)(8 * n);
}

inline bool has_teams(const bpt_plan *P) {
    return P->n_groups > 0 && P->grp_R == TEAM_R && P->grp_members && P->grp_ptr && P->grp_entries && P->grp_chunks &&
           P->grp_max_chunk > 0 && 8 * P->grp_max_chunk >= P->n_groups;
}

inline bool has_groups(const bpt_plan *P) {
    return P->n_groups > 0 && P->grp_R == GROUP_R && P->grp_members && P->grp_ptr && P->grp_entries && P->grp_chunks &&
           P->grp_max_chunk > 0 && 8 * P->grp_max_chunk >= P->n_groups;
}

template <typename T, int H, int D>
int run_attn_fwd(const bpt_plan *P, const void *q, const void *k, const void *v, void *o, float *lse, void *ws, float scale, hipStream_t s) {
    if (P->n_items == 0) return BPT_OK;
    float *ws_acc = (float *)ws;
    float *ws_ml = ws_acc ? ws_acc + (size_t)P->n_slots * H * D : nullptr;
    {
        ProfScope prof(BPT_KERNEL_ATTN_FWD, s);
        if (has_teams(P)) {
            hipLaunchKernelGGL((k_attn_fwd_team<T, H, D>), dim3((int)(8 * P->grp_max_chunk)), dim3(BLOCK), 0, s, *P, (const T *)q,
                               (const T *)k, (const T *)v, (T *)o, lse, ws_acc, ws_ml, scale * LOG2E);
        } else if (has_groups(P)) {
#define LAUNCH_FWD_GRP(B, W)                                                                                                   \
    hipLaunchKernelGGL((k_attn_fwd_grp<T, H, D, GROUP_R, B, W>), dim3(group_grid(P, 0)), dim3(WAVE), 0, s, *P, (const T *)q,   \
                       (const T *)k, (const T *)v, (T *)o, lse, ws_acc, ws_ml, scale * LOG2E)
            const int var = g_group_variant[0].load(std::memory_order_relaxed);
            if (var == 4) LAUNCH_FWD_GRP(4, 1);
            else if (var == 3) LAUNCH_FWD_GRP(2, 3);
            else LAUNCH_FWD_GRP(2, 1);
#undef LAUNCH_FWD_GRP
        } else {
            hipLaunchKernelGGL((k_attn_fwd<T, H, D, FAST_BATCH>), dim3(grid_for(P)), dim3(BLOCK), 0, s, *P, (const T *)q, (const T *)k,
                               (const T *)v, (T *)o, lse, ws_acc, ws_ml, scale * LOG2E);
        }
    }
    int st = launch_status();
    if (st != BPT_OK || P->n_heavy == 0) return st;
    hipLaunchKernelGGL((k_attn_fwd_combine<T, H, D>), dim3((int)P->n_heavy, H * D / WAVE), dim3(BLOCK), 0, s, P->heavy,
                       (const float *)ws_acc, (const float *)ws_ml, (T *)o, lse);
    return launch_status();
}

template <typename T, int H, int D>
int run_attn_bwd_grouped(const bpt_plan *Pin, const bpt_plan *Pout, const void *q, const void *k, const void *v, const void *o,
                         const void *d_o, const float *lse, void *dq, void *dk, void *dv, void *ws, float scale, hipStream_t s) {
    const size_t EH = (size_t)Pin->n_edges * H;
    float2 *pds = (float2 *)ws;
    float *ws_rows = (float *)ws + 2 * (round16((int64_t)EH * 4) / 4);
    {
        ProfScope prof(BPT_KERNEL_ATTN_BWD_DST, s);
#define LAUNCH_DST_GRP(B, W)                                                                                                       \
    hipLaunchKernelGGL((k_attn_bwd_dst_grp<T, H, D, GROUP_R, B, W>), dim3(group_grid(Pin, 1)), dim3(WAVE), 0, s, *Pin, (const T *)q, \
                       (const T *)k, (const T *)v, (const T *)o, (const T *)d_o, lse, (T *)dq, pds, ws_rows, scale, scale * LOG2E)
        const int var = g_group_variant[1].load(std::memory_order_relaxed);
        if (var == 4) LAUNCH_DST_GRP(4, 1);
        else if (var == 3) LAUNCH_DST_GRP(2, 3);
        else LAUNCH_DST_GRP(2, 1);
#undef LAUNCH_DST_GRP
    }
    int st = launch_status();
    if (st != BPT_OK) return st;
    if (Pin->n_heavy > 0) {
        hipLaunchKernelGGL((k_combine_sum<T>), dim3((int)Pin->n_heavy, H * D / WAVE, 1), dim3(BLOCK), 0, s, Pin->heavy,
                           (const float *)ws_rows, (T *)dq, (T *)nullptr, H * D, (size_t)0);
        st = launch_status();
        if (st != BPT_OK) return st;
    }
    float *ws_dk = ws_rows, *ws_dv = ws_rows + (size_t)Pout->n_slots * H * D;
    {
        ProfScope prof(BPT_KERNEL_ATTN_BWD_SRC, s);
#define LAUNCH_SRC_GRP(B, W)                                                                                                          \
    hipLaunchKernelGGL((k_attn_bwd_src_grp<T, H, D, GROUP_R, B, W>), dim3(group_grid(Pout, 2)), dim3(WAVE), 0, s, *Pout, (const T *)q, \
                       (const T *)d_o, (const float2 *)pds, (T *)dk, (T *)dv, ws_dk, ws_dv)
        const int var = g_group_variant[2].load(std::memory_order_relaxed);
        if (var == 4) LAUNCH_SRC_GRP(4, 1);
        else if (var == 3) LAUNCH_SRC_GRP(2, 3);
        else LAUNCH_SRC_GRP(2, 1);
#undef LAUNCH_SRC_GRP
    }
    st = launch_status();
    if (st != BPT_OK || Pout->n_heavy == 0) return st;
    hipLaunchKernelGGL((k_combine_sum<T>), dim3((int)Pout->n_heavy, H * D / WAVE, 2), dim3(BLOCK), 0, s, Pout->heavy,
                       (const float *)ws_dk, (T *)dk, (T *)dv, H * D, (size_t)Pout->n_slots * H * D);
    return launch_status();
}

template <typename T, int H, int D>
int run_attn_bwd_team(const bpt_plan *Pin, const bpt_plan *Pout, const void *q, const void *k, const void *v, const void *o,
                      const void *d_o, const float *lse, void *dq, void *dk, void *dv, void *ws, float scale, hipStream_t s) {
    const size_t EH = (size_t)Pin->n_edges * H;
    float2 *pds = (float2 *)ws;
    float *ws_rows = (float *)ws + 2 * (round16((int64_t)EH * 4) / 4);
    {
        ProfScope prof(BPT_KERNEL_ATTN_BWD_DST, s);
        hipLaunchKernelGGL((k_attn_bwd_dst_team<T, H, D>), dim3((int)(8 * Pin->grp_max_chunk)), dim3(BLOCK), 0, s, *Pin, (const T *)q,
                           (const T *)k, (const T *)v, (const T *)o, (const T *)d_o, lse, (T *)dq, pds, ws_rows, scale, scale * LOG2E);
    }
    int st = launch_status();
    if (st != BPT_OK) return st;
    if (Pin->n_heavy > 0) {
        hipLaunchKernelGGL((k_combine_sum<T>), dim3((int)Pin->n_heavy, H * D / WAVE, 1), dim3(BLOCK), 0, s, Pin->heavy,
                           (const float *)ws_rows, (T *)dq, (T *)nullptr, H * D, (size_t)0);
        st = launch_status();
        if (st != BPT_OK) return st;
    }
    float *ws_dk = ws_rows, *ws_dv = ws_rows + (size_t)Pout->n_slots * H * D;
    {
        ProfScope prof(BPT_KERNEL_ATTN_BWD_SRC, s);
        hipLaunchKernelGGL((k_attn_bwd_src_team<T, H, D>), dim3((int)(8 * Pout->grp_max_chunk)), dim3(BLOCK), 0, s, *Pout, (const T *)q,
                           (const T *)d_o, (const float2 *)pds, (T *)dk, (T *)dv, ws_dk, ws_dv);
    }
    st = launch_status();
    if (st != BPT_OK || Pout->n_heavy == 0) return st;
    hipLaunchKernelGGL((k_combine_sum<T>), dim3((int)Pout->n_heavy, H * D / WAVE, 2), dim3(BLOCK), 0, s, Pout->heavy,
                       (const float *)ws_dk, (T *)dk, (T *)dv, H * D, (size_t)Pout->n_slots * H * D);
    return launch_status();
}

template <typename T, int H, int D>
int run_attn_bwd(const bpt_plan *Pin, const bpt_plan *Pout, const void *q, const void *k, const void *v, const void *o,
                 const void *d_o, const float *lse, void *dq, void *dk, void *dv, void *ws, float scale, hipStream_t s) {
    if (Pin->n_items == 0) return BPT_OK;
    if (has_teams(Pin) && has_teams(Pout) && Pin->grp_pairs)
        return run_attn_bwd_team<T, H, D>(Pin, Pout, q, k, v, o, d_o, lse, dq, dk, dv, ws, scale, s);
    if (has_groups(Pin) && has_groups(Pout) && Pin->grp_pairs)
        return run_attn_bwd_grouped<T, H, D>(Pin, Pout, q, k, v, o, d_o, lse, dq, dk, dv, ws, scale, s);
    const size_t EH = (size_t)Pin->n_edges * H;
    float *pbuf = (float *)ws;
    float *dsbuf = pbuf + round16((int64_t)EH * 4) / 4;
    float *ws_rows = dsbuf + round16((int64_t)EH * 4) / 4;
    {
        ProfScope prof(BPT_KERNEL_ATTN_BWD_DST, s);
        hipLaunchKernelGGL((k_attn_bwd_dst<T, H, D, FAST_BATCH>), dim3(grid_for(Pin)), dim3(BLOCK), 0, s, *Pin, (const T *)q,
                           (const T *)k, (const T *)v, (const T *)o, (const T *)d_o, lse, (T *)dq, pbuf, dsbuf, ws_rows, scale,
                           scale * LOG2E);
    }
    int st = launch_status();
    if (st != BPT_OK) return st;
    if (Pin->n_heavy > 0) {
        hipLaunchKernelGGL((k_combine_sum<T>), dim3((int)Pin->n_heavy, H * D / WAVE, 1), dim3(BLOCK), 0, s, Pin->heavy,
                           (const float *)ws_rows, (T *)dq, (T *)nullptr, H * D, (size_t)0);
        st = launch_status();
        if (st != BPT_OK) return st;
    }
    // source side: dK[src] = sum ds * q[dst], dV[src] = sum p * dO[dst]
    return run_spmm_fast<T, float, H, D, 2>(Pout, dsbuf, q, dk, pbuf, d_o, dv, ws_rows, s);
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
        default: return "unknown bptattn status";
    }
}

int bpt_set_force_generic(int on) { return g_force_generic.exchange(on ? 1 : 0); }

int bpt_set_group_variant(int kernel, int variant) {
    if (kernel < 0 || kernel > 2 || (variant != 2 && variant != 3 && variant != 4)) return BPT_ERR_SIZE;
    g_group_variant[kernel].store(variant);
    return BPT_OK;
}

int bpt_set_group_waves(int kernel, int waves_per_xcd) {
    if (kernel < 0 || kernel > 2 || waves_per_xcd < 0) return BPT_ERR_SIZE;
    g_group_waves[kernel].store(waves_per_xcd);
    return BPT_OK;
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
        case BPT_OP_ATTN_BWD: {
            const int64_t rows = s0 > 2 * s1 ? s0 : 2 * s1;
            return 2 * round16(plan->n_edges * h * 4) + round16(rows * C * 4);
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

int bpt_node_mul_edge_forward(const bpt_plan *plan, const void *A, const void *B, void *y, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan, false));
    CHECK(check_shape(h, d, dtype));
    if (plan->n_edges > 0 && (!A || !B || !y)) return BPT_ERR_NULL;
    return sddmm_edge_generic(plan, A, B, y, h, d, dtype, (hipStream_t)stream);
}

int bpt_node_mul_edge_backward(const bpt_plan *plan, const void *A, const void *B, const void *dy, void *dA, void *dB,
                               void *workspace, int64_t workspace_bytes, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan, false));
    CHECK(check_shape(h, d, dtype));
    if (!dA || (plan->n_edges > 0 && (!A || !B || !dy || !dB))) return BPT_ERR_NULL;
    const int64_t need = bpt_workspace_bytes(BPT_OP_NODE_MUL_EDGE_BWD, plan, nullptr, h, d, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    CHECK(spmm_edge_generic(plan, dy, B, dA, workspace, h, d, dtype, (hipStream_t)stream));
    DISPATCH_DTYPE(dtype, (run_nme_dB<T>(plan, A, dy, dB, h, d, (hipStream_t)stream)))
}

int bpt_sparse_softmax_forward(const bpt_plan *plan, const void *x, void *y, int h, int dtype, void *stream) {
    CHECK(check_plan(plan, false));
    CHECK(check_shape(h, 1, dtype));
    if (plan->n_edges > 0 && (!x || !y)) return BPT_ERR_NULL;
    DISPATCH_DTYPE(dtype, (run_softmax_fwd<T>(plan, x, y, h, (hipStream_t)stream)))
}

int bpt_sparse_softmax_backward(const bpt_plan *plan, const void *y, const void *dy, void *dx, int h, int dtype, void *stream) {
    CHECK(check_plan(plan, false));
    CHECK(check_shape(h, 1, dtype));
    if (plan->n_edges > 0 && (!y || !dy || !dx)) return BPT_ERR_NULL;
    DISPATCH_DTYPE(dtype, (run_softmax_bwd<T>(plan, y, dy, dx, h, (hipStream_t)stream)))
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

int bpt_attention_forward(const bpt_plan *plan_in, const void *q, const void *k, const void *v, void *o, float *lse,
                          void *workspace, int64_t workspace_bytes, float scale, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan_in, true));
    CHECK(check_shape(h, d, dtype));
    if (!q || !k || !v || !o || !lse) return BPT_ERR_NULL;
    if (!fast_shape(h, d, dtype) || !aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(workspace))
        return BPT_ERR_UNSUPPORTED;
    const int64_t need = bpt_workspace_bytes(BPT_OP_ATTN_FWD, plan_in, nullptr, h, d, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
#define X(HH, DD) if (h == HH && d == DD) return run_attn_fwd<T, HH, DD>(plan_in, q, k, v, o, lse, workspace, scale, s);
    if (dtype == BPT_F32) { using T = float; BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { using T = bf16_t; BPT_FAST_SHAPES_BF16(X) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

int bpt_attention_backward(const bpt_plan *plan_in, const bpt_plan *plan_out, const void *q, const void *k, const void *v,
                           const void *o, const void *d_o, const float *lse, void *dq, void *dk, void *dv, void *workspace,
                           int64_t workspace_bytes, float scale, int h, int d, int dtype, void *stream) {
    CHECK(check_plan(plan_in, true));
    CHECK(check_plan(plan_out, true));
    CHECK(check_shape(h, d, dtype));
    if (plan_in->n_edges != plan_out->n_edges || plan_in->n_rows != plan_out->n_rows) return BPT_ERR_PLAN;
    if (!q || !k || !v || !o || !d_o || !lse || !dq || !dk || !dv) return BPT_ERR_NULL;
    if (!fast_shape(h, d, dtype) || !aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(d_o) ||
        !aligned16(dq) || !aligned16(dk) || !aligned16(dv) || !aligned16(workspace))
        return BPT_ERR_UNSUPPORTED;
    const int64_t need = bpt_workspace_bytes(BPT_OP_ATTN_BWD, plan_in, plan_out, h, d, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return BPT_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
#define X(HH, DD) \
    if (h == HH && d == DD) return run_attn_bwd<T, HH, DD>(plan_in, plan_out, q, k, v, o, d_o, lse, dq, dk, dv, workspace, scale, s);
    if (dtype == BPT_F32) { using T = float; BPT_FAST_SHAPES_F32(X) }
    if (dtype == BPT_BF16) { using T = bf16_t; BPT_FAST_SHAPES_BF16(X) }
#undef X
    return BPT_ERR_UNSUPPORTED;
}

}  // extern "C"
