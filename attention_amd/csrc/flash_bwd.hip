// FlashAttention backward entry points: argument checks, kernel choice, launches.
//
// The interface hands over Q, K, V and dO only (no forward output, no softmax statistics), so a backward
// is three launches:
//   1. statistics  per query row i: lse_i = log sum_j exp(scale q_i.k_j) and delta_i = dO_i . O_i
//                  (a forward pass that keeps its output in registers),
//   2. dQ          a workgroup owns query rows and walks the keys:  dS_ij = P_ij (dO_i.v_j - delta_i),
//                  dQ_i = scale * sum_j dS_ij k_j,
//   3. dK, dV      a workgroup owns key rows and walks the queries: dV_j = sum_i P_ij dO_i,
//                  dK_j = scale * sum_i dS_ij q_i  (summed over the query heads of a K/V head);
//                  on the matrix cores, dK and dV in one walk over the query tiles up to d = 128 (launch_dkv).
// with P_ij = exp(scale q_i.k_j - lse_i).  Nothing is accumulated through atomics, so results do not depend
// on launch order.  The statistics live in the caller's workspace: two floats per (sequence, head, row).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdlib>

#include "ahpc_device.hpp"
#include "flash_bwd_mfma.hpp"
#include "mask_pack.hpp"
#include "flash_bwd_f32_mfma.hpp"
#include "tuning.hpp"

namespace ahpc {

struct BwdParams {
    const void* q;
    const void* k;
    const void* v;
    const void* d_out;
    void* d_q;
    void* d_k;
    void* d_v;
    const float* mask;          // [B,N,N] or null
    const int32_t* cu_seqlens;  // ragged batches: sequence b owns token rows cu_seqlens[b] .. cu_seqlens[b+1]-1
    float* lse;                 // [B*H][rows_padded]
    float* delta;               // [B*H][rows_padded]
    int64_t rows_padded;
    int64_t stride_b, stride_n, stride_h;           // Q, dO, dQ
    int64_t kv_stride_b, kv_stride_n, kv_stride_h;  // K, V, dK, dV
    int32_t N, H, d;
    int32_t kv_group;           // query heads per key/value head
    float scale;
    int32_t causal;
};

// ---------------------------------------------------------------------------------------------
// fp32-FMA kernels: any dtype, head dimension up to 256, optional dense mask.  A row (query row in the first
// two kernels, key row in the third) is owned by S neighbouring lanes that keep it in registers, 16-byte
// granules dealt round-robin (S = 1, 2, 4 for padded head dimensions up to 64, 128, 256: at most 64 elements
// of each per-row vector per lane, which is what fits the register file); the rows they walk over are staged in
// LDS as fp32, 16 at a time, by the 128 threads of the workgroup, and dot products are summed across the S
// lanes with shuffles.  Everything between two barriers is straight-line per key with the row's conditions as
// predicates, so that the shuffles run with all lanes.  This is the accuracy path (fp32 tensors, 1e-4
// tolerance) and the fallback for what the matrix-core kernels do not take.
constexpr int kBwdThreads = 128;
constexpr int kBwdTile = 16;

// Stages rows [r0, r0+16) of a [rows][d] tensor (row stride `stride`) into dst[16][DP] as fp32; rows at or
// beyond `n_rows` and columns at or beyond d become zero.
template <typename T, int DP>
__device__ inline void stage_rows(float (*dst)[DP], const T* src, int64_t stride, int r0, int n_rows, int d, int tid) {
    for (int i = tid; i < kBwdTile * DP; i += kBwdThreads) {
        const int r = i / DP, e = i - r * DP;
        const int row = r0 + r;
        dst[r][e] = (row < n_rows && e < d) ? Storage<T>::load(src + (int64_t)row * stride + e) : 0.0f;
    }
}

// Element of the row that register i of lane part `part` holds (S lanes per row, 16-byte granules round-robin).
template <int S>
__device__ inline int row_elem(int i, int part) { return (((i >> 2) * S + part) << 2) + (i & 3); }

// Sum over the S neighbouring lanes of a row; every lane of the wavefront takes part.
template <int S>
__device__ inline float row_sum(float x) {
    if (S >= 2) x += __shfl_xor(x, 1, kWave);
    if (S >= 4) x += __shfl_xor(x, 2, kWave);
    return x;
}

// Length of sequence b and the element offsets of its first row for head h (Q, dO, dQ) and K/V head hk.
__device__ __forceinline__ void bwd_sequence(const BwdParams& p, int b, int h, int hk, int& L, int64_t& base, int64_t& kv_base) {
    if (p.cu_seqlens) {
        const int s0 = p.cu_seqlens[b];
        L = p.cu_seqlens[b + 1] - s0;
        base = (int64_t)s0 * p.stride_n + (int64_t)h * p.stride_h;
        kv_base = (int64_t)s0 * p.kv_stride_n + (int64_t)hk * p.kv_stride_h;
    } else {
        L = p.N;
        base = (int64_t)b * p.stride_b + (int64_t)h * p.stride_h;
        kv_base = (int64_t)b * p.kv_stride_b + (int64_t)hk * p.kv_stride_h;
    }
}

template <typename T, int DP, int S>
__global__ __launch_bounds__(kBwdThreads) void flash_bwd_stats_simple_kernel(const BwdParams p) {
    constexpr int EP = DP / S;            // elements of a row per lane
    constexpr int R = kBwdThreads / S;    // rows per workgroup
    __shared__ float sk[kBwdTile][DP];
    __shared__ float sv[kBwdTile][DP];
    const int tid = threadIdx.x;
    const int part = tid % S;
    const int h = blockIdx.y, b = blockIdx.z;
    const int hk = h / p.kv_group;
    const int d = p.d;
    int L;
    int64_t base, kv_base;
    bwd_sequence(p, b, h, hk, L, base, kv_base);
    const int row0 = blockIdx.x * R;
    if (row0 >= L) return;
    const int n = row0 + tid / S;
    const bool active = n < L;
    const T* gq = static_cast<const T*>(p.q) + base;
    const T* gdo = static_cast<const T*>(p.d_out) + base;
    const T* gk = static_cast<const T*>(p.k) + kv_base;
    const T* gv = static_cast<const T*>(p.v) + kv_base;

    float qv[EP], acc[EP];
#pragma unroll
    for (int i = 0; i < EP; ++i) {
        const int e = row_elem<S>(i, part);
        qv[i] = (active && e < d) ? Storage<T>::load(gq + (int64_t)n * p.stride_n + e) : 0.0f;
        acc[i] = 0.0f;
    }
    float m = -INFINITY, l = 0.0f;
    int k_end = L;
    if (p.causal) k_end = (row0 + R) < L ? (row0 + R) : L;
    const float* mrow = (p.mask && active) ? p.mask + ((int64_t)b * p.N + n) * p.N : nullptr;

    for (int k0 = 0; k0 < k_end; k0 += kBwdTile) {
        __syncthreads();
        stage_rows<T, DP>(sk, gk, p.kv_stride_n, k0, L, d, tid);
        stage_rows<T, DP>(sv, gv, p.kv_stride_n, k0, L, d, tid);
        __syncthreads();
        const int kr_end = (k_end - k0) < kBwdTile ? (k_end - k0) : kBwdTile;
        for (int kr = 0; kr < kr_end; ++kr) {
            const int key = k0 + kr;
            float dot = 0.0f;
#pragma unroll
            for (int i = 0; i < EP; ++i) dot = __builtin_fmaf(qv[i], sk[kr][row_elem<S>(i, part)], dot);
            const float s = row_sum<S>(dot) * p.scale;
            const bool seen = active && !(p.causal && key > n) && !(mrow && mrow[key] == 0.0f);
            if (!seen) continue;
            if (s > m) {
                const float a = __expf(m - s);  // first key: exp(-inf) = 0
                l = l * a + 1.0f;
#pragma unroll
                for (int i = 0; i < EP; ++i) acc[i] = __builtin_fmaf(acc[i], a, sv[kr][row_elem<S>(i, part)]);
                m = s;
            } else {
                const float w = __expf(s - m);
                l += w;
#pragma unroll
                for (int i = 0; i < EP; ++i) acc[i] = __builtin_fmaf(w, sv[kr][row_elem<S>(i, part)], acc[i]);
            }
        }
    }
    // delta = dO . O, summed over the lanes of the row (rows beyond the sequence take part with zeros)
    float dot = 0.0f;
#pragma unroll
    for (int i = 0; i < EP; ++i) {
        const int e = row_elem<S>(i, part);
        if (active && e < d) dot = __builtin_fmaf(acc[i], Storage<T>::load(gdo + (int64_t)n * p.stride_n + e), dot);
    }
    dot = row_sum<S>(dot);
    if (!active || part != 0) return;
    // a row that sees no key: every weight is exp(s - inf) = 0 later on, and nothing flows through it
    const int64_t row = ((int64_t)b * p.H + h) * p.rows_padded + n;
    p.lse[row] = l > 0.0f ? m + logf(l) : INFINITY;
    p.delta[row] = l > 0.0f ? dot / l : 0.0f;
}

template <typename T, int DP, int S>
__global__ __launch_bounds__(kBwdThreads) void flash_bwd_dq_simple_kernel(const BwdParams p) {
    constexpr int EP = DP / S;
    constexpr int R = kBwdThreads / S;
    __shared__ float sk[kBwdTile][DP];
    __shared__ float sv[kBwdTile][DP];
    const int tid = threadIdx.x;
    const int part = tid % S;
    const int h = blockIdx.y, b = blockIdx.z;
    const int hk = h / p.kv_group;
    const int d = p.d;
    int L;
    int64_t base, kv_base;
    bwd_sequence(p, b, h, hk, L, base, kv_base);
    const int row0 = blockIdx.x * R;
    if (row0 >= L) return;
    const int n = row0 + tid / S;
    const bool active = n < L;
    const T* gq = static_cast<const T*>(p.q) + base;
    const T* gdo = static_cast<const T*>(p.d_out) + base;
    const T* gk = static_cast<const T*>(p.k) + kv_base;
    const T* gv = static_cast<const T*>(p.v) + kv_base;

    float qv[EP], dov[EP], dq[EP];
#pragma unroll
    for (int i = 0; i < EP; ++i) {
        const int e = row_elem<S>(i, part);
        const bool in = active && e < d;
        qv[i] = in ? Storage<T>::load(gq + (int64_t)n * p.stride_n + e) : 0.0f;
        dov[i] = in ? Storage<T>::load(gdo + (int64_t)n * p.stride_n + e) : 0.0f;
        dq[i] = 0.0f;
    }
    const int64_t row = ((int64_t)b * p.H + h) * p.rows_padded + (active ? n : 0);
    const float lse = p.lse[row], delta = p.delta[row];
    int k_end = L;
    if (p.causal) k_end = (row0 + R) < L ? (row0 + R) : L;
    const float* mrow = (p.mask && active) ? p.mask + ((int64_t)b * p.N + n) * p.N : nullptr;

    for (int k0 = 0; k0 < k_end; k0 += kBwdTile) {
        __syncthreads();
        stage_rows<T, DP>(sk, gk, p.kv_stride_n, k0, L, d, tid);
        stage_rows<T, DP>(sv, gv, p.kv_stride_n, k0, L, d, tid);
        __syncthreads();
        const int kr_end = (k_end - k0) < kBwdTile ? (k_end - k0) : kBwdTile;
        for (int kr = 0; kr < kr_end; ++kr) {
            const int key = k0 + kr;
            float dot = 0.0f, dp = 0.0f;
#pragma unroll
            for (int i = 0; i < EP; ++i) {
                const int e = row_elem<S>(i, part);
                dot = __builtin_fmaf(qv[i], sk[kr][e], dot);
                dp = __builtin_fmaf(dov[i], sv[kr][e], dp);
            }
            dot = row_sum<S>(dot);
            dp = row_sum<S>(dp);
            const bool seen = active && !(p.causal && key > n) && !(mrow && mrow[key] == 0.0f);
            if (!seen) continue;
            const float ds = __expf(dot * p.scale - lse) * (dp - delta);
#pragma unroll
            for (int i = 0; i < EP; ++i) dq[i] = __builtin_fmaf(ds, sk[kr][row_elem<S>(i, part)], dq[i]);
        }
    }
    if (!active) return;
    T* out = static_cast<T*>(p.d_q) + base + (int64_t)n * p.stride_n;
#pragma unroll
    for (int i = 0; i < EP; ++i) {
        const int e = row_elem<S>(i, part);
        if (e < d) Storage<T>::store(out + e, dq[i] * p.scale);
    }
}

// grid.y = key/value heads: the query heads of a group are walked one after the other
template <typename T, int DP, int S>
__global__ __launch_bounds__(kBwdThreads) void flash_bwd_dkv_simple_kernel(const BwdParams p) {
    constexpr int EP = DP / S;
    constexpr int R = kBwdThreads / S;
    __shared__ float sq[kBwdTile][DP];
    __shared__ float sdo[kBwdTile][DP];
    __shared__ float s_lse[kBwdTile];
    __shared__ float s_delta[kBwdTile];
    const int tid = threadIdx.x;
    const int part = tid % S;
    const int hk = blockIdx.y, b = blockIdx.z;
    const int d = p.d;
    int L;
    int64_t base0, kv_base;
    bwd_sequence(p, b, hk * p.kv_group, hk, L, base0, kv_base);
    const int row0 = blockIdx.x * R;
    if (row0 >= L) return;
    const int j = row0 + tid / S;
    const bool active = j < L;
    const T* gk = static_cast<const T*>(p.k) + kv_base;
    const T* gv = static_cast<const T*>(p.v) + kv_base;

    float kv[EP], vv[EP], dk[EP], dv[EP];
#pragma unroll
    for (int i = 0; i < EP; ++i) {
        const int e = row_elem<S>(i, part);
        const bool in = active && e < d;
        kv[i] = in ? Storage<T>::load(gk + (int64_t)j * p.kv_stride_n + e) : 0.0f;
        vv[i] = in ? Storage<T>::load(gv + (int64_t)j * p.kv_stride_n + e) : 0.0f;
        dk[i] = 0.0f;
        dv[i] = 0.0f;
    }
    // under a causal mask only queries at or after the first key of this workgroup contribute
    const int i_begin = p.causal ? (row0 / kBwdTile) * kBwdTile : 0;

    for (int g = 0; g < p.kv_group; ++g) {
        const int h = hk * p.kv_group + g;
        const int64_t base = base0 + (int64_t)g * p.stride_h;
        const T* gq = static_cast<const T*>(p.q) + base;
        const T* gdo = static_cast<const T*>(p.d_out) + base;
        const int64_t stat0 = ((int64_t)b * p.H + h) * p.rows_padded;
        for (int i0 = i_begin; i0 < L; i0 += kBwdTile) {
            __syncthreads();
            stage_rows<T, DP>(sq, gq, p.stride_n, i0, L, d, tid);
            stage_rows<T, DP>(sdo, gdo, p.stride_n, i0, L, d, tid);
            if (tid < kBwdTile) {
                const int i = i0 + tid;
                s_lse[tid] = i < L ? p.lse[stat0 + i] : INFINITY;
                s_delta[tid] = i < L ? p.delta[stat0 + i] : 0.0f;
            }
            __syncthreads();
            const int r_end = (L - i0) < kBwdTile ? (L - i0) : kBwdTile;
            for (int r = 0; r < r_end; ++r) {
                const int i = i0 + r;
                float dot = 0.0f, dp = 0.0f;
#pragma unroll
                for (int x = 0; x < EP; ++x) {
                    const int e = row_elem<S>(x, part);
                    dot = __builtin_fmaf(sq[r][e], kv[x], dot);
                    dp = __builtin_fmaf(sdo[r][e], vv[x], dp);
                }
                dot = row_sum<S>(dot);
                dp = row_sum<S>(dp);
                const bool seen = active && !(p.causal && i < j) && !(p.mask && p.mask[((int64_t)b * p.N + i) * p.N + j] == 0.0f);
                if (!seen) continue;
                const float pw = __expf(dot * p.scale - s_lse[r]);
                const float ds = pw * (dp - s_delta[r]);
#pragma unroll
                for (int x = 0; x < EP; ++x) {
                    const int e = row_elem<S>(x, part);
                    dv[x] = __builtin_fmaf(pw, sdo[r][e], dv[x]);
                    dk[x] = __builtin_fmaf(ds, sq[r][e], dk[x]);
                }
            }
        }
    }
    if (!active) return;
    T* out_k = static_cast<T*>(p.d_k) + kv_base + (int64_t)j * p.kv_stride_n;
    T* out_v = static_cast<T*>(p.d_v) + kv_base + (int64_t)j * p.kv_stride_n;
#pragma unroll
    for (int x = 0; x < EP; ++x) {
        const int e = row_elem<S>(x, part);
        if (e < d) {
            Storage<T>::store(out_k + e, dk[x] * p.scale);
            Storage<T>::store(out_v + e, dv[x]);
        }
    }
}

template <typename T, int DP>
static int launch_simple_dp(const BwdParams& p, int64_t B, int64_t H_kv, hipStream_t stream) {
    constexpr int S = DP <= 64 ? 1 : DP / 64;  // lanes per row
    constexpr int R = kBwdThreads / S;
    const unsigned tiles = (unsigned)((p.N + R - 1) / R);
    dim3 block(kBwdThreads);
    hipLaunchKernelGGL((flash_bwd_stats_simple_kernel<T, DP, S>), dim3(tiles, (unsigned)p.H, (unsigned)B), block, 0, stream, p);
    hipLaunchKernelGGL((flash_bwd_dq_simple_kernel<T, DP, S>), dim3(tiles, (unsigned)p.H, (unsigned)B), block, 0, stream, p);
    hipLaunchKernelGGL((flash_bwd_dkv_simple_kernel<T, DP, S>), dim3(tiles, (unsigned)H_kv, (unsigned)B), block, 0, stream, p);
    return static_cast<int>(hipGetLastError());
}

template <typename T>
static int launch_simple(const BwdParams& p, int64_t B, int64_t H_kv, hipStream_t stream) {
    if (p.d <= 32) return launch_simple_dp<T, 32>(p, B, H_kv, stream);
    if (p.d <= 64) return launch_simple_dp<T, 64>(p, B, H_kv, stream);
    if (p.d <= 128) return launch_simple_dp<T, 128>(p, B, H_kv, stream);
    if (p.d <= 256) return launch_simple_dp<T, 256>(p, B, H_kv, stream);
    return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
}

// ---------------------------------------------------------------------------------------------
static bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

static int64_t padded_rows(int64_t N) { return (N + kFlashRows - 1) / kFlashRows * kFlashRows; }

// Backward after a forward that kept its row statistics (FlashParams::keep_neg_lse2) and whose output is still there:
// the statistics pass shrinks to -delta = -dO.O per query row, read from the output tensor.  One row per LPR lanes,
// 8 elements per lane; writes both arrays the dQ and dK/dV kernels read, padding rows included (-inf, 0).
constexpr int kDeltaThreads = 256;
template <typename T, int LPR>
__global__ __launch_bounds__(kDeltaThreads) void flash_bwd_delta_kernel(const T* __restrict__ d_out, const T* __restrict__ o,
                                                                         const float* __restrict__ kept, float* __restrict__ neg_lse2,
                                                                         float* __restrict__ neg_delta, int64_t stride_b,
                                                                         int64_t stride_n, int64_t stride_h, int N, int H, int d,
                                                                         int64_t rows_padded, int64_t total_rows) {
    const int64_t r = (int64_t)blockIdx.x * (kDeltaThreads / LPR) + threadIdx.x / LPR;  // (sequence * H + head) * rows_padded + row
    const int piece = threadIdx.x % LPR;
    float part = 0.0f;
    bool live = false;
    if (r < total_rows) {
        const int64_t bh = r / rows_padded;
        const int row = (int)(r - bh * rows_padded);
        live = row < N;
        if (live && 8 * piece < d) {
            const int64_t b = bh / H, h = bh - b * H;
            const int64_t off = b * stride_b + (int64_t)row * stride_n + h * stride_h + 8 * piece;
            const u32x4 a = *reinterpret_cast<const u32x4*>(d_out + off);
            const u32x4 c = *reinterpret_cast<const u32x4*>(o + off);
#pragma unroll
            for (int w = 0; w < 4; ++w) part += lo_f32<T>(a[w]) * lo_f32<T>(c[w]) + hi_f32<T>(a[w]) * hi_f32<T>(c[w]);
        }
    }
    // (every lane of the wavefront takes part in the exchange, rows beyond the end with zeros)
#pragma unroll
    for (int step = LPR / 2; step >= 1; step >>= 1) part += __shfl_xor(part, step, kWave);
    if (piece == 0 && r < total_rows) {
        neg_lse2[r] = live ? kept[r] : -INFINITY;
        neg_delta[r] = live ? -part : 0.0f;
    }
}

// dK and dV: in one walk over the query tiles (four matrix products per tile) up to d = 128, in two walks (dV, then dK:
// five products) at d = 256, where one walk would need more registers than a wavefront has.  At d = 128 the one walk
// runs at one wavefront per SIMD (324 registers) and takes 5 % more cycles than the two walks at two per SIMD; on
// N(0,1) inputs, where the board sits at its power limit and the clock follows the energy spent, it is the faster of
// the two by 4-15 % at every shape timed (fewer products), and it is one launch less.  The tuning value bwd_split
// (0 = this choice, 1 = one walk, 2 = two) overrides.
template <typename T, int D, bool CAUSAL, bool VARLEN, bool MASKED>
static void launch_dkv(const FlashBwdParams& m, dim3 grid, dim3 block, hipStream_t stream) {
    const int64_t choice = tuning().bwd_split.load();
    const bool split = D == 256 || choice == 2;
    if (split) {
        hipLaunchKernelGGL((flash_bwd_dkv_mfma_kernel<T, D, CAUSAL, VARLEN, 1, MASKED>), grid, block, 0, stream, m);
        hipLaunchKernelGGL((flash_bwd_dkv_mfma_kernel<T, D, CAUSAL, VARLEN, 2, MASKED>), grid, block, 0, stream, m);
    } else if constexpr (D != 256) {
        hipLaunchKernelGGL((flash_bwd_dkv_mfma_kernel<T, D, CAUSAL, VARLEN, 0, MASKED>), grid, block, 0, stream, m);
    }
}

// Statistics, dQ, dK and dV.  pm: the packed copy of a dense mask (dense launches only), or null.
template <typename T, int D, bool VARLEN>
static int launch_mfma_dv(const FlashBwdParams& p, const PackedMask* pm, const void* o_kept, const float* stats_kept, int64_t B,
                          int64_t H_kv, bool causal, float* lse2, float* delta, hipStream_t stream) {
    // 1. statistics: the forward kernel with its output kept in registers
    FlashParams f{};
    f.q = p.q; f.k = p.k; f.v = p.v; f.o = nullptr;
    f.stride_b = p.stride_b; f.stride_n = p.stride_n; f.stride_h = p.stride_h;
    f.kv_stride_b = p.kv_stride_b; f.kv_stride_n = p.kv_stride_n; f.kv_stride_h = p.kv_stride_h;
    f.N = p.N; f.H = p.H; f.kv_group = p.kv_group;
    f.cu_seqlens = p.cu_seqlens;
    f.scale_log2 = p.scale_log2;
    f.d_real = p.d_real;
    FlashBwdParams m = p;
    if (pm) {
        f.mask_bits = pm->bits;
        f.mask_kt = pm->tiles;
        m.mask_bits = pm->bits;
        m.mask_bits_t = pm->bits_t;
        m.mask_tiles = pm->tiles;
    }
    if (int rc = flash_plan_launch(f, B, causal, kFlashRows, tuning().flash_pair_min_tiles.load(), VARLEN)) return rc;
    const FlashStatsOut st{p.d_out, lse2, delta, p.rows_padded};
    const dim3 block(kFlashThreads);
    const dim3 grid_stats((unsigned)(f.blocks_per_xcd * 8));
    m.n_tiles = (p.N + kFlashRows - 1) / kFlashRows;
    // causal dense launches: a workgroup takes a long and a short tile of its head, so that all do the same work
    m.paired = (causal && !VARLEN && m.n_tiles >= 2 && tuning().bwd_pair.load() != 0) ? 1 : 0;
    const int64_t units = bwd_units(m);
    const int64_t total_q = B * p.H * units, total_kv = B * H_kv * units;
    if (total_q > 0x7FFFFFF0ll) return AHPC_ERR_BAD_SHAPE;
    m.total_q = (int32_t)total_q; m.per_xcd_q = (int32_t)((total_q + 7) / 8);
    m.total_kv = (int32_t)total_kv; m.per_xcd_kv = (int32_t)((total_kv + 7) / 8);
    const dim3 grid_q((unsigned)(m.per_xcd_q * 8)), grid_kv((unsigned)(m.per_xcd_kv * 8));
    auto launch = [&](auto causal_c, auto masked_c) {
        constexpr bool C = decltype(causal_c)::value, M = decltype(masked_c)::value;
        if constexpr (M && VARLEN) {
            return;  // (a mask belongs to dense launches: never asked for)
        } else {
            if (o_kept && stats_kept && !VARLEN) {
                // the forward kept its row statistics and its output is at hand: no statistics pass
                constexpr int LPR = D / 8;
                const int64_t total_rows = B * p.H * p.rows_padded;
                const int64_t blocks = (total_rows + kDeltaThreads / LPR - 1) / (kDeltaThreads / LPR);
                hipLaunchKernelGGL((flash_bwd_delta_kernel<T, LPR>), dim3((unsigned)blocks), dim3(kDeltaThreads), 0, stream,
                                   static_cast<const T*>(p.d_out), static_cast<const T*>(o_kept), stats_kept, lse2, delta,
                                   p.stride_b, p.stride_n, p.stride_h, (int)p.N, (int)p.H, (int)p.d_real, p.rows_padded, total_rows);
            } else if constexpr (M) {
                hipLaunchKernelGGL((flash_bwd_stats_masked_mfma_kernel<T, D, C>), grid_stats, block, 0, stream, f, st);
            } else {
                hipLaunchKernelGGL((flash_bwd_stats_mfma_kernel<T, D, C, VARLEN>), grid_stats, block, 0, stream, f, st);
            }
            hipLaunchKernelGGL((flash_bwd_dq_mfma_kernel<T, D, C, VARLEN, M>), grid_q, block, 0, stream, m);
            launch_dkv<T, D, C, VARLEN, M>(m, grid_kv, block, stream);
        }
    };
    if (pm && VARLEN) return AHPC_ERR_BAD_SHAPE;
    if (causal) {
        if (pm) launch(std::true_type{}, std::true_type{});
        else launch(std::true_type{}, std::false_type{});
    } else {
        if (pm) launch(std::false_type{}, std::true_type{});
        else launch(std::false_type{}, std::false_type{});
    }
    return static_cast<int>(hipGetLastError());
}

template <typename T>
static int launch_mfma(const FlashBwdParams& p, const PackedMask* pm, const void* o_kept, const float* stats_kept, int64_t B,
                       int64_t H_kv, int d, bool causal, float* lse2, float* delta, hipStream_t stream) {
    if (p.cu_seqlens) {
        if (pm) return AHPC_ERR_BAD_SHAPE;
        if (d == 128) return launch_mfma_dv<T, 128, true>(p, nullptr, nullptr, nullptr, B, H_kv, causal, lse2, delta, stream);
        if (d == 64) return launch_mfma_dv<T, 64, true>(p, nullptr, nullptr, nullptr, B, H_kv, causal, lse2, delta, stream);
        if (d == 256) return launch_mfma_dv<T, 256, true>(p, nullptr, nullptr, nullptr, B, H_kv, causal, lse2, delta, stream);
    } else {
        if (d == 128) return launch_mfma_dv<T, 128, false>(p, pm, o_kept, stats_kept, B, H_kv, causal, lse2, delta, stream);
        if (d == 64) return launch_mfma_dv<T, 64, false>(p, pm, o_kept, stats_kept, B, H_kv, causal, lse2, delta, stream);
        if (d == 256) return launch_mfma_dv<T, 256, false>(p, pm, o_kept, stats_kept, B, H_kv, causal, lse2, delta, stream);
    }
    return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
}

// fp32 tensors: the same three steps on the fp32 matrix instructions (flash_bwd_f32_mfma.hpp), dK and dV always in two walks
template <int D, bool VARLEN>
static int launch_f32_mfma_dv(const FlashBwdParams& p, int64_t B, int64_t H_kv, bool causal, float* lse2, float* delta,
                              hipStream_t stream) {
    FlashParams f{};
    f.q = p.q; f.k = p.k; f.v = p.v; f.o = nullptr;
    f.stride_b = p.stride_b; f.stride_n = p.stride_n; f.stride_h = p.stride_h;
    f.kv_stride_b = p.kv_stride_b; f.kv_stride_n = p.kv_stride_n; f.kv_stride_h = p.kv_stride_h;
    f.N = p.N; f.H = p.H; f.kv_group = p.kv_group;
    f.cu_seqlens = p.cu_seqlens;
    f.scale_log2 = p.scale_log2;
    f.d_real = p.d_real;
    if (int rc = flash_plan_launch(f, B, causal, kFlashRows, tuning().flash_pair_min_tiles.load(), VARLEN)) return rc;
    const FlashStatsOut st{p.d_out, lse2, delta, p.rows_padded};
    const dim3 block(kFlashThreads);
    const dim3 grid_stats((unsigned)(f.blocks_per_xcd * 8));
    FlashBwdParams m = p;
    m.n_tiles = (p.N + kFlashRows - 1) / kFlashRows;
    // causal dense launches: a workgroup takes a long and a short tile of its head, so that all do the same work
    m.paired = (causal && !VARLEN && m.n_tiles >= 2 && tuning().bwd_pair.load() != 0) ? 1 : 0;
    const int64_t units = bwd_units(m);
    const int64_t total_q = B * p.H * units, total_kv = B * H_kv * units;
    if (total_q > 0x7FFFFFF0ll) return AHPC_ERR_BAD_SHAPE;
    m.total_q = (int32_t)total_q; m.per_xcd_q = (int32_t)((total_q + 7) / 8);
    m.total_kv = (int32_t)total_kv; m.per_xcd_kv = (int32_t)((total_kv + 7) / 8);
    const dim3 grid_q((unsigned)(m.per_xcd_q * 8)), grid_kv((unsigned)(m.per_xcd_kv * 8));
    if (causal) {
        hipLaunchKernelGGL((flash_bwd_stats_f32_mfma_kernel<D, true, VARLEN>), grid_stats, block, 0, stream, f, st);
        hipLaunchKernelGGL((flash_bwd_dq_f32_mfma_kernel<D, true, VARLEN>), grid_q, block, 0, stream, m);
        hipLaunchKernelGGL((flash_bwd_dkv_f32_mfma_kernel<D, true, VARLEN, 1>), grid_kv, block, 0, stream, m);
        hipLaunchKernelGGL((flash_bwd_dkv_f32_mfma_kernel<D, true, VARLEN, 2>), grid_kv, block, 0, stream, m);
    } else {
        hipLaunchKernelGGL((flash_bwd_stats_f32_mfma_kernel<D, false, VARLEN>), grid_stats, block, 0, stream, f, st);
        hipLaunchKernelGGL((flash_bwd_dq_f32_mfma_kernel<D, false, VARLEN>), grid_q, block, 0, stream, m);
        hipLaunchKernelGGL((flash_bwd_dkv_f32_mfma_kernel<D, false, VARLEN, 1>), grid_kv, block, 0, stream, m);
        hipLaunchKernelGGL((flash_bwd_dkv_f32_mfma_kernel<D, false, VARLEN, 2>), grid_kv, block, 0, stream, m);
    }
    return static_cast<int>(hipGetLastError());
}

static int launch_f32_mfma(const FlashBwdParams& p, int64_t B, int64_t H_kv, int d, bool causal, float* lse2, float* delta,
                           hipStream_t stream) {
    if (p.cu_seqlens) {
        if (d == 128) return launch_f32_mfma_dv<128, true>(p, B, H_kv, causal, lse2, delta, stream);
        if (d == 64) return launch_f32_mfma_dv<64, true>(p, B, H_kv, causal, lse2, delta, stream);
    } else {
        if (d == 128) return launch_f32_mfma_dv<128, false>(p, B, H_kv, causal, lse2, delta, stream);
        if (d == 64) return launch_f32_mfma_dv<64, false>(p, B, H_kv, causal, lse2, delta, stream);
    }
    return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
}

}  // namespace ahpc

using namespace ahpc;

extern "C" {

size_t ahpc_hip_flash_bwd_workspace_bytes(int64_t B, int64_t N, int64_t H) {
    if (B <= 0 || N <= 0 || H <= 0) return 0;
    // two floats per (sequence, head, row), rows padded to whole query tiles of the matrix-core kernels
    return (size_t)B * (size_t)H * (size_t)padded_rows(N) * 2 * sizeof(float);
}

// B sequences of N tokens (dense), or - cu_seqlens given - B sequences packed one after the other, the longest N tokens.
static int flash_bwd_any(const void* d_out, const void* q, const void* k, const void* v, void* d_q, void* d_k, void* d_v,
                         int dtype, const int32_t* cu_seqlens, int64_t B, int64_t N, int64_t H, int64_t H_kv, int64_t d,
                         int64_t stride_b, int64_t stride_n, int64_t stride_h, int64_t kv_stride_b, int64_t kv_stride_n,
                         int64_t kv_stride_h, float scale, int causal, const float* mask, void* workspace,
                         size_t workspace_bytes, void* stream, const void* o_kept = nullptr, const float* stats_kept = nullptr) {
    if (!d_out || !q || !k || !v || !d_q || !d_k || !d_v) return AHPC_ERR_NULL_POINTER;
    if (!o_kept || !stats_kept || !aligned16(o_kept)) o_kept = nullptr, stats_kept = nullptr;  // both or neither
    if (dtype < AHPC_F32 || dtype > AHPC_BF16) return AHPC_ERR_BAD_DTYPE;
    if (B <= 0 || N <= 0 || H <= 0 || d <= 0 || H_kv <= 0) return AHPC_ERR_BAD_SHAPE;
    if (H % H_kv) return AHPC_ERR_BAD_SHAPE;
    if (B > 65535 || H > 65535 || N > 0x7FFFFF00ll) return AHPC_ERR_BAD_SHAPE;
    if (d > 256) return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
    if (stride_n < d || stride_h < d || stride_b < 0 || kv_stride_n < d || kv_stride_h < d || kv_stride_b < 0)
        return AHPC_ERR_BAD_SHAPE;
    if (!workspace) return AHPC_ERR_NULL_POINTER;
    if (workspace_bytes < ahpc_hip_flash_bwd_workspace_bytes(B, N, H)) return AHPC_ERR_WORKSPACE_TOO_SMALL;
    if (!aligned16(workspace)) return AHPC_ERR_BAD_ALIGNMENT;
    if (!(scale > 0.0f)) scale = 1.0f / std::sqrt((float)d);
    hipStream_t st = static_cast<hipStream_t>(stream);

    BwdParams p{};
    p.q = q; p.k = k; p.v = v; p.d_out = d_out;
    p.d_q = d_q; p.d_k = d_k; p.d_v = d_v;
    p.mask = mask;
    p.cu_seqlens = cu_seqlens;
    p.lse = static_cast<float*>(workspace);
    p.rows_padded = padded_rows(N);
    p.delta = p.lse + (size_t)B * (size_t)H * (size_t)p.rows_padded;
    p.stride_b = stride_b; p.stride_n = stride_n; p.stride_h = stride_h;
    p.kv_stride_b = kv_stride_b; p.kv_stride_n = kv_stride_n; p.kv_stride_h = kv_stride_h;
    p.N = (int32_t)N; p.H = (int32_t)H; p.d = (int32_t)d;
    p.kv_group = (int32_t)(H / H_kv);
    p.scale = scale;
    p.causal = causal ? 1 : 0;
    // fp16 / bf16 with d in {64, 128}, 16-byte aligned rows and no dense mask: the matrix-core kernels
    const bool strides_ok = !(stride_b % 8) && !(stride_n % 8) && !(stride_h % 8) && !(kv_stride_b % 8) && !(kv_stride_n % 8) &&
                            !(kv_stride_h % 8) && stride_n < (int64_t(1) << 24) && kv_stride_n < (int64_t(1) << 24);
    // fp32 with d in {64, 128} likewise (rows of whole 16-byte pieces): the fp32 matrix-core kernels
    const bool strides4_ok = !(stride_b % 4) && !(stride_n % 4) && !(stride_h % 4) && !(kv_stride_b % 4) && !(kv_stride_n % 4) &&
                             !(kv_stride_h % 4) && stride_n < (int64_t(1) << 24) && kv_stride_n < (int64_t(1) << 24);
    const bool is16 = dtype == AHPC_F16 || dtype == AHPC_BF16;
    // head dimensions up to 256 (fp32: 128) in whole 16-byte pieces; one below 64, 128 or 256 runs on the next kernel
    // (FlashParams::d_real)
    const bool d_ok = d <= (is16 ? 256 : 128) && d >= (is16 ? 8 : 4) && d % (is16 ? 8 : 4) == 0;
    const int kernel_d = d <= 64 ? 64 : d <= 128 ? 128 : 256;
    const bool tensors_ok = d_ok && (is16 ? strides_ok : strides4_ok) && aligned16(q) && aligned16(k) && aligned16(v) &&
                            aligned16(d_out) && aligned16(d_q) && aligned16(d_k) && aligned16(d_v);
    if (tensors_ok && (!mask || (is16 && !cu_seqlens && tuning().mask_pack.load() != 0))) {
        FlashBwdParams m{};
        m.q = q; m.k = k; m.v = v; m.d_out = d_out;
        m.d_q = d_q; m.d_k = d_k; m.d_v = d_v;
        m.neg_lse2 = p.lse; m.neg_delta = p.delta; m.rows_padded = p.rows_padded;
        m.cu_seqlens = cu_seqlens;
        m.stride_b = stride_b; m.stride_n = stride_n; m.stride_h = stride_h;
        m.kv_stride_b = kv_stride_b; m.kv_stride_n = kv_stride_n; m.kv_stride_h = kv_stride_h;
        m.N = (int32_t)N; m.H = (int32_t)H; m.kv_group = p.kv_group;
        m.scale = scale;
        m.scale_log2 = scale * kLog2e;
        m.d_real = (int32_t)d;
        if (!mask) {
            if (dtype == AHPC_F32) return launch_f32_mfma(m, B, H_kv, kernel_d, causal != 0, p.lse, p.delta, st);
            return dtype == AHPC_F16 ? launch_mfma<f16_t>(m, nullptr, o_kept, stats_kept, B, H_kv, kernel_d, causal != 0, p.lse, p.delta, st)
                                     : launch_mfma<bf16_t>(m, nullptr, o_kept, stats_kept, B, H_kv, kernel_d, causal != 0, p.lse, p.delta, st);
        }
        // a dense mask on 16-bit tensors: the matrix-core kernels on the mask's packed copy (both layouts), where that
        // can be made (not under graph capture, not beyond the library's buffer limit)
        bool launched = false;
        const int rc = with_packed_mask(mask, B, N, true, st, &launched, [&](const PackedMask& pm) {
            return dtype == AHPC_F16 ? launch_mfma<f16_t>(m, &pm, o_kept, stats_kept, B, H_kv, kernel_d, causal != 0, p.lse, p.delta, st)
                                     : launch_mfma<bf16_t>(m, &pm, o_kept, stats_kept, B, H_kv, kernel_d, causal != 0, p.lse, p.delta, st);
        });
        if (launched || rc != AHPC_OK) return rc;
    }
    switch (dtype) {
        case AHPC_F32: return launch_simple<float>(p, B, H_kv, st);
        case AHPC_F16: return launch_simple<f16_t>(p, B, H_kv, st);
        default: return launch_simple<bf16_t>(p, B, H_kv, st);
    }
}

int ahpc_hip_flash_bwd(const void* d_out, const void* q, const void* k, const void* v, void* d_q, void* d_k, void* d_v,
                       int dtype, int64_t B, int64_t N, int64_t H, int64_t H_kv, int64_t d, int64_t stride_b, int64_t stride_n,
                       int64_t stride_h, int64_t kv_stride_b, int64_t kv_stride_n, int64_t kv_stride_h, float scale, int causal,
                       const float* mask, void* workspace, size_t workspace_bytes, void* stream) {
    return flash_bwd_any(d_out, q, k, v, d_q, d_k, d_v, dtype, nullptr, B, N, H, H_kv, d, stride_b, stride_n, stride_h,
                         kv_stride_b, kv_stride_n, kv_stride_h, scale, causal, mask, workspace, workspace_bytes, stream);
}

size_t ahpc_hip_flash_row_stats_bytes(int64_t B, int64_t N, int64_t H) {
    if (B <= 0 || N <= 0 || H <= 0) return 0;
    return (size_t)B * (size_t)H * (size_t)padded_rows(N) * sizeof(float);
}

int ahpc_hip_flash_bwd_kept(const void* d_out, const void* q, const void* k, const void* v, const void* o, const float* row_stats,
                            void* d_q, void* d_k, void* d_v, int dtype, int64_t B, int64_t N, int64_t H, int64_t H_kv, int64_t d,
                            int64_t stride_b, int64_t stride_n, int64_t stride_h, int64_t kv_stride_b, int64_t kv_stride_n,
                            int64_t kv_stride_h, float scale, int causal, const float* mask, void* workspace,
                            size_t workspace_bytes, void* stream) {
    return flash_bwd_any(d_out, q, k, v, d_q, d_k, d_v, dtype, nullptr, B, N, H, H_kv, d, stride_b, stride_n, stride_h,
                         kv_stride_b, kv_stride_n, kv_stride_h, scale, causal, mask, workspace, workspace_bytes, stream, o,
                         row_stats);
}

int ahpc_hip_flash_bwd_varlen(const void* d_out, const void* q, const void* k, const void* v, void* d_q, void* d_k, void* d_v,
                              int dtype, const int32_t* cu_seqlens, int64_t n_seqs, int64_t max_len, int64_t H, int64_t H_kv,
                              int64_t d, int64_t stride_t, int64_t stride_h, int64_t kv_stride_t, int64_t kv_stride_h,
                              float scale, int causal, void* workspace, size_t workspace_bytes, void* stream) {
    if (!cu_seqlens) return AHPC_ERR_NULL_POINTER;
    return flash_bwd_any(d_out, q, k, v, d_q, d_k, d_v, dtype, cu_seqlens, n_seqs, max_len, H, H_kv, d, 0, stride_t, stride_h, 0,
                         kv_stride_t, kv_stride_h, scale, causal, nullptr, workspace, workspace_bytes, stream);
}

}  // extern "C"
