// FlashAttention backward for fp32 tensors on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32), the counterpart of
// flash_bwd_mfma.hpp for the reference's default data type (FlashAttention::backward,
// src/algorithms/flash_attention.cpp:114-174, 496-580; its gradient test runs in fp32,
// tests/test_flash_attention.cpp:405-480).  Three steps, no atomics, as for 16-bit tensors:
//   1. statistics (flash_bwd_stats_f32_mfma_kernel, flash_fwd_f32_mfma.hpp): -lse2 and -delta per query row,
//   2. dQ: a workgroup owns 128 query rows (a wavefront 32 of them, as columns) and walks the keys 32 at a time:
//          S^T  = K Q^T - lse2      A = K rows (16-byte LDS reads), B = Q^T registers (scaled by scale*log2 e), C = -lse2
//          dP^T = V dO^T - delta    A = V rows,                     B = dO^T registers,                          C = -delta
//          dS^T = exp2(S^T) o dP^T  in registers
//          dQ^T += K^T dS^T         A = K^T: one float of a K row per lane and instruction, B = dS^T where it stands
//   3. dK, dV: a workgroup owns 128 key rows (a wavefront 32, as columns) and walks the queries 32 at a time, once
//      per query head of its K/V head, in two launches (each fits its registers):
//          S  = Q K^T - lse2        A = Q rows, B = K^T registers (scaled), C = -lse2 of the ROW: 4 runs of 4 per lane
//          dV^T += dO^T P           A = dO^T: one float per lane, B = P = exp2(S) where it stands          (dV walk)
//          dP = dO V^T - delta;  dS = P o dP;  dK^T += Q^T dS   A = Q^T: one float per lane               (dK walk)
// The contraction index of an instruction's two halves is chosen as in the forward kernel, so that no operand is
// shuffled: products over d let half h take d = 8m + 4h + e in step 4m + e, products over the 32 rows of a tile let
// half h take row 8g + 4h + e in step 4g + e, the row that result register 4g + e of the first products holds.
//
// Tiles are read both ways (16 bytes along a row, single floats down a column), so every tile carries the row
// swizzle of the forward's K tile (chunk c of row r at c ^ (r % chunks)); the single-float reads then meet a two-way
// bank conflict on half of their instructions, which is nothing next to 64-cycle matrix instructions.
#pragma once

#include "flash_bwd_mfma.hpp"
#include "flash_fwd_f32_mfma.hpp"

namespace ahpc {

// Geometry and addressing of a 32-row fp32 tile in LDS, shared by the kernels below.
template <int D> struct F32Tile {
    static constexpr int RB = 4 * D;               // row bytes
    static constexpr int CH = D / 4;               // 16-byte chunks per row
    static constexpr int RPI = 1024 / RB;          // rows one load instruction covers
    static constexpr int IPW = kF32Keys / RPI / 4; // load instructions per wavefront and tile
    static constexpr int MS = D / 8;               // 16-byte row reads (= register quads) per lane
    static constexpr int MB = D / 32;              // 32-row blocks of a transposed result
    static constexpr int kBytes = kF32Keys * RB;
    __device__ static int f(int r) { return r & (CH - 1); }
    // byte offset of the load instruction i of this wavefront: row, and the chunk that belongs at the lane's place
    // (a head dimension d below D: the columns from d on fetch the row's first chunk again, FlashParams::d_real)
    __device__ static int dma_off(int wave, int lane, int i, int64_t stride_elems, int d) {
        const int r = (wave * IPW + i) * RPI + lane / CH;
        const int ch = (lane % CH) ^ f(r);
        return (int)(r * stride_elems * 4) + ((4 * ch < d ? ch : 0) << 4);
    }
    // 16 bytes of row `col`: logical chunk 2m + half
    __device__ static int row_off(int col, int half, int m) { return col * RB + (((2 * m + half) ^ f(col)) << 4); }
    // One float of column 32 mb + col from the row a lane contracts in step 4g + e, row0 = 8g + e for half 0 and
    // row0 + 4 for half 1.  The swizzle of those rows differs from row0's by 4 half in the chunk index, and row0's own
    // is a compile-time constant: lane part + constant part.
    __device__ static int col_lane_off(int col, int half, int e) {
        return 4 * half * RB + ((((col >> 2) ^ (half << 2)) ^ e) << 4) + ((col & 3) << 2);
    }
    __device__ static constexpr int col_const_off(int row0, int mb) { return row0 * RB + ((((8 * mb) ^ (row0 & (CH - 1))) & ~7) << 4); }
};

template <int D>
__device__ inline void f32_dma_tile(const float* base, unsigned nrec, const int* off, unsigned char* lds, int wave_u) {
#pragma unroll
    for (int i = 0; i < F32Tile<D>::IPW; ++i) dma_instr(base, nrec, off[i], lds + (wave_u * F32Tile<D>::IPW + i) * 1024);
}

// grid: 8 * per_xcd_q workgroups, see bwd_work_of_block
template <int D, bool CAUSAL, bool VARLEN>
__global__ __launch_bounds__(kFlashThreads, (D == 128 ? 1 : 2)) void flash_bwd_dq_f32_mfma_kernel(const FlashBwdParams p) {
    typedef F32Tile<D> TL;
    constexpr int MS = TL::MS, MB = TL::MB, RB = TL::RB;

    __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[TL::kBytes];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 31;
    const int half = lane >> 5;
    const BwdWork work = bwd_work_of_block(blockIdx.x, p.total_q, p.per_xcd_q, bwd_units(p));
    if (!work.valid) return;
    const int b = work.bh / p.H, h = work.bh - b * p.H;
    const int hk = h / p.kv_group;
    int L;
    int64_t base, kv_base;
    if (VARLEN) {
        const int s0 = p.cu_seqlens[b];
        L = p.cu_seqlens[b + 1] - s0;
        base = (int64_t)s0 * p.stride_n + (int64_t)h * p.stride_h;
        kv_base = (int64_t)s0 * p.kv_stride_n + (int64_t)hk * p.kv_stride_h;
    } else {
        L = p.N;
        base = (int64_t)b * p.stride_b + (int64_t)h * p.stride_h;
        kv_base = (int64_t)b * p.kv_stride_b + (int64_t)hk * p.kv_stride_h;
    }
    const float* const gq = static_cast<const float*>(p.q) + base;
    const float* const gdo = static_cast<const float*>(p.d_out) + base;
    const float* const gk = static_cast<const float*>(p.k) + kv_base;
    const float* const gv = static_cast<const float*>(p.v) + kv_base;
    const int64_t sn = p.stride_n;
    const int64_t skv = p.kv_stride_n;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int d_real = (p.d_real > 0 && p.d_real < D) ? p.d_real : D;

    int dma_off[TL::IPW];
#pragma unroll
    for (int i = 0; i < TL::IPW; ++i) dma_off[i] = TL::dma_off(wave, lane, i, skv, d_real);
    auto dma_both = [&](int k0, unsigned char* dst_k, unsigned char* dst_v) {
        const int64_t rem = k0 < L ? (int64_t)(L - k0 - 1) * skv * 4 + 4 * d_real : 0;
        const unsigned nrec = rem > 0xffffffffll ? 0xffffffffu : (unsigned)rem;
        f32_dma_tile<D>(gk + (int64_t)k0 * skv, nrec, dma_off, dst_k, wave_u);
        f32_dma_tile<D>(gv + (int64_t)k0 * skv, nrec, dma_off, dst_v, wave_u);
    };
    int row_off[MS];
#pragma unroll
    for (int m = 0; m < MS; ++m) row_off[m] = TL::row_off(col, half, m);
    int col_off[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) col_off[e] = TL::col_lane_off(col, half, e);

    for (int part = 0; part < 2; ++part) {
        // long tiles first: under a causal mask the late query tiles walk the most keys; a paired workgroup then takes the
        // early tile that completes its share
        const int tile = part == 0 ? work.tile : p.n_tiles - 1 - work.tile;
        if (part == 1 && (!p.paired || tile == work.tile)) break;
        const int q_tile0 = (p.n_tiles - 1 - tile) * kFlashRows;
        if (q_tile0 >= L) continue;  // ragged batches: a sequence shorter than the longest one
        if (part == 1) __syncthreads();  // every wavefront is done with the first pass's last tile
        int k_end = L;
        if (CAUSAL) k_end = (q_tile0 + kFlashRows) < L ? (q_tile0 + kFlashRows) : L;
        const int n_tiles = (k_end + kF32Keys - 1) / kF32Keys;
        dma_both(0, lds_k0, lds_v0);

        const int qw = q_tile0 + wave * 32;
        const int qrow = qw + col;
        f32x4 qreg[MS], doreg[MS];
        {
            const int row = qrow < L ? qrow : L - 1;
            const float c = p.scale_log2;
            const float* sq = gq + (int64_t)row * sn + 4 * half;
            const float* sd = gdo + (int64_t)row * sn + 4 * half;
#pragma unroll
            for (int m = 0; m < MS; ++m) {
                const bool there = 8 * m + 4 * half < d_real;  // columns the tensors have
                const f32x4 raw = there ? *reinterpret_cast<const f32x4*>(sq + 8 * m) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                qreg[m] = f32x4{raw[0] * c, raw[1] * c, raw[2] * c, raw[3] * c};
                doreg[m] = there ? *reinterpret_cast<const f32x4*>(sd + 8 * m) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
        f32x16 neg_lse, neg_delta, zero;
        {
            const int64_t stat = ((int64_t)b * p.H + h) * p.rows_padded + qrow;  // qrow < rows_padded always
            const float a = p.neg_lse2[stat], d0 = p.neg_delta[stat];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                neg_lse[r] = a;
                neg_delta[r] = d0;
                zero[r] = 0.0f;
            }
        }
        f32x16 acc[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[mb] = zero;

        auto compute_tile = [&](const unsigned char* tile_k, const unsigned char* tile_v, int k0) {
            // ---- S^T and dP^T, each in two chains (even and odd quads): four independent chains of matrix instructions
            f32x16 s = neg_lse, s_odd = zero, dp = neg_delta, dp_odd = zero;
            __builtin_amdgcn_s_setprio(1);
            {
                u32x4 kq[MS], vq[MS];
#pragma unroll
                for (int m = 0; m < MS; ++m) {
                    kq[m] = lds_read_b128(tile_k + row_off[m]);
                    vq[m] = lds_read_b128(tile_v + row_off[m]);
                }
#pragma unroll
                for (int m = 0; m < MS; m += 2)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        s = mfma_32x32x2_f32(as_f32(kq[m][e]), qreg[m][e], s);
                        dp = mfma_32x32x2_f32(as_f32(vq[m][e]), doreg[m][e], dp);
                        s_odd = mfma_32x32x2_f32(as_f32(kq[m + 1][e]), qreg[m + 1][e], s_odd);
                        dp_odd = mfma_32x32x2_f32(as_f32(vq[m + 1][e]), doreg[m + 1][e], dp_odd);
                    }
                // the quads of two steps are requested before the first product, those of another behind every 16 products
                __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);  // LDS reads
#pragma unroll
                for (int i = 0; i < MS / 2 - 2; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 16, 0);  // matrix instructions
                    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, 32, 0);
            }
            __builtin_amdgcn_s_setprio(0);
            // ---- dS^T = exp2(S^T) o dP^T; keys the query may not see (key of register r: k0 + 8 (r / 4) + 4 half + r % 4)
            const bool need_mask = (k0 + kF32Keys > L) || (CAUSAL && (k0 + kF32Keys - 1 > qw));
            int lim = 64;
            if (need_mask) {
                lim = L - 1;
                if (CAUSAL) lim = qrow < lim ? qrow : lim;
                lim -= k0 + 4 * half;
            }
            f32x16 ds;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float sv = s[r] + s_odd[r];
                const float pv = (8 * (r >> 2) + (r & 3)) <= lim ? fast_exp2(sv) : 0.0f;
                ds[r] = pv * (dp[r] + dp_odd[r]);
            }
            // ---- dQ^T += K^T dS^T: step r = 4g + e contracts keys 8g + e (half 0) and 8g + 4 + e (half 1)
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row0 = 8 * (r >> 2) + (r & 3);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const float a = *reinterpret_cast<const float*>(tile_k + TL::col_const_off(row0, mb) + col_off[r & 3]);
                    acc[mb] = mfma_32x32x2_f32(a, ds[r], acc[mb]);
                }
            }
            __builtin_amdgcn_s_setprio(0);
        };

        auto step = [&](unsigned char* cur_k, unsigned char* cur_v, unsigned char* nxt_k, unsigned char* nxt_v, int t) {
            const int k0 = t * kF32Keys;
            const bool more = t + 1 < n_tiles;
            if (more) dma_both(k0 + kF32Keys, nxt_k, nxt_v);
            if (!(CAUSAL && k0 > qw + 31)) compute_tile(cur_k, cur_v, k0);
            if (more) {
                __builtin_amdgcn_s_waitcnt(0);
                __syncthreads();
            }
        };

        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        for (int t = 0; t < n_tiles; t += 2) {
            step(lds_k0, lds_v0, lds_k1, lds_v1, t);
            if (t + 1 < n_tiles) step(lds_k1, lds_v1, lds_k0, lds_v0, t + 1);
        }

        if (qrow < L) {
            float* dst = static_cast<float*>(p.d_q) + base + (int64_t)qrow * sn + 4 * half;
            const float sc = p.scale;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4)
                    if (32 * mb + 8 * g4 + 4 * half < d_real)
                        *reinterpret_cast<f32x4*>(dst + 32 * mb + 8 * g4) =
                            f32x4{acc[mb][4 * g4] * sc, acc[mb][4 * g4 + 1] * sc, acc[mb][4 * g4 + 2] * sc, acc[mb][4 * g4 + 3] * sc};
        }
    }
}

// grid: 8 * per_xcd_kv workgroups, see bwd_work_of_block.  PART 1: the dV walk, PART 2: the dK walk.
template <int D, bool CAUSAL, bool VARLEN, int PART>
__global__ __launch_bounds__(kFlashThreads, (PART == 2 ? 1 : 2)) void flash_bwd_dkv_f32_mfma_kernel(const FlashBwdParams p) {
    static_assert(PART == 1 || PART == 2, "one launch per gradient");
    constexpr bool kDoK = PART == 2;
    typedef F32Tile<D> TL;
    constexpr int MS = TL::MS, MB = TL::MB, RB = TL::RB;

    __shared__ __attribute__((aligned(1024))) unsigned char lds_q0[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_o0[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_q1[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_o1[TL::kBytes];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 31;
    const int half = lane >> 5;
    const BwdWork work = bwd_work_of_block(blockIdx.x, p.total_kv, p.per_xcd_kv, bwd_units(p));
    if (!work.valid) return;
    const int heads_kv = p.H / p.kv_group;
    const int b = work.bh / heads_kv, hk = work.bh - b * heads_kv;
    int seq0 = 0;
    int L = p.N;
    if (VARLEN) {
        seq0 = p.cu_seqlens[b];
        L = p.cu_seqlens[b + 1] - seq0;
    }
    const int64_t kv_base = VARLEN ? (int64_t)seq0 * p.kv_stride_n + (int64_t)hk * p.kv_stride_h
                                   : (int64_t)b * p.kv_stride_b + (int64_t)hk * p.kv_stride_h;
    const float* const gk = static_cast<const float*>(p.k) + kv_base;
    const float* const gv = static_cast<const float*>(p.v) + kv_base;
    const int64_t sn = p.stride_n;
    const int64_t skv = p.kv_stride_n;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int d_real = (p.d_real > 0 && p.d_real < D) ? p.d_real : D;

    int dma_off[TL::IPW];
#pragma unroll
    for (int i = 0; i < TL::IPW; ++i) dma_off[i] = TL::dma_off(wave, lane, i, sn, d_real);
    int row_off[MS];
#pragma unroll
    for (int m = 0; m < MS; ++m) row_off[m] = TL::row_off(col, half, m);
    int col_off[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) col_off[e] = TL::col_lane_off(col, half, e);

    for (int part = 0; part < 2; ++part) {
        // under a causal mask the early key tiles see the most queries: they go first; a paired workgroup then takes the
        // late tile that completes its share
        const int tile = part == 0 ? work.tile : p.n_tiles - 1 - work.tile;
        if (part == 1 && (!p.paired || tile == work.tile)) break;
        const int k_tile0 = tile * kFlashRows;
        if (k_tile0 >= L) continue;  // ragged batches: a sequence shorter than the longest one
        const int kw = k_tile0 + wave * 32;  // first key of this wavefront
        const int key = kw + col;
        f32x4 kreg[MS], vreg[kDoK ? MS : 1];
        {
            const int krow = key < L ? key : L - 1;
            const float c = p.scale_log2;
            const float* sk = gk + (int64_t)krow * skv + 4 * half;
            const float* sv = gv + (int64_t)krow * skv + 4 * half;
#pragma unroll
            for (int m = 0; m < MS; ++m) {
                const bool there = 8 * m + 4 * half < d_real;  // columns the tensors have
                const f32x4 raw = there ? *reinterpret_cast<const f32x4*>(sk + 8 * m) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                kreg[m] = f32x4{raw[0] * c, raw[1] * c, raw[2] * c, raw[3] * c};
                if constexpr (kDoK) vreg[m] = there ? *reinterpret_cast<const f32x4*>(sv + 8 * m) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
        f32x16 zero;
#pragma unroll
        for (int r = 0; r < 16; ++r) zero[r] = 0.0f;
        f32x16 acc[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[mb] = zero;

        // queries before the first key of the workgroup see none of its keys under a causal mask
        const int t_begin = CAUSAL ? k_tile0 / kF32Keys : 0;
        const int n_tiles = (L + kF32Keys - 1) / kF32Keys;

        for (int g = 0; g < p.kv_group; ++g) {
            const int h = hk * p.kv_group + g;
            const int64_t base = VARLEN ? (int64_t)seq0 * p.stride_n + (int64_t)h * p.stride_h
                                        : (int64_t)b * p.stride_b + (int64_t)h * p.stride_h;
            const float* const gq = static_cast<const float*>(p.q) + base;
            const float* const gdo = static_cast<const float*>(p.d_out) + base;
            const float* const lse2 = p.neg_lse2 + ((int64_t)b * p.H + h) * p.rows_padded;
            const float* const delta = p.neg_delta + ((int64_t)b * p.H + h) * p.rows_padded;

            auto dma_both = [&](int i0, unsigned char* dst_q, unsigned char* dst_o) {
                const int64_t rem = i0 < L ? (int64_t)(L - i0 - 1) * sn * 4 + 4 * d_real : 0;
                const unsigned nrec = rem > 0xffffffffll ? 0xffffffffu : (unsigned)rem;
                f32_dma_tile<D>(gq + (int64_t)i0 * sn, nrec, dma_off, dst_q, wave_u);
                f32_dma_tile<D>(gdo + (int64_t)i0 * sn, nrec, dma_off, dst_o, wave_u);
            };
            // The statistics of a tile's 32 queries: register r of a result belongs to query i0 + 8 (r / 4) + 4 half + r % 4,
            // i.e. a lane needs 4 runs of 4 consecutive rows (the arrays are padded to whole 128-row tiles, so rows from
            // i0 < L on always exist).  They are loaded one tile ahead, BEFORE the next tile is requested: loads complete in
            // order, and waiting for a load issued behind the tile's requests would wait for the tile.
            auto load_stats = [&](const float* src, int i0, f32x16& out) {
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const f32x4 w = *reinterpret_cast<const f32x4*>(src + i0 + 8 * g4 + 4 * half);
#pragma unroll
                    for (int e = 0; e < 4; ++e) out[4 * g4 + e] = w[e];
                }
            };

            auto compute_tile = [&](const unsigned char* tile_q, const unsigned char* tile_o, int i0, const f32x16& nl, const f32x16& nd) {
                // ---- S = Q K^T - lse2 (and dP = dO V^T - delta), two chains each
                f32x16 s = nl, s_odd = zero, dp = nd, dp_odd = zero;
                __builtin_amdgcn_s_setprio(1);
                {
                    u32x4 qq[MS], oq[kDoK ? MS : 1];
#pragma unroll
                    for (int m = 0; m < MS; ++m) {
                        qq[m] = lds_read_b128(tile_q + row_off[m]);
                        if constexpr (kDoK) oq[m] = lds_read_b128(tile_o + row_off[m]);
                    }
#pragma unroll
                    for (int m = 0; m < MS; m += 2)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            s = mfma_32x32x2_f32(as_f32(qq[m][e]), kreg[m][e], s);
                            if constexpr (kDoK) dp = mfma_32x32x2_f32(as_f32(oq[m][e]), vreg[m][e], dp);
                            s_odd = mfma_32x32x2_f32(as_f32(qq[m + 1][e]), kreg[m + 1][e], s_odd);
                            if constexpr (kDoK) dp_odd = mfma_32x32x2_f32(as_f32(oq[m + 1][e]), vreg[m + 1][e], dp_odd);
                        }
                    constexpr int kReads = kDoK ? 4 : 2, kProducts = kDoK ? 16 : 8;  // per step of two quads
                    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kReads, 0);
#pragma unroll
                    for (int i = 0; i < MS / 2 - 2; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, kProducts, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, kReads, 0);
                    }
                    __builtin_amdgcn_sched_group_barrier(0x008, 2 * kProducts, 0);
                }
                __builtin_amdgcn_s_setprio(0);
                // ---- P = exp2(S) where the query (row of register r: i0 + 8 (r / 4) + 4 half + r % 4) may see the key
                const bool need_mask = CAUSAL && (i0 < kw + 31);   // rows beyond the sequence carry -lse2 = -inf: weight 0
                int first_row = -64;
                if (need_mask) first_row = key - i0 - 4 * half;     // visible iff 8 (r / 4) + r % 4 >= first_row
                f32x16 w;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float pv = (8 * (r >> 2) + (r & 3)) >= first_row ? fast_exp2(s[r] + s_odd[r]) : 0.0f;
                    w[r] = kDoK ? pv * (dp[r] + dp_odd[r]) : pv;
                }
                // ---- dV^T += dO^T P  /  dK^T += Q^T dS: step r = 4g + e contracts queries 8g + e (half 0), 8g + 4 + e (half 1)
                const unsigned char* const tile_a = kDoK ? tile_q : tile_o;
                __builtin_amdgcn_s_setprio(1);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row0 = 8 * (r >> 2) + (r & 3);
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        const float a = *reinterpret_cast<const float*>(tile_a + TL::col_const_off(row0, mb) + col_off[r & 3]);
                        acc[mb] = mfma_32x32x2_f32(a, w[r], acc[mb]);
                    }
                }
                __builtin_amdgcn_s_setprio(0);
            };

            f32x16 nl_a = zero, nd_a = zero, nl_b = zero, nd_b = zero;
            auto step = [&](unsigned char* cur_q, unsigned char* cur_o, unsigned char* nxt_q, unsigned char* nxt_o, int t,
                            const f32x16& nl, const f32x16& nd, f32x16& nl_next, f32x16& nd_next) {
                const int i0 = t * kF32Keys;
                const bool more = t + 1 < n_tiles;
                if (more) {
                    load_stats(lse2, i0 + kF32Keys, nl_next);
                    if constexpr (kDoK) load_stats(delta, i0 + kF32Keys, nd_next);
                    __builtin_amdgcn_sched_barrier(0);
                    dma_both(i0 + kF32Keys, nxt_q, nxt_o);
                }
                // a wavefront whose keys all follow this tile's queries has nothing to add under a causal mask
                if (!(CAUSAL && i0 + 31 < kw)) compute_tile(cur_q, cur_o, i0, nl, nd);
                if (more) {
                    __builtin_amdgcn_s_waitcnt(0);
                    __syncthreads();
                }
            };

            __syncthreads();  // every wavefront is done with the previous head's last tile
            load_stats(lse2, t_begin * kF32Keys, nl_a);
            if constexpr (kDoK) load_stats(delta, t_begin * kF32Keys, nd_a);
            dma_both(t_begin * kF32Keys, lds_q0, lds_o0);
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            for (int t = t_begin; t < n_tiles; t += 2) {
                step(lds_q0, lds_o0, lds_q1, lds_o1, t, nl_a, nd_a, nl_b, nd_b);
                if (t + 1 < n_tiles) step(lds_q1, lds_o1, lds_q0, lds_o0, t + 1, nl_b, nd_b, nl_a, nd_a);
            }
        }

        if (key < L) {
            float* dst = static_cast<float*>(kDoK ? p.d_k : p.d_v) + kv_base + (int64_t)key * skv + 4 * half;
            const float sc = kDoK ? p.scale : 1.0f;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4)
                    if (32 * mb + 8 * g4 + 4 * half < d_real)
                        *reinterpret_cast<f32x4*>(dst + 32 * mb + 8 * g4) =
                            f32x4{acc[mb][4 * g4] * sc, acc[mb][4 * g4 + 1] * sc, acc[mb][4 * g4 + 2] * sc, acc[mb][4 * g4 + 3] * sc};
        }
    }
}

}  // namespace ahpc
