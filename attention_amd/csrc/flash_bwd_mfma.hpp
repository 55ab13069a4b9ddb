// FlashAttention backward on the gfx950 matrix cores (fp16 / bf16 storage, fp32 accumulate), dense batches.
//
// Input: Q, K, V, dO and the per-row statistics of the forward (lse2 = log2 sum_j exp2(c q.k_j) with
// c = scale*log2(e), delta = dO.O; written, negated, by flash_bwd_stats_mfma_kernel).  With P = exp2(c q.k - lse2):
//
//   flash_bwd_dq_mfma_kernel    a workgroup owns 128 query rows (32 per wavefront) and walks the keys in
//       tiles of 64, exactly like the forward:  S^T = K Q^T and dP^T = V dO^T  (A = rows of the K / V tile
//       in LDS, B = Q / dO held in registers; the products start from accumulators holding -lse2 and
//       -delta, so they deliver c q.k - lse2 and dO.v - delta directly),  dS^T = exp2(S^T) o dP^T,
//       dQ^T += K^T dS^T  (A = K^T by transposing LDS reads, B = dS^T straight from the registers it was
//       computed in, as P^T in the forward).  dQ = scale * dQ^T^T.
//
//   flash_bwd_dkv_mfma_kernel   the mirror image: a workgroup owns 128 key rows (32 per wavefront, held in
//       registers as B operands) and walks the queries in tiles of 64:  S = Q K^T, dP = dO V^T  (A = rows
//       of the Q / dO tile in LDS, accumulators start from the tile's -lse2 / -delta per row),
//       P = exp2(S), dS = P o dP,  dV^T += dO^T P,  dK^T += Q^T dS  (A = dO^T / Q^T by transposing LDS reads,
//       B = P / dS from registers).  With grouped heads the query heads of the group are walked one after
//       the other into the same accumulators.  dK = scale * dK^T^T, dV = dV^T^T.
//
// In both kernels a lane owns one row of the output (a query, a key) and the masks are per-lane
// comparisons.  Tiles are streamed with direct-to-LDS loads and double buffered as in the forward; every
// tile is read by rows (first two products) and by transposing reads (last products); its swizzle
// (FlashTile::fb) keeps both kinds of read free of LDS bank conflicts.  No atomics: every output element is written once.
#pragma once

#include "flash_fwd_mfma.hpp"

namespace ahpc {

struct FlashBwdParams {
    const void* q;
    const void* k;
    const void* v;
    const void* d_out;
    void* d_q;
    void* d_k;
    void* d_v;
    const float* neg_lse2;      // [B*H][rows_padded]: -lse2 and -delta, what the accumulators start from
    const float* neg_delta;
    const int32_t* cu_seqlens;  // ragged batches only
    // dense mask, packed (masked kernels only; see PackedMask): 64 keys per word and query for the dQ kernel, 64 queries
    // per word and key for the dK/dV kernels; mask_tiles = ceil(N / 64)
    const uint64_t* mask_bits;
    const uint64_t* mask_bits_t;
    int32_t mask_tiles;
    int64_t rows_padded;
    int64_t stride_b, stride_n, stride_h;           // Q, dO, dQ
    int64_t kv_stride_b, kv_stride_n, kv_stride_h;  // K, V, dK, dV
    int32_t N;                  // sequence length (dense) / longest sequence (ragged)
    int32_t H;                  // query heads
    int32_t kv_group;           // query heads per key/value head
    int32_t n_tiles;            // 128-row tiles per sequence
    int32_t paired;             // 1: a workgroup takes two tiles of a head, a long walk and a short one (causal dense launches:
                                // tile i sees i + 1 tiles' worth of the other side, so i and n_tiles - 1 - i together are the
                                // same work for every workgroup); total_q / total_kv count workgroups accordingly
    int32_t total_q, per_xcd_q;     // dQ kernel: workgroups (B * H * n_tiles) and ceil(that / 8)
    int32_t total_kv, per_xcd_kv;   // dK/dV kernel: workgroups (B * H_kv * n_tiles) and ceil(that / 8)
    float scale;
    float scale_log2;           // scale * log2(e)
    int32_t d_real;             // head dimension of the tensors when smaller than the kernels' D, 0 = D (FlashParams::d_real)
};

// Workgroup id -> (sequence * heads + head, tile).  Both kernels are launched on a 1-D grid of 8 * per_xcd
// workgroups.  Hardware deals consecutive ids to the 8 XCDs in turn; `logical` undoes that, so that the tiles
// of one head (consecutive logical ids) run on one XCD and find the head's K/V (Q/dO) in its L2.
struct BwdWork {
    int bh, tile;
    bool valid;
};
// work units per head: tiles, or pairs of them
__host__ __device__ inline int bwd_units(const FlashBwdParams& p) { return p.paired ? (p.n_tiles + 1) >> 1 : p.n_tiles; }
__host__ __device__ inline BwdWork bwd_work_of_block(unsigned block_id, int total, int per_xcd, int n_tiles) {
    const int logical = (int)(block_id & 7u) * per_xcd + (int)(block_id >> 3);
    if (logical >= total) return BwdWork{0, 0, false};
    const int bh = logical / n_tiles;
    return BwdWork{bh, logical - bh * n_tiles, true};
}

// Byte offset inside a tile swizzled with FlashTile::fb of the 8 bytes a lane hands to a transposing read that fetches
// the 4 tile rows 16*g + 8*a + 4*(lane/32) + 0..3 for column quad (32*mb + 16*((lane/16)%2) + 4*(lane%4)):
// the part that does not depend on g.  Adding 16*g rows keeps the swizzle (it has period 16 rows).
template <int D>
__device__ inline int tr_offset_rowswizzled(int lane, int mb, int a) {
    typedef FlashTile<D> TL;
    const int vi = lane & 15;
    const int row = 8 * a + 4 * (lane >> 5) + (vi >> 2);
    const int cch = 4 * mb + 2 * ((lane >> 4) & 1) + ((vi & 3) >> 1);
    return row * TL::kRowBytes + ((cch ^ TL::fb(row)) << 4) + 8 * (vi & 1);
}

// Packs 8 fp32 of a 32x32 accumulator block (rows r0..r0+7 of the lane's column) as one B operand.
template <typename T>
__device__ inline u32x4 pack_operand(const f32x16& x, int r0) {
    return u32x4{pack2<T>(x[r0 + 0], x[r0 + 1]), pack2<T>(x[r0 + 2], x[r0 + 3]), pack2<T>(x[r0 + 4], x[r0 + 5]),
                 pack2<T>(x[r0 + 6], x[r0 + 7])};
}

// Loads the row `row` of a [rows][d] tensor as B operands (8 consecutive elements per k-step), scaled by c; elements from
// d on (a head dimension below the kernel's) are zero and not read.
template <typename T, int KS>
__device__ inline void load_row_operands(u32x4 (&reg)[KS], const T* row_ptr, int half, float c, int d) {
    const T* src = row_ptr + 8 * half;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const u32x4 raw = 16 * ks + 8 * half < d ? *reinterpret_cast<const u32x4*>(src + 16 * ks) : u32x4{0u, 0u, 0u, 0u};
        u32x4 sc;
#pragma unroll
        for (int w = 0; w < 4; ++w) sc[w] = pack2<T>(lo_f32<T>(raw[w]) * c, hi_f32<T>(raw[w]) * c);
        reg[ks] = sc;
    }
}

// Stores the transposed accumulators of one output row (a lane holds 4 runs of 4 consecutive elements per
// 32-element block), scaled by f; elements from d on do not exist.
template <typename T, int MB>
__device__ inline void store_row(T* dst_row, const f32x16 (&acc)[MB], int half, float f, int d) {
    T* dst = dst_row + 4 * half;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            const f32x16& a = acc[mb];
            const u32x2 w = u32x2{pack2<T>(a[4 * g4 + 0] * f, a[4 * g4 + 1] * f), pack2<T>(a[4 * g4 + 2] * f, a[4 * g4 + 3] * f)};
            if (32 * mb + 8 * g4 + 4 * half < d) *reinterpret_cast<u32x2*>(dst + 32 * mb + 8 * g4) = w;
        }
}

// grid: 8 * per_xcd_q workgroups, see bwd_work_of_block
// MASKED: a dense mask removes keys per query; the lane's word of the packed mask (its query's 64 keys of the tile) is
// loaded in front of the tile requests and tested bit by bit next to the causal / end-of-sequence test.
template <typename T, int D, bool CAUSAL, bool VARLEN, bool MASKED = false>
__global__ __launch_bounds__(kFlashThreads, (D > 128 ? 1 : 2)) void flash_bwd_dq_mfma_kernel(const FlashBwdParams p) {
    static_assert(!(MASKED && VARLEN), "the mask belongs to dense launches");
    typedef FlashTile<D> TL;
    constexpr int KS = D / 16;
    constexpr int MB = D / 32;
    constexpr int RB = TL::kRowBytes;

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
    const T* const gq = static_cast<const T*>(p.q) + base;
    const T* const gdo = static_cast<const T*>(p.d_out) + base;
    const T* const gk = static_cast<const T*>(p.k) + kv_base;
    const T* const gv = static_cast<const T*>(p.v) + kv_base;
    const int64_t sn = p.stride_n;
    const int64_t skv = p.kv_stride_n;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int d_real = (p.d_real > 0 && p.d_real < D) ? p.d_real : D;

    int dma_off[TL::kInstrPerWave];
#pragma unroll
    for (int i = 0; i < TL::kInstrPerWave; ++i) {
        const int r = (wave * TL::kInstrPerWave + i) * TL::kRowsPerInstr + lane / TL::kChunks;
        const int pc = lane % TL::kChunks;
        const int ch = pc ^ TL::fb(r);  // the row's chunk that belongs here; columns from d_real on fetch the first chunk again
        dma_off[i] = (int)(r * skv * 2) + ((8 * ch < d_real ? ch : 0) << 4);
    }
    auto dma_both = [&](int k0, unsigned char* dst_k, unsigned char* dst_v) {
        const int64_t rem = (int64_t)(L - k0 - 1) * skv * 2 + 2 * d_real;
        const unsigned nrec = rem > 0xffffffffll ? 0xffffffffu : (unsigned)rem;
        dma_tile<D>(gk + (int64_t)k0 * skv, nrec, dma_off, dst_k, wave_u);
        dma_tile<D>(gv + (int64_t)k0 * skv, nrec, dma_off, dst_v, wave_u);
    };
    // The tiles behind the first are requested one per step, in order: their addresses and the bytes that remain behind
    // them advance by a tile per request instead of being worked out from the tile number (64-bit products) every step.
    const int64_t tile_elems = (int64_t)kFlashKeys * skv;
    const T* k_next = nullptr;
    const T* v_next = nullptr;
    int64_t rem_next = 0;
    auto dma_next = [&](unsigned char* dst_k, unsigned char* dst_v) {
        const unsigned nrec = rem_next <= 0 ? 0u : rem_next > 0xffffffffll ? 0xffffffffu : (unsigned)rem_next;
        dma_tile<D>(k_next, nrec, dma_off, dst_k, wave_u);
        dma_tile<D>(v_next, nrec, dma_off, dst_v, wave_u);
        k_next += tile_elems;
        v_next += tile_elems;
        rem_next -= 2 * tile_elems;
    };

    int row_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) row_off[ks] = col * RB + (((2 * ks + half) ^ TL::fb(col)) << 4);
    int tr_off[MB][2];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int a = 0; a < 2; ++a) tr_off[mb][a] = tr_offset_rowswizzled<D>(lane, mb, a);

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
        const int n_tiles = (k_end + kFlashKeys - 1) / kFlashKeys;
        dma_both(0, lds_k0, lds_v0);
        k_next = gk + tile_elems;
        v_next = gv + tile_elems;
        rem_next = (int64_t)(L - kFlashKeys - 1) * skv * 2 + 2 * d_real;

        const int qw = q_tile0 + wave * 32;
        const int qrow = qw + col;
        const int row = qrow < L ? qrow : L - 1;
        u32x4 qreg[KS], doreg[KS];
        load_row_operands<T, KS>(qreg, gq + (int64_t)row * sn, half, p.scale_log2, d_real);
        load_row_operands<T, KS>(doreg, gdo + (int64_t)row * sn, half, 1.0f, d_real);
        const int64_t stat = ((int64_t)b * p.H + h) * p.rows_padded + qrow;  // qrow < rows_padded always
        const uint64_t* const mword = MASKED ? p.mask_bits + (int64_t)b * p.mask_tiles * p.N + row : nullptr;
        f32x16 neg_lse, neg_delta;
        {
            const float a = p.neg_lse2[stat], d0 = p.neg_delta[stat];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                neg_lse[r] = a;
                neg_delta[r] = d0;
            }
        }
        f32x16 acc[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][r] = 0.0f;

        auto compute_tile = [&](const unsigned char* tile_k, const unsigned char* tile_v, int k0, uint64_t mw) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const int kblock0 = k0 + 32 * kb;
                if (kblock0 >= L) continue;                        // nothing but padding
                if (CAUSAL && kblock0 > qw + 31) continue;        // every key of the block is in the future
                // (issue priority up while the matrix cores are fed, down for the stretch of exponentials, as in the forward)
                __builtin_amdgcn_s_setprio(1);
                // K^T operands of the block's first 16 keys: requested now, they arrive while the first two products run
                u32x2 kt[2][MB][2];
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    kt[0][mb][0] = TrRead<T>::load(tile_k + (32 * kb) * RB + tr_off[mb][0]);
                    kt[0][mb][1] = TrRead<T>::load(tile_k + (32 * kb) * RB + tr_off[mb][1]);
                }
                f32x16 s = neg_lse, dp = neg_delta;
                {
                    // the operand pairs of the two products are requested kAhead steps ahead of the matrix instructions
                    // that use them (all at once would cost 8 registers per step)
                    u32x4 ak[KS], av[KS];
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        ak[ks] = lds_read_b128(tile_k + 32 * kb * RB + row_off[ks]);
                        av[ks] = lds_read_b128(tile_v + 32 * kb * RB + row_off[ks]);
                    }
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        s = mfma_32x32x16<T>(ak[ks], qreg[ks], s);
                        dp = mfma_32x32x16<T>(av[ks], doreg[ks], dp);
                    }
                    constexpr int kAhead = 2;
                    __builtin_amdgcn_sched_group_barrier(0x100, 2 * MB + 2 * kAhead, 0);  // LDS reads (the K^T ones first)
#pragma unroll
                    for (int i = 0; i < KS - kAhead; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // matrix instructions
                        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                    }
#pragma unroll
                    for (int i = 0; i < kAhead; ++i) __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                }
                // key = kblock0 + 4*half + 8*(r/4) + r%4 is visible iff key <= min(qrow, L-1)
                __builtin_amdgcn_s_setprio(0);
                f32x16 ds;
                // the per-element test is needed only where the block meets the diagonal or the end of the sequence
                // (uniform per wavefront)
                const bool all_on = !MASKED && kblock0 + 31 < L && (!CAUSAL || kblock0 + 31 <= qw);
                if (all_on) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) ds[r] = fast_exp2(s[r]) * dp[r];
                } else {
                    int lim = L - 1;
                    if (CAUSAL) lim = qrow < lim ? qrow : lim;
                    lim -= kblock0 + 4 * half;
                    // the lane's keys of the block as bits 0.. of one word: key kblock0 + 4*half + off <-> bit off
                    const uint32_t bits = MASKED ? (uint32_t)(mw >> (32 * kb)) >> (4 * half) : 0xFFFFFFFFu;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int off = 8 * (r >> 2) + (r & 3);
                        const bool on = off <= lim && (!MASKED || ((bits >> off) & 1u));
                        ds[r] = on ? fast_exp2(s[r]) * dp[r] : 0.0f;
                    }
                }
                __builtin_amdgcn_s_setprio(1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int g2 = 0; g2 < 2; ++g2) {
                    const u32x4 bop = pack_operand<T>(ds, 8 * g2);
                    if (g2 == 0) {
                        // the second 16 keys' operands travel while the first 16 are multiplied
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb) {
                            kt[1][mb][0] = TrRead<T>::load(tile_k + (32 * kb + 16) * RB + tr_off[mb][0]);
                            kt[1][mb][1] = TrRead<T>::load(tile_k + (32 * kb + 16) * RB + tr_off[mb][1]);
                        }
                    }
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        acc[mb] = mfma_32x32x16<T>(u32x4{kt[g2][mb][0][0], kt[g2][mb][0][1], kt[g2][mb][1][0], kt[g2][mb][1][1]}, bop, acc[mb]);
                    __builtin_amdgcn_sched_barrier(0);
                }
                __builtin_amdgcn_s_setprio(0);
            }
        };

        auto step = [&](unsigned char* cur_k, unsigned char* cur_v, unsigned char* nxt_k, unsigned char* nxt_v, int t) {
            const int k0 = t * kFlashKeys;
            const bool more = t + 1 < n_tiles;
            uint64_t mw = 0;
            if constexpr (MASKED) {
                // in front of the tile requests: loads complete in order, a word requested behind them would wait for the tile
                mw = mword[(int64_t)t * p.N];
                __builtin_amdgcn_sched_barrier(0);
            }
            if (more) dma_next(nxt_k, nxt_v);
            compute_tile(cur_k, cur_v, k0, mw);
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
        if (qrow < L) store_row<T, MB>(static_cast<T*>(p.d_q) + base + (int64_t)qrow * sn, acc, half, p.scale, d_real);
    }
}

// grid: 8 * per_xcd_kv workgroups, see bwd_work_of_block
// PART: 0 = dK and dV in one walk over the query tiles (four products per tile; at d = 128 that is 324 registers, one
// wavefront per SIMD), 1 = dV only (S and dV: two products, V and dO.V never touched), 2 = dK only (S, dP, dK).  The
// two partial walks execute five products between them but each fits two wavefronts per SIMD, which hide each
// other's softmax arithmetic and LDS waits: 5 % fewer cycles at d = 128, and still the slower way on inputs that hold
// the board at its power limit, where four products beat five (the launcher picks).  The one walk overlaps its own
// vector arithmetic with its matrix products by pipelining the two blocks of a tile (see compute_tile).
// MASKED: as in the dQ kernel, with the transposed packed mask (the lane's key, 64 queries per word).
template <typename T, int D, bool CAUSAL, bool VARLEN, int PART, bool MASKED = false>
__global__ __launch_bounds__(kFlashThreads, (PART == 0 || D > 128 ? 1 : 2)) void flash_bwd_dkv_mfma_kernel(const FlashBwdParams p) {
    static_assert(!(MASKED && VARLEN), "the mask belongs to dense launches");
    constexpr bool kDoK = PART != 1, kDoV = PART != 2;
    typedef FlashTile<D> TL;
    constexpr int KS = D / 16;
    constexpr int MB = D / 32;
    constexpr int RB = TL::kRowBytes;

    __shared__ __attribute__((aligned(1024))) unsigned char lds_q0[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_o0[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_q1[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_o1[TL::kBytes];
    // the statistics of a tile's 64 queries travel with it: -lse2[64] then -delta[64]
    __shared__ __attribute__((aligned(512))) unsigned char lds_s0[512];
    __shared__ __attribute__((aligned(512))) unsigned char lds_s1[512];

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
    const T* const gk = static_cast<const T*>(p.k) + kv_base;
    const T* const gv = static_cast<const T*>(p.v) + kv_base;
    const int64_t sn = p.stride_n;
    const int64_t skv = p.kv_stride_n;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int d_real = (p.d_real > 0 && p.d_real < D) ? p.d_real : D;

    int dma_off[TL::kInstrPerWave];
#pragma unroll
    for (int i = 0; i < TL::kInstrPerWave; ++i) {
        const int r = (wave * TL::kInstrPerWave + i) * TL::kRowsPerInstr + lane / TL::kChunks;
        const int pc = lane % TL::kChunks;
        const int ch = pc ^ TL::fb(r);
        dma_off[i] = (int)(r * sn * 2) + ((8 * ch < d_real ? ch : 0) << 4);
    }
    int row_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) row_off[ks] = col * RB + (((2 * ks + half) ^ TL::fb(col)) << 4);
    int tr_off[MB][2];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int a = 0; a < 2; ++a) tr_off[mb][a] = tr_offset_rowswizzled<D>(lane, mb, a);

    for (int part = 0; part < 2; ++part) {
        // under a causal mask the early key tiles see the most queries: they go first; a paired workgroup then takes the
        // late tile that completes its share
        const int tile = part == 0 ? work.tile : p.n_tiles - 1 - work.tile;
        if (part == 1 && (!p.paired || tile == work.tile)) break;
        const int k_tile0 = tile * kFlashRows;
        if (k_tile0 >= L) continue;  // ragged batches: a sequence shorter than the longest one
        const int kw = k_tile0 + wave * 32;  // first key of this wavefront
        const int key = kw + col;
        const int krow = key < L ? key : L - 1;
        const uint64_t* const mword = MASKED ? p.mask_bits_t + (int64_t)b * p.mask_tiles * p.N + krow : nullptr;
        u32x4 kreg[KS], vreg[KS];
        load_row_operands<T, KS>(kreg, gk + (int64_t)krow * skv, half, p.scale_log2, d_real);
        if constexpr (kDoK) load_row_operands<T, KS>(vreg, gv + (int64_t)krow * skv, half, 1.0f, d_real);

        f32x16 acc_k[MB], acc_v[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                acc_k[mb][r] = 0.0f;
                acc_v[mb][r] = 0.0f;
            }

        // queries before the first key of the workgroup see none of its keys under a causal mask
        const int t_begin = CAUSAL ? k_tile0 / kFlashKeys : 0;
        const int n_tiles = (L + kFlashKeys - 1) / kFlashKeys;

        for (int g = 0; g < p.kv_group; ++g) {
            const int h = hk * p.kv_group + g;
            const int64_t base = VARLEN ? (int64_t)seq0 * p.stride_n + (int64_t)h * p.stride_h
                                        : (int64_t)b * p.stride_b + (int64_t)h * p.stride_h;
            const T* const gq = static_cast<const T*>(p.q) + base;
            const T* const gdo = static_cast<const T*>(p.d_out) + base;
            const float* const lse2 = p.neg_lse2 + ((int64_t)b * p.H + h) * p.rows_padded;
            const float* const delta = p.neg_delta + ((int64_t)b * p.H + h) * p.rows_padded;

            auto dma_both = [&](int i0, unsigned char* dst_q, unsigned char* dst_o, unsigned char* dst_s) {
                // (a tile that starts at or behind the end of the sequence touches no memory and lands as zeros)
                const int64_t rem = i0 < L ? (int64_t)(L - i0 - 1) * sn * 2 + 2 * d_real : 0;
                const unsigned nrec = rem > 0xffffffffll ? 0xffffffffu : (unsigned)rem;
                dma_tile<D>(gq + (int64_t)i0 * sn, nrec, dma_off, dst_q, wave_u);
                dma_tile<D>(gdo + (int64_t)i0 * sn, nrec, dma_off, dst_o, wave_u);
                // the statistics arrays are padded to whole 128-row tiles: 64 rows from i0 < L on always exist
                if (wave_u == 0) {
                    const unsigned nst = i0 < L ? 256u : 0u;
                    dma_dword(lse2 + i0, nst, 4 * lane, dst_s);
                    dma_dword(delta + i0, nst, 4 * lane, dst_s + 256);
                }
            };
            // (the tiles behind the first: addresses and remaining bytes advance by a tile per request, as in the dQ kernel)
            const int64_t tile_elems = (int64_t)kFlashKeys * sn;
            int64_t off_next = (int64_t)(t_begin + 1) * tile_elems;  // (an element count: Q and dO share it)
            int64_t rem_next = (int64_t)(L - (t_begin + 1) * kFlashKeys - 1) * sn * 2 + 2 * d_real;
            auto dma_next = [&](int i0, unsigned char* dst_q, unsigned char* dst_o, unsigned char* dst_s) {
                const unsigned nrec = rem_next <= 0 ? 0u : rem_next > 0xffffffffll ? 0xffffffffu : (unsigned)rem_next;
                dma_tile<D>(gq + off_next, nrec, dma_off, dst_q, wave_u);
                dma_tile<D>(gdo + off_next, nrec, dma_off, dst_o, wave_u);
                if (wave_u == 0) {
                    const unsigned nst = rem_next > 0 ? 256u : 0u;
                    dma_dword(lse2 + i0, nst, 4 * lane, dst_s);
                    dma_dword(delta + i0, nst, 4 * lane, dst_s + 256);
                }
                off_next += tile_elems;
                rem_next -= 2 * tile_elems;
            };

            auto compute_tile = [&](const unsigned char* tile_q, const unsigned char* tile_o, const unsigned char* tile_s, int i0,
                                    uint64_t mw) {
                if constexpr (PART == 0 && !MASKED) {
                    // Both blocks of 32 queries in full (no end of the sequence, no diagonal in either), which is almost
                    // every tile of a long sequence.  This kernel runs one wavefront per SIMD, so nobody else fills the
                    // matrix pipe while a block's exponentials and products P.dP run (some 100 vector instructions
                    // between 16 + 16 matrix instructions).  The two blocks are therefore laid out as a pipeline:
                    //     first products (S, dP) of block 0
                    //     first products of block 1   among   the exponentials of block 0
                    //     second products (dV, dK) of block 0   among   the exponentials of block 1
                    //     second products of block 1
                    // (the same arithmetic in the same order per element: results are bit for bit those of the loop below).
                    if (i0 + 63 < L && kw + 31 < L && (!CAUSAL || i0 >= kw + 31)) {
                        f32x16 s0, dp0, s1, dp1;
#pragma unroll
                        for (int g4 = 0; g4 < 4; ++g4) {
                            const f32x4 a0 = *reinterpret_cast<const f32x4*>(tile_s + 4 * (8 * g4 + 4 * half));
                            const f32x4 d0 = *reinterpret_cast<const f32x4*>(tile_s + 256 + 4 * (8 * g4 + 4 * half));
                            const f32x4 a1 = *reinterpret_cast<const f32x4*>(tile_s + 4 * (32 + 8 * g4 + 4 * half));
                            const f32x4 d1 = *reinterpret_cast<const f32x4*>(tile_s + 256 + 4 * (32 + 8 * g4 + 4 * half));
#pragma unroll
                            for (int x = 0; x < 4; ++x) {
                                s0[4 * g4 + x] = a0[x];
                                dp0[4 * g4 + x] = d0[x];
                                s1[4 * g4 + x] = a1[x];
                                dp1[4 * g4 + x] = d1[x];
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                        __builtin_amdgcn_s_setprio(1);
                        u32x2 ot[2][MB][2], qt[2][MB][2];
                        auto request_tr = [&](int row0, int g2) __attribute__((always_inline)) {
#pragma unroll
                            for (int mb = 0; mb < MB; ++mb) {
                                ot[g2][mb][0] = TrRead<T>::load(tile_o + row0 * RB + tr_off[mb][0]);
                                ot[g2][mb][1] = TrRead<T>::load(tile_o + row0 * RB + tr_off[mb][1]);
                                qt[g2][mb][0] = TrRead<T>::load(tile_q + row0 * RB + tr_off[mb][0]);
                                qt[g2][mb][1] = TrRead<T>::load(tile_q + row0 * RB + tr_off[mb][1]);
                            }
                        };
                        auto second_products = [&](int row0, const f32x16& pw, const f32x16& ds) __attribute__((always_inline)) {
#pragma unroll
                            for (int g2 = 0; g2 < 2; ++g2) {
                                if (g2 == 0) request_tr(row0 + 16, 1);
                                const u32x4 bp = pack_operand<T>(pw, 8 * g2);
#pragma unroll
                                for (int mb = 0; mb < MB; ++mb)
                                    acc_v[mb] = mfma_32x32x16<T>(u32x4{ot[g2][mb][0][0], ot[g2][mb][0][1], ot[g2][mb][1][0], ot[g2][mb][1][1]}, bp, acc_v[mb]);
                                const u32x4 bs = pack_operand<T>(ds, 8 * g2);
#pragma unroll
                                for (int mb = 0; mb < MB; ++mb)
                                    acc_k[mb] = mfma_32x32x16<T>(u32x4{qt[g2][mb][0][0], qt[g2][mb][0][1], qt[g2][mb][1][0], qt[g2][mb][1][1]}, bs, acc_k[mb]);
                                __builtin_amdgcn_sched_barrier(0);
                            }
                        };
                        constexpr int kAhead = 2;  // (3 and 4 steps ahead time the same)
                        request_tr(0, 0);
                        {   // first products of block 0
                            u32x4 aq[KS], ao[KS];
#pragma unroll
                            for (int ks = 0; ks < KS; ++ks) {
                                aq[ks] = lds_read_b128(tile_q + row_off[ks]);
                                ao[ks] = lds_read_b128(tile_o + row_off[ks]);
                            }
#pragma unroll
                            for (int ks = 0; ks < KS; ++ks) {
                                s0 = mfma_32x32x16<T>(aq[ks], kreg[ks], s0);
                                dp0 = mfma_32x32x16<T>(ao[ks], vreg[ks], dp0);
                            }
                            __builtin_amdgcn_sched_group_barrier(0x100, 4 * MB + 2 * kAhead, 0);
#pragma unroll
                            for (int i = 0; i < KS - kAhead; ++i) {
                                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                            }
#pragma unroll
                            for (int i = 0; i < kAhead; ++i) __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                        f32x16 pw0, ds0;
                        {   // first products of block 1 among the exponentials of block 0
                            u32x4 aq[KS], ao[KS];
#pragma unroll
                            for (int ks = 0; ks < KS; ++ks) {
                                aq[ks] = lds_read_b128(tile_q + 32 * RB + row_off[ks]);
                                ao[ks] = lds_read_b128(tile_o + 32 * RB + row_off[ks]);
                            }
#pragma unroll
                            for (int ks = 0; ks < KS; ++ks) {
                                s1 = mfma_32x32x16<T>(aq[ks], kreg[ks], s1);
                                dp1 = mfma_32x32x16<T>(ao[ks], vreg[ks], dp1);
                            }
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                pw0[r] = fast_exp2(s0[r]);
                                ds0[r] = pw0[r] * dp0[r];
                            }
                            __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
                            for (int i = 0; i < KS - kAhead; ++i) {
                                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                                __builtin_amdgcn_sched_group_barrier(0x402, 32 / KS, 0);
                            }
#pragma unroll
                            for (int i = 0; i < kAhead; ++i) {
                                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                                __builtin_amdgcn_sched_group_barrier(0x402, 32 / KS, 0);
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                        // second products of block 0 among the exponentials of block 1
                        f32x16 pw1, ds1;
#pragma unroll
                        for (int g2 = 0; g2 < 2; ++g2) {
                            if (g2 == 0) request_tr(16, 1);
                            const u32x4 bp = pack_operand<T>(pw0, 8 * g2);
#pragma unroll
                            for (int mb = 0; mb < MB; ++mb)
                                acc_v[mb] = mfma_32x32x16<T>(u32x4{ot[g2][mb][0][0], ot[g2][mb][0][1], ot[g2][mb][1][0], ot[g2][mb][1][1]}, bp, acc_v[mb]);
                            const u32x4 bs = pack_operand<T>(ds0, 8 * g2);
#pragma unroll
                            for (int mb = 0; mb < MB; ++mb)
                                acc_k[mb] = mfma_32x32x16<T>(u32x4{qt[g2][mb][0][0], qt[g2][mb][0][1], qt[g2][mb][1][0], qt[g2][mb][1][1]}, bs, acc_k[mb]);
#pragma unroll
                            for (int r = 8 * g2; r < 8 * g2 + 8; ++r) {
                                pw1[r] = fast_exp2(s1[r]);
                                ds1[r] = pw1[r] * dp1[r];
                            }
                            if (g2 == 1) request_tr(32, 0);  // block 1's first 16 queries (the registers of block 0's are free)
                            __builtin_amdgcn_sched_group_barrier(0x402, 4, 0);
#pragma unroll
                            for (int i = 0; i < 2 * MB; ++i) {
                                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                                __builtin_amdgcn_sched_group_barrier(0x100, 4 * MB / (2 * MB), 0);
                                __builtin_amdgcn_sched_group_barrier(0x402, 5, 0);
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
                        second_products(32, pw1, ds1);
                        __builtin_amdgcn_s_setprio(0);
                        return;
                    }
                }
#pragma unroll
                for (int ib = 0; ib < 2; ++ib) {
                    const int iblock0 = i0 + 32 * ib;
                    if (iblock0 >= L) continue;                      // nothing but padding
                    if (CAUSAL && iblock0 + 31 < kw) continue;      // every query of the block precedes the keys
                    // the block's rows of statistics: this lane's 16 rows are 4 runs of 4 consecutive rows
                    f32x16 s, dp;
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        const f32x4 a = *reinterpret_cast<const f32x4*>(tile_s + 4 * (32 * ib + 8 * g4 + 4 * half));
#pragma unroll
                        for (int x = 0; x < 4; ++x) s[4 * g4 + x] = a[x];
                        if constexpr (kDoK) {
                            const f32x4 d0 = *reinterpret_cast<const f32x4*>(tile_s + 256 + 4 * (32 * ib + 8 * g4 + 4 * half));
#pragma unroll
                            for (int x = 0; x < 4; ++x) dp[4 * g4 + x] = d0[x];
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);  // (the statistics reads stay out of the pipeline laid out below)
                    __builtin_amdgcn_s_setprio(1);
                    // transposed operands of the block's first 16 queries: requested now, they arrive while the first
                    // products run
                    u32x2 ot[2][MB][2], qt[2][MB][2];
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        if constexpr (kDoV) {
                            ot[0][mb][0] = TrRead<T>::load(tile_o + (32 * ib) * RB + tr_off[mb][0]);
                            ot[0][mb][1] = TrRead<T>::load(tile_o + (32 * ib) * RB + tr_off[mb][1]);
                        }
                        if constexpr (kDoK) {
                            qt[0][mb][0] = TrRead<T>::load(tile_q + (32 * ib) * RB + tr_off[mb][0]);
                            qt[0][mb][1] = TrRead<T>::load(tile_q + (32 * ib) * RB + tr_off[mb][1]);
                        }
                    }
                    {
                        // the operands of the first products are requested kAhead steps ahead of the matrix
                        // instructions that use them
                        constexpr int kPer = kDoK ? 2 : 1;  // products (and operand reads) per step
                        constexpr int kAhead = 2;
                        u32x4 aq[KS], ao[KS];
#pragma unroll
                        for (int ks = 0; ks < KS; ++ks) {
                            aq[ks] = lds_read_b128(tile_q + 32 * ib * RB + row_off[ks]);
                            if constexpr (kDoK) ao[ks] = lds_read_b128(tile_o + 32 * ib * RB + row_off[ks]);
                        }
#pragma unroll
                        for (int ks = 0; ks < KS; ++ks) {
                            s = mfma_32x32x16<T>(aq[ks], kreg[ks], s);
                            if constexpr (kDoK) dp = mfma_32x32x16<T>(ao[ks], vreg[ks], dp);
                        }
                        __builtin_amdgcn_sched_group_barrier(0x100, 2 * MB * (kDoK && kDoV ? 2 : 1) + kPer * kAhead, 0);  // LDS reads
#pragma unroll
                        for (int i = 0; i < KS - kAhead; ++i) {
                            __builtin_amdgcn_sched_group_barrier(0x008, kPer, 0);  // matrix instructions
                            __builtin_amdgcn_sched_group_barrier(0x100, kPer, 0);
                        }
#pragma unroll
                        for (int i = 0; i < kAhead; ++i) __builtin_amdgcn_sched_group_barrier(0x008, kPer, 0);
                    }
                    // query = iblock0 + 4*half + 8*(r/4) + r%4 contributes iff it exists, the key exists, and
                    // (causal) query >= key
                    __builtin_amdgcn_s_setprio(0);
                    f32x16 pw, ds;
                    // the per-element tests are needed only where the block meets the diagonal or an end of the sequence
                    // (uniform per wavefront): everywhere else every (query, key) pair of the block counts
                    const bool all_on = !MASKED && iblock0 + 31 < L && kw + 31 < L && (!CAUSAL || iblock0 >= kw + 31);
                    if (all_on) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            pw[r] = fast_exp2(s[r]);
                            if constexpr (kDoK) ds[r] = pw[r] * dp[r];
                        }
                    } else {
                        int first = 0;
                        if (CAUSAL) first = key - (iblock0 + 4 * half);
                        const int last = (key < L ? L : 0) - (iblock0 + 4 * half);  // off < last
                        // the lane's queries of the block as bits 0.. of one word: query iblock0 + 4*half + off <-> bit off
                        const uint32_t bits = MASKED ? (uint32_t)(mw >> (32 * ib)) >> (4 * half) : 0xFFFFFFFFu;
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int off = 8 * (r >> 2) + (r & 3);
                            const bool on = off >= first && off < last && (!MASKED || ((bits >> off) & 1u));
                            pw[r] = on ? fast_exp2(s[r]) : 0.0f;
                            if constexpr (kDoK) ds[r] = on ? pw[r] * dp[r] : 0.0f;
                        }
                    }
                    __builtin_amdgcn_s_setprio(1);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int g2 = 0; g2 < 2; ++g2) {
                        if (g2 == 0) {
                            // the second 16 queries' operands travel while the first 16 are multiplied
#pragma unroll
                            for (int mb = 0; mb < MB; ++mb) {
                                if constexpr (kDoV) {
                                    ot[1][mb][0] = TrRead<T>::load(tile_o + (32 * ib + 16) * RB + tr_off[mb][0]);
                                    ot[1][mb][1] = TrRead<T>::load(tile_o + (32 * ib + 16) * RB + tr_off[mb][1]);
                                }
                                if constexpr (kDoK) {
                                    qt[1][mb][0] = TrRead<T>::load(tile_q + (32 * ib + 16) * RB + tr_off[mb][0]);
                                    qt[1][mb][1] = TrRead<T>::load(tile_q + (32 * ib + 16) * RB + tr_off[mb][1]);
                                }
                            }
                        }
                        if constexpr (kDoV) {
                            const u32x4 bp = pack_operand<T>(pw, 8 * g2);
#pragma unroll
                            for (int mb = 0; mb < MB; ++mb)
                                acc_v[mb] = mfma_32x32x16<T>(u32x4{ot[g2][mb][0][0], ot[g2][mb][0][1], ot[g2][mb][1][0], ot[g2][mb][1][1]}, bp, acc_v[mb]);
                        }
                        if constexpr (kDoK) {
                            const u32x4 bs = pack_operand<T>(ds, 8 * g2);
#pragma unroll
                            for (int mb = 0; mb < MB; ++mb)
                                acc_k[mb] = mfma_32x32x16<T>(u32x4{qt[g2][mb][0][0], qt[g2][mb][0][1], qt[g2][mb][1][0], qt[g2][mb][1][1]}, bs, acc_k[mb]);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    __builtin_amdgcn_s_setprio(0);
                }
            };

            auto step = [&](unsigned char* cur_q, unsigned char* cur_o, unsigned char* cur_s, unsigned char* nxt_q, unsigned char* nxt_o,
                            unsigned char* nxt_s, int t) {
                const int i0 = t * kFlashKeys;
                const bool more = t + 1 < n_tiles;
                uint64_t mw = 0;
                if constexpr (MASKED) {
                    mw = mword[(int64_t)t * p.N];  // (in front of the tile requests, see the dQ kernel)
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (more) dma_next(i0 + kFlashKeys, nxt_q, nxt_o, nxt_s);
                compute_tile(cur_q, cur_o, cur_s, i0, mw);
                if (more) {
                    __builtin_amdgcn_s_waitcnt(0);
                    __syncthreads();
                }
            };

            dma_both(t_begin * kFlashKeys, lds_q0, lds_o0, lds_s0);
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            for (int t = t_begin; t < n_tiles; t += 2) {
                step(lds_q0, lds_o0, lds_s0, lds_q1, lds_o1, lds_s1, t);
                if (t + 1 < n_tiles) step(lds_q1, lds_o1, lds_s1, lds_q0, lds_o0, lds_s0, t + 1);
            }
            __syncthreads();  // the next head's first load reuses the buffers
        }
        if (key < L) {
            if constexpr (kDoK) store_row<T, MB>(static_cast<T*>(p.d_k) + kv_base + (int64_t)key * skv, acc_k, half, p.scale, d_real);
            if constexpr (kDoV) store_row<T, MB>(static_cast<T*>(p.d_v) + kv_base + (int64_t)key * skv, acc_v, half, 1.0f, d_real);
        }
    }
}

}  // namespace ahpc
