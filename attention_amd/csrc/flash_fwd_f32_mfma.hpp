// FlashAttention forward for fp32 tensors on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32: fp32 operands, fp32
// products and sums, so the result keeps the fp32 kernel's accuracy).  fp32 is the reference's default data type
// (DataType::FLOAT32, src/api/attention_interface.hpp:13-19; every case of tests/test_flash_attention.cpp uses it);
// the block it replaces is FlashAttention::compute_attention_block, src/algorithms/flash_attention.cpp:277-350.
//
// Same formulation as the 16-bit kernel (flash_fwd_mfma.hpp): a workgroup of four wavefronts owns 128 query rows,
// a wavefront 32 of them as the COLUMNS of its products, and walks the keys 32 at a time:
//     S^T = K Q^T - m     A = K rows from LDS, B = Q^T from registers (pre-multiplied by scale*log2(e)),
//                         C = -m, the query's reference maximum (lazy, as in the 16-bit kernel)
//     P^T = exp2(S^T)     in the registers S^T arrived in: they ARE the B operand of the next product
//     O^T += V^T P^T      A = V^T: a lane reads one float of a V row per instruction
// A matrix instruction contracts over two values, one per half of the wavefront.  Which two is free as long as A
// and B agree, and both products choose them so that operands need no shuffling:
//   * first product, step 4m+e (m < d/8, e < 4): half h contracts d = 8m + 4h + e.  A lane's four consecutive
//     floats of a K row (one 16-byte LDS read) and of its Q row (one register quad) feed four steps.
//   * second product, step 4g+e: half h contracts key 8g + 4h + e of the tile, which is exactly the key that
//     result register 4g+e of the first product holds for that lane.
// The instruction takes 64 cycles for 4096 FLOP (157 TFLOP/s on the chip), an eighth of the 16-bit rate: next to
// it LDS traffic, the softmax arithmetic and the tile requests are small, so the kernel is as plain as it can be:
// tiles of 32 keys through direct-to-LDS loads into two stages, one barrier per tile, two workgroups per CU.
//
// LDS layout: a tile is 32 rows of d floats; 16-byte chunk c of row r sits at chunk c ^ f(r) (the load writes LDS
// linearly, so the swizzle is applied to the global address a lane fetches):
//   K: f = r % chunks-per-row, so the 16 lanes of a 16-byte read phase (16 rows, same logical chunk) hit 16
//      different chunks;
//   V: f = 8 * ((r / 4) % 2): the two halves of a 4-byte read (rows 4 apart, same 32 floats) hit different banks.
#pragma once

#include "flash_fwd_mfma.hpp"

namespace ahpc {

constexpr int kF32Keys = 32;  // keys per tile

__device__ inline f32x16 mfma_32x32x2_f32(float a, float b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// Work map and launch plan are the 16-bit kernel's (flash_work_of_block, flash_plan_launch): a head's tiles side by side on
// one XCD, long tiles first, causal launches with a late and an early query tile per workgroup.
// MASKED: a dense mask [B,N,N] in its packed form (FlashParams::mask_bits, see flash_fwd_mfma.hpp: one 64-bit word per
// query and 64 keys) removes keys per query; the reference maximum is then set per query when its first key shows up.
// STATS: the first step of the backward.  The output stays in registers; per query row the kernel writes what
// FlashStatsOut describes (flash_fwd_mfma.hpp): -lse2 and -(dO . O), padding rows -inf and 0.
template <int D, bool CAUSAL, bool VARLEN, bool MASKED, bool STATS>
__device__ __forceinline__ void flash_fwd_f32_mfma_body(const FlashParams& p, const FlashStatsOut& st) {
    static_assert(D == 64 || D == 128 || D == 256, "head dimensions of the fp32 matrix-core kernel");
    static_assert(!(MASKED && (VARLEN || STATS)), "the mask belongs to dense forward launches");
    constexpr int RB = 4 * D;                 // row bytes
    constexpr int CH = D / 4;                 // 16-byte chunks per row
    constexpr int RPI = 1024 / RB;            // rows one load instruction covers
    constexpr int IPW = kF32Keys / RPI / 4;   // load instructions per wavefront and tile (K or V)
    constexpr int MS = D / 8;                 // 16-byte K reads (= register quads of Q) per lane
    constexpr int MB = D / 32;                // 32-row blocks of O^T
    constexpr int kTileBytes = kF32Keys * RB;

    __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[kTileBytes];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 31;   // query column / operand row owned by this lane
    const int half = lane >> 5;
    const FlashWork work = flash_work_of_block(blockIdx.x, p);
    if (!work.valid) return;
    // whatever the map says, nothing outside the tensors is ever addressed (uniform per workgroup)
    if (work.bh < 0 || work.bh >= p.n_bh || work.slot < 0 || work.slot >= flash_per_head(p)) return;
    const int slot = work.slot;
    const int b = work.bh / p.H;
    const int h = work.bh - b * p.H;
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
    // query tiles of this sequence, and the slots they fill (a ragged batch hands every sequence as many slots as the
    // longest one needs: the surplus exits here, before anything is requested)
    const int n_q = VARLEN ? (L + kFlashRows - 1) / kFlashRows : p.n_qtiles;
    if (VARLEN && slot >= (p.paired ? (n_q + 1) >> 1 : n_q)) return;
    const float* const gq = static_cast<const float*>(p.q) + base;
    const float* const gk = static_cast<const float*>(p.k) + kv_base;
    const float* const gv = static_cast<const float*>(p.v) + kv_base;
    float* const go = STATS ? nullptr : static_cast<float*>(p.o) + base;  // the statistics pass has no output tensor
    const int64_t sn = p.stride_n;
    const int64_t skv = p.kv_stride_n;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int d_real = (p.d_real > 0 && p.d_real < D) ? p.d_real : D;

    auto fk = [](int r) { return r & (CH - 1); };
    auto fv = [](int r) { return 8 * ((r >> 2) & 1); };  // exchanges the 128-byte blocks 2j and 2j + 1 of a row

    // ---- tile requests: lane's 16 bytes of instruction j land at tile + 1024 j + 16 lane = row RPI j + lane / CH,
    //      chunk lane % CH; the global side picks the chunk that belongs there
    int dma_off_k[IPW], dma_off_v[IPW];
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
        const int r = (wave * IPW + i) * RPI + lane / CH;
        const int pc = lane % CH;
        const int ck = pc ^ fk(r), cv = pc ^ fv(r);  // the 4-float chunk of the row that belongs at this lane's place
        // a head dimension below D (FlashParams::d_real): columns from d_real on fetch the row's first chunk again
        dma_off_k[i] = (int)(r * skv * 4) + ((4 * ck < d_real ? ck : 0) << 4);
        dma_off_v[i] = (int)(r * skv * 4) + ((4 * cv < d_real ? cv : 0) << 4);
    }
    // Bytes from the tile's first row to the end of the sequence's last row bound the descriptor: rows of a ragged last
    // tile that do not exist read as zeros (their scores are masked; zero V rows keep 0 * x finite).
    auto dma_both = [&](int k0, unsigned char* dst_k, unsigned char* dst_v) {
        const int64_t rem = k0 < L ? (int64_t)(L - k0 - 1) * skv * 4 + 4 * d_real : 0;  // the last row ends with its own d
        const unsigned nrec = rem > 0xffffffffll ? 0xffffffffu : (unsigned)rem;
#pragma unroll
        for (int i = 0; i < IPW; ++i) {
            dma_instr(gk + (int64_t)k0 * skv, nrec, dma_off_k[i], dst_k + (wave_u * IPW + i) * 1024);
            dma_instr(gv + (int64_t)k0 * skv, nrec, dma_off_v[i], dst_v + (wave_u * IPW + i) * 1024);
        }
    };

    // ---- operand addresses inside a tile
    int k_off[MS];   // K: row col, logical chunk 2m + half
#pragma unroll
    for (int m = 0; m < MS; ++m) k_off[m] = col * RB + (((2 * m + half) ^ fk(col)) << 4);
    // V: the float at (key, 32 mb + col) sits 128 mb + 4 col bytes into its row; the swizzle of a key that half 1 reads
    // (keys 8g + 4 + e) flips bit 3 of the chunk index, i.e. exchanges the 128-byte blocks mb and mb ^ 1, and the keys
    // half 0 reads are not swizzled.  So a lane reads block mb ^ half of row key0 + 4 half.
    const int v_even = 4 * half * RB + half * 128 + 4 * col;        // blocks 0, 2 of the lane's row, relative to key0's
    const int v_odd = 4 * half * RB + (1 - half) * 128 + 4 * col;   // blocks 1, 3

    for (int part = 0; part < 2; ++part) {
        const int qt = flash_qtile_of_part(p, n_q, slot, part);
        if (qt < 0) break;
        const int q_tile0 = qt * kFlashRows;
        if (part == 1) __syncthreads();  // every wavefront is done with the first pass's last tile
        // ---- Q^T as B operands: quad m holds d = 8m + 4 half .. + 3 of this lane's query, pre-scaled
        const int qw = q_tile0 + wave * 32;
        const int qrow = qw + col;
        f32x4 qreg[MS];
        {
            const float c = p.scale_log2;
            const float* src = gq + (int64_t)(qrow < L ? qrow : L - 1) * sn + 4 * half;
#pragma unroll
            for (int m = 0; m < MS; ++m) {
                const f32x4 raw = 8 * m + 4 * half < d_real ? *reinterpret_cast<const f32x4*>(src + 8 * m) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                qreg[m] = f32x4{raw[0] * c, raw[1] * c, raw[2] * c, raw[3] * c};
            }
        }

        f32x16 oacc[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[mb][r] = 0.0f;
        f32x16 neg_m;
#pragma unroll
        for (int r = 0; r < 16; ++r) neg_m[r] = 0.0f;
        float l_run = 0.0f;
        bool first = true;
        bool seen = false;  // masked launches: this lane's query has met a key it may attend to
        constexpr float kRaise = 8.0f;  // raise the reference maximum only when exceeded by 2^8
        const uint64_t* const mword = MASKED ? p.mask_bits + (int64_t)b * p.mask_kt * p.N + (qrow < L ? qrow : L - 1) : nullptr;

        int k_end = L;
        if (CAUSAL) k_end = (q_tile0 + kFlashRows) < L ? (q_tile0 + kFlashRows) : L;
        const int n_tiles = (k_end + kF32Keys - 1) / kF32Keys;

        auto compute_tile = [&](const unsigned char* tile_k, const unsigned char* tile_v, int k0, uint64_t mw) {
            // ---- S^T = c K Q^T - m in two chains (even and odd quads) so that consecutive matrix instructions are independent
            f32x16 s, s_odd;
            __builtin_amdgcn_s_setprio(1);
            {
                u32x4 kq[MS];
#pragma unroll
                for (int m = 0; m < MS; ++m) kq[m] = lds_read_b128(tile_k + k_off[m]);
#pragma unroll
                for (int r = 0; r < 16; ++r) s_odd[r] = 0.0f;
                s = neg_m;
#pragma unroll
                for (int m = 0; m < MS; m += 2)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        s = mfma_32x32x2_f32(as_f32(kq[m][e]), qreg[m][e], s);
                        s_odd = mfma_32x32x2_f32(as_f32(kq[m + 1][e]), qreg[m + 1][e], s_odd);
                    }
                // two pairs of K quads are requested before the first product, one more pair behind every eight products
                __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);  // LDS reads
#pragma unroll
                for (int i = 0; i < MS / 2 - 2; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);  // matrix instructions
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, 16, 0);
            }
            __builtin_amdgcn_s_setprio(0);
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] += s_odd[r];
            // key of register r: k0 + 8 (r / 4) + 4 half + r % 4; visible iff key <= min(qrow, L - 1)
            const bool need_mask = (k0 + kF32Keys > L) || (CAUSAL && (k0 + kF32Keys - 1 > qw));
            if (need_mask) {
                int lim = L - 1;
                if (CAUSAL) lim = qrow < lim ? qrow : lim;
                lim -= k0 + 4 * half;
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = (8 * (r >> 2) + (r & 3)) <= lim ? s[r] : -INFINITY;
            }
            if constexpr (MASKED) {
                // the word holds 64 keys, the tile is its lower or upper half; the lane's keys are 4 half + 8 (r / 4) + r % 4
                const uint32_t word = (uint32_t)(mw >> ((k0 & 32) + 4 * half));
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int pos = 8 * (r >> 2) + (r & 3);
                    const uint32_t keep = (uint32_t)((int32_t)(word << (31 - pos)) >> 31);
                    s[r] = as_f32((as_u32(s[r]) & keep) | (0xFF800000u & ~keep));
                }
            }
            float mx = s[0];
#pragma unroll
            for (int r = 1; r < 16; r += 2) mx = r + 1 < 16 ? max3(mx, s[r], s[r + 1]) : max3(mx, s[r], s[r]);
            bool adjust;
            if constexpr (MASKED) adjust = __builtin_amdgcn_ballot_w64(seen ? mx > kRaise : mx > -INFINITY) != 0;
            else adjust = first || __builtin_amdgcn_ballot_w64(mx > kRaise) != 0;
            if (adjust) {
                mx = halves_max(mx);  // both lanes of a query agree
                float delta, alpha;
                if constexpr (MASKED) {
                    // a query without a visible key so far has accumulated nothing: its maximum is set exactly, nothing
                    // is rescaled; one that still sees none stays as it is
                    delta = seen ? fmaxf(mx, 0.0f) : (mx > -INFINITY ? mx : 0.0f);
                    alpha = seen ? fast_exp2(-delta) : 1.0f;
                    seen = seen || mx > -INFINITY;
                } else {
                    delta = first ? mx : fmaxf(mx, 0.0f);
                    alpha = fast_exp2(-delta);
                }
                l_run *= alpha;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[mb][r] *= alpha;
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] -= delta;
                const float nm = neg_m[0] - delta;
#pragma unroll
                for (int r = 0; r < 16; ++r) neg_m[r] = nm;
                first = false;
            }
            float sum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                s[r] = fast_exp2(s[r]);
                sum += s[r];
            }
            l_run += sum;
            // ---- O^T += V^T P^T: step r = 4g + e contracts keys 8g + e (half 0) and 8g + 4 + e (half 1)
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const unsigned char* row = tile_v + (8 * (r >> 2) + (r & 3)) * RB;  // key0; half 1 reads 4 rows further down
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const float a = *reinterpret_cast<const float*>(row + ((mb & 1) ? v_odd : v_even) + (mb >> 1) * 256);
                    oacc[mb] = mfma_32x32x2_f32(a, s[r], oacc[mb]);
                }
            }
            __builtin_amdgcn_s_setprio(0);
        };

        auto step = [&](unsigned char* cur_k, unsigned char* cur_v, unsigned char* nxt_k, unsigned char* nxt_v, int t) {
            const int k0 = t * kF32Keys;
            const bool more = t + 1 < n_tiles;
            uint64_t mw = 0;
            if constexpr (MASKED) {
                // The mask word is requested BEFORE the next tile (loads complete in order), and the tile is requested
                // even behind the last one (an empty request), so that the same loads are in flight on every path.
                mw = mword[(int64_t)(k0 >> 6) * p.N];
                __builtin_amdgcn_sched_barrier(0);
                dma_both(k0 + kF32Keys, nxt_k, nxt_v);
            } else {
                if (more) dma_both(k0 + kF32Keys, nxt_k, nxt_v);
            }
            // a wavefront whose queries all precede this tile has nothing to add
            if (!(CAUSAL && k0 > qw + 31)) compute_tile(cur_k, cur_v, k0, mw);
            if (MASKED || more) {
                __builtin_amdgcn_s_waitcnt(0);  // this wavefront's part of the next tile has landed
                __syncthreads();                // everyone's has, and everyone is done with the current one
            }
        };

        dma_both(0, lds_k0, lds_v0);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        for (int t = 0; t < n_tiles; t += 2) {
            step(lds_k0, lds_v0, lds_k1, lds_v1, t);
            if (t + 1 < n_tiles) step(lds_k1, lds_v1, lds_k0, lds_v0, t + 1);
        }

        // ---- normalise and store: per 32-row block a lane holds 4 runs of 4 consecutive d of its query
        const float l = halves_sum(l_run);
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        if constexpr (STATS) {
            // delta = dO . O over the elements this lane holds, then over the two lanes of the query
            float part = 0.0f;
            if (qrow < L) {
                const float* src = static_cast<const float*>(st.d_out) + base + (int64_t)qrow * sn + 4 * half;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        if (32 * mb + 8 * g4 + 4 * half >= d_real) continue;  // columns the tensors do not have
                        const f32x4 w = *reinterpret_cast<const f32x4*>(src + 32 * mb + 8 * g4);
                        part += oacc[mb][4 * g4] * w[0] + oacc[mb][4 * g4 + 1] * w[1] + oacc[mb][4 * g4 + 2] * w[2] +
                                oacc[mb][4 * g4 + 3] * w[3];
                    }
            }
            const float delta = halves_sum(part) * inv;
            if (half == 0) {  // every row of the 128-row tile gets a value: the statistics arrays are padded to whole tiles
                const int64_t row = (int64_t)work.bh * st.rows_padded + qrow;
                const bool live = qrow < L && l > 0.0f;
                st.neg_lse2[row] = live ? neg_m[0] - __builtin_log2f(l) : -INFINITY;
                st.neg_delta[row] = live ? -delta : 0.0f;
            }
        } else if (qrow < L) {
            float* dst = go + (int64_t)qrow * sn + 4 * half;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4)
                    if (32 * mb + 8 * g4 + 4 * half < d_real)
                        *reinterpret_cast<f32x4*>(dst + 32 * mb + 8 * g4) =
                            f32x4{oacc[mb][4 * g4] * inv, oacc[mb][4 * g4 + 1] * inv, oacc[mb][4 * g4 + 2] * inv, oacc[mb][4 * g4 + 3] * inv};
        }
    }
}

template <int D, bool CAUSAL, bool VARLEN, bool MASKED = false>
__global__ __launch_bounds__(kFlashThreads, D == 256 ? 1 : 2) void flash_fwd_f32_mfma_kernel(const FlashParams p) {
    flash_fwd_f32_mfma_body<D, CAUSAL, VARLEN, MASKED, false>(p, FlashStatsOut{});
}

template <int D, bool CAUSAL, bool VARLEN>
__global__ __launch_bounds__(kFlashThreads, 2) void flash_bwd_stats_f32_mfma_kernel(const FlashParams p, const FlashStatsOut st) {
    flash_fwd_f32_mfma_body<D, CAUSAL, VARLEN, false, true>(p, st);
}

}  // namespace ahpc
