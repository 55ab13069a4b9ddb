// FlashAttention forward, "alternating" variant of flash_fwd_mfma.hpp: one workgroup of 8 wavefronts per CU,
// two groups of four that are always in opposite phases.
//
// Same formulation, tiles, swizzles, operand layouts and data movement as the standard kernel (see
// flash_fwd_mfma.hpp); what changes is who does what when.  A wavefront's work on key tile t is cut into
//     matrix phase M(t)   O^T += V^T P^T for tile t-1, then S^T = K Q^T for tile t   (32 matrix instructions at
//                         d = 128, all operand reads from LDS, no softmax arithmetic)
//     softmax phase S(t)  mask, reference maximum, exp2, packing, row sums for tile t (VALU only)
// and every phase ends in a workgroup barrier.  The second group of wavefronts starts one barrier late, so
// between any two barriers one group is in a matrix phase and the other in a softmax phase: each SIMD holds
// one wavefront of either group, its matrix pipe serves one of them and its VALU the other.  (In the standard
// kernel the two wavefronts of a SIMD belong to different workgroups, nothing keeps them out of step, and
// measured phase times add up rather than overlap; a wavefront doing only matrix work and one doing only
// v_exp_f32 on the same SIMD overlap completely.)
//
// Global step j (the time between barrier j-1 and barrier j), n = number of key tiles:
//     first group   j = 2t: M(t)      j = 2t+1: S(t)      j = 2n: the last O^T += V^T P^T      j = 2n+1: idle
//     second group  j = 0: idle       j = 2t+1: M(t)      j = 2t+2: S(t)                       j = 2n+1: the last one
// Tiles: K(t) is read in steps 2t and 2t+1, V(t) in steps 2t+2 and 2t+3.  Two buffers for K and two for V; at
// the start of every even step 2t all 8 wavefronts request their eighth of K(t+1) (into the buffer K(t-1) left
// in step 2t-1) and of V(t) (into the buffer V(t-2) left in step 2t-1), and they wait for these requests at
// the end of step 2t+1, before the barrier that lets step 2t+2 read them: a tile has two steps (one tile time)
// to arrive.  A 256-row workgroup also halves the tile stream from L2 per FLOP.
//
// Barriers are bare s_barrier instructions between compiler-level memory fences: the usual __syncthreads()
// would make every wavefront wait for its outstanding tile requests at every barrier, which is exactly what the
// even steps must not do.  The kernel has no LDS stores other than the tile requests, whose completion is
// waited for explicitly (s_waitcnt) before the barrier that publishes them.
//
// Which wavefronts form a group: waves w and w+4 of a workgroup are taken to share a SIMD (group = w / 4);
// FlashParams::pingpong_low_bit = 1 pairs w and w^1 instead (group = w % 2).
//
// Selected with AHPC_FLASH_PINGPONG=1 (or 2 for the other pairing); dense and ragged batches; the standard kernel
// stays the default until both have been timed.
#pragma once

#include <type_traits>

#include "flash_fwd_mfma.hpp"

namespace ahpc {

constexpr int kPingPongThreads = 512;
constexpr int kPingPongRows = 256;  // query rows per workgroup

// Workgroup barrier that does not wait for outstanding memory requests of the wavefront.
__device__ inline void bare_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <typename T, int D, bool CAUSAL, bool VARLEN>
__global__ __launch_bounds__(kPingPongThreads, 1) void flash_fwd_pingpong_kernel(const FlashParams p) {
    typedef FlashTile<D> TL;
    constexpr int KS = D / 16;
    constexpr int MB = D / 32;
    constexpr int RB = TL::kRowBytes;
    constexpr int kInstr = kFlashKeys / (8 * TL::kRowsPerInstr);  // tile requests per wavefront and tile (8 wavefronts)

    __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[TL::kBytes];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 31;
    const int half = lane >> 5;

    const FlashWork work = flash_work_of_block(blockIdx.x, p);
    if (!work.valid) return;
    // whatever the map says, nothing outside the tensors is ever addressed (uniform per workgroup)
    if (work.bh < 0 || work.bh >= p.n_bh || work.slot < 0 || work.slot >= flash_per_head(p)) return;
    const int bh = work.bh;
    const int slot = work.slot;
    const int b = bh / p.H;
    const int h = bh - b * p.H;
    const int hk = h / p.kv_group;

    int L;
    int64_t base, kv_base;
    if (VARLEN) {  // packed sequences: this one's tokens start at cu_seqlens[b]
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
    const T* const gk = static_cast<const T*>(p.k) + kv_base;
    const T* const gv = static_cast<const T*>(p.v) + kv_base;
    T* const go = static_cast<T*>(p.o) + base;
    const int64_t sn = p.stride_n;
    const int64_t skv = p.kv_stride_n;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const bool second = (p.pingpong_low_bit ? (wave_u & 1) : (wave_u >> 2)) != 0;  // the group that starts a step late

    // ---- per-lane offsets of the tile requests (bytes from the first row of a tile) ----------------
    int dma_off_k[kInstr], dma_off_v[kInstr];
#pragma unroll
    for (int i = 0; i < kInstr; ++i) {
        const int r = (wave * kInstr + i) * TL::kRowsPerInstr + lane / TL::kChunks;
        const int pc = lane % TL::kChunks;
        dma_off_k[i] = (int)(r * skv * 2) + ((pc ^ TL::fk(r)) << 4);
        dma_off_v[i] = (int)(r * skv * 2) + ((pc ^ TL::fv(r)) << 4);
    }
    // This wavefront's eighth of the 64-key tile that starts at key k0.  Rows past the end of the sequence are
    // out of range for the descriptor and arrive as zeros.
    auto request = [&](const T* g, const int* off, int k0, unsigned char* dst) __attribute__((always_inline)) {
        const int64_t rem = (int64_t)(L - k0 - 1) * skv * 2 + 2 * D;
        const unsigned nrec = rem > 0xffffffffll ? 0xffffffffu : (unsigned)rem;
#pragma unroll
        for (int i = 0; i < kInstr; ++i) dma_instr(g + (int64_t)k0 * skv, nrec, off[i], dst + (wave_u * kInstr + i) * 1024);
    };

    // ---- LDS operand addresses (byte offsets inside a tile), as in the standard kernel -----------
    int k_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_off[ks] = col * RB + (((2 * ks + half) ^ TL::fk(col)) << 4);
    const int vi = lane & 15;
    const int vkey = 4 * half + (vi >> 2);
    int v_off[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int cch = 4 * mb + 2 * ((lane >> 4) & 1) + ((vi & 3) >> 1);
        v_off[mb] = vkey * RB + ((cch ^ TL::fv(vkey)) << 4) + 8 * (vi & 1);
    }

    for (int part = 0; part < 2; ++part) {
        int qt;
        if (p.paired) {
            if (part == 1 && 2 * slot == p.n_qtiles - 1) break;
            qt = part == 0 ? p.n_qtiles - 1 - slot : slot;
        } else {
            if (part == 1) break;
            qt = p.n_qtiles - 1 - slot;
        }
        const int q_tile0 = qt * kPingPongRows;
        if (q_tile0 >= L) continue;

        int k_end = L;
        if (CAUSAL) k_end = (q_tile0 + kPingPongRows) < L ? (q_tile0 + kPingPongRows) : L;
        const int n_tiles = (k_end + kFlashKeys - 1) / kFlashKeys;

        // The rest of the query tile, compiled once per group: with the group a run-time value in one copy of the
        // loop, the two phase orders meet at every barrier and the register allocator has to reconcile them
        // (it spills); with two copies each is as lean as the standard kernel.
        auto run = [&](auto group) __attribute__((always_inline)) {
        constexpr bool SECOND = decltype(group)::value;

        request(gk, dma_off_k, 0, lds_k0);  // K(0), before anything else

        // ---- Q^T operands, pre-multiplied by c = scale*log2(e) ------------------------------------
        const int qw = q_tile0 + wave_u * 32;  // first query row of this wavefront (a scalar: conditions on it are branches)
        const int qrow = qw + col;
        u32x4 qreg[KS];
        {
            const int row = qrow < L ? qrow : L - 1;
            const T* src = gq + (int64_t)row * sn + 8 * half;
            const float c = p.scale_log2;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const u32x4 raw = *reinterpret_cast<const u32x4*>(src + 16 * ks);
                u32x4 sc;
#pragma unroll
                for (int w = 0; w < 4; ++w) sc[w] = pack2<T>(lo_f32<T>(raw[w]) * c, hi_f32<T>(raw[w]) * c);
                qreg[ks] = sc;
            }
        }

        f32x16 oacc[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[mb][r] = 0.0f;
        float neg_m = 0.0f;  // -(reference maximum) of the lane's query row, log2 units
        float l_run = 0.0f;
        bool first = true;
        constexpr float kRaise = 8.0f;

        f32x16 s[2];   // scores of the current tile: written by the matrix phase, read by the softmax phase
        u32x4 pb[4];   // P^T of the current tile as B operands: written by the softmax phase, read by the next matrix phase

        // a wavefront whose queries all precede a tile has nothing to add to it
        auto active = [&](int t) __attribute__((always_inline)) { return t >= 0 && t < n_tiles && !(CAUSAL && t * kFlashKeys > qw + 31); };

        // ---- S^T = c*K Q^T - m (log2 units) ---------------------------------------------------------
        // The first product's operands are requested in two goes: the first kAhead pairs early (before the second
        // product of the previous tile, whose tail then hides their latency), the rest between the matrix instructions.
        constexpr int kAhead = KS < 4 ? KS : 4;
        auto scores_head = [&](const unsigned char* tile_k, u32x4* h0, u32x4* h1) __attribute__((always_inline)) {
#pragma unroll
            for (int ks = 0; ks < kAhead; ++ks) {
                h0[ks] = lds_read_b128(tile_k + k_off[ks]);
                h1[ks] = lds_read_b128(tile_k + 32 * RB + k_off[ks]);
            }
        };
        auto scores = [&](const unsigned char* tile_k, const u32x4* h0, const u32x4* h1) __attribute__((always_inline)) {
            u32x4 a0[KS], a1[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                a0[ks] = ks < kAhead ? h0[ks] : lds_read_b128(tile_k + k_off[ks]);
                a1[ks] = ks < kAhead ? h1[ks] : lds_read_b128(tile_k + 32 * RB + k_off[ks]);
            }
            // the products start from accumulators holding -m, so that the matrix core delivers c*s - m (the
            // standard kernel keeps a 16-register copy of -m for this; here the registers are worth more)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[0][r] = s[1][r] = neg_m;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                s[0] = mfma_32x32x16<T>(a0[ks], qreg[ks], s[0]);
                s[1] = mfma_32x32x16<T>(a1[ks], qreg[ks], s[1]);
            }
            // two matrix instructions, then the next operand pair's reads, until the reads run out
#pragma unroll
            for (int i = 0; i < KS - kAhead; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // matrix instructions
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // LDS reads
            }
#pragma unroll
            for (int i = 0; i < kAhead; ++i) __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        };

        // ---- O^T += V^T P^T, 16 keys at a time; the operands of group g+1 are requested before the
        //      matrix instructions of group g ------------------------------------------------------
        auto weighted_values = [&](const unsigned char* tile_v) __attribute__((always_inline)) {
            u32x2 vf[2][MB][2];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                vf[0][mb][0] = TrRead<T>::load(tile_v + v_off[mb]);
                vf[0][mb][1] = TrRead<T>::load(tile_v + v_off[mb] + 8 * RB);
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                if (g < 3) {
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        vf[(g + 1) & 1][mb][0] = TrRead<T>::load(tile_v + v_off[mb] + (16 * (g + 1)) * RB);
                        vf[(g + 1) & 1][mb][1] = TrRead<T>::load(tile_v + v_off[mb] + (16 * (g + 1) + 8) * RB);
                    }
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    oacc[mb] = mfma_32x32x16<T>(u32x4{vf[g & 1][mb][0][0], vf[g & 1][mb][0][1], vf[g & 1][mb][1][0], vf[g & 1][mb][1][1]},
                                                pb[g], oacc[mb]);
                __builtin_amdgcn_sched_barrier(0);  // keeps the groups apart: two sets of V operands in registers, not four
            }
        };

        // ---- mask, reference maximum (raised only when topped by 2^8), P^T = exp2(S^T), row sums ------
        auto softmax = [&](int k0) __attribute__((always_inline)) {
            const bool need_mask = (k0 + kFlashKeys > L) || (CAUSAL && (k0 + kFlashKeys - 1 > qw));
            if (need_mask) {
                // key = k0 + 4*half + off(kb, r); visible iff key <= min(qrow, L-1)  <=>  off <= lim
                int lim = L - 1;
                if (CAUSAL) lim = qrow < lim ? qrow : lim;
                lim -= k0 + 4 * half;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int off = 32 * kb + 8 * (r >> 2) + (r & 3);
                        s[kb][r] = off <= lim ? s[kb][r] : -INFINITY;
                    }
            }
            float mx = fmaxf(s[0][0], s[1][0]);
#pragma unroll
            for (int r = 1; r < 16; ++r) mx = fmaxf(mx, fmaxf(s[0][r], s[1][r]));
            if (first || __builtin_amdgcn_ballot_w64(mx > kRaise) != 0) {
                mx = halves_max(mx);
                const float delta = first ? mx : fmaxf(mx, 0.0f);
                const float alpha = fast_exp2(-delta);
                l_run *= alpha;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[mb][r] *= alpha;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) s[kb][r] -= delta;
                neg_m -= delta;
                first = false;
            }
            float sum = 0.0f;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int kb = g >> 1, r0 = 8 * (g & 1);
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const float p0 = fast_exp2(s[kb][r0 + 2 * w]), p1 = fast_exp2(s[kb][r0 + 2 * w + 1]);
                    pb[g][w] = pack2<T>(p0, p1);
                    sum += p0 + p1;
                }
            }
            l_run += sum;
        };

        auto softmax_or_nothing = [&](int t) __attribute__((always_inline)) {
            if (active(t)) {
                softmax(t * kFlashKeys);
            } else {
#pragma unroll
                for (int g = 0; g < 4; ++g) pb[g] = u32x4{0u, 0u, 0u, 0u};  // as for the scores: dead values, said so
            }
        };
        // Tile requests of an even step 2t: K(t+1) and V(t).  (cur, nxt) are the buffers of parity t and t+1.
        auto requests_of_step = [&](int t, unsigned char* k_nxt, unsigned char* v_cur) __attribute__((always_inline)) {
            if (t + 1 < n_tiles) request(gk, dma_off_k, (t + 1) * kFlashKeys, k_nxt);
            if (t < n_tiles) request(gv, dma_off_v, t * kFlashKeys, v_cur);
        };
        // Matrix phase of tile t: the second product of tile t-1 (its V is in the other buffer), the first of tile t.
        auto matrix_phase = [&](int t, const unsigned char* k_cur, const unsigned char* v_prev) __attribute__((always_inline)) {
            // the wavefront that feeds the matrix cores goes first when its SIMD has to choose: the other one's
            // softmax arithmetic fits into the shadow of the matrix instructions
            __builtin_amdgcn_s_setprio(1);
            // the first operands of this tile's first product are requested before the previous tile's second product,
            // whose matrix instructions then hide their latency
            u32x4 h0[kAhead], h1[kAhead];
            const bool act = active(t);
            if (act) scores_head(k_cur, h0, h1);
            if (active(t - 1)) weighted_values(v_prev);
            if (act) {
                scores(k_cur, h0, h1);
            } else {
                // nobody reads these scores; defining them on this path too tells the register allocator that the
                // previous tile's scores are dead by now
#pragma unroll
                for (int r = 0; r < 16; ++r) s[0][r] = s[1][r] = 0.0f;
            }
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(0);
        };

        // One tile of either group.  (k_cur, v_cur): buffers of parity t; (k_nxt, v_nxt): of parity t+1, which
        // also hold K(t-1) / V(t-1) and later K(t+1) / V(t+1).
        auto tile = [&](int t, unsigned char* k_cur, unsigned char* v_cur, unsigned char* k_nxt, unsigned char* v_nxt) __attribute__((always_inline)) {
            if constexpr (!SECOND) {
                requests_of_step(t, k_nxt, v_cur);         // step 2t
                matrix_phase(t, k_cur, v_nxt);
                bare_barrier();
                softmax_or_nothing(t);                      // step 2t+1
                __builtin_amdgcn_s_waitcnt(0);              // K(t+1) and V(t) have landed (this wavefront's share)
                bare_barrier();
            } else {
                matrix_phase(t, k_cur, v_nxt);              // step 2t+1
                __builtin_amdgcn_s_waitcnt(0);              // the requests of step 2t have landed
                bare_barrier();
                requests_of_step(t + 1, k_cur, v_nxt);      // step 2t+2: K(t+2) over K(t), V(t+1) over V(t-1)
                softmax_or_nothing(t);
                bare_barrier();
            }
        };

        __builtin_amdgcn_s_waitcnt(0);
        bare_barrier();                                     // K(0) is there
        if constexpr (SECOND) {
            requests_of_step(0, lds_k1, lds_v0);            // step 0
            bare_barrier();
        }
        for (int t = 0; t < n_tiles; t += 2) {
            tile(t, lds_k0, lds_v0, lds_k1, lds_v1);
            if (t + 1 < n_tiles) tile(t + 1, lds_k1, lds_v1, lds_k0, lds_v0);
        }
        // the second product of the last tile: step 2n for the first group, 2n+1 for the second
        const unsigned char* v_last = ((n_tiles - 1) & 1) ? lds_v1 : lds_v0;
        if constexpr (!SECOND) {
            if (active(n_tiles - 1)) weighted_values(v_last);
            bare_barrier();
        } else {
            if (active(n_tiles - 1)) weighted_values(v_last);
        }
        __builtin_amdgcn_s_waitcnt(0);
        bare_barrier();  // everyone is done with the buffers: the next query tile's requests reuse them

        // ---- normalise and store ------------------------------------------------------------------------
        const float l = halves_sum(l_run);
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        if (qrow < L) {
            T* dst = go + (int64_t)qrow * sn + 4 * half;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const f32x16& a = oacc[mb];
                    const u32x2 w = u32x2{pack2<T>(a[4 * g4 + 0] * inv, a[4 * g4 + 1] * inv),
                                          pack2<T>(a[4 * g4 + 2] * inv, a[4 * g4 + 3] * inv)};
                    *reinterpret_cast<u32x2*>(dst + 32 * mb + 8 * g4) = w;
                }
        }
        };  // run
        if (second) run(std::true_type{});
        else run(std::false_type{});
    }
}

}  // namespace ahpc
