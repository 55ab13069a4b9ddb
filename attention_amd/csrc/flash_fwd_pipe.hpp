// FlashAttention forward on the gfx950 matrix cores, software pipelined inside the wavefront (fp16 / bf16).
//
// Same tiling and layouts as flash_fwd_mfma.hpp (a wavefront owns 32 query columns, S^T = K Q^T, O^T += V^T P^T, lazily
// raised reference maximum, swizzled tiles requested straight into LDS), but the walk over the keys advances 32 keys (a
// "sub-tile") at a time and overlaps the two products with the softmax arithmetic of neighbouring sub-tiles:
//   phase 1 of sub-step u:  S(u+1)^T = K(u+1) Q^T   on the matrix cores  |  exp2 / pack / row sums of the first 16 keys of S(u)
//   phase 2 of sub-step u:  O^T += V(u)^T P(u)^T    on the matrix cores  |  the other 16 keys of S(u), row maximum of S(u+1)
// so a wavefront has matrix instructions to issue nearly all the time: the only stretches without are the mask of a
// diagonal sub-tile and the (rare) rescale.  K is read 32 keys ahead of V, so the K tiles in LDS start 32 keys later than
// the V tiles (K tile p = keys 64p+32 .. 64p+95, V tile p = keys 64p .. 64p+63): one step over a tile pair reads exactly
// one K and one V buffer, and the request / wait / barrier protocol per step is that of flash_fwd_mfma.hpp.
#pragma once

#include "flash_fwd_mfma.hpp"

namespace ahpc {

#define AHPC_INLINE_LAMBDA __attribute__((always_inline))

template <typename T, int D, bool CAUSAL, bool VARLEN, int WAVES>
__device__ __forceinline__ void flash_fwd_pipe_body(const FlashParams& p) {
    typedef FlashTile<D> TL;
    constexpr int KS = D / 16;  // k-steps of the first product
    constexpr int MB = D / 32;  // 32-row blocks of O^T
    constexpr int RB = TL::kRowBytes;
    constexpr int ROWS = 32 * WAVES;
    constexpr int IPW = kFlashKeys / (WAVES * TL::kRowsPerInstr);
    static_assert(IPW >= 1 && IPW * WAVES * TL::kRowsPerInstr == kFlashKeys, "a tile's requests divide evenly among the wavefronts");
    static_assert(KS == 2 * MB && (KS == 8 || KS == 4), "the interleave below is written for d = 128 and d = 64");

    // two buffers each; the K tiles are 32 keys ahead of the V tiles
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[TL::kBytes];
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

    int L;
    int64_t base, kv_base;
    const int hk = h / p.kv_group;
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
    const int n_q = VARLEN ? (L + ROWS - 1) / ROWS : p.n_qtiles;
    if (VARLEN && slot >= (p.paired ? (n_q + 1) >> 1 : n_q)) return;
    const T* const gq = static_cast<const T*>(p.q) + base;
    const T* const gk = static_cast<const T*>(p.k) + kv_base;
    const T* const gv = static_cast<const T*>(p.v) + kv_base;
    T* const go = static_cast<T*>(p.o) + base;
    const int64_t sn = p.stride_n;
    const int64_t skv = p.kv_stride_n;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int d_real = (p.d_real > 0 && p.d_real < D) ? p.d_real : D;

    // ---- per-lane request offsets (bytes from the first row of a tile), fixed for the whole kernel ------
    int dma_off_k[IPW], dma_off_v[IPW];
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
        const int r = (wave * IPW + i) * TL::kRowsPerInstr + lane / TL::kChunks;
        const int pc = lane % TL::kChunks;
        const int ck = pc ^ TL::fk(r), cv = pc ^ TL::fv(r);
        dma_off_k[i] = (int)(r * skv * 2) + ((8 * ck < d_real ? ck : 0) << 4);
        dma_off_v[i] = (int)(r * skv * 2) + ((8 * cv < d_real ? cv : 0) << 4);
    }
    // Keys k0.. of this head into a buffer.  Bytes from the tile's first row to the end of the sequence's last row bound
    // the descriptor: rows that do not exist read as zeros; a tile at or behind `limit` keys (the end of this query
    // tile's walk) touches no memory at all.
    auto nrec_of = [&](int k0, int limit) AHPC_INLINE_LAMBDA -> unsigned {
        const int64_t rem = k0 < limit ? (int64_t)(L - k0 - 1) * skv * 2 + 2 * d_real : 0;
        return rem > 0xffffffffll ? 0xffffffffu : (unsigned)rem;
    };
    auto dma_k = [&](int k0, int limit, unsigned char* dst) AHPC_INLINE_LAMBDA {
        dma_tile<D, IPW>(gk + (int64_t)(k0 < limit ? k0 : 0) * skv, nrec_of(k0, limit), dma_off_k, dst, wave_u);
    };
    auto dma_v = [&](int k0, int limit, unsigned char* dst) AHPC_INLINE_LAMBDA {
        dma_tile<D, IPW>(gv + (int64_t)(k0 < limit ? k0 : 0) * skv, nrec_of(k0, limit), dma_off_v, dst, wave_u);
    };

    // ---- LDS operand addresses (byte offsets inside a tile) -------------------------------------
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
        const int qt = flash_qtile_of_part(p, n_q, slot, part);
        if (qt < 0) break;
        const int q_tile0 = qt * ROWS;
        if (q_tile0 >= L) continue;

        int k_end = L;
        if (CAUSAL) k_end = (q_tile0 + ROWS) < L ? (q_tile0 + ROWS) : L;
        const int n_sub = (k_end + 31) / 32;    // sub-tiles of 32 keys
        const int n_steps = (n_sub + 1) / 2;    // steps over a (K, V) tile pair

        // first tiles on their way before anything else: keys 0..63 (its first 32 rows give S(0)), K tile 0, V tile 0
        dma_k(0, k_end, lds_k1);
        dma_k(32, k_end, lds_k0);
        dma_v(0, k_end, lds_v0);

        // ---- Q^T operands, pre-multiplied by c = scale*log2(e), kept for the whole query tile --------
        const int qw = q_tile0 + wave * 32;  // first query row of this wavefront
        const int qrow = qw + col;
        u32x4 qreg[KS];
        {
            const int row = qrow < L ? qrow : L - 1;
            const T* src = gq + (int64_t)row * sn + 8 * half;
            const float cs = p.scale_log2;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const u32x4 raw = 16 * ks + 8 * half < d_real ? *reinterpret_cast<const u32x4*>(src + 16 * ks) : u32x4{0u, 0u, 0u, 0u};
                u32x4 sc;
#pragma unroll
                for (int w = 0; w < 4; ++w) sc[w] = pack2<T>(lo_f32<T>(raw[w]) * cs, hi_f32<T>(raw[w]) * cs);
                qreg[ks] = sc;
            }
        }

        // ---- running state (log2 units, see flash_fwd_mfma.hpp) --------------------------------------
        f32x16 oacc[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[mb][r] = 0.0f;
        f32x16 neg_m;
#pragma unroll
        for (int r = 0; r < 16; ++r) neg_m[r] = 0.0f;
        float l_run = 0.0f;
        constexpr float kRaise = 8.0f;

        // a wavefront whose queries all precede a sub-tile has nothing to add to it
        const int qw_u = q_tile0 + wave_u * 32;  // (the same value in a scalar register: the conditions below are wave-uniform)
        auto active = [&](int u) AHPC_INLINE_LAMBDA { return u < n_sub && !(CAUSAL && u * 32 > qw_u + 31); };
        auto needs_mask = [&](int u) AHPC_INLINE_LAMBDA { return (u * 32 + 32 > L) || (CAUSAL && (u * 32 + 31 > qw_u)); };
        // key = 32u + 4*half + off(r); visible iff key <= min(query row, L-1)
        auto apply_mask = [&](f32x16& s, int u) AHPC_INLINE_LAMBDA {
            int lim = L - 1;
            if (CAUSAL) lim = qrow < lim ? qrow : lim;
            lim -= u * 32 + 4 * half;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int off = 8 * (r >> 2) + (r & 3);
                s[r] = off <= lim ? s[r] : -INFINITY;
            }
        };
        auto row_max = [&](const f32x16& s) AHPC_INLINE_LAMBDA {
            float m = fmaxf(s[0], s[1]);
#pragma unroll
            for (int r = 2; r < 16; r += 2) m = max3(m, s[r], s[r + 1]);
            return m;
        };
        // Raises the reference maximum of the rows whose new scores `s` (not yet exponentiated) exceed it by 2^kRaise, or
        // sets it exactly (first sub-tile); everything accumulated so far is rescaled.
        auto adjust = [&](f32x16& s, float mx_in, bool first) AHPC_INLINE_LAMBDA {
            const float mx = halves_max(mx_in);
            const float delta = first ? mx : fmaxf(mx, 0.0f);
            if (!first) {  // (nothing has been accumulated before the first sub-tile)
                const float alpha = fast_exp2(-delta);
                l_run *= alpha;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[mb][r] *= alpha;
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] -= delta;
            const float nm = neg_m[0] - delta;
#pragma unroll
            for (int r = 0; r < 16; ++r) neg_m[r] = nm;
        };

        // exp2 / pack / row sum of element pair w of the 16 keys of group g (0, 1) of a sub-tile
        u32x4 pb[2];
        float sum;
        auto make_p = [&](const f32x16& s, int g, int w) AHPC_INLINE_LAMBDA {
            const float p0 = fast_exp2(s[8 * g + 2 * w]), p1 = fast_exp2(s[8 * g + 2 * w + 1]);
            pb[g][w] = pack2<T>(p0, p1);
            sum += p0 + p1;
        };

        // One sub-step.  sc = scores of sub-tile u (reference maximum applied), sn_ receives those of sub-tile u+1;
        // k_rows = the 32 K rows of sub-tile u+1, v_rows = the 32 V rows of sub-tile u.  The chunks between the
        // scheduling fences are what one matrix instruction's time is filled with.  The steady state (this sub-tile and
        // the next one both belong to the wavefront) is one straight line of code; all conditions are wave-uniform.
        auto substep = [&](f32x16& sc, f32x16& sn_, int u, const unsigned char* k_rows, const unsigned char* v_rows) AHPC_INLINE_LAMBDA {
            if (!active(u)) return;  // (then the next one is not active either)
            const bool act_next = active(u + 1);
            sum = 0.0f;
            u32x2 vf[2][MB][2];
            float mx = -INFINITY;
            if (act_next) {
                // ---- phase 1: S(u+1) on the matrix cores; the first 16 keys of exp(S(u)); V operands of those keys -------
                constexpr int kAhead = KS < 4 ? KS : 4;
                u32x4 a[KS];
#pragma unroll
                for (int ks = 0; ks < kAhead; ++ks) a[ks] = lds_read_b128(k_rows + k_off[ks]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    sn_ = mfma_32x32x16<T>(a[ks], qreg[ks], ks == 0 ? neg_m : sn_);
                    if (ks + kAhead < KS) a[ks + kAhead] = lds_read_b128(k_rows + k_off[ks + kAhead]);
                    if (KS == 8) {
                        if ((ks & 1) == 0) make_p(sc, 0, ks >> 1);
                        else {
                            const int mb = ks >> 1;
                            vf[0][mb][0] = TrRead<T>::load(v_rows + v_off[mb]);
                            vf[0][mb][1] = TrRead<T>::load(v_rows + v_off[mb] + 8 * RB);
                        }
                    } else {
                        make_p(sc, 0, ks);
                        if (ks & 1) {
#pragma unroll
                            for (int mb = ks - 1; mb <= ks && mb < MB; ++mb) {
                                vf[0][mb][0] = TrRead<T>::load(v_rows + v_off[mb]);
                                vf[0][mb][1] = TrRead<T>::load(v_rows + v_off[mb] + 8 * RB);
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                // ---- phase 2: O^T += V(u)^T P^T; the other 16 keys of exp(S(u)); row maximum of S(u+1) -----------------
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const u32x4 av = u32x4{vf[0][mb][0][0], vf[0][mb][0][1], vf[0][mb][1][0], vf[0][mb][1][1]};
                    oacc[mb] = mfma_32x32x16<T>(av, pb[0], oacc[mb]);
                    vf[1][mb][0] = TrRead<T>::load(v_rows + v_off[mb] + 16 * RB);
                    vf[1][mb][1] = TrRead<T>::load(v_rows + v_off[mb] + 24 * RB);
                    if (MB == 4) make_p(sc, 1, mb);
                    else { make_p(sc, 1, 2 * mb); make_p(sc, 1, 2 * mb + 1); }
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const u32x4 av = u32x4{vf[1][mb][0][0], vf[1][mb][0][1], vf[1][mb][1][0], vf[1][mb][1][1]};
                    oacc[mb] = mfma_32x32x16<T>(av, pb[1], oacc[mb]);
                    constexpr int per = 16 / MB;  // elements of S(u+1) folded into the maximum per matrix instruction
#pragma unroll
                    for (int r = per * mb; r < per * (mb + 1); r += 2) mx = max3(mx, sn_[r], sn_[r + 1]);
                    __builtin_amdgcn_sched_barrier(0);
                }
                l_run += sum;
                if (needs_mask(u + 1)) {
                    apply_mask(sn_, u + 1);
                    mx = row_max(sn_);
                }
                if (__builtin_amdgcn_ballot_w64(mx > kRaise) != 0) adjust(sn_, mx, false);
            } else {
                // the wavefront's last sub-tile: nothing to prepare
#pragma unroll
                for (int g = 0; g < 2; ++g)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        vf[g][mb][0] = TrRead<T>::load(v_rows + v_off[mb] + (16 * g) * RB);
                        vf[g][mb][1] = TrRead<T>::load(v_rows + v_off[mb] + (16 * g + 8) * RB);
                    }
#pragma unroll
                for (int g = 0; g < 2; ++g)
#pragma unroll
                    for (int w = 0; w < 4; ++w) make_p(sc, g, w);
#pragma unroll
                for (int g = 0; g < 2; ++g)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        const u32x4 av = u32x4{vf[g][mb][0][0], vf[g][mb][0][1], vf[g][mb][1][0], vf[g][mb][1][1]};
                        oacc[mb] = mfma_32x32x16<T>(av, pb[g], oacc[mb]);
                    }
                l_run += sum;
            }
        };

        f32x16 sa, sb;
        // One step: the two sub-tiles of V tile t, with the K rows 32 keys ahead of them; the next pair of tiles is
        // requested first and has landed for everyone behind the barrier.
        auto step = [&](int t, const unsigned char* k_cur, const unsigned char* v_cur, unsigned char* k_nxt, unsigned char* v_nxt) AHPC_INLINE_LAMBDA {
            dma_k((t + 1) * kFlashKeys + 32, k_end, k_nxt);
            dma_v((t + 1) * kFlashKeys, k_end, v_nxt);
            substep(sa, sb, 2 * t, k_cur, v_cur);
            substep(sb, sa, 2 * t + 1, k_cur + 32 * RB, v_cur + 32 * RB);
            __builtin_amdgcn_s_waitcnt(0);  // this wave's part of the requested tiles has landed
            __syncthreads();                // everyone's has, and everyone is done with the tiles of this step
        };

        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        // scores of the first sub-tile, reference maximum set exactly
        {
            u32x4 a[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) a[ks] = lds_read_b128(lds_k1 + k_off[ks]);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) sa = mfma_32x32x16<T>(a[ks], qreg[ks], ks == 0 ? neg_m : sa);
            if (needs_mask(0)) apply_mask(sa, 0);
            adjust(sa, row_max(sa), true);
        }
        __syncthreads();  // the buffer S(0) came from is free
        for (int t = 0; t < n_steps; t += 2) {
            step(t, lds_k0, lds_v0, lds_k1, lds_v1);
            if (t + 1 < n_steps) step(t + 1, lds_k1, lds_v1, lds_k0, lds_v0);
        }

        // ---- normalise and store: lane holds, per 32-row block, 4 runs of 4 consecutive lanes of d ---
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
                    if (32 * mb + 8 * g4 + 4 * half < d_real) *reinterpret_cast<u32x2*>(dst + 32 * mb + 8 * g4) = w;
                }
        }
        __syncthreads();  // the next query tile's first requests reuse the buffers
    }
}

template <typename T, int D, bool CAUSAL, bool VARLEN>
__global__ __launch_bounds__(64 * kFlashWideWaves, 1) void flash_fwd_pipe_wide_kernel(const FlashParams p) {
    flash_fwd_pipe_body<T, D, CAUSAL, VARLEN, kFlashWideWaves>(p);
}

template <typename T, int D, bool CAUSAL, bool VARLEN>
__global__ __launch_bounds__(kFlashThreads, 2) void flash_fwd_pipe_kernel(const FlashParams p) {
    flash_fwd_pipe_body<T, D, CAUSAL, VARLEN, 4>(p);
}

}  // namespace ahpc
