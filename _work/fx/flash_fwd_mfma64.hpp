// FlashAttention forward on the gfx950 matrix cores, 64 query columns per wavefront (fp16 / bf16, d = 128).
//
// One workgroup = 4 wavefronts = 256 query rows of one (sequence, head), one workgroup per CU: a wavefront has the
// SIMD's whole register file (512 registers per lane) and keeps TWO 32-column blocks of queries.  Every K or V operand
// read from LDS then feeds two matrix instructions, and the CU requests every K/V tile once for 256 rows.
//
// With one wavefront per SIMD nothing else hides the softmax arithmetic, so the walk over the keys is software
// pipelined inside the wavefront, 32 keys (a "sub-tile") at a time:
//   phase 1 of sub-step u:  S(u+1)^T = K(u+1) Q^T   on the matrix cores  |  exp2 / pack / row sums of the first 16 keys of S(u)
//   phase 2 of sub-step u:  O^T += V(u)^T P(u)^T    on the matrix cores  |  the other 16 keys of S(u), row maxima of S(u+1)
// K is therefore read 32 keys ahead of V: the K tiles in LDS start 32 keys later than the V tiles (K tile p = keys
// 64p+32 .. 64p+95, V tile p = keys 64p .. 64p+63), so that one step over a tile pair reads exactly one K and one V buffer.
// Layouts, the lazily raised reference maximum and the LDS swizzles are those of flash_fwd_mfma.hpp; the tile requests,
// the workgroup map and the launch plan are shared with it.
#pragma once

#include "flash_fwd_mfma.hpp"

namespace ahpc {

constexpr int kFlash64Waves = 4;
constexpr int kFlash64Rows = 64 * kFlash64Waves;  // query rows per workgroup

template <typename T, int D, bool CAUSAL, bool VARLEN>
__global__ __launch_bounds__(64 * kFlash64Waves, 1) void flash_fwd_mfma64_kernel(const FlashParams p) {
    typedef FlashTile<D> TL;
    constexpr int KS = D / 16;  // k-steps of the first product
    constexpr int MB = D / 32;  // 32-row blocks of O^T
    constexpr int RB = TL::kRowBytes;
    constexpr int ROWS = kFlash64Rows;
    constexpr int IPW = kFlashKeys / (kFlash64Waves * TL::kRowsPerInstr);
    static_assert(D == 128, "registers are budgeted for d = 128");

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
    // A tile at or behind `limit` keys (the end of this query tile's walk) touches no memory and lands as zeros.
    auto nrec_of = [&](int k0, int limit) __attribute__((always_inline)) -> unsigned {
        const int64_t rem = k0 < limit ? (int64_t)(L - k0 - 1) * skv * 2 + 2 * d_real : 0;
        return rem > 0xffffffffll ? 0xffffffffu : (unsigned)rem;
    };
    auto dma_k = [&](int k0, int limit, unsigned char* dst) __attribute__((always_inline)) { dma_tile<D, IPW>(gk + (int64_t)(k0 < limit ? k0 : 0) * skv, nrec_of(k0, limit), dma_off_k, dst, wave_u); };
    auto dma_v = [&](int k0, int limit, unsigned char* dst) __attribute__((always_inline)) { dma_tile<D, IPW>(gv + (int64_t)(k0 < limit ? k0 : 0) * skv, nrec_of(k0, limit), dma_off_v, dst, wave_u); };

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

        // ---- Q^T operands of the two column blocks, pre-multiplied by c = scale*log2(e) ----------------
        const int qw = q_tile0 + wave * 64;  // first query row of this wavefront
        int qrow[2];
        u32x4 qreg[2][KS];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            qrow[c] = qw + 32 * c + col;
            const int row = qrow[c] < L ? qrow[c] : L - 1;
            const T* src = gq + (int64_t)row * sn + 8 * half;
            const float cs = p.scale_log2;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const u32x4 raw = 16 * ks + 8 * half < d_real ? *reinterpret_cast<const u32x4*>(src + 16 * ks) : u32x4{0u, 0u, 0u, 0u};
                u32x4 sc;
#pragma unroll
                for (int w = 0; w < 4; ++w) sc[w] = pack2<T>(lo_f32<T>(raw[w]) * cs, hi_f32<T>(raw[w]) * cs);
                qreg[c][ks] = sc;
            }
        }

        // ---- running state (log2 units, see flash_fwd_mfma.hpp) --------------------------------------
        f32x16 oacc[2][MB];
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[c][mb][r] = 0.0f;
        f32x16 neg_m[2];
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int r = 0; r < 16; ++r) neg_m[c][r] = 0.0f;
        float l_run[2] = {0.0f, 0.0f};
        constexpr float kRaise = 8.0f;

        // a wavefront whose queries all precede a sub-tile has nothing to add to it
        auto active = [&](int u) __attribute__((always_inline)) { return u < n_sub && !(CAUSAL && u * 32 > qw + 63); };
        auto needs_mask = [&](int u) __attribute__((always_inline)) { return (u * 32 + 32 > L) || (CAUSAL && (u * 32 + 31 > qw)); };
        // key = 32u + 4*half + off(r); visible iff key <= min(query row, L-1)
        auto apply_mask = [&](f32x16 (&s)[2], int u) __attribute__((always_inline)) {
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                int lim = L - 1;
                if (CAUSAL) lim = qrow[c] < lim ? qrow[c] : lim;
                lim -= u * 32 + 4 * half;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int off = 8 * (r >> 2) + (r & 3);
                    s[c][r] = off <= lim ? s[c][r] : -INFINITY;
                }
            }
        };
        auto row_max = [&](const f32x16& s) __attribute__((always_inline)) {
            float m = fmaxf(s[0], s[1]);
#pragma unroll
            for (int r = 2; r < 16; r += 2) m = max3(m, s[r], s[r + 1]);
            return m;
        };
        // Raises the reference maximum of the rows whose new scores `s` (not yet exponentiated) exceed it by 2^kRaise, or
        // sets it exactly (first sub-tile); everything accumulated so far is rescaled.
        auto adjust = [&](f32x16 (&s)[2], const float (&mx_in)[2], bool first) __attribute__((always_inline)) {
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const float mx = halves_max(mx_in[c]);
                const float delta = first ? mx : fmaxf(mx, 0.0f);
                if (!first) {  // (nothing has been accumulated before the first sub-tile)
                    const float alpha = fast_exp2(-delta);
                    l_run[c] *= alpha;
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int r = 0; r < 16; ++r) oacc[c][mb][r] *= alpha;
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) s[c][r] -= delta;
                const float nm = neg_m[c][0] - delta;
#pragma unroll
                for (int r = 0; r < 16; ++r) neg_m[c][r] = nm;
            }
        };

        // exp2 / pack / row sum of element pair w of the 16 keys of group g (0, 1) of a sub-tile, column block c
        u32x4 pb[2][2];
        float sum[2];
        auto make_p = [&](const f32x16 (&s)[2], int c, int g, int w) __attribute__((always_inline)) {
            const float p0 = fast_exp2(s[c][8 * g + 2 * w]), p1 = fast_exp2(s[c][8 * g + 2 * w + 1]);
            pb[c][g][w] = pack2<T>(p0, p1);
            sum[c] += p0 + p1;
        };

        // One sub-step.  sc = scores of sub-tile u (reference maximum applied), sn receives those of sub-tile u+1;
        // k_rows = the 32 K rows of sub-tile u+1, v_rows = the 32 V rows of sub-tile u.
        auto substep = [&](f32x16 (&sc)[2], f32x16 (&sn)[2], int u, const unsigned char* k_rows, const unsigned char* v_rows) __attribute__((always_inline)) {
            const bool act = active(u);
            const bool act_next = active(u + 1);
            sum[0] = sum[1] = 0.0f;
            // ---- phase 1: S(u+1) on the matrix cores, the first 16 keys of exp(S(u)) on the VALU -----------------
            if (act_next) {
                u32x4 a[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) a[ks] = lds_read_b128(k_rows + k_off[ks]);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    sn[0] = mfma_32x32x16<T>(a[ks], qreg[0][ks], ks == 0 ? neg_m[0] : sn[0]);
                    sn[1] = mfma_32x32x16<T>(a[ks], qreg[1][ks], ks == 0 ? neg_m[1] : sn[1]);
                    if (act) make_p(sc, ks >> 2, 0, ks & 3);
                }
                constexpr int kAhead = 4;
                __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);  // LDS reads
#pragma unroll
                for (int i = 0; i < KS; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // matrix instructions
                    if (i < KS - kAhead) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);  // VALU
                }
            } else if (act) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) make_p(sc, ks >> 2, 0, ks & 3);
            }
            __builtin_amdgcn_sched_barrier(0);
            // ---- phase 2: O^T += V(u)^T P^T, the other 16 keys of exp(S(u)), row maxima of S(u+1) -----------------
            float mx[2] = {-INFINITY, -INFINITY};
            if (act) {
                u32x2 vf[2][MB][2];
#pragma unroll
                for (int g = 0; g < 2; ++g)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        vf[g][mb][0] = TrRead<T>::load(v_rows + v_off[mb] + (16 * g) * RB);
                        vf[g][mb][1] = TrRead<T>::load(v_rows + v_off[mb] + (16 * g + 8) * RB);
                    }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const u32x4 av = u32x4{vf[0][mb][0][0], vf[0][mb][0][1], vf[0][mb][1][0], vf[0][mb][1][1]};
                    oacc[0][mb] = mfma_32x32x16<T>(av, pb[0][0], oacc[0][mb]);
                    oacc[1][mb] = mfma_32x32x16<T>(av, pb[1][0], oacc[1][mb]);
                    make_p(sc, 0, 1, mb);
                    make_p(sc, 1, 1, mb);
                }
                __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);  // the first group's V operands
#pragma unroll
                for (int i = 0; i < MB; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // the second group's, behind the matrix instructions
                    __builtin_amdgcn_sched_group_barrier(0x002, 10, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const u32x4 av = u32x4{vf[1][mb][0][0], vf[1][mb][0][1], vf[1][mb][1][0], vf[1][mb][1][1]};
                    oacc[0][mb] = mfma_32x32x16<T>(av, pb[0][1], oacc[0][mb]);
                    oacc[1][mb] = mfma_32x32x16<T>(av, pb[1][1], oacc[1][mb]);
                }
                if (act_next) {
                    mx[0] = row_max(sn[0]);
                    mx[1] = row_max(sn[1]);
                }
#pragma unroll
                for (int i = 0; i < MB; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                l_run[0] += sum[0];
                l_run[1] += sum[1];
            } else if (act_next) {
                mx[0] = row_max(sn[0]);
                mx[1] = row_max(sn[1]);
            }
            if (act_next) {
                if (needs_mask(u + 1)) {
                    apply_mask(sn, u + 1);
                    mx[0] = row_max(sn[0]);
                    mx[1] = row_max(sn[1]);
                }
                if (__builtin_amdgcn_ballot_w64(mx[0] > kRaise || mx[1] > kRaise) != 0) adjust(sn, mx, false);
            }
        };

        f32x16 sa[2], sb[2];
        // One step: the two sub-tiles of V tile t, with the K rows 32 keys ahead of them; the next pair of tiles is
        // requested first and has landed for everyone behind the barrier.
        auto step = [&](int t, const unsigned char* k_cur, const unsigned char* v_cur, unsigned char* k_nxt, unsigned char* v_nxt) __attribute__((always_inline)) {
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
            for (int ks = 0; ks < KS; ++ks) {
                sa[0] = mfma_32x32x16<T>(a[ks], qreg[0][ks], ks == 0 ? neg_m[0] : sa[0]);
                sa[1] = mfma_32x32x16<T>(a[ks], qreg[1][ks], ks == 0 ? neg_m[1] : sa[1]);
            }
            if (needs_mask(0)) apply_mask(sa, 0);
            const float mx[2] = {row_max(sa[0]), row_max(sa[1])};
            adjust(sa, mx, true);
        }
        __syncthreads();  // the buffer S(0) came from is free
        for (int t = 0; t < n_steps; t += 2) {
            step(t, lds_k0, lds_v0, lds_k1, lds_v1);
            if (t + 1 < n_steps) step(t + 1, lds_k1, lds_v1, lds_k0, lds_v0);
        }

        // ---- normalise and store ------------------------------------------------------------------------
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const float l = halves_sum(l_run[c]);
            const float inv = l > 0.0f ? 1.0f / l : 0.0f;
            if (qrow[c] < L) {
                T* dst = go + (int64_t)qrow[c] * sn + 4 * half;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        const f32x16& a = oacc[c][mb];
                        const u32x2 w = u32x2{pack2<T>(a[4 * g4 + 0] * inv, a[4 * g4 + 1] * inv),
                                              pack2<T>(a[4 * g4 + 2] * inv, a[4 * g4 + 3] * inv)};
                        if (32 * mb + 8 * g4 + 4 * half < d_real) *reinterpret_cast<u32x2*>(dst + 32 * mb + 8 * g4) = w;
                    }
            }
        }
        __syncthreads();  // the next query tile's first requests reuse the buffers
    }
}

}  // namespace ahpc
