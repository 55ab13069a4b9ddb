// FlashAttention forward, "wide" variant of flash_fwd_mfma.hpp: a wavefront owns 64 query rows instead of 32.
//
// Same formulation, tiles, swizzles and data movement as the standard kernel (see flash_fwd_mfma.hpp); what
// changes is the register blocking.  Every A operand fetched from LDS (a K row block for S^T = K Q^T, a V^T
// block for O^T += V^T P^T) feeds TWO matrix instructions, one per 32-query block of the wavefront, which
// halves the LDS operand traffic per FLOP; a workgroup of 4 wavefronts covers 256 query rows, which halves
// the K/V tile stream from L2 per FLOP and the barriers per FLOP.  The price is registers (two sets of
// Q^T operands, score blocks and output accumulators: one wavefront per SIMD, one workgroup per CU), so
// the overlap of softmax arithmetic with matrix work has to come from within the wavefront: matrix
// instructions of one 16-key group are issued while the VALU prepares the next.  Above 256 registers the
// output accumulators live in accumulation registers, which the VALU can only reach through copies; the
// hot loop therefore never rescales them (see the two passes below).
//
// Key tiles are streamed two at a time (128 keys per barrier, 128 KiB of LDS at d = 128) and, where no mask is
// needed, processed by a software-pipelined routine (pipelined_super).
//
// Selected with AHPC_FLASH_WIDE=1; the standard kernel stays the default until both have been timed.
#pragma once

#include <type_traits>

#include "flash_fwd_mfma.hpp"

namespace ahpc {

constexpr int kWideRows = 256;  // query rows per workgroup
constexpr int kWideQB = 2;      // 32-query blocks per wavefront

template <typename T, int D, bool CAUSAL, bool VARLEN>
__global__ __launch_bounds__(kFlashThreads, 1) void flash_fwd_wide_kernel(const FlashParams p) {
    typedef FlashTile<D> TL;
    constexpr int KS = D / 16;
    constexpr int MB = D / 32;
    constexpr int RB = TL::kRowBytes;
    constexpr int QB = kWideQB;

    // a "super-tile" is two 64-key tiles, one behind the other (128 rows): one barrier per 128 keys
    constexpr int kSuperKeys = 2 * kFlashKeys;
    constexpr int kSuperBytes = 2 * TL::kBytes;
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[kSuperBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[kSuperBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[kSuperBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[kSuperBytes];
    __shared__ int retry_flags[4];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 31;
    const int half = lane >> 5;

    const FlashWork work = flash_work_of_block(blockIdx.x, p);
    if (!work.valid) return;
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
    const T* const gq = static_cast<const T*>(p.q) + base;
    const T* const gk = static_cast<const T*>(p.k) + kv_base;
    const T* const gv = static_cast<const T*>(p.v) + kv_base;
    T* const go = static_cast<T*>(p.o) + base;
    const int64_t sn = p.stride_n;
    const int64_t skv = p.kv_stride_n;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);

    int dma_off_k[TL::kInstrPerWave], dma_off_v[TL::kInstrPerWave];
#pragma unroll
    for (int i = 0; i < TL::kInstrPerWave; ++i) {
        const int r = (wave * TL::kInstrPerWave + i) * TL::kRowsPerInstr + lane / TL::kChunks;
        const int pc = lane % TL::kChunks;
        dma_off_k[i] = (int)(r * skv * 2) + ((pc ^ TL::fk(r)) << 4);
        dma_off_v[i] = (int)(r * skv * 2) + ((pc ^ TL::fv(r)) << 4);
    }
    auto dma_both = [&](int k0, unsigned char* dst_k, unsigned char* dst_v) {
        const int64_t rem = (int64_t)(L - k0 - 1) * skv * 2 + 2 * D;
        const unsigned nrec = rem > 0xffffffffll ? 0xffffffffu : (unsigned)rem;
        dma_tile<D>(gk + (int64_t)k0 * skv, nrec, dma_off_k, dst_k, wave_u);
        dma_tile<D>(gv + (int64_t)k0 * skv, nrec, dma_off_v, dst_v, wave_u);
    };

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
        const int qt = flash_qtile_of_part(p, slot, part);
        if (qt < 0) break;
        const int q_tile0 = qt * kWideRows;
        if (q_tile0 >= L) continue;

        int k_end = L;
        if (CAUSAL) k_end = (q_tile0 + kWideRows) < L ? (q_tile0 + kWideRows) : L;
        const int n_super = (k_end + kSuperKeys - 1) / kSuperKeys;

        const int qw = q_tile0 + wave * (32 * QB);  // first query row of this wavefront
        int qrow[QB];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) qrow[qb] = qw + 32 * qb + col;
        // Q^T operands of the wavefront's two 32-query blocks, pre-multiplied by scale*log2(e).  Loaded at the
        // start of each pass, so that each pass has its own (short) live range for them.
        u32x4 qreg[QB][KS];
        auto load_q = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
                const int row = qrow[qb] < L ? qrow[qb] : L - 1;
                const T* src = gq + (int64_t)row * sn + 8 * half;
                const float c = p.scale_log2;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const u32x4 raw = *reinterpret_cast<const u32x4*>(src + 16 * ks);
                    u32x4 sc;
#pragma unroll
                    for (int w = 0; w < 4; ++w) sc[w] = pack2<T>(lo_f32<T>(raw[w]) * c, hi_f32<T>(raw[w]) * c);
                    qreg[qb][ks] = sc;
                }
            }
        };

        f32x16 oacc[QB][MB];
        f32x16 neg_m[QB];
        float l_run[QB];
        bool bailed = false;  // wave-uniform: the fast pass met scores it cannot represent in its fixed frame
        // Fast pass: the reference maximum of a query is fixed by the first key block it sees; later scores may top
        // it by up to 2^kFrame and are simply exponentiated (p <= 2^15 fits fp16 and bf16; sums stay far inside
        // fp32).  Nothing in this pass ever rescales the output accumulators, so the VALU never touches them.
        // Slow pass: the lazy-maximum algorithm of the standard kernel (raise the reference when topped by 2^8,
        // rescale accumulators), from scratch, for wavefronts whose fast pass gave up.
        constexpr float kFrame = 15.0f;
        constexpr float kRaise = 8.0f;

        auto reset_state = [&]() {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[qb][mb][r] = 0.0f;
#pragma unroll
                for (int r = 0; r < 16; ++r) neg_m[qb][r] = 0.0f;
                l_run[qb] = 0.0f;
            }
        };

        // One 32-key block of a tile: scores, softmax, and its two 16-key groups of the second product.
        auto compute_block = [&](auto slow_tag, auto first_tag, const unsigned char* tile_k, const unsigned char* tile_v, int kblock0) __attribute__((always_inline)) {
            constexpr bool SLOW = decltype(slow_tag)::value;
            constexpr bool FIRST = decltype(first_tag)::value;  // the first key block of the pass: it fixes the frame
            // ---- S^T = c*K Q^T - m for 32 keys x 64 queries: every K operand feeds both query blocks -----
            f32x16 s[QB];
            {
                const u32x4 a = lds_read_b128(tile_k + k_off[0]);
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) s[qb] = mfma_32x32x16<T>(a, qreg[qb][0], neg_m[qb]);
            }
#pragma unroll
            for (int ks = 1; ks < KS; ++ks) {
                const u32x4 a = lds_read_b128(tile_k + k_off[ks]);
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) s[qb] = mfma_32x32x16<T>(a, qreg[qb][ks], s[qb]);
            }
            // V operands of the first 16 keys: requested now, used after the softmax arithmetic
            u32x2 vf[2][MB][2];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                vf[0][mb][0] = TrRead<T>::load(tile_v + v_off[mb]);
                vf[0][mb][1] = TrRead<T>::load(tile_v + v_off[mb] + 8 * RB);
            }

            const bool need_mask = (kblock0 + 32 > L) || (CAUSAL && (kblock0 + 31 > qw));
            if (need_mask) {
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) {
                    int lim = L - 1;
                    if (CAUSAL) lim = qrow[qb] < lim ? qrow[qb] : lim;
                    lim -= kblock0 + 4 * half;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int off = 8 * (r >> 2) + (r & 3);
                        s[qb][r] = off <= lim ? s[qb][r] : -INFINITY;
                    }
                }
            }
            float mx[QB];
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
                mx[qb] = s[qb][0];
#pragma unroll
                for (int r = 1; r < 16; ++r) mx[qb] = fmaxf(mx[qb], s[qb][r]);
            }
            float top = mx[0];
#pragma unroll
            for (int qb = 1; qb < QB; ++qb) top = fmaxf(top, mx[qb]);
            if constexpr (FIRST) {
                // the first block a wavefront sees fixes the frame: the accumulators are still zero
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) {
                    const float m2 = halves_max(mx[qb]);
                    const float delta = m2 > -INFINITY ? m2 : 0.0f;  // a query block that sees none of these keys yet
#pragma unroll
                    for (int r = 0; r < 16; ++r) s[qb][r] -= delta;
#pragma unroll
                    for (int r = 0; r < 16; ++r) neg_m[qb][r] = -delta;
                }
            } else if constexpr (!SLOW) {
                if (__builtin_amdgcn_ballot_w64(top > kFrame) != 0) {
                    bailed = true;
                    return;
                }
            } else if (__builtin_amdgcn_ballot_w64(top > kRaise) != 0) {
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) {
                    const float delta = fmaxf(halves_max(mx[qb]), 0.0f);
                    const float alpha = fast_exp2(-delta);
                    l_run[qb] *= alpha;
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int r = 0; r < 16; ++r) oacc[qb][mb][r] *= alpha;
#pragma unroll
                    for (int r = 0; r < 16; ++r) s[qb][r] -= delta;
                    const float nm = neg_m[qb][0] - delta;
#pragma unroll
                    for (int r = 0; r < 16; ++r) neg_m[qb][r] = nm;
                }
            }

            // ---- P^T = exp2(S^T) as B operands, O^T += V^T P^T, 16 keys at a time; every V^T operand feeds
            //      both query blocks.  While the matrix core works on one group the VALU prepares the other.
            u32x4 pb[2][QB];
            float sum[QB];
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) sum[qb] = 0.0f;
            auto make_pb = [&](int g) {
#pragma unroll
                for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const float p0 = fast_exp2(s[qb][8 * g + 2 * w]), p1 = fast_exp2(s[qb][8 * g + 2 * w + 1]);
                        pb[g][qb][w] = pack2<T>(p0, p1);
                        sum[qb] += p0 + p1;
                    }
            };
            make_pb(0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < 2; ++g) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const u32x4 a = u32x4{vf[g][mb][0][0], vf[g][mb][0][1], vf[g][mb][1][0], vf[g][mb][1][1]};
#pragma unroll
                    for (int qb = 0; qb < QB; ++qb) oacc[qb][mb] = mfma_32x32x16<T>(a, pb[g][qb], oacc[qb][mb]);
                }
                if (g == 0) {
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        vf[1][mb][0] = TrRead<T>::load(tile_v + v_off[mb] + 16 * RB);
                        vf[1][mb][1] = TrRead<T>::load(tile_v + v_off[mb] + 24 * RB);
                    }
                    make_pb(1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) l_run[qb] += sum[qb];
        };

        // One pass over the key tiles of this query tile.  `active`: whether this wavefront computes (all
        // wavefronts stream tiles and meet at the barriers either way).
        // Streams the super-tile that starts at key k0 (its second half only if it holds keys that are needed).
        auto dma_super = [&](int k0, unsigned char* dst_k, unsigned char* dst_v) __attribute__((always_inline)) {
            dma_both(k0, dst_k, dst_v);
            if (k0 + kFlashKeys < k_end) dma_both(k0 + kFlashKeys, dst_k + TL::kBytes, dst_v + TL::kBytes);
        };

        // Fast pass, a super-tile all of whose 128 keys are visible to all 64 queries of the wavefront (no mask),
        // software-pipelined over its four 32-key blocks: while the matrix cores work on the scores of block b+1 and on
        // the second product of block b, the VALU turns the scores of block b into P and copies the scores of block
        // b+1 out of the accumulation registers.  No branches: a score beyond the frame only sets a flag.
        auto pipelined_super = [&](const unsigned char* tile_k, const unsigned char* tile_v) __attribute__((always_inline)) {
            auto scores = [&](int blk, f32x16 (&dst)[QB]) __attribute__((always_inline)) {
                const unsigned char* tk = tile_k + 32 * blk * RB;
                {
                    const u32x4 a = lds_read_b128(tk + k_off[0]);
#pragma unroll
                    for (int qb = 0; qb < QB; ++qb) dst[qb] = mfma_32x32x16<T>(a, qreg[qb][0], neg_m[qb]);
                }
#pragma unroll
                for (int ks = 1; ks < KS; ++ks) {
                    const u32x4 a = lds_read_b128(tk + k_off[ks]);
#pragma unroll
                    for (int qb = 0; qb < QB; ++qb) dst[qb] = mfma_32x32x16<T>(a, qreg[qb][ks], dst[qb]);
                }
            };
            auto v_operands = [&](int blk, int g, u32x2 (&dst)[MB][2]) __attribute__((always_inline)) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    dst[mb][0] = TrRead<T>::load(tile_v + v_off[mb] + (32 * blk + 16 * g) * RB);
                    dst[mb][1] = TrRead<T>::load(tile_v + v_off[mb] + (32 * blk + 16 * g + 8) * RB);
                }
            };
            auto make_pb = [&](const f32x16 (&s)[QB], int g, u32x4 (&pb)[QB], float (&sum)[QB]) __attribute__((always_inline)) {
#pragma unroll
                for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const float p0 = fast_exp2(s[qb][8 * g + 2 * w]), p1 = fast_exp2(s[qb][8 * g + 2 * w + 1]);
                        pb[qb][w] = pack2<T>(p0, p1);
                        sum[qb] += p0 + p1;
                    }
            };
            auto second_product = [&](const u32x2 (&vf)[MB][2], const u32x4 (&pb)[QB]) __attribute__((always_inline)) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const u32x4 a = u32x4{vf[mb][0][0], vf[mb][0][1], vf[mb][1][0], vf[mb][1][1]};
#pragma unroll
                    for (int qb = 0; qb < QB; ++qb) oacc[qb][mb] = mfma_32x32x16<T>(a, pb[qb], oacc[qb][mb]);
                }
            };
            auto beyond_frame = [&](const f32x16 (&s)[QB]) __attribute__((always_inline)) {
                float top = s[0][0];
#pragma unroll
                for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) top = fmaxf(top, s[qb][r]);
                return top > kFrame;
            };

            f32x16 s_cur[QB], s_nxt[QB];
            u32x2 vf0[MB][2], vf1[MB][2];
            u32x4 pb0[QB], pb1[QB];
            float sum[QB];
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) sum[qb] = 0.0f;
            bool beyond = false;
            scores(0, s_cur);
            v_operands(0, 0, vf0);
            beyond = beyond_frame(s_cur);
            // Each stage below is one scheduling region; the sched_group_barrier sequences ask for its matrix
            // instructions to be issued one or two at a time with the stage's VALU work in between (issue is in
            // order: VALU instructions placed after a run of matrix instructions would wait for all of them).
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                // stage A: scores of the next block | P of this block, first 16 keys.  One k-step of the scores
                // (an operand read, two matrix instructions) alternates with one slice of the P arithmetic; the
                // empty asm statements make, as far as the instruction scheduler can tell, each slice depend on
                // the k-step's operand and the next k-step's operand depend on the slice, which pins that order.
                if (blk < 3) {
                    const unsigned char* tk = tile_k + 32 * (blk + 1) * RB;
                    constexpr int kItems = QB * 4;             // (query block, register pair) items of make_pb
                    constexpr int kPerStep = kItems / KS > 0 ? kItems / KS : 1;
                    float pinned = 0.0f;
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        u32x4 a = lds_read_b128(tk + k_off[ks]);
                        if (ks > 0) asm("" : "+v"(a) : "v"(pinned));
#pragma unroll
                        for (int qb = 0; qb < QB; ++qb)
                            s_nxt[qb] = mfma_32x32x16<T>(a, qreg[qb][ks], ks == 0 ? neg_m[qb] : s_nxt[qb]);
#pragma unroll
                        for (int it = ks * kPerStep; it < (ks + 1) * kPerStep && it < kItems; ++it) {
                            const int qb = it / 4, w = it % 4;
                            float x0 = s_cur[qb][2 * w], x1 = s_cur[qb][2 * w + 1];
                            asm("" : "+v"(x0), "+v"(x1) : "v"(a));
                            const float p0 = fast_exp2(x0), p1 = fast_exp2(x1);
                            pb0[qb][w] = pack2<T>(p0, p1);
                            sum[qb] += p0 + p1;
                            pinned = p1;
                        }
                    }
                    // items the k-steps did not cover (more items than k-steps times kPerStep)
#pragma unroll
                    for (int it = KS * kPerStep; it < kItems; ++it) {
                        const int qb = it / 4, w = it % 4;
                        const float p0 = fast_exp2(s_cur[qb][2 * w]), p1 = fast_exp2(s_cur[qb][2 * w + 1]);
                        pb0[qb][w] = pack2<T>(p0, p1);
                        sum[qb] += p0 + p1;
                    }
                } else {
                    make_pb(s_cur, 0, pb0, sum);
                }
                __builtin_amdgcn_sched_barrier(0);
                // stage B: second product, first 16 keys | P of this block, last 16 keys
                v_operands(blk, 1, vf1);
                second_product(vf0, pb0);
                make_pb(s_cur, 1, pb1, sum);
#pragma unroll
                for (int i = 0; i < MB; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, QB, 1);
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
                    __builtin_amdgcn_sched_group_barrier(0x400, 16 / MB, 1);
                    __builtin_amdgcn_sched_group_barrier(0x002, 24 / MB, 1);
                }
                __builtin_amdgcn_sched_barrier(0);
                // stage C: second product, last 16 keys | the next block's scores copied out and checked
                if (blk < 3) v_operands(blk + 1, 0, vf0);
                second_product(vf1, pb1);
                if (blk < 3) {
                    // (the empty asm ties each copy out of the accumulation registers to a value of stage B, so that
                    // the copies are made here, between this stage's matrix instructions, and not right behind the
                    // matrix instructions that produce the scores, where they would wait for them)
#pragma unroll
                    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            float t = s_nxt[qb][r];
                            asm("" : "+v"(t) : "v"(pb1[qb][r & 3]));
                            s_cur[qb][r] = t;
                        }
                    beyond = beyond | beyond_frame(s_cur);
#pragma unroll
                    for (int i = 0; i < MB; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, QB, 2);
                        __builtin_amdgcn_sched_group_barrier(0x100, 2, 2);
                        __builtin_amdgcn_sched_group_barrier(0x002, 48 / MB, 2);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) l_run[qb] += sum[qb];
            if (__builtin_amdgcn_ballot_w64(beyond) != 0) bailed = true;  // the results of this pass are discarded
        };

        // One pass over the key super-tiles of this query tile.  `active`: whether this wavefront computes (all
        // wavefronts stream tiles and meet at the barriers either way).
        auto run_pass = [&](auto slow_tag, bool active) __attribute__((always_inline)) {
            constexpr bool SLOW = decltype(slow_tag)::value;
            // the four 32-key blocks of a super-tile one after the other, with masks where they are needed
            auto plain_super = [&](auto first_tag, const unsigned char* tile_k, const unsigned char* tile_v, int k0) __attribute__((always_inline)) {
                if (!SLOW && bailed) return;
                compute_block(slow_tag, first_tag, tile_k, tile_v, k0);  // key block 0 is never skipped: every query sees key 0
#pragma unroll
                for (int blk = 1; blk < 4; ++blk) {
                    const int kblock0 = k0 + 32 * blk;
                    if (kblock0 >= L) continue;                               // nothing but padding
                    if (CAUSAL && kblock0 > qw + 32 * QB - 1) continue;      // every key of the block is in the future
                    if (!SLOW && bailed) continue;
                    compute_block(slow_tag, std::false_type{}, tile_k + 32 * blk * RB, tile_v + 32 * blk * RB, kblock0);
                }
            };
            auto step = [&](auto first_tag, unsigned char* cur_k, unsigned char* cur_v, unsigned char* nxt_k, unsigned char* nxt_v, int st) __attribute__((always_inline)) {
                const int k0 = st * kSuperKeys;
                const bool more = st + 1 < n_super;
                if (more) dma_super(k0 + kSuperKeys, nxt_k, nxt_v);
                if (active && !(CAUSAL && k0 > qw + 32 * QB - 1)) {
                    const bool unmasked = k0 + kSuperKeys <= L && !(CAUSAL && k0 + kSuperKeys - 1 > qw);
                    if (!SLOW && !decltype(first_tag)::value && unmasked) {
                        if (!bailed) pipelined_super(cur_k, cur_v);
                    } else {
                        plain_super(first_tag, cur_k, cur_v, k0);
                    }
                }
                if (more) {
                    __builtin_amdgcn_s_waitcnt(0);
                    __syncthreads();
                }
            };
            dma_super(0, lds_k0, lds_v0);
            load_q();
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            step(std::true_type{}, lds_k0, lds_v0, lds_k1, lds_v1, 0);
            for (int st = 1; st < n_super; st += 2) {
                step(std::false_type{}, lds_k1, lds_v1, lds_k0, lds_v0, st);
                if (st + 1 < n_super) step(std::false_type{}, lds_k0, lds_v0, lds_k1, lds_v1, st + 1);
            }
            __syncthreads();  // whatever comes next reuses the buffers
        };

        reset_state();
        run_pass(std::false_type{}, true);
        // does any wavefront of the workgroup need the slow pass?  (all of them must stream its tiles)
        if (lane == 0) retry_flags[wave] = bailed ? 1 : 0;
        __syncthreads();
        const bool any_retry = (retry_flags[0] | retry_flags[1] | retry_flags[2] | retry_flags[3]) != 0;
        __syncthreads();
        if (any_retry) {
            if (bailed) reset_state();
            run_pass(std::true_type{}, bailed);
        }

#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const float l = halves_sum(l_run[qb]);
            const float inv = l > 0.0f ? 1.0f / l : 0.0f;
            if (qrow[qb] < L) {
                T* dst = go + (int64_t)qrow[qb] * sn + 4 * half;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        const f32x16& a = oacc[qb][mb];
                        const u32x2 w = u32x2{pack2<T>(a[4 * g4 + 0] * inv, a[4 * g4 + 1] * inv),
                                              pack2<T>(a[4 * g4 + 2] * inv, a[4 * g4 + 3] * inv)};
                        *reinterpret_cast<u32x2*>(dst + 32 * mb + 8 * g4) = w;
                    }
            }
        }
    }
}

}  // namespace ahpc
