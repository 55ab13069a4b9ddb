// FlashAttention forward on the gfx950 matrix cores, 256 query rows per workgroup, persistent workgroups
// (fp16 / bf16, dense launches without a mask).
//
// Tile arithmetic, layouts and swizzles are those of flash_fwd_mfma.hpp with eight wavefronts: one workgroup per CU,
// 32 query columns per wavefront, one stream of K/V tiles for the 256 rows (half the tile requests and half the
// L2 -> LDS bytes per matrix instruction of the 128-row form).  With a single workgroup on the CU nothing covers the
// start and the end of a query tile, so those are taken off the critical path:
//   * a workgroup is persistent: it walks the block ids i, i + grid, i + 2 grid, ... of the launch's work map, and as
//     soon as every wavefront is through with the last key tile of a query tile it requests the first TWO K/V tiles
//     and the Q rows of the next query tile - before it normalises and stores the finished one;
//   * the output goes through a private stretch of LDS per wavefront: the accumulators hold a query per lane (32 rows,
//     8 bytes each per store otherwise); after the exchange a store instruction writes four whole rows of 256 bytes.
#pragma once

#include "flash_fwd_mfma.hpp"

namespace ahpc {

template <typename T, int D, bool CAUSAL>
__global__ __launch_bounds__(64 * kFlashWideWaves, 1) void flash_fwd_wide_kernel(const FlashParams p) {
    typedef FlashTile<D> TL;
    constexpr int WAVES = kFlashWideWaves;
    constexpr int ROWS = kFlashWideRows;
    constexpr int KS = D / 16;  // k-steps of the first product
    constexpr int MB = D / 32;  // 32-row blocks of O^T
    constexpr int RB = TL::kRowBytes;
    constexpr int CH = TL::kChunks;  // 16-byte chunks per row
    constexpr int IPW = kFlashKeys / (WAVES * TL::kRowsPerInstr);
    static_assert(IPW >= 1 && IPW * WAVES * TL::kRowsPerInstr == kFlashKeys, "a tile's requests divide evenly among the wavefronts");
    static_assert(D == 128 || D == 64, "the output exchange is laid out for rows of 8 or 16 chunks");

    // The tile buffers are aligned more strictly than the output stretch so that they are laid out first: operand reads
    // address them with the instruction's 16-bit offset field, which ends at 64 KiB.
    __shared__ __attribute__((aligned(16384))) unsigned char lds_k0[TL::kBytes];
    __shared__ __attribute__((aligned(16384))) unsigned char lds_v0[TL::kBytes];
    __shared__ __attribute__((aligned(16384))) unsigned char lds_k1[TL::kBytes];
    __shared__ __attribute__((aligned(16384))) unsigned char lds_v1[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_out[WAVES * 32 * RB];  // 32 output rows per wavefront

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 31;
    const int half = lane >> 5;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int64_t sn = p.stride_n;
    const int64_t skv = p.kv_stride_n;
    const int d_real = (p.d_real > 0 && p.d_real < D) ? p.d_real : D;
    const int L = p.N;
    auto set_priority = [&](bool busy) {
        if (busy) __builtin_amdgcn_s_setprio(1); else __builtin_amdgcn_s_setprio(0);
    };

    // ---- per-lane request offsets and LDS operand addresses, fixed for the whole kernel (see flash_fwd_mfma.hpp) ----
    int dma_off_k[IPW], dma_off_v[IPW];
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
        const int r = (wave * IPW + i) * TL::kRowsPerInstr + lane / CH;
        const int pc = lane % CH;
        const int ck = pc ^ TL::fk(r), cv = pc ^ TL::fv(r);
        dma_off_k[i] = (int)(r * skv * 2) + ((8 * ck < d_real ? ck : 0) << 4);
        dma_off_v[i] = (int)(r * skv * 2) + ((8 * cv < d_real ? cv : 0) << 4);
    }
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

    // ---- the work of this workgroup: block ids blockIdx.x, + gridDim.x, ...; each id one or two query tiles ----------
    unsigned id = blockIdx.x;
    int part = -1;
    struct Item { int bh, qt; };
    auto advance = [&](Item& it) -> bool {
        for (;;) {
            if (++part == 2) {
                part = 0;
                id += gridDim.x;
            }
            if (id >= (unsigned)p.n_block_ids) return false;
            const FlashWork w = flash_work_of_block(id, p);
            // whatever the map says, nothing outside the tensors is ever addressed (uniform per workgroup)
            if (!w.valid || w.bh < 0 || w.bh >= p.n_bh || w.slot < 0 || w.slot >= flash_per_head(p)) {
                part = 1;  // (neither part of this id)
                continue;
            }
            const int qt = flash_qtile_of_part(p, p.n_qtiles, w.slot, part);
            if (qt < 0 || qt * ROWS >= L) continue;
            it.bh = w.bh;
            it.qt = qt;
            return true;
        }
    };

    // ---- state of the query tile in hand (set by `request`) ----------------------------------------------------------
    const T* gk = nullptr;
    const T* gv = nullptr;
    T* go = nullptr;
    int q_tile0 = 0, n_tiles = 0, qw = 0, qw_u = 0, qrow = 0, cur_bh = 0;
    u32x4 qreg[KS];  // raw Q rows between `request` and the start of the tile, scaled operands afterwards

    // The K/V tiles of a query tile are requested in order, one per call: the addresses and the bytes that remain behind them
    // (the descriptor's bound: rows behind the sequence's end read as zeros) advance by a tile per request instead of being
    // worked out from the tile number (64-bit products) every time.
    const int64_t tile_elems = (int64_t)kFlashKeys * skv;
    const T* k_next = nullptr;
    const T* v_next = nullptr;
    int64_t rem_next = 0;
    auto dma_next = [&](unsigned char* dst_k, unsigned char* dst_v) {
        const unsigned nrec = rem_next <= 0 ? 0u : rem_next > 0xffffffffll ? 0xffffffffu : (unsigned)rem_next;
        dma_tile<D, IPW>(k_next, nrec, dma_off_k, dst_k, wave_u);
        dma_tile<D, IPW>(v_next, nrec, dma_off_v, dst_v, wave_u);
        k_next += tile_elems;
        v_next += tile_elems;
        rem_next -= 2 * tile_elems;
    };
    // Everything a query tile needs before its first product: addresses, the first two K/V tiles on their way into the
    // four buffers (all free: every wavefront is behind the barrier of the previous tile's last step), its Q rows on
    // their way into registers.
    auto request = [&](const Item& it) {
        const int b = it.bh / p.H;
        const int h = it.bh - b * p.H;
        const int hk = h / p.kv_group;
        const int64_t base = (int64_t)b * p.stride_b + (int64_t)h * p.stride_h;
        const int64_t kv_base = (int64_t)b * p.kv_stride_b + (int64_t)hk * p.kv_stride_h;
        gk = static_cast<const T*>(p.k) + kv_base;
        gv = static_cast<const T*>(p.v) + kv_base;
        go = static_cast<T*>(p.o) + base;
        cur_bh = it.bh;
        q_tile0 = it.qt * ROWS;
        int k_end = L;
        if (CAUSAL) k_end = (q_tile0 + ROWS) < L ? (q_tile0 + ROWS) : L;
        n_tiles = (k_end + kFlashKeys - 1) / kFlashKeys;
        k_next = gk;
        v_next = gv;
        rem_next = (int64_t)(L - 1) * skv * 2 + 2 * d_real;  // the last row ends with its own d
        dma_next(lds_k0, lds_v0);
        dma_next(lds_k1, lds_v1);  // (a tile that starts at or behind the end of the sequence touches no memory and lands as zeros)
        qw = q_tile0 + wave * 32;
        qw_u = q_tile0 + wave_u * 32;
        qrow = qw + col;
        const int row = qrow < L ? qrow : L - 1;
        const T* src = static_cast<const T*>(p.q) + base + (int64_t)row * sn + 8 * half;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            qreg[ks] = 16 * ks + 8 * half < d_real ? *reinterpret_cast<const u32x4*>(src + 16 * ks) : u32x4{0u, 0u, 0u, 0u};
    };

    // The finished tile's output rows wait in registers until the next tile's first barrier is behind the wavefront:
    // stores issued in front of that barrier's wait would be waited for with the tile requests.
    constexpr int kRowsPerStore = 64 / CH, kStores = 32 / kRowsPerStore;
    u32x4 pending[kStores];
    T* pending_out = nullptr;
    int pending_row0 = 0;
    auto store_pending = [&]() {
        const int ch = lane % CH;
#pragma unroll
        for (int j = 0; j < kStores; ++j) {
            const int row = pending_row0 + j * kRowsPerStore + lane / CH;
            if (row < L && 8 * ch < d_real) *reinterpret_cast<u32x4*>(pending_out + (int64_t)row * sn + 8 * ch) = pending[j];
        }
    };

    Item item;
    if (!advance(item)) return;
    request(item);
    for (;;) {
        // ---- Q^T operands: pre-multiplied by c = scale*log2(e), kept for the whole query tile --------
        {
            const float c = p.scale_log2;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const u32x4 raw = qreg[ks];
                u32x4 sc;
#pragma unroll
                for (int w = 0; w < 4; ++w) sc[w] = pack2<T>(lo_f32<T>(raw[w]) * c, hi_f32<T>(raw[w]) * c);
                qreg[ks] = sc;
            }
        }
        // ---- running state (log2 units; see flash_fwd_mfma.hpp) --------------------------------------------------
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
        constexpr float kRaise = 8.0f;  // raise the reference maximum only when exceeded by 2^8

        auto compute_tile = [&](const unsigned char* tile_k, const unsigned char* tile_v, int k0) {
            // ---- S^T = c*K Q^T - m  (log2 units) -----------------------------------------------------------------
            f32x16 s[2];
            set_priority(true);
            {
                u32x4 a0[KS], a1[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    a0[ks] = lds_read_b128(tile_k + k_off[ks]);
                    a1[ks] = lds_read_b128(tile_k + 32 * RB + k_off[ks]);
                }
                s[0] = mfma_32x32x16<T>(a0[0], qreg[0], neg_m);
                s[1] = mfma_32x32x16<T>(a1[0], qreg[0], neg_m);
#pragma unroll
                for (int ks = 1; ks < KS; ++ks) {
                    s[0] = mfma_32x32x16<T>(a0[ks], qreg[ks], s[0]);
                    s[1] = mfma_32x32x16<T>(a1[ks], qreg[ks], s[1]);
                }
                constexpr int kAhead = KS < 4 ? KS : 4;
                __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);  // LDS reads
#pragma unroll
                for (int i = 0; i < KS - kAhead; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // matrix instructions
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                }
#pragma unroll
                for (int i = 0; i < kAhead; ++i) __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            }
            // V operands of the first 16 keys: requested now, used after the softmax arithmetic
            u32x2 vf[4][MB][2];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                vf[0][mb][0] = TrRead<T>::load(tile_v + v_off[mb]);
                vf[0][mb][1] = TrRead<T>::load(tile_v + v_off[mb] + 8 * RB);
            }
            set_priority(false);
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
            // ---- reference maximum: exact on the first tile, afterwards raised only when a score tops it by more
            //      than kRaise (rare, and the only time the accumulators are rescaled) ---------------------------
            float mx = fmaxf(s[0][0], s[1][0]);
#pragma unroll
            for (int r = 1; r < 16; ++r) mx = max3(mx, s[0][r], s[1][r]);
            if (first || __builtin_amdgcn_ballot_w64(mx > kRaise) != 0) {
                mx = halves_max(mx);  // both lanes of a query agree
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
                const float nm = neg_m[0] - delta;
#pragma unroll
                for (int r = 0; r < 16; ++r) neg_m[r] = nm;
                first = false;
            }
            // ---- P^T = exp2(S^T) packed as B operands (row sums in fp32), and O^T += V^T P^T, 16 keys at a time ----
            u32x4 pb[4];
            float sum = 0.0f;
            auto make_pb = [&](int g) {
                const int kb = g >> 1, r0 = 8 * (g & 1);
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const float p0 = fast_exp2(s[kb][r0 + 2 * w]), p1 = fast_exp2(s[kb][r0 + 2 * w + 1]);
                    pb[g][w] = pack2<T>(p0, p1);
                    sum += p0 + p1;
                }
#if defined(__HIP_DEVICE_COMPILE__)
                // the additions stay with their group of keys (left alone, the compiler sinks all of them behind the last
                // matrix instruction, where nothing overlaps them)
                asm volatile("" : "+v"(sum));
#endif
            };
            make_pb(0);
            set_priority(true);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    oacc[mb] = mfma_32x32x16<T>(u32x4{vf[g][mb][0][0], vf[g][mb][0][1], vf[g][mb][1][0], vf[g][mb][1][1]},
                                                pb[g], oacc[mb]);
                if (g < 3) {
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        vf[g + 1][mb][0] = TrRead<T>::load(tile_v + v_off[mb] + (16 * (g + 1)) * RB);
                        vf[g + 1][mb][1] = TrRead<T>::load(tile_v + v_off[mb] + (16 * (g + 1) + 8) * RB);
                    }
                    make_pb(g + 1);
                    // the order of issue: behind every matrix instruction two operand reads for the next 16 keys and a
                    // share of their exponentials (left to itself the compiler bunches the matrix instructions)
#pragma unroll
                    for (int i = 0; i < MB; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // matrix instruction
                        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // LDS reads
                        __builtin_amdgcn_sched_group_barrier(0x402, 4, 0);  // vector arithmetic, exponentials included
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            set_priority(false);
            l_run += sum;
        };

        // One key tile.  Tile t + 1 streams into the other buffer pair meanwhile (tile 1 is already on its way when the
        // walk starts); every step ends with a wait and a barrier, the last one too: behind it the buffers are free.
        auto step = [&](unsigned char* cur_k, unsigned char* cur_v, unsigned char* nxt_k, unsigned char* nxt_v, int t) {
            const int k0 = t * kFlashKeys;
            if (t > 0 && t + 1 < n_tiles) dma_next(nxt_k, nxt_v);
            // a wavefront whose queries all precede this tile has nothing to add
            if (!(CAUSAL && k0 > qw_u + 31)) compute_tile(cur_k, cur_v, k0);
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
        };

        __builtin_amdgcn_s_waitcnt(0);  // the first tiles and Q
        __syncthreads();
        if (pending_out) store_pending();
        for (int t = 0; t < n_tiles; t += 2) {
            step(lds_k0, lds_v0, lds_k1, lds_v1, t);
            if (t + 1 < n_tiles) step(lds_k1, lds_v1, lds_k0, lds_v0, t + 1);
        }

        // ---- the next query tile's requests leave before this one is written out ----------------------------------
        T* const out = go;
        const int out_row0 = qw;  // first output row of this wavefront
        const int out_bh = cur_bh;
        Item next;
        const bool more = advance(next);
        if (more) request(next);

        // ---- normalise, exchange through this wavefront's stretch of LDS, store whole rows -------------------------
        // A lane holds its query's 4 runs of 4 consecutive d per 32-row block of O^T; as 8-byte pieces at
        // row = query, 16-byte chunk (4 mb + g4) ^ (query % CH) they are written free of all but two-way bank conflicts,
        // and read back 16 bytes per lane, 64 / CH rows per instruction.
        {
            const float l = halves_sum(l_run);
            const float inv = l > 0.0f ? 1.0f / l : 0.0f;
            if (p.keep_neg_lse2 != nullptr && half == 0 && out_row0 + col < L)  // (FlashParams::keep_neg_lse2)
                p.keep_neg_lse2[(int64_t)out_bh * p.keep_rows + out_row0 + col] = l > 0.0f ? neg_m[0] - __builtin_log2f(l) : -INFINITY;
            unsigned char* const mine = lds_out + wave_u * (32 * RB);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const f32x16& a = oacc[mb];
                    const u32x2 w = u32x2{pack2<T>(a[4 * g4 + 0] * inv, a[4 * g4 + 1] * inv),
                                          pack2<T>(a[4 * g4 + 2] * inv, a[4 * g4 + 3] * inv)};
                    *reinterpret_cast<u32x2*>(mine + col * RB + (((4 * mb + g4) ^ (col & (CH - 1))) << 4) + 8 * half) = w;
                }
            // (the wavefront's own LDS instructions execute in order: no workgroup barrier between its writes and reads)
            __builtin_amdgcn_wave_barrier();
            const int ch = lane % CH;
#pragma unroll
            for (int j = 0; j < kStores; ++j) {
                const int r = j * kRowsPerStore + lane / CH;
                pending[j] = *reinterpret_cast<const u32x4*>(mine + r * RB + ((ch ^ (r & (CH - 1))) << 4));
            }
            pending_out = out;
            pending_row0 = out_row0;
        }
        if (!more) break;
    }
    store_pending();
}

}  // namespace ahpc
