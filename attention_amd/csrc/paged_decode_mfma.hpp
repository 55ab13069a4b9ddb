// PagedAttention decode for grouped query heads on the gfx950 matrix cores.
//
// With G query heads per pool head the G dot products per K element are what bounds the lane-per-element
// decode kernel (the K/V bytes drop by G, the arithmetic does not).  Here the G query heads of a pool head
// become the columns of the flash-forward formulation: a workgroup of W wavefronts owns one (batch entry, pool
// head, chunk of the context) and shares the chunk's tiles of 32 tokens out (wavefront w: tiles w, w + W, ...);
// per tile
//     S^T = K Q^T        A = the tile's K rows from LDS, B = the group's queries (columns >= G are zero),
//     P^T = exp2(S^T - m) online softmax, one query head per lane column,
//     O^T += V^T P^T     A = V^T by transposing LDS reads, B = P^T from the registers S^T was in.
// Only G of the 32 result columns carry work; the matrix cores have time to spare, because the kernel is
// bound by the K/V stream: 16 matrix instructions per 16 KiB of K and V at d = 128.  What is not to spare is
// instruction issue: a wavefront alone on its SIMD issues every four cycles at best, so the tile loop is kept
// short (one descriptor pair per page, the end-of-sequence mask in a chunk's last tile only, accumulators in
// ordinary registers: the launch bound keeps the kernel within 256).
//
// The LDS reads are asm with their own wait (tr_read_async, lds_read_b128_async): the compiler would otherwise put
// every LDS read behind all direct-to-LDS loads in flight, and the tile on its way could not overlap the tile in hand.
//
// The tile is gathered through the block table with direct-to-LDS loads, one instruction per 1 KiB of a page
// (pages hold 16 tokens): the page id is a lane-uniform readlane, the base address of a page a scalar, the per-lane
// offsets constants.  Every wavefront has two tile slots of its own (one being consumed, one on its way) and
// never waits for another before the end, where the W results (m, l, O) pass through LDS and become one.
// Output: the same (m, l, o) partials per chunk as the lane-per-element kernel, or O itself when the
// context is a single chunk.
//
// Included by paged.hip after DecodeParams and the q/o vector helpers it uses.
#pragma once

#include "flash_fwd_mfma.hpp"

namespace ahpc {

constexpr int kDecodeTile = 32;  // tokens per tile

template <typename T, int D, int W>
__global__ __launch_bounds__(64 * W, D <= 128 ? 2 : 1) void paged_decode_mfma_kernel(const DecodeParams p) {
    typedef FlashTile<D> TL;
    constexpr int KS = D / 16;
    constexpr int MB = D / 32;
    constexpr int RB = TL::kRowBytes;
    constexpr int RPI = TL::kRowsPerInstr;          // token rows one load instruction covers
    constexpr int NI = kDecodeTile / RPI;           // load instructions per tile (K or V)
    constexpr int kTileBytes = kDecodeTile * RB;
    constexpr int P = 16;

    static_assert(W * 4 * kTileBytes <= 160 * 1024, "two tiles (K and V) per wavefront in LDS");
    __shared__ __attribute__((aligned(1024))) unsigned char lds_all[W * 4 * kTileBytes];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    unsigned char* const lds_k0 = lds_all + wave * (4 * kTileBytes);  // this wavefront's own two tile slots
    unsigned char* const lds_v0 = lds_k0 + kTileBytes;
    unsigned char* const lds_k1 = lds_k0 + 2 * kTileBytes;
    unsigned char* const lds_v1 = lds_k0 + 3 * kTileBytes;
    const int col = lane & 31;   // query head of the group (columns >= G idle) / token row of an A operand
    const int half = lane >> 5;
    const int hk = blockIdx.x;
    const int chunk = blockIdx.y;
    const int b = blockIdx.z;
    const int G = p.H / p.H_kv;
    const bool head_ok = col < G;
    const int hq = hk * G + (head_ok ? col : 0);

    // ---- Q^T of this lane's query head: requested first of all (it travels beside the length, the table row and
    // the first tile), converted behind the first tile's requests
    QRaw<KS> qraw;
    q_request<KS>(qraw, p.q, p.qo_dtype, ((int64_t)b * p.H + hq) * D + 8 * half, 16);
    u32x4 qreg[KS];

    const int64_t row = p.batch_rows ? p.batch_rows[b] : b;
    const int L = p.seq_lens[row] < p.max_len ? p.seq_lens[row] : p.max_len;
    const int chunk_len = decode_chunk_len(p, L, P);  // the sequence's own, equal chunks
    const int t0 = chunk * chunk_len;
    const int first_page = t0 / P;
    int my_page = 0;
    if (first_page + lane < p.max_pages) my_page = p.table[row * p.max_pages + first_page + lane];
    if (t0 >= L) {
        // an empty sequence still owns an output row: zeros (with several chunks the merge writes it)
        if (chunk == 0 && p.n_chunks == 1 && head_ok && wave == 0) {
            const float zero[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4)
                    store_qo_vec<4>(p.o, p.qo_dtype, ((int64_t)b * p.H + hq) * D + 32 * mb + 8 * g4 + 4 * half, zero);
        }
        return;
    }
    int t1 = (t0 + chunk_len) < L ? (t0 + chunk_len) : L;
    // a missing page (-1) inside the sequence ends it there (see paged_decode_kernel): the chunk stops in front of it
    const unsigned long long missing = __builtin_amdgcn_ballot_w64(lane < (t1 - t0 + P - 1) / P && my_page < 0);
    const bool stopped = missing != 0;
    if (stopped) {
        const int cut = t0 + (int)__builtin_ctzll(missing) * P;
        t1 = cut < t1 ? cut : t1;
    }
    my_page = my_page < 0 ? 0 : my_page;  // never dereferenced: no token row of such a page is left in the chunk
    const int n_tok = t1 - t0;            // 0 when the chunk's first page is missing
    const int n_tiles = (n_tok + kDecodeTile - 1) / kDecodeTile;

    // ---- gather: per-lane byte offsets inside the span of one load instruction ------------------------
    const int tok_bytes = p.H_kv * D * (int)sizeof(T);
    constexpr int IPP = P / RPI;  // load instructions per page (K or V)
    static_assert(P % RPI == 0 && kDecodeTile % P == 0, "whole instructions per page, whole pages per tile");
    int off_k[NI], off_v[NI];  // relative to the first token row of the instruction's page
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int r = i * RPI + lane / TL::kChunks;  // token row inside the tile
        const int pc = lane % TL::kChunks;
        off_k[i] = (r % P) * tok_bytes + ((pc ^ TL::fk(r)) << 4);
        off_v[i] = (r % P) * tok_bytes + ((pc ^ TL::fv(r)) << 4);
    }
    const unsigned char* const kpool = static_cast<const unsigned char*>(p.k_pool);
    const unsigned char* const vpool = static_cast<const unsigned char*>(p.v_pool);
    // One descriptor pair per page: the scalar unit forms an address and a size once per 16 tokens, and the
    // instructions of a page differ in their per-lane offsets only (a wavefront that works alone on its SIMD
    // issues an instruction every four cycles at best, so every scalar instruction here is time of the tile).
    auto gather_tile = [&](int tile, unsigned char* dst_k, unsigned char* dst_v) __attribute__((always_inline)) {
#pragma unroll
        for (int pg = 0; pg < kDecodeTile / P; ++pg) {
            const int pi = tile * (kDecodeTile / P) + pg;  // chunk-relative page
            const int page_id = __builtin_amdgcn_readlane(my_page, pi);
            const int64_t byte0 = ((int64_t)page_id * P * p.H_kv + hk) * (int64_t)(D * (int)sizeof(T));
            // Token rows at or beyond the end of the chunk are outside the descriptor and land as zeros: what the
            // pool holds there may be any bit pattern, and 0 * NaN in the second product would poison the row.
            // (A page with no token row left touches no memory, whatever its page id is.)
            const int rows = n_tok - pi * P;
            const int rc = rows < P ? rows : P;  // token rows of this page that exist (may be <= 0)
            const unsigned nrec = rc > 0 ? (unsigned)((rc - 1) * tok_bytes + D * (int)sizeof(T)) : 0u;  // bytes it may touch
#pragma unroll
            for (int j = 0; j < IPP; ++j) {
                const int i = pg * IPP + j;
                dma_instr<2>(kpool + byte0, nrec, off_k[i], dst_k + i * 1024);  // non-temporal: every line is used once
                dma_instr<2>(vpool + byte0, nrec, off_v[i], dst_v + i * 1024);
            }
        }
    };

    // ---- LDS operand addresses -----------------------------------------------------------------------
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

    f32x16 oacc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[mb][r] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;

    auto compute_tile = [&](const unsigned char* tile_k, const unsigned char* tile_v, int tile) __attribute__((always_inline)) {
        f32x16 s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.0f;
        {
            u32x4 ka[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) ka[ks] = lds_read_b128_async<0>(tile_k + k_off[ks]);
            b128_wait(ka);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) s = mfma_32x32x16<T>(ka[ks], qreg[ks], s);
        }
        // token = tile*32 + 4*half + 8*(r/4) + r%4 exists iff it is below n_tok: only a chunk's last tile can hold others
        if (n_tok - tile * kDecodeTile < kDecodeTile) {
            const int lim = n_tok - tile * kDecodeTile - 4 * half;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int off = 8 * (r >> 2) + (r & 3);
                s[r] = off < lim ? s[r] : -INFINITY;
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[r]);
        // The reference maximum is raised only when a score tops it by more than 2^8 (and on the first tile):
        // p stays in (0, 256], O/l is unchanged, and the accumulators are rescaled rarely.
        if (__builtin_amdgcn_ballot_w64(mx > m_run + 8.0f) != 0) {  // always on the first tile: m_run is -inf there
            mx = halves_max(mx);  // a tile holds at least one token, so this is finite
            const float m_new = fmaxf(m_run, mx);
            const float alpha = fast_exp2(m_run - m_new);  // first tile: exp2(-inf) = 0
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[mb][r] *= alpha;
        }
        const float m_new = m_run;
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            s[r] = fast_exp2(s[r] - m_new);
            sum += s[r];
        }
        l_run += sum;
#pragma unroll
        for (int g2 = 0; g2 < 2; ++g2) {
            const u32x4 pb = u32x4{pack2<T>(s[8 * g2 + 0], s[8 * g2 + 1]), pack2<T>(s[8 * g2 + 2], s[8 * g2 + 3]),
                                   pack2<T>(s[8 * g2 + 4], s[8 * g2 + 5]), pack2<T>(s[8 * g2 + 6], s[8 * g2 + 7])};
            u32x2 vt[2 * MB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                vt[2 * mb] = tr_read_async<T, 0>(tile_v + v_off[mb] + (16 * g2) * RB);
                vt[2 * mb + 1] = tr_read_async<T, 0>(tile_v + v_off[mb] + (16 * g2 + 8) * RB);
            }
            tr_wait(vt);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                oacc[mb] = mfma_32x32x16<T>(u32x4{vt[2 * mb][0], vt[2 * mb][1], vt[2 * mb + 1][0], vt[2 * mb + 1][1]}, pb, oacc[mb]);
        }
    };

    // The W wavefronts of the workgroup share the chunk's tiles out among themselves (wavefront w takes tiles w, w + W,
    // ...: neighbouring tiles are in flight together) and never wait for each other before the end; each keeps its own
    // (m, l, O).  The waits below are the wavefront's own: its loads complete in order, and the LDS reads are asm
    // statements that the compiler keeps where they stand.
    const int my_tiles = n_tiles > wave ? (n_tiles - wave + W - 1) / W : 0;
    auto step = [&](unsigned char* cur_k, unsigned char* cur_v, unsigned char* nxt_k, unsigned char* nxt_v, int i) __attribute__((always_inline)) {
        const bool more = i + 1 < my_tiles;
        if (more) gather_tile(wave + (i + 1) * W, nxt_k, nxt_v);
        compute_tile(cur_k, cur_v, wave + i * W);
        if (more) {
            __builtin_amdgcn_s_waitcnt(0);  // the next tile has landed
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    if (my_tiles > 0) gather_tile(wave, lds_k0, lds_v0);

    q_convert<T, KS>(qraw, p.qo_dtype, head_ok ? p.scale_log2 : 0.0f, qreg);  // pre-multiplied by scale*log2(e)
    __builtin_amdgcn_s_waitcnt(0);
    __builtin_amdgcn_sched_barrier(0);
    for (int i = 0; i < my_tiles; i += 2) {
        step(lds_k0, lds_v0, lds_k1, lds_v1, i);
        if (i + 1 < my_tiles) step(lds_k1, lds_v1, lds_k0, lds_v0, i + 1);
    }

    float l = halves_sum(l_run);
    if constexpr (W > 1) {
        // ---- the wavefronts' results become one: (m, l, O) of each go through its own tile slots (all its loads have
        // landed and its LDS reads have returned), and wavefront w merges the row blocks mb = w, w + W, ... of O ----
        static_assert(4 * kTileBytes >= MB * 4 * 1024 + 512, "a wavefront's partial fits its tile slots");
        unsigned char* const mine = lds_k0;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4)
                *reinterpret_cast<f32x4*>(mine + ((mb * 4 + g4) * 64 + lane) * 16) =
                    f32x4{oacc[mb][4 * g4 + 0], oacc[mb][4 * g4 + 1], oacc[mb][4 * g4 + 2], oacc[mb][4 * g4 + 3]};
        *reinterpret_cast<f32x2*>(mine + MB * 4 * 1024 + lane * 8) = f32x2{m_run, l};
        __syncthreads();
        float mw[W], lw[W];
        float m_all = -INFINITY;
#pragma unroll
        for (int w = 0; w < W; ++w) {
            const f32x2 ml = *reinterpret_cast<const f32x2*>(lds_all + w * (4 * kTileBytes) + MB * 4 * 1024 + lane * 8);
            mw[w] = ml[0];
            lw[w] = ml[1];
            m_all = fmaxf(m_all, mw[w]);
        }
        l = 0.0f;
#pragma unroll
        for (int w = 0; w < W; ++w) {
            mw[w] = mw[w] == -INFINITY ? 0.0f : fast_exp2(mw[w] - m_all);  // a wavefront without a tile weighs nothing
            l += mw[w] * lw[w];
        }
        m_run = m_all;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            if (mb % W != wave) continue;
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                f32x4 acc = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int w = 0; w < W; ++w) {
                    const f32x4 x = *reinterpret_cast<const f32x4*>(lds_all + w * (4 * kTileBytes) + ((mb * 4 + g4) * 64 + lane) * 16);
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e] += mw[w] * x[e];
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) oacc[mb][4 * g4 + e] = acc[e];
            }
        }
    }
    if (!head_ok) return;
    if (p.n_chunks == 1) {
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            if (mb % W != wave) continue;
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const f32x16& a = oacc[mb];
                const float res[4] = {a[4 * g4 + 0] * inv, a[4 * g4 + 1] * inv, a[4 * g4 + 2] * inv, a[4 * g4 + 3] * inv};
                store_qo_vec<4>(p.o, p.qo_dtype, ((int64_t)b * p.H + hq) * D + 32 * mb + 8 * g4 + 4 * half, res);
            }
        }
    } else {
        const int64_t slot = ((int64_t)b * p.n_chunks + chunk) * p.H + hq;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            if (mb % W != wave) continue;
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const f32x16& a = oacc[mb];
                *reinterpret_cast<f32x4*>(p.part_o + slot * D + 32 * mb + 8 * g4 + 4 * half) =
                    f32x4{a[4 * g4 + 0], a[4 * g4 + 1], a[4 * g4 + 2], a[4 * g4 + 3]};
            }
        }
        if (half == 0 && wave == 0) {
            p.part_ml[slot * 2] = m_run;
            p.part_ml[slot * 2 + 1] = stopped ? -l : l;  // the merge stops after a chunk that met a missing page
        }
    }
}

}  // namespace ahpc
