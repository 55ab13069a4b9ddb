// PagedAttention decode for grouped query heads on the gfx950 matrix cores.
//
// With G query heads per pool head the G dot products per K element are what bounds the lane-per-element
// decode kernel (the K/V bytes drop by G, the arithmetic does not).  Here the G query heads of a pool head
// become the columns of the flash-forward formulation: a workgroup is one wavefront that owns one
// (batch entry, pool head, chunk of the context); per tile of 32 tokens
//     S^T = K Q^T        A = the tile's K rows from LDS, B = the group's queries (columns >= G are zero),
//     P^T = exp2(S^T - m) online softmax, one query head per lane column,
//     O^T += V^T P^T     A = V^T by transposing LDS reads, B = P^T from the registers S^T was in.
// Only G of the 32 result columns carry work; the matrix cores have time to spare, because the kernel is
// bound by the K/V stream: 16 matrix instructions per 16 KiB of K and V at d = 128.
//
// The LDS reads are asm with their own wait (tr_read_async, lds_read_b128_async): the compiler would otherwise put
// every LDS read behind all direct-to-LDS loads in flight, and the tile on its way could not overlap the tile in hand.
//
// The tile is gathered through the block table with direct-to-LDS loads, one instruction per 1 KiB of a page
// (pages hold 16 tokens): the page id is a lane-uniform readlane, the base address of the instruction a
// scalar, the per-lane offsets constants.  Two tiles are in flight (one being consumed, one on its way).
// Output: the same (m, l, o) partials per chunk as the lane-per-element kernel, or O itself when the
// context is a single chunk.
//
// Included by paged.hip after DecodeParams and the q/o vector helpers it uses.
#pragma once

#include "flash_fwd_mfma.hpp"

namespace ahpc {

constexpr int kDecodeTile = 32;  // tokens per tile

template <typename T, int D>
__global__ __launch_bounds__(64) void paged_decode_mfma_kernel(const DecodeParams p) {
    typedef FlashTile<D> TL;
    constexpr int KS = D / 16;
    constexpr int MB = D / 32;
    constexpr int RB = TL::kRowBytes;
    constexpr int RPI = TL::kRowsPerInstr;          // token rows one load instruction covers
    constexpr int NI = kDecodeTile / RPI;           // load instructions per tile (K or V)
    constexpr int kTileBytes = kDecodeTile * RB;
    constexpr int P = 16;

    __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[kTileBytes];

    const int lane = threadIdx.x;
    const int col = lane & 31;   // query head of the group (columns >= G idle) / token row of an A operand
    const int half = lane >> 5;
    const int hk = blockIdx.x;
    const int chunk = blockIdx.y;
    const int b = blockIdx.z;
    const int G = p.H / p.H_kv;
    const bool head_ok = col < G;
    const int hq = hk * G + (head_ok ? col : 0);

    const int64_t row = p.batch_rows ? p.batch_rows[b] : b;
    const int L = p.seq_lens[row] < p.max_len ? p.seq_lens[row] : p.max_len;
    const int chunk_len = decode_chunk_len(p, L, P);  // the sequence's own, equal chunks
    const int t0 = chunk * chunk_len;
    const int first_page = t0 / P;
    int my_page = 0;
    if (first_page + lane < p.max_pages) my_page = p.table[row * p.max_pages + first_page + lane];
    if (t0 >= L) {
        // an empty sequence still owns an output row: zeros (with several chunks the merge writes it)
        if (chunk == 0 && p.n_chunks == 1 && head_ok) {
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

    // ---- Q^T operands of this lane's query head, pre-multiplied by scale*log2(e) ---------------------
    u32x4 qreg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        float x[8];
        load_qo_vec<8>(p.q, p.qo_dtype, ((int64_t)b * p.H + hq) * D + 16 * ks + 8 * half, x);
        const float c = head_ok ? p.scale_log2 : 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) qreg[ks][w] = pack2<T>(x[2 * w] * c, x[2 * w + 1] * c);
    }

    // ---- gather: per-lane byte offsets inside the span of one load instruction ------------------------
    const int tok_bytes = p.H_kv * D * (int)sizeof(T);
    int off_k[NI], off_v[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int r = i * RPI + lane / TL::kChunks;  // token row inside the tile
        const int pc = lane % TL::kChunks;
        off_k[i] = (lane / TL::kChunks) * tok_bytes + ((pc ^ TL::fk(r)) << 4);
        off_v[i] = (lane / TL::kChunks) * tok_bytes + ((pc ^ TL::fv(r)) << 4);
    }
    const unsigned char* const kpool = static_cast<const unsigned char*>(p.k_pool);
    const unsigned char* const vpool = static_cast<const unsigned char*>(p.v_pool);
    auto gather_tile = [&](int tile, unsigned char* dst_k, unsigned char* dst_v) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int ti = tile * kDecodeTile + i * RPI;  // chunk-relative token of the instruction's first row
            const int page_id = __builtin_amdgcn_readlane(my_page, ti >> 4);
            const int64_t byte0 = (((int64_t)page_id * P + (ti & 15)) * p.H_kv + hk) * (int64_t)(D * (int)sizeof(T));
            // Token rows at or beyond the end of the chunk are outside the descriptor and land as zeros: what the
            // pool holds there may be any bit pattern, and 0 * NaN in the second product would poison the row.
            // (An instruction with no token row left touches no memory, whatever its page id is.)
            const int rows = n_tok - ti;
            const int rc = rows < RPI ? rows : RPI;  // token rows of this instruction that exist (may be <= 0)
            const unsigned nrec = rc > 0 ? (unsigned)((rc - 1) * tok_bytes + 2 * D) : 0u;  // bytes it may touch
            dma_instr(kpool + byte0, nrec, off_k[i], dst_k + i * 1024);
            dma_instr(vpool + byte0, nrec, off_v[i], dst_v + i * 1024);
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
        // token = tile*32 + 4*half + 8*(r/4) + r%4 exists iff it is below n_tok
        const int lim = n_tok - tile * kDecodeTile - 4 * half;
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int off = 8 * (r >> 2) + (r & 3);
            s[r] = off < lim ? s[r] : -INFINITY;
            mx = fmaxf(mx, s[r]);
        }
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

    auto step = [&](unsigned char* cur_k, unsigned char* cur_v, unsigned char* nxt_k, unsigned char* nxt_v, int t) __attribute__((always_inline)) {
        const bool more = t + 1 < n_tiles;
        if (more) gather_tile(t + 1, nxt_k, nxt_v);
        compute_tile(cur_k, cur_v, t);
        if (more) {
            __builtin_amdgcn_s_waitcnt(0);  // the next tile has landed
            __syncthreads();                // (one wavefront: only orders the LDS accesses around the loads)
        }
    };

    if (n_tiles > 0) gather_tile(0, lds_k0, lds_v0);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    for (int t = 0; t < n_tiles; t += 2) {
        step(lds_k0, lds_v0, lds_k1, lds_v1, t);
        if (t + 1 < n_tiles) step(lds_k1, lds_v1, lds_k0, lds_v0, t + 1);
    }

    const float l = halves_sum(l_run);
    if (!head_ok) return;
    if (p.n_chunks == 1) {
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const f32x16& a = oacc[mb];
                const float res[4] = {a[4 * g4 + 0] * inv, a[4 * g4 + 1] * inv, a[4 * g4 + 2] * inv, a[4 * g4 + 3] * inv};
                store_qo_vec<4>(p.o, p.qo_dtype, ((int64_t)b * p.H + hq) * D + 32 * mb + 8 * g4 + 4 * half, res);
            }
    } else {
        const int64_t slot = ((int64_t)b * p.n_chunks + chunk) * p.H + hq;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const f32x16& a = oacc[mb];
                *reinterpret_cast<f32x4*>(p.part_o + slot * D + 32 * mb + 8 * g4 + 4 * half) =
                    f32x4{a[4 * g4 + 0], a[4 * g4 + 1], a[4 * g4 + 2], a[4 * g4 + 3]};
            }
        if (half == 0) {
            p.part_ml[slot * 2] = m_run;
            p.part_ml[slot * 2 + 1] = stopped ? -l : l;  // the merge stops after a chunk that met a missing page
        }
    }
}

}  // namespace ahpc
