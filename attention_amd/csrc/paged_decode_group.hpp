// PagedAttention decode for grouped query heads (2 to 16 query heads per pool head) on the gfx950 matrix cores,
// page by page.
//
// A wavefront owns one (batch entry, pool head, chunk of the context); the wavefronts of a workgroup take
// neighbouring pool heads, so that a workgroup reads whole token rows, and never talk to each other (no barrier).
// Per page of 16 tokens
//     S^T = K Q^T        16x16x32 matrix instructions; A = the page's K rows (lane = token, 16 bytes of its row per
//                        instruction), B = the group's queries, pre-scaled (columns >= G are zero),
//     P^T = exp2(S^T - m) online softmax, one query head per lane column, 4 tokens per lane,
//     O^T += V^T P^T     16x16x16 matrix instructions; A = V^T by transposing LDS reads, B = P^T exactly as the
//                        registers of S^T hold it.
// K and V of a page arrive in LDS by direct-to-LDS loads (one instruction per 1 KiB, whole cache lines), in one of
// two page slots per wavefront: one page is consumed while the next is on its way.  That is all the depth the
// memory system can use: a CU keeps about 90 cache-line requests in flight whatever the kernel asks for
// (counters: requests x latency / time), so what counts is that every request is a whole line asked for once.
// (Loading K straight into the operand registers - 64 bytes per token and instruction - makes two instructions
// share every line, and the vector cache asks the L2 for it twice: 3-4 % slower when timed.)
//
// The LDS reads are written as asm, with their own wait: the compiler orders every LDS read it knows of behind ALL
// direct-to-LDS loads in flight once a function holds more than a handful of them, which would serialise the two
// slots.  The direct loads stay builtins and complete in order; the explicit s_waitcnt leaves exactly the next
// page's loads outstanding.
//
// Output: the same (m, l, o) partials per chunk as the lane-per-element kernel, or O itself when the context is a
// single chunk.  A table entry of -1 inside a sequence ends it there (see paged_decode_kernel).
//
// Included by paged.hip after DecodeParams and the q/o vector helpers it uses.
#pragma once

#include <type_traits>

#include "flash_fwd_mfma.hpp"

namespace ahpc {

constexpr int kGroupRing = 2;  // page slots per wavefront
#ifndef AHPC_GROUP_AUX
#define AHPC_GROUP_AUX 2
#endif
constexpr int kStreamAux = AHPC_GROUP_AUX;  // cache policy of the K/V loads: 2 = non-temporal (every line is used once; worth 10 % when timed)

// s_waitcnt immediate that waits until at most N vector-memory loads are outstanding (gfx9 encoding; the other
// counters stay unconstrained).
constexpr int vmcnt_imm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }

// T: pool element type (16 bit).  D: head dimension (64, 128).  W: wavefronts (= pool heads) per workgroup.
template <typename T, int D, int W>
__global__ __launch_bounds__(64 * W) void paged_decode_group_kernel(const DecodeParams p) {
    constexpr int RB = 2 * D;          // bytes of one head of one token
    constexpr int CH = RB / 16;        // 16-byte pieces of such a row
    constexpr int RPI = 1024 / RB;     // token rows one direct-to-LDS instruction covers
    constexpr int NI = 16 / RPI;       // such instructions per page
    constexpr int KS = D / 32;         // matrix instructions of one S^T tile
    constexpr int MB = D / 16;         // 16-row blocks of O^T
    constexpr int R = kGroupRing;
    constexpr int kPart = 16 * RB;     // bytes of V (or K) of one page and head
    constexpr int kSlot = 2 * kPart;   // a page slot: V, then K
    constexpr int P = 16;
    constexpr int kOps = 2 * NI;       // loads per page and wavefront
    static_assert(D == 64 || D == 128 || D == 256, "head dimensions of this kernel");
    static_assert(W * R * kSlot <= 160 * 1024, "page slots of all wavefronts in LDS");

    __shared__ __attribute__((aligned(1024))) unsigned char lds_v[W * R * kSlot];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int col = lane & 15;  // query head of the group (B operands, results) / token of the page (A operand of S^T)
    const int rg = lane >> 4;   // which 8 (or 4) of an instruction's k values / which 4 result rows
    const int hk = (int)blockIdx.x * W + wave;
    if (hk >= p.H_kv) return;   // wavefronts are independent: nothing waits for this one
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
    int my_page = 0;  // lane i: id of page first_page + i (a chunk has at most 64 pages)
    if (first_page + lane < p.max_pages) my_page = p.table[row * p.max_pages + first_page + lane];
    if (t0 >= L) {
        // an empty sequence still owns an output row: zeros (with several chunks the merge writes it)
        if (chunk == 0 && p.n_chunks == 1 && head_ok) {
            const float zero[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) store_qo_vec<4>(p.o, p.qo_dtype, ((int64_t)b * p.H + hq) * D + 16 * mb + 4 * rg, zero);
        }
        return;
    }
    int t1 = (t0 + chunk_len) < L ? (t0 + chunk_len) : L;
    const unsigned long long missing = __builtin_amdgcn_ballot_w64(lane < (t1 - t0 + P - 1) / P && my_page < 0);
    const bool stopped = missing != 0;
    if (stopped) {
        const int cut = t0 + (int)__builtin_ctzll(missing) * P;
        t1 = cut < t1 ? cut : t1;
    }
    my_page = my_page < 0 ? 0 : my_page;  // never dereferenced: no token row of such a page is left in the chunk
    const int n_tok = t1 - t0;            // 0 when the chunk's first page is missing
    const int n_pages = (n_tok + P - 1) / P;

    // ---- Q^T operands: lane (query head col, rg) holds q[32*ks + 8*rg .. +7], times scale*log2(e) ------------
    u32x4 qreg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        float x[8];
        load_qo_vec<8>(p.q, p.qo_dtype, ((int64_t)b * p.H + hq) * D + 32 * ks + 8 * rg, x);
        const float c = head_ok ? p.scale_log2 : 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) qreg[ks][w] = pack2<T>(x[2 * w] * c, x[2 * w + 1] * c);
    }

    // ---- per-lane byte offsets from the first token row of a page (this head) ---------------------------------
    const int tok_bytes = p.H_kv * RB;
    // V lands row-major in its slot; a row's 16-byte pieces are stored permuted (piece c at position c ^ fv(row)), so
    // that the 8 rows which 32 lanes of a transposing read touch fall into different banks (64 banks of 4 bytes;
    // at d = 64 two rows make up one pass over the banks, and rows of equal parity must differ)
    auto fv = [](int r) { return D >= 128 ? 2 * (r & 3) + 8 * ((r >> 2) & 1) : 2 * ((r >> 1) & 3); };
    int v_off[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int r = i * RPI + lane / CH;
        v_off[i] = r * tok_bytes + (((lane % CH) ^ fv(r)) << 4);
    }
    // K: rows are read 16 bytes per lane, 16 rows by 16 lanes at a time: piece c of row r sits at c ^ fk(r)
    auto fk = [](int r) { return D >= 128 ? (r & 15) : ((r >> 1) & 7); };
    int kd_off[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int r = i * RPI + lane / CH;
        kd_off[i] = r * tok_bytes + (((lane % CH) ^ fk(r)) << 4);
    }
    unsigned char* const slot0 = lds_v + wave * (R * kSlot);
    // transposing reads: within 16 lanes, lane j asks for token 4*rg + j/4, elements 16*mb + 4*(j%4) .. +3, and
    // receives element 16*mb + j of tokens 4*rg .. 4*rg+3.  fv is even, so the piece index 2*mb + (j%4)/2 keeps
    // its lowest bit through the permutation.
    const unsigned char* v_rd[MB];
    {
        const int j = lane & 15;
        const int trow = 4 * rg + (j >> 2);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            v_rd[mb] = slot0 + trow * RB + (((2 * mb) ^ fv(trow)) << 4) + 16 * ((j >> 1) & 1) + 8 * (j & 1);
    }

    // lane (token col, rg) reads piece 4*ks + rg of its token's K row
    const unsigned char* k_rd[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_rd[ks] = slot0 + kPart + col * RB + (((4 * ks + rg) ^ fk(col)) << 4);

    const unsigned char* const kpool = static_cast<const unsigned char*>(p.k_pool);
    const unsigned char* const vpool = static_cast<const unsigned char*>(p.v_pool);

    // Requests page `tt` of the chunk into ring slot S.  Token rows at or beyond the end of the chunk (and whole
    // pages beyond it) lie outside the descriptor: they touch no memory and arrive as zeros.
    auto issue = [&](int tt, auto slot_c) __attribute__((always_inline)) {
        constexpr int S = decltype(slot_c)::value;
#if defined(__HIP_DEVICE_COMPILE__)
        const int page_id = __builtin_amdgcn_readlane(my_page, tt < n_pages ? tt : 0);
        const int rows = n_tok - tt * P;
        const int rc = rows < P ? rows : P;
        const unsigned nrec = rc > 0 ? (unsigned)((rc - 1) * tok_bytes + RB) : 0u;
        const int64_t byte0 = ((int64_t)page_id * P * p.H_kv + hk) * (int64_t)RB;
        const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(vpool + byte0), 0, nrec, 0x00020000);
#pragma unroll
        for (int i = 0; i < NI; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (AHPC_LDS void*)(slot0 + S * kSlot + i * 1024), 16, v_off[i], 0, 0, kStreamAux);
        const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(kpool + byte0), 0, nrec, 0x00020000);
#pragma unroll
        for (int i = 0; i < NI; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (AHPC_LDS void*)(slot0 + S * kSlot + kPart + i * 1024), 16, kd_off[i], 0, 0, kStreamAux);
#endif
        // the requests stay ahead of the arithmetic that follows: the wait count below is exact only as long as
        // nothing else slips in between
        __builtin_amdgcn_sched_barrier(0);
    };

    f32x4 oacc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) oacc[mb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY, l_run = 0.0f;

    auto consume = [&](int tt, auto slot_c, auto behind_c) __attribute__((always_inline)) {
        constexpr int S = decltype(slot_c)::value;
        // this page has landed once at most the loads of the page requested behind it are outstanding
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(decltype(behind_c)::value * kOps));
        u32x2 vt[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) vt[mb] = tr_read_async<T, S * kSlot>(v_rd[mb]);
        f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
        u32x4 ka[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) ka[ks] = lds_read_b128_async<S * kSlot>(k_rd[ks]);
        b128_wait(ka);  // (LDS answers in order: V's reads above are done as well)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = mfma_16x16x32<T>(ka[ks], qreg[ks], s);
        // s[r] belongs to token tt*16 + 4*rg + r, which exists iff it is below n_tok
        const int lim = n_tok - tt * P - 4 * rg;
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s[r] = r < lim ? s[r] : -INFINITY;
            mx = fmaxf(mx, s[r]);
        }
        // The reference maximum is raised only when a score tops it by more than 2^8 (and on the first page):
        // p stays in (0, 256], O/l is unchanged, and the accumulators are rescaled rarely.
        if (__builtin_amdgcn_ballot_w64(mx > m_run + 8.0f) != 0) {  // always on the first page: m_run is -inf there
            mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
            mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));  // the four lanes of a query head agree; finite: token 0 of a page exists
            const float m_new = fmaxf(m_run, mx);
            const float alpha = fast_exp2(m_run - m_new);  // first page: exp2(-inf) = 0
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 4; ++r) oacc[mb][r] *= alpha;
        }
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s[r] = fast_exp2(s[r] - m_run);
            sum += s[r];
        }
        l_run += sum;
        const u32x2 pb = u32x2{pack2<T>(s[0], s[1]), pack2<T>(s[2], s[3])};
        tr_wait(vt);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) oacc[mb] = mfma_16x16x16<T>(vt[mb], pb, oacc[mb]);
        __builtin_amdgcn_sched_barrier(0);
    };

    typedef std::integral_constant<int, 0> S0;
    typedef std::integral_constant<int, 1> S1;
    static_assert(R == 2, "the ring below is written out for two slots");
    // The steady loop has no way out in its middle: it requests even behind the last page (empty requests), so the
    // same number of loads is outstanding at every wait.
    int t = 0;
    issue(0, S0{});
    for (; t + R <= n_pages; t += R) {
        issue(t + 1, S1{});
        consume(t, S0{}, S1{});
        issue(t + 2, S0{});
        consume(t + 1, S1{}, S1{});
    }
    // a last odd page is in slot 0 already, with at most an empty request behind it; waiting for everything also keeps
    // that one (a zero fill) from outliving the wavefront's LDS
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    if (t < n_pages) consume(t, S0{}, S0{});

    float l = l_run + __shfl_xor(l_run, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    if (!head_ok) return;
    if (p.n_chunks == 1) {
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const float res[4] = {oacc[mb][0] * inv, oacc[mb][1] * inv, oacc[mb][2] * inv, oacc[mb][3] * inv};
            store_qo_vec<4>(p.o, p.qo_dtype, ((int64_t)b * p.H + hq) * D + 16 * mb + 4 * rg, res);
        }
    } else {
        const int64_t slot = ((int64_t)b * p.n_chunks + chunk) * p.H + hq;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) *reinterpret_cast<f32x4*>(p.part_o + slot * D + 16 * mb + 4 * rg) = oacc[mb];
        if (rg == 0) {
            p.part_ml[slot * 2] = m_run;
            p.part_ml[slot * 2 + 1] = stopped ? -l : l;  // the merge stops after a chunk that met a missing page
        }
    }
}

}  // namespace ahpc
