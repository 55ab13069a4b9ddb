// Paged KV pool kernels: scatter (append), gather (read-back), decode, split merge, index dump.
//
// Pool layout: K and V slabs [page][slot][head][d].  One token of one sequence is H*d contiguous
// elements, so a wavefront reads whole 1-KiB runs: lanes are grouped LPH = d*sizeof(T)/16 per head
// (each lane owns one 16-byte piece of a head's row) and a wavefront covers 64/LPH heads of one
// token with a single 16-byte load per lane.
#include <hip/hip_runtime.h>

#include <atomic>

#include <cmath>
#include <cstdlib>
#include <type_traits>

#include "ahpc_device.hpp"
#include "tuning.hpp"

namespace ahpc {

// Element offset of (token t, head 0, element 0) of table row `row`; -1 when the page is missing or the token
// lies beyond the row's last column.  Used by scatter and gather (append, read-back); the decode kernels do their
// own address arithmetic (one page id per lane, rows a fixed stride apart) and report it themselves when asked
// (DecodeParams::dump_offsets).
__device__ __forceinline__ int64_t kv_token_offset(const int32_t* __restrict__ table, int64_t max_pages, int64_t row,
                                                   int t, int P, int H, int d) {
    const int page_idx = t / P;
    const int pos = t - page_idx * P;
    if (page_idx >= max_pages) return -1;
    const int page_id = table[row * max_pages + page_idx];
    if (page_id < 0) return -1;
    return (((int64_t)page_id * P + pos) * H) * (int64_t)d;
}

// ---------------------------------------------------------------------------------------------
// scatter / gather: one thread per element pair (K and V), dtype conversion on the fly.
template <typename TI, typename TO>
__global__ void kv_scatter_kernel(const TI* __restrict__ k_new, const TI* __restrict__ v_new, TO* __restrict__ k_pool,
                                  TO* __restrict__ v_pool, const int32_t* __restrict__ table, int64_t max_pages,
                                  const int32_t* __restrict__ token_row, const int32_t* __restrict__ token_pos,
                                  int64_t row0, int64_t pos0, int64_t n_tokens, int H, int d, int P) {
    const int64_t hd = (int64_t)H * d;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_tokens * hd) return;
    const int64_t tok = idx / hd;
    const int64_t e = idx - tok * hd;
    const int64_t row = token_row ? token_row[tok] : row0;
    const int t = token_pos ? token_pos[tok] : (int)(pos0 + tok);
    if (row < 0 || t < 0) return;
    const int64_t off = kv_token_offset(table, max_pages, row, t, P, H, d);
    if (off < 0) return;
    Storage<TO>::store(k_pool + off + e, Storage<TI>::load(k_new + idx));
    Storage<TO>::store(v_pool + off + e, Storage<TI>::load(v_new + idx));
}

template <typename TI, typename TO>
__global__ void kv_gather_kernel(TO* __restrict__ k_out, TO* __restrict__ v_out, const TI* __restrict__ k_pool,
                                 const TI* __restrict__ v_pool, const int32_t* __restrict__ table, int64_t max_pages,
                                 int64_t row, int64_t start, int64_t n, int H, int d, int P) {
    const int64_t hd = (int64_t)H * d;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n * hd) return;
    const int64_t tok = idx / hd;
    const int64_t e = idx - tok * hd;
    const int64_t off = kv_token_offset(table, max_pages, row, (int)(start + tok), P, H, d);
    float kx = 0.0f, vx = 0.0f;
    if (off >= 0) {
        kx = Storage<TI>::load(k_pool + off + e);
        vx = Storage<TI>::load(v_pool + off + e);
    }
    Storage<TO>::store(k_out + idx, kx);
    Storage<TO>::store(v_out + idx, vx);
}

// Batched append: the K and V rows of many sequences in one launch, straight from the tensors a prefill
// just attended over.  One wavefront per (sequence, token) moves that token's two H*d rows; when source
// and pool share a type and everything is 16-byte aligned the rows go as 16-byte pieces (a pure copy at
// HBM speed), otherwise element by element with conversion.
struct ScatterBatchParams {
    const void* k_src;
    const void* v_src;
    void* k_pool;
    void* v_pool;
    const int32_t* table;
    const int32_t* seq_rows;    // [B] table row of sequence b
    const int32_t* seq_start;   // [B] position of its first new token, or null = 0
    const int32_t* seq_tokens;  // [B] number of new tokens, or null = N
    const int32_t* cu_seqlens;  // [B+1] packed source: sequence b owns source rows cu[b] .. cu[b+1]-1, or null
    int64_t max_pages;
    int64_t stride_b, stride_n;  // source strides in elements (stride_b unused with cu_seqlens)
    int32_t B, N, H, d, P;
};

template <typename TI, typename TO, bool VEC>
__global__ __launch_bounds__(256) void kv_scatter_batch_kernel(const ScatterBatchParams p) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int b = blockIdx.y;
    const int t = blockIdx.x * 4 + wave;
    int n_new = p.N;
    int64_t src_row0 = 0;
    if (p.cu_seqlens) {
        n_new = p.cu_seqlens[b + 1] - p.cu_seqlens[b];
        src_row0 = (int64_t)p.cu_seqlens[b] * p.stride_n;
    } else {
        if (p.seq_tokens) n_new = p.seq_tokens[b];
        src_row0 = (int64_t)b * p.stride_b;
    }
    if (t >= n_new) return;
    const int64_t row = p.seq_rows[b];
    if (row < 0) return;
    const int pos = (p.seq_start ? p.seq_start[b] : 0) + t;
    const int64_t dst = kv_token_offset(p.table, p.max_pages, row, pos, p.P, p.H, p.d);
    if (dst < 0) return;
    const int64_t src = src_row0 + (int64_t)t * p.stride_n;
    const int hd = p.H * p.d;
    if (VEC) {
        constexpr int EPV = 16 / (int)sizeof(TO);
        const u32x4* ks = reinterpret_cast<const u32x4*>(static_cast<const TI*>(p.k_src) + src);
        const u32x4* vs = reinterpret_cast<const u32x4*>(static_cast<const TI*>(p.v_src) + src);
        u32x4* kd = reinterpret_cast<u32x4*>(static_cast<TO*>(p.k_pool) + dst);
        u32x4* vd = reinterpret_cast<u32x4*>(static_cast<TO*>(p.v_pool) + dst);
        // a token row is moved in rounds of up to 4 KiB of K and 4 KiB of V per wavefront: all of a round's loads are
        // requested before its first store; nothing is reused, so loads and stores are non-temporal
        constexpr int kRound = 4;
        const int n = hd / EPV;
        for (int i0 = lane; i0 < n; i0 += kWave * kRound) {
            u32x4 kx[kRound], vx[kRound];
#pragma unroll
            for (int u = 0; u < kRound; ++u) {
                const int i = i0 + kWave * u;
                if (i < n) {
                    kx[u] = __builtin_nontemporal_load(ks + i);
                    vx[u] = __builtin_nontemporal_load(vs + i);
                }
            }
#pragma unroll
            for (int u = 0; u < kRound; ++u) {
                const int i = i0 + kWave * u;
                if (i < n) {
                    __builtin_nontemporal_store(kx[u], kd + i);
                    __builtin_nontemporal_store(vx[u], vd + i);
                }
            }
        }
    } else {
        const TI* ks = static_cast<const TI*>(p.k_src) + src;
        const TI* vs = static_cast<const TI*>(p.v_src) + src;
        TO* kd = static_cast<TO*>(p.k_pool) + dst;
        TO* vd = static_cast<TO*>(p.v_pool) + dst;
        for (int i = lane; i < hd; i += kWave) {
            Storage<TO>::store(kd + i, Storage<TI>::load(ks + i));
            Storage<TO>::store(vd + i, Storage<TI>::load(vs + i));
        }
    }
}

__global__ void gather_indices_kernel(const int32_t* __restrict__ table, const int32_t* __restrict__ seq_lens,
                                      const int32_t* __restrict__ batch_rows, int64_t B, int H, int d, int P,
                                      int64_t max_pages, int64_t max_len, int64_t* __restrict__ offsets) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= B * max_len) return;
    const int64_t b = idx / max_len;
    const int t = (int)(idx - b * max_len);
    const int64_t row = batch_rows ? batch_rows[b] : b;
    int64_t off = t < seq_lens[row] ? kv_token_offset(table, max_pages, row, t, P, H, d) : -1;
    // a missing page ends the sequence: nothing behind it is read either
    for (int pg = 0; off >= 0 && pg < t / P; ++pg)
        if (table[row * max_pages + pg] < 0) off = -1;
    offsets[idx] = off;
}

// Copies whole pages inside the K and V slabs: page from[i] -> page to[i], i < n (blockIdx.y = 0: K, 1: V).  Sources and
// destinations must be disjoint sets (compaction moves pages in use onto free ones).  Ids outside [0, n_pages) are
// skipped.
__global__ __launch_bounds__(256) void kv_move_pages_kernel(unsigned char* __restrict__ k_pool, unsigned char* __restrict__ v_pool,
                                                            int64_t page_bytes, int64_t n_pages, const int32_t* __restrict__ from,
                                                            const int32_t* __restrict__ to, int64_t n) {
    const int64_t i = blockIdx.x;
    if (i >= n) return;
    const int64_t src = from[i], dst = to[i];
    if (src < 0 || dst < 0 || src >= n_pages || dst >= n_pages || src == dst) return;
    unsigned char* const pool = blockIdx.y == 0 ? k_pool : v_pool;
    const unsigned char* const s = pool + src * page_bytes;
    unsigned char* const d = pool + dst * page_bytes;
    if (((page_bytes | reinterpret_cast<uintptr_t>(pool)) & 15) == 0) {
        for (int64_t o = (int64_t)threadIdx.x * 16; o < page_bytes; o += 256 * 16)
            *reinterpret_cast<u32x4*>(d + o) = *reinterpret_cast<const u32x4*>(s + o);
    } else {
        for (int64_t o = threadIdx.x; o < page_bytes; o += 256) d[o] = s[o];
    }
}

// dst[0..n) = value (a fill in kernel form: callers may be under graph capture)
__global__ __launch_bounds__(256) void fill_i64_kernel(int64_t* __restrict__ dst, int64_t n, int64_t value) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = value;
}

// ---------------------------------------------------------------------------------------------
// decode
struct DecodeParams {
    const void* q;
    void* o;
    const void* k_pool;
    const void* v_pool;
    const int32_t* table;
    const int32_t* seq_lens;
    const int32_t* batch_rows;
    float* part_o;    // [B][n_chunks][H][d]
    float* part_ml;   // [B][n_chunks][H][2]  (m in log2 units, l; l carries a minus sign when the chunk met a missing page)
    int64_t* dump_offsets;  // index-dump launches only: [B][max_len] element offsets of the token rows the kernel addresses
    int64_t max_pages;
    int32_t B, H, d, P;       // H = query heads; d = head dimension of the tensors
    int32_t d_kernel;         // head dimension the lane-per-element kernel is instantiated for: 32, 64, 128 or 256, the
                              // smallest that holds d.  The lanes of a head whose 16-byte piece lies at or beyond d
                              // carry a zero query, re-read the row's first piece and store nothing.
    int32_t H_kv;             // heads in the pool; H / H_kv consecutive query heads share one
    int32_t g0;               // lane-per-element kernel: first query head (within its group) that this launch serves; a group
                              // wider than the kernel is instantiated for is served in several launches
    int32_t chunk_tokens, n_chunks;  // longest chunk (a multiple of P, at most 64 pages) and how many the longest sequence needs
    int32_t balanced;         // 1: a sequence cuts itself into equal chunks (see decode_chunk_len); 0: every chunk is chunk_tokens long
    int32_t max_len;
    int32_t qo_dtype;
    float scale_log2;
};

// Tokens per chunk of a sequence of L tokens.  A sequence needs n = ceil(L / chunk_tokens) chunks; cutting it into n
// EQUAL page-aligned pieces instead of n - 1 full ones and a remainder gives the launch's workgroups similar amounts of
// work (contexts U[512,4096] in chunks of up to 1024: 608 to 1024 tokens each instead of 16 to 1024).  Decode kernels
// and merge evaluate the same function; chunk k of the sequence starts at k * decode_chunk_len and exists iff that is
// below L.
__device__ __forceinline__ int decode_chunk_len(const DecodeParams& p, int L, int P) {
    if (!p.balanced || L <= 0) return p.chunk_tokens;
    const int n = (L + p.chunk_tokens - 1) / p.chunk_tokens;
    const int per = (L + n - 1) / n;
    return ((per + P - 1) / P) * P;  // <= chunk_tokens, which is a multiple of P
}

__device__ __forceinline__ void store_qo(void* base, int dtype, int64_t i, float x) {
    if (dtype == AHPC_F32) static_cast<float*>(base)[i] = x;
    else if (dtype == AHPC_F16) static_cast<f16_t*>(base)[i] = (f16_t)x;
    else static_cast<bf16_t*>(base)[i] = (bf16_t)x;
}

// N (4 or 8) consecutive q/o elements starting at element index i (a multiple of N; the tensors are
// 16-byte aligned), moved with one or two vector accesses whatever the element type.
template <int N> __device__ __forceinline__ void load_qo_vec(const void* base, int dtype, int64_t i, float (&out)[N]) {
    if (dtype == AHPC_F32) {
        const f32x4* src = reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + i);
#pragma unroll
        for (int v = 0; v < N / 4; ++v) {
            const f32x4 x = src[v];
#pragma unroll
            for (int e = 0; e < 4; ++e) out[4 * v + e] = x[e];
        }
    } else {
        uint32_t w[N / 2];
        const uint32_t* src = reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(base) + i);
        if (N == 8) {
            const u32x4 x = *reinterpret_cast<const u32x4*>(src);
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e % (N / 2)] = x[e];
        } else {
            const u32x2 x = *reinterpret_cast<const u32x2*>(src);
            w[0] = x[0];
            w[1] = x[1];
        }
#pragma unroll
        for (int e = 0; e < N / 2; ++e) {
            out[2 * e] = dtype == AHPC_F16 ? lo_f32<f16_t>(w[e]) : lo_f32<bf16_t>(w[e]);
            out[2 * e + 1] = dtype == AHPC_F16 ? hi_f32<f16_t>(w[e]) : hi_f32<bf16_t>(w[e]);
        }
    }
}

// The query operands of the matrix-core decode kernels: KS pieces of 8 consecutive elements (piece ks starts at element
// i0 + ks * step), requested together and converted later.  With the element type tested per piece, every load would be
// followed by its own wait: KS memory round trips in a row in front of a wavefront's first tile.
template <int KS> struct QRaw { u32x4 w[KS][2]; };  // 16-bit types use w[ks][0] only

template <int KS> __device__ __forceinline__ void q_request(QRaw<KS>& r, const void* q, int dtype, int64_t i0, int step) {
    if (dtype == AHPC_F32) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int v = 0; v < 2; ++v) r.w[ks][v] = reinterpret_cast<const u32x4*>(static_cast<const float*>(q) + i0 + ks * step)[v];
    } else {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) r.w[ks][0] = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(q) + i0 + ks * step);
    }
}

// The pieces as pairs of T (the pool's 16-bit type), each element multiplied by c.
template <typename T, int KS> __device__ __forceinline__ void q_convert(const QRaw<KS>& r, int dtype, float c, u32x4 (&out)[KS]) {
    if (dtype == AHPC_F32) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                // (through named words: the bit cast of a vector's element expression reads element 0 with this compiler)
                const uint32_t lo = r.w[ks][w >> 1][2 * (w & 1)], hi = r.w[ks][w >> 1][2 * (w & 1) + 1];
                out[ks][w] = pack2<T>(__builtin_bit_cast(float, lo) * c, __builtin_bit_cast(float, hi) * c);
            }
    } else {
        const bool is_f16 = dtype == AHPC_F16;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t x = r.w[ks][0][w];
                const float lo = is_f16 ? lo_f32<f16_t>(x) : lo_f32<bf16_t>(x);
                const float hi = is_f16 ? hi_f32<f16_t>(x) : hi_f32<bf16_t>(x);
                out[ks][w] = pack2<T>(lo * c, hi * c);
            }
    }
}

template <int N> __device__ __forceinline__ void store_qo_vec(void* base, int dtype, int64_t i, const float (&x)[N]) {
    if (dtype == AHPC_F32) {
        f32x4* dst = reinterpret_cast<f32x4*>(static_cast<float*>(base) + i);
#pragma unroll
        for (int v = 0; v < N / 4; ++v) dst[v] = f32x4{x[4 * v], x[4 * v + 1], x[4 * v + 2], x[4 * v + 3]};
    } else {
        uint32_t w[N / 2];
#pragma unroll
        for (int e = 0; e < N / 2; ++e)
            w[e] = dtype == AHPC_F16 ? pack2<f16_t>(x[2 * e], x[2 * e + 1]) : pack2<bf16_t>(x[2 * e], x[2 * e + 1]);
        uint32_t* dst = reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(base) + i);
        if (N == 8) *reinterpret_cast<u32x4*>(dst) = u32x4{w[0], w[1], w[2 % (N / 2)], w[3 % (N / 2)]};
        else *reinterpret_cast<u32x2*>(dst) = u32x2{w[0], w[1]};
    }
}

// Sum over the LPH lanes that share a head; every one of them gets the total.
template <int LPH> __device__ __forceinline__ float head_allreduce(float x) {
    if (LPH >= 2) x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, true));   // lane ^ 1
    if (LPH >= 4) x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, true));   // lane ^ 2
    if (LPH >= 8) x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, true));  // 7 - lane in each 8
    if (LPH >= 16) x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, true)); // 15 - lane in each 16
    if (LPH >= 32) x += __shfl_xor(x, 16, kWave);
    if (LPH >= 64) x += __shfl_xor(x, 32, kWave);
    return x;
}

// T: pool element type.  D: head dimension.  PT: tokens per page when known at compile time (16), or 0
// for any page size.  G: query heads per pool head (grouped-query attention; 1 = one each).  A lane owns
// EPL = 16/sizeof(T) consecutive elements of one pool head and serves the G query heads of that head
// from the same K and V registers.  Grid: (head group, chunk, batch entry); every wavefront works on
// its own heads and needs no LDS and no barrier.
//
// A chunk starts on a page boundary.  Its page ids are fetched once (one table entry per lane) and
// handed out with v_readlane, so the only per-token address work is a uniform add; K and V rows of
// the next kDecodeBatch tokens are requested before the current ones are consumed.
//
// A table entry of -1 inside a sequence ends the sequence there: keys from that page on are not attended to
// (the reference kernel leaves its page walk at the first negative id, src/backends/cuda/cuda_kernels.cu:417-420).
// The chunk that meets it says so through the sign of its partial l, and the merge stops after that chunk.
//
// DUMP: nothing is loaded or computed; instead the lane that owns (pool head 0, element 0) stores, for every token
// row the kernel would read, the element offset of that row in the pool - taken from the very expression the loads
// use - and -1 for the tokens of its chunk it would not read.  This is what the bit-exact index test compares.
template <typename T, int D, int PT, int G, bool DUMP = false>
__global__ __launch_bounds__(512) void paged_decode_kernel(const DecodeParams p) {
    constexpr int kDecodeBatch = G >= 4 ? 4 : 8;  // tokens whose K and V rows are in flight together, per lane
    constexpr int EPL = 16 / (int)sizeof(T);
    constexpr int LPH = D / EPL;
    constexpr int HPW = kWave / LPH;
    constexpr bool kPacked = sizeof(T) == 2;
    typedef typename std::conditional<kPacked, T, f16_t>::type TP;  // placeholder type for the unused branch

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int waves = blockDim.x >> 6;
    // head group is the fastest grid dimension: the workgroups that together cover the 2*H*D bytes of a
    // token row are dispatched side by side and stream whole pages between them
    const int chunk = blockIdx.y;
    const int b = blockIdx.z;
    const int h_raw = (blockIdx.x * waves + wave) * HPW + lane / LPH;  // pool head
    const bool head_ok = h_raw < p.H_kv;
    const int h = head_ok ? h_raw : p.H_kv - 1;
    const int e0 = (lane % LPH) * EPL;
    const int d = p.d;                    // the tensors' head dimension, D or less
    const int group = G == 1 ? 1 : p.H / p.H_kv;  // query heads per pool head
    const int g0 = G == 1 ? 0 : p.g0;             // the first of them that this launch serves
    const int gr = group - g0 < G ? group - g0 : G;  // how many it serves, G or fewer: the others of the G carry a zero
                                                     // query, are computed along and stored nowhere
    const bool piece_ok = e0 < d;         // this lane's 16-byte piece exists
    const int e_ld = piece_ok ? e0 : 0;   // where it reads K and V from
    const int P = PT ? PT : p.P;

    const int64_t row = p.batch_rows ? p.batch_rows[b] : b;
    const int L = p.seq_lens[row] < p.max_len ? p.seq_lens[row] : p.max_len;
    const int chunk_len = decode_chunk_len(p, L, P);
    const int t0 = chunk * chunk_len;
    // page ids of the chunk (at most 64: the host caps chunk_tokens at 64 pages): lane i holds the id of
    // page (first_page + i)
    const int first_page = t0 / P;
    int my_page = 0;
    if (first_page + lane < p.max_pages) my_page = p.table[row * p.max_pages + first_page + lane];
    bool dumps = DUMP && h_raw == 0 && e0 == 0;  // one lane of the launch's first head group
    if constexpr (DUMP) {
        if (dumps) {  // (the launcher has filled the report with -1: tokens nobody addresses stay that way)
            // what a chunk behind a missing page reads never enters the result (the merge stops in front of it):
            // it is not reported either
            for (int pg = 0; pg < first_page && pg < p.max_pages; ++pg)
                if (p.table[row * p.max_pages + pg] < 0) dumps = false;
        }
    }
    if (t0 >= L) {
        // an empty sequence still owns an output row: zeros (with several chunks the merge writes it)
        if (!DUMP && chunk == 0 && p.n_chunks == 1 && head_ok) {
            float zero[EPL];
#pragma unroll
            for (int e = 0; e < EPL; ++e) zero[e] = 0.0f;
#pragma unroll
            for (int g = 0; g < G; ++g)
                if (piece_ok && g < gr) store_qo_vec<EPL>(p.o, p.qo_dtype, ((int64_t)b * p.H + h * group + g0 + g) * d + e0, zero);
        }
        return;
    }
    int t1 = (t0 + chunk_len) < L ? (t0 + chunk_len) : L;
    // first missing page of the chunk, if any: the chunk ends in front of it
    const unsigned long long missing = __builtin_amdgcn_ballot_w64(lane < (t1 - t0 + P - 1) / P && my_page < 0);
    const bool stopped = missing != 0;
    if (stopped) {
        const int cut = t0 + (int)__builtin_ctzll(missing) * P;
        t1 = cut < t1 ? cut : t1;
    }

    // query pieces of this lane, one per query head of the group
    float qf[G][EPL];
    uint32_t qp[G][4];
    if constexpr (!DUMP) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (piece_ok && g < gr) {
                load_qo_vec<EPL>(p.q, p.qo_dtype, ((int64_t)b * p.H + h * group + g0 + g) * d + e0, qf[g]);
            } else {
#pragma unroll
                for (int e = 0; e < EPL; ++e) qf[g][e] = 0.0f;
            }
            if (kPacked) {
#pragma unroll
                for (int i = 0; i < 4; ++i) qp[g][i] = pack2<TP>(qf[g][2 * i], qf[g][2 * i + 1]);
            }
        }
    }

    // byte offset of this lane's piece inside a token row; token rows are tok_bytes apart
    const uint32_t lane_off = (uint32_t)((h * d + e_ld) * (int)sizeof(T));
    const int64_t tok_bytes = (int64_t)p.H_kv * d * (int64_t)sizeof(T);
    const char* const kbase = static_cast<const char*>(p.k_pool);
    const char* const vbase = static_cast<const char*>(p.v_pool);

    my_page = my_page < 0 ? 0 : my_page;  // never dereferenced: the chunk ends in front of its first missing page

    const int n_tok = t1 - t0;            // 0 when the chunk's first page is missing
    const int n_batches = (n_tok + kDecodeBatch - 1) / kDecodeBatch;

    // Requests the K and V rows of batch `bi` (tokens 8*bi .. 8*bi+7 of the chunk).  Tokens past the
    // end of the chunk re-read the last valid one; their scores are masked when the batch is consumed.
    // The loads are non-temporal: every K/V byte is used exactly once, and keeping the stream out of
    // the caches is worth about 10% of bandwidth here.
    auto issue = [&](u32x4 (&kr)[kDecodeBatch], u32x4 (&vr)[kDecodeBatch], int bi) {
        const int ti0 = bi * kDecodeBatch;
        const int last = n_tok - 1 - ti0;  // index of the last valid token of this batch (>= 0)
        if (PT == 16) {
            // consecutive slots of one page (the batch size divides 16): one page id, rows tok_bytes apart
            const int page_id = __builtin_amdgcn_readlane(my_page, ti0 >> 4);
            const int64_t base = ((int64_t)page_id * 16 + (ti0 & 15)) * tok_bytes;
#pragma unroll
            for (int i = 0; i < kDecodeBatch; ++i) {
                const int ic = i < last ? i : last;
                const int64_t off = base + ic * tok_bytes;
                if constexpr (DUMP) {
                    if (dumps && i <= last) p.dump_offsets[(int64_t)b * p.max_len + t0 + ti0 + i] = (off + lane_off) / (int64_t)sizeof(T);
                } else {
                    kr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kbase + off + lane_off));
                    vr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vbase + off + lane_off));
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < kDecodeBatch; ++i) {
                const int tc = ti0 + (i < last ? i : last);
                const int pg = tc / P;
                const int page_id = __builtin_amdgcn_readlane(my_page, pg);
                const int64_t off = ((int64_t)page_id * P + (tc - pg * P)) * tok_bytes;
                if constexpr (DUMP) {
                    if (dumps && i <= last) p.dump_offsets[(int64_t)b * p.max_len + t0 + ti0 + i] = (off + lane_off) / (int64_t)sizeof(T);
                } else {
                    kr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kbase + off + lane_off));
                    vr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vbase + off + lane_off));
                }
            }
        }
    };

    float acc[G][EPL];
    float m[G], l[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[g][e] = 0.0f;
        m[g] = -INFINITY;
        l[g] = 0.0f;
    }
    const float c = p.scale_log2;

    auto consume = [&](const u32x4 (&kc)[kDecodeBatch], const u32x4 (&vc)[kDecodeBatch], int bi) {
        const int valid = n_tok - bi * kDecodeBatch;  // >= 1; >= kDecodeBatch for all but the last batch
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float s[kDecodeBatch];
            float mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < kDecodeBatch; ++i) {
                float part = 0.0f;
                if (kPacked) {
#pragma unroll
                    for (int w = 0; w < 4; ++w) part = dot2<TP>(qp[g][w], kc[i][w], part);
                } else {
#pragma unroll
                    for (int w = 0; w < 4; ++w) part = __builtin_fmaf(qf[g][w % EPL], as_f32(kc[i][w]), part);
                }
                part = head_allreduce<LPH>(part);
                s[i] = (i < valid) ? part * c : -INFINITY;
                mx = fmaxf(mx, s[i]);
            }
            const float m_new = fmaxf(m[g], mx);            // finite: the batch holds at least one token
            const float alpha = fast_exp2(m[g] - m_new);    // first batch: exp2(-inf) = 0
            float sum = 0.0f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[g][e] *= alpha;
#pragma unroll
            for (int i = 0; i < kDecodeBatch; ++i) {
                const float w = fast_exp2(s[i] - m_new);
                sum += w;
                if (kPacked) {
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        acc[g][(2 * x) % EPL] = __builtin_fmaf(w, lo_f32<TP>(vc[i][x]), acc[g][(2 * x) % EPL]);
                        acc[g][(2 * x + 1) % EPL] = __builtin_fmaf(w, hi_f32<TP>(vc[i][x]), acc[g][(2 * x + 1) % EPL]);
                    }
                } else {
#pragma unroll
                    for (int x = 0; x < 4; ++x) acc[g][x % EPL] = __builtin_fmaf(w, as_f32(vc[i][x]), acc[g][x % EPL]);
                }
            }
            l[g] = l[g] * alpha + sum;
            m[g] = m_new;
        }
    };

    // two register sets in ping-pong: while one batch is consumed the next is in flight
    u32x4 ka[kDecodeBatch], va[kDecodeBatch], kb2[kDecodeBatch], vb2[kDecodeBatch];
    if constexpr (DUMP) {
        for (int bi = 0; bi < n_batches; ++bi) issue(ka, va, bi);
        return;
    }
    if (n_batches > 0) issue(ka, va, 0);
    for (int bi = 0; bi < n_batches; bi += 2) {
        if (bi + 1 < n_batches) issue(kb2, vb2, bi + 1);
        consume(ka, va, bi);
        if (bi + 1 < n_batches) {
            if (bi + 2 < n_batches) issue(ka, va, bi + 2);
            consume(kb2, vb2, bi + 1);
        }
    }

    if (!head_ok) return;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        if (g >= gr) break;
        const int hq = h * group + g0 + g;
        if (p.n_chunks == 1) {
            const float inv = l[g] > 0.0f ? 1.0f / l[g] : 0.0f;
            float res[EPL];
#pragma unroll
            for (int e = 0; e < EPL; ++e) res[e] = acc[g][e] * inv;
            if (piece_ok) store_qo_vec<EPL>(p.o, p.qo_dtype, ((int64_t)b * p.H + hq) * d + e0, res);
        } else {
            const int64_t slot = ((int64_t)b * p.n_chunks + chunk) * p.H + hq;
            f32x4* dst = reinterpret_cast<f32x4*>(p.part_o + slot * d + e_ld);
            if (piece_ok) {
#pragma unroll
                for (int e = 0; e < EPL; e += 4) dst[e / 4] = f32x4{acc[g][e], acc[g][e + 1], acc[g][e + 2], acc[g][e + 3]};
            }
            if (lane % LPH == 0) {
                p.part_ml[slot * 2] = m[g];
                p.part_ml[slot * 2 + 1] = stopped ? -l[g] : l[g];  // l >= 0, and -(0.0f) still carries the sign
            }
        }
    }
}

// One wavefront per (batch entry, head): folds the chunk partials with the rule
// m' = max(m, m2), l' = l*2^(m-m') + l2*2^(m2-m'), accumulators scaled by the same factors.  The round trips to
// memory are what this kernel takes (a long context has 32 chunks and more), so it makes few of them: the (m, l)
// pairs of up to 64 chunks arrive in one, a lane each, and the accumulators in batches of 16 chunks, every load of a
// batch issued before the first is used (a lane holds four consecutive elements of d).
constexpr int kMergeWaves = 4;   // (batch entry, head) pairs per workgroup
constexpr int kMergeBatch = 16;  // chunks whose accumulators are in flight together
__global__ __launch_bounds__(64 * kMergeWaves) void paged_merge_kernel(const DecodeParams p) {
    const int lane = threadIdx.x & 63;
    const int64_t pair = (int64_t)blockIdx.x * kMergeWaves + (threadIdx.x >> 6);
    if (pair >= (int64_t)p.B * p.H) return;  // (uniform per wavefront)
    const int64_t b = pair / p.H;
    const int h = (int)(pair - b * p.H);
    const int64_t row = p.batch_rows ? p.batch_rows[b] : b;
    const int L = p.seq_lens[row] < p.max_len ? p.seq_lens[row] : p.max_len;
    const int chunk_len = decode_chunk_len(p, L, p.P);
    const int n = (L + chunk_len - 1) / chunk_len;
    const float* ml = p.part_ml + ((b * p.n_chunks) * p.H + h) * 2;
    const float* po = p.part_o + ((b * p.n_chunks) * p.H + h) * p.d;
    const int64_t ml_step = (int64_t)p.H * 2, po_step = (int64_t)p.H * p.d;
    const int e0 = 4 * lane;
    const bool active = e0 < p.d;  // d is a multiple of 4

    // A chunk whose l carries a minus sign met a missing page: it is the last one that counts.  Every chunk of the
    // sequence has written its (m, l) pair.  First walk: where the sequence ends, and the largest m up to there.
    float m = -INFINITY;
    int n_used = n;
    for (int c0 = 0; c0 < n; c0 += kWave) {
        const int c = c0 + lane;
        float mc = -INFINITY;
        bool stops = false;
        if (c < n) {
            mc = ml[c * ml_step];
            stops = (__builtin_bit_cast(uint32_t, ml[c * ml_step + 1]) >> 31) != 0;
        }
        const unsigned long long stop = __builtin_amdgcn_ballot_w64(stops);
        if (stop != 0) {
            const int first = c0 + (int)__builtin_ctzll(stop);
            n_used = first + 1;
            if (c > first) mc = -INFINITY;
        }
        m = fmaxf(m, mc);
        if (stop != 0) break;  // (uniform)
    }
#pragma unroll
    for (int s = 1; s < kWave; s <<= 1) m = fmaxf(m, __shfl_xor(m, s, kWave));

    // Second walk: weights 2^(m_c - m), a lane per chunk; the accumulators of a batch of chunks, then their sum.
    float l = 0.0f;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int c0 = 0; c0 < n_used; c0 += kWave) {
        const int c = c0 + lane;
        float f = 0.0f;
        if (c < n_used) {
            f = fast_exp2(ml[c * ml_step] - m);  // (m is -inf only when every m_c is: then l stays 0 below)
            l = __builtin_fmaf(__builtin_fabsf(ml[c * ml_step + 1]), f, l);
        }
        const int cnt = n_used - c0 < kWave ? n_used - c0 : kWave;
        for (int ci = 0; ci < cnt; ci += kMergeBatch) {
            f32x4 v[kMergeBatch];
#pragma unroll
            for (int u = 0; u < kMergeBatch; ++u) {
                v[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                if (ci + u < cnt && active) v[u] = *reinterpret_cast<const f32x4*>(po + (int64_t)(c0 + ci + u) * po_step + e0);
            }
#pragma unroll
            for (int u = 0; u < kMergeBatch; ++u) {
                // (a lane index beyond the batch's chunks is never used: v[u] is zero there)
                const float fc = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(f), (ci + u) & (kWave - 1)));
                if (ci + u < cnt) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(v[u][i], fc, acc[i]);
                }
            }
        }
    }
#pragma unroll
    for (int s = 1; s < kWave; s <<= 1) l += __shfl_xor(l, s, kWave);
    // nothing attended to (empty sequence, or its first page missing): l is 0, or NaN from (-inf) - (-inf)
    if (active) {
        const bool live = l > 0.0f;
        const float inv = live ? 1.0f / l : 0.0f;
        const float res[4] = {live ? acc[0] * inv : 0.0f, live ? acc[1] * inv : 0.0f, live ? acc[2] * inv : 0.0f, live ? acc[3] * inv : 0.0f};
        store_qo_vec<4>(p.o, p.qo_dtype, pair * p.d + e0, res);
    }
}

}  // namespace ahpc

#include "paged_decode_mfma.hpp"  // uses DecodeParams and the q/o vector helpers above
#include "paged_decode_group.hpp"

namespace ahpc {

// Smallest chunk any launch plan below picks for pages of P tokens (sizes the workspace's upper bound).
static int64_t smallest_chunk(int64_t P) { return ((128 + P - 1) / P) * P; }

static int64_t fit_chunk(int64_t chunk, int64_t P) {
    chunk = ((chunk + P - 1) / P) * P;
    if (chunk < P) chunk = P;
    if (chunk > 64 * P) chunk = 64 * P;  // the decode kernel keeps one page id per lane
    return chunk;
}

// Tokens per chunk and wavefronts per workgroup of one decode launch.  row_waves = wavefronts that cover the
// pool heads of one token (each wave works alone; waves only sets how many heads travel together).
struct DecodePlan { int64_t chunk; int waves; };

static DecodePlan plan_decode(int64_t B, int64_t H_kv, int64_t group, int64_t row_waves, int64_t max_len, int64_t P,
                              int64_t requested, bool matrix_kernel = false, int wide_max_waves = 0) {
    DecodePlan plan{requested, (int)tuning().decode_waves.load()};
    if (plan.waves < 0 || plan.waves > 8) plan.waves = 0;
    if (plan.chunk <= 0) plan.chunk = tuning().decode_chunk.load();
    if (wide_max_waves > 0) {
        // The kernel for groups of 17 to 32 query heads: a workgroup of W wavefronts per (pool head, chunk), two tile
        // slots of LDS per wavefront (W = 4 fills a CU at d = 128).  Timed with 32 query heads over one pool head, d =
        // 128: a launch with more workgroups than the CUs hold at once is bound by the stream, and single wavefronts on
        // the longest chunks win (five to a CU, each at its own point of its chunk, few partials: B = 64 with contexts
        // U[16384,32768] 0.158 ms at W = 1, 0.169 at 2, 0.190 at 4).  A launch that fits the CUs in one round is bound
        // by the time of one workgroup, and W wavefronts that share a chunk's tiles out shorten that (B = 8 with the
        // same contexts: 0.042 ms at 256 tokens and W = 1, 0.030 at 1024 and W = 4; B = 16 with contexts U[512,4096]:
        // 0.021 -> 0.017 ms).
        const auto wgs = [&](int64_t chunk) { return B * H_kv * ((max_len + chunk - 1) / chunk); };
        int waves = wgs(1024) > 512 ? 1 : wgs(1024) > 256 ? 2 : 4;
        if (waves > wide_max_waves) waves = wide_max_waves;
        if (plan.chunk > 0) {
            plan.chunk = fit_chunk(plan.chunk, P);
            if (!plan.waves) plan.waves = plan.chunk >= 256 ? waves : plan.chunk >= 128 ? (waves < 2 ? waves : 2) : 1;  // two tiles and more per wavefront
            return plan;
        }
        int64_t chunk = 1024;
        while (waves > 1 && chunk > 256 && wgs(chunk) < 256 && (max_len + chunk / 2 - 1) / (chunk / 2) <= 64) chunk /= 2;
        plan.chunk = fit_chunk(chunk, P);
        if (!plan.waves) plan.waves = waves;
        return plan;
    }
    if (plan.chunk > 0) {
        plan.chunk = fit_chunk(plan.chunk, P);
        if (!plan.waves) plan.waves = 2;
        return plan;
    }
    if (matrix_kernel) {
        // one wavefront per pool head and chunk, bound by the stream like the case below
        // (a sequence in more than 64 chunks costs more in the merge, which walks them one wavefront per head, than
        // the shorter chunks gain: one sequence of 30 000 tokens, 32 heads over 8: 0.050 ms in chunks of 128, 0.034 in 512)
        int64_t chunk = 1024;
        while (chunk > 128 && B * ((max_len + chunk - 1) / chunk) * H_kv < 1024 && (max_len + chunk / 2 - 1) / (chunk / 2) <= 64) chunk /= 2;
        plan.chunk = fit_chunk(chunk, P);
        if (!plan.waves) plan.waves = 2;  // (unused by those kernels)
        return plan;
    }
    if (group == 1) {
        // One query head per pool head is pure streaming: the longest chunks that still leave about four
        // wavefronts for every CU (timed on B=1..256, contexts 128..131072: chunks of 1024 tokens win wherever
        // they leave >= 1024 wavefronts; shorter chunks pay in partials and in part-filled requests).
        // (and no more than 64 chunks to a sequence: the merge walks them one wavefront per head, and beyond that it
        // costs more than the shorter chunks gain: one sequence of 30 000 tokens, 32 heads, 0.105 ms in chunks of 128,
        // 0.091 in 512)
        int64_t chunk = 1024;
        while (chunk > 128 && B * ((max_len + chunk - 1) / chunk) * row_waves < 1024 && (max_len + chunk / 2 - 1) / (chunk / 2) <= 64) chunk /= 2;
        plan.chunk = fit_chunk(chunk, P);
        if (!plan.waves) {
            // Whole token rows per workgroup (8 wavefronts read 8 consecutive KiB and more) when such workgroups
            // still fill the CUs and every sequence spans several of them; single wavefronts otherwise, which
            // spread a few long sequences over more CUs.
            const int64_t n_chunks = (max_len + plan.chunk - 1) / plan.chunk;
            plan.waves = (row_waves >= 8 && n_chunks >= 2 && B * n_chunks >= 256) ? 8 : 1;
        }
        return plan;
    }
    // Several query heads per pool head: the arithmetic per byte is G times higher and more resident
    // workgroups hide it better; enough workgroups to keep every CU busy several times over, while the fp32
    // partials stay below ~1% of the K/V bytes of a chunk.
    int64_t chunk = 256;
    while (chunk > 128 && B * ((max_len + chunk - 1) / chunk) * ((H_kv * group + 3) / 4) < 4096) chunk /= 2;
    plan.chunk = fit_chunk(chunk, P);
    if (!plan.waves) plan.waves = 2;
    return plan;
}

template <typename T, int PT, int G>
static int launch_decode_dpg(const DecodeParams& p, dim3 grid, dim3 block, hipStream_t st) {
    switch (p.d_kernel) {
        case 32: hipLaunchKernelGGL((paged_decode_kernel<T, 32, PT, G>), grid, block, 0, st, p); break;
        case 64: hipLaunchKernelGGL((paged_decode_kernel<T, 64, PT, G>), grid, block, 0, st, p); break;
        case 128: hipLaunchKernelGGL((paged_decode_kernel<T, 128, PT, G>), grid, block, 0, st, p); break;
        case 256: hipLaunchKernelGGL((paged_decode_kernel<T, 256, PT, G>), grid, block, 0, st, p); break;
        default: return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
    }
    return static_cast<int>(hipGetLastError());
}

template <typename T, int PT>
static int launch_decode_dp(const DecodeParams& base, dim3 grid, dim3 block, hipStream_t st) {
    // Instantiated for 1, 2, 4 and 8 query heads per pool head.  A group in between runs on the next size; a wider one
    // in slices of 8 query heads, one launch each (every slice reads the K/V stream again), the last slice on the
    // size that holds it.
    const int group = base.H / base.H_kv;
    if (group == 1) return launch_decode_dpg<T, PT, 1>(base, grid, block, st);
    DecodeParams p = base;
    for (int g0 = 0; g0 < group; g0 += 8) {
        p.g0 = g0;
        const int slice = group - g0 < 8 ? group - g0 : 8;
        const int rc = slice <= 2 ? launch_decode_dpg<T, PT, 2>(p, grid, block, st)
                     : slice <= 4 ? launch_decode_dpg<T, PT, 4>(p, grid, block, st)
                                  : launch_decode_dpg<T, PT, 8>(p, grid, block, st);
        if (rc) return rc;
    }
    return AHPC_OK;
}

// Matrix-core kernel for groups of 17 to 32 query heads: a workgroup of 1, 2 or 4 wavefronts per (pool head, chunk,
// batch entry); the wavefronts share the chunk's tiles out and merge their results in LDS.
template <typename T, int D>
static int launch_decode_mfma_d(const DecodeParams& p, int waves, hipStream_t st) {
    constexpr int kMaxW = D <= 128 ? 4 : 2;  // a wavefront's two tile slots take 256 * D bytes of LDS
    int w = waves >= 4 ? 4 : waves >= 2 ? 2 : 1;
    if (w > kMaxW) w = kMaxW;
    const dim3 grid((unsigned)p.H_kv, (unsigned)p.n_chunks, (unsigned)p.B), block(64 * w);
    if (w == 4) {
        if constexpr (kMaxW >= 4) hipLaunchKernelGGL((paged_decode_mfma_kernel<T, D, 4>), grid, block, 0, st, p);
    } else if (w == 2) {
        hipLaunchKernelGGL((paged_decode_mfma_kernel<T, D, 2>), grid, block, 0, st, p);
    } else {
        hipLaunchKernelGGL((paged_decode_mfma_kernel<T, D, 1>), grid, block, 0, st, p);
    }
    return static_cast<int>(hipGetLastError());
}

template <typename T>
static int launch_decode_mfma(const DecodeParams& p, int waves, hipStream_t st) {
    if (p.d == 128) return launch_decode_mfma_d<T, 128>(p, waves, st);
    if (p.d == 64) return launch_decode_mfma_d<T, 64>(p, waves, st);
    if (p.d == 256) return launch_decode_mfma_d<T, 256>(p, waves, st);
    return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
}

// Matrix-core kernel for groups of up to 16 query heads: a wavefront per (pool head, chunk, batch entry), up to 8
// pool heads side by side in a workgroup.
template <typename T, int D>
static int launch_decode_group_d(const DecodeParams& p, int waves_wanted, hipStream_t st) {
    // (at d = 256 a wavefront's two page slots take 32 KiB of LDS: four wavefronts at most)
    int w = (p.H_kv >= 8 && D <= 128) ? 8 : p.H_kv >= 4 ? 4 : p.H_kv >= 2 ? 2 : 1;
    // A CU draws about 25 GB/s however many wavefronts ask, so a launch with fewer workgroups than CUs is bound by the
    // CUs it reaches: narrower workgroups then, until the launch has one for every CU.  (32 query heads over 8 pool
    // heads, d = 128, contexts U[512,4096]: B = 32 0.086 ms on 8 wavefronts, 0.059 on 4 or 2; B = 16 0.052 -> 0.035;
    // B = 4 0.021 -> 0.017; from B = 64 on whole token rows per workgroup win by 5 %.)
    // (the tuning value decode_waves, when set, says how wide instead)
    if (waves_wanted > 0) {
        while (w > waves_wanted) w /= 2;
    } else {
        while (w > 1 && (int64_t)p.B * p.n_chunks * ((p.H_kv + w - 1) / w) < 256) w /= 2;
    }
    const dim3 grid((unsigned)((p.H_kv + w - 1) / w), (unsigned)p.n_chunks, (unsigned)p.B), block(64 * w);
    switch (w) {
        case 8:
            if constexpr (D <= 128) hipLaunchKernelGGL((paged_decode_group_kernel<T, D, 8>), grid, block, 0, st, p);
            break;
        case 4: hipLaunchKernelGGL((paged_decode_group_kernel<T, D, 4>), grid, block, 0, st, p); break;
        case 2: hipLaunchKernelGGL((paged_decode_group_kernel<T, D, 2>), grid, block, 0, st, p); break;
        default: hipLaunchKernelGGL((paged_decode_group_kernel<T, D, 1>), grid, block, 0, st, p); break;
    }
    return static_cast<int>(hipGetLastError());
}

template <typename T>
static int launch_decode_group(const DecodeParams& p, int waves_wanted, hipStream_t st) {
    if (p.d == 128) return launch_decode_group_d<T, 128>(p, waves_wanted, st);
    if (p.d == 64) return launch_decode_group_d<T, 64>(p, waves_wanted, st);
    if (p.d == 256) return launch_decode_group_d<T, 256>(p, waves_wanted, st);
    return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
}

template <typename T>
static int launch_decode_d(const DecodeParams& p, dim3 grid, dim3 block, hipStream_t st) {
    return p.P == 16 ? launch_decode_dp<T, 16>(p, grid, block, st) : launch_decode_dp<T, 0>(p, grid, block, st);
}

// ---- scratch of ahpc_hip_paged_decode_noalloc -------------------------------------------------------
// Part of the device code, so every GPU that loads the library holds its own copy at its own address.  In
// host code the array's name is only a handle for hipGetSymbolAddress: kernels and memory calls get the
// looked-up device address, never the name.
static __device__ __align__(256) unsigned char scratch[AHPC_NOALLOC_SCRATCH_BYTES];
constexpr int kScratchDevices = 64;
static std::atomic<void*> g_scratch_ptr[kScratchDevices];  // per device; null until looked up

static int scratch_of_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= kScratchDevices) return AHPC_ERR_NO_DEVICE;
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (!ptr) return AHPC_ERR_NO_DEVICE;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // two threads racing here store the same address
    }
    *out = ptr;
    return AHPC_OK;
}

}  // namespace ahpc

using namespace ahpc;

namespace {

template <typename TI>
int scatter_out(int pool_dtype, const void* k_new, const void* v_new, void* k_pool, void* v_pool, const int32_t* table,
                int64_t max_pages, const int32_t* token_row, const int32_t* token_pos, int64_t row0, int64_t pos0,
                int64_t n, int H, int d, int P, hipStream_t st) {
    const int64_t total = n * H * d;
    dim3 block(256), grid((unsigned)((total + 255) / 256));
#define AHPC_SCATTER(TO)                                                                                              \
    hipLaunchKernelGGL((kv_scatter_kernel<TI, TO>), grid, block, 0, st, static_cast<const TI*>(k_new),                \
                       static_cast<const TI*>(v_new), static_cast<TO*>(k_pool), static_cast<TO*>(v_pool), table,      \
                       max_pages, token_row, token_pos, row0, pos0, n, H, d, P)
    switch (pool_dtype) {
        case AHPC_F32: AHPC_SCATTER(float); break;
        case AHPC_F16: AHPC_SCATTER(f16_t); break;
        case AHPC_BF16: AHPC_SCATTER(bf16_t); break;
        default: return AHPC_ERR_BAD_DTYPE;
    }
#undef AHPC_SCATTER
    return static_cast<int>(hipGetLastError());
}

template <typename TI>
int gather_out(int out_dtype, void* k_out, void* v_out, const void* k_pool, const void* v_pool, const int32_t* table,
               int64_t max_pages, int64_t row, int64_t start, int64_t n, int H, int d, int P, hipStream_t st) {
    const int64_t total = n * H * d;
    dim3 block(256), grid((unsigned)((total + 255) / 256));
#define AHPC_GATHER(TO)                                                                                               \
    hipLaunchKernelGGL((kv_gather_kernel<TI, TO>), grid, block, 0, st, static_cast<TO*>(k_out),                       \
                       static_cast<TO*>(v_out), static_cast<const TI*>(k_pool), static_cast<const TI*>(v_pool), table, \
                       max_pages, row, start, n, H, d, P)
    switch (out_dtype) {
        case AHPC_F32: AHPC_GATHER(float); break;
        case AHPC_F16: AHPC_GATHER(f16_t); break;
        case AHPC_BF16: AHPC_GATHER(bf16_t); break;
        default: return AHPC_ERR_BAD_DTYPE;
    }
#undef AHPC_GATHER
    return static_cast<int>(hipGetLastError());
}

bool dims_ok(int64_t H, int64_t d, int64_t P, int64_t max_pages) {
    return H > 0 && d > 0 && P > 0 && max_pages > 0 && H <= 65535 && d <= 1024 && P <= 4096 && max_pages <= 0x7FFFFFFFll;
}

}  // namespace

extern "C" {

int ahpc_hip_kv_scatter(const void* k_new, const void* v_new, int in_dtype, void* k_pool, void* v_pool, int pool_dtype,
                        const int32_t* block_table, int64_t max_pages, const int32_t* token_row, const int32_t* token_pos,
                        int64_t row0, int64_t pos0, int64_t n_tokens, int64_t H, int64_t d, int64_t P, void* stream) {
    if (n_tokens == 0) return AHPC_OK;
    if (!k_new || !v_new || !k_pool || !v_pool || !block_table) return AHPC_ERR_NULL_POINTER;
    if (n_tokens < 0 || row0 < 0 || pos0 < 0 || !dims_ok(H, d, P, max_pages)) return AHPC_ERR_BAD_SHAPE;
    if (n_tokens * H * d > 0xFFFFFFFFll * 256) return AHPC_ERR_BAD_SHAPE;
    // consecutive positions from pos0: all of them must lie inside the table row
    if (!token_pos && (pos0 + n_tokens + P - 1) / P > max_pages) return AHPC_ERR_BAD_SHAPE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (in_dtype) {
        case AHPC_F32: return scatter_out<float>(pool_dtype, k_new, v_new, k_pool, v_pool, block_table, max_pages, token_row, token_pos, row0, pos0, n_tokens, (int)H, (int)d, (int)P, st);
        case AHPC_F16: return scatter_out<f16_t>(pool_dtype, k_new, v_new, k_pool, v_pool, block_table, max_pages, token_row, token_pos, row0, pos0, n_tokens, (int)H, (int)d, (int)P, st);
        case AHPC_BF16: return scatter_out<bf16_t>(pool_dtype, k_new, v_new, k_pool, v_pool, block_table, max_pages, token_row, token_pos, row0, pos0, n_tokens, (int)H, (int)d, (int)P, st);
        default: return AHPC_ERR_BAD_DTYPE;
    }
}

int ahpc_hip_kv_scatter_batch(const void* k_src, const void* v_src, int in_dtype, int64_t stride_b, int64_t stride_n,
                              void* k_pool, void* v_pool, int pool_dtype, const int32_t* block_table, int64_t max_pages,
                              const int32_t* seq_rows, const int32_t* seq_start, const int32_t* seq_tokens,
                              const int32_t* cu_seqlens, int64_t B, int64_t N, int64_t H, int64_t d, int64_t P, void* stream) {
    if (B == 0 || N == 0) return AHPC_OK;
    if (!k_src || !v_src || !k_pool || !v_pool || !block_table || !seq_rows) return AHPC_ERR_NULL_POINTER;
    if (B < 0 || B > 65535 || N < 0 || N > 0x7FFFFFF0ll || !dims_ok(H, d, P, max_pages)) return AHPC_ERR_BAD_SHAPE;
    if (stride_n < H * d || (!cu_seqlens && stride_b < 0)) return AHPC_ERR_BAD_SHAPE;
    if (in_dtype < AHPC_F32 || in_dtype > AHPC_BF16 || pool_dtype < AHPC_F32 || pool_dtype > AHPC_BF16) return AHPC_ERR_BAD_DTYPE;
    ScatterBatchParams p{k_src, v_src, k_pool, v_pool, block_table, seq_rows, seq_start, seq_tokens, cu_seqlens, max_pages,
                         stride_b, stride_n, (int32_t)B, (int32_t)N, (int32_t)H, (int32_t)d, (int32_t)P};
    hipStream_t st = static_cast<hipStream_t>(stream);
    dim3 block(256), grid((unsigned)((N + 3) / 4), (unsigned)B);
    const int esz = in_dtype == AHPC_F32 ? 4 : 2;
    auto aligned = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    const bool vec = in_dtype == pool_dtype && aligned(k_src) && aligned(v_src) && aligned(k_pool) && aligned(v_pool) &&
                     (H * d * esz) % 16 == 0 && (stride_n * esz) % 16 == 0 && (stride_b * esz) % 16 == 0;
#define AHPC_SB(TI, TO, V) hipLaunchKernelGGL((kv_scatter_batch_kernel<TI, TO, V>), grid, block, 0, st, p)
    if (vec) {
        if (in_dtype == AHPC_F32) AHPC_SB(float, float, true);
        else AHPC_SB(f16_t, f16_t, true);  // 16-bit rows are moved as bits: fp16 and bf16 alike
    } else {
        switch (in_dtype * 3 + pool_dtype) {
            case 0: AHPC_SB(float, float, false); break;
            case 1: AHPC_SB(float, f16_t, false); break;
            case 2: AHPC_SB(float, bf16_t, false); break;
            case 3: AHPC_SB(f16_t, float, false); break;
            case 4: AHPC_SB(f16_t, f16_t, false); break;
            case 5: AHPC_SB(f16_t, bf16_t, false); break;
            case 6: AHPC_SB(bf16_t, float, false); break;
            case 7: AHPC_SB(bf16_t, f16_t, false); break;
            default: AHPC_SB(bf16_t, bf16_t, false); break;
        }
    }
#undef AHPC_SB
    return static_cast<int>(hipGetLastError());
}

int ahpc_hip_kv_gather(void* k_out, void* v_out, int out_dtype, const void* k_pool, const void* v_pool, int pool_dtype,
                       const int32_t* block_table, int64_t max_pages, int64_t row, int64_t start, int64_t n, int64_t H,
                       int64_t d, int64_t P, void* stream) {
    if (n == 0) return AHPC_OK;
    if (!k_out || !v_out || !k_pool || !v_pool || !block_table) return AHPC_ERR_NULL_POINTER;
    if (n < 0 || row < 0 || start < 0 || !dims_ok(H, d, P, max_pages)) return AHPC_ERR_BAD_SHAPE;
    if ((start + n + P - 1) / P > max_pages) return AHPC_ERR_BAD_SHAPE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (pool_dtype) {
        case AHPC_F32: return gather_out<float>(out_dtype, k_out, v_out, k_pool, v_pool, block_table, max_pages, row, start, n, (int)H, (int)d, (int)P, st);
        case AHPC_F16: return gather_out<f16_t>(out_dtype, k_out, v_out, k_pool, v_pool, block_table, max_pages, row, start, n, (int)H, (int)d, (int)P, st);
        case AHPC_BF16: return gather_out<bf16_t>(out_dtype, k_out, v_out, k_pool, v_pool, block_table, max_pages, row, start, n, (int)H, (int)d, (int)P, st);
        default: return AHPC_ERR_BAD_DTYPE;
    }
}

size_t ahpc_hip_paged_decode_workspace_bytes(int64_t B, int64_t H, int64_t d, int64_t max_len, int64_t P,
                                             int64_t chunk_tokens) {
    if (B <= 0 || H <= 0 || d <= 0 || max_len <= 0 || P <= 0) return 0;
    // Without the pool's head count and type the launch plan is not known here: an upper bound, the
    // smallest chunk a plan picks (a requested or tuned chunk is taken as it is).
    int64_t chunk = chunk_tokens > 0 ? chunk_tokens : tuning().decode_chunk.load();
    chunk = fit_chunk(chunk > 0 ? chunk : smallest_chunk(P), P);
    const int64_t n_chunks = (max_len + chunk - 1) / chunk;
    if (n_chunks <= 1) return 0;
    return (size_t)(B * n_chunks * H * (d + 2)) * sizeof(float);
}

int ahpc_hip_paged_decode_gqa(const void* q, void* o, int qo_dtype, const void* k_pool, const void* v_pool, int pool_dtype,
                              const int32_t* block_table, const int32_t* seq_lens, const int32_t* batch_rows, int64_t B,
                              int64_t H, int64_t H_kv, int64_t d, int64_t P, int64_t max_pages, int64_t max_len,
                              float scale, int64_t chunk_tokens, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !o || !k_pool || !v_pool || !block_table || !seq_lens) return AHPC_ERR_NULL_POINTER;
    if (H_kv <= 0 || H <= 0 || H % H_kv) return AHPC_ERR_BAD_SHAPE;
    // Up to 8 query heads per pool head: lane-per-element kernel, any pool type (from the tuning value
    // decode_matrix_min_group on: the page-by-page matrix-core kernel, where the pool allows it).  9 to 16: the
    // page-by-page matrix-core kernel; 17 to 32: the 32-column one.  Both need a 16-bit pool, d 64 or 128 and pages
    // of 16 tokens; other pools, and groups beyond 32, go through the lane-per-element kernel in slices of 8 query
    // heads.  The matrix-core kernels take the group size as it is (idle result columns), the lane-per-element
    // kernel runs a group or slice of 3 as 4 and 5 to 7 as 8.
    const int64_t group = H / H_kv;
    const bool mfma_shape = (pool_dtype == AHPC_F16 || pool_dtype == AHPC_BF16) && (d == 64 || d == 128 || d == 256) && P == 16 && H_kv <= 65535 &&
                            group <= 32;
    if (qo_dtype < AHPC_F32 || qo_dtype > AHPC_BF16 || pool_dtype < AHPC_F32 || pool_dtype > AHPC_BF16) return AHPC_ERR_BAD_DTYPE;
    if (B <= 0 || B > 65535 || max_len <= 0 || max_len > 0x7FFFFFFFll || !dims_ok(H, d, P, max_pages)) return AHPC_ERR_BAD_SHAPE;
    if ((max_len + P - 1) / P > max_pages) return AHPC_ERR_BAD_SHAPE;
    // head dimensions up to 256 in whole 16-byte pieces of the pool's type; the lane-per-element kernel is instantiated
    // for 32, 64, 128 and 256 and takes the smallest that holds d (DecodeParams::d_kernel)
    const int64_t piece = pool_dtype == AHPC_F32 ? 4 : 8;
    if (d > 256 || d < piece || (d % piece)) return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
    const int64_t d_kernel = d <= 32 ? 32 : d <= 64 ? 64 : d <= 128 ? 128 : 256;
    if ((reinterpret_cast<uintptr_t>(k_pool) & 15u) || (reinterpret_cast<uintptr_t>(v_pool) & 15u) ||
        (reinterpret_cast<uintptr_t>(q) & 15u) || (reinterpret_cast<uintptr_t>(o) & 15u))
        return AHPC_ERR_BAD_ALIGNMENT;
    if (!(scale > 0.0f)) scale = 1.0f / std::sqrt((float)d);

    const int lph = (int)(d_kernel * (pool_dtype == AHPC_F32 ? 4 : 2) / 16);  // lanes that hold one head of a token
    const int hpw = 64 / lph;
    const int64_t matrix_from = tuning().decode_matrix_min_group.load();
    const bool use_mfma = mfma_shape && (group > 8 || group >= matrix_from);
    const DecodePlan plan = plan_decode(B, H_kv, group < 8 ? group : 8, (H_kv + hpw - 1) / hpw, max_len, P, chunk_tokens, use_mfma,
                                        use_mfma && group > 16 ? (d <= 128 ? 4 : 2) : 0);
    const int64_t chunk = plan.chunk;
    const int waves = plan.waves;
    const int64_t n_chunks = (max_len + chunk - 1) / chunk;
    const size_t need = n_chunks > 1 ? (size_t)(B * n_chunks * H * (d + 2)) * sizeof(float) : 0;
    if (need > 0 && (!workspace || workspace_bytes < need)) return AHPC_ERR_WORKSPACE_TOO_SMALL;
    if (need > 0 && (reinterpret_cast<uintptr_t>(workspace) & 15u)) return AHPC_ERR_BAD_ALIGNMENT;  // partials move in 16-byte pieces
    if (n_chunks > 65535) return AHPC_ERR_BAD_SHAPE;

    DecodeParams p{};
    p.q = q; p.o = o; p.k_pool = k_pool; p.v_pool = v_pool;
    p.table = block_table; p.seq_lens = seq_lens; p.batch_rows = batch_rows;
    p.part_o = static_cast<float*>(workspace);
    p.part_ml = p.part_o ? p.part_o + B * n_chunks * H * d : nullptr;
    p.max_pages = max_pages;
    p.B = (int32_t)B; p.H = (int32_t)H; p.d = (int32_t)d; p.P = (int32_t)P;
    p.d_kernel = (int32_t)d_kernel;
    p.H_kv = (int32_t)H_kv;
    p.chunk_tokens = (int32_t)chunk; p.n_chunks = (int32_t)n_chunks;
    p.balanced = 1;
    p.max_len = (int32_t)max_len;
    p.qo_dtype = qo_dtype;
    p.scale_log2 = scale * kLog2e;

    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t heads_per_wg = (int64_t)hpw * waves;  // pool heads
    const int64_t head_groups = (H_kv + heads_per_wg - 1) / heads_per_wg;
    if (head_groups > 65535) return AHPC_ERR_BAD_SHAPE;

    dim3 eblock(64 * kMergeWaves), egrid((unsigned)((B * H + kMergeWaves - 1) / kMergeWaves));  // the merge: a wavefront per (b, h)

    dim3 grid((unsigned)head_groups, (unsigned)n_chunks, (unsigned)B), block(64 * waves);
    int rc;
    if (use_mfma && group <= 16) {
        const int wanted = (int)tuning().decode_waves.load();
        rc = pool_dtype == AHPC_F16 ? launch_decode_group<f16_t>(p, wanted, st) : launch_decode_group<bf16_t>(p, wanted, st);
    } else if (use_mfma) {
        rc = pool_dtype == AHPC_F16 ? launch_decode_mfma<f16_t>(p, waves, st) : launch_decode_mfma<bf16_t>(p, waves, st);
    } else
    switch (pool_dtype) {
        case AHPC_F32: rc = launch_decode_d<float>(p, grid, block, st); break;
        case AHPC_F16: rc = launch_decode_d<f16_t>(p, grid, block, st); break;
        default: rc = launch_decode_d<bf16_t>(p, grid, block, st); break;
    }
    if (rc) return rc;
    if (n_chunks > 1) {
        hipLaunchKernelGGL(paged_merge_kernel, egrid, eblock, 0, st, p);
        return static_cast<int>(hipGetLastError());
    }
    return AHPC_OK;
}

int ahpc_hip_paged_decode_noalloc(const void* q, void* o, int qo_dtype, const void* k_pool, const void* v_pool, int pool_dtype,
                                  const int32_t* block_table, const int32_t* seq_lens, const int32_t* batch_rows, int64_t B,
                                  int64_t H, int64_t H_kv, int64_t d, int64_t P, int64_t max_pages, int64_t max_len,
                                  float scale, int64_t chunk_tokens, void* stream) {
    void* ptr = nullptr;
    if (int rc = scratch_of_current_device(&ptr)) return rc;
    // The call below plans the launch and knows what its partials need (with chunk_tokens = 0 usually far less than the
    // bound ahpc_hip_paged_decode_workspace_bytes gives): it refuses, before launching anything, a plan that does not fit
    // the array.  The partials need no clearing between calls: the merge reads, per sequence, exactly the chunks whose
    // decode workgroup wrote them in this call (those that start before the sequence's end).
    const int rc = ahpc_hip_paged_decode_gqa(q, o, qo_dtype, k_pool, v_pool, pool_dtype, block_table, seq_lens, batch_rows, B, H,
                                             H_kv, d, P, max_pages, max_len, scale, chunk_tokens, ptr, AHPC_NOALLOC_SCRATCH_BYTES,
                                             stream);
    return rc == AHPC_ERR_WORKSPACE_TOO_SMALL ? AHPC_ERR_SCRATCH_LIMIT : rc;
}

int ahpc_hip_paged_decode(const void* q, void* o, int qo_dtype, const void* k_pool, const void* v_pool, int pool_dtype,
                          const int32_t* block_table, const int32_t* seq_lens, const int32_t* batch_rows, int64_t B,
                          int64_t H, int64_t d, int64_t P, int64_t max_pages, int64_t max_len, float scale,
                          int64_t chunk_tokens, void* workspace, size_t workspace_bytes, void* stream) {
    return ahpc_hip_paged_decode_gqa(q, o, qo_dtype, k_pool, v_pool, pool_dtype, block_table, seq_lens, batch_rows, B, H, H,
                                     d, P, max_pages, max_len, scale, chunk_tokens, workspace, workspace_bytes, stream);
}

int ahpc_hip_kv_move_pages(void* k_pool, void* v_pool, int pool_dtype, int64_t n_pages, const int32_t* from, const int32_t* to,
                           int64_t n, int64_t H, int64_t d, int64_t P, void* stream) {
    if (n == 0) return AHPC_OK;
    if (!k_pool || !v_pool || !from || !to) return AHPC_ERR_NULL_POINTER;
    if (pool_dtype < AHPC_F32 || pool_dtype > AHPC_BF16) return AHPC_ERR_BAD_DTYPE;
    if (n < 0 || n > 0x7FFFFFFFll || n_pages <= 0 || n_pages > 0x7FFFFFFFll || !dims_ok(H, d, P, 1)) return AHPC_ERR_BAD_SHAPE;
    const int64_t page_bytes = P * H * d * (pool_dtype == AHPC_F32 ? 4 : 2);
    hipLaunchKernelGGL(kv_move_pages_kernel, dim3((unsigned)n, 2), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<unsigned char*>(k_pool), static_cast<unsigned char*>(v_pool), page_bytes, n_pages, from, to, n);
    return static_cast<int>(hipGetLastError());
}

int ahpc_hip_paged_gather_indices(const int32_t* block_table, const int32_t* seq_lens, const int32_t* batch_rows, int64_t B,
                                  int64_t H, int64_t d, int64_t P, int64_t max_pages, int64_t max_len, int64_t* offsets,
                                  void* stream) {
    if (!block_table || !seq_lens || !offsets) return AHPC_ERR_NULL_POINTER;
    if (B <= 0 || max_len <= 0 || max_len > 0x7FFFFFFFll || !dims_ok(H, d, P, max_pages)) return AHPC_ERR_BAD_SHAPE;
    if ((max_len + P - 1) / P > max_pages) return AHPC_ERR_BAD_SHAPE;
    if (B > 0x7FFFFFFFll || (B * max_len + 255) / 256 > 0x7FFFFFFFll) return AHPC_ERR_BAD_SHAPE;  // one thread per reported token
    hipStream_t st = static_cast<hipStream_t>(stream);
    if ((d == 32 || d == 64 || d == 128 || d == 256) && B <= 65535 && H <= 65535) {
        // the decode kernel itself (16-bit pool, one query head per pool head), launched for pool head 0 only and with
        // the chunking of a real decode launch (every sequence cut into equal chunks), reports the rows it addresses
        const int64_t chunk = plan_decode(B, H, 1, (H + 3) / 4, max_len, P, 0).chunk;
        const int64_t n_chunks = (max_len + chunk - 1) / chunk;
        if (n_chunks > 65535) return AHPC_ERR_BAD_SHAPE;
        {
            const int64_t total = B * max_len;
            hipLaunchKernelGGL(fill_i64_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, offsets, total, (int64_t)-1);
            if (hipError_t e = hipGetLastError(); e != hipSuccess) return static_cast<int>(e);
        }
        DecodeParams p{};
        p.table = block_table; p.seq_lens = seq_lens; p.batch_rows = batch_rows;
        p.dump_offsets = offsets;
        p.max_pages = max_pages;
        p.B = (int32_t)B; p.H = (int32_t)H; p.H_kv = (int32_t)H; p.d = (int32_t)d; p.P = (int32_t)P;
        p.d_kernel = (int32_t)d;
        p.chunk_tokens = (int32_t)chunk; p.n_chunks = (int32_t)n_chunks;
        p.balanced = 1;
        p.max_len = (int32_t)max_len;
        const dim3 grid(1, (unsigned)n_chunks, (unsigned)B), block(64);
#define AHPC_DUMP(DD)                                                                                                  \
    if (P == 16) hipLaunchKernelGGL((paged_decode_kernel<f16_t, DD, 16, 1, true>), grid, block, 0, st, p);            \
    else hipLaunchKernelGGL((paged_decode_kernel<f16_t, DD, 0, 1, true>), grid, block, 0, st, p)
        switch (d) {
            case 32: AHPC_DUMP(32); break;
            case 64: AHPC_DUMP(64); break;
            case 128: AHPC_DUMP(128); break;
            default: AHPC_DUMP(256); break;
        }
#undef AHPC_DUMP
        return static_cast<int>(hipGetLastError());
    }
    // head dimensions the decode kernel does not take: the index function of append and read-back
    const int64_t total = B * max_len;
    dim3 block(256), grid((unsigned)((total + 255) / 256));
    hipLaunchKernelGGL(gather_indices_kernel, grid, block, 0, st, block_table, seq_lens, batch_rows, B, (int)H, (int)d,
                       (int)P, max_pages, max_len, offsets);
    return static_cast<int>(hipGetLastError());
}

}  // extern "C"
