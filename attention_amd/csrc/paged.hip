// Paged KV pool kernels: scatter (append), gather (read-back), decode, split merge, index dump.
//
// Pool layout: K and V slabs [page][slot][head][d].  One token of one sequence is H*d contiguous
// elements, so a wavefront reads whole 1-KiB runs: lanes are grouped LPH = d*sizeof(T)/16 per head
// (each lane owns one 16-byte piece of a head's row) and a wavefront covers 64/LPH heads of one
// token with a single 16-byte load per lane.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdlib>
#include <type_traits>

#include "ahpc_device.hpp"

namespace ahpc {

// Element offset of (token t, head 0, lane 0) of table row `row`; -1 when the page is missing.
// Shared by the decode kernel, scatter, gather and the index dump, so that what the dump reports
// is what decode reads.
__device__ __forceinline__ int64_t kv_token_offset(const int32_t* __restrict__ table, int64_t max_pages, int64_t row,
                                                   int t, int P, int H, int d) {
    const int page_idx = t / P;
    const int pos = t - page_idx * P;
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

__global__ void gather_indices_kernel(const int32_t* __restrict__ table, const int32_t* __restrict__ seq_lens,
                                      const int32_t* __restrict__ batch_rows, int64_t B, int H, int d, int P,
                                      int64_t max_pages, int64_t max_len, int64_t* __restrict__ offsets) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= B * max_len) return;
    const int64_t b = idx / max_len;
    const int t = (int)(idx - b * max_len);
    const int64_t row = batch_rows ? batch_rows[b] : b;
    offsets[idx] = t < seq_lens[row] ? kv_token_offset(table, max_pages, row, t, P, H, d) : -1;
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
    float* part_ml;   // [B][n_chunks][H][2]  (m in log2 units, l)
    int64_t max_pages;
    int32_t B, H, d, P;
    int32_t chunk_tokens, n_chunks;
    int32_t max_len;
    int32_t qo_dtype;
    float scale_log2;
};

__device__ __forceinline__ float load_qo(const void* base, int dtype, int64_t i) {
    if (dtype == AHPC_F32) return static_cast<const float*>(base)[i];
    if (dtype == AHPC_F16) return (float)static_cast<const f16_t*>(base)[i];
    return (float)static_cast<const bf16_t*>(base)[i];
}

__device__ __forceinline__ void store_qo(void* base, int dtype, int64_t i, float x) {
    if (dtype == AHPC_F32) static_cast<float*>(base)[i] = x;
    else if (dtype == AHPC_F16) static_cast<f16_t*>(base)[i] = (f16_t)x;
    else static_cast<bf16_t*>(base)[i] = (bf16_t)x;
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

constexpr int kDecodeBatch = 8;  // tokens whose K and V rows are in flight together, per lane

// T: pool element type.  D: head dimension.  A lane owns EPL = 16/sizeof(T) consecutive lanes of
// one head.  Grid: (chunk, batch entry, head group); every wavefront works on its own heads and
// needs no LDS and no barrier.
template <typename T, int D>
__global__ __launch_bounds__(256) void paged_decode_kernel(const DecodeParams p) {
    constexpr int EPL = 16 / (int)sizeof(T);
    constexpr int LPH = D / EPL;
    constexpr int HPW = kWave / LPH;
    constexpr bool kPacked = sizeof(T) == 2;
    typedef typename std::conditional<kPacked, T, f16_t>::type TP;  // placeholder type for the unused branch

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int waves = blockDim.x >> 6;
    const int chunk = blockIdx.x;
    const int b = blockIdx.y;
    const int h_raw = (blockIdx.z * waves + wave) * HPW + lane / LPH;
    const bool head_ok = h_raw < p.H;
    const int h = head_ok ? h_raw : p.H - 1;
    const int e0 = (lane % LPH) * EPL;

    const int64_t row = p.batch_rows ? p.batch_rows[b] : b;
    const int L = p.seq_lens[row] < p.max_len ? p.seq_lens[row] : p.max_len;
    const int t0 = chunk * p.chunk_tokens;
    if (t0 >= L) {
        // an empty sequence still owns an output row: zeros (with several chunks the merge writes it)
        if (chunk == 0 && p.n_chunks == 1 && head_ok) {
            const int64_t oi = ((int64_t)b * p.H + h) * D + e0;
#pragma unroll
            for (int e = 0; e < EPL; ++e) store_qo(p.o, p.qo_dtype, oi + e, 0.0f);
        }
        return;
    }
    const int t1 = (t0 + p.chunk_tokens) < L ? (t0 + p.chunk_tokens) : L;

    // query piece of this lane
    float qf[EPL];
    uint32_t qp[4];
    {
        const int64_t qi = ((int64_t)b * p.H + h) * D + e0;
#pragma unroll
        for (int e = 0; e < EPL; ++e) qf[e] = load_qo(p.q, p.qo_dtype, qi + e);
        if (kPacked) {
#pragma unroll
            for (int i = 0; i < 4; ++i) qp[i] = pack2<TP>(qf[2 * i], qf[2 * i + 1]);
        }
    }

    const T* const kp = static_cast<const T*>(p.k_pool) + (int64_t)h * D + e0;
    const T* const vp = static_cast<const T*>(p.v_pool) + (int64_t)h * D + e0;

    auto token_offset = [&](int t) -> int64_t {
        // tokens past the chunk end re-read the last valid token (their score is masked below);
        // a missing page reads page 0 (the host never hands out such a table)
        const int tc = t < t1 ? t : t1 - 1;
        const int64_t off = kv_token_offset(p.table, p.max_pages, row, tc, p.P, p.H, D);
        return off < 0 ? 0 : off;
    };

    u32x4 kreg[kDecodeBatch], vreg[kDecodeBatch];
    auto load_batch = [&](int tb) {
#pragma unroll
        for (int i = 0; i < kDecodeBatch; ++i) {
            const int64_t off = token_offset(tb + i);
            kreg[i] = *reinterpret_cast<const u32x4*>(kp + off);
            vreg[i] = *reinterpret_cast<const u32x4*>(vp + off);
        }
    };

    float acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    const float c = p.scale_log2;

    load_batch(t0);
    for (int tb = t0; tb < t1; tb += kDecodeBatch) {
        u32x4 kc[kDecodeBatch], vc[kDecodeBatch];
#pragma unroll
        for (int i = 0; i < kDecodeBatch; ++i) {
            kc[i] = kreg[i];
            vc[i] = vreg[i];
        }
        if (tb + kDecodeBatch < t1) load_batch(tb + kDecodeBatch);

        float s[kDecodeBatch];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < kDecodeBatch; ++i) {
            float part = 0.0f;
            if (kPacked) {
#pragma unroll
                for (int w = 0; w < 4; ++w) part = dot2<TP>(qp[w], kc[i][w], part);
            } else {
#pragma unroll
                for (int w = 0; w < 4; ++w) part = __builtin_fmaf(qf[w % EPL], as_f32(kc[i][w]), part);
            }
            part = head_allreduce<LPH>(part);
            s[i] = (tb + i < t1) ? part * c : -INFINITY;
            mx = fmaxf(mx, s[i]);
        }
        const float m_new = fmaxf(m, mx);              // finite: the batch holds at least one token
        const float alpha = fast_exp2(m - m_new);      // first batch: exp2(-inf) = 0
        float sum = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[e] *= alpha;
#pragma unroll
        for (int i = 0; i < kDecodeBatch; ++i) {
            const float w = fast_exp2(s[i] - m_new);
            sum += w;
            if (kPacked) {
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    acc[(2 * x) % EPL] = __builtin_fmaf(w, lo_f32<TP>(vc[i][x]), acc[(2 * x) % EPL]);
                    acc[(2 * x + 1) % EPL] = __builtin_fmaf(w, hi_f32<TP>(vc[i][x]), acc[(2 * x + 1) % EPL]);
                }
            } else {
#pragma unroll
                for (int x = 0; x < 4; ++x) acc[x % EPL] = __builtin_fmaf(w, as_f32(vc[i][x]), acc[x % EPL]);
            }
        }
        l = l * alpha + sum;
        m = m_new;
    }

    if (!head_ok) return;
    if (p.n_chunks == 1) {
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        const int64_t oi = ((int64_t)b * p.H + h) * D + e0;
#pragma unroll
        for (int e = 0; e < EPL; ++e) store_qo(p.o, p.qo_dtype, oi + e, acc[e] * inv);
    } else {
        const int64_t slot = ((int64_t)b * p.n_chunks + chunk) * p.H + h;
        f32x4* dst = reinterpret_cast<f32x4*>(p.part_o + slot * D + e0);
#pragma unroll
        for (int e = 0; e < EPL; e += 4) dst[e / 4] = f32x4{acc[e], acc[e + 1], acc[e + 2], acc[e + 3]};
        if (lane % LPH == 0) {
            p.part_ml[slot * 2] = m;
            p.part_ml[slot * 2 + 1] = l;
        }
    }
}

// One thread per output element: folds the chunk partials of its (batch entry, head) with
// m' = max(m, m2), l' = l*2^(m-m') + l2*2^(m2-m') and the same factors on the accumulators.
__global__ void paged_merge_kernel(const DecodeParams p) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t hd = (int64_t)p.H * p.d;
    if (idx >= p.B * hd) return;
    const int64_t b = idx / hd;
    const int64_t he = idx - b * hd;
    const int h = (int)(he / p.d);
    const int64_t row = p.batch_rows ? p.batch_rows[b] : b;
    const int L = p.seq_lens[row] < p.max_len ? p.seq_lens[row] : p.max_len;
    const int n = (L + p.chunk_tokens - 1) / p.chunk_tokens;
    float m = -INFINITY, l = 0.0f, acc = 0.0f;
    for (int ci = 0; ci < n; ++ci) {
        const int64_t slot = (b * p.n_chunks + ci) * p.H + h;
        const float m2 = p.part_ml[slot * 2];
        const float l2 = p.part_ml[slot * 2 + 1];
        const float o2 = p.part_o[slot * p.d + (he - (int64_t)h * p.d)];
        const float m_new = fmaxf(m, m2);
        const float f1 = fast_exp2(m - m_new);
        const float f2 = fast_exp2(m2 - m_new);
        l = l * f1 + l2 * f2;
        acc = acc * f1 + o2 * f2;
        m = m_new;
    }
    store_qo(p.o, p.qo_dtype, idx, l > 0.0f ? acc / l : 0.0f);
}

static int env_int(const char* name, int dflt) {
    const char* e = std::getenv(name);
    return e ? std::atoi(e) : dflt;
}

// Waves per decode workgroup (each wave works alone; this only sets how many heads travel together).
static int decode_waves() {
    static const int v = env_int("AHPC_DECODE_WAVES", 0);
    return v;
}

static int64_t pick_chunk_tokens(int64_t B, int64_t H, int64_t max_len, int64_t P, int64_t requested) {
    int64_t chunk = requested;
    if (chunk <= 0) {
        // enough workgroups to keep every CU busy several times over, while the fp32 partials stay
        // below ~1% of the K/V bytes of a chunk
        chunk = 256;
        while (chunk > 128 && B * ((max_len + chunk - 1) / chunk) * ((H + 3) / 4) < 4096) chunk /= 2;
    }
    chunk = ((chunk + P - 1) / P) * P;
    if (chunk < P) chunk = P;
    return chunk;
}

template <typename T>
static int launch_decode_d(const DecodeParams& p, dim3 grid, dim3 block, hipStream_t st) {
    switch (p.d) {
        case 32: hipLaunchKernelGGL((paged_decode_kernel<T, 32>), grid, block, 0, st, p); break;
        case 64: hipLaunchKernelGGL((paged_decode_kernel<T, 64>), grid, block, 0, st, p); break;
        case 128: hipLaunchKernelGGL((paged_decode_kernel<T, 128>), grid, block, 0, st, p); break;
        case 256: hipLaunchKernelGGL((paged_decode_kernel<T, 256>), grid, block, 0, st, p); break;
        default: return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
    }
    return static_cast<int>(hipGetLastError());
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
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (in_dtype) {
        case AHPC_F32: return scatter_out<float>(pool_dtype, k_new, v_new, k_pool, v_pool, block_table, max_pages, token_row, token_pos, row0, pos0, n_tokens, (int)H, (int)d, (int)P, st);
        case AHPC_F16: return scatter_out<f16_t>(pool_dtype, k_new, v_new, k_pool, v_pool, block_table, max_pages, token_row, token_pos, row0, pos0, n_tokens, (int)H, (int)d, (int)P, st);
        case AHPC_BF16: return scatter_out<bf16_t>(pool_dtype, k_new, v_new, k_pool, v_pool, block_table, max_pages, token_row, token_pos, row0, pos0, n_tokens, (int)H, (int)d, (int)P, st);
        default: return AHPC_ERR_BAD_DTYPE;
    }
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
    const int64_t chunk = pick_chunk_tokens(B, H, max_len, P, chunk_tokens);
    const int64_t n_chunks = (max_len + chunk - 1) / chunk;
    if (n_chunks <= 1) return 0;
    return (size_t)(B * n_chunks * H * (d + 2)) * sizeof(float);
}

int ahpc_hip_paged_decode(const void* q, void* o, int qo_dtype, const void* k_pool, const void* v_pool, int pool_dtype,
                          const int32_t* block_table, const int32_t* seq_lens, const int32_t* batch_rows, int64_t B,
                          int64_t H, int64_t d, int64_t P, int64_t max_pages, int64_t max_len, float scale,
                          int64_t chunk_tokens, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !o || !k_pool || !v_pool || !block_table || !seq_lens) return AHPC_ERR_NULL_POINTER;
    if (qo_dtype < AHPC_F32 || qo_dtype > AHPC_BF16 || pool_dtype < AHPC_F32 || pool_dtype > AHPC_BF16) return AHPC_ERR_BAD_DTYPE;
    if (B <= 0 || B > 65535 || max_len <= 0 || !dims_ok(H, d, P, max_pages)) return AHPC_ERR_BAD_SHAPE;
    if ((max_len + P - 1) / P > max_pages) return AHPC_ERR_BAD_SHAPE;
    if (d != 32 && d != 64 && d != 128 && d != 256) return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
    if ((reinterpret_cast<uintptr_t>(k_pool) & 15u) || (reinterpret_cast<uintptr_t>(v_pool) & 15u)) return AHPC_ERR_BAD_ALIGNMENT;
    if (!(scale > 0.0f)) scale = 1.0f / std::sqrt((float)d);

    const int64_t chunk = pick_chunk_tokens(B, H, max_len, P, chunk_tokens);
    const int64_t n_chunks = (max_len + chunk - 1) / chunk;
    const size_t need = n_chunks > 1 ? (size_t)(B * n_chunks * H * (d + 2)) * sizeof(float) : 0;
    if (need > 0 && (!workspace || workspace_bytes < need)) return AHPC_ERR_WORKSPACE_TOO_SMALL;
    if (n_chunks > 65535) return AHPC_ERR_BAD_SHAPE;

    DecodeParams p{};
    p.q = q; p.o = o; p.k_pool = k_pool; p.v_pool = v_pool;
    p.table = block_table; p.seq_lens = seq_lens; p.batch_rows = batch_rows;
    p.part_o = static_cast<float*>(workspace);
    p.part_ml = p.part_o ? p.part_o + B * n_chunks * H * d : nullptr;
    p.max_pages = max_pages;
    p.B = (int32_t)B; p.H = (int32_t)H; p.d = (int32_t)d; p.P = (int32_t)P;
    p.chunk_tokens = (int32_t)chunk; p.n_chunks = (int32_t)n_chunks;
    p.max_len = (int32_t)max_len;
    p.qo_dtype = qo_dtype;
    p.scale_log2 = scale * kLog2e;

    hipStream_t st = static_cast<hipStream_t>(stream);
    const int elem = pool_dtype == AHPC_F32 ? 4 : 2;
    const int lph = (int)(d * elem / 16);
    if (lph < 1 || lph > 64) return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
    const int hpw = 64 / lph;
    int waves = decode_waves();
    if (waves < 1 || waves > 4) waves = 1;
    const int64_t heads_per_wg = (int64_t)hpw * waves;
    const int64_t head_groups = (H + heads_per_wg - 1) / heads_per_wg;
    if (head_groups > 65535) return AHPC_ERR_BAD_SHAPE;

    const int64_t total = B * H * d;
    dim3 eblock(256), egrid((unsigned)((total + 255) / 256));

    dim3 grid((unsigned)n_chunks, (unsigned)B, (unsigned)head_groups), block(64 * waves);
    int rc;
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

int ahpc_hip_paged_gather_indices(const int32_t* block_table, const int32_t* seq_lens, const int32_t* batch_rows, int64_t B,
                                  int64_t H, int64_t d, int64_t P, int64_t max_pages, int64_t max_len, int64_t* offsets,
                                  void* stream) {
    if (!block_table || !seq_lens || !offsets) return AHPC_ERR_NULL_POINTER;
    if (B <= 0 || max_len <= 0 || !dims_ok(H, d, P, max_pages)) return AHPC_ERR_BAD_SHAPE;
    if ((max_len + P - 1) / P > max_pages) return AHPC_ERR_BAD_SHAPE;
    const int64_t total = B * max_len;
    dim3 block(256), grid((unsigned)((total + 255) / 256));
    hipLaunchKernelGGL(gather_indices_kernel, grid, block, 0, static_cast<hipStream_t>(stream), block_table, seq_lens,
                       batch_rows, B, (int)H, (int)d, (int)P, max_pages, max_len, offsets);
    return static_cast<int>(hipGetLastError());
}

}  // extern "C"
