// FlashAttention forward entry points: argument checks, kernel choice, launches.
#include <hip/hip_runtime.h>

#include <cmath>
#include <atomic>
#include <cstdlib>
#include <functional>
#include <mutex>

#include "ahpc_device.hpp"
#include "flash_fwd_mfma.hpp"
#include "flash_fwd_wide.hpp"
#include "mask_pack.hpp"
#include "flash_fwd_f32_mfma.hpp"
#include "tuning.hpp"

namespace ahpc {

constexpr int kMaxPersistentDevices = 64;

// ---------------------------------------------------------------------------------------------
// fp32-FMA kernel: any dtype, any head dimension up to 256, optional dense mask.  One thread owns
// one query row (q and the output accumulator stay in registers); a workgroup of 128 rows of the
// same (sequence, head) shares key/value tiles of 16 rows staged in LDS as fp32.  This is the
// accuracy path (fp32 inputs, 1e-4 tolerance) and the fallback for shapes the MFMA kernel does
// not take; it is not tuned.
struct SimpleParams {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    const int32_t* cu_seqlens;
    const float* mask;          // [B,N,N] or null
    int64_t stride_b, stride_n, stride_h;           // Q and O
    int64_t kv_stride_b, kv_stride_n, kv_stride_h;  // K and V
    int32_t N, H, d;
    int32_t kv_group;           // query heads per key/value head
    float scale;
    int32_t causal;
};

constexpr int kSimpleRows = 128;
constexpr int kSimpleKeys = 16;

template <typename T, int DP, bool VARLEN>
__global__ __launch_bounds__(kSimpleRows) void flash_fwd_simple_kernel(const SimpleParams p) {
    __shared__ float sk[kSimpleKeys][DP];
    __shared__ float sv[kSimpleKeys][DP];

    const int tid = threadIdx.x;
    const int h = blockIdx.y, b = blockIdx.z;
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
    const int row0 = blockIdx.x * kSimpleRows;
    if (row0 >= L) return;
    const int n = row0 + tid;
    const bool active = n < L;
    const int d = p.d;

    const T* gq = static_cast<const T*>(p.q) + base;
    const T* gk = static_cast<const T*>(p.k) + kv_base;
    const T* gv = static_cast<const T*>(p.v) + kv_base;

    float qv[DP], acc[DP];
#pragma unroll
    for (int e = 0; e < DP; ++e) {
        qv[e] = (active && e < d) ? Storage<T>::load(gq + (int64_t)n * p.stride_n + e) : 0.0f;
        acc[e] = 0.0f;
    }
    float m = -INFINITY, l = 0.0f;

    for (int i = tid; i < kSimpleKeys * DP; i += kSimpleRows) {
        (&sk[0][0])[i] = 0.0f;
        (&sv[0][0])[i] = 0.0f;
    }

    int k_end = L;
    if (p.causal) k_end = (row0 + kSimpleRows) < L ? (row0 + kSimpleRows) : L;
    const float* mrow = (p.mask && active) ? p.mask + ((int64_t)b * p.N + n) * p.N : nullptr;

    for (int k0 = 0; k0 < k_end; k0 += kSimpleKeys) {
        __syncthreads();
        for (int i = tid; i < kSimpleKeys * d; i += kSimpleRows) {
            const int kr = i / d, e = i - kr * d;
            const int key = k0 + kr;
            float kx = 0.0f, vx = 0.0f;
            if (key < L) {
                kx = Storage<T>::load(gk + (int64_t)key * p.kv_stride_n + e);
                vx = Storage<T>::load(gv + (int64_t)key * p.kv_stride_n + e);
            }
            sk[kr][e] = kx;
            sv[kr][e] = vx;
        }
        __syncthreads();
        if (!active) continue;
        for (int kr = 0; kr < kSimpleKeys; ++kr) {
            const int key = k0 + kr;
            if (key >= L) break;
            if (p.causal && key > n) break;
            if (mrow && mrow[key] == 0.0f) continue;
            float dot = 0.0f;
#pragma unroll
            for (int e = 0; e < DP; ++e) dot = __builtin_fmaf(qv[e], sk[kr][e], dot);
            const float s = dot * p.scale;
            if (s > m) {
                const float a = __expf(m - s);  // first key: exp(-inf) = 0
                l = l * a + 1.0f;
#pragma unroll
                for (int e = 0; e < DP; ++e) acc[e] = __builtin_fmaf(acc[e], a, sv[kr][e]);
                m = s;
            } else {
                const float w = __expf(s - m);
                l += w;
#pragma unroll
                for (int e = 0; e < DP; ++e) acc[e] = __builtin_fmaf(w, sv[kr][e], acc[e]);
            }
        }
    }
    if (!active) return;
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    T* go = static_cast<T*>(p.o) + base + (int64_t)n * p.stride_n;
#pragma unroll
    for (int e = 0; e < DP; ++e)
        if (e < d) Storage<T>::store(go + e, acc[e] * inv);
}

template <typename T, bool VARLEN>
static int launch_simple(const SimpleParams& p, int64_t B, hipStream_t stream) {
    dim3 grid((unsigned)((p.N + kSimpleRows - 1) / kSimpleRows), (unsigned)p.H, (unsigned)B);
    dim3 block(kSimpleRows);
    if (p.d <= 16) hipLaunchKernelGGL((flash_fwd_simple_kernel<T, 16, VARLEN>), grid, block, 0, stream, p);
    else if (p.d <= 32) hipLaunchKernelGGL((flash_fwd_simple_kernel<T, 32, VARLEN>), grid, block, 0, stream, p);
    else if (p.d <= 64) hipLaunchKernelGGL((flash_fwd_simple_kernel<T, 64, VARLEN>), grid, block, 0, stream, p);
    else if (p.d <= 128) hipLaunchKernelGGL((flash_fwd_simple_kernel<T, 128, VARLEN>), grid, block, 0, stream, p);
    else if (p.d <= 256) hipLaunchKernelGGL((flash_fwd_simple_kernel<T, 256, VARLEN>), grid, block, 0, stream, p);
    else return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
    return static_cast<int>(hipGetLastError());
}

template <bool VARLEN>
static int dispatch_simple(int dtype, const SimpleParams& p, int64_t B, hipStream_t stream) {
    switch (dtype) {
        case AHPC_F32: return launch_simple<float, VARLEN>(p, B, stream);
        case AHPC_F16: return launch_simple<f16_t, VARLEN>(p, B, stream);
        case AHPC_BF16: return launch_simple<bf16_t, VARLEN>(p, B, stream);
        default: return AHPC_ERR_BAD_DTYPE;
    }
}

// ---------------------------------------------------------------------------------------------
// Query rows per workgroup of the 16-bit forward without a mask: 128 (flash_fwd_mfma.hpp, two workgroups per CU) or 256
// (flash_fwd_wide.hpp, one persistent workgroup per CU: dense launches at d = 64 and 128).  The tuning value when it
// names one, else by shape.  Timed on MI355X over dense shapes from 1x256x32 to 1x32768x32: 256 rows is 3-8 % faster at
// d = 128 from 2048 tokens on once every CU gets a workgroup, and 4-30 % slower on shorter sequences, smaller launches
// and at d = 64 (where three 128-row workgroups share a CU).
static int flash_rows_for(int D, bool varlen, int64_t B, int64_t N, int64_t H) {
    if (D == 256 || varlen) return kFlashRows;
    const int64_t t = tuning().flash_rows.load();
    if (t == kFlashRows || t == kFlashWideRows) return (int)t;
    if (D != 128 || N < 2048) return kFlashRows;
    return B * H * ((N + kFlashWideRows - 1) / kFlashWideRows) >= 256 ? kFlashWideRows : kFlashRows;
}

// Workgroups of a persistent launch: one per CU, a multiple of 8 (a workgroup's block ids then all map to the XCD it
// runs on), and never more than there are block ids.
static int persistent_grid(int n_block_ids) {
    static std::atomic<int> cus[kMaxPersistentDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxPersistentDevices) dev = 0;
    int n = cus[dev].load();
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 8) {
            (void)hipGetLastError();
            n = 8;
        }
        n -= n % 8;
        cus[dev].store(n);
    }
    return n_block_ids < n ? n_block_ids : n;
}

template <typename T, int D, bool VARLEN>
static int launch_mfma(FlashParams p, int64_t B, bool causal, hipStream_t stream) {
    if constexpr (D != 256 && !VARLEN) {
        if (flash_rows_for(D, VARLEN, B, p.N, p.H) == kFlashWideRows) {
            if (int rc = flash_plan_launch(p, B, causal, kFlashWideRows, tuning().flash_pair_min_tiles.load(), false)) return rc;
            dim3 grid((unsigned)persistent_grid(p.n_block_ids)), block(64 * kFlashWideWaves);
            if (causal) hipLaunchKernelGGL((flash_fwd_wide_kernel<T, D, true>), grid, block, 0, stream, p);
            else hipLaunchKernelGGL((flash_fwd_wide_kernel<T, D, false>), grid, block, 0, stream, p);
            return static_cast<int>(hipGetLastError());
        }
    }
    if (int rc = flash_plan_launch(p, B, causal, kFlashRows, tuning().flash_pair_min_tiles.load(), VARLEN)) return rc;
    dim3 grid((unsigned)(p.blocks_per_xcd * 8)), block(kFlashThreads);
    if (causal) hipLaunchKernelGGL((flash_fwd_mfma_kernel<T, D, true, VARLEN>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((flash_fwd_mfma_kernel<T, D, false, VARLEN>), grid, block, 0, stream, p);
    return static_cast<int>(hipGetLastError());
}

template <typename T, int D, int MASK>
static int launch_mfma_masked(FlashParams p, int64_t B, bool causal, hipStream_t stream) {
    if (int rc = flash_plan_launch(p, B, causal, kFlashRows, tuning().flash_pair_min_tiles.load(), false)) return rc;
    dim3 grid((unsigned)(p.blocks_per_xcd * 8)), block(kFlashThreads);
    if (causal) hipLaunchKernelGGL((flash_fwd_mfma_masked_kernel<T, D, true, MASK>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((flash_fwd_mfma_masked_kernel<T, D, false, MASK>), grid, block, 0, stream, p);
    return static_cast<int>(hipGetLastError());
}

template <typename T, int MASK>
static int dispatch_mfma_masked(const FlashParams& p, int64_t B, int d, bool causal, hipStream_t stream) {
    if (d == 128) return launch_mfma_masked<T, 128, MASK>(p, B, causal, stream);
    if (d == 64) return launch_mfma_masked<T, 64, MASK>(p, B, causal, stream);
    if constexpr (MASK == 2) {  // the packed mask only: the in-place mask's 32 registers do not fit beside d = 256
        if (d == 256) return launch_mfma_masked<T, 256, MASK>(p, B, causal, stream);
    }
    return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
}

// Packs a dense fp32 mask [B,N,N] into one bit per (query, key): word [(b * n_kt + tile) * N + query] holds the 64
// keys of the tile, bit j set = mask[b][query][64 * tile + j] != 0 (keys at or beyond N: clear).  A wavefront takes
// 64 queries x 64 keys: per query one coalesced 256-byte read and a ballot; lane r keeps the word of query r, and the
// 64 words leave as one coalesced 512-byte store.  Consecutive wavefronts take consecutive tiles of the same queries.
// With bits_t given the same pass also writes the transposed layout the backward's dK/dV kernels read: word
// [(b * n_rb + query block) * N + key] holds the block's 64 queries, bit r set = mask[b][64 * block + r][key] != 0
// (lane = key collects its own word from the values it loads).
constexpr int kMaskPackThreads = 256;
template <bool TRANSPOSED>
__global__ __launch_bounds__(kMaskPackThreads) void flash_mask_pack_kernel(const float* __restrict__ mask, uint64_t* __restrict__ bits,
                                                                            uint64_t* __restrict__ bits_t, int N, int n_kt, int n_rb,
                                                                            int64_t n_units) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t unit = (int64_t)blockIdx.x * (kMaskPackThreads / kWave) + (threadIdx.x >> 6);
    if (unit >= n_units) return;
    const int kt = (int)(unit % n_kt);
    const int rb = (int)((unit / n_kt) % n_rb);
    const int b = (int)(unit / ((int64_t)n_kt * n_rb));
    const int key = 64 * kt + lane;
    const float* const src = mask + (int64_t)b * N * N + (key < N ? key : 0);
    uint64_t mine = 0, mine_t = 0;
#pragma unroll 16
    for (int r = 0; r < 64; ++r) {
        const int row = 64 * rb + r;
        const float m = (row < N && key < N) ? __builtin_nontemporal_load(src + (int64_t)row * N) : 0.0f;  // read once
        const uint64_t word = __builtin_amdgcn_ballot_w64(m != 0.0f);
        if (lane == r) mine = word;
        if constexpr (TRANSPOSED) mine_t |= (uint64_t)(m != 0.0f) << r;
    }
    const int row = 64 * rb + lane;
    if (row < N) bits[((int64_t)b * n_kt + kt) * N + row] = mine;
    if constexpr (TRANSPOSED) {
        if (key < N) bits_t[((int64_t)b * n_rb + rb) * N + key] = mine_t;
    }
}

// The packed copy of a mask lives in device memory that the library owns: one buffer per device, grown on demand and kept
// until the process ends (B * N * ceil(N / 64) * 8 bytes per layout: an eighth of a byte per mask element).  Calls on one
// device share it: `done` is recorded behind the last launch that reads it, and the next call's stream waits for it
// before the buffer is overwritten; the mutex covers the whole of that.
struct MaskScratch {
    std::mutex mu;
    void* ptr = nullptr;
    size_t bytes = 0;
    hipEvent_t done = nullptr;
};
constexpr int kMaxDevices = 64;
constexpr size_t kMaskScratchLimit = size_t(1) << 30;  // larger masks are read in place
static MaskScratch g_mask_scratch[kMaxDevices];

// Packs `mask` (with_transposed: both layouts) and runs launch_on_bits on the packed copy.  AHPC_OK + *launched = false:
// not possible here (stream under capture, no memory, mask too large), nothing was launched and the caller takes another
// path.
int with_packed_mask(const float* mask, int64_t B, int64_t N, bool with_transposed, hipStream_t stream, bool* launched,
                     const std::function<int(const PackedMask&)>& launch_on_bits) {
    *launched = false;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return AHPC_OK;  // allocation and cross-stream waits do not belong into a captured graph
    }
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return AHPC_OK;
    const int64_t n_kt = (N + 63) / 64, n_rb = (N + 63) / 64;
    const size_t one = (size_t)B * (size_t)n_kt * (size_t)N * sizeof(uint64_t);
    const size_t need = with_transposed ? 2 * one : one;
    if (need > kMaskScratchLimit) return AHPC_OK;
    MaskScratch& sc = g_mask_scratch[dev];
    std::lock_guard<std::mutex> lock(sc.mu);
    if (!sc.done && hipEventCreateWithFlags(&sc.done, hipEventDisableTiming) != hipSuccess) {
        sc.done = nullptr;
        (void)hipGetLastError();
        return AHPC_OK;
    }
    if (need > sc.bytes) {
        if (hipError_t e = hipEventSynchronize(sc.done); e != hipSuccess) return static_cast<int>(e);  // the old buffer's last reader
        if (sc.ptr) (void)hipFree(sc.ptr);
        sc.ptr = nullptr;
        sc.bytes = 0;
        if (hipMalloc(&sc.ptr, need) != hipSuccess) {
            sc.ptr = nullptr;
            (void)hipGetLastError();
            return AHPC_OK;
        }
        sc.bytes = need;
    }
    if (hipError_t e = hipStreamWaitEvent(stream, sc.done, 0); e != hipSuccess) return static_cast<int>(e);
    const int64_t n_units = B * n_rb * n_kt;
    const int64_t blocks = (n_units + kMaskPackThreads / kWave - 1) / (kMaskPackThreads / kWave);
    if (blocks > 0x7FFFFFFFll) return AHPC_OK;
    PackedMask pm{};
    pm.bits = static_cast<const uint64_t*>(sc.ptr);
    pm.bits_t = with_transposed ? pm.bits + one / sizeof(uint64_t) : nullptr;
    pm.tiles = (int32_t)n_kt;
    if (with_transposed)
        hipLaunchKernelGGL(flash_mask_pack_kernel<true>, dim3((unsigned)blocks), dim3(kMaskPackThreads), 0, stream, mask,
                           const_cast<uint64_t*>(pm.bits), const_cast<uint64_t*>(pm.bits_t), (int)N, (int)n_kt, (int)n_rb, n_units);
    else
        hipLaunchKernelGGL(flash_mask_pack_kernel<false>, dim3((unsigned)blocks), dim3(kMaskPackThreads), 0, stream, mask,
                           const_cast<uint64_t*>(pm.bits), nullptr, (int)N, (int)n_kt, (int)n_rb, n_units);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return static_cast<int>(e);
    *launched = true;
    const int rc = launch_on_bits(pm);
    const hipError_t e = hipEventRecord(sc.done, stream);
    return rc != AHPC_OK ? rc : static_cast<int>(e);
}

// The forward on a packed mask.
template <typename Launch>
static int forward_on_packed_mask(FlashParams p, const float* mask, int64_t B, hipStream_t stream, bool* launched,
                                  Launch launch_on_bits) {
    return with_packed_mask(mask, B, p.N, false, stream, launched, [&](const PackedMask& pm) {
        p.mask = nullptr;
        p.mask_bits = pm.bits;
        p.mask_kt = pm.tiles;
        return launch_on_bits(p);
    });
}

template <typename T, bool VARLEN>
static int dispatch_mfma(const FlashParams& p, int64_t B, int d, bool causal, hipStream_t stream) {
    if (d == 128) return launch_mfma<T, 128, VARLEN>(p, B, causal, stream);
    if (d == 64) return launch_mfma<T, 64, VARLEN>(p, B, causal, stream);
    if (d == 256) return launch_mfma<T, 256, VARLEN>(p, B, causal, stream);
    return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
}

static bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

struct Strides {
    int64_t b, n, h;
};

// The head dimension a matrix-core kernel is instantiated for: 64 or 128 (the 16-bit forward without a mask: also 256),
// the tensors' own or the next larger one (the kernels then compute with columns that contribute nothing,
// FlashParams::d_real).
static int kernel_head_dim(int64_t d) { return d <= 64 ? 64 : d <= 128 ? 128 : 256; }

// max_d: 256 for the forward, whose instantiation for 256 keeps one workgroup per CU (its operands need the accumulation
// registers as a second register file, and 128 KiB of LDS); 128 otherwise.
static bool mfma_eligible(int dtype, int64_t d, const void* q, const void* k, const void* v, const void* o,
                          const Strides& sq, const Strides& skv, int64_t max_d = 128) {
    if (dtype != AHPC_F16 && dtype != AHPC_BF16) return false;
    if (d < 8 || d > max_d || (d % 8)) return false;  // rows of whole 16-byte pieces
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o)) return false;
    if ((sq.b % 8) || (sq.n % 8) || (sq.h % 8) || (skv.b % 8) || (skv.n % 8) || (skv.h % 8)) return false;
    // a key tile is addressed with 32-bit byte offsets from its first row, and rows must not overlap
    return sq.n >= d && skv.n >= d && skv.n < (int64_t(1) << 24);
}

// fp32 tensors on the matrix cores: kernels for d = 64, 128 and 256, 16-byte aligned rows.
static bool f32_mfma_eligible(int dtype, int64_t d, const void* q, const void* k, const void* v, const void* o,
                              const Strides& sq, const Strides& skv) {
    if (dtype != AHPC_F32 || d < 4 || d > 256 || (d % 4)) return false;  // rows of whole 16-byte pieces
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o)) return false;
    if ((sq.b % 4) || (sq.n % 4) || (sq.h % 4) || (skv.b % 4) || (skv.n % 4) || (skv.h % 4)) return false;
    // a key tile is addressed with 32-bit byte offsets from its first row, and rows must not overlap
    return sq.n >= d && skv.n >= d && skv.n < (int64_t(1) << 24);
}

template <bool VARLEN, bool MASKED>
static int launch_f32_mfma(FlashParams p, int64_t B, int d, bool causal, hipStream_t stream) {
    if (int rc = flash_plan_launch(p, B, causal, kFlashRows, tuning().flash_pair_min_tiles.load(), VARLEN)) return rc;
    dim3 grid((unsigned)(p.blocks_per_xcd * 8)), block(kFlashThreads);
    if (d == 256) {  // (one workgroup per CU: registers and LDS of twice the size)
        if (causal) hipLaunchKernelGGL((flash_fwd_f32_mfma_kernel<256, true, VARLEN, MASKED>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((flash_fwd_f32_mfma_kernel<256, false, VARLEN, MASKED>), grid, block, 0, stream, p);
    } else if (d == 128) {
        if (causal) hipLaunchKernelGGL((flash_fwd_f32_mfma_kernel<128, true, VARLEN, MASKED>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((flash_fwd_f32_mfma_kernel<128, false, VARLEN, MASKED>), grid, block, 0, stream, p);
    } else {
        if (causal) hipLaunchKernelGGL((flash_fwd_f32_mfma_kernel<64, true, VARLEN, MASKED>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((flash_fwd_f32_mfma_kernel<64, false, VARLEN, MASKED>), grid, block, 0, stream, p);
    }
    return static_cast<int>(hipGetLastError());
}

static int check_dense(const void* q, const void* k, const void* v, void* o, int dtype, int64_t B, int64_t N, int64_t H,
                       int64_t H_kv, int64_t d, const Strides& sq, const Strides& skv) {
    if (!q || !k || !v || !o) return AHPC_ERR_NULL_POINTER;
    if (dtype < AHPC_F32 || dtype > AHPC_BF16) return AHPC_ERR_BAD_DTYPE;
    if (B <= 0 || N <= 0 || H <= 0 || d <= 0 || H_kv <= 0) return AHPC_ERR_BAD_SHAPE;
    if (H % H_kv) return AHPC_ERR_BAD_SHAPE;  // every K/V head serves the same number of query heads
    if (B > 65535 || H > 65535 || N > 0x7FFFFF00ll) return AHPC_ERR_BAD_SHAPE;
    if (d > 256) return AHPC_ERR_UNSUPPORTED_HEAD_DIM;
    if (sq.n < d || sq.h < d || sq.b < 0 || skv.n < d || skv.h < d || skv.b < 0) return AHPC_ERR_BAD_SHAPE;
    return AHPC_OK;
}

}  // namespace ahpc

using namespace ahpc;

extern "C" {

// The dense forward.  row_stats given: the 16-bit matrix-core kernels also write every query row's softmax statistic there
// (FlashParams::keep_neg_lse2) and *stats_written becomes 1; launches that take other kernels leave it 0.
static int flash_fwd_dense(const void* q, const void* k, const void* v, void* o, int dtype, int64_t B, int64_t N, int64_t H,
                           int64_t H_kv, int64_t d, int64_t stride_b, int64_t stride_n, int64_t stride_h,
                           int64_t kv_stride_b, int64_t kv_stride_n, int64_t kv_stride_h, float scale, int causal,
                           const float* mask, float* row_stats, int* stats_written, void* stream) {
    const Strides sq{stride_b, stride_n, stride_h}, skv{kv_stride_b, kv_stride_n, kv_stride_h};
    if (stats_written) *stats_written = 0;
    if (int rc = check_dense(q, k, v, o, dtype, B, N, H, H_kv, d, sq, skv)) return rc;
    if (!(scale > 0.0f)) scale = 1.0f / std::sqrt((float)d);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int32_t group = (int32_t)(H / H_kv);
    if (mfma_eligible(dtype, d, q, k, v, o, sq, skv, 256)) {
        FlashParams p{};
        p.q = q; p.k = k; p.v = v; p.o = o;
        p.mask = mask;
        p.stride_b = sq.b; p.stride_n = sq.n; p.stride_h = sq.h;
        p.kv_stride_b = skv.b; p.kv_stride_n = skv.n; p.kv_stride_h = skv.h;
        p.N = (int32_t)N; p.H = (int32_t)H; p.kv_group = group;
        p.scale_log2 = scale * kLog2e;
        p.d_real = (int32_t)d;
        if (row_stats && stats_written) {
            p.keep_neg_lse2 = row_stats;
            p.keep_rows = (N + kFlashRows - 1) / kFlashRows * kFlashRows;
        }
        auto kept = [&](int rc) {  // (every path below runs a kernel that writes the statistics)
            if (rc == AHPC_OK && p.keep_neg_lse2) *stats_written = 1;
            return rc;
        };
        if (!mask)
            return kept(dtype == AHPC_F16 ? dispatch_mfma<f16_t, false>(p, B, kernel_head_dim(d), causal != 0, st)
                                          : dispatch_mfma<bf16_t, false>(p, B, kernel_head_dim(d), causal != 0, st));
        // The mask, by preference, as a packed copy made in front of the launch (every head reads the mask: packed, a
        // sixteenth of the bytes).  Where that is not possible, or switched off, the kernel reads the mask in place,
        // 16 bytes at a time: rows of a multiple of 4 floats and an aligned base; everything else takes the kernel below.
        if (tuning().mask_pack.load() != 0) {
            bool launched = false;
            const int rc = forward_on_packed_mask(p, mask, B, st, &launched, [&](const FlashParams& pb) {
                return dtype == AHPC_F16 ? dispatch_mfma_masked<f16_t, 2>(pb, B, kernel_head_dim(d), causal != 0, st)
                                         : dispatch_mfma_masked<bf16_t, 2>(pb, B, kernel_head_dim(d), causal != 0, st);
            });
            if (launched || rc != AHPC_OK) return launched ? kept(rc) : rc;
        }
        if (d <= 128 && N % 4 == 0 && aligned16(mask))  // (beyond 128 only the packed mask has a kernel)
            return kept(dtype == AHPC_F16 ? dispatch_mfma_masked<f16_t, 1>(p, B, kernel_head_dim(d), causal != 0, st)
                                          : dispatch_mfma_masked<bf16_t, 1>(p, B, kernel_head_dim(d), causal != 0, st));
    }
    if (f32_mfma_eligible(dtype, d, q, k, v, o, sq, skv)) {
        FlashParams p{};
        p.q = q; p.k = k; p.v = v; p.o = o;
        p.stride_b = sq.b; p.stride_n = sq.n; p.stride_h = sq.h;
        p.kv_stride_b = skv.b; p.kv_stride_n = skv.n; p.kv_stride_h = skv.h;
        p.N = (int32_t)N; p.H = (int32_t)H; p.kv_group = group;
        p.scale_log2 = scale * kLog2e;
        p.d_real = (int32_t)d;
        if (!mask) return launch_f32_mfma<false, false>(p, B, kernel_head_dim(d), causal != 0, st);
        // with a mask: on its packed copy, or not on the matrix cores at all
        if (tuning().mask_pack.load() != 0) {
            bool launched = false;
            const int rc = forward_on_packed_mask(p, mask, B, st, &launched, [&](const FlashParams& pb) {
                return launch_f32_mfma<false, true>(pb, B, kernel_head_dim(d), causal != 0, st);
            });
            if (launched || rc != AHPC_OK) return rc;
        }
    }
    SimpleParams p{q, k, v, o, nullptr, mask, sq.b, sq.n, sq.h, skv.b, skv.n, skv.h, (int32_t)N, (int32_t)H, (int32_t)d, group, scale, causal ? 1 : 0};
    return dispatch_simple<false>(dtype, p, B, st);
}

int ahpc_hip_flash_fwd_gqa(const void* q, const void* k, const void* v, void* o, int dtype, int64_t B, int64_t N, int64_t H,
                           int64_t H_kv, int64_t d, int64_t stride_b, int64_t stride_n, int64_t stride_h,
                           int64_t kv_stride_b, int64_t kv_stride_n, int64_t kv_stride_h, float scale, int causal,
                           const float* mask, void* stream) {
    return flash_fwd_dense(q, k, v, o, dtype, B, N, H, H_kv, d, stride_b, stride_n, stride_h, kv_stride_b, kv_stride_n,
                           kv_stride_h, scale, causal, mask, nullptr, nullptr, stream);
}

int ahpc_hip_flash_fwd_keep(const void* q, const void* k, const void* v, void* o, int dtype, int64_t B, int64_t N, int64_t H,
                            int64_t H_kv, int64_t d, int64_t stride_b, int64_t stride_n, int64_t stride_h,
                            int64_t kv_stride_b, int64_t kv_stride_n, int64_t kv_stride_h, float scale, int causal,
                            const float* mask, float* row_stats, int* stats_written, void* stream) {
    if (!row_stats || !stats_written) return AHPC_ERR_NULL_POINTER;
    if ((reinterpret_cast<uintptr_t>(row_stats) & 3u) != 0) return AHPC_ERR_BAD_ALIGNMENT;
    return flash_fwd_dense(q, k, v, o, dtype, B, N, H, H_kv, d, stride_b, stride_n, stride_h, kv_stride_b, kv_stride_n,
                           kv_stride_h, scale, causal, mask, row_stats, stats_written, stream);
}

int ahpc_hip_flash_block_map(int64_t B, int64_t N, int64_t H, int causal, int64_t capacity, int64_t* n_blocks,
                             int32_t* seq_head, int32_t* first_tile, int32_t* second_tile) {
    if (!n_blocks) return AHPC_ERR_NULL_POINTER;
    if (B <= 0 || N <= 0 || H <= 0 || B > 65535 || H > 65535 || N > 0x7FFFFF00ll) return AHPC_ERR_BAD_SHAPE;
    FlashParams p{};
    p.N = (int32_t)N; p.H = (int32_t)H; p.kv_group = 1;
    const int rows = tuning().flash_rows.load() == kFlashWideRows ? kFlashWideRows : kFlashRows;
    if (int rc = flash_plan_launch(p, B, causal != 0, rows, tuning().flash_pair_min_tiles.load())) return rc;
    const int64_t grid = (int64_t)p.blocks_per_xcd * 8;
    *n_blocks = grid;
    if (!seq_head && !first_tile && !second_tile) return AHPC_OK;
    if (!seq_head || !first_tile || !second_tile || capacity < grid) return AHPC_ERR_BAD_SHAPE;
    for (int64_t i = 0; i < grid; ++i) {
        const FlashWork w = flash_work_of_block((unsigned)i, p);
        seq_head[i] = w.valid ? w.bh : -1;
        first_tile[i] = w.valid ? flash_qtile_of_part(p, p.n_qtiles, w.slot, 0) : -1;
        second_tile[i] = w.valid ? flash_qtile_of_part(p, p.n_qtiles, w.slot, 1) : -1;
    }
    return AHPC_OK;
}

int ahpc_hip_flash_fwd_masked(const void* q, const void* k, const void* v, void* o, int dtype, int64_t B, int64_t N,
                              int64_t H, int64_t d, int64_t stride_b, int64_t stride_n, int64_t stride_h, float scale,
                              int causal, const float* mask, void* stream) {
    if (!mask) {
        // no mask: still the fp32-FMA kernel, as documented for this entry point
        const Strides s{stride_b, stride_n, stride_h};
        if (int rc = check_dense(q, k, v, o, dtype, B, N, H, H, d, s, s)) return rc;
        if (!(scale > 0.0f)) scale = 1.0f / std::sqrt((float)d);
        SimpleParams p{q, k, v, o, nullptr, nullptr, s.b, s.n, s.h, s.b, s.n, s.h, (int32_t)N, (int32_t)H, (int32_t)d, 1, scale, causal ? 1 : 0};
        return dispatch_simple<false>(dtype, p, B, static_cast<hipStream_t>(stream));
    }
    return ahpc_hip_flash_fwd_gqa(q, k, v, o, dtype, B, N, H, H, d, stride_b, stride_n, stride_h, stride_b, stride_n,
                                  stride_h, scale, causal, mask, stream);
}

int ahpc_hip_flash_fwd(const void* q, const void* k, const void* v, void* o, int dtype, int64_t B, int64_t N, int64_t H,
                       int64_t d, int64_t stride_b, int64_t stride_n, int64_t stride_h, float scale, int causal,
                       void* stream) {
    return ahpc_hip_flash_fwd_gqa(q, k, v, o, dtype, B, N, H, H, d, stride_b, stride_n, stride_h, stride_b, stride_n,
                                  stride_h, scale, causal, nullptr, stream);
}

int ahpc_hip_flash_fwd_varlen_gqa(const void* q, const void* k, const void* v, void* o, int dtype,
                                  const int32_t* cu_seqlens, int64_t n_seqs, int64_t max_len, int64_t H, int64_t H_kv,
                                  int64_t d, int64_t stride_t, int64_t stride_h, int64_t kv_stride_t, int64_t kv_stride_h,
                                  float scale, int causal, void* stream) {
    if (!cu_seqlens) return AHPC_ERR_NULL_POINTER;
    const Strides sq{0, stride_t, stride_h}, skv{0, kv_stride_t, kv_stride_h};
    if (int rc = check_dense(q, k, v, o, dtype, n_seqs, max_len, H, H_kv, d, sq, skv)) return rc;
    if (!(scale > 0.0f)) scale = 1.0f / std::sqrt((float)d);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int32_t group = (int32_t)(H / H_kv);
    if (mfma_eligible(dtype, d, q, k, v, o, sq, skv, 256)) {
        FlashParams p{};
        p.q = q; p.k = k; p.v = v; p.o = o;
        p.cu_seqlens = cu_seqlens;
        p.stride_b = 0; p.stride_n = sq.n; p.stride_h = sq.h;
        p.kv_stride_b = 0; p.kv_stride_n = skv.n; p.kv_stride_h = skv.h;
        p.N = (int32_t)max_len; p.H = (int32_t)H; p.kv_group = group;
        p.scale_log2 = scale * kLog2e;
        p.d_real = (int32_t)d;
        return dtype == AHPC_F16 ? dispatch_mfma<f16_t, true>(p, n_seqs, kernel_head_dim(d), causal != 0, st)
                                 : dispatch_mfma<bf16_t, true>(p, n_seqs, kernel_head_dim(d), causal != 0, st);
    }
    if (f32_mfma_eligible(dtype, d, q, k, v, o, sq, skv)) {
        FlashParams p{};
        p.q = q; p.k = k; p.v = v; p.o = o;
        p.cu_seqlens = cu_seqlens;
        p.stride_b = 0; p.stride_n = sq.n; p.stride_h = sq.h;
        p.kv_stride_b = 0; p.kv_stride_n = skv.n; p.kv_stride_h = skv.h;
        p.N = (int32_t)max_len; p.H = (int32_t)H; p.kv_group = group;
        p.scale_log2 = scale * kLog2e;
        p.d_real = (int32_t)d;
        return launch_f32_mfma<true, false>(p, n_seqs, kernel_head_dim(d), causal != 0, st);
    }
    SimpleParams p{q, k, v, o, cu_seqlens, nullptr, 0, sq.n, sq.h, 0, skv.n, skv.h, (int32_t)max_len, (int32_t)H, (int32_t)d, group, scale, causal ? 1 : 0};
    return dispatch_simple<true>(dtype, p, n_seqs, st);
}

int ahpc_hip_flash_fwd_varlen(const void* q, const void* k, const void* v, void* o, int dtype, const int32_t* cu_seqlens,
                              int64_t n_seqs, int64_t max_len, int64_t H, int64_t d, int64_t stride_t, int64_t stride_h,
                              float scale, int causal, void* stream) {
    return ahpc_hip_flash_fwd_varlen_gqa(q, k, v, o, dtype, cu_seqlens, n_seqs, max_len, H, H, d, stride_t, stride_h,
                                         stride_t, stride_h, scale, causal, stream);
}

}  // extern "C"
