// Test infrastructure: small kernels that exist only to check the lane-by-lane executor itself.  Most of
// them are wrong on purpose (a barrier only part of a wavefront reaches, lanes at different cross-lane
// operations, a direct-to-LDS load consumed before its wait); they are compiled for the CPU executor
// only, never for a GPU.  The others are known-answer checks of the cross-lane operations.
#include <hip/hip_runtime.h>

#include "ahpc_hip.h"
#include "flash_fwd_mfma.hpp"

namespace {

// The forward kernel launched with a workgroup map that names more (sequence, head) pairs than the tensors
// hold: the plan is made for `B + extra` batch entries, the tensors and FlashParams::n_bh are those of B.
__global__ __launch_bounds__(ahpc::kFlashThreads) void flash_with_oversized_map(const ahpc::FlashParams p) {
    ahpc::flash_fwd_mfma_body<ahpc::bf16_t, 128, true, false, false>(p, ahpc::FlashStatsOut{});
}

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__global__ void half_wave_at_barrier(float* out) {
    float x = (float)threadIdx.x;
    if (threadIdx.x & 1) __syncthreads();
    else x = __shfl_xor(x, 1, 64);
    out[threadIdx.x] = x;
}

__global__ void lanes_at_different_operations(float* out) {
    float x = (float)threadIdx.x;
    if (threadIdx.x & 1) x = __shfl_xor(x, 2, 64);
    else x = (float)__builtin_amdgcn_ballot_w64(x > 3.0f);
    out[threadIdx.x] = x;
}

__global__ void reads_a_finished_lane(int* out) {
    if (threadIdx.x >= 32) return;
    out[threadIdx.x] = __builtin_amdgcn_readlane((int)threadIdx.x, 40);
}

// every lane copies 16 bytes global -> LDS with the direct load and reads them back; `wait` says whether
// the wait that makes the data visible is executed
__global__ void dma_round_trip(const unsigned char* src, unsigned char* dst, int wait) {
    __shared__ __attribute__((aligned(1024))) unsigned char tile[1024];
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(src), 0, 1000, 0x00020000);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, tile, 16, (int)threadIdx.x * 16, 0, 0, 0);
    if (wait) __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    for (int i = 0; i < 16; ++i) dst[threadIdx.x * 16 + i] = tile[threadIdx.x * 16 + i];
}

// Two wavefronts and one 1 KiB tile.  mode 0 (correct): wavefront 0 loads the tile, waits, barrier, wavefront 1
// reads it.  mode 1: the barrier is missing.  mode 2: after a correct round both wavefronts read the tile and
// wavefront 0 loads into it again without a barrier in between.
__global__ void lds_ordering(const unsigned char* src, unsigned char* dst, int mode) {
    __shared__ __attribute__((aligned(1024))) unsigned char tile[1024];
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(src), 0, 2048, 0x00020000);
    if (wave == 0) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, tile, 16, lane * 16, 0, 0, 0);
        __builtin_amdgcn_s_waitcnt(0);
    }
    if (mode != 1) __syncthreads();
    simt::u32x4 x = simt::lds_read_b128(tile + lane * 16);
    if (mode == 2 && wave == 0) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, tile, 16, 1024 + lane * 16, 0, 0, 0);
        __builtin_amdgcn_s_waitcnt(0);
    }
    if (wave == 1)
        for (int i = 0; i < 4; ++i) reinterpret_cast<unsigned*>(dst)[lane * 4 + i] = x[i];
}

// D = A * B + C with A[i][k] = a[i*16+k], B[k][j] = b[k*32+j], operands and result laid out as documented
// for v_mfma_f32_32x32x16_bf16
__global__ void matrix_instruction(const float* a, const float* b, const float* c, float* d) {
    const int lane = threadIdx.x, col = lane & 31, half = lane >> 5;
    bf16x8 av, bv;
    for (int e = 0; e < 8; ++e) {
        av[e] = (__bf16)a[col * 16 + 8 * half + e];
        bv[e] = (__bf16)b[(8 * half + e) * 32 + col];
    }
    f32x16 acc;
    for (int r = 0; r < 16; ++r) acc[r] = c[(8 * (r / 4) + 4 * half + r % 4) * 32 + col];
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
    for (int r = 0; r < 16; ++r) d[(8 * (r / 4) + 4 * half + r % 4) * 32 + col] = acc[r];
}

// butterfly sums over 2, 4, 8 and 16 neighbouring lanes with the DPP controls the decode kernel uses
__global__ void dpp_sums(const float* in, float* out) {
    float x = in[threadIdx.x];
    auto dpp = [](float v, int ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, true));
    };
    x += dpp(x, 0xB1);
    out[threadIdx.x] = x;
    x += dpp(x, 0x4E);
    out[64 + threadIdx.x] = x;
    x += dpp(x, 0x141);
    out[128 + threadIdx.x] = x;
    x += dpp(x, 0x140);
    out[192 + threadIdx.x] = x;
}

}  // namespace

extern "C" {
int simt_selftest_flash_oversized_map(const void* q, const void* k, const void* v, void* o, int B, int extra, int N, int H,
                                      int kind) {
    ahpc::FlashParams p{};
    p.q = q; p.k = k; p.v = v; p.o = o;
    p.stride_b = p.kv_stride_b = (int64_t)N * H * 128;
    p.stride_n = p.kv_stride_n = (int64_t)H * 128;
    p.stride_h = p.kv_stride_h = 128;
    p.N = N; p.H = H; p.kv_group = 1;
    p.scale_log2 = 0.1275f;
    (void)kind;
    if (int rc = ahpc::flash_plan_launch(p, B + extra, true)) return rc;
    p.n_bh = B * H;  // what the tensors really hold
    hipLaunchKernelGGL(flash_with_oversized_map, dim3(p.blocks_per_xcd * 8), dim3(ahpc::kFlashThreads), 0, nullptr, p);
    return hipGetLastError();
}
int simt_selftest_half_wave_at_barrier(float* out) {
    hipLaunchKernelGGL(half_wave_at_barrier, dim3(1), dim3(64), 0, nullptr, out);
    return hipGetLastError();
}
int simt_selftest_lanes_at_different_operations(float* out) {
    hipLaunchKernelGGL(lanes_at_different_operations, dim3(1), dim3(64), 0, nullptr, out);
    return hipGetLastError();
}
int simt_selftest_reads_a_finished_lane(int* out) {
    hipLaunchKernelGGL(reads_a_finished_lane, dim3(1), dim3(64), 0, nullptr, out);
    return hipGetLastError();
}
int simt_selftest_dma_round_trip(const unsigned char* src, unsigned char* dst, int wait) {
    hipLaunchKernelGGL(dma_round_trip, dim3(1), dim3(64), 0, nullptr, src, dst, wait);
    return hipGetLastError();
}
int simt_selftest_lds_ordering(const unsigned char* src, unsigned char* dst, int mode) {
    hipLaunchKernelGGL(lds_ordering, dim3(1), dim3(128), 0, nullptr, src, dst, mode);
    return hipGetLastError();
}
int simt_selftest_matrix_instruction(const float* a, const float* b, const float* c, float* d) {
    hipLaunchKernelGGL(matrix_instruction, dim3(1), dim3(64), 0, nullptr, a, b, c, d);
    return hipGetLastError();
}
int simt_selftest_dpp_sums(const float* in, float* out) {
    hipLaunchKernelGGL(dpp_sums, dim3(1), dim3(64), 0, nullptr, in, out);
    return hipGetLastError();
}
}
