// Calibration launch for the matrix-bound roofline figures: what the matrix cores of this GPU deliver when every
// SIMD does nothing but v_mfma_f32_32x32x16 on operands that sit in registers, and what they deliver with the VALU
// work of a softmax between the matrix instructions.  No memory traffic inside the loop; nothing here is part of
// the attention path.
#include <hip/hip_runtime.h>

#include "ahpc_device.hpp"
#include "ahpc_hip.h"

namespace ahpc {

constexpr int kProbeThreads = 256;  // 4 wavefronts: one per SIMD and workgroup
constexpr int kProbeChains = 4;     // independent accumulators per wavefront

// Operand words with varied bit patterns (how many bits toggle matters for the clock the chip sustains): small
// normal numbers of either sign in both 16-bit formats.
__device__ inline uint32_t probe_word(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return (x & 0x83ff83ffu) | 0x38003800u;
}

template <typename T, int MIX>
__global__ __launch_bounds__(kProbeThreads) void probe_matrix_rate_kernel(int iterations, float* sink) {
    const uint32_t id = blockIdx.x * kProbeThreads + threadIdx.x;
    u32x4 a[kProbeChains], b;
#pragma unroll
    for (int c = 0; c < kProbeChains; ++c)
#pragma unroll
        for (int w = 0; w < 4; ++w) a[c][w] = probe_word(id * 16u + c * 4u + w);
#pragma unroll
    for (int w = 0; w < 4; ++w) b[w] = probe_word(~id * 4u + w);
    f32x16 acc[kProbeChains];
#pragma unroll
    for (int c = 0; c < kProbeChains; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[c][r] = 0.0f;
    // the VALU part works on its own registers (as a softmax does on the previous tile's scores)
    float x[kProbeChains];
#pragma unroll
    for (int i = 0; i < kProbeChains; ++i) x[i] = -1.0f - 0.125f * (float)((id + i) & 7);
    float sum = 0.0f;

    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int c = 0; c < kProbeChains; ++c) {
            acc[c] = mfma_32x32x16<T>(a[c], b, acc[c]);
            if (MIX) {
                // The flash forward at d = 128 spends, per matrix instruction, one exponential, one row-sum addition,
                // half a maximum and half a packing conversion (32 scores per lane and 32 matrix instructions per
                // 64-key tile).  Here: one exponential, two additions, one maximum, one conversion, one bit
                // operation - somewhat more, so that the figure is a lower bracket for the kernel's ceiling.
                const float p0 = fast_exp2(x[c]);
                sum += p0;
                b[c] ^= pack2<T>(p0, p0) & 0x00010001u;                  // keeps the conversion alive, flips one bit
                x[c] = fmaxf(x[c] - 0.0625f, -6.0f);
            }
        }
    }
    float out = sum;
#pragma unroll
    for (int c = 0; c < kProbeChains; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) out += acc[c][r];
    sink[id] = out;
}

}  // namespace ahpc

extern "C" int ahpc_hip_probe_matrix_rate(int dtype, int mix, int64_t workgroups, int64_t iterations, float* sink,
                                          size_t sink_bytes, double* flop, void* stream) {
    using namespace ahpc;
    if (!sink) return AHPC_ERR_NULL_POINTER;
    if (dtype != AHPC_F16 && dtype != AHPC_BF16) return AHPC_ERR_BAD_DTYPE;
    if (workgroups <= 0 || workgroups > (1 << 20) || iterations <= 0 || iterations > (1 << 24) || (mix != 0 && mix != 1))
        return AHPC_ERR_BAD_SHAPE;
    if (sink_bytes < (size_t)workgroups * kProbeThreads * sizeof(float)) return AHPC_ERR_WORKSPACE_TOO_SMALL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)workgroups), block(kProbeThreads);
    const int it = (int)iterations;
    if (dtype == AHPC_F16) {
        if (mix) hipLaunchKernelGGL((probe_matrix_rate_kernel<f16_t, 1>), grid, block, 0, st, it, sink);
        else hipLaunchKernelGGL((probe_matrix_rate_kernel<f16_t, 0>), grid, block, 0, st, it, sink);
    } else {
        if (mix) hipLaunchKernelGGL((probe_matrix_rate_kernel<bf16_t, 1>), grid, block, 0, st, it, sink);
        else hipLaunchKernelGGL((probe_matrix_rate_kernel<bf16_t, 0>), grid, block, 0, st, it, sink);
    }
    // 32 x 32 x 16 multiply-adds per matrix instruction and wavefront
    if (flop) *flop = 2.0 * 32 * 32 * 16 * kProbeChains * (double)iterations * (kProbeThreads / 64) * (double)workgroups;
    return static_cast<int>(hipGetLastError());
}
