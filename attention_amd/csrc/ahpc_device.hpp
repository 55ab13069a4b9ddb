// Device-side helpers shared by the gfx950 kernels: storage types, conversions, wave intrinsics.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ahpc_hip.h"

namespace ahpc {

typedef _Float16 f16_t;
typedef __bf16 bf16_t;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;

// ---- storage <-> fp32 -----------------------------------------------------------------------
// Conversions to 16 bits are round-to-nearest-even with NaN kept (the compiler lowers them to
// v_cvt_f16_f32 / v_cvt_pk_bf16_f32, both RNE).
template <typename T> struct Storage;
template <> struct Storage<float> {
    static constexpr int code = AHPC_F32;
    __device__ static float load(const float* p) { return *p; }
    __device__ static void store(float* p, float x) { *p = x; }
};
template <> struct Storage<f16_t> {
    static constexpr int code = AHPC_F16;
    typedef f16x8 vec8;
    typedef f16x2 vec2;
    __device__ static float load(const f16_t* p) { return (float)*p; }
    __device__ static void store(f16_t* p, float x) { *p = (f16_t)x; }
};
template <> struct Storage<bf16_t> {
    static constexpr int code = AHPC_BF16;
    typedef bf16x8 vec8;
    typedef bf16x2 vec2;
    __device__ static float load(const bf16_t* p) { return (float)*p; }
    __device__ static void store(bf16_t* p, float x) { *p = (bf16_t)x; }
};

// Bit pattern -> fp32.  Takes the dword BY VALUE on purpose: __builtin_bit_cast applied directly to
// an element of an ext-vector (v[i]) reads element 0 whatever i is with this compiler.
__device__ inline float as_f32(uint32_t w) { return __builtin_bit_cast(float, w); }
__device__ inline uint32_t as_u32(float x) { return __builtin_bit_cast(uint32_t, x); }

// Packs two fp32 into one dword of two 16-bit values (low half = a).
template <typename T> __device__ inline uint32_t pack2(float a, float b);
template <> __device__ inline uint32_t pack2<f16_t>(float a, float b) {
    f16x2 v;
    v[0] = (f16_t)a;
    v[1] = (f16_t)b;
    return __builtin_bit_cast(uint32_t, v);
}
template <> __device__ inline uint32_t pack2<bf16_t>(float a, float b) {
    bf16x2 v;
    v[0] = (bf16_t)a;
    v[1] = (bf16_t)b;
    return __builtin_bit_cast(uint32_t, v);
}

// Unpacks the low / high 16-bit half of a dword to fp32.
template <typename T> __device__ inline float lo_f32(uint32_t w);
template <typename T> __device__ inline float hi_f32(uint32_t w);
template <> __device__ inline float lo_f32<bf16_t>(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
template <> __device__ inline float hi_f32<bf16_t>(uint32_t w) { return __builtin_bit_cast(float, w & 0xFFFF0000u); }
template <> __device__ inline float lo_f32<f16_t>(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[0]; }
template <> __device__ inline float hi_f32<f16_t>(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[1]; }

// acc += dot(two 16-bit pairs), fp32 accumulate (v_dot2_f32_f16 / v_dot2_f32_bf16).
template <typename T> __device__ inline float dot2(uint32_t a, uint32_t b, float acc);
template <> __device__ inline float dot2<f16_t>(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), acc, false);
}
template <> __device__ inline float dot2<bf16_t>(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), acc, false);
}

// ---- LDS ----------------------------------------------------------------------------------------
// 16-byte LDS read (ds_read_b128).  The CPU executor the tests use defines AHPC_TRACED_LDS_READ_B128 to
// a read that also records the lanes' addresses, so that bank conflicts can be counted there.
__device__ inline u32x4 lds_read_b128(const unsigned char* p) {
#if defined(AHPC_TRACED_LDS_READ_B128)
    return AHPC_TRACED_LDS_READ_B128(p);
#else
    return *reinterpret_cast<const u32x4*>(p);
#endif
}

// ---- MFMA ----------------------------------------------------------------------------------
// D(32x32) += A(32x16) * B(16x32).  Lane l supplies A[row l%32][k 8*(l/32)..+7] and
// B[k 8*(l/32)..+7][col l%32]; it receives D[row 8*(r/4) + 4*(l/32) + r%4][col l%32] in acc[r].
template <typename T> __device__ inline f32x16 mfma_32x32x16(u32x4 a, u32x4 b, f32x16 acc);
template <> __device__ inline f32x16 mfma_32x32x16<f16_t>(u32x4 a, u32x4 b, f32x16 acc) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
}
template <> __device__ inline f32x16 mfma_32x32x16<bf16_t>(u32x4 a, u32x4 b, f32x16 acc) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
}

// D(16x16) += A(16xK) * B(Kx16), K = 32 or 16.  Lane l supplies A[row l%16][k KPL*(l/16)..] and
// B[k KPL*(l/16)..][col l%16] (KPL = 8 or 4 values per lane); it receives D[row 4*(l/16) + r][col l%16] in acc[r].
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
template <typename T> __device__ inline f32x4 mfma_16x16x32(u32x4 a, u32x4 b, f32x4 acc);
template <> __device__ inline f32x4 mfma_16x16x32<f16_t>(u32x4 a, u32x4 b, f32x4 acc) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
}
template <> __device__ inline f32x4 mfma_16x16x32<bf16_t>(u32x4 a, u32x4 b, f32x4 acc) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
}
template <typename T> __device__ inline f32x4 mfma_16x16x16(u32x2 a, u32x2 b, f32x4 acc);
template <> __device__ inline f32x4 mfma_16x16x16<f16_t>(u32x2 a, u32x2 b, f32x4 acc) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), acc, 0, 0, 0);
}
template <> __device__ inline f32x4 mfma_16x16x16<bf16_t>(u32x2 a, u32x2 b, f32x4 acc) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), acc, 0, 0, 0);
}

// ---- wave helpers ----------------------------------------------------------------------------
// Value held by lane (l ^ 32).
__device__ inline float swap_halves(float x) {
    return __shfl_xor(x, 32, kWave);
}

__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Largest of three as ONE instruction (v_maximum3_f32).  fmaxf(a, fmaxf(b, c)) on values the compiler cannot
// prove canonical (matrix-instruction results) puts a `v_max_f32 x, x, x` per input in front of the maximum
// itself, three times the instructions in a chain over a tile's scores; the IEEE-754-2019 maximum needs none.
// It propagates NaN where fmaxf drops it: the scores here are finite or -inf.
__device__ inline float max3(float a, float b, float c) {
    return __builtin_elementwise_maximum(__builtin_elementwise_maximum(a, b), c);
}

}  // namespace ahpc
