// Test infrastructure: a stand-in for <hip/hip_runtime.h> that lets the library's kernel sources be
// compiled as ordinary host C++ and executed lane by lane on the CPU (see simt_runtime.cpp).  It is put
// in front of the real header on the include path of the CPU build only; nothing that ships uses it.
//
// What is modelled:
//   * a launch runs its workgroups one after the other; every work-item is a cooperative fiber, a
//     wavefront is 64 consecutive work-items;
//   * __syncthreads and every cross-lane operation the kernels use (matrix instructions, transposing
//     LDS reads, lane swaps, DPP, shuffles, ballot, readlane) exchange operands between the fibers of
//     a wavefront exactly as the instruction set documents; a wavefront whose lanes reach different
//     cross-lane operations, or a workgroup that can make no progress, is reported as an error;
//   * global -> LDS direct loads are asynchronous: their data lands either at issue or only at the next
//     s_waitcnt of the issuing lane (chosen per run), which exposes a missing wait or a buffer reused
//     too early; buffer descriptors clamp out-of-range reads to zero like the hardware;
//   * 16-byte LDS reads made through lds_read_b128 and transposing reads are checked for bank conflicts under
//     a model of 64 banks of 4 bytes (16 lanes per pass for 16-byte reads, 32 for 8-byte reads);
//   * the same reads and the direct loads are checked for ordering between wavefronts: a direct load's write and
//     another wavefront's read (or direct load) of the same LDS word need a workgroup barrier between them,
//     where a load occupies the span from its issue to its lane's wait; violations are reported as errors
//     whatever order the run happened to execute the wavefronts in (plain C++ accesses to LDS are not seen);
//   * __shared__ arrays live in one linker section, filled with a NaN pattern before every workgroup,
//     and LDS accesses made through intrinsics are range-checked against it.
// Plain loads and stores through pointers are ordinary host accesses; run the build under
// AddressSanitizer to bound-check them.
#pragma once

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>

#define __HIP_DEVICE_COMPILE__ 1
#define AHPC_LDS  // LDS pointers are ordinary pointers here

#define __global__
#define __device__
#define __host__
#define __align__(n) __attribute__((aligned(n)))
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __shared__ static __attribute__((section("simt_lds"), used))

struct dim3 {
    unsigned x, y, z;
    constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
extern dim3 threadIdx, blockIdx, blockDim, gridDim;

typedef void* hipStream_t;
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
constexpr hipError_t hipErrorLaunchFailure = 719;

namespace simt {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

void launch(dim3 grid, dim3 block, const std::function<void()>& body);
hipError_t last_error();

void syncthreads();
int lane_id();

f32x16 mfma_32x32x16_f16(f16x8 a, f16x8 b, f32x16 c);
f32x16 mfma_32x32x16_bf16(bf16x8 a, bf16x8 b, f32x16 c);
f32x16 mfma_32x32x2_f32(float a, float b, f32x16 c);
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
f32x4 mfma_16x16x32_f16(f16x8 a, f16x8 b, f32x4 c);
f32x4 mfma_16x16x32_bf16(bf16x8 a, bf16x8 b, f32x4 c);
f32x4 mfma_16x16x16_f16(f16x4 a, f16x4 b, f32x4 c);
f32x4 mfma_16x16x16_bf16(s16x4 a, s16x4 b, f32x4 c);  // operands hold bf16 bit patterns
uint64_t ds_read_tr16_b64(const void* lds_ptr);
u32x4 lds_read_b128(const void* lds_ptr);  // a plain 16-byte LDS read whose addresses are recorded
u32x2 permlane32_swap(unsigned a, unsigned b);
uint64_t ballot(bool pred);
int readfirstlane(int x);
int readlane(int x, int lane);
int update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl);
int shfl_xor_bits(int x, int mask, int width);

struct BufferRsrc {
    const unsigned char* base;
    unsigned num_records;
};
void buffer_load_lds(BufferRsrc r, void* lds_base, int size, int voffset, int soffset, int imm, int aux);
void waitcnt(int imm);

inline float fdot2_f16(f16x2 a, f16x2 b, float c) { return (float)a[0] * (float)b[0] + (float)a[1] * (float)b[1] + c; }
inline float fdot2_bf16(bf16x2 a, bf16x2 b, float c) { return (float)a[0] * (float)b[0] + (float)a[1] * (float)b[1] + c; }

template <typename V> inline V bits_to(uint64_t w) {
    static_assert(sizeof(V) == 8, "64-bit result expected");
    V v;
    std::memcpy(&v, &w, 8);
    return v;
}

template <typename T> inline T shfl_xor(T x, int mask, int width) {
    static_assert(sizeof(T) == 4, "32-bit shuffles only");
    int b;
    std::memcpy(&b, &x, 4);
    b = shfl_xor_bits(b, mask, width);
    std::memcpy(&x, &b, 4);
    return x;
}

}  // namespace simt

typedef simt::BufferRsrc __amdgpu_buffer_rsrc_t;

// ---- runtime services: "device" memory is host memory, streams and events do nothing ------------
typedef void* hipEvent_t;
enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
enum hipMemoryType { hipMemoryTypeHost = 1, hipMemoryTypeDevice = 2, hipMemoryTypeManaged = 3 };
constexpr unsigned hipStreamNonBlocking = 1;
constexpr unsigned hipHostMallocDefault = 0;
struct hipPointerAttribute_t {
    hipMemoryType type;
};
struct hipDeviceProp_t {
    char name[256];
    char gcnArchName[256];
    size_t totalGlobalMem;
    size_t sharedMemPerBlock;
    int multiProcessorCount, warpSize, maxThreadsPerBlock, clockRate;
};
inline const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "success" : "emulated kernel launch failed"; }
inline hipError_t hipGetDeviceCount(int* n) { *n = 1; return hipSuccess; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
#define HIP_SYMBOL(x) (&(x))
template <typename S> inline hipError_t hipGetSymbolAddress(void** p, S* symbol) { *p = (void*)symbol; return hipSuccess; }
inline hipError_t hipRuntimeGetVersion(int* v) { *v = 0; return hipSuccess; }
inline hipError_t hipMemGetInfo(size_t* free_b, size_t* total_b) {
    *free_b = (size_t)4 << 30;  // what callers may really take from the host
    *total_b = (size_t)288 << 30;
    return hipSuccess;
}
inline hipError_t hipGetDeviceProperties(hipDeviceProp_t* p, int) {
    std::memset(p, 0, sizeof *p);
    std::strcpy(p->name, "lane-by-lane CPU executor");
    std::strcpy(p->gcnArchName, "gfx950:emulated");
    p->totalGlobalMem = (size_t)288 << 30;  // the part this stands in for
    p->sharedMemPerBlock = 160 * 1024;
    p->multiProcessorCount = 256;
    p->warpSize = 64;
    p->maxThreadsPerBlock = 1024;
    p->clockRate = 1;
    return hipSuccess;
}
// One allocation can be made to fail (tests of the callers' out-of-memory paths): the countdown is decremented by every
// device allocation, the one that takes it to zero fails.
extern int simt_fail_device_alloc_in;
inline bool simt_alloc_fails() { return simt_fail_device_alloc_in > 0 && --simt_fail_device_alloc_in == 0; }
inline hipError_t hipMalloc(void** p, size_t n) {
    if (simt_alloc_fails()) { *p = nullptr; return 2; }
    *p = std::malloc(n);
    return *p ? hipSuccess : 2;
}
// virtual memory management, emulated with an inaccessible mapping whose front part is made accessible piece by piece
enum hipDeviceAttribute_t { hipDeviceAttributeVirtualMemoryManagementSupported = 1, hipDeviceAttributeMultiprocessorCount = 2 };
inline hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int) { *v = 1; return hipSuccess; }
enum { hipMemAllocationTypePinned = 1, hipMemLocationTypeDevice = 1, hipMemAccessFlagsProtReadWrite = 3 };
struct hipMemLocation { int type; int id; };
struct hipMemAllocationProp { int type; hipMemLocation location; };
struct hipMemAccessDesc { hipMemLocation location; int flags; };
typedef size_t hipMemGenericAllocationHandle_t;
hipError_t hipMemAddressReserve(void** p, size_t n, size_t align, void*, unsigned long long);
hipError_t hipMemAddressFree(void* p, size_t n);
inline hipError_t hipMemCreate(hipMemGenericAllocationHandle_t* h, size_t n, const hipMemAllocationProp*, unsigned long long) {
    if (simt_alloc_fails()) return 2;
    *h = n;
    return hipSuccess;
}
inline hipError_t hipMemRelease(hipMemGenericAllocationHandle_t) { return hipSuccess; }
hipError_t hipMemMap(void* p, size_t n, size_t, hipMemGenericAllocationHandle_t, unsigned long long);
hipError_t hipMemUnmap(void* p, size_t n);
inline hipError_t hipMemSetAccess(void*, size_t, const hipMemAccessDesc*, size_t) { return hipSuccess; }
inline hipError_t hipFree(void* p) { std::free(p); return hipSuccess; }
inline hipError_t hipHostMalloc(void** p, size_t n, unsigned) { *p = std::malloc(n); return *p ? hipSuccess : 2; }
inline hipError_t hipHostFree(void* p) { std::free(p); return hipSuccess; }
inline hipError_t hipMemcpyAsync(void* d, const void* s, size_t n, hipMemcpyKind, hipStream_t) { std::memmove(d, s, n); return hipSuccess; }
inline hipError_t hipMemsetAsync(void* d, int v, size_t n, hipStream_t) { std::memset(d, v, n); return hipSuccess; }
// every pointer counts as device memory: callers then hand their buffers to the kernels as they are
inline hipError_t hipPointerGetAttributes(hipPointerAttribute_t* a, const void*) { a->type = hipMemoryTypeDevice; return hipSuccess; }
inline hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned) { *s = nullptr; return hipSuccess; }
inline hipError_t hipStreamDestroy(hipStream_t) { return hipSuccess; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
inline hipError_t hipDeviceSynchronize() { return hipSuccess; }
inline hipError_t hipEventCreate(hipEvent_t* e) { *e = std::malloc(1); return hipSuccess; }
enum { hipEventDisableTiming = 2 };
inline hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) { *e = std::malloc(1); return hipSuccess; }
inline hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) { return hipSuccess; }
enum hipStreamCaptureStatus { hipStreamCaptureStatusNone = 0, hipStreamCaptureStatusActive = 1 };
inline hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus* s) { *s = hipStreamCaptureStatusNone; return hipSuccess; }
inline hipError_t hipEventDestroy(hipEvent_t e) { std::free(e); return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t, hipEvent_t) { *ms = 0.0f; return hipSuccess; }

#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
    ::simt::launch((grid), (block), [&]() { kernel(__VA_ARGS__); })
inline hipError_t hipGetLastError() { return ::simt::last_error(); }

#define __syncthreads() ::simt::syncthreads()
#define __builtin_amdgcn_s_barrier() ::simt::syncthreads()
#define __shfl_xor(x, mask, width) ::simt::shfl_xor((x), (mask), (width))
#define __expf(x) expf(x)

#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) ::simt::mfma_32x32x16_f16((a), (b), (c))
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) ::simt::mfma_32x32x16_bf16((a), (b), (c))
#define __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, x, y, z) ::simt::mfma_32x32x2_f32((a), (b), (c))
#define __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, x, y, z) ::simt::mfma_16x16x32_f16((a), (b), (c))
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) ::simt::mfma_16x16x32_bf16((a), (b), (c))
#define __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, x, y, z) ::simt::mfma_16x16x16_f16((a), (b), (c))
#define __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, x, y, z) ::simt::mfma_16x16x16_bf16((a), (b), (c))
#define __builtin_amdgcn_ds_read_tr16_b64_v4bf16(p) \
    ::simt::bits_to<__attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16>(::simt::ds_read_tr16_b64((const void*)(p)))
#define __builtin_amdgcn_ds_read_tr16_b64_v4f16(p) \
    ::simt::bits_to<__attribute__((__vector_size__(4 * sizeof(__fp16)))) __fp16>(::simt::ds_read_tr16_b64((const void*)(p)))
#define AHPC_TRACED_LDS_READ_B128(p) ::simt::lds_read_b128((p))
#define __builtin_amdgcn_permlane32_swap(a, b, fi, bc) ::simt::permlane32_swap((a), (b))
#define __builtin_amdgcn_ballot_w64(p) ::simt::ballot((p))
// the lanes of a wavefront meet here (on the GPU they are in step anyway): every lane's LDS writes in front of it are
// visible to the reads behind it
#define __builtin_amdgcn_wave_barrier() ((void)::simt::ballot(true))
#define __builtin_amdgcn_readfirstlane(x) ::simt::readfirstlane((x))
#define __builtin_amdgcn_readlane(x, l) ::simt::readlane((x), (l))
#define __builtin_amdgcn_update_dpp(old, src, ctrl, rm, bm, bc) ::simt::update_dpp((old), (src), (ctrl), (rm), (bm), (bc))
#define __builtin_amdgcn_make_buffer_rsrc(base, stride, num, flags) \
    (::simt::BufferRsrc{static_cast<const unsigned char*>(static_cast<const void*>(base)), (unsigned)(num)})
#define __builtin_amdgcn_raw_ptr_buffer_load_lds(r, lds, size, voff, soff, imm, aux) \
    ::simt::buffer_load_lds((r), (void*)(lds), (size), (voff), (soff), (imm), (aux))
#define __builtin_amdgcn_s_waitcnt(x) ::simt::waitcnt((x))
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)
#define __builtin_amdgcn_sched_barrier(a) ((void)0)
#define __builtin_amdgcn_s_setprio(a) ((void)0)
// hardware register reads: the only one the kernels use is the LDS allocation base, which the executor answers with
// 0 for even workgroups and a non-zero offset for odd ones (both roles of a pair of workgroups get exercised)
#define __builtin_amdgcn_s_getreg(which) ((unsigned)((blockIdx.x & 1u) * 64u))
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_fdot2(a, b, c, clamp) ::simt::fdot2_f16((a), (b), (c))
#define __builtin_amdgcn_fdot2_f32_bf16(a, b, c, clamp) ::simt::fdot2_bf16((a), (b), (c))
