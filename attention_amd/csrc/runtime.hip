// Device, memory, stream and event entry points of the C ABI, and the error strings.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "ahpc_hip.h"
#include "tuning.hpp"

namespace ahpc {

static int64_t env_value(const char* name, int64_t dflt) {
    const char* e = std::getenv(name);
    return e ? std::atoll(e) : dflt;
}

Tuning::Tuning()
    : flash_pair_min_tiles(env_value("AHPC_FLASH_PAIR_MIN", 1024)),
      decode_waves(env_value("AHPC_DECODE_WAVES", 0)),
      decode_chunk(env_value("AHPC_DECODE_CHUNK", 0)),
      decode_matrix_min_group(env_value("AHPC_DECODE_MFMA_MIN_GROUP", 2)),
      bwd_split(env_value("AHPC_BWD_SPLIT", 0)),
      mask_pack(env_value("AHPC_MASK_PACK", 1)),
      bwd_pair(env_value("AHPC_BWD_PAIR", 1)),
      flash_rows(env_value("AHPC_FLASH_ROWS", 0)),
      pool_in_place(env_value("AHPC_POOL_IN_PLACE", 1)) {
    if (flash_pair_min_tiles.load() < 1) flash_pair_min_tiles = 1024;
}

Tuning& tuning() {
    static Tuning t;  // the environment is read here, once
    return t;
}

static std::atomic<int64_t>* tuning_slot(const char* name) {
    if (!name) return nullptr;
    Tuning& t = tuning();
    if (!std::strcmp(name, "flash_pair_min_tiles")) return &t.flash_pair_min_tiles;
    if (!std::strcmp(name, "decode_waves")) return &t.decode_waves;
    if (!std::strcmp(name, "decode_chunk")) return &t.decode_chunk;
    if (!std::strcmp(name, "decode_matrix_min_group")) return &t.decode_matrix_min_group;
    if (!std::strcmp(name, "bwd_split")) return &t.bwd_split;
    if (!std::strcmp(name, "mask_pack")) return &t.mask_pack;
    if (!std::strcmp(name, "bwd_pair")) return &t.bwd_pair;
    if (!std::strcmp(name, "flash_rows")) return &t.flash_rows;
    if (!std::strcmp(name, "pool_in_place")) return &t.pool_in_place;
    return nullptr;
}

}  // namespace ahpc

extern "C" {

int ahpc_hip_set_tuning(const char* name, int64_t value) {
    std::atomic<int64_t>* slot = ahpc::tuning_slot(name);
    if (!slot) return AHPC_ERR_BAD_SHAPE;
    if (value < 0) return AHPC_ERR_BAD_SHAPE;
    slot->store(value);
    return AHPC_OK;
}

int ahpc_hip_get_tuning(const char* name, int64_t* value) {
    if (!value) return AHPC_ERR_NULL_POINTER;
    std::atomic<int64_t>* slot = ahpc::tuning_slot(name);
    if (!slot) return AHPC_ERR_BAD_SHAPE;
    *value = slot->load();
    return AHPC_OK;
}

const char* ahpc_hip_error_string(int code) {
    switch (code) {
        case AHPC_OK: return "success";
        case AHPC_ERR_NULL_POINTER: return "null pointer argument";
        case AHPC_ERR_BAD_SHAPE: return "invalid shape, stride or size argument";
        case AHPC_ERR_BAD_DTYPE: return "unknown data type code";
        case AHPC_ERR_UNSUPPORTED_HEAD_DIM: return "head dimension not supported by this kernel";
        case AHPC_ERR_WORKSPACE_TOO_SMALL: return "workspace too small";
        case AHPC_ERR_NO_DEVICE: return "no HIP device available";
        case AHPC_ERR_BAD_ALIGNMENT: return "pointer or stride not aligned for 16-byte access";
        case AHPC_ERR_UNSUPPORTED_GROUP: return "query heads per key/value head not supported";
        case AHPC_ERR_SCRATCH_LIMIT: return "the call needs more scratch than ahpc_hip_paged_decode_noalloc has built in (16 MiB): use ahpc_hip_paged_decode_gqa with a workspace";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown error code";
}

int ahpc_hip_device_count(int* count) {
    if (!count) return AHPC_ERR_NULL_POINTER;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return AHPC_OK;
}

int ahpc_hip_device_info(int device, ahpc_device_info* out) {
    if (!out) return AHPC_ERR_NULL_POINTER;
    int n = 0;
    ahpc_hip_device_count(&n);
    if (device < 0 || device >= n) return AHPC_ERR_NO_DEVICE;
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return static_cast<int>(e);
    std::memset(out, 0, sizeof(*out));
    std::strncpy(out->name, prop.name, sizeof(out->name) - 1);
    std::strncpy(out->arch, prop.gcnArchName, sizeof(out->arch) - 1);
    if (char* colon = std::strchr(out->arch, ':')) *colon = '\0';
    out->total_memory_bytes = prop.totalGlobalMem;
    size_t free_b = 0, total_b = 0;
    int current = 0;
    if (hipGetDevice(&current) == hipSuccess && current == device && hipMemGetInfo(&free_b, &total_b) == hipSuccess)
        out->free_memory_bytes = free_b;
    out->compute_units = prop.multiProcessorCount;
    out->wavefront_size = prop.warpSize;
    out->lds_bytes_per_workgroup = static_cast<int32_t>(prop.sharedMemPerBlock);
    out->max_threads_per_workgroup = prop.maxThreadsPerBlock;
    out->clock_khz = prop.clockRate;
    int rt = 0;
    if (hipRuntimeGetVersion(&rt) == hipSuccess) out->runtime_version = rt;
    return AHPC_OK;
}

// A failed allocation must not be reported again by whatever asks for the last error next (every kernel launcher
// does): the error is read here, where it is returned.
int ahpc_hip_malloc(void** ptr, size_t bytes) {
    if (!ptr) return AHPC_ERR_NULL_POINTER;
    const hipError_t e = hipMalloc(ptr, bytes ? bytes : 1);
    if (e != hipSuccess) {
        *ptr = nullptr;
        (void)hipGetLastError();
    }
    return static_cast<int>(e);
}

int ahpc_hip_free(void* ptr) { return ptr ? static_cast<int>(hipFree(ptr)) : AHPC_OK; }

int ahpc_hip_host_malloc(void** ptr, size_t bytes) {
    if (!ptr) return AHPC_ERR_NULL_POINTER;
    const hipError_t e = hipHostMalloc(ptr, bytes ? bytes : 1, hipHostMallocDefault);
    if (e != hipSuccess) {
        *ptr = nullptr;
        (void)hipGetLastError();
    }
    return static_cast<int>(e);
}

int ahpc_hip_host_free(void* ptr) { return ptr ? static_cast<int>(hipHostFree(ptr)) : AHPC_OK; }

// ---- address ranges that grow in place ------------------------------------------------------------------------
// A range of device addresses is reserved once; physical memory is mapped behind its front part on demand
// (hipMemAddressReserve / hipMemCreate / hipMemMap / hipMemSetAccess), in chunks of ONE size per range: on this
// runtime hipMemSetAccess refuses a mapping whose size differs from that of the range's earlier mappings.  Pointers
// into the range stay valid while it grows, nothing is copied and no stream is synchronised.  The library keeps the
// physical handles of every range.
namespace {
struct VmemRange {
    size_t reserved = 0;
    size_t chunk = 0;
    size_t committed = 0;
    int device = 0;
    std::vector<hipMemGenericAllocationHandle_t> chunks;
};
std::mutex g_vmem_mu;
std::map<void*, VmemRange> g_vmem;
constexpr size_t kVmemAlign = size_t(2) << 20;  // chunks are multiples of 2 MiB
size_t round_up(size_t n, size_t to) { return (n + to - 1) / to * to; }
}  // namespace

int ahpc_hip_vmem_granularity(size_t* bytes) {
    if (!bytes) return AHPC_ERR_NULL_POINTER;
    *bytes = 0;
    int dev = 0, sup = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&sup, hipDeviceAttributeVirtualMemoryManagementSupported, dev) != hipSuccess || !sup) {
        (void)hipGetLastError();
        return AHPC_OK;
    }
    *bytes = kVmemAlign;
    return AHPC_OK;
}

int ahpc_hip_vmem_reserve(void** base, size_t bytes, size_t chunk_bytes) {
    if (!base) return AHPC_ERR_NULL_POINTER;
    *base = nullptr;
    if (!bytes || !chunk_bytes) return AHPC_ERR_BAD_SHAPE;
    size_t gran = 0;
    ahpc_hip_vmem_granularity(&gran);
    if (!gran) return AHPC_ERR_NO_DEVICE;
    VmemRange r;
    r.chunk = round_up(chunk_bytes, kVmemAlign);
    r.reserved = round_up(bytes, r.chunk);
    if (hipGetDevice(&r.device) != hipSuccess) return AHPC_ERR_NO_DEVICE;
    void* p = nullptr;
    const hipError_t e = hipMemAddressReserve(&p, r.reserved, 0, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return static_cast<int>(e);
    }
    std::lock_guard<std::mutex> lock(g_vmem_mu);
    g_vmem[p] = r;
    *base = p;
    return AHPC_OK;
}

int ahpc_hip_vmem_commit(void* base, size_t bytes, size_t* committed) {
    std::lock_guard<std::mutex> lock(g_vmem_mu);
    auto it = g_vmem.find(base);
    if (it == g_vmem.end()) return AHPC_ERR_NULL_POINTER;
    VmemRange& r = it->second;
    if (committed) *committed = r.committed;
    const size_t want = round_up(bytes, r.chunk);
    if (want > r.reserved) return AHPC_ERR_BAD_SHAPE;
    hipMemAllocationProp prop = {};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = r.device;
    hipMemAccessDesc acc = {};
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = r.device;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    while (r.committed < want) {
        // one chunk at a time: whatever fails, the chunks mapped so far stay usable and nothing half-mapped is left
        hipMemGenericAllocationHandle_t h;
        hipError_t e = hipMemCreate(&h, r.chunk, &prop, 0);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return static_cast<int>(e);  // (out of memory)
        }
        char* at = static_cast<char*>(base) + r.committed;
        e = hipMemMap(at, r.chunk, 0, h, 0);
        if (e == hipSuccess) {
            e = hipMemSetAccess(at, r.chunk, &acc, 1);
            if (e != hipSuccess) (void)hipMemUnmap(at, r.chunk);
        }
        if (e != hipSuccess) {
            (void)hipMemRelease(h);
            (void)hipGetLastError();
            return static_cast<int>(e);
        }
        r.chunks.push_back(h);
        r.committed += r.chunk;
        if (committed) *committed = r.committed;
    }
    return AHPC_OK;
}

int ahpc_hip_vmem_decommit(void* base, size_t keep_bytes, size_t* committed) {
    std::lock_guard<std::mutex> lock(g_vmem_mu);
    auto it = g_vmem.find(base);
    if (it == g_vmem.end()) return AHPC_ERR_NULL_POINTER;
    VmemRange& r = it->second;
    const size_t keep = round_up(keep_bytes, r.chunk);
    hipError_t first = hipSuccess;
    while (r.committed > keep && !r.chunks.empty()) {
        char* at = static_cast<char*>(base) + r.committed - r.chunk;
        hipError_t e = hipMemUnmap(at, r.chunk);
        if (e != hipSuccess) {  // (still mapped: leave the books as they are)
            first = e;
            break;
        }
        e = hipMemRelease(r.chunks.back());
        if (e != hipSuccess && first == hipSuccess) first = e;
        r.chunks.pop_back();
        r.committed -= r.chunk;
    }
    if (committed) *committed = r.committed;
    if (first != hipSuccess) (void)hipGetLastError();
    return static_cast<int>(first);
}

int ahpc_hip_vmem_release(void* base) {
    if (!base) return AHPC_OK;
    std::lock_guard<std::mutex> lock(g_vmem_mu);
    auto it = g_vmem.find(base);
    if (it == g_vmem.end()) return AHPC_ERR_NULL_POINTER;
    VmemRange& r = it->second;
    hipError_t first = hipSuccess;
    for (size_t i = 0; i < r.chunks.size(); ++i) {
        hipError_t e = hipMemUnmap(static_cast<char*>(base) + i * r.chunk, r.chunk);
        if (e != hipSuccess && first == hipSuccess) first = e;
        e = hipMemRelease(r.chunks[i]);
        if (e != hipSuccess && first == hipSuccess) first = e;
    }
    const hipError_t e = hipMemAddressFree(base, r.reserved);
    if (e != hipSuccess && first == hipSuccess) first = e;
    g_vmem.erase(it);
    if (first != hipSuccess) (void)hipGetLastError();
    return static_cast<int>(first);
}

int ahpc_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
    if (!bytes) return AHPC_OK;
    if (!dst || !src) return AHPC_ERR_NULL_POINTER;
    return static_cast<int>(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
}

int ahpc_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
    if (!bytes) return AHPC_OK;
    if (!dst || !src) return AHPC_ERR_NULL_POINTER;
    return static_cast<int>(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
}

int ahpc_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
    if (!bytes) return AHPC_OK;
    if (!dst || !src) return AHPC_ERR_NULL_POINTER;
    return static_cast<int>(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
}

int ahpc_hip_memset(void* dst, int byte_value, size_t bytes, void* stream) {
    if (!bytes) return AHPC_OK;
    if (!dst) return AHPC_ERR_NULL_POINTER;
    return static_cast<int>(hipMemsetAsync(dst, byte_value, bytes, static_cast<hipStream_t>(stream)));
}

int ahpc_hip_ptr_is_device(const void* ptr, int* is_device) {
    if (!is_device) return AHPC_ERR_NULL_POINTER;
    *is_device = 0;
    if (!ptr) return AHPC_OK;
    hipPointerAttribute_t attr;
    hipError_t e = hipPointerGetAttributes(&attr, ptr);
    if (e != hipSuccess) {
        (void)hipGetLastError();  // ordinary host memory is reported as an error: not one for us
        return AHPC_OK;
    }
    *is_device = (attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged) ? 1 : 0;
    return AHPC_OK;
}

int ahpc_hip_stream_create(void** stream) {
    if (!stream) return AHPC_ERR_NULL_POINTER;
    hipStream_t s = nullptr;
    hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
    *stream = s;
    return static_cast<int>(e);
}

int ahpc_hip_stream_destroy(void* stream) {
    return stream ? static_cast<int>(hipStreamDestroy(static_cast<hipStream_t>(stream))) : AHPC_OK;
}

int ahpc_hip_stream_synchronize(void* stream) {
    return static_cast<int>(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
}

int ahpc_hip_device_synchronize(void) { return static_cast<int>(hipDeviceSynchronize()); }

int ahpc_hip_event_create(void** event) {
    if (!event) return AHPC_ERR_NULL_POINTER;
    hipEvent_t ev = nullptr;
    hipError_t e = hipEventCreate(&ev);
    *event = ev;
    return static_cast<int>(e);
}

int ahpc_hip_event_destroy(void* event) {
    return event ? static_cast<int>(hipEventDestroy(static_cast<hipEvent_t>(event))) : AHPC_OK;
}

int ahpc_hip_event_record(void* event, void* stream) {
    if (!event) return AHPC_ERR_NULL_POINTER;
    return static_cast<int>(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
}

int ahpc_hip_event_synchronize(void* event) {
    if (!event) return AHPC_ERR_NULL_POINTER;
    return static_cast<int>(hipEventSynchronize(static_cast<hipEvent_t>(event)));
}

int ahpc_hip_event_elapsed_ms(void* start, void* stop, float* ms) {
    if (!start || !stop || !ms) return AHPC_ERR_NULL_POINTER;
    return static_cast<int>(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
}

}  // extern "C"
