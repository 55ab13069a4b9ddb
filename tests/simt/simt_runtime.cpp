// Test infrastructure: executes kernels compiled against shim/hip/hip_runtime.h on the CPU.
// One operating-system thread; every work-item of the workgroup being executed is a ucontext fiber.
// A fiber runs until it needs the other lanes (cross-lane operation, barrier) and then yields; the
// scheduler resumes fibers whose condition has become true, visiting wavefronts in a seeded random
// order so that different interleavings of the wavefronts of a workgroup are exercised.
#include <hip/hip_runtime.h>
#include <sys/mman.h>
#include <ucontext.h>

#include <algorithm>
#include <cstdio>
#include <mutex>
#include <string>
#include <vector>

#if defined(__has_feature)
#if __has_feature(address_sanitizer)
#define SIMT_ASAN 1
extern "C" void __sanitizer_start_switch_fiber(void** fake_stack_save, const void* bottom, size_t size);
extern "C" void __sanitizer_finish_switch_fiber(void* fake_stack_save, const void** bottom_old, size_t* size_old);
#endif
#endif

dim3 threadIdx, blockIdx, blockDim, gridDim;

extern "C" unsigned char __start_simt_lds[];
extern "C" unsigned char __stop_simt_lds[];

namespace simt {
namespace {

constexpr int kWaveSize = 64;
constexpr int kPayload = 64;          // bytes a lane can publish per cross-lane operation
constexpr size_t kStackBytes = 512 * 1024;

enum Kind : int { K_NONE = 0, K_MFMA, K_TR, K_SWAP, K_BALLOT, K_RFL, K_RL, K_DPP, K_SHFL, K_LDS128, K_WAIT };

struct PendingDma {
    unsigned char* dst;
    const unsigned char* src;  // null: zeros
    int bytes;
};

struct Wave {
    int live = 0;
    int arrived[2] = {0, 0};
    long gen_of[2] = {-1, -1};
    int kind[2] = {K_NONE, K_NONE};
    bool present[2][kWaveSize];
    alignas(16) unsigned char slot[2][kWaveSize][kPayload];
};

struct Fiber {
    ucontext_t ctx;
    unsigned char* stack = nullptr;
    dim3 tid;
    int wave = 0, lane = 0;
    bool done = false;
    const int* wait_counter = nullptr;  // resume when *wait_counter >= *wait_target
    const int* wait_target = nullptr;
    long coll_gen = 0, bar_gen = 0;
    std::vector<PendingDma> dma;
    void* asan_fake = nullptr;
};

struct Block {
    std::vector<Fiber> fibers;
    std::vector<Wave> waves;
    int live = 0;
    int bar_arrived[2] = {0, 0};
    long bar_gen_of[2] = {-1, -1};
};

Block g_block;
Fiber* g_cur = nullptr;
ucontext_t g_main;
void* g_main_fake = nullptr;
const void* g_main_bottom = nullptr;  // the scheduler's stack, as AddressSanitizer reports it
size_t g_main_size = 0;
const std::function<void()>* g_body = nullptr;
std::string g_error;
thread_local hipError_t g_status = hipSuccess;  // what hipGetLastError reports to the launching thread
std::mutex g_launch_mutex;                      // one launch at a time: the executor's state is global
bool g_dma_late = false;
uint64_t g_rng = 0x9E3779B97F4A7C15ull;
std::vector<unsigned char*> g_stacks;  // reused between launches
long g_switches = 0;
long g_lds_stats[4] = {0, 0, 0, 0};  // 16-byte reads, their conflict cycles, transposing reads, theirs

// ---- ordering of LDS traffic between wavefronts ----------------------------------------------------
// A work-item's epoch is the number of workgroup barriers it has passed (at any moment all running
// work-items of a workgroup are in the same epoch).  Per 8-byte granule of LDS: which wavefront last wrote
// it with a direct-to-LDS load and in which epoch the issuing lane waited for it (-1: not yet), and which
// wavefronts have read it with one of the traced reads (16-byte operand reads, transposing reads) in the
// latest epoch it was read in.  Two accesses of different wavefronts to one granule, one of them a load's
// write, are ordered only by a barrier between them; a load is "between" its issue and its wait.  Plain
// C++ accesses to LDS are not seen.
constexpr int kMaxWaves = 16;
constexpr int kGranule = 8;
struct GranuleState {
    uint64_t workgroup = 0;  // serial number of the workgroup this state belongs to; older states count as fresh
    int32_t waited = -1;
    int32_t read_epoch = -1;
    int16_t writer = -1;
    uint16_t readers = 0;    // wavefronts that read it in read_epoch
};
std::vector<GranuleState> g_granules;
uint64_t g_workgroup_serial = 0;

void reset_granule_states() {
    ++g_workgroup_serial;
    const size_t n = (size_t)(__stop_simt_lds - __start_simt_lds + kGranule - 1) / kGranule;
    if (g_granules.size() != n) g_granules.assign(n, GranuleState());
}
// The states of the granules that [p, p + bytes) touches, made fresh if they belong to an earlier workgroup.
GranuleState* granules_of(const void* p, int bytes, int* count) {
    const size_t off = (size_t)(static_cast<const unsigned char*>(p) - __start_simt_lds);
    const size_t first = off / kGranule, last = (off + (size_t)bytes - 1) / kGranule;
    *count = (int)(last - first + 1);
    GranuleState* g = &g_granules[first];
    for (int i = 0; i < *count; ++i)
        if (g[i].workgroup != g_workgroup_serial) {
            g[i] = GranuleState();
            g[i].workgroup = g_workgroup_serial;
        }
    return g;
}

uint64_t next_rand() {
    g_rng ^= g_rng << 13;
    g_rng ^= g_rng >> 7;
    g_rng ^= g_rng << 17;
    return g_rng;
}

void enter_fiber(Fiber* f) {
    g_cur = f;
    threadIdx = f->tid;
    ++g_switches;
#ifdef SIMT_ASAN
    __sanitizer_start_switch_fiber(&g_main_fake, f->stack, kStackBytes);
#endif
    swapcontext(&g_main, &f->ctx);
#ifdef SIMT_ASAN
    __sanitizer_finish_switch_fiber(g_main_fake, nullptr, nullptr);
#endif
    g_cur = nullptr;
}

void yield_to_scheduler() {
    Fiber* f = g_cur;
#ifdef SIMT_ASAN
    __sanitizer_start_switch_fiber(&f->asan_fake, g_main_bottom, g_main_size);
#endif
    swapcontext(&f->ctx, &g_main);
#ifdef SIMT_ASAN
    __sanitizer_finish_switch_fiber(f->asan_fake, &g_main_bottom, &g_main_size);
#endif
    threadIdx = f->tid;
}

[[noreturn]] void leave_for_good() {
    // Used on errors and at the end of a fiber: never comes back to this fiber.
    Fiber* f = g_cur;
#ifdef SIMT_ASAN
    __sanitizer_start_switch_fiber(nullptr, g_main_bottom, g_main_size);
#endif
    swapcontext(&f->ctx, &g_main);
    std::abort();
}

void fail(const std::string& what) {
    if (g_error.empty()) {
        char where[160];
        if (g_cur)
            std::snprintf(where, sizeof where, " [block (%u,%u,%u) thread %u wave %d lane %d]", blockIdx.x, blockIdx.y,
                          blockIdx.z, g_cur->tid.x, g_cur->wave, g_cur->lane);
        else
            where[0] = 0;
        g_error = what + where;
        std::fprintf(stderr, "simt: %s\n", g_error.c_str());
    }
    g_status = hipErrorLaunchFailure;
    if (g_cur) {
        g_cur->done = true;  // the scheduler stops at the first error
        leave_for_good();
    }
}

void note_dma_landed(const struct Fiber* f, const void* p, int bytes);

// Lands this lane's outstanding direct-to-LDS loads, oldest first, until at most `leave` are outstanding
// (loads complete in the order they were issued).
void flush_dma(Fiber* f, size_t leave = 0) {
    size_t n = f->dma.size() > leave ? f->dma.size() - leave : 0;
    for (size_t i = 0; i < n; ++i) {
        const PendingDma& d = f->dma[i];
        if (d.src) std::memcpy(d.dst, d.src, (size_t)d.bytes);
        else std::memset(d.dst, 0, (size_t)d.bytes);
        note_dma_landed(f, d.dst, d.bytes);
    }
    f->dma.erase(f->dma.begin(), f->dma.begin() + (long)n);
}

// A traced read of `bytes` bytes at p by the running work-item.
void note_lds_read(const void* p, int bytes) {
    Fiber* f = g_cur;
    const int e = (int)f->bar_gen;
    int n;
    GranuleState* g = granules_of(p, bytes, &n);
    for (int i = 0; i < n; ++i, ++g) {
        if (g->writer >= 0) {
            if (g->waited < 0)
                fail(g->writer == f->wave ? "LDS read of a direct-to-LDS load that its wavefront has not waited for"
                                          : "LDS read of a direct-to-LDS load of another wavefront that is still in flight");
            else if (g->writer != f->wave && g->waited >= e)
                fail("LDS read races with a direct-to-LDS load of another wavefront: no barrier between the wait for the load and the read");
        }
        if (g->read_epoch != e) {
            g->read_epoch = e;
            g->readers = 0;
        }
        if (f->wave < kMaxWaves) g->readers |= (uint16_t)(1u << f->wave);
    }
}

// A direct-to-LDS load of `bytes` bytes to p issued by the running work-item.
void note_dma_issue(const void* p, int bytes) {
    Fiber* f = g_cur;
    const int e = (int)f->bar_gen;
    const uint16_t me = f->wave < kMaxWaves ? (uint16_t)(1u << f->wave) : 0;
    int n;
    GranuleState* g = granules_of(p, bytes, &n);
    for (int i = 0; i < n; ++i, ++g) {
        if (g->read_epoch == e && (g->readers & ~me) != 0)
            fail("direct-to-LDS load overwrites LDS that another wavefront has read since the last barrier");
        if (g->writer >= 0 && g->writer != f->wave && (g->waited < 0 || g->waited >= e))
            fail("direct-to-LDS loads of two wavefronts write the same LDS without a barrier between them");
        g->writer = (int16_t)f->wave;
        g->waited = -1;
    }
}

void note_dma_landed(const Fiber* f, const void* p, int bytes) {
    int n;
    GranuleState* g = granules_of(p, bytes, &n);
    for (int i = 0; i < n; ++i, ++g)
        if (g->writer == f->wave && g->waited < 0) g->waited = (int32_t)f->bar_gen;
}

void wait_until(const int* counter, const int* target) {
    Fiber* f = g_cur;
    while (*counter < *target) {
        f->wait_counter = counter;
        f->wait_target = target;
        yield_to_scheduler();
        if (g_status != hipSuccess) {
            f->done = true;
            leave_for_good();
        }
    }
    f->wait_counter = f->wait_target = nullptr;
}

void trampoline() {
#ifdef SIMT_ASAN
    __sanitizer_finish_switch_fiber(nullptr, &g_main_bottom, &g_main_size);
#endif
    Fiber* f = g_cur;
    threadIdx = f->tid;
    (*g_body)();
    flush_dma(f);  // the hardware completes outstanding loads of a finished wave as well
    f->done = true;
    g_block.waves[f->wave].live--;
    g_block.live--;
    leave_for_good();
}

// Publishes `n` bytes for the other lanes of the wavefront and waits until every live lane of the
// wavefront has published for the same operation.  Returns the generation's slot table.
struct View {
    const Wave* w;
    int g;
    const unsigned char* of(int lane) const {
        if (!w->present[g][lane]) fail("cross-lane operation reads a lane that is not executing it");
        return w->slot[g][lane];
    }
    bool has(int lane) const { return w->present[g][lane]; }
};

View exchange(int kind, const void* payload, size_t n) {
    Fiber* f = g_cur;
    if (!f) {
        std::fprintf(stderr, "simt: cross-lane operation outside a kernel\n");
        std::abort();
    }
    Wave& w = g_block.waves[f->wave];
    const long gen = f->coll_gen++;
    const int g = (int)(gen & 1);
    if (w.gen_of[g] != gen) {
        w.gen_of[g] = gen;
        w.arrived[g] = 0;
        w.kind[g] = kind;
        std::memset(w.present[g], 0, sizeof w.present[g]);
    }
    if (w.kind[g] != kind) fail("lanes of one wavefront are at different cross-lane operations (divergent control flow)");
    if (n > (size_t)kPayload) fail("internal: payload too large");
    std::memcpy(w.slot[g][f->lane], payload, n);
    w.present[g][f->lane] = true;
    w.arrived[g]++;
    wait_until(&w.arrived[g], &w.live);
    return View{&w, g};
}

bool in_lds(const void* p, size_t n) {
    const unsigned char* q = static_cast<const unsigned char*>(p);
    return q >= __start_simt_lds && q + n <= __stop_simt_lds;
}

// Extra cycles a wave-wide LDS read costs under a model of 64 banks of 4 bytes: the lanes are served
// `lanes_per_pass` at a time (256 bytes per pass); a pass takes as many cycles as the largest number of
// different dwords that fall into one bank.
long conflict_cycles(const View& v, int bytes_per_lane, int lanes_per_pass) {
    long extra = 0;
    for (int first = 0; first < kWaveSize; first += lanes_per_pass) {
        uint64_t dwords[64][16];
        int count[64] = {0};
        for (int l = first; l < first + lanes_per_pass; ++l) {
            if (!v.has(l)) continue;
            uint64_t addr;
            std::memcpy(&addr, v.of(l) + 16, 8);
            addr -= reinterpret_cast<uint64_t>(__start_simt_lds);
            for (int o = 0; o < bytes_per_lane; o += 4) {
                const uint64_t dw = (addr + o) / 4;
                const int bank = (int)(dw % 64);
                bool seen = false;
                for (int i = 0; i < count[bank]; ++i) seen = seen || dwords[bank][i] == dw;
                if (!seen && count[bank] < 16) dwords[bank][count[bank]++] = dw;
            }
        }
        int worst = 1;
        for (int b = 0; b < 64; ++b) worst = std::max(worst, count[b]);
        extra += worst - 1;
    }
    return extra;
}

bool first_live_lane(const View& v, int lane) {
    for (int l = 0; l < lane; ++l)
        if (v.has(l)) return false;
    return true;
}

template <typename T> float to_f32(T x) { return (float)x; }

template <typename V> f32x16 mfma_impl(V a, V b, f32x16 c) {
    struct Ops {
        V a, b;
    } mine{a, b};
    const View v = exchange(K_MFMA, &mine, sizeof mine);
    const Fiber* f = g_cur;
    const int col = f->lane & 31, half = f->lane >> 5;
    f32x16 d = c;
    for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r / 4) + 4 * half + (r % 4);
        double acc = 0.0;
        for (int kh = 0; kh < 2; ++kh) {
            Ops oa, ob;
            std::memcpy(&oa, v.of(row + 32 * kh), sizeof oa);  // A[row][8*kh ..]
            std::memcpy(&ob, v.of(col + 32 * kh), sizeof ob);  // B[8*kh ..][col]
            for (int e = 0; e < 8; ++e) acc += (double)to_f32(oa.a[e]) * (double)to_f32(ob.b[e]);
        }
        d[r] = (float)((double)c[r] + acc);
    }
    return d;
}

// 16x16 matrix instructions: lane l supplies A[row l%16][k KPL*(l/16) ..] and B[k KPL*(l/16) ..][col l%16] and
// receives D[row 4*(l/16) + r][col l%16] in acc[r].
template <int KPL, typename V, typename F> f32x4 mfma16_impl(V a, V b, f32x4 c, F to_float) {
    struct Ops {
        V a, b;
    } mine{a, b};
    const View v = exchange(K_MFMA, &mine, sizeof mine);
    const Fiber* f = g_cur;
    const int col = f->lane & 15, rg = f->lane >> 4;
    f32x4 d = c;
    for (int r = 0; r < 4; ++r) {
        const int row = 4 * rg + r;
        double acc = 0.0;
        for (int kg = 0; kg < 4; ++kg) {
            Ops oa, ob;
            std::memcpy(&oa, v.of(row + 16 * kg), sizeof oa);
            std::memcpy(&ob, v.of(col + 16 * kg), sizeof ob);
            for (int e = 0; e < KPL; ++e) acc += (double)to_float(oa.a[e]) * (double)to_float(ob.b[e]);
        }
        d[r] = (float)((double)c[r] + acc);
    }
    return d;
}

float bf16_bits_to_f32(short bits) {
    const uint32_t w = (uint32_t)(uint16_t)bits << 16;
    float x;
    std::memcpy(&x, &w, 4);
    return x;
}

}  // namespace

// ---- what the shim header declares --------------------------------------------------------------
hipError_t last_error() {
    const hipError_t s = g_status;
    g_status = hipSuccess;
    return s;
}

int lane_id() { return g_cur ? g_cur->lane : 0; }

void syncthreads() {
    Fiber* f = g_cur;
    Block& b = g_block;
    const long gen = f->bar_gen++;
    const int g = (int)(gen & 1);
    if (b.bar_gen_of[g] != gen) {
        b.bar_gen_of[g] = gen;
        b.bar_arrived[g] = 0;
    }
    b.bar_arrived[g]++;
    wait_until(&b.bar_arrived[g], &b.live);
}

f32x16 mfma_32x32x16_f16(f16x8 a, f16x8 b, f32x16 c) { return mfma_impl(a, b, c); }
f32x16 mfma_32x32x16_bf16(bf16x8 a, bf16x8 b, f32x16 c) { return mfma_impl(a, b, c); }

// v_mfma_f32_32x32x2_f32: lane l supplies A[row l%32][k l/32] and B[k l/32][col l%32]; results laid out as above.
f32x16 mfma_32x32x2_f32(float a, float b, f32x16 c) {
    struct Ops {
        float a, b;
    } mine{a, b};
    const View v = exchange(K_MFMA, &mine, sizeof mine);
    const Fiber* f = g_cur;
    const int col = f->lane & 31, half = f->lane >> 5;
    f32x16 d = c;
    for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r / 4) + 4 * half + (r % 4);
        double acc = 0.0;
        for (int kh = 0; kh < 2; ++kh) {
            Ops oa, ob;
            std::memcpy(&oa, v.of(row + 32 * kh), sizeof oa);
            std::memcpy(&ob, v.of(col + 32 * kh), sizeof ob);
            acc += (double)oa.a * (double)ob.b;
        }
        d[r] = (float)((double)c[r] + acc);
    }
    return d;
}
f32x4 mfma_16x16x32_f16(f16x8 a, f16x8 b, f32x4 c) { return mfma16_impl<8>(a, b, c, [](_Float16 x) { return (float)x; }); }
f32x4 mfma_16x16x32_bf16(bf16x8 a, bf16x8 b, f32x4 c) { return mfma16_impl<8>(a, b, c, [](__bf16 x) { return (float)x; }); }
f32x4 mfma_16x16x16_f16(f16x4 a, f16x4 b, f32x4 c) { return mfma16_impl<4>(a, b, c, [](_Float16 x) { return (float)x; }); }
f32x4 mfma_16x16x16_bf16(s16x4 a, s16x4 b, f32x4 c) { return mfma16_impl<4>(a, b, c, bf16_bits_to_f32); }

// ds_read_b64_tr_b16: the 16 lanes of a row each address four 16-bit elements; lane j of the row
// receives element (j % 4) of the lanes 4*r + j/4, r = 0..3 (a 16x4 block handed out transposed).
uint64_t ds_read_tr16_b64(const void* lds_ptr) {
    uint64_t mine = 0;
    if (!in_lds(lds_ptr, 8)) fail("transposing LDS read outside the workgroup's LDS");
    if ((reinterpret_cast<uintptr_t>(lds_ptr) & 7) != 0) fail("transposing LDS read not 8-byte aligned");
    std::memcpy(&mine, lds_ptr, 8);
    unsigned char payload[24] = {0};
    std::memcpy(payload, &mine, 8);
    const uint64_t addr = reinterpret_cast<uint64_t>(lds_ptr);
    std::memcpy(payload + 16, &addr, 8);
    const View v = exchange(K_TR, payload, sizeof payload);
    note_lds_read(lds_ptr, 8);
    const int lane = g_cur->lane, row0 = lane & ~15, j = lane & 15;
    if (first_live_lane(v, lane)) {
        g_lds_stats[2] += 1;
        g_lds_stats[3] += conflict_cycles(v, 8, 32);
    }
    uint16_t out[4];
    for (int r = 0; r < 4; ++r) {
        uint16_t src[4];
        std::memcpy(src, v.of(row0 + 4 * r + j / 4), 8);
        out[r] = src[j % 4];
    }
    uint64_t res;
    std::memcpy(&res, out, 8);
    return res;
}

u32x4 lds_read_b128(const void* lds_ptr) {
    if (!in_lds(lds_ptr, 16)) fail("16-byte LDS read outside the workgroup's LDS");
    if ((reinterpret_cast<uintptr_t>(lds_ptr) & 15) != 0) fail("16-byte LDS read not 16-byte aligned");
    unsigned char payload[24] = {0};
    const uint64_t addr = reinterpret_cast<uint64_t>(lds_ptr);
    std::memcpy(payload + 16, &addr, 8);
    const View v = exchange(K_LDS128, payload, sizeof payload);
    if (first_live_lane(v, g_cur->lane)) {
        g_lds_stats[0] += 1;
        g_lds_stats[1] += conflict_cycles(v, 16, 16);
    }
    note_lds_read(lds_ptr, 16);
    u32x4 r;
    std::memcpy(&r, lds_ptr, 16);
    return r;
}

// v_permlane32_swap a, b: the upper 32 lanes of a and the lower 32 lanes of b change places.
u32x2 permlane32_swap(unsigned a, unsigned b) {
    unsigned mine[2] = {a, b};
    const View v = exchange(K_SWAP, mine, 8);
    const int lane = g_cur->lane;
    unsigned other[2];
    std::memcpy(other, v.of(lane ^ 32), 8);
    u32x2 r;
    if (lane < 32) {
        r[0] = a;
        r[1] = other[0];  // a of lane + 32
    } else {
        r[0] = other[1];  // b of lane - 32
        r[1] = b;
    }
    return r;
}

uint64_t ballot(bool pred) {
    const unsigned char mine = pred ? 1 : 0;
    const View v = exchange(K_BALLOT, &mine, 1);
    uint64_t m = 0;
    for (int l = 0; l < kWaveSize; ++l)
        if (v.has(l) && *v.of(l)) m |= 1ull << l;
    return m;
}

int readfirstlane(int x) {
    const View v = exchange(K_RFL, &x, 4);
    for (int l = 0; l < kWaveSize; ++l)
        if (v.has(l)) {
            int r;
            std::memcpy(&r, v.of(l), 4);
            return r;
        }
    return x;
}

int readlane(int x, int lane) {
    if (lane < 0 || lane >= kWaveSize) fail("readlane: lane index out of range");
    const View v = exchange(K_RL, &x, 4);
    int r;
    std::memcpy(&r, v.of(lane), 4);
    return r;
}

int update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
    (void)old;
    (void)bound_ctrl;
    if (row_mask != 0xF || bank_mask != 0xF) fail("update_dpp: only full row and bank masks are modelled");
    const View v = exchange(K_DPP, &src, 4);
    const int lane = g_cur->lane;
    int from;
    if (ctrl >= 0 && ctrl <= 0xFF) from = (lane & ~3) | ((ctrl >> (2 * (lane & 3))) & 3);  // quad_perm
    else if (ctrl == 0x140) from = (lane & ~15) | (15 - (lane & 15));                       // row_mirror
    else if (ctrl == 0x141) from = (lane & ~7) | (7 - (lane & 7));                          // row_half_mirror
    else {
        fail("update_dpp: control value not modelled");
        return 0;
    }
    int r;
    std::memcpy(&r, v.of(from), 4);
    return r;
}

int shfl_xor_bits(int x, int mask, int width) {
    if (width != kWaveSize) fail("shuffle width other than 64 is not modelled");
    const View v = exchange(K_SHFL, &x, 4);
    const int from = g_cur->lane ^ mask;
    if (from < 0 || from >= kWaveSize) return x;
    int r;
    std::memcpy(&r, v.of(from), 4);
    return r;
}

// buffer_load_dwordx4 ... lds: lane i's 16 bytes go to lds_base + imm + 16*i; a source range that is
// not completely inside the descriptor reads as zeros.
void buffer_load_lds(BufferRsrc r, void* lds_base, int size, int voffset, int soffset, int imm, int aux) {
    (void)aux;
    if (size != 16 && size != 4) fail("buffer_load_lds: only 4- and 16-byte loads are modelled");
    Fiber* f = g_cur;
    unsigned char* dst = static_cast<unsigned char*>(lds_base) + imm + size * f->lane;
    if (!in_lds(dst, (size_t)size)) fail("buffer_load_lds writes outside the workgroup's LDS");
    const uint64_t off = (uint64_t)(uint32_t)voffset + (uint64_t)(uint32_t)soffset + (uint64_t)(uint32_t)imm;
    if (voffset < 0) fail("buffer_load_lds: negative lane offset");
    const bool inside = off + (uint64_t)size <= (uint64_t)r.num_records;
    note_dma_issue(dst, size);
    PendingDma d{dst, inside ? r.base + off : nullptr, size};
    if (g_dma_late) f->dma.push_back(d);
    else {
        f->dma.push_back(d);
        flush_dma(f);
    }
}

// s_waitcnt with the gfx9 encoding: vmcnt in bits 3:0 and 15:14; the other counters are not modelled
// (LDS and scalar accesses are synchronous here).
// The wait belongs to the wavefront: no lane goes on before every lane's loads have landed (a lane may read
// next what another lane's direct-to-LDS load brought in).
void waitcnt(int imm) {
    const int vmcnt = (imm & 0xF) | (((imm >> 14) & 3) << 4);
    if (!g_cur) return;
    flush_dma(g_cur, (size_t)vmcnt);
    unsigned char nothing[8] = {0};
    exchange(K_WAIT, nothing, sizeof nothing);
}

void launch(dim3 grid, dim3 block, const std::function<void()>& body) {
    if (g_status != hipSuccess) return;
    std::lock_guard<std::mutex> guard(g_launch_mutex);
    const int n = (int)(block.x * block.y * block.z);
    if (n <= 0 || n > 1024) {
        g_status = hipErrorLaunchFailure;
        g_error = "launch: bad workgroup size";
        return;
    }
    if (grid.x == 0 || grid.y == 0 || grid.z == 0) {
        g_status = hipErrorLaunchFailure;
        g_error = "launch: empty grid";
        return;
    }
    while ((int)g_stacks.size() < n) g_stacks.push_back(static_cast<unsigned char*>(std::malloc(kStackBytes)));
    const int n_waves = (n + kWaveSize - 1) / kWaveSize;
    gridDim = grid;
    blockDim = block;
    g_body = &body;
    std::vector<int> order(n_waves);
    for (unsigned bz = 0; bz < grid.z && g_status == hipSuccess; ++bz)
        for (unsigned by = 0; by < grid.y && g_status == hipSuccess; ++by)
            for (unsigned bx = 0; bx < grid.x && g_status == hipSuccess; ++bx) {
                blockIdx = dim3(bx, by, bz);
                std::memset(__start_simt_lds, 0xFF, (size_t)(__stop_simt_lds - __start_simt_lds));
                reset_granule_states();
                Block& b = g_block;
                b.fibers.assign(n, Fiber());
                b.waves.assign(n_waves, Wave());
                b.live = n;
                b.bar_arrived[0] = b.bar_arrived[1] = 0;
                b.bar_gen_of[0] = b.bar_gen_of[1] = -1;
                for (int i = 0; i < n; ++i) {
                    Fiber& f = b.fibers[i];
                    f.stack = g_stacks[i];
                    f.tid = dim3(i % block.x, (i / block.x) % block.y, i / (block.x * block.y));
                    f.wave = i / kWaveSize;
                    f.lane = i % kWaveSize;
                    b.waves[f.wave].live++;
                    getcontext(&f.ctx);
                    f.ctx.uc_stack.ss_sp = f.stack;
                    f.ctx.uc_stack.ss_size = kStackBytes;
                    f.ctx.uc_link = nullptr;
                    makecontext(&f.ctx, trampoline, 0);
                }
                while (b.live > 0 && g_status == hipSuccess) {
                    for (int w = 0; w < n_waves; ++w) order[w] = w;
                    for (int w = n_waves - 1; w > 0; --w) std::swap(order[w], order[next_rand() % (uint64_t)(w + 1)]);
                    bool progressed = false;
                    for (int wi = 0; wi < n_waves && g_status == hipSuccess; ++wi) {
                        const int w = order[wi];
                        const int lo = w * kWaveSize, hi = std::min(n, lo + kWaveSize);
                        for (int i = lo; i < hi && g_status == hipSuccess; ++i) {
                            Fiber& f = b.fibers[i];
                            if (f.done) continue;
                            if (f.wait_counter && *f.wait_counter < *f.wait_target) continue;
                            progressed = true;
                            enter_fiber(&f);
                        }
                    }
                    if (!progressed && b.live > 0 && g_status == hipSuccess) {
                        int at_barrier = 0, at_cross = 0;
                        for (const Fiber& f : b.fibers)
                            if (!f.done) {
                                if (f.wait_target == &b.live) ++at_barrier;
                                else ++at_cross;
                            }
                        char msg[200];
                        std::snprintf(msg, sizeof msg,
                                      "workgroup (%u,%u,%u) cannot make progress: %d work-items wait at a barrier, %d at a "
                                      "cross-lane operation",
                                      bx, by, bz, at_barrier, at_cross);
                        g_error = msg;
                        std::fprintf(stderr, "simt: %s\n", msg);
                        g_status = hipErrorLaunchFailure;
                    }
                }
            }
    g_body = nullptr;
}

}  // namespace simt

// ---- emulated virtual memory management: an inaccessible mapping, made accessible piece by piece ------------------
int simt_fail_device_alloc_in = 0;
hipError_t hipMemAddressReserve(void** p, size_t n, size_t, void*, unsigned long long) {
    void* m = mmap(nullptr, n, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (m == MAP_FAILED) return 2;
    *p = m;
    return hipSuccess;
}
hipError_t hipMemAddressFree(void* p, size_t n) { return munmap(p, n) == 0 ? hipSuccess : 1; }
hipError_t hipMemMap(void* p, size_t n, size_t, hipMemGenericAllocationHandle_t, unsigned long long) {
    return mprotect(p, n, PROT_READ | PROT_WRITE) == 0 ? hipSuccess : 1;
}
hipError_t hipMemUnmap(void* p, size_t n) {
    madvise(p, n, MADV_DONTNEED);
    return mprotect(p, n, PROT_NONE) == 0 ? hipSuccess : 1;
}

// ---- control from the tests (ctypes) ---------------------------------------------------------------
extern "C" {
// The n-th device allocation from now on fails (1 = the next one); 0 switches the countdown off.
void simt_fail_device_alloc(int n) { simt_fail_device_alloc_in = n; }
// dma_late != 0: direct-to-LDS loads land at the issuing lane's next s_waitcnt instead of at issue.
// seed: order in which the wavefronts of a workgroup are advanced.
void simt_configure(int dma_late, uint64_t seed) {
    simt::g_dma_late = dma_late != 0;
    simt::g_rng = seed * 0x9E3779B97F4A7C15ull + 0x2545F4914F6CDD1Dull;
    if (simt::g_rng == 0) simt::g_rng = 1;
}
const char* simt_last_error_text() { return simt::g_error.c_str(); }
void simt_clear_error() {
    simt::g_error.clear();
    simt::g_status = hipSuccess;
}
long simt_switch_count() { return simt::g_switches; }
// out[0..3] = 16-byte LDS reads executed (per wavefront), their extra cycles from bank conflicts, transposing
// reads, their extra cycles; counted since the last reset.
void simt_lds_stats(long* out) {
    for (int i = 0; i < 4; ++i) out[i] = simt::g_lds_stats[i];
}
void simt_lds_stats_reset() {
    for (long& x : simt::g_lds_stats) x = 0;
}
}
