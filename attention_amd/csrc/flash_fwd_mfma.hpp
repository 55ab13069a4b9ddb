// FlashAttention forward on the gfx950 matrix cores (fp16 / bf16 storage, fp32 accumulate).
//
// One workgroup = 4 wavefronts = 128 query rows of one (sequence, head); it walks the keys in tiles
// of 64.  Two workgroups share a CU (<= 256 registers per lane, 2 x 64 KiB of LDS), so that one
// wavefront's softmax (VALU) overlaps the other's matrix work on the same SIMD.  Per tile and wave:
//   S^T = K * Q^T      v_mfma_f32_32x32x16: A = K rows from LDS, B = Q^T held in registers for the
//                      whole kernel.  In the 32x32 result a lane owns ONE query column (lane%32)
//                      and 16 of the 32 key rows, so the softmax row reductions are in-lane plus
//                      one exchange between the wave halves (v_permlane32_swap).
//   P^T = exp2(S^T)    online softmax in registers, fp32.  Q is pre-multiplied by c = scale*log2(e) and
//                      the product starts from an accumulator holding -c*m (m = the row's reference
//                      maximum), so the matrix core delivers c*s - c*m and the VALU only has to apply
//                      exp2.  m is a stabiliser, not necessarily the exact running maximum: it is
//                      raised only when a tile's scores exceed it by more than 2^8, which keeps every
//                      p in (0, 256], leaves O/l unchanged, and makes the accumulator rescale rare.
//   O^T += V^T * P^T   A = V^T from LDS, B = P^T straight from the registers S^T was in: the
//                      accumulator layout of the first product is the B-operand layout of the
//                      second once the 16 keys of a k-step are taken in the order
//                      key = 8*(e/4) + 4*(lane/32) + e%4 (e = 0..7).  V stays row-major [key][d] in
//                      LDS; ds_read_b64_tr_b16 (the gfx950 transposing LDS read) hands each lane
//                      4 keys of one d, and two such reads fetch exactly the 8 keys above.
// O^T keeps the query in the lane column, so the per-row rescale factors are per-lane scalars.
//
// Tiles reach LDS without touching registers: buffer_load_dwordx4 ... lds writes 1 KiB per wave
// instruction (lane i -> LDS base + 16*i).  The address is a uniform buffer descriptor (first row of the
// tile, bytes valid from there) plus a per-lane 32-bit offset that never changes, so a tile costs eight
// back-to-back loads and no vector arithmetic, and rows past the end of a sequence are out of range for
// the descriptor and arrive as zeros.  Which global 16-byte chunk a lane fetches is free, so the XOR
// swizzle that makes the later operand reads bank-conflict free is applied on the global side:
// physical chunk = chunk ^ f(row), with f chosen per tile kind (16-byte row reads for K, 8-byte
// transposing reads for V).  LDS is double buffered: tile t+1 streams in while tile t is consumed;
// one barrier per tile.
//
// A wavefront gets ~29 B/clk out of LDS, about what its matrix instructions consume, so operand reads
// are issued ahead of their use: the first product keeps four K operand pairs in flight, and the first
// V operands of the second product are requested before the softmax arithmetic starts.
//
// With `paired` set a workgroup handles query tile (last - i) and then tile i of a head: under a causal
// mask all workgroups then walk the same number of key tiles, which evens out the end of the launch.
#pragma once

#include <cstdlib>

#include "ahpc_device.hpp"

namespace ahpc {

struct FlashParams {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    const int32_t* cu_seqlens;  // ragged batches only
    const float* mask;          // masked kernel only: fp32 [B,N,N], shared by all heads; 0.0f removes the key for the query
    const uint64_t* mask_bits;  // masked kernel on a packed mask: word [(b * mask_kt + key tile) * N + query] holds the 64 keys
                                // of the tile, bit j set = key 64 * tile + j stays (flash_mask_pack_kernel writes it)
    int32_t mask_kt;            // key tiles per row of the packed mask: ceil(N / 64)
    int32_t d_real;             // head dimension of the tensors when it is smaller than the kernel's D (a multiple of 8 for
                                // 16-bit tensors, of 4 for fp32), 0 = D.  The kernel then computes with D columns of which the
                                // last D - d_real contribute nothing: Q's are zero, so whatever K holds there is multiplied
                                // by zero (the tile requests of those columns fetch the row's first chunk again, never
                                // memory behind the row), and V's produce output columns that are not stored.
    int64_t stride_b, stride_n, stride_h;           // Q and O
    int64_t kv_stride_b, kv_stride_n, kv_stride_h;  // K and V
    int32_t N;                  // sequence length (dense) / longest sequence (ragged)
    int32_t H;                  // query heads
    int32_t kv_group;           // query heads per key/value head (1 = every head has its own K/V)
    int32_t n_qtiles;           // query tiles per sequence (of the longest one)
    int32_t paired;             // 1: a workgroup takes two query tiles of a head (see above)
    int32_t total_blocks;       // B * H * n_qtiles, or B * H * ceil(n_qtiles / 2) when paired
    int32_t n_bh;               // B * H: no workgroup may address a (sequence, head) at or beyond this
    int32_t spread_groups;      // ragged batches: 1 = (sequence, head) pairs are dealt to the 8 XCDs in turn (see flash_work_of_block)
    int32_t blocks_per_xcd;     // ceil(total_blocks / 8)
    int32_t n_block_ids;        // 8 * blocks_per_xcd: the block ids of the work map (a persistent kernel walks them with a stride)
    float scale_log2;           // scale * log2(e)
    // Dense launches may keep the softmax statistic of every query row for a later backward: -log2 of the row's sum of
    // exp2(scale_log2 * q.k) over its visible keys (-inf for a row that sees none), at [(b * H + h) * keep_rows + row].
    // Null: nothing is kept.
    float* keep_neg_lse2;
    int64_t keep_rows;          // rows per (sequence, head) of that array: N rounded up to whole 128-row tiles
};

constexpr int kFlashThreads = 256;
constexpr int kFlashRows = 128;  // query rows per workgroup
constexpr int kFlashKeys = 64;   // keys per tile
constexpr int kFlashWideWaves = 8;                    // flash_fwd_wide.hpp: eight wavefronts,
constexpr int kFlashWideRows = 32 * kFlashWideWaves;  // 256 query rows per workgroup

#ifndef AHPC_LDS
#define AHPC_LDS __attribute__((address_space(3)))
#endif

template <typename T> struct TrRead;
template <> struct TrRead<bf16_t> {
    typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 vec;
    __device__ static u32x2 load(const unsigned char* p) {
        return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4bf16((AHPC_LDS vec*)p));
    }
};
template <> struct TrRead<f16_t> {
    typedef __attribute__((__vector_size__(4 * sizeof(__fp16)))) __fp16 vec;
    __device__ static u32x2 load(const unsigned char* p) {
        return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16((AHPC_LDS vec*)p));
    }
};

// ---- LDS reads behind the compiler's back ----------------------------------------------------------------------
// The compiler orders every LDS read it knows of behind ALL direct-to-LDS loads in flight once a function holds more
// than a handful of them (an s_waitcnt vmcnt(0) in front of reads of a tile that landed long ago), which serialises a
// pipeline of tiles.  Kernels with such pipelines issue their LDS reads as asm and complete them with the waits below.
// ds_read_b64_tr_b16 at lds + IMM without the compiler's knowledge; tr_wait() below completes it.
template <typename T, int IMM> __device__ inline u32x2 tr_read_async(const unsigned char* lds) {
#if defined(AHPC_TRACED_LDS_READ_B128)  // the CPU executor: an ordinary (modelled) transposing read
    return TrRead<T>::load(lds + IMM);
#elif defined(__HIP_DEVICE_COMPILE__)
    u32x2 r;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"((uint32_t)(uintptr_t)lds), "n"(IMM) : "memory");
    return r;
#else
    return u32x2{0u, 0u};
#endif
}

// Waits for the LDS reads issued so far; the values pass through it, so nothing that uses them moves above the wait.
template <int N> __device__ inline void tr_wait(u32x2 (&v)[N]) {
#if !defined(AHPC_TRACED_LDS_READ_B128) && defined(__HIP_DEVICE_COMPILE__)
    static_assert(N == 4 || N == 8 || N == 16, "operand sets of d = 64, 128 or 256");
    if constexpr (N == 16) {
        // (an asm statement takes 30 operands at most: the second half passes through an empty one right behind the wait)
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
        asm volatile("" : "+v"(v[8]), "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]), "+v"(v[14]), "+v"(v[15]));
    } else if constexpr (N == 8)
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
    else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]));
#endif
}

// ds_read_b128 at lds + IMM, likewise behind the compiler's back (the CPU executor: the traced read).
template <int IMM> __device__ inline u32x4 lds_read_b128_async(const unsigned char* lds) {
#if defined(AHPC_TRACED_LDS_READ_B128)
    return lds_read_b128(lds + IMM);
#elif defined(__HIP_DEVICE_COMPILE__)
    u32x4 r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"((uint32_t)(uintptr_t)lds), "n"(IMM) : "memory");
    return r;
#else
    return u32x4{0u, 0u, 0u, 0u};
#endif
}
template <int N> __device__ inline void b128_wait(u32x4 (&v)[N]) {
#if !defined(AHPC_TRACED_LDS_READ_B128) && defined(__HIP_DEVICE_COMPILE__)
    static_assert(N == 2 || N == 4 || N == 8 || N == 16, "operand sets of d = 64, 128 or 256");
    if constexpr (N == 16) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
        asm volatile("" : "+v"(v[8]), "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]), "+v"(v[14]), "+v"(v[15]));
    } else if constexpr (N == 8)
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
    else if constexpr (N == 4) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]));
    else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]));
#endif
}

// max / sum of x over the two lanes that share a query column (lane and lane ^ 32).
// v_permlane32_swap(a, b) exchanges the upper 32 lanes of a with the lower 32 lanes of b; with
// a = b = x the two results hold x's lower half and x's upper half in every lane.
__device__ inline float halves_max(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, x), __builtin_bit_cast(unsigned, x), false, false);
    return fmaxf(as_f32(r[0]), as_f32(r[1]));
}
__device__ inline float halves_sum(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, x), __builtin_bit_cast(unsigned, x), false, false);
    return as_f32(r[0]) + as_f32(r[1]);
}

template <int D> struct FlashTile {
    static constexpr int kRowBytes = 2 * D;
    static constexpr int kChunks = D / 8;                 // 16-byte chunks per row
    static constexpr int kRowsPerInstr = 1024 / kRowBytes;  // rows one wave-wide DMA instruction covers
    static constexpr int kInstrPerWave = kFlashKeys / (4 * kRowsPerInstr);
    static constexpr int kBytes = kFlashKeys * kRowBytes;
    // swizzles (XOR on the 16-byte chunk index)
    __device__ static int fk(int row) { return D >= 128 ? (row & 15) : ((row >> 1) & 7); }
    __device__ static int fv(int row) { return D >= 128 ? 4 * (row & 3) : 4 * ((row >> 1) & 1); }
    // for tiles that are read both ways (backward): 16 consecutive rows get 16 different chunks (row reads),
    // and the 4 rows of a transposing read get chunk quads that do not overlap
    __device__ static int fb(int row) {
        const int b0 = row & 1, b1 = (row >> 1) & 1, b2 = (row >> 2) & 1, b3 = (row >> 3) & 1;
        return D >= 128 ? (((b1 ^ b3) << 3) | (b0 << 2) | (b2 << 1) | b1) : (((b1 ^ b0) << 2) | (b2 << 1) | (b3 ^ b0));
    }
};

// Streams one 64-key tile (K or V) from global memory into LDS through a buffer descriptor.
// `base` = first row of the tile, `nrec` = bytes that may be read from there on (anything beyond reads
// as zero), off[i] = this lane's byte offset for its i-th instruction, wave_u = wavefront index (uniform).
// IPW = instructions per wavefront: a tile's instructions are shared out evenly among the workgroup's wavefronts (four
// of them here, eight in flash_fwd_wide.hpp).
template <int D, int IPW = FlashTile<D>::kInstrPerWave>
__device__ inline void dma_tile(const void* base, unsigned nrec, const int* off, unsigned char* lds_tile, int wave_u) {
#if defined(__HIP_DEVICE_COMPILE__)  // the descriptor type exists only in the device pass
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, nrec, 0x00020000);
#pragma unroll
    for (int i = 0; i < IPW; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (AHPC_LDS void*)(lds_tile + (wave_u * IPW + i) * 1024), 16,
                                                 off[i], 0, 0, 0);
#endif
}

// One direct-to-LDS load instruction on its own: lane i's 16 bytes at base + off (bytes; anything not inside
// [0, nrec) reads as zero) land at lds + 16*i.  AUX = the instruction's cache policy bits (2: non-temporal).
template <int AUX = 0> __device__ inline void dma_instr(const void* base, unsigned nrec, int off, unsigned char* lds) {
#if defined(__HIP_DEVICE_COMPILE__)  // the descriptor type exists only in the device pass
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, nrec, 0x00020000);
#if defined(AHPC_TRACED_LDS_READ_B128)  // the CPU executor: LDS is host memory
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (AHPC_LDS void*)lds, 16, off, 0, 0, AUX);
#else
    // (the LDS address is the low half of the generic one; taking it as a number spares the scalar unit the
    // null test that the pointer conversion carries)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (AHPC_LDS void*)(uintptr_t)(uint32_t)(uintptr_t)lds, 16, off, 0, 0, AUX);
#endif
#endif
}

// The 4-byte form of the same instruction: lane i's dword lands at lds + 4*i.
__device__ inline void dma_dword(const void* base, unsigned nrec, int off, unsigned char* lds) {
#if defined(__HIP_DEVICE_COMPILE__)
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, nrec, 0x00020000);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (AHPC_LDS void*)lds, 4, off, 0, 0, 0);
#endif
}

// Workgroup id -> work.  Hardware deals consecutive workgroup ids to the 8 XCDs in turn; `logical` undoes
// that, so that consecutive logical ids run on the same XCD and share its L2.  A head owns `per_head`
// consecutive logical ids (its query tiles, or pairs of them), late (long) tiles first.
// Ragged batches (spread_groups): sequences differ in length, so equal shares of the id range are not equal shares of
// the work.  There the (sequence, head) pairs are dealt to the XCDs in turn - pair g runs on XCD g % 8, its tiles
// still side by side on that XCD - every pair owns as many slots as the LONGEST sequence needs, and a workgroup
// whose slot lies beyond its own sequence's tiles (counted and paired from that sequence's own length) exits at once.
// Host and device evaluate the same code: a host-side dump of this function is what the tests check.
struct FlashWork {
    int bh;     // sequence * H + head
    int slot;   // 0 .. per_head-1
    bool valid;
};
__host__ __device__ inline int flash_per_head(const FlashParams& p) { return p.paired ? (p.n_qtiles + 1) >> 1 : p.n_qtiles; }
__host__ __device__ inline FlashWork flash_work_of_block(unsigned block_id, const FlashParams& p) {
    const int xcd = (int)(block_id & 7u);
    const int per_head = flash_per_head(p);
    if (p.spread_groups) {
        const int k = (int)(block_id >> 3);
        const int round = k / per_head;
        const int g = round * 8 + xcd;
        if (g >= p.n_bh) return FlashWork{0, 0, false};
        return FlashWork{g, k - round * per_head, true};
    }
    const int logical = xcd * p.blocks_per_xcd + (int)(block_id >> 3);
    if (logical >= p.total_blocks) return FlashWork{0, 0, false};
    const int bh = logical / per_head;
    return FlashWork{bh, logical - bh * per_head, true};
}
// Query tile a workgroup handles in its first (part 0) and second (part 1) pass; -1 = none.
// n_qtiles: query tiles of the sequence in hand (p.n_qtiles for dense batches, the sequence's own count in a ragged one).
__host__ __device__ inline int flash_qtile_of_part(const FlashParams& p, int n_qtiles, int slot, int part) {
    if (p.paired) {
        if (part == 1 && 2 * slot == n_qtiles - 1) return -1;  // odd count: the middle tile has no partner
        return part == 0 ? n_qtiles - 1 - slot : slot;
    }
    return part == 0 ? n_qtiles - 1 - slot : -1;
}

// What the statistics variant of the kernel writes instead of O (first step of the backward):
// per (sequence, head, query row)  lse2 = log2 sum_j exp2(c q.k_j)  (c = scale*log2(e), the units the kernel
// works in) and delta = dO . O, both NEGATED: the backward kernels start their accumulators from -lse2 and -delta.
// Rows are laid out [B*H][rows_padded], rows_padded a multiple of the 128-row query tile; rows beyond the sequence
// receive -lse2 = -inf (every weight exp2(s - inf) is 0 later on) and -delta = 0, so that whole tiles of statistics
// can be read without a bounds check.
struct FlashStatsOut {
    const void* d_out;     // dO, laid out like Q and O
    float* neg_lse2;
    float* neg_delta;
    int64_t rows_padded;
};

// MASK != 0: a dense fp32 mask [B,N,N] removes keys per query (0.0f = removed; FlashAttention::apply_attention_mask,
// src/algorithms/flash_attention.cpp:596-607).  Any query may then see its first key in any tile, or none at all
// (zeros come out), so the reference maximum is set per query when its first key shows up.
//   MASK == 1: the kernel reads the caller's mask.  A lane's 32 scores of a tile are 8 runs of 4 consecutive keys of
//              its query: 8 16-byte loads of the mask row (N is a multiple of 4 then, the host checks).  Every head
//              reads the whole mask again: as many bytes through L2 as K and V together.
//   MASK == 2: the kernel reads one 64-bit word per query and tile of a packed copy (flash_mask_pack_kernel made it
//              in front of this launch): a sixteenth of the bytes, one load instead of eight, two registers
//              instead of 32.
template <typename T, int D, bool CAUSAL, bool VARLEN, bool STATS, int MASK = 0>
__device__ __forceinline__ void flash_fwd_mfma_body(const FlashParams& p, const FlashStatsOut& st) {
    constexpr bool MASKED = MASK != 0;
    static_assert(!(MASKED && VARLEN), "the mask belongs to dense launches");
    static_assert(!(STATS && MASK == 1), "the statistics pass reads the packed mask only");
    typedef FlashTile<D> TL;
    constexpr int KS = D / 16;  // k-steps of the first product
    constexpr int MB = D / 32;  // 32-row blocks of O^T
    constexpr int RB = TL::kRowBytes;

    // two buffers, each its own array: the compiler can then tell a DMA into one from reads of the other
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[TL::kBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[TL::kBytes];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 31;   // query column / operand row owned by this lane
    const int half = lane >> 5;

    const FlashWork work = flash_work_of_block(blockIdx.x, p);
    if (!work.valid) return;
    // whatever the map says, nothing outside the tensors is ever addressed (uniform per workgroup)
    if (work.bh < 0 || work.bh >= p.n_bh || work.slot < 0 || work.slot >= flash_per_head(p)) return;
    // A wavefront raises its issue priority while it feeds the matrix cores and lowers it for the stretch of pure
    // softmax arithmetic: of the two wavefronts that share a SIMD the one with matrix instructions ready goes first
    // (worth about 2% on the headline shape).
    auto set_priority = [&](bool busy) {
        if (busy) __builtin_amdgcn_s_setprio(1); else __builtin_amdgcn_s_setprio(0);
    };
    const int bh = work.bh;
    const int slot = work.slot;
    const int b = bh / p.H;
    const int h = bh - b * p.H;

    int L;
    int64_t base, kv_base;
    const int hk = h / p.kv_group;  // grouped-query attention: consecutive query heads share a K/V head
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
    // query tiles of this sequence, and the slots they fill (a ragged batch hands every sequence as many slots as
    // the longest one needs: the surplus exits here, before anything is requested)
    const int n_q = VARLEN ? (L + kFlashRows - 1) / kFlashRows : p.n_qtiles;
    if (VARLEN && slot >= (p.paired ? (n_q + 1) >> 1 : n_q)) return;
    const T* const gq = static_cast<const T*>(p.q) + base;
    const T* const gk = static_cast<const T*>(p.k) + kv_base;
    const T* const gv = static_cast<const T*>(p.v) + kv_base;
    T* const go = STATS ? nullptr : static_cast<T*>(p.o) + base;  // the statistics pass has no output tensor
    const int64_t sn = p.stride_n;
    const int64_t skv = p.kv_stride_n;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int d_real = (p.d_real > 0 && p.d_real < D) ? p.d_real : D;

    // ---- per-lane DMA offsets (bytes from the first row of a tile), fixed for the whole kernel ------
    int dma_off_k[TL::kInstrPerWave], dma_off_v[TL::kInstrPerWave];
#pragma unroll
    for (int i = 0; i < TL::kInstrPerWave; ++i) {
        const int r = (wave * TL::kInstrPerWave + i) * TL::kRowsPerInstr + lane / TL::kChunks;
        const int pc = lane % TL::kChunks;
        const int ck = pc ^ TL::fk(r), cv = pc ^ TL::fv(r);  // the 8-element chunk of the row that belongs at this lane's place
        dma_off_k[i] = (int)(r * skv * 2) + ((8 * ck < d_real ? ck : 0) << 4);
        dma_off_v[i] = (int)(r * skv * 2) + ((8 * cv < d_real ? cv : 0) << 4);
    }
    // Keys k0.. of this head into a buffer pair.  Bytes from the tile's first row to the end of the
    // sequence's last row bound the descriptor, so the rows of a ragged last tile that do not exist
    // read as zeros (their scores are masked; zero V rows keep 0 * x finite).
    auto dma_both = [&](int k0, unsigned char* dst_k, unsigned char* dst_v) {
        // (a tile that starts at or behind the end of the sequence touches no memory and lands as zeros)
        const int64_t rem = k0 < L ? (int64_t)(L - k0 - 1) * skv * 2 + 2 * d_real : 0;  // the last row ends with its own d
        const unsigned nrec = rem > 0xffffffffll ? 0xffffffffu : (unsigned)rem;
        dma_tile<D>(gk + (int64_t)k0 * skv, nrec, dma_off_k, dst_k, wave_u);
        dma_tile<D>(gv + (int64_t)k0 * skv, nrec, dma_off_v, dst_v, wave_u);
    };
    // The tiles behind the first are requested one per step, in order: their addresses and the bytes that remain behind
    // them advance by a tile per request instead of being worked out from the tile number (64-bit products) every step.
    const int64_t tile_elems = (int64_t)kFlashKeys * skv;
    const T* k_next = nullptr;
    const T* v_next = nullptr;
    int64_t rem_next = 0;
    auto dma_next = [&](unsigned char* dst_k, unsigned char* dst_v) {
        const unsigned nrec = rem_next <= 0 ? 0u : rem_next > 0xffffffffll ? 0xffffffffu : (unsigned)rem_next;
        dma_tile<D>(k_next, nrec, dma_off_k, dst_k, wave_u);
        dma_tile<D>(v_next, nrec, dma_off_v, dst_v, wave_u);
        k_next += tile_elems;
        v_next += tile_elems;
        rem_next -= 2 * tile_elems;
    };

    // ---- LDS operand addresses (byte offsets inside a tile) -------------------------------------
    // K: lane reads row (32*kb + col), logical chunk 2*ks + half
    int k_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_off[ks] = col * RB + (((2 * ks + half) ^ TL::fk(col)) << 4);
    // V (transposing read): source lane i = lane%16 points at key (4*half + i/4) of the 16g+8a group,
    // d-quad 32*mb + 16*((lane/16)%2) + 4*(i%4)
    const int vi = lane & 15;
    const int vkey = 4 * half + (vi >> 2);
    int v_off[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int cch = 4 * mb + 2 * ((lane >> 4) & 1) + ((vi & 3) >> 1);
        v_off[mb] = vkey * RB + ((cch ^ TL::fv(vkey)) << 4) + 8 * (vi & 1);
    }

    for (int part = 0; part < 2; ++part) {
        const int qt = flash_qtile_of_part(p, n_q, slot, part);
        if (qt < 0) break;
        const int q_tile0 = qt * kFlashRows;
        if (q_tile0 >= L) continue;

        int k_end = L;
        if (CAUSAL) k_end = (q_tile0 + kFlashRows) < L ? (q_tile0 + kFlashRows) : L;
        const int n_tiles = (k_end + kFlashKeys - 1) / kFlashKeys;

        // first tile on its way before anything else
        dma_both(0, lds_k0, lds_v0);
        k_next = gk + tile_elems;
        v_next = gv + tile_elems;
        rem_next = (int64_t)(L - kFlashKeys - 1) * skv * 2 + 2 * d_real;

        // ---- Q^T operands, pre-multiplied by c = scale*log2(e), kept for the whole query tile --------
        const int qw = q_tile0 + wave * 32;  // first query row of this wavefront
        const int qrow = qw + col;
        u32x4 qreg[KS];
        {
            const int row = qrow < L ? qrow : L - 1;
            const T* src = gq + (int64_t)row * sn + 8 * half;
            const float c = p.scale_log2;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const u32x4 raw = 16 * ks + 8 * half < d_real ? *reinterpret_cast<const u32x4*>(src + 16 * ks) : u32x4{0u, 0u, 0u, 0u};
                u32x4 sc;
#pragma unroll
                for (int w = 0; w < 4; ++w) sc[w] = pack2<T>(lo_f32<T>(raw[w]) * c, hi_f32<T>(raw[w]) * c);
                qreg[ks] = sc;
            }
        }

        // ---- running state ------------------------------------------------------------------------
        // All score arithmetic is in log2 units (c is folded into Q).  `neg_m` = -(reference maximum) of
        // the lane's query row, as a 16-wide vector because it is the C operand of the first k-step.
        f32x16 oacc[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[mb][r] = 0.0f;
        f32x16 neg_m;
#pragma unroll
        for (int r = 0; r < 16; ++r) neg_m[r] = 0.0f;
        float l_run = 0.0f;
        bool first = true;
        bool seen = false;  // masked launches: this lane's query has met a key it may attend to
        constexpr float kRaise = 8.0f;  // raise the reference maximum only when exceeded by 2^8
        const float* const mrow = MASK == 1 ? p.mask + ((int64_t)b * p.N + (qrow < L ? qrow : L - 1)) * p.N : nullptr;
        const uint64_t* const mword = MASK == 2 ? p.mask_bits + (int64_t)b * p.mask_kt * p.N + (qrow < L ? qrow : L - 1) : nullptr;

        // The mask values of this lane's 32 scores of the tile at k0.  A run that starts behind the row's end reads
        // the row's last four values instead: its keys do not exist and are removed by the end-of-sequence test.
        auto load_mask = [&](f32x4 (&mk)[2][4], int k0) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const int key = k0 + 32 * kb + 8 * g4 + 4 * half;
                    mk[kb][g4] = *reinterpret_cast<const f32x4*>(mrow + (key < p.N - 4 ? key : p.N - 4));
                }
        };

        auto compute_tile = [&](const unsigned char* tile_k, const unsigned char* tile_v, int k0, const f32x4 (&mk)[2][4],
                                uint64_t mw) {
            // ---- S^T = c*K Q^T - m  (log2 units).  The two 32-key blocks alternate, kAhead operand
            //      pairs are requested before the first product and one more after every two products.
            f32x16 s[2];
            set_priority(true);
            {
                u32x4 a0[KS], a1[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    a0[ks] = lds_read_b128(tile_k + k_off[ks]);
                    a1[ks] = lds_read_b128(tile_k + 32 * RB + k_off[ks]);
                }
                s[0] = mfma_32x32x16<T>(a0[0], qreg[0], neg_m);
                s[1] = mfma_32x32x16<T>(a1[0], qreg[0], neg_m);
#pragma unroll
                for (int ks = 1; ks < KS; ++ks) {
                    s[0] = mfma_32x32x16<T>(a0[ks], qreg[ks], s[0]);
                    s[1] = mfma_32x32x16<T>(a1[ks], qreg[ks], s[1]);
                }
                constexpr int kAhead = KS < 4 ? KS : 4;
                __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);  // LDS reads
#pragma unroll
                for (int i = 0; i < KS - kAhead; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // matrix instructions
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                }
#pragma unroll
                for (int i = 0; i < kAhead; ++i) __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            }
            // V operands of the first 16 keys: requested now, used after the softmax arithmetic
            u32x2 vf[4][MB][2];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                vf[0][mb][0] = TrRead<T>::load(tile_v + v_off[mb]);
                vf[0][mb][1] = TrRead<T>::load(tile_v + v_off[mb] + 8 * RB);
            }

            set_priority(false);
            const bool need_mask = (k0 + kFlashKeys > L) || (CAUSAL && (k0 + kFlashKeys - 1 > qw));
            if (need_mask) {
                // key = k0 + 4*half + off(kb, r); visible iff key <= min(qrow, L-1)  <=>  off <= lim
                int lim = L - 1;
                if (CAUSAL) lim = qrow < lim ? qrow : lim;
                lim -= k0 + 4 * half;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int off = 32 * kb + 8 * (r >> 2) + (r & 3);
                        s[kb][r] = off <= lim ? s[kb][r] : -INFINITY;
                    }
            }
            if constexpr (MASK == 1) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) s[kb][r] = mk[kb][r >> 2][r & 3] == 0.0f ? -INFINITY : s[kb][r];
            }
            if constexpr (MASK == 2) {
                // the lane's keys of the tile are 4 * half + 32 * kb + 8 * (r / 4) + r % 4: one shift brings them to
                // fixed places of two 32-bit words; a bit spread over a word (all ones: keep) selects between the
                // score and -inf
                const uint64_t w = mw >> (4 * half);
                const uint32_t word[2] = {(uint32_t)w, (uint32_t)(w >> 32)};
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int pos = 8 * (r >> 2) + (r & 3);
                        const uint32_t keep = (uint32_t)((int32_t)(word[kb] << (31 - pos)) >> 31);
                        s[kb][r] = as_f32((as_u32(s[kb][r]) & keep) | (0xFF800000u & ~keep));
                    }
            }
            // ---- reference maximum: exact on the first tile, afterwards raised only when a score tops
            //      it by more than kRaise (rare, and the only time the accumulators are rescaled) ------
            float mx = fmaxf(s[0][0], s[1][0]);
#pragma unroll
            for (int r = 1; r < 16; ++r) mx = max3(mx, s[0][r], s[1][r]);
            bool adjust;
            if constexpr (MASKED) adjust = __builtin_amdgcn_ballot_w64(seen ? mx > kRaise : mx > -INFINITY) != 0;
            else adjust = first || __builtin_amdgcn_ballot_w64(mx > kRaise) != 0;
            if (adjust) {
                mx = halves_max(mx);                       // both lanes of a query agree
                float delta, alpha;
                if constexpr (MASKED) {
                    // a query without a visible key so far has accumulated nothing: its maximum is set exactly,
                    // nothing is rescaled; one that still sees none stays as it is
                    delta = seen ? fmaxf(mx, 0.0f) : (mx > -INFINITY ? mx : 0.0f);
                    alpha = seen ? fast_exp2(-delta) : 1.0f;
                    seen = seen || mx > -INFINITY;
                } else {
                    delta = first ? mx : fmaxf(mx, 0.0f);
                    alpha = fast_exp2(-delta);
                }
                l_run *= alpha;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[mb][r] *= alpha;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) s[kb][r] -= delta;
                const float nm = neg_m[0] - delta;
#pragma unroll
                for (int r = 0; r < 16; ++r) neg_m[r] = nm;
                first = false;
            }

            // ---- P^T = exp2(S^T) packed as B operands (row sums in fp32), and O^T += V^T P^T, 16 keys
            //      at a time: while the matrix core works on group g the VALU prepares group g+1 and LDS
            //      delivers its V operands.  The scheduling fences keep the groups apart.
            u32x4 pb[4];
            float sum = 0.0f;
            auto make_pb = [&](int g) {
                const int kb = g >> 1, r0 = 8 * (g & 1);
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const float p0 = fast_exp2(s[kb][r0 + 2 * w]), p1 = fast_exp2(s[kb][r0 + 2 * w + 1]);
                    pb[g][w] = pack2<T>(p0, p1);
                    sum += p0 + p1;  // plain adds co-issue with the matrix pipe; v_dot2 does not
                }
#if defined(__HIP_DEVICE_COMPILE__)
                // the additions stay with their group of keys (left alone, the compiler sinks all of them behind the last
                // matrix instruction, where nothing overlaps them)
                asm volatile("" : "+v"(sum));
#endif
            };
            make_pb(0);
            set_priority(true);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    oacc[mb] = mfma_32x32x16<T>(u32x4{vf[g][mb][0][0], vf[g][mb][0][1], vf[g][mb][1][0], vf[g][mb][1][1]},
                                                pb[g], oacc[mb]);
                if (g < 3) {
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        vf[g + 1][mb][0] = TrRead<T>::load(tile_v + v_off[mb] + (16 * (g + 1)) * RB);
                        vf[g + 1][mb][1] = TrRead<T>::load(tile_v + v_off[mb] + (16 * (g + 1) + 8) * RB);
                    }
                    make_pb(g + 1);
                    // the order of issue: behind every matrix instruction two operand reads for the next 16 keys and a
                    // share of their exponentials (left to itself the compiler bunches the matrix instructions)
                    constexpr int kValuPerMfma = D >= 256 ? 2 : D == 128 ? 4 : 8;
#pragma unroll
                    for (int i = 0; i < MB; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);             // matrix instruction
                        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);             // LDS reads
                        __builtin_amdgcn_sched_group_barrier(0x402, kValuPerMfma, 0);  // vector arithmetic, exponentials included
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            set_priority(false);
            l_run += sum;
        };

        auto step = [&](unsigned char* cur_k, unsigned char* cur_v, unsigned char* nxt_k, unsigned char* nxt_v, int t) {
            const int k0 = t * kFlashKeys;
            const bool more = t + 1 < n_tiles;
            f32x4 mk[2][4];
            uint64_t mw = 0;
            if constexpr (MASKED) {
                // The mask is requested BEFORE the next tile (loads complete in order: waiting for a load issued
                // behind the tile's would wait for the tile), and the tile is requested even behind the last one
                // (an empty request), so that the compiler counts the same loads in flight on every path.
                if constexpr (MASK == 1) load_mask(mk, k0);
                else mw = mword[(int64_t)t * p.N];
                __builtin_amdgcn_sched_barrier(0);
                dma_next(nxt_k, nxt_v);
            } else {
                if (more) dma_next(nxt_k, nxt_v);
            }
            // a wavefront whose queries all precede this tile has nothing to add
            if (!(CAUSAL && k0 > qw + 31)) compute_tile(cur_k, cur_v, k0, mk, mw);
            if (MASKED || more) {
                __builtin_amdgcn_s_waitcnt(0);  // this wave's part of the next tile has landed
                __syncthreads();                // everyone's has, and everyone is done with the current one
            }
        };

        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        for (int t = 0; t < n_tiles; t += 2) {
            step(lds_k0, lds_v0, lds_k1, lds_v1, t);
            if (t + 1 < n_tiles) step(lds_k1, lds_v1, lds_k0, lds_v0, t + 1);
        }

        // ---- normalise and store: lane holds, per 32-row block, 4 runs of 4 consecutive lanes of d ---
        const float l = halves_sum(l_run);
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        if constexpr (STATS) {
            // delta = dO . O over the elements this lane holds, then over the two lanes of the query
            float part = 0.0f;
            if (qrow < L) {
                const T* src = static_cast<const T*>(st.d_out) + base + (int64_t)qrow * sn + 4 * half;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        if (32 * mb + 8 * g4 + 4 * half >= d_real) continue;  // columns the tensors do not have
                        const u32x2 w = *reinterpret_cast<const u32x2*>(src + 32 * mb + 8 * g4);
                        const f32x16& a = oacc[mb];
                        part += a[4 * g4 + 0] * lo_f32<T>(w[0]) + a[4 * g4 + 1] * hi_f32<T>(w[0]) +
                                a[4 * g4 + 2] * lo_f32<T>(w[1]) + a[4 * g4 + 3] * hi_f32<T>(w[1]);
                    }
            }
            const float delta = halves_sum(part) * inv;
            if (half == 0 && qrow < q_tile0 + kFlashRows) {
                const int64_t row = (int64_t)bh * st.rows_padded + qrow;
                const bool live = qrow < L && l > 0.0f;
                st.neg_lse2[row] = live ? neg_m[0] - __builtin_log2f(l) : -INFINITY;
                st.neg_delta[row] = live ? -delta : 0.0f;
            }
        } else if (qrow < L) {
            T* dst = go + (int64_t)qrow * sn + 4 * half;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const f32x16& a = oacc[mb];
                    const u32x2 w = u32x2{pack2<T>(a[4 * g4 + 0] * inv, a[4 * g4 + 1] * inv),
                                          pack2<T>(a[4 * g4 + 2] * inv, a[4 * g4 + 3] * inv)};
                    if (32 * mb + 8 * g4 + 4 * half < d_real) *reinterpret_cast<u32x2*>(dst + 32 * mb + 8 * g4) = w;
                }
            if constexpr (!VARLEN) {
                if (p.keep_neg_lse2 != nullptr && half == 0)
                    p.keep_neg_lse2[(int64_t)bh * p.keep_rows + qrow] = l > 0.0f ? neg_m[0] - __builtin_log2f(l) : -INFINITY;
            }
        }
        __syncthreads();  // the next query tile's first DMA reuses the buffers
    }
}

// Fills the launch geometry of the MFMA kernel (query tiles, pairing, workgroup count) from N, H and the batch size already in `p`.  Shared by the launcher and by the host-side dump
// of the workgroup map.
inline int flash_plan_launch(FlashParams& p, int64_t B, bool causal, int rows_per_workgroup = kFlashRows, int64_t pair_min_tiles = 1024,
                             bool ragged = false) {
    p.n_qtiles = (p.N + rows_per_workgroup - 1) / rows_per_workgroup;
    int64_t total = B * p.H * (int64_t)p.n_qtiles;
    if (total > 0x7FFFFFF0ll) return AHPC_ERR_BAD_SHAPE;
    // Causal launches with enough workgroups to fill the chip twice over pair a late query tile with an
    // early one, so that every workgroup walks the same number of key tiles
    // (1024 tiles = two rounds of two workgroups on each of 256 CUs).
    p.paired = (causal && p.n_qtiles >= 2 && total * rows_per_workgroup >= pair_min_tiles * kFlashRows) ? 1 : 0;
    if (p.paired) total = B * p.H * (int64_t)((p.n_qtiles + 1) / 2);
    p.total_blocks = (int32_t)total;
    p.n_bh = (int32_t)(B * p.H);
    p.blocks_per_xcd = (int32_t)((total + 7) / 8);
    p.spread_groups = ragged ? 1 : 0;
    if (ragged) {
        const int64_t per_xcd = ((B * p.H + 7) / 8) * (p.paired ? (p.n_qtiles + 1) / 2 : p.n_qtiles);
        if (per_xcd * 8 > 0x7FFFFFF0ll) return AHPC_ERR_BAD_SHAPE;
        p.blocks_per_xcd = (int32_t)per_xcd;
    }
    p.n_block_ids = p.blocks_per_xcd * 8;
    return AHPC_OK;
}

template <typename T, int D, bool CAUSAL, bool VARLEN>
__global__ __launch_bounds__(kFlashThreads, D == 256 ? 1 : 2) void flash_fwd_mfma_kernel(const FlashParams p) {
    flash_fwd_mfma_body<T, D, CAUSAL, VARLEN, false>(p, FlashStatsOut{});
}

// Dense launches with a mask [B,N,N]: MASK 1 reads the caller's fp32 mask, MASK 2 its packed copy.
template <typename T, int D, bool CAUSAL, int MASK>
__global__ __launch_bounds__(kFlashThreads, D == 256 ? 1 : 2) void flash_fwd_mfma_masked_kernel(const FlashParams p) {
    flash_fwd_mfma_body<T, D, CAUSAL, false, false, MASK>(p, FlashStatsOut{});
}

// The forward pass with its output kept in registers: writes the softmax statistics the backward needs.
template <typename T, int D, bool CAUSAL, bool VARLEN>
__global__ __launch_bounds__(kFlashThreads, D == 256 ? 1 : 2) void flash_bwd_stats_mfma_kernel(const FlashParams p, const FlashStatsOut st) {
    flash_fwd_mfma_body<T, D, CAUSAL, VARLEN, true>(p, st);
}
// The same under a dense mask (its packed copy).  A query that sees no key gets -lse2 = -inf and -delta = 0, like a row
// beyond the sequence: every weight of it is exp2(s - inf) = 0 in the backward kernels.
template <typename T, int D, bool CAUSAL>
__global__ __launch_bounds__(kFlashThreads, D == 256 ? 1 : 2) void flash_bwd_stats_masked_mfma_kernel(const FlashParams p, const FlashStatsOut st) {
    flash_fwd_mfma_body<T, D, CAUSAL, false, true, 2>(p, st);
}

}  // namespace ahpc
