// Process-wide tuning values of the launchers.  Each starts from an environment variable that is read once,
// when the first launcher asks; ahpc_hip_set_tuning changes it afterwards (tests use that to reach code paths
// that ordinary problem sizes would need a large GPU job for).  None of them changes results.
#pragma once

#include <atomic>
#include <cstdint>

namespace ahpc {

struct Tuning {
    // forward, causal: a workgroup takes a late query tile and then an early one once the launch has at least
    // this many query tiles (AHPC_FLASH_PAIR_MIN, default 1024: two rounds of two workgroups on each of 256 CUs)
    std::atomic<int64_t> flash_pair_min_tiles;
    // decode: wavefronts per workgroup, 1..8 (AHPC_DECODE_WAVES, default 0 = the launcher's choice)
    std::atomic<int64_t> decode_waves;
    // decode: tokens per context chunk when the caller passes none (AHPC_DECODE_CHUNK, default 0 = by shape)
    std::atomic<int64_t> decode_chunk;
    // decode: query heads per K/V head from which on the matrix-core kernels are taken where they apply (16-bit pool,
    // d 64/128, pages of 16).  Default 2: timed on 8 pool heads, the page-by-page matrix-core kernel reaches 0.65-0.72
    // of 8 TB/s for groups of 2, 4 and 8 where the lane-per-element kernel reaches 0.58, 0.55 and 0.36; with one
    // query head per pool head the lane-per-element kernel stays ahead by 1-2 %.  Groups of 9 to 32 exist on the
    // matrix-core kernels only.  (AHPC_DECODE_MFMA_MIN_GROUP)
    std::atomic<int64_t> decode_matrix_min_group;
    // backward: dK and dV in one walk over the query tiles (1), in two (2), or the launcher's choice (0, the default:
    // one walk up to d = 128, two at d = 256).  (AHPC_BWD_SPLIT)
    std::atomic<int64_t> bwd_split;
    // forward with a dense mask on the matrix-core kernel: 1 (default) = the mask is packed to one bit per element in
    // front of the launch, into device memory the library keeps; 0 = the kernel reads the caller's fp32 mask in place
    // (what a stream under graph capture gets in any case).  (AHPC_MASK_PACK)
    std::atomic<int64_t> mask_pack;
    // backward, causal dense launches: 1 (default) = the dQ and dK/dV workgroups take a long and a short tile of their
    // head each (equal work for all), 0 = one tile per workgroup, long tiles first.  (AHPC_BWD_PAIR)
    std::atomic<int64_t> bwd_pair;
    // forward on the 16-bit matrix-core kernel: query rows per workgroup, 128 (4 wavefronts, two workgroups per CU) or
    // 256 (8 wavefronts, one workgroup per CU: one stream of K/V tiles feeds twice the rows); 0 (default) = by shape.
    // (AHPC_FLASH_ROWS)
    std::atomic<int64_t> flash_rows;
    // KV block pool (host class): 1 (default) = slabs are address ranges that grow in place where the device has virtual
    // memory management; 0 = plain allocations that grow by reallocation and a device copy.  Read when a pool is
    // created.  (AHPC_POOL_IN_PLACE)
    std::atomic<int64_t> pool_in_place;
    Tuning();
};

Tuning& tuning();

}  // namespace ahpc
