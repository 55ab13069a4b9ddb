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
    // decode: query heads per K/V head from which on the matrix-core kernel is taken where it applies (16-bit pool,
    // d 64/128, pages of 16).  Default 16: timed side by side, the lane-per-element kernel is the faster one for
    // groups of 4 and 8 (0.143 ms against 0.147 ms on 32 query heads over 8 pool heads); 16 and 32 exist on the
    // matrix-core kernel only.  (AHPC_DECODE_MFMA_MIN_GROUP)
    std::atomic<int64_t> decode_matrix_min_group;
    Tuning();
};

Tuning& tuning();

}  // namespace ahpc
