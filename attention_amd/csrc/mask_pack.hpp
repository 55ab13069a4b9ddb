// The packed copy of a dense attention mask, shared by the forward and the backward launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <functional>

namespace ahpc {

// One bit per (query, key) of a dense mask [B,N,N], in device memory that the library owns:
//   bits   [(b * tiles + key tile) * N + query]    the tile's 64 keys of one query   (bit j = key 64 * tile + j stays)
//   bits_t [(b * tiles + query block) * N + key]   the block's 64 queries of one key (bit r = query 64 * block + r sees the key);
//          null unless asked for
struct PackedMask {
    const uint64_t* bits;
    const uint64_t* bits_t;
    int32_t tiles;  // ceil(N / 64)
};

// Packs `mask` on `stream` (with_transposed: both layouts) and runs launch_on_bits on the packed copy; everything
// launch_on_bits puts on `stream` may read it.  AHPC_OK with *launched = false: not possible here (stream under capture,
// no memory, mask too large) - nothing was launched and the caller takes another path.
int with_packed_mask(const float* mask, int64_t B, int64_t N, bool with_transposed, hipStream_t stream, bool* launched,
                     const std::function<int(const PackedMask&)>& launch_on_bits);

}  // namespace ahpc
