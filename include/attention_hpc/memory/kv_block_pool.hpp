// Device-resident KV block pool: one HBM slab for K and one for V, laid out
// [page][slot][head][head_dim], plus the host-side free list that hands out page ids.
//
// It takes the place of the reference's PagePool / KVPage (src/algorithms/paged_attention.hpp:19-84,
// src/algorithms/paged_attention.cpp:11-64) and keeps its allocation order exactly, because page ids
// end up in the block table and so in every gather index: pages are numbered in creation order,
// allocate() pops the FRONT of the free queue, an empty queue first grows by `growth` pages, and
// deallocate() pushes to the BACK.  What is new is where the bytes live: each slab is a range of device
// addresses reserved once for the whole budget (sized against the GPU's HBM, 288 GB on MI355X) and backed
// by physical memory only as far as pages exist; growth maps more memory behind it, in place: slab pointers
// never move, nothing is copied, no stream waits.  (On a device without virtual memory management the slabs
// are plain allocations that grow by doubling and a device-to-device copy.)  The host never touches them.  Counters follow the reference's MemoryStats idea
// (src/memory/memory_pool.hpp:29-53): bytes in use, peak, capacity.
#pragma once

#include <cstddef>
#include <cstdint>
#include <deque>
#include <mutex>
#include <utility>
#include <vector>

#include "api/attention_interface.hpp"

namespace attention_hpc {

class MemoryPoolException : public AttentionException {
public:
    explicit MemoryPoolException(const std::string& message)
        : AttentionException(AttentionError::MEMORY_ALLOCATION_FAILED, message) {}
};

struct KVBlockPoolStats {
    size_t total_pages = 0;        // pages created so far (free + allocated)
    size_t free_pages = 0;
    size_t allocated_pages = 0;
    size_t peak_allocated_pages = 0;
    size_t page_bytes = 0;         // K + V bytes of one page
    size_t slab_capacity_pages = 0;
    size_t slab_bytes = 0;         // device bytes currently reserved (K + V)
};

class KVBlockPool {
public:
    // page_tokens x heads x head_dim elements of `dtype` per page and per slab.  `initial_pages`
    // pages exist at once; `growth` more are created whenever the free queue runs dry (0 = fixed).
    // `max_bytes` caps the device reservation (0 = 90% of the free HBM at construction).
    KVBlockPool(size_t page_tokens, size_t heads, size_t head_dim, DataType dtype, size_t initial_pages = 64,
                size_t growth = 16, size_t max_bytes = 0);
    ~KVBlockPool();
    KVBlockPool(const KVBlockPool&) = delete;
    KVBlockPool& operator=(const KVBlockPool&) = delete;

    int32_t allocate_page();             // throws MemoryPoolException when HBM is exhausted
    void deallocate_page(int32_t page);  // unknown / already-free ids are ignored, as in the reference
    // Grows the pool to `new_total_pages`, or shrinks it: pages at the end of the id range that are free are dropped
    // (never below the highest page in use; the device is synchronised first and, where slabs grow in place, the
    // memory of chunks that no longer hold a page goes back to the device).
    void resize_pool(size_t new_total_pages);
    // Compaction in two steps, for the owner of the block tables.  plan_compaction() lists the moves (from, to) that
    // bring every page in use below allocated_pages(): pages in use at or beyond that mark, highest first, onto the
    // free ids below it, lowest first.  After the device copy, apply_compaction(moves) swaps the ids' roles and
    // rebuilds the free queue in ascending id order.
    std::vector<std::pair<int32_t, int32_t>> plan_compaction() const;
    void apply_compaction(const std::vector<std::pair<int32_t, int32_t>>& moves);

    size_t get_pool_size() const;
    size_t get_free_pages() const;
    size_t get_allocated_pages() const;
    KVBlockPoolStats stats() const;

    void* k_slab() const { return k_slab_; }
    void* v_slab() const { return v_slab_; }
    DataType dtype() const { return dtype_; }
    size_t page_tokens() const { return page_tokens_; }
    // Bumped whenever the slabs move: holders of raw slab pointers must re-read them.  Slabs that grow in place
    // (grows_in_place()) never move: the generation then stays 0.
    uint64_t generation() const { return generation_; }
    bool grows_in_place() const { return in_place_; }

private:
    void create_pages_locked(size_t count);
    void reserve_locked(size_t pages);

    const size_t page_tokens_, heads_, head_dim_;
    const DataType dtype_;
    const size_t growth_;
    size_t max_bytes_;
    size_t slab_elems_per_page_;
    size_t capacity_pages_ = 0;
    void* k_slab_ = nullptr;
    void* v_slab_ = nullptr;
    bool in_place_ = false;
    uint64_t generation_ = 0;
    std::deque<int32_t> free_;
    std::vector<uint8_t> in_use_;
    size_t allocated_ = 0, peak_ = 0;
    mutable std::mutex mutex_;
};

}  // namespace attention_hpc
