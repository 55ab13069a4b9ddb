// Device KV block pool: FIFO page ids on the host, K/V slabs in HBM.
#include "memory/kv_block_pool.hpp"

#include <algorithm>

#include "hip_support.hpp"

namespace attention_hpc {

using hipsup::check;

KVBlockPool::KVBlockPool(size_t page_tokens, size_t heads, size_t head_dim, DataType dtype, size_t initial_pages,
                         size_t growth, size_t max_bytes)
    : page_tokens_(page_tokens), heads_(heads), head_dim_(head_dim), dtype_(dtype), growth_(growth), max_bytes_(max_bytes) {
    if (page_tokens == 0 || heads == 0 || head_dim == 0)
        throw AttentionException(AttentionError::INVALID_PARAMETERS, "KVBlockPool: page geometry must be positive");
    slab_elems_per_page_ = page_tokens * heads * head_dim;
    if (max_bytes_ == 0) {
        ahpc_device_info info;
        check(ahpc_hip_device_info(0, &info), "device query");
        const uint64_t avail = info.free_memory_bytes ? info.free_memory_bytes : info.total_memory_bytes;
        max_bytes_ = static_cast<size_t>(avail / 10 * 9);
    }
    // Where the device has virtual memory management the slabs are address ranges sized for the whole budget, backed
    // by physical memory only as far as pages exist: they grow in place.
    const size_t page_bytes_one = slab_elems_per_page_ * hipsup::dtype_size(dtype_);
    size_t granularity = 0;
    int64_t wanted = 1;
    ahpc_hip_get_tuning("pool_in_place", &wanted);
    if (wanted != 0 && ahpc_hip_vmem_granularity(&granularity) == 0 && granularity != 0) {
        const size_t range = std::max<size_t>(max_bytes_ / (2 * page_bytes_one), 1) * page_bytes_one;
        // memory arrives in chunks of one size per slab: 64 MiB, or more where the budget is large (at most 256 chunks)
        size_t chunk = size_t(64) << 20;
        while (chunk * 256 < range) chunk *= 2;
        void* nk = nullptr;
        void* nv = nullptr;
        if (ahpc_hip_vmem_reserve(&nk, range, chunk) == 0 && ahpc_hip_vmem_reserve(&nv, range, chunk) == 0) {
            k_slab_ = nk;
            v_slab_ = nv;
            in_place_ = true;
        } else {
            ahpc_hip_vmem_release(nk);
            ahpc_hip_vmem_release(nv);
        }
    }
    std::lock_guard<std::mutex> lock(mutex_);
    create_pages_locked(initial_pages);
}

KVBlockPool::~KVBlockPool() {
    if (in_place_) {
        ahpc_hip_vmem_release(k_slab_);
        ahpc_hip_vmem_release(v_slab_);
    } else {
        ahpc_hip_free(k_slab_);
        ahpc_hip_free(v_slab_);
    }
}

// Grows the slabs to hold at least `pages` pages.  In place (the usual case): more physical memory is mapped behind
// the slabs' address ranges, in whole chunks, within the budget; nothing moves, no stream waits, the generation stays
// what it is.  Without virtual memory management: new allocation of twice
// the size (at least 64 pages), device-to-device copy of what exists, release of the old slabs.
void KVBlockPool::reserve_locked(size_t pages) {
    if (pages <= capacity_pages_) return;
    const size_t page_bytes_one = slab_elems_per_page_ * hipsup::dtype_size(dtype_);
    const size_t cap_by_budget = max_bytes_ / (2 * page_bytes_one);
    if (pages > cap_by_budget)
        throw MemoryPoolException("KV block pool exhausted: " + std::to_string(pages) + " pages needed, device budget allows " +
                                  std::to_string(cap_by_budget));
    if (in_place_) {
        // whole chunks: what a commit gives beyond the request is capacity for later pages
        size_t got_k = 0, got_v = 0;
        const int rk = ahpc_hip_vmem_commit(k_slab_, pages * page_bytes_one, &got_k);
        const int rv = ahpc_hip_vmem_commit(v_slab_, pages * page_bytes_one, &got_v);
        capacity_pages_ = std::max(capacity_pages_, std::min(std::min(got_k, got_v) / page_bytes_one, cap_by_budget));
        if (rk != 0 || rv != 0 || capacity_pages_ < pages)
            throw MemoryPoolException("KV block pool exhausted: the device cannot back " + std::to_string(pages) + " pages (" +
                                      std::to_string(capacity_pages_) + " backed, status " + std::to_string(rk ? rk : rv) + ")");
        return;
    }
    size_t want = std::max<size_t>(std::max<size_t>(capacity_pages_ * 2, pages), 64);
    if (want > cap_by_budget) want = cap_by_budget;
    // Old and new slabs exist side by side until the copy is done; when the device cannot hold both, fall back
    // to exactly what is needed, and report what is left as the pool being exhausted (not as a failed call).
    void* nk = nullptr;
    void* nv = nullptr;
    for (;;) {
        const int rk = ahpc_hip_malloc(&nk, want * page_bytes_one);
        const int rv = rk == 0 ? ahpc_hip_malloc(&nv, want * page_bytes_one) : rk;
        if (rk == 0 && rv == 0) break;
        if (rk == 0) ahpc_hip_free(nk);
        nk = nv = nullptr;
        if (want == pages)
            throw MemoryPoolException("KV block pool exhausted: the device cannot hold " + std::to_string(pages) +
                                      " pages next to the " + std::to_string(capacity_pages_) + " in use while the pool grows");
        want = pages;
    }
    if (capacity_pages_) {
        // every stream of the device: work that still reads or writes the old slabs ends before they are copied
        check(ahpc_hip_device_synchronize(), "KV slab copy");
        check(ahpc_hip_memcpy_d2d(nk, k_slab_, capacity_pages_ * page_bytes_one, nullptr), "KV slab copy");
        check(ahpc_hip_memcpy_d2d(nv, v_slab_, capacity_pages_ * page_bytes_one, nullptr), "KV slab copy");
        check(ahpc_hip_stream_synchronize(nullptr), "KV slab copy");
        ahpc_hip_free(k_slab_);
        ahpc_hip_free(v_slab_);
    }
    k_slab_ = nk;
    v_slab_ = nv;
    capacity_pages_ = want;
    ++generation_;
}

void KVBlockPool::create_pages_locked(size_t count) {
    if (count == 0) return;
    const size_t first = in_use_.size();
    reserve_locked(first + count);
    in_use_.resize(first + count, 0);
    for (size_t i = 0; i < count; ++i) free_.push_back(static_cast<int32_t>(first + i));
}

int32_t KVBlockPool::allocate_page() {
    std::lock_guard<std::mutex> lock(mutex_);
    if (free_.empty()) {
        if (growth_ == 0) throw MemoryPoolException("KV block pool exhausted (fixed-size pool)");
        create_pages_locked(growth_);
    }
    const int32_t id = free_.front();
    free_.pop_front();
    in_use_[id] = 1;
    ++allocated_;
    peak_ = std::max(peak_, allocated_);
    return id;
}

void KVBlockPool::deallocate_page(int32_t page) {
    std::lock_guard<std::mutex> lock(mutex_);
    if (page < 0 || static_cast<size_t>(page) >= in_use_.size() || !in_use_[page]) return;
    in_use_[page] = 0;
    --allocated_;
    free_.push_back(page);
}

void KVBlockPool::resize_pool(size_t new_total_pages) {
    std::lock_guard<std::mutex> lock(mutex_);
    if (new_total_pages > in_use_.size()) {
        create_pages_locked(new_total_pages - in_use_.size());
        return;
    }
    // shrink: only free pages at the end of the id range can go
    size_t keep = in_use_.size();
    while (keep > new_total_pages && !in_use_[keep - 1]) --keep;
    if (keep == in_use_.size()) return;
    in_use_.resize(keep);
    std::deque<int32_t> still;
    for (int32_t id : free_)
        if (static_cast<size_t>(id) < keep) still.push_back(id);
    free_.swap(still);
    if (in_place_) {
        // work in flight may still read pages that were released a moment ago
        check(ahpc_hip_device_synchronize(), "KV pool shrink");
        const size_t page_bytes_one = slab_elems_per_page_ * hipsup::dtype_size(dtype_);
        size_t got_k = 0, got_v = 0;
        const int rk = ahpc_hip_vmem_decommit(k_slab_, keep * page_bytes_one, &got_k);
        const int rv = ahpc_hip_vmem_decommit(v_slab_, keep * page_bytes_one, &got_v);
        if (rk == 0 && rv == 0) capacity_pages_ = std::min(got_k, got_v) / page_bytes_one;
    }
}

std::vector<std::pair<int32_t, int32_t>> KVBlockPool::plan_compaction() const {
    std::lock_guard<std::mutex> lock(mutex_);
    std::vector<std::pair<int32_t, int32_t>> moves;
    size_t lo = 0;
    for (size_t hi = in_use_.size(); hi-- > allocated_;) {
        if (!in_use_[hi]) continue;
        while (lo < allocated_ && in_use_[lo]) ++lo;
        if (lo >= allocated_) break;  // (cannot happen: as many free ids below the mark as pages in use beyond it)
        moves.emplace_back(static_cast<int32_t>(hi), static_cast<int32_t>(lo));
        ++lo;
    }
    return moves;
}

void KVBlockPool::apply_compaction(const std::vector<std::pair<int32_t, int32_t>>& moves) {
    std::lock_guard<std::mutex> lock(mutex_);
    for (const auto& m : moves) {
        if (m.first < 0 || m.second < 0 || static_cast<size_t>(m.first) >= in_use_.size() ||
            static_cast<size_t>(m.second) >= in_use_.size() || !in_use_[m.first] || in_use_[m.second])
            throw AttentionException(AttentionError::INVALID_INPUT, "KVBlockPool: compaction move does not match the pool's state");
        in_use_[m.first] = 0;
        in_use_[m.second] = 1;
    }
    free_.clear();
    for (size_t id = 0; id < in_use_.size(); ++id)
        if (!in_use_[id]) free_.push_back(static_cast<int32_t>(id));
}

size_t KVBlockPool::get_pool_size() const {
    std::lock_guard<std::mutex> lock(mutex_);
    return in_use_.size();
}
size_t KVBlockPool::get_free_pages() const {
    std::lock_guard<std::mutex> lock(mutex_);
    return free_.size();
}
size_t KVBlockPool::get_allocated_pages() const {
    std::lock_guard<std::mutex> lock(mutex_);
    return allocated_;
}

KVBlockPoolStats KVBlockPool::stats() const {
    std::lock_guard<std::mutex> lock(mutex_);
    KVBlockPoolStats s;
    s.total_pages = in_use_.size();
    s.free_pages = free_.size();
    s.allocated_pages = allocated_;
    s.peak_allocated_pages = peak_;
    s.page_bytes = 2 * slab_elems_per_page_ * hipsup::dtype_size(dtype_);
    s.slab_capacity_pages = capacity_pages_;
    s.slab_bytes = capacity_pages_ * s.page_bytes;
    return s;
}

}  // namespace attention_hpc
