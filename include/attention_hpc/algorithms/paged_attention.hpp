// PagedAttention on the HIP backend: KV cache in a device block pool, block table in HBM, one
// batched decode launch.  Same class name and public methods as the reference's CPU class
// (src/algorithms/paged_attention.hpp:125-149, :176-263), so
// `dynamic_cast<PagedAttention*>(BackendFactory::createPagedAttention(type).get())`
// (examples/basic_usage.cpp:142-145) yields this object and the sequence API below drives it.
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "api/attention_interface.hpp"
#include "api/tensor.hpp"
#include "memory/kv_block_pool.hpp"

namespace attention_hpc {

struct PagedAttentionConfig {
    size_t page_size = 16;                  // overridden by AttentionParams::page_size at configure()
    size_t max_pages_per_sequence = 1024;   // raised automatically to fit AttentionParams::max_sequence_length
    size_t initial_page_pool_size = 64;
    bool enable_page_caching = true;
    bool enable_memory_prefetching = false;
    size_t memory_pool_size = 1024ull * 1024 * 1024;  // soft figure used by get_memory_utilization()
    size_t max_concurrent_sequences = 32;   // rows of the device block table; grows on demand
    size_t block_size = 64;
    bool enable_dynamic_batching = true;
    bool use_kernel_fusion = false;
    bool enable_async_copying = false;
    size_t prefetch_distance = 2;
    bool use_contiguous_layout = true;
    bool enable_memory_coalescing = true;
    // Additions for the device pool
    size_t page_pool_growth = 16;           // pages created when the free queue is empty (reference: 16)
    size_t device_pool_max_bytes = 0;       // 0 = up to 90% of free HBM
    int kv_cache_dtype = -1;                // -1 = the dtype of the first append_kv_cache; else a DataType value
    size_t split_chunk_tokens = 0;          // decode context split, 0 = choose
};

class PagedAttention : public AttentionInterface {
public:
    PagedAttention();
    ~PagedAttention() override;
    PagedAttention(const PagedAttention&) = delete;
    PagedAttention& operator=(const PagedAttention&) = delete;

    void configure(const AttentionParams& params, const PerformanceConfig& perf_config = PerformanceConfig{}) override;
    void configure_paged_attention(const PagedAttentionConfig& paged_config);

    // Convenience decode without a standing cache: K/V [B,N,H,d] are appended to temporary
    // sequences, the single query token per batch entry ([B,1,H,d]) attends to all N keys.
    void forward(const TensorShape& query_shape, const void* query_data, const TensorShape& key_shape,
                 const void* key_data, const TensorShape& value_shape, const void* value_data,
                 const TensorShape& output_shape, void* output_data, const void* attention_mask = nullptr) override;

    void backward(const TensorShape&, const void*, const TensorShape&, const void*, const TensorShape&, const void*,
                  const TensorShape&, const void*, const TensorShape&, void*, const TensorShape&, void*,
                  const TensorShape&, void*, const void* = nullptr) override;

    size_t get_workspace_size(const AttentionParams& params) const override;
    void set_workspace(void* workspace_ptr, size_t workspace_size) override;
    bool supports_data_type(DataType data_type) const override;
    bool supports_memory_layout(MemoryLayout layout) const override;
    std::string get_backend_name() const override;
    std::string get_version() const override;
    void enable_profiling(bool enable) override;
    std::vector<std::pair<std::string, double>> get_profiling_results() const override;
    void reset_profiling() override;
    AttentionError validate_inputs(const TensorShape& query_shape, const TensorShape& key_shape,
                                   const TensorShape& value_shape, const TensorShape& output_shape,
                                   const AttentionParams& params) const override;

    // ---- sequences ---------------------------------------------------------------------------
    size_t create_sequence(size_t max_length);      // ids start at 1
    void destroy_sequence(size_t sequence_id);      // unknown ids are ignored
    void reset_sequence(size_t sequence_id);
    bool is_sequence_active(size_t sequence_id) const;
    void extend_sequence(size_t sequence_id, size_t additional_tokens);  // raises the limit, pre-allocates pages
    void truncate_sequence(size_t sequence_id, size_t new_length);       // frees tail pages
    size_t get_sequence_length(size_t sequence_id) const;
    size_t get_max_sequence_length(size_t sequence_id) const;

    // ---- KV cache ----------------------------------------------------------------------------
    // key/value: [num_tokens, heads, head_dim] of `data_type`, host or device memory.  Pages are
    // taken from the pool as needed.  Unknown sequence -> INVALID_INPUT.
    void append_kv_cache(size_t sequence_id, const void* key_data, const void* value_data, size_t num_tokens,
                         DataType data_type);
    // The prefill -> cache hand-off: the K and V tensors a FlashAttention forward just attended over go into
    // the caches of `sequence_ids` in ONE launch.  Dense: kv_shape = {B, N, key_value_heads, head_dim}, batch
    // entry b feeds sequence_ids[b] with its first num_tokens[b] tokens (empty vector = all N).  Packed:
    // kv_shape = {total_tokens, key_value_heads, head_dim} with cu_seqlens[0..B] as in forward_varlen.
    // Host or device memory; same errors as append_kv_cache.  (The reference appends one sequence per call,
    // src/algorithms/paged_attention.cpp:434-462.)
    void append_kv_cache_batch(const std::vector<size_t>& sequence_ids, const TensorShape& kv_shape, const void* key_data,
                               const void* value_data, const std::vector<size_t>& num_tokens = {});
    void append_kv_cache_packed(const std::vector<size_t>& sequence_ids, const TensorShape& kv_shape, const void* key_data,
                                const void* value_data, const int32_t* cu_seqlens);
    void get_kv_cache(size_t sequence_id, void* key_data, void* value_data, size_t start_token, size_t num_tokens,
                      DataType data_type);
    void clear_kv_cache(size_t sequence_id);

    // ---- decode ------------------------------------------------------------------------------
    // One query token per listed sequence (shape {1,1,H,d}, {1,H,d} or {H,d}); all of them run in
    // one launch.  Vector sizes must agree -> else INVALID_INPUT.  An empty sequence yields zeros.
    void forward_batch(const std::vector<size_t>& sequence_ids, const std::vector<TensorShape>& query_shapes,
                       const std::vector<const void*>& query_data, const std::vector<TensorShape>& output_shapes,
                       const std::vector<void*>& output_data, const std::vector<const void*>& attention_masks = {});

    // ---- statistics ----------------------------------------------------------------------------
    size_t get_total_memory_usage() const;   // bytes of KV pages currently owned by sequences
    size_t get_peak_memory_usage() const;
    float get_memory_utilization() const;    // usage / PagedAttentionConfig::memory_pool_size
    size_t get_active_sequences_count() const;
    KVBlockPoolStats get_pool_stats() const;
    // Page ids of a sequence in order (what its block-table row holds); for tests and tooling.
    std::vector<int32_t> get_sequence_pages(size_t sequence_id) const;

    // Moves the pages in use onto the lowest page ids (device copy + block-table rewrite) and returns the pool's free
    // tail to the device; results of later decodes are unchanged bit for bit.
    void compact_pages();
    void preload_pages(const std::vector<size_t>& sequence_ids); // no-op: the pool is always device-resident

private:
    struct Impl;
    Impl* impl_;
};

}  // namespace attention_hpc
