// FlashAttention forward on the HIP backend.  Same class name, configuration struct and public
// methods as the reference's CPU class (src/algorithms/flash_attention.hpp:17-36, :39-62,
// :85-133), so `std::make_unique<FlashAttention>()` and the factory both hand out this object;
// the work happens in one kernel launch through the C ABI (ahpc_hip_flash_fwd*).
#pragma once

#include <cmath>
#include <limits>
#include <string>
#include <utility>
#include <vector>

#include "api/attention_interface.hpp"
#include "api/tensor.hpp"

namespace attention_hpc {

struct FlashAttentionConfig {
    // Tile sizes are accepted for compatibility; the kernels pick their own tiling and the result
    // does not depend on these (the reference's tests require exactly that,
    // tests/test_flash_attention.cpp:360-402).
    size_t block_size_q = 64;
    size_t block_size_k = 64;
    size_t block_size_v = 64;
    bool use_causal_mask = false;   // OR-ed with AttentionParams::causal_mask
    bool apply_dropout = false;     // must stay false (inference forward only)
    float dropout_probability = 0.0f;
    bool use_safe_softmax = true;
    float softmax_scale = 0.0f;     // 0 = AttentionParams::scale_factor, or 1/sqrt(d) if that is 0 too
    bool prefetch_next_block = true;
    bool use_async_copy = false;
    size_t num_parallel_blocks = 1;
    // Addition: tensors are indexed [B,H,N,d] (as the reference's own test oracle does,
    // tests/test_flash_attention.cpp:46) instead of the declared [B,N,H,d].
    bool tensor_layout_bhnd = false;
    // Addition, for callers that run forward() and then backward() on the same tensors (training): forward() keeps its
    // softmax statistic per query row and where its output lives on the device, and a backward() whose query, key, value
    // and mask pointers, shapes and settings are those of that forward() reads them instead of recomputing both (a fifth
    // less time).  The caller promises that those tensors' contents, and the output if it was given as a device pointer,
    // have not changed in between; any other backward() recomputes as usual.
    bool keep_forward_statistics = false;
};

// The merge rule shared by key tiles, split contexts and (in principle) devices.
struct OnlineSoftmaxState {
    float max_val = -std::numeric_limits<float>::infinity();
    float sum_exp = 0.0f;
    void reset() { *this = OnlineSoftmaxState{}; }
    void update(float new_max, float new_sum) {
        if (new_max > max_val) {
            sum_exp = sum_exp * std::exp(max_val - new_max) + new_sum;
            max_val = new_max;
        } else {
            sum_exp += new_sum * std::exp(new_max - max_val);
        }
    }
    float get_normalizer() const { return sum_exp > 0.0f ? 1.0f / sum_exp : 0.0f; }
};

class FlashAttention : public AttentionInterface {
public:
    FlashAttention();
    ~FlashAttention() override;
    FlashAttention(const FlashAttention&) = delete;
    FlashAttention& operator=(const FlashAttention&) = delete;

    void configure(const AttentionParams& params, const PerformanceConfig& perf_config = PerformanceConfig{}) override;
    void configure_flash_attention(const FlashAttentionConfig& flash_config);

    void forward(const TensorShape& query_shape, const void* query_data, const TensorShape& key_shape,
                 const void* key_data, const TensorShape& value_shape, const void* value_data,
                 const TensorShape& output_shape, void* output_data, const void* attention_mask = nullptr) override;

    // Ragged batch: tensors packed as [total_tokens, heads, head_dim]; sequence i owns tokens
    // cu_seqlens[i] .. cu_seqlens[i+1]-1 (n_seqs+1 host integers).  Not in the reference.
    void forward_varlen(const TensorShape& packed_shape, const void* query_data, const void* key_data,
                        const void* value_data, void* output_data, const int32_t* cu_seqlens, size_t n_seqs);

    // Gradients of forward() for a given grad_output: grad_query has the shape of the query tensor,
    // grad_key / grad_value those of key / value (with grouped heads each K/V head receives the sum over its
    // query heads).  All tensors share one data type; pointers may be host or device memory.  The forward
    // output is not needed (it is recomputed).  Reference: src/algorithms/flash_attention.cpp:114-174, whose
    // gradient loops (:496-580) are placeholders.
    void backward(const TensorShape& grad_output_shape, const void* grad_output_data, const TensorShape& query_shape,
                  const void* query_data, const TensorShape& key_shape, const void* key_data, const TensorShape& value_shape,
                  const void* value_data, const TensorShape& grad_query_shape, void* grad_query_data,
                  const TensorShape& grad_key_shape, void* grad_key_data, const TensorShape& grad_value_shape,
                  void* grad_value_data, const void* attention_mask = nullptr) override;

    // Gradients for a ragged batch packed as in forward_varlen: grad_output, query, grad_query are
    // [total_tokens, num_heads, head_dim]; key, value, grad_key, grad_value [total_tokens, key_value_heads, head_dim].
    void backward_varlen(const TensorShape& packed_shape, const void* grad_output_data, const void* query_data,
                         const void* key_data, const void* value_data, void* grad_query_data, void* grad_key_data,
                         void* grad_value_data, const int32_t* cu_seqlens, size_t n_seqs);

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

private:
    struct Impl;
    Impl* impl_;
};

}  // namespace attention_hpc
