// FlashAttention (HIP backend): validation, host/device pointer staging, one launch per forward, three per backward.
#include "algorithms/flash_attention.hpp"

#include <algorithm>
#include <chrono>
#include <cmath>

#include "hip_support.hpp"

namespace attention_hpc {

using hipsup::check;

struct FlashAttention::Impl {
    FlashAttentionConfig cfg;
    bool configured = false;
    hipsup::Stream stream;
    hipsup::DeviceBuffer dq, dk, dv, dout, dmask, dcu;
    hipsup::DeviceBuffer ddo, gq, gk, gv, ws;  // backward: staged dO, gradients, statistics workspace
    // What the last forward() left for a backward() on the same tensors (FlashAttentionConfig::keep_forward_statistics):
    // the row statistics, the device address of its output, and what identifies the call.
    hipsup::DeviceBuffer row_stats;
    struct Kept {
        bool valid = false;
        const void* q = nullptr;
        const void* k = nullptr;
        const void* v = nullptr;
        const void* mask = nullptr;
        const void* out_on_device = nullptr;
        size_t N = 0;
        DataType type = DataType::FLOAT32;
        int causal = 0;
        float scale = 0.0f;
        bool bhnd = false;
    } kept;
    std::vector<std::pair<std::string, double>> profile;
};

FlashAttention::FlashAttention() : impl_(new Impl) {}
FlashAttention::~FlashAttention() { delete impl_; }

// Reference: FlashAttention::configure, src/algorithms/flash_attention.cpp:32-57 (dimension check and
// INVALID_PARAMETERS).  Unlike the reference, AttentionParams::causal_mask and ::scale_factor are
// honoured (its tests set them and expect them to act, tests/test_flash_attention.cpp:180-181, :108).
void FlashAttention::configure(const AttentionParams& params, const PerformanceConfig& perf_config) {
    if (params.batch_size == 0 || params.sequence_length == 0 || params.num_heads == 0 || params.head_dimension == 0)
        throw AttentionException(AttentionError::INVALID_PARAMETERS, "Invalid attention parameters: dimensions must be positive");
    // Grouped key/value heads (AttentionParams::key_value_heads, src/api/attention_interface.hpp:61; the
    // reference reads the field nowhere): consecutive query heads share a K/V head, so the counts must divide.
    if (params.key_value_heads != 0 && (params.key_value_heads > params.num_heads || params.num_heads % params.key_value_heads))
        throw AttentionException(AttentionError::INVALID_PARAMETERS, "key_value_heads must divide num_heads");
    if (params.apply_rotary_embedding)
        throw AttentionException(AttentionError::UNSUPPORTED_OPERATION, "rotary embedding is not applied by this backend");
    if (params.head_dimension > 256)
        throw AttentionException(AttentionError::UNSUPPORTED_OPERATION, "head_dimension above 256 is not supported");
    int n = 0;
    ahpc_hip_device_count(&n);
    if (n < 1) throw AttentionException(AttentionError::BACKEND_NOT_AVAILABLE, "no HIP device");
    current_params_ = params;
    current_perf_config_ = perf_config;
    impl_->kept.valid = false;
    if (perf_config.enable_profiling) profiling_enabled_ = true;
    impl_->configured = true;
}

void FlashAttention::configure_flash_attention(const FlashAttentionConfig& flash_config) {
    if (flash_config.apply_dropout && flash_config.dropout_probability > 0.0f)
        throw AttentionException(AttentionError::UNSUPPORTED_OPERATION, "dropout is not supported (forward inference only)");
    impl_->cfg = flash_config;
    impl_->kept.valid = false;
}

static size_t kv_heads(const AttentionParams& p) { return p.key_value_heads ? p.key_value_heads : p.num_heads; }

static bool shape_ok(const TensorShape& s, const AttentionParams& p, size_t heads) {
    return s.dimensions.size() == 4 && s.dimensions[0] == p.batch_size && s.dimensions[1] > 0 &&
           s.dimensions[2] == heads && s.dimensions[3] == p.head_dimension;
}

// Reference: FlashAttention::validate_inputs, src/algorithms/flash_attention.cpp:238-275 (4-D, batch,
// heads and head_dim must match the configured parameters; the sequence dimension is free).
AttentionError FlashAttention::validate_inputs(const TensorShape& q, const TensorShape& k, const TensorShape& v,
                                               const TensorShape& o, const AttentionParams& params) const {
    if (!shape_ok(q, params, params.num_heads) || !shape_ok(k, params, kv_heads(params)) ||
        !shape_ok(v, params, kv_heads(params)) || !shape_ok(o, params, params.num_heads))
        return AttentionError::INVALID_INPUT;
    return AttentionError::SUCCESS;
}

namespace {
// Host pointer -> staged device copy; device pointer -> itself.
const void* stage_in(const void* src, size_t bytes, hipsup::DeviceBuffer& buf, void* stream) {
    if (hipsup::is_device_pointer(src)) return src;
    void* d = buf.reserve(bytes);
    check(ahpc_hip_memcpy_h2d(d, src, bytes, stream), "copy to device");
    return d;
}
}  // namespace

// Reference: FlashAttention::forward, src/algorithms/flash_attention.cpp:68-112.  The reference's
// forward does not validate, yet its tests require an AttentionException for a wrong head dimension,
// a wrong batch size and a null pointer (tests/test_flash_attention.cpp:310-357,
// tests/test_backends.cpp:631-680): this one validates first.
void FlashAttention::forward(const TensorShape& qs, const void* q, const TensorShape& ks, const void* k,
                             const TensorShape& vs, const void* v, const TensorShape& os, void* o, const void* mask) {
    if (!impl_->configured)
        throw AttentionException(AttentionError::INVALID_PARAMETERS, "FlashAttention not configured. Call configure() first.");
    if (!q || !k || !v || !o) throw AttentionException(AttentionError::INVALID_INPUT, "null tensor pointer");
    if (validate_inputs(qs, ks, vs, os, current_params_) != AttentionError::SUCCESS)
        throw AttentionException(AttentionError::INVALID_INPUT, "tensor shapes do not match the configured parameters");
    const size_t N = qs.dimensions[1];
    if (ks.dimensions[1] != N || vs.dimensions[1] != N || os.dimensions[1] != N)
        throw AttentionException(AttentionError::INVALID_INPUT, "query, key, value and output must share one sequence length");
    if (ks.data_type != qs.data_type || vs.data_type != qs.data_type || os.data_type != qs.data_type)
        throw AttentionException(AttentionError::INVALID_INPUT, "query, key, value and output must share one data type");
    for (const TensorShape* s : {&qs, &ks, &vs, &os})
        if (s->layout != MemoryLayout::ROW_MAJOR)
            throw AttentionException(AttentionError::UNSUPPORTED_OPERATION, "only ROW_MAJOR tensors are supported");

    const size_t B = current_params_.batch_size, H = current_params_.num_heads, d = current_params_.head_dimension;
    const size_t Hkv = kv_heads(current_params_);
    const size_t bytes = qs.total_bytes(), kv_bytes = ks.total_bytes();
    void* st = impl_->stream.get();
    hipsup::EventTimer timer;
    const auto wall0 = std::chrono::steady_clock::now();

    const void* dq = stage_in(q, bytes, impl_->dq, st);
    const void* dk = stage_in(k, kv_bytes, impl_->dk, st);
    const void* dv = stage_in(v, kv_bytes, impl_->dv, st);
    const bool out_on_device = hipsup::is_device_pointer(o);
    void* dout = out_on_device ? o : impl_->dout.reserve(bytes);
    const float* dmask = nullptr;
    if (mask) dmask = static_cast<const float*>(stage_in(mask, B * N * N * sizeof(float), impl_->dmask, st));

    float scale = impl_->cfg.softmax_scale > 0.0f ? impl_->cfg.softmax_scale : current_params_.scale_factor;
    if (!(scale > 0.0f)) scale = 1.0f / std::sqrt(static_cast<float>(d));
    const int causal = (current_params_.causal_mask || impl_->cfg.use_causal_mask) ? 1 : 0;
    int64_t sb, sn, sh, kb, kn, kh;
    if (impl_->cfg.tensor_layout_bhnd) {
        sb = (int64_t)(H * N * d); sh = (int64_t)(N * d); sn = (int64_t)d;
        kb = (int64_t)(Hkv * N * d); kh = sh; kn = sn;
    } else {
        sb = (int64_t)(N * H * d); sn = (int64_t)(H * d); sh = (int64_t)d;
        kb = (int64_t)(N * Hkv * d); kn = (int64_t)(Hkv * d); kh = sh;
    }
    const int dt = hipsup::dtype_code(qs.data_type);
    impl_->kept.valid = false;
    if (profiling_enabled_) timer.start(st);
    if (impl_->cfg.keep_forward_statistics) {
        float* stats = static_cast<float*>(impl_->row_stats.reserve(ahpc_hip_flash_row_stats_bytes((int64_t)B, (int64_t)N, (int64_t)H)));
        int written = 0;
        check(ahpc_hip_flash_fwd_keep(dq, dk, dv, dout, dt, (int64_t)B, (int64_t)N, (int64_t)H, (int64_t)Hkv, (int64_t)d, sb, sn,
                                      sh, kb, kn, kh, scale, causal, dmask, stats, &written, st), "flash forward");
        if (written) {
            Impl::Kept& kp = impl_->kept;
            kp.valid = true;
            kp.q = q; kp.k = k; kp.v = v; kp.mask = mask;
            kp.out_on_device = dout;
            kp.N = N; kp.type = qs.data_type; kp.causal = causal; kp.scale = scale; kp.bhnd = impl_->cfg.tensor_layout_bhnd;
        }
    } else {
        check(ahpc_hip_flash_fwd_gqa(dq, dk, dv, dout, dt, (int64_t)B, (int64_t)N, (int64_t)H, (int64_t)Hkv, (int64_t)d, sb, sn,
                                     sh, kb, kn, kh, scale, causal, dmask, st), "flash forward");
    }
    if (profiling_enabled_) timer.stop(st);
    if (!out_on_device) check(ahpc_hip_memcpy_d2h(o, dout, bytes, st), "copy from device");
    impl_->stream.sync();

    if (profiling_enabled_) {
        // "forward_pass" keeps the reference's meaning: wall-clock ms of the whole call
        // (src/algorithms/flash_attention.cpp:107-111).  The kernel-only time and the rate it implies follow.
        const double wall_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - wall0).count();
        const double kernel_ms = timer.elapsed_ms();
        const double flop = (causal ? 2.0 : 4.0) * (double)B * (double)H * (double)N * (double)N * (double)d;
        impl_->profile.emplace_back("forward_pass", wall_ms);
        impl_->profile.emplace_back("forward_kernel_ms", kernel_ms);
        impl_->profile.emplace_back("forward_kernel_tflops", kernel_ms > 0 ? flop / (kernel_ms * 1e-3) / 1e12 : 0.0);
    }
}

// `shape` is the packed shape of Q and O, [total_tokens, num_heads, head_dim]; K and V are
// [total_tokens, key_value_heads, head_dim].
void FlashAttention::forward_varlen(const TensorShape& shape, const void* q, const void* k, const void* v, void* o,
                                    const int32_t* cu_seqlens, size_t n_seqs) {
    if (!impl_->configured)
        throw AttentionException(AttentionError::INVALID_PARAMETERS, "FlashAttention not configured. Call configure() first.");
    if (!q || !k || !v || !o || !cu_seqlens) throw AttentionException(AttentionError::INVALID_INPUT, "null pointer");
    const size_t H = current_params_.num_heads, d = current_params_.head_dimension;
    if (shape.dimensions.size() != 3 || shape.dimensions[1] != H || shape.dimensions[2] != d || n_seqs == 0)
        throw AttentionException(AttentionError::INVALID_INPUT, "packed tensors must be [total_tokens, heads, head_dim]");
    int64_t max_len = 0;
    if (cu_seqlens[0] != 0) throw AttentionException(AttentionError::INVALID_INPUT, "cu_seqlens must start at 0");
    for (size_t i = 0; i < n_seqs; ++i) {
        const int64_t len = (int64_t)cu_seqlens[i + 1] - cu_seqlens[i];
        if (len < 0) throw AttentionException(AttentionError::INVALID_INPUT, "cu_seqlens must not decrease");
        max_len = std::max(max_len, len);
    }
    if ((size_t)cu_seqlens[n_seqs] != shape.dimensions[0])
        throw AttentionException(AttentionError::INVALID_INPUT, "cu_seqlens must end at total_tokens");
    if (max_len == 0) return;
    impl_->kept.valid = false;  // (the output staging buffer is about to be reused)
    void* st = impl_->stream.get();
    const size_t Hkv = kv_heads(current_params_);
    const size_t bytes = shape.total_bytes(), kv_bytes = bytes / H * Hkv;
    const void* dq = stage_in(q, bytes, impl_->dq, st);
    const void* dk = stage_in(k, kv_bytes, impl_->dk, st);
    const void* dv = stage_in(v, kv_bytes, impl_->dv, st);
    const bool out_on_device = hipsup::is_device_pointer(o);
    void* dout = out_on_device ? o : impl_->dout.reserve(bytes);
    if (!out_on_device) check(ahpc_hip_memset(dout, 0, bytes, st), "clear output");
    void* dcu = impl_->dcu.reserve((n_seqs + 1) * sizeof(int32_t));
    check(ahpc_hip_memcpy_h2d(dcu, cu_seqlens, (n_seqs + 1) * sizeof(int32_t), st), "copy cu_seqlens");
    float scale = impl_->cfg.softmax_scale > 0.0f ? impl_->cfg.softmax_scale : current_params_.scale_factor;
    if (!(scale > 0.0f)) scale = 1.0f / std::sqrt(static_cast<float>(d));
    const int causal = (current_params_.causal_mask || impl_->cfg.use_causal_mask) ? 1 : 0;
    check(ahpc_hip_flash_fwd_varlen_gqa(dq, dk, dv, dout, hipsup::dtype_code(shape.data_type),
                                        static_cast<const int32_t*>(dcu), (int64_t)n_seqs, max_len, (int64_t)H, (int64_t)Hkv,
                                        (int64_t)d, (int64_t)(H * d), (int64_t)d, (int64_t)(Hkv * d), (int64_t)d, scale, causal,
                                        st), "flash forward (ragged)");
    if (!out_on_device) check(ahpc_hip_memcpy_d2h(o, dout, bytes, st), "copy from device");
    impl_->stream.sync();
}

// Reference: FlashAttention::backward, src/algorithms/flash_attention.cpp:114-174.  The reference converts,
// calls two placeholder gradient loops (:496-580) and converts back; here the gradients are the derivative of
// forward(): three launches behind ahpc_hip_flash_bwd.  Validation as in forward(); the gradient tensors
// must have the shapes of the tensors they belong to.
void FlashAttention::backward(const TensorShape& gos, const void* go, const TensorShape& qs, const void* q,
                              const TensorShape& ks, const void* k, const TensorShape& vs, const void* v,
                              const TensorShape& gqs, void* gq, const TensorShape& gks, void* gk, const TensorShape& gvs,
                              void* gv, const void* mask) {
    if (!impl_->configured)
        throw AttentionException(AttentionError::INVALID_PARAMETERS, "FlashAttention not configured. Call configure() first.");
    if (!go || !q || !k || !v || !gq || !gk || !gv) throw AttentionException(AttentionError::INVALID_INPUT, "null tensor pointer");
    if (validate_inputs(qs, ks, vs, gos, current_params_) != AttentionError::SUCCESS ||
        validate_inputs(gqs, gks, gvs, gos, current_params_) != AttentionError::SUCCESS)
        throw AttentionException(AttentionError::INVALID_INPUT, "tensor shapes do not match the configured parameters");
    const size_t N = qs.dimensions[1];
    for (const TensorShape* s : {&gos, &qs, &ks, &vs, &gqs, &gks, &gvs}) {
        if (s->dimensions[1] != N)
            throw AttentionException(AttentionError::INVALID_INPUT, "all tensors must share one sequence length");
        if (s->data_type != qs.data_type)
            throw AttentionException(AttentionError::INVALID_INPUT, "all tensors must share one data type");
        if (s->layout != MemoryLayout::ROW_MAJOR)
            throw AttentionException(AttentionError::UNSUPPORTED_OPERATION, "only ROW_MAJOR tensors are supported");
    }
    const size_t B = current_params_.batch_size, H = current_params_.num_heads, d = current_params_.head_dimension;
    const size_t Hkv = kv_heads(current_params_);
    const size_t bytes = qs.total_bytes(), kv_bytes = ks.total_bytes();
    void* st = impl_->stream.get();
    hipsup::EventTimer timer;
    const auto wall0 = std::chrono::steady_clock::now();

    const void* d_go = stage_in(go, bytes, impl_->ddo, st);
    const void* d_q = stage_in(q, bytes, impl_->dq, st);
    const void* d_k = stage_in(k, kv_bytes, impl_->dk, st);
    const void* d_v = stage_in(v, kv_bytes, impl_->dv, st);
    const bool gq_dev = hipsup::is_device_pointer(gq), gk_dev = hipsup::is_device_pointer(gk), gv_dev = hipsup::is_device_pointer(gv);
    void* d_gq = gq_dev ? gq : impl_->gq.reserve(bytes);
    void* d_gk = gk_dev ? gk : impl_->gk.reserve(kv_bytes);
    void* d_gv = gv_dev ? gv : impl_->gv.reserve(kv_bytes);
    const float* dmask = nullptr;
    if (mask) dmask = static_cast<const float*>(stage_in(mask, B * N * N * sizeof(float), impl_->dmask, st));
    const size_t ws_bytes = ahpc_hip_flash_bwd_workspace_bytes((int64_t)B, (int64_t)N, (int64_t)H);
    void* ws = impl_->ws.reserve(ws_bytes);

    float scale = impl_->cfg.softmax_scale > 0.0f ? impl_->cfg.softmax_scale : current_params_.scale_factor;
    if (!(scale > 0.0f)) scale = 1.0f / std::sqrt(static_cast<float>(d));
    const int causal = (current_params_.causal_mask || impl_->cfg.use_causal_mask) ? 1 : 0;
    int64_t sb, sn, sh, kb, kn, kh;
    if (impl_->cfg.tensor_layout_bhnd) {
        sb = (int64_t)(H * N * d); sh = (int64_t)(N * d); sn = (int64_t)d;
        kb = (int64_t)(Hkv * N * d); kh = sh; kn = sn;
    } else {
        sb = (int64_t)(N * H * d); sn = (int64_t)(H * d); sh = (int64_t)d;
        kb = (int64_t)(N * Hkv * d); kn = (int64_t)(Hkv * d); kh = sh;
    }
    // the forward's statistics and output, if this is the backward of the last forward()
    const Impl::Kept& kp = impl_->kept;
    const bool same = impl_->cfg.keep_forward_statistics && kp.valid && kp.q == q && kp.k == k && kp.v == v && kp.mask == mask &&
                      kp.N == N && kp.type == qs.data_type && kp.causal == causal && kp.scale == scale &&
                      kp.bhnd == impl_->cfg.tensor_layout_bhnd;
    if (profiling_enabled_) timer.start(st);
    check(ahpc_hip_flash_bwd_kept(d_go, d_q, d_k, d_v, same ? kp.out_on_device : nullptr,
                                  same ? static_cast<const float*>(impl_->row_stats.get()) : nullptr, d_gq, d_gk, d_gv,
                                  hipsup::dtype_code(qs.data_type), (int64_t)B, (int64_t)N, (int64_t)H, (int64_t)Hkv, (int64_t)d, sb,
                                  sn, sh, kb, kn, kh, scale, causal, dmask, ws, ws_bytes, st),
          "flash backward");
    if (profiling_enabled_) timer.stop(st);
    if (!gq_dev) check(ahpc_hip_memcpy_d2h(gq, d_gq, bytes, st), "copy from device");
    if (!gk_dev) check(ahpc_hip_memcpy_d2h(gk, d_gk, kv_bytes, st), "copy from device");
    if (!gv_dev) check(ahpc_hip_memcpy_d2h(gv, d_gv, kv_bytes, st), "copy from device");
    impl_->stream.sync();

    if (profiling_enabled_) {
        // "backward_pass": wall-clock ms of the whole call, as in the reference (src/algorithms/flash_attention.cpp:169-173)
        const double wall_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - wall0).count();
        impl_->profile.emplace_back("backward_pass", wall_ms);
        impl_->profile.emplace_back("backward_kernel_ms", timer.elapsed_ms());
    }
}

void FlashAttention::backward_varlen(const TensorShape& shape, const void* go, const void* q, const void* k, const void* v,
                                     void* gq, void* gk, void* gv, const int32_t* cu_seqlens, size_t n_seqs) {
    if (!impl_->configured)
        throw AttentionException(AttentionError::INVALID_PARAMETERS, "FlashAttention not configured. Call configure() first.");
    if (!go || !q || !k || !v || !gq || !gk || !gv || !cu_seqlens) throw AttentionException(AttentionError::INVALID_INPUT, "null pointer");
    const size_t H = current_params_.num_heads, d = current_params_.head_dimension;
    if (shape.dimensions.size() != 3 || shape.dimensions[1] != H || shape.dimensions[2] != d || n_seqs == 0)
        throw AttentionException(AttentionError::INVALID_INPUT, "packed tensors must be [total_tokens, heads, head_dim]");
    int64_t max_len = 0;
    if (cu_seqlens[0] != 0) throw AttentionException(AttentionError::INVALID_INPUT, "cu_seqlens must start at 0");
    for (size_t i = 0; i < n_seqs; ++i) {
        const int64_t len = (int64_t)cu_seqlens[i + 1] - cu_seqlens[i];
        if (len < 0) throw AttentionException(AttentionError::INVALID_INPUT, "cu_seqlens must not decrease");
        max_len = std::max(max_len, len);
    }
    if ((size_t)cu_seqlens[n_seqs] != shape.dimensions[0])
        throw AttentionException(AttentionError::INVALID_INPUT, "cu_seqlens must end at total_tokens");
    if (max_len == 0) return;
    void* st = impl_->stream.get();
    const size_t Hkv = kv_heads(current_params_);
    const size_t bytes = shape.total_bytes(), kv_bytes = bytes / H * Hkv;
    const void* d_go = stage_in(go, bytes, impl_->ddo, st);
    const void* d_q = stage_in(q, bytes, impl_->dq, st);
    const void* d_k = stage_in(k, kv_bytes, impl_->dk, st);
    const void* d_v = stage_in(v, kv_bytes, impl_->dv, st);
    const bool gq_dev = hipsup::is_device_pointer(gq), gk_dev = hipsup::is_device_pointer(gk), gv_dev = hipsup::is_device_pointer(gv);
    void* d_gq = gq_dev ? gq : impl_->gq.reserve(bytes);
    void* d_gk = gk_dev ? gk : impl_->gk.reserve(kv_bytes);
    void* d_gv = gv_dev ? gv : impl_->gv.reserve(kv_bytes);
    void* dcu = impl_->dcu.reserve((n_seqs + 1) * sizeof(int32_t));
    check(ahpc_hip_memcpy_h2d(dcu, cu_seqlens, (n_seqs + 1) * sizeof(int32_t), st), "copy cu_seqlens");
    const size_t ws_bytes = ahpc_hip_flash_bwd_workspace_bytes((int64_t)n_seqs, max_len, (int64_t)H);
    void* ws = impl_->ws.reserve(ws_bytes);
    float scale = impl_->cfg.softmax_scale > 0.0f ? impl_->cfg.softmax_scale : current_params_.scale_factor;
    if (!(scale > 0.0f)) scale = 1.0f / std::sqrt(static_cast<float>(d));
    const int causal = (current_params_.causal_mask || impl_->cfg.use_causal_mask) ? 1 : 0;
    check(ahpc_hip_flash_bwd_varlen(d_go, d_q, d_k, d_v, d_gq, d_gk, d_gv, hipsup::dtype_code(shape.data_type),
                                    static_cast<const int32_t*>(dcu), (int64_t)n_seqs, max_len, (int64_t)H, (int64_t)Hkv,
                                    (int64_t)d, (int64_t)(H * d), (int64_t)d, (int64_t)(Hkv * d), (int64_t)d, scale, causal, ws,
                                    ws_bytes, st), "flash backward (ragged)");
    if (!gq_dev) check(ahpc_hip_memcpy_d2h(gq, d_gq, bytes, st), "copy from device");
    if (!gk_dev) check(ahpc_hip_memcpy_d2h(gk, d_gk, kv_bytes, st), "copy from device");
    if (!gv_dev) check(ahpc_hip_memcpy_d2h(gv, d_gv, kv_bytes, st), "copy from device");
    impl_->stream.sync();
}

// Device bytes this object stages when every tensor arrives in host memory (nothing when they are
// already on the device).  Reference: FlashAttention::get_workspace_size,
// src/algorithms/flash_attention.cpp:176-199, whose fp32 conversion buffers have no counterpart here.
size_t FlashAttention::get_workspace_size(const AttentionParams& p) const {
    return 4 * p.batch_size * p.sequence_length * p.num_heads * p.head_dimension * sizeof(float);
}

void FlashAttention::set_workspace(void* workspace_ptr, size_t workspace_size) {
    workspace_ptr_ = workspace_ptr;   // kept for API compatibility; the forward kernel needs no scratch
    workspace_size_ = workspace_size;
}

bool FlashAttention::supports_data_type(DataType t) const {
    return t == DataType::FLOAT32 || t == DataType::FLOAT16 || t == DataType::BFLOAT16;
}
bool FlashAttention::supports_memory_layout(MemoryLayout layout) const { return layout == MemoryLayout::ROW_MAJOR; }
std::string FlashAttention::get_backend_name() const { return "HIP_FlashAttention"; }
std::string FlashAttention::get_version() const { return "1.0.0"; }

void FlashAttention::enable_profiling(bool enable) {
    profiling_enabled_ = enable;
    if (!enable) impl_->profile.clear();
}
std::vector<std::pair<std::string, double>> FlashAttention::get_profiling_results() const { return impl_->profile; }
void FlashAttention::reset_profiling() { impl_->profile.clear(); }

}  // namespace attention_hpc
