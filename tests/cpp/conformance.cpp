// Conformance suite for the C++ host classes, written after the reference's own gtest files
// (tests/test_flash_attention.cpp, tests/test_backends.cpp) and its decode example
// (examples/basic_usage.cpp:115-200): same fixtures, same tolerances, same expectations, with the CPU
// oracle (oracle/oracle.h) as the expected value.  gtest is not available, so a few macros stand in.
//
//   ahpc_conformance            all cases (needs a GPU)
//   ahpc_conformance --no-gpu   only the cases that never touch a device
//   ahpc_conformance <filter>   cases whose name contains <filter>
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <atomic>
#include <chrono>
#include <thread>
#include <vector>

#include "algorithms/flash_attention.hpp"
#include "algorithms/paged_attention.hpp"
#include "api/backend_factory.hpp"
#include "api/tensor.hpp"
#include "ahpc_hip.h"
#include "memory/kv_block_pool.hpp"
#include "oracle.h"

using namespace attention_hpc;

// ---- tiny harness --------------------------------------------------------------------------------
struct Case {
    const char* name;
    bool needs_gpu;
    std::function<void()> fn;
};
static std::vector<Case>& cases() {
    static std::vector<Case> c;
    return c;
}
static int g_failures = 0;
struct Registrar {
    Registrar(const char* n, bool gpu, std::function<void()> f) { cases().push_back({n, gpu, std::move(f)}); }
};
#define CASE(name, gpu)                                \
    static void case_##name();                         \
    static Registrar reg_##name(#name, gpu, case_##name); \
    static void case_##name()
#define EXPECT(cond)                                                              \
    do {                                                                          \
        if (!(cond)) {                                                            \
            std::printf("    EXPECT failed %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            ++g_failures;                                                         \
        }                                                                         \
    } while (0)
#define EXPECT_THROWS(stmt, code)                                                                  \
    do {                                                                                           \
        bool thrown = false;                                                                       \
        try {                                                                                      \
            stmt;                                                                                  \
        } catch (const AttentionException& e) {                                                    \
            thrown = true;                                                                         \
            if (e.error_code() != (code)) {                                                        \
                std::printf("    wrong error code %d at %s:%d\n", (int)e.error_code(), __FILE__, __LINE__); \
                ++g_failures;                                                                      \
            }                                                                                      \
        }                                                                                          \
        if (!thrown) {                                                                             \
            std::printf("    expected AttentionException at %s:%d\n", __FILE__, __LINE__);         \
            ++g_failures;                                                                          \
        }                                                                                          \
    } while (0)
#define EXPECT_THROWS_ANY(stmt)                                                            \
    do {                                                                                   \
        bool thrown = false;                                                               \
        try {                                                                              \
            stmt;                                                                          \
        } catch (const AttentionException&) {                                              \
            thrown = true;                                                                 \
        }                                                                                  \
        if (!thrown) {                                                                     \
            std::printf("    expected AttentionException at %s:%d\n", __FILE__, __LINE__); \
            ++g_failures;                                                                  \
        }                                                                                  \
    } while (0)

static std::vector<float> uniform(size_t n, uint64_t seed, uint64_t id, float lo = -1.0f, float hi = 1.0f) {
    std::vector<float> v(n);
    ahpc_oracle_fill_uniform(v.data(), n, seed, id, lo, hi);
    return v;
}
static std::vector<float> normal(size_t n, uint64_t seed, uint64_t id, float sigma = 1.0f) {
    std::vector<float> v(n);
    ahpc_oracle_fill_normal(v.data(), n, seed, id, sigma);
    return v;
}
static float max_abs_diff(const std::vector<float>& a, const std::vector<float>& b) {
    float m = a.size() == b.size() ? 0.0f : INFINITY;
    for (size_t i = 0; i < a.size() && i < b.size(); ++i) m = std::max(m, std::fabs(a[i] - b[i]));
    return m;
}
static std::vector<float> oracle_bnhd(const std::vector<float>& q, const std::vector<float>& k, const std::vector<float>& v,
                                      size_t B, size_t N, size_t H, size_t d, float scale, bool causal,
                                      const float* mask = nullptr) {
    std::vector<float> out(q.size(), 0.0f);
    ahpc_oracle_attention(q.data(), k.data(), v.data(), out.data(), B, N, H, d, N * H * d, H * d, d, scale, causal, mask, 4);
    return out;
}
static TensorShape shape4(size_t B, size_t N, size_t H, size_t d, DataType t = DataType::FLOAT32) {
    return TensorShape({B, N, H, d}, t);
}

// fixture of tests/test_flash_attention.cpp:103-108
static AttentionParams fixture_params() {
    AttentionParams p{};
    p.batch_size = 2;
    p.sequence_length = 16;
    p.num_heads = 4;
    p.head_dimension = 64;
    p.causal_mask = false;
    p.scale_factor = 1.0f / std::sqrt(64.0f);
    return p;
}

static float run_flash_and_compare(FlashAttention& fa, const AttentionParams& p, uint64_t seed) {
    const size_t B = p.batch_size, N = p.sequence_length, H = p.num_heads, d = p.head_dimension, n = B * N * H * d;
    auto q = uniform(n, seed, 1), k = uniform(n, seed, 2), v = uniform(n, seed, 3);
    std::vector<float> out(n, 0.0f);
    const TensorShape s = shape4(B, N, H, d);
    fa.forward(s, q.data(), s, k.data(), s, v.data(), s, out.data());
    return max_abs_diff(out, oracle_bnhd(q, k, v, B, N, H, d, p.scale_factor, p.causal_mask));
}

// ---- tests/test_flash_attention.cpp ---------------------------------------------------------------
CASE(Flash_ForwardPassSmallInput, true) {  // :141-175, tolerance 1e-4
    FlashAttention fa;
    AttentionParams p = fixture_params();
    fa.configure(p);
    EXPECT(run_flash_and_compare(fa, p, 1) <= 1e-4f);
}

CASE(Flash_CausalMaskTest, true) {  // :178-215: params.causal_mask = true must act
    FlashAttention fa;
    AttentionParams p = fixture_params();
    p.causal_mask = true;
    fa.configure(p);
    EXPECT(run_flash_and_compare(fa, p, 2) <= 1e-4f);
}

CASE(Flash_DifferentSequenceLengths, true) {  // :218-260
    FlashAttention fa;
    for (size_t N : {1u, 4u, 32u, 128u}) {
        AttentionParams p = fixture_params();
        p.sequence_length = N;
        fa.configure(p);
        EXPECT(run_flash_and_compare(fa, p, 3 + N) <= 1e-4f);
    }
}

CASE(Flash_DifferentHeadDimensions, true) {  // :263-307, tolerance max(1e-4, 1e-5*sqrt(d))
    FlashAttention fa;
    for (size_t d : {16u, 32u, 64u, 128u}) {
        AttentionParams p = fixture_params();
        p.head_dimension = d;
        p.scale_factor = 1.0f / std::sqrt((float)d);
        fa.configure(p);
        EXPECT(run_flash_and_compare(fa, p, 10 + d) <= std::max(1e-4f, 1e-5f * std::sqrt((float)d)));
    }
}

CASE(Flash_InvalidInputs, true) {  // :310-357
    FlashAttention fa;
    AttentionParams p = fixture_params();
    fa.configure(p);
    const size_t n = 2 * 16 * 4 * 64;
    auto q = uniform(n, 5, 1), k = uniform(n, 5, 2), v = uniform(n, 5, 3);
    std::vector<float> out(n);
    const TensorShape ok = shape4(2, 16, 4, 64);
    EXPECT_THROWS_ANY(fa.forward(shape4(2, 16, 4, 74), q.data(), ok, k.data(), ok, v.data(), ok, out.data()));
    EXPECT_THROWS_ANY(fa.forward(shape4(3, 16, 4, 64), q.data(), ok, k.data(), ok, v.data(), ok, out.data()));
    EXPECT_THROWS_ANY(fa.forward(ok, nullptr, ok, k.data(), ok, v.data(), ok, out.data()));
    EXPECT(fa.validate_inputs(shape4(2, 16, 4, 74), ok, ok, ok, p) == AttentionError::INVALID_INPUT);
    EXPECT(fa.validate_inputs(ok, ok, ok, ok, p) == AttentionError::SUCCESS);
    EXPECT_THROWS_ANY(fa.safe_forward(ok, q.data(), ok, k.data(), shape4(2, 16, 5, 64), v.data(), ok, out.data()));
}

CASE(Flash_DifferentBlockSizes, true) {  // :360-402: result must not depend on the block sizes
    FlashAttention fa;
    AttentionParams p = fixture_params();
    FlashAttentionConfig c;
    c.block_size_q = 32;
    c.block_size_k = 32;
    fa.configure(p);
    fa.configure_flash_attention(c);
    EXPECT(run_flash_and_compare(fa, p, 6) <= 1e-4f);
}

CASE(Flash_BackwardPass, true) {  // :405-480 (forward, then backward; the reference only asks for non-zero gradients)
    FlashAttention fa;
    AttentionParams p = fixture_params();
    fa.configure(p);
    const size_t B = p.batch_size, N = p.sequence_length, H = p.num_heads, d = p.head_dimension, n = B * N * H * d;
    auto q = uniform(n, 11, 1), k = uniform(n, 11, 2), v = uniform(n, 11, 3);
    auto go = uniform(n, 11, 7, 0.01f, 0.1f);  // as in the reference's test
    std::vector<float> out(n), gq(n, 0.0f), gk(n, 0.0f), gv(n, 0.0f);
    const TensorShape s = shape4(B, N, H, d);
    fa.forward(s, q.data(), s, k.data(), s, v.data(), s, out.data());
    fa.backward(s, go.data(), s, q.data(), s, k.data(), s, v.data(), s, gq.data(), s, gk.data(), s, gv.data());
    auto nonzero = [](const std::vector<float>& x) {
        for (float e : x)
            if (std::fabs(e) > 1e-6f) return true;
        return false;
    };
    EXPECT(nonzero(gq) && nonzero(gk) && nonzero(gv));  // :449-478
    std::vector<float> wq(n), wk(n), wv(n);
    ahpc_oracle_attention_backward(q.data(), k.data(), v.data(), go.data(), wq.data(), wk.data(), wv.data(), B, N, H, H, d,
                                   p.scale_factor, 0, nullptr, 4);
    EXPECT(max_abs_diff(gq, wq) <= 1e-4f && max_abs_diff(gk, wk) <= 1e-4f && max_abs_diff(gv, wv) <= 1e-4f);
}

CASE(Flash_BackwardCausalGroupedHalf, true) {  // bf16 tensors, causal, 4 query heads over 2 K/V heads: the matrix-core kernels
    FlashAttention fa;
    AttentionParams p = fixture_params();
    p.sequence_length = 200;
    p.head_dimension = 128;
    p.key_value_heads = 2;
    p.causal_mask = true;
    p.scale_factor = 1.0f / std::sqrt(128.0f);
    fa.configure(p);
    const size_t B = p.batch_size, N = p.sequence_length, H = p.num_heads, Hkv = 2, d = p.head_dimension;
    const size_t n = B * N * H * d, nkv = B * N * Hkv * d;
    auto q = uniform(n, 12, 1), k = uniform(nkv, 12, 2), v = uniform(nkv, 12, 3), go = uniform(n, 12, 7);
    auto to_bf16 = [](std::vector<float>& x) {
        std::vector<bfloat16> y(x.size());
        for (size_t i = 0; i < x.size(); ++i) {
            y[i] = bfloat16(x[i]);
            x[i] = static_cast<float>(y[i]);  // the oracle sees the rounded values
        }
        return y;
    };
    auto hq = to_bf16(q), hk = to_bf16(k), hv = to_bf16(v), hgo = to_bf16(go);
    std::vector<bfloat16> gq(n), gk(nkv), gv(nkv);
    const TensorShape s = shape4(B, N, H, d, DataType::BFLOAT16), skv = shape4(B, N, Hkv, d, DataType::BFLOAT16);
    fa.backward(s, hgo.data(), s, hq.data(), skv, hk.data(), skv, hv.data(), s, gq.data(), skv, gk.data(), skv, gv.data());
    std::vector<float> wq(n), wk(nkv), wv(nkv);
    ahpc_oracle_attention_backward(q.data(), k.data(), v.data(), go.data(), wq.data(), wk.data(), wv.data(), B, N, H, Hkv, d,
                                   p.scale_factor, 1, nullptr, 4);
    auto close = [](const std::vector<bfloat16>& got, const std::vector<float>& want) {
        float top = 1.0f, worst = 0.0f;
        for (float w : want) top = std::max(top, std::fabs(w));
        for (size_t i = 0; i < want.size(); ++i) worst = std::max(worst, std::fabs(static_cast<float>(got[i]) - want[i]));
        return worst <= 2e-2f * top;
    };
    EXPECT(close(gq, wq) && close(gk, wk) && close(gv, wv));
    // wrong gradient shape is refused
    EXPECT_THROWS(fa.backward(s, hgo.data(), s, hq.data(), skv, hk.data(), skv, hv.data(), s, gq.data(), s, gk.data(), skv, gv.data()),
                  AttentionError::INVALID_INPUT);
}

CASE(Flash_BackwardDenseMaskHalfWideHeads, true) {  // fp16 tensors, head dimension 192, dense mask: matrix-core kernels on the packed mask
    FlashAttention fa;
    AttentionParams p = fixture_params();
    p.sequence_length = 90;
    p.head_dimension = 192;
    p.scale_factor = 1.0f / std::sqrt(192.0f);
    fa.configure(p);
    const size_t B = p.batch_size, N = p.sequence_length, H = p.num_heads, d = p.head_dimension, n = B * N * H * d;
    auto q = uniform(n, 14, 1), k = uniform(n, 14, 2), v = uniform(n, 14, 3), go = uniform(n, 14, 7);
    auto to_f16 = [](std::vector<float>& x) {
        std::vector<half> y(x.size());
        for (size_t i = 0; i < x.size(); ++i) {
            y[i] = half(x[i]);
            x[i] = static_cast<float>(y[i]);  // the oracle sees the rounded values
        }
        return y;
    };
    auto hq = to_f16(q), hk = to_f16(k), hv = to_f16(v), hgo = to_f16(go);
    std::vector<float> mask = uniform(B * N * N, 14, 6, 0.0f, 1.0f);
    for (float& m : mask) m = m > 0.4f ? 1.0f : 0.0f;
    for (size_t j = 0; j < N; ++j) mask[(0 * N + 70) * N + j] = 0.0f;  // a query that sees nothing
    for (size_t i = 0; i < N; ++i) mask[(0 * N + i) * N + 33] = 0.0f;  // a key that nobody sees
    std::vector<half> gq(n), gk(n), gv(n);
    const TensorShape s = shape4(B, N, H, d, DataType::FLOAT16);
    fa.backward(s, hgo.data(), s, hq.data(), s, hk.data(), s, hv.data(), s, gq.data(), s, gk.data(), s, gv.data(), mask.data());
    std::vector<float> wq(n), wk(n), wv(n);
    ahpc_oracle_attention_backward(q.data(), k.data(), v.data(), go.data(), wq.data(), wk.data(), wv.data(), B, N, H, H, d,
                                   p.scale_factor, 0, mask.data(), 4);
    auto close = [](const std::vector<half>& got, const std::vector<float>& want) {
        float top = 1.0f, worst = 0.0f;
        for (float w : want) top = std::max(top, std::fabs(w));
        for (size_t i = 0; i < want.size(); ++i) worst = std::max(worst, std::fabs(static_cast<float>(got[i]) - want[i]));
        return worst <= 2e-2f * top;
    };
    EXPECT(close(gq, wq) && close(gk, wk) && close(gv, wv));
    bool dead_query = true, dead_key = true;
    for (size_t h = 0; h < H; ++h)
        for (size_t e = 0; e < d; ++e) {
            dead_query = dead_query && static_cast<float>(gq[((0 * N + 70) * H + h) * d + e]) == 0.0f;
            dead_key = dead_key && static_cast<float>(gk[((0 * N + 33) * H + h) * d + e]) == 0.0f &&
                       static_cast<float>(gv[((0 * N + 33) * H + h) * d + e]) == 0.0f;
        }
    EXPECT(dead_query && dead_key);
}

CASE(Flash_BackwardOnKeptForwardStatistics, true) {  // keep_forward_statistics: backward() of the last forward() skips its statistics pass
    FlashAttention fa;
    AttentionParams p = fixture_params();
    p.sequence_length = 160;
    p.head_dimension = 128;
    p.causal_mask = true;
    p.scale_factor = 1.0f / std::sqrt(128.0f);
    fa.configure(p);
    FlashAttentionConfig c;
    c.keep_forward_statistics = true;
    fa.configure_flash_attention(c);
    const size_t B = p.batch_size, N = p.sequence_length, H = p.num_heads, d = p.head_dimension, n = B * N * H * d;
    auto q = uniform(n, 15, 1), k = uniform(n, 15, 2), v = uniform(n, 15, 3), go = uniform(n, 15, 7);
    auto to_bf16 = [](std::vector<float>& x) {
        std::vector<bfloat16> y(x.size());
        for (size_t i = 0; i < x.size(); ++i) {
            y[i] = bfloat16(x[i]);
            x[i] = static_cast<float>(y[i]);
        }
        return y;
    };
    auto hq = to_bf16(q), hk = to_bf16(k), hv = to_bf16(v), hgo = to_bf16(go);
    std::vector<bfloat16> out(n), gq(n), gk(n), gv(n), gq2(n), gk2(n), gv2(n);
    const TensorShape s = shape4(B, N, H, d, DataType::BFLOAT16);
    fa.forward(s, hq.data(), s, hk.data(), s, hv.data(), s, out.data());
    fa.backward(s, hgo.data(), s, hq.data(), s, hk.data(), s, hv.data(), s, gq.data(), s, gk.data(), s, gv.data());
    std::vector<float> wq(n), wk(n), wv(n);
    ahpc_oracle_attention_backward(q.data(), k.data(), v.data(), go.data(), wq.data(), wk.data(), wv.data(), B, N, H, H, d,
                                   p.scale_factor, 1, nullptr, 4);
    auto close = [](const std::vector<bfloat16>& got, const std::vector<float>& want) {
        float top = 1.0f, worst = 0.0f;
        for (float w : want) top = std::max(top, std::fabs(w));
        for (size_t i = 0; i < want.size(); ++i) worst = std::max(worst, std::fabs(static_cast<float>(got[i]) - want[i]));
        return worst <= 2e-2f * top;
    };
    EXPECT(close(gq, wq) && close(gk, wk) && close(gv, wv));
    // a backward for other tensors (another query pointer) must not use what the forward kept: same values, new address
    std::vector<bfloat16> hq_copy = hq;
    fa.backward(s, hgo.data(), s, hq_copy.data(), s, hk.data(), s, hv.data(), s, gq2.data(), s, gk2.data(), s, gv2.data());
    EXPECT(close(gq2, wq) && close(gk2, wk) && close(gv2, wv));
}

CASE(Flash_BackwardRaggedBatch, true) {  // packed sequences: each one's gradients equal the dense oracle's on it
    FlashAttention fa;
    AttentionParams p = fixture_params();
    p.causal_mask = true;
    fa.configure(p);
    const size_t H = p.num_heads, d = p.head_dimension;
    const std::vector<int32_t> cu = {0, 5, 5, 140, 141};  // lengths 5, 0, 135, 1
    const size_t T = 141, n = T * H * d;
    auto q = uniform(n, 13, 1), k = uniform(n, 13, 2), v = uniform(n, 13, 3), go = uniform(n, 13, 7);
    std::vector<float> gq(n, 9.0f), gk(n, 9.0f), gv(n, 9.0f);
    const TensorShape s({T, H, d}, DataType::FLOAT32);
    fa.backward_varlen(s, go.data(), q.data(), k.data(), v.data(), gq.data(), gk.data(), gv.data(), cu.data(), cu.size() - 1);
    for (size_t i = 0; i + 1 < cu.size(); ++i) {
        const size_t a = (size_t)cu[i] * H * d, len = (size_t)(cu[i + 1] - cu[i]), m = len * H * d;
        if (!len) continue;
        std::vector<float> wq(m), wk(m), wv(m);
        ahpc_oracle_attention_backward(q.data() + a, k.data() + a, v.data() + a, go.data() + a, wq.data(), wk.data(), wv.data(), 1,
                                       len, H, H, d, p.scale_factor, 1, nullptr, 4);
        EXPECT(max_abs_diff(std::vector<float>(gq.begin() + a, gq.begin() + a + m), wq) <= 1e-4f);
        EXPECT(max_abs_diff(std::vector<float>(gk.begin() + a, gk.begin() + a + m), wk) <= 1e-4f);
        EXPECT(max_abs_diff(std::vector<float>(gv.begin() + a, gv.begin() + a + m), wv) <= 1e-4f);
    }
}

CASE(Flash_AttentionMask, true) {  // :483-582: mask [B,N,N] float, 0 = masked
    FlashAttention fa;
    AttentionParams p = fixture_params();
    fa.configure(p);
    const size_t B = 2, N = 16, H = 4, d = 64, n = B * N * H * d;
    auto q = uniform(n, 7, 1), k = uniform(n, 7, 2), v = uniform(n, 7, 3);
    std::vector<float> mask(B * N * N, 1.0f);
    for (size_t b = 0; b < B; ++b)
        for (size_t i = 0; i < N; ++i)
            for (size_t j = 0; j < N; ++j)
                if ((i + 2 * j + b) % 3 == 0) mask[(b * N + i) * N + j] = 0.0f;
    std::vector<float> out(n);
    const TensorShape s = shape4(B, N, H, d);
    fa.forward(s, q.data(), s, k.data(), s, v.data(), s, out.data(), mask.data());
    EXPECT(max_abs_diff(out, oracle_bnhd(q, k, v, B, N, H, d, p.scale_factor, false, mask.data())) <= 1e-4f);
}

CASE(Flash_SingleToken, true) {  // :585-599: N = 1 => output = value
    FlashAttention fa;
    AttentionParams p = fixture_params();
    p.sequence_length = 1;
    fa.configure(p);
    const size_t n = 2 * 1 * 4 * 64;
    auto q = uniform(n, 8, 1), k = uniform(n, 8, 2), v = uniform(n, 8, 3);
    std::vector<float> out(n);
    const TensorShape s = shape4(2, 1, 4, 64);
    fa.forward(s, q.data(), s, k.data(), s, v.data(), s, out.data());
    EXPECT(max_abs_diff(out, v) <= 1e-6f);
}

CASE(Flash_LayoutSwitchAndScaleOverride, true) {
    // tensors indexed [B,H,N,d] as the reference oracle does (tests/test_flash_attention.cpp:46);
    // FlashAttentionConfig::softmax_scale overrides AttentionParams::scale_factor
    FlashAttention fa;
    AttentionParams p = fixture_params();
    p.causal_mask = true;
    fa.configure(p);
    FlashAttentionConfig c;
    c.tensor_layout_bhnd = true;
    c.softmax_scale = 0.2f;
    fa.configure_flash_attention(c);
    const size_t B = 2, N = 16, H = 4, d = 64, n = B * N * H * d;
    auto q = uniform(n, 9, 1), k = uniform(n, 9, 2), v = uniform(n, 9, 3);
    std::vector<float> out(n), want(n);
    const TensorShape s = shape4(B, N, H, d);
    fa.forward(s, q.data(), s, k.data(), s, v.data(), s, out.data());
    ahpc_oracle_attention(q.data(), k.data(), v.data(), want.data(), B, N, H, d, H * N * d, d, N * d, 0.2f, 1, nullptr, 1);
    EXPECT(max_abs_diff(out, want) <= 1e-4f);
}

template <typename T> static std::vector<T> to_storage(const std::vector<float>& x) {
    std::vector<T> y(x.size());
    for (size_t i = 0; i < x.size(); ++i) y[i] = T(x[i]);
    return y;
}
template <typename T> static std::vector<float> from_storage(const std::vector<T>& x) {
    std::vector<float> y(x.size());
    for (size_t i = 0; i < x.size(); ++i) y[i] = (float)x[i];
    return y;
}

template <typename T> static void flash_16bit(size_t d, bool causal) {
    FlashAttention fa;
    AttentionParams p{};
    p.batch_size = 2; p.sequence_length = 200; p.num_heads = 3; p.head_dimension = d; p.causal_mask = causal;
    fa.configure(p);
    const size_t n = 2 * 200 * 3 * d;
    auto qs = to_storage<T>(normal(n, 11, 1)), ks = to_storage<T>(normal(n, 11, 2)), vs = to_storage<T>(normal(n, 11, 3));
    std::vector<T> out(n);
    const TensorShape s = shape4(2, 200, 3, d, DataTypeOf<T>::value);
    fa.forward(s, qs.data(), s, ks.data(), s, vs.data(), s, out.data());
    auto want = oracle_bnhd(from_storage(qs), from_storage(ks), from_storage(vs), 2, 200, 3, d, 1.0f / std::sqrt((float)d), causal);
    EXPECT(max_abs_diff(from_storage(out), want) <= 2e-2f);
}
CASE(Flash_HalfAndBfloat16HostTensors, true) {
    flash_16bit<half>(64, true);
    flash_16bit<half>(128, false);
    flash_16bit<bfloat16>(128, true);
    flash_16bit<bfloat16>(64, false);
}

CASE(Flash_VarlenPackedBatch, true) {
    FlashAttention fa;
    AttentionParams p{};
    p.batch_size = 4; p.sequence_length = 70; p.num_heads = 2; p.head_dimension = 64; p.causal_mask = true;
    fa.configure(p);
    const int32_t cu[5] = {0, 7, 77, 78, 130};
    const size_t T = 130, H = 2, d = 64, n = T * H * d;
    auto qs = to_storage<half>(normal(n, 12, 1, 0.5f)), ks = to_storage<half>(normal(n, 12, 2, 0.5f)), vs = to_storage<half>(normal(n, 12, 3, 0.5f));
    std::vector<half> out(n);
    fa.forward_varlen(TensorShape({T, H, d}, DataType::FLOAT16), qs.data(), ks.data(), vs.data(), out.data(), cu, 4);
    std::vector<float> want(n);
    auto qf = from_storage(qs), kf = from_storage(ks), vf = from_storage(vs);
    ahpc_oracle_attention_varlen(qf.data(), kf.data(), vf.data(), want.data(), cu, 4, H, d, 0.125f, 1, 2);
    EXPECT(max_abs_diff(from_storage(out), want) <= 2e-2f);
    const int32_t bad[5] = {0, 7, 5, 78, 130};
    EXPECT_THROWS(fa.forward_varlen(TensorShape({T, H, d}, DataType::FLOAT16), qs.data(), ks.data(), vs.data(), out.data(), bad, 4),
                  AttentionError::INVALID_INPUT);
}

CASE(Flash_ProfilingResults, true) {  // enable_profiling / get_profiling_results / reset_profiling
    FlashAttention fa;
    AttentionParams p = fixture_params();
    fa.configure(p);
    fa.enable_profiling(true);
    run_flash_and_compare(fa, p, 13);
    auto r = fa.get_profiling_results();
    EXPECT(!r.empty() && r[0].first == "forward_pass" && r[0].second > 0.0);
    fa.reset_profiling();
    EXPECT(fa.get_profiling_results().empty());
    fa.enable_profiling(false);
    run_flash_and_compare(fa, p, 13);
    EXPECT(fa.get_profiling_results().empty());
}

// ---- configuration errors (no device work) ------------------------------------------------------------
CASE(Flash_UnconfiguredAndBadParameters, false) {  // src/algorithms/flash_attention.cpp:37-41, :74-77
    FlashAttention fa;
    const TensorShape s = shape4(2, 16, 4, 64);
    std::vector<float> x(2 * 16 * 4 * 64);
    EXPECT_THROWS(fa.forward(s, x.data(), s, x.data(), s, x.data(), s, x.data()), AttentionError::INVALID_PARAMETERS);
    AttentionParams p = fixture_params();
    p.num_heads = 0;
    EXPECT_THROWS(fa.configure(p), AttentionError::INVALID_PARAMETERS);
    p = fixture_params();
    p.key_value_heads = 3;  // does not divide the four query heads
    EXPECT_THROWS(fa.configure(p), AttentionError::INVALID_PARAMETERS);
    EXPECT(fa.get_backend_name() == "HIP_FlashAttention");
    EXPECT(fa.get_version() == "1.0.0");
    EXPECT(fa.supports_data_type(DataType::FLOAT32) && fa.supports_data_type(DataType::BFLOAT16));
    EXPECT(fa.supports_memory_layout(MemoryLayout::ROW_MAJOR) && !fa.supports_memory_layout(MemoryLayout::COLUMN_MAJOR));
    PagedAttention pa;
    EXPECT_THROWS(pa.create_sequence(16), AttentionError::INVALID_PARAMETERS);
    EXPECT(pa.get_backend_name() == "HIP_PagedAttention");
}

CASE(Types_HalfAndBfloat16MatchOracleBitForBit, false) {
    for (uint32_t i = 0; i < 65536; ++i) {
        half h;
        h.data = (uint16_t)i;
        const float f = (float)h, g = ahpc_oracle_f16_to_f32((uint16_t)i);
        EXPECT(std::memcmp(&f, &g, 4) == 0 || (std::isnan(f) && std::isnan(g)));
        bfloat16 b;
        b.data = (uint16_t)i;
        const float fb = (float)b, gb = ahpc_oracle_bf16_to_f32((uint16_t)i);
        EXPECT(std::memcmp(&fb, &gb, 4) == 0 || (std::isnan(fb) && std::isnan(gb)));
        if (g_failures) return;
    }
    uint64_t z = 88172645463325252ull;
    for (int i = 0; i < 400000; ++i) {
        z ^= z << 13; z ^= z >> 7; z ^= z << 17;
        uint32_t u = (uint32_t)z;
        float f;
        std::memcpy(&f, &u, 4);
        EXPECT(half(f).data == ahpc_oracle_f32_to_f16(f) || std::isnan(f));
        EXPECT(bfloat16(f).data == ahpc_oracle_f32_to_bf16(f) || std::isnan(f));
        if (g_failures) return;
    }
    EXPECT(half(65520.0f).data == 0x7C00 && half(65519.0f).data == 0x7BFF && half(1e-8f).data == 0);
    EXPECT(bfloat16(1.00390625f).data == 0x3F80 && bfloat16(1.01171875f).data == 0x3F82);  // ties to even
}

CASE(Merge_OnlineSoftmaxStateMatchesOracle, false) {  // src/algorithms/flash_attention.hpp:39-62
    OnlineSoftmaxState s;
    float m = -INFINITY, l = 0.0f;
    const float ms[5] = {0.3f, 2.0f, -1.0f, 2.0f, 5.5f}, ls[5] = {1.5f, 0.2f, 7.0f, 1.0f, 0.01f};
    for (int i = 0; i < 5; ++i) {
        s.update(ms[i], ls[i]);
        ahpc_oracle_softmax_merge(&m, &l, ms[i], ls[i]);
        EXPECT(s.max_val == m && s.sum_exp == l);
    }
    EXPECT(OnlineSoftmaxState{}.get_normalizer() == 0.0f);
}

// ---- tests/test_backends.cpp --------------------------------------------------------------------------------
CASE(Factory_NamesAndStrings, false) {
    EXPECT(BackendFactory::backendTypeToString(BackendType::HIP) == "HIP");
    EXPECT(BackendFactory::backendTypeToString(BackendType::CPU) == "CPU");
    EXPECT(BackendFactory::stringToBackendType("hip") == BackendType::HIP);
    EXPECT(BackendFactory::stringToBackendType("CUDA") == BackendType::CUDA);
    bool threw = false;
    try { BackendFactory::stringToBackendType("metal"); } catch (const std::invalid_argument&) { threw = true; }
    EXPECT(threw);
    EXPECT((int)BackendType::AUTO == 5 && (int)BackendType::HIP == 6);  // the reference's values are unchanged
    EXPECT(!BackendFactory::isBackendAvailable(BackendType::CUDA));
    EXPECT_THROWS(BackendFactory::createFlashAttention(BackendType::VULKAN), AttentionError::BACKEND_NOT_AVAILABLE);
    try {
        BackendFactory::createBackend(BackendType::OPENCL);
        EXPECT(false);
    } catch (const BackendException& e) {
        EXPECT(e.backend_type() == BackendType::OPENCL);
        EXPECT(std::string(e.what()).find("OpenCL") != std::string::npos);
    }
    BackendFactory::enableDebugMode(true);
    EXPECT(BackendFactory::isDebugModeEnabled());
    BackendFactory::enableDebugMode(false);
    EXPECT(!BackendFactory::getSystemInfo().empty());
}

// A plug-in CPU backend made of the oracle: exercises registerBackend, and is the second backend of the
// cross-backend consistency case.  It lives in the test, not in the library.
class OracleCpuAttention : public AttentionInterface {
public:
    void configure(const AttentionParams& p, const PerformanceConfig& c = PerformanceConfig{}) override { current_params_ = p; current_perf_config_ = c; ok_ = true; }
    void forward(const TensorShape& qs, const void* q, const TensorShape&, const void* k, const TensorShape&, const void* v,
                 const TensorShape&, void* o, const void* mask = nullptr) override {
        if (!ok_) throw AttentionException(AttentionError::INVALID_PARAMETERS, "not configured");
        if (!q || !k || !v || !o) throw AttentionException(AttentionError::INVALID_INPUT, "null");
        const size_t B = qs.dimensions[0], N = qs.dimensions[1], H = qs.dimensions[2], d = qs.dimensions[3];
        const float scale = current_params_.scale_factor > 0 ? current_params_.scale_factor : 1.0f / std::sqrt((float)d);
        ahpc_oracle_attention((const float*)q, (const float*)k, (const float*)v, (float*)o, B, N, H, d, N * H * d, H * d, d, scale,
                              current_params_.causal_mask, (const float*)mask, 2);
    }
    void backward(const TensorShape&, const void*, const TensorShape&, const void*, const TensorShape&, const void*, const TensorShape&,
                  const void*, const TensorShape&, void*, const TensorShape&, void*, const TensorShape&, void*, const void* = nullptr) override {
        throw AttentionException(AttentionError::UNSUPPORTED_OPERATION, "no backward");
    }
    size_t get_workspace_size(const AttentionParams&) const override { return 0; }
    void set_workspace(void*, size_t) override {}
    bool supports_data_type(DataType t) const override { return t == DataType::FLOAT32; }
    bool supports_memory_layout(MemoryLayout l) const override { return l == MemoryLayout::ROW_MAJOR; }
    std::string get_backend_name() const override { return "CPU_OracleAttention"; }
    std::string get_version() const override { return "test"; }
    void enable_profiling(bool) override {}
    std::vector<std::pair<std::string, double>> get_profiling_results() const override { return {}; }
    void reset_profiling() override {}
    AttentionError validate_inputs(const TensorShape&, const TensorShape&, const TensorShape&, const TensorShape&, const AttentionParams&) const override { return AttentionError::SUCCESS; }

private:
    bool ok_ = false;
};

CASE(Factory_PluginRegistration, false) {  // registerBackend / unregisterBackend, src/api/backend_factory.hpp:68-71
    EXPECT(!BackendFactory::isBackendAvailable(BackendType::CPU));
    BackendFactory::registerBackend(BackendType::CPU, "CPU", [] { return std::unique_ptr<AttentionInterface>(new OracleCpuAttention()); });
    EXPECT(BackendFactory::isBackendAvailable(BackendType::CPU));
    auto cpu = BackendFactory::createFlashAttention(BackendType::CPU);
    EXPECT(cpu && cpu->get_backend_name().find(BackendFactory::backendTypeToString(BackendType::CPU)) == 0);
    EXPECT_THROWS(BackendFactory::createPagedAttention(BackendType::CPU), AttentionError::BACKEND_NOT_AVAILABLE);
    EXPECT(BackendFactory::selectBestBackend(std::vector<BackendType>{BackendType::CUDA, BackendType::CPU}) == BackendType::CPU);
    BackendFactory::unregisterBackend(BackendType::CPU);
    EXPECT(!BackendFactory::isBackendAvailable(BackendType::CPU));
    EXPECT_THROWS(BackendFactory::createFlashAttention(BackendType::CPU), AttentionError::BACKEND_NOT_AVAILABLE);
}

CASE(Backends_AvailabilityAndCapability, true) {  // tests/test_backends.cpp:110-180
    auto avail = BackendFactory::getAvailableBackends();
    EXPECT(std::find(avail.begin(), avail.end(), BackendType::HIP) != avail.end());
    const BackendCapability cap = BackendFactory::getBackendCapability(BackendType::HIP);
    EXPECT(cap.available && !cap.version.empty() && !cap.device_name.empty());
    EXPECT(!cap.supported_data_types.empty() && !cap.supported_layouts.empty());
    EXPECT(cap.memory_size > (size_t)16 << 30 && cap.supports_tensor_cores);
    EXPECT(cap.compute_capability_major == 9 && cap.compute_capability_minor == 50);
    EXPECT(BackendFactory::selectBestBackend() == BackendType::HIP);
    EXPECT(BackendFactory::isBackendAvailable(BackendType::AUTO));
    AttentionParams p = fixture_params();
    EXPECT(BackendFactory::validateBackendCompatibility(BackendType::HIP, p));
    p.head_dimension = 1024;
    EXPECT(!BackendFactory::validateBackendCompatibility(BackendType::HIP, p));
}

CASE(Backends_CreationAndConfiguration, true) {  // tests/test_backends.cpp:183-247
    for (BackendType t : BackendFactory::getAvailableBackends()) {
        auto fa = BackendFactory::createFlashAttention(t);
        EXPECT(fa != nullptr);
        EXPECT(fa->get_backend_name().find(BackendFactory::backendTypeToString(t)) == 0);
        EXPECT(!fa->get_version().empty());
        EXPECT(fa->supports_data_type(DataType::FLOAT32));
        EXPECT(fa->supports_memory_layout(MemoryLayout::ROW_MAJOR));
        auto pa = BackendFactory::createPagedAttention(t);
        EXPECT(pa != nullptr && dynamic_cast<PagedAttention*>(pa.get()) != nullptr);
        AttentionParams p = fixture_params();
        fa->configure(p);
        (void)fa->get_workspace_size(p);
        fa->enable_profiling(true);
        fa->enable_profiling(false);
        const TensorShape s = shape4(2, 16, 4, 64);
        EXPECT(fa->validate_inputs(s, s, s, s, p) == AttentionError::SUCCESS);
    }
    auto any = BackendFactory::createFlashAttention(BackendType::AUTO);  // README.md:150 of the reference
    EXPECT(any && any->get_backend_name() == "HIP_FlashAttention");
}

CASE(Backends_CrossBackendConsistency, true) {  // tests/test_backends.cpp:252-324, tolerance 1e-3
    BackendFactory::registerBackend(BackendType::CPU, "CPU", [] { return std::unique_ptr<AttentionInterface>(new OracleCpuAttention()); });
    AttentionParams p = fixture_params();
    p.sequence_length = 64;
    const size_t n = 2 * 64 * 4 * 64;
    auto q = uniform(n, 21, 1), k = uniform(n, 21, 2), v = uniform(n, 21, 3);
    const TensorShape s = shape4(2, 64, 4, 64);
    std::vector<std::vector<float>> outs;
    for (BackendType t : BackendFactory::getAvailableBackends()) {
        auto a = BackendFactory::createFlashAttention(t);
        a->configure(p);
        outs.emplace_back(n, 0.0f);
        a->forward(s, q.data(), s, k.data(), s, v.data(), s, outs.back().data());
    }
    EXPECT(outs.size() >= 2);
    for (size_t i = 1; i < outs.size(); ++i) EXPECT(max_abs_diff(outs[0], outs[i]) <= 1e-3f);
    BackendFactory::unregisterBackend(BackendType::CPU);
}

CASE(Backends_ConcurrentInstancesAndLifecycles, true) {  // tests/test_backends.cpp:351-449
    std::vector<std::thread> th;
    std::vector<float> errs(4, 1.0f);
    for (int i = 0; i < 4; ++i)
        th.emplace_back([i, &errs] {
            auto a = BackendFactory::createFlashAttention(BackendType::HIP);
            AttentionParams p = fixture_params();
            a->configure(p);
            errs[i] = run_flash_and_compare(*static_cast<FlashAttention*>(a.get()), p, 30 + i);
        });
    for (auto& t : th) t.join();
    for (float e : errs) EXPECT(e <= 1e-4f);
    for (int cycle = 0; cycle < 3; ++cycle) {
        auto a1 = BackendFactory::createFlashAttention(BackendType::HIP);
        auto a2 = BackendFactory::createPagedAttention(BackendType::HIP);
        AttentionParams p = fixture_params();
        a1->configure(p);
        a2->configure(p);
    }
}

CASE(Backends_LargeInput, true) {  // tests/test_backends.cpp:474-516: B=8, N=256, H=8
    FlashAttention fa;
    AttentionParams p = fixture_params();
    p.batch_size = 8; p.sequence_length = 256; p.num_heads = 8;
    fa.configure(p);
    EXPECT(run_flash_and_compare(fa, p, 40) <= 1e-4f);
}

CASE(Backends_ErrorHandling, true) {  // tests/test_backends.cpp:631-680
    auto a = BackendFactory::createFlashAttention(BackendType::HIP);
    const TensorShape s = shape4(2, 16, 4, 64);
    std::vector<float> x(2 * 16 * 4 * 64, 0.5f), o(x.size());
    EXPECT_THROWS_ANY(a->forward(s, x.data(), s, x.data(), s, x.data(), s, o.data()));  // unconfigured
    a->configure(fixture_params());
    EXPECT_THROWS_ANY(a->forward(s, nullptr, s, x.data(), s, x.data(), s, o.data()));
    EXPECT_THROWS_ANY(a->forward(shape4(2, 16, 4, 32), x.data(), s, x.data(), s, x.data(), s, o.data()));
    TensorShape col = s;
    col.layout = MemoryLayout::COLUMN_MAJOR;
    EXPECT_THROWS(a->forward(col, x.data(), s, x.data(), s, x.data(), s, o.data()), AttentionError::UNSUPPORTED_OPERATION);
}

// ---- paged attention ------------------------------------------------------------------------------------------
CASE(Paged_BasicUsageFlow, true) {  // examples/basic_usage.cpp:115-200
    AttentionParams p{};
    p.batch_size = 1; p.sequence_length = 1; p.num_heads = 4; p.head_dimension = 32; p.max_sequence_length = 128;
    auto base = BackendFactory::createPagedAttention(BackendType::HIP);
    auto* pa = dynamic_cast<PagedAttention*>(base.get());
    EXPECT(pa != nullptr);
    pa->configure(p);
    const size_t id = pa->create_sequence(p.max_sequence_length);
    EXPECT(id == 1);  // ids start at 1, src/algorithms/paged_attention.cpp:67, :336
    const size_t L = 32, H = 4, d = 32;
    auto k = uniform(L * H * d, 50, 2), v = uniform(L * H * d, 50, 3), q = uniform(H * d, 50, 1);
    pa->append_kv_cache(id, k.data(), v.data(), L, DataType::FLOAT32);
    EXPECT(pa->get_sequence_length(id) == L && pa->is_sequence_active(id));
    std::vector<float> out(H * d, -1.0f);
    const TensorShape qs = shape4(1, 1, H, d);
    pa->forward_batch({id}, {qs}, {q.data()}, {qs}, {out.data()});
    // expected: dense attention of the last row with the query at position L-1 == decode over all L keys
    std::vector<float> want(H * d);
    const int32_t table[2] = {0, 1};
    const int32_t len = (int32_t)L;
    ahpc_oracle_paged_decode(q.data(), want.data(), k.data(), v.data(), table, &len, nullptr, 1, H, d, 16, 2, 1.0f / std::sqrt((float)d), 1);
    EXPECT(max_abs_diff(out, want) <= 1e-4f);
    pa->destroy_sequence(id);
    EXPECT(!pa->is_sequence_active(id) && pa->get_active_sequences_count() == 0);
    pa->destroy_sequence(id);  // unknown ids are ignored
}

CASE(Paged_PoolOrderMatchesFifoModel, true) {  // src/algorithms/paged_attention.cpp:11-64
    PagedAttention pa;
    AttentionParams p{};
    p.batch_size = 4; p.sequence_length = 1; p.num_heads = 2; p.head_dimension = 32; p.page_size = 4;
    PagedAttentionConfig c;
    c.initial_page_pool_size = 6;
    c.page_pool_growth = 3;
    pa.configure_paged_attention(c);
    pa.configure(p);
    ahpc_oracle_pool* model = ahpc_oracle_pool_create(6, 3);
    const size_t H = 2, d = 32;
    auto tok = [&](size_t n, uint64_t seed) { return uniform(n * H * d, seed, 2); };
    std::vector<std::vector<int32_t>> want(3);
    const size_t a = pa.create_sequence(64), b = pa.create_sequence(64), c3 = pa.create_sequence(64);
    auto append = [&](size_t id, int slot, size_t have, size_t n) {
        auto x = tok(n, id * 100 + have);
        pa.append_kv_cache(id, x.data(), x.data(), n, DataType::FLOAT32);
        for (size_t pg = (have + 3) / 4; pg < (have + n + 3) / 4; ++pg) want[slot].push_back(ahpc_oracle_pool_allocate(model));
    };
    append(a, 0, 0, 9);    // 3 pages
    append(b, 1, 0, 4);    // 1 page
    append(a, 0, 9, 3);    // fills page 3, no new page
    append(c3, 2, 0, 10);  // 3 pages: pool (6) exhausted after 2 -> grows by 3
    EXPECT(pa.get_sequence_pages(a) == want[0] && pa.get_sequence_pages(b) == want[1] && pa.get_sequence_pages(c3) == want[2]);
    pa.truncate_sequence(a, 5);  // keeps 2 pages, frees the third
    ahpc_oracle_pool_release(model, want[0].back());
    want[0].pop_back();
    pa.destroy_sequence(b);
    ahpc_oracle_pool_release(model, want[1][0]);
    append(c3, 2, 10, 9);  // 2 more pages: recycled FIFO
    EXPECT(pa.get_sequence_pages(a) == want[0] && pa.get_sequence_pages(c3) == want[2]);
    const KVBlockPoolStats st = pa.get_pool_stats();
    EXPECT((int32_t)st.total_pages == ahpc_oracle_pool_total(model) && (int32_t)st.free_pages == ahpc_oracle_pool_free_count(model));
    EXPECT(pa.get_total_memory_usage() == st.allocated_pages * st.page_bytes && pa.get_peak_memory_usage() >= pa.get_total_memory_usage());
    EXPECT(pa.get_sequence_length(a) == 5 && pa.get_max_sequence_length(a) == 5);
    ahpc_oracle_pool_destroy(model);
}

CASE(Paged_AppendThenGetRoundTrip, true) {
    PagedAttention pa;
    AttentionParams p{};
    p.batch_size = 1; p.sequence_length = 1; p.num_heads = 4; p.head_dimension = 64;
    pa.configure(p);
    const size_t H = 4, d = 64, id = pa.create_sequence(256);
    auto k1 = normal(21 * H * d, 60, 2), v1 = normal(21 * H * d, 60, 3), k2 = normal(40 * H * d, 61, 2), v2 = normal(40 * H * d, 61, 3);
    pa.append_kv_cache(id, k1.data(), v1.data(), 21, DataType::FLOAT32);
    pa.append_kv_cache(id, k2.data(), v2.data(), 40, DataType::FLOAT32);
    std::vector<float> kg(61 * H * d), vg(61 * H * d);
    pa.get_kv_cache(id, kg.data(), vg.data(), 0, 61, DataType::FLOAT32);
    std::vector<float> kall = k1, vall = v1;
    kall.insert(kall.end(), k2.begin(), k2.end());
    vall.insert(vall.end(), v2.begin(), v2.end());
    EXPECT(kg == kall && vg == vall);  // bit exact
    std::vector<float> part(5 * H * d), partv(5 * H * d);
    pa.get_kv_cache(id, part.data(), partv.data(), 19, 5, DataType::FLOAT32);
    EXPECT(std::equal(part.begin(), part.end(), kall.begin() + 19 * H * d));
    EXPECT_THROWS(pa.get_kv_cache(id, part.data(), partv.data(), 60, 5, DataType::FLOAT32), AttentionError::INVALID_INPUT);
    EXPECT_THROWS(pa.append_kv_cache(999, k1.data(), v1.data(), 1, DataType::FLOAT32), AttentionError::INVALID_INPUT);
    pa.clear_kv_cache(id);
    EXPECT(pa.get_sequence_length(id) == 0 && pa.get_sequence_pages(id).empty());
}

template <typename T> static void paged_batch(DataType dt, float tol) {
    PagedAttention pa;
    AttentionParams p{};
    p.batch_size = 5; p.sequence_length = 1; p.num_heads = 8; p.head_dimension = 128; p.max_sequence_length = 2048;
    PagedAttentionConfig c;
    c.split_chunk_tokens = 128;  // several chunks per sequence: exercises the merge
    pa.configure_paged_attention(c);
    pa.configure(p);
    const size_t H = 8, d = 128, P = 16;
    const size_t lens[5] = {700, 33, 0, 1500, 16};
    std::vector<size_t> ids;
    std::vector<std::vector<float>> ks, vs;
    for (int i = 0; i < 5; ++i) {
        ids.push_back(pa.create_sequence(2048));
        auto k = from_storage(to_storage<T>(normal(lens[i] * H * d, 70 + i, 2)));
        auto v = from_storage(to_storage<T>(normal(lens[i] * H * d, 70 + i, 3)));
        auto kt = to_storage<T>(k), vt = to_storage<T>(v);
        // interleave appends so that the sequences' pages interleave in the pool
        size_t done = 0;
        while (done < lens[i]) {
            const size_t n = std::min<size_t>(lens[i] - done, 300);
            pa.append_kv_cache(ids[i], kt.data() + done * H * d, vt.data() + done * H * d, n, dt);
            done += n;
        }
        ks.push_back(k);
        vs.push_back(v);
    }
    // decode in a different order than creation
    const int order[5] = {3, 0, 4, 2, 1};
    std::vector<size_t> bid;
    std::vector<TensorShape> shp(5, TensorShape({1, 1, H, d}, dt));
    std::vector<std::vector<T>> q(5), out(5);
    std::vector<const void*> qp;
    std::vector<void*> op;
    for (int j = 0; j < 5; ++j) {
        bid.push_back(ids[order[j]]);
        q[j] = to_storage<T>(normal(H * d, 80 + j, 1));
        out[j].assign(H * d, T(7.0f));
        qp.push_back(q[j].data());
        op.push_back(out[j].data());
    }
    pa.forward_batch(bid, shp, qp, shp, op);
    for (int j = 0; j < 5; ++j) {
        const size_t L = lens[order[j]];
        std::vector<float> want(H * d, 0.0f);
        if (L) {
            std::vector<int32_t> table((L + P - 1) / P);
            for (size_t i = 0; i < table.size(); ++i) table[i] = (int32_t)i;
            std::vector<float> kp(table.size() * P * H * d, 0.0f), vp(kp.size(), 0.0f);
            std::copy(ks[order[j]].begin(), ks[order[j]].end(), kp.begin());
            std::copy(vs[order[j]].begin(), vs[order[j]].end(), vp.begin());
            const int32_t len = (int32_t)L;
            auto qf = from_storage(q[j]);
            ahpc_oracle_paged_decode(qf.data(), want.data(), kp.data(), vp.data(), table.data(), &len, nullptr, 1, H, d, P, table.size(),
                                     1.0f / std::sqrt((float)d), 2);
        }
        EXPECT(max_abs_diff(from_storage(out[j]), want) <= tol);
    }
    // vector size mismatch -> INVALID_INPUT (src/algorithms/paged_attention.cpp:511-516)
    std::vector<const void*> short_q(qp.begin(), qp.begin() + 4);
    EXPECT_THROWS(pa.forward_batch(bid, shp, short_q, shp, op), AttentionError::INVALID_INPUT);
    EXPECT_THROWS(pa.forward_batch({12345}, {shp[0]}, {qp[0]}, {shp[0]}, {op[0]}), AttentionError::INVALID_INPUT);
    EXPECT(pa.get_active_sequences_count() == 5);
}
CASE(Paged_ForwardBatchAgainstOracle, true) {
    paged_batch<float>(DataType::FLOAT32, 1e-4f);
    paged_batch<half>(DataType::FLOAT16, 2e-2f);
    paged_batch<bfloat16>(DataType::BFLOAT16, 2e-2f);
}

CASE(Paged_ConvenienceForward, true) {  // src/algorithms/paged_attention.cpp:132-174
    PagedAttention pa;
    AttentionParams p{};
    p.batch_size = 3; p.sequence_length = 50; p.num_heads = 4; p.head_dimension = 64;
    pa.configure(p);
    const size_t B = 3, N = 50, H = 4, d = 64;
    auto q = normal(B * H * d, 90, 1), k = normal(B * N * H * d, 90, 2), v = normal(B * N * H * d, 90, 3);
    std::vector<float> out(B * H * d);
    pa.forward(shape4(B, 1, H, d), q.data(), shape4(B, N, H, d), k.data(), shape4(B, N, H, d), v.data(), shape4(B, 1, H, d), out.data());
    // == last row of causal dense attention whose last query is q
    for (size_t b = 0; b < B; ++b) {
        std::vector<float> qq(N * H * d, 0.0f), want(N * H * d);
        std::copy(q.begin() + b * H * d, q.begin() + (b + 1) * H * d, qq.begin() + (N - 1) * H * d);
        ahpc_oracle_attention(qq.data(), k.data() + b * N * H * d, v.data() + b * N * H * d, want.data(), 1, N, H, d, N * H * d, H * d, d, 0.125f, 1, nullptr, 1);
        float e = 0.0f;
        for (size_t i = 0; i < H * d; ++i) e = std::max(e, std::fabs(out[b * H * d + i] - want[(N - 1) * H * d + i]));
        EXPECT(e <= 1e-4f);
    }
    EXPECT(pa.get_active_sequences_count() == 0 && pa.get_total_memory_usage() == 0);
    EXPECT_THROWS(pa.forward(shape4(B, N, H, d), k.data(), shape4(B, N, H, d), k.data(), shape4(B, N, H, d), v.data(), shape4(B, N, H, d), k.data()),
                  AttentionError::UNSUPPORTED_OPERATION);
}

// Grouped key/value heads (AttentionParams::key_value_heads; read nowhere in the reference, so the only
// yardstick is the definition: query head h uses K/V head h / (H / H_kv)).  The grouped call must equal the
// oracle fed K and V with every head repeated.
static std::vector<float> repeat_heads(const std::vector<float>& x, size_t rows, size_t Hkv, size_t g, size_t d) {
    std::vector<float> y(rows * Hkv * g * d);
    for (size_t r = 0; r < rows; ++r)
        for (size_t h = 0; h < Hkv * g; ++h)
            std::copy(x.begin() + (r * Hkv + h / g) * d, x.begin() + (r * Hkv + h / g + 1) * d, y.begin() + (r * Hkv * g + h) * d);
    return y;
}
CASE(Gqa_FlashForwardEqualsRepeatedHeads, true) {
    const size_t B = 2, N = 96, H = 8, Hkv = 2, d = 64, g = H / Hkv;
    AttentionParams p{};
    p.batch_size = B; p.sequence_length = N; p.num_heads = H; p.key_value_heads = Hkv; p.head_dimension = d; p.causal_mask = true;
    FlashAttention fa;
    fa.configure(p);
    auto q = uniform(B * N * H * d, 95, 1), k = uniform(B * N * Hkv * d, 95, 2), v = uniform(B * N * Hkv * d, 95, 3);
    std::vector<float> out(q.size(), 0.0f);
    fa.forward(shape4(B, N, H, d), q.data(), shape4(B, N, Hkv, d), k.data(), shape4(B, N, Hkv, d), v.data(), shape4(B, N, H, d), out.data());
    auto want = oracle_bnhd(q, repeat_heads(k, B * N, Hkv, g, d), repeat_heads(v, B * N, Hkv, g, d), B, N, H, d, 0.125f, true);
    EXPECT(max_abs_diff(out, want) <= 1e-4f);
    // K/V shaped like Q is now a shape error, and a head count that does not divide is refused at configure
    EXPECT_THROWS(fa.forward(shape4(B, N, H, d), q.data(), shape4(B, N, H, d), q.data(), shape4(B, N, H, d), q.data(), shape4(B, N, H, d), out.data()),
                  AttentionError::INVALID_INPUT);
    p.key_value_heads = 3;
    EXPECT_THROWS(fa.configure(p), AttentionError::INVALID_PARAMETERS);
}
CASE(Gqa_PagedDecodeEqualsRepeatedHeads, true) {
    // groups of 4, 3 and 7 query heads per cached head on the reference's default fp32 cache
    for (const size_t H : {size_t(8), size_t(6), size_t(14)}) {
        const size_t Hkv = 2, d = 128, P = 16, g = H / Hkv, L = 300;
        AttentionParams p{};
        p.batch_size = 1; p.sequence_length = 1; p.num_heads = H; p.key_value_heads = Hkv; p.head_dimension = d; p.max_sequence_length = 512;
        PagedAttention pa;
        pa.configure(p);
        const size_t id = pa.create_sequence(512);
        auto k = normal(L * Hkv * d, 96, 2), v = normal(L * Hkv * d, 96, 3), q = normal(H * d, 96, 1);
        pa.append_kv_cache(id, k.data(), v.data(), L, DataType::FLOAT32);   // [n, key_value_heads, d]
        std::vector<float> out(H * d, 7.0f);
        const TensorShape s({1, 1, H, d}, DataType::FLOAT32);
        pa.forward_batch({id}, {s}, {q.data()}, {s}, {out.data()});
        std::vector<int32_t> table((L + P - 1) / P);
        for (size_t i = 0; i < table.size(); ++i) table[i] = (int32_t)i;
        auto kx = repeat_heads(k, L, Hkv, g, d), vx = repeat_heads(v, L, Hkv, g, d);
        kx.resize(table.size() * P * H * d, 0.0f);
        vx.resize(kx.size(), 0.0f);
        std::vector<float> want(H * d, 0.0f);
        const int32_t len = (int32_t)L;
        ahpc_oracle_paged_decode(q.data(), want.data(), kx.data(), vx.data(), table.data(), &len, nullptr, 1, H, d, P, table.size(),
                                 1.0f / std::sqrt((float)d), 1);
        EXPECT(max_abs_diff(out, want) <= 1e-4f);
    }
    const size_t H = 8, Hkv = 2, d = 128, L = 300;
    AttentionParams p{};
    p.batch_size = 1; p.sequence_length = 1; p.num_heads = H; p.key_value_heads = Hkv; p.head_dimension = d; p.max_sequence_length = 512;
    PagedAttention pa;
    pa.configure(p);
    const size_t id = pa.create_sequence(512);
    auto k = normal(L * Hkv * d, 96, 2), v = normal(L * Hkv * d, 96, 3);
    pa.append_kv_cache(id, k.data(), v.data(), L, DataType::FLOAT32);
    // read-back returns what was appended, in the pool's own head count
    std::vector<float> kb(L * Hkv * d), vb(L * Hkv * d);
    pa.get_kv_cache(id, kb.data(), vb.data(), 0, L, DataType::FLOAT32);
    EXPECT(kb == k && vb == v);
    p.key_value_heads = 3; p.num_heads = 8;  // every cached head serves the same number of query heads
    EXPECT_THROWS(pa.configure(p), AttentionError::INVALID_PARAMETERS);
}

CASE(WideGroups_MultiQueryDecode, true) {
    // 32 query heads over ONE cached head (multi-query attention), fp16 cache: the matrix-core decode kernel
    const size_t H = 32, Hkv = 1, d = 128, P = 16, g = H / Hkv, L = 333;
    AttentionParams p{};
    p.batch_size = 1; p.sequence_length = 1; p.num_heads = H; p.key_value_heads = Hkv; p.head_dimension = d; p.max_sequence_length = 512;
    PagedAttention pa;
    pa.configure(p);
    const size_t id = pa.create_sequence(512);
    auto k = normal(L * Hkv * d, 99, 2), v = normal(L * Hkv * d, 99, 3), q = normal(H * d, 99, 1);
    std::vector<half> hk(k.size()), hv(v.size()), hq(q.size());
    for (size_t i = 0; i < k.size(); ++i) { hk[i] = half(k[i]); k[i] = static_cast<float>(hk[i]); hv[i] = half(v[i]); v[i] = static_cast<float>(hv[i]); }
    for (size_t i = 0; i < q.size(); ++i) { hq[i] = half(q[i]); q[i] = static_cast<float>(hq[i]); }
    pa.append_kv_cache(id, hk.data(), hv.data(), L, DataType::FLOAT16);
    std::vector<half> out(H * d);
    const TensorShape s({1, 1, H, d}, DataType::FLOAT16);
    pa.forward_batch({id}, {s}, {hq.data()}, {s}, {out.data()});
    std::vector<int32_t> table((L + P - 1) / P);
    for (size_t i = 0; i < table.size(); ++i) table[i] = (int32_t)i;
    auto kx = repeat_heads(k, L, Hkv, g, d), vx = repeat_heads(v, L, Hkv, g, d);
    kx.resize(table.size() * P * H * d, 0.0f);
    vx.resize(kx.size(), 0.0f);
    std::vector<float> want(H * d, 0.0f), got(H * d);
    const int32_t len = (int32_t)L;
    ahpc_oracle_paged_decode(q.data(), want.data(), kx.data(), vx.data(), table.data(), &len, nullptr, 1, H, d, P, table.size(),
                             1.0f / std::sqrt((float)d), 1);
    for (size_t i = 0; i < got.size(); ++i) got[i] = static_cast<float>(out[i]);
    EXPECT(max_abs_diff(got, want) <= 2e-2f);
    // the same grouping on an fp32 cache: no matrix-core kernel, the group is served in slices of 8 query heads
    PagedAttention pf;
    pf.configure(p);
    const size_t idf = pf.create_sequence(512);
    pf.append_kv_cache(idf, k.data(), v.data(), L, DataType::FLOAT32);
    std::vector<float> of(H * d, 7.0f);
    const TensorShape sf({1, 1, H, d}, DataType::FLOAT32);
    pf.forward_batch({idf}, {sf}, {q.data()}, {sf}, {of.data()});
    EXPECT(max_abs_diff(of, want) <= 1e-4f);
}

CASE(Paged_PrefillHandOffBatchAndPacked, true) {
    // K/V of a prefill batch go into the caches of several sequences in one call; reading them back and
    // decoding must give what appending sequence by sequence gives.
    const size_t B = 3, N = 40, H = 4, d = 64;
    AttentionParams p{};
    p.batch_size = B; p.sequence_length = 1; p.num_heads = H; p.head_dimension = d; p.max_sequence_length = 256;
    PagedAttention a, b;
    a.configure(p);
    b.configure(p);
    auto k = normal(B * N * H * d, 97, 2), v = normal(B * N * H * d, 97, 3);
    const std::vector<size_t> counts = {40, 7, 33};
    std::vector<size_t> ia, ib;
    for (size_t i = 0; i < B; ++i) {
        ia.push_back(a.create_sequence(256));
        ib.push_back(b.create_sequence(256));
    }
    // both start with a few tokens already cached, so that the new ones land mid-page
    auto k0 = normal(5 * H * d, 98, 2), v0 = normal(5 * H * d, 98, 3);
    for (size_t i = 0; i < B; ++i) {
        a.append_kv_cache(ia[i], k0.data(), v0.data(), 5, DataType::FLOAT32);
        b.append_kv_cache(ib[i], k0.data(), v0.data(), 5, DataType::FLOAT32);
    }
    a.append_kv_cache_batch(ia, shape4(B, N, H, d), k.data(), v.data(), counts);
    for (size_t i = 0; i < B; ++i) b.append_kv_cache(ib[i], k.data() + i * N * H * d, v.data() + i * N * H * d, counts[i], DataType::FLOAT32);
    for (size_t i = 0; i < B; ++i) {
        EXPECT(a.get_sequence_length(ia[i]) == 5 + counts[i]);
        EXPECT(a.get_sequence_pages(ia[i]) == b.get_sequence_pages(ib[i]));
        const size_t L = 5 + counts[i];
        std::vector<float> ka(L * H * d), va(L * H * d), kb(L * H * d), vb(L * H * d);
        a.get_kv_cache(ia[i], ka.data(), va.data(), 0, L, DataType::FLOAT32);
        b.get_kv_cache(ib[i], kb.data(), vb.data(), 0, L, DataType::FLOAT32);
        EXPECT(ka == kb && va == vb);
    }
    // packed: three more chunks of lengths 9, 0, 20 out of one [29,H,d] tensor
    const int32_t cu[4] = {0, 9, 9, 29};
    auto kp = normal(29 * H * d, 99, 2), vp = normal(29 * H * d, 99, 3);
    a.append_kv_cache_packed(ia, TensorShape({29, H, d}, DataType::FLOAT32), kp.data(), vp.data(), cu);
    for (size_t i = 0; i < B; ++i) {
        const size_t n = (size_t)(cu[i + 1] - cu[i]);
        if (n) b.append_kv_cache(ib[i], kp.data() + (size_t)cu[i] * H * d, vp.data() + (size_t)cu[i] * H * d, n, DataType::FLOAT32);
    }
    std::vector<TensorShape> shp(B, TensorShape({1, 1, H, d}, DataType::FLOAT32));
    auto q = normal(B * H * d, 97, 1);
    std::vector<float> oa(B * H * d, 1.0f), ob(B * H * d, 2.0f);
    std::vector<const void*> qp;
    std::vector<void*> pa, pb;
    for (size_t i = 0; i < B; ++i) {
        qp.push_back(q.data() + i * H * d);
        pa.push_back(oa.data() + i * H * d);
        pb.push_back(ob.data() + i * H * d);
    }
    a.forward_batch(ia, shp, qp, shp, pa);
    b.forward_batch(ib, shp, qp, shp, pb);
    EXPECT(oa == ob);
    EXPECT_THROWS(a.append_kv_cache_batch({ia[0], 4242, ia[2]}, shape4(B, N, H, d), k.data(), v.data()), AttentionError::INVALID_INPUT);
    EXPECT_THROWS(a.append_kv_cache_batch({ia[0], ia[0], ia[2]}, shape4(B, N, H, d), k.data(), v.data()), AttentionError::INVALID_INPUT);
    EXPECT_THROWS(a.append_kv_cache_batch(ia, shape4(B, N, H + 1, d), k.data(), v.data()), AttentionError::INVALID_INPUT);
    EXPECT(a.get_sequence_length(ia[0]) == 5 + 40 + 9);  // failed calls changed nothing
}

CASE(Paged_SequenceLifecycle, true) {  // extend / truncate / reset, src/algorithms/paged_attention.cpp:352-418
    PagedAttention pa;
    AttentionParams p{};
    p.batch_size = 1; p.sequence_length = 1; p.num_heads = 2; p.head_dimension = 32;
    pa.configure(p);
    const size_t id = pa.create_sequence(20);
    auto x = normal(20 * 2 * 32, 95, 2);
    pa.append_kv_cache(id, x.data(), x.data(), 20, DataType::FLOAT32);
    EXPECT(pa.get_sequence_pages(id).size() == 2 && pa.get_max_sequence_length(id) == 20);
    pa.extend_sequence(id, 30);  // limit 50 -> 4 pages pre-allocated
    EXPECT(pa.get_max_sequence_length(id) == 50 && pa.get_sequence_pages(id).size() == 4);
    pa.truncate_sequence(id, 17);
    EXPECT(pa.get_sequence_length(id) == 17 && pa.get_sequence_pages(id).size() == 2);
    pa.reset_sequence(id);
    EXPECT(pa.get_sequence_length(id) == 0 && pa.is_sequence_active(id) && pa.get_sequence_pages(id).empty());
    // 40 sequences: more than the default 32 table rows
    std::vector<size_t> ids;
    for (int i = 0; i < 40; ++i) ids.push_back(pa.create_sequence(16));
    EXPECT(pa.get_active_sequences_count() == 41);
    for (size_t s : ids) pa.append_kv_cache(s, x.data(), x.data(), 3, DataType::FLOAT32);
    std::vector<float> out(2 * 32), q = normal(2 * 32, 96, 1);
    const TensorShape qs = shape4(1, 1, 2, 32);
    pa.forward_batch({ids[39]}, {qs}, {q.data()}, {qs}, {out.data()});
    EXPECT(std::isfinite(out[0]));
}

CASE(Paged_PoolGrowsWhileOtherThreadsAppendAndDecode, true) {
    // The pool starts with 4 pages and grows 2 at a time, so the slabs move (device copy, old slabs freed) again and again
    // while one thread appends to a sequence and reads it back, a second one decodes from it, and a third one creates
    // and extends other sequences.  Nothing may be lost or read from a slab that has moved.
    PagedAttention pa;
    AttentionParams p{};
    p.batch_size = 1; p.sequence_length = 1; p.num_heads = 2; p.head_dimension = 32; p.max_sequence_length = 512;
    PagedAttentionConfig c;
    c.initial_page_pool_size = 4;
    c.page_pool_growth = 2;
    pa.configure_paged_attention(c);
    pa.configure(p);
    const size_t H = 2, d = 32, P = 16, total = 320, step = 8;
    const size_t id = pa.create_sequence(512);
    const auto k = normal(total * H * d, 97, 2), v = normal(total * H * d, 97, 3);
    std::atomic<size_t> appended{0};
    std::atomic<bool> stop{false};
    std::atomic<int> bad{0};
    std::thread grower([&] {
        std::vector<size_t> others;
        const auto x = normal(40 * H * d, 98, 2);
        for (int i = 0; i < 24 && !stop.load(); ++i) {
            others.push_back(pa.create_sequence(16));
            pa.extend_sequence(others.back(), 24);          // 40 tokens = 3 pages pre-allocated: the pool grows
            pa.append_kv_cache(others.back(), x.data(), x.data(), 40, DataType::FLOAT32);
            if (i % 3 == 2) {
                pa.destroy_sequence(others.front());
                others.erase(others.begin());
            }
        }
    });
    std::thread decoder([&] {
        const auto q = normal(H * d, 99, 1);
        const TensorShape qs = shape4(1, 1, H, d);
        while (!stop.load()) {
            // the length is whatever the appending thread has reached by the time the decode launches: the result must
            // be finite and must equal the oracle for SOME prefix; it is checked exactly once everything is appended
            std::vector<float> out(H * d, 0.0f);
            if (appended.load() == 0) continue;
            pa.forward_batch({id}, {qs}, {q.data()}, {qs}, {out.data()});
            for (float y : out)
                if (!std::isfinite(y)) bad.fetch_add(1);
        }
    });
    for (size_t done = 0; done < total; done += step) {
        pa.append_kv_cache(id, k.data() + done * H * d, v.data() + done * H * d, step, DataType::FLOAT32);
        appended.store(done + step);
        if (done % 64 == 0) {
            std::vector<float> kg((done + step) * H * d), vg(kg.size());
            pa.get_kv_cache(id, kg.data(), vg.data(), 0, done + step, DataType::FLOAT32);
            if (!std::equal(kg.begin(), kg.end(), k.begin()) || !std::equal(vg.begin(), vg.end(), v.begin())) bad.fetch_add(1);
        }
    }
    stop.store(true);
    grower.join();
    decoder.join();
    EXPECT(bad.load() == 0);
    std::vector<float> kg(total * H * d), vg(kg.size());
    pa.get_kv_cache(id, kg.data(), vg.data(), 0, total, DataType::FLOAT32);
    EXPECT(kg == k && vg == v);  // bit exact after all the moves
    const auto q = normal(H * d, 99, 1);
    const TensorShape qs = shape4(1, 1, H, d);
    std::vector<float> out(H * d), want(H * d);
    pa.forward_batch({id}, {qs}, {q.data()}, {qs}, {out.data()});
    std::vector<int32_t> table(total / P);
    for (size_t i = 0; i < table.size(); ++i) table[i] = (int32_t)i;
    const int32_t len = (int32_t)total;
    ahpc_oracle_paged_decode(q.data(), want.data(), k.data(), v.data(), table.data(), &len, nullptr, 1, H, d, P, table.size(),
                             1.0f / std::sqrt((float)d), 2);
    EXPECT(max_abs_diff(out, want) <= 1e-4f);
}

CASE(Paged_CompactPagesRehomesPagesAndShrinksThePool, true) {
    // Six sequences of three pages each, every other one destroyed: the survivors' pages are scattered over the id range.
    // compact_pages() moves them onto the lowest ids (on the device), rewrites the block table and drops the pool's free
    // tail; cache contents and decode results are what they were, bit for bit, and the pool goes on working.
    PagedAttention pa;
    AttentionParams p{};
    p.batch_size = 1; p.sequence_length = 1; p.num_heads = 2; p.head_dimension = 32; p.max_sequence_length = 256;
    PagedAttentionConfig c;
    c.initial_page_pool_size = 8;
    c.page_pool_growth = 4;
    pa.configure_paged_attention(c);
    pa.configure(p);
    const size_t H = 2, d = 32, T = 40;
    std::vector<size_t> ids;
    std::vector<std::vector<float>> ks, vs;
    for (int i = 0; i < 6; ++i) {
        ids.push_back(pa.create_sequence(64));
        ks.push_back(normal(T * H * d, 130 + i, 2));
        vs.push_back(normal(T * H * d, 130 + i, 3));
        pa.append_kv_cache(ids.back(), ks.back().data(), vs.back().data(), T, DataType::FLOAT32);
    }
    for (int i : {0, 2, 4}) pa.destroy_sequence(ids[i]);
    const std::vector<size_t> keep = {ids[1], ids[3], ids[5]};
    const auto q = normal(3 * H * d, 140, 1);
    const TensorShape qs = shape4(1, 1, H, d);
    auto decode_all = [&]() {
        std::vector<float> out(3 * H * d);
        pa.forward_batch(keep, {qs, qs, qs}, {q.data(), q.data() + H * d, q.data() + 2 * H * d}, {qs, qs, qs},
                         {out.data(), out.data() + H * d, out.data() + 2 * H * d});
        return out;
    };
    const auto before = decode_all();
    std::vector<std::vector<int32_t>> pages_before;
    for (size_t id : keep) pages_before.push_back(pa.get_sequence_pages(id));
    EXPECT(pa.get_pool_stats().total_pages >= 18);
    int32_t highest = 0;
    for (auto& pg : pages_before) for (int32_t x : pg) highest = std::max(highest, x);
    EXPECT(highest >= 9);  // scattered: some page in use lies beyond the count of pages in use

    pa.compact_pages();

    const KVBlockPoolStats st = pa.get_pool_stats();
    EXPECT(st.allocated_pages == 9 && st.total_pages == 9 && st.free_pages == 0);
    std::vector<int32_t> seen;
    for (size_t i = 0; i < keep.size(); ++i) {
        const auto pg = pa.get_sequence_pages(keep[i]);
        EXPECT(pg.size() == 3);
        for (int32_t x : pg) { EXPECT(x >= 0 && x < 9); seen.push_back(x); }
        std::vector<float> kg(T * H * d), vg(T * H * d);
        pa.get_kv_cache(keep[i], kg.data(), vg.data(), 0, T, DataType::FLOAT32);
        EXPECT(kg == ks[2 * i + 1] && vg == vs[2 * i + 1]);
    }
    std::sort(seen.begin(), seen.end());
    EXPECT(std::adjacent_find(seen.begin(), seen.end()) == seen.end() && seen.size() == 9);  // every id once
    EXPECT(decode_all() == before);
    // compacting a compact pool changes nothing
    pa.compact_pages();
    EXPECT(decode_all() == before && pa.get_pool_stats().total_pages == 9);
    // the pool goes on: a new sequence takes the next ids (the pool grows again) and appends to a survivor still work
    const size_t fresh = pa.create_sequence(64);
    pa.append_kv_cache(fresh, ks[0].data(), vs[0].data(), T, DataType::FLOAT32);
    const auto pg = pa.get_sequence_pages(fresh);
    EXPECT(pg.size() == 3 && pg[0] == 9 && pg[1] == 10 && pg[2] == 11);
    std::vector<float> kg(T * H * d), vg(T * H * d);
    pa.get_kv_cache(fresh, kg.data(), vg.data(), 0, T, DataType::FLOAT32);
    EXPECT(kg == ks[0] && vg == vs[0]);
    EXPECT(decode_all() == before);
}

// ---- KV block pool growth ---------------------------------------------------------------------------------------
static bool on_cpu_executor() {
    ahpc_device_info info;
    return ahpc_hip_device_info(0, &info) == 0 && std::strstr(info.name, "CPU executor") != nullptr;
}

// Fills pages [0, pages) of a pool from seeded host data through the scatter entry point and returns what was written.
static void fill_pool_pages(KVBlockPool& pool, size_t pages, size_t H, size_t d, size_t P, std::vector<float>& k, std::vector<float>& v) {
    const size_t tokens = pages * P;
    k = normal(tokens * H * d, 123, 2);
    v = normal(tokens * H * d, 123, 3);
    std::vector<int32_t> table(pages);
    for (size_t i = 0; i < pages; ++i) table[i] = (int32_t)i;
    void *dk = nullptr, *dv = nullptr, *dt = nullptr;
    EXPECT(ahpc_hip_malloc(&dk, k.size() * 4) == 0 && ahpc_hip_malloc(&dv, v.size() * 4) == 0 && ahpc_hip_malloc(&dt, pages * 4) == 0);
    ahpc_hip_memcpy_h2d(dk, k.data(), k.size() * 4, nullptr);
    ahpc_hip_memcpy_h2d(dv, v.data(), v.size() * 4, nullptr);
    ahpc_hip_memcpy_h2d(dt, table.data(), pages * 4, nullptr);
    EXPECT(ahpc_hip_kv_scatter(dk, dv, AHPC_F32, pool.k_slab(), pool.v_slab(), (int)pool.dtype(), (const int32_t*)dt, (int64_t)pages,
                               nullptr, nullptr, 0, 0, (int64_t)tokens, (int64_t)H, (int64_t)d, (int64_t)P, nullptr) == 0);
    ahpc_hip_stream_synchronize(nullptr);
    ahpc_hip_free(dk); ahpc_hip_free(dv); ahpc_hip_free(dt);
}

static void gather_pool_pages(KVBlockPool& pool, size_t pages, size_t H, size_t d, size_t P, std::vector<float>& k, std::vector<float>& v) {
    const size_t tokens = pages * P;
    k.assign(tokens * H * d, -1.0f);
    v.assign(tokens * H * d, -1.0f);
    std::vector<int32_t> table(pages);
    for (size_t i = 0; i < pages; ++i) table[i] = (int32_t)i;
    void *dk = nullptr, *dv = nullptr, *dt = nullptr;
    EXPECT(ahpc_hip_malloc(&dk, k.size() * 4) == 0 && ahpc_hip_malloc(&dv, v.size() * 4) == 0 && ahpc_hip_malloc(&dt, pages * 4) == 0);
    ahpc_hip_memcpy_h2d(dt, table.data(), pages * 4, nullptr);
    EXPECT(ahpc_hip_kv_gather(dk, dv, AHPC_F32, pool.k_slab(), pool.v_slab(), (int)pool.dtype(), (const int32_t*)dt, (int64_t)pages, 0, 0,
                              (int64_t)tokens, (int64_t)H, (int64_t)d, (int64_t)P, nullptr) == 0);
    ahpc_hip_memcpy_d2h(k.data(), dk, k.size() * 4, nullptr);
    ahpc_hip_memcpy_d2h(v.data(), dv, v.size() * 4, nullptr);
    ahpc_hip_stream_synchronize(nullptr);
    ahpc_hip_free(dk); ahpc_hip_free(dv); ahpc_hip_free(dt);
}

CASE(Pool_GrowsInPlace, true) {
    // Slabs are address ranges backed on demand: growth keeps their addresses and their contents, the generation stays 0,
    // and the page order is the FIFO order whatever the capacity steps are.
    size_t granularity = 0;
    EXPECT(ahpc_hip_vmem_granularity(&granularity) == 0);
    if (granularity == 0) { std::printf("    (no virtual memory management on this device: skipped)\n"); return; }
    const size_t H = 2, d = 32, P = 16;
    KVBlockPool pool(P, H, d, DataType::FLOAT32, 8, 4, size_t(1) << 30);
    EXPECT(pool.grows_in_place());
    void* const k0 = pool.k_slab();
    void* const v0 = pool.v_slab();
    std::vector<float> k, v, kg, vg;
    fill_pool_pages(pool, 8, H, d, P, k, v);
    for (int i = 0; i < 8; ++i) EXPECT(pool.allocate_page() == i);
    EXPECT(pool.allocate_page() == 8);  // grows by 4
    EXPECT(pool.get_pool_size() == 12);
    pool.resize_pool(40000);            // 40000 pages x 4 KiB x 2 slabs = 312 MiB: several chunks (an exception ends the case here)
    EXPECT(pool.get_pool_size() == 40000 && pool.k_slab() == k0 && pool.v_slab() == v0 && pool.generation() == 0);
    EXPECT(pool.stats().slab_capacity_pages >= 40000);
    if (pool.stats().slab_capacity_pages < 40000) return;
    gather_pool_pages(pool, 8, H, d, P, kg, vg);
    EXPECT(kg == k && vg == v);
    // the last page is usable
    EXPECT(ahpc_hip_memset(static_cast<char*>(pool.k_slab()) + (40000 - 1) * P * H * d * 4, 0, P * H * d * 4, nullptr) == 0);
    EXPECT(ahpc_hip_stream_synchronize(nullptr) == 0);
    // the budget is the limit, and running into it loses nothing
    EXPECT_THROWS(pool.resize_pool((size_t(1) << 30) / (2 * P * H * d * 4) + 1), AttentionError::MEMORY_ALLOCATION_FAILED);
    EXPECT(pool.get_pool_size() == 40000);
    gather_pool_pages(pool, 8, H, d, P, kg, vg);
    EXPECT(kg == k && vg == v);
    // shrinking drops the free pages at the end of the id range (the nine in use stay) and gives their chunks back;
    // growing again maps new memory at the same addresses
    const size_t bytes_big = pool.stats().slab_bytes;
    pool.resize_pool(4);
    EXPECT(pool.get_pool_size() == 9 && pool.get_free_pages() == 0 && pool.k_slab() == k0);
    EXPECT(pool.stats().slab_bytes < bytes_big && pool.stats().slab_capacity_pages >= 9);
    gather_pool_pages(pool, 8, H, d, P, kg, vg);
    EXPECT(kg == k && vg == v);
    EXPECT(pool.allocate_page() == 9);  // grows by 4 again: ids follow on
    pool.resize_pool(40000);
    EXPECT(pool.get_pool_size() == 40000 && pool.k_slab() == k0 && pool.stats().slab_capacity_pages >= 40000);
    if (pool.stats().slab_capacity_pages < 40000) return;
    EXPECT(ahpc_hip_memset(static_cast<char*>(pool.v_slab()) + (40000 - 1) * P * H * d * 4, 0, P * H * d * 4, nullptr) == 0);
    EXPECT(ahpc_hip_stream_synchronize(nullptr) == 0);
    gather_pool_pages(pool, 8, H, d, P, kg, vg);
    EXPECT(kg == k && vg == v);
}

CASE(Pool_GrowsByCopyWhenInPlaceIsSwitchedOff, true) {
    // The path of devices without virtual memory management: the slabs move, the generation counts it, contents survive.
    int64_t before = 1;
    ahpc_hip_get_tuning("pool_in_place", &before);
    ahpc_hip_set_tuning("pool_in_place", 0);
    {
        const size_t H = 2, d = 32, P = 16;
        KVBlockPool pool(P, H, d, DataType::FLOAT32, 8, 4, size_t(1) << 28);
        EXPECT(!pool.grows_in_place());
        std::vector<float> k, v, kg, vg;
        fill_pool_pages(pool, 8, H, d, P, k, v);
        const uint64_t g0 = pool.generation();
        pool.resize_pool(4000);
        EXPECT(pool.generation() > g0 && pool.get_pool_size() == 4000);
        gather_pool_pages(pool, 8, H, d, P, kg, vg);
        EXPECT(kg == k && vg == v);
    }
    ahpc_hip_set_tuning("pool_in_place", before);
}

CASE(Pool_GrowsPast8GiBWhileDecodeRunsOnAnotherStream, true) {
    // A decode loop on its own stream keeps reading the first pages of the pool while the pool grows to more than 8 GiB
    // in place, 64 MiB per slab at a time: every result is bit-identical with the one before the growth, the slabs stay
    // where they are, and no decode waits for the growth (the longest iteration is printed next to the median).
    size_t granularity = 0;
    ahpc_hip_vmem_granularity(&granularity);
    if (granularity == 0) { std::printf("    (no virtual memory management on this device: skipped)\n"); return; }
    const bool small = on_cpu_executor();
    const size_t H = small ? 2 : 8, d = small ? 32 : 128, P = 16, B = small ? 2 : 8, ctx = small ? 64 : 2048;
    const size_t pages0 = B * ctx / P;
    const size_t page_bytes = P * H * d * 2;                     // fp16, one slab
    const size_t target_pages = small ? 4096 : (size_t(9) << 30) / (2 * page_bytes);  // 9 GiB of K + V
    KVBlockPool pool(P, H, d, DataType::FLOAT16, pages0, 16, size_t(16) << 30);  // (a budget of 16 GiB: chunks of 64 MiB)
    EXPECT(pool.grows_in_place());
    std::vector<float> k, v;
    fill_pool_pages(pool, pages0, H, d, P, k, v);
    for (size_t i = 0; i < pages0; ++i) pool.allocate_page();
    std::vector<int32_t> table(pages0), lens(B, (int32_t)ctx);
    for (size_t i = 0; i < pages0; ++i) table[i] = (int32_t)i;
    const auto q = normal(B * H * d, 124, 1);
    void *dq = nullptr, *dout = nullptr, *dt = nullptr, *dl = nullptr, *dws = nullptr, *stream = nullptr;
    const size_t ws = ahpc_hip_paged_decode_workspace_bytes(B, H, d, ctx, P, 0);
    EXPECT(ahpc_hip_malloc(&dq, q.size() * 4) == 0 && ahpc_hip_malloc(&dout, q.size() * 4) == 0 && ahpc_hip_malloc(&dt, pages0 * 4) == 0 &&
           ahpc_hip_malloc(&dl, B * 4) == 0 && ahpc_hip_malloc(&dws, ws ? ws : 16) == 0 && ahpc_hip_stream_create(&stream) == 0);
    ahpc_hip_memcpy_h2d(dq, q.data(), q.size() * 4, nullptr);
    ahpc_hip_memcpy_h2d(dt, table.data(), pages0 * 4, nullptr);
    ahpc_hip_memcpy_h2d(dl, lens.data(), B * 4, nullptr);
    ahpc_hip_stream_synchronize(nullptr);
    void* const k0 = pool.k_slab();
    auto decode = [&](std::vector<float>& out) {
        const int rc = ahpc_hip_paged_decode(dq, dout, AHPC_F32, pool.k_slab(), pool.v_slab(), AHPC_F16, (const int32_t*)dt, (const int32_t*)dl, nullptr,
                                             (int64_t)B, (int64_t)H, (int64_t)d, (int64_t)P, (int64_t)(ctx / P), (int64_t)ctx,
                                             1.0f / std::sqrt((float)d), 0, dws, ws, stream);
        ahpc_hip_memcpy_d2h(out.data(), dout, out.size() * 4, stream);
        ahpc_hip_stream_synchronize(stream);
        return rc;
    };
    std::vector<float> want(q.size());
    EXPECT(decode(want) == 0);
    std::atomic<bool> stop{false};
    std::atomic<int> bad{0};
    std::vector<double> ms;
    std::thread reader([&] {
        std::vector<float> out(q.size());
        while (!stop.load()) {
            const auto t0 = std::chrono::steady_clock::now();
            if (decode(out) != 0 || out != want) bad.fetch_add(1);
            ms.push_back(std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count());
        }
    });
    double grow_ms = 0.0;
    int steps = 0;
    std::string grow_error;
    try {
        for (size_t total = pages0; total < target_pages;) {
            total = std::min(target_pages, total + target_pages / 72);
            const auto t0 = std::chrono::steady_clock::now();
            pool.resize_pool(total);
            grow_ms += std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
            ++steps;
            std::this_thread::sleep_for(std::chrono::microseconds(300));  // (so that decodes fall between the steps)
        }
    } catch (const std::exception& e) {
        grow_error = e.what();
    }
    stop.store(true);
    reader.join();
    if (!grow_error.empty()) std::printf("    growth failed: %s\n", grow_error.c_str());
    EXPECT(grow_error.empty());
    if (!grow_error.empty()) return;  // (nothing behind the backed part of the slabs is touched)
    EXPECT(bad.load() == 0);
    EXPECT(pool.k_slab() == k0 && pool.generation() == 0 && pool.get_pool_size() == target_pages);
    EXPECT(pool.stats().slab_bytes >= target_pages * 2 * page_bytes);
    // the far end of the grown slabs is real memory
    EXPECT(ahpc_hip_memset(static_cast<char*>(pool.v_slab()) + (target_pages - 1) * page_bytes, 0, page_bytes, nullptr) == 0);
    EXPECT(ahpc_hip_stream_synchronize(nullptr) == 0);
    std::vector<float> after(q.size());
    EXPECT(decode(after) == 0 && after == want);
    if (!ms.empty()) {
        std::vector<double> sorted = ms;
        std::sort(sorted.begin(), sorted.end());
        std::printf("    pool grown to %.2f GiB in %d steps, %.2f ms of host time in all; %zu decodes meanwhile: median %.3f ms, longest %.3f ms\n",
                    pool.stats().slab_bytes / 1073741824.0, steps, grow_ms, ms.size(), sorted[sorted.size() / 2], sorted.back());
        // growth by reallocation would stop every stream for the copy of gigabytes (tens of milliseconds per step)
        if (!small) EXPECT(sorted.back() < 10.0 * sorted[sorted.size() / 2] + 2.0);
    }
    ahpc_hip_free(dq); ahpc_hip_free(dout); ahpc_hip_free(dt); ahpc_hip_free(dl); ahpc_hip_free(dws);
    ahpc_hip_stream_destroy(stream);
}

// ---- main ------------------------------------------------------------------------------------------------------
int main(int argc, char** argv) {
    bool no_gpu = false;
    std::string filter, skip;   // run cases whose name contains `filter`, leave out those containing `skip`
    for (int i = 1; i < argc; ++i) {
        if (std::string(argv[i]) == "--no-gpu") no_gpu = true;
        else if (std::string(argv[i]) == "--skip" && i + 1 < argc) skip = argv[++i];  // comma-separated substrings
        else filter = argv[i];
    }
    int ran = 0, failed = 0;
    for (const Case& c : cases()) {
        if (no_gpu && c.needs_gpu) continue;
        if (!filter.empty() && std::string(c.name).find(filter) == std::string::npos) continue;
        bool skipped = false;
        for (size_t a = 0; a < skip.size();) {
            const size_t e = std::min(skip.find(',', a), skip.size());
            if (e > a && std::string(c.name).find(skip.substr(a, e - a)) != std::string::npos) skipped = true;
            a = e + 1;
        }
        if (skipped) continue;
        std::printf("[ RUN  ] %s\n", c.name);
        std::fflush(stdout);
        const int before = g_failures;
        try {
            c.fn();
        } catch (const std::exception& e) {
            std::printf("    unexpected exception: %s\n", e.what());
            ++g_failures;
        }
        ++ran;
        if (g_failures != before) {
            ++failed;
            std::printf("[ FAIL ] %s\n", c.name);
        } else {
            std::printf("[  OK  ] %s\n", c.name);
        }
        std::fflush(stdout);
    }
    std::printf("%d cases run, %d failed\n", ran, failed);
    return failed == 0 ? 0 : 1;
}
