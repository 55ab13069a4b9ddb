// Sweep benchmark of the HIP FlashAttention backend in the shape of the reference's own harness:
// RunComprehensiveBenchmarks / benchmark_attention_config / GeneratePerformanceReport / SaveResultsToJSON,
// benchmarks/benchmark_attention.cpp:129-255, :462-669.  Same grid (BenchmarkConfig, :27-38: batch
// {1,2,4,8} x sequence {64..2048} x heads {1,4,8,12,16} x head_dim {64,128}, configurations above 50 M
// elements skipped, :490-493), same warm-up 5 / 10 timed iterations, same derived figures and the same JSON
// field names, so that its results file can be laid beside one produced by the reference.
//
// The backward pass is timed into backward_time_ms and total_time_ms exactly as the reference does (:215-235), and
// "gflops" is the reference's figure: B*H*N^2*d*2 over the TOTAL time (:241-242).  --csv FILE also writes the table of
// examples/performance_comparison.cpp:431-463 (same columns, same precisions).
//
// PagedAttention rows follow BM_PagedAttention (benchmarks/benchmark_attention.cpp:336-385, registered at :436-457 for
// batch 2 x sequence {256, 512, 1024} x heads {4, 8} x head_dim {64, 128}): createPagedAttention -> configure (page
// size 16, max_sequence_length = 2 x sequence) -> the convenience forward, timed as a whole (temporary sequences, cache
// append, one decode token per batch entry, release), with bytes_per_second as that benchmark's SetBytesProcessed
// counts them (4 tensors of B x N x H x d elements).  One figure is added: decode_time_ms, the decode of one token per
// sequence over caches that are already resident (PagedAttention::forward_batch), which is what a serving loop pays.
// They go into "paged_results" of the JSON file and a second table of the report.
//
// Differences, all forced: the backend is BackendType::HIP; inputs are seeded, not std::random_device.  Two extra
// JSON fields per row say where the tensors lived: with --device the tensors are resident in HBM (the kernel rate),
// without it they are host vectors exactly as in the reference and the times include the PCIe copies.
//
//   ahpc_bench_report [--device] [--dtype fp32|fp16|bf16] [--causal] [--quick] [--json FILE] [--csv FILE]
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iomanip>
#include <iostream>
#include <string>
#include <vector>

#include "ahpc_hip.h"
#include "algorithms/flash_attention.hpp"
#include "algorithms/paged_attention.hpp"
#include "api/backend_factory.hpp"
#include "api/tensor.hpp"

using namespace attention_hpc;

namespace {

struct Options {
    bool device = false, causal = false, quick = false;
    DataType dtype = DataType::FLOAT32;
    std::string json = "benchmark_results.json";
    std::string csv;   // empty: no CSV file
    int warmup = 5, iters = 10;  // BenchmarkConfig::warmup_iterations / benchmark_iterations
};

struct Metrics {  // PerformanceMetrics, benchmarks/benchmark_attention.cpp:41-51
    double forward_time_ms = 0.0, backward_time_ms = 0.0, total_time_ms = 0.0;
    size_t memory_usage_bytes = 0, peak_memory_bytes = 0;
    double gflops = 0.0, throughput_tokens_per_sec = 0.0;
    bool success = false;
    std::string error_message;
};

struct Result {
    size_t B, N, H, d;
    Metrics m;
    size_t total_elements() const { return B * N * H * d; }
    // BenchmarkResult::get_theoretical_flops, benchmarks/benchmark_attention.cpp:68-77
    double theoretical_flops() const {
        const double bhnn = (double)B * H * N * N;
        return bhnn * d + bhnn * 4 + bhnn * d;
    }
};

size_t elem_size(DataType t) { return t == DataType::FLOAT32 ? 4 : 2; }

// seeded U(-1, 1), stored in `t`
std::vector<unsigned char> random_tensor(size_t n, DataType t, uint32_t seed) {
    std::vector<unsigned char> out(n * elem_size(t));
    uint32_t s = seed * 2654435761u + 12345u;
    for (size_t i = 0; i < n; ++i) {
        s = s * 1664525u + 1013904223u;
        const float x = (float)((s >> 8) & 0xFFFFFF) / 8388608.0f - 1.0f;
        if (t == DataType::FLOAT32) std::memcpy(&out[4 * i], &x, 4);
        else if (t == DataType::FLOAT16) { const half h(x); std::memcpy(&out[2 * i], &h, 2); }
        else { const bfloat16 h(x); std::memcpy(&out[2 * i], &h, 2); }
    }
    return out;
}

struct DeviceTensor {
    void* p = nullptr;
    explicit DeviceTensor(const std::vector<unsigned char>& host) {
        if (ahpc_hip_malloc(&p, host.size()) != 0) throw std::runtime_error("device allocation failed");
        if (ahpc_hip_memcpy_h2d(p, host.data(), host.size(), nullptr) != 0 || ahpc_hip_stream_synchronize(nullptr) != 0)
            throw std::runtime_error("copy to device failed");
    }
    ~DeviceTensor() { ahpc_hip_free(p); }
    DeviceTensor(const DeviceTensor&) = delete;
    DeviceTensor& operator=(const DeviceTensor&) = delete;
};

Metrics run_config(size_t B, size_t N, size_t H, size_t d, const Options& opt) {
    Metrics m;
    try {
        auto attention = BackendFactory::createFlashAttention(BackendType::HIP);
        AttentionParams params;
        params.batch_size = B;
        params.sequence_length = N;
        params.num_heads = H;
        params.head_dimension = d;
        params.causal_mask = opt.causal;
        params.scale_factor = 1.0f / std::sqrt((float)d);
        attention->configure(params);

        const size_t n = B * N * H * d, bytes = n * elem_size(opt.dtype);
        auto q = random_tensor(n, opt.dtype, 1), k = random_tensor(n, opt.dtype, 2), v = random_tensor(n, opt.dtype, 3);
        std::vector<unsigned char> o(bytes, 0);
        const TensorShape shape({B, N, H, d}, opt.dtype, MemoryLayout::ROW_MAJOR);
        const void *pq = q.data(), *pk = k.data(), *pv = v.data();
        void* po = o.data();
        // backward operands: dO in, dQ, dK, dV out (:178-184)
        auto go = random_tensor(n, opt.dtype, 4);
        std::vector<unsigned char> gq(bytes, 0), gk(bytes, 0), gv(bytes, 0);
        const void* pgo = go.data();
        void *pgq = gq.data(), *pgk = gk.data(), *pgv = gv.data();
        std::unique_ptr<DeviceTensor> dq, dk, dv, dout, dgo, dgq, dgk, dgv;
        if (opt.device) {
            dq.reset(new DeviceTensor(q)); dk.reset(new DeviceTensor(k)); dv.reset(new DeviceTensor(v)); dout.reset(new DeviceTensor(o));
            dgo.reset(new DeviceTensor(go)); dgq.reset(new DeviceTensor(gq)); dgk.reset(new DeviceTensor(gk)); dgv.reset(new DeviceTensor(gv));
            pq = dq->p; pk = dk->p; pv = dv->p; po = dout->p;
            pgo = dgo->p; pgq = dgq->p; pgk = dgk->p; pgv = dgv->p;
        }
        m.memory_usage_bytes = m.peak_memory_bytes = 8 * bytes;  // Q, K, V, O, dO, dQ, dK, dV (the tracker of :186-191)

        for (int i = 0; i < opt.warmup; ++i) attention->forward(shape, pq, shape, pk, shape, pv, shape, po);
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < opt.iters; ++i) attention->forward(shape, pq, shape, pk, shape, pv, shape, po);
        const auto t1 = std::chrono::steady_clock::now();
        m.forward_time_ms = std::chrono::duration<double, std::milli>(t1 - t0).count() / opt.iters;
        // backward pass, timed like the forward (:215-235); one untimed call first
        attention->backward(shape, pgo, shape, pq, shape, pk, shape, pv, shape, pgq, shape, pgk, shape, pgv);
        const auto t2 = std::chrono::steady_clock::now();
        for (int i = 0; i < opt.iters; ++i)
            attention->backward(shape, pgo, shape, pq, shape, pk, shape, pv, shape, pgq, shape, pgk, shape, pgv);
        const auto t3 = std::chrono::steady_clock::now();
        m.backward_time_ms = std::chrono::duration<double, std::milli>(t3 - t2).count() / opt.iters;
        m.total_time_ms = m.forward_time_ms + m.backward_time_ms;
        const double flops = (double)B * H * N * N * d * 2;  // :241
        m.gflops = (flops / 1e9) / (m.total_time_ms / 1000.0);
        m.throughput_tokens_per_sec = (double)(B * N) / (m.forward_time_ms / 1000.0);
        m.success = true;
    } catch (const std::exception& e) {
        m.error_message = e.what();
        m.success = false;
    }
    return m;
}

struct PagedResult {
    size_t B = 0, N = 0, H = 0, d = 0;
    double forward_time_ms = 0.0, decode_time_ms = 0.0, bytes_per_second = 0.0, decode_kv_bytes_per_second = 0.0;
    bool success = false;
    std::string error_message;
};

// BM_PagedAttention, benchmarks/benchmark_attention.cpp:336-385
PagedResult run_paged_config(size_t B, size_t N, size_t H, size_t d, const Options& opt) {
    PagedResult r;
    r.B = B; r.N = N; r.H = H; r.d = d;
    try {
        auto attention = BackendFactory::createPagedAttention(BackendType::HIP);
        AttentionParams params;
        params.batch_size = B;
        params.sequence_length = 1;           // one query token per batch entry
        params.num_heads = H;
        params.head_dimension = d;
        params.max_sequence_length = N * 2;   // "allow for growth", :361
        params.page_size = 16;
        attention->configure(params);
        const size_t n_kv = B * N * H * d, n_q = B * H * d, es = elem_size(opt.dtype);
        auto q = random_tensor(n_q, opt.dtype, 11), k = random_tensor(n_kv, opt.dtype, 12), v = random_tensor(n_kv, opt.dtype, 13);
        std::vector<unsigned char> o(n_q * es, 0);
        const TensorShape q_shape({B, 1, H, d}, opt.dtype, MemoryLayout::ROW_MAJOR), kv_shape({B, N, H, d}, opt.dtype, MemoryLayout::ROW_MAJOR);
        const void *pq = q.data(), *pk = k.data(), *pv = v.data();
        void* po = o.data();
        std::unique_ptr<DeviceTensor> dq, dk, dv, dout;
        if (opt.device) {
            dq.reset(new DeviceTensor(q)); dk.reset(new DeviceTensor(k)); dv.reset(new DeviceTensor(v)); dout.reset(new DeviceTensor(o));
            pq = dq->p; pk = dk->p; pv = dv->p; po = dout->p;
        }
        for (int i = 0; i < opt.warmup; ++i) attention->forward(q_shape, pq, kv_shape, pk, kv_shape, pv, q_shape, po);
        auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < opt.iters; ++i) attention->forward(q_shape, pq, kv_shape, pk, kv_shape, pv, q_shape, po);
        auto t1 = std::chrono::steady_clock::now();
        r.forward_time_ms = std::chrono::duration<double, std::milli>(t1 - t0).count() / opt.iters;
        r.bytes_per_second = (double)(n_kv * es * 4) / (r.forward_time_ms / 1000.0);  // SetBytesProcessed, :381-382
        // the serving loop's step: caches resident, one token per sequence decoded
        PagedAttention& pa = dynamic_cast<PagedAttention&>(*attention);
        std::vector<size_t> ids(B);
        std::vector<TensorShape> shapes(B, TensorShape({1, 1, H, d}, opt.dtype, MemoryLayout::ROW_MAJOR));
        std::vector<const void*> qp(B);
        std::vector<void*> op(B);
        for (size_t b = 0; b < B; ++b) {
            ids[b] = pa.create_sequence(N * 2);
            pa.append_kv_cache(ids[b], static_cast<const unsigned char*>(pk) + b * N * H * d * es,
                               static_cast<const unsigned char*>(pv) + b * N * H * d * es, N, opt.dtype);
            qp[b] = static_cast<const unsigned char*>(pq) + b * H * d * es;
            op[b] = static_cast<unsigned char*>(po) + b * H * d * es;
        }
        for (int i = 0; i < opt.warmup; ++i) pa.forward_batch(ids, shapes, qp, shapes, op);
        t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < opt.iters; ++i) pa.forward_batch(ids, shapes, qp, shapes, op);
        t1 = std::chrono::steady_clock::now();
        r.decode_time_ms = std::chrono::duration<double, std::milli>(t1 - t0).count() / opt.iters;
        r.decode_kv_bytes_per_second = (double)(2 * n_kv * es) / (r.decode_time_ms / 1000.0);
        for (size_t id : ids) pa.destroy_sequence(id);
        r.success = true;
    } catch (const std::exception& e) {
        r.error_message = e.what();
    }
    return r;
}

void report_paged(const std::vector<PagedResult>& results) {
    std::cout << "\n=== PagedAttention (BM_PagedAttention configurations) ===\n";
    std::cout << std::left << std::setw(12) << "Backend" << std::setw(18) << "Config" << std::setw(15) << "Forward(ms)" << std::setw(15)
              << "Decode(ms)" << std::setw(16) << "Bytes/s (ref.)" << "KV GB/s (decode)\n";
    for (const PagedResult& r : results) {
        if (!r.success) continue;
        const std::string cfg = std::to_string(r.B) + "x" + std::to_string(r.N) + "x" + std::to_string(r.H) + "x" + std::to_string(r.d);
        std::cout << std::left << std::setw(12) << "HIP" << std::setw(18) << cfg << std::setw(15) << std::fixed << std::setprecision(3)
                  << r.forward_time_ms << std::setw(15) << r.decode_time_ms << std::setw(16) << std::scientific << std::setprecision(3)
                  << r.bytes_per_second << std::fixed << std::setprecision(2) << r.decode_kv_bytes_per_second / 1e9 << "\n";
    }
}

const char* dtype_name(DataType t) { return t == DataType::FLOAT32 ? "fp32" : t == DataType::FLOAT16 ? "fp16" : "bf16"; }

void report(const std::vector<Result>& results) {  // GeneratePerformanceReport, :529-620
    std::cout << "\n=== Performance Report ===\n";
    std::cout << std::left << std::setw(12) << "Backend" << std::setw(18) << "Config" << std::setw(15) << "Forward(ms)"
              << std::setw(15) << "Backward(ms)" << std::setw(14) << "GFLOPS" << std::setw(15) << "Tokens/sec" << std::setw(12)
              << "Memory(MB)" << "\n";
    const Result *best_tp = nullptr, *best_gf = nullptr;
    for (const Result& r : results) {
        if (!r.m.success) continue;
        const std::string cfg = std::to_string(r.B) + "x" + std::to_string(r.N) + "x" + std::to_string(r.H) + "x" + std::to_string(r.d);
        std::cout << std::left << std::setw(12) << "HIP" << std::setw(18) << cfg << std::setw(15) << std::fixed << std::setprecision(3)
                  << r.m.forward_time_ms << std::setw(15) << r.m.backward_time_ms << std::setw(14) << std::setprecision(1) << r.m.gflops
                  << std::setw(15) << std::setprecision(0) << r.m.throughput_tokens_per_sec << std::setw(12) << std::setprecision(1)
                  << r.m.peak_memory_bytes / 1024.0 / 1024.0 << "\n";
        if (!best_tp || r.m.throughput_tokens_per_sec > best_tp->m.throughput_tokens_per_sec) best_tp = &r;
        if (!best_gf || r.m.gflops > best_gf->m.gflops) best_gf = &r;
    }
    std::cout << "\n=== Best Performing Configurations ===\n";
    if (best_tp) std::cout << "Best Throughput: HIP with " << std::fixed << std::setprecision(0) << best_tp->m.throughput_tokens_per_sec << " tokens/sec\n";
    if (best_gf) std::cout << "Best GFLOPS: HIP with " << std::fixed << std::setprecision(2) << best_gf->m.gflops << " GFLOPS\n";
}

bool save_json(const std::vector<Result>& results, const std::vector<PagedResult>& paged, const Options& opt) {  // SaveResultsToJSON, :625-669
    std::ofstream f(opt.json);
    if (!f) return false;
    f << "{\n  \"benchmark_results\": [\n";
    for (size_t i = 0; i < results.size(); ++i) {
        const Result& r = results[i];
        f << "    {\n";
        f << "      \"backend\": \"HIP\",\n";
        f << "      \"batch_size\": " << r.B << ",\n      \"sequence_length\": " << r.N << ",\n      \"num_heads\": " << r.H
          << ",\n      \"head_dimension\": " << r.d << ",\n      \"total_elements\": " << r.total_elements() << ",\n";
        f << "      \"data_type\": \"" << dtype_name(opt.dtype) << "\",\n      \"tensors_resident_on_device\": " << (opt.device ? "true" : "false") << ",\n";
        f << "      \"success\": " << (r.m.success ? "true" : "false") << ",\n";
        if (r.m.success) {
            f << "      \"forward_time_ms\": " << r.m.forward_time_ms << ",\n      \"backward_time_ms\": " << r.m.backward_time_ms
              << ",\n      \"total_time_ms\": " << r.m.total_time_ms << ",\n      \"memory_usage_bytes\": " << r.m.memory_usage_bytes
              << ",\n      \"peak_memory_bytes\": " << r.m.peak_memory_bytes << ",\n      \"gflops\": " << r.m.gflops
              << ",\n      \"throughput_tokens_per_sec\": " << r.m.throughput_tokens_per_sec << ",\n      \"theoretical_flops\": "
              << r.theoretical_flops() << "\n";
        } else {
            f << "      \"error_message\": \"" << r.m.error_message << "\"\n";
        }
        f << "    }" << (i + 1 < results.size() ? "," : "") << "\n";
    }
    f << "  ],\n  \"paged_results\": [\n";
    for (size_t i = 0; i < paged.size(); ++i) {
        const PagedResult& r = paged[i];
        f << "    {\n      \"backend\": \"HIP\",\n      \"batch_size\": " << r.B << ",\n      \"sequence_length\": " << r.N
          << ",\n      \"num_heads\": " << r.H << ",\n      \"head_dimension\": " << r.d << ",\n      \"page_size\": 16,\n";
        f << "      \"data_type\": \"" << dtype_name(opt.dtype) << "\",\n      \"tensors_resident_on_device\": " << (opt.device ? "true" : "false") << ",\n";
        f << "      \"success\": " << (r.success ? "true" : "false") << ",\n";
        if (r.success)
            f << "      \"forward_time_ms\": " << r.forward_time_ms << ",\n      \"bytes_per_second\": " << r.bytes_per_second
              << ",\n      \"decode_time_ms\": " << r.decode_time_ms << ",\n      \"decode_kv_bytes_per_second\": "
              << r.decode_kv_bytes_per_second << "\n";
        else
            f << "      \"error_message\": \"" << r.error_message << "\"\n";
        f << "    }" << (i + 1 < paged.size() ? "," : "") << "\n";
    }
    f << "  ],\n  \"config\": {\n    \"warmup_iterations\": " << opt.warmup << ",\n    \"benchmark_iterations\": " << opt.iters
      << ",\n    \"causal_mask\": " << (opt.causal ? "true" : "false") << "\n  }\n}\n";
    return true;
}

// save_results_to_csv, examples/performance_comparison.cpp:431-463: same header, same precisions
bool save_csv(const std::vector<Result>& results, const std::string& filename) {
    std::ofstream file(filename);
    if (!file.is_open()) return false;
    file << "Backend,BatchSize,SequenceLength,NumHeads,HeadDimension,";
    file << "ForwardTimeMs,BackwardTimeMs,TotalTimeMs,MemoryUsageMB,PeakMemoryMB,";
    file << "ThroughputTokensPerSec,GFLOPS,Success,ErrorMessage" << std::endl;
    for (const Result& r : results) {
        file << "HIP" << "," << r.B << "," << r.N << "," << r.H << "," << r.d << ","
             << std::fixed << std::setprecision(6) << r.m.forward_time_ms << ","
             << std::fixed << std::setprecision(6) << r.m.backward_time_ms << ","
             << std::fixed << std::setprecision(6) << r.m.total_time_ms << ","
             << std::fixed << std::setprecision(2) << r.m.memory_usage_bytes / 1024.0 / 1024.0 << ","
             << std::fixed << std::setprecision(2) << r.m.peak_memory_bytes / 1024.0 / 1024.0 << ","
             << std::fixed << std::setprecision(0) << r.m.throughput_tokens_per_sec << ","
             << std::fixed << std::setprecision(4) << r.m.gflops << ","
             << (r.m.success ? "true" : "false") << ","
             << "\"" << r.m.error_message << "\"" << std::endl;
    }
    return true;
}

}  // namespace

int main(int argc, char** argv) {
    Options opt;
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        if (a == "--device") opt.device = true;
        else if (a == "--causal") opt.causal = true;
        else if (a == "--quick") opt.quick = true;
        else if (a == "--json" && i + 1 < argc) opt.json = argv[++i];
        else if (a == "--csv" && i + 1 < argc) opt.csv = argv[++i];
        else if (a == "--dtype" && i + 1 < argc) {
            const std::string t = argv[++i];
            opt.dtype = t == "fp16" ? DataType::FLOAT16 : t == "bf16" ? DataType::BFLOAT16 : DataType::FLOAT32;
        } else {
            std::cerr << "usage: ahpc_bench_report [--device] [--dtype fp32|fp16|bf16] [--causal] [--quick] [--json FILE] [--csv FILE]\n";
            return 2;
        }
    }
    if (!BackendFactory::isBackendAvailable(BackendType::HIP)) {
        std::cerr << "ahpc_bench_report: the HIP backend is not available (no GPU)\n";
        return 1;
    }
    // BenchmarkConfig, benchmarks/benchmark_attention.cpp:27-32
    std::vector<size_t> batches = {1, 2, 4, 8}, seqs = {64, 128, 256, 512, 1024, 2048}, heads = {1, 4, 8, 12, 16}, dims = {64, 128};
    if (opt.quick) { batches = {1, 4}; seqs = {128, 1024, 2048}; heads = {8, 16}; dims = {64, 128}; }
    std::cout << "Running comprehensive attention benchmarks (HIP backend, " << dtype_name(opt.dtype) << ", tensors "
              << (opt.device ? "resident on the device" : "in host memory") << ")...\n";
    std::vector<Result> results;
    for (size_t B : batches)
        for (size_t N : seqs)
            for (size_t H : heads)
                for (size_t d : dims) {
                    if (B * N * H * d > 50000000) continue;  // :490-493
                    Result r{B, N, H, d, run_config(B, N, H, d, opt)};
                    std::cout << "  Testing config: batch=" << B << ", seq_len=" << N << ", heads=" << H << ", head_dim=" << d;
                    if (r.m.success) std::cout << " - OK (" << std::fixed << std::setprecision(3) << r.m.forward_time_ms << "ms)\n";
                    else std::cout << " - FAILED (" << r.m.error_message << ")\n";
                    results.push_back(r);
                }
    report(results);
    // PagedAttention: the subset BM_PagedAttention is registered for, benchmarks/benchmark_attention.cpp:436-457
    std::vector<PagedResult> paged;
    for (size_t N : {256, 512, 1024})
        for (size_t H : {4, 8})
            for (size_t d : {64, 128}) {
                paged.push_back(run_paged_config(2, N, H, d, opt));
                const PagedResult& r = paged.back();
                std::cout << "  Testing paged config: batch=2, seq_len=" << N << ", heads=" << H << ", head_dim=" << d;
                if (r.success) std::cout << " - OK (" << std::fixed << std::setprecision(3) << r.forward_time_ms << "ms)\n";
                else std::cout << " - FAILED (" << r.error_message << ")\n";
            }
    report_paged(paged);
    if (!save_json(results, paged, opt)) {
        std::cerr << "Failed to open file for writing: " << opt.json << "\n";
        return 1;
    }
    std::cout << "Results saved to " << opt.json << "\n";
    if (!opt.csv.empty()) {
        if (!save_csv(results, opt.csv)) {
            std::cerr << "Failed to open file for writing: " << opt.csv << "\n";
            return 1;
        }
        std::cout << "\nResults saved to: " << opt.csv << "\n";
    }
    for (const Result& r : results)
        if (!r.m.success) return 1;
    for (const PagedResult& r : paged)
        if (!r.success) return 1;
    return 0;
}
