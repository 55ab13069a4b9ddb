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

bool save_json(const std::vector<Result>& results, const Options& opt) {  // SaveResultsToJSON, :625-669
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
    if (!save_json(results, opt)) {
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
    return 0;
}
