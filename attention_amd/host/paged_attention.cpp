// PagedAttention (HIP backend): sequence bookkeeping on the host, KV pages and block table in HBM,
// batched decode through the C ABI.
#include "algorithms/paged_attention.hpp"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>
#include <mutex>
#include <unordered_map>

#include "hip_support.hpp"

namespace attention_hpc {

using hipsup::check;

namespace {
struct Sequence {
    size_t id = 0;
    int32_t row = -1;                 // row of the device block table
    std::vector<int32_t> pages;
    size_t total_tokens = 0;
    size_t max_length = 0;
    bool active = true;
};
}  // namespace

struct PagedAttention::Impl {
    PagedAttentionConfig cfg;
    bool configured = false;
    size_t H = 0, d = 0, P = 16;  // H = query heads
    size_t Hkv = 0;               // heads stored in the pool (AttentionParams::key_value_heads, 0 = H)
    size_t max_pages = 0;             // columns of the block table
    size_t n_rows = 0;                // rows of the block table

    std::unique_ptr<KVBlockPool> pool;
    std::unordered_map<size_t, Sequence> seqs;
    std::vector<int32_t> free_rows;
    size_t next_id = 1;
    mutable std::mutex seq_mutex;     // sequences, table mirror, pool pointer
    std::mutex run_mutex;             // serialises device work of this instance

    // host mirror (the truth) and device copy of the block table and lengths
    std::vector<int32_t> table;       // [n_rows][max_pages], -1 = none
    std::vector<int32_t> lens;        // [n_rows]
    hipsup::DeviceBuffer d_table, d_lens;
    bool table_dirty = true;

    hipsup::Stream stream;
    hipsup::DeviceBuffer d_in_k, d_in_v, d_q, d_o, d_rows, d_ws, d_tmp_k, d_tmp_v;
    hipsup::PinnedBuffer h_q, h_o, h_rows;
    size_t peak_bytes = 0;
    std::vector<std::pair<std::string, double>> profile;

    size_t page_bytes() const { return pool ? pool->stats().page_bytes : 0; }

    void resize_table_locked(size_t rows, size_t cols) {
        std::vector<int32_t> nt(rows * cols, -1);
        for (size_t r = 0; r < std::min(rows, n_rows); ++r)
            std::copy_n(table.begin() + r * max_pages, std::min(cols, max_pages), nt.begin() + r * cols);
        table.swap(nt);
        lens.resize(rows, 0);
        for (size_t r = n_rows; r < rows; ++r) free_rows.push_back(static_cast<int32_t>(r));
        // lowest row first, so that rows are handed out in ascending order
        std::sort(free_rows.begin(), free_rows.end(), std::greater<int32_t>());
        n_rows = rows;
        max_pages = cols;
        table_dirty = true;
    }

    void ensure_pool_locked(DataType dtype) {
        if (pool) return;
        const DataType dt = cfg.kv_cache_dtype >= 0 ? static_cast<DataType>(cfg.kv_cache_dtype) : dtype;
        pool.reset(new KVBlockPool(P, Hkv, d, dt, cfg.initial_page_pool_size, cfg.page_pool_growth, cfg.device_pool_max_bytes));
    }

    void release_pages_locked(Sequence& s, size_t keep_pages) {
        while (s.pages.size() > keep_pages) {
            pool->deallocate_page(s.pages.back());
            s.pages.pop_back();
            table[s.row * max_pages + s.pages.size()] = -1;
        }
        table_dirty = true;
    }

    void grow_pages_locked(Sequence& s, size_t want_pages) {
        if (want_pages > max_pages) resize_table_locked(n_rows, std::max(want_pages, max_pages * 2));
        while (s.pages.size() < want_pages) {
            const int32_t id = pool->allocate_page();
            table[s.row * max_pages + s.pages.size()] = id;
            s.pages.push_back(id);
        }
        table_dirty = true;
        peak_bytes = std::max(peak_bytes, pool->get_allocated_pages() * page_bytes());
    }

    // Uploads the mirror when it changed.  Synchronous: the mirror may be modified right after.
    void sync_table_locked() {
        if (!table_dirty) return;
        void* dt = d_table.reserve(std::max<size_t>(table.size(), 1) * sizeof(int32_t));
        void* dl = d_lens.reserve(std::max<size_t>(lens.size(), 1) * sizeof(int32_t));
        check(ahpc_hip_memcpy_h2d(dt, table.data(), table.size() * sizeof(int32_t), stream.get()), "block table upload");
        check(ahpc_hip_memcpy_h2d(dl, lens.data(), lens.size() * sizeof(int32_t), stream.get()), "sequence lengths upload");
        stream.sync();
        table_dirty = false;
    }

    void append_many(const std::vector<size_t>& ids, const std::vector<size_t>& counts, const void* key_data,
                     const void* value_data, size_t total_rows, DataType dt, int64_t stride_b, int64_t stride_n,
                     const int32_t* cu_seqlens, size_t n_max);

    Sequence& find_locked(size_t id) {
        auto it = seqs.find(id);
        if (it == seqs.end()) throw AttentionException(AttentionError::INVALID_INPUT, "Sequence not found");
        return it->second;
    }
};

PagedAttention::PagedAttention() : impl_(new Impl) {}
PagedAttention::~PagedAttention() { delete impl_; }

// Reference: PagedAttention::configure, src/algorithms/paged_attention.cpp:98-117.  The pool itself is
// created at the first append (its element type is the type of the data that arrives, unless
// PagedAttentionConfig::kv_cache_dtype fixes it).
void PagedAttention::configure(const AttentionParams& params, const PerformanceConfig& perf_config) {
    if (params.batch_size == 0 || params.sequence_length == 0 || params.num_heads == 0 || params.head_dimension == 0)
        throw AttentionException(AttentionError::INVALID_PARAMETERS, "Invalid attention parameters: dimensions must be positive");
    // Grouped key/value heads: the pool stores key_value_heads heads per token and every one of them serves
    // num_heads / key_value_heads consecutive query heads (any number of them; see ahpc_hip_paged_decode_gqa for the
    // kernel a group size runs on).
    if (params.key_value_heads != 0) {
        if (params.key_value_heads > params.num_heads || params.num_heads % params.key_value_heads)
            throw AttentionException(AttentionError::INVALID_PARAMETERS, "key_value_heads must divide num_heads");
    }
    if (params.page_size == 0) throw AttentionException(AttentionError::INVALID_PARAMETERS, "page_size must be positive");
    const size_t d = params.head_dimension;
    // whole 16-byte pieces of the cache's type, which is known at the first append only: a multiple of 4 passes here,
    // a 16-bit cache then needs a multiple of 8 (the decode call reports it otherwise)
    if (d > 256 || d % 4)
        throw AttentionException(AttentionError::UNSUPPORTED_OPERATION,
                                 "paged decode supports head_dimension up to 256 in whole 16-byte pieces");
    int n = 0;
    ahpc_hip_device_count(&n);
    if (n < 1) throw AttentionException(AttentionError::BACKEND_NOT_AVAILABLE, "no HIP device");

    std::lock_guard<std::mutex> run(impl_->run_mutex);
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    current_params_ = params;
    current_perf_config_ = perf_config;
    if (perf_config.enable_profiling) profiling_enabled_ = true;
    Impl& m = *impl_;
    m.seqs.clear();
    m.pool.reset();
    m.free_rows.clear();
    m.table.clear();
    m.lens.clear();
    m.n_rows = m.max_pages = 0;
    m.next_id = 1;
    m.H = params.num_heads;
    m.Hkv = params.key_value_heads ? params.key_value_heads : params.num_heads;
    m.d = d;
    m.P = params.page_size;
    m.cfg.page_size = m.P;
    const size_t longest = std::max(params.max_sequence_length, params.sequence_length);
    const size_t cols = std::max(m.cfg.max_pages_per_sequence, (longest + m.P - 1) / m.P);
    const size_t rows = std::max(m.cfg.max_concurrent_sequences, params.batch_size);
    m.resize_table_locked(rows, cols);
    m.configured = true;
}

void PagedAttention::configure_paged_attention(const PagedAttentionConfig& paged_config) {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    impl_->cfg = paged_config;
    if (impl_->configured) {
        // takes effect for the table immediately; pool geometry changes need a new configure()
        impl_->cfg.page_size = impl_->P;
        const size_t rows = std::max(impl_->n_rows, paged_config.max_concurrent_sequences);
        const size_t cols = std::max(impl_->max_pages, paged_config.max_pages_per_sequence);
        if (rows != impl_->n_rows || cols != impl_->max_pages) impl_->resize_table_locked(rows, cols);
    }
}

// ---- sequences (reference: src/algorithms/paged_attention.cpp:333-432) -------------------------------

size_t PagedAttention::create_sequence(size_t max_length) {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    Impl& m = *impl_;
    if (!m.configured) throw AttentionException(AttentionError::INVALID_PARAMETERS, "PagedAttention not configured. Call configure() first.");
    if (m.free_rows.empty()) m.resize_table_locked(std::max<size_t>(m.n_rows * 2, 1), m.max_pages);
    Sequence s;
    s.id = m.next_id++;
    s.row = m.free_rows.back();
    m.free_rows.pop_back();
    s.max_length = max_length;
    m.lens[s.row] = 0;
    m.table_dirty = true;
    m.seqs.emplace(s.id, std::move(s));
    return m.next_id - 1;
}

void PagedAttention::destroy_sequence(size_t sequence_id) {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    Impl& m = *impl_;
    auto it = m.seqs.find(sequence_id);
    if (it == m.seqs.end()) return;
    if (m.pool) m.release_pages_locked(it->second, 0);
    m.lens[it->second.row] = 0;
    m.free_rows.push_back(it->second.row);
    m.table_dirty = true;
    m.seqs.erase(it);
}

void PagedAttention::reset_sequence(size_t sequence_id) {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    Impl& m = *impl_;
    auto it = m.seqs.find(sequence_id);
    if (it == m.seqs.end()) return;
    if (m.pool) m.release_pages_locked(it->second, 0);
    it->second.total_tokens = 0;
    it->second.active = true;
    m.lens[it->second.row] = 0;
    m.table_dirty = true;
}

bool PagedAttention::is_sequence_active(size_t sequence_id) const {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    auto it = impl_->seqs.find(sequence_id);
    return it != impl_->seqs.end() && it->second.active;
}

void PagedAttention::extend_sequence(size_t sequence_id, size_t additional_tokens) {
    // taking pages can move the pool's slabs (growth copies them and frees the old ones): no append, read-back or
    // decode of this instance may be between reading the slab pointers and the end of its device work meanwhile
    std::lock_guard<std::mutex> run(impl_->run_mutex);
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    Impl& m = *impl_;
    auto it = m.seqs.find(sequence_id);
    if (it == m.seqs.end()) return;
    Sequence& s = it->second;
    s.max_length += additional_tokens;
    if (m.pool) m.grow_pages_locked(s, (s.max_length + m.P - 1) / m.P);  // pre-allocate, as the reference does
}

void PagedAttention::truncate_sequence(size_t sequence_id, size_t new_length) {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    Impl& m = *impl_;
    auto it = m.seqs.find(sequence_id);
    if (it == m.seqs.end()) return;
    Sequence& s = it->second;
    if (new_length < s.total_tokens) {
        s.total_tokens = new_length;
        m.lens[s.row] = static_cast<int32_t>(new_length);
        if (m.pool) m.release_pages_locked(s, (new_length + m.P - 1) / m.P);
        m.table_dirty = true;
    }
    s.max_length = new_length;
}

size_t PagedAttention::get_sequence_length(size_t sequence_id) const {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    auto it = impl_->seqs.find(sequence_id);
    return it != impl_->seqs.end() ? it->second.total_tokens : 0;
}

size_t PagedAttention::get_max_sequence_length(size_t sequence_id) const {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    auto it = impl_->seqs.find(sequence_id);
    return it != impl_->seqs.end() ? it->second.max_length : 0;
}

std::vector<int32_t> PagedAttention::get_sequence_pages(size_t sequence_id) const {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    auto it = impl_->seqs.find(sequence_id);
    return it != impl_->seqs.end() ? it->second.pages : std::vector<int32_t>{};
}

// ---- KV cache (reference: src/algorithms/paged_attention.cpp:434-494) ---------------------------------

void PagedAttention::append_kv_cache(size_t sequence_id, const void* key_data, const void* value_data, size_t num_tokens,
                                     DataType data_type) {
    if (num_tokens == 0) return;
    if (!key_data || !value_data) throw AttentionException(AttentionError::INVALID_INPUT, "null key/value pointer");
    std::lock_guard<std::mutex> run(impl_->run_mutex);
    Impl& m = *impl_;
    int32_t row;
    size_t start;
    {
        std::lock_guard<std::mutex> lock(m.seq_mutex);
        Sequence& s = m.find_locked(sequence_id);
        m.ensure_pool_locked(data_type);
        m.grow_pages_locked(s, (s.total_tokens + num_tokens + m.P - 1) / m.P);
        row = s.row;
        start = s.total_tokens;
        m.sync_table_locked();
    }
    void* st = m.stream.get();
    const size_t bytes = num_tokens * m.Hkv * m.d * hipsup::dtype_size(data_type);
    const void* dk = key_data;
    const void* dv = value_data;
    if (!hipsup::is_device_pointer(key_data)) {
        check(ahpc_hip_memcpy_h2d(m.d_in_k.reserve(bytes), key_data, bytes, st), "copy keys to device");
        dk = m.d_in_k.get();
    }
    if (!hipsup::is_device_pointer(value_data)) {
        check(ahpc_hip_memcpy_h2d(m.d_in_v.reserve(bytes), value_data, bytes, st), "copy values to device");
        dv = m.d_in_v.get();
    }
    check(ahpc_hip_kv_scatter(dk, dv, hipsup::dtype_code(data_type), m.pool->k_slab(), m.pool->v_slab(),
                              hipsup::dtype_code(m.pool->dtype()), static_cast<const int32_t*>(m.d_table.get()),
                              (int64_t)m.max_pages, nullptr, nullptr, row, (int64_t)start, (int64_t)num_tokens, (int64_t)m.Hkv,
                              (int64_t)m.d, (int64_t)m.P, st), "KV scatter");
    m.stream.sync();
    {
        std::lock_guard<std::mutex> lock(m.seq_mutex);
        auto it = m.seqs.find(sequence_id);
        if (it != m.seqs.end()) {
            it->second.total_tokens = start + num_tokens;
            m.lens[row] = static_cast<int32_t>(start + num_tokens);
            m.table_dirty = true;
        }
    }
}

namespace {
struct BatchAppend {
    std::vector<int32_t> rows, start, count;
};
}  // namespace

void PagedAttention::append_kv_cache_batch(const std::vector<size_t>& sequence_ids, const TensorShape& kv_shape,
                                           const void* key_data, const void* value_data, const std::vector<size_t>& num_tokens) {
    Impl& m = *impl_;
    if (!m.configured) throw AttentionException(AttentionError::INVALID_PARAMETERS, "PagedAttention not configured. Call configure() first.");
    if (!key_data || !value_data) throw AttentionException(AttentionError::INVALID_INPUT, "null key/value pointer");
    const auto& dm = kv_shape.dimensions;
    if (dm.size() != 4 || dm[0] != sequence_ids.size() || dm[2] != m.Hkv || dm[3] != m.d || (!num_tokens.empty() && num_tokens.size() != dm[0]))
        throw AttentionException(AttentionError::INVALID_INPUT, "expected [sequences, tokens, key_value_heads, head_dim] and one count per sequence");
    const size_t B = dm[0], N = dm[1];
    std::vector<size_t> counts(B, N);
    for (size_t b = 0; b < num_tokens.size(); ++b) {
        if (num_tokens[b] > N) throw AttentionException(AttentionError::INVALID_INPUT, "num_tokens exceeds the tensor's sequence dimension");
        counts[b] = num_tokens[b];
    }
    if (B == 0 || N == 0) return;
    m.append_many(sequence_ids, counts, key_data, value_data, B * N, kv_shape.data_type, (int64_t)(N * m.Hkv * m.d),
                (int64_t)(m.Hkv * m.d), nullptr, N);
}

void PagedAttention::append_kv_cache_packed(const std::vector<size_t>& sequence_ids, const TensorShape& kv_shape,
                                            const void* key_data, const void* value_data, const int32_t* cu_seqlens) {
    Impl& m = *impl_;
    if (!m.configured) throw AttentionException(AttentionError::INVALID_PARAMETERS, "PagedAttention not configured. Call configure() first.");
    if (!key_data || !value_data || !cu_seqlens) throw AttentionException(AttentionError::INVALID_INPUT, "null pointer");
    const auto& dm = kv_shape.dimensions;
    const size_t B = sequence_ids.size();
    if (dm.size() != 3 || dm[1] != m.Hkv || dm[2] != m.d)
        throw AttentionException(AttentionError::INVALID_INPUT, "packed tensors must be [total_tokens, key_value_heads, head_dim]");
    if (B == 0) return;
    if (cu_seqlens[0] != 0 || (size_t)cu_seqlens[B] != dm[0]) throw AttentionException(AttentionError::INVALID_INPUT, "cu_seqlens must run from 0 to total_tokens");
    std::vector<size_t> counts(B);
    size_t n_max = 0;
    for (size_t b = 0; b < B; ++b) {
        if (cu_seqlens[b + 1] < cu_seqlens[b]) throw AttentionException(AttentionError::INVALID_INPUT, "cu_seqlens must not decrease");
        counts[b] = (size_t)(cu_seqlens[b + 1] - cu_seqlens[b]);
        n_max = std::max(n_max, counts[b]);
    }
    if (n_max == 0) return;
    m.append_many(sequence_ids, counts, key_data, value_data, dm[0], kv_shape.data_type, 0, (int64_t)(m.Hkv * m.d), cu_seqlens, n_max);
}

// Shared by the dense and the packed hand-off: reserves pages for every sequence, uploads the table and the
// index arrays, scatters with one launch, then publishes the new lengths.
void PagedAttention::Impl::append_many(const std::vector<size_t>& ids, const std::vector<size_t>& counts, const void* key_data,
                                       const void* value_data, size_t total_rows, DataType dt, int64_t stride_b,
                                       int64_t stride_n, const int32_t* cu_seqlens, size_t n_max) {
    Impl& m = *this;
    std::lock_guard<std::mutex> run(m.run_mutex);
    const size_t B = ids.size();
    BatchAppend ba;
    {
        std::lock_guard<std::mutex> lock(m.seq_mutex);
        for (size_t b = 0; b < B; ++b)  // every id must exist before anything is changed
            m.find_locked(ids[b]);
        for (size_t b = 0; b < B; ++b)
            for (size_t c = b + 1; c < B; ++c)
                if (ids[b] == ids[c]) throw AttentionException(AttentionError::INVALID_INPUT, "a sequence may appear only once in a batched append");
        m.ensure_pool_locked(dt);
        for (size_t b = 0; b < B; ++b) {
            Sequence& s = m.find_locked(ids[b]);
            m.grow_pages_locked(s, (s.total_tokens + counts[b] + m.P - 1) / m.P);
            ba.rows.push_back(s.row);
            ba.start.push_back((int32_t)s.total_tokens);
            ba.count.push_back((int32_t)counts[b]);
        }
        m.sync_table_locked();
    }
    void* st = m.stream.get();
    const size_t bytes = total_rows * m.Hkv * m.d * hipsup::dtype_size(dt);
    const void* dk = key_data;
    const void* dv = value_data;
    if (!hipsup::is_device_pointer(key_data)) {
        check(ahpc_hip_memcpy_h2d(m.d_in_k.reserve(bytes), key_data, bytes, st), "copy keys to device");
        dk = m.d_in_k.get();
    }
    if (!hipsup::is_device_pointer(value_data)) {
        check(ahpc_hip_memcpy_h2d(m.d_in_v.reserve(bytes), value_data, bytes, st), "copy values to device");
        dv = m.d_in_v.get();
    }
    // index arrays: rows | start | count | cu_seqlens, one upload
    std::vector<int32_t> idx;
    idx.insert(idx.end(), ba.rows.begin(), ba.rows.end());
    idx.insert(idx.end(), ba.start.begin(), ba.start.end());
    idx.insert(idx.end(), ba.count.begin(), ba.count.end());
    if (cu_seqlens) idx.insert(idx.end(), cu_seqlens, cu_seqlens + B + 1);
    int32_t* didx = static_cast<int32_t*>(m.d_rows.reserve(idx.size() * sizeof(int32_t)));
    check(ahpc_hip_memcpy_h2d(didx, idx.data(), idx.size() * sizeof(int32_t), st), "copy index arrays");
    check(ahpc_hip_kv_scatter_batch(dk, dv, hipsup::dtype_code(dt), stride_b, stride_n, m.pool->k_slab(), m.pool->v_slab(),
                                    hipsup::dtype_code(m.pool->dtype()), static_cast<const int32_t*>(m.d_table.get()),
                                    (int64_t)m.max_pages, didx, didx + B, cu_seqlens ? nullptr : didx + 2 * B,
                                    cu_seqlens ? didx + 3 * B : nullptr, (int64_t)B, (int64_t)n_max, (int64_t)m.Hkv, (int64_t)m.d,
                                    (int64_t)m.P, st), "batched KV scatter");
    m.stream.sync();
    {
        std::lock_guard<std::mutex> lock(m.seq_mutex);
        for (size_t b = 0; b < B; ++b) {
            auto it = m.seqs.find(ids[b]);
            if (it == m.seqs.end()) continue;
            it->second.total_tokens = (size_t)ba.start[b] + counts[b];
            m.lens[ba.rows[b]] = (int32_t)it->second.total_tokens;
        }
        m.table_dirty = true;
    }
}

void PagedAttention::get_kv_cache(size_t sequence_id, void* key_data, void* value_data, size_t start_token, size_t num_tokens,
                                  DataType data_type) {
    if (num_tokens == 0) return;
    if (!key_data || !value_data) throw AttentionException(AttentionError::INVALID_INPUT, "null key/value pointer");
    std::lock_guard<std::mutex> run(impl_->run_mutex);
    Impl& m = *impl_;
    int32_t row;
    {
        std::lock_guard<std::mutex> lock(m.seq_mutex);
        Sequence& s = m.find_locked(sequence_id);
        if (start_token + num_tokens > s.total_tokens)
            throw AttentionException(AttentionError::INVALID_INPUT, "requested tokens are beyond the cached length");
        row = s.row;
        m.sync_table_locked();
    }
    void* st = m.stream.get();
    const size_t bytes = num_tokens * m.Hkv * m.d * hipsup::dtype_size(data_type);
    const bool kdev = hipsup::is_device_pointer(key_data), vdev = hipsup::is_device_pointer(value_data);
    void* dk = kdev ? key_data : m.d_tmp_k.reserve(bytes);
    void* dv = vdev ? value_data : m.d_tmp_v.reserve(bytes);
    check(ahpc_hip_kv_gather(dk, dv, hipsup::dtype_code(data_type), m.pool->k_slab(), m.pool->v_slab(),
                             hipsup::dtype_code(m.pool->dtype()), static_cast<const int32_t*>(m.d_table.get()),
                             (int64_t)m.max_pages, row, (int64_t)start_token, (int64_t)num_tokens, (int64_t)m.Hkv, (int64_t)m.d,
                             (int64_t)m.P, st), "KV gather");
    if (!kdev) check(ahpc_hip_memcpy_d2h(key_data, dk, bytes, st), "copy keys from device");
    if (!vdev) check(ahpc_hip_memcpy_d2h(value_data, dv, bytes, st), "copy values from device");
    m.stream.sync();
}

void PagedAttention::clear_kv_cache(size_t sequence_id) { reset_sequence(sequence_id); }

// ---- decode ---------------------------------------------------------------------------------------------

static bool decode_shape_ok(const TensorShape& s, size_t H, size_t d) {
    const auto& v = s.dimensions;
    if (v.size() < 2 || v.size() > 4) return false;
    if (v[v.size() - 1] != d || v[v.size() - 2] != H) return false;
    for (size_t i = 0; i + 2 < v.size(); ++i)
        if (v[i] != 1) return false;
    return true;
}

// Reference: PagedAttention::forward_batch, src/algorithms/paged_attention.cpp:496-547 (size check and
// INVALID_INPUT :511-516).  The reference walks the sequences one by one on the host; here the queries
// are packed to [B,H,d] and the whole batch is one launch.
void PagedAttention::forward_batch(const std::vector<size_t>& ids, const std::vector<TensorShape>& q_shapes,
                                   const std::vector<const void*>& q_data, const std::vector<TensorShape>& o_shapes,
                                   const std::vector<void*>& o_data, const std::vector<const void*>& masks) {
    Impl& m = *impl_;
    if (!m.configured)
        throw AttentionException(AttentionError::INVALID_PARAMETERS, "PagedAttention not configured. Call configure() first.");
    const size_t B = ids.size();
    if (B != q_shapes.size() || B != q_data.size() || B != o_shapes.size() || B != o_data.size())
        throw AttentionException(AttentionError::INVALID_INPUT, "Batch input sizes mismatch");
    if (B == 0) return;
    for (const void* mk : masks)
        if (mk) throw AttentionException(AttentionError::UNSUPPORTED_OPERATION, "decode attends to the whole cached context; masks are not supported");
    const DataType qdt = q_shapes[0].data_type;
    for (size_t i = 0; i < B; ++i) {
        if (!q_data[i] || !o_data[i]) throw AttentionException(AttentionError::INVALID_INPUT, "null query/output pointer");
        if (!decode_shape_ok(q_shapes[i], m.H, m.d) || !decode_shape_ok(o_shapes[i], m.H, m.d))
            throw AttentionException(AttentionError::INVALID_INPUT, "decode tensors must be one token of [heads, head_dim]");
        if (q_shapes[i].data_type != qdt || o_shapes[i].data_type != qdt)
            throw AttentionException(AttentionError::INVALID_INPUT, "all decode tensors of a batch must share one data type");
    }

    std::lock_guard<std::mutex> run(m.run_mutex);
    const auto wall0 = std::chrono::steady_clock::now();
    void* st = m.stream.get();
    const size_t row_bytes = m.H * m.d * hipsup::dtype_size(qdt);
    int32_t* rows = static_cast<int32_t*>(m.h_rows.reserve(B * sizeof(int32_t)));
    size_t max_len = 0;
    {
        std::lock_guard<std::mutex> lock(m.seq_mutex);
        for (size_t i = 0; i < B; ++i) {
            Sequence& s = m.find_locked(ids[i]);
            rows[i] = s.row;
            max_len = std::max(max_len, s.total_tokens);
        }
        m.sync_table_locked();
    }
    unsigned char* dq = static_cast<unsigned char*>(m.d_q.reserve(B * row_bytes));
    unsigned char* dout = static_cast<unsigned char*>(m.d_o.reserve(B * row_bytes));
    if (max_len == 0 || !m.pool) {  // nothing cached anywhere: zero rows
        check(ahpc_hip_memset(dout, 0, B * row_bytes, st), "clear output");
    } else {
        // gather the per-sequence query pointers into one [B,H,d] block
        unsigned char* hq = static_cast<unsigned char*>(m.h_q.reserve(B * row_bytes));
        bool any_host = false;
        for (size_t i = 0; i < B; ++i) {
            if (hipsup::is_device_pointer(q_data[i])) {
                check(ahpc_hip_memcpy_d2d(dq + i * row_bytes, q_data[i], row_bytes, st), "gather queries");
            } else {
                std::memcpy(hq + i * row_bytes, q_data[i], row_bytes);
                any_host = true;
            }
        }
        if (any_host) {
            for (size_t i = 0; i < B;) {  // contiguous runs of host rows go up in one copy each
                if (hipsup::is_device_pointer(q_data[i])) { ++i; continue; }
                size_t j = i;
                while (j < B && !hipsup::is_device_pointer(q_data[j])) ++j;
                check(ahpc_hip_memcpy_h2d(dq + i * row_bytes, hq + i * row_bytes, (j - i) * row_bytes, st), "copy queries to device");
                i = j;
            }
        }
        void* drows = m.d_rows.reserve(B * sizeof(int32_t));
        check(ahpc_hip_memcpy_h2d(drows, rows, B * sizeof(int32_t), st), "copy batch rows");
        const int64_t chunk = (int64_t)m.cfg.split_chunk_tokens;
        const size_t ws_bytes = ahpc_hip_paged_decode_workspace_bytes((int64_t)B, (int64_t)m.H, (int64_t)m.d, (int64_t)max_len, (int64_t)m.P, chunk);
        if (ws_bytes > current_perf_config_.max_workspace_size)
            throw AttentionException(AttentionError::MEMORY_ALLOCATION_FAILED, "decode partials exceed PerformanceConfig::max_workspace_size");
        void* ws = nullptr;
        if (ws_bytes) ws = (workspace_ptr_ && workspace_size_ >= ws_bytes && hipsup::is_device_pointer(workspace_ptr_)) ? workspace_ptr_ : m.d_ws.reserve(ws_bytes);
        float scale = current_params_.scale_factor > 0.0f ? current_params_.scale_factor : 1.0f / std::sqrt(static_cast<float>(m.d));
        hipsup::EventTimer timer;
        if (profiling_enabled_) timer.start(st);
        check(ahpc_hip_paged_decode_gqa(dq, dout, hipsup::dtype_code(qdt), m.pool->k_slab(), m.pool->v_slab(),
                                        hipsup::dtype_code(m.pool->dtype()), static_cast<const int32_t*>(m.d_table.get()),
                                        static_cast<const int32_t*>(m.d_lens.get()), static_cast<const int32_t*>(drows),
                                        (int64_t)B, (int64_t)m.H, (int64_t)m.Hkv, (int64_t)m.d, (int64_t)m.P,
                                        (int64_t)m.max_pages, (int64_t)max_len, scale, chunk, ws, ws_bytes, st), "paged decode");
        if (profiling_enabled_) {
            timer.stop(st);
            m.profile.emplace_back("decode_kernel_ms", timer.elapsed_ms());
        }
    }
    // scatter the output rows back to the caller's buffers
    unsigned char* ho = static_cast<unsigned char*>(m.h_o.reserve(B * row_bytes));
    bool any_host_out = false;
    for (size_t i = 0; i < B; ++i) {
        if (hipsup::is_device_pointer(o_data[i])) check(ahpc_hip_memcpy_d2d(o_data[i], dout + i * row_bytes, row_bytes, st), "scatter outputs");
        else any_host_out = true;
    }
    if (any_host_out) check(ahpc_hip_memcpy_d2h(ho, dout, B * row_bytes, st), "copy outputs from device");
    m.stream.sync();
    if (any_host_out)
        for (size_t i = 0; i < B; ++i)
            if (!hipsup::is_device_pointer(o_data[i])) std::memcpy(o_data[i], ho + i * row_bytes, row_bytes);
    if (profiling_enabled_)
        m.profile.emplace_back("forward_batch", std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - wall0).count());
}

// Reference: PagedAttention::forward, src/algorithms/paged_attention.cpp:132-174 (temporary sequence,
// append, one decode, destroy) - done per batch entry here.
void PagedAttention::forward(const TensorShape& qs, const void* q, const TensorShape& ks, const void* k, const TensorShape& vs,
                             const void* v, const TensorShape& os, void* o, const void* mask) {
    if (!impl_->configured)
        throw AttentionException(AttentionError::INVALID_PARAMETERS, "PagedAttention not configured. Call configure() first.");
    if (!q || !k || !v || !o) throw AttentionException(AttentionError::INVALID_INPUT, "null tensor pointer");
    if (mask) throw AttentionException(AttentionError::UNSUPPORTED_OPERATION, "decode attends to the whole cached context; masks are not supported");
    if (validate_inputs(qs, ks, vs, os, current_params_) != AttentionError::SUCCESS)
        throw AttentionException(AttentionError::INVALID_INPUT, "tensor shapes do not match the configured parameters");
    if (qs.dimensions[1] != 1 || os.dimensions[1] != 1)
        throw AttentionException(AttentionError::UNSUPPORTED_OPERATION, "PagedAttention::forward decodes ONE query token per batch entry; use FlashAttention for prefill");
    if (ks.data_type != vs.data_type) throw AttentionException(AttentionError::INVALID_INPUT, "key and value must share one data type");
    const size_t B = qs.dimensions[0], N = ks.dimensions[1], H = impl_->H, d = impl_->d;
    const auto wall0 = std::chrono::steady_clock::now();
    std::vector<size_t> ids(B);
    std::vector<TensorShape> qsh(B, TensorShape({1, 1, H, d}, qs.data_type)), osh(B, TensorShape({1, 1, H, d}, os.data_type));
    std::vector<const void*> qp(B);
    std::vector<void*> op(B);
    const size_t kv_stride = N * impl_->Hkv * d * ks.element_size();
    const size_t q_stride = H * d * qs.element_size();
    try {
        for (size_t b = 0; b < B; ++b) {
            ids[b] = create_sequence(N);
            append_kv_cache(ids[b], static_cast<const unsigned char*>(k) + b * kv_stride,
                            static_cast<const unsigned char*>(v) + b * kv_stride, N, ks.data_type);
            qp[b] = static_cast<const unsigned char*>(q) + b * q_stride;
            op[b] = static_cast<unsigned char*>(o) + b * q_stride;
        }
        forward_batch(ids, qsh, qp, osh, op);
    } catch (...) {
        for (size_t id : ids) destroy_sequence(id);
        throw;
    }
    for (size_t id : ids) destroy_sequence(id);
    if (profiling_enabled_)
        impl_->profile.emplace_back("forward_pass", std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - wall0).count());
}

void PagedAttention::backward(const TensorShape&, const void*, const TensorShape&, const void*, const TensorShape&, const void*,
                              const TensorShape&, const void*, const TensorShape&, void*, const TensorShape&, void*,
                              const TensorShape&, void*, const void*) {
    throw AttentionException(AttentionError::UNSUPPORTED_OPERATION, "HIP PagedAttention implements decode only");
}

// Bytes of decode partials for this batch at the configured maximum context (device scratch; allocated
// on demand unless a device workspace of this size was lent through set_workspace).
size_t PagedAttention::get_workspace_size(const AttentionParams& p) const {
    const size_t longest = std::max(p.max_sequence_length, p.sequence_length);
    return ahpc_hip_paged_decode_workspace_bytes((int64_t)p.batch_size, (int64_t)p.num_heads, (int64_t)p.head_dimension,
                                                 (int64_t)std::max<size_t>(longest, 1), (int64_t)std::max<size_t>(p.page_size, 1),
                                                 (int64_t)impl_->cfg.split_chunk_tokens);
}

void PagedAttention::set_workspace(void* workspace_ptr, size_t workspace_size) {
    workspace_ptr_ = workspace_ptr;
    workspace_size_ = workspace_size;
}

bool PagedAttention::supports_data_type(DataType t) const {
    return t == DataType::FLOAT32 || t == DataType::FLOAT16 || t == DataType::BFLOAT16;
}
bool PagedAttention::supports_memory_layout(MemoryLayout layout) const { return layout == MemoryLayout::ROW_MAJOR; }
std::string PagedAttention::get_backend_name() const { return "HIP_PagedAttention"; }
std::string PagedAttention::get_version() const { return "1.0.0"; }

void PagedAttention::enable_profiling(bool enable) {
    profiling_enabled_ = enable;
    if (!enable) impl_->profile.clear();
}
std::vector<std::pair<std::string, double>> PagedAttention::get_profiling_results() const { return impl_->profile; }
void PagedAttention::reset_profiling() { impl_->profile.clear(); }

// Reference: PagedAttention::validate_inputs, src/algorithms/paged_attention.cpp:301-331 (only the query
// and output shapes are examined).
AttentionError PagedAttention::validate_inputs(const TensorShape& q, const TensorShape&, const TensorShape&,
                                               const TensorShape& o, const AttentionParams& p) const {
    for (const TensorShape* s : {&q, &o}) {
        if (s->dimensions.size() != 4) return AttentionError::INVALID_INPUT;
        if (s->dimensions[0] != p.batch_size || s->dimensions[2] != p.num_heads || s->dimensions[3] != p.head_dimension)
            return AttentionError::INVALID_INPUT;
    }
    return AttentionError::SUCCESS;
}

// ---- statistics (reference getters: src/algorithms/paged_attention.cpp:549-575, whose counters are never
// updated there; here they come from the pool) -----------------------------------------------------------
size_t PagedAttention::get_total_memory_usage() const {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    return impl_->pool ? impl_->pool->get_allocated_pages() * impl_->page_bytes() : 0;
}
size_t PagedAttention::get_peak_memory_usage() const {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    return impl_->peak_bytes;
}
float PagedAttention::get_memory_utilization() const {
    const size_t used = get_total_memory_usage();
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    return impl_->cfg.memory_pool_size ? static_cast<float>(used) / static_cast<float>(impl_->cfg.memory_pool_size) : 0.0f;
}
size_t PagedAttention::get_active_sequences_count() const {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    size_t n = 0;
    for (const auto& kv : impl_->seqs) n += kv.second.active ? 1 : 0;
    return n;
}
KVBlockPoolStats PagedAttention::get_pool_stats() const {
    std::lock_guard<std::mutex> lock(impl_->seq_mutex);
    return impl_->pool ? impl_->pool->stats() : KVBlockPoolStats{};
}

// Re-homes the pages in use onto the lowest page ids (one device launch moves them, then the block table is rewritten)
// and hands the pool's free tail back: after sequences have come and gone the pages of the survivors are scattered
// over the whole id range, and only a pool whose high ids are free can shrink.  Pages keep their order inside every
// sequence; decode results do not change by a bit.  Reference: PagedAttention::compact_pages,
// src/algorithms/paged_attention.cpp:577-583 (its per-sequence helper is not defined in the reference's sources).
void PagedAttention::compact_pages() {
    Impl& m = *impl_;
    std::lock_guard<std::mutex> run(m.run_mutex);
    std::lock_guard<std::mutex> lock(m.seq_mutex);
    if (!m.pool) return;
    const auto moves = m.pool->plan_compaction();
    if (!moves.empty()) {
        std::vector<int32_t> ids(2 * moves.size());
        std::unordered_map<int32_t, int32_t> new_id;
        for (size_t i = 0; i < moves.size(); ++i) {
            ids[i] = moves[i].first;
            ids[moves.size() + i] = moves[i].second;
            new_id.emplace(moves[i].first, moves[i].second);
        }
        void* d_ids = m.d_rows.reserve(ids.size() * sizeof(int32_t));
        check(ahpc_hip_memcpy_h2d(d_ids, ids.data(), ids.size() * sizeof(int32_t), m.stream.get()), "compaction move list");
        const KVBlockPoolStats st = m.pool->stats();
        check(ahpc_hip_kv_move_pages(m.pool->k_slab(), m.pool->v_slab(), hipsup::dtype_code(m.pool->dtype()),
                                     static_cast<int64_t>(st.slab_capacity_pages), static_cast<const int32_t*>(d_ids),
                                     static_cast<const int32_t*>(d_ids) + moves.size(), static_cast<int64_t>(moves.size()),
                                     static_cast<int64_t>(m.Hkv), static_cast<int64_t>(m.d), static_cast<int64_t>(m.P), m.stream.get()),
              "compaction page moves");
        m.stream.sync();  // (the move list lives in host memory until here)
        for (auto& kv : m.seqs) {
            Sequence& s = kv.second;
            for (size_t i = 0; i < s.pages.size(); ++i) {
                auto it = new_id.find(s.pages[i]);
                if (it == new_id.end()) continue;
                s.pages[i] = it->second;
                m.table[s.row * m.max_pages + i] = it->second;
            }
        }
        m.table_dirty = true;
        m.pool->apply_compaction(moves);
    }
    // the free tail goes back, down to what the configuration starts a pool with
    m.pool->resize_pool(std::max(m.pool->get_allocated_pages(), m.cfg.initial_page_pool_size));
}
void PagedAttention::preload_pages(const std::vector<size_t>&) {}

}  // namespace attention_hpc
