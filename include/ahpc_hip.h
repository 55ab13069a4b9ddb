/*
 * ahpc_hip.h - C ABI of the gfx950 (MI355X) attention kernels.
 *
 * This is the only door between host code and the GPU: plain pointers and sizes, no C++
 * types, no exceptions.  The C++ classes in include/attention_hpc/ (HipFlashAttention,
 * HipPagedAttention) call these functions and turn a non-zero return into
 * AttentionException(COMPUTATION_FAILED), the way the reference's CUDA_CHECK does
 * (src/backends/cuda/cuda_flash_attention.hpp:16-22).  The reference's precedent for such a
 * layer is its `extern "C" launch_*` block, src/backends/cuda/cuda_flash_attention.hpp:41-68;
 * each entry point below cites what it stands in for.  Paths are relative to the reference
 * checkout.
 *
 * Conventions
 *   - every function returns 0 on success, otherwise an ahpc_status (negative: rejected
 *     arguments, nothing launched) or a positive hipError_t value;
 *     ahpc_hip_error_string() explains either.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Launches are
 *     asynchronous on that stream; nothing here synchronises unless it says so.
 *   - all tensor pointers are DEVICE pointers unless a parameter says "host".
 *   - dtype codes equal the reference's DataType enumerators
 *     (src/api/attention_interface.hpp:16-20): 0 fp32, 1 fp16, 2 bf16.  16-bit values are
 *     produced with round-to-nearest-even.
 *   - strides are in elements.
 */
#ifndef AHPC_HIP_H
#define AHPC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { AHPC_F32 = 0, AHPC_F16 = 1, AHPC_BF16 = 2 };

typedef enum ahpc_status {
    AHPC_OK = 0,
    AHPC_ERR_NULL_POINTER = -1,
    AHPC_ERR_BAD_SHAPE = -2,       /* zero / negative / overflowing dimension, stride too small */
    AHPC_ERR_BAD_DTYPE = -3,
    AHPC_ERR_UNSUPPORTED_HEAD_DIM = -4,
    AHPC_ERR_WORKSPACE_TOO_SMALL = -5,
    AHPC_ERR_NO_DEVICE = -6,
    AHPC_ERR_BAD_ALIGNMENT = -7,   /* pointers/strides must allow 16-byte vector access */
    AHPC_ERR_UNSUPPORTED_GROUP = -8, /* query heads per K/V head not supported (kept for callers that test for it: decode takes any group size now) */
    AHPC_ERR_SCRATCH_LIMIT = -9     /* ahpc_hip_paged_decode_noalloc: the call needs more than AHPC_NOALLOC_SCRATCH_BYTES */
} ahpc_status;

const char* ahpc_hip_error_string(int code);

/* ---- device, memory, streams, events ------------------------------------------------------
 * Stand in for CudaMemoryManager / CudaStreamManager,
 * src/backends/cuda/cuda_flash_attention.hpp:71-122, and for the capability probe
 * BackendFactory::detectBackendCapabilities, src/api/backend_factory.cpp (BackendCapability,
 * src/api/backend_factory.hpp:24-37). */
typedef struct ahpc_device_info {
    char     name[128];
    char     arch[32];               /* e.g. "gfx950" */
    uint64_t total_memory_bytes;
    uint64_t free_memory_bytes;
    int32_t  compute_units;
    int32_t  wavefront_size;
    int32_t  lds_bytes_per_workgroup;
    int32_t  max_threads_per_workgroup;
    int32_t  clock_khz;
    int32_t  runtime_version;
} ahpc_device_info;

/* Launcher tuning values ("flash_pair_min_tiles", "flash_rows", "decode_waves", "decode_chunk", "decode_matrix_min_group",
 * "bwd_split", "bwd_pair", "mask_pack", "pool_in_place"): process-wide, each starts from its environment variable
 * (AHPC_FLASH_PAIR_MIN, AHPC_FLASH_ROWS, AHPC_DECODE_WAVES, AHPC_DECODE_CHUNK, AHPC_DECODE_MFMA_MIN_GROUP, AHPC_BWD_SPLIT,
 * AHPC_BWD_PAIR, AHPC_MASK_PACK, AHPC_POOL_IN_PLACE), which is read once.  No value
 * changes results; unknown names and negative values are refused.  The reference has no counterpart: its tile sizes
 * sit in PerformanceConfig (src/api/attention_interface.hpp:29-53), which the host classes still honour. */
int ahpc_hip_set_tuning(const char* name, int64_t value);
int ahpc_hip_get_tuning(const char* name, int64_t* value);
int ahpc_hip_device_count(int* count);                       /* never fails: count = 0 without a GPU */
int ahpc_hip_device_info(int device, ahpc_device_info* out);
int ahpc_hip_malloc(void** ptr, size_t bytes);
int ahpc_hip_free(void* ptr);
int ahpc_hip_host_malloc(void** ptr, size_t bytes);           /* pinned host staging memory */
int ahpc_hip_host_free(void* ptr);
/* Device address ranges that grow in place (what the KV block pool's slabs live in): reserve `bytes` of addresses
 * once, then commit physical memory behind the first `bytes` of the range, as often as needed.  Memory arrives in
 * chunks of `chunk_bytes` (rounded up to 2 MiB; one size per range, which this runtime's virtual memory management
 * insists on): committed only ever grows, *committed, when given, receives the bytes now backed - the request
 * rounded up to whole chunks, or less when the device ran out of memory part-way (then the call returns the
 * runtime's out-of-memory code and what was committed stays usable).  Pointers into the range never move, nothing
 * is copied and no stream is synchronised: kernels on other streams keep running while a range grows.
 * ahpc_hip_vmem_granularity reports 0 on a device without virtual memory management (then reserve returns
 * AHPC_ERR_NO_DEVICE and callers fall back to ahpc_hip_malloc).  Takes the place of the reference's
 * grow-by-reallocation of host vectors (PagePool::allocate_new_pages, src/algorithms/paged_attention.cpp:41-48). */
int ahpc_hip_vmem_granularity(size_t* bytes);
int ahpc_hip_vmem_reserve(void** base, size_t bytes, size_t chunk_bytes);
int ahpc_hip_vmem_commit(void* base, size_t bytes, size_t* committed);
/* Gives back the physical memory of the chunks that lie wholly behind the first `keep_bytes` of the range (the caller
 * vouches that no work in flight touches them: synchronise first). */
int ahpc_hip_vmem_decommit(void* base, size_t keep_bytes, size_t* committed);
int ahpc_hip_vmem_release(void* base);                        /* unmaps, frees the physical memory and the addresses */
int ahpc_hip_memcpy_h2d(void* dst, const void* src_host, size_t bytes, void* stream);
int ahpc_hip_memcpy_d2h(void* dst_host, const void* src, size_t bytes, void* stream);
int ahpc_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream);
int ahpc_hip_memset(void* dst, int byte_value, size_t bytes, void* stream);
int ahpc_hip_ptr_is_device(const void* ptr, int* is_device);  /* 0 for ordinary host memory */
int ahpc_hip_stream_create(void** stream);
int ahpc_hip_stream_destroy(void* stream);
int ahpc_hip_stream_synchronize(void* stream);
int ahpc_hip_device_synchronize(void);                      /* every stream of the current device */
int ahpc_hip_event_create(void** event);
int ahpc_hip_event_destroy(void* event);
int ahpc_hip_event_record(void* event, void* stream);
int ahpc_hip_event_synchronize(void* event);
int ahpc_hip_event_elapsed_ms(void* start, void* stop, float* ms);

/* ---- FlashAttention forward -------------------------------------------------------------------
 * O = softmax(scale * Q K^T [+ causal]) V in one launch; replaces
 * FlashAttention::forward -> compute_multihead_attention -> compute_attention_block,
 * src/algorithms/flash_attention.cpp:68-112, :379-450, :277-350, and the
 * launch_flash_attention_kernel slot of src/backends/cuda/cuda_flash_attention.hpp:42-48.
 *
 * Element (b, n, h, e) is at  b*stride_b + n*stride_n + h*stride_h + e; the last dimension
 * is contiguous.  The API layout [B,N,H,d] (FlashAttention::validate_inputs,
 * src/algorithms/flash_attention.cpp:238-275) is stride_b = N*H*d, stride_n = H*d,
 * stride_h = d; [B,H,N,d] is stride_b = H*N*d, stride_h = N*d, stride_n = d, so no transpose
 * pass (src/backends/cuda/cuda_kernels.cu:668-687) is ever needed.  Q, K, V and O share one
 * dtype and one set of strides.  d <= 256 with 16-byte aligned rows (d a multiple of 8 for fp16/bf16, of 4 for fp32)
 * runs on the matrix cores: fp16/bf16 on 16-bit matrix instructions, fp32 (the reference's default,
 * DataType::FLOAT32) on fp32 ones (fp32 products and sums: same accuracy as the fp32-FMA kernel).  The kernels are
 * built for d = 64, 128 and 256 (the last at one workgroup per CU); any other d runs on the next one with columns that
 * contribute nothing (beyond 128 with a dense mask: on its packed copy only).  Every other
 * case (d up to 256, unaligned tensors) runs on the fp32-FMA kernel.  Accumulation is fp32 throughout.  A row with no visible key yields zeros
 * (OnlineSoftmaxState::get_normalizer, src/algorithms/flash_attention.hpp:59-61).
 * scale <= 0 means 1/sqrt(d) (AttentionParams::scale_factor,
 * src/api/attention_interface.hpp:64). */
int ahpc_hip_flash_fwd(const void* q, const void* k, const void* v, void* o, int dtype,
                       int64_t B, int64_t N, int64_t H, int64_t d,
                       int64_t stride_b, int64_t stride_n, int64_t stride_h,
                       float scale, int causal, void* stream);

/* Grouped-query attention: H query heads over H_kv <= H key/value heads (H % H_kv == 0); query
 * head h reads K/V head h / (H / H_kv), i.e. consecutive query heads share one.  This is what
 * AttentionParams::key_value_heads announces (src/api/attention_interface.hpp:61; 0 = H) and the
 * reference never implements (the field is read nowhere; README.md:367-368 lists it as planned).
 * Q and O use (stride_b, stride_n, stride_h), K and V their own strides; with H_kv == H and equal
 * strides this is ahpc_hip_flash_fwd.  mask: NULL, or fp32 [B,N,N] as in the masked entry point. */
int ahpc_hip_flash_fwd_gqa(const void* q, const void* k, const void* v, void* o, int dtype,
                           int64_t B, int64_t N, int64_t H, int64_t H_kv, int64_t d,
                           int64_t stride_b, int64_t stride_n, int64_t stride_h,
                           int64_t kv_stride_b, int64_t kv_stride_n, int64_t kv_stride_h,
                           float scale, int causal, const float* mask, void* stream);

/* Same with a dense fp32 mask [B,N,N] shared by all heads, 0.0f removes the key
 * (FlashAttention::apply_attention_mask, src/algorithms/flash_attention.cpp:596-607;
 * indexing :432-435).  A query whose keys are all removed gets a zero output row.  Tensors that qualify for the
 * matrix cores (see ahpc_hip_flash_fwd) stay there, everything else runs on the fp32-FMA kernel.  The matrix-core kernels read a packed copy
 * of the mask (one bit per element) that a small kernel writes in front of it, into device memory the LIBRARY owns:
 * one buffer per device, grown on demand (hipMalloc; B * N * ceil(N / 64) * 8 bytes, at most 1 GiB) and kept until the
 * process ends; calls on one device share it and are ordered through an event, on whatever streams they run.  A
 * stream under graph capture, a larger mask, a failed allocation or the tuning value mask_pack = 0 make the 16-bit
 * kernel read the mask in place instead (N a multiple of 4 and a 16-byte aligned mask; otherwise, and for fp32
 * tensors, the fp32-FMA kernel): no allocation, more traffic.  mask may be NULL: then the fp32-FMA kernel runs whatever the type (the way to ask for
 * it). */
int ahpc_hip_flash_fwd_masked(const void* q, const void* k, const void* v, void* o, int dtype,
                              int64_t B, int64_t N, int64_t H, int64_t d,
                              int64_t stride_b, int64_t stride_n, int64_t stride_h,
                              float scale, int causal, const float* mask, void* stream);

/* Ragged batch packed as [T,H,d] (token stride stride_t, head stride stride_h); sequence i
 * owns tokens cu_seqlens[i] .. cu_seqlens[i+1]-1 (int32, device, n_seqs+1 entries) and
 * attends only within itself.  max_len = longest sequence (sizes the grid).  The reference
 * has no ragged entry point; the nearest declared shape is
 * CudaFlashAttention::forward_multi_sequence,
 * src/backends/cuda/cuda_flash_attention.hpp:270-279. */
int ahpc_hip_flash_fwd_varlen(const void* q, const void* k, const void* v, void* o, int dtype,
                              const int32_t* cu_seqlens, int64_t n_seqs, int64_t max_len,
                              int64_t H, int64_t d, int64_t stride_t, int64_t stride_h,
                              float scale, int causal, void* stream);

/* Ragged batch with grouped K/V heads: Q, O packed [T,H,d], K, V packed [T,H_kv,d]. */
int ahpc_hip_flash_fwd_varlen_gqa(const void* q, const void* k, const void* v, void* o, int dtype,
                                  const int32_t* cu_seqlens, int64_t n_seqs, int64_t max_len,
                                  int64_t H, int64_t H_kv, int64_t d,
                                  int64_t stride_t, int64_t stride_h, int64_t kv_stride_t, int64_t kv_stride_h,
                                  float scale, int causal, void* stream);

/* Debug twin of the MFMA kernel's launch geometry, evaluated on the HOST by the very function the kernel
 * uses (no GPU needed): for a dense fp16/bf16 launch of B sequences, N tokens, H heads it reports the grid
 * size in *n_blocks and, when the three arrays (capacity entries each) are given, for every workgroup id
 * its (sequence * H + head), the query tile it handles first and the one it handles second (-1 = none; all -1
 * for padding workgroups).  Tiles are 128 query rows, or 256 while the tuning value "flash_rows" is 256 (the
 * launcher itself takes 256 rows at d = 128 for dense launches of at least 2048 tokens that fill the chip).  Lets a test check that every query tile of every head is
 * handled exactly once, whatever the pairing and interleaving in force.  No counterpart in the reference
 * (its kernels are launched one tile per block, src/backends/cuda/cuda_kernels.cu:125-127). */
int ahpc_hip_flash_block_map(int64_t B, int64_t N, int64_t H, int causal, int64_t capacity, int64_t* n_blocks,
                             int32_t* seq_head, int32_t* first_tile, int32_t* second_tile);

/* ---- FlashAttention backward ------------------------------------------------------------------
 * Gradients of ahpc_hip_flash_fwd_gqa: given d_out = dLoss/dO it writes d_q = dLoss/dQ (layout and strides
 * of Q) and d_k, d_v (layout and strides of K, V; with grouped heads each K/V head receives the sum over
 * its query heads).  Replaces FlashAttention::backward -> compute_query_gradients /
 * compute_key_value_gradients, src/algorithms/flash_attention.cpp:114-174, :496-580, and the
 * launch_flash_attention_backward_kernel slot of src/backends/cuda/cuda_flash_attention.hpp:50-56
 * (flash_attention_backward_kernel, src/backends/cuda/cuda_kernels.cu:280-365).  Those are placeholders
 * (sums that ignore the attention weights; a kernel that expects stored N x N weights): what is computed
 * here is the derivative of the forward,  P = softmax(scale Q K^T + mask),  dV = P^T dO,
 * dS = P o (dO V^T - rowsum(dO o O)),  dQ = scale dS K,  dK = scale dS^T Q,  with the softmax statistics
 * recomputed (the interface passes neither O nor them).  All seven tensors share one dtype; fp32
 * accumulation throughout; the gradient tensors are fully overwritten, rows that see no key get zeros.
 * workspace: device memory of at least ahpc_hip_flash_bwd_workspace_bytes(B, N, H) bytes, 16-byte aligned,
 * for two floats per (sequence, head, row of a whole 128-row tile); its contents afterwards are unspecified.
 * Head dimensions in whole 16-byte pieces (fp16/bf16: a multiple of 8 up to 256; fp32: a multiple of 4 up to 128) with
 * 16-byte aligned rows run on the matrix cores (fp16/bf16 on 16-bit matrix instructions, fp32 on fp32 ones; kernels exist
 * for 64, 128 and, 16-bit only, 256, a smaller head dimension runs on the next one), everything else on fp32-FMA kernels.
 * mask: NULL or fp32 [B,N,N] as in the forward.  fp16/bf16 tensors with a mask stay on the matrix cores, on the
 * packed copy of the mask that ahpc_hip_flash_fwd_masked describes (here in two layouts, a quarter of a byte per
 * element; same owner, same limits, same conditions); fp32 tensors with a mask take the fp32-FMA kernels. */
size_t ahpc_hip_flash_bwd_workspace_bytes(int64_t B, int64_t N, int64_t H);
int ahpc_hip_flash_bwd(const void* d_out, const void* q, const void* k, const void* v,
                       void* d_q, void* d_k, void* d_v, int dtype,
                       int64_t B, int64_t N, int64_t H, int64_t H_kv, int64_t d,
                       int64_t stride_b, int64_t stride_n, int64_t stride_h,
                       int64_t kv_stride_b, int64_t kv_stride_n, int64_t kv_stride_h,
                       float scale, int causal, const float* mask,
                       void* workspace, size_t workspace_bytes, void* stream);

/* The same for a ragged batch packed as in ahpc_hip_flash_fwd_varlen_gqa: token t, head h, element e of Q, dO and
 * dQ is at t*stride_t + h*stride_h + e (K, V, dK, dV: kv_stride_t, kv_stride_h); sequence i owns tokens
 * cu_seqlens[i] .. cu_seqlens[i+1]-1 (n_seqs+1 device integers) and max_len is the longest sequence.
 * Workspace: ahpc_hip_flash_bwd_workspace_bytes(n_seqs, max_len, H).  No counterpart in the reference. */
int ahpc_hip_flash_bwd_varlen(const void* d_out, const void* q, const void* k, const void* v,
                              void* d_q, void* d_k, void* d_v, int dtype,
                              const int32_t* cu_seqlens, int64_t n_seqs, int64_t max_len,
                              int64_t H, int64_t H_kv, int64_t d,
                              int64_t stride_t, int64_t stride_h, int64_t kv_stride_t, int64_t kv_stride_h,
                              float scale, int causal,
                              void* workspace, size_t workspace_bytes, void* stream);

/* Forward and backward as a pair, for callers that run both on the same tensors (training): the forward keeps one float
 * per query row, the statistic its online softmax ends with (OnlineSoftmaxState::max_val / sum_exp,
 * src/algorithms/flash_attention.hpp:50-57, as -log2 of the row's sum of exp2(scale * log2(e) * q.k)), and the backward reads
 * it and the forward's output instead of recomputing both: its statistics launch, two of the backward's nine matrix products,
 * shrinks to one pass over dO and O.  The reference's backward has no such inputs
 * (FlashAttention::backward, src/algorithms/flash_attention.cpp:114-174, takes dO, Q, K, V only); the pair is an extension
 * of that interface.
 *   ahpc_hip_flash_row_stats_bytes(B, N, H): size of row_stats (4-byte aligned device memory).
 *   ahpc_hip_flash_fwd_keep: ahpc_hip_flash_fwd_gqa that also fills row_stats.  *stats_written = 1 when the launch did
 *     (fp16 / bf16 tensors on the matrix-core kernels), 0 when it ran on kernels that keep nothing (fp32, unaligned
 *     tensors): the backward must then be called without them.
 *   ahpc_hip_flash_bwd_kept: ahpc_hip_flash_bwd with o (the forward's output, layout and strides of Q) and row_stats, both
 *     as that forward left them for the same q, k, v, mask, scale and causal flag; anything else computes wrong gradients
 *     without notice.  o = NULL or row_stats = NULL: exactly ahpc_hip_flash_bwd.  Launches the matrix-core kernels cannot
 *     take ignore both and recompute. */
size_t ahpc_hip_flash_row_stats_bytes(int64_t B, int64_t N, int64_t H);
int ahpc_hip_flash_fwd_keep(const void* q, const void* k, const void* v, void* o, int dtype,
                            int64_t B, int64_t N, int64_t H, int64_t H_kv, int64_t d,
                            int64_t stride_b, int64_t stride_n, int64_t stride_h,
                            int64_t kv_stride_b, int64_t kv_stride_n, int64_t kv_stride_h,
                            float scale, int causal, const float* mask,
                            float* row_stats, int* stats_written, void* stream);
int ahpc_hip_flash_bwd_kept(const void* d_out, const void* q, const void* k, const void* v,
                            const void* o, const float* row_stats,
                            void* d_q, void* d_k, void* d_v, int dtype,
                            int64_t B, int64_t N, int64_t H, int64_t H_kv, int64_t d,
                            int64_t stride_b, int64_t stride_n, int64_t stride_h,
                            int64_t kv_stride_b, int64_t kv_stride_n, int64_t kv_stride_h,
                            float scale, int causal, const float* mask,
                            void* workspace, size_t workspace_bytes, void* stream);

/* ---- paged KV pool ---------------------------------------------------------------------------
 * Pool layout: K and V are separate slabs  [page][slot 0..P-1][head][d]  (the layout
 * update_kv_cache_kernel writes, src/backends/cuda/cuda_kernels.cu:547-556).
 * block_table is int32 [n_rows][max_pages], -1 = no page (sentinel of
 * src/backends/cuda/cuda_kernels.cu:420).  Token t of table row r, head h lives at element
 *     ((block_table[r*max_pages + t/P] * P + t%P) * H + h) * d.
 */

/* Write n_tokens new K/V rows ([n_tokens,H,d], dtype in_dtype) into the pool (dtype
 * pool_dtype, converted with RNE).  Token i goes to table row token_row[i] at position
 * token_pos[i]; token_row == NULL means every token belongs to `row0`, token_pos == NULL
 * means positions pos0, pos0+1, ...  Tokens whose table entry is negative are skipped.
 * Replaces PagedAttention::append_kv_cache -> scatter_keys_values,
 * src/algorithms/paged_attention.cpp:434-462, and update_kv_cache_kernel with its
 * slot_mapping, src/backends/cuda/cuda_kernels.cu:518-563. */
int ahpc_hip_kv_scatter(const void* k_new, const void* v_new, int in_dtype,
                        void* k_pool, void* v_pool, int pool_dtype,
                        const int32_t* block_table, int64_t max_pages,
                        const int32_t* token_row, const int32_t* token_pos,
                        int64_t row0, int64_t pos0, int64_t n_tokens,
                        int64_t H, int64_t d, int64_t P, void* stream);

/* Batched append, one launch for B sequences: the hand-off from a prefill to the cache.  Sequence b
 * receives seq_tokens[b] new tokens (NULL = N each) at positions seq_start[b].. (NULL = 0..) of table
 * row seq_rows[b]; its source rows are k_src/v_src + b*stride_b + t*stride_n (elements; each row is
 * H*d contiguous elements), i.e. the [B,N,H,d] K and V tensors a FlashAttention forward just read, or -
 * with cu_seqlens (int32[B+1], device) - rows cu_seqlens[b].. of a packed [T,H,d] batch (lengths from
 * cu_seqlens, stride_b ignored).  N bounds the tokens per sequence (it sizes the grid).  All index
 * arrays live on the device.  Same layout, conversion and skipping rules as ahpc_hip_kv_scatter; the
 * reference appends one sequence at a time (PagedAttention::append_kv_cache,
 * src/algorithms/paged_attention.cpp:434-462). */
int ahpc_hip_kv_scatter_batch(const void* k_src, const void* v_src, int in_dtype,
                              int64_t stride_b, int64_t stride_n,
                              void* k_pool, void* v_pool, int pool_dtype,
                              const int32_t* block_table, int64_t max_pages,
                              const int32_t* seq_rows, const int32_t* seq_start, const int32_t* seq_tokens,
                              const int32_t* cu_seqlens,
                              int64_t B, int64_t N, int64_t H, int64_t d, int64_t P, void* stream);

/* Read tokens [start, start+n) of table row `row` back as [n,H,d] in out_dtype.  Replaces
 * PagedAttention::get_kv_cache -> gather_keys_values,
 * src/algorithms/paged_attention.cpp:464-490. */
int ahpc_hip_kv_gather(void* k_out, void* v_out, int out_dtype,
                       const void* k_pool, const void* v_pool, int pool_dtype,
                       const int32_t* block_table, int64_t max_pages,
                       int64_t row, int64_t start, int64_t n,
                       int64_t H, int64_t d, int64_t P, void* stream);

/* Moves whole pages inside the pool: page from[i] -> page to[i] for i < n, K and V slabs alike, in one launch
 * (from, to: int32[n] in device memory; n_pages = pages the slabs hold; the two id sets must be disjoint; ids outside
 * the pool are skipped).  What PagedAttention::compact_pages re-homes pages with before it rewrites the block table
 * (reference: PagedAttention::compact_pages, src/algorithms/paged_attention.cpp:577-583, whose per-sequence helper
 * is declared at paged_attention.hpp:262 and not defined in the reference's sources). */
int ahpc_hip_kv_move_pages(void* k_pool, void* v_pool, int pool_dtype, int64_t n_pages, const int32_t* from,
                           const int32_t* to, int64_t n, int64_t H, int64_t d, int64_t P, void* stream);

/* ---- PagedAttention decode --------------------------------------------------------------------
 * One query token per batch entry attends to all seq_lens[row] cached tokens of its sequence:
 * replaces PagedAttention::forward_batch -> compute_paged_attention,
 * src/algorithms/paged_attention.cpp:496-547, :596-680, and paged_attention_kernel,
 * src/backends/cuda/cuda_kernels.cu:370-515 (with the query at the last position, which that
 * kernel's causal test :434 reduces to "all cached keys").
 *
 * q, o: [B,H,d] in qo_dtype.  batch_rows (int32[B], device, may be NULL = identity) maps
 * batch entry b to its row of block_table / seq_lens.  seq_lens: int32 per table row.
 * A sequence of length 0 gets a zero output row (the reference skips it, :613-615).
 *
 * Long contexts are cut into chunks of `chunk_tokens` tokens (a multiple of P; 0 = choose),
 * each chunk reduced by its own workgroup into an fp32 partial (m, l, o[d]) per head, then
 * merged with the rule of OnlineSoftmaxState::update, src/algorithms/flash_attention.hpp:50-57.
 * `max_len` bounds seq_lens (it sizes the grid; tokens beyond it are not read).
 * workspace must hold ahpc_hip_paged_decode_workspace_bytes() bytes: with chunk_tokens = 0 that is an upper
 * bound over the chunk lengths the launch may choose (128 to 1024 tokens, by batch, context and head count); 16-byte
 * aligned (AHPC_ERR_BAD_ALIGNMENT otherwise). */
size_t ahpc_hip_paged_decode_workspace_bytes(int64_t B, int64_t H, int64_t d, int64_t max_len,
                                             int64_t P, int64_t chunk_tokens);
int ahpc_hip_paged_decode(const void* q, void* o, int qo_dtype,
                          const void* k_pool, const void* v_pool, int pool_dtype,
                          const int32_t* block_table, const int32_t* seq_lens, const int32_t* batch_rows,
                          int64_t B, int64_t H, int64_t d, int64_t P, int64_t max_pages, int64_t max_len,
                          float scale, int64_t chunk_tokens,
                          void* workspace, size_t workspace_bytes, void* stream);

/* Decode with grouped K/V heads: the pool holds H_kv heads per token (its kv_scatter / kv_gather /
 * gather_indices calls take H = H_kv), q and o hold H = g * H_kv heads, any g; query head h reads pool head h / g.
 * Up to g = 8 every K/V byte is read once and serves the g query heads.  g from 9 to 32 (up to multi-query attention
 * with 32 heads) does the same on matrix-core kernels when the pool is fp16/bf16, d is 64, 128 or 256 and P = 16; on other
 * pools, and beyond 32, the group is served in slices of 8 query heads that each read the K/V stream.  The head dimension
 * may be anything up to 256 in whole 16-byte pieces of the pool's type (a multiple of 8 for fp16/bf16 pools, of 4 for
 * fp32 ones); AHPC_ERR_UNSUPPORTED_HEAD_DIM otherwise.
 * Workspace size: ahpc_hip_paged_decode_workspace_bytes with the QUERY head count. */
int ahpc_hip_paged_decode_gqa(const void* q, void* o, int qo_dtype,
                              const void* k_pool, const void* v_pool, int pool_dtype,
                              const int32_t* block_table, const int32_t* seq_lens, const int32_t* batch_rows,
                              int64_t B, int64_t H, int64_t H_kv, int64_t d, int64_t P, int64_t max_pages,
                              int64_t max_len, float scale, int64_t chunk_tokens,
                              void* workspace, size_t workspace_bytes, void* stream);

/* Decode for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  No counterpart in the reference.  Same arguments, kernels and results as
 * ahpc_hip_paged_decode_gqa, without the workspace: the chunk partials live in an array that is part of the
 * library's device code (AHPC_NOALLOC_SCRATCH_BYTES per GPU, held until the process ends).  The call performs no
 * hipMalloc / hipFree and calls no allocating library routine; its first call on a device looks the array's
 * address up (make that call outside a capture).  A call whose partials, at the chunk length the launch picks
 * (with chunk_tokens = 0 far fewer than the bound ahpc_hip_paged_decode_workspace_bytes reports: 64 sequences of up
 * to 4096 tokens, 32 heads of 128, take 4.3 MB), do not fit AHPC_NOALLOC_SCRATCH_BYTES returns AHPC_ERR_SCRATCH_LIMIT and
 * launches nothing.  Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (different
 * streams, different threads) race; calls on one stream do not.  Nothing in the array has to start at zero. */
#define AHPC_NOALLOC_SCRATCH_BYTES ((size_t)16 << 20)
int ahpc_hip_paged_decode_noalloc(const void* q, void* o, int qo_dtype,
                                  const void* k_pool, const void* v_pool, int pool_dtype,
                                  const int32_t* block_table, const int32_t* seq_lens, const int32_t* batch_rows,
                                  int64_t B, int64_t H, int64_t H_kv, int64_t d, int64_t P, int64_t max_pages,
                                  int64_t max_len, float scale, int64_t chunk_tokens, void* stream);

/* What the decode kernel gathers: offsets[b*max_len + t] = the element offset in the pool of (token t, head 0,
 * element 0) of batch entry b, or -1 for a token the decode does not attend to (t >= seq_lens[row], or at and behind
 * the first negative table entry of the row).  For the head dimensions the decode kernel is instantiated for (32, 64, 128, 256) the
 * values are written by that kernel itself, launched in a reporting mode in which the expression that addresses a
 * token row feeds a store instead of the loads; for other head dimensions by the index function of append and
 * read-back.  Lets a test hold the GPU's gather indices bit for bit against the index math of the reference
 * (src/backends/cuda/cuda_kernels.cu:417-440).  offsets: int64 [B][max_len] in device memory. */
int ahpc_hip_paged_gather_indices(const int32_t* block_table, const int32_t* seq_lens, const int32_t* batch_rows,
                                  int64_t B, int64_t H, int64_t d, int64_t P, int64_t max_pages, int64_t max_len,
                                  int64_t* offsets, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AHPC_HIP_H */
