/*
 * CPU oracle for the FlashAttention-forward and PagedAttention-decode paths.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is a plain-C restatement of the
 * arithmetic the reference repository's own test oracle and kernels define, used only
 * as the checker in tests, in the smoke run, and as the timed CPU baseline in the
 * benchmark.  The shipped library never calls into it.
 *
 * Every function below names the reference file:line whose behaviour it restates
 * (paths are relative to the reference checkout).  How each one is pinned
 * (closed forms, float64 brute force, invariants) is listed at the top of oracle.c and
 * exercised by tests/test_oracle_*.py.
 *
 * All tensors are fp32.  16-bit experiments feed the oracle values that were already
 * rounded to fp16/bf16 (see ahpc_oracle_round_*), so oracle and device see the same
 * numbers.
 */
#ifndef AHPC_ORACLE_H
#define AHPC_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- deterministic inputs ------------------------------------------------------ */

/* splitmix64 counter hash -> two 24-bit uniforms -> Box-Muller -> N(0, sigma^2).
 * (The reference seeds every generator from std::random_device,
 * tests/test_flash_attention.cpp:16-27, so there is nothing to restate: this only has to
 * be reproducible.) */
void ahpc_oracle_fill_normal(float* out, size_t n, uint64_t seed, uint64_t tensor_id, float sigma);
/* The same stream from element `first` on: a tensor generated in pieces holds the same values. */
void ahpc_oracle_fill_normal_at(float* out, size_t n, uint64_t seed, uint64_t tensor_id, float sigma, uint64_t first);
/* Same counter hash, uniform in [lo, hi) (the reference's tests draw U(-1,1),
 * tests/test_flash_attention.cpp:16-27). */
void ahpc_oracle_fill_uniform(float* out, size_t n, uint64_t seed, uint64_t tensor_id, float lo, float hi);
/* Uniform integers in [lo, hi] (inclusive), and a Fisher-Yates permutation of 0..n-1. */
void ahpc_oracle_fill_lengths(int32_t* out, size_t n, uint64_t seed, uint64_t tensor_id, int32_t lo, int32_t hi);
void ahpc_oracle_permutation(int32_t* out, size_t n, uint64_t seed, uint64_t tensor_id);

/* ---- 16-bit storage types ------------------------------------------------------- */
/* The reference declares half(float)/bfloat16(float) but never defines them
 * (src/api/tensor.hpp:39-66), so the rounding mode is this build's choice:
 * round-to-nearest-even, NaN preserved (quiet), overflow to infinity. */
uint16_t ahpc_oracle_f32_to_f16(float x);
float    ahpc_oracle_f16_to_f32(uint16_t h);
uint16_t ahpc_oracle_f32_to_bf16(float x);
float    ahpc_oracle_bf16_to_f32(uint16_t h);
/* In-place: x <- dtype(x) back to fp32.  dtype: 0 fp32 (no-op), 1 fp16, 2 bf16. */
void ahpc_oracle_round_inplace(float* x, size_t n, int dtype);

/* ---- dense attention ----------------------------------------------------------- */
/* softmax(scale * Q K^T [+ causal] [+ dense mask]) V, one query row at a time, fp32,
 * max-subtracted, sequential sums: restates compute_reference_attention,
 * tests/test_flash_attention.cpp:30-97 (and its dense-mask twin, :519-578, where a mask
 * value of 0.0f removes the key).  A row whose keys are all masked yields zeros, the rule
 * of OnlineSoftmaxState::get_normalizer, src/algorithms/flash_attention.hpp:59-61.
 *
 * Element (b, n, h, e) of a tensor lives at  b*stride_b + n*stride_n + h*stride_h + e
 * (in elements), so the same routine serves the API layout [B,N,H,d]
 * (FlashAttention::validate_inputs, src/algorithms/flash_attention.cpp:238-275) and the
 * [B,H,N,d] indexing the reference oracle itself uses (tests/test_flash_attention.cpp:46).
 * mask is NULL or fp32 [B,N,N] shared by all heads
 * (src/algorithms/flash_attention.cpp:432-435).
 * n_threads <= 1 runs serially (the reference has no threading); more threads split the
 * (b, h, row) space without changing any row's arithmetic. */
void ahpc_oracle_attention(const float* q, const float* k, const float* v, float* out,
                           int64_t B, int64_t N, int64_t H, int64_t d,
                           int64_t stride_b, int64_t stride_n, int64_t stride_h,
                           float scale, int causal, const float* mask, int n_threads);

/* Only the listed rows: rows[i] = (b*H + h)*N + n.  out is [n_rows, d]. */
void ahpc_oracle_attention_rows(const float* q, const float* k, const float* v, float* out,
                                int64_t B, int64_t N, int64_t H, int64_t d,
                                int64_t stride_b, int64_t stride_n, int64_t stride_h,
                                float scale, int causal,
                                const int64_t* rows, int64_t n_rows, int n_threads);

/* Packed ragged batch: tensors are [T,H,d] with token stride H*d, sequence i owns tokens
 * cu_seqlens[i] .. cu_seqlens[i+1]-1 and attends only within itself (per-sequence causal
 * diagonal).  The reference has no ragged API; each sequence is the dense routine above
 * with B = 1. */
void ahpc_oracle_attention_varlen(const float* q, const float* k, const float* v, float* out,
                                  const int32_t* cu_seqlens, int64_t n_seqs, int64_t H, int64_t d,
                                  float scale, int causal, int n_threads);
/* Listed rows of the ragged batch: rows[i] = token*H + h. out is [n_rows, d]. */
void ahpc_oracle_attention_varlen_rows(const float* q, const float* k, const float* v, float* out,
                                       const int32_t* cu_seqlens, int64_t n_seqs, int64_t H, int64_t d,
                                       float scale, int causal,
                                       const int64_t* rows, int64_t n_rows, int n_threads);

/* Gradients of ahpc_oracle_attention with respect to q, k and v for a given d_out, in double precision
 * (the reference's own backward, src/algorithms/flash_attention.cpp:496-580, is a placeholder).
 * q, d_out, d_q: contiguous [B,N,H,d]; k, v, d_k, d_v: contiguous [B,N,H_kv,d], H_kv divides H. */
void ahpc_oracle_attention_backward(const float* q, const float* k, const float* v, const float* d_out,
                                    float* d_q, float* d_k, float* d_v,
                                    int64_t B, int64_t N, int64_t H, int64_t H_kv, int64_t d,
                                    float scale, int causal, const float* mask, int n_threads);

/* ---- online-softmax merge --------------------------------------------------------- */
/* (m, l) <- merge((m, l), (m2, l2)): restates OnlineSoftmaxState::update,
 * src/algorithms/flash_attention.hpp:50-57. */
void ahpc_oracle_softmax_merge(float* m, float* l, float m2, float l2);
/* Attention of one query row computed in `n_splits` key ranges that are merged with the
 * rule above (accumulator rescaled by the same factors); used to show that the split
 * count does not change the result. */
void ahpc_oracle_attention_row_split(const float* q, const float* k, const float* v, float* out,
                                     int64_t L, int64_t d, int64_t stride_k, float scale, int n_splits);

/* ---- paged KV pool ------------------------------------------------------------------- */
/* Element offset of (token t, head h, lane 0) of sequence row `row` in a pool laid out
 * [page][slot][head][d]: restates the index math of paged_attention_kernel and
 * update_kv_cache_kernel, src/backends/cuda/cuda_kernels.cu:417-440 and :543-556
 * (page_idx = t / P, pos = t % P, page_id = table[row*max_pages + page_idx],
 *  offset = ((page_id*P + pos)*H + h)*d).  Returns -1 when the table entry is negative. */
int64_t ahpc_oracle_kv_offset(const int32_t* block_table, int64_t max_pages, int64_t row,
                              int64_t t, int64_t h, int64_t P, int64_t H, int64_t d);
/* Tokens of a sequence of length L that a decode attends to: all L, or those in front of the first negative
 * entry of its table row - the reference kernel's page walk ends there (`if (page_id < 0) break;`,
 * src/backends/cuda/cuda_kernels.cu:417-420). */
int64_t ahpc_oracle_attended_tokens(const int32_t* block_table, int64_t max_pages, int64_t row, int64_t L, int64_t P);
/* offsets[b*max_len + t] = ahpc_oracle_kv_offset(row = rows ? rows[b] : b, t, h = 0) for the tokens
 * a decode attends to (t < ahpc_oracle_attended_tokens(min(seq_lens[row], max_len))), else -1. */
void ahpc_oracle_gather_offsets(const int32_t* block_table, const int32_t* seq_lens, const int32_t* rows,
                                int64_t B, int64_t max_pages, int64_t max_len,
                                int64_t P, int64_t H, int64_t d, int64_t* offsets);
/* Write / read tokens [start, start+n) of one sequence: the scatter_keys_values /
 * gather_keys_values pair the reference declares but never defines
 * (src/algorithms/paged_attention.hpp:280-288), with the device layout above.
 * src/dst are [n,H,d] as in examples/basic_usage.cpp:160-165. */
void ahpc_oracle_kv_scatter(const float* k_new, const float* v_new, float* k_pool, float* v_pool,
                            const int32_t* block_table, int64_t max_pages, int64_t row,
                            int64_t start, int64_t n, int64_t P, int64_t H, int64_t d);
void ahpc_oracle_kv_gather(float* k_out, float* v_out, const float* k_pool, const float* v_pool,
                           const int32_t* block_table, int64_t max_pages, int64_t row,
                           int64_t start, int64_t n, int64_t P, int64_t H, int64_t d);

/* Decode: one query token per sequence attends to all L cached keys of that sequence.
 * Per (sequence, head): gather the keys through the block table, s_k = (q . K_k)*scale,
 * softmax, o = sum_k p_k V_k - the loop of PagedAttention::compute_paged_attention,
 * src/algorithms/paged_attention.cpp:596-680, without its lines :665-667 (which set every
 * score but the first to -inf) and completed where the file is cut off by the same
 * max-subtracted softmax as the dense routine.  q, out: [B,H,d].  A sequence of length 0
 * leaves its output row at zero (the reference skips it, :613-615). */
void ahpc_oracle_paged_decode(const float* q, float* out, const float* k_pool, const float* v_pool,
                              const int32_t* block_table, const int32_t* seq_lens, const int32_t* rows,
                              int64_t B, int64_t H, int64_t d, int64_t P, int64_t max_pages,
                              float scale, int n_threads);

/* FIFO page allocator model: restates PagePool, src/algorithms/paged_attention.cpp:11-64
 * (pages are numbered in creation order; allocate pops the front of the free queue and
 * creates `grow` more when it is empty; deallocate pushes to the back). */
typedef struct ahpc_oracle_pool ahpc_oracle_pool;
ahpc_oracle_pool* ahpc_oracle_pool_create(int32_t initial_pages, int32_t grow);
void    ahpc_oracle_pool_destroy(ahpc_oracle_pool* p);
int32_t ahpc_oracle_pool_allocate(ahpc_oracle_pool* p);
void    ahpc_oracle_pool_release(ahpc_oracle_pool* p, int32_t page);
int32_t ahpc_oracle_pool_free_count(const ahpc_oracle_pool* p);
int32_t ahpc_oracle_pool_total(const ahpc_oracle_pool* p);

#ifdef __cplusplus
}
#endif
#endif
