/*
 * CPU oracle - TEST INFRASTRUCTURE ONLY (see oracle.h).  Nothing that ships links this.
 *
 * How each function is pinned (tests/test_oracle_*.py), since the reference holds no golden
 * vectors for this path and its own sources do not compile:
 *   ahpc_oracle_attention[_rows|_varlen]   float64 brute force (numpy) at the reference fixture
 *        shape B=2,N=16,H=4,d=64 and others; closed forms: V constant => O constant,
 *        Q = 0 => mean of V (prefix mean when causal), N = 1 => O = V, one dominant logit =>
 *        that V row, key-permutation invariance, fully masked row => 0; committed fixtures.
 *   ahpc_oracle_attention_backward          central differences of an independent float64 forward (numpy)
 *        in sampled entries of q, k and v; torch autograd in float64 on whole tensors; closed forms:
 *        N = 1 => dV = dO and dQ = dK = 0; V with equal rows => dQ = dK = 0; K with equal rows =>
 *        dQ = 0 and dV_j = mean_i dO_i; sum_j dV_j = sum_i dO_i; sum_i q_i.dQ_i = sum_j k_j.dK_j;
 *        grouped heads = repeated heads with the group's dK, dV summed.  The reference has no
 *        backward to compare with (placeholder): parity unpinned by the reference.
 *   ahpc_oracle_softmax_merge / _row_split  equals direct softmax for any split count;
 *        commutative/associative up to rounding.
 *   ahpc_oracle_kv_offset / gather_offsets  brute-force enumeration on a tiny pool.
 *   ahpc_oracle_kv_scatter / kv_gather      append -> read-back identity.
 *   ahpc_oracle_paged_decode                identity block table == dense attention of the last
 *        row; a page permutation leaves the output bit-identical.  No test of the reference
 *        covers paged decode: its parity is pinned by these equivalences only.
 *   ahpc_oracle_f32_to_f16 / bf16           all 65 536 bit patterns against numpy.float16 and a
 *        bit-manipulated bf16; round-trip identity.
 *   ahpc_oracle_pool_*                       hand-traced allocation order.
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------ */
/* generators                                                                             */

static inline uint64_t mix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

static inline uint64_t draw(uint64_t seed, uint64_t tensor_id, uint64_t i) {
    return mix64(mix64(seed ^ (tensor_id * 0x9E3779B97F4A7C15ull)) + i);
}

/* Elements first .. first+n-1 of the stream (every element depends on its index only, so any split of a tensor
 * into pieces, and any number of threads, gives the same values). */
void ahpc_oracle_fill_normal_at(float* out, size_t n, uint64_t seed, uint64_t tensor_id, float sigma, uint64_t first) {
    const double two_pi = 6.283185307179586476925286766559;
#pragma omp parallel for schedule(static) if (n > 65536)
    for (size_t i = 0; i < n; ++i) {
        uint64_t z = draw(seed, tensor_id, first + (uint64_t)i);
        double u1 = (double)((z >> 40) + 1) * (1.0 / 16777216.0);       /* (0, 1] */
        double u2 = (double)((z >> 16) & 0xFFFFFFu) * (1.0 / 16777216.0); /* [0, 1) */
        double r = sqrt(-2.0 * log(u1));
        out[i] = (float)(r * cos(two_pi * u2)) * sigma;
    }
}

void ahpc_oracle_fill_normal(float* out, size_t n, uint64_t seed, uint64_t tensor_id, float sigma) {
    ahpc_oracle_fill_normal_at(out, n, seed, tensor_id, sigma, 0);
}

void ahpc_oracle_fill_uniform(float* out, size_t n, uint64_t seed, uint64_t tensor_id, float lo, float hi) {
    for (size_t i = 0; i < n; ++i) {
        uint64_t z = draw(seed, tensor_id, (uint64_t)i);
        float u = (float)(z >> 40) * (1.0f / 16777216.0f);
        out[i] = lo + (hi - lo) * u;
    }
}

void ahpc_oracle_fill_lengths(int32_t* out, size_t n, uint64_t seed, uint64_t tensor_id, int32_t lo, int32_t hi) {
    uint64_t span = (uint64_t)(hi - lo) + 1;
    for (size_t i = 0; i < n; ++i) out[i] = lo + (int32_t)(draw(seed, tensor_id, (uint64_t)i) % span);
}

void ahpc_oracle_permutation(int32_t* out, size_t n, uint64_t seed, uint64_t tensor_id) {
    for (size_t i = 0; i < n; ++i) out[i] = (int32_t)i;
    for (size_t i = n; i > 1; --i) {
        size_t j = (size_t)(draw(seed, tensor_id, (uint64_t)i) % (uint64_t)i);
        int32_t t = out[i - 1]; out[i - 1] = out[j]; out[j] = t;
    }
}

/* ------------------------------------------------------------------------------------ */
/* fp16 / bf16, round-to-nearest-even                                                     */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

uint16_t ahpc_oracle_f32_to_bf16(float x) {
    uint32_t u = f2u(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u); /* NaN stays NaN */
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float ahpc_oracle_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

uint16_t ahpc_oracle_f32_to_f16(float x) {
    uint32_t u = f2u(x);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((a >> 13) & 0x1FFu)); /* NaN */
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);  /* >= 65536 (and inf) -> inf; 65520..65536 handled below */
    if (a >= 0x38800000u) {                                    /* normal half range */
        uint32_t m = a - 0x38000000u;                          /* rebias 127 -> 15 */
        uint32_t r = m + 0x0FFFu + ((m >> 13) & 1u);           /* RNE on the 13 dropped bits */
        return (uint16_t)(sign | (r >> 13));                   /* a carry into the exponent, up to inf, is correct */
    }
    if (a < 0x33000000u) return sign;                          /* below half the smallest subnormal -> 0 (tie at 2^-25 -> 0 even) */
    /* subnormal half: value = mant * 2^-24 */
    int e = (int)(a >> 23);                                    /* 102 .. 112 */
    uint32_t m = (a & 0x7FFFFFu) | 0x800000u;                  /* 24-bit significand */
    int shift = 126 - e;                                       /* 14 .. 24 */
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) ++q;
    return (uint16_t)(sign | q);
}

float ahpc_oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    if (e == 0x1Fu) return u2f(sign | 0x7F800000u | (m << 13));
    if (e != 0) return u2f(sign | ((e + 112u) << 23) | (m << 13));
    if (m == 0) return u2f(sign);
    float f = (float)m * (1.0f / 16777216.0f); /* m * 2^-24, exact */
    return sign ? -f : f;
}

void ahpc_oracle_round_inplace(float* x, size_t n, int dtype) {
    if (dtype == 1) for (size_t i = 0; i < n; ++i) x[i] = ahpc_oracle_f16_to_f32(ahpc_oracle_f32_to_f16(x[i]));
    else if (dtype == 2) for (size_t i = 0; i < n; ++i) x[i] = ahpc_oracle_bf16_to_f32(ahpc_oracle_f32_to_bf16(x[i]));
}

/* ------------------------------------------------------------------------------------ */
/* one attention row                                                                      */

/* Keys 0..n_keys-1 at kbase + j*stride_k, values likewise; `keep` (may be NULL) has one
 * fp32 per key, 0.0f removes it.  scores/weights are caller scratch of n_keys floats. */
static void attend_row(const float* qrow, const float* kbase, const float* vbase, float* orow,
                       int64_t n_keys, int64_t d, int64_t stride_k, float scale,
                       const float* keep, float* scores, float* acc) {
    float top = -INFINITY;
    for (int64_t j = 0; j < n_keys; ++j) {
        if (keep && keep[j] == 0.0f) { scores[j] = -INFINITY; continue; }
        const float* kr = kbase + j * stride_k;
        float dot = 0.0f;
        for (int64_t e = 0; e < d; ++e) dot += qrow[e] * kr[e];
        float s = dot * scale;
        scores[j] = s;
        if (s > top) top = s;
    }
    for (int64_t e = 0; e < d; ++e) acc[e] = 0.0f;
    if (top == -INFINITY) {            /* nothing to attend to: zero row */
        for (int64_t e = 0; e < d; ++e) orow[e] = 0.0f;
        return;
    }
    float total = 0.0f;
    for (int64_t j = 0; j < n_keys; ++j) {
        float w = expf(scores[j] - top);
        scores[j] = w;
        total += w;
    }
    for (int64_t j = 0; j < n_keys; ++j) scores[j] /= total;
    /* per output lane the sum runs over keys in order, as in the reference; the loops are
     * swapped only so that V is read row by row */
    for (int64_t j = 0; j < n_keys; ++j) {
        float w = scores[j];
        const float* vr = vbase + j * stride_k;
        for (int64_t e = 0; e < d; ++e) acc[e] += w * vr[e];
    }
    for (int64_t e = 0; e < d; ++e) orow[e] = acc[e];
}

static void dense_row(const float* q, const float* k, const float* v, float* orow,
                      int64_t b, int64_t h, int64_t n, int64_t N, int64_t d,
                      int64_t sb, int64_t sn, int64_t sh, float scale, int causal,
                      const float* mask, float* scores, float* acc) {
    int64_t base = b * sb + h * sh;
    int64_t n_keys = causal ? n + 1 : N;
    const float* keep = mask ? mask + (b * N + n) * N : NULL;
    attend_row(q + base + n * sn, k + base, v + base, orow, n_keys, d, sn, scale, keep, scores, acc);
}

void ahpc_oracle_attention(const float* q, const float* k, const float* v, float* out,
                           int64_t B, int64_t N, int64_t H, int64_t d,
                           int64_t sb, int64_t sn, int64_t sh,
                           float scale, int causal, const float* mask, int n_threads) {
    int64_t total = B * H * N;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel num_threads(n_threads)
    {
        float* scores = (float*)malloc(sizeof(float) * (size_t)(N + d));
        float* acc = scores + N;
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < total; ++r) {
            int64_t n = r % N, h = (r / N) % H, b = r / (N * H);
            dense_row(q, k, v, out + b * sb + n * sn + h * sh, b, h, n, N, d, sb, sn, sh, scale, causal, mask, scores, acc);
        }
        free(scores);
    }
}

void ahpc_oracle_attention_rows(const float* q, const float* k, const float* v, float* out,
                                int64_t B, int64_t N, int64_t H, int64_t d,
                                int64_t sb, int64_t sn, int64_t sh,
                                float scale, int causal,
                                const int64_t* rows, int64_t n_rows, int n_threads) {
    (void)B;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel num_threads(n_threads)
    {
        float* scores = (float*)malloc(sizeof(float) * (size_t)(N + d));
        float* acc = scores + N;
#pragma omp for schedule(dynamic, 4)
        for (int64_t i = 0; i < n_rows; ++i) {
            int64_t r = rows[i];
            int64_t n = r % N, h = (r / N) % H, b = r / (N * H);
            dense_row(q, k, v, out + i * d, b, h, n, N, d, sb, sn, sh, scale, causal, NULL, scores, acc);
        }
        free(scores);
    }
}

/* ------------------------------------------------------------------------------------ */
/* backward: the derivative of the function above.  The reference's backward is a placeholder
 * (src/algorithms/flash_attention.cpp:496-580 sums products that ignore the attention weights, and its
 * test only asks for non-zero gradients, tests/test_flash_attention.cpp:447-479), so there is nothing to
 * follow line by line: this differentiates compute_reference_attention (tests/test_flash_attention.cpp:30-97)
 *   P = softmax(scale * Q K^T + mask),  O = P V
 *   dV = P^T dO,  dP = dO V^T,  dS = P o (dP - rowsum(P o dP)),  dQ = scale * dS K,  dK = scale * dS^T Q
 * in double precision, rounding once at the end.  q, d_out, d_q are [B,N,H,d]; k, v, d_k, d_v are
 * [B,N,H_kv,d] and query head h uses key/value head h / (H / H_kv), whose gradient sums over its group. */
void ahpc_oracle_attention_backward(const float* q, const float* k, const float* v, const float* d_out,
                                    float* d_q, float* d_k, float* d_v,
                                    int64_t B, int64_t N, int64_t H, int64_t H_kv, int64_t d,
                                    float scale, int causal, const float* mask, int n_threads) {
    const int64_t G = H / H_kv;
    const int64_t sq = H * d, skv = H_kv * d;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel num_threads(n_threads)
    {
        double* p = (double*)malloc(sizeof(double) * (size_t)(2 * N + d + 2 * N * d));
        double* dp = p + N;
        double* dq_row = dp + N;
        double* dk_acc = dq_row + d;
        double* dv_acc = dk_acc + N * d;
#pragma omp for schedule(dynamic, 1)
        for (int64_t bh = 0; bh < B * H_kv; ++bh) {
            const int64_t b = bh / H_kv, hk = bh % H_kv;
            const float* kb = k + b * N * skv + hk * d;
            const float* vb = v + b * N * skv + hk * d;
            for (int64_t x = 0; x < 2 * N * d; ++x) dk_acc[x] = 0.0;
            for (int64_t g = 0; g < G; ++g) {
                const int64_t h = hk * G + g;
                for (int64_t i = 0; i < N; ++i) {
                    const float* qi = q + (b * N + i) * sq + h * d;
                    const float* doi = d_out + (b * N + i) * sq + h * d;
                    float* dqi = d_q + (b * N + i) * sq + h * d;
                    const float* keep = mask ? mask + (b * N + i) * N : NULL;
                    const int64_t n_keys = causal ? i + 1 : N;
                    double top = -INFINITY;
                    for (int64_t j = 0; j < n_keys; ++j) {
                        if (keep && keep[j] == 0.0f) { p[j] = -INFINITY; continue; }
                        double s = 0.0;
                        for (int64_t e = 0; e < d; ++e) s += (double)qi[e] * (double)kb[j * skv + e];
                        p[j] = s * (double)scale;
                        if (p[j] > top) top = p[j];
                    }
                    for (int64_t e = 0; e < d; ++e) dq_row[e] = 0.0;
                    if (top != -INFINITY) {
                        double total = 0.0, delta = 0.0;
                        for (int64_t j = 0; j < n_keys; ++j) { p[j] = exp(p[j] - top); total += p[j]; }
                        for (int64_t j = 0; j < n_keys; ++j) {
                            p[j] /= total;
                            double t = 0.0;
                            for (int64_t e = 0; e < d; ++e) t += (double)doi[e] * (double)vb[j * skv + e];
                            dp[j] = t;
                            delta += p[j] * t;
                        }
                        for (int64_t j = 0; j < n_keys; ++j) {
                            if (p[j] == 0.0) continue;
                            const double ds = p[j] * (dp[j] - delta) * (double)scale;
                            for (int64_t e = 0; e < d; ++e) {
                                dq_row[e] += ds * (double)kb[j * skv + e];
                                dk_acc[j * d + e] += ds * (double)qi[e];
                                dv_acc[j * d + e] += p[j] * (double)doi[e];
                            }
                        }
                    }
                    for (int64_t e = 0; e < d; ++e) dqi[e] = (float)dq_row[e];
                }
            }
            for (int64_t j = 0; j < N; ++j)
                for (int64_t e = 0; e < d; ++e) {
                    d_k[(b * N + j) * skv + hk * d + e] = (float)dk_acc[j * d + e];
                    d_v[(b * N + j) * skv + hk * d + e] = (float)dv_acc[j * d + e];
                }
        }
        free(p);
    }
}

static int64_t find_seq(const int32_t* cu, int64_t n_seqs, int64_t tok) {
    int64_t lo = 0, hi = n_seqs - 1;
    while (lo < hi) {
        int64_t mid = (lo + hi + 1) / 2;
        if (cu[mid] <= tok) lo = mid; else hi = mid - 1;
    }
    return lo;
}

static void varlen_row(const float* q, const float* k, const float* v, float* orow,
                       const int32_t* cu, int64_t n_seqs, int64_t tok, int64_t h, int64_t H, int64_t d,
                       float scale, int causal, float* scores, float* acc) {
    int64_t s = find_seq(cu, n_seqs, tok);
    int64_t first = cu[s], len = cu[s + 1] - cu[s], n = tok - first;
    int64_t st = H * d;
    int64_t n_keys = causal ? n + 1 : len;
    attend_row(q + tok * st + h * d, k + first * st + h * d, v + first * st + h * d, orow,
               n_keys, d, st, scale, NULL, scores, acc);
}

void ahpc_oracle_attention_varlen(const float* q, const float* k, const float* v, float* out,
                                  const int32_t* cu, int64_t n_seqs, int64_t H, int64_t d,
                                  float scale, int causal, int n_threads) {
    int64_t T = cu[n_seqs], max_len = 0;
    for (int64_t s = 0; s < n_seqs; ++s) if (cu[s + 1] - cu[s] > max_len) max_len = cu[s + 1] - cu[s];
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel num_threads(n_threads)
    {
        float* scores = (float*)malloc(sizeof(float) * (size_t)(max_len + d + 1));
        float* acc = scores + max_len;
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < T * H; ++r) {
            int64_t tok = r / H, h = r % H;
            varlen_row(q, k, v, out + tok * H * d + h * d, cu, n_seqs, tok, h, H, d, scale, causal, scores, acc);
        }
        free(scores);
    }
}

void ahpc_oracle_attention_varlen_rows(const float* q, const float* k, const float* v, float* out,
                                       const int32_t* cu, int64_t n_seqs, int64_t H, int64_t d,
                                       float scale, int causal,
                                       const int64_t* rows, int64_t n_rows, int n_threads) {
    int64_t max_len = 0;
    for (int64_t s = 0; s < n_seqs; ++s) if (cu[s + 1] - cu[s] > max_len) max_len = cu[s + 1] - cu[s];
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel num_threads(n_threads)
    {
        float* scores = (float*)malloc(sizeof(float) * (size_t)(max_len + d + 1));
        float* acc = scores + max_len;
#pragma omp for schedule(dynamic, 4)
        for (int64_t i = 0; i < n_rows; ++i) {
            int64_t tok = rows[i] / H, h = rows[i] % H;
            varlen_row(q, k, v, out + i * d, cu, n_seqs, tok, h, H, d, scale, causal, scores, acc);
        }
        free(scores);
    }
}

/* ------------------------------------------------------------------------------------ */
/* online-softmax merge                                                                   */

void ahpc_oracle_softmax_merge(float* m, float* l, float m2, float l2) {
    if (m2 > *m) {
        *l = *l * expf(*m - m2) + l2;
        *m = m2;
    } else {
        *l += l2 * expf(m2 - *m);
    }
}

void ahpc_oracle_attention_row_split(const float* q, const float* k, const float* v, float* out,
                                     int64_t L, int64_t d, int64_t stride_k, float scale, int n_splits) {
    float run_m = -INFINITY, run_l = 0.0f;
    float* acc = (float*)calloc((size_t)d, sizeof(float));
    float* part = (float*)malloc(sizeof(float) * (size_t)d);
    float* s = (float*)malloc(sizeof(float) * (size_t)(L > 0 ? L : 1));
    if (n_splits < 1) n_splits = 1;
    int64_t per = (L + n_splits - 1) / n_splits;
    for (int64_t lo = 0; lo < L; lo += per) {
        int64_t hi = lo + per < L ? lo + per : L;
        float pm = -INFINITY, pl = 0.0f;
        for (int64_t j = lo; j < hi; ++j) {
            float dot = 0.0f;
            for (int64_t e = 0; e < d; ++e) dot += q[e] * k[j * stride_k + e];
            s[j] = dot * scale;
            if (s[j] > pm) pm = s[j];
        }
        for (int64_t e = 0; e < d; ++e) part[e] = 0.0f;
        for (int64_t j = lo; j < hi; ++j) {
            float w = expf(s[j] - pm);
            pl += w;
            for (int64_t e = 0; e < d; ++e) part[e] += w * v[j * stride_k + e];
        }
        /* fold the partial into the running state with the factors the merge rule uses */
        float new_m = pm > run_m ? pm : run_m;
        float f_old = run_m == -INFINITY ? 0.0f : expf(run_m - new_m);
        float f_new = expf(pm - new_m);
        for (int64_t e = 0; e < d; ++e) acc[e] = acc[e] * f_old + part[e] * f_new;
        ahpc_oracle_softmax_merge(&run_m, &run_l, pm, pl);
    }
    float inv = run_l > 0.0f ? 1.0f / run_l : 0.0f;
    for (int64_t e = 0; e < d; ++e) out[e] = acc[e] * inv;
    free(acc); free(part); free(s);
}

/* ------------------------------------------------------------------------------------ */
/* paged pool                                                                             */

int64_t ahpc_oracle_kv_offset(const int32_t* table, int64_t max_pages, int64_t row,
                              int64_t t, int64_t h, int64_t P, int64_t H, int64_t d) {
    int64_t page_idx = t / P, pos = t % P;
    int64_t page_id = table[row * max_pages + page_idx];
    if (page_id < 0) return -1;
    return ((page_id * P + pos) * H + h) * d;
}

/* Tokens a decode attends to: the page walk of the reference kernel leaves its loop at the first negative
 * page id (`if (page_id < 0) break;`, src/backends/cuda/cuda_kernels.cu:417-420), so a missing page ends the
 * sequence there whatever follows it in the row. */
int64_t ahpc_oracle_attended_tokens(const int32_t* table, int64_t max_pages, int64_t row, int64_t L, int64_t P) {
    int64_t num_pages = (L + P - 1) / P;
    for (int64_t page_idx = 0; page_idx < num_pages; ++page_idx)
        if (table[row * max_pages + page_idx] < 0) return page_idx * P;
    return L;
}

void ahpc_oracle_gather_offsets(const int32_t* table, const int32_t* seq_lens, const int32_t* rows,
                                int64_t B, int64_t max_pages, int64_t max_len,
                                int64_t P, int64_t H, int64_t d, int64_t* offsets) {
    for (int64_t b = 0; b < B; ++b) {
        int64_t row = rows ? rows[b] : b;
        int64_t L = seq_lens[row] < max_len ? seq_lens[row] : max_len;
        int64_t n = ahpc_oracle_attended_tokens(table, max_pages, row, L, P);
        for (int64_t t = 0; t < max_len; ++t)
            offsets[b * max_len + t] = t < n ? ahpc_oracle_kv_offset(table, max_pages, row, t, 0, P, H, d) : -1;
    }
}

void ahpc_oracle_kv_scatter(const float* k_new, const float* v_new, float* k_pool, float* v_pool,
                            const int32_t* table, int64_t max_pages, int64_t row,
                            int64_t start, int64_t n, int64_t P, int64_t H, int64_t d) {
    for (int64_t i = 0; i < n; ++i) {
        int64_t off = ahpc_oracle_kv_offset(table, max_pages, row, start + i, 0, P, H, d);
        if (off < 0) continue;
        memcpy(k_pool + off, k_new + i * H * d, sizeof(float) * (size_t)(H * d));
        memcpy(v_pool + off, v_new + i * H * d, sizeof(float) * (size_t)(H * d));
    }
}

void ahpc_oracle_kv_gather(float* k_out, float* v_out, const float* k_pool, const float* v_pool,
                           const int32_t* table, int64_t max_pages, int64_t row,
                           int64_t start, int64_t n, int64_t P, int64_t H, int64_t d) {
    for (int64_t i = 0; i < n; ++i) {
        int64_t off = ahpc_oracle_kv_offset(table, max_pages, row, start + i, 0, P, H, d);
        if (off < 0) continue;
        memcpy(k_out + i * H * d, k_pool + off, sizeof(float) * (size_t)(H * d));
        memcpy(v_out + i * H * d, v_pool + off, sizeof(float) * (size_t)(H * d));
    }
}

void ahpc_oracle_paged_decode(const float* q, float* out, const float* k_pool, const float* v_pool,
                              const int32_t* table, const int32_t* seq_lens, const int32_t* rows,
                              int64_t B, int64_t H, int64_t d, int64_t P, int64_t max_pages,
                              float scale, int n_threads) {
    if (n_threads < 1) n_threads = 1;
    int64_t max_len = 0;
    for (int64_t b = 0; b < B; ++b) {
        int64_t L = seq_lens[rows ? rows[b] : b];
        if (L > max_len) max_len = L;
    }
#pragma omp parallel num_threads(n_threads)
    {
        /* per-thread gather buffers: the keys and values of one (sequence, head) made contiguous */
        float* kbuf = (float*)malloc(sizeof(float) * (size_t)(2 * max_len * d + max_len + d + 1));
        float* vbuf = kbuf + max_len * d;
        float* scores = vbuf + max_len * d;
        float* acc = scores + max_len;
#pragma omp for schedule(dynamic, 1)
        for (int64_t bh = 0; bh < B * H; ++bh) {
            int64_t b = bh / H, h = bh % H;
            int64_t row = rows ? rows[b] : b;
            int64_t L = ahpc_oracle_attended_tokens(table, max_pages, row, seq_lens[row], P);
            float* orow = out + (b * H + h) * d;
            if (L == 0) { for (int64_t e = 0; e < d; ++e) orow[e] = 0.0f; continue; }
            for (int64_t t = 0; t < L; ++t) {
                int64_t off = ahpc_oracle_kv_offset(table, max_pages, row, t, h, P, H, d);
                memcpy(kbuf + t * d, k_pool + off, sizeof(float) * (size_t)d);
                memcpy(vbuf + t * d, v_pool + off, sizeof(float) * (size_t)d);
            }
            attend_row(q + (b * H + h) * d, kbuf, vbuf, orow, L, d, d, scale, NULL, scores, acc);
        }
        free(kbuf);
    }
}

/* ------------------------------------------------------------------------------------ */
/* FIFO pool model                                                                        */

struct ahpc_oracle_pool {
    int32_t* ring;      /* free queue storage */
    int32_t cap, head, count;
    int32_t total, grow;
    uint8_t* in_use;
    int32_t in_use_cap;
};

static void pool_push(ahpc_oracle_pool* p, int32_t id) {
    if (p->count == p->cap) {
        int32_t ncap = p->cap ? p->cap * 2 : 64;
        int32_t* nr = (int32_t*)malloc(sizeof(int32_t) * (size_t)ncap);
        for (int32_t i = 0; i < p->count; ++i) nr[i] = p->ring[(p->head + i) % p->cap];
        free(p->ring); p->ring = nr; p->cap = ncap; p->head = 0;
    }
    p->ring[(p->head + p->count) % p->cap] = id;
    ++p->count;
}

static void pool_create_pages(ahpc_oracle_pool* p, int32_t n) {
    if (p->total + n > p->in_use_cap) {
        int32_t ncap = (p->total + n) * 2;
        p->in_use = (uint8_t*)realloc(p->in_use, (size_t)ncap);
        memset(p->in_use + p->in_use_cap, 0, (size_t)(ncap - p->in_use_cap));
        p->in_use_cap = ncap;
    }
    for (int32_t i = 0; i < n; ++i) pool_push(p, p->total++);
}

ahpc_oracle_pool* ahpc_oracle_pool_create(int32_t initial_pages, int32_t grow) {
    ahpc_oracle_pool* p = (ahpc_oracle_pool*)calloc(1, sizeof(*p));
    p->grow = grow;
    pool_create_pages(p, initial_pages);
    return p;
}

void ahpc_oracle_pool_destroy(ahpc_oracle_pool* p) {
    if (!p) return;
    free(p->ring); free(p->in_use); free(p);
}

int32_t ahpc_oracle_pool_allocate(ahpc_oracle_pool* p) {
    if (p->count == 0) {
        if (p->grow <= 0) return -1;
        pool_create_pages(p, p->grow);
    }
    int32_t id = p->ring[p->head];
    p->head = (p->head + 1) % p->cap;
    --p->count;
    p->in_use[id] = 1;
    return id;
}

void ahpc_oracle_pool_release(ahpc_oracle_pool* p, int32_t page) {
    if (page < 0 || page >= p->total || !p->in_use[page]) return; /* unknown page: ignored, as the reference does */
    p->in_use[page] = 0;
    pool_push(p, page);
}

int32_t ahpc_oracle_pool_free_count(const ahpc_oracle_pool* p) { return p->count; }
int32_t ahpc_oracle_pool_total(const ahpc_oracle_pool* p) { return p->total; }
