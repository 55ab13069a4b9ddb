// FlashAttention forward on the gfx950 matrix cores (fp16 / bf16 storage, fp32 accumulate).
//
// One workgroup = 4 wavefronts = 128*QB query rows of one (sequence, head); it walks the keys in
// tiles of 64.  Per tile and wavefront:
//   S^T = K * Q^T      v_mfma_f32_32x32x16: A = K rows from LDS, B = Q^T held in registers for the
//                      whole kernel.  In the 32x32 result a lane owns ONE query column (lane%32)
//                      and 16 of the 32 key rows, so the softmax row reductions are in-lane plus
//                      one exchange with lane^32.
//   P^T = exp2(c*S^T - c*m)   online softmax in registers (c = scale*log2 e), fp32.
//   O^T += V^T * P^T   A = V^T rows from LDS, B = P^T straight from the registers S^T was in: the
//                      accumulator layout of the first product is the B-operand layout of the
//                      second once the 16 keys of a k-step are taken in the order
//                      key = 8*(e/4) + 4*(lane/32) + e%4 (e = 0..7); V^T is written to LDS in that
//                      same order, so no data moves between the two products.
// O^T keeps the query in the lane column, so the per-row rescale factors are per-lane scalars.
//
// LDS: K tile [64][D] with rows padded by 16 B (bank-conflict-free 16-B row reads); V^T tile
// [D][64] built by a 4x8 in-register transpose (v_perm_b32) of what each thread loaded, XOR-swizzled
// in 16-B columns so that both the 8-B transpose writes and the 16-B operand reads are conflict free.
// The next tile's global loads are issued before the current tile's math and parked in registers.
#pragma once

#include "ahpc_device.hpp"

namespace ahpc {

struct FlashParams {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    const int32_t* cu_seqlens;  // ragged batches only
    int64_t stride_b, stride_n, stride_h;
    int32_t N;                  // sequence length (dense) / longest sequence (ragged)
    int32_t H;
    int32_t n_qtiles;           // query tiles per sequence (of the longest one)
    int32_t total_blocks;       // B * H * n_qtiles
    int32_t blocks_per_xcd;     // ceil(total_blocks / 8)
    float scale_log2;           // scale * log2(e)
};

constexpr int kFlashThreads = 256;
constexpr int kFlashKeys = 64;  // keys per tile

template <int D> struct FlashLds {
    static constexpr int kRowBytes = D * 2 + 16;
    static constexpr int kBytesK = kFlashKeys * kRowBytes;
    static constexpr int kBytesV = D * 128;
    static constexpr int kBytes = kBytesK + kBytesV;
};

template <typename T, int D, int QB, bool CAUSAL, bool VARLEN>
__global__ __launch_bounds__(kFlashThreads) void flash_fwd_mfma_kernel(const FlashParams p) {
    constexpr int BM = 128 * QB;       // query rows per workgroup
    constexpr int CPR = D / 8;         // 16-byte chunks per row
    constexpr int KS = D / 16;         // k-steps of the first product
    constexpr int MB = D / 32;         // 32-row blocks of O^T
    constexpr int KROWS = kFlashThreads / CPR;            // K rows covered by one pass of the block
    constexpr int KPASS = kFlashKeys / KROWS;             // passes to cover 64 keys
    constexpr int KROW = FlashLds<D>::kRowBytes;
    constexpr int VTHREADS = 16 * CPR;                    // threads that carry a 4-key x 8-lane V patch

    __shared__ __attribute__((aligned(16))) unsigned char lds[FlashLds<D>::kBytes];
    unsigned char* const lds_k = lds;
    unsigned char* const lds_v = lds + FlashLds<D>::kBytesK;

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int col = lane & 31;   // query column / operand row owned by this lane
    const int half = lane >> 5;

    // Workgroup id -> (sequence*head, query tile).  Consecutive logical ids run on the same XCD so
    // that the tiles of one head share that XCD's L2; within a head the long (late) tiles go first.
    const int xcd = blockIdx.x & 7;
    const int logical = xcd * p.blocks_per_xcd + (blockIdx.x >> 3);
    if (logical >= p.total_blocks) return;
    const int bh = logical / p.n_qtiles;
    const int qt = p.n_qtiles - 1 - (logical - bh * p.n_qtiles);
    const int b = bh / p.H;
    const int h = bh - b * p.H;

    int L;
    int64_t base;
    if (VARLEN) {
        const int s0 = p.cu_seqlens[b];
        L = p.cu_seqlens[b + 1] - s0;
        base = (int64_t)s0 * p.stride_n + (int64_t)h * p.stride_h;
    } else {
        L = p.N;
        base = (int64_t)b * p.stride_b + (int64_t)h * p.stride_h;
    }
    const int q_tile0 = qt * BM;
    if (q_tile0 >= L) return;

    const T* const gq = static_cast<const T*>(p.q) + base;
    const T* const gk = static_cast<const T*>(p.k) + base;
    const T* const gv = static_cast<const T*>(p.v) + base;
    T* const go = static_cast<T*>(p.o) + base;
    const int64_t sn = p.stride_n;

    // ---- Q^T operands, kept for the whole kernel --------------------------------------------
    const int qw = q_tile0 + wave * 32 * QB;  // first query row of this wavefront
    u32x4 qreg[QB][KS];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        int row = qw + 32 * qb + col;
        row = row < L ? row : L - 1;
        const T* src = gq + (int64_t)row * sn + 8 * half;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qreg[qb][ks] = *reinterpret_cast<const u32x4*>(src + 16 * ks);
    }

    // ---- per-thread tile-load geometry ----------------------------------------------------------
    const int chunk = tid % CPR;          // 16-byte chunk of the row
    const int krow0 = tid / CPR;          // first K row this thread carries
    const int vquad = tid / CPR;          // V: keys 4*vquad .. 4*vquad+3 (threads < VTHREADS)
    // V^T position of the quad: key 16g + 8a + 4hh + b  ->  position 16g + 8hh + 4a + b
    const int vpos = 16 * (vquad >> 2) + 8 * (vquad & 1) + 4 * ((vquad >> 1) & 1);
    const int vcx = (chunk & 7);          // (row/8)%8 of the rows 8*chunk + j this thread writes

    u32x4 kreg[KPASS];
    u32x4 vreg[4];

    auto load_tile = [&](int k0) {
#pragma unroll
        for (int i = 0; i < KPASS; ++i) {
            int key = k0 + krow0 + i * KROWS;
            key = key < L ? key : L - 1;
            kreg[i] = *reinterpret_cast<const u32x4*>(gk + (int64_t)key * sn + 8 * chunk);
        }
        if (tid < VTHREADS) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = k0 + 4 * vquad + r;
                const int ck = key < L ? key : L - 1;
                u32x4 t = *reinterpret_cast<const u32x4*>(gv + (int64_t)ck * sn + 8 * chunk);
                if (key >= L) t = u32x4{0u, 0u, 0u, 0u};
                vreg[r] = t;
            }
        }
    };

    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < KPASS; ++i)
            *reinterpret_cast<u32x4*>(lds_k + (krow0 + i * KROWS) * KROW + chunk * 16) = kreg[i];
        if (tid < VTHREADS) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // dword i of each key row holds lanes 2i (low) and 2i+1 (high)
                const uint32_t lo01 = __builtin_amdgcn_perm(vreg[1][i], vreg[0][i], 0x05040100u);
                const uint32_t lo23 = __builtin_amdgcn_perm(vreg[3][i], vreg[2][i], 0x05040100u);
                const uint32_t hi01 = __builtin_amdgcn_perm(vreg[1][i], vreg[0][i], 0x07060302u);
                const uint32_t hi23 = __builtin_amdgcn_perm(vreg[3][i], vreg[2][i], 0x07060302u);
                const int row_lo = 8 * chunk + 2 * i;
                const int row_hi = row_lo + 1;
                const int x_lo = ((2 * i) ^ vcx) << 4;
                const int x_hi = ((2 * i + 1) ^ vcx) << 4;
                *reinterpret_cast<u32x2*>(lds_v + row_lo * 128 + ((2 * vpos) ^ x_lo)) = u32x2{lo01, lo23};
                *reinterpret_cast<u32x2*>(lds_v + row_hi * 128 + ((2 * vpos) ^ x_hi)) = u32x2{hi01, hi23};
            }
        }
    };

    // ---- running state ----------------------------------------------------------------------------
    f32x16 oacc[MB][QB];
    float m_run[QB], l_run[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.0f;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[mb][qb][r] = 0.0f;
    }

    int k_end = L;
    if (CAUSAL) k_end = (q_tile0 + BM) < L ? (q_tile0 + BM) : L;
    const int n_tiles = (k_end + kFlashKeys - 1) / kFlashKeys;
    const float c = p.scale_log2;

    load_tile(0);
    for (int t = 0; t < n_tiles; ++t) {
        const int k0 = t * kFlashKeys;
        __syncthreads();  // every wavefront is done reading the previous tile
        store_tile();
        __syncthreads();
        if (t + 1 < n_tiles) load_tile(k0 + kFlashKeys);

        // a wavefront whose queries all precede this tile has nothing to add
        if (CAUSAL && k0 > qw + 32 * QB - 1) continue;

        // ---- S^T = K Q^T ---------------------------------------------------------------------------
        f32x16 s[2][QB];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                for (int r = 0; r < 16; ++r) s[kb][qb][r] = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            const unsigned char* arow = lds_k + (32 * kb + col) * KROW + 16 * half;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const u32x4 a = *reinterpret_cast<const u32x4*>(arow + 32 * ks);
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) s[kb][qb] = mfma_32x32x16<T>(a, qreg[qb][ks], s[kb][qb]);
            }
        }

        // ---- online softmax, P^T packed as the B operand of the second product ---------------
        const bool need_mask = (k0 + kFlashKeys > L) || (CAUSAL && (k0 + kFlashKeys - 1 > qw));
        u32x4 pb[QB][4];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const int qrow = qw + 32 * qb + col;
            if (need_mask) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int key = k0 + 32 * kb + 8 * (r >> 2) + 4 * half + (r & 3);
                        const bool ok = key < L && (!CAUSAL || key <= qrow);
                        s[kb][qb][r] = ok ? s[kb][qb][r] : -INFINITY;
                    }
            }
            float mx = s[0][qb][0];
#pragma unroll
            for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[0][qb][r]);
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[1][qb][r]);
            mx = fmaxf(mx, swap_halves(mx));
            const float m_new = fmaxf(m_run[qb], mx);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = fast_exp2((m_run[qb] - m_use) * c);
            const float neg = -m_use * c;
            float sum = 0.0f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float pv = fast_exp2(__builtin_fmaf(s[kb][qb][r], c, neg));
                    s[kb][qb][r] = pv;
                    sum += pv;
                }
            l_run[qb] = l_run[qb] * alpha + sum;
            m_run[qb] = m_new;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[mb][qb][r] *= alpha;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int kb = g >> 1, r0 = 8 * (g & 1);
                pb[qb][g] = u32x4{pack2<T>(s[kb][qb][r0 + 0], s[kb][qb][r0 + 1]), pack2<T>(s[kb][qb][r0 + 2], s[kb][qb][r0 + 3]),
                                  pack2<T>(s[kb][qb][r0 + 4], s[kb][qb][r0 + 5]), pack2<T>(s[kb][qb][r0 + 6], s[kb][qb][r0 + 7])};
            }
        }

        // ---- O^T += V^T P^T ------------------------------------------------------------------------
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int row = 32 * mb + col;
            const int x = (row & 7) ^ ((row >> 3) & 7);
            const unsigned char* vrow = lds_v + row * 128;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x4 a = *reinterpret_cast<const u32x4*>(vrow + (((2 * g + half) ^ x) << 4));
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) oacc[mb][qb] = mfma_32x32x16<T>(a, pb[qb][g], oacc[mb][qb]);
            }
        }
    }

    // ---- normalise and store: lane holds, per 32-row block, 4 runs of 4 consecutive lanes of d -----
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const float l = l_run[qb] + swap_halves(l_run[qb]);
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        const int qrow = qw + 32 * qb + col;
        if (qrow < L) {
            T* dst = go + (int64_t)qrow * sn + 4 * half;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const f32x16& a = oacc[mb][qb];
                    const u32x2 w = u32x2{pack2<T>(a[4 * g4 + 0] * inv, a[4 * g4 + 1] * inv),
                                          pack2<T>(a[4 * g4 + 2] * inv, a[4 * g4 + 3] * inv)};
                    *reinterpret_cast<u32x2*>(dst + 32 * mb + 8 * g4) = w;
                }
        }
    }
}

}  // namespace ahpc
