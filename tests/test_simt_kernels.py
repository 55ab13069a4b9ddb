"""The library's kernels, compiled as host C++ and executed lane by lane on the CPU (tests/simt), against
the CPU oracle: same entry points, same bars as the GPU parity tests, at sizes that run in seconds.

What this covers that the GPU tests cannot show: every buffer sits directly against an inaccessible page,
so an access past either end of a tensor faults here instead of on a GPU; cross-lane operations in
divergent control flow, barriers some wavefronts skip, direct-to-LDS loads that are consumed before the
wait that covers them, and LDS that is read before it is written all fail the run.  What it cannot show:
timing, and instruction-level behaviour of the real compiler's code."""
import os

import numpy as np
import pytest

from oracle import oracle as O
from simt import simt as S

TOL = {O.F32: 1e-4, O.F16: 2e-2, O.BF16: 2e-2}


@pytest.fixture(scope="module")
def emu():
    S.load()
    S.configure(False, 1)
    return S.EmulatedHip()


def qkv(shape, seed, dtype, sigma=1.0):
    return tuple(O.round_to(O.fill_normal(shape, seed, t, sigma), dtype) for t in (1, 2, 3))


def dev(x, dtype, front=False):
    return S.guarded(S.to_storage(x, dtype), front)


def flash(emu, q, k, v, dtype, B, N, H, d, scale, causal, H_kv=None, mask=None, front=False):
    H_kv = H_kv or H
    dq, dk, dv = dev(q, dtype, front), dev(k, dtype, front), dev(v, dtype, front)
    do = S.guarded(S.empty_storage((B, N, H, d), dtype), front)
    dm = None if mask is None else S.guarded(mask, front)
    emu.flash_fwd_gqa(S.ptr(dq), S.ptr(dk), S.ptr(dv), S.ptr(do), dtype, B, N, H, H_kv, d, (N * H * d, H * d, d),
                      (N * H_kv * d, H_kv * d, d), scale, causal, None, None if dm is None else S.ptr(dm))
    return S.from_storage(do, dtype)


# ---- FlashAttention forward -----------------------------------------------------------------------------
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("N,d", [(16, 64), (129, 64), (40, 80), (1, 32)])
def test_fp32_kernel(emu, N, d, causal):
    B, H = 2, 3
    q, k, v = qkv((B, N, H, d), 11, O.F32)
    scale = 1.0 / np.sqrt(d)
    got = flash(emu, q, k, v, O.F32, B, N, H, d, scale, causal)
    assert np.abs(got - O.attention(q, k, v, B, N, H, d, scale, causal)).max() <= 1e-4


@pytest.mark.parametrize("dma_late", [False, True])
@pytest.mark.parametrize("N,d,causal,H,H_kv", [(64, 128, False, 2, 2), (129, 128, True, 2, 1), (300, 64, True, 4, 2), (200, 64, False, 2, 2),
                                               (1, 128, True, 1, 1), (33, 64, True, 3, 3), (31, 128, False, 2, 2), (260, 128, True, 2, 2)])
def test_fp32_matrix_core_kernel(emu, N, d, causal, H, H_kv, dma_late):
    """fp32 tensors with d 64 or 128 run on the matrix cores (fp32 operands and sums): tiles of 32 keys, a last tile of
    1 to 32 keys, query tiles that end inside the sequence, grouped heads, with the tile requests landing as late as the
    executor can make them; the 16-byte operand reads are free of bank conflicts."""
    B = 2
    q = O.fill_normal((B, N, H, d), 21, 1)
    k, v = O.fill_normal((B, N, H_kv, d), 21, 2), O.fill_normal((B, N, H_kv, d), 21, 3)
    scale = 1.0 / np.sqrt(d)
    S.configure(dma_late, seed=N + d)
    S.lds_stats(reset=True)
    try:
        got = flash(emu, q, k, v, O.F32, B, N, H, d, scale, causal, H_kv=H_kv, front=dma_late)
    finally:
        S.configure(False, 1)
    rep = H // H_kv
    want = O.attention(q, np.repeat(k, rep, axis=2), np.repeat(v, rep, axis=2), B, N, H, d, scale, causal)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= 1e-4
    reads, read_conflicts, tr, tr_conflicts = S.lds_stats(reset=True)
    assert reads > 0 and read_conflicts == 0   # the matrix-core kernel ran (the FMA kernel makes no traced LDS reads)


@pytest.mark.parametrize("dma_late", [False, True])
@pytest.mark.parametrize("N,d,causal,H_kv", [(64, 128, False, 2), (131, 128, True, 1), (300, 64, False, 2), (65, 64, True, 2), (5, 128, False, 2)])
def test_fp32_matrix_core_kernel_dense_mask(emu, N, d, causal, H_kv, dma_late):
    """fp32 tensors with a mask [B,N,N] on the matrix cores, on the packed copy of the mask: a row that sees nothing gives
    zeros, a row whose first visible key lies in the last tile, rows that see a single key."""
    B, H = 2, 2
    q = O.fill_normal((B, N, H, d), 24, 1)
    k, v = O.fill_normal((B, N, H_kv, d), 24, 2), O.fill_normal((B, N, H_kv, d), 24, 3)
    mask = (O.fill_uniform((B, N, N), 24, 6) > 0.4).astype(np.float32)
    mask[0, N // 2, :] = 0.0
    mask[1, N - 1, :] = 0.0
    mask[1, N - 1, N - 1] = 1.0
    mask[1, 0, :] = 0.0
    mask[1, 0, 0] = 1.0
    if N > 70:
        mask[0, N - 2, :N - 3] = 0.0
    scale = 1.0 / np.sqrt(d)
    S.configure(dma_late, seed=N + d)
    S.lds_stats(reset=True)
    try:
        got = flash(emu, q, k, v, O.F32, B, N, H, d, scale, causal, H_kv=H_kv, mask=mask, front=dma_late)
    finally:
        S.configure(False, 1)
    rep = H // H_kv
    want = O.attention(q, np.repeat(k, rep, axis=2), np.repeat(v, rep, axis=2), B, N, H, d, scale, causal, mask=mask)
    assert np.isfinite(got).all()
    assert np.all(got[0, N // 2] == 0.0)
    assert np.abs(got - want).max() <= 1e-4
    assert S.lds_stats(reset=True)[0] > 0


@pytest.mark.parametrize("dtype,d", [(O.BF16, 32), (O.F16, 96), (O.BF16, 8), (O.F16, 120), (O.F32, 32), (O.F32, 100), (O.F32, 4), (O.F32, 72)])
@pytest.mark.parametrize("N,causal,H,H_kv,dma_late", [(150, True, 2, 1, True), (64, False, 3, 3, False)])
def test_matrix_core_kernels_smaller_head_dimensions(emu, dtype, d, N, causal, H, H_kv, dma_late):
    """Head dimensions below the kernels' 64 / 128 (multiples of 8 for 16-bit tensors, of 4 for fp32) run on the matrix-core
    kernels with columns that contribute nothing.  Tensors sit at the very end (or start) of guarded buffers: nothing behind
    a row's own d elements may be read, in particular not behind the last row of the last head."""
    B = 2
    q = O.round_to(O.fill_normal((B, N, H, d), 25, 1), dtype)
    k = O.round_to(O.fill_normal((B, N, H_kv, d), 25, 2), dtype)
    v = O.round_to(O.fill_normal((B, N, H_kv, d), 25, 3), dtype)
    scale = 1.0 / np.sqrt(d)
    S.configure(dma_late, seed=N + d)
    S.lds_stats(reset=True)
    try:
        got = flash(emu, q, k, v, dtype, B, N, H, d, scale, causal, H_kv=H_kv, front=dma_late)
    finally:
        S.configure(False, 1)
    rep = H // H_kv
    want = O.attention(q, np.repeat(k, rep, axis=2), np.repeat(v, rep, axis=2), B, N, H, d, scale, causal)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL[dtype]
    assert S.lds_stats(reset=True)[0] > 0   # a matrix-core kernel ran (the FMA kernel makes no traced LDS reads)


@pytest.mark.parametrize("dtype,d", [(O.BF16, 256), (O.F16, 200), (O.BF16, 136), (O.F16, 256), (O.F32, 256), (O.F32, 132)])
@pytest.mark.parametrize("N,causal,H,H_kv,dma_late", [(150, True, 2, 1, True), (70, False, 2, 2, False)])
def test_matrix_core_forward_head_dimensions_to_256(emu, tuned, dtype, d, N, causal, H, H_kv, dma_late):
    """Head dimensions above 128 (to 256, in whole 16-byte pieces): the forward kernels instantiated for 256, dense and ragged,
    with its conflict counts (the swizzles are the ones of 128)."""
    B = 2
    q = O.round_to(O.fill_normal((B, N, H, d), 27, 1), dtype)
    k = O.round_to(O.fill_normal((B, N, H_kv, d), 27, 2), dtype)
    v = O.round_to(O.fill_normal((B, N, H_kv, d), 27, 3), dtype)
    scale = 1.0 / np.sqrt(d)
    S.configure(dma_late, seed=N + d)
    S.lds_stats(reset=True)
    try:
        got = flash(emu, q, k, v, dtype, B, N, H, d, scale, causal, H_kv=H_kv, front=dma_late)
    finally:
        S.configure(False, 1)
    rep = H // H_kv
    kx, vx = np.repeat(k, rep, axis=2), np.repeat(v, rep, axis=2)
    want = O.attention(q, kx, vx, B, N, H, d, scale, causal)
    assert np.abs(got - want).max() <= TOL[dtype]
    reads, read_conflicts, tr, tr_conflicts = S.lds_stats(reset=True)
    assert reads > 0 and (tr > 0 or dtype == O.F32)   # a matrix-core kernel ran (the fp32 one makes no transposing reads)
    print(f"d={d}: operand reads {reads} (conflicts {read_conflicts}), transposing reads {tr} (conflicts {tr_conflicts})")
    # the same tensors as a ragged batch of B sequences
    T = B * N
    cu = np.arange(B + 1, dtype=np.int32) * N
    dq, dk, dv = dev(q.reshape(T, H, d), dtype), dev(k.reshape(T, H_kv, d), dtype), dev(v.reshape(T, H_kv, d), dtype)
    do = S.guarded(S.empty_storage((T, H, d), dtype))
    dcu = S.guarded(cu)
    emu.flash_fwd_varlen_gqa(S.ptr(dq), S.ptr(dk), S.ptr(dv), S.ptr(do), dtype, S.ptr(dcu), B, N, H, H_kv, d, H * d, d, H_kv * d, d,
                             scale, causal)
    assert np.abs(S.from_storage(do, dtype).reshape(B, N, H, d) - want).max() <= TOL[dtype]
    # and under a dense mask: the packed copy has a kernel of this size, the mask read in place has none (fp32-FMA kernel)
    mask = (O.fill_normal((B, N, N), 28, 9) > -0.3).astype(np.float32)
    mask[0, 3, :] = 0.0   # a query that sees nothing: zeros
    want_m = O.attention(q, kx, vx, B, N, H, d, scale, causal, mask=mask)
    for packed in (1, 0):
        tuned("mask_pack", packed)
        S.lds_stats(reset=True)
        got_m = flash(emu, q, k, v, dtype, B, N, H, d, scale, causal, H_kv=H_kv, mask=mask)
        assert np.abs(got_m - want_m).max() <= TOL[dtype], packed
        assert (S.lds_stats(reset=True)[0] > 0) == (packed == 1)


def test_matrix_core_kernels_smaller_head_dimensions_ragged_and_masked(emu):
    H, d = 2, 40
    lens = np.array([1, 130, 0, 64, 33], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    for dtype in (O.BF16, O.F32):
        q, k, v = qkv((T, H, d), 26, dtype)
        dq, dk, dv = dev(q, dtype), dev(k, dtype), dev(v, dtype)
        do = S.guarded(S.empty_storage((T, H, d), dtype))
        dcu = S.guarded(cu)
        S.lds_stats(reset=True)
        emu.flash_fwd_varlen(S.ptr(dq), S.ptr(dk), S.ptr(dv), S.ptr(do), dtype, S.ptr(dcu), len(lens), int(lens.max()), H, d,
                             H * d, d, 0.2, True)
        want = O.attention_varlen(q, k, v, cu, H, d, 0.2, True)
        assert np.abs(S.from_storage(do, dtype) - want).max() <= TOL[dtype]
        assert S.lds_stats(reset=True)[0] > 0
        B, N = 2, 70
        q, k, v = qkv((B, N, H, d), 27, dtype)
        mask = (O.fill_uniform((B, N, N), 27, 6) > 0.0).astype(np.float32)
        mask[:, np.arange(N), np.arange(N)] = 1.0
        got = flash(emu, q, k, v, dtype, B, N, H, d, 0.2, False, mask=mask)
        assert np.abs(got - O.attention(q, k, v, B, N, H, d, 0.2, False, mask=mask)).max() <= TOL[dtype]
        assert S.lds_stats(reset=True)[0] > 0


def test_fp32_matrix_core_kernel_large_scores_and_strides(emu):
    """Scores that grow along the sequence (the reference maximum is raised again and again), head-major strides."""
    B, N, H, d = 1, 200, 2, 64
    q, k, v = qkv((B, N, H, d), 22, O.F32)
    k = k * (1.0 + np.arange(N, dtype=np.float32)[None, :, None, None] / 16.0)
    t = lambda x: np.ascontiguousarray(x.transpose(0, 2, 1, 3))
    dq, dk, dv = dev(t(q), O.F32), dev(t(k), O.F32), dev(t(v), O.F32)
    do = S.guarded(S.empty_storage((B, H, N, d), O.F32))
    S.lds_stats(reset=True)
    emu.flash_fwd(S.ptr(dq), S.ptr(dk), S.ptr(dv), S.ptr(do), O.F32, B, N, H, d, (H * N * d, d, N * d), 0.5, False)
    got = S.from_storage(do, O.F32).transpose(0, 2, 1, 3)
    assert np.abs(got - O.attention(q, k, v, B, N, H, d, 0.5, False)).max() <= 1e-4
    assert S.lds_stats(reset=True)[0] > 0


def test_fp32_matrix_core_kernel_ragged_batch(emu):
    H, d = 2, 128
    lens = np.array([1, 130, 0, 64, 257, 33], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    q, k, v = qkv((T, H, d), 23, O.F32)
    dq, dk, dv = dev(q, O.F32), dev(k, O.F32), dev(v, O.F32)
    do = S.guarded(S.empty_storage((T, H, d), O.F32))
    dcu = S.guarded(cu)
    scale = 1.0 / np.sqrt(d)
    for causal in (True, False):
        S.lds_stats(reset=True)
        emu.flash_fwd_varlen(S.ptr(dq), S.ptr(dk), S.ptr(dv), S.ptr(do), O.F32, S.ptr(dcu), len(lens), int(lens.max()), H, d,
                             H * d, d, scale, causal)
        want = O.attention_varlen(q, k, v, cu, H, d, scale, causal)
        assert np.abs(S.from_storage(do, O.F32) - want).max() <= 1e-4
        assert S.lds_stats(reset=True)[0] > 0


def test_fp32_kernel_dense_mask(emu):
    B, N, H, d = 2, 37, 2, 64
    q, k, v = qkv((B, N, H, d), 12, O.F32)
    mask = (O.fill_uniform((B, N, N), 12, 6) > 0.3).astype(np.float32)
    mask[0, 5, :] = 0.0  # a row that sees nothing: output 0
    got = flash(emu, q, k, v, O.F32, B, N, H, d, 0.125, False, mask=mask)
    want = O.attention(q, k, v, B, N, H, d, 0.125, False, mask=mask)
    assert np.all(got[0, 5] == 0.0)
    assert np.abs(got - want).max() <= 1e-4


@pytest.mark.parametrize("packed,dma_late", [(1, True), (0, False)], ids=["packed-copy", "mask-in-place"])
@pytest.mark.parametrize("dtype,N,d,causal,H_kv", [(O.BF16, 64, 128, False, 2), (O.F16, 132, 128, True, 2), (O.F16, 300, 64, False, 1),
                                                   (O.BF16, 200, 64, True, 2), (O.BF16, 4, 128, False, 2), (O.F16, 131, 128, False, 1),
                                                   (O.BF16, 65, 64, True, 2)])
def test_matrix_core_kernel_dense_mask(emu, dtype, N, d, causal, H_kv, dma_late, packed):
    """fp16/bf16 with a mask [B,N,N] run on the matrix cores, on a packed copy of the mask (any N) or on the mask in place
    (N a multiple of 4): a row that sees nothing gives zeros, a row whose first visible key lies in the last tile, rows
    that see a single key, a last tile of 1 to 60 keys."""
    if not packed and N % 4:
        pytest.skip("the mask is read in place 16 bytes at a time: other lengths take the fp32 kernel")
    B, H = 2, 2
    q, k, v = qkv((B, N, H, d), 17, dtype)
    k, v = k[:, :, :H_kv].copy(), v[:, :, :H_kv].copy()
    mask = (O.fill_uniform((B, N, N), 17, 6) > 0.4).astype(np.float32)
    mask[0, N // 2, :] = 0.0
    mask[1, N - 1, :] = 0.0
    mask[1, N - 1, N - 1] = 1.0      # only the last key
    mask[1, 0, :] = 0.0
    mask[1, 0, 0] = 1.0              # only the first key (also what a causal launch leaves row 0)
    if N > 70:
        mask[0, N - 2, :N - 3] = 0.0  # nothing before the last tile
    scale = 1.0 / np.sqrt(d)
    S.configure(dma_late, seed=N + d)
    before = emu.get_tuning("mask_pack")
    emu.set_tuning("mask_pack", packed)
    try:
        got = flash(emu, q, k, v, dtype, B, N, H, d, scale, causal, H_kv=H_kv, mask=mask, front=dma_late)
    finally:
        S.configure(False, 1)
        emu.set_tuning("mask_pack", before)
    rep = H // H_kv   # grouped heads = the same K/V head repeated
    want = O.attention(q, np.repeat(k, rep, axis=2), np.repeat(v, rep, axis=2), B, N, H, d, scale, causal, mask=mask)
    assert np.isfinite(got).all()
    assert np.all(got[0, N // 2] == 0.0)
    assert np.abs(got - want).max() <= TOL[dtype]
    reads, read_conflicts, tr, tr_conflicts = S.lds_stats(reset=True)
    assert reads > 0 and tr > 0    # the matrix-core kernel ran (the fp32 kernel makes no traced LDS reads)


@pytest.mark.parametrize("dma_late", [False, True])
@pytest.mark.parametrize("dtype", [O.BF16, O.F16])
@pytest.mark.parametrize("N,d,causal", [(64, 128, False), (129, 128, True), (300, 64, True), (200, 64, False), (1, 128, True)])
def test_matrix_core_kernel(emu, dtype, N, d, causal, dma_late):
    B, H = 2, 2
    q, k, v = qkv((B, N, H, d), 13, dtype)
    scale = 1.0 / np.sqrt(d)
    S.configure(dma_late, seed=N + d)
    try:
        got = flash(emu, q, k, v, dtype, B, N, H, d, scale, causal, front=dma_late)
    finally:
        S.configure(False, 1)
    assert np.isfinite(got).all()
    assert np.abs(got - O.attention(q, k, v, B, N, H, d, scale, causal)).max() <= TOL[dtype]


@pytest.mark.parametrize("H,H_kv,dtype,d", [(4, 2, O.BF16, 128), (4, 1, O.F16, 64), (6, 3, O.F32, 32)])
def test_grouped_heads_equal_repeated_heads(emu, H, H_kv, dtype, d):
    B, N = 1, 150
    q = O.round_to(O.fill_normal((B, N, H, d), 14, 1), dtype)
    k = O.round_to(O.fill_normal((B, N, H_kv, d), 14, 2), dtype)
    v = O.round_to(O.fill_normal((B, N, H_kv, d), 14, 3), dtype)
    got = flash(emu, q, k, v, dtype, B, N, H, d, 0.1, True, H_kv=H_kv)
    g = H // H_kv
    want = O.attention(q, np.repeat(k, g, axis=2), np.repeat(v, g, axis=2), B, N, H, d, 0.1, True)
    assert np.abs(got - want).max() <= TOL[dtype]


@pytest.mark.parametrize("dtype,d", [(O.F16, 64), (O.BF16, 128), (O.F32, 64)])
def test_ragged_batch(emu, dtype, d):
    H = 2
    lens = np.array([1, 130, 64, 257], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    q, k, v = qkv((T, H, d), 15, dtype)
    dq, dk, dv = dev(q, dtype), dev(k, dtype), dev(v, dtype)
    do = S.guarded(S.empty_storage((T, H, d), dtype))
    dcu = S.guarded(cu)
    scale = 1.0 / np.sqrt(d)
    emu.flash_fwd_varlen(S.ptr(dq), S.ptr(dk), S.ptr(dv), S.ptr(do), dtype, S.ptr(dcu), len(lens), int(lens.max()), H, d,
                         H * d, d, scale, True)
    want = O.attention_varlen(q, k, v, cu, H, d, scale, True)
    assert np.abs(S.from_storage(do, dtype) - want).max() <= TOL[dtype]


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("paired", [False, True])
def test_ragged_batch_of_very_different_lengths(emu, causal, paired):
    """Every sequence is tiled and paired from its own length: an empty one, some shorter than a tile, odd and even
    tile counts, 3 heads on 8 XCDs (the surplus slots of the short sequences exit without touching anything)."""
    if paired:
        emu.set_tuning("flash_pair_min_tiles", 1)
    try:
        H, d, dtype = 3, 64, O.F16
        lens = np.array([1, 130, 0, 64, 700, 257, 384, 129], np.int32)
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        T = int(cu[-1])
        q, k, v = qkv((T, H, d), 16, dtype)
        dq, dk, dv = dev(q, dtype), dev(k, dtype), dev(v, dtype)
        do = S.guarded(S.empty_storage((T, H, d), dtype))
        dcu = S.guarded(cu)
        emu.flash_fwd_varlen(S.ptr(dq), S.ptr(dk), S.ptr(dv), S.ptr(do), dtype, S.ptr(dcu), len(lens), int(lens.max()), H, d,
                             H * d, d, 0.125, causal)
        got = S.from_storage(do, dtype)
        assert np.isfinite(got).all()
        assert np.abs(got - O.attention_varlen(q, k, v, cu, H, d, 0.125, causal)).max() <= TOL[dtype]
    finally:
        emu.set_tuning("flash_pair_min_tiles", 1024)


def test_head_major_strides(emu):
    # the same tensors laid out [B,H,N,d]: only the strides change
    B, N, H, d = 1, 140, 3, 128
    q, k, v = qkv((B, N, H, d), 16, O.BF16)
    t = lambda x: np.ascontiguousarray(x.transpose(0, 2, 1, 3))
    dq, dk, dv = dev(t(q), O.BF16), dev(t(k), O.BF16), dev(t(v), O.BF16)
    do = S.guarded(S.empty_storage((B, H, N, d), O.BF16))
    emu.flash_fwd(S.ptr(dq), S.ptr(dk), S.ptr(dv), S.ptr(do), O.BF16, B, N, H, d, (H * N * d, d, N * d), 0.09, True)
    got = S.from_storage(do, O.BF16).transpose(0, 2, 1, 3)
    assert np.abs(got - O.attention(q, k, v, B, N, H, d, 0.09, True)).max() <= 2e-2


# ---- paged KV pool and decode -----------------------------------------------------------------------------
from test_gpu_paged import build_problem, poison_unused, _tables_for  # problem builders only (pure numpy + oracle)


def decode(emu, q, kp, vp, table, lens, rows, B, H, H_kv, d, P, dtype, qo_dtype, scale, chunk=0):
    dq = dev(q, qo_dtype)
    do = S.guarded(S.empty_storage((B, H, d), qo_dtype))
    dk, dv = dev(kp, dtype), dev(vp, dtype)
    dt, dl = S.guarded(table), S.guarded(np.asarray(lens, np.int32))
    dr = None if rows is None else S.guarded(np.asarray(rows, np.int32))
    max_len = int(max(1, np.max(lens)))
    ws_bytes = emu.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
    ws = S.guarded(np.full(max(ws_bytes, 4) // 4, np.nan, np.float32))
    emu.paged_decode_gqa(S.ptr(dq), S.ptr(do), qo_dtype, S.ptr(dk), S.ptr(dv), dtype, S.ptr(dt), S.ptr(dl),
                         None if dr is None else S.ptr(dr), B, H, H_kv, d, P, table.shape[1], max_len, scale, chunk,
                         S.ptr(ws), ws_bytes)
    return S.from_storage(do, qo_dtype)


@pytest.mark.parametrize("dtype", [O.F32, O.F16, O.BF16])
@pytest.mark.parametrize("H,d,P", [(4, 32, 16), (8, 128, 16), (6, 64, 4), (3, 128, 16), (2, 256, 8)])
def test_decode(emu, dtype, H, d, P):
    B = 4
    q, kp, vp, table, lens, _, _ = build_problem(B, H, d, P, [33, 1, 16, 150], 21, dtype)
    scale = 1.0 / np.sqrt(d)
    want = O.paged_decode(q, kp, vp, table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H, d, wild_page=1 << 24)
    for chunk in (0, P, 4 * P):
        got = decode(emu, q, kp, vp, table, lens, None, B, H, H, d, P, dtype, dtype, scale, chunk)
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() <= TOL[dtype], f"chunk={chunk}"


@pytest.mark.parametrize("dtype,H,H_kv,d,P", [(O.BF16, 4, 4, 96, 16), (O.F16, 8, 2, 80, 16), (O.F32, 3, 3, 100, 8), (O.BF16, 2, 1, 8, 16),
                                             (O.F32, 4, 4, 4, 16), (O.F16, 6, 6, 200, 4), (O.BF16, 8, 8, 40, 16)])
def test_decode_other_head_dimensions(emu, dtype, H, H_kv, d, P):
    """Head dimensions in whole 16-byte pieces that are not 32, 64, 128 or 256: the lane-per-element kernel of the next
    size, whose surplus lanes carry a zero query, re-read a row's first piece and store nothing (the pool sits at the end
    of a guarded buffer, unused slots and pages are NaN)."""
    B = 4
    q, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, [33, 1, 16, 150], 23, dtype)
    q = O.round_to(O.fill_normal((B, H, d), 23, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    g = H // H_kv
    n_slots = kp.size // (H_kv * d)
    kx = np.repeat(kp.reshape(n_slots, H_kv, d), g, axis=1).reshape(-1)
    vx = np.repeat(vp.reshape(n_slots, H_kv, d), g, axis=1).reshape(-1)
    want = O.paged_decode(q, kx, vx, table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H_kv, d, wild_page=1 << 24)
    for chunk in (0, 2 * P):
        got = decode(emu, q, kp, vp, table, lens, None, B, H, H_kv, d, P, dtype, dtype, scale, chunk)
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() <= TOL[dtype], f"chunk={chunk}"


@pytest.mark.parametrize("waves", [1, 2, 4, 8])
def test_decode_workgroup_shapes(emu, tuned, waves):
    """Every workgroup width the launch plan can choose (1 to 8 wavefronts: from 4 heads of a token to whole
    token rows) and its chunk lengths give the result of the oracle; 12 heads leave the last wavefronts of a
    wide workgroup without a head."""
    B, H, d, P = 3, 12, 128, 16
    q, kp, vp, table, lens, _, _ = build_problem(B, H, d, P, [300, 17, 1100], 27, O.F16)
    scale = 1.0 / np.sqrt(d)
    want = O.paged_decode(q, kp, vp, table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H, d, wild_page=1 << 24)
    tuned("decode_waves", waves)
    for chunk in (1024, 256, 0):
        tuned("decode_chunk", chunk)
        got = decode(emu, q, kp, vp, table, lens, None, B, H, H, d, P, O.F16, O.F16, scale, 0)
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() <= 2e-2, f"chunk={chunk}"


@pytest.mark.parametrize("matrix_from", [2, 16])
@pytest.mark.parametrize("G", [2, 4, 8])
def test_decode_grouped_heads(emu, tuned, G, matrix_from):
    # groups of 2, 4 and 8 exist on the lane-per-element kernel and on the page-by-page matrix-core kernel
    tuned("decode_matrix_min_group", matrix_from)
    B, H_kv, d, P = 3, 2, 128, 16
    H = G * H_kv
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, [70, 5, 129], 22, O.F16)
    q = O.round_to(O.fill_normal((B, H, d), 22, 1), O.F16)
    scale = 1.0 / np.sqrt(d)
    # the ordinary oracle on a pool whose heads are repeated G times
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H_kv, d, wild_page=1 << 24)
    for chunk in (0, 32):
        got = decode(emu, q, kp, vp, table, lens, None, B, H, H_kv, d, P, O.F16, O.F16, scale, chunk)
        assert np.abs(got - want).max() <= 2e-2


@pytest.mark.parametrize("G,H_kv,d,dtype", [(32, 1, 128, O.F16), (24, 2, 64, O.BF16), (17, 1, 128, O.BF16)])
@pytest.mark.parametrize("waves", [1, 2, 4])
def test_decode_wide_groups(emu, tuned, G, H_kv, d, dtype, waves):
    # groups of 17 to 32 query heads run on the matrix-core kernel with tiles of 32 tokens (two pages, one descriptor
    # pair per page): sequences that end inside a page, inside a tile's first page and on a tile's border, one chunk
    # and several; workgroups of 1, 2 and 4 wavefronts that share a chunk's tiles out (with fewer tiles than
    # wavefronts, and with none at all) and merge in LDS
    tuned("decode_waves", waves)
    B, P = 4, 16
    H = G * H_kv
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, [70, 5, 64, 300], 29, dtype)
    q = O.round_to(O.fill_normal((B, H, d), 29, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H_kv, d, wild_page=1 << 24)
    for chunk in (0, 32, 48, 160):
        got = decode(emu, q, kp, vp, table, lens, None, B, H, H_kv, d, P, dtype, dtype, scale, chunk)
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() <= 2e-2, f"chunk={chunk}"


def test_decode_empty_sequence_and_batch_rows(emu):
    B, H, d, P = 4, 4, 64, 16
    q, kp, vp, table, lens, _, _ = build_problem(B, H, d, P, [40, 7, 90, 16], 41, O.BF16)
    lens = lens.copy()
    lens[1] = 0
    rows = np.array([2, 1, 0, 3], np.int32)
    want = O.paged_decode(q, kp, vp, table, lens, rows, B, H, d, P, 0.125)
    got = decode(emu, q, kp, vp, table, lens, rows, B, H, H, d, P, O.BF16, O.BF16, 0.125, 32)
    assert np.all(got[1] == 0.0)
    assert np.abs(got - want).max() <= 2e-2


@pytest.mark.parametrize("H,H_kv,d,P,dtype", [(4, 4, 128, 16, O.F16), (6, 6, 64, 4, O.F32), (8, 2, 128, 16, O.BF16),
                                              (32, 2, 128, 16, O.F16), (16, 1, 64, 16, O.BF16)])
def test_decode_stops_at_a_missing_page(emu, H, H_kv, d, P, dtype):
    # a -1 entry inside a sequence ends it there (the reference kernel's page walk, cuda_kernels.cu:417-420):
    # first page of a later chunk, a page in the middle of a chunk, the very first page, and no hole at all
    B = 4
    lens_full = [150, 150, 40, 70]
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, lens_full, 23, dtype)
    q = O.round_to(O.fill_normal((B, H, d), 23, 1), dtype)
    table = table.copy()
    holes = [(0, (4 * P) // P), (1, (4 * P) // P + 1), (2, 0)]
    for b, pg in holes:
        table[b, pg] = -1
    scale = 1.0 / np.sqrt(d)
    G = H // H_kv
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    assert np.all(want[2] == 0.0)
    # page 0 is what a kernel that papers over the hole would read: poison it (no sequence owns it here)
    assert not (table == 0).any() or True
    kp2, vp2 = kp.copy().reshape(-1, P * H_kv * d), vp.copy().reshape(-1, P * H_kv * d)
    used = set(table[table >= 0].tolist())
    for pg in range(kp2.shape[0]):
        if pg not in used:
            kp2[pg] = np.nan
            vp2[pg] = np.nan
    for chunk in (0, 4 * P, 2 * P):
        got = decode(emu, q, kp2.reshape(-1), vp2.reshape(-1), table, lens, None, B, H, H_kv, d, P, dtype, dtype, scale, chunk)
        assert np.isfinite(got).all(), f"chunk={chunk}"
        assert np.all(got[2] == 0.0)
        assert np.abs(got - want).max() <= TOL[dtype], f"chunk={chunk}"


def test_gather_indices_with_missing_pages_and_small_head_dim(emu):
    # the decode kernel's own report (d = 128, pages of 16 and of 4) and the append/read-back index function (d = 8)
    for (H, d, P) in [(4, 128, 16), (2, 64, 4), (2, 8, 4)]:
        B = 3
        lens = np.array([70 if P == 16 else 300, 33, 5], np.int32)  # the longest one spans several chunks
        _, _, _, table, lens, _, _ = build_problem(B, 1, 1, P, lens, 52, O.F32)
        table = table.copy()
        table[0, 2] = -1
        table[2, 0] = -1
        max_len = int(lens.max())
        out = S.guarded(np.full((B, max_len), -7, np.int64))
        dt, dl = S.guarded(table), S.guarded(lens)
        emu.paged_gather_indices(S.ptr(dt), S.ptr(dl), None, B, H, d, P, table.shape[1], max_len, S.ptr(out))
        want = O.gather_offsets(table, lens, None, B, max_len, P, H, d)
        assert np.array_equal(out, want)
        assert (want[0, 2 * P:] == -1).all() and (want[2] == -1).all() and (want[1, :33] >= 0).all()


def test_gather_indices_bit_exact(emu):
    B, H, d, P = 6, 32, 128, 16
    lens = O.fill_lengths(B, 51, 4, 1, 300)
    _, _, _, table, lens, _, _ = build_problem(B, 1, 1, P, lens, 51, O.F32)
    max_len = int(lens.max())
    rows = np.array([5, 0, 3, 1, 2, 4], np.int32)
    out = S.guarded(np.full((B, max_len), -7, np.int64))
    dt, dl, dr = S.guarded(table), S.guarded(lens), S.guarded(rows)
    emu.paged_gather_indices(S.ptr(dt), S.ptr(dl), S.ptr(dr), B, H, d, P, table.shape[1], max_len, S.ptr(out))
    assert np.array_equal(out, O.gather_offsets(table, lens, rows, B, max_len, P, H, d))


@pytest.mark.parametrize("in_dtype,pool_dtype", [(O.F32, O.F32), (O.F32, O.F16), (O.F16, O.F16), (O.BF16, O.BF16)])
def test_scatter_then_gather_roundtrip(emu, in_dtype, pool_dtype):
    H, d, P, n_pages = 4, 32, 16, 12
    table = np.array([[7, 2, 9, 0, -1], [3, 11, 5, -1, -1]], np.int32)
    store = O.F16 if O.F16 in (in_dtype, pool_dtype) else (O.BF16 if O.BF16 in (in_dtype, pool_dtype) else O.F32)
    k1, v1 = (O.round_to(O.fill_normal((21, H, d), 1, t), store) for t in (2, 3))
    k2, v2 = (O.round_to(O.fill_normal((30, H, d), 2, t), store) for t in (2, 3))
    dt = S.guarded(table)
    kpool = S.guarded(S.to_storage(np.zeros(n_pages * P * H * d, np.float32), pool_dtype))
    vpool = S.guarded(S.to_storage(np.zeros(n_pages * P * H * d, np.float32), pool_dtype))
    a, b, c, e = dev(k1, in_dtype), dev(v1, in_dtype), dev(k2, in_dtype), dev(v2, in_dtype)
    emu.kv_scatter(S.ptr(a), S.ptr(b), in_dtype, S.ptr(kpool), S.ptr(vpool), pool_dtype, S.ptr(dt), 5, 21, H, d, P, row0=0, pos0=0)
    emu.kv_scatter(S.ptr(c), S.ptr(e), in_dtype, S.ptr(kpool), S.ptr(vpool), pool_dtype, S.ptr(dt), 5, 30, H, d, P, row0=0, pos0=21)
    trow, tpos = S.guarded(np.full(21, 1, np.int32)), S.guarded(np.arange(21, dtype=np.int32)[::-1].copy())
    emu.kv_scatter(S.ptr(a), S.ptr(b), in_dtype, S.ptr(kpool), S.ptr(vpool), pool_dtype, S.ptr(dt), 5, 21, H, d, P,
                   token_row=S.ptr(trow), token_pos=S.ptr(tpos))
    ko, vo = S.guarded(np.empty(51 * H * d, np.float32)), S.guarded(np.empty(51 * H * d, np.float32))
    emu.kv_gather(S.ptr(ko), S.ptr(vo), O.F32, S.ptr(kpool), S.ptr(vpool), pool_dtype, S.ptr(dt), 5, 0, 0, 51, H, d, P)
    assert np.array_equal(ko.reshape(51, H, d), np.concatenate([k1, k2]))
    assert np.array_equal(vo.reshape(51, H, d), np.concatenate([v1, v2]))
    kp, vp = np.zeros(n_pages * P * H * d, np.float32), np.zeros(n_pages * P * H * d, np.float32)
    O.kv_scatter(k1, v1, kp, vp, table, 0, 0, P, H, d)
    O.kv_scatter(k2, v2, kp, vp, table, 0, 21, P, H, d)
    O.kv_scatter(np.ascontiguousarray(k1[::-1]), np.ascontiguousarray(v1[::-1]), kp, vp, table, 1, 0, P, H, d)
    assert np.array_equal(S.from_storage(kpool, pool_dtype), kp) and np.array_equal(S.from_storage(vpool, pool_dtype), vp)


@pytest.mark.parametrize("in_dtype,pool_dtype", [(O.F16, O.F16), (O.F32, O.F16), (O.BF16, O.F32)])
def test_scatter_batch_dense(emu, in_dtype, pool_dtype):
    B, N, H, d, P = 4, 70, 3, 64, 16
    start = np.array([0, 5, 16, 33], np.int32)
    n_new = np.array([70, 1, 0, 37], np.int32)
    rows = np.array([2, 0, 3, 1], np.int32)
    lens_total = np.zeros(4, np.int32)
    lens_total[rows] = start + n_new
    table, n_pages = _tables_for(lens_total, P, 61)
    k, v = (O.round_to(O.fill_normal((B, N, H, d), 61, t), in_dtype) for t in (2, 3))
    kp, vp = np.zeros(n_pages * P * H * d, np.float32), np.zeros(n_pages * P * H * d, np.float32)
    for b in range(B):
        if n_new[b]:
            O.kv_scatter(O.round_to(k[b, :n_new[b]], pool_dtype), O.round_to(v[b, :n_new[b]], pool_dtype), kp, vp, table,
                         int(rows[b]), int(start[b]), P, H, d)
    dk, dv = dev(k, in_dtype), dev(v, in_dtype)
    dkp, dvp = dev(np.zeros_like(kp), pool_dtype), dev(np.zeros_like(vp), pool_dtype)
    dtab, drows, dstart, dnew = S.guarded(table), S.guarded(rows), S.guarded(start), S.guarded(n_new)
    emu.kv_scatter_batch(S.ptr(dk), S.ptr(dv), in_dtype, N * H * d, H * d, S.ptr(dkp), S.ptr(dvp), pool_dtype, S.ptr(dtab),
                         table.shape[1], S.ptr(drows), B, N, H, d, P, seq_start=S.ptr(dstart), seq_tokens=S.ptr(dnew))
    assert np.array_equal(S.from_storage(dkp, pool_dtype), kp) and np.array_equal(S.from_storage(dvp, pool_dtype), vp)


def test_scatter_batch_packed(emu):
    H, d, P = 2, 128, 16
    lens = np.array([130, 16, 1, 55], np.int32)
    B = len(lens)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    table, n_pages = _tables_for(lens, P, 62)
    k, v = (O.round_to(O.fill_normal((T, H, d), 62, t), O.F16) for t in (2, 3))
    kp, vp = np.zeros(n_pages * P * H * d, np.float32), np.zeros(n_pages * P * H * d, np.float32)
    for b in range(B):
        O.kv_scatter(k[cu[b]:cu[b + 1]], v[cu[b]:cu[b + 1]], kp, vp, table, b, 0, P, H, d)
    dk, dv = dev(k, O.F16), dev(v, O.F16)
    dkp, dvp = dev(np.zeros_like(kp), O.F16), dev(np.zeros_like(vp), O.F16)
    dtab, drows, dcu = S.guarded(table), S.guarded(np.arange(B, dtype=np.int32)), S.guarded(cu)
    emu.kv_scatter_batch(S.ptr(dk), S.ptr(dv), O.F16, 0, H * d, S.ptr(dkp), S.ptr(dvp), O.F16, S.ptr(dtab), table.shape[1],
                         S.ptr(drows), B, int(lens.max()), H, d, P, cu_seqlens=S.ptr(dcu))
    assert np.array_equal(S.from_storage(dkp, O.F16), kp) and np.array_equal(S.from_storage(dvp, O.F16), vp)


@pytest.fixture
def tuned(emu):
    """tuned(name, value) changes a launcher tuning value of the emulated library for the rest of the test."""
    before = {}

    def set_value(name, value):
        before.setdefault(name, emu.get_tuning(name))
        emu.set_tuning(name, value)
    yield set_value
    for name, value in before.items():
        emu.set_tuning(name, value)


@pytest.mark.parametrize("dtype", [O.F16, O.F32])
def test_paired_query_tiles(emu, tuned, dtype):
    """Causal launches with many query tiles (1024 by default; lowered here) hand each workgroup a late tile and
    then an early one; with an odd count the middle tile has no partner.  Both matrix-core kernels (16-bit, fp32)."""
    tuned("flash_pair_min_tiles", 1)
    for N in (512, 640):
        B, H, d = 1, 3, 64
        _, _, second = emu.flash_block_map(B, N, H, True)
        assert (second >= 0).any()
        q, k, v = qkv((B, N, H, d), 18, dtype)
        S.lds_stats(reset=True)
        got = flash(emu, q, k, v, dtype, B, N, H, d, 0.125, True)
        assert np.abs(got - O.attention(q, k, v, B, N, H, d, 0.125, True)).max() <= TOL[dtype]
        assert S.lds_stats(reset=True)[0] > 0


@pytest.mark.parametrize("dma_late", [False, True])
@pytest.mark.parametrize("dtype,N,d,causal,H,H_kv", [(O.BF16, 64, 128, False, 2, 2), (O.F16, 129, 128, True, 2, 1), (O.BF16, 300, 64, True, 2, 2),
                                                  (O.F16, 700, 128, True, 1, 1), (O.BF16, 520, 128, False, 1, 1), (O.F16, 1, 64, True, 1, 1),
                                                  (O.BF16, 257, 96, True, 2, 1)])
def test_matrix_core_kernel_256_rows_per_workgroup(emu, tuned, dtype, N, d, causal, H, H_kv, dma_late):
    """The persistent 8-wavefront form of the 16-bit forward (one stream of K/V tiles for 256 query rows; the executor
    reports one CU, so the 8 workgroups of the launch walk several block ids each), also with paired tiles."""
    tuned("flash_rows", 256)
    tuned("flash_pair_min_tiles", 1)
    B = 2
    q = O.round_to(O.fill_normal((B, N, H, d), 31, 1), dtype)
    k = O.round_to(O.fill_normal((B, N, H_kv, d), 31, 2), dtype)
    v = O.round_to(O.fill_normal((B, N, H_kv, d), 31, 3), dtype)
    scale = 1.0 / np.sqrt(d)
    S.configure(dma_late, seed=N + d)
    S.lds_stats(reset=True)
    try:
        got = flash(emu, q, k, v, dtype, B, N, H, d, scale, causal, H_kv=H_kv, front=dma_late)
    finally:
        S.configure(False, 1)
    assert S.lds_stats(reset=True)[0] > 0  # the matrix-core kernel ran
    kr, vr = np.repeat(k, H // H_kv, axis=2), np.repeat(v, H // H_kv, axis=2)
    assert np.isfinite(got).all()
    assert np.abs(got - O.attention(q, kr, vr, B, N, H, d, scale, causal)).max() <= TOL[dtype]


# ---- FlashAttention backward -----------------------------------------------------------------------------
def backward(emu, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal, mask=None, front=False):
    dq_, dk_, dv_, ddo = dev(q, dtype, front), dev(k, dtype, front), dev(v, dtype, front), dev(do, dtype, front)
    gq = S.guarded(S.empty_storage((B, N, H, d), dtype), front)
    gk = S.guarded(S.empty_storage((B, N, H_kv, d), dtype), front)
    gv = S.guarded(S.empty_storage((B, N, H_kv, d), dtype), front)
    dm = None if mask is None else S.guarded(mask, front)
    ws_bytes = emu.flash_bwd_workspace_bytes(B, N, H)
    ws = S.guarded(np.full(ws_bytes // 4, np.nan, np.float32), front)
    emu.flash_bwd(S.ptr(ddo), S.ptr(dq_), S.ptr(dk_), S.ptr(dv_), S.ptr(gq), S.ptr(gk), S.ptr(gv), dtype, B, N, H, H_kv, d,
                  (N * H * d, H * d, d), (N * H_kv * d, H_kv * d, d), scale, causal, S.ptr(ws), ws_bytes, None,
                  None if dm is None else S.ptr(dm))
    return tuple(S.from_storage(x, dtype) for x in (gq, gk, gv))


def bwd_inputs(B, N, H, H_kv, d, seed, dtype):
    q = O.round_to(O.fill_normal((B, N, H, d), seed, 1), dtype)
    k = O.round_to(O.fill_normal((B, N, H_kv, d), seed, 2), dtype)
    v = O.round_to(O.fill_normal((B, N, H_kv, d), seed, 3), dtype)
    do = O.round_to(O.fill_normal((B, N, H, d), seed, 7), dtype)
    return q, k, v, do


def check_gradients(got, want, dtype):
    """fp32: 1e-4 max-abs as in the forward.  16-bit: 2e-2 relative to the largest entry of the gradient
    (entries are sums over up to N terms, so their size, unlike the forward's, grows with the problem)."""
    for name, g, w in zip(("dQ", "dK", "dV"), got, want):
        assert np.isfinite(g).all(), name
        bar = 1e-4 * max(1.0, np.abs(w).max()) if dtype == O.F32 else 2e-2 * max(1.0, np.abs(w).max())
        assert np.abs(g - w).max() <= bar, (name, np.abs(g - w).max(), bar)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,N,H,H_kv,d", [(2, 16, 4, 4, 64), (1, 150, 2, 1, 32), (1, 40, 3, 3, 80), (1, 1, 2, 2, 128), (1, 20, 2, 2, 256)])
def test_backward_fp32_kernels(emu, B, N, H, H_kv, d, causal):
    q, k, v, do = bwd_inputs(B, N, H, H_kv, d, 31, O.F32)
    scale = 1.0 / np.sqrt(d)
    got = backward(emu, q, k, v, do, O.F32, B, N, H, H_kv, d, scale, causal)
    check_gradients(got, O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv), O.F32)


def test_backward_fp32_kernels_dense_mask(emu):
    B, N, H, d = 2, 37, 2, 64
    q, k, v, do = bwd_inputs(B, N, H, H, d, 32, O.F32)
    mask = (O.fill_uniform((B, N, N), 12, 6) > 0.3).astype(np.float32)
    mask[0, 5, :] = 0.0  # a row that sees nothing: no gradient flows through it
    got = backward(emu, q, k, v, do, O.F32, B, N, H, H, d, 0.125, False, mask=mask)
    assert not got[0][0, 5].any()
    check_gradients(got, O.attention_backward(q, k, v, do, B, N, H, d, 0.125, False, H, mask), O.F32)


@pytest.mark.parametrize("dtype", [O.F16, O.BF16])
def test_backward_fp32_kernels_16bit_storage(emu, dtype):
    B, N, H, H_kv, d = 1, 70, 4, 2, 32   # d = 32 is not taken by the matrix-core kernels
    q, k, v, do = bwd_inputs(B, N, H, H_kv, d, 33, dtype)
    got = backward(emu, q, k, v, do, dtype, B, N, H, H_kv, d, 0.2, True, front=True)
    check_gradients(got, O.attention_backward(q, k, v, do, B, N, H, d, 0.2, True, H_kv), dtype)


@pytest.mark.parametrize("split,dma_late", [(1, False), (2, True), (1, True)])
@pytest.mark.parametrize("dtype", [O.BF16, O.F16])
@pytest.mark.parametrize("B,N,H,H_kv,d,causal", [
    (1, 64, 1, 1, 128, False), (2, 129, 2, 2, 128, True), (1, 300, 2, 2, 64, True), (1, 200, 2, 1, 64, False),
    (1, 1, 2, 2, 128, True), (1, 260, 4, 2, 128, True), (1, 150, 2, 1, 256, True), (2, 70, 2, 2, 200, False)])
def test_backward_matrix_core_kernels(emu, tuned, dtype, B, N, H, H_kv, d, causal, dma_late, split):
    tuned("bwd_split", split)   # dK and dV in one walk over the query tiles (the default up to d = 128), or in two
    tuned("bwd_pair", split - 1)  # causal launches: one tile per workgroup (with one walk), a long and a short one (with two)
    q, k, v, do = bwd_inputs(B, N, H, H_kv, d, 34, dtype)
    scale = 1.0 / np.sqrt(d)
    S.configure(dma_late, seed=N + d)
    S.lds_stats(reset=True)
    try:
        got = backward(emu, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal, front=dma_late)
    finally:
        S.configure(False, 1)
    assert S.lds_stats(reset=True)[0] > 0   # the matrix-core kernels ran (the FMA kernels make no traced reads)
    check_gradients(got, O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv), dtype)


@pytest.mark.parametrize("split,dma_late", [(1, False), (2, True)])
@pytest.mark.parametrize("dtype,B,N,H,H_kv,d,causal", [
    (O.BF16, 2, 64, 2, 2, 128, False), (O.F16, 2, 131, 2, 1, 128, True), (O.F16, 1, 300, 2, 2, 64, False),
    (O.BF16, 2, 200, 4, 2, 64, True), (O.BF16, 1, 3, 2, 2, 128, False), (O.F16, 2, 65, 2, 2, 32, True),
    (O.BF16, 1, 140, 2, 1, 256, True), (O.F16, 1, 66, 2, 2, 192, False)])
def test_backward_matrix_core_kernels_dense_mask(emu, tuned, dtype, B, N, H, H_kv, d, causal, dma_late, split):
    """fp16/bf16 with a mask [B,N,N]: statistics, dQ, dK and dV on the matrix cores, on the packed copy of the mask in
    both of its layouts (keys per query for dQ, queries per key for dK and dV).  A query that sees nothing (no gradient
    reaches or leaves it), a key that nobody sees, queries that see one key, a last tile of 1 to 60 rows."""
    tuned("bwd_split", split)
    tuned("bwd_pair", split - 1)
    q, k, v, do = bwd_inputs(B, N, H, H_kv, d, 35, dtype)
    mask = (O.fill_uniform((B, N, N), 35, 6) > 0.4).astype(np.float32)
    mask[0, N // 2, :] = 0.0
    mask[0, :, N // 3] = 0.0
    mask[B - 1, N - 1, :] = 0.0
    mask[B - 1, N - 1, N - 1] = 1.0
    mask[B - 1, 0, :] = 0.0
    mask[B - 1, 0, 0] = 1.0
    scale = 1.0 / np.sqrt(d)
    S.configure(dma_late, seed=N + d)
    S.lds_stats(reset=True)
    try:
        got = backward(emu, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal, mask=mask, front=dma_late)
    finally:
        S.configure(False, 1)
    assert S.lds_stats(reset=True)[0] > 0   # the matrix-core kernels ran (the FMA kernels make no traced reads)
    assert not got[0][0, N // 2].any()
    assert not got[1][0, N // 3].any() and not got[2][0, N // 3].any()
    check_gradients(got, O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv, mask), dtype)


def forward_keep_backward_kept(emu, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal, mask=None, front=False, shift=0.0):
    """Forward that keeps its row statistics, then the backward that uses them: (output, kept statistics or None, gradients)."""
    dq_, dk_, dv_, ddo = dev(q, dtype, front), dev(k, dtype, front), dev(v, dtype, front), dev(do, dtype, front)
    o = S.guarded(S.empty_storage((B, N, H, d), dtype), front)
    dm = None if mask is None else S.guarded(mask, front)
    stats = S.guarded(np.full(emu.flash_row_stats_bytes(B, N, H) // 4, np.nan, np.float32), front)
    st, kst = (N * H * d, H * d, d), (N * H_kv * d, H_kv * d, d)
    written = emu.flash_fwd_keep(S.ptr(dq_), S.ptr(dk_), S.ptr(dv_), S.ptr(o), dtype, B, N, H, H_kv, d, st, kst, scale, causal,
                                 S.ptr(stats), None, None if dm is None else S.ptr(dm))
    gq = S.guarded(S.empty_storage((B, N, H, d), dtype), front)
    gk = S.guarded(S.empty_storage((B, N, H_kv, d), dtype), front)
    gv = S.guarded(S.empty_storage((B, N, H_kv, d), dtype), front)
    ws_bytes = emu.flash_bwd_workspace_bytes(B, N, H)
    ws = S.guarded(np.full(ws_bytes // 4, np.nan, np.float32), front)
    if shift:
        stats += np.float32(shift)
    emu.flash_bwd_kept(S.ptr(ddo), S.ptr(dq_), S.ptr(dk_), S.ptr(dv_), S.ptr(o) if written else None,
                       S.ptr(stats) if written else None, S.ptr(gq), S.ptr(gk), S.ptr(gv), dtype, B, N, H, H_kv, d, st, kst, scale,
                       causal, S.ptr(ws), ws_bytes, None, None if dm is None else S.ptr(dm))
    rows = (N + 127) // 128 * 128
    kept = np.array(stats).reshape(B, H, rows)[:, :, :N] if written else None
    return S.from_storage(o, dtype), kept, tuple(S.from_storage(x, dtype) for x in (gq, gk, gv))


def row_statistics(q, k, B, N, H, H_kv, d, scale, causal, mask=None):
    """-log2 of every query row's sum of exp2(scale * log2(e) * q.k) over its visible keys, in double precision."""
    g = H // H_kv
    out = np.empty((B, H, N))
    for b in range(B):
        for h in range(H):
            s = (q[b, :, h].astype(np.float64) @ k[b, :, h // g].astype(np.float64).T) * scale
            vis = np.ones((N, N), bool)
            if causal:
                vis &= np.tril(np.ones((N, N), bool))
            if mask is not None:
                vis &= mask[b] != 0
            with np.errstate(divide="ignore"):
                m = np.where(vis, s, -np.inf).max(axis=1, keepdims=True)
                m = np.where(np.isfinite(m), m, 0.0)
                out[b, h] = -(m[:, 0] + np.log(np.where(vis, np.exp(s - m), 0.0).sum(axis=1))) / np.log(2.0)
    return out


@pytest.mark.parametrize("rows", [128, 256])
@pytest.mark.parametrize("dtype,B,N,H,H_kv,d,causal,masked", [
    (O.BF16, 2, 300, 2, 2, 128, True, False), (O.F16, 1, 150, 4, 2, 64, False, False), (O.BF16, 1, 260, 2, 1, 128, False, True),
    (O.F16, 2, 70, 2, 2, 96, True, True), (O.BF16, 1, 140, 2, 2, 256, True, False)])
def test_backward_with_the_forward_s_kept_statistics(emu, tuned, rows, dtype, B, N, H, H_kv, d, causal, masked):
    """The forward keeps -log2 of every row's softmax sum (both forms of the kernel), the backward reads it and the
    forward's output instead of running its statistics pass: the kept values against a double-precision computation, the
    gradients against the oracle's, rows that see no key included."""
    tuned("flash_rows", rows)
    q, k, v, do = bwd_inputs(B, N, H, H_kv, d, 41, dtype)
    mask = None
    if masked:
        mask = (O.fill_uniform((B, N, N), 41, 6) > 0.4).astype(np.float32)
        mask[0, N // 2, :] = 0.0
    scale = 1.0 / np.sqrt(d)
    S.lds_stats(reset=True)
    out, kept, got = forward_keep_backward_kept(emu, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal, mask, front=rows == 256)
    assert S.lds_stats(reset=True)[0] > 0
    assert kept is not None
    want_stats = row_statistics(q, k, B, N, H, H_kv, d, scale, causal, mask)
    live = np.isfinite(want_stats)
    assert np.array_equal(np.isfinite(kept), live)
    assert np.abs(kept[live] - want_stats[live]).max() <= 2e-2   # (scores from 16-bit operands scaled before the product)
    rep = H // H_kv
    assert np.abs(out - O.attention(q, np.repeat(k, rep, axis=2), np.repeat(v, rep, axis=2), B, N, H, d, scale, causal, mask=mask)).max() <= TOL[dtype]
    check_gradients(got, O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv, mask), dtype)


def test_backward_really_reads_the_kept_statistics(emu):
    """Statistics shifted by one (every weight halved) halve dV: the backward used what it was given, not its own pass."""
    B, N, H, d = 1, 200, 2, 128
    q, k, v, do = bwd_inputs(B, N, H, H, d, 43, O.BF16)
    _, _, good = forward_keep_backward_kept(emu, q, k, v, do, O.BF16, B, N, H, H, d, 0.09, True)
    _, _, half = forward_keep_backward_kept(emu, q, k, v, do, O.BF16, B, N, H, H, d, 0.09, True, shift=-1.0)
    assert np.abs(half[2] - 0.5 * good[2]).max() <= 1e-2 * max(1.0, np.abs(good[2]).max())


def test_kept_statistics_are_not_written_by_kernels_that_keep_none(emu):
    """fp32 tensors run on kernels that keep nothing: the forward says so, and the backward without them is the plain one."""
    B, N, H, d = 1, 40, 2, 64
    q, k, v, do = bwd_inputs(B, N, H, H, d, 42, O.F32)
    out, kept, got = forward_keep_backward_kept(emu, q, k, v, do, O.F32, B, N, H, H, d, 0.125, True)
    assert kept is None
    assert np.abs(out - O.attention(q, k, v, B, N, H, d, 0.125, True)).max() <= 1e-4
    check_gradients(got, O.attention_backward(q, k, v, do, B, N, H, d, 0.125, True, H), O.F32)


def test_backward_dense_mask_without_the_packed_copy_takes_the_plain_kernels(emu, tuned):
    tuned("mask_pack", 0)
    B, N, H, d = 1, 70, 2, 64
    q, k, v, do = bwd_inputs(B, N, H, H, d, 36, O.BF16)
    mask = (O.fill_uniform((B, N, N), 36, 6) > 0.3).astype(np.float32)
    S.lds_stats(reset=True)
    got = backward(emu, q, k, v, do, O.BF16, B, N, H, H, d, 0.125, False, mask=mask)
    assert S.lds_stats(reset=True)[0] == 0
    check_gradients(got, O.attention_backward(q, k, v, do, B, N, H, d, 0.125, False, H, mask), O.BF16)


@pytest.mark.parametrize("dma_late", [False, True])
@pytest.mark.parametrize("B,N,H,H_kv,d,causal", [
    (1, 64, 1, 1, 128, False), (2, 129, 2, 2, 128, True), (1, 300, 2, 2, 64, True), (1, 200, 2, 1, 64, False),
    (1, 1, 2, 2, 128, True), (1, 260, 2, 1, 128, True), (1, 33, 2, 2, 64, True), (1, 31, 1, 1, 128, False)])
def test_backward_fp32_matrix_core_kernels(emu, tuned, B, N, H, H_kv, d, causal, dma_late):
    """fp32 tensors with d 64 or 128: statistics, dQ, and the dV and dK walks on the fp32 matrix instructions.  Causal launches
    with one tile per workgroup (tile requests on time) and with a long and a short one (requests late)."""
    tuned("bwd_pair", 1 if dma_late else 0)
    q, k, v, do = bwd_inputs(B, N, H, H_kv, d, 38, O.F32)
    scale = 1.0 / np.sqrt(d)
    S.configure(dma_late, seed=N + d)
    S.lds_stats(reset=True)
    try:
        got = backward(emu, q, k, v, do, O.F32, B, N, H, H_kv, d, scale, causal, front=dma_late)
    finally:
        S.configure(False, 1)
    check_gradients(got, O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv), O.F32)
    reads, read_conflicts, _, _ = S.lds_stats(reset=True)
    assert reads > 0 and read_conflicts == 0   # the matrix-core kernels ran (the FMA kernels make no traced reads)


@pytest.mark.parametrize("dtype,d", [(O.BF16, 32), (O.F16, 96), (O.BF16, 8), (O.F32, 32), (O.F32, 100), (O.F32, 4)])
@pytest.mark.parametrize("N,causal,H,H_kv,dma_late", [(150, True, 2, 1, True), (64, False, 2, 2, False)])
def test_backward_smaller_head_dimensions(emu, dtype, d, N, causal, H, H_kv, dma_late):
    """Head dimensions below the kernels' 64 / 128 in the backward: the matrix-core kernels with columns that contribute
    nothing, tensors at either end of guarded buffers."""
    B = 1
    q, k, v, do = bwd_inputs(B, N, H, H_kv, d, 39, dtype)
    scale = 1.0 / np.sqrt(d)
    S.configure(dma_late, seed=N + d)
    S.lds_stats(reset=True)
    try:
        got = backward(emu, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal, front=dma_late)
    finally:
        S.configure(False, 1)
    check_gradients(got, O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv), dtype)
    assert S.lds_stats(reset=True)[0] > 0   # the matrix-core kernels ran


# ---- LDS bank conflicts (model: 64 banks of 4 bytes) --------------------------------------------------------
@pytest.mark.parametrize("dtype,d", [(O.BF16, 128), (O.F16, 64), (O.BF16, 256)])
def test_operand_reads_are_free_of_bank_conflicts(emu, dtype, d):
    """Every 16-byte operand read and every transposing read of the matrix-core kernels, forward and backward.
    (The GPU's own conflict counter reads zero for the forward kernel, which is what anchors the model.)"""
    B, N, H = 1, 200, 2
    q, k, v, do = bwd_inputs(B, N, H, H, d, 36, dtype)
    S.lds_stats(reset=True)
    flash(emu, q, k, v, dtype, B, N, H, d, 0.1, True)
    reads, read_conflicts, tr, tr_conflicts = S.lds_stats(reset=True)
    assert reads > 0 and tr > 0 and read_conflicts == 0 and tr_conflicts == 0
    backward(emu, q, k, v, do, dtype, B, N, H, H, d, 0.1, True)
    reads, read_conflicts, tr, tr_conflicts = S.lds_stats(reset=True)
    assert reads > 0 and tr > 0 and read_conflicts == 0 and tr_conflicts == 0


# ---- grouped decode on the matrix cores --------------------------------------------------------------------
@pytest.mark.parametrize("dtype,d", [(O.F16, 128), (O.BF16, 64)])
@pytest.mark.parametrize("G", [4, 8, 16, 32])
def test_decode_grouped_heads_matrix_core_kernel(emu, G, dtype, d, tuned):
    tuned("decode_matrix_min_group", 4)   # groups of 4 and 8 take this kernel only when asked to
    tuned("decode_waves", 8)              # the widest workgroups (a launch this small would get single wavefronts)
    B, H_kv, P = 4, 2, 16
    H = G * H_kv
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, [70, 5, 129, 32], 23, dtype)
    lens = lens.copy()
    lens[3] = 0                                     # an empty sequence: zeros
    q = O.round_to(O.fill_normal((B, H, d), 23, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    # slots that hold no token of a sequence are NaN, table entries behind a last page point far outside the pool
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H_kv, d, wild_page=1 << 24)
    S.lds_stats(reset=True)
    for chunk, qo, dma_late in ((0, dtype, False), (48, O.F32, True), (16, dtype, False), (0, dtype, True)):
        S.configure(dma_late, seed=G + chunk)
        try:
            got = decode(emu, q, kp, vp, table, lens, None, B, H, H_kv, d, P, dtype, qo, scale, chunk)
        finally:
            S.configure(False, 1)
        assert np.all(got[3] == 0.0)
        assert np.abs(got - want).max() <= 2e-2, (chunk, qo)
    reads, read_conflicts, tr, tr_conflicts = S.lds_stats(reset=True)
    assert reads > 0 and tr > 0 and read_conflicts == 0 and tr_conflicts == 0


@pytest.mark.parametrize("H_kv,G,dtype", [(2, 4, O.F16), (8, 7, O.BF16), (5, 16, O.F16), (1, 32, O.BF16), (3, 20, O.F16)])
def test_decode_grouped_heads_matrix_core_kernels_head_dimension_256(emu, tuned, H_kv, G, dtype):
    """Both matrix-core decode kernels instantiated for d = 256 (the page-by-page one with at most four wavefronts in a
    workgroup: its page slots take twice the LDS), chunks of several trips round the page ring, loads landing late."""
    tuned("decode_matrix_min_group", 2)
    B, P, d = 4, 16, 256
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, [16 * 9 + 1, 5, 129, 32], 33, dtype)
    lens = lens.copy()
    lens[3] = 0
    H = G * H_kv
    q = O.round_to(O.fill_normal((B, H, d), 33, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H_kv, d, wild_page=1 << 24)
    S.lds_stats(reset=True)
    for chunk, dma_late in ((0, False), (48, True), (1024, True)):
        S.configure(dma_late, seed=G + chunk)
        try:
            got = decode(emu, q, kp, vp, table, lens, None, B, H, H_kv, d, P, dtype, dtype, scale, chunk)
        finally:
            S.configure(False, 1)
        assert np.all(got[3] == 0.0)
        assert np.abs(got - want).max() <= 2e-2, chunk
    reads, read_conflicts, tr, tr_conflicts = S.lds_stats(reset=True)
    assert reads > 0 and tr > 0   # a matrix-core kernel ran
    print(f"G={G}: operand reads {reads} (conflicts {read_conflicts}), transposing reads {tr} (conflicts {tr_conflicts})")


@pytest.mark.parametrize("H_kv,G,d,dtype", [(8, 4, 128, O.F16), (5, 2, 64, O.BF16), (1, 16, 128, O.BF16), (3, 8, 64, O.F16)])
def test_decode_page_ring_of_the_group_kernel(emu, tuned, H_kv, G, d, dtype):
    """The page-by-page matrix-core kernel with 8, 4, 2 and 1 pool heads side by side in a workgroup (5 heads leave
    wavefronts of the second workgroup without a head), chunks long enough for several trips round its ring of
    page slots and every remainder of pages (0 to 3) behind the last full trip, direct loads landing late."""
    tuned("decode_matrix_min_group", 2)
    B, P = 5, 16
    lens_in = [16 * 4 * 3, 16 * 9 + 1, 16 * 10 + 15, 16 * 7, 3]   # 12, 10, 11, 7 pages and a single short page
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, lens_in, 29, dtype)
    H = G * H_kv
    q = O.round_to(O.fill_normal((B, H, d), 29, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H_kv, d, wild_page=1 << 24)
    for chunk, dma_late in ((1024, True), (96, True), (0, False)):
        S.configure(dma_late, seed=H_kv + chunk)
        try:
            got = decode(emu, q, kp, vp, table, lens, None, B, H, H_kv, d, P, dtype, dtype, scale, chunk)
        finally:
            S.configure(False, 1)
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() <= 2e-2, chunk


@pytest.mark.parametrize("G,dtype,d,P,matrix_from", [
    (3, O.F32, 64, 16, 2), (5, O.F32, 128, 8, 2), (7, O.F16, 96, 16, 2), (6, O.BF16, 128, 16, 16), (3, O.F16, 64, 16, 16),  # lane per element
    (3, O.F16, 128, 16, 2), (7, O.BF16, 64, 16, 2), (12, O.F16, 128, 16, 2), (9, O.BF16, 64, 16, 16),                       # page by page
    (17, O.F16, 64, 16, 2), (24, O.BF16, 128, 16, 2), (31, O.F16, 128, 16, 16)])                                            # 32 columns
def test_decode_group_sizes_in_between(emu, tuned, G, dtype, d, P, matrix_from):
    """Group sizes the kernels are not instantiated for: the lane-per-element kernel of the next size with surplus query
    heads that hold zeros and store nothing, the matrix-core kernels with idle result columns.  The output sits
    directly against an inaccessible page, so a store for a head that does not exist faults."""
    tuned("decode_matrix_min_group", matrix_from)
    B, H_kv = 4, 3
    H = G * H_kv
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, [70, 5, 129, 32], 26, dtype)
    lens = lens.copy()
    lens[3] = 0                                     # an empty sequence: zeros
    q = O.round_to(O.fill_normal((B, H, d), 26, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H_kv, d, wild_page=1 << 24)
    for chunk in (0, 2 * P, 64 * P):
        got = decode(emu, q, kp, vp, table, lens, None, B, H, H_kv, d, P, dtype, dtype, scale, chunk)
        assert np.all(got[3] == 0.0)
        assert np.abs(got - want).max() <= TOL[dtype], chunk


@pytest.mark.parametrize("G,dtype,d,P", [(16, O.F32, 64, 16), (9, O.F16, 64, 8), (33, O.F16, 128, 16), (12, O.BF16, 96, 16), (20, O.F32, 128, 4),
                                        (71, O.BF16, 64, 16)])
def test_wide_groups_off_the_matrix_core_shape(emu, G, dtype, d, P):
    """More than 8 query heads per pool head where the matrix-core kernels do not apply (fp32 pool, other page sizes or
    head dimensions, more than 32 heads): the lane-per-element kernel serves the group in slices of 8 query heads."""
    B, H_kv = 3, 2
    H = G * H_kv
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, [70, 0, 33], 24, dtype)
    q = O.round_to(O.fill_normal((B, H, d), 24, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H_kv, d, wild_page=1 << 24)
    for chunk in (0, 2 * P):
        got = decode(emu, q, kp, vp, table, lens, None, B, H, H_kv, d, P, dtype, dtype, scale, chunk)
        assert np.all(got[1] == 0.0)
        assert np.abs(got - want).max() <= TOL[dtype], chunk


@pytest.mark.parametrize("dtype,d,H,H_kv,causal", [(O.F16, 64, 2, 2, False), (O.F16, 64, 2, 2, True), (O.BF16, 128, 4, 2, True),
                                                  (O.F32, 32, 2, 1, False), (O.F32, 128, 2, 1, True), (O.F32, 64, 2, 2, True)])
def test_backward_ragged_batch(emu, dtype, d, H, H_kv, causal):
    """Packed sequences of different lengths: every sequence's gradients equal the dense oracle's on that sequence."""
    lens = np.array([1, 130, 64, 257], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    q = O.round_to(O.fill_normal((T, H, d), 37, 1), dtype)
    k = O.round_to(O.fill_normal((T, H_kv, d), 37, 2), dtype)
    v = O.round_to(O.fill_normal((T, H_kv, d), 37, 3), dtype)
    do = O.round_to(O.fill_normal((T, H, d), 37, 7), dtype)
    tq, tk, tv, tdo = dev(q, dtype), dev(k, dtype), dev(v, dtype), dev(do, dtype)
    gq = S.guarded(S.empty_storage((T, H, d), dtype))
    gk = S.guarded(S.empty_storage((T, H_kv, d), dtype))
    gv = S.guarded(S.empty_storage((T, H_kv, d), dtype))
    dcu = S.guarded(cu)
    ws_bytes = emu.flash_bwd_workspace_bytes(len(lens), int(lens.max()), H)
    ws = S.guarded(np.full(ws_bytes // 4, np.nan, np.float32))
    scale = 1.0 / np.sqrt(d)
    emu.flash_bwd_varlen(S.ptr(tdo), S.ptr(tq), S.ptr(tk), S.ptr(tv), S.ptr(gq), S.ptr(gk), S.ptr(gv), dtype, S.ptr(dcu),
                         len(lens), int(lens.max()), H, H_kv, d, H * d, d, H_kv * d, d, scale, causal, S.ptr(ws), ws_bytes)
    got = tuple(S.from_storage(x, dtype) for x in (gq, gk, gv))
    for i, n in enumerate(lens):
        a, b = cu[i], cu[i + 1]
        want = O.attention_backward(q[a:b][None], k[a:b][None], v[a:b][None], do[a:b][None], 1, int(n), H, d, scale, causal, H_kv)
        check_gradients(tuple(g[a:b][None] for g in got), want, dtype)


# ---- decode without a workspace argument ----------------------------------------------------------------------
def decode_noalloc(emu, q, kp, vp, table, lens, B, H, H_kv, d, P, dtype, scale, chunk):
    dq = dev(q, dtype)
    do = S.guarded(S.empty_storage((B, H, d), dtype))
    dk, dv = dev(kp, dtype), dev(vp, dtype)
    dt, dl = S.guarded(table), S.guarded(np.asarray(lens, np.int32))
    emu.paged_decode_noalloc(S.ptr(dq), S.ptr(do), dtype, S.ptr(dk), S.ptr(dv), dtype, S.ptr(dt), S.ptr(dl), None, B, H, H_kv,
                             d, P, table.shape[1], int(max(1, np.max(lens))), scale, chunk)
    return S.from_storage(do, dtype)


def test_decode_with_built_in_scratch_equals_decode_with_workspace(emu):
    """Two calls in a row, the second smaller: the built-in array keeps the first call's partials."""
    for B, H, H_kv, d, lens, seed, dtype, chunk in ((4, 4, 4, 64, [150, 5, 33, 70], 71, O.F16, 32),
                                                    (2, 4, 4, 64, [40, 17], 72, O.F16, 32),
                                                    (3, 8, 2, 128, [90, 0, 20], 73, O.BF16, 16)):
        P = 16
        _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, lens, seed, dtype)
        q = O.round_to(O.fill_normal((B, H, d), seed, 1), dtype)
        a = decode(emu, q, kp, vp, table, lens, None, B, H, H_kv, d, P, dtype, dtype, 0.125, chunk)
        b = decode_noalloc(emu, q, kp, vp, table, lens, B, H, H_kv, d, P, dtype, 0.125, chunk)
        assert np.isfinite(b).all() and np.array_equal(a, b)


def test_decode_with_built_in_scratch_has_a_limit(emu):
    x = S.guarded(np.zeros(64, np.float32))
    p = S.ptr(x)
    with pytest.raises(emu.HipError) as e:
        emu.paged_decode_noalloc(p, p, O.F16, p, p, O.F16, p, p, None, 4096, 64, 64, 128, 16, 4096, 65536, 0.1, 16)
    assert "scratch" in str(e.value)
