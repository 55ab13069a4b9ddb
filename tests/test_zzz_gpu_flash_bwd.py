"""FlashAttention backward on the GPU (through the C ABI) against the CPU oracle's double-precision gradients.

Bars: fp32 tensors 1e-4 max-abs (relative to the largest entry when that exceeds 1); fp16/bf16 tensors 2e-2 of
the largest entry of the gradient (gradient entries are sums over up to N terms, so their size grows with
the problem, unlike the forward's convex combinations).  The reference has no working backward to compare with
(src/algorithms/flash_attention.cpp:496-580 is a placeholder): parity is to the oracle, which is pinned by
tests/test_oracle_backward.py."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def inputs(B, N, H, H_kv, d, seed, dtype):
    q = O.round_to(O.fill_normal((B, N, H, d), seed, 1), dtype)
    k = O.round_to(O.fill_normal((B, N, H_kv, d), seed, 2), dtype)
    v = O.round_to(O.fill_normal((B, N, H_kv, d), seed, 3), dtype)
    do = O.round_to(O.fill_normal((B, N, H, d), seed, 7), dtype)
    return q, k, v, do


def run_backward(hip, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal, mask=None):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr
    tq, tk, tv, tdo = (to_dev(x, dtype) for x in (q, k, v, do))
    gq, gk, gv = torch.full_like(tq, float("nan")), torch.full_like(tk, float("nan")), torch.full_like(tv, float("nan"))
    tm = None if mask is None else torch.from_numpy(mask).cuda()
    ws_bytes = hip.flash_bwd_workspace_bytes(B, N, H)
    ws = torch.full((ws_bytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
    hip.flash_bwd(tdo.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), gq.data_ptr(), gk.data_ptr(), gv.data_ptr(),
                  dtype, B, N, H, H_kv, d, (N * H * d, H * d, d), (N * H_kv * d, H_kv * d, d), scale, causal, ws.data_ptr(),
                  ws_bytes, stream_ptr(), None if tm is None else tm.data_ptr())
    torch.cuda.synchronize()
    return to_host(gq), to_host(gk), to_host(gv)


def check(got, want, dtype):
    for name, g, w in zip(("dQ", "dK", "dV"), got, want):
        assert np.isfinite(g).all(), name
        bar = (1e-4 if dtype == O.F32 else 2e-2) * max(1.0, np.abs(w).max())
        assert np.abs(g - w).max() <= bar, (name, float(np.abs(g - w).max()), bar)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,N,H,H_kv,d", [(2, 16, 4, 4, 64), (1, 150, 2, 1, 32), (1, 40, 3, 3, 80), (1, 1, 2, 2, 128), (1, 300, 2, 2, 128)])
def test_fp32_tensors(gpu, B, N, H, H_kv, d, causal):
    # the first shape is the fixture of tests/test_flash_attention.cpp:103-108, whose backward test (:405-480)
    # only asks for non-zero gradients
    q, k, v, do = inputs(B, N, H, H_kv, d, 31, O.F32)
    scale = 1.0 / np.sqrt(d)
    got = run_backward(gpu, q, k, v, do, O.F32, B, N, H, H_kv, d, scale, causal)
    assert all(np.abs(g).max() > 1e-6 for g in got) or N == 1
    check(got, O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv), O.F32)


@pytest.mark.parametrize("dtype,d", [(O.BF16, 32), (O.F16, 96), (O.BF16, 8), (O.F16, 120), (O.F32, 100), (O.F32, 4), (O.F32, 72)])
@pytest.mark.parametrize("N,causal,H,H_kv", [(150, True, 2, 1), (64, False, 3, 3), (517, True, 4, 2)])
def test_smaller_head_dimensions_on_the_matrix_cores(gpu, dtype, d, N, causal, H, H_kv):
    """Head dimensions below 64 / 128 (multiples of 8 for 16-bit tensors, of 4 for fp32): the matrix-core kernels with
    columns that contribute nothing; gradients are pre-filled with NaN, every element must have been written."""
    B = 2
    q, k, v, do = inputs(B, N, H, H_kv, d, 33, dtype)
    scale = 1.0 / np.sqrt(d)
    got = run_backward(gpu, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal)
    check(got, O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv), dtype)


def test_dense_mask(gpu):
    B, N, H, d = 2, 37, 2, 64
    q, k, v, do = inputs(B, N, H, H, d, 32, O.F32)
    mask = (O.fill_uniform((B, N, N), 12, 6) > 0.3).astype(np.float32)
    mask[0, 5, :] = 0.0
    got = run_backward(gpu, q, k, v, do, O.F32, B, N, H, H, d, 0.125, False, mask=mask)
    assert not got[0][0, 5].any()
    check(got, O.attention_backward(q, k, v, do, B, N, H, d, 0.125, False, H, mask), O.F32)


@pytest.mark.parametrize("dtype", [O.F16, O.BF16])
@pytest.mark.parametrize("B,N,H,H_kv,d,causal", [
    (1, 64, 1, 1, 128, False), (2, 129, 2, 2, 128, True), (1, 300, 2, 2, 64, True), (1, 200, 2, 1, 64, False),
    (1, 1, 2, 2, 128, True), (1, 260, 4, 2, 128, True), (2, 1024, 4, 4, 128, True), (1, 517, 3, 3, 64, False),
    (1, 70, 4, 2, 32, True), (1, 300, 2, 1, 256, True), (2, 517, 2, 2, 200, False), (1, 1024, 4, 4, 256, True)])
def test_16bit_tensors(gpu, dtype, B, N, H, H_kv, d, causal):
    # matrix-core kernels for 64, 128 and 256 (smaller head dimensions run on the next one)
    q, k, v, do = inputs(B, N, H, H_kv, d, 34, dtype)
    scale = 1.0 / np.sqrt(d)
    got = run_backward(gpu, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal)
    check(got, O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv), dtype)


@pytest.mark.parametrize("dtype,B,N,H,H_kv,d,causal", [
    (O.BF16, 2, 64, 2, 2, 128, False), (O.F16, 2, 131, 2, 1, 128, True), (O.F16, 1, 300, 2, 2, 64, False),
    (O.BF16, 2, 517, 4, 2, 64, True), (O.BF16, 1, 3, 2, 2, 128, False), (O.F16, 2, 65, 2, 2, 32, True),
    (O.BF16, 1, 1030, 2, 2, 128, False), (O.F16, 1, 300, 2, 1, 256, True), (O.BF16, 2, 130, 2, 2, 192, False)])
def test_16bit_tensors_dense_mask(gpu, dtype, B, N, H, H_kv, d, causal):
    """fp16/bf16 with a mask [B,N,N]: the matrix-core kernels on the packed copy of the mask.  A query that sees nothing,
    a key that nobody sees, queries that see one key."""
    q, k, v, do = inputs(B, N, H, H_kv, d, 36, dtype)
    mask = (O.fill_uniform((B, N, N), 36, 6) > 0.4).astype(np.float32)
    mask[0, N // 2, :] = 0.0
    mask[0, :, N // 3] = 0.0
    mask[B - 1, N - 1, :] = 0.0
    mask[B - 1, N - 1, N - 1] = 1.0
    mask[B - 1, 0, :] = 0.0
    mask[B - 1, 0, 0] = 1.0
    scale = 1.0 / np.sqrt(d)
    got = run_backward(gpu, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal, mask=mask)
    assert not got[0][0, N // 2].any()
    assert not got[1][0, N // 3].any() and not got[2][0, N // 3].any()
    check(got, O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv, mask), dtype)


def test_16bit_dense_mask_runs_at_matrix_core_speed(gpu):
    """B=1, N=2048, H=8, d=128, bf16 with a mask: within 4x of the same launch without a mask (the plain kernels this
    case used to take were some 50 times slower), and equal to it where the mask hides nothing."""
    import torch
    from gpu_util import stream_ptr
    B, N, H, d = 1, 2048, 8, 128
    g = torch.Generator(device="cuda").manual_seed(0xA77E0007)
    tq, tk, tv, tdo = (torch.randn((B, N, H, d), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
                       for _ in range(4))
    ones = torch.ones((B, N, N), dtype=torch.float32, device="cuda")
    ws_bytes = gpu.flash_bwd_workspace_bytes(B, N, H)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device="cuda")
    scale = 1.0 / np.sqrt(d)

    def run(mask):
        out = tuple(torch.full_like(tq, float("nan")) for _ in range(3))
        def call():
            gpu.flash_bwd(tdo.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), *(t.data_ptr() for t in out), O.BF16,
                          B, N, H, H, d, (N * H * d, H * d, d), (N * H * d, H * d, d), scale, False, ws.data_ptr(), ws_bytes,
                          stream_ptr(), None if mask is None else mask.data_ptr())
        for _ in range(3):
            call()
        torch.cuda.synchronize()
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        for _ in range(10):
            call()
        t1.record()
        torch.cuda.synchronize()
        return out, t0.elapsed_time(t1) / 10

    plain, ms_plain = run(None)
    masked, ms_masked = run(ones)
    print(f"backward B=1 N=2048 H=8 d=128 bf16: {ms_plain:.3f} ms without a mask, {ms_masked:.3f} ms with one")
    for a, b in zip(plain, masked):
        assert (a.float() - b.float()).abs().max().item() <= 1e-2 * max(1.0, a.float().abs().max().item())
    assert ms_masked <= 4 * ms_plain


def run_kept(hip, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal, mask=None):
    """Forward that keeps its row statistics, backward that uses them: (output, statistics were kept, gradients)."""
    import torch
    from gpu_util import to_dev, to_host, stream_ptr
    tq, tk, tv, tdo = (to_dev(x, dtype) for x in (q, k, v, do))
    to = torch.full_like(tq, float("nan"))
    gq, gk, gv = torch.full_like(tq, float("nan")), torch.full_like(tk, float("nan")), torch.full_like(tv, float("nan"))
    tm = None if mask is None else torch.from_numpy(mask).cuda()
    stats = torch.full((hip.flash_row_stats_bytes(B, N, H) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    ws_bytes = hip.flash_bwd_workspace_bytes(B, N, H)
    ws = torch.full((ws_bytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
    st, kst = (N * H * d, H * d, d), (N * H_kv * d, H_kv * d, d)
    mp = None if tm is None else tm.data_ptr()
    kept = hip.flash_fwd_keep(tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), to.data_ptr(), dtype, B, N, H, H_kv, d, st, kst, scale,
                              causal, stats.data_ptr(), stream_ptr(), mp)
    hip.flash_bwd_kept(tdo.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), to.data_ptr() if kept else None,
                       stats.data_ptr() if kept else None, gq.data_ptr(), gk.data_ptr(), gv.data_ptr(), dtype, B, N, H, H_kv, d, st,
                       kst, scale, causal, ws.data_ptr(), ws_bytes, stream_ptr(), mp)
    torch.cuda.synchronize()
    return to_host(to), kept, (to_host(gq), to_host(gk), to_host(gv))


@pytest.mark.parametrize("dtype,B,N,H,H_kv,d,causal,masked", [
    (O.BF16, 2, 300, 2, 2, 128, True, False), (O.F16, 1, 150, 4, 2, 64, False, False), (O.BF16, 1, 260, 2, 1, 128, False, True),
    (O.F16, 2, 70, 2, 2, 96, True, True), (O.BF16, 1, 140, 2, 2, 256, True, False), (O.BF16, 2, 2048, 8, 8, 128, True, False),
    (O.F16, 1, 2304, 16, 4, 128, False, False), (O.F32, 1, 40, 2, 2, 64, True, False)])
def test_backward_with_the_forward_s_kept_statistics(gpu, dtype, B, N, H, H_kv, d, causal, masked):
    """ahpc_hip_flash_fwd_keep + ahpc_hip_flash_bwd_kept: output and gradients against the oracle (the 2048- and 2304-token
    cases take the 256-row forward); fp32 tensors keep nothing and fall back to the plain backward."""
    from gpu_util import TOL
    q, k, v, do = inputs(B, N, H, H_kv, d, 44, dtype)
    mask = None
    if masked:
        mask = (O.fill_uniform((B, N, N), 44, 6) > 0.4).astype(np.float32)
        mask[0, N // 2, :] = 0.0
    scale = 1.0 / np.sqrt(d)
    out, kept, got = run_kept(gpu, q, k, v, do, dtype, B, N, H, H_kv, d, scale, causal, mask)
    assert kept == (dtype != O.F32)
    rep = H // H_kv
    want = O.attention(q, np.repeat(k, rep, axis=2), np.repeat(v, rep, axis=2), B, N, H, d, scale, causal, mask=mask)
    assert np.abs(out - want).max() <= TOL[dtype]
    check(got, O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv, mask), dtype)


def test_kept_statistics_headline_shape_timing(gpu):
    """B=4 N=4096 H=32 d=128 bf16 causal: the backward on kept statistics agrees with the plain one and is faster."""
    import torch
    from gpu_util import stream_ptr
    B, N, H, d = 4, 4096, 32, 128
    g = torch.Generator(device="cuda").manual_seed(0xA77E000A)
    tq, tk, tv, tdo = (torch.randn((B, N, H, d), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
                       for _ in range(4))
    to = torch.empty_like(tq)
    stats = torch.empty(gpu.flash_row_stats_bytes(B, N, H) // 4, dtype=torch.float32, device="cuda")
    ws_bytes = gpu.flash_bwd_workspace_bytes(B, N, H)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device="cuda")
    st = (N * H * d, H * d, d)
    scale = 1.0 / np.sqrt(d)
    assert gpu.flash_fwd_keep(tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), to.data_ptr(), O.BF16, B, N, H, H, d, st, st, scale, True,
                              stats.data_ptr(), stream_ptr())

    def run(kept):
        out = tuple(torch.full_like(tq, float("nan")) for _ in range(3))
        def call():
            gpu.flash_bwd_kept(tdo.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), to.data_ptr() if kept else None,
                               stats.data_ptr() if kept else None, *(t.data_ptr() for t in out), O.BF16, B, N, H, H, d, st, st,
                               scale, True, ws.data_ptr(), ws_bytes, stream_ptr())
        for _ in range(5):
            call()
        torch.cuda.synchronize()
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        for _ in range(10):
            call()
        t1.record()
        torch.cuda.synchronize()
        return out, t0.elapsed_time(t1) / 10

    plain, ms_plain = run(False)
    kept, ms_kept = run(True)
    print(f"backward B=4 N=4096 H=32 d=128 bf16 causal: {ms_plain:.3f} ms recomputing the statistics, {ms_kept:.3f} ms on kept ones")
    for a, b in zip(plain, kept):
        assert (a.float() - b.float()).abs().max().item() <= 2e-2 * max(1.0, a.float().abs().max().item())
    assert ms_kept < ms_plain


def test_closed_forms_16bit(gpu):
    B, N, H, d = 1, 256, 2, 128
    q, k, v, do = inputs(B, N, H, H, d, 35, O.BF16)
    # V with equal rows => dP is constant along a row => dS = 0 => dQ = dK = 0
    vc = np.repeat(v[:, :1], N, axis=1)
    gq, gk, gv = run_backward(gpu, q, k, vc, do, O.BF16, B, N, H, H, d, 0.1, True)
    assert np.abs(gq).max() <= 2e-2 and np.abs(gk).max() <= 2e-2
    # K with equal rows => uniform weights: dQ = 0 and (no mask) dV_j = mean_i dO_i
    kc = np.repeat(k[:, :1], N, axis=1)
    gq, gk, gv = run_backward(gpu, q, kc, v, do, O.BF16, B, N, H, H, d, 0.1, False)
    assert np.abs(gq).max() <= 2e-2
    assert np.abs(gv - do.mean(axis=1, keepdims=True)).max() <= 2e-2


def test_headline_shape_bf16_causal(gpu):
    """B=4, N=4096, H=32, d=128, causal, bf16: properties that hold at any size over the whole result, and one
    (sequence, head) against the oracle."""
    import torch
    from gpu_util import stream_ptr
    B, N, H, d = 4, 4096, 32, 128
    g = torch.Generator(device="cuda").manual_seed(0xA77E0006)
    tq, tk, tv, tdo = (torch.randn((B, N, H, d), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
                       for _ in range(4))
    gq, gk, gv = (torch.full_like(tq, float("nan")) for _ in range(3))
    ws_bytes = gpu.flash_bwd_workspace_bytes(B, N, H)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device="cuda")
    scale = 1.0 / np.sqrt(d)
    gpu.flash_bwd(tdo.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), gq.data_ptr(), gk.data_ptr(), gv.data_ptr(),
                  O.BF16, B, N, H, H, d, (N * H * d, H * d, d), (N * H * d, H * d, d), scale, True, ws.data_ptr(), ws_bytes,
                  stream_ptr())
    torch.cuda.synchronize()
    for t in (gq, gk, gv):
        assert torch.isfinite(t.float()).all()
    # the weights of a query row sum to one: sum_j dV_j = sum_i dO_i per (sequence, head)
    lhs, rhs = gv.double().sum(dim=1), tdo.double().sum(dim=1)
    assert (lhs - rhs).abs().max().item() <= 2e-2 * max(1.0, rhs.abs().max().item())
    # sum_i q_i.dQ_i = sum_j k_j.dK_j (both are scale * sum_ij dS_ij q_i.k_j)
    a = (tq.double() * gq.double()).sum(dim=(1, 3))
    b = (tk.double() * gk.double()).sum(dim=(1, 3))
    assert (a - b).abs().max().item() <= 2e-2 * max(1.0, a.abs().max().item(), b.abs().max().item())
    # the last key is seen by the last query only: dV_last = P_last,last * dO_last, a multiple of dO_last
    # one (sequence, head) against the oracle
    bi, hi = 2, 17
    sl = lambda t: t[bi:bi + 1, :, hi:hi + 1].float().cpu().numpy()
    want = O.attention_backward(sl(tq), sl(tk), sl(tv), sl(tdo), 1, N, 1, d, scale, True)
    for name, got, w in zip(("dQ", "dK", "dV"), (sl(gq), sl(gk), sl(gv)), want):
        assert np.abs(got - w).max() <= 2e-2 * max(1.0, np.abs(w).max()), name


def test_bad_arguments_are_rejected_without_launch(gpu):
    import torch
    x = torch.zeros(1 << 16, device="cuda")
    p = x.data_ptr()
    ok = dict(dtype=O.F32, B=1, N=16, H=2, H_kv=2, d=64, strides=(2048, 128, 64), kv_strides=(2048, 128, 64), scale=0.1,
              causal=False, workspace=p, workspace_bytes=1 << 16)
    call = lambda **kw: gpu.flash_bwd(p, p, p, p, p, p, p, **{**ok, **kw})
    with pytest.raises(gpu.HipError):
        call(H_kv=3)
    with pytest.raises(gpu.HipError):
        call(d=300)
    with pytest.raises(gpu.HipError):
        call(workspace_bytes=16)
    with pytest.raises(gpu.HipError):
        call(workspace=None)
    with pytest.raises(gpu.HipError):
        gpu.flash_bwd(p, p, p, p, 0, p, p, **ok)
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype,d,H,H_kv", [(O.F16, 64, 4, 4), (O.BF16, 128, 4, 2), (O.F32, 32, 2, 1), (O.BF16, 256, 2, 1)])
@pytest.mark.parametrize("causal", [False, True])
def test_ragged_batch(gpu, dtype, d, H, H_kv, causal):
    """Packed sequences of different lengths: every sequence's gradients equal the dense oracle's on that sequence."""
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32
    lens = np.array([5, 130, 1, 64, 257, 128], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    q = O.round_to(O.fill_normal((T, H, d), 37, 1), dtype)
    k = O.round_to(O.fill_normal((T, H_kv, d), 37, 2), dtype)
    v = O.round_to(O.fill_normal((T, H_kv, d), 37, 3), dtype)
    do = O.round_to(O.fill_normal((T, H, d), 37, 7), dtype)
    tq, tk, tv, tdo = (to_dev(x, dtype) for x in (q, k, v, do))
    gq, gk, gv = torch.full_like(tq, float("nan")), torch.full_like(tk, float("nan")), torch.full_like(tv, float("nan"))
    dcu = dev_i32(cu)
    ws_bytes = gpu.flash_bwd_workspace_bytes(len(lens), int(lens.max()), H)
    ws = torch.full((ws_bytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
    scale = 1.0 / np.sqrt(d)
    gpu.flash_bwd_varlen(tdo.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), gq.data_ptr(), gk.data_ptr(),
                         gv.data_ptr(), dtype, dcu.data_ptr(), len(lens), int(lens.max()), H, H_kv, d, H * d, d, H_kv * d, d,
                         scale, causal, ws.data_ptr(), ws_bytes, stream_ptr())
    torch.cuda.synchronize()
    got = (to_host(gq), to_host(gk), to_host(gv))
    for i, n in enumerate(lens):
        a, b = cu[i], cu[i + 1]
        want = O.attention_backward(q[a:b][None], k[a:b][None], v[a:b][None], do[a:b][None], 1, int(n), H, d, scale, causal, H_kv)
        check(tuple(g[a:b][None] for g in got), want, dtype)


def test_golden_backward_vectors(gpu):
    """tests/golden/*.npz: gradients from a float64 computation that shares no code with the oracle."""
    import os
    from test_golden_vectors import FILES, load, dense_inputs
    for path in FILES:
        c = load(path)
        if "dq" not in c:
            continue
        (B, N, H, Hkv, d), q, k, v, do, mask = dense_inputs(c)
        got = run_backward(gpu, q, k, v, do, O.F32, B, N, H, Hkv, d, float(c["scale"]), bool(c["causal"]), mask)
        for g, name in zip(got, ("dq", "dk", "dv")):
            assert np.abs(g - c[name]).max() <= 1e-4, (os.path.basename(path), name)
