"""Seeded sweeps over shapes nobody picked by hand: forward (dense, grouped heads, dense mask, ragged batches), backward and
paged decode on the GPU through the C ABI against the CPU oracle, bars as everywhere (fp32 1e-4, 16-bit 2e-2; gradients
relative to the gradient's largest entry).  The shapes come from numpy's PCG64 with fixed seeds, so a failure names a
reproducible case; sizes stay small enough for the oracle to finish the whole file in seconds.

What the hand-picked cases do not reach and these do: sequence lengths around every tile edge at once (1, 31..33, 63..65,
127..129, 255..257), head counts that do not divide the XCD count, odd batch sizes, empty sequences inside a ragged batch,
contexts that end on a page edge, chunk sizes that do not divide the context, every legal group size on both decode kernels."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

EDGE_LENGTHS = [1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 95, 127, 128, 129, 191, 255, 256, 257, 300, 511, 513]


def expand_heads(x, g, axis):
    return np.ascontiguousarray(np.repeat(x, g, axis=axis))


def pick(rng, xs):
    return xs[int(rng.integers(len(xs)))]


def forward_cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        dtype = pick(rng, [O.F32, O.F16, O.BF16])
        d = pick(rng, [64, 128] if dtype != O.F32 else [16, 32, 64, 128])
        Hkv = int(rng.integers(1, 4))
        g = pick(rng, [1, 1, 2, 3, 4])
        N = pick(rng, EDGE_LENGTHS) if rng.random() < 0.7 else int(rng.integers(1, 600))
        B = int(rng.integers(1, 4))
        causal = bool(rng.integers(2))
        masked = rng.random() < 0.3
        if masked and rng.random() < 0.7:
            N = (N + 3) // 4 * 4  # the matrix-core mask path wants rows of whole 16-byte pieces; others take the fp32 kernel
        out.append(pytest.param(dtype, B, N, Hkv * g, Hkv, d, causal, masked, 1000 + i,
                                id=f"{i}-{['f32', 'f16', 'bf16'][dtype]}-B{B}-N{N}-H{Hkv * g}over{Hkv}-d{d}-{'c' if causal else 'f'}{'-mask' if masked else ''}"))
    return out


@pytest.mark.parametrize("dtype,B,N,H,Hkv,d,causal,masked,seed", forward_cases(96, 20261))
def test_forward_random_shapes(gpu, dtype, B, N, H, Hkv, d, causal, masked, seed):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, TOL
    g = H // Hkv
    q = O.round_to(O.fill_normal((B, N, H, d), seed, 1), dtype)
    k = O.round_to(O.fill_normal((B, N, Hkv, d), seed, 2), dtype)
    v = O.round_to(O.fill_normal((B, N, Hkv, d), seed, 3), dtype)
    mask = None
    if masked:
        mask = (O.fill_uniform((B, N, N), seed, 9) > -0.2).astype(np.float32)
        mask[:, np.arange(N), np.arange(N)] = 1.0  # every query keeps its own key: no empty rows
    scale = 1.0 / np.sqrt(d)
    want = O.attention(q, expand_heads(k, g, 2), expand_heads(v, g, 2), B, N, H, d, scale, causal, mask=mask)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    dm = None if mask is None else torch.from_numpy(mask).cuda()
    do = torch.full_like(dq, float("nan"))
    gpu.flash_fwd_gqa(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), dtype, B, N, H, Hkv, d,
                      (N * H * d, H * d, d), (N * Hkv * d, Hkv * d, d), scale, causal, stream_ptr(),
                      None if dm is None else dm.data_ptr())
    torch.cuda.synchronize()
    got = to_host(do)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL[dtype]


def varlen_cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        dtype = pick(rng, [O.F16, O.BF16, O.F32])
        d = pick(rng, [64, 128])
        Hkv = int(rng.integers(1, 3))
        g = pick(rng, [1, 2, 4])
        n_seqs = int(rng.integers(1, 7))
        lens = [pick(rng, [0] + EDGE_LENGTHS[:18]) if rng.random() < 0.8 else int(rng.integers(0, 400)) for _ in range(n_seqs)]
        if sum(lens) == 0:
            lens[0] = 5
        out.append(pytest.param(dtype, lens, Hkv * g, Hkv, d, bool(rng.integers(2)), 2000 + i,
                                id=f"{i}-{['f32', 'f16', 'bf16'][dtype]}-lens{'_'.join(map(str, lens))}-H{Hkv * g}over{Hkv}-d{d}"))
    return out


@pytest.mark.parametrize("dtype,lens,H,Hkv,d,causal,seed", varlen_cases(48, 20262))
def test_ragged_forward_random_batches(gpu, dtype, lens, H, Hkv, d, causal, seed):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32, TOL
    g = H // Hkv
    lens = np.asarray(lens, np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    q = O.round_to(O.fill_normal((T, H, d), seed, 1, 0.7), dtype)
    k = O.round_to(O.fill_normal((T, Hkv, d), seed, 2, 0.7), dtype)
    v = O.round_to(O.fill_normal((T, Hkv, d), seed, 3, 0.7), dtype)
    scale = 1.0 / np.sqrt(d)
    want = O.attention_varlen(q, expand_heads(k, g, 1), expand_heads(v, g, 1), cu, H, d, scale, causal)
    dq, dk, dv, dcu = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), dev_i32(cu)
    do = torch.full_like(dq, float("nan"))
    gpu.flash_fwd_varlen_gqa(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), dtype, dcu.data_ptr(), len(lens),
                             int(lens.max()), H, Hkv, d, H * d, d, Hkv * d, d, scale, causal, stream_ptr())
    torch.cuda.synchronize()
    got = to_host(do)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL[dtype]


def backward_cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        dtype = pick(rng, [O.F32, O.F16, O.BF16])
        d = pick(rng, [64, 128] if dtype != O.F32 else [32, 64, 128])
        Hkv = int(rng.integers(1, 3))
        g = pick(rng, [1, 2, 4])
        N = pick(rng, EDGE_LENGTHS[:20])
        B = int(rng.integers(1, 3))
        split = int(rng.integers(0, 3))
        out.append(pytest.param(dtype, B, N, Hkv * g, Hkv, d, bool(rng.integers(2)), split, 3000 + i,
                                id=f"{i}-{['f32', 'f16', 'bf16'][dtype]}-B{B}-N{N}-H{Hkv * g}over{Hkv}-d{d}-split{split}"))
    return out


@pytest.mark.parametrize("dtype,B,N,H,Hkv,d,causal,split,seed", backward_cases(48, 20263))
def test_backward_random_shapes(gpu, dtype, B, N, H, Hkv, d, causal, split, seed):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr
    q = O.round_to(O.fill_normal((B, N, H, d), seed, 1, 0.8), dtype)
    k = O.round_to(O.fill_normal((B, N, Hkv, d), seed, 2, 0.8), dtype)
    v = O.round_to(O.fill_normal((B, N, Hkv, d), seed, 3, 0.8), dtype)
    go = O.round_to(O.fill_normal((B, N, H, d), seed, 4, 0.8), dtype)
    scale = 1.0 / np.sqrt(d)
    want = O.attention_backward(q, k, v, go, B, N, H, d, scale, causal, H_kv=Hkv)
    dq, dk, dv, dgo = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), to_dev(go, dtype)
    gq, gk, gv = (torch.full_like(t, float("nan")) for t in (dq, dk, dv))
    wsb = gpu.flash_bwd_workspace_bytes(B, N, H)
    ws = torch.empty(max(wsb, 4) // 4, dtype=torch.float32, device="cuda")
    before = gpu.get_tuning("bwd_split")
    before_pair = gpu.get_tuning("bwd_pair")
    gpu.set_tuning("bwd_split", split)
    gpu.set_tuning("bwd_pair", seed % 2)   # causal launches: one tile per workgroup, or a long and a short one
    try:
        gpu.flash_bwd(dgo.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), gq.data_ptr(), gk.data_ptr(), gv.data_ptr(),
                      dtype, B, N, H, Hkv, d, (N * H * d, H * d, d), (N * Hkv * d, Hkv * d, d), scale, causal,
                      ws.data_ptr(), wsb, stream_ptr())
        torch.cuda.synchronize()
    finally:
        gpu.set_tuning("bwd_split", before)
        gpu.set_tuning("bwd_pair", before_pair)
    bar = 1e-4 if dtype == O.F32 else 2e-2
    for name, got, ref in zip(("dq", "dk", "dv"), (gq, gk, gv), want):
        got = to_host(got)
        assert np.isfinite(got).all(), name
        assert np.abs(got - ref).max() <= bar * max(1.0, np.abs(ref).max()), name


def decode_cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        dtype = pick(rng, [O.F32, O.F16, O.BF16])
        d = pick(rng, [64, 128]) if rng.random() < 0.8 else pick(rng, [32, 256])
        P = 16 if rng.random() < 0.75 else pick(rng, [4, 8, 32])
        Hkv = int(rng.integers(1, 4))
        g = pick(rng, list(range(1, 33)) + [40, 71]) if rng.random() < 0.85 else 1
        B = int(rng.integers(1, 6))
        lens = []
        for _ in range(B):
            r = rng.random()
            lens.append(0 if r < 0.08 else pick(rng, [1, P - 1, P, P + 1, 2 * P, 8 * P, 8 * P + 1, 16 * P, 17 * P - 1]) if r < 0.6
                        else int(rng.integers(1, 1500)))
        if max(lens) == 0:
            lens[0] = 3
        chunk = pick(rng, [0, 0, 2 * P, 6 * P, 128, 256, 1024])
        chunk = chunk // P * P
        waves = pick(rng, [0, 0, 1, 2, 4, 8])
        matrix_from = pick(rng, [2, 16])
        out.append(pytest.param(dtype, B, lens, Hkv * g, Hkv, d, P, chunk, waves, matrix_from, 4000 + i,
                                id=f"{i}-{['f32', 'f16', 'bf16'][dtype]}-H{Hkv * g}over{Hkv}-d{d}-P{P}-c{chunk}-w{waves}-m{matrix_from}-L{'_'.join(map(str, lens))}"))
    return out


@pytest.mark.parametrize("dtype,B,lens,H,Hkv,d,P,chunk,waves,matrix_from,seed", decode_cases(128, 20264))
def test_decode_random_shapes(gpu, dtype, B, lens, H, Hkv, d, P, chunk, waves, matrix_from, seed):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32, TOL
    from test_gpu_gqa import build_pool
    from test_gpu_paged import poison_unused
    g = H // Hkv
    kp, vp, table, lens, n_pages = build_pool(B, Hkv, d, P, lens, seed, dtype)
    q = O.round_to(O.fill_normal((B, H, d), seed, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    kx = expand_heads(kp.reshape(n_pages * P, Hkv, d), g, 1).reshape(-1)
    vx = expand_heads(vp.reshape(n_pages * P, Hkv, d), g, 1).reshape(-1)
    want = O.paged_decode(q, kx, vx, table, lens, None, B, H, d, P, scale)
    # what no sequence owns is NaN on the device
    kp_n, vp_n, table_n = poison_unused(kp, vp, table, lens, P, Hkv, d, wild_page=None)
    kd, vd, dt, dl = to_dev(kp_n, dtype), to_dev(vp_n, dtype), dev_i32(table_n), dev_i32(lens)
    dq = to_dev(q, dtype)
    do = torch.full_like(dq, float("nan"))
    max_len = int(lens.max())
    ws_bytes = gpu.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
    ws = torch.empty(max(ws_bytes, 4) // 4, dtype=torch.float32, device="cuda")
    saved = {name: gpu.get_tuning(name) for name in ("decode_waves", "decode_matrix_min_group")}
    gpu.set_tuning("decode_waves", waves)
    gpu.set_tuning("decode_matrix_min_group", matrix_from)
    try:
        gpu.paged_decode_gqa(dq.data_ptr(), do.data_ptr(), dtype, kd.data_ptr(), vd.data_ptr(), dtype, dt.data_ptr(),
                             dl.data_ptr(), None, B, H, Hkv, d, P, table.shape[1], max_len, scale, chunk, ws.data_ptr(),
                             ws_bytes, stream_ptr())
        torch.cuda.synchronize()
    finally:
        for name, value in saved.items():
            gpu.set_tuning(name, value)
    got = to_host(do)
    live = lens > 0
    assert np.isfinite(got[live]).all()
    assert np.abs(got[live] - want[live]).max() <= TOL[dtype]
    assert (got[~live] == 0).all()  # an empty context yields zeros, as the oracle's does
