"""Grouped key/value heads (AttentionParams::key_value_heads, src/api/attention_interface.hpp:61) on the
GPU, through the C ABI.

The reference announces the field and reads it nowhere, so there is nothing of its own to compare with:
PARITY UNPINNED BY THE REFERENCE.  What pins these kernels is the definition itself - query head h uses
K/V head h // (H / H_kv) - checked as: the grouped call must equal the ordinary oracle (one K/V head per
query head) fed K and V with every head repeated H / H_kv times.  Tolerances as everywhere: fp32 1e-4,
16-bit 2e-2 max-abs against the fp32 oracle on the same rounded inputs."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def expand_heads(x, g, axis):
    """[..., H_kv, ...] -> [..., H_kv * g, ...]: head j of the result is head j // g of x."""
    return np.ascontiguousarray(np.repeat(x, g, axis=axis))


@pytest.mark.parametrize("dtype", [O.F32, O.F16, O.BF16])
@pytest.mark.parametrize("B,N,H,Hkv,d,causal", [
    (2, 200, 8, 2, 64, True),
    (1, 333, 6, 3, 128, False),
    (2, 130, 4, 1, 128, True),   # multi-query: one K/V head
    (1, 64, 8, 8, 64, True),     # g = 1 through the grouped entry point
])
def test_flash_gqa_equals_expanded_heads(gpu, dtype, B, N, H, Hkv, d, causal):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, TOL
    g = H // Hkv
    q = O.round_to(O.fill_normal((B, N, H, d), 31, 1), dtype)
    k = O.round_to(O.fill_normal((B, N, Hkv, d), 31, 2), dtype)
    v = O.round_to(O.fill_normal((B, N, Hkv, d), 31, 3), dtype)
    scale = 1.0 / np.sqrt(d)
    want = O.attention(q, expand_heads(k, g, 2), expand_heads(v, g, 2), B, N, H, d, scale, causal)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    do = torch.full_like(dq, float("nan"))
    gpu.flash_fwd_gqa(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), dtype, B, N, H, Hkv, d,
                      (N * H * d, H * d, d), (N * Hkv * d, Hkv * d, d), scale, causal, stream_ptr())
    torch.cuda.synchronize()
    got = to_host(do)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL[dtype]


def test_flash_gqa_masked_fp32(gpu):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr
    B, N, H, Hkv, d = 2, 48, 4, 2, 32
    q = O.fill_uniform((B, N, H, d), 32, 1)
    k = O.fill_uniform((B, N, Hkv, d), 32, 2)
    v = O.fill_uniform((B, N, Hkv, d), 32, 3)
    mask = (O.fill_uniform((B, N, N), 32, 9) > -0.4).astype(np.float32)
    mask[:, np.arange(N), np.arange(N)] = 1.0
    want = O.attention(q, expand_heads(k, 2, 2), expand_heads(v, 2, 2), B, N, H, d, 0.2, False, mask=mask)
    dq, dk, dv = to_dev(q, O.F32), to_dev(k, O.F32), to_dev(v, O.F32)
    dm = torch.from_numpy(mask).cuda()
    do = torch.full_like(dq, float("nan"))
    gpu.flash_fwd_gqa(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), O.F32, B, N, H, Hkv, d,
                      (N * H * d, H * d, d), (N * Hkv * d, Hkv * d, d), 0.2, False, stream_ptr(), dm.data_ptr())
    torch.cuda.synchronize()
    assert np.abs(to_host(do) - want).max() <= 1e-4


@pytest.mark.parametrize("dtype", [O.F16, O.BF16])
def test_flash_varlen_gqa(gpu, dtype):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32, TOL
    H, Hkv, d = 8, 2, 64
    lens = np.array([70, 1, 129, 300], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    q = O.round_to(O.fill_normal((T, H, d), 33, 1, 0.5), dtype)
    k = O.round_to(O.fill_normal((T, Hkv, d), 33, 2, 0.5), dtype)
    v = O.round_to(O.fill_normal((T, Hkv, d), 33, 3, 0.5), dtype)
    scale = 1.0 / np.sqrt(d)
    want = O.attention_varlen(q, expand_heads(k, 4, 1), expand_heads(v, 4, 1), cu, H, d, scale, True)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    do = torch.full_like(dq, float("nan"))
    dcu = dev_i32(cu)
    gpu.flash_fwd_varlen_gqa(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), dtype, dcu.data_ptr(), len(lens),
                             int(lens.max()), H, Hkv, d, H * d, d, Hkv * d, d, scale, True, stream_ptr())
    torch.cuda.synchronize()
    got = to_host(do)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL[dtype]


def test_flash_gqa_rejects_uneven_groups(gpu):
    import torch
    from attention_amd.hip import HipError
    x = torch.zeros(1 * 16 * 6 * 64, dtype=torch.float16, device="cuda")
    with pytest.raises(HipError) as e:
        gpu.flash_fwd_gqa(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), O.F16, 1, 16, 6, 4, 64,
                          (16 * 6 * 64, 6 * 64, 64), (16 * 4 * 64, 4 * 64, 64), 0.0, False, None)
    assert e.value.code == -2


def build_pool(B, Hkv, d, P, lens, seed, dtype):
    lens = np.asarray(lens, np.int32)
    pages_per = (lens + P - 1) // P
    max_pages = max(1, int(pages_per.max()))
    n_pages = int(pages_per.sum()) + 3
    ids = O.permutation(n_pages, seed, 5)
    table = np.full((B, max_pages), -1, np.int32)
    c = 0
    for b in range(B):
        table[b, :pages_per[b]] = ids[c:c + pages_per[b]]
        c += pages_per[b]
    kp = np.zeros(n_pages * P * Hkv * d, np.float32)
    vp = np.zeros_like(kp)
    for b in range(B):
        kb = O.round_to(O.fill_normal((int(lens[b]), Hkv, d), seed + 10 + b, 2), dtype)
        vb = O.round_to(O.fill_normal((int(lens[b]), Hkv, d), seed + 10 + b, 3), dtype)
        O.kv_scatter(kb, vb, kp, vp, table, b, 0, P, Hkv, d)
    return kp, vp, table, lens, n_pages


@pytest.fixture(params=[2, 16], ids=["matrix-core-from-2", "lane-per-element-to-8"])
def kernel_choice(gpu, request):
    """Groups of 2, 4 and 8 heads on 16-bit pools (d 64/128, pages of 16) exist on both decode kernels: the tuning value
    decides, and both settings are run."""
    before = gpu.get_tuning("decode_matrix_min_group")
    gpu.set_tuning("decode_matrix_min_group", request.param)
    yield request.param
    gpu.set_tuning("decode_matrix_min_group", before)


@pytest.mark.parametrize("dtype", [O.F32, O.F16, O.BF16])
@pytest.mark.parametrize("H,Hkv,d,P", [(8, 4, 128, 16), (8, 2, 64, 16), (16, 2, 128, 16), (4, 1, 128, 8), (6, 3, 32, 16),
                                       (9, 3, 64, 16), (10, 2, 128, 16), (14, 2, 128, 16), (6, 1, 96, 8), (21, 3, 128, 16)])
def test_decode_gqa_equals_expanded_pool(gpu, dtype, H, Hkv, d, P, kernel_choice):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32, TOL
    g = H // Hkv
    B = 4
    lens = [45, 1, 260, 16]
    kp, vp, table, lens, n_pages = build_pool(B, Hkv, d, P, lens, 41, dtype)
    q = O.round_to(O.fill_normal((B, H, d), 41, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    # the oracle sees a pool with H heads per token: every pool head repeated g times
    kx = expand_heads(kp.reshape(n_pages * P, Hkv, d), g, 1).reshape(-1)
    vx = expand_heads(vp.reshape(n_pages * P, Hkv, d), g, 1).reshape(-1)
    want = O.paged_decode(q, kx, vx, table, lens, None, B, H, d, P, scale)
    kd, vd = to_dev(kp, dtype), to_dev(vp, dtype)
    dt, dl = dev_i32(table), dev_i32(lens)
    for chunk in (0, 2 * P, 1024):
        dq = to_dev(q, dtype)
        do = torch.full_like(dq, float("nan"))
        max_len = int(lens.max())
        ws_bytes = gpu.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
        ws = torch.empty(max(ws_bytes, 4) // 4, dtype=torch.float32, device="cuda")
        gpu.paged_decode_gqa(dq.data_ptr(), do.data_ptr(), dtype, kd.data_ptr(), vd.data_ptr(), dtype, dt.data_ptr(),
                             dl.data_ptr(), None, B, H, Hkv, d, P, table.shape[1], max_len, scale, chunk, ws.data_ptr(),
                             ws_bytes, stream_ptr())
        torch.cuda.synchronize()
        got = to_host(do)
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() <= TOL[dtype], f"chunk={chunk}"


@pytest.mark.parametrize("dtype,H,Hkv,d,P", [(O.F16, 66, 2, 64, 16), (O.F32, 32, 2, 128, 16), (O.BF16, 18, 2, 64, 8), (O.F32, 71, 1, 64, 16)])
def test_decode_gqa_wide_groups_in_slices(gpu, dtype, H, Hkv, d, P):
    """More than 8 query heads per cached head where the matrix-core kernels do not apply (more than 32, an fp32 pool,
    pages of 8 tokens): slices of 8 query heads on the lane-per-element kernel."""
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32, TOL
    g = H // Hkv
    B = 3
    kp, vp, table, lens, n_pages = build_pool(B, Hkv, d, P, [45, 0, 260], 43, dtype)
    q = O.round_to(O.fill_normal((B, H, d), 43, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    kx = expand_heads(kp.reshape(n_pages * P, Hkv, d), g, 1).reshape(-1)
    vx = expand_heads(vp.reshape(n_pages * P, Hkv, d), g, 1).reshape(-1)
    want = O.paged_decode(q, kx, vx, table, lens, None, B, H, d, P, scale)
    kd, vd = to_dev(kp, dtype), to_dev(vp, dtype)
    dt, dl = dev_i32(table), dev_i32(lens)
    max_len = int(lens.max())
    for chunk in (0, 4 * P):
        dq = to_dev(q, dtype)
        do = torch.full_like(dq, float("nan"))
        ws_bytes = gpu.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
        ws = torch.empty(max(ws_bytes, 4) // 4, dtype=torch.float32, device="cuda")
        gpu.paged_decode_gqa(dq.data_ptr(), do.data_ptr(), dtype, kd.data_ptr(), vd.data_ptr(), dtype, dt.data_ptr(),
                             dl.data_ptr(), None, B, H, Hkv, d, P, table.shape[1], max_len, scale, chunk, ws.data_ptr(),
                             ws_bytes, stream_ptr())
        torch.cuda.synchronize()
        got = to_host(do)
        assert np.all(got[1] == 0.0)
        assert np.abs(got - want).max() <= TOL[dtype], f"chunk={chunk}"
