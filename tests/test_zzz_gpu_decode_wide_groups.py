"""Grouped-head decode on the matrix-core kernel, on the GPU through the C ABI, against the CPU oracle fed a pool
whose heads are repeated (the definition of grouped heads).  16 and 32 query heads per pool head exist on this
kernel only; 4 and 8 take it when the tuning value decode_matrix_min_group says so."""
import numpy as np
import pytest

from oracle import oracle as O
from test_gpu_paged import build_problem, poison_unused, gpu_decode  # noqa: F401  (builders; gpu_decode documents the call)

pytestmark = pytest.mark.gpu


def run(hip, q, kp, vp, table, lens, B, H, H_kv, d, P, dtype, qo_dtype, scale, chunk):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32
    dq = to_dev(q, qo_dtype)
    do = torch.full_like(dq, float("nan"))
    kd, vd = to_dev(kp, dtype), to_dev(vp, dtype)
    dt, dl = dev_i32(table), dev_i32(lens)
    max_len = int(max(1, lens.max()))
    ws_bytes = hip.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
    ws = torch.full((max(ws_bytes, 4) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    hip.paged_decode_gqa(dq.data_ptr(), do.data_ptr(), qo_dtype, kd.data_ptr(), vd.data_ptr(), dtype, dt.data_ptr(),
                         dl.data_ptr(), None, B, H, H_kv, d, P, table.shape[1], max_len, scale, chunk, ws.data_ptr(), ws_bytes,
                         stream_ptr())
    torch.cuda.synchronize()
    return to_host(do)


@pytest.fixture
def matrix_kernel_from_four(gpu):
    before = gpu.get_tuning("decode_matrix_min_group")
    gpu.set_tuning("decode_matrix_min_group", 4)
    yield
    gpu.set_tuning("decode_matrix_min_group", before)


@pytest.mark.parametrize("dtype,d", [(O.F16, 128), (O.BF16, 64), (O.BF16, 128), (O.F16, 256), (O.BF16, 256)])
@pytest.mark.parametrize("G", [4, 5, 7, 8, 12, 16, 17, 24, 31, 32])
def test_matrix_core_decode_equals_repeated_heads(gpu, G, dtype, d, matrix_kernel_from_four):
    B, H_kv, P = 5, 2, 16
    H = G * H_kv
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, [700, 5, 129, 32, 1000], 23, dtype)
    lens = lens.copy()
    lens[3] = 0
    q = O.round_to(O.fill_normal((B, H, d), 23, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H_kv, d)   # NaN wherever the pool holds no token of a sequence
    for chunk, qo in ((0, dtype), (48, O.F32), (16, dtype), (1024, dtype)):
        got = run(gpu, q, kp, vp, table, lens, B, H, H_kv, d, P, dtype, qo, scale, chunk)
        assert np.isfinite(got).all()
        assert np.all(got[3] == 0.0)
        assert np.abs(got - want).max() <= 2e-2, (chunk, qo)


@pytest.mark.parametrize("waves", [1, 2, 4])
@pytest.mark.parametrize("G,H_kv,d,dtype", [(32, 1, 128, O.F16), (24, 2, 64, O.BF16), (17, 1, 256, O.BF16), (32, 3, 128, O.BF16)])
def test_wide_groups_workgroup_widths(gpu, G, H_kv, d, dtype, waves):
    """Groups of 17 to 32 query heads in workgroups of 1, 2 and 4 wavefronts (at d = 256: 1 and 2) that share a chunk's
    tiles out and merge in LDS: chunks with fewer tiles than wavefronts, with one tile more than a multiple, a sequence
    that ends on a tile's border, an empty one, and a page that is missing inside a chunk."""
    B, P = 6, 16
    H = G * H_kv
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, [1500, 33, 1024, 7, 2049, 300], 31, dtype)
    lens = lens.copy()
    lens[3] = 0
    q = O.round_to(O.fill_normal((B, H, d), 31, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    holed = table.copy()
    holed[5, 9] = -1           # sequence 5 ends in front of its tenth page: 144 tokens
    want = O.paged_decode(q, rep(kp), rep(vp), holed, lens, None, B, H, d, P, scale)
    kp, vp, _ = poison_unused(kp, vp, table, lens, P, H_kv, d)
    table = holed
    before = gpu.get_tuning("decode_waves")
    gpu.set_tuning("decode_waves", waves)
    try:
        for chunk in (0, 1024, 288, 64):
            got = run(gpu, q, kp, vp, table, lens, B, H, H_kv, d, P, dtype, dtype, scale, chunk)
            assert np.isfinite(got).all()
            assert np.all(got[3] == 0.0)
            assert np.abs(got - want).max() <= 2e-2, chunk
    finally:
        gpu.set_tuning("decode_waves", before)


@pytest.mark.parametrize("H_kv,G,d,dtype", [(8, 4, 128, O.F16), (5, 2, 64, O.BF16), (1, 16, 128, O.BF16), (3, 8, 64, O.F16)])
def test_page_ring_of_the_group_kernel(gpu, H_kv, G, d, dtype):
    """8, 4, 2 and 1 pool heads side by side in a workgroup of the page-by-page kernel, chunks of several trips round its
    ring of page slots with every remainder of pages behind the last full trip."""
    B, P = 5, 16
    lens_in = [16 * 4 * 3, 16 * 9 + 1, 16 * 10 + 15, 16 * 7, 3]
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, lens_in, 29, dtype)
    H = G * H_kv
    q = O.round_to(O.fill_normal((B, H, d), 29, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H_kv, d)
    before = gpu.get_tuning("decode_matrix_min_group"), gpu.get_tuning("decode_waves")
    gpu.set_tuning("decode_matrix_min_group", 2)
    try:
        # (a launch this small would get single wavefronts: 8 asks for the widest workgroup the pool's heads fill)
        for waves in (8, 0):
            gpu.set_tuning("decode_waves", waves)
            for chunk in (1024, 96, 0):
                got = run(gpu, q, kp, vp, table, lens, B, H, H_kv, d, P, dtype, dtype, scale, chunk)
                assert np.isfinite(got).all()
                assert np.abs(got - want).max() <= 2e-2, (waves, chunk)
    finally:
        gpu.set_tuning("decode_matrix_min_group", before[0])
        gpu.set_tuning("decode_waves", before[1])


def test_both_kernels_agree_for_groups_of_four(gpu):
    B, H_kv, d, P, G = 3, 8, 128, 16, 4
    H = G * H_kv
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, [2000, 77, 513], 25, O.F16)
    q = O.round_to(O.fill_normal((B, H, d), 25, 1), O.F16)
    scale = 1.0 / np.sqrt(d)
    before = gpu.get_tuning("decode_matrix_min_group")
    try:
        gpu.set_tuning("decode_matrix_min_group", 16)
        a = run(gpu, q, kp, vp, table, lens, B, H, H_kv, d, P, O.F16, O.F32, scale, 0)
        gpu.set_tuning("decode_matrix_min_group", 4)
        b = run(gpu, q, kp, vp, table, lens, B, H, H_kv, d, P, O.F16, O.F32, scale, 0)
    finally:
        gpu.set_tuning("decode_matrix_min_group", before)
    assert np.abs(a - b).max() <= 5e-3   # same inputs, fp32 outputs: only P's rounding to 16 bits differs
