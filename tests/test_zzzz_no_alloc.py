"""ahpc_hip_paged_decode_noalloc: the decode entry point that allocates nothing (chunk partials in an array that is
part of the library's device code).  Through the C ABI, against ahpc_hip_paged_decode_gqa on the same inputs - same
kernels, same chunking, so bit for bit - on two calls in a row, the second with a smaller problem (the array keeps
the first call's contents).  Collected last on purpose."""
import numpy as np
import pytest

from oracle import oracle as O
from test_gpu_paged import build_problem, poison_unused

pytestmark = pytest.mark.gpu


def both(hip, B, H, H_kv, d, P, lens, seed, dtype, chunk):
    """(existing entry point with a workspace, new entry point, oracle) on one problem."""
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32
    _, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, lens, seed, dtype)
    q = O.round_to(O.fill_normal((B, H, d), seed, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    G = H // H_kv
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H_kv, d)
    dq = to_dev(q, dtype)
    kd, vd = to_dev(kp, dtype), to_dev(vp, dtype)
    dt, dl = dev_i32(table), dev_i32(lens)
    max_len = int(max(1, lens.max()))
    ws_bytes = hip.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
    ws = torch.full((max(ws_bytes, 4) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    a = torch.full_like(dq, float("nan"))
    b = torch.full_like(dq, float("nan"))
    hip.paged_decode_gqa(dq.data_ptr(), a.data_ptr(), dtype, kd.data_ptr(), vd.data_ptr(), dtype, dt.data_ptr(), dl.data_ptr(),
                         None, B, H, H_kv, d, P, table.shape[1], max_len, scale, chunk, ws.data_ptr(), ws_bytes, stream_ptr())
    torch.cuda.synchronize()
    # everything the new entry point needs exists by now: from here on it must not allocate
    hip.paged_decode_noalloc(dq.data_ptr(), b.data_ptr(), dtype, kd.data_ptr(), vd.data_ptr(), dtype, dt.data_ptr(),
                             dl.data_ptr(), None, B, H, H_kv, d, P, table.shape[1], max_len, scale, chunk, stream_ptr())
    torch.cuda.synchronize()
    return to_host(a), to_host(b), want


def test_two_calls_in_a_row_the_second_smaller(gpu):
    # several chunks per sequence, so the partials and the merge are in play; then a smaller batch with shorter contexts
    first = both(gpu, 6, 8, 8, 128, 16, [900, 5, 129, 2048, 1, 640], 61, O.F16, 128)
    second = both(gpu, 3, 8, 8, 128, 16, [300, 17, 64], 62, O.F16, 128)
    for a, b, want in (first, second):
        assert np.isfinite(b).all()
        assert np.array_equal(a, b)
        assert np.abs(b - want).max() <= 2e-2


def test_grouped_heads_and_single_chunk(gpu):
    a, b, want = both(gpu, 4, 16, 4, 64, 16, [700, 40, 0, 333], 63, O.BF16, 64)
    assert np.array_equal(a, b) and np.all(b[2] == 0.0) and np.abs(b - want).max() <= 2e-2
    a, b, want = both(gpu, 2, 4, 4, 128, 16, [100, 60], 64, O.F16, 1024)   # one chunk: no partials at all
    assert np.array_equal(a, b) and np.abs(b - want).max() <= 2e-2


def test_headline_decode_shape_with_the_launchers_own_chunking(gpu):
    # 64 sequences of 512..4096 tokens, 32 heads of 128: the upper bound of the size query (34 MB) is beyond the
    # array, what the launch plan really needs (chunks of 1024 tokens: 4.3 MB) is not
    rng = np.random.default_rng(65)
    lens = [int(x) for x in rng.integers(512, 4097, 64)]
    assert gpu.paged_decode_workspace_bytes(64, 32, 128, max(lens), 16, 0) > (16 << 20)
    a, b, want = both(gpu, 64, 32, 32, 128, 16, lens, 65, O.F16, 0)
    assert np.isfinite(b).all() and np.array_equal(a, b) and np.abs(b - want).max() <= 2e-2


def test_beyond_the_built_in_scratch_is_refused(gpu):
    import torch
    x = torch.zeros(1 << 16, device="cuda")
    p = x.data_ptr()
    B, H, d, P, max_len, chunk = 4096, 64, 128, 16, 65536, 16
    assert gpu.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk) > (16 << 20)
    with pytest.raises(gpu.HipError) as e:
        gpu.paged_decode_noalloc(p, p, O.F16, p, p, O.F16, p, p, None, B, H, H, d, P, max_len // P, max_len, 0.1, chunk, None)
    assert "scratch" in str(e.value)
    torch.cuda.synchronize()
