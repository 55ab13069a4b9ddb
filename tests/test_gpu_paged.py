"""Paged KV pool and decode on the GPU (through the C ABI) against the CPU oracle: bit-exact gather
indices and scatter/gather round trips, decode within 1e-4 (fp32 pool) / 2e-2 (fp16, bf16 pools)."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def build_problem(B, H, d, P, lens, seed, dtype, extra_pages=5):
    """Seeded shuffled block table + pool filled through the oracle's scatter (fp32 view, rounded)."""
    lens = np.asarray(lens, np.int32)
    pages_per = (lens + P - 1) // P
    max_pages = max(1, int(pages_per.max()))
    n_pages = int(pages_per.sum()) + extra_pages
    ids = O.permutation(n_pages, seed, 5)
    table = np.full((B, max_pages), -1, np.int32)
    c = 0
    for b in range(B):
        table[b, :pages_per[b]] = ids[c:c + pages_per[b]]
        c += pages_per[b]
    kp = np.zeros(n_pages * P * H * d, np.float32)
    vp = np.zeros_like(kp)
    news = []
    for b in range(B):
        kb = O.round_to(O.fill_normal((int(lens[b]), H, d), seed + 10 + b, 2), dtype)
        vb = O.round_to(O.fill_normal((int(lens[b]), H, d), seed + 10 + b, 3), dtype)
        O.kv_scatter(kb, vb, kp, vp, table, b, 0, P, H, d)
        news.append((kb, vb))
    q = O.round_to(O.fill_normal((B, H, d), seed, 1), dtype)
    return q, kp, vp, table, lens, news, n_pages


def poison_unused(kp, vp, table, lens, P, H, d, wild_page=None):
    """Copies of the pools with NaN in every token slot that no sequence owns (the tail of a last page, free pages,
    the pages of a sequence whose length was set to zero), and of the table with `wild_page` (if given) in the
    entries behind each sequence's last page.  A decode must neither read the former into its result nor
    dereference the latter."""
    kp, vp, table = kp.copy(), vp.copy(), table.copy()
    used = np.zeros(kp.size // (H * d), bool)
    for b, n in enumerate(np.asarray(lens)):
        t = np.arange(int(n))
        used[table[b, t // P].astype(np.int64) * P + t % P] = True
        if wild_page is not None:
            table[b, (int(n) + P - 1) // P:] = wild_page
    kp.reshape(-1, H * d)[~used] = np.nan
    vp.reshape(-1, H * d)[~used] = np.nan
    return kp, vp, table


def gpu_decode(hip, q, kp_dev, vp_dev, table, lens, rows, B, H, d, P, dtype, qo_dtype, scale, chunk=0, max_len=None):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32
    dq = to_dev(q, qo_dtype)
    do = torch.full_like(dq, float("nan"))
    dt, dl = dev_i32(table), dev_i32(lens)
    dr = None if rows is None else dev_i32(rows)
    max_len = int(max_len or max(1, lens.max()))
    ws_bytes = hip.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
    ws = torch.empty(max(ws_bytes, 4) // 4, dtype=torch.float32, device="cuda")
    hip.paged_decode(dq.data_ptr(), do.data_ptr(), qo_dtype, kp_dev.data_ptr(), vp_dev.data_ptr(), dtype, dt.data_ptr(),
                     dl.data_ptr(), None if dr is None else dr.data_ptr(), B, H, d, P, table.shape[1], max_len, scale,
                     chunk, ws.data_ptr(), ws_bytes, stream_ptr())
    torch.cuda.synchronize()
    return to_host(do)


@pytest.mark.parametrize("dtype", [O.F32, O.F16, O.BF16])
@pytest.mark.parametrize("H,d,P", [(4, 32, 16), (32, 128, 16), (6, 64, 4), (3, 128, 16), (2, 256, 8)])
def test_decode_small(gpu, dtype, H, d, P):
    from gpu_util import to_dev
    B = 5
    lens = [33, 1, 16, 100, 257]
    q, kp, vp, table, lens, _, _ = build_problem(B, H, d, P, lens, 21, dtype)
    kd, vd = to_dev(kp, dtype), to_dev(vp, dtype)
    scale = 1.0 / np.sqrt(d)
    want = O.paged_decode(q, kp, vp, table, lens, None, B, H, d, P, scale)
    tol = 1e-4 if dtype == O.F32 else 2e-2
    for chunk in (0, P, 4 * P, 1024):
        got = gpu_decode(gpu, q, kd, vd, table, lens, None, B, H, d, P, dtype, dtype, scale, chunk)
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() <= tol, f"chunk={chunk}"


@pytest.mark.parametrize("dtype,H,d,P", [(O.BF16, 4, 96, 16), (O.F16, 8, 80, 16), (O.F32, 3, 100, 8), (O.BF16, 2, 8, 16), (O.F32, 4, 4, 16),
                                        (O.F16, 6, 200, 4), (O.BF16, 32, 112, 16)])
def test_decode_other_head_dimensions(gpu, dtype, H, d, P):
    """Head dimensions in whole 16-byte pieces that are not 32, 64, 128 or 256 run on the kernel of the next size; unused
    slots and pages of the pool are NaN."""
    from gpu_util import to_dev
    B = 5
    q, kp, vp, table, lens, _, _ = build_problem(B, H, d, P, [33, 1, 16, 150, 700], 43, dtype)
    scale = 1.0 / np.sqrt(d)
    want = O.paged_decode(q, kp, vp, table, lens, None, B, H, d, P, scale)
    kp_n, vp_n, _ = poison_unused(kp, vp, table, lens, P, H, d)
    kd, vd = to_dev(kp_n, dtype), to_dev(vp_n, dtype)
    for chunk in (0, 2 * P, 16 * P):
        got = gpu_decode(gpu, q, kd, vd, table, lens, None, B, H, d, P, dtype, dtype, scale, chunk)
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() <= (1e-4 if dtype == O.F32 else 2e-2), f"chunk={chunk}"


def test_decode_split_count_invariance_and_fp32_query_on_fp16_pool(gpu):
    from gpu_util import to_dev
    B, H, d, P = 3, 8, 128, 16
    lens = [700, 45, 1000]
    q, kp, vp, table, lens, _, _ = build_problem(B, H, d, P, lens, 31, O.F16)
    kd, vd = to_dev(kp, O.F16), to_dev(vp, O.F16)
    scale = 1.0 / np.sqrt(d)
    want = O.paged_decode(q, kp, vp, table, lens, None, B, H, d, P, scale)
    outs = [gpu_decode(gpu, q, kd, vd, table, lens, None, B, H, d, P, O.F16, O.F32, scale, chunk) for chunk in (16, 112, 512, 1008)]
    for o in outs:
        assert np.abs(o - want).max() <= 2e-3  # fp32 outputs: only the kernel's own rounding is left
    assert np.abs(outs[0] - outs[-1]).max() <= 1e-4


def test_decode_empty_sequence_and_batch_rows(gpu):
    from gpu_util import to_dev
    B, H, d, P = 4, 4, 64, 16
    q, kp, vp, table, lens, _, _ = build_problem(B, H, d, P, [40, 7, 90, 16], 41, O.BF16)
    lens = lens.copy()
    lens[1] = 0
    kd, vd = to_dev(kp, O.BF16), to_dev(vp, O.BF16)
    rows = np.array([2, 1, 0, 3], np.int32)
    want = O.paged_decode(q, kp, vp, table, lens, rows, B, H, d, P, 0.125)
    for chunk in (0, 32):
        got = gpu_decode(gpu, q, kd, vd, table, lens, rows, B, H, d, P, O.BF16, O.BF16, 0.125, chunk)
        assert np.all(got[1] == 0.0)
        assert np.abs(got - want).max() <= 2e-2


@pytest.mark.parametrize("H,H_kv,d,P,dtype", [(4, 4, 128, 16, O.F16), (6, 6, 64, 4, O.F32), (8, 2, 128, 16, O.BF16),
                                              (32, 2, 128, 16, O.F16), (16, 1, 64, 16, O.BF16)])
def test_decode_stops_at_a_missing_page(gpu, H, H_kv, d, P, dtype):
    """A -1 entry inside a sequence ends it there, as the reference kernel's page walk does
    (src/backends/cuda/cuda_kernels.cu:417-420): the first page of a later chunk, a page in the middle of a chunk, the
    very first page.  Every page no sequence owns (page ids a kernel that papers over the hole might fall back to,
    page 0 among them) holds NaN."""
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32
    B = 4
    _, kp, vp, table, lens, _, n_pages = build_problem(B, H_kv, d, P, [600, 600, 40, 70], 23, dtype, extra_pages=9)
    q = O.round_to(O.fill_normal((B, H, d), 23, 1), dtype)
    table = table.copy()
    for b, pg in [(0, 16), (1, 21), (2, 0)]:
        table[b, pg] = -1
    scale = 1.0 / np.sqrt(d)
    G = H // H_kv
    rep = lambda pool: np.repeat(pool.reshape(-1, H_kv, d), G, axis=1).reshape(-1)
    want = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    assert np.all(want[2] == 0.0)
    kp2, vp2 = kp.copy().reshape(n_pages, -1), vp.copy().reshape(n_pages, -1)
    owned = set(table[table >= 0].tolist())
    for pg in range(n_pages):
        if pg not in owned:
            kp2[pg] = np.nan
            vp2[pg] = np.nan
    assert 0 not in owned or True
    kd, vd = to_dev(kp2.reshape(-1), dtype), to_dev(vp2.reshape(-1), dtype)
    dq = to_dev(q, dtype)
    dt, dl = dev_i32(table), dev_i32(lens)
    max_len = int(lens.max())
    for chunk in (0, 16 * P, 4 * P):
        do = torch.full_like(dq, float("nan"))
        ws_bytes = gpu.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
        ws = torch.full((max(ws_bytes, 4) // 4,), float("nan"), dtype=torch.float32, device="cuda")
        gpu.paged_decode_gqa(dq.data_ptr(), do.data_ptr(), dtype, kd.data_ptr(), vd.data_ptr(), dtype, dt.data_ptr(), dl.data_ptr(),
                             None, B, H, H_kv, d, P, table.shape[1], max_len, scale, chunk, ws.data_ptr(), ws_bytes, stream_ptr())
        torch.cuda.synchronize()
        got = to_host(do)
        assert np.isfinite(got).all(), f"chunk={chunk}"
        assert np.all(got[2] == 0.0)
        assert np.abs(got - want).max() <= (1e-4 if dtype == O.F32 else 2e-2), f"chunk={chunk}"
    # and the kernel's own report of what it reads ends at the hole
    out = torch.full((B, max_len), -7, dtype=torch.int64, device="cuda")
    gpu.paged_gather_indices(dt.data_ptr(), dl.data_ptr(), None, B, H_kv, d, P, table.shape[1], max_len, out.data_ptr(), stream_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), O.gather_offsets(table, lens, None, B, max_len, P, H_kv, d))


def test_gather_indices_bit_exact(gpu):
    import torch
    from gpu_util import stream_ptr, dev_i32
    B, H, d, P = 6, 32, 128, 16
    lens = O.fill_lengths(B, 51, 4, 1, 900)
    _, _, _, table, lens, _, _ = build_problem(B, 1, 1, P, lens, 51, O.F32)
    max_len = int(lens.max())
    rows = np.array([5, 0, 3, 1, 2, 4], np.int32)
    dt, dl, dr = dev_i32(table), dev_i32(lens), dev_i32(rows)
    out = torch.full((B, max_len), -7, dtype=torch.int64, device="cuda")
    gpu.paged_gather_indices(dt.data_ptr(), dl.data_ptr(), dr.data_ptr(), B, H, d, P, table.shape[1], max_len,
                             out.data_ptr(), stream_ptr())
    torch.cuda.synchronize()
    want = O.gather_offsets(table, lens, rows, B, max_len, P, H, d)
    assert np.array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("in_dtype,pool_dtype", [(O.F32, O.F32), (O.F32, O.F16), (O.F16, O.F16), (O.BF16, O.BF16), (O.F32, O.BF16)])
def test_scatter_then_gather_roundtrip(gpu, in_dtype, pool_dtype):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32, torch_dtype
    H, d, P = 4, 32, 16
    n_pages = 12
    table = np.array([[7, 2, 9, 0, -1], [3, 11, 5, -1, -1]], np.int32)
    dt = dev_i32(table)
    kpool = torch.zeros(n_pages * P * H * d, dtype=torch_dtype(pool_dtype), device="cuda")
    vpool = torch.zeros_like(kpool)
    store = O.F16 if (in_dtype == O.F16 or pool_dtype == O.F16) else (O.BF16 if (in_dtype == O.BF16 or pool_dtype == O.BF16) else O.F32)
    k1 = O.round_to(O.fill_normal((21, H, d), 1, 2), store)
    v1 = O.round_to(O.fill_normal((21, H, d), 1, 3), store)
    k2 = O.round_to(O.fill_normal((30, H, d), 2, 2), store)
    v2 = O.round_to(O.fill_normal((30, H, d), 2, 3), store)
    # sequence row 0: two appends; row 1: one append through explicit per-token row/position arrays
    a, b = to_dev(k1, in_dtype), to_dev(v1, in_dtype)
    gpu.kv_scatter(a.data_ptr(), b.data_ptr(), in_dtype, kpool.data_ptr(), vpool.data_ptr(), pool_dtype, dt.data_ptr(), 5, 21, H, d, P, row0=0, pos0=0, stream=stream_ptr())
    c, e = to_dev(k2, in_dtype), to_dev(v2, in_dtype)
    gpu.kv_scatter(c.data_ptr(), e.data_ptr(), in_dtype, kpool.data_ptr(), vpool.data_ptr(), pool_dtype, dt.data_ptr(), 5, 30, H, d, P, row0=0, pos0=21, stream=stream_ptr())
    trow = dev_i32(np.full(21, 1))
    tpos = dev_i32(np.arange(21)[::-1].copy())
    gpu.kv_scatter(a.data_ptr(), b.data_ptr(), in_dtype, kpool.data_ptr(), vpool.data_ptr(), pool_dtype, dt.data_ptr(), 5, 21, H, d, P, token_row=trow.data_ptr(), token_pos=tpos.data_ptr(), stream=stream_ptr())
    ko = torch.empty(51 * H * d, dtype=torch.float32, device="cuda")
    vo = torch.empty_like(ko)
    gpu.kv_gather(ko.data_ptr(), vo.data_ptr(), O.F32, kpool.data_ptr(), vpool.data_ptr(), pool_dtype, dt.data_ptr(), 5, 0, 0, 51, H, d, P, stream_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(to_host(ko).reshape(51, H, d), np.concatenate([k1, k2]))
    assert np.array_equal(to_host(vo).reshape(51, H, d), np.concatenate([v1, v2]))
    ko2 = torch.empty(21 * H * d, dtype=torch.float32, device="cuda")
    vo2 = torch.empty_like(ko2)
    gpu.kv_gather(ko2.data_ptr(), vo2.data_ptr(), O.F32, kpool.data_ptr(), vpool.data_ptr(), pool_dtype, dt.data_ptr(), 5, 1, 0, 21, H, d, P, stream_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(to_host(ko2).reshape(21, H, d), k1[::-1])
    # the device pool equals the oracle's pool bit for bit, including pages nobody owns
    kp = np.zeros(n_pages * P * H * d, np.float32)
    vp = np.zeros_like(kp)
    O.kv_scatter(k1, v1, kp, vp, table, 0, 0, P, H, d)
    O.kv_scatter(k2, v2, kp, vp, table, 0, 21, P, H, d)
    O.kv_scatter(np.ascontiguousarray(k1[::-1]), np.ascontiguousarray(v1[::-1]), kp, vp, table, 1, 0, P, H, d)
    assert np.array_equal(to_host(kpool), kp) and np.array_equal(to_host(vpool), vp)


def _full_size_decode(gpu, dtype, B, lo, hi, seed, chunk=0):
    """Full-size decode: pool filled on the device, parity on a sample of sequences against the oracle,
    and gather indices bit-exact over everything."""
    import torch
    from gpu_util import stream_ptr, dev_i32, torch_dtype, to_host
    H, d, P = 32, 128, 16
    lens = O.fill_lengths(B, seed, 4, lo, hi)
    pages_per = (lens + P - 1) // P
    max_pages = int(pages_per.max())
    n_pages = int(pages_per.sum()) + 64
    ids = O.permutation(n_pages, seed, 5)
    table = np.full((B, max_pages), -1, np.int32)
    c = 0
    for b in range(B):
        table[b, :pages_per[b]] = ids[c:c + pages_per[b]]
        c += pages_per[b]
    g = torch.Generator(device="cuda").manual_seed(seed)
    tdt = torch_dtype(dtype)
    kpool = torch.randn(n_pages * P * H * d, generator=g, device="cuda", dtype=torch.float32).to(tdt)
    vpool = torch.randn(n_pages * P * H * d, generator=g, device="cuda", dtype=torch.float32).to(tdt)
    dq = torch.randn((B, H, d), generator=g, device="cuda", dtype=torch.float32).to(tdt)
    do = torch.full_like(dq, float("nan"))
    dt, dl = dev_i32(table), dev_i32(lens)
    max_len = int(lens.max())
    ws_bytes = gpu.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
    ws = torch.empty(max(ws_bytes, 4) // 4, dtype=torch.float32, device="cuda")
    scale = 1.0 / np.sqrt(d)
    gpu.paged_decode(dq.data_ptr(), do.data_ptr(), dtype, kpool.data_ptr(), vpool.data_ptr(), dtype, dt.data_ptr(),
                     dl.data_ptr(), None, B, H, d, P, max_pages, max_len, scale, chunk, ws.data_ptr(), ws_bytes, stream_ptr())
    idx = torch.empty((B, max_len), dtype=torch.int64, device="cuda")
    gpu.paged_gather_indices(dt.data_ptr(), dl.data_ptr(), None, B, H, d, P, max_pages, max_len, idx.data_ptr(), stream_ptr())
    torch.cuda.synchronize()
    assert torch.isfinite(do.float()).all()
    assert np.array_equal(idx.cpu().numpy(), O.gather_offsets(table, lens, None, B, max_len, P, H, d))
    # oracle on a sample of sequences: copy only their pages to the host
    got = to_host(do)
    sample = sorted({0, B - 1, int(np.argmax(lens)), int(np.argmin(lens))})
    for b in sample:
        npg = int(pages_per[b])
        pg = torch.from_numpy(table[b, :npg].astype(np.int64)).cuda()
        ksub = kpool.view(n_pages, -1)[pg].float().cpu().numpy().reshape(-1)
        vsub = vpool.view(n_pages, -1)[pg].float().cpu().numpy().reshape(-1)
        sub_table = np.arange(npg, dtype=np.int32)[None, :]
        want = O.paged_decode(to_host(dq[b:b + 1]), ksub, vsub, sub_table, lens[b:b + 1], None, 1, H, d, P, scale)
        assert np.abs(got[b] - want[0]).max() <= 2e-2, f"sequence {b} (len {lens[b]})"


@pytest.mark.parametrize("chunk,waves", [(1024, 8), (1024, 1), (512, 4), (128, 2), (0, 0)])
def test_decode_workgroup_shapes(gpu, chunk, waves):
    """The launch shapes the plan chooses from (chunk length, wavefronts per workgroup), forced through the tuning
    values, every sequence against the oracle."""
    B, H, d, P = 6, 32, 128, 16
    lens = [2500, 1, 1024, 1025, 300, 4000]
    q, kp, vp, table, lens, _, _ = build_problem(B, H, d, P, lens, 61, O.F16)
    scale = 1.0 / np.sqrt(d)
    want = O.paged_decode(q, kp, vp, table, lens, None, B, H, d, P, scale)
    kp, vp, table = poison_unused(kp, vp, table, lens, P, H, d)
    from gpu_util import to_dev
    before = gpu.get_tuning("decode_chunk"), gpu.get_tuning("decode_waves")
    gpu.set_tuning("decode_chunk", chunk)
    gpu.set_tuning("decode_waves", waves)
    try:
        got = gpu_decode(gpu, q, to_dev(kp, O.F16), to_dev(vp, O.F16), table, lens, None, B, H, d, P, O.F16, O.F16, scale)
    finally:
        gpu.set_tuning("decode_chunk", before[0])
        gpu.set_tuning("decode_waves", before[1])
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= 2e-2


def test_config3_decode_fp16_b64(gpu):
    # fp16, B=64, H=32, d=128, P=16, context lengths U[512, 4096], shuffled block table
    _full_size_decode(gpu, O.F16, 64, 512, 4096, 0xA77E0003)


def test_config4_decode_bf16_long_context(gpu):
    # bf16, B=8, context lengths U[16384, 32768]: split-context reduction
    _full_size_decode(gpu, O.BF16, 8, 16384, 32768, 0xA77E0004)


def test_bad_arguments_are_rejected_without_launch(gpu):
    import torch
    x = torch.zeros(4096, device="cuda")
    p = x.data_ptr()
    with pytest.raises(gpu.HipError):
        gpu.paged_decode(p, p, O.F32, p, p, O.F32, p, p, None, 1, 4, 50, 16, 4, 64, 0.1)  # head dim: not whole 16-byte pieces
    with pytest.raises(gpu.HipError):
        gpu.paged_decode(p, p, O.F32, p, p, O.F32, p, p, None, 1, 4, 64, 16, 4, 6400, 0.1)  # max_len needs more pages than the table has
    with pytest.raises(gpu.HipError):
        gpu.paged_decode(p, p, O.F32, 0, p, O.F32, p, p, None, 1, 4, 64, 16, 4, 64, 0.1)
    with pytest.raises(gpu.HipError):
        gpu.paged_decode(p, p, O.F32, p, p, O.F32, p, p, None, 1, 4, 64, 16, 64, 1024, 0.1, chunk_tokens=16, workspace=None, workspace_bytes=0)
    torch.cuda.synchronize()


# ---- batched append: the prefill -> cache hand-off ---------------------------------------------------
def _tables_for(lens_total, P, seed, extra=3):
    lens_total = np.asarray(lens_total, np.int32)
    pages_per = (lens_total + P - 1) // P
    n_pages = int(pages_per.sum()) + extra
    ids = O.permutation(n_pages, seed, 5)
    table = np.full((len(lens_total), max(1, int(pages_per.max()))), -1, np.int32)
    c = 0
    for b in range(len(lens_total)):
        table[b, :pages_per[b]] = ids[c:c + pages_per[b]]
        c += pages_per[b]
    return table, n_pages


@pytest.mark.parametrize("in_dtype,pool_dtype", [(O.F16, O.F16), (O.BF16, O.BF16), (O.F32, O.F32), (O.F32, O.F16), (O.BF16, O.F32)])
def test_scatter_batch_dense_prefill_matches_oracle_bit_for_bit(gpu, in_dtype, pool_dtype):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32
    B, N, H, d, P = 4, 70, 3, 64, 16
    start = np.array([0, 5, 16, 33], np.int32)       # tokens already cached per sequence
    n_new = np.array([70, 1, 0, 37], np.int32)       # new tokens taken from the [B,N,H,d] prefill tensors
    rows = np.array([2, 0, 3, 1], np.int32)          # batch entry -> table row
    lens_total = np.zeros(4, np.int32)
    lens_total[rows] = start + n_new
    table, n_pages = _tables_for(lens_total, P, 61)
    k = O.round_to(O.fill_normal((B, N, H, d), 61, 2), in_dtype)
    v = O.round_to(O.fill_normal((B, N, H, d), 61, 3), in_dtype)
    kp = np.zeros(n_pages * P * H * d, np.float32)
    vp = np.zeros_like(kp)
    for b in range(B):
        if n_new[b]:
            O.kv_scatter(O.round_to(k[b, :n_new[b]], pool_dtype), O.round_to(v[b, :n_new[b]], pool_dtype), kp, vp, table,
                         int(rows[b]), int(start[b]), P, H, d)
    dk, dv = to_dev(k, in_dtype), to_dev(v, in_dtype)
    dkp, dvp = to_dev(np.zeros_like(kp), pool_dtype), to_dev(np.zeros_like(vp), pool_dtype)
    # the index arrays must stay alive until the launch has run: keep the tensors, not just their addresses
    dtab, drows, dstart, dnew = dev_i32(table), dev_i32(rows), dev_i32(start), dev_i32(n_new)
    gpu.kv_scatter_batch(dk.data_ptr(), dv.data_ptr(), in_dtype, N * H * d, H * d, dkp.data_ptr(), dvp.data_ptr(), pool_dtype,
                         dtab.data_ptr(), table.shape[1], drows.data_ptr(), B, N, H, d, P,
                         seq_start=dstart.data_ptr(), seq_tokens=dnew.data_ptr(), stream=stream_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(to_host(dkp), kp) and np.array_equal(to_host(dvp), vp)


def test_scatter_batch_packed_prefill_then_decode(gpu):
    """Ragged prefill tensors [T,H,d] + cu_seqlens -> pool in one launch; a decode over the pool then
    matches the oracle's decode over the oracle-filled pool."""
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32
    H, d, P = 8, 128, 16
    lens = np.array([130, 16, 1, 255], np.int32)
    B = len(lens)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    table, n_pages = _tables_for(lens, P, 62)
    k = O.round_to(O.fill_normal((T, H, d), 62, 2), O.F16)
    v = O.round_to(O.fill_normal((T, H, d), 62, 3), O.F16)
    kp = np.zeros(n_pages * P * H * d, np.float32)
    vp = np.zeros_like(kp)
    for b in range(B):
        O.kv_scatter(k[cu[b]:cu[b + 1]], v[cu[b]:cu[b + 1]], kp, vp, table, b, 0, P, H, d)
    dk, dv = to_dev(k, O.F16), to_dev(v, O.F16)
    dkp, dvp = to_dev(np.zeros_like(kp), O.F16), to_dev(np.zeros_like(vp), O.F16)
    dtab, drows, dcu = dev_i32(table), dev_i32(np.arange(B, dtype=np.int32)), dev_i32(cu)
    gpu.kv_scatter_batch(dk.data_ptr(), dv.data_ptr(), O.F16, 0, H * d, dkp.data_ptr(), dvp.data_ptr(), O.F16,
                         dtab.data_ptr(), table.shape[1], drows.data_ptr(), B, int(lens.max()), H, d, P,
                         cu_seqlens=dcu.data_ptr(), stream=stream_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(to_host(dkp), kp) and np.array_equal(to_host(dvp), vp)
    q = O.round_to(O.fill_normal((B, H, d), 62, 1), O.F16)
    scale = 1.0 / np.sqrt(d)
    got = gpu_decode(gpu, q, dkp, dvp, table, lens, None, B, H, d, P, O.F16, O.F16, scale)
    want = O.paged_decode(q, kp, vp, table, lens, None, B, H, d, P, scale)
    assert np.abs(got - want).max() <= 2e-2
