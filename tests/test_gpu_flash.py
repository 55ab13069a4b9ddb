"""FlashAttention forward on the GPU (through the C ABI) against the CPU oracle.

Tolerances: fp32 <= 1e-4 max-abs (tests/test_flash_attention.cpp:174 of the reference), fp16/bf16
<= 2e-2 max-abs against the fp32 oracle fed the same, already rounded, inputs."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def run_dense(hip, q, k, v, dtype, B, N, H, d, scale, causal, layout="BNHD", mask=None):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr
    dq, dk, dv = (to_dev(x, dtype) for x in (q, k, v))
    do = torch.full_like(dq, float("nan"))
    strides = (N * H * d, H * d, d) if layout == "BNHD" else (H * N * d, d, N * d)
    dm = None if mask is None else torch.from_numpy(mask).cuda()
    hip.flash_fwd(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), dtype, B, N, H, d, strides, scale, causal,
                  stream_ptr(), None if dm is None else dm.data_ptr())
    torch.cuda.synchronize()
    return to_host(do)


def make_qkv(shape, seed, dtype, sigma=1.0, uniform=False):
    gen = (lambda t: O.fill_uniform(shape, seed, t)) if uniform else (lambda t: O.fill_normal(shape, seed, t, sigma))
    return tuple(O.round_to(gen(t), dtype) for t in (1, 2, 3))


@pytest.mark.parametrize("causal", [False, True])
def test_reference_fixture_shape_fp32(gpu, causal):
    # B=2,N=16,H=4,d=64: the fixture of tests/test_flash_attention.cpp:103-108, U(-1,1) inputs
    B, N, H, d = 2, 16, 4, 64
    q, k, v = make_qkv((B, N, H, d), 1, O.F32, uniform=True)
    scale = 1.0 / np.sqrt(d)
    got = run_dense(gpu, q, k, v, O.F32, B, N, H, d, scale, causal)
    want = O.attention(q, k, v, B, N, H, d, scale, causal)
    assert np.abs(got - want).max() <= 1e-4


@pytest.mark.parametrize("N", [1, 4, 32, 128, 129, 300])
def test_sequence_lengths_fp32(gpu, N):
    # tests/test_flash_attention.cpp:218-260 uses {1,4,32,128}; 129 and 300 add ragged tails
    B, H, d = 2, 4, 64
    q, k, v = make_qkv((B, N, H, d), 2, O.F32, uniform=True)
    got = run_dense(gpu, q, k, v, O.F32, B, N, H, d, 0.125, False)
    want = O.attention(q, k, v, B, N, H, d, 0.125, False)
    assert np.abs(got - want).max() <= 1e-4
    if N == 1:
        assert np.abs(got - v).max() <= 1e-6  # N = 1 => O = V (tests/test_flash_attention.cpp:585-588)


@pytest.mark.parametrize("d", [16, 32, 64, 128, 80, 256])
def test_head_dimensions_fp32(gpu, d):
    # tests/test_flash_attention.cpp:263-307, tolerance max(1e-4, 1e-5*sqrt(d)); 80 and 256 are extra
    B, N, H = 2, 16, 4
    q, k, v = make_qkv((B, N, H, d), 3, O.F32, uniform=True)
    scale = 1.0 / np.sqrt(d)
    got = run_dense(gpu, q, k, v, O.F32, B, N, H, d, scale, True)
    want = O.attention(q, k, v, B, N, H, d, scale, True)
    assert np.abs(got - want).max() <= max(1e-4, 1e-5 * np.sqrt(d))


def test_config1_fp32_noncausal(gpu):
    # fp32, non-causal, B=2, N=512, H=8, d=64, N(0,1) inputs
    B, N, H, d = 2, 512, 8, 64
    q, k, v = make_qkv((B, N, H, d), 0xA77E0001, O.F32)
    scale = 1.0 / np.sqrt(d)
    got = run_dense(gpu, q, k, v, O.F32, B, N, H, d, scale, False)
    want = O.attention(q, k, v, B, N, H, d, scale, False)
    assert np.abs(got - want).max() <= 1e-4


def test_layout_bhnd_fp32(gpu):
    B, N, H, d = 2, 40, 3, 32
    q, k, v = make_qkv((B, H, N, d), 4, O.F32)
    got = run_dense(gpu, q, k, v, O.F32, B, N, H, d, 0.2, True, layout="BHND")
    want = O.attention(q, k, v, B, N, H, d, 0.2, True, layout="BHND")
    assert np.abs(got - want).max() <= 1e-4


def test_dense_mask_fp32(gpu):
    # tests/test_flash_attention.cpp:483-582: mask [B,N,N], 0 = masked; a fully masked row gives zeros
    B, N, H, d = 2, 48, 2, 32
    q, k, v = make_qkv((B, N, H, d), 5, O.F32)
    rng = np.random.default_rng(7)
    mask = (rng.random((B, N, N)) > 0.5).astype(np.float32)
    mask[1, 3, :] = 0.0
    got = run_dense(gpu, q, k, v, O.F32, B, N, H, d, 0.2, False, mask=mask)
    want = O.attention(q, k, v, B, N, H, d, 0.2, False, mask=mask)
    assert np.abs(got - want).max() <= 1e-4
    assert np.all(got[1, 3] == 0.0)


@pytest.fixture(params=[1, 0], ids=["packed-copy", "mask-in-place"])
def mask_path(gpu, request):
    """The matrix-core kernel takes a dense mask as a packed copy made in front of the launch (any N) or reads it in
    place (N a multiple of 4; other lengths go to the fp32-FMA kernel then): the tuning value decides, both are run."""
    before = gpu.get_tuning("mask_pack")
    gpu.set_tuning("mask_pack", request.param)
    yield request.param
    gpu.set_tuning("mask_pack", before)


@pytest.mark.parametrize("dtype,d", [(O.F16, 128), (O.BF16, 64), (O.BF16, 128), (O.BF16, 256), (O.F16, 200)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("N", [4, 64, 132, 520, 1028, 517, 63, 129])
def test_dense_mask_16bit(gpu, dtype, d, causal, N, mask_path):
    """16-bit inputs with a mask [B,N,N].  Rows that see nothing (zeros), a single key, or nothing before the last key
    tile; sequence ends inside a 64-bit mask word, on its edge and one behind it."""
    B, H = 2, 3
    q, k, v = make_qkv((B, N, H, d), 6, dtype)
    mask = (O.fill_uniform((B, N, N), 6, 6) > 0.3).astype(np.float32)
    mask[0, N // 2, :] = 0.0
    mask[1, N - 1, :] = 0.0
    mask[1, N - 1, N - 1] = 1.0
    mask[1, 0, :] = 0.0
    mask[1, 0, 0] = 1.0
    if N > 70:
        mask[0, N - 2, :N - 3] = 0.0
    scale = 1.0 / np.sqrt(d)
    got = run_dense(gpu, q, k, v, dtype, B, N, H, d, scale, causal, mask=mask)
    want = O.attention(q, k, v, B, N, H, d, scale, causal, mask=mask)
    assert np.isfinite(got).all()
    assert np.all(got[0, N // 2] == 0.0)
    assert np.abs(got - want).max() <= 2e-2


def test_dense_mask_full_size_properties(gpu, mask_path):
    """B=2 N=4096 H=8 d=128 bf16 with a mask: (1) an all-ones mask reproduces the unmasked launch bit for bit;
    (2) a lower-triangular mask reproduces the causal launch within rounding (the same keys, the reference maximum set
    by another rule); (3) sampled rows of a random mask against the oracle."""
    import torch
    from gpu_util import to_dev, to_host, stream_ptr
    B, N, H, d = 2, 4096, 8, 128
    g = torch.Generator(device="cuda").manual_seed(606)
    q, k, v = (torch.randn((B, N, H, d), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16) for _ in range(3))
    scale = 1.0 / np.sqrt(d)
    st = (N * H * d, H * d, d)

    def launch(causal, mask):
        o = torch.full_like(q, float("nan"))
        gpu.flash_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), O.BF16, B, N, H, d, st, scale, causal, stream_ptr(),
                      None if mask is None else mask.data_ptr())
        torch.cuda.synchronize()
        return o

    plain, causal = launch(False, None), launch(True, None)
    ones = torch.ones((B, N, N), device="cuda")
    assert torch.equal(launch(False, ones), plain)
    tril = torch.tril(torch.ones((N, N), device="cuda")).expand(B, N, N).contiguous()
    assert (launch(False, tril).float() - causal.float()).abs().max().item() <= 2e-2
    rnd = (torch.rand((B, N, N), generator=g, device="cuda") > 0.5).float()
    got = launch(False, rnd)
    assert torch.isfinite(got.float()).all()
    rows = [(0, 0, 0), (1, 7, 4095), (0, 3, 2048), (1, 5, 63)]
    qh, kh, vh, mh = (x.float().cpu().numpy() for x in (q, k, v, rnd))
    for b, h, n in rows:
        s = (kh[b, :, h] @ qh[b, n, h]) * scale
        s[mh[b, n] == 0.0] = -np.inf
        w = np.exp(s - s.max())
        want = (w[:, None] * vh[b, :, h]).sum(0) / w.sum()
        assert np.abs(got[b, n, h].float().cpu().numpy() - want).max() <= 2e-2, (b, h, n)


def test_dense_mask_packed_copy_shared_between_streams_and_sizes(gpu):
    """The packed copy of the mask is one buffer per device: launches with different masks on two streams, queued without
    a synchronisation in between and with the sizes growing (the buffer is replaced while earlier launches may still run),
    each give their own result."""
    import torch
    from gpu_util import to_dev, to_host
    H, d = 2, 128
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    jobs = []
    for i, N in enumerate([64, 200, 132, 520, 260, 1028]):
        B = 1 + i % 2
        q, k, v = make_qkv((B, N, H, d), 70 + i, O.BF16)
        mask = (O.fill_uniform((B, N, N), 70 + i, 6) > (-0.5 + 0.2 * i)).astype(np.float32)
        mask[:, np.arange(N), np.arange(N)] = 1.0
        dq, dk, dv = to_dev(q, O.BF16), to_dev(k, O.BF16), to_dev(v, O.BF16)
        dm = torch.from_numpy(mask).cuda()
        do = torch.full_like(dq, float("nan"))
        jobs.append((B, N, q, k, v, mask, dq, dk, dv, dm, do))
    torch.cuda.synchronize()
    for rep in range(3):
        for i, (B, N, q, k, v, mask, dq, dk, dv, dm, do) in enumerate(jobs):
            st = streams[(i + rep) % 2]
            gpu.flash_fwd(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), O.BF16, B, N, H, d, (N * H * d, H * d, d),
                          1.0 / np.sqrt(d), False, st.cuda_stream, dm.data_ptr())
    torch.cuda.synchronize()
    for B, N, q, k, v, mask, dq, dk, dv, dm, do in jobs:
        want = O.attention(q, k, v, B, N, H, d, 1.0 / np.sqrt(d), False, mask=mask)
        assert np.abs(to_host(do) - want).max() <= 2e-2, N


def test_dense_mask_under_graph_capture_allocates_nothing(gpu):
    """A stream under graph capture gets the kernel that reads the mask in place (the packed copy would need an allocation
    and a wait on another stream's event): the captured graph replays correctly, with new inputs between the replays."""
    import torch
    from gpu_util import to_dev, to_host
    B, N, H, d = 2, 260, 2, 128
    q, k, v = make_qkv((B, N, H, d), 81, O.BF16)
    mask = (O.fill_uniform((B, N, N), 81, 6) > -0.2).astype(np.float32)
    mask[:, np.arange(N), np.arange(N)] = 1.0
    dq, dk, dv, dm = to_dev(q, O.BF16), to_dev(k, O.BF16), to_dev(v, O.BF16), torch.from_numpy(mask).cuda()
    do = torch.full_like(dq, float("nan"))
    scale = 1.0 / np.sqrt(d)
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        gpu.flash_fwd(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), O.BF16, B, N, H, d, (N * H * d, H * d, d),
                      scale, False, torch.cuda.current_stream().cuda_stream, dm.data_ptr())
    for rep in range(3):
        if rep:
            q, k, v = make_qkv((B, N, H, d), 81 + rep, O.BF16)
            mask = (O.fill_uniform((B, N, N), 81 + rep, 6) > 0.1 * rep).astype(np.float32)
            mask[:, np.arange(N), np.arange(N)] = 1.0
            dq.copy_(to_dev(q, O.BF16)); dk.copy_(to_dev(k, O.BF16)); dv.copy_(to_dev(v, O.BF16)); dm.copy_(torch.from_numpy(mask).cuda())
        do.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = O.attention(q, k, v, B, N, H, d, scale, False, mask=mask)
        assert np.abs(to_host(do) - want).max() <= 2e-2, rep


@pytest.mark.parametrize("dtype,d", [(O.BF16, 32), (O.F16, 96), (O.BF16, 8), (O.F16, 120), (O.BF16, 80), (O.F32, 32), (O.F32, 100),
                                     (O.F32, 4), (O.F32, 72), (O.BF16, 256), (O.F16, 200), (O.BF16, 136), (O.F16, 256), (O.F32, 256), (O.F32, 132)])
@pytest.mark.parametrize("N,causal,H,H_kv", [(150, True, 2, 1), (64, False, 3, 3), (517, True, 4, 2)])
def test_smaller_head_dimensions_on_the_matrix_cores(gpu, dtype, d, N, causal, H, H_kv):
    """Head dimensions other than 64 / 128 (multiples of 8 for 16-bit tensors, of 4 for fp32; up to 256) run
    on the matrix-core kernels of the next size with columns that contribute nothing; the output tensor is pre-filled with
    NaN, every element must have been written."""
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, TOL
    B = 2
    q = O.round_to(O.fill_normal((B, N, H, d), 91, 1), dtype)
    k = O.round_to(O.fill_normal((B, N, H_kv, d), 91, 2), dtype)
    v = O.round_to(O.fill_normal((B, N, H_kv, d), 91, 3), dtype)
    scale = 1.0 / np.sqrt(d)
    rep = H // H_kv
    want = O.attention(q, np.repeat(k, rep, axis=2), np.repeat(v, rep, axis=2), B, N, H, d, scale, causal)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    do = torch.full_like(dq, float("nan"))
    gpu.flash_fwd_gqa(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), dtype, B, N, H, H_kv, d,
                      (N * H * d, H * d, d), (N * H_kv * d, H_kv * d, d), scale, causal, stream_ptr())
    torch.cuda.synchronize()
    got = to_host(do)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL[dtype]


@pytest.mark.parametrize("dtype", [O.F16, O.BF16])
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("N", [1, 37, 64, 128, 200, 517])
def test_mfma_small(gpu, dtype, d, causal, N):
    B, H = 2, 3
    q, k, v = make_qkv((B, N, H, d), 100 + N, dtype)
    scale = 1.0 / np.sqrt(d)
    got = run_dense(gpu, q, k, v, dtype, B, N, H, d, scale, causal)
    want = O.attention(q, k, v, B, N, H, d, scale, causal)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= 2e-2


@pytest.fixture
def flash_rows(gpu):
    """flash_rows(n) pins the query rows per workgroup of the 16-bit forward (128 or 256) for the rest of the test."""
    before = gpu.get_tuning("flash_rows")
    yield lambda n: gpu.set_tuning("flash_rows", n)
    gpu.set_tuning("flash_rows", before)


@pytest.mark.parametrize("dtype,d", [(O.BF16, 128), (O.F16, 128), (O.F16, 64), (O.BF16, 96)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("N", [1, 64, 255, 256, 257, 517, 1300])
def test_256_row_workgroups_against_oracle_and_128_row_form(gpu, flash_rows, dtype, d, causal, N):
    """The forward with 8 wavefronts per workgroup (256 query rows share one stream of K/V tiles): against the oracle,
    and bit-identical with the 4-wavefront form (a wavefront does the same arithmetic on the same keys in both)."""
    from gpu_util import TOL
    B, H = 2, 3
    q, k, v = make_qkv((B, N, H, d), 300 + N, dtype)
    scale = 1.0 / np.sqrt(d)
    flash_rows(256)
    wide = run_dense(gpu, q, k, v, dtype, B, N, H, d, scale, causal)
    flash_rows(128)
    narrow = run_dense(gpu, q, k, v, dtype, B, N, H, d, scale, causal)
    assert np.isfinite(wide).all()
    assert np.abs(wide - O.attention(q, k, v, B, N, H, d, scale, causal)).max() <= TOL[dtype]
    assert np.array_equal(wide, narrow)


def test_256_row_workgroups_grouped_heads_and_more_block_ids_than_workgroups(gpu, flash_rows):
    """Grouped K/V heads on the persistent kernel, in a launch whose block ids outnumber the CUs (every workgroup walks
    several ids, paired tiles included)."""
    import torch
    from gpu_util import stream_ptr, to_dev, to_host, TOL
    flash_rows(256)
    dtype, B, N, H, H_kv, d = O.BF16, 3, 1100, 40, 10, 128      # 3 * 40 * 5 = 600 query tiles of 256 rows
    q = O.round_to(O.fill_normal((B, N, H, d), 78, 1), dtype)
    k = O.round_to(O.fill_normal((B, N, H_kv, d), 78, 2), dtype)
    v = O.round_to(O.fill_normal((B, N, H_kv, d), 78, 3), dtype)
    for causal, pair_min in ((True, 1), (False, 1024)):
        gpu.set_tuning("flash_pair_min_tiles", pair_min)
        try:
            dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
            do = torch.full_like(dq, float("nan"))
            gpu.flash_fwd_gqa(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), dtype, B, N, H, H_kv, d, (N * H * d, H * d, d),
                              (N * H_kv * d, H_kv * d, d), 0.09, causal, stream_ptr())
            torch.cuda.synchronize()
        finally:
            gpu.set_tuning("flash_pair_min_tiles", 1024)
        got = to_host(do)
        assert np.isfinite(got).all()
        rng = np.random.default_rng(5)
        rows = np.unique(np.concatenate([rng.integers(0, B * H * N, 200), [0, N - 1, B * H * N - 1, 255, 256, 1099]])).astype(np.int64)
        kr, vr = np.repeat(k, H // H_kv, axis=2), np.repeat(v, H // H_kv, axis=2)
        want = O.attention_rows(q, kr, vr, B, N, H, d, 0.09, rows, causal)
        have = np.stack([got[r // (N * H), r % N, (r // N) % H] for r in rows])
        assert np.abs(have - want).max() <= TOL[dtype]


def test_256_row_workgroups_one_long_sequence(gpu, flash_rows):
    """B=1 N=32768 H=8 d=128 bf16 causal (128 query tiles a head, every workgroup walks several): the two forms of the
    kernel agree bit for bit over the whole output, and sampled rows (first, last, tile edges, random) match the oracle."""
    import torch
    from gpu_util import stream_ptr, TOL
    B, N, H, d = 1, 32768, 8, 128
    g = torch.Generator(device="cuda").manual_seed(0xA77E0008)
    q, k, v = (torch.randn((B, N, H, d), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16) for _ in range(3))
    scale = 1.0 / np.sqrt(d)
    outs = []
    for rows in (256, 128):
        flash_rows(rows)
        o = torch.full_like(q, float("nan"))
        gpu.flash_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), O.BF16, B, N, H, d, (N * H * d, H * d, d), scale, True,
                      stream_ptr())
        torch.cuda.synchronize()
        outs.append(o)
    assert torch.isfinite(outs[0].float()).all()
    assert torch.equal(outs[0], outs[1])
    rng = np.random.default_rng(9)
    rows = np.unique(np.concatenate([rng.integers(0, H * N, 48), [0, 255, 256, N - 1, H * N - 1, 7 * N + 16383]])).astype(np.int64)
    qh, kh, vh = (t.float().cpu().numpy() for t in (q, k, v))
    want = O.attention_rows(qh, kh, vh, B, N, H, d, scale, rows, True)
    got = outs[0].float().cpu().numpy()
    have = np.stack([got[0, r % N, r // N] for r in rows])
    assert np.abs(have - want).max() <= TOL[O.BF16]


@pytest.mark.parametrize("dtype", [O.F16, O.BF16])
def test_mfma_closed_forms(gpu, dtype):
    B, N, H, d = 1, 256, 2, 128
    q, k, v = make_qkv((B, N, H, d), 9, dtype)
    # V constant => O constant (exactly representable value)
    vc = np.full_like(v, 0.625)
    got = run_dense(gpu, q, k, vc, dtype, B, N, H, d, 0.1, True)
    assert np.abs(got - 0.625).max() <= 4e-3
    # Q = 0 => prefix mean of V
    got = run_dense(gpu, np.zeros_like(q), k, v, dtype, B, N, H, d, 0.1, True)
    prefix = np.cumsum(v.astype(np.float64), axis=1) / np.arange(1, N + 1)[None, :, None, None]
    assert np.abs(got - prefix).max() <= 2e-2
    # one dominant logit => that V row
    q1 = np.zeros_like(q)
    k1 = np.zeros_like(k)
    q1[..., 0] = 1.0
    k1[:, 77, :, 0] = 80.0
    got = run_dense(gpu, q1, k1, v, dtype, B, N, H, d, 1.0, False)
    assert np.abs(got - v[:, 77:78]).max() <= 1e-2
    # key-permutation invariance (non causal)
    perm = np.random.default_rng(1).permutation(N)
    a = run_dense(gpu, q, k, v, dtype, B, N, H, d, 0.1, False)
    b = run_dense(gpu, q, np.ascontiguousarray(k[:, perm]), np.ascontiguousarray(v[:, perm]), dtype, B, N, H, d, 0.1, False)
    assert np.abs(a - b).max() <= 1e-2


@pytest.mark.parametrize("dtype", [O.F16, O.BF16])
def test_mfma_layout_bhnd(gpu, dtype):
    B, N, H, d = 2, 96, 2, 64
    q, k, v = make_qkv((B, H, N, d), 6, dtype)
    got = run_dense(gpu, q, k, v, dtype, B, N, H, d, 0.125, True, layout="BHND")
    want = O.attention(q, k, v, B, N, H, d, 0.125, True, layout="BHND")
    assert np.abs(got - want).max() <= 2e-2


def test_config2_shape_bf16_causal_sampled_rows(gpu):
    # bf16, causal, B=4, N=4096, H=32, d=128 at full size: a seeded sample of rows against the oracle,
    # plus size-independent properties over the whole output
    import torch
    from gpu_util import stream_ptr
    B, N, H, d = 4, 4096, 32, 128
    dtype = O.BF16
    g = torch.Generator(device="cuda").manual_seed(0xA77E0002)
    dq, dk, dv = (torch.randn((B, N, H, d), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16) for _ in range(3))
    do = torch.full_like(dq, float("nan"))
    scale = 1.0 / np.sqrt(d)
    gpu.flash_fwd(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), dtype, B, N, H, d, (N * H * d, H * d, d),
                  scale, True, stream_ptr())
    torch.cuda.synchronize()
    assert torch.isfinite(do.float()).all()
    # row 0 of every (b, h) sees only key 0 => equals V row 0 exactly
    assert torch.equal(do[:, 0], dv[:, 0])
    # outputs are convex combinations of V rows: bounded by the running min/max of V along the sequence
    vmax = torch.cummax(dv.float(), dim=1).values
    vmin = torch.cummin(dv.float(), dim=1).values
    assert (do.float() <= vmax + 2e-2).all() and (do.float() >= vmin - 2e-2).all()
    rng = np.random.default_rng(2)
    rows = np.unique(np.concatenate([rng.integers(0, B * H * N, 384), [N - 1, B * H * N - 1, 127, 128, 4095]])).astype(np.int64)
    q, k, v = (t.float().cpu().numpy() for t in (dq, dk, dv))
    want = O.attention_rows(q, k, v, B, N, H, d, scale, rows, True)
    out = do.float().cpu().numpy()
    got = np.stack([out[r // (N * H), r % N, (r // N) % H] for r in rows])
    assert np.abs(got - want).max() <= 2e-2


@pytest.mark.parametrize("d,causal", [(128, True), (64, False)])
def test_headline_shape_fp32_sampled_rows(gpu, d, causal):
    """fp32 at the headline shape (B=4 N=4096 H=32), the fp32 matrix-core kernel at its real size: a seeded sample of
    rows against the oracle within 1e-4, and what holds for every output row (finite, inside the range of V)."""
    import torch
    from gpu_util import stream_ptr
    B, N, H = 4, 4096, 32
    g = torch.Generator(device="cuda").manual_seed(0xA77E0012)
    dq, dk, dv = (torch.randn((B, N, H, d), generator=g, device="cuda", dtype=torch.float32) for _ in range(3))
    do = torch.full_like(dq, float("nan"))
    scale = 1.0 / np.sqrt(d)
    gpu.flash_fwd(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), O.F32, B, N, H, d, (N * H * d, H * d, d),
                  scale, causal, stream_ptr())
    torch.cuda.synchronize()
    assert torch.isfinite(do).all()
    if causal:
        assert torch.equal(do[:, 0], dv[:, 0])   # row 0 sees only key 0
        vmax, vmin = torch.cummax(dv, dim=1).values, torch.cummin(dv, dim=1).values
    else:
        vmax, vmin = dv.amax(dim=1, keepdim=True), dv.amin(dim=1, keepdim=True)
    assert (do <= vmax + 1e-4).all() and (do >= vmin - 1e-4).all()
    rng = np.random.default_rng(12)
    rows = np.unique(np.concatenate([rng.integers(0, B * H * N, 256), [N - 1, B * H * N - 1, 127, 128, 4095]])).astype(np.int64)
    q, k, v = (t.cpu().numpy() for t in (dq, dk, dv))
    want = O.attention_rows(q, k, v, B, N, H, d, scale, rows, causal)
    out = do.cpu().numpy()
    got = np.stack([out[r // (N * H), r % N, (r // N) % H] for r in rows])
    assert np.abs(got - want).max() <= 1e-4


@pytest.mark.parametrize("dtype,d", [(O.F16, 64), (O.BF16, 128), (O.F32, 64), (O.F16, 32)])
@pytest.mark.parametrize("causal", [True, False])
def test_varlen_small(gpu, dtype, d, causal):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32
    H = 4
    lens = [5, 130, 1, 64, 257, 128]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    q, k, v = make_qkv((T, H, d), 11, dtype, sigma=0.5)
    dq, dk, dv = (to_dev(x, dtype) for x in (q, k, v))
    do = torch.full_like(dq, float("nan"))
    dcu = dev_i32(cu)
    scale = 1.0 / np.sqrt(d)
    gpu.flash_fwd_varlen(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), dtype, dcu.data_ptr(), len(lens),
                         max(lens), H, d, H * d, d, scale, causal, stream_ptr())
    torch.cuda.synchronize()
    got = to_host(do)
    want = O.attention_varlen(q, k, v, cu, H, d, scale, causal)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= (1e-4 if dtype == O.F32 else 2e-2)


def test_config5_varlen_fp16_causal_sampled_rows(gpu):
    # fp16 causal ragged batch: 16 sequences, lengths U[128, 8192], H=32, d=64, sigma = 0.5
    import torch
    from gpu_util import stream_ptr, dev_i32
    H, d = 32, 64
    lens = O.fill_lengths(16, 0xA77E0005, 4, 128, 8192)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    g = torch.Generator(device="cuda").manual_seed(0xA77E0005)
    dq, dk, dv = ((0.5 * torch.randn((T, H, d), generator=g, device="cuda", dtype=torch.float32)).to(torch.float16) for _ in range(3))
    do = torch.full_like(dq, float("nan"))
    dcu = dev_i32(cu)
    scale = 1.0 / np.sqrt(d)
    gpu.flash_fwd_varlen(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), O.F16, dcu.data_ptr(), 16,
                         int(lens.max()), H, d, H * d, d, scale, True, stream_ptr())
    torch.cuda.synchronize()
    assert torch.isfinite(do.float()).all()
    # first token of every sequence sees only itself
    first = torch.from_numpy(cu[:-1].astype(np.int64)).cuda()
    assert torch.equal(do[first], dv[first])
    rng = np.random.default_rng(5)
    toks = np.concatenate([rng.integers(0, T, 300), cu[1:] - 1, cu[:-1]])
    rows = (toks.astype(np.int64) * H + rng.integers(0, H, toks.size)).astype(np.int64)
    q, k, v = (t.float().cpu().numpy() for t in (dq, dk, dv))
    want = O.attention_varlen_rows(q, k, v, cu, H, d, scale, rows, True)
    out = do.float().cpu().numpy()
    got = np.stack([out[r // H, r % H] for r in rows])
    assert np.abs(got - want).max() <= 2e-2


def test_bad_arguments_are_rejected_without_launch(gpu):
    import torch
    x = torch.zeros(2 * 16 * 4 * 64, device="cuda")
    p = x.data_ptr()
    with pytest.raises(gpu.HipError):
        gpu.flash_fwd(0, p, p, p, O.F32, 2, 16, 4, 64, (16 * 4 * 64, 4 * 64, 64), 0.1, False)
    with pytest.raises(gpu.HipError):
        gpu.flash_fwd(p, p, p, p, 7, 2, 16, 4, 64, (16 * 4 * 64, 4 * 64, 64), 0.1, False)
    with pytest.raises(gpu.HipError):
        gpu.flash_fwd(p, p, p, p, O.F32, 2, 0, 4, 64, (16 * 4 * 64, 4 * 64, 64), 0.1, False)
    with pytest.raises(gpu.HipError):
        gpu.flash_fwd(p, p, p, p, O.F32, 2, 16, 4, 512, (16 * 4 * 512, 4 * 512, 512), 0.1, False)
    torch.cuda.synchronize()
