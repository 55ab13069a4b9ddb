"""Pins the oracle's 16-bit conversions, block-table index math, pool model and paged decode."""
import numpy as np
import pytest

from oracle import oracle as O


def test_f16_all_patterns_roundtrip_and_numpy_agreement():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    ours = np.array([O.lib.ahpc_oracle_f16_to_f32(int(b)) for b in bits], np.float32)
    theirs = bits.view(np.float16).astype(np.float32)
    same = (ours == theirs) | (np.isnan(ours) & np.isnan(theirs))
    assert same.all()
    back = np.array([O.lib.ahpc_oracle_f32_to_f16(float(x)) for x in theirs], np.uint16)
    ok = (back == bits) | np.isnan(theirs)
    assert ok.all()


def test_f32_to_f16_rne_against_numpy():
    rng = np.random.default_rng(1)
    # random bit patterns cover normals, subnormals, overflow and ties
    u = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    # add exact ties and boundaries
    extra = np.array([0x33000000, 0x33000001, 0x32FFFFFF, 0x38800000, 0x387FFFFF, 0x477FE000, 0x477FF000,
                      0x477FEFFF, 0x47800000, 0x7F800000, 0x00000001, 0x3F801000, 0x3F803000, 0x3F802000],
                     np.uint32)
    u = np.concatenate([u, extra, extra | 0x80000000])
    x = u.view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([O.lib.ahpc_oracle_f32_to_f16(float(v)) for v in x], np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    gotf = got[nan].view(np.float16)
    assert np.isnan(gotf).all()


def test_bf16_rne_closed_form():
    rng = np.random.default_rng(2)
    u = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    extra = np.array([0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0x7F7FFFFF, 0x7F800000], np.uint32)
    u = np.concatenate([u, extra, extra | 0x80000000])
    x = u.view(np.float32)
    got = np.array([O.lib.ahpc_oracle_f32_to_bf16(float(v)) for v in x], np.uint16)
    # closed form in float64: nearest multiple of 2^(e-7), ties to even mantissa
    nan = np.isnan(x)
    lo = (u >> 16).astype(np.uint32)
    rem = u & 0xFFFF
    up = (rem > 0x8000) | ((rem == 0x8000) & ((lo & 1) == 1))
    want = (lo + up.astype(np.uint32)).astype(np.uint16)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(O.from_bits16(got[nan], O.BF16)).all()
    # every bf16 pattern survives a round trip
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = O.from_bits16(bits, O.BF16)
    back = np.array([O.lib.ahpc_oracle_f32_to_bf16(float(v)) for v in f], np.uint16)
    assert ((back == bits) | np.isnan(f)).all()


def test_round_inplace_idempotent():
    x = O.fill_normal((1000,), 3, 1)
    for dt in (O.F16, O.BF16):
        y = O.round_to(x, dt)
        assert np.array_equal(O.round_to(y, dt), y)
        assert np.abs(y - x).max() < (1e-3 if dt == O.F16 else 8e-3) * max(1.0, np.abs(x).max())
        assert np.array_equal(O.from_bits16(O.to_bits16(y, dt), dt), y)


def test_kv_offset_bruteforce_tiny_pool():
    P, H, d = 4, 2, 8
    table = np.array([[3, 0, -1], [1, 2, 4]], np.int32)
    for row in range(2):
        for t in range(12):
            for h in range(H):
                page = table[row, t // P]
                want = -1 if page < 0 else ((page * P + t % P) * H + h) * d
                assert O.kv_offset(table, row, t, h, P, H, d) == want
    lens = np.array([7, 12], np.int32)
    offs = O.gather_offsets(table, lens, None, 2, 12, P, H, d)
    assert offs[0, 7:].tolist() == [-1] * 5
    assert offs[0, 5] == ((0 * P + 1) * H) * d
    offs2 = O.gather_offsets(table, lens, np.array([1, 0], np.int32), 2, 12, P, H, d)
    assert np.array_equal(offs2[0], offs[1]) and np.array_equal(offs2[1], offs[0])


def test_scatter_gather_roundtrip():
    P, H, d = 4, 3, 8
    n_pages = 10
    table = np.array([[7, 2, 9, 0]], np.int32)
    kp = np.zeros(n_pages * P * H * d, np.float32)
    vp = np.zeros_like(kp)
    k1 = O.fill_normal((6, H, d), 1, 2)
    v1 = O.fill_normal((6, H, d), 1, 3)
    k2 = O.fill_normal((9, H, d), 2, 2)
    v2 = O.fill_normal((9, H, d), 2, 3)
    O.kv_scatter(k1, v1, kp, vp, table, 0, 0, P, H, d)
    O.kv_scatter(k2, v2, kp, vp, table, 0, 6, P, H, d)
    kg, vg = O.kv_gather(kp, vp, table, 0, 0, 15, P, H, d)
    assert np.array_equal(kg, np.concatenate([k1, k2])) and np.array_equal(vg, np.concatenate([v1, v2]))
    kg, vg = O.kv_gather(kp, vp, table, 0, 5, 4, P, H, d)
    assert np.array_equal(kg, np.concatenate([k1, k2])[5:9])
    # pages the table does not name stay untouched
    pool = kp.reshape(n_pages, -1)
    assert np.all(pool[[1, 3, 4, 5, 6, 8]] == 0)


def test_pool_fifo_order():
    # src/algorithms/paged_attention.cpp:11-64: ids ascend on first use, freed pages recycle FIFO,
    # an empty queue grows by `grow`
    p = O.Pool(4, 2)
    assert [p.allocate() for _ in range(4)] == [0, 1, 2, 3]
    p.release(2)
    p.release(0)
    assert p.free == 2
    assert [p.allocate() for _ in range(2)] == [2, 0]
    assert p.allocate() == 4 and p.total == 6 and p.free == 1
    p.release(9)  # unknown page ignored
    p.release(3)
    p.release(3)  # double free ignored
    assert [p.allocate(), p.allocate()] == [5, 3]
    fixed = O.Pool(2, 0)
    assert [fixed.allocate() for _ in range(3)] == [0, 1, -1]


def _paged_problem(B, H, d, P, lens, seed, n_pages=None, shuffle=True):
    lens = np.asarray(lens, np.int32)
    pages_per = (lens + P - 1) // P
    max_pages = int(pages_per.max())
    total = int(pages_per.sum())
    n_pages = n_pages or total + 3
    ids = O.permutation(n_pages, seed, 5) if shuffle else np.arange(n_pages, dtype=np.int32)
    table = np.full((B, max_pages), -1, np.int32)
    c = 0
    for b in range(B):
        table[b, :pages_per[b]] = ids[c:c + pages_per[b]]
        c += pages_per[b]
    kp = np.zeros(n_pages * P * H * d, np.float32)
    vp = np.zeros_like(kp)
    ks, vs = [], []
    for b in range(B):
        kb = O.fill_normal((lens[b], H, d), seed + b, 2)
        vb = O.fill_normal((lens[b], H, d), seed + b, 3)
        O.kv_scatter(kb, vb, kp, vp, table, b, 0, P, H, d)
        ks.append(kb)
        vs.append(vb)
    q = O.fill_normal((B, H, d), seed, 1)
    return q, kp, vp, table, lens, ks, vs


def test_paged_decode_equals_dense_last_row_and_page_permutation_is_bit_invariant():
    B, H, d, P = 3, 2, 16, 4
    lens = [9, 1, 16]
    scale = 0.25
    q, kp, vp, table, lens_a, ks, vs = _paged_problem(B, H, d, P, lens, 77, shuffle=True)
    got = O.paged_decode(q, kp, vp, table, lens_a, None, B, H, d, P, scale)
    for b in range(B):
        L = lens[b]
        qq = np.zeros((1, L, H, d), np.float32)
        qq[0, -1] = q[b]
        want = O.attention(qq, ks[b][None], vs[b][None], 1, L, H, d, scale, True)[0, -1]
        assert np.array_equal(got[b], want)
    # identity table gives the same bits
    q2, kp2, vp2, table2, _, _, _ = _paged_problem(B, H, d, P, lens, 77, shuffle=False)
    got2 = O.paged_decode(q2, kp2, vp2, table2, lens_a, None, B, H, d, P, scale)
    assert np.array_equal(got, got2)
    # batch order indirection
    rows = np.array([2, 0, 1], np.int32)
    got3 = O.paged_decode(q[rows], kp, vp, table, lens_a, rows, B, H, d, P, scale)
    assert np.array_equal(got3, got[rows])


def test_paged_decode_empty_sequence_is_zero():
    B, H, d, P = 2, 2, 8, 4
    q, kp, vp, table, lens, _, _ = _paged_problem(B, H, d, P, [5, 3], 5)
    lens = lens.copy()
    lens[1] = 0
    out = O.paged_decode(q, kp, vp, table, lens, None, B, H, d, P, 0.3)
    assert np.all(out[1] == 0) and np.any(out[0] != 0)


def _reference_page_walk(table_row, L, P):
    """The key positions the reference decode kernel visits for one sequence: its loop over pages, written out in
    Python statement by statement (src/backends/cuda/cuda_kernels.cu:417-427; decode = the query is the last token)."""
    visited = []
    num_pages = (L + P - 1) // P
    for page_idx in range(num_pages):
        page_id = int(table_row[page_idx])
        if page_id < 0:
            break
        page_start = page_idx * P
        page_end = min(page_start + P, L)
        for k_idx in range(page_end - page_start):
            visited.append((page_id, k_idx))
    return visited


def test_missing_page_ends_the_sequence_as_the_reference_page_walk_does():
    P, H, d = 4, 2, 8
    table = np.array([[3, 0, -1, 5, 6], [-1, 2, 4, 1, 7], [1, 2, 4, 7, -1], [6, -1, -1, 2, 3]], np.int32)
    lens = np.array([18, 9, 16, 20], np.int32)
    for row in range(4):
        walk = _reference_page_walk(table[row], int(lens[row]), P)
        assert O.attended_tokens(table, row, int(lens[row]), P) == len(walk)
    assert [O.attended_tokens(table, r, int(lens[r]), P) for r in range(4)] == [8, 0, 16, 4]
    offs = O.gather_offsets(table, lens, None, 4, 20, P, H, d)
    for row in range(4):
        walk = _reference_page_walk(table[row], int(lens[row]), P)
        want = [((pg * P + slot) * H) * d for pg, slot in walk] + [-1] * (20 - len(walk))
        assert offs[row].tolist() == want
    # the decode attends to exactly those tokens: same bits as a sequence truncated there; page 0 .. are poisoned with
    # NaN wherever the walk does not go
    n_pages = 8
    kp = O.fill_normal((n_pages * P * H * d,), 9, 2)
    vp = O.fill_normal((n_pages * P * H * d,), 9, 3)
    q = O.fill_normal((4, H, d), 9, 1)
    got = O.paged_decode(q, kp, vp, table, lens, None, 4, H, d, P, 0.3)
    cut = np.array([8, 0, 16, 4], np.int32)
    clean = np.where(table < 0, 0, table).astype(np.int32)
    want = O.paged_decode(q, kp, vp, clean, cut, None, 4, H, d, P, 0.3)
    assert np.array_equal(got, want)
    assert np.all(got[1] == 0.0)


def test_generators_are_reproducible_and_sane():
    a = O.fill_normal((100000,), 0xA77E0002, 1)
    b = O.fill_normal((100000,), 0xA77E0002, 1)
    c = O.fill_normal((100000,), 0xA77E0002, 2)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    assert abs(a.mean()) < 0.02 and abs(a.std() - 1.0) < 0.02
    h = O.fill_normal((100000,), 4, 1, 0.5)
    assert abs(h.std() - 0.5) < 0.01
    L = O.fill_lengths(10000, 3, 4, 512, 4096)
    assert L.min() >= 512 and L.max() <= 4096 and abs(L.mean() - 2304) < 60
    p = O.permutation(1000, 3, 5)
    assert sorted(p.tolist()) == list(range(1000)) and p.tolist() != list(range(1000))
