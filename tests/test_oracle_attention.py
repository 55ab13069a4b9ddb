"""Pins the dense / ragged attention oracle without the reference's (uncompilable) code:
float64 brute force, closed forms and invariances named in oracle/oracle.c."""
import numpy as np
import pytest

from oracle import oracle as O


def brute_f64(q, k, v, scale, causal, mask=None):
    """q,k,v: [B,N,H,d] float64 brute force, independent of the oracle's loop structure."""
    B, N, H, d = q.shape
    out = np.zeros_like(q, dtype=np.float64)
    for b in range(B):
        for h in range(H):
            s = (q[b, :, h, :].astype(np.float64) @ k[b, :, h, :].astype(np.float64).T) * scale
            if causal:
                s = np.where(np.tril(np.ones((N, N), bool)), s, -np.inf)
            if mask is not None:
                s = np.where(mask[b] == 0.0, -np.inf, s)
            m = s.max(axis=1, keepdims=True)
            dead = ~np.isfinite(m)
            m = np.where(dead, 0.0, m)
            p = np.exp(s - m)
            den = p.sum(axis=1, keepdims=True)
            p = np.where(den > 0, p / np.where(den > 0, den, 1.0), 0.0)
            out[b, :, h, :] = p @ v[b, :, h, :].astype(np.float64)
    return out


@pytest.mark.parametrize("B,N,H,d", [(2, 16, 4, 64), (1, 1, 2, 16), (2, 33, 3, 32), (1, 128, 2, 128)])
@pytest.mark.parametrize("causal", [False, True])
def test_dense_matches_float64_bruteforce(B, N, H, d, causal):
    # (2,16,4,64) is the reference fixture shape, tests/test_flash_attention.cpp:103-106
    q = O.fill_uniform((B, N, H, d), 11, 1)
    k = O.fill_uniform((B, N, H, d), 11, 2)
    v = O.fill_uniform((B, N, H, d), 11, 3)
    scale = 1.0 / np.sqrt(d)
    got = O.attention(q, k, v, B, N, H, d, scale, causal)
    want = brute_f64(q, k, v, scale, causal)
    assert np.abs(got - want).max() < 2e-6


def test_layout_switch_is_a_transpose():
    B, N, H, d = 2, 9, 3, 16
    q, k, v = (O.fill_normal((B, N, H, d), 5, t) for t in (1, 2, 3))
    a = O.attention(q, k, v, B, N, H, d, 0.25, True, layout="BNHD")
    tq, tk, tv = (np.ascontiguousarray(x.transpose(0, 2, 1, 3)) for x in (q, k, v))
    b = O.attention(tq, tk, tv, B, N, H, d, 0.25, True, layout="BHND")
    assert np.array_equal(a, b.transpose(0, 2, 1, 3))


def test_dense_mask_matches_bruteforce_and_dead_rows_are_zero():
    B, N, H, d = 2, 12, 2, 16
    q, k, v = (O.fill_normal((B, N, H, d), 7, t) for t in (1, 2, 3))
    rng = np.random.default_rng(3)
    mask = (rng.random((B, N, N)) > 0.4).astype(np.float32)
    mask[0, 5, :] = 0.0  # fully masked row
    got = O.attention(q, k, v, B, N, H, d, 0.3, False, mask=mask)
    want = brute_f64(q, k, v, 0.3, False, mask)
    assert np.abs(got - want).max() < 2e-6
    assert np.all(got[0, 5] == 0.0)


def test_closed_forms():
    B, N, H, d = 2, 24, 3, 32
    q, k, v = (O.fill_normal((B, N, H, d), 21, t) for t in (1, 2, 3))
    # V constant => O constant
    vc = np.full_like(v, 0.625)
    out = O.attention(q, k, vc, B, N, H, d, 0.2, False)
    assert np.abs(out - 0.625).max() < 1e-6
    # Q = 0 => uniform weights => mean of V (prefix mean when causal)
    z = np.zeros_like(q)
    out = O.attention(z, k, v, B, N, H, d, 0.2, False)
    assert np.abs(out - v.mean(axis=1, keepdims=True)).max() < 1e-6
    out = O.attention(z, k, v, B, N, H, d, 0.2, True)
    prefix = np.cumsum(v.astype(np.float64), axis=1) / np.arange(1, N + 1)[None, :, None, None]
    assert np.abs(out - prefix).max() < 1e-6
    # one dominant logit => that V row
    q1 = np.zeros_like(q)
    k1 = np.zeros_like(k)
    q1[..., 0] = 1.0
    k1[:, 7, :, 0] = 80.0
    out = O.attention(q1, k1, v, B, N, H, d, 1.0, False)
    assert np.abs(out - v[:, 7:8]).max() < 1e-6
    # N = 1 => O = V  (tests/test_flash_attention.cpp:585-588)
    out = O.attention(q[:, :1].copy(), k[:, :1].copy(), v[:, :1].copy(), B, 1, H, d, 0.2, True)
    assert np.array_equal(out, v[:, :1])


def test_key_permutation_invariance():
    B, N, H, d = 1, 40, 2, 16
    q, k, v = (O.fill_normal((B, N, H, d), 33, t) for t in (1, 2, 3))
    perm = np.random.default_rng(0).permutation(N)
    a = O.attention(q, k, v, B, N, H, d, 0.25, False)
    b = O.attention(q, np.ascontiguousarray(k[:, perm]), np.ascontiguousarray(v[:, perm]), B, N, H, d, 0.25, False)
    assert np.abs(a - b).max() < 1e-6


def test_rows_subset_equals_full():
    B, N, H, d = 2, 20, 3, 16
    q, k, v = (O.fill_normal((B, N, H, d), 8, t) for t in (1, 2, 3))
    full = O.attention(q, k, v, B, N, H, d, 0.25, True)
    rows = np.array([0, 7, 59, 119, 60], np.int64)
    got = O.attention_rows(q, k, v, B, N, H, d, 0.25, rows, True)
    for i, r in enumerate(rows):
        n, h, b = r % N, (r // N) % H, r // (N * H)
        assert np.array_equal(got[i], full[b, n, h])


def test_threads_do_not_change_bits():
    B, N, H, d = 2, 50, 4, 32
    q, k, v = (O.fill_normal((B, N, H, d), 9, t) for t in (1, 2, 3))
    a = O.attention(q, k, v, B, N, H, d, 0.17, True, threads=1)
    b = O.attention(q, k, v, B, N, H, d, 0.17, True, threads=4)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("causal", [False, True])
def test_varlen_equals_per_sequence_dense(causal):
    H, d = 3, 16
    lens = [5, 1, 17, 8]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    q, k, v = (O.fill_normal((T, H, d), 17, t) for t in (1, 2, 3))
    got = O.attention_varlen(q, k, v, cu, H, d, 0.25, causal)
    for i, L in enumerate(lens):
        s, e = cu[i], cu[i + 1]
        want = brute_f64(q[None, s:e], k[None, s:e], v[None, s:e], 0.25, causal)[0]
        assert np.abs(got[s:e] - want).max() < 2e-6
    rows = np.array([0, 4 * H + 2, (T - 1) * H + 1, 6 * H], np.int64)
    sub = O.attention_varlen_rows(q, k, v, cu, H, d, 0.25, rows, causal)
    for i, r in enumerate(rows):
        assert np.array_equal(sub[i], got[r // H, r % H])


def test_merge_rule_matches_direct_softmax():
    rng = np.random.default_rng(5)
    s = rng.normal(size=100).astype(np.float32) * 4
    m, l = -np.inf, 0.0
    for lo in range(0, 100, 13):
        blk = s[lo:lo + 13]
        bm = blk.max()
        m, l = O.softmax_merge(m, l, float(bm), float(np.exp(blk - bm).sum()))
    assert m == s.max()
    assert abs(l - np.exp(s.astype(np.float64) - s.max()).sum()) < 1e-4 * l
    # order of the two operands does not matter beyond rounding
    a = O.softmax_merge(1.0, 2.0, 3.0, 0.5)
    b = O.softmax_merge(3.0, 0.5, 1.0, 2.0)
    assert a[0] == b[0] and abs(a[1] - b[1]) < 1e-6
    # merging with the empty state is the identity
    assert O.softmax_merge(-np.inf, 0.0, 2.0, 3.0) == (2.0, 3.0)


@pytest.mark.parametrize("splits", [1, 2, 7])
def test_split_count_invariance(splits):
    L, d = 300, 64
    q = O.fill_normal((d,), 41, 1)
    k = O.fill_normal((L, d), 41, 2)
    v = O.fill_normal((L, d), 41, 3)
    got = O.attention_row_split(q, k, v, 0.125, splits)
    # q is a single row: compare against the last causal row of a dense problem whose last query is q
    qq = np.zeros((L, d), np.float32)
    qq[-1] = q
    want = O.attention(qq, k, v, 1, L, 1, d, 0.125, True).reshape(L, d)[-1]
    assert np.abs(got - want).max() < 2e-6
