"""Grouped K/V heads have no implementation in the reference (AttentionParams::key_value_heads,
src/api/attention_interface.hpp:61, is read nowhere), so the GPU tests compare the grouped kernels with the
ordinary oracle fed K/V whose heads are repeated.  This file pins that yardstick itself: repeating heads and
running the oracle is the same as computing, in float64 and straight from the definition, attention where query
head h uses K/V head h // (H / H_kv) - and it is NOT the same as the other plausible convention (h % H_kv), so a
kernel that picked the wrong one would be caught."""
import numpy as np
import pytest

from oracle import oracle as O


def brute_force_gqa(q, k, v, scale, causal, pick):
    B, N, H, d = q.shape
    out = np.zeros((B, N, H, d))
    for b in range(B):
        for h in range(H):
            hk = pick(h)
            s = (q[b, :, h].astype(np.float64) @ k[b, :, hk].astype(np.float64).T) * scale
            if causal:
                s = np.where(np.tril(np.ones((N, N), bool)), s, -np.inf)
            p = np.exp(s - s.max(axis=1, keepdims=True))
            out[b, :, h] = (p / p.sum(axis=1, keepdims=True)) @ v[b, :, hk].astype(np.float64)
    return out


@pytest.mark.parametrize("H,Hkv", [(8, 2), (6, 3), (4, 1), (4, 4)])
@pytest.mark.parametrize("causal", [False, True])
def test_repeated_heads_equal_the_definition(H, Hkv, causal):
    B, N, d = 2, 19, 16
    g = H // Hkv
    q = O.fill_normal((B, N, H, d), 51, 1)
    k = O.fill_normal((B, N, Hkv, d), 51, 2)
    v = O.fill_normal((B, N, Hkv, d), 51, 3)
    scale = 0.25
    got = O.attention(q, np.ascontiguousarray(np.repeat(k, g, axis=2)), np.ascontiguousarray(np.repeat(v, g, axis=2)), B, N, H, d,
                      scale, causal)
    want = brute_force_gqa(q, k, v, scale, causal, lambda h: h // g)
    assert np.abs(got - want).max() <= 2e-6
    if 1 < Hkv < H:
        other = brute_force_gqa(q, k, v, scale, causal, lambda h: h % Hkv)
        assert np.abs(got - other).max() > 1e-2  # the interleaved convention gives a different answer


def test_repeated_pool_heads_equal_the_definition_for_decode():
    B, H, Hkv, d, P = 3, 8, 2, 32, 4
    g = H // Hkv
    lens = np.array([9, 1, 14], np.int32)
    pages = (lens + P - 1) // P
    n_pages = int(pages.sum())
    table = np.full((B, int(pages.max())), -1, np.int32)
    ids = O.permutation(n_pages, 52, 5)
    c = 0
    for b in range(B):
        table[b, :pages[b]] = ids[c:c + pages[b]]
        c += pages[b]
    kp = np.zeros(n_pages * P * Hkv * d, np.float32)
    vp = np.zeros_like(kp)
    ks, vs = [], []
    for b in range(B):
        kb, vb = O.fill_normal((int(lens[b]), Hkv, d), 60 + b, 2), O.fill_normal((int(lens[b]), Hkv, d), 60 + b, 3)
        O.kv_scatter(kb, vb, kp, vp, table, b, 0, P, Hkv, d)
        ks.append(kb)
        vs.append(vb)
    q = O.fill_normal((B, H, d), 52, 1)
    kx = np.ascontiguousarray(np.repeat(kp.reshape(-1, Hkv, d), g, axis=1)).reshape(-1)
    vx = np.ascontiguousarray(np.repeat(vp.reshape(-1, Hkv, d), g, axis=1)).reshape(-1)
    got = O.paged_decode(q, kx, vx, table, lens, None, B, H, d, P, 0.3)
    for b in range(B):
        for h in range(H):
            s = ks[b][:, h // g].astype(np.float64) @ q[b, h].astype(np.float64) * 0.3
            p = np.exp(s - s.max())
            want = (p / p.sum()) @ vs[b][:, h // g].astype(np.float64)
            assert np.abs(got[b, h] - want).max() <= 2e-6
