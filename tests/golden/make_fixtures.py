"""Writes the known-answer vectors of tests/golden/*.npz.

The reference holds no golden vectors for this path (every test input comes from std::random_device), so these are
made here: inputs from the seeded generator the oracle and the GPU tests share (oracle.fill_*, a counter-based
generator, so only seeds are stored), expected outputs from a float64 numpy computation written independently of
oracle/oracle.c (no code shared with it).  tests/test_golden_vectors.py checks the oracle, and the kernels on the
CPU executor, against them.  Run:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as O  # noqa: E402  (input generator only)


def softmax64(s):
    top = s.max(axis=-1, keepdims=True)
    top = np.where(np.isfinite(top), top, 0.0)
    e = np.exp(s - top)
    tot = e.sum(axis=-1, keepdims=True)
    return np.where(tot > 0, e / np.where(tot > 0, tot, 1.0), 0.0)


def scores64(q, k, scale, causal, mask):
    B, N, H, d = q.shape
    g = H // k.shape[2]
    s = np.empty((B, H, N, N))
    for h in range(H):
        s[:, h] = scale * np.einsum("bid,bjd->bij", q[:, :, h].astype(np.float64), k[:, :, h // g].astype(np.float64))
    if causal:
        s = np.where(np.tril(np.ones((N, N), bool))[None, None], s, -np.inf)
    if mask is not None:
        s = np.where(mask[:, None] != 0, s, -np.inf)
    return s


def forward64(q, k, v, scale, causal, mask=None):
    g = q.shape[2] // k.shape[2]
    p = softmax64(scores64(q, k, scale, causal, mask))
    vv = np.repeat(v.astype(np.float64), g, axis=2)
    return np.einsum("bhij,bjhd->bihd", p, vv)


def backward64(q, k, v, do, scale, causal, mask=None):
    B, N, H, d = q.shape
    Hkv = k.shape[2]
    g = H // Hkv
    p = softmax64(scores64(q, k, scale, causal, mask))
    vv = np.repeat(v.astype(np.float64), g, axis=2)
    kk = np.repeat(k.astype(np.float64), g, axis=2)
    do64 = do.astype(np.float64)
    dp = np.einsum("bihd,bjhd->bhij", do64, vv)
    ds = p * (dp - (p * dp).sum(axis=-1, keepdims=True))
    dq = scale * np.einsum("bhij,bjhd->bihd", ds, kk)
    dk = scale * np.einsum("bhij,bihd->bjhd", ds, q.astype(np.float64))
    dv = np.einsum("bhij,bihd->bjhd", p, do64)
    fold = lambda x: x.reshape(B, N, Hkv, g, d).sum(axis=3)
    return dq, fold(dk), fold(dv)


def decode64(q, k_rows, v_rows, scale):
    """q [H,d]; k_rows, v_rows [L,H_kv,d] in token order."""
    H, d = q.shape
    g = H // k_rows.shape[1]
    out = np.zeros((H, d))
    for h in range(H):
        s = scale * k_rows[:, h // g].astype(np.float64) @ q[h].astype(np.float64)
        p = softmax64(s[None])[0]
        out[h] = p @ v_rows[:, h // g].astype(np.float64)
    return out


def main():
    cases = {}
    # dense forward and backward: (B, N, H, H_kv, d, causal, with_mask, seed)
    for name, (B, N, H, Hkv, d, causal, with_mask, seed) in {
        "dense_reference_fixture_shape": (2, 16, 4, 4, 64, False, False, 0x601),   # tests/test_flash_attention.cpp:103-108
        "dense_causal": (1, 16, 4, 4, 64, True, False, 0x602),
        "dense_causal_grouped_heads": (1, 24, 6, 2, 32, True, False, 0x603),
        "dense_masked": (1, 20, 2, 2, 16, False, True, 0x604),
    }.items():
        q = O.fill_uniform((B, N, H, d), seed, 1)
        k = O.fill_uniform((B, N, Hkv, d), seed, 2)
        v = O.fill_uniform((B, N, Hkv, d), seed, 3)
        do = O.fill_uniform((B, N, H, d), seed, 7)
        mask = None
        if with_mask:
            mask = (O.fill_uniform((B, N, N), seed, 6) > -0.4).astype(np.float32)
            mask[0, 3, :] = 0.0  # a row that sees nothing
        scale = float(1.0 / np.sqrt(d))
        o = forward64(q, k, v, scale, causal, mask)
        dq, dk, dv = backward64(q, k, v, do, scale, causal, mask)
        cases[name] = dict(kind="dense", shape=np.array([B, N, H, Hkv, d]), causal=causal, with_mask=with_mask, seed=seed,
                           scale=scale, o=o.astype(np.float32))
        if name != "dense_reference_fixture_shape":  # forward only at the largest shape: keeps the files small
            cases[name].update(dq=dq.astype(np.float32), dk=dk.astype(np.float32), dv=dv.astype(np.float32))
    # paged decode: tokens of each sequence scattered over shuffled pages
    for name, (lens, H, Hkv, d, P, seed) in {
        "decode_shuffled_pages": ([33, 1, 16, 70], 4, 4, 32, 16, 0x611),
        "decode_grouped_heads_small_pages": ([9, 30], 8, 2, 64, 4, 0x612),
    }.items():
        lens = np.array(lens, np.int32)
        scale = float(1.0 / np.sqrt(d))
        q = O.fill_normal((len(lens), H, d), seed, 1)
        outs = []
        for b, n in enumerate(lens):
            kb = O.fill_normal((int(n), Hkv, d), seed + 10 + b, 2)
            vb = O.fill_normal((int(n), Hkv, d), seed + 10 + b, 3)
            outs.append(decode64(q[b], kb, vb, scale))
        cases[name] = dict(kind="decode", lens=lens, shape=np.array([H, Hkv, d, P]), seed=seed, scale=scale,
                           o=np.stack(outs).astype(np.float32))
    for name, c in cases.items():
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **c)
        print(name, os.path.getsize(os.path.join(HERE, name + ".npz")), "bytes")


if __name__ == "__main__":
    main()
