"""Known-answer vectors (tests/golden/*.npz, written by tests/golden/make_fixtures.py from a float64 computation that
shares no code with the oracle) against the oracle and against the kernels on the CPU executor.  The reference itself
holds no golden vectors for this path: all its test inputs are unseeded random numbers."""
import glob
import os

import numpy as np
import pytest

from oracle import oracle as O
from simt import simt as S

HERE = os.path.dirname(os.path.abspath(__file__))
FILES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))


def load(path):
    with np.load(path, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def dense_inputs(c):
    B, N, H, Hkv, d = (int(x) for x in c["shape"])
    seed = int(c["seed"])
    q = O.fill_uniform((B, N, H, d), seed, 1)
    k = O.fill_uniform((B, N, Hkv, d), seed, 2)
    v = O.fill_uniform((B, N, Hkv, d), seed, 3)
    do = O.fill_uniform((B, N, H, d), seed, 7)
    mask = None
    if bool(c["with_mask"]):
        mask = (O.fill_uniform((B, N, N), seed, 6) > -0.4).astype(np.float32)
        mask[0, 3, :] = 0.0
    return (B, N, H, Hkv, d), q, k, v, do, mask


def test_fixtures_are_present():
    assert len(FILES) >= 6


@pytest.mark.parametrize("path", [f for f in FILES if "dense" in os.path.basename(f)], ids=os.path.basename)
def test_dense_vectors(path):
    c = load(path)
    (B, N, H, Hkv, d), q, k, v, do, mask = dense_inputs(c)
    scale, causal = float(c["scale"]), bool(c["causal"])
    g = H // Hkv
    # the oracle (its forward knows one K/V head per query head: repeated heads are the definition of grouped heads)
    o = O.attention(q, np.repeat(k, g, axis=2), np.repeat(v, g, axis=2), B, N, H, d, scale, causal, mask=mask)
    assert np.abs(o - c["o"]).max() <= 2e-6
    if "dq" in c:
        dq, dk, dv = O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, Hkv, mask)
        for got, name in ((dq, "dq"), (dk, "dk"), (dv, "dv")):
            assert np.abs(got - c[name]).max() <= 2e-6, name
    # the fp32 kernels on the CPU executor, through the C ABI
    S.load()
    emu = S.EmulatedHip()
    dev = lambda x: S.guarded(np.ascontiguousarray(x, np.float32))
    tq, tk, tv, tdo = dev(q), dev(k), dev(v), dev(do)
    to = S.guarded(np.full((B, N, H, d), np.nan, np.float32))
    tm = None if mask is None else dev(mask)
    sq, skv = (N * H * d, H * d, d), (N * Hkv * d, Hkv * d, d)
    emu.flash_fwd_gqa(S.ptr(tq), S.ptr(tk), S.ptr(tv), S.ptr(to), O.F32, B, N, H, Hkv, d, sq, skv, scale, causal, None,
                      None if tm is None else S.ptr(tm))
    assert np.abs(to - c["o"]).max() <= 1e-4
    if "dq" in c:
        gq = S.guarded(np.full((B, N, H, d), np.nan, np.float32))
        gk = S.guarded(np.full((B, N, Hkv, d), np.nan, np.float32))
        gv = S.guarded(np.full((B, N, Hkv, d), np.nan, np.float32))
        ws_bytes = emu.flash_bwd_workspace_bytes(B, N, H)
        ws = S.guarded(np.full(ws_bytes // 4, np.nan, np.float32))
        emu.flash_bwd(S.ptr(tdo), S.ptr(tq), S.ptr(tk), S.ptr(tv), S.ptr(gq), S.ptr(gk), S.ptr(gv), O.F32, B, N, H, Hkv, d, sq,
                      skv, scale, causal, S.ptr(ws), ws_bytes, None, None if tm is None else S.ptr(tm))
        for got, name in ((gq, "dq"), (gk, "dk"), (gv, "dv")):
            assert np.abs(got - c[name]).max() <= 1e-4, name


def decode_inputs(c):
    """Rebuilds the decode problem of a fixture: queries, the two pools (fp32, `Hkv` heads per token), block table, lengths."""
    H, Hkv, d, P = (int(x) for x in c["shape"])
    lens, seed = c["lens"].astype(np.int32), int(c["seed"])
    B = len(lens)
    q = O.fill_normal((B, H, d), seed, 1)
    pages_per = (lens + P - 1) // P
    n_pages = int(pages_per.sum()) + 3
    ids = O.permutation(n_pages, seed, 5)
    table = np.full((B, int(pages_per.max())), -1, np.int32)
    at = 0
    for b in range(B):
        table[b, :pages_per[b]] = ids[at:at + pages_per[b]]
        at += pages_per[b]
    kp, vp = np.zeros(n_pages * P * Hkv * d, np.float32), np.zeros(n_pages * P * Hkv * d, np.float32)
    for b, n in enumerate(lens):
        kb = O.fill_normal((int(n), Hkv, d), seed + 10 + b, 2)
        vb = O.fill_normal((int(n), Hkv, d), seed + 10 + b, 3)
        O.kv_scatter(kb, vb, kp, vp, table, b, 0, P, Hkv, d)
    return (B, H, Hkv, d, P), q, kp, vp, table, lens


@pytest.mark.parametrize("path", [f for f in FILES if "decode" in os.path.basename(f)], ids=os.path.basename)
def test_decode_vectors(path):
    c = load(path)
    (B, H, Hkv, d, P), q, kp, vp, table, lens = decode_inputs(c)
    scale, g = float(c["scale"]), H // Hkv
    rep = lambda pool: np.repeat(pool.reshape(-1, Hkv, d), g, axis=1).reshape(-1)
    o = O.paged_decode(q, rep(kp), rep(vp), table, lens, None, B, H, d, P, scale)
    assert np.abs(o - c["o"]).max() <= 2e-6
    S.load()
    emu = S.EmulatedHip()
    dq_, dk_, dv_ = S.guarded(q), S.guarded(kp), S.guarded(vp)
    do_ = S.guarded(np.full((B, H, d), np.nan, np.float32))
    dt, dl = S.guarded(table), S.guarded(lens)
    max_len = int(lens.max())
    ws_bytes = emu.paged_decode_workspace_bytes(B, H, d, max_len, P, P)
    ws = S.guarded(np.full(max(ws_bytes, 4) // 4, np.nan, np.float32))
    emu.paged_decode_gqa(S.ptr(dq_), S.ptr(do_), O.F32, S.ptr(dk_), S.ptr(dv_), O.F32, S.ptr(dt), S.ptr(dl), None, B, H, Hkv, d,
                         P, table.shape[1], max_len, scale, P, S.ptr(ws), ws_bytes)
    assert np.abs(do_ - c["o"]).max() <= 1e-4
