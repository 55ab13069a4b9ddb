"""Element offsets beyond 4 GiB, on the CPU executor: a batch or head stride, or a page id, that puts part of
a tensor further than 2^32 bytes from its base pointer.  The buffers are sparse anonymous mappings (address
space only; just the pages the test touches are ever backed by memory), so the shapes stay tiny while every
address the kernels form for the far part needs more than 32 bits.  An offset computed in 32 bits lands in
the untouched (zero) part of a mapping or outside it: wrong results or a fault here, not on a GPU."""
import mmap

import numpy as np
import pytest

from oracle import oracle as O
from simt import simt as S

TOL = {O.F32: 1e-4, O.F16: 2e-2, O.BF16: 2e-2}
NP_OF = {O.F32: np.float32, O.F16: np.float16, O.BF16: np.uint16}
_MAP_NORESERVE = 0x4000

_keep = []  # the mappings live as long as the views on them


@pytest.fixture(scope="module")
def emu():
    S.load()
    S.configure(False, 1)
    return S.EmulatedHip()


def sparse(n_elems, dtype):
    """n_elems of storage type `dtype`, all zero, none of it resident until touched."""
    nbytes = int(n_elems) * np.dtype(NP_OF[dtype]).itemsize
    nbytes = (nbytes + mmap.PAGESIZE - 1) // mmap.PAGESIZE * mmap.PAGESIZE
    m = mmap.mmap(-1, nbytes, flags=mmap.MAP_PRIVATE | mmap.MAP_ANONYMOUS | _MAP_NORESERVE)
    _keep.append(m)
    return np.frombuffer(m, dtype=NP_OF[dtype], count=int(n_elems))


def place(buf, x, dtype, strides):
    """Writes the dense fp32 array x [B,N,H,d] into buf at element strides (b, n, h)."""
    s = S.to_storage(x, dtype).reshape(x.shape)
    B, N, H, d = x.shape
    for b in range(B):
        for h in range(H):
            for n in range(N):
                o = b * strides[0] + n * strides[1] + h * strides[2]
                buf[o:o + d] = s[b, n, h]


def pick(buf, shape, dtype, strides):
    B, N, H, d = shape
    out = np.empty(shape, np.float32)
    for b in range(B):
        for h in range(H):
            for n in range(N):
                o = b * strides[0] + n * strides[1] + h * strides[2]
                out[b, n, h] = S.from_storage(buf[o:o + d], dtype)
    return out


def far_strides(kind, N, H, d, itemsize):
    """(b, n, h) element strides with the second batch entry, or the second head, 4 GiB and a bit away."""
    far = (1 << 32) // itemsize + 8 * d
    if kind == "batch":
        return (far, H * d, d)
    return (2 * far, d, far)  # head-major layout, heads far apart


@pytest.mark.parametrize("kind", ["batch", "head"])
@pytest.mark.parametrize("dtype,d,causal", [(O.BF16, 128, True), (O.F16, 64, False), (O.F32, 128, True), (O.F32, 40, False),
                                            (O.F32, 256, True)])
def test_forward_and_backward_with_strides_beyond_4_gib(emu, kind, dtype, d, causal):
    B, N, H = 2, 70, 2
    item = np.dtype(NP_OF[dtype]).itemsize
    st = far_strides(kind, N, H, d, item)
    span = (B - 1) * st[0] + (N - 1) * st[1] + (H - 1) * st[2] + d
    q, k, v, do = (O.round_to(O.fill_normal((B, N, H, d), 91, t), dtype) for t in (1, 2, 3, 7))
    bq, bk, bv, bdo, bo, gq, gk, gv = (sparse(span, dtype) for _ in range(8))
    for buf, x in ((bq, q), (bk, k), (bv, v), (bdo, do)):
        place(buf, x, dtype, st)
    scale = 1.0 / np.sqrt(d)
    emu.flash_fwd(S.ptr(bq), S.ptr(bk), S.ptr(bv), S.ptr(bo), dtype, B, N, H, d, st, scale, causal)
    got = pick(bo, (B, N, H, d), dtype, st)
    assert np.abs(got - O.attention(q, k, v, B, N, H, d, scale, causal)).max() <= TOL[dtype]

    ws_bytes = emu.flash_bwd_workspace_bytes(B, N, H)
    ws = S.guarded(np.full(ws_bytes // 4, np.nan, np.float32))
    emu.flash_bwd(S.ptr(bdo), S.ptr(bq), S.ptr(bk), S.ptr(bv), S.ptr(gq), S.ptr(gk), S.ptr(gv), dtype, B, N, H, H, d, st, st,
                  scale, causal, S.ptr(ws), ws_bytes, None, None)
    want = O.attention_backward(q, k, v, do, B, N, H, d, scale, causal)
    for name, buf, w in zip(("dQ", "dK", "dV"), (gq, gk, gv), want):
        g = pick(buf, (B, N, H, d), dtype, st)
        bar = (1e-4 if dtype == O.F32 else 2e-2) * max(1.0, np.abs(w).max())
        assert np.abs(g - w.reshape(B, N, H, d)).max() <= bar, name


@pytest.mark.parametrize("dtype,H,H_kv,d", [(O.F16, 4, 4, 128), (O.BF16, 8, 2, 64), (O.F32, 2, 2, 96), (O.F16, 16, 1, 128)])
def test_pool_pages_beyond_4_gib(emu, dtype, H, H_kv, d):
    """Scatter, gather, the index dump and decode on pages whose byte offset in the pool needs more than 32 bits."""
    P, B = 16, 2
    item = np.dtype(NP_OF[dtype]).itemsize
    page_elems = P * H_kv * d
    first_far = (1 << 32) // (page_elems * item) + 3          # first page id wholly beyond 4 GiB
    lens = np.array([70, 33], np.int32)
    ids = [first_far + 40, 2, first_far + 7, first_far + 1000, 5, first_far, 1, first_far + 999]
    table = np.full((B, 6), -1, np.int32)
    table[0, :5] = ids[:5]
    table[1, :3] = ids[5:]
    n_pages = max(ids) + 1
    kpool, vpool = sparse(n_pages * page_elems, dtype), sparse(n_pages * page_elems, dtype)
    dt, dl = S.guarded(table), S.guarded(lens)

    # the same tokens in a compact pool (pages renumbered 0..7) for the oracle
    remap = {pid: i for i, pid in enumerate(ids)}
    ctable = np.vectorize(lambda p: remap.get(int(p), -1))(table).astype(np.int32)
    ck, cv = np.zeros(len(ids) * page_elems, np.float32), np.zeros(len(ids) * page_elems, np.float32)
    for row in range(B):
        n = int(lens[row])
        kn, vn = (O.round_to(O.fill_normal((n, H_kv, d), 40 + row, t), dtype) for t in (2, 3))
        O.kv_scatter(kn, vn, ck, cv, ctable, row, 0, P, H_kv, d)
        a, b = S.guarded(S.to_storage(kn, dtype)), S.guarded(S.to_storage(vn, dtype))
        emu.kv_scatter(S.ptr(a), S.ptr(b), dtype, S.ptr(kpool), S.ptr(vpool), dtype, S.ptr(dt), table.shape[1], n, H_kv, d, P,
                       row0=row, pos0=0)
    # what the scatter wrote, page by page, straight from the sparse pool
    for pid, i in remap.items():
        for pool, cpool in ((kpool, ck), (vpool, cv)):
            got = S.from_storage(pool[pid * page_elems:(pid + 1) * page_elems], dtype)
            assert np.array_equal(got, cpool[i * page_elems:(i + 1) * page_elems]), pid

    # gather reads them back
    for row in range(B):
        n = int(lens[row])
        ko, vo = S.guarded(np.empty(n * H_kv * d, np.float32)), S.guarded(np.empty(n * H_kv * d, np.float32))
        emu.kv_gather(S.ptr(ko), S.ptr(vo), O.F32, S.ptr(kpool), S.ptr(vpool), dtype, S.ptr(dt), table.shape[1], row, 0, n,
                      H_kv, d, P)
        want_k = np.empty(n * H_kv * d, np.float32)
        for t in range(n):
            src = (ctable[row, t // P] * P + t % P) * H_kv * d
            want_k[t * H_kv * d:(t + 1) * H_kv * d] = ck[src:src + H_kv * d]
        assert np.array_equal(ko, want_k)

    # the offsets decode reads at, bit for bit
    max_len = int(lens.max())
    out = S.guarded(np.full((B, max_len), -7, np.int64))
    emu.paged_gather_indices(S.ptr(dt), S.ptr(dl), None, B, H_kv, d, P, table.shape[1], max_len, S.ptr(out))
    want_off = O.gather_offsets(table, lens, None, B, max_len, P, H_kv, d)
    assert np.array_equal(out, want_off) and int(want_off.max()) * item > (1 << 32)

    # decode, whole and in chunks
    q = O.round_to(O.fill_normal((B, H, d), 44, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    G = H // H_kv
    want = np.empty((B, H, d), np.float32)
    for g in range(G):  # the oracle decodes ungrouped heads: query head h reads pool head h // G
        sel = np.arange(H_kv) * G + g
        want[:, sel] = O.paged_decode(np.ascontiguousarray(q[:, sel]), ck, cv, ctable, lens, None, B, H_kv, d, P, scale)
    dq = S.guarded(S.to_storage(q, dtype))
    for chunk in (0, 2 * P):
        do = S.guarded(S.empty_storage((B, H, d), dtype))
        ws_bytes = emu.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
        ws = S.guarded(np.full(max(ws_bytes, 4) // 4, np.nan, np.float32))
        emu.paged_decode_gqa(S.ptr(dq), S.ptr(do), dtype, S.ptr(kpool), S.ptr(vpool), dtype, S.ptr(dt), S.ptr(dl), None, B, H,
                             H_kv, d, P, table.shape[1], max_len, scale, chunk, S.ptr(ws), ws_bytes)
        got = S.from_storage(do, dtype)
        assert np.abs(got - want).max() <= TOL[dtype], chunk
