"""Element offsets beyond 4 GiB on the GPU: tensors whose second batch entry or second head, and pool pages whose
first byte, lie further than 2^32 bytes from the base pointer (a 288 GB part holds pools and batches of that size).
The allocations are real (a few GiB each, mostly untouched); the shapes that are computed stay small, so the oracle
checks every element.  The same cases run on the CPU executor first (test_simt_large_offsets.py), where an address
formed in 32 bits cannot fault a GPU."""
import numpy as np
import pytest

from oracle import oracle as O
from gpu_util import TOL, torch_dtype, to_host, stream_ptr, dev_i32

pytestmark = pytest.mark.gpu

ITEM = {O.F32: 4, O.F16: 2, O.BF16: 2}


def far_strides(kind, H, d, itemsize):
    far = (1 << 32) // itemsize + 8 * d
    if kind == "batch":
        return (far, H * d, d)
    return (2 * far, d, far)  # head-major layout, heads far apart


def strided(buf, shape, st):
    import torch
    return torch.as_strided(buf, shape, (st[0], st[1], st[2], 1))


@pytest.mark.parametrize("kind", ["batch", "head"])
@pytest.mark.parametrize("dtype,d,causal", [(O.BF16, 128, True), (O.F16, 64, False), (O.F32, 128, True), (O.F32, 40, False),
                                            (O.F32, 256, True)])
def test_forward_and_backward_with_strides_beyond_4_gib(gpu, kind, dtype, d, causal):
    import torch
    B, N, H = 2, 300, 2
    st = far_strides(kind, H, d, ITEM[dtype])
    span = (B - 1) * st[0] + (N - 1) * st[1] + (H - 1) * st[2] + d
    q, k, v, do = (O.round_to(O.fill_normal((B, N, H, d), 91, t), dtype) for t in (1, 2, 3, 7))
    td = torch_dtype(dtype)
    bufs = [torch.empty(span, dtype=td, device="cuda") for _ in range(8)]
    bq, bk, bv, bdo, bo, gq, gk, gv = bufs
    for buf, x in ((bq, q), (bk, k), (bv, v), (bdo, do)):
        strided(buf, (B, N, H, d), st).copy_(torch.from_numpy(x).to(td))
    for buf in (bo, gq, gk, gv):
        strided(buf, (B, N, H, d), st).fill_(float("nan"))
    scale = 1.0 / np.sqrt(d)
    print(f"large offsets: forward {kind} dtype={dtype} d={d} causal={causal}", flush=True)
    gpu.flash_fwd(bq.data_ptr(), bk.data_ptr(), bv.data_ptr(), bo.data_ptr(), dtype, B, N, H, d, st, scale, causal, stream_ptr())
    torch.cuda.synchronize()
    got = to_host(strided(bo, (B, N, H, d), st))
    assert np.abs(got - O.attention(q, k, v, B, N, H, d, scale, causal)).max() <= TOL[dtype]

    ws_bytes = gpu.flash_bwd_workspace_bytes(B, N, H)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device="cuda")
    print(f"large offsets: backward {kind} dtype={dtype} d={d} causal={causal}", flush=True)
    gpu.flash_bwd(bdo.data_ptr(), bq.data_ptr(), bk.data_ptr(), bv.data_ptr(), gq.data_ptr(), gk.data_ptr(), gv.data_ptr(),
                  dtype, B, N, H, H, d, st, st, scale, causal, ws.data_ptr(), ws_bytes, stream_ptr())
    torch.cuda.synchronize()
    want = O.attention_backward(q, k, v, do, B, N, H, d, scale, causal)
    for name, buf, w in zip(("dQ", "dK", "dV"), (gq, gk, gv), want):
        g = to_host(strided(buf, (B, N, H, d), st))
        bar = (1e-4 if dtype == O.F32 else 2e-2) * max(1.0, np.abs(w).max())
        assert np.abs(g - w.reshape(B, N, H, d)).max() <= bar, name
    del bufs, bq, bk, bv, bdo, bo, gq, gk, gv
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype,H,H_kv,d", [(O.F16, 4, 4, 128), (O.BF16, 8, 2, 64), (O.F32, 2, 2, 96), (O.F16, 16, 1, 128)])
def test_pool_pages_beyond_4_gib(gpu, dtype, H, H_kv, d):
    """Scatter, gather, the index dump and decode on pages whose byte offset in the pool needs more than 32 bits."""
    import torch
    P, B = 16, 2
    item = ITEM[dtype]
    td = torch_dtype(dtype)
    page_elems = P * H_kv * d
    first_far = (1 << 32) // (page_elems * item) + 3
    lens = np.array([70, 33], np.int32)
    ids = [first_far + 40, 2, first_far + 7, first_far + 1000, 5, first_far, 1, first_far + 999]
    table = np.full((B, 6), -1, np.int32)
    table[0, :5] = ids[:5]
    table[1, :3] = ids[5:]
    n_pages = max(ids) + 1
    kpool = torch.empty(n_pages * page_elems, dtype=td, device="cuda")
    vpool = torch.empty_like(kpool)
    dt, dl = dev_i32(table), dev_i32(lens)

    remap = {pid: i for i, pid in enumerate(ids)}
    ctable = np.vectorize(lambda p: remap.get(int(p), -1))(table).astype(np.int32)
    ck, cv = np.zeros(len(ids) * page_elems, np.float32), np.zeros(len(ids) * page_elems, np.float32)
    for pid in ids:  # the pages start as zeros, as in the compact pool
        kpool[pid * page_elems:(pid + 1) * page_elems].zero_()
        vpool[pid * page_elems:(pid + 1) * page_elems].zero_()
    print(f"large offsets: pool dtype={dtype} H={H} H_kv={H_kv} d={d} first far page {first_far}", flush=True)
    for row in range(B):
        n = int(lens[row])
        kn, vn = (O.round_to(O.fill_normal((n, H_kv, d), 40 + row, t), dtype) for t in (2, 3))
        O.kv_scatter(kn, vn, ck, cv, ctable, row, 0, P, H_kv, d)
        a, b = torch.from_numpy(kn).to(td).cuda(), torch.from_numpy(vn).to(td).cuda()
        gpu.kv_scatter(a.data_ptr(), b.data_ptr(), dtype, kpool.data_ptr(), vpool.data_ptr(), dtype, dt.data_ptr(), table.shape[1],
                       n, H_kv, d, P, row0=row, pos0=0, stream=stream_ptr())
    torch.cuda.synchronize()
    for pid, i in remap.items():
        for pool, cpool in ((kpool, ck), (vpool, cv)):
            got = to_host(pool[pid * page_elems:(pid + 1) * page_elems])
            assert np.array_equal(got, cpool[i * page_elems:(i + 1) * page_elems]), pid

    for row in range(B):
        n = int(lens[row])
        ko = torch.empty(n * H_kv * d, dtype=torch.float32, device="cuda")
        vo = torch.empty_like(ko)
        gpu.kv_gather(ko.data_ptr(), vo.data_ptr(), O.F32, kpool.data_ptr(), vpool.data_ptr(), dtype, dt.data_ptr(), table.shape[1],
                      row, 0, n, H_kv, d, P, stream_ptr())
        torch.cuda.synchronize()
        want_k = np.empty(n * H_kv * d, np.float32)
        for t in range(n):
            src = (ctable[row, t // P] * P + t % P) * H_kv * d
            want_k[t * H_kv * d:(t + 1) * H_kv * d] = ck[src:src + H_kv * d]
        assert np.array_equal(ko.cpu().numpy(), want_k)

    max_len = int(lens.max())
    out = torch.full((B, max_len), -7, dtype=torch.int64, device="cuda")
    gpu.paged_gather_indices(dt.data_ptr(), dl.data_ptr(), None, B, H_kv, d, P, table.shape[1], max_len, out.data_ptr(), stream_ptr())
    torch.cuda.synchronize()
    want_off = O.gather_offsets(table, lens, None, B, max_len, P, H_kv, d)
    assert np.array_equal(out.cpu().numpy(), want_off) and int(want_off.max()) * item > (1 << 32)

    q = O.round_to(O.fill_normal((B, H, d), 44, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    G = H // H_kv
    want = np.empty((B, H, d), np.float32)
    for g in range(G):  # the oracle decodes ungrouped heads: query head h reads pool head h // G
        sel = np.arange(H_kv) * G + g
        want[:, sel] = O.paged_decode(np.ascontiguousarray(q[:, sel]), ck, cv, ctable, lens, None, B, H_kv, d, P, scale)
    dq = torch.from_numpy(q).to(td).cuda()
    for chunk in (0, 2 * P):
        do = torch.full((B, H, d), float("nan"), dtype=td, device="cuda")
        ws_bytes = gpu.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
        ws = torch.empty(max(ws_bytes, 4) // 4, dtype=torch.float32, device="cuda")
        gpu.paged_decode_gqa(dq.data_ptr(), do.data_ptr(), dtype, kpool.data_ptr(), vpool.data_ptr(), dtype, dt.data_ptr(),
                             dl.data_ptr(), None, B, H, H_kv, d, P, table.shape[1], max_len, scale, chunk, ws.data_ptr(), ws_bytes,
                             stream_ptr())
        torch.cuda.synchronize()
        assert np.abs(to_host(do) - want).max() <= TOL[dtype], chunk
    del kpool, vpool
    torch.cuda.empty_cache()
