"""Sequences far longer than the benchmark configurations: a prefill of 40 013 tokens (313 query tiles, a count
that is odd and not a multiple of anything in the work map) and a decode over a context of 150 001 tokens
(9 376 pages, some 150 context chunks).  The oracle checks a seeded sample of the prefill's rows and all of
the decode's output."""
import numpy as np
import pytest

from oracle import oracle as O
from gpu_util import TOL, torch_dtype, to_host, stream_ptr, dev_i32
from test_gpu_paged import build_problem

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,d,causal,H,H_kv", [(O.BF16, 128, True, 2, 2), (O.F16, 64, False, 2, 1), (O.F32, 128, True, 2, 2),
                                                  (O.BF16, 96, True, 4, 2)])
def test_prefill_of_40013_tokens(gpu, dtype, d, causal, H, H_kv):
    import torch
    B, N = 1, 40013
    td = torch_dtype(dtype)
    g = torch.Generator(device="cuda").manual_seed(0xA77E0020)
    dq = torch.randn((B, N, H, d), generator=g, device="cuda", dtype=torch.float32).to(td)
    dk, dv = (torch.randn((B, N, H_kv, d), generator=g, device="cuda", dtype=torch.float32).to(td) for _ in range(2))
    do = torch.full_like(dq, float("nan"))
    scale = 1.0 / np.sqrt(d)
    print(f"long prefill: dtype={dtype} d={d} causal={causal} H={H} H_kv={H_kv}", flush=True)
    gpu.flash_fwd_gqa(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), dtype, B, N, H, H_kv, d, (N * H * d, H * d, d),
                      (N * H_kv * d, H_kv * d, d), scale, causal, stream_ptr())
    torch.cuda.synchronize()
    out = do.float()
    assert torch.isfinite(out).all()
    G = H // H_kv
    vfull = dv.float().repeat_interleave(G, dim=2)
    if causal:
        assert torch.allclose(out[:, 0], vfull[:, 0])  # row 0 sees only key 0
        vmax, vmin = torch.cummax(vfull, dim=1).values, torch.cummin(vfull, dim=1).values
    else:
        vmax, vmin = vfull.amax(dim=1, keepdim=True), vfull.amin(dim=1, keepdim=True)
    assert (out <= vmax + TOL[dtype]).all() and (out >= vmin - TOL[dtype]).all()
    rng = np.random.default_rng(20)
    rows = np.unique(np.concatenate([rng.integers(0, B * H * N, 192), [0, N - 1, H * N - 1, 127, 128, 40012 - 128, 20006, 20007]]))
    q = to_host(dq)
    k, v = to_host(dk.repeat_interleave(G, dim=2)), to_host(vfull)
    want = O.attention_rows(q, k, v, B, N, H, d, scale, rows.astype(np.int64), causal)
    host = to_host(do)
    got = np.stack([host[r // (N * H), r % N, (r // N) % H] for r in rows])
    assert np.abs(got - want).max() <= TOL[dtype]


@pytest.mark.parametrize("dtype,H,H_kv,d", [(O.F16, 4, 4, 128), (O.BF16, 16, 2, 128), (O.F16, 32, 1, 128), (O.F32, 2, 2, 64)])
def test_decode_over_150001_tokens(gpu, dtype, H, H_kv, d):
    import torch
    P, B = 16, 2
    lens = [150001, 77]
    qk, kp, vp, table, lens, _, _ = build_problem(B, H_kv, d, P, lens, 61, dtype)
    q = O.round_to(O.fill_normal((B, H, d), 62, 1), dtype)
    scale = 1.0 / np.sqrt(d)
    G = H // H_kv
    want = np.empty((B, H, d), np.float32)
    for g in range(G):  # the oracle decodes ungrouped heads: query head h reads pool head h // G
        sel = np.arange(H_kv) * G + g
        want[:, sel] = O.paged_decode(np.ascontiguousarray(q[:, sel]), kp, vp, table, lens, None, B, H_kv, d, P, scale)
    td = torch_dtype(dtype)
    dk, dv = torch.from_numpy(kp).to(td).cuda(), torch.from_numpy(vp).to(td).cuda()
    dq = torch.from_numpy(q).to(td).cuda()
    dt, dl = dev_i32(table), dev_i32(lens)
    max_len = int(lens.max())
    for chunk in (0, 64 * P):
        do = torch.full((B, H, d), float("nan"), dtype=td, device="cuda")
        ws_bytes = gpu.paged_decode_workspace_bytes(B, H, d, max_len, P, chunk)
        ws = torch.empty(max(ws_bytes, 4) // 4, dtype=torch.float32, device="cuda")
        print(f"long decode: dtype={dtype} H={H} H_kv={H_kv} d={d} chunk={chunk} workspace={ws_bytes}", flush=True)
        gpu.paged_decode_gqa(dq.data_ptr(), do.data_ptr(), dtype, dk.data_ptr(), dv.data_ptr(), dtype, dt.data_ptr(), dl.data_ptr(),
                             None, B, H, H_kv, d, P, table.shape[1], max_len, scale, chunk, ws.data_ptr(), ws_bytes, stream_ptr())
        torch.cuda.synchronize()
        assert np.abs(to_host(do) - want).max() <= TOL[dtype], chunk


def _row_gradients(q, k, v, do, h, hk, rows, scale, causal):
    """dQ rows and softmax weights of single query rows in float64, from the definition (one row needs only its own
    scores): p = softmax(scale q_i K^T), dP = dO_i V^T, dS = p (dP - p.dP), dQ_i = scale dS K."""
    K, V = k[0, :, hk].astype(np.float64), v[0, :, hk].astype(np.float64)
    out, last_w = [], []
    for i in rows:
        n = i + 1 if causal else K.shape[0]
        s = scale * (K[:n] @ q[0, i, h].astype(np.float64))
        p = np.exp(s - s.max())
        p /= p.sum()
        dp = V[:n] @ do[0, i, h].astype(np.float64)
        ds = p * (dp - (p * dp).sum())
        out.append(scale * (ds @ K[:n]))
        last_w.append(p[-1])
    return np.stack(out), np.array(last_w)


@pytest.mark.parametrize("dtype,d,causal,H,H_kv", [(O.BF16, 128, True, 2, 1), (O.F32, 64, False, 2, 2), (O.F16, 64, True, 2, 2)])
def test_backward_of_40013_tokens(gpu, dtype, d, causal, H, H_kv):
    """Properties that hold at any size over the whole result, and sampled dQ rows from the definition."""
    import torch
    B, N = 1, 40013
    td = torch_dtype(dtype)
    g = torch.Generator(device="cuda").manual_seed(0xA77E0021)
    tq, tdo = (torch.randn((B, N, H, d), generator=g, device="cuda", dtype=torch.float32).to(td) for _ in range(2))
    tk, tv = (torch.randn((B, N, H_kv, d), generator=g, device="cuda", dtype=torch.float32).to(td) for _ in range(2))
    gq = torch.full_like(tq, float("nan"))
    gk, gv = torch.full_like(tk, float("nan")), torch.full_like(tv, float("nan"))
    ws_bytes = gpu.flash_bwd_workspace_bytes(B, N, H)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device="cuda")
    scale = 1.0 / np.sqrt(d)
    print(f"long backward: dtype={dtype} d={d} causal={causal} H={H} H_kv={H_kv}", flush=True)
    gpu.flash_bwd(tdo.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), gq.data_ptr(), gk.data_ptr(), gv.data_ptr(),
                  dtype, B, N, H, H_kv, d, (N * H * d, H * d, d), (N * H_kv * d, H_kv * d, d), scale, causal, ws.data_ptr(),
                  ws_bytes, stream_ptr())
    torch.cuda.synchronize()
    for t in (gq, gk, gv):
        assert torch.isfinite(t.float()).all()
    rel = 1e-4 if dtype == O.F32 else 2e-2
    G = H // H_kv
    # the weights of a query row sum to one: sum_j dV_j = sum_i dO_i, per pool head over its group of query heads
    lhs = gv.double().sum(dim=1)
    rhs = tdo.double().sum(dim=1).reshape(B, H_kv, G, d).sum(dim=2)
    # (bars: the relative bar of the element-wise checks on the sums of magnitudes, which is what rounding of the
    # single entries can add up to; a wrong kernel is off by the magnitudes themselves)
    assert (lhs - rhs).abs().max().item() <= rel * max(1.0, gv.double().abs().sum(dim=1).max().item())
    # sum_i q_i.dQ_i = sum_j k_j.dK_j (both are scale * sum_ij dS_ij q_i.k_j), per pool head
    a = (tq.double() * gq.double()).sum(dim=(1, 3)).reshape(B, H_kv, G).sum(dim=2)
    b = (tk.double() * gk.double()).sum(dim=(1, 3))
    mag = ((tq.double() * gq.double()).abs().sum(dim=(1, 3)).reshape(B, H_kv, G).sum(dim=2)
           + (tk.double() * gk.double()).abs().sum(dim=(1, 3)))
    assert ((a - b).abs() <= rel * mag.clamp(min=1.0)).all()
    # sampled dQ rows from the definition
    q, k, v, do = (to_host(t) for t in (tq, tk, tv, tdo))
    rows = np.unique(np.concatenate([np.random.default_rng(21).integers(0, N, 24), [0, 127, 128, N - 1, N - 2, 20006]]))
    host_gq = to_host(gq)
    for h in range(H):
        want, last_w = _row_gradients(q, k, v, do, h, h // G, rows, scale, causal)
        got = host_gq[0, rows, h]
        assert np.abs(got - want).max() <= rel * max(1.0, np.abs(want).max()), h
    if causal and G == 1:
        # the last key is seen by the last query only: dV_last = P_last,last * dO_last
        for h in range(H):
            _, w = _row_gradients(q, k, v, do, h, h, [N - 1], scale, True)
            assert np.abs(to_host(gv)[0, N - 1, h] - w[0] * do[0, N - 1, h]).max() <= rel
