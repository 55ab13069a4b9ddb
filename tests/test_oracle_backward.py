"""Pins of the oracle's attention backward (oracle/oracle.c).  The reference's backward is a placeholder
(src/algorithms/flash_attention.cpp:496-580) and its test only asks for non-zero gradients
(tests/test_flash_attention.cpp:447-479), so the oracle is pinned by mathematics: numerical derivatives of an
independent float64 forward, torch's autograd as a library routine, and closed forms."""
import numpy as np
import pytest

from oracle import oracle as O


def forward64(q, k, v, scale, causal, mask=None):
    """softmax(scale q k^T) v per (batch, head) in float64; k, v may carry fewer heads (grouped)."""
    B, N, H, d = q.shape
    g = H // k.shape[2]
    out = np.zeros((B, N, H, d))
    for b in range(B):
        for h in range(H):
            s = scale * q[b, :, h].astype(np.float64) @ k[b, :, h // g].astype(np.float64).T
            if causal:
                s = np.where(np.tril(np.ones((N, N), bool)), s, -np.inf)
            if mask is not None:
                s = np.where(mask[b] != 0, s, -np.inf)
            s = s - s.max(axis=1, keepdims=True)
            p = np.exp(s)
            p /= p.sum(axis=1, keepdims=True)
            out[b, :, h] = p @ v[b, :, h // g].astype(np.float64)
    return out


def inputs(B, N, H, H_kv, d, seed):
    q = O.fill_normal((B, N, H, d), seed, 1)
    k = O.fill_normal((B, N, H_kv, d), seed, 2)
    v = O.fill_normal((B, N, H_kv, d), seed, 3)
    do = O.fill_normal((B, N, H, d), seed, 7)
    return q, k, v, do


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,N,H,H_kv,d,with_mask", [(2, 7, 2, 2, 8, False), (1, 12, 4, 2, 16, False), (1, 9, 2, 1, 4, True)])
def test_central_differences(B, N, H, H_kv, d, with_mask, causal):
    q, k, v, do = inputs(B, N, H, H_kv, d, 100 + N)
    mask = None
    if with_mask:
        mask = (O.fill_uniform((B, N, N), 5, 6) > 0.3).astype(np.float32)
        mask[:, np.arange(N), np.arange(N)] = 1.0  # every row keeps its own key
    scale = 0.37
    dq, dk, dv = O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv, mask)
    loss = lambda q_, k_, v_: float((forward64(q_, k_, v_, scale, causal, mask) * do).sum())
    rng = np.random.default_rng(N)
    eps = 1e-4
    for name, x, grad in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        for _ in range(12):
            idx = tuple(rng.integers(0, s) for s in x.shape)
            xp, xm = x.astype(np.float64).copy(), x.astype(np.float64).copy()
            xp[idx] += eps
            xm[idx] -= eps
            args_p = {"q": (xp, k, v), "k": (q, xp, v), "v": (q, k, xp)}[name]
            args_m = {"q": (xm, k, v), "k": (q, xm, v), "v": (q, k, xm)}[name]
            num = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(num - grad[idx]) <= 1e-5 + 1e-4 * abs(num), (name, idx, num, grad[idx])


@pytest.mark.parametrize("causal", [False, True])
def test_against_autograd_float64(causal):
    import torch
    B, N, H, H_kv, d = 2, 33, 4, 2, 16
    q, k, v, do = inputs(B, N, H, H_kv, d, 7)
    scale = 1.0 / np.sqrt(d)
    tq, tk, tv = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (q, k, v))
    kk = tk.repeat_interleave(H // H_kv, dim=2)
    vv = tv.repeat_interleave(H // H_kv, dim=2)
    s = scale * torch.einsum("bihd,bjhd->bhij", tq, kk)
    if causal:
        s = s.masked_fill(~torch.tril(torch.ones(N, N, dtype=torch.bool)), float("-inf"))
    o = torch.einsum("bhij,bjhd->bihd", torch.softmax(s, dim=-1), vv)
    o.backward(torch.tensor(do, dtype=torch.float64))
    dq, dk, dv = O.attention_backward(q, k, v, do, B, N, H, d, scale, causal, H_kv)
    for got, want in ((dq, tq.grad), (dk, tk.grad), (dv, tv.grad)):
        assert np.abs(got - want.numpy()).max() <= 2e-6


def test_single_token():
    q, k, v, do = inputs(2, 1, 3, 3, 8, 1)
    dq, dk, dv = O.attention_backward(q, k, v, do, 2, 1, 3, 8, 0.5)
    assert np.array_equal(dv, do) and not dq.any() and not dk.any()


def test_equal_value_rows_give_no_query_or_key_gradient():
    B, N, H, d = 1, 10, 2, 8
    q, k, v, do = inputs(B, N, H, H, d, 2)
    v[:] = v[:, :1]
    dq, dk, dv = O.attention_backward(q, k, v, do, B, N, H, d, 0.3, True)
    assert np.abs(dq).max() <= 1e-6 and np.abs(dk).max() <= 1e-6


def test_equal_key_rows_give_uniform_weights():
    B, N, H, d = 1, 10, 2, 8
    q, k, v, do = inputs(B, N, H, H, d, 3)
    k[:] = k[:, :1]
    dq, dk, dv = O.attention_backward(q, k, v, do, B, N, H, d, 0.3, False)
    assert np.abs(dq).max() <= 1e-6
    assert np.abs(dv - do.mean(axis=1, keepdims=True)).max() <= 1e-6


@pytest.mark.parametrize("causal", [False, True])
def test_sum_rules(causal):
    B, N, H, d = 2, 21, 3, 16
    q, k, v, do = inputs(B, N, H, H, d, 4)
    dq, dk, dv = O.attention_backward(q, k, v, do, B, N, H, d, 0.2, causal)
    # weights of a row sum to one
    assert np.abs(dv.sum(axis=1) - do.sum(axis=1)).max() <= 1e-4
    # both equal scale * sum_ij dS_ij (q_i . k_j)
    lhs = (q.astype(np.float64) * dq).sum(axis=(1, 3))
    rhs = (k.astype(np.float64) * dk).sum(axis=(1, 3))
    assert np.abs(lhs - rhs).max() <= 1e-4


def test_grouped_heads_sum_the_groups_gradients():
    B, N, H, H_kv, d = 1, 14, 6, 2, 8
    q, k, v, do = inputs(B, N, H, H_kv, d, 5)
    g = H // H_kv
    dq, dk, dv = O.attention_backward(q, k, v, do, B, N, H, d, 0.25, True, H_kv)
    dq2, dk2, dv2 = O.attention_backward(q, np.repeat(k, g, axis=2), np.repeat(v, g, axis=2), do, B, N, H, d, 0.25, True)
    assert np.abs(dq - dq2).max() <= 1e-6
    assert np.abs(dk - dk2.reshape(B, N, H_kv, g, d).sum(axis=3)).max() <= 1e-5
    assert np.abs(dv - dv2.reshape(B, N, H_kv, g, d).sum(axis=3)).max() <= 1e-5


def test_fully_masked_row_contributes_nothing():
    B, N, H, d = 1, 6, 1, 4
    q, k, v, do = inputs(B, N, H, H, d, 6)
    mask = np.ones((B, N, N), np.float32)
    mask[0, 2, :] = 0.0
    dq, dk, dv = O.attention_backward(q, k, v, do, B, N, H, d, 0.5, False, mask=mask)
    assert not dq[0, 2].any()
    do2 = do.copy()
    do2[0, 2] = 0.0
    dq2, dk2, dv2 = O.attention_backward(q, k, v, do2, B, N, H, d, 0.5, False, mask=mask)
    assert np.array_equal(dk, dk2) and np.array_equal(dv, dv2)
