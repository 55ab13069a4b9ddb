"""ctypes binding of the CPU oracle (oracle/liboracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke run and by the benchmark's
CPU-baseline leg.  The shipped package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F32, F16, BF16 = 0, 1, 2


def build(force=False):
    """Compile liboracle.so with the Makefile beside this file."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    fp = C.POINTER(C.c_float)
    ip = C.POINTER(C.c_int32)
    lp = C.POINTER(C.c_int64)
    i64, u64, f32, ci = C.c_int64, C.c_uint64, C.c_float, C.c_int
    sig = {
        "ahpc_oracle_fill_normal": (None, [fp, C.c_size_t, u64, u64, f32]),
        "ahpc_oracle_fill_normal_at": (None, [fp, C.c_size_t, u64, u64, f32, C.c_uint64]),
        "ahpc_oracle_fill_uniform": (None, [fp, C.c_size_t, u64, u64, f32, f32]),
        "ahpc_oracle_fill_lengths": (None, [ip, C.c_size_t, u64, u64, C.c_int32, C.c_int32]),
        "ahpc_oracle_permutation": (None, [ip, C.c_size_t, u64, u64]),
        "ahpc_oracle_f32_to_f16": (C.c_uint16, [f32]),
        "ahpc_oracle_f16_to_f32": (f32, [C.c_uint16]),
        "ahpc_oracle_f32_to_bf16": (C.c_uint16, [f32]),
        "ahpc_oracle_bf16_to_f32": (f32, [C.c_uint16]),
        "ahpc_oracle_round_inplace": (None, [fp, C.c_size_t, ci]),
        "ahpc_oracle_attention": (None, [fp, fp, fp, fp, i64, i64, i64, i64, i64, i64, i64, f32, ci, fp, ci]),
        "ahpc_oracle_attention_rows": (None, [fp, fp, fp, fp, i64, i64, i64, i64, i64, i64, i64, f32, ci, lp, i64, ci]),
        "ahpc_oracle_attention_varlen": (None, [fp, fp, fp, fp, ip, i64, i64, i64, f32, ci, ci]),
        "ahpc_oracle_attention_varlen_rows": (None, [fp, fp, fp, fp, ip, i64, i64, i64, f32, ci, lp, i64, ci]),
        "ahpc_oracle_attention_backward": (None, [fp, fp, fp, fp, fp, fp, fp, i64, i64, i64, i64, i64, f32, ci, fp, ci]),
        "ahpc_oracle_softmax_merge": (None, [fp, fp, f32, f32]),
        "ahpc_oracle_attention_row_split": (None, [fp, fp, fp, fp, i64, i64, i64, f32, ci]),
        "ahpc_oracle_kv_offset": (i64, [ip, i64, i64, i64, i64, i64, i64, i64]),
        "ahpc_oracle_attended_tokens": (i64, [ip, i64, i64, i64, i64]),
        "ahpc_oracle_gather_offsets": (None, [ip, ip, ip, i64, i64, i64, i64, i64, i64, lp]),
        "ahpc_oracle_kv_scatter": (None, [fp, fp, fp, fp, ip, i64, i64, i64, i64, i64, i64, i64]),
        "ahpc_oracle_kv_gather": (None, [fp, fp, fp, fp, ip, i64, i64, i64, i64, i64, i64, i64]),
        "ahpc_oracle_paged_decode": (None, [fp, fp, fp, fp, ip, ip, ip, i64, i64, i64, i64, i64, f32, ci]),
        "ahpc_oracle_pool_create": (C.c_void_p, [C.c_int32, C.c_int32]),
        "ahpc_oracle_pool_destroy": (None, [C.c_void_p]),
        "ahpc_oracle_pool_allocate": (C.c_int32, [C.c_void_p]),
        "ahpc_oracle_pool_release": (None, [C.c_void_p, C.c_int32]),
        "ahpc_oracle_pool_free_count": (C.c_int32, [C.c_void_p]),
        "ahpc_oracle_pool_total": (C.c_int32, [C.c_void_p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def _f(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _i(a):
    if a is None:
        return None
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.POINTER(C.c_int32))


def _l(a):
    assert a.dtype == np.int64 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.POINTER(C.c_int64))


def cpu_threads():
    return max(1, min(16, len(os.sched_getaffinity(0))))


# ---- generators -------------------------------------------------------------------------
def fill_normal(shape, seed, tensor_id, sigma=1.0):
    out = np.empty(shape, np.float32)
    lib.ahpc_oracle_fill_normal(_f(out), out.size, seed, tensor_id, sigma)
    return out


def fill_uniform(shape, seed, tensor_id, lo=-1.0, hi=1.0):
    out = np.empty(shape, np.float32)
    lib.ahpc_oracle_fill_uniform(_f(out), out.size, seed, tensor_id, lo, hi)
    return out


def fill_normal_at(out, seed, tensor_id, sigma, first):
    """Fills the float32 array `out` with elements first .. first+out.size-1 of the stream fill_normal draws from."""
    lib.ahpc_oracle_fill_normal_at(_f(out), out.size, seed, tensor_id, sigma, first)
    return out


def fill_lengths(n, seed, tensor_id, lo, hi):
    out = np.empty(n, np.int32)
    lib.ahpc_oracle_fill_lengths(_i(out), n, seed, tensor_id, lo, hi)
    return out


def permutation(n, seed, tensor_id):
    out = np.empty(n, np.int32)
    lib.ahpc_oracle_permutation(_i(out), n, seed, tensor_id)
    return out


def round_to(x, dtype):
    """fp32 array -> values representable in `dtype` (still fp32)."""
    y = np.ascontiguousarray(x, np.float32).copy()
    lib.ahpc_oracle_round_inplace(_f(y), y.size, dtype)
    return y


def to_bits16(x, dtype):
    """fp32 array (already representable) -> uint16 storage bits of fp16 / bf16."""
    x = np.ascontiguousarray(x, np.float32)
    if dtype == F16:
        return x.astype(np.float16).view(np.uint16)
    assert dtype == BF16
    return (x.view(np.uint32) >> 16).astype(np.uint16)


def from_bits16(u, dtype):
    u = np.ascontiguousarray(u, np.uint16)
    if dtype == F16:
        return u.view(np.float16).astype(np.float32)
    assert dtype == BF16
    return (u.astype(np.uint32) << 16).view(np.float32)


# ---- attention ----------------------------------------------------------------------------
def _strides(B, N, H, d, layout):
    if layout == "BNHD":
        return N * H * d, H * d, d
    assert layout == "BHND"
    return H * N * d, d, N * d


def attention(q, k, v, B, N, H, d, scale, causal=False, mask=None, layout="BNHD", threads=None):
    sb, sn, sh = _strides(B, N, H, d, layout)
    out = np.zeros(B * N * H * d, np.float32)
    q, k, v = (np.ascontiguousarray(a, np.float32).reshape(-1) for a in (q, k, v))
    m = None if mask is None else _f(np.ascontiguousarray(mask, np.float32).reshape(-1))
    lib.ahpc_oracle_attention(_f(q), _f(k), _f(v), _f(out), B, N, H, d, sb, sn, sh, scale, int(causal), m,
                              threads or cpu_threads())
    return out.reshape((B, N, H, d) if layout == "BNHD" else (B, H, N, d))


def attention_backward(q, k, v, d_out, B, N, H, d, scale, causal=False, H_kv=None, mask=None, threads=None):
    """Gradients (d_q [B,N,H,d], d_k and d_v [B,N,H_kv,d]) of attention() for the given d_out."""
    H_kv = H_kv or H
    q, k, v, d_out = (np.ascontiguousarray(a, np.float32).reshape(-1) for a in (q, k, v, d_out))
    dq = np.zeros(B * N * H * d, np.float32)
    dk = np.zeros(B * N * H_kv * d, np.float32)
    dv = np.zeros(B * N * H_kv * d, np.float32)
    m = None if mask is None else _f(np.ascontiguousarray(mask, np.float32).reshape(-1))
    lib.ahpc_oracle_attention_backward(_f(q), _f(k), _f(v), _f(d_out), _f(dq), _f(dk), _f(dv), B, N, H, H_kv, d, scale,
                                       int(causal), m, threads or cpu_threads())
    return dq.reshape(B, N, H, d), dk.reshape(B, N, H_kv, d), dv.reshape(B, N, H_kv, d)


def attention_rows(q, k, v, B, N, H, d, scale, rows, causal=False, layout="BNHD", threads=None):
    """rows[i] = (b*H + h)*N + n; returns [len(rows), d]."""
    sb, sn, sh = _strides(B, N, H, d, layout)
    rows = np.ascontiguousarray(rows, np.int64)
    out = np.zeros((rows.size, d), np.float32)
    q, k, v = (np.ascontiguousarray(a, np.float32).reshape(-1) for a in (q, k, v))
    lib.ahpc_oracle_attention_rows(_f(q), _f(k), _f(v), _f(out), B, N, H, d, sb, sn, sh, scale, int(causal),
                                   _l(rows), rows.size, threads or cpu_threads())
    return out


def attention_varlen(q, k, v, cu_seqlens, H, d, scale, causal=False, threads=None):
    cu = np.ascontiguousarray(cu_seqlens, np.int32)
    q, k, v = (np.ascontiguousarray(a, np.float32).reshape(-1) for a in (q, k, v))
    out = np.zeros(q.size, np.float32)
    lib.ahpc_oracle_attention_varlen(_f(q), _f(k), _f(v), _f(out), _i(cu), cu.size - 1, H, d, scale, int(causal),
                                     threads or cpu_threads())
    return out.reshape(-1, H, d)


def attention_varlen_rows(q, k, v, cu_seqlens, H, d, scale, rows, causal=False, threads=None):
    """rows[i] = token*H + h; returns [len(rows), d]."""
    cu = np.ascontiguousarray(cu_seqlens, np.int32)
    rows = np.ascontiguousarray(rows, np.int64)
    q, k, v = (np.ascontiguousarray(a, np.float32).reshape(-1) for a in (q, k, v))
    out = np.zeros((rows.size, d), np.float32)
    lib.ahpc_oracle_attention_varlen_rows(_f(q), _f(k), _f(v), _f(out), _i(cu), cu.size - 1, H, d, scale,
                                          int(causal), _l(rows), rows.size, threads or cpu_threads())
    return out


def softmax_merge(m, l, m2, l2):
    cm, cl = C.c_float(m), C.c_float(l)
    lib.ahpc_oracle_softmax_merge(C.byref(cm), C.byref(cl), m2, l2)
    return cm.value, cl.value


def attention_row_split(q, k, v, scale, n_splits):
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    q = np.ascontiguousarray(q, np.float32)
    L, d = k.shape
    out = np.zeros(d, np.float32)
    lib.ahpc_oracle_attention_row_split(_f(q), _f(k), _f(v), _f(out), L, d, d, scale, n_splits)
    return out


# ---- paged pool -----------------------------------------------------------------------------
def kv_offset(table, row, t, h, P, H, d):
    table = np.ascontiguousarray(table, np.int32)
    return lib.ahpc_oracle_kv_offset(_i(table), table.shape[1], row, t, h, P, H, d)


def attended_tokens(table, row, L, P):
    table = np.ascontiguousarray(table, np.int32)
    return lib.ahpc_oracle_attended_tokens(_i(table), table.shape[1], row, L, P)


def gather_offsets(table, seq_lens, rows, B, max_len, P, H, d):
    table = np.ascontiguousarray(table, np.int32)
    seq_lens = np.ascontiguousarray(seq_lens, np.int32)
    rows = None if rows is None else np.ascontiguousarray(rows, np.int32)
    out = np.empty((B, max_len), np.int64)
    lib.ahpc_oracle_gather_offsets(_i(table), _i(seq_lens), _i(rows), B, table.shape[1], max_len, P, H, d, _l(out))
    return out


def kv_scatter(k_new, v_new, k_pool, v_pool, table, row, start, P, H, d):
    table = np.ascontiguousarray(table, np.int32)
    n = k_new.size // (H * d)
    lib.ahpc_oracle_kv_scatter(_f(k_new), _f(v_new), _f(k_pool), _f(v_pool), _i(table), table.shape[1], row,
                               start, n, P, H, d)


def kv_gather(k_pool, v_pool, table, row, start, n, P, H, d):
    table = np.ascontiguousarray(table, np.int32)
    k_out = np.zeros((n, H, d), np.float32)
    v_out = np.zeros((n, H, d), np.float32)
    lib.ahpc_oracle_kv_gather(_f(k_out), _f(v_out), _f(k_pool), _f(v_pool), _i(table), table.shape[1], row,
                              start, n, P, H, d)
    return k_out, v_out


def paged_decode(q, k_pool, v_pool, table, seq_lens, rows, B, H, d, P, scale, threads=None):
    table = np.ascontiguousarray(table, np.int32)
    seq_lens = np.ascontiguousarray(seq_lens, np.int32)
    rows = None if rows is None else np.ascontiguousarray(rows, np.int32)
    q = np.ascontiguousarray(q, np.float32).reshape(-1)
    out = np.zeros((B, H, d), np.float32)
    lib.ahpc_oracle_paged_decode(_f(q), _f(out), _f(k_pool.reshape(-1)), _f(v_pool.reshape(-1)), _i(table),
                                 _i(seq_lens), _i(rows), B, H, d, P, table.shape[1], scale,
                                 threads or cpu_threads())
    return out


class Pool:
    """FIFO page-allocator model."""

    def __init__(self, initial_pages=64, grow=16):
        self._p = lib.ahpc_oracle_pool_create(initial_pages, grow)

    def allocate(self):
        return lib.ahpc_oracle_pool_allocate(self._p)

    def release(self, page):
        lib.ahpc_oracle_pool_release(self._p, page)

    @property
    def free(self):
        return lib.ahpc_oracle_pool_free_count(self._p)

    @property
    def total(self):
        return lib.ahpc_oracle_pool_total(self._p)

    def __del__(self):
        if getattr(self, "_p", None):
            lib.ahpc_oracle_pool_destroy(self._p)
            self._p = None
