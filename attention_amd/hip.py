"""ctypes view of the C ABI in include/ahpc_hip.h (lib/libahpc_hip.so).

Pointers are plain integers (e.g. torch.Tensor.data_ptr()); nothing here allocates or copies
unless the function name says so.  A non-zero status raises HipError.
"""
import ctypes as C
import os

F32, F16, BF16 = 0, 1, 2

_HERE = os.path.dirname(os.path.abspath(__file__))
# AHPC_HIP_LIB points at another build of the same library (kernel experiments)
LIB_PATH = os.environ.get("AHPC_HIP_LIB") or os.path.join(_HERE, "lib", "libahpc_hip.so")


class HipError(RuntimeError):
    def __init__(self, code, what):
        super().__init__(f"{what}: status {code}: {error_string(code)}")
        self.code = code


class DeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128),
        ("arch", C.c_char * 32),
        ("total_memory_bytes", C.c_uint64),
        ("free_memory_bytes", C.c_uint64),
        ("compute_units", C.c_int32),
        ("wavefront_size", C.c_int32),
        ("lds_bytes_per_workgroup", C.c_int32),
        ("max_threads_per_workgroup", C.c_int32),
        ("clock_khz", C.c_int32),
        ("runtime_version", C.c_int32),
    ]


_vp, _i64, _f32, _ci, _sz = C.c_void_p, C.c_int64, C.c_float, C.c_int, C.c_size_t

# name -> (restype, argtypes); every symbol the header declares
SIGNATURES = {
    "ahpc_hip_error_string": (C.c_char_p, [_ci]),
    "ahpc_hip_set_tuning": (_ci, [C.c_char_p, _i64]),
    "ahpc_hip_get_tuning": (_ci, [C.c_char_p, C.POINTER(_i64)]),
    "ahpc_hip_device_count": (_ci, [C.POINTER(_ci)]),
    "ahpc_hip_device_info": (_ci, [_ci, C.POINTER(DeviceInfo)]),
    "ahpc_hip_malloc": (_ci, [C.POINTER(_vp), _sz]),
    "ahpc_hip_free": (_ci, [_vp]),
    "ahpc_hip_host_malloc": (_ci, [C.POINTER(_vp), _sz]),
    "ahpc_hip_host_free": (_ci, [_vp]),
    "ahpc_hip_vmem_granularity": (_ci, [C.POINTER(_sz)]),
    "ahpc_hip_vmem_reserve": (_ci, [C.POINTER(_vp), _sz, _sz]),
    "ahpc_hip_vmem_commit": (_ci, [_vp, _sz, C.POINTER(_sz)]),
    "ahpc_hip_vmem_decommit": (_ci, [_vp, _sz, C.POINTER(_sz)]),
    "ahpc_hip_vmem_release": (_ci, [_vp]),
    "ahpc_hip_kv_move_pages": (_ci, [_vp, _vp, _ci, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "ahpc_hip_memcpy_h2d": (_ci, [_vp, _vp, _sz, _vp]),
    "ahpc_hip_memcpy_d2h": (_ci, [_vp, _vp, _sz, _vp]),
    "ahpc_hip_memcpy_d2d": (_ci, [_vp, _vp, _sz, _vp]),
    "ahpc_hip_memset": (_ci, [_vp, _ci, _sz, _vp]),
    "ahpc_hip_ptr_is_device": (_ci, [_vp, C.POINTER(_ci)]),
    "ahpc_hip_stream_create": (_ci, [C.POINTER(_vp)]),
    "ahpc_hip_stream_destroy": (_ci, [_vp]),
    "ahpc_hip_stream_synchronize": (_ci, [_vp]),
    "ahpc_hip_device_synchronize": (_ci, []),
    "ahpc_hip_event_create": (_ci, [C.POINTER(_vp)]),
    "ahpc_hip_event_destroy": (_ci, [_vp]),
    "ahpc_hip_event_record": (_ci, [_vp, _vp]),
    "ahpc_hip_event_synchronize": (_ci, [_vp]),
    "ahpc_hip_event_elapsed_ms": (_ci, [_vp, _vp, C.POINTER(_f32)]),
    "ahpc_hip_flash_fwd": (_ci, [_vp, _vp, _vp, _vp, _ci, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _ci, _vp]),
    "ahpc_hip_flash_fwd_gqa": (_ci, [_vp, _vp, _vp, _vp, _ci, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _ci, _vp, _vp]),
    "ahpc_hip_flash_block_map": (_ci, [_i64, _i64, _i64, _ci, _i64, C.POINTER(_i64), _vp, _vp, _vp]),
    "ahpc_hip_flash_bwd_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "ahpc_hip_flash_bwd": (_ci, [_vp] * 7 + [_ci] + [_i64] * 11 + [_f32, _ci, _vp, _vp, _sz, _vp]),
    "ahpc_hip_flash_row_stats_bytes": (_sz, [_i64, _i64, _i64]),
    "ahpc_hip_flash_fwd_keep": (_ci, [_vp, _vp, _vp, _vp, _ci] + [_i64] * 11 + [_f32, _ci, _vp, _vp, C.POINTER(_ci), _vp]),
    "ahpc_hip_flash_bwd_kept": (_ci, [_vp] * 9 + [_ci] + [_i64] * 11 + [_f32, _ci, _vp, _vp, _sz, _vp]),
    "ahpc_hip_flash_bwd_varlen": (_ci, [_vp] * 7 + [_ci, _vp] + [_i64] * 9 + [_f32, _ci, _vp, _sz, _vp]),
    "ahpc_hip_flash_fwd_masked": (_ci, [_vp, _vp, _vp, _vp, _ci, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _ci, _vp, _vp]),
    "ahpc_hip_flash_fwd_varlen": (_ci, [_vp, _vp, _vp, _vp, _ci, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _ci, _vp]),
    "ahpc_hip_flash_fwd_varlen_gqa": (_ci, [_vp, _vp, _vp, _vp, _ci, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _ci, _vp]),
    "ahpc_hip_kv_scatter": (_ci, [_vp, _vp, _ci, _vp, _vp, _ci, _vp, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp]),
    "ahpc_hip_kv_scatter_batch": (_ci, [_vp, _vp, _ci, _i64, _i64, _vp, _vp, _ci, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "ahpc_hip_kv_gather": (_ci, [_vp, _vp, _ci, _vp, _vp, _ci, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _vp]),
    "ahpc_hip_paged_decode_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64, _i64]),
    "ahpc_hip_paged_decode": (_ci, [_vp, _vp, _ci, _vp, _vp, _ci, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i64, _vp, _sz, _vp]),
    "ahpc_hip_paged_decode_gqa": (_ci, [_vp, _vp, _ci, _vp, _vp, _ci, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i64, _vp, _sz, _vp]),
    "ahpc_hip_paged_decode_noalloc": (_ci, [_vp, _vp, _ci, _vp, _vp, _ci, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i64, _vp]),
    "ahpc_hip_paged_gather_indices": (_ci, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp, _vp]),
}

_lib = None


def load():
    """Load lib/libahpc_hip.so (once).  Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `make -C attention_amd/csrc` "
                              "(or __graft_entry__.build()); this package has no CPU fallback")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def error_string(code):
    return load().ahpc_hip_error_string(int(code)).decode()


def _check(code, what):
    if code != 0:
        raise HipError(code, what)


def device_count():
    n = _ci(0)
    _check(load().ahpc_hip_device_count(C.byref(n)), "device_count")
    return n.value


def set_tuning(name, value):
    _check(load().ahpc_hip_set_tuning(name.encode(), value), "set_tuning")


def get_tuning(name):
    v = _i64()
    _check(load().ahpc_hip_get_tuning(name.encode(), C.byref(v)), "get_tuning")
    return v.value


def vmem_granularity():
    """Bytes address ranges that grow in place are rounded to; 0 = the device has no virtual memory management."""
    n = _sz(0)
    _check(load().ahpc_hip_vmem_granularity(C.byref(n)), "vmem_granularity")
    return n.value


def vmem_reserve(nbytes, chunk_bytes):
    p = _vp()
    _check(load().ahpc_hip_vmem_reserve(C.byref(p), nbytes, chunk_bytes), "vmem_reserve")
    return p.value


def vmem_commit(base, nbytes):
    """Backs the first nbytes of the range with memory; returns the bytes now backed."""
    n = _sz(0)
    _check(load().ahpc_hip_vmem_commit(base, nbytes, C.byref(n)), "vmem_commit")
    return n.value


def vmem_release(base):
    _check(load().ahpc_hip_vmem_release(base), "vmem_release")


def device_info(device=0):
    info = DeviceInfo()
    _check(load().ahpc_hip_device_info(device, C.byref(info)), "device_info")
    return info


def flash_fwd(q, k, v, o, dtype, B, N, H, d, strides, scale, causal, stream=None, mask=None):
    sb, sn, sh = strides
    if mask is None:
        rc = load().ahpc_hip_flash_fwd(q, k, v, o, dtype, B, N, H, d, sb, sn, sh, scale, int(causal), stream)
    else:
        rc = load().ahpc_hip_flash_fwd_masked(q, k, v, o, dtype, B, N, H, d, sb, sn, sh, scale, int(causal), mask, stream)
    _check(rc, "flash_fwd")


def flash_block_map(B, N, H, causal):
    """Host-side dump of the MFMA kernel's workgroup -> (sequence*head, first tile, second tile) map (numpy)."""
    import numpy as np
    n = _i64(0)
    _check(load().ahpc_hip_flash_block_map(B, N, H, int(causal), 0, C.byref(n), None, None, None), "flash_block_map")
    bh, t0, t1 = (np.empty(n.value, np.int32) for _ in range(3))
    _check(load().ahpc_hip_flash_block_map(B, N, H, int(causal), n.value, C.byref(n), bh.ctypes.data, t0.ctypes.data,
                                          t1.ctypes.data), "flash_block_map")
    return bh, t0, t1


def flash_fwd_gqa(q, k, v, o, dtype, B, N, H, H_kv, d, strides, kv_strides, scale, causal, stream=None, mask=None):
    sb, sn, sh = strides
    kb, kn, kh = kv_strides
    _check(load().ahpc_hip_flash_fwd_gqa(q, k, v, o, dtype, B, N, H, H_kv, d, sb, sn, sh, kb, kn, kh, scale, int(causal),
                                        mask, stream), "flash_fwd_gqa")


def flash_bwd_workspace_bytes(B, N, H):
    return load().ahpc_hip_flash_bwd_workspace_bytes(B, N, H)


def flash_bwd(d_out, q, k, v, d_q, d_k, d_v, dtype, B, N, H, H_kv, d, strides, kv_strides, scale, causal, workspace,
              workspace_bytes, stream=None, mask=None):
    sb, sn, sh = strides
    kb, kn, kh = kv_strides
    _check(load().ahpc_hip_flash_bwd(d_out, q, k, v, d_q, d_k, d_v, dtype, B, N, H, H_kv, d, sb, sn, sh, kb, kn, kh, scale,
                                    int(causal), mask, workspace, workspace_bytes, stream), "flash_bwd")


def flash_row_stats_bytes(B, N, H):
    return load().ahpc_hip_flash_row_stats_bytes(B, N, H)


def flash_fwd_keep(q, k, v, o, dtype, B, N, H, H_kv, d, strides, kv_strides, scale, causal, row_stats, stream=None, mask=None):
    """The dense forward that also keeps its row statistics for flash_bwd_kept; returns True when it did."""
    sb, sn, sh = strides
    kb, kn, kh = kv_strides
    written = _ci(0)
    _check(load().ahpc_hip_flash_fwd_keep(q, k, v, o, dtype, B, N, H, H_kv, d, sb, sn, sh, kb, kn, kh, scale, int(causal), mask,
                                         row_stats, C.byref(written), stream), "flash_fwd_keep")
    return bool(written.value)


def flash_bwd_kept(d_out, q, k, v, o, row_stats, d_q, d_k, d_v, dtype, B, N, H, H_kv, d, strides, kv_strides, scale, causal,
                   workspace, workspace_bytes, stream=None, mask=None):
    sb, sn, sh = strides
    kb, kn, kh = kv_strides
    _check(load().ahpc_hip_flash_bwd_kept(d_out, q, k, v, o, row_stats, d_q, d_k, d_v, dtype, B, N, H, H_kv, d, sb, sn, sh, kb, kn,
                                         kh, scale, int(causal), mask, workspace, workspace_bytes, stream), "flash_bwd_kept")


def flash_bwd_varlen(d_out, q, k, v, d_q, d_k, d_v, dtype, cu_seqlens, n_seqs, max_len, H, H_kv, d, stride_t, stride_h,
                     kv_stride_t, kv_stride_h, scale, causal, workspace, workspace_bytes, stream=None):
    _check(load().ahpc_hip_flash_bwd_varlen(d_out, q, k, v, d_q, d_k, d_v, dtype, cu_seqlens, n_seqs, max_len, H, H_kv, d,
                                           stride_t, stride_h, kv_stride_t, kv_stride_h, scale, int(causal), workspace,
                                           workspace_bytes, stream), "flash_bwd_varlen")


def flash_fwd_varlen_gqa(q, k, v, o, dtype, cu_seqlens, n_seqs, max_len, H, H_kv, d, stride_t, stride_h, kv_stride_t,
                         kv_stride_h, scale, causal, stream=None):
    _check(load().ahpc_hip_flash_fwd_varlen_gqa(q, k, v, o, dtype, cu_seqlens, n_seqs, max_len, H, H_kv, d, stride_t,
                                               stride_h, kv_stride_t, kv_stride_h, scale, int(causal), stream),
           "flash_fwd_varlen_gqa")


def flash_fwd_varlen(q, k, v, o, dtype, cu_seqlens, n_seqs, max_len, H, d, stride_t, stride_h, scale, causal, stream=None):
    _check(load().ahpc_hip_flash_fwd_varlen(q, k, v, o, dtype, cu_seqlens, n_seqs, max_len, H, d, stride_t, stride_h,
                                           scale, int(causal), stream), "flash_fwd_varlen")


def kv_scatter(k_new, v_new, in_dtype, k_pool, v_pool, pool_dtype, table, max_pages, n_tokens, H, d, P,
               token_row=None, token_pos=None, row0=0, pos0=0, stream=None):
    _check(load().ahpc_hip_kv_scatter(k_new, v_new, in_dtype, k_pool, v_pool, pool_dtype, table, max_pages, token_row,
                                     token_pos, row0, pos0, n_tokens, H, d, P, stream), "kv_scatter")


def kv_scatter_batch(k_src, v_src, in_dtype, stride_b, stride_n, k_pool, v_pool, pool_dtype, table, max_pages, seq_rows, B, N,
                     H, d, P, seq_start=None, seq_tokens=None, cu_seqlens=None, stream=None):
    _check(load().ahpc_hip_kv_scatter_batch(k_src, v_src, in_dtype, stride_b, stride_n, k_pool, v_pool, pool_dtype, table,
                                           max_pages, seq_rows, seq_start, seq_tokens, cu_seqlens, B, N, H, d, P, stream),
           "kv_scatter_batch")


def kv_gather(k_out, v_out, out_dtype, k_pool, v_pool, pool_dtype, table, max_pages, row, start, n, H, d, P, stream=None):
    _check(load().ahpc_hip_kv_gather(k_out, v_out, out_dtype, k_pool, v_pool, pool_dtype, table, max_pages, row, start,
                                    n, H, d, P, stream), "kv_gather")


def paged_decode_workspace_bytes(B, H, d, max_len, P, chunk_tokens=0):
    return load().ahpc_hip_paged_decode_workspace_bytes(B, H, d, max_len, P, chunk_tokens)


def paged_decode(q, o, qo_dtype, k_pool, v_pool, pool_dtype, table, seq_lens, batch_rows, B, H, d, P, max_pages, max_len,
                 scale, chunk_tokens=0, workspace=None, workspace_bytes=0, stream=None):
    _check(load().ahpc_hip_paged_decode(q, o, qo_dtype, k_pool, v_pool, pool_dtype, table, seq_lens, batch_rows, B, H, d,
                                       P, max_pages, max_len, scale, chunk_tokens, workspace, workspace_bytes, stream),
           "paged_decode")


def paged_decode_gqa(q, o, qo_dtype, k_pool, v_pool, pool_dtype, table, seq_lens, batch_rows, B, H, H_kv, d, P, max_pages,
                     max_len, scale, chunk_tokens=0, workspace=None, workspace_bytes=0, stream=None):
    _check(load().ahpc_hip_paged_decode_gqa(q, o, qo_dtype, k_pool, v_pool, pool_dtype, table, seq_lens, batch_rows, B, H,
                                           H_kv, d, P, max_pages, max_len, scale, chunk_tokens, workspace,
                                           workspace_bytes, stream), "paged_decode_gqa")


def paged_decode_noalloc(q, o, qo_dtype, k_pool, v_pool, pool_dtype, table, seq_lens, batch_rows, B, H, H_kv, d, P, max_pages,
                         max_len, scale, chunk_tokens=0, stream=None):
    """ahpc_hip_paged_decode_gqa without a workspace argument: partials in the library's built-in scratch array."""
    _check(load().ahpc_hip_paged_decode_noalloc(q, o, qo_dtype, k_pool, v_pool, pool_dtype, table, seq_lens, batch_rows, B,
                                               H, H_kv, d, P, max_pages, max_len, scale, chunk_tokens, stream),
           "paged_decode_noalloc")


def paged_gather_indices(table, seq_lens, batch_rows, B, H, d, P, max_pages, max_len, offsets, stream=None):
    _check(load().ahpc_hip_paged_gather_indices(table, seq_lens, batch_rows, B, H, d, P, max_pages, max_len, offsets,
                                               stream), "paged_gather_indices")
