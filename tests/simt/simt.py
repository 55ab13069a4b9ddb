"""Test infrastructure: loads tests/simt/libahpc_simt.so, the library's kernel sources compiled as host
C++ and executed lane by lane on the CPU.  It exports the same compute entry points as
attention_amd/lib/libahpc_hip.so; "device" pointers are numpy buffers.  Only tests import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from attention_amd import hip

_HERE = os.path.dirname(os.path.abspath(__file__))
# AHPC_SIMT_LIB names another build of the same library (the sanitizer build of the Makefile's `ubsan` target)
LIB_PATH = os.environ.get("AHPC_SIMT_LIB") or os.path.join(_HERE, "libahpc_simt.so")

F32, F16, BF16 = 0, 1, 2
_lib = None


def build():
    if os.environ.get("AHPC_SIMT_LIB"):
        return  # a build the caller made
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def load():
    """The emulated library with every entry point it exports bound to the signature of the real one."""
    global _lib
    if _lib is None:
        build()
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in hip.SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError:
                continue  # runtime services (malloc, streams, events) are not part of the emulated build
            fn.restype = res
            fn.argtypes = args
        lib.simt_configure.restype = None
        lib.simt_configure.argtypes = [C.c_int, C.c_uint64]
        lib.simt_last_error_text.restype = C.c_char_p
        lib.simt_clear_error.restype = None
        _lib = lib
    return _lib


def configure(dma_late=False, seed=1):
    """dma_late: direct-to-LDS loads land only at the issuing lane's next wait; seed: wavefront order."""
    load().simt_configure(int(dma_late), seed)


def check(rc, what):
    if rc != 0:
        lib = load()
        text = lib.simt_last_error_text().decode()
        lib.simt_clear_error()
        raise AssertionError(f"{what}: status {rc} {text}")


def to_storage(x_f32, dtype):
    """fp32 numpy (values already representable in `dtype`) -> numpy array holding that storage type."""
    x = np.ascontiguousarray(x_f32, np.float32)
    if dtype == F32:
        return x.copy()
    if dtype == F16:
        return x.astype(np.float16)
    return (x.view(np.uint32) >> 16).astype(np.uint16)


def from_storage(a, dtype):
    if dtype == F32:
        return np.array(a, np.float32)
    if dtype == F16:
        return a.astype(np.float32)
    return (a.astype(np.uint32) << 16).view(np.float32)


def empty_storage(shape, dtype):
    """Output buffer filled with a pattern that reads as NaN in every storage type."""
    if dtype == F32:
        return np.full(shape, np.nan, np.float32)
    if dtype == F16:
        return np.full(shape, np.nan, np.float16)
    return np.full(shape, 0x7FC0, np.uint16)


def ptr(a):
    return a.ctypes.data


class EmulatedHip:
    """The call wrappers of attention_amd.hip, bound to the emulated library for the duration of a call."""
    HipError = hip.HipError

    def __getattr__(self, name):
        target = getattr(hip, name)
        if not callable(target) or isinstance(target, type):
            return target

        def call(*args, **kwargs):
            saved = hip._lib
            hip._lib = load()
            try:
                return target(*args, **kwargs)
            finally:
                hip._lib = saved
                err = load().simt_last_error_text().decode()
                if err:
                    load().simt_clear_error()
                    raise AssertionError("emulated launch failed: " + err)
        return call


_libc = C.CDLL(None, use_errno=True)
_libc.mprotect.argtypes = [C.c_void_p, C.c_size_t, C.c_int]
_libc.mprotect.restype = C.c_int


def guarded(a, front=False):
    """A copy of `a` whose last byte is directly followed by an inaccessible page (front=True: whose
    first byte directly follows one), so that a kernel reading or writing past the end faults on the spot."""
    import mmap
    a = np.ascontiguousarray(a)
    page = mmap.PAGESIZE
    body = max(page, (a.nbytes + page - 1) // page * page)
    m = mmap.mmap(-1, body + 2 * page)
    base = C.addressof(C.c_char.from_buffer(m))
    for addr in (base, base + page + body):
        if _libc.mprotect(addr, page, 0) != 0:
            raise OSError(C.get_errno(), "mprotect")
    off = page if front else page + body - a.nbytes
    out = np.frombuffer(m, dtype=a.dtype, count=a.size, offset=off).reshape(a.shape)
    out[...] = a
    return out


def lds_stats(reset=False):
    """(16-byte LDS reads, their bank-conflict cycles, transposing reads, their bank-conflict cycles) per
    wavefront instruction, under the executor's model of 64 banks of 4 bytes."""
    lib = load()
    out = (C.c_long * 4)()
    lib.simt_lds_stats(out)
    if reset:
        lib.simt_lds_stats_reset()
    return tuple(out)
