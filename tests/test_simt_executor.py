"""The lane-by-lane CPU executor (tests/simt) checked on its own: kernels that are wrong on purpose must be
reported, and the cross-lane operations must give the documented results on known inputs."""
import ctypes as C

import numpy as np
import pytest

from simt import simt as S


@pytest.fixture(scope="module")
def lib():
    lib = S.load()
    S.configure(False, 1)
    return lib


def failing(lib, fn, *args):
    rc = fn(*args)
    text = lib.simt_last_error_text().decode()
    lib.simt_clear_error()
    assert rc != 0
    return text


def test_barrier_reached_by_half_a_wavefront_is_reported(lib):
    out = np.zeros(64, np.float32)
    text = failing(lib, lib.simt_selftest_half_wave_at_barrier, C.c_void_p(out.ctypes.data))
    assert "cannot make progress" in text


def test_lanes_at_different_cross_lane_operations_are_reported(lib):
    out = np.zeros(64, np.float32)
    text = failing(lib, lib.simt_selftest_lanes_at_different_operations, C.c_void_p(out.ctypes.data))
    assert "different cross-lane operations" in text


def test_reading_a_lane_that_has_finished_is_reported(lib):
    out = np.zeros(64, np.int32)
    text = failing(lib, lib.simt_selftest_reads_a_finished_lane, C.c_void_p(out.ctypes.data))
    assert "not executing" in text


def test_direct_to_lds_load_without_wait_is_exposed(lib):
    src = S.guarded(np.arange(1024, dtype=np.uint8))  # the descriptor covers 1000 bytes only
    want = src.copy()
    want[992:] = 0       # the lane whose 16 bytes cross the descriptor's end gets zeros

    def run(wait):
        dst = np.zeros(1024, np.uint8)
        assert lib.simt_selftest_dma_round_trip(C.c_void_p(src.ctypes.data), C.c_void_p(dst.ctypes.data), wait) == 0
        return dst

    for late in (False, True):
        S.configure(late, 3)
        assert np.array_equal(run(1), want)
    S.configure(True, 3)
    assert not np.array_equal(run(0), want)  # the data has not landed: the LDS still holds the fill pattern
    S.configure(False, 1)


def test_lds_traffic_of_two_wavefronts_needs_a_barrier_between(lib):
    src = S.guarded(np.arange(2048, dtype=np.uint16).view(np.uint8)[:2048].copy())
    for seed in (1, 2, 3, 4):
        for late in (False, True):
            S.configure(late, seed)
            dst = np.zeros(1024, np.uint8)
            assert lib.simt_selftest_lds_ordering(C.c_void_p(src.ctypes.data), C.c_void_p(dst.ctypes.data), 0) == 0
            assert np.array_equal(dst, src[:1024])
            # no barrier between the wait for a load and another wavefront's read of its data
            text = failing(lib, lib.simt_selftest_lds_ordering, C.c_void_p(src.ctypes.data), C.c_void_p(dst.ctypes.data), 1)
            assert "direct-to-LDS load" in text and "another wavefront" in text
            # a load into LDS that the other wavefront reads in the same barrier interval
            text = failing(lib, lib.simt_selftest_lds_ordering, C.c_void_p(src.ctypes.data), C.c_void_p(dst.ctypes.data), 2)
            assert "direct-to-LDS load" in text and "another wavefront" in text
    S.configure(False, 1)


def test_matrix_instruction_equals_matmul(lib):
    rng = np.random.default_rng(5)
    a = rng.integers(-8, 9, (32, 16)).astype(np.float32)
    b = rng.integers(-8, 9, (16, 32)).astype(np.float32)
    c = rng.integers(-50, 50, (32, 32)).astype(np.float32)
    d = np.zeros((32, 32), np.float32)
    rc = lib.simt_selftest_matrix_instruction(*(C.c_void_p(x.ctypes.data) for x in (a, b, c, d)))
    assert rc == 0
    assert np.array_equal(d, a @ b + c)


def test_dpp_butterflies(lib):
    x = np.random.default_rng(6).integers(-100, 100, 64).astype(np.float32)
    out = np.zeros((4, 64), np.float32)
    assert lib.simt_selftest_dpp_sums(C.c_void_p(x.ctypes.data), C.c_void_p(out.ctypes.data)) == 0
    for i, width in enumerate((2, 4, 8, 16)):
        want = np.repeat(x.reshape(-1, width).sum(axis=1), width)
        assert np.array_equal(out[i], want)


def test_forward_kernel_ignores_workgroups_its_tensors_do_not_cover(lib, kind=0):
    """A workgroup map that names more (sequence, head) pairs than the tensors hold (here: one batch entry too many)
    must leave the surplus workgroups without a single access: the tensors sit against inaccessible pages, and the
    heads that do exist get the same result as from an honest launch."""
    from oracle import oracle as O
    B, N, H, d = 1, 300, 2, 128
    q, k, v = (O.round_to(O.fill_normal((B, N, H, d), 81, t), O.BF16) for t in (1, 2, 3))
    dq, dk, dv = (S.guarded(S.to_storage(x, S.BF16)) for x in (q, k, v))
    out = S.guarded(S.empty_storage((B, N, H, d), S.BF16))
    ptr = lambda a: C.c_void_p(a.ctypes.data)
    for late in (False, True):
        S.configure(late, 5)
        rc = lib.simt_selftest_flash_oversized_map(ptr(dq), ptr(dk), ptr(dv), ptr(out), B, 1, N, H, kind)
        S.check(rc, "forward with an oversized map")
    S.configure(False, 1)
    want = O.attention(q, k, v, B, N, H, d, 0.1275 / np.log2(np.e), True)
    assert np.abs(S.from_storage(out, S.BF16) - want).max() <= 2e-2
