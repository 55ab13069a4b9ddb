"""The MFMA flash kernel's workgroup -> work map, dumped on the host by the function the kernel itself uses
(ahpc_hip_flash_block_map): whatever the shape and the pairing of query tiles under a causal mask, every
(sequence*head, query tile) must be handled by exactly one workgroup pass, and nothing else may be handled.  A map that misses or repeats a tile computes wrong
attention; one that names a head that does not exist reads outside the tensors."""
import numpy as np
import pytest

ROWS = 128  # query rows per workgroup pass (256 while the tuning value flash_rows says so)


def check_exact_cover(B, N, H, causal, ROWS=ROWS):
    from attention_amd import hip
    bh, t0, t1 = hip.flash_block_map(B, N, H, causal)
    n_tiles = (N + ROWS - 1) // ROWS
    assert len(bh) % 8 == 0
    valid = bh >= 0
    assert ((t0 >= 0) == valid).all() and (t1[~valid] == -1).all()
    assert bh[valid].max() < B * H and t0[valid].max() < n_tiles and t1.max() < n_tiles
    pairs = np.concatenate([bh[valid].astype(np.int64) * n_tiles + t0[valid], (bh.astype(np.int64) * n_tiles + t1)[t1 >= 0]])
    assert len(pairs) == B * H * n_tiles
    assert np.array_equal(np.sort(pairs), np.arange(B * H * n_tiles))
    return bh, t0, t1


SHAPES = [(1, 1, 1), (1, 128, 1), (2, 129, 3), (1, 1000, 3), (2, 2144, 16), (4, 4096, 32), (1, 777, 5), (3, 640, 7),
          (64, 300, 8), (1, 8192, 9), (5, 1152, 13)]


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,N,H", SHAPES)
def test_default_map_covers_every_tile_once_and_keeps_its_order(B, N, H, causal):
    bh, t0, t1 = check_exact_cover(B, N, H, causal)
    # the default order: consecutive logical ids (= 8 workgroup ids apart) walk one head's tiles, late tiles first
    n_tiles = (N + ROWS - 1) // ROWS
    paired = causal and n_tiles >= 2 and B * H * n_tiles >= 1024
    per_head = (n_tiles + 1) // 2 if paired else n_tiles
    per_xcd = len(bh) // 8
    for block in range(len(bh)):
        logical = (block & 7) * per_xcd + (block >> 3)
        if logical >= B * H * per_head:
            assert bh[block] == -1
            continue
        slot = logical % per_head
        assert bh[block] == logical // per_head and t0[block] == n_tiles - 1 - slot
        want_second = slot if paired and 2 * slot != n_tiles - 1 else -1
        assert t1[block] == want_second


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,N,H", SHAPES)
def test_map_of_256_row_workgroups_covers_every_tile_once(B, N, H, causal):
    from attention_amd import hip
    before = hip.get_tuning("flash_rows")
    hip.set_tuning("flash_rows", 256)
    try:
        check_exact_cover(B, N, H, causal, ROWS=256)
    finally:
        hip.set_tuning("flash_rows", before)


def test_rejects_bad_shapes_without_a_gpu():
    from attention_amd import hip
    import ctypes as C
    n = C.c_int64(0)
    assert hip.load().ahpc_hip_flash_block_map(0, 16, 4, 0, 0, C.byref(n), None, None, None) == -2
    assert hip.load().ahpc_hip_flash_block_map(1, 16, 4, 0, 0, None, None, None, None) == -1
    buf = np.empty(4, np.int32)
    assert hip.load().ahpc_hip_flash_block_map(4, 4096, 32, 1, 4, C.byref(n), buf.ctypes.data, buf.ctypes.data, buf.ctypes.data) == -2
