"""Every compute entry point of the C ABI refuses bad arguments BEFORE it touches the GPU, so these checks
run anywhere.  The codes are the AHPC_ERR_* values of include/ahpc_hip.h.  (The C++ classes turn them into
the reference's AttentionException codes; tests/cpp/conformance.cpp covers that side, following
tests/test_flash_attention.cpp:310-357 and tests/test_backends.cpp:631-680 of the reference.)"""
import pytest

NULL_POINTER, BAD_SHAPE, BAD_DTYPE, HEAD_DIM, WORKSPACE, BAD_ALIGNMENT, BAD_GROUP = -1, -2, -3, -4, -5, -7, -8
P = 4096  # a non-null, 16-byte aligned "pointer": never dereferenced, the calls below all fail first
F16 = 1


@pytest.fixture(scope="module")
def lib():
    from attention_amd import hip
    return hip.load()


def dense(lib, q=P, k=P, v=P, o=P, dtype=F16, B=2, N=16, H=4, d=64, sb=None, sn=None, sh=None):
    sb = N * H * d if sb is None else sb
    sn = H * d if sn is None else sn
    sh = d if sh is None else sh
    return lib.ahpc_hip_flash_fwd(q, k, v, o, dtype, B, N, H, d, sb, sn, sh, 0.0, 0, None)


def test_flash_forward_argument_checks(lib):
    assert dense(lib, q=None) == NULL_POINTER and dense(lib, o=None) == NULL_POINTER
    assert dense(lib, dtype=3) == BAD_DTYPE and dense(lib, dtype=-1) == BAD_DTYPE
    for bad in (dict(B=0), dict(N=0), dict(H=0), dict(d=0), dict(B=70000), dict(sn=8), dict(sh=8), dict(sb=-1)):
        assert dense(lib, **bad) == BAD_SHAPE, bad
    assert dense(lib, d=512, sn=4 * 512, sh=512, sb=16 * 4 * 512) == HEAD_DIM
    # masked entry point: the same checks, mask may be null
    assert lib.ahpc_hip_flash_fwd_masked(P, P, None, P, F16, 2, 16, 4, 64, 4096, 256, 64, 0.0, 0, None, None) == NULL_POINTER


def test_grouped_heads_argument_checks(lib):
    def gqa(H=8, Hkv=2, **kw):
        N, d = 16, 64
        return lib.ahpc_hip_flash_fwd_gqa(P, P, P, P, F16, 1, N, H, Hkv, d, N * H * d, H * d, d, N * Hkv * d, Hkv * d, d, 0.0, 0, None, None)
    assert gqa(H=6, Hkv=4) == BAD_SHAPE      # every K/V head must serve the same number of query heads
    assert gqa(H=8, Hkv=0) == BAD_SHAPE
    # ragged: cu_seqlens is required
    assert lib.ahpc_hip_flash_fwd_varlen_gqa(P, P, P, P, F16, None, 2, 16, 8, 2, 64, 8 * 64, 64, 2 * 64, 64, 0.0, 1, None) == NULL_POINTER
    assert lib.ahpc_hip_flash_fwd_varlen(P, P, P, P, F16, None, 2, 16, 8, 64, 8 * 64, 64, 0.0, 1, None) == NULL_POINTER


def test_flash_backward_argument_checks(lib):
    def bwd(go=P, q=P, gq=P, dtype=F16, B=1, N=16, H=4, Hkv=2, d=64, ws=P, ws_bytes=1 << 20, sn=None):
        sn = H * d if sn is None else sn
        return lib.ahpc_hip_flash_bwd(go, q, P, P, gq, P, P, dtype, B, N, H, Hkv, d, N * H * d, sn, d, N * Hkv * d, Hkv * d, d,
                                      0.0, 1, None, ws, ws_bytes, None)
    assert bwd(go=None) == NULL_POINTER and bwd(q=None) == NULL_POINTER and bwd(gq=None) == NULL_POINTER
    assert bwd(ws=None) == NULL_POINTER
    assert bwd(dtype=7) == BAD_DTYPE
    assert bwd(N=0) == BAD_SHAPE and bwd(H=6, Hkv=4) == BAD_SHAPE and bwd(sn=8) == BAD_SHAPE
    assert bwd(d=512, sn=4 * 512) == HEAD_DIM
    need = lib.ahpc_hip_flash_bwd_workspace_bytes(1, 16, 4)
    assert need == 1 * 4 * 128 * 2 * 4          # rows padded to a whole 128-row tile, two floats each
    assert bwd(ws_bytes=need - 1) == WORKSPACE
    assert bwd(ws=P + 4) == BAD_ALIGNMENT
    assert lib.ahpc_hip_flash_bwd_workspace_bytes(0, 16, 4) == 0
    # ragged: cu_seqlens is required, the rest is checked like the dense call
    rag = lambda cu, H=4, Hkv=2: lib.ahpc_hip_flash_bwd_varlen(P, P, P, P, P, P, P, F16, cu, 2, 16, H, Hkv, 64, H * 64, 64, Hkv * 64, 64,
                                                                0.0, 1, P, 1 << 20, None)
    assert rag(None) == NULL_POINTER and rag(P, H=6, Hkv=4) == BAD_SHAPE


def decode(lib, q=P, o=P, kp=P, vp=P, table=P, lens=P, qo=F16, pool=F16, B=2, H=8, Hkv=8, d=128, Pg=16, max_pages=4, max_len=64,
           ws=None, ws_bytes=0, chunk=0):
    return lib.ahpc_hip_paged_decode_gqa(q, o, qo, kp, vp, pool, table, lens, None, B, H, Hkv, d, Pg, max_pages, max_len, 0.0, chunk,
                                         ws, ws_bytes, None)


def test_paged_decode_argument_checks(lib):
    assert decode(lib, q=None) == NULL_POINTER and decode(lib, lens=None) == NULL_POINTER
    assert decode(lib, qo=5) == BAD_DTYPE and decode(lib, pool=-2) == BAD_DTYPE
    assert decode(lib, B=0) == BAD_SHAPE and decode(lib, max_len=0) == BAD_SHAPE
    assert decode(lib, max_len=65, max_pages=4) == BAD_SHAPE           # the table row cannot hold that many tokens
    # lengths are 32-bit in the kernels: a bound beyond that is refused, not truncated
    assert decode(lib, Pg=4096, max_pages=1 << 20, max_len=(1 << 31) + 4096, chunk=262144, ws=P, ws_bytes=1 << 40) == BAD_SHAPE
    assert decode(lib, d=44) == HEAD_DIM and decode(lib, d=264) == HEAD_DIM   # whole 16-byte pieces of an fp16 row, up to 256
    assert decode(lib, kp=P + 8) == BAD_ALIGNMENT and decode(lib, o=P + 2) == BAD_ALIGNMENT
    assert decode(lib, H=6, Hkv=4) == BAD_SHAPE                        # does not divide
    # several chunks need the workspace the size query reports
    need = lib.ahpc_hip_paged_decode_workspace_bytes(2, 8, 128, 64, 16, 16)
    assert need == 2 * 4 * 8 * 130 * 4
    assert decode(lib, chunk=16, ws=None, ws_bytes=0) == WORKSPACE
    assert decode(lib, chunk=16, ws=P, ws_bytes=need - 1) == WORKSPACE
    assert lib.ahpc_hip_paged_decode(None, P, F16, P, P, F16, P, P, None, 2, 8, 128, 16, 4, 64, 0.0, 0, None, 0, None) == NULL_POINTER


def test_pool_copy_argument_checks(lib):
    sc = lib.ahpc_hip_kv_scatter
    assert sc(P, P, F16, P, P, F16, P, 4, None, None, 0, 0, 0, 8, 64, 16, None) == 0              # nothing to do
    assert sc(None, P, F16, P, P, F16, P, 4, None, None, 0, 0, 5, 8, 64, 16, None) == NULL_POINTER
    assert sc(P, P, F16, P, P, F16, P, 4, None, None, -1, 0, 5, 8, 64, 16, None) == BAD_SHAPE
    assert sc(P, P, 9, P, P, F16, P, 4, None, None, 0, 0, 5, 8, 64, 16, None) == BAD_DTYPE
    ga = lib.ahpc_hip_kv_gather
    assert ga(P, P, F16, P, P, F16, P, 4, 0, 0, 0, 8, 64, 16, None) == 0
    assert ga(P, P, F16, P, P, F16, P, 4, 0, 60, 10, 8, 64, 16, None) == BAD_SHAPE                 # past the row's last page
    sb = lib.ahpc_hip_kv_scatter_batch
    assert sb(P, P, F16, 0, 8 * 64, P, P, F16, P, 4, P, None, None, None, 0, 16, 8, 64, 16, None) == 0
    assert sb(P, P, F16, 0, 8 * 64, P, P, F16, P, 4, None, None, None, None, 2, 16, 8, 64, 16, None) == NULL_POINTER
    assert sb(P, P, F16, 0, 100, P, P, F16, P, 4, P, None, None, None, 2, 16, 8, 64, 16, None) == BAD_SHAPE  # rows overlap
    assert sb(P, P, F16, 0, 8 * 64, P, P, 4, P, 4, P, None, None, None, 2, 16, 8, 64, 16, None) == BAD_DTYPE
    mv = lib.ahpc_hip_kv_move_pages
    assert mv(P, P, F16, 64, P, P, 0, 8, 64, 16, None) == 0                                        # nothing to move
    assert mv(P, None, F16, 64, P, P, 3, 8, 64, 16, None) == NULL_POINTER and mv(P, P, F16, 64, None, P, 3, 8, 64, 16, None) == NULL_POINTER
    assert mv(P, P, 7, 64, P, P, 3, 8, 64, 16, None) == BAD_DTYPE and mv(P, P, F16, 0, P, P, 3, 8, 64, 16, None) == BAD_SHAPE
    gi = lib.ahpc_hip_paged_gather_indices
    assert gi(P, P, None, 2, 8, 64, 16, 4, 64, None, None) == NULL_POINTER
    assert gi(P, P, None, 2, 8, 64, 16, 4, 65, P, None) == BAD_SHAPE
    assert gi(P, P, None, 2, 8, 64, 4096, 1 << 20, (1 << 31) + 4096, P, None) == BAD_SHAPE


def test_error_strings_cover_every_code(lib):
    from attention_amd import hip
    seen = set()
    for code in range(0, -9, -1):
        text = hip.error_string(code)
        assert text and text != "unknown error code", code
        seen.add(text)
    assert len(seen) == 9
    assert hip.error_string(-99) == "unknown error code"
