"""The known-answer vectors of tests/golden/*.npz on the GPU, through the C ABI (forward and decode; the backward ones
are in tests/test_zzz_gpu_flash_bwd.py)."""
import os

import numpy as np
import pytest

from oracle import oracle as O
from test_golden_vectors import FILES, load, dense_inputs, decode_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("path", [f for f in FILES if "dense" in os.path.basename(f)], ids=os.path.basename)
def test_dense_forward_vectors(gpu, path):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr
    c = load(path)
    (B, N, H, Hkv, d), q, k, v, _, mask = dense_inputs(c)
    tq, tk, tv = (to_dev(x, O.F32) for x in (q, k, v))
    to = torch.full_like(tq, float("nan"))
    tm = None if mask is None else torch.from_numpy(mask).cuda()
    gpu.flash_fwd_gqa(tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), to.data_ptr(), O.F32, B, N, H, Hkv, d, (N * H * d, H * d, d),
                      (N * Hkv * d, Hkv * d, d), float(c["scale"]), bool(c["causal"]), stream_ptr(),
                      None if tm is None else tm.data_ptr())
    torch.cuda.synchronize()
    assert np.abs(to_host(to) - c["o"]).max() <= 1e-4


@pytest.mark.parametrize("path", [f for f in FILES if "decode" in os.path.basename(f)], ids=os.path.basename)
def test_decode_vectors(gpu, path):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32
    c = load(path)
    (B, H, Hkv, d, P), q, kp, vp, table, lens = decode_inputs(c)
    tq, tk, tv = (to_dev(x, O.F32) for x in (q, kp, vp))
    to = torch.full_like(tq, float("nan"))
    tt, tl = dev_i32(table), dev_i32(lens)
    max_len = int(lens.max())
    ws_bytes = gpu.paged_decode_workspace_bytes(B, H, d, max_len, P, P)
    ws = torch.full((max(ws_bytes, 4) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    # chunks of one page: every context is split and merged
    gpu.paged_decode_gqa(tq.data_ptr(), to.data_ptr(), O.F32, tk.data_ptr(), tv.data_ptr(), O.F32, tt.data_ptr(), tl.data_ptr(),
                         None, B, H, Hkv, d, P, table.shape[1], max_len, float(c["scale"]), P, ws.data_ptr(), ws_bytes,
                         stream_ptr())
    torch.cuda.synchronize()
    assert np.abs(to_host(to) - c["o"]).max() <= 1e-4
