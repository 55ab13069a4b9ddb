"""The opt-in forward kernels and tuning knobs on the GPU, through the C ABI: each must reproduce the standard kernel
bit for bit (same arithmetic per wavefront, different schedule or workgroup order).  Collected after the established GPU
tests; the kernels that have run on the CPU executor only wait for a first run by hand (gpu_util.first_hardware_run)."""
import numpy as np
import pytest

from oracle import oracle as O
from gpu_util import first_hardware_run

pytestmark = pytest.mark.gpu


def forward(hip, q, k, v, dtype, B, N, H, d, scale, causal):
    import torch
    from gpu_util import to_dev, to_host, stream_ptr
    tq, tk, tv = (to_dev(x, dtype) for x in (q, k, v))
    to = torch.full_like(tq, float("nan"))
    hip.flash_fwd(tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), to.data_ptr(), dtype, B, N, H, d, (N * H * d, H * d, d), scale,
                  causal, stream_ptr())
    torch.cuda.synchronize()
    return to_host(to)


SHAPES = [(O.BF16, 2, 700, 3, 128, True), (O.F16, 1, 520, 2, 64, False), (O.BF16, 1, 2048 + 96, 16, 128, True),
          (O.F16, 2, 257, 2, 128, False)]


@first_hardware_run
@pytest.mark.parametrize("knob,value", [("AHPC_FLASH_PINGPONG", "1"), ("AHPC_FLASH_PINGPONG", "2"), ("AHPC_FLASH_VARIANT", "1"),
                                        ("AHPC_FLASH_VARIANT", "2"), ("AHPC_FLASH_VARIANT", "3"), ("AHPC_FLASH_VARIANT", "4"),
                                        ("AHPC_FLASH_VARIANT", "6"), ("AHPC_FLASH_HEADS_TOGETHER", "4")])
@pytest.mark.parametrize("dtype,B,N,H,d,causal", SHAPES)
def test_knob_reproduces_the_standard_kernel(gpu, dtype, B, N, H, d, causal, knob, value, monkeypatch):
    q, k, v = (O.round_to(O.fill_normal((B, N, H, d), 41, t), dtype) for t in (1, 2, 3))
    scale = 1.0 / np.sqrt(d)
    plain = forward(gpu, q, k, v, dtype, B, N, H, d, scale, causal)
    assert np.abs(plain - O.attention(q, k, v, B, N, H, d, scale, causal)).max() <= 2e-2
    monkeypatch.setenv(knob, value)
    got = forward(gpu, q, k, v, dtype, B, N, H, d, scale, causal)
    assert np.isfinite(got).all()
    assert np.array_equal(got, plain), (knob, value, float(np.abs(got - plain).max()))


@first_hardware_run
@pytest.mark.parametrize("mode", ["1", "2"])
@pytest.mark.parametrize("dtype,d", [(O.F16, 64), (O.BF16, 128)])
def test_alternating_kernel_on_a_ragged_batch(gpu, dtype, d, mode, monkeypatch):
    """Packed sequences (cu_seqlens), causal: the alternating kernel against the oracle and, bit for bit, the standard one."""
    import torch
    from gpu_util import to_dev, to_host, stream_ptr, dev_i32
    H = 4
    lens = np.array([1, 130, 64, 700, 257, 1500], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    q, k, v = (O.round_to(O.fill_normal((T, H, d), 43, t), dtype) for t in (1, 2, 3))
    tq, tk, tv = (to_dev(x, dtype) for x in (q, k, v))
    tcu = dev_i32(cu)
    scale = 1.0 / np.sqrt(d)
    outs = []
    for knob in (None, mode):
        if knob:
            monkeypatch.setenv("AHPC_FLASH_PINGPONG", knob)
        to = torch.full_like(tq, float("nan"))
        gpu.flash_fwd_varlen(tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), to.data_ptr(), dtype, tcu.data_ptr(), len(lens),
                             int(lens.max()), H, d, H * d, d, scale, True, stream_ptr())
        torch.cuda.synchronize()
        outs.append(to_host(to))
    assert np.abs(outs[1] - O.attention_varlen(q, k, v, cu, H, d, scale, True)).max() <= 2e-2
    assert np.array_equal(outs[0], outs[1])
