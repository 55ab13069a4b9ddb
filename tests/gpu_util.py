"""Helpers for the GPU parity tests: device buffers come from torch (plumbing only); every compute
call goes through the C ABI (attention_amd.hip)."""
import os

import numpy as np
import pytest

from oracle import oracle as O

# Kernels that have so far run only on the CPU executor (tests/simt) get their first run on hardware by hand:
# one case at a time, each under its own time limit, with AHPC_GPU_FIRST_RUN=1.  An unattended run of the
# suite leaves their launching tests out until that has happened, because a kernel that misbehaves on its
# first run can take the whole machine with it and hide the results of every established test.
first_hardware_run = pytest.mark.skipif(
    os.environ.get("AHPC_GPU_FIRST_RUN") != "1",
    reason="kernel verified on the CPU executor only; its first run on hardware is made by hand (AHPC_GPU_FIRST_RUN=1)")

TOL = {O.F32: 1e-4, O.F16: 2e-2, O.BF16: 2e-2}  # max-abs bars: fp32 vs oracle, 16-bit vs fp32 oracle


def torch_dtype(code):
    import torch
    return {O.F32: torch.float32, O.F16: torch.float16, O.BF16: torch.bfloat16}[code]


def to_dev(x_f32, code):
    """fp32 numpy (already representable in `code`) -> device tensor of that storage type."""
    import torch
    t = torch.from_numpy(np.ascontiguousarray(x_f32, np.float32))
    return t.to(torch_dtype(code)).cuda()


def to_host(t):
    import torch
    return t.detach().to(torch.float32).cpu().numpy()


def stream_ptr():
    import torch
    return torch.cuda.current_stream().cuda_stream


def dev_i32(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a, np.int32)).cuda()
