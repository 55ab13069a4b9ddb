"""Helpers for the GPU parity tests: device buffers come from torch (plumbing only); every compute
call goes through the C ABI (attention_amd.hip)."""
import numpy as np
import pytest

from oracle import oracle as O

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
