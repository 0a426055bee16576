"""Helpers shared by the GPU parity tests: load the product through its C ABI, move oracle
arrays (numpy, 16-bit floats as uint16 bit patterns) to the device and back."""
import importlib

import numpy as np

import oracle as orc

mynn = importlib.import_module("my-nn-engine_amd")

TOL = {orc.F32: 2e-5, orc.BF16: 1e-2, orc.F16: 1e-2}  # max-abs-rel bound for float outputs


def torch_dtype(dt):
    import torch

    return {orc.F32: torch.float32, orc.BF16: torch.bfloat16, orc.F16: torch.float16}[dt]


def to_dev(a, dt=None):
    """numpy storage array -> cuda tensor (uint16 bit patterns become bf16/f16 per dt)."""
    import torch

    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        t = torch.from_numpy(a.view(np.int16)).cuda().view(torch_dtype(dt))
    else:
        t = torch.from_numpy(a).cuda()
    return t


def to_host(t):
    """cuda tensor -> numpy storage array (bf16/f16 come back as uint16 bit patterns)."""
    import torch

    t = t.detach().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def f32(a, dt):
    return orc.to_f32(a, dt)
