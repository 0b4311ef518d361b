"""Plumbing for the GPU parity tests: device buffers (torch) + calls through the C ABI."""
import ctypes as C

import numpy as np

from smallframework_amd import capi


def torch_mod():
    import torch
    return torch


def dev(a):
    """numpy -> device tensor (flat)."""
    torch = torch_mod()
    return torch.from_numpy(np.ascontiguousarray(a).ravel()).to("cuda")


def dev_empty(n, dtype):
    torch = torch_mod()
    td = {np.float32: torch.float32, np.uint8: torch.uint8}[dtype]
    return torch.empty(int(n), dtype=td, device="cuda")


def host(t):
    torch_mod().cuda.synchronize()
    return t.cpu().numpy()


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def stream():
    return C.c_void_p(torch_mod().cuda.current_stream().cuda_stream)


def q(zero=0, multiplier=1 << 30, lshift=0, rshift=0):
    return capi.Quant(zero, multiplier, lshift, rshift)


def qref(x):
    return C.byref(x)
