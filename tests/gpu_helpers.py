"""Plumbing for the GPU parity tests: load the HIP library through its C ABI and move numpy arrays to HBM."""
import importlib

import numpy as np

tfk = importlib.import_module("turbo-fieldfare_amd")

_ctx = None


def ctx():
    global _ctx
    if _ctx is None:
        _ctx = tfk.Context(0)
    return _ctx


def dev(a, byte_offset: int = 0):
    """numpy array -> uint8 CUDA tensor holding its bytes at `byte_offset` inside a padded allocation."""
    import torch
    raw = np.ascontiguousarray(a).view(np.uint8).ravel()
    if byte_offset:
        raw = np.concatenate([np.full(byte_offset, 0xA5, np.uint8), raw, np.full(32, 0x5A, np.uint8)])
    return torch.from_numpy(raw.copy()).cuda()


def zeros_bytes(n: int, fill: int = 0):
    import torch
    return torch.full((n,), fill, dtype=torch.uint8, device="cuda")


def host(t, dtype, count=None, byte_offset: int = 0):
    import torch
    torch.cuda.synchronize()
    raw = t.cpu().numpy().view(np.uint8)[byte_offset:]
    out = raw.view(dtype) if raw.size % np.dtype(dtype).itemsize == 0 else raw[: raw.size // np.dtype(dtype).itemsize * np.dtype(dtype).itemsize].view(dtype)
    return out[:count].copy() if count is not None else out.copy()


def within_north_star(actual, reference, rel=1e-2, abs_=1e-3):
    """BASELINE tolerance: |a - r| <= 1e-3 + 1e-2 * |r| elementwise."""
    a = np.asarray(actual, np.float64)
    r = np.asarray(reference, np.float64)
    return bool(np.all(np.abs(a - r) <= abs_ + rel * np.abs(r)))


class _RawDeviceArray:
    """Exposes a raw device pointer to torch through the CUDA array interface (read-only use in tests)."""

    def __init__(self, ptr: int, count: int, typestr: str):
        self.__cuda_array_interface__ = {"shape": (count,), "typestr": typestr, "data": (ptr, False), "version": 2}


def device_view(ptr: int, count: int, typestr: str):
    """Copy `count` elements starting at a library-owned device pointer back to the host."""
    import torch
    torch.cuda.synchronize()
    return torch.as_tensor(_RawDeviceArray(ptr, count, typestr), device="cuda").cpu().numpy().copy()
