"""Column-major device arrays on top of torch tensors (memory and streams only)."""
from __future__ import annotations

import numpy as np


def colmajor_empty(shape, dtype, device="cuda"):
    """An uninitialised column-major (first index fastest) tensor of the given logical shape."""
    import torch
    return torch.empty(tuple(reversed(shape)), dtype=dtype, device=device).permute(*reversed(range(len(shape))))


def colmajor(array: np.ndarray, dtype=None, device="cuda"):
    """Copy a numpy array to the device in column-major order, keeping its logical shape.
    float16 complex data is passed as a real array with a trailing dimension of 2; bfloat16 data as
    uint16 bit patterns together with dtype=torch.bfloat16."""
    import torch
    host = np.ascontiguousarray(array.transpose())                   # C-order of the transpose == F-order
    if host.dtype == np.uint16 and dtype is torch.bfloat16:
        t = torch.from_numpy(host.view(np.int16)).view(torch.bfloat16)   # bit patterns, not values
    else:
        t = torch.from_numpy(host)
        if dtype is not None:
            t = t.to(dtype)
    t = t.to(device)
    return t.permute(*reversed(range(t.dim())))


def to_numpy(t) -> np.ndarray:
    """Device tensor (any strides) -> numpy array with the same logical shape."""
    import torch
    if t.dtype == torch.bfloat16:
        t = t.to(torch.float32)
    return t.detach().cpu().numpy()


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 values -> bfloat16 bit patterns (uint16), round to nearest even; keeps the memory order."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32)
    return ((u + (((u >> 16) & 1) + 0x7FFF)) >> 16).astype(np.uint16)


def bf16_values(bits: np.ndarray) -> np.ndarray:
    """bfloat16 bit patterns (uint16) -> float32 values; keeps the memory order."""
    return (np.asarray(bits).astype(np.uint32, order="K") << 16).view(np.float32)
