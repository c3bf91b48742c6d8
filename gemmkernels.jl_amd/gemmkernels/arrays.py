"""Column-major device arrays on top of torch tensors (memory and streams only)."""
from __future__ import annotations

import numpy as np


def colmajor_empty(shape, dtype, device="cuda"):
    """An uninitialised column-major (first index fastest) tensor of the given logical shape."""
    import torch
    return torch.empty(tuple(reversed(shape)), dtype=dtype, device=device).permute(*reversed(range(len(shape))))


def colmajor(array: np.ndarray, dtype=None, device="cuda"):
    """Copy a numpy array to the device in column-major order, keeping its logical shape.
    float16 complex data is passed as a real array with a trailing dimension of 2."""
    import torch
    t = torch.from_numpy(np.ascontiguousarray(array.transpose()))   # C-order of the transpose == F-order
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
