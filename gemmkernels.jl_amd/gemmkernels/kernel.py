"""Kernels (reference src/kernel.jl).  The three names are kept; on gfx950 all of them run the
LDS-DMA software pipeline for tile-sized aligned layouts, and ``matmul_singlestage`` is the one
that accepts bounds-checked layouts and honours ``threadblock_condition`` (diagonal A)."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

from . import _lib
from .errors import ConfigError


@dataclass(frozen=True)
class KernelKind:
    code: int
    name: str

    def __repr__(self):
        return f"Kernel.{self.name}"


matmul_singlestage = KernelKind(0, "matmul_singlestage")     # src/kernel.jl:10-129
matmul_pipelined = KernelKind(1, "matmul_pipelined")         # src/kernel.jl:147-350
matmul_pipelined_ng = KernelKind(2, "matmul_pipelined_ng")   # src/kernel.jl:368-574
# no counterpart in the reference: the pipelined kernel with the K range cut into slices that run as
# separate workgroups of one launch, for problems with too few output tiles to fill the chip; the slices of
# a tile meet in a workspace and are added in slice order, so results do not change from run to run
matmul_split_k = KernelKind(3, "matmul_split_k")


def shmem_size(conf, kernel: KernelKind = matmul_singlestage) -> int:
    """LDS bytes requested by the kernel instance of ``conf`` (src/kernel.jl:131-145, 352-366, 576-590)."""
    c = conf.to_c()
    n = _lib.lib().gk_shmem_size(ctypes.byref(c), kernel.code)
    if n < 0:
        raise ConfigError(_lib.last_error(), _lib.GK_ERR_UNSUPPORTED)
    return int(n)


def reference_shmem_size(conf) -> int:
    """The reference's own formula (src/kernel.jl:131-145, 352-366): max(size_c, size_a + size_b, size_d)
    over the shared layouts of ``conf`` in their physical sizes.  Host arithmetic only."""
    c = conf.to_c()
    n = _lib.lib().gk_reference_shmem_size(ctypes.byref(c))
    if n < 0:
        raise ConfigError(_lib.last_error(), _lib.GK_ERR_INVALID_ARGUMENT)
    return int(n)
