"""CTA swizzles: blockIdx -> tile origin (reference src/cta-swizzle.jl).

The maps are evaluated by the library (``gk_cta_swizzle`` runs the very function the kernels
inline), so what is tested on the host is what the device executes.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

from . import _lib
from .errors import ConfigError
from .tiling import NT

IDENTITY, HORIZONTALLY_TILED, VERTICALLY_TILED, LEBESGUE, XCD = range(5)
_NAMES = {IDENTITY: "Identity", HORIZONTALLY_TILED: "HorizontallyTiled", VERTICALLY_TILED: "VerticallyTiled",
          LEBESGUE: "LebesgueCurve", XCD: "XCDAware"}


@dataclass(frozen=True)
class SwizzleType:
    kind: int
    param: int = 0

    def __repr__(self):
        return f"CTASwizzle.{_NAMES[self.kind]}" + (f"{{{self.param}}}" if self.param else "")


class _Tiled:
    def __init__(self, kind):
        self.kind = kind

    def __getitem__(self, tile_size: int) -> SwizzleType:
        return SwizzleType(self.kind, int(tile_size))


Identity = SwizzleType(IDENTITY)                 # src/cta-swizzle.jl:26-41
HorizontallyTiled = _Tiled(HORIZONTALLY_TILED)   # :67-82
VerticallyTiled = _Tiled(VERTICALLY_TILED)       # :102-117
LebesgueCurve = SwizzleType(LEBESGUE)            # :147-160
# MI355X: workgroup n of a launch lands on XCD n % 8 and each XCD has its own L2.  XCDAware[G]
# regroups consecutive ids per XCD, then walks the tile grid in panels G tiles high.
XCDAware = _Tiled(XCD)


def _mini_config(swizzle: SwizzleType, block_shape, matmul_shape) -> _lib.gk_config:
    c = _lib.gk_config()
    c.matmul_shape.M, c.matmul_shape.N = int(matmul_shape["M"]), int(matmul_shape["N"])
    c.block_shape.M, c.block_shape.N = int(block_shape["M"]), int(block_shape["N"])
    c.cta_swizzle.kind, c.cta_swizzle.param = swizzle.kind, swizzle.param
    return c


def number_of_blocks(swizzle: SwizzleType, block_shape, matmul_shape):
    """Grid dimensions (x, y) of the launch."""
    c = _mini_config(swizzle, block_shape, matmul_shape)
    bx, by = ctypes.c_int32(), ctypes.c_int32()
    rc = _lib.lib().gk_number_of_blocks(ctypes.byref(c), ctypes.byref(bx), ctypes.byref(by))
    if rc != 0:
        raise ConfigError(_lib.last_error(), rc)
    return bx.value, by.value


def cta_swizzle(swizzle: SwizzleType, blockIdx, block_shape, matmul_shape=None):
    """(block_i, block_j): element offsets of the tile of the 1-based ``blockIdx`` (``.x``, ``.y``),
    as in the reference.  ``matmul_shape`` is needed by XCDAware, which depends on the grid."""
    if matmul_shape is None:
        matmul_shape = NT(M=1 << 30, N=1 << 30)
    c = _mini_config(swizzle, block_shape, matmul_shape)
    bi, bj = ctypes.c_int32(), ctypes.c_int32()
    rc = _lib.lib().gk_cta_swizzle(ctypes.byref(c), int(blockIdx["x"]) - 1, int(blockIdx["y"]) - 1,
                                   ctypes.byref(bi), ctypes.byref(bj))
    if rc != 0:
        raise ConfigError(_lib.last_error(), rc)
    return bi.value, bj.value


def visualise_cta_swizzle(swizzle: SwizzleType, block_shape=None, matmul_shape=None):
    """reference src/cta-swizzle.jl:7-19: which (bx, by) computes each tile, as a 2-D list of strings."""
    block_shape = NT(M=128, N=128) if block_shape is None else block_shape
    matmul_shape = NT(M=1024, N=1024) if matmul_shape is None else matmul_shape
    rows = -(-matmul_shape["M"] // block_shape["M"])
    cols = -(-matmul_shape["N"] // block_shape["N"])
    res = [["" for _ in range(cols)] for _ in range(rows)]
    BX, BY = number_of_blocks(swizzle, block_shape, matmul_shape)
    for bx in range(1, BX + 1):
        for by in range(1, BY + 1):
            bi, bj = cta_swizzle(swizzle, NT(x=bx, y=by), block_shape, matmul_shape)
            i, j = bi // block_shape["M"], bj // block_shape["N"]
            if i < rows and j < cols:
                res[i][j] = f"({bx}, {by})"
    return res
