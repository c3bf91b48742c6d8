"""Config and get_config (reference src/config.jl), with defaults re-derived for the MI355X:
64-lane wavefronts, 160 KiB of LDS per workgroup, MFMA 32x32x16 blocks."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, fields
from typing import Optional

from . import _lib
from . import layout as Layout
from . import operator as Operator
from . import cta_swizzle as CTASwizzle
from .errors import ConfigError
from .tiling import NT

WARP_SIZE = 64   # lanes per wavefront; the reference's 32 (src/matmul.jl:24) becomes 64 here


@dataclass
class Config:
    """reference src/config.jl:3-41, field for field."""
    matmul_shape: NT
    block_shape: NT
    warps_per_block: int
    mem_a_warp: NT
    mem_a_thread: NT
    mem_b_warp: NT
    mem_b_thread: NT
    mem_cd_warp: NT
    mem_cd_thread: NT
    compute_warp: NT
    compute_op_shape: NT
    global_a_layout: Layout.LayoutType
    global_b_layout: Layout.LayoutType
    global_c_layout: Layout.LayoutType
    global_d_layout: Layout.LayoutType
    shared_a_layout: Layout.LayoutType
    shared_b_layout: Layout.LayoutType
    shared_c_layout: Layout.LayoutType
    shared_d_layout: Layout.LayoutType
    operator: Operator.OperatorType
    is_a_col_major: bool
    is_b_col_major: bool
    cta_swizzle: CTASwizzle.SwizzleType

    def __str__(self):
        # reference src/config.jl:43-76
        width = max(len(f.name) for f in fields(self)) + 2
        return "\n".join(f"{(f.name + ':').ljust(width)}{getattr(self, f.name)}" for f in fields(self)) + "\n"

    def to_c(self, lda: int = 0, ldb: int = 0, ldc: int = 0, ldd: int = 0) -> _lib.gk_config:
        """Lower to the POD of the C ABI; leading dimensions come from the arrays of the call.
        The result is cached per set of leading dimensions (a Config is immutable once built)."""
        cache = self.__dict__.setdefault("_c_cache", {})
        key = (lda, ldb, ldc, ldd)
        hit = cache.get(key)
        if hit is not None:
            return hit
        c = _lib.gk_config()
        cache[key] = c

        def shape(dst, src):
            dst.M, dst.N, dst.K = int(src.get("M", 0)), int(src.get("N", 0)), int(src.get("K", 0))

        shape(c.matmul_shape, self.matmul_shape)
        shape(c.block_shape, self.block_shape)
        c.warps_per_block = int(self.warps_per_block)
        for name in ("mem_a_warp", "mem_a_thread", "mem_b_warp", "mem_b_thread", "mem_cd_warp", "mem_cd_thread",
                     "compute_warp", "compute_op_shape"):
            shape(getattr(c, name), getattr(self, name))

        def lay(dst, src: Layout.LayoutType, ld=0):
            dst.kind, dst.eltype, dst.pad, dst.ld = src.kind, src.T.code, src.pad, int(ld)

        lay(c.global_a_layout, self.global_a_layout, lda)
        lay(c.global_b_layout, self.global_b_layout, ldb)
        lay(c.global_c_layout, self.global_c_layout, ldc)
        lay(c.global_d_layout, self.global_d_layout, ldd)
        lay(c.shared_a_layout, self.shared_a_layout)
        lay(c.shared_b_layout, self.shared_b_layout)
        lay(c.shared_c_layout, self.shared_c_layout)
        lay(c.shared_d_layout, self.shared_d_layout)
        op = self.operator
        c.op.kind, c.op.M, c.op.N, c.op.K = op.kind, op.M, op.N, op.K
        c.op.mb, c.op.nb, c.op.kb = op.mb, op.nb, op.kb
        c.op.compute_type, c.op.accum_type = op.CT.code, op.AT.code
        c.is_a_col_major, c.is_b_col_major = int(self.is_a_col_major), int(self.is_b_col_major)
        c.cta_swizzle.kind, c.cta_swizzle.param = self.cta_swizzle.kind, self.cta_swizzle.param
        gmap = None
        for l in (self.global_a_layout, self.global_b_layout, self.global_c_layout, self.global_d_layout):
            if l.kind == Layout.GETT_KIND and l.gett is not None:
                gmap = l.gett
        if gmap is not None:
            for dst, src in ((c.gett.m, gmap.m), (c.gett.n, gmap.n), (c.gett.k, gmap.k)):
                if len(src) > _lib.GK_MAX_MODES:
                    raise ConfigError(f"at most {_lib.GK_MAX_MODES} tensor modes per GEMM dimension")
                dst.nmodes = len(src)
                for i, (e, s0, s1) in enumerate(src):
                    dst.extent[i], dst.stride0[i], dst.stride1[i] = int(e), int(s0), int(s1)
        return c


def heuristic_block_shape(shared_a_layout, shared_b_layout, shared_c_layout, shared_d_layout) -> NT:
    """The reference's block-shape heuristic, unchanged (src/config.jl:84-120): grow M and N while
    a C/D tile fits 64 KiB, then K while the A and B tiles fit 64 KiB together."""
    def nbytes(layout, a, b):
        size = Layout.physical_size(layout, (a, b))
        n = 1
        for s in size:
            n *= s
        return n * layout.T.size

    def num_bytes_cd(M, N, K):
        return max(nbytes(shared_c_layout, M, N), nbytes(shared_d_layout, M, N))

    def num_bytes_ab(M, N, K):
        return nbytes(shared_a_layout, M, K) + nbytes(shared_b_layout, K, N)

    def next_mn(M, N, K):
        return (2 * M, N, K) if M == N else (M, 2 * N, K)

    cur = (1, 1, 1)
    nxt = next_mn(*cur)
    while num_bytes_cd(*nxt) <= 64 * 1024:
        cur, nxt = nxt, next_mn(*nxt)
    nxt = (cur[0], cur[1], 2 * cur[2])
    while num_bytes_ab(*nxt) <= 64 * 1024:
        cur, nxt = nxt, (nxt[0], nxt[1], 2 * nxt[2])
    return NT(M=cur[0], N=cur[1], K=cur[2])


def adjacent_elements(num: int, parent_size: NT, is_col_major: bool) -> NT:
    """reference src/config.jl:124-134."""
    p = tuple(parent_size.values())
    if is_col_major:
        t = (min(num, p[0]), num // min(num, p[0]))
    else:
        t = (num // min(num, p[1]), min(num, p[1]))
    return NT(zip(parent_size.keys(), t))


# MFMA tile table of the library: block shape -> waves (M x N).  The wave tile (compute_warp) is
# block / waves; every entry is made of 32x32 MFMA blocks.
_MFMA_TILES = [
    ((256, 256, 64), (2, 4)),
    ((256, 256, 32), (2, 4)),     # for K that is a multiple of 32 only (6 % behind 256x256x64; 4 x 2 waves: 10 %)
    ((256, 128, 64), (2, 2)),
    ((128, 256, 64), (2, 2)),
    ((128, 128, 32), (2, 2)),     # four stages: measured ahead of 128x128x64 with two stages on 2048-sized problems
    ((128, 128, 64), (2, 2)),
    ((64, 64, 64), (2, 2)),
    ((64, 64, 32), (2, 2)),       # four stages; the one-wave instance (the tensor-contraction kernels have only that) is 1.5 - 2.7 times slower
]
# Tiles with a side of 192: they fill the chip where 256 x 256 leaves CUs idle (3072^2: 192 tiles instead of 144,
# 56 us instead of 68).  Compiled per transpose: 256 x 192 for 'N','N', 'T','N' and 'N','T'; 192 x 256 for
# 'T','N' and 'T','T' (the third entry says whether a transpose (a_kmajor, b_kmajor) has the tile).
_MFMA_TILES_192 = [((256, 192, 64), (4, 2), lambda a_kmajor, b_kmajor: b_kmajor or not a_kmajor),
                   ((192, 256, 64), (2, 4), lambda a_kmajor, b_kmajor: a_kmajor)]
NUM_CUS = 256

# measured winners by problem (filled by gemmkernels.tuning.install / load, or from the JSON file
# named by the environment variable GEMMKERNELS_TUNING_TABLE)
TUNED = {}


# tiles compiled with tensor-contraction addressing
_GETT_TILES = [(256, 256, 64), (128, 128, 64), (64, 64, 32)]


def default_block_shape(operator, gemm_shape, tile_sized: bool = True, gett: bool = False, planar: bool = False,
                        a_kmajor: bool = False, b_kmajor: bool = True) -> NT:
    """MI355X block shape: of the tiles of the table that divide the problem, the one with the shortest
    estimated launch (tiles per CU times the cost of a tile).  ``a_kmajor``: A is stored K x M ('T');
    ``b_kmajor``: B is stored K x N ('N'); they admit the tiles with a side of 192."""
    M, N, K = gemm_shape["M"], gemm_shape["N"], gemm_shape["K"]
    if operator.kind in (Operator.FPU, Operator.FPU_TROPICAL):
        # a small Float32 product in whole 32 x 32 x 32 tiles: four times the workgroups of the 64 x 64 tile
        # (256^3: 64 workgroups instead of 16) with 2 x 2 outputs per lane on four waves, so that a lane works
        # through 4 fma chains instead of 16 (every output is still one fma chain in k: the same bits)
        if (operator.kind == Operator.FPU and operator.CT.name == "Float32" and operator.AT.name == "Float32" and tile_sized
                and M % 32 == 0 and N % 32 == 0 and K % 32 == 0 and -(-M // 64) * -(-N // 64) < NUM_CUS // 2):
            return NT(M=32, N=32, K=32)
        return NT(M=64, N=64, K=32)
    if operator.kind in (Operator.MFMA_COMPLEX, Operator.MFMA_DUAL):
        # complex tiles, in complex elements
        table = _complex_tiles(operator, planar, a_kmajor, b_kmajor)
        fitting = [t for t, _ in table if M % t[0] == 0 and N % t[1] == 0 and K % t[2] == 0]
        for t in fitting:
            if (M // t[0]) * (N // t[1]) >= NUM_CUS:
                return NT(M=t[0], N=t[1], K=t[2])
        t = fitting[-1] if fitting else (64, 64, 32)
        return NT(M=t[0], N=t[1], K=t[2])
    # sizes need not be whole tiles when the layouts are the bounds-checked ones (the aligned kernels mask the
    # last tile row / column and zero the end of the last K tile)
    table = [t for t, _ in _MFMA_TILES] + [t for t, _, has in _MFMA_TILES_192 if has(a_kmajor, b_kmajor)]
    fitting = [t for t in table if not tile_sized or (M % t[0] == 0 and N % t[1] == 0 and K % t[2] == 0)]
    if gett:
        fitting = [t for t in fitting if t in _GETT_TILES]
    if not fitting:
        return NT(M=64, N=64, K=32)
    # time of the launch in units of "one CU multiplying at the rate of the 256 x 256 x 64 tile": a tile costs its area
    # over the rate of its kernel when it has a CU to itself (_MFMA_TILE_RATE), and a CU works through its share of the
    # tiles in rounds (_rounds: whole rounds for the tiles of which a CU holds one at a time, overlapping ones for the
    # smaller tiles).  Ties go to the tile listed first.
    def cost(t):
        tiles = -(-M // t[0]) * -(-N // t[1])
        per_cu = tiles / NUM_CUS
        rate = _MFMA_TILE_RATE.get(t, 0.3)
        if isinstance(rate, tuple):
            rate = rate[0] if per_cu <= 1 else rate[1]
        if t == (256, 192, 64) and not a_kmajor and not b_kmajor and (M % t[0] or N % t[1] or K % t[2]):
            rate = 0.70      # 'N','T' on eight waves (tiles over the edges): the 192 side is read with transposing LDS reads
        if t == (64, 64, 32) and per_cu <= 1 and K >= 2048:
            rate = 0.24      # a lone workgroup on a long K: four stages in flight instead of two (1024 x 1024 x 4096: 23.4 us, 64 x 64 x 64: 34.1)
        return _rounds(t, tiles) * t[0] * t[1] / rate
    best = min(fitting, key=lambda t: (cost(t), fitting.index(t)))
    return NT(M=best[0], N=best[1], K=best[2])


# Throughput of a CU that has one tile at a time, relative to 256 x 256 x 64 on four waves; a pair: a launch with at most
# one tile per CU, a launch with several (the small tiles are bound by latency when alone).  From timings of every tile
# and panel height at 1024^3 ... 6144^3 and eight rectangular problems ('N','N', three interleaved passes each):
# e.g. 4096^3 takes 99 us on 256 x 256 x 64, 131 on 128 x 128 x 64, 134 on 128 x 256 x 64, 194 on 64 x 64 x 64;
# 2560^3 42.2 us on 128 x 128 x 64 (400 tiles), 45.5 on 128 x 256 x 64 (200), 53.1 on 256 x 256 x 64 (100).
_MFMA_TILE_RATE = {(256, 256, 64): 1.0, (256, 256, 32): 0.68, (256, 128, 64): (0.61, 0.70), (128, 256, 64): (0.62, 0.72),
                   (128, 128, 32): (0.415, 0.345), (128, 128, 64): 0.39, (64, 64, 64): 0.169, (64, 64, 32): (0.163, 0.13),
                   (256, 192, 64): 0.86, (192, 256, 64): 0.86}


def _rounds(t, tiles):
    """How many tile times a launch of ``tiles`` tiles of shape ``t`` takes.  A CU holds one workgroup of the tiles with
    144 or 128 KiB of LDS at a time: whole rounds.  Of the 128 x 128 tiles it holds two, which run side by side in 1.15
    times the time of one (2560^3, 400 tiles: 1.17; 4096^3, 1024 tiles: 2.27 = two such rounds); of the 64 x 64 tiles
    four and more, whose time grows by about a third of a tile time per further tile of a CU (1536^3, 2.25 per CU: 1.43;
    3072^3, 9 per CU: 3.8)."""
    per_cu = tiles / NUM_CUS
    if t[0] * t[1] >= 128 * 256:
        return -(-tiles // NUM_CUS)
    if per_cu <= 1:
        return 1.0
    if t[0] * t[1] >= 128 * 128:
        return 1.15 * -(-tiles // (2 * NUM_CUS))
    return 1.0 + 0.36 * (per_cu - 1.0)


# complex / dual tiles (complex elements) -> waves: one real product of the real views of A and B, whose real tile
# has twice the rows and columns; the same table for every transpose
_COMPLEX_PAIR_TILES = [((128, 128, 64), (2, 4)), ((64, 64, 64), (2, 2)), ((64, 64, 32), (2, 2)), ((32, 32, 32), (2, 2))]

# complex tiles (complex elements) of the kernel for planar global matrices -> waves; the real tile has twice
# the rows and columns (both planes of A, B and D)
_PLANAR_TILES = [((128, 128, 64), (2, 4)), ((64, 64, 64), (2, 2)), ((64, 64, 32), (2, 2)), ((32, 32, 32), (2, 2))]

# tiles of the vector-ALU kernel and of the bounds-checked MFMA kernel
_FPU_TILES = [((64, 64, 32), (2, 2)), ((128, 128, 16), (2, 2)), ((32, 32, 32), (2, 2)), ((32, 32, 32), (1, 1))]
_CHECKED_TILES = [((64, 64, 32), (2, 2))]


def _complex_tiles(operator, planar, a_kmajor, b_kmajor):
    """(tile, waves) of the complex / dual instances for these layouts, in order of preference."""
    return _PLANAR_TILES if planar else _COMPLEX_PAIR_TILES


# One wave per SIMD: 256 x 256 x 64 on four waves with 128 x 128 wave tiles (a third fewer LDS reads per MFMA than
# 2 x 4 waves, and a K loop written out slot by slot: 105 against 116 us at 4096^3).  Compiled for plain products
# without hooks (whole tiles, or any extents with an FP32 C / D) and with hooks of D in closed form; the library runs
# the 2 x 4 arrangement of the same block shape, with the same bits, for any other launch of such a configuration.
_SOLO_TILE, _SOLO_WAVES = (256, 256, 64), (2, 2)
_SOLO_COMPLEX_TILE = (128, 128, 64)        # in complex elements


def _default_waves(operator, block_shape, checked=False, planar=False, gett=False, a_kmajor=False, b_kmajor=True, whole_tiles=False):
    key = (block_shape["M"], block_shape["N"], block_shape["K"])
    if gett and key == (64, 64, 32):
        return (1, 1)
    if operator.kind == Operator.MFMA and key == _SOLO_TILE and whole_tiles:
        return _SOLO_WAVES
    # ... and the tiles with a side of 192 (wave tiles of 128 x 96 / 96 x 128; 3072^3: 56 us against 62 on eight waves,
    # 'N','T' 57 against 65); the library runs the eight waves for what these instances do not cover (hooks, a bias,
    # tiles over the edges, a C / D that does not take 16-byte accesses)
    if operator.kind == Operator.MFMA and not gett and whole_tiles and any(key == t for t, _, _ in _MFMA_TILES_192):
        return _SOLO_WAVES
    # ... and the complex / dual product on interleaved matrices of an 'N','N' launch, whose real tile is that tile
    # (planar matrices: every transpose)
    if (operator.kind in (Operator.MFMA_COMPLEX, Operator.MFMA_DUAL) and key == _SOLO_COMPLEX_TILE and whole_tiles
            and (planar or (not a_kmajor and b_kmajor))):
        return _SOLO_WAVES
    if operator.kind in (Operator.FPU, Operator.FPU_TROPICAL):
        table = _FPU_TILES
    elif operator.kind == Operator.MFMA and checked and any(t == key for t, _ in _CHECKED_TILES):
        table = _CHECKED_TILES
    elif operator.kind in (Operator.MFMA_COMPLEX, Operator.MFMA_DUAL):
        table = _complex_tiles(operator, planar, a_kmajor, b_kmajor)
    else:
        table = _MFMA_TILES + [(t, w) for t, w, _ in _MFMA_TILES_192]
    for t, w in table:
        if t == key:
            return w
    return None


def require_tile_sized_global(layout) -> bool:
    """reference src/config.jl:175-178."""
    return layout.kind not in (Layout.ZERO, Layout.COL_MAJOR, Layout.ROW_MAJOR)


def get_config(*, gemm_shape, operator, global_a_layout, global_c_layout, **params) -> Config:
    """reference src/config.jl:180-316.  Same keywords; defaults for the parameters the caller
    leaves out are chosen for the MI355X.  All checks of the reference are run (by the library,
    through gk_validate) and raise ConfigError."""
    gemm_shape = NT(gemm_shape)
    global_b_layout = params.get("global_b_layout", global_a_layout)
    global_d_layout = params.get("global_d_layout", global_c_layout)

    def padded(l):
        return Layout.Padded[l, 16 // l.T.size] if l.kind not in (Layout.ZERO, Layout.DIAGONAL, Layout.GETT_KIND) else l

    shared_a_layout = params.get("shared_a_layout", padded(global_a_layout))
    shared_b_layout = params.get("shared_b_layout", padded(global_b_layout))
    shared_c_layout = params.get("shared_c_layout", global_c_layout)
    shared_d_layout = params.get("shared_d_layout", global_d_layout)

    tile_sized = any(require_tile_sized_global(l) for l in (global_a_layout, global_b_layout, global_c_layout, global_d_layout))
    block_shape = params.get("block_shape")
    if block_shape is None and operator.kind == Operator.MFMA and TUNED:
        # a measured winner for exactly this problem (gemmkernels.tuning), unless the caller chose otherwise
        key = (f"mfma/{global_a_layout.T.name}/{'N' if params.get('is_a_col_major', True) else 'T'}"
               f"{'N' if params.get('is_b_col_major', True) else 'T'}/{gemm_shape.M}x{gemm_shape.N}x{gemm_shape.K}")
        hit = TUNED.get(key)
        aligned = all(l.kind in (Layout.ALIGNED_COL_MAJOR, Layout.ALIGNED_ROW_MAJOR, Layout.ZERO)
                      for l in (global_a_layout, global_b_layout, global_c_layout, global_d_layout))
        if hit is not None and aligned:
            bm, bn, bk = hit["block"]
            wm, wn = hit["waves"]
            block_shape = NT(M=bm, N=bn, K=bk)
            params.setdefault("warps_per_block", wm * wn)
            params.setdefault("compute_warp", NT(M=bm // wm, N=bn // wn, K=16))
            params.setdefault("cta_swizzle", CTASwizzle.XCDAware[int(hit.get("panel", 4))])
    if block_shape is None and global_a_layout.kind == Layout.DIAGONAL and gemm_shape.M % 64 == 0 and gemm_shape.N % 64 == 0:
        # a diagonal A makes the product a streaming pass over B and D: many small workgroups keep more
        # memory requests in flight than a few large ones (measured against HBM with rotating buffers)
        block_shape = NT(M=64, N=64, K=32 if gemm_shape.K % 32 == 0 else gemm_shape.K)
        params.setdefault("warps_per_block", 4)
        params.setdefault("compute_warp", NT(M=32, N=32, K=16))
        # consecutive workgroups on consecutive pieces of memory: the XCD-aware walk (made for tiles that
        # share operands) costs a streaming kernel 8 % here
        params.setdefault("cta_swizzle", CTASwizzle.Identity)
    is_gett = any(l.kind == Layout.GETT_KIND for l in (global_a_layout, global_b_layout, global_c_layout, global_d_layout))
    planar = global_a_layout.kind in (Layout.SPLIT_COL_MAJOR, Layout.SPLIT_ROW_MAJOR)
    a_kmajor = global_a_layout.kind in (Layout.ROW_MAJOR, Layout.ALIGNED_ROW_MAJOR, Layout.INTERLEAVED_ROW_MAJOR, Layout.SPLIT_ROW_MAJOR)
    b_kmajor = global_b_layout.kind in (Layout.COL_MAJOR, Layout.ALIGNED_COL_MAJOR, Layout.INTERLEAVED_COL_MAJOR, Layout.SPLIT_COL_MAJOR)
    block_shape = (default_block_shape(operator, gemm_shape, tile_sized, is_gett, planar, a_kmajor=a_kmajor, b_kmajor=b_kmajor)
                   if block_shape is None else NT(block_shape))
    op_shape = Operator.shape(operator)

    checked = any(l.kind in (Layout.COL_MAJOR, Layout.ROW_MAJOR) for l in (global_a_layout, global_b_layout, global_c_layout, global_d_layout))
    whole_tiles = gemm_shape.M % block_shape.M == 0 and gemm_shape.N % block_shape.N == 0 and gemm_shape.K % block_shape.K == 0
    if operator.kind == Operator.MFMA and not is_gett:
        # (the plain product also where tiles stick out over the edges; the library runs the eight-wave arrangement
        # where C / D are not FP32)
        whole_tiles = whole_tiles or (gemm_shape.M >= 8 and gemm_shape.K >= 64)
    waves = _default_waves(operator, block_shape, checked, planar, is_gett, a_kmajor, b_kmajor, whole_tiles)
    if waves is not None:
        warps_default = waves[0] * waves[1]
        compute_warp_default = NT(M=block_shape.M // waves[0], N=block_shape.N // waves[1], K=op_shape.K)
    else:
        # reference src/config.jl:216-229: 8 warps as 4 x 2 unless the block is too small for that
        warps_default = 8
        compute_warp_default = NT(M=block_shape.M // 4, N=block_shape.N // 2, K=op_shape.K)
        if op_shape.M > 0 and op_shape.N > 0 and ((block_shape.M // op_shape.M) < 4 or (block_shape.N // op_shape.N) < 2):
            compute_warp_default = NT(M=max(op_shape.M, block_shape.M // 4), N=max(op_shape.N, block_shape.N // 2), K=op_shape.K)
            warps_default = min(block_shape.M // op_shape.M, 4) * min(block_shape.N // op_shape.N, 2)
    warps_per_block = params.get("warps_per_block", warps_default)
    compute_warp = NT(params.get("compute_warp", compute_warp_default))
    if "warps_per_block" in params and "compute_warp" not in params and waves is not None and warps_per_block != warps_default:
        # keep the reference's 4 x 2 style split for a caller-chosen wave count
        wm = 4 if warps_per_block % 4 == 0 and warps_per_block >= 8 else (2 if warps_per_block % 2 == 0 else 1)
        compute_warp = NT(M=block_shape.M // wm, N=block_shape.N // max(1, warps_per_block // wm), K=op_shape.K)

    is_a_col_major = params.get("is_a_col_major", True)
    is_b_col_major = params.get("is_b_col_major", True)
    is_cd_col_major = params.get("is_cd_col_major", True)

    # reference src/config.jl:240-260 with 64 lanes: 16 bytes per lane, as few lanes per row as possible
    lanes = WARP_SIZE * max(1, warps_per_block)
    n_a = max(1, min(16 // global_a_layout.T.size, (block_shape.M * block_shape.K) // lanes))
    n_b = max(1, min(16 // global_b_layout.T.size, (block_shape.K * block_shape.N) // lanes))
    n_c = max(1, min(16 // global_c_layout.T.size, (block_shape.M * block_shape.N) // lanes))
    mk, kn, mn = NT(M=block_shape.M, K=block_shape.K), NT(K=block_shape.K, N=block_shape.N), NT(M=block_shape.M, N=block_shape.N)
    mem_a_warp = NT(params.get("mem_a_warp", adjacent_elements(WARP_SIZE * n_a, mk, is_a_col_major)))
    mem_b_warp = NT(params.get("mem_b_warp", adjacent_elements(WARP_SIZE * n_b, kn, is_b_col_major)))
    mem_cd_warp = NT(params.get("mem_cd_warp", adjacent_elements(WARP_SIZE * n_c, mn, is_cd_col_major)))
    mem_a_thread = NT(params.get("mem_a_thread", adjacent_elements(n_a, mk, is_a_col_major)))
    mem_b_thread = NT(params.get("mem_b_thread", adjacent_elements(n_b, kn, is_b_col_major)))
    mem_cd_thread = NT(params.get("mem_cd_thread", adjacent_elements(n_c, mn, is_cd_col_major)))

    # src/config.jl:277-279 defaults to Identity; on the MI355X the XCD-aware walk is the default
    # (panels 4 tiles high; 8 once every CU has a tile: 4096^3 is 0.2 - 1.0 us faster with it in every transpose, 8192^3
    # 10 %; 16 from four thousand tiles on: 16384 x 16384 x 4096 1771 us against 1789 and 1871 us with 8 and 4)
    n_tiles = -(-gemm_shape.M // block_shape.M) * -(-gemm_shape.N // block_shape.N)
    cta_swizzle = params.get("cta_swizzle", CTASwizzle.XCDAware[16 if n_tiles >= 4096 else (8 if n_tiles >= NUM_CUS else 4)])

    conf = Config(gemm_shape, block_shape, warps_per_block, mem_a_warp, mem_a_thread, mem_b_warp, mem_b_thread,
                  mem_cd_warp, mem_cd_thread, compute_warp, op_shape,
                  global_a_layout, global_b_layout, global_c_layout, global_d_layout,
                  shared_a_layout, shared_b_layout, shared_c_layout, shared_d_layout,
                  operator, is_a_col_major, is_b_col_major, cta_swizzle)
    if not params.get("specialize", False):
        # ``specialize=True``: the block shape need not be in the library's table because the kernel
        # will be compiled at run time (gemmkernels.specialize); that compilation and every launch run
        # the same checks, minus the table lookup
        check_config(conf, params.get("kernel"))
    return conf


def check_config(conf: Config, kernel=None) -> None:
    """Every ConfigError of the reference (src/config.jl:203-275, src/matmul.jl:28-41), decided by
    the library on the host."""
    c = conf.to_c()
    code = 0 if kernel is None else kernel.code
    rc = _lib.lib().gk_validate(ctypes.byref(c), code)
    if rc != _lib.GK_OK:
        raise ConfigError(_lib.last_error(), rc)


def _load_tuning_table_from_environment() -> None:
    import json
    import os
    path = os.environ.get("GEMMKERNELS_TUNING_TABLE")
    if path and os.path.exists(path):
        with open(path) as f:
            TUNED.update(json.load(f))


_load_tuning_table_from_environment()
