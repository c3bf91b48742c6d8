"""Planner for tensor contractions written the TCCG way, e.g. ``"abc-bda-dc"`` for
``D[a,b,c] = sum_d A[b,d,a] * B[d,c]`` (the contraction of the reference's benchmark script,
benchmarks/tensor-contractions/run.jl:10-21, where the index arithmetic is hand-written into four
Layout types, :22-85).  Here the arithmetic is derived from the mode strings:

1. modes are classified (M: in A and D, N: in B and D, K: in A and B);
2. neighbouring modes that are neighbours, in the same order, in both tensors that hold them are
   fused into one longer mode (longer first modes are what the kernel's 16-byte vectors and 32-wide
   accumulator blocks need);
3. both assignments of the two inputs to the kernel's A and B operands are tried (swapping them
   swaps the roles of M and N; the sum is the same);
4. a tile with tensor-contraction addressing is chosen whose BLOCK_K divides the first K mode;
5. the library validates the result; if no candidate passes, the reasons are reported.

Tensors are dense and column-major (first index fastest), as Julia arrays are.  Nothing is copied
or permuted: a contraction either maps onto one launch of the GEMM kernel or is refused.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

from . import kernel as Kernel
from . import layout as Layout
from . import operator as Operator
from .config import _GETT_TILES, NUM_CUS, get_config
from .dtypes import BFloat16, DType, Float16, Float32
from .errors import ConfigError
from .tiling import NT


def parse(spec: str) -> Tuple[str, str, str]:
    """``"D-A-B"`` -> (d_modes, a_modes, b_modes); one letter per mode."""
    parts = spec.replace(" ", "").split("-")
    if len(parts) != 3 or not all(parts):
        raise ValueError(f"a contraction is written 'D-A-B' with one letter per mode, got {spec!r}")
    d, a, b = parts
    for name, modes in (("D", d), ("A", a), ("B", b)):
        if len(set(modes)) != len(modes):
            raise ValueError(f"mode repeated in {name}: {modes!r}")
    return d, a, b


def classify(d: str, a: str, b: str) -> Tuple[List[str], List[str], List[str]]:
    """M, N and K modes; batch modes (in all three tensors) and modes summed over a single tensor are
    not GEMM-shaped and are refused."""
    m = [ch for ch in a if ch in d and ch not in b]
    n = [ch for ch in b if ch in d and ch not in a]
    k = [ch for ch in a if ch in b and ch not in d]
    odd = [ch for ch in set(a + b + d) if ch not in m + n + k]
    if odd:
        raise ValueError("modes " + ", ".join(sorted(odd)) + " appear in all three tensors or in only one: not a GEMM-shaped contraction")
    if not m or not n or not k:
        raise ValueError("a contraction needs at least one M mode (A and D), one N mode (B and D) and one K mode (A and B)")
    return m, n, k


def fuse(d: str, a: str, b: str, extents: Dict[str, int]) -> Tuple[str, str, str, Dict[str, int], Dict[str, str]]:
    """Fuses modes x, y that directly follow each other (x before y) in every tensor that holds them.
    Returns the new mode strings and extents, and for every surviving letter the letters it stands for."""
    groups = {ch: ch for ch in set(d + a + b)}
    ext = dict(extents)
    tensors = [d, a, b]
    changed = True
    while changed:
        changed = False
        for t in tensors:
            for i in range(len(t) - 1):
                x, y = t[i], t[i + 1]
                holders = [u for u in tensors if x in u or y in u]
                if all((x in u) and (y in u) and u.index(y) == u.index(x) + 1 for u in holders):
                    ext[x] = ext[x] * ext[y]
                    groups[x] = groups[x] + groups[y]
                    del ext[y], groups[y]
                    tensors = [u.replace(y, "") for u in tensors]
                    changed = True
                    break
            if changed:
                break
    d2, a2, b2 = tensors
    return d2, a2, b2, ext, groups


@dataclass
class ContractionPlan:
    """What the planner decided, and the launch (``plan(...)`` returns it ready to call)."""
    spec: str
    swapped: bool                 # the second input runs as the kernel's A operand
    fused: Dict[str, str]         # surviving mode -> original modes it stands for
    conf: object
    gemm_shape: Tuple[int, int, int]
    kernel_name: str
    _launch: object = None

    def __call__(self, stream=None):
        return self._launch(stream)


def _shape_extents(modes: str, x, extents: Dict[str, int], name: str) -> None:
    shape = tuple(int(s) for s in x.shape)
    if len(shape) != len(modes):
        raise ConfigError(f"{name} has {len(shape)} dimensions, its mode string {modes!r} has {len(modes)}")
    stride = 1
    for ch, e, s in zip(modes, shape, x.stride()):
        if extents.setdefault(ch, e) != e:
            raise ConfigError(f"mode {ch!r} has extent {extents[ch]} in one tensor and {e} in {name}")
        if e > 1 and int(s) != stride:
            raise ConfigError(f"{name} must be dense and column-major (first index fastest); see gemmkernels.colmajor")
        stride *= e


def candidates(spec: str, extents: Dict[str, int], ab_type: DType = Float16, cd_type: DType = Float32, zero_c: bool = True):
    """Yields (swapped, fused groups, configuration or None, reason) for both operand assignments and
    every tile with contraction addressing, best first.  Needs no GPU."""
    from .matmul import kernel_name
    d, a, b = parse(spec)
    classify(d, a, b)
    d2, a2, b2, ext, groups = fuse(d, a, b, extents)
    for swapped in (False, True):
        am, bm = (b2, a2) if swapped else (a2, b2)
        gmap = Layout.gett_map(am, bm, d2, ext)
        M, N, K = gmap.extent("m"), gmap.extent("n"), gmap.extent("k")
        tiles = [t for t in _GETT_TILES if M % t[0] == 0 and N % t[1] == 0 and gmap.k[0][0] % t[2] == 0]
        if not tiles:
            yield swapped, groups, None, (f"no tile divides M = {M}, N = {N} and the first K mode of {gmap.k[0][0]} "
                                          f"(tiles {_GETT_TILES})")
            continue
        filling = [t for t in tiles if (M // t[0]) * (N // t[1]) >= NUM_CUS]
        for t in (filling[:1] or tiles[-1:]) + [u for u in tiles if u not in (filling[:1] or tiles[-1:])]:
            try:
                conf = get_config(gemm_shape=NT(M=M, N=N, K=K), operator=Operator.MFMAOp[32, 32, 16, ab_type, Float32],
                                  global_a_layout=Layout.GETT[ab_type, gmap], global_b_layout=Layout.GETT[ab_type, gmap],
                                  global_c_layout=Layout.Zero[cd_type] if zero_c else Layout.GETT[cd_type, gmap],
                                  global_d_layout=Layout.GETT[cd_type, gmap],
                                  shared_a_layout=Layout.UnsafeAlignedColMajor[ab_type], shared_b_layout=Layout.UnsafeAlignedColMajor[ab_type],
                                  shared_c_layout=Layout.Zero[cd_type] if zero_c else Layout.UnsafeAlignedColMajor[cd_type],
                                  shared_d_layout=Layout.UnsafeAlignedColMajor[cd_type],
                                  block_shape=NT(M=t[0], N=t[1], K=t[2]), kernel=Kernel.matmul_pipelined)
                yield swapped, groups, conf, kernel_name(conf, Kernel.matmul_pipelined)
            except ConfigError as e:
                yield swapped, groups, None, f"tile {t}: {e.message}"


def plan(spec: str, a, b, d, c=None, ab_type: Optional[DType] = None, cd_type: Optional[DType] = None) -> ContractionPlan:
    """Plans ``D = sum A * B (+ C)`` for device tensors (dense, column-major) and returns the launch.
    ``c`` has the modes and the element type of ``d``; ``d`` may be ``c``."""
    from .dtypes import from_torch
    from .matmul import Plan, _DEFAULT_EPILOGUE, _IDENTITY, _HOOKS
    dm, am, bm = parse(spec)
    extents: Dict[str, int] = {}
    _shape_extents(am, a, extents, "A")
    _shape_extents(bm, b, extents, "B")
    _shape_extents(dm, d, extents, "D")
    if c is not None:
        _shape_extents(dm, c, extents, "C")
    ab_type = ab_type or from_torch(a.dtype)
    cd_type = cd_type or from_torch(d.dtype)
    if ab_type not in (Float16, BFloat16) or from_torch(b.dtype) != ab_type:
        raise ConfigError("contractions run on the matrix cores: A and B must both be Float16 or both BFloat16")
    reasons = []
    for swapped, groups, conf, info in candidates(spec, extents, ab_type, cd_type, zero_c=c is None):
        if conf is None:
            reasons.append(("B as the A operand: " if swapped else "") + info)
            continue
        x, y = (b, a) if swapped else (a, b)
        launch = Plan(conf, x, y, c, d, {k: _IDENTITY for k in _HOOKS}, _DEFAULT_EPILOGUE, Kernel.matmul_pipelined)
        ms = conf.matmul_shape
        return ContractionPlan(spec, swapped, groups, conf, (ms.M, ms.N, ms.K), info, launch)
    raise ConfigError("contraction " + spec + " does not map onto the GEMM kernel: " + "; ".join(reasons))


def contract(spec: str, a, b, d, c=None, stream=None):
    """``D[...] = sum A[...] * B[...] (+ C[...])`` in one launch on the current stream; returns ``d``."""
    plan(spec, a, b, d, c)(stream)
    return d
