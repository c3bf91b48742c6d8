"""Layouts: how a logical tile maps to memory (reference src/layout.jl).

A layout is written ``Layout.UnsafeAlignedColMajor[Float16]`` where the reference writes
``Layout.UnsafeAlignedColMajor{Float16}``; ``Layout.Padded[L, P]`` mirrors ``Padded{L, P}``.
The objects only describe; the loads and stores they stand for are in the HIP kernels.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Sequence, Tuple

from .dtypes import DType

# gk_layout_kind
ZERO, COL_MAJOR, ROW_MAJOR, ALIGNED_COL_MAJOR, ALIGNED_ROW_MAJOR, DIAGONAL, INTERLEAVED_COL_MAJOR, \
    INTERLEAVED_ROW_MAJOR, SPLIT_COL_MAJOR, SPLIT_ROW_MAJOR, GETT_KIND = range(11)

_NAMES = {ZERO: "Zero", COL_MAJOR: "ColMajor", ROW_MAJOR: "RowMajor", ALIGNED_COL_MAJOR: "UnsafeAlignedColMajor",
          ALIGNED_ROW_MAJOR: "UnsafeAlignedRowMajor", DIAGONAL: "Diagonal", INTERLEAVED_COL_MAJOR: "InterleavedColMajor",
          INTERLEAVED_ROW_MAJOR: "InterleavedRowMajor", SPLIT_COL_MAJOR: "SplitColMajor", SPLIT_ROW_MAJOR: "SplitRowMajor",
          GETT_KIND: "GETT"}


@dataclass(frozen=True)
class LayoutType:
    kind: int
    T: DType
    pad: int = 0                       # Padded{L, P}
    gett: Optional["GETTMap"] = None   # tensor-contraction index map (GETT_KIND only)

    def __repr__(self):
        base = f"Layout.{_NAMES[self.kind]}{{{self.T}}}"
        return f"Layout.Padded{{{base}, {self.pad}}}" if self.pad else base

    # reference src/layout.jl:75-76
    @property
    def eltype(self) -> DType:
        return self.T

    @property
    def is_row_major(self) -> bool:
        return self.kind in (ROW_MAJOR, ALIGNED_ROW_MAJOR, INTERLEAVED_ROW_MAJOR, SPLIT_ROW_MAJOR)

    @property
    def is_aligned(self) -> bool:
        return self.kind in (ALIGNED_COL_MAJOR, ALIGNED_ROW_MAJOR)

    @property
    def base(self) -> "LayoutType":
        return LayoutType(self.kind, self.T, 0, self.gett)


class _Family:
    def __init__(self, kind: int):
        self.kind = kind

    def __getitem__(self, T: DType) -> LayoutType:
        return LayoutType(self.kind, T)

    def __repr__(self):
        return f"Layout.{_NAMES[self.kind]}"


Zero = _Family(ZERO)                                    # src/layout.jl:82-89
ColMajor = _Family(COL_MAJOR)                           # :111-148
RowMajor = _Family(ROW_MAJOR)                           # :156-184
UnsafeAlignedColMajor = _Family(ALIGNED_COL_MAJOR)      # :192-219
UnsafeAlignedRowMajor = _Family(ALIGNED_ROW_MAJOR)      # :244-270
Diagonal = _Family(DIAGONAL)                            # :225-236
InterleavedColMajor = _Family(INTERLEAVED_COL_MAJOR)    # :276-302
InterleavedRowMajor = _Family(INTERLEAVED_ROW_MAJOR)    # :310-334
SplitColMajor = _Family(SPLIT_COL_MAJOR)                # :340-372
SplitRowMajor = _Family(SPLIT_ROW_MAJOR)                # :380-411


class _Padded:
    """``Layout.Padded[L, P]``: P elements of padding on the leading physical dimension (:95-105)."""

    def __getitem__(self, args) -> LayoutType:
        layout, pad = args
        return LayoutType(layout.kind, layout.T, int(pad), layout.gett)


Padded = _Padded()


@dataclass(frozen=True)
class GETTMap:
    """Index map of a tensor contraction.  Each GEMM dimension is a mixed-radix number over tensor
    modes, fastest digit first: ``m``, ``n``, ``k`` are sequences of (extent, stride0, stride1) with
    the strides of the mode in (A, D) for m, (B, D) for n and (A, B) for k.  The pattern follows the
    custom Layout subtypes of reference benchmarks/tensor-contractions/run.jl:22-85, where the
    contraction's index arithmetic lives in Layout.load / Layout.store!."""
    m: Tuple[Tuple[int, int, int], ...]
    n: Tuple[Tuple[int, int, int], ...]
    k: Tuple[Tuple[int, int, int], ...]

    def extent(self, which: str) -> int:
        out = 1
        for e, _, _ in getattr(self, which):
            out *= e
        return out


class _GETT:
    def __getitem__(self, args) -> LayoutType:
        T, gmap = args
        return LayoutType(GETT_KIND, T, 0, gmap)


GETT = _GETT()


def eltype(layout: LayoutType) -> DType:
    return layout.T


def physical_size(layout: LayoutType, logical_size) -> tuple:
    """reference src/layout.jl:76, :113, :152, :194, :246, :342-345, :381-383."""
    t = tuple(logical_size.values()) if hasattr(logical_size, "values") else tuple(logical_size)
    if layout.kind in (ROW_MAJOR, ALIGNED_ROW_MAJOR):
        return (t[1] + layout.pad, t[0]) if layout.pad else t
    if layout.kind == SPLIT_ROW_MAJOR:
        return (t[1] + layout.pad, t[0], 2) if layout.pad else (*t, 2)
    if layout.kind == SPLIT_COL_MAJOR:
        return (t[0] + layout.pad, *t[1:], 2)
    return (t[0] + layout.pad, *t[1:])


def gett_map(a_modes: str, b_modes: str, d_modes: str, extents: dict) -> GETTMap:
    """Index map of the contraction ``D[d_modes] = sum A[a_modes] * B[b_modes]`` over dense
    column-major tensors (first index fastest), einsum-style mode letters.

    M modes are those shared by A and D, N modes by B and D, K modes by A and B.  Within each GEMM
    dimension the mode that is contiguous in A (for M, K) or B (for N, K) goes first, so that the
    loader can move 16-byte vectors; the others follow by increasing stride."""
    def strides(modes):
        out, s = {}, 1
        for ch in modes:
            out[ch] = s
            s *= extents[ch]
        return out

    sa, sb, sd = strides(a_modes), strides(b_modes), strides(d_modes)
    m_modes = [ch for ch in a_modes if ch in d_modes]
    n_modes = [ch for ch in b_modes if ch in d_modes]
    k_modes = [ch for ch in a_modes if ch in b_modes]
    if set(m_modes) | set(n_modes) != set(d_modes) or set(m_modes) & set(n_modes):
        raise ValueError("every mode of D must come from exactly one of A and B")
    m_modes.sort(key=lambda ch: sa[ch])
    n_modes.sort(key=lambda ch: sb[ch])
    # K: a mode that is contiguous in A or in B must lead
    k_modes.sort(key=lambda ch: min(sa[ch], sb[ch]))
    return GETTMap(m=tuple((extents[ch], sa[ch], sd[ch]) for ch in m_modes),
                   n=tuple((extents[ch], sb[ch], sd[ch]) for ch in n_modes),
                   k=tuple((extents[ch], sa[ch], sb[ch]) for ch in k_modes))
