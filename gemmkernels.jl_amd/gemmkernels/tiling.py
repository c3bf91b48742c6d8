"""Host-side Tiling API: named multi-dimensional tiles and their split across cooperating
entities (reference src/tiling.jl).  On the device the same index math is closed-form inside the
HIP kernels; this module keeps the reference's host-visible behaviour (and its known-answer
tests, reference test/tiling.jl:5-81).

Coordinates are 0-based ``dict``-like named tuples exactly as in the reference; ``linearise``
returns the reference's 1-based linear index.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Iterator, Mapping, Tuple


class NT(OrderedDict):
    """A tiny ordered named tuple: ``NT(M=1, N=2)``; fields by attribute, ordered, comparable."""

    def __getattr__(self, name):
        try:
            return self[name]
        except KeyError as e:
            raise AttributeError(name) from e

    def __eq__(self, other):
        if isinstance(other, Mapping):
            return list(self.items()) == list(other.items())
        return NotImplemented

    def __ne__(self, other):
        r = self.__eq__(other)
        return r if r is NotImplemented else not r

    __hash__ = None

    def names(self) -> Tuple[str, ...]:
        return tuple(self.keys())

    def __repr__(self):
        return "(" + ", ".join(f"{k} = {v}" for k, v in self.items()) + ")"


def _nt(names, values) -> NT:
    return NT(zip(names, values))


class Tile:
    """reference src/tiling.jl:34-37: ``size`` (static), ``base`` (run-time part of the index) and
    ``offset`` (compile-time part); ``index = base + offset``.  Projections are attributes named
    after the kept dimensions (``tile.MN``, ``tile.KMN`` ...), :88-113."""

    __slots__ = ("size", "base", "offset")

    def __init__(self, size=None, base=None, offset=None, **kw):
        if size is None:
            size = NT(kw)
        elif not isinstance(size, NT):
            size = NT(size)
        object.__setattr__(self, "size", size)
        object.__setattr__(self, "base", _nt(size.names(), [0] * len(size)) if base is None else NT(base))
        object.__setattr__(self, "offset", _nt(size.names(), [0] * len(size)) if offset is None else NT(offset))

    def __setattr__(self, *_):
        raise AttributeError("Tile is immutable")

    @property
    def index(self) -> NT:
        return _nt(self.size.names(), [self.base[k] + self.offset[k] for k in self.size])

    def __getattr__(self, name):
        # projection: every character names a dimension to keep, in that order
        size = object.__getattribute__(self, "size")
        if name and all(ch in size for ch in name):
            names = tuple(name)
            return Tile(_nt(names, [size[k] for k in names]),
                        _nt(names, [self.base[k] for k in names]),
                        _nt(names, [self.offset[k] for k in names]))
        raise AttributeError(name)

    def __eq__(self, other):
        return (isinstance(other, Tile) and self.size == other.size and self.base == other.base
                and self.offset == other.offset)

    __hash__ = None

    def __repr__(self):
        return f"base:   {self.base}\noffset: {self.offset}\nsize:   {self.size}"


def transpose(tile: Tile) -> Tile:
    """reference src/tiling.jl:107-110: reverse the order of the dimensions."""
    names = tuple(reversed(tile.size.names()))
    return Tile(_nt(names, [tile.size[k] for k in names]), _nt(names, [tile.base[k] for k in names]),
                _nt(names, [tile.offset[k] for k in names]))


def linearise(coord: Mapping, dims: Mapping) -> int:
    """reference src/tiling.jl:131-134: 1-based column-major linear index of a 0-based coordinate."""
    idx, stride = 0, 1
    for c, d in zip(coord.values(), dims.values()):
        idx += c * stride
        stride *= d
    return idx + 1


def _as_offset(tile: Tile, offset) -> NT:
    if isinstance(offset, Mapping):
        if tuple(offset.keys()) != tile.size.names():
            raise ValueError("offset names must match the tile's")
        return NT(offset)
    return _nt(tile.size.names(), offset)


def translate_base(tile: Tile, offset) -> Tile:
    """reference src/tiling.jl:166-171."""
    off = _as_offset(tile, offset)
    return Tile(tile.size, _nt(tile.size.names(), [tile.base[k] + off[k] for k in tile.size]), tile.offset)


def translate_offset(tile: Tile, offset) -> Tile:
    """reference src/tiling.jl:173-178."""
    off = _as_offset(tile, offset)
    return Tile(tile.size, tile.base, _nt(tile.size.names(), [tile.offset[k] + off[k] for k in tile.size]))


def _subtile_index(linear: int, num_tiles) -> Tuple[int, ...]:
    """0-based column-major multi-index of the 1-based ``linear`` among ``num_tiles``."""
    lin = linear - 1
    out = []
    for n in num_tiles:
        out.append(lin % n)
        lin //= n
    return tuple(out)


def parallelise(tile: Tile, tiling_size: Tile, idx: int, count: int, col_major: bool = True) -> Iterator[Tile]:
    """reference src/tiling.jl:224-236 + iterator :263-286: entity ``idx`` (1-based) of ``count``
    visits sub-tiles idx, idx+count, ...; its own number goes to ``base``, the iteration to
    ``offset``; row-major variants walk the transposed tile."""
    t = tile if col_major else transpose(tile)
    ts = tiling_size if col_major else transpose(tiling_size)
    names = t.size.names()
    num_tiles = [t.size[k] // ts.size[k] for k in names]
    total = 1
    for n in num_tiles:
        total *= n
    if count > total and idx > total:
        return
    state = 1
    while state <= total:
        bi = _subtile_index(idx, num_tiles)
        oi = _subtile_index(state, num_tiles)
        base = _nt(names, [t.base[k] + bi[i] * ts.size[k] for i, k in enumerate(names)])
        offset = _nt(names, [t.offset[k] + oi[i] * ts.size[k] for i, k in enumerate(names)])
        sub = Tile(_nt(names, [ts.size[k] for k in names]), base, offset)
        yield sub if col_major else transpose(sub)
        state += count


def subdivide(tile: Tile, tiling_size: Tile, idx: int, count: int) -> Tile:
    """reference src/tiling.jl:255-261: the single sub-tile of entity ``idx``."""
    for t in parallelise(tile, tiling_size, idx, count):
        return t
    raise IndexError("subdivide: more entities than sub-tiles")
