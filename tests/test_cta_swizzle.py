"""CTA swizzles on the host: the library evaluates the very function the kernels inline.
Known answers: the example tables in the comments of reference src/cta-swizzle.jl."""
import json
import os

import pytest

from gemmkernels import CTASwizzle, NT

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "cta_swizzle_tables.json")))
BLOCK = NT(M=128, N=128)
SHAPE = NT(M=1024, N=1024)


@pytest.mark.parametrize("swz,key", [(CTASwizzle.HorizontallyTiled[4], "HorizontallyTiled4"),
                                     (CTASwizzle.VerticallyTiled[4], "VerticallyTiled4"),
                                     (CTASwizzle.LebesgueCurve, "LebesgueCurve")])
def test_reference_tables(swz, key):
    assert CTASwizzle.visualise_cta_swizzle(swz, BLOCK, SHAPE) == GOLDEN[key]


def test_number_of_blocks():
    # reference src/cta-swizzle.jl:28-31, 69-72, 104-107, 149-151
    assert CTASwizzle.number_of_blocks(CTASwizzle.Identity, BLOCK, SHAPE) == (8, 8)
    assert CTASwizzle.number_of_blocks(CTASwizzle.HorizontallyTiled[4], BLOCK, SHAPE) == (32, 2)
    assert CTASwizzle.number_of_blocks(CTASwizzle.VerticallyTiled[4], BLOCK, SHAPE) == (2, 32)
    assert CTASwizzle.number_of_blocks(CTASwizzle.LebesgueCurve, BLOCK, SHAPE) == (64, 1)
    assert CTASwizzle.number_of_blocks(CTASwizzle.XCDAware[4], BLOCK, SHAPE) == (64, 1)
    assert CTASwizzle.number_of_blocks(CTASwizzle.Identity, BLOCK, NT(M=1000, N=10)) == (8, 1)   # cld


def test_identity_origin():
    assert CTASwizzle.cta_swizzle(CTASwizzle.Identity, NT(x=3, y=5), BLOCK) == (256, 512)


def _tiles(swz, block, shape):
    gx, gy = CTASwizzle.number_of_blocks(swz, block, shape)
    out = []
    for by in range(1, gy + 1):
        for bx in range(1, gx + 1):
            bi, bj = CTASwizzle.cta_swizzle(swz, NT(x=bx, y=by), block, shape)
            out.append((bi // block.M, bj // block.N))
    return out


@pytest.mark.parametrize("swz", [CTASwizzle.Identity, CTASwizzle.HorizontallyTiled[2], CTASwizzle.HorizontallyTiled[8],
                                 CTASwizzle.VerticallyTiled[4], CTASwizzle.LebesgueCurve, CTASwizzle.XCDAware[4],
                                 CTASwizzle.XCDAware[3], CTASwizzle.XCDAware[1]])
@pytest.mark.parametrize("shape", [NT(M=1024, N=1024), NT(M=4096, N=4096), NT(M=2048, N=512)])
def test_bijection_onto_the_tile_grid(swz, shape):
    block = NT(M=128, N=128) if shape.M < 4096 else NT(M=256, N=256)
    nbm, nbn = shape.M // block.M, shape.N // block.N
    if swz == CTASwizzle.LebesgueCurve and nbm != nbn:
        pytest.skip("the Lebesgue curve covers square power-of-two grids only (reference quirk)")
    tiles = [t for t in _tiles(swz, block, shape) if t[0] < nbm and t[1] < nbn]
    assert sorted(tiles) == [(i, j) for i in range(nbm) for j in range(nbn)]


def test_xcd_walk_odd_grid_is_a_bijection():
    block, shape = NT(M=128, N=128), NT(M=128 * 7, N=128 * 5)     # 35 tiles: not a multiple of 8
    assert sorted(_tiles(CTASwizzle.XCDAware[4], block, shape)) == [(i, j) for i in range(7) for j in range(5)]


def test_xcd_walk_locality():
    """With 256 tiles of a 16 x 16 grid, the 32 workgroups that share an XCD (ids congruent mod 8)
    cover a 4 x 8 patch of tiles: 4 row panels of A and 8 column panels of B per L2."""
    block, shape = NT(M=256, N=256), NT(M=4096, N=4096)
    tiles = _tiles(CTASwizzle.XCDAware[4], block, shape)
    for xcd in range(8):
        mine = [tiles[i] for i in range(xcd, 256, 8)]
        rows, cols = {t[0] for t in mine}, {t[1] for t in mine}
        assert len(rows) == 4 and len(cols) == 8


def test_xcd_walk_locality_when_the_tile_count_is_not_a_multiple_of_8():
    """225 tiles (15 x 15, e.g. 3840^2 on 256 x 256 tiles): the ids of one XCD (congruent mod 8) still
    cover consecutive positions of the panel walk, so they share rows of A and columns of B."""
    block, shape = NT(M=256, N=256), NT(M=3840, N=3840)
    tiles = _tiles(CTASwizzle.XCDAware[4], block, shape)
    assert sorted(tiles) == [(i, j) for i in range(15) for j in range(15)]
    # position of a tile in the panel walk (panels 4 tiles high, the last one 3 high)
    def walk_pos(t):
        i, j = t
        first = (i // 4) * 4
        gsz = min(4, 15 - first)
        return first * 15 + j * gsz + (i - first)
    for xcd in range(8):
        pos = sorted(walk_pos(tiles[n]) for n in range(xcd, 225, 8))
        assert pos == list(range(pos[0], pos[0] + len(pos))), xcd
        rows = {tiles[n][0] for n in range(xcd, 225, 8)}
        assert len(rows) <= 8
