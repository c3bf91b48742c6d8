"""Known-answer tests of the Tiling API, the reference's own (reference test/tiling.jl:5-81)."""
from gemmkernels.tiling import NT, Tile, linearise, parallelise, subdivide, translate_base, translate_offset, transpose


def test_index():
    assert Tile(M=4, N=4, K=4).index == NT(M=0, N=0, K=0)


def test_projection():
    assert Tile(M=1, N=2, K=3).MN == Tile(M=1, N=2)
    assert Tile(M=1, N=2, K=3).NM == Tile(N=2, M=1)
    assert Tile(M=1, N=2, K=3).M == Tile(M=1)
    assert Tile(M=1, N=2, K=3).KMN == Tile(K=3, M=1, N=2)


def test_transposition():
    assert transpose(Tile(M=1, N=2)) == Tile(N=2, M=1)
    assert transpose(Tile(M=1, N=2, K=3)) == Tile(K=3, N=2, M=1)


def test_translate_base():
    tile = translate_base(Tile(M=10, N=20), NT(M=1, N=2))
    assert tile.size == NT(M=10, N=20)
    assert tile.base == NT(M=1, N=2)
    assert tile.offset == NT(M=0, N=0)


def test_translate_offset():
    tile = translate_offset(Tile(M=10, N=20), NT(M=1, N=2))
    assert tile.size == NT(M=10, N=20)
    assert tile.base == NT(M=0, N=0)
    assert tile.offset == NT(M=1, N=2)


def test_linearise():
    tile = Tile(M=3, N=5)
    for i in range(3):
        for j in range(5):
            t = translate_offset(tile, NT(M=i, N=j))
            assert linearise(t.index, NT(M=100, N=200)) == j * 100 + i + 1
            assert linearise(t.NM.index, NT(N=200, M=100)) == i * 200 + j + 1


def test_subdivide():
    tile_size = NT(M=8, N=4)
    num_tiles = NT(M=2, N=4)
    tile = Tile(M=num_tiles.M * tile_size.M, N=num_tiles.N * tile_size.N)
    for i in range(1, num_tiles.M * num_tiles.N + 1):
        t = subdivide(tile, Tile(tile_size), i, num_tiles.M * num_tiles.N)
        assert t.offset == NT(M=0, N=0)
        assert t.base == NT(M=tile_size.M * ((i - 1) % num_tiles.M), N=tile_size.N * ((i - 1) // num_tiles.M))
        assert t.size == tile_size


def test_parallelise():
    tile_size = NT(M=8, N=4)
    num_tiles = NT(M=2, N=8)
    tile = Tile(M=num_tiles.M * tile_size.M, N=num_tiles.N * tile_size.N)
    count = (num_tiles.M * num_tiles.N) // 2
    for i in range(1, count + 1):
        t1, t2 = list(parallelise(tile, Tile(tile_size), i, count))
        assert t1.offset == NT(M=0, N=0)
        assert t2.offset == NT(M=0, N=4 * tile_size.N)
        base = NT(M=tile_size.M * ((i - 1) % num_tiles.M), N=tile_size.N * ((i - 1) // num_tiles.M))
        assert t1.base == base and t2.base == base
        assert t1.size == tile_size and t2.size == tile_size


def test_parallelise_row_major_walks_the_transposed_tile():
    # reference src/tiling.jl:226-227, 283: row-major iteration transposes, splits, transposes back
    tile = Tile(M=4, K=16)
    subs = list(parallelise(tile, Tile(M=1, K=8), 1, 2, False))
    assert [s.index for s in subs] == [NT(M=0, K=0), NT(M=1, K=0), NT(M=2, K=0), NT(M=3, K=0)]
    subs = list(parallelise(tile, Tile(M=1, K=8), 2, 2, False))
    assert [s.index for s in subs] == [NT(M=0, K=8), NT(M=1, K=8), NT(M=2, K=8), NT(M=3, K=8)]
    assert all(s.size == NT(M=1, K=8) for s in subs)


def test_more_entities_than_subtiles_yields_nothing():
    # reference src/tiling.jl:264-269
    assert list(parallelise(Tile(M=8, N=8), Tile(M=8, N=8), 2, 4)) == []
    assert len(list(parallelise(Tile(M=8, N=8), Tile(M=8, N=8), 1, 4))) == 1
