"""The tuning table (counterpart of the reference's tuning/ directory): get_config takes a measured
winner for exactly the problem at hand when the caller leaves the block shape open."""
import json

import pytest

import gemmkernels as gk
from gemmkernels import configs, tuning, Kernel, NT
from gemmkernels import config as cfg


def test_table_round_trip_and_lookup(tmp_path):
    key = tuning.table_key(1024, 512, 256, False, True)
    assert key == "mfma/Float16/NT/1024x512x256"
    table = {key: {"block": [128, 128, 32], "waves": [2, 2], "panel": 2}}
    path = tmp_path / "table.json"
    tuning.save(str(path), table)
    assert json.loads(path.read_text()) == table
    before = configs.mfma_config(1024, 512, 256, False, True)
    try:
        tuning.load(str(path))
        conf = configs.mfma_config(1024, 512, 256, False, True)
        assert conf.block_shape == NT(M=128, N=128, K=32) and conf.warps_per_block == 4
        assert conf.cta_swizzle.param == 2
        assert "128x128x32_w2x2" in gk.kernel_name(conf, Kernel.matmul_pipelined)
        # an explicit block shape wins over the table; other problems are untouched
        assert configs.mfma_config(1024, 512, 256, False, True, block_shape=(64, 64, 64)).block_shape == NT(M=64, N=64, K=64)
        assert configs.mfma_config(1024, 512, 512, False, True).block_shape == configs.mfma_config(1024, 512, 512, False, True).block_shape
    finally:
        cfg.TUNED.clear()
    assert configs.mfma_config(1024, 512, 256, False, True).block_shape == before.block_shape


def test_every_candidate_of_the_tuner_is_a_compiled_instance():
    for block, waves in tuning.MFMA_CANDIDATES:
        # a tile with a side of 192 exists where the operand on that side is contiguous along k: 'T','N' has both
        ta = 192 in block[:2]
        conf = tuning.mfma_config(2 * block[0], 2 * block[1], 4 * block[2], ta, False, block, waves, 4)
        assert f"{block[0]}x{block[1]}x{block[2]}_w{waves[0]}x{waves[1]}" in gk.kernel_name(conf, Kernel.matmul_pipelined)
    # ... and nowhere else: the tuner skips it there
    with pytest.raises(gk.ConfigError):
        tuning.mfma_config(384, 512, 256, False, True, (192, 256, 64), (2, 4), 4)      # 'N','T' has 256 x 192 instead


@pytest.mark.gpu
def test_tune_a_small_problem(gpu):
    results = tuning.tune_mfma(512, 512, 256, candidates=[((128, 128, 64), (2, 2)), ((64, 64, 64), (2, 2)), ((256, 256, 64), (2, 4))],
                               panels=(1, 4), launches=5, warmup=2)
    assert len(results) == 6 and results == sorted(results, key=lambda r: r["us"])
    assert all(r["us"] > 0 for r in results)
