"""Config, get_config and every launch-time error, decided on the host (no GPU).
Known answers are hand-evaluated from the reference source lines cited at each test."""
import ctypes

import pytest

import gemmkernels as gk
from gemmkernels import CTASwizzle, Kernel, Layout, Operator, NT, Float16, Float32, ConfigError, DimensionMismatch, _lib
from gemmkernels import config as cfgmod
from gemmkernels.matmul import create_config

F16, F32 = Float16, Float32
ACM, ARM = Layout.UnsafeAlignedColMajor, Layout.UnsafeAlignedRowMajor


def test_heuristic_block_shape_reference_answers():
    # reference src/config.jl:84-120 with Padded{.,8} FP16 A/B: C/D FP32 128x128x4 = 64 KiB, then
    # K = 64: 136*64*2 + 72*128*2 = 35840 B fits, K = 128: 69632 B does not
    pa, pb = Layout.Padded[ACM[F16], 8], Layout.Padded[ACM[F16], 8]
    assert gk.heuristic_block_shape(pa, pb, ACM[F32], ACM[F32]) == NT(M=128, N=128, K=64)
    # FP16 C/D: 256 x 128 x 2 = 64 KiB
    assert gk.heuristic_block_shape(pa, pb, ACM[F16], ACM[F16]) == NT(M=256, N=128, K=64)
    # row-major A pads the K extent instead (src/layout.jl:246)
    assert gk.heuristic_block_shape(Layout.Padded[ARM[F16], 8], pb, ACM[F32], ACM[F32]) == NT(M=128, N=128, K=64)


def test_heuristic_block_shape_of_the_library_matches_the_python_mirror():
    """gk_heuristic_block_shape (what a Julia binding would call) against gk.heuristic_block_shape."""
    import ctypes
    from gemmkernels import ComplexF16, ComplexF32

    def c_layout(l):
        out = _lib.gk_layout()
        out.kind, out.eltype, out.pad, out.ld = l.kind, l.T.code, l.pad, 0
        return out

    SCM, SRM = Layout.SplitColMajor, Layout.SplitRowMajor
    cases = [
        (Layout.Padded[ACM[F16], 8], Layout.Padded[ACM[F16], 8], ACM[F32], ACM[F32]),
        (Layout.Padded[ACM[F16], 8], Layout.Padded[ACM[F16], 8], ACM[F16], ACM[F16]),
        (Layout.Padded[ARM[F16], 8], Layout.Padded[ARM[F16], 8], ACM[F32], ACM[F32]),
        (ACM[F32], ACM[F32], ACM[F32], ACM[F32]),
        (ACM[gk.Float64], ARM[gk.Float64], ACM[gk.Float64], ACM[gk.Float64]),
        (Layout.Padded[SCM[F16], 8], Layout.Padded[SCM[F16], 8], SCM[F32], SCM[F32]),     # configs/configs.jl:397-401
        (Layout.Padded[SRM[F16], 8], Layout.Padded[SCM[F16], 8], SCM[F32], SCM[F32]),
    ]
    for layouts in cases:
        want = gk.heuristic_block_shape(*layouts)
        cl = [c_layout(l) for l in layouts]
        got = _lib.gk_shape()
        rc = _lib.lib().gk_heuristic_block_shape(*(ctypes.byref(x) for x in cl), ctypes.byref(got))
        assert rc == _lib.GK_OK
        assert (got.M, got.N, got.K) == (want.M, want.N, want.K), layouts


def test_physical_size():
    # src/layout.jl:113, :194 / :152, :246 / :342-345 / :381-383
    assert Layout.physical_size(Layout.Padded[ACM[F16], 8], NT(M=128, K=64)) == (136, 64)
    assert Layout.physical_size(Layout.Padded[ARM[F16], 8], NT(M=128, K=64)) == (72, 128)
    assert Layout.physical_size(ACM[F32], NT(M=128, N=128)) == (128, 128)
    assert Layout.physical_size(Layout.SplitColMajor[F32], NT(M=64, N=64)) == (64, 64, 2)
    assert Layout.physical_size(Layout.Padded[Layout.SplitRowMajor[F16], 8], NT(M=64, K=32)) == (40, 64, 2)
    assert Layout.physical_size(Layout.Padded[Layout.SplitColMajor[F16], 8], NT(M=64, K=32)) == (72, 32, 2)


def test_adjacent_elements_reference_answers():
    # src/config.jl:124-134; the mem tiles of the reference's default 128x128x64 config with 32 lanes
    assert gk.adjacent_elements(256, NT(M=128, K=64), True) == NT(M=128, K=2)
    assert gk.adjacent_elements(256, NT(M=128, K=64), False) == NT(M=4, K=64)
    assert gk.adjacent_elements(8, NT(M=128, K=64), True) == NT(M=8, K=1)
    assert gk.adjacent_elements(8, NT(M=128, K=64), False) == NT(M=1, K=8)
    assert gk.adjacent_elements(256, NT(K=64, N=128), True) == NT(K=64, N=4)
    assert gk.adjacent_elements(128, NT(M=128, N=128), True) == NT(M=128, N=1)
    assert gk.adjacent_elements(4, NT(M=128, N=128), True) == NT(M=4, N=1)


def base_kwargs(M=4096, N=4096, K=4096, **kw):
    d = dict(gemm_shape=NT(M=M, N=N, K=K), operator=Operator.MFMAOp[32, 32, 16, F16, F32],
             global_a_layout=ACM[F16], global_c_layout=ACM[F32])
    d.update(kw)
    return d


def test_get_config_defaults_for_the_headline_problem():
    conf = gk.get_config(**base_kwargs())
    assert conf.block_shape == NT(M=256, N=256, K=64)
    # whole 256 x 256 x 64 tiles: four waves, one per SIMD, with 128 x 128 wave tiles
    assert conf.warps_per_block == 4 and conf.compute_warp == NT(M=128, N=128, K=16)
    # ... also with tiles over the edges; eight waves with 128 x 64 wave tiles for a K of less than one tile
    col = Layout.ColMajor
    for size in (4000, 4001):
        ragged = gk.get_config(**base_kwargs(M=size, N=size + 2, K=size + 4, global_a_layout=col[F16], global_c_layout=col[F32],
                                             block_shape=NT(M=256, N=256, K=64)))
        assert ragged.warps_per_block == 4 and ragged.compute_warp == NT(M=128, N=128, K=16)
    short = gk.get_config(**base_kwargs(M=4000, N=4000, K=40, global_a_layout=col[F16], global_c_layout=col[F32],
                                        block_shape=NT(M=256, N=256, K=64)))
    assert short.warps_per_block == 8 and short.compute_warp == NT(M=128, N=64, K=16)
    assert conf.compute_op_shape == NT(M=32, N=32, K=16)
    # 64-lane waves, 16 bytes per lane (src/config.jl:240-260 with 64 lanes)
    assert conf.mem_a_warp == NT(M=256, K=2) and conf.mem_a_thread == NT(M=8, K=1)
    assert conf.mem_b_warp == NT(K=64, N=8) and conf.mem_b_thread == NT(K=8, N=1)
    assert conf.mem_cd_warp == NT(M=256, N=1) and conf.mem_cd_thread == NT(M=4, N=1)
    assert conf.global_b_layout == conf.global_a_layout and conf.global_d_layout == conf.global_c_layout
    assert conf.shared_a_layout == Layout.Padded[ACM[F16], 8]           # src/config.jl:191-194
    assert conf.cta_swizzle == CTASwizzle.XCDAware[8]            # (every CU has a tile: panels 8 tiles high)
    assert Kernel.shmem_size(conf, Kernel.matmul_pipelined) == 2 * (256 * 64 * 2 + 256 * 64 * 2)
    assert "block_shape:" in str(conf) and "(M = 256, N = 256, K = 64)" in str(conf)


def test_default_block_shape_shrinks_to_fill_the_chip():
    assert gk.default_block_shape(Operator.MFMAOp[32, 32, 16, F16, F32], NT(M=4096, N=4096, K=4096)) == NT(M=256, N=256, K=64)
    assert gk.default_block_shape(Operator.MFMAOp[32, 32, 16, F16, F32], NT(M=4096, N=4096, K=2048)) == NT(M=256, N=256, K=64)
    assert gk.default_block_shape(Operator.MFMAOp[32, 32, 16, F16, F32], NT(M=2048, N=2048, K=2048)) == NT(M=128, N=128, K=32)
    assert gk.default_block_shape(Operator.MFMAOp[32, 32, 16, F16, F32], NT(M=256, N=256, K=256)) == NT(M=64, N=64, K=64)
    assert gk.default_block_shape(Operator.MFMAOp[32, 32, 16, F16, F32], NT(M=256, N=256, K=96)) == NT(M=64, N=64, K=32)
    assert gk.default_block_shape(Operator.MFMAOp[32, 32, 16, F16, F32], NT(M=4096, N=4096, K=2048 + 32)) == NT(M=256, N=256, K=32)


ERROR_CASES = [
    # (name, kwargs overrides, expected status)
    ("block too small (src/config.jl:203-205)", dict(block_shape=NT(M=64, N=64, K=4), compute_warp=NT(M=32, N=32, K=16)), _lib.GK_ERR_BLOCK_SHAPE),
    ("block < 2 x operator (src/config.jl:209-212)", dict(block_shape=NT(M=32, N=128, K=64), compute_warp=NT(M=32, N=32, K=16), warps_per_block=4), _lib.GK_ERR_BLOCK_SHAPE),
    ("unsupported matrix-core shape (src/config.jl:159-169)", dict(operator=Operator.MFMAOp[16, 16, 4, F16, F32]), _lib.GK_ERR_OP_SHAPE),
    ("FPU base shape is not one wave (src/config.jl:147-149)", dict(operator=Operator.FPUOp[8, 8, 1, 4, 8, 1, F32, F32], block_shape=NT(M=64, N=64, K=32)), _lib.GK_ERR_OP_SHAPE),
    ("FPU lane grid other than 8 x 8 (one wave, but not the grid the kernels are compiled for)", dict(operator=Operator.FPUOp[16, 4, 1, 16, 4, 1, F32, F32], block_shape=NT(M=64, N=64, K=32)), _lib.GK_ERR_OP_SHAPE),
    ("FPU kb != 1 (src/config.jl:151-153)", dict(operator=Operator.FPUOp[8, 8, 2, 8, 8, 2, F32, F32], block_shape=NT(M=64, N=64, K=32)), _lib.GK_ERR_OP_SHAPE),
    ("FPU operator smaller than a wave (src/config.jl:142-145)", dict(operator=Operator.FPUOp[4, 8, 1, 4, 8, 1, F32, F32], block_shape=NT(M=64, N=64, K=32)), _lib.GK_ERR_OP_SHAPE),
    ("FPU shape not a multiple of its base (src/config.jl:155-157)", dict(operator=Operator.FPUOp[12, 8, 1, 8, 8, 1, F32, F32], block_shape=NT(M=64, N=64, K=32)), _lib.GK_ERR_OP_SHAPE),
    ("mem_a_warp too big (src/config.jl:263)", dict(block_shape=NT(M=128, N=128, K=64), mem_a_warp=NT(M=128, K=64)), _lib.GK_ERR_MEM_TILE),
    ("mem_b_warp too big (src/config.jl:264)", dict(block_shape=NT(M=128, N=128, K=64), mem_b_warp=NT(K=64, N=128)), _lib.GK_ERR_MEM_TILE),
    ("mem_cd_warp too big (src/config.jl:265)", dict(block_shape=NT(M=128, N=128, K=64), mem_cd_warp=NT(M=128, N=128)), _lib.GK_ERR_MEM_TILE),
    ("block not a multiple of compute_warp (src/config.jl:270)", dict(block_shape=NT(M=128, N=128, K=64), compute_warp=NT(M=96, N=64, K=16)), _lib.GK_ERR_TILE_MULTIPLE),
    ("compute_warp not a multiple of the operator (src/config.jl:271)", dict(block_shape=NT(M=128, N=128, K=64), compute_warp=NT(M=64, N=16, K=16), warps_per_block=16), _lib.GK_ERR_TILE_MULTIPLE),
    ("gemm not a multiple of the block, aligned layouts (src/config.jl:272-275)", dict(gemm_shape=NT(M=1000, N=1024, K=1024), block_shape=NT(M=128, N=128, K=64)), _lib.GK_ERR_TILE_MULTIPLE),
    ("FP64 D with the matrix cores", dict(global_d_layout=ACM[gk.Float64]), _lib.GK_ERR_UNSUPPORTED),
    ("FP16 D on the vector ALUs", dict(operator=Operator.FPUOp[8, 8, 1, 8, 8, 1, F32, F32], block_shape=NT(M=64, N=64, K=32),
                                       global_a_layout=ACM[F32], global_b_layout=ACM[F32], global_d_layout=ACM[F16]), _lib.GK_ERR_UNSUPPORTED),
    ("no compiled instance", dict(block_shape=NT(M=192, N=192, K=64), compute_warp=NT(M=96, N=96, K=16), warps_per_block=4, gemm_shape=NT(M=384, N=384, K=128)), _lib.GK_ERR_UNSUPPORTED),
    ("warps_per_block disagrees with block / compute_warp", dict(block_shape=NT(M=128, N=128, K=64), compute_warp=NT(M=64, N=64, K=16), warps_per_block=8), _lib.GK_ERR_UNSUPPORTED),
]


@pytest.mark.parametrize("name,over,status", ERROR_CASES, ids=[c[0] for c in ERROR_CASES])
def test_config_errors(name, over, status):
    with pytest.raises(ConfigError) as ei:
        gk.get_config(**base_kwargs(**over))
    assert ei.value.status == status, ei.value.message
    assert len(ei.value.message) > 10


def test_checked_layouts_lift_the_divisibility_rule():
    # src/config.jl:175-178: Zero / ColMajor / RowMajor do not need tile-sized operands
    with pytest.raises(ConfigError) as ei:
        gk.get_config(**base_kwargs(M=1000, N=1000, K=1000, block_shape=NT(M=64, N=64, K=32),
                                    global_a_layout=Layout.ColMajor[F16], global_b_layout=Layout.ColMajor[F16],
                                    global_c_layout=Layout.ColMajor[F32], global_d_layout=ACM[F32]))
    assert ei.value.status == _lib.GK_ERR_TILE_MULTIPLE      # D is still an aligned layout


def test_lds_stage_and_thread_limits():
    conf = gk.get_config(**base_kwargs())
    try:
        _lib.lib().gk_set_device_limits(64 * 1024, 0)          # src/matmul.jl:28-31
        with pytest.raises(ConfigError) as ei:
            gk.check_config(conf, Kernel.matmul_pipelined)
        assert ei.value.status == _lib.GK_ERR_LDS and "shared memory" in ei.value.message
        _lib.lib().gk_set_device_limits(0, 128)                # src/matmul.jl:41 (the configuration runs 256 threads)
        with pytest.raises(ConfigError) as ei:
            gk.check_config(conf, Kernel.matmul_pipelined)
        assert ei.value.status == _lib.GK_ERR_THREADS
    finally:
        _lib.lib().gk_set_device_limits(0, 0)
    gk.check_config(conf, Kernel.matmul_pipelined)
    # src/matmul.jl:34-36: pipelined kernels need BLOCK_K >= 2 * OPERATOR_K; single-stage does not
    kw = base_kwargs(block_shape=NT(M=64, N=64, K=16), compute_warp=NT(M=32, N=32, K=16), warps_per_block=4, kernel=Kernel.matmul_pipelined)
    with pytest.raises(ConfigError) as ei:
        gk.get_config(**kw)
    assert ei.value.status == _lib.GK_ERR_STAGES


def test_alignment_and_null_pointer_checks_happen_before_any_launch():
    conf = gk.get_config(**base_kwargs(M=256, N=256, K=256, block_shape=NT(M=128, N=128, K=64)))
    c = conf.to_c(256, 256, 256, 256)
    lib = _lib.lib()
    call = lambda a, b, cc, d: lib.gk_matmul(ctypes.byref(c), a, b, cc, d, None, None, Kernel.matmul_pipelined.code, None)
    assert call(0x1008, 0x2000, 0x3000, 0x4000) == _lib.GK_ERR_ALIGNMENT and "A is not aligned" in _lib.last_error()
    assert call(0x1000, 0x2000, 0x3000, 0x4004) == _lib.GK_ERR_ALIGNMENT
    assert call(None, 0x2000, 0x3000, 0x4000) == _lib.GK_ERR_INVALID_ARGUMENT
    assert call(0x1000, 0x2000, None, 0x4000) == _lib.GK_ERR_INVALID_ARGUMENT      # C is not Zero
    c_bad = conf.to_c(260, 256, 256, 256)                                            # lda * 2 B not a multiple of 16
    assert lib.gk_matmul(ctypes.byref(c_bad), 0x1000, 0x2000, 0x3000, 0x4000, None, None, 1, None) == _lib.GK_ERR_ALIGNMENT
    c_small = conf.to_c(128, 256, 256, 256)                                          # lda < M
    assert lib.gk_matmul(ctypes.byref(c_small), 0x1000, 0x2000, 0x3000, 0x4000, None, None, 1, None) == _lib.GK_ERR_DIMENSION_MISMATCH


def test_create_config_choices():
    # reference src/matmul.jl:66-183
    args = (F16, (4096, 4096), (1, 4096), False, F16, (4096, 4096), (1, 4096), False, F32, (4096, 4096), (1, 4096), float, False, float, False, None)
    conf, compute_type, kernel = create_config(*args)
    assert compute_type == F16 and kernel == Kernel.matmul_pipelined
    assert conf.operator.kind == Operator.MFMA and conf.block_shape == NT(M=256, N=256, K=64)
    assert conf.global_a_layout == ACM[F16] and conf.global_c_layout == ACM[F32]
    # transposed operands pick the row-major family and flip is_*_col_major (:79-83, :160-161)
    conf, _, _ = create_config(F16, (4096, 4096), (1, 4096), True, F16, (4096, 4096), (1, 4096), True, F32, (4096, 4096), (1, 4096), float, False, float, False, None)
    assert conf.global_a_layout == ARM[F16] and conf.global_b_layout == ARM[F16] and not conf.is_a_col_major
    # beta == 0 elides the C load (:139-145)
    conf, _, _ = create_config(F16, (4096, 4096), (1, 4096), False, F16, (4096, 4096), (1, 4096), False, F32, (4096, 4096), (1, 4096), float, False, float, True, None)
    assert conf.global_c_layout == Layout.Zero[F32] and conf.shared_c_layout == Layout.Zero[F32]
    with pytest.raises(DimensionMismatch):                                           # :75-77
        create_config(F16, (128, 64), (1, 128), False, F16, (128, 128), (1, 128), False, F32, (128, 128), (1, 128), float, False, float, False, None)


def test_which_launches_of_the_headline_tile_run_on_four_waves():
    """What the library runs for a configuration of the 256 x 256 x 64 tile with four waves (one per SIMD): that
    arrangement where it is compiled for the launch, the eight-wave arrangement of the same tile elsewhere (same bits)."""
    from gemmkernels import Transform, Epilogue
    col = Layout.ColMajor

    def name(M, N, K, c=F32, d=F32, checked=False, **kw):
        lay = col if checked else ACM
        conf = gk.get_config(gemm_shape=NT(M=M, N=N, K=K), block_shape=NT(M=256, N=256, K=64), warps_per_block=4,
                             compute_warp=NT(M=128, N=128, K=16), operator=Operator.MFMAOp[32, 32, 16, F16, F32],
                             global_a_layout=lay[F16], global_b_layout=lay[F16], global_c_layout=lay[c], global_d_layout=lay[d])
        return gk.kernel_name(conf, Kernel.matmul_pipelined, **kw)

    assert name(4096, 4096, 4096) == "mfma_gemm_nn_256x256x64_w2x2_s2__Float16"
    assert name(4096, 4096, 4096, c=F16, d=F16) == "mfma_gemm_nn_256x256x64_w2x2_s2__Float16"
    # tiles over the edges, a partial last K tile, odd extents: an instance of its own
    for size in ((4000, 4000, 4000), (4001, 4003, 4005), (8, 1032, 64)):
        assert name(*size, checked=True) == "mfma_gemm_nn_256x256x64_w2x2_s2__Float16_edges"
    # ... for FP32 C / D and at least one whole K tile
    assert "_w2x4_" in name(4000, 4000, 4000, d=F16, checked=True)
    assert "_w2x4_" in name(4000, 4000, 40, checked=True)
    # hooks of D in closed form and a bias; any other hook runs on eight waves
    E = Transform.Elementwise
    assert name(512, 512, 512, transforms=dict(transform_shared_to_global_d=E(Transform.relu)), epilogue=Epilogue.Bias(None)).endswith("_w2x2_s2__Float16_fused_d")
    assert "_w2x4_" in name(512, 512, 512, transforms=dict(transform_global_to_shared_c=E(lambda x: x * 0.25)))
    assert "_w2x4_" in name(4000, 4000, 4000, checked=True, transforms=dict(transform_shared_to_global_d=E(Transform.relu)))


def test_every_tile_of_the_python_tables_has_a_compiled_instance():
    """The tile tables the defaults are drawn from and the instances compiled into the library
    must not drift apart: every entry resolves to a kernel name."""
    from gemmkernels import config as cfg, configs
    for (bm, bn, bk), (wm, wn) in cfg._MFMA_TILES:
        conf = configs.mfma_config(2 * bm, 2 * bn, 4 * bk, block_shape=(bm, bn, bk), warps_per_block=wm * wn,
                                   compute_warp=NT(M=bm // wm, N=bn // wn, K=16))
        assert f"{bm}x{bn}x{bk}_w{wm}x{wn}" in gk.kernel_name(conf, Kernel.matmul_pipelined)
    for (bm, bn, bk), (wm, wn) in cfg._FPU_TILES:
        conf = gk.get_config(gemm_shape=NT(M=2 * bm, N=2 * bn, K=2 * bk), block_shape=NT(M=bm, N=bn, K=bk), warps_per_block=wm * wn,
                             compute_warp=NT(M=bm // wm, N=bn // wn, K=bk),
                             operator=Operator.FPUOp[8, 8, 1, 8, 8, 1, F32, F32], global_a_layout=ACM[F32], global_c_layout=ACM[F32])
        assert f"{bm}x{bn}x{bk}_w{wm}x{wn}" in gk.kernel_name(conf, Kernel.matmul_pipelined)
    for dual in (False, True):
        for ta in (False, True):
            for tb in (False, True):
                op = Operator.MFMADualOp if dual else Operator.MFMAComplexOp
                for (bm, bn, bk), (wm, wn) in cfg._complex_tiles(op[16, 16, 16, F16, F32], False, ta, not tb):
                    conf = configs.complex_config(2 * bm, 2 * bn, 4 * bk, ta, tb, dual=dual, block_shape=NT(M=bm, N=bn, K=bk))
                    name = gk.kernel_name(conf, Kernel.matmul_pipelined)
                    if (bm, bn, bk) == cfg._SOLO_COMPLEX_TILE and not ta and not tb:
                        wm, wn = cfg._SOLO_WAVES          # whole tiles of an 'N','N' launch: one wave per SIMD
                    assert f"_{'nt'[ta]}{'nt'[tb]}_{bm}x{bn}x{bk}_w{wm}x{wn}" in name, name
                    assert "pair" in name, name
    for (bm, bn, bk), (wm, wn) in cfg._PLANAR_TILES:
        conf = configs.complex_planar_config(2 * bm, 2 * bn, 4 * bk, block_shape=NT(M=bm, N=bn, K=bk))
        if (bm, bn, bk) == cfg._SOLO_COMPLEX_TILE:
            wm, wn = cfg._SOLO_WAVES          # whole tiles: one wave per SIMD
        assert f"{bm}x{bn}x{bk}_w{wm}x{wn}" in gk.kernel_name(conf, Kernel.matmul_pipelined)


@pytest.mark.parametrize("size", [(64, 64, 32), (128, 128, 64), (256, 256, 96), (512, 768, 128), (2048, 2048, 2048), (4096, 4096, 4096)])
def test_default_tiles_resolve_to_compiled_instances_for_every_kind_of_config(size):
    """Whatever tile the defaults pick for a problem, the library holds the instance: plain, with
    transforms on the fragments (the fused levels), BF16, 16-bit C/D, and tensor-contraction layouts
    (which are compiled for fewer tiles than the plain kernel)."""
    from gemmkernels import configs, BFloat16, Transform
    M, N, K = size
    for ta in (False, True):
        for tb in (False, True):
            conf = configs.mfma_config(M, N, K, ta=ta, tb=tb)
            assert gk.kernel_name(conf, Kernel.matmul_pipelined).startswith("mfma_gemm_")
            scale = Transform.Elementwise(lambda x: x * 2.0)
            for hook in ("transform_shared_to_regs_a", "transform_shared_to_regs_c"):
                assert gk.kernel_name(conf, Kernel.matmul_pipelined, transforms={hook: scale}).startswith("mfma_gemm_")
    conf = configs.mfma_config(M, N, K, operator=Operator.MFMAOp[32, 32, 16, BFloat16, F32],
                               global_a_layout=ACM[BFloat16], global_b_layout=ACM[BFloat16])
    assert "bf16" in gk.kernel_name(conf, Kernel.matmul_pipelined)
    conf = configs.mfma_config(M, N, K, global_c_layout=ACM[F16], global_d_layout=ACM[F16])
    assert gk.kernel_name(conf, Kernel.matmul_pipelined).startswith("mfma_gemm_")
    # a contraction with the same GEMM extents: M = a*b, N = c, K = d
    ext = dict(a=M // 32, b=32, c=N, d=K)
    conf, _ = configs.gett_config("bda", "dc", "abc", ext)
    assert gk.kernel_name(conf, Kernel.matmul_pipelined).endswith("_gett")


def test_complex_layout_rules_of_the_library():
    """Complex matrices are interleaved (the reference's global form) or planar, never a mix; planar
    ones are for the complex operator only, and only for tiles compiled with planar addressing."""
    from gemmkernels import configs
    M, N, K = 256, 256, 128
    conf = configs.complex_planar_config(M, N, K)
    assert "mfma_complex_planar_nn_" in gk.kernel_name(conf, Kernel.matmul_pipelined)
    assert "mfma_complex_pair_nn_" in gk.kernel_name(configs.complex_config(M, N, K), Kernel.matmul_pipelined)
    assert "mfma_complex_pair_tn_" in gk.kernel_name(configs.complex_config(M, N, K, True, False), Kernel.matmul_pipelined)
    cases = [
        dict(global_b_layout=Layout.InterleavedColMajor[F16]),                                   # planar A, interleaved B
        dict(global_d_layout=Layout.InterleavedColMajor[F32]),                                   # planar inputs, interleaved D
        dict(operator=Operator.MFMADualOp[16, 16, 16, F16, F32]),                                # dual numbers have no planar form
        dict(block_shape=NT(M=32, N=64, K=32)),                                                  # an interleaved-only tile
    ]
    for over in cases:
        with pytest.raises(ConfigError) as ei:
            configs.complex_planar_config(M, N, K, **over)
        assert ei.value.status in (_lib.GK_ERR_UNSUPPORTED, _lib.GK_ERR_BLOCK_SHAPE), ei.value.message
    with pytest.raises(ConfigError):                                                            # K not a multiple of the tile
        configs.complex_planar_config(M, N, 48)


def test_reference_shmem_size_known_answers():
    """Kernel.shmem_size as the reference computes it (src/kernel.jl:131-145, 352-366):
    max(size_c, size_a + size_b, size_d) over the shared layouts.  Answers evaluated by hand from the source:
    the 128 x 128 x 64 WMMA configuration (Padded F16 A / B by 8, F32 C / D): A (128+8)*64*2 = 17 408,
    B (64+8)*128*2 = 18 432, C = D = 128*128*4 = 65 536; the complex configuration of
    configs/configs.jl:385-416 (64 x 64 x 32, padded planar F16 A / B, planar F32 C / D): A (64+8)*32*2*2 = 9 216,
    B (32+8)*64*2*2 = 10 240, C = D = 64*64*2*4 = 32 768."""
    from gemmkernels import configs
    from gemmkernels.kernel import reference_shmem_size
    conf = gk.get_config(**base_kwargs(block_shape=NT(M=128, N=128, K=64), warps_per_block=4, compute_warp=NT(M=64, N=64, K=16)))
    assert conf.shared_a_layout == Layout.Padded[ACM[F16], 8]
    assert reference_shmem_size(conf) == 65536
    # with FP16 C and D the operand tiles decide: 17 408 + 18 432 against 32 768
    conf16 = gk.get_config(**base_kwargs(block_shape=NT(M=128, N=128, K=64), warps_per_block=4, compute_warp=NT(M=64, N=64, K=16),
                                         global_c_layout=ACM[F16], global_d_layout=ACM[F16]))
    assert reference_shmem_size(conf16) == 17408 + 18432
    cplx = configs.complex_config(128, 128, 128, zero_c=False, block_shape=NT(M=64, N=64, K=32))
    assert reference_shmem_size(cplx) == 32768
    # the operand part alone, through a configuration whose C / D tiles are smaller: B transposed keeps 10 240
    cplx_t = configs.complex_config(128, 128, 128, tb=True, zero_c=False, block_shape=NT(M=64, N=64, K=32))
    assert reference_shmem_size(cplx_t) == 32768
    c = cplx.to_c()
    from gemmkernels import _lib
    import ctypes
    c.shared_c_layout.kind = Layout.ZERO; c.shared_c_layout.eltype = 0; c.shared_c_layout.pad = 0
    c.shared_d_layout.kind = Layout.ALIGNED_COL_MAJOR; c.shared_d_layout.eltype = 0
    # C as a 64 x 64 F16 tile (8 192 B), D the same: now A + B = 9 216 + 10 240 wins
    assert _lib.lib().gk_reference_shmem_size(ctypes.byref(c)) == 9216 + 10240
