"""gk_matmul_split_k_noalloc: the K-split launch whose workspace is a device array inside the library, for
callers that cannot allocate.  Called through the C ABI with raw addresses and compared, bit for bit, with
gk_matmul_split_k on a caller-owned workspace; two calls in a row, the second on a smaller product (the shared
array keeps what the first call left: the arrival counters must be back at zero)."""
import ctypes

import numpy as np
import pytest
import torch

import gemmkernels as gk
from gemmkernels import Kernel, _lib, configs, rng
from oracle import oracle

pytestmark = pytest.mark.gpu


def _both_ways(M, N, K, block, seed, with_c=True):
    lib = _lib.lib()
    conf = configs.mfma_config(M, N, K, block_shape=block)
    a = rng.matrix("upm1_f16", seed + 1, (M, K))
    b = rng.matrix("upm1_f16", seed + 2, (K, N))
    c = rng.matrix("upm1_f32", seed + 3, (M, N))
    A, B, C = gk.colmajor(a), gk.colmajor(b), gk.colmajor(c)
    cconf = conf.to_c(M, K, M, M)
    need = ctypes.c_size_t()
    assert lib.gk_split_k_workspace_size(ctypes.byref(cconf), ctypes.byref(need)) == _lib.GK_OK
    assert 0 < need.value <= lib.gk_split_k_noalloc_capacity()
    ws = torch.zeros(need.value, dtype=torch.uint8, device="cuda")
    d_ws = gk.colmajor_empty((M, N), torch.float32)
    d_na = gk.colmajor_empty((M, N), torch.float32)
    d_ws.fill_(float("nan"))
    d_na.fill_(float("nan"))
    torch.cuda.synchronize()
    rc = lib.gk_matmul_split_k(ctypes.byref(cconf), A.data_ptr(), B.data_ptr(), C.data_ptr(), d_ws.data_ptr(), None, None,
                               ws.data_ptr(), ws.numel(), None)
    assert rc == _lib.GK_OK, _lib.last_error()
    before = torch.cuda.memory_allocated()
    rc = lib.gk_matmul_split_k_noalloc(ctypes.byref(cconf), A.data_ptr(), B.data_ptr(), C.data_ptr(), d_na.data_ptr(), None, None, None)
    assert rc == _lib.GK_OK, _lib.last_error()
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    got_ws, got_na = gk.to_numpy(d_ws), gk.to_numpy(d_na)
    assert np.array_equal(got_na.view(np.uint32), got_ws.view(np.uint32))          # same kernel, same order of the sum
    assert oracle.rel_frobenius(got_na, oracle.gemm_f64(a, b, c, 1.0, 1.0)) <= 1e-3
    return got_na


def test_two_calls_in_a_row_the_second_smaller(gpu):
    print("no-alloc K-split: 4096 x 64 x 4096 on 64 x 64 x 64 tiles", flush=True)
    _both_ways(4096, 64, 4096, (64, 64, 64), 7100)
    print("no-alloc K-split: 128 x 192 x 2048 on 64 x 64 x 64 tiles", flush=True)
    _both_ways(128, 192, 2048, (64, 64, 64), 7200)
    print("no-alloc K-split: 256 x 256 x 8192 on 128 x 128 x 64 tiles", flush=True)
    _both_ways(256, 256, 8192, (128, 128, 64), 7300)
    print("no-alloc K-split: 64 x 64 x 4096", flush=True)
    _both_ways(64, 64, 4096, (64, 64, 64), 7400)
    # more tiles than any call before: the counters of the tiles 64 .. 127 lie where, with a counter region sized by
    # the tile count, the partial sums of the calls above would have been
    print("no-alloc K-split: 1024 x 512 x 2048 (128 tiles)", flush=True)
    _both_ways(1024, 512, 2048, (64, 64, 64), 7500)
    print("no-alloc K-split: 4096 x 64 x 4096 again", flush=True)
    _both_ways(4096, 64, 4096, (64, 64, 64), 7600)


def test_a_product_beyond_the_static_workspace_is_refused(gpu):
    lib = _lib.lib()
    M, N, K = 1024, 1024, 32768          # 64 tiles of 128 x 128 in 8 slices: 32 MiB of partial tiles plus the counters
    conf = configs.mfma_config(M, N, K, block_shape=(128, 128, 64))
    cconf = conf.to_c(M, K, M, M)
    A = torch.zeros(M * K, dtype=torch.float16, device="cuda")
    B = torch.zeros(K * N, dtype=torch.float16, device="cuda")
    D = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    rc = lib.gk_matmul_split_k_noalloc(ctypes.byref(cconf), A.data_ptr(), B.data_ptr(), D.data_ptr(), D.data_ptr(), None, None, None)
    assert rc == _lib.GK_ERR_INVALID_ARGUMENT
    msg = _lib.last_error()
    assert "static workspace" in msg and str(lib.gk_split_k_noalloc_capacity()) in msg
    torch.cuda.synchronize()
    assert float(D.abs().max()) == 0.0          # nothing ran
