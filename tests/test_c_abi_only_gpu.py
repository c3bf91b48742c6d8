"""The drop-in boundary used the way a non-Python caller would: numpy host arrays, device memory from
the library's own helpers, integer addresses into gk_matmul.  No torch tensor is involved, so the
test also shows that torch is plumbing for the other tests and not part of the product path."""
import ctypes

import numpy as np
import pytest

import gemmkernels as gk
from gemmkernels import _lib, configs, rng, Kernel
from oracle import oracle

pytestmark = pytest.mark.gpu


class DeviceBuffer:
    def __init__(self, host: np.ndarray = None, nbytes: int = 0):
        self.lib = _lib.lib()
        self.nbytes = host.nbytes if host is not None else nbytes
        p = ctypes.c_void_p()
        assert self.lib.gk_dev_alloc(self.nbytes, ctypes.byref(p)) == _lib.GK_OK, _lib.last_error()
        self.ptr = p.value
        if host is not None:
            src = np.asfortranarray(host)
            assert self.lib.gk_copy_to_device(self.ptr, src.ctypes.data, src.nbytes) == _lib.GK_OK, _lib.last_error()

    def download(self, shape, dtype) -> np.ndarray:
        out = np.empty(shape, dtype=dtype, order="F")
        assert self.lib.gk_copy_to_host(out.ctypes.data, self.ptr, out.nbytes) == _lib.GK_OK, _lib.last_error()
        return out

    def free(self):
        assert self.lib.gk_dev_free(self.ptr) == _lib.GK_OK


def test_gemm_through_the_c_abi_without_torch(gpu):
    M, N, K = 512, 256, 384
    a, b, c = rng.matrix("upm1_f16", 1, (M, K)), rng.matrix("upm1_f16", 2, (K, N)), rng.matrix("upm1_f32", 3, (M, N))
    conf = configs.mfma_config(M, N, K)
    cconf = conf.to_c(M, K, M, M)
    A, B, C = DeviceBuffer(a), DeviceBuffer(b), DeviceBuffer(c)
    D = DeviceBuffer(nbytes=M * N * 4)
    lib = _lib.lib()
    rc = lib.gk_matmul(ctypes.byref(cconf), A.ptr, B.ptr, C.ptr, D.ptr, None, None, Kernel.matmul_pipelined.code, None)
    assert rc == _lib.GK_OK, _lib.last_error()
    assert lib.gk_synchronize() == _lib.GK_OK
    d = D.download((M, N), np.float32)
    assert oracle.rel_frobenius(d, oracle.gemm_f64(a, b, c, 1.0, 1.0)) <= 1e-3
    # a NULL operand is refused before anything is launched
    rc = lib.gk_matmul(ctypes.byref(cconf), A.ptr, None, C.ptr, D.ptr, None, None, Kernel.matmul_pipelined.code, None)
    assert rc == _lib.GK_ERR_INVALID_ARGUMENT
    for buf in (A, B, C, D):
        buf.free()


def test_matrix_rate_probe(gpu):
    """The measurement aid of the benchmark: a register-only MFMA loop.  Its rate lies between what no MI355X could fall
    below while it runs at all and the data-sheet peak of 2516.6 TFLOP/s; zeros draw less power than values spread over
    [-1, 1) and are at least as fast; arguments out of range are refused."""
    lib = _lib.lib()
    rates = {}
    for rnd in (1, 0):
        t = ctypes.c_double(0.0)
        for _ in range(2):
            assert lib.gk_probe_matrix_rate(10, 1000, rnd, None, ctypes.byref(t)) == _lib.GK_OK, _lib.last_error()
        rates[rnd] = t.value
    print("matrix-core rate: %.0f TFLOP/s on random FP16 values, %.0f on zeros" % (rates[1], rates[0]), flush=True)
    assert 500.0 < rates[1] <= 2516.6 * 1.01 and 500.0 < rates[0] <= 2516.6 * 1.01
    assert rates[0] >= 0.97 * rates[1]
    t = ctypes.c_double(0.0)
    assert lib.gk_probe_matrix_rate(0, 1000, 1, None, ctypes.byref(t)) == _lib.GK_ERR_INVALID_ARGUMENT
    assert lib.gk_probe_matrix_rate(10, 1000, 1, None, None) == _lib.GK_ERR_INVALID_ARGUMENT
