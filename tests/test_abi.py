"""The C-ABI library loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

from gemmkernels import _lib

HEADER = os.path.join(os.path.dirname(__file__), "..", "include", "gemmkernels_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gk_[a-z_0-9]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    names = declared_functions()
    assert len(names) >= 12
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(handle, name), f"{name} is declared in the header but not exported"
    assert sorted(_lib.EXPORTED_SYMBOLS) == names, "the Python binding must cover exactly the header"


def test_struct_sizes_match_the_library():
    lib = _lib.lib()     # lib() itself raises on any mismatch
    for which, struct in enumerate((_lib.gk_config, _lib.gk_layout, _lib.gk_operator, _lib.gk_transforms, _lib.gk_epilogue, _lib.gk_gett)):
        assert lib.gk_sizeof(which) == ctypes.sizeof(struct)
    assert lib.gk_sizeof(99) == -1


def test_version_and_status_strings():
    lib = _lib.lib()
    assert lib.gk_version() == 100
    assert _lib.status_string(0) == "GK_OK"
    assert _lib.status_string(_lib.GK_ERR_LDS) == "GK_ERR_LDS"
    assert _lib.status_string(12345) == "GK_ERR_UNKNOWN"


def test_null_config_is_an_error_not_a_crash():
    lib = _lib.lib()
    assert lib.gk_validate(None, 0) == _lib.GK_ERR_INVALID_ARGUMENT
    assert "NULL" in _lib.last_error()
    assert lib.gk_shmem_size(None, 0) == -1
    assert lib.gk_matmul(None, None, None, None, None, None, None, 0, None) == _lib.GK_ERR_INVALID_ARGUMENT


def test_malformed_transforms_and_epilogues_are_refused():
    import gemmkernels as gk
    from gemmkernels import configs, Kernel
    conf = configs.mfma_config(256, 256, 128).to_c()
    lib = _lib.lib()
    t = _lib.gk_transforms()
    t.hook[2].n_ops = 5                                    # more than a hook holds
    buf = ctypes.create_string_buffer(64)
    assert lib.gk_kernel_name(ctypes.byref(conf), ctypes.byref(t), None, Kernel.matmul_pipelined.code, buf, 64) == _lib.GK_ERR_INVALID_ARGUMENT
    t.hook[2].n_ops = 1
    t.hook[2].ops[0].kind = 42                              # not an op of the vocabulary
    assert lib.gk_kernel_name(ctypes.byref(conf), ctypes.byref(t), None, Kernel.matmul_pipelined.code, buf, 64) == _lib.GK_ERR_INVALID_ARGUMENT
    e = _lib.gk_epilogue()
    e.kind = 7
    assert lib.gk_kernel_name(ctypes.byref(conf), None, ctypes.byref(e), Kernel.matmul_pipelined.code, buf, 64) == _lib.GK_ERR_INVALID_ARGUMENT
    assert "epilogue" in _lib.last_error()


def test_error_messages_are_per_thread():
    """gk_last_error is thread-local: concurrent callers never read each other's message."""
    import threading
    import gemmkernels as gk
    from gemmkernels import configs, Kernel, NT
    good = configs.mfma_config(256, 256, 128).to_c()
    lds_hungry = configs.mfma_config(512, 512, 128, block_shape=(256, 256, 64)).to_c()
    bad_block = _lib.gk_config.from_buffer_copy(good)
    bad_block.block_shape.K = 4
    lib = _lib.lib()
    failures = []

    def worker(conf, want_status, needle):
        for _ in range(300):
            rc = lib.gk_validate(ctypes.byref(conf), Kernel.matmul_pipelined.code)
            msg = _lib.last_error() if rc != _lib.GK_OK else ""
            if rc != want_status or needle not in msg:
                failures.append((rc, msg))
                return

    threads = [threading.Thread(target=worker, args=(good, _lib.GK_OK, "")),
               threading.Thread(target=worker, args=(bad_block, _lib.GK_ERR_BLOCK_SHAPE, "block shape")),
               threading.Thread(target=worker, args=(lds_hungry, _lib.GK_OK, ""))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures[:2]
