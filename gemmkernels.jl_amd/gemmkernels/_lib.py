"""ctypes binding of libgemmkernels_hip.so (the C ABI declared in include/gemmkernels_hip.h).

The library is required: there is no CPU fallback.  Loading fails loudly when it has not been
built (``python -c "import __graft_entry__ as g; g.build()"`` or ``make -C gemmkernels.jl_amd/csrc``).
"""
from __future__ import annotations

import ctypes
import os

GK_MAX_OPS = 4
GK_MAX_MODES = 4

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.normpath(os.path.join(_HERE, "..", "lib", "libgemmkernels_hip.so"))

# status codes
GK_OK = 0
GK_ERR_INVALID_ARGUMENT = 1
GK_ERR_LDS = 2
GK_ERR_STAGES = 3
GK_ERR_THREADS = 4
GK_ERR_BLOCK_SHAPE = 5
GK_ERR_OP_SHAPE = 6
GK_ERR_MEM_TILE = 7
GK_ERR_TILE_MULTIPLE = 8
GK_ERR_ALIGNMENT = 9
GK_ERR_UNSUPPORTED = 10
GK_ERR_DIMENSION_MISMATCH = 11
GK_ERR_HIP = 12


class gk_shape(ctypes.Structure):
    _fields_ = [("M", ctypes.c_int32), ("N", ctypes.c_int32), ("K", ctypes.c_int32)]


class gk_operator(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("M", ctypes.c_int32), ("N", ctypes.c_int32), ("K", ctypes.c_int32),
                ("mb", ctypes.c_int32), ("nb", ctypes.c_int32), ("kb", ctypes.c_int32),
                ("compute_type", ctypes.c_int32), ("accum_type", ctypes.c_int32)]


class gk_layout(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("eltype", ctypes.c_int32), ("pad", ctypes.c_int32),
                ("reserved", ctypes.c_int32), ("ld", ctypes.c_int64)]


class gk_swizzle(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("param", ctypes.c_int32)]


class gk_gett_dim(ctypes.Structure):
    _fields_ = [("nmodes", ctypes.c_int32), ("extent", ctypes.c_int32 * GK_MAX_MODES),
                ("stride0", ctypes.c_int64 * GK_MAX_MODES), ("stride1", ctypes.c_int64 * GK_MAX_MODES)]


class gk_gett(ctypes.Structure):
    _fields_ = [("m", gk_gett_dim), ("n", gk_gett_dim), ("k", gk_gett_dim)]


class gk_config(ctypes.Structure):
    _fields_ = [("matmul_shape", gk_shape), ("block_shape", gk_shape), ("warps_per_block", ctypes.c_int32),
                ("mem_a_warp", gk_shape), ("mem_a_thread", gk_shape),
                ("mem_b_warp", gk_shape), ("mem_b_thread", gk_shape),
                ("mem_cd_warp", gk_shape), ("mem_cd_thread", gk_shape),
                ("compute_warp", gk_shape), ("compute_op_shape", gk_shape),
                ("global_a_layout", gk_layout), ("global_b_layout", gk_layout),
                ("global_c_layout", gk_layout), ("global_d_layout", gk_layout),
                ("shared_a_layout", gk_layout), ("shared_b_layout", gk_layout),
                ("shared_c_layout", gk_layout), ("shared_d_layout", gk_layout),
                ("op", gk_operator), ("is_a_col_major", ctypes.c_int32), ("is_b_col_major", ctypes.c_int32),
                ("cta_swizzle", gk_swizzle), ("gett", gk_gett)]


class gk_op(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("p0", ctypes.c_float), ("p1", ctypes.c_float)]


class gk_transform(ctypes.Structure):
    _fields_ = [("n_ops", ctypes.c_int32), ("ops", gk_op * GK_MAX_OPS)]


class gk_transforms(ctypes.Structure):
    _fields_ = [("hook", gk_transform * 8)]


class gk_epilogue(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("reserved", ctypes.c_int32), ("bias", ctypes.c_void_p)]


# every symbol the header declares, with its signature
_SIGNATURES = {
    "gk_version": (ctypes.c_int, []),
    "gk_last_error": (ctypes.c_size_t, [ctypes.c_char_p, ctypes.c_size_t]),
    "gk_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "gk_set_device_limits": (ctypes.c_int, [ctypes.c_int64, ctypes.c_int32]),
    "gk_validate": (ctypes.c_int, [ctypes.POINTER(gk_config), ctypes.c_int32]),
    "gk_number_of_blocks": (ctypes.c_int, [ctypes.POINTER(gk_config), ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32)]),
    "gk_cta_swizzle": (ctypes.c_int, [ctypes.POINTER(gk_config), ctypes.c_int32, ctypes.c_int32,
                                      ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32)]),
    "gk_shmem_size": (ctypes.c_int64, [ctypes.POINTER(gk_config), ctypes.c_int32]),
    "gk_reference_shmem_size": (ctypes.c_int64, [ctypes.POINTER(gk_config)]),
    "gk_threads_per_block": (ctypes.c_int32, [ctypes.POINTER(gk_config)]),
    "gk_heuristic_block_shape": (ctypes.c_int, [ctypes.POINTER(gk_layout), ctypes.POINTER(gk_layout), ctypes.POINTER(gk_layout),
                                                ctypes.POINTER(gk_layout), ctypes.POINTER(gk_shape)]),
    "gk_kernel_name": (ctypes.c_int, [ctypes.POINTER(gk_config), ctypes.POINTER(gk_transforms), ctypes.POINTER(gk_epilogue),
                                      ctypes.c_int32, ctypes.c_char_p, ctypes.c_size_t]),
    "gk_matmul": (ctypes.c_int, [ctypes.POINTER(gk_config), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                 ctypes.POINTER(gk_transforms), ctypes.POINTER(gk_epilogue), ctypes.c_int32, ctypes.c_void_p]),
    "gk_split_k_workspace_size": (ctypes.c_int, [ctypes.POINTER(gk_config), ctypes.POINTER(ctypes.c_size_t)]),
    "gk_matmul_split_k": (ctypes.c_int, [ctypes.POINTER(gk_config), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                         ctypes.POINTER(gk_transforms), ctypes.POINTER(gk_epilogue), ctypes.c_void_p, ctypes.c_size_t,
                                         ctypes.c_void_p]),
    "gk_split_k_noalloc_capacity": (ctypes.c_size_t, []),
    "gk_matmul_split_k_noalloc": (ctypes.c_int, [ctypes.POINTER(gk_config), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                 ctypes.POINTER(gk_transforms), ctypes.POINTER(gk_epilogue), ctypes.c_void_p]),
    "gk_probe_matrix_rate": (ctypes.c_int, [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.POINTER(ctypes.c_double)]),
    "gk_rtc_compile": (ctypes.c_int, [ctypes.POINTER(gk_config), ctypes.POINTER(ctypes.c_char_p), ctypes.c_int32,
                                      ctypes.POINTER(ctypes.c_void_p)]),
    "gk_rtc_matmul": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(gk_config), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                     ctypes.c_void_p, ctypes.POINTER(gk_epilogue), ctypes.c_void_p]),
    "gk_rtc_kernel_name": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t]),
    "gk_dev_alloc": (ctypes.c_int, [ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]),
    "gk_dev_free": (ctypes.c_int, [ctypes.c_void_p]),
    "gk_copy_to_device": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
    "gk_copy_to_host": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]),
    "gk_synchronize": (ctypes.c_int, []),
    "gk_sizeof": (ctypes.c_int32, [ctypes.c_int32]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it is missing (no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP library first (make -C gemmkernels.jl_amd/csrc, "
                "or __graft_entry__.build()). There is no CPU fallback.")
        try:
            # torch carries its own copy of the HIP runtime; a process must hold exactly one, so when
            # torch is installed it is loaded first and this library binds to that copy.  (Loading the
            # library first would make a later `import torch` find a runtime it was not built with.)
            import torch  # noqa: F401
        except ImportError:
            pass
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        mirrors = (gk_config, gk_layout, gk_operator, gk_transforms, gk_epilogue, gk_gett)
        for which, struct in enumerate(mirrors):
            if handle.gk_sizeof(which) != ctypes.sizeof(struct):
                raise RuntimeError(f"ABI mismatch for {struct.__name__}: library {handle.gk_sizeof(which)} B, binding {ctypes.sizeof(struct)} B")
        _lib = handle
    return _lib


def last_error() -> str:
    buf = ctypes.create_string_buffer(1024)
    lib().gk_last_error(buf, len(buf))
    return buf.value.decode("utf-8", "replace")


def status_string(status: int) -> str:
    return lib().gk_status_string(status).decode()
