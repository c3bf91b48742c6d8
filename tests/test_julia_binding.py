"""The Julia host layer (gemmkernels.jl_amd/julia/GemmKernelsHIP) cannot be executed in the build image (no Julia).
These checks read it as text: struct mirrors and enum tables against the C header and the tested Python binding,
ccalls against the exported symbols, block structure, and the names the integration notes rely on."""
import ctypes
import os
import re

from gemmkernels import _lib

ROOT = os.path.join(os.path.dirname(__file__), "..")
JL = os.path.join(ROOT, "gemmkernels.jl_amd", "julia", "GemmKernelsHIP", "src", "GemmKernelsHIP.jl")
HEADER = os.path.join(ROOT, "include", "gemmkernels_hip.h")
INTEGRATION = os.path.join(ROOT, "INTEGRATION.md")


def _strip(text):
    """Julia source without comments and string contents (docstrings included)."""
    out, i, n = [], 0, len(text)
    while i < n:
        if text.startswith('"""', i):
            j = text.index('"""', i + 3)
            out.append('""')
            i = j + 3
        elif text[i] == '"':
            j = i + 1
            while text[j] != '"':
                j += 2 if text[j] == "\\" else 1
            out.append('""')
            i = j + 1
        elif text[i] == "#":
            while i < n and text[i] != "\n":
                i += 1
        else:
            out.append(text[i])
            i += 1
    return "".join(out)


SRC = open(JL).read()
CODE = _strip(SRC)

_JL_TYPES = {"Int32": ctypes.c_int32, "Int64": ctypes.c_int64, "Float32": ctypes.c_float, "Ptr{Cvoid}": ctypes.c_void_p}


def _julia_structs():
    structs = {}
    for m in re.finditer(r"^struct (Gk\w+)(.*?)\bend$", CODE, re.S | re.M):
        structs[m.group(1)] = re.findall(r"(\w+)::([\w{},]+)", m.group(2))
    return structs


def _ctype(jl_type, structs_c):
    if jl_type in _JL_TYPES:
        return _JL_TYPES[jl_type]
    m = re.fullmatch(r"NTuple\{(\d+),(\w+)\}", jl_type)
    if m:
        return _ctype(m.group(2), structs_c) * int(m.group(1))
    return structs_c[jl_type]


def test_struct_mirrors_match_the_python_binding_field_by_field():
    jl = _julia_structs()
    pairs = {"GkShape": _lib.gk_shape, "GkOperator": _lib.gk_operator, "GkLayout": _lib.gk_layout, "GkSwizzle": _lib.gk_swizzle,
             "GkGettDim": _lib.gk_gett_dim, "GkGett": _lib.gk_gett, "GkConfig": _lib.gk_config, "GkOp": _lib.gk_op,
             "GkTransform": _lib.gk_transform, "GkTransforms": _lib.gk_transforms, "GkEpilogue": _lib.gk_epilogue}
    assert set(pairs) <= set(jl), sorted(set(pairs) - set(jl))
    built = {}
    for name in ("GkShape", "GkOperator", "GkLayout", "GkSwizzle", "GkGettDim", "GkGett", "GkOp", "GkTransform", "GkTransforms",
                 "GkEpilogue", "GkConfig"):
        py = pairs[name]
        fields = jl[name]
        assert [f for f, _ in fields] == [f for f, _ in py._fields_], name
        cls = type(name, (ctypes.Structure,), {"_fields_": [(f, _ctype(t, built)) for f, t in fields]})
        built[name] = cls
        assert ctypes.sizeof(cls) == ctypes.sizeof(py), name
        for (f, _), (g, _) in zip(fields, py._fields_):
            assert getattr(cls, f).offset == getattr(py, g).offset and getattr(cls, f).size == getattr(py, g).size, (name, f)
    lib = _lib.lib()
    for which, name in enumerate(("GkConfig", "GkLayout", "GkOperator", "GkTransforms", "GkEpilogue", "GkGett")):
        assert lib.gk_sizeof(which) == ctypes.sizeof(built[name])


def _header_enum(name):
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    body = re.search(r"typedef enum %s \{(.*?)\}" % name, text, re.S).group(1)
    out, nxt = {}, 0
    for item in body.split(","):
        item = item.strip()
        if not item:
            continue
        if "=" in item:
            k, v = item.split("=")
            nxt = int(v)
            out[k.strip()] = nxt
        else:
            out[item] = nxt
        nxt += 1
    return out


def _julia_dict(name):
    body = re.search(r"const %s = Dict\{Symbol,Int32\}\((.*?)\)\n" % name, SRC, re.S).group(1)
    return {k: int(v) for k, v in re.findall(r":(\w+) => (\d+)", body)}


def test_enum_tables_match_the_header():
    dt = _header_enum("gk_dtype")
    assert _julia_dict("DTYPE") == {"Float16": dt["GK_F16"], "BFloat16": dt["GK_BF16"], "Float32": dt["GK_F32"], "Float64": dt["GK_F64"],
                                    "Int16": dt["GK_I16"], "Int32": dt["GK_I32"], "Int64": dt["GK_I64"]}
    lay = _header_enum("gk_layout_kind")
    want = {"Zero": "ZERO", "ColMajor": "COL_MAJOR", "RowMajor": "ROW_MAJOR", "UnsafeAlignedColMajor": "ALIGNED_COL_MAJOR",
            "UnsafeAlignedRowMajor": "ALIGNED_ROW_MAJOR", "Diagonal": "DIAGONAL", "InterleavedColMajor": "INTERLEAVED_COL_MAJOR",
            "InterleavedRowMajor": "INTERLEAVED_ROW_MAJOR", "SplitColMajor": "SPLIT_COL_MAJOR", "SplitRowMajor": "SPLIT_ROW_MAJOR", "GETT": "GETT"}
    assert _julia_dict("LAYOUT_KIND") == {k: lay["GK_LAYOUT_" + v] for k, v in want.items()}
    ker = _header_enum("gk_kernel_kind")
    assert _julia_dict("KERNEL_KIND") == {"matmul_singlestage": ker["GK_KERNEL_SINGLESTAGE"], "matmul_pipelined": ker["GK_KERNEL_PIPELINED"],
                                          "matmul_pipelined_ng": ker["GK_KERNEL_PIPELINED_NG"], "matmul_split_k": ker["GK_KERNEL_SPLIT_K"]}
    ops = _header_enum("gk_op_kind")
    assert _julia_dict("OP_KIND") == {k.replace("GK_T_", "").lower(): v for k, v in ops.items()}
    opk = _header_enum("gk_operator_kind")
    jo = _julia_dict("OPERATOR_KIND")
    assert jo["MFMAOp"] == jo["WMMAOp"] == opk["GK_OP_MFMA"] and jo["FPUOp"] == opk["GK_OP_FPU"] and jo["TropicalFPUOp"] == opk["GK_OP_FPU_TROPICAL"]
    assert jo["MFMAComplexOp"] == jo["WMMAComplexOp"] == opk["GK_OP_MFMA_COMPLEX"] and jo["MFMADualOp"] == jo["WMMADualOp"] == opk["GK_OP_MFMA_DUAL"]
    swz = _header_enum("gk_swizzle_kind")
    assert _julia_dict("SWIZZLE_KIND") == {"Identity": swz["GK_SWIZZLE_IDENTITY"], "HorizontallyTiled": swz["GK_SWIZZLE_HORIZONTALLY_TILED"],
                                           "VerticallyTiled": swz["GK_SWIZZLE_VERTICALLY_TILED"], "LebesgueCurve": swz["GK_SWIZZLE_LEBESGUE"],
                                           "XCDAware": swz["GK_SWIZZLE_XCD"]}
    epi = _header_enum("gk_epilogue_kind")
    assert _julia_dict("EPILOGUE_KIND") == {"Default": epi["GK_EPILOGUE_DEFAULT"], "Bias": epi["GK_EPILOGUE_BIAS"], "BiasRow": epi["GK_EPILOGUE_BIAS_ROW"]}


def test_every_ccall_names_an_exported_symbol_with_the_right_number_of_arguments():
    calls = re.findall(r"ccall\(\(:(gk_\w+), libgk\[\]\),\s*(\w+),\s*\(([^()]*(?:\([^()]*\)[^()]*)*)\)", CODE)
    assert len(calls) >= 15
    for sym, ret, argtypes in calls:
        assert sym in _lib._SIGNATURES, sym
        restype, args = _lib._SIGNATURES[sym]
        given = [a for a in (x.strip() for x in argtypes.split(",")) if a]
        assert len(given) == len(args), (sym, given, len(args))
    used = {c[0] for c in calls}
    # the launcher, its K-split form, validation and the run-time compiler are all reachable from Julia
    assert {"gk_matmul", "gk_matmul_split_k", "gk_split_k_workspace_size", "gk_validate", "gk_rtc_compile", "gk_rtc_matmul",
            "gk_heuristic_block_shape", "gk_shmem_size", "gk_reference_shmem_size", "gk_number_of_blocks", "gk_last_error", "gk_sizeof"} <= used


def test_blocks_are_balanced():
    """Every block opener has its `end` (`end` inside brackets is an index, `x = if ...`-style openers are counted too)."""
    depth_brackets = 0
    openers = ends = 0
    tokens = re.findall(r"[\[\]]|\b(?:module|struct|function|if|for|while|let|begin|try|do|quote|macro|end|primitive type|abstract type)\b", CODE)
    prev_line_oneliner = 0
    for tok in tokens:
        if tok == "[":
            depth_brackets += 1
        elif tok == "]":
            depth_brackets -= 1
        elif tok == "end":
            if depth_brackets == 0:
                ends += 1
        elif depth_brackets == 0:
            openers += 1
    # `function name end` declarations (Kernel module) have an opener and an end of their own: already balanced
    assert depth_brackets == 0
    # comprehension `for` / `if` inside brackets were skipped with their brackets; generator `for` in parentheses:
    gen_for = len(re.findall(r"\((?:[^()\n]|\([^()\n]*\))* for \w+ in ", CODE))
    assert openers - gen_for == ends, (openers, gen_for, ends)


def _defined_names():
    names = set(re.findall(r"^\s*(?:mutable )?struct (\w+)", CODE, re.M))
    names |= set(re.findall(r"^\s*function (?:Base\.)?(\w+!?)", CODE, re.M))
    names |= set(re.findall(r"^\s*(\w+!?)\([^=\n]*\)(?: where \{[^}]*\})? *=", CODE, re.M))
    names |= set(re.findall(r"^\s*const (\w+)", CODE, re.M))
    names |= set(re.findall(r"^\s*module (\w+)", CODE, re.M))
    names |= set(re.findall(r"^\s*primitive type (\w+)", CODE, re.M))
    return names


def test_every_name_the_integration_notes_use_is_defined():
    text = open(INTEGRATION).read()
    blocks = re.findall(r"```julia\n(.*?)```", text, re.S)
    assert blocks
    used = set()
    for b in blocks:
        used |= set(re.findall(r"GemmKernelsHIP\.(\w+!?)", b))
    used |= set(re.findall(r"`GemmKernelsHIP\.(\w+!?)", text))
    defined = _defined_names()
    missing = sorted(u for u in used if u not in defined)
    assert not missing, missing
    # names used unqualified after `using GemmKernelsHIP` must be exported
    exported = set(re.findall(r"\w+!?", re.search(r"^export (.*?)\n\n", SRC, re.S | re.M).group(1)))
    for name in ("Layout", "Operator", "Transform", "Epilogue", "Kernel", "to_device", "DeviceArray", "get_config", "matmul", "mul!", "matmatmul!"):
        assert name in exported and name in defined, name
    # what the reference's API needs from the host layer (reference src/matmul.jl:58-215, src/config.jl:180-316)
    for name in ("Config", "get_config", "create_config", "matmatmul!", "mul!", "matmul", "lower", "lower_layout", "lower_operator",
                 "lower_swizzle", "lower_transform", "lower_epilogue", "empty_gett", "devptr", "heuristic_block_shape", "adjacent_elements",
                 "validate", "shmem_size", "specialize", "last_error"):
        assert name in defined, name


def test_get_config_keywords_are_the_reference_keywords():
    """reference src/config.jl:180-316: every keyword get_config reads there is read here (as params[:name])."""
    for kw in ("global_b_layout", "global_d_layout", "shared_a_layout", "shared_b_layout", "shared_c_layout", "shared_d_layout",
               "block_shape", "warps_per_block", "compute_warp", "is_a_col_major", "is_b_col_major", "mem_a_warp", "mem_b_warp",
               "mem_cd_warp", "mem_a_thread", "mem_b_thread", "mem_cd_thread", "cta_swizzle"):
        assert re.search(r"get\(params, :%s," % kw, CODE), kw
    assert re.search(r"function get_config\(; gemm_shape, operator, global_a_layout, global_c_layout, kwargs\.\.\.\)", CODE)


def test_tile_tables_match_the_python_tables():
    """The tables from which both host layers draw their default block shapes and wave grids."""
    from gemmkernels import config as cfg

    def jl_table(name):
        m = re.search(r"const " + name + r" = \[(.*?)\]\n", SRC, flags=re.S)
        assert m, name
        return [((int(a), int(b), int(c)), (int(d), int(e)))
                for a, b, c, d, e in re.findall(r"\(\((\d+), (\d+), (\d+)\), \((\d+), (\d+)\)\)", m.group(1))]

    assert jl_table("MFMA_TILES") == [(t, w) for t, w in cfg._MFMA_TILES]
    assert jl_table("COMPLEX_PAIR_TILES") == cfg._COMPLEX_PAIR_TILES == cfg._PLANAR_TILES
    assert jl_table("FPU_TILES") == cfg._FPU_TILES
