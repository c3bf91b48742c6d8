"""The compiled gfx950 kernels of the library, read from the code-object metadata of the built shared
object (no GPU): the MFMA kernels read their LDS fragments with inline assembly and hand-placed waits,
which is only sound while no fragment register is spilled between a read and its wait -- so an MFMA
kernel may use scratch memory only if it is one of those whose reads wait inside the assembly statement
that issues them (MfmaGemmConfig::SYNC_FRAGS) -- and every kernel must fit the 160 KiB of LDS and the
512-register file of a wave."""
import os
import re
import shutil
import struct
import subprocess

import pytest

LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gemmkernels.jl_amd", "lib", "libgemmkernels_hip.so")
LLVM = "/opt/rocm/llvm/bin"
MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"


COMPRESSED_MAGIC = b"CCOB"


def code_objects(tmp_path):
    """The gfx950 code objects bundled into the library (one per translation unit).  The library is built with
    --offload-compress: every bundle is a compressed one (magic CCOB, total size in its header), which the bundler of
    the toolchain unpacks; plain bundles (magic __CLANG_OFFLOAD_BUNDLE__) are read directly."""
    fat = tmp_path / "fatbin"
    subprocess.run([f"{LLVM}/llvm-objcopy", f"--dump-section=.hip_fatbin={fat}", LIB, os.devnull], check=True)
    data = fat.read_bytes()
    out = []
    for m in re.finditer(re.escape(COMPRESSED_MAGIC), data):
        p = m.start()
        version, method = struct.unpack_from("<HH", data, p + 4)
        if version >= 3:
            (total,) = struct.unpack_from("<Q", data, p + 8)
        else:
            (total,) = struct.unpack_from("<I", data, p + 8)
        if method not in (0, 1) or total < 24 or p + total > len(data):       # (a chance match inside other data)
            continue
        piece = tmp_path / f"bundle{len(out)}.ccob"
        piece.write_bytes(data[p:p + total])
        path = tmp_path / f"co{len(out)}.elf"
        r = subprocess.run([f"{LLVM}/clang-offload-bundler", "--type=o", f"--input={piece}", "--targets=hipv4-amdgcn-amd-amdhsa--gfx950",
                            f"--output={path}", "--unbundle"], capture_output=True, text=True)
        if r.returncode == 0 and path.exists() and path.stat().st_size > 0:
            out.append(path)
    for m in re.finditer(re.escape(MAGIC), data):
        p = m.start()
        (count,) = struct.unpack_from("<Q", data, p + len(MAGIC))
        off = p + len(MAGIC) + 8
        for _ in range(count):
            o, size, tlen = struct.unpack_from("<QQQ", data, off)
            off += 24
            triple = data[off:off + tlen].decode()
            off += tlen
            if "gfx950" in triple and size > 0:
                path = tmp_path / f"co{len(out)}.elf"
                path.write_bytes(data[p + o:p + o + size])
                out.append(path)
    return out


def kernel_metadata(path):
    """[(name, {field: int})] from the AMDGPU metadata note of one code object."""
    text = subprocess.run([f"{LLVM}/llvm-readelf", "--notes", str(path)], check=True, capture_output=True, text=True).stdout
    kernels, cur = [], None
    for line in text.splitlines():
        s = line.strip()
        m = re.match(r"-?\s*\.(\w+):\s*(.*)$", s)
        if not m:
            continue
        key, val = m.group(1), m.group(2).strip().strip("'\"")
        if s.startswith("- .") and key in ("agpr_count", "args"):      # first field of a kernel entry
            cur = {}
            kernels.append(cur)
        if cur is not None:
            cur[key] = val
    return [(k.get("name", "?"), k) for k in kernels if "name" in k and "vgpr_count" in k]


@pytest.mark.skipif(not (os.path.exists(LIB) and shutil.which(f"{LLVM}/llvm-readelf")), reason="library or LLVM tools not present")
def test_no_mfma_kernel_uses_scratch_and_every_kernel_fits_the_cu(tmp_path):
    objs = code_objects(tmp_path)
    assert len(objs) >= 8                                   # one per kernel translation unit
    seen = mfma = 0
    for obj in objs:
        for name, k in kernel_metadata(obj):
            seen += 1
            lds = int(k.get("group_segment_fixed_size", 0))
            scratch = int(k.get("private_segment_fixed_size", 0))
            spills = int(k.get("vgpr_spill_count", 0)) + int(k.get("sgpr_spill_count", 0))
            assert lds <= 160 * 1024, (name, lds)
            assert int(k["vgpr_count"]) <= 512, name          # vector and accumulation registers together
            m = re.search(r"mfma_gemm_kernelINS_14MfmaGemmConfigILi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)E[A-Za-z0-9_]+?Li(\d+)E", name)
            if m:
                mfma += 1
                bm, bn, _, wm, wn = (int(x) for x in m.groups()[:5])
                fuse = int(m.group(9))
                sync_reads = fuse == 2 or (bm // wm // 32) * (bn // wn // 32) > 8       # MfmaGemmConfig::SYNC_FRAGS
                if not sync_reads:
                    assert scratch == 0 and spills == 0, f"{name}: scratch {scratch} B, {spills} spills"
    assert seen > 100 and mfma > 100, (seen, mfma)
