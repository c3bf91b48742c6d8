"""On-box tuning of the launch parameters, the counterpart of the reference's ``tuning/`` directory
(tuning/tune.jl, tuning/wmma.jl:34-47: a search over block shapes, warp counts and kernels whose best
configurations are kept in a file).  Here the search space is the set of kernel instances compiled
into the library times the panel height of the XCD-aware CTA swizzle; every candidate is timed on the
device with seeded data and the winners are kept in a JSON table that ``get_config`` consults when
the caller leaves the block shape open.

    python -m gemmkernels.tuning --shape 4096 4096 4096 --transposes NN --save table.json
    GEMMKERNELS_TUNING_TABLE=table.json python your_program.py
"""
from __future__ import annotations

import argparse
import json
import sys
from typing import Iterable, Optional

from . import config as _config
from . import cta_swizzle as CTASwizzle
from . import kernel as Kernel
from . import layout as Layout
from . import operator as Operator
from . import rng
from .dtypes import Float16, Float32
from .errors import ConfigError
from .tiling import NT

# every MFMA instance of the library: (block shape, waves M x N)
MFMA_CANDIDATES = [
    ((256, 256, 64), (2, 4)), ((256, 256, 64), (2, 2)),     # (2, 2): one wave per SIMD, plain products only
    ((256, 256, 32), (2, 4)), ((256, 256, 32), (4, 2)),
    ((256, 128, 64), (2, 2)), ((128, 256, 64), (2, 2)),
    ((128, 128, 64), (2, 2)), ((128, 128, 64), (4, 2)), ((128, 128, 32), (2, 2)),
    ((64, 64, 64), (2, 2)), ((64, 64, 32), (2, 2)), ((64, 64, 32), (1, 1)),
    ((256, 192, 64), (4, 2)), ((192, 256, 64), (2, 4)),     # compiled for the transposes whose 192 side is contiguous along k; skipped elsewhere
    ((256, 192, 64), (2, 2)), ((192, 256, 64), (2, 2)),     # ... and on one wave per SIMD (plain products in whole tiles)
]
SWIZZLE_PANELS = (1, 2, 4, 8, 16)


def mfma_config(M, N, K, ta, tb, block, waves, panel, zero_c=False, ab=Float16, cd=Float32):
    """The configuration of one candidate."""
    col, row = Layout.UnsafeAlignedColMajor, Layout.UnsafeAlignedRowMajor
    return _config.get_config(
        gemm_shape=NT(M=M, N=N, K=K), operator=Operator.MFMAOp[32, 32, 16, ab, Float32],
        global_a_layout=(row if ta else col)[ab], global_b_layout=(row if tb else col)[ab],
        global_c_layout=Layout.Zero[cd] if zero_c else col[cd], global_d_layout=col[cd],
        is_a_col_major=not ta, is_b_col_major=not tb,
        block_shape=NT(M=block[0], N=block[1], K=block[2]), warps_per_block=waves[0] * waves[1],
        compute_warp=NT(M=block[0] // waves[0], N=block[1] // waves[1], K=16),
        cta_swizzle=CTASwizzle.XCDAware[panel], kernel=Kernel.matmul_pipelined)


def tune_mfma(M: int, N: int, K: int, ta: bool = False, tb: bool = False, zero_c: bool = False,
              candidates: Optional[Iterable] = None, panels: Iterable[int] = SWIZZLE_PANELS,
              launches: int = 20, warmup: int = 3, rounds: int = 3, verbose: bool = False) -> list:
    """Times every candidate that the library accepts for the problem (the others raise ConfigError,
    like the skipped configurations of the reference's sweep) and returns the measurements, fastest
    first: dicts with block, waves, panel, us, tflops.

    The part is power-limited, so what a candidate measures depends on what ran just before it.  All
    candidates are therefore timed in ``rounds`` interleaved passes (after one untimed pass that warms
    the chip up) and the median of a candidate's passes is its result."""
    import torch
    from .arrays import colmajor, colmajor_empty
    from .matmul import plan
    a = colmajor(rng.matrix("upm1_f16", 1, (K, M) if ta else (M, K)))
    b = colmajor(rng.matrix("upm1_f16", 2, (N, K) if tb else (K, N)))
    c = None if zero_c else colmajor(rng.matrix("upm1_f32", 3, (M, N)))
    d = colmajor_empty((M, N), torch.float32)
    steps = []
    for block, waves in (MFMA_CANDIDATES if candidates is None else candidates):
        for panel in panels:
            try:
                conf = mfma_config(M, N, K, ta, tb, block, waves, panel, zero_c)
            except ConfigError:
                break                      # the tile does not fit the problem: no panel height will
            steps.append((block, waves, panel, plan(conf, a, b, c, d, kernel=Kernel.matmul_pipelined)))

    def timed(step, n):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(n):
            step()
        stop.record()
        stop.synchronize()
        return start.elapsed_time(stop) * 1e3 / n

    for _, _, _, step in steps:            # untimed pass: first launches, clocks and caches settle
        timed(step, warmup)
    samples = [[] for _ in steps]
    for _ in range(max(1, rounds)):
        for i, (_, _, _, step) in enumerate(steps):
            samples[i].append(timed(step, launches))
    results = []
    for (block, waves, panel, _), s in zip(steps, samples):
        us = sorted(s)[len(s) // 2]
        results.append(dict(block=list(block), waves=list(waves), panel=panel, us=round(us, 2),
                            tflops=round(2.0 * M * N * K / us / 1e6, 1)))
        if verbose:
            print(results[-1], file=sys.stderr, flush=True)
    results.sort(key=lambda r: r["us"])
    return results


def table_key(M, N, K, ta, tb, ab=Float16) -> str:
    return f"mfma/{ab.name}/{'T' if ta else 'N'}{'T' if tb else 'N'}/{M}x{N}x{K}"


def install(table: dict) -> None:
    """Makes ``get_config`` use the table for problems it holds (when the caller gives no block shape)."""
    _config.TUNED.update(table)


def load(path: str) -> dict:
    with open(path) as f:
        table = json.load(f)
    install(table)
    return table


def save(path: str, table: dict) -> None:
    with open(path, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)


def main(argv=None):
    p = argparse.ArgumentParser(description="time every compiled MFMA instance on one problem")
    p.add_argument("--shape", type=int, nargs=3, default=[4096, 4096, 4096], metavar=("M", "N", "K"))
    p.add_argument("--transposes", default="NN", choices=["NN", "NT", "TN", "TT"])
    p.add_argument("--zero-c", action="store_true")
    p.add_argument("--launches", type=int, default=20)
    p.add_argument("--save", help="JSON table to create or extend with the winner")
    args = p.parse_args(argv)
    M, N, K = args.shape
    ta, tb = args.transposes[0] == "T", args.transposes[1] == "T"
    results = tune_mfma(M, N, K, ta, tb, args.zero_c, launches=args.launches, verbose=True)
    if not results:
        print("no compiled instance fits this problem", file=sys.stderr)
        return 1
    best = results[0]
    print(json.dumps({"problem": table_key(M, N, K, ta, tb), "best": best, "candidates": len(results)}))
    if args.save:
        try:
            with open(args.save) as f:
                table = json.load(f)
        except FileNotFoundError:
            table = {}
        table[table_key(M, N, K, ta, tb)] = {k: best[k] for k in ("block", "waves", "panel")}
        save(args.save, table)
    return 0


if __name__ == "__main__":
    sys.exit(main())
