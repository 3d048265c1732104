"""dynamic_tiling's sweep protocol for this library: time every candidate tiling of a shape, write the reference's
result.csv, pick the best row per shape.

Reference pieces mirrored (paths relative to the reference tree):
  warm-up 10 launches, 3 timed launches, mean        examples/dynamic_tiling/include/info.h:22-23,
                                                     examples/dynamic_tiling/utils/process_data.py:32-45
  result.csv header and row layout                   examples/dynamic_tiling/include/tiling.h:107-144
  best row = minimum Time(us) per (Op, M, K, N)      examples/dynamic_tiling/utils/get_best_res.py:73-83

The reference's own search space (commInterval x commTileM x core split, tiling.h:19-22) moves work between its cube and
vector cores; here the reduce runs in the GEMM's epilogue and those knobs do not change the kernel.  What does change it
on an MI355X: the macro tile (m0 = 128 two workgroups per CU, m0 = 256 one eight-wave workgroup), the tile order
(XCD-block order or the reference's linear order, swizzle offset / direction), commInterval through the round structure
of the launch order, and the k slices of few-tile launches.  The sweep walks those and keeps the reference's columns,
with the MI355X knobs and the achieved rate appended as extra columns.
"""
import csv

import torch

from . import lib as _l
from . import ops

REF_COLUMNS = ["Op", "M", "K", "N", "Transpose A", "Transpose B", "commInterval", "commTileM", "commBlockM", "commNpuSplit",
               "commDataSplit", "Time(us)"]
EXTRA_COLUMNS = ["m0", "swizzleOffset", "swizzleDirection", "linearOrder", "kSlices", "TOPS", "peakFraction"]
WARM_UP_TIMES = 10          # info.h:22
PERF_TEST_CYCLE_TIMES = 3   # info.h:23


def candidates(rows_per_rank, full_tiles):
    """The MI355X-side search space for one shape: (m0, (swizzle offset, direction), linear order, commInterval)."""
    # (256-row tiles take ragged problems too, from one whole tile of rows per rank on; the library rejects what it cannot run)
    m0s = [128] + ([256] if rows_per_rank >= 256 else []) + ([64] if rows_per_rank <= 64 else [])
    out = []
    for m0 in m0s:
        for swz in ((7, 1), (3, 0)):
            for linear in (False, True):
                for ci in (1, 4):
                    out.append((m0, swz, linear, ci))
    return out


def time_launch(fn, warm_up=WARM_UP_TIMES, cycles=PERF_TEST_CYCLE_TIMES):
    """Mean duration in microseconds of `cycles` launches after `warm_up` untimed ones (HIP events on the current stream)."""
    for _ in range(warm_up):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(cycles):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / cycles


def sweep_shape(op, make_launch, m, k, n, rank_size, trans_a, trans_b, peak_tops, full_tiles=True, warm_up=WARM_UP_TIMES,
                cycles=PERF_TEST_CYCLE_TIMES, progress=None):
    """Time every candidate of one shape.  make_launch(tiling, swizzle, linear) -> callable enqueuing one launch, or raises
    CatcocError for a candidate the library rejects (skipped).  Returns result rows (dicts keyed by the CSV columns)."""
    rows = []
    for m0, swz, linear, ci in candidates(m // max(rank_size, 1), full_tiles):
        t = ops.default_tiling(m, k, n, rank_size, m0=m0, n0=256, k0=256, commInterval=ci)
        try:
            fn = make_launch(t, swz, linear)
            fn()
            _l.check()
        except _l.CatcocError:
            continue
        us = time_launch(fn, warm_up, cycles)
        tops = 2.0 * m * n * k / us / 1e6
        if progress is not None:
            progress("[TEST] %s M=%d K=%d N=%d m0=%d swizzle=<%d,%d> linear=%d commInterval=%d: %.1f us" % (
                op, m, k, n, m0, swz[0], swz[1], int(linear), ci, us))
        rows.append({"Op": op, "M": m, "K": k, "N": n, "Transpose A": int(trans_a), "Transpose B": int(trans_b),
                     "commInterval": t.commInterval, "commTileM": t.commTileM, "commBlockM": t.commBlockM,
                     "commNpuSplit": t.commNpuSplit, "commDataSplit": t.commDataSplit, "Time(us)": round(us, 2),
                     "m0": m0, "swizzleOffset": swz[0], "swizzleDirection": swz[1], "linearOrder": int(linear), "kSlices": 1,
                     "TOPS": round(tops, 1), "peakFraction": round(tops / peak_tops, 4)})
    return rows


def write_result_csv(path, rows):
    """result.csv with the reference's header first (its post-processing reads those columns by name)."""
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=REF_COLUMNS + EXTRA_COLUMNS)
        w.writeheader()
        for r in rows:
            w.writerow(r)


def best_results(rows):
    """get_best_res.py: per (Op, M, K, N) the row with the smallest Time(us)."""
    best = {}
    for r in rows:
        key = (r["Op"], r["M"], r["K"], r["N"])
        if key not in best or r["Time(us)"] < best[key]["Time(us)"]:
            best[key] = r
    return list(best.values())
