"""CPU tests of the C-ABI library: exports, host-side scheduling and tiling logic (the same
integer code the kernels run) against the oracle, and argument validation.  No kernel is launched."""
import ctypes as C
import re
import os

import numpy as np
import pytest

import oracle
from mm_rs_with_catlass_amd import lib as L

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
u32 = C.c_uint32


@pytest.fixture(scope="module")
def so():
    return L.load()


def test_library_exports_every_declared_symbol(so):
    hdr = open(os.path.join(ROOT, "include", "catcoc_hip.h")).read()
    declared = set(re.findall(r"\b(catcoc_[a-z0-9_]+)\s*\(", hdr))
    assert declared, "no declarations found"
    assert declared == set(L.EXPORTS)
    for name in declared:
        assert hasattr(so, name), name


def test_struct_layout_matches_reference_tiling_params():
    # twelve uint32 in the reference's order (examples/dynamic_tiling/include/info.h:29-42)
    names = [f[0] for f in L.CocTilingParams._fields_]
    assert names == ["m", "k", "n", "m0", "k0", "n0", "commTileM", "commInterval", "commNpuSplit",
                     "commDataSplit", "commBlockM", "rankSize"]
    assert C.sizeof(L.CocTilingParams) == 48
    assert [getattr(L.CocTilingParams, n).offset for n in names] == list(range(0, 48, 4))


def test_registry_matches_reference_dispatcher(so):
    # launch_map.h:60-66 registers the three ops for FP16 and BF16; anything else is NULL
    for ct in (L.MATMUL_ALLREDUCE, L.ALLGATHER_MATMUL, L.MATMUL_REDUCE_SCATTER):
        for dt in (L.FP16, L.BF16):
            assert so.catcoc_get_kernel(ct, dt)
        assert not so.catcoc_get_kernel(ct, 0)
        assert not so.catcoc_get_kernel(ct, L.INT8)
    assert not so.catcoc_get_kernel(7, L.FP16)
    names = {(L.MATMUL_ALLREDUCE, L.FP16): "catcoc_launch_matmul_allreduce_fp16",
             (L.ALLGATHER_MATMUL, L.BF16): "catcoc_launch_allgather_matmul_bf16",
             (L.MATMUL_REDUCE_SCATTER, L.BF16): "catcoc_launch_matmul_reduce_scatter_bf16"}
    for (ct, dt), nm in names.items():
        assert so.catcoc_get_kernel(ct, dt) == C.cast(getattr(so, nm), C.c_void_p).value


def test_host_schedulers_equal_oracle(so):
    m, n, k, s = u32(), u32(), u32(), u32()
    for off, d, lm, ln in [(7, 1, 8, 16), (7, 1, 4, 16), (7, 0, 16, 4), (3, 0, 11, 3), (3, 1, 11, 9), (1, 0, 3, 2),
                           (2, 1, 5, 5), (4, 0, 1, 1), (7, 1, 1, 32)]:
        for t in range(2 * lm * ln):
            so.catcoc_swizzle_block_coord(off, d, lm, ln, t, C.byref(m), C.byref(n))
            assert (m.value, n.value) == oracle.swizzle_block_coord(off, d, lm, ln, t)
    for off, d, lm, ln, kt, f in [(7, 1, 1, 32, 32, 8), (3, 0, 4, 32, 32, 2), (3, 0, 1, 3, 8, 3), (1, 1, 1, 2, 9, 4),
                                  (7, 1, 1, 4, 8, 5)]:
        for t in range(lm * ln * f):
            so.catcoc_splitk_block_coord(off, d, lm, ln, kt, f, t, C.byref(m), C.byref(n), C.byref(k), C.byref(s))
            assert (m.value, n.value, k.value, s.value) == oracle.splitk_block_coord(off, d, lm, ln, kt, f, t)
        for sl in range(f):
            for K in (kt * 256, kt * 256 - 100):
                assert so.catcoc_splitk_actual_k(K, 256, f, sl) == oracle.splitk_actual_k(K, 256, f, sl)
    for off, d, P, ci, lmr, ln in [(7, 1, 8, 1, 4, 4), (7, 1, 8, 3, 4, 4), (7, 1, 2, 2, 6, 3), (3, 0, 4, 2, 5, 4)]:
        for t in range(lmr * P * ln):
            so.catcoc_allgather_block_coord(off, d, P, ci, lmr, ln, t, C.byref(m), C.byref(n))
            assert (m.value, n.value) == oracle.allgather_block_coord(off, d, P, ci, lmr, ln, t)
    for d, P, sr, sc, dl in [(0, 8, 20, 1, 50), (0, 8, 16, 1, 7), (0, 4, 2, 2, 9), (1, 8, 4, 2, 13), (1, 2, 3, 1, 5)]:
        for t in range(dl * P + 5):
            so.catcoc_comm_block_idx(d, P, sr, sc, dl, t, C.byref(m), C.byref(n))
            assert (m.value, n.value) == oracle.comm_block_idx(d, P, sr, sc, dl, t)


def _desc(P, rank=0, **kw):
    return L.make_desc(rank, P, [16] * (P - 1), **kw)


def test_task_tile_equals_oracle_reduce_scatter_and_allreduce(so):
    tr, row, col, ws = u32(), u32(), u32(), u32()
    for (M, N, P, m0, n0, bn, ci, st) in [(8192, 4096, 8, 128, 256, 20, 10, 2), (8192, 4096, 8, 128, 256, 256, 1, 2),
                                          (4096, 4096, 8, 128, 256, 256, 4, 2), (800, 260, 8, 64, 256, 16, 1, 3)]:
        t = L.CocTilingParams(m=M, k=64, n=N, m0=m0, n0=n0, k0=256, commInterval=ci, rankSize=P)
        d = _desc(P, block_num=bn, stages=st)
        cnt = so.catcoc_get_task_count(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d))
        assert cnt == -(-(M // P) // m0) * -(-N // n0) * P
        for task in list(range(0, cnt, max(1, cnt // 97))) + [cnt - 1]:
            assert so.catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr),
                                       C.byref(row), C.byref(col), C.byref(ws))
            o = oracle.rs_task(M, N, P, m0, n0, bn, ci, st, task)
            assert (tr.value, row.value, col.value, ws.value) == (o[0], o[3], o[4], o[5])
        assert not so.catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), cnt, C.byref(tr),
                                       C.byref(row), C.byref(col), C.byref(ws))
    t = L.CocTilingParams(m=512, k=2048, n=1024, m0=128, n0=256, k0=256, commInterval=3, rankSize=2)
    d = _desc(2, block_num=20)
    for task in range(16):
        assert so.catcoc_task_tile(L.MATMUL_ALLREDUCE, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row),
                                   C.byref(col), C.byref(ws))
        mi, ni, w = oracle.ar_task(512, 1024, 128, 256, 20, 3, 2, task)
        assert (row.value, col.value, ws.value) == (mi * 128, ni * 256, w)


def test_workgroup_task_is_a_bijection(so):
    for tasks in (1, 7, 127, 128, 129, 1024, 1000, 2048, 4097):
        for flags in (0, L.FLAG_LINEAR_ORDER):
            got = sorted(so.catcoc_workgroup_task(w, tasks, flags) for w in range(tasks))
            assert got == list(range(tasks))
    # chunks of 16 consecutive tasks share an XCD (workgroup id modulo 8)
    xcd = {}
    for w in range(1024):
        xcd.setdefault(so.catcoc_workgroup_task(w, 1024, 0) // 16, set()).add(w % 8)
    assert all(len(v) == 1 for v in xcd.values())
    # every XCD gets the same number of each rank's 128 tasks
    for r in range(8):
        per = [0] * 8
        for w in range(1024):
            if so.catcoc_workgroup_task(w, 1024, 0) // 128 == r:
                per[w % 8] += 1
        assert per == [16] * 8


def test_launch_order_is_a_bijection_with_kept_tiles_first_or_last(so):
    from mm_rs_with_catlass_amd import ops
    for (M, K, N, P, rank, m0) in [(8192, 1792, 4096, 8, 0, 128), (8192, 1792, 4096, 8, 5, 256), (2048, 256, 1024, 4, 3, 128)]:
        t = ops.default_tiling(M, K, N, P, m0=m0, n0=256, k0=256)
        for ws in (False, True):
            d = L.make_desc(rank, P)
            if ws:
                d.workspace, d.workspaceBytes = 4096, 1 << 40    # never dereferenced on the host
            n = so.catcoc_get_task_count(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d))
            tasks = [so.catcoc_launch_task(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), wg) for wg in range(n)]
            assert sorted(tasks) == list(range(n))
            assert so.catcoc_launch_task(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), n) == 0xffffffff
            tr = u32()
            kept = []
            for task in tasks:
                so.catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), None, None, None)
                kept.append(tr.value == rank)
            nk = sum(kept)
            assert nk == n // P
            # the kept tiles are the first workgroups to be dispatched, up to the permutation inside a block of
            # 128 workgroups that the XCD-aware orders apply
            span = -(-nk // 128) * 128
            assert max(wg for wg in range(n) if kept[wg]) < span


def test_launch_tile_equals_launch_task_then_task_tile(so):
    # the kernels work out workgroup -> task and tile through per-launch constants and reciprocal multiplies; the
    # result has to be what the plain integer route gives, for every workgroup, operator, swizzle and round layout
    from mm_rs_with_catlass_amd import ops
    cases = [(L.QUANT_MATMUL_REDUCE_SCATTER, 8192, 1792, 4096, 8, 0, 128, {}),
             (L.QUANT_MATMUL_REDUCE_SCATTER, 8192, 1792, 4096, 8, 5, 256, {}),
             (L.QUANT_MATMUL_REDUCE_SCATTER, 4096, 512, 2048, 4, 3, 128, dict(block_num=20, stages=3, swizzle=(3, 0))),
             (L.QUANT_MATMUL_REDUCE_SCATTER, 6144, 256, 1280, 2, 1, 128, dict(block_num=6, swizzle=(5, 1))),
             (L.QUANT_MATMUL_REDUCE_SCATTER, 2048, 256, 1024, 1, 0, 128, {}),
             (L.MATMUL_REDUCE_SCATTER, 4096, 1792, 4096, 8, 7, 128, {}),
             (L.MATMUL_ALLREDUCE, 2048, 1024, 2048, 2, 0, 128, dict(block_num=20, stages=2, swizzle=(2, 1))),
             (L.MATMUL_ALLREDUCE, 512, 1024, 1024, 2, 1, 128, {}),
             (L.ALLGATHER_MATMUL, 512, 4096, 1024, 8, 2, 128, {})]
    task, tr, row, col, wsr = (u32() for _ in range(5))
    tr2, row2, col2, wsr2 = (u32() for _ in range(4))
    for comm, M, K, N, P, rank, m0, kw in cases:
        t = ops.default_tiling(M, K, N, P, m0=m0, n0=256, k0=256)
        d = L.make_desc(rank, P, **kw)
        n = so.catcoc_get_task_count(comm, C.byref(t), C.byref(d))
        assert n > 0, L.last_error()
        seen = set()
        for wg in range(n):
            assert so.catcoc_launch_tile(comm, C.byref(t), C.byref(d), wg, C.byref(task), C.byref(tr), C.byref(row), C.byref(col), C.byref(wsr)) == 1
            assert task.value == so.catcoc_launch_task(comm, C.byref(t), C.byref(d), wg), (comm, M, N, P, wg)
            assert so.catcoc_task_tile(comm, C.byref(t), C.byref(d), task.value, C.byref(tr2), C.byref(row2), C.byref(col2), C.byref(wsr2)) == 1
            assert (tr.value, row.value, col.value, wsr.value) == (tr2.value, row2.value, col2.value, wsr2.value), (comm, M, N, P, wg)
            seen.add(task.value)
        assert len(seen) == n
        assert so.catcoc_launch_tile(comm, C.byref(t), C.byref(d), n, None, None, None, None, None) == 0


def test_launch_tile_random_shapes(so):
    # the same comparison over random grids, rank counts, swizzles and round layouts (sampled workgroups)
    from mm_rs_with_catlass_amd import ops
    rng = np.random.default_rng(11)
    task, tr, row, col, wsr = (u32() for _ in range(5))
    tr2, row2, col2, wsr2 = (u32() for _ in range(4))
    done = 0
    for _ in range(60):
        P = int(rng.choice([1, 2, 4, 8]))
        comm = int(rng.choice([L.QUANT_MATMUL_REDUCE_SCATTER, L.MATMUL_REDUCE_SCATTER, L.MATMUL_ALLREDUCE]))
        m0 = int(rng.choice([128, 256]))
        rows_per_rank = m0 * int(rng.integers(1, 9))
        M = rows_per_rank * (P if comm != L.MATMUL_ALLREDUCE else 1)
        N = 256 * int(rng.integers(1, 12))
        kw = dict(block_num=int(rng.choice([0, 4, 8, 20])) * P, stages=int(rng.integers(0, 4)),
                  swizzle=(int(rng.integers(1, 9)), int(rng.integers(0, 2))))
        t = ops.default_tiling(M, 512, N, P, m0=m0, n0=256, k0=256, commInterval=int(rng.integers(1, 4)))
        d = L.make_desc(int(rng.integers(0, P)), P, **kw)
        n = so.catcoc_get_task_count(comm, C.byref(t), C.byref(d))
        if n == 0:
            continue        # a layout the library rejects (it says why); nothing to compare
        for wg in sorted(set(int(x) for x in rng.integers(0, n, 40)) | {0, n - 1}):
            assert so.catcoc_launch_tile(comm, C.byref(t), C.byref(d), wg, C.byref(task), C.byref(tr), C.byref(row), C.byref(col), C.byref(wsr)) == 1
            assert task.value == so.catcoc_launch_task(comm, C.byref(t), C.byref(d), wg)
            assert so.catcoc_task_tile(comm, C.byref(t), C.byref(d), task.value, C.byref(tr2), C.byref(row2), C.byref(col2), C.byref(wsr2)) == 1
            assert (tr.value, row.value, col.value, wsr.value) == (tr2.value, row2.value, col2.value, wsr2.value), (comm, M, N, P, m0, kw, wg)
        done += 1
    assert done >= 30


def test_reciprocal_division_is_exact():
    # the formula of the schedulers' FastDiv (m = floor(2^32 / d), estimate mulhi(n, m), two corrections)
    rng = np.random.default_rng(3)
    ds = np.concatenate([np.arange(1, 300), rng.integers(1, 2 ** 32, 300), [2 ** 31, 2 ** 32 - 1, 65535, 65536, 65537]]).astype(np.uint64)
    ns = np.concatenate([np.arange(0, 300), rng.integers(0, 2 ** 32, 500), [2 ** 32 - 1, 2 ** 31, 2 ** 31 - 1]]).astype(np.uint64)
    for d in ds:
        m = min((1 << 32) // int(d), 0xffffffff)
        q = (ns * np.uint64(m)) >> np.uint64(32)
        r = ns - q * d
        for _ in range(2):
            up = r >= d
            q = q + up
            r = r - up * d
        assert np.array_equal(q, ns // d) and np.array_equal(r, ns % d), int(d)


def test_splitk_launch_order_is_a_permutation_that_groups_b_readers(so):
    import ctypes as C
    for loopsM, loopsN, f in [(1, 64, 4), (4, 64, 1), (2, 16, 3), (1, 8, 1), (3, 24, 2), (1, 3, 4), (2, 5, 1)]:
        total = loopsM * loopsN * f
        tasks = [so.catcoc_splitk_launch_task(7, 1, loopsM, loopsN, f, wg) for wg in range(total)]
        assert sorted(tasks) == list(range(total))
        assert so.catcoc_splitk_launch_task(7, 1, loopsM, loopsN, f, total + 5) == total + 5
        if (loopsN * f) % 8 or loopsM < 2:
            assert tasks == list(range(total))      # the order does not apply: identity
            continue
        m, n, k, sl = (C.c_uint32() for _ in range(4))
        where = {}
        for wg, task in enumerate(tasks):
            so.catcoc_splitk_block_coord(7, 1, loopsM, loopsN, 32, f, task, C.byref(m), C.byref(n), C.byref(k), C.byref(sl))
            where.setdefault((n.value, sl.value), []).append(wg)
        for wgs in where.values():
            # the loopsM row tiles that stream one (column tile, k slice) of B sit on one XCD, dispatched back to back
            assert len(wgs) == loopsM and len({w % 8 for w in wgs}) == 1
            assert max(wgs) - min(wgs) == 8 * (loopsM - 1)


def test_workspace_size_queries(so):
    from mm_rs_with_catlass_amd import ops
    import torch
    # k slices of few-tile launches: fill the CUs once, at least eight k steps per slice, two slices at most for floats
    assert ops.kslice_plan(L.ALLGATHER_MATMUL, torch.bfloat16, 512, 4096, 1024, 0, 8) == (128 * 2 * 131072 + 65536, 2)
    assert ops.kslice_plan(L.MATMUL_ALLREDUCE, torch.float16, 512, 1024, 1024, 0, 2) == (16 * 2 * 131072 + 65536, 2)
    assert ops.kslice_plan(L.QUANT_MATMUL_REDUCE_SCATTER, torch.int8, 8192, 1792, 4096, 0, 8) == (0, 1)       # 1024 tiles
    assert ops.kslice_plan(L.QUANT_MATMUL_REDUCE_SCATTER, torch.int8, 1024, 4096, 1024, 0, 8) == (32 * 8 * 131072 + 65536, 8)
    assert ops.kslice_plan(L.QUANT_MATMUL_REDUCE_SCATTER, torch.int8, 1024, 4096, 1024, 0, 8, split_k=2)[1] == 2
    assert ops.kslice_plan(L.QUANT_MATMUL_REDUCE_SCATTER, torch.int8, 1024 + 8, 4096, 1024, 0, 8) == (0, 1)   # ragged rows
    # the caller's own count: up to eight for floats too (three or more partials are added in slice order)
    assert ops.kslice_plan(L.MATMUL_ALLREDUCE, torch.float16, 512, 1024, 1024, 0, 2, split_k=4) == (16 * 4 * 131072 + 65536, 4)
    with pytest.raises(L.CatcocError, match="at most 8 k slices"):
        ops.kslice_plan(L.MATMUL_ALLREDUCE, torch.float16, 512, 1024, 1024, 0, 2, split_k=16)
    # explicit kept rows on a shape outside the streaming kernels (k not in 64-byte steps): whole tiles, no workspace
    assert ops.splitk_plan(40, 100, 200, 4, 5, 20) == (0, 1, 2)
    need, f, tiles = ops.splitk_plan(16, 8192, 8192, 8, 0, 2)
    assert (f, tiles) == (oracle.splitk_factor(16, 8192, 8192, 256, 128, 128, 256), 64)
    assert need == f * tiles * 128 * 128 * 4 + 65536    # counter block of a fixed size first, then the partial tiles
    # from 256 rows on (full tiles, kept rows in whole 32-row blocks): 128x256 tiles, k slices that fill the CUs once
    assert ops.splitk_plan(512, 8192, 8192, 8, 0, 64) == (65536 + 128 * 2 * 131072, 2, 256)
    assert ops.splitk_plan(256, 8192, 8192, 8, 0, 32) == (65536 + 64 * 4 * 131072, 4, 128)
    assert ops.splitk_plan(256, 8192, 8192, 8, 0, 32, n0=128)[1:] == (oracle.splitk_factor(256, 8192, 8192, 256, 128, 128, 256), 128)
    assert ops.splitk_plan(128, 8192, 8192, 4, 0, 32)[0] != 65536 + 32 * 8 * 131072     # below that the split-K kernel, unless asked
    assert ops.splitk_plan(512, 8192, 8192, 8, 0, 64, n0=128) == (0, 1, 256)        # on request: the 128x128 split-K kernel
    assert ops.splitk_plan(512, 8192, 8192, 8, 0, 60)[1:] == (1, 256)               # kept rows not in 32-row blocks: split-K kernel
    assert ops.splitk_plan(1024, 8192, 8192, 8, 0, 128) == (0, 1, 512)              # many rows: 256 tiles of 128x256, no slices
    assert ops.splitk_plan(1024, 8192, 8192, 8, 0, 128, n0=128)[1:] == (1, 512)
    assert ops.splitk_plan(128, 8192, 8192, 8, 0, 32, n0=256) == (65536 + 32 * 8 * 131072, 8, 64)
    assert ops.splitk_plan(128, 8192, 8192, 8, 0, 16)[1:] == (oracle.splitk_factor(128, 8192, 8192, 256, 128, 128, 256), 64)
    assert ops.splitk_plan(2048, 8192, 8192, 8, 8, 64)[1:] == (1, 1024)             # kept rows off the 32-row grid: split-K kernel
    with pytest.raises(L.CatcocError, match="128x256 tiles with explicit kept rows"):
        ops.splitk_plan(128, 8192, 8192, 8, 0, 16, n0=256)
    need, f, tiles = ops.splitk_plan(200, 1088, 256, 4, 100, 50, split_k=3)
    assert (f, tiles) == (3, 4) and need == 3 * 4 * 65536 + 65536
    with pytest.raises(L.CatcocError, match="kept rows"):
        ops.splitk_plan(16, 8192, 8192, 8, 10, 7)


def test_tiling_search_equals_oracle(so):
    for ct, octx in ((L.MATMUL_ALLREDUCE, oracle.MATMUL_ALLREDUCE), (L.ALLGATHER_MATMUL, oracle.ALLGATHER_MATMUL),
                     (L.MATMUL_REDUCE_SCATTER, oracle.MATMUL_REDUCE_SCATTER)):
        for P in (2, 3, 8):
            for (m, k, n) in ((8192, 1792, 4096), (8192, 27392, 4096), (7936, 12544, 6656)):
                base = L.CocTilingParams()
                so.catcoc_default_tiling(C.byref(base), m, k, n, P)
                assert (base.m0, base.k0, base.n0, base.commTileM, base.commInterval, base.commNpuSplit,
                        base.commDataSplit, base.commBlockM) == (128, 256, 256, 64, 20, 1, 2, 64)
                out = (L.CocTilingParams * 64)()
                cnt = so.catcoc_get_tilings(C.byref(base), ct, P, 20, out, 64)
                ob = oracle.TilingParams(*[getattr(base, f[0]) for f in L.CocTilingParams._fields_])
                want = oracle.get_tilings(ob, octx, P, 20)
                assert cnt == len(want)
                for i in range(cnt):
                    for f, _ in L.CocTilingParams._fields_:
                        assert getattr(out[i], f) == getattr(want[i], f)


def test_splitk_factor_equals_oracle(so):
    for (m, n, k, cores) in [(16, 8192, 8192, 20), (16, 8192, 8192, 256), (512, 8192, 8192, 256), (128, 256, 1024, 20),
                             (128, 256, 256, 20), (4096, 4096, 9000, 20), (4096, 4096, 40000, 20), (768, 256, 4096, 20),
                             (1, 8192, 8192, 256), (64, 8192, 8192, 256), (128, 8192, 8192, 256)]:
        assert so.catcoc_get_splitk_factor(m, n, k, cores, 128, 256, 256) == oracle.splitk_factor(m, n, k, cores, 128, 256, 256)


def test_validation_errors(so):
    t = L.CocTilingParams(m=1024, k=256, n=512, rankSize=8, commInterval=1)
    d = _desc(8)
    chk = lambda ct, dt, tt, dd, ta=0, tb=0: so.catcoc_can_implement(ct, dt, C.byref(tt) if tt else None,
                                                                     C.byref(dd) if dd else None, ta, tb)
    assert chk(L.QUANT_MATMUL_REDUCE_SCATTER, L.INT8, t, d) == 0 and L.last_error() == ""
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t, d) == 0
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, None, d) != 0 and "NULL" in L.last_error()
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t, None) != 0
    bad = _desc(8); bad.magic = 0
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t, bad) != 0 and "magic" in L.last_error()
    assert chk(L.MATMUL_REDUCE_SCATTER, L.INT8, t, d) != 0          # int8 is only registered for the quant op
    assert chk(L.QUANT_MATMUL_REDUCE_SCATTER, L.FP16, t, d) != 0
    t2 = L.CocTilingParams(m=1001, k=256, n=512, rankSize=8, commInterval=1)
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t2, d) != 0 and "rankSize" in L.last_error()   # m % P != 0
    t3 = L.CocTilingParams(m=1024, k=256, n=512, rankSize=4, commInterval=1)
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t3, d) != 0          # tiling and descriptor disagree on rankSize
    d3 = _desc(3, block_num=20)
    t4 = L.CocTilingParams(m=3 * 128, k=256, n=512, rankSize=3, commInterval=4)
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t4, d3) != 0 and "multiple of rankSize" in L.last_error()  # 80 % 3
    t4.commInterval = 6
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t4, d3) == 0
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, L.CocTilingParams(m=0, k=1, n=1), d) != 0     # empty problem
    dnp = L.make_desc(0, 8, [16] * 3)
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t, dnp) != 0 and "peers[3]" in L.last_error()   # missing peer
    dr = L.make_desc(9, 8, [16] * 7)
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t, dr) != 0
    dst = L.make_desc(0, 8, [16] * 7, flags=L.OUTBOUND_STORE)
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t, dst) != 0 and "outbound" in L.last_error()
    need = so.catcoc_get_workspace_size(L.MATMUL_REDUCE_SCATTER, L.FP16, C.byref(t), C.byref(dst))
    assert need == 2 * 256 * 128 * 256 * 4
    dst.outbound, dst.outboundBytes = 4096, need - 1
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t, dst) != 0 and "too small" in L.last_error()
    dst.outboundBytes = need
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t, dst) == 0
    dri = L.make_desc(0, 8, [16] * 7, flags=L.FLAG_REDUCE_INT32)
    assert chk(L.MATMUL_REDUCE_SCATTER, L.FP16, t, dri) != 0        # int32 reduce is a W8A8 mode
    assert chk(L.QUANT_MATMUL_REDUCE_SCATTER, L.INT8, t, dri) == 0


def test_rejected_launch_launches_nothing_and_reports(so):
    # a launcher called with a bad descriptor must return without touching the GPU
    t = L.CocTilingParams(m=1024, k=256, n=512, rankSize=8, commInterval=1)
    bad = L.make_desc(0, 8, [16] * 7); bad.magic = 1
    so.catcoc_launch_matmul_reduce_scatter_fp16(None, 0, 16, 16, 16, None, None, C.addressof(bad), C.byref(t), 0, 0)
    assert so.catcoc_last_status() != 0 and "magic" in L.last_error()
    with pytest.raises(L.CatcocError):
        L.check()
    so.catcoc_quant_matmul_reduce_scatter(None, 0, 16, 16, 16, 16, None, None, 16, None, 1024, 512, 256)
    assert so.catcoc_last_status() != 0


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout == ""


def test_python_entry_points_reject_mistyped_or_short_operands():
    # The C ABI sees raw pointers, so element types and sizes are checked by the Python mirror before any launch;
    # every rejection below is raised on host tensors, before the device check and without touching a GPU.
    import torch
    from mm_rs_with_catlass_amd import ops
    M, K, N, P = 1024, 256, 512, 8
    rows = M // P
    x1 = torch.zeros((M, K), dtype=torch.int8)
    x2 = torch.zeros((K, N), dtype=torch.int8)
    s1 = torch.ones(M)
    s2 = torch.ones(N)
    peers = [torch.zeros((rows, N)) for _ in range(P - 1)]
    q = ops.prepare_quant_matmul_reduce_scatter

    def rejects(match, *a, **kw):
        with pytest.raises(L.CatcocError, match=match):
            q(*a, **kw)

    rejects("x1 must be", x1.float(), x2, s1, s2, None, peers, 0, P)
    rejects("scale_x1 must be", x1, x2, s1.half(), s2, None, peers, 0, P)
    rejects("scale_x2 holds", x1, x2, s1, s2[:N - 1], None, peers, 0, P)
    rejects("bias must be", x1, x2, s1, s2, torch.zeros(N), peers, 0, P)
    rejects("k extent", x1, torch.zeros((K + 64, N), dtype=torch.int8), s1, s2, None, peers, 0, P)
    rejects("k extent", x1, x2, s1, s2, None, peers, 0, P, trans_b=True)
    rejects("rank_size - 1", x1, x2, s1, s2, None, peers[:-1], 0, P)
    rejects(r"peers\[6\] has shape", x1, x2, s1, s2, None, peers[:-1] + [torch.zeros((rows - 1, N))], 0, P)
    rejects(r"peers\[0\] has shape", x1, x2, s1, s2, None, peers, 0, P, peer_row_offset=1)
    rejects(r"peers\[2\] must be", x1, x2, s1, s2, None, peers[:2] + [peers[2].int()] + peers[3:], 0, P)
    rejects(r"peers\[0\] must be", x1, x2, s1, s2, None, peers, 0, P, reduce_int32=True)
    rejects("m % rank_size", x1[:1020], x2, s1, s2, None, peers, 0, P)
    rejects("out of range", x1, x2, s1, s2, None, peers, 8, P)
    rejects("out must have shape", x1, x2, s1, s2, None, peers, 0, P, out=torch.zeros((rows, N - 1), dtype=torch.bfloat16))
    rejects("out must be", x1, x2, s1, s2, None, peers, 0, P, out=torch.zeros((rows, N)))
    rejects("c_accum holds", x1, x2, s1, s2, None, peers, 0, P, c_accum=torch.zeros((rows - 1, N), dtype=torch.int32))
    rejects("acc_dump must be", x1, x2, s1, s2, None, peers, 0, P, acc_dump=torch.zeros((M, N)))
    rejects("checksum holds", x1, x2, s1, s2, None, peers, 0, P, checksum=torch.zeros(15, dtype=torch.int64))   # 16 tasks
    rejects("tiling says", x1, x2, s1, s2, None, peers, 0, P, tiling=ops.default_tiling(M, K, N + 256, P))
    rejects("must live on the GPU", x1, x2, s1, s2, None, peers, 0, P)          # everything else in order: only the device is wrong

    sk = ops.prepare_quant_matmul_splitk
    a1 = torch.zeros((16, 256), dtype=torch.int8)
    b1 = torch.zeros((256, 256), dtype=torch.int8)
    with pytest.raises(L.CatcocError, match="kept rows"):
        sk(a1, b1, torch.ones(16), torch.ones(256), None, [], 1, 10, 7)
    with pytest.raises(L.CatcocError, match=r"peers\[0\] has shape"):
        sk(a1, b1, torch.ones(16), torch.ones(256), None, [torch.zeros((1, 256))], 2, 0, 2)
    with pytest.raises(L.CatcocError, match="checksum holds"):
        sk(a1, b1, torch.ones(16), torch.ones(256), None, [], 1, 0, 2, checksum=torch.zeros(1, dtype=torch.int64))
    with pytest.raises(L.CatcocError, match="scale_x1 holds"):
        sk(a1, b1, torch.ones(15), torch.ones(256), None, [], 1, 0, 2)

    a = torch.zeros((M, K), dtype=torch.float16)
    b = torch.zeros((K, N), dtype=torch.float16)
    with pytest.raises(L.CatcocError, match="both be float16 or both bfloat16"):
        ops.matmul_reduce_scatter(a, b.bfloat16(), peers, 0, P)
    with pytest.raises(L.CatcocError, match=r"peers\[0\] has shape"):
        ops.matmul_allreduce(a, b, [torch.zeros((rows, N))], 0, 2)          # all-reduce peers are full [m,n]
    with pytest.raises(L.CatcocError, match="k extent"):
        ops.matmul_reduce_scatter(a, b, peers, 0, P, trans_a=True)
    with pytest.raises(L.CatcocError, match=r"peer_shards\[0\] has shape"):
        ops.allgather_matmul(a, [torch.zeros((M - 1, K), dtype=torch.float16)], b, 0, 2)
    with pytest.raises(L.CatcocError, match=r"peer_shards\[0\] must be"):
        ops.allgather_matmul(a, [torch.zeros((M, K))], b, 0, 2)
    with pytest.raises(L.CatcocError, match="acc_dump holds"):
        ops.allgather_matmul(a, [a.clone()], b, 0, 2, acc_dump=torch.zeros((M, N)))      # the gathered product has 2M rows
    with pytest.raises(L.CatcocError, match="must live on the GPU"):
        ops.matmul_reduce_scatter(a, b, peers, 0, P)


def test_verify_gate_equals_oracle(so):
    # catcoc_verify is host code of the product (the reference's verify_result.py runs on the host too); it must agree
    # with the oracle's restatement on random data, on the tolerance edges and on NaN / Inf handling
    from mm_rs_with_catlass_amd import ops
    rng = np.random.default_rng(3)
    for dtype, ct in ((L.FP16, 100), (L.FP16, 4096), (L.BF16, 100), (L.BF16, 4096)):
        gold = (rng.standard_normal(5000) * 50).astype(np.float32)
        for noise in (0.0, 1e-3, 5e-3, 2e-2):
            out = (gold * (1 + noise * rng.standard_normal(5000))).astype(np.float32)
            out[::97] = np.nan
            gold2 = gold.copy()
            gold2[5::131] = np.inf
            want = oracle.verify(out, gold2, dtype, ct)
            got = ops.verify(out, gold2, dtype, ct)
            assert got[0] == want[0] and got[1] == want[1] and abs(got[2] - want[2]) <= 1e-12, (dtype, ct, noise)
    # exactly on the element-wise bound passes, one step beyond fails (rtol 2^-8 for fp16, computeTimes < 2048)
    g = np.array([4.0, 0.5], np.float32)
    assert ops.verify(g + np.array([4.0 / 256, 1.0 / 256], np.float32), g, L.FP16, 10)[1] == 0
    over = np.array([np.nextafter(np.float32(4.0 + 4.0 / 256), np.float32(5)), 0.5], np.float32)
    assert ops.verify(over, g, L.FP16, 10)[1] == 1
    # a bias below the element-wise bound still fails the mean test (2^-10 for fp16)
    g = np.full(1000, 2.0, np.float32)
    ok_, bad, eb = ops.verify(g * (1 + 1.0 / 512), g, L.FP16, 10)
    assert bad == 0 and not ok_ and eb > 2.0 ** -10
    with pytest.raises(L.CatcocError):
        ops.verify(g, g, 5, 10)


def test_comm_swizzle_variants_equal_oracle(so):
    d, r = u32(), u32()
    for (P, sr, sc, dl) in [(8, 20, 1, 50), (8, 10, 2, 50), (4, 3, 1, 7), (8, 256, 1, 16), (2, 5, 2, 11)]:
        assert so.catcoc_comm_core_loop(1, P, sr, sc, dl) == oracle.comm_core_loop(True, P, sr, sc, dl)
        assert so.catcoc_comm_core_loop(0, P, sr, sc, dl) == dl * P
        for t in range(oracle.comm_core_loop(True, P, sr, sc, dl) + 5):
            so.catcoc_comm_block_idx_ex(0, 1, P, sr, sc, dl, t, C.byref(d), C.byref(r))
            assert (d.value, r.value) == oracle.comm_block_idx_det(P, sr, sc, dl, t), (P, sr, sc, dl, t)
        if P % sc == 0:
            for t in range(dl * P):
                so.catcoc_comm_block_idx_ex(0, 0, P, sr, sc, dl, t, C.byref(d), C.byref(r))
                assert (d.value, r.value) == oracle.comm_block_idx(0, P, sr, sc, dl, t)


def test_pipelined_entry_points_reject_bad_arguments(so):
    t = L.CocTilingParams(m=1024, k=256, n=512, rankSize=8, commInterval=1, commBlockM=48)
    d = L.make_desc(0, 8, [16] * 7, outbound=4096, outbound_bytes=1 << 40)
    so.catcoc_pipelined_quant_matmul_reduce_scatter(None, None, 0, 16, 16, 16, 16, None, 16, 16, C.addressof(d), C.byref(t), 0, 0, L.BF16, 1)
    assert so.catcoc_last_status() != 0 and "commBlockM" in L.last_error()
    t.commBlockM = 64
    so.catcoc_pipelined_quant_matmul_reduce_scatter(None, None, 0, 16, 16, 16, 16, None, None, 16, C.addressof(d), C.byref(t), 0, 0, L.BF16, 1)
    assert so.catcoc_last_status() != 0 and "c_accum" in L.last_error()
    d2 = L.make_desc(0, 8, [16] * 7)
    so.catcoc_pipelined_matmul_reduce_scatter(None, None, L.FP16, 16, 16, 16, C.addressof(d2), C.byref(t), 0, 0, 1)
    assert so.catcoc_last_status() != 0 and "outbound" in L.last_error()
    so.catcoc_reduce_add(None, 16, 16, 10, 2, 0)
    assert so.catcoc_last_status() != 0 and "multiple of 4" in L.last_error()
    so.catcoc_reduce_add(None, 16, 16, 16, 0, 0)
    assert so.catcoc_last_status() != 0


def test_sweep_csv_has_the_reference_columns_and_best_pick(tmp_path):
    # examples/dynamic_tiling/include/tiling.h:114 header, get_best_res.py:73-83 best row = min Time(us) per (Op, M, K, N)
    import csv
    from mm_rs_with_catlass_amd import tuning
    rows = []
    for i, us in enumerate((90.0, 71.5, 80.0)):
        rows.append({"Op": "QuantMatmulReduceScatter", "M": 8192, "K": 1792, "N": 4096, "Transpose A": 0, "Transpose B": 0, "commInterval": 1 + i,
                     "commTileM": 64, "commBlockM": 64, "commNpuSplit": 1, "commDataSplit": 2, "Time(us)": us, "m0": 128, "swizzleOffset": 7,
                     "swizzleDirection": 1, "linearOrder": 0, "kSlices": 1, "TOPS": 1.0, "peakFraction": 0.1})
    rows.append(dict(rows[0], Op="MatmulReduceScatter", **{"Time(us)": 5.0}))
    path = tmp_path / "result.csv"
    tuning.write_result_csv(str(path), rows)
    with open(path) as f:
        header = f.readline().strip().split(",")
        assert header[:12] == ["Op", "M", "K", "N", "Transpose A", "Transpose B", "commInterval", "commTileM", "commBlockM", "commNpuSplit",
                               "commDataSplit", "Time(us)"]
        assert len(list(csv.reader(f))) == 4
    best = tuning.best_results(rows)
    assert len(best) == 2 and {b["Time(us)"] for b in best} == {71.5, 5.0}
    assert (tuning.WARM_UP_TIMES, tuning.PERF_TEST_CYCLE_TIMES) == (10, 3)      # examples/dynamic_tiling/include/info.h:22-23
    assert (256, (7, 1), False, 1) in tuning.candidates(1024, True) and (256, (3, 0), True, 4) in tuning.candidates(1018, False)
    assert all(c[0] != 256 for c in tuning.candidates(200, False)) and (64, (7, 1), False, 1) in tuning.candidates(64, True)


def test_task_tiles_batch_query_equals_single_queries(so):
    t = L.CocTilingParams(m=8192, k=1792, n=4096, m0=128, n0=256, k0=256, commInterval=10, rankSize=8)
    d = L.make_desc(3, 8, [16] * 7, block_num=20)
    n = so.catcoc_get_task_count(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d))
    arr = [(u32 * n)() for _ in range(4)]
    got = so.catcoc_task_tiles(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), 0, n, *arr)
    assert got == n == 1024
    one = [u32() for _ in range(4)]
    for task in (0, 1, 199, 200, 777, 1023):
        assert so.catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, *[C.byref(x) for x in one])
        assert tuple(a[task] for a in arr) == tuple(x.value for x in one)
        assert tuple(a[task] for a in arr) == (lambda r: (r[0], r[3], r[4], r[5]))(oracle.rs_task(8192, 4096, 8, 128, 256, 20, 10, 2, task))
    assert so.catcoc_task_tiles(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), 1000, 100, None, arr[1], None, None) == 24


def test_kept_split_choice_by_tile_count_and_k_length():
    # which reduce-scatter launches run their kept tiles as two 64-row workgroups (catcoc_kept_split_tiles): fewer than 256
    # tiles, or up to 512 tiles with up to 80 k steps of 64 bytes; whole tiles, A as [m,k], XCD-block order; flags override
    from mm_rs_with_catlass_amd import ops
    so = L.load()

    def split(comm, dt, m, k, n, p, flags=0, ta=0, tb=0, rank=0):
        t = ops.default_tiling(m, k, n, p, m0=0, n0=0, k0=0)
        d = L.make_desc(rank, p, [16] * (p - 1))
        d.flags = flags
        r = so.catcoc_kept_split_tiles(comm, dt, C.byref(t), C.byref(d), ta, tb)
        L.check()
        return r
    Q, RS = L.QUANT_MATMUL_REDUCE_SCATTER, L.MATMUL_REDUCE_SCATTER
    assert split(Q, L.INT8, 8192, 1792, 4096, 8) == 0                 # config 4: 1024 tiles, two rounds
    assert split(Q, L.INT8, 8192, 1792, 4096, 8, L.FLAG_KEPT_SPLIT) == 128
    assert split(Q, L.INT8, 4096, 1792, 4096, 8) == 64                # 512 tiles, 28 k steps
    assert split(Q, L.INT8, 4096, 1792, 4096, 8, tb=1) == 64          # either layout of B
    assert split(Q, L.INT8, 4096, 1792, 4096, 8, ta=1) == 0           # A as [k,m]: whole tiles only
    assert split(Q, L.INT8, 4096, 1792, 4096, 8, L.FLAG_KEPT_WHOLE) == 0
    assert split(Q, L.INT8, 4096, 1792, 4096, 8, L.FLAG_LINEAR_ORDER) == 0
    assert split(Q, L.INT8, 4096, 5120, 4096, 8) == 64                # 80 k steps
    assert split(Q, L.INT8, 4096, 5184, 4096, 8) == 0                 # 81
    assert split(Q, L.INT8, 1024, 7168, 4096, 8) == 16                # 128 tiles: fewer than CUs, any k
    assert split(RS, L.FP16, 4096, 1792, 4096, 8) == 64               # config 3: 512 tiles, 56 k steps
    assert split(RS, L.FP16, 4096, 2592, 4096, 8) == 0                # 81 k steps

    # the tiles by which tasks + kept halves exceed the 512 workgroup slots run as halves too (catcoc_tail_split_tiles); their
    # checksum halves need the counter block of a workspace
    def tail(comm, dt, m, k, n, p, flags=0, checksum=False, workspace=False):
        t = ops.default_tiling(m, k, n, p, m0=0, n0=0, k0=0)
        d = L.make_desc(0, p, [16] * (p - 1))
        d.flags = flags
        if checksum:
            d.checksum = 4096
        if workspace:
            d.workspace, d.workspaceBytes = 4096, 65536
        r = so.catcoc_tail_split_tiles(comm, dt, C.byref(t), C.byref(d), 0, 0)
        L.check()
        return r
    assert tail(Q, L.INT8, 4096, 1792, 4096, 8) == 64                               # 512 + 64 - 512
    assert tail(Q, L.INT8, 4096, 1792, 4096, 8, checksum=True) == 0                 # no workspace for the checksum halves
    assert tail(Q, L.INT8, 4096, 1792, 4096, 8, checksum=True, workspace=True) == 64
    assert tail(Q, L.INT8, 4096, 1792, 4096, 8, L.FLAG_TAIL_WHOLE) == 0
    assert tail(Q, L.INT8, 4096, 1792, 4096, 8, L.FLAG_KEPT_WHOLE) == 0
    assert tail(Q, L.INT8, 3072, 1792, 4096, 8) == 0                                # 384 + 48 workgroups fit
    assert tail(Q, L.INT8, 4096, 1792, 3584, 8) == 0                                # 448 + 56 workgroups fit
    assert tail(Q, L.INT8, 8192, 1792, 4096, 8) == 0                                # no split kept tiles, no tail
    assert tail(RS, L.FP16, 4096, 1792, 4096, 8, checksum=True, workspace=True) == 64
    assert split(RS, L.FP16, 8 * 296, 512, 1344, 8) == 0              # ragged problems keep whole tiles
    assert split(L.MATMUL_ALLREDUCE, L.FP16, 1024, 512, 1024, 2) == 0 # no kept-rank block to split
    assert split(Q, L.INT8, 4096, 1792, 4096, 1) == 0                 # no peers to stream
