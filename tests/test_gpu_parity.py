"""GPU parity tests: the HIP library, called through its C ABI, against the CPU oracle on the same
seeded inputs.  Bars: int32 accumulators bit-exact; W8A8 outputs within 1 ulp of the 16-bit output
type (the build reduces in the oracle's order, so they are normally equal); float GEMMs within
rel-err 1e-2 of the fp32 k-sequential oracle and inside the reference's own rtol gate."""
import os

import numpy as np
import pytest
import torch

import oracle
from mm_rs_with_catlass_amd import lib as L
from mm_rs_with_catlass_amd import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _need_gpu():
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    L.load()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def dev16(bits, dtype):
    """uint16 bit patterns -> fp16 / bf16 tensor on the GPU."""
    t = torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(DEV)
    return t.view(torch.float16 if dtype == oracle.FP16 else torch.bfloat16)


def host16(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def ulp_diff16(a_bits, b_bits):
    """Distance in units of last place between two arrays of fp16/bf16 bit patterns."""
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


TORCH_DT = {oracle.FP16: torch.float16, oracle.BF16: torch.bfloat16}


def _report_ulp(what, ulp, share=0.999):
    """Float outputs: the share of elements within 1 ulp of the oracle's (blocked fp32 accumulation differs from the oracle's
    k-sequential one) must exceed `share`; the figures are printed so that a drift shows in the log before it fails."""
    within = float((ulp <= 1).mean())
    print("%s: %.5f of %d elements within 1 ulp, worst %d ulp" % (what, within, ulp.size, int(ulp.max())))
    assert within > share, "%s: only %.5f within 1 ulp (worst %d)" % (what, within, int(ulp.max()))


def quant_case(rng, M, N, K, P, rank, *, bias=False, out_dtype=oracle.BF16, trans_b=False, trans_a=False, reduce_int32=False,
               full_peers=False, tiling=None, outbound=False, block_num=0, stages=0, swizzle=None, linear=False,
               launches=1, kslices=None):
    _need_gpu()
    x1 = rng.integers(-127, 128, (M, K), dtype=np.int8)
    x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s1 = rng.uniform(0.005, 0.02, M).astype(np.float32)
    s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.integers(-1000, 1000, N, dtype=np.int32) if bias else None
    rows = M // P
    prow0 = rank * rows if full_peers else 0
    prow = M if full_peers else rows
    if reduce_int32:
        peers = [rng.integers(-2 ** 24, 2 ** 24, (prow, N), dtype=np.int32) for _ in range(P - 1)]
    else:
        peers = [rng.standard_normal((prow, N)).astype(np.float32) for _ in range(P - 1)]
    acc_want, out_want = oracle.quant_matmul_reduce_scatter(
        x1, x2, s1, s2, b, rank * rows, rows, peers, out_dtype, peer_row0=prow0, reduce_int32=reduce_int32)

    x2d = dev(np.ascontiguousarray(x2.T)) if trans_b else dev(x2)
    x1d = dev(np.ascontiguousarray(x1.T)) if trans_a else dev(x1)
    acc_dump = torch.full((M, N), -7, dtype=torch.int32, device=DEV)
    c_accum = torch.full((rows, N), -7, dtype=torch.int32, device=DEV)
    dpeers = [dev(p) for p in peers]
    import ctypes as C
    kw = {}
    ob = None
    t = tiling if tiling is not None else ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
    d = L.make_desc(rank, P, [16] * (P - 1), block_num=block_num, stages=stages, swizzle=swizzle)
    ntasks = L.load().catcoc_get_task_count(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d))
    if outbound:
        need = L.load().catcoc_get_workspace_size(L.QUANT_MATMUL_REDUCE_SCATTER, L.INT8, C.byref(t), C.byref(d))
        ob = torch.zeros(need // 4, dtype=torch.int32 if reduce_int32 else torch.float32, device=DEV)
        kw["outbound"] = ob
    checksum = torch.zeros(ntasks, dtype=torch.int64, device=DEV)
    if not outbound:
        kw["checksum"] = checksum
    ws = None
    if kslices is not None:      # (forced count or 0 = the library's choice, count expected)
        need, f = ops.kslice_plan(L.QUANT_MATMUL_REDUCE_SCATTER, torch.int8, M, K, N, rank, P, tiling=tiling, split_k=kslices[0])
        assert f == kslices[1]
        assert need == (ntasks * f * 128 * 256 * 4 + 65536 if f > 1 else 0)
        if f > 1:
            ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
            kw["workspace"] = ws
        kw["split_k"] = kslices[0]
    for it in range(launches):
        out = ops.quant_matmul_reduce_scatter(
            x1d, x2d, dev(s1), dev(s2), dev(b) if bias else None, dpeers, rank, P, out_dtype=TORCH_DT[out_dtype],
            tiling=tiling, trans_b=trans_b, trans_a=trans_a, peer_row_offset=prow0, reduce_int32=reduce_int32, acc_dump=acc_dump,
            c_accum=c_accum, block_num=block_num, stages=stages, swizzle=swizzle, linear_order=linear, **kw)
        torch.cuda.synchronize()
        if it + 1 < launches:
            out.zero_()
    if ws is not None:
        assert not ws[:65536].any(), "tile counters were not re-armed"
    acc_got = acc_dump.cpu().numpy()
    assert np.array_equal(acc_got, acc_want), "int32 accumulators differ from the oracle"
    kept = acc_want[rank * rows:(rank + 1) * rows]
    if reduce_int32:
        kept = kept + sum(p[prow0:prow0 + rows] for p in peers)
    assert np.array_equal(c_accum.cpu().numpy(), kept)
    got = host16(out)
    d_ulp = ulp_diff16(got, out_want)
    assert d_ulp.max() <= 1, "output differs by %d ulp" % d_ulp.max()
    return dict(x1=x1, x2=x2, s1=s1, s2=s2, bias=b, acc=acc_want, out=got, out_want=out_want, checksum=checksum,
                outbound=ob, ntasks=ntasks, exact=int((d_ulp == 0).sum()), total=d_ulp.size)


# ------------------------------------------------------------------- W8A8 path
@pytest.mark.parametrize("rank", [0, 3, 7])
def test_quant_rs_full_tiles_bit_exact(rank):
    r = quant_case(np.random.default_rng(100 + rank), 2048, 512, 256, 8, rank)
    assert r["exact"] == r["total"]          # same reduce order as the oracle: equality, not just 1 ulp


def test_quant_rs_bias_fp16_out_and_full_size_peers():
    quant_case(np.random.default_rng(1), 1024, 768, 320, 8, 5, bias=True, out_dtype=oracle.FP16, full_peers=True)


def test_quant_rs_reference_order_int32_reduce():
    quant_case(np.random.default_rng(2), 1024, 512, 192, 4, 1, bias=True, reduce_int32=True)


def test_quant_rs_transposed_b():
    quant_case(np.random.default_rng(3), 1024, 512, 256, 8, 2, trans_b=True)


@pytest.mark.parametrize("case", [(4096, 1024, 1792, 8, 3, None), (2048, 2048, 320, 2, 1, None), (1024, 1024, 2048, 4, 1, (0, 4)),
                                  (1024, 512, 1024, 2, 0, (3, 3))])
def test_quant_rs_weights_stored_n_by_k(case):
    # B given as [n,k] (the usual layout of a weight matrix): full tiles run the direct-to-LDS kernel, which then
    # stages B like A and needs no transposing reads; also cut into k slices; everything stays bit-exact
    M, N, K, P, rank, ks = case
    r = quant_case(np.random.default_rng(80 + rank), M, N, K, P, rank, bias=True, trans_b=True, launches=2, kslices=ks)
    assert r["exact"] == r["total"]


@pytest.mark.parametrize("shape", [(800, 260, 208), (8 * 130, 516, 80), (64, 256, 16), (8, 4, 16)])
def test_quant_rs_ragged_edges(shape):
    M, N, K = shape
    quant_case(np.random.default_rng(4), M, N, K, 8, 6, bias=True)


@pytest.mark.parametrize("case", [(8 * 296, 1344, 512, 8, 6, False), (8 * 296, 1280, 192, 8, 0, True), (4 * 1064, 1088, 128, 4, 3, False),
                                  (2 * 1024, 2112, 256, 2, 1, True)])
def test_quant_rs_ragged_problem_on_many_tiles(case):
    # ragged rows and/or columns with 64 or more full tiles: two launches over one launch order, the direct-to-LDS
    # kernel on the full tiles and the bounds-checked kernel on the ragged ones; every tile's accumulators, the kept
    # block, the checksums and the outbound tiles must come out as from one launch
    import ctypes as C
    M, N, K, P, rank, outbound = case
    stages = 0      # (every case is a single round of at most 256 tasks: no workspace stage is reused)
    r = quant_case(np.random.default_rng(90 + rank), M, N, K, P, rank, bias=True, launches=2, outbound=outbound, stages=stages)
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
    d = L.make_desc(rank, P, [16] * (P - 1), stages=stages)
    so = L.load()
    tr, row, col, ws = (C.c_uint32() for _ in range(4))
    rows = M // P
    seen_ragged = seen_full = 0
    deq = oracle.dequant(r["acc"], r["s2"], r["s1"]) if outbound else None
    ob = r["outbound"].cpu().numpy().reshape(-1, 256) if outbound else None
    cs = r["checksum"].cpu().numpy()
    for task in range(r["ntasks"]):
        so.catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row), C.byref(col), C.byref(ws))
        rv = min(128, (tr.value + 1) * rows - row.value)
        cv = min(256, N - col.value)
        seen_ragged += rv < 128 or cv < 256
        seen_full += rv == 128 and cv == 256
        if tr.value == rank:
            continue
        blk = r["acc"][row.value:row.value + rv, col.value:col.value + cv]
        if outbound:
            want = deq[row.value:row.value + rv, col.value:col.value + cv]
            assert np.array_equal(ob[ws.value:ws.value + rv, :cv].view(np.uint32), want.view(np.uint32)), task
        else:
            assert cs[task] == int(blk.astype(np.int64).sum()), task
    assert seen_ragged > 0 and seen_full >= 64 and r["ntasks"] <= 256


# (M, N, K, P, rank, weights as [n,k], outbound tiles instead of checksums)
@pytest.mark.parametrize("case", [(8 * 296, 1344, 512, 8, 6, False, False), (8 * 296, 1280, 256, 8, 0, True, True),
                                  (4 * 1064, 1088, 128, 4, 3, True, False), (2 * 1000, 2120, 384, 2, 1, False, True),
                                  (8 * 300, 520, 1024, 8, 7, True, False)])
def test_quant_rs_ragged_problem_on_256_row_tiles(case):
    """Ragged rows and / or columns on 256x256 tiles (m0 = 256): edge tiles are computed as whole tiles moved up / left until
    they end at the edge, on the direct-to-LDS kernel in both layouts of B.  Accumulators of every element, the kept
    block, and every other tile's own part through its checksum or its outbound tile."""
    import ctypes as C
    M, N, K, P, rank, tb, outbound = case
    t = ops.default_tiling(M, K, N, P, m0=256, n0=256, k0=256, commInterval=1)
    r = quant_case(np.random.default_rng(95 + rank), M, N, K, P, rank, bias=True, tiling=t, trans_b=tb, outbound=outbound, stages=4)
    d = L.make_desc(rank, P, [16] * (P - 1), stages=4)
    so = L.load()
    tr, row, col, ws = (C.c_uint32() for _ in range(4))
    rows = M // P
    seen_ragged = 0
    deq = oracle.dequant(r["acc"], r["s2"], r["s1"]) if outbound else None
    ob = r["outbound"].cpu().numpy().reshape(-1, 256) if outbound else None
    cs = r["checksum"].cpu().numpy()
    for task in range(r["ntasks"]):
        so.catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row), C.byref(col), C.byref(ws))
        rv = min(256, (tr.value + 1) * rows - row.value)
        cv = min(256, N - col.value)
        seen_ragged += rv < 256 or cv < 256
        if tr.value == rank:
            continue
        blk = r["acc"][row.value:row.value + rv, col.value:col.value + cv]
        if outbound:
            want = deq[row.value:row.value + rv, col.value:col.value + cv]
            assert np.array_equal(ob[ws.value:ws.value + rv, :cv].view(np.uint32), want.view(np.uint32)), task
        else:
            assert cs[task] == int(blk.astype(np.int64).sum()), task
    assert seen_ragged > 0


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
@pytest.mark.parametrize("tb", [False, True])
def test_float_ragged_problems_on_256_row_tiles(dtype, tb):
    # reduce-scatter with ragged rows and columns and all-reduce with ragged rows on 256x256 tiles, both layouts of B
    _need_gpu()
    rng = np.random.default_rng(27)
    M, N, K, P, rank = 8 * 296, 1344, 448, 8, 5
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.02)
    rows = M // P
    peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
    part, want = oracle.matmul_reduce(A, B, dtype, rank * rows, rows, peers, want_partial=True)
    dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    t = ops.default_tiling(M, K, N, P, m0=256, n0=256, k0=256)
    Bd = dev16(np.ascontiguousarray(B.T) if tb else B, dtype)
    out = ops.matmul_reduce_scatter(dev16(A, dtype), Bd, [dev(p) for p in peers], rank, P, tiling=t, trans_b=tb, acc_dump=dump)
    L.check()
    torch.cuda.synchronize()
    _check_float(host16(out), want, part[rank * rows:(rank + 1) * rows] + sum(peers), dtype, K)
    assert np.abs(dump.cpu().numpy() - part).max() <= 1e-2 * max(1.0, np.abs(part).max())
    M, N, K = 1100, 2048, 320
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.02)
    p1 = rng.standard_normal((M, N)).astype(np.float32)
    part, want = oracle.matmul_reduce(A, B, dtype, 0, M, [p1], want_partial=True)
    t = ops.default_tiling(M, K, N, 2, m0=256, n0=256, k0=256)
    out = ops.matmul_allreduce(dev16(A, dtype), dev16(np.ascontiguousarray(B.T) if tb else B, dtype), [dev(p1)], 0, 2, tiling=t, trans_b=tb)
    L.check()
    torch.cuda.synchronize()
    _check_float(host16(out), want, part + p1, dtype, K)


@pytest.mark.parametrize("tb", [False, True])
def test_quant_rs_kept_tiles_whole_or_split_give_the_same_bits(tb):
    # CATCOC_FLAG_KEPT_WHOLE / CATCOC_FLAG_KEPT_SPLIT are tuning knobs: output, kept accumulators and checksums must not change
    _need_gpu()
    import ctypes as C
    M, N, K, P, rank = 8192, 1024, 448, 8, 5          # 256 tiles; also forced on 1024 tiles below
    for (M, N) in ((8192, 1024), (8192, 4096)):
        g = torch.Generator(device=DEV).manual_seed(11)
        x1 = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=DEV, generator=g)
        x2 = torch.randint(-127, 128, (N, K) if tb else (K, N), dtype=torch.int8, device=DEV, generator=g)
        s1 = torch.empty(M, device=DEV).uniform_(0.005, 0.02, generator=g)
        s2 = torch.empty(N, device=DEV).uniform_(0.001, 0.01, generator=g)
        peers = [torch.randn((M // P, N), device=DEV, generator=g) for _ in range(P - 1)]
        t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
        d = L.make_desc(rank, P, [16] * (P - 1))
        ntasks = L.load().catcoc_get_task_count(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d))
        res = []
        for ks in (False, True, None):
            cs = torch.zeros(ntasks, dtype=torch.int64, device=DEV)
            ca = torch.zeros((M // P, N), dtype=torch.int32, device=DEV)
            out = ops.quant_matmul_reduce_scatter(x1, x2, s1, s2, None, peers, rank, P, trans_b=tb, checksum=cs, c_accum=ca, kept_split=ks)
            torch.cuda.synchronize()
            res.append((out.view(torch.int16).clone(), cs, ca))
        for r in res[1:]:
            assert torch.equal(res[0][0], r[0]) and torch.equal(res[0][1], r[1]) and torch.equal(res[0][2], r[2])
        assert int(res[0][1].ne(0).sum()) >= ntasks * 7 // 8 - 2


@pytest.mark.parametrize("kind", ["int8", "fp16"])
def test_rs_tiles_that_wait_for_kept_halves_run_as_halves(kind):
    """512 tiles with split kept tiles are 576 workgroups on 512 slots; with a workspace (the checksum halves of a task meet
    through its counter block) the 64 tiles that wait run as two 64-row workgroups.  Outputs and per-task checksums equal those
    of the launch with whole tiles bit for bit, the counter block is clean again, and without a workspace the launch falls back."""
    _need_gpu()
    import ctypes as C
    M, N, K, P, rank = 4096, 4096, 320, 8, 5
    g = torch.Generator(device=DEV).manual_seed(77)
    rows = M // P
    peers = [torch.randn((rows, N), device=DEV, generator=g) for _ in range(P - 1)]
    if kind == "int8":
        x1 = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=DEV, generator=g)
        x2 = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=DEV, generator=g)
        s1 = torch.empty(M, device=DEV).uniform_(0.005, 0.02, generator=g)
        s2 = torch.empty(N, device=DEV).uniform_(0.001, 0.01, generator=g)
        comm, dt, csdt = L.QUANT_MATMUL_REDUCE_SCATTER, L.INT8, torch.int64
        run = lambda **kw: ops.quant_matmul_reduce_scatter(x1, x2, s1, s2, None, peers, rank, P, **kw)
    else:
        A = torch.randn((M, K), device=DEV, generator=g).half()
        B = (torch.randn((K, N), device=DEV, generator=g) * 0.02).half()
        comm, dt, csdt = L.MATMUL_REDUCE_SCATTER, L.FP16, torch.float64
        run = lambda **kw: ops.matmul_reduce_scatter(A, B, peers, rank, P, **kw)
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
    d = L.make_desc(rank, P, [16] * (P - 1))
    d.checksum, d.workspace, d.workspaceBytes = 4096, 4096, 65536
    so = L.load()
    assert so.catcoc_kept_split_tiles(comm, dt, C.byref(t), C.byref(d), 0, 0) == 64
    assert so.catcoc_tail_split_tiles(comm, dt, C.byref(t), C.byref(d), 0, 0) == 64
    res = {}
    for name, kw in (("whole", dict(kept_split=False)), ("kept halves", dict(kept_split="kept-only")), ("kept and waiting halves", dict()),
                     ("no workspace", dict(workspace=None))):
        cs = torch.full((512,), -1, dtype=csdt, device=DEV)
        ws = torch.zeros(65536, dtype=torch.uint8, device=DEV)
        kw.setdefault("workspace", ws)
        for _ in range(2):   # (the second launch finds the counter block as the first left it)
            out = run(checksum=cs, **kw)
        torch.cuda.synchronize()
        assert not ws.any(), name
        res[name] = (host16(out), cs.cpu().numpy())
    for name in res:
        assert np.array_equal(res[name][0], res["whole"][0]), name
        assert np.array_equal(res[name][1], res["whole"][1]), name
    # and the outbound mode: halves store their own rows of the workspace tile
    need = so.catcoc_get_workspace_size(comm, dt, C.byref(t), C.byref(d))
    obs = []
    for kw in (dict(kept_split=False), dict()):
        ob = torch.zeros(need // 4, dtype=torch.float32, device=DEV)
        run(outbound=ob, **kw)
        torch.cuda.synchronize()
        obs.append(ob.cpu().numpy())
    assert np.array_equal(obs[0].view(np.uint32), obs[1].view(np.uint32))


@pytest.mark.parametrize("shape", [(32, 129, 100), (24, 7, 3), (4 * 23, 45, 68), (4, 128, 512)])
def test_quant_rs_general_shapes(shape):
    # K not a multiple of 16 or N not a multiple of 4: the general kernel (incl. the reference's own
    # quant test shape 4x128x512 and the 23/45/68 sizes its issue list names)
    M, N, K = shape
    quant_case(np.random.default_rng(5), M, N, K, 4, 3, bias=True)


def test_quant_rs_m0_64_and_reference_launch_geometry():
    t = ops.default_tiling(2048, 256, 1024, 8, m0=64, n0=256, k0=256, commInterval=10)
    quant_case(np.random.default_rng(6), 2048, 1024, 256, 8, 4, tiling=t, block_num=20, stages=2)
    t = ops.default_tiling(2048, 256, 1024, 8, m0=128, n0=256, k0=256, commInterval=2)
    quant_case(np.random.default_rng(7), 2048, 1024, 256, 8, 4, tiling=t, block_num=4, swizzle=(3, 0), linear=True)


@pytest.mark.parametrize("rank", [0, 6])
def test_quant_rs_m0_256_eight_wave_tile(rank):
    t = ops.default_tiling(4096, 512, 1024, 8, m0=256, n0=256, k0=256, commInterval=1)
    r = quant_case(np.random.default_rng(30 + rank), 4096, 1024, 512, 8, rank, tiling=t, bias=True)
    assert r["exact"] == r["total"]
    t = ops.default_tiling(2048, 128, 512, 4, m0=256, n0=256, k0=256, commInterval=1)
    quant_case(np.random.default_rng(32), 2048, 512, 128, 4, 1, tiling=t, outbound=True, stages=4)
    # k not a multiple of 128: m0 = 256 falls back to the general kernel, same results
    t = ops.default_tiling(2048, 448, 512, 8, m0=256, n0=256, k0=256, commInterval=1)
    quant_case(np.random.default_rng(33), 2048, 512, 448, 8, rank, tiling=t)


# (M, N, K, P, rank): k of one pair of steps, of two, three (an odd number of pairs), four and many; one and several tiles per rank
@pytest.mark.parametrize("case", [(2048, 512, 128, 8, 0), (2048, 256, 256, 4, 3), (4096, 1024, 384, 8, 6), (2048, 512, 512, 2, 1),
                                  (4096, 1024, 1920, 8, 5), (2048, 768, 8192, 8, 7)])
def test_quant_rs_m0_256_weights_stored_n_by_k(case):
    """The 256x256 tile with B as [n,k]: both operands in pair buffers of whole cache lines (two of A, three of B), copies
    at even steps only.  Accumulators of every tile bit for bit, kept rows against the oracle, the other ranks' tiles
    through their checksums; then the int32 reduce order, bias and outbound tiles on the same route."""
    M, N, K, P, rank = case
    t = ops.default_tiling(M, K, N, P, m0=256, n0=256, k0=256, commInterval=1)
    r = quant_case(np.random.default_rng(40 + K), M, N, K, P, rank, tiling=t, trans_b=True, bias=(K % 256 == 0))
    assert r["exact"] == r["total"]
    if K == 1920:
        quant_case(np.random.default_rng(41), M, N, K, P, rank, tiling=t, trans_b=True, reduce_int32=True, outbound=True, stages=4)


@pytest.mark.parametrize("case", [(8192, 1024, 512, 8, 0), (8192, 1024, 512, 8, 5), (4096, 2048, 128, 4, 3),
                                  (4096, 2048, 1792, 8, 7), (8192, 1024, 3584, 2, 1)])
def test_quant_rs_many_tiles_two_launches(case):
    # 256 tiles and more: every XCD walks its own block of the tile grid, kept rows first; the second launch
    # must rewrite the zeroed output
    M, N, K, P, rank = case
    quant_case(np.random.default_rng(40 + rank), M, N, K, P, rank, bias=True, launches=2)


@pytest.mark.parametrize("case", [(1024, 1024, 4096, 4, 1, (0, 8)), (1024, 1024, 2048, 4, 3, (0, 4)), (2048, 512, 1792, 8, 7, (0, 2)),
                                  (1024, 512, 1024, 2, 0, (3, 3)), (2048, 1024, 576, 8, 3, (0, 1)), (1024, 768, 64, 4, 2, (1, 1))])
def test_quant_rs_few_tiles_k_sliced(case):
    # fewer tiles than CUs: with a workspace every tile's k range is cut into slices that meet through memory;
    # int32 partials add exactly, so everything stays bit-exact, and the second launch finds the counters re-armed
    M, N, K, P, rank, ks = case
    r = quant_case(np.random.default_rng(70 + rank), M, N, K, P, rank, bias=True, launches=2, kslices=ks)
    cs = r["checksum"].cpu().numpy()
    rows = M // P
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
    d = L.make_desc(rank, P, [16] * (P - 1))
    import ctypes as C
    tr, row, col = C.c_uint32(), C.c_uint32(), C.c_uint32()
    for task in range(r["ntasks"]):
        L.load().catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row), C.byref(col), None)
        if tr.value != rank:
            blk = r["acc"][row.value:row.value + 128, col.value:col.value + 256].astype(np.int64)
            assert cs[task] == blk.sum(), task


def test_one_workspace_shared_by_launches_of_different_shapes():
    # The arrival counters sit in a block of fixed size at the start of the workspace, so a workspace zeroed once serves
    # launches of different tile counts and slice counts, k-sliced large tiles and skinny-M split-K alike, in any order.
    _need_gpu()
    rng = np.random.default_rng(77)
    ws = torch.zeros(96 << 20, dtype=torch.uint8, device=DEV)

    def ksliced(M, N, K, P, rank):
        x1 = rng.integers(-127, 128, (M, K), dtype=np.int8)
        x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
        s1 = rng.uniform(0.005, 0.02, M).astype(np.float32)
        s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
        rows = M // P
        peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
        _, want = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, None, rank * rows, rows, peers, oracle.BF16, want_acc=False)
        need, f = ops.kslice_plan(L.QUANT_MATMUL_REDUCE_SCATTER, torch.int8, M, K, N, rank, P)
        assert f > 1 and need <= ws.numel()
        out = ops.quant_matmul_reduce_scatter(dev(x1), dev(x2), dev(s1), dev(s2), None, [dev(p) for p in peers], rank, P, workspace=ws)
        torch.cuda.synchronize()
        assert np.array_equal(host16(out), want), (M, N, K)
        return f

    def skinny(M, N, K, P, kr):
        x1 = rng.integers(-127, 128, (M, K), dtype=np.int8)
        x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
        s1 = rng.uniform(0.005, 0.02, M).astype(np.float32)
        s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
        peers = [rng.standard_normal((kr, N)).astype(np.float32) for _ in range(P - 1)]
        _, want = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, None, 0, kr, peers, oracle.BF16, want_acc=False)
        need, f, tiles = ops.splitk_plan(M, K, N, P, 0, kr)
        assert f > 1 and need <= ws.numel()
        out = ops.quant_matmul_splitk(dev(x1), dev(x2), dev(s1), dev(s2), None, [dev(p) for p in peers], P, 0, kr, workspace=ws)
        torch.cuda.synchronize()
        assert np.array_equal(host16(out), want), (M, N, K)
        return f

    fs = [ksliced(1024, 1024, 4096, 4, 1),      # 32 tiles x 8 slices
          skinny(16, 1024, 4096, 8, 2),         # 8 tiles of 128x128, split-K
          ksliced(2048, 512, 1792, 8, 7),       # 32 tiles x 2 slices: counters where the first launch had partials
          skinny(64, 2048, 2048, 4, 16),
          ksliced(1024, 1024, 4096, 4, 2)]
    assert fs[0] == 8 and fs[2] == 2
    assert not ws[:65536].any(), "tile counters were not re-armed"


def test_quant_rs_few_tiles_k_sliced_outbound_store():
    # the sliced launch with the other ranks' tiles stored (not just summed): the last slice writes the fp32 tile
    M, N, K, P, rank = 1024, 512, 2048, 4, 2
    r = quant_case(np.random.default_rng(77), M, N, K, P, rank, bias=True, outbound=True, launches=2, kslices=(0, 4))
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
    d = L.make_desc(rank, P, [16] * (P - 1))
    import ctypes as C
    tr, row, col, wsr = (C.c_uint32() for _ in range(4))
    ob = r["outbound"].cpu().numpy().reshape(-1, 256)
    deq = oracle.dequant(r["acc"], r["s2"], r["s1"])
    for task in range(r["ntasks"]):
        L.load().catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row), C.byref(col), C.byref(wsr))
        if tr.value == rank:
            continue
        want = deq[row.value:row.value + 128, col.value:col.value + 256]
        assert np.array_equal(ob[wsr.value:wsr.value + 128].view(np.uint32), want.view(np.uint32)), task


def test_k_slice_rejections():
    _need_gpu()
    a = torch.zeros((512, 1024), dtype=torch.float16, device=DEV)
    b = torch.zeros((1024, 1024), dtype=torch.float16, device=DEV)
    with pytest.raises(L.CatcocError, match="at most 8 k slices"):
        ops.matmul_allreduce(a, b, [], 0, 1, split_k=16, workspace=torch.zeros(1 << 24, dtype=torch.uint8, device=DEV))
    with pytest.raises(L.CatcocError, match="needs a workspace"):
        ops.matmul_allreduce(a, b, [], 0, 1, split_k=2)
    with pytest.raises(L.CatcocError, match="workspace too small"):
        ops.matmul_allreduce(a, b, [], 0, 1, workspace=torch.zeros(4096, dtype=torch.uint8, device=DEV))


@pytest.mark.parametrize("case", [(1, 512, 1024, 8, 0, 1, 0), (16, 512, 2048, 8, 0, 2, 0), (16, 384, 1024, 8, 6, 10, 4),
                                  (64, 256, 4096, 8, 8, 8, 0), (128, 640, 2048, 8, 112, 16, 0), (200, 256, 1088, 4, 100, 50, 3),
                                  (33, 128, 64, 2, 0, 33, 0), (512, 1024, 1024, 8, 0, 64, 2), (64, 256, 2048, 4, 0, 16, 8),
                                  (48, 384, 1536, 1, 0, 48, 6), (256, 256, 320, 2, 128, 128, 0),
                                  # many rows with kept rows in whole 32-row blocks: 128x256 tiles, epilogue per 32-row block
                                  (512, 512, 512, 4, 96, 160, 0), (384, 768, 1024, 8, 352, 32, 4), (512, 1024, 2048, 8, 448, 64, 0),
                                  (512, 512, 512, 4, 100, 160, 0)])    # the same off the 32-row grid: split-K kernel
def test_quant_skinny_m_splitk(case):
    # decode shapes: any m, explicit kept rows, k slices meet through the workspace; int32 sums are exact
    _need_gpu()
    M, N, K, P, kb, kr, f = case
    rng = np.random.default_rng(60 + M)
    x1 = rng.integers(-127, 128, (M, K), dtype=np.int8)
    x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s1 = rng.uniform(0.005, 0.02, M).astype(np.float32)
    s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.integers(-1000, 1000, N, dtype=np.int32)
    peers = [rng.standard_normal((kr, N)).astype(np.float32) for _ in range(P - 1)]
    acc_want, out_want = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, b, kb, kr, peers, oracle.BF16)
    need, fac, tiles = ops.splitk_plan(M, K, N, P, kb, kr, split_k=f)
    assert tiles == -(-M // 128) * (N // 128) and fac >= 1 and (f == 0 or fac == min(f, -(-K // 256)))
    ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=DEV)
    acc_dump = torch.full((M, N), -7, dtype=torch.int32, device=DEV)
    c_accum = torch.full((kr, N), -7, dtype=torch.int32, device=DEV)
    checksum = torch.zeros(tiles, dtype=torch.int64, device=DEV)
    n0 = 256 if (M % 128 == 0 and N % 256 == 0 and kb % 32 == 0 and kr % 32 == 0 and M >= 256) else 0   # exercise the large-tile route
    if n0:
        need, fac, tiles = ops.splitk_plan(M, K, N, P, kb, kr, split_k=f, n0=n0)
        ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=DEV)
    launch, out = ops.prepare_quant_matmul_splitk(dev(x1), dev(x2), dev(s1), dev(s2), dev(b), [dev(p) for p in peers], P,
                                                  kb, kr, split_k=f, workspace=ws, checksum=checksum, acc_dump=acc_dump,
                                                  c_accum=c_accum, n0=n0)
    for it in range(2):                      # the second launch reuses the workspace the first one re-armed
        out.zero_()
        launch()
        L.check()
        torch.cuda.synchronize()
        assert np.array_equal(acc_dump.cpu().numpy(), acc_want), "int32 accumulators differ from the oracle"
        assert np.array_equal(c_accum.cpu().numpy(), acc_want[kb:kb + kr])
        assert np.array_equal(host16(out), out_want), "kept rows differ from the oracle"
    cs = checksum.cpu().numpy()
    keep = np.zeros(M, bool)
    keep[kb:kb + kr] = True
    for t in range(tiles):
        mi, ni = divmod(t, N // 128)
        blk = acc_want[mi * 128:(mi + 1) * 128, ni * 128:(ni + 1) * 128].astype(np.int64)
        assert cs[t] == blk[~keep[mi * 128:(mi + 1) * 128]].sum(), t


@pytest.mark.parametrize("case", [(1, 8192, 8192, 8, 0, 1), (16, 8192, 8192, 8, 0, 2), (128, 8192, 8192, 8, 16, 16), (64, 1024, 4160, 4, 40, 24),
                                  (512, 8192, 8192, 8, 64, 64), (100, 384, 1088, 2, 3, 90)])
@pytest.mark.parametrize("mode", ["weights_n_by_k", "int32_reduce", "both"])
def test_quant_skinny_m_weight_layout_and_reference_reduce_order(case, mode):
    """The decode path in the layouts and modes the reference uses: B stored as [n,k] (transB, the layout of its sweep shapes,
    examples/dynamic_tiling/scripts/test_shapes.csv, and of a weight matrix) and int32 peers that join the accumulators before
    the dequantisation (quant_matmul_reduce_scatter.hpp:285-351), at K = N = 8192 for M = 1, 16, 128 and 512 (the large-tile
    route) and on odd shapes.  Accumulators, reduced int32 block and output bit for bit against the oracle."""
    _need_gpu()
    M, N, K, P, kb, kr = case
    tb, ri = mode != "int32_reduce", mode != "weights_n_by_k"
    rng = np.random.default_rng(260 + M)
    x1 = rng.integers(-127, 128, (M, K), dtype=np.int8)
    x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s1 = rng.uniform(0.005, 0.02, M).astype(np.float32)
    s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.integers(-1000, 1000, N, dtype=np.int32)
    if ri:
        peers = [rng.integers(-2 ** 24, 2 ** 24, (kr, N), dtype=np.int32) for _ in range(P - 1)]
    else:
        peers = [rng.standard_normal((kr, N)).astype(np.float32) for _ in range(P - 1)]
    acc_k, out_want = oracle.quant_matmul_reduce_scatter(x1[kb:kb + kr], x2, s1[kb:kb + kr], s2, b, 0, kr, peers, oracle.BF16, reduce_int32=ri)
    need, fac, tiles = ops.splitk_plan(M, K, N, P, kb, kr)
    ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=DEV)
    c_accum = torch.full((kr, N), -7, dtype=torch.int32, device=DEV)
    x2d = dev(np.ascontiguousarray(x2.T)) if tb else dev(x2)
    launch, out = ops.prepare_quant_matmul_splitk(dev(x1), x2d, dev(s1), dev(s2), dev(b), [dev(p) for p in peers], P, kb, kr,
                                                  workspace=ws, c_accum=c_accum, trans_b=tb, reduce_int32=ri)
    for it in range(2):
        out.zero_()
        launch()
        L.check()
        torch.cuda.synchronize()
        kept = acc_k + (sum(peers) if ri else 0)
        assert np.array_equal(c_accum.cpu().numpy(), kept), "kept int32 block differs from the oracle"
        assert np.array_equal(host16(out), out_want), "kept rows differ from the oracle"
    assert not ws[:65536].any()


# (M, N, K, P, kept_begin, kept_rows, peer_row_offset, fp16 output, bias, int32 peers)
@pytest.mark.parametrize("case", [(1, 128, 128, 1, 0, 1, 0, False, False, False), (1, 8192, 8192, 8, 0, 1, 0, False, True, False),
                                  (8, 256, 384, 8, 5, 3, 0, False, True, True), (9, 1024, 1152, 16, 0, 9, 2, True, True, False),
                                  (16, 8192, 8192, 8, 14, 2, 0, False, True, False), (17, 640, 2048, 4, 7, 10, 0, True, False, True),
                                  (24, 384, 640, 16, 20, 4, 1, False, True, False), (32, 8192, 8192, 8, 0, 32, 0, False, True, True),
                                  (31, 128, 256, 2, 30, 1, 0, True, True, False), (32, 4096, 512, 9, 8, 16, 0, False, False, True),
                                  (33, 128, 256, 2, 31, 2, 0, False, True, False), (64, 8192, 8192, 8, 8, 8, 0, False, True, False),
                                  (100, 640, 1152, 4, 20, 70, 3, True, True, True), (128, 8192, 8192, 8, 112, 16, 0, False, True, False),
                                  (128, 256, 512, 16, 0, 128, 0, False, False, True), (96, 384, 384, 3, 60, 36, 0, True, True, False),
                                  (65, 128, 128, 1, 64, 1, 0, False, True, False)])
def test_quant_decode_rows_against_stored_weights(case):
    """B stored as [n,k].  At most 32 rows: a workgroup owns 32 columns over the whole k range (no k slices, no workspace),
    its four waves deal the 128-byte chunks of k round-robin and start the walk at a place of their own.  One to 32 rows
    (every A-copy width), k of one chunk, of fewer chunks than waves have stages and of many, one to sixteen ranks (more
    than one batch of eight peers), kept rows at the start, in the middle and at the end of the block, peers read at a row
    offset, fp16 and bf16 output, with and without bias, fp32 peers and int32 peers.  33 to 128 rows: the same options on
    the split-K kernel (with its workspace), kept rows across 32-row blocks and a last block of one row.  The accumulators
    of every row, the kept int32 block and the output bit for bit against the oracle, twice in a row."""
    _need_gpu()
    M, N, K, P, kb, kr, pro, f16, has_bias, ri = case
    rng = np.random.default_rng(460 + M + K)
    x1 = rng.integers(-127, 128, (M, K), dtype=np.int8)
    x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s1 = rng.uniform(0.005, 0.02, M).astype(np.float32)
    s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.integers(-1000, 1000, N, dtype=np.int32) if has_bias else None
    peers = [rng.integers(-2 ** 24, 2 ** 24, (kr, N), dtype=np.int32) if ri else rng.standard_normal((kr, N)).astype(np.float32)
             for _ in range(P - 1)]
    acc_want, out_want = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, b, kb, kr, peers, oracle.FP16 if f16 else oracle.BF16,
                                                            reduce_int32=ri)
    # peers as the launch sees them: `pro` rows of filler in front of the rows that line up with the kept ones
    staged = [np.concatenate([np.full((pro, N), 77, p.dtype), p]) for p in peers]
    acc_dump = torch.full((M, N), -7, dtype=torch.int32, device=DEV)
    c_accum = torch.full((kr, N), -7, dtype=torch.int32, device=DEV)
    ws = None
    if M > 32:
        need, fac, tiles = ops.splitk_plan(M, K, N, P, kb, kr)
        ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=DEV)
    launch, out = ops.prepare_quant_matmul_splitk(dev(x1), dev(np.ascontiguousarray(x2.T)), dev(s1), dev(s2), dev(b) if has_bias else None,
                                                  [dev(p) for p in staged], P, kb, kr, out_dtype=torch.float16 if f16 else torch.bfloat16,
                                                  acc_dump=acc_dump, c_accum=c_accum, peer_row_offset=pro, trans_b=True, reduce_int32=ri,
                                                  workspace=ws)
    for it in range(2):
        out.zero_()
        launch()
        L.check()
        torch.cuda.synchronize()
        assert np.array_equal(acc_dump.cpu().numpy(), acc_want), "int32 accumulators differ from the oracle"
        assert np.array_equal(c_accum.cpu().numpy(), acc_want[kb:kb + kr] + (sum(peers) if ri else 0)), "kept int32 block differs"
        assert np.array_equal(host16(out), out_want), "kept rows differ from the oracle"


@pytest.mark.parametrize("case", [(40, 200, 100, 4, 5, 20, False, False), (130, 264, 192, 2, 100, 30, True, False), (17, 128, 72, 8, 0, 17, False, True),
                                  (260, 136, 1000, 4, 120, 140, True, True)])
def test_quant_explicit_kept_rows_on_odd_shapes(case):
    # k that is not whole 64-byte steps or n that is not whole 128-column tiles: the explicit-kept-rows launch runs the
    # one-thread-per-element kernel on the same 128x128 grid (kept rows need not line up with tiles); everything it writes
    # against the oracle: accumulators, kept int32 block, output, checksums of the rows that are not kept
    _need_gpu()
    M, N, K, P, kb, kr, tb, ri = case
    rng = np.random.default_rng(360 + M)
    x1 = rng.integers(-127, 128, (M, K), dtype=np.int8)
    x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s1 = rng.uniform(0.005, 0.02, M).astype(np.float32)
    s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.integers(-1000, 1000, N, dtype=np.int32)
    peers = [rng.integers(-2 ** 24, 2 ** 24, (kr, N), dtype=np.int32) if ri else rng.standard_normal((kr, N)).astype(np.float32) for _ in range(P - 1)]
    acc_want, out_want = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, b, kb, kr, peers, oracle.BF16, reduce_int32=ri)
    need, fac, tiles = ops.splitk_plan(M, K, N, P, kb, kr)
    assert need == 0 and fac == 1 and tiles == -(-M // 128) * -(-N // 128)
    acc_dump = torch.full((M, N), -7, dtype=torch.int32, device=DEV)
    c_accum = torch.full((kr, N), -7, dtype=torch.int32, device=DEV)
    checksum = torch.zeros(tiles, dtype=torch.int64, device=DEV)
    x2d = dev(np.ascontiguousarray(x2.T)) if tb else dev(x2)
    out = ops.quant_matmul_splitk(dev(x1), x2d, dev(s1), dev(s2), dev(b), [dev(p) for p in peers], P, kb, kr, checksum=checksum,
                                  acc_dump=acc_dump, c_accum=c_accum, trans_b=tb, reduce_int32=ri)
    torch.cuda.synchronize()
    assert np.array_equal(acc_dump.cpu().numpy(), acc_want)
    assert np.array_equal(c_accum.cpu().numpy(), acc_want[kb:kb + kr] + (sum(peers) if ri else 0))
    assert np.array_equal(host16(out), out_want)
    cs = checksum.cpu().numpy()
    keep = np.zeros(M, bool)
    keep[kb:kb + kr] = True
    nt = -(-N // 128)
    for t in range(tiles):
        mi, ni = divmod(t, nt)
        blk = acc_want[mi * 128:(mi + 1) * 128, ni * 128:(ni + 1) * 128].astype(np.int64)
        assert cs[t] == blk[~keep[mi * 128:(mi + 1) * 128]].sum(), t
    with pytest.raises(L.CatcocError, match="runs whole tiles on the general kernel"):
        ops.quant_matmul_splitk(dev(x1), x2d, dev(s1), dev(s2), dev(b), [dev(p) for p in peers], P, kb, kr, trans_b=tb, reduce_int32=ri,
                                split_k=2, workspace=torch.zeros(1 << 20, dtype=torch.uint8, device=DEV))


@pytest.mark.parametrize("case", [(64, 256, 4096, 8, 8, 8, 0), (128, 640, 2048, 8, 112, 16, 0), (200, 256, 1088, 4, 100, 50, 3),
                                  (100, 384, 1024, 8, 37, 13, 4), (256, 256, 2048, 2, 130, 60, 2), (33, 128, 512, 2, 0, 33, 2),
                                  (128, 256, 1024, 1, 0, 128, 4), (190, 128, 768, 8, 0, 5, 3)])
def test_quant_skinny_m_splitk_checksums_without_dump(case):
    """Checksums without a dump of the accumulators: the k slices then hand over only the groups of eight rows that hold kept
    rows, and every lane's sum of what it holds of the other groups.  Kept ranges that start and end inside a group, rows
    of A that end inside a group, every row kept, k slices of an odd number of steps: the checksum of every tile equals the
    oracle's sum over the rows that are not kept, the kept rows its output, on two launches through one workspace."""
    _need_gpu()
    M, N, K, P, kb, kr, f = case
    rng = np.random.default_rng(160 + M)
    x1 = rng.integers(-127, 128, (M, K), dtype=np.int8)
    x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s1 = rng.uniform(0.005, 0.02, M).astype(np.float32)
    s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.integers(-1000, 1000, N, dtype=np.int32)
    peers = [rng.standard_normal((kr, N)).astype(np.float32) for _ in range(P - 1)]
    acc_want, out_want = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, b, kb, kr, peers, oracle.BF16)
    need, fac, tiles = ops.splitk_plan(M, K, N, P, kb, kr, split_k=f, n0=128)
    ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=DEV)
    checksum = torch.zeros(tiles, dtype=torch.int64, device=DEV)
    launch, out = ops.prepare_quant_matmul_splitk(dev(x1), dev(x2), dev(s1), dev(s2), dev(b), [dev(p) for p in peers], P,
                                                  kb, kr, split_k=f, workspace=ws, checksum=checksum, n0=128)
    keep = np.zeros(M, bool)
    keep[kb:kb + kr] = True
    for it in range(2):
        out.zero_()
        checksum.fill_(-1)
        launch()
        L.check()
        torch.cuda.synchronize()
        assert np.array_equal(host16(out), out_want), "kept rows differ from the oracle"
        cs = checksum.cpu().numpy()
        for t in range(tiles):
            mi, ni = divmod(t, N // 128)
            blk = acc_want[mi * 128:(mi + 1) * 128, ni * 128:(ni + 1) * 128].astype(np.int64)
            assert cs[t] == blk[~keep[mi * 128:(mi + 1) * 128]].sum(), (it, t)


def test_quant_skinny_m_rejections():
    _need_gpu()
    s1 = torch.ones(16, device=DEV)
    s2 = torch.ones(256, device=DEV)
    x1 = torch.zeros((16, 2048), dtype=torch.int8, device=DEV)
    x2 = torch.zeros((2048, 256), dtype=torch.int8, device=DEV)
    with pytest.raises(L.CatcocError, match="workspace"):
        ops.quant_matmul_splitk(x1, x2, s1, s2, None, [], 1, 0, 2, split_k=4)
    with pytest.raises(L.CatcocError, match="kept rows"):
        ops.quant_matmul_splitk(x1, x2, s1, s2, None, [], 1, 10, 7, split_k=1)


def test_quant_rs_checksum_and_outbound_tiles():
    import ctypes as C
    M, N, K, P, rank = 2048, 512, 128, 8, 2
    r = quant_case(np.random.default_rng(8), M, N, K, P, rank)
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
    d = L.make_desc(rank, P, [16] * (P - 1))
    so = L.load()
    tr, row, col, ws = (C.c_uint32() for _ in range(4))
    cs = r["checksum"].cpu().numpy()
    m0 = 128
    for task in range(r["ntasks"]):
        so.catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row),
                            C.byref(col), C.byref(ws))
        want = 0 if tr.value == rank else int(r["acc"][row.value:row.value + m0, col.value:col.value + 256].astype(np.int64).sum())
        assert cs[task] == want, task
    # outbound store: every non-kept tile lands at its tile-linear workspace row, dequantised in fp32
    stages = 4  # enough stages that no round overwrites another
    r = quant_case(np.random.default_rng(8), M, N, K, P, rank, outbound=True, stages=stages)
    d = L.make_desc(rank, P, [16] * (P - 1), stages=stages)
    ob = r["outbound"].cpu().numpy().reshape(-1, 256)
    deq = oracle.dequant(r["acc"], r["s2"], r["s1"])
    for task in range(r["ntasks"]):
        so.catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row),
                            C.byref(col), C.byref(ws))
        if tr.value == rank:
            continue
        want = deq[row.value:row.value + m0, col.value:col.value + 256]
        assert np.array_equal(ob[ws.value:ws.value + m0].view(np.uint32), want.view(np.uint32)), task


def test_quant_checksum_with_most_negative_operands_and_long_k():
    # int8 admits -128: accumulators reach 128*128*k, and the checksum's 32-bit partial sums must still hold them
    _need_gpu()
    M, N, K, P, rank = 256, 256, 32704, 2, 1
    x1 = torch.full((M, K), -128, dtype=torch.int8, device=DEV)
    x2 = torch.full((K, N), -128, dtype=torch.int8, device=DEV)
    s1 = torch.full((M,), 2.0 ** -20, device=DEV)
    s2 = torch.full((N,), 2.0 ** -10, device=DEV)
    peers = [torch.zeros((M // P, N), device=DEV)]
    cs = torch.zeros(2, dtype=torch.int64, device=DEV)
    dump = torch.zeros((M, N), dtype=torch.int32, device=DEV)
    out = ops.quant_matmul_reduce_scatter(x1, x2, s1, s2, None, peers, rank, P, checksum=cs, acc_dump=dump)
    torch.cuda.synchronize()
    acc = 128 * 128 * K
    assert acc < 2 ** 31 and 4 * acc < 2 ** 31
    assert torch.all(dump == acc)
    assert sorted(cs.tolist()) == [0, 128 * 256 * acc]
    want = torch.tensor(float(acc) * 2.0 ** -30).to(torch.bfloat16)     # power-of-two scales: only the final cast rounds
    assert torch.all(out == want.to(DEV))

def test_quant_fixed_config_entry_point():
    # catcoc_quant_matmul_reduce_scatter: the example's signature (m, n, k by value, bf16 out, tile 128x256,
    # commInterval 10); the 256-slot schedule needs 2560 % P == 0
    import ctypes as C
    _need_gpu()
    rng = np.random.default_rng(9)
    M, N, K, P, rank = 1024, 512, 128, 8, 1
    x1 = rng.integers(-16, 16, (M, K), dtype=np.int8)       # the reference's own input range
    x2 = rng.integers(-16, 16, (K, N), dtype=np.int8)
    s1 = (rng.standard_normal(M) * 0.01).astype(np.float32)  # can be negative, as in gen_quant_data.py:37-38
    s2 = (rng.standard_normal(N) * 0.01).astype(np.float32)
    bias = np.ones(N, np.int32)
    rows = M // P
    peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
    _, want = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, bias, rank * rows, rows, peers, oracle.BF16)
    dp = [dev(p) for p in peers]
    d = L.make_desc(rank, P, [p.data_ptr() for p in dp], peer_ld=N)
    out = torch.zeros((rows, N), dtype=torch.bfloat16, device=DEV)
    tx1, tx2, ts1, ts2, tb = dev(x1), dev(x2), dev(s1), dev(s2), dev(bias)
    L.load().catcoc_quant_matmul_reduce_scatter(
        torch.cuda.current_stream().cuda_stream, 0, tx1.data_ptr(), tx2.data_ptr(), ts1.data_ptr(), ts2.data_ptr(),
        tb.data_ptr(), None, out.data_ptr(), C.addressof(d), M, N, K)
    L.check()
    torch.cuda.synchronize()
    assert ulp_diff16(host16(out), want).max() <= 1


def test_quant_debug_mode_closed_form_on_gpu():
    # examples/utils/gen_quant_data.py debug data: ones, scales 0.01, bias 1..N; P identical partials
    _need_gpu()
    M, N, K, P = 1024, 256, 128, 8
    rows = M // P
    x1 = torch.ones((M, K), dtype=torch.int8, device=DEV)
    x2 = torch.ones((K, N), dtype=torch.int8, device=DEV)
    s1 = torch.full((M,), 0.01, dtype=torch.float32, device=DEV)
    s2 = torch.full((N,), 0.01, dtype=torch.float32, device=DEV)
    bias = torch.arange(1, N + 1, dtype=torch.int32, device=DEV)
    part = ((K + bias.float()) * 0.01 * 0.01).expand(rows, N).contiguous()
    out = ops.quant_matmul_reduce_scatter(x1, x2, s1, s2, bias, [part] * (P - 1), 0, P, out_dtype=torch.float16)
    torch.cuda.synchronize()
    want = P * (K + np.arange(1, N + 1)) * 1e-4
    assert np.allclose(out.float().cpu().numpy(), np.broadcast_to(want, (rows, N)), rtol=2 ** -9, atol=0)


# ------------------------------------------------------------------ float paths
def _rand16(rng, shape, dtype, scale=1.0, uniform=False):
    x = rng.uniform(-1, 1, shape) if uniform else rng.standard_normal(shape) * scale
    return oracle.f32_to_half(x.astype(np.float32), dtype)


def _check_float(got_bits, want_bits, partial_f32, dtype, K):
    got = oracle.half_to_f32(got_bits, dtype)
    want = oracle.half_to_f32(want_bits, dtype)
    err = np.abs(got - want) / np.maximum(1.0, np.abs(want))
    assert err.max() <= 1e-2, "rel err %g" % err.max()      # the stated tolerance for fp32-accumulate float GEMMs
    ok, bad, eb = oracle.verify(got, partial_f32, dtype, K)  # the reference's own gate, against unrounded fp32
    assert ok, (bad, eb)


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
@pytest.mark.parametrize("shape", [(1024, 512, 256, 8, 3), (800, 260, 208, 8, 7), (24, 7, 30, 4, 1)])
def test_float_reduce_scatter(dtype, shape):
    _need_gpu()
    M, N, K, P, rank = shape
    rng = np.random.default_rng(20)
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.02)
    rows = M // P
    peers = [rng.standard_normal((M, N)).astype(np.float32) for _ in range(P - 1)]   # full size, rows of the block read
    part, want = oracle.matmul_reduce(A, B, dtype, rank * rows, rows, peers, peer_row0=rank * rows, want_partial=True)
    dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    out = ops.matmul_reduce_scatter(dev16(A, dtype), dev16(B, dtype), [dev(p) for p in peers], rank, P,
                                    peer_row_offset=rank * rows, acc_dump=dump)
    torch.cuda.synchronize()
    full = part[rank * rows:(rank + 1) * rows] + sum(p[rank * rows:(rank + 1) * rows] for p in peers)
    _check_float(host16(out), want, full, dtype, K)
    pd = dump.cpu().numpy()
    assert np.abs(pd - part).max() <= 1e-2 * max(1.0, np.abs(part).max())


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
def test_float_single_round_launch_splits_kept_tiles(dtype):
    # at most 512 tiles and short k: every kept tile runs as two 64-row workgroups (a second tile body inside the kernel);
    # kept block, accumulators of every tile, checksums of the other ranks' tiles
    _need_gpu()
    import ctypes as C
    M, N, K, P, rank = 4096, 2048, 640, 8, 3          # 256 tiles, 20 k steps
    rng = np.random.default_rng(28)
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.02)
    rows = M // P
    peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
    part, want = oracle.matmul_reduce(A, B, dtype, rank * rows, rows, peers, want_partial=True)
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
    d = L.make_desc(rank, P, [16] * (P - 1))
    so = L.load()
    ntasks = so.catcoc_get_task_count(L.MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d))
    cs = torch.zeros(ntasks, dtype=torch.float64, device=DEV)
    dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    for _ in range(2):
        out = ops.matmul_reduce_scatter(dev16(A, dtype), dev16(B, dtype), [dev(p) for p in peers], rank, P, checksum=cs, acc_dump=dump)
        torch.cuda.synchronize()
    _check_float(host16(out), want, part[rank * rows:(rank + 1) * rows] + sum(peers), dtype, K)
    assert np.abs(dump.cpu().numpy() - part).max() <= 1e-2 * max(1.0, np.abs(part).max())
    tr, row, col, ws = (C.c_uint32() for _ in range(4))
    for task in range(ntasks):
        so.catcoc_task_tile(L.MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row), C.byref(col), C.byref(ws))
        blk = part[row.value:row.value + 128, col.value:col.value + 256]
        want_cs = 0.0 if tr.value == rank else float(blk.astype(np.float64).sum())
        assert abs(float(cs[task]) - want_cs) <= 1e-2 * max(1.0, np.abs(blk).sum()), task


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
def test_float_ragged_problems_on_many_tiles(dtype):
    # full tiles on the direct-to-LDS kernel, ragged ones on the bounds-checked kernel, in two launches
    _need_gpu()
    rng = np.random.default_rng(26)
    # reduce-scatter: 8 ranks x (2 full + 1 ragged) tile rows x (5 full + 1 ragged) tile columns
    M, N, K, P, rank = 8 * 296, 1344, 224, 8, 5
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.02)
    rows = M // P
    peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
    part, want = oracle.matmul_reduce(A, B, dtype, rank * rows, rows, peers, want_partial=True)
    dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    out = ops.matmul_reduce_scatter(dev16(A, dtype), dev16(B, dtype), [dev(p) for p in peers], rank, P, acc_dump=dump)
    torch.cuda.synchronize()
    _check_float(host16(out), want, part[rank * rows:(rank + 1) * rows] + sum(peers), dtype, K)
    assert np.abs(dump.cpu().numpy() - part).max() <= 1e-2 * max(1.0, np.abs(part).max())
    # all-gather with ragged shards and B as [n,k]
    ml, N, K, P, rank = 424, 1024, 512, 8, 2
    shards = [_rand16(rng, (ml, K), dtype) for _ in range(P)]
    B = _rand16(rng, (K, N), dtype, 0.02)
    want = oracle.allgather_matmul(shards, B, dtype)
    dsh = [dev16(s, dtype) for s in shards]
    Bt = dev16(np.ascontiguousarray(B.T), dtype)
    out = ops.allgather_matmul(dsh[rank], [dsh[r] for r in range(P) if r != rank], Bt, rank, P, trans_b=True)
    torch.cuda.synchronize()
    _check_float(host16(out), want, oracle.gemm_half_f32(np.concatenate(shards, 0), B, dtype), dtype, K)
    # all-reduce, ragged rows only
    M, N, K = 1100, 2048, 320
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.02)
    p1 = rng.standard_normal((M, N)).astype(np.float32)
    part, want = oracle.matmul_reduce(A, B, dtype, 0, M, [p1], want_partial=True)
    out = ops.matmul_allreduce(dev16(A, dtype), dev16(B, dtype), [dev(p1)], 0, 2)
    torch.cuda.synchronize()
    _check_float(host16(out), want, part + p1, dtype, K)


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
def test_float_reduce_scatter_256_row_tiles_outbound_and_checksum(dtype):
    # the direct-to-LDS kernel on 256x256 tiles; tiles of the other ranks checked through outbound stores / checksums
    _need_gpu()
    import ctypes as C
    M, N, K, P, rank = 4096, 512, 320, 8, 6
    rng = np.random.default_rng(21)
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.02)
    rows = M // P
    peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
    part, want = oracle.matmul_reduce(A, B, dtype, rank * rows, rows, peers, want_partial=True)
    t = ops.default_tiling(M, K, N, P, m0=256, n0=256, k0=256)
    d = L.make_desc(rank, P, [16] * (P - 1))
    so = L.load()
    ntasks = so.catcoc_get_task_count(L.MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d))
    need = so.catcoc_get_workspace_size(L.MATMUL_REDUCE_SCATTER, L.FP16, C.byref(t), C.byref(d))
    full = part[rank * rows:(rank + 1) * rows] + sum(peers)
    for mode in ("checksum", "outbound"):
        kw = {"checksum": torch.zeros(ntasks, dtype=torch.float64, device=DEV)} if mode == "checksum" else \
             {"outbound": torch.zeros(need // 4, dtype=torch.float32, device=DEV)}
        out = ops.matmul_reduce_scatter(dev16(A, dtype), dev16(B, dtype), [dev(p) for p in peers], rank, P, tiling=t, **kw)
        torch.cuda.synchronize()
        _check_float(host16(out), want, full, dtype, K)
        tr, row, col, ws = (C.c_uint32() for _ in range(4))
        for task in range(ntasks):
            so.catcoc_task_tile(L.MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row), C.byref(col), C.byref(ws))
            blk = part[row.value:row.value + 256, col.value:col.value + 256]
            if mode == "checksum":
                got = float(kw["checksum"][task])
                want_cs = 0.0 if tr.value == rank else float(blk.astype(np.float64).sum())
                assert abs(got - want_cs) <= 1e-2 * max(1.0, np.abs(blk).sum()), task
            elif tr.value != rank:
                ob = kw["outbound"].cpu().numpy().reshape(-1, 256)[ws.value:ws.value + 256]
                assert np.abs(ob - blk).max() <= 1e-2 * max(1.0, np.abs(blk).max()), task


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
@pytest.mark.parametrize("shape", [(4096, 512, 320, 8, 6), (2048, 1024, 4096, 4, 0), (1024, 256, 64, 2, 1)])
def test_float_reduce_scatter_256_row_tiles_weights_stored_n_by_k(dtype, shape):
    # 256x256 tiles with B as [n,k] (the layout of the reference's dynamic_tiling sweep shapes): pair buffers for both operands
    _need_gpu()
    M, N, K, P, rank = shape
    rng = np.random.default_rng(23 + K)
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.02)
    rows = M // P
    peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
    part, want = oracle.matmul_reduce(A, B, dtype, rank * rows, rows, peers, want_partial=True)
    t = ops.default_tiling(M, K, N, P, m0=256, n0=256, k0=256)
    dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    out = ops.matmul_reduce_scatter(dev16(A, dtype), dev16(np.ascontiguousarray(B.T), dtype), [dev(p) for p in peers], rank, P, tiling=t,
                                    trans_b=True, acc_dump=dump)
    L.check()
    torch.cuda.synchronize()
    _check_float(host16(out), want, part[rank * rows:(rank + 1) * rows] + sum(peers), dtype, K)
    _report_ulp("256-row tiles, B as [n,k]", ulp_diff16(host16(out), want))
    assert np.abs(dump.cpu().numpy() - part).max() <= 1e-2 * max(1.0, np.abs(part).max())


def test_float_allreduce_config1_full_size():
    # BASELINE config 1: A[512,2048], B[2048,1024] fp16 ~U(-1,1), K halves as the two ranks' partials
    _need_gpu()
    rng = np.random.default_rng(21)
    M, N, K = 512, 1024, 2048
    A = _rand16(rng, (M, K), oracle.FP16, uniform=True)
    B = _rand16(rng, (K, N), oracle.FP16, uniform=True)
    A0, B0 = np.ascontiguousarray(A[:, :K // 2]), np.ascontiguousarray(B[:K // 2])
    p1 = oracle.gemm_half_f32(np.ascontiguousarray(A[:, K // 2:]), np.ascontiguousarray(B[K // 2:]), oracle.FP16)
    part, want = oracle.matmul_reduce(A0, B0, oracle.FP16, 0, M, [p1], want_partial=True)
    out = ops.matmul_allreduce(dev16(A0, oracle.FP16), dev16(B0, oracle.FP16), [dev(p1)], 0, 2)
    torch.cuda.synchronize()
    _check_float(host16(out), want, part + p1, oracle.FP16, K)
    _report_ulp("config 1", ulp_diff16(host16(out), want))


@pytest.mark.parametrize("dtype", [oracle.BF16, oracle.FP16])
@pytest.mark.parametrize("shape", [(256, 512, 256, 8, 2), (100, 260, 72, 4, 0), (512, 1024, 4096, 8, 5)])
def test_allgather_matmul_reads_shards_in_place(dtype, shape):
    _need_gpu()
    ml, N, K, P, rank = shape
    rng = np.random.default_rng(22)
    shards = [_rand16(rng, (ml, K), dtype) for _ in range(P)]
    B = _rand16(rng, (K, N), dtype, 0.02)
    want = oracle.allgather_matmul(shards, B, dtype)
    dsh = [dev16(s, dtype) for s in shards]          # P separate allocations
    out = ops.allgather_matmul(dsh[rank], [dsh[r] for r in range(P) if r != rank], dev16(B, dtype), rank, P)
    torch.cuda.synchronize()
    full = oracle.gemm_half_f32(np.concatenate(shards, 0), B, dtype)
    _check_float(host16(out), want, full, dtype, K)
    if ml % 256 == 0 and N % 256 == 0:     # the same on 256x256 tiles, in both layouts of B
        t = ops.default_tiling(ml, K, N, P, m0=256, n0=256, k0=256)
        for tb in (False, True):
            Bd = dev16(np.ascontiguousarray(B.T) if tb else B, dtype)
            out = ops.allgather_matmul(dsh[rank], [dsh[r] for r in range(P) if r != rank], Bd, rank, P, tiling=t, trans_b=tb)
            L.check()
            torch.cuda.synchronize()
            _check_float(host16(out), want, full, dtype, K)


@pytest.mark.parametrize("kslices", [False, True])
def test_allgather_matmul_operands_streamed_from_hbm(kslices):
    """All-gather matmul whose operands stream from HBM (four shards of [256, 8192] bf16 in separate allocations against
    B [8192, 4096], 72 MB, 128 tiles): the six-stage ring with A copied in pairs of k steps out of the shard each tile row
    belongs to, whole and in two k slices.  A sample of rows from every shard against the oracle, the rest of the output
    through column sums against fp64."""
    _need_gpu()
    dtype = oracle.BF16
    ml, N, K, P, rank = 256, 4096, 8192, 4, 1
    g = torch.Generator(device=DEV).manual_seed(301)
    dsh = [torch.randn((ml, K), device=DEV, generator=g).bfloat16() for _ in range(P)]     # P separate allocations
    B = (torch.randn((K, N), device=DEV, generator=g) * 0.02).bfloat16()
    ws = None
    if kslices:
        need, f = ops.kslice_plan(L.ALLGATHER_MATMUL, torch.bfloat16, ml, K, N, rank, P)
        assert f == 2
        ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    # the operator takes this rank's shard first, then the others in rank order: the gathered A is dsh in rank order
    out = ops.allgather_matmul(dsh[rank], [dsh[r] for r in range(P) if r != rank], B, rank, P, workspace=ws)
    torch.cuda.synchronize()
    sel = np.arange(7, ml, 37)
    shards_sel = [host16(d[sel]) for d in dsh]
    want = oracle.allgather_matmul(shards_sel, host16(B), dtype)
    full = oracle.gemm_half_f32(np.concatenate(shards_sel, 0), host16(B), dtype)
    got = np.concatenate([host16(out[r * ml:(r + 1) * ml][sel]) for r in range(P)], 0)
    _check_float(got, want, full, dtype, K)
    a_all = torch.cat(dsh, 0).double()
    col_sums = a_all.sum(0) @ B.double()                     # sum over all rows of every output column
    got_sums = out.double().sum(0)
    # every output element carries a bf16 rounding of at most 2^-9 relative
    bound = (a_all.abs().sum(0) @ B.double().abs()) * 2.0 ** -8
    assert bool(((got_sums - col_sums).abs() <= bound).all())


@pytest.mark.parametrize("dtype", [oracle.BF16, oracle.FP16])
def test_float_few_tiles_k_sliced(dtype):
    # two k slices per tile: an fp32 sum of two partials, the same whichever slice arrives last, so repeated
    # launches agree bit for bit, and the result stays inside the float tolerance of the unsliced oracle
    _need_gpu()
    rng = np.random.default_rng(24)
    tdt = TORCH_DT[dtype]
    # all-gather: 8 shards of 128 rows, 32 tiles
    ml, N, K, P, rank = 128, 512, 2048, 8, 3
    shards = [_rand16(rng, (ml, K), dtype) for _ in range(P)]
    B = _rand16(rng, (K, N), dtype, 0.02)
    want = oracle.allgather_matmul(shards, B, dtype)
    need, f = ops.kslice_plan(L.ALLGATHER_MATMUL, tdt, ml, K, N, rank, P)
    assert f == 2
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    dsh = [dev16(x, dtype) for x in shards]
    outs = []
    for _ in range(3):
        out = ops.allgather_matmul(dsh[rank], [dsh[r] for r in range(P) if r != rank], dev16(B, dtype), rank, P, workspace=ws)
        torch.cuda.synchronize()
        outs.append(host16(out))
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    _check_float(outs[0], want, oracle.gemm_half_f32(np.concatenate(shards, 0), B, dtype), dtype, K)
    # reduce-scatter with peers and all-reduce, 16 tiles each
    M, N, K, P, rank = 1024, 512, 1024, 4, 2
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.02)
    rows = M // P
    peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
    part, want = oracle.matmul_reduce(A, B, dtype, rank * rows, rows, peers, want_partial=True)
    need, f = ops.kslice_plan(L.MATMUL_REDUCE_SCATTER, tdt, M, K, N, rank, P)
    assert f == 2
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    out = ops.matmul_reduce_scatter(dev16(A, dtype), dev16(B, dtype), [dev(p) for p in peers], rank, P, acc_dump=dump, workspace=ws)
    torch.cuda.synchronize()
    _check_float(host16(out), want, part[rank * rows:(rank + 1) * rows] + sum(peers), dtype, K)
    assert np.abs(dump.cpu().numpy() - part).max() <= 1e-2 * max(1.0, np.abs(part).max())
    fullp = [rng.standard_normal((M, N)).astype(np.float32)]
    part, want = oracle.matmul_reduce(A, B, dtype, 0, M, fullp, want_partial=True)
    need, f = ops.kslice_plan(L.MATMUL_ALLREDUCE, tdt, M, K, N, 0, 2)
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    out = ops.matmul_allreduce(dev16(A, dtype), dev16(B, dtype), [dev(fullp[0])], 0, 2, workspace=ws)
    torch.cuda.synchronize()
    _check_float(host16(out), want, part + fullp[0], dtype, K)
    # three and more slices (the caller's choice): their fp32 partials are added in slice order whichever slice arrives last,
    # so repeated launches still agree bit for bit, outputs and dumped partials alike
    for f in (3, 4, 8):
        need, got_f = ops.kslice_plan(L.MATMUL_ALLREDUCE, tdt, M, K, N, 0, 2, split_k=f)
        assert got_f == f
        ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
        outs, dumps = [], []
        for _ in range(3):
            dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
            out = ops.matmul_allreduce(dev16(A, dtype), dev16(B, dtype), [dev(fullp[0])], 0, 2, workspace=ws, split_k=f, acc_dump=dump)
            torch.cuda.synchronize()
            outs.append(host16(out))
            dumps.append(dump.cpu().numpy())
        assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2]), f
        assert np.array_equal(dumps[0], dumps[1]) and np.array_equal(dumps[0], dumps[2]), f
        _check_float(outs[0], want, part + fullp[0], dtype, K)
        assert not ws[:65536].any()


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
def test_float_weights_stored_n_by_k(dtype):
    _need_gpu()
    rng = np.random.default_rng(25)
    tdt = TORCH_DT[dtype]
    M, N, K, P, rank = 1024, 768, 640, 4, 3
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.02)
    Bt = np.ascontiguousarray(B.T)
    rows = M // P
    peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
    part, want = oracle.matmul_reduce(A, B, dtype, rank * rows, rows, peers, want_partial=True)
    dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    out = ops.matmul_reduce_scatter(dev16(A, dtype), dev16(Bt, dtype), [dev(p) for p in peers], rank, P, trans_b=True, acc_dump=dump)
    torch.cuda.synchronize()
    _check_float(host16(out), want, part[rank * rows:(rank + 1) * rows] + sum(peers), dtype, K)
    assert np.abs(dump.cpu().numpy() - part).max() <= 1e-2 * max(1.0, np.abs(part).max())
    # the same operands through the row-major path: same MFMAs in the same k order, so the fp32 partials are identical
    dump2 = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    ops.matmul_reduce_scatter(dev16(A, dtype), dev16(B, dtype), [dev(p) for p in peers], rank, P, acc_dump=dump2)
    torch.cuda.synchronize()
    assert torch.equal(dump, dump2)
    # all-gather with [n,k] weights and two k slices
    ml, N, K, P, rank = 128, 512, 2048, 8, 6
    shards = [_rand16(rng, (ml, K), dtype) for _ in range(P)]
    B = _rand16(rng, (K, N), dtype, 0.02)
    want = oracle.allgather_matmul(shards, B, dtype)
    need, f = ops.kslice_plan(L.ALLGATHER_MATMUL, tdt, ml, K, N, rank, P)
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    dsh = [dev16(x, dtype) for x in shards]
    out = ops.allgather_matmul(dsh[rank], [dsh[r] for r in range(P) if r != rank], dev16(np.ascontiguousarray(B.T), dtype), rank, P,
                               trans_b=True, workspace=ws)
    torch.cuda.synchronize()
    _check_float(host16(out), want, oracle.gemm_half_f32(np.concatenate(shards, 0), B, dtype), dtype, K)


@pytest.mark.parametrize("case", [(2048, 512, 320, 4, 1, False, None), (2048, 512, 320, 4, 2, True, None), (8 * 304, 1344, 192, 8, 5, False, None),
                                  (8 * 304, 1344, 192, 8, 0, True, None), (1024, 1024, 2048, 4, 1, False, (0, 4)), (32, 129, 100, 4, 3, False, None)])
def test_quant_rs_activations_stored_k_by_m(case):
    # A given as [k,m]: full and ragged problems on the direct-to-LDS kernel (A staged as rows of k and read through the
    # transposing LDS reads), with either layout of B, also cut into k slices; anything else on the general kernel
    M, N, K, P, rank, tb, ks = case
    r = quant_case(np.random.default_rng(60 + rank), M, N, K, P, rank, bias=True, trans_a=True, trans_b=tb, launches=2, kslices=ks)
    if M >= 1024:
        assert r["exact"] == r["total"]


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
def test_float_activations_stored_k_by_m(dtype):
    _need_gpu()
    rng = np.random.default_rng(27)
    for (M, N, K, P, rank) in ((2048, 512, 224, 4, 3), (8 * 296, 1344, 96, 8, 6)):
        A = _rand16(rng, (M, K), dtype)
        B = _rand16(rng, (K, N), dtype, 0.02)
        rows = M // P
        peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
        part, want = oracle.matmul_reduce(A, B, dtype, rank * rows, rows, peers, want_partial=True)
        full = part[rank * rows:(rank + 1) * rows] + sum(peers)
        At = dev16(np.ascontiguousarray(A.T), dtype)
        for tb in (0, 1):
            b = dev16(np.ascontiguousarray(B.T) if tb else B, dtype)
            dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
            out = ops.matmul_reduce_scatter(At, b, [dev(p) for p in peers], rank, P, trans_a=True, trans_b=bool(tb), acc_dump=dump)
            torch.cuda.synchronize()
            _check_float(host16(out), want, full, dtype, K)
            assert np.abs(dump.cpu().numpy() - part).max() <= 1e-2 * max(1.0, np.abs(part).max())
    # all-reduce, cut into two k slices
    M, N, K = 1024, 512, 1024
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.02)
    p1 = rng.standard_normal((M, N)).astype(np.float32)
    part, want = oracle.matmul_reduce(A, B, dtype, 0, M, [p1], want_partial=True)
    need, f = ops.kslice_plan(L.MATMUL_ALLREDUCE, TORCH_DT[dtype], M, K, N, 0, 2)
    assert f == 2
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    out = ops.matmul_allreduce(dev16(np.ascontiguousarray(A.T), dtype), dev16(B, dtype), [dev(p1)], 0, 2, trans_a=True, workspace=ws)
    torch.cuda.synchronize()
    _check_float(host16(out), want, part + p1, dtype, K)


def test_float_transposed_operands_general_kernel():
    _need_gpu()
    rng = np.random.default_rng(23)
    M, N, K, P, rank = 256, 260, 96, 4, 2
    A = _rand16(rng, (M, K), oracle.FP16)
    B = _rand16(rng, (K, N), oracle.FP16, 0.05)
    rows = M // P
    peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
    part, want = oracle.matmul_reduce(A, B, oracle.FP16, rank * rows, rows, peers, want_partial=True)
    full = part[rank * rows:(rank + 1) * rows] + sum(peers)
    for ta, tb in ((0, 1), (1, 0), (1, 1)):
        a = np.ascontiguousarray(A.T) if ta else A
        b = np.ascontiguousarray(B.T) if tb else B
        out = ops.matmul_reduce_scatter(dev16(a, oracle.FP16), dev16(b, oracle.FP16), [dev(p) for p in peers], rank, P,
                                        trans_a=bool(ta), trans_b=bool(tb))
        torch.cuda.synchronize()
        _check_float(host16(out), want, full, oracle.FP16, K)


# ------------------------------------------------ round-pipelined, reference-faithful form
def _outbound_for(comm, dt_code, t, rank, P, dtype):
    import ctypes as C
    d = L.make_desc(rank, P, [16] * (P - 1))
    need = L.load().catcoc_get_workspace_size(comm, dt_code, C.byref(t), C.byref(d))
    L.check()
    return torch.zeros(need // 4, dtype=dtype, device=DEV)


@pytest.mark.parametrize("case", [(2048, 512, 256, 8, 3, 16, 1, 64, True), (2048, 512, 256, 8, 3, 16, 1, 64, False),
                                  (4096, 1024, 320, 8, 7, 64, 2, 32, True), (1024, 768, 192, 4, 0, 20, 3, 128, False),
                                  (800, 264, 208, 8, 5, 8, 1, 64, True)])
def test_pipelined_quant_equals_fused_int32_reduce_and_oracle(case):
    # GEMM rounds on one stream, comm rounds (BlockCommSwizzle task list, int32 adds into c_accum) and the dequant pass on
    # another, stage reuse guarded by events.  int32 adds are exact in any order, so both comm schedules must equal the
    # oracle and the fused kernel's int32-reduce mode bit for bit.
    _need_gpu()
    M, N, K, P, rank, block_num, ci, cb, det = case
    rng = np.random.default_rng(900 + M + ci)
    x1 = rng.integers(-127, 128, (M, K), dtype=np.int8)
    x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s1 = rng.uniform(0.005, 0.02, M).astype(np.float32)
    s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.integers(-1000, 1000, N, dtype=np.int32)
    rows = M // P
    peers = [rng.integers(-2 ** 24, 2 ** 24, (rows, N), dtype=np.int32) for _ in range(P - 1)]
    acc_want, out_want = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, b, rank * rows, rows, peers, oracle.BF16, reduce_int32=True)
    t = ops.default_tiling(M, K, N, P, m0=128, n0=256, k0=256, commInterval=ci, commBlockM=cb, commDataSplit=20, commNpuSplit=1)
    import ctypes as C
    d = L.make_desc(rank, P, [16] * (P - 1), block_num=block_num)
    need = L.load().catcoc_get_workspace_size(L.QUANT_MATMUL_REDUCE_SCATTER, L.INT8, C.byref(t), C.byref(d))
    ob = torch.zeros(need // 4, dtype=torch.int32, device=DEV)
    side = torch.cuda.Stream()
    dx = [dev(x1), dev(x2), dev(s1), dev(s2), dev(b)]
    dp = [dev(p) for p in peers]
    for it in range(2):
        out, cacc = ops.pipelined_quant_matmul_reduce_scatter(*dx, dp, rank, P, ob, tiling=t, deterministic=det, comm_stream=side,
                                                              block_num=block_num)
        torch.cuda.synchronize()
        kept = acc_want[rank * rows:(rank + 1) * rows] + sum(peers)
        assert np.array_equal(cacc.cpu().numpy(), kept), "reduced int32 block differs"
        assert np.array_equal(host16(out), out_want), "dequantised output differs from the oracle"
    fused = ops.quant_matmul_reduce_scatter(*dx, dp, rank, P, tiling=t, reduce_int32=True, block_num=block_num)
    torch.cuda.synchronize()
    assert torch.equal(fused.view(torch.int16), out.view(torch.int16))
    # the other ranks' int32 tiles sit in the workspace ring where the reference puts them (stage = round % 2)
    so = L.load()
    ntasks = so.catcoc_get_task_count(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d))
    obh = ob.cpu().numpy().reshape(-1, 256)
    bpc = (block_num or 256) * ci
    last_round = (ntasks - 1) // bpc
    tr, row, col, ws = (C.c_uint32() for _ in range(4))
    checked = 0
    for task in range(ntasks):
        so.catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row), C.byref(col), C.byref(ws))
        rnd = task // bpc
        if tr.value == rank or rnd + 2 <= last_round:        # kept tiles go to c_accum; older rounds were overwritten
            continue
        r0, c0 = row.value, col.value
        rv, cv = min(128, (tr.value + 1) * rows - r0), min(256, N - c0)
        assert np.array_equal(obh[ws.value:ws.value + rv, :cv], acc_want[r0:r0 + rv, c0:c0 + cv]), task
        checked += 1
    assert checked > 0


@pytest.mark.parametrize("tb", [False, True])
def test_pipelined_quant_on_the_librarys_256_row_tiles(tb):
    """A shape large enough for the library to choose 256x256 tiles by itself (8192x4096x8192, tiling m0 = 0), in both weight
    layouts: the round-pipelined operator (GEMM rounds of 256-row tiles, comm rounds, int32 reduce) against the fused
    int32-reduce launch bit for bit, and a sample of kept rows against the oracle."""
    _need_gpu()
    import ctypes as C
    M, N, K, P, rank = 8192, 8192, 4096, 8, 6
    g = torch.Generator(device=DEV).manual_seed(77)
    x1 = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=DEV, generator=g)
    x2 = torch.randint(-127, 128, (N, K) if tb else (K, N), dtype=torch.int8, device=DEV, generator=g)
    s1 = torch.empty(M, device=DEV).uniform_(0.005, 0.02, generator=g)
    s2 = torch.empty(N, device=DEV).uniform_(0.001, 0.01, generator=g)
    rows = M // P
    peers = [torch.randint(-2 ** 24, 2 ** 24, (rows, N), dtype=torch.int32, device=DEV, generator=g) for _ in range(P - 1)]
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0, commInterval=1)
    d = L.make_desc(rank, P, [16] * (P - 1))
    ntasks = L.load().catcoc_get_task_count(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d))
    assert ntasks == 1024          # 32 x 32 tiles of 256 x 256
    ob = _outbound_for(L.QUANT_MATMUL_REDUCE_SCATTER, L.INT8, t, rank, P, torch.int32)
    side = torch.cuda.Stream()
    out, cacc = ops.pipelined_quant_matmul_reduce_scatter(x1, x2, s1, s2, None, peers, rank, P, ob, tiling=t, comm_stream=side, trans_b=tb)
    L.check()
    torch.cuda.synchronize()
    fused = ops.quant_matmul_reduce_scatter(x1, x2, s1, s2, None, peers, rank, P, tiling=t, trans_b=tb, reduce_int32=True)
    torch.cuda.synchronize()
    assert torch.equal(fused.view(torch.int16), out.view(torch.int16))
    sel = np.array([0, 1, 255, 256, 511, 700, rows - 1])
    idx = torch.as_tensor(sel, device=DEV)
    x2h = x2.cpu().numpy()
    if tb:
        x2h = np.ascontiguousarray(x2h.T)
    acc, want = oracle.quant_matmul_reduce_scatter(x1[idx + rank * rows].cpu().numpy(), x2h, s1[idx + rank * rows].cpu().numpy(), s2.cpu().numpy(),
                                                   None, 0, len(sel), [p[idx].cpu().numpy() for p in peers], oracle.BF16, reduce_int32=True)
    assert np.array_equal(host16(out[idx]), want)
    assert np.array_equal(cacc[idx].cpu().numpy(), acc + sum(p[idx].cpu().numpy() for p in peers))


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
@pytest.mark.parametrize("case", [(2048, 512, 256, 8, 2, 16, 1, 64), (1024, 1024, 320, 4, 3, 0, 1, 32), (4096, 512, 128, 8, 6, 32, 2, 128)])
def test_pipelined_float_reduces_in_half_precision_deterministically(dtype, case):
    # the reference's float reduce: local partial rounded to the 16-bit type, 16-bit peers, one rounding per add
    # (matmul_reduce_scatter.hpp:261).  With the deterministic comm swizzle the order of every block's adds is fixed,
    # so the result equals the oracle's replay of the comm rounds bit for bit, launch after launch.
    _need_gpu()
    M, N, K, P, rank, block_num, ci, cb = case
    rng = np.random.default_rng(950 + M)
    A = _rand16(rng, (M, K), dtype)
    B = _rand16(rng, (K, N), dtype, 0.05)
    rows = M // P
    peers = [oracle.f32_to_half(rng.standard_normal((rows, N)).astype(np.float32), dtype) for _ in range(P - 1)]
    t = ops.default_tiling(M, K, N, P, m0=128, n0=256, k0=256, commInterval=ci, commBlockM=cb, commDataSplit=24, commNpuSplit=1)
    import ctypes as C
    d = L.make_desc(rank, P, [16] * (P - 1), block_num=block_num)
    need = L.load().catcoc_get_workspace_size(L.MATMUL_REDUCE_SCATTER, dtype, C.byref(t), C.byref(d))
    ob = torch.zeros(need // 4, dtype=torch.float32, device=DEV)
    dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    side = torch.cuda.Stream()
    dA, dB, dP = dev16(A, dtype), dev16(B, dtype), [dev16(p, dtype) for p in peers]
    outs = []
    for it in range(3):
        out = ops.pipelined_matmul_reduce_scatter(dA, dB, dP, rank, P, ob, tiling=t, deterministic=True, comm_stream=side,
                                                  block_num=block_num, acc_dump=dump)
        torch.cuda.synchronize()
        outs.append(host16(out))
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    local = dump.cpu().numpy()
    part = oracle.gemm_half_f32(A, B, dtype)
    assert np.abs(local - part).max() <= 1e-2 * max(1.0, np.abs(part).max())         # the GEMM itself, fp32 accumulate
    want = oracle.pipelined_reduce_half(local[rank * rows:(rank + 1) * rows], peers, dtype, M, P, rank, 128, 256, block_num or 256, ci, cb, 24, 1)
    assert np.array_equal(outs[0], want), "half-precision reduce differs from the replay of the comm rounds"
    # against the unrounded sum: the textbook bound of recursive summation with unit roundoff u of the 16-bit type,
    # |error| <= P * u * (|local| + sum |peers|) (P roundings; the reference's own element-wise gate, two ulps of the
    # result, is tighter than what reducing in half precision can promise when partials cancel), and no bias
    pf = [oracle.half_to_f32(p, dtype) for p in peers]
    full = part[rank * rows:(rank + 1) * rows] + sum(pf)
    mag = np.abs(part[rank * rows:(rank + 1) * rows]) + sum(np.abs(x) for x in pf)
    u = 2.0 ** -11 if dtype == oracle.FP16 else 2.0 ** -8
    err = np.abs(oracle.half_to_f32(outs[0], dtype) - full)
    assert (err <= 1.01 * P * u * mag + 1e-6).all()
    _, _, eb = oracle.verify(oracle.half_to_f32(outs[0], dtype), full, dtype, K)
    assert eb <= 2.0 ** -12, eb


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
def test_pipelined_float_atomic_schedule_on_exactly_summable_data(dtype):
    # BlockCommSwizzle<0,false> with hardware 16-bit atomic adds, arrival order: checked where every partial sum is exactly
    # representable (small integers), so any order gives the same bits
    _need_gpu()
    M, N, K, P, rank = 2048, 512, 64, 8, 4
    rng = np.random.default_rng(77)
    A = oracle.f32_to_half(rng.integers(-1, 2, (M, K)).astype(np.float32), dtype)
    B = oracle.f32_to_half(rng.integers(-1, 2, (K, N)).astype(np.float32), dtype)
    rows = M // P
    peers = [oracle.f32_to_half(rng.integers(-8, 9, (rows, N)).astype(np.float32), dtype) for _ in range(P - 1)]
    t = ops.default_tiling(M, K, N, P, m0=128, n0=256, k0=256, commInterval=1, commBlockM=64, commDataSplit=16, commNpuSplit=2)
    import ctypes as C
    d = L.make_desc(rank, P, [16] * (P - 1), block_num=16)
    need = L.load().catcoc_get_workspace_size(L.MATMUL_REDUCE_SCATTER, dtype, C.byref(t), C.byref(d))
    ob = torch.zeros(need // 4, dtype=torch.float32, device=DEV)
    out = ops.pipelined_matmul_reduce_scatter(dev16(A, dtype), dev16(B, dtype), [dev16(p, dtype) for p in peers], rank, P, ob, tiling=t,
                                              deterministic=False, comm_stream=torch.cuda.Stream(), block_num=16)
    torch.cuda.synchronize()
    part = oracle.half_to_f32(A, dtype)[rank * rows:(rank + 1) * rows] @ oracle.half_to_f32(B, dtype)
    want = part + sum(oracle.half_to_f32(p, dtype) for p in peers)
    assert np.abs(want).max() <= 256                                   # integers below 2^8: exact in bf16 and fp16
    assert np.array_equal(oracle.half_to_f32(host16(out), dtype), want.astype(np.float32))


@pytest.mark.parametrize("case", [(4, 1024 * 1024, None), (2, 4096 * 13, torch.float16), (7, 1000 * 4, torch.bfloat16), (1, 515, torch.bfloat16),
                                  (3, 64, None)])
def test_splitk_reduce_add_kernel(case):
    # SplitkMatmul's ReduceAdd as a kernel of its own: slices summed in slice order in fp32, one cast
    _need_gpu()
    f, count, dt = case
    rng = np.random.default_rng(f * 31 + count % 97)
    src = (rng.standard_normal((f, count)) * 10).astype(np.float32)
    got = ops.reduce_add(dev(src), dt)
    torch.cuda.synchronize()
    code = 0 if dt is None else (oracle.FP16 if dt == torch.float16 else oracle.BF16)
    want = oracle.reduce_add(src, code)
    if dt is None:
        assert np.array_equal(got.cpu().numpy(), want)
    else:
        assert np.array_equal(host16(got), want)


def test_cpp_host_written_against_the_kernel_template_facade():
    # include/catcoc_hip/dgemm.hpp: the reference's Catcoc::DGemm::Kernel::* class templates with their Params, forwarding
    # to the C ABI; the host program compares each operator bit for bit with the direct C-ABI launch
    _need_gpu()
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(L.LIB_PATH)), "catcoc_facade_host")
    assert os.path.exists(exe), "catcoc_facade_host is not built"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    for name in ("QuantMatmulReduceScatter", "MatmulReduceScatter fp16", "MatmulAllReduce fp16", "AllGatherMatmul fp16",
                 "MatmulReduceScatter bf16", "MatmulAllReduce bf16", "AllGatherMatmul bf16"):
        assert "PASS " + name in r.stdout, r.stdout
    assert "facade ok" in r.stdout


# ------------------------------------------------------------ full benchmark size
def test_quant_config4_full_size_properties():
    """W8A8 benchmark config (M=8192, K=1792, N=4096, P=8) at full size.  The oracle checks a row sample
    bit-exactly; the whole output is checked through size-independent properties: int32 accumulators
    against torch's exact integer row/column sums, and linearity in the peer partials."""
    _need_gpu()
    M, N, K, P, rank = 8192, 4096, 1792, 8, 3
    g = torch.Generator(device=DEV).manual_seed(4)
    x1 = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=DEV, generator=g)
    x2 = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=DEV, generator=g)
    s1 = torch.empty(M, device=DEV).uniform_(0.005, 0.02, generator=g)
    s2 = torch.empty(N, device=DEV).uniform_(0.001, 0.01, generator=g)
    rows = M // P
    peers = [torch.randn((rows, N), device=DEV, generator=g) for _ in range(P - 1)]
    dump = torch.zeros((M, N), dtype=torch.int32, device=DEV)
    out = ops.quant_matmul_reduce_scatter(x1, x2, s1, s2, None, peers, rank, P, acc_dump=dump)
    torch.cuda.synchronize()
    # checksum of checksums: sum_j acc[i,j] == x1[i,:] . rowsum(x2), exact in int64
    # (fp64 holds these integers exactly: every partial sum is below 2^53)
    want_rows = x1.double() @ x2.double().sum(1)
    assert torch.equal(dump.to(torch.int64).sum(1), want_rows.to(torch.int64))
    want_cols = x1.double().sum(0) @ x2.double()
    assert torch.equal(dump.to(torch.int64).sum(0), want_cols.to(torch.int64))
    # oracle on a row sample of the kept block, bit for bit
    sel = np.arange(rank * rows, (rank + 1) * rows, 37)
    acc_s, out_s = oracle.quant_matmul_reduce_scatter(
        x1[sel].cpu().numpy(), x2.cpu().numpy(), s1[sel].cpu().numpy(), s2.cpu().numpy(), None, 0, len(sel),
        [p[sel - rank * rows].cpu().numpy() for p in peers], oracle.BF16)
    assert np.array_equal(dump[sel].cpu().numpy(), acc_s)
    assert ulp_diff16(host16(out[sel - rank * rows]), out_s).max() <= 1
    # zero peers leave the pure dequantised block: out0 == bf16(float(acc) * s2 * s1)
    zeros = [torch.zeros_like(peers[0])] * (P - 1)
    out0 = ops.quant_matmul_reduce_scatter(x1, x2, s1, s2, None, zeros, rank, P)
    torch.cuda.synchronize()
    blk = dump[rank * rows:(rank + 1) * rows].float()
    want0 = ((blk * s2[None, :]) * s1[rank * rows:(rank + 1) * rows, None]).to(torch.bfloat16)
    assert torch.equal(out0.view(torch.int16), want0.view(torch.int16))


def test_quant_config4_full_size_int32_reduce():
    """The reference's own W8A8 data flow at the benchmark size (M=8192, K=1792, N=4096, P=8): int32 peers join the
    accumulators before the dequantisation (quant_matmul_reduce_scatter.hpp:285-351), the other ranks' tiles leave as raw
    int32.  Exact integer checks of the whole kept block and of the workspace tiles, the output against the same fp32
    products in torch, a row sample against the oracle, and the round-pipelined operator against the fused launch."""
    _need_gpu()
    import ctypes as C
    M, N, K, P, rank = 8192, 4096, 1792, 8, 5
    g = torch.Generator(device=DEV).manual_seed(44)
    x1 = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=DEV, generator=g)
    x2 = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=DEV, generator=g)
    s1 = torch.empty(M, device=DEV).uniform_(0.005, 0.02, generator=g)
    s2 = torch.empty(N, device=DEV).uniform_(0.001, 0.01, generator=g)
    bias = torch.randint(-1000, 1000, (N,), dtype=torch.int32, device=DEV, generator=g)
    rows = M // P
    peers = [torch.randint(-2 ** 24, 2 ** 24, (rows, N), dtype=torch.int32, device=DEV, generator=g) for _ in range(P - 1)]
    # (one comm round holds all 1024 tasks: a single launch runs them in its own order, so no workspace stage may be reused)
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0, commInterval=4)
    d = L.make_desc(rank, P, [16] * (P - 1))
    so = L.load()
    need = so.catcoc_get_workspace_size(L.QUANT_MATMUL_REDUCE_SCATTER, L.INT8, C.byref(t), C.byref(d))
    ntasks = so.catcoc_get_task_count(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d))
    ob = torch.zeros(need // 4, dtype=torch.int32, device=DEV)
    dump = torch.zeros((M, N), dtype=torch.int32, device=DEV)
    cacc = torch.full((rows, N), -7, dtype=torch.int32, device=DEV)
    out = ops.quant_matmul_reduce_scatter(x1, x2, s1, s2, bias, peers, rank, P, reduce_int32=True, acc_dump=dump, c_accum=cacc, outbound=ob,
                                          tiling=t)
    torch.cuda.synchronize()
    # accumulators (bias included) through exact row sums; the kept block = accumulators + peers, exactly
    want_rows = x1.double() @ x2.double().sum(1) + float(bias.to(torch.int64).sum())
    assert torch.equal(dump.to(torch.int64).sum(1), want_rows.to(torch.int64))
    kept = dump[rank * rows:(rank + 1) * rows].clone()
    for p in peers:
        kept += p
    assert torch.equal(cacc, kept)
    want = ((kept.float() * s2[None, :]) * s1[rank * rows:(rank + 1) * rows, None]).to(torch.bfloat16)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    # row sample against the oracle, bit for bit
    sel = np.arange(rank * rows, (rank + 1) * rows, 61)
    acc_s, out_s = oracle.quant_matmul_reduce_scatter(
        x1[sel].cpu().numpy(), x2.cpu().numpy(), s1[sel].cpu().numpy(), s2.cpu().numpy(), bias.cpu().numpy(), 0, len(sel),
        [p[sel - rank * rows].cpu().numpy() for p in peers], oracle.BF16, reduce_int32=True)
    assert np.array_equal(dump[sel].cpu().numpy(), acc_s)
    assert np.array_equal(host16(out[sel - rank * rows]), out_s)
    # raw int32 tiles of the other ranks where the reference puts them
    obv = ob.view(-1, 256)
    tr, row, col, ws = (C.c_uint32() for _ in range(4))
    checked = 0
    for task in range(0, ntasks, 7):
        so.catcoc_task_tile(L.QUANT_MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row), C.byref(col), C.byref(ws))
        if tr.value == rank:
            continue
        assert torch.equal(obv[ws.value:ws.value + 128], dump[row.value:row.value + 128, col.value:col.value + 256]), task
        checked += 1
    assert checked > 100
    # the round-pipelined operator (GEMM rounds and comm rounds on two streams) gives the same bits
    del ob
    t1 = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)   # four rounds of 256 tasks on two workspace stages
    ob2 = _outbound_for(L.QUANT_MATMUL_REDUCE_SCATTER, L.INT8, t1, rank, P, torch.int32)
    side = torch.cuda.Stream()
    for det in (True, False):
        out2, cacc2 = ops.pipelined_quant_matmul_reduce_scatter(x1, x2, s1, s2, bias, peers, rank, P, ob2, tiling=t1, deterministic=det,
                                                                comm_stream=side)
        torch.cuda.synchronize()
        assert torch.equal(cacc2, kept)
        assert torch.equal(out2.view(torch.int16), out.view(torch.int16))


def test_float_config3_full_size_properties():
    """fp16 matmul-reduce-scatter benchmark config (A[4096,1792] N(0,1), B[1792,4096] N(0,0.02), P=8, 7 fp32 peers,
    kept block [512,4096]) at full size: 512 tiles of 128x256, the launch order of the many-tile regime.  A row sample
    of the kept block against the oracle; the whole local partial through row / column sums against fp64 GEMVs; the
    other ranks' tiles through their per-task checksums."""
    _need_gpu()
    import ctypes as C
    M, N, K, P, rank = 4096, 4096, 1792, 8, 5
    g = torch.Generator(device=DEV).manual_seed(33)
    A = torch.randn((M, K), device=DEV, generator=g).half()
    B = (torch.randn((K, N), device=DEV, generator=g) * 0.02).half()
    rows = M // P
    peers = [torch.randn((rows, N), device=DEV, generator=g) for _ in range(P - 1)]
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
    d = L.make_desc(rank, P, [16] * (P - 1))
    so = L.load()
    ntasks = so.catcoc_get_task_count(L.MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d))
    assert ntasks == 512
    dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    cs = torch.zeros(ntasks, dtype=torch.float64, device=DEV)
    out = ops.matmul_reduce_scatter(A, B, peers, rank, P, acc_dump=dump, checksum=cs)
    torch.cuda.synchronize()
    Ad, Bd = A.double(), B.double()
    # sum_j C[i,j] = A[i,:] . rowsum(B); |C| ~ 0.85, fp32 accumulation error of a 1792-term dot ~1e-5 per element
    want_rows = Ad @ Bd.sum(1)
    assert (dump.double().sum(1) - want_rows).abs().max().item() <= 2e-2
    want_cols = Ad.sum(0) @ Bd
    assert (dump.double().sum(0) - want_cols).abs().max().item() <= 2e-2
    # oracle on a row sample of the kept block
    sel = np.arange(rank * rows, (rank + 1) * rows, 29)
    part, want = oracle.matmul_reduce(host16(A[sel]), host16(B), oracle.FP16, 0, len(sel),
                                      [p[sel - rank * rows].cpu().numpy() for p in peers], want_partial=True)
    full = part + sum(p[sel - rank * rows].cpu().numpy() for p in peers)
    _check_float(host16(out[sel - rank * rows]), want, full, oracle.FP16, K)
    _report_ulp("row sample", ulp_diff16(host16(out[sel - rank * rows]), want))
    assert np.abs(dump[sel].cpu().numpy() - part).max() <= 1e-3
    # every task of another rank left the sum of its tile; kept tasks leave their slot untouched
    csh = cs.cpu().numpy()
    tile_sums = dump.double().view(M // 128, 128, N // 256, 256).sum((1, 3)).cpu().numpy()
    tr, row, col, ws = (C.c_uint32() for _ in range(4))
    for task in range(ntasks):
        assert so.catcoc_task_tile(L.MATMUL_REDUCE_SCATTER, C.byref(t), C.byref(d), task, C.byref(tr), C.byref(row), C.byref(col), C.byref(ws))
        want_cs = 0.0 if tr.value == rank else tile_sums[row.value // 128, col.value // 256]
        assert abs(csh[task] - want_cs) <= 1e-6 * 128 * 256, task


# the shapes the reference's own sweeps run (M, K, N[, Transpose A, Transpose B] rows of its test_shapes.csv files)
_REFERENCE_SWEEP = [
    ("allreduce", 16384, 27392, 4096, False, 2, 1, oracle.FP16),       # examples/00_matmul_allreduce/scripts/test_shapes.csv
    ("allreduce", 131072, 8192, 3072, False, 2, 0, oracle.BF16),
    ("allgather", 1024, 6148, 5120, False, 8, 3, oracle.FP16),         # examples/01_allgather_matmul/scripts/test_shapes.csv
    ("reduce_scatter", 16384, 27392, 4096, False, 8, 5, oracle.BF16),  # examples/02_matmul_reduce_scatter/scripts/test_shapes.csv
    ("reduce_scatter", 131072, 8192, 3072, False, 8, 2, oracle.FP16),
    ("reduce_scatter", 8192, 27392, 4096, True, 8, 7, oracle.FP16),    # examples/dynamic_tiling/scripts/test_shapes.csv (B as [n,k])
    ("reduce_scatter", 7936, 12544, 6656, True, 8, 0, oracle.BF16),
    ("reduce_scatter", 8144, 5120, 1696, True, 8, 4, oracle.FP16),
]


@pytest.mark.parametrize("case", _REFERENCE_SWEEP, ids=lambda c: "%s-%dx%dx%d" % (c[0], c[1], c[2], c[3]))
def test_float_shapes_of_the_reference_sweeps(case):
    """Every shape of the reference's test_shapes.csv files at full size (up to 131072 rows, k up to 27392, a k that is
    not a whole number of 16-byte pieces, row blocks that are not whole tiles, weights as [n,k]): operands of up to
    2 GiB, so every offset the kernels form is exercised near the top of its range.  A sample of output rows -- the
    first and the last of the kept block, rows either side of tile boundaries, the rest spread evenly -- against the oracle
    within the reference's gate and the stated 1e-2."""
    _need_gpu()
    op, M, K, N, tb, P, rank, dtype = case
    tdt = TORCH_DT[dtype]
    g = torch.Generator(device=DEV).manual_seed(1000 + M % 997)

    def operand(rows, cols, scale):   # generated in slabs: the fp32 draw of a 2 GiB operand would be 4 GiB at once
        t = torch.empty((rows, cols), dtype=tdt, device=DEV)
        for r0 in range(0, rows, 8192):
            r1 = min(rows, r0 + 8192)
            t[r0:r1] = (torch.randn((r1 - r0, cols), device=DEV, generator=g) * scale).to(tdt)
        return t
    Bst = operand(N, K, 0.02) if tb else operand(K, N, 0.02)
    Bh = host16(Bst)
    if op == "allgather":
        shards = [operand(M, K, 1.0) for _ in range(P)]
        out = ops.allgather_matmul(shards[rank], [shards[r] for r in range(P) if r != rank], Bst, rank, P)
        torch.cuda.synchronize()
        rows_all = M * P
        sel = np.unique(np.concatenate([[0, 127, 128, rows_all - 1, M - 1, M, 3 * M + 5], np.linspace(0, rows_all - 1, 40).astype(np.int64)]))
        Asel = np.stack([host16(shards[r // M][r % M]) for r in sel])
        part, want = oracle.matmul_reduce(Asel, Bh, dtype, 0, len(sel), [], want_partial=True)
        _check_float(host16(out[torch.as_tensor(sel, device=DEV)]), want, part, dtype, K)
        return
    A = operand(M, K, 1.0)
    kept0, kept = (0, M) if op == "allreduce" else (rank * (M // P), M // P)
    peers = [torch.randn((kept, N), device=DEV, generator=g) for _ in range(P - 1)]
    if op == "allreduce":
        out = ops.matmul_allreduce(A, Bst, peers, rank, P, trans_b=tb)
    else:
        out = ops.matmul_reduce_scatter(A, Bst, peers, rank, P, trans_b=tb)
    L.check()
    torch.cuda.synchronize()
    assert tuple(out.shape) == (kept, N)
    rel = np.unique(np.concatenate([[0, 1, 127, 128, 255, 256, kept - 129, kept - 128, kept - 2, kept - 1],
                                    np.linspace(0, kept - 1, 38).astype(np.int64)]))
    rel = rel[(rel >= 0) & (rel < kept)]
    idx = torch.as_tensor(rel, device=DEV)
    Asel = host16(A[idx + kept0])
    psel = [p[idx].cpu().numpy() for p in peers]
    part, want = oracle.matmul_reduce(Asel, Bh, dtype, 0, len(rel), psel, transB=tb, want_partial=True)
    _check_float(host16(out[idx]), want, part + sum(psel), dtype, K)
    # (sums of up to 27392 products: the blocked fp32 accumulation drifts further from the oracle's k-sequential one than at
    # the benchmark configs, and elements near zero count many ulps; the gates above are the criterion)
    _report_ulp("%s %dx%dx%d row sample" % (op, M, K, N), ulp_diff16(host16(out[idx]), want), share=0.99)


# (M, K, N, weights as [n,k], int32 peers, P, rank or None for explicit kept rows (kept_begin, kept_rows))
@pytest.mark.parametrize("case", [(16384, 27392, 4096, False, False, 8, 5), (131072, 8192, 3072, False, True, 8, 7),
                                  (8192, 27392, 4096, True, False, 8, 0), (7936, 12544, 6656, True, False, 8, 3),
                                  (16, 27392, 16384, True, False, 8, (6, 2)), (128, 27392, 16384, False, True, 8, (96, 32)),
                                  (512, 16384, 32768, False, False, 8, (448, 64))],
                         ids=lambda c: "%dx%dx%d" % (c[0], c[1], c[2]))
def test_quant_shapes_of_the_reference_sweeps(case):
    """The W8A8 operator at the sizes of the reference's sweeps (its float examples' test_shapes.csv; the quant example's own
    csv holds the 4x128x512 debug shape, tested elsewhere) and the decode form at the same k with wide n: operands of up
    to 1 GiB, kept rows anywhere.  A sample of kept rows bit for bit against the oracle."""
    _need_gpu()
    M, K, N, tb, ri, P, where = case
    g = torch.Generator(device=DEV).manual_seed(2000 + M % 997)

    def operand(rows, cols):
        t = torch.empty((rows, cols), dtype=torch.int8, device=DEV)
        for r0 in range(0, rows, 16384):
            r1 = min(rows, r0 + 16384)
            t[r0:r1] = torch.randint(-127, 128, (r1 - r0, cols), dtype=torch.int8, device=DEV, generator=g)
        return t
    x1 = operand(M, K)
    x2 = operand(N, K) if tb else operand(K, N)
    s1 = torch.empty(M, device=DEV).uniform_(0.005, 0.02, generator=g)
    s2 = torch.empty(N, device=DEV).uniform_(0.001, 0.01, generator=g)
    bias = torch.randint(-1000, 1000, (N,), dtype=torch.int32, device=DEV, generator=g)
    kb, kr = where if isinstance(where, tuple) else (where * (M // P), M // P)
    if ri:
        peers = [torch.randint(-2 ** 24, 2 ** 24, (kr, N), dtype=torch.int32, device=DEV, generator=g) for _ in range(P - 1)]
    else:
        peers = [torch.randn((kr, N), device=DEV, generator=g) for _ in range(P - 1)]
    if isinstance(where, tuple):
        need, fac, tiles = ops.splitk_plan(M, K, N, P, kb, kr)
        ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=DEV)
        out = ops.quant_matmul_splitk(x1, x2, s1, s2, bias, peers, P, kb, kr, workspace=ws, trans_b=tb, reduce_int32=ri)
    else:
        out = ops.quant_matmul_reduce_scatter(x1, x2, s1, s2, bias, peers, where, P, trans_b=tb, reduce_int32=ri)
    L.check()
    torch.cuda.synchronize()
    assert tuple(out.shape) == (kr, N)
    rel = np.unique(np.concatenate([[0, 1, 31, 32, 127, 128, kr - 129, kr - 128, kr - 2, kr - 1], np.linspace(0, kr - 1, 30).astype(np.int64)]))
    rel = rel[(rel >= 0) & (rel < kr)]
    idx = torch.as_tensor(rel, device=DEV)
    x2h = x2.cpu().numpy()
    if tb:
        x2h = np.ascontiguousarray(x2h.T)
    acc, want = oracle.quant_matmul_reduce_scatter(x1[idx + kb].cpu().numpy(), x2h, s1[idx + kb].cpu().numpy(), s2.cpu().numpy(),
                                                   bias.cpu().numpy(), 0, len(rel), [p[idx].cpu().numpy() for p in peers], oracle.BF16,
                                                   reduce_int32=ri)
    assert np.array_equal(host16(out[idx]), want), "kept rows differ from the oracle"


@pytest.mark.parametrize("case", [(1024, 8192, 8192, 8, 3, None), (512, 8192, 8192, 4, 1, (0, 2)), (1024, 8192, 6144, 2, 0, None)])
def test_quant_rs_operands_streamed_from_hbm(case):
    """At most one workgroup per CU and 48 MB of operands or more: the launch runs the six-stage ring with the pipelined
    row-layout peer loads (whole tiles kept; one case k-sliced through a workspace, one with a single peer).  Same bits as
    every other route: int32 accumulators, kept int32 block and every output element equal the oracle's."""
    M, N, K, P, rank, ks = case
    r = quant_case(np.random.default_rng(90 + rank), M, N, K, P, rank, bias=True, launches=2, kslices=ks)
    assert r["exact"] == r["total"]


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
def test_float_reduce_scatter_operands_streamed_from_hbm(dtype):
    """The same route for 2-byte operands: 256 tiles, 72 MB of A and B, a row sample against the oracle and the whole local
    partial through row sums against fp64."""
    _need_gpu()
    M, N, K, P, rank = 1024, 8192, 4096, 8, 6
    g = torch.Generator(device=DEV).manual_seed(71)
    td = TORCH_DT[dtype]
    A = torch.randn((M, K), device=DEV, generator=g).to(td)
    B = (torch.randn((K, N), device=DEV, generator=g) * 0.02).to(td)
    rows = M // P
    peers = [torch.randn((rows, N), device=DEV, generator=g) for _ in range(P - 1)]
    dump = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    out = ops.matmul_reduce_scatter(A, B, peers, rank, P, acc_dump=dump)
    torch.cuda.synchronize()
    want_rows = A.double() @ B.double().sum(1)
    assert (dump.double().sum(1) - want_rows).abs().max().item() <= 5e-2
    sel = np.arange(rank * rows, (rank + 1) * rows, 5)
    part, want = oracle.matmul_reduce(host16(A[sel]), host16(B), dtype, 0, len(sel),
                                      [p[sel - rank * rows].cpu().numpy() for p in peers], want_partial=True)
    full = part + sum(p[sel - rank * rows].cpu().numpy() for p in peers)
    _check_float(host16(out[sel - rank * rows]), want, full, dtype, K)
    _report_ulp("row sample", ulp_diff16(host16(out[sel - rank * rows]), want))
    assert np.abs(dump[sel].cpu().numpy() - part).max() <= 2e-3


@pytest.mark.parametrize("M", [1, 16, 64, 128, 512])
def test_quant_config5_full_size(M):
    """W8A8 decode sweep config at full size (K = N = 8192, P = 8, rank 0 keeps rows [0, ceil(M/8))): kept rows bit
    for bit against the oracle, the full int32 accumulators through exact row / column sums."""
    _need_gpu()
    K = N = 8192
    P = 8
    kr = -(-M // P)
    g = torch.Generator(device=DEV).manual_seed(500 + M)
    x1 = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=DEV, generator=g)
    x2 = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=DEV, generator=g)
    s1 = torch.empty(M, device=DEV).uniform_(0.005, 0.02, generator=g)
    s2 = torch.empty(N, device=DEV).uniform_(0.001, 0.01, generator=g)
    peers = [torch.randn((kr, N), device=DEV, generator=g) for _ in range(P - 1)]
    need, f, tiles = ops.splitk_plan(M, K, N, P, 0, kr)
    ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=DEV)
    dump = torch.zeros((M, N), dtype=torch.int32, device=DEV)
    out = ops.quant_matmul_splitk(x1, x2, s1, s2, None, peers, P, 0, kr, workspace=ws, acc_dump=dump)
    torch.cuda.synchronize()
    want_rows = x1.double() @ x2.double().sum(1)          # exact: every partial sum is an integer below 2^53
    assert torch.equal(dump.to(torch.int64).sum(1), want_rows.to(torch.int64))
    want_cols = x1.double().sum(0) @ x2.double()
    assert torch.equal(dump.to(torch.int64).sum(0), want_cols.to(torch.int64))
    acc_k, want = oracle.quant_matmul_reduce_scatter(x1[:kr].cpu().numpy(), x2.cpu().numpy(), s1[:kr].cpu().numpy(),
                                                     s2.cpu().numpy(), None, 0, kr, [p.cpu().numpy() for p in peers], oracle.BF16)
    assert np.array_equal(dump[:kr].cpu().numpy(), acc_k)
    assert np.array_equal(host16(out), want), "kept rows differ from the oracle"


@pytest.mark.parametrize("case", [(1024, 16, 0, 64, 8192),     # whole tiles, 128 k steps per workgroup: A copied in pairs of steps
                                  (512, 8, 448, 64, 8192), (768, 3, 256, 96, 8192),
                                  (128, 4, 64, 32, 8192),      # eight k slices of 16 steps
                                  (512, 8, 64, 64, 16384),     # two k slices of 128 steps: A in pairs with k slices
                                  (1024, 8, 128, 128, 8256)])  # an odd number of k steps: A step by step
def test_quant_explicit_kept_rows_large_tiles_streamed_operands(case):
    """Explicit kept rows on the 128x256 tiles with operands that stream from HBM (K = 8192 or more, N = 8192): six-stage ring
    on eight waves, the peers' partials in row layout through the ring of register buffers, A copied in pairs of k steps
    where a workgroup's k range is long enough -- with 15, 7, 3 and 2 peers, kept rows at the start, at the end and in the
    middle of A, whole tiles and k slices.  Kept rows bit for bit against the oracle, the other rows through the per-block
    checksums."""
    _need_gpu()
    M, P, kb, kr, K = case
    N = 8192
    g = torch.Generator(device=DEV).manual_seed(900 + M)
    x1 = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=DEV, generator=g)
    x2 = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=DEV, generator=g)
    s1 = torch.empty(M, device=DEV).uniform_(0.005, 0.02, generator=g)
    s2 = torch.empty(N, device=DEV).uniform_(0.001, 0.01, generator=g)
    peers = [torch.randn((kr, N), device=DEV, generator=g) for _ in range(P - 1)]
    need, f, blocks = ops.splitk_plan(M, K, N, P, kb, kr, n0=256)
    ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=DEV)
    cs = torch.zeros(blocks, dtype=torch.int64, device=DEV)
    out = ops.quant_matmul_splitk(x1, x2, s1, s2, None, peers, P, kb, kr, workspace=ws, checksum=cs, n0=256)
    torch.cuda.synchronize()
    acc_k, want = oracle.quant_matmul_reduce_scatter(x1[kb:kb + kr].cpu().numpy(), x2.cpu().numpy(), s1[kb:kb + kr].cpu().numpy(),
                                                     s2.cpu().numpy(), None, 0, kr, [p.cpu().numpy() for p in peers], oracle.BF16)
    assert np.array_equal(host16(out), want), "kept rows differ from the oracle"
    # rows that are not kept, per 128 x 128 block: exact through row sums of A against column blocks of B
    notkept = torch.ones(M, dtype=torch.float64, device=DEV)
    notkept[kb:kb + kr] = 0
    a_blocks = (x1.double() * notkept[:, None]).view(M // 128, 128, K).sum(1)            # [M/128, K]
    want_cs = (a_blocks @ x2.double()).view(M // 128, N // 128, 128).sum(2)              # [M/128, N/128]
    assert torch.equal(cs.view(M // 128, N // 128), want_cs.to(torch.int64))
    assert not ws[:65536].any()
    if f > 1:
        # the k slices were the library's own choice: a caller without a workspace gets the same tiles run whole, not an error
        cs2 = torch.zeros_like(cs)
        out2 = ops.quant_matmul_splitk(x1, x2, s1, s2, None, peers, P, kb, kr, workspace=None, checksum=cs2, n0=256)
        torch.cuda.synchronize()
        assert torch.equal(out2.view(torch.int16), out.view(torch.int16)) and torch.equal(cs2, cs)
        if M >= 256:      # (fewer rows take the split-K kernel by default, whose factor is SplitkMatmul's and needs its workspace)
            out3 = ops.quant_matmul_splitk(x1, x2, s1, s2, None, peers, P, kb, kr, workspace=None)   # the route the library picks by itself
            torch.cuda.synchronize()
            assert torch.equal(out3.view(torch.int16), out.view(torch.int16))
        with pytest.raises(L.CatcocError, match="workspace"):                                    # an explicit count insists
            ops.quant_matmul_splitk(x1, x2, s1, s2, None, peers, P, kb, kr, workspace=None, n0=256, split_k=f)


@pytest.mark.parametrize("case", [(256, 256, 64, 2, 0, 32, 1, False, False, True), (256, 512, 128, 8, 32, 32, 2, True, False, True),
                                  (384, 512, 192, 4, 96, 96, 3, False, True, False), (256, 512, 448, 16, 224, 32, 2, True, True, True),
                                  (512, 256, 1088, 8, 448, 64, 4, False, False, False), (256, 768, 320, 3, 64, 128, 1, True, False, False),
                                  (1024, 512, 832, 8, 128, 128, 0, False, False, False),
                                  (256, 256, 8192, 8, 32, 32, 1, True, False, False),      # 128 steps: A in pairs, B as [n,k]
                                  (256, 512, 16384, 4, 64, 64, 2, False, True, True)])     # two slices of 128 steps: A in pairs
def test_quant_explicit_kept_rows_eight_wave_ring_short_k_ranges(case):
    """Explicit kept rows on the 128x256 tiles at sizes where a workgroup's k range is shorter than the six-stage ring, odd, or
    unequal between the k slices (1 to 17 steps of 64), and two where it is long enough for A to be copied in pairs of steps:
    eight waves per workgroup, both layouts of B, fp32 and int32 peers at a
    row offset, with and without a dump of the accumulators (without one only the kept 32-row blocks travel between the
    slices).  Everything the launch writes against the oracle: accumulators, kept int32 block, output, checksums per
    128 x 128 block of the rows that are not kept."""
    _need_gpu()
    M, N, K, P, kb, kr, f, tb, ri, dump = case
    rng = np.random.default_rng(770 + M + K)
    x1 = rng.integers(-127, 128, (M, K), dtype=np.int8)
    x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s1 = rng.uniform(0.005, 0.02, M).astype(np.float32)
    s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.integers(-1000, 1000, N, dtype=np.int32)
    pro = 5
    peers = [rng.integers(-2 ** 24, 2 ** 24, (kr, N), dtype=np.int32) if ri else rng.standard_normal((kr, N)).astype(np.float32) for _ in range(P - 1)]
    staged = [np.concatenate([np.full((pro, N), 77, p.dtype), p]) for p in peers]
    acc_want, out_want = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, b, kb, kr, peers, oracle.BF16, reduce_int32=ri)
    need, fac, blocks = ops.splitk_plan(M, K, N, P, kb, kr, n0=256, split_k=f)
    assert blocks == (M // 128) * (N // 128) and (f == 0 or fac == f)
    ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=DEV)
    acc_dump = torch.full((M, N), -7, dtype=torch.int32, device=DEV) if dump else None
    c_accum = torch.full((kr, N), -7, dtype=torch.int32, device=DEV)
    checksum = torch.zeros(blocks, dtype=torch.int64, device=DEV)
    x2d = dev(np.ascontiguousarray(x2.T)) if tb else dev(x2)
    launch, out = ops.prepare_quant_matmul_splitk(dev(x1), x2d, dev(s1), dev(s2), dev(b), [dev(p) for p in staged], P, kb, kr, checksum=checksum,
                                                  acc_dump=acc_dump, c_accum=c_accum, trans_b=tb, reduce_int32=ri, n0=256, split_k=f,
                                                  workspace=ws, peer_row_offset=pro)
    keep = np.zeros(M, bool)
    keep[kb:kb + kr] = True
    want_cs = np.array([[acc_want[mi * 128:(mi + 1) * 128, ni * 128:(ni + 1) * 128].astype(np.int64)[~keep[mi * 128:(mi + 1) * 128]].sum()
                         for ni in range(N // 128)] for mi in range(M // 128)])
    for it in range(2):   # (twice: the counters of the k slices go back to zero)
        out.zero_()
        checksum.zero_()
        launch()
        L.check()
        torch.cuda.synchronize()
        if dump:
            assert np.array_equal(acc_dump.cpu().numpy(), acc_want), "int32 accumulators differ from the oracle"
        assert np.array_equal(c_accum.cpu().numpy(), acc_want[kb:kb + kr] + (sum(peers) if ri else 0)), "kept int32 block differs"
        assert np.array_equal(host16(out), out_want), "kept rows differ from the oracle"
        assert np.array_equal(checksum.cpu().numpy().reshape(M // 128, N // 128), want_cs)
    assert not ws[:65536].any()


# ------------------------------------------------------- C ABI from a plain C++ host
def test_launches_replay_from_a_hip_graph():
    # serving loops capture their launches: the library allocates nothing and never synchronises, the split-K path
    # re-arms its counters inside the kernel, so a captured launch replays; every replay must equal the eager result
    _need_gpu()
    g = torch.Generator(device=DEV).manual_seed(5)
    M, K, N, P = 1024, 512, 512, 4
    x1 = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=DEV, generator=g)
    x2 = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=DEV, generator=g)
    s1 = torch.empty(M, device=DEV).uniform_(0.005, 0.02, generator=g)
    s2 = torch.empty(N, device=DEV).uniform_(0.001, 0.01, generator=g)
    peers = [torch.randn((M // P, N), device=DEV, generator=g) for _ in range(P - 1)]
    big, out_big = ops.prepare_quant_matmul_reduce_scatter(x1, x2, s1, s2, None, peers, 1, P)
    xs = torch.randint(-127, 128, (16, 2048), dtype=torch.int8, device=DEV, generator=g)
    w = torch.randint(-127, 128, (2048, 512), dtype=torch.int8, device=DEV, generator=g)
    ss = torch.empty(16, device=DEV).uniform_(0.005, 0.02, generator=g)
    pk = [torch.randn((2, N), device=DEV, generator=g) for _ in range(P - 1)]
    need, fac, tiles = ops.splitk_plan(16, 2048, 512, P, 4, 2, split_k=4)
    assert fac == 4
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    small, out_small = ops.prepare_quant_matmul_splitk(xs, w, ss, s2, None, pk, P, 4, 2, split_k=4, workspace=ws)
    # the same rows against the weights stored as [n,k]: whole k per column strip, no workspace at all
    strips, out_strips = ops.prepare_quant_matmul_splitk(xs, w.t().contiguous(), ss, s2, None, pk, P, 4, 2, trans_b=True)
    # a launch of 512 tiles with split kept tiles, whose waiting tiles run as halves: their checksum halves meet through
    # the counter block of a workspace and clear it again
    xh = torch.randint(-127, 128, (4096, 128), dtype=torch.int8, device=DEV, generator=g)
    wh = torch.randint(-127, 128, (128, 4096), dtype=torch.int8, device=DEV, generator=g)
    sh1 = torch.empty(4096, device=DEV).uniform_(0.005, 0.02, generator=g)
    sh2 = torch.empty(4096, device=DEV).uniform_(0.001, 0.01, generator=g)
    ph = [torch.randn((512, 4096), device=DEV, generator=g) for _ in range(7)]
    csh = torch.zeros(512, dtype=torch.int64, device=DEV)
    wsh = torch.zeros(65536, dtype=torch.uint8, device=DEV)
    halves, out_halves = ops.prepare_quant_matmul_reduce_scatter(xh, wh, sh1, sh2, None, ph, 3, 8, checksum=csh, workspace=wsh)
    # explicit kept rows on the 128x256 tiles in two k slices: the eight-wave ring, whose slices meet through tile counters
    xr = torch.randint(-127, 128, (256, 2048), dtype=torch.int8, device=DEV, generator=g)
    sr1 = torch.empty(256, device=DEV).uniform_(0.005, 0.02, generator=g)
    pr = [torch.randn((32, N), device=DEV, generator=g) for _ in range(P - 1)]
    need_r, fac_r, _ = ops.splitk_plan(256, 2048, N, P, 32, 32, n0=256, split_k=2)
    assert fac_r == 2
    wsr = torch.zeros(need_r, dtype=torch.uint8, device=DEV)
    ring, out_ring = ops.prepare_quant_matmul_splitk(xr, w, sr1, s2, None, pr, P, 32, 32, split_k=2, workspace=wsr, n0=256)
    # the round-pipelined W8A8 operator (three comm rounds on two streams) with its events in a plan of the caller's: the call
    # then creates nothing, and the second stream joins the capture through the plan's events
    ipeers = [torch.randint(-2 ** 20, 2 ** 20, (M // P, N), dtype=torch.int32, device=DEV, generator=g) for _ in range(P - 1)]
    tp = ops.default_tiling(M, K, N, P, m0=128, n0=256, k0=256, commInterval=1)
    rounds = ops.pipelined_round_count(L.QUANT_MATMUL_REDUCE_SCATTER, tp, 1, P, block_num=8)
    assert rounds == 2
    plan = ops.PipelinedPlan(rounds)
    obp = _outbound_for(L.QUANT_MATMUL_REDUCE_SCATTER, L.INT8, tp, 1, P, torch.int32)
    out_pipe = torch.zeros((M // P, N), dtype=torch.bfloat16, device=DEV)
    cacc_pipe = torch.zeros((M // P, N), dtype=torch.int32, device=DEV)
    comm = torch.cuda.Stream()

    def pipe():
        ops.pipelined_quant_matmul_reduce_scatter(x1, x2, s1, s2, None, ipeers, 1, P, obp, c_accum=cacc_pipe, tiling=tp, comm_stream=comm,
                                                  block_num=8, out=out_pipe, plan=plan)
    big(); small(); strips(); halves(); ring(); pipe(); L.check()
    torch.cuda.synchronize()
    want_big, want_small, want_halves, want_cs = out_big.clone(), out_small.clone(), out_halves.clone(), csh.clone()
    want_ring = out_ring.clone()
    _, ring_oracle = oracle.quant_matmul_reduce_scatter(xr[32:64].cpu().numpy(), w.cpu().numpy(), sr1[32:64].cpu().numpy(), s2.cpu().numpy(),
                                                        None, 0, 32, [p.cpu().numpy() for p in pr], oracle.BF16)
    assert np.array_equal(host16(want_ring), ring_oracle)
    assert torch.equal(out_strips, want_small), "the two weight layouts give the same rows"
    want_pipe, want_cacc = out_pipe.clone(), cacc_pipe.clone()
    fused = ops.quant_matmul_reduce_scatter(x1, x2, s1, s2, None, ipeers, 1, P, reduce_int32=True)
    assert torch.equal(fused.view(torch.int16), want_pipe.view(torch.int16))
    with pytest.raises(L.CatcocError, match="plan holds events for"):
        ops.pipelined_quant_matmul_reduce_scatter(x1, x2, s1, s2, None, ipeers, 1, P, obp, c_accum=cacc_pipe, tiling=tp, comm_stream=comm,
                                                  block_num=4, out=out_pipe, plan=plan)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        big(); small(); strips(); halves(); ring(); pipe()     # warm the side stream before capture
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            out_big.zero_()
            out_small.zero_()
            out_strips.zero_()
            out_halves.zero_()
            out_ring.zero_()
            csh.zero_()
            big()
            small()
            strips()
            halves()
            ring()
            pipe()
    L.check()
    for _ in range(3):
        out_big.fill_(1.0)                   # eager work between the replays
        out_small.fill_(1.0)
        out_strips.fill_(1.0)
        out_halves.fill_(1.0)
        out_ring.fill_(1.0)
        out_pipe.fill_(1.0)
        cacc_pipe.fill_(3)
        csh.fill_(7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_big, want_big) and torch.equal(out_small, want_small) and torch.equal(out_strips, want_small)
        assert torch.equal(out_halves, want_halves) and torch.equal(csh, want_cs)
        assert torch.equal(out_ring, want_ring) and not wsr[:65536].any()
        assert torch.equal(out_pipe, want_pipe) and torch.equal(cacc_pipe, want_cacc)
        assert not ws[:65536].any(), "tile counters were not re-armed"
        assert not wsh.any(), "the words the checksum halves meet through were not cleared"
    plan.close()


def test_cpp_host_drives_the_library_through_the_c_abi(tmp_path):
    # the stand-alone host (no Python, no torch in the process) reads the reference's raw .bin files, launches
    # catcoc_quant_matmul_reduce_scatter and writes this rank's block of output.bin at its offset
    _need_gpu()
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(L.LIB_PATH), "catcoc_quant_rs_host")
    assert os.path.exists(exe), "build the package first (python -m mm_rs_with_catlass_amd._build)"
    M, N, K, P, rank = 1024, 512, 256, 4, 2
    rng = np.random.default_rng(77)
    x1 = rng.integers(-127, 128, (M, K), dtype=np.int8)
    x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s1 = rng.uniform(0.005, 0.02, M).astype(np.float32)
    s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.integers(-1000, 1000, N, dtype=np.int32)
    rows = M // P
    peers = [rng.standard_normal((rows, N)).astype(np.float32) for _ in range(P - 1)]
    for name, arr in (("x1_gm", x1), ("x2_gm", x2), ("scale_x1_gm", s1), ("scale_x2_gm", s2), ("bias_gm", b)):
        arr.tofile(tmp_path / (name + ".bin"))
    for i, p in enumerate(peers):
        p.tofile(tmp_path / ("peer_%d.bin" % i))
    r = subprocess.run([exe, str(P), str(rank), str(M), str(N), str(K), str(tmp_path)], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr + r.stdout
    _, want = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, b, rank * rows, rows, peers, oracle.BF16, want_acc=False)
    got = np.fromfile(tmp_path / "output.bin", dtype=np.uint16)
    assert got.size == (rank + 1) * rows * N
    assert np.array_equal(got[rank * rows * N:].reshape(rows, N), want)
    assert not got[:rank * rows * N].any()
    # a rejected launch is reported, not executed
    r = subprocess.run([exe, str(P), str(rank), str(M), str(N), str(K), str(tmp_path / "missing")], capture_output=True, text=True, timeout=100)
    assert r.returncode == 1 and "cannot read" in r.stderr


def test_bench_prints_one_json_line_with_roofline():
    # the measurement contract: one JSON line, whole-job throughput, the roofline object of the dominant kernel
    _need_gpu()
    import json
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--steps", "3", "--warmup", "1", "--no-cpu", "--sustained", "40"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["unit"] == "TOPS" and d["vs_baseline"] is None and d["dtype"] == "int8"
    assert "workload" in d["config"] and d["config"]["parity_sample_ok"] is True
    rf = d["roofline"]
    assert rf["bound"] == "mfma" and rf["peak"] == 5000.0 and abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3
    assert 100.0 < d["value"] < 5000.0
    assert rf["kernel_us_sustained"] > 0 and len(rf["sustained_series_us"]) == 10 and rf["kernel_us_avg_same_buffers"] > 0
    ob = d["outbound"]          # the reference's store mode rides along as a secondary object
    assert ob["kept_block_equals_main_mode"] is True and ob["TOPS"] > 100.0 and ob["algorithmic_bytes"] > rf["algorithmic_bytes"]
