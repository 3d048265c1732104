"""CPU tests that pin the oracle (oracle/catcoc_oracle.c).

Each oracle function is checked against something it did not come from:
the reference's own golden / scheduler code compiled from source (oracle/_ref,
only where the reference tree is present), fixtures that build emitted
(tests/golden/sched_fixtures.json), numpy, brute force, and closed forms.
"""
import ctypes as C
import json
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
REF_G = oracle.ref_golden()
REF_S = oracle.ref_sched()
needs_ref_golden = pytest.mark.skipif(REF_G is None, reason="oracle/_ref golden not built (no reference tree)")
needs_ref_sched = pytest.mark.skipif(REF_S is None, reason="oracle/_ref scheduler not built (no reference tree)")
u32 = C.c_uint32


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


# ------------------------------------------------------------------ rounding
def test_bf16_round_matches_bit_trick_and_ties():
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(100.0),
        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, -3.3895314e38, np.inf, -np.inf,
                  1e-40, 65504.0], np.float32),
    ])
    got = oracle.f32_to_half(x, oracle.BF16)
    # independent statement: nearest of the two neighbouring bf16 values, ties to even mantissa
    u = x.view(np.uint32).astype(np.uint64)
    lo = (u >> 16) << 16
    hi = lo + (1 << 16)
    rem = u - lo
    pick_hi = (rem > 0x8000) | ((rem == 0x8000) & (((lo >> 16) & 1) == 1))
    want = np.where(pick_hi, hi, lo) >> 16
    assert np.array_equal(got.astype(np.uint64), want)
    # exact ties: 1 + 2^-8 -> 1.0 (even), 1 + 3*2^-8 -> 1 + 2^-6
    assert oracle.f32_to_half(np.array([1.00390625], np.float32), oracle.BF16)[0] == 0x3F80
    assert oracle.f32_to_half(np.array([1.01171875], np.float32), oracle.BF16)[0] == 0x3F82
    assert oracle.f32_to_half(np.array([np.nan], np.float32), oracle.BF16)[0] == 0x7FC0


@needs_ref_golden
def test_bf16_round_matches_reference_bfloat16_h():
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(5000) * 10.0 ** rng.integers(-6, 6, 5000)).astype(np.float32)
    got = oracle.f32_to_half(x, oracle.BF16)
    want = np.array([REF_G.ref_round_to_bf16(C.c_float(float(v))) for v in x], np.uint16)
    assert np.array_equal(got, want)


def test_fp16_round_matches_numpy_everywhere():
    # every finite fp16 value round-trips, and every midpoint between neighbours rounds like numpy
    allh = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    f = allh.view(np.float16).astype(np.float32)
    back = oracle.half_to_f32(allh, oracle.FP16)
    fin = np.isfinite(f)
    assert np.array_equal(back[fin].view(np.uint32), f[fin].view(np.uint32))
    assert np.array_equal(oracle.f32_to_half(f[fin], oracle.FP16), allh[fin])
    pos = np.arange(0x0000, 0x7C00, dtype=np.uint16)
    a = pos.view(np.float16).astype(np.float64)
    b = (pos + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    b[-1] = 65536.0  # neighbour above the largest finite value
    mid = ((a + b) / 2).astype(np.float32)
    pts = np.concatenate([mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf))])
    pts = np.concatenate([pts, -pts])
    with np.errstate(over="ignore"):
        want = pts.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_half(pts, oracle.FP16), want)
    rng = np.random.default_rng(3)
    r = (rng.standard_normal(50000) * 10.0 ** rng.integers(-9, 6, 50000)).astype(np.float32)
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.f32_to_half(r, oracle.FP16), r.astype(np.float16).view(np.uint16))


# ----------------------------------------------------------------- int8 GEMM
def test_gemm_i8_brute_force_and_numpy():
    rng = np.random.default_rng(4)
    for (M, N, K) in [(1, 1, 1), (3, 5, 7), (17, 33, 129), (64, 96, 300)]:
        A = rng.integers(-128, 128, (M, K), dtype=np.int8)
        B = rng.integers(-128, 128, (K, N), dtype=np.int8)
        bias = rng.integers(-1000, 1000, N, dtype=np.int32)
        want = A.astype(np.int64) @ B.astype(np.int64)
        assert np.array_equal(oracle.gemm_i8_i32(A, B), want.astype(np.int32))
        assert np.array_equal(oracle.gemm_i8_i32_literal(A, B), want.astype(np.int32))
        assert np.array_equal(oracle.gemm_i8_i32(A, B, bias=bias), (want + bias).astype(np.int32))
        assert np.array_equal(oracle.gemm_i8_i32(A, np.ascontiguousarray(B.T), transB=True), want.astype(np.int32))
    # a transposed operand or a dropped k fails these: asymmetric one-hot inputs
    A = np.zeros((4, 6), np.int8); A[1, 5] = 3
    B = np.zeros((6, 5), np.int8); B[5, 2] = -7
    out = oracle.gemm_i8_i32(A, B)
    assert out[1, 2] == -21 and np.count_nonzero(out) == 1


def test_gemm_i8_extreme_values_do_not_overflow_int32():
    K = 1792
    A = np.full((2, K), -128, np.int8)
    B = np.full((K, 3), -128, np.int8)
    assert np.all(oracle.gemm_i8_i32(A, B) == K * 16384)


@needs_ref_golden
def test_quant_golden_matches_reference_matmul_hpp():
    rng = np.random.default_rng(5)
    M, N, K = 37, 53, 301
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s_n = rng.uniform(0.001, 0.01, N).astype(np.float32)
    s_m = rng.uniform(0.005, 0.02, M).astype(np.float32)
    want = np.empty((M, N), np.float32)
    REF_G.ref_quant_matmul(u32(M), u32(N), u32(K), _p(A), _p(B), _p(s_n), _p(s_m), _p(want))
    got = oracle.dequant(oracle.gemm_i8_i32(A, B), s_n, s_m)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    bias = rng.integers(-50, 50, N, dtype=np.int32)
    wb = np.empty((M, N), np.int32)
    REF_G.ref_compute_matmul_bias_i8(u32(M), u32(N), u32(K), _p(A), _p(B), _p(bias), _p(wb))
    assert np.array_equal(oracle.gemm_i8_i32(A, B, bias=bias), wb)


def test_dequant_order_and_rounding():
    # float(acc) must round to nearest even above 2^24, per-channel scale is applied first
    acc = np.array([[2 ** 24 + 1, 2 ** 24 + 3, -(2 ** 25 + 6), 123456789]], np.int32)
    s_n = np.array([0.1, 0.3, 0.007, 0.0123], np.float32)
    s_m = np.array([0.77], np.float32)
    got = oracle.dequant(acc, s_n, s_m)
    want = (acc.astype(np.float32) * s_n[None, :]) * s_m[:, None]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert acc.astype(np.float32)[0, 0] == np.float32(2 ** 24) and acc.astype(np.float32)[0, 1] == np.float32(2 ** 24 + 4)
    # the other order differs somewhere on random data: the test would notice a swap
    rng = np.random.default_rng(6)
    acc = rng.integers(-3 * 10 ** 7, 3 * 10 ** 7, (64, 64), dtype=np.int32)
    s_n = rng.uniform(0.001, 0.01, 64).astype(np.float32)
    s_m = rng.uniform(0.005, 0.02, 64).astype(np.float32)
    a = oracle.dequant(acc, s_n, s_m)
    other = (acc.astype(np.float32) * s_m[:, None]) * s_n[None, :]
    assert np.array_equal(a.view(np.uint32), ((acc.astype(np.float32) * s_n[None, :]) * s_m[:, None]).view(np.uint32))
    assert not np.array_equal(a.view(np.uint32), other.view(np.uint32))


def test_quant_debug_mode_closed_form():
    # examples/utils/gen_quant_data.py:10-16,43-52 debug data: all-ones int8, scales 0.01, bias 1..N.
    # Every rank contributes (K + j + 1) * 0.01 * 0.01, so P identical partials sum to P times that.
    M, N, K, P = 16, 40, 128, 4
    x1 = np.ones((M, K), np.int8)
    x2 = np.ones((K, N), np.int8)
    s1 = np.full(M, 0.01, np.float32)
    s2 = np.full(N, 0.01, np.float32)
    bias = np.arange(1, N + 1, dtype=np.int32)
    rows = M // P
    acc, _ = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, bias, 0, rows, [], oracle.FP16)
    assert np.array_equal(acc, np.broadcast_to(K + bias, (M, N)))
    part = oracle.dequant(acc[:rows], s2, s1[:rows])
    _, out = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, bias, 0, rows, [part] * (P - 1), oracle.FP16)
    got = oracle.half_to_f32(out, oracle.FP16)
    want = P * (K + bias).astype(np.float64) * 1e-4
    assert np.allclose(got, np.broadcast_to(want, (rows, N)), rtol=2 ** -10, atol=0)
    # reference order (int32 reduce first) gives the same closed form
    _, out2 = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, bias, 0, rows, [acc[:rows]] * (P - 1), oracle.FP16,
                                                 reduce_int32=True)
    assert np.allclose(oracle.half_to_f32(out2, oracle.FP16), np.broadcast_to(want, (rows, N)), rtol=2 ** -10, atol=0)


def test_reduce_cast_order_is_local_then_peers_ascending():
    # fp32 addition is not associative: 1e8 + 1 - 1e8 depends on the order
    local = np.array([[1.0e8]], np.float32)
    peers = [np.array([[1.0]], np.float32), np.array([[-1.0e8]], np.float32), np.array([[0.5]], np.float32)]
    out = oracle.half_to_f32(oracle.reduce_cast(local, peers, oracle.BF16), oracle.BF16)
    want = np.float32(np.float32(np.float32(np.float32(1.0e8) + np.float32(1.0)) + np.float32(-1.0e8)) + np.float32(0.5))
    assert out[0, 0] == oracle.half_to_f32(oracle.f32_to_half(np.array([want]), oracle.BF16), oracle.BF16)[0]
    assert want == np.float32(0.5)
    # peer_row0 selects the row of a taller peer buffer
    local = np.zeros((2, 3), np.float32)
    peer = np.arange(15, dtype=np.float32).reshape(5, 3)
    out = oracle.half_to_f32(oracle.reduce_cast(local, [peer], oracle.FP16, peer_row0=2), oracle.FP16)
    assert np.array_equal(out, peer[2:4])


# ---------------------------------------------------------------- float GEMM
def _rand_half(rng, shape, dtype, scale=1.0):
    return oracle.f32_to_half((rng.standard_normal(shape) * scale).astype(np.float32), dtype)


@pytest.mark.parametrize("dtype", [oracle.FP16, oracle.BF16])
def test_gemm_half_is_k_sequential_fp32(dtype):
    rng = np.random.default_rng(7)
    M, N, K = 9, 11, 200
    A = _rand_half(rng, (M, K), dtype)
    B = _rand_half(rng, (K, N), dtype)
    got = oracle.gemm_half_f32(A, B, dtype)
    Af, Bf = oracle.half_to_f32(A, dtype), oracle.half_to_f32(B, dtype)
    want = np.zeros((M, N), np.float32)
    for k in range(K):  # numpy float32 ops round once per op: the same sequence
        want = want + Af[:, k:k + 1] * Bf[k:k + 1, :]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # layouts
    assert np.array_equal(oracle.gemm_half_f32(A, np.ascontiguousarray(B.T), dtype, transB=True), got)
    assert np.array_equal(oracle.gemm_half_f32(np.ascontiguousarray(A.T), B, dtype, transA=True), got)
    # identity B returns A exactly; all-ones A gives column sums of powers of two exactly
    eye = oracle.f32_to_half(np.eye(K, dtype=np.float32), dtype)
    assert np.array_equal(oracle.gemm_half_f32(A, eye, dtype), Af)
    pw = oracle.f32_to_half(np.float32(2.0) ** rng.integers(-3, 4, (K, N)).astype(np.float32), dtype)
    ones = oracle.f32_to_half(np.ones((M, K), np.float32), dtype)
    assert np.array_equal(oracle.gemm_half_f32(ones, pw, dtype),
                          np.broadcast_to(oracle.half_to_f32(pw, dtype).astype(np.float64).sum(0), (M, N)).astype(np.float32))


@needs_ref_golden
def test_gemm_half_matches_reference_compute_matmul():
    rng = np.random.default_rng(8)
    M, N, K = 21, 19, 333
    for dtype in (oracle.FP16, oracle.BF16):
        A = _rand_half(rng, (M, K), dtype)
        B = _rand_half(rng, (K, N), dtype, 0.02)
        Af, Bf = oracle.half_to_f32(A, dtype), oracle.half_to_f32(B, dtype)
        want = np.empty((M, N), np.float32)
        REF_G.ref_compute_matmul_f32(u32(M), u32(N), u32(K), _p(Af), _p(Bf), _p(want))
        got = oracle.gemm_half_f32(A, B, dtype)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    A = _rand_half(rng, (M, K), oracle.BF16)
    B = _rand_half(rng, (K, N), oracle.BF16)
    want = np.empty((M, N), np.float32)
    REF_G.ref_compute_matmul_bf16(u32(M), u32(N), u32(K), _p(A), _p(B), _p(want))
    assert np.array_equal(oracle.gemm_half_f32(A, B, oracle.BF16).view(np.uint32), want.view(np.uint32))


def test_allreduce_config1_split_k_partials():
    # BASELINE config 1 at reduced size: K split into 2 contiguous halves as rank partials
    rng = np.random.default_rng(9)
    M, N, K = 32, 48, 256
    A = oracle.f32_to_half(rng.uniform(-1, 1, (M, K)).astype(np.float32), oracle.FP16)
    B = oracle.f32_to_half(rng.uniform(-1, 1, (K, N)).astype(np.float32), oracle.FP16)
    p0 = oracle.gemm_half_f32(A[:, :K // 2], B[:K // 2], oracle.FP16)
    p1 = oracle.gemm_half_f32(A[:, K // 2:], B[K // 2:], oracle.FP16)
    _, out = oracle.matmul_reduce(np.ascontiguousarray(A[:, :K // 2]), B[:K // 2], oracle.FP16, 0, M, [p1])
    want = oracle.f32_to_half(p0 + p1, oracle.FP16)
    assert np.array_equal(out, want)
    full = oracle.half_to_f32(A, oracle.FP16).astype(np.float64) @ oracle.half_to_f32(B, oracle.FP16).astype(np.float64)
    ok, bad, eb = oracle.verify(oracle.half_to_f32(out, oracle.FP16), full.astype(np.float32), oracle.FP16, K)
    assert ok, (bad, eb)


def test_allgather_matmul_matches_concatenation():
    rng = np.random.default_rng(10)
    P, ml, K, N = 4, 6, 64, 10
    shards = [_rand_half(rng, (ml, K), oracle.BF16) for _ in range(P)]
    B = _rand_half(rng, (K, N), oracle.BF16, 0.02)
    out = oracle.allgather_matmul(shards, B, oracle.BF16)
    cat = np.concatenate(shards, 0)
    want = oracle.f32_to_half(oracle.gemm_half_f32(cat, B, oracle.BF16), oracle.BF16)
    assert np.array_equal(out, want)


# ---------------------------------------------------------------- schedulers
with open(os.path.join(HERE, "golden", "sched_fixtures.json")) as _f:
    FX = json.load(_f)


def test_swizzle_matches_reference_fixtures():
    for case in FX["swizzle"]:
        M, N, m0, n0 = case["M"], case["N"], case["m0"], case["n0"]
        lm, ln = -(-M // m0), -(-N // n0)
        assert len(case["coords"]) == lm * ln
        seen = set()
        area = 0
        for t, (m, n, ma, na) in enumerate(case["coords"]):
            assert oracle.swizzle_block_coord(case["off"], case["dir"], lm, ln, t) == (m, n)
            assert oracle.swizzle_actual_shape(M, N, m0, n0, m, n) == (ma, na)
            seen.add((m, n))
            area += ma * na
        assert len(seen) == lm * ln and area == M * N  # bijection onto the grid, shapes tile the matrix


def test_swizzle_serpentine_closed_form():
    # direction 1, offset 7 on a 8x16 grid: band 0 = columns 0..6 walking n fastest, m ascending;
    # band 1 = columns 7..13 with m descending; last band has 2 columns.
    lm, ln = 8, 16
    assert [oracle.swizzle_block_coord(7, 1, lm, ln, t) for t in range(8)] == \
        [(0, 0), (0, 1), (0, 2), (0, 3), (0, 4), (0, 5), (0, 6), (1, 0)]
    assert oracle.swizzle_block_coord(7, 1, lm, ln, 56) == (7, 7)      # first task of odd band starts at the bottom
    assert oracle.swizzle_block_coord(7, 1, lm, ln, 56 + 7) == (6, 7)
    assert oracle.swizzle_block_coord(7, 1, lm, ln, 112) == (0, 14)    # last band: 2 columns
    assert oracle.swizzle_block_coord(7, 1, lm, ln, 113) == (0, 15)
    assert oracle.swizzle_block_coord(7, 1, lm, ln, 114) == (1, 14)
    assert oracle.swizzle_block_coord(7, 1, lm, ln, 128 + 5) == (0, 5)  # wraps modulo coreLoops


@needs_ref_sched
def test_swizzle_matches_reference_live_random_grids():
    rng = np.random.default_rng(11)
    o = (u32 * 5)()
    for _ in range(60):
        off = int(rng.choice([1, 2, 3, 4, 7]))
        d = int(rng.integers(0, 2))
        M, N = int(rng.integers(1, 3000)), int(rng.integers(1, 5000))
        m0, n0 = int(rng.choice([16, 64, 128, 256])), int(rng.choice([128, 256]))
        lm, ln = -(-M // m0), -(-N // n0)
        for t in rng.integers(0, 2 * lm * ln, 25):
            REF_S.ref_swizzle_coord(u32(off), u32(d), u32(M), u32(N), u32(m0), u32(n0), u32(int(t)), o)
            assert oracle.swizzle_block_coord(off, d, lm, ln, int(t)) == (o[0], o[1])
            assert oracle.swizzle_actual_shape(M, N, m0, n0, o[0], o[1]) == (o[2], o[3])


def test_splitk_matches_reference_fixtures():
    for case in FX["splitk"]:
        M, N, K, m0, n0, k0, f = (case[k] for k in ("M", "N", "K", "m0", "n0", "k0", "f"))
        lm, ln, kt = -(-M // m0), -(-N // n0), -(-K // k0)
        cover = {}
        for t, (m, n, k, s, ma, na, ka) in enumerate(case["coords"]):
            assert oracle.splitk_block_coord(case["off"], case["dir"], lm, ln, kt, f, t) == (m, n, k, s)
            assert oracle.splitk_actual_k(K, k0, f, s) == ka
            cover.setdefault((m, n), []).append((k * k0, ka))
        for segs in cover.values():  # slices of a tile partition [0,K) in order
            segs.sort()
            pos = 0
            for start, ln_ in segs:
                assert start == pos
                pos += ln_
            assert pos == K


def test_splitk_factor_hand_cases():
    # 3rdparty/catlass/include/catlass/gemm/kernel/splitk_matmul.hpp:219-265, worked by hand:
    # M=16,N=K=8192, tile 128x256x256: 32 base tiles, cap 16 (k>4096).
    assert oracle.splitk_factor(16, 8192, 8192, 20, 128, 256, 256) == 1     # 20/32 = 0 -> 1; 32 >= 20 cores
    assert oracle.splitk_factor(16, 8192, 8192, 256, 128, 256, 256) == 8    # min(256/32, 16)
    assert oracle.splitk_factor(512, 8192, 8192, 256, 128, 256, 256) == 2   # 128 tiles -> 2; 3 would add a wave
    assert oracle.splitk_factor(128, 256, 1024, 20, 128, 256, 256) == 2     # 1 tile, cap 2 (k<=1024)
    assert oracle.splitk_factor(128, 256, 2048, 20, 128, 256, 256) == 4     # cap 4
    assert oracle.splitk_factor(128, 256, 512, 20, 128, 256, 256) == 2      # cap 2, k tiles 2
    assert oracle.splitk_factor(128, 256, 256, 20, 128, 256, 256) == 1      # only one k tile
    assert oracle.splitk_factor(4096, 4096, 9000, 20, 128, 256, 256) == 2   # k>8192 forces 2
    assert oracle.splitk_factor(4096, 4096, 40000, 20, 128, 256, 256) == 4  # k>32768 forces 4
    # growth loop: 6 tiles on 20 cores, k=4096 (cap 8): 20/6=3, then 4..8 keep one wave? ceil(6f/20) >= f only while false
    assert oracle.splitk_factor(128 * 6, 256, 4096, 20, 128, 256, 256) == 3


def test_allgather_swizzle_matches_reference_fixtures():
    for case in FX["allgather"]:
        P, ci, ml, N, m0, n0 = (case[k] for k in ("P", "commInterval", "mLocal", "N", "m0", "n0"))
        lmr, ln = -(-ml // m0), -(-N // n0)
        assert len(case["coords"]) == lmr * P * ln
        seen = set()
        for t, (m, n, ma, na) in enumerate(case["coords"]):
            assert oracle.allgather_block_coord(case["off"], case["dir"], P, ci, lmr, ln, t) == (m, n)
            assert oracle.swizzle_actual_shape(ml, N, m0, n0, m % lmr, n) == (ma, na)
            seen.add((m, n))
        assert len(seen) == lmr * P * ln


def test_comm_swizzle_hand_cases_and_invariants():
    # include/catcoc/comm_epilogue/block/comm_block_swizzle.hpp:147-186, worked by hand for
    # P=8, coreSplit (20,1) (the quant example), 50 data loops per rank, direction 0:
    # swizzleOffset = 20, nStride = 8; tasks 0..19 walk dataIdx 0..19 with the rank rotated by dataIdx.
    P, sr, sc, dl = 8, 20, 1, 50
    got = [oracle.comm_block_idx(0, P, sr, sc, dl, t) for t in range(22)]
    assert got[:9] == [(0, 0), (1, 1), (2, 2), (3, 3), (4, 4), (5, 5), (6, 6), (7, 7), (8, 0)]
    assert got[20] == (0, 1) and got[21] == (1, 2)     # next rank step: (1*8)%8 + (1*8)/8 = 1, plus dataIdx
    # last band has 10 rows: task 2*160 .. : band 2 -> dataIdx 40..49
    assert oracle.comm_block_idx(0, P, sr, sc, dl, 320) == (40, 0)
    assert oracle.comm_block_idx(0, P, sr, sc, dl, 330) == (40, 1)
    for (d, P, sr, sc, dl) in [(0, 8, 20, 1, 50), (0, 8, 16, 1, 7), (0, 4, 2, 2, 9), (1, 8, 4, 2, 13), (1, 2, 3, 1, 5),
                               (0, 8, 10, 2, 25)]:
        pairs = [oracle.comm_block_idx(d, P, sr, sc, dl, t) for t in range(dl * P)]
        assert len(set(pairs)) == dl * P                               # bijection onto data x rank
        assert all(0 <= a < dl and 0 <= b < P for a, b in pairs)
        assert oracle.comm_block_idx(d, P, sr, sc, dl, dl * P + 3) == pairs[3]
    assert oracle.lib().oracle_comm_block_row(u32(3), u32(5), u32(50), u32(64)) == 3 * 50 * 64 + 5 * 64


def test_rs_task_schedule_config4():
    # W8A8 benchmark config with the reference launch (20 cores, commInterval 10, 128x256 tiles, P=8):
    # 8x16 tiles per rank, 1024 tasks, 200 per round (25 per rank), 6 rounds, last round 24 (3 per rank).
    M, N, P = 8192, 4096, 8
    args = (M, N, P, 128, 256, 20, 10, 2)
    seen = set()
    for t in range(1024):
        tr, mi, ni, row, col, ws = oracle.rs_task(*args, t)
        assert row == tr * 1024 + mi * 128 and col == ni * 256
        seen.add((row, col))
        rnd, b = divmod(t, 200)
        assert ws == ((rnd % 2) * 200 + b) * 128
        per = 25 if rnd < 5 else 3
        assert tr == b // per
        assert (mi, ni) == oracle.swizzle_block_coord(7, 1, 8, 16, rnd * 25 + b % per)
    assert len(seen) == 1024 and oracle.rs_task(*args, 1024) is None
    assert oracle.rs_task(*args, 0)[:3] == (0, 0, 0) and oracle.rs_task(*args, 25)[:3] == (1, 0, 0)
    assert oracle.rs_task(*args, 200)[:3] == (0, 3, 4)  # loopIdxInRank 25 -> (25 // 7, 25 % 7)


def test_ar_task_hand_worked_cases():
    # include/catcoc/dgemm/kernel/matmul_allreduce.hpp:146-179 worked by hand.
    # (a) BASELINE config 1 with the reference launch: 512x1024 in 128x256 tiles = 4x4 tiles, 20 cores x
    # commInterval 3 = 60 tiles per round, so all 16 tasks are round 0 / stage 0 and tile t sits at workspace
    # row t*128; swizzle <7,1> on 4 tile columns is a single (last, narrower) band of width 4: task -> (t/4, t%4).
    for t in range(16):
        assert oracle.ar_task(512, 1024, 128, 256, 20, 3, 2, t) == (t // 4, t % 4, t * 128)
    assert oracle.ar_task(512, 1024, 128, 256, 20, 3, 2, 16) is None
    # (b) several rounds and a narrow reversed last band: 512x2304 -> 4x9 tiles, 5 cores x commInterval 2 = 10
    # tiles per round, 2 stages.  Band 0 = tile columns 0..6 (28 tasks, n fastest); band 1 = columns 7,8 with
    # the tile rows walked backwards.
    args = (512, 2304, 128, 256, 5, 2, 2)
    assert oracle.ar_task(*args, 0) == (0, 0, 0)
    assert oracle.ar_task(*args, 9) == (1, 2, 9 * 128)                   # round 0, b = 9
    assert oracle.ar_task(*args, 17) == (2, 3, (10 + 7) * 128)           # round 1 -> stage 1, b = 7
    assert oracle.ar_task(*args, 23) == (3, 2, 3 * 128)                  # round 2 -> stage 0 again, b = 3
    assert oracle.ar_task(*args, 28) == (3, 7, (0 + 8) * 128)            # first task of the reversed band
    assert oracle.ar_task(*args, 29) == (3, 8, (0 + 9) * 128)
    assert oracle.ar_task(*args, 30) == (2, 7, (10 + 0) * 128)           # round 3 -> stage 1
    assert oracle.ar_task(*args, 35) == (0, 8, (10 + 5) * 128)
    assert oracle.ar_task(*args, 36) is None
    assert len({oracle.ar_task(*args, t)[:2] for t in range(36)}) == 36


def test_splitk_slices_hand_worked_case():
    # block_swizzle.hpp:151-158,220-235 by hand: 9 k tiles over 4 slices -> the FIRST 9 % 4 = 1 slice owns one
    # extra tile: slices start at k tiles 0, 3, 5, 7 and hold 3, 2, 2, 2 tiles; the last slice's extent is what
    # is left of K (ragged K = 9*256 - 100).
    assert [oracle.lib().oracle_splitk_first_ktile(u32(9), u32(4), u32(s)) for s in range(4)] == [0, 3, 5, 7]
    K = 9 * 256 - 100
    assert [oracle.splitk_actual_k(K, 256, 4, s) for s in range(4)] == [768, 512, 512, K - 7 * 256]
    # 10 k tiles over 4: two slices with an extra tile -> starts 0, 3, 6, 8
    assert [oracle.lib().oracle_splitk_first_ktile(u32(10), u32(4), u32(s)) for s in range(4)] == [0, 3, 6, 8]
    # task -> (m, n, first k tile, slice) on a 2x3 tile grid, swizzle <7,1> (one band of width 3: m = i/3, n = i%3):
    # the slice is the task's index divided by the 6 tiles of the grid
    assert oracle.splitk_block_coord(7, 1, 2, 3, 9, 4, 13) == (0, 1, 5, 2)
    assert oracle.splitk_block_coord(7, 1, 2, 3, 9, 4, 23) == (1, 2, 7, 3)
    assert oracle.splitk_block_coord(7, 1, 2, 3, 9, 4, 5) == (1, 2, 0, 0)
    assert oracle.splitk_block_coord(7, 1, 2, 3, 9, 4, 24 + 6) == (0, 0, 3, 1)    # wraps modulo the 24 tasks


def test_allgather_swizzle_hand_worked_ragged_last_round():
    # include/catcoc/dgemm/block/block_swizzle_allgather.hpp:88-108 by hand: P = 2 ranks with 3 tile rows each,
    # 2 tile columns, commInterval 2 -> rounds of 4 tile rows (2 per rank), then a last round of 2 (1 per rank).
    # Inside a round the base swizzle <7,1> on 2 columns is one band of width 2: (cm, cn) = (i/2, i%2); the row is
    # re-based rank-major: m = rank*3 + round*2 + cm % rowsPerRankThisRound.
    f = lambda t: oracle.allgather_block_coord(7, 1, 2, 2, 3, 2, t)
    assert f(0) == (0, 0) and f(3) == (1, 1)
    assert f(4) == (3, 0) and f(5) == (3, 1) and f(7) == (4, 1)      # second half of round 0 = rank 1
    assert f(8) == (2, 0) and f(9) == (2, 1)                          # last round: one row per rank
    assert f(10) == (5, 0) and f(11) == (5, 1)
    assert sorted(f(t) for t in range(12)) == [(m, n) for m in range(6) for n in range(2)]
    # direction 0, band width 3 on the 4 rows of round 0: band 0 = rows 0..2 (m fastest), band 1 = row 3 with the
    # columns walked backwards
    g = lambda t: oracle.allgather_block_coord(3, 0, 2, 2, 3, 2, t)
    assert [g(t) for t in range(8)] == [(0, 0), (1, 0), (3, 0), (0, 1), (1, 1), (3, 1), (4, 1), (4, 0)]


def test_reduce_i32_distinct_peers_and_row_offset():
    rng = np.random.default_rng(11)
    M, N, ld, r0 = 5, 7, 9, 3
    acc = rng.integers(-10 ** 6, 10 ** 6, (M, N), dtype=np.int32)
    peers = [rng.integers(-10 ** 6, 10 ** 6, (M + r0 + 2, ld), dtype=np.int32) for _ in range(3)]
    got = acc.copy()
    arr = (C.c_void_p * 3)(*[p.ctypes.data for p in peers])
    oracle.lib().oracle_reduce_i32(u32(M), u32(N), _p(got), C.c_int64(N), u32(3), arr, C.c_int64(ld), C.c_int64(r0))
    want = acc + sum(p[r0:r0 + M, :N] for p in peers)
    assert np.array_equal(got, want)
    # through the whole-operator entry: int32 peers with a row offset against numpy
    x1 = rng.integers(-127, 128, (8, 16), dtype=np.int8)
    x2 = rng.integers(-127, 128, (16, N), dtype=np.int8)
    s1 = rng.uniform(0.005, 0.02, 8).astype(np.float32)
    s2 = rng.uniform(0.001, 0.01, N).astype(np.float32)
    pk = [rng.integers(-10 ** 5, 10 ** 5, (2 + r0, N), dtype=np.int32) for _ in range(3)]
    _, out = oracle.quant_matmul_reduce_scatter(x1, x2, s1, s2, None, 4, 2, pk, oracle.FP16, peer_row0=r0, reduce_int32=True)
    tot = (x1[4:6].astype(np.int64) @ x2.astype(np.int64) + sum(p[r0:r0 + 2].astype(np.int64) for p in pk)).astype(np.int32)
    want = ((tot.astype(np.float32) * s2[None, :]) * s1[4:6, None]).astype(np.float16)
    assert np.array_equal(out, want.view(np.uint16))


def test_tiling_search_space():
    base = oracle.TilingParams(m=8192, k=1792, n=4096, m0=128, k0=256, n0=256, commTileM=64, commInterval=20,
                               commNpuSplit=1, commDataSplit=2, commBlockM=64, rankSize=8)
    rs = oracle.get_tilings(base, oracle.MATMUL_REDUCE_SCATTER, 8)
    assert len(rs) == 50                                    # 20*{4,6,8,12,14} all divide by 8
    assert [(t.commInterval, t.commTileM, t.commNpuSplit, t.commDataSplit) for t in rs[:3]] == \
        [(4, 4, 1, 16), (4, 4, 1, 20), (4, 8, 1, 16)]
    assert all(t.commBlockM == t.commTileM for t in rs)
    assert len(oracle.get_tilings(base, oracle.MATMUL_REDUCE_SCATTER, 3)) == 20   # only 6 and 12 divide by 3
    ar = oracle.get_tilings(base, oracle.MATMUL_ALLREDUCE, 8)
    # bound (204 MiB - 2.5 MiB)/2/8/2 = 6602752 elements vs commInterval*128*256*20 = 655360*ci: 4,6,8 pass
    assert sorted({t.commInterval for t in ar}) == [4, 6, 8] and len(ar) == 30
    ag = oracle.get_tilings(base, oracle.ALLGATHER_MATMUL, 8)
    # ci*128*256*ceil(1792/256)=229376*ci < 6602752 for every ci in the space
    assert len(ag) == 50
    base.k = 27392
    assert sorted({t.commInterval for t in oracle.get_tilings(base, oracle.ALLGATHER_MATMUL, 8)}) == []


# ------------------------------------------------------------- accuracy gate
def test_verify_rule():
    gold = np.array([0.5, 10.0, -300.0, 0.0], np.float32)
    ok, bad, eb = oracle.verify(gold, gold, oracle.FP16, 100)
    assert ok and bad == 0 and eb == 0
    out = gold + np.array([1 / 256, 10 / 256, 300 / 256, 0], np.float32)      # exactly at rtol*max(1,|g|): passes
    ok, bad, _ = oracle.verify(out, gold, oracle.FP16, 100)
    assert bad == 0
    out = gold + np.array([1 / 200, 0, 0, 0], np.float32)                     # above 2^-8 for K<2048 ...
    assert oracle.verify(out, gold, oracle.FP16, 100)[1] == 1
    assert oracle.verify(out, gold, oracle.FP16, 4096)[1] == 0                # ... but within 2^-7 for K>=2048
    assert oracle.verify(out, gold, oracle.BF16, 100)[1] == 0                 # bf16 rtol is 2^-7
    bias = gold + np.float32(0.002) * np.maximum(1, np.abs(gold))             # each within rtol, mean error 2e-3 > 2^-10
    ok, bad, eb = oracle.verify(bias, gold, oracle.FP16, 100)
    assert bad == 0 and not ok and abs(eb - 0.002) < 1e-4
    out = np.array([np.nan, 10.0, -300.0, np.inf], np.float32)                # NaN/Inf are zeroed first
    assert oracle.verify(out, gold, oracle.FP16, 100)[1] == 1


@needs_ref_golden
def test_verify_elementwise_rule_matches_reference_compare_data():
    rng = np.random.default_rng(12)
    gold = (rng.standard_normal(4000) * 50).astype(np.float32)
    out = gold + (rng.standard_normal(4000) * 0.05).astype(np.float32)
    for ct in (100, 4096):
        want = REF_G.ref_compare_data(_p(out), _p(gold), C.c_uint64(out.size), u32(ct))
        assert oracle.verify(out, gold, oracle.FP16, ct)[1] == want


# ------------------------------------------- deterministic comm swizzle, 16-bit adds, split-K reduce-add
def test_comm_swizzle_deterministic_hand_cases():
    # comm_block_swizzle.hpp:25-31,54-56,106-118,147-186 with IS_DETERMINISTIC worked by hand for the quant example's
    # split (20 x 1 cores), P = 8, 50 data blocks per rank: the band width is the core count (20), the last band is
    # padded to it (60 blocks -> 480 tasks), nStride = P, so task t of band b is (data b*20 + t%20, rank (t/20 + data) % 8).
    assert oracle.comm_core_loop(True, 8, 20, 1, 50) == 480 and oracle.comm_core_loop(False, 8, 20, 1, 50) == 400
    f = lambda t: oracle.comm_block_idx_det(8, 20, 1, 50, t)
    assert f(0) == (0, 0) and f(1) == (1, 1) and f(19) == (19, 3)
    assert f(20) == (0, 1) and f(21) == (1, 2)                       # same data blocks, next rank step
    assert f(160) == (20, 4) and f(170) == (30, 6)                   # band 1
    assert f(320 + 15) == (55, 7) and f(320 + 20 + 15) == (55, 0)    # band 2: data 50..59 are padding (>= 50)
    # the npu split folds into the data split: (10 x 2) behaves exactly like (20 x 1)
    assert all(oracle.comm_block_idx_det(8, 10, 2, 50, t) == f(t) for t in range(480))
    # what makes it deterministic: core c (tasks c, c + cores, ...) owns data blocks c, c + 20, ... and meets the ranks of a
    # block in the fixed sequence (data + i) % P
    for c in (0, 7, 19):
        tasks = [f(t) for t in range(c, 480, 20)]
        for band in range(3):
            seq = tasks[band * 8:(band + 1) * 8]
            d = band * 20 + c
            assert seq == [(d, (d + i) % 8) for i in range(8)]
    pairs = {f(t) for t in range(480)}
    assert len(pairs) == 480 and {p for p in pairs if p[0] < 50} == {(d, r) for d in range(50) for r in range(8)}


def test_add_half_is_the_correctly_rounded_sum():
    rng = np.random.default_rng(5)
    a = rng.integers(0, 1 << 16, 200000).astype(np.uint16)
    b = rng.integers(0, 1 << 16, 200000).astype(np.uint16)
    fin = np.isfinite(a.view(np.float16)) & np.isfinite(b.view(np.float16))
    a, b = a[fin], b[fin]
    with np.errstate(over="ignore"):
        want = (a.view(np.float16) + b.view(np.float16))            # numpy float16 addition is IEEE round-to-nearest-even
    got = oracle.add_half(a, b, oracle.FP16).view(np.float16)
    ok = np.isfinite(want)
    assert np.array_equal(got[ok].view(np.uint16), want[ok].view(np.uint16))
    # bf16 against exact rational arithmetic: the sum of two bf16 values, rounded once to 8 significand bits
    from fractions import Fraction
    a = rng.integers(0, 1 << 16, 3000).astype(np.uint16)
    b = rng.integers(0, 1 << 16, 3000).astype(np.uint16)
    fa, fb = oracle.half_to_f32(a, oracle.BF16), oracle.half_to_f32(b, oracle.BF16)
    got = oracle.half_to_f32(oracle.add_half(a, b, oracle.BF16), oracle.BF16)
    checked = 0
    for x, y, g in zip(fa, fb, got):
        if not (np.isfinite(x) and np.isfinite(y) and np.isfinite(g)) or abs(float(x) + float(y)) < 2.0 ** -120:
            continue
        s = Fraction(float(x)) + Fraction(float(y))
        if s == 0:
            assert g == 0
            continue
        e = 0                                                        # s = m * 2^e with 2^7 <= |m| < 2^8, m rounded to nearest even
        mag = abs(s)
        while mag >= 256:
            mag /= 2; e += 1
        while mag < 128:
            mag *= 2; e -= 1
        fl = mag.numerator // mag.denominator
        rem = mag - fl
        if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
            fl += 1
        want = float(fl) * 2.0 ** e * (1 if s > 0 else -1)
        assert float(g) == want, (x, y, g, want)
        checked += 1
    assert checked > 2000


def test_reduce_add_is_slice_sequential_fp32_with_one_cast():
    rng = np.random.default_rng(6)
    src = (rng.standard_normal((5, 37, 11)) * 100).astype(np.float32)
    want = src[0].copy()
    for k in range(1, 5):
        want = (want + src[k]).astype(np.float32)
    assert np.array_equal(oracle.reduce_add(src, 0), want)
    assert np.array_equal(oracle.reduce_add(src, oracle.FP16), want.astype(np.float16).view(np.uint16))
    assert np.array_equal(oracle.reduce_add(src, oracle.BF16), oracle.f32_to_half(want, oracle.BF16))
    # order matters in fp32: the oracle adds slice 0 first
    tricky = np.array([[1.0e8], [1.0], [-1.0e8]], np.float32)
    assert oracle.reduce_add(tricky, 0)[0] == np.float32(np.float32(np.float32(1.0e8) + np.float32(1.0)) + np.float32(-1.0e8))


def test_pipelined_order_tiles_the_kept_block_and_skips_self():
    # config-4-like geometry at small scale: every comm block covered exactly once, P - 1 ranks each, never this rank
    M, N, P, rank = 2048, 1024, 8, 5
    blocks = oracle.pipelined_reduce_scatter_order(M, N, P, rank, 128, 256, 16, 1, 64, 20, 1)
    cover = np.zeros((M // P, N), np.int32)
    for row0, rows, col0, cols, ranks in blocks:
        cover[row0:row0 + rows, col0:col0 + cols] += 1
        assert sorted(ranks) == [r for r in range(P) if r != rank]
    assert (cover == 1).all()
    # the rotation: different blocks start with different ranks
    assert len({tuple(b[4]) for b in blocks}) > 1
