"""ctypes loader for the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` import this module; the product package never does.  The oracle
restates the reference's golden math (see the header of ``catcoc_oracle.c`` for
the file:line map).  ``ref_golden()`` / ``ref_sched()`` return the reference's
own golden and scheduler code compiled from its sources into ``oracle/_ref/``
when that build exists, else ``None``.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

FP16 = 1
BF16 = 27
MATMUL_ALLREDUCE = 0
ALLGATHER_MATMUL = 1
MATMUL_REDUCE_SCATTER = 2

u32 = C.c_uint32
i64 = C.c_int64
vp = C.c_void_p


class TilingParams(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "m", "k", "n", "m0", "k0", "n0", "commTileM", "commInterval",
        "commNpuSplit", "commDataSplit", "commBlockM", "rankSize")]


def build(force=False):
    """Compile the oracle (and oracle/_ref when the reference tree is present)."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libcatcoc_oracle.so")
        if not os.path.exists(path):
            build()
        _LIB = C.CDLL(path)
        _LIB.oracle_bf16_to_f32.restype = C.c_float
        _LIB.oracle_f16_to_f32.restype = C.c_float
        _LIB.oracle_f32_to_bf16.restype = C.c_uint16
        _LIB.oracle_f32_to_f16.restype = C.c_uint16
        _LIB.oracle_f32_to_bf16.argtypes = [C.c_float]
        _LIB.oracle_f32_to_f16.argtypes = [C.c_float]
        _LIB.oracle_bf16_to_f32.argtypes = [C.c_uint16]
        _LIB.oracle_f16_to_f32.argtypes = [C.c_uint16]
        for name in ("oracle_splitk_first_ktile", "oracle_splitk_actual_k", "oracle_splitk_factor",
                     "oracle_comm_block_row", "oracle_comm_core_loop"):
            getattr(_LIB, name).restype = C.c_uint32
    return _LIB


def _load_ref(name):
    path = os.path.join(_HERE, "_ref", name)
    return C.CDLL(path) if os.path.exists(path) else None


def ref_golden():
    r = _load_ref("libcatcoc_ref_golden.so")
    if r is not None:
        r.ref_compare_data.restype = C.c_uint64
        r.ref_round_to_bf16.restype = C.c_uint16
        r.ref_round_to_bf16.argtypes = [C.c_float]
    return r


def ref_sched():
    return _load_ref("libcatcoc_ref_sched.so")


def _p(a):
    return a.ctypes.data_as(vp) if a is not None else None


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


# ---------------------------------------------------------------- conversions
def f32_to_half(x, dtype):
    """float32 array -> uint16 bit patterns (RNE) of fp16 / bf16."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_cast_f32_to_half(_p(x), _p(out), C.c_size_t(x.size), C.c_int(dtype))
    return out


def half_to_f32(h, dtype):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().oracle_cast_half_to_f32(_p(h), _p(out), C.c_size_t(h.size), C.c_int(dtype))
    return out


# ---------------------------------------------------------------------- GEMMs
def gemm_i8_i32(A, B, bias=None, transB=False):
    A = _c(A, np.int8)
    B = _c(B, np.int8)
    M, K = A.shape
    N = B.shape[0] if transB else B.shape[1]
    out = np.empty((M, N), np.int32)
    b = _c(bias, np.int32) if bias is not None else None
    lib().oracle_gemm_i8_i32(u32(M), u32(N), u32(K), _p(A), i64(K), _p(B), i64(B.shape[1]), C.c_int(int(transB)),
                             _p(b), _p(out), i64(N))
    return out


def gemm_i8_i32_literal(A, B):
    A = _c(A, np.int8)
    B = _c(B, np.int8)
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N), np.int32)
    lib().oracle_gemm_i8_i32_literal(u32(M), u32(N), u32(K), _p(A), _p(B), _p(out))
    return out


def gemm_half_f32(A, B, dtype, transA=False, transB=False):
    """A, B as uint16 bit patterns; returns the fp32 k-sequential accumulation."""
    A = _c(A, np.uint16)
    B = _c(B, np.uint16)
    M, K = (A.shape[1], A.shape[0]) if transA else A.shape
    N = B.shape[0] if transB else B.shape[1]
    out = np.empty((M, N), np.float32)
    lib().oracle_gemm_half_f32(u32(M), u32(N), u32(K), _p(A), i64(A.shape[1]), C.c_int(int(transA)),
                               _p(B), i64(B.shape[1]), C.c_int(int(transB)), C.c_int(dtype), _p(out), i64(N))
    return out


def dequant(acc, scale_n, scale_m):
    acc = _c(acc, np.int32)
    M, N = acc.shape
    sn = _c(scale_n, np.float32)
    sm = _c(scale_m, np.float32)
    out = np.empty((M, N), np.float32)
    lib().oracle_dequant(u32(M), u32(N), _p(acc), i64(N), _p(sn), _p(sm), _p(out), i64(N))
    return out


def _ptr_array(arrs):
    arr = (vp * max(1, len(arrs)))()
    for i, a in enumerate(arrs):
        arr[i] = a.ctypes.data
    return arr


def reduce_cast(local, peers, dtype, peer_row0=0):
    local = _c(local, np.float32)
    peers = [_c(p, np.float32) for p in peers]
    M, N = local.shape
    out = np.empty((M, N), np.uint16)
    ldp = peers[0].shape[1] if peers else N
    lib().oracle_reduce_cast(u32(M), u32(N), _p(local), i64(N), u32(len(peers)), _ptr_array(peers), i64(ldp),
                             i64(peer_row0), C.c_int(dtype), _p(out), i64(N))
    return out


def quant_matmul_reduce_scatter(x1, x2, scale_x1, scale_x2, bias, row0, rows_kept, peers, out_dtype,
                                peer_row0=0, reduce_int32=False, transB=False, want_acc=True):
    """Returns (acc_full int32 [M,N] or None, d_out uint16 [rows_kept,N])."""
    x1 = _c(x1, np.int8)
    x2 = _c(x2, np.int8)
    M, K = x1.shape
    N = x2.shape[0] if transB else x2.shape[1]
    s1 = _c(scale_x1, np.float32)
    s2 = _c(scale_x2, np.float32)
    b = _c(bias, np.int32) if bias is not None else None
    pdt = np.int32 if reduce_int32 else np.float32
    peers = [_c(p, pdt) for p in peers]
    ldp = peers[0].shape[1] if peers else N
    acc = np.empty((M, N), np.int32) if want_acc else None
    out = np.empty((rows_kept, N), np.uint16)
    lib().oracle_quant_matmul_reduce_scatter(
        u32(M), u32(N), u32(K), _p(x1), _p(x2), C.c_int(int(transB)), _p(s1), _p(s2), _p(b),
        u32(row0), u32(rows_kept), u32(len(peers)), _ptr_array(peers), i64(ldp), i64(peer_row0),
        C.c_int(int(reduce_int32)), C.c_int(out_dtype), _p(acc), _p(out))
    return acc, out


def matmul_reduce(A, B, dtype, row0, rows_kept, peers, peer_row0=0, transA=False, transB=False, want_partial=False):
    """Float matmul + fp32 peer reduce of the kept rows.  Returns (partial fp32 or None, d_out uint16)."""
    A = _c(A, np.uint16)
    B = _c(B, np.uint16)
    M, K = (A.shape[1], A.shape[0]) if transA else A.shape
    N = B.shape[0] if transB else B.shape[1]
    peers = [_c(p, np.float32) for p in peers]
    ldp = peers[0].shape[1] if peers else N
    part = np.empty((M, N), np.float32) if want_partial else None
    out = np.empty((rows_kept, N), np.uint16)
    lib().oracle_matmul_reduce(u32(M), u32(N), u32(K), _p(A), C.c_int(int(transA)), _p(B), C.c_int(int(transB)),
                               C.c_int(dtype), u32(row0), u32(rows_kept), u32(len(peers)), _ptr_array(peers),
                               i64(ldp), i64(peer_row0), _p(part), _p(out))
    return part, out


def allgather_matmul(a_shards, B, dtype, transB=False):
    shards = [_c(a, np.uint16) for a in a_shards]
    B = _c(B, np.uint16)
    m_local, K = shards[0].shape
    N = B.shape[0] if transB else B.shape[1]
    P = len(shards)
    out = np.empty((P * m_local, N), np.uint16)
    lib().oracle_allgather_matmul(u32(m_local), u32(N), u32(K), u32(P), _ptr_array(shards), _p(B),
                                  C.c_int(int(transB)), C.c_int(dtype), _p(out))
    return out


# ----------------------------------------------------------------- schedulers
def swizzle_block_coord(off, direction, loopsM, loopsN, task):
    m, n = u32(), u32()
    lib().oracle_swizzle_block_coord(u32(off), u32(direction), u32(loopsM), u32(loopsN), u32(task),
                                     C.byref(m), C.byref(n))
    return m.value, n.value


def swizzle_actual_shape(M, N, m0, n0, mIdx, nIdx):
    a, b = u32(), u32()
    lib().oracle_swizzle_actual_shape(u32(M), u32(N), u32(m0), u32(n0), u32(mIdx), u32(nIdx), C.byref(a), C.byref(b))
    return a.value, b.value


def splitk_block_coord(off, direction, loopsM, loopsN, kTiles, f, task):
    m, n, k, s = u32(), u32(), u32(), u32()
    lib().oracle_splitk_block_coord(u32(off), u32(direction), u32(loopsM), u32(loopsN), u32(kTiles), u32(f),
                                    u32(task), C.byref(m), C.byref(n), C.byref(k), C.byref(s))
    return m.value, n.value, k.value, s.value


def splitk_actual_k(K, k0, f, s):
    return lib().oracle_splitk_actual_k(u32(K), u32(k0), u32(f), u32(s))


def splitk_factor(m, n, k, cores, m0, n0, k0):
    return lib().oracle_splitk_factor(u32(m), u32(n), u32(k), u32(cores), u32(m0), u32(n0), u32(k0))


def allgather_block_coord(off, direction, P, commInterval, loopsMRank, loopsN, task):
    m, n = u32(), u32()
    lib().oracle_allgather_block_coord(u32(off), u32(direction), u32(P), u32(commInterval), u32(loopsMRank),
                                       u32(loopsN), u32(task), C.byref(m), C.byref(n))
    return m.value, n.value


def comm_block_idx(direction, P, splitRow, splitCol, dataLoopsInRank, task):
    d, r = u32(), u32()
    lib().oracle_comm_block_idx(u32(direction), u32(P), u32(splitRow), u32(splitCol), u32(dataLoopsInRank),
                                u32(task), C.byref(d), C.byref(r))
    return d.value, r.value


def comm_core_loop(deterministic, P, splitRow, splitCol, dataLoopsInRank):
    return lib().oracle_comm_core_loop(C.c_int(int(deterministic)), u32(P), u32(splitRow), u32(splitCol), u32(dataLoopsInRank))


def comm_block_idx_det(P, splitRow, splitCol, dataLoopsInRank, task):
    d, r = u32(), u32()
    lib().oracle_comm_block_idx_det(u32(P), u32(splitRow), u32(splitCol), u32(dataLoopsInRank), u32(task), C.byref(d), C.byref(r))
    return d.value, r.value


def add_half(a_bits, b_bits, dtype):
    a = _c(a_bits, np.uint16)
    b = _c(b_bits, np.uint16)
    out = np.empty(a.shape, np.uint16)
    lib().oracle_add_half(_p(a), _p(b), C.c_size_t(a.size), C.c_int(dtype), _p(out))
    return out


def reduce_add(src_f32, dtype):
    """src [slices, ...] fp32 -> the slices' sum in slice order, cast once (dtype 0: fp32)."""
    src = _c(src_f32, np.float32)
    f = src.shape[0]
    count = src[0].size
    out = np.empty(src.shape[1:], np.float32 if dtype == 0 else np.uint16)
    lib().oracle_reduce_add(_p(src), C.c_size_t(count), u32(f), C.c_int(dtype), _p(out))
    return out


def pipelined_reduce_scatter_order(M, N, P, rank, m0, n0, blockNum, commInterval, commBlockM, splitRow, splitCol, off=7,
                                   direction=1):
    """The reference's comm rounds replayed on the CPU with the deterministic comm swizzle
    (KQ:262-320 / KRS:237-296 with CSW's BlockCommSwizzle<0,true>): for every data block of every round, the rows and
    columns of the kept block it covers and the ranks whose blocks are added to it, in the order its core meets them.
    -> list of (row0, rows, col0, cols, [ranks])."""
    mRank = M // P
    loopsM, loopsN = -(-mRank // m0), -(-N // n0)
    coreLoops = loopsM * loopsN * P
    bpc = blockNum * commInterval
    perRank = bpc // P
    rounds = -(-coreLoops // bpc)
    bpt = m0 // commBlockM
    cores = splitRow * splitCol
    blocks = []
    for rnd in range(rounds):
        actual = min(bpc, coreLoops - rnd * bpc)
        dl = (actual // P) * bpt
        loop = comm_core_loop(True, P, splitRow, splitCol, dl)
        seq = {}
        for core in range(cores):                      # a core runs its tasks one after the other (KQ:291)
            for t in range(core, loop, cores):
                d, r = comm_block_idx_det(P, splitRow, splitCol, dl, t)
                if d >= dl or r == rank:               # padding block / this rank's own data (KQ:300)
                    continue
                seq.setdefault(d, []).append(r)
        for d in range(dl):
            tile, sub = divmod(d, bpt)
            mi, ni = swizzle_block_coord(off, direction, loopsM, loopsN, rnd * perRank + tile)
            row0 = mi * m0 + sub * commBlockM
            rows = max(0, min(commBlockM, mRank - row0))
            cols = min(n0, N - ni * n0)
            blocks.append((row0, rows, ni * n0, cols, seq.get(d, [])))
    return blocks


def pipelined_reduce_half(local_f32, peers_bits, dtype, M, P, rank, m0, n0, blockNum, commInterval, commBlockM, splitRow,
                          splitCol):
    """Float reduce-scatter in the reference's precision: the local fp32 partial of the kept block [M/P, N] is rounded to
    the 16-bit type, then each peer's 16-bit block is added with one rounding per add, ranks in the deterministic comm
    order.  peers_bits[s] is the block of rank s (s < rank) or s + 1.  -> uint16 [M/P, N]."""
    local = _c(local_f32, np.float32)
    N = local.shape[1]
    out = f32_to_half(local, dtype)
    covered = np.zeros(local.shape, np.int32)
    for row0, rows, col0, cols, ranks in pipelined_reduce_scatter_order(M, N, P, rank, m0, n0, blockNum, commInterval,
                                                                        commBlockM, splitRow, splitCol):
        if rows <= 0:
            continue
        sl = (slice(row0, row0 + rows), slice(col0, col0 + cols))
        covered[sl] += 1
        v = out[sl]
        for r in ranks:
            v = add_half(v, _c(peers_bits[r if r < rank else r - 1][sl], np.uint16), dtype)
        out[sl] = v
    assert (covered == 1).all(), "the comm blocks must tile the kept block exactly once"
    return out


def rs_task(M, N, P, m0, n0, blockNum, commInterval, stages, t, off=7, direction=1):
    """-> (targetRank, mIdx, nIdx, row, col, wsRow) or None past the end."""
    o = [u32() for _ in range(6)]
    ok = lib().oracle_rs_task(u32(M), u32(N), u32(P), u32(m0), u32(n0), u32(blockNum), u32(commInterval),
                              u32(stages), u32(off), u32(direction), u32(t), *[C.byref(x) for x in o])
    return tuple(x.value for x in o) if ok else None


def ar_task(M, N, m0, n0, blockNum, commInterval, stages, t, off=7, direction=1):
    o = [u32() for _ in range(3)]
    ok = lib().oracle_ar_task(u32(M), u32(N), u32(m0), u32(n0), u32(blockNum), u32(commInterval), u32(stages),
                              u32(off), u32(direction), u32(t), *[C.byref(x) for x in o])
    return tuple(x.value for x in o) if ok else None


def get_tilings(base, commType, rankSize, blockNum=20):
    out = (TilingParams * 64)()
    n = lib().oracle_get_tilings(C.byref(base), C.c_int(commType), C.c_int(rankSize), C.c_int(blockNum), out, 64)
    return [out[i] for i in range(n)]


def verify(out_f32, gold_f32, dtype, compute_times):
    """The reference's accuracy gate.  -> (passed, n_bad, eb)."""
    o = _c(out_f32, np.float32).ravel()
    g = _c(gold_f32, np.float32).ravel()
    nb, eb = C.c_uint64(), C.c_double()
    ok = lib().oracle_verify(_p(o), _p(g), C.c_size_t(o.size), C.c_int(dtype), u32(compute_times),
                             C.byref(nb), C.byref(eb))
    return bool(ok), nb.value, eb.value


def num_threads():
    return lib().oracle_num_threads()
