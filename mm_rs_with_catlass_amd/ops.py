"""Host-side mirror of the reference's operator entry points, on torch tensors resident in HBM.

Each function fills the reference's ``CocTilingParams`` and the one-GPU symmetric
descriptor, then calls the matching C-ABI launcher of ``libcatcoc_hip.so``
(``include/catcoc_hip.h``) on torch's current stream.  torch is used for device
memory and streams only; all arithmetic happens in the HIP kernels.

Reference entry points mirrored (paths relative to the reference tree):
  ShmemQuantMatmulReduceScatter   examples/02_matmul_reduce_scatter/quant_matmul_reduce_scatter.cpp:54-60
  LaunchMatmulReduceScatter*      examples/dynamic_tiling/impl/kernel_fp16.cpp:64-86
  LaunchMatmulAllReduce*          examples/dynamic_tiling/impl/kernel_fp16.cpp:22-44
  LaunchAllGatherMatmul*          examples/dynamic_tiling/impl/kernel_fp16.cpp:46-62
"""
import ctypes as C

import torch

from . import lib as _l

_TORCH_TO_DT = {torch.float16: _l.FP16, torch.bfloat16: _l.BF16}


def default_tiling(m, k, n, rank_size, **over):
    """The defaults of examples/dynamic_tiling/dynamic_tiling.cpp:215-227, with overrides.
    m0/n0/k0 = 0 lets the library pick its own macro tile."""
    t = _l.CocTilingParams()
    _l.load().catcoc_default_tiling(C.byref(t), m, k, n, rank_size)
    t.commInterval = 1
    for key, val in over.items():
        setattr(t, key, val)
    return t


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def _check_dev(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise _l.CatcocError("all operands must live on the GPU (got a %s tensor)" % t.device)
        if t is not None and not t.is_contiguous():
            raise _l.CatcocError("operands must be contiguous")


def _fail(msg, *a):
    raise _l.CatcocError(msg % a if a else msg)


def _want(t, name, dtype=None, ndim=None, numel=None, shape=None):
    """One operand against what the kernels will read or write: the C ABI sees raw pointers only, so sizes and element
    types can be checked here and nowhere else (a short or mistyped buffer is an out-of-bounds access on the GPU)."""
    if t is None:
        return
    if dtype is not None and t.dtype not in (dtype if isinstance(dtype, tuple) else (dtype,)):
        _fail("%s must be %s (got %s)", name, dtype, t.dtype)
    if ndim is not None and t.dim() != ndim:
        _fail("%s must have %d dimensions (got shape %s)", name, ndim, tuple(t.shape))
    if shape is not None and tuple(t.shape) != tuple(shape):
        _fail("%s must have shape %s (got %s)", name, tuple(shape), tuple(t.shape))
    if numel is not None and t.numel() < numel:
        _fail("%s holds %d elements, the launch needs %d", name, t.numel(), numel)


def _check_peers(peers, count, dtype, rows_needed, n, what="peers"):
    if len(peers) != count:
        _fail("%s: %d buffers given, rank_size - 1 = %d needed", what, len(peers), count)
    for i, p in enumerate(peers):
        _want(p, "%s[%d]" % (what, i), dtype, 2)
        if p.shape[1] != peers[0].shape[1]:
            _fail("%s[%d] has %d columns, %s[0] has %d: one leading dimension serves all", what, i, p.shape[1], what, peers[0].shape[1])
        if p.shape[1] < n or p.shape[0] < rows_needed:
            _fail("%s[%d] has shape %s, the launch reads rows [0,%d) x %d columns", what, i, tuple(p.shape), rows_needed, n)


def _check_rank(rank, rank_size):
    if rank_size < 1 or rank_size > _l.MAX_RANKS or not 0 <= rank < rank_size:
        _fail("rank %d / rank_size %d out of range (1..%d ranks)", rank, rank_size, _l.MAX_RANKS)


def _task_count(comm_type, t, d):
    n = int(_l.load().catcoc_get_task_count(comm_type, C.byref(t), C.byref(d)))
    _l.check()
    return n


def _kept_flag(kept_split):
    """kept_split: None = the library decides, False = kept tiles whole, True = two 64-row workgroups where allowed,
    "kept-only" = as None but the tiles that wait for the kept halves' slots stay whole (CATCOC_FLAG_TAIL_WHOLE)."""
    if kept_split == "kept-only":
        return _l.FLAG_TAIL_WHOLE
    return 0 if kept_split is None else (_l.FLAG_KEPT_SPLIT if kept_split else _l.FLAG_KEPT_WHOLE)


def _attach_workspace(d, workspace, split_k):
    """Optional scratch for k-sliced launches (kslice_plan() says how large) and the caller's own slice count."""
    d.splitK = split_k
    if workspace is not None:
        _check_dev(workspace)
        d.workspace = workspace.data_ptr()
        d.workspaceBytes = workspace.numel() * workspace.element_size()


def _desc(rank, rank_size, peers, peer_row_offset, flags, block_num, stages, swizzle, outbound, checksum, acc_dump):
    peer_ld = peers[0].shape[1] if peers else 0
    return _l.make_desc(
        rank, rank_size, [p.data_ptr() for p in peers], peer_ld, peer_row_offset, flags, block_num, stages, swizzle,
        _ptr(outbound), outbound.numel() * outbound.element_size() if outbound is not None else 0,
        _ptr(checksum), _ptr(acc_dump))


def prepare_quant_matmul_reduce_scatter(x1, x2, scale_x1, scale_x2, bias=None, peers=(), rank=0, rank_size=1,
                                        out_dtype=torch.bfloat16, tiling=None, trans_b=False, peer_row_offset=0,
                                        reduce_int32=False, outbound=None, checksum=None, acc_dump=None,
                                        c_accum=None, block_num=0, stages=0, swizzle=None, linear_order=False,
                                        out=None, workspace=None, split_k=0, trans_a=False, kept_split=None):
    """Validate and bind the arguments once; returns (launch, out) where launch() enqueues one call of
    catcoc_launch_quant_matmul_reduce_scatter on torch's current stream (for launch-rate-sensitive loops)."""
    _check_rank(rank, rank_size)
    _want(x1, "x1", torch.int8, 2)
    _want(x2, "x2", torch.int8, 2)
    m, k = (x1.shape[1], x1.shape[0]) if trans_a else x1.shape
    n = x2.shape[0] if trans_b else x2.shape[1]
    if (x2.shape[1] if trans_b else x2.shape[0]) != k:
        _fail("x2 has shape %s: its k extent does not match x1's k = %d", tuple(x2.shape), k)
    if m % rank_size != 0:
        _fail("reduce-scatter needs m %% rank_size == 0 (m=%d, rank_size=%d)", m, rank_size)
    if peer_row_offset < 0:
        _fail("peer_row_offset must be >= 0")
    rows = m // rank_size
    _want(scale_x1, "scale_x1", torch.float32, 1, m)
    _want(scale_x2, "scale_x2", torch.float32, 1, n)
    _want(bias, "bias", torch.int32, 1, n)
    _check_peers(list(peers), rank_size - 1, torch.int32 if reduce_int32 else torch.float32, peer_row_offset + rows, n)
    _want(c_accum, "c_accum", torch.int32, None, rows * n)
    _want(acc_dump, "acc_dump", torch.int32, None, m * n)
    _want(outbound, "outbound", (torch.float32, torch.int32))
    t = tiling if tiling is not None else default_tiling(m, k, n, rank_size, m0=0, n0=0, k0=0)
    if (t.m, t.k, t.n) != (m, k, n):
        _fail("tiling says m,k,n = %d,%d,%d; the operands say %d,%d,%d", t.m, t.k, t.n, m, k, n)
    flags = (_l.OUTBOUND_STORE if outbound is not None else 0) | (_l.FLAG_REDUCE_INT32 if reduce_int32 else 0) | \
        (_l.FLAG_LINEAR_ORDER if linear_order else 0) | _kept_flag(kept_split)
    d = _desc(rank, rank_size, list(peers), peer_row_offset, flags, block_num, stages, swizzle, outbound, checksum, acc_dump)
    _attach_workspace(d, workspace, split_k)
    if checksum is not None:
        _want(checksum, "checksum", torch.int64, None, _task_count(_l.QUANT_MATMUL_REDUCE_SCATTER, t, d))
    if out is None:
        out = torch.empty((rows, n), dtype=out_dtype, device=x1.device)
    _want(out, "out", (torch.float16, torch.bfloat16), 2, None, (rows, n))
    _check_dev(x1, x2, scale_x1, scale_x2, bias, outbound, checksum, acc_dump, c_accum, out, *peers)
    L = _l.load()
    keep = (x1, x2, scale_x1, scale_x2, bias, tuple(peers), outbound, checksum, acc_dump, c_accum, out, d, t, workspace)
    fn = L.catcoc_launch_quant_matmul_reduce_scatter
    argv = (0, x1.data_ptr(), x2.data_ptr(), scale_x1.data_ptr(), scale_x2.data_ptr(), _ptr(bias), _ptr(c_accum),
            out.data_ptr(), C.addressof(d), C.byref(t), int(trans_a), int(trans_b), _TORCH_TO_DT[out.dtype])

    def launch(_keep=keep):
        fn(_stream(), *argv)

    return launch, out


def quant_matmul_reduce_scatter(x1, x2, scale_x1, scale_x2, bias=None, peers=(), rank=0, rank_size=1,
                                out_dtype=torch.bfloat16, tiling=None, trans_b=False, peer_row_offset=0,
                                reduce_int32=False, outbound=None, checksum=None, acc_dump=None, c_accum=None,
                                block_num=0, stages=0, swizzle=None, linear_order=False, out=None, workspace=None,
                                split_k=0, trans_a=False, kept_split=None):
    """W8A8 matmul -> reduce-scatter share of one rank.

    x1 [m,k] int8 ([k,m] with trans_a), x2 [k,n] int8 ([n,k] with trans_b), scale_x1 [m] fp32 per token, scale_x2 [n] fp32 per
    channel, bias [n] int32 or None.  peers: rank_size-1 staged partials for the kept rows (fp32, or int32
    with reduce_int32), added in list order after the local partial.  workspace: optional zero-initialised uint8
    tensor of kslice_plan() bytes with which a launch of few tiles cuts its k range into slices.
    Returns d_out [m/rank_size, n].
    """
    launch, out = prepare_quant_matmul_reduce_scatter(
        x1, x2, scale_x1, scale_x2, bias, peers, rank, rank_size, out_dtype, tiling, trans_b, peer_row_offset,
        reduce_int32, outbound, checksum, acc_dump, c_accum, block_num, stages, swizzle, linear_order, out, workspace, split_k,
        trans_a, kept_split)
    launch()
    _l.check()
    return out


def splitk_plan(m, k, n, rank_size, kept_row_begin, kept_rows, split_k=0, block_num=0, n0=0):
    """(workspace bytes, k slices, 128x128 blocks) of the explicit-kept-rows path for this problem.  n0 = 128 asks for the
    128x128 split-K kernel, 256 for the 128x256 kernel, 0 lets the library choose by the number of rows."""
    t = default_tiling(m, k, n, rank_size, m0=128 if n0 else 0, n0=n0, k0=0)
    d = _l.make_desc(0, rank_size, block_num=block_num)
    d.keptRowBegin, d.keptRows, d.splitK = kept_row_begin, kept_rows, split_k
    f, tiles = C.c_uint32(), C.c_uint32()
    need = _l.load().catcoc_get_splitk_workspace_size(C.byref(t), C.byref(d), C.byref(f), C.byref(tiles))
    _l.check()
    return int(need), f.value, tiles.value


def prepare_quant_matmul_splitk(x1, x2, scale_x1, scale_x2, bias=None, peers=(), rank_size=1, kept_row_begin=0,
                                kept_rows=None, out_dtype=torch.bfloat16, split_k=0, workspace=None, checksum=None,
                                acc_dump=None, c_accum=None, peer_row_offset=0, block_num=0, swizzle=None, out=None, n0=0,
                                trans_b=False, reduce_int32=False):
    """Skinny-M (decode) form of the W8A8 operator: x1 [m,k] with any m, x2 [k,n] (or [n,k] with trans_b, the layout of a
    stored weight matrix), the rank keeps rows [kept_row_begin, +kept_rows); peers are rank_size-1 partials [kept_rows, n],
    fp32 added after the dequantisation or, with reduce_int32, int32 added before it.  Returns (launch, out)."""
    _check_rank(0, rank_size)
    _want(x1, "x1", torch.int8, 2)
    _want(x2, "x2", torch.int8, 2)
    m, k = x1.shape
    n = x2.shape[0] if trans_b else x2.shape[1]
    if (x2.shape[1] if trans_b else x2.shape[0]) != k:
        _fail("x2 has shape %s: its k extent does not match x1's k = %d", tuple(x2.shape), k)
    kr = kept_rows if kept_rows is not None else m
    if kept_row_begin < 0 or kr < 1 or kept_row_begin + kr > m:
        _fail("kept rows [%d,+%d) outside [0,%d)", kept_row_begin, kr, m)
    if peer_row_offset < 0:
        _fail("peer_row_offset must be >= 0")
    _want(scale_x1, "scale_x1", torch.float32, 1, m)
    _want(scale_x2, "scale_x2", torch.float32, 1, n)
    _want(bias, "bias", torch.int32, 1, n)
    _check_peers(list(peers), rank_size - 1, torch.int32 if reduce_int32 else torch.float32, peer_row_offset + kr, n)
    _want(c_accum, "c_accum", torch.int32, None, kr * n)
    _want(acc_dump, "acc_dump", torch.int32, None, m * n)
    _want(checksum, "checksum", torch.int64, None, -(-m // 128) * -(-n // 128))
    _want(out, "out", (torch.float16, torch.bfloat16), 2, None, (kr, n))
    _check_dev(x1, x2, scale_x1, scale_x2, bias, checksum, acc_dump, c_accum, workspace, out, *peers)
    t = default_tiling(m, k, n, rank_size, m0=128 if n0 else 0, n0=n0, k0=0)
    d = _desc(0, rank_size, list(peers), peer_row_offset, _l.FLAG_REDUCE_INT32 if reduce_int32 else 0, block_num, 0, swizzle, None,
              checksum, acc_dump)
    d.keptRowBegin = kept_row_begin
    d.keptRows = kept_rows if kept_rows is not None else m
    d.splitK = split_k
    if workspace is not None:
        d.workspace = workspace.data_ptr()
        d.workspaceBytes = workspace.numel() * workspace.element_size()
    if out is None:
        out = torch.empty((d.keptRows, n), dtype=out_dtype, device=x1.device)
    keep = (x1, x2, scale_x1, scale_x2, bias, tuple(peers), checksum, acc_dump, c_accum, out, d, t, workspace)
    fn = _l.load().catcoc_launch_quant_matmul_reduce_scatter
    argv = (0, x1.data_ptr(), x2.data_ptr(), scale_x1.data_ptr(), scale_x2.data_ptr(), _ptr(bias), _ptr(c_accum),
            out.data_ptr(), C.addressof(d), C.byref(t), 0, int(trans_b), _TORCH_TO_DT[out.dtype])

    def launch(_keep=keep):
        fn(_stream(), *argv)

    return launch, out


def quant_matmul_splitk(*args, **kw):
    """One launch of prepare_quant_matmul_splitk(); returns d_out [kept_rows, n]."""
    launch, out = prepare_quant_matmul_splitk(*args, **kw)
    launch()
    _l.check()
    return out


def _float_op(comm_type, a, b, c_shape, peers, rank, rank_size, tiling, trans_a, trans_b, peer_row_offset, outbound,
              checksum, acc_dump, block_num, stages, swizzle, linear_order, out, m_for_tiling, workspace=None, split_k=0,
              kept_split=None):
    if a.dtype not in _TORCH_TO_DT or b.dtype != a.dtype:
        raise _l.CatcocError("a and b must both be float16 or both bfloat16")
    _check_rank(rank, rank_size)
    _want(a, "a", None, 2)
    _want(b, "b", None, 2)
    k = a.shape[0] if trans_a else a.shape[1]
    n = b.shape[0] if trans_b else b.shape[1]
    if (b.shape[1] if trans_b else b.shape[0]) != k:
        _fail("b has shape %s: its k extent does not match a's k = %d", tuple(b.shape), k)
    if peer_row_offset < 0:
        _fail("peer_row_offset must be >= 0")
    out_shape = c_shape(n)
    if comm_type == _l.ALLGATHER_MATMUL:
        _check_peers(list(peers), rank_size - 1, a.dtype, a.shape[0], k, "peer_shards")
        for i, p in enumerate(peers):
            if tuple(p.shape) != tuple(a.shape):
                _fail("peer_shards[%d] has shape %s, this rank's shard %s", i, tuple(p.shape), tuple(a.shape))
    else:
        if comm_type == _l.MATMUL_REDUCE_SCATTER and m_for_tiling % rank_size != 0:
            _fail("reduce-scatter needs m %% rank_size == 0 (m=%d, rank_size=%d)", m_for_tiling, rank_size)
        _check_peers(list(peers), rank_size - 1, torch.float32, peer_row_offset + out_shape[0], n)
    rows_all = m_for_tiling * (rank_size if comm_type == _l.ALLGATHER_MATMUL else 1)
    _want(acc_dump, "acc_dump", torch.float32, None, rows_all * n)
    _want(outbound, "outbound", torch.float32)
    t = tiling if tiling is not None else default_tiling(m_for_tiling, k, n, rank_size, m0=0, n0=0, k0=0)
    if (t.m, t.k, t.n) != (m_for_tiling, k, n):
        _fail("tiling says m,k,n = %d,%d,%d; the operands say %d,%d,%d", t.m, t.k, t.n, m_for_tiling, k, n)
    flags = (_l.OUTBOUND_STORE if outbound is not None else 0) | (_l.FLAG_LINEAR_ORDER if linear_order else 0) | _kept_flag(kept_split)
    d = _desc(rank, rank_size, list(peers), peer_row_offset, flags, block_num, stages, swizzle, outbound, checksum, acc_dump)
    _attach_workspace(d, workspace, split_k)
    if checksum is not None:
        _want(checksum, "checksum", torch.float64, None, _task_count(comm_type, t, d))
    if out is None:
        out = torch.empty(out_shape, dtype=a.dtype, device=a.device)
    _want(out, "out", a.dtype, 2, None, out_shape)
    _check_dev(a, b, outbound, checksum, acc_dump, out, *peers)
    L = _l.load()
    fn = L.catcoc_get_kernel(comm_type, _TORCH_TO_DT[a.dtype])
    if not fn:
        raise _l.CatcocError("no kernel registered for commType %d dtype %s" % (comm_type, a.dtype))
    _l.KernelFuncPtr(fn)(_stream(), 0, a.data_ptr(), b.data_ptr(), out.data_ptr(), None, None, C.addressof(d),
                         C.byref(t), int(trans_a), int(trans_b))
    _l.check()
    return out


def matmul_reduce_scatter(a, b, peers=(), rank=0, rank_size=1, tiling=None, trans_a=False, trans_b=False,
                          peer_row_offset=0, outbound=None, checksum=None, acc_dump=None, block_num=0, stages=0,
                          swizzle=None, linear_order=False, out=None, workspace=None, split_k=0, kept_split=None):
    """fp16/bf16 matmul -> reduce-scatter share: a [m,k], b [k,n], peers fp32; returns [m/rank_size, n]."""
    m = a.shape[1] if trans_a else a.shape[0]
    return _float_op(_l.MATMUL_REDUCE_SCATTER, a, b, lambda n: (m // max(rank_size, 1), n), peers, rank, rank_size,
                     tiling, trans_a, trans_b, peer_row_offset, outbound, checksum, acc_dump, block_num, stages,
                     swizzle, linear_order, out, m, workspace, split_k, kept_split)


def matmul_allreduce(a, b, peers=(), rank=0, rank_size=1, tiling=None, trans_a=False, trans_b=False,
                     peer_row_offset=0, acc_dump=None, block_num=0, stages=0, swizzle=None, linear_order=False,
                     out=None, workspace=None, split_k=0):
    """fp16/bf16 matmul -> all-reduce share: every row is kept; peers are full [m,n] fp32 partials."""
    m = a.shape[1] if trans_a else a.shape[0]
    return _float_op(_l.MATMUL_ALLREDUCE, a, b, lambda n: (m, n), peers, rank, rank_size, tiling, trans_a, trans_b,
                     peer_row_offset, None, None, acc_dump, block_num, stages, swizzle, linear_order, out, m, workspace, split_k)


def allgather_matmul(a_local, peer_shards, b, rank=0, rank_size=1, tiling=None, trans_b=False, acc_dump=None,
                     block_num=0, stages=0, swizzle=None, linear_order=False, out=None, workspace=None, split_k=0):
    """all-gather -> matmul: a_local [m,k] is this rank's shard, peer_shards the other ranks' shards in
    ascending rank order (separate buffers, read in place); returns [m*rank_size, n]."""
    m = a_local.shape[0]
    return _float_op(_l.ALLGATHER_MATMUL, a_local, b, lambda n: (m * rank_size, n), peer_shards, rank, rank_size,
                     tiling, False, trans_b, 0, None, None, acc_dump, block_num, stages, swizzle, linear_order, out, m,
                     workspace, split_k)


class PipelinedPlan:
    """The events of the round-pipelined operators, made once (catcoc_pipelined_plan_create) and reused by every call
    that is given the plan: such a call creates nothing and can be captured into a HIP graph."""

    def __init__(self, max_rounds):
        self.handle = _l.load().catcoc_pipelined_plan_create(int(max_rounds))
        if not self.handle:
            raise _l.CatcocError(_l.last_error())
        self.max_rounds = int(max_rounds)

    def close(self):
        if self.handle:
            _l.load().catcoc_pipelined_plan_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def pipelined_round_count(comm_type, tiling, rank, rank_size, block_num=0, stages=0):
    """Comm rounds a round-pipelined call with this tiling has (catcoc_pipelined_round_count)."""
    d = _l.make_desc(rank, rank_size, [16] * (rank_size - 1), block_num=block_num, stages=stages)
    n = _l.load().catcoc_pipelined_round_count(comm_type, C.byref(tiling), C.byref(d))
    _l.check()
    return n


def pipelined_quant_matmul_reduce_scatter(x1, x2, scale_x1, scale_x2, bias, peers, rank, rank_size, outbound, c_accum=None,
                                          out_dtype=torch.bfloat16, tiling=None, trans_b=False, peer_row_offset=0, deterministic=True,
                                          comm_stream=None, block_num=0, stages=0, swizzle=None, out=None, plan=None):
    """The W8A8 operator in the reference's round-pipelined form (catcoc_pipelined_quant_matmul_reduce_scatter): GEMM rounds
    on torch's current stream, comm rounds (int32 peers added into c_accum) and the dequant pass on comm_stream.
    peers: rank_size-1 int32 partials [m/rank_size, n]; outbound: the symmetric workspace (bytes per
    catcoc_get_workspace_size).  Returns (d_out, c_accum)."""
    _check_rank(rank, rank_size)
    _want(x1, "x1", torch.int8, 2)
    _want(x2, "x2", torch.int8, 2)
    m, k = x1.shape
    n = x2.shape[0] if trans_b else x2.shape[1]
    if (x2.shape[1] if trans_b else x2.shape[0]) != k:
        _fail("x2 has shape %s: its k extent does not match x1's k = %d", tuple(x2.shape), k)
    if m % rank_size != 0:
        _fail("reduce-scatter needs m %% rank_size == 0 (m=%d, rank_size=%d)", m, rank_size)
    rows = m // rank_size
    _want(scale_x1, "scale_x1", torch.float32, 1, m)
    _want(scale_x2, "scale_x2", torch.float32, 1, n)
    _want(bias, "bias", torch.int32, 1, n)
    _check_peers(list(peers), rank_size - 1, torch.int32, peer_row_offset + rows, n)
    _want(outbound, "outbound", (torch.int32, torch.float32))
    if c_accum is None:
        c_accum = torch.empty((rows, n), dtype=torch.int32, device=x1.device)
    _want(c_accum, "c_accum", torch.int32, 2, None, (rows, n))
    if out is None:
        out = torch.empty((rows, n), dtype=out_dtype, device=x1.device)
    _want(out, "out", (torch.float16, torch.bfloat16), 2, None, (rows, n))
    _check_dev(x1, x2, scale_x1, scale_x2, bias, outbound, c_accum, out, *peers)
    t = tiling if tiling is not None else default_tiling(m, k, n, rank_size, m0=0, n0=0, k0=0)
    d = _desc(rank, rank_size, list(peers), peer_row_offset, 0, block_num, stages, swizzle, outbound, None, None)
    if plan is not None:
        d.pipelinedPlan = plan.handle
    cs = comm_stream if comm_stream is not None else torch.cuda.current_stream()
    _l.load().catcoc_pipelined_quant_matmul_reduce_scatter(
        _stream(), cs.cuda_stream, 0, x1.data_ptr(), x2.data_ptr(), scale_x1.data_ptr(), scale_x2.data_ptr(), _ptr(bias),
        c_accum.data_ptr(), out.data_ptr(), C.addressof(d), C.byref(t), 0, int(trans_b), _TORCH_TO_DT[out.dtype], int(deterministic))
    _l.check()
    return out, c_accum


def pipelined_matmul_reduce_scatter(a, b, peers, rank, rank_size, outbound, tiling=None, trans_a=False, trans_b=False,
                                    peer_row_offset=0, deterministic=True, comm_stream=None, block_num=0, stages=0, swizzle=None,
                                    out=None, acc_dump=None, plan=None):
    """fp16 / bf16 reduce-scatter in the reference's round-pipelined form and precision: the local partial is rounded to the
    16-bit type, peers are 16-bit partials [m/rank_size, n] of the same type, every add rounds to that type."""
    if a.dtype not in _TORCH_TO_DT or b.dtype != a.dtype:
        _fail("a and b must both be float16 or both bfloat16")
    _check_rank(rank, rank_size)
    _want(a, "a", None, 2)
    _want(b, "b", None, 2)
    m = a.shape[1] if trans_a else a.shape[0]
    k = a.shape[0] if trans_a else a.shape[1]
    n = b.shape[0] if trans_b else b.shape[1]
    if (b.shape[1] if trans_b else b.shape[0]) != k:
        _fail("b has shape %s: its k extent does not match a's k = %d", tuple(b.shape), k)
    if m % rank_size != 0:
        _fail("reduce-scatter needs m %% rank_size == 0 (m=%d, rank_size=%d)", m, rank_size)
    rows = m // rank_size
    _check_peers(list(peers), rank_size - 1, a.dtype, peer_row_offset + rows, n)
    _want(outbound, "outbound", torch.float32)
    if out is None:
        out = torch.empty((rows, n), dtype=a.dtype, device=a.device)
    _want(out, "out", a.dtype, 2, None, (rows, n))
    _want(acc_dump, "acc_dump", torch.float32, None, m * n)
    _check_dev(a, b, outbound, out, acc_dump, *peers)
    t = tiling if tiling is not None else default_tiling(m, k, n, rank_size, m0=0, n0=0, k0=0)
    d = _desc(rank, rank_size, list(peers), peer_row_offset, 0, block_num, stages, swizzle, outbound, None, acc_dump)
    if plan is not None:
        d.pipelinedPlan = plan.handle
    cs = comm_stream if comm_stream is not None else torch.cuda.current_stream()
    _l.load().catcoc_pipelined_matmul_reduce_scatter(_stream(), cs.cuda_stream, _TORCH_TO_DT[a.dtype], a.data_ptr(), b.data_ptr(),
                                                     out.data_ptr(), C.addressof(d), C.byref(t), int(trans_a), int(trans_b), int(deterministic))
    _l.check()
    return out


def reduce_add(src, out_dtype=None, out=None):
    """SplitkMatmul's ReduceAdd: src [slices, ...] fp32 -> sum over the slices in slice order, cast once to out_dtype
    (None keeps fp32)."""
    _want(src, "src", torch.float32)
    if src.dim() < 2:
        _fail("src must have the slices as its first dimension")
    f, count = src.shape[0], src[0].numel()
    dt = torch.float32 if out_dtype is None else out_dtype
    if out is None:
        out = torch.empty(src.shape[1:], dtype=dt, device=src.device)
    _want(out, "out", dt, None, count)
    _check_dev(src, out)
    _l.load().catcoc_reduce_add(_stream(), out.data_ptr(), src.data_ptr(), count, f, 0 if dt == torch.float32 else _TORCH_TO_DT[dt])
    _l.check()
    return out


def verify(out, gold, dtype, compute_times):
    """The reference's accuracy gate on host data (float32 numpy arrays or CPU tensors).  -> (passed, n_bad, mean_rel_err)."""
    import numpy as np
    o = np.ascontiguousarray(out.numpy() if hasattr(out, "numpy") else out, dtype=np.float32).ravel()
    g = np.ascontiguousarray(gold.numpy() if hasattr(gold, "numpy") else gold, dtype=np.float32).ravel()
    if o.size != g.size:
        _fail("out has %d elements, gold %d", o.size, g.size)
    nb, eb = C.c_uint64(), C.c_double()
    okv = _l.load().catcoc_verify(o.ctypes.data, g.ctypes.data, o.size, _TORCH_TO_DT.get(dtype, dtype), compute_times, C.byref(nb), C.byref(eb))
    _l.check()
    return bool(okv), nb.value, eb.value


def kslice_plan(comm_type, dtype, m, k, n, rank=0, rank_size=1, tiling=None, split_k=0):
    """(workspace bytes, k slices) with which a launch of this shape would cut its tiles' k range; (0, 1) = it would not.
    m is the first dimension the operator's tiling takes (all-gather: one shard's rows)."""
    t = tiling if tiling is not None else default_tiling(m, k, n, rank_size, m0=0, n0=0, k0=0)
    d = _l.make_desc(rank, rank_size)
    d.splitK = split_k
    f = C.c_uint32(1)
    need = int(_l.load().catcoc_get_kslice_workspace_size(comm_type, _TORCH_TO_DT.get(dtype, _l.INT8), C.byref(t), C.byref(d), C.byref(f)))
    _l.check()
    return need, f.value


def device_info():
    cu, mhz = C.c_int(), C.c_int()
    name = C.create_string_buffer(64)
    if _l.load().catcoc_device_info(C.byref(cu), C.byref(mhz), name, 64) != 0:
        raise _l.CatcocError(_l.last_error())
    return {"cu_count": cu.value, "clock_mhz": mhz.value, "arch": name.value.decode()}
