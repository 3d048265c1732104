"""ctypes binding of libcatcoc_hip.so (declarations: include/catcoc_hip.h)."""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libcatcoc_hip.so")

# CocCommType / CocDataType of the reference (examples/dynamic_tiling/include/launch_map.h:6-16)
MATMUL_ALLREDUCE = 0
ALLGATHER_MATMUL = 1
MATMUL_REDUCE_SCATTER = 2
QUANT_MATMUL_REDUCE_SCATTER = 3
FP16 = 1
INT8 = 2
BF16 = 27

MAX_RANKS = 16
WORKSPACE_COUNTER_BYTES = 65536
STATIC_SCRATCH_BYTES = WORKSPACE_COUNTER_BYTES + (32 << 20)
DESC_MAGIC = 0x43544343
OUTBOUND_CHECKSUM = 0
OUTBOUND_STORE = 1
FLAG_REDUCE_INT32 = 4
FLAG_LINEAR_ORDER = 8
FLAG_KEPT_WHOLE = 0x10
FLAG_KEPT_SPLIT = 0x20
FLAG_TAIL_WHOLE = 0x40


class CatcocError(RuntimeError):
    pass


class CocTilingParams(C.Structure):
    """examples/dynamic_tiling/include/info.h:29-42."""
    _fields_ = [(n, C.c_uint32) for n in (
        "m", "k", "n", "m0", "k0", "n0", "commTileM", "commInterval",
        "commNpuSplit", "commDataSplit", "commBlockM", "rankSize")]


class CatcocSymmetricDesc(C.Structure):
    _fields_ = [
        ("magic", C.c_uint32), ("rankIdx", C.c_uint32), ("rankSize", C.c_uint32), ("blockNum", C.c_uint32),
        ("workspaceStages", C.c_uint32), ("swizzleOffset", C.c_uint32), ("swizzleDirection", C.c_uint32),
        ("flags", C.c_uint32), ("keptRowBegin", C.c_uint32), ("keptRows", C.c_uint32), ("splitK", C.c_uint32),
        ("peers", C.c_void_p * MAX_RANKS),
        ("peerLd", C.c_int64), ("peerRowOffset", C.c_int64),
        ("outbound", C.c_void_p), ("outboundBytes", C.c_uint64),
        ("checksum", C.c_void_p), ("accDump", C.c_void_p),
        ("workspace", C.c_void_p), ("workspaceBytes", C.c_uint64),
        ("pipelinedPlan", C.c_void_p),
    ]


KernelFuncPtr = C.CFUNCTYPE(None, C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                            C.c_void_p, C.POINTER(CocTilingParams), C.c_uint32, C.c_uint32)

_LAUNCHER_ARGS = [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                  C.POINTER(CocTilingParams), C.c_uint32, C.c_uint32]

# every symbol include/catcoc_hip.h declares
EXPORTS = [
    "catcoc_get_kernel",
    "catcoc_launch_matmul_allreduce_fp16", "catcoc_launch_matmul_allreduce_bf16",
    "catcoc_launch_allgather_matmul_fp16", "catcoc_launch_allgather_matmul_bf16",
    "catcoc_launch_matmul_reduce_scatter_fp16", "catcoc_launch_matmul_reduce_scatter_bf16",
    "catcoc_quant_matmul_reduce_scatter", "catcoc_launch_quant_matmul_reduce_scatter",
    "catcoc_launch_quant_matmul_reduce_scatter_static_scratch",
    "catcoc_last_error", "catcoc_last_status", "catcoc_can_implement", "catcoc_get_workspace_size",
    "catcoc_get_splitk_workspace_size", "catcoc_get_kslice_workspace_size",
    "catcoc_get_task_count", "catcoc_get_tilings", "catcoc_check_comm_interval_reduce_scatter",
    "catcoc_check_comm_interval_allreduce", "catcoc_check_comm_interval_allgather", "catcoc_get_splitk_factor",
    "catcoc_default_tiling", "catcoc_swizzle_block_coord", "catcoc_splitk_block_coord", "catcoc_splitk_actual_k", "catcoc_splitk_launch_task",
    "catcoc_allgather_block_coord", "catcoc_comm_block_idx", "catcoc_task_tile", "catcoc_workgroup_task", "catcoc_launch_task", "catcoc_launch_tile", "catcoc_kept_split_tiles", "catcoc_tail_split_tiles",
    "catcoc_device_info", "catcoc_version",
    "catcoc_pipelined_quant_matmul_reduce_scatter", "catcoc_pipelined_matmul_reduce_scatter", "catcoc_reduce_add",
    "catcoc_verify", "catcoc_comm_block_idx_ex", "catcoc_comm_core_loop", "catcoc_task_tiles",
    "catcoc_pipelined_plan_create", "catcoc_pipelined_plan_destroy", "catcoc_pipelined_round_count",
]

_lib = None


def _preload_hip_runtime():
    """libcatcoc_hip.so names no HIP runtime of its own; it binds to the one already in the process.
    Make that runtime's symbols global first: torch's bundled copy when torch is importable (so that the
    library and torch share one runtime and one set of streams), else the system ROCm one."""
    import sys
    cands = []
    try:
        import torch  # noqa: F401  (device memory and streams come from torch in this package)
        cands.append(os.path.join(os.path.dirname(sys.modules["torch"].__file__), "lib", "libamdhip64.so"))
    except ImportError:
        pass
    cands += ["/opt/rocm/lib/libamdhip64.so", "libamdhip64.so"]
    for c in cands:
        try:
            C.CDLL(c, mode=C.RTLD_GLOBAL)
            return c
        except OSError:
            continue
    raise CatcocError("no HIP runtime (libamdhip64.so) could be loaded")


def load():
    """Load libcatcoc_hip.so.  There is no fallback: a missing library is an error."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise CatcocError(
            "libcatcoc_hip.so is not built (%s). Build it with `python -m mm_rs_with_catlass_amd._build` "
            "or __graft_entry__.build()." % LIB_PATH)
    _preload_hip_runtime()
    L = C.CDLL(LIB_PATH)
    u32, vp = C.c_uint32, C.c_void_p
    pu = C.POINTER(u32)
    for name in EXPORTS:
        if name.startswith("catcoc_launch_") and not name.startswith("catcoc_launch_quant_") and name not in (
                "catcoc_launch_task", "catcoc_launch_tile"):
            f = getattr(L, name)
            f.argtypes = _LAUNCHER_ARGS
            f.restype = None
    L.catcoc_get_kernel.argtypes = [C.c_int, C.c_int]
    L.catcoc_get_kernel.restype = C.c_void_p
    L.catcoc_quant_matmul_reduce_scatter.argtypes = [vp, C.c_uint64] + [vp] * 8 + [u32, u32, u32]
    L.catcoc_quant_matmul_reduce_scatter.restype = None
    L.catcoc_launch_quant_matmul_reduce_scatter.argtypes = [vp, C.c_uint64] + [vp] * 8 + [
        C.POINTER(CocTilingParams), u32, u32, u32]
    L.catcoc_launch_quant_matmul_reduce_scatter.restype = None
    L.catcoc_launch_quant_matmul_reduce_scatter_static_scratch.argtypes = L.catcoc_launch_quant_matmul_reduce_scatter.argtypes
    L.catcoc_launch_quant_matmul_reduce_scatter_static_scratch.restype = None
    L.catcoc_last_error.restype = C.c_char_p
    L.catcoc_last_status.restype = C.c_int
    L.catcoc_can_implement.argtypes = [C.c_int, C.c_int, C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc), u32, u32]
    L.catcoc_can_implement.restype = C.c_int
    L.catcoc_get_workspace_size.argtypes = [C.c_int, C.c_int, C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc)]
    L.catcoc_get_workspace_size.restype = C.c_uint64
    L.catcoc_get_kslice_workspace_size.argtypes = [C.c_int, C.c_int, C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc), pu]
    L.catcoc_get_kslice_workspace_size.restype = C.c_uint64
    L.catcoc_get_splitk_workspace_size.argtypes = [C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc), pu, pu]
    L.catcoc_get_splitk_workspace_size.restype = C.c_uint64
    L.catcoc_launch_task.argtypes = [C.c_int, C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc), u32]
    L.catcoc_launch_task.restype = u32
    L.catcoc_kept_split_tiles.argtypes = [C.c_int, C.c_int, C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc), u32, u32]
    L.catcoc_kept_split_tiles.restype = u32
    L.catcoc_tail_split_tiles.argtypes = [C.c_int, C.c_int, C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc), u32, u32]
    L.catcoc_tail_split_tiles.restype = u32
    L.catcoc_get_task_count.argtypes = [C.c_int, C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc)]
    L.catcoc_get_task_count.restype = u32
    L.catcoc_get_tilings.argtypes = [C.POINTER(CocTilingParams), C.c_int, C.c_int, C.c_int, C.POINTER(CocTilingParams), C.c_int]
    L.catcoc_get_tilings.restype = C.c_int
    for n in ("catcoc_check_comm_interval_reduce_scatter", "catcoc_check_comm_interval_allreduce"):
        getattr(L, n).argtypes = [C.POINTER(CocTilingParams), C.c_int, C.c_int]
        getattr(L, n).restype = C.c_int
    L.catcoc_check_comm_interval_allgather.argtypes = [C.POINTER(CocTilingParams), C.c_int]
    L.catcoc_check_comm_interval_allgather.restype = C.c_int
    L.catcoc_get_splitk_factor.argtypes = [u32] * 7
    L.catcoc_get_splitk_factor.restype = u32
    L.catcoc_default_tiling.argtypes = [C.POINTER(CocTilingParams), u32, u32, u32, u32]
    L.catcoc_default_tiling.restype = None
    L.catcoc_swizzle_block_coord.argtypes = [u32] * 5 + [pu, pu]
    L.catcoc_splitk_block_coord.argtypes = [u32] * 7 + [pu] * 4
    L.catcoc_splitk_actual_k.argtypes = [u32] * 4
    L.catcoc_splitk_actual_k.restype = u32
    L.catcoc_splitk_launch_task.argtypes = [u32] * 6
    L.catcoc_splitk_launch_task.restype = u32
    L.catcoc_allgather_block_coord.argtypes = [u32] * 7 + [pu, pu]
    L.catcoc_comm_block_idx.argtypes = [u32] * 6 + [pu, pu]
    L.catcoc_task_tile.argtypes = [C.c_int, C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc), u32] + [pu] * 4
    L.catcoc_task_tile.restype = C.c_int
    L.catcoc_launch_tile.argtypes = [C.c_int, C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc), u32] + [pu] * 5
    L.catcoc_launch_tile.restype = C.c_int
    L.catcoc_workgroup_task.argtypes = [u32, u32, u32]
    L.catcoc_workgroup_task.restype = u32
    L.catcoc_device_info.argtypes = [C.POINTER(C.c_int), C.POINTER(C.c_int), C.c_char_p, C.c_int]
    L.catcoc_device_info.restype = C.c_int
    L.catcoc_version.restype = C.c_char_p
    L.catcoc_pipelined_quant_matmul_reduce_scatter.argtypes = [vp, vp, C.c_uint64] + [vp] * 8 + [C.POINTER(CocTilingParams), u32, u32, u32, u32]
    L.catcoc_pipelined_quant_matmul_reduce_scatter.restype = None
    L.catcoc_pipelined_matmul_reduce_scatter.argtypes = [vp, vp, C.c_int] + [vp] * 4 + [C.POINTER(CocTilingParams), u32, u32, u32]
    L.catcoc_pipelined_matmul_reduce_scatter.restype = None
    L.catcoc_reduce_add.argtypes = [vp, vp, vp, C.c_uint64, u32, u32]
    L.catcoc_reduce_add.restype = None
    L.catcoc_verify.argtypes = [vp, vp, C.c_uint64, C.c_int, u32, C.POINTER(C.c_uint64), C.POINTER(C.c_double)]
    L.catcoc_verify.restype = C.c_int
    L.catcoc_comm_block_idx_ex.argtypes = [u32] * 7 + [pu, pu]
    L.catcoc_comm_block_idx_ex.restype = None
    L.catcoc_comm_core_loop.argtypes = [u32] * 5
    L.catcoc_comm_core_loop.restype = u32
    L.catcoc_task_tiles.argtypes = [C.c_int, C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc), u32, u32] + [pu] * 4
    L.catcoc_task_tiles.restype = u32
    L.catcoc_pipelined_plan_create.argtypes = [u32]
    L.catcoc_pipelined_plan_create.restype = vp
    L.catcoc_pipelined_plan_destroy.argtypes = [vp]
    L.catcoc_pipelined_plan_destroy.restype = None
    L.catcoc_pipelined_round_count.argtypes = [C.c_int, C.POINTER(CocTilingParams), C.POINTER(CatcocSymmetricDesc)]
    L.catcoc_pipelined_round_count.restype = u32
    _lib = L
    return L


def last_error():
    return load().catcoc_last_error().decode()


def check():
    """Raise CatcocError if the last launcher call on this thread was rejected."""
    L = load()
    if L.catcoc_last_status() != 0:
        raise CatcocError(L.catcoc_last_error().decode())


def make_desc(rank, rank_size, peers=(), peer_ld=0, peer_row_offset=0, flags=0, block_num=0, stages=0,
              swizzle=None, outbound=None, outbound_bytes=0, checksum=None, acc_dump=None):
    """Build a CatcocSymmetricDesc from raw device addresses (ints)."""
    d = CatcocSymmetricDesc()
    d.magic = DESC_MAGIC
    d.rankIdx = rank
    d.rankSize = rank_size
    d.blockNum = block_num
    d.workspaceStages = stages
    if swizzle is not None:
        d.swizzleOffset, d.swizzleDirection = swizzle
    d.flags = flags
    for i, p in enumerate(peers):
        d.peers[i] = p
    d.peerLd = peer_ld
    d.peerRowOffset = peer_row_offset
    d.outbound = outbound
    d.outboundBytes = outbound_bytes
    d.checksum = checksum
    d.accDump = acc_dump
    return d
