"""MI355X-native per-rank fused GEMM path of CATCOC (matmul + all-reduce / all-gather /
reduce-scatter shares, W8A8 dequant + peer-reduce epilogue) behind a C ABI.

``lib`` loads ``libcatcoc_hip.so`` (hand-written gfx950 kernels) through ctypes and fails
loudly when it is missing; ``ops`` mirrors the reference's operator entry points on
torch tensors that live on the GPU.  There is no CPU path in this package.
"""
from . import lib  # noqa: F401
from .lib import (BF16, FP16, INT8, ALLGATHER_MATMUL, MATMUL_ALLREDUCE, MATMUL_REDUCE_SCATTER,  # noqa: F401
                  QUANT_MATMUL_REDUCE_SCATTER, CocTilingParams, CatcocSymmetricDesc, CatcocError)

__all__ = ["lib", "ops", "BF16", "FP16", "INT8", "ALLGATHER_MATMUL", "MATMUL_ALLREDUCE", "MATMUL_REDUCE_SCATTER",
           "QUANT_MATMUL_REDUCE_SCATTER", "CocTilingParams", "CatcocSymmetricDesc", "CatcocError"]
