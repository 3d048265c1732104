/*
 * catcoc_hip.h -- C ABI of libcatcoc_hip.so: the per-rank fused GEMM path of
 * CATCOC (tile GEMM + dequant + peer-partial reduce epilogue) for AMD MI355X
 * (gfx950), on ONE GPU.  Peer ranks' data are buffers staged in this GPU's HBM.
 *
 * Every entry point names the reference interface it stands in for (paths are
 * relative to the reference tree).  Plain C types only; `stream` is a
 * hipStream_t passed as void*.  All launches are asynchronous on `stream`; the
 * caller owns every buffer and the library allocates nothing on a launch.
 */
#ifndef CATCOC_HIP_H
#define CATCOC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CATCOC_API __attribute__((visibility("default")))

/* ----------------------------------------------------------------------- */
/* Types kept binary-identical to the reference                              */
/* ----------------------------------------------------------------------- */

/* examples/dynamic_tiling/include/info.h:29-42 -- twelve uint32_t, same order.
 * m,k,n: problem (for ALLGATHER_MATMUL m is the rows of ONE rank's shard).
 * m0,n0,k0: workgroup macro tile; 0 lets the library choose (m0: 64 for at most 64 rows per rank, else 128, or 256 when
 * the problem is whole 256x256 tiles, 512 or more of them with 4 KiB or more of k per row, or 1024 with 2 KiB; the choice does not depend on the
 * operands' layouts, so catcoc_get_task_count / catcoc_get_workspace_size see the same tiles as the launch).
 * commInterval x blockNum: tiles per scheduling round (blockNum, the
 * reference's BLOCK_NUM = 20 AI cores, comes from CatcocSymmetricDesc).
 * commTileM, commBlockM, commNpuSplit, commDataSplit: comm-epilogue chunking of
 * the reference; accepted, validated like the reference does, and otherwise
 * unused because the reduce runs in registers in the GEMM's own epilogue. */
typedef struct CocTilingParams {
    uint32_t m;
    uint32_t k;
    uint32_t n;
    uint32_t m0;
    uint32_t k0;
    uint32_t n0;
    uint32_t commTileM;
    uint32_t commInterval;
    uint32_t commNpuSplit;
    uint32_t commDataSplit;
    uint32_t commBlockM;
    uint32_t rankSize;
} CocTilingParams;

/* examples/dynamic_tiling/include/launch_map.h:6-11 (values 0..2 unchanged). */
typedef enum CocCommType {
    MATMUL_ALLREDUCE = 0,
    ALLGATHER_MATMUL = 1,
    MATMUL_REDUCE_SCATTER = 2,
    QUANT_MATMUL_REDUCE_SCATTER = 3, /* examples/02_matmul_reduce_scatter/quant_matmul_reduce_scatter.cpp */
    TYPE_NUM
} CocCommType;

/* examples/dynamic_tiling/include/launch_map.h:13-16; INT8 = 2 is the ACL code. */
typedef enum CocDataType {
    FP16 = 1,
    INT8 = 2,
    BF16 = 27
} CocDataType;

/* examples/dynamic_tiling/include/launch_map.h:18-19  KernelFuncPtr.  The C++
 * reference passes `CocTilingParams &`; at the ABI level that is this pointer.
 * aW, bW are reserved and ignored (examples/dynamic_tiling/impl/kernel_fp16.cpp:29-30).
 * fftsAddr is accepted and ignored (no cross-core flags on a GPU).
 *   MATMUL_ALLREDUCE     : a [m,k], b [k,n], c [m,n]
 *   ALLGATHER_MATMUL     : a [m,k] = this rank's shard, b [k,n], c [m*rankSize,n]
 *   MATMUL_REDUCE_SCATTER: a [m,k], b [k,n], c [m/rankSize,n]
 * transA / transB != 0 mean the operand is stored transposed ([k,m] / [n,k]),
 * the ColumnMajor instantiations of kernel_fp16.cpp:31-43.
 * symmetricPtr points at a CatcocSymmetricDesc in HOST memory (see below). */
typedef void (*CatcocKernelFuncPtr)(void *stream, uint64_t fftsAddr, uint8_t *a, uint8_t *b, uint8_t *c,
                                    uint8_t *aW, uint8_t *bW, uint8_t *symmetricPtr, CocTilingParams *tiling,
                                    uint32_t transA, uint32_t transB);

/* ----------------------------------------------------------------------- */
/* One-GPU stand-in for the symmetric heap                                   */
/* ----------------------------------------------------------------------- */

#define CATCOC_MAX_RANKS 16
#define CATCOC_WORKSPACE_COUNTER_BYTES 65536u /* counter block at the start of CatcocSymmetricDesc.workspace */
#define CATCOC_DESC_MAGIC 0x43544343u /* "CCTC" */

/* What happens to tiles whose rows belong to another rank (the reference stores
 * them to the symmetric workspace, quant_matmul_reduce_scatter.hpp:196-201). */
#define CATCOC_OUTBOUND_CHECKSUM 0u /* fold each tile's accumulators into `checksum` (keeps the MACs observable) */
#define CATCOC_OUTBOUND_STORE 1u    /* store the tile to `outbound` in the reference's tile-linear layout, as fp32
                                       (dequantised for W8A8), or int32 when CATCOC_FLAG_REDUCE_INT32 is set */
#define CATCOC_OUTBOUND_MASK 0x3u
/* W8A8 only: peers hold int32 partials that are added BEFORE the dequant (the
 * reference's order, quant_matmul_reduce_scatter.hpp:285-351); default is fp32
 * partials added after the dequant. */
#define CATCOC_FLAG_REDUCE_INT32 0x4u
/* Keep the linear workgroup -> task order (no XCD-aware chunking). */
#define CATCOC_FLAG_LINEAR_ORDER 0x8u
/* Reduce-scatter launches of one round of workgroups (at most 512 tiles of 128x256 with at most 80 k steps of 64 bytes,
 * or fewer than 256 tiles) run every kept tile as two 64-row workgroups, which halves the chain of peer partials a
 * workgroup adds; the library decides by those two numbers.  KEPT_WHOLE never splits, KEPT_SPLIT splits whenever the launch allows it (whole
 * tiles, A as [m,k], XCD-aware order): tuning knobs like the tiling's, results are bit-identical either way. */
#define CATCOC_FLAG_KEPT_WHOLE 0x10u
#define CATCOC_FLAG_KEPT_SPLIT 0x20u
/* A launch with split kept tiles has more workgroups than the GPU has slots for; the tiles that wait for a slot (they get the
 * ones the kept halves leave) run as two 64-row workgroups as well, unless this flag is set.  With checksums (the default
 * outbound mode) the two halves of such a task meet through the counter block of desc.workspace: without a workspace of at
 * least CATCOC_WORKSPACE_COUNTER_BYTES (zeroed once, shared like any other) they stay whole.  Results are bit-identical. */
#define CATCOC_FLAG_TAIL_WHOLE 0x40u

/* Replaces the reference's `symmetricPtr` workspace + shmem_my_pe()/shmem_n_pes()
 * (examples/dynamic_tiling/impl/kernel/matmul_reduce_scatter.h:155-156): which
 * rank this GPU plays and where the other ranks' staged data live.  Zero-filled
 * fields take the documented defaults. */
struct CatcocPipelinedPlan;
typedef struct CatcocSymmetricDesc {
    uint32_t magic;           /* CATCOC_DESC_MAGIC */
    uint32_t rankIdx;         /* shmem_my_pe() */
    uint32_t rankSize;        /* shmem_n_pes(); must match tiling.rankSize when that is non-zero */
    uint32_t blockNum;        /* BLOCK_NUM of the schedule; 0 = 256 (one per CU) */
    uint32_t workspaceStages; /* WORKSPACE_STAGES; 0 = 2 */
    uint32_t swizzleOffset;   /* GemmIdentityBlockSwizzle<offset,direction>; 0 = <7,1> as in every example */
    uint32_t swizzleDirection;
    uint32_t flags;           /* CATCOC_OUTBOUND_* | CATCOC_FLAG_* */
    uint32_t keptRowBegin;    /* keptRows == 0: the rank keeps rows [rankIdx*m/rankSize, +m/rankSize) as in the reference. */
    uint32_t keptRows;        /* keptRows != 0 (W8A8 only): the rank keeps rows [keptRowBegin, +keptRows) of an m that need not
                                 divide by rankSize, and the launch takes the skinny-M split-K path (decode shapes) */
    uint32_t splitK;          /* k slices per tile; 0 = the library's choice (split-K path: GetSplitkFactor with blockNum cores
                                 and 128x128x256 tiles; large-tile kernel: see catcoc_get_kslice_workspace_size) */
    /* Reduce paths: peers[s], s = 0..rankSize-2, are the other ranks' partial
     * results for this rank's kept rows (fp32, or int32 with REDUCE_INT32), added
     * in slot order after the local partial.  Row `peerRowOffset + i` of a peer
     * buffer lines up with kept row i; peerLd is its leading dimension in elements.
     * ALLGATHER_MATMUL: peers[s] are the other ranks' A shards in ascending rank
     * order (this rank's own shard is the `a` argument), each [m,k], read in place. */
    const void *peers[CATCOC_MAX_RANKS];
    int64_t peerLd;
    int64_t peerRowOffset;
    void *outbound;           /* OUTBOUND_STORE target, rows (stage*blockPerComm + blockIdxInComm)*m0, n0 columns */
    uint64_t outboundBytes;   /* capacity of `outbound` */
    int64_t *checksum;        /* OUTBOUND_CHECKSUM target: one int64 per task (W8A8) / one double per task (float) */
    void *accDump;            /* optional full [m,n] int32 (W8A8) or fp32 (float) local partial, for bit-exact checks */
    /* Scratch in HBM for launches whose k range is cut into slices: the skinny-M split-K path
     * (catcoc_get_splitk_workspace_size() bytes) and few-tile launches of the large-tile kernel
     * (catcoc_get_kslice_workspace_size() bytes, optional there).  256-byte aligned.  Layout: the first
     * CATCOC_WORKSPACE_COUNTER_BYTES hold one arrival counter per tile, at the same place for every shape and slice
     * count; the partial tiles follow.  The caller ZEROES the counter block (or simply the whole buffer) once before
     * the first use; every launch leaves the counters at zero again, so launches of any shapes may share one
     * workspace that is large enough for each of them.  Launches that share a workspace must not overlap (same
     * stream, or ordered by events). */
    void *workspace;
    uint64_t workspaceBytes;
    /* Round-pipelined operators only: the events they order their two streams with, made once by
     * catcoc_pipelined_plan_create and reused by every call that is given the plan (NULL = the call makes and destroys
     * its own).  Calls that share a plan must not overlap. */
    struct CatcocPipelinedPlan *pipelinedPlan;
} CatcocSymmetricDesc;

/* ----------------------------------------------------------------------- */
/* Registry and launchers                                                    */
/* ----------------------------------------------------------------------- */

/* KernelDispatcher::GetKernelFunc (examples/dynamic_tiling/include/launch_map.h:35-42).
 * Returns NULL for an unregistered (commType, dataType) pair, as the reference does. */
CATCOC_API CatcocKernelFuncPtr catcoc_get_kernel(int commType, int dataType);

/* LaunchMatmulAllReduceFP16 / BF16      (examples/dynamic_tiling/impl/kernel_fp16.cpp:22-44, kernel_bf16.cpp) */
CATCOC_API void catcoc_launch_matmul_allreduce_fp16(void *stream, uint64_t fftsAddr, uint8_t *a, uint8_t *b,
    uint8_t *c, uint8_t *aW, uint8_t *bW, uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA,
    uint32_t transB);
CATCOC_API void catcoc_launch_matmul_allreduce_bf16(void *stream, uint64_t fftsAddr, uint8_t *a, uint8_t *b,
    uint8_t *c, uint8_t *aW, uint8_t *bW, uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA,
    uint32_t transB);
/* LaunchAllGatherMatmulFP16 / BF16      (kernel_fp16.cpp:46-62) */
CATCOC_API void catcoc_launch_allgather_matmul_fp16(void *stream, uint64_t fftsAddr, uint8_t *a, uint8_t *b,
    uint8_t *c, uint8_t *aW, uint8_t *bW, uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA,
    uint32_t transB);
CATCOC_API void catcoc_launch_allgather_matmul_bf16(void *stream, uint64_t fftsAddr, uint8_t *a, uint8_t *b,
    uint8_t *c, uint8_t *aW, uint8_t *bW, uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA,
    uint32_t transB);
/* LaunchMatmulReduceScatterFP16 / BF16  (kernel_fp16.cpp:64-86) */
CATCOC_API void catcoc_launch_matmul_reduce_scatter_fp16(void *stream, uint64_t fftsAddr, uint8_t *a, uint8_t *b,
    uint8_t *c, uint8_t *aW, uint8_t *bW, uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA,
    uint32_t transB);
CATCOC_API void catcoc_launch_matmul_reduce_scatter_bf16(void *stream, uint64_t fftsAddr, uint8_t *a, uint8_t *b,
    uint8_t *c, uint8_t *aW, uint8_t *bW, uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA,
    uint32_t transB);

/* ShmemQuantMatmulReduceScatter<<<...>>>(fftsAddr, x1, x2, scale_x1, scale_x2, bias, c_accum, d_out,
 * symmetricPtr, m, n, k)   (examples/02_matmul_reduce_scatter/quant_matmul_reduce_scatter.cpp:54-60).
 * x1 [m,k] int8, x2 [k,n] int8, scale_x1 [m] fp32 per token, scale_x2 [n] fp32 per channel,
 * bias [n] int32 or NULL, c_accum [m/P,n] int32 or NULL (receives the kept block's local
 * accumulators incl. bias), d_out [m/P,n].  Fixed configuration of the example:
 * tile 128x256, commInterval 10, swizzle <7,1>; rank and rankSize come from the descriptor.
 * d_out is bf16 (the kernel's ElementD, quant_matmul_reduce_scatter.hpp:48). */
CATCOC_API void catcoc_quant_matmul_reduce_scatter(void *stream, uint64_t fftsAddr, uint8_t *x1, uint8_t *x2,
    uint8_t *scale_x1, uint8_t *scale_x2, uint8_t *bias, uint8_t *c_accum, uint8_t *d_out, uint8_t *symmetricPtr,
    uint32_t m, uint32_t n, uint32_t k);

/* Same operator driven by CocTilingParams, as the dynamic_tiling wrappers do for the float ops
 * (examples/dynamic_tiling/impl/kernel/matmul_reduce_scatter.h:126-170).  outDataType is FP16 or
 * BF16 (the example instantiates the dequant epilogue with half, quant_matmul_reduce_scatter.cpp:129). */
CATCOC_API void catcoc_launch_quant_matmul_reduce_scatter(void *stream, uint64_t fftsAddr, uint8_t *x1, uint8_t *x2,
    uint8_t *scale_x1, uint8_t *scale_x2, uint8_t *bias, uint8_t *c_accum, uint8_t *d_out, uint8_t *symmetricPtr,
    CocTilingParams *tiling, uint32_t transA, uint32_t transB, uint32_t outDataType);

/* The same operator for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Arguments and results are exactly those
 * of catcoc_launch_quant_matmul_reduce_scatter, except that desc->workspace / workspaceBytes are ignored: launches that
 * cut their k range into slices (the skinny-M split-K path; few-tile launches of the large-tile kernel) meet through a
 * scratch array built into the library, CATCOC_STATIC_SCRATCH_BYTES per GPU, which each GPU the library runs on holds
 * until the process ends.  The call allocates nothing.  A launch that needs more scratch than that is rejected
 * (catcoc_last_error() says how much it needs).  All calls on one GPU share that GPU's array: calls that overlap on
 * one GPU (different streams, no ordering between them) race; calls on one stream, or ordered by events, are fine.
 * Nothing is cleared at run time: the array is zero when the library's code is loaded on a GPU, and every launch leaves
 * its counter block at zero again for the next, also when it is replayed from a HIP graph. */
#define CATCOC_STATIC_SCRATCH_BYTES (CATCOC_WORKSPACE_COUNTER_BYTES + (32u << 20))
CATCOC_API void catcoc_launch_quant_matmul_reduce_scatter_static_scratch(void *stream, uint64_t fftsAddr, uint8_t *x1,
    uint8_t *x2, uint8_t *scale_x1, uint8_t *scale_x2, uint8_t *bias, uint8_t *c_accum, uint8_t *d_out,
    uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA, uint32_t transB, uint32_t outDataType);

/* ----------------------------------------------------------------------- */
/* Round-pipelined, reference-faithful form                                  */
/* ----------------------------------------------------------------------- */

/* The reduce-scatter operators with the reference's own structure instead of the fused epilogue
 * (include/catcoc/dgemm/kernel/quant_matmul_reduce_scatter.hpp:159-164,219,282,319 and matmul_reduce_scatter.hpp:155-199,
 * 237-296): comm rounds of blockNum x commInterval tiles; per round the GEMM (on computeStream) stores the round's tiles --
 * the kept rank's into the local block, the others into stage `round % workspaceStages` of desc->outbound in the
 * tile-linear layout -- then the comm side (on commStream) adds the peers' blocks into the local block along
 * BlockCommSwizzle's task list; the GEMM of round + workspaceStages waits for that before it reuses the stage.  The two
 * cross-core flags per stage are HIP events between the two streams (created and destroyed inside the call unless the
 * descriptor names a CatcocPipelinedPlan, below); on return
 * computeStream is ordered after the finished output.  commBlockM (0 = 64) must divide m0; commDataSplit x commNpuSplit
 * is the number of comm "cores" (workgroups), raised to 256 x 1 when below 16.
 *   W8A8: int32 tiles; peers[] are int32 partials [m/P, n] added into c_accum (required, receives the reduced int32
 *   block) with integer adds, then one dequant pass writes d_out (quant_matmul_reduce_scatter.hpp:285-351).  Bit-identical
 *   to catcoc_launch_quant_matmul_reduce_scatter with CATCOC_FLAG_REDUCE_INT32.
 *   fp16 / bf16: the local partial is rounded to the output type and peers[] are 16-bit partials [m/P, n] of that type,
 *   each added with one rounding to that type (matmul_reduce_scatter.hpp:261; the fp32 -> 16-bit cast of
 *   3rdparty/catlass/include/catlass/gemm/tile/copy_l0c_to_gm.hpp:39-57).
 * deterministic != 0 runs BlockCommSwizzle<0, true> (comm_block_swizzle.hpp:25-31,54-56,114-118): one core owns a data
 * block and adds the ranks in the order (dataIdx + i) % rankSize, so 16-bit results are reproducible; 0 runs
 * BlockCommSwizzle<0, false> with hardware atomic adds in arrival order, like the reference. */
CATCOC_API void catcoc_pipelined_quant_matmul_reduce_scatter(void *computeStream, void *commStream, uint64_t fftsAddr,
    uint8_t *x1, uint8_t *x2, uint8_t *scale_x1, uint8_t *scale_x2, uint8_t *bias, uint8_t *c_accum, uint8_t *d_out,
    uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA, uint32_t transB, uint32_t outDataType,
    uint32_t deterministic);
CATCOC_API void catcoc_pipelined_matmul_reduce_scatter(void *computeStream, void *commStream, int dataType, uint8_t *a,
    uint8_t *b, uint8_t *c, uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA, uint32_t transB,
    uint32_t deterministic);

/* The events of the round-pipelined operators as an object of the caller's.  The reference needs nothing of the kind:
 * its two flags per workspace stage live in the symmetric workspace and the one kernel waits on them itself
 * (quant_matmul_reduce_scatter.hpp:159-164,219,282,319); here they are HIP events between two streams, and a call that
 * has to create them cannot run under stream capture or in a loop that must not allocate.  A plan holds the events for
 * calls of up to maxRounds comm rounds (catcoc_pipelined_round_count says how many a call has) on the device that is
 * current when it is made; a call whose descriptor names the plan creates and destroys nothing, so it can be captured
 * into a HIP graph (capture on computeStream; commStream joins the capture through the first event and is joined back
 * before the call returns).  catcoc_pipelined_plan_create returns NULL on failure (catcoc_last_error() says why). */
typedef struct CatcocPipelinedPlan CatcocPipelinedPlan;
CATCOC_API CatcocPipelinedPlan *catcoc_pipelined_plan_create(uint32_t maxRounds);
CATCOC_API void catcoc_pipelined_plan_destroy(CatcocPipelinedPlan *plan);
/* Comm rounds of a round-pipelined call with this tiling and descriptor: ceil(tasks / (blockNum * commInterval)); 0 on error. */
CATCOC_API uint32_t catcoc_pipelined_round_count(int commType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc);

/* SplitkMatmul's ReduceAdd as a kernel of its own (3rdparty/catlass/include/catlass/gemm/kernel/splitk_matmul.hpp:24-161):
 * src holds splitkFactor fp32 slices of elementCount elements each, back to back; dst[i] = the slices' sum in slice order
 * (fp32 adds), rounded once to outDataType (FP16 / BF16, or 0 to keep fp32).  16-byte aligned buffers. */
CATCOC_API void catcoc_reduce_add(void *stream, uint8_t *dst, uint8_t *src, uint64_t elementCount, uint32_t splitkFactor,
                                  uint32_t outDataType);

/* The reference's accuracy gate (examples/utils/verify_result.py:26-43,88-117 with the tolerances of
 * examples/utils/utils.py:44-52) on host arrays: every element |out - gold| <= rtol * max(1, |gold|) with
 * rtol = 2^-8 (fp16) / 2^-7 (bf16) for computeTimes < 2048 and twice that otherwise, and
 * |mean((out - gold) / max(1, |gold|))| <= 2^-10 (fp16) / 2^-7 (bf16); NaN and Inf count as 0.  Returns 1 on pass. */
CATCOC_API int catcoc_verify(const float *out, const float *gold, uint64_t count, int dataType, uint32_t computeTimes,
                             uint64_t *nBad, double *meanRelErr);

/* ----------------------------------------------------------------------- */
/* Validation, errors, sizes                                                 */
/* ----------------------------------------------------------------------- */

/* The launchers return void like the reference's; a rejected call launches nothing and records
 * an error.  catcoc_last_error(): message of the calling thread's last rejected call ("" if none);
 * catcoc_last_status(): 0 = the last call on this thread was accepted. */
CATCOC_API const char *catcoc_last_error(void);
CATCOC_API int catcoc_last_status(void);

/* Catlass::Status-style pre-flight check (3rdparty/catlass/include/catlass/gemm/device/device_gemm.hpp:46-53):
 * 0 if the launcher would accept these arguments, else non-zero with catcoc_last_error() set. */
CATCOC_API int catcoc_can_implement(int commType, int dataType, const CocTilingParams *tiling,
                                    const CatcocSymmetricDesc *desc, uint32_t transA, uint32_t transB);

/* Bytes of `outbound` needed for OUTBOUND_STORE with this tiling / descriptor (the reference
 * sizes layoutSymmetric = m0*commInterval*BLOCK_NUM*WORKSPACE_STAGES x n0, matmul_reduce_scatter.h:161). */
CATCOC_API uint64_t catcoc_get_workspace_size(int commType, int dataType, const CocTilingParams *tiling,
                                              const CatcocSymmetricDesc *desc);

/* Launches with few 128x256 tiles (fewer than half the CUs' worth) can cut every tile's k range into k slices, one
 * workgroup each, that meet through `workspace` (partial tiles in 32-bit words + one counter per tile, zeroed once
 * by the caller, re-armed by every launch): returns the bytes needed and the slice count (1 and 0 bytes when the
 * launch would not be sliced: other tile shapes, ragged problems, enough tiles already; the operands' layouts do
 * not matter).  The count
 * is 2, 4 or 8 for W8A8 (integer partials add exactly) and 2 for fp16/bf16; desc->splitK, when non-zero, is taken as the
 * caller's own count (up to 8; three or more fp32 partials are added in slice order whichever slice arrives last, so
 * the result is reproducible for any count).  A launch
 * slices only when `workspace` is given.  Counterpart in the reference: SplitkMatmul's k split
 * (3rdparty/catlass/include/catlass/gemm/kernel/splitk_matmul.hpp:68-148), which its communication kernels do not
 * use. */
CATCOC_API uint64_t catcoc_get_kslice_workspace_size(int commType, int dataType, const CocTilingParams *tiling,
                                                     const CatcocSymmetricDesc *desc, uint32_t *kSlices);

/* Split-K path (descriptor with keptRows != 0): bytes of `workspace` the launch needs (0 when the split factor
 * is 1), the split factor it will use and its number of 128x128 tiles (`checksum`, if given, needs one int64 per
 * tile and receives the sum of the accumulators of the tile's rows that are not kept).  The path takes int8 A [m,k]
 * and B [k,n] (or, with transB, [n,k]: a weight matrix stored output-major), peers [keptRows, n] as fp32 added after
 * the dequantisation or, with CATCOC_FLAG_REDUCE_INT32, int32 added before it.  k in whole 64-byte steps and n in whole
 * 128-column tiles run the streaming kernels; any other k or n runs whole tiles on a one-thread-per-element kernel
 * (correct, slow, no k split).  At most 32 rows against B as [n,k] (k in whole 128-byte chunks, desc->splitK 0 or 1, no
 * `checksum`) need no k split at all: one workgroup per 32 columns walks the whole k range, and such a launch neither needs
 * nor touches the workspace, whatever this query (which does not know the layout) reports.  CATCOC_OUTBOUND_STORE does not apply (explicit kept rows have no rank structure to lay
 * tiles out by).  It stands in for SplitkMatmul (3rdparty/catlass/include/catlass/gemm/kernel/splitk_matmul.hpp:68-330)
 * in front of the dequant / reduce epilogue. */
CATCOC_API uint64_t catcoc_get_splitk_workspace_size(const CocTilingParams *tiling, const CatcocSymmetricDesc *desc,
                                                     uint32_t *splitK, uint32_t *tiles);

/* Number of tasks (tiles) a launch runs; `checksum` needs this many entries. */
CATCOC_API uint32_t catcoc_get_task_count(int commType, const CocTilingParams *tiling,
                                          const CatcocSymmetricDesc *desc);

/* ----------------------------------------------------------------------- */
/* dynamic_tiling host logic                                                 */
/* ----------------------------------------------------------------------- */

/* GetTilings (examples/dynamic_tiling/include/tiling.h:83-105): fills `out` (capacity maxOut) with the
 * candidates of the 5x5x2 search space that pass the op's check; returns how many exist. */
CATCOC_API int catcoc_get_tilings(const CocTilingParams *base, int commType, int rankSize, int blockNum,
                                  CocTilingParams *out, int maxOut);
/* CheckCommIntervalReduceScatter / AllReduce / AllGather (tiling.h:32-62); 1 = valid. */
CATCOC_API int catcoc_check_comm_interval_reduce_scatter(const CocTilingParams *t, int rankSize, int blockNum);
CATCOC_API int catcoc_check_comm_interval_allreduce(const CocTilingParams *t, int rankSize, int blockNum);
CATCOC_API int catcoc_check_comm_interval_allgather(const CocTilingParams *t, int rankSize);
/* SplitkMatmul::GetSplitkFactor (3rdparty/catlass/include/catlass/gemm/kernel/splitk_matmul.hpp:219-265). */
CATCOC_API uint32_t catcoc_get_splitk_factor(uint32_t m, uint32_t n, uint32_t k, uint32_t coreNum, uint32_t m0,
                                             uint32_t n0, uint32_t k0);
/* The defaults dynamic_tiling.cpp:215-227 fills in before the search (m0,k0,n0 = 128,256,256; commTileM 64;
 * commInterval 20; npuSplit 1; dataSplit 2; commBlockM 64). */
CATCOC_API void catcoc_default_tiling(CocTilingParams *t, uint32_t m, uint32_t k, uint32_t n, uint32_t rankSize);

/* ----------------------------------------------------------------------- */
/* Block schedulers (the same integer code the kernels run, callable on the host) */
/* ----------------------------------------------------------------------- */

/* GemmIdentityBlockSwizzle<off,dir>::GetBlockCoord on a loopsM x loopsN tile grid
 * (3rdparty/catlass/include/catlass/gemm/block/block_swizzle.hpp:79-113). */
CATCOC_API void catcoc_swizzle_block_coord(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN,
                                           uint32_t task, uint32_t *mIdx, uint32_t *nIdx);
/* SplitkGemmIdentityBlockSwizzle::GetBlockCoord / slice k extent (block_swizzle.hpp:151-235). */
CATCOC_API void catcoc_splitk_block_coord(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN,
                                          uint32_t kTiles, uint32_t f, uint32_t task, uint32_t *mIdx,
                                          uint32_t *nIdx, uint32_t *kIdx, uint32_t *slice);
CATCOC_API uint32_t catcoc_splitk_actual_k(uint32_t K, uint32_t k0, uint32_t f, uint32_t slice);
/* Which task of SplitkGemmIdentityBlockSwizzle workgroup `wg` of a split-K launch runs: a permutation that puts
 * the row tiles sharing a slice of B on one XCD.  No counterpart in the reference (its cores share one L2). */
CATCOC_API uint32_t catcoc_splitk_launch_task(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN,
                                              uint32_t f, uint32_t wg);
/* GemmIdentityBlockSwizzleAllGather::GetBlockCoord (include/catcoc/dgemm/block/block_swizzle_allgather.hpp:88-108). */
CATCOC_API void catcoc_allgather_block_coord(uint32_t off, uint32_t dir, uint32_t P, uint32_t commInterval,
                                             uint32_t loopsMRank, uint32_t loopsN, uint32_t task, uint32_t *mIdx,
                                             uint32_t *nIdx);
/* BlockCommSwizzle<dir>::GetBlockIdx (include/catcoc/comm_epilogue/block/comm_block_swizzle.hpp:147-186). */
CATCOC_API void catcoc_comm_block_idx(uint32_t dir, uint32_t P, uint32_t splitRow, uint32_t splitCol,
                                      uint32_t dataLoopsInRank, uint32_t task, uint32_t *dataIdx,
                                      uint32_t *rankIdx);
/* BlockCommSwizzle<dir, deterministic>::GetBlockIdx / GetCoreLoop (comm_block_swizzle.hpp:25-31,54-56,106-118,147-186).
 * With deterministic != 0 (direction 0 only) the npu split folds into the data split and the last band is padded:
 * data indices >= dataLoopsInRank are padding tasks. */
CATCOC_API void catcoc_comm_block_idx_ex(uint32_t dir, uint32_t deterministic, uint32_t P, uint32_t splitRow,
                                         uint32_t splitCol, uint32_t dataLoopsInRank, uint32_t task, uint32_t *dataIdx,
                                         uint32_t *rankIdx);
CATCOC_API uint32_t catcoc_comm_core_loop(uint32_t deterministic, uint32_t P, uint32_t splitRow, uint32_t splitCol,
                                          uint32_t dataLoopsInRank);
/* The tile a task computes in each operator (quant_matmul_reduce_scatter.hpp:172-201,
 * matmul_allreduce.hpp:154-179, allgather_matmul.hpp:142-163): target rank, first row/col of the tile in
 * the global problem, and the workspace row of the reference's tile-linear layout.  Returns 0 past the end. */
CATCOC_API int catcoc_task_tile(int commType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc,
                                uint32_t task, uint32_t *targetRank, uint32_t *row, uint32_t *col,
                                uint32_t *wsRow);
/* The same for tasks [firstTask, firstTask + count) in one call (the launch is planned once): fills the arrays that are not
 * NULL and returns how many tasks of the range exist. */
CATCOC_API uint32_t catcoc_task_tiles(int commType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc,
                                      uint32_t firstTask, uint32_t count, uint32_t *targetRank, uint32_t *row, uint32_t *col,
                                      uint32_t *wsRow);
/* The task workgroup `wg` of a launch runs: an XCD-aware order with the kept rank's tiles first (they are the
 * long ones).  A bijection on [0, task count);
 * 0xffffffff for wg out of range or rejected arguments.  (A reduce-scatter launch that splits its kept tiles, see
 * CATCOC_FLAG_KEPT_SPLIT, runs each as two 64-row workgroups placed first in the same order; this function still
 * describes the order by tile.)  No counterpart in the reference, where AI core i
 * simply runs tasks i, i + BLOCK_NUM, ... (quant_matmul_reduce_scatter.hpp:166-170). */
CATCOC_API uint32_t catcoc_launch_task(int commType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc,
                                       uint32_t wg);
/* How many kept tiles a launch of this shape would run as two 64-row workgroups each (see CATCOC_FLAG_KEPT_SPLIT;
 * 0 = none: the launch then has one workgroup per task, else that many workgroups more).  For tools that size or
 * reason about the grid.  No counterpart in the reference. */
CATCOC_API uint32_t catcoc_kept_split_tiles(int commType, int dataType, const CocTilingParams *tiling,
                                            const CatcocSymmetricDesc *desc, uint32_t transA, uint32_t transB);
/* How many tiles at the end of the launch order such a launch also runs as two 64-row workgroups each (see
 * CATCOC_FLAG_TAIL_WHOLE): the tiles by which tasks + kept halves exceed the 512 workgroup slots of the GPU; 0 when the
 * launch asks for checksums and desc carries no workspace.  The checksum buffer itself does not enter: pass the descriptor
 * the launch will use (desc.checksum non-NULL or not).  No counterpart in the reference. */
CATCOC_API uint32_t catcoc_tail_split_tiles(int commType, int dataType, const CocTilingParams *tiling,
                                            const CatcocSymmetricDesc *desc, uint32_t transA, uint32_t transB);
/* The same with the tile: what workgroup `wg` of the launch computes, exactly as the kernel works it out (the
 * large-tile kernels take a division-free route through constants prepared per launch; this entry point is how
 * tests compare that route with catcoc_launch_task + catcoc_task_tile).  Returns 0 past the end of the launch. */
CATCOC_API int catcoc_launch_tile(int commType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc, uint32_t wg,
                                  uint32_t *task, uint32_t *targetRank, uint32_t *row, uint32_t *col, uint32_t *wsRow);
/* The task workgroup `wg` of a launch with `tasks` tasks runs (XCD-aware chunking unless
 * CATCOC_FLAG_LINEAR_ORDER); a bijection on [0,tasks). */
CATCOC_API uint32_t catcoc_workgroup_task(uint32_t wg, uint32_t tasks, uint32_t flags);

/* Library / device information: fills cuCount, clockMHz of the current device; returns 0 on success. */
CATCOC_API int catcoc_device_info(int *cuCount, int *clockMHz, char *name, int nameLen);
CATCOC_API const char *catcoc_version(void);

#ifdef __cplusplus
}
#endif

#endif /* CATCOC_HIP_H */
