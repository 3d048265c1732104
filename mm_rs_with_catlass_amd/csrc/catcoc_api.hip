// C ABI of libcatcoc_hip.so: argument validation, tiling selection and dispatch
// to the fused GEMM kernels.  Declarations and the reference interfaces they
// replace are in include/catcoc_hip.h.
#include <hip/hip_runtime.h>
#include <pthread.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <math.h>

#include <new>
#include <vector>

#include "catcoc_hip.h"
#include "comm_reduce.h"
#include "gemm_args.h"
#include "tile_sched.h"

namespace catcoc {
int launch_gemm_i8(const GemmArgs &args, int variant, bool edge, void *stream);
int launch_gemm_dma_i8(const GemmArgs &args, void *stream);
int launch_gemm_splitk_i8(const GemmArgs &args, int rowBlocks, uint32_t tasks, void *stream);
int launch_gemm_decode_nk_i8(const GemmArgs &args, void *stream);
int launch_gemm_f16(const GemmArgs &args, int variant, bool edge, void *stream);
int launch_gemm_bf16(const GemmArgs &args, int variant, bool edge, void *stream);
int launch_gemm_dma_f16(const GemmArgs &args, void *stream);
int launch_gemm_dma_bf16(const GemmArgs &args, void *stream);

static int launch_gemm(uint32_t dtype, const GemmArgs &args, int variant, bool edge, void *stream)
{
    switch (dtype) {
        case DT_I8: return launch_gemm_i8(args, variant, edge, stream);
        case DT_F16: return launch_gemm_f16(args, variant, edge, stream);
        case DT_BF16: return launch_gemm_bf16(args, variant, edge, stream);
        default: return (int)hipErrorInvalidValue;
    }
}
}

using namespace catcoc;

namespace {

thread_local char g_err[512] = "";
thread_local int g_status = 0;

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    g_status = code;
    return code;
}

void ok()
{
    g_err[0] = 0;
    g_status = 0;
}

enum { E_NULL = 1, E_DESC = 2, E_SHAPE = 3, E_RANK = 4, E_TILING = 5, E_DTYPE = 6, E_WORKSPACE = 7, E_LAUNCH = 8 };

constexpr uint32_t kDefaultBlockNum = 256;  // one scheduling slot per CU of an MI355X
constexpr uint32_t kDefaultStages = 2;      // WORKSPACE_STAGES, examples/dynamic_tiling/include/info.h:18
// Every workspace starts with one block of per-tile arrival counters at a fixed place and of a fixed size, whatever the
// shape or slice count of the launch: launches of different shapes can then share one workspace that was zeroed once
// (each launch leaves its counters at zero again; the partial tiles behind the block are written before they are read).
constexpr uint64_t kCounterBlockBytes = CATCOC_WORKSPACE_COUNTER_BYTES;
constexpr uint32_t kMaxCountedTiles = (uint32_t)(kCounterBlockBytes / 4u);

struct Plan {
    GemmArgs args;
    int variant;  // 0 = general kernel, else tile rows / 64 of the fast kernel
    bool edge;
    uint32_t dtype;
    uint32_t blockNum;
    bool dma;     // full tiles, row-major operands: the direct-to-LDS kernel applies
    uint32_t kSlices;        // k slices per tile this launch would run with a workspace (1 = none)
    uint64_t kSliceBytes;    // workspace for that: partial tiles + counters
};

uint32_t elem_size(uint32_t dt) { return dt == DT_I8 ? 1u : 2u; }

// Everything a launcher checks before it launches; fills `plan` except the buffer pointers.
int make_plan(int commType, int dataType, const CocTilingParams *t, const CatcocSymmetricDesc *d, uint32_t transA,
              uint32_t transB, Plan &plan)
{
    if (t == nullptr) return fail(E_NULL, "tiling is NULL");
    if (d == nullptr) return fail(E_NULL, "symmetricPtr is NULL (it must point at a CatcocSymmetricDesc)");
    if (d->magic != CATCOC_DESC_MAGIC) return fail(E_DESC, "symmetricPtr does not point at a CatcocSymmetricDesc (bad magic)");
    if (commType < 0 || commType >= TYPE_NUM) return fail(E_DTYPE, "unknown commType %d", commType);
    const bool quant = commType == QUANT_MATMUL_REDUCE_SCATTER;
    if (quant ? dataType != INT8 : (dataType != FP16 && dataType != BF16))
        return fail(E_DTYPE, "dataType %d is not registered for commType %d", dataType, commType);
    if (t->m == 0 || t->n == 0 || t->k == 0) return fail(E_SHAPE, "empty problem m=%u n=%u k=%u", t->m, t->n, t->k);
    const uint32_t P = d->rankSize;
    if (P == 0 || P > CATCOC_MAX_RANKS) return fail(E_RANK, "rankSize %u out of range 1..%d", P, CATCOC_MAX_RANKS);
    if (t->rankSize != 0 && t->rankSize != P) return fail(E_RANK, "tiling.rankSize %u != descriptor rankSize %u", t->rankSize, P);
    if (d->rankIdx >= P) return fail(E_RANK, "rankIdx %u >= rankSize %u", d->rankIdx, P);

    const uint32_t op = (commType == MATMUL_ALLREDUCE) ? OP_ALLREDUCE : (commType == ALLGATHER_MATMUL) ? OP_ALLGATHER : OP_REDUCE_SCATTER;
    if (op == OP_REDUCE_SCATTER && t->m % P != 0)
        return fail(E_SHAPE, "reduce-scatter needs m %% rankSize == 0 (m=%u, rankSize=%u)", t->m, P);

    const uint32_t blockNum = d->blockNum ? d->blockNum : kDefaultBlockNum;
    const uint32_t stages = d->workspaceStages ? d->workspaceStages : kDefaultStages;
    const uint32_t commInterval = t->commInterval ? t->commInterval : 1u;
    // examples/dynamic_tiling/include/tiling.h:32-41: a round's tiles are dealt evenly to the ranks
    if (op == OP_REDUCE_SCATTER && ((uint64_t)blockNum * commInterval) % P != 0)
        return fail(E_TILING, "blockNum*commInterval = %u*%u is not a multiple of rankSize %u", blockNum, commInterval, P);
    const uint32_t off = d->swizzleOffset ? d->swizzleOffset : 7u;
    const uint32_t dir = d->swizzleOffset ? d->swizzleDirection : 1u;
    if (dir > 1) return fail(E_TILING, "swizzleDirection %u must be 0 or 1", dir);

    const uint32_t dt = (uint32_t)dataType;
    const uint32_t es = elem_size(dt);
    const uint32_t che = 16 / es;
    const uint32_t mRank = op == OP_REDUCE_SCATTER ? t->m / P : t->m;

    // tile selection: the fast kernels have n0 = 256 and m0 in {64,128}, or 256 for W8A8 on full tiles
    uint32_t m0 = t->m0, n0 = t->n0;
    if (n0 == 0) n0 = 256;
    // 256-row tiles: k in whole pairs of 64-byte steps; full tiles, or ragged rows / columns with a whole tile to move an edge
    // tile into and the moved tile's first column on the 16-byte grid of B, D and the peers (as for 128-row tiles below)
    const bool full256 = mRank % 256 == 0 && t->n % 256 == 0;
    const bool can256 = n0 == 256 && !transA && ((uint64_t)t->k * es) % 128 == 0 &&
                        (full256 || (mRank >= 256 && t->n >= 256 && t->n % 8 == 0 && (transB || ((uint64_t)t->n * es) % 16 == 0)));
    if (m0 == 0) {
        // The library's choice: 128-row tiles (two workgroups per CU) unless the launch has at least two 256x256 tiles per CU
        // and a row of k holds 4 KiB or more (or four per CU and 2 KiB): there 256 rows measured 3-10 % faster with B as
        // [k,n] and 15-25 % with B as [n,k] (8192-row launches, both element types, launches alternating); with two tiles
        // per CU and 1792 bytes of k (the benchmark shards) 128 rows stay ahead, 68.8 against 75.7 us.  The
        // rule does not look at the layout of B (with [n,k] the larger tile already pays from 2 KiB of k on): the queries for
        // task counts and workspace sizes do not know the layout and must see the same tiles.  All-gather keeps 128 rows
        // unless the caller asks.
        const uint64_t kBytes = (uint64_t)t->k * es;
        const uint64_t tiles256 = (uint64_t)(t->m / 256u) * (t->n / 256u);
        const bool pays = (tiles256 >= 512 && kBytes >= 4096) || (tiles256 >= 1024 && kBytes >= 2048);
        // (full tiles only: ragged problems take 256 rows on request, since the pipelined operators run those on other kernels)
        m0 = (mRank <= 64) ? 64 : (can256 && full256 && pays && op != OP_ALLGATHER) ? 256 : 128;
    }
    const bool dmaShape = can256 && m0 == 256;
    // (A as [k,m] exists in the 128-row direct-to-LDS kernel only: rows of m in whole 16-byte pieces, a rank's block on that grid)
    const bool taOk = !transA || (m0 == 128 && ((uint64_t)t->m * es) % 16 == 0 && ((uint64_t)mRank * es) % 16 == 0);
    const bool fastShape = dmaShape || n0 == 256 && (m0 == 64 || m0 == 128) && taOk && t->k % che == 0 && t->n % 4 == 0;
    plan.variant = fastShape ? (int)(m0 / 64) : 0;   // 4 (m0 = 256) exists only as the direct-to-LDS kernel
    plan.edge = !(mRank % m0 == 0 && t->n % n0 == 0 && t->k % (64 / es) == 0);
    plan.dtype = dt;
    plan.blockNum = blockNum;
    // (B as [n,k] runs the 128-row direct-to-LDS kernel when its rows of k are 16-byte multiples)
    // Ragged rows / columns on 128-row tiles: the direct-to-LDS kernel moves the edge tiles inwards (GF_RAGGED).  It needs a whole
    // tile to move into, k in whole 64-byte steps, and the moved tile's first column on the 16-byte grid of B, D and the peers.
    const bool ragged = plan.edge && ((m0 == 128 && mRank >= m0 && t->n >= n0 && ((uint64_t)t->k * es) % 64 == 0 && t->n % 8 == 0 &&
                                       (transB || ((uint64_t)t->n * es) % 16 == 0)) ||
                                      (m0 == 256 && can256));
    plan.dma = fastShape && (!plan.edge || ragged) && (m0 == 256 || (m0 == 128 && (!transB || ((uint64_t)t->k * es) % 16 == 0))) &&
               (m0 == 128 || !transA);
    if (transA && !plan.dma) plan.variant = 0;   // the other fast kernels take A as [m,k] only

    GemmArgs &a = plan.args;
    memset(&a, 0, sizeof(a));
    a.M = t->m;
    a.N = t->n;
    a.K = t->k;
    a.lda = transA ? t->m : t->k;
    a.ldb = transB ? t->k : t->n;
    a.ldd = t->n;
    a.transA = transA ? 1 : 0;
    a.transB = transB ? 1 : 0;
    a.outDtype = dt == DT_I8 ? DT_BF16 : dt;
    a.sched = make_sched(op, t->m, t->n, P, m0, n0, blockNum, commInterval, stages, off, dir);
    if (a.sched.coreLoops == 0) return fail(E_SHAPE, "no tiles to compute");

    if ((d->flags & CATCOC_OUTBOUND_MASK) == CATCOC_OUTBOUND_STORE) a.flags |= GF_OUTBOUND_STORE;
    if (d->flags & CATCOC_FLAG_REDUCE_INT32) {
        if (!quant) return fail(E_DESC, "CATCOC_FLAG_REDUCE_INT32 only applies to the W8A8 operator");
        a.flags |= GF_REDUCE_INT32;
    }
    if (d->flags & CATCOC_FLAG_LINEAR_ORDER) a.flags |= GF_LINEAR_ORDER;
    if (d->flags & CATCOC_FLAG_KEPT_WHOLE) a.flags |= GF_KEPT_WHOLE;
    if (d->flags & CATCOC_FLAG_KEPT_SPLIT) a.flags |= GF_KEPT_SPLIT;
    if (plan.dma && plan.edge) a.flags |= GF_RAGGED;

    // kept rows
    if (op == OP_REDUCE_SCATTER) {
        a.keptBegin = d->rankIdx * mRank;
        a.keptRows = mRank;
        a.keptRank = d->rankIdx;
    } else if (op == OP_ALLREDUCE) {
        a.keptBegin = 0;
        a.keptRows = t->m;
    } else {
        a.keptBegin = 0;
        a.keptRows = t->m * P;
    }

    // peers
    const uint32_t nPeers = P - 1;
    if (op == OP_ALLGATHER) {
        a.nPeers = 0;
        uint32_t s = 0;
        for (uint32_t r = 0; r < P; ++r) {
            if (r == d->rankIdx) continue;
            if (d->peers[s] == nullptr) return fail(E_NULL, "all-gather needs %u peer shards; peers[%u] is NULL", nPeers, s);
            a.a[r] = d->peers[s++];
        }
    } else {
        a.nPeers = nPeers;
        for (uint32_t s = 0; s < nPeers; ++s) {
            if (d->peers[s] == nullptr) return fail(E_NULL, "reduce needs %u staged peer partials; peers[%u] is NULL", nPeers, s);
            a.peers[s] = d->peers[s];
        }
        a.peerLd = d->peerLd ? d->peerLd : t->n;
        a.peerRowOffset = d->peerRowOffset;
        if (nPeers && a.peerLd < (int64_t)t->n) return fail(E_DESC, "peerLd %lld < n %u", (long long)a.peerLd, t->n);
        if (a.peerRowOffset < 0) return fail(E_DESC, "peerRowOffset must be >= 0");
        if (fastShape && nPeers && (a.peerLd % 4 != 0)) plan.variant = 0;  // 16-byte peer loads need aligned rows
    }

    if (a.flags & GF_OUTBOUND_STORE) {
        if (op == OP_REDUCE_SCATTER && P > 1) {
            if (d->outbound == nullptr) return fail(E_NULL, "CATCOC_OUTBOUND_STORE needs an outbound buffer");
            const uint64_t need = (uint64_t)stages * a.sched.blockPerComm * m0 * n0 * 4u;
            if (d->outboundBytes < need)
                return fail(E_WORKSPACE, "outbound buffer too small: %llu < %llu bytes", (unsigned long long)d->outboundBytes,
                            (unsigned long long)need);
        }
        a.outbound = d->outbound;
    } else {
        a.checksum = d->checksum;
    }
    a.accDump = d->accDump;

    // Few tiles: the 128-row direct-to-LDS kernel can cut every tile's k range into slices, one workgroup each, that
    // meet through a workspace (partial tiles [tiles][slices][128*256] as 32-bit words, then one counter per tile).
    // Chosen so that the slices fill the 256 CUs once, each with at least eight k steps; float launches take
    // two slices by themselves (see fauto below).  desc.splitK overrides the choice.
    plan.kSlices = 1;
    plan.kSliceBytes = 0;
    if (plan.dma && !plan.edge && m0 == 128 && d->keptRows == 0) {
        const uint32_t T = a.sched.coreLoops, nkAll = (uint32_t)((uint64_t)t->k * es / 64u);
        const uint32_t fmax = 8u;
        // the library's own choice stays at two slices for float operands (more are reproducible too -- three or more float
        // partials are added in slice order -- but did not measure faster: the last slice then fetches every partial)
        const uint32_t fauto = dt == DT_I8 ? 8u : 2u;
        uint32_t f = 1;
        if (d->splitK != 0) {
            if (d->splitK > fmax || d->splitK > nkAll)
                return fail(E_TILING, "splitK %u: at most %u k slices for this k", d->splitK, umin(fmax, nkAll));
            f = d->splitK;
        } else {
            while (f * 2u <= fauto && T * f * 2u <= 256u && nkAll / (f * 2u) >= 8u) f *= 2u;
        }
        if (f > 1) {
            plan.kSlices = f;
            if (T > kMaxCountedTiles) return fail(E_TILING, "k slices: %u tiles exceed the %u the workspace counts", T, kMaxCountedTiles);
            plan.kSliceBytes = kCounterBlockBytes + (uint64_t)T * f * (128u * 256u * 4u);
            if (d->workspace != nullptr) {
                if ((uintptr_t)d->workspace % 256 != 0) return fail(E_WORKSPACE, "workspace must be 256-byte aligned");
                if (d->workspaceBytes < plan.kSliceBytes)
                    return fail(E_WORKSPACE, "workspace too small for %u k slices: %llu < %llu bytes", f,
                                (unsigned long long)d->workspaceBytes, (unsigned long long)plan.kSliceBytes);
                a.splitK = f;
                a.skCount = (uint32_t *)d->workspace;
                a.skPart = (int32_t *)((unsigned char *)d->workspace + kCounterBlockBytes);
            } else if (d->splitK != 0) {
                return fail(E_WORKSPACE, "splitK %u needs a workspace of %llu bytes", f, (unsigned long long)plan.kSliceBytes);
            }
        }
    }
    // a workspace also lets the checksum halves of tiles that run as two workgroups meet (its counter block)
    if (a.skCount == nullptr && d->workspace != nullptr && (uintptr_t)d->workspace % 256 == 0 && d->workspaceBytes >= kCounterBlockBytes)
        a.skCount = (uint32_t *)d->workspace;
    if (d->flags & CATCOC_FLAG_TAIL_WHOLE) a.flags |= GF_TAIL_WHOLE;
    return 0;
}

int check_ptr_align(const Plan &p, const void *a, const void *b)
{
    if (p.variant == 0) return 1;
    const uint32_t es = elem_size(p.dtype);
    bool okA = ((uintptr_t)a % 16 == 0) && ((p.args.lda * es) % 16 == 0);
    bool okB = p.args.transB ? (((uintptr_t)b % 16 == 0) && ((p.args.ldb * es) % 16 == 0))
                             : (((uintptr_t)b % (4 * es) == 0) && (p.args.ldb % 4 == 0));
    for (uint32_t r = 0; r < p.args.sched.P && okA; ++r)
        if (p.args.a[r] && (uintptr_t)p.args.a[r] % 16 != 0) okA = false;
    return okA && okB;
}

void launch_float(int commType, int dataType, void *stream, uint8_t *a, uint8_t *b, uint8_t *c, uint8_t *symmetricPtr,
                  CocTilingParams *tiling, uint32_t transA, uint32_t transB)
{
    Plan p;
    const CatcocSymmetricDesc *d = (const CatcocSymmetricDesc *)symmetricPtr;
    if (make_plan(commType, dataType, tiling, d, transA, transB, p)) return;
    if (!a || !b || !c) { fail(E_NULL, "a, b and c must be non-NULL"); return; }
    if (commType == ALLGATHER_MATMUL) p.args.a[d->rankIdx] = a;
    else p.args.a[0] = a;
    p.args.b = b;
    p.args.d = c;
    if (!check_ptr_align(p, a, b)) p.variant = 0;
    const bool dma = p.dma && p.variant != 0 && (uintptr_t)b % 16 == 0 && (p.args.ldb * 2) % 16 == 0 && (uintptr_t)c % 16 == 0;
    if (!dma) p.args.splitK = 0;   // the other kernels run every tile whole
    if (!dma && p.variant == 4) { fail(E_TILING, "m0 = 256 needs full tiles and 16-byte aligned row-major operands"); return; }
    if (!dma && p.args.transA) p.variant = 0;
    const int e = dma ? (p.dtype == DT_F16 ? launch_gemm_dma_f16(p.args, stream) : launch_gemm_dma_bf16(p.args, stream))
                      : launch_gemm(p.dtype, p.args, p.variant, p.edge, stream);
    if (e) { fail(E_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)e)); return; }
    ok();
}

// ---- skinny-M split-K path (explicit kept rows) ----------------------------------------------
struct SplitkPlan {
    GemmArgs args;
    uint32_t f, tiles, rowBlocks;
    uint64_t workspaceBytes;   // partial tiles + counters (0 when f == 1)
    bool general;              // shape outside the fast routes: gemm_general_kernel on the 128x128 grid
    bool wholeK;               // at most 32 rows against B as [n,k]: gemm_decode_nk_kernel, no k slices, no workspace
    bool large;                // many rows: the 128x256 direct-to-LDS kernel in row-mask mode runs instead of the split-K kernel
};

// Explicit kept rows with at least this many rows of A run the 128x256 direct-to-LDS kernel (k-sliced through the same
// workspace) when the shape has full tiles and the kept rows are whole 32-row blocks.  Such launches have at most one
// workgroup per CU and run the kernel's six-stage ring with the pipelined peer loads.  Measured at K = N = 8192 with kept
// rows = M / 8, the two routes alternating launch by launch and B coming from HBM (six copies, another one every launch):
// M = 1024 106 against 166 us, M = 512 69 (two k slices) against 77 us, M = 256 50 (four k slices) against 48 us (since then
// both routes fetch A as whole cache lines per pair of k steps and hand only kept blocks between k slices: M = 512 59 against 74 us,
// M = 384 56 against 103 (three rows of 128x128 tiles in four slices are three waves of workgroups), M = 256 42 against 50, and with
// 32 kept rows M = 128 45 (eight k slices) against 36, so the large tile starts at 256 rows).  n0 = 256
// (with m0 0 or 128) in the tiling asks for the large tile explicitly, n0 = 128 for the split-K kernel.
constexpr uint32_t kLargeTileRows = 256;

int make_splitk_plan(const CocTilingParams *t, const CatcocSymmetricDesc *d, uint32_t transA, uint32_t transB, SplitkPlan &sp)
{
    if (t == nullptr) return fail(E_NULL, "tiling is NULL");
    if (d == nullptr || d->magic != CATCOC_DESC_MAGIC) return fail(E_DESC, "symmetricPtr does not point at a CatcocSymmetricDesc");
    if (t->m == 0 || t->n == 0 || t->k == 0) return fail(E_SHAPE, "empty problem m=%u n=%u k=%u", t->m, t->n, t->k);
    const uint32_t P = d->rankSize;
    if (P == 0 || P > CATCOC_MAX_RANKS) return fail(E_RANK, "rankSize %u out of range 1..%d", P, CATCOC_MAX_RANKS);
    if (transA) return fail(E_SHAPE, "the explicit-kept-rows (split-K) path takes A as [m,k] (B as [k,n] or, with transB, as [n,k])");
    // shapes the two fast routes cannot take (k not in whole 64-byte steps, n not in whole 128-column tiles) run the
    // one-thread-per-element kernel on the same 128x128 grid: a correctness path, whole tiles, no workspace
    sp.general = t->k % 64 != 0 || t->n % 128 != 0;
    sp.wholeK = false;
    const bool canLarge = !sp.general && t->m % 128 == 0 && t->n % 256 == 0 && d->keptRowBegin % 32 == 0 && d->keptRows % 32 == 0;
    const bool wantLarge = t->n0 == 256 && (t->m0 == 0 || t->m0 == 128);
    if (wantLarge && !canLarge)
        return fail(E_TILING, "128x256 tiles with explicit kept rows need m %% 128 == 0, n %% 256 == 0 and kept rows in whole 32-row blocks "
                              "(m=%u, n=%u, kept [%u,+%u))", t->m, t->n, d->keptRowBegin, d->keptRows);
    sp.large = wantLarge || (t->n0 == 0 && t->m0 == 0 && canLarge && t->m >= kLargeTileRows);
    if (!sp.large && ((t->m0 != 0 && t->m0 != 128) || (t->n0 != 0 && t->n0 != 128)))
        return fail(E_TILING, "explicit kept rows run 128x128 tiles (split-K kernel) or 128x256 tiles; leave m0/n0 zero or pass one of those "
                              "(m0=%u, n0=%u)", t->m0, t->n0);
    if (d->keptRows == 0 || (uint64_t)d->keptRowBegin + d->keptRows > t->m)
        return fail(E_DESC, "kept rows [%u,+%u) outside [0,%u)", d->keptRowBegin, d->keptRows, t->m);
    if ((d->flags & CATCOC_OUTBOUND_MASK) == CATCOC_OUTBOUND_STORE)
        return fail(E_DESC, "the split-K path folds non-kept rows into checksums; CATCOC_OUTBOUND_STORE is not supported there");
    const uint32_t off = d->swizzleOffset ? d->swizzleOffset : 7u;
    const uint32_t dir = d->swizzleOffset ? d->swizzleDirection : 1u;
    if (dir > 1) return fail(E_TILING, "swizzleDirection %u must be 0 or 1", dir);

    GemmArgs &a = sp.args;
    memset(&a, 0, sizeof(a));
    a.M = t->m; a.N = t->n; a.K = t->k;
    a.lda = t->k; a.ldb = transB ? t->k : t->n; a.ldd = t->n;
    a.transB = transB ? 1 : 0;
    if (d->flags & CATCOC_FLAG_REDUCE_INT32) a.flags |= GF_REDUCE_INT32;   // int32 peers join the accumulators before the dequant
    a.outDtype = DT_BF16;
    a.sched.off = off; a.sched.dir = dir;
    a.keptBegin = d->keptRowBegin;
    a.keptRows = d->keptRows;
    a.nPeers = P - 1;
    for (uint32_t s = 0; s < a.nPeers; ++s) {
        if (d->peers[s] == nullptr) return fail(E_NULL, "reduce needs %u staged peer partials; peers[%u] is NULL", a.nPeers, s);
        a.peers[s] = d->peers[s];
    }
    a.peerLd = d->peerLd ? d->peerLd : t->n;
    a.peerRowOffset = d->peerRowOffset;
    if (a.nPeers && a.peerLd < (int64_t)t->n) return fail(E_DESC, "peerLd %lld < n %u", (long long)a.peerLd, t->n);
    if (a.peerRowOffset < 0) return fail(E_DESC, "peerRowOffset must be >= 0");
    if ((uint64_t)(a.peerRowOffset + a.keptRows) * (uint64_t)a.peerLd * 4u > 0x7fffffffull)
        return fail(E_DESC, "the split-K path addresses each peer partial with 31-bit byte offsets: (peerRowOffset + keptRows) * peerLd * 4 must stay below 2 GiB");
    a.checksum = d->checksum;
    a.accDump = d->accDump;

    const uint32_t cores = d->blockNum ? d->blockNum : kDefaultBlockNum;
    const uint32_t kTiles = ceil_div(t->k, 256u);
    sp.tiles = ceil_div(t->m, 128u) * ceil_div(t->n, 128u);
    if (sp.general) {
        if (d->splitK > 1) return fail(E_TILING, "k %% 64 != 0 or n %% 128 != 0: this shape runs whole tiles on the general kernel; splitK %u is not available", d->splitK);
        const uint32_t stages = d->workspaceStages ? d->workspaceStages : kDefaultStages;
        a.sched = make_sched(OP_ALLREDUCE, t->m, t->n, 1, 128, 128, cores, 1, stages, off, dir);
        a.flags |= GF_ROW_MASK;
        sp.f = 1;
        a.splitK = 0;
        sp.rowBlocks = 4;
        sp.workspaceBytes = 0;
        return 0;
    }
    if (sp.large) {
        // one grid of 128x256 tiles over all of A's rows (no rank structure), k slices as for any few-tile launch
        const uint32_t stages = d->workspaceStages ? d->workspaceStages : kDefaultStages;
        a.sched = make_sched(OP_ALLREDUCE, t->m, t->n, 1, 128, 256, cores, 1, stages, off, dir);
        a.flags |= GF_ROW_MASK;
        const uint32_t T = a.sched.coreLoops, nkAll = t->k / 64u;
        uint32_t f = 1;
        if (d->splitK != 0) {
            if (d->splitK > 8u || d->splitK > nkAll) return fail(E_TILING, "splitK %u: at most %u k slices here", d->splitK, umin(8u, nkAll));
            f = d->splitK;
        } else {
            while (f * 2u <= 8u && T * f * 2u <= 256u && nkAll / (f * 2u) >= 8u) f *= 2u;
        }
        if (f > 1 && T > kMaxCountedTiles) return fail(E_TILING, "k slices: %u tiles exceed the %u the workspace counts", T, kMaxCountedTiles);
        sp.f = f;
        a.splitK = f > 1 ? f : 0;
        sp.rowBlocks = 4;
        sp.workspaceBytes = f > 1 ? kCounterBlockBytes + (uint64_t)T * f * (128u * 256u * 4u) : 0;
        return 0;
    }
    // B as [n,k] against at most 32 rows: a workgroup can own 32 columns over the whole k range and still read whole cache
    // lines, so nothing is handed between workgroups (unless the caller asks for k slices or for per-tile checksums, which
    // are per 128 columns)
    sp.wholeK = transB && t->m <= 32 && t->k % 128 == 0 && d->splitK <= 1 && d->checksum == nullptr;
    if (sp.wholeK) {
        sp.f = 1;
        a.splitK = 0;
        sp.rowBlocks = 1;
        sp.workspaceBytes = 0;
        return 0;
    }
    uint32_t f = d->splitK ? d->splitK : splitk_factor(t->m, t->n, t->k, cores, 128, 128, 256);
    if (f > kTiles) f = kTiles;
    if (f == 0) f = 1;
    sp.f = f;
    a.splitK = f;
    sp.rowBlocks = t->m <= 32 ? 1 : t->m <= 64 ? 2 : 4;
    if (f > 1 && sp.tiles > kMaxCountedTiles)
        return fail(E_TILING, "split-K: %u tiles exceed the %u the workspace counts", sp.tiles, kMaxCountedTiles);
    sp.workspaceBytes = f > 1 ? kCounterBlockBytes + (uint64_t)f * sp.tiles * 128u * 128u * 4u : 0;
    return 0;
}

void launch_quant_splitk(void *stream, uint8_t *x1, uint8_t *x2, uint8_t *scale_x1, uint8_t *scale_x2, uint8_t *bias,
                         uint8_t *c_accum, uint8_t *d_out, const CatcocSymmetricDesc *d, CocTilingParams *tiling,
                         uint32_t transA, uint32_t transB, uint32_t outDataType)
{
    SplitkPlan sp;
    if (make_splitk_plan(tiling, d, transA, transB, sp)) return;
    if (!x1 || !x2 || !scale_x1 || !scale_x2 || !d_out) { fail(E_NULL, "x1, x2, scale_x1, scale_x2 and d_out must be non-NULL"); return; }
    if (outDataType != FP16 && outDataType != BF16) { fail(E_DTYPE, "outDataType %u must be FP16 (1) or BF16 (27)", outDataType); return; }
    GemmArgs &a = sp.args;
    if (sp.general) {
        a.a[0] = x1; a.b = x2; a.d = d_out;
        a.scaleM = (const float *)scale_x1; a.scaleN = (const float *)scale_x2;
        a.bias = (const int32_t *)bias; a.cAccum = (int32_t *)c_accum;
        a.outDtype = outDataType;
        const int eg = launch_gemm(DT_I8, a, 0, true, stream);
        if (eg) { fail(E_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)eg)); return; }
        ok();
        return;
    }
    if ((uintptr_t)x1 % 16 != 0 || (uintptr_t)x2 % 16 != 0 || sp.args.lda % 16 != 0 || sp.args.ldb % 16 != 0) {
        fail(E_SHAPE, "the split-K path needs 16-byte aligned x1, x2 and row pitches");
        return;
    }
    // The large-tile route picked its k slices by itself (no desc.splitK): they need a workspace to meet through, and without
    // one that fits the tiles run whole, as any other few-tile launch of that kernel does.  Only an explicit splitK insists.
    if (sp.large && sp.f > 1 && d->splitK == 0 &&
        (d->workspace == nullptr || (uintptr_t)d->workspace % 256 != 0 || d->workspaceBytes < sp.workspaceBytes)) {
        sp.f = 1;
        a.splitK = 0;
    }
    if (sp.f > 1) {
        if (d->workspace == nullptr || d->workspaceBytes < sp.workspaceBytes) {
            fail(E_WORKSPACE, "split factor %u needs a zero-initialised workspace of %llu bytes (catcoc_get_splitk_workspace_size)",
                 sp.f, (unsigned long long)sp.workspaceBytes);
            return;
        }
        if ((uintptr_t)d->workspace % 256 != 0) { fail(E_WORKSPACE, "workspace must be 256-byte aligned"); return; }
        a.skCount = (uint32_t *)d->workspace;
        a.skPart = (int32_t *)((unsigned char *)d->workspace + kCounterBlockBytes);
    }
    a.a[0] = x1;
    a.b = x2;
    a.d = d_out;
    a.scaleM = (const float *)scale_x1;
    a.scaleN = (const float *)scale_x2;
    a.bias = (const int32_t *)bias;
    a.cAccum = (int32_t *)c_accum;
    a.outDtype = outDataType;
    if (sp.large) {
        bool aligned = (uintptr_t)scale_x2 % 16 == 0 && (uintptr_t)d_out % 16 == 0 && (!bias || (uintptr_t)bias % 16 == 0) && a.peerLd % 4 == 0;
        for (uint32_t s = 0; s < a.nPeers && aligned; ++s) aligned = (uintptr_t)a.peers[s] % 16 == 0;
        if (!aligned) { fail(E_SHAPE, "128x256 tiles with explicit kept rows need 16-byte aligned scales, bias, peers and output"); return; }
        const int el = launch_gemm_dma_i8(a, stream);
        if (el) { fail(E_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)el)); return; }
        ok();
        return;
    }
    const int e = sp.wholeK ? launch_gemm_decode_nk_i8(a, stream) : launch_gemm_splitk_i8(a, (int)sp.rowBlocks, sp.tiles * sp.f, stream);
    if (e) { fail(E_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)e)); return; }
    ok();
}

void launch_quant(void *stream, uint8_t *x1, uint8_t *x2, uint8_t *scale_x1, uint8_t *scale_x2, uint8_t *bias,
                  uint8_t *c_accum, uint8_t *d_out, uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA,
                  uint32_t transB, uint32_t outDataType)
{
    Plan p;
    const CatcocSymmetricDesc *d = (const CatcocSymmetricDesc *)symmetricPtr;
    if (d != nullptr && d->magic == CATCOC_DESC_MAGIC && d->keptRows != 0) {
        launch_quant_splitk(stream, x1, x2, scale_x1, scale_x2, bias, c_accum, d_out, d, tiling, transA, transB, outDataType);
        return;
    }
    if (make_plan(QUANT_MATMUL_REDUCE_SCATTER, INT8, tiling, d, transA, transB, p)) return;
    if (!x1 || !x2 || !scale_x1 || !scale_x2 || !d_out) { fail(E_NULL, "x1, x2, scale_x1, scale_x2 and d_out must be non-NULL"); return; }
    if (outDataType != FP16 && outDataType != BF16) { fail(E_DTYPE, "outDataType %u must be FP16 (1) or BF16 (27)", outDataType); return; }
    p.args.a[0] = x1;
    p.args.b = x2;
    p.args.d = d_out;
    p.args.scaleM = (const float *)scale_x1;
    p.args.scaleN = (const float *)scale_x2;
    p.args.bias = (const int32_t *)bias;
    p.args.cAccum = (int32_t *)c_accum;
    p.args.outDtype = outDataType;
    if (!check_ptr_align(p, x1, x2) || (uintptr_t)scale_x2 % 16 != 0 || (bias && (uintptr_t)bias % 16 != 0) ||
        (c_accum && (uintptr_t)c_accum % 16 != 0) || (uintptr_t)d_out % 8 != 0)
        p.variant = 0;
    bool dma = p.dma && p.variant != 0 && (uintptr_t)x2 % 16 == 0 && p.args.ldb % 16 == 0 && (uintptr_t)d_out % 16 == 0;
    for (uint32_t s = 0; s < p.args.nPeers && dma; ++s) dma = (uintptr_t)p.args.peers[s] % 16 == 0;
    if (!dma && p.variant == 4) { fail(E_TILING, "m0 = 256 needs full tiles, 16-byte aligned row-major operands and fp32 peers"); return; }
    if (!dma) p.args.splitK = 0;   // the other kernels run every tile whole
    if (!dma && p.args.transA) p.variant = 0;
    const int e = dma ? launch_gemm_dma_i8(p.args, stream) : launch_gemm(p.dtype, p.args, p.variant, p.edge, stream);
    if (e) { fail(E_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)e)); return; }
    ok();
}

}  // namespace

// The events of a round-pipelined call: "store finished" and "compute finished" per round, and the join at the end.
struct CatcocPipelinedPlan {
    uint32_t magic = 0;
    std::vector<hipEvent_t> ready, done;
    hipEvent_t fin = nullptr;
};

namespace {

constexpr uint32_t kPlanMagic = 0x4350504cu;   // "CPPL"

void plan_destroy_events(CatcocPipelinedPlan &p)
{
    for (hipEvent_t e : p.ready) if (e) (void)hipEventDestroy(e);
    for (hipEvent_t e : p.done) if (e) (void)hipEventDestroy(e);
    if (p.fin) (void)hipEventDestroy(p.fin);
    p.ready.clear();
    p.done.clear();
    p.fin = nullptr;
    p.magic = 0;
}

bool plan_make_events(CatcocPipelinedPlan &p, uint32_t rounds)
{
    p.ready.assign(rounds, nullptr);
    p.done.assign(rounds, nullptr);
    hipError_t he = hipEventCreateWithFlags(&p.fin, hipEventDisableTiming);
    for (uint32_t r = 0; r < rounds && he == hipSuccess; ++r) {
        he = hipEventCreateWithFlags(&p.ready[r], hipEventDisableTiming);
        if (he == hipSuccess) he = hipEventCreateWithFlags(&p.done[r], hipEventDisableTiming);
    }
    if (he != hipSuccess) {
        plan_destroy_events(p);
        fail(E_LAUNCH, "hipEventCreate failed: %s", hipGetErrorString(he));
        return false;
    }
    p.magic = kPlanMagic;
    return true;
}

// ---- round-pipelined, reference-faithful form of the reduce-scatter operators ------------------
// The reference's structure kept as it is (quant_matmul_reduce_scatter.hpp:159-164,219,282,319; matmul_reduce_scatter.hpp
// the same): per comm round the GEMM stores the round's tiles (kept rank's into the local block, the others into stage
// `round % stages` of the workspace) and raises "store finished"; the comm side waits for it, adds the peers' blocks into
// the local block along BlockCommSwizzle's task list and raises "compute finished", which the GEMM of round + stages
// waits for before it reuses the stage.  The two sides are two HIP streams here and the flags are events.
void launch_pipelined(bool quant, int dataType, void *computeStream, void *commStream, uint8_t *a, uint8_t *b, uint8_t *scale_x1,
                      uint8_t *scale_x2, uint8_t *bias, uint8_t *c_accum, uint8_t *d_out, uint8_t *symmetricPtr,
                      CocTilingParams *tiling, uint32_t transA, uint32_t transB, uint32_t outDataType, uint32_t deterministic)
{
    const CatcocSymmetricDesc *given = (const CatcocSymmetricDesc *)symmetricPtr;
    if (given == nullptr || given->magic != CATCOC_DESC_MAGIC) { fail(E_DESC, "symmetricPtr does not point at a CatcocSymmetricDesc"); return; }
    if (given->keptRows != 0) { fail(E_DESC, "the round-pipelined form keeps the reference's row blocks (keptRows must be 0)"); return; }
    CatcocSymmetricDesc d = *given;
    d.flags = (d.flags & ~CATCOC_OUTBOUND_MASK) | CATCOC_OUTBOUND_STORE | CATCOC_FLAG_LINEAR_ORDER;
    if (quant) d.flags |= CATCOC_FLAG_REDUCE_INT32;
    d.workspace = nullptr;
    d.splitK = 0;
    Plan p;
    const int commType = quant ? QUANT_MATMUL_REDUCE_SCATTER : MATMUL_REDUCE_SCATTER;
    if (make_plan(commType, dataType, tiling, &d, transA, transB, p)) return;
    if (!a || !b || !d_out) { fail(E_NULL, "operands and output must be non-NULL"); return; }
    if (quant && (!scale_x1 || !scale_x2 || !c_accum)) { fail(E_NULL, "the pipelined W8A8 operator needs scale_x1, scale_x2 and c_accum"); return; }
    const uint32_t outDt = quant ? outDataType : (uint32_t)dataType;
    if (outDt != FP16 && outDt != BF16) { fail(E_DTYPE, "outDataType %u must be FP16 (1) or BF16 (27)", outDt); return; }
    if (d.outbound == nullptr && d.rankSize > 1) { fail(E_NULL, "the pipelined form stores the other ranks' tiles: outbound (the symmetric workspace) is needed"); return; }

    GemmArgs &g = p.args;
    const SchedParams &sp = g.sched;
    const uint32_t P = sp.P, m0 = sp.m0, n0 = sp.n0;
    const uint32_t cb = tiling->commBlockM ? tiling->commBlockM : umin(64u, m0);
    if (m0 % cb != 0) { fail(E_TILING, "commBlockM %u must divide m0 %u", cb, m0); return; }
    uint32_t splitRow = tiling->commDataSplit, splitCol = tiling->commNpuSplit ? tiling->commNpuSplit : 1u;
    if (splitRow == 0 || splitRow * splitCol < 16u) { splitRow = 256u; splitCol = 1u; }   // the reference's 2..20 cores would idle this GPU
    if (!deterministic && P % splitCol != 0) { fail(E_TILING, "commNpuSplit %u must divide rankSize %u", splitCol, P); return; }
    const uint32_t es = quant ? 4u : 2u;
    const uint32_t vec = 16u / es;
    if (tiling->n % vec != 0 || n0 % vec != 0) { fail(E_SHAPE, "the pipelined form moves 16-byte pieces: n and n0 must be multiples of %u", vec); return; }
    const int64_t peerLd = d.peerLd ? d.peerLd : tiling->n;
    void *local = quant ? (void *)c_accum : (void *)d_out;
    if ((uintptr_t)local % 16 != 0 || (peerLd * es) % 16 != 0) { fail(E_SHAPE, "the pipelined form needs 16-byte aligned blocks and peer rows"); return; }
    for (uint32_t s = 0; s + 1 < P; ++s)
        if ((uintptr_t)d.peers[s] % 16 != 0) { fail(E_SHAPE, "peers[%u] must be 16-byte aligned", s); return; }

    // GEMM side: every round is one launch of the ordinary kernels over the round's tasks, with no peers to add
    if (quant) {
        g.a[0] = a; g.b = b; g.d = d_out;
        g.scaleM = (const float *)scale_x1; g.scaleN = (const float *)scale_x2;
        g.bias = (const int32_t *)bias; g.cAccum = (int32_t *)c_accum;
        g.outDtype = outDt;
        if (!check_ptr_align(p, a, b) || (uintptr_t)scale_x2 % 16 != 0 || (bias && (uintptr_t)bias % 16 != 0) || (uintptr_t)d_out % 8 != 0) p.variant = 0;
    } else {
        g.a[0] = a; g.b = b; g.d = d_out;
        if (!check_ptr_align(p, a, b)) p.variant = 0;
    }
    g.nPeers = 0;
    const bool dma = p.dma && !p.edge && p.variant != 0 && (uintptr_t)b % 16 == 0 && (g.ldb * (quant ? 1 : 2)) % 16 == 0 && (uintptr_t)d_out % 16 == 0;
    g.flags &= ~(uint32_t)GF_RAGGED;   // (ragged problems run the bounds-checked kernel here)
    if (!dma && p.variant == 4) { fail(E_TILING, "m0 = 256 needs full tiles and 16-byte aligned row-major operands"); return; }
    if (!dma && g.transA) p.variant = 0;
    const bool commWritesOutput = quant && deterministic != 0 && P > 1 && (uintptr_t)scale_x2 % 16 == 0 && (uintptr_t)d_out % 8 == 0;
    if (dma && commWritesOutput) g.flags |= GF_KEPT_INT32_ONLY;   // (the comm rounds write every kept row's output)

    CommArgs c;
    memset(&c, 0, sizeof(c));
    c.local = local;
    c.localLd = tiling->n;
    for (uint32_t s = 0; s + 1 < P; ++s) c.peers[s] = d.peers[s];
    c.peerLd = peerLd;
    c.peerRowOffset = d.peerRowOffset;
    c.P = P; c.rank = d.rankIdx;
    c.mRank = sp.mRank; c.N = tiling->n;
    c.m0 = m0; c.n0 = n0; c.loopsM = sp.loopsM; c.loopsN = sp.loopsN; c.off = sp.off; c.dir = sp.dir;
    c.commBlockM = cb;
    c.splitRow = splitRow; c.splitCol = splitCol;
    c.swizzleDir = 0;
    c.dtype = quant ? (uint32_t)CT_INT32 : outDt;
    const uint32_t cores = splitRow * splitCol;
    // deterministic W8A8 rounds finish their blocks themselves (int32 sums and the dequantised rows in one pass over them)
    const bool fuseDequant = commWritesOutput;
    if (fuseDequant) {
        c.dOut = d_out;
        c.ldd = tiling->n;
        c.scaleN = (const float *)scale_x2;
        c.scaleM = (const float *)scale_x1 + (size_t)d.rankIdx * sp.mRank;
        c.outDtype = outDt;
    }

    const uint32_t bpc = sp.blockPerComm, perRank = bpc / P, stages = sp.stages;
    const uint32_t rounds = ceil_div(sp.coreLoops, bpc);
    // the events: the caller's plan, or a set made for this call alone
    CatcocPipelinedPlan own;
    CatcocPipelinedPlan *plan = given->pipelinedPlan;
    if (plan != nullptr) {
        if (plan->magic != kPlanMagic) { fail(E_DESC, "desc.pipelinedPlan does not point at a CatcocPipelinedPlan"); return; }
        if (plan->ready.size() < rounds) {
            fail(E_WORKSPACE, "this call has %u comm rounds; the plan holds events for %u", rounds, (uint32_t)plan->ready.size());
            return;
        }
    } else if (rounds > 1 && computeStream != commStream) {   // (a single round, or one stream, needs no event)
        plan = &own;
        if (!plan_make_events(own, rounds)) return;
    } else {
        plan = &own;
        own.ready.assign(rounds, nullptr);
        own.done.assign(rounds, nullptr);
    }
    std::vector<hipEvent_t> &ready = plan->ready, &done = plan->done;
    hipEvent_t fin = plan->fin;
    auto destroy = [&]() { if (plan == &own) plan_destroy_events(own); };
    hipError_t he = hipSuccess;
    // A single round has nothing to overlap: its comm side then runs on computeStream behind the GEMM and no event is needed.
    const bool oneStream = rounds == 1 || computeStream == commStream;
    hipStream_t cs = (hipStream_t)computeStream, ms = oneStream ? cs : (hipStream_t)commStream;
    int e = 0;
    for (uint32_t r = 0; r < rounds && e == 0 && he == hipSuccess; ++r) {
        const uint32_t first = r * bpc, actual = umin(bpc, sp.coreLoops - first);
        if (r >= stages && !oneStream) he = hipStreamWaitEvent(cs, done[r - stages], 0);   // "compute finished" of the stage's last user
        g.taskBase = first;
        g.taskCount = actual;
        if (he == hipSuccess)
            e = dma ? (p.dtype == DT_I8 ? launch_gemm_dma_i8(g, computeStream)
                       : p.dtype == DT_F16 ? launch_gemm_dma_f16(g, computeStream) : launch_gemm_dma_bf16(g, computeStream))
                    : launch_gemm(p.dtype, g, p.variant, p.edge, computeStream);
        if (e == 0 && he == hipSuccess && !oneStream) he = hipEventRecord(ready[r], cs);   // "store finished"
        if (e == 0 && he == hipSuccess && !oneStream) he = hipStreamWaitEvent(ms, ready[r], 0);
        c.roundFirstIdx = r * perRank;
        c.dataLoops = (actual / P) * (m0 / cb);
        if (e == 0 && he == hipSuccess && P > 1 && c.dataLoops > 0) e = launch_comm_reduce(c, cores, deterministic != 0, ms);
        if (e == 0 && he == hipSuccess && !oneStream) he = hipEventRecord(done[r], ms);
    }
    if (e == 0 && he == hipSuccess && quant && !fuseDequant)   // the pass after all rounds: dequantise the reduced int32 block
        e = launch_dequant_rows((const int32_t *)c_accum, tiling->n, (const float *)scale_x2, (const float *)scale_x1 + (size_t)d.rankIdx * sp.mRank,
                                d_out, tiling->n, sp.mRank, tiling->n, outDt, ms);
    if (e == 0 && he == hipSuccess && !oneStream) he = hipEventRecord(fin, ms);
    if (e == 0 && he == hipSuccess && !oneStream) he = hipStreamWaitEvent(cs, fin, 0);   // the caller's stream sees the finished output
    destroy();
    if (e) { fail(E_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)e)); return; }
    if (he != hipSuccess) { fail(E_LAUNCH, "stream/event call failed: %s", hipGetErrorString(he)); return; }
    ok();
}

// ---- built-in scratch for callers that cannot allocate ---------------------------------------
// One array per GPU, part of the library's code object: it exists from the moment the library is loaded on a device
// until the process ends.  In host code the array's name is only a handle for hipGetSymbolAddress; everything that
// needs the memory (kernel arguments, the fill below) uses the per-device address obtained from it.
static __device__ __align__(256) unsigned char scratch[CATCOC_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
struct ScratchState { void *ptr; };
ScratchState g_scratch[kMaxDevices];
pthread_mutex_t g_scratchLock = PTHREAD_MUTEX_INITIALIZER;

// Address of the current device's copy of `scratch`; NULL on failure.  Nothing has to be cleared: a __device__ array is
// zero when the code object is loaded, and every launch leaves the counter block at zero again for the next.
void *scratch_for_current_device()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        fail(E_LAUNCH, "no current HIP device (or more than %d devices)", kMaxDevices);
        return nullptr;
    }
    pthread_mutex_lock(&g_scratchLock);
    ScratchState &st = g_scratch[dev];
    if (st.ptr == nullptr) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr) {
            pthread_mutex_unlock(&g_scratchLock);
            fail(E_LAUNCH, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        st.ptr = p;
    }
    void *p = st.ptr;
    pthread_mutex_unlock(&g_scratchLock);
    return p;
}

}  // namespace

extern "C" {

void catcoc_launch_quant_matmul_reduce_scatter_static_scratch(void *stream, uint64_t fftsAddr, uint8_t *x1, uint8_t *x2,
                                                              uint8_t *scale_x1, uint8_t *scale_x2, uint8_t *bias,
                                                              uint8_t *c_accum, uint8_t *d_out, uint8_t *symmetricPtr,
                                                              CocTilingParams *tiling, uint32_t transA, uint32_t transB,
                                                              uint32_t outDataType)
{
    (void)fftsAddr;
    const CatcocSymmetricDesc *given = (const CatcocSymmetricDesc *)symmetricPtr;
    if (given == nullptr || given->magic != CATCOC_DESC_MAGIC) {
        fail(E_DESC, "symmetricPtr does not point at a CatcocSymmetricDesc");
        return;
    }
    CatcocSymmetricDesc d = *given;
    d.workspace = nullptr;
    d.workspaceBytes = 0;
    // how much scratch would this launch use?  Plan it first, with the sizes only.
    uint64_t need = 0;
    {
        CatcocSymmetricDesc q = d;
        for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!q.peers[i]) q.peers[i] = (const void *)16;
        if (q.keptRows != 0) {
            SplitkPlan sp;
            if (make_splitk_plan(tiling, &q, transA, transB, sp)) return;
            need = sp.workspaceBytes;
        } else {
            Plan p;
            q.flags &= ~CATCOC_OUTBOUND_MASK;
            if (make_plan(QUANT_MATMUL_REDUCE_SCATTER, INT8, tiling, &q, transA, transB, p)) return;
            need = p.kSliceBytes;
        }
    }
    if (need > (uint64_t)CATCOC_STATIC_SCRATCH_BYTES) {
        fail(E_WORKSPACE, "this launch needs %llu bytes of scratch; the built-in scratch holds %llu "
                          "(use catcoc_launch_quant_matmul_reduce_scatter with a workspace of your own)",
             (unsigned long long)need, (unsigned long long)CATCOC_STATIC_SCRATCH_BYTES);
        return;
    }
    if (need != 0) {
        void *p = scratch_for_current_device();
        if (p == nullptr) return;
        d.workspace = p;
        d.workspaceBytes = CATCOC_STATIC_SCRATCH_BYTES;
    }
    launch_quant(stream, x1, x2, scale_x1, scale_x2, bias, c_accum, d_out, (uint8_t *)&d, tiling, transA, transB, outDataType);
}

#define FLOAT_LAUNCHER(name, commType, dataType)                                                                      \
    void name(void *stream, uint64_t fftsAddr, uint8_t *a, uint8_t *b, uint8_t *c, uint8_t *aW, uint8_t *bW,           \
              uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA, uint32_t transB)                        \
    {                                                                                                                  \
        (void)fftsAddr; (void)aW; (void)bW;                                                                            \
        launch_float(commType, dataType, stream, a, b, c, symmetricPtr, tiling, transA, transB);                       \
    }

FLOAT_LAUNCHER(catcoc_launch_matmul_allreduce_fp16, MATMUL_ALLREDUCE, FP16)
FLOAT_LAUNCHER(catcoc_launch_matmul_allreduce_bf16, MATMUL_ALLREDUCE, BF16)
FLOAT_LAUNCHER(catcoc_launch_allgather_matmul_fp16, ALLGATHER_MATMUL, FP16)
FLOAT_LAUNCHER(catcoc_launch_allgather_matmul_bf16, ALLGATHER_MATMUL, BF16)
FLOAT_LAUNCHER(catcoc_launch_matmul_reduce_scatter_fp16, MATMUL_REDUCE_SCATTER, FP16)
FLOAT_LAUNCHER(catcoc_launch_matmul_reduce_scatter_bf16, MATMUL_REDUCE_SCATTER, BF16)

CatcocKernelFuncPtr catcoc_get_kernel(int commType, int dataType)
{
    switch ((commType << 8) | dataType) {  // key of KernelDispatcher::Hash, launch_map.h:30-33
        case (MATMUL_ALLREDUCE << 8) | FP16: return catcoc_launch_matmul_allreduce_fp16;
        case (MATMUL_ALLREDUCE << 8) | BF16: return catcoc_launch_matmul_allreduce_bf16;
        case (ALLGATHER_MATMUL << 8) | FP16: return catcoc_launch_allgather_matmul_fp16;
        case (ALLGATHER_MATMUL << 8) | BF16: return catcoc_launch_allgather_matmul_bf16;
        case (MATMUL_REDUCE_SCATTER << 8) | FP16: return catcoc_launch_matmul_reduce_scatter_fp16;
        case (MATMUL_REDUCE_SCATTER << 8) | BF16: return catcoc_launch_matmul_reduce_scatter_bf16;
        default: return nullptr;
    }
}

void catcoc_launch_quant_matmul_reduce_scatter(void *stream, uint64_t fftsAddr, uint8_t *x1, uint8_t *x2,
                                               uint8_t *scale_x1, uint8_t *scale_x2, uint8_t *bias, uint8_t *c_accum,
                                               uint8_t *d_out, uint8_t *symmetricPtr, CocTilingParams *tiling,
                                               uint32_t transA, uint32_t transB, uint32_t outDataType)
{
    (void)fftsAddr;
    launch_quant(stream, x1, x2, scale_x1, scale_x2, bias, c_accum, d_out, symmetricPtr, tiling, transA, transB, outDataType);
}

void catcoc_quant_matmul_reduce_scatter(void *stream, uint64_t fftsAddr, uint8_t *x1, uint8_t *x2, uint8_t *scale_x1,
                                        uint8_t *scale_x2, uint8_t *bias, uint8_t *c_accum, uint8_t *d_out,
                                        uint8_t *symmetricPtr, uint32_t m, uint32_t n, uint32_t k)
{
    (void)fftsAddr;
    // the example's fixed configuration (quant_matmul_reduce_scatter.cpp:93-147): tile 128x256, commInterval 10
    CocTilingParams t;
    memset(&t, 0, sizeof(t));
    t.m = m; t.n = n; t.k = k;
    t.m0 = 128; t.n0 = 256; t.k0 = 256;
    t.commInterval = 10;
    t.commTileM = 64; t.commBlockM = 64; t.commNpuSplit = 1; t.commDataSplit = 20;
    const CatcocSymmetricDesc *d = (const CatcocSymmetricDesc *)symmetricPtr;
    t.rankSize = (d && d->magic == CATCOC_DESC_MAGIC) ? d->rankSize : 0;
    launch_quant(stream, x1, x2, scale_x1, scale_x2, bias, c_accum, d_out, symmetricPtr, &t, 0, 0, BF16);
}

const char *catcoc_last_error(void) { return g_err; }
int catcoc_last_status(void) { return g_status; }

int catcoc_can_implement(int commType, int dataType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc,
                         uint32_t transA, uint32_t transB)
{
    Plan p;
    const int e = make_plan(commType, dataType, tiling, desc, transA, transB, p);
    if (!e) ok();
    return e;
}

uint64_t catcoc_get_workspace_size(int commType, int dataType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc)
{
    Plan p;
    CatcocSymmetricDesc d;
    if (desc == nullptr || tiling == nullptr) { fail(E_NULL, "tiling and desc must be non-NULL"); return 0; }
    d = *desc;
    d.flags &= ~CATCOC_OUTBOUND_MASK;  // size query must not require the buffer it sizes
    for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!d.peers[i]) d.peers[i] = (const void *)16;
    if (make_plan(commType, dataType, tiling, &d, 0, 0, p)) return 0;
    ok();
    return (uint64_t)p.args.sched.stages * p.args.sched.blockPerComm * p.args.sched.m0 * p.args.sched.n0 * 4u;
}

uint64_t catcoc_get_kslice_workspace_size(int commType, int dataType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc,
                                          uint32_t *kSlices)
{
    Plan p;
    CatcocSymmetricDesc d;
    if (desc == nullptr || tiling == nullptr) { fail(E_NULL, "tiling and desc must be non-NULL"); return 0; }
    d = *desc;
    d.flags &= ~CATCOC_OUTBOUND_MASK;
    d.workspace = nullptr;
    const uint32_t forced = d.splitK;
    d.splitK = 0;
    for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!d.peers[i]) d.peers[i] = (const void *)16;
    if (forced != 0) {   // size for the caller's own slice count: plan it with a workspace that is large enough
        d.splitK = forced;
        d.workspace = (void *)256;
        d.workspaceBytes = ~0ull;
    }
    if (make_plan(commType, dataType, tiling, &d, 0, 0, p)) return 0;
    ok();
    if (kSlices) *kSlices = p.kSlices;
    return p.kSliceBytes;
}

uint64_t catcoc_get_splitk_workspace_size(const CocTilingParams *tiling, const CatcocSymmetricDesc *desc, uint32_t *splitK,
                                          uint32_t *tiles)
{
    SplitkPlan sp;
    CatcocSymmetricDesc d;
    if (desc == nullptr || tiling == nullptr) { fail(E_NULL, "tiling and desc must be non-NULL"); return 0; }
    d = *desc;
    for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!d.peers[i]) d.peers[i] = (const void *)16;
    if (make_splitk_plan(tiling, &d, 0, 0, sp)) return 0;
    ok();
    if (splitK) *splitK = sp.f;
    if (tiles) *tiles = sp.tiles;
    return sp.workspaceBytes;
}

uint32_t catcoc_get_task_count(int commType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc)
{
    Plan p;
    CatcocSymmetricDesc d;
    if (desc == nullptr || tiling == nullptr) { fail(E_NULL, "tiling and desc must be non-NULL"); return 0; }
    d = *desc;
    d.flags &= ~CATCOC_OUTBOUND_MASK;
    for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!d.peers[i]) d.peers[i] = (const void *)16;
    const int dataType = commType == QUANT_MATMUL_REDUCE_SCATTER ? INT8 : FP16;
    if (make_plan(commType, dataType, tiling, &d, 0, 0, p)) return 0;
    ok();
    return p.args.sched.coreLoops;
}

int catcoc_task_tile(int commType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc, uint32_t task,
                     uint32_t *targetRank, uint32_t *row, uint32_t *col, uint32_t *wsRow)
{
    Plan p;
    CatcocSymmetricDesc d;
    if (desc == nullptr || tiling == nullptr) { fail(E_NULL, "tiling and desc must be non-NULL"); return 0; }
    d = *desc;
    d.flags &= ~CATCOC_OUTBOUND_MASK;
    for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!d.peers[i]) d.peers[i] = (const void *)16;
    const int dataType = commType == QUANT_MATMUL_REDUCE_SCATTER ? INT8 : FP16;
    if (make_plan(commType, dataType, tiling, &d, 0, 0, p)) return 0;
    ok();
    TileInfo ti;
    if (!task_tile(p.args.sched, task, ti)) return 0;
    if (targetRank) *targetRank = ti.targetRank;
    if (row) *row = ti.row;
    if (col) *col = ti.col;
    if (wsRow) *wsRow = ti.wsRow;
    return 1;
}

uint32_t catcoc_task_tiles(int commType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc, uint32_t firstTask, uint32_t count,
                           uint32_t *targetRank, uint32_t *row, uint32_t *col, uint32_t *wsRow)
{
    Plan p;
    CatcocSymmetricDesc d;
    if (desc == nullptr || tiling == nullptr) { fail(E_NULL, "tiling and desc must be non-NULL"); return 0; }
    d = *desc;
    d.flags &= ~CATCOC_OUTBOUND_MASK;
    for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!d.peers[i]) d.peers[i] = (const void *)16;
    const int dataType = commType == QUANT_MATMUL_REDUCE_SCATTER ? INT8 : FP16;
    if (make_plan(commType, dataType, tiling, &d, 0, 0, p)) return 0;   // planned once for the whole range
    ok();
    uint32_t n = 0;
    for (; n < count; ++n) {
        TileInfo ti;
        if (!task_tile(p.args.sched, firstTask + n, ti)) break;
        if (targetRank) targetRank[n] = ti.targetRank;
        if (row) row[n] = ti.row;
        if (col) col[n] = ti.col;
        if (wsRow) wsRow[n] = ti.wsRow;
    }
    return n;
}

int catcoc_launch_tile(int commType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc, uint32_t wg, uint32_t *task,
                       uint32_t *targetRank, uint32_t *row, uint32_t *col, uint32_t *wsRow)
{
    Plan p;
    CatcocSymmetricDesc d;
    if (desc == nullptr || tiling == nullptr) { fail(E_NULL, "tiling and desc must be non-NULL"); return 0; }
    d = *desc;
    d.flags &= ~CATCOC_OUTBOUND_MASK;
    for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!d.peers[i]) d.peers[i] = (const void *)16;
    const int dataType = commType == QUANT_MATMUL_REDUCE_SCATTER ? INT8 : FP16;
    if (make_plan(commType, dataType, tiling, &d, 0, 0, p)) return 0;
    ok();
    const SchedParams &s = p.args.sched;
    const bool linear = (p.args.flags & GF_LINEAR_ORDER) != 0;
    uint32_t t;
    TileInfo ti;
    if (p.dma) {
        if (!launch_tile(s, wg, linear, p.args.keptRank, t, ti)) return 0;
    } else {
        if (wg >= s.coreLoops) return 0;
        t = launch_order_task(s, wg, linear, p.args.keptRank);
        if (!task_tile(s, t, ti)) return 0;
    }
    if (task) *task = t;
    if (targetRank) *targetRank = ti.targetRank;
    if (row) *row = ti.row;
    if (col) *col = ti.col;
    if (wsRow) *wsRow = ti.wsRow;
    return 1;
}

uint32_t catcoc_launch_task(int commType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc, uint32_t wg)
{
    Plan p;
    CatcocSymmetricDesc d;
    if (desc == nullptr || tiling == nullptr) { fail(E_NULL, "tiling and desc must be non-NULL"); return 0xffffffffu; }
    d = *desc;
    d.flags &= ~CATCOC_OUTBOUND_MASK;
    for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!d.peers[i]) d.peers[i] = (const void *)16;
    const int dataType = commType == QUANT_MATMUL_REDUCE_SCATTER ? INT8 : FP16;
    if (make_plan(commType, dataType, tiling, &d, 0, 0, p)) return 0xffffffffu;
    ok();
    const SchedParams &s = p.args.sched;
    if (wg >= s.coreLoops) return 0xffffffffu;
    if (!p.dma) return launch_order_task(s, wg, (p.args.flags & GF_LINEAR_ORDER) != 0, p.args.keptRank);
    return launch_task(s, wg, (p.args.flags & GF_LINEAR_ORDER) != 0, p.args.keptRank);
}

uint32_t catcoc_kept_split_tiles(int commType, int dataType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc,
                                 uint32_t transA, uint32_t transB)
{
    Plan p;
    CatcocSymmetricDesc d;
    if (desc == nullptr || tiling == nullptr) { fail(E_NULL, "tiling and desc must be non-NULL"); return 0; }
    d = *desc;
    for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!d.peers[i]) d.peers[i] = (const void *)16;
    if (make_plan(commType, dataType, tiling, &d, transA, transB, p)) return 0;
    ok();
    if (!p.dma || p.args.sched.m0 != 128) return 0;
    return 8u * split_kept_tiles(p.args, p.args.K * elem_size(p.dtype) / 64u);
}

uint32_t catcoc_tail_split_tiles(int commType, int dataType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc,
                                 uint32_t transA, uint32_t transB)
{
    Plan p;
    CatcocSymmetricDesc d;
    if (desc == nullptr || tiling == nullptr) { fail(E_NULL, "tiling and desc must be non-NULL"); return 0; }
    d = *desc;
    for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!d.peers[i]) d.peers[i] = (const void *)16;
    if (make_plan(commType, dataType, tiling, &d, transA, transB, p)) return 0;
    ok();
    if (!p.dma || p.args.sched.m0 != 128) return 0;
    return 8u * split_tail_tiles(p.args, split_kept_tiles(p.args, p.args.K * elem_size(p.dtype) / 64u));
}

uint32_t catcoc_workgroup_task(uint32_t wg, uint32_t tasks, uint32_t flags)
{
    return workgroup_task(wg, tasks, (flags & CATCOC_FLAG_LINEAR_ORDER) != 0);
}

// ---- dynamic_tiling host logic ------------------------------------------------

int catcoc_check_comm_interval_reduce_scatter(const CocTilingParams *t, int rankSize, int blockNum)
{
    return rankSize > 0 && ((int64_t)blockNum * t->commInterval) % rankSize == 0;
}

static int32_t max_peer_mem_per_rank(int rankSize)
{
    // (LCAL_BUFF_BYTES - FLAG_BUFF_BYTES) / INPUT_DTYPE / rankSize / MAX_BLOCK_COUNT, info.h:24-27
    return (204 * 1024 * 1024 - 5 * 512 * 1024) / 2 / rankSize / 2;
}

int catcoc_check_comm_interval_allreduce(const CocTilingParams *t, int rankSize, int blockNum)
{
    if (rankSize <= 0) return 0;
    return t->commInterval * t->m0 * t->n0 * (uint32_t)blockNum < (uint32_t)max_peer_mem_per_rank(rankSize);
}

int catcoc_check_comm_interval_allgather(const CocTilingParams *t, int rankSize)
{
    if (rankSize <= 0) return 0;
    const uint32_t kLoop = t->k0 ? ceil_div(t->k, t->k0) : 0u;
    return t->commInterval * t->m0 * t->k0 * kLoop < (uint32_t)max_peer_mem_per_rank(rankSize);
}

int catcoc_get_tilings(const CocTilingParams *base, int commType, int rankSize, int blockNum, CocTilingParams *out, int maxOut)
{
    // search space of tiling.h:19-22 in its nesting order: interval (outer), tile M, then the split pairs
    static const uint32_t intervals[] = {4, 6, 8, 12, 14};
    static const uint32_t tileMs[] = {4, 8, 16, 32, 64};
    static const uint32_t splits[][2] = {{1, 16}, {1, 20}};
    if (base == nullptr) { fail(E_NULL, "base tiling is NULL"); return 0; }
    int n = 0;
    for (uint32_t ci : intervals)
        for (uint32_t tm : tileMs)
            for (auto &sp : splits) {
                CocTilingParams t = *base;
                t.commInterval = ci;
                t.commTileM = tm;
                t.commBlockM = tm;
                t.commNpuSplit = sp[0];
                t.commDataSplit = sp[1];
                bool valid = true;
                if (commType == ALLGATHER_MATMUL) valid = catcoc_check_comm_interval_allgather(&t, rankSize);
                else if (commType == MATMUL_REDUCE_SCATTER || commType == QUANT_MATMUL_REDUCE_SCATTER)
                    valid = catcoc_check_comm_interval_reduce_scatter(&t, rankSize, blockNum);
                else if (commType == MATMUL_ALLREDUCE) valid = catcoc_check_comm_interval_allreduce(&t, rankSize, blockNum);
                if (!valid) continue;
                if (out && n < maxOut) out[n] = t;
                ++n;
            }
    return n;
}

uint32_t catcoc_get_splitk_factor(uint32_t m, uint32_t n, uint32_t k, uint32_t coreNum, uint32_t m0, uint32_t n0, uint32_t k0)
{
    if (!m0 || !n0 || !k0 || !coreNum) return 1;
    return splitk_factor(m, n, k, coreNum, m0, n0, k0);
}

void catcoc_default_tiling(CocTilingParams *t, uint32_t m, uint32_t k, uint32_t n, uint32_t rankSize)
{
    t->m = m; t->k = k; t->n = n;
    t->m0 = 128; t->k0 = 256; t->n0 = 256;
    t->commTileM = 64;
    t->commInterval = 20;
    t->commNpuSplit = 1;
    t->commDataSplit = 2;
    t->commBlockM = 64;
    t->rankSize = rankSize;
}

// ---- schedulers on the host ---------------------------------------------------

void catcoc_swizzle_block_coord(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN, uint32_t task, uint32_t *mIdx, uint32_t *nIdx)
{
    swizzle_block_coord(off, dir, loopsM, loopsN, task, *mIdx, *nIdx);
}

void catcoc_splitk_block_coord(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN, uint32_t kTiles, uint32_t f,
                               uint32_t task, uint32_t *mIdx, uint32_t *nIdx, uint32_t *kIdx, uint32_t *slice)
{
    splitk_block_coord(off, dir, loopsM, loopsN, kTiles, f, task, *mIdx, *nIdx, *kIdx, *slice);
}

uint32_t catcoc_splitk_actual_k(uint32_t K, uint32_t k0, uint32_t f, uint32_t slice) { return splitk_actual_k(K, k0, f, slice); }

uint32_t catcoc_splitk_launch_task(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN, uint32_t f, uint32_t wg)
{
    return splitk_launch_task(off, dir, loopsM, loopsN, f, wg);
}

void catcoc_allgather_block_coord(uint32_t off, uint32_t dir, uint32_t P, uint32_t commInterval, uint32_t loopsMRank,
                                  uint32_t loopsN, uint32_t task, uint32_t *mIdx, uint32_t *nIdx)
{
    allgather_block_coord(off, dir, P, commInterval, loopsMRank, loopsN, task, *mIdx, *nIdx);
}

void catcoc_comm_block_idx(uint32_t dir, uint32_t P, uint32_t splitRow, uint32_t splitCol, uint32_t dataLoopsInRank,
                           uint32_t task, uint32_t *dataIdx, uint32_t *rankIdx)
{
    comm_block_idx(dir, P, splitRow, splitCol, dataLoopsInRank, task, *dataIdx, *rankIdx);
}

int catcoc_device_info(int *cuCount, int *clockMHz, char *name, int nameLen)
{
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
        return fail(E_LAUNCH, "no HIP device");
    if (cuCount) *cuCount = prop.multiProcessorCount;
    if (clockMHz) *clockMHz = prop.clockRate / 1000;
    if (name && nameLen > 0) { strncpy(name, prop.gcnArchName, nameLen - 1); name[nameLen - 1] = 0; }
    ok();
    return 0;
}

const char *catcoc_version(void) { return "catcoc-hip 0.2 (gfx950)"; }

void catcoc_pipelined_quant_matmul_reduce_scatter(void *computeStream, void *commStream, uint64_t fftsAddr, uint8_t *x1, uint8_t *x2,
                                                  uint8_t *scale_x1, uint8_t *scale_x2, uint8_t *bias, uint8_t *c_accum, uint8_t *d_out,
                                                  uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA, uint32_t transB,
                                                  uint32_t outDataType, uint32_t deterministic)
{
    (void)fftsAddr;
    launch_pipelined(true, INT8, computeStream, commStream, x1, x2, scale_x1, scale_x2, bias, c_accum, d_out, symmetricPtr, tiling, transA,
                     transB, outDataType, deterministic);
}

CatcocPipelinedPlan *catcoc_pipelined_plan_create(uint32_t maxRounds)
{
    if (maxRounds == 0 || maxRounds > 65536u) { fail(E_TILING, "maxRounds %u out of range 1..65536", maxRounds); return nullptr; }
    CatcocPipelinedPlan *p = new (std::nothrow) CatcocPipelinedPlan();
    if (p == nullptr) { fail(E_LAUNCH, "out of host memory"); return nullptr; }
    if (!plan_make_events(*p, maxRounds)) { delete p; return nullptr; }
    ok();
    return p;
}

void catcoc_pipelined_plan_destroy(CatcocPipelinedPlan *plan)
{
    if (plan == nullptr) return;
    plan_destroy_events(*plan);
    delete plan;
}

uint32_t catcoc_pipelined_round_count(int commType, const CocTilingParams *tiling, const CatcocSymmetricDesc *desc)
{
    if (desc == nullptr || desc->magic != CATCOC_DESC_MAGIC) { fail(E_DESC, "desc does not point at a CatcocSymmetricDesc"); return 0; }
    if (commType != MATMUL_REDUCE_SCATTER && commType != QUANT_MATMUL_REDUCE_SCATTER) {
        fail(E_DTYPE, "the round-pipelined form exists for the reduce-scatter operators (commType %d)", commType);
        return 0;
    }
    CatcocSymmetricDesc q = *desc;
    for (int i = 0; i < CATCOC_MAX_RANKS; ++i) if (!q.peers[i]) q.peers[i] = (const void *)16;
    q.flags &= ~CATCOC_OUTBOUND_MASK;
    q.workspace = nullptr;
    q.splitK = 0;
    Plan p;
    if (make_plan(commType, commType == QUANT_MATMUL_REDUCE_SCATTER ? INT8 : FP16, tiling, &q, 0, 0, p)) return 0;
    ok();
    return ceil_div(p.args.sched.coreLoops, p.args.sched.blockPerComm);
}

void catcoc_pipelined_matmul_reduce_scatter(void *computeStream, void *commStream, int dataType, uint8_t *a, uint8_t *b, uint8_t *c,
                                            uint8_t *symmetricPtr, CocTilingParams *tiling, uint32_t transA, uint32_t transB,
                                            uint32_t deterministic)
{
    launch_pipelined(false, dataType, computeStream, commStream, a, b, nullptr, nullptr, nullptr, nullptr, c, symmetricPtr, tiling, transA,
                     transB, (uint32_t)dataType, deterministic);
}

void catcoc_reduce_add(void *stream, uint8_t *dst, uint8_t *src, uint64_t elementCount, uint32_t splitkFactor, uint32_t outDataType)
{
    if (!dst || !src) { fail(E_NULL, "dst and src must be non-NULL"); return; }
    if (splitkFactor == 0) { fail(E_TILING, "splitkFactor must be at least 1"); return; }
    if (outDataType != 0 && outDataType != FP16 && outDataType != BF16) { fail(E_DTYPE, "outDataType %u must be 0 (fp32), FP16 or BF16", outDataType); return; }
    if (elementCount == 0) { ok(); return; }
    if ((uintptr_t)src % 16 != 0 || (uintptr_t)dst % 16 != 0 || (splitkFactor > 1 && elementCount % 4 != 0)) {
        fail(E_SHAPE, "reduce-add needs 16-byte aligned buffers and, with more than one slice, an element count that is a multiple of 4");
        return;
    }
    const int e = launch_reduce_add(dst, (const float *)src, elementCount, splitkFactor, outDataType, stream);
    if (e) { fail(E_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)e)); return; }
    ok();
}

int catcoc_verify(const float *out, const float *gold, uint64_t count, int dataType, uint32_t computeTimes, uint64_t *nBad, double *meanRelErr)
{
    // examples/utils/utils.py:44-52 and verify_result.py:34-43,88-117
    if ((!out || !gold) && count) { fail(E_NULL, "out and gold must be non-NULL"); return 0; }
    if (dataType != FP16 && dataType != BF16) { fail(E_DTYPE, "dataType %d must be FP16 or BF16", dataType); return 0; }
    const float rtol = dataType == FP16 ? (computeTimes < 2048 ? 1.0f / 256 : 1.0f / 128) : (computeTimes < 2048 ? 1.0f / 128 : 1.0f / 64);
    const double meanLimit = dataType == FP16 ? 1.0 / 1024 : 1.0 / 128;
    uint64_t bad = 0;
    double sum = 0.0;
    for (uint64_t i = 0; i < count; ++i) {
        float o = out[i], g = gold[i];
        if (isnan(o) || isinf(o)) o = 0.0f;       // NaN / Inf are zeroed before the comparison
        if (isnan(g) || isinf(g)) g = 0.0f;
        const float scale = fabsf(g) > 1.0f ? fabsf(g) : 1.0f;
        const float diff = o - g;
        if (fabsf(diff) - rtol * scale > 0.0f) ++bad;
        sum += (double)(diff / scale);
    }
    const double mean = count ? fabs(sum / (double)count) : 0.0;
    if (nBad) *nBad = bad;
    if (meanRelErr) *meanRelErr = mean;
    ok();
    return bad == 0 && mean <= meanLimit;
}

void catcoc_comm_block_idx_ex(uint32_t dir, uint32_t deterministic, uint32_t P, uint32_t splitRow, uint32_t splitCol,
                              uint32_t dataLoopsInRank, uint32_t task, uint32_t *dataIdx, uint32_t *rankIdx)
{
    comm_block_idx_ex(dir, deterministic != 0, P, splitRow, splitCol, dataLoopsInRank, task, *dataIdx, *rankIdx);
}

uint32_t catcoc_comm_core_loop(uint32_t deterministic, uint32_t P, uint32_t splitRow, uint32_t splitCol, uint32_t dataLoopsInRank)
{
    return comm_core_loop(deterministic != 0, P, splitRow, splitCol, dataLoopsInRank);
}

}  // extern "C"
