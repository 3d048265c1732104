// Kernel argument block shared by the fused GEMM kernels and the host launcher.
#pragma once
#include <stdint.h>

#include "tile_sched.h"

namespace catcoc {

constexpr int kMaxRanks = 16;

// Element type codes: the CocDataType values of the C ABI.
enum : uint32_t { DT_F16 = 1, DT_I8 = 2, DT_BF16 = 27 };

enum : uint32_t {
    GF_OUTBOUND_STORE = 1u << 0,  // non-kept tiles are stored to `outbound` (else folded into `checksum`)
    GF_REDUCE_INT32 = 1u << 1,    // W8A8: peers are int32 and are added before the dequant
    GF_LINEAR_ORDER = 1u << 2,    // workgroup i runs task i
    GF_ROW_MASK = 1u << 3,        // kept rows [keptBegin, +keptRows) are whole 32-row blocks that need not line up with tiles: the
                                  // epilogue works per 32-row block, and `checksum` takes the rows that are not kept per 128 x 128
                                  // block, index (row / 128) * (N / 128) + col / 128
    GF_KEPT_WHOLE = 1u << 5,      // never run kept tiles as two 64-row workgroups
    GF_KEPT_SPLIT = 1u << 6,      // do so whenever the launch allows it (default: by tile count and k length)
    GF_TAIL_WHOLE = 1u << 7,      // never run the tiles that wait for the slots of kept halves as two 64-row workgroups
    GF_KEPT_INT32_ONLY = 1u << 8, // W8A8, direct-to-LDS kernels: kept tiles store c_accum and nothing else (the caller dequantises later)
    GF_RAGGED = 1u << 4,          // the last tile row of a rank and / or the last tile column are not full: such tiles are computed as
                                  // whole tiles moved up / left so that they end at the edge (they overlap their neighbours, whose
                                  // values they reproduce bit for bit); sums and workspace stores leave the overlap out
};

struct GemmArgs {
    const void *a[kMaxRanks];      // A operand per rank (all-gather: the P shards; otherwise a[0])
    const void *b;
    void *d;                       // kept rows, 16-bit output [keptRows, N]
    const void *peers[kMaxRanks];  // staged peer partials for the kept rows
    const float *scaleM;           // W8A8 per-token scale, indexed by global A row
    const float *scaleN;           // W8A8 per-channel scale
    const int32_t *bias;           // W8A8 optional int32 bias[N]
    int32_t *cAccum;               // W8A8 optional int32 [keptRows, N]
    void *accDump;                 // optional full [M, N] local partial (int32 / fp32)
    void *outbound;                // tile-linear workspace for non-kept tiles
    void *checksum;                // per-task int64 (W8A8) / double (float) sums of non-kept tiles
    int64_t lda, ldb, ldd;         // leading dimensions in elements
    int64_t peerLd, peerRowOffset;
    uint32_t M, N, K;              // M = rows of the local A operand
    uint32_t nPeers;
    uint32_t keptRank;             // rank whose row block is kept (launch order puts its tiles first)
    uint32_t keptBegin, keptRows;  // global rows [keptBegin, keptBegin + keptRows) are reduced and written to d
    uint32_t flags;                // GF_*
    uint32_t outDtype;             // DT_F16 / DT_BF16
    uint32_t transA, transB;
    uint32_t taskBase, taskCount;  // positions [taskBase, taskBase + taskCount) of the launch order (round-by-round launches); taskCount 0 = all
    // Skinny-M split-K launch: k slices per tile, int32 partial tiles [splitK][tiles][128][128], one counter per tile.
    uint32_t splitK;
    int32_t *skPart;
    uint32_t *skCount;
    SchedParams sched;
};

// Workgroups (before k slicing) a launch starts.
inline uint32_t launch_positions(const GemmArgs &a) { return a.taskCount ? a.taskCount : a.sched.coreLoops; }

// Kept tiles per XCD when a launch qualifies for gemm_dma_split_kept_kernel, else 0: a whole reduce-scatter launch in the
// XCD-block order, A as [m,k], the kept rows exactly the kept rank's block with peers to stream, and by default either
// fewer tiles than CUs or at most one round of workgroups (512 tiles) with at most 80 k steps per tile.  Measured with
// the two variants alternating launch by launch and the inputs rotating over several sets (W8A8, N = 4096, 512 tiles, whole ->
// split with the waiting tiles as halves, us): 28 / 56 / 64 / 72 / 80 / 112 k steps 55.6 -> 42.7 / 77.4 -> 70.7 / 87.1 -> 84.4 /
// 90.4 -> 86.9 / 97.6 -> 95.9 / 125.8 -> 130.7; fp16 56 / 64 / 80 / 112 steps 78.5 -> 72.8 / 87.9 -> 84.8 / 98.1 -> 97.5 / 126.9 ->
// 131.8; 128 tiles with 112 steps 67.3 -> 49.8; 768 tiles 59.3 -> 59.1; 1024 tiles 74.8 -> 83.3.  GF_KEPT_WHOLE / GF_KEPT_SPLIT
// override.
inline uint32_t split_kept_tiles(const GemmArgs &a, uint32_t kSteps)
{
    const SchedParams &s = a.sched;
    if (s.m0 != 128 || a.splitK > 1 || a.taskBase != 0 || a.taskCount != 0 || (a.flags & (GF_LINEAR_ORDER | GF_ROW_MASK | GF_RAGGED)) ||
        a.transA || a.nPeers == 0 || a.keptBegin != a.keptRank * s.mRank || a.keptRows != s.mRank)
        return 0;
    if (a.flags & GF_KEPT_WHOLE) return 0;
    if (!(a.flags & GF_KEPT_SPLIT) && !(s.coreLoops < 256u || (s.coreLoops <= 512u && kSteps <= 80u))) return 0;
    return xcd_uniform_kept(s, a.keptRank);
}

// Tiles per XCD at the END of the launch order that a launch with split kept tiles also runs as two 64-row workgroups: the
// tiles by which the launch exceeds the 512 workgroup slots of the GPU (each of them inherits the slot of a kept half).
// Their checksum halves meet through the counter block of a workspace: without one (and with checksums asked for) they
// stay whole.
inline uint32_t split_tail_tiles(const GemmArgs &a, uint32_t keptPerXcd)
{
    const SchedParams &s = a.sched;
    if (keptPerXcd == 0 || (a.flags & GF_TAIL_WHOLE)) return 0;
    if (!(a.flags & GF_OUTBOUND_STORE) && a.checksum != nullptr && (a.skCount == nullptr || s.coreLoops > 8192u)) return 0;
    const uint32_t wgs = s.coreLoops + 8u * keptPerXcd;
    if (wgs <= 512u) return 0;
    const uint32_t over = (wgs - 512u) >> 3;
    return over <= keptPerXcd && over + keptPerXcd <= (s.coreLoops >> 3) ? over : 0;
}

}  // namespace catcoc
