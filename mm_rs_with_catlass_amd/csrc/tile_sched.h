// Tile schedulers of the fused GEMM path, as integer functions that compile for
// both the host (C ABI, CPU tests) and the device (kernels).  Written from the
// behaviour of the reference's schedulers, cited per function (paths relative to
// the reference tree).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define CATCOC_HD __host__ __device__ inline
#else
#define CATCOC_HD inline
#endif

namespace catcoc {

CATCOC_HD uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1u) / b; }
CATCOC_HD uint32_t umin(uint32_t a, uint32_t b) { return a < b ? a : b; }

// Division by a launch constant without the float round trip a 32-bit division compiles to on the GPU (every
// workgroup runs a few dozen of them before its first load).  m = floor(2^32 / d); the estimate mulhi(n, m) is at
// most two short of n / d for any 32-bit n, so two conditional corrections make it exact.
struct FastDiv { uint32_t d, m; };
CATCOC_HD FastDiv make_fast_div(uint32_t d)
{
    FastDiv f;
    f.d = d ? d : 1u;
    const uint64_t m = 0x100000000ull / f.d;
    f.m = m > 0xffffffffull ? 0xffffffffu : (uint32_t)m;
    return f;
}
CATCOC_HD uint32_t fast_div(uint32_t n, const FastDiv &f, uint32_t &rem)
{
    uint32_t q = (uint32_t)(((uint64_t)n * f.m) >> 32);
    uint32_t r = n - q * f.d;
    if (r >= f.d) { ++q; r -= f.d; }
    if (r >= f.d) { ++q; r -= f.d; }
    rem = r;
    return q;
}

// Walk a 2-D grid in bands of `width` lines along the banded axis: inside a band
// the banded axis runs fastest; with `serpentine` the other axis runs backwards
// on odd bands.  The last band may be narrower.
CATCOC_HD void banded_walk(uint32_t width, uint32_t lenBanded, uint32_t lenOther, uint32_t idx, bool serpentine,
                           uint32_t &posBanded, uint32_t &posOther)
{
    const uint32_t perBand = width * lenOther;
    const uint32_t band = idx / perBand;
    const uint32_t in = idx - band * perBand;
    const uint32_t w = umin(width, lenBanded - band * width);
    const uint32_t q = in / w;
    posBanded = band * width + (in - q * w);
    posOther = (serpentine && (band & 1u)) ? lenOther - 1u - q : q;
}

// GemmIdentityBlockSwizzle<off,dir>::GetBlockCoord
// (3rdparty/catlass/include/catlass/gemm/block/block_swizzle.hpp:79-113).
// dir 0 bands tile rows, dir 1 bands tile columns.
CATCOC_HD void swizzle_block_coord(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN, uint32_t task,
                                   uint32_t &mIdx, uint32_t &nIdx)
{
    const uint32_t inner = task % (loopsM * loopsN);
    if (dir == 0) banded_walk(off, loopsM, loopsN, inner, true, mIdx, nIdx);
    else banded_walk(off, loopsN, loopsM, inner, true, nIdx, mIdx);
}

// Inverse of banded_walk / swizzle_block_coord: the position of tile (mIdx, nIdx) in the swizzled order.
CATCOC_HD uint32_t banded_index(uint32_t width, uint32_t lenBanded, uint32_t lenOther, bool serpentine, uint32_t posBanded,
                                uint32_t posOther)
{
    const uint32_t band = posBanded / width;
    const uint32_t w = umin(width, lenBanded - band * width);
    const uint32_t q = (serpentine && (band & 1u)) ? lenOther - 1u - posOther : posOther;
    return band * width * lenOther + q * w + (posBanded - band * width);
}

CATCOC_HD uint32_t swizzle_block_index(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN, uint32_t mIdx, uint32_t nIdx)
{
    return dir == 0 ? banded_index(off, loopsM, loopsN, true, mIdx, nIdx) : banded_index(off, loopsN, loopsM, true, nIdx, mIdx);
}

// SplitkGemmIdentityBlockSwizzle (block_swizzle.hpp:151-158): first k tile of slice s.
CATCOC_HD uint32_t splitk_first_ktile(uint32_t kTiles, uint32_t f, uint32_t s)
{
    const uint32_t base = kTiles / f, extra = kTiles % f;
    return s * base + umin(s, extra);
}

// block_swizzle.hpp:160-165,179-216.
CATCOC_HD void splitk_block_coord(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN, uint32_t kTiles,
                                  uint32_t f, uint32_t task, uint32_t &mIdx, uint32_t &nIdx, uint32_t &kIdx,
                                  uint32_t &slice)
{
    const uint32_t mn = loopsM * loopsN;
    slice = (task % (mn * f)) / mn;
    kIdx = splitk_first_ktile(kTiles, f, slice);
    swizzle_block_coord(off, dir, loopsM, loopsN, task % mn, mIdx, nIdx);
}

// Workgroup -> task of a split-K launch.  Workgroups are dealt round-robin to the eight XCDs, each with its own
// L2; the row tiles that read the same columns of B over the same k slice are given to one XCD, next to each
// other, so that B crosses the fabric once per slice instead of once per row tile.  With a single row of tiles
// nothing is shared and the reference's order stays (regrouping it measured 10-15 % slower at 8192 x 8192).
// A permutation of the reference's task indices: which task a workgroup runs does not change any result.
CATCOC_HD uint32_t splitk_launch_task(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN, uint32_t f, uint32_t wg)
{
    const uint32_t mn = loopsM * loopsN, total = mn * f;
    if (wg >= total || loopsM < 2u || (loopsN * f) % 8u != 0) return wg;
    const uint32_t x = wg & 7u, j = wg >> 3;
    const uint32_t grp = j / loopsM, mIdx = j - grp * loopsM;
    const uint32_t g = x * (loopsN * f / 8u) + grp;          // (slice, column tile) pair
    const uint32_t slice = g / loopsN, nIdx = g - slice * loopsN;
    return slice * mn + swizzle_block_index(off, dir, loopsM, loopsN, mIdx, nIdx);
}

// block_swizzle.hpp:220-235: k extent of a slice (the last slice takes what is left of K).
CATCOC_HD uint32_t splitk_actual_k(uint32_t K, uint32_t k0, uint32_t f, uint32_t s)
{
    const uint32_t kTiles = ceil_div(K, k0);
    if (s == f - 1u) return K - splitk_first_ktile(kTiles, f, s) * k0;
    return (kTiles / f + (s < kTiles % f ? 1u : 0u)) * k0;
}

// GemmIdentityBlockSwizzleAllGather::GetBlockCoord
// (include/catcoc/dgemm/block/block_swizzle_allgather.hpp:88-108): tiles of one comm
// round (commInterval tile rows from every rank) are swizzled as one grid, then the
// row index is re-based rank-major.
CATCOC_HD void allgather_block_coord(uint32_t off, uint32_t dir, uint32_t P, uint32_t commInterval,
                                     uint32_t loopsMRank, uint32_t loopsN, uint32_t task, uint32_t &mIdx,
                                     uint32_t &nIdx)
{
    const uint32_t rowsPerRound = commInterval * P;
    const uint32_t rowsAll = loopsMRank * P;
    const uint32_t rounds = ceil_div(rowsAll, rowsPerRound);
    const uint32_t round = task / (rowsPerRound * loopsN);
    const uint32_t inRound = task - round * rowsPerRound * loopsN;
    const uint32_t rowsHere = (round == rounds - 1u) ? rowsAll - round * rowsPerRound : rowsPerRound;
    const uint32_t perRank = rowsHere / P;
    uint32_t cm, cn;
    swizzle_block_coord(off, dir, rowsHere, loopsN, inRound, cm, cn);
    const uint32_t r = cm / perRank;
    mIdx = r * loopsMRank + round * commInterval + (cm - r * perRank);
    nIdx = cn;
}

// BlockCommSwizzle<dir,false>::GetBlockIdx
// (include/catcoc/comm_epilogue/block/comm_block_swizzle.hpp:147-186).
CATCOC_HD void comm_block_idx(uint32_t dir, uint32_t P, uint32_t splitRow, uint32_t splitCol,
                              uint32_t dataLoopsInRank, uint32_t task, uint32_t &dataIdx, uint32_t &rankIdx)
{
    const uint32_t inner = task % (dataLoopsInRank * P);
    uint32_t d, r;
    if (dir == 0) banded_walk(splitRow, dataLoopsInRank, P, inner, false, d, r);
    else banded_walk(splitCol, P, dataLoopsInRank, inner, false, r, d);
    const uint32_t stepped = r * (P / splitCol);
    r = (stepped % P + stepped / P + d) % P;
    dataIdx = d;
    rankIdx = r;
}

// BlockCommSwizzle<dir, deterministic> (comm_block_swizzle.hpp:25-31,54-56,114-118,147-186).  The deterministic
// variant folds the npu split into the data split (coreSplit = {row * col, 1}) and pads the last band to the full
// band width, so that core c of `row * col` cores meets every data block c, c + cores, ... with the ranks in a fixed
// sequence; data indices at or beyond dataLoopsInRank are padding (GetActualBlockShape returns an empty block there).
CATCOC_HD uint32_t comm_core_loop(bool deterministic, uint32_t P, uint32_t splitRow, uint32_t splitCol, uint32_t dataLoopsInRank)
{
    if (!deterministic) return dataLoopsInRank * P;
    const uint32_t cores = splitRow * splitCol;
    return ceil_div(dataLoopsInRank, cores) * cores * P;
}

CATCOC_HD void comm_block_idx_ex(uint32_t dir, bool deterministic, uint32_t P, uint32_t splitRow, uint32_t splitCol,
                                 uint32_t dataLoopsInRank, uint32_t task, uint32_t &dataIdx, uint32_t &rankIdx)
{
    if (!deterministic) {
        comm_block_idx(dir, P, splitRow, splitCol, dataLoopsInRank, task, dataIdx, rankIdx);
        return;
    }
    const uint32_t cores = splitRow * splitCol;                    // direction 0 only: bands of `cores` data blocks
    const uint32_t padded = ceil_div(dataLoopsInRank, cores) * cores;
    const uint32_t inner = task % (padded * P);
    uint32_t d, r;
    banded_walk(cores, padded, P, inner, false, d, r);
    dataIdx = d;
    rankIdx = (r + d) % P;                                         // nStride = P / 1: (r * P) % P + (r * P) / P = r
}

// ---------------------------------------------------------------------------
// Task -> tile of each operator
// ---------------------------------------------------------------------------

enum : uint32_t { OP_ALLREDUCE = 0, OP_ALLGATHER = 1, OP_REDUCE_SCATTER = 2 };

struct SchedParams {
    uint32_t op;            // OP_*
    uint32_t P;             // rankSize
    uint32_t mRank;         // rows of one rank's sub-problem (RS: M/P, AG: shard rows, AR: M)
    uint32_t N;
    uint32_t m0, n0;
    uint32_t loopsM, loopsN;  // tile grid of ONE rank's sub-problem
    uint32_t coreLoops;       // tasks of the launch
    uint32_t blockPerComm;    // blockNum * commInterval
    uint32_t commInterval;
    uint32_t stages;
    uint32_t off, dir;
    // XCD-block launch order worked out once per launch (xcd_launch_tile): the cut of the tile grid and the
    // divisors of the workgroup -> tile arithmetic
    uint32_t xOk;                 // the order applies to this launch
    uint32_t xRxLog, xCxLog;      // row parts x column parts = 8, as powers of two
    uint32_t xRowsPer, xColsPer;  // tile rows / tile columns of one XCD's block
    uint32_t xPerRank, xCommLoops, xLastPerRank;   // tasks of one rank in a full round; rounds; the same in the last round
    FastDiv dColsPer, dLoopsM, dBand, dPerRank, dStages, dBpc;
};

struct TileInfo {
    uint32_t targetRank;  // rank whose row block the tile belongs to (AG: rank whose shard feeds it)
    uint32_t rowInRank;   // first row inside that rank's sub-problem
    uint32_t row;         // first row in the global problem
    uint32_t col;         // first column
    uint32_t rowsValid, colsValid;
    uint32_t wsRow;       // first row of the tile in the reference's tile-linear workspace
};

CATCOC_HD void fill_xcd_order(SchedParams &s);

CATCOC_HD SchedParams make_sched(uint32_t op, uint32_t M, uint32_t N, uint32_t P, uint32_t m0, uint32_t n0,
                                 uint32_t blockNum, uint32_t commInterval, uint32_t stages, uint32_t off,
                                 uint32_t dir)
{
    SchedParams s;
    s.op = op;
    s.P = P;
    s.mRank = (op == OP_REDUCE_SCATTER) ? M / P : M;  // AG: M is already the shard's rows
    s.N = N;
    s.m0 = m0;
    s.n0 = n0;
    s.loopsM = ceil_div(s.mRank, m0);
    s.loopsN = ceil_div(N, n0);
    s.coreLoops = s.loopsM * s.loopsN * (op == OP_ALLREDUCE ? 1u : P);
    s.blockPerComm = blockNum * commInterval;
    s.commInterval = commInterval;
    s.stages = stages;
    s.off = off;
    s.dir = dir;
    fill_xcd_order(s);
    return s;
}

// quant_matmul_reduce_scatter.hpp:159-201 / matmul_reduce_scatter.hpp (same mapping),
// matmul_allreduce.hpp:146-179, allgather_matmul.hpp:131-163.
CATCOC_HD bool task_tile(const SchedParams &s, uint32_t t, TileInfo &ti)
{
    if (t >= s.coreLoops) return false;
    uint32_t mi, ni;
    if (s.op == OP_REDUCE_SCATTER) {
        const uint32_t perRank = s.blockPerComm / s.P;
        const uint32_t commLoops = ceil_div(s.coreLoops, s.blockPerComm);
        const uint32_t round = t / s.blockPerComm;
        const uint32_t b = t - round * s.blockPerComm;
        const uint32_t actual = (round == commLoops - 1u) ? s.coreLoops - round * s.blockPerComm : s.blockPerComm;
        const uint32_t actualInRank = actual / s.P;
        ti.targetRank = b / actualInRank;
        swizzle_block_coord(s.off, s.dir, s.loopsM, s.loopsN, round * perRank + b % actualInRank, mi, ni);
        ti.wsRow = ((round % s.stages) * s.blockPerComm + b) * s.m0;
    } else if (s.op == OP_ALLREDUCE) {
        const uint32_t round = t / s.blockPerComm;
        ti.targetRank = 0;
        swizzle_block_coord(s.off, s.dir, s.loopsM, s.loopsN, t, mi, ni);
        ti.wsRow = ((round % s.stages) * s.blockPerComm + (t - round * s.blockPerComm)) * s.m0;
    } else {
        uint32_t mAll;
        allgather_block_coord(s.off, s.dir, s.P, s.commInterval, s.loopsM, s.loopsN, t, mAll, ni);
        ti.targetRank = mAll / s.loopsM;
        mi = mAll - ti.targetRank * s.loopsM;
        // workspace row of the A block in the reference (allgather_matmul.hpp:150-161):
        // (stage * commInterval*P + rank * tileRowsPerRankThisRound + inCommIdx) * m0
        const uint32_t round = mi / s.commInterval;
        const uint32_t rounds = ceil_div(s.loopsM, s.commInterval);
        const uint32_t perRank = (round == rounds - 1u) ? s.loopsM - round * s.commInterval : s.commInterval;
        ti.wsRow = ((round % s.stages) * s.commInterval * s.P + ti.targetRank * perRank + mi % s.commInterval) * s.m0;
    }
    ti.rowInRank = mi * s.m0;
    ti.row = ti.targetRank * s.mRank + ti.rowInRank;
    ti.col = ni * s.n0;
    ti.rowsValid = umin(s.m0, s.mRank - ti.rowInRank);
    ti.colsValid = umin(s.n0, s.N - ti.col);
    return true;
}

// Workgroup -> task.  Hardware deals consecutive workgroups round-robin over the 8
// XCDs (each with its own L2); chunks of 16 consecutive tasks (neighbours in the
// swizzle, sharing A rows and B columns) are dealt to one XCD each, and successive
// chunks rotate over the XCDs so that every XCD gets the same share of each rank's
// tiles, including the expensive kept ones.  A bijection on [0,tasks).
CATCOC_HD uint32_t workgroup_task(uint32_t wg, uint32_t tasks, bool linear)
{
    const uint32_t X = 8u, CH = 16u;
    const uint32_t full = tasks / (X * CH) * (X * CH);
    if (linear || wg >= full) return wg;
    const uint32_t x = wg % X, s = wg / X;
    return ((s / CH) * X + x) * CH + s % CH;
}

// Reduce-scatter launches run the kept rank's tiles first: they are the long ones (their epilogue
// streams the peers' partials), so starting them first lets the short tiles fill in behind them.
// seq -> task: the kept tasks in their original order, then all others in theirs.  A bijection.
CATCOC_HD uint32_t kept_first_task(const SchedParams &s, uint32_t keptRank, uint32_t seq)
{
    if (s.op != OP_REDUCE_SCATTER || s.P <= 1) return seq;
    const uint32_t bpc = s.blockPerComm;
    const uint32_t perRank = bpc / s.P;                 // kept tasks in a full round
    const uint32_t fullRounds = s.coreLoops / bpc;
    const uint32_t lastInRank = (s.coreLoops - fullRounds * bpc) / s.P;
    const uint32_t keptCount = s.coreLoops / s.P;
    uint32_t round, inRank, idx;
    if (seq < keptCount) {
        if (seq < fullRounds * perRank) { round = seq / perRank; inRank = perRank; idx = seq - round * perRank; }
        else { round = fullRounds; inRank = lastInRank; idx = seq - fullRounds * perRank; }
        return round * bpc + keptRank * inRank + idx;
    }
    const uint32_t j = seq - keptCount;
    const uint32_t otherFull = bpc - perRank;
    if (j < fullRounds * otherFull) { round = j / otherFull; inRank = perRank; idx = j - round * otherFull; }
    else { round = fullRounds; inRank = lastInRank; idx = j - fullRounds * otherFull; }
    const uint32_t b = idx < keptRank * inRank ? idx : idx + inRank;
    return round * bpc + b;
}

// XCD-block launch order for reduce-scatter and all-reduce launches.  Consecutive workgroups go round-robin to the
// 8 XCDs, each with its own L2, so XCD x = wg mod 8 is given one block of the global tile grid (all ranks' rows):
// the grid is cut RX x CX = 8 ways, rows dealt round-robin to the RX row parts (every part then holds the same share
// of each rank's rows, kept ones included) and columns cut into CX contiguous parts, with RX x CX chosen to minimise
// the A rows plus B columns one XCD touches.  Inside its block an XCD walks row by row with the kept rank's rows
// first, so the tiles in flight on an XCD at any time share a few A row blocks and all of the block's B columns.
// Returns false when the grid does not divide evenly (callers fall back to the chunked order).
struct XcdBlock {
    uint32_t RX, CX;          // row parts x column parts = 8
    uint32_t rowsPer, colsPer;  // tile rows / tile columns of one XCD's block
    uint32_t rp, cp;          // this XCD's row part and column part
    uint32_t i0, i1;          // the block's tile rows rp + RX*i with i in [i0, i1) belong to the kept rank
};

// Geometry of XCD x's block; false when the order does not apply to this launch.
CATCOC_HD bool xcd_block(const SchedParams &s, uint32_t keptRank, uint32_t x, XcdBlock &g)
{
    if (s.op == OP_ALLGATHER || (s.coreLoops & 7u) != 0) return false;
    const bool rs = s.op == OP_REDUCE_SCATTER;
    const uint32_t GM = (rs ? s.P : 1u) * s.loopsM;
    if (GM * s.loopsN != s.coreLoops) return false;
    uint32_t RX = 0, best = 0xffffffffu;
    for (uint32_t r = 1; r <= 8; r <<= 1) {
        const uint32_t c = 8u / r;
        if (GM % r != 0 || s.loopsN % c != 0) continue;
        const uint32_t cost = (GM / r) * s.m0 + (s.loopsN / c) * s.n0;
        if (cost < best) { best = cost; RX = r; }
    }
    if (RX == 0) return false;
    g.RX = RX;
    g.CX = 8u / RX;
    g.rowsPer = GM / RX;
    g.colsPer = s.loopsN / g.CX;
    g.rp = x / g.CX;
    g.cp = x - g.rp * g.CX;
    g.i0 = g.i1 = 0;
    if (rs && s.P > 1) {
        const uint32_t lo = keptRank * s.loopsM, hi = lo + s.loopsM;
        g.i0 = umin(lo > g.rp ? ceil_div(lo - g.rp, RX) : 0u, g.rowsPer);
        g.i1 = umin(hi > g.rp ? ceil_div(hi - g.rp, RX) : 0u, g.rowsPer);
    }
    return true;
}

CATCOC_HD bool xcd_block_task(const SchedParams &s, uint32_t keptRank, uint32_t wg, uint32_t &task)
{
    XcdBlock g;
    if (wg >= s.coreLoops || !xcd_block(s, keptRank, wg & 7u, g)) return false;
    const uint32_t j = wg >> 3;
    const uint32_t ri = j / g.colsPer, ci = j - ri * g.colsPer;
    const uint32_t nk = g.i1 - g.i0;
    uint32_t i;
    if (ri < nk) i = g.i0 + ri;
    else { const uint32_t t = ri - nk; i = t < g.i0 ? t : t + nk; }
    const uint32_t gr = g.rp + g.RX * i, nIdx = g.cp * g.colsPer + ci;
    const uint32_t rank = gr / s.loopsM, mIdx = gr - rank * s.loopsM;
    const uint32_t inRank = swizzle_block_index(s.off, s.dir, s.loopsM, s.loopsN, mIdx, nIdx);
    if (s.op != OP_REDUCE_SCATTER) { task = inRank; return true; }
    const uint32_t perRank = s.blockPerComm / s.P;
    const uint32_t round = inRank / perRank, idx = inRank - round * perRank;
    const uint32_t commLoops = ceil_div(s.coreLoops, s.blockPerComm);
    const uint32_t actual = (round == commLoops - 1u) ? s.coreLoops - round * s.blockPerComm : s.blockPerComm;
    task = round * s.blockPerComm + rank * (actual / s.P) + idx;
    return true;
}

// The launch constants of the XCD-block order (part of SchedParams, filled by make_sched).
CATCOC_HD void fill_xcd_order(SchedParams &s)
{
    XcdBlock g;
    s.xOk = (s.stages != 0 && s.blockPerComm != 0 && s.blockPerComm % (s.op == OP_REDUCE_SCATTER ? s.P : 1u) == 0 &&
             xcd_block(s, 0, 0, g)) ? 1u : 0u;
    s.xRxLog = s.xCxLog = s.xRowsPer = s.xColsPer = s.xPerRank = s.xCommLoops = s.xLastPerRank = 0;
    s.dColsPer = s.dLoopsM = s.dBand = s.dPerRank = s.dStages = s.dBpc = make_fast_div(1);
    if (!s.xOk) return;
    while ((1u << s.xRxLog) < g.RX) ++s.xRxLog;
    s.xCxLog = 3u - s.xRxLog;
    s.xRowsPer = g.rowsPer;
    s.xColsPer = g.colsPer;
    const uint32_t ranks = s.op == OP_REDUCE_SCATTER ? s.P : 1u;
    s.xPerRank = s.blockPerComm / ranks;
    s.xCommLoops = ceil_div(s.coreLoops, s.blockPerComm);
    s.xLastPerRank = (s.coreLoops - (s.xCommLoops - 1u) * s.blockPerComm) / ranks;
    s.dColsPer = make_fast_div(g.colsPer);
    s.dLoopsM = make_fast_div(s.loopsM);
    s.dBand = make_fast_div(s.off);
    s.dPerRank = make_fast_div(s.xPerRank);
    s.dStages = make_fast_div(s.stages);
    s.dBpc = make_fast_div(s.blockPerComm);
}

// xcd_block_task followed by task_tile, from the launch constants and without a division: workgroup -> task and tile.
// Only for launches with s.xOk.
CATCOC_HD void xcd_launch_tile(const SchedParams &s, uint32_t keptRank, uint32_t wg, uint32_t &task, TileInfo &ti)
{
    const bool rs = s.op == OP_REDUCE_SCATTER;
    const uint32_t x = wg & 7u, j = wg >> 3;
    const uint32_t rp = x >> s.xCxLog, cp = x - (rp << s.xCxLog);
    uint32_t i0 = 0, i1 = 0;
    if (rs && s.P > 1) {
        const uint32_t lo = keptRank * s.loopsM, hi = lo + s.loopsM, up = (1u << s.xRxLog) - 1u;
        i0 = umin(lo > rp ? (lo - rp + up) >> s.xRxLog : 0u, s.xRowsPer);
        i1 = umin(hi > rp ? (hi - rp + up) >> s.xRxLog : 0u, s.xRowsPer);
    }
    uint32_t ci;
    const uint32_t ri = fast_div(j, s.dColsPer, ci);
    const uint32_t nk = i1 - i0;
    uint32_t i;
    if (ri < nk) i = i0 + ri;
    else { const uint32_t t = ri - nk; i = t < i0 ? t : t + nk; }
    const uint32_t gr = rp + (i << s.xRxLog), nIdx = cp * s.xColsPer + ci;
    uint32_t mIdx;
    const uint32_t rank = fast_div(gr, s.dLoopsM, mIdx);
    // position of (mIdx, nIdx) in the swizzled order of one rank's grid (banded_index with the band width s.off)
    const uint32_t posBanded = s.dir == 0 ? mIdx : nIdx, posOther = s.dir == 0 ? nIdx : mIdx;
    const uint32_t lenBanded = s.dir == 0 ? s.loopsM : s.loopsN, lenOther = s.dir == 0 ? s.loopsN : s.loopsM;
    uint32_t inBand;
    const uint32_t band = fast_div(posBanded, s.dBand, inBand);
    const uint32_t w = umin(s.off, lenBanded - band * s.off);
    const uint32_t q = (band & 1u) ? lenOther - 1u - posOther : posOther;
    const uint32_t inRank = band * s.off * lenOther + q * w + inBand;
    uint32_t round, b;
    if (rs) {
        uint32_t idx;
        round = fast_div(inRank, s.dPerRank, idx);
        b = rank * (round == s.xCommLoops - 1u ? s.xLastPerRank : s.xPerRank) + idx;
        task = round * s.blockPerComm + b;
    } else {
        task = inRank;
        round = fast_div(task, s.dBpc, b);
    }
    uint32_t stage;
    fast_div(round, s.dStages, stage);
    ti.targetRank = rank;
    ti.rowInRank = mIdx * s.m0;
    ti.row = rank * s.mRank + ti.rowInRank;
    ti.col = nIdx * s.n0;
    ti.rowsValid = umin(s.m0, s.mRank - ti.rowInRank);
    ti.colsValid = umin(s.n0, s.N - ti.col);
    ti.wsRow = (stage * s.blockPerComm + b) * s.m0;
}

// Kept tiles of one XCD's block under the XCD-block order when all eight XCDs hold the same number (they are then the first
// positions of every XCD), else 0.
inline uint32_t xcd_uniform_kept(const SchedParams &s, uint32_t keptRank)
{
    if (!s.xOk || s.op != OP_REDUCE_SCATTER || s.P <= 1 || (s.coreLoops & 7u) != 0) return 0;
    uint32_t per = 0;
    for (uint32_t x = 0; x < 8; ++x) {
        const uint32_t rp = x >> s.xCxLog;
        const uint32_t lo = keptRank * s.loopsM, hi = lo + s.loopsM, up = (1u << s.xRxLog) - 1u;
        const uint32_t i0 = umin(lo > rp ? (lo - rp + up) >> s.xRxLog : 0u, s.xRowsPer);
        const uint32_t i1 = umin(hi > rp ? (hi - rp + up) >> s.xRxLog : 0u, s.xRowsPer);
        const uint32_t k = (i1 - i0) * s.xColsPer;
        if (x == 0) per = k;
        else if (k != per) return 0;
    }
    return per;
}

// Workgroup -> task and tile of a launch of the direct-to-LDS kernels; false past the end of the launch.
CATCOC_HD bool launch_tile(const SchedParams &s, uint32_t wg, bool linear, uint32_t keptRank, uint32_t &task, TileInfo &ti);

// Workgroup -> task of a launch: the XCD-block order where it applies, else XCD-aware chunking with the kept
// rank's tiles first.  Either way the kept tiles are among the first ceil(kept / 128) * 128 workgroups.
CATCOC_HD uint32_t launch_task(const SchedParams &s, uint32_t wg, bool linear, uint32_t keptRank)
{
    if (linear) return wg;
    uint32_t task;
    if (xcd_block_task(s, keptRank, wg, task)) return task;
    return kept_first_task(s, keptRank, workgroup_task(wg, s.coreLoops, false));
}

CATCOC_HD bool launch_tile(const SchedParams &s, uint32_t wg, bool linear, uint32_t keptRank, uint32_t &task, TileInfo &ti)
{
    if (wg >= s.coreLoops) return false;
    if (!linear && s.xOk) {
        xcd_launch_tile(s, keptRank, wg, task, ti);
        return true;
    }
    task = launch_task(s, wg, linear, keptRank);
    return task_tile(s, task, ti);
}

// Workgroup -> task of a launch: XCD-aware chunking, then kept-first ordering.
CATCOC_HD uint32_t launch_order_task(const SchedParams &s, uint32_t wg, bool linear, uint32_t keptRank)
{
    if (linear) return wg;
    return kept_first_task(s, keptRank, workgroup_task(wg, s.coreLoops, false));
}

// SplitkMatmul::GetSplitkFactor (3rdparty/catlass/include/catlass/gemm/kernel/splitk_matmul.hpp:219-265).
inline uint32_t splitk_factor(uint32_t m, uint32_t n, uint32_t k, uint32_t cores, uint32_t m0, uint32_t n0,
                              uint32_t k0)
{
    const uint32_t cap = k <= 1024 ? 2u : k <= 2048 ? 4u : k <= 4096 ? 8u : 16u;
    const uint32_t base = ceil_div(m, m0) * ceil_div(n, n0);
    uint32_t f = umin(cores / base, cap);
    if (f == 0) f = 1;
    if (base < cores) {
        // keep growing while one more slice does not cost an extra wave of tiles
        while (f < cap && ceil_div(base * f, cores) >= ceil_div(base, cores) * f) ++f;
    }
    f = umin(f, ceil_div(k, k0));
    if (k > 8192 && f < 2) f = 2;
    if (k > 32768 && f < 4) f = 4;
    return f;
}

}  // namespace catcoc
