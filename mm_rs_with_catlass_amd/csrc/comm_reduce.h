// Arguments of the stand-alone comm-round, dequant and split-K reduce kernels (comm_reduce.hip).
#pragma once
#include <stdint.h>

#include "gemm_args.h"

namespace catcoc {

enum : uint32_t { CT_INT32 = 0 };   // CommArgs.dtype: CT_INT32, or DT_F16 / DT_BF16 for 16-bit blocks

struct CommArgs {
    void *local;                   // this rank's kept block [mRank, N]: int32 accumulators or 16-bit partial sums
    int64_t localLd;               // its leading dimension in elements
    const void *peers[kMaxRanks];  // the other ranks' staged blocks, slot s = rank s (s < rank) or s + 1
    int64_t peerLd, peerRowOffset;
    uint32_t P, rank;
    uint32_t mRank, N;             // extent of the kept block
    uint32_t m0, n0, loopsM, loopsN, off, dir;   // tile grid and swizzle of one rank's sub-problem
    uint32_t roundFirstIdx;        // position in that swizzle of the round's first tile
    uint32_t dataLoops;            // data blocks of this rank in the round: tiles in the round x (m0 / commBlockM)
    uint32_t commBlockM;           // rows of a comm block (divides m0)
    uint32_t splitRow, splitCol;   // CommCoreSplit (data split, npu split)
    uint32_t swizzleDir;           // BlockCommSwizzle direction (non-deterministic schedule)
    uint32_t dtype;                // CT_INT32, DT_F16 or DT_BF16
    // Deterministic int32 rounds can finish their blocks: once a core has added every rank's block the sums are final (a kept
    // tile belongs to exactly one round), so it writes the dequantised 16-bit rows next to the int32 ones and the pass after
    // all rounds falls away.  dOut NULL = leave that to the separate pass.
    void *dOut;                    // [mRank, N] 16-bit output, or NULL
    int64_t ldd;
    const float *scaleN;           // per channel, [N]
    const float *scaleM;           // per token, already at the kept block's first row
    uint32_t outDtype;             // DT_F16 / DT_BF16
    uint32_t passes;               // deterministic schedule: pieces of 256 x 4 sixteen-byte accesses a data block is cut into
};

int launch_comm_reduce(const CommArgs &a, uint32_t cores, bool deterministic, void *stream);
int launch_dequant_rows(const int32_t *acc, int64_t ldAcc, const float *scaleN, const float *scaleM, void *out, int64_t ldOut,
                        uint32_t rows, uint32_t cols, uint32_t outDtype, void *stream);
int launch_reduce_add(void *dst, const float *src, uint64_t elementCount, uint32_t slices, uint32_t outDtype, void *stream);

}  // namespace catcoc
