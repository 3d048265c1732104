// Full-tile fast path of the fused GEMM for gfx950: A and B tiles stream from
// global memory straight into LDS (no VGPR staging) three k-steps ahead of the
// MFMAs, and the row-major B tile is transposed on the way out of LDS with the
// transpose-read instruction, so the main loop issues almost nothing but LDS reads
// and MFMAs.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "gemm_fused_kernel.h"

namespace catcoc {

typedef short v4s16 __attribute__((ext_vector_type(4)));

#define CATCOC_LDS __attribute__((address_space(3)))
#define CATCOC_GLB __attribute__((address_space(1)))

// Wait until at most n of this wave's vector-memory operations (the LDS copies below) are outstanding.
#define CATCOC_WAIT_VMCNT(n) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(n) : "memory")

// Workgroup barrier that does not drain the vector-memory queue: loads that are
// still in flight for LATER stages must stay in flight across it.  The empty asm
// statements keep the compiler from moving LDS accesses across the barrier.
__device__ __forceinline__ void barrier_keep_vmem()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// 16 bytes per lane, global -> LDS, lane l lands at lds + 16*l (lds is wave-uniform).
// Issued as an asm statement on purpose: the kernel orders these copies against LDS reads itself
// (CATCOC_WAIT_VMCNT + barrier), with several stages in flight across barriers and loop iterations.
__device__ __forceinline__ void dma16(const unsigned char *g, unsigned char *lds)
{
    const uint32_t l = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(CATCOC_LDS unsigned char *)lds);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(l) : "memory", "m0");
}

// The same with the LDS destination given as a byte address that is already wave-uniform (built from scalars).
__device__ __forceinline__ void dma16_at(const unsigned char *g, uint32_t ldsAddr)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(ldsAddr) : "memory", "m0");
}

// Same as dma16 with the streaming cache hint: for data that is read exactly once.
__device__ __forceinline__ void dma16_stream(const unsigned char *g, unsigned char *lds)
{
    const uint32_t l = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(CATCOC_LDS unsigned char *)lds);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" : : "v"(g), "s"(l) : "memory", "m0");
}

// LDS layouts per stage (k step = 64 bytes of K):
//   A: [row][4 x 16-byte k chunks], chunk slot = chunk ^ ((row >> 2) & 3)            (as in gemm_fused_kernel)
//   B: raw row-major [k row][16 x 16-byte column chunks] (64 rows x 256 B),
//      column chunk slot = chunk ^ ((k row & 7) << 1); the swizzle is applied on the global side of
//      the copy, and makes the 8-row x 16-column transpose reads of a half-wave hit all 64 banks once.
//
// Geometries (every wave computes 64 x 128: MB = 2 row blocks of 32, 4 column blocks of 32; two wave columns):
//   WM 2 -> 128x256 tile, 4 waves, 3 stages (72 KiB LDS, two workgroups per CU);
//   WM 4 -> 256x256 tile, 8 waves (128 KiB LDS, one workgroup per CU): half the L2 -> LDS traffic per MAC.
//   W8   -> the 128x256 tile on EIGHT waves (four wave rows of 32 rows, MB = 1; WM stays 2: every tile-level rule of the
//           128-row geometry applies): for the six-stage ring, whose launches have one workgroup per CU -- with four waves
//           every wave is alone on its SIMD and pays barrier, LDS latency and copy issue of every k step one after the other.
//   TB   -> B is given as [n][k] (k contiguous, the layout of a weight matrix stored output-major): its tiles are then
//           staged and read exactly like A's, rows of 64 bytes of k, and need no transposing LDS reads.
//   RM   -> explicit kept rows (GF_ROW_MASK): the kept rows are whole 32-row blocks anywhere in the row range, so a tile can
//           hold kept and not-kept blocks; every per-row step of the epilogue is then decided per 32-row block of a wave
//           (wave-uniform branches, no per-lane selects).  A separate instantiation: the other launches pay nothing for it.
//   RG   -> ragged problems (GF_RAGGED): a tile with fewer than m0 valid rows or n0 valid columns is computed as a whole tile
//           moved up / left until it ends at the edge of its rank's row block / of the matrix.  Every load stays in bounds,
//           the main loop is unchanged, and the rows and columns it shares with the neighbouring tile come out bit for bit as
//           that tile computes them (same operands, same k order), so writing them twice is harmless; only what is counted
//           per task (checksums) or laid out per task (workspace stores) has to leave the overlap out.
//   TA   -> A is given as [k][m] (m contiguous): its tiles are then staged as rows of k, 128 bytes or 128 two-byte elements
//           of m each, and read with the transposing LDS reads B uses (an MFMA's A operand wants k contiguous per lane for
//           its row, exactly as its B operand does for its column).
// One LDS pool per workgroup, carved by constant offsets:
//   128-row tile: three A stages (8 KiB each), then three B stages (16 KiB each)            = 72 KiB
//   256-row tile: two A pair buffers (32 KiB each), then four B stages (16 KiB each)         = 128 KiB
//   256-row tile, B as [n][k]: two A pair buffers, then three B pair buffers (32 KiB each)   = 160 KiB, the whole LDS
// (a 64-row tile of the four-wave geometry uses the first 60 KiB of the 72)
//   128-row tile, six stages, A in pairs (AQ): four A pair buffers (16 KiB each), then six B stages = 160 KiB, the whole LDS
template <int WM, int NS = 3, bool AQ = false, bool TB = false> struct DmaPool
{
    static constexpr int BYTES = (WM == 4) ? (TB ? 5 * 256 * 128 : 4 * 256 * 64 + 4 * 64 * 256) : AQ ? ((NS / 2 + 1) * 128 * 128 + NS * 64 * 256) : NS * (128 * 64 + 64 * 256);
};

// One tile (or one k slice of a tile) of the launch: position `pos` of the launch order, in the caller's LDS pool.
// MB = 32-row blocks per wave (2; 1 = a 64-row tile of the four-wave geometry, or the eight-wave geometry W8); subRow =
// first row of a 64-row tile inside its 128-row tile of the schedule.
// AQ = A is copied per pair of k steps, 128 bytes per row (whole cache lines: half as many requests to L2 as two 64-byte
// halves), as the 256-row geometry does; for the six-stage ring, whose launches have one workgroup per CU and feel every
// request (with three stages and two workgroups per CU the same change measured slower).
template <uint32_t DT, int WM, bool TB, bool RM, bool RG, bool TA, int MB, int NS = 3, bool PP = false, bool AQ = false, bool W8 = false>
__device__ __forceinline__ void dma_tile(const GemmArgs &args, unsigned char *smem, uint32_t pos, uint32_t slice, uint32_t kSlices,
                                         uint32_t subRow)
{
    static_assert(!RM || (DT == DT_I8 && WM == 2), "row-mask mode exists for the W8A8 128-row kernel");
    static_assert(!RG || !RM, "ragged mode and row-mask mode exclude each other");
    static_assert(!TA || (WM == 2 && !RM), "transposed A exists for the 128-row kernel");
    static_assert(WM == 2 || WM == 4, "supported geometries");
    static_assert(NS == 3 || (WM == 2 && NS >= 3 && NS <= 8), "deeper rings exist for the 128-row kernel");
    static_assert(MB == 2 || (MB == 1 && WM == 2 && (!RM || W8) && !RG && !TA), "64-row tiles exist for the four-wave geometry with A as [m,k]");
    static_assert(!W8 || (WM == 2 && MB == 1 && !RG && !TA), "eight waves on the 128-row tile: 32 rows per wave");
    static_assert(!AQ || (WM == 2 && NS == 6 && (MB == 2 || W8) && !TA), "pairs of A steps exist for the six-stage 128-row kernel with A as [m,k]");
    using Acc = typename AccOf<DT>::type;
    constexpr int ES = (DT == DT_I8) ? 1 : 2;   // bytes per operand element; a k step is 64 BYTES of K
    constexpr int WR = W8 ? 4 : WM;     // wave rows (two wave columns)
    constexpr int NW = 2 * WR;          // waves
    constexpr int NT = 64 * NW;         // threads
    constexpr int BM = 32 * MB * WR;
    constexpr bool HALF = MB == 1 && !W8;   // a 64-row half of a 128-row tile of the schedule
    constexpr int A_STAGE = BM * 64;
    constexpr int B_STAGE = 64 * 256;
    constexpr int A_DMA = BM / 16 / NW;  // 1 KiB copies per wave per stage
    constexpr int B_DMA = 16 / NW;
    constexpr int STEP_DMA = A_DMA + B_DMA;
    constexpr int POOL = DmaPool<WM, NS, AQ, TB>::BYTES;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = tid >> 6;
    const int wm = w >> 1, wn = w & 1;
    const int c32 = lane & 31, h = lane >> 5;

    const SchedParams &sp = args.sched;
    // the launch constants are all needed within the next few hundred instructions: naming them here lets the compiler
    // fetch them as a few wide scalar loads instead of one load and one wait per use
    asm volatile("" : : "s"(sp.xOk), "s"(sp.xRxLog), "s"(sp.xCxLog), "s"(sp.xRowsPer), "s"(sp.xColsPer), "s"(sp.xPerRank),
                 "s"(sp.xCommLoops), "s"(sp.xLastPerRank), "s"(sp.coreLoops), "s"(sp.loopsM), "s"(sp.loopsN), "s"(sp.blockPerComm),
                 "s"(sp.m0), "s"(sp.n0), "s"(sp.mRank), "s"(sp.off));
    asm volatile("" : : "s"(sp.dColsPer.d), "s"(sp.dColsPer.m), "s"(sp.dLoopsM.d), "s"(sp.dLoopsM.m), "s"(sp.dBand.d), "s"(sp.dBand.m),
                 "s"(sp.dPerRank.d), "s"(sp.dPerRank.m), "s"(sp.dStages.d), "s"(sp.dStages.m), "s"(sp.dBpc.d), "s"(sp.dBpc.m),
                 "s"(args.keptRank), "s"(args.flags), "s"(args.K), "s"(args.N));
    const bool linear = (args.flags & GF_LINEAR_ORDER) != 0;
    if (pos >= sp.coreLoops) return;
    uint32_t task;
    TileInfo ti;
    if (!linear && sp.xOk) {
        xcd_launch_tile(sp, args.keptRank, pos, task, ti);
    } else {
        task = launch_task(sp, pos, linear, args.keptRank);
        TileInfo tg;   // (a separate object: filled in place, the tile of both routes ends up in memory instead of registers)
        task_tile(sp, task, tg);
        ti = tg;
    }
    if constexpr (HALF) {
        ti.row += subRow;
        ti.rowInRank += subRow;
        ti.wsRow += subRow;
    }
    uint32_t shiftM = 0, shiftN = 0;   // RG: rows / columns at the start of the tile that belong to the neighbouring tile
    if constexpr (RG) {
        shiftM = sp.m0 - ti.rowsValid;
        shiftN = sp.n0 - ti.colsValid;
        ti.row -= shiftM;
        ti.rowInRank -= shiftM;
        ti.col -= shiftN;
    }
    // The kept tiles are the longest chain of a reduce-scatter launch (main loop, then the peers' partials):
    // their waves get priority over the other workgroup on the CU so that the chain starts its streaming early.
    if (sp.op == OP_REDUCE_SCATTER && sp.P > 1 && ti.row >= args.keptBegin && ti.row < args.keptBegin + args.keptRows)
        __builtin_amdgcn_s_setprio(3);

    const int64_t ldaB = args.lda * ES, ldbB = args.ldb * ES;  // row pitches in bytes
    const bool gather = sp.op == OP_ALLGATHER;
    const unsigned char *Ag = (const unsigned char *)args.a[gather ? ti.targetRank : 0] +
                              (TA ? (int64_t)(gather ? ti.rowInRank : ti.row) * ES : (int64_t)(gather ? ti.rowInRank : ti.row) * ldaB);
    const unsigned char *Bg = (const unsigned char *)args.b + (TB ? (size_t)ti.col * ldbB : (size_t)ti.col * ES);
    // k steps (64 bytes of K each) of this workgroup: all of them, or its slice
    const uint32_t nkAll = args.K * ES / 64;
    uint32_t nk = nkAll;
    if (kSlices > 1) {   // (at most 16 slices of fewer than 2^24 steps: 32-bit products)
        const uint32_t kFirst = nkAll * slice / kSlices;
        nk = nkAll * (slice + 1u) / kSlices - kFirst;
        Ag += TA ? (size_t)kFirst * (64 / ES) * ldaB : (size_t)kFirst * 64;
        Bg += TB ? (size_t)kFirst * 64 : (size_t)kFirst * (64 / ES) * ldbB;
    }

    // ---- copy descriptors ---------------------------------------------------
    // Every copy a wave issues has its own global pointer, advanced after each issue, and a scalar LDS address:
    // issuing a copy is then a pointer add, an M0 write and the load.  Steps are issued in increasing order.
    const uint32_t ws = __builtin_amdgcn_readfirstlane((uint32_t)w);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(CATCOC_LDS unsigned char *)smem;
    // A (128-row tiles): copy j covers rows 16j..16j+15; lane -> row 16j + lane/4, LDS chunk slot lane&3 holds k chunk slot^swz
    // A given as [k][m], 1-byte elements (64 k rows x 128 bytes): copy j covers k rows 8j..8j+7; lane -> row 8j + lane/8, slot
    // lane&7 holds chunk slot ^ (((row>>1)&3)<<1).  2-byte elements (32 k rows x 256 bytes): copy j covers k rows 4j..4j+3;
    // lane -> row 4j + lane/16, slot lane&15 holds chunk slot ^ ((row&3)<<2).
    const unsigned char *gA[A_DMA];
#pragma unroll
    for (int jj = 0; jj < A_DMA; ++jj) {
        if constexpr (!TA) {
            gA[jj] = Ag + (size_t)(16 * (w + NW * jj) + (lane >> 2)) * ldaB + (((lane & 3) ^ ((lane >> 4) & 3)) * 16);
        } else if constexpr (ES == 1) {
            const int row = 8 * (w + NW * jj) + (lane >> 3);
            gA[jj] = Ag + (size_t)row * ldaB + (((lane & 7) ^ (((row >> 1) & 3) << 1)) * 16);
        } else {
            const int row = 4 * (w + NW * jj) + (lane >> 4);
            gA[jj] = Ag + (size_t)row * ldaB + (((lane & 15) ^ ((row & 3) << 2)) * 16);
        }
    }
    const size_t aStep = TA ? (size_t)(64 / ES) * ldaB : (size_t)64;
    auto issue_a = [&](uint32_t ldsStage) {   // next k step of A into the stage at LDS byte offset ldsStage
#pragma unroll
        for (int jj = 0; jj < A_DMA; ++jj) {
            dma16_at(gA[jj], lds0 + ldsStage + (ws + NW * jj) * 1024);
            gA[jj] += aStep;
        }
    };
    // B, 1-byte elements: copy j covers k rows 4j..4j+3; lane -> row 4j + lane/16, LDS slot lane&15 holds column
    // chunk slot^((row&7)<<1).  2-byte elements (32 k rows x 512 bytes): copy j covers k rows 2j, 2j+1; lane -> row
    // 2j + lane/32, slot lane&31 holds chunk slot^((row&3)<<2).
    // B given as [n][k]: copy j covers tile columns 16j..16j+15, one 64-byte row of k each, laid out like A.
    const unsigned char *gB[B_DMA];
#pragma unroll
    for (int jj = 0; jj < B_DMA; ++jj) {
        if constexpr (TB) {
            gB[jj] = Bg + (size_t)(16 * (w + NW * jj) + (lane >> 2)) * ldbB + (((lane & 3) ^ ((lane >> 4) & 3)) * 16);
        } else if constexpr (ES == 1) {
            const int row = 4 * (w + NW * jj) + (lane >> 4);
            gB[jj] = Bg + (size_t)row * ldbB + (((lane & 15) ^ ((row & 7) << 1)) * 16);
        } else {
            const int row = 2 * (w + NW * jj) + (lane >> 5);
            gB[jj] = Bg + (size_t)row * ldbB + (((lane & 31) ^ ((row & 3) << 2)) * 16);
        }
    }
    const size_t bStep = TB ? (size_t)64 : (size_t)(64 / ES) * ldbB;
    auto issue_b = [&](uint32_t ldsStage) {   // next k step of B
#pragma unroll
        for (int jj = 0; jj < B_DMA; ++jj) {
            dma16_at(gB[jj], lds0 + ldsStage + (ws + NW * jj) * 1024);
            gB[jj] += bStep;
        }
    };

    Acc acc[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][nb][r] = 0;

    // fragment addresses
    // 1-byte transpose read: within a 16-lane group, lane i supplies 8 bytes of k row (i>>1), column half (i&1)
    // of a 16-column chunk, and receives column i of the chunk for 8 consecutive k rows.
    // 2-byte transpose read: lane i supplies 4 elements of k row (i>>2), column quad (i&3) of a 16-column (32-byte)
    // chunk pair, and receives column i for 4 consecutive k rows.  Two reads make the 16 bytes of k a lane feeds
    // the MFMA with; groups 0/1 of a half-wave take the two 16-column halves of a 32-column block, the upper
    // half-wave the upper half of the k slab.
    const int ti16 = lane & 15, tch = (lane >> 4) & 1;
    uint32_t b_lds[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
        if constexpr (ES == 1) {
            const int trow = ti16 >> 1, thalf = ti16 & 1;
            const int q = wn * 8 + nb * 2 + tch;
            b_lds[nb] = (16 * h + trow) * 256 + ((q ^ (2 * trow)) * 16) + thalf * 8;
        } else {
            const int trow = ti16 >> 2, tq = ti16 & 3;
            const int q = wn * 16 + nb * 4 + tch * 2 + (tq >> 1);
            b_lds[nb] = (8 * h + trow) * 512 + ((q ^ (trow << 2)) * 16) + (tq & 1) * 8;
        }
    }
    constexpr int B_KK = (ES == 1) ? 32 * 256 : 16 * 512;     // bytes of a stage per 32-byte k slab
    constexpr int B_HALF = (ES == 1) ? 8 * 256 : 4 * 512;     // second transpose read of a fragment
    const uint32_t bt_lds = (wn * 128 + c32) * 64, bt_sw = (c32 >> 2) & 3;   // [n][k] stage: row of column c32, chunk swizzle
    // 256-row tile with B as [n][k]: B sits in pair buffers like A (rows of 128 bytes, two k steps); bpar = step of the pair
    uint32_t bpar = 0;
    const uint32_t bp4_lds = (wn * 128 + c32) * 128, bp4_sw = (c32 >> 1) & 7;
    auto read_b1 = [&](v4i (&bf)[4], const unsigned char *sb, int kk, int nb) {
        if constexpr (TB && WM == 4) {
            bf[nb] = *(const v4i *)(sb + bp4_lds + nb * 32 * 128 + (((bpar * 4 + 2 * kk + h) ^ bp4_sw) * 16));
            return;
        }
        if constexpr (TB) {
            bf[nb] = *(const v4i *)(sb + bt_lds + nb * 32 * 64 + (((2 * kk + h) ^ bt_sw) * 16));
            return;
        }
        const unsigned char *p = sb + b_lds[nb] + kk * B_KK;
        v2i t0, t1;
        if constexpr (ES == 1) {
            t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)p);
            t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)(p + B_HALF));
        } else {
            t0 = __builtin_bit_cast(v2i, __builtin_amdgcn_ds_read_tr16_b64_v4i16((CATCOC_LDS v4s16 *)p));
            t1 = __builtin_bit_cast(v2i, __builtin_amdgcn_ds_read_tr16_b64_v4i16((CATCOC_LDS v4s16 *)(p + B_HALF)));
        }
        bf[nb] = v4i{t0.x, t0.y, t1.x, t1.y};
    };
    auto load_b = [&](v4i (&bf)[4], const unsigned char *sb, int kk) {
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) read_b1(bf, sb, kk, nb);
    };
    auto mma = [&](const v4i (&af)[MB], const v4i (&bf)[4]) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) acc[mb][nb] = mfma32<DT>(af[mb], bf[nb], acc[mb][nb]);
    };

    // One k step, hand-scheduled: the 16 MFMAs of a wave are issued back to back, and every other
    // instruction of the step (fragment reads for the NEXT eight MFMAs, the copies for later steps)
    // sits between two MFMAs, where it issues while the matrix pipe is busy.  The first
    // eight MFMAs finish the previous step (fragments fa1/fb1, read during the previous step), the second
    // eight use fa0/fb0 read during the first eight; the MFMAs lag the fragment reads by half a step, so
    // LDS latency is never exposed.  The fences keep the compiler from regrouping the sequence.
    v4i fa0[MB], fb0[4], fa1[MB], fb1[4];
#define CATCOC_FENCE() __builtin_amdgcn_sched_barrier(0)
#define CATCOC_MMA(FA, FB, MBI, NBI)                                              \
    acc[MBI][NBI] = mfma32<DT>(FA[MBI], FB[NBI], acc[MBI][NBI]);                  \
    CATCOC_FENCE();
    // read_a(af, kk): A fragments of this step; sb: B stage of this step; slot1/2/3/4: the step's other work
    auto sched_step = [&](auto read_a, const unsigned char *sb, auto slot1, auto slot2, auto slot3, auto slot4) {
        if constexpr (MB == 1) {   // eight MFMAs per step: the same lag of half a step, two reads per gap
            CATCOC_MMA(fa1, fb1, 0, 0)
            read_a(fa0, 0);
            read_b1(fb0, sb, 0, 0);
            CATCOC_FENCE();
            CATCOC_MMA(fa1, fb1, 0, 1)
            read_b1(fb0, sb, 0, 1);
            read_b1(fb0, sb, 0, 2);
            CATCOC_FENCE();
            CATCOC_MMA(fa1, fb1, 0, 2)
            read_b1(fb0, sb, 0, 3);
            slot1();
            CATCOC_FENCE();
            CATCOC_MMA(fa1, fb1, 0, 3)
            slot2();
            slot3();
            CATCOC_FENCE();
            CATCOC_MMA(fa0, fb0, 0, 0)
            read_a(fa1, 1);
            read_b1(fb1, sb, 1, 0);
            CATCOC_FENCE();
            CATCOC_MMA(fa0, fb0, 0, 1)
            read_b1(fb1, sb, 1, 1);
            read_b1(fb1, sb, 1, 2);
            CATCOC_FENCE();
            CATCOC_MMA(fa0, fb0, 0, 2)
            read_b1(fb1, sb, 1, 3);
            slot4();
            CATCOC_FENCE();
            CATCOC_MMA(fa0, fb0, 0, 3)
        } else {
        CATCOC_MMA(fa1, fb1, 0, 0)
        read_a(fa0, 0);
        CATCOC_FENCE();
        CATCOC_MMA(fa1, fb1, 1, 0)
        read_b1(fb0, sb, 0, 0);
        CATCOC_FENCE();
        CATCOC_MMA(fa1, fb1, 0, 1)
        read_b1(fb0, sb, 0, 1);
        CATCOC_FENCE();
        CATCOC_MMA(fa1, fb1, 1, 1)
        read_b1(fb0, sb, 0, 2);
        CATCOC_FENCE();
        CATCOC_MMA(fa1, fb1, 0, 2)
        read_b1(fb0, sb, 0, 3);
        CATCOC_FENCE();
        CATCOC_MMA(fa1, fb1, 1, 2)
        slot1();
        CATCOC_FENCE();
        CATCOC_MMA(fa1, fb1, 0, 3)
        slot2();
        CATCOC_FENCE();
        CATCOC_MMA(fa1, fb1, 1, 3)
        slot3();
        CATCOC_FENCE();
        CATCOC_MMA(fa0, fb0, 0, 0)
        read_a(fa1, 1);
        CATCOC_FENCE();
        CATCOC_MMA(fa0, fb0, 1, 0)
        read_b1(fb1, sb, 1, 0);
        CATCOC_FENCE();
        CATCOC_MMA(fa0, fb0, 0, 1)
        read_b1(fb1, sb, 1, 1);
        CATCOC_FENCE();
        CATCOC_MMA(fa0, fb0, 1, 1)
        read_b1(fb1, sb, 1, 2);
        CATCOC_FENCE();
        CATCOC_MMA(fa0, fb0, 0, 2)
        read_b1(fb1, sb, 1, 3);
        CATCOC_FENCE();
        CATCOC_MMA(fa0, fb0, 1, 2)
        slot4();
        CATCOC_FENCE();
        CATCOC_MMA(fa0, fb0, 0, 3)
        CATCOC_MMA(fa0, fb0, 1, 3)
        }
    };
#undef CATCOC_MMA
    auto nothing = [] {};

    if constexpr (WM == 2 && AQ) {
        // ---- NS B stages, NS / 2 + 1 A pair buffers.  B runs NS - 1 steps ahead as in the plain ring; pair q (steps 2q,
        // 2q + 1) is issued at step 2q - NS into buffer q mod (NS / 2 + 1), which pair q - NS / 2 - 1 left before that
        // step's barrier.  Copies a wave issues in step kt, in this order: B(kt + NS - 1), then on even kt the pair
        // (kt + NS) / 2; the prologue issues what the steps -NS .. -1 would have.  The vector-memory counter retires in
        // order, so at the barrier of step s everything issued after B(s) may still be in flight: the B copies of the NS - 2
        // steps after s and the pairs issued at the even steps s - (NS - 1) .. s - 1 (three of them when s is odd, two when
        // it is even), fewer towards the end of the k range.  A pair and a B step are the same number of copies per wave.
        constexpr int NPB = NS / 2 + 1;
        constexpr int AP = BM * 128;
        constexpr int APC = BM / 8 / NW;
        static_assert(APC == B_DMA, "the waits count pairs and B steps in one unit");
        static_assert(NPB * AP + NS * B_STAGE <= POOL, "pair buffers and B stages fit the pool");
        static_assert((NS - 2 + NS / 2) * B_DMA <= 63, "the wait counter holds 63");
        auto stB = [&](uint32_t st) { return smem + NPB * AP + st * B_STAGE; };
        auto offB = [&](uint32_t st) { return NPB * AP + st * B_STAGE; };
        // pair copy j covers rows 8j..8j+7: lane -> row 8j + lane/8, slot lane&7 holds chunk slot ^ ((row>>1)&7)
        const unsigned char *gP[APC];
#pragma unroll
        for (int jj = 0; jj < APC; ++jj) {
            const int row = 8 * (w + NW * jj) + (lane >> 3);
            gP[jj] = Ag + (size_t)row * ldaB + (((lane & 7) ^ ((row >> 1) & 7)) * 16);
        }
        auto issue_ap = [&](uint32_t q) {   // pairs are issued in increasing q
#pragma unroll
            for (int jj = 0; jj < APC; ++jj) {
                dma16_at(gP[jj], lds0 + (q % NPB) * AP + (ws + NW * jj) * 1024);
                gP[jj] += 128;
            }
        };
        const uint32_t ap_lds = (wm * 32 * MB + c32) * 128;
        const uint32_t ap_sw = (c32 >> 1) & 7;
        auto load_ap = [&](v4i (&af)[MB], uint32_t kt, int kk) {
            const unsigned char *sa = smem + ((kt >> 1) % NPB) * AP + ap_lds + ((((kt & 1) * 4 + 2 * kk + h) ^ ap_sw) * 16);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) af[mb] = *(const v4i *)(sa + mb * 32 * 128);
        };
        auto wait_units = [&](uint32_t n) {   // at most n x B_DMA copies (the youngest) outstanding
            switch (n) {
                case 0: CATCOC_WAIT_VMCNT(0); break;
                case 1: CATCOC_WAIT_VMCNT(1 * B_DMA); break;
                case 2: CATCOC_WAIT_VMCNT(2 * B_DMA); break;
                case 3: CATCOC_WAIT_VMCNT(3 * B_DMA); break;
                case 4: CATCOC_WAIT_VMCNT(4 * B_DMA); break;
                case 5: CATCOC_WAIT_VMCNT(5 * B_DMA); break;
                case 6: CATCOC_WAIT_VMCNT(6 * B_DMA); break;
                default: CATCOC_WAIT_VMCNT(7 * B_DMA); break;
            }
        };
        auto units_after = [&](uint32_t s) {   // B steps and pairs issued after B(s) by the time step s starts
            const uint32_t nB = umin((uint32_t)(NS - 2), nk - 1u - s);
            // pairs: issued at the even (possibly virtual, negative) steps t with s - (NS - 1) <= t <= min(s - 1, nk - NS - 2);
            // counted with t shifted by NS + 2, which keeps the parity and makes every term non-negative
            const uint32_t lo = s + 3u, hiA = s + (uint32_t)NS + 1u, hiB = nk;
            const uint32_t hi = umin(hiA, hiB);
            const uint32_t nP = hi >= lo ? (hi >> 1) - ((lo + 1u) >> 1) + 1u : 0u;
            return nB + nP;
        };
        // the prologue: what the steps -NS .. -1 would have issued
#pragma unroll
        for (int v = -NS; v < 0; ++v) {
            if (v + NS - 1 >= 0 && (uint32_t)(v + NS - 1) < nk) issue_b(offB(v + NS - 1));
            if ((v & 1) == 0 && (uint32_t)(v + NS + 2) <= nk) issue_ap((uint32_t)(v + NS) >> 1);
        }
        // step 0 (peeled: no MFMAs pending yet)
        wait_units(units_after(0));
        barrier_keep_vmem();
        if ((uint32_t)(NS - 1) < nk) issue_b(offB(NS - 1));
        if ((uint32_t)(NS + 2) <= nk) issue_ap(NS >> 1);
        load_ap(fa0, 0, 0);
        load_b(fb0, stB(0), 0);
        load_ap(fa1, 0, 1);
        load_b(fb1, stB(0), 1);
        CATCOC_FENCE();
        mma(fa0, fb0);
        CATCOC_FENCE();
        // step kt reads B stage kt % NS and refills stage (kt - 1) % NS with B(kt + NS - 1)
        uint32_t kt = 1, cur = 1, nxt = 0;
        auto step = [&]() {
            const uint32_t k = kt;
            const bool moreB = k + (uint32_t)(NS - 1) < nk, moreP = (k & 1u) == 0 && k + (uint32_t)(NS + 2) <= nk;
            sched_step([&](v4i (&af)[MB], int kk) { load_ap(af, k, kk); }, stB(cur), [&] { if (moreB) issue_b(offB(nxt)); },
                       [&] { if (moreP) issue_ap((k + (uint32_t)NS) >> 1); }, nothing, nothing);
            ++kt;
            cur = cur == NS - 1 ? 0 : cur + 1;
            nxt = nxt == NS - 1 ? 0 : nxt + 1;
        };
        while (kt + (uint32_t)(NS + 2) <= nk) {   // kt is odd here: an odd and an even step in full flight
            CATCOC_WAIT_VMCNT((NS - 2 + NS / 2) * B_DMA);
            barrier_keep_vmem();
            step();
            CATCOC_WAIT_VMCNT((NS - 3 + NS / 2) * B_DMA);
            barrier_keep_vmem();
            step();
        }
        while (kt < nk) {
            wait_units(units_after(kt));
            barrier_keep_vmem();
            step();
        }
        mma(fa1, fb1);
    } else if constexpr (WM == 2) {
        // ---- NS stages, copies run NS - 1 k steps ahead.  NS = 3: 72 KiB LDS, two workgroups per CU, for operands that come
        // out of L2 or the Infinity Cache.  NS = 6: 144 KiB, one workgroup per CU, 120 KiB in flight per CU: for launches of at
        // most one workgroup per CU anyway, whose operands stream from HBM (two steps ahead do not cover that latency) ----
        auto stA = [&](uint32_t st) { return smem + st * A_STAGE; };
        auto stB = [&](uint32_t st) { return smem + NS * A_STAGE + st * B_STAGE; };
        auto offA = [&](uint32_t st) { return st * A_STAGE; };
        auto offB = [&](uint32_t st) { return NS * A_STAGE + st * B_STAGE; };
        // wait until at most r whole steps of copies (the youngest) are outstanding, r < NS - 1
        auto wait_steps = [&](uint32_t r) {
            if constexpr (NS == 3) {
                if (r) CATCOC_WAIT_VMCNT(STEP_DMA);
                else CATCOC_WAIT_VMCNT(0);
            } else {
                switch (r) {
                    case 0: CATCOC_WAIT_VMCNT(0); break;
                    case 1: CATCOC_WAIT_VMCNT(STEP_DMA); break;
                    case 2: CATCOC_WAIT_VMCNT(2 * STEP_DMA); break;
                    case 3: CATCOC_WAIT_VMCNT(3 * STEP_DMA); break;
                    case 4: CATCOC_WAIT_VMCNT((NS > 5 ? 4 : 0) * STEP_DMA); break;
                    case 5: CATCOC_WAIT_VMCNT((NS > 6 ? 5 : 0) * STEP_DMA); break;
                    default: CATCOC_WAIT_VMCNT((NS > 7 ? 6 : 0) * STEP_DMA); break;
                }
            }
        };
        static_assert((NS - 2) * STEP_DMA <= 63, "the wait counter holds 63");
        const uint32_t a_lds = (wm * 32 * MB + c32) * 64;
        const uint32_t a_sw = (c32 >> 2) & 3;
        // A as [k][m]: the transposing reads of B, with this wave's 32-row blocks in place of 32-column blocks
        uint32_t at_lds[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            if constexpr (ES == 1) {
                const int trow = ti16 >> 1, thalf = ti16 & 1;
                const int q = wm * 2 * MB + mb * 2 + tch;
                at_lds[mb] = (16 * h + trow) * 128 + ((q ^ (((trow >> 1) & 3) << 1)) * 16) + thalf * 8;
            } else {
                const int trow = ti16 >> 2, tq = ti16 & 3;
                const int q = wm * 4 * MB + mb * 4 + tch * 2 + (tq >> 1);
                at_lds[mb] = (8 * h + trow) * 256 + ((q ^ (trow << 2)) * 16) + (tq & 1) * 8;
            }
        }
        constexpr int AT_KK = (ES == 1) ? 32 * 128 : 16 * 256;   // bytes of a stage per 32-byte k slab
        constexpr int AT_HALF = (ES == 1) ? 8 * 128 : 4 * 256;   // second transpose read of a fragment
        auto load_a = [&](v4i (&af)[MB], const unsigned char *sa, int kk) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                if constexpr (!TA) {
                    af[mb] = *(const v4i *)(sa + a_lds + mb * 32 * 64 + (((2 * kk + h) ^ a_sw) * 16));
                } else {
                    const unsigned char *p = sa + at_lds[mb] + kk * AT_KK;
                    v2i t0, t1;
                    if constexpr (ES == 1) {
                        t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)p);
                        t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)(p + AT_HALF));
                    } else {
                        t0 = __builtin_bit_cast(v2i, __builtin_amdgcn_ds_read_tr16_b64_v4i16((CATCOC_LDS v4s16 *)p));
                        t1 = __builtin_bit_cast(v2i, __builtin_amdgcn_ds_read_tr16_b64_v4i16((CATCOC_LDS v4s16 *)(p + AT_HALF)));
                    }
                    af[mb] = v4i{t0.x, t0.y, t1.x, t1.y};
                }
            }
        };
#pragma unroll
        for (int st = 0; st < NS - 1; ++st)
            if (nk > (uint32_t)st) {
                issue_a(offA(st));
                issue_b(offB(st));
            }
        // step 0 (peeled: no MFMAs pending yet)
        wait_steps(umin(NS - 2, nk - 1));
        barrier_keep_vmem();
        if (nk > NS - 1) {
            issue_a(offA(NS - 1));
            issue_b(offB(NS - 1));
        }
        load_a(fa0, stA(0), 0);
        load_b(fb0, stB(0), 0);
        load_a(fa1, stA(0), 1);
        load_b(fb1, stB(0), 1);
        CATCOC_FENCE();
        mma(fa0, fb0);
        CATCOC_FENCE();
        // step kt reads stage kt % NS and refills stage (kt - 1) % NS, which every wave left at the barrier
        uint32_t kt = 1, cur = 1, nxt = 0;
        auto step = [&](bool more) {
            const unsigned char *sa = stA(cur);
            sched_step([&](v4i (&af)[MB], int kk) { load_a(af, sa, kk); }, stB(cur),
                       [&] { if (more) issue_a(offA(nxt)); }, [&] { if (more) issue_b(offB(nxt)); }, nothing, nothing);
            ++kt;
            cur = cur == NS - 1 ? 0 : cur + 1;
            nxt = nxt == NS - 1 ? 0 : nxt + 1;
        };
        while (kt + (NS - 1) < nk) {
            CATCOC_WAIT_VMCNT((NS - 2) * STEP_DMA);
            barrier_keep_vmem();
            step(true);
        }
        while (kt < nk) {
            wait_steps(nk - 1 - kt);
            barrier_keep_vmem();
            step(false);
        }
        mma(fa1, fb1);
    } else if constexpr (TB) {
        // ---- 256x256, B as [n][k] ---------------------------------------------------------------------
        // Both operands are rows of k: both sit in pair buffers (256 rows x 128 bytes = two k steps, whole 128-byte lines per
        // row), A in two of them, B in three.  Copies are issued at even steps only, after the barrier, in this order:
        // A pair (kt+2)/2, then B pair (kt+4)/2 -- B runs a pair further ahead.  The barrier of an even step s needs A pair
        // s/2 (issued in step s-2) and B pair s/2 (in step s-4): younger than both are only the copies of B pair s/2+1.
        // Odd steps issue nothing, read the buffers their even step waited for and need neither wait nor barrier.
        // (K in whole pairs of steps: the host requires k * element size to be a multiple of 128.)
        constexpr int AP = 256 * 128;   // bytes of a pair buffer
        constexpr int APC = 32 / NW;    // pair copies per wave and operand
        auto stAP = [&](uint32_t q) { return smem + (q & 1) * AP; };
        auto stBP = [&](uint32_t q) { return smem + 2 * AP + (q % 3u) * AP; };
        // pair copy j covers rows 8j..8j+7: lane -> row 8j + lane/8, slot lane&7 holds chunk slot ^ ((row>>1)&7)
        const unsigned char *gP[APC], *gQ[APC];
#pragma unroll
        for (int jj = 0; jj < APC; ++jj) {
            const int row = 8 * (w + NW * jj) + (lane >> 3);
            gP[jj] = Ag + (size_t)row * ldaB + (((lane & 7) ^ ((row >> 1) & 7)) * 16);
            gQ[jj] = Bg + (size_t)row * ldbB + (((lane & 7) ^ ((row >> 1) & 7)) * 16);
        }
        auto issue_ap = [&](uint32_t q) {   // pairs are issued in increasing q
#pragma unroll
            for (int jj = 0; jj < APC; ++jj) {
                dma16_at(gP[jj], lds0 + (q & 1) * AP + (ws + NW * jj) * 1024);
                gP[jj] += 128;
            }
        };
        auto issue_bp = [&](uint32_t q) {
#pragma unroll
            for (int jj = 0; jj < APC; ++jj) {
                dma16_at(gQ[jj], lds0 + 2 * AP + (q % 3u) * AP + (ws + NW * jj) * 1024);
                gQ[jj] += 128;
            }
        };
        const uint32_t ap_lds = (wm * 32 * MB + c32) * 128;
        const uint32_t ap_sw = (c32 >> 1) & 7;
        auto load_ap = [&](v4i (&af)[MB], uint32_t kt, int kk) {
            const unsigned char *sa = stAP(kt >> 1) + ap_lds + ((((kt & 1) * 4 + 2 * kk + h) ^ ap_sw) * 16);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) af[mb] = *(const v4i *)(sa + mb * 32 * 128);
        };
        auto issue_even_a = [&](uint32_t kt, bool guard) {
            if ((kt & 1) == 0 && (!guard || kt + 2 < nk)) issue_ap((kt + 2) >> 1);
        };
        auto issue_even_b = [&](uint32_t kt, bool guard) {
            if ((kt & 1) == 0 && (!guard || kt + 4 < nk)) issue_bp((kt + 4) >> 1);
        };
        // prologue in steady-state order: A pair 0, B pairs 0 and 1
        issue_ap(0);
        issue_bp(0);
        if (nk > 2) issue_bp(1);
        // step 0 (peeled: no MFMAs pending yet)
        if (nk > 2) CATCOC_WAIT_VMCNT(APC);
        else CATCOC_WAIT_VMCNT(0);
        barrier_keep_vmem();
        issue_even_a(0, true);
        issue_even_b(0, true);
        bpar = 0;
        load_ap(fa0, 0, 0);
        load_b(fb0, stBP(0), 0);
        load_ap(fa1, 0, 1);
        load_b(fb1, stBP(0), 1);
        CATCOC_FENCE();
        mma(fa0, fb0);
        CATCOC_FENCE();

        auto compute = [&](uint32_t kt, bool guard) {
            // The two waves that share a SIMD (w and w + 4) issue their copies in different halves of the step,
            // so that one of them always has MFMAs to feed the matrix pipe while the other computes addresses.
            const bool early = ws < NW / 2;
            bpar = kt & 1u;
            sched_step([&](v4i (&af)[MB], int kk) { load_ap(af, kt, kk); }, stBP(kt >> 1),
                       [&] { if (early) issue_even_a(kt, guard); }, [&] { if (early) issue_even_b(kt, guard); }, nothing,
                       [&] {
                           if (!early) {
                               issue_even_a(kt, guard);
                               issue_even_b(kt, guard);
                           }
                       });
        };
        uint32_t kt = 1;
        for (; kt + 6 <= nk; kt += 2) {   // (the even step kt + 1 issues A pair (kt+3)/2 and B pair (kt+5)/2 unguarded)
            compute(kt, false);
            CATCOC_WAIT_VMCNT(APC);
            barrier_keep_vmem();
            compute(kt + 1, false);
        }
        for (; kt < nk; ++kt) {   // tail: drain fully at every even step
            if ((kt & 1u) == 0) {
                CATCOC_WAIT_VMCNT(0);
                barrier_keep_vmem();
            }
            compute(kt, true);
        }
        mma(fa1, fb1);
    } else {
        // ---- 256x256 ---------------------------------------------------------------------------------
        // B: four 64-row stages, copies issued three steps ahead.  A: two "pair" buffers of 256 rows x 128
        // bytes (two k steps, whole 128-byte lines per row), pair q = steps 2q, 2q+1, issued at step 2q-2.
        // The MFMAs lag the fragment reads by half a step: after the barrier of step kt the fragments of
        // (kt, kk=0) are read while the MFMAs of (kt-1, kk=1) run, so LDS latency is never exposed and a
        // stage only has to have landed at its own barrier.
        // Copies a wave issues in step kt, in this order: B(kt+3) [B_DMA], then on even kt the A pair (kt+2)/2
        // [APC].  The vector-memory counter retires in order, so "at most n outstanding" at the barrier of step
        // s means everything older than the last n copies has landed:
        //   even s needs A pair s/2 (issued in step s-2): younger are the copies of step s-1;
        //   odd s needs B(s) (issued in step s-3): younger are all of steps s-2 and s-1.
        constexpr int AP = 256 * 128;   // bytes of an A pair buffer
        constexpr int APC = 32 / NW;    // pair copies per wave
        constexpr int WAIT_EVEN = B_DMA;
        constexpr int WAIT_ODD = B_DMA + (B_DMA + APC);
        auto stAP = [&](uint32_t q) { return smem + (q & 1) * AP; };
        auto stB = [&](uint32_t step) { return smem + 2 * AP + (step & 3) * B_STAGE; };
        // pair copy j covers rows 8j..8j+7: lane -> row 8j + lane/8, slot lane&7 holds chunk slot ^ ((row>>1)&7)
        const unsigned char *gP[APC];
#pragma unroll
        for (int jj = 0; jj < APC; ++jj) {
            const int row = 8 * (w + NW * jj) + (lane >> 3);
            gP[jj] = Ag + (size_t)row * ldaB + (((lane & 7) ^ ((row >> 1) & 7)) * 16);
        }
        auto issue_ap = [&](uint32_t q) {   // pairs are issued in increasing q
#pragma unroll
            for (int jj = 0; jj < APC; ++jj) {
                dma16_at(gP[jj], lds0 + (q & 1) * AP + (ws + NW * jj) * 1024);
                gP[jj] += 128;
            }
        };
        auto offB4 = [&](uint32_t step) { return 2 * AP + (step & 3) * B_STAGE; };
        const uint32_t ap_lds = (wm * 32 * MB + c32) * 128;
        const uint32_t ap_sw = (c32 >> 1) & 7;
        auto load_ap = [&](v4i (&af)[MB], uint32_t kt, int kk) {
            const unsigned char *sa = stAP(kt >> 1) + ap_lds + ((((kt & 1) * 4 + 2 * kk + h) ^ ap_sw) * 16);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) af[mb] = *(const v4i *)(sa + mb * 32 * 128);
        };

        auto issue_step_b = [&](uint32_t kt, bool guard) {
            if (!guard || kt + 3 < nk) issue_b(offB4(kt + 3));
        };
        auto issue_step_a = [&](uint32_t kt, bool guard) {
            if ((kt & 1) == 0 && (!guard || kt + 2 < nk)) issue_ap((kt + 2) >> 1);
        };
        // prologue in steady-state order: B0, B1, pair 0, B2
        issue_b(offB4(0));
        if (nk > 1) issue_b(offB4(1));
        issue_ap(0);
        if (nk > 2) issue_b(offB4(2));
        // step 0 (peeled: no MFMAs pending yet)
        if (nk > 2) CATCOC_WAIT_VMCNT(B_DMA);
        else CATCOC_WAIT_VMCNT(0);
        barrier_keep_vmem();
        issue_step_b(0, true);
        issue_step_a(0, true);
        load_ap(fa0, 0, 0);
        load_b(fb0, stB(0), 0);
        load_ap(fa1, 0, 1);
        load_b(fb1, stB(0), 1);
        CATCOC_FENCE();
        mma(fa0, fb0);
        CATCOC_FENCE();

        auto compute = [&](uint32_t kt, bool guard) {
            // The two waves that share a SIMD (w and w + 4) issue their copies in different halves of the step,
            // so that one of them always has MFMAs to feed the matrix pipe while the other computes addresses.
            const bool early = ws < NW / 2;
            sched_step([&](v4i (&af)[MB], int kk) { load_ap(af, kt, kk); }, stB(kt),
                       [&] { if (early) issue_step_b(kt, guard); }, [&] { if (early) issue_step_a(kt, guard); }, nothing,
                       [&] {
                           if (!early) {
                               issue_step_b(kt, guard);
                               issue_step_a(kt, guard);
                           }
                       });
        };
        uint32_t kt = 1;
        for (; kt + 5 <= nk; kt += 2) {
            CATCOC_WAIT_VMCNT(WAIT_ODD);
            barrier_keep_vmem();
            compute(kt, false);
            CATCOC_WAIT_VMCNT(WAIT_EVEN);
            barrier_keep_vmem();
            compute(kt + 1, false);
        }
        for (; kt < nk; ++kt) {   // tail: drain fully at every step
            CATCOC_WAIT_VMCNT(0);
            barrier_keep_vmem();
            compute(kt, true);
        }
        mma(fa1, fb1);
    }

#undef CATCOC_FENCE

    // ---- k slices meet --------------------------------------------------------------
    // Every slice writes its partial tile through to memory (device-scope stores, 16 bytes per lane, the tile in
    // register order: index (((mb*4 + nb)*4 + g)*256 + thread)*4 + j holds register r = 4g + j), a per-tile counter
    // elects the last slice to arrive, and that workgroup adds the others' partials and goes on to the epilogue.
    // (the order of the additions: below, where the partials meet)
    // RM: only the 32-row blocks with kept rows travel (unless the caller wants a dump of every accumulator): of the others
    // a checksum needs the sum alone, and sums of sums are exact, so every lane adds up what it holds of such a block and
    // the eight bytes travel in the place of the block's first 16.  At M = 512 with 64 kept rows three tiles in four then
    // hand over 4 KiB instead of 128 and the fourth 64 KiB.
    uint32_t travelMb = (1u << MB) - 1u;   // bit mb: block mb of this wave travels whole (wave-uniform)
    long long othersSum[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) othersSum[mb] = 0;
    if constexpr (RM) {
        if (args.accDump == nullptr) {
            travelMb = 0;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                if ((ti.row + wm * 32 * MB + mb * 32 - args.keptBegin) < args.keptRows) travelMb |= 1u << mb;
        }
    }
    // RM with the pipelined peer loads (launches of one round of workgroups): the kept tiles are few, and what ends the launch
    // is the one workgroup per kept tile that streams the peers' partials of its kept rows through one CU (about 60 GB/s).
    // Every other workgroup of the same tile column -- the tiles of the other row blocks and the k slices that do not
    // finish the kept tile -- is done at about the moment that stream starts.  On its way out it reads one word of every
    // 128-byte line of ONE peer's kept rows in its 256 columns (workgroup number u of the column takes peer nPeers - 1 - u:
    // the stream starts at peer 0), so that the line is in the L2 (same XCD) or at least in the memory-side cache when the
    // stream arrives there.  Nothing is done with the words.
    auto prefetch_peers = [&]() {
        if constexpr (RM && PP) {
            const uint32_t lines = args.keptRows * 8u;   // of one peer's kept rows in this tile's columns
            const uint32_t u = (ti.row / (uint32_t)BM) * kSlices + slice;
            if (args.nPeers == 0 || (args.flags & GF_REDUCE_INT32) || u >= args.nPeers || lines > 8u * NT) return;
            const float *peer = (const float *)args.peers[args.nPeers - 1u - u] + args.peerRowOffset * args.peerLd + ti.col;
            for (uint32_t l = tid; l < lines; l += NT) {
                const float word = *(volatile const float *)(peer + (size_t)(l >> 3) * args.peerLd + (l & 7u) * 32u);
                (void)word;
            }
            CATCOC_WAIT_VMCNT(0);
        }
    };
    if constexpr (WM == 2) {
        if (kSlices > 1) {
            constexpr int DEVICE_SCOPE = 16;   // sc1
            constexpr uint32_t TILE_WORDS = BM * 256;
            const __amdgpu_buffer_rsrc_t mine = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(args.skPart + ((size_t)task * kSlices + slice) * TILE_WORDS), 0, (int)(TILE_WORDS * 4), 0x00020000);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                if (travelMb & (1u << mb)) {
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const auto e0 = acc[mb][nb][4 * g], e1 = acc[mb][nb][4 * g + 1], e2 = acc[mb][nb][4 * g + 2], e3 = acc[mb][nb][4 * g + 3];
                            const v4i iv = {__builtin_bit_cast(int, e0), __builtin_bit_cast(int, e1), __builtin_bit_cast(int, e2), __builtin_bit_cast(int, e3)};
                            __builtin_amdgcn_raw_buffer_store_b128(iv, mine, (((mb * 4 + nb) * 4 + g) * NT + tid) * 16, 0, DEVICE_SCOPE);
                        }
                } else if constexpr (RM) {
                    if (args.checksum != nullptr) {
                        long long sb = 0;
#pragma unroll
                        for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                            for (int r = 0; r < 16; ++r) sb += acc[mb][nb][r];
                        const v2i sv = {(int)(uint32_t)(unsigned long long)sb, (int)(uint32_t)((unsigned long long)sb >> 32)};
                        __builtin_amdgcn_raw_buffer_store_b64(sv, mine, ((mb * 16) * NT + tid) * 16, 0, DEVICE_SCOPE);
                    }
                }
            }
            CATCOC_WAIT_VMCNT(0);   // once the stores are acknowledged the slice may be counted
            __syncthreads();
            volatile uint32_t *flag = (volatile uint32_t *)smem;
            if (tid == 0) *flag = __hip_atomic_fetch_add(args.skCount + task, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            if (*flag != kSlices - 1u) {
                prefetch_peers();
                return;
            }
            if (tid == 0) __hip_atomic_store(args.skCount + task, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // Integer partials add exactly in any order, and so do two float partials: the last slice to arrive keeps its own in
            // registers and adds the others.  Three or more float partials are added in SLICE order whichever slice arrives
            // last (the result then does not depend on timing): the accumulators restart at zero and every slice's partial,
            // the workgroup's own included, comes back from the workspace, slice 0 first.
            const bool ordered = DT != DT_I8 && kSlices > 2u;
            if constexpr (DT != DT_I8) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const float keep = acc[mb][nb][r];
                            acc[mb][nb][r] = ordered ? 0.0f : keep;   // (a select, not a branch around the accumulators)
                        }
            }
            const uint32_t nOthers = ordered ? kSlices : kSlices - 1u;
            for (uint32_t o = 0; o < nOthers; ++o) {
                const uint32_t sl = ordered ? o : (o < slice ? o : o + 1);
                const __amdgpu_buffer_rsrc_t other = __builtin_amdgcn_make_buffer_rsrc(
                    (void *)(args.skPart + ((size_t)task * kSlices + sl) * TILE_WORDS), 0, (int)(TILE_WORDS * 4), 0x00020000);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {   // one 32-row block (64 registers) per round trip
                    if (!(travelMb & (1u << mb))) {
                        if constexpr (RM) {
                            if (args.checksum != nullptr) {
                                const v2i sv = __builtin_amdgcn_raw_buffer_load_b64(other, ((mb * 16) * NT + tid) * 16, 0, DEVICE_SCOPE);
                                othersSum[mb] += (long long)(((unsigned long long)(uint32_t)sv.y << 32) | (uint32_t)sv.x);
                            }
                        }
                        continue;
                    }
                    v4i pv[4][4];
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                        for (int g = 0; g < 4; ++g)
                            pv[nb][g] = __builtin_amdgcn_raw_buffer_load_b128(other, (((mb * 4 + nb) * 4 + g) * NT + tid) * 16, 0, DEVICE_SCOPE);
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const int p0 = pv[nb][g].x, p1 = pv[nb][g].y, p2 = pv[nb][g].z, p3 = pv[nb][g].w;
                            if constexpr (DT == DT_I8) {
                                acc[mb][nb][4 * g] += p0;
                                acc[mb][nb][4 * g + 1] += p1;
                                acc[mb][nb][4 * g + 2] += p2;
                                acc[mb][nb][4 * g + 3] += p3;
                            } else {
                                acc[mb][nb][4 * g] += __builtin_bit_cast(float, p0);
                                acc[mb][nb][4 * g + 1] += __builtin_bit_cast(float, p1);
                                acc[mb][nb][4 * g + 2] += __builtin_bit_cast(float, p2);
                                acc[mb][nb][4 * g + 3] += __builtin_bit_cast(float, p3);
                            }
                        }
                }
            }
        }
    }

    // ---- epilogue -----------------------------------------------------------------
    // acc[mb][nb][r] is element (row, col) of the tile with
    //   row = wm*32*MB + mb*32 + (r>>2)*8 + h*4 + (r&3),  col = wn*128 + nb*32 + c32
    const uint32_t col0 = wn * 128 + c32;       // + 32*nb
    const uint32_t gcol0 = ti.col + col0;
    const uint32_t row_base = wm * 32 * MB + h * 4;
    bool kept = ti.row >= args.keptBegin && ti.row < args.keptBegin + args.keptRows;
    // RM: bit mb is set when 32-row block mb of this wave is kept (the unsigned compare also rejects blocks above keptBegin:
    // the difference wraps); the tile counts as kept when any of its rows is
    uint32_t keptMb = 0;
    if constexpr (RM) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            if ((ti.row + wm * 32 * MB + mb * 32 - args.keptBegin) < args.keptRows) keptMb |= 1u << mb;
        kept = ti.row < args.keptBegin + args.keptRows && ti.row + BM > args.keptBegin;
        if (!kept) prefetch_peers();
    }
    // W8A8 accumulators are dequantised in place (the registers then hold fp32 bit patterns); element accesses go
    // through scalar temporaries
    auto getf = [&](int mb, int nb, int r) -> float {
        if constexpr (DT == DT_I8) {
            const int iv = acc[mb][nb][r];
            return i2f(iv);
        } else {
            const float fv = acc[mb][nb][r];
            return fv;
        }
    };
    auto setf = [&](int mb, int nb, int r, float v) {
        if constexpr (DT == DT_I8) acc[mb][nb][r] = f2i(v);
        else acc[mb][nb][r] = v;
    };

    if constexpr (DT == DT_I8) {
        if (args.bias != nullptr) {
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
                const int bv = args.bias[gcol0 + 32 * nb];
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[mb][nb][r] += bv;
            }
        }
    }

    if (args.accDump != nullptr) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                if constexpr (DT == DT_I8) {
                    int32_t *o = (int32_t *)args.accDump + (size_t)(ti.row + lrow) * args.N + gcol0;
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) {
                        const int iv = acc[mb][nb][r];
                        o[32 * nb] = iv;
                    }
                } else {
                    float *o = (float *)args.accDump + (size_t)(ti.row + lrow) * args.N + gcol0;
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) o[32 * nb] = getf(mb, nb, r);
                }
            }
    }

    // W8A8 scales of this lane's rows and columns, fetched in one batch (32 + 4 loads in flight together;
    // fetched one row at a time next to their use they cost a memory round trip per row)
    float sN[4] = {1.f, 1.f, 1.f, 1.f};
    float sMv[MB][16];
    if constexpr (DT == DT_I8) {
        if (kept || (args.flags & GF_OUTBOUND_STORE)) {
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) sN[nb] = args.scaleN[gcol0 + 32 * nb];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) sMv[mb][r] = args.scaleM[ti.row + row_base + mb * 32 + (r >> 2) * 8 + (r & 3)];
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    if constexpr (RM) {
        if (args.checksum != nullptr) {
            // the accumulators of the 32-row blocks that are not kept, per 128 x 128 block (one wave column each)
            long long si = 0;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                long long sb = 0;   // (summed for every block and dropped for kept ones: no control flow around the accumulators)
#pragma unroll
                for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) sb += acc[mb][nb][r];
                si += (kept && (keptMb & (1u << mb))) ? 0ll : sb + othersSum[mb];
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) si += __shfl_xor(si, o, 64);
            long long *red = (long long *)smem;
            __syncthreads();   // every wave has left the main loop's LDS reads behind
            if (lane == 0) red[w] = si;
            __syncthreads();
            if (tid < 2) {
                long long t = 0;
#pragma unroll
                for (int i = 0; i < WR; ++i) t += red[2 * i + tid];
                ((long long *)args.checksum)[(size_t)(ti.row / 128u) * (args.N / 128u) + ti.col / 128u + tid] = t;
            }
        }
    }

    // W8A8 with GF_REDUCE_INT32 (the reference's data flow, quant_matmul_reduce_scatter.hpp:191-201,285-351): the peers'
    // partials are int32 and join the accumulators before the dequantisation; tiles of other ranks leave as raw int32
    const bool redI32 = DT == DT_I8 && (args.flags & GF_REDUCE_INT32) != 0;
    const uint32_t nPeersI32 = redI32 ? args.nPeers : 0u, nPeersF32 = redI32 ? 0u : args.nPeers;
    if (kept) {
        // (RM: a tile that starts above keptBegin makes this wrap; it is only added to rows of kept blocks, where the sum
        // is the row's index in the kept range again)
        const uint32_t out_row0 = ti.row - args.keptBegin;
        if constexpr (DT == DT_I8) {
            // one int32 partial of the tile, 32 rows (64 loads per lane) at a time, as add_partial below does for fp32
            for (uint32_t p = 0; p < nPeersI32; ++p) {
                const int32_t *peer = (const int32_t *)args.peers[p] + args.peerRowOffset * args.peerLd;
                const int32_t *src = peer + (int64_t)(int32_t)out_row0 * args.peerLd + (size_t)row_base * args.peerLd + gcol0;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const int32_t *srcb = src + (size_t)(mb * 32) * args.peerLd;
                    if constexpr (RM) srcb = (keptMb & (1u << mb)) ? srcb : peer + (size_t)(h * 4) * args.peerLd + gcol0;   // (as add_partial)
                    int pv[16][4];
#pragma unroll
                    for (int r = 0; r < 16; ++r)
#pragma unroll
                        for (int nb = 0; nb < 4; ++nb)
                            pv[r][nb] = __builtin_nontemporal_load(srcb + (size_t)((r >> 2) * 8 + (r & 3)) * args.peerLd + 32 * nb);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int r = 0; r < 16; ++r)
#pragma unroll
                        for (int nb = 0; nb < 4; ++nb) acc[mb][nb][r] += pv[r][nb];
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if (args.cAccum != nullptr) {
                // the int32 block, turned around in the wave's 16 KiB of LDS 32 rows at a time like the workspace tiles below:
                // sixteen-byte stores that cover whole 512-byte row segments instead of 128 four-byte stores per lane
                static_assert(NW * 16384 <= POOL, "one 16 KiB staging area per wave");
                unsigned char *stc = smem + w * 16384;
                __syncthreads();   // every wave has left the main loop's LDS reads behind
                int32_t *cw = args.cAccum + ((int64_t)(int32_t)out_row0 + wm * 32 * MB) * (int64_t)args.N + ti.col + wn * 128;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t wrow = (r >> 2) * 8 + h * 4 + (r & 3);
#pragma unroll
                        for (int nb = 0; nb < 4; ++nb) {
                            const int iv = acc[mb][nb][r];
                            *(int *)(stc + wrow * 512 + (((nb * 32 + c32) * 4) ^ (h << 7))) = iv;
                        }
                    }
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        const uint32_t wrow = j * 2 + (lane >> 5), chunk = lane & 31;
                        const v4i v = *(const v4i *)(stc + wrow * 512 + ((chunk * 16) ^ (((wrow >> 2) & 1) << 7)));
                        if (RM && !(keptMb & (1u << mb))) continue;   // (stores only)
                        *(v4i *)(cw + (int64_t)(mb * 32 + wrow) * args.N + chunk * 4) = v;
                    }
                }
            }
            // a round of the pipelined operator whose comm side also writes the dequantised rows: the int32 block is all
            // this tile owes
            if (args.flags & GF_KEPT_INT32_ONLY) return;
            // dequantise in place: per-channel scale first, then per-token, each product rounded on its own
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float sM = sMv[mb][r];
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) {
                        const int iv = acc[mb][nb][r];
                        acc[mb][nb][r] = f2i(__fmul_rn(__fmul_rn((float)iv, sN[nb]), sM));
                    }
                }
        }

        if constexpr (PP) {
            // One workgroup per CU (the deep ring): few tiles, so few kept tiles, and their peer partials are bound by memory
            // latency, not bandwidth.  Fetched in accumulator layout (64 four-byte loads per 32-row block and peer) a wave
            // cannot have more than its 63 outstanding loads = 16 KiB in flight, and every block costs a memory round trip per
            // peer.  So the block is turned around in the wave's 16 KiB of LDS first (4-byte writes in accumulator layout,
            // 16-byte reads along the rows: a lane then holds four consecutive columns of rows 2j + lane/32, j = 0..15), and a
            // peer's values are 16 sixteen-byte loads per lane, issued eight at a time ("units") into a ring of six register
            // buffers, five units (40 KiB per wave) in flight.  Every element sees the same additions in the same order as in
            // accumulator layout.
            static_assert(NW * 16384 <= POOL, "one 16 KiB staging area per wave");
            constexpr int NBUF = W8 ? 4 : 6;   // (eight waves: 256 registers per wave; the count must be even)
            unsigned char *st = smem + w * 16384;
            __syncthreads();   // every wave has left the main loop's LDS reads behind
            const uint32_t U = 2u * nPeersF32;   // units: peer u / 2, rows 16 (u & 1) .. of the block
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                if constexpr (RM)
                    if (!(keptMb & (1u << mb))) continue;
                const uint32_t lrow = lane >> 5, chunk = lane & 31;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t wrow = (r >> 2) * 8 + h * 4 + (r & 3);
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) *(float *)(st + wrow * 512 + (((nb * 32 + c32) * 4) ^ (h << 7))) = getf(mb, nb, r);
                }
                v4f cur[16];
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const uint32_t wrow = j * 2 + lrow;
                    cur[j] = *(const v4f *)(st + wrow * 512 + ((chunk * 16) ^ (((wrow >> 2) & 1) << 7)));
                }
                // peers and output go through buffer descriptors: a wave-uniform base per unit, one per-lane offset for all
                // of them, and the row step as a scalar offset, so that a load costs no address arithmetic in vector registers
                const int64_t rowInKept = (int64_t)(int32_t)out_row0 + (ws >> 1) * 32 * MB + mb * 32;
                const uint32_t colW = ti.col + (ws & 1u) * 128;
                const uint32_t pitchB = (uint32_t)args.peerLd * 4u;
                const uint32_t voff = lrow * pitchB + chunk * 16u;
                v4f buf[NBUF][8];
                // (a unit past the last one is issued with an empty descriptor: its loads return zeros without touching memory,
                // so every turn of the ring issues and counts the same number of loads whatever the number of peers)
                auto issue = [&](v4f (&b)[8], uint32_t u) {
                    const float *base = (const float *)args.peers[umin(u >> 1, (uint32_t)kMaxRanks - 1u)] +
                                        (args.peerRowOffset + rowInKept + (int64_t)((u & 1u) * 16u)) * args.peerLd + colW;
                    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, u < U ? 0x7ffffff0 : 0, 0x00020000);
#pragma unroll
                    for (int jj = 0; jj < 8; ++jj)
                        b[jj] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rs, voff, (2 * jj) * pitchB, 2 /* nt */));
                };
                if (U > 0) {
#pragma unroll
                    for (int q = 0; q < NBUF - 1; ++q) issue(buf[q], q);
                    for (uint32_t u = 0; u < U; u += NBUF) {
#pragma unroll
                        for (int q = 0; q < NBUF; ++q) {   // unit u + q sits in buffer q and adds to rows 16 (q & 1) ..
                            __builtin_amdgcn_sched_barrier(0);
                            issue(buf[(q + NBUF - 1) % NBUF], u + q + NBUF - 1);
                            __builtin_amdgcn_sched_barrier(0);
                            if (u + q < U) {
#pragma unroll
                                for (int jj = 0; jj < 8; ++jj) {
                                    v4f &c = cur[(q & 1) * 8 + jj];
                                    c.x = __fadd_rn(c.x, buf[q][jj].x);
                                    c.y = __fadd_rn(c.y, buf[q][jj].y);
                                    c.z = __fadd_rn(c.z, buf[q][jj].z);
                                    c.w = __fadd_rn(c.w, buf[q][jj].w);
                                }
                            }
                        }
                    }
                }
                // 16-bit output: a lane's four columns are eight bytes, a wave instruction covers two 256-byte row segments
                const uint32_t pitchD = (uint32_t)args.ldd * 2u;
                const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(
                    (void *)((unsigned char *)args.d + (rowInKept * args.ldd + colW) * 2), 0, 0x7ffffff0, 0x00020000);
                const uint32_t voffD = lrow * pitchD + chunk * 8u;
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    uint32_t q0, q1, q2, q3;
                    if (args.outDtype == DT_BF16) {
                        q0 = f32_to_bf16_bits(cur[j].x); q1 = f32_to_bf16_bits(cur[j].y); q2 = f32_to_bf16_bits(cur[j].z); q3 = f32_to_bf16_bits(cur[j].w);
                    } else {
                        q0 = f32_to_f16_bits(cur[j].x); q1 = f32_to_f16_bits(cur[j].y); q2 = f32_to_f16_bits(cur[j].z); q3 = f32_to_f16_bits(cur[j].w);
                    }
                    const v2i pk = {(int)((q0 & 0xffffu) | (q1 << 16)), (int)((q2 & 0xffffu) | (q3 << 16))};
                    __builtin_amdgcn_raw_buffer_store_b64(pk, rd, voffD, (2 * j) * pitchD, 0);
                }
            }
        } else {
        // one fp32 partial of the tile, added from global memory 32 rows (64 loads per lane) at a time
        // (RM: a block that is not kept adds the first 32 kept rows of the peer instead -- valid memory, and its sums are
        // never stored; skipping it would put control flow around the accumulators, which costs far more than the loads)
        auto add_partial = [&](const float *base, int64_t ld, const float *firstKept) {
            const float *src = base + (size_t)row_base * ld + gcol0;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const float *srcb = src + (size_t)(mb * 32) * ld;
                if constexpr (RM) srcb = (keptMb & (1u << mb)) ? srcb : firstKept + (size_t)(h * 4) * ld + gcol0;
                float pv[16][4];
#pragma unroll
                for (int r = 0; r < 16; ++r)
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb)
                        pv[r][nb] = __builtin_nontemporal_load(srcb + (size_t)((r >> 2) * 8 + (r & 3)) * ld + 32 * nb);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int r = 0; r < 16; ++r)
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) setf(mb, nb, r, __fadd_rn(getf(mb, nb, r), pv[r][nb]));
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        for (uint32_t p = 0; p < nPeersF32; ++p) {
            const float *peer = (const float *)args.peers[p] + args.peerRowOffset * args.peerLd;
            add_partial(peer + (int64_t)(int32_t)out_row0 * args.peerLd, args.peerLd, peer);
        }

        // 16-bit output.  A lane holds single columns 32 apart, so storing from registers would write 64-byte
        // pieces (half a cache line each, 128 store instructions per lane).  Instead every wave turns its 64 x 128
        // block around in a private 16 KiB LDS area: 2-byte writes in accumulator layout, 16-byte reads along the
        // rows, and 16 stores per lane that each cover four whole 256-byte row segments.  Rows with bit 2 set
        // (the upper half-wave of a write) are shifted by 128 bytes, which keeps both half-waves on different banks.
        static_assert(NW * 16384 <= POOL, "one 16 KiB staging area per wave");
        unsigned char *st = smem + w * 16384;
        __syncthreads();   // every wave has left the main loop's LDS reads behind
        auto stage_all = [&](auto cvt) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t wrow = mb * 32 + (r >> 2) * 8 + h * 4 + (r & 3);
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb)
                        *(unsigned short *)(st + wrow * 256 + (((nb * 32 + c32) * 2) ^ (h << 7))) = (unsigned short)cvt(getf(mb, nb, r));
                }
        };
        if (args.outDtype == DT_BF16) stage_all([](float f) { return f32_to_bf16_bits(f); });
        else stage_all([](float f) { return f32_to_f16_bits(f); });
        unsigned char *dwave = (unsigned char *)args.d + (((int64_t)(int32_t)out_row0 + wm * 32 * MB) * args.ldd + ti.col + wn * 128) * 2;
#pragma unroll
        for (int j = 0; j < 8 * MB; ++j) {
            if constexpr (RM) if (!(keptMb & (1u << (j >> 3)))) continue;   // rows 4j .. 4j+3 of the wave: 32-row block j / 8
            const uint32_t wrow = j * 4 + (lane >> 4), chunk = lane & 15;
            const v4i v = *(const v4i *)(st + wrow * 256 + ((chunk * 16) ^ (((wrow >> 2) & 1) << 7)));
            *(v4i *)(dwave + (size_t)wrow * args.ldd * 2 + chunk * 16) = v;
        }
        }
    } else if (args.flags & GF_OUTBOUND_STORE) {
        // fp32 tile of another rank, to the tile-linear workspace (rows wsRow .., n0 columns).  A lane holds single columns
        // 32 apart, so storing from registers takes 128 four-byte stores per lane, and a wave can only have 63 memory
        // operations outstanding: the tile would leave in three write round trips.  Instead every wave turns its block
        // around in its private 16 KiB of LDS, 32 rows at a time (4-byte writes in accumulator layout, 16-byte reads along
        // the rows), and leaves in 32 sixteen-byte streaming stores per lane that each cover two whole 512-byte row
        // segments.  Rows with bit 2 set (the upper half-wave of a write) are shifted by 128 bytes to other banks.
        static_assert(NW * 16384 <= POOL, "one 16 KiB staging area per wave");
        unsigned char *st = smem + w * 16384;
        __syncthreads();   // every wave has left the main loop's LDS reads behind
        // (RG: the tile's own rows and columns start at (shiftM, shiftN) and go to workspace position (0, 0))
        float *obw = (float *)args.outbound + ((int64_t)ti.wsRow + wm * 32 * MB - (int64_t)shiftM) * sp.n0 + wn * 128 - (int64_t)shiftN;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t wrow = (r >> 2) * 8 + h * 4 + (r & 3);   // row inside the 32-row block
                float sM = 1.f;
                if constexpr (DT == DT_I8) sM = sMv[mb][r];
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) {
                    float v;
                    if constexpr (DT == DT_I8) {
                        const int iv = acc[mb][nb][r];
                        v = redI32 ? i2f(iv) : __fmul_rn(__fmul_rn((float)iv, sN[nb]), sM);   // (raw int32: the bit pattern travels)
                    } else {
                        v = getf(mb, nb, r);
                    }
                    *(float *)(st + wrow * 512 + (((nb * 32 + c32) * 4) ^ (h << 7))) = v;
                }
            }
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const uint32_t wrow = j * 2 + (lane >> 5), chunk = lane & 31;
                const v4f v = *(const v4f *)(st + wrow * 512 + ((chunk * 16) ^ (((wrow >> 2) & 1) << 7)));
                if constexpr (RG)
                    if (wm * 32 * MB + mb * 32 + wrow < shiftM || wn * 128 + chunk * 4 < shiftN) continue;
                __builtin_nontemporal_store(v, (v4f *)(obw + (size_t)(mb * 32 + wrow) * sp.n0 + chunk * 4));
            }
        }
    } else if (!RM && args.checksum != nullptr) {
        // int64 sum of the int32 accumulators (W8A8) or double sum of the fp32 ones
        using Sum = typename std::conditional<DT == DT_I8, long long, double>::type;
        Sum *red = (Sum *)smem;   // the pool is free again
        Sum si = 0;
        bool summed = false;
        if constexpr (RG) {
            if ((shiftM | shiftN) != 0) {   // the tile's own part only
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const bool rowOwn = row_base + mb * 32 + (r >> 2) * 8 + (r & 3) >= shiftM;
#pragma unroll
                        for (int nb = 0; nb < 4; ++nb) {
                            const bool own = rowOwn && col0 + 32 * nb >= shiftN;
                            if constexpr (DT == DT_I8) {
                                const int iv = acc[mb][nb][r];
                                si += own ? iv : 0;
                            } else {
                                si += own ? (double)getf(mb, nb, r) : 0.0;
                            }
                        }
                    }
                summed = true;
            }
        }
        if constexpr (DT == DT_I8) {
            // |accumulator| <= 128 * 128 * k (int8 admits -128), so without a bias four of them add in 32 bits for
            // k < 32768 (4 * 2^14 * 32767 < 2^31): a third of the 64-bit additions
            if (!summed && args.bias == nullptr && args.K < 32768u) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                        for (int g = 0; g < 4; ++g)
                            si += (acc[mb][nb][4 * g] + acc[mb][nb][4 * g + 1]) + (acc[mb][nb][4 * g + 2] + acc[mb][nb][4 * g + 3]);
                summed = true;
            }
        }
        if (!summed) {
            if constexpr (DT == DT_I8) {
                // exact in 32-bit arithmetic: a = (a >> 16) * 65536 + (a & 0xffff), and 128 of either part add without overflow
                int hi = 0, lo = 0;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int a = acc[mb][nb][r];
                            hi += a >> 16;
                            lo += a & 0xffff;
                        }
                si = (long long)hi * 65536 + lo;
            } else {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                        for (int r = 0; r < 16; ++r) si += (double)getf(mb, nb, r);
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) si += __shfl_xor(si, o, 64);
        __syncthreads();   // every wave has left the main loop's LDS reads behind
        if (lane == 0) red[w] = si;
        __syncthreads();
        if (tid == 0) {
            Sum t = 0;
#pragma unroll
            for (int i = 0; i < NW; ++i) t += red[i];
            if constexpr (HALF) {
                // The two 64-row halves of a task meet through a 64-bit word per task (the workspace's counter block, all zero
                // between launches): each exchanges its sum, encoded so that it is never zero, into the word; the half that
                // finds the other's sum there adds the two (either order gives the same bits), writes the task's checksum
                // and clears the word.
                unsigned long long enc;
                if constexpr (DT == DT_I8) {
                    enc = (unsigned long long)(t + (1ll << 62));   // |t| < 2^47
                } else {
                    enc = __builtin_bit_cast(unsigned long long, t);
                    if (t != t) enc = 0x7ff8000000000000ull;
                    enc += 1ull;
                }
                unsigned long long *word = (unsigned long long *)args.skCount + task;
                const unsigned long long other = __hip_atomic_exchange(word, enc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (other != 0ull) {
                    Sum o;
                    if constexpr (DT == DT_I8) o = (long long)other - (1ll << 62);
                    else o = __builtin_bit_cast(double, other - 1ull);
                    ((Sum *)args.checksum)[task] = t + o;
                    __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            } else {
                ((Sum *)args.checksum)[task] = t;
            }
        }
    }

}

// One workgroup per tile, or per k slice of a tile.
template <uint32_t DT, int WM, bool TB = false, bool RM = false, bool RG = false, bool TA = false, int NS = 3, bool PP = false, bool AQ = false, bool W8 = false>
__global__ void __launch_bounds__(128 * WM * (W8 ? 2 : 1), NS == 3 ? 2 : 1) gemm_dma_kernel(const GemmArgs args)
{
    __shared__ __attribute__((aligned(1024))) unsigned char smem[DmaPool<WM, NS, AQ, TB>::BYTES];
    // A launch with few tiles can cut every tile's k range into kSlices pieces, one workgroup each (128-row tiles
    // only): position `pos` of the launch order runs as kSlices workgroups that stay in the position's XCD column.
    uint32_t pos = blockIdx.x + args.taskBase, slice = 0;   // (taskBase is zero for k-sliced launches)
    const uint32_t kSlices = (WM == 2 && args.splitK > 1) ? args.splitK : 1u;
    if (kSlices > 1) {
        if ((args.sched.coreLoops & 7u) == 0) {
            const uint32_t q = blockIdx.x >> 3;
            slice = q % kSlices;
            pos = (q / kSlices) * 8u + (blockIdx.x & 7u);
        } else {
            slice = blockIdx.x % kSlices;
            pos = blockIdx.x / kSlices;
        }
    }
    dma_tile<DT, WM, TB, RM, RG, TA, W8 ? 1 : 2, NS, PP, AQ, W8>(args, smem, pos, slice, kSlices, 0);
}

// Reduce-scatter launches of a single round of workgroups (no more tiles than the 512 slots of the GPU) run some tiles as two
// 64-row workgroups.  Positions of an XCD in launch order (workgroup id = 8 * j + xcd):
//   the first keptPerXcd positions, the kept tiles: a kept tile is the longest chain of such a launch (its main loop, then the
//     peers' partials from HBM) and nothing follows it, so the launch lasts as long as that chain; cut in two, each half
//     streams half the peers, on two CUs;
//   the last tailPerXcd positions: the kept halves make the launch larger than the workgroup slots of the GPU, and the tiles
//     that have to wait for a slot get the ones the kept halves leave, about one tile time before the end; as halves they
//     fill those slots for half a tile time (their checksum halves meet through the workspace's counter block).
// Requires the XCD-block order, whole tiles, A as [m,k], one launch for all tasks.
template <uint32_t DT, bool TB>
__global__ void __launch_bounds__(256, 2) gemm_dma_split_kept_kernel(const GemmArgs args, const uint32_t keptPerXcd, const uint32_t tailPerXcd)
{
    __shared__ __attribute__((aligned(1024))) unsigned char smem[DmaPool<2>::BYTES];
    const uint32_t x = blockIdx.x & 7u, j = blockIdx.x >> 3, n = args.sched.coreLoops >> 3;
    const uint32_t whole = n - keptPerXcd - tailPerXcd;   // positions keptPerXcd .. keptPerXcd + whole - 1 run whole
    uint32_t posJ, sub = 0;
    bool half = true;
    if (j < 2u * keptPerXcd) {
        posJ = j >> 1;
        sub = (j & 1u) * 64u;
    } else if (j < 2u * keptPerXcd + whole) {
        posJ = j - keptPerXcd;
        half = false;
    } else {
        const uint32_t t = j - (2u * keptPerXcd + whole);
        posJ = keptPerXcd + whole + (t >> 1);
        sub = (t & 1u) * 64u;
    }
    if (half) dma_tile<DT, 2, TB, false, false, false, 1>(args, smem, posJ * 8u + x, 0, 1, sub);
    else dma_tile<DT, 2, TB, false, false, false, 2>(args, smem, posJ * 8u + x, 0, 1, 0);
}

// A launch of at most one workgroup per CU has the whole LDS of a CU for each workgroup.  When its operands are too large to
// come out of the L2s (48 MB of A and B or more: they stream from HBM or the Infinity Cache, whose latency the two steps of
// look-ahead of the three-stage ring do not cover) it runs the six-stage ring with the pipelined peer loads.  Measured with
// the variants alternating launch by launch, W8A8 with explicit kept rows at K = N = 8192, B from HBM on every launch (six
// copies): M = 512 140 us on three stages, 75 with six, 70 with the pipelined peer loads as well; M = 1024 158 / 102 / 106.
// Small operands do not gain: config 2 (42 MB) 47.9 -> 49.6 us, config 1 18.2 -> 20.7 (and 23.6 with the pipelined peer loads).
inline bool deep_ring(const GemmArgs &a, uint32_t workgroups, uint64_t es /* bytes per operand element */)
{
    return workgroups <= 256u && (uint64_t)a.K * es * ((uint64_t)a.M * (a.sched.op == OP_ALLGATHER ? a.sched.P : 1u) + a.N) >= (48ull << 20);
}

// The six-stage ring copies A in pairs of k steps (whole 128-byte lines per row) when every workgroup's k range is whole
// pairs and long enough for the ring to fill (A as [m,k]).  Same measurement, both variants alternating: M = 512 (two k
// slices) 71.2 -> 65.4 us, M = 1024 105.8 -> 98.4 us.
inline bool deep_ring_pairs(const GemmArgs &a, uint64_t es)
{
    const uint64_t nkAll = (uint64_t)a.K * es / 64u, f = a.splitK > 1 ? a.splitK : 1u;
    return !a.transA && ((uint64_t)a.K * es) % 64u == 0 && nkAll % (2u * f) == 0 && nkAll / f >= 16u;
}

// Launch of the 128-row geometry: one instantiation per operand layout (A as [m][k] or [k][m], B as [k][n] or [n][k]) and
// for ragged problems; one workgroup per tile, or per k slice of a tile.
template <uint32_t DT>
inline int launch_dma_128(const GemmArgs &args, hipStream_t s)
{
    const dim3 grid(launch_positions(args) * (args.splitK > 1 ? args.splitK : 1u)), block(256);
    switch ((args.transA ? 4 : 0) | (args.transB ? 2 : 0) | ((args.flags & GF_RAGGED) ? 1 : 0)) {
        case 0:
            if (const uint32_t keptPerXcd = split_kept_tiles(args, args.K * (DT == DT_I8 ? 1u : 2u) / 64u))
{
                const uint32_t tailPerXcd = split_tail_tiles(args, keptPerXcd);
                hipLaunchKernelGGL((gemm_dma_split_kept_kernel<DT, false>), dim3(args.sched.coreLoops + 8u * (keptPerXcd + tailPerXcd)), block, 0, s, args,
                                   keptPerXcd, tailPerXcd);
            }
            else if (deep_ring(args, grid.x, DT == DT_I8 ? 1u : 2u)) {
                if (deep_ring_pairs(args, DT == DT_I8 ? 1u : 2u))
                    hipLaunchKernelGGL((gemm_dma_kernel<DT, 2, false, false, false, false, 6, true, true>), grid, block, 0, s, args);
                else
                    hipLaunchKernelGGL((gemm_dma_kernel<DT, 2, false, false, false, false, 6, true>), grid, block, 0, s, args);
            }
            else
                hipLaunchKernelGGL((gemm_dma_kernel<DT, 2, false, false, false, false>), grid, block, 0, s, args);
            break;
        case 1: hipLaunchKernelGGL((gemm_dma_kernel<DT, 2, false, false, true, false>), grid, block, 0, s, args); break;
        case 2:
            if (const uint32_t keptPerXcd = split_kept_tiles(args, args.K * (DT == DT_I8 ? 1u : 2u) / 64u))
{
                const uint32_t tailPerXcd = split_tail_tiles(args, keptPerXcd);
                hipLaunchKernelGGL((gemm_dma_split_kept_kernel<DT, true>), dim3(args.sched.coreLoops + 8u * (keptPerXcd + tailPerXcd)), block, 0, s, args,
                                   keptPerXcd, tailPerXcd);
            }
            else
                hipLaunchKernelGGL((gemm_dma_kernel<DT, 2, true, false, false, false>), grid, block, 0, s, args);
            break;
        case 3: hipLaunchKernelGGL((gemm_dma_kernel<DT, 2, true, false, true, false>), grid, block, 0, s, args); break;
        case 4: hipLaunchKernelGGL((gemm_dma_kernel<DT, 2, false, false, false, true>), grid, block, 0, s, args); break;
        case 5: hipLaunchKernelGGL((gemm_dma_kernel<DT, 2, false, false, true, true>), grid, block, 0, s, args); break;
        case 6: hipLaunchKernelGGL((gemm_dma_kernel<DT, 2, true, false, false, true>), grid, block, 0, s, args); break;
        default: hipLaunchKernelGGL((gemm_dma_kernel<DT, 2, true, false, true, true>), grid, block, 0, s, args); break;
    }
    return (int)hipGetLastError();
}

}  // namespace catcoc
