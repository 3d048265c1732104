// Skinny-M W8A8 GEMM for gfx950: few rows of A against a large B, which makes the
// launch HBM-bound on B.  The tile grid of SplitkMatmul is kept (tasks = tiles x k
// slices through SplitkGemmIdentityBlockSwizzle), with 128 x 128 tiles so that a
// decode-sized problem still spreads over every CU with a small split factor.
//
// A workgroup (4 waves) streams its k slice of B (64 k rows x 128 columns = 8 KiB per
// step) and of A straight into an LDS ring of 8 or 12 stages with direct-to-LDS copies,
// so 60 to 80 KiB per CU is in flight; every wave multiplies all rows of the tile by
// its own 32 columns, two or four steps per barrier.  Partial tiles of the k slices are written
// through to memory as int32 (device-scope stores), a per-tile counter elects the
// last slice to arrive, and that workgroup adds the other partials (integer adds:
// exact in any order), then runs the same epilogue as the large-M kernels on the
// rows that exist: bias, dequant, peers, 16-bit store for kept rows, checksum for
// the others.
//
// Stands in for SplitkMatmul + ReduceAdd
// (3rdparty/catlass/include/catlass/gemm/kernel/splitk_matmul.hpp:68-148,267-330)
// feeding the epilogue of quant_matmul_reduce_scatter.hpp:285-351.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "gemm_dma_kernel.h"

namespace catcoc {

// MBW: 32-row blocks staged per tile (1, 2 or 4); rows past the end of A are clamped to the last row
// on the way in and masked on the way out.
// AP: A is fetched per group of two k steps, 128 bytes per row (whole cache lines: half as many requests to L2 as two
// 64-byte halves), into one "pair" area per group; for 64- and 128-row tiles whose k slices are whole pairs of steps.
// TB: B is given as [n][k] (k contiguous, the layout of a stored weight matrix): a step's B stage is then 128 rows of 64
// bytes of k, copied and read exactly like A's (plain 16-byte fragment reads, no transposing reads).  A line of B is
// asked for in two halves one step apart; the second finds it in L2, so these copies carry no streaming hint.
// KP: eight waves, two per SIMD: waves 4-7 own the same columns as waves 0-3 and take the second step of every pair
// (accumulators of their own, added to the others' through LDS after the loop).  A wave alone on its SIMD reads its
// fragments, multiplies, waits at the barrier and issues copies one after the other, and the four waves do so in lockstep,
// so LDS, matrix pipe and copy path take turns; with a second wave per SIMD on the other step they overlap.
template <int MBW, bool AP = false, bool TB = false, bool KP = false>
__global__ void __launch_bounds__(KP ? 512 : 256, 1) gemm_splitk_kernel(const GemmArgs args)
{
    static_assert(!AP || MBW >= 2, "pairs of steps are the groups of the 64- and 128-row tiles");
    static_assert(!KP || AP, "the step-parity split works on pairs of steps");
    constexpr int NW = KP ? 8 : 4;             // waves that issue copies
    constexpr int PB = KP ? 4 : 8;             // peers whose values a wave holds at a time
    constexpr int G = (MBW == 1) ? 4 : 2;      // k steps per barrier
    constexpr int NS = (MBW == 1) ? 12 : 8;    // LDS stages (a multiple of G, at least 2G)
    constexpr int ROWS = 32 * MBW;
    constexpr int A_STAGE = ROWS * 64;
    constexpr int B_STAGE = 64 * 128;
    constexpr int STAGE = A_STAGE + B_STAGE;
    constexpr int A_CP = (MBW >= 2) ? MBW / 2 : 1;   // A copies per wave per step (MBW 1: waves 2,3 repeat 0,1)
    constexpr int B_CP = 8 / NW;
    constexpr int PAIR_CP = MBW * 4 / NW + 2 * B_CP;   // pair instantiations: copies per wave per pair of steps
    constexpr int STEP_CP = A_CP + B_CP;
    __shared__ __attribute__((aligned(1024))) unsigned char smem[NS * STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wc = tid >> 6;                   // wave of the workgroup: which copies it issues
    const int w = wc & 3;                      // its 32 columns of the tile
    const int kp = KP ? wc >> 2 : 0;           // its step of every pair
    const int c32 = lane & 31, h = lane >> 5;

    const uint32_t M = args.M, N = args.N, K = args.K, f = args.splitK;
    const uint32_t loopsM = ceil_div(M, 128u), loopsN = N / 128u, kTiles = ceil_div(K, 256u);
    uint32_t mi, ni, kIdx, slice;
    const uint32_t task = splitk_launch_task(args.sched.off, args.sched.dir, loopsM, loopsN, f, blockIdx.x);
    splitk_block_coord(args.sched.off, args.sched.dir, loopsM, loopsN, kTiles, f, task, mi, ni, kIdx, slice);
    const uint32_t kBeg = kIdx * 256u;
    const uint32_t nsteps = splitk_actual_k(K, 256u, f, slice) / 64u;
    const uint32_t row0 = mi * 128u, colT = ni * 128u;
    const uint32_t rowsValid = umin(128u, M - row0);
    const uint32_t tile = mi * loopsN + ni;

    const int64_t lda = args.lda, ldb = args.ldb;
    const unsigned char *Ag = (const unsigned char *)args.a[0] + (size_t)row0 * lda + kBeg;
    const unsigned char *Bg = TB ? (const unsigned char *)args.b + (size_t)colT * ldb + kBeg
                                 : (const unsigned char *)args.b + (size_t)kBeg * ldb + colT;
    // B copy j of a step: [k][n] covers k rows 8j..8j+7 (lane -> row 8j + lane/8, slot lane&7 holds chunk slot ^ (((row>>1)&3)<<1));
    // [n][k] covers tile columns 16j..16j+15, one 64-byte row of k each, laid out like A
    auto copy_b = [&](const unsigned char *Bgk, unsigned char *sb) {
#pragma unroll
        for (int jj = 0; jj < B_CP; ++jj) {
            const int j = wc + NW * jj;
            if constexpr (TB) {
                const uint32_t lrow = 16 * j + (lane >> 2);
                dma16(Bgk + (size_t)lrow * ldb + (((lane & 3) ^ ((lane >> 4) & 3)) * 16), sb + j * 1024);
            } else {
                const int row = 8 * j + (lane >> 3);
                dma16_stream(Bgk + (size_t)row * ldb + (((lane & 7) ^ (((row >> 1) & 3) << 1)) * 16), sb + j * 1024);
            }
        }
    };

    // A: copy j covers tile rows 16j..16j+15; lane -> row 16j + lane/4, LDS chunk slot lane&3 holds k chunk slot^swz
    // Every workgroup of a k slice reads the same 64-byte column of A at the same step, and the rows of A are a
    // power of two apart, so those reads would all queue at one L2 channel.  Each workgroup therefore walks its k
    // steps from a different starting point (integer sums do not care about the order); workgroups that share an
    // XCD (blockIdx mod 8) get consecutive starting points, which spreads them over the channels.
    const uint32_t rot = AP ? 2u * ((blockIdx.x >> 3) % (nsteps / 2u)) : (blockIdx.x >> 3) % nsteps;
    auto issue = [&](uint32_t st, uint32_t step) {
        unsigned char *sa = smem + st * STAGE, *sb = sa + A_STAGE;
        const uint32_t kt = step + rot < nsteps ? step + rot : step + rot - nsteps;
        const unsigned char *Agk = Ag + (size_t)kt * 64;
        const unsigned char *Bgk = TB ? Bg + (size_t)kt * 64 : Bg + (size_t)kt * 64 * ldb;
#pragma unroll
        for (int jj = 0; jj < A_CP; ++jj) {
            const int j = (MBW == 1) ? (w & 1) : w + NW * jj;
            const uint32_t lrow = 16 * j + (lane >> 2);
            const uint32_t srow = umin(lrow, rowsValid - 1u);
            dma16(Agk + (size_t)srow * lda + (((lane & 3) ^ ((lane >> 4) & 3)) * 16), sa + j * 1024);
        }
        copy_b(Bgk, sb);
    };
    // AP: steps `step` and `step + 1` (st even).  The group's area holds the pair of A first (rows of 128 bytes: copy j covers
    // rows 8j..8j+7, lane -> row 8j + lane/8, chunk slot lane&7 holds k chunk slot ^ ((row>>1)&7)), then B of the two steps.
    auto issue_pair = [&](uint32_t st, uint32_t step) {
        unsigned char *sp = smem + st * STAGE;
        const uint32_t kt = step + rot < nsteps ? step + rot : step + rot - nsteps;
        const unsigned char *Agk = Ag + (size_t)kt * 64;
#pragma unroll
        for (int jj = 0; jj < MBW * 4 / NW; ++jj) {
            const int j = wc + NW * jj;
            const uint32_t lrow = 8 * j + (lane >> 3);
            const uint32_t srow = umin(lrow, rowsValid - 1u);
            dma16(Agk + (size_t)srow * lda + (((lane & 7) ^ ((lrow >> 1) & 7)) * 16), sp + j * 1024);
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const unsigned char *Bgk = TB ? Bg + (size_t)(kt + t) * 64 : Bg + (size_t)(kt + t) * 64 * ldb;
            copy_b(Bgk, sp + 2 * A_STAGE + t * B_STAGE);
        }
    };
    auto issue_more = [&](uint32_t &issuedSteps) {   // the next step, or the next pair of steps
        if constexpr (AP) {
            issue_pair(issuedSteps % NS, issuedSteps);
            issuedSteps += 2;
        } else {
            issue(issuedSteps % NS, issuedSteps);
            ++issuedSteps;
        }
    };

    // ---- everything the epilogue reads is requested while the stream is still in flight ---------
    // The tail of this kernel is a chain of memory round trips (publish, count, fetch the other slices); bias,
    // scales and the peers' values of the tile's first 32-row block with kept rows would add two more, so every
    // slice asks for them as soon as its last copy of B is on its way (request_epilogue_operands below) and holds
    // them in registers (the peers of a decode tile are a few KiB).  A wave can have 63 memory operations
    // outstanding and this code runs once, so it is kept short: one load per 32-row block for the per-token
    // scales (lane l fetches row l of the block; the lanes pick their rows from each other in the epilogue), and
    // peer loads only for the register slots whose rows can be kept rows.
    //
    // acc[mb][r] is element (lrow, lcol) with lrow = mb*32 + slot_row(r) + 4h, lcol = w*32 + c32.  Inside block mb
    // the kept rows are the local rows [kLo, kHi) (wave-uniform); lane and slot then decide with one unsigned
    // compare, (slot_row(r) + rel) < kHi - kLo with rel = 4h - kLo, and a peer offset is base + slot_row(r) * pitch.
    const uint32_t lcol = w * 32 + c32;
    const uint32_t gcol = colT + lcol;
    const uint32_t keptEnd = args.keptBegin + args.keptRows;
    const uint64_t peerBytes = (uint64_t)(args.peerRowOffset + args.keptRows) * args.peerLd * 4;
    const int peerRange = peerBytes > 0x7fffffffull ? 0x7fffffff : (int)peerBytes;
    const uint32_t peerPitch = (uint32_t)args.peerLd * 4u;
    constexpr uint32_t OUT_OF_RANGE = 0x7fffffffu;   // a buffer load at this offset touches no memory and reads zero
    auto slot_row = [](int r) { return (uint32_t)((r >> 2) * 8 + (r & 3)); };
    struct KeptRows { uint32_t lo, n, rel, base; };   // of one 32-row block
    auto kept_rows = [&](uint32_t mb) {
        const uint32_t blk0 = row0 + mb * 32, blkEnd = row0 + umin(rowsValid, mb * 32 + 32);
        const uint32_t lo = args.keptBegin > blk0 ? args.keptBegin : blk0, hi = umin(keptEnd, blkEnd);
        KeptRows k;
        k.lo = lo - blk0;
        k.n = hi > lo ? hi - lo : 0u;
        k.rel = 4u * h - k.lo;
        k.base = ((uint32_t)(args.peerRowOffset + blk0 - args.keptBegin) + 4u * h) * peerPitch + gcol * 4u;
        return k;
    };
    auto slot_active = [&](const KeptRows &k, int r) { return slot_row(r) < k.lo + k.n && slot_row(r) + 4u >= k.lo; };   // uniform
    auto lane_kept = [&](const KeptRows &k, int r) { return slot_row(r) + k.rel < k.n; };
    // PB peers of one block (eight; four where two waves share a SIMD's registers), slot by slot: one uniform test, then
    // the loads back to back
    auto fetch_peers = [&](const KeptRows &k, uint32_t p0, float (&pv)[PB][16]) {
        __amdgpu_buffer_rsrc_t prs[PB];   // a peer that does not exist gets an empty range
#pragma unroll
        for (int q = 0; q < PB; ++q) {
            const bool use = p0 + q < args.nPeers && k.n != 0;
            prs[q] = __builtin_amdgcn_make_buffer_rsrc((void *)args.peers[use ? p0 + q : 0], 0, use ? peerRange : 0, 0x00020000);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            if (k.n != 0 && slot_active(k, r)) {
                const uint32_t off = lane_kept(k, r) ? k.base + slot_row(r) * peerPitch : OUT_OF_RANGE;
#pragma unroll
                for (int q = 0; q < PB; ++q)
                    pv[q][r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(prs[q], off, 0, 2 /* streaming */));
            } else {
#pragma unroll
                for (int q = 0; q < PB; ++q) pv[q][r] = 0.0f;
            }
        }
    };
    uint32_t mbK = 0;   // first 32-row block of the tile with kept rows (none: block 0, which then has nothing to fetch)
#pragma unroll
    for (int mb = MBW - 1; mb >= 0; --mb)
        if (kept_rows(mb).n != 0) mbK = mb;
    int bv;
    float sN;
    float sMrow[MBW];
    float pv0[PB][16];
    auto request_epilogue_operands = [&]() {
        bv = args.bias ? args.bias[gcol] : 0;
        sN = args.scaleN[gcol];
#pragma unroll
        for (int mb = 0; mb < MBW; ++mb) {
            const uint32_t lrow = mb * 32 + c32;
            sMrow[mb] = lrow < rowsValid ? args.scaleM[row0 + lrow] : 0.0f;
        }
        fetch_peers(kept_rows(mbK), 0, pv0);
    };

    v16i acc[MBW];
#pragma unroll
    for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mb][r] = 0;

    const uint32_t a_lds = c32 * 64;
    const uint32_t a_sw = (c32 >> 2) & 3;
    const uint32_t ap_lds = c32 * 128, ap_sw = (c32 >> 1) & 7;   // pair area: rows of 128 bytes
    // transpose read of this wave's 32 columns (two 16-column chunks, one per half of a 32-lane group)
    const int ti16 = lane & 15, tch = (lane >> 4) & 1, trow = ti16 >> 1, thalf = ti16 & 1;
    const uint32_t b_lds = (16 * h + trow) * 128 + (((2 * w + tch) ^ (((trow >> 1) & 3) << 1)) * 16) + thalf * 8;
    const uint32_t bt_lds = (w * 32 + c32) * 64;   // [n][k] stage: the row of this lane's column (chunk swizzle a_sw, as for A)

    // The loop is paced by latencies, not by bandwidth (one wave per SIMD: barrier, LDS round trip and the MFMA
    // chain of a step add up), so G steps share one barrier and one LDS round trip.  `issued` counts the steps
    // whose copies have been issued; before a group is read, the copies of later steps may stay in flight.
    const uint32_t ahead = umin(nsteps, (uint32_t)(NS - G));
    uint32_t issued = 0;
    while (issued < ahead) issue_more(issued);
    auto wait_steps_in_flight = [&](uint32_t n) {
        if constexpr (AP) {   // whole pairs
            switch (n / 2) {
                case 0: CATCOC_WAIT_VMCNT(0); break;
                case 1: CATCOC_WAIT_VMCNT(1 * PAIR_CP); break;
                case 2: CATCOC_WAIT_VMCNT(2 * PAIR_CP); break;
                case 3: CATCOC_WAIT_VMCNT(3 * PAIR_CP); break;
                default: CATCOC_WAIT_VMCNT(4 * PAIR_CP); break;
            }
            return;
        }
        switch (n) {
            case 0: CATCOC_WAIT_VMCNT(0); break;
            case 1: CATCOC_WAIT_VMCNT(1 * STEP_CP); break;
            case 2: CATCOC_WAIT_VMCNT(2 * STEP_CP); break;
            case 3: CATCOC_WAIT_VMCNT(3 * STEP_CP); break;
            case 4: CATCOC_WAIT_VMCNT(4 * STEP_CP); break;
            case 5: CATCOC_WAIT_VMCNT(5 * STEP_CP); break;
            case 6: CATCOC_WAIT_VMCNT(6 * STEP_CP); break;
            case 7: CATCOC_WAIT_VMCNT(7 * STEP_CP); break;
            default: CATCOC_WAIT_VMCNT(8 * STEP_CP); break;
        }
    };
    static_assert(NS - G <= 8 && NS >= 2 * G && NS % G == 0, "ring geometry");
    auto k_group = [&](uint32_t s, auto count) {   // steps s .. s + GG - 1
        constexpr int GG = decltype(count)::value;
        wait_steps_in_flight(issued - (s + GG));
        barrier_keep_vmem();
        // every wave has left the steps before s: their stages take the next copies
        while (issued < nsteps && issued < s + NS) issue_more(issued);
        // all fragment reads of the group first, then the MFMAs: one LDS round trip per group (left to itself the
        // compiler reuses two fragment registers and serialises them)
        constexpr int GJ = KP ? 1 : GG;   // steps of the group this wave multiplies (KP: the one of its parity)
        v4i bf[GJ][2], af[GJ][2][MBW];
#pragma unroll
        for (int jj = 0; jj < GJ; ++jj) {
            const int j = KP ? kp : jj;
            // (AP: the group's area starts at the stage of its first step: the pair of A, then B of step j)
            const unsigned char *sa = AP ? smem + (s % NS) * STAGE : smem + ((s + j) % NS) * STAGE;
            const unsigned char *sb = AP ? sa + 2 * A_STAGE + j * B_STAGE : sa + A_STAGE;
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                if constexpr (TB) {
                    bf[jj][kk] = *(const v4i *)(sb + bt_lds + (((2 * kk + h) ^ a_sw) * 16));
                } else {
                    const unsigned char *p = sb + b_lds + kk * 32 * 128;
                    const v2i t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)p);
                    const v2i t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)(p + 8 * 128));
                    bf[jj][kk] = v4i{t0.x, t0.y, t1.x, t1.y};
                }
#pragma unroll
                for (int mb = 0; mb < MBW; ++mb) {
                    if constexpr (AP) af[jj][kk][mb] = *(const v4i *)(sa + ap_lds + mb * 32 * 128 + (((4 * j + 2 * kk + h) ^ ap_sw) * 16));
                    else af[jj][kk][mb] = *(const v4i *)(sa + a_lds + mb * 32 * 64 + (((2 * kk + h) ^ a_sw) * 16));
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int jj = 0; jj < GJ; ++jj)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                for (int mb = 0; mb < MBW; ++mb) acc[mb] = mfma32<DT_I8>(af[jj][kk][mb], bf[jj][kk], acc[mb]);
        __builtin_amdgcn_sched_barrier(0);
    };
    // The groups that still issue copies, then the request for the epilogue's operands (younger than every copy,
    // so the waits of the remaining groups, which count outstanding operations, stay on the safe side), then the
    // rest; steps left over by a k slice that is not a multiple of G go one at a time.
    uint32_t s = 0;
    for (; issued < nsteps && s + G <= nsteps; s += G) k_group(s, std::integral_constant<int, G>{});
    if (!KP || kp == 0) request_epilogue_operands();
    for (; s + G <= nsteps; s += G) k_group(s, std::integral_constant<int, G>{});
    if constexpr (!AP) {   // (with pairs the host guarantees whole groups)
        for (; s < nsteps; ++s) k_group(s, std::integral_constant<int, 1>{});
    }

    if constexpr (KP) {   // the two step parities meet: waves 4-7 hand their sums to waves 0-3 and leave
        CATCOC_WAIT_VMCNT(0);
        __syncthreads();   // every wave has left the ring
        int *meet = (int *)smem;   // [4][MBW][16][64]
        if (kp == 1) {
#pragma unroll
            for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) meet[((w * MBW + mb) * 16 + r) * 64 + lane] = acc[mb][r];
        }
        __syncthreads();
        if (kp == 1) return;
#pragma unroll
        for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][r] += meet[((w * MBW + mb) * 16 + r) * 64 + lane];
    }

    // ---- k slices meet -------------------------------------------------------------
    long long csumOthers = 0;   // what the other slices hold of the groups that did not travel (checksums only)
    if (f > 1) {
        // Partial tiles travel through memory at device scope (cache policy sc1: written through / read past
        // the XCD-local L2), as ordinary buffer accesses so that the loads of a slice are issued together.  Inside
        // the workspace a tile is kept in register order: int32 index ((mb*4 + g)*256 + thread)*4 + j holds register
        // r = 4g + j of block mb, so every access is 16 bytes per lane and 1 KiB per wave.  Groups of rows past the
        // end of A are neither written nor read.
        constexpr int DEVICE_SCOPE = 16;   // sc1
        const size_t tileBytes = 128 * 128 * 4;
        // A group of eight rows travels when it has rows of A and somebody will look at them: kept rows (the output), or
        // every row when the caller asked for a dump of the accumulators.  The partials of the other groups stay where
        // they are: at M = 128 with 16 kept rows a workgroup publishes 8 KiB instead of 64, and the last slice fetches
        // 24 KiB instead of 192.  A checksum needs only their sum, and sums of sums are exact: every lane adds up what
        // it holds of those groups and the eight bytes travel in the place of the first group that stays behind.
        // (Tiles of up to 32 rows have four groups at most: there every row travels when checksums are asked for.)
        const bool allRows = args.accDump != nullptr || (MBW == 1 && args.checksum != nullptr);
        auto group_valid = [&](int mb, int g) {   // wave-uniform
            const uint32_t g0 = (uint32_t)(mb * 32 + g * 8);
            if (g0 >= rowsValid) return false;
            return allRows || (row0 + g0 < keptEnd && row0 + g0 + 8u > args.keptBegin);
        };
        const __amdgpu_buffer_rsrc_t mine = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(args.skPart + ((size_t)slice * loopsM * loopsN + tile) * (128 * 128)), 0, (int)tileBytes, 0x00020000);
        int sumSlot = -1;   // first group with rows of A that does not travel (wave-uniform)
        long long behind = 0;
        if (MBW >= 2 && args.checksum != nullptr) {
#pragma unroll
            for (int mb = MBW - 1; mb >= 0; --mb)
#pragma unroll
                for (int g = 3; g >= 0; --g)
                    if ((uint32_t)(mb * 32 + g * 8) < rowsValid && !group_valid(mb, g)) {
                        sumSlot = mb * 4 + g;
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            behind += (uint32_t)(mb * 32 + g * 8 + j) + 4u * h < rowsValid ? acc[mb][4 * g + j] : 0;
                    }
            if (sumSlot >= 0) {
                const v2i sv = {(int)(uint32_t)(unsigned long long)behind, (int)(uint32_t)((unsigned long long)behind >> 32)};
                __builtin_amdgcn_raw_buffer_store_b64(sv, mine, (sumSlot * 256 + tid) * 16, 0, DEVICE_SCOPE);
            }
        }
#pragma unroll
        for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                if (group_valid(mb, g)) {
                    const v4i iv = {acc[mb][4 * g], acc[mb][4 * g + 1], acc[mb][4 * g + 2], acc[mb][4 * g + 3]};
                    __builtin_amdgcn_raw_buffer_store_b128(iv, mine, ((mb * 4 + g) * 256 + tid) * 16, 0, DEVICE_SCOPE);
                }
        // once the stores are acknowledged the slice may be counted
        CATCOC_WAIT_VMCNT(0);
        __syncthreads();
        volatile uint32_t *flag = (volatile uint32_t *)smem;
        if (tid == 0) *flag = __hip_atomic_fetch_add(args.skCount + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*flag != f - 1u) return;
        if (tid == 0) __hip_atomic_store(args.skCount + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // the other slices' partials: every 32-row block of up to QG slices per round trip
        const int32_t *tile0 = args.skPart + (size_t)tile * (128 * 128);
        const size_t sliceStride = (size_t)loopsM * loopsN * (128 * 128);
        constexpr int QG = (KP && MBW == 4) ? 1 : 3;   // (two waves per SIMD have half the registers each)
        for (uint32_t o0 = 0; o0 + 1 < f; o0 += QG) {
            v4i pv[QG][MBW][4];
            v2i sums[QG];
#pragma unroll
            for (int q = 0; q < QG; ++q) {
                const uint32_t o = o0 + q;                       // o-th of the f - 1 other slices
                const bool use = o + 1 < f;
                const uint32_t sl = o < slice ? o : o + 1;
                const __amdgpu_buffer_rsrc_t other = __builtin_amdgcn_make_buffer_rsrc(
                    (void *)(tile0 + (use ? sl : slice) * sliceStride), 0, use ? (int)tileBytes : 0, 0x00020000);
                sums[q] = v2i{0, 0};
                if (use && sumSlot >= 0) sums[q] = __builtin_amdgcn_raw_buffer_load_b64(other, (sumSlot * 256 + tid) * 16, 0, DEVICE_SCOPE);
#pragma unroll
                for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        pv[q][mb][g] = v4i{0, 0, 0, 0};
                        if (use && group_valid(mb, g))
                            pv[q][mb][g] = __builtin_amdgcn_raw_buffer_load_b128(other, ((mb * 4 + g) * 256 + tid) * 16, 0, DEVICE_SCOPE);
                    }
            }
#pragma unroll
            for (int q = 0; q < QG; ++q) {
                csumOthers += (long long)(((unsigned long long)(uint32_t)sums[q].y << 32) | (uint32_t)sums[q].x);
#pragma unroll
                for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        acc[mb][4 * g] += pv[q][mb][g].x;
                        acc[mb][4 * g + 1] += pv[q][mb][g].y;
                        acc[mb][4 * g + 2] += pv[q][mb][g].z;
                        acc[mb][4 * g + 3] += pv[q][mb][g].w;
                    }
            }
        }
    }

    // ---- epilogue on the rows that exist -----------------------------------------------
    // First a cheap pass over every 32-row block: bias, dumps, checksum of the rows that are not kept.  Then ONE loop
    // body, run once per block with kept rows (a run-time loop: this code executes once per tile, and unrolled per
    // block it was several times the size of the instruction cache): the block's registers are selected, dequantised,
    // the peers added in slot order eight at a time (the first block's first eight are in registers already, the
    // others are fetched into the same registers in one round trip) and the 16-bit rows stored.
    // GF_REDUCE_INT32 (the reference's order, quant_matmul_reduce_scatter.hpp:285-351): the peers hold int32 partials that join
    // the accumulators before the dequantisation, and c_accum receives the reduced block
    const bool redI32 = (args.flags & GF_REDUCE_INT32) != 0;
    long long csum = csumOthers;
#pragma unroll
    for (int mb = 0; mb < MBW; ++mb) {
        if ((uint32_t)mb * 32 >= rowsValid) break;
        const KeptRows k = kept_rows(mb);
        const uint32_t vrel = mb * 32 + 4u * h;   // slot r is a row of A when slot_row(r) + vrel < rowsValid
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mb][r] += bv;
        if (args.checksum != nullptr) {   // rows that are not kept are only summed, and only on request
#pragma unroll
            for (int r = 0; r < 16; ++r) csum += (slot_row(r) + vrel < rowsValid && !lane_kept(k, r)) ? acc[mb][r] : 0;
        }
        if (args.accDump) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (slot_row(r) + vrel < rowsValid) ((int32_t *)args.accDump)[(size_t)(row0 + vrel + slot_row(r)) * N + gcol] = acc[mb][r];
        }
        if (k.n != 0 && args.cAccum && !redI32) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (lane_kept(k, r)) args.cAccum[(size_t)(row0 + vrel + slot_row(r) - args.keptBegin) * N + gcol] = acc[mb][r];
        }
    }
#pragma nounroll
    for (uint32_t t = mbK; t < (uint32_t)MBW; ++t) {
        const KeptRows k = kept_rows(t);
        if (k.n == 0) continue;
        // this block's accumulators and per-token scale, picked with uniform selects
        int iv[16];
        float sMt = sMrow[0];
#pragma unroll
        for (int r = 0; r < 16; ++r) iv[r] = acc[0][r];
#pragma unroll
        for (int mb = 1; mb < MBW; ++mb)
            if (t == (uint32_t)mb) {
                sMt = sMrow[mb];
#pragma unroll
                for (int r = 0; r < 16; ++r) iv[r] = acc[mb][r];
            }
        float v[16];
        if (redI32) {
            for (uint32_t p0 = 0; p0 < args.nPeers; p0 += PB) {
                if (t != mbK || p0 != 0) fetch_peers(k, p0, pv0);
#pragma unroll
                for (int q = 0; q < PB; ++q)
                    if (p0 + q < args.nPeers) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) iv[r] += f2i(pv0[q][r]);   // (the loads carry bit patterns)
                    }
            }
            if (args.cAccum) {
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (lane_kept(k, r)) args.cAccum[(size_t)(row0 + t * 32 + 4u * h + slot_row(r) - args.keptBegin) * N + gcol] = iv[r];
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] = __fmul_rn(__fmul_rn((float)iv[r], sN), __shfl(sMt, slot_row(r) + 4 * h, 64));
        for (uint32_t p0 = 0; p0 < (redI32 ? 0u : args.nPeers); p0 += PB) {
            if (t != mbK || p0 != 0) fetch_peers(k, p0, pv0);
#pragma unroll
            for (int q = 0; q < PB; ++q)
                if (p0 + q < args.nPeers) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) v[r] = __fadd_rn(v[r], pv0[q][r]);
                }
        }
        // signed: the block may start above the first kept row (only kept lanes dereference)
        unsigned short *drow = (unsigned short *)args.d + ((int64_t)(row0 + t * 32 + 4u * h) - (int64_t)args.keptBegin) * args.ldd + gcol;
#pragma unroll
        for (int r = 0; r < 16; ++r)
            if (lane_kept(k, r)) drow[(int64_t)slot_row(r) * args.ldd] = (unsigned short)f32_to_out16(v[r], args.outDtype);
    }
    if (args.checksum != nullptr) {
        long long *red = (long long *)smem + 8;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) csum += __shfl_xor(csum, o, 64);
        __syncthreads();
        if (lane == 0) red[w] = csum;
        __syncthreads();
        if (tid == 0) ((long long *)args.checksum)[tile] = red[0] + red[1] + red[2] + red[3];
    }
}

}  // namespace catcoc
