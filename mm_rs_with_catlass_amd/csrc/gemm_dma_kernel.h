// Full-tile fast path of the fused GEMM for gfx950: A and B tiles stream from
// global memory straight into LDS (no VGPR staging) three k-steps ahead of the
// MFMAs, and the row-major B tile is transposed on the way out of LDS with the
// transpose-read instruction, so the main loop issues almost nothing but LDS reads
// and MFMAs.  The kept tiles' peer partials are staged through the same LDS
// buffers, again without VGPRs, which keeps a deep queue of HBM reads in flight
// while the accumulators stay in registers.
//
// Same per-tile contract as gemm_fused_kernel (see gemm_fused_kernel.h); used when
// every tile is full, A is [rows,K] and B is [K,N], both row-major.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_fused_kernel.h"

namespace catcoc {

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

// LDS layouts per stage (k step = 64 bytes of K):
//   A: [row][4 x 16-byte k chunks], chunk slot = chunk ^ ((row >> 2) & 3)            (as in gemm_fused_kernel)
//   B: raw row-major [k row][16 x 16-byte column chunks] for int8 (64 rows x 256 B),
//      column chunk slot = chunk ^ ((k row & 7) << 1); the swizzle is applied on the global side of
//      the copy, and makes the 8-row x 16-column transpose reads of a half-wave hit all 64 banks once.
//   fp16/bf16: 32 k rows x 512 B, 32 chunks per row, slot = chunk ^ ((k row & 3) << 1 ... see b_slot16)
//
// Geometries (MB = 32-row blocks per wave, WM = wave rows; every wave is 128 columns wide, two wave columns):
//   MB 2, WM 2 -> 128x256 tile, 4 waves of 64x128, 3 stages (72 KiB LDS, two workgroups per CU);
//   MB 2, WM 4 -> 256x256 tile, 8 waves of 64x128 (128 KiB LDS, one workgroup per CU): half the L2 -> LDS
//                 traffic per MAC;
//   MB 4, WM 2 -> 256x256 tile, 4 waves of 128x128, one wave per SIMD: also a third less LDS read traffic
//                 per MFMA, which is what bounds the 64x128 waves.
template <uint32_t DT, int MB, int WM>
__global__ void __launch_bounds__(128 * WM, (MB == 4) ? 1 : 2) gemm_dma_kernel(const GemmArgs args)
{
    static_assert(DT == DT_I8, "transpose-read path is written for int8 operands");
    static_assert((MB == 2 && (WM == 2 || WM == 4)) || (MB == 4 && WM == 2), "supported geometries");
    using Acc = typename AccOf<DT>::type;
    constexpr int NW = 2 * WM;          // waves
    constexpr int BM = 32 * MB * WM;
    constexpr int NS = (BM == 256) ? 4 : 3;
    constexpr int A_STAGE = BM * 64;
    constexpr int B_STAGE = 64 * 256;
    constexpr int A_DMA = BM / 16 / NW;  // 1 KiB copies per wave per stage
    constexpr int B_DMA = 16 / NW;
    constexpr int STEP_DMA = A_DMA + B_DMA;

    // One LDS pool, carved by constant offsets:
    //   BM = 128: three A stages (8 KiB each), then three B stages (16 KiB each)            = 72 KiB
    //   BM = 256: two A pair buffers (32 KiB each), then four B stages (16 KiB each)         = 128 KiB
    // After the main loop the pool is reused as per-wave staging rings for the peers' partials.
    constexpr int NSA4 = 4, NSB4 = 4;   // BM = 256: A area = two pair buffers of 2 x 16 KiB
    constexpr int LDS_BYTES = (BM == 256) ? (NSA4 * A_STAGE + NSB4 * B_STAGE) : 3 * (A_STAGE + B_STAGE);
    __shared__ __attribute__((aligned(1024))) unsigned char smem[LDS_BYTES];
    unsigned char *const smem4 = smem;
    unsigned char *const sA0 = smem, *const sA1 = smem + A_STAGE, *const sA2 = smem + 2 * A_STAGE;        // BM = 128
    unsigned char *const sB0 = smem + 3 * A_STAGE, *const sB1 = sB0 + B_STAGE, *const sB2 = sB0 + 2 * B_STAGE;  // BM = 128

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = tid >> 6;
    const int wm = w >> 1, wn = w & 1;
    const int c32 = lane & 31, h = lane >> 5;

    const SchedParams &sp = args.sched;
    const uint32_t task = launch_order_task(sp, blockIdx.x, (args.flags & GF_LINEAR_ORDER) != 0, args.keptRank);
    TileInfo ti;
    if (!task_tile(sp, task, ti)) return;

    const int64_t ldaB = args.lda, ldbB = args.ldb;  // int8: elements == bytes
    const bool gather = sp.op == OP_ALLGATHER;
    const unsigned char *Ag = (const unsigned char *)args.a[gather ? ti.targetRank : 0] +
                              (int64_t)(gather ? ti.rowInRank : ti.row) * ldaB;
    const unsigned char *Bg = (const unsigned char *)args.b + ti.col;

    // ---- copy descriptors ---------------------------------------------------
    // A: copy j covers rows 16j..16j+15; lane -> row 16j + lane/4, LDS chunk slot lane&3 holds k chunk slot^swz
    const uint32_t a_goff = (uint32_t)(lane >> 2) * (uint32_t)ldaB + (((lane & 3) ^ ((lane >> 4) & 3)) * 16);
    // B: copy j covers k rows 4j..4j+3; lane -> row 4j + lane/16, LDS slot lane&15 holds column chunk slot^((row&7)<<1)
    auto issue_a = [&](unsigned char *sa, uint32_t kt) {
        const unsigned char *Agk = Ag + (size_t)kt * 64;
#pragma unroll
        for (int jj = 0; jj < A_DMA; ++jj) {
            const int j = w + NW * jj;
            dma16(Agk + (size_t)(16 * j) * ldaB + a_goff, sa + j * 1024);
        }
    };
    auto issue_b = [&](unsigned char *sb, uint32_t kt) {
        const unsigned char *Bgk = Bg + (size_t)kt * 64 * ldbB;
#pragma unroll
        for (int jj = 0; jj < B_DMA; ++jj) {
            const int j = w + NW * jj;
            const int row = 4 * j + (lane >> 4);
            dma16(Bgk + (size_t)row * ldbB + (((lane & 15) ^ ((row & 7) << 1)) * 16), sb + j * 1024);
        }
    };
    auto issue = [&](unsigned char *sa, unsigned char *sb, uint32_t kt) {
        issue_a(sa, kt);
        issue_b(sb, kt);
    };

    Acc acc[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][nb][r] = 0;

    // fragment addresses
    const uint32_t a_lds = (wm * 32 * MB + c32) * 64;
    const uint32_t a_sw = (c32 >> 2) & 3;
    // transpose read: within a 16-lane group, lane i supplies 8 bytes of k row (i>>1), column half (i&1)
    // of a 16-column chunk, and receives column i of the chunk for 8 consecutive k rows.
    const int ti16 = lane & 15, tch = (lane >> 4) & 1, trow = ti16 >> 1, thalf = ti16 & 1;
    uint32_t b_lds[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
        const int q = wn * 8 + nb * 2 + tch;
        b_lds[nb] = (16 * h + trow) * 256 + ((q ^ (2 * trow)) * 16) + thalf * 8;
    }

    auto load_a = [&](v4i (&af)[MB], const unsigned char *sa, int kk) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) af[mb] = *(const v4i *)(sa + a_lds + mb * 32 * 64 + (((2 * kk + h) ^ a_sw) * 16));
    };
    auto load_b = [&](v4i (&bf)[4], const unsigned char *sb, int kk) {
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            const unsigned char *p = sb + b_lds[nb] + kk * 32 * 256;
            const v2i t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)p);
            const v2i t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)(p + 8 * 256));
            bf[nb] = v4i{t0.x, t0.y, t1.x, t1.y};
        }
    };
    auto mma = [&](const v4i (&af)[MB], const v4i (&bf)[4]) {
        if (args.debug & 2) return;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) acc[mb][nb] = mfma32<DT>(af[mb], bf[nb], acc[mb][nb]);
    };

    const uint32_t nk = args.K / 64;
    if constexpr (NS == 3) {
        // ---- 3 stages: copies run two k steps ahead; fragments are read right after the barrier ----
        auto compute = [&](const unsigned char *sa, const unsigned char *sb) {
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                v4i af[MB], bf[4];
                load_a(af, sa, kk);
                load_b(bf, sb, kk);
                mma(af, bf);
            }
        };
        issue(sA0, sB0, 0);
        if (nk > 1) issue(sA1, sB1, 1);
        uint32_t kt = 0;
        // FULL: two more steps exist behind this one, so every condition is known to hold
#define CATCOC_STEP(FULL, SA, SB, NA, NB)                                      \
    {                                                                          \
        if (FULL || kt + 1 < nk) CATCOC_WAIT_VMCNT(STEP_DMA);                  \
        else CATCOC_WAIT_VMCNT(0);                                             \
        barrier_keep_vmem();                                                   \
        if (FULL || kt + 2 < nk) issue(NA, NB, kt + 2);                        \
        compute(SA, SB);                                                       \
        ++kt;                                                                  \
    }
        while (kt + 5 <= nk) {   // steps kt, kt+1, kt+2 all have two successors
            CATCOC_STEP(1, sA0, sB0, sA2, sB2)
            CATCOC_STEP(1, sA1, sB1, sA0, sB0)
            CATCOC_STEP(1, sA2, sB2, sA1, sB1)
        }
        while (true) {
            if (kt >= nk) break;
            CATCOC_STEP(0, sA0, sB0, sA2, sB2)
            if (kt >= nk) break;
            CATCOC_STEP(0, sA1, sB1, sA0, sB0)
            if (kt >= nk) break;
            CATCOC_STEP(0, sA2, sB2, sA1, sB1)
        }
#undef CATCOC_STEP
    } else {
        // ---- 256x256 ---------------------------------------------------------------------------------
        // B: four 64-row stages, copies issued three steps ahead.  A: two "pair" buffers of 256 rows x 128
        // bytes (two k steps, whole 128-byte lines per row), pair q = steps 2q, 2q+1, issued at step 2q-2.
        // The MFMAs lag the fragment reads by half a step: after the barrier of step kt the fragments of
        // (kt, kk=0) are read while the MFMAs of (kt-1, kk=1) run, so LDS latency is never exposed and a
        // stage only has to have landed at its own barrier.
        // Issue order per wave: even step [B(kt+3): 2 copies, A pair (kt+2)/2: 4 copies], odd step [B(kt+3)].
        // At the barrier of an even step 2 copies may be in flight (B(kt+2)), at an odd step 8
        // (B(kt+1), B(kt+2), A pair (kt+1)/2+... issued at kt-1).
        constexpr int AP = 256 * 128;   // bytes of an A pair buffer
        static_assert(2 * AP == NSA4 * A_STAGE, "A pair buffers fill the A stage area");
        auto stAP = [&](uint32_t q) { return smem4 + (q & 1) * AP; };
        auto stB = [&](uint32_t step) { return smem4 + 2 * AP + (step & 3) * B_STAGE; };
        // pair copy j covers rows 8j..8j+7: lane -> row 8j + lane/8, slot lane&7 holds chunk slot ^ ((row>>1)&7)
        constexpr int APC = 32 / NW;   // pair copies per wave
        auto issue_ap = [&](uint32_t q) {
            const unsigned char *Agq = Ag + (size_t)q * 128;
            unsigned char *dst = stAP(q);
#pragma unroll
            for (int jj = 0; jj < APC; ++jj) {
                const int j = w + NW * jj;
                const int row = 8 * j + (lane >> 3);
                dma16(Agq + (size_t)row * ldaB + (((lane & 7) ^ ((row >> 1) & 7)) * 16), dst + j * 1024);
            }
        };
        const uint32_t ap_lds = (wm * 32 * MB + c32) * 128;
        const uint32_t ap_sw = (c32 >> 1) & 7;
        auto load_ap = [&](v4i (&af)[MB], uint32_t kt, int kk) {
            const unsigned char *sa = stAP(kt >> 1) + ap_lds + ((((kt & 1) * 4 + 2 * kk + h) ^ ap_sw) * 16);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) af[mb] = *(const v4i *)(sa + mb * 32 * 128);
        };
        auto issue_step = [&](uint32_t kt, bool guard) {
            if (args.debug & 1) return;
            if (!guard || kt + 3 < nk) issue_b(stB(kt + 3), kt + 3);
            if ((kt & 1) == 0 && (!guard || kt + 2 < nk)) issue_ap((kt + 2) >> 1);
        };
        v4i fa0[MB], fb0[4], fa1[MB], fb1[4];
        // prologue in steady-state order: B0, B1, pair 0, B2
        issue_b(stB(0), 0);
        if (nk > 1) issue_b(stB(1), 1);
        issue_ap(0);
        if (nk > 2) issue_b(stB(2), 2);
        // step 0 (peeled: no MFMAs pending yet)
        if (nk > 2) CATCOC_WAIT_VMCNT(B_DMA);
        else CATCOC_WAIT_VMCNT(0);
        barrier_keep_vmem();
        issue_step(0, true);
        load_ap(fa0, 0, 0);
        load_b(fb0, stB(0), 0);
        load_ap(fa1, 0, 1);
        load_b(fb1, stB(0), 1);
        __builtin_amdgcn_sched_barrier(0);
        mma(fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        auto compute = [&](uint32_t kt) {
            load_ap(fa0, kt, 0);
            load_b(fb0, stB(kt), 0);
            __builtin_amdgcn_sched_barrier(0);
            mma(fa1, fb1);      // second half of the previous step
            __builtin_amdgcn_sched_barrier(0);
            load_ap(fa1, kt, 1);
            load_b(fb1, stB(kt), 1);
            __builtin_amdgcn_sched_barrier(0);
            mma(fa0, fb0);
            __builtin_amdgcn_sched_barrier(0);
        };
        uint32_t kt = 1;
        for (; kt + 5 <= nk; kt += 2) {
            CATCOC_WAIT_VMCNT(2 * B_DMA + APC);   // odd step
            barrier_keep_vmem();
            issue_step(kt, false);
            compute(kt);
            CATCOC_WAIT_VMCNT(B_DMA);           // even step
            barrier_keep_vmem();
            issue_step(kt + 1, false);
            compute(kt + 1);
        }
        for (; kt < nk; ++kt) {   // tail: drain fully at every step
            CATCOC_WAIT_VMCNT(0);
            barrier_keep_vmem();
            issue_step(kt, true);
            compute(kt);
        }
        mma(fa1, fb1);
    }

    // ---- epilogue -----------------------------------------------------------------
    // acc[mb][nb][r] is element (row, col) of the tile with
    //   row = wm*32*MB + mb*32 + (r>>2)*8 + h*4 + (r&3),  col = wn*128 + nb*32 + c32
    const uint32_t col0 = wn * 128 + c32;       // + 32*nb
    const uint32_t gcol0 = ti.col + col0;
    const uint32_t row_base = wm * 32 * MB + h * 4;
    const bool kept = ti.row >= args.keptBegin && ti.row < args.keptBegin + args.keptRows;

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

    if (args.accDump != nullptr) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                int32_t *o = (int32_t *)args.accDump + (size_t)(ti.row + lrow) * args.N + gcol0;
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) {
                    const int iv = acc[mb][nb][r];
                    o[32 * nb] = iv;
                }
            }
    }

    float sN[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) sN[nb] = args.scaleN[gcol0 + 32 * nb];

    if (kept) {
        const uint32_t out_row0 = ti.row - args.keptBegin;
        if (args.cAccum != nullptr) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                    int32_t *o = args.cAccum + (size_t)(out_row0 + lrow) * args.N + gcol0;
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) {
                        const int iv = acc[mb][nb][r];
                        o[32 * nb] = iv;
                    }
                }
        }
        // dequantise in place: per-channel scale first, then per-token, each product rounded on its own
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                const float sM = args.scaleM[ti.row + lrow];
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) {
                    const int iv = acc[mb][nb][r];
                    acc[mb][nb][r] = f2i(__fmul_rn(__fmul_rn((float)iv, sN[nb]), sM));
                }
            }

        // peers, in slot order.  Every wave streams the peers' values for its own 64*MB/2... x 128 sub-tile
        // through a private 16 KiB LDS ring of four 4 KiB slots, with no barriers: a sub-batch is the 8 rows of
        // one accumulator row group (mb, r>>2) x the wave's 128 columns, copied as four 1 KiB pieces of
        // 2 rows x 512 bytes; three sub-batches are in flight while one is added.  Pieces of rows 4..7 are
        // stored with their 128-byte halves swapped so the two half-waves of a read hit different banks.
        const uint32_t nP = args.nPeers;
        if (nP != 0) {
            static_assert(NW * 16384 <= LDS_BYTES, "peer staging rings fit the pool");
            constexpr int SP = MB * 4;                 // sub-batches per peer; a multiple of the ring size
            const int64_t prow0 = args.peerRowOffset + out_row0 + wm * 32 * MB;
            unsigned char *const ring = smem + w * 16384;
            // lane -> row (lane>>5) of the piece, 16-byte chunk (lane&31) of the wave's 512-byte row segment
            const size_t src_lane = (size_t)(lane >> 5) * args.peerLd * 4 + (size_t)(ti.col + wn * 128) * 4;
            auto issue_sb = [&](uint32_t p, int s) {
                const int mb = s / 4, rq = s % 4;
                const unsigned char *src = (const unsigned char *)args.peers[p] +
                                           (size_t)(prow0 + mb * 32 + rq * 8) * args.peerLd * 4 + src_lane;
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    dma16(src + (size_t)(2 * c) * args.peerLd * 4 + (((lane & 31) ^ ((c >> 1) * 8)) * 16),
                          ring + rq * 4096 + c * 1024);
            };
            const uint32_t rd_lane = (2 * h) * 1024 + c32 * 4;
            const uint32_t Q = nP * SP;
            barrier_keep_vmem();   // every wave is done with the main loop's LDS reads
            issue_sb(0, 0);
            issue_sb(0, 1);
            issue_sb(0, 2);
            for (uint32_t p = 0; p < nP; ++p) {
#pragma unroll
                for (int s = 0; s < SP; ++s) {
                    const int mb = s / 4, rq = s % 4;
                    const uint32_t ahead = Q - 1 - (p * SP + s);
                    if (ahead >= 2) CATCOC_WAIT_VMCNT(8);
                    else if (ahead == 1) CATCOC_WAIT_VMCNT(4);
                    else CATCOC_WAIT_VMCNT(0);
                    if (s + 3 < SP) issue_sb(p, s + 3);
                    else if (p + 1 < nP) issue_sb(p + 1, s + 3 - SP);
                    const unsigned char *slot = ring + rq * 4096 + rd_lane;
#pragma unroll
                    for (int ri = 0; ri < 4; ++ri) {
                        const int r = rq * 4 + ri;
                        const unsigned char *rowp = slot + (ri >> 1) * 1024 + (ri & 1) * 512;
#pragma unroll
                        for (int nb = 0; nb < 4; ++nb) {
                            const float pv = *(const float *)(rowp + ((nb ^ h) * 128));
                            const int iv = acc[mb][nb][r];
                            acc[mb][nb][r] = f2i(__fadd_rn(i2f(iv), pv));
                        }
                    }
                }
            }
        }

        unsigned short *dptr = (unsigned short *)args.d + (size_t)out_row0 * args.ldd + gcol0;
        auto store_all = [&](auto cvt) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) {
                        const int iv = acc[mb][nb][r];
                        dptr[(size_t)lrow * args.ldd + 32 * nb] = (unsigned short)cvt(i2f(iv));
                    }
                }
        };
        if (args.outDtype == DT_BF16) store_all([](float f) { return f32_to_bf16_bits(f); });
        else store_all([](float f) { return f32_to_f16_bits(f); });
    } else if (args.flags & GF_OUTBOUND_STORE) {
        float *ob = (float *)args.outbound + (size_t)ti.wsRow * sp.n0 + col0;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                const float sM = args.scaleM[ti.row + lrow];
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) {
                    const int iv = acc[mb][nb][r];
                    __builtin_nontemporal_store(__fmul_rn(__fmul_rn((float)iv, sN[nb]), sM), ob + (size_t)lrow * sp.n0 + 32 * nb);
                }
            }
    } else if (args.checksum != nullptr) {
        __shared__ long long red[NW];
        long long si = 0;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                for (int r = 0; r < 16; ++r) si += acc[mb][nb][r];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) si += __shfl_xor(si, o, 64);
        if (lane == 0) red[w] = si;
        __syncthreads();
        if (tid == 0) {
            long long t = 0;
#pragma unroll
            for (int i = 0; i < NW; ++i) t += red[i];
            ((long long *)args.checksum)[task] = t;
        }
    }
}

}  // namespace catcoc
