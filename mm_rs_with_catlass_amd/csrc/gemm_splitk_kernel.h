// Skinny-M W8A8 GEMM for gfx950: few rows of A against a large B, which makes the
// launch HBM-bound on B.  The tile grid of SplitkMatmul is kept (tasks = tiles x k
// slices through SplitkGemmIdentityBlockSwizzle), with 128 x 128 tiles so that a
// decode-sized problem still spreads over every CU with a small split factor.
//
// A workgroup (4 waves) streams its k slice of B (64 k rows x 128 columns = 8 KiB per
// step) and of A straight into an 8-stage LDS ring with direct-to-LDS copies, seven
// steps ahead, so about 100 KiB per CU is in flight; every wave multiplies all rows
// of the tile by its own 32 columns.  Partial tiles of the k slices are written
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

#include "gemm_dma_kernel.h"

namespace catcoc {

// MBW: 32-row blocks staged per tile (1, 2 or 4); rows past the end of A are clamped to the last row
// on the way in and masked on the way out.
template <int MBW>
__global__ void __launch_bounds__(256, 1) gemm_splitk_kernel(const GemmArgs args)
{
    constexpr int NW = 4;
    constexpr int NS = 8;
    constexpr int ROWS = 32 * MBW;
    constexpr int A_STAGE = ROWS * 64;
    constexpr int B_STAGE = 64 * 128;
    constexpr int STAGE = A_STAGE + B_STAGE;
    constexpr int A_CP = (MBW >= 2) ? MBW / 2 : 1;   // A copies per wave per step (MBW 1: waves 2,3 repeat 0,1)
    constexpr int B_CP = 2;
    constexpr int STEP_CP = A_CP + B_CP;
    __shared__ __attribute__((aligned(1024))) unsigned char smem[NS * STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = tid >> 6;
    const int c32 = lane & 31, h = lane >> 5;

    const uint32_t M = args.M, N = args.N, K = args.K, f = args.splitK;
    const uint32_t loopsM = ceil_div(M, 128u), loopsN = N / 128u, kTiles = ceil_div(K, 256u);
    uint32_t mi, ni, kIdx, slice;
    splitk_block_coord(args.sched.off, args.sched.dir, loopsM, loopsN, kTiles, f, blockIdx.x, mi, ni, kIdx, slice);
    const uint32_t kBeg = kIdx * 256u;
    const uint32_t nsteps = splitk_actual_k(K, 256u, f, slice) / 64u;
    const uint32_t row0 = mi * 128u, colT = ni * 128u;
    const uint32_t rowsValid = umin(128u, M - row0);
    const uint32_t tile = mi * loopsN + ni;

    const int64_t lda = args.lda, ldb = args.ldb;
    const unsigned char *Ag = (const unsigned char *)args.a[0] + (size_t)row0 * lda + kBeg;
    const unsigned char *Bg = (const unsigned char *)args.b + (size_t)kBeg * ldb + colT;

    // A: copy j covers tile rows 16j..16j+15; lane -> row 16j + lane/4, LDS chunk slot lane&3 holds k chunk slot^swz
    // Every workgroup of a k slice reads the same 64-byte column of A at the same step, and the rows of A are a
    // power of two apart, so those reads would all queue at one L2 channel.  Each workgroup therefore walks its k
    // steps from a different starting point (integer sums do not care about the order); workgroups that share an
    // XCD (blockIdx mod 8) get consecutive starting points, which spreads them over the channels.
    const uint32_t rot = (blockIdx.x >> 3) % nsteps;
    auto issue = [&](uint32_t st, uint32_t step) {
        unsigned char *sa = smem + st * STAGE, *sb = sa + A_STAGE;
        const uint32_t kt = step + rot < nsteps ? step + rot : step + rot - nsteps;
        const unsigned char *Agk = Ag + (size_t)kt * 64;
        const unsigned char *Bgk = Bg + (size_t)kt * 64 * ldb;
#pragma unroll
        for (int jj = 0; jj < A_CP; ++jj) {
            const int j = (MBW == 1) ? (w & 1) : w + NW * jj;
            const uint32_t lrow = 16 * j + (lane >> 2);
            const uint32_t srow = umin(lrow, rowsValid - 1u);
            dma16(Agk + (size_t)srow * lda + (((lane & 3) ^ ((lane >> 4) & 3)) * 16), sa + j * 1024);
        }
        // B: copy j covers k rows 8j..8j+7; lane -> row 8j + lane/8, slot lane&7 holds chunk slot ^ (((row>>1)&3)<<1)
#pragma unroll
        for (int jj = 0; jj < B_CP; ++jj) {
            const int j = w + NW * jj;
            const int row = 8 * j + (lane >> 3);
            dma16_stream(Bgk + (size_t)row * ldb + (((lane & 7) ^ (((row >> 1) & 3) << 1)) * 16), sb + j * 1024);
        }
    };

    v16i acc[MBW];
#pragma unroll
    for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mb][r] = 0;

    const uint32_t a_lds = c32 * 64;
    const uint32_t a_sw = (c32 >> 2) & 3;
    // transpose read of this wave's 32 columns (two 16-column chunks, one per half of a 32-lane group)
    const int ti16 = lane & 15, tch = (lane >> 4) & 1, trow = ti16 >> 1, thalf = ti16 & 1;
    const uint32_t b_lds = (16 * h + trow) * 128 + (((2 * w + tch) ^ (((trow >> 1) & 3) << 1)) * 16) + thalf * 8;

    const uint32_t pre = umin(nsteps, NS - 1);
    for (uint32_t i = 0; i < pre; ++i) issue(i, i);
    for (uint32_t kt = 0; kt < nsteps; ++kt) {
        const uint32_t ahead = umin(nsteps - 1u - kt, NS - 2u);   // later steps whose copies may still be in flight
        switch (ahead) {
            case 6: CATCOC_WAIT_VMCNT(6 * STEP_CP); break;
            case 5: CATCOC_WAIT_VMCNT(5 * STEP_CP); break;
            case 4: CATCOC_WAIT_VMCNT(4 * STEP_CP); break;
            case 3: CATCOC_WAIT_VMCNT(3 * STEP_CP); break;
            case 2: CATCOC_WAIT_VMCNT(2 * STEP_CP); break;
            case 1: CATCOC_WAIT_VMCNT(1 * STEP_CP); break;
            default: CATCOC_WAIT_VMCNT(0); break;
        }
        barrier_keep_vmem();
        // stage (kt + NS - 1) % NS was read in step kt - 1, which every wave has left
        if (kt + NS - 1 < nsteps) issue((kt + NS - 1) & (NS - 1), kt + NS - 1);
        const unsigned char *sa = smem + (kt & (NS - 1)) * STAGE, *sb = sa + A_STAGE;
        // all fragment reads of the step first, then the MFMAs: one LDS round trip per step instead of one per
        // 32-row block (left to itself the compiler reuses two fragment registers and serialises them)
        v4i bf[2], af[2][MBW];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const unsigned char *p = sb + b_lds + kk * 32 * 128;
            const v2i t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)p);
            const v2i t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)(p + 8 * 128));
            bf[kk] = v4i{t0.x, t0.y, t1.x, t1.y};
#pragma unroll
            for (int mb = 0; mb < MBW; ++mb)
                af[kk][mb] = *(const v4i *)(sa + a_lds + mb * 32 * 64 + (((2 * kk + h) ^ a_sw) * 16));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int mb = 0; mb < MBW; ++mb) acc[mb] = mfma32<DT_I8>(af[kk][mb], bf[kk], acc[mb]);
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- k slices meet -------------------------------------------------------------
    // acc[mb][r] is element (lrow, lcol) with lrow = mb*32 + (r>>2)*8 + h*4 + (r&3), lcol = w*32 + c32
    const uint32_t lcol = w * 32 + c32;
    if (f > 1) {
        // Partial tiles travel through memory at device scope (cache policy sc1: written through / read past
        // the XCD-local L2), as ordinary buffer accesses so that the loads of a slice are issued together.
        constexpr int DEVICE_SCOPE = 16;   // sc1
        const size_t tileBytes = 128 * 128 * 4;
        const __amdgpu_buffer_rsrc_t mine = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(args.skPart + ((size_t)slice * loopsM * loopsN + tile) * (128 * 128)), 0, (int)tileBytes, 0x00020000);
#pragma unroll
        for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t lrow = mb * 32 + (r >> 2) * 8 + h * 4 + (r & 3);
                const int iv = acc[mb][r];
                if (lrow < rowsValid) __builtin_amdgcn_raw_buffer_store_b32(iv, mine, (lrow * 128 + lcol) * 4, 0, DEVICE_SCOPE);
            }
        // once the stores are acknowledged the slice may be counted
        CATCOC_WAIT_VMCNT(0);
        __syncthreads();
        volatile uint32_t *flag = (volatile uint32_t *)smem;
        if (tid == 0) *flag = __hip_atomic_fetch_add(args.skCount + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*flag != f - 1u) return;
        if (tid == 0) __hip_atomic_store(args.skCount + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // the other slices' partials, one 32-row block at a time and up to four slices per round trip
        const int32_t *tile0 = args.skPart + (size_t)tile * (128 * 128);
        const size_t sliceStride = (size_t)loopsM * loopsN * (128 * 128);
#pragma unroll
        for (int mb = 0; mb < MBW; ++mb) {
            for (uint32_t s0 = 0; s0 < f; s0 += 4) {
                int pv[4][16];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t s = s0 + q;
                    const bool use = s < f && s != slice;
                    const __amdgpu_buffer_rsrc_t other = __builtin_amdgcn_make_buffer_rsrc(
                        (void *)(tile0 + (use ? s : slice) * sliceStride), 0, (int)tileBytes, 0x00020000);
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t lrow = mb * 32 + (r >> 2) * 8 + h * 4 + (r & 3);
                        // unused slots and rows past the end read as zero: the offset is pushed out of the descriptor's range
                        pv[q][r] = __builtin_amdgcn_raw_buffer_load_b32(other, (use && lrow < rowsValid) ? (lrow * 128 + lcol) * 4 : 0x7fffffff, 0, DEVICE_SCOPE);
                    }
                }
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[mb][r] += pv[q][r];
            }
        }
    }

    // ---- epilogue on the rows that exist -----------------------------------------------
    // Per 32-row block: bias, dumps, dequant; then the peers' values of the block's kept rows are fetched eight
    // peers at a time in ONE round trip (out-of-range offsets of a buffer load cost nothing and return zero, which
    // masks rows that are not kept and peers that do not exist) and added in slot order; then the 16-bit store.
    const uint32_t gcol = colT + lcol;
    const int bv = args.bias ? args.bias[gcol] : 0;
    const float sN = args.scaleN[gcol];
    const uint32_t keptEnd = args.keptBegin + args.keptRows;
    const uint64_t peerBytes = (uint64_t)(args.peerRowOffset + args.keptRows) * args.peerLd * 4;
    const int peerRange = peerBytes > 0x7fffffffull ? 0x7fffffff : (int)peerBytes;
    long long csum = 0;
#pragma unroll
    for (int mb = 0; mb < MBW; ++mb) {
        const uint32_t blk0 = row0 + mb * 32;
        if (blk0 >= row0 + rowsValid) break;
        float v[16];
        uint32_t poff[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t lrow = mb * 32 + (r >> 2) * 8 + h * 4 + (r & 3);
            const uint32_t grow = row0 + lrow;
            const bool valid = lrow < rowsValid;
            const bool kept = valid && grow >= args.keptBegin && grow < keptEnd;
            const int iv = acc[mb][r] + bv;
            if (valid && args.accDump) ((int32_t *)args.accDump)[(size_t)grow * N + gcol] = iv;
            if (kept && args.cAccum) args.cAccum[(size_t)(grow - args.keptBegin) * N + gcol] = iv;
            if (valid && !kept) csum += iv;
            v[r] = __fmul_rn(__fmul_rn((float)iv, sN), args.scaleM[valid ? grow : row0]);
            poff[r] = kept ? (uint32_t)(((args.peerRowOffset + grow - args.keptBegin) * args.peerLd + gcol) * 4) : 0x7fffffffu;
        }
        if (blk0 < keptEnd && blk0 + 32 > args.keptBegin) {   // the block holds kept rows
            for (uint32_t p0 = 0; p0 < args.nPeers; p0 += 8) {
                float pv[8][16];
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const bool use = p0 + q < args.nPeers;
                    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
                        (void *)args.peers[use ? p0 + q : 0], 0, use ? peerRange : 0, 0x00020000);
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        pv[q][r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, poff[r], 0, 2 /* streaming */));
                }
#pragma unroll
                for (int q = 0; q < 8; ++q)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (p0 + q < args.nPeers) v[r] = __fadd_rn(v[r], pv[q][r]);
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t grow = blk0 + (r >> 2) * 8 + h * 4 + (r & 3);
                if (poff[r] != 0x7fffffffu)
                    ((unsigned short *)args.d)[(size_t)(grow - args.keptBegin) * args.ldd + gcol] = (unsigned short)f32_to_out16(v[r], args.outDtype);
            }
        }
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
