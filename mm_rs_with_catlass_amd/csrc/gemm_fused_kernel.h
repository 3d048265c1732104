// Fused tile GEMM + dequant + peer-reduce epilogue for gfx950 (MI355X).
//
// One workgroup (256 threads = 4 wavefronts, 2x2) computes one (64*MB) x 256 tile
// of the local partial product with MFMA, k in steps of 64 bytes, A and B tiles
// double-buffered in LDS.  It then applies the epilogue the reference runs as
// separate vector-core passes (reduce of the peers' partials, per-token dequant,
// cast) while the accumulators are still in registers, and writes only what the
// rank keeps; tiles that belong to other ranks are stored to the outbound
// workspace or folded into a checksum.
//
// Stands in for, per tile: BlockMmad<MmadAtlasA2Pingpong[Bias]>
// (3rdparty/catlass/include/catlass/gemm/block/block_mmad_pingpong.hpp:144-320,
// block_mmad_pingpong_bias.hpp:279-315), the atomic-add reduce of
// include/catcoc/comm_epilogue/block/comm_block_epilogue_to_local_mem.hpp:162-224 and
// BlockEpilogue<EpilogueAtlasA2PerTokenDequant>
// (3rdparty/catlass/include/catlass/epilogue/block/block_epilogue_per_token_dequant.hpp:498-606).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_args.h"

namespace catcoc {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef unsigned short v4u16 __attribute__((ext_vector_type(4)));

template <uint32_t DT> struct AccOf { using type = v16f; };
template <> struct AccOf<DT_I8> { using type = v16i; };

// One 32x32 MFMA over a 32-byte k slab: int8 32x32x32, fp16/bf16 32x32x16.
// Lane l supplies 16 bytes of row (l%32) for k-chunk (l/32) of each operand.
template <uint32_t DT>
__device__ __forceinline__ typename AccOf<DT>::type mfma32(v4i a, v4i b, typename AccOf<DT>::type c)
{
    if constexpr (DT == DT_I8) {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
    } else if constexpr (DT == DT_F16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
    }
}

__device__ __forceinline__ int f2i(float f) { return __builtin_bit_cast(int, f); }
__device__ __forceinline__ float i2f(int i) { return __builtin_bit_cast(float, i); }

// fp32 -> bf16, round to nearest even, NaN -> 0x7fc0.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f)
{
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return (f != f) ? 0x7fc0u : r;
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f)
{
    _Float16 h = (_Float16)f;  // v_cvt_f16_f32, round to nearest even
    return (uint32_t)__builtin_bit_cast(unsigned short, h);
}

__device__ __forceinline__ uint32_t f32_to_out16(float f, uint32_t outDtype)
{
    return outDtype == DT_BF16 ? f32_to_bf16_bits(f) : f32_to_f16_bits(f);
}

// Transpose a 4x4 byte block held as four dwords (row r = dword r, byte c = column c).
__device__ __forceinline__ void transpose4x4_b8(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3, uint32_t &c0,
                                                uint32_t &c1, uint32_t &c2, uint32_t &c3)
{
    // v_perm_b32(hi, lo, sel): selector byte values 0-3 pick from lo, 4-7 from hi
    const uint32_t lo01 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);  // r0.b0 r1.b0 r0.b1 r1.b1
    const uint32_t hi01 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);  // r0.b2 r1.b2 r0.b3 r1.b3
    const uint32_t lo23 = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
    const uint32_t hi23 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    c0 = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
    c1 = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
    c2 = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
    c3 = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

// ---------------------------------------------------------------------------
// Fast kernel.  Requirements checked by the host: A stored [rows, K] (k
// contiguous); K a multiple of 16 bytes of elements; N a multiple of 4; leading
// dimensions and base pointers 16-byte aligned (A, and B when TRANSB) / 4-element
// aligned (B row-major).  EDGE = false additionally assumes full tiles and K a
// multiple of the k step, and drops every bounds check.
//
// LDS layouts (per stage), all in 16-byte chunks of 16/ES consecutive k:
//   A: [row][4 chunks], chunk slot = chunk ^ ((row >> 2) & 3)
//   B: [k-chunk g][column phase i = n & 3][slot p = (n >> 7) * 32 + ((n & 127) >> 2)]
//      so that the lane reading slot p for the four phases holds four ADJACENT
//      output columns, and writers of a row-major B tile (one k row per load,
//      4 columns per lane, transposed in registers) write 1 KiB contiguous.
// ---------------------------------------------------------------------------
template <uint32_t DT, int MB, bool TRANSB, bool EDGE>
__global__ void __launch_bounds__(256, (MB <= 2) ? 2 : 1) gemm_fused_kernel(const GemmArgs args)
{
    using Acc = typename AccOf<DT>::type;
    constexpr int ES = (DT == DT_I8) ? 1 : 2;
    constexpr int BM = 64 * MB;
    constexpr int BKE = 64 / ES;   // elements per k step
    constexpr int CHE = 16 / ES;   // elements per 16-byte chunk
    constexpr int RW = 16 / ES;    // k rows of a row-major B tile handled by one wave
    constexpr int A_STAGE = BM * 64;
    constexpr int B_STAGE = 256 * 64;

    __shared__ __attribute__((aligned(16))) unsigned char smem[2 * (A_STAGE + B_STAGE)];
    unsigned char *const As = smem;
    unsigned char *const Bs = smem + 2 * A_STAGE;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = tid >> 6;
    const int wm = w >> 1, wn = w & 1;
    const int c32 = lane & 31, h = lane >> 5;

    const SchedParams &sp = args.sched;
    const uint32_t task = launch_order_task(sp, blockIdx.x + args.taskBase, (args.flags & GF_LINEAR_ORDER) != 0, args.keptRank);
    TileInfo ti;
    if (!task_tile(sp, task, ti)) return;

    const uint32_t K = args.K;
    const int64_t ldaB = args.lda * ES, ldbB = args.ldb * ES;
    const bool gather = sp.op == OP_ALLGATHER;
    const unsigned char *Ag = (const unsigned char *)args.a[gather ? ti.targetRank : 0] +
                              (int64_t)(gather ? ti.rowInRank : ti.row) * ldaB;
    const unsigned char *Bg = (const unsigned char *)args.b + (TRANSB ? (int64_t)ti.col * ldbB : (int64_t)ti.col * ES);

    // ---- per-thread load coordinates -------------------------------------
    const int a_row = tid >> 2, a_kc = tid & 3;
    const uint32_t a_off = (uint32_t)a_row * (uint32_t)ldaB + a_kc * 16;
    const uint32_t a_sts = a_row * 64 + ((a_kc ^ ((a_row >> 2) & 3)) * 16);
    // row-major B: wave w owns k rows [RW*w, RW*w + RW) of the step, lane owns 4 columns
    const uint32_t b_off = TRANSB ? 0u : (uint32_t)(RW * w) * (uint32_t)ldbB + lane * 4 * ES;
    const bool b_col_ok = !EDGE || (uint32_t)(lane * 4) < ti.colsValid;
    // transposed B ([N,K], k contiguous): 4 chunks per thread: q = (tid>>2) + 64*s -> phase i = q>>6... see below

    v4i areg[MB];
    uint32_t braw[16];
    v4i btr[4];

    auto gload = [&](uint32_t kt) {
        const unsigned char *Agk = Ag + (size_t)kt * 64;
#pragma unroll
        for (int s = 0; s < MB; ++s) {
            bool ok = true;
            if constexpr (EDGE) ok = (uint32_t)(a_row + 64 * s) < ti.rowsValid && (kt * BKE + a_kc * CHE) < K;
            areg[s] = ok ? *(const v4i *)(Agk + a_off + (size_t)(64 * s) * ldaB) : v4i{0, 0, 0, 0};
        }
        if constexpr (!TRANSB) {
            const unsigned char *Bgk = Bg + (size_t)kt * BKE * ldbB;
            if constexpr (DT == DT_I8) {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    bool ok = true;
                    if constexpr (EDGE) ok = b_col_ok && (kt * BKE + RW * w + j) < K;
                    braw[j] = ok ? *(const uint32_t *)(Bgk + b_off + (size_t)j * ldbB) : 0u;
                }
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    bool ok = true;
                    if constexpr (EDGE) ok = b_col_ok && (kt * BKE + RW * w + j) < K;
                    v2i t = ok ? *(const v2i *)(Bgk + b_off + (size_t)j * ldbB) : v2i{0, 0};
                    braw[2 * j] = (uint32_t)t.x;
                    braw[2 * j + 1] = (uint32_t)t.y;
                }
            }
        } else {
            // chunk q = (tid >> 2) + 64*s, k-chunk g = tid & 3: slot p = q & 63, phase i = s
            const unsigned char *Bgk = Bg + (size_t)kt * 64;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const uint32_t p = tid >> 2;
                const uint32_t n = (p >> 5) * 128 + (p & 31) * 4 + s;
                bool ok = true;
                if constexpr (EDGE) ok = n < ti.colsValid && (kt * BKE + (tid & 3) * CHE) < K;
                btr[s] = ok ? *(const v4i *)(Bgk + (size_t)n * ldbB + (tid & 3) * 16) : v4i{0, 0, 0, 0};
            }
        }
    };

    auto lds_store = [&](int stage) {
        unsigned char *as = As + stage * A_STAGE;
        unsigned char *bs = Bs + stage * B_STAGE;
#pragma unroll
        for (int s = 0; s < MB; ++s) *(v4i *)(as + a_sts + s * 64 * 64) = areg[s];
        if constexpr (!TRANSB) {
            uint32_t t[4][4];  // [column phase i][dword q of the 16-byte chunk]
            if constexpr (DT == DT_I8) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    transpose4x4_b8(braw[4 * q], braw[4 * q + 1], braw[4 * q + 2], braw[4 * q + 3], t[0][q], t[1][q],
                                    t[2][q], t[3][q]);
            } else {
                // rows 2q, 2q+1; dword 0 of a row = columns 0,1; dword 1 = columns 2,3
#pragma unroll
                for (int q = 0; q < 4; ++q) {
#pragma unroll
                    for (int pr = 0; pr < 2; ++pr) {
                        const uint32_t d0 = braw[2 * (2 * q) + pr], d1 = braw[2 * (2 * q + 1) + pr];
                        t[2 * pr][q] = __builtin_amdgcn_perm(d1, d0, 0x05040100u);
                        t[2 * pr + 1][q] = __builtin_amdgcn_perm(d1, d0, 0x07060302u);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
                *(v4i *)(bs + ((w * 4 + i) * 64 + lane) * 16) = v4i{(int)t[i][0], (int)t[i][1], (int)t[i][2], (int)t[i][3]};
        } else {
            // transposed-B stage layout: [phase i][slot p][4 chunks], chunk slot = g ^ ((p >> 2) & 3)
            const uint32_t p = tid >> 2, g = tid & 3;
#pragma unroll
            for (int s = 0; s < 4; ++s) *(v4i *)(bs + ((s * 64 + p) * 4 + (g ^ ((p >> 2) & 3))) * 16) = btr[s];
        }
    };

    Acc acc[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][nb][r] = 0;

    const uint32_t a_lds = (wm * 32 * MB + c32) * 64;
    const uint32_t a_sw = (c32 >> 2) & 3;
    const uint32_t b_slot = wn * 32 + c32;

    auto compute = [&](int stage) {
        const unsigned char *as = As + stage * A_STAGE;
        const unsigned char *bs = Bs + stage * B_STAGE;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const uint32_t g = 2 * kk + h;
            v4i af[MB], bf[4];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) af[mb] = *(const v4i *)(as + a_lds + mb * 32 * 64 + ((g ^ a_sw) * 16));
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
                if constexpr (!TRANSB) bf[nb] = *(const v4i *)(bs + ((g * 4 + nb) * 64 + b_slot) * 16);
                else bf[nb] = *(const v4i *)(bs + ((nb * 64 + b_slot) * 4 + (g ^ ((b_slot >> 2) & 3))) * 16);
            }
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) acc[mb][nb] = mfma32<DT>(af[mb], bf[nb], acc[mb][nb]);
        }
    };

    // ---- main loop: one barrier per k step ------------------------------
    const uint32_t nk = (K + BKE - 1) / BKE;
    gload(0);
    lds_store(0);
    __syncthreads();
    for (uint32_t kt = 0; kt < nk; ++kt) {
        const bool more = kt + 1 < nk;
        if (more) gload(kt + 1);
        compute(kt & 1);
        if (more) lds_store((kt + 1) & 1);
        __syncthreads();
    }

    // ---- epilogue ----------------------------------------------------------
    // acc[mb][nb][r] is element (row, col) of the tile with
    //   row = wm*32*MB + mb*32 + (r>>2)*8 + h*4 + (r&3),  col = wn*128 + 4*c32 + nb
    const uint32_t col4 = wn * 128 + 4 * c32;
    const uint32_t gcol = ti.col + col4;
    const bool col_ok = !EDGE || col4 < ti.colsValid;
    const uint32_t row_base = wm * 32 * MB + h * 4;
    const bool quant = DT == DT_I8;
    const bool kept = ti.row >= args.keptBegin && ti.row < args.keptBegin + args.keptRows;
    const uint32_t rowsValid = EDGE ? ti.rowsValid : (uint32_t)BM;

    if constexpr (DT == DT_I8) {
        if (args.bias != nullptr && col_ok) {
            const v4i bv = *(const v4i *)(args.bias + gcol);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[mb][nb][r] += bv[nb];
        }
    }

    if (args.accDump != nullptr && col_ok) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                if (lrow < rowsValid) {
                    const size_t o = (size_t)(ti.row + lrow) * args.N + gcol;
                    if constexpr (DT == DT_I8)
                        *(v4i *)((int32_t *)args.accDump + o) = v4i{acc[mb][0][r], acc[mb][1][r], acc[mb][2][r], acc[mb][3][r]};
                    else
                        *(v4f *)((float *)args.accDump + o) = v4f{acc[mb][0][r], acc[mb][1][r], acc[mb][2][r], acc[mb][3][r]};
                }
            }
    }

    v4f sN = {1.f, 1.f, 1.f, 1.f};
    if constexpr (DT == DT_I8) {
        if (col_ok) sN = *(const v4f *)(args.scaleN + gcol);
    }

    if (kept) {
        const uint32_t out_row0 = ti.row - args.keptBegin;
        const uint32_t keptLeft = args.keptBegin + args.keptRows - ti.row;
        const uint32_t rowsK = rowsValid < keptLeft ? rowsValid : keptLeft;
        const bool redI32 = quant && (args.flags & GF_REDUCE_INT32);

        if constexpr (DT == DT_I8) {
            if (redI32) {
                for (uint32_t p = 0; p < args.nPeers; ++p) {
                    const int32_t *pp = (const int32_t *)args.peers[p] + (args.peerRowOffset + out_row0) * args.peerLd + gcol;
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                            if (col_ok && lrow < rowsK) {
                                const v4i t = *(const v4i *)(pp + (size_t)lrow * args.peerLd);
#pragma unroll
                                for (int nb = 0; nb < 4; ++nb) acc[mb][nb][r] += t[nb];
                            }
                        }
                }
            }
            if (args.cAccum != nullptr && col_ok) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                        if (lrow < rowsK)
                            *(v4i *)(args.cAccum + (size_t)(out_row0 + lrow) * args.N + gcol) =
                                v4i{acc[mb][0][r], acc[mb][1][r], acc[mb][2][r], acc[mb][3][r]};
                    }
            }
        }

        // local partial in fp32, kept in the accumulator registers (dequantised for W8A8:
        // per-channel scale first, then per-token, each product rounded on its own)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                if constexpr (DT == DT_I8) {
                    const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                    const float sM = (lrow < rowsK) ? args.scaleM[ti.row + lrow] : 0.f;
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) {
                        const int iv = acc[mb][nb][r];
                        acc[mb][nb][r] = f2i(__fmul_rn(__fmul_rn((float)iv, sN[nb]), sM));
                    }
                }
            }
        auto getf = [&](int mb, int nb, int r) -> float {
            if constexpr (DT == DT_I8) {
                const int iv = acc[mb][nb][r];  // bit casts go through a scalar, never a vector-element lvalue
                return i2f(iv);
            } else {
                return acc[mb][nb][r];
            }
        };
        auto setf = [&](int mb, int nb, int r, float v) {
            if constexpr (DT == DT_I8) acc[mb][nb][r] = f2i(v);
            else acc[mb][nb][r] = v;
        };

        if (!redI32) {
            // peers in slot order; 16 rows (16 x 16-byte loads per lane) in flight at a time
            for (uint32_t p = 0; p < args.nPeers; ++p) {
                const float *pp = (const float *)args.peers[p] + (args.peerRowOffset + out_row0) * args.peerLd + gcol;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int rh = 0; rh < 2; ++rh) {
                        v4f t[8];
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            const uint32_t lrow = row_base + mb * 32 + (rh * 2 + (i >> 2)) * 8 + (i & 3);
                            bool okp = true;
                            if constexpr (EDGE) okp = col_ok && lrow < rowsK;
                            t[i] = okp ? __builtin_nontemporal_load((const v4f *)(pp + (size_t)lrow * args.peerLd)) : v4f{0.f, 0.f, 0.f, 0.f};
                        }
#pragma unroll
                        for (int i = 0; i < 8; ++i)
#pragma unroll
                            for (int nb = 0; nb < 4; ++nb) {
                                const int r = rh * 8 + i;
                                setf(mb, nb, r, __fadd_rn(getf(mb, nb, r), t[i][nb]));
                            }
                        __builtin_amdgcn_sched_barrier(0);
                    }
            }
        }

        if (col_ok) {
            unsigned short *dptr = (unsigned short *)args.d + (size_t)out_row0 * args.ldd + gcol;
            auto store_all = [&](auto cvt) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                        if (!EDGE || lrow < rowsK) {
                            const uint32_t lo = cvt(getf(mb, 0, r)) | (cvt(getf(mb, 1, r)) << 16);
                            const uint32_t hi = cvt(getf(mb, 2, r)) | (cvt(getf(mb, 3, r)) << 16);
                            *(v2i *)(dptr + (size_t)lrow * args.ldd) = v2i{(int)lo, (int)hi};
                        }
                    }
            };
            if (args.outDtype == DT_BF16) store_all([](float f) { return f32_to_bf16_bits(f); });
            else store_all([](float f) { return f32_to_f16_bits(f); });
        }
    } else if (args.flags & GF_OUTBOUND_STORE) {
        // tile-linear workspace of the reference: rows wsRow .. wsRow+m0, n0 columns
        const size_t base = (size_t)ti.wsRow * sp.n0 + col4;
        if (col_ok) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                    if (lrow < rowsValid) {
                        const size_t o = base + (size_t)lrow * sp.n0;
                        if constexpr (DT == DT_I8) {
                            if (args.flags & GF_REDUCE_INT32) {
                                *(v4i *)((int32_t *)args.outbound + o) = v4i{acc[mb][0][r], acc[mb][1][r], acc[mb][2][r], acc[mb][3][r]};
                            } else {
                                const float sM = args.scaleM[ti.row + lrow];
                                v4f o4;
#pragma unroll
                                for (int nb = 0; nb < 4; ++nb) o4[nb] = __fmul_rn(__fmul_rn((float)acc[mb][nb][r], sN[nb]), sM);
                                __builtin_nontemporal_store(o4, (v4f *)((float *)args.outbound + o));
                            }
                        } else {
                            __builtin_nontemporal_store(v4f{acc[mb][0][r], acc[mb][1][r], acc[mb][2][r], acc[mb][3][r]},
                                                        (v4f *)((float *)args.outbound + o));
                        }
                    }
                }
        }
    } else if (args.checksum != nullptr) {
        // fold the tile into one number so the work stays observable without the store traffic
        __shared__ double red[4];
        double s = 0.0;
        long long si = 0;
        if (col_ok) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t lrow = row_base + mb * 32 + (r >> 2) * 8 + (r & 3);
                    if (lrow < rowsValid) {
#pragma unroll
                        for (int nb = 0; nb < 4; ++nb) {
                            if constexpr (DT == DT_I8) si += acc[mb][nb][r];
                            else s += (double)acc[mb][nb][r];
                        }
                    }
                }
        }
        if constexpr (DT == DT_I8) {
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) si += __shfl_xor(si, o, 64);
            if (lane == 0) ((long long *)red)[w] = si;
            __syncthreads();
            if (tid == 0) {
                const long long *ri = (const long long *)red;
                ((long long *)args.checksum)[task] = ri[0] + ri[1] + ri[2] + ri[3];
            }
        } else {
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
            if (lane == 0) red[w] = s;
            __syncthreads();
            if (tid == 0) ((double *)args.checksum)[task] = ((red[0] + red[1]) + red[2]) + red[3];
        }
    }
}

// ---------------------------------------------------------------------------
// General kernel: any shape, alignment and operand layout.  One workgroup per
// task of the same schedule, one thread per output element, scalar k loop.
// It exists so that every shape the API accepts has a device implementation;
// it is not tuned.
// ---------------------------------------------------------------------------
template <uint32_t DT>
__global__ void __launch_bounds__(256) gemm_general_kernel(const GemmArgs args)
{
    const SchedParams &sp = args.sched;
    const uint32_t task = blockIdx.x + args.taskBase;
    TileInfo ti;
    if (!task_tile(sp, task, ti)) return;
    const bool gather = sp.op == OP_ALLGATHER;
    const uint32_t arow0 = gather ? ti.rowInRank : ti.row;
    // GF_ROW_MASK (explicit kept rows, which need not line up with tiles): every row decides for itself, and `checksum` takes
    // the rows that are not kept per tile of the plain grid, index (row / m0) * ceil(N / n0) + col / n0
    const bool rowMask = (args.flags & GF_ROW_MASK) != 0;
    const bool kept = rowMask ? (ti.row < args.keptBegin + args.keptRows && ti.row + ti.rowsValid > args.keptBegin)
                              : (ti.row >= args.keptBegin && ti.row < args.keptBegin + args.keptRows);
    const uint32_t keptLeft = kept && !rowMask ? args.keptBegin + args.keptRows - ti.row : 0;
    __shared__ double red[256];
    double csum = 0.0;
    long long isum = 0;

    for (uint32_t e = threadIdx.x; e < ti.rowsValid * ti.colsValid; e += 256) {
        const uint32_t lrow = e / ti.colsValid, lcol = e % ti.colsValid;
        const uint32_t col = ti.col + lcol;
        const size_t ar = arow0 + lrow;
        float facc = 0.f;
        int32_t iacc = 0;
        if constexpr (DT == DT_I8) {
            const int8_t *A = (const int8_t *)args.a[gather ? ti.targetRank : 0];
            const int8_t *B = (const int8_t *)args.b;
            if (args.bias) iacc = args.bias[col];
            for (uint32_t k = 0; k < args.K; ++k) {
                const int32_t av = args.transA ? A[(size_t)k * args.lda + ar] : A[ar * args.lda + k];
                const int32_t bv = args.transB ? B[(size_t)col * args.ldb + k] : B[(size_t)k * args.ldb + col];
                iacc += av * bv;
            }
        } else {
            const unsigned short *A = (const unsigned short *)args.a[gather ? ti.targetRank : 0];
            const unsigned short *B = (const unsigned short *)args.b;
            for (uint32_t k = 0; k < args.K; ++k) {
                const unsigned short ah = args.transA ? A[(size_t)k * args.lda + ar] : A[ar * args.lda + k];
                const unsigned short bh = args.transB ? B[(size_t)col * args.ldb + k] : B[(size_t)k * args.ldb + col];
                float af, bf;
                if constexpr (DT == DT_BF16) {
                    af = __builtin_bit_cast(float, (uint32_t)ah << 16);
                    bf = __builtin_bit_cast(float, (uint32_t)bh << 16);
                } else {
                    af = (float)__builtin_bit_cast(_Float16, ah);
                    bf = (float)__builtin_bit_cast(_Float16, bh);
                }
                facc = __fadd_rn(facc, __fmul_rn(af, bf));
            }
        }
        if (args.accDump) {
            const size_t o = (size_t)(ti.row + lrow) * args.N + col;
            if constexpr (DT == DT_I8) ((int32_t *)args.accDump)[o] = iacc;
            else ((float *)args.accDump)[o] = facc;
        }
        const bool rowKept = rowMask ? (ti.row + lrow - args.keptBegin) < args.keptRows : (kept && lrow < keptLeft);   // (unsigned: rows above keptBegin wrap)
        if (rowKept) {
            const uint32_t orow = ti.row - args.keptBegin + lrow;
            float v;
            if constexpr (DT == DT_I8) {
                const bool redI32 = args.flags & GF_REDUCE_INT32;
                if (redI32)
                    for (uint32_t p = 0; p < args.nPeers; ++p)
                        iacc += ((const int32_t *)args.peers[p])[(args.peerRowOffset + orow) * args.peerLd + col];
                if (args.cAccum) args.cAccum[(size_t)orow * args.N + col] = iacc;
                v = __fmul_rn(__fmul_rn((float)iacc, args.scaleN[col]), args.scaleM[ti.row + lrow]);
                if (!redI32)
                    for (uint32_t p = 0; p < args.nPeers; ++p)
                        v = __fadd_rn(v, ((const float *)args.peers[p])[(args.peerRowOffset + orow) * args.peerLd + col]);
            } else {
                v = facc;
                for (uint32_t p = 0; p < args.nPeers; ++p)
                    v = __fadd_rn(v, ((const float *)args.peers[p])[(args.peerRowOffset + orow) * args.peerLd + col]);
            }
            ((unsigned short *)args.d)[(size_t)orow * args.ldd + col] = (unsigned short)f32_to_out16(v, args.outDtype);
        } else if (args.flags & GF_OUTBOUND_STORE) {
            const size_t o = (size_t)(ti.wsRow + lrow) * sp.n0 + lcol;
            if constexpr (DT == DT_I8) {
                if (args.flags & GF_REDUCE_INT32) ((int32_t *)args.outbound)[o] = iacc;
                else ((float *)args.outbound)[o] = __fmul_rn(__fmul_rn((float)iacc, args.scaleN[col]), args.scaleM[ti.row + lrow]);
            } else {
                ((float *)args.outbound)[o] = facc;
            }
        } else {
            if constexpr (DT == DT_I8) isum += iacc;
            else csum += (double)facc;
        }
    }
    if ((!kept || rowMask) && !(args.flags & GF_OUTBOUND_STORE) && args.checksum != nullptr) {
        const size_t slot = rowMask ? (size_t)(ti.row / sp.m0) * sp.loopsN + ti.col / sp.n0 : (size_t)task;
        if constexpr (DT == DT_I8) ((long long *)red)[threadIdx.x] = isum;
        else red[threadIdx.x] = csum;
        __syncthreads();
        if (threadIdx.x == 0) {
            if constexpr (DT == DT_I8) {
                long long t = 0;
                for (int i = 0; i < 256; ++i) t += ((long long *)red)[i];
                ((long long *)args.checksum)[slot] = t;
            } else {
                double t = 0;
                for (int i = 0; i < 256; ++i) t += red[i];
                ((double *)args.checksum)[slot] = t;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Host-side variant selection (one translation unit per element type)
// ---------------------------------------------------------------------------

template <uint32_t DT, int MB, bool TRANSB>
static hipError_t launch_fast(const GemmArgs &args, bool edge, hipStream_t stream)
{
    const dim3 grid(launch_positions(args)), block(256);
    if (edge) hipLaunchKernelGGL((gemm_fused_kernel<DT, MB, TRANSB, true>), grid, block, 0, stream, args);
    else hipLaunchKernelGGL((gemm_fused_kernel<DT, MB, TRANSB, false>), grid, block, 0, stream, args);
    return hipGetLastError();
}

// variant: 0 = general kernel; otherwise tile rows / 64 of the fast kernel (1 or 2).
template <uint32_t DT>
static int launch_dt(const GemmArgs &args, int variant, bool edge, void *stream)
{
    hipStream_t s = (hipStream_t)stream;
    if (variant == 0) {
        hipLaunchKernelGGL((gemm_general_kernel<DT>), dim3(launch_positions(args)), dim3(256), 0, s, args);
        return (int)hipGetLastError();
    }
    if (args.transB) {
        if (variant == 1) return (int)launch_fast<DT, 1, true>(args, edge, s);
        return (int)launch_fast<DT, 2, true>(args, edge, s);
    }
    if (variant == 1) return (int)launch_fast<DT, 1, false>(args, edge, s);
    return (int)launch_fast<DT, 2, false>(args, edge, s);
}

}  // namespace catcoc
