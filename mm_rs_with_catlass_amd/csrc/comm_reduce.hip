// The reference's vector-core work as kernels of their own, for the round-pipelined form of the operators:
//   * comm_reduce_kernel   -- one comm round of KQ/KRS's AIV loop (quant_matmul_reduce_scatter.hpp:262-320,
//                             matmul_reduce_scatter.hpp:237-296): walk BlockCommSwizzle's task list, skip this rank, add
//                             the peer's block into the local block (comm_block_epilogue_to_local_mem.hpp:162-224 under
//                             SetAtomicAdd).  Peers' data are staged buffers in this GPU's HBM.
//   * dequant_rows_kernel  -- the pass after all rounds (quant_matmul_reduce_scatter.hpp:322-351,
//                             block_epilogue_per_token_dequant.hpp:574-594): int32 -> fp32, x per-channel scale, x per-token
//                             scale, one rounding to fp16 / bf16.
//   * reduce_add_kernel    -- catlass' split-K ReduceAdd (gemm/kernel/splitk_matmul.hpp:24-161): sum of the k slices'
//                             fp32 workspaces in slice order, one rounding to the output type.
// All three are HBM-bound streaming kernels: 16-byte accesses per lane, whole rows of a block per wave.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "comm_reduce.h"
#include "gemm_fused_kernel.h"   // rounding helpers

namespace catcoc {

typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

namespace {

__device__ __forceinline__ float half_bits_to_f32(uint32_t bits, uint32_t dt)
{
    if (dt == DT_BF16) return __builtin_bit_cast(float, bits << 16);
    return (float)__builtin_bit_cast(_Float16, (unsigned short)bits);
}

// One 16-bit add as the hardware atomic does it: exact sum of the two values, one rounding (RNE) to the 16-bit type.
// (fp32 holds the sum of two fp16 / bf16 values to well beyond twice their precision, so rounding the fp32 sum is
// the correctly rounded 16-bit sum.)
__device__ __forceinline__ uint32_t add16(uint32_t a, uint32_t b, uint32_t dt)
{
    return f32_to_out16(__fadd_rn(half_bits_to_f32(a, dt), half_bits_to_f32(b, dt)), dt);
}

// Geometry of data block `d` of the round: the reference's comm blocks are commBlockM rows of the tile-linear slab of
// this rank, i.e. block d = rows [sub * cb, +cb) of the round's tile number d / (m0 / cb) (in swizzle order).
struct BlockGeom { uint32_t row0, rows, col0, cols; };

__device__ __forceinline__ BlockGeom block_geom(const CommArgs &a, uint32_t d)
{
    const uint32_t bpt = a.m0 / a.commBlockM;
    const uint32_t t = d / bpt, sub = d - t * bpt;
    uint32_t mi, ni;
    swizzle_block_coord(a.off, a.dir, a.loopsM, a.loopsN, a.roundFirstIdx + t, mi, ni);
    BlockGeom g;
    g.row0 = mi * a.m0 + sub * a.commBlockM;
    g.col0 = ni * a.n0;
    g.rows = g.row0 < a.mRank ? umin(a.commBlockM, a.mRank - g.row0) : 0u;
    g.cols = umin(a.n0, a.N - g.col0);
    return g;
}

}  // namespace

// ELEM: 0 = int32 blocks (the W8A8 operator reduces its int32 accumulators), 1 = 16-bit blocks (fp16 / bf16 partials
// added in that precision, as the float operators do).
// DET: the deterministic schedule.  Workgroup c is "core" c of the comm schedule.  With DET it owns data blocks
// c, c + cores, ...: it reads the local block once, adds the ranks' blocks in the schedule's order in registers and
// writes the block back, so the result does not depend on timing.  Without DET every (block, rank) task adds its
// peer block into memory with atomic adds, in whatever order the cores get there, like the reference.
template <int ELEM, bool DET>
__global__ void __launch_bounds__(256) comm_reduce_kernel(const CommArgs a)
{
    const uint32_t cores = gridDim.x;
    const uint32_t coreLoop = comm_core_loop(DET, a.P, a.splitRow, a.splitCol, a.dataLoops);
    const uint32_t tid = threadIdx.x;
    constexpr uint32_t VEC = ELEM == 0 ? 4u : 8u;      // elements per 16-byte access
    constexpr uint32_t ES = ELEM == 0 ? 4u : 2u;

    if constexpr (DET) {
        // tasks c, c + cores, ... of the deterministic order are (block c + band * cores, rank sequence): walk blocks.  Which
        // workgroup adds a block does not change any result, so the blocks are dealt out in pieces of 256 x 4 sixteen-byte
        // accesses (a.passes per block) over as many workgroups as the launch has: more loads in flight per CU.
        for (uint32_t unit = blockIdx.x; unit < a.dataLoops * a.passes; unit += cores) {
            const uint32_t d = unit / a.passes;
            const BlockGeom g = block_geom(a, d);
            const uint32_t vecPerRow = g.cols / VEC;                  // (host: n0 and N are multiples of 8)
            const uint32_t total = g.rows * vecPerRow;
            const uint32_t e0 = (unit - d * a.passes) * (256u * 4u);  // up to four 16-byte pieces per thread per piece
            if (e0 < total) {
                v4i acc[4];
                uint32_t offs[4];
                bool ok[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t e = e0 + u * 256 + tid;
                    ok[u] = e < total;
                    const uint32_t r = ok[u] ? e / vecPerRow : 0u, c = ok[u] ? e - r * vecPerRow : 0u;
                    const size_t lo = ((size_t)(g.row0 + r) * a.localLd + g.col0 + c * VEC) * ES;
                    acc[u] = ok[u] ? *(const v4i *)((const unsigned char *)a.local + lo) : v4i{0, 0, 0, 0};
                    offs[u] = e;   // (the element index: local and peer pitches differ, so offsets are rebuilt per buffer)
                }
                for (uint32_t i = 0; i < a.P; ++i) {
                    const uint32_t rk = (i + d) % a.P;                // the rank the deterministic order visits i-th for block d
                    if (rk == a.rank) continue;
                    const unsigned char *pb = (const unsigned char *)a.peers[rk < a.rank ? rk : rk - 1u];
                    v4i pv[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const uint32_t e = offs[u];
                        const uint32_t r = ok[u] ? e / vecPerRow : 0u, c = ok[u] ? e - r * vecPerRow : 0u;
                        const size_t po = ((size_t)(a.peerRowOffset + g.row0 + r) * a.peerLd + g.col0 + c * VEC) * ES;
                        pv[u] = ok[u] ? __builtin_nontemporal_load((const v4i *)(pb + po)) : v4i{0, 0, 0, 0};
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if constexpr (ELEM == 0) {
                            acc[u] += pv[u];
                        } else {
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                const uint32_t x = (uint32_t)acc[u][q], y = (uint32_t)pv[u][q];
                                const uint32_t lo = add16(x & 0xffffu, y & 0xffffu, a.dtype);
                                const uint32_t hi = add16(x >> 16, y >> 16, a.dtype);
                                acc[u][q] = (int)(lo | (hi << 16));
                            }
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (!ok[u]) continue;
                    const uint32_t e = offs[u];
                    const uint32_t r = e / vecPerRow, c = e - r * vecPerRow;
                    const size_t lo = ((size_t)(g.row0 + r) * a.localLd + g.col0 + c * VEC) * ES;
                    *(v4i *)((unsigned char *)a.local + lo) = acc[u];
                    if constexpr (ELEM == 0) {
                        if (a.dOut != nullptr) {   // the block is final: per-channel scale, then per-token, one rounding
                            const uint32_t col = g.col0 + c * VEC;
                            const v4f sn = *(const v4f *)(a.scaleN + col);
                            const float sm = a.scaleM[g.row0 + r];
                            uint32_t o[4];
#pragma unroll
                            for (int q = 0; q < 4; ++q) o[q] = f32_to_out16(__fmul_rn(__fmul_rn((float)acc[u][q], sn[q]), sm), a.outDtype);
                            *(v2i *)((unsigned short *)a.dOut + (size_t)(g.row0 + r) * a.ldd + col) = v2i{(int)(o[0] | (o[1] << 16)), (int)(o[2] | (o[3] << 16))};
                        }
                    }
                }
            }
        }
    } else {
        for (uint32_t t = blockIdx.x; t < coreLoop; t += cores) {
            uint32_t d, rk;
            comm_block_idx_ex(a.swizzleDir, false, a.P, a.splitRow, a.splitCol, a.dataLoops, t, d, rk);
            if (rk == a.rank || d >= a.dataLoops) continue;
            const BlockGeom g = block_geom(a, d);
            const unsigned char *pb = (const unsigned char *)a.peers[rk < a.rank ? rk : rk - 1u];
            const uint32_t vecPerRow = g.cols / VEC;
            const uint32_t total = g.rows * vecPerRow;
            for (uint32_t e = tid; e < total; e += 256) {
                const uint32_t r = e / vecPerRow, c = e - r * vecPerRow;
                const size_t po = ((size_t)(a.peerRowOffset + g.row0 + r) * a.peerLd + g.col0 + c * VEC) * ES;
                const size_t lo = ((size_t)(g.row0 + r) * a.localLd + g.col0 + c * VEC) * ES;
                const v4i pv = __builtin_nontemporal_load((const v4i *)(pb + po));
                unsigned char *lp = (unsigned char *)a.local + lo;
                if constexpr (ELEM == 0) {
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        __hip_atomic_fetch_add((int *)lp + q, pv[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                } else {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int w = pv[q];   // (bit casts go through a scalar: casting a vector element in place picks element 0)
                        if (a.dtype == DT_BF16)
                            __builtin_amdgcn_global_atomic_fadd_v2bf16((v2bf *)lp + q, __builtin_bit_cast(v2bf, w));
                        else
                            __builtin_amdgcn_global_atomic_fadd_v2f16((v2h *)lp + q, __builtin_bit_cast(v2h, w));
                    }
                }
            }
        }
    }
}

// D[i, j] = cast(float(acc[i, j]) * scaleN[j] * scaleM[i]) for the kept block, four columns per thread.
__global__ void __launch_bounds__(256) dequant_rows_kernel(const int32_t *acc, int64_t ldAcc, const float *scaleN, const float *scaleM,
                                                           void *out, int64_t ldOut, uint32_t rows, uint32_t cols, uint32_t outDtype)
{
    const uint32_t vecPerRow = cols / 4u;
    const uint64_t total = (uint64_t)rows * vecPerRow;
    for (uint64_t e = (uint64_t)blockIdx.x * 256u + threadIdx.x; e < total; e += (uint64_t)gridDim.x * 256u) {
        const uint32_t r = (uint32_t)(e / vecPerRow), c = (uint32_t)(e - (uint64_t)r * vecPerRow) * 4u;
        const v4i v = *(const v4i *)(acc + (size_t)r * ldAcc + c);
        const v4f sn = *(const v4f *)(scaleN + c);
        const float sm = scaleM[r];
        uint32_t o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) o[q] = f32_to_out16(__fmul_rn(__fmul_rn((float)v[q], sn[q]), sm), outDtype);
        *(v2i *)((unsigned short *)out + (size_t)r * ldOut + c) = v2i{(int)(o[0] | (o[1] << 16)), (int)(o[2] | (o[3] << 16))};
    }
}

// dst[i] = cast(((src[0][i] + src[1][i]) + src[2][i]) + ...), slices `elementCount` apart; OUT: 0 = fp32 copy of the
// sum, else the 16-bit type.  Four elements per thread per step.
__global__ void __launch_bounds__(256) reduce_add_kernel(void *dst, const float *src, uint64_t elementCount, uint32_t slices, uint32_t outDtype)
{
    const uint64_t vecs = elementCount / 4u;
    for (uint64_t e = (uint64_t)blockIdx.x * 256u + threadIdx.x; e < vecs; e += (uint64_t)gridDim.x * 256u) {
        v4f s = __builtin_nontemporal_load((const v4f *)src + e);
        for (uint32_t k = 1; k < slices; ++k) {
            const v4f t = __builtin_nontemporal_load((const v4f *)(src + (uint64_t)k * elementCount) + e);
#pragma unroll
            for (int q = 0; q < 4; ++q) s[q] = __fadd_rn(s[q], t[q]);
        }
        if (outDtype == 0) {
            *((v4f *)dst + e) = s;
        } else {
            uint32_t o[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) o[q] = f32_to_out16(s[q], outDtype);
            *((v2i *)dst + e) = v2i{(int)(o[0] | (o[1] << 16)), (int)(o[2] | (o[3] << 16))};
        }
    }
    // tail (elementCount not a multiple of four): one thread each
    const uint64_t tail0 = vecs * 4u;
    if (blockIdx.x == 0 && threadIdx.x < elementCount - tail0) {
        const uint64_t i = tail0 + threadIdx.x;
        float s = src[i];
        for (uint32_t k = 1; k < slices; ++k) s = __fadd_rn(s, src[(uint64_t)k * elementCount + i]);
        if (outDtype == 0) ((float *)dst)[i] = s;
        else ((unsigned short *)dst)[i] = (unsigned short)f32_to_out16(s, outDtype);
    }
}

int launch_comm_reduce(const CommArgs &a0, uint32_t cores, bool deterministic, void *stream)
{
    CommArgs a = a0;
    const uint32_t vec = a.dtype == CT_INT32 ? 4u : 8u;
    a.passes = ceil_div(a.commBlockM * (a.n0 / vec), 256u * 4u);
    if (a.passes == 0) a.passes = 1;
    if (deterministic) {   // (the deterministic result does not depend on the number of workgroups)
        const uint64_t units = (uint64_t)a.dataLoops * a.passes;
        cores = (uint32_t)(units < 2048u ? (units ? units : 1u) : 2048u);
    }
    const dim3 grid(cores), block(256);
    hipStream_t s = (hipStream_t)stream;
    if (a.dtype == CT_INT32) {
        if (deterministic) hipLaunchKernelGGL((comm_reduce_kernel<0, true>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((comm_reduce_kernel<0, false>), grid, block, 0, s, a);
    } else {
        if (deterministic) hipLaunchKernelGGL((comm_reduce_kernel<1, true>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((comm_reduce_kernel<1, false>), grid, block, 0, s, a);
    }
    return (int)hipGetLastError();
}

int launch_dequant_rows(const int32_t *acc, int64_t ldAcc, const float *scaleN, const float *scaleM, void *out, int64_t ldOut,
                        uint32_t rows, uint32_t cols, uint32_t outDtype, void *stream)
{
    const uint64_t total = (uint64_t)rows * (cols / 4u);
    const uint32_t blocks = (uint32_t)((total + 255u) / 256u);
    hipLaunchKernelGGL(dequant_rows_kernel, dim3(blocks < 4096u ? (blocks ? blocks : 1u) : 4096u), dim3(256), 0, (hipStream_t)stream, acc, ldAcc,
                       scaleN, scaleM, out, ldOut, rows, cols, outDtype);
    return (int)hipGetLastError();
}

int launch_reduce_add(void *dst, const float *src, uint64_t elementCount, uint32_t slices, uint32_t outDtype, void *stream)
{
    const uint64_t vecs = elementCount / 4u;
    const uint64_t blocks = (vecs + 255u) / 256u;
    hipLaunchKernelGGL(reduce_add_kernel, dim3((uint32_t)(blocks < 8192u ? (blocks ? blocks : 1u) : 8192u)), dim3(256), 0, (hipStream_t)stream, dst,
                       src, elementCount, slices, outDtype);
    return (int)hipGetLastError();
}

}  // namespace catcoc
