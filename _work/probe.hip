// Measurement helpers, not operators.  First: the inner loop of the 128x256 W8A8 kernel with the global-memory side taken
// away.  512 workgroups of four waves (two per CU, as the real launch), each wave issuing the main loop's sixteen
// 32x32x32 int8 MFMAs per k step, with or without the LDS fragment reads that feed them (four 16-byte reads for A,
// sixteen transposing 8-byte reads for B per step), on whatever bytes the caller puts into LDS.  What it sustains is
// the ceiling of the matrix pipes for that data on the box at hand: the pipes are power-limited, and how hard depends
// on how many operand bits toggle.  bench.py --mode ceiling reports it.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "catcoc_hip.h"
#include "gemm_dma_kernel.h"

namespace catcoc {

template <bool LDS_READS>
__global__ void __launch_bounds__(256, 2) probe_mfma_kernel(const unsigned char *pattern, uint32_t steps, int *sink)
{
    constexpr int POOL = 72 * 1024;   // three stages of A (8 KiB) and B (16 KiB), as the 128-row kernel
    __shared__ __attribute__((aligned(1024))) unsigned char smem[POOL];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int wm = w >> 1, wn = w & 1, c32 = lane & 31, h = lane >> 5;
    for (int i = tid; i < POOL / 16; i += 256) *(v4i *)(smem + i * 16) = *(const v4i *)(pattern + i * 16);
    __syncthreads();
    // the fragment addresses of gemm_dma_kernel (1-byte elements)
    const uint32_t a_lds = (wm * 64 + c32) * 64, a_sw = (c32 >> 2) & 3;
    const int ti16 = lane & 15, tch = (lane >> 4) & 1, trow = ti16 >> 1, thalf = ti16 & 1;
    uint32_t b_lds[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) b_lds[nb] = (16 * h + trow) * 256 + (((wn * 8 + nb * 2 + tch) ^ (2 * trow)) * 16) + thalf * 8;
    v16i acc[2][4];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][nb][r] = 0;
    v4i fa[2], fb[4];
    auto read_frags = [&](uint32_t stage, int kk) {
        const unsigned char *sa = smem + stage * 8192, *sb = smem + 3 * 8192 + stage * 16384;
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) fa[mb] = *(const v4i *)(sa + a_lds + mb * 32 * 64 + (((2 * kk + h) ^ a_sw) * 16));
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            const unsigned char *p = sb + b_lds[nb] + kk * (32 * 256);
            const v2i t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)p);
            const v2i t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((CATCOC_LDS v2i *)(p + 8 * 256));
            fb[nb] = v4i{t0.x, t0.y, t1.x, t1.y};
        }
    };
    read_frags(0, 0);
    uint32_t stage = 0;
    for (uint32_t s = 0; s < steps; ++s) {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            if constexpr (LDS_READS) read_frags(stage, kk);
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) acc[mb][nb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[mb], fb[nb], acc[mb][nb], 0, 0, 0);
        }
        stage = stage == 2 ? 0 : stage + 1;
    }
    int sum = 0;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) sum += acc[mb][nb][r];
    sink[blockIdx.x * 256 + tid] = sum;
}


// ---- peer-partial stream on its own ------------------------------------------------------------------------------
// What a reduce-scatter launch's kept tiles do after their main loops, and nothing else: one workgroup per 128x256 tile of
// a [rows, n] block (row pitch n floats) adds up `P` fp32 partials.  LAYOUT 0: accumulator layout, per peer and 32-row
// block 64 four-byte loads per lane, all awaited before they are added (the kept epilogue of the 128-row kernel).
// LAYOUT 1: row layout, sixteen-byte loads, eight per unit, D units in flight (the pipelined epilogue).
template <int I, int N_, typename F> __device__ __forceinline__ void probe_static_for(F &&f)
{
    if constexpr (I < N_) {
        f(std::integral_constant<int, I>{});
        probe_static_for<I + 1, N_>(f);
    }
}

__global__ void __launch_bounds__(256) probe_stream_acc_kernel(const float *const *peers, uint32_t nPeers, uint32_t n, float *out)
{
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, wm = w >> 1, wn = w & 1, c32 = lane & 31, h = lane >> 5;
    const uint32_t tilesPerRow = n / 256u, tr = blockIdx.x / tilesPerRow, tc = blockIdx.x % tilesPerRow;
    float acc[2][16][4];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) acc[mb][r][nb] = 0.f;
    for (uint32_t p = 0; p < nPeers; ++p) {
        const float *src = peers[p] + (size_t)(tr * 128 + wm * 64 + h * 4) * n + tc * 256 + wn * 128 + c32;
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
            float pv[16][4];
#pragma unroll
            for (int r = 0; r < 16; ++r)
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) pv[r][nb] = __builtin_nontemporal_load(src + (size_t)(mb * 32 + (r >> 2) * 8 + (r & 3)) * n + 32 * nb);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < 16; ++r)
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) acc[mb][r][nb] += pv[r][nb];
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float sum = 0;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) sum += acc[mb][r][nb];
    out[blockIdx.x * 256 + tid] = sum;
}

// (seven peers: the pipeline is unrolled over its 14 units per 32-row block)
template <int D>
__global__ void __launch_bounds__(256) probe_stream_row_kernel(const float *const *peers, uint32_t n, float *out)
{
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, wm = w >> 1, wn = w & 1, lrow = lane >> 5, chunk = lane & 31;
    const uint32_t tilesPerRow = n / 256u, tr = blockIdx.x / tilesPerRow, tc = blockIdx.x % tilesPerRow;
    float total = 0;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
        const size_t off = (size_t)(tr * 128 + wm * 64 + mb * 32 + lrow) * n + tc * 256 + wn * 128 + chunk * 4;
        v4f cur[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) cur[j] = v4f{0, 0, 0, 0};
        constexpr int U = 14;
        v4f buf[D][8];
        auto issue = [&](auto uc) {
            constexpr int u = decltype(uc)::value;
            const float *src = peers[u / 2] + off + (size_t)((u & 1) * 16) * n;
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) buf[u % D][jj] = __builtin_nontemporal_load((const v4f *)(src + (size_t)(2 * jj) * n));
        };
        probe_static_for<0, (D - 1 < U ? D - 1 : U)>(issue);
        probe_static_for<0, U>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (u + D - 1 < U) issue(std::integral_constant<int, u + D - 1>{});
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) cur[(u & 1) * 8 + jj] += buf[u % D][jj];
        });
        v4f sv = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 16; ++j) sv += cur[j];
        total += sv.x + sv.y + sv.z + sv.w;
    }
    out[blockIdx.x * 256 + tid] = total;
}

// ---- LDS and copy-path rates of a CU ---------------------------------------------------------------------------------
// Four waves per workgroup, `wgs` workgroups (256 = one per CU, 512 = two), 72 KiB of LDS each.  Per iteration and wave, by
// MODE bit: 1 -> eight 16-byte LDS reads (8 KiB); 2 -> sixteen transposing 8-byte reads (8 KiB); 4 -> six 1 KiB
// direct-to-LDS copies from a 24 KiB region of global memory that stays in the caches.  The reads are asm statements, so
// none of them is hoisted or merged.
template <int MODE>
__global__ void __launch_bounds__(256, 2) probe_lds_kernel(const unsigned char *src, uint32_t iters, int *sink)
{
    __shared__ __attribute__((aligned(1024))) unsigned char smem[72 * 1024];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    for (int i = tid; i < 72 * 1024 / 16; i += 256) *(v4i *)(smem + i * 16) = v4i{i, i, i, i};
    __syncthreads();
    const uint32_t lds0 = (uint32_t)(uintptr_t)(CATCOC_LDS unsigned char *)smem;
    const uint32_t ws = __builtin_amdgcn_readfirstlane((uint32_t)w);
    const unsigned char *g = src + (size_t)(ws * 6) * 1024 + lane * 16;
    v4i a128[8];
    v2i a64[16];
    for (uint32_t it = 0; it < iters; ++it) {
        const uint32_t base = lds0 + (it & 1u) * 32768u + ws * 8192u;
        if constexpr (MODE & 1) {
#pragma unroll
            for (int j = 0; j < 8; ++j) asm volatile("ds_read_b128 %0, %1" : "=v"(a128[j]) : "v"(base + j * 1024 + lane * 16));
        }
        if constexpr (MODE & 2) {
#pragma unroll
            for (int j = 0; j < 16; ++j) asm volatile("ds_read_b64_tr_b8 %0, %1" : "=v"(a64[j]) : "v"(base + j * 512 + lane * 8));
        }
        if constexpr (MODE & 4) {
#pragma unroll
            for (int j = 0; j < 6; ++j) dma16_at(g + j * 1024, lds0 + 65536 + ((ws * 6 + j) & 7u) * 1024);   // (the last 8 KiB: never read)
            CATCOC_WAIT_VMCNT(12);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    CATCOC_WAIT_VMCNT(0);
    int x = 0;
    if constexpr (MODE & 1) x ^= a128[0].x ^ a128[7].w;
    if constexpr (MODE & 2) x ^= a64[0].x ^ a64[15].y;
    sink[blockIdx.x * 256 + tid] = x;
}

// ---- a streaming neighbour on the CU ---------------------------------------------------------------------------------
// 512 workgroups with 72 KiB of LDS each, two per CU (workgroups w and w + 256 land on one CU; their HW_ID words are
// returned so that the caller can check).  The first 256 run the copy side of a main loop and time themselves: per step six
// 1 KiB direct-to-LDS copies per wave from a per-workgroup region that stays in L2, two steps ahead, a barrier and a pause of
// the length of a step's MFMAs.  The other 256 exit at once (mode 0) or, like a kept tile's epilogue, fetch batches of 64
// four-byte loads per lane and await each batch, from 4 MiB of their own each (mode 1: HBM) or from 64 KiB each (mode 2: L2).
__global__ void __launch_bounds__(256, 2) probe_neighbour_kernel(const unsigned char *hot, const float *big, uint32_t mode, uint32_t steps,
                                                                 float *sink, unsigned long long *ticks, uint32_t *hwid)
{
    __shared__ __attribute__((aligned(1024))) unsigned char smem[72 * 1024];
    const int tid = threadIdx.x, lane = tid & 63;
    const uint32_t ws = __builtin_amdgcn_readfirstlane((uint32_t)(tid >> 6));
    const uint32_t lds0 = (uint32_t)(uintptr_t)(CATCOC_LDS unsigned char *)smem;
    if (tid == 0) {
        uint32_t hw, xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        hwid[blockIdx.x] = ((hw >> 8) & 0xffu) | (xcc << 8);   // CU, shader array, shader engine; XCD
    }
    if (blockIdx.x < 256) {
        const unsigned char *g = hot + (size_t)blockIdx.x * 98304 + (ws * 6) * 1024 + lane * 16;
        const unsigned long long t0 = wall_clock64();
        auto issue = [&](uint32_t step) {
            const unsigned char *p = g + (step & 3u) * 24576;
#pragma unroll
            for (int j = 0; j < 6; ++j) dma16_at(p + j * 1024, lds0 + (step % 3u) * 24576 + (ws * 6 + j) * 1024);
        };
        issue(0);
        issue(1);
        for (uint32_t it = 0; it < steps; ++it) {
            CATCOC_WAIT_VMCNT(6);
            barrier_keep_vmem();
            issue(it + 2);
            __builtin_amdgcn_s_sleep(7);   // about 500 cycles
        }
        CATCOC_WAIT_VMCNT(0);
        const unsigned long long t1 = wall_clock64();
        if (tid == 0) ticks[blockIdx.x] = t1 - t0;   // 100 MHz ticks
    } else if (mode != 0) {
        const uint32_t v = blockIdx.x - 256;
        const float *src = mode == 1 ? big + (size_t)v * (1u << 20) : (const float *)(hot + 256 * 98304) + (size_t)v * 16384;
        const uint32_t span = mode == 1 ? (1u << 20) : 16384u;   // floats
        float acc = 0;
        for (uint32_t b = 0; b < steps / 2; ++b) {
            float pv[64];
            const float *p = src + (b * 16384u + ws * 4096u + lane) % span;
#pragma unroll
            for (int r = 0; r < 64; ++r) pv[r] = __builtin_nontemporal_load(p + r * 64);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < 64; ++r) acc += pv[r];
            __builtin_amdgcn_sched_barrier(0);
        }
        sink[v * 256 + tid] = acc;
    }
}

}  // namespace catcoc

extern "C" int catcoc_probe_mfma_int8(void *stream, uint32_t ldsReads, uint32_t steps, const uint8_t *pattern, uint8_t *sink)
{
    if (pattern == nullptr || sink == nullptr || (uintptr_t)pattern % 16 != 0) return 1;
    if (ldsReads) hipLaunchKernelGGL((catcoc::probe_mfma_kernel<true>), dim3(512), dim3(256), 0, (hipStream_t)stream, pattern, steps, (int *)sink);
    else hipLaunchKernelGGL((catcoc::probe_mfma_kernel<false>), dim3(512), dim3(256), 0, (hipStream_t)stream, pattern, steps, (int *)sink);
    return (int)hipGetLastError();
}

extern "C" int catcoc_probe_peer_stream(void *stream, uint32_t layout, uint32_t depth, const void *const *peers, uint32_t nPeers, uint32_t rows,
                                        uint32_t n, uint8_t *sink)
{
    if (peers == nullptr || sink == nullptr || rows % 128 != 0 || n % 256 != 0 || rows == 0 || n == 0) return 1;
    const dim3 grid((rows / 128) * (n / 256)), block(256);
    hipStream_t s = (hipStream_t)stream;
    if (layout == 0) {
        hipLaunchKernelGGL(catcoc::probe_stream_acc_kernel, grid, block, 0, s, (const float *const *)peers, nPeers, n, (float *)sink);
    } else {
        if (nPeers != 7) return 1;
        switch (depth) {
            case 2: hipLaunchKernelGGL(catcoc::probe_stream_row_kernel<2>, grid, block, 0, s, (const float *const *)peers, n, (float *)sink); break;
            case 3: hipLaunchKernelGGL(catcoc::probe_stream_row_kernel<3>, grid, block, 0, s, (const float *const *)peers, n, (float *)sink); break;
            case 4: hipLaunchKernelGGL(catcoc::probe_stream_row_kernel<4>, grid, block, 0, s, (const float *const *)peers, n, (float *)sink); break;
            case 6: hipLaunchKernelGGL(catcoc::probe_stream_row_kernel<6>, grid, block, 0, s, (const float *const *)peers, n, (float *)sink); break;
            default: return 1;
        }
    }
    return (int)hipGetLastError();
}

extern "C" int catcoc_probe_lds(void *stream, uint32_t mode, uint32_t workgroups, uint32_t iters, const uint8_t *src, uint8_t *sink)
{
    if (src == nullptr || sink == nullptr || (uintptr_t)src % 16 != 0 || workgroups == 0 || workgroups > 512) return 1;
    const dim3 grid(workgroups), block(256);
    hipStream_t s = (hipStream_t)stream;
    switch (mode) {
        case 1: hipLaunchKernelGGL(catcoc::probe_lds_kernel<1>, grid, block, 0, s, src, iters, (int *)sink); break;
        case 2: hipLaunchKernelGGL(catcoc::probe_lds_kernel<2>, grid, block, 0, s, src, iters, (int *)sink); break;
        case 3: hipLaunchKernelGGL(catcoc::probe_lds_kernel<3>, grid, block, 0, s, src, iters, (int *)sink); break;
        case 4: hipLaunchKernelGGL(catcoc::probe_lds_kernel<4>, grid, block, 0, s, src, iters, (int *)sink); break;
        case 7: hipLaunchKernelGGL(catcoc::probe_lds_kernel<7>, grid, block, 0, s, src, iters, (int *)sink); break;
        default: return 1;
    }
    return (int)hipGetLastError();
}

extern "C" int catcoc_probe_neighbour(void *stream, uint32_t mode, uint32_t steps, const uint8_t *hot, const uint8_t *big, uint8_t *sink,
                                      uint64_t *ticks, uint32_t *hwid)
{
    if (hot == nullptr || big == nullptr || sink == nullptr || ticks == nullptr || hwid == nullptr || mode > 2 || (uintptr_t)hot % 16 != 0) return 1;
    hipLaunchKernelGGL(catcoc::probe_neighbour_kernel, dim3(512), dim3(256), 0, (hipStream_t)stream, hot, (const float *)big, mode, steps, (float *)sink,
                       (unsigned long long *)ticks, hwid);
    return (int)hipGetLastError();
}
