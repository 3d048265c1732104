// Measurement helper, not an operator: the inner loop of the 128x256 W8A8 kernel with the global-memory side taken
// away.  512 workgroups of four waves (two per CU, as the real launch), each wave issuing the main loop's sixteen
// 32x32x32 int8 MFMAs per k step, with or without the LDS fragment reads that feed them (four 16-byte reads for A,
// sixteen transposing 8-byte reads for B per step), on whatever bytes the caller puts into LDS.  What it sustains is
// the ceiling of the matrix pipes for that data on the box at hand: the pipes are power-limited, and how hard depends
// on how many operand bits toggle.  bench.py --mode ceiling reports it.
#include <hip/hip_runtime.h>
#include <stdint.h>

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

}  // namespace catcoc

extern "C" int catcoc_probe_mfma_int8(void *stream, uint32_t ldsReads, uint32_t steps, const uint8_t *pattern, uint8_t *sink)
{
    if (pattern == nullptr || sink == nullptr || (uintptr_t)pattern % 16 != 0) return 1;
    if (ldsReads) hipLaunchKernelGGL((catcoc::probe_mfma_kernel<true>), dim3(512), dim3(256), 0, (hipStream_t)stream, pattern, steps, (int *)sink);
    else hipLaunchKernelGGL((catcoc::probe_mfma_kernel<false>), dim3(512), dim3(256), 0, (hipStream_t)stream, pattern, steps, (int *)sink);
    return (int)hipGetLastError();
}
