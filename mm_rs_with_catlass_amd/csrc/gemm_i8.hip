// Instantiates the fused GEMM kernels for int8 operands.
#include "gemm_dma_kernel.h"
#include "gemm_fused_kernel.h"

namespace catcoc {
int launch_gemm_i8(const GemmArgs &args, int variant, bool edge, void *stream)
{
    return launch_dt<DT_I8>(args, variant, edge, stream);
}

// Full-tile paths with direct-to-LDS copies (see gemm_dma_kernel.h for their requirements):
// m0 = 128 (4 waves, two workgroups per CU) or m0 = 256 (8 waves).
int launch_gemm_dma_i8(const GemmArgs &args, void *stream)
{
    if (args.sched.m0 == 256) {
        const dim3 grid(launch_positions(args)), block(512);
        const bool ragged = (args.flags & GF_RAGGED) != 0;   // edge tiles moved inwards, as on 128-row tiles
        if (args.transB && ragged) hipLaunchKernelGGL((gemm_dma_kernel<DT_I8, 4, true, false, true>), grid, block, 0, (hipStream_t)stream, args);
        else if (args.transB) hipLaunchKernelGGL((gemm_dma_kernel<DT_I8, 4, true>), grid, block, 0, (hipStream_t)stream, args);
        else if (ragged) hipLaunchKernelGGL((gemm_dma_kernel<DT_I8, 4, false, false, true>), grid, block, 0, (hipStream_t)stream, args);
        else hipLaunchKernelGGL((gemm_dma_kernel<DT_I8, 4>), grid, block, 0, (hipStream_t)stream, args);
        return (int)hipGetLastError();
    }
    if (args.flags & GF_ROW_MASK) {   // explicit kept rows in whole 32-row blocks
        const uint32_t wgs = launch_positions(args) * (args.splitK > 1 ? args.splitK : 1u);
        // Launches of at most 512 workgroups (one or two rounds of one workgroup per CU) run the six-stage ring (the whole
        // LDS of the CU) on EIGHT waves, 32 rows of the tile each, with the peers' partials pipelined through register buffers:
        //  - two waves per SIMD overlap what a wave alone on its SIMD pays one after the other in every k step (barrier, LDS
        //    latency, copy issue).  Same box, variants alternating, K = N = 8192, operands from HBM, the library's own k
        //    slices, four -> eight waves: M = 256 41.5 -> 33.9 us, M = 512 60.6 -> 53.4, M = 1024 98.4 -> 92.4 (B as [n,k]:
        //    43.7 -> 36.4, 66.4 -> 59.3, 112.2 -> 104.9);
        //  - the kept tiles of such a launch are few and their peer stream ends the launch: fetched batch by batch into
        //    registers (the three-stage kernel) it takes 35 us at M = 512 with seven peers, pipelined 8-10.  Three-stage
        //    kernel -> this one, operands of less than 48 MB: M = 512, K = 4096 / 2048 79.9 -> 35.9 / 70.8 -> 27.4 us,
        //    M = 256, K = 4096 74.7 -> 24.8, M = 1024, K = 2048 80.2 -> 42.0, M = 512, K = 8192, N = 4096 81.7 -> 36.9.
        // More workgroups, eight-wave ring against the three-stage kernel with two workgroups per CU (K = N = 8192): 384 (M = 1536)
        // 156.1 -> 142.1 us, 512 (M = 512 in four k slices / M = 2048) 102.6 -> 55.8 / 174.7 -> 168.0, 1024 (M = 4096) 293.3 -> 334.2.
        // A goes in pairs of k steps from 128 steps per workgroup on (K = 16384, M = 512, one / two slices: 142.5 -> 121.1 /
        // 85.5 -> 83.2 us; B as [n,k] 152.6 -> 139.0 / 106.4 -> 96.6; shorter loops lose 2-5 % with pairs).
        if (wgs <= 512u) {
            const uint32_t stepsPerWg = args.K / 64u / (args.splitK > 1 ? args.splitK : 1u);
            const bool pairs = stepsPerWg >= 128u && deep_ring_pairs(args, 1u);
            if (args.transB && pairs)
                hipLaunchKernelGGL((gemm_dma_kernel<DT_I8, 2, true, true, false, false, 6, true, true, true>), dim3(wgs), dim3(512), 0, (hipStream_t)stream, args);
            else if (args.transB)
                hipLaunchKernelGGL((gemm_dma_kernel<DT_I8, 2, true, true, false, false, 6, true, false, true>), dim3(wgs), dim3(512), 0, (hipStream_t)stream, args);
            else if (pairs)
                hipLaunchKernelGGL((gemm_dma_kernel<DT_I8, 2, false, true, false, false, 6, true, true, true>), dim3(wgs), dim3(512), 0, (hipStream_t)stream, args);
            else
                hipLaunchKernelGGL((gemm_dma_kernel<DT_I8, 2, false, true, false, false, 6, true, false, true>), dim3(wgs), dim3(512), 0, (hipStream_t)stream, args);
        }
        else if (args.transB)
            hipLaunchKernelGGL((gemm_dma_kernel<DT_I8, 2, true, true>), dim3(wgs), dim3(256), 0, (hipStream_t)stream, args);
        else
            hipLaunchKernelGGL((gemm_dma_kernel<DT_I8, 2, false, true>), dim3(wgs), dim3(256), 0, (hipStream_t)stream, args);
        return (int)hipGetLastError();
    }
    return launch_dma_128<DT_I8>(args, (hipStream_t)stream);
}
}  // namespace catcoc
