// Instantiates the fused GEMM kernels for one element type.
#include "gemm_dma_kernel.h"
#include "gemm_fused_kernel.h"

namespace catcoc {
int launch_gemm_f16(const GemmArgs &args, int variant, bool edge, void *stream)
{
    return launch_dt<DT_F16>(args, variant, edge, stream);
}

// Full-tile path with direct-to-LDS copies (row-major operands, see gemm_dma_kernel.h): m0 = 128 or 256.
int launch_gemm_dma_f16(const GemmArgs &args, void *stream)
{
    if (args.sched.m0 == 256) {
        const dim3 grid(launch_positions(args)), block(512);
        const bool ragged = (args.flags & GF_RAGGED) != 0;   // edge tiles moved inwards, as on 128-row tiles
        if (args.transB && ragged) hipLaunchKernelGGL((gemm_dma_kernel<DT_F16, 4, true, false, true>), grid, block, 0, (hipStream_t)stream, args);
        else if (args.transB) hipLaunchKernelGGL((gemm_dma_kernel<DT_F16, 4, true>), grid, block, 0, (hipStream_t)stream, args);
        else if (ragged) hipLaunchKernelGGL((gemm_dma_kernel<DT_F16, 4, false, false, true>), grid, block, 0, (hipStream_t)stream, args);
        else hipLaunchKernelGGL((gemm_dma_kernel<DT_F16, 4>), grid, block, 0, (hipStream_t)stream, args);
        return (int)hipGetLastError();
    }
    return launch_dma_128<DT_F16>(args, (hipStream_t)stream);
}
}  // namespace catcoc
