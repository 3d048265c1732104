// Instantiates the skinny-M W8A8 kernels: split K, and whole K for weights stored as [n,k].
#include "gemm_decode_nk_kernel.h"
#include "gemm_splitk_kernel.h"

namespace catcoc {
// rowBlocks: 32-row blocks of A a tile stages (1, 2 or 4); grid = tiles x k slices.
int launch_gemm_splitk_i8(const GemmArgs &args, int rowBlocks, uint32_t tasks, void *stream)
{
    const dim3 grid(tasks), block(256), block8(512);
    // k slices are whole 256-byte k tiles except the last one, which takes what is left of K: with K a multiple of 128
    // every slice is a whole number of pairs of 64-byte steps, and A can be fetched as whole 128-byte lines.  128-row
    // tiles on pairs run eight waves, one of each SIMD's two per step of a pair (measured against four waves, launches
    // alternating: 128 rows 29.1 -> 27.4 us, 96 rows 29.2 -> 27.0; 64-row tiles do not gain, 22.2 -> 22.4).
    const bool pairs = args.K % 128u == 0;
    hipStream_t s = (hipStream_t)stream;
    if (args.transB) {   // B as [n][k]
        if (rowBlocks == 1) hipLaunchKernelGGL((gemm_splitk_kernel<1, false, true>), grid, block, 0, s, args);
        else if (rowBlocks == 2 && pairs) hipLaunchKernelGGL((gemm_splitk_kernel<2, true, true>), grid, block, 0, s, args);
        else if (rowBlocks == 2) hipLaunchKernelGGL((gemm_splitk_kernel<2, false, true>), grid, block, 0, s, args);
        else if (pairs) hipLaunchKernelGGL((gemm_splitk_kernel<4, true, true, true>), grid, block8, 0, s, args);
        else hipLaunchKernelGGL((gemm_splitk_kernel<4, false, true>), grid, block, 0, s, args);
        return (int)hipGetLastError();
    }
    if (rowBlocks == 1) hipLaunchKernelGGL((gemm_splitk_kernel<1>), grid, block, 0, s, args);
    else if (rowBlocks == 2 && pairs) hipLaunchKernelGGL((gemm_splitk_kernel<2, true>), grid, block, 0, s, args);
    else if (rowBlocks == 2) hipLaunchKernelGGL((gemm_splitk_kernel<2>), grid, block, 0, s, args);
    else if (pairs) hipLaunchKernelGGL((gemm_splitk_kernel<4, true, false, true>), grid, block8, 0, s, args);
    else hipLaunchKernelGGL((gemm_splitk_kernel<4>), grid, block, 0, s, args);
    return (int)hipGetLastError();
}

// At most 32 rows of A against B as [n][k] (K in whole 128-byte chunks, N in whole 32-column strips): one workgroup per strip.
int launch_gemm_decode_nk_i8(const GemmArgs &args, void *stream)
{
    const dim3 grid(args.N / 32u), block(256);
    hipStream_t s = (hipStream_t)stream;
    if (args.M > 32u || args.K % 128u != 0 || args.N % 32u != 0 || args.K == 0) return (int)hipErrorInvalidValue;
    if (args.M <= 8) hipLaunchKernelGGL((gemm_decode_nk_kernel<1>), grid, block, 0, s, args);
    else if (args.M <= 16) hipLaunchKernelGGL((gemm_decode_nk_kernel<2>), grid, block, 0, s, args);
    else hipLaunchKernelGGL((gemm_decode_nk_kernel<4>), grid, block, 0, s, args);
    return (int)hipGetLastError();
}
}  // namespace catcoc
