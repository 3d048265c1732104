// Instantiates the fused GEMM kernels for one element type.
#include "gemm_fused_kernel.h"

namespace catcoc {
int launch_gemm_bf16(const GemmArgs &args, int variant, bool edge, void *stream)
{
    return launch_dt<DT_BF16>(args, variant, edge, stream);
}
}  // namespace catcoc
