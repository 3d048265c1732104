// Instantiates the fused GEMM kernels for one element type.
#include "gemm_fused_kernel.h"

namespace catcoc {
int launch_gemm_i8(const GemmArgs &args, int variant, bool edge, void *stream)
{
    return launch_dt<DT_I8>(args, variant, edge, stream);
}
}  // namespace catcoc
