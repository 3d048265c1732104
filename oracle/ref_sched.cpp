// Driver that compiles the REFERENCE's tile schedulers, in place, into
// oracle/_ref/libcatcoc_ref_sched.so.  Test infrastructure only.
//
// The scheduler headers mark their methods with the Ascend compiler's function
// attributes (3rdparty/catlass/include/catlass/detail/macros.hpp:15-21).  The
// Makefile defines those three attribute macros as plain `inline` on the g++
// command line; no header is replaced or added, and the index arithmetic that is
// compiled is the reference's own text:
//   GemmIdentityBlockSwizzle, SplitkGemmIdentityBlockSwizzle
//        3rdparty/catlass/include/catlass/gemm/block/block_swizzle.hpp:24-236
//   GemmIdentityBlockSwizzleAllGather
//        include/catcoc/dgemm/block/block_swizzle_allgather.hpp:28-117
// BlockCommSwizzle (include/catcoc/comm_epilogue/block/comm_block_swizzle.hpp)
// includes the Ascend toolkit's kernel_operator.h through catcoc.hpp and is
// therefore NOT built here.
#include <cstdint>
#include <algorithm>

#include "catlass/gemm/block/block_swizzle.hpp"
#include "catcoc/dgemm/block/block_swizzle_allgather.hpp"

using namespace Catlass;

namespace {

template <uint32_t OFF, uint32_t DIR>
void BaseCoord(uint32_t M, uint32_t N, uint32_t m0, uint32_t n0, uint32_t task, uint32_t *o)
{
    Gemm::Block::GemmIdentityBlockSwizzle<OFF, DIR> s(GemmCoord{M, N, 1u}, MatrixCoord{m0, n0});
    GemmCoord c = s.GetBlockCoord(task);
    GemmCoord a = s.GetActualBlockShape(c);
    o[0] = c.m(); o[1] = c.n(); o[2] = a.m(); o[3] = a.n(); o[4] = s.GetCoreLoops();
}

template <uint32_t OFF, uint32_t DIR>
void SplitCoord(uint32_t M, uint32_t N, uint32_t K, uint32_t m0, uint32_t n0, uint32_t k0, uint32_t f,
                uint32_t task, uint32_t *o)
{
    Gemm::Block::SplitkGemmIdentityBlockSwizzle<OFF, DIR> s(GemmCoord{M, N, K}, GemmCoord{m0, n0, k0}, f);
    GemmCoord c = s.GetBlockCoord(task);
    uint32_t slice = s.GetSplitkSliceIdx(task);
    GemmCoord a = s.GetActualBlockShape(c, slice);
    o[0] = c.m(); o[1] = c.n(); o[2] = c.k(); o[3] = slice; o[4] = a.m(); o[5] = a.n(); o[6] = a.k();
    o[7] = s.GetCoreLoops();
}

template <uint32_t OFF, uint32_t DIR>
void AgCoord(uint32_t P, uint32_t commInterval, uint32_t mLocal, uint32_t N, uint32_t m0, uint32_t n0,
             uint32_t task, uint32_t *o)
{
    Catcoc::DGemm::Block::GemmIdentityBlockSwizzleAllGather<OFF, DIR> s(
        P, commInterval, GemmCoord{mLocal, N, 1u}, MatrixCoord{m0, n0});
    GemmCoord c = s.GetBlockCoord(task);
    GemmCoord a = s.GetActualBlockShape(c);
    o[0] = c.m(); o[1] = c.n(); o[2] = a.m(); o[3] = a.n(); o[4] = s.GetCoreLoops();
}

}  // namespace

#define DISPATCH(FN, ...)                                              \
    switch (off * 2 + dir) {                                           \
        case 1 * 2 + 0: FN<1, 0>(__VA_ARGS__); return 1;               \
        case 1 * 2 + 1: FN<1, 1>(__VA_ARGS__); return 1;               \
        case 2 * 2 + 0: FN<2, 0>(__VA_ARGS__); return 1;               \
        case 2 * 2 + 1: FN<2, 1>(__VA_ARGS__); return 1;               \
        case 3 * 2 + 0: FN<3, 0>(__VA_ARGS__); return 1;               \
        case 3 * 2 + 1: FN<3, 1>(__VA_ARGS__); return 1;               \
        case 4 * 2 + 0: FN<4, 0>(__VA_ARGS__); return 1;               \
        case 4 * 2 + 1: FN<4, 1>(__VA_ARGS__); return 1;               \
        case 7 * 2 + 0: FN<7, 0>(__VA_ARGS__); return 1;               \
        case 7 * 2 + 1: FN<7, 1>(__VA_ARGS__); return 1;               \
        default: return 0;                                             \
    }

extern "C" {

// o[5]: mIdx, nIdx, mActual, nActual, coreLoops.  Returns 0 if (off,dir) is not instantiated.
__attribute__((visibility("default")))
int ref_swizzle_coord(uint32_t off, uint32_t dir, uint32_t M, uint32_t N, uint32_t m0, uint32_t n0,
                      uint32_t task, uint32_t *o)
{
    DISPATCH(BaseCoord, M, N, m0, n0, task, o)
}

// o[8]: mIdx, nIdx, kIdx, slice, mActual, nActual, kActual, coreLoops.
__attribute__((visibility("default")))
int ref_splitk_coord(uint32_t off, uint32_t dir, uint32_t M, uint32_t N, uint32_t K,
                     uint32_t m0, uint32_t n0, uint32_t k0, uint32_t f, uint32_t task, uint32_t *o)
{
    DISPATCH(SplitCoord, M, N, K, m0, n0, k0, f, task, o)
}

// o[5]: mIdx (over all ranks), nIdx, mActual, nActual, coreLoops.
__attribute__((visibility("default")))
int ref_allgather_coord(uint32_t off, uint32_t dir, uint32_t P, uint32_t commInterval, uint32_t mLocal,
                        uint32_t N, uint32_t m0, uint32_t n0, uint32_t task, uint32_t *o)
{
    DISPATCH(AgCoord, P, commInterval, mLocal, N, m0, n0, task, o)
}

}  // extern "C"
