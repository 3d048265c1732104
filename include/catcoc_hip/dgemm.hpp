// catcoc_hip/dgemm.hpp -- the reference's kernel-template entry points as a thin C++17 facade over the C ABI of
// libcatcoc_hip.so (catcoc_hip.h).  Host code written against
//     Catcoc::DGemm::Kernel::{MatmulAllReduce, AllGatherMatmul, MatmulReduceScatter, QuantMatmulReduceScatter}
// (include/catcoc/dgemm/kernel/*.hpp of the reference) keeps its type definitions and its `Params{...}` construction;
// the one difference is where the kernel object is called: the reference calls it inside a __global__ wrapper on the
// device, here `kernel(params, stream)` is a HOST call that validates, picks the gfx950 kernel and enqueues it.
//
// What each template argument means here:
//   BlockMmad<Policy, L1TileShape, L0TileShape, AType, BType, CType[, BiasType]>
//       L1TileShape::M/N/K -> CocTilingParams.m0/n0/k0; element types pick int8 / fp16 / bf16 kernels; a ColumnMajor
//       AType / BType means the operand is stored transposed (transA / transB of the launchers).
//   BlockScheduler = GemmIdentityBlockSwizzle<offset, direction>  -> the tile order (descriptor swizzle fields).
//   CommBlockEpilogue<...>::Params  -> the comm-epilogue chunking (commDataSplit, commNpuSplit, commBlockM, commTileM),
//       validated like the reference does and otherwise unused: the reduce runs in the GEMM's own epilogue.
//   ptrSymmetric -> a CatcocSymmetricDesc in host memory (which rank this GPU plays, where the peers' staged partials
//       or A shards live), standing in for the symmetric heap + shmem_my_pe()/shmem_n_pes().
// Nothing here touches the GPU by itself; every call ends in one of the extern "C" launchers.
#ifndef CATCOC_HIP_DGEMM_HPP
#define CATCOC_HIP_DGEMM_HPP

#include <cstddef>
#include <cstdint>
#include <type_traits>

#include "../catcoc_hip.h"

#ifndef GM_ADDR
using GM_ADDR = uint8_t *;   // the reference's global-memory byte pointer
#endif

// 16-bit element tags.  They only select kernels; host code never does arithmetic on them.
struct bfloat16_t { uint16_t bits; };
#if !defined(HIP_INCLUDE_HIP_AMD_DETAIL_HIP_FP16_H) && !defined(CATCOC_HIP_NO_GLOBAL_HALF)
struct half { uint16_t bits; };
#endif

namespace Catlass {

enum class Status { kSuccess, kInvalid };   // 3rdparty/catlass/include/catlass/status.hpp:16

template <class T>
constexpr T CeilDiv(T a, T b) { return (a + b - 1) / b; }
template <class T>
constexpr T RoundUp(T a, T b) { return CeilDiv(a, b) * b; }

// 3rdparty/catlass/include/catlass/gemm_coord.hpp, matrix_coord.hpp: (m, n, k) and (row, column)
struct MatrixCoord {
    uint32_t v[2]{0, 0};
    constexpr MatrixCoord() = default;
    constexpr MatrixCoord(uint32_t r, uint32_t c) : v{r, c} {}
    constexpr uint32_t row() const { return v[0]; }
    constexpr uint32_t column() const { return v[1]; }
    constexpr uint32_t operator[](int i) const { return v[i]; }
};
struct GemmCoord {
    uint32_t v[3]{0, 0, 0};
    constexpr GemmCoord() = default;
    constexpr GemmCoord(uint32_t m, uint32_t n, uint32_t k) : v{m, n, k} {}
    constexpr uint32_t m() const { return v[0]; }
    constexpr uint32_t n() const { return v[1]; }
    constexpr uint32_t k() const { return v[2]; }
    constexpr MatrixCoord GetCoordMN() const { return {v[0], v[1]}; }
    constexpr GemmCoord operator*(GemmCoord const &o) const { return {v[0] * o.v[0], v[1] * o.v[1], v[2] * o.v[2]}; }
    constexpr GemmCoord operator/(GemmCoord const &o) const { return {v[0] / o.v[0], v[1] / o.v[1], v[2] / o.v[2]}; }
};
template <class T = uint32_t>
constexpr MatrixCoord MakeCoord(T a, T b) { return {(uint32_t)a, (uint32_t)b}; }
template <class T = uint32_t>
constexpr GemmCoord MakeCoord(T a, T b, T c) { return {(uint32_t)a, (uint32_t)b, (uint32_t)c}; }

template <uint32_t M_, uint32_t N_, uint32_t K_>
struct GemmShape {
    static constexpr uint32_t M = M_, N = N_, K = K_;
    static constexpr GemmCoord ToCoord() { return {M, N, K}; }
};
template <uint32_t ROW_, uint32_t COLUMN_>
struct MatrixShape {
    static constexpr uint32_t ROW = ROW_, COLUMN = COLUMN_;
    static constexpr MatrixCoord ToCoord() { return {ROW, COLUMN}; }
};

namespace layout {
// 3rdparty/catlass/include/catlass/layout/matrix.hpp:22-140 (shape + leading dimension), layout/vector.hpp
struct RowMajor {
    static constexpr bool kTransposed = false;
    uint32_t rows{0}, cols{0};
    int64_t ldm{0};
    constexpr RowMajor() = default;
    constexpr RowMajor(uint32_t r, uint32_t c) : rows(r), cols(c), ldm(c) {}
    constexpr RowMajor(uint32_t r, uint32_t c, int64_t ld) : rows(r), cols(c), ldm(ld) {}
    constexpr int64_t GetOffset(MatrixCoord const &c) const { return (int64_t)c.row() * ldm + c.column(); }
};
struct ColumnMajor {
    static constexpr bool kTransposed = true;
    uint32_t rows{0}, cols{0};
    int64_t ldm{0};
    constexpr ColumnMajor() = default;
    constexpr ColumnMajor(uint32_t r, uint32_t c) : rows(r), cols(c), ldm(r) {}
    constexpr ColumnMajor(uint32_t r, uint32_t c, int64_t ld) : rows(r), cols(c), ldm(ld) {}
    constexpr int64_t GetOffset(MatrixCoord const &c) const { return (int64_t)c.column() * ldm + c.row(); }
};
struct VectorLayout {
    uint32_t size{0};
    constexpr VectorLayout() = default;
    constexpr VectorLayout(uint32_t n) : size(n) {}
};
}  // namespace layout

namespace Arch { struct AtlasA2 {}; }   // accepted as a selector; the code runs on gfx950

namespace Gemm {

template <class Element_, class Layout_>
struct GemmType {
    using Element = Element_;
    using Layout = Layout_;
};

// 3rdparty/catlass/include/catlass/gemm/dispatch_policy.hpp:31-35,108-112: the two policies the communication kernels
// use; the bias variant adds an int32 bias[n] to the accumulators
template <bool ENABLE_UNIT_FLAG_ = false>
struct MmadAtlasA2Pingpong {
    static constexpr uint32_t STAGES = 2;
    static constexpr bool ENABLE_UNIT_FLAG = ENABLE_UNIT_FLAG_;
    static constexpr bool HAS_BIAS = false;
};
template <bool ENABLE_UNIT_FLAG_ = false>
struct MmadAtlasA2PingpongBias {
    static constexpr uint32_t STAGES = 2;
    static constexpr bool ENABLE_UNIT_FLAG = ENABLE_UNIT_FLAG_;
    static constexpr bool HAS_BIAS = true;
};

namespace Block {

struct NoBias { using Element = void; using Layout = layout::VectorLayout; };

// 3rdparty/catlass/include/catlass/gemm/block/block_mmad.hpp: here a bundle of types, the MAC loop itself is the
// library's MFMA kernel
template <class DispatchPolicy_, class L1TileShape_, class L0TileShape_, class AType_, class BType_, class CType_,
          class BiasType_ = NoBias>
struct BlockMmad {
    using DispatchPolicy = DispatchPolicy_;
    using ArchTag = Arch::AtlasA2;
    using L1TileShape = L1TileShape_;
    using L0TileShape = L0TileShape_;
    using ElementA = typename AType_::Element;
    using LayoutA = typename AType_::Layout;
    using ElementB = typename BType_::Element;
    using LayoutB = typename BType_::Layout;
    using ElementC = typename CType_::Element;
    using LayoutC = typename CType_::Layout;
    using ElementBias = typename BiasType_::Element;
    using LayoutBias = typename BiasType_::Layout;
};

// GemmIdentityBlockSwizzle<offset, direction> (3rdparty/catlass/include/catlass/gemm/block/block_swizzle.hpp:24-125);
// the coordinates come from the same integer code the kernels run, through the C ABI
template <uint32_t SwizzleOffset = 1, uint32_t SwizzleDirection = 0>
struct GemmIdentityBlockSwizzle {
    static constexpr uint32_t OFFSET = SwizzleOffset, DIRECTION = SwizzleDirection;
    GemmCoord problemShape;
    MatrixCoord tileMN, loopsMN;
    GemmIdentityBlockSwizzle() = default;
    GemmIdentityBlockSwizzle(GemmCoord const &problemShape_, MatrixCoord const &tileMN_)
        : problemShape(problemShape_), tileMN(tileMN_),
          loopsMN(CeilDiv(problemShape_.m(), tileMN_.row()), CeilDiv(problemShape_.n(), tileMN_.column())) {}
    uint32_t GetCoreLoops() const { return loopsMN.row() * loopsMN.column(); }
    GemmCoord GetBlockCoord(uint32_t taskIdx) const
    {
        uint32_t m = 0, n = 0;
        catcoc_swizzle_block_coord(OFFSET, DIRECTION, loopsMN.row(), loopsMN.column(), taskIdx, &m, &n);
        return {m, n, 0};
    }
    GemmCoord GetActualBlockShape(GemmCoord const &blockCoord) const
    {
        const uint32_t mAct = blockCoord.m() == loopsMN.row() - 1 ? problemShape.m() - blockCoord.m() * tileMN.row() : tileMN.row();
        const uint32_t nAct = blockCoord.n() == loopsMN.column() - 1 ? problemShape.n() - blockCoord.n() * tileMN.column() : tileMN.column();
        return {mAct, nAct, problemShape.k()};
    }
};

}  // namespace Block
}  // namespace Gemm

namespace Epilogue {

template <uint32_t UB_STAGES_>
struct EpilogueAtlasA2PerTokenDequant { static constexpr uint32_t UB_STAGES = UB_STAGES_; };

namespace Tile {
struct EpilogueIdentityTileSwizzle {};
template <class... T> struct TileRowBroadcastMul {};
template <class ArchTag, class ComputeType, uint32_t N> struct TileBroadcastOneBlk {};
template <class... T> struct TileOneBlkColumnBroadcastMul {};
template <class... T> struct TileCopy {};
}  // namespace Tile

namespace Block {
// BlockEpilogue<EpilogueAtlasA2PerTokenDequant, ...> (3rdparty/catlass/include/catlass/epilogue/block/
// block_epilogue_per_token_dequant.hpp:339-640, float-scale specialisation): the per-channel scale is applied first,
// then the per-token scale, then one rounding to the 16-bit output type.  The tile helpers are accepted and ignored.
template <class DispatchPolicy, class CType_, class ScaleType_, class PerTokenScaleType_, class DType_, class... TileOps>
struct BlockEpilogue {
    using ElementC = typename CType_::Element;
    using ElementScale = typename ScaleType_::Element;
    using ElementPerTokenScale = typename PerTokenScaleType_::Element;
    using ElementD = typename DType_::Element;
    using LayoutD = typename DType_::Layout;
    struct Params {
        ElementScale *ptrScale{nullptr};
        layout::VectorLayout layoutScale;
        ElementPerTokenScale *ptrPerTokenScale{nullptr};   // first kept row's scale (the reference pre-offsets by rank * m / P)
        layout::VectorLayout layoutPerTokenScale;
        ElementD *ptrD{nullptr};
        LayoutD layoutD;
        Params() = default;
        Params(ElementScale *ptrScale_, layout::VectorLayout const &layoutScale_, ElementPerTokenScale *ptrPerTokenScale_,
               layout::VectorLayout const &layoutPerTokenScale_, ElementD *ptrD_, LayoutD const &layoutD_)
            : ptrScale(ptrScale_), layoutScale(layoutScale_), ptrPerTokenScale(ptrPerTokenScale_),
              layoutPerTokenScale(layoutPerTokenScale_), ptrD(ptrD_), layoutD(layoutD_) {}
    };
};
}  // namespace Block
}  // namespace Epilogue
}  // namespace Catlass

namespace Catcoc {

using Catlass::GemmCoord;
using Catlass::MatrixCoord;

namespace detail {
enum class CopyMode { P2P, Scatter, Gather };   // include/catcoc/detail/remote_copy_type.hpp:6-7
enum class CopyDirect { Put, Get };

template <class T> struct ElementCode;          // element type -> CocDataType of the C ABI
template <> struct ElementCode<int8_t> { static constexpr int value = INT8; };
template <> struct ElementCode<::bfloat16_t> { static constexpr int value = BF16; };
#if !defined(HIP_INCLUDE_HIP_AMD_DETAIL_HIP_FP16_H) && !defined(CATCOC_HIP_NO_GLOBAL_HALF)
template <> struct ElementCode<::half> { static constexpr int value = FP16; };
#else
template <> struct ElementCode<__half> { static constexpr int value = FP16; };
#endif
}  // namespace detail

namespace CommEpilogue {

// include/catcoc/comm_epilogue/comm_dispatch_policy.hpp:21-36
template <uint32_t UB_STAGES_, detail::CopyMode CopyMode_, bool IsDynamic_ = false>
struct EpilogueAtlasA2CommToLocalMem {
    static constexpr uint32_t UB_STAGES = UB_STAGES_;
    static constexpr detail::CopyMode COPY_MODE = CopyMode_;
    static constexpr bool IS_DYNAMIC = IsDynamic_;
};
template <uint32_t UB_STAGES_, detail::CopyMode CopyMode_, bool IsDynamic_ = false>
struct EpilogueAtlasA2CommToShareMem {
    static constexpr uint32_t UB_STAGES = UB_STAGES_;
    static constexpr detail::CopyMode COPY_MODE = CopyMode_;
    static constexpr bool IS_DYNAMIC = IsDynamic_;
};

namespace Tile {
template <class ArchTag, class SrcType, class DstType, detail::CopyDirect Direct>
struct TileRemoteCopy { static constexpr detail::CopyDirect RemoteCopyDirect = Direct; };
}  // namespace Tile

namespace Block {

// BlockCommSwizzle<direction, deterministic> (include/catcoc/comm_epilogue/block/comm_block_swizzle.hpp:25-215):
// comm task -> (data block, peer rank).  The deterministic variant folds the npu split into the data split and pads
// the last band, so that one core visits the ranks of a data block in a fixed order.
template <uint32_t SWIZZLE_DIRECTION_ = 0, bool IS_DETERMINISTIC_ = false>
struct BlockCommSwizzle {
    static constexpr uint32_t SWIZZLE_DIRECTION = SWIZZLE_DIRECTION_;
    static constexpr bool IS_DETERMINISTIC = IS_DETERMINISTIC_;
    static_assert(!IS_DETERMINISTIC || SWIZZLE_DIRECTION == 0, "the deterministic order needs swizzle direction 0");
    uint32_t curRankIdx{0}, rankSize{1}, dataLoopsInRank{0};
    MatrixCoord coreSplit;
    BlockCommSwizzle() = default;
    BlockCommSwizzle(uint32_t curRankIdx_, uint32_t rankSize_, MatrixCoord const &coreSplit_, uint32_t dataLoopsInRank_ = 0)
        : curRankIdx(curRankIdx_), rankSize(rankSize_), dataLoopsInRank(dataLoopsInRank_),
          coreSplit(IS_DETERMINISTIC ? MatrixCoord{coreSplit_.row() * coreSplit_.column(), 1} : coreSplit_) {}
    uint32_t GetRealCore() const { return coreSplit.row() * coreSplit.column(); }
    uint32_t GetCoreLoop() const
    {
        return (IS_DETERMINISTIC ? Catlass::RoundUp(dataLoopsInRank, coreSplit.row()) : dataLoopsInRank) * rankSize;
    }
    MatrixCoord GetBlockIdx(uint32_t taskIdx) const
    {
        uint32_t d = 0, r = 0;
        catcoc_comm_block_idx_ex(SWIZZLE_DIRECTION, IS_DETERMINISTIC ? 1u : 0u, rankSize, coreSplit.row(), coreSplit.column(),
                                 dataLoopsInRank, taskIdx, &d, &r);
        return {d, r};
    }
};

// CommBlockEpilogue<Dispatch, SrcType, DstType, CoreSplit, BlockShape, TileShape, TileRemoteCopy, TileScheduler,
// GemmReMapper> (include/catcoc/comm_epilogue/block/comm_block_epilogue_to_local_mem.hpp:29-232, ..._to_share_mem.hpp):
// static split/shape types, or `void` with the dynamic dispatch policies and the three extra Params members.
template <class DispatchPolicy_, class SrcType_, class DstType_, class CoreSplit_, class BlockShape_, class TileShape_,
          class TileRemoteCopy_, class EpilogueTileSwizzle_, class GemmReMapper_ = void>
struct CommBlockEpilogue {
    using DispatchPolicy = DispatchPolicy_;
    using ElementSrc = typename SrcType_::Element;
    using ElementDst = typename DstType_::Element;
    using LayoutDst = typename DstType_::Layout;
    using GemmReMapper = GemmReMapper_;
    static constexpr bool IS_DYNAMIC = DispatchPolicy::IS_DYNAMIC;

    struct Params {
        void *shmemPtr{nullptr};
        Catlass::layout::RowMajor shmemLayout;
        MatrixCoord coreSplit, blockShape, tileShape;
        Params() = default;
        // static form: (ptr, layout[, gemmReMapper])
        template <class Ptr>
        Params(Ptr *shmemPtr_, Catlass::layout::RowMajor const &shmemLayout_) : shmemPtr((void *)shmemPtr_), shmemLayout(shmemLayout_)
        {
            fill_static();
        }
        template <class Ptr, class ReMapper>
        Params(Ptr *shmemPtr_, Catlass::layout::RowMajor const &shmemLayout_, ReMapper const &) : shmemPtr((void *)shmemPtr_), shmemLayout(shmemLayout_)
        {
            fill_static();
        }
        // dynamic form: (ptr, layout, [gemmReMapper,] coreSplit, blockShape, tileShape)
        template <class Ptr>
        Params(Ptr *shmemPtr_, Catlass::layout::RowMajor const &shmemLayout_, MatrixCoord coreSplit_, MatrixCoord blockShape_, MatrixCoord tileShape_)
            : shmemPtr((void *)shmemPtr_), shmemLayout(shmemLayout_), coreSplit(coreSplit_), blockShape(blockShape_), tileShape(tileShape_) {}
        template <class Ptr, class ReMapper>
        Params(Ptr *shmemPtr_, Catlass::layout::RowMajor const &shmemLayout_, ReMapper const &, MatrixCoord coreSplit_, MatrixCoord blockShape_,
               MatrixCoord tileShape_)
            : shmemPtr((void *)shmemPtr_), shmemLayout(shmemLayout_), coreSplit(coreSplit_), blockShape(blockShape_), tileShape(tileShape_) {}

    private:
        void fill_static()
        {
            if constexpr (!std::is_void<CoreSplit_>::value) coreSplit = CoreSplit_::ToCoord();
            if constexpr (!std::is_void<BlockShape_>::value) blockShape = BlockShape_::ToCoord();
            if constexpr (!std::is_void<TileShape_>::value) tileShape = TileShape_::ToCoord();
        }
    };
};

}  // namespace Block
}  // namespace CommEpilogue

namespace DGemm {

namespace Block {
// GemmIdentityBlockSwizzleAllGather<offset, direction, buffers> (include/catcoc/dgemm/block/block_swizzle_allgather.hpp:28-117):
// inside a comm round (pValue tile rows from every rank) the base swizzle walks the round's grid, then the row index is
// re-based rank-major.  problemShape is ONE rank's shard.
template <uint32_t SwizzleOffset = 1, uint32_t SwizzleDirection = 0, uint32_t BufferNum = 1>
struct GemmIdentityBlockSwizzleAllGather {
    static constexpr uint32_t OFFSET = SwizzleOffset, DIRECTION = SwizzleDirection;
    uint32_t rankSize{1}, pValue{1};
    MatrixCoord loopsInRank;
    GemmIdentityBlockSwizzleAllGather() = default;
    GemmIdentityBlockSwizzleAllGather(uint32_t rankSize_, uint32_t pValue_, GemmCoord const &problemShape_, MatrixCoord const &tileMN_)
        : rankSize(rankSize_), pValue(pValue_),
          loopsInRank(Catlass::CeilDiv(problemShape_.m(), tileMN_.row()), Catlass::CeilDiv(problemShape_.n(), tileMN_.column())) {}
    uint32_t GetMLoops() const { return loopsInRank.row() * rankSize; }
    uint32_t GetNLoops() const { return loopsInRank.column(); }
    uint32_t GetCoreLoops() const { return GetMLoops() * GetNLoops(); }
    GemmCoord GetBlockCoord(uint32_t taskIdx) const
    {
        uint32_t m = 0, n = 0;
        catcoc_allgather_block_coord(OFFSET, DIRECTION, rankSize, pValue, loopsInRank.row(), loopsInRank.column(), taskIdx, &m, &n);
        return {m, n, 0};
    }
};
}  // namespace Block

namespace Kernel {

namespace impl {

// the three shapes of a comm epilogue's Params, whichever epilogue type they came from
struct CommShape {
    MatrixCoord coreSplit, blockShape, tileShape;
    template <class P>
    CommShape(P const &p) : coreSplit(p.coreSplit), blockShape(p.blockShape), tileShape(p.tileShape) {}
};

inline void fill_comm(CocTilingParams &t, MatrixCoord coreSplit, MatrixCoord blockShape, MatrixCoord tileShape)
{
    // the dynamic wrappers' derivation read backwards (examples/dynamic_tiling/impl/kernel/matmul_reduce_scatter.h:151-153):
    // commCoreSplit = {dataSplit, npuSplit}, commBlockShape = {commBlockM, n0}, commTileShape = {commTileM / 2, n0}
    t.commDataSplit = coreSplit.row();
    t.commNpuSplit = coreSplit.column();
    t.commBlockM = blockShape.row();
    t.commTileM = tileShape.row() * 2;
}

template <class BlockMmad>
CocTilingParams make_tiling(GemmCoord const &problem, uint32_t rankSize, uint32_t commInterval)
{
    CocTilingParams t{};
    t.m = problem.m();
    t.n = problem.n();
    t.k = problem.k();
    t.m0 = BlockMmad::L1TileShape::M;
    t.n0 = BlockMmad::L1TileShape::N;
    t.k0 = BlockMmad::L1TileShape::K;
    t.commInterval = commInterval;
    t.rankSize = rankSize;
    return t;
}

// The caller's descriptor with what the template arguments and Params fix: rank, rank count, tile order.
template <class BlockScheduler>
bool make_desc(GM_ADDR ptrSymmetric, uint32_t rankIdx, uint32_t rankSize, CatcocSymmetricDesc &d)
{
    const CatcocSymmetricDesc *given = reinterpret_cast<const CatcocSymmetricDesc *>(ptrSymmetric);
    if (given == nullptr || given->magic != CATCOC_DESC_MAGIC) return false;
    d = *given;
    d.rankIdx = rankIdx;
    d.rankSize = rankSize;
    d.swizzleOffset = BlockScheduler::OFFSET;
    d.swizzleDirection = BlockScheduler::DIRECTION;
    return true;
}

}  // namespace impl

// Common shape of the three float kernels: `commType` picks the launcher family.
template <int COMM_TYPE, class BlockMmad_, class CommEpilogue_, class BlockScheduler_, class CommScheduler_, uint32_t WORKSPACE_STAGES_>
class FloatKernelBase {
public:
    using BlockMmad = BlockMmad_;
    using L1TileShape = typename BlockMmad::L1TileShape;
    using ElementA = typename BlockMmad::ElementA;
    using LayoutA = typename BlockMmad::LayoutA;
    using ElementB = typename BlockMmad::ElementB;
    using LayoutB = typename BlockMmad::LayoutB;
    using ElementD = typename CommEpilogue_::ElementDst;
    using LayoutD = typename CommEpilogue_::LayoutDst;
    using BlockScheduler = BlockScheduler_;
    using CommScheduler = CommScheduler_;
    using CommParams = typename CommEpilogue_::Params;
    static constexpr uint32_t WORKSPACE_STAGES = WORKSPACE_STAGES_;
    static_assert(std::is_same<ElementA, ElementB>::value, "A and B share one element type");

protected:
    static void launch(GemmCoord const &problemShape, uint32_t rankIdx, uint32_t rankSize, GM_ADDR ptrA, GM_ADDR ptrB,
                       GM_ADDR ptrSymmetric, impl::CommShape const &comm, GM_ADDR ptrD, uint32_t commInterval, void *stream)
    {
        CocTilingParams t = impl::make_tiling<BlockMmad>(problemShape, rankSize, commInterval);
        impl::fill_comm(t, comm.coreSplit, comm.blockShape, comm.tileShape);
        CatcocSymmetricDesc d;
        if (!impl::make_desc<BlockScheduler>(ptrSymmetric, rankIdx, rankSize, d)) {
            // let the launcher produce the error for a bad descriptor
            CatcocKernelFuncPtr fn = catcoc_get_kernel(COMM_TYPE, detail::ElementCode<ElementA>::value);
            fn(stream, 0, ptrA, ptrB, ptrD, nullptr, nullptr, ptrSymmetric, &t, LayoutA::kTransposed, LayoutB::kTransposed);
            return;
        }
        d.workspaceStages = WORKSPACE_STAGES;
        CatcocKernelFuncPtr fn = catcoc_get_kernel(COMM_TYPE, detail::ElementCode<ElementA>::value);
        fn(stream, 0, ptrA, ptrB, ptrD, nullptr, nullptr, reinterpret_cast<uint8_t *>(&d), &t, LayoutA::kTransposed, LayoutB::kTransposed);
    }
    static Catlass::Status check(GemmCoord const &problemShape, uint32_t rankIdx, uint32_t rankSize, GM_ADDR ptrSymmetric,
                                 impl::CommShape const &comm, uint32_t commInterval)
    {
        CocTilingParams t = impl::make_tiling<BlockMmad>(problemShape, rankSize, commInterval);
        impl::fill_comm(t, comm.coreSplit, comm.blockShape, comm.tileShape);
        CatcocSymmetricDesc d;
        if (!impl::make_desc<BlockScheduler>(ptrSymmetric, rankIdx, rankSize, d)) return Catlass::Status::kInvalid;
        d.workspaceStages = WORKSPACE_STAGES;
        return catcoc_can_implement(COMM_TYPE, detail::ElementCode<ElementA>::value, &t, &d, LayoutA::kTransposed, LayoutB::kTransposed) == 0
                   ? Catlass::Status::kSuccess : Catlass::Status::kInvalid;
    }
};

// include/catcoc/dgemm/kernel/matmul_reduce_scatter.hpp:17-89
template <class BlockMmad_, class BlockEpilogueReduceScatter_, class BlockScheduler_, class BlockEpilogueScheduler_, uint32_t WORKSPACE_STAGES_>
class MatmulReduceScatter : public FloatKernelBase<MATMUL_REDUCE_SCATTER, BlockMmad_, BlockEpilogueReduceScatter_, BlockScheduler_,
                                                    BlockEpilogueScheduler_, WORKSPACE_STAGES_> {
    using Base = FloatKernelBase<MATMUL_REDUCE_SCATTER, BlockMmad_, BlockEpilogueReduceScatter_, BlockScheduler_, BlockEpilogueScheduler_, WORKSPACE_STAGES_>;

public:
    using ReduceScatterParams = typename BlockEpilogueReduceScatter_::Params;
    using typename Base::LayoutA;
    using typename Base::LayoutB;
    using typename Base::LayoutD;
    struct Params {
        GemmCoord problemShape;
        uint32_t rankIdx{0}, rankSize{1};
        GM_ADDR ptrA{nullptr};
        LayoutA layoutA;
        GM_ADDR ptrB{nullptr};
        LayoutB layoutB;
        GM_ADDR ptrSymmetric{nullptr};
        ReduceScatterParams reduceScatterParams;
        GM_ADDR ptrD{nullptr};
        LayoutD layoutD;
        uint32_t commInterval{1};
        Params() = default;
        Params(GemmCoord const &problemShape_, uint32_t rank_, uint32_t rankSize_, GM_ADDR ptrA_, LayoutA const &layoutA_, GM_ADDR ptrB_,
               LayoutB const &layoutB_, GM_ADDR ptrSymmetric_, ReduceScatterParams const &reduceScatterParams_, GM_ADDR ptrD_,
               LayoutD const &layoutD_, uint32_t commInterval_)
            : problemShape(problemShape_), rankIdx(rank_), rankSize(rankSize_), ptrA(ptrA_), layoutA(layoutA_), ptrB(ptrB_), layoutB(layoutB_),
              ptrSymmetric(ptrSymmetric_), reduceScatterParams(reduceScatterParams_), ptrD(ptrD_), layoutD(layoutD_), commInterval(commInterval_) {}
    };
    static Catlass::Status CanImplement(Params const &p)
    {
        return Base::check(p.problemShape, p.rankIdx, p.rankSize, p.ptrSymmetric, p.reduceScatterParams, p.commInterval);
    }
    void operator()(Params const &p, void *stream = nullptr) const
    {
        Base::launch(p.problemShape, p.rankIdx, p.rankSize, p.ptrA, p.ptrB, p.ptrSymmetric, p.reduceScatterParams, p.ptrD, p.commInterval, stream);
    }
};

// include/catcoc/dgemm/kernel/matmul_allreduce.hpp:17-96 (two comm epilogues: reduce-scatter into the owner's slab, then all-gather)
template <class BlockMmad_, class BlockEpilogueReduceScatter_, class BlockEpilogueAllGather_, class BlockScheduler_,
          class BlockEpilogueScheduler_, uint32_t WORKSPACE_STAGES_>
class MatmulAllReduce : public FloatKernelBase<MATMUL_ALLREDUCE, BlockMmad_, BlockEpilogueAllGather_, BlockScheduler_,
                                                BlockEpilogueScheduler_, WORKSPACE_STAGES_> {
    using Base = FloatKernelBase<MATMUL_ALLREDUCE, BlockMmad_, BlockEpilogueAllGather_, BlockScheduler_, BlockEpilogueScheduler_, WORKSPACE_STAGES_>;

public:
    using ReduceScatterParams = typename BlockEpilogueReduceScatter_::Params;
    using AllGatherParams = typename BlockEpilogueAllGather_::Params;
    using typename Base::LayoutA;
    using typename Base::LayoutB;
    using typename Base::LayoutD;
    struct Params {
        GemmCoord problemShape;
        uint32_t rankIdx{0}, rankSize{1};
        GM_ADDR ptrA{nullptr};
        LayoutA layoutA;
        GM_ADDR ptrB{nullptr};
        LayoutB layoutB;
        GM_ADDR ptrSymmetric{nullptr};
        ReduceScatterParams reduceScatterParams;
        AllGatherParams allGatherParams;
        GM_ADDR ptrD{nullptr};
        LayoutD layoutD;
        uint32_t commInterval{1};
        Params() = default;
        Params(GemmCoord const &problemShape_, uint32_t rank_, uint32_t rankSize_, GM_ADDR ptrA_, LayoutA const &layoutA_, GM_ADDR ptrB_,
               LayoutB const &layoutB_, GM_ADDR ptrSymmetric_, ReduceScatterParams const &reduceScatterParams_,
               AllGatherParams const &allGatherParams_, GM_ADDR ptrD_, LayoutD const &layoutD_, uint32_t commInterval_)
            : problemShape(problemShape_), rankIdx(rank_), rankSize(rankSize_), ptrA(ptrA_), layoutA(layoutA_), ptrB(ptrB_), layoutB(layoutB_),
              ptrSymmetric(ptrSymmetric_), reduceScatterParams(reduceScatterParams_), allGatherParams(allGatherParams_), ptrD(ptrD_),
              layoutD(layoutD_), commInterval(commInterval_) {}
    };
    static Catlass::Status CanImplement(Params const &p)
    {
        return Base::check(p.problemShape, p.rankIdx, p.rankSize, p.ptrSymmetric, p.reduceScatterParams, p.commInterval);
    }
    void operator()(Params const &p, void *stream = nullptr) const
    {
        Base::launch(p.problemShape, p.rankIdx, p.rankSize, p.ptrA, p.ptrB, p.ptrSymmetric, p.reduceScatterParams, p.ptrD, p.commInterval, stream);
    }
};

// include/catcoc/dgemm/kernel/allgather_matmul.hpp:17-90.  problemShape.m() is ONE rank's shard; ptrA is this rank's shard.
template <class BlockMmad_, class BlockEpilogueAllGather_, class BlockScheduler_, class BlockEpilogueScheduler_, uint32_t WORKSPACE_STAGES_>
class AllGatherMatmul : public FloatKernelBase<ALLGATHER_MATMUL, BlockMmad_, BlockEpilogueAllGather_, BlockScheduler_,
                                                BlockEpilogueScheduler_, WORKSPACE_STAGES_> {
    using Base = FloatKernelBase<ALLGATHER_MATMUL, BlockMmad_, BlockEpilogueAllGather_, BlockScheduler_, BlockEpilogueScheduler_, WORKSPACE_STAGES_>;

public:
    using AllGatherParams = typename BlockEpilogueAllGather_::Params;
    using typename Base::LayoutA;
    using typename Base::LayoutB;
    using typename Base::LayoutD;
    struct Params {
        GemmCoord problemShape;
        uint32_t rankIdx{0}, rankSize{1};
        GM_ADDR ptrA{nullptr};
        LayoutA layoutA;
        GM_ADDR ptrB{nullptr};
        LayoutB layoutB;
        GM_ADDR ptrSymmetric{nullptr};
        AllGatherParams allGatherParams;
        GM_ADDR ptrD{nullptr};
        LayoutD layoutD;
        uint32_t commInterval{1};
        Params() = default;
        Params(GemmCoord const &problemShape_, uint32_t rank_, uint32_t rankSize_, GM_ADDR ptrA_, LayoutA const &layoutA_, GM_ADDR ptrB_,
               LayoutB const &layoutB_, GM_ADDR ptrSymmetric_, AllGatherParams const &allGatherParams_, GM_ADDR ptrD_, LayoutD const &layoutD_,
               uint32_t commInterval_)
            : problemShape(problemShape_), rankIdx(rank_), rankSize(rankSize_), ptrA(ptrA_), layoutA(layoutA_), ptrB(ptrB_), layoutB(layoutB_),
              ptrSymmetric(ptrSymmetric_), allGatherParams(allGatherParams_), ptrD(ptrD_), layoutD(layoutD_), commInterval(commInterval_) {}
    };
    static Catlass::Status CanImplement(Params const &p)
    {
        return Base::check(p.problemShape, p.rankIdx, p.rankSize, p.ptrSymmetric, p.allGatherParams, p.commInterval);
    }
    void operator()(Params const &p, void *stream = nullptr) const
    {
        Base::launch(p.problemShape, p.rankIdx, p.rankSize, p.ptrA, p.ptrB, p.ptrSymmetric, p.allGatherParams, p.ptrD, p.commInterval, stream);
    }
};

// include/catcoc/dgemm/kernel/quant_matmul_reduce_scatter.hpp:21-94.  The reduce runs on int32 partials before the
// dequant in the reference; which domain this launch reduces in follows the descriptor's flags (CATCOC_FLAG_REDUCE_INT32).
template <class BlockMmad_, class BlockEpilogueReduceScatter_, class BlockEpilogueDequant_, class BlockScheduler_,
          class BlockEpilogueScheduler_, uint32_t WORKSPACE_STAGES_>
class QuantMatmulReduceScatter {
public:
    using BlockMmad = BlockMmad_;
    using L1TileShape = typename BlockMmad::L1TileShape;
    using ElementA = typename BlockMmad::ElementA;
    using LayoutA = typename BlockMmad::LayoutA;
    using ElementB = typename BlockMmad::ElementB;
    using LayoutB = typename BlockMmad::LayoutB;
    using ElementC = typename BlockMmad::ElementC;
    using LayoutC = typename BlockMmad::LayoutC;
    using LayoutBias = typename BlockMmad::LayoutBias;
    using ReduceScatterParams = typename BlockEpilogueReduceScatter_::Params;
    using Dequant = BlockEpilogueDequant_;
    using DequantParams = typename Dequant::Params;
    using LayoutD = Catlass::layout::RowMajor;
    using BlockScheduler = BlockScheduler_;
    using CommScheduler = BlockEpilogueScheduler_;
    static constexpr uint32_t WORKSPACE_STAGES = WORKSPACE_STAGES_;
    static_assert(std::is_same<ElementA, int8_t>::value && std::is_same<ElementB, int8_t>::value, "W8A8: int8 operands");

    struct Params {
        GemmCoord problemShape;
        uint32_t rankIdx{0}, rankSize{1};
        GM_ADDR ptrA{nullptr};
        LayoutA layoutA;
        GM_ADDR ptrB{nullptr};
        LayoutB layoutB;
        GM_ADDR ptrBias{nullptr};
        LayoutBias layoutBias;
        GM_ADDR ptrSymmetric{nullptr};
        ReduceScatterParams reduceScatterParams;
        DequantParams dequantParams;
        GM_ADDR ptrC_accum{nullptr};
        LayoutC layoutC_accum;
        GM_ADDR ptrD_out{nullptr};
        LayoutD layoutD_out;
        uint32_t commInterval{1};
        Params() = default;
        Params(GemmCoord const &problemShape_, uint32_t rank_, uint32_t rankSize_, GM_ADDR ptrA_, LayoutA const &layoutA_, GM_ADDR ptrB_,
               LayoutB const &layoutB_, GM_ADDR ptrBias_, LayoutBias const &layoutBias_, GM_ADDR ptrSymmetric_,
               ReduceScatterParams const &reduceScatterParams_, DequantParams const &dequantParams_, GM_ADDR ptrC_accum_,
               LayoutC const &layoutC_accum_, GM_ADDR ptrD_out_, LayoutD const &layoutD_out_, uint32_t commInterval_)
            : problemShape(problemShape_), rankIdx(rank_), rankSize(rankSize_), ptrA(ptrA_), layoutA(layoutA_), ptrB(ptrB_), layoutB(layoutB_),
              ptrBias(ptrBias_), layoutBias(layoutBias_), ptrSymmetric(ptrSymmetric_), reduceScatterParams(reduceScatterParams_),
              dequantParams(dequantParams_), ptrC_accum(ptrC_accum_), layoutC_accum(layoutC_accum_), ptrD_out(ptrD_out_),
              layoutD_out(layoutD_out_), commInterval(commInterval_) {}
    };

    static Catlass::Status CanImplement(Params const &p)
    {
        CocTilingParams t;
        CatcocSymmetricDesc d;
        if (!prepare(p, t, d)) return Catlass::Status::kInvalid;
        return catcoc_can_implement(QUANT_MATMUL_REDUCE_SCATTER, INT8, &t, &d, LayoutA::kTransposed, LayoutB::kTransposed) == 0
                   ? Catlass::Status::kSuccess : Catlass::Status::kInvalid;
    }

    void operator()(Params const &p, void *stream = nullptr) const
    {
        CocTilingParams t;
        CatcocSymmetricDesc d;
        uint8_t *desc = reinterpret_cast<uint8_t *>(&d);
        if (!prepare(p, t, d)) desc = p.ptrSymmetric;   // the launcher reports what is wrong with it
        // the reference hands the dequant epilogue the per-token scales of the kept rows (scale_x1 + rank * m / P,
        // examples/02_matmul_reduce_scatter/quant_matmul_reduce_scatter.cpp:176-182); the launcher indexes them by global row
        const uint32_t mRank = p.rankSize ? p.problemShape.m() / p.rankSize : 0;
        uint8_t *perToken = reinterpret_cast<uint8_t *>(p.dequantParams.ptrPerTokenScale - (size_t)p.rankIdx * mRank);
        catcoc_launch_quant_matmul_reduce_scatter(stream, 0, p.ptrA, p.ptrB, perToken, reinterpret_cast<uint8_t *>(p.dequantParams.ptrScale),
                                                  p.ptrBias, p.ptrC_accum, p.ptrD_out, desc, &t, LayoutA::kTransposed, LayoutB::kTransposed,
                                                  detail::ElementCode<typename Dequant::ElementD>::value);
    }

private:
    static bool prepare(Params const &p, CocTilingParams &t, CatcocSymmetricDesc &d)
    {
        t = impl::make_tiling<BlockMmad>(p.problemShape, p.rankSize, p.commInterval);
        impl::fill_comm(t, p.reduceScatterParams.coreSplit, p.reduceScatterParams.blockShape, p.reduceScatterParams.tileShape);
        if (!impl::make_desc<BlockScheduler>(p.ptrSymmetric, p.rankIdx, p.rankSize, d)) return false;
        d.workspaceStages = WORKSPACE_STAGES;
        return true;
    }
};

}  // namespace Kernel
}  // namespace DGemm
}  // namespace Catcoc

#endif  // CATCOC_HIP_DGEMM_HPP
