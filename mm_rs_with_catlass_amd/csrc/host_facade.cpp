// Plain C++ host (g++, no hipcc) that drives the four operators through the template facade of
// include/catcoc_hip/dgemm.hpp, written the way the reference's wrappers set their types up
// (examples/02_matmul_reduce_scatter/quant_matmul_reduce_scatter.cpp:63-201,
// examples/dynamic_tiling/impl/kernel/matmul_reduce_scatter.h:36-118, examples/00_matmul_allreduce/matmul_allreduce.cpp,
// examples/01_allgather_matmul/allgather_matmul.cpp), and checks every result bit for bit against the same launch made
// through the C ABI directly.  Prints one "PASS <operator>" line per operator; exit code 0 when all pass.
#include <hip/hip_runtime_api.h>

#include <climits>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "catcoc_hip/dgemm.hpp"

using namespace Catcoc;

#define HIP_OK(call)                                                                                \
    do {                                                                                            \
        hipError_t e_ = (call);                                                                     \
        if (e_ != hipSuccess) {                                                                     \
            std::fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
            return 2;                                                                               \
        }                                                                                           \
    } while (0)

static uint32_t g_seed = 12345u;
static uint32_t rnd() { g_seed = g_seed * 1664525u + 1013904223u; return g_seed >> 8; }

template <class T>
static T *to_device(const std::vector<T> &h)
{
    T *d = nullptr;
    if (hipMalloc((void **)&d, h.size() * sizeof(T)) != hipSuccess) return nullptr;
    if (hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
    return d;
}

static uint16_t small_half(bool bf16)   // a small integer value in fp16 / bf16: products and sums stay exact
{
    static const uint16_t f16[5] = {0xC000, 0xBC00, 0x0000, 0x3C00, 0x4000};   // -2 -1 0 1 2
    static const uint16_t b16[5] = {0xC000, 0xBF80, 0x0000, 0x3F80, 0x4000};
    return (bf16 ? b16 : f16)[rnd() % 5];
}

static bool same(const void *devA, const void *devB, size_t bytes)
{
    std::vector<unsigned char> a(bytes), b(bytes);
    if (hipMemcpy(a.data(), devA, bytes, hipMemcpyDeviceToHost) != hipSuccess) return false;
    if (hipMemcpy(b.data(), devB, bytes, hipMemcpyDeviceToHost) != hipSuccess) return false;
    bool nonzero = false;
    for (unsigned char c : a) nonzero |= c != 0;
    return nonzero && std::memcmp(a.data(), b.data(), bytes) == 0;
}

static CatcocSymmetricDesc make_desc(uint32_t rank, uint32_t P)
{
    CatcocSymmetricDesc d;
    std::memset(&d, 0, sizeof(d));
    d.magic = CATCOC_DESC_MAGIC;
    d.rankIdx = rank;
    d.rankSize = P;
    return d;
}

using LayoutA = Catlass::layout::RowMajor;
using LayoutB = Catlass::layout::RowMajor;
using LayoutC = Catlass::layout::RowMajor;
using LayoutD = Catlass::layout::RowMajor;
using ArchTag = Catlass::Arch::AtlasA2;
constexpr uint32_t BLOCK_NUM = 256;   // scheduling slots per round: one per CU (the reference launches 20 AI cores)

static int run_quant(hipStream_t stream)
{
    const uint32_t m = 2048, n = 512, k = 256, rankSize = 8, rank = 3;
    std::vector<int8_t> hx1((size_t)m * k), hx2((size_t)k * n);
    for (auto &v : hx1) v = (int8_t)(rnd() % 255 - 127);
    for (auto &v : hx2) v = (int8_t)(rnd() % 255 - 127);
    std::vector<float> hs1(m), hs2(n);
    for (auto &v : hs1) v = 0.005f + (rnd() % 1000) * 1.5e-5f;
    for (auto &v : hs2) v = 0.001f + (rnd() % 1000) * 9e-6f;
    std::vector<int32_t> hbias(n);
    for (auto &v : hbias) v = (int32_t)(rnd() % 2001) - 1000;
    const uint32_t rows = m / rankSize;
    CatcocSymmetricDesc desc = make_desc(rank, rankSize);
    for (uint32_t s = 0; s + 1 < rankSize; ++s) {
        std::vector<float> hp((size_t)rows * n);
        for (auto &v : hp) v = ((int)(rnd() % 2001) - 1000) * 1e-3f;
        desc.peers[s] = to_device(hp);
    }
    uint8_t *x1 = (uint8_t *)to_device(hx1), *x2 = (uint8_t *)to_device(hx2), *scale_x1 = (uint8_t *)to_device(hs1),
            *scale_x2 = (uint8_t *)to_device(hs2), *bias = (uint8_t *)to_device(hbias);
    uint8_t *c_accum, *d_out, *d_ref;
    HIP_OK(hipMalloc((void **)&c_accum, (size_t)rows * n * 4));
    HIP_OK(hipMalloc((void **)&d_out, (size_t)rows * n * 2));
    HIP_OK(hipMalloc((void **)&d_ref, (size_t)rows * n * 2));
    HIP_OK(hipMemset(d_out, 0, (size_t)rows * n * 2));
    HIP_OK(hipMemset(d_ref, 0, (size_t)rows * n * 2));
    uint8_t *symmetricPtr = (uint8_t *)&desc;

    // ---- the reference wrapper's type set-up -----------------------------------------------------------------
    Catlass::GemmCoord problemShape{m, n, k};
    Catlass::layout::RowMajor layoutA{m, k, k};
    Catlass::layout::RowMajor layoutB{k, n, n};
    Catlass::layout::RowMajor layoutC_accum{m / rankSize, n, n};
    Catlass::layout::RowMajor layoutD_out{m / rankSize, n, n};
    Catlass::layout::VectorLayout layout_bias(n);

    using AType = Catlass::Gemm::GemmType<int8_t, LayoutA>;
    using BType = Catlass::Gemm::GemmType<int8_t, LayoutB>;
    using CType = Catlass::Gemm::GemmType<int32_t, LayoutC>;
    using BiasType = Catlass::Gemm::GemmType<int32_t, Catlass::layout::VectorLayout>;
    constexpr bool enableUnitFlag = true;
    using MmadDispatchPolicy = Catlass::Gemm::MmadAtlasA2PingpongBias<enableUnitFlag>;
    using L1TileShape = Catlass::GemmShape<128, 256, 256>;
    using L0TileShape = Catlass::GemmShape<128, 256, 64>;
    using BlockMmad = Catlass::Gemm::Block::BlockMmad<MmadDispatchPolicy, L1TileShape, L0TileShape, AType, BType, CType, BiasType>;
    using BlockScheduler = typename Catlass::Gemm::Block::GemmIdentityBlockSwizzle<7, 1>;
    using CommBlockScheduler = CommEpilogue::Block::BlockCommSwizzle<0>;
    using TileRemoteCopy = CommEpilogue::Tile::TileRemoteCopy<ArchTag, CType, CType, Catcoc::detail::CopyDirect::Get>;
    using TileScheduler = Catlass::Epilogue::Tile::EpilogueIdentityTileSwizzle;
    using CommBlockShape = Catlass::MatrixShape<64, 256>;
    using CommCoreSplit = Catlass::MatrixShape<20, 1>;
    constexpr uint32_t ubStages = 2;
    using ReduceScatterTileShape = Catlass::MatrixShape<32, 256>;
    using ReduceScatterDispatch = CommEpilogue::EpilogueAtlasA2CommToLocalMem<ubStages, Catcoc::detail::CopyMode::Scatter>;
    using BlockEpilogueReduceScatter = CommEpilogue::Block::CommBlockEpilogue<ReduceScatterDispatch, CType, CType, CommCoreSplit, CommBlockShape,
                                                                              ReduceScatterTileShape, TileRemoteCopy, TileScheduler, BlockScheduler>;
    using DequantScaleType = Catlass::Gemm::GemmType<float, Catlass::layout::VectorLayout>;
    using DequantDType = Catlass::Gemm::GemmType<bfloat16_t, LayoutD>;
    using BlockEpilogueDequant = Catlass::Epilogue::Block::BlockEpilogue<Catlass::Epilogue::EpilogueAtlasA2PerTokenDequant<2>, CType,
                                                                          DequantScaleType, DequantScaleType, DequantDType>;
    constexpr uint32_t workspaceStages = 2;
    constexpr uint32_t commInterval = 10;
    using Kernel = DGemm::Kernel::QuantMatmulReduceScatter<BlockMmad, BlockEpilogueReduceScatter, BlockEpilogueDequant, BlockScheduler,
                                                           CommBlockScheduler, workspaceStages>;
    Catlass::GemmCoord problemShapeInRank = problemShape / Catlass::MakeCoord<uint32_t>(rankSize, 1, 1);
    BlockScheduler matmulBlockScheduler(problemShapeInRank, Catlass::MakeCoord(L1TileShape::M, L1TileShape::N));
    Catlass::layout::RowMajor layoutPeerMemStore{L1TileShape::M * commInterval * BLOCK_NUM * workspaceStages, L1TileShape::N, L1TileShape::N};
    typename BlockEpilogueReduceScatter::Params reduceScatterParams{reinterpret_cast<int32_t *>(symmetricPtr), layoutPeerMemStore, matmulBlockScheduler};
    const uint32_t m_per_rank = m / rankSize;
    typename BlockEpilogueDequant::Params dequantParams{reinterpret_cast<float *>(scale_x2), Catlass::layout::VectorLayout(n),
                                                        reinterpret_cast<float *>(scale_x1) + rank * m_per_rank,
                                                        Catlass::layout::VectorLayout(m_per_rank), reinterpret_cast<bfloat16_t *>(d_out), layoutD_out};
    typename Kernel::Params params{problemShape, rank, rankSize, x1, layoutA, x2, layoutB, bias, layout_bias, symmetricPtr, reduceScatterParams,
                                   dequantParams, c_accum, layoutC_accum, d_out, layoutD_out, commInterval};
    if (Kernel::CanImplement(params) != Catlass::Status::kSuccess) {
        std::fprintf(stderr, "quant: CanImplement says no: %s\n", catcoc_last_error());
        return 1;
    }
    Kernel matmulCommKernel;
    matmulCommKernel(params, stream);
    if (catcoc_last_status() != 0) { std::fprintf(stderr, "quant facade rejected: %s\n", catcoc_last_error()); return 1; }

    // the same launch through the C ABI (the fixed configuration of the reference's example: 128x256 tiles, commInterval 10)
    catcoc_quant_matmul_reduce_scatter(stream, 0, x1, x2, scale_x1, scale_x2, bias, nullptr, d_ref, symmetricPtr, m, n, k);
    if (catcoc_last_status() != 0) { std::fprintf(stderr, "quant C ABI rejected: %s\n", catcoc_last_error()); return 1; }
    HIP_OK(hipStreamSynchronize(stream));
    if (!same(d_out, d_ref, (size_t)rows * n * 2)) { std::fprintf(stderr, "quant: facade and C ABI results differ\n"); return 1; }
    // the scheduler types answer on the host with the library's own index code
    const Catlass::GemmCoord c25 = matmulBlockScheduler.GetBlockCoord(3);
    uint32_t mi = 0, ni = 0;
    catcoc_swizzle_block_coord(7, 1, 2, 2, 3, &mi, &ni);
    if (matmulBlockScheduler.GetCoreLoops() != 4 || c25.m() != mi || c25.n() != ni) { std::fprintf(stderr, "quant: scheduler facade mismatch\n"); return 1; }
    std::printf("PASS QuantMatmulReduceScatter\n");
    return 0;
}

template <class Element, bool BF16>
static int run_float(hipStream_t stream)
{
    const uint32_t m = 1024, n = 512, k = 256, rankSize = 4, rank = 1;
    std::vector<uint16_t> ha((size_t)m * k), hb((size_t)k * n);
    for (auto &v : ha) v = small_half(BF16);
    for (auto &v : hb) v = small_half(BF16);
    uint8_t *a = (uint8_t *)to_device(ha), *b = (uint8_t *)to_device(hb);
    const int dt = BF16 ? (int)::BF16 : (int)::FP16;
    using AType = Catlass::Gemm::GemmType<Element, LayoutA>;
    using BType = Catlass::Gemm::GemmType<Element, LayoutB>;
    using CType = Catlass::Gemm::GemmType<Element, LayoutC>;
    using DType = Catlass::Gemm::GemmType<Element, LayoutD>;
    using L1TileShape = Catlass::GemmShape<128, 256, 256>;
    using L0TileShape = Catlass::GemmShape<128, 256, 64>;
    using BlockMmad = Catlass::Gemm::Block::BlockMmad<Catlass::Gemm::MmadAtlasA2Pingpong<true>, L1TileShape, L0TileShape, AType, BType, CType>;
    using BlockScheduler = typename Catlass::Gemm::Block::GemmIdentityBlockSwizzle<7, 1>;
    using CommBlockScheduler = CommEpilogue::Block::BlockCommSwizzle<0>;
    using TileScheduler = Catlass::Epilogue::Tile::EpilogueIdentityTileSwizzle;
    constexpr uint32_t commInterval = 2;
    Catlass::GemmCoord problemShape{m, n, k};

    // ---- reduce-scatter, dynamic comm parameters (the dynamic_tiling wrapper) ---------------------------------
    {
        const uint32_t rows = m / rankSize;
        CatcocSymmetricDesc desc = make_desc(rank, rankSize);
        for (uint32_t s = 0; s + 1 < rankSize; ++s) {
            std::vector<float> hp((size_t)rows * n);
            for (auto &v : hp) v = (float)((int)(rnd() % 9) - 4);
            desc.peers[s] = to_device(hp);
        }
        uint8_t *d_out, *d_ref;
        HIP_OK(hipMalloc((void **)&d_out, (size_t)rows * n * 2));
        HIP_OK(hipMalloc((void **)&d_ref, (size_t)rows * n * 2));
        HIP_OK(hipMemset(d_out, 0, (size_t)rows * n * 2));
        HIP_OK(hipMemset(d_ref, 0, (size_t)rows * n * 2));
        using TileRemoteCopy = CommEpilogue::Tile::TileRemoteCopy<ArchTag, CType, DType, Catcoc::detail::CopyDirect::Get>;
        using ReduceScatterDispatch = CommEpilogue::EpilogueAtlasA2CommToLocalMem<2, Catcoc::detail::CopyMode::Scatter, true>;
        using BlockEpilogueReduceScatter = CommEpilogue::Block::CommBlockEpilogue<ReduceScatterDispatch, CType, DType, void, void, void,
                                                                                  TileRemoteCopy, TileScheduler, BlockScheduler>;
        using Kernel = DGemm::Kernel::MatmulReduceScatter<BlockMmad, BlockEpilogueReduceScatter, BlockScheduler, CommBlockScheduler, 2>;
        BlockScheduler matmulBlockScheduler(problemShape / Catlass::MakeCoord<uint32_t>(rankSize, 1, 1), Catlass::MakeCoord<uint32_t>(128, 256));
        Catlass::layout::RowMajor layoutSymmetric{128 * commInterval * BLOCK_NUM * 2, 256, 256};
        typename BlockEpilogueReduceScatter::Params reduceScatterParams{reinterpret_cast<Element *>(&desc), layoutSymmetric, matmulBlockScheduler,
                                                                        Catlass::MatrixCoord{16, 1}, Catlass::MatrixCoord{64, 256},
                                                                        Catlass::MatrixCoord{32, 256}};
        typename Kernel::Params params{problemShape, rank, rankSize, a, LayoutA{m, k}, b, LayoutB{k, n}, (uint8_t *)&desc, reduceScatterParams,
                                       d_out, LayoutD{rows, n}, commInterval};
        if (Kernel::CanImplement(params) != Catlass::Status::kSuccess) { std::fprintf(stderr, "RS: CanImplement says no: %s\n", catcoc_last_error()); return 1; }
        Kernel kernel;
        kernel(params, stream);
        if (catcoc_last_status() != 0) { std::fprintf(stderr, "RS facade rejected: %s\n", catcoc_last_error()); return 1; }
        CocTilingParams t;
        catcoc_default_tiling(&t, m, k, n, rankSize);
        t.commInterval = commInterval; t.commDataSplit = 16; t.commNpuSplit = 1; t.commBlockM = 64; t.commTileM = 64;
        catcoc_get_kernel(MATMUL_REDUCE_SCATTER, dt)(stream, 0, a, b, d_ref, nullptr, nullptr, (uint8_t *)&desc, &t, 0, 0);
        if (catcoc_last_status() != 0) { std::fprintf(stderr, "RS C ABI rejected: %s\n", catcoc_last_error()); return 1; }
        HIP_OK(hipStreamSynchronize(stream));
        if (!same(d_out, d_ref, (size_t)rows * n * 2)) { std::fprintf(stderr, "RS: facade and C ABI results differ\n"); return 1; }
        std::printf("PASS MatmulReduceScatter %s\n", BF16 ? "bf16" : "fp16");
    }
    // ---- all-reduce: two static comm epilogues (reduce-scatter into the owner's slab, all-gather) ----------------
    {
        CatcocSymmetricDesc desc = make_desc(rank, rankSize);
        for (uint32_t s = 0; s + 1 < rankSize; ++s) {
            std::vector<float> hp((size_t)m * n);
            for (auto &v : hp) v = (float)((int)(rnd() % 9) - 4);
            desc.peers[s] = to_device(hp);
        }
        uint8_t *d_out, *d_ref;
        HIP_OK(hipMalloc((void **)&d_out, (size_t)m * n * 2));
        HIP_OK(hipMalloc((void **)&d_ref, (size_t)m * n * 2));
        HIP_OK(hipMemset(d_out, 0, (size_t)m * n * 2));
        HIP_OK(hipMemset(d_ref, 0, (size_t)m * n * 2));
        using CommBlockShape = Catlass::MatrixShape<64, 256>;
        using CommCoreSplit = Catlass::MatrixShape<20, 1>;
        using TileShape = Catlass::MatrixShape<32, 256>;
        using RemoteGet = CommEpilogue::Tile::TileRemoteCopy<ArchTag, CType, DType, Catcoc::detail::CopyDirect::Get>;
        using ReduceScatterDispatch = CommEpilogue::EpilogueAtlasA2CommToShareMem<2, Catcoc::detail::CopyMode::Scatter>;
        using AllGatherDispatch = CommEpilogue::EpilogueAtlasA2CommToLocalMem<2, Catcoc::detail::CopyMode::Gather>;
        using BlockEpilogueReduceScatter = CommEpilogue::Block::CommBlockEpilogue<ReduceScatterDispatch, CType, DType, CommCoreSplit, CommBlockShape,
                                                                                  TileShape, RemoteGet, TileScheduler>;
        using BlockEpilogueAllGather = CommEpilogue::Block::CommBlockEpilogue<AllGatherDispatch, CType, DType, CommCoreSplit, CommBlockShape, TileShape,
                                                                              RemoteGet, TileScheduler, BlockScheduler>;
        using Kernel = DGemm::Kernel::MatmulAllReduce<BlockMmad, BlockEpilogueReduceScatter, BlockEpilogueAllGather, BlockScheduler,
                                                      CommBlockScheduler, 2>;
        BlockScheduler matmulBlockScheduler(problemShape, Catlass::MakeCoord<uint32_t>(128, 256));
        Catlass::layout::RowMajor layoutPeerMemStore{128 * commInterval * BLOCK_NUM * 2, 256, 256};
        typename BlockEpilogueReduceScatter::Params rsParams{reinterpret_cast<Element *>(&desc), layoutPeerMemStore};
        typename BlockEpilogueAllGather::Params agParams{reinterpret_cast<Element *>(&desc), layoutPeerMemStore, matmulBlockScheduler};
        typename Kernel::Params params{problemShape, rank, rankSize, a, LayoutA{m, k}, b, LayoutB{k, n}, (uint8_t *)&desc, rsParams, agParams,
                                       d_out, LayoutD{m, n}, commInterval};
        Kernel kernel;
        kernel(params, stream);
        if (catcoc_last_status() != 0) { std::fprintf(stderr, "AR facade rejected: %s\n", catcoc_last_error()); return 1; }
        CocTilingParams t;
        catcoc_default_tiling(&t, m, k, n, rankSize);
        t.commInterval = commInterval; t.commDataSplit = 20; t.commNpuSplit = 1; t.commBlockM = 64; t.commTileM = 64;
        catcoc_get_kernel(MATMUL_ALLREDUCE, dt)(stream, 0, a, b, d_ref, nullptr, nullptr, (uint8_t *)&desc, &t, 0, 0);
        if (catcoc_last_status() != 0) { std::fprintf(stderr, "AR C ABI rejected: %s\n", catcoc_last_error()); return 1; }
        HIP_OK(hipStreamSynchronize(stream));
        if (!same(d_out, d_ref, (size_t)m * n * 2)) { std::fprintf(stderr, "AR: facade and C ABI results differ\n"); return 1; }
        std::printf("PASS MatmulAllReduce %s\n", BF16 ? "bf16" : "fp16");
    }
    // ---- all-gather matmul: this rank's shard is `a`, the others' shards sit in the descriptor ----------------------
    {
        const uint32_t ms = 256;   // rows of one shard
        CatcocSymmetricDesc desc = make_desc(rank, rankSize);
        for (uint32_t s = 0; s + 1 < rankSize; ++s) {
            std::vector<uint16_t> hs((size_t)ms * k);
            for (auto &v : hs) v = small_half(BF16);
            desc.peers[s] = to_device(hs);
        }
        uint8_t *d_out, *d_ref;
        HIP_OK(hipMalloc((void **)&d_out, (size_t)ms * rankSize * n * 2));
        HIP_OK(hipMalloc((void **)&d_ref, (size_t)ms * rankSize * n * 2));
        HIP_OK(hipMemset(d_out, 0, (size_t)ms * rankSize * n * 2));
        HIP_OK(hipMemset(d_ref, 0, (size_t)ms * rankSize * n * 2));
        using AGScheduler = typename Catcoc::DGemm::Block::GemmIdentityBlockSwizzleAllGather<7, 1, 2>;
        using BlockRemapper = typename Catlass::Gemm::Block::GemmIdentityBlockSwizzle<7, 1>;
        using RemotePut = CommEpilogue::Tile::TileRemoteCopy<ArchTag, CType, DType, Catcoc::detail::CopyDirect::Put>;
        using CommBlockShape = Catlass::MatrixShape<64, UINT_MAX / 2>;
        using CommCoreSplit = Catlass::MatrixShape<20, 1>;
        using AllGatherDispatch = CommEpilogue::EpilogueAtlasA2CommToShareMem<2, Catcoc::detail::CopyMode::Gather, false>;
        using BlockEpilogueAllGather = CommEpilogue::Block::CommBlockEpilogue<AllGatherDispatch, CType, DType, CommCoreSplit, CommBlockShape,
                                                                              Catlass::MatrixShape<32, 256>, RemotePut, TileScheduler, BlockRemapper>;
        using Kernel = DGemm::Kernel::AllGatherMatmul<BlockMmad, BlockEpilogueAllGather, AGScheduler, CommBlockScheduler, 2>;
        Catlass::GemmCoord shardShape{ms, n, k};
        BlockRemapper reMapper(Catlass::GemmCoord{ms, k, k}, Catlass::MakeCoord<uint32_t>(128, k));
        Catlass::layout::RowMajor layoutPeerMemStore{128 * 1 * rankSize * 2, k, k};
        typename BlockEpilogueAllGather::Params agParams{reinterpret_cast<Element *>(&desc), layoutPeerMemStore, reMapper};
        typename Kernel::Params params{shardShape, rank, rankSize, a, LayoutA{ms, k}, b, LayoutB{k, n}, (uint8_t *)&desc, agParams,
                                       d_out, LayoutD{ms * rankSize, n}, 1};
        Kernel kernel;
        kernel(params, stream);
        if (catcoc_last_status() != 0) { std::fprintf(stderr, "AG facade rejected: %s\n", catcoc_last_error()); return 1; }
        CocTilingParams t;
        catcoc_default_tiling(&t, ms, k, n, rankSize);
        t.commInterval = 1; t.commDataSplit = 20; t.commNpuSplit = 1; t.commBlockM = 64; t.commTileM = 64;
        catcoc_get_kernel(ALLGATHER_MATMUL, dt)(stream, 0, a, b, d_ref, nullptr, nullptr, (uint8_t *)&desc, &t, 0, 0);
        if (catcoc_last_status() != 0) { std::fprintf(stderr, "AG C ABI rejected: %s\n", catcoc_last_error()); return 1; }
        HIP_OK(hipStreamSynchronize(stream));
        if (!same(d_out, d_ref, (size_t)ms * rankSize * n * 2)) { std::fprintf(stderr, "AG: facade and C ABI results differ\n"); return 1; }
        AGScheduler sched(rankSize, 1, shardShape, Catlass::MakeCoord<uint32_t>(128, 256));
        uint32_t mi = 0, ni = 0;
        catcoc_allgather_block_coord(7, 1, rankSize, 1, 2, 2, 5, &mi, &ni);
        if (sched.GetCoreLoops() != 16 || sched.GetBlockCoord(5).m() != mi || sched.GetBlockCoord(5).n() != ni) {
            std::fprintf(stderr, "AG: scheduler facade mismatch\n");
            return 1;
        }
        std::printf("PASS AllGatherMatmul %s\n", BF16 ? "bf16" : "fp16");
    }
    return 0;
}

int main()
{
    hipStream_t stream;
    HIP_OK(hipSetDevice(0));
    HIP_OK(hipStreamCreate(&stream));
    int rc = run_quant(stream);
    if (rc == 0) rc = run_float<half, false>(stream);
    if (rc == 0) rc = run_float<bfloat16_t, true>(stream);
    if (rc == 0) std::printf("facade ok\n");
    (void)hipStreamDestroy(stream);
    return rc;
}
