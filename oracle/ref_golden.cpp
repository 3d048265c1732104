// Driver that compiles the REFERENCE's own CPU golden, unmodified and in place,
// into oracle/_ref/libcatcoc_ref_golden.so.  Test infrastructure only: it is used
// to validate oracle/catcoc_oracle.c and is never loaded by the product path.
// The reference sources are included from /root/reference (see oracle/Makefile);
// nothing of them is copied here.
//
// Wrapped functions (paths relative to the reference tree):
//   Catlass::golden::QuantMatmul        3rdparty/catlass/examples/common/golden/matmul.hpp:274-302
//   Catlass::golden::ComputeMatmul      3rdparty/catlass/examples/common/golden/matmul.hpp:22-42
//   Catlass::golden::ComputeMatmulBias  3rdparty/catlass/examples/common/golden/matmul.hpp:343-364
//   Catlass::golden::CompareData        3rdparty/catlass/examples/common/golden/compare_data.hpp:20-39
//   op::bfloat16::round_to_bfloat16     3rdparty/catlass/examples/common/bfloat16.h:151-173
#include <cstdint>
#include <cstring>
#include <vector>

#include "bfloat16.h"
#include "golden/matmul.hpp"
#include "golden/compare_data.hpp"

using namespace Catlass;

extern "C" {

__attribute__((visibility("default")))
void ref_quant_matmul(uint32_t M, uint32_t N, uint32_t K, const int8_t *A, const int8_t *B,
                      const float *scale, const float *perTokenScale, float *out)
{
    std::vector<int8_t> a(A, A + (size_t)M * K), b(B, B + (size_t)K * N);
    std::vector<float> s(scale, scale + N), p(perTokenScale, perTokenScale + M), g((size_t)M * N);
    golden::QuantMatmul(GemmCoord{M, N, K}, a, layout::RowMajor{M, K}, b, layout::RowMajor{K, N},
                        s, layout::VectorLayout{N}, p, layout::VectorLayout{M}, g, layout::RowMajor{M, N});
    std::memcpy(out, g.data(), g.size() * sizeof(float));
}

// Inputs already widened to float (the widening of fp16/bf16 is exact), golden in float.
__attribute__((visibility("default")))
void ref_compute_matmul_f32(uint32_t M, uint32_t N, uint32_t K, const float *A, const float *B, float *out)
{
    std::vector<float> a(A, A + (size_t)M * K), b(B, B + (size_t)K * N), g((size_t)M * N);
    golden::ComputeMatmul(GemmCoord{M, N, K}, a, layout::RowMajor{M, K}, b, layout::RowMajor{K, N},
                          g, layout::RowMajor{M, N});
    std::memcpy(out, g.data(), g.size() * sizeof(float));
}

// Same with the reference's own bfloat16 element type (inputs given as bit patterns).
__attribute__((visibility("default")))
void ref_compute_matmul_bf16(uint32_t M, uint32_t N, uint32_t K, const uint16_t *A, const uint16_t *B, float *out)
{
    std::vector<op::bfloat16> a((size_t)M * K), b((size_t)K * N);
    for (size_t i = 0; i < a.size(); ++i) a[i] = op::bfloat16(A[i], op::bfloat16::from_bits());
    for (size_t i = 0; i < b.size(); ++i) b[i] = op::bfloat16(B[i], op::bfloat16::from_bits());
    std::vector<float> g((size_t)M * N);
    golden::ComputeMatmul(GemmCoord{M, N, K}, a, layout::RowMajor{M, K}, b, layout::RowMajor{K, N},
                          g, layout::RowMajor{M, N});
    std::memcpy(out, g.data(), g.size() * sizeof(float));
}

__attribute__((visibility("default")))
void ref_compute_matmul_bias_i8(uint32_t M, uint32_t N, uint32_t K, const int8_t *A, const int8_t *B,
                                const int32_t *bias, int32_t *out)
{
    std::vector<int8_t> a(A, A + (size_t)M * K), b(B, B + (size_t)K * N);
    std::vector<int32_t> bi(bias, bias + N), g((size_t)M * N);
    golden::ComputeMatmulBias(GemmCoord{M, N, K}, a, layout::RowMajor{M, K}, b, layout::RowMajor{K, N},
                              bi, g, layout::RowMajor{M, N});
    std::memcpy(out, g.data(), g.size() * sizeof(int32_t));
}

__attribute__((visibility("default")))
uint64_t ref_compare_data(const float *result, const float *expect, uint64_t n, uint32_t computeNum)
{
    std::vector<float> r(result, result + n), e(expect, expect + n);
    return golden::CompareData(r, e, computeNum).size();
}

__attribute__((visibility("default")))
uint16_t ref_round_to_bf16(float v)
{
    return op::bfloat16::round_to_bfloat16(v).value;
}

}  // extern "C"
