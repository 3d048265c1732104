/*
 * catcoc_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, CPU-only restatement of the arithmetic and index math of the
 * CATCOC per-rank fused GEMM path.  It exists so that the HIP library can be
 * checked against it; nothing in the product path links, loads or calls it.
 * Only tests, the smoke check and the benchmark's cpu-baseline leg use it.
 *
 * Every function names the reference file:line whose behaviour it restates
 * (paths relative to the reference tree):
 *   GOLD = 3rdparty/catlass/examples/common/golden/matmul.hpp
 *   BF16 = 3rdparty/catlass/examples/common/bfloat16.h
 *   SWZ  = 3rdparty/catlass/include/catlass/gemm/block/block_swizzle.hpp
 *   SWAG = include/catcoc/dgemm/block/block_swizzle_allgather.hpp
 *   CSW  = include/catcoc/comm_epilogue/block/comm_block_swizzle.hpp
 *   KQ   = include/catcoc/dgemm/kernel/quant_matmul_reduce_scatter.hpp
 *   KAR  = include/catcoc/dgemm/kernel/matmul_allreduce.hpp
 *   KAG  = include/catcoc/dgemm/kernel/allgather_matmul.hpp
 *   DEQ  = 3rdparty/catlass/include/catlass/epilogue/block/block_epilogue_per_token_dequant.hpp
 *   SPK  = 3rdparty/catlass/include/catlass/gemm/kernel/splitk_matmul.hpp
 *   TIL  = examples/dynamic_tiling/include/tiling.h
 *   VER  = examples/utils/verify_result.py, examples/utils/utils.py
 *
 * Pinning status (what each function is checked against, in tests/):
 *   int8 GEMM, float GEMM, dequant      : the reference's own golden compiled
 *                                         from source (oracle/_ref), brute force,
 *                                         closed forms (debug-mode data).
 *   bf16 / fp16 rounding                : reference bfloat16.h via oracle/_ref,
 *                                         numpy float16, exhaustive tie cases.
 *   GemmIdentityBlockSwizzle, split-K   : reference headers via oracle/_ref,
 *   swizzle, all-gather swizzle           committed fixtures, bijection checks.
 *   BlockCommSwizzle                    : reference header needs the Ascend
 *                                         toolkit header, so it is not built;
 *                                         pinned by hand-worked cases and
 *                                         bijection / rotation invariants.
 *   GetSplitkFactor, tiling search      : hand-enumerated cases.
 *   reduce-scatter / all-reduce task    : cases worked by hand from KQ:159-201
 *   maps, int32 peer reduce               and KAR:146-179 (several rounds, a
 *                                         reversed narrow band); numpy with
 *                                         distinct peers and a row offset.
 *   deterministic BlockCommSwizzle,     : cases worked by hand from CSW:114-118,
 *   comm core loop                        166-170 (rank of step d is (i + d) mod P),
 *                                         every (rank, block) pair visited once.
 *   half-precision add (one rounding    : numpy float16, exact rational sums
 *   per add), ReduceAdd                   rounded once (fractions), numpy fp32
 *                                         slice-sequential sums.
 *   peer reduce order                   : defined by this build (local partial
 *                                         first, then peers in ascending slot
 *                                         order); the reference reduces with
 *                                         unordered atomics, so there is no
 *                                         reference order to pin against.
 *
 * Build: see oracle/Makefile (gcc -O3 -march=native -ffp-contract=off -fopenmp).
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <stdlib.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* 16-bit float conversions                                                   */
/* ------------------------------------------------------------------------- */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* BF16:151-173  round_to_bfloat16: NaN -> 0x7fc0, else add 0x7fff + lsb and truncate. */
ORACLE_API uint16_t oracle_f32_to_bf16(float v)
{
    uint32_t u = f32_bits(v);
    if (v != v) return 0x7fc0;
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

ORACLE_API float oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* IEEE binary16 round-to-nearest-even from binary32.  The reference's fp16 host
 * type (fp16_t.h) only declares its conversions, so this follows IEEE 754 and is
 * pinned against numpy.float16 in the tests. */
ORACLE_API uint16_t oracle_f32_to_f16(float v)
{
    uint32_t u = f32_bits(v);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t absu = u & 0x7fffffffu;
    if (absu > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);          /* NaN */
    if (absu >= 0x47800000u) {                                           /* >= 65536: inf (65520 rounds up too) */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absu >= 0x38800000u) {                                           /* normal half range */
        uint32_t mant = absu & 0x7fffffu;
        uint32_t exp = (absu >> 23) - 112u;                              /* rebias 127 -> 15 */
        uint32_t h = (exp << 10) | (mant >> 13);
        uint32_t rem = mant & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h += 1u;      /* may carry into exponent / inf: correct */
        return (uint16_t)(sign | h);
    }
    if (absu < 0x33000000u) return (uint16_t)sign;                       /* < 2^-25: rounds to zero */
    /* subnormal half: value = mant24 * 2^(e-150); target unit 2^-24 */
    uint32_t e = absu >> 23;
    uint32_t mant = (absu & 0x7fffffu) | 0x800000u;
    uint32_t shift = 126u - e;                                           /* 14..24 */
    uint32_t h = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1u);
    if (rem > half || (rem == half && (h & 1u))) h += 1u;
    return (uint16_t)(sign | h);
}

ORACLE_API float oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t mant = h & 0x3ffu;
    if (exp == 0x1f) return bits_f32(sign | 0x7f800000u | (mant << 13));
    if (exp != 0) return bits_f32(sign | ((exp + 112u) << 23) | (mant << 13));
    if (mant == 0) return bits_f32(sign);
    float f = (float)mant * (1.0f / 16777216.0f);                        /* mant * 2^-24, exact */
    return (sign ? -f : f);
}

/* dtype codes follow examples/dynamic_tiling/include/launch_map.h:13-16 and
 * examples/utils/utils.py:14-17 (FP16 = 1, BF16 = 27). */
enum { ORACLE_FP16 = 1, ORACLE_BF16 = 27 };

static inline float half_to_f32(uint16_t h, int dtype)
{
    return dtype == ORACLE_BF16 ? oracle_bf16_to_f32(h) : oracle_f16_to_f32(h);
}
static inline uint16_t f32_to_half(float f, int dtype)
{
    return dtype == ORACLE_BF16 ? oracle_f32_to_bf16(f) : oracle_f32_to_f16(f);
}

ORACLE_API void oracle_cast_f32_to_half(const float *src, uint16_t *dst, size_t n, int dtype)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) dst[i] = f32_to_half(src[i], dtype);
}

ORACLE_API void oracle_cast_half_to_f32(const uint16_t *src, float *dst, size_t n, int dtype)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) dst[i] = half_to_f32(src[i], dtype);
}

/* ------------------------------------------------------------------------- */
/* GEMMs                                                                      */
/* ------------------------------------------------------------------------- */

/* GOLD:274-302 (integer part) and GOLD:343-364 (bias seeds the accumulator).
 * acc[i][j] = bias[j] + sum_k int32(A[i][k]) * int32(B[k][j]).
 * A is row-major [M,K] with leading dimension lda.  B is row-major [K,N]
 * (transB = 0, element (k,j) at k*ldb + j) or stored transposed [N,K]
 * (transB = 1, element (k,j) at j*ldb + k), the two layouts of
 * examples/dynamic_tiling/impl/kernel_fp16.cpp:31-43.
 * Integer sums are exact, so the loop order is free; i-k-j is used so the
 * inner loop vectorises. */
ORACLE_API void oracle_gemm_i8_i32(uint32_t M, uint32_t N, uint32_t K,
                                   const int8_t *A, int64_t lda,
                                   const int8_t *B, int64_t ldb, int transB,
                                   const int32_t *bias,
                                   int32_t *C, int64_t ldc)
{
#pragma omp parallel for schedule(dynamic, 4)
    for (uint32_t i = 0; i < M; ++i) {
        int32_t *c = C + (int64_t)i * ldc;
        for (uint32_t j = 0; j < N; ++j) c[j] = bias ? bias[j] : 0;
        const int8_t *a = A + (int64_t)i * lda;
        if (!transB) {
            for (uint32_t k = 0; k < K; ++k) {
                const int32_t av = a[k];
                const int8_t *b = B + (int64_t)k * ldb;
                for (uint32_t j = 0; j < N; ++j) c[j] += av * (int32_t)b[j];
            }
        } else {
            for (uint32_t j = 0; j < N; ++j) {
                const int8_t *b = B + (int64_t)j * ldb;
                int32_t s = 0;
                for (uint32_t k = 0; k < K; ++k) s += (int32_t)a[k] * (int32_t)b[k];
                c[j] += s;
            }
        }
    }
}

/* The literal triple loop of GOLD:288-296 (k innermost, one scalar accumulator),
 * single thread: used for the labelled single-core timing and as a brute-force
 * cross-check of the vectorised loop above. */
ORACLE_API void oracle_gemm_i8_i32_literal(uint32_t M, uint32_t N, uint32_t K,
                                           const int8_t *A, const int8_t *B, int32_t *C)
{
    for (uint32_t i = 0; i < M; ++i)
        for (uint32_t j = 0; j < N; ++j) {
            int32_t acc = 0;
            for (uint32_t k = 0; k < K; ++k)
                acc += (int32_t)A[(size_t)i * K + k] * (int32_t)B[(size_t)k * N + j];
            C[(size_t)i * N + j] = acc;
        }
}

/* GOLD:22-42 with ElementGolden = float: accumulator starts at 0 and adds
 * float(a)*float(b) for k ascending.  The product of two fp16 (or bf16) values is
 * exact in fp32, so each step rounds once.  Loop order i-k-j keeps every output
 * element's additions in ascending k, i.e. the reference's order. */
ORACLE_API void oracle_gemm_half_f32(uint32_t M, uint32_t N, uint32_t K,
                                     const uint16_t *A, int64_t lda, int transA,
                                     const uint16_t *B, int64_t ldb, int transB,
                                     int dtype, float *C, int64_t ldc)
{
    float *Bf = (float *)malloc((size_t)K * N * sizeof(float));
#pragma omp parallel for schedule(static)
    for (uint32_t k = 0; k < K; ++k)
        for (uint32_t j = 0; j < N; ++j) {
            uint16_t h = transB ? B[(int64_t)j * ldb + k] : B[(int64_t)k * ldb + j];
            Bf[(size_t)k * N + j] = half_to_f32(h, dtype);
        }
#pragma omp parallel for schedule(dynamic, 4)
    for (uint32_t i = 0; i < M; ++i) {
        float *c = C + (int64_t)i * ldc;
        for (uint32_t j = 0; j < N; ++j) c[j] = 0.0f;
        for (uint32_t k = 0; k < K; ++k) {
            uint16_t h = transA ? A[(int64_t)k * lda + i] : A[(int64_t)i * lda + k];
            const float av = half_to_f32(h, dtype);
            const float *b = Bf + (size_t)k * N;
            for (uint32_t j = 0; j < N; ++j) c[j] += av * b[j];
        }
    }
    free(Bf);
}

/* ------------------------------------------------------------------------- */
/* Epilogues                                                                  */
/* ------------------------------------------------------------------------- */

/* DEQ:575-594 and GOLD:297-299: c32 = float(acc) (round to nearest even),
 * t = c32 * scale[n] (per-channel first), u = t * perTokenScale[m]. */
ORACLE_API void oracle_dequant(uint32_t M, uint32_t N, const int32_t *acc, int64_t ldacc,
                               const float *scale_n, const float *scale_m,
                               float *out, int64_t ldo)
{
#pragma omp parallel for schedule(static)
    for (uint32_t i = 0; i < M; ++i)
        for (uint32_t j = 0; j < N; ++j) {
            float c32 = (float)acc[(int64_t)i * ldacc + j];
            float t = c32 * scale_n[j];
            out[(int64_t)i * ldo + j] = t * scale_m[i];
        }
}

/* The reduce the comm epilogue performs with atomic add (KQ:285-308, KAR:253-282),
 * restated on staged peer partials: s = local; s += peer[0]; s += peer[1]; ...
 * in fp32, then one round-to-nearest-even cast (KAR/KRS store in the output
 * dtype; DEQ:594 casts with CAST_RINT).  peers[p] points at a row-major fp32
 * matrix whose row `peer_row0 + i` lines up with local row i. */
ORACLE_API void oracle_reduce_cast(uint32_t M, uint32_t N, const float *local, int64_t ldl,
                                   uint32_t n_peers, const float *const *peers, int64_t ldp,
                                   int64_t peer_row0, int dtype, uint16_t *out, int64_t ldo)
{
#pragma omp parallel for schedule(static)
    for (uint32_t i = 0; i < M; ++i)
        for (uint32_t j = 0; j < N; ++j) {
            float s = local[(int64_t)i * ldl + j];
            for (uint32_t p = 0; p < n_peers; ++p) s += peers[p][(peer_row0 + i) * ldp + j];
            out[(int64_t)i * ldo + j] = f32_to_half(s, dtype);
        }
}

/* Reference-faithful quantised reduce: peers' int32 partials are added before
 * the dequant (KQ:285-308 then KQ:322-351).  Integer adds are exact. */
ORACLE_API void oracle_reduce_i32(uint32_t M, uint32_t N, int32_t *acc, int64_t ldacc,
                                  uint32_t n_peers, const int32_t *const *peers, int64_t ldp,
                                  int64_t peer_row0)
{
#pragma omp parallel for schedule(static)
    for (uint32_t i = 0; i < M; ++i)
        for (uint32_t j = 0; j < N; ++j) {
            int32_t s = acc[(int64_t)i * ldacc + j];
            for (uint32_t p = 0; p < n_peers; ++p) s += peers[p][(peer_row0 + i) * ldp + j];
            acc[(int64_t)i * ldacc + j] = s;
        }
}

/* ------------------------------------------------------------------------- */
/* Whole-operator restatements                                                */
/* ------------------------------------------------------------------------- */

/* W8A8 matmul -> reduce-scatter, this rank's share (KQ:116-351 with the peers
 * staged): full [M,N] int32 accumulators (optionally returned), dequant of the
 * kept row block [rows_kept, N] starting at row0, fp32 peer reduce, cast.
 * reduce_int32 != 0 selects the reference's order (int32 reduce, then dequant). */
ORACLE_API void oracle_quant_matmul_reduce_scatter(
    uint32_t M, uint32_t N, uint32_t K,
    const int8_t *x1, const int8_t *x2, int transB,
    const float *scale_x1, const float *scale_x2, const int32_t *bias,
    uint32_t row0, uint32_t rows_kept,
    uint32_t n_peers, const void *const *peers, int64_t ldp, int64_t peer_row0,
    int reduce_int32, int out_dtype,
    int32_t *acc_full /* [M,N] or NULL */, uint16_t *d_out /* [rows_kept,N] */)
{
    int32_t *acc = acc_full ? acc_full : (int32_t *)malloc((size_t)M * N * sizeof(int32_t));
    oracle_gemm_i8_i32(M, N, K, x1, K, x2, transB ? K : N, transB, bias, acc, N);
    if (d_out && rows_kept) {
        float *deq = (float *)malloc((size_t)rows_kept * N * sizeof(float));
        if (reduce_int32) {
            int32_t *tmp = (int32_t *)malloc((size_t)rows_kept * N * sizeof(int32_t));
            memcpy(tmp, acc + (size_t)row0 * N, (size_t)rows_kept * N * sizeof(int32_t));
            oracle_reduce_i32(rows_kept, N, tmp, N, n_peers, (const int32_t *const *)peers, ldp, peer_row0);
            oracle_dequant(rows_kept, N, tmp, N, scale_x2, scale_x1 + row0, deq, N);
            oracle_reduce_cast(rows_kept, N, deq, N, 0, NULL, 0, 0, out_dtype, d_out, N);
            free(tmp);
        } else {
            oracle_dequant(rows_kept, N, acc + (size_t)row0 * N, N, scale_x2, scale_x1 + row0, deq, N);
            oracle_reduce_cast(rows_kept, N, deq, N, n_peers, (const float *const *)peers, ldp, peer_row0,
                               out_dtype, d_out, N);
        }
        free(deq);
    }
    if (!acc_full) free(acc);
}

/* Float matmul -> reduce-scatter / all-reduce share: fp32 partial [M,N]
 * (optionally returned), kept rows [row0, row0+rows_kept) reduced with the
 * peers in fp32 and cast once.  All-reduce is the case row0 = 0, rows_kept = M
 * (KAR keeps every row on every rank). */
ORACLE_API void oracle_matmul_reduce(
    uint32_t M, uint32_t N, uint32_t K,
    const uint16_t *A, int transA, const uint16_t *B, int transB, int dtype,
    uint32_t row0, uint32_t rows_kept,
    uint32_t n_peers, const float *const *peers, int64_t ldp, int64_t peer_row0,
    float *partial_full /* [M,N] or NULL */, uint16_t *d_out)
{
    float *c = partial_full ? partial_full : (float *)malloc((size_t)M * N * sizeof(float));
    oracle_gemm_half_f32(M, N, K, A, transA ? M : K, transA, B, transB ? K : N, transB, dtype, c, N);
    if (d_out && rows_kept)
        oracle_reduce_cast(rows_kept, N, c + (size_t)row0 * N, N, n_peers, peers, ldp, peer_row0, dtype, d_out, N);
    if (!partial_full) free(c);
}

/* All-gather -> matmul (KAG:106-179): P row shards of A, each [m_local,K] in its
 * own buffer, are logically concatenated; C[p*m_local + i, :] = A_p[i,:] * B. */
ORACLE_API void oracle_allgather_matmul(
    uint32_t m_local, uint32_t N, uint32_t K, uint32_t P,
    const uint16_t *const *a_shards, const uint16_t *B, int transB, int dtype, uint16_t *C)
{
    float *c = (float *)malloc((size_t)m_local * N * sizeof(float));
    for (uint32_t p = 0; p < P; ++p) {
        oracle_gemm_half_f32(m_local, N, K, a_shards[p], K, 0, B, transB ? K : N, transB, dtype, c, N);
        oracle_cast_f32_to_half(c, C + (size_t)p * m_local * N, (size_t)m_local * N, dtype);
    }
    free(c);
}

/* ------------------------------------------------------------------------- */
/* Schedulers (pure index math)                                               */
/* ------------------------------------------------------------------------- */

static inline uint32_t ceil_div_u32(uint32_t a, uint32_t b) { return (a + b - 1u) / b; }

/* SWZ:79-113  GemmIdentityBlockSwizzle<off,dir>::GetBlockCoord on a grid of
 * loopsM x loopsN tiles.  dir 0 ("Zn"): bands of `off` tile rows, m fastest,
 * n reversed on odd bands.  dir 1 ("Nz"): bands of `off` tile columns, n
 * fastest, m reversed on odd bands.  The last band is narrower. */
ORACLE_API void oracle_swizzle_block_coord(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN,
                                           uint32_t task, uint32_t *mIdx, uint32_t *nIdx)
{
    uint32_t inner = task % (loopsM * loopsN);
    if (dir == 0) {
        uint32_t bands = ceil_div_u32(loopsM, off);
        uint32_t band = inner / (off * loopsN);
        uint32_t inBand = inner % (off * loopsN);
        uint32_t nRow = off;
        if (band == bands - 1) nRow = loopsM - off * band;
        uint32_t m = band * off + inBand % nRow;
        uint32_t n = inBand / nRow;
        if (band % 2 == 1) n = loopsN - n - 1;
        *mIdx = m; *nIdx = n;
    } else {
        uint32_t bands = ceil_div_u32(loopsN, off);
        uint32_t band = inner / (off * loopsM);
        uint32_t inBand = inner % (off * loopsM);
        uint32_t nCol = off;
        if (band == bands - 1) nCol = loopsN - off * band;
        uint32_t m = inBand / nCol;
        uint32_t n = band * off + inBand % nCol;
        if (band % 2 == 1) m = loopsM - m - 1;
        *mIdx = m; *nIdx = n;
    }
}

/* SWZ:116-124  edge tiles are the remainder. */
ORACLE_API void oracle_swizzle_actual_shape(uint32_t M, uint32_t N, uint32_t m0, uint32_t n0,
                                            uint32_t mIdx, uint32_t nIdx, uint32_t *mAct, uint32_t *nAct)
{
    uint32_t loopsM = ceil_div_u32(M, m0), loopsN = ceil_div_u32(N, n0);
    *mAct = (mIdx == loopsM - 1) ? (M - mIdx * m0) : m0;
    *nAct = (nIdx == loopsN - 1) ? (N - nIdx * n0) : n0;
}

/* SWZ:151-158  first k-tile of split-K slice s: the first kTiles % f slices own
 * one extra k-tile. */
ORACLE_API uint32_t oracle_splitk_first_ktile(uint32_t kTiles, uint32_t f, uint32_t s)
{
    if (s < kTiles % f) return (kTiles / f + 1) * s;
    return s * (kTiles / f) + kTiles % f;
}

/* SWZ:179-216 + 160-165  SplitkGemmIdentityBlockSwizzle::GetBlockCoord:
 * slice = task % coreLoops / (loopsM*loopsN); (m,n) swizzled as above. */
ORACLE_API void oracle_splitk_block_coord(uint32_t off, uint32_t dir, uint32_t loopsM, uint32_t loopsN,
                                          uint32_t kTiles, uint32_t f, uint32_t task,
                                          uint32_t *mIdx, uint32_t *nIdx, uint32_t *kIdx, uint32_t *slice)
{
    uint32_t mn = loopsM * loopsN;
    uint32_t s = task % (mn * f) / mn;
    *slice = s;
    *kIdx = oracle_splitk_first_ktile(kTiles, f, s);
    oracle_swizzle_block_coord(off, dir, loopsM, loopsN, task % mn, mIdx, nIdx);
}

/* SWZ:220-235  k extent of a split-K slice. */
ORACLE_API uint32_t oracle_splitk_actual_k(uint32_t K, uint32_t k0, uint32_t f, uint32_t s)
{
    uint32_t kTiles = ceil_div_u32(K, k0);
    uint32_t len = (s < kTiles % f) ? (kTiles / f + 1) * k0 : (kTiles / f) * k0;
    if (s == f - 1) return K - oracle_splitk_first_ktile(kTiles, f, s) * k0;
    return len;
}

/* SPK:219-265  GetSplitkFactor(m,n,k,cores) with tile (m0,n0,k0). */
ORACLE_API uint32_t oracle_splitk_factor(uint32_t m, uint32_t n, uint32_t k, uint32_t cores,
                                         uint32_t m0, uint32_t n0, uint32_t k0)
{
    uint32_t maxF = (k <= 1024) ? 2 : (k <= 2048) ? 4 : (k <= 4096) ? 8 : 16;
    uint32_t base = ceil_div_u32(m, m0) * ceil_div_u32(n, n0);
    uint32_t f = cores / base;
    if (f > maxF) f = maxF;
    if (f < 1) f = 1;
    if (base < cores) {
        while (f + 1 <= maxF && ceil_div_u32(base * f, cores) >= ceil_div_u32(base, cores) * f) f += 1;
    }
    uint32_t kt = ceil_div_u32(k, k0);
    if (f > kt) f = kt;
    if (k > 8192 && f < 2) f = 2;
    if (k > 32768 && f < 4) f = 4;
    return f;
}

/* SWAG:88-108  GemmIdentityBlockSwizzleAllGather::GetBlockCoord.
 * loopsMRank = tile rows of ONE rank's shard, loopsN = tile columns,
 * mLoopsPerComm = commInterval * P.  Within a comm round the base swizzle runs
 * on a (actualMLoops x loopsN) grid and m is remapped rank-major. */
ORACLE_API void oracle_allgather_block_coord(uint32_t off, uint32_t dir, uint32_t P, uint32_t commInterval,
                                             uint32_t loopsMRank, uint32_t loopsN, uint32_t task,
                                             uint32_t *mIdx, uint32_t *nIdx)
{
    uint32_t loopsMAll = loopsMRank * P;
    uint32_t mLoopsPerComm = commInterval * P;
    uint32_t commCount = ceil_div_u32(loopsMAll, mLoopsPerComm);
    uint32_t commIdx = task / (mLoopsPerComm * loopsN);
    uint32_t inComm = task % (mLoopsPerComm * loopsN);
    uint32_t actualMLoops = (commIdx == commCount - 1) ? loopsMAll - commIdx * mLoopsPerComm : mLoopsPerComm;
    uint32_t perRank = actualMLoops / P;
    uint32_t cm, cn;
    oracle_swizzle_block_coord(off, dir, actualMLoops, loopsN, inComm, &cm, &cn);
    uint32_t rankIdx = cm / perRank;
    *mIdx = rankIdx * loopsMRank + commIdx * (mLoopsPerComm / P) + cm % perRank;
    *nIdx = cn;
}

/* CSW:147-186  BlockCommSwizzle<dir,false>::GetBlockIdx: task -> (dataIdx, rank).
 * coreSplit = (row = data split, col = npu split); swizzleOffset = row for dir 0,
 * col for dir 1; nStride = P / col; rank is stepped by nStride then rotated by
 * dataIdx so concurrent cores address different peers. */
ORACLE_API void oracle_comm_block_idx(uint32_t dir, uint32_t P, uint32_t splitRow, uint32_t splitCol,
                                      uint32_t dataLoopsInRank, uint32_t task,
                                      uint32_t *dataIdx, uint32_t *rankIdx)
{
    uint32_t rankLoops = P;
    uint32_t nStride = P / splitCol;
    uint32_t coreLoop = dataLoopsInRank * rankLoops;
    uint32_t inner = task % coreLoop;
    uint32_t d, r;
    if (dir == 0) {
        uint32_t off = splitRow;
        uint32_t bands = ceil_div_u32(dataLoopsInRank, off);
        uint32_t band = inner / (off * rankLoops);
        uint32_t inBand = inner % (off * rankLoops);
        uint32_t nRow = off;
        if (band == bands - 1) nRow = dataLoopsInRank - off * band;
        d = band * off + inBand % nRow;
        r = inBand / nRow;
    } else {
        uint32_t off = splitCol;
        uint32_t bands = ceil_div_u32(rankLoops, off);
        uint32_t band = inner / (off * dataLoopsInRank);
        uint32_t inBand = inner % (off * dataLoopsInRank);
        uint32_t nCol = off;
        if (band == bands - 1) nCol = rankLoops - off * band;
        d = inBand / nCol;
        r = band * off + inBand % nCol;
    }
    r = (r * nStride) % rankLoops + (r * nStride) / rankLoops;
    r = (r + d) % rankLoops;
    *dataIdx = d; *rankIdx = r;
}

/* CSW:25-31,54-56,106-118,147-186  BlockCommSwizzle<0, true>: the deterministic variant.  coreSplit becomes
 * (row * col, 1), so swizzleOffset = row * col and nStride = P; GetCoreLoop pads dataLoopsInRank up to a multiple of
 * the core count and the last band is NOT narrowed, so data indices >= dataLoopsInRank occur (empty blocks). */
ORACLE_API uint32_t oracle_comm_core_loop(int deterministic, uint32_t P, uint32_t splitRow, uint32_t splitCol,
                                          uint32_t dataLoopsInRank)
{
    if (!deterministic) return dataLoopsInRank * P;
    uint32_t cores = splitRow * splitCol;
    return (dataLoopsInRank + cores - 1) / cores * cores * P;
}

ORACLE_API void oracle_comm_block_idx_det(uint32_t P, uint32_t splitRow, uint32_t splitCol, uint32_t dataLoopsInRank,
                                          uint32_t task, uint32_t *dataIdx, uint32_t *rankIdx)
{
    uint32_t off = splitRow * splitCol;
    uint32_t rankLoops = P, nStride = P / 1;
    uint32_t inner = task % oracle_comm_core_loop(1, P, splitRow, splitCol, dataLoopsInRank);
    uint32_t band = inner / (off * rankLoops);
    uint32_t inBand = inner % (off * rankLoops);
    uint32_t d = band * off + inBand % off;
    uint32_t r = inBand / off;
    r = (r * nStride) % rankLoops + (r * nStride) / rankLoops;
    r = (r + d) % rankLoops;
    *dataIdx = d; *rankIdx = r;
}

/* One 16-bit add as a hardware atomic add on fp16 / bf16 memory does it (KRS:261 under SetAtomicAdd<half>): the exact
 * sum rounded once, to nearest even, to the 16-bit type.  Computed as the fp32 sum rounded to 16 bits: fp32 carries
 * 24 significand bits, at least 2p + 2 for p = 11 (fp16) and p = 8 (bf16), so the double rounding is innocuous. */
ORACLE_API void oracle_add_half(const uint16_t *a, const uint16_t *b, size_t n, int dtype, uint16_t *out)
{
    for (size_t i = 0; i < n; ++i) out[i] = f32_to_half(half_to_f32(a[i], dtype) + half_to_f32(b[i], dtype), dtype);
}

/* SPK:24-161  ReduceAdd: dst[i] = cast(((s0[i] + s1[i]) + s2[i]) + ...), slices `count` apart, fp32 adds, one RNE cast
 * (dtype 0 keeps fp32 and writes 4-byte elements). */
ORACLE_API void oracle_reduce_add(const float *src, size_t count, uint32_t slices, int dtype, void *dst)
{
    for (size_t i = 0; i < count; ++i) {
        float s = src[i];
        for (uint32_t k = 1; k < slices; ++k) s = s + src[(size_t)k * count + i];
        if (dtype == 0) ((float *)dst)[i] = s;
        else ((uint16_t *)dst)[i] = f32_to_half(s, dtype);
    }
}

/* CSW:188-201 with layoutComm = Packed(1, dLoopsInRank, commBlockM) (KQ:257-258):
 * first row of a comm block inside one round's comm shape.  Scatter+Get and
 * Gather+Put address the slab of the CURRENT rank, the other two pairs the slab
 * of the block's rank. */
ORACLE_API uint32_t oracle_comm_block_row(uint32_t slabRank, uint32_t dataIdx,
                                          uint32_t dLoopsInRank, uint32_t commBlockM)
{
    return slabRank * dLoopsInRank * commBlockM + dataIdx * commBlockM;
}

/* KQ:122-201  reduce-scatter tile schedule.  Task t of the whole launch is
 * (commIdx = t / blockPerComm, blockIdxInComm = t % blockPerComm).  Outputs:
 * the target rank whose row block the tile belongs to, the tile coordinate
 * inside that rank's (M/P, N) sub-problem (swizzle <7,1> in every example), the
 * first global row/col of the tile, and the workspace row the reference would
 * store a non-kept tile at: (stage*blockPerComm + blockIdxInComm) * m0.
 * Returns 0 when t is past the last task. */
ORACLE_API int oracle_rs_task(uint32_t M, uint32_t N, uint32_t P, uint32_t m0, uint32_t n0,
                              uint32_t blockNum, uint32_t commInterval, uint32_t stages,
                              uint32_t off, uint32_t dir, uint32_t t,
                              uint32_t *targetRank, uint32_t *mIdx, uint32_t *nIdx,
                              uint32_t *row, uint32_t *col, uint32_t *wsRow)
{
    uint32_t mRank = M / P;
    uint32_t loopsM = ceil_div_u32(mRank, m0), loopsN = ceil_div_u32(N, n0);
    uint32_t coreLoops = loopsM * loopsN * P;
    uint32_t blockPerComm = blockNum * commInterval;
    uint32_t perRank = blockPerComm / P;
    uint32_t commLoops = ceil_div_u32(coreLoops, blockPerComm);
    if (t >= coreLoops) return 0;
    uint32_t commIdx = t / blockPerComm;
    uint32_t b = t % blockPerComm;
    uint32_t actual = (commIdx == commLoops - 1) ? (coreLoops - blockPerComm * commIdx) : blockPerComm;
    uint32_t actualInRank = actual / P;
    uint32_t loopIdxInRank = commIdx * perRank + b % actualInRank;
    uint32_t tr = b / actualInRank;
    uint32_t mi, ni;
    oracle_swizzle_block_coord(off, dir, loopsM, loopsN, loopIdxInRank, &mi, &ni);
    *targetRank = tr; *mIdx = mi; *nIdx = ni;
    *row = tr * mRank + mi * m0;
    *col = ni * n0;
    *wsRow = ((commIdx % stages) * blockPerComm + b) * m0;
    return 1;
}

/* KAR:146-179  all-reduce tile schedule: loopIdx = commIdx*blockPerComm + b over
 * the full (M,N) grid; every tile goes to workspace row (stage, b). */
ORACLE_API int oracle_ar_task(uint32_t M, uint32_t N, uint32_t m0, uint32_t n0,
                              uint32_t blockNum, uint32_t commInterval, uint32_t stages,
                              uint32_t off, uint32_t dir, uint32_t t,
                              uint32_t *mIdx, uint32_t *nIdx, uint32_t *wsRow)
{
    uint32_t loopsM = ceil_div_u32(M, m0), loopsN = ceil_div_u32(N, n0);
    if (t >= loopsM * loopsN) return 0;
    uint32_t blockPerComm = blockNum * commInterval;
    uint32_t commIdx = t / blockPerComm, b = t % blockPerComm;
    oracle_swizzle_block_coord(off, dir, loopsM, loopsN, t, mIdx, nIdx);
    *wsRow = ((commIdx % stages) * blockPerComm + b) * m0;
    return 1;
}

/* ------------------------------------------------------------------------- */
/* dynamic_tiling search space                                                */
/* ------------------------------------------------------------------------- */

typedef struct {
    uint32_t m, k, n, m0, k0, n0, commTileM, commInterval, commNpuSplit, commDataSplit, commBlockM, rankSize;
} OracleCocTilingParams; /* examples/dynamic_tiling/include/info.h:29-42 */

enum { ORACLE_MATMUL_ALLREDUCE = 0, ORACLE_ALLGATHER_MATMUL = 1, ORACLE_MATMUL_REDUCE_SCATTER = 2 };

/* TIL:32-41  blockNum * commInterval must divide by rankSize. */
ORACLE_API int oracle_check_comm_interval_reduce_scatter(const OracleCocTilingParams *t, int rankSize, int blockNum)
{
    int64_t product = (int64_t)blockNum * t->commInterval;
    return product % rankSize == 0;
}

/* TIL:43-51  per-rank peer memory = (204 MiB - 2.5 MiB) / 2 / P / 2 elements. */
ORACLE_API int oracle_check_comm_interval_allreduce(const OracleCocTilingParams *t, int rankSize, int blockNum)
{
    int32_t maxPeer = (204 * 1024 * 1024 - 5 * 512 * 1024) / 2 / rankSize / 2;
    return !(t->commInterval * t->m0 * t->n0 * (uint32_t)blockNum >= (uint32_t)maxPeer);
}

/* TIL:53-62 */
ORACLE_API int oracle_check_comm_interval_allgather(const OracleCocTilingParams *t, int rankSize)
{
    int32_t maxPeer = (204 * 1024 * 1024 - 5 * 512 * 1024) / 2 / rankSize / 2;
    uint32_t kLoop = t->k0 ? (t->k + t->k0 - 1) / t->k0 : 0;
    return !(t->commInterval * t->m0 * t->k0 * kLoop >= (uint32_t)maxPeer);
}

/* TIL:19-22,64-105  enumerate commInterval {4,6,8,12,14} x commTileM {4,8,16,32,64}
 * x (npuSplit,dataSplit) {(1,16),(1,20)} in the reference's nesting order, set
 * commBlockM = commTileM, keep those that pass the op's check.  Returns count. */
ORACLE_API int oracle_get_tilings(const OracleCocTilingParams *base, int commType, int rankSize, int blockNum,
                                  OracleCocTilingParams *out, int maxOut)
{
    static const uint32_t vInterval[5] = {4, 6, 8, 12, 14};
    static const uint32_t vTileM[5] = {4, 8, 16, 32, 64};
    static const uint32_t vSplit[2][2] = {{1, 16}, {1, 20}};
    int n = 0;
    for (int a = 0; a < 5; ++a)
        for (int b = 0; b < 5; ++b)
            for (int c = 0; c < 2; ++c) {
                OracleCocTilingParams t = *base;
                t.commInterval = vInterval[a];
                t.commTileM = vTileM[b];
                t.commBlockM = t.commTileM;
                t.commNpuSplit = vSplit[c][0];
                t.commDataSplit = vSplit[c][1];
                if (commType == ORACLE_ALLGATHER_MATMUL && !oracle_check_comm_interval_allgather(&t, rankSize)) continue;
                if (commType == ORACLE_MATMUL_REDUCE_SCATTER &&
                    !oracle_check_comm_interval_reduce_scatter(&t, rankSize, blockNum)) continue;
                if (commType == ORACLE_MATMUL_ALLREDUCE &&
                    !oracle_check_comm_interval_allreduce(&t, rankSize, blockNum)) continue;
                if (n < maxOut) out[n] = t;
                ++n;
            }
    return n;
}

/* ------------------------------------------------------------------------- */
/* Accuracy gate                                                              */
/* ------------------------------------------------------------------------- */

/* VER: utils.py:44-52 (rtol) and verify_result.py:34-43,88-117: every element
 * |out-gold| <= rtol*max(1,|gold|), and |mean((out-gold)/max(1,|gold|))| <= eb
 * with eb = 2^-10 (fp16) / 2^-7 (bf16); NaN/Inf are zeroed first.
 * Returns 1 on pass; *n_bad = failing elements, *eb = the mean relative error. */
ORACLE_API int oracle_verify(const float *out, const float *gold, size_t n, int dtype, uint32_t computeTimes,
                             uint64_t *n_bad, double *eb)
{
    double rtol, ebThr;
    if (dtype == ORACLE_FP16) { rtol = computeTimes < 2048 ? 1.0 / 256 : 1.0 / 128; ebThr = 1.0 / 1024; }
    else { rtol = computeTimes < 2048 ? 1.0 / 128 : 1.0 / 64; ebThr = 1.0 / 128; }
    uint64_t bad = 0;
    double acc = 0.0;
    for (size_t i = 0; i < n; ++i) {
        float o = out[i], g = gold[i];
        if (isnan(o) || isinf(o)) o = 0.0f;
        if (isnan(g) || isinf(g)) g = 0.0f;
        float diff = o - g;
        float mx = fabsf(g) > 1.0f ? fabsf(g) : 1.0f;
        if (fabsf(diff) - (float)rtol * mx > 0.0f) ++bad;
        acc += (double)(diff / mx);
    }
    double e = n ? fabs(acc / (double)n) : 0.0;
    if (n_bad) *n_bad = bad;
    if (eb) *eb = e;
    return bad == 0 && e <= ebThr;
}

ORACLE_API int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
