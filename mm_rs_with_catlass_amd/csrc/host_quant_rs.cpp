// Stand-alone C++ host for the W8A8 matmul-reduce-scatter entry point of libcatcoc_hip.so: the role of
// main() in examples/02_matmul_reduce_scatter/quant_matmul_reduce_scatter.cpp:253-365 of the reference,
// for one rank on one GPU.  It shows the library driven through its C ABI alone (no Python, no torch):
// the host links the HIP runtime itself, fills a CatcocSymmetricDesc where the reference calls the
// SHMEM runtime, and uses the reference's raw file conventions:
//
//   <dir>/x1_gm.bin        int8  [m,k]          <dir>/scale_x1_gm.bin  fp32 [m]
//   <dir>/x2_gm.bin        int8  [k,n]          <dir>/scale_x2_gm.bin  fp32 [n]
//   <dir>/bias_gm.bin      int32 [n]  (optional)
//   <dir>/peer_<s>.bin     fp32  [m/rankSize, n], s = 0..rankSize-2: the other ranks' dequantised partials
//                          for this rank's rows (what the SHMEM gets would have pulled)
//   <dir>/output.bin       bf16  [m,n]: this rank's [m/rankSize, n] block is written at its offset
//   <dir>/golden.bin       fp32  [m,n]  (optional): when present, this rank's rows are checked against it with the
//                          reference's accuracy gate (examples/utils/verify_quant_result.py) and the exit code is 4 on failure
//
// usage: catcoc_quant_rs_host <rankSize> <rankId> <m> <n> <k> [dir=./output]
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "catcoc_hip.h"

#define HIP_OK(call)                                                                                \
    do {                                                                                            \
        hipError_t e_ = (call);                                                                     \
        if (e_ != hipSuccess) {                                                                     \
            std::fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
            return 2;                                                                               \
        }                                                                                           \
    } while (0)

static bool read_file(const std::string &path, void *dst, size_t bytes)
{
    FILE *f = std::fopen(path.c_str(), "rb");
    if (!f) return false;
    const size_t got = std::fread(dst, 1, bytes, f);
    std::fclose(f);
    return got == bytes;
}

static bool write_file_at(const std::string &path, const void *src, size_t bytes, size_t offset)
{
    FILE *f = std::fopen(path.c_str(), "r+b");
    if (!f) f = std::fopen(path.c_str(), "w+b");
    if (!f) return false;
    bool ok = std::fseek(f, (long)offset, SEEK_SET) == 0 && std::fwrite(src, 1, bytes, f) == bytes;
    std::fclose(f);
    return ok;
}

template <typename T>
static int upload(const std::string &path, size_t count, T **dev, bool optional = false)
{
    std::vector<T> host(count);
    *dev = nullptr;
    if (!read_file(path, host.data(), count * sizeof(T))) {
        if (optional) return 0;
        std::fprintf(stderr, "cannot read %zu bytes from %s\n", count * sizeof(T), path.c_str());
        return 1;
    }
    HIP_OK(hipMalloc((void **)dev, count * sizeof(T)));
    HIP_OK(hipMemcpy(*dev, host.data(), count * sizeof(T), hipMemcpyHostToDevice));
    return 0;
}

int main(int argc, char **argv)
{
    if (argc < 6) {
        std::fprintf(stderr, "usage: %s <rankSize> <rankId> <m> <n> <k> [dir]\n", argv[0]);
        return 1;
    }
    const uint32_t rankSize = (uint32_t)std::atoi(argv[1]), rankId = (uint32_t)std::atoi(argv[2]);
    const uint32_t m = (uint32_t)std::atoi(argv[3]), n = (uint32_t)std::atoi(argv[4]), k = (uint32_t)std::atoi(argv[5]);
    const std::string dir = argc > 6 ? argv[6] : "./output";
    if (rankSize == 0 || rankSize > CATCOC_MAX_RANKS || rankId >= rankSize || m % rankSize != 0) {
        std::fprintf(stderr, "bad rank arguments\n");
        return 1;
    }
    const uint32_t rows = m / rankSize;

    hipStream_t stream;
    HIP_OK(hipSetDevice(0));
    HIP_OK(hipStreamCreate(&stream));

    int8_t *x1, *x2;
    float *s1, *s2;
    int32_t *bias;
    if (upload(dir + "/x1_gm.bin", (size_t)m * k, &x1) || upload(dir + "/x2_gm.bin", (size_t)k * n, &x2) ||
        upload(dir + "/scale_x1_gm.bin", (size_t)m, &s1) || upload(dir + "/scale_x2_gm.bin", (size_t)n, &s2) ||
        upload(dir + "/bias_gm.bin", (size_t)n, &bias, true))
        return 1;

    CatcocSymmetricDesc desc = {};
    desc.magic = CATCOC_DESC_MAGIC;
    desc.rankIdx = rankId;
    desc.rankSize = rankSize;
    desc.peerLd = n;
    std::vector<float *> peers(rankSize - 1);
    for (uint32_t s = 0; s + 1 < rankSize; ++s) {
        if (upload(dir + "/peer_" + std::to_string(s) + ".bin", (size_t)rows * n, &peers[s])) return 1;
        desc.peers[s] = peers[s];
    }

    int32_t *cAccum;
    uint16_t *dOut;
    HIP_OK(hipMalloc((void **)&cAccum, (size_t)rows * n * sizeof(int32_t)));
    HIP_OK(hipMemset(cAccum, 0, (size_t)rows * n * sizeof(int32_t)));
    HIP_OK(hipMalloc((void **)&dOut, (size_t)rows * n * sizeof(uint16_t)));

    if (std::getenv("CATCOC_HOST_VERBOSE")) std::printf("%s\n", catcoc_version());
    catcoc_quant_matmul_reduce_scatter(stream, 0, (uint8_t *)x1, (uint8_t *)x2, (uint8_t *)s1, (uint8_t *)s2, (uint8_t *)bias,
                                       (uint8_t *)cAccum, (uint8_t *)dOut, (uint8_t *)&desc, m, n, k);
    if (catcoc_last_status() != 0) {
        std::fprintf(stderr, "launch rejected: %s\n", catcoc_last_error());
        return 3;
    }
    HIP_OK(hipStreamSynchronize(stream));

    std::vector<uint16_t> out((size_t)rows * n);
    HIP_OK(hipMemcpy(out.data(), dOut, out.size() * sizeof(uint16_t), hipMemcpyDeviceToHost));
    if (!write_file_at(dir + "/output.bin", out.data(), out.size() * sizeof(uint16_t), (size_t)rankId * out.size() * sizeof(uint16_t))) {
        std::fprintf(stderr, "cannot write %s/output.bin\n", dir.c_str());
        return 1;
    }
    if (rankId == 0) std::printf("test finished\n");

    // verify_quant_result.py's check, when the reference's golden.bin (fp32 [m,n]) sits next to the inputs: this rank's rows
    // of the output against the golden's, through the library's own accuracy gate
    int verdict = 0;
    {
        std::vector<float> gold((size_t)rows * n);
        FILE *f = std::fopen((dir + "/golden.bin").c_str(), "rb");
        if (f != nullptr) {
            const bool got = std::fseek(f, (long)((size_t)rankId * gold.size() * sizeof(float)), SEEK_SET) == 0 &&
                             std::fread(gold.data(), sizeof(float), gold.size(), f) == gold.size();
            std::fclose(f);
            if (got) {
                std::vector<float> outF(out.size());
                for (size_t i = 0; i < out.size(); ++i) {   // bf16 bit pattern -> fp32
                    const uint32_t u = (uint32_t)out[i] << 16;
                    std::memcpy(&outF[i], &u, 4);
                }
                uint64_t nBad = 0;
                double mean = 0.0;
                const int pass = catcoc_verify(outF.data(), gold.data(), outF.size(), BF16, k, &nBad, &mean);
                std::printf("[verify] rank %u: %s (%llu of %zu elements outside rtol, mean relative error %.3e)\n", rankId,
                            pass ? "PASS" : "FAIL", (unsigned long long)nBad, outF.size(), mean);
                verdict = pass ? 0 : 4;
            }
        }
    }

    for (float *p : peers) (void)hipFree(p);
    (void)hipFree(x1); (void)hipFree(x2); (void)hipFree(s1); (void)hipFree(s2);
    if (bias) (void)hipFree(bias);
    (void)hipFree(cAccum); (void)hipFree(dOut);
    (void)hipStreamDestroy(stream);
    return verdict;
}
