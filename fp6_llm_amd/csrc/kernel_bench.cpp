// Command-line benchmark / smoke driver over the C ABI, the counterpart of the reference's C++ harness
// (tests/cpp/kernel_test_fpx.cu:8-17: `kernel_test_fpx E M OC IC BS SplitK`).
//   kernel_bench E M OC IC BS SplitK [iters=200] [warmup=20] [pool_MiB=1024]
// Weights are random bytes in the native layout (every bit pattern is a valid code), rotated through a pool of distinct
// buffers larger than the 256 MB last-level cache so that every launch streams its weights from HBM.
// Prints microseconds per GEMM, TFLOP/s = 2*OC*IC*BS/t (tests/cpp/kernel_test.h:59-66) and weight GB/s.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <random>
#include <string>
#include <vector>

#include "fp6_linear.h"

#define HIP_OK(x)                                                                      \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            std::fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));        \
            return 2;                                                                  \
        }                                                                              \
    } while (0)

// `kernel_bench check E M OC IC BS SplitK`: the flow of the reference's C++ test (tests/cpp/kernel_test_fpx.cu:19-33,128-149)
// through the reference-named C++ API: random raw bytes, dequantize on the CPU BEFORE prepacking in place, upload the
// reference-layout buffer, run the GEMM, and print sum|err|/sum|ref| against a double-precision product of the
// dequantized weights (tests/cpp/kernel_test.h:48-57).  Exit status 0 iff that ratio is below 2e-3.
static int check_main(int argc, char **argv)
{
    if (argc < 8) { std::fprintf(stderr, "usage: %s check E M OC IC BS SplitK\n", argv[0]); return 1; }
    int    E = std::atoi(argv[2]), Mb = std::atoi(argv[3]);
    size_t OC = std::strtoull(argv[4], nullptr, 10), IC = std::strtoull(argv[5], nullptr, 10), BS = std::strtoull(argv[6], nullptr, 10);
    int    splitK = std::atoi(argv[7]);
    size_t wbytes = OC * IC * (1 + E + Mb) / 8;
    std::vector<unsigned char> raw(wbytes);
    std::mt19937               rng(7);
    for (auto &b : raw) b = (unsigned char)(rng() & 255);
    std::vector<fp6mi_half> sc(OC), x(BS * IC), wdq(OC * IC), out(BS * OC);
    for (auto &v : sc) v = (fp6mi_half)((float)(rng() % 256 + 1) / 4096.0f);
    for (auto &v : x) v = (fp6mi_half)(((int)(rng() % 5) - 2) * 0.1f - 0.1f);
    if (int rc = dequant_matrix_fp_eXmY_to_fp16(E, Mb, wdq.data(), raw.data(), OC, IC, sc.data())) { std::fprintf(stderr, "dequant: %s\n", fp6mi_error_string(rc)); return 2; }
    if (int rc = weight_matrix_prepacking_fp_eXmY(E, Mb, reinterpret_cast<int *>(raw.data()), reinterpret_cast<int *>(raw.data()), OC, IC)) {
        std::fprintf(stderr, "prepack: %s\n", fp6mi_error_string(rc));
        return 2;
    }
    void  *dW, *dS, *dX, *dC;
    float *dWs = nullptr;
    HIP_OK(hipMalloc(&dW, wbytes));
    HIP_OK(hipMalloc(&dS, OC * 2));
    HIP_OK(hipMalloc(&dX, BS * IC * 2));
    HIP_OK(hipMalloc(&dC, BS * OC * 2));
    HIP_OK(hipMemcpy(dW, raw.data(), wbytes, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dS, sc.data(), OC * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dX, x.data(), BS * IC * 2, hipMemcpyHostToDevice));
    if (splitK > 1) HIP_OK(hipMalloc(reinterpret_cast<void **>(&dWs), fp6mi_workspace_bytes(OC, BS, splitK)));
    for (int rep = 0; rep < 2; rep++) { // the second call reuses the native twin made by the first
        int rc = fp_eXmY_linear_kernel(E, Mb, nullptr, dW, static_cast<fp6mi_half *>(dS), static_cast<fp6mi_half *>(dX), static_cast<fp6mi_half *>(dC), OC,
                                       BS, IC, dWs, splitK);
        if (rc) { std::fprintf(stderr, "fp_eXmY_linear_kernel: %s\n", fp6mi_error_string(rc)); return 2; }
    }
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(out.data(), dC, BS * OC * 2, hipMemcpyDeviceToHost));
    long double err = 0, ref = 0;
    for (size_t n = 0; n < BS; n++)
        for (size_t m = 0; m < OC; m++) {
            double acc = 0;
            for (size_t k = 0; k < IC; k++) acc += (double)wdq[m * IC + k] * (double)x[n * IC + k];
            err += std::fabs((double)out[n * OC + m] - acc);
            ref += std::fabs(acc);
        }
    double ratio = (double)(err / ref);
    std::printf("check E%dM%d OC=%zu IC=%zu BS=%zu splitK=%d: sum|err|/sum|ref| = %.3e\n", E, Mb, OC, IC, BS, splitK, ratio);
    if (int rc = fp6mi_twin_clear()) { std::fprintf(stderr, "twin_clear: %s\n", fp6mi_error_string(rc)); return 2; }
    return ratio < 2e-3 ? 0 : 3;
}

int main(int argc, char **argv)
{
    if (argc > 1 && std::string(argv[1]) == "check") return check_main(argc, argv);
    if (argc < 7) {
        std::fprintf(stderr, "usage: %s E M OC IC BS SplitK [iters] [warmup] [pool_MiB]\n", argv[0]);
        return 1;
    }
    int    E = std::atoi(argv[1]), Mb = std::atoi(argv[2]);
    size_t OC = std::strtoull(argv[3], nullptr, 10), IC = std::strtoull(argv[4], nullptr, 10), BS = std::strtoull(argv[5], nullptr, 10);
    int    splitK = std::atoi(argv[6]);
    int    iters = argc > 7 ? std::atoi(argv[7]) : 200, warmup = argc > 8 ? std::atoi(argv[8]) : 20;
    size_t pool = (argc > 9 ? std::strtoull(argv[9], nullptr, 10) : 1024) << 20;

    size_t nbytes = fp6mi_native_bytes(E, Mb, OC, IC);
    if (!nbytes) { std::fprintf(stderr, "unsupported format or shape\n"); return 1; }
    size_t nbuf = pool / nbytes;
    if (nbuf < 1) nbuf = 1;
    if (nbuf > 256) nbuf = 256;

    std::vector<uint32_t> hw(nbytes / 4);
    std::mt19937          rng(1234);
    for (auto &w : hw) w = rng();
    std::vector<_Float16> hs(OC), hx(BS * IC);
    std::uniform_real_distribution<float> us(1e-3f, 1e-2f);
    std::normal_distribution<float>       nx(0.f, 1.f);
    for (auto &v : hs) v = (_Float16)us(rng);
    for (auto &v : hx) v = (_Float16)nx(rng);

    std::vector<void *> dW(nbuf);
    for (size_t i = 0; i < nbuf; i++) {
        HIP_OK(hipMalloc(&dW[i], nbytes));
        HIP_OK(hipMemcpy(dW[i], hw.data(), nbytes, hipMemcpyHostToDevice));
    }
    void  *dS, *dX, *dC;
    float *dWs = nullptr;
    HIP_OK(hipMalloc(&dS, OC * 2));
    HIP_OK(hipMalloc(&dX, BS * IC * 2));
    HIP_OK(hipMalloc(&dC, BS * OC * 2));
    HIP_OK(hipMemcpy(dS, hs.data(), OC * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dX, hx.data(), BS * IC * 2, hipMemcpyHostToDevice));
    if (splitK > 1) HIP_OK(hipMalloc(reinterpret_cast<void **>(&dWs), fp6mi_workspace_bytes(OC, BS, splitK)));

    hipStream_t st;
    HIP_OK(hipStreamCreate(&st));
    for (int i = 0; i < warmup; i++) {
        int rc = fp6mi_linear_native(E, Mb, st, dW[i % nbuf], dS, dX, dC, OC, BS, IC, dWs, splitK);
        if (rc) { std::fprintf(stderr, "fp6mi_linear_native: %s\n", fp6mi_error_string(rc)); return 2; }
    }
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    HIP_OK(hipStreamSynchronize(st));
    HIP_OK(hipEventRecord(e0, st));
    for (int i = 0; i < iters; i++) {
        int rc = fp6mi_linear_native(E, Mb, st, dW[i % nbuf], dS, dX, dC, OC, BS, IC, dWs, splitK);
        if (rc) { std::fprintf(stderr, "fp6mi_linear_native: %s\n", fp6mi_error_string(rc)); return 2; }
    }
    HIP_OK(hipEventRecord(e1, st));
    HIP_OK(hipEventSynchronize(e1));
    float ms = 0;
    HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    double us_per = ms * 1e3 / iters, wbytes = (double)OC * IC * (1 + E + Mb) / 8.0;
    std::printf("E%dM%d OC=%zu IC=%zu BS=%zu splitK=%d buffers=%zu: %.2f us/GEMM  %.2f TFLOP/s  %.0f GB/s (weight bytes)\n", E, Mb, OC, IC, BS,
                splitK, nbuf, us_per, 2.0 * OC * IC * BS / us_per / 1e6, wbytes / us_per / 1e3);
    return 0;
}
