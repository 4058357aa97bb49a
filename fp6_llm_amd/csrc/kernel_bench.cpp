// Command-line benchmark / smoke driver over the C ABI, the counterpart of the reference's C++ harness
// (tests/cpp/kernel_test_fpx.cu:8-17: `kernel_test_fpx E M OC IC BS SplitK`).
//   kernel_bench E M OC IC BS SplitK [iters=200] [warmup=20] [pool_MiB=1024]
// Weights are random bytes in the native layout (every bit pattern is a valid code), rotated through a pool of distinct
// buffers larger than the 256 MB last-level cache so that every launch streams its weights from HBM.
// Prints microseconds per GEMM, TFLOP/s = 2*OC*IC*BS/t (tests/cpp/kernel_test.h:59-66) and weight GB/s, then the same for an
// FP16 GEMM of that shape through rocblas_gemm_ex (FP32 accumulation; rocBLAS dispatches to hipBLASLt on this part) with
// its FP16 weights rotating the same way -- the part cublasGemmEx plays in tests/cpp/kernel_test_fpx.cu:80-103 -- and the speed-up.
#include <hip/hip_runtime.h>
#include <rocblas/rocblas.h>

#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <random>
#include <string>
#include <vector>

#include "fp6_linear.h"

#define BLAS_OK(x)                                                                     \
    do {                                                                               \
        rocblas_status s_ = (x);                                                       \
        if (s_ != rocblas_status_success) {                                            \
            std::fprintf(stderr, "%s failed: rocblas status %d\n", #x, (int)s_);       \
            return 2;                                                                  \
        }                                                                              \
    } while (0)

// out[BS, OC] (row-major) = X[BS, IC] * W16[OC, IC]^T in FP16 with FP32 accumulation.  In rocBLAS' column-major terms:
// C[OC x BS] = op_T(A = W16 as IC x OC, ld IC) * (B = X as IC x BS, ld IC).
static rocblas_status fp16_gemm(rocblas_handle h, const void *W16, const void *X, void *C, size_t OC, size_t BS, size_t IC)
{
    const float alpha = 1.0f, beta = 0.0f;
    return rocblas_gemm_ex(h, rocblas_operation_transpose, rocblas_operation_none, (rocblas_int)OC, (rocblas_int)BS, (rocblas_int)IC, &alpha, W16,
                           rocblas_datatype_f16_r, (rocblas_int)IC, X, rocblas_datatype_f16_r, (rocblas_int)IC, &beta, C, rocblas_datatype_f16_r,
                           (rocblas_int)OC, C, rocblas_datatype_f16_r, (rocblas_int)OC, rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
}

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
    { // the reference prints the same ratio against the FP16 library GEMM of the dequantized weights (tests/cpp/kernel_test_fpx.cu:150-160)
        void *dW16, *dC16;
        std::vector<fp6mi_half> out16(BS * OC);
        HIP_OK(hipMalloc(&dW16, OC * IC * 2));
        HIP_OK(hipMalloc(&dC16, BS * OC * 2));
        HIP_OK(hipMemcpy(dW16, wdq.data(), OC * IC * 2, hipMemcpyHostToDevice));
        rocblas_handle h;
        BLAS_OK(rocblas_create_handle(&h));
        BLAS_OK(fp16_gemm(h, dW16, dX, dC16, OC, BS, IC));
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(out16.data(), dC16, BS * OC * 2, hipMemcpyDeviceToHost));
        long double e2 = 0, r2 = 0;
        for (size_t i = 0; i < BS * OC; i++) { e2 += std::fabs((double)out[i] - (double)out16[i]); r2 += std::fabs((double)out16[i]); }
        std::printf("      against the FP16 rocBLAS GEMM of the dequantized weights: sum|err|/sum|ref| = %.3e\n", (double)(e2 / r2));
        BLAS_OK(rocblas_destroy_handle(h));
        HIP_OK(hipFree(dW16));
        HIP_OK(hipFree(dC16));
    }
    if (int rc = fp6mi_twin_clear()) { std::fprintf(stderr, "twin_clear: %s\n", fp6mi_error_string(rc)); return 2; }
    return ratio < 2e-3 ? 0 : 3;
}

// FP16 baseline: same shape, FP16 weights (arbitrary finite values) rotating through a pool of the same size, launched
// back to back on one stream like the FPx GEMM above.
static int fp16_baseline(size_t OC, size_t IC, size_t BS, int iters, int warmup, size_t pool, void *dX, void *dC, hipStream_t st, double *us_out)
{
    size_t n16 = pool / (OC * IC * 2);
    if (n16 < 2) n16 = 2;
    if (n16 > 64) n16 = 64;
    std::mt19937          rng(99);
    std::vector<_Float16> hw16(OC * IC);
    for (auto &v : hw16) v = (_Float16)(((int)(rng() % 57) - 28) * 0.01f);
    std::vector<void *> dW16(n16);
    for (size_t i = 0; i < n16; i++) {
        HIP_OK(hipMalloc(&dW16[i], OC * IC * 2));
        HIP_OK(hipMemcpy(dW16[i], hw16.data(), OC * IC * 2, hipMemcpyHostToDevice));
    }
    rocblas_handle h;
    BLAS_OK(rocblas_create_handle(&h));
    BLAS_OK(rocblas_set_stream(h, st));
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    for (int i = 0; i < warmup; i++) BLAS_OK(fp16_gemm(h, dW16[i % n16], dX, dC, OC, BS, IC));
    double best = 1e30;
    for (int rep = 0; rep < 5; rep++) { // the first repetitions also settle the clocks; the median-like minimum of the last three counts
        HIP_OK(hipStreamSynchronize(st));
        HIP_OK(hipEventRecord(e0, st));
        for (int i = 0; i < iters; i++) BLAS_OK(fp16_gemm(h, dW16[i % n16], dX, dC, OC, BS, IC));
        HIP_OK(hipEventRecord(e1, st));
        HIP_OK(hipEventSynchronize(e1));
        float ms = 0;
        HIP_OK(hipEventElapsedTime(&ms, e0, e1));
        if (rep >= 2 && ms * 1e3 / iters < best) best = ms * 1e3 / iters;
    }
    std::printf("FP16 rocblas_gemm_ex OC=%zu IC=%zu BS=%zu buffers=%zu: %.2f us/GEMM  %.2f TFLOP/s\n", OC, IC, BS, n16, best,
                2.0 * OC * IC * BS / best / 1e6);
    BLAS_OK(rocblas_destroy_handle(h));
    for (void *p : dW16) HIP_OK(hipFree(p));
    *us_out = best;
    return 0;
}

// `kernel_bench fp16 OC IC BS [iters] [warmup] [pool_MiB]`: only the FP16 library GEMM (what the Python benchmark calls to time
// the system's rocBLAS/hipBLASLt in a process of its own).
static int fp16_main(int argc, char **argv)
{
    if (argc < 5) { std::fprintf(stderr, "usage: %s fp16 OC IC BS [iters] [warmup] [pool_MiB]\n", argv[0]); return 1; }
    size_t OC = std::strtoull(argv[2], nullptr, 10), IC = std::strtoull(argv[3], nullptr, 10), BS = std::strtoull(argv[4], nullptr, 10);
    int    iters = argc > 5 ? std::atoi(argv[5]) : 200, warmup = argc > 6 ? std::atoi(argv[6]) : 20;
    size_t pool = (argc > 7 ? std::strtoull(argv[7], nullptr, 10) : 1024) << 20;
    std::vector<_Float16> hx(BS * IC);
    std::mt19937          rng(5);
    std::normal_distribution<float> nx(0.f, 1.f);
    for (auto &v : hx) v = (_Float16)nx(rng);
    void *dX, *dC;
    HIP_OK(hipMalloc(&dX, BS * IC * 2));
    HIP_OK(hipMalloc(&dC, BS * OC * 2));
    HIP_OK(hipMemcpy(dX, hx.data(), BS * IC * 2, hipMemcpyHostToDevice));
    hipStream_t st;
    HIP_OK(hipStreamCreate(&st));
    double us = 0;
    return fp16_baseline(OC, IC, BS, iters, warmup, pool, dX, dC, st, &us);
}

int main(int argc, char **argv)
{
    if (argc > 1 && std::string(argv[1]) == "check") return check_main(argc, argv);
    if (argc > 1 && std::string(argv[1]) == "fp16") return fp16_main(argc, argv);
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

    for (void *p : dW) HIP_OK(hipFree(p));
    double us16 = 0;
    if (int rc = fp16_baseline(OC, IC, BS, iters, warmup, pool, dX, dC, st, &us16)) return rc;
    std::printf("      speed-up of the FPx GEMM over it: %.2f\n", us16 / us_per);
    return 0;
}
