// Sanitizer run of the CPU code: the engine's host functions (fp6_llm_amd/csrc/fp6mi_host.cpp) and the test oracle
// (oracle/fpx_oracle.c), built with AddressSanitizer and UndefinedBehaviorSanitizer and driven over every format, shapes
// with K not a multiple of 256, in-place packing and the grouped dequantizer; the two implementations are compared on the way.
// Role: the CPU-side sanitizer build of the reference's development practice (no GPU is involved).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../fp6_llm_amd/csrc/fp6mi_internal.h"

extern "C" {
int orc_prepack(int E, int M, uint8_t *out, const uint8_t *in, size_t rows, size_t K);
int orc_dequant(int E, int M, uint16_t *out, const uint8_t *raw, size_t rows, size_t K, const uint16_t *scale);
int orc_unpack_codes(int E, int M, uint8_t *codes, const uint8_t *raw, size_t rows, size_t K);
int orc_gemm(uint16_t *out, const uint16_t *Wdq, const uint16_t *X, size_t M, size_t N, size_t K, int splitK);
uint16_t orc_float_to_half(float f);
}
using namespace fp6mi;

#define CHECK(cond)                                                                                      \
    do {                                                                                                 \
        if (!(cond)) { std::printf("FAILED %s (line %d): E=%d M=%d rows=%zu K=%zu\n", #cond, __LINE__, E, Mb, M, K); return 1; } \
    } while (0)

int main()
{
    const int    fmts[4][2] = { { 3, 2 }, { 2, 2 }, { 2, 3 }, { 2, 1 } };
    const size_t shapes[][2] = { { 64, 64 }, { 64, 320 }, { 128, 192 }, { 256, 1024 }, { 64, 4160 } };
    std::srand(12345);
    for (auto &f : fmts)
        for (auto &s : shapes) {
            const int    E = f[0], Mb = f[1], x = 1 + E + Mb;
            const size_t M = s[0], K = s[1], rb = K * x / 8;
            std::vector<uint8_t> raw(M * rb), packed(M * rb), want(M * rb), back(M * rb), back2(M * rb);
            for (auto &b : raw) b = (uint8_t)std::rand();
            CHECK(prepack_ref(E, Mb, packed.data(), raw.data(), M, K) == 0);
            CHECK(orc_prepack(E, Mb, want.data(), raw.data(), M, K) == 0 && want == packed);
            CHECK(unpack_ref(E, Mb, back.data(), packed.data(), M, K) == 0 && back == raw);
            std::vector<uint8_t> nat(native_bytes(E, Mb, M, K)), nat2(nat.size());
            CHECK(prepack_native(E, Mb, nat.data(), raw.data(), M, K) == 0);
            CHECK(unpack_native(E, Mb, back2.data(), nat.data(), M, K) == 0 && back2 == raw);
            CHECK(relayout_ref_to_native(E, Mb, nat2.data(), packed.data(), M, K) == 0 && nat2 == nat);
            std::vector<uint16_t> sc(M), out(M * K), out_orc(M * K), out_g(M * K);
            for (auto &v : sc) v = orc_float_to_half(0.001f + 0.009f * (float)std::rand() / (float)RAND_MAX);
            CHECK(dequant(E, Mb, out.data(), raw.data(), M, K, sc.data()) == 0);
            CHECK(orc_dequant(E, Mb, out_orc.data(), raw.data(), M, K, sc.data()) == 0 && out == out_orc);
            const size_t groups = (K + 127) / 128;
            std::vector<uint8_t> ex(M * groups, 127), exn(group_exps_bytes(M, K));
            CHECK(dequant_grouped(E, Mb, out_g.data(), raw.data(), M, K, sc.data(), ex.data()) == 0 && out_g == out); // factor 2^0
            for (auto &b : ex) b = (uint8_t)(112 + std::rand() % 16);
            CHECK(dequant_grouped(E, Mb, out_g.data(), raw.data(), M, K, sc.data(), ex.data()) == 0);
            CHECK(pack_group_exps(exn.data(), ex.data(), M, K) == 0);
            std::vector<uint8_t> codes(M * K);
            CHECK(orc_unpack_codes(E, Mb, codes.data(), raw.data(), M, K) == 0);
            std::vector<uint8_t> inpl = raw; // packing in place, as the reference's callers do
            CHECK(prepack_ref(E, Mb, inpl.data(), inpl.data(), M, K) == 0 && inpl == packed);
            if (M * K <= 64 * 320) { // the oracle's GEMM with and without a split
                const size_t          N = 3;
                std::vector<uint16_t> X(N * K), y1(N * M), y2(N * M);
                for (auto &v : X) v = orc_float_to_half((float)(std::rand() % 17 - 8) / 8.0f);
                CHECK(orc_gemm(y1.data(), out.data(), X.data(), M, N, K, 1) == 0 && orc_gemm(y2.data(), out.data(), X.data(), M, N, K, 2) == 0);
            }
            // bad arguments come back as error codes
            CHECK(prepack_ref(4, 3, packed.data(), raw.data(), M, K) != 0 && prepack_ref(E, Mb, packed.data(), raw.data(), M + 1, K) != 0);
        }
    std::puts("host code and oracle clean under ASan + UBSan");
    return 0;
}
