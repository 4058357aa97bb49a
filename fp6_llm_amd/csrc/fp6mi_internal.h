// Internal declarations shared by the host code and the kernel translation unit.
#ifndef FP6MI_INTERNAL_H
#define FP6MI_INTERNAL_H

#include <cmath>
#include <cstddef>
#include <cstdint>

#include "../../include/fp6mi.h"

namespace fp6mi {

// FP6_e3m2 and FP5_e2m2 (the formats of the reference's entry points), FP6_e2m3 and FP4_e2m1 (through the same paths)
inline bool supported(int E, int Mbits) { return (E == 3 && Mbits == 2) || (E == 2 && (Mbits == 1 || Mbits == 2 || Mbits == 3)); }

// fp6mi_gemm.hip, compiled once per format: the entry functions of one weight format (stream = hipStream_t)
// kind 0: gemm_stream (wr == 1, wk = wavefronts per workgroup);  kind 1: gemm_tile (wr x wk wavefronts)
struct LaunchCfg { int kind, nt, rt, wr, wk; };
struct FormatOps {
    int bits;
    // gexp: group exponents in their native layout (one byte per row and 128 columns), or null
    int (*gemm)(const LaunchCfg &c, void *stream, const void *W, const void *sc, const void *gexp, const void *B, void *C, float *ws, size_t M,
                size_t N, size_t K, int splitK);
    int (*relayout)(void *stream, void *native, const void *packed_ref, size_t M, size_t K);
    int (*dequant)(void *stream, void *out_f16, const void *W, const void *sc, const void *gexp, size_t M, size_t K);
    int (*quantize)(void *stream, void *native, void *scales, void *gexp, const void *weights, int dtype, size_t M, size_t K); // gexp may be null
};
const FormatOps &format_ops_32(), &format_ops_22(), &format_ops_23(), &format_ops_21(); // named by 10*E + M
inline const FormatOps *ops_for(int E, int Mbits)
{
    return E == 3 ? &format_ops_32() : Mbits == 2 ? &format_ops_22() : Mbits == 3 ? &format_ops_23() : &format_ops_21();
}

// fp6mi_host.cpp
int    prepack_ref(int E, int Mb, void *packed, const void *raw, size_t M, size_t K);
int    unpack_ref(int E, int Mb, void *raw, const void *packed, size_t M, size_t K);
int    dequant(int E, int Mb, void *out_f16, const void *raw, size_t M, size_t K, const void *scales_f16);
size_t native_block_bytes(int x);
size_t native_bytes(int E, int Mb, size_t M, size_t K);
int    prepack_native(int E, int Mb, void *native, const void *raw, size_t M, size_t K);
int    unpack_native(int E, int Mb, void *raw, const void *native, size_t M, size_t K);
int    relayout_ref_to_native(int E, int Mb, void *native, const void *packed_ref, size_t M, size_t K);
size_t group_exps_bytes(size_t M, size_t K);
int    pack_group_exps(void *native_exps, const void *exps, size_t M, size_t K);
int    dequant_grouped(int E, int Mb, void *out_f16, const void *raw, size_t M, size_t K, const void *scales_f16, const void *exps);

} // namespace fp6mi
#endif
