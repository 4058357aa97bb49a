// C++ API with the names and argument meaning of the reference's fp6_llm/csrc/fp6_linear.cuh:8-43, as inline wrappers
// over the C ABI (include/fp6mi.h).  Differences a caller sees: the stream is a hipStream_t, half is _Float16, and the
// functions return the C ABI's int status (0 = success; see fp6mi_error_string) instead of cudaError_t / aborting.
//
//   reference                                   here
//   fp6_linear_kernel(stream, W, ...)           same; W = output of weight_matrix_prepacking uploaded to the device
//   fp_eXmY_linear_kernel(E, M, stream, ...)    same
//   weight_matrix_prepacking[_fp_eXmY]          same (bit-identical bytes, may be called in place)
//   DeQuantMatrix_FP6_To_FP16 / dequant_matrix_fp_eXmY_to_fp16   same (bit-identical fp16)
#ifndef FP6MI_FP6_LINEAR_H
#define FP6MI_FP6_LINEAR_H

#include <hip/hip_runtime.h>

#include "../../include/fp6mi.h"

typedef _Float16 fp6mi_half;

inline int fp_eXmY_linear_kernel(int EXPONENT, int MANTISSA, hipStream_t stream, const void *Weight, const fp6mi_half *Scales,
                                 const fp6mi_half *B, fp6mi_half *C, size_t M_Global, size_t N_Global, size_t K_Global,
                                 float *Reduction_Workspace, int Split_K)
{
    return fp6mi_linear(EXPONENT, MANTISSA, stream, Weight, Scales, B, C, M_Global, N_Global, K_Global, Reduction_Workspace, Split_K);
}

inline int fp6_linear_kernel(hipStream_t stream, const void *Weight, const fp6mi_half *Scales, const fp6mi_half *B, fp6mi_half *C,
                             size_t M_Global, size_t N_Global, size_t K_Global, float *Reduction_Workspace, int Split_K)
{
    return fp_eXmY_linear_kernel(3, 2, stream, Weight, Scales, B, C, M_Global, N_Global, K_Global, Reduction_Workspace, Split_K);
}

inline int weight_matrix_prepacking_fp_eXmY(int EXPONENT, int MANTISSA, int *packed_weights, int *FPxWeights, size_t M, size_t K)
{
    return fp6mi_prepack_ref(EXPONENT, MANTISSA, packed_weights, FPxWeights, M, K);
}

inline int weight_matrix_prepacking(int *packed_weights, int *FP6Weights, size_t M, size_t K)
{
    return weight_matrix_prepacking_fp_eXmY(3, 2, packed_weights, FP6Weights, M, K);
}

inline int dequant_matrix_fp_eXmY_to_fp16(int EXPONENT, int MANTISSA, fp6mi_half *A_16bit_h, unsigned char *A_x_bit_h, size_t M, size_t K,
                                          fp6mi_half *scale)
{
    return fp6mi_dequant(EXPONENT, MANTISSA, A_16bit_h, A_x_bit_h, M, K, scale);
}

inline int DeQuantMatrix_FP6_To_FP16(fp6mi_half *A_16bit_h, unsigned char *A_6bit_h, size_t M, size_t K, fp6mi_half *scale)
{
    return dequant_matrix_fp_eXmY_to_fp16(3, 2, A_16bit_h, A_6bit_h, M, K, scale);
}

#endif
