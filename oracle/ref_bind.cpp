// TEST INFRASTRUCTURE ONLY.  C bindings around the reference's own CPU prepacking routine, compiled from the
// reference checkout where it lies (-I$(REF)/fp6_llm/csrc); no reference source is copied.  The result
// (oracle/_ref/libref_prepack.so) validates oracle/fpx_oracle.c and writes the fixtures under tests/golden/.
//
// Only utils/weight_prepacking.h is built: utils/weight_dequant.h includes <cuda_fp16.h>, whose copy in this image
// needs <nv/target>, which the image does not have, so the reference dequantizer is unbuildable here.
#include <cstddef>
#include "utils/weight_prepacking.h"

extern "C" void ref_weight_matrix_prepacking(int *packed, int *raw, size_t M, size_t K)
{
    weight_matrix_prepacking(packed, raw, M, K); // utils/weight_prepacking.h:199-201
}
extern "C" void ref_weight_matrix_prepacking_fp_eXmY(int E, int Mbits, int *packed, int *raw, size_t M, size_t K)
{
    weight_matrix_prepacking_fp_eXmY(E, Mbits, packed, raw, M, K); // utils/weight_prepacking.h:204-211
}
