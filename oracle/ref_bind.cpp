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
// The reference's prepacking template instantiated for any supported (E,M): utils/weight_prepacking.h:118-196 is generic in
// the bit width (1-, 2- and 4-bit segments as the width has them); its own dispatcher above admits e3m2 and e2m2 only.
extern "C" int ref_weight_matrix_prepacking_x_bit(int E, int Mbits, int *packed, int *raw, size_t M, size_t K)
{
    if (E == 3 && Mbits == 2) { weight_matrix_prepacking_x_bit<3, 2>(packed, raw, M, K); return 0; }
    if (E == 2 && Mbits == 2) { weight_matrix_prepacking_x_bit<2, 2>(packed, raw, M, K); return 0; }
    if (E == 2 && Mbits == 3) { weight_matrix_prepacking_x_bit<2, 3>(packed, raw, M, K); return 0; }
    if (E == 2 && Mbits == 1) { weight_matrix_prepacking_x_bit<2, 1>(packed, raw, M, K); return 0; }
    return -1;
}
