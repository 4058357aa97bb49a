/*
 * fp6mi.h -- C ABI of the MI355X (gfx950) FPx x FP16 linear-layer engine.
 *
 * Plain C: pointers, sizes and ints only.  This is the boundary a host binding (ctypes, pybind, cgo, JNI ...)
 * attaches to; the C++ header fp6_llm_amd/csrc/fp6_linear.h and the Python package fp6_llm_amd are thin layers
 * over exactly these symbols.  Citations name the interface of usyd-fsalab/fp6_llm that each entry replaces
 * (paths relative to that repository).
 *
 * Conventions (same as the reference, fp6_llm/csrc/fp6_linear.cu:149-159):
 *   M = OC (weight rows), K = IC, N = batch.  Weights are x = 1+E+M bit codes: (E,M) = (3,2) FP6_e3m2 and (2,2) FP5_e2m2,
 *   the formats the reference's entry points admit (fp6_llm/csrc/fp6_linear.cu:133-138), and through the same entry points
 *   (2,3) FP6_e2m3 and (2,1) FP4_e2m1, which the reference's templates allow (utils/weight_prepacking.h:43) but its
 *   dispatchers reject.
 *   "raw" weights     : row-major [M,K] codes, per-row MSB-first bitstream, M*K*x/8 bytes.
 *   "ref" layout      : the reference's prepacked layout (utils/weight_prepacking.h:118-196), same byte count.
 *   "native" layout   : this engine's gfx950 layout, fp6mi_native_bytes() bytes (K padded to 256).
 *   activations B     : fp16 [N,K] row-major;  output C : fp16 [N,M] row-major;  scales : fp16 [M], 2-byte aligned
 *   (a view into a larger scale tensor is fine; 8-byte alignment lets the large-batch kernel fetch four at a time).
 *
 * Return value of every int function: 0 on success, a negative FP6MI_ERR_* for rejected arguments, or a positive
 * hipError_t from the runtime.  Nothing here aborts the process.  GPU entry points enqueue on `stream`
 * (a hipStream_t passed as void*, NULL = the default stream) and do not synchronize.
 */
#ifndef FP6MI_H
#define FP6MI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FP6MI_OK 0
#define FP6MI_ERR_FORMAT (-1)    /* (E,M) is not (3,2), (2,2), (2,3), (2,1) */
#define FP6MI_ERR_SHAPE (-2)     /* M % 256, K % 64, N > 0 or size overflow */
#define FP6MI_ERR_NULL (-3)      /* a required pointer is NULL              */
#define FP6MI_ERR_WORKSPACE (-4) /* splitK > 1 without a workspace          */
#define FP6MI_ERR_SPLITK (-5)    /* splitK < 1                              */
#define FP6MI_ERR_ALIGN (-6)     /* a device pointer is not 16-byte aligned (scales, group exponents: 2-byte) */
#define FP6MI_ERR_TOO_LARGE (-7) /* the problem exceeds the static workspace of fp6mi_linear_native_static */
#define FP6MI_ERR_CAPTURE (-8)   /* the call would have to allocate while its stream is being captured */

const char *fp6mi_error_string(int code);
int         fp6mi_version(void);
/* What the measured launch-shape table of this build was measured on: entry count, and per group of entries the library
 * version and ROCm release of the measuring run.  The table answers only for 256-CU parts; elsewhere the rules decide.
 * (No counterpart in the reference, whose tile choice is a fixed bucketing of the batch, fp6_llm/csrc/fp6_linear.cu:58-99.) */
const char *fp6mi_tuning_info(void);

/* ------------------------------------------------------------------------------------------------ CPU side */

/* Replaces weight_matrix_prepacking / weight_matrix_prepacking_fp_eXmY (fp6_llm/csrc/fp6_linear.cuh:36-37,
 * utils/weight_prepacking.h:199-211): raw -> reference layout, bit-exact.  `packed` may alias `raw`.
 * Requires M % 64 == 0 and K % 64 == 0 like the reference (utils/weight_prepacking.h:121-122). */
int fp6mi_prepack_ref(int E, int Mbits, void *packed, const void *raw, size_t M, size_t K);

/* Replaces DeQuantMatrix_FP6_To_FP16 / dequant_matrix_fp_eXmY_to_fp16 (fp6_llm/csrc/fp6_linear.cuh:42-43,
 * utils/weight_dequant.h:10-61): raw -> fp16 [M,K], out = fp16_rn(value(code) * scale[row]), bit-exact. */
int fp6mi_dequant(int E, int Mbits, void *out_f16, const void *raw, size_t M, size_t K, const void *scales_f16);

/* Inverse of fp6mi_prepack_ref (no counterpart in the reference): reference layout -> raw. */
int fp6mi_unpack_ref(int E, int Mbits, void *raw, const void *packed, size_t M, size_t K);

/* Native gfx950 layout (no counterpart in the reference; the reference's layout targets 32-lane warps and
 * mma.m16n8k16 fragments, utils/weight_prepacking.h:39-85).  Requires M % 16 == 0, K % 64 == 0. */
size_t fp6mi_native_bytes(int E, int Mbits, size_t M, size_t K);
int    fp6mi_prepack_native(int E, int Mbits, void *native, const void *raw, size_t M, size_t K);
int    fp6mi_relayout_ref_to_native(int E, int Mbits, void *native, const void *packed_ref, size_t M, size_t K);
int    fp6mi_unpack_native(int E, int Mbits, void *raw, const void *native, size_t M, size_t K);

/* Split-K choice for an MI355X-class part with `num_cus` compute units (replaces the role of
 * HeuristicFuntion_SplitK, fp6_llm/__init__.py:13-23, whose model of one CTA per 512x64 outputs does not fit
 * this kernel).  Returns a value in [1, 64]. */
int fp6mi_heuristic_splitk(size_t M, size_t N, size_t K, int num_cus);
/* The same for a given weight format (the measured table is per bit width; the function above answers for FP6). */
int fp6mi_heuristic_splitk_format(int E, int Mbits, size_t M, size_t N, size_t K, int num_cus);

/* Bytes of the split-K workspace the GEMM entry points need: splitK*M*N floats (fp6_llm/csrc/fp6_linear.cuh:17),
 * 0 when splitK == 1. */
size_t fp6mi_workspace_bytes(size_t M, size_t N, int splitK);

/* ------------------------------------------------------------------------------------------------ GPU side */

/* The GEMM on native-layout weights: C[N,M] = B[N,K] . dequant(W)[M,K]^T, FP32 accumulation, fp16 output.
 * Same argument meaning as fp_eXmY_linear_kernel (fp6_llm/csrc/fp6_linear.cuh:20-32) except that W is the
 * native layout.  splitK > 1 splits K across workgroups; partial sums go to `workspace`
 * ([splitK][N][M] floats, layout of include/kernel_matmul.cuh:183) and a reduction kernel
 * (role of include/kernel_reduction.cuh:28-47) produces C.  M % 256 == 0, K % 64 == 0, N >= 1. */
int fp6mi_linear_native(int E, int Mbits, void *stream, const void *W_native, const void *scales_f16,
                        const void *B_f16, void *C_f16, size_t M, size_t N, size_t K, float *workspace, int splitK);

/* Allocation-free variant of fp6mi_linear_native.  It has no counterpart in the reference (whose callers bring the
 * workspace, fp6_llm/csrc/fp6_linear.cuh:17); it is for callers that can neither allocate nor keep a workspace: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same kernels and results as
 * fp6mi_linear_native; the split-K partial sums go to a static device array of the library,
 * fp6mi_static_workspace_bytes() bytes (32 MiB) per GPU, instead of a caller workspace.  It calls no hipMalloc/hipFree.
 * splitK * M * N floats beyond that size return FP6MI_ERR_TOO_LARGE.  All calls on one GPU share the array: calls with
 * splitK > 1 that overlap in time on one GPU (different streams) race; calls on one stream are ordered.
 * fp6mi_init() looks the array's device address up for the current device ahead of time (the first call on a device does
 * it otherwise); call it once per device outside any stream capture. */
int    fp6mi_linear_native_static(int E, int Mbits, void *stream, const void *W_native, const void *scales_f16,
                                  const void *B_f16, void *C_f16, size_t M, size_t N, size_t K, int splitK);
size_t fp6mi_static_workspace_bytes(void);
int    fp6mi_init(void);

/* Drop-in for fp_eXmY_linear_kernel / fp6_linear_kernel (fp6_llm/csrc/fp6_linear.cuh:8-32): W is the REFERENCE
 * prepacked layout on the device, exactly what a caller of the reference already holds.  On the first call with a
 * given W pointer the library allocates a native-layout twin (hipMalloc), fills it with one relayout kernel on
 * `stream` and waits for that kernel (so that the twin is complete before any other stream can be handed it); later
 * calls with the same (pointer, format, M, K) reuse it from any stream without allocating or waiting.  A first call
 * whose stream is being captured returns FP6MI_ERR_CAPTURE instead of allocating (the reference's entry point
 * allocates nothing, fp6_llm/csrc/fp6_linear.cu:104-117): make the first call, or fp6mi_relayout_ref_to_native_gpu,
 * before the capture.  The twin is keyed by ADDRESS: if the caller overwrites or frees-and-reuses the weight buffer
 * it must call fp6mi_twin_evict(W) (or fp6mi_twin_clear()) first.  The first call per weight allocates and synchronizes
 * `stream` (outside the library's lock: calls on other weights from other threads are not held up), so it must not
 * overlap another thread's stream capture in global mode.  Callers that cannot tolerate the hidden allocation convert
 * explicitly and use fp6mi_linear_native. */
int fp6mi_linear(int E, int Mbits, void *stream, const void *W_ref, const void *scales_f16, const void *B_f16,
                 void *C_f16, size_t M, size_t N, size_t K, float *workspace, int splitK);
int fp6mi_twin_evict(const void *W_ref);
int fp6mi_twin_clear(void);

/* The same drop-in with the reference's contract kept to the letter (fp6_llm/csrc/fp6_linear.cu:104-139: the entry point
 * allocates nothing and remembers nothing): W_ref is the REFERENCE layout, and the caller lends a device buffer of
 * fp6mi_native_bytes(E, Mbits, M, K) bytes into which the weights are re-laid out on `stream` by every call, right before
 * the GEMM reads them there.  No library state, safe under stream capture, any stream; the price is one more pass over the
 * weights per call (read + write, about as long again as a batch-8 GEMM), so callers that can keep the converted copy
 * should convert once (fp6mi_relayout_ref_to_native_gpu) and call fp6mi_linear_native. */
int fp6mi_linear_stateless(int E, int Mbits, void *stream, const void *W_ref, const void *scales_f16, const void *B_f16,
                           void *C_f16, size_t M, size_t N, size_t K, float *workspace, int splitK, void *native_scratch);

/* Tuning hook: the same GEMM with the launch shape chosen by the caller instead of the built-in selection
 * (no counterpart in the reference, whose TilingConfig is picked inside fpx_linear_kernel, fp6_linear.cu:61-81).
 * kind 0 = stream kernel (row_waves must be 1, k_waves in {4,8,16} wavefronts split K inside the workgroup; row_tiles = 1..8, where
 *          3, 5, 6 and 7 need not divide M/16: the last workgroup holds the tiles that are left),
 * kind 1 = tile kernel (row_waves x k_waves wavefronts, activations staged in LDS),
 * kind 2 = wave-specialized tile kernel (row_waves arithmetic wavefronts; k_waves = 4 loading wavefronts that move weights and
 *          activations into LDS for them);
 * n_tiles = 16-column batch tiles per workgroup, row_tiles = 16-row weight tiles per wavefront.
 * Combinations that are not compiled in, or that do not divide M, return FP6MI_ERR_SHAPE. */
int fp6mi_linear_native_cfg(int E, int Mbits, void *stream, const void *W_native, const void *scales_f16,
                            const void *B_f16, void *C_f16, size_t M, size_t N, size_t K, float *workspace, int splitK,
                            int kind, int n_tiles, int row_tiles, int row_waves, int k_waves);

/* The same hook for weights with group exponents (fp6mi_linear_native_grouped with the launch shape chosen by the caller). */
int fp6mi_linear_native_grouped_cfg(int E, int Mbits, void *stream, const void *W_native, const void *scales_f16,
                                    const void *group_exps_native, const void *B_f16, void *C_f16, size_t M, size_t N, size_t K,
                                    float *workspace, int splitK, int kind, int n_tiles, int row_tiles, int row_waves, int k_waves);

/* Which kernel shape fp6mi_linear_native would launch for this problem: shape[0..4] = kind, n_tiles, row_tiles,
 * row_waves, k_waves, with the meaning they have in fp6mi_linear_native_cfg.  Pure host code, no GPU needed.  The
 * choice comes from a table measured on the MI355X (python -m fp6_llm_amd.tune) where the problem is near a measured
 * one, else from a rule; it plays the part of the reference's compile-time TilingConfig dispatch
 * (fp6_llm/csrc/fp6_linear.cu:61-81). */
int fp6mi_query_launch(int E, int Mbits, size_t M, size_t N, size_t K, int splitK, int *shape);
/* Where that choice comes from on a 256-CU part: 0 = this (M, K) was measured (at this batch or the next larger measured
 * one), 1 = carried over from measured problems up to a factor 1.5 away in M and in K, 2 = the rules (no measured
 * neighbour, or a splitK the table does not hold).  Negative: FP6MI_ERR_*.  (No counterpart in the reference.) */
int fp6mi_launch_source(int E, int Mbits, size_t M, size_t N, size_t K, int splitK);

/* Device-side conversion reference layout -> native layout (both device pointers), run once per weight matrix. */
int fp6mi_relayout_ref_to_native_gpu(int E, int Mbits, void *stream, void *native_dev, const void *packed_ref_dev,
                                     size_t M, size_t K);

/* Device-side dequantisation of native-layout weights to fp16 [M,K]: the same arithmetic the GEMM applies in
 * registers, made visible.  Bit-exact to fp6mi_dequant of the corresponding raw weights. */
int fp6mi_dequant_native_gpu(int E, int Mbits, void *stream, void *out_f16_dev, const void *W_native_dev,
                             const void *scales_f16_dev, size_t M, size_t K);

/* Device-side quantizer: float weights [M,K] (dtype 0 = fp16, 1 = bf16, 2 = fp32; device pointer, row-major) to
 * per-row fp16 scales [M] (absmax / format maximum, 1.0 for an all-zero row) and native-layout FPx codes
 * (round to nearest, ties to the even code, clamped at the format maximum).  The step BEFORE the reference's path: the
 * reference only ships a truncating fp16->fp6 cast that no API calls (fp6_llm/csrc/utils/weight_quant.h:9-105,
 * "weight_prepacking_fp16_to_fp6"); this replaces quantize-on-CPU + weight_matrix_prepacking for checkpoints that are
 * already on the GPU.  M % 16 == 0 (256 for the GEMM), K % 64 == 0; native_dev holds fp6mi_native_bytes(E,M,...) bytes. */
int fp6mi_quantize_native_gpu(int E, int Mbits, void *stream, void *native_dev, void *scales_f16_dev,
                              const void *weights_dev, int dtype, size_t M, size_t K);

/* ---------------------------------------------------------------------------------- per-group scales (beyond the reference)
 * The reference scales per output row only (fp6_llm/csrc/fp6_linear.cuh:24, one half per row).  Here a weight matrix may
 * carry, besides its row scales, one exponent byte b per (row, group of 128 columns): the weights of the group count
 * value * 2^(b-127) * scale[row]  (b is the E8M0 scale type of the OCP MX formats; 127 = factor 1).  The gfx950 conversion
 * instruction applies the power of two while it converts, so a grouped GEMM runs at the speed of an ungrouped one.
 * b must keep value * 2^(b-127) inside fp16 (112 <= b <= 135 always does); the quantizer of the Python package emits
 * 112..127.  `exps` is row-major [M][ceil(K/128)] bytes; the kernels read the "native" order produced by
 * fp6mi_pack_group_exps: fp6mi_group_exps_bytes(M, K) bytes, M % 16 == 0, K % 64 == 0. */
size_t fp6mi_group_exps_bytes(size_t M, size_t K);
int    fp6mi_pack_group_exps(void *native_exps, const void *exps, size_t M, size_t K);
/* fp6mi_dequant with group exponents (host; raw weights, exps row-major). */
int fp6mi_dequant_grouped(int E, int Mbits, void *out_f16, const void *raw, size_t M, size_t K, const void *scales_f16,
                          const void *exps);
/* fp6mi_linear_native / fp6mi_dequant_native_gpu with group exponents (device pointer, native order, 2-byte aligned). */
int fp6mi_linear_native_grouped(int E, int Mbits, void *stream, const void *W_native, const void *scales_f16,
                                const void *group_exps_native, const void *B_f16, void *C_f16, size_t M, size_t N, size_t K,
                                float *workspace, int splitK);
int fp6mi_dequant_native_grouped_gpu(int E, int Mbits, void *stream, void *out_f16_dev, const void *W_native_dev,
                                     const void *scales_f16_dev, const void *group_exps_native_dev, size_t M, size_t K);
/* fp6mi_quantize_native_gpu that also chooses the group exponents: per group the smallest 2^(b-127), 112 <= b <= 127, that
 * holds the group's largest |weight| / scale[row]; codes are rounded against scale * 2^(b-127).  Writes
 * fp6mi_group_exps_bytes(M, K) bytes in native order. */
int fp6mi_quantize_native_grouped_gpu(int E, int Mbits, void *stream, void *native_dev, void *scales_f16_dev,
                                      void *group_exps_native_dev, const void *weights_dev, int dtype, size_t M, size_t K);

#ifdef __cplusplus
}
#endif
#endif /* FP6MI_H */
