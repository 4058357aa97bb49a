// gfx950 (MI355X) kernels of the FPx x FP16 linear layer, their launchers and the C ABI.
//
// Roles taken over from the reference (usyd-fsalab/fp6_llm, paths relative to it):
//   gemm_stream   <- QUANT_GEMM_Kernel        fp6_llm/csrc/include/kernel_matmul.cuh:29-191
//   splitk_reduce <- SplitK_Reduction         fp6_llm/csrc/include/kernel_reduction.cuh:28-47
//   launchers     <- fpx_linear_kernel        fp6_llm/csrc/fp6_linear.cu:44-102
// The design is not a translation: weights use the native layout described in fp6mi_host.cpp, go from HBM straight
// to VGPRs with 128-bit non-temporal loads, FP6 codes are converted by the CDNA4 instruction
// v_cvt_scalef32_pk32_f16_bf6 (BF6 = e3m2, bias 3, no inf/nan: the very format of the reference), FP5 codes by the same
// instruction after a zero bit is slipped in above their exponent (an e2m2 code read as e3m2 is a quarter of its value),
// FP6_e2m3 codes by v_cvt_scalef32_pk32_f16_fp6 and FP4_e2m1 codes by that instruction after two zero bits are appended
// to their mantissa, and v_mfma_f32_16x16x32_f16 accumulates in FP32.  The per-row scale (and the factor 4 of FP5) is
// applied once to the FP32 sums instead of to every weight.
#include <hip/hip_runtime.h>

#include <mutex>
#include <type_traits>
#include <unordered_map>
#include <vector>

#include "fp6mi_internal.h"

namespace {

typedef _Float16 half_t;
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v32h __attribute__((ext_vector_type(32)));
typedef float    v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef uint32_t v6u __attribute__((ext_vector_type(6)));

constexpr int kWave = 64;

// Formats are named by the tag FM = 10*E + M.  `hw_e3m2` says which conversion instruction reads the 6-bit fields that the
// native layout holds (BF6 = e3m2 or FP6 = e2m3); post_scale is the factor the epilogue owes the sums.
template <int FM> struct Fmt;
template <> struct Fmt<32> { static constexpr int bits = 6, man = 2, bias = 3, block_bytes = 3072; static constexpr bool hw_e3m2 = true;
                             static constexpr float post_scale = 1.0f; static constexpr double max_value = 28.0; };
template <> struct Fmt<22> { static constexpr int bits = 5, man = 2, bias = 1, block_bytes = 2560; static constexpr bool hw_e3m2 = true;
                             static constexpr float post_scale = 4.0f; static constexpr double max_value = 7.0; };
template <> struct Fmt<23> { static constexpr int bits = 6, man = 3, bias = 1, block_bytes = 3072; static constexpr bool hw_e3m2 = false;
                             static constexpr float post_scale = 1.0f; static constexpr double max_value = 7.5; };
template <> struct Fmt<21> { static constexpr int bits = 4, man = 1, bias = 1, block_bytes = 2048; static constexpr bool hw_e3m2 = false;
                             static constexpr float post_scale = 1.0f; static constexpr double max_value = 6.0; };

// The weights of one lane for one 16x256 block, as loaded from memory.
template <int FM> struct WFrag;
template <> struct WFrag<32> { v4u a, b, c; };
template <> struct WFrag<23> { v4u a, b, c; };
template <> struct WFrag<22> { v4u a, b; v2u s; };
template <> struct WFrag<21> { v4u a, b; };

template <int FM> __device__ __forceinline__ WFrag<FM> load_wfrag(const uint8_t *block, int lane)
{
    const v4u *p = reinterpret_cast<const v4u *>(block) + lane;
    WFrag<FM>  f;
    f.a = __builtin_nontemporal_load(p);
    f.b = __builtin_nontemporal_load(p + 64);
    if constexpr (Fmt<FM>::bits == 6) f.c = __builtin_nontemporal_load(p + 128);
    if constexpr (Fmt<FM>::bits == 5) f.s = __builtin_nontemporal_load(reinterpret_cast<const v2u *>(block + 2048) + lane);
    return f;
}

// A operands (8 halfs = k 8q..8q+7 of this lane's row) of the eight MFMA steps of a block.
// FP5: a quarter of the values (exact; the epilogue multiplies the sums by 4).  The other formats: exact values.
template <int FM> struct AOps { v8h s[8]; };

__device__ __forceinline__ v8h slice8(const v32h &v, int i)
{
    switch (i) {
    case 0: return __builtin_shufflevector(v, v, 0, 1, 2, 3, 4, 5, 6, 7);
    case 1: return __builtin_shufflevector(v, v, 8, 9, 10, 11, 12, 13, 14, 15);
    case 2: return __builtin_shufflevector(v, v, 16, 17, 18, 19, 20, 21, 22, 23);
    default: return __builtin_shufflevector(v, v, 24, 25, 26, 27, 28, 29, 30, 31);
    }
}

// FP5: 32 codes are stored in five dwords; the sixth dword of the 6-bit string the conversion instruction reads is parked
// in the fixed-zero bits ("holes", bit 4 of every 6-bit field) of the other five and is put back here (layout: fp6mi_host.cpp).
__device__ __forceinline__ v6u fp5_expand(uint32_t s0, uint32_t s1, uint32_t s2, uint32_t s3, uint32_t s4)
{
    constexpr uint32_t A = 0x10410410u, B = 0x04104104u, C = 0x41041041u;
    uint32_t lo = (s0 & A) | (s1 & B), hi = (s2 & C) | (s3 & A) | (s4 & B);
    return (v6u){ s0 & ~A, s1 & ~B, s2 & ~C, s3 & ~A, s4 & ~B, (hi << 1) | lo };
}

// FP4: 32 codes are stored in four dwords; the fifth and sixth dword of the 6-bit string sit in the fixed-zero bit pairs (the
// two bits appended below every mantissa) of the other four, at their own bit positions (layout: fp6mi_host.cpp).
__device__ __forceinline__ v6u fp4_expand(v4u s)
{
    constexpr uint32_t P = 0xC30C30C3u, Q = 0x30C30C30u, R = 0x0C30C30Cu;
    return (v6u){ s[0] & ~P, s[1] & ~Q, s[2] & ~R, s[3] & ~P, (s[0] & P) | (s[2] & R), (s[1] & Q) | (s[3] & P) };
}

// The 192-bit string of 6-bit fields of MFMA steps 4h..4h+3 (half of a K block) of one lane, and its conversion.
template <int FM> __device__ __forceinline__ v6u field_string(const WFrag<FM> &f, int h)
{
    if constexpr (Fmt<FM>::bits == 6)
        return h == 0 ? (v6u){ f.a[0], f.a[1], f.a[2], f.a[3], f.b[0], f.b[1] } : (v6u){ f.b[2], f.b[3], f.c[0], f.c[1], f.c[2], f.c[3] };
    else if constexpr (Fmt<FM>::bits == 5)
        return h == 0 ? fp5_expand(f.a[0], f.a[1], f.a[2], f.a[3], f.s[0]) : fp5_expand(f.b[0], f.b[1], f.b[2], f.b[3], f.s[1]);
    else
        return fp4_expand(h == 0 ? f.a : f.b);
}

template <int FM> __device__ __forceinline__ v32h fields_to_halfs(v6u src)
{
    if constexpr (Fmt<FM>::hw_e3m2)
        return __builtin_amdgcn_cvt_scalef32_pk32_f16_bf6(src, 1.0f);
    else
        return __builtin_amdgcn_cvt_scalef32_pk32_f16_fp6(src, 1.0f);
}

template <int FM> __device__ __forceinline__ void convert(const WFrag<FM> &f, AOps<FM> &o)
{
    v32h h0 = fields_to_halfs<FM>(field_string<FM>(f, 0));
    v32h h1 = fields_to_halfs<FM>(field_string<FM>(f, 1));
#pragma unroll
    for (int i = 0; i < 4; i++) {
        o.s[i]     = slice8(h0, i);
        o.s[4 + i] = slice8(h1, i);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// gemm_stream: weight-bandwidth-bound GEMM for small batches.
//   grid  = (M/(16*RT) row groups, splitK, ceil(N / (16*NT)))      block = WAVES wavefronts
// A workgroup owns 16*RT output rows and 16*NT batch columns over the K blocks of its split; its wavefronts take the
// blocks round-robin (K is split inside the workgroup), each streaming its weights HBM -> VGPR and its slice of the
// activations L2 -> VGPR directly in MFMA B-operand order (reused for the RT row tiles); the partial accumulators are
// summed through LDS.
// ---------------------------------------------------------------------------------------------------------------
// Batches of at most 8 leave MFMA B columns 8..15 unused, and with them the lanes that would load those columns.  Those
// lanes fetch the operand of the FOLLOWING MFMA step instead: lane (col, q) reads batch row col % 8 at step offset col / 8,
// so one instruction brings two steps and touches whole 128-byte lines; a DPP rotation of each 16-lane row by 8 then moves
// the second step's data down to columns 0..7.  Columns 8..15 end up holding the other step's (real, finite) data and only
// feed output columns that are never stored.  (Four or eight steps per load for batches <= 4 or <= 2 measured no faster.)
template <int NT> __device__ __forceinline__ void load_x_paired(v8h (&x)[8][NT], const half_t *src)
{
#pragma unroll
    for (int sl = 0; sl < 4; sl++) {
        v4u v = *reinterpret_cast<const v4u *>(src + 64 * sl), w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v[i], 0x128, 0xf, 0xf, false); // row_ror:8
        x[2 * sl][0]     = __builtin_bit_cast(v8h, v);
        x[2 * sl + 1][0] = __builtin_bit_cast(v8h, w);
    }
}

template <int FM, int NT, int RT> struct Stage {
    WFrag<FM> w[RT];
    v8h       x[8][NT];
};

template <int FM, int NT, int RT>
__device__ __forceinline__ void load_stage(Stage<FM, NT, RT> &st, const uint8_t *wgroup, size_t tile_stride, uint32_t u, int lane,
                                           const half_t *const (&xrow)[NT], int q, uint32_t K, bool xpack, const half_t *xrow_packed)
{
#pragma unroll
    for (int r = 0; r < RT; r++) st.w[r] = load_wfrag<FM>(wgroup + r * tile_stride + (size_t)u * Fmt<FM>::block_bytes, lane);
    // Every lane loads, without branches.  Batch columns beyond N read the last real row: an MFMA output column depends only
    // on its own B column, and those columns are never stored.  K positions beyond K (only in the last block when K is not
    // a multiple of 256) read position 0 of the row: the native layout holds zero weights there.
    if (NT == 1 && xpack && (u + 1) * 256 <= K) { // uniform
        load_x_paired(st.x, xrow_packed + u * 256);
    } else
    if ((u + 1) * 256 <= K) { // uniform: whole block inside K, one base address and immediate offsets
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int t = 0; t < NT; t++) st.x[s][t] = *reinterpret_cast<const v8h *>(xrow[t] + u * 256 + 32 * s);
    } else {
#pragma unroll
        for (int s = 0; s < 8; s++) {
            uint32_t k = u * 256 + 32 * s;
            if (k + 8 * q >= K) k = 0;
#pragma unroll
            for (int t = 0; t < NT; t++) st.x[s][t] = *reinterpret_cast<const v8h *>(xrow[t] + k);
        }
    }
    __builtin_amdgcn_sched_barrier(0); // keep every load of the block issued before the first conversion waits
}

template <int FM, int NT, int RT>
__device__ __forceinline__ void consume_stage(const Stage<FM, NT, RT> &st, v4f (&acc)[RT][NT])
{
#pragma unroll
    for (int r = 0; r < RT; r++) {
        AOps<FM> a;
        convert(st.w[r], a);
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int t = 0; t < NT; t++) acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.s[s], st.x[s][t], acc[r][t], 0, 0, 0);
    }
}

template <int FM, int NT, int RT, int WAVES>
__global__ __launch_bounds__(WAVES *kWave) void gemm_stream(const uint8_t *__restrict__ W, const half_t *__restrict__ scales,
                                                            const half_t *__restrict__ X, half_t *__restrict__ C,
                                                            float *__restrict__ ws, uint32_t M, uint32_t N, uint32_t K,
                                                            uint32_t units, uint32_t splitK)
{
    __shared__ float red[WAVES][RT * NT][256];

    const int      lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int      col = lane & 15, q = lane >> 4;
    const uint32_t R0 = blockIdx.x * RT, split = blockIdx.y, nbase = blockIdx.z * (16 * NT);

    const uint32_t avg = units / splitK, extra = units % splitK;
    const uint32_t u0 = split * avg + (split < extra ? split : extra);
    const uint32_t u1 = u0 + avg + (split < extra ? 1u : 0u);

    const size_t   tile_stride = (size_t)units * Fmt<FM>::block_bytes;
    const uint8_t *wgroup = W + (size_t)R0 * tile_stride;

    v4f acc[RT][NT];
#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int t = 0; t < NT; t++) acc[r][t] = (v4f){ 0.f, 0.f, 0.f, 0.f };

    const half_t *xrow[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        uint32_t n = nbase + 16 * t + col;
        xrow[t]    = X + (size_t)(n < N ? n : N - 1) * K + 8 * q;
    }
    // batches up to 8: two MFMA steps per activation load (see load_x_paired)
    const bool    xpack = NT == 1 && N <= 8;
    const int     prow = col & 7, pstep = col >> 3;
    const half_t *xrow_packed = X + (size_t)((uint32_t)prow < N ? prow : N - 1) * K + 8 * q + 32 * pstep;

    // The epilogue gives thread e the output (row tile e/(256*NT), column tile, batch column, row e%16); its row scale is
    // fetched now so that no global load sits on the tail of the kernel.
    constexpr int kOutPerThread = (RT * NT * 256 + WAVES * kWave - 1) / (WAVES * kWave);
    half_t        my_scale[kOutPerThread]; // kept as loaded: converting here would wait for the load before the weight loads issue
#pragma unroll
    for (int j = 0; j < kOutPerThread; j++) {
        int e = threadIdx.x + j * WAVES * kWave;
        my_scale[j] = scales[(R0 + (e < RT * NT * 256 ? (e >> 8) / NT : 0)) * 16 + (e & 15)];
    }

    // workgroups that share an L2 (ids congruent mod 8) start on different K blocks, so that the chip does not ask
    // the same activation lines of the same L2 channel at the same moment
    // One K block at a time and no register double-buffering: the other wavefronts of the workgroup keep the memory system
    // busy while this one converts, and a second stage in registers measured slower at every size.
    for (uint32_t u = u0 + ((wave + (blockIdx.x >> 3)) % WAVES); u < u1; u += WAVES) {
        Stage<FM, NT, RT> cur;
        load_stage<FM, NT, RT>(cur, wgroup, tile_stride, u, lane, xrow, q, K, xpack, xrow_packed);
        consume_stage<FM, NT, RT>(cur, acc);
    }

    // acc[r][t][i] = sum for output row 16r + 4q+i, batch column 16t+col
#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int t = 0; t < NT; t++) *reinterpret_cast<v4f *>(&red[wave][r * NT + t][lane * 4]) = acc[r][t];
    __syncthreads();

#pragma unroll
    for (int j = 0; j < kOutPerThread; j++) {
        const int e = threadIdx.x + j * WAVES * kWave;
        if (e >= RT * NT * 256) break;
        int   rt = e >> 8, i8 = e & 255, n = i8 >> 4, mm = i8 & 15;
        int   r = rt / NT, t = rt % NT;
        int   idx = (((mm >> 2) * 16 + n) << 2) | (mm & 3);
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) sum += red[w][rt][idx];
        uint32_t ng = nbase + 16 * t + n, mg = (R0 + r) * 16 + mm;
        if (ng < N) {
            float v = sum * ((float)my_scale[j] * Fmt<FM>::post_scale);
            if (splitK == 1)
                C[(size_t)ng * M + mg] = (half_t)v;
            else
                ws[((size_t)split * N + ng) * M + mg] = v;
        }
    }
}

// A operands of MFMA steps 4h..4h+3 (half of a K block) of one lane.
template <int FM> __device__ __forceinline__ void convert_half(const WFrag<FM> &f, int h, v8h (&o)[4])
{
    v32h v = fields_to_halfs<FM>(field_string<FM>(f, h));
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = slice8(v, i);
}

// ---------------------------------------------------------------------------------------------------------------
// gemm_tile: GEMM for batches above 16, where every weight must meet many activation columns.
//   workgroup = WR x WK wavefronts; tile = (WR*RT*16) rows x (NT*16) columns
//   grid.x enumerates (row block, column block, split) with column blocks of one row block adjacent on one XCD
// The K blocks of a split are walked in chunks of WK blocks.  Per chunk the workgroup stages the activation chunk
// [WK][NT*16][256] in LDS (double-buffered, filled by fully coalesced 16-byte loads); wavefront (wr, wk) streams the
// weights of its RT row tiles for K block wk straight from HBM into VGPRs (prefetched one chunk ahead), converts them
// half a block at a time and runs RT*NT MFMAs per step against B operands read once per step from LDS.  The LDS row
// stride is 256+16 halfs (544 bytes): measured on the MI355X, the 16-column x 4-k-group operand read (ds_read_b128) then runs at
// the conflict-free rate of 7 cycles per wavefront, against 8.8 cycles at 528 bytes and 32 cycles without padding.
// The WK partial accumulators are summed through LDS at the end (WK > 1), then scaled and stored.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kXsRowBytes = 544;

template <int FM, int NT, int RT, int WR, int WK>
__global__ __launch_bounds__(WR *WK *kWave) void gemm_tile(const uint8_t *__restrict__ W, const half_t *__restrict__ scales,
                                                           const half_t *__restrict__ X, half_t *__restrict__ C,
                                                           float *__restrict__ ws, uint32_t M, uint32_t N, uint32_t K,
                                                           uint32_t units, uint32_t splitK, uint32_t nblocks)
{
    constexpr int  TN = NT * 16, NTHREADS = WR * WK * kWave;
    constexpr int  kBufBytes = WK * TN * kXsRowBytes;
    constexpr int  kPieces = WK * TN * 32, kPerThread = (kPieces + NTHREADS - 1) / NTHREADS;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wr = wave % WR, wk = wave / WR;
    const int col = lane & 15, q = lane >> 4;

    // grid.x -> (row block, column block, split): ids that are congruent mod 8 run on one XCD and share its L2, so
    // the column blocks of a row block (which read the same weights) are given such ids
    uint32_t id = blockIdx.x;
    if ((gridDim.x & 7u) == 0) id = (id & 7u) * (gridDim.x >> 3) + (id >> 3);
    const uint32_t nb = id % nblocks, rest = id / nblocks, split = rest % splitK, mb = rest / splitK;
    const uint32_t nbase = nb * TN, R0 = (mb * WR + wr) * RT; // first row tile of this wavefront

    const uint32_t avg = units / splitK, extra = units % splitK;
    const uint32_t u0 = split * avg + (split < extra ? split : extra);
    const uint32_t u1 = u0 + avg + (split < extra ? 1u : 0u);

    const size_t   tile_stride = (size_t)units * Fmt<FM>::block_bytes;
    const uint8_t *wgroup = W + (size_t)R0 * tile_stride;

    v4f acc[RT][NT];
#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int t = 0; t < NT; t++) acc[r][t] = (v4f){ 0.f, 0.f, 0.f, 0.f };

    WFrag<FM> wcur[RT], wnxt[RT];
    v4u       xr[kPerThread];

    // row scales of this lane's outputs (rows 4q..4q+3 of each of its row tiles), fetched before the main loop so that no
    // global load sits on the tail of the kernel
    typedef _Float16 v4h __attribute__((ext_vector_type(4)));
    v4h sc4[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) sc4[r] = *reinterpret_cast<const v4h *>(scales + (R0 + r) * 16 + 4 * q);

    auto load_w = [&](WFrag<FM>(&dst)[RT], uint32_t c0) {
        const uint32_t u = c0 + wk;
        if (u < u1) {
#pragma unroll
            for (int r = 0; r < RT; r++) dst[r] = load_wfrag<FM>(wgroup + r * tile_stride + (size_t)u * Fmt<FM>::block_bytes, lane);
        }
    };
    // Per-thread pieces of the activation chunk: piece p = tid + NTHREADS*j is 16 bytes, (K block p / (TN*32) of the chunk,
    // batch column (p/32) % TN, halfs 8*(p%32)..+7).  Row pointers and LDS offsets are fixed for the whole kernel.
    // There is no zero fill: columns beyond N read the last real row (their outputs are never stored); positions beyond K or
    // beyond the split read position 0 of the row (zero weights there, or a wavefront that does not compute).
    const half_t *xrow[kPerThread];
    uint32_t      xlds[kPerThread];
#pragma unroll
    for (int j = 0; j < kPerThread; j++) {
        const uint32_t p = tid + NTHREADS * j, n = nbase + (p >> 5) % TN;
        xrow[j] = X + (size_t)(n < N ? n : N - 1) * K + (p & 31) * 8 + (size_t)(p / (TN * 32)) * 256;
        xlds[j] = (p >> 5) * kXsRowBytes + (p & 31) * 16;
    }
    auto load_x = [&](uint32_t c0) {
        if ((c0 + WK) * 256 <= K && c0 + WK <= u1) { // uniform: the whole chunk lies inside K and inside the split
#pragma unroll
            for (int j = 0; j < kPerThread; j++)
                if (kPieces % NTHREADS == 0 || tid + NTHREADS * j < kPieces) xr[j] = *reinterpret_cast<const v4u *>(xrow[j] + (size_t)c0 * 256);
        } else {
#pragma unroll
            for (int j = 0; j < kPerThread; j++) {
                const uint32_t p = tid + NTHREADS * j;
                if (kPieces % NTHREADS == 0 || p < (uint32_t)kPieces) {
                    const uint32_t u = c0 + p / (TN * 32), k = u * 256 + (p & 31) * 8;
                    const bool     ok = k < K && u < u1;
                    xr[j] = *reinterpret_cast<const v4u *>(ok ? xrow[j] + (size_t)c0 * 256 : xrow[j] - ((p & 31) * 8 + (size_t)(p / (TN * 32)) * 256));
                }
            }
        }
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int j = 0; j < kPerThread; j++)
            if (kPieces % NTHREADS == 0 || tid + NTHREADS * j < kPieces) *reinterpret_cast<v4u *>(lds + buf * kBufBytes + xlds[j]) = xr[j];
    };

    if (u0 < u1) {
        load_x(u0);
        load_w(wcur, u0);
        store_x(0);
        __syncthreads();
        int buf = 0;
        for (uint32_t c0 = u0; c0 < u1; c0 += WK, buf ^= 1) {
            const bool more = c0 + WK < u1;
            if (more) {
                load_x(c0 + WK);
                load_w(wnxt, c0 + WK);
            }
            if (c0 + wk < u1) {
                const uint8_t *xs = lds + buf * kBufBytes + (wk * TN + col) * kXsRowBytes + q * 16;
                v8h            a0[RT][4], a1[RT][4];
#pragma unroll
                for (int r = 0; r < RT; r++) convert_half(wcur[r], 0, a0[r]);
                // second half converted ahead of the first half's MFMAs: the VALU work then runs under the matrix pipe
#pragma unroll
                for (int r = 0; r < RT; r++) convert_half(wcur[r], 1, a1[r]);
#pragma unroll
                for (int h = 0; h < 2; h++) {
#pragma unroll
                    for (int s = 0; s < 4; s++) {
                        v8h b[NT];
#pragma unroll
                        for (int t = 0; t < NT; t++) b[t] = *reinterpret_cast<const v8h *>(xs + t * 16 * kXsRowBytes + (4 * h + s) * 64);
#pragma unroll
                        for (int r = 0; r < RT; r++)
#pragma unroll
                            for (int t = 0; t < NT; t++)
                                acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(h == 0 ? a0[r][s] : a1[r][s], b[t], acc[r][t], 0, 0, 0);
                    }
                }
            }
            if (more) {
                store_x(buf ^ 1); // that buffer was last read before the barrier that ended the previous iteration
#pragma unroll
                for (int r = 0; r < RT; r++) wcur[r] = wnxt[r];
            }
            __syncthreads();
        }
    }

    // acc[r][t][i]: output row (R0+r)*16 + 4q+i, batch column nbase + 16t + col
    if (WK > 1) {
        float *red = reinterpret_cast<float *>(lds); // [WK][WR][RT*NT][256]; the last barrier above freed the buffers
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int t = 0; t < NT; t++) *reinterpret_cast<v4f *>(&red[(((wk * WR + wr) * RT + r) * NT + t) * 256 + lane * 4]) = acc[r][t];
        __syncthreads();
        if (wk == 0) {
#pragma unroll
            for (int r = 0; r < RT; r++)
#pragma unroll
                for (int t = 0; t < NT; t++)
#pragma unroll
                    for (int k2 = 1; k2 < WK; k2++)
                        acc[r][t] += *reinterpret_cast<const v4f *>(&red[(((k2 * WR + wr) * RT + r) * NT + t) * 256 + lane * 4]);
        }
    }
    if (wk == 0) {
#pragma unroll
        for (int r = 0; r < RT; r++) {
            const uint32_t mg = (R0 + r) * 16 + 4 * q;
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const uint32_t ng = nbase + 16 * t + col;
                if (ng < N) {
                    v4f v;
#pragma unroll
                    for (int i = 0; i < 4; i++) v[i] = acc[r][t][i] * ((float)sc4[r][i] * Fmt<FM>::post_scale);
                    if (splitK == 1) {
                        v4h o = { (half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3] };
                        *reinterpret_cast<v4h *>(C + (size_t)ng * M + mg) = o;
                    } else {
                        *reinterpret_cast<v4f *>(ws + ((size_t)split * N + ng) * M + mg) = v;
                    }
                }
            }
        }
    }
}

// C[i] = fp16_rn(sum over splits, in split order, of ws[s][i]); four outputs per thread.
__global__ __launch_bounds__(256) void splitk_reduce(half_t *__restrict__ C, const float *__restrict__ ws, size_t MN, int splitK)
{
    size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= MN) return;
    v4f sum = { 0.f, 0.f, 0.f, 0.f };
    for (int s = 0; s < splitK; s++) sum += *reinterpret_cast<const v4f *>(ws + (size_t)s * MN + i);
    typedef _Float16 v4h __attribute__((ext_vector_type(4)));
    v4h o = { (half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3] };
    *reinterpret_cast<v4h *>(C + i) = o;
}

// Native layout -> fp16 [M,K], with the GEMM's own conversion code.  One lane per (row tile, K block, lane) triple.
template <int FM>
__global__ __launch_bounds__(256) void dequant_native(half_t *__restrict__ out, const uint8_t *__restrict__ W,
                                                     const half_t *__restrict__ scales, uint32_t M, uint32_t K, uint32_t units)
{
    const int      lane = threadIdx.x & 63;
    const uint32_t blk = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= (M / 16) * units) return;
    const uint32_t R = blk / units, U = blk % units;
    const int      m = lane & 15, q = lane >> 4;
    WFrag<FM>      wf = load_wfrag<FM>(W + (size_t)blk * Fmt<FM>::block_bytes, lane);
    AOps<FM>       a;
    convert(wf, a);
    const half_t sc = scales[R * 16 + m], post = (half_t)Fmt<FM>::post_scale;
#pragma unroll
    for (int s = 0; s < 8; s++) {
        uint32_t k = U * 256 + 32 * s + 8 * q;
        if (k < K) {
            v8h v = a.s[s];
            if (Fmt<FM>::post_scale != 1.0f) v = v * post; // exact: a power of two, results are at most 7
            v = v * sc;                // one round-to-nearest-even, like fp16_rn(value * scale)
            *reinterpret_cast<v8h *>(out + (size_t)(R * 16 + m) * K + k) = v;
        }
    }
}

// Writes the 64 codes of one lane (c[8*s + j] = code of its row at column 32*s + 8*q + j of the K block) as the lane's
// 12 (6-bit formats), 10 (FP5) or 8 (FP4) dwords of a native block.
template <int FM> __device__ __forceinline__ void store_native_lane(const uint8_t (&c)[64], uint8_t *dst, int lane)
{
    if (Fmt<FM>::bits == 6) {
        uint32_t d[12];
        for (int h = 0; h < 2; h++) {
            uint64_t accb = 0;
            int      nb = 0, w = 0;
            for (int i = 0; i < 32; i++) {
                accb |= (uint64_t)c[32 * h + i] << nb;
                nb += 6;
                if (nb >= 32) { d[6 * h + w++] = (uint32_t)accb; accb >>= 32; nb -= 32; }
            }
        }
        for (int i = 0; i < 3; i++) {
            v4u v = { d[4 * i], d[4 * i + 1], d[4 * i + 2], d[4 * i + 3] };
            reinterpret_cast<v4u *>(dst)[i * 64 + lane] = v;
        }
    } else if (Fmt<FM>::bits == 4) {
        constexpr uint32_t P = 0xC30C30C3u, Q = 0x30C30C30u, R = 0x0C30C30Cu;
        for (int h = 0; h < 2; h++) {
            uint32_t D[6];
            uint64_t accb = 0;
            int      nb = 0, w = 0;
            for (int i = 0; i < 32; i++) {
                accb |= (uint64_t)((c[32 * h + i] & 15u) << 2) << nb;
                nb += 6;
                if (nb >= 32) { D[w++] = (uint32_t)accb; accb >>= 32; nb -= 32; }
            }
            v4u v = { D[0] | (D[4] & P), D[1] | (D[5] & Q), D[2] | (D[4] & R), D[3] | (D[5] & P) };
            reinterpret_cast<v4u *>(dst)[h * 64 + lane] = v;
        }
    } else {
        constexpr uint32_t A = 0x10410410u, B = 0x04104104u, C = 0x41041041u;
        uint32_t           S[2][5];
        for (int h = 0; h < 2; h++) {
            uint32_t D[6];
            uint64_t accb = 0;
            int      nb = 0, w = 0;
            for (int i = 0; i < 32; i++) {
                uint32_t code = c[32 * h + i], field = (code & 15u) | (((code >> 4) & 1u) << 5);
                accb |= (uint64_t)field << nb;
                nb += 6;
                if (nb >= 32) { D[w++] = (uint32_t)accb; accb >>= 32; nb -= 32; }
            }
            S[h][0] = D[0] | (D[5] & A);
            S[h][1] = D[1] | (D[5] & B);
            S[h][2] = D[2] | ((D[5] >> 1) & C);
            S[h][3] = D[3] | ((D[5] >> 1) & A);
            S[h][4] = D[4] | ((D[5] >> 1) & B);
        }
        for (int h = 0; h < 2; h++) {
            v4u v = { S[h][0], S[h][1], S[h][2], S[h][3] };
            reinterpret_cast<v4u *>(dst)[h * 64 + lane] = v;
        }
        v2u sv = { S[0][4], S[1][4] };
        reinterpret_cast<v2u *>(dst + 2048)[lane] = sv;
    }
}

// Reference layout -> native layout on the device.  One thread per (row tile, K block, lane): it gathers its 64
// codes bit piece by bit piece from the reference's segment arrays and writes its 8, 10 or 12 native dwords.
__constant__ uint8_t kInvOrder4[8]  = { 4, 0, 6, 2, 5, 1, 7, 3 };
__constant__ uint8_t kInvOrder2[16] = { 8, 0, 12, 4, 9, 1, 13, 5, 10, 2, 14, 6, 11, 3, 15, 7 };

template <int FM>
__global__ __launch_bounds__(256) void relayout_ref_to_native(uint8_t *__restrict__ native, const uint8_t *__restrict__ ref,
                                                             uint32_t M, uint32_t K, uint32_t units)
{
    const int      lane = threadIdx.x & 63;
    const uint32_t blk = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= (M / 16) * units) return;
    const uint32_t R = blk / units, U = blk % units;
    const int      m = lane & 15, q = lane >> 4;
    const uint32_t row = R * 16 + m, tile = row >> 6, block = (row >> 4) & 3, rin = row & 15, g = rin & 7, rowhalf = rin >> 3;
    // segment arrays: 6 bits = [2-bit | 4-bit], 5 bits = [1-bit | 4-bit], 4 bits = [4-bit]
    constexpr int   bits = Fmt<FM>::bits;
    const uint32_t *seg_hi = reinterpret_cast<const uint32_t *>(ref);
    const uint32_t *seg4   = reinterpret_cast<const uint32_t *>(ref + (size_t)M * K * (bits - 4) / 8);
    uint8_t         c[64];
#pragma unroll 1
    for (int s = 0; s < 8; s++) {
        uint32_t k0 = U * 256 + 32 * s + 8 * q;
        for (int j = 0; j < 8; j++) {
            uint32_t col = k0 + j, code = 0;
            if (col < K) {
                uint32_t slice = col >> 4, cc = col & 15, t = (cc & 7) >> 1;
                uint32_t el = (cc & 1) | (rowhalf << 1) | ((cc >> 3) << 2);
                uint32_t l32 = 4 * g + t;
                { // 4-bit piece: q4 = block, pre = el
                    uint32_t word = seg4[((size_t)(tile * (K / 16) + slice) * 4 + block) * 32 + l32];
                    code |= (word >> (28 - 4 * kInvOrder4[el])) & 15u;
                }
                if (bits == 6) { // 2-bit piece: q2 = block/2, pre = (block%2)*8 + el
                    uint32_t word = seg_hi[((size_t)(tile * (K / 16) + slice) * 2 + (block >> 1)) * 32 + l32];
                    code |= ((word >> (30 - 2 * kInvOrder2[(block & 1) * 8 + el])) & 3u) << 4;
                } else if (bits == 5) { // 1-bit piece: q1 = 0, pre = block*8 + el; order_1 maps p -> pre, inverted arithmetically:
                    // order_1[p]-1 = 4*(p%8) + {1,3,0,2}[p/8]  =>  p = 8*{2,0,3,1}[pre%4] + pre/4
                    uint32_t pre = block * 8 + el;
                    uint32_t p   = 8 * ((0x1302u >> (4 * (pre & 3))) & 3u) + (pre >> 2);
                    uint32_t word = seg_hi[((size_t)(tile * (K / 16) + slice)) * 32 + l32];
                    code |= ((word >> (31 - p)) & 1u) << 4;
                }
            }
            c[8 * s + j] = (uint8_t)code;
        }
    }
    store_native_lane<FM>(c, native + (size_t)blk * Fmt<FM>::block_bytes, lane);
}

// ---------------------------------------------------------------------------------------------------------------
// Quantizer on the device: float weights [M,K] (fp16, bf16 or fp32) -> per-row fp16 scales + native-layout FPx codes.
// Same arithmetic as the host quantizer of this package, so that both give identical bits:
//   scale[row] = fp16_rn(absmax(row) / max_value) (1.0 where that rounds to zero), computed from a double quotient;
//   code       = nearest representable magnitude to |w / scale| (a double quotient, clamped at max_value), ties to the even
//                code, with the sign bit of w.
// (The reference's only quantizer truncates and is not wired to any API: fp6_llm/csrc/utils/weight_quant.h:9-105.)
// ---------------------------------------------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ float to_float(T v);
template <> __device__ __forceinline__ float to_float<half_t>(half_t v) { return (float)v; }
template <> __device__ __forceinline__ float to_float<float>(float v) { return v; }
struct bf16_t { uint16_t bits; };
template <> __device__ __forceinline__ float to_float<bf16_t>(bf16_t v) { return __builtin_bit_cast(float, (uint32_t)v.bits << 16); }

// round-to-nearest-even of a non-negative double to fp16 without passing through float (no double rounding)
__device__ __forceinline__ half_t half_rn_from_double(double q)
{
    if (!(q > 0.0)) return (half_t)0.0f;
    int e = ilogb(q);                               // q = 1.xxx * 2^e
    int ulp_exp = (e < -14 ? -14 : e) - 10;          // fp16 spacing at q (subnormals share the spacing 2^-24)
    double r = rint(scalbn(q, -ulp_exp));            // exact scaling, then round to nearest even integer
    double v = scalbn(r, ulp_exp);                   // representable in fp16 unless it overflows
    return v >= 65520.0 ? (half_t)__builtin_inff() : (half_t)(float)v;
}

template <typename T>
__global__ __launch_bounds__(256) void quant_row_scales(half_t *__restrict__ scales, const T *__restrict__ Wf, uint32_t M, uint32_t K,
                                                       double max_value)
{
    const int      lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    const T *p = Wf + (size_t)row * K;
    float    amax = 0.f;
    for (uint32_t k = lane * 8; k < K; k += 512)
#pragma unroll
        for (int j = 0; j < 8; j++) amax = fmaxf(amax, fabsf(to_float<T>(p[k + j])));
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if (lane == 0) {
        half_t sc = half_rn_from_double((double)amax / max_value);
        scales[row] = (float)sc == 0.f ? (half_t)1.0f : sc;
    }
}

// index (= magnitude bits of the code) of the representable magnitude nearest to a, 0 <= a <= max_value
template <int FM> __device__ __forceinline__ uint32_t nearest_magnitude(double a)
{
    constexpr int bias = Fmt<FM>::bias, MB = Fmt<FM>::man;
    int           e = a > 0.0 ? ilogb(a) : -1000;
    if (e < 1 - bias) e = 1 - bias;                        // subnormals use the spacing of the first binade
    double   t = scalbn(a, MB - e);                        // in units of the spacing 2^(e-MB): [0,2^MB) subnormal, [2^MB,2^(MB+1)) normal
    double   fl = floor(t), frac = t - fl;
    uint32_t lo = (uint32_t)fl + ((uint32_t)(e + bias - 1) << MB);
    // (normal: index = (e+bias)*2^MB + (fl-2^MB); subnormal: e = 1-bias, so index = fl)
    if (frac > 0.5 || (frac == 0.5 && (lo & 1u))) lo += 1;
    return lo;
}

template <int FM, typename T>
__global__ __launch_bounds__(256) void quant_to_native(uint8_t *__restrict__ native, const half_t *__restrict__ scales,
                                                      const T *__restrict__ Wf, uint32_t M, uint32_t K, uint32_t units, double max_value)
{
    const int      lane = threadIdx.x & 63;
    const uint32_t blk = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= (M / 16) * units) return;
    const uint32_t R = blk / units, U = blk % units;
    const int      m = lane & 15, q = lane >> 4;
    const uint32_t row = R * 16 + m;
    const double   sc = (double)(float)scales[row];
    const T       *p = Wf + (size_t)row * K;
    uint8_t        c[64];
#pragma unroll 1
    for (int s = 0; s < 8; s++) {
        const uint32_t k0 = U * 256 + 32 * s + 8 * q;
        for (int j = 0; j < 8; j++) {
            uint32_t code = 0;
            if (k0 + j < K) {
                float  w = to_float<T>(p[k0 + j]);
                double a = fabs((double)w / sc);
                if (!(a <= max_value)) a = max_value; // clamps, and sends NaN to the maximum like a saturating cast
                code = nearest_magnitude<FM>(a) | ((__builtin_bit_cast(uint32_t, w) >> 31) << (Fmt<FM>::bits - 1));
            }
            c[8 * s + j] = (uint8_t)code;
        }
    }
    store_native_lane<FM>(c, native + (size_t)blk * Fmt<FM>::block_bytes, lane);
}

// ------------------------------------------------------------------------------------------------ launch helpers

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Calls fn with the format tag of a supported (E, M) as an integral constant.
template <class Fn> inline int with_format(int E, int Mb, Fn &&fn)
{
    if (E == 3) return fn(std::integral_constant<int, 32>{});
    if (Mb == 2) return fn(std::integral_constant<int, 22>{});
    if (Mb == 3) return fn(std::integral_constant<int, 23>{});
    return fn(std::integral_constant<int, 21>{});
}

template <int FM, int NT, int RT, int WAVES>
int launch_stream(hipStream_t st, const void *W, const void *sc, const void *B, void *C, float *ws, size_t M, size_t N, size_t K,
                  int splitK)
{
    uint32_t units = (uint32_t)((K + 255) / 256);
    dim3     grid((uint32_t)(M / (16 * RT)), (uint32_t)splitK, (uint32_t)((N + 16 * NT - 1) / (16 * NT)));
    hipLaunchKernelGGL((gemm_stream<FM, NT, RT, WAVES>), grid, dim3(WAVES * kWave), 0, st, static_cast<const uint8_t *>(W),
                       static_cast<const half_t *>(sc), static_cast<const half_t *>(B), static_cast<half_t *>(C), ws, (uint32_t)M,
                       (uint32_t)N, (uint32_t)K, units, (uint32_t)splitK);
    return (int)hipGetLastError();
}

template <int FM, int NT, int RT, int WR, int WK>
int launch_tile(hipStream_t st, const void *W, const void *sc, const void *B, void *C, float *ws, size_t M, size_t N, size_t K, int splitK)
{
    constexpr int TN = NT * 16, TM = WR * RT * 16;
    constexpr size_t x_bytes = 2 * (size_t)WK * TN * kXsRowBytes, red_bytes = WK > 1 ? (size_t)WK * WR * RT * NT * 1024 : 0;
    constexpr size_t lds_bytes = x_bytes > red_bytes ? x_bytes : red_bytes;
    static_assert(lds_bytes <= 160 * 1024, "tile does not fit in LDS");
    if (M % TM) return FP6MI_ERR_SHAPE;
    static bool attr_set = false; // idempotent, so a race between host threads is harmless
    if (!attr_set && lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_tile<FM, NT, RT, WR, WK>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return (int)e;
        attr_set = true;
    }
    uint32_t units = (uint32_t)((K + 255) / 256), nblocks = (uint32_t)((N + TN - 1) / TN);
    size_t   wgs = (M / TM) * (size_t)splitK * nblocks;
    if (wgs > 0x7fffffffu) return FP6MI_ERR_SHAPE;
    hipLaunchKernelGGL((gemm_tile<FM, NT, RT, WR, WK>), dim3((uint32_t)wgs), dim3(WR * WK * kWave), lds_bytes, st,
                       static_cast<const uint8_t *>(W), static_cast<const half_t *>(sc), static_cast<const half_t *>(B), static_cast<half_t *>(C),
                       ws, (uint32_t)M, (uint32_t)N, (uint32_t)K, units, (uint32_t)splitK, nblocks);
    return (int)hipGetLastError();
}

// kind 0: gemm_stream (wr == 1, wk = wavefronts per workgroup);  kind 1: gemm_tile (wr x wk wavefronts)
struct LaunchCfg { int kind, nt, rt, wr, wk; };

// Rule for batches above 16 where no measured neighbour exists: score the six tile shapes that exhaustive sweeps showed to
// cover every case (64x32 with four K wavefronts; 128x32 with one or two; 128x64 with two; 256x64; 256x128) and take the
// best.  The score is the product of
//   * how full the chip is: workgroups / slots (one workgroup per CU, two for four-wavefront workgroups), divided by the
//     number of rounds that takes when there are more workgroups than slots;
//   * the share of the tile's columns that are real batch columns;
//   * pipeline fill: chunks / (chunks + 2), a workgroup with few K chunks is mostly prologue and epilogue;
//   * 1 / (1 + 32 * bytes through the CU's L1 per multiply-accumulate), which favours large tiles.
// Against an exhaustive sweep (99 problems, all compiled shapes) the choice loses 0.6 % on average and 15 % at worst.
struct TileShape { int nt, rt, wr, wk; };
constexpr TileShape kRuleShapes[] = { { 2, 1, 4, 4 }, { 2, 2, 4, 1 }, { 2, 2, 4, 2 }, { 4, 2, 4, 2 }, { 4, 2, 8, 1 }, { 8, 2, 8, 1 } };

inline double tile_score(size_t M, size_t N, size_t K, int splitK, const TileShape &t, int cus)
{
    const size_t TM = (size_t)t.wr * t.rt * 16, TN = (size_t)t.nt * 16, units = (K + 255) / 256, per_split = (units + splitK - 1) / splitK;
    if (M % TM || (size_t)t.wk > per_split) return 0.0;
    const size_t nblocks = (N + TN - 1) / TN;
    const double wgs = (double)(M / TM) * nblocks * splitK, slots = (double)cus * (t.wr * t.wk <= 4 ? 2 : 1);
    const double fill = wgs / slots, eff = fill >= 1.0 ? fill / std::ceil(fill) : fill;
    const double cover = (double)N / (double)(nblocks * TN);
    const double chunks = (double)per_split / t.wk, pipe = chunks / (chunks + 2.0);
    const double traffic = (0.75 * TM + 2.0 * TN) / ((double)TM * TN);
    return eff * cover * pipe / (1.0 + 32.0 * traffic);
}

// Estimated time in ns of the best shape for a given splitK: weight bytes at 6 TB/s divided by the score, plus, for a split, a
// second launch (2 us) and the FP32 partial sums written and read back (8 bytes per output per split at 8 TB/s).
inline double tile_estimate_ns(size_t M, size_t N, size_t K, int splitK, int cus, const TileShape **best_shape)
{
    double best = 0.0;
    for (const TileShape &t : kRuleShapes) {
        double sc = tile_score(M, N, K, splitK, t, cus);
        if (sc > best) { best = sc; if (best_shape) *best_shape = &t; }
    }
    if (best <= 0.0) return 1e30;
    double ns = (double)M * K * 0.75 / 6000.0 / best;
    if (splitK > 1) ns += 2000.0 + (double)splitK * M * N * 8.0 / 8000.0;
    return ns;
}

// ---- measured launch shapes (generated by `python -m fp6_llm_amd.tune`, MI355X, 256 CUs) ----
struct TuneCfg { uint8_t kind, nt, rt, wr, wk; uint16_t t; };              // t in 0.02 us; kind 255 = not measured
struct TuneEntry { uint8_t xb; uint16_t m256, k64, n; TuneCfg sk[4]; };    // sk[i]: best shape for splitK = 1 << i
const TuneEntry kTune[] = {
    { 0, 0, 0, 0, { { 255, 0, 0, 0, 0, 0 }, { 255, 0, 0, 0, 0, 0 }, { 255, 0, 0, 0, 0, 0 }, { 255, 0, 0, 0, 0, 0 } } }, // keeps the array non-empty
#include "fp6mi_tuning.inc"
};

inline bool cfg_fits(const TuneCfg &c, size_t M) { return c.kind != 255 && M % (16u * c.rt * (c.kind == 1 ? c.wr : 1u)) == 0; }

// Nearest measured problem: the batch is rounded UP to a measured batch of the same kernel family (a shape's cost steps at
// column-tile boundaries), M and K go to the nearest measured value in ratio, at most a factor 1.5 away.
struct TuneGroup { int xb; size_t n, begin, end; }; // entries [begin, end) of kTune share format and batch (the table is sorted by them)

const std::vector<TuneGroup> &tune_groups()
{
    static const std::vector<TuneGroup> groups = [] {
        std::vector<TuneGroup> g;
        const size_t           count = sizeof(kTune) / sizeof(kTune[0]);
        for (size_t i = 1; i < count; i++) {
            if (g.empty() || g.back().xb != kTune[i].xb || g.back().n != kTune[i].n) g.push_back(TuneGroup{ kTune[i].xb, kTune[i].n, i, i });
            g.back().end = i + 1;
        }
        return g;
    }();
    return groups;
}

const TuneEntry *tune_lookup(int xbits, size_t M, size_t N, size_t K)
{
    // a serving loop asks for the same few layer shapes at whatever batch size the scheduler formed: remember answers
    struct Memo { int xb; size_t M, N, K; const TuneEntry *e; };
    static thread_local Memo memo[256];
    Memo &slot = memo[(M * 0x9E3779B97F4A7C15ull + N * 0xC2B2AE3D27D4EB4Full + K * 0x165667B19E3779F9ull + (size_t)xbits) >> 56];
    if (slot.xb == xbits && slot.M == M && slot.N == N && slot.K == K) return slot.e;
    const TuneGroup *group = nullptr, *widest = nullptr;
    for (const TuneGroup &g : tune_groups()) {
        if (g.xb != xbits || (g.n <= 16) != (N <= 16)) continue;
        if (g.n >= N && (!group || g.n < group->n)) group = &g;
        if (!widest || g.n > widest->n) widest = &g;
    }
    if (!group) group = widest; // batches beyond the largest measured one behave like it, only with more column blocks
    const TuneEntry *best = nullptr;
    float            best_d = 0.f;
    if (group) {
        const float lm = std::log2((float)M / 256.f), lk = std::log2((float)K / 64.f);
        for (size_t i = group->begin; i < group->end; i++) {
            const TuneEntry &e = kTune[i];
            float dm = std::fabs(lm - std::log2((float)e.m256)), dk = std::fabs(lk - std::log2((float)e.k64));
            if (dm > 0.585f || dk > 0.585f) continue;
            if (!best || dm + dk < best_d) { best = &e; best_d = dm + dk; }
        }
    }
    slot = Memo{ xbits, M, N, K, best };
    return best;
}

// Launch shape for a given splitK.
//  N <= 16: stream kernel.  Row tiles per wavefront (rt) reuse the activation registers, so rt grows with M; wavefronts
//           per workgroup follow the K blocks of one split and the register budget (16 wavefronts leave 128 VGPRs each).
//  N > 16:  tile kernel, 128 rows x 32 or 64 columns, with the K parallelism that splitK leaves open given to the
//           wavefronts of the workgroup (at most what its LDS holds).
inline LaunchCfg pick_cfg(int xbits, size_t M, size_t N, size_t K, int splitK, int cus)
{
    LaunchCfg c;
    if (cus == 256 && (splitK == 1 || splitK == 2 || splitK == 4 || splitK == 8)) {
        if (const TuneEntry *e = tune_lookup(xbits, M, N, K)) {
            const TuneCfg &t = e->sk[splitK == 1 ? 0 : splitK == 2 ? 1 : splitK == 4 ? 2 : 3];
            if (cfg_fits(t, M)) return LaunchCfg{ t.kind, t.nt, t.rt, t.wr, t.wk };
        }
    }
    size_t    tiles = M / 16, units = (K + 255) / 256, per_split = (units + splitK - 1) / splitK;
    if (N <= 16) {
        c.kind = 0;
        c.nt = 1;
        c.wr = 1;
        // Fitted to a sweep of every compiled shape over M in 2048..28672, K in 4096..28672, N in 1..16, both formats, on
        // the MI355X.  What it encodes: about eight to eleven wavefronts per CU keep the memory system full; small
        // workgroups (four wavefronts) balance better than large ones once there are several per CU; sharing the
        // activation registers among row tiles (rt) pays in proportion to the batch, because every workgroup pulls the
        // whole activation matrix through its CU's L1.
        const double per_cu = (double)tiles * splitK / cus; // 16-row tiles per CU
        if (N <= 4) {
            if (per_cu < 1.5)        { c.rt = 1; c.wk = N <= 2 ? 16 : 8; }
            else if (per_cu < 2.5)   { c.rt = 2; c.wk = 8; }
            else if (per_cu < 3.125) { c.rt = 1; c.wk = 4; }
            else if (per_cu < 5.5)   { c.rt = 2; c.wk = 4; }
            else                     { c.rt = 2; c.wk = 8; }
        } else if (N <= 8) {
            if (per_cu < 1.5)        { c.rt = 1; c.wk = 8; }
            else if (per_cu < 2.5)   { c.rt = 2; c.wk = 8; }
            else if (per_cu < 3.125) { c.rt = 4; c.wk = 8; }
            else if (per_cu < 5.5)   { c.rt = 2; c.wk = 4; }
            else                     { c.rt = 4; c.wk = 4; }
        } else {
            if (per_cu < 1.5)        { c.rt = 1; c.wk = 8; }
            else if (per_cu < 2.5)   { c.rt = 2; c.wk = 4; }
            else                     { c.rt = 4; c.wk = 4; }
        }
        while (c.rt > 1 && tiles % c.rt) c.rt /= 2;
        const int cap = per_split > 8 ? 16 : per_split > 4 ? 8 : 4; // no more wavefronts than K blocks to hand out
        if (c.wk > cap) c.wk = cap;
        if (c.rt == 4 && c.wk == 16) c.wk = 8; // not compiled: 16 wavefronts leave too few registers for four row tiles
        (void)xbits;
        return c;
    }
    c.kind = 1;
    const TileShape *t = nullptr;
    tile_estimate_ns(M, N, K, splitK, cus, &t);
    if (!t) t = &kRuleShapes[1]; // 128 x 32, one K wavefront: divides every legal M and needs a single K block
    c.nt = t->nt, c.rt = t->rt, c.wr = t->wr, c.wk = t->wk;
    return c;
}

template <int FM>
int launch_cfg(const LaunchCfg &c, hipStream_t st, const void *W, const void *sc, const void *B, void *C, float *ws, size_t M, size_t N,
               size_t K, int splitK)
{
    if (c.kind == 0) {
#define FP6MI_CASE(NT, RT, WV) \
    if (c.nt == NT && c.rt == RT && c.wk == WV && c.wr == 1) return launch_stream<FM, NT, RT, WV>(st, W, sc, B, C, ws, M, N, K, splitK);
        FP6MI_CASE(1, 1, 4) FP6MI_CASE(1, 1, 8) FP6MI_CASE(1, 1, 16)
        FP6MI_CASE(1, 2, 4) FP6MI_CASE(1, 2, 8) FP6MI_CASE(1, 2, 16)
        FP6MI_CASE(1, 4, 4) FP6MI_CASE(1, 4, 8)
        FP6MI_CASE(2, 1, 4) FP6MI_CASE(2, 1, 8)
        FP6MI_CASE(2, 2, 4) FP6MI_CASE(2, 2, 8)
        FP6MI_CASE(4, 1, 4) FP6MI_CASE(4, 1, 8)
        FP6MI_CASE(4, 2, 4) FP6MI_CASE(4, 2, 8)
#undef FP6MI_CASE
    } else if (c.kind == 1) {
#define FP6MI_CASE(NT, RT, WR, WK) \
    if (c.nt == NT && c.rt == RT && c.wr == WR && c.wk == WK) return launch_tile<FM, NT, RT, WR, WK>(st, W, sc, B, C, ws, M, N, K, splitK);
        FP6MI_CASE(2, 1, 4, 4) FP6MI_CASE(2, 2, 4, 4) FP6MI_CASE(2, 2, 4, 2) FP6MI_CASE(2, 2, 4, 1) FP6MI_CASE(2, 4, 4, 1) FP6MI_CASE(2, 4, 4, 2)
        FP6MI_CASE(4, 2, 4, 2) FP6MI_CASE(4, 2, 4, 1) FP6MI_CASE(4, 4, 4, 1) FP6MI_CASE(4, 4, 2, 1) FP6MI_CASE(4, 4, 2, 2)
        FP6MI_CASE(8, 2, 4, 1) FP6MI_CASE(8, 2, 2, 1) FP6MI_CASE(4, 2, 8, 1) FP6MI_CASE(4, 2, 8, 2) FP6MI_CASE(2, 2, 8, 1) FP6MI_CASE(2, 2, 8, 2) FP6MI_CASE(8, 2, 8, 1) FP6MI_CASE(4, 1, 8, 2) FP6MI_CASE(4, 1, 8, 1) FP6MI_CASE(4, 1, 4, 2) FP6MI_CASE(2, 1, 2, 4)
#undef FP6MI_CASE
    }
    return FP6MI_ERR_SHAPE;
}

template <int FM>
int linear_native(hipStream_t st, const void *W, const void *sc, const void *B, void *C, size_t M, size_t N, size_t K, float *ws,
                  int splitK, const LaunchCfg *forced)
{
    LaunchCfg c = forced ? *forced : pick_cfg(Fmt<FM>::bits, M, N, K, splitK, 256);
    if (c.kind == 0 && (M / 16) % c.rt) return FP6MI_ERR_SHAPE;
    int rc = launch_cfg<FM>(c, st, W, sc, B, C, ws, M, N, K, splitK);
    if (rc != 0) return rc;
    if (splitK > 1) {
        size_t MN = M * N; // M % 256 == 0, so MN % 4 == 0
        hipLaunchKernelGGL(splitk_reduce, dim3((uint32_t)((MN / 4 + 255) / 256)), dim3(256), 0, st, static_cast<half_t *>(C), ws, MN,
                           splitK);
        rc = (int)hipGetLastError();
    }
    return rc;
}

} // namespace

// ------------------------------------------------------------------------------------------------ C ABI

extern "C" {

const char *fp6mi_error_string(int code)
{
    switch (code) {
    case FP6MI_OK: return "success";
    case FP6MI_ERR_FORMAT: return "unsupported (E,M): only FP6_e3m2 (3,2), FP5_e2m2 (2,2), FP6_e2m3 (2,3) and FP4_e2m1 (2,1)";
    case FP6MI_ERR_SHAPE: return "unsupported shape: need M % 256 == 0 (64 for CPU packers, 16 for native packers), K % 64 == 0, N >= 1, distinct in/out";
    case FP6MI_ERR_NULL: return "a required pointer is NULL";
    case FP6MI_ERR_WORKSPACE: return "splitK > 1 needs a workspace of splitK*M*N floats";
    case FP6MI_ERR_SPLITK: return "splitK must be >= 1";
    case FP6MI_ERR_ALIGN: return "device pointers must be 16-byte aligned";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown fp6mi error";
    }
}

int fp6mi_version(void) { return 100; }

int fp6mi_prepack_ref(int E, int Mb, void *packed, const void *raw, size_t M, size_t K) { return fp6mi::prepack_ref(E, Mb, packed, raw, M, K); }
int fp6mi_unpack_ref(int E, int Mb, void *raw, const void *packed, size_t M, size_t K) { return fp6mi::unpack_ref(E, Mb, raw, packed, M, K); }
int fp6mi_dequant(int E, int Mb, void *out, const void *raw, size_t M, size_t K, const void *sc) { return fp6mi::dequant(E, Mb, out, raw, M, K, sc); }
size_t fp6mi_native_bytes(int E, int Mb, size_t M, size_t K) { return fp6mi::native_bytes(E, Mb, M, K); }
int fp6mi_prepack_native(int E, int Mb, void *native, const void *raw, size_t M, size_t K) { return fp6mi::prepack_native(E, Mb, native, raw, M, K); }
int fp6mi_unpack_native(int E, int Mb, void *raw, const void *native, size_t M, size_t K) { return fp6mi::unpack_native(E, Mb, raw, native, M, K); }
int fp6mi_relayout_ref_to_native(int E, int Mb, void *native, const void *ref, size_t M, size_t K)
{
    return fp6mi::relayout_ref_to_native(E, Mb, native, ref, M, K);
}

size_t fp6mi_workspace_bytes(size_t M, size_t N, int splitK) { return splitK > 1 ? (size_t)splitK * M * N * sizeof(float) : 0; }

// Split-K choice.  Batches up to 16 (stream kernel): a cost model in microseconds on a part with `num_cus` compute
// units -- workgroups run in rounds of one per CU, a workgroup streams its weights at what one CU sustains, the whole
// chip cannot beat HBM, and a split costs a second launch plus writing and re-reading the FP32 partial sums; K is
// already split inside the workgroup, so a split rarely pays.  Larger batches (tile kernel): as much of the wanted K
// parallelism as keeps the FP32 partial-sum traffic (8 bytes per output per split) under half of the weight bytes.
int fp6mi_heuristic_splitk(size_t M, size_t N, size_t K, int num_cus)
{
    if (M == 0 || N == 0 || K == 0 || num_cus <= 0) return 1;
    size_t units = (K + 255) / 256;
    if (num_cus == 256) { // a measured neighbour knows better than any model: take its fastest split (3 % hysteresis towards fewer splits)
        if (const TuneEntry *e = tune_lookup(6, M, N, K)) {
            int      best_s = 0;
            unsigned best_t = 0;
            for (int i = 0; i < 4; i++) {
                const TuneCfg &t = e->sk[i];
                if (!cfg_fits(t, M) || (size_t)(1 << i) > units) continue;
                if (best_s == 0 || (unsigned)t.t * 103u < best_t * 100u) { best_s = 1 << i; best_t = t.t; }
            }
            if (best_s) return best_s;
        }
    }
    if (N > 16) {
        int    best_s = 1;
        double best_ns = 1e30;
        for (int sp = 1; sp <= 8 && (size_t)sp <= units; sp *= 2) {
            if (sp > 1 && (double)sp * 8.0 * (double)N > 0.75 * (double)K) break; // partial sums would outweigh the weights
            double ns = tile_estimate_ns(M, N, K, sp, num_cus, nullptr);
            if (ns < best_ns * 0.97) { best_ns = ns; best_s = sp; }
        }
        return best_s;
    }
    const double cu_gbps = 60.0, hbm_gbps = 6000.0, launch_us = 3.0;
    size_t       wgs = M / 16 ? M / 16 : 1;
    double       best = 1e30;
    int          best_s = 1;
    for (int s = 1; s <= 64 && (size_t)s <= units; s++) {
        double per_wg_bytes = (double)((units + s - 1) / s) * 3072.0;
        double rounds = std::ceil((double)(wgs * (size_t)s) / (double)num_cus);
        double t_cu = rounds * per_wg_bytes / (cu_gbps * 1e3);
        double t_hbm = (double)wgs * (double)units * 3072.0 / (hbm_gbps * 1e3);
        double t = launch_us + (t_cu > t_hbm ? t_cu : t_hbm);
        if (s > 1) t += launch_us + 2.0 * (double)s * (double)M * (double)N * 4.0 / (hbm_gbps * 1e3);
        if (t < best * 0.97) { best = t; best_s = s; }
    }
    return best_s;
}

static int check_gemm_args(int E, int Mb, const void *W, const void *sc, const void *B, const void *C, size_t M, size_t N, size_t K,
                           const float *ws, int splitK)
{
    if (!fp6mi::supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!W || !sc || !B || !C) return FP6MI_ERR_NULL;
    if (M == 0 || M % 256 || K == 0 || K % 64 || N == 0) return FP6MI_ERR_SHAPE;
    if (M > 0x7fffffffu || N > 0x7fffffffu || K > 0x7fffffffu || (N + 15) / 16 > 65535) return FP6MI_ERR_SHAPE;
    if (splitK < 1 || splitK > 65535) return FP6MI_ERR_SPLITK;
    if (splitK > 1 && !ws) return FP6MI_ERR_WORKSPACE;
    if (!aligned16(W) || !aligned16(B) || !aligned16(C) || (ws && !aligned16(ws))) return FP6MI_ERR_ALIGN;
    return FP6MI_OK;
}

int fp6mi_linear_native(int E, int Mb, void *stream, const void *W, const void *sc, const void *B, void *C, size_t M, size_t N, size_t K,
                        float *ws, int splitK)
{
    int rc = check_gemm_args(E, Mb, W, sc, B, C, M, N, K, ws, splitK);
    if (rc != FP6MI_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return with_format(E, Mb, [&](auto fm) { return linear_native<decltype(fm)::value>(st, W, sc, B, C, M, N, K, ws, splitK, nullptr); });
}

int fp6mi_linear_native_cfg(int E, int Mb, void *stream, const void *W, const void *sc, const void *B, void *C, size_t M, size_t N, size_t K,
                            float *ws, int splitK, int kind, int n_tiles, int row_tiles, int row_waves, int k_waves)
{
    int rc = check_gemm_args(E, Mb, W, sc, B, C, M, N, K, ws, splitK);
    if (rc != FP6MI_OK) return rc;
    LaunchCfg   c = { kind, n_tiles, row_tiles, row_waves, k_waves };
    hipStream_t st = static_cast<hipStream_t>(stream);
    return with_format(E, Mb, [&](auto fm) { return linear_native<decltype(fm)::value>(st, W, sc, B, C, M, N, K, ws, splitK, &c); });
}

int fp6mi_query_launch(int E, int Mb, size_t M, size_t N, size_t K, int splitK, int *shape)
{
    if (!fp6mi::supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!shape) return FP6MI_ERR_NULL;
    if (M == 0 || M % 256 || K == 0 || K % 64 || N == 0) return FP6MI_ERR_SHAPE;
    if (splitK < 1) return FP6MI_ERR_SPLITK;
    LaunchCfg c = pick_cfg(1 + E + Mb, M, N, K, splitK, 256);
    shape[0] = c.kind, shape[1] = c.nt, shape[2] = c.rt, shape[3] = c.wr, shape[4] = c.wk;
    return FP6MI_OK;
}

// ---- drop-in entry on REFERENCE-layout weights: native twins are made on first sight of a weight pointer and kept ----
namespace {
struct Twin { void *native; int E, Mb; size_t M, K; int device; };
std::mutex                              g_twin_mutex;
std::unordered_map<const void *, Twin>  g_twins;
} // namespace

int fp6mi_linear(int E, int Mb, void *stream, const void *W_ref, const void *sc, const void *B, void *C, size_t M, size_t N, size_t K,
                 float *ws, int splitK)
{
    int rc = check_gemm_args(E, Mb, W_ref, sc, B, C, M, N, K, ws, splitK);
    if (rc != FP6MI_OK) return rc;
    int device = 0;
    if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return (int)e;
    void *native = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_twin_mutex);
        auto it = g_twins.find(W_ref);
        if (it != g_twins.end()) {
            const Twin &t = it->second;
            if (t.E == E && t.Mb == Mb && t.M == M && t.K == K && t.device == device) {
                native = t.native;
            } else { // the address now holds a different matrix
                (void)hipFree(t.native);
                g_twins.erase(it);
            }
        }
        if (!native) {
            size_t bytes = fp6mi::native_bytes(E, Mb, M, K);
            if (hipError_t e = hipMalloc(&native, bytes); e != hipSuccess) return (int)e;
            rc = fp6mi_relayout_ref_to_native_gpu(E, Mb, stream, native, W_ref, M, K); // same stream: ordered before the GEMM
            if (rc != 0) {
                (void)hipFree(native);
                return rc;
            }
            g_twins[W_ref] = Twin{ native, E, Mb, M, K, device };
        }
    }
    return fp6mi_linear_native(E, Mb, stream, native, sc, B, C, M, N, K, ws, splitK);
}

int fp6mi_twin_evict(const void *W_ref)
{
    std::lock_guard<std::mutex> lock(g_twin_mutex);
    auto it = g_twins.find(W_ref);
    if (it == g_twins.end()) return FP6MI_OK;
    hipError_t e = hipFree(it->second.native); // hipFree waits for work that may still read the buffer
    g_twins.erase(it);
    return (int)e;
}

int fp6mi_twin_clear(void)
{
    std::lock_guard<std::mutex> lock(g_twin_mutex);
    int rc = 0;
    for (auto &kv : g_twins) {
        hipError_t e = hipFree(kv.second.native);
        if (e != hipSuccess) rc = (int)e;
    }
    g_twins.clear();
    return rc;
}

int fp6mi_relayout_ref_to_native_gpu(int E, int Mb, void *stream, void *native, const void *ref, size_t M, size_t K)
{
    if (!fp6mi::supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!native || !ref) return FP6MI_ERR_NULL;
    if (M == 0 || M % 64 || K == 0 || K % 64 || M > 0x7fffffffu || K > 0x7fffffffu || native == ref) return FP6MI_ERR_SHAPE;
    if (!aligned16(native) || !aligned16(ref)) return FP6MI_ERR_ALIGN;
    uint32_t units = (uint32_t)((K + 255) / 256);
    size_t   blocks = (M / 16) * units;
    dim3     grid((uint32_t)((blocks + 3) / 4));
    hipStream_t st = static_cast<hipStream_t>(stream);
    return with_format(E, Mb, [&](auto fm) {
        hipLaunchKernelGGL(relayout_ref_to_native<decltype(fm)::value>, grid, dim3(256), 0, st, static_cast<uint8_t *>(native),
                           static_cast<const uint8_t *>(ref), (uint32_t)M, (uint32_t)K, units);
        return (int)hipGetLastError();
    });
}

int fp6mi_dequant_native_gpu(int E, int Mb, void *stream, void *out, const void *W, const void *sc, size_t M, size_t K)
{
    if (!fp6mi::supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!out || !W || !sc) return FP6MI_ERR_NULL;
    if (M == 0 || M % 16 || K == 0 || K % 64 || M > 0x7fffffffu || K > 0x7fffffffu) return FP6MI_ERR_SHAPE;
    if (!aligned16(out) || !aligned16(W)) return FP6MI_ERR_ALIGN;
    uint32_t units = (uint32_t)((K + 255) / 256);
    size_t   blocks = (M / 16) * units;
    dim3     grid((uint32_t)((blocks + 3) / 4));
    hipStream_t st = static_cast<hipStream_t>(stream);
    return with_format(E, Mb, [&](auto fm) {
        hipLaunchKernelGGL(dequant_native<decltype(fm)::value>, grid, dim3(256), 0, st, static_cast<half_t *>(out), static_cast<const uint8_t *>(W),
                           static_cast<const half_t *>(sc), (uint32_t)M, (uint32_t)K, units);
        return (int)hipGetLastError();
    });
}

int fp6mi_quantize_native_gpu(int E, int Mb, void *stream, void *native, void *scales, const void *weights, int dtype, size_t M, size_t K)
{
    if (!fp6mi::supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!native || !scales || !weights) return FP6MI_ERR_NULL;
    if (dtype < 0 || dtype > 2) return FP6MI_ERR_FORMAT;
    if (M == 0 || M % 16 || K == 0 || K % 64 || M > 0x7fffffffu || K > 0x7fffffffu) return FP6MI_ERR_SHAPE;
    if (!aligned16(native) || !aligned16(weights)) return FP6MI_ERR_ALIGN;
    const uint32_t units = (uint32_t)((K + 255) / 256);
    const size_t   blocks = (M / 16) * units;
    const dim3     grid_rows((uint32_t)((M + 3) / 4)), grid_blocks((uint32_t)((blocks + 3) / 4));
    hipStream_t    st = static_cast<hipStream_t>(stream);
    uint8_t       *nat = static_cast<uint8_t *>(native);
    half_t        *sc = static_cast<half_t *>(scales);
    return with_format(E, Mb, [&](auto fm) {
        constexpr int    FM = decltype(fm)::value;
        constexpr double max_value = Fmt<FM>::max_value;
        auto             run = [&](auto *typed) {
            typedef std::remove_cv_t<std::remove_pointer_t<decltype(typed)>> T;
            hipLaunchKernelGGL(quant_row_scales<T>, grid_rows, dim3(256), 0, st, sc, typed, (uint32_t)M, (uint32_t)K, max_value);
            hipLaunchKernelGGL((quant_to_native<FM, T>), grid_blocks, dim3(256), 0, st, nat, sc, typed, (uint32_t)M, (uint32_t)K, units, max_value);
        };
        if (dtype == 0)
            run(static_cast<const half_t *>(weights));
        else if (dtype == 1)
            run(static_cast<const bf16_t *>(weights));
        else
            run(static_cast<const float *>(weights));
        return (int)hipGetLastError();
    });
}

} // extern "C"
