// gfx950 (MI355X) kernels of the FPx x FP16 linear layer and their launchers, for ONE weight format per translation unit:
// the build compiles this file once per format with -DFP6MI_FORMAT=<10*E+M> (32, 22, 23, 21), in parallel, and each object
// exports one table of entry functions (fp6mi::FormatOps) that the C ABI in fp6mi_api.hip dispatches to.
//
// Roles taken over from the reference (usyd-fsalab/fp6_llm, paths relative to it):
//   gemm_stream, gemm_tile, gemm_ws <- QUANT_GEMM_Kernel   fp6_llm/csrc/include/kernel_matmul.cuh:29-191
//                    (small batches / batches above 16 / large batches: three organisations of the same GEMM)
//   splitk_reduce <- SplitK_Reduction         fp6_llm/csrc/include/kernel_reduction.cuh:28-47   (in fp6mi_api.hip)
//   launchers     <- fpx_linear_kernel        fp6_llm/csrc/fp6_linear.cu:44-102
// The design is not a translation: weights use the native layout described in fp6mi_host.cpp, go from HBM straight
// to VGPRs with 128-bit non-temporal loads, FP6 codes are converted by the CDNA4 instruction
// v_cvt_scalef32_pk32_f16_bf6 (BF6 = e3m2, bias 3, no inf/nan: the very format of the reference), FP5 codes by the same
// instruction after a zero bit is slipped in above their exponent (an e2m2 code read as e3m2 is a quarter of its value),
// FP6_e2m3 codes by v_cvt_scalef32_pk32_f16_fp6 and FP4_e2m1 codes by that instruction after two zero bits are appended
// to their mantissa, and v_mfma_f32_16x16x32_f16 accumulates in FP32.  The per-row scale (and the factor 4 of FP5) is
// applied once to the FP32 sums instead of to every weight.
#include <hip/hip_runtime.h>

#include <atomic>
#include <type_traits>

#include "fp6mi_internal.h"

#ifndef FP6MI_FORMAT
#error "compile with -DFP6MI_FORMAT=32, 22, 23 or 21 (10*E + M of the weight format)"
#endif

namespace {

using fp6mi::LaunchCfg;

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

// One of the two or three loads of load_wfrag, for a kernel that spreads them over its compute.
template <int FM> __device__ __forceinline__ void load_wfrag_part(WFrag<FM> &f, const uint8_t *block, int lane, int part)
{
    const v4u *p = reinterpret_cast<const v4u *>(block) + lane;
    if (part == 0) f.a = __builtin_nontemporal_load(p);
    if (part == 1) f.b = __builtin_nontemporal_load(p + 64);
    if constexpr (Fmt<FM>::bits == 6) { if (part == 2) f.c = __builtin_nontemporal_load(p + 128); }
    if constexpr (Fmt<FM>::bits == 5) { if (part == 2) f.s = __builtin_nontemporal_load(reinterpret_cast<const v2u *>(block + 2048) + lane); }
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

// The conversion instruction multiplies its 32 values by the power of two in the exponent field of `scale` at no cost.
template <int FM> __device__ __forceinline__ v32h fields_to_halfs(v6u src, float scale)
{
    if constexpr (Fmt<FM>::hw_e3m2)
        return __builtin_amdgcn_cvt_scalef32_pk32_f16_bf6(src, scale);
    else
        return __builtin_amdgcn_cvt_scalef32_pk32_f16_fp6(src, scale);
}

// Group exponents: one byte b per (row, 128 columns), meaning the factor 2^(b-127) on those weights (the E8M0 scale type of
// the OCP MX formats).  A lane's 32-code string is exactly its row's share of one 128-column group, so the factor rides on
// the conversion instruction.  Native layout of the bytes: [row tile][K block][row in tile][half of the block], 32 bytes per
// block; `g` below is the lane's pair of bytes (half 0 in the low byte).  GS = false: no group exponents, factor 1.
template <bool GS> __device__ __forceinline__ float group_factor(uint32_t g, int h)
{
    if constexpr (GS)
        return __builtin_bit_cast(float, (h == 0 ? (g & 0xffu) : (g >> 8)) << 23);
    else
        return 1.0f;
}
// block = index of the 16x256 block counted from `gexp` (32 bytes each); nothing is computed or read without group exponents
template <bool GS> __device__ __forceinline__ uint32_t load_group_exps(const uint8_t *gexp, size_t block, int lane)
{
    if constexpr (GS)
        return *reinterpret_cast<const uint16_t *>(gexp + block * 32 + 2 * (lane & 15));
    else
        return 0;
}

template <int FM, bool GS> __device__ __forceinline__ void convert(const WFrag<FM> &f, AOps<FM> &o, uint32_t g)
{
    v32h h0 = fields_to_halfs<FM>(field_string<FM>(f, 0), group_factor<GS>(g, 0));
    v32h h1 = fields_to_halfs<FM>(field_string<FM>(f, 1), group_factor<GS>(g, 1));
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
// activations L2 -> VGPR -> LDS -> VGPR (reused for the RT row tiles); the partial accumulators are summed through LDS.
//
// Why the activations take the detour through LDS.  The MFMA wants lane (col, q) to hold 16 bytes of batch row `col`, so a
// load in operand order makes the 16 lanes of every quarter-wavefront touch 16 different 128-byte lines, 16 bytes of each.
// The vector memory pipeline looks up one line per cycle: measured on the MI355X with nothing else in the kernel, the
// operand-order loads of a 4096-wide K for batch 16 on all 256 CUs take 3.1 us, the same bytes loaded as whole rows
// (32 consecutive lanes = 512 consecutive bytes) 0.9 us; batch 8 with two MFMA steps per load 1.4 us against 0.25 us.
// So from batch 5 up every wavefront loads its slice as whole rows, writes it to an LDS area of its own (no barrier: nobody
// else reads it) and reads it back in operand order; LDS rows are padded to 544 bytes, the stride at which that read is
// conflict-free.  Batches of 5 to 8 stage 8 rows (B columns 8..15 re-read rows 0..7 and feed outputs that are never stored).
// Batches up to 4 keep operand-order loads: a quarter-wavefront then touches at most 4 lines, and the trip through LDS
// would only add latency (measured: 1-4 % slower there).
// ---------------------------------------------------------------------------------------------------------------
constexpr int kXsRowBytes = 544;

template <int FM, int RT> struct StageW {
    WFrag<FM> w[RT];
    uint32_t  g[RT]; // group exponents of the block (unused without them)
};

// LDS bytes per wavefront: the activation rows of one K block, or the RT*NT partial tiles of the epilogue (they share it)
__host__ __device__ constexpr uint32_t stream_wave_bytes(int rows, int RT, int NT)
{
    return (uint32_t)(rows * kXsRowBytes > RT * NT * 1024 ? rows * kXsRowBytes : RT * NT * 1024);
}

template <int FM, bool GS, int NT, int RT, int WAVES, bool SPLIT>
__global__ __launch_bounds__(WAVES *kWave) void gemm_stream(const uint8_t *__restrict__ W, const half_t *__restrict__ scales,
                                                            const uint8_t *__restrict__ gexp, const half_t *__restrict__ X, half_t *__restrict__ C,
                                                            float *__restrict__ ws, uint32_t M, uint32_t N, uint32_t K,
                                                            uint32_t units, uint32_t splitK)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    // every kernel argument is fetched by one batch of scalar loads at the top (left alone, the compiler fetches them in
    // three batches, each a round trip to memory, as the code reaches their first use)
    asm volatile("" ::"s"(W), "s"(scales), "s"(gexp), "s"(X), "s"(C), "s"(ws), "s"(M), "s"(N), "s"(K), "s"(units), "s"(splitK));
    // the wavefront's index as a scalar: the K-block loop, its bounds and its branches then run on the scalar unit
    const int      lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int      col = lane & 15, q = lane >> 4;
    const uint32_t R0 = blockIdx.x * RT, split = blockIdx.y, nbase = blockIdx.z * (16 * NT);

    // SPLIT = false is the launch with splitK == 1: its range is the whole of K and its epilogue writes fp16
    uint32_t u0 = 0, u1 = units;
    if constexpr (SPLIT) {
        const uint32_t avg = units / splitK, extra = units % splitK;
        u0 = split * avg + (split < extra ? split : extra);
        u1 = u0 + avg + (split < extra ? 1u : 0u);
    }

    const size_t   tile_stride = (size_t)units * Fmt<FM>::block_bytes;
    const uint8_t *wgroup = W + (size_t)R0 * tile_stride;
    const uint8_t *ggroup = GS ? gexp + (size_t)R0 * units * 32 : nullptr;
    // M is a multiple of 256, so 1, 2, 4 and 8 row tiles per workgroup divide its M/16 row tiles; 3, 5, 6 and 7 need not, and
    // the last workgroup then holds fewer.  Its missing tiles stand in as copies of its last real one (same loads, same arithmetic,
    // nothing stored): rlast is the largest r that names a real tile.
    constexpr bool kRagged = (RT & (RT - 1)) != 0;
    const uint32_t rlast = kRagged && R0 + RT > (M >> 4) ? (M >> 4) - 1 - R0 : RT - 1;
    auto           real = [&](int r) -> uint32_t { return kRagged && (uint32_t)r > rlast ? rlast : (uint32_t)r; };

    v4f acc[RT][NT];
#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int t = 0; t < NT; t++) acc[r][t] = (v4f){ 0.f, 0.f, 0.f, 0.f };

    // The epilogue gives thread e the output (row tile e/(256*NT), column tile, batch column, row e%16); its row scale is
    // fetched now so that no global load sits on the tail of the kernel.
    constexpr int kOutPerThread = (RT * NT * 256 + WAVES * kWave - 1) / (WAVES * kWave);
    half_t        my_scale[kOutPerThread]; // kept as loaded: converting here would wait for the load before the weight loads issue
#pragma unroll
    for (int j = 0; j < kOutPerThread; j++) {
        int e = threadIdx.x + j * WAVES * kWave;
        my_scale[j] = scales[(R0 + real(e < RT * NT * 256 ? (e >> 8) / NT : 0)) * 16 + (e & 15)];
    }

    const uint32_t ncols = N - nbase;              // batch columns of this column block that exist (the launcher made sure of >= 1)
    const bool     small = NT == 1 && ncols <= 8;  // 8 rows are staged instead of 16
    const uint32_t wave_bytes = small ? stream_wave_bytes(8, RT, NT) : stream_wave_bytes(16 * NT, RT, NT);
    uint8_t       *mine = lds + wave * wave_bytes;  // this wavefront's LDS area

    // One K block at a time and no register double-buffering: the other wavefronts of the workgroup keep the memory system
    // busy while this one converts, and a second stage in registers measured slower at every size.
    // workgroups that share an L2 (ids congruent mod 8) start on different K blocks, so that the chip does not ask
    // the same activation lines of the same L2 channel at the same moment
    const uint32_t ufull = K / 256 < u1 ? K / 256 : u1; // the blocks before this one lie wholly inside K
    uint32_t       u = u0 + ((wave + (blockIdx.x >> 3)) % WAVES);
    // MODE 0: batches up to 4 load in operand order (a quarter-wavefront then touches at most 4 lines, and the detour through
    // LDS would only add latency); MODE 1: 8 rows through LDS; MODE 2: 16*NT rows through LDS.  TAIL: the block is cut by K
    // (only the last block of a K that is no multiple of 256).  The kernel chooses outside its K loop: a choice made per
    // block inside the loop cost 0.2 us of a 4.9 us launch.
    auto run = [&](auto mode_c, auto tail_c, uint32_t end) {
        constexpr int  MODE = decltype(mode_c)::value, ROWS = MODE == 2 ? 16 * NT : 8, LOADS = MODE == 0 ? 4 : ROWS / 2;
        constexpr bool TAIL = decltype(tail_c)::value;
        static_assert(!(MODE == 0 && (TAIL || NT != 1)), "operand-order loads serve whole blocks of one column tile");
        // MODE 0: lane (col, q) reads batch row col % 8 at MFMA step offset col / 8
        const uint32_t prow = (uint32_t)(col & 7) < ncols ? col & 7 : ncols - 1;
        const half_t  *xpaired = X + (size_t)(nbase + prow) * K + 8 * q + 32 * (col >> 3);
        // MODE 1, 2: load i of a block brings rows 2i and 2i+1, lane l takes bytes 16*(l%32).. of row 2i + l/32: a scalar base per
        // load plus one per-lane offset for the whole kernel.  Rows beyond the batch repeat its last row (an MFMA output column
        // depends only on its own B column, and those columns are never stored).
        const uint8_t *xbase = reinterpret_cast<const uint8_t *>(X + (size_t)nbase * K);
        const uint32_t off_one = (lane & 31) * 16, off_pair = (lane >> 5) * (K * 2) + off_one; // K < 2^31
        uint8_t       *xw = mine + (lane >> 5) * kXsRowBytes + (lane & 31) * 16;
        const uint8_t *xr = mine + (ROWS == 8 ? col & 7 : col) * kXsRowBytes + q * 16;
        constexpr int  kWParts = Fmt<FM>::bits == 4 ? 2 : 3;
        // Through LDS, the activation loads are issued BEFORE the weight loads: the memory pipeline returns loads in order, so
        // activations asked for first are back (from L2) long before the weights (from HBM), and their trip through LDS
        // is over when the weights arrive.  Issued after the weights they cost 5-10 % at batch 16.  In operand order they go
        // between the second and the third weight load of the first row tile.
        constexpr int kWBeforeX = MODE == 0 ? 2 : 0;
        for (; u < end; u += WAVES) {
            StageW<FM, RT> cur;
            v4u            xv[LOADS];
            auto           wpart = [&](int i) {
                const int r = i / kWParts, part = i % kWParts;
                load_wfrag_part<FM>(cur.w[r], wgroup + real(r) * tile_stride + (size_t)u * Fmt<FM>::block_bytes, lane, part);
            };
#pragma unroll
            for (int i = 0; i < kWBeforeX; i++) wpart(i);
            // K positions beyond K count as zero activations against the zero weights the native layout holds there (0 x 0,
            // whatever the row holds elsewhere: an infinite activation must not meet a padding weight): such a piece is read
            // at the row's start (a valid address) and replaced by zeros
            const bool beyond = TAIL && u * 256 + 8 * (lane & 31) >= K;
#pragma unroll
            for (int i = 0; i < LOADS; i++) {
                if constexpr (MODE == 0) {
                    xv[i] = *reinterpret_cast<const v4u *>(xpaired + (size_t)u * 256 + 64 * i);
                } else {
                    const uint32_t r0 = (uint32_t)(2 * i) < ncols ? 2 * i : ncols - 1;
                    const uint8_t *sb = xbase + ((size_t)r0 * K + (size_t)u * 256) * 2;
                    uint32_t       vo = (uint32_t)(2 * i + 1) < ncols ? off_pair : off_one;
                    if (beyond) vo -= off_one;
                    const v4u v = *reinterpret_cast<const v4u *>(sb + vo);
                    xv[i] = beyond ? (v4u){ 0u, 0u, 0u, 0u } : v;
                }
            }
#pragma unroll
            for (int i = kWBeforeX; i < RT * kWParts; i++) wpart(i);
#pragma unroll
            for (int r = 0; r < RT; r++) cur.g[r] = load_group_exps<GS>(ggroup, (size_t)real(r) * units + u, lane);
            __builtin_amdgcn_sched_barrier(0); // keep every load of the block issued before anything waits
            v8h x[8][NT];
            if constexpr (MODE == 0) {
                // one load brought two MFMA steps: a DPP rotation of each 16-lane row by 8 moves the second step's data down to
                // columns 0..7 (columns 8..15 then hold the other step's real, finite data and feed outputs never stored)
#pragma unroll
                for (int sl = 0; sl < 4; sl++) {
                    v4u w;
#pragma unroll
                    for (int i = 0; i < 4; i++) w[i] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)xv[sl][i], 0x128, 0xf, 0xf, false); // row_ror:8
                    x[2 * sl][0]     = __builtin_bit_cast(v8h, xv[sl]);
                    x[2 * sl + 1][0] = __builtin_bit_cast(v8h, w);
                }
            } else {
#pragma unroll
                for (int i = 0; i < LOADS; i++) *reinterpret_cast<v4u *>(xw + 2 * i * kXsRowBytes) = xv[i];
#pragma unroll
                for (int s = 0; s < 8; s++)
#pragma unroll
                    for (int t = 0; t < NT; t++) x[s][t] = *reinterpret_cast<const v8h *>(xr + t * 16 * kXsRowBytes + 64 * s);
                // the trip through LDS is issued before anything that waits for weights (left alone, the compiler moves register
                // copies that feed the conversion above the LDS writes, and with them the wait for the weight loads)
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int r = 0; r < RT; r++) {
                AOps<FM> a;
                convert<FM, GS>(cur.w[r], a, cur.g[r]);
#pragma unroll
                for (int s = 0; s < 8; s++)
#pragma unroll
                    for (int t = 0; t < NT; t++) acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.s[s], x[s][t], acc[r][t], 0, 0, 0);
            }
        }
    };
    typedef std::integral_constant<int, 0> Direct;
    typedef std::integral_constant<int, 1> Staged8;
    typedef std::integral_constant<int, 2> StagedAll;
    auto staged = [&](auto mode_c, bool whole_blocks) {
        if (whole_blocks) run(mode_c, std::false_type{}, ufull);
        run(mode_c, std::true_type{}, u1); // at most one block, and only when K is not a multiple of 256
    };
    if (small) {
        if constexpr (NT == 1) {
            if (ncols <= 4) {
                run(Direct{}, std::false_type{}, ufull);
                staged(Staged8{}, false);
            } else {
                staged(Staged8{}, true);
            }
        }
    } else {
        staged(StagedAll{}, true);
    }

    // acc[r][t][i] = sum for output row 16r + 4q+i, batch column 16t+col.  Each wavefront parks its tiles in its own LDS
    // area (its activation rows are dead by now; nobody else ever touched them), then the workgroup sums them.
#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int t = 0; t < NT; t++) *reinterpret_cast<v4f *>(mine + (r * NT + t) * 1024 + lane * 16) = acc[r][t];
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
        for (int w = 0; w < WAVES; w++) sum += *reinterpret_cast<const float *>(lds + w * wave_bytes + rt * 1024 + idx * 4);
        uint32_t ng = nbase + 16 * t + n, mg = (R0 + r) * 16 + mm;
        if (ng < N && (!kRagged || (uint32_t)r <= rlast)) {
            float v = sum * ((float)my_scale[j] * Fmt<FM>::post_scale);
            if constexpr (!SPLIT)
                C[(size_t)ng * M + mg] = (half_t)v;
            else
                ws[((size_t)split * N + ng) * M + mg] = v;
        }
    }
}

// A operands of MFMA steps 4h..4h+3 (half of a K block) of one lane.
template <int FM, bool GS> __device__ __forceinline__ void convert_half(const WFrag<FM> &f, int h, v8h (&o)[4], uint32_t g)
{
    v32h v = fields_to_halfs<FM>(field_string<FM>(f, h), group_factor<GS>(g, h));
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

// One segment of a tile's K range: K blocks [u0, u1) of row block `mb` against the batch columns from `nbase`, accumulated
// into acc.  On return the wavefronts with wk == 0 hold the sums of all WK K-wavefronts; the LDS buffers are free again
// once every wavefront of the workgroup has passed a barrier.
template <int FM, bool GS, int NT, int RT, int WR, int WK>
__device__ __forceinline__ void tile_segment(v4f (&acc)[RT][NT], const uint8_t *__restrict__ W, const uint8_t *__restrict__ gexp,
                                             const half_t *__restrict__ X, uint32_t N, uint32_t K, uint32_t units, uint32_t mb, uint32_t nbase,
                                             uint32_t u0, uint32_t u1, uint8_t *lds, int tid, int lane, int wr, int wk, int col, int q)
{
    constexpr int  TN = NT * 16, NTHREADS = WR * WK * kWave;
    constexpr int  kBufBytes = WK * TN * kXsRowBytes;
    constexpr int  kPieces = WK * TN * 32, kPerThread = (kPieces + NTHREADS - 1) / NTHREADS;
    const uint32_t R0 = (mb * WR + wr) * RT; // first row tile of this wavefront
    const size_t   tile_stride = (size_t)units * Fmt<FM>::block_bytes;
    const uint8_t *wgroup = W + (size_t)R0 * tile_stride;
    const uint8_t *ggroup = GS ? gexp + (size_t)R0 * units * 32 : nullptr;

#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int t = 0; t < NT; t++) acc[r][t] = (v4f){ 0.f, 0.f, 0.f, 0.f };

    WFrag<FM> wcur[RT], wnxt[RT];
    uint32_t  gcur[RT], gnxt[RT]; // group exponents travel with the weights (unused without them)
    v4u       xr[kPerThread];

    auto load_w = [&](WFrag<FM>(&dst)[RT], uint32_t(&gdst)[RT], uint32_t c0) {
        const uint32_t u = c0 + wk;
        if (u < u1) {
#pragma unroll
            for (int r = 0; r < RT; r++) {
                dst[r]  = load_wfrag<FM>(wgroup + r * tile_stride + (size_t)u * Fmt<FM>::block_bytes, lane);
                gdst[r] = load_group_exps<GS>(ggroup, (size_t)r * units + u, lane);
            }
        }
    };
    // Per-thread pieces of the activation chunk: piece p = tid + NTHREADS*j is 16 bytes, (K block p / (TN*32) of the chunk,
    // batch column (p/32) % TN, halfs 8*(p%32)..+7).  Row pointers and LDS offsets are fixed for the whole kernel.
    // Columns beyond N read the last real row (their outputs are never stored); positions beyond K or beyond the split are
    // read at position 0 of the row (a valid address) and staged as zeros (zero weights meet them, or no wavefront does).
    const half_t *xrow[kPerThread];
    uint32_t      xlds[kPerThread];
#pragma unroll
    for (int j = 0; j < kPerThread; j++) {
        const uint32_t p = tid + NTHREADS * j, n = nbase + (p >> 5) % TN;
        xrow[j] = X + (size_t)(n < N ? n : N - 1) * K + (p & 31) * 8 + (size_t)(p / (TN * 32)) * 256;
        xlds[j] = (p >> 5) * kXsRowBytes + (p & 31) * 16;
    }
    // `full` (a compile-time flag): the whole chunk lies inside K and inside the segment, so every piece is a plain load.  The
    // K loop below is written out per case: one choice per chunk inside the loop costs a wait for the activation loads before
    // the weight loads can be issued.
    auto load_x = [&](auto full, uint32_t c0) {
        if constexpr (decltype(full)::value) {
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
                    const v4u      v = *reinterpret_cast<const v4u *>(ok ? xrow[j] + (size_t)c0 * 256 : xrow[j] - ((p & 31) * 8 + (size_t)(p / (TN * 32)) * 256));
                    xr[j] = ok ? v : (v4u){ 0u, 0u, 0u, 0u };
                }
            }
        }
    };
    // The same loads one at a time (i = 0 .. kLoads-1: weights first, then activation pieces).  The 256 x 128 tile spreads them
    // over its MFMA steps instead of issuing them in one burst: measured 10-12 % faster for batches from 1024 up (the burst keeps
    // a wavefront, which issues in order, from starting its MFMAs until the CU has accepted its last load); for the smaller
    // tiles, with fewer MFMAs between two loads, spreading measured 0-8 % slower and they keep the burst.
    constexpr bool kSpreadLoads = NT >= 8 && WR * WK >= 8;
    constexpr int  kWParts = Fmt<FM>::bits == 4 ? 2 : 3, kWLoads = RT * kWParts, kLoads = kWLoads + kPerThread, kPerStep = (kLoads + 7) / 8;
    auto load_one = [&](auto full, int i, uint32_t c0) {
        if (i < kWLoads) {
            const int      r = i / kWParts, part = i % kWParts;
            const uint32_t u = c0 + wk;
            if (u < u1) {
                load_wfrag_part<FM>(wnxt[r], wgroup + r * tile_stride + (size_t)u * Fmt<FM>::block_bytes, lane, part);
                if (part == 0) gnxt[r] = load_group_exps<GS>(ggroup, (size_t)r * units + u, lane);
            }
        } else if (i < kLoads) {
            const int      j = i - kWLoads;
            const uint32_t p = tid + NTHREADS * j;
            if (kPieces % NTHREADS == 0 || p < (uint32_t)kPieces) {
                if constexpr (decltype(full)::value) {
                    xr[j] = *reinterpret_cast<const v4u *>(xrow[j] + (size_t)c0 * 256);
                } else {
                    const uint32_t u = c0 + p / (TN * 32), k = u * 256 + (p & 31) * 8;
                    const bool     ok = k < K && u < u1;
                    const v4u      v = *reinterpret_cast<const v4u *>(ok ? xrow[j] + (size_t)c0 * 256 : xrow[j] - ((p & 31) * 8 + (size_t)(p / (TN * 32)) * 256));
                    xr[j] = ok ? v : (v4u){ 0u, 0u, 0u, 0u };
                }
            }
        }
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int j = 0; j < kPerThread; j++)
            if (kPieces % NTHREADS == 0 || tid + NTHREADS * j < kPieces) *reinterpret_cast<v4u *>(lds + buf * kBufBytes + xlds[j]) = xr[j];
    };
    typedef std::integral_constant<int, 0> NoNext;       // the last chunk: nothing to fetch
    typedef std::integral_constant<int, 1> FullNext;     // the next chunk is a full one
    typedef std::integral_constant<int, 2> PartialNext;  // the next chunk is cut by K or by the end of the segment
    typedef std::integral_constant<bool, true> Full;
    typedef std::integral_constant<bool, false> Partial;

    if (u0 < u1) {
        const uint32_t ufull = K / 256 < u1 ? K / 256 : u1; // chunks that end at or before this block are full
        if (u0 + WK <= ufull)
            load_x(Full{}, u0);
        else
            load_x(Partial{}, u0);
        load_w(wcur, gcur, u0);
        store_x(0);
        __syncthreads();
        int      buf = 0;
        uint32_t c0 = u0;
        // one chunk: fetch the next one (if any), compute this one, stage the next one's activations, barrier
        auto chunk = [&](auto next) {
            constexpr int  kNext = decltype(next)::value;
            constexpr bool more = kNext != 0;
            typedef std::integral_constant<bool, kNext == 1> NextIsFull;
            if (more && (!kSpreadLoads || c0 + wk >= u1)) { // (a wavefront without a K block in this chunk has no MFMAs to spread over)
                load_x(NextIsFull{}, c0 + WK);
                load_w(wnxt, gnxt, c0 + WK);
            }
            if (c0 + wk < u1) {
                const uint8_t *xs = lds + buf * kBufBytes + (wk * TN + col) * kXsRowBytes + q * 16;
                v8h            a0[RT][4], a1[RT][4];
#pragma unroll
                for (int r = 0; r < RT; r++) convert_half<FM, GS>(wcur[r], 0, a0[r], gcur[r]);
                // second half converted ahead of the first half's MFMAs: the VALU work then runs under the matrix pipe
#pragma unroll
                for (int r = 0; r < RT; r++) convert_half<FM, GS>(wcur[r], 1, a1[r], gcur[r]);
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
                        if constexpr (kSpreadLoads && more) {
#pragma unroll
                            for (int i = (4 * h + s) * kPerStep; i < (4 * h + s + 1) * kPerStep; i++) load_one(NextIsFull{}, i, c0 + WK);
                        }
                    }
                }
            }
            if (more) {
                store_x(buf ^ 1); // that buffer was last read before the barrier that ended the previous iteration
#pragma unroll
                for (int r = 0; r < RT; r++) wcur[r] = wnxt[r], gcur[r] = gnxt[r];
            }
            __syncthreads();
            c0 += WK, buf ^= 1;
        };
        while (c0 + 2 * WK <= ufull) chunk(FullNext{});
        while (c0 + WK < u1) chunk(PartialNext{});
        chunk(NoNext{});
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
}

// The tile kernel's output goes through LDS.  An MFMA accumulator holds four consecutive rows of ONE batch column per lane, so
// a store straight from the accumulators makes the 16 lanes of a quarter-wavefront write 8 or 16 bytes into each of 16
// different lines (C and the partial sums are [N][M], rows contiguous); the memory pipeline takes a line at a time, and with
// every workgroup finishing at the same moment nothing hides it: measured, those stores were 10-16 % of the GEMMs that split K
// at batches 32-128 and 4-5 % at batch 512.  So the wavefronts that hold results scale them and park them in LDS as a
// [column][row] tile (fp16 for the final output, fp32 for partial sums), and after a barrier every thread of the workgroup
// stores 16 consecutive bytes of one column: a wavefront writes whole lines.
//   stage: TN columns of TM rows, column stride TM * (2 or 4) + 16 bytes
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
template <int NT, int RT, int WR> constexpr size_t tile_stage_bytes(bool partial) { return (size_t)NT * 16 * (WR * RT * 16 * (partial ? 4 : 2) + 16); }

// first half: a wavefront that holds results scales them and parks them in the stage
template <int FM, int NT, int RT, int WR, typename OutT>
__device__ __forceinline__ void tile_park(const v4f (&acc)[RT][NT], const v4h (&sc4)[RT], uint8_t *stage, int wr, int col, int q)
{
    constexpr int TM = WR * RT * 16, kStride = TM * (int)sizeof(OutT) + 16;
#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int t = 0; t < NT; t++) {
            v4f v;
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = acc[r][t][i] * ((float)sc4[r][i] * Fmt<FM>::post_scale);
            uint8_t *dst = stage + (16 * t + col) * kStride + ((wr * RT + r) * 16 + 4 * q) * (int)sizeof(OutT);
            if constexpr (sizeof(OutT) == 2)
                *reinterpret_cast<v4h *>(dst) = (v4h){ (half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3] };
            else
                *reinterpret_cast<v4f *>(dst) = v;
        }
}
// second half, after a barrier: every thread of the workgroup stores 16-byte pieces of the stage's columns
template <int NT, int RT, int WR, int NTHREADS, typename OutT>
__device__ __forceinline__ void tile_flush(OutT *__restrict__ out, const uint8_t *stage, uint32_t M, uint32_t N, uint32_t mb, uint32_t nbase, int tid)
{
    constexpr int TM = WR * RT * 16, TN = NT * 16, kStride = TM * (int)sizeof(OutT) + 16, kPer16 = 16 / (int)sizeof(OutT); // outputs per 16 bytes
    constexpr int kPiecesPerCol = TM / kPer16, kPieces = TN * kPiecesPerCol;
#pragma unroll
    for (int p = tid; p < kPieces; p += NTHREADS) {
        const int      c = p / kPiecesPerCol, piece = p % kPiecesPerCol;
        const uint32_t ng = nbase + c;
        if (ng < N) {
            const v4u d = *reinterpret_cast<const v4u *>(stage + c * kStride + piece * 16);
            *reinterpret_cast<v4u *>(out + (size_t)ng * M + (size_t)mb * TM + piece * kPer16) = d;
        }
    }
}

template <int FM, int NT, int RT, int WR, int NTHREADS, typename OutT>
__device__ __forceinline__ void tile_store(const v4f (&acc)[RT][NT], const v4h (&sc4)[RT], OutT *__restrict__ out, uint8_t *stage, bool holds_results,
                                           uint32_t M, uint32_t N, uint32_t mb, uint32_t nbase, int tid, int wr, int col, int q)
{
    if (holds_results) tile_park<FM, NT, RT, WR, OutT>(acc, sc4, stage, wr, col, q);
    __syncthreads();
    tile_flush<NT, RT, WR, NTHREADS, OutT>(out, stage, M, N, mb, nbase, tid);
}

template <int FM, bool GS, int NT, int RT, int WR, int WK>
__global__ __launch_bounds__(WR *WK *kWave) void gemm_tile(const uint8_t *__restrict__ W, const half_t *__restrict__ scales,
                                                           const uint8_t *__restrict__ gexp, const half_t *__restrict__ X, half_t *__restrict__ C,
                                                           float *__restrict__ ws, uint32_t M, uint32_t N, uint32_t K,
                                                           uint32_t units, uint32_t splitK, uint32_t nblocks)
{
    constexpr int  TN = NT * 16, NTHREADS = WR * WK * kWave;
    constexpr int  kBufBytes = WK * TN * kXsRowBytes;
    constexpr int  kPieces = WK * TN * 32, kPerThread = (kPieces + NTHREADS - 1) / NTHREADS;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    asm volatile("" ::"s"(W), "s"(scales), "s"(gexp), "s"(X), "s"(C), "s"(ws), "s"(M), "s"(N), "s"(K), "s"(units), "s"(splitK), "s"(nblocks)); // one batch of argument loads
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6); // a scalar, like all that follows from it
    const int wr = wave % WR, wk = wave / WR;
    const int col = lane & 15, q = lane >> 4;

    // grid.x -> (row block, split, column block): workgroup ids that are congruent mod 8 run on one XCD and share its L2, so
    // XCD x is given a run of consecutive triples (the column blocks of a row block read the same weights, its splits write
    // partial sums that one reduction workgroup reads): the first (gridDim.x mod 8) XCDs take one triple more than the others
    uint32_t id = blockIdx.x;
    {
        const uint32_t q = gridDim.x >> 3, r = gridDim.x & 7u, x = id & 7u;
        id = x * q + (x < r ? x : r) + (id >> 3);
    }
    const uint32_t nb = id % nblocks, rest = id / nblocks, split = rest % splitK, mb = rest / splitK;
    const uint32_t nbase = nb * TN, R0 = (mb * WR + wr) * RT; // first row tile of this wavefront

    uint32_t u0 = 0, u1 = units;
    if (splitK > 1) {
        const uint32_t avg = units / splitK, extra = units % splitK;
        u0 = split * avg + (split < extra ? split : extra);
        u1 = u0 + avg + (split < extra ? 1u : 0u);
    }

    v4f acc[RT][NT];
    // row scales of this lane's outputs (rows 4q..4q+3 of each of its row tiles), fetched before the main loop so that no
    // global load sits on the tail of the kernel
    v4h sc4[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) {
        const half_t *p = scales + (R0 + r) * 16 + 4 * q;
        if ((reinterpret_cast<uintptr_t>(scales) & 7u) == 0) // uniform: one 8-byte load where the caller's pointer allows it
            sc4[r] = *reinterpret_cast<const v4h *>(p);
        else
            sc4[r] = (v4h){ p[0], p[1], p[2], p[3] };
    }

    tile_segment<FM, GS, NT, RT, WR, WK>(acc, W, gexp, X, N, K, units, mb, nbase, u0, u1, lds, tid, lane, wr, wk, col, q);

    // the output tile is parked where the partial sums of the K wavefronts met: everybody has read those first
    if (WK > 1) __syncthreads();
    uint8_t *stage = lds;
    if (splitK == 1)
        tile_store<FM, NT, RT, WR, NTHREADS>(acc, sc4, C, stage, wk == 0, M, N, mb, nbase, tid, wr, col, q);
    else
        tile_store<FM, NT, RT, WR, NTHREADS>(acc, sc4, ws + (size_t)split * N * M, stage, wk == 0, M, N, mb, nbase, tid, wr, col, q);
}

// ---------------------------------------------------------------------------------------------------------------
// gemm_ws: the tile GEMM with the wavefronts of a workgroup divided into two kinds.
//   workgroup = WR arithmetic wavefronts + PW loading wavefronts; tile = (WR*RT*16) rows x (NT*16) columns; same grid as gemm_tile
// The loading wavefronts move K blocks from memory into LDS without passing through registers (global_load_lds_dwordx4):
// the tile's weight blocks exactly as they lie in memory (native blocks of raw codes, 16-byte pieces in lane order) and the
// activation rows of the block.  The arithmetic wavefronts never touch global memory inside the K loop: they read their
// weight pieces and their B operands from LDS, convert and run the MFMAs.  In gemm_tile every wavefront does both, a
// wavefront issues its instructions in order, and the CU's memory pipeline accepts a chunk's loads at its own pace: there
// the second wavefront of every SIMD starts its MFMAs a third of a K step late, and a block has to arrive within the one
// step before it is used.  Here the weights travel SW-1 blocks ahead of the arithmetic and the activations SX-1 blocks
// (SW >= SX >= 2: the weights come from HBM, the activations from L2), during the whole of those steps.
// LDS: a ring of SW weight stages [WR*RT tiles x block bytes] and a ring of SX activation stages [NT*16 rows x 512 bytes].
// The activation rows are not padded (256 x 64 with FP6 weights and two stages each fills the 160 KB to the byte): piece p
// of row n (16 bytes) lies at slot p ^ (n & 15) of its row, which makes the operand read of eight batch columns at one K
// position touch eight different slots.  One barrier per K block: before it the loading wavefronts wait until the NEXT
// block has landed (s_waitcnt with the number of transfers issued after it: they complete in order).
// ---------------------------------------------------------------------------------------------------------------
template <int FM, int NT, int RT, int WR, int SW, int SX> constexpr size_t ws_ring_bytes()
{
    return (size_t)SW * WR * RT * Fmt<FM>::block_bytes + (size_t)SX * NT * 16 * 512;
}

template <int N> __device__ __forceinline__ void wait_transfers_and_barrier()
{
    static_assert(N >= 0 && N <= 63, "s_waitcnt vmcnt holds six bits");
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

template <int FM, bool GS, int NT, int RT, int WR, int PW, int SW, int SX>
__global__ __launch_bounds__((WR + PW) * kWave) void gemm_ws(const uint8_t *__restrict__ W, const half_t *__restrict__ scales,
                                                             const uint8_t *__restrict__ gexp, const half_t *__restrict__ X, half_t *__restrict__ C,
                                                             float *__restrict__ ws, uint32_t M, uint32_t N, uint32_t K,
                                                             uint32_t units, uint32_t splitK, uint32_t nblocks)
{
    static_assert(SW >= SX && SX >= 2, "weights run at least as far ahead as activations; a stage is filled while another is read");
    constexpr int TN = NT * 16, TILES = WR * RT, NTHREADS = (WR + PW) * kWave;
    constexpr int kBlock = Fmt<FM>::block_bytes, kWStage = TILES * kBlock, kXStage = TN * 512, kXRing = SW * kWStage; // the activation ring follows the weight ring
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    asm volatile("" ::"s"(W), "s"(scales), "s"(gexp), "s"(X), "s"(C), "s"(ws), "s"(M), "s"(N), "s"(K), "s"(units), "s"(splitK), "s"(nblocks)); // one batch of argument loads
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15, q = lane >> 4;

    // grid.x -> (row block, split, column block), every XCD a run of consecutive triples: as in gemm_tile
    uint32_t id = blockIdx.x;
    {
        const uint32_t per = gridDim.x >> 3, r = gridDim.x & 7u, x = id & 7u;
        id = x * per + (x < r ? x : r) + (id >> 3);
    }
    const uint32_t nb = id % nblocks, rest = id / nblocks, split = rest % splitK, mb = rest / splitK;
    const uint32_t nbase = nb * TN;
    uint32_t       u0 = 0, u1 = units;
    if (splitK > 1) {
        const uint32_t avg = units / splitK, extra = units % splitK;
        u0 = split * avg + (split < extra ? split : extra);
        u1 = u0 + avg + (split < extra ? 1u : 0u);
    }
    const int nk = (int)(u1 - u0); // K blocks of this workgroup, numbered 0 .. nk-1 below

    v4f acc[RT][NT];
    v4h sc4[RT];
#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int t = 0; t < NT; t++) acc[r][t] = (v4f){ 0.f, 0.f, 0.f, 0.f };

    if (wave >= WR) {
        // ---------------------------------------------------------------- loading wavefronts
        // One instruction moves 64 x 16 bytes from memory straight into 1 KB of LDS, lane l to byte 16*l of the destination;
        // each lane chooses its source address.  Instruction i of a weight (activation) stage fills its pieces 64*i .. 64*i+63;
        // this wavefront issues the instructions pw, pw + PW, ...
        typedef __attribute__((address_space(1))) void gvoid;
        typedef __attribute__((address_space(3))) void lvoid;
        const int     pw = wave - WR;
        constexpr int PB = kBlock / 16, kWPieces = TILES * PB, kXPieces = TN * 32;
        static_assert(kWPieces % 64 == 0 && kXPieces % 64 == 0, "a stage is a whole number of 1 KB instructions");
        constexpr int kWInst = kWPieces / 64, kXInst = kXPieces / 64;
        static_assert(kWInst % PW == 0 && kXInst % PW == 0, "every loading wavefront issues the same number of transfers (the waits count them)");
        constexpr int kWPer = kWInst / PW, kXPer = kXInst / PW;
        // transfers issued after those of block j+1 when step j ends: the later of its two transfers is the activation one, issued
        // SX-2 steps ago and followed there by that step's weight transfers when the weight ring is the deeper one
        constexpr int kAhead = (SW > SX ? kWPer : 0) + (SX - 2) * (kWPer + kXPer);
        // weight piece P (16 bytes) of a stage = piece P % PB of the block of tile P / PB: a straight copy
        const uint8_t *wsrc[kWPer];
#pragma unroll
        for (int j = 0; j < kWPer; j++) {
            const uint32_t P = (pw + PW * j) * 64 + lane, tile = P / PB, within = P % PB;
            wsrc[j] = W + ((size_t)(mb * TILES + tile) * units + u0) * kBlock + within * 16;
        }
        // activation piece P of a stage = slot P % 32 of row P / 32, which holds piece slot ^ (row & 15) of that batch column's
        // 256 halfs (columns beyond N repeat the last real one: their outputs are never stored)
        const uint8_t *xsrc[kXPer];
        uint32_t       xpiece[kXPer];
#pragma unroll
        for (int j = 0; j < kXPer; j++) {
            const uint32_t P = (pw + PW * j) * 64 + lane, n = P >> 5, piece = (P & 31) ^ (n & 15);
            const uint32_t row = nbase + n < N ? nbase + n : N - 1;
            xsrc[j] = reinterpret_cast<const uint8_t *>(X + (size_t)row * K + (size_t)u0 * 256) + piece * 16;
            xpiece[j] = piece;
        }
        auto fetch_w = [&](int k, int slot) { // weights of block k -> stage `slot` of the weight ring
            uint8_t *st = lds + slot * kWStage;
#pragma unroll
            for (int j = 0; j < kWPer; j++)
                __builtin_amdgcn_global_load_lds((gvoid *)(wsrc[j] + (size_t)k * kBlock), (lvoid *)(st + (pw + PW * j) * 1024), 16, 0, 0);
        };
        auto fetch_x = [&](int k, int slot) { // activations of block k -> stage `slot` of the activation ring
            uint8_t *st = lds + kXRing + slot * kXStage;
            if ((u0 + k + 1) * 256 <= K) {
#pragma unroll
                for (int j = 0; j < kXPer; j++)
                    __builtin_amdgcn_global_load_lds((gvoid *)(xsrc[j] + (size_t)k * 512), (lvoid *)(st + (pw + PW * j) * 1024), 16, 0, 0);
            } else { // the block that K cuts goes through registers: positions beyond K are read at the block's start (a valid address) and stored as zeros
#pragma unroll
                for (int j = 0; j < kXPer; j++) {
                    const bool ok = (u0 + k) * 256 + xpiece[j] * 8 < K;
                    const v4u  v = *reinterpret_cast<const v4u *>(xsrc[j] + (size_t)k * 512 - (ok ? 0u : xpiece[j] * 16));
                    *reinterpret_cast<v4u *>(st + (pw + PW * j) * 1024 + lane * 16) = ok ? v : (v4u){ 0u, 0u, 0u, 0u };
                }
            }
        };
        if (nk > 0) {
            // step j (j = -(SW-1) .. nk-1; the negative ones fill the rings) issues the activations of block j+SX-1 and then the
            // weights of block j+SW-1; it ends with a barrier before which block j+1 must have landed
            int wslot = 0, xslot = 0; // ring positions the next transfers go to
            for (int j = 1 - SW; j < nk; j++) {
                const int kx = j + SX - 1, kw = j + SW - 1;
                if (kx >= 0 && kx < nk) {
                    fetch_x(kx, xslot);
                    xslot = xslot + 1 == SX ? 0 : xslot + 1;
                }
                if (kw < nk) {
                    fetch_w(kw, wslot);
                    wslot = wslot + 1 == SW ? 0 : wslot + 1;
                }
                if (j >= -1) {
                    // the count is exact only while every transfer it assumes was issued; at the end of K wait for everything
                    // (block j+1's last transfer is followed by exactly kAhead others as long as this step still had weights to fetch)
                    if (kw < nk)
                        wait_transfers_and_barrier<kAhead>();
                    else
                        wait_transfers_and_barrier<0>();
                }
            }
        }
    } else {
        // ---------------------------------------------------------------- arithmetic wavefronts
        const int      wr = wave;
        const uint32_t R0 = (mb * WR + wr) * RT; // first row tile of this wavefront
#pragma unroll
        for (int r = 0; r < RT; r++) {
            const half_t *p = scales + (R0 + r) * 16 + 4 * q;
            if ((reinterpret_cast<uintptr_t>(scales) & 7u) == 0)
                sc4[r] = *reinterpret_cast<const v4h *>(p);
            else
                sc4[r] = (v4h){ p[0], p[1], p[2], p[3] };
        }
        const uint8_t *ggroup = GS ? gexp + ((size_t)R0 * units + u0) * 32 : nullptr;
        uint32_t       xoff[8]; // B operand of MFMA step s: row col, piece 4s+q, at its swizzled slot
#pragma unroll
        for (int s8 = 0; s8 < 8; s8++) xoff[s8] = kXRing + col * 512 + 16 * ((4 * s8 + q) ^ col);
        const uint32_t woff = wr * RT * kBlock + lane * 16;
        if (nk > 0) {
            uint32_t gnext[RT];
#pragma unroll
            for (int r = 0; r < RT; r++) gnext[r] = load_group_exps<GS>(ggroup, (size_t)r * units, lane);
            __syncthreads(); // block 0 has landed
            int wslot = 0, xslot = 0;
            for (int k = 0; k < nk; k++) {
                const uint8_t *wst = lds + wslot * kWStage, *xst = lds + xslot * kXStage;
                wslot = wslot + 1 == SW ? 0 : wslot + 1;
                xslot = xslot + 1 == SX ? 0 : xslot + 1;
                WFrag<FM> wf[RT];
                uint32_t  g[RT];
#pragma unroll
                for (int r = 0; r < RT; r++) {
                    const uint8_t *b = wst + woff + r * kBlock;
                    wf[r].a = *reinterpret_cast<const v4u *>(b);
                    wf[r].b = *reinterpret_cast<const v4u *>(b + 1024);
                    if constexpr (Fmt<FM>::bits == 6) wf[r].c = *reinterpret_cast<const v4u *>(b + 2048);
                    if constexpr (Fmt<FM>::bits == 5) wf[r].s = *reinterpret_cast<const v2u *>(wst + (wr * RT + r) * kBlock + 2048 + lane * 8);
                    g[r] = gnext[r];
                    if (GS && k + 1 < nk) gnext[r] = load_group_exps<GS>(ggroup, (size_t)r * units + k + 1, lane);
                }
                v8h a0[RT][4], a1[RT][4];
#pragma unroll
                for (int r = 0; r < RT; r++) convert_half<FM, GS>(wf[r], 0, a0[r], g[r]);
#pragma unroll
                for (int r = 0; r < RT; r++) convert_half<FM, GS>(wf[r], 1, a1[r], g[r]);
#pragma unroll
                for (int h = 0; h < 2; h++) {
#pragma unroll
                    for (int s = 0; s < 4; s++) {
                        v8h b[NT];
#pragma unroll
                        for (int t = 0; t < NT; t++) b[t] = *reinterpret_cast<const v8h *>(xst + xoff[4 * h + s] + t * 16 * 512);
#pragma unroll
                        for (int r = 0; r < RT; r++)
#pragma unroll
                            for (int t = 0; t < NT; t++)
                                acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(h == 0 ? a0[r][s] : a1[r][s], b[t], acc[r][t], 0, 0, 0);
                    }
                }
                __syncthreads();
            }
        }
    }
    // every wavefront has passed the last barrier of the K loop: the rings are free, the output tile is parked there
    uint8_t *stage = lds;
    if (splitK == 1) {
        if (wave < WR) tile_park<FM, NT, RT, WR, half_t>(acc, sc4, stage, wave, col, q);
        __syncthreads();
        tile_flush<NT, RT, WR, NTHREADS, half_t>(C, stage, M, N, mb, nbase, tid);
    } else {
        if (wave < WR) tile_park<FM, NT, RT, WR, float>(acc, sc4, stage, wave, col, q);
        __syncthreads();
        tile_flush<NT, RT, WR, NTHREADS, float>(ws + (size_t)split * N * M, stage, M, N, mb, nbase, tid);
    }
}

// Native layout -> fp16 [M,K], with the GEMM's own conversion code.  One lane per (row tile, K block, lane) triple.
template <int FM, bool GS>
__global__ __launch_bounds__(256) void dequant_native(half_t *__restrict__ out, const uint8_t *__restrict__ W, const half_t *__restrict__ scales,
                                                     const uint8_t *__restrict__ gexp, uint32_t M, uint32_t K, uint32_t units)
{
    const int      lane = threadIdx.x & 63;
    const uint32_t blk = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= (M / 16) * units) return;
    const uint32_t R = blk / units, U = blk % units;
    const int      m = lane & 15, q = lane >> 4;
    WFrag<FM>      wf = load_wfrag<FM>(W + (size_t)blk * Fmt<FM>::block_bytes, lane);
    AOps<FM>       a;
    convert<FM, GS>(wf, a, load_group_exps<GS>(gexp, blk, lane));
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
//                code, with the sign bit of w.  NaN weights become +0, +-Inf saturates, and neither takes part in absmax.
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

// |v| for finite v, 0 for NaN and +-Inf: neither sets a scale
__device__ __forceinline__ float finite_abs(float v)
{
    const float a = fabsf(v);
    return a <= 3.4028234663852886e38f ? a : 0.f;
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
        for (int j = 0; j < 8; j++) amax = fmaxf(amax, finite_abs(to_float<T>(p[k + j])));
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

// gexp (native order) non-null: besides the row scale every group of 128 columns of a row gets the smallest factor 2^k,
// -15 <= k <= 0, that still holds its largest magnitude, stored as the byte 127 + k, and its codes are chosen against
// scale * 2^k.  A wavefront's lanes (m, q = 0..3) hold the group's 128 values between them, 32 each.
template <int FM, typename T>
__global__ __launch_bounds__(256) void quant_to_native(uint8_t *__restrict__ native, const half_t *__restrict__ scales, uint8_t *__restrict__ gexp,
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
    double         factor[2] = { sc, sc };
    if (gexp) { // uniform
        for (int h = 0; h < 2; h++) {
            float amax = 0.f;
            for (int s = 4 * h; s < 4 * h + 4; s++) {
                const uint32_t k0 = U * 256 + 32 * s + 8 * q;
                for (int j = 0; j < 8; j++)
                    if (k0 + j < K) amax = fmaxf(amax, finite_abs(to_float<T>(p[k0 + j])));
            }
            amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
            amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
            const double gmax = (double)amax / sc;
            int          k = -15;
            while (k < 0 && !(gmax <= scalbn(max_value, k))) k++;
            if (U * 256 + 128 * h >= K) k = 0; // a half block beyond K: factor 1 by convention
            factor[h] = scalbn(sc, k);
            if (q == 0) gexp[((size_t)blk * 16 + m) * 2 + h] = (uint8_t)(127 + k);
        }
    }
    uint8_t c[64];
#pragma unroll 1
    for (int s = 0; s < 8; s++) {
        const uint32_t k0 = U * 256 + 32 * s + 8 * q;
        const double   f = factor[s >> 2];
        for (int j = 0; j < 8; j++) {
            uint32_t code = 0;
            if (k0 + j < K) {
                float  w = to_float<T>(p[k0 + j]);
                double a = fabs((double)w / f);
                if (a > max_value) a = max_value; // clamps; +-Inf saturates
                if (w == w) code = nearest_magnitude<FM>(a) | ((__builtin_bit_cast(uint32_t, w) >> 31) << (Fmt<FM>::bits - 1)); // NaN: +0
            }
            c[8 * s + j] = (uint8_t)code;
        }
    }
    store_native_lane<FM>(c, native + (size_t)blk * Fmt<FM>::block_bytes, lane);
}
// ------------------------------------------------------------------------------------------------ launch helpers

// Lets `Kernel` use up to `bytes` of dynamic LDS.  The attribute belongs to the device's copy of the kernel: set once per device.
template <auto Kernel> int allow_dynamic_lds(size_t bytes)
{
    static std::atomic<uint64_t> attr_set{ 0 }; // bit d: done on device d; setting it twice is harmless, so no lock
    int                          dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
    const uint64_t bit = dev >= 0 && dev < 64 ? 1ull << dev : 0;
    if (!(attr_set.load(std::memory_order_relaxed) & bit)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) return (int)e;
        attr_set.fetch_or(bit, std::memory_order_relaxed);
    }
    return 0;
}

template <int FM, bool GS, int NT, int RT, int WAVES>
int launch_stream(hipStream_t st, const void *W, const void *sc, const void *gexp, const void *B, void *C, float *ws, size_t M, size_t N, size_t K,
                  int splitK)
{
    constexpr size_t kMaxLds = (size_t)WAVES * stream_wave_bytes(16 * NT, RT, NT);
    static_assert(kMaxLds <= 160 * 1024, "the wavefronts' activation rows do not fit in LDS");
    uint32_t     units = (uint32_t)((K + 255) / 256);
    dim3         grid((uint32_t)((M / 16 + RT - 1) / RT), (uint32_t)splitK, (uint32_t)((N + 16 * NT - 1) / (16 * NT)));
    const size_t lds_bytes = NT == 1 && N <= 8 ? (size_t)WAVES * stream_wave_bytes(8, RT, NT) : kMaxLds;
    auto         go = [&](auto kernel_c) -> int {
        constexpr auto kernel = decltype(kernel_c)::value;
        if (kMaxLds > 48 * 1024)
            if (int rc = allow_dynamic_lds<kernel>(kMaxLds)) return rc;
        hipLaunchKernelGGL(kernel, grid, dim3(WAVES * kWave), lds_bytes, st, static_cast<const uint8_t *>(W), static_cast<const half_t *>(sc),
                           static_cast<const uint8_t *>(gexp), static_cast<const half_t *>(B), static_cast<half_t *>(C), ws, (uint32_t)M, (uint32_t)N,
                           (uint32_t)K, units, (uint32_t)splitK);
        return (int)hipGetLastError();
    };
    if (splitK > 1) return go(std::integral_constant<decltype(&gemm_stream<FM, GS, NT, RT, WAVES, true>), &gemm_stream<FM, GS, NT, RT, WAVES, true>>{});
    return go(std::integral_constant<decltype(&gemm_stream<FM, GS, NT, RT, WAVES, false>), &gemm_stream<FM, GS, NT, RT, WAVES, false>>{});
}

template <int FM, bool GS, int NT, int RT, int WR, int WK>
int launch_tile(hipStream_t st, const void *W, const void *sc, const void *gexp, const void *B, void *C, float *ws, size_t M, size_t N, size_t K,
                int splitK)
{
    constexpr int TN = NT * 16, TM = WR * RT * 16;
    constexpr size_t x_bytes = 2 * (size_t)WK * TN * kXsRowBytes, red_bytes = WK > 1 ? (size_t)WK * WR * RT * NT * 1024 : 0;
    constexpr size_t kLoopLds = x_bytes > red_bytes ? x_bytes : red_bytes, out_max = tile_stage_bytes<NT, RT, WR>(true);
    constexpr size_t kMaxLds = kLoopLds > out_max ? kLoopLds : out_max;
    static_assert(kMaxLds <= 160 * 1024, "tile does not fit in LDS");
    const size_t out_bytes = tile_stage_bytes<NT, RT, WR>(splitK > 1), lds_bytes = kLoopLds > out_bytes ? kLoopLds : out_bytes;
    if (M % TM) return FP6MI_ERR_SHAPE;
    if (kMaxLds > 48 * 1024)
        if (int rc = allow_dynamic_lds<&gemm_tile<FM, GS, NT, RT, WR, WK>>(kMaxLds)) return rc;
    uint32_t units = (uint32_t)((K + 255) / 256), nblocks = (uint32_t)((N + TN - 1) / TN);
    size_t   wgs = (M / TM) * (size_t)splitK * nblocks;
    if (wgs > 0x7fffffffu) return FP6MI_ERR_SHAPE;
    hipLaunchKernelGGL((gemm_tile<FM, GS, NT, RT, WR, WK>), dim3((uint32_t)wgs), dim3(WR * WK * kWave), lds_bytes, st,
                       static_cast<const uint8_t *>(W), static_cast<const half_t *>(sc), static_cast<const uint8_t *>(gexp), static_cast<const half_t *>(B),
                       static_cast<half_t *>(C), ws, (uint32_t)M, (uint32_t)N, (uint32_t)K, units, (uint32_t)splitK, nblocks);
    return (int)hipGetLastError();
}
template <int FM, bool GS, int NT, int RT, int WR, int PW, int SW, int SX>
int launch_ws(hipStream_t st, const void *W, const void *sc, const void *gexp, const void *B, void *C, float *ws, size_t M, size_t N, size_t K,
              int splitK)
{
    constexpr int    TN = NT * 16, TM = WR * RT * 16;
    constexpr size_t kLoopLds = ws_ring_bytes<FM, NT, RT, WR, SW, SX>(), out_max = tile_stage_bytes<NT, RT, WR>(true);
    constexpr size_t kMaxLds = kLoopLds > out_max ? kLoopLds : out_max;
    static_assert(kMaxLds <= 160 * 1024, "the rings do not fit in LDS");
    static_assert((WR + PW) * kWave <= 1024, "too many wavefronts");
    // a weight stage must be a whole number of 1 KB transfers per loading wavefront (FP5 blocks are 2.5 KB: 64-row tiles are out)
    constexpr bool kDivides = (WR * RT * Fmt<FM>::block_bytes) % (1024 * PW) == 0 && (TN * 512) % (1024 * PW) == 0;
    if constexpr (!kDivides) {
        return FP6MI_ERR_SHAPE;
    } else {
        const size_t out_bytes = tile_stage_bytes<NT, RT, WR>(splitK > 1), lds_bytes = kLoopLds > out_bytes ? kLoopLds : out_bytes;
        if (M % TM) return FP6MI_ERR_SHAPE;
        if (kMaxLds > 48 * 1024)
            if (int rc = allow_dynamic_lds<&gemm_ws<FM, GS, NT, RT, WR, PW, SW, SX>>(kMaxLds)) return rc;
        uint32_t units = (uint32_t)((K + 255) / 256), nblocks = (uint32_t)((N + TN - 1) / TN);
        size_t   wgs = (M / TM) * (size_t)splitK * nblocks;
        if (wgs > 0x7fffffffu) return FP6MI_ERR_SHAPE;
        hipLaunchKernelGGL((gemm_ws<FM, GS, NT, RT, WR, PW, SW, SX>), dim3((uint32_t)wgs), dim3((WR + PW) * kWave), lds_bytes, st,
                           static_cast<const uint8_t *>(W), static_cast<const half_t *>(sc), static_cast<const uint8_t *>(gexp), static_cast<const half_t *>(B),
                           static_cast<half_t *>(C), ws, (uint32_t)M, (uint32_t)N, (uint32_t)K, units, (uint32_t)splitK, nblocks);
        return (int)hipGetLastError();
    }
}
// kind 0: gemm_stream (wr == 1, wk = wavefronts per workgroup);  kind 1: gemm_tile (wr x wk wavefronts);  kind 2: gemm_ws (wr arithmetic + wk loading wavefronts)
template <int FM, bool GS>
int launch_cfg(const LaunchCfg &c, hipStream_t st, const void *W, const void *sc, const void *gexp, const void *B, void *C, float *ws, size_t M,
               size_t N, size_t K, int splitK)
{
    if (c.kind == 0) {
#define FP6MI_CASE(NT, RT, WV) \
    if (c.nt == NT && c.rt == RT && c.wk == WV && c.wr == 1) return launch_stream<FM, GS, NT, RT, WV>(st, W, sc, gexp, B, C, ws, M, N, K, splitK);
        FP6MI_CASE(1, 1, 4) FP6MI_CASE(1, 1, 8) FP6MI_CASE(1, 1, 16)
        FP6MI_CASE(1, 2, 4) FP6MI_CASE(1, 2, 8) FP6MI_CASE(1, 2, 16)
        FP6MI_CASE(1, 3, 4) FP6MI_CASE(1, 3, 8)
        FP6MI_CASE(1, 4, 4) FP6MI_CASE(1, 4, 8)
        FP6MI_CASE(1, 5, 4) FP6MI_CASE(1, 5, 8) FP6MI_CASE(1, 6, 4) FP6MI_CASE(1, 6, 8) FP6MI_CASE(1, 7, 4) FP6MI_CASE(1, 8, 4)
        FP6MI_CASE(2, 1, 4) FP6MI_CASE(2, 1, 8)
        FP6MI_CASE(2, 2, 4) FP6MI_CASE(2, 2, 8)
        FP6MI_CASE(2, 3, 4) FP6MI_CASE(2, 3, 8)
        FP6MI_CASE(2, 4, 4) FP6MI_CASE(2, 4, 8)
        FP6MI_CASE(2, 5, 4) FP6MI_CASE(2, 5, 8) FP6MI_CASE(2, 6, 4) FP6MI_CASE(2, 7, 4) FP6MI_CASE(2, 8, 4)
#undef FP6MI_CASE
    } else if (c.kind == 1) {
#define FP6MI_CASE(NT, RT, WR, WK) \
    if (c.nt == NT && c.rt == RT && c.wr == WR && c.wk == WK) return launch_tile<FM, GS, NT, RT, WR, WK>(st, W, sc, gexp, B, C, ws, M, N, K, splitK);
        FP6MI_CASE(2, 1, 4, 4) FP6MI_CASE(2, 2, 4, 4) FP6MI_CASE(2, 2, 4, 2) FP6MI_CASE(2, 2, 4, 1) FP6MI_CASE(2, 4, 4, 1) FP6MI_CASE(2, 4, 4, 2)
        FP6MI_CASE(4, 2, 4, 2) FP6MI_CASE(4, 2, 4, 1) FP6MI_CASE(4, 4, 4, 1) FP6MI_CASE(4, 4, 2, 1) FP6MI_CASE(4, 4, 2, 2)
        FP6MI_CASE(8, 2, 4, 1) FP6MI_CASE(8, 2, 2, 1) FP6MI_CASE(4, 2, 8, 1) FP6MI_CASE(4, 2, 8, 2) FP6MI_CASE(2, 2, 8, 1) FP6MI_CASE(2, 2, 8, 2) FP6MI_CASE(8, 2, 8, 1) FP6MI_CASE(4, 1, 8, 2) FP6MI_CASE(4, 1, 8, 1) FP6MI_CASE(4, 1, 4, 2) FP6MI_CASE(2, 1, 2, 4)
#undef FP6MI_CASE
    } else if (c.kind == 2) {
        // ring depths (2,2): deeper rings on smaller tiles (128 x 64 with (4,2), 128 x 32 and 64 x 64 with (4,3)) measured no faster than
        // gemm_tile at batches 32-64, where the time goes to the partial sums and the second launch, and are not built
#define FP6MI_CASE(NT, RT, WR, PW) \
    if (c.nt == NT && c.rt == RT && c.wr == WR && c.wk == PW) return launch_ws<FM, GS, NT, RT, WR, PW, 2, 2>(st, W, sc, gexp, B, C, ws, M, N, K, splitK);
        FP6MI_CASE(4, 2, 8, 4) FP6MI_CASE(4, 2, 4, 4) FP6MI_CASE(2, 2, 8, 4)
#undef FP6MI_CASE
    }
    return FP6MI_ERR_SHAPE;
}

// ------------------------------------------------------------------------------------------------ entry functions of this format
// (arguments are checked by the C ABI before it comes here)
// gexp: group exponents in their native layout, or null for none
template <int FM>
int op_gemm(const LaunchCfg &c, void *stream, const void *W, const void *sc, const void *gexp, const void *B, void *C, float *ws, size_t M,
            size_t N, size_t K, int splitK)
{
    hipStream_t st = static_cast<hipStream_t>(stream);
    return gexp ? launch_cfg<FM, true>(c, st, W, sc, gexp, B, C, ws, M, N, K, splitK) : launch_cfg<FM, false>(c, st, W, sc, nullptr, B, C, ws, M, N, K, splitK);
}

template <int FM> int op_relayout(void *stream, void *native, const void *ref, size_t M, size_t K)
{
    uint32_t units = (uint32_t)((K + 255) / 256);
    size_t   blocks = (M / 16) * units;
    hipLaunchKernelGGL(relayout_ref_to_native<FM>, dim3((uint32_t)((blocks + 3) / 4)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint8_t *>(native), static_cast<const uint8_t *>(ref), (uint32_t)M, (uint32_t)K, units);
    return (int)hipGetLastError();
}

template <int FM> int op_dequant(void *stream, void *out, const void *W, const void *sc, const void *gexp, size_t M, size_t K)
{
    uint32_t    units = (uint32_t)((K + 255) / 256);
    size_t      blocks = (M / 16) * units;
    dim3        grid((uint32_t)((blocks + 3) / 4));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (gexp)
        hipLaunchKernelGGL((dequant_native<FM, true>), grid, dim3(256), 0, st, static_cast<half_t *>(out), static_cast<const uint8_t *>(W),
                           static_cast<const half_t *>(sc), static_cast<const uint8_t *>(gexp), (uint32_t)M, (uint32_t)K, units);
    else
        hipLaunchKernelGGL((dequant_native<FM, false>), grid, dim3(256), 0, st, static_cast<half_t *>(out), static_cast<const uint8_t *>(W),
                           static_cast<const half_t *>(sc), static_cast<const uint8_t *>(nullptr), (uint32_t)M, (uint32_t)K, units);
    return (int)hipGetLastError();
}

// dtype: 0 = fp16, 1 = bf16, 2 = fp32
template <int FM> int op_quantize(void *stream, void *native, void *scales, void *gexp, const void *weights, int dtype, size_t M, size_t K)
{
    const uint32_t   units = (uint32_t)((K + 255) / 256);
    const size_t     blocks = (M / 16) * units;
    const dim3       grid_rows((uint32_t)((M + 3) / 4)), grid_blocks((uint32_t)((blocks + 3) / 4));
    constexpr double max_value = Fmt<FM>::max_value;
    hipStream_t      st = static_cast<hipStream_t>(stream);
    uint8_t         *nat = static_cast<uint8_t *>(native);
    half_t          *sc = static_cast<half_t *>(scales);
    auto             run = [&](auto *typed) {
        typedef std::remove_cv_t<std::remove_pointer_t<decltype(typed)>> T;
        hipLaunchKernelGGL(quant_row_scales<T>, grid_rows, dim3(256), 0, st, sc, typed, (uint32_t)M, (uint32_t)K, max_value);
        hipLaunchKernelGGL((quant_to_native<FM, T>), grid_blocks, dim3(256), 0, st, nat, sc, static_cast<uint8_t *>(gexp), typed, (uint32_t)M,
                           (uint32_t)K, units, max_value);
    };
    if (dtype == 0)
        run(static_cast<const half_t *>(weights));
    else if (dtype == 1)
        run(static_cast<const bf16_t *>(weights));
    else
        run(static_cast<const float *>(weights));
    return (int)hipGetLastError();
}

} // namespace

namespace fp6mi {
#define FP6MI_OPS_NAME_(f) format_ops_##f
#define FP6MI_OPS_NAME(f) FP6MI_OPS_NAME_(f)
const FormatOps &FP6MI_OPS_NAME(FP6MI_FORMAT)() // a host function, so that the table of host pointers stays out of the device code
{
    static const FormatOps ops = { Fmt<FP6MI_FORMAT>::bits, &op_gemm<FP6MI_FORMAT>, &op_relayout<FP6MI_FORMAT>, &op_dequant<FP6MI_FORMAT>,
                                   &op_quantize<FP6MI_FORMAT> };
    return ops;
}
} // namespace fp6mi
