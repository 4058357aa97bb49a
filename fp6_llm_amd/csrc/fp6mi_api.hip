// C ABI of the FPx x FP16 linear-layer engine (include/fp6mi.h), the choice of the launch shape, and the split-K reduction.
// The kernels live in fp6mi_gemm.hip, compiled once per weight format; this file reaches them through fp6mi::FormatOps.
//
// Roles taken over from the reference (usyd-fsalab/fp6_llm, paths relative to it):
//   splitk_reduce      <- SplitK_Reduction        fp6_llm/csrc/include/kernel_reduction.cuh:28-47
//   pick_cfg           <- the N bucketing of      fp6_llm/csrc/fp6_linear.cu:58-99
//   fp6mi_linear*      <- fpx_linear_kernel       fp6_llm/csrc/fp6_linear.cu:44-102
#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>
#include <type_traits>
#include <unordered_map>
#include <vector>

#include "fp6mi_internal.h"

namespace {

typedef _Float16 half_t;
typedef float    v4f __attribute__((ext_vector_type(4)));

using fp6mi::LaunchCfg;

// C[i] = fp16_rn(sum over splits, in split order, of ws[s][i]) for the four outputs from index i.
__device__ __forceinline__ void reduce_four(half_t *__restrict__ C, const float *__restrict__ ws, size_t MN, int splitK, size_t i)
{
    v4f sum = { 0.f, 0.f, 0.f, 0.f };
    // up to eight loads in flight instead of one round trip to memory per split; the order of the sum is unchanged.  The
    // remainder after the groups of eight is one group of its exact size (a 3 done as 2 + 1 would be two round trips).
    auto chunk = [&](auto count, int s0) {
        constexpr int C = decltype(count)::value;
        v4f           part[C];
#pragma unroll
        for (int k = 0; k < C; k++) part[k] = *reinterpret_cast<const v4f *>(ws + (size_t)(s0 + k) * MN + i);
#pragma unroll
        for (int k = 0; k < C; k++) sum += part[k];
    };
    int s = 0;
    for (; s + 8 <= splitK; s += 8) chunk(std::integral_constant<int, 8>{}, s);
    switch (splitK - s) {
    case 7: chunk(std::integral_constant<int, 7>{}, s); break;
    case 6: chunk(std::integral_constant<int, 6>{}, s); break;
    case 5: chunk(std::integral_constant<int, 5>{}, s); break;
    case 4: chunk(std::integral_constant<int, 4>{}, s); break;
    case 3: chunk(std::integral_constant<int, 3>{}, s); break;
    case 2: chunk(std::integral_constant<int, 2>{}, s); break;
    case 1: chunk(std::integral_constant<int, 1>{}, s); break;
    default: break;
    }
    typedef _Float16 v4h __attribute__((ext_vector_type(4)));
    v4h o = { (half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3] };
    *reinterpret_cast<v4h *>(C + i) = o;
}

// four outputs per thread, in the order of the output
__global__ __launch_bounds__(256) void splitk_reduce(half_t *__restrict__ C, const float *__restrict__ ws, size_t MN, int splitK)
{
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i < MN) reduce_four(C, ws, MN, splitK, i);
}

// The same sums with the workgroups placed where the partial sums were written.  gemm_tile hands XCD x (workgroup ids
// congruent to x mod 8) the consecutive (row block, split, column block) triples from start(x) = x * q + min(x, r) on, where
// q = grid / 8 and r = grid mod 8, i.e. the row blocks from start(x) / per_block (per_block = splits x column blocks; a row block
// cut by the boundary counts for the later XCD).  Workgroup b of this kernel also runs on XCD b mod 8 and takes the rows that
// XCD produced, for every batch column: its loads hit the L2 that the partial sums were written through, where the
// output-order kernel above finds most of them behind another XCD's L2 (measured: 4 MB written by one kernel are read by
// the next in 0.7 us from the writer's XCD and in 2.6 us from another).
__global__ __launch_bounds__(256) void splitk_reduce_by_xcd(half_t *__restrict__ C, const float *__restrict__ ws, uint32_t M, uint32_t N, int splitK,
                                                             uint32_t tile_rows, uint32_t q, uint32_t r, uint32_t per_block)
{
    const uint32_t x = blockIdx.x & 7u, j = blockIdx.x >> 3;
    const uint32_t s0 = x * q + (x < r ? x : r), s1 = (x + 1) * q + (x + 1 < r ? x + 1 : r);
    const uint32_t lo = s0 / per_block * tile_rows, hi = s1 / per_block * tile_rows, quads = (hi - lo) / 4;
    const uint32_t g = j * 256 + threadIdx.x;
    if (g >= quads * N) return;
    const uint32_t n = g / quads, m = lo + (g - n * quads) * 4;
    reduce_four(C, ws, (size_t)M * N, splitK, (size_t)n * M + m);
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Compute units of the current device, asked of the runtime once per device (the launch-shape rules and the measured table
// are written for 256; another count takes the rules).
int current_device_cus()
{
    static std::atomic<int> cus[64];
    int                     dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

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
constexpr int kSplits[] = { 1, 2, 3, 4, 6, 8 };                             // the splits the table knows
constexpr int kNumSplits = sizeof(kSplits) / sizeof(kSplits[0]);
inline int split_index(int splitK) { for (int i = 0; i < kNumSplits; i++) if (kSplits[i] == splitK) return i; return -1; }
struct TuneEntry { uint8_t xb; uint16_t m256, k64, n; TuneCfg sk[kNumSplits]; };    // sk[i]: best shape for splitK = kSplits[i]
const TuneEntry kTune[] = {
    { 0, 0, 0, 0, { { 255, 0, 0, 0, 0, 0 }, { 255, 0, 0, 0, 0, 0 }, { 255, 0, 0, 0, 0, 0 }, { 255, 0, 0, 0, 0, 0 }, { 255, 0, 0, 0, 0, 0 }, { 255, 0, 0, 0, 0, 0 } } }, // keeps the array non-empty
#include "fp6mi_tuning.inc"
};

// (the stream kernel takes any number of row tiles per workgroup for any M: its last workgroup may hold fewer)
inline bool cfg_fits(const TuneCfg &c, size_t M) { return c.kind != 255 && (c.kind == 0 || M % (16u * c.rt * c.wr) == 0); }

// What the table says about a problem that need not be in it: per splitK the shape expected to be fastest and its expected
// time.  The batch is rounded UP to a measured batch of the same kernel family (a shape's cost steps at column-tile
// boundaries).  A measured (M, K) answers for itself; otherwise the up to four nearest measured problems (in ratio, at most a
// factor 1.5 away in M and in K) each propose their best shape per splitK, and a proposal's time is carried over to the
// query: in proportion to K, and for M by the number of rounds the shape's workgroups need on the chip.  Two matrices with
// 16384 and 17920 rows differ by 9 % in size but by a whole round of 64-row workgroups; sweeps off the grid showed that
// this, not the distance, decides which neighbour's shape is right.  Farther neighbours pay 15 % per octave of distance.
struct TuneGroup { int xb; size_t n, begin, end; }; // entries [begin, end) of kTune share format and batch (the table is sorted by them)
struct TuneAnswer { bool valid, measured; LaunchCfg cfg[kNumSplits]; float t[kNumSplits]; }; // index i: splitK = kSplits[i]; t in 0.02 us, 0 = no proposal; measured: this very (M, K) at this or the next larger measured batch

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

inline double rounds_on_chip(const TuneCfg &c, size_t M, size_t N, int splitK)
{
    const size_t TM = (size_t)(c.kind >= 1 ? c.wr : 1) * c.rt * 16, TN = (size_t)c.nt * 16;
    const double wgs = (double)((M + TM - 1) / TM) * (double)((N + TN - 1) / TN) * splitK;
    // tile kernel: one workgroup per CU, two for four-wavefront workgroups.  Stream kernel: several workgroups share a CU, but
    // they share its memory pipeline too, so what counts is the largest number of workgroups any CU is given.
    const double slots = 256.0 * (c.kind == 1 && c.wr * c.wk <= 4 ? 2 : 1);
    return std::ceil(wgs / slots);
}

const TuneAnswer *tune_lookup(int xbits, size_t M, size_t N, size_t K)
{
    // a serving loop asks for the same few layer shapes at whatever batch size the scheduler formed: remember answers
    struct Memo { int xb; size_t M, N, K; TuneAnswer a; };
    static thread_local Memo memo[256];
    Memo &slot = memo[(M * 0x9E3779B97F4A7C15ull + N * 0xC2B2AE3D27D4EB4Full + K * 0x165667B19E3779F9ull + (size_t)xbits) >> 56];
    if (slot.xb == xbits && slot.M == M && slot.N == N && slot.K == K) return slot.a.valid ? &slot.a : nullptr;
    const TuneGroup *group = nullptr, *widest = nullptr;
    for (const TuneGroup &g : tune_groups()) {
        if (g.xb != xbits || (g.n <= 16) != (N <= 16)) continue;
        if (g.n >= N && (!group || g.n < group->n)) group = &g;
        if (!widest || g.n > widest->n) widest = &g;
    }
    if (!group) group = widest; // batches beyond the largest measured one behave like it, only with more column blocks
    constexpr int    kNear = 4;
    const TuneEntry *near[kNear] = {};
    float            dist[kNear] = {};
    int              count = 0;
    if (group) {
        const float lm = std::log2((float)M / 256.f), lk = std::log2((float)K / 64.f);
        for (size_t i = group->begin; i < group->end; i++) {
            const TuneEntry &e = kTune[i];
            float dm = std::fabs(lm - std::log2((float)e.m256)), dk = std::fabs(lk - std::log2((float)e.k64));
            if (dm > 0.585f || dk > 0.585f) continue;
            int pos = count < kNear ? count : kNear - 1; // insertion into the sorted list of the nearest
            if (count == kNear && dm + dk >= dist[pos]) continue;
            while (pos > 0 && dist[pos - 1] > dm + dk) { near[pos] = near[pos - 1]; dist[pos] = dist[pos - 1]; pos--; }
            near[pos] = &e, dist[pos] = dm + dk;
            if (count < kNear) count++;
        }
    }
    TuneAnswer a = {};
    if (count > 0 && dist[0] == 0.f) count = 1, a.measured = true; // measured: nothing to carry over
    const size_t units = (K + 255) / 256;
    for (int j = 0; j < count; j++) {
        const TuneEntry &e = *near[j];
        const size_t     Me = (size_t)e.m256 * 256, Ke = (size_t)e.k64 * 64, Nq = N > group->n ? N : group->n;
        for (int i = 0; i < kNumSplits; i++) {
            const TuneCfg &c = e.sk[i];
            if (!cfg_fits(c, M) || (size_t)kSplits[i] > units) continue;
            double t = (double)c.t * (double)K / (double)Ke * (1.0 + 0.15 * dist[j]);
            t *= rounds_on_chip(c, M, Nq, kSplits[i]) / rounds_on_chip(c, Me, group->n, kSplits[i]);
            if (a.t[i] == 0.f || (float)t < a.t[i]) {
                a.t[i] = (float)t;
                a.cfg[i] = LaunchCfg{ c.kind, c.nt, c.rt, c.wr, c.wk };
                a.valid = true;
            }
        }
    }
    slot = Memo{ xbits, M, N, K, a };
    return a.valid ? &slot.a : nullptr;
}

// Launch shape for a given splitK.
//  N <= 16: stream kernel.  Row tiles per wavefront (rt) reuse the activation registers, so rt grows with M; wavefronts
//           per workgroup follow the K blocks of one split and the register budget (16 wavefronts leave 128 VGPRs each).
//  N > 16:  tile kernel, 128 rows x 32 or 64 columns, with the K parallelism that splitK leaves open given to the
//           wavefronts of the workgroup (at most what its LDS holds).
inline LaunchCfg pick_cfg(int xbits, size_t M, size_t N, size_t K, int splitK, int cus)
{
    LaunchCfg c;
    if (const int i = split_index(splitK); cus == 256 && i >= 0) {
        if (const TuneAnswer *a = tune_lookup(xbits, M, N, K)) {
            if (a->t[i] > 0.f) return a->cfg[i];
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
        } else {
            // Batches 5..16: every row tile a workgroup adds re-uses its activation registers, and a CU is done when its last
            // workgroup is, so give each CU its share of the row tiles in as few workgroups as hold them (at most eight tiles):
            // cost of rt tiles per workgroup = rounds of the 256 CUs x rt.  10240, 11008 and 12288 rows take 3, 17920 and 19968
            // rows 5, 22016 rows 6, 28672 rows 7 (measured: 5-20 % better than the power of two next to them).  Ties go to the
            // larger workgroup (12288 rows: three tiles at once beat three workgroups of one by 7 %).
            int    best = 1;
            size_t best_cost = ~(size_t)0;
            for (int rt = 1; rt <= 8; rt++) {
                const size_t wgs = (tiles + rt - 1) / rt * splitK, cost = (wgs + cus - 1) / cus * rt;
                if (cost <= best_cost) best = rt, best_cost = cost;
            }
            c.rt = best;
            c.wk = best >= 5 || (best == 4 && N > 8) ? 4 : 8;
        }
        while ((c.rt == 2 || c.rt == 4 || c.rt == 8) && tiles % c.rt) c.rt /= 2; // (the other counts need not divide: the last workgroup holds the rest)
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
int linear_native(const fp6mi::FormatOps &ops, hipStream_t st, const void *W, const void *sc, const void *gexp, const void *B, void *C, size_t M, size_t N, size_t K, float *ws,
                  int splitK, const LaunchCfg *forced)
{
    LaunchCfg c = forced ? *forced : pick_cfg(ops.bits, M, N, K, splitK, current_device_cus());
    if (c.kind == 0 && !(c.rt & (c.rt - 1)) && (M / 16) % c.rt) return FP6MI_ERR_SHAPE; // (3, 5, 6, 7 tiles per workgroup end in a workgroup with fewer)
    int rc = ops.gemm(c, st, W, sc, gexp, B, C, ws, M, N, K, splitK);
    if (rc != 0) return rc;
    if (splitK > 1) {
        size_t MN = M * N; // M % 256 == 0, so MN % 4 == 0
        const size_t tile_rows = (size_t)c.wr * c.rt * 16, nblocks = (N + (size_t)c.nt * 16 - 1) / ((size_t)c.nt * 16);
        const size_t grid = c.kind >= 1 && M % tile_rows == 0 ? M / tile_rows * nblocks * splitK : 0; // gemm_tile and gemm_ws share the tile order
        if (grid && MN / 4 < ((size_t)1 << 31)) {
            // gemm_tile gave every XCD a run of consecutive triples: reduce where the partial sums lie
            const uint32_t q = (uint32_t)(grid / 8), r = (uint32_t)(grid % 8), per_block = (uint32_t)(nblocks * splitK);
            size_t         most = 0;
            for (uint32_t x = 0; x < 8; x++) {
                const size_t s0 = (size_t)x * q + (x < r ? x : r), s1 = (size_t)(x + 1) * q + (x + 1 < r ? x + 1 : r);
                const size_t rows = (s1 / per_block - s0 / per_block) * tile_rows;
                most = rows > most ? rows : most;
            }
            const size_t per_xcd = (most / 4 * N + 255) / 256;
            hipLaunchKernelGGL(splitk_reduce_by_xcd, dim3((uint32_t)(per_xcd * 8)), dim3(256), 0, st, static_cast<half_t *>(C), ws, (uint32_t)M, (uint32_t)N,
                               splitK, (uint32_t)tile_rows, q, r, per_block);
        } else {
            hipLaunchKernelGGL(splitk_reduce, dim3((uint32_t)((MN / 4 + 255) / 256)), dim3(256), 0, st, static_cast<half_t *>(C), ws, MN, splitK);
        }
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
    case FP6MI_ERR_ALIGN: return "weights, activations, output and workspace must be 16-byte aligned (scales: 2-byte, group exponents: 2-byte)";
    case FP6MI_ERR_TOO_LARGE: return "splitK*M*N floats exceed the library's static workspace (fp6mi_static_workspace_bytes)";
    case FP6MI_ERR_CAPTURE: return "the stream is being captured and this call would have to allocate: convert the weights first (fp6mi_relayout_ref_to_native_gpu) or make the first call outside the capture";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown fp6mi error";
    }
}

const char *fp6mi_tuning_info(void)
{
    return
#include "fp6mi_tuning_info.inc"
        ;
}

int fp6mi_version(void) { return 134; } // 134: three row tiles per workgroup in the small-batch kernel (any M: the last workgroup takes what is left), no other kernel changed; 133: wave-specialized tile kernel (launch kind 2) for large batches; 132: split-K reduction runs on the XCD that wrote the partial sums, every grid size gets XCD-contiguous tiles; 131: tile kernel stores through LDS; 130: small-batch kernel loads activations as whole rows and turns them into operand order through LDS

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

size_t fp6mi_group_exps_bytes(size_t M, size_t K) { return fp6mi::group_exps_bytes(M, K); }
int fp6mi_pack_group_exps(void *native_exps, const void *exps, size_t M, size_t K) { return fp6mi::pack_group_exps(native_exps, exps, M, K); }
int fp6mi_dequant_grouped(int E, int Mb, void *out, const void *raw, size_t M, size_t K, const void *sc, const void *exps)
{
    return fp6mi::dequant_grouped(E, Mb, out, raw, M, K, sc, exps);
}

size_t fp6mi_workspace_bytes(size_t M, size_t N, int splitK) { return splitK > 1 ? (size_t)splitK * M * N * sizeof(float) : 0; }

// Split-K choice.  Batches up to 16 (stream kernel): a cost model in microseconds on a part with `num_cus` compute
// units -- workgroups run in rounds of one per CU, a workgroup streams its weights at what one CU sustains, the whole
// chip cannot beat HBM, and a split costs a second launch plus writing and re-reading the FP32 partial sums; K is
// already split inside the workgroup, so a split rarely pays.  Larger batches (tile kernel): as much of the wanted K
// parallelism as keeps the FP32 partial-sum traffic (8 bytes per output per split) under half of the weight bytes.
static int heuristic_splitk(int xbits, size_t M, size_t N, size_t K, int num_cus);

int fp6mi_heuristic_splitk(size_t M, size_t N, size_t K, int num_cus) { return heuristic_splitk(6, M, N, K, num_cus); }

int fp6mi_heuristic_splitk_format(int E, int Mb, size_t M, size_t N, size_t K, int num_cus)
{
    return heuristic_splitk(fp6mi::supported(E, Mb) ? 1 + E + Mb : 6, M, N, K, num_cus);
}

static int heuristic_splitk(int xbits, size_t M, size_t N, size_t K, int num_cus)
{
    if (M == 0 || N == 0 || K == 0 || num_cus <= 0) return 1;
    size_t units = (K + 255) / 256;
    if (num_cus == 256) { // a measured neighbour knows better than any model: take its fastest split (3 % hysteresis towards fewer splits)
        if (const TuneAnswer *a = tune_lookup(xbits, M, N, K)) {
            int   best_s = 0;
            float best_t = 0.f;
            for (int i = 0; i < kNumSplits; i++) {
                if (a->t[i] == 0.f) continue;
                if (best_s == 0 || a->t[i] * 1.03f < best_t) { best_s = kSplits[i]; best_t = a->t[i]; }
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
    const double block_bytes = (double)fp6mi::native_block_bytes(xbits); // one 16-row x 256-column block of the format
    size_t       wgs = M / 16 ? M / 16 : 1;
    double       best = 1e30;
    int          best_s = 1;
    for (int s = 1; s <= 64 && (size_t)s <= units; s++) {
        double per_wg_bytes = (double)((units + s - 1) / s) * block_bytes;
        double rounds = std::ceil((double)(wgs * (size_t)s) / (double)num_cus);
        double t_cu = rounds * per_wg_bytes / (cu_gbps * 1e3);
        double t_hbm = (double)wgs * (double)units * block_bytes / (hbm_gbps * 1e3);
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
    if (reinterpret_cast<uintptr_t>(sc) & 1u) return FP6MI_ERR_ALIGN; // halfs; the tile kernel uses 8-byte loads where the pointer allows them
    return FP6MI_OK;
}

int fp6mi_linear_native(int E, int Mb, void *stream, const void *W, const void *sc, const void *B, void *C, size_t M, size_t N, size_t K,
                        float *ws, int splitK)
{
    int rc = check_gemm_args(E, Mb, W, sc, B, C, M, N, K, ws, splitK);
    if (rc != FP6MI_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return linear_native(*fp6mi::ops_for(E, Mb), st, W, sc, nullptr, B, C, M, N, K, ws, splitK, nullptr);
}

int fp6mi_linear_native_grouped(int E, int Mb, void *stream, const void *W, const void *sc, const void *group_exps, const void *B, void *C, size_t M,
                                size_t N, size_t K, float *ws, int splitK)
{
    int rc = check_gemm_args(E, Mb, W, sc, B, C, M, N, K, ws, splitK);
    if (rc != FP6MI_OK) return rc;
    if (!group_exps) return FP6MI_ERR_NULL;
    if (reinterpret_cast<uintptr_t>(group_exps) & 1u) return FP6MI_ERR_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return linear_native(*fp6mi::ops_for(E, Mb), st, W, sc, group_exps, B, C, M, N, K, ws, splitK, nullptr);
}

int fp6mi_linear_native_cfg(int E, int Mb, void *stream, const void *W, const void *sc, const void *B, void *C, size_t M, size_t N, size_t K,
                            float *ws, int splitK, int kind, int n_tiles, int row_tiles, int row_waves, int k_waves)
{
    int rc = check_gemm_args(E, Mb, W, sc, B, C, M, N, K, ws, splitK);
    if (rc != FP6MI_OK) return rc;
    LaunchCfg   c = { kind, n_tiles, row_tiles, row_waves, k_waves };
    hipStream_t st = static_cast<hipStream_t>(stream);
    return linear_native(*fp6mi::ops_for(E, Mb), st, W, sc, nullptr, B, C, M, N, K, ws, splitK, &c);
}

int fp6mi_linear_native_grouped_cfg(int E, int Mb, void *stream, const void *W, const void *sc, const void *group_exps, const void *B, void *C, size_t M,
                                    size_t N, size_t K, float *ws, int splitK, int kind, int n_tiles, int row_tiles, int row_waves, int k_waves)
{
    int rc = check_gemm_args(E, Mb, W, sc, B, C, M, N, K, ws, splitK);
    if (rc != FP6MI_OK) return rc;
    if (!group_exps) return FP6MI_ERR_NULL;
    if (reinterpret_cast<uintptr_t>(group_exps) & 1u) return FP6MI_ERR_ALIGN;
    LaunchCfg   c = { kind, n_tiles, row_tiles, row_waves, k_waves };
    hipStream_t st = static_cast<hipStream_t>(stream);
    return linear_native(*fp6mi::ops_for(E, Mb), st, W, sc, group_exps, B, C, M, N, K, ws, splitK, &c);
}

int fp6mi_launch_source(int E, int Mb, size_t M, size_t N, size_t K, int splitK)
{
    if (!fp6mi::supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (M == 0 || M % 256 || K == 0 || K % 64 || N == 0) return FP6MI_ERR_SHAPE;
    if (splitK < 1) return FP6MI_ERR_SPLITK;
    const int i = split_index(splitK);
    if (i >= 0)
        if (const TuneAnswer *a = tune_lookup(1 + E + Mb, M, N, K))
            if (a->t[i] > 0.f) return a->measured ? 0 : 1;
    return 2;
}

int fp6mi_query_launch(int E, int Mb, size_t M, size_t N, size_t K, int splitK, int *shape)
{
    if (!fp6mi::supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!shape) return FP6MI_ERR_NULL;
    if (M == 0 || M % 256 || K == 0 || K % 64 || N == 0) return FP6MI_ERR_SHAPE;
    if (splitK < 1) return FP6MI_ERR_SPLITK;
    LaunchCfg c = pick_cfg(1 + E + Mb, M, N, K, splitK, current_device_cus()); // the count the launch path uses (256 where no device answers)
    shape[0] = c.kind, shape[1] = c.nt, shape[2] = c.rt, shape[3] = c.wr, shape[4] = c.wk;
    return FP6MI_OK;
}

// ---- allocation-free variant of fp6mi_linear_native: the split-K workspace is a static device array of the library ----
namespace {
constexpr size_t kStaticWsFloats = (size_t)8 << 20; // 32 MiB per GPU, held from the first use of the library on that GPU until the process ends
__device__ __align__(256) float g_static_ws[kStaticWsFloats];

// Device address of g_static_ws on the current device (every GPU holds its own copy of the array at its own address); asked
// of the runtime once per device.  The array's name is only a host-side handle: kernels get this pointer as an argument.
int static_ws_ptr(float **out)
{
    static std::mutex mu;
    static float     *ptrs[64];
    int               dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return FP6MI_ERR_SHAPE;
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void *p = nullptr;
        if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_ws)); e != hipSuccess) return (int)e;
        ptrs[dev] = static_cast<float *>(p);
    }
    *out = ptrs[dev];
    return FP6MI_OK;
}
} // namespace

size_t fp6mi_static_workspace_bytes(void) { return kStaticWsFloats * sizeof(float); }

int fp6mi_init(void)
{
    float *p = nullptr;
    (void)current_device_cus();
    return static_ws_ptr(&p);
}

int fp6mi_linear_native_static(int E, int Mb, void *stream, const void *W, const void *sc, const void *B, void *C, size_t M, size_t N, size_t K,
                               int splitK)
{
    float *ws = nullptr;
    if (splitK > 1) {
        // checked before the multiplication can overflow: M, N <= 2^31 and splitK <= 65535 are enforced by check_gemm_args below
        if (M > 0x7fffffffu || N > 0x7fffffffu || splitK > 65535) return FP6MI_ERR_SHAPE;
        if ((size_t)splitK * M > kStaticWsFloats || (size_t)splitK * M * N > kStaticWsFloats) return FP6MI_ERR_TOO_LARGE;
        if (int rc = static_ws_ptr(&ws); rc != FP6MI_OK) return rc;
    }
    int rc = check_gemm_args(E, Mb, W, sc, B, C, M, N, K, ws, splitK);
    if (rc != FP6MI_OK) return rc;
    return linear_native(*fp6mi::ops_for(E, Mb), static_cast<hipStream_t>(stream), W, sc, nullptr, B, C, M, N, K, ws, splitK, nullptr);
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
    void *native = nullptr, *stale = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_twin_mutex);
        auto it = g_twins.find(W_ref);
        if (it != g_twins.end()) {
            const Twin &t = it->second;
            if (t.E == E && t.Mb == Mb && t.M == M && t.K == K && t.device == device) {
                native = t.native;
            } else { // the address now holds a different matrix
                stale = t.native;
                g_twins.erase(it);
            }
        }
    }
    // Everything slow happens outside the lock (allocation, the relayout kernel, the wait for it, freeing a stale twin), so
    // that other threads' calls, cache hits on other weights above all, never queue behind one caller's stream.
    if (stale) (void)hipFree(stale);
    if (!native) {
        // A twin has to be allocated and filled: not possible while the stream is being captured (the allocation would end
        // the capture with an error, and a replay would not repeat it).
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipError_t e = hipStreamIsCapturing(static_cast<hipStream_t>(stream), &cap); e != hipSuccess) return (int)e;
        if (cap != hipStreamCaptureStatusNone) return FP6MI_ERR_CAPTURE;
        size_t bytes = fp6mi::native_bytes(E, Mb, M, K);
        if (hipError_t e = hipMalloc(&native, bytes); e != hipSuccess) return (int)e;
        rc = fp6mi_relayout_ref_to_native_gpu(E, Mb, stream, native, W_ref, M, K);
        // The twin becomes visible to other callers (and other streams) only once it is completely written: this
        // one-time path waits for the relayout kernel before it publishes the pointer.
        if (rc == 0) rc = (int)hipStreamSynchronize(static_cast<hipStream_t>(stream));
        if (rc != 0) {
            (void)hipFree(native);
            return rc;
        }
        void *duplicate = nullptr;
        {
            std::lock_guard<std::mutex> lock(g_twin_mutex);
            auto ins = g_twins.emplace(W_ref, Twin{ native, E, Mb, M, K, device });
            if (!ins.second) { // another thread converted the same weights meanwhile
                const Twin &t = ins.first->second;
                if (t.E == E && t.Mb == Mb && t.M == M && t.K == K && t.device == device) {
                    duplicate = native;   // keep theirs, which may already be in use
                    native = t.native;
                } else {                  // theirs describes another matrix at this address: ours is the newer truth
                    duplicate = t.native;
                    ins.first->second = Twin{ native, E, Mb, M, K, device };
                }
            }
        }
        if (duplicate) (void)hipFree(duplicate);
    }
    return fp6mi_linear_native(E, Mb, stream, native, sc, B, C, M, N, K, ws, splitK);
}

int fp6mi_linear_stateless(int E, int Mb, void *stream, const void *W_ref, const void *sc, const void *B, void *C, size_t M, size_t N, size_t K,
                           float *ws, int splitK, void *native_scratch)
{
    if (!native_scratch) return FP6MI_ERR_NULL;
    if (!aligned16(native_scratch) || native_scratch == W_ref) return native_scratch == W_ref ? FP6MI_ERR_SHAPE : FP6MI_ERR_ALIGN;
    int rc = check_gemm_args(E, Mb, W_ref, sc, B, C, M, N, K, ws, splitK);
    if (rc != FP6MI_OK) return rc;
    rc = fp6mi_relayout_ref_to_native_gpu(E, Mb, stream, native_scratch, W_ref, M, K);
    if (rc != FP6MI_OK) return rc;
    return fp6mi_linear_native(E, Mb, stream, native_scratch, sc, B, C, M, N, K, ws, splitK);
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
    return fp6mi::ops_for(E, Mb)->relayout(stream, native, ref, M, K);
}

int fp6mi_dequant_native_gpu(int E, int Mb, void *stream, void *out, const void *W, const void *sc, size_t M, size_t K)
{
    if (!fp6mi::supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!out || !W || !sc) return FP6MI_ERR_NULL;
    if (M == 0 || M % 16 || K == 0 || K % 64 || M > 0x7fffffffu || K > 0x7fffffffu) return FP6MI_ERR_SHAPE;
    if (!aligned16(out) || !aligned16(W)) return FP6MI_ERR_ALIGN;
    return fp6mi::ops_for(E, Mb)->dequant(stream, out, W, sc, nullptr, M, K);
}

int fp6mi_dequant_native_grouped_gpu(int E, int Mb, void *stream, void *out, const void *W, const void *sc, const void *group_exps, size_t M, size_t K)
{
    if (!fp6mi::supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!out || !W || !sc || !group_exps) return FP6MI_ERR_NULL;
    if (M == 0 || M % 16 || K == 0 || K % 64 || M > 0x7fffffffu || K > 0x7fffffffu) return FP6MI_ERR_SHAPE;
    if (!aligned16(out) || !aligned16(W) || (reinterpret_cast<uintptr_t>(group_exps) & 1u)) return FP6MI_ERR_ALIGN;
    return fp6mi::ops_for(E, Mb)->dequant(stream, out, W, sc, group_exps, M, K);
}

int fp6mi_quantize_native_gpu(int E, int Mb, void *stream, void *native, void *scales, const void *weights, int dtype, size_t M, size_t K)
{
    if (!fp6mi::supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!native || !scales || !weights) return FP6MI_ERR_NULL;
    if (dtype < 0 || dtype > 2) return FP6MI_ERR_FORMAT;
    if (M == 0 || M % 16 || K == 0 || K % 64 || M > 0x7fffffffu || K > 0x7fffffffu) return FP6MI_ERR_SHAPE;
    if (!aligned16(native) || !aligned16(weights)) return FP6MI_ERR_ALIGN;
    return fp6mi::ops_for(E, Mb)->quantize(stream, native, scales, nullptr, weights, dtype, M, K);
}

int fp6mi_quantize_native_grouped_gpu(int E, int Mb, void *stream, void *native, void *scales, void *group_exps, const void *weights, int dtype,
                                      size_t M, size_t K)
{
    if (!fp6mi::supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!native || !scales || !weights || !group_exps) return FP6MI_ERR_NULL;
    if (dtype < 0 || dtype > 2) return FP6MI_ERR_FORMAT;
    if (M == 0 || M % 16 || K == 0 || K % 64 || M > 0x7fffffffu || K > 0x7fffffffu) return FP6MI_ERR_SHAPE;
    if (!aligned16(native) || !aligned16(weights)) return FP6MI_ERR_ALIGN;
    return fp6mi::ops_for(E, Mb)->quantize(stream, native, scales, group_exps, weights, dtype, M, K);
}

} // extern "C"
