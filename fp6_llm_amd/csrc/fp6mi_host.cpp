// CPU half of the FPx linear-layer engine: reference-layout prepacking (bit-exact), dequantisation (bit-exact),
// and the packers for the native gfx950 layout.  No GPU headers; built into the same shared library as the kernels.
//
// Formats: x = 1+E+M bit codes, (E,M) = (3,2) "FP6_e3m2", (2,2) "FP5_e2m2", (2,3) "FP6_e2m3" or (2,1) "FP4_e2m1".
// Raw tensor: row-major [M,K] codes, each row an MSB-first bitstream (code c = bits [c*x,(c+1)*x), bit 0 = MSB of
// byte 0), the format defined by fp6_llm/csrc/utils/common.h:4-19 of the reference.
#include "fp6mi_internal.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

namespace fp6mi {

// ------------------------------------------------------------------------------------------------ small helpers

template <class F>
static void parallel_for(size_t n, F &&body)
{
    unsigned hw = std::thread::hardware_concurrency();
    size_t   nt = std::min<size_t>({ (size_t)(hw ? hw : 1), (size_t)16, n });
    if (nt <= 1) {
        for (size_t i = 0; i < n; i++) body(i);
        return;
    }
    std::vector<std::thread> pool;
    for (size_t t = 0; t < nt; t++)
        pool.emplace_back([&, t] {
            for (size_t i = t; i < n; i += nt) body(i);
        });
    for (auto &th : pool) th.join();
}

// Reads `count` codes (count % 8 == 0) starting at code index `first` (first % 8 == 0) of a row bitstream.
// Eight codes occupy exactly x bytes, so the reader never touches a byte outside the row.
static inline void read_codes(const uint8_t *row, int x, size_t first, size_t count, uint8_t *codes)
{
    const uint8_t *p    = row + first / 8 * x;
    const uint64_t mask = (1u << x) - 1u;
    for (size_t g = 0; g < count / 8; g++, p += x, codes += 8) {
        uint64_t v = 0;
        for (int b = 0; b < x; b++) v = (v << 8) | p[b]; // x bytes, big-endian = MSB-first bit order
        for (int i = 0; i < 8; i++) codes[i] = (uint8_t)((v >> (x * (7 - i))) & mask);
    }
}

static inline void write_codes(uint8_t *row, int x, size_t first, size_t count, const uint8_t *codes)
{
    uint8_t *p = row + first / 8 * x;
    for (size_t g = 0; g < count / 8; g++, p += x, codes += 8) {
        uint64_t v = 0;
        for (int i = 0; i < 8; i++) v = (v << x) | codes[i];
        for (int b = x - 1; b >= 0; b--) { p[b] = (uint8_t)v; v >>= 8; }
    }
}

// ------------------------------------------------------------------------------------------------ reference layout
//
// The reference's layout (utils/weight_prepacking.h:118-196) in closed form.  The buffer is the concatenation of one
// array per segment width w in {1,2,4} that the bit width uses (x & w), in that order; segments are cut from the
// code MSB-down in the same order.  Every array is little-endian 32-bit words,
//     word = ((i*(K/16) + j)*w + q)*32 + lane,        i = 64-row tile, j = 16-column slice, q in [0,w), lane = 4g+t
// and the fragment at MSB-first position p of a word belongs to
//     pre = order_w[p]-1,  block = q*(4/w) + pre/8,  el = pre%8,
//     row = 64i + 16*block + g + 8*((el>>1)&1),      col = 16j + 2t + (el&1) + 8*(el>>2).
struct FragPos { uint8_t row_off, col_off; }; // row offset without g, column offset without 2t

struct RefTables {
    // [w index 0..2][q][p]
    FragPos pos[3][4][32];
    RefTables()
    {
        static const int order1[32] = { 2, 6, 10, 14, 18, 22, 26, 30, 4, 8, 12, 16, 20, 24, 28, 32,
                                        1, 5, 9, 13, 17, 21, 25, 29, 3, 7, 11, 15, 19, 23, 27, 31 };
        static const int order2[16] = { 2, 6, 10, 14, 4, 8, 12, 16, 1, 5, 9, 13, 3, 7, 11, 15 };
        static const int order4[8]  = { 2, 6, 4, 8, 1, 5, 3, 7 };
        const int *orders[3] = { order1, order2, order4 };
        for (int wi = 0; wi < 3; wi++) {
            int w = 1 << wi;
            for (int q = 0; q < w; q++)
                for (int p = 0; p < 32 / w; p++) {
                    int pre = orders[wi][p] - 1, block = q * (4 / w) + pre / 8, el = pre % 8;
                    pos[wi][q][p].row_off = (uint8_t)(16 * block + 8 * ((el >> 1) & 1));
                    pos[wi][q][p].col_off = (uint8_t)((el & 1) + 8 * (el >> 2));
                }
        }
    }
};
static const RefTables &ref_tables()
{
    static const RefTables t;
    return t;
}

struct SegInfo { int w, shift; size_t offset_bytes; };
// Segments present for bit width x, with the right shift that isolates each piece and its array offset.
static int segments_of(int x, size_t M, size_t K, SegInfo seg[3])
{
    int    n = 0, consumed = 0;
    size_t off = 0;
    for (int w = 1; w <= 4; w <<= 1) {
        if (!(x & w)) continue;
        consumed += w;
        seg[n++] = { w, x - consumed, off };
        off += M * K * (size_t)w / 8;
    }
    return n;
}

// One 64-row tile: codes [64][K] -> words of every segment array for tile i.
static void ref_pack_tile(int x, size_t M, size_t K, size_t i, const uint8_t *codes, uint8_t *out)
{
    const RefTables &T = ref_tables();
    SegInfo seg[3];
    int     ns = segments_of(x, M, K, seg);
    for (int s = 0; s < ns; s++) {
        int       w = seg[s].w, wi = (w == 1) ? 0 : (w == 2) ? 1 : 2, nfrag = 32 / w;
        uint32_t  pmask = (1u << w) - 1u;
        uint32_t *words = reinterpret_cast<uint32_t *>(out + seg[s].offset_bytes) + i * (K / 16) * (size_t)w * 32;
        for (size_t j = 0; j < K / 16; j++)
            for (int q = 0; q < w; q++)
                for (int lane = 0; lane < 32; lane++) {
                    int      g = lane >> 2, t = lane & 3;
                    uint32_t word = 0;
                    for (int p = 0; p < nfrag; p++) {
                        const FragPos &fp = T.pos[wi][q][p];
                        uint32_t c = codes[(size_t)(fp.row_off + g) * K + 16 * j + 2 * t + fp.col_off];
                        word |= ((c >> seg[s].shift) & pmask) << (32 - w * (p + 1));
                    }
                    words[(j * w + q) * 32 + lane] = word;
                }
    }
}

static void ref_unpack_tile(int x, size_t M, size_t K, size_t i, const uint8_t *in, uint8_t *codes)
{
    const RefTables &T = ref_tables();
    SegInfo seg[3];
    int     ns = segments_of(x, M, K, seg);
    std::memset(codes, 0, 64 * K);
    for (int s = 0; s < ns; s++) {
        int             w = seg[s].w, wi = (w == 1) ? 0 : (w == 2) ? 1 : 2, nfrag = 32 / w;
        uint32_t        pmask = (1u << w) - 1u;
        const uint32_t *words = reinterpret_cast<const uint32_t *>(in + seg[s].offset_bytes) + i * (K / 16) * (size_t)w * 32;
        for (size_t j = 0; j < K / 16; j++)
            for (int q = 0; q < w; q++)
                for (int lane = 0; lane < 32; lane++) {
                    int      g = lane >> 2, t = lane & 3;
                    uint32_t word = words[(j * w + q) * 32 + lane];
                    for (int p = 0; p < nfrag; p++) {
                        const FragPos &fp = T.pos[wi][q][p];
                        uint8_t piece = (uint8_t)((word >> (32 - w * (p + 1))) & pmask);
                        codes[(size_t)(fp.row_off + g) * K + 16 * j + 2 * t + fp.col_off] |= (uint8_t)(piece << seg[s].shift);
                    }
                }
    }
}

int prepack_ref(int E, int Mb, void *packed, const void *raw, size_t M, size_t K)
{
    if (!supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!packed || !raw) return FP6MI_ERR_NULL;
    if (M == 0 || K == 0 || M % 64 || K % 64) return FP6MI_ERR_SHAPE;
    int    x = 1 + E + Mb;
    size_t row_bytes = K * x / 8, total = M * row_bytes;
    // The output of a tile lands all over the buffer, so an aliased call is staged through a private copy.
    const uint8_t       *src = static_cast<const uint8_t *>(raw);
    std::vector<uint8_t> staged;
    if (packed == raw) {
        staged.assign(src, src + total);
        src = staged.data();
    }
    uint8_t *dst = static_cast<uint8_t *>(packed);
    parallel_for(M / 64, [&](size_t i) {
        std::vector<uint8_t> codes(64 * K);
        for (size_t r = 0; r < 64; r++) read_codes(src + (i * 64 + r) * row_bytes, x, 0, K, codes.data() + r * K);
        ref_pack_tile(x, M, K, i, codes.data(), dst);
    });
    return FP6MI_OK;
}

int unpack_ref(int E, int Mb, void *raw, const void *packed, size_t M, size_t K)
{
    if (!supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!packed || !raw) return FP6MI_ERR_NULL;
    if (M == 0 || K == 0 || M % 64 || K % 64 || raw == packed) return FP6MI_ERR_SHAPE;
    int    x = 1 + E + Mb;
    size_t row_bytes = K * x / 8;
    parallel_for(M / 64, [&](size_t i) {
        std::vector<uint8_t> codes(64 * K);
        ref_unpack_tile(x, M, K, i, static_cast<const uint8_t *>(packed), codes.data());
        for (size_t r = 0; r < 64; r++)
            write_codes(static_cast<uint8_t *>(raw) + (i * 64 + r) * row_bytes, x, 0, K, codes.data() + r * K);
    });
    return FP6MI_OK;
}

// ------------------------------------------------------------------------------------------------ dequantisation
//
// value(code) = (-1)^s 2^(e-b) (1+m/2^M), e = 0: (-1)^s 2^(1-b) m/2^M, b = 2^(E-1)-1; every exponent is an ordinary value.
// out = fp16_rn(value * float(scale)): the product of an at most 4-bit and an 11-bit significand is exact in FP32, so there is
// one rounding, which is what utils/weight_dequant.h:30-43 of the reference computes.
// exps (may be null): one byte b per (row, 128 columns), row-major [M][ceil(K/128)], the factor 2^(b-127) on those weights;
// then out = fp16_rn(value * 2^(b-127) * float(scale)), still one rounding (the power of two is exact in double).
static int dequant_any(int E, int Mb, void *out_f16, const void *raw, size_t M, size_t K, const void *scales_f16, const uint8_t *exps)
{
    if (!supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!out_f16 || !raw || !scales_f16) return FP6MI_ERR_NULL;
    if (M == 0 || K == 0 || K % 8) return FP6MI_ERR_SHAPE;
    int    x = 1 + E + Mb, ncodes = 1 << x;
    size_t row_bytes = K * x / 8, groups = (K + 127) / 128;
    float  value[64];
    for (int c = 0; c < ncodes; c++) {
        int   s = c >> (x - 1), e = (c >> Mb) & ((1 << E) - 1), m = c & ((1 << Mb) - 1), b = (1 << (E - 1)) - 1;
        float v = e ? std::ldexp(1.0f + (float)m / (float)(1 << Mb), e - b) : std::ldexp((float)m / (float)(1 << Mb), 1 - b);
        value[c] = s ? -v : v; // s ? -0.0f : 0.0f for the zero magnitude
    }
    const uint8_t  *src = static_cast<const uint8_t *>(raw);
    const _Float16 *sc  = static_cast<const _Float16 *>(scales_f16);
    _Float16       *dst = static_cast<_Float16 *>(out_f16);
    parallel_for((M + 15) / 16, [&](size_t blk) {
        std::vector<uint8_t> codes(K);
        for (size_t r = blk * 16; r < std::min(M, blk * 16 + 16); r++) {
            _Float16 table[64];
            float    s = (float)sc[r];
            read_codes(src + r * row_bytes, x, 0, K, codes.data());
            _Float16 *o = dst + r * K;
            for (size_t g = 0; g < (exps ? groups : 1); g++) {
                // value * 2^k * scale has at most 4 + 11 significant bits: exact in double for every k, and exact in float
                // wherever fp16 can tell the result from zero or infinity; so the float -> half step is the one rounding
                double f = exps ? std::ldexp(1.0, (int)exps[r * groups + g] - 127) : 1.0;
                for (int c = 0; c < ncodes; c++) table[c] = (_Float16)(float)((double)value[c] * f * (double)s);
                size_t c0 = exps ? g * 128 : 0, c1 = exps ? std::min(K, c0 + 128) : K;
                for (size_t c = c0; c < c1; c++) o[c] = table[codes[c]];
            }
        }
    });
    return FP6MI_OK;
}

int dequant(int E, int Mb, void *out_f16, const void *raw, size_t M, size_t K, const void *scales_f16)
{
    return dequant_any(E, Mb, out_f16, raw, M, K, scales_f16, nullptr);
}

int dequant_grouped(int E, int Mb, void *out_f16, const void *raw, size_t M, size_t K, const void *scales_f16, const void *exps)
{
    if (!exps) return FP6MI_ERR_NULL;
    return dequant_any(E, Mb, out_f16, raw, M, K, scales_f16, static_cast<const uint8_t *>(exps));
}

// Group exponents in the order the kernels read them: [row tile][K block][row in tile][half of the block], 32 bytes per
// 16x256 block; halves beyond K hold 127 (factor 1; the weights there are zero codes anyway).
size_t group_exps_bytes(size_t M, size_t K) { return (M % 16 || K % 64) ? 0 : (M / 16) * ((K + 255) / 256) * 32; }

int pack_group_exps(void *native_exps, const void *exps, size_t M, size_t K)
{
    if (!native_exps || !exps) return FP6MI_ERR_NULL;
    if (M == 0 || K == 0 || M % 16 || K % 64 || native_exps == exps) return FP6MI_ERR_SHAPE;
    const size_t   units = (K + 255) / 256, groups = (K + 127) / 128;
    const uint8_t *src = static_cast<const uint8_t *>(exps);
    uint8_t       *dst = static_cast<uint8_t *>(native_exps);
    for (size_t R = 0; R < M / 16; R++)
        for (size_t U = 0; U < units; U++)
            for (size_t m = 0; m < 16; m++)
                for (size_t h = 0; h < 2; h++) {
                    size_t g = 2 * U + h;
                    dst[((R * units + U) * 16 + m) * 2 + h] = g < groups ? src[(R * 16 + m) * groups + g] : (uint8_t)127;
                }
    return FP6MI_OK;
}

// ------------------------------------------------------------------------------------------------ native layout
//
// Unit of the layout: a block = 16 rows x 256 columns, stored contiguously; blocks are ordered
// [row tile R = row/16][K block U = col/256]; K is padded to a multiple of 256 with zero codes.
// Inside a block, wavefront lane l = (m = l%16, q = l/16) owns row 16R+m and, for MFMA step s = 0..7,
// the eight codes of columns 256U + 32s + 8q + 0..7: exactly its A operand of v_mfma_f32_16x16x32_f16.
// Its 64 codes are numbered ci = 8s + j.
//
// FP6_e3m2 block (3072 B): lane l's codes are packed as two 192-bit little-endian strings of 32 six-bit codes
// (code ci%32 at bits [6(ci%32), +6) of string ci/32), the source format of v_cvt_scalef32_pk32_f16_bf6;
// the twelve dwords d = 0..11 of a lane sit at byte (d/4)*1024 + 16*l + 4*(d%4), so three 16-byte loads per lane,
// each contiguous over the wavefront, fetch a block.
//
// FP5_e2m2 block (2560 B): the same two strings of 32 six-bit fields per lane, each field = the FP5 code with a zero
// inserted above its two exponent bits (sign, 0, e1 e0 m1 m0): read as e3m2 that field is exactly a quarter of the e2m2
// value, subnormals included, so the same hardware conversion applies.  A string would take six dwords D0..D5 with one
// fixed-zero bit (a "hole", bit 4 of each field) per code; storage keeps five dwords S0..S4 per string by parking the 26
// payload bits of D5 in the 26 holes of D0..D4, a residue class of bit positions per dword so that one mask (and one shared
// shift) moves them back:
//   S0 = D0 | (D5 & A)   S1 = D1 | (D5 & B)   S2 = D2 | ((D5 >> 1) & C)   S3 = D3 | ((D5 >> 1) & A)   S4 = D4 | ((D5 >> 1) & B)
//   A = 0x10410410 (bits 4,10,..,28)   B = 0x04104104 (bits 2,8,..,26)   C = 0x41041041 (bits 0,6,..,30)
//   D5 = (S0 & A) | (S1 & B) | (((S2 & C) | (S3 & A) | (S4 & B)) << 1),   Dk = Sk & ~(its hole mask)
// Eleven integer instructions rebuild the six dwords of 32 codes.  Lane dwords: string h has S0..S3 in dwords 4h..4h+3
// and S4 in dword 8+h; dwords 0..7 sit at (d/4)*1024 + 16*l + 4*(d%4), dwords 8,9 at 2048 + 8*l + 4*(d-8).
//
// FP6_e2m3 block (3072 B): the FP6_e3m2 block with e2m3 codes, the source format of v_cvt_scalef32_pk32_f16_fp6.
//
// FP4_e2m1 block (2048 B): again two strings of 32 six-bit fields per lane, each field = the FP4 code with two zeros appended
// below its mantissa bit (s e1 e0 m 0 0): read as e2m3 that field is exactly the e2m1 value.  The two fixed-zero bits of the
// 22 fields that start in D0..D3 are as many holes (44) as D4 and D5 have payload bits, at the same positions within a
// dword, so storage keeps four dwords S0..S3 per string and no bit has to shift:
//   S0 = D0 | (D4 & P)   S1 = D1 | (D5 & Q)   S2 = D2 | (D4 & R)   S3 = D3 | (D5 & P)
//   P = 0xC30C30C3 (bit pairs 0,6,..,30)   Q = 0x30C30C30 (pairs 4,10,..,28)   R = 0x0C30C30C (pairs 2,8,..,26)
//   D4 = (S0 & P) | (S2 & R),   D5 = (S1 & Q) | (S3 & P),   D0 = S0 & ~P,  D1 = S1 & ~Q,  D2 = S2 & ~R,  D3 = S3 & ~P
// Lane dwords: string h has S0..S3 in dwords 4h..4h+3 at (d/4)*1024 + 16*l + 4*(d%4).
size_t native_block_bytes(int x) { return x == 6 ? 3072 : x == 5 ? 2560 : 2048; }
static inline int native_lane_dwords(int x) { return x == 6 ? 12 : x == 5 ? 10 : 8; }

static const uint32_t kHoleA = 0x10410410u, kHoleB = 0x04104104u, kHoleC = 0x41041041u;
static const uint32_t kPairP = 0xC30C30C3u, kPairQ = 0x30C30C30u, kPairR = 0x0C30C30Cu;

// 32 six-bit fields -> six dwords (little-endian bit string), and back
static void fields_to_dwords(const uint8_t f[32], uint32_t o[6])
{
    for (int w = 0; w < 6; w++) o[w] = 0;
    for (int i = 0; i < 32; i++) {
        int      bit = 6 * i, w = bit >> 5, off = bit & 31;
        uint32_t v   = f[i] & 63u;
        o[w] |= v << off;
        if (off > 26) o[w + 1] |= v >> (32 - off);
    }
}
static void dwords_to_fields(const uint32_t o[6], uint8_t f[32])
{
    for (int i = 0; i < 32; i++) {
        int      bit = 6 * i, w = bit >> 5, off = bit & 31;
        uint32_t v   = o[w] >> off;
        if (off > 26) v |= o[w + 1] << (32 - off);
        f[i] = (uint8_t)(v & 63u);
    }
}

static inline size_t native_dword_offset(int x, int lane, int d)
{
    if (x != 5 || d < 8) return (size_t)(d / 4) * 1024 + (size_t)lane * 16 + (size_t)(d % 4) * 4;
    return 2048 + (size_t)lane * 8 + (size_t)(d - 8) * 4;
}

static void native_pack_lane(int x, const uint8_t c[64], uint32_t d[12])
{
    for (int h = 0; h < 2; h++) {
        if (x == 6) {
            fields_to_dwords(c + 32 * h, d + 6 * h);
        } else if (x == 4) {
            uint8_t  f[32];
            uint32_t D[6];
            for (int i = 0; i < 32; i++) f[i] = (uint8_t)((c[32 * h + i] & 15u) << 2);
            fields_to_dwords(f, D);
            d[4 * h + 0] = D[0] | (D[4] & kPairP);
            d[4 * h + 1] = D[1] | (D[5] & kPairQ);
            d[4 * h + 2] = D[2] | (D[4] & kPairR);
            d[4 * h + 3] = D[3] | (D[5] & kPairP);
        } else {
            uint8_t  f[32];
            uint32_t D[6];
            for (int i = 0; i < 32; i++) f[i] = (uint8_t)((c[32 * h + i] & 15u) | (((c[32 * h + i] >> 4) & 1u) << 5));
            fields_to_dwords(f, D);
            d[4 * h + 0] = D[0] | (D[5] & kHoleA);
            d[4 * h + 1] = D[1] | (D[5] & kHoleB);
            d[4 * h + 2] = D[2] | ((D[5] >> 1) & kHoleC);
            d[4 * h + 3] = D[3] | ((D[5] >> 1) & kHoleA);
            d[8 + h]     = D[4] | ((D[5] >> 1) & kHoleB);
        }
    }
}

static void native_unpack_lane(int x, const uint32_t d[12], uint8_t c[64])
{
    for (int h = 0; h < 2; h++) {
        if (x == 6) {
            dwords_to_fields(d + 6 * h, c + 32 * h);
        } else if (x == 4) {
            const uint32_t S0 = d[4 * h], S1 = d[4 * h + 1], S2 = d[4 * h + 2], S3 = d[4 * h + 3];
            uint32_t       D[6] = { S0 & ~kPairP, S1 & ~kPairQ, S2 & ~kPairR, S3 & ~kPairP, (S0 & kPairP) | (S2 & kPairR), (S1 & kPairQ) | (S3 & kPairP) };
            uint8_t        f[32];
            dwords_to_fields(D, f);
            for (int i = 0; i < 32; i++) c[32 * h + i] = (uint8_t)(f[i] >> 2);
        } else {
            const uint32_t S0 = d[4 * h], S1 = d[4 * h + 1], S2 = d[4 * h + 2], S3 = d[4 * h + 3], S4 = d[8 + h];
            uint32_t       D[6] = { S0 & ~kHoleA, S1 & ~kHoleB, S2 & ~kHoleC, S3 & ~kHoleA, S4 & ~kHoleB,
                                    (S0 & kHoleA) | (S1 & kHoleB) | (((S2 & kHoleC) | (S3 & kHoleA) | (S4 & kHoleB)) << 1) };
            uint8_t        f[32];
            dwords_to_fields(D, f);
            for (int i = 0; i < 32; i++) c[32 * h + i] = (uint8_t)((f[i] & 15u) | (((f[i] >> 5) & 1u) << 4));
        }
    }
}

size_t native_bytes(int E, int Mb, size_t M, size_t K)
{
    if (!supported(E, Mb) || M % 16 || K % 64) return 0;
    return (M / 16) * ((K + 255) / 256) * native_block_bytes(1 + E + Mb);
}

// codes: [16][K] of row tile R -> all blocks of that row tile
static void native_pack_rowtile(int x, size_t K, const uint8_t *codes, uint8_t *tile_out)
{
    size_t units = (K + 255) / 256, bb = native_block_bytes(x);
    int    nd = native_lane_dwords(x);
    for (size_t U = 0; U < units; U++)
        for (int lane = 0; lane < 64; lane++) {
            int     m = lane & 15, q = lane >> 4;
            uint8_t c[64];
            for (int s = 0; s < 8; s++) {
                size_t k0 = U * 256 + 32 * (size_t)s + 8 * (size_t)q;
                for (int j = 0; j < 8; j++) c[8 * s + j] = (k0 + j < K) ? codes[(size_t)m * K + k0 + j] : 0;
            }
            uint32_t d[12];
            native_pack_lane(x, c, d);
            for (int i = 0; i < nd; i++) std::memcpy(tile_out + U * bb + native_dword_offset(x, lane, i), &d[i], 4);
        }
}

static void native_unpack_rowtile(int x, size_t K, const uint8_t *tile_in, uint8_t *codes)
{
    size_t units = (K + 255) / 256, bb = native_block_bytes(x);
    int    nd = native_lane_dwords(x);
    for (size_t U = 0; U < units; U++)
        for (int lane = 0; lane < 64; lane++) {
            int      m = lane & 15, q = lane >> 4;
            uint32_t d[12] = { 0 };
            for (int i = 0; i < nd; i++) std::memcpy(&d[i], tile_in + U * bb + native_dword_offset(x, lane, i), 4);
            uint8_t c[64];
            native_unpack_lane(x, d, c);
            for (int s = 0; s < 8; s++) {
                size_t k0 = U * 256 + 32 * (size_t)s + 8 * (size_t)q;
                for (int j = 0; j < 8; j++)
                    if (k0 + j < K) codes[(size_t)m * K + k0 + j] = c[8 * s + j];
            }
        }
}

int prepack_native(int E, int Mb, void *native, const void *raw, size_t M, size_t K)
{
    if (!supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!native || !raw) return FP6MI_ERR_NULL;
    if (M == 0 || K == 0 || M % 16 || K % 64 || native == raw) return FP6MI_ERR_SHAPE;
    int    x = 1 + E + Mb;
    size_t row_bytes = K * x / 8, tile_bytes = ((K + 255) / 256) * native_block_bytes(x);
    parallel_for(M / 16, [&](size_t R) {
        std::vector<uint8_t> codes(16 * K);
        for (size_t r = 0; r < 16; r++)
            read_codes(static_cast<const uint8_t *>(raw) + (R * 16 + r) * row_bytes, x, 0, K, codes.data() + r * K);
        native_pack_rowtile(x, K, codes.data(), static_cast<uint8_t *>(native) + R * tile_bytes);
    });
    return FP6MI_OK;
}

int unpack_native(int E, int Mb, void *raw, const void *native, size_t M, size_t K)
{
    if (!supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!native || !raw) return FP6MI_ERR_NULL;
    if (M == 0 || K == 0 || M % 16 || K % 64 || native == raw) return FP6MI_ERR_SHAPE;
    int    x = 1 + E + Mb;
    size_t row_bytes = K * x / 8, tile_bytes = ((K + 255) / 256) * native_block_bytes(x);
    parallel_for(M / 16, [&](size_t R) {
        std::vector<uint8_t> codes(16 * K);
        native_unpack_rowtile(x, K, static_cast<const uint8_t *>(native) + R * tile_bytes, codes.data());
        for (size_t r = 0; r < 16; r++)
            write_codes(static_cast<uint8_t *>(raw) + (R * 16 + r) * row_bytes, x, 0, K, codes.data() + r * K);
    });
    return FP6MI_OK;
}

int relayout_ref_to_native(int E, int Mb, void *native, const void *packed_ref, size_t M, size_t K)
{
    if (!supported(E, Mb)) return FP6MI_ERR_FORMAT;
    if (!native || !packed_ref) return FP6MI_ERR_NULL;
    if (M == 0 || K == 0 || M % 64 || K % 64 || native == packed_ref) return FP6MI_ERR_SHAPE;
    int    x = 1 + E + Mb;
    size_t tile_bytes = ((K + 255) / 256) * native_block_bytes(x);
    parallel_for(M / 64, [&](size_t i) {
        std::vector<uint8_t> codes(64 * K);
        ref_unpack_tile(x, M, K, i, static_cast<const uint8_t *>(packed_ref), codes.data());
        for (size_t t = 0; t < 4; t++)
            native_pack_rowtile(x, K, codes.data() + t * 16 * K, static_cast<uint8_t *>(native) + (i * 4 + t) * tile_bytes);
    });
    return FP6MI_OK;
}

} // namespace fp6mi
