// Bit-exact unpack helpers for the AutoGPTQ int4 / int3 packed formats.
//
// Everything here is plain integer and fp16 arithmetic written with clang
// vector types, so the same functions build for gfx950 and for the host
// (the host build is what the CPU-side tests check against the oracle).
//
// Format (reference: auto_gptq/nn_modules/qlinear.py:105-139 pack,
// :211-236 unpack): along the packed axis, every `bits` consecutive int32
// words form one little-endian bit stream holding 32 codes; code j sits at
// bit bits*j.  For 3 bits, codes 10 and 21 straddle word boundaries.
#pragma once
#include <stdint.h>

#if defined(__HIP__) || defined(__HIPCC__)
#define GPTQ_HD __host__ __device__ __forceinline__
#else
#define GPTQ_HD inline
#endif

namespace gptq {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));

GPTQ_HD h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }
GPTQ_HD uint32_t as_u32(h2 v) { return __builtin_bit_cast(uint32_t, v); }

// 32 bits of the 64-bit value hi:lo starting at bit `sh` (0 < sh < 32)
GPTQ_HD uint32_t funnel(uint32_t hi, uint32_t lo, int sh)
{
    return (uint32_t)((((uint64_t)hi << 32) | (uint64_t)lo) >> sh);
}

// ---- plain integer extraction (the definition everything else must equal) ----
GPTQ_HD int code4(uint32_t w, int j) { return (int)((w >> (4 * j)) & 0xfu); }

GPTQ_HD int code3(uint32_t w0, uint32_t w1, uint32_t w2, int j)
{
    const int bit = 3 * j;
    const int word = bit >> 5;
    const int sh = bit & 31;
    const uint32_t lo = word == 0 ? w0 : (word == 1 ? w1 : w2);
    const uint32_t hi = word == 0 ? w1 : (word == 1 ? w2 : 0u);
    const uint64_t v = (((uint64_t)hi << 32) | (uint64_t)lo) >> sh;
    return (int)(v & 0x7u);
}

// Widths that divide a word (2, 4, 8 bits): code j of a block of 32 codes held in `BITS` words.
template <int BITS>
GPTQ_HD int code_pow2(const uint32_t *w, int j)
{
    static_assert(BITS == 2 || BITS == 4 || BITS == 8, "width must divide 32");
    return (int)((w[(BITS * j) >> 5] >> ((BITS * j) & 31)) & ((1u << BITS) - 1u));
}

// Zero point (already +1) of column n from a packed qzeros row
// (reference: qlinear.py:202-209, :217-227).
GPTQ_HD int zero4(const uint32_t *zrow, int n) { return code4(zrow[n >> 3], n & 7) + 1; }

GPTQ_HD int zero3(const uint32_t *zrow, int n)
{
    const uint32_t *b = zrow + 3 * (n >> 5);
    return code3(b[0], b[1], b[2], n & 31) + 1;
}

// ---- "magic number" unpack: codes land in fp16 mantissas ----------------------
// OR-ing a code into the mantissa of 0x6400 (= 1024.0) yields 1024 + code * 2^p
// where p is the code's bit position inside its 16-bit half.  The halves of one
// 32-bit register therefore carry two codes that sit 16 (+-) bits apart in the
// stream; SLOT4 / SLOT3 give, for every (register, half), which code that is.
//
// int4: four registers per word.  Register r, half h holds code SLOT4[2r + h].
//   r = 0: p = 0 ;  r = 1: p = 4 ;  r = 2: p = 0 ;  r = 3: p = 4
static constexpr int SLOT4[8] = {0, 4, 1, 5, 2, 6, 3, 7};

GPTQ_HD void magic4(uint32_t w, uint32_t out[4])
{
    const uint32_t w8 = w >> 8;
    out[0] = (w & 0x000f000fu) | 0x64006400u;
    out[1] = (w & 0x00f000f0u) | 0x64006400u;
    out[2] = (w8 & 0x000f000fu) | 0x64006400u;
    out[3] = (w8 & 0x00f000f0u) | 0x64006400u;
}

// magic -> exact code value as fp16 (no rounding happens: all values are small integers)
GPTQ_HD h2 code_from_magic4(uint32_t m, int r)
{
    const h2 v = as_h2(m);
    if ((r & 1) == 0) {
        return v - (h2){(_Float16)1024.0f, (_Float16)1024.0f};
    }
    return v * (h2){(_Float16)0.0625f, (_Float16)0.0625f} - (h2){(_Float16)64.0f, (_Float16)64.0f};
}

// int3: sixteen registers per 3-word block.  Register r, half h holds code SLOT3[2r + h].
// Even registers: low half p = 0, high half p = 2.  Odd registers: low p = 3, high p = 5.
static constexpr int SLOT3[32] = {0,  6,  1,  7,  2,  8,  3,  9,  4,  10, 5,  11, 12, 18, 13, 19,
                                  14, 20, 15, 21, 16, 22, 17, 23, 24, 30, 25, 31, 26, 28, 27, 29};

GPTQ_HD void magic3(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t out[16])
{
    uint32_t win[8];
    win[0] = w0;                    // stream bit 0
    win[1] = w0 >> 6;               // 6
    win[2] = funnel(w1, w0, 12);    // 12
    win[3] = funnel(w2, w1, 4);     // 36
    win[4] = funnel(w2, w1, 10);    // 42
    win[5] = funnel(w2, w1, 16);    // 48
    win[6] = w2 >> 8;               // 72
    const uint32_t t = w2 >> 14;    // 78: codes 26..29 all in the low half
    win[7] = (t << 12) | t;         // move codes 28, 29 up into the high half
#pragma unroll
    for (int i = 0; i < 8; i++) {
        out[2 * i] = (win[i] & 0x001c0007u) | 0x64006400u;
        out[2 * i + 1] = (win[i] & 0x00e00038u) | 0x64006400u;
    }
}

GPTQ_HD h2 code_from_magic3(uint32_t m, int r)
{
    const h2 v = as_h2(m);
    if ((r & 1) == 0) {
        return v * (h2){(_Float16)1.0f, (_Float16)0.25f} - (h2){(_Float16)1024.0f, (_Float16)256.0f};
    }
    return v * (h2){(_Float16)0.125f, (_Float16)0.03125f} - (h2){(_Float16)128.0f, (_Float16)32.0f};
}


// ---- "biased" unpack: every code with unit weight, no arithmetic after the OR -----------
// Choosing the fp16 exponent per half so that the code's lowest bit has weight one makes the
// register read (base + code) directly: a code at mantissa bit p wants exponent 2^(10 - p),
// i.e. base = 1024 >> p.  The bases differ per slot but not per weight, so a product against
// x picks up sum_k x[k] * base(slot(k)), which one extra MFMA against the constant vector
// BASE4 / BASE3 measures and the epilogue subtracts.
//
// v_and_or_b32 takes one scalar constant at most, so the magic constant must sit in a vector
// register for the compiler to fuse the AND and the OR: opaque_vgpr() hides its value.
GPTQ_HD uint32_t opaque_vgpr(uint32_t v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" : "+v"(v));
#endif
    return v;
}

GPTQ_HD uint32_t and_or(uint32_t x, uint32_t mask, uint32_t magic) { return (x & mask) | magic; }

// int4: register r, half h holds BASE4[2r + h] + code SLOT4[2r + h]
static constexpr float BASE4[8] = {1024.f, 1024.f, 64.f, 64.f, 1024.f, 1024.f, 64.f, 64.f};

// The outputs are whole MFMA operands (four consecutive registers each) so that the register
// allocator can build them in place.
GPTQ_HD void biased4(uint32_t w, u4 out[1], uint32_t magic_lo, uint32_t magic_hi)
{
    const uint32_t w8 = w >> 8;
    out[0][0] = and_or(w, 0x000f000fu, magic_lo);   // 0x64006400: 1024 + code
    out[0][1] = and_or(w, 0x00f000f0u, magic_hi);   // 0x54005400: 64 + code
    out[0][2] = and_or(w8, 0x000f000fu, magic_lo);
    out[0][3] = and_or(w8, 0x00f000f0u, magic_hi);
}
static constexpr uint32_t MAGIC4_LO = 0x64006400u;
static constexpr uint32_t MAGIC4_HI = 0x54005400u;

// int3: register r, half h holds BASE3[2r + h] + code SLOT3[2r + h]; even registers carry
// (p = 0, p = 2) -> bases (1024, 256); odd registers (p = 3, p = 5) -> bases (128, 32).
static constexpr float BASE3[8] = {1024.f, 256.f, 128.f, 32.f, 1024.f, 256.f, 128.f, 32.f};
static constexpr uint32_t MAGIC3_EVEN = 0x5c006400u;
static constexpr uint32_t MAGIC3_ODD = 0x50005800u;

GPTQ_HD void biased3(uint32_t w0, uint32_t w1, uint32_t w2, u4 out[4], uint32_t magic_even,
                     uint32_t magic_odd)
{
    uint32_t win[8];
    win[0] = w0;
    win[1] = w0 >> 6;
    win[2] = funnel(w1, w0, 12);
    win[3] = funnel(w2, w1, 4);
    win[4] = funnel(w2, w1, 10);
    win[5] = funnel(w2, w1, 16);
    win[6] = w2 >> 8;
    const uint32_t t = w2 >> 14;
    win[7] = (t << 12) | t;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        out[i >> 1][2 * (i & 1)] = and_or(win[i], 0x001c0007u, magic_even);
        out[i >> 1][2 * (i & 1) + 1] = and_or(win[i], 0x00e00038u, magic_odd);
    }
}

// One quarter of biased3: the four registers (8 codes) of MFMA block nb of the 3-word block.
GPTQ_HD void biased3_block(uint32_t w0, uint32_t w1, uint32_t w2, int nb, u4 &out, uint32_t magic_even,
                           uint32_t magic_odd)
{
    uint32_t lo, hi;
    if (nb == 0) {
        lo = w0;
        hi = w0 >> 6;
    } else if (nb == 1) {
        lo = funnel(w1, w0, 12);
        hi = funnel(w2, w1, 4);
    } else if (nb == 2) {
        lo = funnel(w2, w1, 10);
        hi = funnel(w2, w1, 16);
    } else {
        lo = w2 >> 8;
        const uint32_t t = w2 >> 14;
        hi = (t << 12) | t;
    }
    out[0] = and_or(lo, 0x001c0007u, magic_even);
    out[1] = and_or(lo, 0x00e00038u, magic_odd);
    out[2] = and_or(hi, 0x001c0007u, magic_even);
    out[3] = and_or(hi, 0x00e00038u, magic_odd);
}

// int8: two registers per word.  Register r of a word holds fields (r, r + 2): both halves carry their code at
// mantissa bit 0, so every base is 1024.
static constexpr int SLOT8[4] = {0, 2, 1, 3};
static constexpr uint32_t MAGIC8 = 0x64006400u;

// int2: eight registers per word.  The word, and the word shifted right by 8, each give four registers:
// register r masks bits 2 r, 2 r + 1 of both halves, so its codes sit at mantissa bit 2 r and read
// (1024 >> 2 r) + code.  Register r of the unshifted word holds fields (r, 8 + r), of the shifted word
// (4 + r, 12 + r).
static constexpr int SLOT2[16] = {0, 8, 1, 9, 2, 10, 3, 11, 4, 12, 5, 13, 6, 14, 7, 15};
static constexpr uint32_t MAGIC2[4] = {0x64006400u, 0x5c005c00u, 0x54005400u, 0x4c004c00u};

// ---- the tiled format, per width ------------------------------------------------------------------
// A lane of the tiled format holds 32 codes in BITS words; operand j (j = 0..3) is the lane's positions
// 8 j .. 8 j + 7 as four registers of (base + code) pairs, register r holding positions (8 j + 2 r, 8 j + 2 r + 1).
//   field(s)   the stream field (of the lane's 32) that the unpack hands out as position s
//   base(e)    the base of position e (period 8)
//   KINDS      registers r and r + KINDS of an operand share their magic constant and their bases
//   operand()  the unpack of operand j; mg[k] = MAGIC[k] held in a vector register
template <int BITS>
struct TileCodec;

template <>
struct TileCodec<4> {
    static constexpr int KINDS = 2;
    static constexpr uint32_t MAGIC[4] = {MAGIC4_LO, MAGIC4_HI, MAGIC4_LO, MAGIC4_HI};
    static GPTQ_HD constexpr float base(int e) { return ((e >> 1) & 1) ? 64.f : 1024.f; }
    static GPTQ_HD constexpr int field(int s) { return (s & ~7) + SLOT4[s & 7]; }
    static GPTQ_HD void operand(const uint32_t (&w)[4], int j, u4 &q, const uint32_t (&mg)[KINDS])
    {
        u4 t[1];
        biased4(w[j], t, mg[0], mg[1]);
        q = t[0];
    }
};

template <>
struct TileCodec<3> {
    static constexpr int KINDS = 2;
    static constexpr uint32_t MAGIC[4] = {MAGIC3_EVEN, MAGIC3_ODD, MAGIC3_EVEN, MAGIC3_ODD};
    static GPTQ_HD constexpr float base(int e) { return BASE3[e & 7]; }
    static GPTQ_HD constexpr int field(int s) { return SLOT3[s]; }
    static GPTQ_HD void operand(const uint32_t (&w)[3], int j, u4 &q, const uint32_t (&mg)[KINDS])
    {
        biased3_block(w[0], w[1], w[2], j, q, mg[0], mg[1]);
    }
};

template <>
struct TileCodec<8> {
    static constexpr int KINDS = 1;
    static constexpr uint32_t MAGIC[4] = {MAGIC8, MAGIC8, MAGIC8, MAGIC8};
    static GPTQ_HD constexpr float base(int) { return 1024.f; }
    static GPTQ_HD constexpr int field(int s) { return (s & ~3) + SLOT8[s & 3]; }
    static GPTQ_HD void operand(const uint32_t (&w)[8], int j, u4 &q, const uint32_t (&mg)[KINDS])
    {
        q[0] = and_or(w[2 * j], 0x00ff00ffu, mg[0]);
        q[1] = and_or(w[2 * j] >> 8, 0x00ff00ffu, mg[0]);
        q[2] = and_or(w[2 * j + 1], 0x00ff00ffu, mg[0]);
        q[3] = and_or(w[2 * j + 1] >> 8, 0x00ff00ffu, mg[0]);
    }
};

template <>
struct TileCodec<2> {
    static constexpr int KINDS = 4;
    static constexpr uint32_t MAGIC[4] = {MAGIC2[0], MAGIC2[1], MAGIC2[2], MAGIC2[3]};
    static GPTQ_HD constexpr float base(int e) { return (float)(1024 >> (2 * ((e >> 1) & 3))); }
    static GPTQ_HD constexpr int field(int s) { return (s & ~15) + SLOT2[s & 15]; }
    static GPTQ_HD void operand(const uint32_t (&w)[2], int j, u4 &q, const uint32_t (&mg)[KINDS])
    {
        const uint32_t t = (j & 1) ? w[j >> 1] >> 8 : w[j >> 1];
        q[0] = and_or(t, 0x00030003u, mg[0]);
        q[1] = and_or(t, 0x000c000cu, mg[1]);
        q[2] = and_or(t, 0x00300030u, mg[2]);
        q[3] = and_or(t, 0x00c000c0u, mg[3]);
    }
};

// The dequantised weight of the reference (qlinear.py:242): fp16 scale times the
// integer (q - zero), rounded once.  (q - zero) is exact in fp16, so one fp16 multiply
// is that rounding, signed zeros and subnormals included.  (Going through an fp32
// product and a conversion is equal in value, but the compiler fuses it into a
// mixed-precision fma with a +0 addend, which turns -0 results into +0.)
GPTQ_HD _Float16 dequant_one(_Float16 scale, int q, int zero)
{
    return scale * (_Float16)(float)(q - zero);
}

}  // namespace gptq
