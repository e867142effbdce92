// Host build of csrc/gptq_unpack.h: checks the magic-number unpack against plain bit
// extraction on random words.  Reads nothing; prints "ok <count>" or the first mismatch.
#include <stdint.h>
#include <stdio.h>

#include <initializer_list>

#include "gptq_unpack.h"

using namespace gptq;

static uint64_t state = 0x9e3779b97f4a7c15ull;
static uint32_t rnd()
{
    state ^= state << 13;
    state ^= state >> 7;
    state ^= state << 17;
    return (uint32_t)(state >> 16);
}

// field f (BITS wide) of the little-endian stream held in the lane's words
template <int BITS>
static int stream_field(const uint32_t *w, int f)
{
    const int bit = BITS * f, wd = bit >> 5, sh = bit & 31;
    uint64_t v = w[wd];
    if (wd + 1 < BITS) v |= (uint64_t)w[wd + 1] << 32;
    return (int)((v >> sh) & ((1u << BITS) - 1u));
}

// The tiled format's codec: register r, half h of operand j reads base(2 r + h) + the code in stream field
// field(8 j + 2 r + h), and field() is a permutation of the lane's 32 fields.
template <int BITS>
static bool check_codec(const uint32_t (&w)[BITS], long &checked)
{
    using C = TileCodec<BITS>;
    uint32_t mg[C::KINDS];
    for (int k = 0; k < C::KINDS; k++) mg[k] = C::MAGIC[k];
    uint32_t seen = 0u;
    for (int j = 0; j < 4; j++) {
        u4 q;
        C::operand(w, j, q, mg);
        for (int r = 0; r < 4; r++) {
            const h2 v = as_h2(q[r]);
            for (int h = 0; h < 2; h++) {
                const int s = 8 * j + 2 * r + h;
                seen |= 1u << C::field(s);
                if (C::base(2 * r + h) != C::base(s) ||
                    (float)v[h] - C::base(s) != (float)stream_field<BITS>(w, C::field(s))) {
                    printf("codec<%d> mismatch operand %d reg %d half %d got %f\n", BITS, j, r, h, (float)v[h]);
                    return false;
                }
                // the matmul's dequantisation: (v - (base + zero)) is exact for every zero point of the width
                for (int z = 1; z <= (1 << BITS); z += (1 << BITS) - 1) {
                    const _Float16 zb = (_Float16)(C::base(s) + (float)z);
                    if ((float)(_Float16)(v[h] - zb) != (float)(stream_field<BITS>(w, C::field(s)) - z)) {
                        printf("codec<%d> zero-point subtraction is not exact\n", BITS);
                        return false;
                    }
                }
                checked++;
            }
        }
    }
    if (seen != 0xffffffffu) {
        printf("codec<%d>: field() is not a permutation\n", BITS);
        return false;
    }
    return true;
}

int main()
{
    long checked = 0;
    for (int it = 0; it < 20000; it++) {
        uint32_t w0 = rnd(), w1 = rnd(), w2 = rnd();
        if (it == 0) { w0 = w1 = w2 = 0xffffffffu; }
        if (it == 1) { w0 = w1 = w2 = 0u; }
        if (it == 2) { w0 = 0x80000000u; w1 = 0x80000001u; w2 = 0x00000003u; }
        uint32_t m4[4];
        magic4(w0, m4);
        for (int r = 0; r < 4; r++) {
            const h2 v = code_from_magic4(m4[r], r);
            for (int h = 0; h < 2; h++) {
                const int want = code4(w0, SLOT4[2 * r + h]);
                if ((float)v[h] != (float)want) {
                    printf("int4 mismatch w=%08x reg %d half %d got %f want %d\n", w0, r, h, (float)v[h], want);
                    return 1;
                }
                checked++;
            }
        }
        uint32_t m3[16];
        magic3(w0, w1, w2, m3);
        for (int r = 0; r < 16; r++) {
            const h2 v = code_from_magic3(m3[r], r);
            for (int h = 0; h < 2; h++) {
                const int want = code3(w0, w1, w2, SLOT3[2 * r + h]);
                if ((float)v[h] != (float)want) {
                    printf("int3 mismatch w=%08x %08x %08x reg %d half %d got %f want %d\n", w0, w1, w2, r, h,
                           (float)v[h], want);
                    return 1;
                }
                checked++;
            }
        }
        // biased unpack: register value minus its slot's base is the code
        u4 b4[1];
        biased4(w0, b4, MAGIC4_LO, MAGIC4_HI);
        for (int r = 0; r < 4; r++) {
            const h2 v = as_h2(b4[0][r]);
            for (int h = 0; h < 2; h++) {
                if ((float)v[h] - BASE4[2 * r + h] != (float)code4(w0, SLOT4[2 * r + h])) {
                    printf("biased4 mismatch w=%08x reg %d half %d got %f\n", w0, r, h, (float)v[h]);
                    return 1;
                }
                checked++;
            }
        }
        u4 b3[4];
        biased3(w0, w1, w2, b3, MAGIC3_EVEN, MAGIC3_ODD);
        for (int r = 0; r < 16; r++) {
            const h2 v = as_h2(b3[r >> 2][r & 3]);
            for (int h = 0; h < 2; h++) {
                if ((float)v[h] - BASE3[(2 * r + h) & 7] != (float)code3(w0, w1, w2, SLOT3[2 * r + h])) {
                    printf("biased3 mismatch w=%08x %08x %08x reg %d half %d got %f\n", w0, w1, w2, r, h,
                           (float)v[h]);
                    return 1;
                }
                checked++;
            }
        }
        {
            const uint32_t a2[2] = {w0, w1}, a3[3] = {w0, w1, w2}, a4[4] = {w0, w1, w2, rnd()};
            uint32_t a8[8] = {w0, w1, w2, rnd(), rnd(), rnd(), rnd(), rnd()};
            if (it == 0) for (auto &v : a8) v = 0xffffffffu;
            if (!check_codec<2>(a2, checked) || !check_codec<3>(a3, checked) || !check_codec<4>(a4, checked) ||
                !check_codec<8>(a8, checked))
                return 1;
        }
        // code3 itself against the reference's straddle formulas (qlinear.py:233-234)
        const int c10 = (int)(((w0 >> 30) & 0x3u) | ((w1 << 2) & 0x4u));
        const int c21 = (int)(((w1 >> 31) & 0x1u) | ((w2 << 1) & 0x6u));
        if (code3(w0, w1, w2, 10) != c10 || code3(w0, w1, w2, 21) != c21) {
            printf("straddle mismatch %08x %08x %08x\n", w0, w1, w2);
            return 1;
        }
        // exact dequant: product in fp32 rounded once
        const _Float16 s = (_Float16)(0.001f + (float)(rnd() & 0xffff) / 65536.0f * 0.009f);
        const int q = (int)(rnd() & 15), z = 1 + (int)(rnd() & 15);
        const _Float16 d = dequant_one(s, q, z);
        const _Float16 e = (_Float16)((float)s * (float)(q - z));  // exact fp32 product, one rounding
        if (__builtin_bit_cast(uint16_t, d) != __builtin_bit_cast(uint16_t, e)) {
            printf("dequant mismatch s=%f q=%d z=%d\n", (float)s, q, z);
            return 1;
        }
    }
    // SLOT tables are permutations
    int seen4 = 0;
    uint32_t seen3 = 0;
    for (int i = 0; i < 8; i++) seen4 |= 1 << SLOT4[i];
    for (int i = 0; i < 32; i++) seen3 |= 1u << SLOT3[i];
    if (seen4 != 0xff || seen3 != 0xffffffffu) {
        printf("slot tables are not permutations\n");
        return 1;
    }
    printf("ok %ld\n", checked);
    printf("slot4");
    for (int i = 0; i < 8; i++) printf(" %d", SLOT4[i]);
    printf("\nslot3");
    for (int i = 0; i < 32; i++) printf(" %d", SLOT3[i]);
    printf("\nslot8");
    for (int i = 0; i < 4; i++) printf(" %d", SLOT8[i]);
    printf("\nslot2");
    for (int i = 0; i < 16; i++) printf(" %d", SLOT2[i]);
    for (int bits : {2, 3, 4, 8}) {
        printf("\nbase%d", bits);
        for (int e = 0; e < 8; e++)
            printf(" %d", (int)(bits == 2 ? TileCodec<2>::base(e) : bits == 3 ? TileCodec<3>::base(e) : bits == 4 ? TileCodec<4>::base(e) : TileCodec<8>::base(e)));
        printf("\nfield%d", bits);
        for (int s = 0; s < 32; s++)
            printf(" %d", bits == 2 ? TileCodec<2>::field(s) : bits == 3 ? TileCodec<3>::field(s) : bits == 4 ? TileCodec<4>::field(s) : TileCodec<8>::field(s));
    }
    printf("\n");
    return 0;
}
