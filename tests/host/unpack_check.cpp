// Host build of csrc/gptq_unpack.h: checks the magic-number unpack against plain bit
// extraction on random words.  Reads nothing; prints "ok <count>" or the first mismatch.
#include <stdint.h>
#include <stdio.h>

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
    printf("\n");
    return 0;
}
