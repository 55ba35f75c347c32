/* Integer-only C restatement of the Q4_0 codec.  TEST INFRASTRUCTURE ONLY.
 *
 * Nothing in the product links or loads this file: it exists so that the torch/numpy oracle
 * (oracle/q40_oracle.py) and the HIP kernels can be checked against arithmetic that shares no
 * floating-point library with either.  fp16 values travel as uint16_t bit patterns; the fp16
 * multiply and divide are done on float (exact for the operand ranges used, see below) and
 * rounded to fp16 by hand with round-to-nearest-even, subnormals kept.
 *
 * Follows fp16_to_int4.py:52-96 of the reference (same maths at triton_kernels.py:12-56).
 * Parity pins for this file: tests/test_oracle_codec.py compares it with numpy float16 and with
 * torch on every (nibble, scale) pair and on every fp16 absmax.
 */
#include <stdint.h>
#include <string.h>
#include <math.h>

static float h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {                      /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* float -> fp16, round to nearest even, subnormals kept, overflow to inf, NaN stays NaN */
static uint16_t f2h(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) {                      /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((absx > 0x7F800000u) ? 0x200u : 0u));
    }
    int32_t exp = (int32_t)(absx >> 23) - 127 + 15;
    uint32_t man = absx & 0x7FFFFFu;
    if (exp >= 31) return (uint16_t)(sign | 0x7C00u);
    if (exp <= 0) {
        if (exp < -10) return sign;                 /* below half the smallest subnormal */
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - exp);      /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half_man = man >> 13;
    uint32_t rem = man & 0x1FFFu;
    uint16_t h = (uint16_t)(sign | ((uint32_t)exp << 10) | half_man);
    if (rem > 0x1000u || (rem == 0x1000u && (half_man & 1u))) h++;   /* may carry into exponent */
    return h;
}

uint16_t q40_ref_f2h(float f) { return f2h(f); }
float q40_ref_h2f(uint16_t h) { return h2f(h); }

/* nibble pattern (0..15, two's complement) times fp16 scale, one fp16 rounding.
 * |code| <= 8 needs 4 bits and an fp16 significand 11, so the float product is exact. */
uint16_t q40_ref_mul(int nibble, uint16_t scale) {
    int q = (nibble & 8) ? (nibble & 15) - 16 : (nibble & 15);
    return f2h((float)q * h2f(scale));
}

/* table[p * 65536 + s] for all 16 nibble patterns and all fp16 scale patterns */
void q40_ref_dequant_table(uint16_t *table) {
    for (int p = 0; p < 16; ++p)
        for (uint32_t s = 0; s < 65536u; ++s)
            table[(size_t)p * 65536u + s] = q40_ref_mul(p, (uint16_t)s);
}

/* rows: number of 64-byte packed rows; out: rows*128 fp16 patterns, high-nibble group first */
void q40_ref_dequantize(const int8_t *w, const uint16_t *s, long rows, uint16_t *out) {
    for (long r = 0; r < rows; ++r) {
        for (int j = 0; j < 64; ++j) {
            uint8_t b = (uint8_t)w[r * 64 + j];
            out[r * 128 + j] = q40_ref_mul(b >> 4, s[2 * r]);
            out[r * 128 + 64 + j] = q40_ref_mul(b & 15, s[2 * r + 1]);
        }
    }
}

/* scale = fp16(absmax / 7) with a true float division */
uint16_t q40_ref_scale(uint16_t absmax) { return f2h(h2f(absmax) / 7.0f); }

/* one code: fp16(w / scale) rounded half-to-even to an integer; NaN (0/0) gives 0 */
int q40_ref_code(uint16_t w, uint16_t scale) {
    float q = h2f(f2h(h2f(w) / h2f(scale)));
    if (q != q) return 0;
    return (int)nearbyintf(q);       /* default rounding mode: to nearest even */
}

/* groups: number of 64-value groups (even); in: fp16 patterns; w: groups/2 rows of 64 bytes */
void q40_ref_quantize(const uint16_t *in, long groups, int8_t *w, uint16_t *s) {
    for (long g = 0; g < groups; ++g) {
        uint16_t amax = 0;
        for (int j = 0; j < 64; ++j) {
            uint16_t a = (uint16_t)(in[g * 64 + j] & 0x7FFFu);
            if (a > amax) amax = a;                 /* magnitude order == bit order for finite */
        }
        uint16_t sc = q40_ref_scale(amax);
        s[g] = sc;
        for (int j = 0; j < 64; ++j) {
            int c = q40_ref_code(in[g * 64 + j], sc) & 15;
            uint8_t *dst = (uint8_t *)&w[(g / 2) * 64 + j];
            if ((g & 1) == 0) *dst = (uint8_t)(c << 4);
            else *dst = (uint8_t)(*dst | c);
        }
    }
}
