/*
 * iom_oracle.c — CPU restatement of the reference CPU backend (see
 * iom_oracle.h).  TEST INFRASTRUCTURE ONLY: nothing shipped may link this.
 *
 * Build without FMA contraction and without ISA flags (plain -O2
 * -ffp-contract=off): the reference's sequential F32 recurrences
 * `sum + v*v` and `(v*inverse)*scale` must stay two roundings.
 */
#include "iom_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define TILE 16u
#define TILE_SLOTS 256u

/* ------------------------------------------------------------------ */
/* Layout (src/tensor.cpp:76-164)                                       */
/* ------------------------------------------------------------------ */

unsigned iomo_leaf_bits(int dtype) {
    switch (dtype) {
        case IOMO_DT_I2: case IOMO_DT_U2: return 2;
        case IOMO_DT_I4: case IOMO_DT_U4: case IOMO_DT_F4_E2M1: return 4;
        case IOMO_DT_F6_E2M3: case IOMO_DT_F6_E3M2: return 6;
        case IOMO_DT_BOOL: case IOMO_DT_I8: case IOMO_DT_U8: case IOMO_DT_F8_E4M3FN:
        case IOMO_DT_F8_E5M2: case IOMO_DT_F8_E8M0: return 8;
        case IOMO_DT_I16: case IOMO_DT_U16: case IOMO_DT_F16: case IOMO_DT_BF16: return 16;
        case IOMO_DT_I32: case IOMO_DT_U32: case IOMO_DT_F32: return 32;
        case IOMO_DT_I64: case IOMO_DT_U64: case IOMO_DT_F64: return 64;
        default: return 0;
    }
}

size_t iomo_leaf_bytes(int dtype) {
    const unsigned bits = iomo_leaf_bits(dtype);
    return bits % 8 == 0 ? bits / 8 : 0;
}

static uint64_t tiles_of(uint64_t extent) { return (extent + TILE - 1) / TILE; }

uint64_t iomo_plane_elems(uint64_t rows, uint64_t cols) {
    return tiles_of(rows) * tiles_of(cols) * TILE_SLOTS;
}

uint64_t iomo_plane_slot(uint64_t rows, uint64_t cols, uint64_t plane,
                         uint64_t row, uint64_t col) {
    const uint64_t tile_cols = tiles_of(cols);
    const uint64_t tiles_per_plane = tiles_of(rows) * tile_cols;
    const uint64_t tile = plane * tiles_per_plane + (row / TILE) * tile_cols
            + col / TILE;
    return tile * TILE_SLOTS + (row % TILE) * TILE + col % TILE;
}

/* Packed elements: element `slot` occupies bits [slot*bits, (slot+1)*bits) of a
 * little-endian bit stream, least significant bit first
 * (src/cpu/transfer_helpers.hpp:14-40). */
static uint64_t load_leaf(const void* base, uint64_t slot, unsigned bits) {
    const unsigned char* p = (const unsigned char*)base;
    if (bits % 8 == 0) {
        uint64_t v = 0;
        memcpy(&v, p + slot * (bits / 8), bits / 8);
        return v;
    }
    uint64_t v = 0;
    const uint64_t first = slot * bits;
    for (unsigned i = 0; i < bits; ++i) {
        const uint64_t bit = first + i;
        v |= (uint64_t)((p[bit >> 3] >> (bit & 7)) & 1u) << i;
    }
    return v;
}

static void store_leaf(void* base, uint64_t slot, unsigned bits, uint64_t raw) {
    unsigned char* p = (unsigned char*)base;
    if (bits % 8 == 0) {
        memcpy(p + slot * (bits / 8), &raw, bits / 8);
        return;
    }
    const uint64_t first = slot * bits;
    for (unsigned i = 0; i < bits; ++i) {
        const uint64_t bit = first + i;
        const unsigned char mask = (unsigned char)(1u << (bit & 7));
        if ((raw >> i) & 1u) p[bit >> 3] |= mask;
        else p[bit >> 3] &= (unsigned char)~mask;
    }
}

/* ------------------------------------------------------------------ */
/* Named-format codec (src/shared/scalar_binary_codec.hpp:30-148)       */
/* ------------------------------------------------------------------ */

typedef struct {
    unsigned ebits, fbits;
    int bias;
    int finite_only; /* no infinities; NaN only when ebits >= 4 (all of the top exponent) */
    int infs;
} fmt_t;

/* :30-43 */
static int float_format(int dtype, fmt_t* f) {
    switch (dtype) {
        case IOMO_DT_F4_E2M1:   *f = (fmt_t){2, 1, 1, 1, 0}; return 1;
        case IOMO_DT_F6_E2M3:   *f = (fmt_t){2, 3, 1, 1, 0}; return 1;
        case IOMO_DT_F6_E3M2:   *f = (fmt_t){3, 2, 3, 1, 0}; return 1;
        case IOMO_DT_F8_E4M3FN: *f = (fmt_t){4, 3, 7, 1, 0}; return 1;
        case IOMO_DT_F8_E5M2:   *f = (fmt_t){5, 2, 15, 0, 1}; return 1;
        case IOMO_DT_F16:       *f = (fmt_t){5, 10, 15, 0, 1}; return 1;
        case IOMO_DT_BF16:      *f = (fmt_t){8, 7, 127, 0, 1}; return 1;
        case IOMO_DT_F32:       *f = (fmt_t){8, 23, 127, 0, 1}; return 1;
        case IOMO_DT_F64:       *f = (fmt_t){11, 52, 1023, 0, 1}; return 1;
        default: return 0;
    }
}

static unsigned integer_width(int dtype) {
    switch (dtype) {
        case IOMO_DT_I2: case IOMO_DT_U2: case IOMO_DT_I4: case IOMO_DT_U4:
        case IOMO_DT_I8: case IOMO_DT_U8: case IOMO_DT_I16: case IOMO_DT_U16:
        case IOMO_DT_I32: case IOMO_DT_U32: case IOMO_DT_I64: case IOMO_DT_U64:
            return iomo_leaf_bits(dtype);
        default: return 0;
    }
}

/* The top exponent is special (infinity / NaN) unless the format is one of the
 * finite-only ones narrower than four exponent bits (:50-55). */
static int top_exponent_is_special(fmt_t f) { return !f.finite_only || f.ebits >= 4; }

/* :45-65 */
static long double codec_decode(uint64_t raw, fmt_t f) {
    const uint64_t emask = (1ull << f.ebits) - 1;
    const uint64_t sign = (raw >> (f.ebits + f.fbits)) & 1;
    const uint64_t frac = raw & ((1ull << f.fbits) - 1);
    const uint64_t exp = (raw >> f.fbits) & emask;
    long double v;
    if (exp == emask && top_exponent_is_special(f)) {
        if (f.infs && frac == 0) return sign ? -(long double)INFINITY : (long double)INFINITY;
        return (long double)NAN;
    }
    if (exp != 0) {
        v = ldexpl((long double)((1ull << f.fbits) + frac),
                   (int)exp - f.bias - (int)f.fbits);
    } else {
        v = ldexpl((long double)frac, 1 - f.bias - (int)f.fbits);
    }
    return sign ? -v : v;
}

/* :110-118 */
static uint64_t codec_round_even(long double v) {
    const long double whole = floorl(v);
    const long double rest = v - whole;
    uint64_t q = (uint64_t)whole;
    if (rest > 0.5L || (rest == 0.5L && (q & 1))) ++q;
    return q;
}

/* :67-108.  Overflow stores infinity where the format has one and the largest
 * finite magnitude otherwise; NaN stores exponent all-ones with the top
 * fraction bit (every fraction bit for F8_E4M3FN), and the largest finite
 * magnitude in the formats that have no NaN at all. */
static uint64_t codec_encode(long double v, fmt_t f) {
    const uint64_t sign = signbit(v) ? 1 : 0;
    const uint64_t emask = (1ull << f.ebits) - 1;
    const uint64_t fmask = (1ull << f.fbits) - 1;
    const unsigned shift = f.ebits + f.fbits;
    const uint64_t finite_emax = top_exponent_is_special(f) ? emask - 1 : emask;
    const uint64_t overflow = (sign << shift)
            | (f.infs ? emask << f.fbits : (finite_emax << f.fbits) | fmask);
    v = fabsl(v);
    if (isnan(v)) {
        if (!top_exponent_is_special(f)) return overflow;
        return (sign << shift) | (emask << f.fbits)
                | (f.finite_only ? fmask : 1ull << (f.fbits - 1));
    }
    if (isinf(v)) return overflow;
    if (v == 0) return sign << shift;
    const int min_sub = 1 - f.bias - (int)f.fbits;
    const int max_exp = (int)finite_emax - f.bias;
    int e = 0;
    (void)frexpl(v, &e);
    --e;
    if (e < min_sub + (int)f.fbits) {
        const uint64_t q = codec_round_even(ldexpl(v, -min_sub));
        if (q == (1ull << f.fbits)) return (sign << shift) | (1ull << f.fbits);
        return (sign << shift) | q;
    }
    if (e > max_exp) return overflow;
    uint64_t frac = codec_round_even(
            ldexpl(v, (int)f.fbits - e) - (long double)(1ull << f.fbits));
    if (frac == (1ull << f.fbits)) { ++e; frac = 0; }
    if (e > max_exp) return overflow;
    return (sign << shift) | ((uint64_t)(e + f.bias) << f.fbits) | frac;
}

/* :120-148 */
static long double codec_arith(int op, long double x, long double y) {
    if (isnan(x) || isnan(y)) return (long double)NAN;
    if (op == IOMO_OP_ADD) {
        if (isinf(x) && isinf(y) && signbit(x) != signbit(y)) return (long double)NAN;
        if (x == 0 && y == 0) return (signbit(x) && signbit(y)) ? -0.0L : 0.0L;
        const long double r = x + y;
        return r == 0 ? 0.0L : r;
    }
    if (op == IOMO_OP_MUL) {
        if ((isinf(x) && y == 0) || (isinf(y) && x == 0)) return (long double)NAN;
        return x * y;
    }
    if (op == IOMO_OP_SUB) {
        if (isinf(x) && isinf(y) && signbit(x) == signbit(y)) return (long double)NAN;
        return x - y;
    }
    if ((x == 0 && y == 0) || (isinf(x) && isinf(y))) return (long double)NAN;
    return x / y;
}

static long double positive_nan(void) { return fabsl((long double)NAN); }

/* The codec stores every NaN as sign 0, exponent all-ones, top fraction bit
 * (:79-84, quiet_nan() has a clear sign on x86-64). */
uint64_t iomo_scalar_binary(int op, int dtype, uint64_t a, uint64_t b) {
    const unsigned width = integer_width(dtype);
    if (width) {
        const uint64_t mask = width == 64 ? ~0ull : (1ull << width) - 1;
        if (op == IOMO_OP_DIV) return 0;   /* :166; refused before it is reached */
        if (op == IOMO_OP_ADD) return (a + b) & mask;
        if (op == IOMO_OP_MUL) return (a * b) & mask;
        return (a - b) & mask;
    }
    fmt_t f;
    if (!float_format(dtype, &f)) return 0;
    long double r = codec_arith(op, codec_decode(a, f), codec_decode(b, f));
    if (isnan(r)) r = positive_nan();
    return codec_encode(r, f);
}

uint16_t iomo_encode_bf16(float value) {
    fmt_t f;
    float_format(IOMO_DT_BF16, &f);
    if (isnan(value)) return 0x7FC0u;
    return (uint16_t)codec_encode((long double)value, f);
}

/* ---- closed form: one IEEE-754 operation and one rounding ------------ */

static float f32_from_bits(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }
static uint32_t f32_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }
static double f64_from_bits(uint64_t b) { double f; memcpy(&f, &b, 8); return f; }
static uint64_t f64_bits(double f) { uint64_t b; memcpy(&b, &f, 8); return b; }

static uint16_t bf16_rne_bits(uint32_t bits) {
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0u;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

/* Value of a narrow encoding as a binary64 number, by integer construction
 * (every format of at most 32 bits is a subset of binary64).  *special: 0 finite,
 * 1 infinity, 2 NaN. */
static double narrow_value(uint64_t raw, fmt_t f, int* special) {
    const uint64_t emask = (1ull << f.ebits) - 1;
    const int negative = (int)((raw >> (f.ebits + f.fbits)) & 1);
    const uint64_t frac = raw & ((1ull << f.fbits) - 1);
    const uint64_t exp = (raw >> f.fbits) & emask;
    *special = 0;
    if (exp == emask && top_exponent_is_special(f)) {
        *special = (f.infs && frac == 0) ? 1 : 2;
        if (*special == 2) return NAN;
        return negative ? -INFINITY : INFINITY;
    }
    const int64_t m = (int64_t)(exp ? (1ull << f.fbits) + frac : frac);
    const int scale = (int)(exp ? exp : 1) - f.bias - (int)f.fbits;
    const double v = ldexp((double)m, scale);
    return negative ? -v : v;
}

/* One round-to-nearest-even of a finite binary64 value onto a narrow format's
 * grid, done on the integer significand (no floating-point operation rounds
 * here).  `v` must be a normal binary64 number or zero. */
static uint64_t narrow_round(double v, fmt_t f) {
    const uint64_t emask = (1ull << f.ebits) - 1;
    const uint64_t fmask = (1ull << f.fbits) - 1;
    const unsigned shift = f.ebits + f.fbits;
    const uint64_t b = f64_bits(v);
    const uint64_t sign = (b >> 63) << shift;
    const uint64_t finite_emax = top_exponent_is_special(f) ? emask - 1 : emask;
    const uint64_t overflow = sign | (f.infs ? emask << f.fbits : (finite_emax << f.fbits) | fmask);
    const uint64_t mag = b & 0x7FFFFFFFFFFFFFFFull;
    if (mag == 0) return sign;
    const int e = (int)(mag >> 52) - 1023;                  /* unbiased, v = 1.m * 2^e */
    const uint64_t m = (mag & 0xFFFFFFFFFFFFFull) | (1ull << 52);
    const int emin = 1 - f.bias;                             /* smallest normal exponent */
    /* the kept integer q counts units of 2^(max(e,emin) - fbits) */
    int drop = 52 - (int)f.fbits + (e < emin ? emin - e : 0);
    uint64_t q, rest, half;
    if (drop > 62) { q = 0; rest = 1; half = 2; }            /* far below half a unit */
    else {
        q = m >> drop;
        rest = m & ((1ull << drop) - 1);
        half = 1ull << (drop - 1);
    }
    if (rest > half || (rest == half && (q & 1))) ++q;
    /* a normal q carries the implicit bit, which adds one to the exponent field;
     * a subnormal q that reaches 2^fbits becomes the smallest normal the same way */
    const uint64_t field = e < emin ? q : ((uint64_t)(e + f.bias - 1) << f.fbits) + q;
    if ((field >> f.fbits) > finite_emax) return overflow;
    return sign | field;
}

static uint64_t narrow_nan(fmt_t f) {
    const uint64_t emask = (1ull << f.ebits) - 1;
    const uint64_t fmask = (1ull << f.fbits) - 1;
    if (!top_exponent_is_special(f)) return (emask << f.fbits) | fmask;   /* saturates */
    return (emask << f.fbits) | (f.finite_only ? fmask : 1ull << (f.fbits - 1));
}

/* Quotient of two finite non-zero values of a format of at most 16 bits, rounded once:
 * the operands are integers times powers of two (at most 11 significand bits), so the
 * quotient's leading 40-odd bits come from one integer division, and the remainder
 * becomes a sticky bit below them.  That integer, scaled, is an exact binary64 number
 * which lies strictly between the same pair of neighbours of the narrow grid, and on
 * the same side of their midpoint, as the true quotient; narrow_round does the rest. */
static uint64_t narrow_quotient(uint64_t a, uint64_t b, fmt_t f) {
    const uint64_t emask = (1ull << f.ebits) - 1, fmask = (1ull << f.fbits) - 1;
    const uint64_t ea = (a >> f.fbits) & emask, eb = (b >> f.fbits) & emask;
    const uint64_t ma = ea ? (1ull << f.fbits) + (a & fmask) : (a & fmask);
    const uint64_t mb = eb ? (1ull << f.fbits) + (b & fmask) : (b & fmask);
    const int sa = (int)(ea ? ea : 1), sb = (int)(eb ? eb : 1);   /* the bias and fbits cancel */
    const int negative = (int)(((a ^ b) >> (f.ebits + f.fbits)) & 1);
    const uint64_t n = ma << 40;
    const uint64_t q = ((n / mb) << 1) | (n % mb != 0);
    const double v = ldexp((double)q, sa - sb - 41);             /* q < 2^53: exact */
    return narrow_round(negative ? -v : v, f);
}

uint64_t iomo_scalar_binary_ieee(int op, int dtype, uint64_t a, uint64_t b) {
    const unsigned width = integer_width(dtype);
    if (width && op == IOMO_OP_DIV) return 0;
    if (width == 64) {
        if (op == IOMO_OP_ADD) return a + b;
        if (op == IOMO_OP_MUL) return a * b;
        return a - b;
    }
    if (width) {
        /* two's-complement wrap in the native width */
        const uint32_t x = (uint32_t)a, y = (uint32_t)b;
        const uint32_t mask = width == 32 ? 0xFFFFFFFFu : (1u << width) - 1;
        if (op == IOMO_OP_ADD) return (uint32_t)(x + y) & mask;
        if (op == IOMO_OP_MUL) return (uint32_t)(x * y) & mask;
        return (uint32_t)(x - y) & mask;
    }
    if (dtype == IOMO_DT_F32) {
        const volatile float x = f32_from_bits((uint32_t)a);
        const volatile float y = f32_from_bits((uint32_t)b);
        volatile float r;
        if (op == IOMO_OP_ADD) r = x + y;
        else if (op == IOMO_OP_MUL) r = x * y;
        else if (op == IOMO_OP_SUB) r = x - y;
        else r = x / y;
        if (r != r) return 0x7FC00000u;
        return f32_bits(r);
    }
    if (dtype == IOMO_DT_F64) {
        /* binary64 carrier: the rule of a backend without an extended type
         * (src/shared/standard_tiled_add.inl:116).  The x87 carrier of the host
         * codec rounds twice here and may differ in the last place. */
        const volatile double x = f64_from_bits(a), y = f64_from_bits(b);
        volatile double r;
        if (op == IOMO_OP_ADD) r = x + y;
        else if (op == IOMO_OP_MUL) r = x * y;
        else if (op == IOMO_OP_SUB) r = x - y;
        else r = x / y;
        if (r != r) return 0x7FF8000000000000ull;
        return f64_bits(r);
    }
    if (dtype == IOMO_DT_BF16 && op != IOMO_OP_DIV) {
        const float x = f32_from_bits((uint32_t)a << 16);
        const float y = f32_from_bits((uint32_t)b << 16);
        if (op == IOMO_OP_MUL) {
            /* The product of two 8-bit significands is exact in binary64 and
             * binary64 has the exponent range for it, so one rounding from the
             * exact value is what remains.  Round on the BF16 grid directly. */
            const double p = (double)x * (double)y;
            if (p != p) return 0x7FC0u;
            if (isinf(p)) return p < 0 ? 0xFF80u : 0x7F80u;
            const double m = fabs(p);
            const uint64_t sign = signbit(p) ? 0x8000u : 0;
            if (m == 0) return sign;
            int e;
            (void)frexp(m, &e); /* m = f * 2^e, f in [0.5,1) */
            --e;
            int quantum = e - 7;              /* normal BF16 ulp exponent */
            if (quantum < -133) quantum = -133; /* subnormal grid 2^-133   */
            const double scaled = ldexp(m, -quantum); /* exact */
            double q = floor(scaled);
            const double rest = scaled - q;
            if (rest > 0.5 || (rest == 0.5 && fmod(q, 2.0) != 0)) q += 1;
            const double rounded = ldexp(q, quantum);
            if (rounded > 3.3895313892515355e38) return sign | 0x7F80u;
            const float back = (float)rounded; /* exact: on the BF16 grid */
            return sign | (f32_bits(back) >> 16);
        }
        const volatile float r = (op == IOMO_OP_ADD) ? x + y : x - y;
        return bf16_rne_bits(f32_bits(r));
    }
    fmt_t f;
    if (!float_format(dtype, &f)) return 0;
    /* F16 and the 4/6/8-bit formats: sums, differences and products of two
     * values are exact in binary64 (at most 11 significand bits each, exponents
     * within 2^-24 .. 2^16), so the single rounding below is the only one. */
    int sx, sy;
    const double x = narrow_value(a, f, &sx), y = narrow_value(b, f, &sy);
    if (sx == 2 || sy == 2) return narrow_nan(f);
    if (op == IOMO_OP_DIV) {
        const uint64_t emask = (1ull << f.ebits) - 1, fmask = (1ull << f.fbits) - 1;
        const uint64_t finite_emax = top_exponent_is_special(f) ? emask - 1 : emask;
        const uint64_t sign = ((a ^ b) >> (f.ebits + f.fbits) & 1) << (f.ebits + f.fbits);
        if ((sx == 1 && sy == 1) || (x == 0 && y == 0)) return narrow_nan(f);
        if (sx == 1 || y == 0)   /* infinite quotient: infinity, or the largest finite value */
            return sign | (f.infs ? emask << f.fbits : (finite_emax << f.fbits) | fmask);
        if (sy == 1 || x == 0) return sign;
        return narrow_quotient(a, b, f);
    }
    if (op == IOMO_OP_MUL) {
        if ((sx == 1 && y == 0) || (sy == 1 && x == 0)) return narrow_nan(f);
    } else if (sx == 1 && sy == 1) {
        const int same = signbit(x) == signbit(y);
        if ((op == IOMO_OP_ADD) != same) return narrow_nan(f);
    }
    double r;
    if (op == IOMO_OP_ADD) {
        if (x == 0 && y == 0) r = (signbit(x) && signbit(y)) ? -0.0 : 0.0;
        else { r = x + y; if (r == 0) r = 0.0; }
    } else if (op == IOMO_OP_MUL) {
        r = x * y;
    } else {
        r = x - y;
    }
    if (isinf(r)) {
        const uint64_t emask = (1ull << f.ebits) - 1;
        return ((uint64_t)(signbit(r) ? 1 : 0) << (f.ebits + f.fbits)) | (emask << f.fbits);
    }
    return narrow_round(r, f);
}

/* ------------------------------------------------------------------ */
/* SiLU (src/shared/scalar_silu.hpp:69-97, float carrier)               */
/* ------------------------------------------------------------------ */

static float silu_f32(float x) {
    if (isnan(x)) return NAN;
    if (isinf(x)) return signbit(x) ? -0.0f : INFINITY;
    if (x == 0.0f) return x;
    if (x >= 0.0f) {
        const volatile float e = expf(-x);
        const volatile float d = 1.0f + e;
        return x / d;
    }
    const volatile float t = expf(x * 0.5f);
    const volatile float xt = x * t;
    const volatile float num = xt * t;
    const volatile float tt = t * t;
    const volatile float den = 1.0f + tt;
    return num / den;
}

static double silu_f64(double x) {
    if (isnan(x)) return NAN;
    if (isinf(x)) return signbit(x) ? -0.0 : INFINITY;
    if (x == 0.0) return x;
    if (x >= 0.0) {
        const volatile double e = exp(-x);
        const volatile double d = 1.0 + e;
        return x / d;
    }
    const volatile double t = exp(x * 0.5);
    const volatile double xt = x * t;
    const volatile double num = xt * t;
    const volatile double tt = t * t;
    const volatile double den = 1.0 + tt;
    return num / den;
}

/* Carrier: binary32 for every leaf below F64, binary64 for F64
 * (src/cpu/queue.cpp:1769-1773). */
uint64_t iomo_scalar_silu(int dtype, uint64_t raw) {
    fmt_t f;
    if (!float_format(dtype, &f)) return 0;
    long double y;
    if (dtype == IOMO_DT_F64) y = (long double)silu_f64((double)codec_decode(raw, f));
    else y = (long double)silu_f32((float)codec_decode(raw, f));
    if (isnan(y)) y = positive_nan();
    return codec_encode(y, f);
}

/* ------------------------------------------------------------------ */
/* View helpers                                                         */
/* ------------------------------------------------------------------ */

static int view_ok(const iomo_view* v) {
    if (!v || !v->base || v->rank < 2 || v->rank > 8) return 0;
    for (uint32_t i = 0; i < v->rank; ++i) if (v->dims[i] == 0) return 0;
    return 1;
}

static uint64_t view_rows(const iomo_view* v) { return v->dims[v->rank - 2]; }
static uint64_t view_cols(const iomo_view* v) { return v->dims[v->rank - 1]; }

/* Row-major walk over the leading coordinates of `dims[0..leading)`. */
static int next_coord(uint64_t* coord, const uint64_t* dims, uint32_t leading) {
    for (uint32_t i = leading; i-- > 0;) {
        if (++coord[i] < dims[i]) return 1;
        coord[i] = 0;
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* Binary (src/cpu/queue.cpp:414-536)                                   */
/* ------------------------------------------------------------------ */

typedef struct {
    uint64_t strides[6]; /* result-aligned, 0 on broadcast / missing axes */
    int bcast_rows, bcast_cols;
} bsnap_t;

/* src/device_ops_binary.cpp:61-100 */
static void snapshot(const iomo_view* v, const uint64_t* rdims, uint32_t rrank,
                     bsnap_t* s) {
    const uint32_t offset = rrank - v->rank;
    const uint32_t rleading = rrank - 2;
    for (uint32_t axis = 0; axis < rleading; ++axis) {
        s->strides[axis] = 0;
        if (axis < offset) continue;
        const uint32_t src = axis - offset;
        if (v->dims[src] == 1 && rdims[axis] != 1) continue;
        s->strides[axis] = v->plane_strides[src];
    }
    s->bcast_rows = view_rows(v) == 1 && rdims[rrank - 2] != 1;
    s->bcast_cols = view_cols(v) == 1 && rdims[rrank - 1] != 1;
}

int iomo_binary(int op, int dtype, const iomo_view* lhs, const iomo_view* rhs,
                const iomo_view* out, int use_ieee) {
    const unsigned bits = iomo_leaf_bits(dtype);
    fmt_t numeric;
    if (!bits || (!integer_width(dtype) && !float_format(dtype, &numeric)))
        return IOMO_ERR_UNSUPPORTED;   /* BOOL and F8_E8M0 (src/device_ops_binary.cpp:26-46) */
    if (op < IOMO_OP_ADD || op > IOMO_OP_DIV) return IOMO_ERR_INVALID;
    if (!view_ok(lhs) || !view_ok(rhs) || !view_ok(out)) return IOMO_ERR_INVALID;
    /* src/device_ops_binary.cpp:121-143: right-aligned broadcast */
    const uint32_t rank = lhs->rank > rhs->rank ? lhs->rank : rhs->rank;
    uint64_t rdims[8];
    for (uint32_t i = 0; i < rank; ++i) {
        const uint64_t l = i < rank - lhs->rank ? 1 : lhs->dims[i - (rank - lhs->rank)];
        const uint64_t r = i < rank - rhs->rank ? 1 : rhs->dims[i - (rank - rhs->rank)];
        if (l != r && l != 1 && r != 1) return IOMO_ERR_INVALID;
        rdims[i] = l > r ? l : r;
    }
    if (out->rank != rank) return IOMO_ERR_INVALID;
    for (uint32_t i = 0; i < rank; ++i)
        if (out->dims[i] != rdims[i]) return IOMO_ERR_INVALID;
    /* src/device_ops_binary.cpp:174-175: division on the floating leaves only, refused
     * after the shape checks */
    if (op == IOMO_OP_DIV && integer_width(dtype)) return IOMO_ERR_UNSUPPORTED;

    bsnap_t ls, rs, os;
    snapshot(lhs, rdims, rank, &ls);
    snapshot(rhs, rdims, rank, &rs);
    snapshot(out, rdims, rank, &os);
    const uint32_t leading = rank - 2;
    const uint64_t rows = rdims[rank - 2], cols = rdims[rank - 1];
    uint64_t coord[8] = {0};
    do {
        uint64_t lp = lhs->plane_offset, rp = rhs->plane_offset, op_ = out->plane_offset;
        for (uint32_t a = 0; a < leading; ++a) {
            lp += coord[a] * ls.strides[a];
            rp += coord[a] * rs.strides[a];
            op_ += coord[a] * os.strides[a];
        }
        for (uint64_t r = 0; r < rows; ++r) {
            for (uint64_t c = 0; c < cols; ++c) {
                const uint64_t lslot = iomo_plane_slot(
                        view_rows(lhs), view_cols(lhs), lp,
                        ls.bcast_rows ? 0 : r, ls.bcast_cols ? 0 : c);
                const uint64_t rslot = iomo_plane_slot(
                        view_rows(rhs), view_cols(rhs), rp,
                        rs.bcast_rows ? 0 : r, rs.bcast_cols ? 0 : c);
                const uint64_t oslot = iomo_plane_slot(rows, cols, op_, r, c);
                const uint64_t a = load_leaf(lhs->base, lslot, bits);
                const uint64_t b = load_leaf(rhs->base, rslot, bits);
                const uint64_t y = use_ieee
                        ? iomo_scalar_binary_ieee(op, dtype, a, b)
                        : iomo_scalar_binary(op, dtype, a, b);
                store_leaf(out->base, oslot, bits, y);
            }
        }
    } while (next_coord(coord, rdims, leading));
    return IOMO_OK;
}

/* ------------------------------------------------------------------ */
/* RMSNorm (src/cpu/queue.cpp:1144-1296, float carrier)                 */
/* ------------------------------------------------------------------ */

#define RMSNORM_ROWS(T, SQRT)                                                              \
    do {                                                                                  \
        const T divisor = (T)feats;                                                       \
        const T epsilon = (T)eps;                                                         \
        for (uint64_t r = 0; r < rows; ++r) {                                             \
            volatile T sum = 0;                                                           \
            for (uint64_t c = 0; c < feats; ++c) {                                        \
                const T v = (T)codec_decode(                                              \
                        load_leaf(x->base, iomo_plane_slot(rows, feats, xp, r, c), bits), f); \
                const volatile T sq = v * v;                                              \
                sum = sum + sq;                                                           \
            }                                                                             \
            const volatile T mean = sum / divisor;                                        \
            const volatile T shifted = mean + epsilon;                                    \
            const volatile T root = SQRT(shifted);                                        \
            const volatile T inverse = (T)1 / root;                                       \
            for (uint64_t c = 0; c < feats; ++c) {                                        \
                const T v = (T)codec_decode(                                              \
                        load_leaf(x->base, iomo_plane_slot(rows, feats, xp, r, c), bits), f); \
                const T w = (T)codec_decode(                                              \
                        load_leaf(scale->base,                                            \
                                  iomo_plane_slot(1, feats, scale->plane_offset, 0, c), bits), f); \
                const volatile T normalized = v * inverse;                                \
                const volatile T y = normalized * w;                                      \
                /* a NaN result is stored in its positive form (:1124-1134) */           \
                const long double enc = (y != y) ? positive_nan() : (long double)y;       \
                store_leaf(out->base, iomo_plane_slot(rows, feats, yp, r, c), bits,       \
                           codec_encode(enc, f));                                         \
            }                                                                             \
        }                                                                                 \
    } while (0)

int iomo_rmsnorm(int dtype, const iomo_view* x, const iomo_view* scale,
                 const iomo_view* out, float eps) {
    fmt_t f;
    if (!view_ok(x) || !view_ok(scale) || !view_ok(out)) return IOMO_ERR_INVALID;
    if (x->rank != out->rank) return IOMO_ERR_INVALID;
    for (uint32_t i = 0; i < x->rank; ++i)
        if (x->dims[i] != out->dims[i]) return IOMO_ERR_INVALID;
    const uint64_t rows = view_rows(x), feats = view_cols(x);
    if (scale->rank != 2 || scale->dims[0] != 1 || scale->dims[1] != feats)
        return IOMO_ERR_INVALID;
    if (out->base == x->base || out->base == scale->base) return IOMO_ERR_INVALID;
    if (!float_format(dtype, &f)) return IOMO_ERR_UNSUPPORTED;
    if (!isfinite(eps) || eps < 0.0f) return IOMO_ERR_INVALID;
    const unsigned bits = iomo_leaf_bits(dtype);
    const uint32_t leading = x->rank - 2;
    uint64_t coord[8] = {0};
    do {
        uint64_t xp = x->plane_offset, yp = out->plane_offset;
        for (uint32_t a = 0; a < leading; ++a) {
            xp += coord[a] * x->plane_strides[a];
            yp += coord[a] * out->plane_strides[a];
        }
        /* carrier: binary64 for the F64 leaf, binary32 below (:1312-1317) */
        if (dtype == IOMO_DT_F64) RMSNORM_ROWS(double, sqrt);
        else RMSNORM_ROWS(float, sqrtf);
    } while (next_coord(coord, x->dims, leading));
    return IOMO_OK;
}

/* ------------------------------------------------------------------ */
/* SiLU / copy: two-view plane walks                                    */
/* ------------------------------------------------------------------ */

static int same_shape(const iomo_view* a, const iomo_view* b) {
    if (a->rank != b->rank) return 0;
    for (uint32_t i = 0; i < a->rank; ++i) if (a->dims[i] != b->dims[i]) return 0;
    return 1;
}

int iomo_silu(int dtype, const iomo_view* x, const iomo_view* y) {
    fmt_t f;
    if (!view_ok(x) || !view_ok(y) || !same_shape(x, y)) return IOMO_ERR_INVALID;
    if (!float_format(dtype, &f)) return IOMO_ERR_UNSUPPORTED;
    const unsigned bits = iomo_leaf_bits(dtype);
    const uint64_t rows = view_rows(x), cols = view_cols(x);
    const uint32_t leading = x->rank - 2;
    uint64_t coord[8] = {0};
    do {
        uint64_t xp = x->plane_offset, yp = y->plane_offset;
        for (uint32_t a = 0; a < leading; ++a) {
            xp += coord[a] * x->plane_strides[a];
            yp += coord[a] * y->plane_strides[a];
        }
        for (uint64_t r = 0; r < rows; ++r)
            for (uint64_t c = 0; c < cols; ++c)
                store_leaf(y->base, iomo_plane_slot(rows, cols, yp, r, c), bits,
                           iomo_scalar_silu(dtype, load_leaf(
                                   x->base, iomo_plane_slot(rows, cols, xp, r, c), bits)));
    } while (next_coord(coord, x->dims, leading));
    return IOMO_OK;
}

int iomo_copy(int dtype, const iomo_view* src, const iomo_view* dst) {
    const unsigned bits = iomo_leaf_bits(dtype);
    if (!bits) return IOMO_ERR_UNSUPPORTED;
    if (!view_ok(src) || !view_ok(dst) || !same_shape(src, dst)) return IOMO_ERR_INVALID;
    const uint64_t rows = view_rows(src), cols = view_cols(src);
    const uint32_t leading = src->rank - 2;
    uint64_t coord[8] = {0};
    do {
        uint64_t sp = src->plane_offset, dp = dst->plane_offset;
        for (uint32_t a = 0; a < leading; ++a) {
            sp += coord[a] * src->plane_strides[a];
            dp += coord[a] * dst->plane_strides[a];
        }
        for (uint64_t r = 0; r < rows; ++r)
            for (uint64_t c = 0; c < cols; ++c)
                store_leaf(dst->base, iomo_plane_slot(rows, cols, dp, r, c), bits,
                           load_leaf(src->base, iomo_plane_slot(rows, cols, sp, r, c), bits));
    } while (next_coord(coord, src->dims, leading));
    return IOMO_OK;
}

/* src/cpu/tensor.cpp:79-167: the logical side is dense row-major over the
 * view's own shape. */
int iomo_scatter(int dtype, const iomo_view* dst, const void* logical) {
    const unsigned bits = iomo_leaf_bits(dtype);
    if (!bits) return IOMO_ERR_UNSUPPORTED;
    if (!view_ok(dst) || !logical) return IOMO_ERR_INVALID;
    const uint64_t rows = view_rows(dst), cols = view_cols(dst);
    const uint32_t leading = dst->rank - 2;
    uint64_t coord[8] = {0};
    uint64_t index = 0;
    do {
        uint64_t dp = dst->plane_offset;
        for (uint32_t a = 0; a < leading; ++a) dp += coord[a] * dst->plane_strides[a];
        for (uint64_t r = 0; r < rows; ++r)
            for (uint64_t c = 0; c < cols; ++c, ++index)
                store_leaf(dst->base, iomo_plane_slot(rows, cols, dp, r, c), bits,
                           load_leaf(logical, index, bits));
    } while (next_coord(coord, dst->dims, leading));
    return IOMO_OK;
}

int iomo_gather(int dtype, const iomo_view* src, void* logical) {
    const unsigned bits = iomo_leaf_bits(dtype);
    if (!bits) return IOMO_ERR_UNSUPPORTED;
    if (!view_ok(src) || !logical) return IOMO_ERR_INVALID;
    const uint64_t rows = view_rows(src), cols = view_cols(src);
    const uint32_t leading = src->rank - 2;
    uint64_t coord[8] = {0};
    uint64_t index = 0;
    /* the unused high bits of a final partial byte read as zero
     * (src/cpu/tensor.cpp:126-135) */
    uint64_t count = 1;
    for (uint32_t i = 0; i < src->rank; ++i) count *= src->dims[i];
    if ((count * bits) % 8 != 0) ((unsigned char*)logical)[count * bits / 8] = 0;
    do {
        uint64_t sp = src->plane_offset;
        for (uint32_t a = 0; a < leading; ++a) sp += coord[a] * src->plane_strides[a];
        for (uint64_t r = 0; r < rows; ++r)
            for (uint64_t c = 0; c < cols; ++c, ++index)
                store_leaf(logical, index, bits,
                           load_leaf(src->base, iomo_plane_slot(rows, cols, sp, r, c), bits));
    } while (next_coord(coord, src->dims, leading));
    return IOMO_OK;
}

/* ------------------------------------------------------------------ */
/* Cache append, embedding, RoPE                                        */
/* ------------------------------------------------------------------ */

/* src/cpu/queue.cpp:2227-2272, admission of src/device_ops_cache_append.cpp:160-270
 * (what can be checked without owner identities). */
int iomo_cache_append(int dtype, const iomo_view* src, const iomo_view* dst, uint64_t a) {
    const unsigned bits = iomo_leaf_bits(dtype);
    if (!view_ok(src) || !view_ok(dst)) return IOMO_ERR_INVALID;
    if (src->rank < 3 || src->rank != dst->rank) return IOMO_ERR_INVALID;
    const uint32_t rank = src->rank;
    for (uint32_t i = 0; i + 2 < rank; ++i)
        if (src->dims[i] != dst->dims[i]) return IOMO_ERR_INVALID;
    if (view_cols(src) != view_cols(dst)) return IOMO_ERR_INVALID;
    const uint64_t capacity = view_rows(dst), rows = view_rows(src), feats = view_cols(src);
    if (a > capacity || rows > capacity - a) return IOMO_ERR_INVALID;
    if (src->base == dst->base) return IOMO_ERR_INVALID;
    if (!bits) return IOMO_ERR_UNSUPPORTED;
    const uint32_t leading = rank - 2;
    uint64_t coord[8] = {0};
    do {
        uint64_t sp = src->plane_offset, dp = dst->plane_offset;
        for (uint32_t k = 0; k < leading; ++k) {
            sp += coord[k] * src->plane_strides[k];
            dp += coord[k] * dst->plane_strides[k];
        }
        for (uint64_t r = 0; r < rows; ++r)
            for (uint64_t c = 0; c < feats; ++c)
                store_leaf(dst->base, iomo_plane_slot(capacity, feats, dp, a + r, c), bits,
                           load_leaf(src->base, iomo_plane_slot(rows, feats, sp, r, c), bits));
    } while (next_coord(coord, src->dims, leading));
    return IOMO_OK;
}

/* src/cpu/queue.cpp:941-1038.  table [V,F] (rank two, one selected plane), indices
 * [...,1,R] of an integer leaf, out [...,R,F].  Every index is checked before
 * anything is written; a negative or out-of-vocabulary one gives
 * IOMO_ERR_INVALID (the CPU worker's deferred std::invalid_argument). */
int iomo_embedding(int dtype, int index_dtype, const iomo_view* table, const iomo_view* indices,
                   const iomo_view* out) {
    const unsigned bits = iomo_leaf_bits(dtype);
    const unsigned ibits = integer_width(index_dtype);
    if (!view_ok(table) || !view_ok(indices) || !view_ok(out)) return IOMO_ERR_INVALID;
    if (table->rank != 2 || indices->rank != out->rank) return IOMO_ERR_INVALID;
    const uint32_t rank = out->rank;
    for (uint32_t i = 0; i + 2 < rank; ++i)
        if (indices->dims[i] != out->dims[i]) return IOMO_ERR_INVALID;
    const uint64_t run = view_cols(indices), vocab = table->dims[0], feats = table->dims[1];
    if (view_rows(indices) != 1 || view_rows(out) != run || view_cols(out) != feats)
        return IOMO_ERR_INVALID;
    if (out->base == table->base || out->base == indices->base) return IOMO_ERR_INVALID;
    if (!bits || !ibits) return IOMO_ERR_UNSUPPORTED;
    const int is_signed = index_dtype == IOMO_DT_I2 || index_dtype == IOMO_DT_I4
            || index_dtype == IOMO_DT_I8 || index_dtype == IOMO_DT_I16
            || index_dtype == IOMO_DT_I32 || index_dtype == IOMO_DT_I64;
    const uint32_t leading = rank - 2;
    for (int pass = 0; pass < 2; ++pass) {
        uint64_t coord[8] = {0};
        do {
            uint64_t ip = indices->plane_offset, op = out->plane_offset;
            for (uint32_t k = 0; k < leading; ++k) {
                ip += coord[k] * indices->plane_strides[k];
                op += coord[k] * out->plane_strides[k];
            }
            for (uint64_t r = 0; r < run; ++r) {
                const uint64_t raw = load_leaf(indices->base, iomo_plane_slot(1, run, ip, 0, r), ibits);
                if (pass == 0) {
                    if (is_signed && ((raw >> (ibits - 1)) & 1)) return IOMO_ERR_INVALID;
                    if (raw >= vocab) return IOMO_ERR_INVALID;
                    continue;
                }
                for (uint64_t f = 0; f < feats; ++f)
                    store_leaf(out->base, iomo_plane_slot(run, feats, op, r, f), bits,
                               load_leaf(table->base,
                                         iomo_plane_slot(vocab, feats, table->plane_offset, raw, f), bits));
            }
        } while (next_coord(coord, out->dims, leading));
    }
    return IOMO_OK;
}

/* src/cpu/queue.cpp:1341-1581: split-half rotary encoding of [...,H,R,D] in the
 * carrier T (binary32 below F64, binary64 for F64).  A row at absolute position 0
 * is a raw copy; otherwise for c < D/2: frequency = pow(theta, -2c/D),
 * angle = position * frequency, and the four products and the following
 * subtraction / addition stay separate roundings. */
#define ROPE_ROWS(T, POW, SIN, COS)                                                        \
    do {                                                                                  \
        const T base = (T)theta;                                                          \
        for (uint64_t r = 0; r < rows; ++r) {                                             \
            const uint64_t position = a + r;                                              \
            if (position == 0) {                                                          \
                for (uint64_t c = 0; c < width; ++c)                                      \
                    store_leaf(out->base, iomo_plane_slot(rows, width, yp, r, c), bits,   \
                               load_leaf(x->base, iomo_plane_slot(rows, width, xp, r, c), bits)); \
                continue;                                                                 \
            }                                                                             \
            for (uint64_t c = 0; c < half; ++c) {                                         \
                const T first = (T)codec_decode(                                          \
                        load_leaf(x->base, iomo_plane_slot(rows, width, xp, r, c), bits), f); \
                const T second = (T)codec_decode(                                         \
                        load_leaf(x->base, iomo_plane_slot(rows, width, xp, r, c + half), bits), f); \
                const T exponent = (T)((-2.0 * (double)c) / (double)width);               \
                const T frequency = POW(base, exponent);                                  \
                const T angle = (T)position * frequency;                                  \
                const T sine = SIN(angle), cosine = COS(angle);                           \
                const volatile T p0 = first * cosine;                                     \
                const volatile T p1 = second * sine;                                      \
                const volatile T o0 = p0 - p1;                                            \
                const volatile T p2 = second * cosine;                                    \
                const volatile T p3 = first * sine;                                       \
                const volatile T o1 = p2 + p3;                                            \
                store_leaf(out->base, iomo_plane_slot(rows, width, yp, r, c), bits,       \
                           codec_encode((long double)o0, f));                             \
                store_leaf(out->base, iomo_plane_slot(rows, width, yp, r, c + half), bits, \
                           codec_encode((long double)o1, f));                             \
            }                                                                             \
        }                                                                                 \
    } while (0)

int iomo_rope(int dtype, const iomo_view* x, const iomo_view* out, uint64_t a, double theta) {
    fmt_t f;
    if (!view_ok(x) || !view_ok(out) || !same_shape(x, out) || x->rank < 3) return IOMO_ERR_INVALID;
    const uint64_t rows = view_rows(x), width = view_cols(x), half = width / 2;
    if (width % 2 != 0) return IOMO_ERR_INVALID;
    if (a + (rows - 1) > (1ull << 24)) return IOMO_ERR_INVALID;   /* binary32-exact positions */
    if (out->base == x->base) return IOMO_ERR_INVALID;
    if (!isfinite(theta) || theta < 1.0 || theta > 3.4028234663852886e38) return IOMO_ERR_INVALID;
    if (!float_format(dtype, &f)) return IOMO_ERR_UNSUPPORTED;
    const unsigned bits = iomo_leaf_bits(dtype);
    const uint32_t leading = x->rank - 2;
    uint64_t coord[8] = {0};
    do {
        uint64_t xp = x->plane_offset, yp = out->plane_offset;
        for (uint32_t k = 0; k < leading; ++k) {
            xp += coord[k] * x->plane_strides[k];
            yp += coord[k] * out->plane_strides[k];
        }
        if (dtype == IOMO_DT_F64) ROPE_ROWS(double, pow, sin, cos);
        else ROPE_ROWS(float, powf, sinf, cosf);
    } while (next_coord(coord, x->dims, leading));
    return IOMO_OK;
}

/* ------------------------------------------------------------------ */
/* Linear projection (src/cpu/queue.cpp:1905-2051)                      */
/* ------------------------------------------------------------------ */

/* out[b,r,o] = sum_i x[b,s+r,i] * w[o,i] (ordinary, H = 1, D = O) or
 * out[b,h,r,d] = sum_i x[b,s+r,i] * w[h*D+d,i] (head planar, O = H*D): integers
 * modulo 2^N; floating leaves start at +0 and take one correctly rounded fused
 * multiply-add per increasing i in binary32 (binary64 for F64), encoded once.
 * Admission of docs/BACKEND_CONTRACT/linear-projections.md:86-112 as far as it can
 * be checked without owner identities. */
int iomo_linear(int dtype, const iomo_view* x, const iomo_view* w, const iomo_view* out,
                uint64_t s, uint64_t R, int head_planar, uint64_t H, uint64_t D) {
    const unsigned bits = iomo_leaf_bits(dtype);
    fmt_t f;
    if (!view_ok(x) || !view_ok(w) || !view_ok(out)) return IOMO_ERR_INVALID;
    if (w->rank != 2) return IOMO_ERR_INVALID;
    const uint64_t T = view_rows(x), I = view_cols(x), O = w->dims[0];
    if (w->dims[1] != I) return IOMO_ERR_INVALID;
    if (R == 0 || s > T || R > T - s) return IOMO_ERR_INVALID;
    if (head_planar) {
        if (H == 0 || D == 0 || H * D != O) return IOMO_ERR_INVALID;
        if (out->rank != x->rank + 1 || out->rank > 8) return IOMO_ERR_INVALID;
    } else {
        if (H != 1 || D != O) return IOMO_ERR_INVALID;
        if (out->rank != x->rank) return IOMO_ERR_INVALID;
    }
    const uint32_t leading = x->rank - 2;
    for (uint32_t i = 0; i < leading; ++i)
        if (x->dims[i] != out->dims[i]) return IOMO_ERR_INVALID;
    if (head_planar && out->dims[leading] != H) return IOMO_ERR_INVALID;
    if (view_rows(out) != R || view_cols(out) != D) return IOMO_ERR_INVALID;
    if (out->base == x->base || out->base == w->base) return IOMO_ERR_INVALID;
    const unsigned width = integer_width(dtype);
    if (!bits || (!width && !float_format(dtype, &f))) return IOMO_ERR_UNSUPPORTED;
    const uint64_t mask = width == 64 ? ~0ull : (1ull << width) - 1;
    const uint64_t heads = head_planar ? H : 1;
    const uint64_t head_stride = head_planar ? out->plane_strides[leading] : 0;
    uint64_t coord[8] = {0};
    do {
        uint64_t xp = x->plane_offset, op = out->plane_offset;
        for (uint32_t a = 0; a < leading; ++a) {
            xp += coord[a] * x->plane_strides[a];
            op += coord[a] * out->plane_strides[a];
        }
        for (uint64_t r = 0; r < R; ++r)
        for (uint64_t h = 0; h < heads; ++h)
        for (uint64_t d = 0; d < D; ++d) {
            const uint64_t o = h * D + d;
            uint64_t raw;
            if (width) {
                uint64_t acc = 0;
                for (uint64_t i = 0; i < I; ++i) {
                    const uint64_t a = load_leaf(x->base, iomo_plane_slot(T, I, xp, s + r, i), bits) & mask;
                    const uint64_t b = load_leaf(w->base, iomo_plane_slot(O, I, w->plane_offset, o, i), bits) & mask;
                    acc = (acc + a * b) & mask;
                }
                raw = acc;
            } else if (dtype == IOMO_DT_F64) {
                double acc = 0.0;
                for (uint64_t i = 0; i < I; ++i)
                    acc = fma((double)codec_decode(load_leaf(x->base, iomo_plane_slot(T, I, xp, s + r, i), bits), f),
                              (double)codec_decode(load_leaf(w->base, iomo_plane_slot(O, I, w->plane_offset, o, i), bits), f),
                              acc);
                raw = codec_encode(acc != acc ? positive_nan() : (long double)acc, f);
            } else {
                float acc = 0.0f;
                for (uint64_t i = 0; i < I; ++i)
                    acc = fmaf((float)codec_decode(load_leaf(x->base, iomo_plane_slot(T, I, xp, s + r, i), bits), f),
                               (float)codec_decode(load_leaf(w->base, iomo_plane_slot(O, I, w->plane_offset, o, i), bits), f),
                               acc);
                raw = codec_encode(acc != acc ? positive_nan() : (long double)acc, f);
            }
            store_leaf(out->base, iomo_plane_slot(R, D, op + h * head_stride, r, d), bits, raw);
        }
    } while (next_coord(coord, x->dims, leading));
    return IOMO_OK;
}

/* ------------------------------------------------------------------ */
/* Scaled dot-product attention (src/cpu/sdpa.cpp:132-336)              */
/* ------------------------------------------------------------------ */

/* The matrix-operand flush of src/cpu/sdpa.cpp:57-60: a nonzero magnitude below the
 * smallest normal becomes a zero of the same sign. */
static float matrix_daz(float v) {
    return (v != 0.0f && fabsf(v) < 0x1p-126f) ? copysignf(0.0f, v) : v;
}

static float bf16_value(const iomo_view* v, uint64_t rows, uint64_t cols, uint64_t plane,
                        uint64_t row, uint64_t col) {
    const uint32_t bits = (uint32_t)load_leaf(v->base, iomo_plane_slot(rows, cols, plane, row, col), 16);
    return f32_from_bits(bits << 16);
}

/* q [B..,Hq,R,D], k and v [B..,Hkv,C,D], out [B..,R,Hq*D]; BF16 only.  Per head and
 * row, over the visible tokens t < min(L, a+r+1): score = (sum_d q*k in binary32,
 * one product and one sum per increasing d) / sqrtf(D); the special rows and the
 * max-subtracted softmax of src/cpu/sdpa.cpp:214-309 with the probability rounded
 * once to BF16; out = sum_t P*V in binary32 per increasing t, -0 stored as +0, one
 * BF16 rounding (src/cpu/sdpa.cpp:317-336).  Admission follows
 * docs/BACKEND_CONTRACT/scaled-dot-product-attention.md:28-57 as far as it can be
 * checked without owner identities. */
int iomo_sdpa(int dtype, const iomo_view* q, const iomo_view* k, const iomo_view* v,
              const iomo_view* out, uint64_t a, uint64_t L) {
    if (!view_ok(q) || !view_ok(k) || !view_ok(v) || !view_ok(out)) return IOMO_ERR_INVALID;
    if (q->rank < 3 || k->rank != q->rank || v->rank != q->rank || out->rank != q->rank - 1)
        return IOMO_ERR_INVALID;
    const uint32_t leading = q->rank - 3;
    const uint64_t Hq = q->dims[leading], R = view_rows(q), D = view_cols(q);
    const uint64_t Hkv = k->dims[leading], C = view_rows(k);
    if (view_cols(k) != D || v->dims[leading] != Hkv || view_rows(v) != C || view_cols(v) != D)
        return IOMO_ERR_INVALID;
    if (Hq == 0 || Hkv == 0 || Hq % Hkv != 0) return IOMO_ERR_INVALID;
    if (view_rows(out) != R || view_cols(out) != Hq * D) return IOMO_ERR_INVALID;
    for (uint32_t i = 0; i < leading; ++i)
        if (k->dims[i] != q->dims[i] || v->dims[i] != q->dims[i] || out->dims[i] != q->dims[i])
            return IOMO_ERR_INVALID;
    if (L == 0 || L > C || a >= C || R > C - a) return IOMO_ERR_INVALID;
    if (out->base == q->base || out->base == k->base || out->base == v->base) return IOMO_ERR_INVALID;
    if (dtype != IOMO_DT_BF16) return IOMO_ERR_UNSUPPORTED;
    const uint64_t grouping = Hq / Hkv;
    const float scale = sqrtf((float)D);
    float* score = (float*)malloc((size_t)L * sizeof(float));
    uint16_t* prob = (uint16_t*)malloc((size_t)L * sizeof(uint16_t));
    if (!score || !prob) { free(score); free(prob); return IOMO_ERR_INVALID; }
    uint64_t coord[8] = {0};
    do {
        uint64_t qp = q->plane_offset, kp = k->plane_offset, vp = v->plane_offset, op = out->plane_offset;
        for (uint32_t i = 0; i < leading; ++i) {
            qp += coord[i] * q->plane_strides[i];
            kp += coord[i] * k->plane_strides[i];
            vp += coord[i] * v->plane_strides[i];
            op += coord[i] * out->plane_strides[i];
        }
        for (uint64_t head = 0; head < Hq; ++head) {
            const uint64_t qh = qp + head * q->plane_strides[leading];
            const uint64_t kh = kp + (head / grouping) * k->plane_strides[leading];
            const uint64_t vh = vp + (head / grouping) * v->plane_strides[leading];
            for (uint64_t row = 0; row < R; ++row) {
                const uint64_t visible = L < a + row + 1 ? L : a + row + 1;
                int has_nan = 0, all_ninf = 1;
                uint64_t pinf = 0;
                for (uint64_t t = 0; t < visible; ++t) {
                    float dot = 0.0f;
                    for (uint64_t d = 0; d < D; ++d) {
                        const volatile float product = matrix_daz(bf16_value(q, R, D, qh, row, d))
                                * matrix_daz(bf16_value(k, C, D, kh, t, d));
                        const volatile float next = dot + product;
                        dot = next;
                    }
                    const volatile float scaled = dot / scale;
                    score[t] = scaled;
                    has_nan = has_nan || isnan(scaled);
                    pinf += (scaled == INFINITY) ? 1 : 0;
                    all_ninf = all_ninf && isinf(scaled) && signbit(scaled);
                }
                if (has_nan || all_ninf) {
                    for (uint64_t f = 0; f < D; ++f)
                        store_leaf(out->base, iomo_plane_slot(R, Hq * D, op, row, head * D + f), 16, 0x7FC0u);
                    continue;
                }
                if (pinf != 0) {
                    const volatile float p = 1.0f / (float)pinf;
                    for (uint64_t t = 0; t < visible; ++t)
                        prob[t] = iomo_encode_bf16(score[t] == INFINITY ? p : 0.0f);
                } else {
                    float maximum = -INFINITY;
                    for (uint64_t t = 0; t < visible; ++t)
                        if (score[t] > maximum) maximum = score[t];
                    float sum = 0.0f;
                    for (uint64_t t = 0; t < visible; ++t) {
                        if (isinf(score[t]) && signbit(score[t])) { score[t] = 0.0f; continue; }
                        const volatile float shifted = score[t] - maximum;
                        const volatile float e = expf(shifted);
                        const volatile float next = sum + e;
                        sum = next;
                        score[t] = e;
                    }
                    for (uint64_t t = 0; t < visible; ++t) {
                        const volatile float normalized = score[t] / sum;
                        prob[t] = iomo_encode_bf16(normalized);
                    }
                }
                for (uint64_t f = 0; f < D; ++f) {
                    float result = 0.0f;
                    for (uint64_t t = 0; t < visible; ++t) {
                        const volatile float product = matrix_daz(f32_from_bits((uint32_t)prob[t] << 16))
                                * matrix_daz(bf16_value(v, C, D, vh, t, f));
                        const volatile float next = result + product;
                        result = next;
                    }
                    if (result == 0.0f) result = 0.0f;   /* -0 is stored as +0 */
                    store_leaf(out->base, iomo_plane_slot(R, Hq * D, op, row, head * D + f), 16,
                               iomo_encode_bf16(result));
                }
            }
        }
    } while (next_coord(coord, q->dims, leading));
    free(score);
    free(prob);
    return IOMO_OK;
}

/* ------------------------------------------------------------------ */
/* Softmax stage (src/cpu/sdpa.cpp:214-309)                             */
/* ------------------------------------------------------------------ */

static uint64_t stage_offset(const iomo_stage_layout* l, uint64_t plane,
                             uint64_t head, uint64_t row, uint64_t col) {
    return l->plane_offset + plane * l->plane_stride + head * l->head_stride
            + row * l->row_stride + col * l->column_stride;
}

int iomo_softmax(const iomo_softmax_desc* d) {
    if (!d || !d->scores || !d->p_bf16) return IOMO_ERR_INVALID;
    if (d->L == 0 || d->rows == 0 || d->heads == 0 || d->planes == 0) return IOMO_ERR_INVALID;
    const iomo_stage_layout* sl = &d->scores_layout;
    const iomo_stage_layout* pl = &d->probability_layout;
    if (pl->rows < d->rows || pl->columns < d->L) return IOMO_ERR_INVALID;
    for (uint64_t plane = 0; plane < d->planes; ++plane)
    for (uint64_t head = 0; head < d->heads; ++head)
    for (uint64_t row = 0; row < pl->rows; ++row) {
        uint16_t* prow = d->p_bf16;
        if (row >= d->rows) {
            /* physical rows past the logical extent are canonical +0
             * (src/rocm/sdpa_softmax.hpp:24-27) */
            for (uint64_t t = 0; t < pl->columns; ++t)
                prow[stage_offset(pl, plane, head, row, t)] = 0;
            continue;
        }
        const uint64_t reach = d->a + row + 1;
        const uint64_t visible = reach < d->L ? reach : d->L;
        int has_nan = 0, all_ninf = 1;
        uint64_t pinf = 0;
        for (uint64_t t = 0; t < visible; ++t) {
            const volatile float s =
                    d->scores[stage_offset(sl, plane, head, row, t)] * d->scale;
            has_nan = has_nan || isnan(s);
            pinf += (s == INFINITY) ? 1 : 0;
            all_ninf = all_ninf && isinf(s) && signbit(s);
        }
        if (has_nan || all_ninf) {
            for (uint64_t t = 0; t < pl->columns; ++t)
                prow[stage_offset(pl, plane, head, row, t)] =
                        t < visible ? 0x7FC0u : 0;
            continue;
        }
        if (pinf != 0) {
            const volatile float p = 1.0f / (float)pinf;
            for (uint64_t t = 0; t < pl->columns; ++t) {
                uint16_t e = 0;
                if (t < visible) {
                    const volatile float s =
                            d->scores[stage_offset(sl, plane, head, row, t)] * d->scale;
                    e = iomo_encode_bf16(s == INFINITY ? p : 0.0f);
                }
                prow[stage_offset(pl, plane, head, row, t)] = e;
            }
            continue;
        }
        float maximum = -INFINITY;
        for (uint64_t t = 0; t < visible; ++t) {
            const volatile float s =
                    d->scores[stage_offset(sl, plane, head, row, t)] * d->scale;
            if (s > maximum) maximum = s;
        }
        volatile float sum = 0.0f;
        for (uint64_t t = 0; t < visible; ++t) {
            const volatile float s =
                    d->scores[stage_offset(sl, plane, head, row, t)] * d->scale;
            if (isinf(s) && signbit(s)) continue;
            const volatile float shifted = s - maximum;
            const volatile float e = expf(shifted);
            sum = sum + e;
        }
        for (uint64_t t = 0; t < pl->columns; ++t) {
            uint16_t enc = 0;
            if (t < visible) {
                const volatile float s =
                        d->scores[stage_offset(sl, plane, head, row, t)] * d->scale;
                if (!(isinf(s) && signbit(s))) {
                    const volatile float shifted = s - maximum;
                    const volatile float e = expf(shifted);
                    const volatile float p = e / sum;
                    enc = iomo_encode_bf16(p);
                }
            }
            prow[stage_offset(pl, plane, head, row, t)] = enc;
        }
    }
    return IOMO_OK;
}
