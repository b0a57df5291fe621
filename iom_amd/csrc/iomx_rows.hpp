// Tile-row helpers shared by the every-leaf kernels: leaf tables, a tile row of
// sixteen packed elements as an array of 32-bit words, the little-endian bit
// stream of the host format, and the per-element arithmetic of every leaf.
#pragma once

#include "iomx_common.hpp"

namespace iomx {

enum {
    DT_BOOL = 0, DT_I2 = 1, DT_U2 = 2, DT_I4 = 3, DT_U4 = 4, DT_I8 = 5, DT_U8 = 6, DT_I16 = 7,
    DT_U16 = 8, DT_I32 = 9, DT_U32 = 10, DT_I64 = 11, DT_U64 = 12, DT_F4_E2M1 = 13,
    DT_F6_E2M3 = 14, DT_F6_E3M2 = 15, DT_F8_E4M3FN = 16, DT_F8_E5M2 = 17, DT_F8_E8M0 = 18,
    DT_F16 = 19, DT_BF16 = 20, DT_F32 = 21, DT_F64 = 22
};

constexpr int bits_of(int dt) {
    switch (dt) {
        case DT_I2: case DT_U2: return 2;
        case DT_I4: case DT_U4: case DT_F4_E2M1: return 4;
        case DT_F6_E2M3: case DT_F6_E3M2: return 6;
        case DT_BOOL: case DT_I8: case DT_U8: case DT_F8_E4M3FN: case DT_F8_E5M2:
        case DT_F8_E8M0: return 8;
        case DT_I16: case DT_U16: case DT_F16: case DT_BF16: return 16;
        case DT_I32: case DT_U32: case DT_F32: return 32;
        case DT_I64: case DT_U64: case DT_F64: return 64;
        default: return 0;
    }
}

constexpr bool is_float_leaf(int dt) { return dt >= DT_F4_E2M1 && dt != DT_F8_E8M0; }

struct Fmt {
    int ebits, fbits, bias;
    bool finite_only, infs;
};

constexpr Fmt fmt_of(int dt) {
    switch (dt) {
        case DT_F4_E2M1: return {2, 1, 1, true, false};
        case DT_F6_E2M3: return {2, 3, 1, true, false};
        case DT_F6_E3M2: return {3, 2, 3, true, false};
        case DT_F8_E4M3FN: return {4, 3, 7, true, false};
        case DT_F8_E5M2: return {5, 2, 15, false, true};
        case DT_F16: return {5, 10, 15, false, true};
        case DT_BF16: return {8, 7, 127, false, true};
        case DT_F32: return {8, 23, 127, false, true};
        default: return {11, 52, 1023, false, true};
    }
}

// The top exponent encodes infinity / NaN unless the leaf is finite-only with
// fewer than four exponent bits.
constexpr bool top_special(Fmt f) { return !f.finite_only || f.ebits >= 4; }

// The packing helpers and the element arithmetic are plain C++ (usable from host
// code as well), so they can be exercised without a device.
#define IOMX_HD __host__ __device__ __forceinline__

// ---------------------------------------------------------------------------
// Tile rows as word arrays
// ---------------------------------------------------------------------------

// STREAM: read past the caches (an operand that no other lane reads again).
template <int BITS, bool STREAM = false>
IOMX_HD void load_row(const uint8_t* p, uint32_t (&w)[BITS / 2]) {
    constexpr int K = BITS / 2;
    if constexpr (K == 1) {
        w[0] = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p))
                      : *reinterpret_cast<const uint32_t*>(p);
    } else if constexpr (K == 2) {
        const u32x2 v = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p))
                               : *reinterpret_cast<const u32x2*>(p);
        w[0] = v.x;
        w[1] = v.y;
    } else if constexpr (K == 3) {
#pragma unroll
        for (int j = 0; j < 3; ++j)
            w[j] = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p) + j)
                          : reinterpret_cast<const uint32_t*>(p)[j];
    } else {
#pragma unroll
        for (int j = 0; j < K / 4; ++j) {
            const u32x4 v = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p) + j)
                                   : reinterpret_cast<const u32x4*>(p)[j];
            w[4 * j] = v.x;
            w[4 * j + 1] = v.y;
            w[4 * j + 2] = v.z;
            w[4 * j + 3] = v.w;
        }
    }
}

// Element i of a tile row (i is a compile-time constant after unrolling).
template <int BITS>
IOMX_HD uint64_t get(const uint32_t (&w)[BITS / 2], int i) {
    if constexpr (BITS == 64) {
        return (uint64_t)w[2 * i] | ((uint64_t)w[2 * i + 1] << 32);
    } else if constexpr (32 % BITS == 0) {
        constexpr int per = 32 / BITS;
        const uint32_t v = w[i / per] >> ((i % per) * BITS);
        return BITS == 32 ? v : (v & ((1u << (BITS & 31)) - 1u));
    } else {
        const int bit = i * BITS, j = bit >> 5, sh = bit & 31;
        uint64_t v = w[j];
        if (sh + BITS > 32) v |= (uint64_t)w[j + 1] << 32;
        return (v >> sh) & ((1u << BITS) - 1u);
    }
}

// ORs element i into a zero-initialised tile row.
template <int BITS>
IOMX_HD void put(uint32_t (&w)[BITS / 2], int i, uint64_t v) {
    if constexpr (BITS == 64) {
        w[2 * i] = (uint32_t)v;
        w[2 * i + 1] = (uint32_t)(v >> 32);
    } else if constexpr (32 % BITS == 0) {
        constexpr int per = 32 / BITS;
        w[i / per] |= (uint32_t)v << ((i % per) * BITS);
    } else {
        const int bit = i * BITS, j = bit >> 5, sh = bit & 31;
        w[j] |= (uint32_t)v << sh;
        if (sh + BITS > 32) w[j + 1] |= (uint32_t)v >> (32 - sh);
    }
}

// Stores the first ncols elements of a tile row and nothing else: whole words
// where they are covered, a read-modify-write of the one partly covered word.
template <int BITS, bool STREAM = false>
IOMX_HD void store_row(uint8_t* p, const uint32_t (&w)[BITS / 2], uint32_t ncols) {
    constexpr int K = BITS / 2;
    if (ncols == kTile) {
        if constexpr (K == 1) {
            if constexpr (STREAM) __builtin_nontemporal_store(w[0], reinterpret_cast<uint32_t*>(p));
            else *reinterpret_cast<uint32_t*>(p) = w[0];
        } else if constexpr (K == 2) {
            if constexpr (STREAM) __builtin_nontemporal_store(u32x2{w[0], w[1]}, reinterpret_cast<u32x2*>(p));
            else *reinterpret_cast<u32x2*>(p) = u32x2{w[0], w[1]};
        } else if constexpr (K == 3) {
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                if constexpr (STREAM) __builtin_nontemporal_store(w[j], reinterpret_cast<uint32_t*>(p) + j);
                else reinterpret_cast<uint32_t*>(p)[j] = w[j];
            }
        } else {
#pragma unroll
            for (int j = 0; j < K / 4; ++j) {
                const u32x4 v = u32x4{w[4 * j], w[4 * j + 1], w[4 * j + 2], w[4 * j + 3]};
                if constexpr (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p) + j);
                else reinterpret_cast<u32x4*>(p)[j] = v;
            }
        }
        return;
    }
    const uint32_t nbits = ncols * BITS;
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const uint32_t lo = j * 32u;
        if (lo >= nbits) break;
        uint32_t* dst = reinterpret_cast<uint32_t*>(p) + j;
        if (lo + 32u <= nbits) {
            *dst = w[j];
        } else {
            const uint32_t mask = (1u << (nbits - lo)) - 1u;
            *dst = (*dst & ~mask) | (w[j] & mask);
        }
    }
}

// BITS bits of a little-endian bit stream held in 32-bit words.
template <int BITS>
IOMX_HD uint64_t read_bits(const uint32_t* words, uint64_t bit) {
    if constexpr (BITS == 64) {
        return read_bits<32>(words, bit) | (read_bits<32>(words, bit + 32) << 32);
    } else {
        const uint64_t j = bit >> 5;
        const uint32_t sh = (uint32_t)bit & 31u;
        uint32_t v = words[j] >> sh;
        if (sh + BITS > 32) v |= words[j + 1] << (32u - sh);
        return BITS == 32 ? v : (v & ((1u << (BITS & 31)) - 1u));
    }
}

// ---------------------------------------------------------------------------
// Element arithmetic
// ---------------------------------------------------------------------------

IOMX_HD double as_f64(uint64_t b) { return __builtin_bit_cast(double, b); }
IOMX_HD uint64_t as_u64(double d) { return __builtin_bit_cast(uint64_t, d); }

constexpr uint64_t kQuietNanF64 = 0x7FF8000000000000ull;

template <int DT>
IOMX_HD double decode(uint64_t raw64) {
    if constexpr (DT == DT_F64) {
        return as_f64(raw64);
    } else {
        constexpr Fmt f = fmt_of(DT);
        constexpr uint32_t emask = (1u << f.ebits) - 1u, fmask = (1u << f.fbits) - 1u;
        const uint32_t raw = (uint32_t)raw64;
        const uint32_t frac = raw & fmask, exp = (raw >> f.fbits) & emask;
        double v;
        if (top_special(f) && exp == emask) {
            v = (f.infs && frac == 0) ? __builtin_inf() : __builtin_nan("");
        } else {
            const int m = exp ? (int)((1u << f.fbits) + frac) : (int)frac;
            const int scale = (int)(exp ? exp : 1u) - f.bias - f.fbits;
            v = ldexp((double)m, scale);
        }
        return ((raw >> (f.ebits + f.fbits)) & 1u) ? -v : v;
    }
}

// One rounding of a binary64 value (zero, normal, infinite or NaN) onto the leaf.
template <int DT>
IOMX_HD uint64_t encode(double r) {
    if constexpr (DT == DT_F64) {
        return (r != r) ? kQuietNanF64 : as_u64(r);
    } else {
        constexpr Fmt f = fmt_of(DT);
        constexpr uint32_t emask = (1u << f.ebits) - 1u, fmask = (1u << f.fbits) - 1u;
        constexpr int shift = f.ebits + f.fbits;
        constexpr uint32_t finite_emax = top_special(f) ? emask - 1u : emask;
        constexpr uint32_t over = f.infs ? (emask << f.fbits) : ((finite_emax << f.fbits) | fmask);
        constexpr uint32_t nan = !top_special(f) ? over
                : (emask << f.fbits) | (f.finite_only ? fmask : 1u << (f.fbits - 1));
        const uint64_t b = as_u64(r);
        const uint32_t sign = (uint32_t)(b >> 63) << shift;
        const uint64_t mag = b & 0x7FFFFFFFFFFFFFFFull;
        if (mag > 0x7FF0000000000000ull) return nan;
        if (mag == 0x7FF0000000000000ull) return sign | over;
        if (mag == 0) return sign;
        const int e = (int)(mag >> 52) - 1023;
        const uint64_t m = (mag & 0xFFFFFFFFFFFFFull) | (1ull << 52);
        constexpr int emin = 1 - f.bias;
        const int drop = 52 - f.fbits + (e < emin ? emin - e : 0);
        uint64_t q = 0, rest = 1, half = 2;  // far below half a unit unless set below
        if (drop <= 62) {
            q = m >> drop;
            rest = m & ((1ull << drop) - 1ull);
            half = 1ull << (drop - 1);
        }
        if (rest > half || (rest == half && (q & 1ull))) ++q;
        // a normal q carries the implicit bit, which adds one to the exponent field; a
        // subnormal q that reaches 2^fbits becomes the smallest normal the same way
        const uint32_t field = e < emin ? (uint32_t)q
                                        : ((uint32_t)(e + f.bias - 1) << f.fbits) + (uint32_t)q;
        if ((field >> f.fbits) > finite_emax) return sign | over;
        return sign | field;
    }
}

// The same two steps in binary32, for the leaves of at most 8 bits.  Their values are
// exact in binary32; a product of two is exact (at most 8 significand bits), and a
// sum or difference is exact or rounded with so many guard bits (24 >= 2*4 + 2)
// that the rounding below still equals one rounding of the exact result.  The
// binary32 path equals the binary64 one for every operand pair (checked
// exhaustively on the host and on the device).
IOMX_HD float as_f32_hd(uint32_t b) { return __builtin_bit_cast(float, b); }
IOMX_HD uint32_t as_u32_hd(float f) { return __builtin_bit_cast(uint32_t, f); }

template <int DT>
IOMX_HD float decode_f32(uint32_t raw) {
    constexpr Fmt f = fmt_of(DT);
    constexpr uint32_t emask = (1u << f.ebits) - 1u, fmask = (1u << f.fbits) - 1u;
    const uint32_t frac = raw & fmask, exp = (raw >> f.fbits) & emask;
    const uint32_t sign = ((raw >> (f.ebits + f.fbits)) & 1u) << 31;
    if (top_special(f) && exp == emask)
        return as_f32_hd(sign | ((f.infs && frac == 0) ? 0x7F800000u : 0x7FC00000u));
    // a normal value re-biased into binary32 (every leaf exponent is inside its range), a
    // subnormal one as its integer fraction times the leaf's smallest step: both exact
    constexpr float kStep = 1.0f / (float)(1u << (f.bias - 1 + f.fbits));       // 2^(1 - bias - fbits)
    const uint32_t normal = ((exp + 127u - (uint32_t)f.bias) << 23) | (frac << (23 - f.fbits));
    const float magnitude = exp ? as_f32_hd(normal) : (float)frac * kStep;
    return as_f32_hd(as_u32_hd(magnitude) | sign);
}

template <int DT>
IOMX_HD uint32_t encode_f32(float r) {
    constexpr Fmt f = fmt_of(DT);
    constexpr uint32_t emask = (1u << f.ebits) - 1u, fmask = (1u << f.fbits) - 1u;
    constexpr int shift = f.ebits + f.fbits;
    constexpr uint32_t finite_emax = top_special(f) ? emask - 1u : emask;
    constexpr uint32_t over = f.infs ? (emask << f.fbits) : ((finite_emax << f.fbits) | fmask);
    constexpr uint32_t nan = !top_special(f) ? over
            : (emask << f.fbits) | (f.finite_only ? fmask : 1u << (f.fbits - 1));
    const uint32_t b = as_u32_hd(r);
    const uint32_t sign = (b >> 31) << shift;
    const uint32_t mag = b & 0x7FFFFFFFu;
    if (mag > 0x7F800000u) return nan;
    if (mag == 0x7F800000u) return sign | over;
    if (mag < 0x00800000u) return sign;   // zero, or below 2^-126: far under half the smallest step
    const int e = (int)(mag >> 23) - 127;
    const uint32_t m = (mag & 0x7FFFFFu) | 0x800000u;
    constexpr int emin = 1 - f.bias;
    const int drop = 23 - f.fbits + (e < emin ? emin - e : 0);
    uint32_t q = 0, rest = 1, half = 2;
    if (drop <= 30) {
        q = m >> drop;
        rest = m & ((1u << drop) - 1u);
        half = 1u << (drop - 1);
    }
    if (rest > half || (rest == half && (q & 1u))) ++q;
    const uint32_t field = e < emin ? q : ((uint32_t)(e + f.bias - 1) << f.fbits) + q;
    if ((field >> f.fbits) > finite_emax) return sign | over;
    return sign | field;
}

template <int OP, typename T>
IOMX_HD T leaf_arith(T x, T y) {
    if constexpr (OP == IOMX_OP_ADD) return x + y;
    else if constexpr (OP == IOMX_OP_MUL) return x * y;
    else if constexpr (OP == IOMX_OP_SUB) return x - y;
    else return x / y;
}

template <int DT, int OP>
IOMX_HD uint64_t leaf_binary(uint64_t a, uint64_t b) {
    constexpr int BITS = bits_of(DT);
    if constexpr (!is_float_leaf(DT)) {
        if constexpr (BITS == 64) {
            return OP == IOMX_OP_ADD ? a + b : (OP == IOMX_OP_MUL ? a * b : a - b);
        } else {
            const uint32_t x = (uint32_t)a, y = (uint32_t)b;
            const uint32_t r = OP == IOMX_OP_ADD ? x + y : (OP == IOMX_OP_MUL ? x * y : x - y);
            return BITS == 32 ? r : (r & ((1u << (BITS & 31)) - 1u));
        }
    } else {
        // IEEE arithmetic supplies the special cases of the reference rule: opposite
        // infinities, infinity times zero, 0/0 and inf/inf give NaN, an exact zero sum
        // is +0 unless both operands are -0, NaN operands give NaN.  A quotient is not
        // exact in the carrier, but it is correctly rounded to at least 2p + 2 bits for
        // a leaf of p significand bits (24 for p <= 11, 53 for F32), so the encode's
        // rounding still equals one rounding of the exact quotient.
        if constexpr (BITS <= 8) {
            const float x = decode_f32<DT>((uint32_t)a), y = decode_f32<DT>((uint32_t)b);
            return encode_f32<DT>(leaf_arith<OP>(x, y));
        }
        const double x = decode<DT>(a), y = decode<DT>(b);
        return encode<DT>(leaf_arith<OP>(x, y));
    }
}

// A whole word of 2- or 4-bit integers at once (sixteen or eight lanes; the wrap of
// two's complement does not see the sign).  Sum and difference keep carries and
// borrows inside a lane by handling each lane's top bit apart; the 2-bit product is
// two bits of boolean algebra; the 4-bit products are formed two at a time, on nibbles
// j and j + 4 moved to the bottom of the two 16-bit halves of a word.
template <int BITS>
IOMX_HD uint32_t splat_lane(uint32_t w) {
    return BITS == 2 ? (w & 3u) * 0x55555555u : (w & 15u) * 0x11111111u;
}

template <int BITS, int OP>
IOMX_HD uint32_t swar_word(uint32_t a, uint32_t b) {
    static_assert(BITS == 2 || BITS == 4, "sub-byte integer lanes");
    constexpr uint32_t H = BITS == 2 ? 0xAAAAAAAAu : 0x88888888u, L = ~H;
    if constexpr (OP == IOMX_OP_ADD) {
        return ((a & L) + (b & L)) ^ ((a ^ b) & H);
    } else if constexpr (OP == IOMX_OP_SUB) {
        return ((a | H) - (b & L)) ^ ((a ^ ~b) & H);
    } else if constexpr (BITS == 2) {
        // (2*a1 + a0)(2*b1 + b0) mod 4 = 2*(a1 b0 xor a0 b1) + a0 b0
        const uint32_t low = a & b & 0x55555555u;
        const uint32_t high = (((a >> 1) & b) ^ (a & (b >> 1))) & 0x55555555u;
        return low | (high << 1);
    } else {
        uint32_t r = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t x = (a >> (4 * j)) & 0x000F000Fu, y = (b >> (4 * j)) & 0x000F000Fu;
            const uint32_t p = ((x & 0xFFFFu) * (y & 0xFFFFu)) | (((x >> 16) * (y >> 16)) << 16);
            r |= (p & 0x000F000Fu) << (4 * j);
        }
        return r;
    }
}

// x * sigmoid(x), two-branch form of src/shared/scalar_silu.hpp:69-97; one
// exponential of a non-positive argument serves both branches.
IOMX_HD float silu_carrier(float x) {
    const bool pos = x >= 0.0f;
    const float e = expf(pos ? -x : x * 0.5f);
    const float xe = x * e;
    float num = pos ? x : xe * e;
    const float den = 1.0f + (pos ? e : e * e);
    if (!pos && e == 0.0f) num = -0.0f;
    return num / den;
}
IOMX_HD double silu_carrier(double x) {
    const bool pos = x >= 0.0;
    const double e = exp(pos ? -x : x * 0.5);
    const double xe = x * e;
    double num = pos ? x : xe * e;
    const double den = 1.0 + (pos ? e : e * e);
    if (!pos && e == 0.0) num = -0.0;
    return num / den;
}

// Carrier: binary32 below F64, binary64 for F64 (src/cpu/queue.cpp:1769-1773).
template <int DT>
IOMX_HD uint64_t leaf_silu(uint64_t a) {
    if constexpr (DT == DT_F64) return encode<DT>(silu_carrier(decode<DT>(a)));
    else if constexpr (bits_of(DT) <= 8) return encode_f32<DT>(silu_carrier(decode_f32<DT>((uint32_t)a)));
    else return encode<DT>((double)silu_carrier((float)decode<DT>(a)));
}

// A leaf value in the carrier T (float or double) and back, by the cheaper route.
template <int DT, typename T>
IOMX_HD T decode_as(uint64_t raw) {
    if constexpr (bits_of(DT) <= 8) return (T)decode_f32<DT>((uint32_t)raw);
    else return (T)decode<DT>(raw);
}
template <int DT, typename T>
IOMX_HD uint64_t encode_from(T v) {
    if constexpr (bits_of(DT) <= 8) return encode_f32<DT>((float)v);
    else return encode<DT>((double)v);
}

#if defined(__HIPCC__)

// The conversion instructions of the two 8-bit floating leaves.  They agree with the
// leaf's own rule on every value up to the largest finite one (the same grid, the same
// round-to-nearest-even, subnormals included).  Outside that they do not: the top
// exponent of F8_E4M3FN holds values up to 448 for the hardware and is all NaN for the
// leaf (src/shared/scalar_binary_codec.hpp:51,73), and what an overflow or a NaN
// becomes is the leaf's choice.  So a caller converts by hardware only what
// hw_f8_limit bounds and sends every other element through decode_f32 / encode_f32.
constexpr bool has_hw_f8(int dt) { return dt == DT_F8_E4M3FN || dt == DT_F8_E5M2; }

template <int DT>
constexpr float hw_f8_limit() { return DT == DT_F8_E4M3FN ? 240.0f : 57344.0f; }

// Element `byte` (a constant after unrolling) of a word of four.
template <int DT>
__device__ __forceinline__ float hw_f8_value(uint32_t word, int byte) {
    if constexpr (DT == DT_F8_E4M3FN) {
        switch (byte) {
            case 0: return __builtin_amdgcn_cvt_f32_fp8(word, 0);
            case 1: return __builtin_amdgcn_cvt_f32_fp8(word, 1);
            case 2: return __builtin_amdgcn_cvt_f32_fp8(word, 2);
            default: return __builtin_amdgcn_cvt_f32_fp8(word, 3);
        }
    } else {
        switch (byte) {
            case 0: return __builtin_amdgcn_cvt_f32_bf8(word, 0);
            case 1: return __builtin_amdgcn_cvt_f32_bf8(word, 1);
            case 2: return __builtin_amdgcn_cvt_f32_bf8(word, 2);
            default: return __builtin_amdgcn_cvt_f32_bf8(word, 3);
        }
    }
}

// Two rounded values into the lower or upper half of a word, the other half kept.
template <int DT>
__device__ __forceinline__ uint32_t hw_f8_pack(float first, float second, uint32_t word, bool upper) {
    if constexpr (DT == DT_F8_E4M3FN) {
        return upper ? __builtin_amdgcn_cvt_pk_fp8_f32(first, second, word, true)
                     : __builtin_amdgcn_cvt_pk_fp8_f32(first, second, word, false);
    } else {
        return upper ? __builtin_amdgcn_cvt_pk_bf8_f32(first, second, word, true)
                     : __builtin_amdgcn_cvt_pk_bf8_f32(first, second, word, false);
    }
}

// True if one of the four bytes has all four exponent bits of F8_E4M3FN set.
__device__ __forceinline__ bool e4m3_top_exponent(uint32_t word) {
    return (((word & 0x78787878u) + 0x08080808u) & 0x80808080u) != 0;
}

// The scaled conversions of the 4- and 6-bit floating leaves, at scale 1: their decode
// is exact, and their encode is the leaf's own rule for every binary32 input (the same
// round-to-nearest-even, subnormals included, saturation at the largest finite magnitude,
// infinities too) except that a NaN keeps its sign where the leaf stores the positive
// largest magnitude (src/shared/scalar_binary_codec.hpp:80) - the caller replaces a NaN
// by that value first.  Checked against decode_f32 / encode_f32 on the device for all
// encodings and a dense sweep of binary32 values.
constexpr bool has_hw_f46(int dt) { return dt == DT_F4_E2M1 || dt == DT_F6_E2M3 || dt == DT_F6_E3M2; }

template <int DT>
constexpr float hw_f46_largest() { return DT == DT_F4_E2M1 ? 6.0f : DT == DT_F6_E2M3 ? 7.5f : 28.0f; }

typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x32_t __attribute__((ext_vector_type(32)));
typedef uint32_t u32x6_t __attribute__((ext_vector_type(6)));

// Sixteen values of one tile row (two words of F4, three of F6).
template <int DT>
__device__ __forceinline__ void hw_f46_decode(const uint32_t (&w)[bits_of(DT) / 2], float (&v)[kTile]) {
    if constexpr (DT == DT_F4_E2M1) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const f32x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 0);
            const f32x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 1);
            const f32x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 2);
            const f32x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 3);
            v[8 * j] = p0.x; v[8 * j + 1] = p0.y; v[8 * j + 2] = p1.x; v[8 * j + 3] = p1.y;
            v[8 * j + 4] = p2.x; v[8 * j + 5] = p2.y; v[8 * j + 6] = p3.x; v[8 * j + 7] = p3.y;
        }
    } else {
        // the instruction converts thirty-two: the upper sixteen are zeros here
        const u32x6_t s = {w[0], w[1], w[2], 0u, 0u, 0u};
        f32x32_t d;
        if constexpr (DT == DT_F6_E2M3) d = __builtin_amdgcn_cvt_scalef32_pk32_f32_fp6(s, 1.0f);
        else d = __builtin_amdgcn_cvt_scalef32_pk32_f32_bf6(s, 1.0f);
#pragma unroll
        for (int i = 0; i < (int)kTile; ++i) v[i] = d[i];
    }
}

template <int DT>
__device__ __forceinline__ void hw_f46_encode(const float (&r)[kTile], uint32_t (&w)[bits_of(DT) / 2]) {
    if constexpr (DT == DT_F4_E2M1) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            uint32_t x = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, r[8 * j], r[8 * j + 1], 1.0f, 0);
            x = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(x, r[8 * j + 2], r[8 * j + 3], 1.0f, 1);
            x = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(x, r[8 * j + 4], r[8 * j + 5], 1.0f, 2);
            w[j] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(x, r[8 * j + 6], r[8 * j + 7], 1.0f, 3);
        }
    } else {
        // result 2i comes from the first operand's element i, result 2i + 1 from the second's
        f32x16_t even, odd;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            even[i] = i < 8 ? r[2 * i] : 0.0f;
            odd[i] = i < 8 ? r[2 * i + 1] : 0.0f;
        }
        u32x6_t e;
        if constexpr (DT == DT_F6_E2M3) e = __builtin_amdgcn_cvt_scalef32_2xpk16_fp6_f32(even, odd, 1.0f);
        else e = __builtin_amdgcn_cvt_scalef32_2xpk16_bf6_f32(even, odd, 1.0f);
        w[0] = e[0]; w[1] = e[1]; w[2] = e[2];
    }
}

// A tile row of one of the five leaves above, decoded and rounded by the conversion
// instructions wherever they agree with the leaf's rule, by decode_f32 / encode_f32
// elsewhere: exact for every encoding, the leaf's rounding for every binary32 value.
constexpr bool has_hw_convert(int dt) { return has_hw_f8(dt) || has_hw_f46(dt); }

template <int DT>
__device__ __forceinline__ void hw_decode_row(const uint32_t (&w)[bits_of(DT) / 2], float (&v)[kTile]) {
    if constexpr (has_hw_f46(DT)) {
        hw_f46_decode<DT>(w, v);
    } else {
        // The top exponent of F8_E4M3FN is all NaN for the leaf and holds numbers for the
        // instruction: in a row that has such a byte every element is still converted by the
        // instruction, and the bytes in question are replaced by the leaf's NaN (with the
        // byte's sign, as decode_f32 gives it).
        bool special = false;
        if constexpr (DT == DT_F8_E4M3FN)
            special = e4m3_top_exponent(w[0]) | e4m3_top_exponent(w[1]) | e4m3_top_exponent(w[2]) | e4m3_top_exponent(w[3]);
        // (decided for the wave as a whole: lanes that took different sides would make the wave
        // walk both, and the replacement below is harmless for a row that needs none)
        if (__any(special)) {
            // a byte with the top exponent gets all three fraction bits set, four bytes at a time:
            // that is the one encoding of the top exponent the instruction reads as NaN as well
            // (the empty statement keeps this side a branch: folded into selects it would run, and
            // cost its instructions, in every row)
            asm volatile("");
            uint32_t fixed[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t top = (((w[j] & 0x78787878u) + 0x08080808u) & 0x80808080u) >> 7;   // 1 per such byte
                fixed[j] = w[j] | (top * 7u);
            }
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i) v[i] = hw_f8_value<DT>(fixed[i >> 2], i & 3);
        } else {
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i) v[i] = hw_f8_value<DT>(w[i >> 2], i & 3);
        }
    }
}

// NANS = false: the caller knows that no value is a NaN (sums, differences and products of the
// finite 4- and 6-bit values), which spares those leaves the replacement of a NaN.
template <int DT, bool NANS = true>
__device__ __forceinline__ void hw_encode_row(const float (&r)[kTile], uint32_t (&w)[bits_of(DT) / 2]) {
    if constexpr (has_hw_f46(DT)) {
        if constexpr (NANS) {
            float s[kTile];
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i) s[i] = (r[i] != r[i]) ? hw_f46_largest<DT>() : r[i];
            hw_f46_encode<DT>(s, w);
        } else {
            hw_f46_encode<DT>(r, w);
        }
    } else {
        // the instructions when all sixteen are numbers within the finite range (false for a NaN)
        bool plain = true;
#pragma unroll
        for (int i = 0; i < (int)kTile; ++i) plain &= __builtin_fabsf(r[i]) <= hw_f8_limit<DT>();
        if (__all(plain)) {       // for the wave as a whole, as in hw_decode_row
#pragma unroll
            for (int j = 0; j < 4; ++j)
                w[j] = hw_f8_pack<DT>(r[4 * j + 2], r[4 * j + 3], hw_f8_pack<DT>(r[4 * j], r[4 * j + 1], 0u, false), true);
        } else {
            // Some element is a NaN, an infinity or beyond the largest finite value.
            asm volatile("");     // stays a branch, as in hw_decode_row
            if constexpr (DT == DT_F8_E4M3FN) {
                // Every number, infinities included, clamped to the largest finite magnitude first
                // (240: what lies above rounds or saturates there); a NaN stays one.  No number
                // then lands in the top exponent, so a byte that has it came from a NaN: the
                // instruction stored 0x7F or 0xFF for it, and the leaf's NaN is 0x7F.
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float t[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const float x = r[4 * j + k];
                        const float clamped = __builtin_fminf(__builtin_fmaxf(x, -240.0f), 240.0f);
                        t[k] = (x != x) ? as_f32_hd(0x7FC00000u) : clamped;
                    }
                    const uint32_t word = hw_f8_pack<DT>(t[2], t[3], hw_f8_pack<DT>(t[0], t[1], 0u, false), true);
                    w[j] = word & ~(((word & 0x78787878u) + 0x08080808u) & 0x80808080u);
                }
                return;
            }
            constexpr Fmt f = fmt_of(DT);
            constexpr uint32_t emask = (1u << f.ebits) - 1u, fmask = (1u << f.fbits) - 1u;
            constexpr uint32_t largest = ((emask - 1u) << f.fbits) | fmask;
            constexpr uint32_t over = f.infs ? (emask << f.fbits) : largest;
            constexpr uint32_t nan = (emask << f.fbits) | (f.finite_only ? fmask : 1u << (f.fbits - 1));
            // F8_E5M2: the rest still goes through the instructions (a zero stands in for the odd
            // ones), and the bytes of the odd ones are what encode_f32 stores for them: the leaf's
            // NaN, or the signed overflow value -- 57344 below the halfway point to 2^16 and
            // infinity from there on (the tie goes to the even neighbour, the infinity's place).
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float t[4];
                uint32_t keep = 0xFFFFFFFFu, put = 0u;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float x = r[4 * j + k];
                    const bool odd = !(__builtin_fabsf(x) <= hw_f8_limit<DT>());
                    const uint32_t sign = (as_u32_hd(x) >> 31) << 7;
                    uint32_t code = sign | over;
                    if constexpr (DT == DT_F8_E5M2) code = __builtin_fabsf(x) < 61440.0f ? (sign | largest) : code;
                    code = (x != x) ? nan : code;
                    t[k] = odd ? 0.0f : x;
                    keep = odd ? keep & ~(0xFFu << (8 * k)) : keep;
                    put = odd ? put | (code << (8 * k)) : put;
                }
                const uint32_t word = hw_f8_pack<DT>(t[2], t[3], hw_f8_pack<DT>(t[0], t[1], 0u, false), true);
                w[j] = (word & keep) | put;
            }
        }
    }
}

struct TileRow {
    uint32_t row, tc, ncols;
    bool live;
};

__device__ __forceinline__ TileRow tile_row_of(uint32_t g, uint32_t rows_per_plane, uint32_t tile_cols,
                                               FastDiv div, uint32_t rows, uint32_t cols) {
    TileRow t;
    const uint32_t r = g & 15u, q = g >> 4;
    const uint32_t tr = tile_cols > 1 ? fast_div(q, div) : q;
    t.tc = q - tr * tile_cols;
    t.row = tr * kTile + r;
    t.live = g < rows_per_plane && t.row < rows;
    const uint32_t left = cols - t.tc * kTile;
    t.ncols = left < kTile ? left : kTile;
    return t;
}

#endif  // __HIPCC__

// Grid of the kernels that give one lane to every padded tile row of a plane:
// x covers one plane, y walks the planes.
inline int plane_grid(uint64_t tile_rows, uint64_t tile_cols, uint64_t planes, uint32_t* rows_per_plane,
                      dim3* grid) {
    uint64_t per;
    if (mul_overflows(tile_rows, tile_cols, &per) || mul_overflows(per, kTile, &per))
        return IOMX_ERR_OVERFLOW;
    if (per > 0xFFFFFF00ull || tile_cols > 0x0FFFFFFFull || planes > 0xFFFFFFFFull)
        return IOMX_ERR_OVERFLOW;
    *rows_per_plane = (uint32_t)per;
    *grid = dim3((uint32_t)((per + 255) / 256), (uint32_t)(planes < 65535 ? planes : 65535));
    return IOMX_OK;
}

}  // namespace iomx
