// Every-leaf kernels: the binary operations over the integer leaves of 2..64
// bits and the floating leaves F4_E2M1, F6_E2M3, F6_E3M2, F8_E4M3FN, F8_E5M2,
// F16 and F64; SiLU and RMSNorm over those floating leaves; copy of any leaf
// under tile padding; host-transfer staging of any leaf, packed 2/4/6-bit ones
// included.  (I32 / U32 / F32 / BF16 arithmetic runs on the streaming kernels.)
//
// The unit of work is one tile row: sixteen consecutive elements = 2*bits
// bytes = bits/2 whole 32-bit words, contiguous in the tiled layout, so
// consecutive lanes touch consecutive memory for every leaf width.  A lane
// unpacks its sixteen elements, computes, repacks, and stores whole words; in a
// partial tile row it keeps the padding bits of the one word it shares with
// them.  Inputs are read before the output is stored, so an exact alias is safe.
//
// Element rule of the floating leaves (src/shared/scalar_binary_codec.hpp:45-148):
// decode to binary64, where every sum, difference and product of two values of
// at most 11 significand bits is exact; one round-to-nearest-even onto the
// leaf's grid, done on the integer significand; overflow to infinity where the
// leaf has one and to the largest finite magnitude otherwise; every NaN result
// as the leaf's positive canonical NaN (or, in the 4- and 6-bit leaves, which
// have none, the largest finite magnitude).  F64 computes in binary64 itself
// (the carrier of a device without an extended type,
// src/shared/standard_tiled_add.inl:116).
#include "iomx_leaves.hpp"

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

template <int BITS>
IOMX_HD void load_row(const uint8_t* p, uint32_t (&w)[BITS / 2]) {
    constexpr int K = BITS / 2;
    if constexpr (K == 1) {
        w[0] = *reinterpret_cast<const uint32_t*>(p);
    } else if constexpr (K == 2) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(p);
        w[0] = v.x;
        w[1] = v.y;
    } else if constexpr (K == 3) {
#pragma unroll
        for (int j = 0; j < 3; ++j) w[j] = reinterpret_cast<const uint32_t*>(p)[j];
    } else {
#pragma unroll
        for (int j = 0; j < K / 4; ++j) {
            const u32x4 v = reinterpret_cast<const u32x4*>(p)[j];
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
template <int BITS>
IOMX_HD void store_row(uint8_t* p, const uint32_t (&w)[BITS / 2], uint32_t ncols) {
    constexpr int K = BITS / 2;
    if (ncols == kTile) {
        if constexpr (K == 1) {
            *reinterpret_cast<uint32_t*>(p) = w[0];
        } else if constexpr (K == 2) {
            *reinterpret_cast<u32x2*>(p) = u32x2{w[0], w[1]};
        } else if constexpr (K == 3) {
#pragma unroll
            for (int j = 0; j < 3; ++j) reinterpret_cast<uint32_t*>(p)[j] = w[j];
        } else {
#pragma unroll
            for (int j = 0; j < K / 4; ++j)
                reinterpret_cast<u32x4*>(p)[j] = u32x4{w[4 * j], w[4 * j + 1], w[4 * j + 2], w[4 * j + 3]};
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
        // infinities and infinity times zero give NaN, an exact zero sum is +0 unless
        // both operands are -0, NaN operands give NaN.
        const double x = decode<DT>(a), y = decode<DT>(b);
        const double r = OP == IOMX_OP_ADD ? x + y : (OP == IOMX_OP_MUL ? x * y : x - y);
        return encode<DT>(r);
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
    else return encode<DT>((double)silu_carrier((float)decode<DT>(a)));
}

// ---------------------------------------------------------------------------
// Elementwise kernel: one lane per result tile row
// ---------------------------------------------------------------------------

struct RowsArgs {
    const uint8_t* src[2];
    uint8_t* out;
    PlaneWalk<3> walk;
    uint64_t plane_bytes[3];
    uint32_t tile_cols[3];
    uint32_t rows, cols;
    uint32_t rows_per_plane;  // padded tile rows of one result plane
    FastDiv div_tile_cols;    // by tile_cols[2]
    uint32_t planes;
    uint32_t brow[2], bcol[2];
};

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

template <int DT, int OP>
__global__ __launch_bounds__(256) void rows_kernel(const RowsArgs a) {
    constexpr int BITS = bits_of(DT);
    constexpr int K = BITS / 2;
    constexpr int kInputs = (OP == ROWS_OP_SILU || OP == ROWS_OP_COPY) ? 1 : 2;
    constexpr uint32_t kRowBytes = 2 * BITS, kTileBytes = 32 * BITS;
    const TileRow t = tile_row_of(blockIdx.x * 256u + threadIdx.x, a.rows_per_plane, a.tile_cols[2],
                                  a.div_tile_cols, a.rows, a.cols);
    if (!t.live) return;
    for (uint32_t p = blockIdx.y; p < a.planes; p += gridDim.y) {
        uint64_t plane[3];
        walk_planes(a.walk, p, plane);
        uint32_t in[kInputs][K];
#pragma unroll
        for (int k = 0; k < kInputs; ++k) {
            const uint32_t rk = a.brow[k] ? 0u : t.row;
            const uint32_t tck = a.bcol[k] ? 0u : t.tc;
            const uint8_t* src = a.src[k] + plane[k] * a.plane_bytes[k]
                    + ((uint64_t)(rk >> 4) * a.tile_cols[k] + tck) * kTileBytes + (rk & 15u) * kRowBytes;
            load_row<BITS>(src, in[k]);
        }
        uint32_t res[K];
        if constexpr (OP == ROWS_OP_COPY) {
#pragma unroll
            for (int j = 0; j < K; ++j) res[j] = in[0][j];
        } else {
#pragma unroll
            for (int j = 0; j < K; ++j) res[j] = 0;
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i) {
                const uint64_t x = a.bcol[0] ? get<BITS>(in[0], 0) : get<BITS>(in[0], i);
                uint64_t y;
                if constexpr (kInputs == 2) {
                    const uint64_t z = a.bcol[1] ? get<BITS>(in[1], 0) : get<BITS>(in[1], i);
                    y = leaf_binary<DT, OP>(x, z);
                } else {
                    y = leaf_silu<DT>(x);
                }
                put<BITS>(res, i, y);
            }
        }
        uint8_t* dst = a.out + plane[2] * a.plane_bytes[2]
                + ((uint64_t)(t.row >> 4) * a.tile_cols[2] + t.tc) * kTileBytes + (t.row & 15u) * kRowBytes;
        store_row<BITS>(dst, res, t.ncols);
    }
}

// ---------------------------------------------------------------------------
// RMSNorm: one workgroup per logical row, one lane per tile of the row
// ---------------------------------------------------------------------------

struct RowsRmsArgs {
    const uint8_t* x;
    const uint8_t* scale;
    uint8_t* out;
    PlaneWalk<2> walk;
    uint64_t plane_bytes;
    uint32_t rows, feats, tile_cols;
    uint32_t total_rows;  // view planes * rows
    FastDiv div_rows;
    float eps;
};

__device__ __forceinline__ float carrier_sqrt(float v) { return __builtin_sqrtf(v); }
__device__ __forceinline__ double carrier_sqrt(double v) { return __builtin_sqrt(v); }

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = v + __shfl_xor(v, off, 64);
    return v;
}

// Order of src/cpu/queue.cpp:1187-1234 in the carrier T: mean = sum / F,
// shifted = mean + eps, root = sqrt, inverse = 1 / root, y = (x*inverse)*scale;
// a NaN result is stored in its positive form (:1124-1134).
template <int DT, typename T>
__global__ __launch_bounds__(256) void rows_rmsnorm_kernel(const RowsRmsArgs a) {
    constexpr int BITS = bits_of(DT);
    constexpr int K = BITS / 2;
    constexpr uint32_t kRowBytes = 2 * BITS, kTileBytes = 32 * BITS;
    __shared__ T part[4];
    const uint32_t tid = threadIdx.x;
    for (uint32_t lin = blockIdx.x; lin < a.total_rows; lin += gridDim.x) {
        const uint32_t p = a.rows > 1 ? fast_div(lin, a.div_rows) : lin;
        const uint32_t row = lin - p * a.rows;
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint64_t inplane = (uint64_t)(row >> 4) * a.tile_cols * kTileBytes + (row & 15u) * kRowBytes;
        const uint8_t* xrow = a.x + plane[0] * a.plane_bytes + inplane;
        uint8_t* orow = a.out + plane[1] * a.plane_bytes + inplane;
        T acc = 0;
        for (uint32_t tc = tid; tc < a.tile_cols; tc += 256) {
            uint32_t w[K];
            load_row<BITS>(xrow + (uint64_t)tc * kTileBytes, w);
            const uint32_t left = a.feats - tc * kTile;
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i) {
                if ((uint32_t)i < left) {
                    const T v = (T)decode<DT>(get<BITS>(w, i));
                    acc = acc + v * v;
                }
            }
        }
        acc = wave_sum(acc);
        if ((tid & 63u) == 0) part[tid >> 6] = acc;
        __syncthreads();
        const T total = ((part[0] + part[1]) + part[2]) + part[3];
        const T mean = total / (T)a.feats;
        const T shifted = mean + (T)a.eps;
        const T root = carrier_sqrt(shifted);
        const T inverse = (T)1 / root;
        for (uint32_t tc = tid; tc < a.tile_cols; tc += 256) {
            uint32_t w[K], s[K], res[K];
            load_row<BITS>(xrow + (uint64_t)tc * kTileBytes, w);
            load_row<BITS>(a.scale + (uint64_t)tc * kTileBytes, s);
#pragma unroll
            for (int j = 0; j < K; ++j) res[j] = 0;
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i) {
                const T v = (T)decode<DT>(get<BITS>(w, i));
                const T g = (T)decode<DT>(get<BITS>(s, i));
                const T normalized = v * inverse;
                const T y = normalized * g;
                put<BITS>(res, i, encode<DT>((double)y));
            }
            const uint32_t left = a.feats - tc * kTile;
            store_row<BITS>(orow + (uint64_t)tc * kTileBytes, res, left < kTile ? left : kTile);
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------
// Host-transfer staging on the packed logical bit stream
// ---------------------------------------------------------------------------

struct BitArgs {
    uint8_t* tiled;
    uint32_t* words;
    PlaneWalk<1> walk;
    uint64_t plane_bytes;
    uint32_t rows, cols, tile_cols;
    uint32_t rows_per_plane;
    FastDiv div_tile_cols;
    uint32_t planes;
    uint64_t total_elems, total_words;
};

// One lane per destination tile row.
template <int BITS>
__global__ __launch_bounds__(256) void scatter_bits_kernel(const BitArgs a) {
    constexpr int K = BITS / 2;
    constexpr uint32_t kRowBytes = 2 * BITS, kTileBytes = 32 * BITS;
    const TileRow t = tile_row_of(blockIdx.x * 256u + threadIdx.x, a.rows_per_plane, a.tile_cols,
                                  a.div_tile_cols, a.rows, a.cols);
    if (!t.live) return;
    for (uint32_t p = blockIdx.y; p < a.planes; p += gridDim.y) {
        uint64_t plane[1];
        walk_planes(a.walk, p, plane);
        const uint64_t first = ((uint64_t)p * a.rows + t.row) * a.cols + (uint64_t)t.tc * kTile;
        uint32_t w[K];
#pragma unroll
        for (int j = 0; j < K; ++j) w[j] = 0;
#pragma unroll
        for (int i = 0; i < (int)kTile; ++i)
            if ((uint32_t)i < t.ncols) put<BITS>(w, i, read_bits<BITS>(a.words, (first + i) * BITS));
        uint8_t* dst = a.tiled + plane[0] * a.plane_bytes
                + ((uint64_t)(t.row >> 4) * a.tile_cols + t.tc) * kTileBytes + (t.row & 15u) * kRowBytes;
        store_row<BITS>(dst, w, t.ncols);
    }
}

// One lane per 32-bit word of the logical stream; bits past the last element
// are stored as zero (src/cpu/tensor.cpp:126-135).
template <int BITS>
__global__ __launch_bounds__(256) void gather_bits_kernel(const BitArgs a) {
    for (uint64_t j = blockIdx.x * 256ull + threadIdx.x; j < a.total_words;
         j += (uint64_t)gridDim.x * 256ull) {
        const uint64_t first_bit = j * 32ull;
        uint64_t e = first_bit / BITS;
        const uint64_t q = e / a.cols;
        uint32_t col = (uint32_t)(e - q * a.cols);
        uint64_t pl = q / a.rows;
        uint32_t row = (uint32_t)(q - pl * a.rows);
        uint32_t word = 0;
        while (e < a.total_elems && e * BITS < first_bit + 32ull) {
            uint64_t plane[1];
            walk_planes(a.walk, (uint32_t)pl, plane);
            const uint64_t slot = ((uint64_t)(row >> 4) * a.tile_cols + (col >> 4)) * kTileSlots
                    + (row & 15u) * kTile + (col & 15u);
            const uint64_t v = read_bits<BITS>(
                    reinterpret_cast<const uint32_t*>(a.tiled + plane[0] * a.plane_bytes), slot * BITS);
            const int64_t pos = (int64_t)(e * BITS) - (int64_t)first_bit;
            word |= pos >= 0 ? (uint32_t)(v << pos) : (uint32_t)(v >> -pos);
            ++e;
            if (++col == a.cols) {
                col = 0;
                if (++row == a.rows) { row = 0; ++pl; }
            }
        }
        a.words[j] = word;
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

namespace {

// signed and unsigned integers of one width share their kernels
int kernel_leaf(int dtype) {
    switch (dtype) {
        case DT_U2: return DT_I2;
        case DT_U4: return DT_I4;
        case DT_U8: return DT_I8;
        case DT_U16: return DT_I16;
        case DT_U32: return DT_I32;
        case DT_U64: return DT_I64;
        default: return dtype;
    }
}

// copies move raw bits: one kernel per width
int raw_leaf(int bits) {
    switch (bits) {
        case 2: return DT_I2;
        case 4: return DT_I4;
        case 6: return DT_F6_E2M3;
        case 8: return DT_I8;
        case 16: return DT_I16;
        case 32: return DT_I32;
        default: return DT_I64;
    }
}

template <int DT, int OP>
void launch_rows_kernel(const RowsArgs& a, dim3 grid, hipStream_t s) {
    hipLaunchKernelGGL((rows_kernel<DT, OP>), grid, dim3(256), 0, s, a);
}

template <int DT>
int dispatch_rows(int op, const RowsArgs& a, dim3 grid, hipStream_t s) {
    switch (op) {
        case IOMX_OP_ADD: launch_rows_kernel<DT, IOMX_OP_ADD>(a, grid, s); return IOMX_OK;
        case IOMX_OP_MUL: launch_rows_kernel<DT, IOMX_OP_MUL>(a, grid, s); return IOMX_OK;
        case IOMX_OP_SUB: launch_rows_kernel<DT, IOMX_OP_SUB>(a, grid, s); return IOMX_OK;
        default: break;
    }
    if constexpr (is_float_leaf(DT)) {
        if (op == ROWS_OP_SILU) { launch_rows_kernel<DT, ROWS_OP_SILU>(a, grid, s); return IOMX_OK; }
    }
    return IOMX_ERR_UNSUPPORTED;
}

template <int DT>
void launch_copy_rows(const RowsArgs& a, dim3 grid, hipStream_t s) {
    launch_rows_kernel<DT, ROWS_OP_COPY>(a, grid, s);
}

int plane_grid(uint64_t tile_rows, uint64_t tile_cols, uint64_t planes, uint32_t* rows_per_plane,
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

}  // namespace

int launch_rows(int op, int dtype, const RowsRequest& r, hipStream_t stream) {
    const int bits = bits_of(dtype);
    if (!bits) return IOMX_ERR_UNSUPPORTED;
    RowsArgs a = {};
    a.src[0] = r.src[0];
    a.src[1] = r.src[1];
    a.out = r.out;
    a.walk = r.walk;
    for (int k = 0; k < 3; ++k) {
        a.plane_bytes[k] = r.m[k].plane_elems * bits / 8;
        if (r.m[k].tile_cols > 0x0FFFFFFFull) return IOMX_ERR_OVERFLOW;
        a.tile_cols[k] = (uint32_t)r.m[k].tile_cols;
    }
    if (r.m[2].rows > 0xFFFFFFFFull || r.m[2].cols > 0xFFFFFFFFull) return IOMX_ERR_OVERFLOW;
    a.rows = (uint32_t)r.m[2].rows;
    a.cols = (uint32_t)r.m[2].cols;
    a.div_tile_cols = make_fast_div(a.tile_cols[2]);
    a.planes = (uint32_t)r.walk.planes;
    for (int k = 0; k < 2; ++k) { a.brow[k] = r.brow[k]; a.bcol[k] = r.bcol[k]; }
    dim3 grid;
    IOMX_TRY(plane_grid(r.m[2].tile_rows, r.m[2].tile_cols, r.walk.planes, &a.rows_per_plane, &grid));
    const char* name = "rows_binary";
    if (op == ROWS_OP_COPY) {
        switch (bits) {
            case 2: launch_copy_rows<DT_I2>(a, grid, stream); break;
            case 4: launch_copy_rows<DT_I4>(a, grid, stream); break;
            case 6: launch_copy_rows<DT_F6_E2M3>(a, grid, stream); break;
            case 8: launch_copy_rows<DT_I8>(a, grid, stream); break;
            case 16: launch_copy_rows<DT_I16>(a, grid, stream); break;
            case 32: launch_copy_rows<DT_I32>(a, grid, stream); break;
            default: launch_copy_rows<DT_I64>(a, grid, stream); break;
        }
        name = "rows_copy";
    } else {
        int rc = IOMX_ERR_UNSUPPORTED;
        switch (kernel_leaf(dtype)) {
            case DT_I2: rc = dispatch_rows<DT_I2>(op, a, grid, stream); break;
            case DT_I4: rc = dispatch_rows<DT_I4>(op, a, grid, stream); break;
            case DT_I8: rc = dispatch_rows<DT_I8>(op, a, grid, stream); break;
            case DT_I16: rc = dispatch_rows<DT_I16>(op, a, grid, stream); break;
            case DT_I64: rc = dispatch_rows<DT_I64>(op, a, grid, stream); break;
            case DT_F4_E2M1: rc = dispatch_rows<DT_F4_E2M1>(op, a, grid, stream); break;
            case DT_F6_E2M3: rc = dispatch_rows<DT_F6_E2M3>(op, a, grid, stream); break;
            case DT_F6_E3M2: rc = dispatch_rows<DT_F6_E3M2>(op, a, grid, stream); break;
            case DT_F8_E4M3FN: rc = dispatch_rows<DT_F8_E4M3FN>(op, a, grid, stream); break;
            case DT_F8_E5M2: rc = dispatch_rows<DT_F8_E5M2>(op, a, grid, stream); break;
            case DT_F16: rc = dispatch_rows<DT_F16>(op, a, grid, stream); break;
            case DT_F64: rc = dispatch_rows<DT_F64>(op, a, grid, stream); break;
            default: break;  // BOOL, F8_E8M0: no arithmetic; I32/U32/F32/BF16: streaming kernels
        }
        IOMX_TRY(rc);
        if (op == ROWS_OP_SILU) name = "rows_silu";
    }
    record_launch(name, grid.x, 256, (uint64_t)a.rows_per_plane * a.planes);
    return IOMX_OK;
}

int launch_rows_rmsnorm(int dtype, const RowsRmsnormRequest& r, hipStream_t stream) {
    const int bits = bits_of(dtype);
    if (!bits || !is_float_leaf(dtype) || dtype == DT_BF16 || dtype == DT_F32)
        return IOMX_ERR_UNSUPPORTED;
    RowsRmsArgs a = {};
    a.x = r.x;
    a.scale = r.scale;
    a.out = r.out;
    a.walk = r.walk;
    a.plane_bytes = r.m.plane_elems * bits / 8;
    uint64_t total;
    if (mul_overflows(r.walk.planes, r.m.rows, &total)) return IOMX_ERR_OVERFLOW;
    if (total > 0xFFFFFFFFull || r.m.cols > 0xFFFFFFFFull || r.m.tile_cols > 0x0FFFFFFFull)
        return IOMX_ERR_OVERFLOW;
    a.rows = (uint32_t)r.m.rows;
    a.feats = (uint32_t)r.m.cols;
    a.tile_cols = (uint32_t)r.m.tile_cols;
    a.total_rows = (uint32_t)total;
    a.div_rows = make_fast_div(a.rows);
    a.eps = r.eps;
    const uint32_t grid = a.total_rows < (1u << 20) ? a.total_rows : (1u << 20);
#define IOMX_RMS(DTV, T) \
    hipLaunchKernelGGL((rows_rmsnorm_kernel<DTV, T>), dim3(grid), dim3(256), 0, stream, a)
    switch (dtype) {
        case DT_F4_E2M1: IOMX_RMS(DT_F4_E2M1, float); break;
        case DT_F6_E2M3: IOMX_RMS(DT_F6_E2M3, float); break;
        case DT_F6_E3M2: IOMX_RMS(DT_F6_E3M2, float); break;
        case DT_F8_E4M3FN: IOMX_RMS(DT_F8_E4M3FN, float); break;
        case DT_F8_E5M2: IOMX_RMS(DT_F8_E5M2, float); break;
        case DT_F16: IOMX_RMS(DT_F16, float); break;
        default: IOMX_RMS(DT_F64, double); break;
    }
#undef IOMX_RMS
    record_launch("rows_rmsnorm", grid, 256, a.total_rows);
    return IOMX_OK;
}

int launch_bit_transfer(int dtype, const iomx_view* view, void* stream_words, bool scatter,
                        hipStream_t stream) {
    const int bits = bits_of(dtype);
    if (!bits) return IOMX_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(stream_words) & 3u) != 0) return IOMX_ERR_INVALID;
    const Matrix m = matrix_of(*view);
    BitArgs a = {};
    uint64_t strides[1][kMaxLead] = {};
    uint64_t offsets[1] = {view->plane_offset};
    for (uint32_t i = 0; i + 2 < view->rank; ++i) strides[0][i] = view->plane_strides[i];
    IOMX_TRY(build_walk<1>(view->rank - 2, view->dims, strides, offsets, &a.walk));
    a.tiled = static_cast<uint8_t*>(view->base);
    a.words = static_cast<uint32_t*>(stream_words);
    a.plane_bytes = m.plane_elems * bits / 8;
    if (m.rows > 0xFFFFFFFFull || m.cols > 0xFFFFFFFFull) return IOMX_ERR_OVERFLOW;
    a.rows = (uint32_t)m.rows;
    a.cols = (uint32_t)m.cols;
    a.tile_cols = (uint32_t)m.tile_cols;
    a.div_tile_cols = make_fast_div(a.tile_cols);
    a.planes = (uint32_t)a.walk.planes;
    dim3 grid;
    IOMX_TRY(plane_grid(m.tile_rows, m.tile_cols, a.walk.planes, &a.rows_per_plane, &grid));
    uint64_t t;
    if (mul_overflows(a.walk.planes, m.rows, &t) || mul_overflows(t, m.cols, &a.total_elems))
        return IOMX_ERR_OVERFLOW;
    if (mul_overflows(a.total_elems, (uint64_t)bits, &t)) return IOMX_ERR_OVERFLOW;
    a.total_words = (t + 31) / 32;
    if (scatter) {
#define IOMX_SC(B) hipLaunchKernelGGL((scatter_bits_kernel<B>), grid, dim3(256), 0, stream, a)
        switch (bits) {
            case 2: IOMX_SC(2); break;
            case 4: IOMX_SC(4); break;
            case 6: IOMX_SC(6); break;
            case 8: IOMX_SC(8); break;
            case 16: IOMX_SC(16); break;
            case 32: IOMX_SC(32); break;
            default: IOMX_SC(64); break;
        }
#undef IOMX_SC
        record_launch("scatter_bits", grid.x, 256, (uint64_t)a.rows_per_plane * a.planes);
    } else {
        const uint64_t blocks = (a.total_words + 255) / 256;
        const uint32_t gx = (uint32_t)(blocks < (1u << 20) ? blocks : (1u << 20));
#define IOMX_GA(B) hipLaunchKernelGGL((gather_bits_kernel<B>), dim3(gx), dim3(256), 0, stream, a)
        switch (bits) {
            case 2: IOMX_GA(2); break;
            case 4: IOMX_GA(4); break;
            case 6: IOMX_GA(6); break;
            case 8: IOMX_GA(8); break;
            case 16: IOMX_GA(16); break;
            case 32: IOMX_GA(32); break;
            default: IOMX_GA(64); break;
        }
#undef IOMX_GA
        record_launch("gather_bits", gx, 256, a.total_words);
    }
    return IOMX_OK;
}

}  // namespace iomx
