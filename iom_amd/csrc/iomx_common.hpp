// Shared host and device helpers of libiomx (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>

#include "iomx.h"

namespace iomx {

constexpr uint32_t kTile = 16;
constexpr uint32_t kTileSlots = 256;
constexpr uint32_t kMaxLead = 6;
constexpr uint32_t kWave = 64;

// ---------------------------------------------------------------------------
// Host: status plumbing
// ---------------------------------------------------------------------------

#define IOMX_HIP(call)                                   \
    do {                                                 \
        const hipError_t iomx_e_ = (call);               \
        if (iomx_e_ != hipSuccess) return (int)iomx_e_;  \
    } while (0)

#define IOMX_TRY(call)                      \
    do {                                    \
        const int iomx_s_ = (call);         \
        if (iomx_s_ != IOMX_OK) return iomx_s_; \
    } while (0)

inline hipStream_t native(iomx_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

void record_launch(const char* kernel, uint32_t grid, uint32_t block, uint64_t work);

// Bit width of every leaf (src/tensor.cpp:107-134); 0 for an unknown code.
inline uint32_t leaf_bits(int dtype) {
    static const uint8_t kBits[23] = {8, 2, 2, 4, 4, 8, 8, 16, 16, 32, 32, 64, 64, 4, 6, 6,
                                      8, 8, 8, 16, 16, 32, 64};
    return (dtype >= 0 && dtype < 23) ? kBits[dtype] : 0;
}

// The leaves whose arithmetic runs on the streaming kernels: the integers of 8 to
// 64 bits, F16, BF16, F32 and F64.
inline bool streaming_leaf(int dtype) {
    switch (dtype) {
        case IOMX_DT_I8: case IOMX_DT_U8: case IOMX_DT_I16: case IOMX_DT_U16:
        case IOMX_DT_I32: case IOMX_DT_U32: case IOMX_DT_I64: case IOMX_DT_U64:
        case IOMX_DT_F16: case IOMX_DT_BF16: case IOMX_DT_F32: case IOMX_DT_F64:
            return true;
        default:
            return false;
    }
}

inline uint32_t leaf_bytes(int dtype) {
    return streaming_leaf(dtype) ? leaf_bits(dtype) / 8 : 0;
}

inline bool mul_overflows(uint64_t a, uint64_t b, uint64_t* out) {
    return __builtin_mul_overflow(a, b, out);
}
inline bool add_overflows(uint64_t a, uint64_t b, uint64_t* out) {
    return __builtin_add_overflow(a, b, out);
}

// Geometry of the final two axes of one owner.
struct Matrix {
    uint64_t rows, cols;
    uint64_t tile_rows, tile_cols;
    uint64_t plane_elems;  // padded elements of one plane
};

inline Matrix matrix_of(const iomx_view& v) {
    Matrix m;
    m.rows = v.dims[v.rank - 2];
    m.cols = v.dims[v.rank - 1];
    m.tile_rows = (m.rows + kTile - 1) / kTile;
    m.tile_cols = (m.cols + kTile - 1) / kTile;
    m.plane_elems = m.tile_rows * m.tile_cols * kTileSlots;
    return m;
}

// Structural checks every operand must pass before any address is formed
// (same facts as validate_checked_view, src/device_ops.cpp:112-206, minus the
// owner identity that only the C++ layer knows).
inline int check_view(const iomx_view* v, uint32_t bits) {
    if (!v || !v->base) return IOMX_ERR_INVALID;
    if (v->rank < 2 || v->rank > 8) return IOMX_ERR_INVALID;
    for (uint32_t i = 0; i < v->rank; ++i)
        if (v->dims[i] == 0) return IOMX_ERR_INVALID;
    uint64_t max_plane = v->plane_offset;
    for (uint32_t i = 0; i + 2 < v->rank; ++i) {
        if (v->plane_strides[i] == 0) return IOMX_ERR_INVALID;
        uint64_t span;
        if (mul_overflows(v->dims[i] - 1, v->plane_strides[i], &span)) return IOMX_ERR_OVERFLOW;
        if (add_overflows(max_plane, span, &max_plane)) return IOMX_ERR_OVERFLOW;
    }
    const uint64_t rows = v->dims[v->rank - 2], cols = v->dims[v->rank - 1];
    if (rows > (1ull << 40) || cols > (1ull << 40)) return IOMX_ERR_OVERFLOW;
    const Matrix m = matrix_of(*v);
    uint64_t end;
    if (add_overflows(max_plane, 1, &end)) return IOMX_ERR_OVERFLOW;
    if (mul_overflows(end, m.plane_elems, &end)) return IOMX_ERR_OVERFLOW;
    if (mul_overflows(end, bits, &end)) return IOMX_ERR_OVERFLOW;
    if (end / 8 > (1ull << 47)) return IOMX_ERR_OVERFLOW;
    if ((reinterpret_cast<uintptr_t>(v->base) & 15u) != 0) return IOMX_ERR_INVALID;
    return IOMX_OK;
}

// ---------------------------------------------------------------------------
// Leading-plane mapping shared by every kernel: a row-major walk over up to six
// (coalesced) leading extents, with one plane stride per operand and axis.
// Passed to kernels by value.
// ---------------------------------------------------------------------------

// Division of a 32-bit value by a launch-invariant divisor d >= 2 as a multiply
// and two shifts (round-up method): with l = ceil(log2 d) and
// m = floor(2^32 (2^l - d) / d) + 1, n / d = (t + ((n - t) >> 1)) >> (l - 1) where
// t = mulhi(m, n), exact for every 32-bit n.  A wave that needs a plane
// coordinate pays five scalar operations instead of a reciprocal sequence.
struct FastDiv {
    uint32_t mul;
    uint32_t shift;  // l - 1
};

inline FastDiv make_fast_div(uint32_t d) {
    FastDiv f = {0, 0};
    if (d < 2) return f;
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    f.mul = (uint32_t)((((1ull << l) - d) << 32) / d + 1);
    f.shift = l - 1;
    return f;
}

template <int N>
struct PlaneWalk {
    uint32_t nlead;                 // axes in use
    uint32_t dims[kMaxLead];        // extents, outermost first
    FastDiv div[kMaxLead];          // division by dims[a]
    uint64_t stride[N][kMaxLead];   // owner planes per step, 0 = broadcast
    uint64_t offset[N];             // first owner plane
    uint64_t planes;                // product of dims
};

// Builds the walk from result-aligned strides, dropping unit axes and merging
// neighbours that every operand steps through contiguously.
template <int N>
inline int build_walk(uint32_t nlead, const uint64_t* dims,
                      const uint64_t (*strides)[kMaxLead], const uint64_t* offsets,
                      PlaneWalk<N>* w) {
    std::memset(w, 0, sizeof(*w));
    uint64_t planes = 1;
    uint32_t n = 0;
    uint64_t d[kMaxLead];
    uint64_t s[N][kMaxLead];
    for (uint32_t a = 0; a < nlead; ++a) {
        if (dims[a] == 1) continue;
        if (mul_overflows(planes, dims[a], &planes)) return IOMX_ERR_OVERFLOW;
        bool merge = n > 0;
        if (merge) {
            for (int k = 0; k < N; ++k) {
                uint64_t expect;
                if (mul_overflows(strides[k][a], dims[a], &expect)
                    || s[k][n - 1] != expect) { merge = false; break; }
            }
        }
        if (merge) {
            d[n - 1] *= dims[a];
            for (int k = 0; k < N; ++k) s[k][n - 1] = strides[k][a];
        } else {
            d[n] = dims[a];
            for (int k = 0; k < N; ++k) s[k][n] = strides[k][a];
            ++n;
        }
    }
    if (planes > 0xFFFFFFFFull) return IOMX_ERR_OVERFLOW;
    for (uint32_t a = 0; a < n; ++a) {
        if (d[a] > 0xFFFFFFFFull) return IOMX_ERR_OVERFLOW;
        w->dims[a] = static_cast<uint32_t>(d[a]);
        w->div[a] = make_fast_div(w->dims[a]);
        for (int k = 0; k < N; ++k) w->stride[k][a] = s[k][a];
    }
    w->nlead = n;
    w->planes = planes;
    for (int k = 0; k < N; ++k) w->offset[k] = offsets[k];
    return IOMX_OK;
}

// True when operand k walks its planes back to back (so the whole selection is
// one dense range starting at offset[k]).
template <int N>
inline bool walk_is_dense(const PlaneWalk<N>& w, int k) {
    if (w.nlead == 0) return true;
    return w.nlead == 1 && w.stride[k][0] == 1;
}

#if defined(__HIPCC__)

// ---------------------------------------------------------------------------
// Device helpers
// ---------------------------------------------------------------------------

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr uint32_t kQuietNanF32 = 0x7FC00000u;

__device__ __forceinline__ float as_f32(uint32_t b) { return __uint_as_float(b); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __float_as_uint(f); }

// Every NaN becomes the positive canonical quiet NaN (sign 0, top fraction bit).
__device__ __forceinline__ float canonical(float r) {
    return (r != r) ? as_f32(kQuietNanF32) : r;
}

// Software BF16 round-to-nearest-even of one binary32 encoding (NaN -> 0x7FC0).
__device__ __forceinline__ uint32_t bf16_rne_sw(uint32_t bits) {
    const uint32_t r = (bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16;
    return ((bits & 0x7FFFFFFFu) > 0x7F800000u) ? 0x7FC0u : r;
}

// Two binary32 values -> one packed BF16 pair (lo in bits 0..15).  The hardware
// conversion rounds to nearest even with gradual underflow; NaNs are replaced
// by the canonical encoding first so no payload or sign survives.
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 v = {canonical(lo), canonical(hi)};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// Two F16 values of one word as binary32 and back.  The widening is exact; the
// narrowing is the hardware's round-to-nearest-even with gradual underflow, and
// one binary32 operation between them rounds innocuously (24 >= 2*11 + 2), so
// the pair equals one correctly rounded binary16 operation.  NaN results are
// made canonical (0x7E00) before the narrowing.
__device__ __forceinline__ f32x2 f16_pair(uint32_t w) {
    return __builtin_convertvector(__builtin_bit_cast(f16x2, w), f32x2);
}
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
    const f32x2 v = {canonical(lo), canonical(hi)};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return as_f32(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return as_f32(w & 0xFFFF0000u); }

__device__ __forceinline__ uint32_t fast_div(uint32_t n, FastDiv f) {
    const uint32_t t = __umulhi(f.mul, n);
    return (t + ((n - t) >> 1)) >> f.shift;
}

// e^x for x <= 0 (-inf gives 0; NaN gives a finite value, callers handle NaN
// themselves), to about two units in the last place for |x| < 32, with gradual
// underflow.  n is the nearest integer to x*log2(e) and one FMA forms x*log2(e) - n
// from the exact product, so the rounding error of the product never reaches the
// fraction; the power of two is applied by v_ldexp_f32, which denormalises
// correctly where v_exp_f32 alone would flush.
__device__ __forceinline__ float exp_nonpos(float x) {
    const float a = fmaxf(x, -256.0f);  // bounds the integer part
    const float n = __builtin_rintf(a * 1.44269502e+00f);
    const float f = __builtin_fmaf(a, 1.44269502e+00f, -n);
    return __builtin_amdgcn_ldexpf(__builtin_amdgcn_exp2f(f), (int)n);
}

// Owner plane of operand k for the linear result plane p.  The outermost
// coordinate needs no division, and the loop stays rolled so that a launch with
// one leading axis (the common case) pays for none.
template <int N>
__device__ __forceinline__ void walk_planes(const PlaneWalk<N>& w, uint32_t p, uint64_t* out) {
#pragma unroll
    for (int k = 0; k < N; ++k) out[k] = w.offset[k];
    if (w.nlead == 0) return;
    uint32_t rem = p;
#pragma clang loop unroll(disable)
    for (uint32_t a = w.nlead - 1; a >= 1; --a) {
        const uint32_t d = w.dims[a];
        const uint32_t q = fast_div(rem, w.div[a]);
        const uint32_t c = rem - q * d;
        rem = q;
#pragma unroll
        for (int k = 0; k < N; ++k) out[k] += (uint64_t)c * w.stride[k][a];
    }
#pragma unroll
    for (int k = 0; k < N; ++k) out[k] += (uint64_t)rem * w.stride[k][0];
}

#endif  // __HIPCC__

}  // namespace iomx
