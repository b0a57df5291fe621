// The arithmetic of the chunk kernels, one 32-bit word (or one 64-bit element) at a time:
// ADD / SUB / MUL / DIV over the integers of 8 to 64 bits, F16, BF16, F32 and F64; SiLU and
// SiLU*up over the floating ones; copy.  Shared by the elementwise kernels, by the fused
// residual-add + RMSNorm kernel (which must form the very sum the ADD kernel stores) and by the
// device self-tests.
#pragma once

#include "iomx_leaves.hpp"
#include "iomx_rows.hpp"

namespace iomx {

// Internal operation codes: the four public binary operations keep their ABI
// values; the rest are private to the library.
enum { OP_SILU = 4, OP_COPY = 5, OP_SILU_MUL = 6 };

// The binary operations that broadcast (everything else takes whole planes only).
constexpr bool is_arithmetic(int op) { return op >= IOMX_OP_ADD && op <= IOMX_OP_DIV; }

// One IEEE operation in the carrier T.  Division needs no special cases beside
// IEEE's own: 0/0 and inf/inf are NaN, x/0 is a signed infinity, x/inf a signed zero.
template <int OP, typename T>
__device__ __forceinline__ T arith(T x, T y) {
    if constexpr (OP == IOMX_OP_ADD) return x + y;
    else if constexpr (OP == IOMX_OP_MUL) return x * y;
    else if constexpr (OP == IOMX_OP_SUB) return x - y;
    else return x / y;
}

template <int OP>
struct Arity { static constexpr int kInputs = (OP == OP_SILU || OP == OP_COPY) ? 1 : 2; };

// x * sigmoid(x) in binary32.  Both branches of the reference form
// (x >= 0: x / (1 + exp(-x)); x < 0: ((x*t)*t) / (1 + t*t), t = exp(x/2)) need
// one exponential of a non-positive argument, so one evaluation serves both.
// -inf maps to -0, +inf to +inf, zeros keep their sign, NaN stays NaN.
__device__ __forceinline__ float silu_f32(float x) {
    const bool pos = x >= 0.0f;
    const float e = expf(pos ? -x : x * 0.5f);
    const float xe = x * e;
    float num = pos ? x : xe * e;
    const float den = 1.0f + (pos ? e : e * e);
    if (!pos && e == 0.0f) num = -0.0f;  // covers -inf (inf*0) and the flushed tail
    return num / den;
}

// The same function for a BF16 result, where a few binary32 units in the last
// place show only at a rounding boundary: t = exp(-|x|/2) serves both signs (for
// x >= 0 the denominator 1 + t*t equals 1 + exp(-x)), the exponential is one
// multiply and one v_exp_f32 (relative error about 2^-21 for |x| < 16), and the
// quotient is a reciprocal multiply.  t underflows to zero only where the result
// is below every BF16 subnormal; the product t*t keeps its gradual underflow.
// A third of the instructions of silu_f32; within one BF16 unit of it.
__device__ __forceinline__ float silu_for_bf16(float x) {
    const float t = __builtin_amdgcn_exp2f(__builtin_fabsf(x) * -0.72134752f);
    const float tt = t * t;
    float num = (x >= 0.0f) ? x : (x * t) * t;
    if (x == -__builtin_inff()) num = -0.0f;  // -inf * 0
    return num * __builtin_amdgcn_rcpf(1.0f + tt);
}

// Leaf classes of the chunk kernels: signed and unsigned integers of one width
// share a class (two's-complement wrap does not see the sign).
constexpr bool is_float_class(int dt) {
    return dt == IOMX_DT_F16 || dt == IOMX_DT_BF16 || dt == IOMX_DT_F32 || dt == IOMX_DT_F64;
}

template <int DT, int OP>
__device__ __forceinline__ uint32_t op_word(uint32_t a, uint32_t b) {
    if constexpr (OP == OP_COPY) {
        return a;
    } else if constexpr (OP == OP_SILU) {
        if constexpr (DT == IOMX_DT_F32) return as_u32(canonical(silu_f32(as_f32(a))));
        else if constexpr (DT == IOMX_DT_F16) {
            const f32x2 x = f16_pair(a);
            return pack_f16(silu_for_bf16(x.x), silu_for_bf16(x.y));
        } else return pack_bf16(silu_for_bf16(bf16_lo(a)), silu_for_bf16(bf16_hi(a)));
    } else if constexpr (OP == OP_SILU_MUL) {
        // the activation is rounded to the leaf before the product, exactly as
        // the stored intermediate of the two-operation sequence
        if constexpr (DT == IOMX_DT_F32) {
            const float act = canonical(silu_f32(as_f32(a)));
            return as_u32(canonical(act * as_f32(b)));
        } else if constexpr (DT == IOMX_DT_F16) {
            const f32x2 x = f16_pair(a);
            const f32x2 act = f16_pair(pack_f16(silu_for_bf16(x.x), silu_for_bf16(x.y))), y = f16_pair(b);
            return pack_f16(act.x * y.x, act.y * y.y);
        } else {
            const uint32_t act = pack_bf16(silu_for_bf16(bf16_lo(a)), silu_for_bf16(bf16_hi(a)));
            return pack_bf16(bf16_lo(act) * bf16_lo(b), bf16_hi(act) * bf16_hi(b));
        }
    } else if constexpr (DT == IOMX_DT_I32) {
        if constexpr (OP == IOMX_OP_ADD) return a + b;
        else if constexpr (OP == IOMX_OP_MUL) return a * b;
        else return a - b;
    } else if constexpr (DT == IOMX_DT_I16) {
        // two 16-bit lanes: carries are kept out of the neighbour's top bit
        constexpr uint32_t H = 0x80008000u, L7 = 0x7FFF7FFFu;
        if constexpr (OP == IOMX_OP_ADD) return ((a & L7) + (b & L7)) ^ ((a ^ b) & H);
        else if constexpr (OP == IOMX_OP_SUB) return ((a | H) - (b & L7)) ^ ((a ^ ~b) & H);
        else return ((a & 0xFFFFu) * (b & 0xFFFFu) & 0xFFFFu) | ((a >> 16) * (b >> 16) << 16);
    } else if constexpr (DT == IOMX_DT_I8) {
        constexpr uint32_t H = 0x80808080u, L7 = 0x7F7F7F7Fu;
        if constexpr (OP == IOMX_OP_ADD) return ((a & L7) + (b & L7)) ^ ((a ^ b) & H);
        else if constexpr (OP == IOMX_OP_SUB) return ((a | H) - (b & L7)) ^ ((a ^ ~b) & H);
        else {
            uint32_t r = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                r |= ((((a >> (8 * i)) & 0xFFu) * ((b >> (8 * i)) & 0xFFu)) & 0xFFu) << (8 * i);
            return r;
        }
    } else if constexpr (DT == IOMX_DT_F32) {
        return as_u32(canonical(arith<OP>(as_f32(a), as_f32(b))));
    } else if constexpr (DT == IOMX_DT_F16) {
        // a binary32 quotient of two F16 values narrows with one rounding as well:
        // 24 significand bits are the 2*11 + 2 that make the second rounding harmless
        const f32x2 x = f16_pair(a), y = f16_pair(b);
        return pack_f16(arith<OP>(x.x, y.x), arith<OP>(x.y, y.y));
    } else {
        // BF16 pair.  The binary32 result of one operation on two BF16 values
        // is exact or correctly rounded with enough guard bits that the single
        // narrowing below is the only rounding that matters; binary32
        // subnormals are kept, so tiny products and quotients round once as well
        // (a quotient is correctly rounded to 24 >= 2*8 + 2 bits; in the binary32
        // subnormal range the BF16 grid is coarser by the same 16 bits).
        return pack_bf16(arith<OP>(bf16_lo(a), bf16_lo(b)), arith<OP>(bf16_hi(a), bf16_hi(b)));
    }
}

// One 64-bit element (two words of a chunk).
template <int DT, int OP>
__device__ __forceinline__ uint64_t op_wide(uint64_t a, uint64_t b) {
    if constexpr (OP == OP_COPY) {
        return a;
    } else if constexpr (DT == IOMX_DT_I64) {
        if constexpr (OP == IOMX_OP_ADD) return a + b;
        else if constexpr (OP == IOMX_OP_MUL) return a * b;
        else return a - b;
    } else {
        const double x = as_f64(a), y = as_f64(b);
        double r;
        if constexpr (OP == OP_SILU) r = silu_carrier(x);
        else if constexpr (OP == OP_SILU_MUL) {
            const double act = silu_carrier(x);
            r = ((act != act) ? as_f64(kQuietNanF64) : act) * y;
        } else r = arith<OP>(x, y);
        return (r != r) ? kQuietNanF64 : as_u64(r);
    }
}

template <int DT, int OP>
__device__ __forceinline__ u32x4 op_chunk(u32x4 a, u32x4 b) {
    u32x4 r;
    if constexpr (DT == IOMX_DT_I64 || DT == IOMX_DT_F64) {
        const uint64_t lo = op_wide<DT, OP>((uint64_t)a.x | ((uint64_t)a.y << 32), (uint64_t)b.x | ((uint64_t)b.y << 32));
        const uint64_t hi = op_wide<DT, OP>((uint64_t)a.z | ((uint64_t)a.w << 32), (uint64_t)b.z | ((uint64_t)b.w << 32));
        r.x = (uint32_t)lo; r.y = (uint32_t)(lo >> 32); r.z = (uint32_t)hi; r.w = (uint32_t)(hi >> 32);
    } else {
        r.x = op_word<DT, OP>(a.x, b.x);
        r.y = op_word<DT, OP>(a.y, b.y);
        r.z = op_word<DT, OP>(a.z, b.z);
        r.w = op_word<DT, OP>(a.w, b.w);
    }
    return r;
}

constexpr uint32_t class_bytes(int dt) {
    return dt == IOMX_DT_I8 ? 1 : (dt == IOMX_DT_I16 || dt == IOMX_DT_F16 || dt == IOMX_DT_BF16) ? 2
            : (dt == IOMX_DT_I64 || dt == IOMX_DT_F64) ? 8 : 4;
}

}  // namespace iomx
