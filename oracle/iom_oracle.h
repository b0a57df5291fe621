/*
 * iom_oracle.h — CPU restatement of IOM's reference CPU backend for the
 * memory-bound tensor ops (binary ADD/SUB/MUL/DIV, RMSNorm, SiLU, the softmax
 * stage of SDPA, tiled copy, host transfer scatter/gather).
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker the GPU path is compared
 * against.  Nothing shipped may call it: only tests, the smoke check and the
 * benchmark's CPU-baseline leg link or load this library.
 *
 * Each function names the reference file:line whose algorithm it follows
 * (paths relative to the rlewczuk/iom tree).
 *
 * Pinning status (what fixes each function's results, beyond this file):
 *   iomo_scalar_binary   reference KATs test/backend/test_scalar_add.cpp:42-132,
 *                        closed form (IEEE-754 single rounding, two's-complement
 *                        wrap), and the compiled reference CPU backend.  DIV:
 *                        the KATs of :50-53,94,101, an integer quotient with a
 *                        sticky bit, numpy's binary16/binary32 division, and the
 *                        compiled reference over every pair of the narrow leaves.
 *   iomo_binary          broadcast fixtures of backend_conformance_add_gpu.hpp:242-394,
 *                        brute-force index invariant, compiled reference.
 *   iomo_rmsnorm         closed form for all-ones rows
 *                        (backend_conformance_rmsnorm_reference.hpp:1347-1367),
 *                        float64 cross-check, compiled reference (bit-exact).
 *   iomo_silu            tails and ulp ceilings of test/backend/test_scalar_silu.cpp,
 *                        float64 cross-check, compiled reference (bit-exact, same libm).
 *   iomo_softmax         special-row KATs test/rocm/test_rocm_sdpa_nonmatrix.cpp:607-648,
 *                        sum-to-one invariant, and the compiled reference's sdpa
 *                        driven with identity K and V.
 *   iomo_cache_append / iomo_embedding / iomo_rope
 *                        compiled reference, bit for bit (rope with the same libm);
 *                        rope also against a float64 evaluation and the identity
 *                        at position 0.
 *   iomo_copy / scatter / gather
 *                        bit identity and the closed-form slot formula
 *                        (test/test_iom.cpp:614-706), compiled reference.
 */
#ifndef IOM_ORACLE_H
#define IOM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Leaf codes: numeric values of iom::DataType (include/iom/tensor.hpp:10-33). */
enum {
    IOMO_DT_BOOL = 0,
    IOMO_DT_I2 = 1, IOMO_DT_U2 = 2, IOMO_DT_I4 = 3, IOMO_DT_U4 = 4,
    IOMO_DT_I8 = 5, IOMO_DT_U8 = 6, IOMO_DT_I16 = 7, IOMO_DT_U16 = 8,
    IOMO_DT_I32 = 9, IOMO_DT_U32 = 10, IOMO_DT_I64 = 11, IOMO_DT_U64 = 12,
    IOMO_DT_F4_E2M1 = 13, IOMO_DT_F6_E2M3 = 14, IOMO_DT_F6_E3M2 = 15,
    IOMO_DT_F8_E4M3FN = 16, IOMO_DT_F8_E5M2 = 17, IOMO_DT_F8_E8M0 = 18,
    IOMO_DT_F16 = 19, IOMO_DT_BF16 = 20, IOMO_DT_F32 = 21, IOMO_DT_F64 = 22
};

/* Binary operations in the order of scalar_binary_codec.hpp:9. */
enum { IOMO_OP_ADD = 0, IOMO_OP_MUL = 1, IOMO_OP_SUB = 2, IOMO_OP_DIV = 3 };

enum {
    IOMO_OK = 0,
    IOMO_ERR_INVALID = -1,     /* std::invalid_argument in the reference */
    IOMO_ERR_UNSUPPORTED = -2  /* UnsupportedOperation */
};

/*
 * A tensor view over 16x16-tiled owner storage
 * (include/iom/tensor.hpp:262-335).  dims is the view's logical shape; the
 * final two dims equal the owner's.  plane_offset and plane_strides count
 * whole owner planes.
 */
typedef struct iomo_view {
    void* base;
    uint32_t rank;
    uint64_t dims[8];
    uint64_t plane_offset;
    uint64_t plane_strides[6];
} iomo_view;

/* src/tensor.cpp:107-134: bit width of a leaf (0 for an unknown code); bytes for
 * the byte-sized ones (0 otherwise). */
unsigned iomo_leaf_bits(int dtype);
size_t iomo_leaf_bytes(int dtype);
/* src/tensor.cpp:136-164: element slot of (plane,row,column). */
uint64_t iomo_plane_slot(uint64_t rows, uint64_t cols, uint64_t plane,
                         uint64_t row, uint64_t col);
/* src/tensor.cpp:95-102: elements of one padded plane. */
uint64_t iomo_plane_elems(uint64_t rows, uint64_t cols);

/* src/shared/scalar_binary_codec.hpp:163-178 with the long-double host traits
 * of src/shared/scalar_add.hpp:15-39. */
uint64_t iomo_scalar_binary(int op, int dtype, uint64_t a, uint64_t b);
/* Closed form: one IEEE-754 operation in a carrier wide enough to be exact or
 * innocuously rounded (binary32 for F32/BF16, binary64 for the narrower formats
 * and for F64 itself), one rounding on the integer significand, canonical NaN,
 * two's-complement wrap.  Must equal the codec for every leaf but F64, where
 * the host codec's 64-bit-significand carrier rounds twice. */
uint64_t iomo_scalar_binary_ieee(int op, int dtype, uint64_t a, uint64_t b);
/* src/shared/scalar_silu.hpp:69-97 with the float carrier of
 * src/cpu/device_internal.hpp:20-49. */
uint64_t iomo_scalar_silu(int dtype, uint64_t raw);
/* BF16 round-to-nearest-even encode of a float through the codec
 * (scalar_binary_codec.hpp:67-108). */
uint16_t iomo_encode_bf16(float value);

/* src/cpu/queue.cpp:414-536 + src/device_ops_binary.cpp:61-181 (shape rules).
 * use_ieee != 0 selects the closed-form element rule (fast). */
int iomo_binary(int op, int dtype, const iomo_view* lhs, const iomo_view* rhs,
                const iomo_view* out, int use_ieee);
/* src/cpu/queue.cpp:1144-1296 (portable path), src/device_ops_rmsnorm.cpp:75-127. */
int iomo_rmsnorm(int dtype, const iomo_view* x, const iomo_view* scale,
                 const iomo_view* out, float eps);
/* src/cpu/queue.cpp:1774-1838. */
int iomo_silu(int dtype, const iomo_view* x, const iomo_view* y);
/* src/cpu/queue.cpp:2274-2303, src/device_ops_copy.cpp:9-52. */
int iomo_copy(int dtype, const iomo_view* src, const iomo_view* dst);
/* src/cpu/tensor.cpp:79-167: logical row-major packed bits <-> tiled view. */
int iomo_scatter(int dtype, const iomo_view* dst, const void* logical);
int iomo_gather(int dtype, const iomo_view* src, void* logical);

/* destination[..., h, a + r, d] = source[..., h, r, d]
 * (src/cpu/queue.cpp:2227-2272, src/device_ops_cache_append.cpp:160-270). */
int iomo_cache_append(int dtype, const iomo_view* src, const iomo_view* dst, uint64_t a);
/* out[..., r, f] = table[indices[..., 0, r], f] (src/cpu/queue.cpp:941-1038);
 * IOMO_ERR_INVALID for a negative or out-of-vocabulary index. */
int iomo_embedding(int dtype, int index_dtype, const iomo_view* table,
                   const iomo_view* indices, const iomo_view* out);
/* Split-half rotary position encoding (src/cpu/queue.cpp:1341-1581,
 * src/device_ops_neural.cpp:241-362). */
int iomo_rope(int dtype, const iomo_view* x, const iomo_view* out, uint64_t a, double theta);

/* Linear projection out[b,r,o] = sum_i x[b,s+r,i] * w[o,i] and its head-planar
 * form (src/cpu/queue.cpp:1905-2051, docs/BACKEND_CONTRACT/linear-projections.md):
 * one fused multiply-add per increasing i in binary32 (binary64 for F64), integers
 * modulo 2^N, one encode.  NaN results are stored positive (NaN signs are outside
 * the contract). */
int iomo_linear(int dtype, const iomo_view* x, const iomo_view* w, const iomo_view* out,
                uint64_t s, uint64_t R, int head_planar, uint64_t H, uint64_t D);

/*
 * Causal grouped-query attention, BF16 (src/cpu/sdpa.cpp:132-336): q [B..,Hq,R,D],
 * k and v [B..,Hkv,C,D], out [B..,R,Hq*D]; row r sees tokens t < min(L, a+r+1).
 */
int iomo_sdpa(int dtype, const iomo_view* q, const iomo_view* k, const iomo_view* v,
              const iomo_view* out, uint64_t a, uint64_t L);

/*
 * Softmax stage.  Request shape follows src/rocm/sdpa_softmax.hpp:14-62
 * (strides in elements); arithmetic follows src/cpu/sdpa.cpp:214-309 with
 * scaled = score * scale as in src/rocm/sdpa_softmax.hip:131-132.
 */
typedef struct iomo_stage_layout {
    uint64_t plane_offset, plane_stride, head_stride, row_stride,
            column_stride, rows, columns;
} iomo_stage_layout;

typedef struct iomo_softmax_desc {
    uint64_t planes, heads, rows; /* logical rows per head            */
    uint64_t a;                   /* absolute position of row 0       */
    uint64_t L;                   /* initialized prefix length        */
    float scale;
    const float* scores;
    uint16_t* p_bf16;
    iomo_stage_layout scores_layout;
    iomo_stage_layout probability_layout;
} iomo_softmax_desc;

int iomo_softmax(const iomo_softmax_desc* desc);

#ifdef __cplusplus
}
#endif
#endif
