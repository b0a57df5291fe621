// Linear projection out[b,r,o] = sum_i x[b,s+r,i] * w[o,i] (and its head-planar
// form out[b,h,r,d], o = h*D + d) on tiled operands.
//
//   linear_rows      every numeric leaf, the contract's scalar recurrence: integers
//                    modulo 2^N, floating leaves one fused multiply-add per
//                    increasing i in binary32 (binary64 for F64) from +0, one
//                    encode.  A lane owns one output tile row (16 outputs of one
//                    row) and walks the inner axis tile by tile.
//   linear_mfma      BF16 on the matrix cores (v_mfma_f32_16x16x16_bf16): products
//                    exact, binary32 accumulation, one round-to-nearest-even
//                    store.  A 16x16 tile of either operand is one MFMA operand as
//                    it lies in memory: lane l reads four consecutive inner
//                    elements of tile row l%16, so no staging or transposition is
//                    needed; the weight tile is the A operand so that a lane ends
//                    up with four consecutive outputs of one row.
#include "iomx_rows.hpp"

namespace iomx {

struct LinearArgs {
    const uint8_t* x;
    const uint8_t* w;         // the selected weight plane
    uint8_t* out;
    PlaneWalk<2> walk;        // 0 x, 1 out: the leading tuple shared by both
    uint64_t x_plane_bytes, out_plane_bytes;
    uint64_t head_stride;     // out planes per head (0 in ordinary mode)
    uint32_t T, I, O;         // x rows, inner extent, weight rows
    uint32_t s, R;            // row window
    uint32_t H, D;            // heads (1 in ordinary mode) and outputs per head
    uint32_t x_tile_cols, w_tile_cols, out_tile_cols;   // tiles along I (x, w) and D (out)
    uint32_t row_tiles;       // ceil(R / 16)
    uint32_t lanes_per_plane; // row_tiles * 16 * H * out_tile_cols
    uint32_t planes;
};

// ---------------------------------------------------------------------------
// Scalar recurrence
// ---------------------------------------------------------------------------

template <int DT>
struct Acc {
    using type = float;
};
template <> struct Acc<DT_F64> { using type = double; };
template <> struct Acc<DT_I64> { using type = uint64_t; };
template <> struct Acc<DT_I2> { using type = uint32_t; };
template <> struct Acc<DT_I4> { using type = uint32_t; };
template <> struct Acc<DT_I8> { using type = uint32_t; };
template <> struct Acc<DT_I16> { using type = uint32_t; };
template <> struct Acc<DT_I32> { using type = uint32_t; };

template <int DT, typename T>
__device__ __forceinline__ T operand(uint64_t raw) {
    if constexpr (!is_float_leaf(DT)) return (T)raw;
    else if constexpr (DT == DT_BF16) return (T)as_f32((uint32_t)raw << 16);
    else if constexpr (DT == DT_F32) return (T)as_f32((uint32_t)raw);
    else return decode_as<DT, T>(raw);
}

__device__ __forceinline__ float step(float a, float b, float acc) { return __builtin_fmaf(a, b, acc); }
__device__ __forceinline__ double step(double a, double b, double acc) { return __builtin_fma(a, b, acc); }
__device__ __forceinline__ uint32_t step(uint32_t a, uint32_t b, uint32_t acc) { return acc + a * b; }
__device__ __forceinline__ uint64_t step(uint64_t a, uint64_t b, uint64_t acc) { return acc + a * b; }

template <int DT, typename T>
__device__ __forceinline__ uint64_t result(T acc) {
    constexpr int BITS = bits_of(DT);
    if constexpr (!is_float_leaf(DT)) {
        if constexpr (BITS == 64) return (uint64_t)acc;
        else return (uint64_t)((uint32_t)acc & (BITS == 32 ? 0xFFFFFFFFu : ((1u << (BITS & 31)) - 1u)));
    } else if constexpr (DT == DT_BF16) {
        return bf16_rne_sw(as_u32((float)acc));
    } else if constexpr (DT == DT_F32) {
        return as_u32(canonical((float)acc));
    } else {
        return encode_from<DT, T>(acc);
    }
}

// One lane = one output tile row: row r of the window, head h, outputs
// d0 .. d0+15 of that head.  Lanes run over the rows of a row tile first, so the
// x tile rows they read and the output tile rows they write are contiguous.
template <int DT>
__global__ __launch_bounds__(256) void linear_rows_kernel(const LinearArgs a) {
    using T = typename Acc<DT>::type;
    constexpr int BITS = bits_of(DT);
    constexpr int K = BITS / 2;
    constexpr uint32_t kRowBytes = 2 * BITS, kTileBytes = 32 * BITS;
    const uint32_t g = blockIdx.x * 256u + threadIdx.x;
    if (g >= a.lanes_per_plane) return;
    const uint32_t r16 = g & 15u;
    uint32_t q = g >> 4;
    const uint32_t tr = q % a.row_tiles;
    q /= a.row_tiles;
    const uint32_t dt = q % a.out_tile_cols;
    const uint32_t h = q / a.out_tile_cols;
    const uint32_t r = tr * kTile + r16;
    if (r >= a.R) return;
    const uint32_t d0 = dt * kTile;
    const uint32_t nout = a.D - d0 < kTile ? a.D - d0 : kTile;
    const uint32_t srow = a.s + r;
    const uint64_t x_row = (uint64_t)(srow >> 4) * a.x_tile_cols * kTileBytes + (srow & 15u) * kRowBytes;
    const uint32_t o0 = h * a.D + d0;
    for (uint32_t p = blockIdx.y; p < a.planes; p += gridDim.y) {
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint8_t* xb = a.x + plane[0] * a.x_plane_bytes + x_row;
        T acc[kTile];
#pragma unroll
        for (int j = 0; j < (int)kTile; ++j) acc[j] = (T)0;
        for (uint32_t ti = 0; ti < a.x_tile_cols; ++ti) {
            const uint32_t extent = a.I - ti * kTile < kTile ? a.I - ti * kTile : kTile;
            uint32_t xw[K];
            load_row<BITS>(xb + (uint64_t)ti * kTileBytes, xw);
            T xv[kTile];
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i) xv[i] = operand<DT, T>(get<BITS>(xw, i));
#pragma unroll
            for (int j = 0; j < (int)kTile; ++j) {
                if ((uint32_t)j < nout) {
                    const uint32_t o = o0 + j;
                    uint32_t ww[K];
                    load_row<BITS>(a.w + ((uint64_t)(o >> 4) * a.w_tile_cols + ti) * kTileBytes
                                           + (o & 15u) * kRowBytes, ww);
                    if (extent == kTile) {
#pragma unroll
                        for (int i = 0; i < (int)kTile; ++i)
                            acc[j] = step(xv[i], operand<DT, T>(get<BITS>(ww, i)), acc[j]);
                    } else {
#pragma unroll
                        for (int i = 0; i < (int)kTile; ++i)
                            if ((uint32_t)i < extent)
                                acc[j] = step(xv[i], operand<DT, T>(get<BITS>(ww, i)), acc[j]);
                    }
                }
            }
        }
        uint32_t res[K];
#pragma unroll
        for (int j = 0; j < K; ++j) res[j] = 0;
#pragma unroll
        for (int j = 0; j < (int)kTile; ++j) put<BITS>(res, j, result<DT, T>(acc[j]));
        uint8_t* dst = a.out + (plane[1] + (uint64_t)h * a.head_stride) * a.out_plane_bytes
                + ((uint64_t)(r >> 4) * a.out_tile_cols + dt) * kTileBytes + (r & 15u) * kRowBytes;
        store_row<BITS>(dst, res, nout);
    }
}

// ---------------------------------------------------------------------------
// BF16 on the matrix cores
// ---------------------------------------------------------------------------

typedef short bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// Four consecutive BF16 of one tile row, columns c0..c0+3 of inner tile ti, zero
// where the inner index is past I (tile padding is never an operand).
__device__ __forceinline__ bf16x4_t load_k4(const uint8_t* tile_row, uint32_t c0, uint32_t i0, uint32_t I) {
    bf16x4_t v = {0, 0, 0, 0};
    if (i0 + 4 <= I) {
        v = *reinterpret_cast<const bf16x4_t*>(tile_row + c0 * 2);
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (i0 + j < I) v[j] = *reinterpret_cast<const short*>(tile_row + (c0 + j) * 2);
    }
    return v;
}

// One wave = MT row tiles x NT output tiles; a workgroup = 2 x 2 waves.
template <int MT, int NT>
__global__ __launch_bounds__(256) void linear_mfma_bf16_kernel(const LinearArgs a) {
    constexpr uint32_t kTileBytes = 512, kRowBytes = 32;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t l16 = lane & 15u, kg = lane >> 4;          // tile row, inner group of four
    const uint32_t rt0 = (blockIdx.x * 2 + (wave & 1u)) * MT;  // first row tile of this wave
    const uint32_t ot0 = (blockIdx.y * 2 + (wave >> 1)) * NT;  // first output tile (over O = H*D)
    const uint32_t o_tiles = (a.O + kTile - 1) / kTile;
    if (rt0 >= a.row_tiles || ot0 >= o_tiles) return;
    for (uint32_t p = blockIdx.z; p < a.planes; p += gridDim.z) {
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint8_t* xb = a.x + plane[0] * a.x_plane_bytes;
        // per-lane operand rows: x row for each row tile, w row for each output tile
        const uint8_t* xrow[MT];
        bool xok[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const uint32_t r = (rt0 + m) * kTile + l16;
            xok[m] = r < a.R;
            const uint32_t srow = a.s + (xok[m] ? r : 0);
            xrow[m] = xb + (uint64_t)(srow >> 4) * a.x_tile_cols * kTileBytes + (srow & 15u) * kRowBytes;
        }
        const uint8_t* wrow[NT];
        bool wok[NT];
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            const uint32_t o = (ot0 + n) * kTile + l16;
            wok[n] = o < a.O;
            const uint32_t oo = wok[n] ? o : 0;
            wrow[n] = a.w + (uint64_t)(oo >> 4) * a.w_tile_cols * kTileBytes + (oo & 15u) * kRowBytes;
        }
        f32x4_t acc[MT][NT];
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[m][n] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        for (uint32_t ti = 0; ti < a.x_tile_cols; ++ti) {
            const uint32_t i0 = ti * kTile + kg * 4;
            bf16x4_t xf[MT], wf[NT];
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                xf[m] = bf16x4_t{0, 0, 0, 0};
                if (xok[m]) xf[m] = load_k4(xrow[m] + (uint64_t)ti * kTileBytes, kg * 4, i0, a.I);
            }
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                wf[n] = bf16x4_t{0, 0, 0, 0};
                if (wok[n]) wf[n] = load_k4(wrow[n] + (uint64_t)ti * kTileBytes, kg * 4, i0, a.I);
            }
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int n = 0; n < NT; ++n)
                    acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(wf[n], xf[m], acc[m][n], 0, 0, 0);
        }
        // lane holds outputs o = tile*16 + 4*kg + j (j < 4) of row r = tile*16 + l16
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const uint32_t r = (rt0 + m) * kTile + l16;
            if (r >= a.R) continue;
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                const uint32_t o = (ot0 + n) * kTile + kg * 4;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t oj = o + j;
                    if (oj >= a.O) continue;
                    const uint32_t h = oj / a.D, d = oj - h * a.D;
                    uint8_t* dst = a.out + (plane[1] + (uint64_t)h * a.head_stride) * a.out_plane_bytes
                            + ((uint64_t)(r >> 4) * a.out_tile_cols + (d >> 4)) * kTileBytes
                            + (r & 15u) * kRowBytes + (d & 15u) * 2;
                    *reinterpret_cast<uint16_t*>(dst) = (uint16_t)bf16_rne_sw(as_u32(acc[m][n][j]));
                }
            }
        }
    }
}

namespace {

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

}  // namespace
}  // namespace iomx

using namespace iomx;

// Admission of docs/BACKEND_CONTRACT/linear-projections.md:86-112 (everything that
// can be checked without owner identities).  path: 0 = fastest conforming kernel
// (matrix cores for BF16), 1 = the scalar recurrence for every leaf.
extern "C" int iomx_launch_linear(int dtype, const iomx_view* x, const iomx_view* w,
                                  const iomx_view* out, uint64_t s, uint64_t R, int head_planar,
                                  uint64_t H, uint64_t D, int path, iomx_stream_t stream) {
    const uint32_t bits = leaf_bits(dtype);
    if (!bits) return IOMX_ERR_UNSUPPORTED;
    IOMX_TRY(check_view(x, bits));
    IOMX_TRY(check_view(w, bits));
    IOMX_TRY(check_view(out, bits));
    if (w->rank != 2) return IOMX_ERR_INVALID;
    const Matrix xm = matrix_of(*x), wm = matrix_of(*w), om = matrix_of(*out);
    if (wm.cols != xm.cols) return IOMX_ERR_INVALID;
    if (R == 0 || s > xm.rows || R > xm.rows - s) return IOMX_ERR_INVALID;
    if (head_planar) {
        uint64_t hd;
        if (H == 0 || D == 0 || mul_overflows(H, D, &hd) || hd != wm.rows) return IOMX_ERR_INVALID;
        if (out->rank != x->rank + 1 || out->rank > 8) return IOMX_ERR_INVALID;
    } else {
        if (H != 1 || D != wm.rows) return IOMX_ERR_INVALID;
        if (out->rank != x->rank) return IOMX_ERR_INVALID;
    }
    const uint32_t leading = x->rank - 2;
    for (uint32_t i = 0; i < leading; ++i) if (x->dims[i] != out->dims[i]) return IOMX_ERR_INVALID;
    if (head_planar && out->dims[leading] != H) return IOMX_ERR_INVALID;
    if (om.rows != R || om.cols != D) return IOMX_ERR_INVALID;
    if (out->base == x->base || out->base == w->base) return IOMX_ERR_INVALID;
    if (dtype == DT_BOOL || dtype == DT_F8_E8M0) return IOMX_ERR_UNSUPPORTED;
    if (xm.rows > 0xFFFFFFF0ull || xm.cols > 0xFFFFFFF0ull || wm.rows > 0xFFFFFFF0ull)
        return IOMX_ERR_OVERFLOW;

    LinearArgs a = {};
    uint64_t strides[2][kMaxLead] = {};
    uint64_t offsets[2] = {x->plane_offset, out->plane_offset};
    for (uint32_t i = 0; i < leading; ++i) {
        strides[0][i] = x->plane_strides[i];
        strides[1][i] = out->plane_strides[i];
    }
    IOMX_TRY(build_walk<2>(leading, x->dims, strides, offsets, &a.walk));
    a.x = static_cast<const uint8_t*>(x->base);
    a.w = static_cast<const uint8_t*>(w->base) + w->plane_offset * (wm.plane_elems * bits / 8);
    a.out = static_cast<uint8_t*>(out->base);
    a.x_plane_bytes = xm.plane_elems * bits / 8;
    a.out_plane_bytes = om.plane_elems * bits / 8;
    a.head_stride = head_planar ? out->plane_strides[leading] : 0;
    a.T = (uint32_t)xm.rows;
    a.I = (uint32_t)xm.cols;
    a.O = (uint32_t)wm.rows;
    a.s = (uint32_t)s;
    a.R = (uint32_t)R;
    a.H = (uint32_t)(head_planar ? H : 1);
    a.D = (uint32_t)D;
    a.x_tile_cols = (uint32_t)xm.tile_cols;
    a.w_tile_cols = (uint32_t)wm.tile_cols;
    a.out_tile_cols = (uint32_t)om.tile_cols;
    a.row_tiles = (uint32_t)((R + kTile - 1) / kTile);
    a.planes = (uint32_t)a.walk.planes;
    uint64_t lanes = (uint64_t)a.row_tiles * kTile * a.H;
    if (mul_overflows(lanes, (uint64_t)a.out_tile_cols, &lanes) || lanes > 0xFFFFFF00ull)
        return IOMX_ERR_OVERFLOW;
    a.lanes_per_plane = (uint32_t)lanes;
    const hipStream_t st = native(stream);
    const uint32_t gy = a.planes < 65535u ? a.planes : 65535u;

    if (dtype == DT_BF16 && path == 0) {
        const uint32_t o_tiles = (a.O + kTile - 1) / kTile;
        if (a.row_tiles <= 2) {
            // few rows (decode, last-row logits): one row tile per wave, more output tiles
            const dim3 grid((a.row_tiles + 1) / 2, (o_tiles + 15) / 16, gy);
            hipLaunchKernelGGL((linear_mfma_bf16_kernel<1, 8>), grid, dim3(256), 0, st, a);
        } else {
            const dim3 grid((a.row_tiles + 3) / 4, (o_tiles + 7) / 8, gy);
            hipLaunchKernelGGL((linear_mfma_bf16_kernel<2, 4>), grid, dim3(256), 0, st, a);
        }
        record_launch("linear_mfma", (a.row_tiles + 3) / 4, 256, (uint64_t)a.row_tiles * o_tiles * a.planes);
        IOMX_HIP(hipGetLastError());
        return IOMX_OK;
    }

    const dim3 grid((a.lanes_per_plane + 255) / 256, gy);
#define IOMX_LINEAR(DTV) hipLaunchKernelGGL((linear_rows_kernel<DTV>), grid, dim3(256), 0, st, a)
    switch (kernel_leaf(dtype)) {
        case DT_I2: IOMX_LINEAR(DT_I2); break;
        case DT_I4: IOMX_LINEAR(DT_I4); break;
        case DT_I8: IOMX_LINEAR(DT_I8); break;
        case DT_I16: IOMX_LINEAR(DT_I16); break;
        case DT_I32: IOMX_LINEAR(DT_I32); break;
        case DT_I64: IOMX_LINEAR(DT_I64); break;
        case DT_F4_E2M1: IOMX_LINEAR(DT_F4_E2M1); break;
        case DT_F6_E2M3: IOMX_LINEAR(DT_F6_E2M3); break;
        case DT_F6_E3M2: IOMX_LINEAR(DT_F6_E3M2); break;
        case DT_F8_E4M3FN: IOMX_LINEAR(DT_F8_E4M3FN); break;
        case DT_F8_E5M2: IOMX_LINEAR(DT_F8_E5M2); break;
        case DT_F16: IOMX_LINEAR(DT_F16); break;
        case DT_BF16: IOMX_LINEAR(DT_BF16); break;
        case DT_F32: IOMX_LINEAR(DT_F32); break;
        default: IOMX_LINEAR(DT_F64); break;
    }
#undef IOMX_LINEAR
    record_launch("linear_rows", grid.x, 256, (uint64_t)a.lanes_per_plane * a.planes);
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}
