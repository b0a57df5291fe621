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
#include "iomx_rows.hpp"

namespace iomx {

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

template <int DT, int OP>
__global__ __launch_bounds__(256) void rows_kernel(const RowsArgs a) {
    constexpr int BITS = bits_of(DT);
    constexpr int K = BITS / 2;
    constexpr int kInputs = (OP == ROWS_OP_SILU || OP == ROWS_OP_COPY) ? 1 : 2;
    constexpr uint32_t kRowBytes = 2 * BITS, kTileBytes = 32 * BITS;
    const TileRow t = tile_row_of(blockIdx.x * 256u + threadIdx.x, a.rows_per_plane, a.tile_cols[2],
                                  a.div_tile_cols, a.rows, a.cols);
    if (!t.live) return;
    // the 2- and 4-bit leaves (4 and 8 bytes a tile row) request the rows of two planes before
    // the first is computed: U4 12.1 -> 11.4 us, F4 14.7 -> 13.9 us on [64,512,2048]; the 6- and
    // 8-bit floating leaves lost 4-10 % to it
    constexpr int kAhead = BITS <= 4 ? 2 : 1;
    for (uint32_t p0 = blockIdx.y; p0 < a.planes; p0 += gridDim.y * kAhead) {
      uint64_t planes_of[kAhead][3];
      uint32_t rows_of[kAhead][kInputs][K];
#pragma unroll
      for (int b = 0; b < kAhead; ++b) {
        const uint32_t p = p0 + b * gridDim.y;
        if (p >= a.planes) break;
        walk_planes(a.walk, p, planes_of[b]);
#pragma unroll
        for (int k = 0; k < kInputs; ++k) {
            const uint32_t rk = a.brow[k] ? 0u : t.row;
            const uint32_t tck = a.bcol[k] ? 0u : t.tc;
            const uint8_t* src = a.src[k] + planes_of[b][k] * a.plane_bytes[k]
                    + ((uint64_t)(rk >> 4) * a.tile_cols[k] + tck) * kTileBytes + (rk & 15u) * kRowBytes;
            // an operand that broadcasts is read again by other lanes and stays cached
            if (a.brow[k] | a.bcol[k]) load_row<BITS>(src, rows_of[b][k]);
            else load_row<BITS, true>(src, rows_of[b][k]);
        }
      }
#pragma unroll
      for (int b = 0; b < kAhead; ++b) {
        if (p0 + b * gridDim.y >= a.planes) break;
        const uint64_t (&plane)[3] = planes_of[b];
        const uint32_t (&in)[kInputs][K] = rows_of[b];
        uint32_t res[K];
        if constexpr (OP == ROWS_OP_COPY) {
#pragma unroll
            for (int j = 0; j < K; ++j) res[j] = in[0][j];
        } else if constexpr (has_hw_convert(DT)) {
            // the 4-, 6- and 8-bit floating leaves: one binary32 operation between the conversions.
            // Their operands are finite or (F8) decode to the infinity or NaN they stand for.
            float v[kInputs][kTile], r[kTile];
#pragma unroll
            for (int k = 0; k < kInputs; ++k) hw_decode_row<DT>(in[k], v[k]);
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i) {
                const float x = a.bcol[0] ? v[0][0] : v[0][i];
                if constexpr (kInputs == 2) r[i] = leaf_arith<OP>(x, a.bcol[1] ? v[1][0] : v[1][i]);
                else r[i] = silu_carrier(x);
            }
            // finite operands: only a quotient (0/0) can be a NaN
            hw_encode_row<DT, OP == IOMX_OP_DIV || has_hw_f8(DT)>(r, res);
        } else if constexpr (!is_float_leaf(DT) && BITS <= 4) {
#pragma unroll
            for (int j = 0; j < K; ++j)
                res[j] = swar_word<BITS, OP>(a.bcol[0] ? splat_lane<BITS>(in[0][0]) : in[0][j],
                                             a.bcol[1] ? splat_lane<BITS>(in[1][0]) : in[1][j]);
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
        store_row<BITS, true>(dst, res, t.ncols);
      }
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

// Sixteen elements of a tile row in the carrier T and back: by the conversion instructions
// for the narrow floating leaves, element by element otherwise.
template <int DT, typename T>
__device__ __forceinline__ void decode_row(const uint32_t (&w)[bits_of(DT) / 2], T (&v)[kTile]) {
    if constexpr (has_hw_convert(DT)) {
        hw_decode_row<DT>(w, v);
    } else {
#pragma unroll
        for (int i = 0; i < (int)kTile; ++i) v[i] = decode_as<DT, T>(get<bits_of(DT)>(w, i));
    }
}
template <int DT, typename T>
__device__ __forceinline__ void encode_row(const T (&y)[kTile], uint32_t (&w)[bits_of(DT) / 2]) {
    if constexpr (has_hw_convert(DT)) {
        hw_encode_row<DT>(y, w);
    } else {
#pragma unroll
        for (int j = 0; j < bits_of(DT) / 2; ++j) w[j] = 0;
#pragma unroll
        for (int i = 0; i < (int)kTile; ++i) put<bits_of(DT)>(w, i, encode_from<DT, T>(y[i]));
    }
}

// Order of src/cpu/queue.cpp:1187-1234 in the carrier T: mean = sum / F,
// shifted = mean + eps, root = sqrt, inverse = 1 / root, y = (x*inverse)*scale;
// a NaN result is stored in its positive form (:1124-1134).
// PER_WAVE: a wave per row, four rows per workgroup, no LDS and no barrier - for rows of at most
// 8192 features, where a workgroup per row would leave most lanes idle (2048 features are 128 tile
// rows: two a lane).  Otherwise a workgroup per row.
template <int DT, typename T, bool PER_WAVE>
__global__ __launch_bounds__(256) void rows_rmsnorm_kernel(const RowsRmsArgs a) {
    constexpr int BITS = bits_of(DT);
    constexpr int K = BITS / 2;
    constexpr uint32_t kRowBytes = 2 * BITS, kTileBytes = 32 * BITS;
    constexpr uint32_t kLanes = PER_WAVE ? 64 : 256, kRowsPerGroup = PER_WAVE ? 4 : 1;
    __shared__ T part[4];
    const uint32_t tid = PER_WAVE ? (threadIdx.x & 63u) : threadIdx.x;
    const uint32_t first = PER_WAVE ? blockIdx.x * 4u + (threadIdx.x >> 6) : blockIdx.x;
    for (uint64_t lin64 = first; lin64 < a.total_rows; lin64 += (uint64_t)gridDim.x * kRowsPerGroup) {
        const uint32_t lin = (uint32_t)lin64;
        const uint32_t p = a.rows > 1 ? fast_div(lin, a.div_rows) : lin;
        const uint32_t row = lin - p * a.rows;
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint64_t inplane = (uint64_t)(row >> 4) * a.tile_cols * kTileBytes + (row & 15u) * kRowBytes;
        const uint8_t* xrow = a.x + plane[0] * a.plane_bytes + inplane;
        uint8_t* orow = a.out + plane[1] * a.plane_bytes + inplane;
        T acc = 0;
        for (uint32_t tc = tid; tc < a.tile_cols; tc += kLanes) {
            uint32_t w[K];
            load_row<BITS>(xrow + (uint64_t)tc * kTileBytes, w);
            const uint32_t left = a.feats - tc * kTile;
            T v[kTile];
            decode_row<DT, T>(w, v);
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i)
                if ((uint32_t)i < left) acc = acc + v[i] * v[i];
        }
        acc = wave_sum(acc);
        T total = acc;
        if constexpr (!PER_WAVE) {
            if ((tid & 63u) == 0) part[tid >> 6] = acc;
            __syncthreads();
            total = ((part[0] + part[1]) + part[2]) + part[3];
        }
        const T mean = total / (T)a.feats;
        const T shifted = mean + (T)a.eps;
        const T root = carrier_sqrt(shifted);
        const T inverse = (T)1 / root;
        for (uint32_t tc = tid; tc < a.tile_cols; tc += kLanes) {
            uint32_t w[K], s[K], res[K];
            load_row<BITS>(xrow + (uint64_t)tc * kTileBytes, w);
            load_row<BITS>(a.scale + (uint64_t)tc * kTileBytes, s);
            T v[kTile], g[kTile], y[kTile];
            decode_row<DT, T>(w, v);
            decode_row<DT, T>(s, g);
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i) {
                const T normalized = v[i] * inverse;
                y[i] = normalized * g[i];
            }
            encode_row<DT, T>(y, res);
            const uint32_t left = a.feats - tc * kTile;
            store_row<BITS>(orow + (uint64_t)tc * kTileBytes, res, left < kTile ? left : kTile);
        }
        if constexpr (!PER_WAVE) __syncthreads();
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
        if (op == IOMX_OP_DIV) { launch_rows_kernel<DT, IOMX_OP_DIV>(a, grid, s); return IOMX_OK; }
        if (op == ROWS_OP_SILU) { launch_rows_kernel<DT, ROWS_OP_SILU>(a, grid, s); return IOMX_OK; }
    }
    return IOMX_ERR_UNSUPPORTED;
}

template <int DT>
void launch_copy_rows(const RowsArgs& a, dim3 grid, hipStream_t s) {
    launch_rows_kernel<DT, ROWS_OP_COPY>(a, grid, s);
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
    // A lane's tile row is 4 to 16 bytes for the leaves of at most 8 bits: where the launch has
    // workgroups to spare a lane walks four planes (two for the 8-bit leaves) with the one
    // decomposition of its index (measured on [64,512,2048]: F6 21.8 -> 17.5 us, F4 16.9 -> 14.1,
    // U4 14.2 -> 12.0, F8 24.4 -> 22.5; eight planes a lane were slower again)
    if (bits <= 8) {
        uint32_t per = bits == 8 ? 2 : 4;
        while (per > 1 && (uint64_t)grid.x * ((grid.y + per - 1) / per) < 4096) per /= 2;
        grid.y = (grid.y + per - 1) / per;
    }
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
    const bool per_wave = a.tile_cols <= 512;
    const uint32_t groups = per_wave ? (a.total_rows + 3) / 4 : a.total_rows;
    const uint32_t grid = groups < (1u << 20) ? groups : (1u << 20);
#define IOMX_RMS(DTV, T)                                                                                       \
    do {                                                                                                       \
        if (per_wave) hipLaunchKernelGGL((rows_rmsnorm_kernel<DTV, T, true>), dim3(grid), dim3(256), 0, stream, a); \
        else hipLaunchKernelGGL((rows_rmsnorm_kernel<DTV, T, false>), dim3(grid), dim3(256), 0, stream, a);     \
    } while (0)
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
