// Linear projection out[b,r,o] = sum_i x[b,s+r,i] * w[o,i] (and its head-planar
// form out[b,h,r,d], o = h*D + d) on tiled operands.
//
//   linear_rows      every numeric leaf, the contract's scalar recurrence: integers
//                    modulo 2^N, floating leaves one fused multiply-add per
//                    increasing i in binary32 (binary64 for F64) from +0, one
//                    encode.  A lane owns one output tile row (16 outputs of one
//                    row) and walks the inner axis tile by tile.
//   linear_mfma      BF16 on the matrix cores (v_mfma_f32_16x16x32_bf16): products
//                    exact, binary32 accumulation, one round-to-nearest-even
//                    store.  Two neighbouring 16x16 tiles of either operand are one
//                    MFMA operand as they lie in memory: lane l reads eight
//                    consecutive inner elements (16 bytes) of tile row l%16, so no
//                    transposition is needed; the weight tile is the A operand so
//                    that a lane ends up with four consecutive outputs of one row.
//                    The rows of all planes form one row axis.  Three kernels share
//                    this operand mapping: linear_mfma (operands straight from
//                    global memory, any shape), linear_mfma_splitk (few rows: the
//                    inner axis split over the waves of a workgroup so that every
//                    CU streams weights) and linear_mfma_lds (256 rows or more:
//                    256x256 workgroup tiles staged through LDS).
#include "iomx_rows.hpp"
#include "iomx_mfma.hpp"
#include <type_traits>

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
    uint32_t row_blocks, out_blocks, blocks_per_xcd;   // workgroup-tiled kernels: blocks of rows / of outputs
    uint32_t out_tile0;                         // ... and the first output tile of this launch
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

// The rows of every plane form one row axis (row index = plane * R + r), so a
// decode step of many sequences fills whole row tiles and reads the weight once.
// One wave = MT row tiles x NT output tiles, one v_mfma_f32_16x16x32_bf16 per pair
// and per 32 inner elements (two inner tiles); a workgroup = 2 x 2 waves.
template <int MT, int NT>
__global__ __launch_bounds__(256) void linear_mfma_bf16_kernel(const LinearArgs a) {
    constexpr uint32_t kTileBytes = 512, kRowBytes = 32;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t l16 = lane & 15u, kg = lane >> 4;          // tile row, group of eight inner elements
    const uint32_t total_rows = a.planes * a.R;
    const uint32_t row_tiles = (total_rows + kTile - 1) / kTile;
    const uint32_t o_tiles = (a.O + kTile - 1) / kTile;
    const uint32_t rt0 = (blockIdx.x * 2 + (wave & 1u)) * MT;
    const uint32_t ot0 = (blockIdx.y * 2 + (wave >> 1)) * NT;
    if (rt0 >= row_tiles || ot0 >= o_tiles) return;
    // per-lane operand rows
    const uint8_t* xrow[MT];
    uint8_t* orow[MT];     // output plane of the lane's row (head 0), advanced per head below
    uint32_t orow_r[MT];
    bool xok[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const uint32_t idx = (rt0 + m) * kTile + l16;
        xok[m] = idx < total_rows;
        const uint32_t p = xok[m] ? idx / a.R : 0;
        const uint32_t r = xok[m] ? idx - p * a.R : 0;
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint32_t srow = a.s + r;
        xrow[m] = a.x + plane[0] * a.x_plane_bytes
                + (uint64_t)(srow >> 4) * a.x_tile_cols * kTileBytes + (srow & 15u) * kRowBytes;
        orow[m] = a.out + plane[1] * a.out_plane_bytes
                + (uint64_t)(r >> 4) * a.out_tile_cols * kTileBytes + (r & 15u) * kRowBytes;
        orow_r[m] = r;
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
    const uint32_t tile_off = (kg >> 1) * kTileBytes, c0 = (kg & 1u) * 8u;
    // Rows and outputs past the end read row 0 / output 0 instead (valid memory):
    // an MFMA column only ever feeds its own outputs, which are not stored.  Only the
    // inner tail needs zeros.
    const uint32_t lane_off = tile_off + c0 * 2;
    const uint32_t full_steps = a.I >> 5;
#pragma unroll 1
    for (uint32_t step = 0; step < full_steps; ++step) {
        const uint64_t off = (uint64_t)step * (2 * kTileBytes) + lane_off;
        bf16x8_t xf[MT], wf[NT];
#pragma unroll
        for (int m = 0; m < MT; ++m)
            xf[m] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(xrow[m] + off));
#pragma unroll
        for (int n = 0; n < NT; ++n)
            wf[n] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(wrow[n] + off));
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n)
                acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[n], xf[m], acc[m][n], 0, 0, 0);
    }
    if ((a.I & 31u) != 0) {
        const uint32_t i0 = full_steps * 32 + kg * 8;
        const uint64_t off = (uint64_t)full_steps * (2 * kTileBytes) + tile_off;
        bf16x8_t xf[MT], wf[NT];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            xf[m] = __builtin_bit_cast(bf16x8_t, u32x4{0, 0, 0, 0});
            if (i0 < a.I) xf[m] = load_k8(xrow[m] + off, c0, i0, a.I);
        }
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            wf[n] = __builtin_bit_cast(bf16x8_t, u32x4{0, 0, 0, 0});
            if (i0 < a.I) wf[n] = load_k8(wrow[n] + off, c0, i0, a.I);
        }
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n)
                acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[n], xf[m], acc[m][n], 0, 0, 0);
    }
    // lane holds outputs o = tile*16 + 4*(lane/16) + j (j < 4) of its row
    const uint32_t og = (lane >> 4) * 4;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        if (!xok[m]) continue;
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            const uint32_t o = (ot0 + n) * kTile + og;
            if (o >= a.O) continue;
            if ((a.D & 15u) == 0) {
                // heads and output tiles are aligned: the four outputs are contiguous
                const uint32_t h = o / a.D, d = o - h * a.D;
                uint8_t* dst = orow[m] + (uint64_t)h * a.head_stride * a.out_plane_bytes
                        + (uint64_t)(d >> 4) * kTileBytes + (d & 15u) * 2;
                *reinterpret_cast<u32x2*>(dst) = u32x2{pack_bf16(acc[m][n][0], acc[m][n][1]),
                                                      pack_bf16(acc[m][n][2], acc[m][n][3])};
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t oj = o + j;
                    if (oj >= a.O) continue;
                    const uint32_t h = oj / a.D, d = oj - h * a.D;
                    uint8_t* dst = orow[m] + (uint64_t)h * a.head_stride * a.out_plane_bytes
                            + (uint64_t)(d >> 4) * kTileBytes + (d & 15u) * 2;
                    *reinterpret_cast<uint16_t*>(dst) = (uint16_t)bf16_rne_sw(as_u32(acc[m][n][j]));
                }
            }
        }
    }
    (void)orow_r;
}

// Few rows (a decode step, last-row logits): the weight is the traffic, read once,
// and the job is to have every CU streaming it.  One workgroup = NT output tiles
// against MT row tiles; its four waves take every fourth 32-element slice of the
// inner axis, so together they read each tile's weight rows as one contiguous
// stream, and their partial sums meet in LDS (added in wave order, so the result
// does not depend on timing).  When each row is the only row of its plane (one
// token per sequence) a 128-byte line of x holds 32 useful bytes, so x costs MT x
// 4 bytes of line traffic per weight byte-row it meets: with one or two row tiles
// the launch picks MT = 1 and lets NT output tiles share each x fragment; with more
// row tiles and many output tiles, 2 x 2, 2 x 4 or 4 x 4 tiles per workgroup read
// both operands less often from L2, which is what bounds those launches.
template <int MT, int NT, int SETS>
__global__ __launch_bounds__(256) void linear_mfma_splitk_bf16_kernel(const LinearArgs a) {
    constexpr uint32_t kTileBytes = 512, kRowBytes = 32;
    __shared__ f32x4_t partial[3][MT][NT][64];
    const uint32_t lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t l16 = lane & 15u, kg = lane >> 4;
    const uint32_t total_rows = a.planes * a.R;
    // workgroup id % 8 is the XCD: the row blocks of one output block run next to each
    // other on one XCD, so the weight rows they share come from that XCD's L2
    const uint32_t in_xcd = blockIdx.x >> 3;
    const uint32_t out_block = (in_xcd / a.row_blocks) * 8 + (blockIdx.x & 7u);
    if (out_block >= a.out_blocks) return;
    const uint32_t ot0 = out_block * NT, rt0 = (in_xcd % a.row_blocks) * MT;
    const uint8_t* xrow[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        uint32_t idx = (rt0 + m) * kTile + l16;
        if (idx >= total_rows) idx = 0;            // valid memory; its results are not stored
        const uint32_t p = idx / a.R, r = idx - p * a.R;
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint32_t srow = a.s + r;
        xrow[m] = a.x + plane[0] * a.x_plane_bytes
                + (uint64_t)(srow >> 4) * a.x_tile_cols * kTileBytes + (srow & 15u) * kRowBytes;
    }
    const uint8_t* wrow[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        uint32_t o_row = (ot0 + n) * kTile + l16;
        if (o_row >= a.O) o_row = 0;
        wrow[n] = a.w + (uint64_t)(o_row >> 4) * a.w_tile_cols * kTileBytes + (o_row & 15u) * kRowBytes;
    }
    f32x4_t acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    const uint32_t tile_off = (kg >> 1) * kTileBytes, c0 = (kg & 1u) * 8u;
    const uint32_t lane_off = tile_off + c0 * 2;
    const uint32_t full_steps = a.I >> 5;
    // SETS == 2 where a launch has at most one workgroup per CU (nothing else covers a wave's
    // waits there); with more workgroups than that the single set, which leaves registers for
    // a second workgroup per CU, was faster (64 rows x [32000,2048]: 43 against 48-50 us)
    uint32_t step;
    if constexpr (SETS == 2) {
        // Two register sets of kBatch slices each: while one set is multiplied the other is on
        // its way, so a wave always has kBatch to 2 x kBatch slices in flight -- what a wave waits
        // for is memory latency, and with one set it waited once per set.  The slices are still
        // multiplied in increasing order.
        constexpr uint32_t kBatch = (MT + NT) <= 3 ? 8 : 4;
        bf16x8_t wf0[kBatch][NT], xf0[kBatch][MT], wf1[kBatch][NT], xf1[kBatch][MT];
        auto request = [&](uint32_t at, bf16x8_t (&wf)[kBatch][NT], bf16x8_t (&xf)[kBatch][MT]) {
#pragma unroll
            for (uint32_t u = 0; u < kBatch; ++u) {
                const uint64_t off = (uint64_t)(at + 4 * u) * (2 * kTileBytes) + lane_off;
#pragma unroll
                for (int n = 0; n < NT; ++n)
                    wf[u][n] = __builtin_bit_cast(bf16x8_t, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[n] + off)));
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    xf[u][m] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(xrow[m] + off));
            }
        };
        auto multiply = [&](const bf16x8_t (&wf)[kBatch][NT], const bf16x8_t (&xf)[kBatch][MT]) {
#pragma unroll
            for (uint32_t u = 0; u < kBatch; ++u)
#pragma unroll
                for (int m = 0; m < MT; ++m)
#pragma unroll
                    for (int n = 0; n < NT; ++n)
                        acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][n], xf[u][m], acc[m][n], 0, 0, 0);
        };
        constexpr uint32_t kSpan = 4 * kBatch;                 // inner steps between the sets of one wave
        step = wave;
        bool whole = step + 4 * (kBatch - 1) < full_steps;     // a whole set starts at step
        if (whole) request(step, wf0, xf0);
        while (whole) {
            bool next = step + kSpan + 4 * (kBatch - 1) < full_steps;
            if (next) request(step + kSpan, wf1, xf1);
            multiply(wf0, xf0);
            step += kSpan;
            if (!next) break;
            next = step + kSpan + 4 * (kBatch - 1) < full_steps;
            if (next) request(step + kSpan, wf0, xf0);
            multiply(wf1, xf1);
            step += kSpan;
            whole = next;
        }
    } else {
        // kBatch slices a wave are requested before the first is multiplied: a wave has
        // only a few slices, and what it waits for is memory latency
        constexpr uint32_t kBatch = (MT + NT) <= 5 ? 8 : 4;
        step = wave;
        for (; step + 4 * (kBatch - 1) < full_steps; step += 4 * kBatch) {
            bf16x8_t wf[kBatch][NT], xf[kBatch][MT];
#pragma unroll
            for (uint32_t u = 0; u < kBatch; ++u) {
                const uint64_t off = (uint64_t)(step + 4 * u) * (2 * kTileBytes) + lane_off;
#pragma unroll
                for (int n = 0; n < NT; ++n)
                    wf[u][n] = __builtin_bit_cast(bf16x8_t, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[n] + off)));
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    xf[u][m] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(xrow[m] + off));
            }
#pragma unroll
            for (uint32_t u = 0; u < kBatch; ++u)
#pragma unroll
                for (int m = 0; m < MT; ++m)
#pragma unroll
                    for (int n = 0; n < NT; ++n)
                        acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][n], xf[u][m], acc[m][n], 0, 0, 0);
        }
    }
    for (; step < full_steps; step += 4) {
        const uint64_t off = (uint64_t)step * (2 * kTileBytes) + lane_off;
        bf16x8_t wf[NT], xf[MT];
#pragma unroll
        for (int n = 0; n < NT; ++n)
            wf[n] = __builtin_bit_cast(bf16x8_t, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[n] + off)));
#pragma unroll
        for (int m = 0; m < MT; ++m)
            xf[m] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(xrow[m] + off));
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n)
                acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[n], xf[m], acc[m][n], 0, 0, 0);
    }
    if ((a.I & 31u) != 0 && (full_steps & 3u) == wave) {
        const uint32_t i0 = full_steps * 32 + kg * 8;
        const uint64_t off = (uint64_t)full_steps * (2 * kTileBytes) + tile_off;
        bf16x8_t wf[NT], xf[MT];
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            wf[n] = __builtin_bit_cast(bf16x8_t, u32x4{0, 0, 0, 0});
            if (i0 < a.I) wf[n] = load_k8(wrow[n] + off, c0, i0, a.I);
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            xf[m] = __builtin_bit_cast(bf16x8_t, u32x4{0, 0, 0, 0});
            if (i0 < a.I) xf[m] = load_k8(xrow[m] + off, c0, i0, a.I);
        }
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n)
                acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[n], xf[m], acc[m][n], 0, 0, 0);
    }
    if (wave != 0) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) partial[wave - 1][m][n][lane] = acc[m][n];
    }
    __syncthreads();
    if (wave != 0) return;
    // lane holds outputs o = tile*16 + 4*(lane/16) + j (j < 4) of row l16 of its row tiles
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const uint32_t idx = (rt0 + m) * kTile + l16;
        if (idx >= total_rows) continue;
        const uint32_t p = idx / a.R, r = idx - p * a.R;
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        uint8_t* orow = a.out + plane[1] * a.out_plane_bytes
                + (uint64_t)(r >> 4) * a.out_tile_cols * kTileBytes + (r & 15u) * kRowBytes;
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            const uint32_t o = (ot0 + n) * kTile + kg * 4;
            if (o >= a.O) continue;
            f32x4_t v = acc[m][n];
#pragma unroll
            for (int k = 0; k < 3; ++k) v += partial[k][m][n][lane];
            if ((a.D & 3u) == 0 && o + 4 <= a.O) {
                // the four outputs lie in one head and one tile row
                const uint32_t h = o / a.D, d = o - h * a.D;
                uint8_t* dst = orow + (uint64_t)h * a.head_stride * a.out_plane_bytes
                        + (uint64_t)(d >> 4) * kTileBytes + (d & 15u) * 2;
                *reinterpret_cast<u32x2*>(dst) = u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
                continue;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t oj = o + j;
                if (oj >= a.O) continue;
                const uint32_t h = oj / a.D, d = oj - h * a.D;
                uint8_t* dst = orow + (uint64_t)h * a.head_stride * a.out_plane_bytes
                        + (uint64_t)(d >> 4) * kTileBytes + (d & 15u) * 2;
                *reinterpret_cast<uint16_t*>(dst) = (uint16_t)bf16_rne_sw(as_u32(v[j]));
            }
        }
    }
}

// ---------------------------------------------------------------------------
// BF16 on the matrix cores, operands staged through LDS
// ---------------------------------------------------------------------------
//
// A workgroup of eight waves owns 256 rows x 256 outputs; a wave owns 128 rows x
// 64 outputs (8 x 4 MFMA tiles, 128 accumulator registers).  The inner axis is
// walked in stages of 32*KS elements.  One "fragment" is the pair of neighbouring
// 16x16 tiles (1 KiB, contiguous in memory) that feeds one MFMA operand; a stage
// holds 16 row-tile and 16 output-tile fragments per 32 inner elements.  Fragments
// go from global memory to LDS with the direct loader (global_load_lds, 16 bytes a
// lane, no registers) into a ring of stage buffers, several stages ahead of the
// matrix cores, so every operand crosses L2->CU once per workgroup instead of once
// per wave.
//
// The direct loader puts lane i's 16 bytes at fragment + 16*i, so a fragment lies in
// LDS as it lies in memory.  ds_read_b128 serves the lanes {0-3, 12-15, 20-23, 24-27},
// {4-7, 8-11, 16-19, 28-31} (and the same +32) together; with lane l reading row l%16,
// inner elements 8*(l/16).., of the plain tiled fragment each such group touches 16
// different 16-byte bank groups, so the operand reads are conflict-free as stored.

// blockIdx.x -> (row block, output block).  The blocks are put in one sequence: panels of
// eight row blocks, inside a panel output block by output block; XCD id % 8 takes the id/8-th
// block of its eighth of the sequence.  So every XCD gets the same number of blocks (give or
// take one), and the 32 or 64 workgroups that run together on it cover about 8 row blocks x
// 4 or 8 output blocks: its L2 serves every operand slice to several workgroups for one fetch.
__device__ __forceinline__ bool block_of_workgroup(const LinearArgs& a, uint32_t* bx, uint32_t* by) {
    const uint32_t xcd = blockIdx.x & 7u, idx = blockIdx.x >> 3;
    const uint32_t at = xcd * a.blocks_per_xcd + idx;
    if (at >= a.row_blocks * a.out_blocks) return false;
    const uint32_t panel_blocks = 8 * a.out_blocks;
    const uint32_t panel = at / panel_blocks, rem = at - panel * panel_blocks;
    const uint32_t left = a.row_blocks - panel * 8, height = left < 8 ? left : 8;
    *by = rem / height;
    *bx = panel * 8 + (rem - *by * height);
    return true;
}

// GROUPS > 1: that many sets of WVM x WVN waves in one workgroup, each with a ring of its own
// over a GROUPS-th of the inner axis (I / 32 divisible by GROUPS); the partial sums meet in LDS
// at the end, in group order.  For launches with fewer blocks than CUs, whose duration is the
// time one workgroup needs for its chain of stages.
template <int WM, int WVM, int WVN, int DEPTH, int GROUPS = 1>
__global__ __launch_bounds__(WVM * WVN * 64 * GROUPS) __attribute__((amdgpu_waves_per_eu(2, 2)))
void linear_mfma_lds_bf16_kernel(const LinearArgs a) {
    constexpr int WN = 4;                                   // wave tile WM x WN, in 16x16 tiles
    constexpr int NW = WVM * WVN;                           // waves of a group, WVM along the rows
    constexpr uint32_t BM = WM * WVM, BN = WN * WVN;        // workgroup tile, in 16x16 tiles
    constexpr int KS = 1, HALF = WM / 2;                    // DEPTH stage buffers of 32 inner elements
    constexpr int LPS = (BM + BN) / NW;                     // direct loads per wave and stage
    static_assert(LPS == 4 && BM == 2 * NW && BN == 2 * NW, "two row and two output fragments per wave");
    static_assert(WM >= 4 && WM % 2 == 0 && LPS % HALF == 0, "loads spread over the second half of a stage");
    constexpr uint32_t kTileBytes = 512, kRowBytes = 32, kFrag = 1024;
    constexpr uint32_t kStageFrags = (BM + BN) * KS, kStageBytes = kStageFrags * kFrag;
    __shared__ __attribute__((aligned(16))) uint8_t all_rings[GROUPS * DEPTH * kStageBytes];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t group = GROUPS > 1 ? (threadIdx.x >> 6) / NW : 0, wave = (threadIdx.x >> 6) % NW;
    uint8_t* lds = all_rings + group * (DEPTH * kStageBytes);
    const uint32_t l16 = lane & 15u, kg = lane >> 4;
    const uint32_t total_rows = a.planes * a.R;
    uint32_t bx, by;
    if (!block_of_workgroup(a, &bx, &by)) return;
    const uint32_t bm0 = bx * BM, bn0 = a.out_tile0 + by * BN;   // first row tile / output tile
    const uint32_t wm = wave % WVM, wn = wave / WVM;
    // this group's part of the inner axis: stages [group * stages, (group + 1) * stages)
    const uint32_t stages = a.I / 32 / GROUPS;
    const uint64_t group_off = (uint64_t)group * stages * kFrag;

    // loader role: this wave brings in row fragments wave, wave+NW and output fragments
    // wave, wave+NW of every 32-element slice; lane i fetches 16-byte chunk i
    const uint32_t ld_tile = lane >> 5, ld_row = (lane & 31u) >> 1;
    const uint32_t ld_off = ld_tile * kTileBytes + (lane & 1u) * 16;
    const uint8_t* src[4];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        uint32_t idx = (bm0 + wave + NW * j) * kTile + ld_row;
        if (idx >= total_rows) idx = 0;            // valid memory; its results are not stored
        const uint32_t p = idx / a.R, r = idx - p * a.R;
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint32_t srow = a.s + r;
        src[j] = a.x + plane[0] * a.x_plane_bytes + (uint64_t)(srow >> 4) * a.x_tile_cols * kTileBytes
                + (srow & 15u) * kRowBytes + ld_off + group_off;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        uint32_t o = (bn0 + wave + NW * j) * kTile + ld_row;
        if (o >= a.O) o = 0;
        src[2 + j] = a.w + (uint64_t)(o >> 4) * a.w_tile_cols * kTileBytes + (o & 15u) * kRowBytes + ld_off
                + group_off;
    }
    auto issue = [&](uint32_t stage, uint32_t buf) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const uint64_t goff = (uint64_t)(stage * KS + ks) * kFrag;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t frag = ks * (BM + BN) + (j < 2 ? wave + NW * j : BM + wave + NW * (j - 2));
                __builtin_amdgcn_global_load_lds((gptr_t)(src[j] + goff),
                                                 (lptr_t)(lds + buf * kStageBytes + frag * kFrag), 16, 0, 0);
            }
        }
    };

    f32x4_t acc[WM][WN];
#pragma unroll
    for (int m = 0; m < WM; ++m)
#pragma unroll
        for (int n = 0; n < WN; ++n) acc[m][n] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // reader role: position of the lane's eight inner elements inside a fragment
    const uint32_t rd_off = (kg >> 1) * kTileBytes + l16 * kRowBytes + (kg & 1u) * 16;
    // A ring of DEPTH stage buffers (one stage = 32 inner elements; four for the large tile,
    // five for the small one whose stages are half as long) and two register sets of operand
    // fragments.  At the top of stage st every wave waits for its own loads of stage st+1 and
    // meets the others at the barrier: from there on stage st+1 is complete in LDS.  During the
    // stage the MFMAs run on the register set of stage st while the other set is read from the
    // buffer of stage st+1, one row fragment per step -- the matrix core never waits for LDS at a
    // stage boundary -- and the second half of the steps requests stage st+DEPTH-1 with direct
    // loads between the MFMA groups (a direct load holds its wave at issue until the memory
    // pipeline takes it; the MFMAs issued before it keep the matrix core busy meanwhile) into a
    // buffer whose stage everyone has long read into registers.
    const uint32_t last = stages - 1;
#pragma unroll
    for (uint32_t d = 0; d < DEPTH - 1; ++d) issue(d < stages ? d : last, d);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 2) * LPS) : "memory");
    __builtin_amdgcn_s_barrier();
    static_assert(WN <= WM, "WM + WN fragment reads fit two a step");
    bf16x8_t wf[2][WN], xf[2][WM];
    auto rd = [&](uint32_t ring, uint32_t frag) {
        return __builtin_bit_cast(bf16x8_t,
                *reinterpret_cast<const u32x4*>(lds + ring * kStageBytes + rd_off + frag * kFrag));
    };
#pragma unroll
    for (int n = 0; n < WN; ++n) wf[0][n] = rd(0, BM + wn * WN + n);
#pragma unroll
    for (int m = 0; m < WM; ++m) xf[0][m] = rd(0, wm * WM + m);
    // P = parity of the stage (which register set holds its fragments)
    auto stage = [&](auto parity, uint32_t st) {
        constexpr int P = decltype(parity)::value;
        // ring positions of the next stage and of the one requested now
        const uint32_t ring1 = (st + 1) % DEPTH, ring3 = (st + DEPTH - 1) % DEPTH;
        const uint64_t gnext = (uint64_t)(st + DEPTH - 1 < stages ? st + DEPTH - 1 : last) * kFrag;
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 3) * LPS) : "memory");
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int step = 0; step < WM; ++step) {
#pragma unroll
            for (int n = 0; n < WN; ++n)
                acc[step][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[P][n], xf[P][step], acc[step][n], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            // the WM + WN fragments of the next stage, two a step behind the step's MFMAs, the
            // last ones two steps before the stage ends: the wait for them at the top of the
            // next stage finds them landed
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                constexpr int kReads = WM + WN;
                const int f = 2 * step + i;
                if (f < 2 * WN) {
                    if (f & 1) wf[P ^ 1][f >> 1] = rd(ring1, BM + wn * WN + (f >> 1));
                    else xf[P ^ 1][f >> 1] = rd(ring1, wm * WM + (f >> 1));
                } else if (f < kReads) {
                    xf[P ^ 1][f - WN] = rd(ring1, wm * WM + (f - WN));
                }
            }
            if (step >= HALF) {
#pragma unroll
                for (int i = 0; i < LPS / HALF; ++i) {
                    const int j = (step - HALF) * (LPS / HALF) + i;
                    const uint32_t frag = j < 2 ? wave + NW * j : BM + wave + NW * (j - 2);
                    __builtin_amdgcn_global_load_lds((gptr_t)(src[j] + gnext),
                                                     (lptr_t)(lds + ring3 * kStageBytes + frag * kFrag), 16, 0, 0);
                }
            }
            // the step stays as written: left to itself the scheduler sinks the LDS reads of the
            // next stage to just before their use, and the matrix core waits for LDS there
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    uint32_t st = 0;
    for (; st + 1 < stages; st += 2) {
        stage(std::integral_constant<int, 0>{}, st);
        stage(std::integral_constant<int, 1>{}, st + 1);
    }
    if (st < stages) stage(std::integral_constant<int, 0>{}, st);
    // nothing may still be landing in LDS when the workgroup gives it back
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (GROUPS > 1) {
        // the other groups' partial sums through the (now idle) rings: [group - 1][wave][tile][lane]
        __syncthreads();
        f32x4_t* part = reinterpret_cast<f32x4_t*>(all_rings);
        static_assert((GROUPS - 1) * NW * WM * WN * 1024 <= GROUPS * DEPTH * kStageBytes, "partial sums fit the rings");
        if (group > 0) {
#pragma unroll
            for (int m = 0; m < WM; ++m)
#pragma unroll
                for (int n = 0; n < WN; ++n)
                    part[((((group - 1) * NW + wave) * WM + m) * WN + n) * 64 + lane] = acc[m][n];
        }
        __syncthreads();
        if (group > 0) return;
#pragma unroll 1
        for (uint32_t g = 0; g + 1 < GROUPS; ++g)
#pragma unroll
            for (int m = 0; m < WM; ++m)
#pragma unroll
                for (int n = 0; n < WN; ++n)
                    acc[m][n] += part[(((g * NW + wave) * WM + m) * WN + n) * 64 + lane];
    }

    // lane holds outputs o = tile*16 + 4*(lane/16) + j (j < 4) of row l16 of its row tiles.
    // Heads are whole tiles wide here, so head and tile of an output tile are the same
    // for the whole wave.
    const uint32_t d_tiles = a.D >> 4;
    uint64_t col_off[WN];
    bool col_ok[WN];
#pragma unroll
    for (int n = 0; n < WN; ++n) {
        const uint32_t ot = bn0 + wn * WN + n;
        col_ok[n] = ot * kTile < a.O;
        const uint32_t h = ot / d_tiles, dt = ot - h * d_tiles;
        col_off[n] = (uint64_t)h * a.head_stride * a.out_plane_bytes + (uint64_t)dt * kTileBytes + kg * 8;
    }
#pragma unroll
    for (int m = 0; m < WM; ++m) {
        const uint32_t idx = (bm0 + wm * WM + m) * kTile + l16;
        if (idx >= total_rows) continue;
        const uint32_t p = idx / a.R, r = idx - p * a.R;
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        uint8_t* orow = a.out + plane[1] * a.out_plane_bytes
                + (uint64_t)(r >> 4) * a.out_tile_cols * kTileBytes + (r & 15u) * kRowBytes;
#pragma unroll
        for (int n = 0; n < WN; ++n) {
            if (!col_ok[n]) continue;
            *reinterpret_cast<u32x2*>(orow + col_off[n]) = u32x2{pack_bf16(acc[m][n][0], acc[m][n][1]),
                                                                 pack_bf16(acc[m][n][2], acc[m][n][3])};
        }
    }
}

// 64 rows x 64 outputs per workgroup of four waves (a wave: 2 x 2 MFMA tiles): for
// problems whose larger tiles would leave CUs idle.  A stage of 32 inner elements is
// 8 KiB; with a ring of DEPTH stages four or five workgroups share a CU, and their
// waves cover each other's waits, so a stage is simply: wait for the own loads of the
// stage, barrier (the stage is complete and nobody reads the one before it any more),
// request the stage DEPTH-1 ahead into the freed buffer, read four fragments, four MFMAs.
// The fragments of a wave are 4 KiB per 4 MFMAs: the LDS ports, not the matrix cores,
// bound this kernel (at about half the matrix rate).
//
// KS > 1: when even these blocks are fewer than the CUs, KS groups of four waves each walk a
// KS-th of the inner axis with a ring of their own, and the partial sums meet in LDS at the end
// (in group order; the sum is then not the single sequence of the other kernels).
template <int DEPTH, int KS>
__global__ __launch_bounds__(256 * KS)
void linear_mfma_lds64_bf16_kernel(const LinearArgs a) {
    constexpr uint32_t BM = 4, BN = 4, NW = 4, LPS = 2;
    constexpr uint32_t kTileBytes = 512, kRowBytes = 32, kFrag = 1024;
    constexpr uint32_t kStageBytes = (BM + BN) * kFrag;
    __shared__ __attribute__((aligned(16))) uint8_t all_rings[KS * DEPTH * kStageBytes];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t slice = (threadIdx.x >> 6) / NW, wave = (threadIdx.x >> 6) % NW;   // group and role in it
    uint8_t* lds = all_rings + slice * DEPTH * kStageBytes;
    const uint32_t l16 = lane & 15u, kg = lane >> 4;
    const uint32_t total_rows = a.planes * a.R;
    uint32_t bx, by;
    if (!block_of_workgroup(a, &bx, &by)) return;
    const uint32_t bm0 = bx * BM, bn0 = a.out_tile0 + by * BN;
    const uint32_t wm = wave & 1u, wn = wave >> 1;

    // loader role: row fragment `wave` and output fragment `wave` of every stage
    const uint32_t ld_tile = lane >> 5, ld_row = (lane & 31u) >> 1;
    const uint32_t ld_off = ld_tile * kTileBytes + (lane & 1u) * 16;
    const uint8_t* src_x;
    const uint8_t* src_w;
    {
        uint32_t idx = (bm0 + wave) * kTile + ld_row;
        if (idx >= total_rows) idx = 0;            // valid memory; its results are not stored
        const uint32_t p = idx / a.R, r = idx - p * a.R;
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint32_t srow = a.s + r;
        src_x = a.x + plane[0] * a.x_plane_bytes + (uint64_t)(srow >> 4) * a.x_tile_cols * kTileBytes
                + (srow & 15u) * kRowBytes + ld_off;
        uint32_t o = (bn0 + wave) * kTile + ld_row;
        if (o >= a.O) o = 0;
        src_w = a.w + (uint64_t)(o >> 4) * a.w_tile_cols * kTileBytes + (o & 15u) * kRowBytes + ld_off;
    }
    // this group's stages: [s_lo, s_hi) of the I / 32; every group runs `per` iterations
    const uint32_t stages = a.I / 32, per = (stages + KS - 1) / KS;
    const uint32_t s_lo = slice * per < stages ? slice * per : stages;
    const uint32_t s_hi = s_lo + per < stages ? s_lo + per : stages;
    const uint32_t last = s_hi > s_lo ? s_hi - 1 : 0;
    auto issue = [&](uint32_t stage, uint32_t buf) {
        const uint64_t goff = (uint64_t)(stage < s_hi ? stage : last) * kFrag;
        uint8_t* base = lds + buf * kStageBytes;
        __builtin_amdgcn_global_load_lds((gptr_t)(src_x + goff), (lptr_t)(base + wave * kFrag), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr_t)(src_w + goff), (lptr_t)(base + (BM + wave) * kFrag), 16, 0, 0);
    };
    f32x4_t acc[2][2];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n) acc[m][n] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    const uint32_t rd_off = (kg >> 1) * kTileBytes + l16 * kRowBytes + (kg & 1u) * 16;
    auto rd = [&](uint32_t ring, uint32_t frag) {
        return __builtin_bit_cast(bf16x8_t,
                *reinterpret_cast<const u32x4*>(lds + ring * kStageBytes + rd_off + frag * kFrag));
    };
#pragma unroll
    for (uint32_t d = 0; d < DEPTH - 1; ++d) issue(s_lo + d, d);
    uint32_t ring = 0, free_ring = DEPTH - 1;
    for (uint32_t st = s_lo; st < s_lo + per; ++st) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 2) * LPS) : "memory");
        __builtin_amdgcn_s_barrier();
        issue(st + DEPTH - 1, free_ring);
        if (KS == 1 || st < s_hi) {                        // (the last group may have fewer stages)
            const bf16x8_t x0 = rd(ring, wm * 2), x1 = rd(ring, wm * 2 + 1);
            const bf16x8_t w0 = rd(ring, BM + wn * 2), w1 = rd(ring, BM + wn * 2 + 1);
            acc[0][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, x0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, x0, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, x1, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, x1, acc[1][1], 0, 0, 0);
        }
        free_ring = ring;
        ring = ring + 1 == DEPTH ? 0 : ring + 1;
    }
    // nothing may still be landing in LDS when the workgroup gives it back
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (KS > 1) {
        // the groups' partial sums through the (now idle) rings: [group - 1][wave][tile][lane]
        __syncthreads();
        f32x4_t* part = reinterpret_cast<f32x4_t*>(all_rings);
        if (slice > 0) {
#pragma unroll
            for (int t = 0; t < 4; ++t) part[(((slice - 1) * NW + wave) * 4 + t) * 64 + lane] = acc[t >> 1][t & 1];
        }
        __syncthreads();
        if (slice > 0) return;
#pragma unroll 1
        for (uint32_t g = 0; g + 1 < KS; ++g)
#pragma unroll
            for (int t = 0; t < 4; ++t) acc[t >> 1][t & 1] += part[((g * NW + wave) * 4 + t) * 64 + lane];
    }

    const uint32_t d_tiles = a.D >> 4;
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        const uint32_t idx = (bm0 + wm * 2 + m) * kTile + l16;
        if (idx >= total_rows) continue;
        const uint32_t p = idx / a.R, r = idx - p * a.R;
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        uint8_t* orow = a.out + plane[1] * a.out_plane_bytes
                + (uint64_t)(r >> 4) * a.out_tile_cols * kTileBytes + (r & 15u) * kRowBytes;
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            const uint32_t ot = bn0 + wn * 2 + n;
            if (ot * kTile >= a.O) continue;
            const uint32_t h = ot / d_tiles, dt = ot - h * d_tiles;
            *reinterpret_cast<u32x2*>(orow + (uint64_t)h * a.head_stride * a.out_plane_bytes
                                      + (uint64_t)dt * kTileBytes + kg * 8) =
                    u32x2{pack_bf16(acc[m][n][0], acc[m][n][1]), pack_bf16(acc[m][n][2], acc[m][n][3])};
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

    if (dtype == DT_BF16 && path != 1) {
        const uint64_t total_rows = (uint64_t)a.planes * a.R;
        const uint32_t o_tiles = (a.O + kTile - 1) / kTile;
        if (total_rows <= 0x7FFFFFFFull && o_tiles <= 65535u * 8u) {
            const uint32_t row_tiles = (uint32_t)((total_rows + kTile - 1) / kTile);
            if (path != 2 && row_tiles >= 8 && (a.I % 32) == 0 && (a.D & 15u) == 0) {
                // enough rows for workgroup tiles: operands staged through LDS.  256 x 256
                // outputs per workgroup (one workgroup per CU) when those fill at least
                // 65 % of the CU slots of the rounds they take, 128 x 128 (two per CU)
                // otherwise; 64 x 64 (four or five per CU) when there is not even one
                // 128 x 128 block per CU
                const uint64_t big = (uint64_t)((row_tiles + 15) / 16) * ((o_tiles + 15) / 16);
                const uint64_t mid = (uint64_t)((row_tiles + 7) / 8) * ((o_tiles + 7) / 8);
                const uint64_t rounds = (big + 255) / 256;
                uint32_t bt = big * 100 >= rounds * 256 * 65 ? 16 : mid >= 256 ? 8 : 4;
                if (path == 3 && row_tiles >= 16) bt = 16;
                if (path == 4) bt = 8;
                if (path == 5) bt = 4;
                // output tiles [first, first + count) with workgroup tiles of bt x bt 16x16 tiles
                // 130 to 256 blocks of 128 x 128 are one round in which each CU has a single workgroup
                // and the launch lasts as long as that workgroup's chain of stages: two groups of
                // waves then each take half of the inner axis (measured at 384-640 rows x
                // [4096..8192, 2048 or 4096]: 12-38 % faster than the 64 x 64 blocks, e.g. 512 rows x
                // [5632,2048] 21.4 -> 17.5 us, 640 rows x [5632,4096] 50.7 -> 31.8 us; with 128
                // blocks or fewer the 64 x 64 blocks with their own groups stay ahead)
                uint32_t groups = 1;
                const bool halves = (a.I / 32) % 2 == 0 && a.I >= 128;
                if (halves && (path == 6 || (path == 0 && bt != 16 && mid >= 130 && mid <= 256 && a.I >= 1024))) {
                    bt = 8;
                    groups = 2;
                }
                auto launch_part = [&](uint32_t first, uint32_t count, uint32_t tile) -> int {
                    LinearArgs b = a;
                    b.out_tile0 = first;
                    b.row_blocks = (row_tiles + tile - 1) / tile;
                    b.out_blocks = (count + tile - 1) / tile;
                    const uint64_t blocks = (uint64_t)b.row_blocks * b.out_blocks;
                    if (blocks > 0x7FFFFFF0ull) return IOMX_ERR_OVERFLOW;
                    b.blocks_per_xcd = (uint32_t)((blocks + 7) / 8);
                    const uint64_t wgs = (uint64_t)b.blocks_per_xcd * 8;
                    const dim3 grid((uint32_t)wgs);
                    uint32_t threads = 256;
                    if (tile == 16) {
                        threads = 512;
                        hipLaunchKernelGGL((linear_mfma_lds_bf16_kernel<8, 2, 4, 4>), grid, dim3(512), 0, st, b);
                    } else if (tile == 8 && groups == 2) {
                        threads = 512;
                        hipLaunchKernelGGL((linear_mfma_lds_bf16_kernel<4, 2, 2, 4, 2>), grid, dim3(512), 0, st, b);
                    } else if (tile == 8) {
                        hipLaunchKernelGGL((linear_mfma_lds_bf16_kernel<4, 2, 2, 5>), grid, dim3(256), 0, st, b);
                    } else {
                        // fewer blocks than CUs: two or four groups of waves share the inner axis
                        const uint32_t stages = a.I / 32;
                        // (measured at 512 rows: [2048,5632] 26 -> 20 us and [2048,2048] 12 -> 10 us with
                        // four groups instead of two; 256 rows x [5632,2048], 352 blocks, 14 -> 13 us with two)
                        const uint32_t ks = path == 5 ? 1
                                : (blocks <= 128 && stages >= 32) || (blocks <= 256 && stages >= 64) ? 4
                                : (blocks <= 256 && stages >= 16) || (blocks <= 384 && stages >= 32) ? 2 : 1;
                        threads = 256 * ks;
                        if (ks == 4) hipLaunchKernelGGL((linear_mfma_lds64_bf16_kernel<4, 4>), grid, dim3(1024), 0, st, b);
                        else if (ks == 2) hipLaunchKernelGGL((linear_mfma_lds64_bf16_kernel<4, 2>), grid, dim3(512), 0, st, b);
                        else hipLaunchKernelGGL((linear_mfma_lds64_bf16_kernel<4, 1>), grid, dim3(256), 0, st, b);
                    }
                    record_launch("linear_mfma_lds", grid.x, threads, (uint64_t)row_tiles * count);
                    return IOMX_OK;
                };
                // 256 x 256 blocks that fill whole rounds of the 256 CUs, and the rest of the
                // output range with smaller tiles in a second launch, when the last round of the
                // large tiles would run on few CUs (say 352 blocks: 256 + 96 -> 256 large blocks,
                // then 384 blocks of 128 x 128 at half the duration)
                const uint32_t rb16 = (row_tiles + 15) / 16, ob16 = (o_tiles + 15) / 16;
                const uint32_t ob_whole = (uint32_t)((big / 256) * 256 / rb16);
                if (path == 0 && bt == 16 && big > 256 && big * 100 < rounds * 256 * 85
                    && ob_whole >= 1 && ob_whole < ob16 && (uint64_t)ob_whole * rb16 * 100 >= (big / 256) * 256 * 90) {
                    const uint32_t rest = o_tiles - ob_whole * 16;
                    const uint64_t rest_mid = (uint64_t)((row_tiles + 7) / 8) * ((rest + 7) / 8);
                    IOMX_TRY(launch_part(0, ob_whole * 16, 16));
                    IOMX_TRY(launch_part(ob_whole * 16, rest, rest_mid >= 256 ? 8 : 4));
                } else {
                    IOMX_TRY(launch_part(0, o_tiles, bt));
                }
            } else if (path != 2 && row_tiles < 16 && o_tiles <= 0x3FFFFFu) {
                // few rows (decode, last-row logits): one output tile per workgroup, the
                // inner axis split over its waves
                // rows that are alone in their plane (R == 1 of many planes) make x the
                // expensive operand: then one row tile against four output tiles;
                // otherwise up to four row tiles against one or two
                const bool sparse_rows = a.R < kTile && a.planes > 1;
                uint32_t mt, nt;
                if (sparse_rows) {
                    // ... as long as that still leaves a workgroup for every CU
                    mt = 1;
                    nt = 4;
                    while (nt > 1 && (uint64_t)((o_tiles + nt - 1) / nt) * row_tiles < 256) nt /= 2;
                } else {
                    mt = row_tiles == 1 ? 1 : row_tiles == 2 ? 2 : 4;
                    nt = mt == 1 && (o_tiles + 1) / 2 >= 256 ? 2 : 1;      // a workgroup for every CU first
                }
                // two to four row tiles (a decode step of 17-64 sequences) against many
                // outputs: larger workgroup tiles, where enough of them remain for the CUs
                // (measured: 64 rows x [5632,2048] 18 -> 15 us, x [4096,4096] 30 -> 22 us,
                // x [32000,2048] 97 -> 43 us)
                if (row_tiles >= 3 && row_tiles <= 4) {
                    if (o_tiles >= 640 && (uint64_t)o_tiles * a.I >= 2500000u) { mt = 4; nt = 4; }
                    else if (o_tiles >= 352) { mt = 2; nt = 4; }
                    else if (o_tiles >= 256) { mt = 2; nt = 2; }
                } else if (row_tiles == 2 && o_tiles >= 1024) {
                    mt = 2; nt = 4;
                }
                LinearArgs b = a;
                b.row_blocks = (row_tiles + mt - 1) / mt;
                b.out_blocks = (uint32_t)((o_tiles + nt - 1) / nt);
                const dim3 grid((b.out_blocks + 7) / 8 * 8 * b.row_blocks);
                const bool two_sets = grid.x <= 256 && !(mt == 4 && nt == 4);
#define IOMX_SPLITK(M, N) \
    if (mt == M && nt == N) { \
        if (two_sets) hipLaunchKernelGGL((linear_mfma_splitk_bf16_kernel<M, N, 2>), grid, dim3(256), 0, st, b); \
        else hipLaunchKernelGGL((linear_mfma_splitk_bf16_kernel<M, N, 1>), grid, dim3(256), 0, st, b); \
    }
                IOMX_SPLITK(1, 1); IOMX_SPLITK(1, 2); IOMX_SPLITK(1, 4); IOMX_SPLITK(2, 1); IOMX_SPLITK(4, 1);
                IOMX_SPLITK(2, 2); IOMX_SPLITK(2, 4); IOMX_SPLITK(4, 4);
#undef IOMX_SPLITK
                record_launch("linear_mfma_splitk", grid.x, 256, (uint64_t)row_tiles * o_tiles);
            } else if (row_tiles <= 4) {
                const dim3 grid((row_tiles + 1) / 2, (o_tiles + 15) / 16);
                hipLaunchKernelGGL((linear_mfma_bf16_kernel<1, 8>), grid, dim3(256), 0, st, a);
                record_launch("linear_mfma", grid.x * grid.y, 256, (uint64_t)row_tiles * o_tiles);
            } else {
                const dim3 grid((row_tiles + 7) / 8, (o_tiles + 7) / 8);
                hipLaunchKernelGGL((linear_mfma_bf16_kernel<4, 4>), grid, dim3(256), 0, st, a);
                record_launch("linear_mfma", grid.x * grid.y, 256, (uint64_t)row_tiles * o_tiles);
            }
            IOMX_HIP(hipGetLastError());
            return IOMX_OK;
        }
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
