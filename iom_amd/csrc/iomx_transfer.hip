// Host-transfer staging kernels: dense logical row-major data of a view's shape
// (in device memory) <-> the view's 16x16-tiled planes.  One lane moves one
// 16-byte piece of one logical row; a row of tiles is 32 or 64 bytes contiguous
// on both sides, so both sides coalesce per piece.  Also the BF16 conversion
// self test.
#include "iomx_leaves.hpp"

namespace iomx {

struct TransferArgs {
    uint8_t* tiled;
    uint8_t* logical;
    PlaneWalk<1> walk;
    uint64_t plane_elems;
    uint64_t rows, cols, tile_cols;
    uint64_t pieces_per_row;
    uint64_t total_pieces;
    uint32_t vector_ok;  // logical rows are 16-byte aligned
};

template <int BYTES, bool SCATTER>
__global__ __launch_bounds__(256) void transfer_kernel(const TransferArgs a) {
    constexpr uint32_t kPer = 16 / BYTES;
    for (uint64_t g = blockIdx.x * 256ull + threadIdx.x; g < a.total_pieces;
         g += (uint64_t)gridDim.x * 256) {
        const uint64_t piece = g % a.pieces_per_row;
        const uint64_t rowlin = g / a.pieces_per_row;
        const uint64_t row = rowlin % a.rows;
        const uint32_t p = (uint32_t)(rowlin / a.rows);
        const uint64_t col0 = piece * kPer;
        if (col0 >= a.cols) continue;
        const uint32_t valid = (a.cols - col0) < kPer ? (uint32_t)(a.cols - col0) : kPer;
        uint64_t plane[1];
        walk_planes(a.walk, p, plane);
        const uint64_t slot = plane[0] * a.plane_elems
                + ((row / kTile) * a.tile_cols + col0 / kTile) * kTileSlots
                + (row % kTile) * kTile + col0 % kTile;
        uint8_t* t = a.tiled + slot * BYTES;
        uint8_t* l = a.logical + (rowlin * a.cols + col0) * BYTES;
        if (valid == kPer && a.vector_ok) {
            if (SCATTER) *reinterpret_cast<u32x4*>(t) = *reinterpret_cast<const u32x4*>(l);
            else *reinterpret_cast<u32x4*>(l) = *reinterpret_cast<const u32x4*>(t);
        } else {
            for (uint32_t e = 0; e < valid; ++e) {
                if constexpr (BYTES == 2) {
                    if (SCATTER) reinterpret_cast<uint16_t*>(t)[e] = reinterpret_cast<const uint16_t*>(l)[e];
                    else reinterpret_cast<uint16_t*>(l)[e] = reinterpret_cast<const uint16_t*>(t)[e];
                } else {
                    if (SCATTER) reinterpret_cast<uint32_t*>(t)[e] = reinterpret_cast<const uint32_t*>(l)[e];
                    else reinterpret_cast<uint32_t*>(l)[e] = reinterpret_cast<const uint32_t*>(t)[e];
                }
            }
        }
    }
}

namespace {

int run_transfer(int dtype, const iomx_view* view, const void* logical, bool scatter,
                 iomx_stream_t stream) {
    const uint32_t bits = leaf_bits(dtype);
    if (!bits) return IOMX_ERR_UNSUPPORTED;
    IOMX_TRY(check_view(view, bits));
    if (!logical) return IOMX_ERR_INVALID;
    if (bits != 16 && bits != 32) {
        // every other width moves through the packed bit stream
        IOMX_TRY(launch_bit_transfer(dtype, view, const_cast<void*>(logical), scatter, native(stream)));
        IOMX_HIP(hipGetLastError());
        return IOMX_OK;
    }
    const uint32_t bytes = bits / 8;
    const Matrix m = matrix_of(*view);
    TransferArgs a = {};
    uint64_t strides[1][kMaxLead] = {};
    uint64_t offsets[1] = {view->plane_offset};
    for (uint32_t i = 0; i + 2 < view->rank; ++i) strides[0][i] = view->plane_strides[i];
    IOMX_TRY(build_walk<1>(view->rank - 2, view->dims, strides, offsets, &a.walk));
    a.tiled = static_cast<uint8_t*>(view->base);
    a.logical = static_cast<uint8_t*>(const_cast<void*>(logical));
    a.plane_elems = m.plane_elems;
    a.rows = m.rows;
    a.cols = m.cols;
    a.tile_cols = m.tile_cols;
    a.pieces_per_row = m.tile_cols * (kTile * bytes / 16);
    uint64_t t;
    if (mul_overflows(a.walk.planes, m.rows, &t)) return IOMX_ERR_OVERFLOW;
    if (mul_overflows(t, a.pieces_per_row, &a.total_pieces)) return IOMX_ERR_OVERFLOW;
    a.vector_ok = ((m.cols * bytes) % 16 == 0)
            && (reinterpret_cast<uintptr_t>(logical) & 15u) == 0;
    const uint64_t blocks = (a.total_pieces + 255) / 256;
    const uint32_t grid = (uint32_t)(blocks < (1u << 20) ? blocks : (1u << 20));
    const hipStream_t s = native(stream);
    if (bytes == 2) {
        if (scatter) hipLaunchKernelGGL((transfer_kernel<2, true>), dim3(grid), dim3(256), 0, s, a);
        else hipLaunchKernelGGL((transfer_kernel<2, false>), dim3(grid), dim3(256), 0, s, a);
    } else {
        if (scatter) hipLaunchKernelGGL((transfer_kernel<4, true>), dim3(grid), dim3(256), 0, s, a);
        else hipLaunchKernelGGL((transfer_kernel<4, false>), dim3(grid), dim3(256), 0, s, a);
    }
    record_launch(scatter ? "scatter" : "gather", grid, 256, a.total_pieces);
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}

}  // namespace
}  // namespace iomx

using namespace iomx;

extern "C" {

int iomx_launch_scatter(int dtype, const iomx_view* dst, const void* logical, iomx_stream_t stream) {
    return run_transfer(dtype, dst, logical, true, stream);
}

int iomx_launch_gather(int dtype, const iomx_view* src, void* logical, iomx_stream_t stream) {
    return run_transfer(dtype, src, logical, false, stream);
}

}  // extern "C"
