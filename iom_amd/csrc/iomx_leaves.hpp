// The every-leaf path of libiomx: requests the streaming kernels do not take
// (leaves other than I32 / U32 / F32 / BF16, and packed 2/4/6-bit storage) are
// served by kernels whose unit of work is one tile row: sixteen consecutive
// elements, 2*bits bytes, always a whole number of 32-bit words.
#pragma once

#include "iomx_common.hpp"

namespace iomx {

// Internal operation codes shared with the streaming kernels.
enum { ROWS_OP_SILU = 4, ROWS_OP_COPY = 5 };

struct RowsRequest {
    const uint8_t* src[2];
    uint8_t* out;
    PlaneWalk<3> walk;   // 0 lhs, 1 rhs, 2 out
    Matrix m[3];
    bool brow[2], bcol[2];
};

// op: IOMX_OP_ADD / MUL / SUB / DIV (DIV on floating leaves), ROWS_OP_SILU (one input), ROWS_OP_COPY (one input).
int launch_rows(int op, int dtype, const RowsRequest& r, hipStream_t stream);

struct RowsRmsnormRequest {
    const uint8_t* x;
    const uint8_t* scale;   // plane of the [1,F] vector
    uint8_t* out;
    PlaneWalk<2> walk;      // 0 x, 1 out
    Matrix m;
    float eps;
};

int launch_rows_rmsnorm(int dtype, const RowsRmsnormRequest& r, hipStream_t stream);

// Packed logical bit stream (32-bit words) <-> tiled view, any leaf width.
int launch_bit_transfer(int dtype, const iomx_view* view, void* stream_words, bool scatter,
                        hipStream_t stream);

}  // namespace iomx
