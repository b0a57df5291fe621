// Operand types and loads shared by the BF16 matrix-core kernels
// (v_mfma_f32_16x16x32_bf16: lane l supplies eight consecutive inner elements
// 8*(l/16).. of operand row l%16 and receives D[4*(l/16)+j][l%16], j < 4).
#pragma once
#include "iomx_common.hpp"

namespace iomx {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
// operands of the direct global -> LDS loader (global_load_lds: 16 bytes a lane, lane i's
// piece lands at the LDS address + 16*i)
typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// Eight consecutive BF16 of one tile row starting at column c0 (0 or 8), inner
// indices i0..i0+7, zero where the inner index is past I (tile padding is never
// an operand and is not read).
__device__ __forceinline__ u32x4 load_k8_bits(const uint8_t* tile_row, uint32_t c0, uint32_t i0, uint32_t I) {
    u32x4 v = {0, 0, 0, 0};
    if (i0 + 8 <= I) {
        v = *reinterpret_cast<const u32x4*>(tile_row + c0 * 2);
    } else if (i0 < I) {
        uint32_t h[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            h[j] = (i0 + j < I) ? *reinterpret_cast<const uint16_t*>(tile_row + (c0 + j) * 2) : 0u;
        v = u32x4{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
    }
    return v;
}

__device__ __forceinline__ bf16x8_t load_k8(const uint8_t* tile_row, uint32_t c0, uint32_t i0, uint32_t I) {
    return __builtin_bit_cast(bf16x8_t, load_k8_bits(tile_row, c0, i0, I));
}

}  // namespace iomx
