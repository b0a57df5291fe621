// RMSNorm over the rows of tiled [..., R, F] views, binary32 accumulation.
//
// In the 16x16-tiled layout one tile-row band (16 logical rows x F features)
// is one contiguous range, and inside it a wave that reads 64 consecutive
// 128-bit chunks always sees the same logical row in the same lane.  So a
// workgroup owns one band at a time, streams it once with fully coalesced
// loads, keeps it in registers, reduces per lane, combines the lanes of a row
// inside the wave and the waves through LDS, then scales the registers and
// stores: HBM sees x once and out once.
//
//   rmsnorm_band     F a multiple of 16 and a band that fits the register
//                    budget (at most 16 chunks per lane of a 1024-lane workgroup).
//   rmsnorm_generic  any F and any band size: two passes over the band, the
//                    second served by L2, with per-element column masks.
#include "iomx_leaves.hpp"

namespace iomx {

struct RmsArgs {
    const uint8_t* x;
    const uint8_t* scale;  // already advanced to the scale plane
    uint8_t* out;
    PlaneWalk<2> walk;     // 0 x, 1 out
    uint64_t plane_bytes;
    uint64_t band_bytes;
    uint32_t rows, feats;
    uint32_t tile_rows;
    uint32_t band_chunks;
    uint32_t total_bands;
    float eps;
};

template <int DT>
struct RLeaf {
    static constexpr uint32_t kBytes = (DT == IOMX_DT_BF16 || DT == IOMX_DT_F16) ? 2 : 4;
    static constexpr uint32_t kPerChunk = 16 / kBytes;
    static constexpr uint32_t kChunksPerRow = kTile / kPerChunk;     // 2 | 4
    static constexpr uint32_t kChunksPerTile = kTileSlots / kPerChunk; // 32 | 64
};

template <int DT>
__device__ __forceinline__ void unpack(const u32x4& v, float* f) {
    if constexpr (DT == IOMX_DT_BF16) {
        f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x); f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
        f[4] = bf16_lo(v.z); f[5] = bf16_hi(v.z); f[6] = bf16_lo(v.w); f[7] = bf16_hi(v.w);
    } else if constexpr (DT == IOMX_DT_F16) {
        const f32x2 a = f16_pair(v.x), b = f16_pair(v.y), c = f16_pair(v.z), d = f16_pair(v.w);
        f[0] = a.x; f[1] = a.y; f[2] = b.x; f[3] = b.y; f[4] = c.x; f[5] = c.y; f[6] = d.x; f[7] = d.y;
    } else {
        f[0] = as_f32(v.x); f[1] = as_f32(v.y); f[2] = as_f32(v.z); f[3] = as_f32(v.w);
    }
}

template <int DT>
__device__ __forceinline__ u32x4 pack(const float* f) {
    u32x4 r;
    if constexpr (DT == IOMX_DT_BF16) {
        r.x = pack_bf16(f[0], f[1]); r.y = pack_bf16(f[2], f[3]);
        r.z = pack_bf16(f[4], f[5]); r.w = pack_bf16(f[6], f[7]);
    } else if constexpr (DT == IOMX_DT_F16) {
        r.x = pack_f16(f[0], f[1]); r.y = pack_f16(f[2], f[3]);
        r.z = pack_f16(f[4], f[5]); r.w = pack_f16(f[6], f[7]);
    } else {
        r.x = as_u32(canonical(f[0])); r.y = as_u32(canonical(f[1]));
        r.z = as_u32(canonical(f[2])); r.w = as_u32(canonical(f[3]));
    }
    return r;
}

// Row of the band that lane `tid` sees in every chunk it loads, and the sum of
// the lanes of one wave that share a row.
template <int DT>
__device__ __forceinline__ uint32_t lane_row(uint32_t tid) {
    if constexpr (RLeaf<DT>::kBytes == 2) return (tid & 31u) >> 1;
    else return (tid & 63u) >> 2;
}

template <int DT>
__device__ __forceinline__ float row_sum_in_wave(float acc) {
    if constexpr (RLeaf<DT>::kBytes == 2) {
        acc += __shfl_xor(acc, 1);
        acc += __shfl_xor(acc, 32);
    } else {
        acc += __shfl_xor(acc, 1);
        acc += __shfl_xor(acc, 2);
    }
    return acc;
}

template <int DT>
__device__ __forceinline__ bool row_leader(uint32_t tid) {
    if constexpr (RLeaf<DT>::kBytes == 2) return (tid & 33u) == 0;
    else return (tid & 3u) == 0;
}

// inverse = 1 / sqrt(sum/F + eps), each step rounded to binary32
// (src/cpu/queue.cpp:1193-1196).
__device__ __forceinline__ float inverse_rms(float sum, uint32_t feats, float eps) {
    const float mean = sum / (float)feats;
    const float shifted = mean + eps;
    const float root = sqrtf(shifted);
    return 1.0f / root;
}

// The band kernel: one band per workgroup, K 128-bit chunks per lane held in
// registers between the two passes.  Whole-band loads and stores stream past
// the caches; the scale row stays cached.  Keeping the register count low keeps
// two 1024-lane workgroups resident per compute unit, so one band's loads
// overlap the other's arithmetic and stores.  (Variants measured and dropped on
// MI355X, [32768,2048]: a persistent workgroup that prefetches its next band
// into a second register set, the scale row decoded once into registers, sixteen
// lanes finishing the row totals for everyone, and a barrier-free kernel with
// four rows per wave, and two passes with the second read served by the caches:
// all slower, by 3-20 %.)
//
// The sum of squares uses a fused multiply-add per element (one rounding instead
// of the reference's two): the total differs from the sequential reference
// recurrence by a few units in the last place either way, far inside the bar.
template <int DT, int K, int THREADS>
__global__ __launch_bounds__(THREADS) void rmsnorm_band_kernel(const RmsArgs a) {
    using L = RLeaf<DT>;
    constexpr int kWaves = THREADS / 64;
    __shared__ __attribute__((aligned(16))) float partial[kTile][kWaves];
    const uint32_t tid = threadIdx.x;
    const uint32_t row = lane_row<DT>(tid);
    const uint32_t band = blockIdx.x;
    uint32_t p = 0, tr = band;
    if (a.walk.nlead != 0) {
        p = band / a.tile_rows;
        tr = band - p * a.tile_rows;
    }
    uint64_t plane[2];
    walk_planes(a.walk, p, plane);
    const uint8_t* xb = a.x + plane[0] * a.plane_bytes + (uint64_t)tr * a.band_bytes;
    uint8_t* ob = a.out + plane[1] * a.plane_bytes + (uint64_t)tr * a.band_bytes;
    u32x4 cur[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t c = tid + k * THREADS;
        cur[k] = u32x4{0, 0, 0, 0};
        if (c < a.band_chunks)
            cur[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xb + (uint64_t)c * 16));
    }
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        float f[L::kPerChunk];
        unpack<DT>(cur[k], f);
#pragma unroll
        for (uint32_t e = 0; e < L::kPerChunk; ++e) acc = __builtin_fmaf(f[e], f[e], acc);
    }
    acc = row_sum_in_wave<DT>(acc);
    float inverse;
    if constexpr (kWaves > 1) {
        if (row_leader<DT>(tid)) partial[row][tid / 64] = acc;
        __syncthreads();
        float total = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kWaves; ++wv) total = total + partial[row][wv];
        inverse = inverse_rms(total, a.feats, a.eps);
    } else {
        inverse = inverse_rms(acc, a.feats, a.eps);
    }
    if (tr * kTile + row >= a.rows) return;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t c = tid + k * THREADS;
        if (c < a.band_chunks) {
            const uint32_t soff = ((c / L::kChunksPerTile) * L::kChunksPerTile
                                   + (c % L::kChunksPerRow)) * 16;
            float f[L::kPerChunk], sc[L::kPerChunk];
            unpack<DT>(cur[k], f);
            unpack<DT>(*reinterpret_cast<const u32x4*>(a.scale + soff), sc);
#pragma unroll
            for (uint32_t e = 0; e < L::kPerChunk; ++e) {
                const float normalized = f[e] * inverse;
                f[e] = normalized * sc[e];
            }
            u32x4* dst = reinterpret_cast<u32x4*>(ob + (uint64_t)c * 16);
            __builtin_nontemporal_store(pack<DT>(f), dst);
        }
    }
}

// Wide rows: the band is cut into S parts of 16/S rows each, one workgroup per
// part, so that a workgroup still holds only K chunks per lane (two workgroups
// stay resident per compute unit) however large F is.  Inside a tile the rows
// of one part are one contiguous run of kChunksPerTile/S chunks; a lane's chunk
// index within its part maps to (tile, chunk in the run), and the lanes of a
// wave that share a row differ in the position inside the row piece (low bits)
// and in the tile (bits above the run).
template <int DT, int K, int S>
__global__ __launch_bounds__(1024) void rmsnorm_split_kernel(const RmsArgs a) {
    using L = RLeaf<DT>;
    constexpr int THREADS = 1024;
    constexpr int kWaves = THREADS / 64;
    constexpr uint32_t SUB = L::kChunksPerTile / S;   // chunks of one part in one tile
    constexpr uint32_t RP = kTile / S;                // rows of one part
    static_assert(SUB >= L::kChunksPerRow, "a part holds whole row pieces");
    __shared__ __attribute__((aligned(16))) float partial[RP][kWaves];
    const uint32_t tid = threadIdx.x;
    const uint32_t band = blockIdx.x / S, part = blockIdx.x % S;
    const uint32_t w = tid % SUB;
    const uint32_t row = w / L::kChunksPerRow;        // within the part
    uint32_t p = 0, tr = band;
    if (a.walk.nlead != 0) {
        p = band / a.tile_rows;
        tr = band - p * a.tile_rows;
    }
    uint64_t plane[2];
    walk_planes(a.walk, p, plane);
    const uint8_t* xb = a.x + plane[0] * a.plane_bytes + (uint64_t)tr * a.band_bytes;
    uint8_t* ob = a.out + plane[1] * a.plane_bytes + (uint64_t)tr * a.band_bytes;
    const uint32_t part_chunks = a.band_chunks / S;
    uint32_t chunk[K];
    u32x4 cur[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t c = tid + k * THREADS;
        chunk[k] = (c / SUB) * L::kChunksPerTile + part * SUB + w;
        cur[k] = u32x4{0, 0, 0, 0};
        if (c < part_chunks)
            cur[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xb + (uint64_t)chunk[k] * 16));
    }
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        float f[L::kPerChunk];
        unpack<DT>(cur[k], f);
#pragma unroll
        for (uint32_t e = 0; e < L::kPerChunk; ++e) acc = __builtin_fmaf(f[e], f[e], acc);
    }
    // lanes of the wave that hold the same row: every lane bit that is not a row bit
    uint32_t shared_bits = 0;
#pragma unroll
    for (uint32_t bit = 1; bit < 64; bit <<= 1) {
        if (bit < L::kChunksPerRow || bit >= SUB) {
            acc += __shfl_xor(acc, (int)bit);
            shared_bits |= bit;
        }
    }
    if ((tid & shared_bits) == 0) partial[row][tid / 64] = acc;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int wv = 0; wv < kWaves; ++wv) total = total + partial[row][wv];
    const float inverse = inverse_rms(total, a.feats, a.eps);
    if (tr * kTile + part * RP + row >= a.rows) return;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (tid + k * THREADS < part_chunks) {
            const uint32_t c = chunk[k];
            const uint32_t soff = ((c / L::kChunksPerTile) * L::kChunksPerTile
                                   + (c % L::kChunksPerRow)) * 16;
            float f[L::kPerChunk], sc[L::kPerChunk];
            unpack<DT>(cur[k], f);
            unpack<DT>(*reinterpret_cast<const u32x4*>(a.scale + soff), sc);
#pragma unroll
            for (uint32_t e = 0; e < L::kPerChunk; ++e) {
                const float normalized = f[e] * inverse;
                f[e] = normalized * sc[e];
            }
            __builtin_nontemporal_store(pack<DT>(f), reinterpret_cast<u32x4*>(ob + (uint64_t)c * 16));
        }
    }
}

template <int DT>
__global__ __launch_bounds__(256) void rmsnorm_generic_kernel(const RmsArgs a) {
    using L = RLeaf<DT>;
    constexpr int THREADS = 256;
    constexpr int kWaves = THREADS / 64;
    __shared__ float partial[kWaves][kTile];
    const uint32_t tid = threadIdx.x;
    const uint32_t row = lane_row<DT>(tid);
    for (uint32_t band = blockIdx.x; band < a.total_bands; band += gridDim.x) {
        const uint32_t p = band / a.tile_rows;
        const uint32_t tr = band - p * a.tile_rows;
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint8_t* xb = a.x + plane[0] * a.plane_bytes + (uint64_t)tr * a.band_bytes;
        uint8_t* ob = a.out + plane[1] * a.plane_bytes + (uint64_t)tr * a.band_bytes;
        float acc = 0.0f;
        for (uint32_t c = tid; c < a.band_chunks; c += THREADS) {
            const uint32_t col0 = (c / L::kChunksPerTile) * kTile + (c % L::kChunksPerRow) * L::kPerChunk;
            const u32x4 v = *reinterpret_cast<const u32x4*>(xb + (uint64_t)c * 16);
            float f[L::kPerChunk];
            unpack<DT>(v, f);
#pragma unroll
            for (uint32_t e = 0; e < L::kPerChunk; ++e)
                if (col0 + e < a.feats) acc = acc + f[e] * f[e];
        }
        acc = row_sum_in_wave<DT>(acc);
        if (row_leader<DT>(tid)) partial[tid / 64][row] = acc;
        __syncthreads();
        acc = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kWaves; ++wv) acc = acc + partial[wv][row];
        const float inverse = inverse_rms(acc, a.feats, a.eps);
        const bool live = tr * kTile + row < a.rows;
        for (uint32_t c = tid; c < a.band_chunks && live; c += THREADS) {
            const uint32_t col0 = (c / L::kChunksPerTile) * kTile + (c % L::kChunksPerRow) * L::kPerChunk;
            if (col0 >= a.feats) continue;
            const uint32_t soff = ((c / L::kChunksPerTile) * L::kChunksPerTile
                                   + (c % L::kChunksPerRow)) * 16;
            const u32x4 v = *reinterpret_cast<const u32x4*>(xb + (uint64_t)c * 16);
            const u32x4 wk = *reinterpret_cast<const u32x4*>(a.scale + soff);
            float f[L::kPerChunk], s[L::kPerChunk];
            unpack<DT>(v, f);
            unpack<DT>(wk, s);
#pragma unroll
            for (uint32_t e = 0; e < L::kPerChunk; ++e) {
                const float normalized = f[e] * inverse;
                f[e] = normalized * s[e];
            }
            const u32x4 r = pack<DT>(f);
            uint8_t* dst = ob + (uint64_t)c * 16;
            const uint32_t valid = a.feats - col0;
            if (valid >= L::kPerChunk) {
                *reinterpret_cast<u32x4*>(dst) = r;
            } else {
                const uint32_t words[4] = {r.x, r.y, r.z, r.w};
                for (uint32_t e = 0; e < valid; ++e) {
                    if constexpr (L::kBytes == 2)
                        reinterpret_cast<uint16_t*>(dst)[e] = (uint16_t)(words[e >> 1] >> ((e & 1) * 16));
                    else
                        reinterpret_cast<uint32_t*>(dst)[e] = words[e];
                }
            }
        }
        __syncthreads();
    }
}

namespace {

template <int DT, int K, int THREADS>
void launch_band(const RmsArgs& a, hipStream_t s) {
    hipLaunchKernelGGL((rmsnorm_band_kernel<DT, K, THREADS>), dim3(a.total_bands), dim3(THREADS), 0,
                       s, a);
    record_launch("rmsnorm_band", a.total_bands, THREADS, a.total_bands);
}

template <int DT, int K, int S>
void launch_split(const RmsArgs& a, hipStream_t s) {
    hipLaunchKernelGGL((rmsnorm_split_kernel<DT, K, S>), dim3(a.total_bands * S), dim3(1024), 0, s, a);
    record_launch("rmsnorm_split", a.total_bands * S, 1024, (uint64_t)a.total_bands * S);
}

// Chunks one 1024-lane workgroup can hold in registers without spilling: K = 8 per
// lane for BF16 (whose unpacked chunk is eight floats), 16 for F32.  Measured on
// MI355X with rows of 4096..16384 features: the fewest, largest parts win (runs of
// 256 bytes or more per tile), and sixteen parts (32-byte runs) lose even to the
// two-pass kernel, so the split stops at eight.
template <int DT>
constexpr uint32_t kResidentChunks = (RLeaf<DT>::kBytes == 2 ? 8u : 16u) * 1024u;

template <int DT>
int launch(const RmsArgs& a, bool band_ok, hipStream_t s) {
    const uint32_t n = a.band_chunks;
    constexpr int KS = RLeaf<DT>::kBytes == 2 ? 8 : 16;
    if (band_ok && n > kResidentChunks<DT> && n <= 8 * kResidentChunks<DT>
        && (uint64_t)a.total_bands * 8 <= 0x7FFFFFFFull) {
        if (n <= 2 * kResidentChunks<DT>) launch_split<DT, KS, 2>(a, s);
        else if (n <= 4 * kResidentChunks<DT>) launch_split<DT, KS, 4>(a, s);
        else launch_split<DT, KS, 8>(a, s);
        return IOMX_OK;
    }
    if (!band_ok || n > kResidentChunks<DT> || a.total_bands > 0x7FFFFFFFu) {
        const uint32_t cap = 1u << 20;
        const uint32_t grid = a.total_bands < cap ? a.total_bands : cap;
        hipLaunchKernelGGL((rmsnorm_generic_kernel<DT>), dim3(grid), dim3(256), 0, s, a);
        record_launch("rmsnorm_generic", grid, 256, a.total_bands);
    } else if (n <= 64) launch_band<DT, 1, 64>(a, s);
    else if (n <= 256) launch_band<DT, 1, 256>(a, s);
    else if (n <= 512) launch_band<DT, 1, 512>(a, s);
    else if (n <= 1024) launch_band<DT, 1, 1024>(a, s);
    else if (n <= 2048) launch_band<DT, 2, 1024>(a, s);
    else if (n <= 4096) launch_band<DT, 4, 1024>(a, s);
    else if (n <= 8192) launch_band<DT, 8, 1024>(a, s);
    else if constexpr (RLeaf<DT>::kBytes != 2) launch_band<DT, 16, 1024>(a, s);
    else return IOMX_ERR_INVALID;          // unreachable: BF16 bands this wide are split above
    return IOMX_OK;
}

}  // namespace
}  // namespace iomx

using namespace iomx;

// Admission of src/device_ops_rmsnorm.cpp:75-127 (everything that can be
// checked without owner identities).
extern "C" int iomx_launch_rmsnorm(int dtype, const iomx_view* x, const iomx_view* scale,
                                   const iomx_view* out, float eps, iomx_stream_t stream) {
    const uint32_t bits = leaf_bits(dtype);
    if (!bits) return IOMX_ERR_UNSUPPORTED;
    const uint32_t bytes = bits / 8;
    IOMX_TRY(check_view(x, bits));
    IOMX_TRY(check_view(scale, bits));
    IOMX_TRY(check_view(out, bits));
    if (x->rank != out->rank) return IOMX_ERR_INVALID;
    for (uint32_t i = 0; i < x->rank; ++i) if (x->dims[i] != out->dims[i]) return IOMX_ERR_INVALID;
    const Matrix m = matrix_of(*x);
    if (scale->rank != 2 || scale->dims[0] != 1 || scale->dims[1] != m.cols) return IOMX_ERR_INVALID;
    if (out->base == x->base || out->base == scale->base) return IOMX_ERR_INVALID;
    if (!(eps >= 0.0f) || eps > 3.4028234e38f) return IOMX_ERR_INVALID;
    if (dtype != IOMX_DT_BF16 && dtype != IOMX_DT_F32 && dtype != IOMX_DT_F16) {
        // the other floating leaves: one workgroup per row on packed tile rows
        RowsRmsnormRequest r = {};
        uint64_t rstrides[2][kMaxLead] = {};
        uint64_t roffsets[2] = {x->plane_offset, out->plane_offset};
        for (uint32_t i = 0; i + 2 < x->rank; ++i) {
            rstrides[0][i] = x->plane_strides[i];
            rstrides[1][i] = out->plane_strides[i];
        }
        IOMX_TRY(build_walk<2>(x->rank - 2, x->dims, rstrides, roffsets, &r.walk));
        r.x = static_cast<const uint8_t*>(x->base);
        r.out = static_cast<uint8_t*>(out->base);
        r.scale = static_cast<const uint8_t*>(scale->base)
                + scale->plane_offset * matrix_of(*scale).plane_elems * bits / 8;
        r.m = m;
        r.eps = eps;
        IOMX_TRY(launch_rows_rmsnorm(dtype, r, native(stream)));
        IOMX_HIP(hipGetLastError());
        return IOMX_OK;
    }

    RmsArgs a = {};
    uint64_t strides[2][kMaxLead] = {};
    uint64_t offsets[2] = {x->plane_offset, out->plane_offset};
    for (uint32_t i = 0; i + 2 < x->rank; ++i) {
        strides[0][i] = x->plane_strides[i];
        strides[1][i] = out->plane_strides[i];
    }
    IOMX_TRY(build_walk<2>(x->rank - 2, x->dims, strides, offsets, &a.walk));
    const uint64_t band_chunks = m.tile_cols * (kTileSlots * bytes / 16);
    uint64_t total_bands;
    if (mul_overflows(a.walk.planes, m.tile_rows, &total_bands)) return IOMX_ERR_OVERFLOW;
    if (total_bands > 0xFFFFFFFFull || band_chunks > 0x0FFFFFFFull || m.rows > 0xFFFFFFFFull
        || m.cols > 0xFFFFFFFFull)
        return IOMX_ERR_OVERFLOW;
    a.x = static_cast<const uint8_t*>(x->base);
    a.out = static_cast<uint8_t*>(out->base);
    const Matrix sm = matrix_of(*scale);
    a.scale = static_cast<const uint8_t*>(scale->base) + scale->plane_offset * sm.plane_elems * bytes;
    a.plane_bytes = m.plane_elems * bytes;
    a.band_bytes = band_chunks * 16;
    a.rows = (uint32_t)m.rows;
    a.feats = (uint32_t)m.cols;
    a.tile_rows = (uint32_t)m.tile_rows;
    a.band_chunks = (uint32_t)band_chunks;
    a.total_bands = (uint32_t)total_bands;
    a.eps = eps;
    // Dense selections of whole bands fold all planes into one run of bands.
    if (a.walk.nlead <= 1 && walk_is_dense(a.walk, 0) && walk_is_dense(a.walk, 1)
        && m.rows % kTile == 0 && total_bands * kTile <= 0xFFFFFFFFull) {
        a.x += a.walk.offset[0] * a.plane_bytes;
        a.out += a.walk.offset[1] * a.plane_bytes;
        a.walk.offset[0] = a.walk.offset[1] = 0;
        a.walk.nlead = 0;
        a.tile_rows = (uint32_t)total_bands;
        a.rows = (uint32_t)(total_bands * kTile);
    }
    const bool band_ok = m.cols % kTile == 0;
    const hipStream_t s = native(stream);
    if (dtype == IOMX_DT_BF16) IOMX_TRY(launch<IOMX_DT_BF16>(a, band_ok, s));
    else if (dtype == IOMX_DT_F16) IOMX_TRY(launch<IOMX_DT_F16>(a, band_ok, s));
    else IOMX_TRY(launch<IOMX_DT_F32>(a, band_ok, s));
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}
