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
//   rmsnorm_band     F a multiple of 16: a band, or one of 2..8 row groups of it,
//                    resident in the registers of one workgroup.
//   rmsnorm_generic  any F and any band size: two passes over the band, the
//                    second served by L2, with per-element column masks.
#include "iomx_arith.hpp"

namespace iomx {

// N = 2: x and out.  N = 4 (residual add fused in front): x + y is stored to `sum` and normalised.
template <int N>
struct RmsArgsT {
    const uint8_t* x;
    const uint8_t* scale;  // already advanced to the scale plane
    uint8_t* out;
    const uint8_t* y;      // N = 4 only
    uint8_t* sum;          // N = 4 only
    PlaneWalk<N> walk;     // 0 x, 1 out, 2 y, 3 sum
    uint64_t plane_bytes;
    uint64_t band_bytes;
    uint32_t rows, feats;
    uint32_t tile_rows;
    uint32_t band_chunks;
    uint32_t total_bands;
    float eps;
};
using RmsArgs = RmsArgsT<2>;

constexpr bool is_f8(int dt) { return dt == IOMX_DT_F8_E4M3FN || dt == IOMX_DT_F8_E5M2; }

// (The two 8-bit floating leaves take the resident kernel as well: a 16-byte chunk is one tile
// row of sixteen elements, decoded and encoded by the conversion instructions of the tile-row
// kernels.)
template <int DT>
struct RLeaf {
    static constexpr uint32_t kBytes = is_f8(DT) ? 1 : (DT == IOMX_DT_BF16 || DT == IOMX_DT_F16) ? 2 : 4;
    static constexpr uint32_t kPerChunk = 16 / kBytes;
    static constexpr uint32_t kChunksPerRow = kTile / kPerChunk;     // 1 | 2 | 4
    static constexpr uint32_t kChunksPerTile = kTileSlots / kPerChunk; // 16 | 32 | 64
};

template <int DT>
__device__ __forceinline__ void unpack(const u32x4& v, float* f) {
    if constexpr (is_f8(DT)) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        float row[kTile];
        hw_decode_row<DT>(w, row);
#pragma unroll
        for (int i = 0; i < (int)kTile; ++i) f[i] = row[i];
    } else if constexpr (DT == IOMX_DT_BF16) {
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
    if constexpr (is_f8(DT)) {
        float row[kTile];
#pragma unroll
        for (int i = 0; i < (int)kTile; ++i) row[i] = f[i];
        uint32_t w[4];
        hw_encode_row<DT>(row, w);
        r = u32x4{w[0], w[1], w[2], w[3]};
    } else if constexpr (DT == IOMX_DT_BF16) {
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

// The resident kernel.  A band is cut into S parts of 16/S rows (S = 1: the whole
// band); one workgroup of THREADS lanes owns one part and holds its K 128-bit chunks per
// lane in registers between the two passes, so HBM sees x once and out once.  Inside a
// tile the rows of a part are one contiguous run of kChunksPerTile/S chunks; a lane's
// chunk index within its part maps to (tile, chunk in the run), the same lane always
// sees the same row, and the lanes of a wave that share a row differ in the position
// inside the row piece (low lane bits) and in the tile (bits above the run).
//
// What the order of the code is for (each point measured on MI355X at [32768,2048]):
//  * x and the scale row are requested together, before anything waits: a scale chunk
//    fetched after the barrier sits in the path between the last load and the first
//    store of a workgroup, and the compiler otherwise waits for each store's
//    acknowledgement before it fetches the next scale chunk (stores and loads share
//    one counter);
//  * the values unpacked for the sum of squares are not kept: the raw chunks are made
//    opaque after pass 1, so a lane holds 2*K*4 raw registers instead of K*8 decoded
//    ones plus the scale, and two 1024-lane workgroups stay resident per compute unit
//    (at most 64 registers) with K = 4;
//  * all results are formed first and stored back to back.
// FULL says that K*THREADS chunks cover a part exactly, which removes every bounds test.
// PRE is the early scale request: a lane has room for it with up to four chunks of a
// 2-byte leaf or eight of a 4-byte leaf (128 registers at most for 1024 lanes); without it
// the scale chunk is fetched where it is used.
//
// The sum of squares uses a fused multiply-add per element (one rounding instead of the
// reference's two): the total differs from the sequential reference recurrence by a few
// units in the last place either way, far inside the bar.
//
// ADD: the residual add fused in front.  A lane loads the chunks of x and y, forms x + y with the
// arithmetic of the ADD kernel (op_chunk: one IEEE addition per element, one rounding to the
// leaf), stores it to `sum` at once -- those stores are under way while the row totals meet at
// the barrier -- and normalises the rounded sum it holds.  Bit for bit the result of the ADD
// launch followed by the RMSNorm launch, with x + y crossing HBM once instead of three times.
template <int DT, int K, int S, int THREADS, bool FULL, bool PRE, bool ADD = false>
__global__ __launch_bounds__(THREADS) void rmsnorm_band_kernel(const RmsArgsT<ADD ? 4 : 2> a) {
    using L = RLeaf<DT>;
    constexpr int kWaves = THREADS / 64;
    constexpr uint32_t SUB = L::kChunksPerTile / S;   // chunks of one part in one tile
    constexpr uint32_t RP = kTile / S;                // rows of one part
    static_assert(SUB >= L::kChunksPerRow, "a part holds whole row pieces");
    static_assert(THREADS % 64 == 0 && (SUB >= 64 ? SUB % 64 == 0 : 64 % SUB == 0), "lane keeps its row");
    __shared__ __attribute__((aligned(16))) float partial[RP][kWaves];
    const uint32_t tid = threadIdx.x;
    const uint32_t band = S == 1 ? blockIdx.x : blockIdx.x / S;
    const uint32_t part = S == 1 ? 0u : blockIdx.x % S;
    const uint32_t w = tid % SUB;
    const uint32_t row = w / L::kChunksPerRow;        // within the part
    uint32_t p = 0, tr = band;
    if (a.walk.nlead != 0) {
        p = band / a.tile_rows;
        tr = band - p * a.tile_rows;
    }
    uint64_t plane[ADD ? 4 : 2];
    walk_planes(a.walk, p, plane);
    const uint8_t* xb = a.x + plane[0] * a.plane_bytes + (uint64_t)tr * a.band_bytes;
    uint8_t* ob = a.out + plane[1] * a.plane_bytes + (uint64_t)tr * a.band_bytes;
    const uint32_t part_chunks = a.band_chunks / S;
    uint32_t chunk[K];
    u32x4 cur[K], scl[PRE ? K : 1];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t c = tid + k * THREADS;
        chunk[k] = S == 1 ? c : (c / SUB) * L::kChunksPerTile + part * SUB + w;
        cur[k] = u32x4{0, 0, 0, 0};
        if (FULL || c < part_chunks)
            cur[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xb + (uint64_t)chunk[k] * 16));
    }
    if constexpr (ADD) {
        const uint8_t* yb = a.y + plane[2] * a.plane_bytes + (uint64_t)tr * a.band_bytes;
        uint8_t* sb = a.sum + plane[3] * a.plane_bytes + (uint64_t)tr * a.band_bytes;
        u32x4 other[K];
#pragma unroll
        for (int k = 0; k < K; ++k) {
            other[k] = u32x4{0, 0, 0, 0};
            if (FULL || tid + k * THREADS < part_chunks)
                other[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(yb + (uint64_t)chunk[k] * 16));
        }
#pragma unroll
        for (int k = 0; k < K; ++k) cur[k] = op_chunk<DT, IOMX_OP_ADD>(cur[k], other[k]);
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (FULL || tid + k * THREADS < part_chunks)
                __builtin_nontemporal_store(cur[k], reinterpret_cast<u32x4*>(sb + (uint64_t)chunk[k] * 16));
        }
    }
    if constexpr (PRE) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint32_t soff = ((chunk[k] / L::kChunksPerTile) * L::kChunksPerTile
                                   + (chunk[k] % L::kChunksPerRow)) * 16;
            scl[k] = u32x4{0, 0, 0, 0};
            if (FULL || tid + k * THREADS < part_chunks)
                scl[k] = *reinterpret_cast<const u32x4*>(a.scale + soff);
        }
    }
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        float f[L::kPerChunk];
        unpack<DT>(cur[k], f);
#pragma unroll
        for (uint32_t e = 0; e < L::kPerChunk; ++e) acc = __builtin_fmaf(f[e], f[e], acc);
    }
    if constexpr (L::kBytes <= 2) {
#pragma unroll
        for (int k = 0; k < K; ++k) asm volatile("" : "+v"(cur[k]));
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
    float total = acc;
    if constexpr (kWaves > 1) {
        if ((tid & shared_bits) == 0) partial[row][tid / 64] = acc;
        __syncthreads();
        total = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kWaves; ++wv) total = total + partial[row][wv];
    }
    const float inverse = inverse_rms(total, a.feats, a.eps);
    if (tr * kTile + part * RP + row >= a.rows) return;
    if constexpr (PRE) {
        u32x4 res[K];
#pragma unroll
        for (int k = 0; k < K; ++k) {
            float f[L::kPerChunk], sc[L::kPerChunk];
            unpack<DT>(cur[k], f);
            unpack<DT>(scl[k], sc);
#pragma unroll
            for (uint32_t e = 0; e < L::kPerChunk; ++e) {
                const float normalized = f[e] * inverse;
                f[e] = normalized * sc[e];
            }
            res[k] = pack<DT>(f);
        }
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (FULL || tid + k * THREADS < part_chunks)
                __builtin_nontemporal_store(res[k], reinterpret_cast<u32x4*>(ob + (uint64_t)chunk[k] * 16));
        }
    } else {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (FULL || tid + k * THREADS < part_chunks) {
                const uint32_t soff = ((chunk[k] / L::kChunksPerTile) * L::kChunksPerTile
                                       + (chunk[k] % L::kChunksPerRow)) * 16;
                float f[L::kPerChunk], sc[L::kPerChunk];
                unpack<DT>(cur[k], f);
                unpack<DT>(*reinterpret_cast<const u32x4*>(a.scale + soff), sc);
#pragma unroll
                for (uint32_t e = 0; e < L::kPerChunk; ++e) {
                    const float normalized = f[e] * inverse;
                    f[e] = normalized * sc[e];
                }
                __builtin_nontemporal_store(pack<DT>(f), reinterpret_cast<u32x4*>(ob + (uint64_t)chunk[k] * 16));
            }
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

template <int DT, int K, int S, int THREADS, bool ADD, bool PRE = (K * (int)RLeaf<DT>::kPerChunk <= 32)>
void launch_band(const RmsArgsT<ADD ? 4 : 2>& a, hipStream_t s) {
    const uint32_t grid = a.total_bands * S;
    // Workgroups per CU.  A workgroup of the 2-byte leaves that holds 32 KiB on 512 lanes would fit a
    // CU four times (2048 lanes); three of them stream faster: four loads of 32 KiB each in flight,
    // then four bursts of stores, is more than the memory side of a CU takes without queueing.  An
    // LDS request nobody uses, of a size that fits three times into a CU's 160 KiB, sets that
    // (BF16 [32768,2048]: 5830 -> 5950 GB/s, [65536,1024]: 6010 -> 6060; with two, 5800; the
    // 16 KiB and 64 KiB workgroups of the other shapes and the F32 shapes of any size: no change or
    // a loss).  The fused add + norm holds twice the bytes and takes two per CU (5560 -> 5610).
    uint32_t lds = 0;
    if (RLeaf<DT>::kBytes == 2 && K == 4 && THREADS == 512) lds = ADD ? 72u * 1024 : 48u * 1024;
    if ((uint32_t)(K * THREADS * S) == a.band_chunks)
        hipLaunchKernelGGL((rmsnorm_band_kernel<DT, K, S, THREADS, true, PRE, ADD>), dim3(grid), dim3(THREADS), lds, s, a);
    else
        hipLaunchKernelGGL((rmsnorm_band_kernel<DT, K, S, THREADS, false, PRE, ADD>), dim3(grid), dim3(THREADS), lds, s, a);
    record_launch(ADD ? (S == 1 ? "add_rmsnorm_band" : "add_rmsnorm_split") : (S == 1 ? "rmsnorm_band" : "rmsnorm_split"),
                  grid, THREADS, grid);
}

// Which shape of the resident kernel: n = 128-bit chunks of one band (2F for the 2-byte
// leaves, 4F for F32).  Measured on MI355X over 128 MiB of rows of 512..16384 features
// (GB/s of x + out, average of three runs of 40 launches):
//   * four chunks per lane is the sweet spot; at equal bytes per workgroup 512 lanes do as
//     well as 1024 (BF16 n = 2048: K4 T512 5890, K2 T1024 5440; F32 n = 4096: K4 S2 T512
//     5930, K4 S1 T1024 5780), more chunks per lane cost 5-10 % (F32 n = 8192: K4 S2 5950,
//     K8 S1 5420), except for very wide F32 rows, where sixteen chunks on two parts beat
//     eight on four (n = 32768: 5890 against 5220);
//   * a part's runs should stay at 256 bytes or more per tile: 128-byte runs cost 5-20 %
//     and 32-byte runs (sixteen parts) lose even to the two-pass kernel;
//   * a shape whose K * THREADS * S chunks exceed n idles lanes in proportion, so the
//     four-part shapes are kept for the widths they fit exactly.
// Whether the resident kernel serves n chunks per band of a leaf.
template <int DT>
bool band_kernel_serves(uint32_t n, uint32_t total_bands) {
    constexpr bool wide = RLeaf<DT>::kBytes != 2;      // 64 chunks per tile instead of 32
    return total_bands <= 0x7FFFFFFFu / 8 && n <= (wide ? 131072u : 65536u);
}

// (The fused add + norm takes the shape the norm alone takes: the order in which a row's squares
// are summed follows from K, S and the lanes, and the fused result is to be the two launches'
// result bit for bit.  Two chunks per lane on 1024 lanes would be 2 % faster for the fused kernel
// at [32768,2048] BF16, 94.2 against 95.8 us.)
template <int DT, bool ADD>
void launch_resident(const RmsArgsT<ADD ? 4 : 2>& a, hipStream_t s) {
    const uint32_t n = a.band_chunks;
    constexpr bool wide = RLeaf<DT>::kBytes != 2;
    if (n <= 64) launch_band<DT, 1, 1, 64, ADD>(a, s);
    else if (n <= 256) launch_band<DT, 1, 1, 256, ADD>(a, s);
    else if (n <= 512) launch_band<DT, 2, 1, 256, ADD>(a, s);
    else if (n <= 1024) launch_band<DT, 2, 1, 512, ADD>(a, s);
    else if (n <= 2048) launch_band<DT, 4, 1, 512, ADD>(a, s);
    else if (n <= 4096) launch_band<DT, 4, 2, 512, ADD>(a, s);
    else if (n <= 8192) launch_band<DT, 4, 2, 1024, ADD>(a, s);
    else if (n == 16384) launch_band<DT, 4, 4, 1024, ADD>(a, s);
    else if (n <= 16384) launch_band<DT, 8, 2, 1024, ADD>(a, s);
    else if (n <= 32768) {
        if constexpr (wide) launch_band<DT, 16, 2, 1024, ADD>(a, s);
        else launch_band<DT, 8, 4, 1024, ADD, true>(a, s);
    } else if (n <= 65536) {
        launch_band<DT, 8, 8, 1024, ADD>(a, s);
    } else {
        if constexpr (wide) launch_band<DT, 16, 8, 1024, ADD>(a, s);
    }
}

// The 8-bit floating leaves: n = F chunks per band (a tile is 256 bytes, sixteen chunks); whole
// bands per workgroup up to 8192 features, two parts of eight rows beyond.
constexpr uint32_t kF8BandLimit = 16384;
template <int DT>
void launch_resident_f8(const RmsArgs& a, hipStream_t s) {
    const uint32_t n = a.band_chunks;
    if (n <= 64) launch_band<DT, 1, 1, 64, false, true>(a, s);
    else if (n <= 256) launch_band<DT, 1, 1, 256, false, true>(a, s);
    else if (n <= 512) launch_band<DT, 2, 1, 256, false, true>(a, s);
    else if (n <= 1024) launch_band<DT, 2, 1, 512, false, true>(a, s);
    else if (n <= 2048) launch_band<DT, 4, 1, 512, false, true>(a, s);
    else if (n <= 4096) launch_band<DT, 4, 1, 1024, false, true>(a, s);
    else if (n <= 8192) launch_band<DT, 8, 1, 1024, false, false>(a, s);
    else launch_band<DT, 8, 2, 1024, false, false>(a, s);
}

template <int DT>
int launch(const RmsArgs& a, bool band_ok, hipStream_t s) {
    if (!band_ok || !band_kernel_serves<DT>(a.band_chunks, a.total_bands)) {
        const uint32_t cap = 1u << 20;
        const uint32_t grid = a.total_bands < cap ? a.total_bands : cap;
        hipLaunchKernelGGL((rmsnorm_generic_kernel<DT>), dim3(grid), dim3(256), 0, s, a);
        record_launch("rmsnorm_generic", grid, 256, a.total_bands);
        return IOMX_OK;
    }
    launch_resident<DT, false>(a, s);
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
    // (the 8-bit floating leaves take the resident kernel where a band is whole tiles and fits it)
    bool f8_resident = is_f8(dtype) && m.cols % kTile == 0 && m.tile_cols * 16 <= kF8BandLimit;
    if (f8_resident) {
        uint64_t bands = m.tile_rows;            // of all leading planes: two workgroups a band at most
        for (uint32_t i = 0; i + 2 < x->rank; ++i)
            if (mul_overflows(bands, x->dims[i], &bands)) bands = ~0ull;
        f8_resident = bands <= 0x7FFFFFFFull / 8;
    }
    if (dtype != IOMX_DT_BF16 && dtype != IOMX_DT_F32 && dtype != IOMX_DT_F16 && !f8_resident) {
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
    else if (dtype == IOMX_DT_F8_E4M3FN) launch_resident_f8<IOMX_DT_F8_E4M3FN>(a, s);
    else if (dtype == IOMX_DT_F8_E5M2) launch_resident_f8<IOMX_DT_F8_E5M2>(a, s);
    else IOMX_TRY(launch<IOMX_DT_F32>(a, band_ok, s));
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}

// x + y -> sum, rmsnorm(sum, scale) -> out in one launch (a private fusion: IOM has no such
// operation; the public path is iomx_launch_binary(ADD) followed by iomx_launch_rmsnorm, and
// this entry point produces the same bits in both outputs).  Served where the resident kernel
// serves the shape without padding: BF16 / F16 / F32, features and rows multiples of 16, all four
// tensors of one shape (no broadcast); anything else is IOMX_ERR_UNSUPPORTED and the caller
// makes the two launches.  `sum` may be x or y itself (the exact alias the ADD allows: every
// lane reads both inputs of a chunk before it stores the chunk); `out` must share storage with
// none of the others.
extern "C" int iomx_launch_add_rmsnorm(int dtype, const iomx_view* x, const iomx_view* y,
                                       const iomx_view* sum, const iomx_view* scale,
                                       const iomx_view* out, float eps, iomx_stream_t stream) {
    if (dtype != IOMX_DT_BF16 && dtype != IOMX_DT_F32 && dtype != IOMX_DT_F16) return IOMX_ERR_UNSUPPORTED;
    const uint32_t bits = leaf_bits(dtype);
    const uint32_t bytes = bits / 8;
    const iomx_view* full[4] = {x, out, y, sum};
    for (const iomx_view* v : full) IOMX_TRY(check_view(v, bits));
    IOMX_TRY(check_view(scale, bits));
    for (int k = 1; k < 4; ++k) {
        if (full[k]->rank != x->rank) return IOMX_ERR_INVALID;
        for (uint32_t i = 0; i < x->rank; ++i) if (full[k]->dims[i] != x->dims[i]) return IOMX_ERR_INVALID;
    }
    const Matrix m = matrix_of(*x);
    if (scale->rank != 2 || scale->dims[0] != 1 || scale->dims[1] != m.cols) return IOMX_ERR_INVALID;
    if (out->base == x->base || out->base == y->base || out->base == sum->base || out->base == scale->base
        || sum->base == scale->base)
        return IOMX_ERR_INVALID;
    // an input that shares the sum's storage must be the identical window
    for (const iomx_view* in : {x, y}) {
        if (in->base != sum->base) continue;
        if (in->plane_offset != sum->plane_offset) return IOMX_ERR_INVALID;
        for (uint32_t i = 0; i + 2 < x->rank; ++i)
            if (in->plane_strides[i] != sum->plane_strides[i]) return IOMX_ERR_INVALID;
    }
    if (!(eps >= 0.0f) || eps > 3.4028234e38f) return IOMX_ERR_INVALID;
    if (m.cols % kTile != 0 || m.rows % kTile != 0) return IOMX_ERR_UNSUPPORTED;

    RmsArgsT<4> a = {};
    uint64_t strides[4][kMaxLead] = {};
    uint64_t offsets[4];
    for (int k = 0; k < 4; ++k) {
        offsets[k] = full[k]->plane_offset;
        for (uint32_t i = 0; i + 2 < x->rank; ++i) strides[k][i] = full[k]->plane_strides[i];
    }
    IOMX_TRY(build_walk<4>(x->rank - 2, x->dims, strides, offsets, &a.walk));
    const uint64_t band_chunks = m.tile_cols * (kTileSlots * bytes / 16);
    uint64_t total_bands;
    if (mul_overflows(a.walk.planes, m.tile_rows, &total_bands)) return IOMX_ERR_OVERFLOW;
    if (total_bands > 0xFFFFFFFFull || band_chunks > 0x0FFFFFFFull || m.rows > 0xFFFFFFFFull
        || m.cols > 0xFFFFFFFFull)
        return IOMX_ERR_OVERFLOW;
    a.x = static_cast<const uint8_t*>(x->base);
    a.out = static_cast<uint8_t*>(out->base);
    a.y = static_cast<const uint8_t*>(y->base);
    a.sum = static_cast<uint8_t*>(sum->base);
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
    bool dense = a.walk.nlead <= 1 && total_bands * kTile <= 0xFFFFFFFFull;
    for (int k = 0; k < 4; ++k) dense = dense && walk_is_dense(a.walk, k);
    if (dense) {
        // whole bands of a dense selection: all planes fold into one run of bands
        a.x += a.walk.offset[0] * a.plane_bytes;
        a.out += a.walk.offset[1] * a.plane_bytes;
        a.y += a.walk.offset[2] * a.plane_bytes;
        a.sum += a.walk.offset[3] * a.plane_bytes;
        for (int k = 0; k < 4; ++k) a.walk.offset[k] = 0;
        a.walk.nlead = 0;
        a.tile_rows = (uint32_t)total_bands;
        a.rows = (uint32_t)(total_bands * kTile);
    }
    const hipStream_t s = native(stream);
    if (dtype == IOMX_DT_BF16) {
        if (!band_kernel_serves<IOMX_DT_BF16>(a.band_chunks, a.total_bands)) return IOMX_ERR_UNSUPPORTED;
        launch_resident<IOMX_DT_BF16, true>(a, s);
    } else if (dtype == IOMX_DT_F16) {
        if (!band_kernel_serves<IOMX_DT_F16>(a.band_chunks, a.total_bands)) return IOMX_ERR_UNSUPPORTED;
        launch_resident<IOMX_DT_F16, true>(a, s);
    } else {
        if (!band_kernel_serves<IOMX_DT_F32>(a.band_chunks, a.total_bands)) return IOMX_ERR_UNSUPPORTED;
        launch_resident<IOMX_DT_F32, true>(a, s);
    }
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}
