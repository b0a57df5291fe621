// The remaining non-contraction operations of a transformer layer: cache-row
// append, embedding row lookup, split-half rotary position encoding.  All three
// work on tile rows (sixteen packed elements, whole 32-bit words) of any leaf.
#include "iomx_rows.hpp"

namespace iomx {

// ---------------------------------------------------------------------------
// Cache append: destination[..., a + r, :] = source[..., r, :]
// ---------------------------------------------------------------------------

struct AppendArgs {
    const uint8_t* src;
    uint8_t* dst;
    PlaneWalk<2> walk;  // 0 source, 1 destination
    uint64_t plane_bytes[2];
    uint32_t tile_cols, rows, cols;
    uint32_t rows_per_plane;  // padded tile rows of one source plane
    FastDiv div_tile_cols;
    uint32_t planes;
    uint32_t a;
};

template <int BITS>
__global__ __launch_bounds__(256) void cache_append_kernel(const AppendArgs a) {
    constexpr int K = BITS / 2;
    constexpr uint32_t kRowBytes = 2 * BITS, kTileBytes = 32 * BITS;
    const TileRow t = tile_row_of(blockIdx.x * 256u + threadIdx.x, a.rows_per_plane, a.tile_cols,
                                  a.div_tile_cols, a.rows, a.cols);
    if (!t.live) return;
    const uint32_t drow = a.a + t.row;
    const uint64_t soff = ((uint64_t)(t.row >> 4) * a.tile_cols + t.tc) * kTileBytes + (t.row & 15u) * kRowBytes;
    const uint64_t doff = ((uint64_t)(drow >> 4) * a.tile_cols + t.tc) * kTileBytes + (drow & 15u) * kRowBytes;
    for (uint32_t p = blockIdx.y; p < a.planes; p += gridDim.y) {
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        uint32_t w[K];
        load_row<BITS>(a.src + plane[0] * a.plane_bytes[0] + soff, w);
        store_row<BITS>(a.dst + plane[1] * a.plane_bytes[1] + doff, w, t.ncols);
    }
}

// ---------------------------------------------------------------------------
// Embedding: out[..., r, :] = table[indices[..., 0, r], :]
// ---------------------------------------------------------------------------

struct EmbedArgs {
    const uint8_t* table;    // the selected table plane
    const uint8_t* indices;
    uint8_t* out;
    uint32_t* status;        // set to 1 by any lane that meets an invalid id
    PlaneWalk<2> walk;       // 0 indices, 1 out
    uint64_t index_plane_bytes, out_plane_bytes;
    uint32_t tile_cols, run, feats;
    uint32_t rows_per_plane;
    FastDiv div_tile_cols;
    uint32_t planes;
    uint32_t index_signed;
    uint64_t vocabulary;
};

__global__ void store_word_kernel(uint32_t* p, uint32_t v) { *p = v; }

// An id is decoded at its full width, its sign bit is inspected before any
// conversion and the unsigned value is compared with the vocabulary before any
// address is formed (docs/BACKEND_CONTRACT/embedding-lookup.md:262-268); an
// invalid id raises the status word and its output row is left alone.
template <int BITS, int IBITS>
__global__ __launch_bounds__(256) void embedding_kernel(const EmbedArgs a) {
    constexpr int K = BITS / 2;
    constexpr uint32_t kRowBytes = 2 * BITS, kTileBytes = 32 * BITS;
    const TileRow t = tile_row_of(blockIdx.x * 256u + threadIdx.x, a.rows_per_plane, a.tile_cols,
                                  a.div_tile_cols, a.run, a.feats);
    if (!t.live) return;
    // element r of an [1,R] plane: row 0 of tile r/16
    const uint64_t index_bit = ((uint64_t)(t.row >> 4) * kTileSlots + (t.row & 15u)) * IBITS;
    const uint64_t ooff = ((uint64_t)(t.row >> 4) * a.tile_cols + t.tc) * kTileBytes + (t.row & 15u) * kRowBytes;
    for (uint32_t p = blockIdx.y; p < a.planes; p += gridDim.y) {
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint64_t raw = read_bits<IBITS>(
                reinterpret_cast<const uint32_t*>(a.indices + plane[0] * a.index_plane_bytes), index_bit);
        const bool negative = a.index_signed && ((raw >> (IBITS - 1)) & 1ull);
        if (negative || raw >= a.vocabulary) {
            *a.status = 1u;
            continue;
        }
        const uint64_t toff = ((raw >> 4) * a.tile_cols + t.tc) * kTileBytes + (raw & 15ull) * kRowBytes;
        uint32_t w[K];
        load_row<BITS>(a.table + toff, w);
        store_row<BITS>(a.out + plane[1] * a.out_plane_bytes + ooff, w, t.ncols);
    }
}

// ---------------------------------------------------------------------------
// RoPE (split halves): for c < D/2 and position = a + row,
//   frequency = pow(theta, -2c/D), angle = position * frequency,
//   out[c]       = x[c] * cos - x[c + D/2] * sin
//   out[c + D/2] = x[c + D/2] * cos + x[c] * sin
// in binary32 (binary64 for F64), four products and one subtraction / addition
// as separate roundings, one encode per result; a row at position 0 is a raw
// copy (src/cpu/queue.cpp:1357-1411,1498-1521).  The angle depends on the row
// and the column only, so a lane evaluates its sixteen sine / cosine pairs once
// and reuses them for every plane it walks.
// ---------------------------------------------------------------------------

struct RopeArgs {
    const uint8_t* x;
    uint8_t* out;
    PlaneWalk<2> walk;  // 0 x, 1 out
    uint64_t plane_bytes;
    uint32_t rows, width, half, tile_cols;
    uint32_t col_tiles;       // tiles a lane index runs over: pair tiles (aligned) or all tiles
    uint32_t lanes_per_plane;
    FastDiv div_col_tiles;
    uint32_t planes;
    uint32_t a;
    double theta;
};

template <int DT, typename T>
__device__ __forceinline__ T rope_decode(uint64_t raw) {
    if constexpr (DT == DT_BF16) return (T)as_f32((uint32_t)raw << 16);
    else if constexpr (DT == DT_F32) return (T)as_f32((uint32_t)raw);
    else return decode_as<DT, T>(raw);
}

template <int DT, typename T>
__device__ __forceinline__ uint64_t rope_encode(T v) {
    if constexpr (DT == DT_BF16) return bf16_rne_sw(as_u32((float)v));
    else if constexpr (DT == DT_F32) return as_u32(canonical((float)v));
    else return encode_from<DT, T>(v);
}

__device__ __forceinline__ float rope_frequency(uint32_t column, uint32_t width, float theta) {
    return powf(theta, (float)((-2.0 * (double)column) / (double)width));
}
__device__ __forceinline__ double rope_frequency(uint32_t column, uint32_t width, double theta) {
    return pow(theta, (-2.0 * (double)column) / (double)width);
}
__device__ __forceinline__ void rope_sincos(uint32_t position, float frequency, float* sine, float* cosine) {
    sincosf((float)position * frequency, sine, cosine);
}
__device__ __forceinline__ void rope_sincos(uint32_t position, double frequency, double* sine, double* cosine) {
    sincos((double)position * frequency, sine, cosine);
}
template <typename T>
__device__ __forceinline__ void rope_angle(uint32_t column, uint32_t width, uint32_t position,
                                           T theta, T* sine, T* cosine) {
    rope_sincos(position, rope_frequency(column, width, theta), sine, cosine);
}

// D/2 a multiple of 16: a lane owns tile rows tc and tc + D/32 of one row.
template <int DT, typename T>
__global__ __launch_bounds__(256) void rope_pairs_kernel(const RopeArgs a) {
    constexpr int BITS = bits_of(DT);
    constexpr int K = BITS / 2;
    constexpr uint32_t kRowBytes = 2 * BITS, kTileBytes = 32 * BITS;
    const uint32_t g = blockIdx.x * 256u + threadIdx.x;
    const uint32_t r = g & 15u, q = g >> 4;
    const uint32_t tr = a.col_tiles > 1 ? fast_div(q, a.div_col_tiles) : q;
    const uint32_t ptc = q - tr * a.col_tiles;
    const uint32_t row = tr * kTile + r;
    // the 16 lanes of a pair tile need the same 16 frequencies: one power each, exchanged
    // (every lane of the wave takes part, also those without a row)
    const T own_frequency = rope_frequency(ptc * kTile + r, a.width, (T)a.theta);
    T frequency[kTile];
#pragma unroll
    for (int i = 0; i < (int)kTile; ++i) frequency[i] = __shfl(own_frequency, i, 16);
    if (g >= a.lanes_per_plane || row >= a.rows) return;
    const uint32_t position = a.a + row;
    T sine[kTile], cosine[kTile];
    if (position != 0) {
#pragma unroll
        for (int i = 0; i < (int)kTile; ++i) rope_sincos(position, frequency[i], &sine[i], &cosine[i]);
    }
    const uint64_t off0 = ((uint64_t)tr * a.tile_cols + ptc) * kTileBytes + r * kRowBytes;
    const uint64_t off1 = off0 + (uint64_t)(a.half >> 4) * kTileBytes;
    for (uint32_t p = blockIdx.y; p < a.planes; p += gridDim.y) {
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint8_t* xb = a.x + plane[0] * a.plane_bytes;
        uint8_t* ob = a.out + plane[1] * a.plane_bytes;
        uint32_t w0[K], w1[K];
        load_row<BITS>(xb + off0, w0);
        load_row<BITS>(xb + off1, w1);
        if (position != 0) {
            uint32_t r0[K], r1[K];
#pragma unroll
            for (int j = 0; j < K; ++j) { r0[j] = 0; r1[j] = 0; }
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i) {
                const T first = rope_decode<DT, T>(get<BITS>(w0, i));
                const T second = rope_decode<DT, T>(get<BITS>(w1, i));
                const T fc = first * cosine[i], ss = second * sine[i];
                const T sc = second * cosine[i], fs = first * sine[i];
                put<BITS>(r0, i, rope_encode<DT, T>(fc - ss));
                put<BITS>(r1, i, rope_encode<DT, T>(sc + fs));
            }
            store_row<BITS>(ob + off0, r0, kTile);
            store_row<BITS>(ob + off1, r1, kTile);
        } else {
            store_row<BITS>(ob + off0, w0, kTile);
            store_row<BITS>(ob + off1, w1, kTile);
        }
    }
}

// BF16, D/2 a multiple of 16: a lane owns one 16-byte chunk (eight columns of one row) of pair
// tile tc and the matching chunk of tile tc + D/32, so a wave's request is 1 KiB of consecutive
// memory.  A word holds columns 2j and 2j + 1, and the hardware conversion packs two results
// with the rounding of the software encode (nearest even, gradual underflow; NaN made
// canonical first).  The planes a lane walks are independent of each other, so the next
// plane's chunks are requested before the present ones are rotated and stored.
__global__ __launch_bounds__(256) void rope_pairs_bf16_kernel(const RopeArgs a) {
    constexpr uint32_t kRowBytes = 32, kTileBytes = 512;
    const uint32_t g = blockIdx.x * 256u + threadIdx.x;
    const uint32_t h = g & 1u, r = (g >> 1) & 15u, q = g >> 5;
    const uint32_t tr = a.col_tiles > 1 ? fast_div(q, a.div_col_tiles) : q;
    const uint32_t ptc = q - tr * a.col_tiles;
    const uint32_t row = tr * kTile + r;
    // the 32 lanes of a pair tile need its 16 frequencies: one power each, exchanged
    const float own_frequency = rope_frequency(ptc * kTile + (g & 15u), a.width, (float)a.theta);
    float frequency[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) frequency[i] = __shfl(own_frequency, (int)(8u * h) + i, 32);
    if (g >= 2u * a.lanes_per_plane || row >= a.rows) return;
    const uint32_t position = a.a + row;
    float sine[8], cosine[8];
    if (position != 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) rope_sincos(position, frequency[i], &sine[i], &cosine[i]);
    }
    const uint64_t off0 = ((uint64_t)tr * a.tile_cols + ptc) * kTileBytes + r * kRowBytes + h * 16u;
    const uint64_t off1 = off0 + (uint64_t)(a.half >> 4) * kTileBytes;
    uint32_t p = blockIdx.y;
    if (p >= a.planes) return;
    auto request = [&](uint32_t which, u32x4* first, u32x4* second) {
        uint64_t pl[2];
        walk_planes(a.walk, which, pl);
        const uint8_t* xb = a.x + pl[0] * a.plane_bytes;
        *first = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xb + off0));
        *second = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xb + off1));
    };
    u32x4 f, s2, nf = {}, ns = {};
    request(p, &f, &s2);
    for (;;) {
        const uint32_t following = p + gridDim.y;
        const bool more = following < a.planes;
        if (more) request(following, &nf, &ns);
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        uint8_t* ob = a.out + plane[1] * a.plane_bytes;
        if (position != 0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int i = 2 * j;
                const float fa = bf16_lo(f[j]), fb = bf16_hi(f[j]);
                const float sa = bf16_lo(s2[j]), sb = bf16_hi(s2[j]);
                const float fca = fa * cosine[i], ssa = sa * sine[i];
                const float sca = sa * cosine[i], fsa = fa * sine[i];
                const float fcb = fb * cosine[i + 1], ssb = sb * sine[i + 1];
                const float scb = sb * cosine[i + 1], fsb = fb * sine[i + 1];
                f[j] = pack_bf16(fca - ssa, fcb - ssb);
                s2[j] = pack_bf16(sca + fsa, scb + fsb);
            }
        }
        __builtin_nontemporal_store(f, reinterpret_cast<u32x4*>(ob + off0));
        __builtin_nontemporal_store(s2, reinterpret_cast<u32x4*>(ob + off1));
        if (!more) break;
        f = nf;
        s2 = ns;
        p = following;
    }
}

// One row per plane (a decode step): every plane has the same position, so the 16
// lanes of a group evaluate one angle each, exchange them, and then rotate the row
// of 16 different planes: no lane repeats the powf / sincos work of another.
template <int DT, typename T>
__global__ __launch_bounds__(256) void rope_row_kernel(const RopeArgs a) {
    constexpr int BITS = bits_of(DT);
    constexpr int K = BITS / 2;
    constexpr uint32_t kTileBytes = 32 * BITS;
    const uint32_t g = blockIdx.x * 256u + threadIdx.x;
    const uint32_t r = g & 15u, q = g >> 4;
    const uint32_t pg = a.col_tiles > 1 ? fast_div(q, a.div_col_tiles) : q;   // group of 16 planes
    const uint32_t ptc = q - pg * a.col_tiles;
    const uint32_t position = a.a;
    T my_sine = (T)0, my_cosine = (T)1;
    if (position != 0) rope_angle(ptc * kTile + r, a.width, position, (T)a.theta, &my_sine, &my_cosine);
    T sine[kTile], cosine[kTile];
    const int base = (int)(threadIdx.x & 63u & ~15u);
#pragma unroll
    for (int i = 0; i < (int)kTile; ++i) {          // every lane of the wave takes part
        sine[i] = __shfl(my_sine, base + i);
        cosine[i] = __shfl(my_cosine, base + i);
    }
    const uint64_t p = (uint64_t)pg * kTile + r;
    if (p >= a.planes) return;
    const uint64_t off0 = (uint64_t)ptc * kTileBytes;                 // row 0 of the first tile row
    const uint64_t off1 = off0 + (uint64_t)(a.half >> 4) * kTileBytes;
    uint64_t plane[2];
    walk_planes(a.walk, (uint32_t)p, plane);
    const uint8_t* xb = a.x + plane[0] * a.plane_bytes;
    uint8_t* ob = a.out + plane[1] * a.plane_bytes;
    uint32_t w0[K], w1[K];
    load_row<BITS>(xb + off0, w0);
    load_row<BITS>(xb + off1, w1);
    if (position != 0) {
        uint32_t r0[K], r1[K];
#pragma unroll
        for (int j = 0; j < K; ++j) { r0[j] = 0; r1[j] = 0; }
#pragma unroll
        for (int i = 0; i < (int)kTile; ++i) {
            const T first = rope_decode<DT, T>(get<BITS>(w0, i));
            const T second = rope_decode<DT, T>(get<BITS>(w1, i));
            const T fc = first * cosine[i], ss = second * sine[i];
            const T sc = second * cosine[i], fs = first * sine[i];
            put<BITS>(r0, i, rope_encode<DT, T>(fc - ss));
            put<BITS>(r1, i, rope_encode<DT, T>(sc + fs));
        }
        store_row<BITS>(ob + off0, r0, kTile);
        store_row<BITS>(ob + off1, r1, kTile);
    } else {
        store_row<BITS>(ob + off0, w0, kTile);
        store_row<BITS>(ob + off1, w1, kTile);
    }
}

// Any even D: a lane owns one output tile row and fetches each partner element
// from wherever the other half puts it.
template <int DT, typename T>
__global__ __launch_bounds__(256) void rope_general_kernel(const RopeArgs a) {
    constexpr int BITS = bits_of(DT);
    constexpr int K = BITS / 2;
    constexpr uint32_t kRowBytes = 2 * BITS, kTileBytes = 32 * BITS;
    const TileRow t = tile_row_of(blockIdx.x * 256u + threadIdx.x, a.lanes_per_plane, a.tile_cols,
                                  a.div_col_tiles, a.rows, a.width);
    if (!t.live) return;
    const uint32_t position = a.a + t.row;
    T sine[kTile], cosine[kTile];
    if (position != 0) {
#pragma unroll
        for (int i = 0; i < (int)kTile; ++i) {
            const uint32_t c = t.tc * kTile + i;
            if (c < a.width)
                rope_angle(c < a.half ? c : c - a.half, a.width, position, (T)a.theta, &sine[i], &cosine[i]);
        }
    }
    const uint64_t row_base = (uint64_t)(t.row >> 4) * a.tile_cols * kTileBytes + (t.row & 15u) * kRowBytes;
    const uint64_t off = row_base + (uint64_t)t.tc * kTileBytes;
    for (uint32_t p = blockIdx.y; p < a.planes; p += gridDim.y) {
        uint64_t plane[2];
        walk_planes(a.walk, p, plane);
        const uint8_t* xb = a.x + plane[0] * a.plane_bytes;
        uint32_t w[K], res[K];
        load_row<BITS>(xb + off, w);
        if (position != 0) {
#pragma unroll
            for (int j = 0; j < K; ++j) res[j] = 0;
#pragma unroll
            for (int i = 0; i < (int)kTile; ++i) {
                const uint32_t c = t.tc * kTile + i;
                if (c >= a.width) continue;
                const bool low = c < a.half;
                const uint32_t partner = low ? c + a.half : c - a.half;
                // bit address of the partner inside this row of tiles
                const uint64_t bit = (row_base + (uint64_t)(partner >> 4) * kTileBytes) * 8ull
                        + (uint64_t)(partner & 15u) * BITS;
                const T own = rope_decode<DT, T>(get<BITS>(w, i));
                const T other = rope_decode<DT, T>(read_bits<BITS>(reinterpret_cast<const uint32_t*>(xb), bit));
                // low half: first*cos - second*sin; high half: second*cos + first*sin, where
                // this lane's own element is `first` in the low half and `second` in the high
                const T oc = own * cosine[i], os = other * sine[i];
                const T y = low ? oc - os : oc + os;
                put<BITS>(res, i, rope_encode<DT, T>(y));
            }
        } else {
#pragma unroll
            for (int j = 0; j < K; ++j) res[j] = w[j];
        }
        store_row<BITS>(a.out + plane[1] * a.plane_bytes + off, res, t.ncols);
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

namespace {

bool same_leading(const iomx_view* a, const iomx_view* b, uint32_t axes) {
    for (uint32_t i = 0; i < axes; ++i) if (a->dims[i] != b->dims[i]) return false;
    return true;
}

template <int N>
int walk_of(const iomx_view* const (&v)[N], const uint64_t* dims, uint32_t nlead, PlaneWalk<N>* w) {
    uint64_t strides[N][kMaxLead] = {};
    uint64_t offsets[N];
    for (int k = 0; k < N; ++k) {
        offsets[k] = v[k]->plane_offset;
        for (uint32_t i = 0; i < nlead; ++i) strides[k][i] = v[k]->plane_strides[i];
    }
    return build_walk<N>(nlead, dims, strides, offsets, w);
}

bool is_signed_index(int dtype) {
    return dtype == DT_I2 || dtype == DT_I4 || dtype == DT_I8 || dtype == DT_I16 || dtype == DT_I32
            || dtype == DT_I64;
}

bool is_index_leaf(int dtype) { return dtype >= DT_I2 && dtype <= DT_U64; }

// Enough planes per lane to reuse its angles, enough lanes to fill the device.
uint32_t planes_in_grid(uint64_t lanes_per_plane, uint64_t planes) {
    const uint64_t target = 1ull << 17;  // measured best on [64,32,512,64] BF16: 16 planes per lane
    uint64_t y = (target + lanes_per_plane - 1) / lanes_per_plane;
    if (y < 1) y = 1;
    if (y > planes) y = planes;
    if (y > 65535) y = 65535;
    return (uint32_t)y;
}

template <int DT, typename T>
void launch_rope(const RopeArgs& a, bool aligned, dim3 grid, hipStream_t s) {
    if (aligned && a.rows == 1) hipLaunchKernelGGL((rope_row_kernel<DT, T>), grid, dim3(256), 0, s, a);
    else if (aligned && DT == DT_BF16 && a.lanes_per_plane <= 0x7FFFFF00u) {
        const dim3 chunks((uint32_t)((2ull * a.lanes_per_plane + 255) / 256), grid.y, 1);
        hipLaunchKernelGGL(rope_pairs_bf16_kernel, chunks, dim3(256), 0, s, a);
    } else if (aligned) hipLaunchKernelGGL((rope_pairs_kernel<DT, T>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((rope_general_kernel<DT, T>), grid, dim3(256), 0, s, a);
}

}  // namespace
}  // namespace iomx

using namespace iomx;

extern "C" {

// Admission of src/device_ops_cache_append.cpp:160-270 (everything checkable
// without owner identities).
int iomx_launch_cache_append(int dtype, const iomx_view* source, const iomx_view* destination,
                             uint64_t a, iomx_stream_t stream) {
    const uint32_t bits = leaf_bits(dtype);
    if (!bits) return IOMX_ERR_UNSUPPORTED;
    IOMX_TRY(check_view(source, bits));
    IOMX_TRY(check_view(destination, bits));
    if (source->rank < 3 || source->rank != destination->rank) return IOMX_ERR_INVALID;
    const uint32_t rank = source->rank;
    if (!same_leading(source, destination, rank - 2)) return IOMX_ERR_INVALID;
    const Matrix sm = matrix_of(*source), dm = matrix_of(*destination);
    if (sm.cols != dm.cols) return IOMX_ERR_INVALID;
    if (a > dm.rows || sm.rows > dm.rows - a) return IOMX_ERR_INVALID;   // in this order
    if (source->base == destination->base) return IOMX_ERR_INVALID;
    if (dm.rows > 0xFFFFFFFFull || sm.cols > 0xFFFFFFFFull) return IOMX_ERR_OVERFLOW;
    AppendArgs k = {};
    const iomx_view* v[2] = {source, destination};
    IOMX_TRY(walk_of<2>(v, source->dims, rank - 2, &k.walk));
    k.src = static_cast<const uint8_t*>(source->base);
    k.dst = static_cast<uint8_t*>(destination->base);
    k.plane_bytes[0] = sm.plane_elems * bits / 8;
    k.plane_bytes[1] = dm.plane_elems * bits / 8;
    k.tile_cols = (uint32_t)sm.tile_cols;
    k.rows = (uint32_t)sm.rows;
    k.cols = (uint32_t)sm.cols;
    k.div_tile_cols = make_fast_div(k.tile_cols);
    k.planes = (uint32_t)k.walk.planes;
    k.a = (uint32_t)a;
    dim3 grid;
    IOMX_TRY(plane_grid(sm.tile_rows, sm.tile_cols, k.walk.planes, &k.rows_per_plane, &grid));
    const hipStream_t s = native(stream);
#define IOMX_APPEND(B) hipLaunchKernelGGL((cache_append_kernel<B>), grid, dim3(256), 0, s, k)
    switch (bits) {
        case 2: IOMX_APPEND(2); break;
        case 4: IOMX_APPEND(4); break;
        case 6: IOMX_APPEND(6); break;
        case 8: IOMX_APPEND(8); break;
        case 16: IOMX_APPEND(16); break;
        case 32: IOMX_APPEND(32); break;
        default: IOMX_APPEND(64); break;
    }
#undef IOMX_APPEND
    record_launch("cache_append", grid.x, 256, (uint64_t)k.rows_per_plane * k.planes);
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}

// Structural admission of src/device_ops_embedding.cpp (shape rules of
// include/iom/iom.hpp:188-200).
int iomx_launch_embedding(int dtype, int index_dtype, const iomx_view* table,
                          const iomx_view* indices, const iomx_view* out, uint32_t* status,
                          iomx_stream_t stream) {
    const uint32_t bits = leaf_bits(dtype), ibits = leaf_bits(index_dtype);
    if (!bits || !ibits) return IOMX_ERR_UNSUPPORTED;
    IOMX_TRY(check_view(table, bits));
    IOMX_TRY(check_view(indices, ibits));
    IOMX_TRY(check_view(out, bits));
    if (!status || (reinterpret_cast<uintptr_t>(status) & 3u)) return IOMX_ERR_INVALID;
    if (table->rank != 2 || indices->rank != out->rank) return IOMX_ERR_INVALID;
    const uint32_t rank = out->rank;
    if (!same_leading(indices, out, rank - 2)) return IOMX_ERR_INVALID;
    const Matrix tm = matrix_of(*table), im = matrix_of(*indices), om = matrix_of(*out);
    if (im.rows != 1 || om.rows != im.cols || om.cols != tm.cols) return IOMX_ERR_INVALID;
    if (out->base == table->base || out->base == indices->base) return IOMX_ERR_INVALID;
    if (!is_index_leaf(index_dtype)) return IOMX_ERR_UNSUPPORTED;
    if (om.rows > 0xFFFFFFFFull || om.cols > 0xFFFFFFFFull) return IOMX_ERR_OVERFLOW;
    EmbedArgs k = {};
    const iomx_view* v[2] = {indices, out};
    IOMX_TRY(walk_of<2>(v, out->dims, rank - 2, &k.walk));
    k.table = static_cast<const uint8_t*>(table->base) + table->plane_offset * (tm.plane_elems * bits / 8);
    k.indices = static_cast<const uint8_t*>(indices->base);
    k.out = static_cast<uint8_t*>(out->base);
    k.status = status;
    k.index_plane_bytes = im.plane_elems * ibits / 8;
    k.out_plane_bytes = om.plane_elems * bits / 8;
    k.tile_cols = (uint32_t)om.tile_cols;
    k.run = (uint32_t)om.rows;
    k.feats = (uint32_t)om.cols;
    k.div_tile_cols = make_fast_div(k.tile_cols);
    k.planes = (uint32_t)k.walk.planes;
    k.index_signed = is_signed_index(index_dtype);
    k.vocabulary = tm.rows;
    dim3 grid;
    IOMX_TRY(plane_grid(om.tile_rows, om.tile_cols, k.walk.planes, &k.rows_per_plane, &grid));
    const hipStream_t s = native(stream);
    hipLaunchKernelGGL(store_word_kernel, dim3(1), dim3(1), 0, s, status, 0u);
#define IOMX_EMBED_I(B)                                                                          \
    switch (ibits) {                                                                             \
        case 2: hipLaunchKernelGGL((embedding_kernel<B, 2>), grid, dim3(256), 0, s, k); break;   \
        case 4: hipLaunchKernelGGL((embedding_kernel<B, 4>), grid, dim3(256), 0, s, k); break;   \
        case 8: hipLaunchKernelGGL((embedding_kernel<B, 8>), grid, dim3(256), 0, s, k); break;   \
        case 16: hipLaunchKernelGGL((embedding_kernel<B, 16>), grid, dim3(256), 0, s, k); break; \
        case 32: hipLaunchKernelGGL((embedding_kernel<B, 32>), grid, dim3(256), 0, s, k); break; \
        default: hipLaunchKernelGGL((embedding_kernel<B, 64>), grid, dim3(256), 0, s, k); break; \
    }
    switch (bits) {
        case 2: IOMX_EMBED_I(2); break;
        case 4: IOMX_EMBED_I(4); break;
        case 6: IOMX_EMBED_I(6); break;
        case 8: IOMX_EMBED_I(8); break;
        case 16: IOMX_EMBED_I(16); break;
        case 32: IOMX_EMBED_I(32); break;
        default: IOMX_EMBED_I(64); break;
    }
#undef IOMX_EMBED_I
    record_launch("embedding", grid.x, 256, (uint64_t)k.rows_per_plane * k.planes);
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}

// Admission of src/device_ops_neural.cpp:241-362.
int iomx_launch_rope(int dtype, const iomx_view* x, const iomx_view* out, uint64_t a, double theta,
                     iomx_stream_t stream) {
    const uint32_t bits = leaf_bits(dtype);
    if (!bits) return IOMX_ERR_UNSUPPORTED;
    IOMX_TRY(check_view(x, bits));
    IOMX_TRY(check_view(out, bits));
    if (x->rank < 3 || x->rank != out->rank) return IOMX_ERR_INVALID;
    if (!same_leading(x, out, x->rank)) return IOMX_ERR_INVALID;
    const Matrix m = matrix_of(*x);
    if (m.cols % 2 != 0) return IOMX_ERR_INVALID;
    uint64_t last;
    if (add_overflows(a, m.rows - 1, &last)) return IOMX_ERR_OVERFLOW;
    if (last > (1ull << 24)) return IOMX_ERR_INVALID;   // positions stay exact in binary32
    if (out->base == x->base) return IOMX_ERR_INVALID;
    if (!(theta >= 1.0) || theta > 3.4028234663852886e38) return IOMX_ERR_INVALID;
    if (!is_float_leaf(dtype)) return IOMX_ERR_UNSUPPORTED;
    if (m.cols > 0xFFFFFFFFull) return IOMX_ERR_OVERFLOW;
    RopeArgs k = {};
    const iomx_view* v[2] = {x, out};
    IOMX_TRY(walk_of<2>(v, x->dims, x->rank - 2, &k.walk));
    k.x = static_cast<const uint8_t*>(x->base);
    k.out = static_cast<uint8_t*>(out->base);
    k.plane_bytes = m.plane_elems * bits / 8;
    k.rows = (uint32_t)m.rows;
    k.width = (uint32_t)m.cols;
    k.half = k.width / 2;
    k.tile_cols = (uint32_t)m.tile_cols;
    const bool aligned = k.half % kTile == 0;
    k.col_tiles = aligned ? k.half / kTile : k.tile_cols;
    k.div_col_tiles = make_fast_div(k.col_tiles);
    k.planes = (uint32_t)k.walk.planes;
    k.a = (uint32_t)a;
    k.theta = theta;
    dim3 grid;
    IOMX_TRY(plane_grid(m.tile_rows, k.col_tiles, k.walk.planes, &k.lanes_per_plane, &grid));
    grid.y = planes_in_grid(k.lanes_per_plane, k.walk.planes);
    const bool single_row = aligned && k.rows == 1;
    if (single_row) {
        // 16 lanes = 16 planes of one pair tile
        const uint64_t lanes = ((k.walk.planes + kTile - 1) / kTile) * k.col_tiles * kTile;
        if (lanes > 0x7FFFFF00ull * 256) return IOMX_ERR_OVERFLOW;
        grid = dim3((uint32_t)((lanes + 255) / 256), 1, 1);
    }
    const hipStream_t s = native(stream);
    switch (dtype) {
        case DT_F4_E2M1: launch_rope<DT_F4_E2M1, float>(k, aligned, grid, s); break;
        case DT_F6_E2M3: launch_rope<DT_F6_E2M3, float>(k, aligned, grid, s); break;
        case DT_F6_E3M2: launch_rope<DT_F6_E3M2, float>(k, aligned, grid, s); break;
        case DT_F8_E4M3FN: launch_rope<DT_F8_E4M3FN, float>(k, aligned, grid, s); break;
        case DT_F8_E5M2: launch_rope<DT_F8_E5M2, float>(k, aligned, grid, s); break;
        case DT_F16: launch_rope<DT_F16, float>(k, aligned, grid, s); break;
        case DT_BF16: launch_rope<DT_BF16, float>(k, aligned, grid, s); break;
        case DT_F32: launch_rope<DT_F32, float>(k, aligned, grid, s); break;
        default: launch_rope<DT_F64, double>(k, aligned, grid, s); break;
    }
    record_launch(single_row ? "rope_row" : aligned ? "rope_pairs" : "rope_general", grid.x, 256,
                  (uint64_t)k.lanes_per_plane * k.planes);
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}

}  // extern "C"
