// Elementwise operations on tiled, plane-strided, broadcast views:
// ADD / SUB / MUL over the integers of 8 to 64 bits, F16, BF16, F32 and F64; SiLU
// and SiLU*up over the four floating ones; same-spec copy.  (The 2/4/6-bit leaves
// and the 8-bit floats run on the tile-row kernels.)  Kernel families, selected on
// the host:
//
//   *_planes        every operand either covers whole 16x16-tiled planes
//                   (FULL) or is a [.,1,F] row vector broadcast over rows
//                   (ROWVEC); no padding.  Each lane moves 128-bit chunks of a
//                   contiguous plane range: loads and stores are fully
//                   coalesced, the plane index math runs on the scalar unit.
//   *_general       anything else: tile padding, column broadcast, scalars.
//                   One lane owns one 16-byte piece of one logical row and
//                   masks the tail.
//
// Both read every input of a chunk before storing it, so an input that is the
// exact alias of the output is safe without staging.
#include "iomx_arith.hpp"

namespace iomx {

// Operand shapes relative to the result plane: whole planes, a [.,1,F] row vector,
// a [.,R,1] column vector, a [.,1,1] scalar (the last two on the padded kernel only).
enum { MODE_FULL = 0, MODE_ROWVEC = 1, MODE_COLVEC = 2, MODE_SCALAR = 3 };

// Work decomposition of the streaming kernel: a result plane (z) is cut into
// segments (y) of seg_chunks 128-bit chunks, and a wave takes 64 consecutive
// chunks of one segment (x).  With whole-plane operands only, the segment is the
// plane (or every plane at once when the selection is dense).  With a row-vector
// operand the segment is one tile-row band, so the vector chunk a lane needs
// follows from its position in the segment by bit operations alone.
struct BinaryArgs {
    const uint8_t* src[2];
    uint8_t* out;
    uint64_t seg_chunks;
    uint32_t segments;        // per plane
    uint32_t planes;
    uint64_t plane_bytes[3];  // bytes of one owner plane
    PlaneWalk<3> walk;        // 0 lhs, 1 rhs, 2 out
};

struct GeneralArgs {
    const uint8_t* src[2];
    uint8_t* out;
    PlaneWalk<3> walk;
    uint64_t plane_elems[3];
    uint64_t rows, cols;          // result matrix
    uint64_t tile_cols[3];        // per operand
    uint64_t pieces_per_row;      // 16-byte pieces covering one padded row
    uint64_t total_pieces;
    uint32_t brow[2], bcol[2];
};


// One element replicated over a chunk, and the first `valid` elements of a chunk
// stored one by one.
template <int BYTES>
__device__ __forceinline__ u32x4 splat_element(const uint8_t* p) {
    if constexpr (BYTES == 8) {
        const u32x2 e = *reinterpret_cast<const u32x2*>(p);
        return u32x4{e.x, e.y, e.x, e.y};
    } else {
        uint32_t word;
        if constexpr (BYTES == 1) word = *p * 0x01010101u;
        else if constexpr (BYTES == 2) word = *reinterpret_cast<const uint16_t*>(p) * 0x00010001u;
        else word = *reinterpret_cast<const uint32_t*>(p);
        return u32x4{word, word, word, word};
    }
}

template <int BYTES>
__device__ __forceinline__ void store_elements(uint8_t* dst, u32x4 r, uint32_t valid) {
    const uint32_t words[4] = {r.x, r.y, r.z, r.w};
    for (uint32_t e = 0; e < valid; ++e) {
        if constexpr (BYTES == 1) dst[e] = (uint8_t)(words[e >> 2] >> ((e & 3) * 8));
        else if constexpr (BYTES == 2) reinterpret_cast<uint16_t*>(dst)[e] = (uint16_t)(words[e >> 1] >> ((e & 1) * 16));
        else if constexpr (BYTES == 4) reinterpret_cast<uint32_t*>(dst)[e] = words[e];
        else *reinterpret_cast<u32x2*>(dst + e * 8) = u32x2{words[2 * e], words[2 * e + 1]};
    }
}

template <int DT>
struct Leaf {
    static constexpr uint32_t kBytes = class_bytes(DT);
    static constexpr uint32_t kPerChunk = 16 / kBytes;          // elements per 16 bytes
    static constexpr uint32_t kChunksPerRow = kTile / kPerChunk; // per tile row
    static constexpr uint32_t kChunksPerTile = kTileSlots / kPerChunk;
};

// Launch shape of the streaming kernel.  Measured on MI355X with 64..1024 MiB
// operands: one wave per workgroup, one 128-bit chunk per lane and streaming
// (nontemporal) loads and stores sustain the most HBM bandwidth; larger
// workgroups or deeper unrolling lose 3-15 %.
constexpr uint32_t kPlanesBlock = 64;
constexpr uint32_t kBlock = 256;  // general kernel

__device__ __forceinline__ u32x4 load_stream(const uint8_t* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void store_stream(uint8_t* p, u32x4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

// Kernel arguments of the two cheap shapes: everything in one dense range
// (FLAT), or one dense range cut into tile-row bands (BANDS).  A wave of these
// kernels reads its few arguments, forms three addresses and issues its loads:
// nothing else stands before the memory system.
struct FlatArgs {
    const uint8_t* src[2];
    uint8_t* out;
    uint64_t seg_chunks;
    uint32_t segments;
    // one or two leading axes, as byte steps per coordinate (0 = broadcast)
    uint32_t n0, n1;
    uint64_t step0[3], step1[3];
    FastDiv div_segments;
};

// FLAT    one dense range.
// BANDS   one dense range cut into tile-row bands (row-vector operand).
// AXIS1   one strided leading axis on blockIdx.z, segments on blockIdx.y.
// AXIS2   two strided leading axes on blockIdx.z / blockIdx.y, one segment.
// AXIS2B  two strided leading axes with bands: axis 0 on blockIdx.z, (axis 1, band) on
//         blockIdx.y, split by one scalar multiply-shift division.
// PLANES  anything else: the generic plane walk.
enum { SHAPE_FLAT = 0, SHAPE_BANDS = 1, SHAPE_AXIS1 = 2, SHAPE_AXIS2 = 3, SHAPE_PLANES = 4,
       SHAPE_AXIS2B = 5 };

// chunk of row 0 of the lane's tile column, for row-vector operands
template <int DT>
__device__ __forceinline__ uint64_t rowvec_offset(uint64_t cb) {
    using L = Leaf<DT>;
    return ((cb & ~(uint64_t)(L::kChunksPerTile - 1)) | (cb & (L::kChunksPerRow - 1))) * 16;
}

// Whole-plane operands stream past the caches; the row vector is reused by every row and stays
// cached.  (Fetching the vector's 64 bytes a wave through the scalar cache instead, each lane
// selecting its chunk, was built: a bare copy-plus-add probe gained 3 % from it, the real
// operations lost 2-3 %, because the selects are vector instructions and a wave of these kernels
// has about 680 cycles of its SIMD per KiB at full bandwidth -- sixty instructions are a third of
// that.  Four lanes fetching and a cross-lane read per word: +0.5 % on ADD, -1 % on DIV.)
template <int DT, int OP, int LM, int RM>
__device__ __forceinline__ void stream_chunk(const uint8_t* lbase, const uint8_t* rbase,
                                             uint8_t* obase, uint64_t off, uint64_t voff) {
    constexpr int kInputs = Arity<OP>::kInputs;
    u32x4 va, vb = u32x4{0, 0, 0, 0};
    if constexpr (LM == MODE_ROWVEC) va = *reinterpret_cast<const u32x4*>(lbase + voff);
    else va = load_stream(lbase + off);
    if constexpr (kInputs == 2) {
        if constexpr (RM == MODE_ROWVEC) vb = *reinterpret_cast<const u32x4*>(rbase + voff);
        else vb = load_stream(rbase + off);
    }
    store_stream(obase + off, op_chunk<DT, OP>(va, vb));
}

// ONCE: the grid has a workgroup for every (axis 0, axis 1 / band) pair -- no extent above 65535 --
// so nothing loops: the wave reads one batch of arguments, loads, computes, stores and ends.  The
// bandwidth of these kernels is the bytes in flight over the lifetime of a wave, and the loop
// bounds and the grid's extents (fetched for the loops' steps) were two more trips to the scalar
// cache in that lifetime: broadcast ADD BF16 [64,512,2048] 6490 -> 6570 GB/s, DIV 6480 -> 6550.
template <int DT, int OP, int LM, int RM, int SHAPE, bool ONCE>
__global__ __launch_bounds__(kPlanesBlock) void elementwise_stream_kernel(const FlatArgs a) {
    const uint64_t cb = (uint64_t)blockIdx.x * kPlanesBlock + threadIdx.x;
    if (cb >= a.seg_chunks) return;
    // with a row-vector operand and a single segment (a plane of one band) FLAT and AXIS2 still
    // need the lane's chunk of the vector
    constexpr bool kVector = LM == MODE_ROWVEC || RM == MODE_ROWVEC;
    const uint64_t voff = kVector ? rowvec_offset<DT>(cb) : 0;
    // the (z, y) pairs of this workgroup: one, or a stride of the grid's extents
    const uint32_t z_step = ONCE ? 1u : gridDim.z, y_step = ONCE ? 1u : gridDim.y;
    if constexpr (SHAPE == SHAPE_FLAT) {
        stream_chunk<DT, OP, LM, RM>(a.src[0], a.src[1], a.out, cb * 16, voff);
    } else if constexpr (SHAPE == SHAPE_BANDS) {
        const uint32_t y_end = ONCE ? blockIdx.y + 1 : a.segments;
        for (uint32_t y = blockIdx.y; y < y_end; y += y_step)
            stream_chunk<DT, OP, LM, RM>(a.src[0], a.src[1], a.out,
                                         ((uint64_t)y * a.seg_chunks + cb) * 16, voff);
    } else if constexpr (SHAPE == SHAPE_AXIS1) {
        const uint32_t z_end = ONCE ? blockIdx.z + 1 : a.n0, y_end = ONCE ? blockIdx.y + 1 : a.segments;
        for (uint32_t z = blockIdx.z; z < z_end; z += z_step)
            for (uint32_t y = blockIdx.y; y < y_end; y += y_step)
                stream_chunk<DT, OP, LM, RM>(a.src[0] + z * a.step0[0], a.src[1] + z * a.step0[1],
                                             a.out + z * a.step0[2],
                                             ((uint64_t)y * a.seg_chunks + cb) * 16, voff);
    } else if constexpr (SHAPE == SHAPE_AXIS2B) {
        const uint32_t z_end = ONCE ? blockIdx.z + 1 : a.n0, y_end = ONCE ? blockIdx.y + 1 : a.n1 * a.segments;
        for (uint32_t z = blockIdx.z; z < z_end; z += z_step)
            for (uint32_t y = blockIdx.y; y < y_end; y += y_step) {
                const uint32_t j = fast_div(y, a.div_segments);  // segments >= 2 here
                const uint32_t seg = y - j * a.segments;
                stream_chunk<DT, OP, LM, RM>(a.src[0] + z * a.step0[0] + j * a.step1[0],
                                             a.src[1] + z * a.step0[1] + j * a.step1[1],
                                             a.out + z * a.step0[2] + j * a.step1[2],
                                             ((uint64_t)seg * a.seg_chunks + cb) * 16, voff);
            }
    } else {
        const uint32_t z_end = ONCE ? blockIdx.z + 1 : a.n0, y_end = ONCE ? blockIdx.y + 1 : a.n1;
        for (uint32_t z = blockIdx.z; z < z_end; z += z_step)
            for (uint32_t y = blockIdx.y; y < y_end; y += y_step)
                stream_chunk<DT, OP, LM, RM>(a.src[0] + z * a.step0[0] + y * a.step1[0],
                                             a.src[1] + z * a.step0[1] + y * a.step1[1],
                                             a.out + z * a.step0[2] + y * a.step1[2], cb * 16, voff);
    }
}

template <int DT, int OP, int LM, int RM>
__global__ __launch_bounds__(kPlanesBlock) void elementwise_planes_kernel(const BinaryArgs a) {
    const uint64_t cb = (uint64_t)blockIdx.x * kPlanesBlock + threadIdx.x;
    if (cb >= a.seg_chunks) return;
    const uint64_t voff = rowvec_offset<DT>(cb);
    for (uint32_t z = blockIdx.z; z < a.planes; z += gridDim.z) {
        uint64_t plane[3];
        walk_planes(a.walk, z, plane);
        const uint8_t* lbase = a.src[0] + plane[0] * a.plane_bytes[0];
        const uint8_t* rbase = a.src[1] + plane[1] * a.plane_bytes[1];
        uint8_t* obase = a.out + plane[2] * a.plane_bytes[2];
        for (uint32_t y = blockIdx.y; y < a.segments; y += gridDim.y)
            stream_chunk<DT, OP, LM, RM>(lbase, rbase, obase,
                                         ((uint64_t)y * a.seg_chunks + cb) * 16, voff);
    }
}

// Tile padding (rows or columns that are not multiples of 16): the padded planes
// are still whole contiguous bands, so the lanes keep the streaming kernel's chunk
// mapping; a lane drops out where its chunk lies in the padding (columns: once per
// launch; rows: in the last band of a plane) and stores element by element where a
// chunk straddles the last logical column.  Padding is neither loaded nor stored.
struct PaddedArgs {
    BinaryArgs b;             // seg_chunks = chunks of one band, segments = bands walked per plane
    uint32_t rows, cols;
    uint32_t tile_rows;       // bands of one plane
    FastDiv div_tile_rows;
    uint32_t folded;          // segments run over several planes: band = segment mod tile_rows
    uint32_t row_shift;       // lanes cover 2^row_shift rows of a band (4: all sixteen)
    uint64_t lanes;           // lanes of one band: tile columns * 2^row_shift rows * chunks per row
};

// One operand's chunk: streamed for whole planes; for the broadcast shapes the one
// element a lane needs (row 0 of its tile column is a whole chunk; a column vector
// holds element (row, 0) of tile (band, 0); a scalar is element 0 of its plane),
// replicated across the chunk.
template <int DT, int MODE>
__device__ __forceinline__ u32x4 padded_operand(const uint8_t* base, uint64_t off, uint64_t voff,
                                                uint32_t band, uint32_t row) {
    using L = Leaf<DT>;
    if constexpr (MODE == MODE_FULL) {
        return load_stream(base + off);
    } else if constexpr (MODE == MODE_ROWVEC) {
        return *reinterpret_cast<const u32x4*>(base + voff);
    } else {
        const uint64_t slot = MODE == MODE_COLVEC ? (uint64_t)band * kTileSlots + row * kTile : 0;
        return splat_element<L::kBytes>(base + slot * L::kBytes);
    }
}

template <int DT, int OP, int LM, int RM>
__global__ __launch_bounds__(kPlanesBlock) void elementwise_padded_kernel(const PaddedArgs a) {
    using L = Leaf<DT>;
    constexpr int kInputs = Arity<OP>::kInputs;
    // A plane of one band with eight rows or fewer (a decode step's [.,1,F] planes) gets lanes for
    // the first 1, 2, 4 or 8 rows of its tiles only: the others would drop out at once, fifteen
    // lanes in sixteen for a single row.  row_shift = 4 is the plain chunk order of the band.
    const uint64_t lane_id = (uint64_t)blockIdx.x * kPlanesBlock + threadIdx.x;
    if (lane_id >= a.lanes) return;
    constexpr uint32_t kRowBits = L::kChunksPerRow == 1 ? 0 : L::kChunksPerRow == 2 ? 1 : L::kChunksPerRow == 4 ? 2 : 3;
    static_assert((1u << kRowBits) == L::kChunksPerRow, "chunks per row: a power of two up to eight");
    const uint32_t piece = (uint32_t)lane_id & (L::kChunksPerRow - 1);
    const uint32_t row = (uint32_t)(lane_id >> kRowBits) & ((1u << a.row_shift) - 1);
    const uint64_t tile = lane_id >> (kRowBits + a.row_shift);
    const uint64_t cb = tile * L::kChunksPerTile + row * L::kChunksPerRow + piece;
    const uint32_t col0 = (uint32_t)tile * kTile + piece * L::kPerChunk;
    if (col0 >= a.cols) return;
    const uint32_t left = a.cols - col0;
    const uint32_t valid = left < L::kPerChunk ? left : L::kPerChunk;
    const uint64_t voff = rowvec_offset<DT>(cb);
    for (uint32_t z = blockIdx.z; z < a.b.planes; z += gridDim.z) {
        uint64_t plane[3];
        walk_planes(a.b.walk, z, plane);
        const uint8_t* lbase = a.b.src[0] + plane[0] * a.b.plane_bytes[0];
        const uint8_t* rbase = a.b.src[1] + plane[1] * a.b.plane_bytes[1];
        uint8_t* obase = a.b.out + plane[2] * a.b.plane_bytes[2];
        for (uint32_t y = blockIdx.y; y < a.b.segments; y += gridDim.y) {
            uint32_t tr = y;
            if (a.folded && a.tile_rows > 1) tr = y - fast_div(y, a.div_tile_rows) * a.tile_rows;
            else if (a.folded) tr = 0;
            if (tr * kTile + row >= a.rows) continue;
            const uint64_t off = ((uint64_t)y * a.b.seg_chunks + cb) * 16;
            const u32x4 va = padded_operand<DT, LM>(lbase, off, voff, tr, row);
            u32x4 vb = u32x4{0, 0, 0, 0};
            if constexpr (kInputs == 2) vb = padded_operand<DT, RM>(rbase, off, voff, tr, row);
            const u32x4 r = op_chunk<DT, OP>(va, vb);
            uint8_t* dst = obase + off;
            if (valid == L::kPerChunk) {
                store_stream(dst, r);
            } else {
                store_elements<L::kBytes>(dst, r, valid);
            }
        }
    }
}

// One lane = one 16-byte piece (kPerChunk elements) of one logical result row.
template <int DT, int OP>
__global__ __launch_bounds__(kBlock) void elementwise_general_kernel(const GeneralArgs a) {
    using L = Leaf<DT>;
    constexpr int kInputs = Arity<OP>::kInputs;
    for (uint64_t g = blockIdx.x * (uint64_t)kBlock + threadIdx.x; g < a.total_pieces;
         g += (uint64_t)gridDim.x * kBlock) {
        const uint64_t piece = g % a.pieces_per_row;
        const uint64_t rowlin = g / a.pieces_per_row;
        const uint64_t row = rowlin % a.rows;
        const uint32_t p = (uint32_t)(rowlin / a.rows);
        const uint64_t col0 = piece * L::kPerChunk;
        if (col0 >= a.cols) continue;
        const uint32_t valid = (a.cols - col0) < L::kPerChunk ? (uint32_t)(a.cols - col0) : L::kPerChunk;
        uint64_t plane[3];
        walk_planes(a.walk, p, plane);
        u32x4 v[2] = {u32x4{0, 0, 0, 0}, u32x4{0, 0, 0, 0}};
#pragma unroll
        for (int k = 0; k < kInputs; ++k) {
            const uint64_t r = a.brow[k] ? 0 : row;
            const uint64_t c = a.bcol[k] ? 0 : col0;
            const uint64_t slot = plane[k] * a.plane_elems[k]
                    + ((r / kTile) * a.tile_cols[k] + c / kTile) * kTileSlots
                    + (r % kTile) * kTile + c % kTile;
            if (a.bcol[k]) {
                v[k] = splat_element<L::kBytes>(a.src[k] + slot * L::kBytes);
            } else {
                v[k] = *reinterpret_cast<const u32x4*>(a.src[k] + slot * L::kBytes);
            }
        }
        const u32x4 r = op_chunk<DT, OP>(v[0], v[1]);
        const uint64_t oslot = plane[2] * a.plane_elems[2]
                + ((row / kTile) * a.tile_cols[2] + col0 / kTile) * kTileSlots
                + (row % kTile) * kTile + col0 % kTile;
        uint8_t* dst = a.out + oslot * L::kBytes;
        if (valid == L::kPerChunk) {
            *reinterpret_cast<u32x4*>(dst) = r;
        } else {
            store_elements<L::kBytes>(dst, r, valid);
        }
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

namespace {

struct Snapshot {
    uint64_t stride[kMaxLead];
    bool brow, bcol, broadcasts;
};

// Result-aligned plane strides with 0 on broadcast axes
// (src/device_ops_binary.cpp:61-100).
Snapshot snapshot(const iomx_view& v, const uint64_t* rdims, uint32_t rrank) {
    Snapshot s = {};
    const uint32_t offset = rrank - v.rank;
    s.broadcasts = v.rank != rrank;
    for (uint32_t axis = 0; axis + 2 < rrank; ++axis) {
        if (axis < offset) { s.broadcasts = s.broadcasts || rdims[axis] != 1; continue; }
        const uint32_t src = axis - offset;
        if (v.dims[src] == 1 && rdims[axis] != 1) { s.broadcasts = true; continue; }
        s.stride[axis] = v.plane_strides[src];
    }
    s.brow = v.dims[v.rank - 2] == 1 && rdims[rrank - 2] != 1;
    s.bcol = v.dims[v.rank - 1] == 1 && rdims[rrank - 1] != 1;
    s.broadcasts = s.broadcasts || s.brow || s.bcol;
    return s;
}

bool same_window(const iomx_view& a, const iomx_view& b) {
    if (a.rank != b.rank || a.plane_offset != b.plane_offset) return false;
    for (uint32_t i = 0; i < a.rank; ++i) if (a.dims[i] != b.dims[i]) return false;
    for (uint32_t i = 0; i + 2 < a.rank; ++i)
        if (a.plane_strides[i] != b.plane_strides[i]) return false;
    return true;
}

uint32_t grid_for(uint64_t blocks) {
    // One workgroup per block of work: the hardware dispatcher keeps the access
    // stream in address order; the kernels loop only beyond the grid limit.
    const uint64_t cap = 0x7FFFFFFFull;
    return (uint32_t)(blocks < cap ? blocks : cap);
}

const char* family(int op, bool planes, bool rowvec) {
    const bool unary = op == OP_SILU || op == OP_COPY;
    if (op == OP_SILU) return planes ? "silu_planes" : "silu_general";
    if (op == OP_COPY) return planes ? "copy_planes" : "copy_general";
    if (op == OP_SILU_MUL) return planes ? "silu_mul_planes" : "silu_mul_general";
    (void)unary;
    if (!planes) return "binary_general";
    return rowvec ? "binary_rowvec" : "binary_planes";
}

// The loop-free instance where the grid has a workgroup for every (axis, band) pair; FLAT has
// no loops to begin with.
template <int DT, int OP, int LM, int RM, int SH>
void launch_stream(bool once, dim3 grid3, hipStream_t s, const FlatArgs& fa) {
    if constexpr (SH == SHAPE_FLAT) {
        hipLaunchKernelGGL((elementwise_stream_kernel<DT, OP, LM, RM, SH, true>), grid3, dim3(kPlanesBlock), 0, s, fa);
    } else {
        if (once)
            hipLaunchKernelGGL((elementwise_stream_kernel<DT, OP, LM, RM, SH, true>), grid3, dim3(kPlanesBlock), 0, s, fa);
        else
            hipLaunchKernelGGL((elementwise_stream_kernel<DT, OP, LM, RM, SH, false>), grid3, dim3(kPlanesBlock), 0, s, fa);
    }
}

template <int DT, int OP>
int launch(bool planes, int lm, int rm, const BinaryArgs& pa, const GeneralArgs& ga,
           hipStream_t s) {
    if (planes) {
        const uint64_t gx = (pa.seg_chunks + kPlanesBlock - 1) / kPlanesBlock;
        if (gx > 0x7FFFFFFFull) return IOMX_ERR_OVERFLOW;
        const uint32_t grid = (uint32_t)gx;
        FlatArgs fa = {};
        fa.src[0] = pa.src[0];
        fa.src[1] = pa.src[1];
        fa.out = pa.out;
        fa.seg_chunks = pa.seg_chunks;
        fa.segments = pa.segments;
        int shape = SHAPE_PLANES;
        dim3 grid3((uint32_t)gx, pa.segments < 65535u ? pa.segments : 65535u,
                   pa.planes < 65535u ? pa.planes : 65535u);
        uint64_t y_extent = pa.segments, z_extent = pa.planes;    // what grid3.y and grid3.z stand for
        if (pa.planes == 1 && pa.walk.nlead == 0) {
            shape = pa.segments == 1 ? SHAPE_FLAT : SHAPE_BANDS;
        } else if (pa.walk.nlead == 1 || pa.walk.nlead == 2) {
            shape = pa.walk.nlead == 1 ? SHAPE_AXIS1 : (pa.segments == 1 ? SHAPE_AXIS2 : SHAPE_AXIS2B);
            fa.n0 = pa.walk.dims[0];
            fa.n1 = pa.walk.nlead == 2 ? pa.walk.dims[1] : 1;
            fa.src[0] += pa.walk.offset[0] * pa.plane_bytes[0];
            fa.src[1] += pa.walk.offset[1] * pa.plane_bytes[1];
            fa.out += pa.walk.offset[2] * pa.plane_bytes[2];
            for (int k = 0; k < 3; ++k) {
                fa.step0[k] = pa.walk.stride[k][0] * pa.plane_bytes[k];
                fa.step1[k] = pa.walk.nlead == 2 ? pa.walk.stride[k][1] * pa.plane_bytes[k] : 0;
            }
            z_extent = fa.n0;
            if (shape == SHAPE_AXIS2) {
                grid3 = dim3((uint32_t)gx, fa.n1 < 65535u ? fa.n1 : 65535u, fa.n0 < 65535u ? fa.n0 : 65535u);
                y_extent = fa.n1;
            } else if (shape == SHAPE_AXIS2B) {
                const uint64_t ys = (uint64_t)fa.n1 * pa.segments;
                fa.div_segments = make_fast_div(pa.segments);
                grid3 = dim3((uint32_t)gx, (uint32_t)(ys < 65535u ? ys : 65535u),
                             fa.n0 < 65535u ? fa.n0 : 65535u);
                y_extent = ys;
                if (ys > 0xFFFFFFFFull) shape = SHAPE_PLANES;
            }
            else grid3.z = fa.n0 < 65535u ? fa.n0 : 65535u;
        }
        // a workgroup for every (axis 0, axis 1 / band) pair: the kernel without loops
        const bool once = grid3.y == y_extent && grid3.z == z_extent;
#define IOMX_STREAM(LMV, RMV, SH) launch_stream<DT, OP, LMV, RMV, SH>(once, grid3, s, fa)
#define IOMX_PLANES(LMV, RMV)                                                                   \
    do {                                                                                        \
        if (shape == SHAPE_FLAT) IOMX_STREAM(LMV, RMV, SHAPE_FLAT);                             \
        else if (shape == SHAPE_BANDS) IOMX_STREAM(LMV, RMV, SHAPE_BANDS);                      \
        else if (shape == SHAPE_AXIS1) IOMX_STREAM(LMV, RMV, SHAPE_AXIS1);                      \
        else if (shape == SHAPE_AXIS2) IOMX_STREAM(LMV, RMV, SHAPE_AXIS2);                      \
        else if (shape == SHAPE_AXIS2B) IOMX_STREAM(LMV, RMV, SHAPE_AXIS2B);                    \
        else                                                                                    \
            hipLaunchKernelGGL((elementwise_planes_kernel<DT, OP, LMV, RMV>), grid3,            \
                               dim3(kPlanesBlock), 0, s, pa);                                   \
    } while (0)
        if (lm == MODE_FULL && rm == MODE_FULL) IOMX_PLANES(MODE_FULL, MODE_FULL);
        else if constexpr (is_arithmetic(OP)) {
            if (lm == MODE_FULL) IOMX_PLANES(MODE_FULL, MODE_ROWVEC);
            else IOMX_PLANES(MODE_ROWVEC, MODE_FULL);
        } else {
            return IOMX_ERR_INVALID;
        }
#undef IOMX_PLANES
#undef IOMX_STREAM
        record_launch(family(OP, true, lm != MODE_FULL || rm != MODE_FULL), grid, kPlanesBlock,
                      gx * pa.segments * pa.planes);
    } else {
        const uint64_t blocks = (ga.total_pieces + kBlock - 1) / kBlock;
        const uint32_t grid = grid_for(blocks);
        hipLaunchKernelGGL((elementwise_general_kernel<DT, OP>), dim3(grid), dim3(kBlock), 0, s, ga);
        record_launch(family(OP, false, false), grid, kBlock, ga.total_pieces);
    }
    return IOMX_OK;
}

template <int DT>
int dispatch(int op, bool planes, int lm, int rm, const BinaryArgs& pa, const GeneralArgs& ga,
             hipStream_t s) {
    switch (op) {
        case IOMX_OP_ADD: return launch<DT, IOMX_OP_ADD>(planes, lm, rm, pa, ga, s);
        case IOMX_OP_MUL: return launch<DT, IOMX_OP_MUL>(planes, lm, rm, pa, ga, s);
        case IOMX_OP_SUB: return launch<DT, IOMX_OP_SUB>(planes, lm, rm, pa, ga, s);
        case OP_COPY: return launch<DT, OP_COPY>(planes, lm, rm, pa, ga, s);
        default: break;
    }
    if constexpr (is_float_class(DT)) {
        if (op == IOMX_OP_DIV) return launch<DT, IOMX_OP_DIV>(planes, lm, rm, pa, ga, s);
        if (op == OP_SILU) return launch<DT, OP_SILU>(planes, lm, rm, pa, ga, s);
        if (op == OP_SILU_MUL) return launch<DT, OP_SILU_MUL>(planes, lm, rm, pa, ga, s);
    }
    return IOMX_ERR_UNSUPPORTED;
}

template <int DT, int OP>
int launch_padded(int lm, int rm, const PaddedArgs& pa, hipStream_t s) {
    const uint64_t gx = (pa.lanes + kPlanesBlock - 1) / kPlanesBlock;
    if (gx > 0x7FFFFFFFull) return IOMX_ERR_OVERFLOW;
    const dim3 grid((uint32_t)gx, pa.b.segments < 65535u ? pa.b.segments : 65535u,
                    pa.b.planes < 65535u ? pa.b.planes : 65535u);
#define IOMX_PADDED(LMV, RMV)                                                                  \
    hipLaunchKernelGGL((elementwise_padded_kernel<DT, OP, LMV, RMV>), grid, dim3(kPlanesBlock), 0, s, pa)
    if (lm == MODE_FULL && rm == MODE_FULL) IOMX_PADDED(MODE_FULL, MODE_FULL);
    else if constexpr (is_arithmetic(OP)) {
        if (lm == MODE_FULL && rm == MODE_ROWVEC) IOMX_PADDED(MODE_FULL, MODE_ROWVEC);
        else if (lm == MODE_FULL && rm == MODE_COLVEC) IOMX_PADDED(MODE_FULL, MODE_COLVEC);
        else if (lm == MODE_FULL && rm == MODE_SCALAR) IOMX_PADDED(MODE_FULL, MODE_SCALAR);
        else if (lm == MODE_ROWVEC && rm == MODE_FULL) IOMX_PADDED(MODE_ROWVEC, MODE_FULL);
        else if (lm == MODE_COLVEC && rm == MODE_FULL) IOMX_PADDED(MODE_COLVEC, MODE_FULL);
        else if (lm == MODE_SCALAR && rm == MODE_FULL) IOMX_PADDED(MODE_SCALAR, MODE_FULL);
        else return IOMX_ERR_INVALID;
    } else {
        return IOMX_ERR_INVALID;
    }
#undef IOMX_PADDED
    const char* name = OP == OP_SILU ? "silu_padded" : OP == OP_COPY ? "copy_padded"
            : OP == OP_SILU_MUL ? "silu_mul_padded" : "binary_padded";
    record_launch(name, (uint32_t)gx, kPlanesBlock, gx * pa.b.segments * pa.b.planes);
    return IOMX_OK;
}

template <int DT>
int dispatch_padded(int op, int lm, int rm, const PaddedArgs& pa, hipStream_t s) {
    switch (op) {
        case IOMX_OP_ADD: return launch_padded<DT, IOMX_OP_ADD>(lm, rm, pa, s);
        case IOMX_OP_MUL: return launch_padded<DT, IOMX_OP_MUL>(lm, rm, pa, s);
        case IOMX_OP_SUB: return launch_padded<DT, IOMX_OP_SUB>(lm, rm, pa, s);
        case OP_COPY: return launch_padded<DT, OP_COPY>(lm, rm, pa, s);
        default: break;
    }
    if constexpr (is_float_class(DT)) {
        if (op == IOMX_OP_DIV) return launch_padded<DT, IOMX_OP_DIV>(lm, rm, pa, s);
        if (op == OP_SILU) return launch_padded<DT, OP_SILU>(lm, rm, pa, s);
        if (op == OP_SILU_MUL) return launch_padded<DT, OP_SILU_MUL>(lm, rm, pa, s);
    }
    return IOMX_ERR_UNSUPPORTED;
}

// Shared admission + planning of every elementwise operation.  `rhs` is null
// for the one-input operations.
enum AliasPolicy { ALIAS_NONE, ALIAS_EXACT, ALIAS_ANY };

int run(int op, int dtype, const iomx_view* lhs, const iomx_view* rhs, const iomx_view* out,
        AliasPolicy alias, iomx_stream_t stream) {
    const uint32_t bits = leaf_bits(dtype);
    if (!bits) return IOMX_ERR_UNSUPPORTED;
    IOMX_TRY(check_view(lhs, bits));
    if (rhs) IOMX_TRY(check_view(rhs, bits));
    IOMX_TRY(check_view(out, bits));
    const bool unary = rhs == nullptr;
    if (unary) rhs = lhs;

    // right-aligned broadcast and exact output shape (src/device_ops_binary.cpp:121-143)
    const uint32_t rank = lhs->rank > rhs->rank ? lhs->rank : rhs->rank;
    uint64_t rdims[8];
    for (uint32_t i = 0; i < rank; ++i) {
        const uint64_t l = i < rank - lhs->rank ? 1 : lhs->dims[i - (rank - lhs->rank)];
        const uint64_t r = i < rank - rhs->rank ? 1 : rhs->dims[i - (rank - rhs->rank)];
        if (l != r && l != 1 && r != 1) return IOMX_ERR_INVALID;
        rdims[i] = l > r ? l : r;
    }
    if (out->rank != rank) return IOMX_ERR_INVALID;
    for (uint32_t i = 0; i < rank; ++i) if (out->dims[i] != rdims[i]) return IOMX_ERR_INVALID;

    const iomx_view* v[3] = {lhs, rhs, out};
    Snapshot snap[3];
    for (int k = 0; k < 3; ++k) snap[k] = snapshot(*v[k], rdims, rank);
    // alias rule (src/device_ops_binary.cpp:152-169)
    for (int k = 0; k < 2; ++k) {
        if (v[k]->base != out->base || alias == ALIAS_ANY) continue;
        if (alias == ALIAS_NONE || snap[k].broadcasts || !same_window(*v[k], *out))
            return IOMX_ERR_INVALID;
    }
    // division is defined on the floating leaves only, refused after the shape and alias
    // checks (src/device_ops_binary.cpp:170-176)
    if (op == IOMX_OP_DIV && (dtype < IOMX_DT_F4_E2M1 || dtype == IOMX_DT_F8_E8M0))
        return IOMX_ERR_UNSUPPORTED;

    Matrix m[3];
    for (int k = 0; k < 3; ++k) m[k] = matrix_of(*v[k]);
    uint64_t strides[3][kMaxLead];
    uint64_t offsets[3];
    for (int k = 0; k < 3; ++k) {
        std::memcpy(strides[k], snap[k].stride, sizeof(strides[k]));
        offsets[k] = v[k]->plane_offset;
    }
    PlaneWalk<3> walk;
    IOMX_TRY(build_walk<3>(rank - 2, rdims, strides, offsets, &walk));

    const uint64_t rows = rdims[rank - 2], cols = rdims[rank - 1];
    const bool no_pad = rows % kTile == 0 && cols % kTile == 0;
    int mode[2] = {MODE_FULL, MODE_FULL};
    for (int k = 0; k < 2; ++k) {
        if (!snap[k].brow && !snap[k].bcol) mode[k] = MODE_FULL;
        else if (snap[k].brow && !snap[k].bcol) mode[k] = MODE_ROWVEC;
        else if (!snap[k].brow && snap[k].bcol) mode[k] = MODE_COLVEC;
        else mode[k] = MODE_SCALAR;
    }
    // the chunk-mapped kernels take at most one operand that is not whole planes
    bool modes_ok = mode[0] == MODE_FULL || mode[1] == MODE_FULL;
    if (!is_arithmetic(op) && (mode[0] != MODE_FULL || mode[1] != MODE_FULL)) modes_ok = false;
    const bool lean_modes = mode[0] <= MODE_ROWVEC && mode[1] <= MODE_ROWVEC;
    bool planes_ok = modes_ok && lean_modes && no_pad;

    // A copy of whole planes is a move of bytes whatever the leaf.  Everything else
    // outside the four streaming leaves goes to the tile-row kernels.
    const bool byte_copy = op == OP_COPY && planes_ok;
    // kernel class: integers by width, floats by leaf; a copy moves raw bits of its width
    int cls;
    if (op == OP_COPY) {
        cls = bits == 8 ? IOMX_DT_I8 : bits == 16 ? IOMX_DT_I16 : bits == 32 ? IOMX_DT_I32
                : bits == 64 ? IOMX_DT_I64 : -1;
    } else {
        switch (dtype) {
            case IOMX_DT_I8: case IOMX_DT_U8: cls = IOMX_DT_I8; break;
            case IOMX_DT_I16: case IOMX_DT_U16: cls = IOMX_DT_I16; break;
            case IOMX_DT_I32: case IOMX_DT_U32: cls = IOMX_DT_I32; break;
            case IOMX_DT_I64: case IOMX_DT_U64: cls = IOMX_DT_I64; break;
            case IOMX_DT_F16: case IOMX_DT_BF16: case IOMX_DT_F32: case IOMX_DT_F64: cls = dtype; break;
            default: cls = -1; break;
        }
    }
    const bool streaming = cls >= 0;
    if (!byte_copy && !streaming) {
        RowsRequest r = {};
        r.src[0] = static_cast<const uint8_t*>(lhs->base);
        r.src[1] = static_cast<const uint8_t*>(rhs->base);
        r.out = static_cast<uint8_t*>(out->base);
        r.walk = walk;
        for (int k = 0; k < 3; ++k) r.m[k] = m[k];
        for (int k = 0; k < 2; ++k) { r.brow[k] = snap[k].brow; r.bcol[k] = snap[k].bcol; }
        IOMX_TRY(launch_rows(op, dtype, r, native(stream)));
        IOMX_HIP(hipGetLastError());
        return IOMX_OK;
    }
    // byte counts below: exact for every width since a plane holds a multiple of 256 slots
    const uint64_t bytes8 = bits;  // bits per element; sizes are formed as elems * bits / 8

    if (modes_ok && (!no_pad || !lean_modes) && rows <= 0xFFFFFFFFull && cols <= 0xFFFFFFFFull) {
        // padded planes, column vectors, scalars: whole bands, chunk validity decided per lane
        PaddedArgs pd = {};
        BinaryArgs& b = pd.b;
        b.src[0] = static_cast<const uint8_t*>(lhs->base);
        b.src[1] = static_cast<const uint8_t*>(rhs->base);
        b.out = static_cast<uint8_t*>(out->base);
        b.walk = walk;
        for (int k = 0; k < 3; ++k) b.plane_bytes[k] = m[k].plane_elems * bytes8 / 8;
        b.seg_chunks = m[2].tile_cols * (kTileSlots * bytes8 / 128);
        uint64_t planes = walk.planes, segments = m[2].tile_rows;
        bool fold = walk.nlead <= 1;
        for (int k = 0; k < 3 && fold; ++k) {
            const bool vec = k < 2 && mode[k] != MODE_FULL;
            if (vec) fold = walk.nlead == 0 || walk.stride[k][0] == 0;
            else fold = walk_is_dense(walk, k);
        }
        if (fold) {
            b.src[0] += offsets[0] * b.plane_bytes[0];
            b.src[1] += offsets[1] * b.plane_bytes[1];
            b.out += offsets[2] * b.plane_bytes[2];
            for (int k = 0; k < 3; ++k) b.walk.offset[k] = 0;
            b.walk.nlead = 0;
            if (mul_overflows(segments, planes, &segments)) return IOMX_ERR_OVERFLOW;
            planes = 1;
            pd.folded = 1;
        }
        if (segments > 0xFFFFFFFFull || planes > 0xFFFFFFFFull || m[2].tile_rows > 0xFFFFFFFFull)
            return IOMX_ERR_OVERFLOW;
        b.segments = (uint32_t)segments;
        b.planes = (uint32_t)planes;
        pd.rows = (uint32_t)rows;
        pd.cols = (uint32_t)cols;
        pd.tile_rows = (uint32_t)m[2].tile_rows;
        pd.div_tile_rows = make_fast_div(pd.tile_rows);
        pd.row_shift = 4;
        if (m[2].tile_rows == 1 && rows <= 8) pd.row_shift = rows <= 1 ? 0 : rows <= 2 ? 1 : rows <= 4 ? 2 : 3;
        pd.lanes = (b.seg_chunks >> 4) << pd.row_shift;
        const hipStream_t ps = native(stream);
        int prc = IOMX_ERR_UNSUPPORTED;
        switch (cls) {
            case IOMX_DT_I8: prc = dispatch_padded<IOMX_DT_I8>(op, mode[0], mode[1], pd, ps); break;
            case IOMX_DT_I16: prc = dispatch_padded<IOMX_DT_I16>(op, mode[0], mode[1], pd, ps); break;
            case IOMX_DT_I32: prc = dispatch_padded<IOMX_DT_I32>(op, mode[0], mode[1], pd, ps); break;
            case IOMX_DT_I64: prc = dispatch_padded<IOMX_DT_I64>(op, mode[0], mode[1], pd, ps); break;
            case IOMX_DT_F16: prc = dispatch_padded<IOMX_DT_F16>(op, mode[0], mode[1], pd, ps); break;
            case IOMX_DT_BF16: prc = dispatch_padded<IOMX_DT_BF16>(op, mode[0], mode[1], pd, ps); break;
            case IOMX_DT_F32: prc = dispatch_padded<IOMX_DT_F32>(op, mode[0], mode[1], pd, ps); break;
            default: prc = dispatch_padded<IOMX_DT_F64>(op, mode[0], mode[1], pd, ps); break;
        }
        IOMX_TRY(prc);
        IOMX_HIP(hipGetLastError());
        return IOMX_OK;
    }

    BinaryArgs pa = {};
    GeneralArgs ga = {};
    if (planes_ok) {
        pa.src[0] = static_cast<const uint8_t*>(lhs->base);
        pa.src[1] = static_cast<const uint8_t*>(rhs->base);
        pa.out = static_cast<uint8_t*>(out->base);
        pa.walk = walk;
        for (int k = 0; k < 3; ++k) pa.plane_bytes[k] = m[k].plane_elems * bytes8 / 8;
        const bool rowvec = mode[0] == MODE_ROWVEC || mode[1] == MODE_ROWVEC;
        const uint64_t plane_chunks = m[2].plane_elems * bytes8 / 128;
        const uint64_t band_chunks = m[2].tile_cols * (kTileSlots * bytes8 / 128);
        uint64_t planes = walk.planes;
        uint64_t segments = rowvec ? m[2].tile_rows : 1;
        pa.seg_chunks = rowvec ? band_chunks : plane_chunks;
        // A dense selection on every whole-plane operand (and a row vector shared by
        // all planes) folds the planes into one range.
        bool fold = walk.nlead <= 1;
        for (int k = 0; k < 3 && fold; ++k) {
            const bool vec = k < 2 && mode[k] == MODE_ROWVEC;
            if (vec) fold = walk.nlead == 0 || walk.stride[k][0] == 0;
            else fold = walk_is_dense(walk, k);
        }
        if (fold) {
            pa.src[0] += offsets[0] * pa.plane_bytes[0];
            pa.src[1] += offsets[1] * pa.plane_bytes[1];
            pa.out += offsets[2] * pa.plane_bytes[2];
            for (int k = 0; k < 3; ++k) pa.walk.offset[k] = 0;
            pa.walk.nlead = 0;
            if (rowvec) {
                if (mul_overflows(segments, planes, &segments)) return IOMX_ERR_OVERFLOW;
            } else if (mul_overflows(pa.seg_chunks, planes, &pa.seg_chunks)) {
                return IOMX_ERR_OVERFLOW;
            }
            planes = 1;
        }
        if (segments > 0xFFFFFFFFull || planes > 0xFFFFFFFFull) return IOMX_ERR_OVERFLOW;
        pa.segments = (uint32_t)segments;
        pa.planes = (uint32_t)planes;
    } else {
        ga.src[0] = static_cast<const uint8_t*>(lhs->base);
        ga.src[1] = static_cast<const uint8_t*>(rhs->base);
        ga.out = static_cast<uint8_t*>(out->base);
        ga.walk = walk;
        for (int k = 0; k < 3; ++k) { ga.plane_elems[k] = m[k].plane_elems; ga.tile_cols[k] = m[k].tile_cols; }
        ga.rows = rows;
        ga.cols = cols;
        ga.pieces_per_row = m[2].tile_cols * (kTile * bytes8 / 128);
        for (int k = 0; k < 2; ++k) { ga.brow[k] = snap[k].brow; ga.bcol[k] = snap[k].bcol; }
        uint64_t t;
        if (mul_overflows(walk.planes, rows, &t)) return IOMX_ERR_OVERFLOW;
        if (mul_overflows(t, ga.pieces_per_row, &ga.total_pieces)) return IOMX_ERR_OVERFLOW;
    }

    const hipStream_t s = native(stream);
    int rc;
    // whole planes of any width move as 32-bit words
    if (byte_copy) cls = IOMX_DT_I32;
    switch (cls) {
        case IOMX_DT_I8: rc = dispatch<IOMX_DT_I8>(op, planes_ok, mode[0], mode[1], pa, ga, s); break;
        case IOMX_DT_I16: rc = dispatch<IOMX_DT_I16>(op, planes_ok, mode[0], mode[1], pa, ga, s); break;
        case IOMX_DT_I32: rc = dispatch<IOMX_DT_I32>(op, planes_ok, mode[0], mode[1], pa, ga, s); break;
        case IOMX_DT_I64: rc = dispatch<IOMX_DT_I64>(op, planes_ok, mode[0], mode[1], pa, ga, s); break;
        case IOMX_DT_F16: rc = dispatch<IOMX_DT_F16>(op, planes_ok, mode[0], mode[1], pa, ga, s); break;
        case IOMX_DT_BF16: rc = dispatch<IOMX_DT_BF16>(op, planes_ok, mode[0], mode[1], pa, ga, s); break;
        case IOMX_DT_F32: rc = dispatch<IOMX_DT_F32>(op, planes_ok, mode[0], mode[1], pa, ga, s); break;
        default: rc = dispatch<IOMX_DT_F64>(op, planes_ok, mode[0], mode[1], pa, ga, s); break;
    }
    IOMX_TRY(rc);
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}

bool same_shape(const iomx_view* a, const iomx_view* b) {
    if (!a || !b || a->rank != b->rank || a->rank > 8) return false;
    for (uint32_t i = 0; i < a->rank; ++i) if (a->dims[i] != b->dims[i]) return false;
    return true;
}

}  // namespace
}  // namespace iomx

using namespace iomx;

extern "C" {

int iomx_launch_binary(int op, int dtype, const iomx_view* lhs, const iomx_view* rhs,
                       const iomx_view* out, iomx_stream_t stream) {
    if (!is_arithmetic(op)) return IOMX_ERR_INVALID;
    if (!rhs) return IOMX_ERR_INVALID;
    return run(op, dtype, lhs, rhs, out, ALIAS_EXACT, stream);
}

// Admission of src/device_ops_neural.cpp:363-438: identical shapes, a floating
// leaf, and an output that shares no storage with the input.
int iomx_launch_silu(int dtype, const iomx_view* x, const iomx_view* y, iomx_stream_t stream) {
    // the nine floating leaves (F8_E8M0 is a scale, not a number)
    if (dtype < 13 || dtype > 22 || dtype == 18) return IOMX_ERR_UNSUPPORTED;
    if (!same_shape(x, y)) return IOMX_ERR_INVALID;
    return run(OP_SILU, dtype, x, nullptr, y, ALIAS_NONE, stream);
}

int iomx_launch_silu_mul(int dtype, const iomx_view* gate, const iomx_view* up,
                         const iomx_view* y, iomx_stream_t stream) {
    if (dtype != IOMX_DT_BF16 && dtype != IOMX_DT_F32 && dtype != IOMX_DT_F16 && dtype != IOMX_DT_F64)
        return IOMX_ERR_UNSUPPORTED;
    if (!same_shape(gate, y) || !same_shape(up, y)) return IOMX_ERR_INVALID;
    return run(OP_SILU_MUL, dtype, gate, up, y, ALIAS_EXACT, stream);
}

// src/device_ops_copy.cpp:9-52: identical specs; an identical window is a
// no-op.  Distinct windows of one owner are accepted as the reference accepts
// them; windows that overlap partially have no defined result.
int iomx_launch_copy(int dtype, const iomx_view* src, const iomx_view* dst, iomx_stream_t stream) {
    if (!leaf_bits(dtype)) return IOMX_ERR_UNSUPPORTED;
    if (!same_shape(src, dst)) return IOMX_ERR_INVALID;
    if (src->base == dst->base && same_window(*src, *dst)) {
        IOMX_TRY(check_view(src, leaf_bits(dtype)));
        record_launch("copy_noop", 0, 0, 0);
        return IOMX_OK;
    }
    return run(OP_COPY, dtype, src, nullptr, dst, ALIAS_ANY, stream);
}

}  // extern "C"
