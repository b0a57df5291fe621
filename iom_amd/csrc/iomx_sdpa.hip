// Causal grouped-query attention, BF16: q [B..,Hq,R,D], k and v [B..,Hkv,C,D],
// out [B..,R,Hq*D]; row r sees tokens t < min(L, a+r+1).
//
//   sdpa_pack       V of the visible prefix, transposed into matrix-core operand
//                   fragments in the caller's workspace (subnormals flushed to signed
//                   zero, zeros past L and past D), K copied tile for tile with the
//                   same flush, and a flag raised when a V value of the prefix is
//                   infinite or NaN.
//   sdpa_mfma       one wave = one head x 16 rows.  Pass 1 forms the scores
//                   (K tile x Q tile on the matrix cores, binary32) and the row's
//                   maximum and sum of exponentials; pass 2 forms them again, turns
//                   them into the normalised probability rounded once to BF16, and
//                   multiplies by the packed V fragments (binary32 accumulation),
//                   one BF16 rounding at the store.  Scores never leave registers.
//   sdpa_decode     few rows per KV head (a decode step): one launch, no workspace.
//   sdpa_rows       the scalar recurrence in the reference's order (one wave per
//                   row: sequential sums over features and over tokens): the path
//                   for head sizes the fragments do not cover.  sdpa_mfma forms its
//                   rows the same way where the flag of their KV head is up: a
//                   masked probability is +0, and +0 times an infinite V of a token
//                   the row must not see would poison the row on the matrix cores.
#include <atomic>
#include <type_traits>
#include <utility>

#include "iomx_mfma.hpp"

namespace iomx {

struct SdpaArgs {
    const uint8_t* q;
    const uint8_t* k;
    const uint8_t* v;
    uint8_t* out;
    PlaneWalk<4> walk;          // 0 q, 1 k, 2 v, 3 out: the shared leading tuple
    uint64_t q_plane_bytes, kv_plane_bytes, out_plane_bytes;
    uint64_t q_head_stride, k_head_stride, v_head_stride;   // owner planes per head
    uint32_t Hq, Hkv, grouping, R, C, D, a, L;
    uint32_t d_tiles, out_tile_cols, kv_tile_rows;
    uint32_t planes, groups;    // leading planes; 32-token groups of the prefix
    uint32_t plane0;            // first plane of this launch
    float* decode_stats;        // sdpa_decode in shares: [pair][share][row][8] statistics
    float* decode_sums;         // ... and [pair][share][row][D] partial output sums
    uint32_t kept_wave_bytes;   // sdpa_decode with kept scores: bytes of a wave's area in dynamic LDS
    uint8_t* packed_v;          // [plane][kv head][group][d tile] fragments of 1 KiB
    uint8_t* packed_k;          // [plane][kv head][token tile][d tile] flushed tiles (null: not packed)
    uint32_t* flags;            // [plane][kv head][pack split]: nonzero = that part of the V prefix
                                // holds an infinity or NaN
    uint32_t pack_splits;       // workgroups sharing the fragments of one KV head
    float scale;                // sqrtf(D)
    float inv_scale;            // 1 / scale, rounded
    uint32_t scale_pow2;        // scale is a power of two: the product with inv_scale is the quotient
    float exp_scale;            // log2(e) / scale, rounded once: exp((dot - max) / scale) = 2^((dot - max) * exp_scale)
};

constexpr uint32_t kTileBytes = 512, kRowBytes = 32, kFrag = 1024;

// Subnormal operands of the matrix stages become zeros of the same sign
// (src/cpu/sdpa.cpp:57-60), two BF16 per word.
__device__ __forceinline__ uint32_t daz2(uint32_t w) {
    // bit 15 of a half of `normal` is set where that half's exponent field is not zero (the field
    // sits in bits 7..14, so adding 0x7FFF carries into bit 15 exactly then and never past it)
    const uint32_t normal = ((w & 0x7F807F80u) + 0x7FFF7FFFu) & 0x80008000u;
    // 0x7FFF under every such bit, and the sign bits always
    return w & ((normal - (normal >> 15)) | 0x80008000u);
}
__device__ __forceinline__ bf16x8_t daz8(u32x4 v) {
    return __builtin_bit_cast(bf16x8_t, u32x4{daz2(v[0]), daz2(v[1]), daz2(v[2]), daz2(v[3])});
}
// The smaller exponent field of each half, over a run of words: zero in a half exactly if some
// word of the run has a zero exponent field there (a zero or a subnormal).
typedef unsigned short u16x2_min_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t least_exponents(uint32_t least, uint32_t w) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2_min_t, least),
                                                                  __builtin_bit_cast(u16x2_min_t, w & 0x7F807F80u)));
}
// N operand words with their subnormals flushed.  Two instructions a word find out whether any
// lane of the wave holds a zero exponent field at all; only then the six-instruction flush runs
// (operands of a model hold neither zeros nor subnormals as a rule).
template <int N>
__device__ __forceinline__ void daz_words(u32x4 (&v)[N]) {
    uint32_t least = 0xFFFFFFFFu;
#pragma unroll
    for (int i = 0; i < N; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) least = least_exponents(least, v[i][j]);
    if (__any((least & 0xFFFFu) == 0u || (least >> 16) == 0u)) {
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = u32x4{daz2(v[i][0]), daz2(v[i][1]), daz2(v[i][2]), daz2(v[i][3])};
    }
}
__device__ __forceinline__ float daz_bf16(uint32_t h) {
    return as_f32(((h & 0x7F80u) ? h : (h & 0x8000u)) << 16);
}

// LDS reads written out as instructions (see the shared-ring walk of sdpa_mfma): the 32-bit LDS
// address of a pointer into a __shared__ array, one 128-bit read at a constant offset from it,
// and the wait that makes every such read issued so far usable.
__device__ __forceinline__ uint32_t lds_address(const void* shared) {
    return (uint32_t)(uintptr_t)(lptr_t)shared;
}
template <int OFFSET>
__device__ __forceinline__ u32x4 lds_read_b128(uint32_t address) {
    static_assert(OFFSET >= 0 && OFFSET < 65536 && OFFSET % 16 == 0, "immediate offset of ds_read_b128");
    u32x4 value;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(value) : "v"(address), "n"(OFFSET));
    return value;
}
__device__ __forceinline__ void lds_reads_landed() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// one 32-bit word, waited for
__device__ __forceinline__ uint32_t lds_read_b32(uint32_t address) {
    uint32_t value;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(value) : "v"(address) : "memory");
    return value;
}

// One workgroup packs a share of the fragments of one KV head of one plane and writes
// that share's flag word (every word is written on every call, so the workspace needs
// no clearing).
//
// V fragment (group g, d tile dt) holds, for lane (d = l%16, kg = l/16), the eight
// values V[32g + 4kg + j][16dt + d] (j < 4) and V[32g + 16 + 4kg + j][16dt + d]: the
// token order in which a lane of sdpa_mfma holds its probabilities.  K is copied tile
// for tile (token tiles 2g and 2g+1, d tile dt) with the same flush, rows past the
// prefix and columns past D as zeros, so that the many waves that meet a K tile do not
// each flush it again.
__global__ __launch_bounds__(256) void sdpa_pack_kernel(const SdpaArgs a) {
    // a wave's staging area for the transposition: the two 16x16 V tiles of a fragment as they lie
    __shared__ __attribute__((aligned(16))) uint8_t turn[4][2 * kTileBytes];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t l16 = lane & 15u, kg = lane >> 4;
    const uint32_t hkv = blockIdx.x / a.pack_splits, split = blockIdx.x - hkv * a.pack_splits;
    const uint32_t frags = a.groups * a.d_tiles;
    // lane = 16-byte chunk of the two tiles of a group: tile lane/32, row (lane%32)/2, half lane%2
    const uint32_t in_tile = lane >> 5, r = (lane & 31u) >> 1, half = lane & 1u;
    // the transposing read: the sixteen lanes of quarter kg supply the 8-byte pieces of rows
    // 4kg .. 4kg+3 (lane 4i + c: row 4kg + i, columns 4c .. 4c+3), and lane (kg, d) receives
    // column d of those four rows -- tokens 4kg .. 4kg+3 of feature d, the fragment's order
    const uint32_t turn_at = lds_address(&turn[wave][0]) + (4 * kg + (l16 >> 2)) * kRowBytes + (l16 & 3u) * 8;
    for (uint32_t p = blockIdx.y; p < a.planes; p += gridDim.y) {
        uint64_t plane[4];
        walk_planes(a.walk, p, plane);
        const uint8_t* vb = a.v + (plane[2] + (uint64_t)hkv * a.v_head_stride) * a.kv_plane_bytes;
        const uint8_t* kb = a.k + (plane[1] + (uint64_t)hkv * a.k_head_stride) * a.kv_plane_bytes;
        const uint64_t head_frags = ((uint64_t)p * a.Hkv + hkv) * frags;
        bool special = false;
        for (uint32_t frag = split * 4 + wave; frag < frags; frag += 4 * a.pack_splits) {
            const uint32_t g = frag / a.d_tiles, dt = frag - g * a.d_tiles;
            const uint32_t tt = 2 * g + in_tile;
            const uint64_t tile_row = ((uint64_t)tt * a.d_tiles + dt) * kTileBytes + r * kRowBytes;
            // both operands are requested before anything is stored (a load is not moved across a
            // store it cannot be told apart from: that would be two trips to memory in a row);
            // tokens past the prefix and columns past D are zeros
            u32x4 vw = {0, 0, 0, 0}, kw = {0, 0, 0, 0};
            if (tt * kTile + r < a.L) {
                vw = load_k8_bits(vb + tile_row, half * 8, dt * kTile + half * 8, a.D);
                if (a.packed_k) kw = load_k8_bits(kb + tile_row, half * 8, dt * kTile + half * 8, a.D);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
                special = special || (vw[i] & 0x7F80u) == 0x7F80u || (vw[i] & 0x7F800000u) == 0x7F800000u;
            vw = u32x4{daz2(vw[0]), daz2(vw[1]), daz2(vw[2]), daz2(vw[3])};
            *reinterpret_cast<u32x4*>(&turn[wave][lane * 16]) = vw;
            u32x2 lo, hi;
            // (the "memory" clobber keeps the store above ahead of the reads; a wave's LDS
            // instructions execute in order, so the reads see all sixty-four lanes' pieces)
            asm volatile("ds_read_b64_tr_b16 %0, %2\n\t"
                         "ds_read_b64_tr_b16 %1, %2 offset:512\n\t"
                         "s_waitcnt lgkmcnt(0)"
                         : "=&v"(lo), "=&v"(hi) : "v"(turn_at) : "memory");
            *reinterpret_cast<u32x4*>(a.packed_v + (head_frags + frag) * kFrag + lane * 16) = u32x4{lo.x, lo.y, hi.x, hi.y};
            if (a.packed_k) {
                kw = u32x4{daz2(kw[0]), daz2(kw[1]), daz2(kw[2]), daz2(kw[3])};
                *reinterpret_cast<u32x4*>(a.packed_k + ((head_frags * 2 + (uint64_t)tt * a.d_tiles + dt) * kTileBytes)
                                          + (lane & 31u) * 16) = kw;
            }
        }
        const int any = __syncthreads_or(special ? 1 : 0);
        if (threadIdx.x == 0) a.flags[((uint64_t)p * a.Hkv + hkv) * a.pack_splits + split] = any ? 1u : 0u;
    }
}

// Running maximum and sum of exp(score - maximum) over the finite scores of a row,
// and what the special rows need (docs/BACKEND_CONTRACT/scaled-dot-product-attention.md:
// "Formed-score special values").
struct RowStats {
    float m, sum;
    uint32_t pinf;
    bool nan, finite;
    __device__ __forceinline__ void merge(float m2, float sum2, uint32_t pinf2, bool nan2, bool finite2) {
        const float mm = m > m2 ? m : m2;
        if (mm == -__builtin_inff()) sum = 0.0f;
        else sum = sum * __expf(m - mm) + sum2 * __expf(m2 - mm);
        m = mm;
        pinf += pinf2;
        nan = nan || nan2;
        finite = finite || finite2;
    }
};

// Orders the LDS traffic of one wave: its lanes run in lockstep and its LDS operations
// complete in order.
__device__ __forceinline__ void wave_sync() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
}

// One row of one head in the reference's own order of operations (src/cpu/sdpa.cpp:132-336):
// sequential sums over features and over tokens, by one wave; pbuf = 64 floats of LDS of this wave.
__device__ __forceinline__ void sdpa_reference_row(const SdpaArgs& a, uint32_t p, uint32_t hkv, uint32_t head,
                                                uint32_t row, uint32_t lane, float* pbuf) {
    const float inf = __builtin_inff();
    const uint32_t reach = a.a + row + 1;
    const uint32_t vis = reach < a.L ? reach : a.L;
    uint64_t plane[4];
    walk_planes(a.walk, p, plane);
    const uint8_t* qb = a.q + (plane[0] + (uint64_t)head * a.q_head_stride) * a.q_plane_bytes
            + (uint64_t)(row >> 4) * a.d_tiles * kTileBytes + (row & 15u) * kRowBytes;
    const uint8_t* kb = a.k + (plane[1] + (uint64_t)hkv * a.k_head_stride) * a.kv_plane_bytes;
    const uint8_t* vb = a.v + (plane[2] + (uint64_t)hkv * a.v_head_stride) * a.kv_plane_bytes;
    auto element = [&](const uint8_t* row_base, uint32_t d) {
        return daz_bf16(*reinterpret_cast<const uint16_t*>(row_base + (uint64_t)(d >> 4) * kTileBytes + (d & 15u) * 2));
    };
    auto score = [&](uint32_t t) {
        const uint8_t* kr = kb + (uint64_t)(t >> 4) * a.d_tiles * kTileBytes + (t & 15u) * kRowBytes;
        float dot = 0.0f;
        for (uint32_t d = 0; d < a.D; ++d) dot = dot + element(qb, d) * element(kr, d);   // products are exact
        return dot / a.scale;
    };
    // classes and maximum
    float m = -inf;
    uint32_t pinf = 0;
    bool nan = false, not_ninf = false;
    for (uint32_t t = lane; t < vis; t += 64) {
        const float s = score(t);
        nan = nan || s != s;
        pinf += s == inf ? 1u : 0u;
        not_ninf = not_ninf || s != -inf;
        if (s > m) m = s;
    }
#pragma unroll
    for (int off = 1; off < 64; off *= 2) {
        // every lane takes part in every exchange (no short-circuit around a shuffle)
        const float m2 = __shfl_xor(m, off);
        const uint32_t p2 = __shfl_xor(pinf, off);
        const int n2 = __shfl_xor((int)nan, off), f2 = __shfl_xor((int)not_ninf, off);
        m = m2 > m ? m2 : m;
        pinf += p2;
        nan = nan || n2 != 0;
        not_ninf = not_ninf || f2 != 0;
    }
    uint8_t* ob = a.out + plane[3] * a.out_plane_bytes
            + (uint64_t)(row >> 4) * a.out_tile_cols * kTileBytes + (row & 15u) * kRowBytes;
    auto store = [&](uint32_t d, uint32_t bits) {
        const uint32_t col = head * a.D + d;
        *reinterpret_cast<uint16_t*>(ob + (uint64_t)(col >> 4) * kTileBytes + (col & 15u) * 2) = (uint16_t)bits;
    };
    if (nan || !not_ninf) {
        for (uint32_t d = lane; d < a.D; d += 64) store(d, 0x7FC0u);
        return;
    }
    // sum of exponentials in token order
    float sum = 0.0f;
    if (pinf == 0) {
        for (uint32_t t0 = 0; t0 < vis; t0 += 64) {
            const uint32_t t = t0 + lane;
            float e = 0.0f;
            if (t < vis) {
                const float s = score(t);
                if (s != -inf) e = expf(s - m);
            }
            for (int i = 0; i < 64; ++i) sum = sum + __shfl(e, i);     // adding +0 changes nothing
        }
    }
    const float pinf_p = pinf ? 1.0f / (float)pinf : 0.0f;
    // out = sum over tokens of P * V, features over lanes (up to 256)
    float result[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t t0 = 0; t0 < vis; t0 += 64) {
        const uint32_t t = t0 + lane;
        float pr = 0.0f;
        if (t < vis) {
            const float s = score(t);
            if (pinf) pr = s == inf ? pinf_p : 0.0f;
            else if (s != -inf) pr = expf(s - m) / sum;
        }
        wave_sync();                                   // the previous chunk's readers are done
        pbuf[lane] = daz_bf16(bf16_rne_sw(as_u32(pr)));
        wave_sync();
        const uint32_t n = vis - t0 < 64 ? vis - t0 : 64;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t d = lane + 64 * c;
            if (d >= a.D) continue;
            for (uint32_t i = 0; i < n; ++i) {
                const uint32_t tt = t0 + i;
                const uint8_t* vr = vb + (uint64_t)(tt >> 4) * a.d_tiles * kTileBytes + (tt & 15u) * kRowBytes;
                result[c] = result[c] + pbuf[i] * element(vr, d);             // products are exact
            }
        }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t d = lane + 64 * c;
        if (d >= a.D) continue;
        float val = result[c];
        if (val == 0.0f) val = 0.0f;
        store(d, bf16_rne_sw(as_u32(val)));
    }
}

// KV heads of plane p whose V prefix holds an infinity or NaN (any share's flag up)
// The flag words of one (plane, KV head), a word per lane (there are 64 pack splits at most), as one
// vector load that stays in flight with whatever the caller requests next; any lane's result
// non-zero = the flag is up.  (Read one after the other through the scalar cache they were a chain
// of up to 64 dependent loads at the head of every workgroup.)
__device__ __forceinline__ uint32_t sdpa_flag_words(const SdpaArgs& a, uint32_t p, uint32_t hkv, uint32_t lane) {
    const uint64_t pair = (uint64_t)p * a.Hkv + hkv;
    uint32_t up = 0;
    for (uint32_t i = lane; i < a.pack_splits; i += 64) up |= a.flags[pair * a.pack_splits + i];
    return up;
}

// MODE 0: a workgroup of four waves = four heads of one row tile, each wave walks
// all visible tokens (prefill: many row tiles, K and V shared through the caches).
// MODE 1: one head, the 4 or 8 waves share out the 32-token groups and meet in LDS (few
// rows against a long prefix would otherwise be one wave's chain of dependent loads).
// MODE 2: MODE 0 for four heads that share one KV head (grouping a multiple of 4) and D = 64
// or 128: the workgroup brings every K and V group into LDS once, with the direct loader,
// three groups deep, and its four waves read their operands from there -- the vector
// memory pipeline of the CU, which bounds MODE 0, carries a quarter of the bytes.
// MODE 3: the same ring for any grouping: the four waves are four consecutive row tiles of one
// head (the workgroup walks the groups of its last tile; a wave sits out the groups past its own).
// FULLD: D is a multiple of 32, no operand load needs a guard against the columns past D.
//
// Both passes exist twice.  The plain one assumes what almost every row satisfies -- no
// NaN and no +infinity among its visible scores and at least one finite score -- and
// spends two or three vector instructions per score; its sum of exponentials turns NaN
// or its maximum infinite exactly when the assumption fails, and then the whole tile
// repeats both passes with the bookkeeping of the special rows
// (docs/BACKEND_CONTRACT/scaled-dot-product-attention.md: "Formed-score special values").
// waves of a workgroup: four heads, or as many token shares as LDS holds partial outputs for
constexpr int sdpa_waves(int dt16, int mode) { return mode != 1 ? 4 : dt16 <= 4 ? 8 : 4; }

typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
// two finite floats to two BF16, round to nearest even (the conversion instruction of gfx950)
__device__ __forceinline__ uint32_t cvt_bf16x2(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}

// max(a, b, c) as the one instruction (the compiler's own maximum first makes every operand a
// quiet NaN or itself, an instruction apiece; the scores here come out of multiplications and
// selects and need none of that).
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Results of the matrix instructions that are about to be read by instructions the compiler
// cannot see (max3 / max2 above).  A vector instruction may read a register the matrix pipeline
// writes only a fixed number of issue slots after the matrix instruction; the compiler counts those
// slots for the instructions it schedules and knows nothing of the ones inside an asm statement,
// so the wait is written out here (sixteen slots cover the eight passes of a 16x16x32 product),
// tied to the values so that it stays between their producers and their readers.
__device__ __forceinline__ void settle_matrix_results(f32x4_t (&s)[2]) {
    asm volatile("s_nop 7\n\ts_nop 7" : "+v"(s[0]), "+v"(s[1]));
}

__device__ __forceinline__ float max2(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

// Eight products e[i] * scale, those below the smallest normal number as zeros, rounded to BF16
// (nearest even) and packed in order.  The multiplications run with the mode register's binary32
// denormal field on "flush", which makes the zeroing part of the multiplication instead of a
// compare and a select per product; the field is set back before anything else executes.
__device__ __forceinline__ u32x4 scaled_flushed_bf16x8(const float (&e)[8], float scale) {
    float p[8];
    asm volatile(
            "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 4, 2), 0\n\t"
            "v_mul_f32 %0, %8, %16\n\t"
            "v_mul_f32 %1, %9, %16\n\t"
            "v_mul_f32 %2, %10, %16\n\t"
            "v_mul_f32 %3, %11, %16\n\t"
            "v_mul_f32 %4, %12, %16\n\t"
            "v_mul_f32 %5, %13, %16\n\t"
            "v_mul_f32 %6, %14, %16\n\t"
            "v_mul_f32 %7, %15, %16\n\t"
            "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 4, 2), 3"
            : "=&v"(p[0]), "=&v"(p[1]), "=&v"(p[2]), "=&v"(p[3]), "=&v"(p[4]), "=&v"(p[5]), "=&v"(p[6]), "=&v"(p[7])
            : "v"(e[0]), "v"(e[1]), "v"(e[2]), "v"(e[3]), "v"(e[4]), "v"(e[5]), "v"(e[6]), "v"(e[7]), "v"(scale));
    return u32x4{cvt_bf16x2(p[0], p[1]), cvt_bf16x2(p[2], p[3]), cvt_bf16x2(p[4], p[5]), cvt_bf16x2(p[6], p[7])};
}

template <class F, int... I>
__device__ __forceinline__ void static_for_each(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_each(f, std::make_integer_sequence<int, N>{});
}

template <int DT16, int MODE, bool FULLD>
__global__ __launch_bounds__(sdpa_waves(DT16, MODE) * 64) __attribute__((amdgpu_waves_per_eu(MODE != 1 ? 3 : 2)))
void sdpa_mfma_bf16_kernel(const SdpaArgs a) {
    // MODE 0 hides the K latency with many waves per SIMD; the token-sharing mode has few
    // waves and requests the next group ahead instead
    constexpr bool AHEAD = MODE == 1;
    constexpr bool SPLIT = MODE == 1;
    constexpr bool SHARE = MODE == 2 || MODE == 3;
    static_assert(!SHARE || (DT16 % 4 == 0 && FULLD), "shared groups: whole KiB chunks per wave");
    constexpr uint32_t kStage = 2 * DT16 * 1024;           // K group + V group
    __shared__ __attribute__((aligned(16))) uint8_t kv_ring[SHARE ? 3 * kStage : 16];
    constexpr int NW = sdpa_waves(DT16, MODE);
    constexpr int D32 = (DT16 + 1) / 2;
    // FULLD: D is a multiple of 32, i.e. exactly DT16 whole tiles -- a constant to the compiler
    const uint32_t head_dim = FULLD ? (uint32_t)DT16 * kTile : a.D;
    const uint32_t d_tiles = FULLD ? (uint32_t)DT16 : a.d_tiles;
    constexpr float kLog2e = 1.44269504088896340736f;
    // stands in for a maximum of -infinity (nothing seen yet) in exponent arguments
    constexpr float kFloor = -1.0e30f;
    __shared__ float wave_stats[NW][16][5];
    __shared__ f32x4_t wave_out[SPLIT ? NW - 1 : 1][SPLIT ? DT16 : 1][64];
    // raised by a wave whose rows need the passes of the special rows (the waves that share a ring
    // decide together); cleared here, and the barriers of pass 1 lie between this and its first use
    __shared__ uint32_t special_rows;
    if (SHARE && threadIdx.x == 0) special_rows = 0;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t l16 = lane & 15u, kg = lane >> 4;
    // which (head, row) the lane's tile row is
    const uint32_t head = (MODE == 1 || MODE == 3) ? blockIdx.x : blockIdx.x * 4 + wave;
    if (MODE == 0 && head >= a.Hq) return;          // no barrier on this path (MODE 2: Hq is a multiple of 4)
    const uint32_t hkv = head / a.grouping;
    // grid = (heads, planes, row tiles): the row tiles with the longest prefixes are dispatched
    // first, for every head and plane, and the short ones fill the end of the launch
    const uint32_t slab = gridDim.z - 1 - blockIdx.z;
    const uint32_t first_row = (MODE == 3 ? slab * 4 + wave : slab) * kTile, row = first_row + l16;
    const bool ghost = MODE == 3 && first_row >= a.R;       // a wave past the last row tile: barriers only
    const uint32_t last_row = first_row + 15 < a.R ? first_row + 15 : a.R - 1;
    const bool row_ok = row < a.R;
    const uint32_t qrow = row_ok ? row : a.R - 1;
    const uint32_t reach = a.a + row + 1, reach_min = a.a + first_row + 1, reach_max = a.a + last_row + 1;
    const uint32_t vis = row_ok ? (reach < a.L ? reach : a.L) : 0;     // tokens this lane's row sees
    const uint32_t vis_max = reach_max < a.L ? reach_max : a.L;        // ... and the tile's last row
    const uint32_t groups = ghost ? 0 : (vis_max + 31) / 32;
    // the groups the workgroup brings in: those of its last row tile (MODE 3), else the wave's own
    const uint32_t slab_last = slab * 64 + 63 < a.R ? slab * 64 + 63 : a.R - 1;
    const uint32_t slab_reach = a.a + slab_last + 1;
    const uint32_t ring_groups = MODE == 3 ? ((slab_reach < a.L ? slab_reach : a.L) + 31) / 32 : groups;
    // groups that every row of the tile sees whole need no mask
    const uint32_t full_groups = (reach_min < a.L ? reach_min : a.L) / 32;
    // the plain passes let the rows past R mirror the last row (their results are dropped)
    const uint32_t vis_plain = row_ok ? vis : vis_max;
    const uint32_t g_first = SPLIT ? wave : 0, g_step = SPLIT ? NW : 1;
    const uint32_t c0 = (kg & 1u) * 8u;
    const float inf = __builtin_inff();
    // one plane per grid layer (a loop over planes here would make the compiler keep every
    // lane offset of the body alive across it, far beyond the register file)
    {
        const uint32_t p = a.plane0 + blockIdx.y;
        // requested now, looked at once Q and the first K groups are on their way too
        const uint32_t flag_words = sdpa_flag_words(a, p, hkv, lane);
        uint64_t plane[4];
        walk_planes(a.walk, p, plane);
        const uint8_t* qb = a.q + (plane[0] + (uint64_t)head * a.q_head_stride) * a.q_plane_bytes;
        // wave-uniform bases and 32-bit lane offsets: the packed region of one KV head is far
        // below 4 GiB, and 64-bit addresses per load would cost the registers of a whole wave slot
        const uint8_t* vf = a.packed_v + (((uint64_t)p * a.Hkv + hkv) * a.groups) * d_tiles * kFrag;
        const uint32_t vf_lane = lane * 16;
        const uint8_t* kp = a.packed_k + (((uint64_t)p * a.Hkv + hkv) * a.groups * 2) * d_tiles * kTileBytes;
        const uint32_t kp_lane = l16 * kRowBytes + c0 * 2;
        // One direct load of a wave's share of the K group (and of the V group) g into ring stage buf:
        // wave w brings in KiB chunks w, w+4, .. ; lane i fetches 16-byte piece i of a chunk, and the
        // loader puts it at chunk + 16*i, so a group lies in LDS as it lies in the packed regions.
        auto issue = [&](auto with_v, uint32_t g, uint32_t buf) {
            if constexpr (SHARE) {
                const uint32_t gg = g < ring_groups ? g : ring_groups - 1;   // past the end: a valid group again, unused
                uint8_t* stage = kv_ring + buf * kStage;
#pragma unroll
                for (int j = 0; j < DT16 / 4; ++j) {
                    const uint32_t chunk = wave + 4 * j;
                    __builtin_amdgcn_global_load_lds((gptr_t)(kp + ((gg * DT16 + chunk) * kFrag + vf_lane)),
                                                     (lptr_t)(stage + chunk * kFrag), 16, 0, 0);
                    if constexpr (decltype(with_v)::value)
                        __builtin_amdgcn_global_load_lds((gptr_t)(vf + ((gg * DT16 + chunk) * kFrag + vf_lane)),
                                                         (lptr_t)(stage + (DT16 + chunk) * kFrag), 16, 0, 0);
                }
            }
        };
        // the first two K groups of pass 1 are on their way while Q is fetched and flushed
        if (SHARE && ring_groups != 0) {
            issue(std::false_type{}, 0, 0);
            issue(std::false_type{}, 1, 1);
        }
        // the row tile of Q, flushed, as the B operand of every score tile
        u32x4 q_bits[D32];
#pragma unroll
        for (int c = 0; c < D32; ++c) {
            const uint32_t i0 = 32 * c + 8 * kg, tile = 2 * c + (kg >> 1);
            q_bits[c] = u32x4{0, 0, 0, 0};
            if (FULLD || i0 < a.D)
                q_bits[c] = load_k8_bits(qb + ((uint64_t)(qrow >> 4) * d_tiles + tile) * kTileBytes
                                            + (qrow & 15u) * kRowBytes, c0, i0, head_dim);
        }
        if (__any(flag_words != 0)) {
            // V of this KV head holds an infinity or NaN.  A masked probability is +0, and on the
            // matrix cores +0 times an infinite V of a token the row must not see would poison
            // the row: these rows are formed in the reference's order instead.  (All waves of a
            // workgroup that meets at barriers share the KV head and leave together; the K groups
            // requested above land in the ring, which nothing reads on this path.)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            float* pbuf = &wave_stats[wave][0][0];
            for (uint32_t r = SPLIT ? wave : 0; r < kTile; r += SPLIT ? NW : 1)
                if (first_row + r < a.R) sdpa_reference_row(a, p, hkv, head, first_row + r, lane, pbuf);
            return;
        }
        bf16x8_t qf[D32];
#pragma unroll
        for (int c = 0; c < D32; ++c) qf[c] = daz8(q_bits[c]);
        // K of the 32 tokens of group g, from the flushed copy: two 16-token tiles, lane
        // (token l16, features 8*kg..); tokens past the prefix and columns past D are zeros there
        struct KGroup { u32x4 w[2][D32]; };
        auto load_k = [&](uint32_t g, KGroup& kgp) {
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int c = 0; c < D32; ++c) {
                    const uint32_t i0 = 32 * c + 8 * kg, tile = 2 * c + (kg >> 1);
                    kgp.w[half][c] = u32x4{0, 0, 0, 0};
                    if (FULLD || i0 < a.D)
                        kgp.w[half][c] = *reinterpret_cast<const u32x4*>(
                                kp + (((2 * g + half) * d_tiles + tile) * kTileBytes + kp_lane));
                }
        };
        // scores: lane gets tokens 32g + 16*half + 4*kg + j (j < 4) of row l16.  `bare` (the plain
        // passes): the dot products themselves; the division by sqrt(D) is folded into the constant
        // of the passes' exponent argument (see there).  Otherwise (the passes of the special rows,
        // whose values are compared and counted as scores): dot / sqrt(D).
        auto scores = [&](const KGroup& kgp, f32x4_t (&s)[2], bool bare) {
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int c = 0; c < D32; ++c)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kgp.w[half][c]), qf[c], acc, 0, 0, 0);
                if (bare) {
                    s[half] = acc;
                    continue;
                }
                // dot / sqrt(D): the product with the reciprocal is the quotient when sqrt(D) is
                // a power of two; otherwise one correction step of the remainder makes it the
                // correctly rounded quotient in all but halfway cases of the last bit
                f32x4_t q = acc * a.inv_scale;
                if (!a.scale_pow2) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float refined = __builtin_fmaf(__builtin_fmaf(-q[j], a.scale, acc[j]), a.inv_scale, q[j]);
                        q[j] = __builtin_fabsf(q[j]) < __builtin_inff() ? refined : q[j];   // inf - inf is not a remainder
                    }
                }
                s[half] = q;
            }
        };
        // the visible groups of this wave, K one group ahead where the mode says so; WITH_V: the
        // V fragments of the group are requested before its scores are formed
        // `primed`: the first two stages of the ring have been requested already
        // `edge` (plain passes): the groups below full_groups get body(.., false_type) and the ones
        // from there on body(.., true_type), which masks -- as two loops over one step, because a
        // mask under a branch inside one loop costs a register copy per score in every group.  The
        // special rows' passes do their own bookkeeping per score and take one loop.
        auto walk_groups = [&](auto with_v, bool bare, bool primed, auto edge, auto&& body) {
            constexpr bool WITH_V = decltype(with_v)::value;
            constexpr bool EDGE = decltype(edge)::value;
            if constexpr (SHARE) {
                constexpr int LPS = (WITH_V ? 2 : 1) * (DT16 / 4);        // direct loads per wave and stage
                if (!primed) {
                    issue(with_v, 0, 0);
                    issue(with_v, 1, 1);
                }
                uint32_t buf = 0;
                auto step = [&](uint32_t g, auto masked) {
                    // the own loads of group g have landed; past the barrier everybody's have, and
                    // nobody reads the buffer of group g-1 any more: it takes group g+2
                    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPS) : "memory");
                    __builtin_amdgcn_s_barrier();
                    issue(with_v, g + 2, buf == 0 ? 2 : buf - 1);
                    const uint8_t* stage = kv_ring + buf * kStage;
                    buf = buf == 2 ? 0 : buf + 1;
                    if (MODE == 3 && g >= groups) return;                 // uniform: past this wave's own tile
                    // The operands come out of LDS through ds_read instructions the compiler does
                    // not see as such.  Left to itself it waits, before every LDS read, for every
                    // direct load still in flight (it cannot tell the ring's stages apart), which
                    // is a full trip to the cache per group, every group; the counted wait and the
                    // barrier above already say exactly what this stage needs.
                    KGroup cur;
                    const uint32_t k_at = lds_address(stage + ((kg >> 1) * kTileBytes + kp_lane));
                    static_for<2 * D32>([&](auto index) {
                        constexpr int half = decltype(index)::value / D32, c = decltype(index)::value % D32;
                        cur.w[half][c] = lds_read_b128<(half * DT16 + 2 * c) * (int)kTileBytes>(k_at);
                    });
                    u32x4 vfr[WITH_V ? DT16 : 1];
                    if constexpr (WITH_V) {
                        const uint32_t v_at = lds_address(stage + vf_lane);
                        static_for<DT16>([&](auto index) {
                            constexpr int dt = decltype(index)::value;
                            vfr[dt] = lds_read_b128<(DT16 + dt) * (int)kFrag>(v_at);
                        });
                    }
                    lds_reads_landed();
#pragma unroll
                    for (int half = 0; half < 2; ++half)
#pragma unroll
                        for (int c = 0; c < D32; ++c) asm volatile("" : "+v"(cur.w[half][c]));
                    if constexpr (WITH_V) {
#pragma unroll
                        for (int dt = 0; dt < DT16; ++dt) asm volatile("" : "+v"(vfr[dt]));
                    }
                    f32x4_t s[2];
                    scores(cur, s, bare);
                    body(g, s, vfr, masked);
                };
                uint32_t g = 0;
                if constexpr (EDGE) {
                    const uint32_t whole = full_groups < ring_groups ? full_groups : ring_groups;
#pragma unroll 1
                    for (; g < whole; ++g) step(g, std::false_type{});
                }
#pragma unroll 1
                for (; g < ring_groups; ++g) step(g, std::true_type{});
                // nothing in flight and nobody reading when the next pass (or the next workgroup)
                // takes the ring
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __builtin_amdgcn_s_barrier();
                return;
            }
            KGroup cur, nxt;
            if (AHEAD && g_first < groups) load_k(g_first, cur);
            auto step = [&](uint32_t g, auto masked) {
                if (!AHEAD) load_k(g, cur);
                else if (g + g_step < groups) load_k(g + g_step, nxt);     // the next group is in flight meanwhile
                u32x4 vfr[WITH_V ? DT16 : 1];
                if constexpr (WITH_V) {
#pragma unroll
                    for (int dt = 0; dt < DT16; ++dt)
                        vfr[dt] = *reinterpret_cast<const u32x4*>(vf + ((g * d_tiles + dt) * kFrag + vf_lane));
                }
                f32x4_t s[2];
                scores(cur, s, bare);
                body(g, s, vfr, masked);
                if (AHEAD) cur = nxt;
            };
            uint32_t g = g_first;
            if constexpr (EDGE) {
                const uint32_t whole = full_groups < groups ? full_groups : groups;
#pragma unroll 1
                for (; g < whole; g += g_step) step(g, std::false_type{});
            }
#pragma unroll 1
            for (; g < groups; g += g_step) step(g, std::true_type{});
        };
        // scores of tokens the lane's row must not see become -infinity (plain passes)
        auto mask_group = [&](uint32_t g, f32x4_t (&s)[2]) {
            const int rem = (int)vis_plain - (int)(32 * g + 4 * kg);
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int j = 0; j < 4; ++j) s[half][j] = 16 * half + j < rem ? s[half][j] : -inf;
        };
        // The plain passes work on the dot products themselves: the division by sqrt(D) moves into
        // the constant of the exponent argument, 2^(dot * c - max * c) with c = log2(e) / sqrt(D)
        // rounded once, and the running maximum is a maximum of dot products.  Where sqrt(D) is a
        // power of two that is the same binary32 value as 2^((dot / sqrt(D)) * log2 e - ...) bit for
        // bit (scaling by a power of two commutes with rounding); for the other head sizes the
        // argument differs from the divided form's by a few units of its last place, which is the
        // size of the rounding of dot / sqrt(D) itself and far inside the contract's allowance for
        // a native kernel, and costs three vector instructions per score and pass less than a
        // correctly rounded quotient.
        constexpr bool bare = true;
        const float kls = a.exp_scale;
        // (maximum, sum) of one part of a row joined with another part's
        auto join = [&](float& m, float& sum, float m2, float sum2) {
            const float mm = __builtin_fmaxf(m, m2), base = __builtin_fmaxf(mm, kFloor);
            sum = sum * __builtin_amdgcn_exp2f((__builtin_fmaxf(m, kFloor) - base) * kls)
                + sum2 * __builtin_amdgcn_exp2f((__builtin_fmaxf(m2, kFloor) - base) * kls);
            m = mm;
        };
        auto mma_v = [&](f32x4_t (&o)[DT16], const u32x4 (&vfr)[DT16], const u32x4& pw) {
            const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, pw);
#pragma unroll
            for (int dt = 0; dt < DT16; ++dt)
                o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vfr[dt]), pf, o[dt], 0, 0, 0);
        };

        // ---- plain pass 1: running maximum and sum of exp(score - maximum)
        float pm = -inf, psum = 0.0f;
        walk_groups(std::false_type{}, bare, true, std::true_type{}, [&](uint32_t g, f32x4_t (&s)[2], const u32x4 (&)[1], auto masked) {
            if constexpr (decltype(masked)::value) mask_group(g, s);     // (selects the compiler schedules)
            else settle_matrix_results(s);
            // (the maximum instruction itself: a NaN among its operands is passed over, and the
            // row's sum below turns NaN from that score's exponential all the same)
            const float newm = max3(max3(s[0][0], s[0][1], s[0][2]), max3(s[0][3], s[1][0], s[1][1]),
                                    max3(s[1][2], s[1][3], pm));
            const float base = max2(newm, kFloor);
            psum *= __builtin_amdgcn_exp2f((max2(pm, kFloor) - base) * kls);
            const float nb = -base * kls;
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int j = 0; j < 4; ++j) psum += __builtin_amdgcn_exp2f(__builtin_fmaf(s[half][j], kls, nb));
            pm = newm;
        });
        // the first two groups of pass 2 (K and V) are on their way while the statistics are
        // joined: the ring is free (pass 1 ended at a barrier with nothing in flight).  Should the
        // tile turn out to need the special rows' passes, those request their own first groups
        // over these: the same K bytes into the same places.
        if (SHARE && ring_groups != 0) {
            issue(std::true_type{}, 0, 0);
            issue(std::true_type{}, 1, 1);
        }
#pragma unroll
        for (int off = 16; off <= 32; off *= 2) {
            const float m2 = __shfl_xor(pm, off), s2 = __shfl_xor(psum, off);
            join(pm, psum, m2, s2);
        }
        if (SPLIT) {
            if (kg == 0) {
                wave_stats[wave][l16][0] = pm;
                wave_stats[wave][l16][1] = psum;
            }
            __syncthreads();
            pm = wave_stats[0][l16][0];
            psum = wave_stats[0][l16][1];
#pragma unroll
            for (int w = 1; w < NW; ++w) join(pm, psum, wave_stats[w][l16][0], wave_stats[w][l16][1]);
        }
        // a NaN or +infinity score, or no finite score at all, shows here; every wave of the
        // workgroup holds the same joined values and decides alike
        const bool odd = !ghost && !(psum > 0.0f && psum < inf && pm < inf);
        // (sharing the groups, the four waves also share the decision: they meet at barriers)
        bool plain = !__any(odd);
        if constexpr (SHARE) {
            // (a bare barrier and a read the compiler does not see as one: a fence here, or an LDS
            // read it knows of, would first wait for the groups of pass 2 requested above)
            if (!plain && lane == 0) special_rows = 1;
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            plain = __builtin_amdgcn_readfirstlane(lds_read_b32(lds_address(&special_rows))) == 0;
        }

        f32x4_t o[DT16];
#pragma unroll
        for (int dt = 0; dt < DT16; ++dt) o[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        bool nan_row = false;
        if (plain) {
            // ---- plain pass 2: probabilities, rounded once to BF16 and flushed, times V
            const float inv_sum = 1.0f / psum, nb = -pm * kls;
            walk_groups(std::true_type{}, bare, SHARE, std::true_type{}, [&](uint32_t g, f32x4_t (&s)[2], const u32x4 (&vfr)[DT16], auto masked) {
                if constexpr (decltype(masked)::value) mask_group(g, s);
                float e[8];
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        e[half * 4 + j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[half][j], kls, nb));
                // probabilities below the BF16 normals are zeros as matrix operands
                mma_v(o, vfr, scaled_flushed_bf16x8(e, inv_sum));
            });
        } else {
            // ---- pass 1 with the bookkeeping of the special rows
            RowStats st = {-inf, 0.0f, 0u, false, false};
            walk_groups(std::false_type{}, false, false, std::false_type{}, [&](uint32_t g, f32x4_t (&s)[2], const u32x4 (&)[1], auto) {
                // the finite maximum of the lane's eight scores first, then one rescale; written
                // with selects only (a branch per element would cost more than the arithmetic)
                float local = -inf;
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const bool seen = 32 * g + 16 * half + 4 * kg + j < vis;
                        const float v = s[half][j];
                        st.nan = st.nan | (seen & (v != v));
                        st.pinf += (seen & (v == inf)) ? 1u : 0u;
                        // masked, NaN and infinite scores take no part in the sum
                        s[half][j] = (seen & (__builtin_fabsf(v) < inf)) ? v : -inf;
                        local = __builtin_fmaxf(local, s[half][j]);
                    }
                const float newm = __builtin_fmaxf(st.m, local);
                st.sum = newm == st.m ? st.sum : st.sum * __expf(st.m - newm);   // exp(-inf) = 0
                st.m = newm;
                st.finite = st.finite | (local > -inf);
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        st.sum += s[half][j] == -inf ? 0.0f : __expf(s[half][j] - newm);
            });
#pragma unroll
            for (int off = 16; off <= 32; off *= 2) {
                const float m2 = __shfl_xor(st.m, off), s2 = __shfl_xor(st.sum, off);
                const uint32_t p2 = __shfl_xor(st.pinf, off);
                const int n2 = __shfl_xor((int)st.nan, off), f2 = __shfl_xor((int)st.finite, off);
                st.merge(m2, s2, p2, n2 != 0, f2 != 0);
            }
            if (SPLIT) {
                __syncthreads();                       // the readers of the plain statistics are done
                if (kg == 0) {
                    wave_stats[wave][l16][0] = st.m;
                    wave_stats[wave][l16][1] = st.sum;
                    wave_stats[wave][l16][2] = as_f32(st.pinf);
                    wave_stats[wave][l16][3] = st.nan ? 1.0f : 0.0f;
                    wave_stats[wave][l16][4] = st.finite ? 1.0f : 0.0f;
                }
                __syncthreads();
                st = RowStats{-inf, 0.0f, 0u, false, false};
#pragma unroll
                for (int w = 0; w < NW; ++w)
                    st.merge(wave_stats[w][l16][0], wave_stats[w][l16][1], as_u32(wave_stats[w][l16][2]),
                             wave_stats[w][l16][3] != 0.0f, wave_stats[w][l16][4] != 0.0f);
            }
            nan_row = st.nan || (st.pinf == 0 && !st.finite);      // NaN score or all -inf
            const float pinf_p = st.pinf ? 1.0f / (float)st.pinf : 0.0f;
            const float inv_sum = 1.0f / st.sum;
            // ---- pass 2 of the special rows
            walk_groups(std::true_type{}, false, false, std::false_type{}, [&](uint32_t g, f32x4_t (&s)[2], const u32x4 (&vfr)[DT16], auto) {
                float pr[8];
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float v = s[half][j];
                        const bool seen = (32 * g + 16 * half + 4 * kg + j < vis) & !nan_row;
                        const float regular = v == -inf ? 0.0f : __expf(v - st.m) * inv_sum;
                        const float special = v == inf ? pinf_p : 0.0f;
                        pr[half * 4 + j] = seen ? (st.pinf ? special : regular) : 0.0f;
                    }
                // one rounding to BF16, then flushed like every matrix operand (p >= 0)
                mma_v(o, vfr, u32x4{daz2(pack_bf16(pr[0], pr[1])), daz2(pack_bf16(pr[2], pr[3])),
                                    daz2(pack_bf16(pr[4], pr[5])), daz2(pack_bf16(pr[6], pr[7]))});
            });
        }
        if (SPLIT) {
            if (wave != 0) {
#pragma unroll
                for (int dt = 0; dt < DT16; ++dt) wave_out[wave - 1][dt][lane] = o[dt];
            }
            __syncthreads();
            if (wave != 0) return;
            // one wave's partial at a time (unrolled, the loads of all of them would be
            // hoisted and would not fit the register file)
#pragma unroll 1
            for (int w = 0; w < NW - 1; ++w)
#pragma unroll
                for (int dt = 0; dt < DT16; ++dt) o[dt] += wave_out[w][dt][lane];
        }
        // lane holds out[row][head*D + 16*dt + 4*kg + j]
        if (!row_ok) return;
        uint8_t* ob = a.out + plane[3] * a.out_plane_bytes
                + (uint64_t)(row >> 4) * a.out_tile_cols * kTileBytes + (row & 15u) * kRowBytes;
        if (FULLD && plain) {
            // whole tiles and no special row: a lane's four outputs of a tile are one 8-byte piece of
            // tile head * DT16 + dt.  Adding +0 stores -0 as +0; the sums are no NaN here (finite V,
            // probabilities that add up to about one).
            uint8_t* ot = ob + (uint64_t)head * (DT16 * kTileBytes) + kg * 8;
#pragma unroll
            for (int dt = 0; dt < DT16; ++dt)
                *reinterpret_cast<u32x2*>(ot + dt * kTileBytes) =
                        u32x2{cvt_bf16x2(o[dt][0] + 0.0f, o[dt][1] + 0.0f), cvt_bf16x2(o[dt][2] + 0.0f, o[dt][3] + 0.0f)};
            return;
        }
#pragma unroll
        for (int dt = 0; dt < DT16; ++dt) {
            float val[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                val[j] = o[dt][j];
                if (val[j] == 0.0f) val[j] = 0.0f;                    // -0 is stored as +0
            }
            const uint32_t d = dt * kTile + 4 * kg, col = head * head_dim + d;
            if ((head_dim & 3u) == 0) {
                // the four outputs lie in one tile row of out
                if (d >= head_dim) continue;
                const u32x2 bits = nan_row ? u32x2{0x7FC07FC0u, 0x7FC07FC0u}
                                           : u32x2{pack_bf16(val[0], val[1]), pack_bf16(val[2], val[3])};
                *reinterpret_cast<u32x2*>(ob + (uint64_t)(col >> 4) * kTileBytes + (col & 15u) * 2) = bits;
                continue;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (d + j >= head_dim) continue;
                const uint32_t bits = nan_row ? 0x7FC0u : bf16_rne_sw(as_u32(val[j]));
                const uint32_t cj = col + j;
                *reinterpret_cast<uint16_t*>(ob + (uint64_t)(cj >> 4) * kTileBytes + (cj & 15u) * 2) = (uint16_t)bits;
            }
        }
    }
}

// The shared-ring mapping (MODE 2 above: four heads of one KV head per workgroup, D = 64 or 128)
// with TWO neighbouring row tiles per wave: every K and V group read from LDS feeds two score tiles
// and two output tiles, which halves the LDS traffic per product (what bounds the one-tile kernel
// at D = 128) and gives a wave two independent chains of matrix and exponent instructions per group
// where few waves fit a SIMD.  (Pairing tile j with tile N-1-j instead, which makes every
// workgroup's walk equally long, was measured and lost: half of its steps have one tile's work.)
// Plain passes only: a workgroup whose rows turn out special (a NaN or +infinity score, no finite
// score, or an infinity / NaN in V) forms its rows in the reference's order instead
// (sdpa_reference_row), all four waves together.  Grid (Hq / 4, planes, ceil(N / 2)); with N odd
// the last tile is alone.  The walk below does not assume the two tiles are neighbours: tile 0 is
// any tile above tile 1.
struct TileAbsent {};
struct TilePlain {};
struct TileMasked {};

template <int DT16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
void sdpa_mfma_pair_bf16_kernel(const SdpaArgs a) {
    static_assert(DT16 % 4 == 0, "whole KiB chunks per wave");
    constexpr int T = 2;                                   // row tiles per wave: 0 the short one, 1 the long one
    constexpr uint32_t kStage = 2 * DT16 * 1024;           // K group + V group
    constexpr int D32 = DT16 / 2;
    constexpr float kFloor = -1.0e30f;                     // stands in for a maximum of -infinity
    __shared__ __attribute__((aligned(16))) uint8_t kv_ring[3 * kStage];
    __shared__ float row_buffer[4][64];
    __shared__ uint32_t special_rows;
    if (threadIdx.x == 0) special_rows = 0;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t l16 = lane & 15u, kg = lane >> 4;
    const uint32_t head = blockIdx.x * 4 + wave;
    const uint32_t hkv = head / a.grouping;
    const uint32_t row_tiles = (a.R + kTile - 1) / kTile;
    // pairs of neighbouring tiles, the pairs with the longest prefixes dispatched first
    const uint32_t pair = gridDim.z - 1 - blockIdx.z;
    const uint32_t slab[T] = {2 * pair, 2 * pair + 1 < row_tiles ? 2 * pair + 1 : 2 * pair};
    const bool both = slab[0] < slab[1];
    const float inf = __builtin_inff();
    // per tile: the lane's row, what it sees (rows past R mirror the tile's last row: their results
    // are dropped), the groups its rows reach and the groups all of them see whole
    uint32_t row[T], vis_plain[T], groups[T], full[T], first_row[T], last_row[T];
    bool row_ok[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        first_row[t] = slab[t] * kTile;
        last_row[t] = first_row[t] + kTile - 1 < a.R ? first_row[t] + kTile - 1 : a.R - 1;
        const uint32_t vis_last = a.a + last_row[t] + 1 < a.L ? a.a + last_row[t] + 1 : a.L;
        row[t] = first_row[t] + l16;
        row_ok[t] = row[t] < a.R && (t == 1 || both);
        const uint32_t reach = a.a + row[t] + 1;
        vis_plain[t] = row[t] < a.R ? (reach < a.L ? reach : a.L) : vis_last;
        const uint32_t reach_min = a.a + first_row[t] + 1;
        groups[t] = (vis_last + 31) / 32;
        full[t] = (reach_min < a.L ? reach_min : a.L) / 32;
    }
    if (!both) {
        groups[0] = 0;
        full[0] = 0;
    }
    const uint32_t ring_groups = groups[1];
    const uint32_t c0 = (kg & 1u) * 8u;
    const uint32_t p = a.plane0 + blockIdx.y;
    const uint32_t flag_words = sdpa_flag_words(a, p, hkv, lane);
    uint64_t plane[4];
    walk_planes(a.walk, p, plane);
    const uint8_t* qb = a.q + (plane[0] + (uint64_t)head * a.q_head_stride) * a.q_plane_bytes;
    const uint8_t* vf = a.packed_v + (((uint64_t)p * a.Hkv + hkv) * a.groups) * DT16 * kFrag;
    const uint32_t vf_lane = lane * 16;
    const uint8_t* kp = a.packed_k + (((uint64_t)p * a.Hkv + hkv) * a.groups * 2) * DT16 * kTileBytes;
    const uint32_t kp_lane = l16 * kRowBytes + c0 * 2;
    // a wave's share of K group g (and V group g) into ring stage buf, as in sdpa_mfma
    auto issue = [&](auto with_v, uint32_t g, uint32_t buf) {
        const uint32_t gg = g < ring_groups ? g : ring_groups - 1;
        uint8_t* stage = kv_ring + buf * kStage;
#pragma unroll
        for (int j = 0; j < DT16 / 4; ++j) {
            const uint32_t chunk = wave + 4 * j;
            __builtin_amdgcn_global_load_lds((gptr_t)(kp + ((gg * DT16 + chunk) * kFrag + vf_lane)),
                                             (lptr_t)(stage + chunk * kFrag), 16, 0, 0);
            if constexpr (decltype(with_v)::value)
                __builtin_amdgcn_global_load_lds((gptr_t)(vf + ((gg * DT16 + chunk) * kFrag + vf_lane)),
                                                 (lptr_t)(stage + (DT16 + chunk) * kFrag), 16, 0, 0);
        }
    };
    issue(std::false_type{}, 0, 0);
    issue(std::false_type{}, 1, 1);
    u32x4 q_bits[T][D32];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const uint32_t qrow = row[t] < a.R ? row[t] : a.R - 1;
#pragma unroll
        for (int c = 0; c < D32; ++c)
            q_bits[t][c] = *reinterpret_cast<const u32x4*>(
                    qb + ((uint64_t)(qrow >> 4) * DT16 + (2 * c + (kg >> 1))) * kTileBytes + (qrow & 15u) * kRowBytes + c0 * 2);
    }
    // every row of the wave's tiles in the reference's order
    auto reference_rows = [&]() {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        for (int t = both ? 0 : 1; t < T; ++t)
            for (uint32_t r = first_row[t]; r <= last_row[t]; ++r)
                sdpa_reference_row(a, p, hkv, head, r, lane, &row_buffer[wave][0]);
    };
    if (__any(flag_words != 0)) {           // an infinity or NaN in V of this KV head: all four waves alike
        reference_rows();
        return;
    }
    bf16x8_t qf[T][D32];
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int c = 0; c < D32; ++c) qf[t][c] = daz8(q_bits[t][c]);

    // One pass over the groups of the long tile: group g's K (and V) out of the ring, then
    // body(g, k, v, state of tile 0, state of tile 1).  Tile 0 sees its groups whole, then masked,
    // then not at all; tile 1 whole, then masked; the combinations that occur, in their order:
    auto walk = [&](auto with_v, bool primed, auto&& body) {
        constexpr bool WITH_V = decltype(with_v)::value;
        constexpr int LPS = (WITH_V ? 2 : 1) * (DT16 / 4);
        if (!primed) {
            issue(with_v, 0, 0);
            issue(with_v, 1, 1);
        }
        uint32_t buf = 0;
        auto step = [&](uint32_t g, auto tile0, auto tile1) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPS) : "memory");
            __builtin_amdgcn_s_barrier();
            issue(with_v, g + 2, buf == 0 ? 2 : buf - 1);
            const uint8_t* stage = kv_ring + buf * kStage;
            buf = buf == 2 ? 0 : buf + 1;
            u32x4 kw[2][D32];
            const uint32_t k_at = lds_address(stage + ((kg >> 1) * kTileBytes + kp_lane));
            static_for<2 * D32>([&](auto index) {
                constexpr int half = decltype(index)::value / D32, c = decltype(index)::value % D32;
                kw[half][c] = lds_read_b128<(half * DT16 + 2 * c) * (int)kTileBytes>(k_at);
            });
            u32x4 vfr[WITH_V ? DT16 : 1];
            if constexpr (WITH_V) {
                const uint32_t v_at = lds_address(stage + vf_lane);
                static_for<DT16>([&](auto index) {
                    constexpr int dt = decltype(index)::value;
                    vfr[dt] = lds_read_b128<(DT16 + dt) * (int)kFrag>(v_at);
                });
            }
            lds_reads_landed();
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int c = 0; c < D32; ++c) asm volatile("" : "+v"(kw[half][c]));
            if constexpr (WITH_V) {
#pragma unroll
                for (int dt = 0; dt < DT16; ++dt) asm volatile("" : "+v"(vfr[dt]));
            }
            body(g, kw, vfr, tile0, tile1);
        };
        const uint32_t meet = groups[0] < full[1] ? groups[0] : full[1];
        uint32_t g = 0;
#pragma unroll 1
        for (; g < full[0]; ++g) step(g, TilePlain{}, TilePlain{});
#pragma unroll 1
        for (; g < meet; ++g) step(g, TileMasked{}, TilePlain{});
#pragma unroll 1
        for (; g < full[1]; ++g) step(g, TileAbsent{}, TilePlain{});       // (runs when groups[0] < full[1])
#pragma unroll 1
        for (; g < groups[0]; ++g) step(g, TileMasked{}, TileMasked{});    // (runs when full[1] < groups[0])
#pragma unroll 1
        for (; g < groups[1]; ++g) step(g, TileAbsent{}, TileMasked{});
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
    };
    // the dot products of tile t's rows with the 32 tokens of the group (lane: tokens
    // 16*half + 4*kg + j of row l16), masked where the row must not see the token
    auto scores = [&](auto tile, auto state, const u32x4 (&kw)[2][D32], uint32_t g, f32x4_t (&s)[2]) {
        constexpr int t = decltype(tile)::value;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int c = 0; c < D32; ++c)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kw[half][c]), qf[t][c], acc, 0, 0, 0);
            s[half] = acc;
        }
        if constexpr (std::is_same_v<decltype(state), TileMasked>) {
            const int rem = (int)vis_plain[t] - (int)(32 * g + 4 * kg);
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int j = 0; j < 4; ++j) s[half][j] = 16 * half + j < rem ? s[half][j] : -inf;
        } else {
            settle_matrix_results(s);
        }
    };
    const float kls = a.exp_scale;
    auto join = [&](float& m, float& sum, float m2, float sum2) {
        const float mm = __builtin_fmaxf(m, m2), base = __builtin_fmaxf(mm, kFloor);
        sum = sum * __builtin_amdgcn_exp2f((__builtin_fmaxf(m, kFloor) - base) * kls)
            + sum2 * __builtin_amdgcn_exp2f((__builtin_fmaxf(m2, kFloor) - base) * kls);
        m = mm;
    };

    // ---- pass 1: running maximum and sum of exponentials of both tiles
    float pm[T], psum[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        pm[t] = -inf;
        psum[t] = 0.0f;
    }
    auto statistics = [&](auto tile, auto state, const u32x4 (&kw)[2][D32], uint32_t g) {
        constexpr int t = decltype(tile)::value;
        if constexpr (!std::is_same_v<decltype(state), TileAbsent>) {
            f32x4_t s[2];
            scores(tile, state, kw, g, s);
            const float newm = max3(max3(s[0][0], s[0][1], s[0][2]), max3(s[0][3], s[1][0], s[1][1]),
                                    max3(s[1][2], s[1][3], pm[t]));
            const float base = max2(newm, kFloor);
            psum[t] *= __builtin_amdgcn_exp2f((max2(pm[t], kFloor) - base) * kls);
            const float nb = -base * kls;
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int j = 0; j < 4; ++j) psum[t] += __builtin_amdgcn_exp2f(__builtin_fmaf(s[half][j], kls, nb));
            pm[t] = newm;
        }
    };
    walk(std::false_type{}, true, [&](uint32_t g, const u32x4 (&kw)[2][D32], const u32x4 (&)[1], auto tile0, auto tile1) {
        statistics(std::integral_constant<int, 0>{}, tile0, kw, g);
        statistics(std::integral_constant<int, 1>{}, tile1, kw, g);
    });
    // pass 2's first groups are on their way while the statistics are joined
    issue(std::true_type{}, 0, 0);
    issue(std::true_type{}, 1, 1);
    bool odd = false;
#pragma unroll
    for (int t = 0; t < T; ++t) {
#pragma unroll
        for (int off = 16; off <= 32; off *= 2) {
            const float m2 = __shfl_xor(pm[t], off), s2 = __shfl_xor(psum[t], off);
            join(pm[t], psum[t], m2, s2);
        }
        if (t == 1 || both) odd = odd || !(psum[t] > 0.0f && psum[t] < inf && pm[t] < inf);
    }
    bool plain = !__any(odd);
    if (!plain && lane == 0) special_rows = 1;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    plain = __builtin_amdgcn_readfirstlane(lds_read_b32(lds_address(&special_rows))) == 0;
    if (!plain) {
        reference_rows();
        return;
    }

    // ---- pass 2: probabilities, rounded once to BF16 and flushed, times V
    f32x4_t o[T][DT16];
    float inv_sum[T], nb[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
#pragma unroll
        for (int dt = 0; dt < DT16; ++dt) o[t][dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        inv_sum[t] = 1.0f / psum[t];
        nb[t] = -pm[t] * kls;
    }
    auto products = [&](auto tile, auto state, const u32x4 (&kw)[2][D32], const u32x4 (&vfr)[DT16], uint32_t g) {
        constexpr int t = decltype(tile)::value;
        if constexpr (!std::is_same_v<decltype(state), TileAbsent>) {
            f32x4_t s[2];
            scores(tile, state, kw, g, s);
            float e[8];
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int j = 0; j < 4; ++j) e[half * 4 + j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[half][j], kls, nb[t]));
            const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, scaled_flushed_bf16x8(e, inv_sum[t]));
#pragma unroll
            for (int dt = 0; dt < DT16; ++dt)
                o[t][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vfr[dt]), pf, o[t][dt], 0, 0, 0);
        }
    };
    walk(std::true_type{}, true, [&](uint32_t g, const u32x4 (&kw)[2][D32], const u32x4 (&vfr)[DT16], auto tile0, auto tile1) {
        products(std::integral_constant<int, 0>{}, tile0, kw, vfr, g);
        products(std::integral_constant<int, 1>{}, tile1, kw, vfr, g);
    });
    // lane holds out[row][head*D + 16*dt + 4*kg + j]: one 8-byte piece of tile head * DT16 + dt
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (!row_ok[t]) continue;
        uint8_t* ot = a.out + plane[3] * a.out_plane_bytes + (uint64_t)(row[t] >> 4) * a.out_tile_cols * kTileBytes
                + (row[t] & 15u) * kRowBytes + (uint64_t)head * (DT16 * kTileBytes) + kg * 8;
#pragma unroll
        for (int dt = 0; dt < DT16; ++dt)
            *reinterpret_cast<u32x2*>(ot + dt * kTileBytes) =
                    u32x2{cvt_bf16x2(o[t][dt][0] + 0.0f, o[t][dt][1] + 0.0f), cvt_bf16x2(o[t][dt][2] + 0.0f, o[t][dt][3] + 0.0f)};
    }
}

// Few rows per KV head (grouping * R <= 16: a decode step): one workgroup of eight waves
// = one KV head of one plane, the 16 rows of its tile = the rows of all query heads of
// that KV head, the waves share out the 32-token groups.  Scores come from the matrix
// cores as in sdpa_mfma (K read from the cache as it lies, flushed in registers); the
// product with V runs on the vector units straight from the cache -- lane = feature,
// the probabilities of a group broadcast from LDS -- so nothing is packed or
// transposed, no workspace is used, and a token a row must not see is left out of that
// row's sum by a select (an infinite V there cannot reach it).
// PHASE 0: the whole step in one launch.  A long prefix of few sequences leaves most CUs idle
// that way, so the token groups can also be shared out over several workgroups per KV head
// (grid z), in two launches that keep the arithmetic of the one: PHASE 1 forms the statistics of
// a share of the groups and leaves them in the workspace; PHASE 2 joins the statistics of all
// shares (every workgroup in the same order, so all hold the same values), forms the
// probabilities of its share and leaves its partial output sums; sdpa_decode_join_kernel adds the
// partial sums in share order and stores the rows.
//
// KEPT (one launch, prefixes past what the K ring holds): the scores of pass 1 stay in LDS
// (128 bytes per group and tile row in use: [tile row][kg][8] binary32; every wave its own
// groups), and pass 2 takes them from there instead of reading K and multiplying a second time
// -- the same bits, a third less traffic.  KEPT = 1: the scores lie behind the kernel's own
// arrays, [group] by [group].  KEPT = 2, for prefixes that do not fit that way: every wave has
// an area of its own for its groups, and its probabilities of the vector path and its partial
// outputs take the start of that area over once the wave is through with its scores (a wave's
// LDS operations complete in order, and no other wave looks at the area before the barrier
// behind the partial outputs).
// FULLD: D is DT16 whole tiles and a multiple of 32 -- a constant to the compiler, and no operand
// load needs a path for a head that ends inside its eight features.
template <int DT16, int PHASE, int KEPT = 0, bool FULLD = false>
__global__ __launch_bounds__(512) void sdpa_decode_bf16_kernel(const SdpaArgs a) {
    static_assert(KEPT == 0 || PHASE == 0, "scores are kept inside one launch");
    static_assert(!FULLD || DT16 % 2 == 0, "whole 32-feature slices");
    extern __shared__ __attribute__((aligned(16))) uint8_t kept_scores[];
    constexpr int D32 = (DT16 + 1) / 2;
    constexpr int NW = 8;
    constexpr int DL = (DT16 + 3) / 4;                 // features per lane (lane, lane + 64)
    constexpr int PD = DT16 > 6 ? 1 : 2;               // groups in flight per wave (registers allow one at D > 96)
    __shared__ float wave_stats[NW][16][5];
    // the probabilities of a group on the vector path and the waves' partial outputs
    constexpr uint32_t kPBytes = 16 * 32 * 4;
    __shared__ __attribute__((aligned(16))) float p_tile_own[KEPT == 2 ? 1 : NW][16][32];
    __shared__ float o_part_own[KEPT == 2 ? 1 : NW][16][DL * 64];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t l16 = lane & 15u, kg = lane >> 4;
    const uint32_t hkv = blockIdx.x;
    const uint32_t row = l16 / a.grouping;                            // the lane's tile row: (row, query head)
    const uint32_t head = hkv * a.grouping + (l16 - row * a.grouping);
    const bool row_ok = row < a.R;
    const uint32_t qrow = row_ok ? row : a.R - 1;
    const uint32_t nrows = a.grouping * a.R;                          // tile rows in use
    const uint32_t head_dim = FULLD ? (uint32_t)DT16 * kTile : a.D;
    const uint32_t d_tiles = FULLD ? (uint32_t)DT16 : a.d_tiles;
    auto p_tile = [&](uint32_t r, uint32_t t) -> float* {
        if constexpr (KEPT == 2) return reinterpret_cast<float*>(kept_scores + wave * a.kept_wave_bytes + (r * 32 + t) * 4);
        else return &p_tile_own[wave][r][t];
    };
    auto o_part = [&](uint32_t w, uint32_t r, uint32_t d) -> float& {
        if constexpr (KEPT == 2)
            return *reinterpret_cast<float*>(kept_scores + w * a.kept_wave_bytes + kPBytes + (r * (DL * 64) + d) * 4);
        else return o_part_own[w][r][d];
    };
    // where the lane's eight scores of group g are kept
    auto kept_at = [&](uint32_t g, uint32_t r) -> f32x4_t* {
        if constexpr (KEPT == 2)
            return reinterpret_cast<f32x4_t*>(kept_scores + wave * a.kept_wave_bytes + (((g / NW) * nrows + r) * 4 + kg) * 32);
        else return reinterpret_cast<f32x4_t*>(kept_scores + ((g * nrows + r) * 4 + kg) * 32);
    };
    const uint32_t reach = a.a + row + 1, reach_max = a.a + a.R;
    const uint32_t vis = row_ok ? (reach < a.L ? reach : a.L) : 0;
    const uint32_t vis_max = reach_max < a.L ? reach_max : a.L;
    const uint32_t groups = (vis_max + 31) / 32;
    // this workgroup's share of the groups: [g_lo, g_hi)
    const uint32_t shares = PHASE == 0 ? 1 : gridDim.z, share = PHASE == 0 ? 0 : blockIdx.z;
    const uint32_t per_share = (groups + shares - 1) / shares;
    const uint32_t g_lo = share * per_share < groups ? share * per_share : groups;
    const uint32_t g_hi = g_lo + per_share < groups ? g_lo + per_share : groups;
    const uint32_t c0 = (kg & 1u) * 8u;
    const float inf = __builtin_inff();
    // one plane per grid row, as in sdpa_mfma
    {
        const uint32_t p = a.plane0 + blockIdx.y;
        uint64_t plane[4];
        walk_planes(a.walk, p, plane);
        const uint8_t* qb = a.q + (plane[0] + (uint64_t)head * a.q_head_stride) * a.q_plane_bytes;
        const uint8_t* kb = a.k + (plane[1] + (uint64_t)hkv * a.k_head_stride) * a.kv_plane_bytes;
        const uint8_t* vb = a.v + (plane[2] + (uint64_t)hkv * a.v_head_stride) * a.kv_plane_bytes;
        // the raw bits of q: flushed after K and V have been requested, so that nothing waits
        // for q alone
        u32x4 q_bits[D32];
        bf16x8_t qf[D32];
#pragma unroll
        for (int c = 0; c < D32; ++c) {
            const uint32_t i0 = 32 * c + 8 * kg, tile = 2 * c + (kg >> 1);
            q_bits[c] = u32x4{0, 0, 0, 0};
            if (FULLD || i0 < head_dim)
                q_bits[c] = load_k8_bits(qb + ((uint64_t)(qrow >> 4) * d_tiles + tile) * kTileBytes
                                            + (qrow & 15u) * kRowBytes, c0, i0, head_dim);
        }
        // K of group g (two 16-token tiles), requested one group ahead of its use
        struct KGroup { u32x4 w[2][D32]; };
        auto load_k = [&](uint32_t g, KGroup& kgp) {
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                uint32_t token = 32 * g + 16 * half + l16;
                if (token >= a.L) token = a.L - 1;                    // the cache tail is never touched
                const uint8_t* krow = kb + (uint64_t)(token >> 4) * d_tiles * kTileBytes + (token & 15u) * kRowBytes;
#pragma unroll
                for (int c = 0; c < D32; ++c) {
                    const uint32_t i0 = 32 * c + 8 * kg, tile = 2 * c + (kg >> 1);
                    kgp.w[half][c] = u32x4{0, 0, 0, 0};
                    if (FULLD || i0 < head_dim)
                        kgp.w[half][c] = load_k8_bits(krow + (uint64_t)tile * kTileBytes, c0, i0, head_dim);
                }
            }
        };
        // scores: lane gets tokens 32g + 16*half + 4*kg + j (j < 4) of tile row l16
        auto scores = [&](const KGroup& kgp, f32x4_t (&s)[2]) {
            // (whole heads: one test for the group's words, the flush only if a lane asks for it)
            u32x4 kw[2 * D32];
#pragma unroll
            for (int i = 0; i < 2 * D32; ++i) kw[i] = kgp.w[i / D32][i % D32];
            if constexpr (FULLD) daz_words(kw);
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int c = 0; c < D32; ++c)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            FULLD ? __builtin_bit_cast(bf16x8_t, kw[half * D32 + c]) : daz8(kw[half * D32 + c]), qf[c], acc, 0, 0, 0);
                f32x4_t q = acc * a.inv_scale;
                if (!a.scale_pow2) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float refined = __builtin_fmaf(__builtin_fmaf(-q[j], a.scale, acc[j]), a.inv_scale, q[j]);
                        q[j] = __builtin_fabsf(q[j]) < inf ? refined : q[j];
                    }
                }
                s[half] = q;
            }
        };
        // V of group g, lane = feature: the raw bits of the 32 tokens
        // V of eight tokens from token t0 of group g on, lane = feature: flushed values
        auto load_v8 = [&](uint32_t g, uint32_t t0, float (&value)[8][DL]) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                uint32_t token = 32 * g + t0 + i;
                if (token >= vis_max) token = vis_max - 1;            // its probability is +0 and it is masked below
                const uint8_t* vrow = vb + (uint64_t)(token >> 4) * d_tiles * kTileBytes + (token & 15u) * kRowBytes;
#pragma unroll
                for (int c = 0; c < DL; ++c) {
                    const uint32_t d = lane + 64 * c;
                    value[i][c] = (FULLD || d < head_dim) ? daz_bf16(*reinterpret_cast<const uint16_t*>(
                                                    vrow + (uint64_t)(d >> 4) * kTileBytes + (d & 15u) * 2))
                                          : 0.0f;
                }
            }
        };
        // pass 2 sends a group that every row in use sees whole through the matrix cores with V
        // loaded straight from the cache in the operand order (lane (feature l16, kg): tokens
        // 32g + 4kg + j and 32g + 16 + 4kg + j), flushed in registers
        const uint32_t vis_min = a.a + 1 < a.L ? a.a + 1 : a.L;          // what row 0 sees: the least
        // Where every row in use sees the same prefix (one row per sequence -- the decode step --
        // or every row reaches the end of the prefix) no visible token is hidden from any row, so
        // the ragged last group takes the matrix cores as well: its tokens past the prefix get a
        // probability of +0 and their V, whatever the cache holds there, is taken as zero.
        const bool one_prefix = vis_min == vis_max;
        const uint32_t full_groups = one_prefix ? groups : vis_min / 32;
        // of this share: the fully visible groups end at full_hi, the others start at tail_lo
        const uint32_t full_hi = full_groups < g_hi ? full_groups : g_hi;
        const uint32_t tail_lo = full_groups > g_lo ? full_groups : g_lo;
        struct VFrag { u32x4 w[DT16]; };
        // (the ragged last group may end in the cache's last token tile: the second tile of the
        // group is then not there, and its lanes read the first tile again -- their tokens lie past
        // the prefix and are taken as zero below.  A wave-uniform offset, so every address stays a
        // group base plus constants.)
        const uint32_t last_token_tile = (vis_max - 1) >> 4;
        auto load_vf = [&](uint32_t g, VFrag& vf) {
            const uint32_t second = 2 * g + 1 <= last_token_tile ? 2 * g + 1 : 2 * g;
            const uint8_t* tiles[2] = {vb + (uint64_t)(2 * g) * d_tiles * kTileBytes,
                                       vb + (uint64_t)second * d_tiles * kTileBytes};
#pragma unroll
            for (int dt = 0; dt < DT16; ++dt) {
                // pairs of 16-bit loads into the halves of one register
                u16x2_t h[4];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    uint16_t bits = 0;
                    if (FULLD || dt * kTile + l16 < head_dim)
                        bits = *reinterpret_cast<const uint16_t*>(
                                tiles[j >> 2] + dt * kTileBytes + (4 * kg + (j & 3)) * kRowBytes + l16 * 2);
                    h[j >> 1][j & 1] = bits;
                }
                // raw bits: they are flushed where they are used, so a request does not wait here
                vf.w[dt] = u32x4{__builtin_bit_cast(uint32_t, h[0]), __builtin_bit_cast(uint32_t, h[1]),
                                 __builtin_bit_cast(uint32_t, h[2]), __builtin_bit_cast(uint32_t, h[3])};
            }
        };
        // pass 1: the rows' statistics over this wave's groups, then over the waves
        RowStats st = {-inf, 0.0f, 0u, false, false};
        // a ring of PD groups of K (and of V in pass 2): group g + PD*NW is requested as soon as
        // group g has been multiplied, so PD groups per wave are in flight -- one wave's chain of
        // dependent loads is what a long prefix costs here
        // (with kept scores every pass streams one operand, and one group per wave in flight is
        // enough: measured at 2048 tokens, 64 sequences, two groups 31.2 us, four 33.1, one 29.5)
        constexpr int PR = KEPT != 0 ? 1 : PD;
        KGroup kr[PR];
        VFrag vr[PR];
        // a wave whose groups all fit the ring still holds their K after pass 1; V of the first
        // groups of pass 2 is requested here, together with K, so the step waits for memory once
        const bool ring_kept = PHASE == 0 && g_lo + wave + PD * NW >= g_hi;
        if (PHASE != 2) {
#pragma unroll
        for (int slot = 0; slot < PR; ++slot)
            if (g_lo + wave + slot * NW < g_hi) load_k(g_lo + wave + slot * NW, kr[slot]);
        if (PHASE == 0 && KEPT == 0) {
#pragma unroll
            for (int slot = 0; slot < PD; ++slot)
                if (g_lo + wave + slot * NW < full_hi) load_vf(g_lo + wave + slot * NW, vr[slot]);
        }
        }
#pragma unroll
        for (int c = 0; c < D32; ++c) qf[c] = daz8(q_bits[c]);
        if (PHASE != 2) {
        // The statistics of a group, with everything the special scores need: which tokens the
        // row sees, NaN, the count of +infinity, non-finite scores kept out of maximum and sum.
        auto careful_stats = [&](uint32_t g, f32x4_t (&s)[2]) {
            float local = -inf;
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const bool seen = 32 * g + 16 * half + 4 * kg + j < vis;
                    const float v = s[half][j];
                    st.nan = st.nan | (seen & (v != v));
                    st.pinf += (seen & (v == inf)) ? 1u : 0u;
                    s[half][j] = (seen & (__builtin_fabsf(v) < inf)) ? v : -inf;
                    local = __builtin_fmaxf(local, s[half][j]);
                }
            const float newm = __builtin_fmaxf(st.m, local);
            st.sum = newm == st.m ? st.sum : st.sum * __expf(st.m - newm);
            st.m = newm;
            st.finite = st.finite | (local > -inf);
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int e = 0; e < 4; ++e) st.sum += s[half][e] == -inf ? 0.0f : __expf(s[half][e] - newm);
        };
        // The same statistics, bit for bit, for a group that every row in use sees whole and whose
        // scores are finite or -infinity -- less than half the instructions: no per-token test, and
        // exp(-infinity) is the +0 the careful form selects.  kFloor stands in for a maximum of
        // -infinity in the exponent arguments.  A NaN, a +infinity or a maximum below kFloor raises
        // `suspicious`, and the wave then forms all its statistics again in the careful form.
        constexpr float kFloor = -1.0e30f;
        bool suspicious = false;
        auto fast_stats = [&](const f32x4_t (&s)[2]) {
            suspicious = suspicious | __builtin_isunordered(s[0][0], s[0][1]) | __builtin_isunordered(s[0][2], s[0][3])
                    | __builtin_isunordered(s[1][0], s[1][1]) | __builtin_isunordered(s[1][2], s[1][3]);
            const float local = __builtin_fmaxf(__builtin_fmaxf(__builtin_fmaxf(s[0][0], s[0][1]), __builtin_fmaxf(s[0][2], s[0][3])),
                                                __builtin_fmaxf(__builtin_fmaxf(s[1][0], s[1][1]), __builtin_fmaxf(s[1][2], s[1][3])));
            const float newm = __builtin_fmaxf(st.m, local);
            suspicious = suspicious | (local == inf) | ((newm < kFloor) & (newm > -inf));
            const float m_eff = __builtin_fmaxf(newm, kFloor);
            st.sum = st.sum * __expf(__builtin_fmaxf(st.m, kFloor) - m_eff);
            st.m = newm;
            st.finite = st.finite | (local > -inf);
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int e = 0; e < 4; ++e) st.sum += __expf(s[half][e] - m_eff);
        };
        // groups below whole_hi are seen whole by every row in use
        const uint32_t whole_groups = vis_min / 32, whole_hi = whole_groups < g_hi ? whole_groups : g_hi;
        uint32_t g0 = g_lo + wave;
#pragma unroll 1
        for (; g0 + (PR - 1) * NW < whole_hi; g0 += PR * NW) {
#pragma unroll
          for (int slot = 0; slot < PR; ++slot) {
            const uint32_t g = g0 + slot * NW;
            f32x4_t s[2];
            scores(kr[slot], s);
            if (g + PR * NW < g_hi) load_k(g + PR * NW, kr[slot]);
            if constexpr (KEPT != 0) {
                if (l16 < nrows) {
                    f32x4_t* dst = kept_at(g, l16);
                    dst[0] = s[0];
                    dst[1] = s[1];
                }
            }
            fast_stats(s);
          }
        }
#pragma unroll 1
        for (; g0 < g_hi; g0 += PR * NW) {
#pragma unroll
          for (int slot = 0; slot < PR; ++slot) {
            const uint32_t g = g0 + slot * NW;
            if (g >= g_hi) break;                                     // uniform
            f32x4_t s[2];
            scores(kr[slot], s);
            if (g + PR * NW < g_hi) load_k(g + PR * NW, kr[slot]);
            if constexpr (KEPT != 0) {
                if (l16 < nrows) {
                    f32x4_t* dst = kept_at(g, l16);
                    dst[0] = s[0];
                    dst[1] = s[1];
                }
            }
            careful_stats(g, s);
          }
        }
        if (__any(suspicious)) {
            // rare: a special score among the whole groups -- all of the wave's groups again
            st = RowStats{-inf, 0.0f, 0u, false, false};
#pragma unroll 1
            for (uint32_t g = g_lo + wave; g < g_hi; g += NW) {
                KGroup kt;
                load_k(g, kt);
                f32x4_t s[2];
                scores(kt, s);
                careful_stats(g, s);
            }
        }
#pragma unroll
        for (int off = 16; off <= 32; off *= 2) {
            const float m2 = __shfl_xor(st.m, off), s2 = __shfl_xor(st.sum, off);
            const uint32_t p2 = __shfl_xor(st.pinf, off);
            const int n2 = __shfl_xor((int)st.nan, off), f2 = __shfl_xor((int)st.finite, off);
            st.merge(m2, s2, p2, n2 != 0, f2 != 0);
        }
        if (kg == 0) {
            wave_stats[wave][l16][0] = st.m;
            wave_stats[wave][l16][1] = st.sum;
            wave_stats[wave][l16][2] = as_f32(st.pinf);
            wave_stats[wave][l16][3] = st.nan ? 1.0f : 0.0f;
            wave_stats[wave][l16][4] = st.finite ? 1.0f : 0.0f;
        }
        __syncthreads();
        st = RowStats{-inf, 0.0f, 0u, false, false};
#pragma unroll
        for (int w = 0; w < NW; ++w)
            st.merge(wave_stats[w][l16][0], wave_stats[w][l16][1], as_u32(wave_stats[w][l16][2]),
                     wave_stats[w][l16][3] != 0.0f, wave_stats[w][l16][4] != 0.0f);
        }
        // the statistics of a share: [pair][share][row][8] floats of the workspace
        float* share_stats = a.decode_stats + (((uint64_t)p * a.Hkv + hkv) * shares) * 16 * 8;
        if (PHASE == 1) {
            if (threadIdx.x < 16) {
                float* dst = share_stats + ((uint64_t)share * 16 + l16) * 8;
                dst[0] = st.m;
                dst[1] = st.sum;
                dst[2] = as_f32(st.pinf);
                dst[3] = st.nan ? 1.0f : 0.0f;
                dst[4] = st.finite ? 1.0f : 0.0f;
            }
            return;
        }
        if (PHASE == 2) {
            st = RowStats{-inf, 0.0f, 0u, false, false};
            for (uint32_t sh = 0; sh < shares; ++sh) {
                const float* src = share_stats + ((uint64_t)sh * 16 + l16) * 8;
                st.merge(src[0], src[1], as_u32(src[2]), src[3] != 0.0f, src[4] != 0.0f);
            }
        }
        const bool nan_row = st.nan || (st.pinf == 0 && !st.finite);
        const float pinf_p = st.pinf ? 1.0f / (float)st.pinf : 0.0f;
        const float inv_sum = 1.0f / st.sum;
        // pass 2.  A group that every row in use sees whole goes through the matrix cores: the
        // probabilities stay in the lanes that formed the scores, V is loaded straight from the
        // cache in the operand order (lane (feature l16, kg): tokens 32g + 4kg + j and
        // 32g + 16 + 4kg + j), flushed in registers.  The group on the diagonal and the ragged last
        // group take the vector units: probabilities to LDS, lane = feature, and a token a row
        // must not see is left out of that row's sum by a select.
        f32x4_t om[DT16];                                   // matrix-core part: out[row l16][16 dt + 4 kg + j]
#pragma unroll
        for (int dt = 0; dt < DT16; ++dt) om[dt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        // the probabilities of a group, rounded once to BF16 and flushed like every operand of the
        // product (p >= 0), two to a word
        auto probabilities = [&](uint32_t g, const f32x4_t (&s)[2]) -> u32x4 {
            float pr[8];
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float v = s[half][j];
                    const bool seen = (32 * g + 16 * half + 4 * kg + j < vis) & !nan_row;
                    const float regular = v == -inf ? 0.0f : __expf(v - st.m) * inv_sum;
                    const float special = v == inf ? pinf_p : 0.0f;
                    pr[half * 4 + j] = seen ? (st.pinf ? special : regular) : 0.0f;
                }
            return u32x4{daz2(pack_bf16(pr[0], pr[1])), daz2(pack_bf16(pr[2], pr[3])),
                         daz2(pack_bf16(pr[4], pr[5])), daz2(pack_bf16(pr[6], pr[7]))};
        };
        // The same probabilities, bit for bit, where no row of the tile is special (no NaN, no
        // +infinity, a finite maximum) and every row in use sees the whole group: the careful
        // form's selects all pick exp(v - max) / sum there, and exp(-infinity) is its +0.  (Tile
        // rows not in use get probabilities too; their outputs are never stored.)
        const bool plain_rows = !__any(nan_row || st.pinf != 0);
        auto plain_probabilities = [&](const f32x4_t (&s)[2]) -> u32x4 {
            float pr[8];
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int j = 0; j < 4; ++j) pr[half * 4 + j] = __expf(s[half][j] - st.m) * inv_sum;
            return u32x4{daz2(pack_bf16(pr[0], pr[1])), daz2(pack_bf16(pr[2], pr[3])),
                         daz2(pack_bf16(pr[4], pr[5])), daz2(pack_bf16(pr[6], pr[7]))};
        };
        {
#pragma unroll
            for (int slot = 0; slot < PR; ++slot)
                if (g_lo + wave + slot * NW < full_hi) {
                    if (!ring_kept && KEPT == 0) load_k(g_lo + wave + slot * NW, kr[slot]);
                    if (PHASE != 0 || KEPT != 0) load_vf(g_lo + wave + slot * NW, vr[slot]);
                }
#pragma unroll 1
            for (uint32_t g0 = g_lo + wave; g0 < full_hi; g0 += PR * NW) {
#pragma unroll
                for (int slot = 0; slot < PR; ++slot) {
                    const uint32_t g = g0 + slot * NW;
                    if (g >= full_hi) break;                                  // uniform
                    f32x4_t s[2];
                    if constexpr (KEPT != 0) {
                        // (a wave reads what it wrote itself; rows not in use get no probability)
                        const f32x4_t* src = kept_at(g, l16 < nrows ? l16 : 0);
                        s[0] = src[0];
                        s[1] = src[1];
                    } else {
                        scores(kr[slot], s);
                        if (g + PR * NW < full_hi) load_k(g + PR * NW, kr[slot]);
                    }
                    const bf16x8_t pf = __builtin_bit_cast(
                            bf16x8_t, plain_rows && 32 * g + 32 <= vis_min ? plain_probabilities(s) : probabilities(g, s));
                    if (32 * g + 32 > vis_max) {                              // uniform: the ragged last group
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const uint32_t t0 = 32 * g + (q < 2 ? 4 * kg + 2 * q : 16 + 4 * kg + 2 * (q - 2));
                            const uint32_t keep = (t0 < vis_max ? 0x0000FFFFu : 0u) | (t0 + 1 < vis_max ? 0xFFFF0000u : 0u);
#pragma unroll
                            for (int dt = 0; dt < DT16; ++dt) vr[slot].w[dt][q] &= keep;
                        }
                    }
                    if constexpr (FULLD) daz_words(vr[slot].w);
#pragma unroll
                    for (int dt = 0; dt < DT16; ++dt)
                        om[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                                FULLD ? __builtin_bit_cast(bf16x8_t, vr[slot].w[dt]) : daz8(vr[slot].w[dt]), pf, om[dt], 0, 0, 0);
                    if (g + PR * NW < full_hi) load_vf(g + PR * NW, vr[slot]);
                }
            }
        }
        float o[16][DL];                                    // vector part: out[row r][lane + 64 c]
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
            for (int c = 0; c < DL; ++c) o[r][c] = 0.0f;
        // the one or two groups past the fully visible ones, one per wave
#pragma unroll 1
        for (uint32_t g = tail_lo + wave; g < g_hi; g += NW) {
            KGroup kt;
            load_k(g, kt);
            f32x4_t s[2];
            scores(kt, s);
            const u32x4 pw = probabilities(g, s);
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                f32x4_t pe;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t pair = pw[half * 2 + (j >> 1)];
                    pe[j] = as_f32((j & 1) ? (pair & 0xFFFF0000u) : (pair << 16));
                }
                *reinterpret_cast<f32x4_t*>(p_tile(l16, 16 * half + 4 * kg)) = pe;
            }
            // the wave reads only what it wrote itself: LDS operations of a wave complete in order
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            // every tile row in use takes its probabilities (16-byte broadcasts) and adds
#pragma unroll
            for (int t0 = 0; t0 < 32; t0 += 8) {
                float value[8][DL];
                load_v8(g, t0, value);
#pragma unroll
                for (int r4 = 0; r4 < 16; r4 += 4) {
                    if ((uint32_t)r4 >= nrows) break;                         // uniform; rows past nrows hold +0
                    // four rows at a time: their eight broadcasts are requested together
                    f32x4_t pa[4], pb[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        pa[q] = *reinterpret_cast<const f32x4_t*>(p_tile(r4 + q, t0));
                        pb[q] = *reinterpret_cast<const f32x4_t*>(p_tile(r4 + q, t0 + 4));
                    }
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t rr = (uint32_t)(r4 + q) / a.grouping;
                        const uint32_t reach_r = a.a + rr + 1;
                        const uint32_t vis_r = reach_r < a.L ? reach_r : a.L; // uniform: what this row may see
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            const bool seen = 32 * g + t0 + i < vis_r;
#pragma unroll
                            for (int c = 0; c < DL; ++c)
                                o[r4 + q][c] = seen ? __builtin_fmaf(i < 4 ? pa[q][i & 3] : pb[q][i & 3], value[i][c], o[r4 + q][c])
                                                    : o[r4 + q][c];
                        }
                    }
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // p_tile is rewritten by the next group
        }
        // the waves' partial outputs meet in LDS: the vector part, then the matrix-core part on
        // top of it (LDS operations of a wave complete in order)
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
            for (int c = 0; c < DL; ++c) o_part(wave, r, lane + 64 * c) = o[r][c];
#pragma unroll
        for (int dt = 0; dt < DT16; ++dt)
#pragma unroll
            for (int j = 0; j < 4; ++j) o_part(wave, l16, dt * 16 + 4 * kg + j) += om[dt][j];
        __syncthreads();
        // thread = (tile row, feature): 16 x D outputs over 512 threads
        for (uint32_t idx = threadIdx.x; idx < 16 * DL * 64; idx += 512) {
            const uint32_t r = idx / (DL * 64), d = idx - r * (DL * 64);
            if (r >= nrows || d >= head_dim) continue;
            float sum = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; ++w) sum += o_part(w, r, d);
            if (PHASE == 2) {
                // [pair][share][row][D] partial sums of the workspace
                a.decode_sums[((((uint64_t)p * a.Hkv + hkv) * shares + share) * 16 + r) * head_dim + d] = sum;
                continue;
            }
            if (sum == 0.0f) sum = 0.0f;                                   // -0 is stored as +0
            const uint32_t rr = r / a.grouping, hh = hkv * a.grouping + (r - rr * a.grouping);
            const float* ws = &wave_stats[0][r][0];
            // the row's class again, from the merged per-wave statistics
            bool nan = false, finite = false;
            uint32_t pinf = 0;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                nan = nan || ws[w * 16 * 5 + 3] != 0.0f;
                finite = finite || ws[w * 16 * 5 + 4] != 0.0f;
                pinf += as_u32(ws[w * 16 * 5 + 2]);
            }
            const bool nan_out = nan || (pinf == 0 && !finite);
            const uint32_t col = hh * head_dim + d;
            uint8_t* ob = a.out + plane[3] * a.out_plane_bytes
                    + (uint64_t)(rr >> 4) * a.out_tile_cols * kTileBytes + (rr & 15u) * kRowBytes;
            *reinterpret_cast<uint16_t*>(ob + (uint64_t)(col >> 4) * kTileBytes + (col & 15u) * 2) =
                    (uint16_t)(nan_out ? 0x7FC0u : bf16_rne_sw(as_u32(sum)));
        }
    }
}

// The partial sums of the shares of one KV head, added in share order, and the rows' classes
// from the joined statistics: the rows of sdpa_decode in two launches.
__global__ __launch_bounds__(512) void sdpa_decode_join_kernel(const SdpaArgs a, uint32_t shares) {
    const uint32_t hkv = blockIdx.x, p = a.plane0 + blockIdx.y;
    const uint32_t nrows = a.grouping * a.R;
    const uint64_t pair = (uint64_t)p * a.Hkv + hkv;
    uint64_t plane[4];
    walk_planes(a.walk, p, plane);
    for (uint32_t idx = threadIdx.x; idx < nrows * a.D; idx += 512) {
        const uint32_t r = idx / a.D, d = idx - r * a.D;
        float sum = 0.0f;
        bool nan = false, finite = false;
        uint32_t pinf = 0;
        for (uint32_t sh = 0; sh < shares; ++sh) {
            sum += a.decode_sums[((pair * shares + sh) * 16 + r) * a.D + d];
            const float* st = a.decode_stats + ((pair * shares + sh) * 16 + r) * 8;
            nan = nan || st[3] != 0.0f;
            finite = finite || st[4] != 0.0f;
            pinf += as_u32(st[2]);
        }
        if (sum == 0.0f) sum = 0.0f;                                       // -0 is stored as +0
        const bool nan_out = nan || (pinf == 0 && !finite);
        const uint32_t rr = r / a.grouping, hh = hkv * a.grouping + (r - rr * a.grouping);
        const uint32_t col = hh * a.D + d;
        uint8_t* ob = a.out + plane[3] * a.out_plane_bytes
                + (uint64_t)(rr >> 4) * a.out_tile_cols * kTileBytes + (rr & 15u) * kRowBytes;
        *reinterpret_cast<uint16_t*>(ob + (uint64_t)(col >> 4) * kTileBytes + (col & 15u) * 2) =
                (uint16_t)(nan_out ? 0x7FC0u : bf16_rne_sw(as_u32(sum)));
    }
}

// One wave per (row, head, plane), the arithmetic and the order of
// src/cpu/sdpa.cpp:186-336: every score a sequential sum over the features, the sum
// of exponentials sequential over the tokens, every output a sequential sum over
// the tokens; lanes only divide the tokens (scores) or the features (outputs).
__global__ __launch_bounds__(64) void sdpa_rows_kernel(const SdpaArgs a) {
    __shared__ float pbuf[64];
    const uint32_t lane = threadIdx.x;
    // blockIdx.y walks the (plane, KV head) pairs, blockIdx.x the rows of the pair's query heads
    const uint32_t pairs = a.planes * a.Hkv, per_pair = a.grouping * a.R;
    for (uint32_t pair = blockIdx.y; pair < pairs; pair += gridDim.y) {
        const uint32_t p = pair / a.Hkv, hkv = pair - p * a.Hkv;
        for (uint32_t it = blockIdx.x; it < per_pair; it += gridDim.x) {
            const uint32_t hg = it / a.R, row = it - hg * a.R;
            sdpa_reference_row(a, p, hkv, hkv * a.grouping + hg, row, lane, pbuf);
        }
    }
}

namespace {

struct SdpaShape {
    uint64_t Hq, Hkv, R, C, D, planes;
    uint32_t leading;
};

int sdpa_shape(const iomx_view* q, const iomx_view* k, const iomx_view* v, const iomx_view* out,
               uint64_t a, uint64_t L, SdpaShape* s) {
    IOMX_TRY(check_view(q, 16));
    IOMX_TRY(check_view(k, 16));
    IOMX_TRY(check_view(v, 16));
    IOMX_TRY(check_view(out, 16));
    if (q->rank < 3 || k->rank != q->rank || v->rank != q->rank || out->rank != q->rank - 1) return IOMX_ERR_INVALID;
    const uint32_t leading = q->rank - 3;
    const Matrix qm = matrix_of(*q), km = matrix_of(*k), vm = matrix_of(*v), om = matrix_of(*out);
    s->leading = leading;
    s->Hq = q->dims[leading];
    s->Hkv = k->dims[leading];
    s->R = qm.rows;
    s->D = qm.cols;
    s->C = km.rows;
    if (km.cols != s->D || v->dims[leading] != s->Hkv || vm.rows != s->C || vm.cols != s->D) return IOMX_ERR_INVALID;
    if (s->Hq == 0 || s->Hkv == 0 || s->Hq % s->Hkv != 0) return IOMX_ERR_INVALID;
    uint64_t width;
    if (mul_overflows(s->Hq, s->D, &width) || om.rows != s->R || om.cols != width) return IOMX_ERR_INVALID;
    s->planes = 1;
    for (uint32_t i = 0; i < leading; ++i) {
        if (k->dims[i] != q->dims[i] || v->dims[i] != q->dims[i] || out->dims[i] != q->dims[i]) return IOMX_ERR_INVALID;
        if (mul_overflows(s->planes, q->dims[i], &s->planes)) return IOMX_ERR_OVERFLOW;
    }
    if (L == 0 || L > s->C || a >= s->C || s->R > s->C - a) return IOMX_ERR_INVALID;
    if (out->base == q->base || out->base == k->base || out->base == v->base) return IOMX_ERR_INVALID;
    if (s->C > 0x7FFFFFF0ull || width > 0x7FFFFFF0ull || s->planes > 0x7FFFFFF0ull) return IOMX_ERR_OVERFLOW;
    return IOMX_OK;
}

constexpr uint64_t kMaxMfmaHeadDim = 128;

// all rows of the query heads of one KV head fit one 16-row tile: the decode kernel
bool sdpa_few_rows(const SdpaShape& s) { return (s.Hq / s.Hkv) * s.R <= kTile && s.D <= kMaxMfmaHeadDim; }

// Workgroups that share the token groups of one KV head in a decode step (sdpa_decode): one,
// unless the prefix is long and planes * Hkv workgroups would leave most CUs idle; then enough
// for about one workgroup per CU, each with at least 16 groups (two per wave).
uint32_t sdpa_decode_shares(const SdpaShape& s, uint64_t a, uint64_t L) {
    const uint64_t reach = a + s.R, vis = reach < L ? reach : L;
    const uint64_t groups = (vis + 31) / 32, heads = s.planes * s.Hkv;
    if (groups < 64 || heads >= 128) return 1;
    uint64_t shares = 256 / heads;
    if (shares > groups / 16) shares = groups / 16;
    if (shares > 64) shares = 64;
    return (uint32_t)(shares > 1 ? shares : 1);
}

// Workspace of a decode step in shares: [pair][share][16 rows][8] statistics, then
// [pair][share][16 rows][D] partial sums, binary32.
uint64_t sdpa_decode_stats_floats(const SdpaShape& s, uint32_t shares) { return s.planes * s.Hkv * shares * 16 * 8; }
uint64_t sdpa_decode_workspace(const SdpaShape& s, uint32_t shares) {
    return (sdpa_decode_stats_floats(s, shares) + s.planes * s.Hkv * shares * 16 * s.D) * 4;
}

// Workgroups that share the packing of one KV head: enough of them to occupy the
// chip when planes * Hkv alone would not.
uint32_t sdpa_pack_splits(const SdpaShape& s, uint64_t L) {
    const uint64_t frags = ((L + 31) / 32) * ((s.D + 15) / 16);
    const uint64_t heads = s.planes * s.Hkv;
    uint64_t splits = heads >= 4096 ? 1 : (4096 + heads - 1) / heads;
    const uint64_t most = (frags + 3) / 4;
    if (splits > most) splits = most;
    if (splits > 64) splits = 64;
    return (uint32_t)(splits ? splits : 1);
}

// header (one flag word per plane, KV head and pack split, rounded up to 256 bytes),
// the V fragments, then the flushed K tiles (the same number of bytes)
int sdpa_layout(const SdpaShape& s, uint64_t L, uint64_t* header, uint64_t* region, uint64_t* bytes) {
    uint64_t heads = s.planes, n, h, total;
    if (mul_overflows(heads, s.Hkv, &heads)) return IOMX_ERR_OVERFLOW;
    if (mul_overflows(heads, (uint64_t)sdpa_pack_splits(s, L) * 4, &h) || h > ~0ull - 255) return IOMX_ERR_OVERFLOW;
    h = (h + 255) & ~255ull;
    if (mul_overflows(heads, (L + 31) / 32, &n) || mul_overflows(n, (s.D + 15) / 16, &n)
        || mul_overflows(n, (uint64_t)kFrag, &n) || mul_overflows(n, (uint64_t)2, &total)
        || total > ~0ull - h)
        return IOMX_ERR_OVERFLOW;
    *header = h;
    *region = n;
    *bytes = total + h;
    return IOMX_OK;
}

}  // namespace

}  // namespace iomx

using namespace iomx;

extern "C" int iomx_sdpa_workspace(int dtype, const iomx_view* q, const iomx_view* k, const iomx_view* v,
                                   const iomx_view* out, uint64_t a, uint64_t L, uint64_t* bytes,
                                   uint64_t* alignment) {
    if (!bytes || !alignment) return IOMX_ERR_INVALID;
    SdpaShape s;
    IOMX_TRY(sdpa_shape(q, k, v, out, a, L, &s));
    if (dtype != IOMX_DT_BF16) return IOMX_ERR_UNSUPPORTED;
    *alignment = 256;
    if (s.D <= kMaxMfmaHeadDim && sdpa_few_rows(s)) {
        const uint32_t shares = sdpa_decode_shares(s, a, L);
        if (shares > 1) { *bytes = sdpa_decode_workspace(s, shares); return IOMX_OK; }
    }
    if (s.D > kMaxMfmaHeadDim || sdpa_few_rows(s)) { *bytes = 0; *alignment = 1; return IOMX_OK; }
    uint64_t header, region;
    return sdpa_layout(s, L, &header, &region, bytes);
}

// The launches of one attention request; `workspace` is the caller's buffer
// (iomx_launch_sdpa) or this device's copy of the fixed array (iomx_launch_sdpa_static).
static int sdpa_launch(int dtype, const iomx_view* q, const iomx_view* k, const iomx_view* v,
                       const iomx_view* out, uint64_t a, uint64_t L, void* workspace,
                       uint64_t workspace_bytes, int path, iomx_stream_t stream) {
    SdpaShape s;
    IOMX_TRY(sdpa_shape(q, k, v, out, a, L, &s));
    if (dtype != IOMX_DT_BF16) return IOMX_ERR_UNSUPPORTED;
    if (s.D > 256) return IOMX_ERR_UNSUPPORTED;
    // path 2 = path 0 with the two-tile kernel wherever its mapping applies, however few the rows
    const bool pairs_always = path == 2;
    if (path == 2) path = 0;
    const Matrix qm = matrix_of(*q), km = matrix_of(*k), om = matrix_of(*out);
    SdpaArgs g = {};
    uint64_t strides[4][kMaxLead] = {};
    uint64_t offsets[4] = {q->plane_offset, k->plane_offset, v->plane_offset, out->plane_offset};
    for (uint32_t i = 0; i < s.leading; ++i) {
        strides[0][i] = q->plane_strides[i];
        strides[1][i] = k->plane_strides[i];
        strides[2][i] = v->plane_strides[i];
        strides[3][i] = out->plane_strides[i];
    }
    IOMX_TRY(build_walk<4>(s.leading, q->dims, strides, offsets, &g.walk));
    g.q = static_cast<const uint8_t*>(q->base);
    g.k = static_cast<const uint8_t*>(k->base);
    g.v = static_cast<const uint8_t*>(v->base);
    g.out = static_cast<uint8_t*>(out->base);
    g.q_plane_bytes = qm.plane_elems * 2;
    g.kv_plane_bytes = km.plane_elems * 2;
    g.out_plane_bytes = om.plane_elems * 2;
    g.q_head_stride = q->plane_strides[s.leading];
    g.k_head_stride = k->plane_strides[s.leading];
    g.v_head_stride = v->plane_strides[s.leading];
    g.Hq = (uint32_t)s.Hq;
    g.Hkv = (uint32_t)s.Hkv;
    g.grouping = (uint32_t)(s.Hq / s.Hkv);
    g.R = (uint32_t)s.R;
    g.C = (uint32_t)s.C;
    g.D = (uint32_t)s.D;
    g.a = (uint32_t)a;
    g.L = (uint32_t)L;
    g.d_tiles = (uint32_t)qm.tile_cols;
    g.out_tile_cols = (uint32_t)om.tile_cols;
    g.kv_tile_rows = (uint32_t)km.tile_rows;
    g.planes = (uint32_t)g.walk.planes;
    g.groups = (uint32_t)((L + 31) / 32);
    g.scale = sqrtf((float)s.D);
    {
        int e = 0;
        g.scale_pow2 = frexpf(g.scale, &e) == 0.5f ? 1u : 0u;
        g.inv_scale = 1.0f / g.scale;
        g.exp_scale = (float)(1.4426950408889634074 / (double)g.scale);
    }
    if (s.Hq > 65535u || s.R > 0x7FFFFFFFull) return IOMX_ERR_OVERFLOW;
    const hipStream_t st = native(stream);
    const uint32_t gz = g.planes < 65535u ? g.planes : 65535u;

    if (path == 0 && sdpa_few_rows(s) && s.Hkv <= 0x7FFFFFFFull) {
        const uint32_t shares = sdpa_decode_shares(s, a, L);
        if (shares > 1) {
            // (shares > 1 implies fewer than 128 planes: one launch of each phase)
            if (!workspace || workspace_bytes < sdpa_decode_workspace(s, shares)
                || (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
                return IOMX_ERR_INVALID;
            g.decode_stats = static_cast<float*>(workspace);
            g.decode_sums = g.decode_stats + sdpa_decode_stats_floats(s, shares);
        }
        // The scores of pass 1 kept in LDS for pass 2, where the K ring does not hold the whole prefix
        // anyway (more than 16 groups; 8 where the ring has one slot) and they fit beside the
        // kernel's own arrays (160 KiB per workgroup, one workgroup per CU): 128 bytes per group and
        // tile row in use.
        uint32_t kept_bytes = 0, kept_mode = 0;
        {
            const uint64_t reach = a + s.R, vis = reach < L ? reach : L, groups = (vis + 31) / 32;
            const uint64_t ring = g.d_tiles > 6 ? 8 : 16, room = 159 * 1024;
            const uint64_t arrays = 16 * 32 * 4 + 16 * ((g.d_tiles + 3) / 4) * 64 * 4;   // probabilities, partial outputs: per wave
            const uint64_t group_bytes = (uint64_t)(g.grouping * s.R) * 128;
            // a wave's area (mode 2): its ceil(groups / 8) groups, and not less than the two arrays
            uint64_t per_wave = ((groups + 7) / 8) * group_bytes;
            if (per_wave < arrays) per_wave = arrays;
            if (shares == 1 && groups > ring) {
                if (2560 + 8 * arrays + groups * group_bytes <= room) {
                    kept_mode = 1;
                    kept_bytes = (uint32_t)(groups * group_bytes);
                } else if (2560 + 8 * per_wave <= room) {
                    kept_mode = 2;
                    kept_bytes = (uint32_t)(8 * per_wave);
                    g.kept_wave_bytes = (uint32_t)per_wave;
                }
            }
        }
        for (g.plane0 = 0; g.plane0 < g.planes; g.plane0 += 65535u) {
            const dim3 grid(g.Hkv, g.planes - g.plane0 < 65535u ? g.planes - g.plane0 : 65535u, shares);
#define IOMX_SDPA_DECODE_AS(N, F) \
        if (shares == 1 && kept_mode == 1) { \
            hipLaunchKernelGGL((sdpa_decode_bf16_kernel<N, 0, 1, F>), grid, dim3(512), kept_bytes, st, g); \
        } else if (shares == 1 && kept_mode == 2) { \
            hipLaunchKernelGGL((sdpa_decode_bf16_kernel<N, 0, 2, F>), grid, dim3(512), kept_bytes, st, g); \
        } else if (shares == 1) { \
            hipLaunchKernelGGL((sdpa_decode_bf16_kernel<N, 0, 0, F>), grid, dim3(512), 0, st, g); \
        } else { \
            hipLaunchKernelGGL((sdpa_decode_bf16_kernel<N, 1, 0, F>), grid, dim3(512), 0, st, g); \
            hipLaunchKernelGGL((sdpa_decode_bf16_kernel<N, 2, 0, F>), grid, dim3(512), 0, st, g); \
            hipLaunchKernelGGL(sdpa_decode_join_kernel, dim3(grid.x, grid.y), dim3(512), 0, st, g, shares); \
        }
#define IOMX_SDPA_DECODE(N) \
    case N: \
        IOMX_SDPA_DECODE_AS(N, false) \
        break;
#define IOMX_SDPA_DECODE_EVEN(N) \
    case N: \
        if (whole_head) { IOMX_SDPA_DECODE_AS(N, true) } else { IOMX_SDPA_DECODE_AS(N, false) } \
        break;
            // head sizes that are whole multiples of 32 (64 and 128 are the model families') as
            // compile-time constants
            const bool whole_head = g.D == g.d_tiles * 16;
            switch (g.d_tiles) {
                IOMX_SDPA_DECODE(1) IOMX_SDPA_DECODE_EVEN(2) IOMX_SDPA_DECODE(3) IOMX_SDPA_DECODE_EVEN(4)
                IOMX_SDPA_DECODE(5) IOMX_SDPA_DECODE_EVEN(6) IOMX_SDPA_DECODE(7)
                default:
                    if (whole_head) { IOMX_SDPA_DECODE_AS(8, true) } else { IOMX_SDPA_DECODE_AS(8, false) }
                    break;
            }
#undef IOMX_SDPA_DECODE
#undef IOMX_SDPA_DECODE_EVEN
#undef IOMX_SDPA_DECODE_AS
        }
        record_launch("sdpa_decode", g.Hkv * gz * shares, 512, (uint64_t)g.planes * g.Hq * g.R);
        IOMX_HIP(hipGetLastError());
        return IOMX_OK;
    }
    bool matrix_cores = path == 0 && s.D <= kMaxMfmaHeadDim;
    uint64_t header = 0, region = 0;
    if (matrix_cores) {
        uint64_t need;
        IOMX_TRY(sdpa_layout(s, L, &header, &region, &need));
        if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
            return IOMX_ERR_INVALID;
        if (s.Hkv > 65535u || (s.R + kTile - 1) / kTile > 65535u) matrix_cores = false;
    }
    if (matrix_cores) {
        // few row tiles against a long prefix: the waves of a workgroup split the tokens,
        // and when all rows of a KV head's query heads fit one tile they share it
        const uint32_t row_tiles = (g.R + kTile - 1) / kTile;
        int mode = 0;
        const bool four_heads_share = (g.D == 64 || g.D == 128) && g.grouping % 4 == 0;
        if (pairs_always && four_heads_share) mode = 2;
        else if ((uint64_t)row_tiles * g.Hq * g.planes < 4096 && g.groups >= 8) mode = 1;
        else if (four_heads_share) mode = 2;
        else if ((g.D == 64 || g.D == 128) && row_tiles >= 4) mode = 3;
        g.flags = static_cast<uint32_t*>(workspace);
        g.packed_v = static_cast<uint8_t*>(workspace) + header;
        g.packed_k = g.packed_v + region;
        g.pack_splits = sdpa_pack_splits(s, L);
        hipLaunchKernelGGL(sdpa_pack_kernel, dim3(g.Hkv * g.pack_splits, gz), dim3(256), 0, st, g);
        const bool full_d = (g.D & 31u) == 0;
        // two row tiles per wave from 1024 rows on (measured on one sequence of 4096 rows against the
        // one-tile kernel in the same process: 2 % at D = 64, 8 % at D = 128; at 512 rows no gain)
        const bool in_pairs = mode == 2 && (pairs_always || row_tiles >= 64);
        for (g.plane0 = 0; g.plane0 < g.planes; g.plane0 += 65535u) {
        const uint32_t layers = g.planes - g.plane0 < 65535u ? g.planes - g.plane0 : 65535u;
        const dim3 grid(mode == 1 || mode == 3 ? g.Hq : (g.Hq + 3) / 4, layers, mode == 3 ? (row_tiles + 3) / 4 : row_tiles);
#define IOMX_SDPA_MODE(N, M) \
    if (full_d) hipLaunchKernelGGL((sdpa_mfma_bf16_kernel<N, M, true>), grid, dim3(sdpa_waves(N, M) * 64), 0, st, g); \
    else hipLaunchKernelGGL((sdpa_mfma_bf16_kernel<N, M, false>), grid, dim3(sdpa_waves(N, M) * 64), 0, st, g)
#define IOMX_SDPA(N) \
    case N: \
        if (mode == 1) { IOMX_SDPA_MODE(N, 1); } \
        else { IOMX_SDPA_MODE(N, 0); } \
        break;
        if (in_pairs) {
            const dim3 pairs(g.Hq / 4, layers, (row_tiles + 1) / 2);
            if (g.d_tiles == 4) hipLaunchKernelGGL((sdpa_mfma_pair_bf16_kernel<4>), pairs, dim3(256), 0, st, g);
            else hipLaunchKernelGGL((sdpa_mfma_pair_bf16_kernel<8>), pairs, dim3(256), 0, st, g);
        } else if (mode == 2 && g.d_tiles == 4)
            hipLaunchKernelGGL((sdpa_mfma_bf16_kernel<4, 2, true>), grid, dim3(256), 0, st, g);
        else if (mode == 2)
            hipLaunchKernelGGL((sdpa_mfma_bf16_kernel<8, 2, true>), grid, dim3(256), 0, st, g);
        else if (mode == 3 && g.d_tiles == 4)
            hipLaunchKernelGGL((sdpa_mfma_bf16_kernel<4, 3, true>), grid, dim3(256), 0, st, g);
        else if (mode == 3)
            hipLaunchKernelGGL((sdpa_mfma_bf16_kernel<8, 3, true>), grid, dim3(256), 0, st, g);
        else switch (g.d_tiles) {
            IOMX_SDPA(1) IOMX_SDPA(2) IOMX_SDPA(3) IOMX_SDPA(4)
            IOMX_SDPA(5) IOMX_SDPA(6) IOMX_SDPA(7)
            default: IOMX_SDPA(8)
        }
#undef IOMX_SDPA_MODE
#undef IOMX_SDPA
        }
        if (in_pairs) record_launch("sdpa_mfma_pair", (row_tiles + 1) / 2 * (g.Hq / 4) * gz, 256, (uint64_t)g.planes * g.Hq * g.R);
        else record_launch("sdpa_mfma", (mode == 3 ? (row_tiles + 3) / 4 : row_tiles) * (mode == 1 || mode == 3 ? g.Hq : (g.Hq + 3) / 4) * gz, 256,
                           (uint64_t)g.planes * g.Hq * g.R);
        IOMX_HIP(hipGetLastError());
        return IOMX_OK;
    }
    // the reference-order kernel: one grid row per (plane, KV head) pair
    const uint64_t pairs = (uint64_t)g.planes * g.Hkv, per_pair = (uint64_t)g.grouping * g.R;
    if (pairs > 0x7FFFFFFFull || per_pair > 0x7FFFFFFFull) return IOMX_ERR_OVERFLOW;
    const uint32_t gy = (uint32_t)(pairs < 65535 ? pairs : 65535);
    const dim3 rows_grid((uint32_t)(per_pair < 65535 ? per_pair : 65535), gy);
    hipLaunchKernelGGL(sdpa_rows_kernel, rows_grid, dim3(64), 0, st, g);
    record_launch("sdpa_rows", rows_grid.x * rows_grid.y, 64, pairs * per_pair);
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}

extern "C" int iomx_launch_sdpa(int dtype, const iomx_view* q, const iomx_view* k, const iomx_view* v,
                                const iomx_view* out, uint64_t a, uint64_t L, void* workspace,
                                uint64_t workspace_bytes, int path, iomx_stream_t stream) {
    return sdpa_launch(dtype, q, k, v, out, a, L, workspace, workspace_bytes, path, stream);
}

// ---- attention without a caller workspace and without any allocation ----------
//
// The packed V fragments / flushed K tiles of a prefill (or the shares' statistics
// and partial sums of a long-prefix decode step) go into a fixed array that the code
// object itself carries, one copy per GPU.  In host code the array's name is only a
// handle for hipGetSymbolAddress: the address a kernel may use is looked up once per
// device, with that device current, and kept.

static __device__ __align__(256) unsigned char scratch[IOMX_SDPA_STATIC_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_address[kMaxDevices];

// The first call on a device looks the address up, and a symbol lookup is not a call to make
// under stream capture: there the request is refused (make one eager call first, or any call on
// another stream), so that a captured call is launches only.
int scratch_of_current_device(hipStream_t stream, void** address) {
    int device = -1;
    IOMX_HIP(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return IOMX_ERR_UNSUPPORTED;
    void* known = g_scratch_address[device].load(std::memory_order_acquire);
    if (known == nullptr) {
        if (stream != nullptr) {
            hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
            IOMX_HIP(hipStreamIsCapturing(stream, &capture));
            if (capture != hipStreamCaptureStatusNone) return IOMX_ERR_INVALID;
        }
        IOMX_HIP(hipGetSymbolAddress(&known, HIP_SYMBOL(scratch)));
        if (known == nullptr || (reinterpret_cast<uintptr_t>(known) & 255u) != 0) return IOMX_ERR_INVALID;
        g_scratch_address[device].store(known, std::memory_order_release);
    }
    *address = known;
    return IOMX_OK;
}
}  // namespace

extern "C" int iomx_launch_sdpa_static(int dtype, const iomx_view* q, const iomx_view* k,
                                       const iomx_view* v, const iomx_view* out, uint64_t a,
                                       uint64_t L, int path, iomx_stream_t stream) {
    uint64_t need = 0, alignment = 1;
    IOMX_TRY(iomx_sdpa_workspace(dtype, q, k, v, out, a, L, &need, &alignment));
    if (path == 1) need = 0;  // the reference-order kernel keeps nothing outside its operands
    if (need > IOMX_SDPA_STATIC_BYTES) return IOMX_ERR_EXHAUSTED;
    void* address = nullptr;
    IOMX_TRY(scratch_of_current_device(native(stream), &address));
    // Every word of the part in use is written by the pack kernel (or by the first two
    // decode phases) before it is read in the same call, so what an earlier call left
    // in the array needs no clearing.
    return sdpa_launch(dtype, q, k, v, out, a, L, address, IOMX_SDPA_STATIC_BYTES, path, stream);
}
