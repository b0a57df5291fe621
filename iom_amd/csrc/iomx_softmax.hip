// The softmax stage of attention: binary32 scores in, BF16 probabilities out.
//
// One wave owns one row.  In the fast kernel the lane holds the whole row in
// registers (K 128-bit loads, fully coalesced across the wave), so HBM sees
// every visible score once and every probability once; the maximum and the sum
// are wave-wide butterfly reductions.  Rows are independent: a workgroup is one wave
// with one row, without LDS or barriers.
//
//   softmax_rows     unit column strides, 16-byte aligned score rows, at most
//                    4096 physical columns.
//   softmax_generic  any strides and lengths: three strided passes per row.
#include "iomx_common.hpp"

namespace iomx {

struct SoftmaxArgs {
    const float* scores;
    uint16_t* p;
    iomx_stage_layout sl, pl;
    uint64_t rows;       // logical rows per head
    uint64_t a, L;
    uint64_t heads;
    uint64_t total_rows; // planes * heads * pl.rows
    float scale;
    // 32-bit copies for the row kernel (all fit when it is selected)
    uint32_t rows32, prows32, heads32, pcols32, scols32, L32, a32;
    FastDiv div_prows, div_heads;
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m));
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = v + __shfl_xor(v, m);
    return v;
}

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = v + __shfl_xor(v, m);
    return v;
}

constexpr uint32_t kNegInf = 0xFF800000u;
constexpr uint32_t kPosInf = 0x7F800000u;

__device__ __forceinline__ uint64_t stage_offset(const iomx_stage_layout& l, uint64_t plane,
                                                 uint64_t head, uint64_t row) {
    return l.plane_offset + plane * l.plane_stride + head * l.head_stride + row * l.row_stride;
}

template <int K>
__global__ __launch_bounds__(64) void softmax_rows_kernel(const SoftmaxArgs a) {
    const uint32_t lane = threadIdx.x;
    const uint32_t g = blockIdx.x;   // the grid has one workgroup of one wave per row
    // row -> (plane, head, r) with multiply-shift divisions
    uint32_t ph = g, r = 0;
    if (a.prows32 > 1) {
        ph = fast_div(g, a.div_prows);
        r = g - ph * a.prows32;
    }
    uint32_t plane = ph, head = 0;
    if (a.heads32 > 1) {
        plane = fast_div(ph, a.div_heads);
        head = ph - plane * a.heads32;
    }
    uint16_t* prow = a.p + stage_offset(a.pl, plane, head, r);
    uint32_t visible = 0;
    if (r < a.rows32) {
        const uint32_t reach = a.a32 + r + 1;  // a32 <= L32 <= 4096: no wrap
        visible = reach < a.L32 ? reach : a.L32;
    }
    const float* srow = a.scores + stage_offset(a.sl, plane, head, r < a.rows32 ? r : 0);

    // All K loads are issued before anything looks at a loaded value: with a branch or a
    // select on the loaded registers between two loads the compiler waits for each load
    // before it issues the next, and a wave then has one 1 KiB request in flight instead
    // of K.  So every lane loads unconditionally -- from its own chunk where at least one
    // of its four scores is visible and the chunk lies inside the physical row, from the
    // start of the row otherwise (always readable: the row has at least four columns; one
    // cache line for all such lanes) -- and the masks are applied afterwards.  A 256-column
    // chunk past the visible limit (the same for every lane) thus costs one line instead of
    // 1 KiB of traffic, and nothing is compared or, below, exponentiated for it.
    u32x4 raw[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = (k * 64u + lane) * 4u;
        const bool mine = col < visible && col + 4 <= a.scols32;
        raw[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(srow + (mine ? col : 0u)));
    }
    float s[K][4];
    bool has_nan = false;
    float vmax = as_f32(kNegInf);
#pragma unroll
    for (int k = 0; k < K; ++k) {
        if (k * 256u >= visible) {                         // uniform: nothing of this chunk is seen
#pragma unroll
            for (int j = 0; j < 4; ++j) s[k][j] = as_f32(kNegInf);
            continue;
        }
        float x[4] = {as_f32(raw[k].x) * a.scale, as_f32(raw[k].y) * a.scale,
                      as_f32(raw[k].z) * a.scale, as_f32(raw[k].w) * a.scale};
        if ((k + 1) * 256u > visible || (k + 1) * 256u > a.scols32) {
            // uniform: the visible range or the physical row ends inside this chunk
            const uint32_t col = (k * 64u + lane) * 4u;
            const uint32_t nvis = visible > col ? visible - col : 0u;
            if (col < visible && col + 4 > a.scols32) {
                // the physical row ends inside this lane's four scores: element by element (at
                // most one lane of a row, and only where the row length is not a multiple of four)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if ((uint32_t)j < nvis) x[j] = srow[col + j] * a.scale;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) x[j] = (uint32_t)j < nvis ? x[j] : as_f32(kNegInf);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) s[k][j] = x[j];
        // one unordered compare sees a NaN in either of two scores; fmaxf skips NaN
        has_nan = has_nan || __builtin_isunordered(x[0], x[1]) || __builtin_isunordered(x[2], x[3]);
        vmax = fmaxf(fmaxf(vmax, x[0]), fmaxf(x[1], fmaxf(x[2], x[3])));
    }
    const bool row_nan = __any(has_nan);
    const float m = wave_max(vmax);
    const bool poisoned = row_nan || as_u32(m) == kNegInf;
    if (poisoned || as_u32(m) == kPosInf) {
        // rare rows: NaN / all -inf -> NaN over the visible range; k scores of +inf
        // share 1/k; everything at or beyond the visible limit is +0
        float share = as_f32(kQuietNanF32);
        if (!poisoned) {
            uint32_t cnt = 0;
#pragma unroll
            for (int k = 0; k < K; ++k)
#pragma unroll
                for (int j = 0; j < 4; ++j) cnt += as_u32(s[k][j]) == kPosInf ? 1u : 0u;
            share = 1.0f / (float)wave_sum_u32(cnt);
        }
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool seen = (k * 64u + lane) * 4u + j < visible;
                const float v = (poisoned || as_u32(s[k][j]) == kPosInf) ? share : 0.0f;
                s[k][j] = seen ? v : 0.0f;
            }
    } else {
        float part = 0.0f;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (k * 256u >= visible) continue;            // uniform; stored as +0 below
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float e = exp_nonpos(s[k][j] - m);  // +0 for masked and -inf scores
                s[k][j] = e;
                part = part + e;
            }
        }
        // e * (1/sum) instead of e / sum: at most one binary32 unit apart, which a
        // BF16 result shows only at a rounding boundary.  A masked score's +0 stays +0.
        const float inv_sum = 1.0f / wave_sum(part);
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (k * 256u >= visible) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j) s[k][j] = s[k][j] * inv_sum;
        }
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint32_t col = (k * 64u + lane) * 4u;
        if (col >= a.pcols32) continue;
        uint32_t lo = 0, hi = 0;                           // a chunk nobody sees is +0
        if (k * 256u < visible) {                          // uniform
            lo = pack_bf16(s[k][0], s[k][1]);
            hi = pack_bf16(s[k][2], s[k][3]);
        }
        if (col + 4 <= a.pcols32) {
            __builtin_nontemporal_store(u32x2{lo, hi}, reinterpret_cast<u32x2*>(prow + col));
        } else {
            const uint32_t words[2] = {lo, hi};
            for (int j = 0; j < 4; ++j)
                if (col + j < a.pcols32)
                    prow[col + j] = (uint16_t)(words[j >> 1] >> ((j & 1) * 16));
        }
    }
}

__global__ __launch_bounds__(256) void softmax_generic_kernel(const SoftmaxArgs a) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint64_t wave = (blockIdx.x * (uint64_t)blockDim.x + threadIdx.x) >> 6;
    const uint64_t waves = ((uint64_t)gridDim.x * blockDim.x) >> 6;
    for (uint64_t g = wave; g < a.total_rows; g += waves) {
        const uint64_t r = g % a.pl.rows;
        const uint64_t ph = g / a.pl.rows;
        const uint64_t head = ph % a.heads;
        const uint64_t plane = ph / a.heads;
        uint16_t* prow = a.p + stage_offset(a.pl, plane, head, r);
        uint64_t visible = 0;
        if (r < a.rows) {
            const uint64_t reach = a.a + r + 1;
            visible = reach < a.L ? reach : a.L;
        }
        const float* srow = a.scores + stage_offset(a.sl, plane, head, r < a.rows ? r : 0);
        bool has_nan = false;
        float vmax = as_f32(kNegInf);
        uint32_t cnt = 0;
        for (uint64_t t = lane; t < visible; t += 64) {
            const float x = srow[t * a.sl.column_stride] * a.scale;
            has_nan = has_nan || (x != x);
            vmax = fmaxf(vmax, x);
            cnt += as_u32(x) == kPosInf ? 1u : 0u;
        }
        const bool row_nan = __any(has_nan);
        const float m = wave_max(vmax);
        const bool poisoned = row_nan || as_u32(m) == kNegInf;
        const uint32_t pinf = wave_sum_u32(cnt);
        float sum = 1.0f;
        if (!poisoned && pinf == 0) {
            float part = 0.0f;
            for (uint64_t t = lane; t < visible; t += 64) {
                const float x = srow[t * a.sl.column_stride] * a.scale;
                part = part + expf(x - m);
            }
            sum = wave_sum(part);
        }
        const float inv_share = pinf ? 1.0f / (float)pinf : 0.0f;
        for (uint64_t t = lane; t < a.pl.columns; t += 64) {
            float v = 0.0f;
            if (t < visible) {
                const float x = srow[t * a.sl.column_stride] * a.scale;
                if (poisoned) v = as_f32(kQuietNanF32);
                else if (pinf != 0) v = as_u32(x) == kPosInf ? inv_share : 0.0f;
                else v = expf(x - m) / sum;
            }
            prow[t * a.pl.column_stride] = (uint16_t)(pack_bf16(v, 0.0f) & 0xFFFFu);
        }
    }
}

}  // namespace iomx

using namespace iomx;

// Request checks of validate_sdpa_softmax_request (src/rocm/sdpa_softmax.hpp:64-69).
extern "C" int iomx_launch_softmax(const iomx_softmax_desc* d, iomx_stream_t stream) {
    if (!d || !d->scores || !d->p_bf16) return IOMX_ERR_INVALID;
    if (d->planes == 0 || d->heads == 0 || d->rows == 0 || d->L == 0) return IOMX_ERR_INVALID;
    const iomx_stage_layout& sl = d->scores_layout;
    const iomx_stage_layout& pl = d->probability_layout;
    if (pl.rows < d->rows || pl.columns < d->L) return IOMX_ERR_INVALID;
    if (sl.rows < d->rows || sl.columns < d->L) return IOMX_ERR_INVALID;
    if (sl.column_stride == 0 || pl.column_stride == 0) return IOMX_ERR_INVALID;
    if (!(d->scale == d->scale)) return IOMX_ERR_INVALID;
    uint64_t total;
    if (mul_overflows(d->planes, d->heads, &total) || mul_overflows(total, pl.rows, &total))
        return IOMX_ERR_OVERFLOW;
    // the largest element offset either buffer can reach must stay addressable
    const iomx_stage_layout* ls[2] = {&sl, &pl};
    for (const iomx_stage_layout* l : ls) {
        uint64_t reach = l->plane_offset, t;
        if (mul_overflows(d->planes - 1, l->plane_stride, &t) || add_overflows(reach, t, &reach)
            || mul_overflows(d->heads - 1, l->head_stride, &t) || add_overflows(reach, t, &reach)
            || mul_overflows(l->rows - 1, l->row_stride, &t) || add_overflows(reach, t, &reach)
            || mul_overflows(l->columns - 1, l->column_stride, &t) || add_overflows(reach, t, &reach)
            || reach > (1ull << 44))
            return IOMX_ERR_OVERFLOW;
    }

    SoftmaxArgs a = {};
    a.scores = d->scores;
    a.p = d->p_bf16;
    a.sl = sl;
    a.pl = pl;
    a.rows = d->rows;
    a.a = d->a;
    a.L = d->L;
    a.heads = d->heads;
    a.total_rows = total;
    a.scale = d->scale;

    const bool aligned = sl.column_stride == 1 && pl.column_stride == 1
            && (reinterpret_cast<uintptr_t>(d->scores) & 15u) == 0
            && (reinterpret_cast<uintptr_t>(d->p_bf16) & 7u) == 0
            && sl.plane_offset % 4 == 0 && sl.plane_stride % 4 == 0 && sl.head_stride % 4 == 0
            && sl.row_stride % 4 == 0
            && pl.plane_offset % 4 == 0 && pl.plane_stride % 4 == 0 && pl.head_stride % 4 == 0
            && pl.row_stride % 4 == 0;
    const hipStream_t s = native(stream);
    const uint64_t cols = pl.columns;
    if (aligned && cols <= 4096 && sl.columns >= 4 && total <= 0x7FFFFFFFull && d->rows <= 0xFFFFFFFFull
        && pl.rows <= 0xFFFFFFFFull && d->heads <= 0xFFFFFFFFull) {
        const uint32_t grid = (uint32_t)total;  // one wave per row, one-shot
        a.rows32 = (uint32_t)d->rows;
        a.prows32 = (uint32_t)pl.rows;
        a.heads32 = (uint32_t)d->heads;
        a.pcols32 = (uint32_t)cols;
        a.scols32 = (uint32_t)(sl.columns < 0xFFFFFFFFull ? sl.columns : 0xFFFFFFFFull);
        a.L32 = (uint32_t)d->L;
        a.a32 = (uint32_t)(d->a < d->L ? d->a : d->L);
        a.div_prows = make_fast_div(a.prows32);
        a.div_heads = make_fast_div(a.heads32);
        // One wave per workgroup (the dispatcher then starts and retires rows one by one instead
        // of four at a time), and fewer of them on a compute unit than its 32 wave slots: a wave
        // has K KiB of loads in flight, and past about 100 KiB per compute unit more requests in
        // flight only lengthen every wave's wait.  Measured on 2^32 scores, GB/s at the best
        // count against four-wave workgroups at theirs: rows of 4096 columns 6170 (10 per compute
        // unit) against 5400, 2048 columns 6500 (12) against 6110, 1024 columns 6250 (20) against
        // 6250, 512 columns 6500 (32) against 6330; where a row sees only a part of its columns
        // (half of them on average with a = 0) the best counts are 16, 16, 28 and 32.  The limit
        // is an LDS request that nobody uses (160 KiB per compute unit).
        const bool sees_all = a.a32 + 1 >= a.L32;
        const auto lds_for = [](uint32_t per_cu) { return (163840u / per_cu) & ~511u; };
        if (cols <= 256) hipLaunchKernelGGL(softmax_rows_kernel<1>, dim3(grid), dim3(64), 0, s, a);
        else if (cols <= 512) hipLaunchKernelGGL(softmax_rows_kernel<2>, dim3(grid), dim3(64), 0, s, a);
        else if (cols <= 1024)
            hipLaunchKernelGGL(softmax_rows_kernel<4>, dim3(grid), dim3(64), lds_for(sees_all ? 20 : 28), s, a);
        else if (cols <= 2048)
            hipLaunchKernelGGL(softmax_rows_kernel<8>, dim3(grid), dim3(64), lds_for(sees_all ? 12 : 16), s, a);
        else
            hipLaunchKernelGGL(softmax_rows_kernel<16>, dim3(grid), dim3(64), lds_for(sees_all ? 10 : 16), s, a);
        record_launch("softmax_rows", grid, 64, total);
    } else {
        const uint64_t blocks = (total + 3) / 4;
        const uint32_t grid = (uint32_t)(blocks < (1u << 20) ? blocks : (1u << 20));
        hipLaunchKernelGGL(softmax_generic_kernel, dim3(grid), dim3(256), 0, s, a);
        record_launch("softmax_generic", grid, 256, total);
    }
    IOMX_HIP(hipGetLastError());
    return IOMX_OK;
}
