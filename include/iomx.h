/*
 * iomx.h — C ABI of the MI355X (gfx950) tensor-op library, libiomx.so.
 *
 * This is the only place where HIP is reached: an IOM backend's C++ host code
 * (Device / Tensor / DeviceOps subclasses) includes this header and nothing of
 * hip_runtime.  Each entry point names the interface of the rlewczuk/iom tree
 * it stands in for (paths relative to that tree).  All functions return 0 on
 * success, a NEGATIVE iomx_status for a request this library rejects before
 * any launch, or a POSITIVE HIP error code; iomx_error_string() explains both.
 *
 * Tensors are owner storages in IOM's standard layout: leading planes in the
 * owner's row-major order, each plane 16x16-tiled (tile row, tile column, row
 * in tile, column in tile), padded to whole tiles.  A view selects planes with
 * an offset and per-axis strides counted in whole planes
 * (include/iom/tensor.hpp:262-335).  Padding slots are never written and never
 * influence a logical result.
 */
#ifndef IOMX_H
#define IOMX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status ------------------------------------------------------------- */

/* Negative values mirror the OID error classes of include/iom/oid.hpp:16-23. */
typedef enum iomx_status {
    IOMX_OK = 0,
    IOMX_ERR_INVALID = -1,     /* malformed request (std::invalid_argument)   */
    IOMX_ERR_UNSUPPORTED = -2, /* leaf or shape outside this library's scope  */
    IOMX_ERR_OVERFLOW = -3,    /* address arithmetic would overflow           */
    IOMX_ERR_EXHAUSTED = -4    /* needs more scratch than a fixed array holds */
} iomx_status;

const char* iomx_error_string(int status);

/* ---- leaves and operations --------------------------------------------- */

/* Numeric values of iom::DataType (include/iom/tensor.hpp:10-33): the 23 leaves
 * every standard tiled backend advertises (src/shared/standard_tiled_copy.hpp:17-31).
 * Elements of 2, 4 and 6 bits are packed back to back, least significant bit
 * first (src/cpu/transfer_helpers.hpp:14-40); a tile row of 16 elements is
 * always a whole number of 32-bit words.  I32, U32, F32 and BF16 arithmetic runs
 * on the bandwidth-tuned streaming kernels, every other leaf on the tile-row
 * kernels. */
enum {
    IOMX_DT_BOOL = 0,
    IOMX_DT_I2 = 1, IOMX_DT_U2 = 2, IOMX_DT_I4 = 3, IOMX_DT_U4 = 4,
    IOMX_DT_I8 = 5, IOMX_DT_U8 = 6, IOMX_DT_I16 = 7, IOMX_DT_U16 = 8,
    IOMX_DT_I32 = 9, IOMX_DT_U32 = 10, IOMX_DT_I64 = 11, IOMX_DT_U64 = 12,
    IOMX_DT_F4_E2M1 = 13, IOMX_DT_F6_E2M3 = 14, IOMX_DT_F6_E3M2 = 15,
    IOMX_DT_F8_E4M3FN = 16, IOMX_DT_F8_E5M2 = 17, IOMX_DT_F8_E8M0 = 18,
    IOMX_DT_F16 = 19, IOMX_DT_BF16 = 20, IOMX_DT_F32 = 21, IOMX_DT_F64 = 22
};

/* Order of BinaryOp in src/shared/scalar_binary_codec.hpp:9. */
enum { IOMX_OP_ADD = 0, IOMX_OP_MUL = 1, IOMX_OP_SUB = 2, IOMX_OP_DIV = 3 };

/*
 * One operand: what DeviceOps::BinaryViewSnapshot / CopyViewSnapshot carry
 * (include/iom/iom.hpp:382-401,480-511) and what the reference uploads as
 * BinaryMetadata / RmsnormMetadata / SiluMetadata
 * (src/shared/standard_tiled_add.inl:43-65,
 *  src/shared/standard_tiled_rmsnorm.inl:73-90, src/shared/gpu_queue.hpp:59-73).
 * Passed by pointer on the host and by value to the kernels: no descriptor
 * upload, no allocation.
 */
typedef struct iomx_view {
    void* base;                /* device address of the OWNER storage          */
    uint32_t rank;             /* 2..8                                         */
    uint64_t dims[8];          /* the view's logical shape                     */
    uint64_t plane_offset;     /* first selected owner plane                   */
    uint64_t plane_strides[6]; /* per leading axis, in owner planes, nonzero   */
} iomx_view;

/* ---- runtime: device, memory, streams, events --------------------------- */

typedef struct iomx_stream_s* iomx_stream_t; /* NULL = the default stream */
typedef struct iomx_event_s* iomx_event_t;

typedef struct iomx_device_props {
    char name[64];     /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
    int compute_units;
    int wavefront_size;
    int lds_bytes_per_cu;
    uint64_t global_bytes;
} iomx_device_props;

/* Stand in for the hip* calls of src/rocm/driver.hpp:20-81 and
 * src/rocm/copy.hpp:121-185. */
int iomx_device_count(int* count);
int iomx_set_device(int ordinal);
int iomx_get_device(int* ordinal);
int iomx_get_device_props(int ordinal, iomx_device_props* props);
int iomx_device_synchronize(void);

int iomx_malloc(void** ptr, size_t bytes);
int iomx_free(void* ptr);
int iomx_host_alloc(void** ptr, size_t bytes); /* pinned, for staging mirrors */
int iomx_host_free(void* ptr);
/* src/rocm/device_tensor.cpp:22-41: is this a device allocation of `ordinal`? */
int iomx_pointer_device(const void* ptr, int* ordinal);
int iomx_fill_async(void* ptr, uint8_t value, size_t bytes, iomx_stream_t stream);
int iomx_memcpy_h2d(void* dst, const void* src, size_t bytes);
int iomx_memcpy_d2h(void* dst, const void* src, size_t bytes);
int iomx_memcpy_h2d_async(void* dst, const void* src, size_t bytes, iomx_stream_t stream);
int iomx_memcpy_d2h_async(void* dst, const void* src, size_t bytes, iomx_stream_t stream);
int iomx_memcpy_d2d_async(void* dst, const void* src, size_t bytes, iomx_stream_t stream);

/* Non-blocking stream at the default priority (src/rocm/copy.hpp:151-185). */
int iomx_stream_create(iomx_stream_t* stream);
int iomx_stream_destroy(iomx_stream_t stream);
int iomx_stream_synchronize(iomx_stream_t stream);
int iomx_event_create(iomx_event_t* event, int enable_timing);
int iomx_event_destroy(iomx_event_t event);
int iomx_event_record(iomx_event_t event, iomx_stream_t stream);
int iomx_event_synchronize(iomx_event_t event);
/* *done = 1 when the event has completed, 0 while it is pending. */
int iomx_event_query(iomx_event_t event, int* done);
int iomx_event_elapsed_ms(iomx_event_t start, iomx_event_t stop, float* ms);
/*
 * Completion word: after everything submitted to the stream before this call has
 * finished, the device stores `value` to a 32-bit word in memory of iomx_host_alloc,
 * which the host may poll directly.  `device_word` is the word's address as the device
 * sees it, from iomx_host_device_address (asked once: the lookup costs more than the
 * store).  No counterpart in the reference, whose queue learns of completion from an
 * event (src/shared/gpu_queue_operations.inl:717-818); a host that waits for one short
 * operation at a time sees the word about 2 us earlier than the event.  The store is a
 * one-lane kernel (hipStreamWriteValue32 reaches the host as early, but on this runtime
 * every launch that follows one takes 10 us longer); the call costs a launch, more than
 * iomx_event_record.
 */
int iomx_host_device_address(void* host, void** device);
int iomx_stream_write_word(iomx_stream_t stream, void* device_word, uint32_t value);

/*
 * Recording and replay of a fixed sequence of launches (HIP graph).  No counterpart in
 * the reference, which submits every operation separately: a caller that repeats the
 * same sequence on the same buffers (a decode step is ~20 launches of a few
 * microseconds each) records it once between begin and end on a stream created here
 * and replays it with one submission.  Every iomx_launch_* entry point may be recorded
 * (none allocates or clears memory with a memset node); host transfers and
 * synchronisation calls may not.  Views, sizes and pointers are frozen into the
 * recording.
 */
typedef struct iomx_graph_s* iomx_graph_t;
int iomx_stream_begin_capture(iomx_stream_t stream);
int iomx_stream_end_capture(iomx_stream_t stream, iomx_graph_t* graph);
int iomx_graph_launch(iomx_graph_t graph, iomx_stream_t stream);
int iomx_graph_destroy(iomx_graph_t graph);

/* ---- operations ---------------------------------------------------------- */

/*
 * out = lhs (op) rhs with right-aligned broadcasting.  Replaces
 * launch_grid_stride_binary / launch_alias_safe_binary
 * (src/shared/standard_tiled_add.inl:445-464,297-441) behind
 * DeviceOps::binary_impl (include/iom/iom.hpp:846-956); element rule of
 * src/shared/scalar_binary_codec.hpp:120-178 over the 21 numeric leaves
 * (src/device_ops_binary.cpp:26-46; BOOL and F8_E8M0 are IOMX_ERR_UNSUPPORTED).
 * IOMX_OP_DIV takes the nine floating leaves only (src/device_ops_binary.cpp:174-175):
 * a zero or an infinity divided by its like is NaN, any other division by zero is
 * the signed overflow value of the leaf.
 * Integers wrap modulo 2^width.  Floating leaves are one IEEE operation with
 * one round-to-nearest-even encode and gradual underflow; overflow gives
 * infinity where the leaf has one and the largest finite magnitude otherwise
 * (F8_E4M3FN reserves its whole top exponent for NaN and saturates at 240, as
 * the reference codec does); every NaN result is the leaf's positive canonical
 * NaN, or the largest finite magnitude in the 4- and 6-bit leaves, which have
 * none.  F64 computes in binary64, the carrier of a device without an extended
 * type (src/shared/standard_tiled_add.inl:116).  An input that shares out's
 * storage must select exactly out's window (src/device_ops_binary.cpp:152-169);
 * anything else is rejected.
 */
int iomx_launch_binary(int op, int dtype, const iomx_view* lhs, const iomx_view* rhs,
                       const iomx_view* out, iomx_stream_t stream);

/*
 * out[...,r,:] = (x[...,r,:] / sqrt(mean(x^2)+eps)) * scale[0,:] over the 9
 * floating leaves, accumulated in F32 (in F64 for the F64 leaf,
 * src/cpu/queue.cpp:1312-1317).  Replaces standard_tiled_rmsnorm_kernel
 * (src/shared/standard_tiled_rmsnorm.inl:436-637) behind
 * DeviceOps::rmsnorm_impl; arithmetic order of src/cpu/queue.cpp:1187-1234:
 * mean = sum/F, shifted = mean+eps, root = sqrt, inverse = 1/root,
 * out = (x*inverse)*scale, no fused multiply-add.
 */
int iomx_launch_rmsnorm(int dtype, const iomx_view* x, const iomx_view* scale,
                        const iomx_view* out, float eps, iomx_stream_t stream);

/*
 * y = x * sigmoid(x) over the 9 floating leaves, evaluated in F32 (F64 for the
 * F64 leaf) with the stable two-branch form of
 * src/shared/scalar_silu.hpp:69-97.  Replaces silu_kernel
 * (src/rocm/copy.hip:1317-1454) behind DeviceOps::silu_impl.
 */
int iomx_launch_silu(int dtype, const iomx_view* x, const iomx_view* y, iomx_stream_t stream);

/*
 * y = silu(gate) * up with the intermediate rounded to the leaf exactly as the
 * two-kernel sequence stores it (src/session.cpp:2022-2028 calls silu then
 * mul).  A private fast path with no counterpart operation in the reference:
 * its result equals iomx_launch_silu followed by iomx_launch_binary(MUL).
 */
int iomx_launch_silu_mul(int dtype, const iomx_view* gate, const iomx_view* up,
                         const iomx_view* y, iomx_stream_t stream);

/*
 * sum = x + y and out = rmsnorm(sum, scale, eps) in one launch: the residual add and
 * the norm that follows it in a decoder layer (src/session.cpp:2500 then :1996).  A
 * private fast path with no counterpart operation in the reference: both outputs equal,
 * bit for bit, iomx_launch_binary(ADD) followed by iomx_launch_rmsnorm on its result,
 * while the sum crosses HBM once instead of three times.  BF16, F16 and F32; all four
 * tensors of one shape whose two matrix extents are multiples of 16; `sum` may be the
 * identical window of x or y, `out` shares storage with none of the others.  Any other
 * request is IOMX_ERR_UNSUPPORTED (make the two launches) or IOMX_ERR_INVALID.
 */
int iomx_launch_add_rmsnorm(int dtype, const iomx_view* x, const iomx_view* y,
                            const iomx_view* sum, const iomx_view* scale,
                            const iomx_view* out, float eps, iomx_stream_t stream);

/*
 * Same-spec copy of the selected planes' logical elements, any leaf.  Replaces
 * grid_stride_copy_kernel (src/shared/standard_tiled_copy_metadata.inl:241-282)
 * behind DeviceOps::copy_impl (src/device_ops_copy.cpp:9-52).
 */
int iomx_launch_copy(int dtype, const iomx_view* src, const iomx_view* dst, iomx_stream_t stream);

/*
 * Host-transfer staging: the dense logical row-major bit stream of the view's
 * shape (already in device memory) <-> the tiled view, any leaf.  Replace
 * scatter_plane_kernel / gather_plane_kernel
 * (src/shared/standard_tiled_copy.inl:286-310) under Tensor::region_from_host /
 * region_to_host (src/rocm/device_tensor.cpp:145-167).  `logical` is 4-byte
 * aligned and spans the logical byte count rounded up to 4, the size of the
 * reference's transfer workspace (src/rocm/device_tensor.cpp:136-143): the
 * kernels move whole 32-bit words, and gather stores the unused bits of the
 * last word as zero (src/cpu/tensor.cpp:126-135).
 */
int iomx_launch_scatter(int dtype, const iomx_view* dst, const void* logical, iomx_stream_t stream);
int iomx_launch_gather(int dtype, const iomx_view* src, void* logical, iomx_stream_t stream);

/*
 * destination[..., h, a + r, d] = source[..., h, r, d]: appends R rows to a cache
 * of capacity C at the explicit row offset a, any leaf, raw bits.  Replaces the
 * cache-append kernel of the standard tiled backends (src/rocm/copy.hip:132)
 * behind DeviceOps::cache_append_impl; admission of
 * src/device_ops_cache_append.cpp:160-270: ranks three to eight, equal leading
 * tuples, head counts and feature widths, a <= C and then R <= C - a, distinct
 * storages.
 */
int iomx_launch_cache_append(int dtype, const iomx_view* source, const iomx_view* destination,
                             uint64_t a, iomx_stream_t stream);

/*
 * out[..., r, f] = table[indices[..., 0, r], f]: table [V,F] of rank two, indices
 * [...,1,R] of one of the twelve integer leaves, out [...,R,F] of the table's
 * leaf; payload bits are copied unchanged.  Replaces the gather kernel of
 * src/shared/standard_tiled_embedding.inl behind DeviceOps::embedding_impl.
 * `status` is one 32-bit word of device memory (the first word of the 32-byte
 * control packet of docs/BACKEND_CONTRACT/embedding-lookup.md:178-201): the call
 * resets it to 0 in stream order, and any negative or out-of-vocabulary id sets it
 * to 1 without forming a table address; the caller transfers and interprets it
 * after completion.
 */
int iomx_launch_embedding(int dtype, int index_dtype, const iomx_view* table,
                          const iomx_view* indices, const iomx_view* out, uint32_t* status,
                          iomx_stream_t stream);

/*
 * Split-half rotary position encoding of x[..., H, R, D] into out (same shape,
 * distinct storage), row r at absolute position a + r, base theta in
 * [1, FLT_MAX], over the 9 floating leaves: frequency = pow(theta, -2c/D),
 * angle = position * frequency, out[c] = x[c] cos - x[c+D/2] sin,
 * out[c+D/2] = x[c+D/2] cos + x[c] sin, evaluated in F32 (F64 for the F64 leaf)
 * with separately rounded products; a row at position 0 is copied unchanged.
 * Replaces the kernels of src/shared/standard_tiled_rope.inl behind
 * DeviceOps::rope_impl; arithmetic of src/cpu/queue.cpp:1357-1411, admission of
 * src/device_ops_neural.cpp:241-362.
 */
int iomx_launch_rope(int dtype, const iomx_view* x, const iomx_view* out, uint64_t a, double theta,
                     iomx_stream_t stream);

/*
 * out[b,r,o] = sum_i x[b,s+r,i] * w[o,i] (ordinary: H = 1, D = O, out [...,R,O]) or
 * out[b,h,r,d] = sum_i x[b,s+r,i] * w[h*D+d,i] (head planar: O = H*D, out
 * [...,H,R,D]); w is rank two in the [out,in] orientation and is never transposed.
 * Replaces the linear kernels of the standard tiled backends behind
 * DeviceOps::linear_impl; contract docs/BACKEND_CONTRACT/linear-projections.md,
 * arithmetic of src/cpu/queue.cpp:1905-2003: integers modulo 2^N; floating leaves
 * one fused multiply-add per increasing i in F32 (F64 for F64) from +0 and one
 * encode.  path 0 lets BF16 run on the matrix cores (exact products, F32
 * accumulation in the hardware's order, one round-to-nearest-even store: the
 * "native BF16" allowance of linear-projections.md:213-218) and picks the kernel by
 * the number of rows (rows of all planes count as one row axis): 256 rows or more
 * with I % 32 == 0 and D % 16 == 0 take the workgroup-tiled kernel that stages
 * operands through LDS, fewer rows the kernel that splits the inner axis over the
 * waves of a workgroup; path 1 forces the scalar recurrence for every leaf; path 2
 * forces the BF16 matrix-core kernel that loads operands straight from global
 * memory (any shape; the fallback of path 0 and the cross-check of the other two);
 * paths 3, 4 and 5 are path 0 with the workgroup tile forced to 256 x 256 (wherever
 * there are 256 rows), 128 x 128 and 64 x 64 (path 0 picks by how many CUs the
 * problem fills), path 6 forces 128 x 128 with two groups of waves that each take
 * half of the inner axis (I % 64 == 0, else as path 0): for tests.
 */
int iomx_launch_linear(int dtype, const iomx_view* x, const iomx_view* w, const iomx_view* out,
                       uint64_t s, uint64_t R, int head_planar, uint64_t H, uint64_t D, int path,
                       iomx_stream_t stream);

/*
 * Causal grouped-query attention: q [B..,Hq,R,D], k and v [B..,Hkv,C,D] (Hq % Hkv
 * == 0, kv head of h = h / (Hq/Hkv)), out [B..,R,Hq*D]; row r attends to the
 * tokens t < min(L, a+r+1) of the initialised prefix L <= C.  Replaces the attention
 * kernels behind DeviceOps::sdpa_impl (include/iom/iom.hpp:368-373,913-922; the
 * reference's ROCm chain src/rocm/sdpa*.hip is wave32 WMMA for gfx12 only).
 * Contract docs/BACKEND_CONTRACT/scaled-dot-product-attention.md, arithmetic of
 * src/cpu/sdpa.cpp:186-336: BF16 only (any other leaf -2); scores in F32 divided by
 * sqrtf(D); NaN / +inf / all -inf rows by the special-row rules; the normalised
 * probability rounded once to BF16; P x V in F32, -0 stored as +0, one BF16
 * rounding; subnormal Q, K, P and V operands flushed to signed zero; the cache
 * tail [L,C), future tokens and tile padding are never read.
 *
 * iomx_sdpa_workspace is the pure requirement query (sdpa_workspace_requirements):
 * the bytes and alignment of caller workspace iomx_launch_sdpa needs for these
 * operands.  Requests whose rows fit one 16-row tile per KV head ((Hq/Hkv)*R <= 16, a
 * decode step) and heads wider than 128 need none (0 bytes, alignment 1) -- except a
 * decode step of few sequences against a long prefix (2048 tokens or more, fewer than
 * 128 planes x KV heads), whose token groups are shared out over several workgroups per
 * KV head: that one needs 32 + 4*D bytes per plane, KV head, share and tile row for the
 * shares' statistics and partial sums (256-byte aligned, no initialisation); every other
 * request needs the packed V fragments and flushed K tiles of the visible prefix and
 * one flag word per plane, KV head and pack share (256-byte aligned, no
 * initialisation).  path 0: the decode kernel (one launch: scores on the matrix cores,
 * P*V on the vector units straight from the cache) for the few-row requests, else the
 * pack kernel and the matrix-core kernel (D <= 128), which forms the rows of a KV head
 * whose V holds an infinity or NaN in the reference's order instead; path 1 runs the
 * reference-order kernel alone (D <= 256, no workspace); path 2 is path 0 with the kernel
 * that gives a wave two row tiles (chosen by path 0 from 1024 rows on, where four query
 * heads share a KV head and D is 64 or 128) for any number of rows: for tests.
 */
int iomx_sdpa_workspace(int dtype, const iomx_view* q, const iomx_view* k, const iomx_view* v,
                        const iomx_view* out, uint64_t a, uint64_t L, uint64_t* bytes,
                        uint64_t* alignment);
int iomx_launch_sdpa(int dtype, const iomx_view* q, const iomx_view* k, const iomx_view* v,
                     const iomx_view* out, uint64_t a, uint64_t L, void* workspace,
                     uint64_t workspace_bytes, int path, iomx_stream_t stream);

/*
 * iomx_launch_sdpa for callers that cannot allocate or bring a workspace (code under
 * HIP graph capture, serving loops and harnesses in which hipMalloc is forbidden).  It
 * has no counterpart in the reference, where the caller always leases the workspace
 * from the device arena.  Same operands, same kernels, same bits as iomx_launch_sdpa;
 * what that entry point keeps in the caller's workspace goes into a fixed array of
 * IOMX_SDPA_STATIC_BYTES that the library's code object carries once per GPU until the
 * process ends.  No hipMalloc, hipFree or allocating call is made.  A request whose
 * iomx_sdpa_workspace figure exceeds IOMX_SDPA_STATIC_BYTES returns IOMX_ERR_EXHAUSTED
 * before any launch.  The address of the array on the current device is looked up on
 * the first call made on that device (not under capture; later calls may be captured).
 * All calls on one GPU share the one array: calls that overlap in time on the same GPU,
 * from several streams or threads, race; calls in one stream's order do not.
 */
#define IOMX_SDPA_STATIC_BYTES (16u << 20)
int iomx_launch_sdpa_static(int dtype, const iomx_view* q, const iomx_view* k, const iomx_view* v,
                            const iomx_view* out, uint64_t a, uint64_t L, int path,
                            iomx_stream_t stream);

/* Element strides of one softmax-stage buffer (src/rocm/sdpa_softmax.hpp:14-22). */
typedef struct iomx_stage_layout {
    uint64_t plane_offset, plane_stride, head_stride, row_stride, column_stride;
    uint64_t rows, columns; /* physical region the stage may write */
} iomx_stage_layout;

/*
 * The softmax stage of attention: F32 scores in, BF16 probabilities out.
 * Replaces launch_sdpa_softmax (src/rocm/sdpa_softmax.hpp:36-80,
 * src/rocm/sdpa_softmax.hip:109-198); arithmetic of src/cpu/sdpa.cpp:214-309.
 * Row r sees tokens t < min(L, a+r+1).  A row with a NaN or with only -inf
 * becomes NaN; k scores of +inf share 1/k; otherwise exp(s-max)/sum, rounded to
 * BF16 once.  Everything outside the visible range, and every physical row or
 * column beyond the logical extent, is stored as +0.
 */
typedef struct iomx_softmax_desc {
    uint64_t planes, heads, rows;
    uint64_t a, L;
    float scale;
    const float* scores;
    uint16_t* p_bf16;
    iomx_stage_layout scores_layout;
    iomx_stage_layout probability_layout;
} iomx_softmax_desc;

int iomx_launch_softmax(const iomx_softmax_desc* desc, iomx_stream_t stream);

/* ---- introspection (no counterpart in the reference) --------------------- */

/* Which kernel family the last successful launch on this thread selected
 * ("binary_planes", "binary_rowvec", "binary_general", "rows_binary", ...), and
 * its grid. */
typedef struct iomx_launch_info {
    char kernel[48];
    uint32_t grid, block;
    uint64_t work_items;
} iomx_launch_info;
int iomx_last_launch(iomx_launch_info* info);

#ifdef __cplusplus
}
#endif
#endif /* IOMX_H */
