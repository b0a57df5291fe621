/*
 * iomx_probe.h -- measurement and self-test entry points of libiomx_probe.so.
 *
 * Not part of the backend: libiomx.so holds the operations and the runtime, this
 * library holds what the benchmark and the tests need beside them -- bare bandwidth
 * streams in the launch shape of the elementwise kernels, and device self-tests of the
 * conversions and packed arithmetic those kernels are built from.  Nothing in the
 * reference corresponds to it.  Status codes and iomx_stream_t are those of iomx.h.
 */
#ifndef IOMX_PROBE_H
#define IOMX_PROBE_H

#include "iomx.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Bandwidth probes (no counterpart in the reference): one launch of a bare stream over
 * `bytes` bytes per operand (a multiple of 4096, operands 16-byte aligned), in the launch
 * shape of the elementwise kernels -- one 128-bit chunk per lane, one-shot grid,
 * nontemporal access -- and with nothing else in the kernel.  They measure what this GPU
 * gives a read-only stream (a), a write-only stream (out), a copy (a -> out) and a
 * two-read-one-write stream (a + b -> out, 32-bit integer adds), which is the practical
 * ceiling the operation kernels are compared with.  READ needs `out` only as a pointer to
 * 4 KiB of writable memory that it never writes.  HELD_COPY is the memory side of the
 * resident RMSNorm kernel alone (a -> out; bytes a multiple of 64 KiB): 1024-lane workgroups
 * that load four chunks per lane, meet at a barrier and store.
 */
enum { IOMX_PROBE_READ = 0, IOMX_PROBE_WRITE = 1, IOMX_PROBE_COPY = 2, IOMX_PROBE_ADD = 3,
       IOMX_PROBE_HELD_COPY = 4 };
int iomx_probe_stream(int mode, const void* a, const void* b, void* out, uint64_t bytes,
                      iomx_stream_t stream);

/* Compares the hardware BF16 conversion with the software round-to-nearest-
 * even rule over all 2^32 binary32 encodings; *mismatches receives the count. */
int iomx_selftest_bf16_convert(uint64_t* mismatches, iomx_stream_t stream);

/* Compares the packed F16 arithmetic of the streaming kernels (hardware F16 <->
 * binary32 conversions around one binary32 operation) with the integer-rounded
 * binary64 rule for all 2^32 operand pairs and ADD, MUL, SUB, DIV; *mismatches receives
 * the count. */
int iomx_selftest_f16_binary(uint64_t* mismatches, iomx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* IOMX_PROBE_H */
