/* Measurement aids of the benchmark (libksmm_bench.so).  Not part of the drop-in ABI of
 * libksmm_hip.so; status codes are those of ksmm_hip.h.  No counterpart in the reference. */
#ifndef KSMM_PROBE_H
#define KSMM_PROBE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* Measurement aid, no counterpart in the reference: launches a kernel of 256 workgroups x 8 waves
 * that only issues matrix-core instructions on register operands (KSMM_F16: 32x32x16 fp16,
 * KSMM_F32: 16x16x4 fp32; `random` != 0: operands uniform in [-1, 1], else all ones) and
 * returns the flops it performs in *flops; timed by the caller, it gives the rate the matrix
 * cores sustain, which a benchmark prints beside the published peak.  `out` receives
 * ksbench_mfma_probe_bytes() bytes of checksums (so that the work cannot be optimised away). */
int64_t ksbench_mfma_probe_bytes(void);
int ksbench_mfma_probe(int dtype, int iters, int random, void *out, int64_t out_bytes, double *flops, void *stream);

/* Measurement aid, no counterpart in the reference: a copy with the access pattern of a
 * batch-size-last factor with square blocks.  x and y are (a * rows * d) rows of `row_bytes` bytes;
 * one workgroup moves the `rows` x `tile_bytes` tile of block (a_i, d_i) and one batch tile from x
 * to the same place in y (the rows of a block are d rows apart), all loads before the first
 * store.  Timed by the caller, it gives the rate of a copy that moves whole tiles with those
 * addresses, which a benchmark prints beside the rate of a streaming copy (with d = 1 and
 * row_bytes = tile_bytes the same tiles lie in linear memory).  tile_bytes: a power of two,
 * 16..4096; rows <= 48 * (4096 / tile_bytes). */
int ksbench_tilecopy_probe(const void *x, void *y, int64_t row_bytes, int a, int rows, int d, int tile_bytes, void *stream);

/* A streaming copy of `bytes` bytes (a multiple of 16, both pointers 16-byte aligned) by a
 * persistent grid of `workgroups` x 256 threads, four 16-byte vectors per thread and round,
 * non-temporal loads and stores.  Timed by the caller, it is the rate a benchmark prints as what
 * this memory system gives a kernel that only moves bytes. */
int ksbench_stream_copy(const void *x, void *y, int64_t bytes, int workgroups, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* KSMM_PROBE_H */
