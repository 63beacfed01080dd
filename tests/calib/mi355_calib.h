/* Measurement kernels behind bench.py's --calib-* switches (tests/bin/libmi355_calib.so).
 * Not part of the library's boundary: nothing here computes a matmul.  Every
 * function is asynchronous on `stream` (a hipStream_t, NULL = the default
 * stream) and returns 0, 1 (bad arguments) or 2 (launch failed). */
#ifndef MI355_CALIB_H
#define MI355_CALIB_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* Plain device-to-device copy (one 16-byte load + store per lane): the
 * known-size dispatch that FETCH_SIZE / WRITE_SIZE counter passes are scaled by. */
int mi355_calib_copy(void *dst, const void *src, size_t bytes, void *stream);

/* Read-modify-write sweep over `buf`: evicts the caches between timed launches. */
int mi355_calib_flush(void *buf, size_t bytes, void *stream);

/* A kernel that does nothing, `blocks` workgroups of `threads` lanes: the cost of a dispatch. */
int mi355_calib_empty(int blocks, int threads, void *stream);

/* Read-only kernel with the access shape of the weight-only decode kernel
 * (128 KiB per workgroup, 16 wavefronts of eight 1 KiB non-temporal runs):
 * what streaming `bytes` (a multiple of 128 KiB) of weights costs by itself.
 * `sink` holds 4 bytes per 128 KiB and is not written in practice. */
int mi355_calib_read_stream(const void *src, size_t bytes, void *sink, void *stream);

/* The same stream plus the decode kernel's ending: the wavefronts' values meet
 * in LDS and 64 floats are stored per workgroup (`out`: 256 bytes per 128 KiB). */
int mi355_calib_read_reduce(const void *src, size_t bytes, void *out, void *stream);

/* Access-shape probe for kernels that stream rows (the grouped matmul tiles):
 * `slabs` workgroups of four wavefronts each read a slab of 256 rows x K bytes
 * (K a multiple of 1024) once, K-major, a load instruction fetching 1024 / run
 * rows x `run` contiguous bytes (run = 64, 128, 256 or 1024).  `sink`: 1 KiB. */
int mi355_calib_read_pattern(const void *src, int64_t slabs, int64_t K, int run, void *sink, void *stream);

/* What an MFMA instruction of the GEMM kernels sustains by itself: 1024
 * workgroups x 4 wavefronts, operands and accumulators in registers, 8 or 16
 * independent accumulator chains, `iters` rounds.  instr: 0 i32_32x32x32_i8,
 * 1 i32_16x16x64_i8, 2 f32_32x32x64 fp8, 3 f32_16x16x128 fp8, 4 f32_32x32x64
 * fp4, 5 f32_16x16x128 fp4, 6 f32_32x32x16_bf16, 7 f32_16x16x32_bf16,
 * 8 f32_32x32x2_f32.  `bits`: 16 KiB of operand bits (their toggling decides
 * the clock the power manager grants), `out`: 1 MiB.  *ops_per_launch receives
 * the operation count to divide by the measured time. */
int mi355_calib_mfma_rate(int instr, int iters, void *out, const void *bits, double *ops_per_launch, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355_CALIB_H */
