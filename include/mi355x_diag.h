/*
 * mi355x_diag -- measurement aids of the benchmark (libmi355x_diag.so).  Not part of the drop-in boundary: nothing
 * here has a counterpart in the reference, and no provider kernel links it.  Two plain HBM movers with a known byte
 * count and a matrix-pipe exerciser: the read stream gives the bandwidth a kernel that only reads (the decode GEMV)
 * can reach on this device, the copy calibrates the profiler's FETCH_SIZE / WRITE_SIZE counters, the matrix-pipe
 * loop gives the rate the int8 MFMA sustains for given operand data.  Status codes as in mi355x_int8.h; the HIP device
 * is the caller's current one; `stream` is a hipStream_t passed as void*.
 */
#ifndef MI355X_DIAG_H_
#define MI355X_DIAG_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* bytes must be a multiple of 16, pointers 16-byte aligned. */
int mi_diag_stream_read(const void *src_dev, int64_t bytes, void *stream);
int mi_diag_copy(void *dst_dev, const void *src_dev, int64_t bytes, void *stream);
/* The matrix pipe alone: `workgroups` x 4 waves each issue iters x 16 v_mfma_i32_32x32x32_i8 (65536 ops each) on
 * register operands read once from operands_dev (32 KiB), in the order and with the accumulator start value the
 * 256 x 256 GEMM tile uses (accumulators restart every 128 iterations = K 4096).  The sustained shader clock, and
 * with it the rate, depends on the operand data (bit toggling -> power), so the benchmark passes bytes drawn like
 * the GEMM's.  clocks_dev[0] = shader cycles, clocks_dev[1] = 100 MHz ticks spent in the loop (device memory). */
int mi_diag_mfma_rate(const void *operands_dev, int32_t iters, int32_t workgroups, uint64_t *clocks_dev,
                      void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355X_DIAG_H_ */
