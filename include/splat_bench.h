/*
 * splat_bench.h -- C ABI of libsplat_bench.so: measurement aids for bench.py.
 *
 * Nothing here has a counterpart in the reference (spikerheado1234/triton-fun) and nothing on the operator path
 * calls it: the operator ABI a maintainer binds is include/splat_hip.h.  These are the ceilings bench.py quotes the
 * kernels against, built from the same sources and with the same flags as the operators.
 *
 * Conventions as in splat_hip.h: device pointers, `stream` a hipStream_t passed as void*, calls only enqueue work and
 * never allocate; 0 on success, negative SPLAT_E_* codes (same values as in splat_hip.h) for rejected arguments,
 * positive = hipError_t; splat_bench_last_error() gives the text of the last non-zero return on this thread.
 */
#ifndef SPLAT_BENCH_H
#define SPLAT_BENCH_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPLAT_BENCH_VERSION 200

int splat_bench_version(void);
const char* splat_bench_last_error(void);

/* Copy `bytes` (a multiple of 16; both pointers 16-byte aligned) from src to dst with the access forms of the HBM-bound
 * kernels (16 bytes per lane, non-temporal, several requests in flight).  Its rate is the read + write streaming
 * ceiling that bench.py quotes splat_softmax against. */
int splat_bench_stream_copy(const void* src, void* dst, int64_t bytes, void* stream);

/* The matrix work of the fused forward's tile loop with nothing else around it: `workgroups` workgroups run `tiles`
 * times the LDS fragment reads and MFMAs of one 64-key tile at d = 128 in bf16 (both products), with no global loads,
 * copies, exponentials or barriers in the loop.  `shape` selects how the work is cut:
 *   0: 32x32x16 MFMA, 32 query rows per wavefront, 4 wavefronts per workgroup, 2 wavefronts per SIMD (the fused
 *      forward's own shape; one fresh 1 KiB LDS fragment per MFMA);
 *   1: 32x32x16 MFMA, 64 query rows per wavefront, 4 wavefronts per workgroup, 1 wavefront per SIMD (every LDS
 *      fragment feeds two MFMAs);
 *   2: 16x16x32 MFMA, 16 query rows per wavefront, 8 wavefronts per workgroup, 4 wavefronts per SIMD (twice the LDS
 *      bytes per operation).
 * The 64 KiB at `data` (16-byte aligned; give it random bf16 values: the switching activity of the operands decides
 * the clock a power-limited part reaches) fill the LDS; `out` receives one float per thread (256 threads per workgroup
 * for shapes 0 and 1, 512 for shape 2).  splat_bench_mfma_lds_probe_flops gives the floating-point operations of one
 * such call (0 for an unknown shape). */
int splat_bench_mfma_lds_probe(const void* data, int64_t data_bytes, void* out, int64_t out_bytes, int32_t shape,
                               int32_t workgroups, int32_t tiles, void* stream);
int64_t splat_bench_mfma_lds_probe_flops(int32_t shape, int32_t workgroups, int32_t tiles);

/* The fused forward's tile loop at d = 64 in bf16 with its exponentials and nothing else around it: per 64-key tile both
 * products out of LDS tiles and, per score, one multiply-add, one exponential, one add into the row sum and one
 * conversion (the loop's work once every row has its reference), one workgroup barrier per tile; no global loads, no
 * masks.  `shape` 0: 32 query rows per wavefront (32x32x16 MFMA, 256 threads per workgroup); 1: 16 rows per wavefront
 * (16x16x32 MFMA, 512 threads).  Both are launched with 53 KiB of LDS, so that three workgroups share a compute unit:
 * 3 and 6 wavefronts per SIMD.  `exponentials` 0 replaces the exponential and the sum by a multiplication.  data, out
 * and the limits as for splat_bench_mfma_lds_probe; splat_bench_softmax_loop_probe_flops gives the matrix operations of
 * one call (128 rows x 64 keys x 64 x 4 per workgroup and tile). */
int splat_bench_softmax_loop_probe(const void* data, int64_t data_bytes, void* out, int64_t out_bytes, int32_t shape,
                                   int32_t exponentials, int32_t workgroups, int32_t tiles, void* stream);
int64_t splat_bench_softmax_loop_probe_flops(int32_t workgroups, int32_t tiles);

#ifdef __cplusplus
}
#endif
#endif /* SPLAT_BENCH_H */
