/*
 * Test and tuning hook of libmi355gq.so; NOT part of the public C ABI (include/mi355gq.h does not declare it).
 *
 * Forces which kernel family / launch shape the dispatcher picks, so that tests can run every kernel on every
 * shape and sweeps can A/B launch shapes.  The state it sets is thread-local: it steers only calls made later on
 * the calling thread, and a thread that never calls it always gets the heuristics.  value < 0 restores the
 * heuristic.  Names and ranges:
 *   "gemv_rows_per_wave"  1, 2, 4, 8     rows per row set of the register GEMV
 *   "gemv_variant"        0..15          kernel family for up to 16 rows (2..5 a skinny form, 6..8 the quad-row kernel, 9 its
 *                                        form with x in registers)
 *   "gemv_waves"          4..16384       persistent waves of the register GEMV / quad-row kernel
 *   "gemv_ksplit"         0, 1           K of a row shared between two waves of the register GEMV (off / on)
 *   "quad_ksplit"         0, 1, 2, 3     log2 of the waves of a quad-row kernel that share a quad's K range (3: the form
 *                                        with x in registers only)
 *   "quad_pairs"          1, 2           weight quads per item of the quad-row kernel
 *   "gemm_variant"        0..15          GEMM tile (1: GEMM only, 2: GEMV up to 8 rows, others pick a tile)
 *   "gemm_split_k"        1..4096        split of K in the few-row GEMM
 *   "gemm_fast_loop"      0              0 forces the GEMM's general K loop (zero-selects kept)
 * Returns 0, or MI355GQ_ERR_ARG for an unknown name or a value out of range.
 * Because the state is thread-local, mi355gq_linear_workspace_bytes (which reads "gemm_split_k") and the matmul call
 * it sizes a workspace for must run on the same thread while an option is set.
 */
#ifndef MI355GQ_TESTING_H_
#define MI355GQ_TESTING_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

__attribute__((visibility("default"))) int mi355gq_testing_set_option(const char* name, int value);

/* Name and template arguments of the kernel the calling thread's last matmul call launched ("" before any),
 * e.g. "gq::gemv_reg_kernel<4,1,2,2,0,false>": lets a benchmark label its timings from the run. */
__attribute__((visibility("default"))) const char* mi355gq_testing_last_kernel(void);

/* Measurement aid, no counterpart in the reference: one launch that only reads the byte ranges a and b (sizes
 * multiples of 16, pointers 16-byte aligned) with 128-bit loads and discards them; sink is 4 bytes of device memory
 * or NULL; stream is a hipStream_t.  The benchmark times it on a GEMV's weight and scale tensors to quote what the
 * device delivers for those bytes without any arithmetic. */
__attribute__((visibility("default"))) int mi355gq_testing_stream_read(const void* a, int64_t a_bytes, const void* b,
                                                                       int64_t b_bytes, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355GQ_TESTING_H_ */
