/*
 * Test and tuning hook of libmi355gq.so; NOT part of the public C ABI (include/mi355gq.h does not declare it).
 *
 * Forces which kernel family / launch shape the dispatcher picks, so that tests can run every kernel on every
 * shape and sweeps can A/B launch shapes.  The state it sets is thread-local: it steers only calls made later on
 * the calling thread, and a thread that never calls it always gets the heuristics.  value < 0 restores the
 * heuristic.  Names: "gemv_rows_per_wave" (1, 2, 4, 8), "gemv_variant", "gemm_variant" (0..15),
 * "gemv_waves" (4..16384), "gemm_split_k" (1..4096).  Returns 0, or MI355GQ_ERR_ARG for an unknown name or a value
 * out of range.
 */
#ifndef MI355GQ_TESTING_H_
#define MI355GQ_TESTING_H_

#ifdef __cplusplus
extern "C" {
#endif

__attribute__((visibility("default"))) int mi355gq_testing_set_option(const char* name, int value);

/* Name and template arguments of the kernel the calling thread's last matmul call launched ("" before any),
 * e.g. "gq::gemv_reg_kernel<4,1,2,2,0,false>": lets a benchmark label its timings from the run. */
__attribute__((visibility("default"))) const char* mi355gq_testing_last_kernel(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355GQ_TESTING_H_ */
