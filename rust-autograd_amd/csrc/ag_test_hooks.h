/* Test hooks: exported only by libag_hip_test.so, the flavour of the kernel library that build.sh compiles with
 * -DAG_TEST_HOOKS for the test-suite and tuning runs.  The shipped libag_hip.so is built without them and exports
 * exactly the operator boundary (include/ag_hip.h).  Every hook sets an override that is local to the calling
 * thread, so other threads' calls are never affected. */
#ifndef AG_TEST_HOOKS_H
#define AG_TEST_HOOKS_H

#ifdef __cplusplus
extern "C" {
#endif
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

/* Force GEMM tile configuration `cfg` for later calls of this thread (-1 = automatic choice). */
void ag_test_gemm_force_config(int cfg);
/* Force the split count of accumulated-batch GEMMs (0 = automatic). */
void ag_test_gemm_force_splits(int splits);
/* Blocks per CU of the persistent GEMM grid (0 = as many as stay resident). */
void ag_test_gemm_force_grid(int blocks_per_cu);
/* Output rows per chunk of the stride-2 pooling kernels (0 = automatic); a negative value instead keeps 2 x 2
   windows off the one-thread-per-window kernels, so that the staged and register kernels see those geometries too. */
void ag_test_pool_chunk_rows(int rows);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* AG_TEST_HOOKS_H */
