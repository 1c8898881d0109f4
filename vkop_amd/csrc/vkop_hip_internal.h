/*
 * Measurement hooks that are NOT part of the public interface (include/vkop_hip.h):
 * for this repository's benchmarks and tests only.  vkop_hip_measure_path is a pure
 * query and part of libvkop_hip.so; vkop_hip_measure_stages changes what a call
 * launches and exists only in the benchmark build of the library
 * (libvkop_hip_bench.so: the same objects, the C ABI source compiled with
 * -DVKOP_BENCH_HOOKS).
 */
#ifndef VKOP_HIP_INTERNAL_H_
#define VKOP_HIP_INTERNAL_H_

#ifdef __cplusplus
extern "C" {
#endif

/* Which kernels of a two-kernel streaming call are launched from now on, in every
 * thread of the process: 3 = both (the state the library starts in), 1 = only the
 * first, 2 = only the second (it reads the workspace an earlier whole call left).
 * With 1 or 2 the top-k and fused entry points do NOT produce valid results: the
 * settings exist so that a benchmark can time each kernel by itself with the
 * launches a real call makes.  Not thread-safe; set it back to 3.
 * libvkop_hip_bench.so only. */
#ifdef VKOP_BENCH_HOOKS
int vkop_hip_measure_stages(int stages);
#endif

/* Which streaming kernels a fused / top-k (largest) call on this tensor would run
 * with the current tuning settings: 4 = rows_tiny_kernel (one wave per row), 2 =
 * rows_scan_kernel + rows_pick_kernel, 3 = rows_scan_kernel + bigpick_gather_kernel +
 * bigpick_rank_kernel, 1 = rows_chunk_kernel (+ rows_merge_kernel when a row is
 * split), 0 = other kernels, -1 = bad arguments. */
int vkop_hip_measure_path(int dtype, const int *shape, int ndim, int axis, int k);

#ifdef __cplusplus
}
#endif
#endif /* VKOP_HIP_INTERNAL_H_ */
