/*
 * vkop_hip.h -- C ABI of the MI355X (gfx950) softmax / top-k post-processing
 * library (libvkop_hip.so, built from vkop_amd/csrc).
 *
 * This is the boundary the reference's two operators sit on once their Vulkan
 * plumbing is taken away: where `Softmax::execute` (ops/Softmax.hpp:61-141) and
 * `Topk::execute` (ops/Topk.hpp:95-218) bind storage buffers, fill push
 * constants and call `Operator::submit` (ops/Operator.hpp:225-238), a HIP build
 * calls one function of this header with device pointers and a stream.
 *
 * Conventions
 *  - plain C: pointers, sizes, ints; no C++ or framework types.
 *  - every function returns an int status (0 = VKOP_HIP_OK) unless it returns a
 *    size; no exception crosses the boundary; vkop_hip_last_error() gives the
 *    calling thread's last failure text.
 *  - `in`, `out*`, `workspace` are DEVICE pointers; `stream` is a hipStream_t
 *    passed as void* (NULL = the default stream).  Calls only enqueue work.
 *  - tensors are dense row-major with `ndim` (1..4) extents in `shape`, the
 *    layout of the reference's storage-buffer tensors (core/Tensor.hpp:722-729,
 *    765-801); `axis` may be negative (ops/Softmax.hpp:111-113).
 *  - dtype VKOP_HIP_F16 means IEEE binary16 bits in uint16_t, the reference's
 *    Tensor<uint16_t> (core/Tensor.hpp:116-198).  Arithmetic is float32 either way.
 *  - a workspace must have been cleared once with vkop_hip_workspace_init()
 *    before its first use (it holds per-row arrival counters that every call
 *    returns to zero); clear it again after a call failed with
 *    VKOP_HIP_ERR_DEVICE.  Two calls that are in flight at the same time must
 *    not share a workspace.
 */
#ifndef VKOP_HIP_H_
#define VKOP_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum vkop_hip_status {
    VKOP_HIP_OK = 0,
    VKOP_HIP_ERR_INVALID = 1,     /* bad argument: null pointer, dtype, rank, axis, k */
    VKOP_HIP_ERR_DEVICE = 2,      /* a HIP runtime call failed */
    VKOP_HIP_ERR_WORKSPACE = 3,   /* workspace missing or smaller than *_workspace_bytes() */
    VKOP_HIP_ERR_UNSUPPORTED = 4  /* valid request this build does not cover (k too large) */
};

enum vkop_hip_dtype { VKOP_HIP_F32 = 0, VKOP_HIP_F16 = 1 };

/* Largest k the top-k entry points accept (the reference asserts k < 256,
 * ops/Topk.hpp:103). */
#define VKOP_HIP_MAX_K 2048

/* ---- device, memory, streams: replaces VulkanDevice / VulkanBuffer /
 * VulkanCommandPool + staging (vulkan/, core/Tensor.hpp:765-832) for this path. */
int vkop_hip_init(int device);
int vkop_hip_shutdown(void);
const char *vkop_hip_last_error(void);
/* name: caller buffer of name_len bytes; any out pointer may be NULL. */
int vkop_hip_device_info(char *name, size_t name_len, int *compute_units,
                         size_t *memory_bytes);

int vkop_hip_malloc(void **ptr, size_t bytes);
int vkop_hip_free(void *ptr);
/* Host pointers may be pageable; the copy is ordered on `stream` and has
 * completed on return (Tensor::copyToGPU / copyToCPU block the same way). */
int vkop_hip_memcpy_h2d(void *dst_device, const void *src_host, size_t bytes, void *stream);
int vkop_hip_memcpy_d2h(void *dst_host, const void *src_device, size_t bytes, void *stream);
int vkop_hip_memcpy_d2d(void *dst_device, const void *src_device, size_t bytes, void *stream);

int vkop_hip_stream_create(void **stream);
int vkop_hip_stream_destroy(void *stream);
int vkop_hip_stream_sync(void *stream);

/* Timeline points (VulkanCommandBuffer's timeline semaphore wait/signal,
 * core/runtime.cpp:421-446) and timing. */
int vkop_hip_event_create(void **event);
int vkop_hip_event_destroy(void *event);
int vkop_hip_event_record(void *event, void *stream);
int vkop_hip_event_sync(void *event);
int vkop_hip_stream_wait_event(void *stream, void *event);
int vkop_hip_event_elapsed_ms(void *start, void *stop, float *ms);

/* Recorded work: everything enqueued on `stream` between begin and end is
 * recorded instead of run, the way Operator::onExecute only records into a
 * VulkanCommandBuffer between begin() and end() (ops/Operator.hpp:124-134) and
 * Runtime::Run submits the recorded buffers (core/runtime.cpp:435-440).
 * vkop_hip_graph_launch submits the recording; it may be launched any number
 * of times.  Implemented with HIP stream capture. */
int vkop_hip_graph_begin(void *stream);
int vkop_hip_graph_end(void *stream, void **graph);
int vkop_hip_graph_launch(void *graph, void *stream);
int vkop_hip_graph_destroy(void *graph);

/* Clears a workspace with a fill kernel (safe to capture in a HIP graph). */
int vkop_hip_workspace_init(void *workspace, size_t bytes, void *stream);

/* ---- Softmax: ops/Softmax.hpp:61-141 over shaders/softmax2.comp:50-184 and
 * shaders/softmax.comp:31-207.  out has the shape and dtype of in; in == out is
 * allowed.  nan_where != 0 replaces NaN results by nan_value (the shader's
 * `nan_optimization`, shaders/softmax2.comp:177-181), on every axis. */
size_t vkop_hip_softmax_workspace_bytes(int dtype, const int *shape, int ndim, int axis);
int vkop_hip_softmax(const void *in, void *out, int dtype, const int *shape,
                     int ndim, int axis, int nan_where, float nan_value,
                     void *workspace, size_t workspace_bytes, void *stream);

/* ---- TopK: ops/Topk.hpp:95-218 over shaders/topk.comp:110-262.
 * out_values: dtype of in, out_indices: int32 positions along `axis`; both have
 * the shape of in with [axis] = k.  With sorted != 0: descending for
 * largest != 0, ascending otherwise; ties: lower index first; NaN ranks above
 * +inf.  With sorted == 0 (the reference parses the attribute and ignores it,
 * ops/Topk.hpp:73-75; ONNX leaves the order open then) the same k elements
 * come in an order the library chooses, the same from run to run: on the
 * multi-pass radix select (smallest first on long rows, and rows no other
 * route takes) as that select lists them, which saves its last step; on
 * every other route in sorted order, which costs nothing there.
 * 1 <= k <= min(extent of axis, VKOP_HIP_MAX_K). */
size_t vkop_hip_topk_workspace_bytes(int dtype, const int *shape, int ndim, int axis, int k);
int vkop_hip_topk(const void *in, void *out_values, int32_t *out_indices,
                  int dtype, const int *shape, int ndim, int axis, int k,
                  int largest, int sorted, void *workspace,
                  size_t workspace_bytes, void *stream);

/* ---- Fused post-proc: TOPK applied to the SOFTMAX output, the pair
 * benchmark/main.cpp:85-101 registers through Runtime::RegisterPostProcess
 * (core/runtime.cpp:480-520).  Result = top-k (value order, then lower index)
 * of the softmax tensor, without writing that tensor.  out_probs may be NULL;
 * when given it receives the full softmax tensor as well. */
size_t vkop_hip_softmax_topk_workspace_bytes(int dtype, const int *shape, int ndim, int axis, int k);
int vkop_hip_softmax_topk(const void *in, void *out_probs, void *out_values,
                          int32_t *out_indices, int dtype, const int *shape,
                          int ndim, int axis, int k, int largest,
                          void *workspace, size_t workspace_bytes, void *stream);

/* ---- Sampling-style variant of the fused post-proc (no counterpart in the
 * reference; its TopK parses k, axis, largest and sorted, ops/Topk.hpp:62-79, and
 * the benchmark scales nothing, benchmark/main.cpp:85-101).  Every logit is first
 * multiplied by `scale` (1 / temperature; positive and finite) in single
 * precision, x' = fl32(x * scale); out_values / out_indices are the fused
 * softmax -> top-k, largest first, of x', to the bars of vkop_hip_softmax_topk
 * on a tensor holding x' (bit for bit its result on long last-axis rows, where
 * both run the same streaming kernels; to the same bar against an exact softmax elsewhere).  out_counts (int32 per
 * row, may be NULL; last axis only) receives the nucleus cut of each row's
 * result for top_p, the number vkop_hip_topp_count gives on out_values.
 * Workspace: vkop_hip_softmax_topk_workspace_bytes().
 * Cost by shape (MI355X, one call at a time): on the long last-axis rows the
 * scan + pick kernels take -- the shapes this entry point is for, e.g.
 * [64,128256] k = 50 -- it costs the plain fused call plus about a tenth
 * (17.2 against 15.5 us).  Last-axis rows that one workgroup holds (up to
 * 32768 elements, k up to 408) run that workgroup's kernel with the scale and
 * the count inside, short rows with k up to 32 the one-wave kernel:
 * [64,8192] k = 40 takes 9.6 us (9.4 for the plain fused call), [256,1000]
 * k = 5 takes 5.5 us (4.7).  What is left -- other axes, k beyond 511 on
 * long rows -- is correct but runs the one-workgroup-per-line kernels, two
 * passes and an exact select per line and then the count (tens of
 * microseconds). */
int vkop_hip_softmax_topk_sampling(const void *in, void *out_values, int32_t *out_indices,
                                   int32_t *out_counts, int dtype, const int *shape, int ndim,
                                   int axis, int k, float scale, float top_p, void *workspace,
                                   size_t workspace_bytes, void *stream);

/* ---- The fused post-proc for callers that cannot allocate device memory (work
 * recorded into a HIP graph, tight serving loops, harnesses that forbid
 * hipMalloc): vkop_hip_softmax_topk without out_probs and without a workspace
 * argument.  No counterpart in the reference.  Its scratch is an array of
 * VKOP_HIP_STATIC_SCRATCH_BYTES that the library holds on every GPU it runs on
 * until the process ends; the call allocates and frees nothing.  A tensor whose
 * vkop_hip_softmax_topk_workspace_bytes() exceeds that size is refused with
 * VKOP_HIP_ERR_WORKSPACE.  Results are bit for bit those of
 * vkop_hip_softmax_topk.  All calls on one GPU share that GPU's array: calls
 * that overlap in time on one GPU (different streams or threads) race; calls
 * on one stream, or ordered by events, are fine.  The stream must belong to the
 * current device; call vkop_hip_init(device) first (it looks up the array's
 * address; otherwise the first call on a device does). */
#define VKOP_HIP_STATIC_SCRATCH_BYTES (4u << 20)
int vkop_hip_softmax_topk_static(const void *in, void *out_values, int32_t *out_indices,
                                 int dtype, const int *shape, int ndim, int axis, int k,
                                 int largest, void *stream);

/* ---- Max along an axis, (.., n, ..) -> (.., ..): the per-anchor class max
 * between softmax and top-k in the detection-style post-proc
 * (example/yolo/main.cpp:60-127; ops/Reduce.hpp covers only 4-D images). */
int vkop_hip_reduce_max(const void *in, void *out, int dtype, const int *shape,
                        int ndim, int axis, void *stream);

/* ---- Softmax along `axis` followed by the max over the same axis, without the
 * softmax tensor: the first two steps of the detection-style post-proc
 * (per-anchor class max of the class probabilities, example/yolo/main.cpp:60-127)
 * in one read of the input.  out has the shape of in without `axis` and is bit
 * for bit what vkop_hip_softmax + vkop_hip_reduce_max give. */
size_t vkop_hip_softmax_reduce_max_workspace_bytes(int dtype, const int *shape, int ndim, int axis);
int vkop_hip_softmax_reduce_max(const void *in, void *out, int dtype, const int *shape,
                                int ndim, int axis, void *workspace, size_t workspace_bytes, void *stream);

/* ---- Nucleus (top-p) cut on the output of a sorted top-k: counts[row] = the
 * smallest m >= 1 such that values[row][0..m) sum to at least p, or k when they
 * never do (also when a NaN enters the sum).  The sum is taken in float, front
 * to back, so the count is reproducible bit for bit.  values: rows x k
 * probabilities in descending order, rows row_stride elements apart (the
 * benchmark's arrangement writes top-k into full-width rows,
 * benchmark/main.cpp:92-94).  No counterpart in the reference: a sampling-style
 * extension on the softmax -> top-k path. */
int vkop_hip_topp_count(const void *values, int32_t *counts, int dtype, int rows,
                        int k, int row_stride, float p, void *stream);

/* ---- Non-maximum suppression: replaces Nms::execute (ops/Nms.hpp:73-118) and
 * shaders/nms.comp, the operator that follows the top-k in the detection-style
 * post-processing.  boxes [B][N][4] and scores [B][C][N] of `dtype`; per (batch,
 * class) the boxes whose score is greater than score_threshold are walked from
 * the best score down (equal scores: lower box index first), a box still active
 * is selected and deactivates every later box whose IoU with it is greater than
 * iou_threshold; max_output_boxes_per_class > 0 limits the selections per pair;
 * center_point_box != 0: boxes are (x_center, y_center, width, height).
 * out receives (batch, class, box index) records, [out_capacity][3] int32, in
 * order of batch, then class, then selection (the reference appends them through
 * an atomic counter in scheduling order, with a (-1,-1,-1) record somewhere among
 * them; here that record follows the last one, when out_capacity has room for it).
 * out_count: two int32 on the device: the number of records (all
 * of them, also when out_capacity holds fewer) and 1 if some pair had more than
 * VKOP_HIP_NMS_MAX_CANDIDATES boxes above the score threshold (the later ones by
 * box index were left out; the reference's shader keeps 1024). */
#define VKOP_HIP_NMS_MAX_CANDIDATES 2048
size_t vkop_hip_nms_workspace_bytes(int B, int C, int N, int max_output_boxes_per_class);
int vkop_hip_nms(const void *boxes, const void *scores, int32_t *out, int out_capacity,
                 int32_t *out_count, int dtype, int B, int C, int N, int center_point_box,
                 int max_output_boxes_per_class, float iou_threshold, float score_threshold,
                 void *workspace, size_t workspace_bytes, void *stream);

/* ---- Tuning knobs (no counterpart in the reference, whose shaders fix their
 * workgroup shapes at compile time).  Only the kernels and launch shapes chosen
 * differ.  What is identical for every setting: the softmax operator's output,
 * plain top-k values and indices, and the indices of the fused call wherever the
 * k+1 largest probabilities of a row differ by more than the kernels' sums do.
 * What is equal to within the bar (2 ulp of float against the CPU definition, one
 * unit of a half): the fused call's probabilities -- each route adds a row's
 * terms up in its own order, and two routes may round a row's sum one ulp apart.
 * The settings are
 * process-wide and read when a call is made: set them before the threads that
 * call the operators start, not while calls are being made (a call that sees a
 * setting change between its workspace query and its launch is refused with
 * VKOP_HIP_ERR_WORKSPACE at worst, never runs out of bounds: *_workspace_bytes()
 * covers every setting).
 *   "rows.path": 0 (default) = short last-axis rows with k up to 32 go through
 *       the one-wave-per-row kernel, rows too long for one workgroup through the
 *       scan + pick kernel pair where it applies (k up to 511; beyond that, scan +
 *       gather + rank); 1 = never (the chunk + merge kernels, the multi-pass radix
 *       select: with the default, rows of several chunks never take chunk + merge,
 *       which the tests compare every other route with).
 *   "rows.threads", "rows.loads", "rows.chunks": force the launch shape of the
 *       chunk kernel (threads per workgroup, 128-bit loads per thread,
 *       workgroups per row); all three must be set, 0 = automatic (default).
 *   "rows.fused": 0 (default) = rows split over several chunk workgroups are
 *       merged by a second kernel; 1 = one kernel, whose workgroups merge each
 *       row as its last chunk completes (measured slower on MI355X).
 *   "nms.threads": threads per workgroup of the Nms kernel: 0 (default) = 256
 *       from 1024 (batch, class) pairs on, else 1024; 256 or 1024 force one.
 * Unknown names return VKOP_HIP_ERR_INVALID. */
int vkop_hip_tune(const char *name, int value);

/* Launch shape the fused / top-k entry points would use for this tensor:
 * threads per workgroup, 128-bit loads per thread and workgroups per row of the
 * streaming kernel (a second kernel per row follows when chunks > 1); all three
 * are 0 when the general one-workgroup-per-line kernels would run.  Any out
 * pointer may be NULL. */
int vkop_hip_rows_plan(int dtype, const int *shape, int ndim, int axis, int k,
                       int *threads, int *loads, int *chunks);

#ifdef __cplusplus
}
#endif
#endif /* VKOP_HIP_H_ */
