/*
 * CPU oracle for the softmax -> top-k logits post-processing path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the library ships may include, link or
 * call this file: it exists so that tests, the smoke check and the benchmark's
 * CPU-baseline leg have something independent of the HIP kernels to compare
 * with.  Plain C99, no GPU, no third-party dependency.
 *
 * Every tensor is addressed as (outer, n, inner): `n` is the extent of the
 * axis the operator works along, `inner` the product of the extents after it
 * (1 when the axis is the last one), `outer` the product of those before it.
 * Element (o, j, i) lives at  o*n*inner + j*inner + i.
 *
 * Half precision tensors are carried as uint16_t holding IEEE binary16 bits,
 * the way the reference carries them (core/Tensor.hpp:116-198, Tensor<uint16_t>).
 */
#ifndef VKOP_ORACLE_H_
#define VKOP_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* binary16 <-> binary32, round-to-nearest-even, NaN/inf/subnormals kept
 * (what _cvtss_sh(f,0) / _cvtsh_ss do, core/Tensor.hpp:133,174). */
float vkop_oracle_half_to_float(uint16_t h);
uint16_t vkop_oracle_float_to_half(float f);

/* Softmax along the middle axis of (outer, n, inner).
 * Follows ops/Softmax.hpp:61-141 for shape/axis meaning and
 * shaders/softmax2.comp:50-117 / shaders/softmax.comp:31-207 for the math
 * (max, sum of exp(x-max), exp(x-max)/sum), with three stated deviations:
 * the running max starts at -inf (not -1e9), the sum is accumulated in
 * double over correctly rounded single-precision exp terms, and the NaN
 * replacement option applies to every axis (the shader has it on axis 0 only,
 * shaders/softmax2.comp:177-181).
 * nan_where != 0: outputs that are NaN are replaced by nan_value. */
void vkop_oracle_softmax_f32(const float *in, float *out, int outer, int n,
                             int inner, int nan_where, float nan_value);
void vkop_oracle_softmax_f16(const uint16_t *in, uint16_t *out, int outer,
                             int n, int inner, int nan_where, float nan_value);

/* Top-k along the middle axis.  Output tensors are (outer, k, inner).
 * Follows ops/Topk.hpp:95-125 (values keep the input type, indices are int32
 * positions along the axis) and torch::topk(input,k,axis,largest,sorted=true)
 * as called by tests/TopkTest.cpp:73 for the ordering of distinct values.
 * Ties: the element with the lower index comes first.  NaN ranks above +inf
 * for largest != 0 and last for largest == 0; -0 and +0 are equal.
 * Requires 0 <= k <= n. */
void vkop_oracle_topk_f32(const float *in, float *values, int32_t *indices,
                          int outer, int n, int inner, int k, int largest);
void vkop_oracle_topk_f16(const uint16_t *in, uint16_t *values,
                          int32_t *indices, int outer, int n, int inner, int k,
                          int largest);

/* Fused post-proc = top-k of the softmax output, the sequence
 * benchmark/main.cpp:85-101 registers (SOFTMAX then TOPK on its result).
 * probs may be NULL; when given it receives the full softmax tensor. */
void vkop_oracle_softmax_topk_f32(const float *in, float *probs, float *values,
                                  int32_t *indices, int outer, int n,
                                  int inner, int k, int largest);
void vkop_oracle_softmax_topk_f16(const uint16_t *in, uint16_t *probs,
                                  uint16_t *values, int32_t *indices,
                                  int outer, int n, int inner, int k,
                                  int largest);

/* Sampling-style variant (no counterpart in the reference; the attribute
 * parsing such options would hang on is ops/Topk.hpp:62-79): every logit is
 * first multiplied by `scale` (1 / temperature) in single precision, then the
 * fused softmax -> top-k, largest first, of the scaled logits; counts (may be
 * NULL) receives per line the nucleus cut of vkop_oracle_topp_count_f32 for
 * top_p on the line's k sorted probabilities (halves widened for f16). */
void vkop_oracle_softmax_topk_sampling_f32(const float *in, float scale,
                                           float top_p, float *values,
                                           int32_t *indices, int32_t *counts,
                                           int outer, int n, int inner, int k);
void vkop_oracle_softmax_topk_sampling_f16(const uint16_t *in, float scale,
                                           float top_p, uint16_t *values,
                                           int32_t *indices, int32_t *counts,
                                           int outer, int n, int inner, int k);

/* Same as vkop_oracle_softmax_topk_f32 with the (outer*inner) lines spread
 * over OpenMP threads; used only to time a multi-core CPU baseline.
 * Returns the number of threads used. */
int vkop_oracle_softmax_topk_f32_mt(const float *in, float *values,
                                    int32_t *indices, int outer, int n,
                                    int inner, int k, int largest,
                                    int threads);

/* Maximum along the middle axis, (outer, n, inner) -> (outer, inner):
 * the "per-anchor class max" step of the detection-style post-proc
 * (example/yolo/main.cpp:60-127 does it on the CPU).  NaN propagates. */
void vkop_oracle_reduce_max_f32(const float *in, float *out, int outer, int n,
                                int inner);

/* Restatement of Function::get_top_k_predictions (core/function.cpp:150-183):
 * single row, float exp, sequential float sum, divide, sort by probability
 * descending, truncate to k.  std::sort leaves the order of equal
 * probabilities unspecified; here the lower index comes first.
 * Returns the number of pairs written (min(k, n)). */
int vkop_oracle_get_top_k_predictions(const float *logits, int n, int k,
                                      int32_t *indices, float *probs);

/* Non-maximum suppression, the Nms operator (ops/Nms.hpp:73-118,
 * shaders/nms.comp:74-201).  boxes is [B][N][4], scores is [B][C][N].
 * Per (batch, class), as the shader's workgroup does: the boxes whose score is
 * greater than score_threshold (shaders/nms.comp:89; at most max_candidates of
 * them, the first by box index -- the shader's shared arrays hold 1024) are
 * ordered by score, largest first (a selection sort that keeps the earlier of
 * two equal scores first, shaders/nms.comp:107-127), then walked in that
 * order: a box still active is selected and deactivates every later box whose
 * IoU with it is greater than iou_threshold (shaders/nms.comp:155-188, IoU as
 * in shaders/nms.comp:61-72: 0 for an empty intersection or a union that is
 * not positive); at most max_output_boxes_per_class selections when that is
 * positive.  center_point_box != 0: boxes are (x_center, y_center, width,
 * height) (shaders/nms.comp:51-59).
 * Stated deviation: the records (batch, class, box index) are written in order
 * of batch, then class, then selection -- the shader appends them through a
 * global atomic counter, so its order across (batch, class) pairs is whatever
 * the scheduling gives, and it adds a (-1,-1,-1) record this function does not.
 * Returns the number of records; at most out_capacity are written to out. */
int vkop_oracle_nms_f32(const float *boxes, const float *scores, int32_t *out,
                        int out_capacity, int B, int C, int N,
                        int center_point_box, int max_output_boxes_per_class,
                        float iou_threshold, float score_threshold,
                        int max_candidates);

/* Nucleus (top-p) cut: counts[r] = smallest m >= 1 with values[r][0..m) summing
 * (float, front to back) to at least p; k when they never do.  Not in the
 * reference: a sampling-style extension on its softmax -> top-k path. */
void vkop_oracle_topp_count_f32(const float *values, int rows, int k,
                                int row_stride, float p, int32_t *counts);

#ifdef __cplusplus
}
#endif
#endif /* VKOP_ORACLE_H_ */
