/*
 * CPU oracle for the softmax -> top-k logits post-processing path.
 * TEST INFRASTRUCTURE ONLY -- see vkop_oracle.h.  The shipped library never
 * links or calls anything in this file.
 *
 * What pins each function (tests/test_oracle_*.py):
 *   half conversions  exhaustive over all 65536 halves and a boundary/random
 *                     sweep of floats against numpy's float16.
 *   softmax           libtorch 2.10.0 CPU goldens for the six SoftmaxTest
 *                     shapes (tests/SoftmaxTest.cpp:193-231, seed 42), closed
 *                     forms (constant line -> 1/n, n = 1 -> 1, two elements ->
 *                     logistic in long double), an 80-bit brute force on small
 *                     lines, sum-to-one, shift invariance, permutation
 *                     equivariance.
 *   top-k             libtorch goldens for the five TopkTest shapes
 *                     (tests/TopkTest.cpp:91-128, seed 56; tie free, so
 *                     indices are comparable), a stable-sort brute force,
 *                     structural invariants on tie-heavy lines.
 *   fused             composition of the two, checked the same way.
 *   get_top_k_predictions  numpy restatement on tie-free rows.
 *   reduce max        numpy's maximum (a maximum has no rounding), NaN lines.
 *   nms               the expectation of the reference's own test re-derived
 *                     in numpy on its three cases (tests/NmsTest.cpp:62-169),
 *                     invariants (kept boxes of a pair do not overlap above
 *                     the threshold, every dropped candidate overlaps an
 *                     earlier kept one), closed forms (disjoint boxes, equal
 *                     boxes, threshold >= 1, per-class limit = prefix), centre
 *                     format = corner format after conversion.
 *   topp_count        not in the reference: closed forms with exact partial
 *                     sums, numpy's sequential float32 cumsum, monotone in p.
 * Parity unpinned (no reference test or fixture fixes them, the behaviour is a
 * stated choice): the order of tied values (lower index first; libtorch's own
 * tie order is implementation defined), NaN ranking, largest == 0, rank-3
 * shapes, k >= 256; for nms the order of equal scores (lower box index first),
 * more than 1024 candidates per (batch, class) pair (the shader's array ends
 * there) and scores exactly at the threshold (left out, as the shader's >).
 */
#include "vkop_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ */
/* binary16 <-> binary32                                               */
/* ------------------------------------------------------------------ */

static uint32_t f2u(float f) {
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    return u;
}
static float u2f(uint32_t u) {
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

float vkop_oracle_half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t ex = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (ex == 0x1fu) /* inf / NaN: payload moves to the top of the fraction */
        return u2f(sign | 0x7f800000u | (man << 13));
    if (ex == 0) {
        if (man == 0)
            return u2f(sign);
        /* subnormal half = man * 2^-24, exact in float */
        float v = (float)man * 5.9604644775390625e-08f;
        return u2f(f2u(v) | sign);
    }
    return u2f(sign | ((ex + 112u) << 23) | (man << 13));
}

uint16_t vkop_oracle_float_to_half(float f) {
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) /* NaN: keep it a NaN (quiet), keep top payload bits */
        return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x1ffu));
    if (a >= 0x477ff000u) /* >= 65520 rounds to inf (65504 is the max half) */
        return (uint16_t)(sign | 0x7c00u);
    if (a < 0x33000001u) /* <= 2^-25 rounds to zero (tie at 2^-25 -> even = 0) */
        return sign;
    int e = (int)(a >> 23) - 127; /* unbiased */
    uint32_t man = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift;                                  /* bits dropped */
    uint32_t base;
    if (e < -14) { /* result is a subnormal half: value = q * 2^-24 */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7fffffu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u)))
        q++; /* may carry into the exponent field, which is the right result */
    return (uint16_t)(sign | (base + q));
}

/* ------------------------------------------------------------------ */
/* softmax                                                             */
/* ------------------------------------------------------------------ */

/* One line of n elements with element stride `st`.  x[] are the inputs widened
 * to float; y[] receives float results (rounded to half by the f16 caller). */
static void softmax_line(const float *x, float *y, int n) {
    float m = -INFINITY;
    for (int j = 0; j < n; j++)
        if (x[j] > m)
            m = x[j]; /* a NaN never wins here; it poisons the sum below */
    double s = 0.0;
    for (int j = 0; j < n; j++) {
        float d = x[j] - m; /* single precision subtraction, as the shader does */
        float e = (float)exp((double)d); /* correctly rounded float exp */
        y[j] = e;
        s += (double)e;
    }
    for (int j = 0; j < n; j++)
        y[j] = (float)((double)y[j] / s);
}

static void apply_nan_option(float *y, int n, int nan_where, float nan_value) {
    if (!nan_where)
        return;
    for (int j = 0; j < n; j++)
        if (isnan(y[j]))
            y[j] = nan_value;
}

void vkop_oracle_softmax_f32(const float *in, float *out, int outer, int n,
                             int inner, int nan_where, float nan_value) {
    if (outer <= 0 || n <= 0 || inner <= 0)
        return;
    float *x = (float *)malloc(sizeof(float) * (size_t)n * 2);
    float *y = x + n;
    for (int o = 0; o < outer; o++)
        for (int i = 0; i < inner; i++) {
            size_t base = (size_t)o * n * inner + i;
            for (int j = 0; j < n; j++)
                x[j] = in[base + (size_t)j * inner];
            softmax_line(x, y, n);
            apply_nan_option(y, n, nan_where, nan_value);
            for (int j = 0; j < n; j++)
                out[base + (size_t)j * inner] = y[j];
        }
    free(x);
}

void vkop_oracle_softmax_f16(const uint16_t *in, uint16_t *out, int outer,
                             int n, int inner, int nan_where,
                             float nan_value) {
    if (outer <= 0 || n <= 0 || inner <= 0)
        return;
    float *x = (float *)malloc(sizeof(float) * (size_t)n * 2);
    float *y = x + n;
    for (int o = 0; o < outer; o++)
        for (int i = 0; i < inner; i++) {
            size_t base = (size_t)o * n * inner + i;
            for (int j = 0; j < n; j++)
                x[j] = vkop_oracle_half_to_float(in[base + (size_t)j * inner]);
            softmax_line(x, y, n);
            apply_nan_option(y, n, nan_where, nan_value);
            for (int j = 0; j < n; j++)
                out[base + (size_t)j * inner] = vkop_oracle_float_to_half(y[j]);
        }
    free(x);
}

/* ------------------------------------------------------------------ */
/* top-k                                                               */
/* ------------------------------------------------------------------ */

/* "a ranks strictly before b" for the largest-first order: NaN above
 * everything, -0 == +0, otherwise the float comparison. */
static int ranks_before(float a, float b, int largest) {
    int an = isnan(a), bn = isnan(b);
    if (largest) {
        if (an)
            return !bn;
        if (bn)
            return 0;
        return a > b;
    }
    /* smallest first: NaN is still the largest value, so it comes last */
    if (an)
        return 0;
    if (bn)
        return 1;
    return a < b;
}

/* Keeps the best k seen so far, ordered, in (v[], ix[]).  Elements are offered
 * in index order and only a strictly better one moves ahead of an entry, so
 * equal values stay in increasing-index order and a later equal value never
 * evicts an earlier one. */
static void topk_line(const float *x, int n, int k, int largest, float *v,
                      int32_t *ix) {
    int cnt = 0;
    for (int j = 0; j < n; j++) {
        float c = x[j];
        if (cnt == k) {
            if (k == 0 || !ranks_before(c, v[k - 1], largest))
                continue;
        }
        int pos = cnt < k ? cnt : k - 1; /* slot that opens up */
        while (pos > 0 && ranks_before(c, v[pos - 1], largest)) {
            v[pos] = v[pos - 1];
            ix[pos] = ix[pos - 1];
            pos--;
        }
        v[pos] = c;
        ix[pos] = j;
        if (cnt < k)
            cnt++;
    }
}

void vkop_oracle_topk_f32(const float *in, float *values, int32_t *indices,
                          int outer, int n, int inner, int k, int largest) {
    if (outer <= 0 || n <= 0 || inner <= 0 || k <= 0)
        return;
    if (k > n)
        k = n;
    float *x = (float *)malloc(sizeof(float) * ((size_t)n + k));
    float *v = x + n;
    int32_t *ix = (int32_t *)malloc(sizeof(int32_t) * (size_t)k);
    for (int o = 0; o < outer; o++)
        for (int i = 0; i < inner; i++) {
            size_t ibase = (size_t)o * n * inner + i;
            size_t obase = (size_t)o * k * inner + i;
            for (int j = 0; j < n; j++)
                x[j] = in[ibase + (size_t)j * inner];
            topk_line(x, n, k, largest, v, ix);
            for (int j = 0; j < k; j++) {
                /* the value is a bit copy of the chosen input element */
                values[obase + (size_t)j * inner] =
                    in[ibase + (size_t)ix[j] * inner];
                indices[obase + (size_t)j * inner] = ix[j];
            }
        }
    free(x);
    free(ix);
}

void vkop_oracle_topk_f16(const uint16_t *in, uint16_t *values,
                          int32_t *indices, int outer, int n, int inner, int k,
                          int largest) {
    if (outer <= 0 || n <= 0 || inner <= 0 || k <= 0)
        return;
    if (k > n)
        k = n;
    float *x = (float *)malloc(sizeof(float) * ((size_t)n + k));
    float *v = x + n;
    int32_t *ix = (int32_t *)malloc(sizeof(int32_t) * (size_t)k);
    for (int o = 0; o < outer; o++)
        for (int i = 0; i < inner; i++) {
            size_t ibase = (size_t)o * n * inner + i;
            size_t obase = (size_t)o * k * inner + i;
            for (int j = 0; j < n; j++)
                x[j] = vkop_oracle_half_to_float(in[ibase + (size_t)j * inner]);
            topk_line(x, n, k, largest, v, ix);
            for (int j = 0; j < k; j++) {
                values[obase + (size_t)j * inner] =
                    in[ibase + (size_t)ix[j] * inner];
                indices[obase + (size_t)j * inner] = ix[j];
            }
        }
    free(x);
    free(ix);
}

/* ------------------------------------------------------------------ */
/* fused softmax -> top-k                                              */
/* ------------------------------------------------------------------ */

static void fused_line_f32(const float *in, size_t ibase, size_t obase,
                           float *probs, float *values, int32_t *indices,
                           int n, int inner, int k, int largest, float *x,
                           float *y, float *v, int32_t *ix) {
    for (int j = 0; j < n; j++)
        x[j] = in[ibase + (size_t)j * inner];
    softmax_line(x, y, n);
    if (probs)
        for (int j = 0; j < n; j++)
            probs[ibase + (size_t)j * inner] = y[j];
    topk_line(y, n, k, largest, v, ix);
    for (int j = 0; j < k; j++) {
        values[obase + (size_t)j * inner] = y[ix[j]];
        indices[obase + (size_t)j * inner] = ix[j];
    }
}

void vkop_oracle_softmax_topk_f32(const float *in, float *probs, float *values,
                                  int32_t *indices, int outer, int n,
                                  int inner, int k, int largest) {
    if (outer <= 0 || n <= 0 || inner <= 0 || k <= 0)
        return;
    if (k > n)
        k = n;
    float *x = (float *)malloc(sizeof(float) * ((size_t)2 * n + k));
    int32_t *ix = (int32_t *)malloc(sizeof(int32_t) * (size_t)k);
    for (int o = 0; o < outer; o++)
        for (int i = 0; i < inner; i++)
            fused_line_f32(in, (size_t)o * n * inner + i,
                           (size_t)o * k * inner + i, probs, values, indices,
                           n, inner, k, largest, x, x + n, x + 2 * (size_t)n,
                           ix);
    free(x);
    free(ix);
}

int vkop_oracle_softmax_topk_f32_mt(const float *in, float *values,
                                    int32_t *indices, int outer, int n,
                                    int inner, int k, int largest,
                                    int threads) {
    if (outer <= 0 || n <= 0 || inner <= 0 || k <= 0)
        return 0;
    if (k > n)
        k = n;
    int used = 1;
    long lines = (long)outer * inner;
#ifdef _OPENMP
    if (threads > 0)
        omp_set_num_threads(threads);
#pragma omp parallel
    {
#pragma omp single
        used = omp_get_num_threads();
        float *x = (float *)malloc(sizeof(float) * ((size_t)2 * n + k));
        int32_t *ix = (int32_t *)malloc(sizeof(int32_t) * (size_t)k);
#pragma omp for schedule(dynamic, 1)
        for (long l = 0; l < lines; l++) {
            int o = (int)(l / inner), i = (int)(l % inner);
            fused_line_f32(in, (size_t)o * n * inner + i,
                           (size_t)o * k * inner + i, NULL, values, indices, n,
                           inner, k, largest, x, x + n, x + 2 * (size_t)n, ix);
        }
        free(x);
        free(ix);
    }
#else
    (void)threads;
    (void)lines;
    vkop_oracle_softmax_topk_f32(in, NULL, values, indices, outer, n, inner, k,
                                 largest);
#endif
    return used;
}

void vkop_oracle_softmax_topk_f16(const uint16_t *in, uint16_t *probs,
                                  uint16_t *values, int32_t *indices,
                                  int outer, int n, int inner, int k,
                                  int largest) {
    if (outer <= 0 || n <= 0 || inner <= 0 || k <= 0)
        return;
    if (k > n)
        k = n;
    float *x = (float *)malloc(sizeof(float) * ((size_t)2 * n + k));
    float *y = x + n, *v = x + 2 * (size_t)n;
    uint16_t *yh = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)n);
    int32_t *ix = (int32_t *)malloc(sizeof(int32_t) * (size_t)k);
    for (int o = 0; o < outer; o++)
        for (int i = 0; i < inner; i++) {
            size_t ibase = (size_t)o * n * inner + i;
            size_t obase = (size_t)o * k * inner + i;
            for (int j = 0; j < n; j++)
                x[j] = vkop_oracle_half_to_float(in[ibase + (size_t)j * inner]);
            softmax_line(x, y, n);
            /* the softmax operator stores halves; top-k sees those halves */
            for (int j = 0; j < n; j++) {
                yh[j] = vkop_oracle_float_to_half(y[j]);
                y[j] = vkop_oracle_half_to_float(yh[j]);
                if (probs)
                    probs[ibase + (size_t)j * inner] = yh[j];
            }
            topk_line(y, n, k, largest, v, ix);
            for (int j = 0; j < k; j++) {
                values[obase + (size_t)j * inner] = yh[ix[j]];
                indices[obase + (size_t)j * inner] = ix[j];
            }
        }
    free(x);
    free(yh);
    free(ix);
}

/* ------------------------------------------------------------------ */
/* sampling-style variant of the fused post-proc                        */
/* ------------------------------------------------------------------ */

/* No counterpart in the reference (extensions on its softmax -> top-k path,
 * benchmark/main.cpp:85-101; the attribute parsing they would hang on is
 * ops/Topk.hpp:62-79): every logit is first multiplied by `scale` (1 /
 * temperature) in single precision, x' = fl32(x * scale); the result is the
 * fused softmax -> top-k (largest first) of x'; counts, when given, receives
 * per line the nucleus cut of vkop_oracle_topp_count_f32 on that line's k
 * sorted probabilities for top_p. */
void vkop_oracle_softmax_topk_sampling_f32(const float *in, float scale,
                                           float top_p, float *values,
                                           int32_t *indices, int32_t *counts,
                                           int outer, int n, int inner,
                                           int k) {
    if (outer <= 0 || n <= 0 || inner <= 0 || k <= 0)
        return;
    if (k > n)
        k = n;
    float *x = (float *)malloc(sizeof(float) * ((size_t)2 * n + 2 * (size_t)k));
    float *y = x + n, *v = x + 2 * (size_t)n, *pv = v + k;
    int32_t *ix = (int32_t *)malloc(sizeof(int32_t) * (size_t)k);
    for (int o = 0; o < outer; o++)
        for (int i = 0; i < inner; i++) {
            size_t ibase = (size_t)o * n * inner + i;
            size_t obase = (size_t)o * k * inner + i;
            for (int j = 0; j < n; j++) {
                volatile float t = in[ibase + (size_t)j * inner] * scale;
                x[j] = t; /* (volatile: the product rounded to float) */
            }
            softmax_line(x, y, n);
            topk_line(y, n, k, 1, v, ix);
            for (int j = 0; j < k; j++) {
                pv[j] = y[ix[j]];
                values[obase + (size_t)j * inner] = pv[j];
                indices[obase + (size_t)j * inner] = ix[j];
            }
            if (counts)
                vkop_oracle_topp_count_f32(pv, 1, k, k, top_p,
                                           counts + (size_t)o * inner + i);
        }
    free(x);
    free(ix);
}

void vkop_oracle_softmax_topk_sampling_f16(const uint16_t *in, float scale,
                                           float top_p, uint16_t *values,
                                           int32_t *indices, int32_t *counts,
                                           int outer, int n, int inner,
                                           int k) {
    if (outer <= 0 || n <= 0 || inner <= 0 || k <= 0)
        return;
    if (k > n)
        k = n;
    float *x = (float *)malloc(sizeof(float) * ((size_t)2 * n + 2 * (size_t)k));
    float *y = x + n, *v = x + 2 * (size_t)n, *pv = v + k;
    uint16_t *yh = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)n);
    int32_t *ix = (int32_t *)malloc(sizeof(int32_t) * (size_t)k);
    for (int o = 0; o < outer; o++)
        for (int i = 0; i < inner; i++) {
            size_t ibase = (size_t)o * n * inner + i;
            size_t obase = (size_t)o * k * inner + i;
            for (int j = 0; j < n; j++) {
                volatile float t =
                    vkop_oracle_half_to_float(in[ibase + (size_t)j * inner]) * scale;
                x[j] = t;
            }
            softmax_line(x, y, n);
            /* the softmax operator stores halves; top-k sees those halves */
            for (int j = 0; j < n; j++) {
                yh[j] = vkop_oracle_float_to_half(y[j]);
                y[j] = vkop_oracle_half_to_float(yh[j]);
            }
            topk_line(y, n, k, 1, v, ix);
            for (int j = 0; j < k; j++) {
                pv[j] = y[ix[j]];
                values[obase + (size_t)j * inner] = yh[ix[j]];
                indices[obase + (size_t)j * inner] = ix[j];
            }
            if (counts)
                vkop_oracle_topp_count_f32(pv, 1, k, k, top_p,
                                           counts + (size_t)o * inner + i);
        }
    free(x);
    free(yh);
    free(ix);
}

/* ------------------------------------------------------------------ */
/* reduce max, CPU post-proc restatement                               */
/* ------------------------------------------------------------------ */

void vkop_oracle_reduce_max_f32(const float *in, float *out, int outer, int n,
                                int inner) {
    if (outer <= 0 || n <= 0 || inner <= 0)
        return;
    for (int o = 0; o < outer; o++)
        for (int i = 0; i < inner; i++) {
            size_t base = (size_t)o * n * inner + i;
            float m = in[base];
            for (int j = 1; j < n; j++) {
                float c = in[base + (size_t)j * inner];
                if (isnan(c) || (!isnan(m) && c > m))
                    m = c;
            }
            out[(size_t)o * inner + i] = m;
        }
}

int vkop_oracle_get_top_k_predictions(const float *logits, int n, int k,
                                      int32_t *indices, float *probs) {
    if (n <= 0 || k <= 0)
        return 0;
    if (k > n)
        k = n;
    float *p = (float *)malloc(sizeof(float) * ((size_t)n + k));
    float maxv = logits[0]; /* std::max_element, core/function.cpp:154-155 */
    for (int j = 1; j < n; j++)
        if (logits[j] > maxv)
            maxv = logits[j];
    float sum = 0.0f;
    for (int j = 0; j < n; j++) { /* core/function.cpp:157-160 */
        p[j] = expf(logits[j] - maxv);
        sum += p[j];
    }
    for (int j = 0; j < n; j++) /* core/function.cpp:162-164 */
        p[j] /= sum;
    /* sort by probability descending and keep k, core/function.cpp:172-180 */
    topk_line(p, n, k, 1, p + n, indices);
    for (int j = 0; j < k; j++)
        probs[j] = p[indices[j]];
    free(p);
    return k;
}

/* ---- non-maximum suppression (ops/Nms.hpp, shaders/nms.comp) ---- */

static float nms_iou(const float *a, const float *b) {
    /* shaders/nms.comp:61-72 */
    float x1 = a[0] > b[0] ? a[0] : b[0];
    float y1 = a[1] > b[1] ? a[1] : b[1];
    float x2 = a[2] < b[2] ? a[2] : b[2];
    float y2 = a[3] < b[3] ? a[3] : b[3];
    if (x2 <= x1 || y2 <= y1)
        return 0.0f;
    float inter = (x2 - x1) * (y2 - y1);
    float area_a = (a[2] - a[0]) * (a[3] - a[1]);
    float area_b = (b[2] - b[0]) * (b[3] - b[1]);
    float uni = area_a + area_b - inter;
    return uni > 0.0f ? inter / uni : 0.0f;
}

int vkop_oracle_nms_f32(const float *boxes, const float *scores, int32_t *out,
                        int out_capacity, int B, int C, int N,
                        int center_point_box, int max_output_boxes_per_class,
                        float iou_threshold, float score_threshold,
                        int max_candidates) {
    int total = 0;
    float *cb = (float *)malloc((size_t)(max_candidates > 0 ? max_candidates : 1) * 4 * sizeof(float));
    float *cs = (float *)malloc((size_t)(max_candidates > 0 ? max_candidates : 1) * sizeof(float));
    int *ci = (int *)malloc((size_t)(max_candidates > 0 ? max_candidates : 1) * sizeof(int));
    char *active = (char *)malloc((size_t)(max_candidates > 0 ? max_candidates : 1));
    for (int b = 0; b < B; b++) {
        for (int c = 0; c < C; c++) {
            /* shaders/nms.comp:83-104: collect, in box order */
            int count = 0;
            for (int i = 0; i < N && count < max_candidates; i++) {
                float s = scores[((size_t)b * C + c) * N + i];
                if (s > score_threshold) {
                    const float *r = boxes + ((size_t)b * N + i) * 4;
                    float *d = cb + (size_t)count * 4;
                    if (center_point_box == 0) {
                        d[0] = r[0], d[1] = r[1], d[2] = r[2], d[3] = r[3];
                    } else { /* shaders/nms.comp:55-58 */
                        d[0] = r[0] - r[2] * 0.5f, d[1] = r[1] - r[3] * 0.5f;
                        d[2] = r[0] + r[2] * 0.5f, d[3] = r[1] + r[3] * 0.5f;
                    }
                    cs[count] = s;
                    ci[count] = i;
                    count++;
                }
            }
            /* shaders/nms.comp:107-127: selection sort, strict > keeps the
             * earlier of equal scores first */
            for (int i = 0; i < count; i++) {
                int best = i;
                for (int j = i + 1; j < count; j++)
                    if (cs[j] > cs[best])
                        best = j;
                if (best != i) {
                    /* the shader swaps; a rotation keeps the order of the others
                     * too, which is what "earlier of equal scores first" needs to
                     * hold beyond the pair -- with distinct scores both give the
                     * same list */
                    float ts = cs[best], tb[4];
                    int ti = ci[best];
                    memcpy(tb, cb + (size_t)best * 4, sizeof tb);
                    for (int j = best; j > i; j--) {
                        cs[j] = cs[j - 1];
                        ci[j] = ci[j - 1];
                        memcpy(cb + (size_t)j * 4, cb + (size_t)(j - 1) * 4, sizeof tb);
                    }
                    cs[i] = ts;
                    ci[i] = ti;
                    memcpy(cb + (size_t)i * 4, tb, sizeof tb);
                }
                active[i] = 1;
            }
            /* shaders/nms.comp:148-188 */
            int max_out = count;
            if (max_output_boxes_per_class > 0 && max_output_boxes_per_class < count)
                max_out = max_output_boxes_per_class;
            int selected = 0;
            for (int i = 0; i < count && selected < max_out; i++) {
                if (!active[i])
                    continue;
                if (total < out_capacity) {
                    out[(size_t)total * 3 + 0] = b;
                    out[(size_t)total * 3 + 1] = c;
                    out[(size_t)total * 3 + 2] = ci[i];
                }
                total++;
                selected++;
                for (int j = i + 1; j < count; j++)
                    if (active[j] && nms_iou(cb + (size_t)j * 4, cb + (size_t)i * 4) > iou_threshold)
                        active[j] = 0;
            }
        }
    }
    free(cb);
    free(cs);
    free(ci);
    free(active);
    return total;
}

/* ------------------------------------------------------------------ */
/* nucleus (top-p) cut on sorted top-k probabilities                   */
/* ------------------------------------------------------------------ */

/* No counterpart in the reference (a sampling-style extension on its softmax ->
 * top-k path, benchmark/main.cpp:85-101): the usual sampler rule, keep leading
 * values until their running float sum reaches p, the one that crosses included. */
void vkop_oracle_topp_count_f32(const float *values, int rows, int k,
                                int row_stride, float p, int32_t *counts) {
    for (int r = 0; r < rows; r++) {
        const float *v = values + (size_t)r * row_stride;
        volatile float sum = 0.0f; /* (volatile: every partial sum rounded to float) */
        int count = k;
        for (int j = 0; j < k; j++) {
            sum = sum + v[j];
            if (sum >= p) {
                count = j + 1;
                break;
            }
        }
        counts[r] = count;
    }
}
