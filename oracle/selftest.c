/* Memory-safety self-test of the CPU oracle (test infrastructure, like the oracle
 * itself): every function is called on heap buffers of exactly the size its
 * contract names, at the edge shapes (k = 0, k = n, n = 1, inner > 1, all-NaN
 * lines, an output capacity smaller than the result), so that a read or write
 * past a buffer is caught when this file is built with -fsanitize=address,undefined
 * (`make -C oracle asan`).  A few value checks that need no second implementation
 * ride along: softmax lines sum to 1, top-k values descend and carry their indices.
 * Exit status 0 = clean. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "vkop_oracle.h"

static int g_failed = 0, g_checked = 0;
#define EXPECT(c)                                                     \
    do {                                                              \
        g_checked++;                                                  \
        if (!(c)) {                                                   \
            g_failed++;                                               \
            printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #c);       \
        }                                                             \
    } while (0)

static uint32_t g_rng = 12345u;
static float rnd(void) { /* uniform in [-4, 4) */
    g_rng = g_rng * 1664525u + 1013904223u;
    return (float)(g_rng >> 8) / (float)(1u << 24) * 8.f - 4.f;
}

static void *exact(size_t bytes) { /* malloc(0) may return NULL: keep one byte */
    void *p = malloc(bytes ? bytes : 1);
    if (!p) {
        printf("out of memory\n");
        exit(2);
    }
    return p;
}

static void fill(float *x, size_t cnt, int kind) {
    for (size_t i = 0; i < cnt; i++) {
        float v = rnd();
        if (kind == 1) v = (float)((int)(v * 2.f)) * 0.5f;     /* many ties */
        if (kind == 2 && (i % 7) == 3) v = NAN;                 /* NaNs inside */
        if (kind == 3) v = NAN;                                 /* all NaN */
        if (kind == 4) v = (i % 5) == 0 ? INFINITY : ((i % 5) == 1 ? -INFINITY : v);
        x[i] = v;
    }
}

static void one_shape(int outer, int n, int inner, int k, int kind) {
    const size_t cnt = (size_t)outer * n * inner, kcnt = (size_t)outer * k * inner, lines = (size_t)outer * inner;
    float *x = exact(cnt * 4), *p = exact(cnt * 4), *v = exact(kcnt * 4);
    int32_t *ix = exact(kcnt * 4), *counts = exact(lines * 4);
    uint16_t *hx = exact(cnt * 2), *hp = exact(cnt * 2), *hv = exact(kcnt * 2);
    fill(x, cnt, kind);
    for (size_t i = 0; i < cnt; i++) hx[i] = vkop_oracle_float_to_half(x[i]);

    vkop_oracle_softmax_f32(x, p, outer, n, inner, 0, 0.f);
    if (kind <= 1)
        for (int o = 0; o < outer; o++)
            for (int in = 0; in < inner; in++) {
                double s = 0;
                for (int j = 0; j < n; j++) s += p[((size_t)o * n + j) * inner + in];
                EXPECT(fabs(s - 1.0) < 1e-5);
            }
    vkop_oracle_softmax_f32(x, p, outer, n, inner, 1, 0.25f);
    for (size_t i = 0; i < cnt; i++) EXPECT(!isnan(p[i]));
    vkop_oracle_softmax_f16(hx, hp, outer, n, inner, 0, 0.f);
    vkop_oracle_softmax_f16(hx, hp, outer, n, inner, 1, 0.25f);

    for (int largest = 0; largest < 2; largest++) {
        vkop_oracle_topk_f32(x, v, ix, outer, n, inner, k, largest);
        for (int o = 0; o < outer; o++)
            for (int in = 0; in < inner; in++)
                for (int j = 0; j < k; j++) {
                    const size_t at = ((size_t)o * k + j) * inner + in;
                    EXPECT(ix[at] >= 0 && ix[at] < n);
                    const float src = x[((size_t)o * n + ix[at]) * inner + in];
                    EXPECT(memcmp(&src, &v[at], 4) == 0 || (isnan(src) && isnan(v[at])));
                    if (j && kind <= 1) {
                        const float prev = v[at - inner];
                        EXPECT(largest ? prev >= v[at] : prev <= v[at]);
                        if (prev == v[at]) EXPECT(ix[at - inner] < ix[at]);
                    }
                }
        vkop_oracle_topk_f16(hx, hv, ix, outer, n, inner, k, largest);
        vkop_oracle_softmax_topk_f32(x, NULL, v, ix, outer, n, inner, k, largest);
        vkop_oracle_softmax_topk_f32(x, p, v, ix, outer, n, inner, k, largest);
        vkop_oracle_softmax_topk_f16(hx, NULL, hv, ix, outer, n, inner, k, largest);
        vkop_oracle_softmax_topk_f16(hx, hp, hv, ix, outer, n, inner, k, largest);
        EXPECT(vkop_oracle_softmax_topk_f32_mt(x, v, ix, outer, n, inner, k, largest, 3) >= (k > 0));
    }
    vkop_oracle_softmax_topk_sampling_f32(x, 1.25f, 0.9f, v, ix, NULL, outer, n, inner, k);
    vkop_oracle_softmax_topk_sampling_f32(x, 0.5f, 0.9f, v, ix, counts, outer, n, inner, k);
    if (k > 0)
        for (size_t l = 0; l < lines; l++) EXPECT(counts[l] >= 1 && counts[l] <= k);
    vkop_oracle_softmax_topk_sampling_f16(hx, 1.25f, 0.5f, hv, ix, counts, outer, n, inner, k);

    float *mx = exact(lines * 4);
    vkop_oracle_reduce_max_f32(x, mx, outer, n, inner);
    free(mx);

    if (k > 0 && inner == 1) {
        vkop_oracle_softmax_topk_f32(x, NULL, v, ix, outer, n, 1, k, 1);
        vkop_oracle_topp_count_f32(v, outer, k, k, 0.5f, counts);
        vkop_oracle_topp_count_f32(v, outer, k, k, 2.0f, counts);
        for (int o = 0; o < outer; o++) EXPECT(counts[o] == k);
    }
    free(x); free(p); free(v); free(ix); free(counts); free(hx); free(hp); free(hv);
}

static void predictions(void) {
    for (int n = 1; n <= 9; n += 4)
        for (int k = 0; k <= n + 2; k += (n > 4 ? 3 : 1)) {
            const int w = k < n ? k : n;
            float *x = exact((size_t)n * 4), *pr = exact((size_t)w * 4);
            int32_t *ix = exact((size_t)w * 4);
            fill(x, (size_t)n, 1);
            EXPECT(vkop_oracle_get_top_k_predictions(x, n, k, ix, pr) == w);
            for (int j = 1; j < w; j++) EXPECT(pr[j - 1] >= pr[j]);
            free(x); free(pr); free(ix);
        }
}

static void nms(void) {
    const int B = 2, C = 3, N = 40;
    float *boxes = exact((size_t)B * N * 4 * 4), *scores = exact((size_t)B * C * N * 4);
    for (int i = 0; i < B * N; i++) {
        const float cx = rnd() + 4.f, cy = rnd() + 4.f, w = fabsf(rnd()) * 0.5f + 0.1f, h = fabsf(rnd()) * 0.5f + 0.1f;
        boxes[i * 4 + 0] = cx - w; boxes[i * 4 + 1] = cy - h; boxes[i * 4 + 2] = cx + w; boxes[i * 4 + 3] = cy + h;
    }
    for (int i = 0; i < B * C * N; i++) scores[i] = (rnd() + 4.f) / 8.f;
    for (int cpb = 0; cpb < 2; cpb++)
        for (int cap = 0; cap <= 3 * B * C * N; cap += B * C * N) {
            int32_t *out = exact((size_t)cap * 3 * 4);
            const int total = vkop_oracle_nms_f32(boxes, scores, out, cap, B, C, N, cpb, 0, 0.5f, 0.2f, 1024);
            EXPECT(total >= 0 && total <= B * C * N);
            const int wrote = total < cap ? total : cap;
            for (int r = 0; r < wrote; r++) {
                EXPECT(out[r * 3] >= 0 && out[r * 3] < B);
                EXPECT(out[r * 3 + 1] >= 0 && out[r * 3 + 1] < C);
                EXPECT(out[r * 3 + 2] >= 0 && out[r * 3 + 2] < N);
            }
            free(out);
        }
    {   /* fewer candidate slots than boxes above the threshold, and a per-class limit */
        int32_t *out = exact((size_t)B * C * N * 3 * 4);
        const int a = vkop_oracle_nms_f32(boxes, scores, out, B * C * N, B, C, N, 0, 2, 0.5f, 0.0f, 7);
        EXPECT(a <= 2 * B * C);
        free(out);
    }
    free(boxes); free(scores);
}

static void halves(void) {
    for (uint32_t h = 0; h < 65536u; h++) {
        const float f = vkop_oracle_half_to_float((uint16_t)h);
        const uint16_t back = vkop_oracle_float_to_half(f);
        if (isnan(f)) EXPECT((back & 0x7C00u) == 0x7C00u && (back & 0x3FFu) != 0);
        else EXPECT(back == (uint16_t)h);
    }
}

int main(void) {
    static const int shapes[][4] = {
        /* outer, n, inner, k */
        {1, 1, 1, 1}, {1, 1, 1, 0}, {3, 17, 1, 17}, {3, 17, 1, 5}, {2, 9, 4, 3}, {1, 300, 1, 256},
        {2, 1000, 1, 50}, {2, 5, 3, 0}, {1, 1030, 2, 40}, {4, 64, 1, 1},
    };
    for (size_t s = 0; s < sizeof(shapes) / sizeof(shapes[0]); s++)
        for (int kind = 0; kind <= 4; kind++) one_shape(shapes[s][0], shapes[s][1], shapes[s][2], shapes[s][3], kind);
    predictions();
    nms();
    halves();
    printf("%d checks, %d failed\n", g_checked, g_failed);
    return g_failed ? 1 : 0;
}
