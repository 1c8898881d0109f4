// General kernels: correct for every shape, axis, dtype and k the C ABI accepts.
// One workgroup per line (or one thread per line for the strided variants).
// The streaming kernels in kernels_rows.hpp take over for the shapes that
// matter for throughput; these stay as the path for everything else and as the
// exact fallback.
#pragma once

#include "device_utils.hpp"
#include "select.hpp"

namespace vkop {

// A line of the (outer, n, inner) view: element j lives at base + j * inner.
struct LineGeom {
    uint32_t outer, n, inner;
    __device__ __forceinline__ size_t base(uint32_t line) const {
        const uint32_t o = line / inner, i = line - o * inner;
        return static_cast<size_t>(o) * n * inner + i;
    }
};

struct LineStats {
    float m;      // max of the line (NaN ignored)
    float pad;
    double rinv;  // 1 / sum of exp(x - m), the sum taken in double
};

// max and sum of exp(x - max) of one line, by all NT threads of the block.
// scale: every element counts times scale (1: as it is).
template <typename T, int NT>
__device__ __forceinline__ LineStats line_stats(const T *x, size_t base, uint32_t n, uint32_t stride,
                                                float *fscratch, double *dscratch, float scale = 1.f) {
    const uint32_t tid = threadIdx.x;
    float m = -INFINITY;
    for (uint32_t j = tid; j < n; j += NT) m = fmaxf(m, scaled(load_elem(x, base + static_cast<size_t>(j) * stride), scale));
    m = block_max<NT>(m, fscratch);
    // every term is a float (as the softmax definition rounds it); the sum of
    // the terms is exact to double rounding, in a fixed order
    double a0 = 0.0, a1 = 0.0;
    uint32_t j = tid;
    for (; j + NT < n; j += 2u * NT) {
        a0 += static_cast<double>(softmax_term(scaled(load_elem(x, base + static_cast<size_t>(j) * stride), scale), m));
        a1 += static_cast<double>(softmax_term(scaled(load_elem(x, base + static_cast<size_t>(j + NT) * stride), scale), m));
    }
    if (j < n) a0 += static_cast<double>(softmax_term(scaled(load_elem(x, base + static_cast<size_t>(j) * stride), scale), m));
    const double s = block_sum<NT>(a0 + a1, dscratch);
    return LineStats{m, 0.f, 1.0 / s};
}

// Probability of one element given its line's statistics: the single formula
// every kernel uses, so separately computed results agree bit for bit.  The
// term is rounded to float first, then scaled in double and rounded once.
__device__ __forceinline__ float softmax_prob(float x, LineStats st) {
    return static_cast<float>(static_cast<double>(softmax_term(x, st.m)) * st.rinv);
}
template <typename T> __device__ __forceinline__ float softmax_prob_as(float x, LineStats st) {
    return scale_term<T>(softmax_term_as<T>(x, st.m), st.rinv);
}

// ---- softmax, one workgroup per line ---------------------------------------
template <typename T, int NT>
__global__ __launch_bounds__(NT) void softmax_lines_kernel(const T *in, T *out, LineGeom g, int nan_where,
                                                           float nan_value, LineStats *stats_out, float scale = 1.f) {
    __shared__ float fscratch[NT / kWave];
    __shared__ double dscratch[NT / kWave];
    const uint32_t line = blockIdx.x;
    const size_t base = g.base(line);
    const LineStats st = line_stats<T, NT>(in, base, g.n, g.inner, fscratch, dscratch, scale);
    if (stats_out != nullptr && threadIdx.x == 0) stats_out[line] = st;
    if (out == nullptr) return;
    for (uint32_t j = threadIdx.x; j < g.n; j += NT) {
        const size_t at = base + static_cast<size_t>(j) * g.inner;
        float p = round_to_storage<T>(softmax_prob(scaled(load_elem(in, at), scale), st));
        if (nan_where && p != p) p = nan_value;
        store_elem(out, at, p);
    }
}

// ---- softmax along a non-last axis, one thread per line --------------------
// Threads run along `inner` (contiguous), so each step over j is a coalesced
// row of the (n, inner) slab.
template <typename T, int NT>
__global__ __launch_bounds__(NT) void softmax_strided_kernel(const T *in, T *out, LineGeom g, int nan_where,
                                                             float nan_value) {
    const uint32_t line = blockIdx.x * NT + threadIdx.x;
    if (line >= g.outer * g.inner) return;
    const size_t base = g.base(line);
    float m = -INFINITY;
    for (uint32_t j = 0; j < g.n; j++) m = fmaxf(m, load_elem(in, base + static_cast<size_t>(j) * g.inner));
    double s = 0.0;
    for (uint32_t j = 0; j < g.n; j++)
        s += static_cast<double>(softmax_term(load_elem(in, base + static_cast<size_t>(j) * g.inner), m));
    const LineStats st{m, 0.f, 1.0 / s};
    for (uint32_t j = 0; j < g.n; j++) {
        const size_t at = base + static_cast<size_t>(j) * g.inner;
        float p = round_to_storage<T>(softmax_prob(load_elem(in, at), st));
        if (nan_where && p != p) p = nan_value;
        store_elem(out, at, p);
    }
}

// ---- max along an axis ------------------------------------------------------
// Strided lines: lanes run along the contiguous inner axis (coalesced rows of the
// slab); four lanes of a wave share a line (lane l, l + 16, l + 32, l + 48 take
// every fourth element), eight loads in flight per lane, so that few and short
// lines still keep the memory system busy.
template <typename T, int NT>
__global__ __launch_bounds__(NT) void reduce_max_strided_kernel(const T *__restrict__ in, T *out, LineGeom g) {
    constexpr uint32_t P = 4, LPW = kWave / P, U = 8;
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t part = lane / LPW;
    const uint32_t wave_id = (xcd_grouped_block() * NT + threadIdx.x) / kWave;  // (neighbouring lines share cache lines)
    const uint32_t lines = g.outer * g.inner;
    const uint32_t line_raw = wave_id * LPW + (lane % LPW);
    const bool live = line_raw < lines;
    const size_t base = g.base(live ? line_raw : 0u);
    float m = -INFINITY;
    bool nan = false;
    for (uint32_t j0 = part; j0 < g.n; j0 += P * U) {
        float v[U];
#pragma unroll
        for (uint32_t u = 0; u < U; u++) {
            const uint32_t j = j0 + u * P;
            v[u] = load_elem(in, base + static_cast<size_t>(j < g.n ? j : part) * g.inner);  // (re-reads one of its own)
        }
#pragma unroll
        for (uint32_t u = 0; u < U; u++) {
            nan |= (v[u] != v[u]);
            m = fmaxf(m, v[u]);
        }
    }
    float nanf = nan ? 1.f : 0.f;
#pragma unroll
    for (uint32_t o = LPW; o < kWave; o <<= 1) {
        m = fmaxf(m, __shfl_xor(m, o, kWave));
        nanf = fmaxf(nanf, __shfl_xor(nanf, o, kWave));
    }
    if (live && part == 0) store_elem(out, line_raw, nanf != 0.f ? __uint_as_float(0x7FC00000u) : m);
}

template <typename T, int NT>
__global__ __launch_bounds__(NT) void reduce_max_lines_kernel(const T *__restrict__ in, T *out, LineGeom g) {
    __shared__ float fscratch[NT / kWave];
    const uint32_t line = blockIdx.x;
    const size_t base = g.base(line);
    float m = -INFINITY;
    float nan = 0.f;
    for (uint32_t j = threadIdx.x; j < g.n; j += NT) {
        const float v = load_elem(in, base + static_cast<size_t>(j) * g.inner);
        if (v != v) nan = 1.f;
        m = fmaxf(m, v);
    }
    m = block_max<NT>(m, fscratch);
    nan = block_max<NT>(nan, fscratch);
    if (threadIdx.x == 0) store_elem(out, line, nan != 0.f ? __uint_as_float(0x7FC00000u) : m);
}

// ---- nucleus cut on sorted top-k probabilities --------------------------------
// counts[row] = the smallest m >= 1 whose first m values sum to at least p, k when
// none does.  The sum runs in float, one value after the other from the front,
// so that it is the same number on every machine: a wave reads 64 values at once
// and walks them through the lanes in order.  Launch: one wave per row.
template <typename T>
__global__ __launch_bounds__(kWave) void topp_count_kernel(const T *__restrict__ values, int32_t *__restrict__ counts, uint32_t k,
                                                            size_t row_stride, float p) {
    const T *row = values + static_cast<size_t>(blockIdx.x) * row_stride;
    const uint32_t count = nucleus_count_wave(k, p, [&](uint32_t r) { return load_elem(row, r); });
    if (threadIdx.x == 0) counts[blockIdx.x] = static_cast<int32_t>(count);
}

// ---- top-k, one workgroup per line -----------------------------------------
template <typename T, int NT>
__global__ __launch_bounds__(NT) void topk_lines_kernel(const T *__restrict__ in, T *__restrict__ values,
                                                        int32_t *__restrict__ indices, LineGeom g, uint32_t k,
                                                        int largest) {
    __shared__ SelectShared sh;
    const uint32_t line = blockIdx.x;
    const size_t base = g.base(line);
    const uint32_t flip = largest ? 0u : 0xFFFFFFFFu;
    select_topk_line<NT>(sh, g.n, k, [&](uint32_t j) {
        return order_key(load_elem(in, base + static_cast<size_t>(j) * g.inner)) ^ flip;
    });
    const uint32_t o = line / g.inner, i = line - o * g.inner;
    const size_t obase = static_cast<size_t>(o) * k * g.inner + i;
    for (uint32_t r = threadIdx.x; r < k; r += NT) {
        const uint32_t idx = composite_index(sh.sel[r]);
        values[obase + static_cast<size_t>(r) * g.inner] = in[base + static_cast<size_t>(idx) * g.inner];  // bit copy
        indices[obase + static_cast<size_t>(r) * g.inner] = static_cast<int32_t>(idx);
    }
}

// ---- top-k of the softmax of a line, from precomputed line statistics -------
// The key of element j is its probability as the output tensor would store it,
// so the result is exactly top-k (value order, then lower index) of the softmax
// tensor, including probabilities that collide after rounding.
template <typename T, int NT>
__global__ __launch_bounds__(NT) void softmax_topk_lines_kernel(const T *__restrict__ in,
                                                                const LineStats *__restrict__ stats,
                                                                T *__restrict__ values, int32_t *__restrict__ indices,
                                                                LineGeom g, uint32_t k, int largest, float scale = 1.f) {
    __shared__ SelectShared sh;
    const uint32_t line = blockIdx.x;
    const size_t base = g.base(line);
    const LineStats st = stats[line];
    const uint32_t flip = largest ? 0u : 0xFFFFFFFFu;
    select_topk_line<NT>(sh, g.n, k, [&](uint32_t j) {
        const float p = softmax_prob(scaled(load_elem(in, base + static_cast<size_t>(j) * g.inner), scale), st);
        return order_key(round_to_storage<T>(p)) ^ flip;
    });
    const uint32_t o = line / g.inner, i = line - o * g.inner;
    const size_t obase = static_cast<size_t>(o) * k * g.inner + i;
    for (uint32_t r = threadIdx.x; r < k; r += NT) {
        const uint32_t idx = composite_index(sh.sel[r]);
        const float p = softmax_prob(scaled(load_elem(in, base + static_cast<size_t>(idx) * g.inner), scale), st);
        store_elem(values, obase + static_cast<size_t>(r) * g.inner, p);
        indices[obase + static_cast<size_t>(r) * g.inner] = static_cast<int32_t>(idx);
    }
}

// ---- largest softmax entry of a line from its statistics ---------------------------------
// The line's maximum has the term exp_accurate(0) = 1, so its probability is
// (float)(1 / S); NaN statistics (NaN or +inf in the line) give NaN, as the
// softmax tensor itself would.
template <typename T> __global__ void stats_to_max_kernel(const LineStats *__restrict__ stats, T *out, uint32_t lines) {
    const uint32_t line = blockIdx.x * blockDim.x + threadIdx.x;
    if (line >= lines) return;
    const LineStats st = stats[line];
    store_elem(out, line, softmax_prob(st.m, st));
}

}  // namespace vkop
