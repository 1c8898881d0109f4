// Throughput kernels for the plain softmax operator.
//
// Contiguous rows (the reduced axis is the last one):
//   softmax_row_kernel      one workgroup holds a whole row in registers: one
//                           read, one write (rows up to NT * V vectors).
//   softmax_stats_kernel +  long rows, or too few rows to fill the chip: a row
//   softmax_scale_kernel    is split into chunks, one workgroup each.  The first
//                           kernel leaves (maximum, sum of exp(x - maximum)) per
//                           chunk, the second combines a row's chunk results and
//                           writes exp(x - M) / S for its chunk.  The second
//                           read of the input comes from the Infinity Cache for
//                           tensors that fit it.
// Strided lines (another axis, short lines):
//   softmax_strided_lds_kernel  one thread per line, threads along the
//                           contiguous inner axis; the line's elements are staged
//                           in LDS ([element][thread], conflict free), so the
//                           input is read once and the loops stay loops.
// All of them produce what kernels_general.hpp defines: terms exp_accurate(x - M),
// the sum in double, one rounding of term * (1 / sum).  The chunked variant sums
// hardware-exp terms (argument scaled with a two-part log2 e, so the scaling adds
// no bias); the sum's relative error of ~1e-8 is far below a float ulp.
#pragma once

#include "device_utils.hpp"
#include "kernels_general.hpp"
#include "kernels_rows.hpp"

namespace vkop {

// exp(x - m) on the hardware unit with an unbiased argument: (x - m) * log2 e
// evaluated with log2 e split in two floats.
__device__ __forceinline__ float fast_term_unbiased(float x, float m) {
    const float d = x - m;
    constexpr float kHi = 1.44269502162933349609375f;    // float(log2 e)
    constexpr float kLo = 1.925963033500011e-8f;         // log2 e - kHi
    return __builtin_amdgcn_exp2f(fmaf(d, kHi, d * kLo));
}

struct ChunkStat {
    double s;   // sum of exp(x - ref) over the chunk
    float m;    // maximum of the chunk (NaN ignored; -inf for an empty chunk)
    float ref;  // reference of the sum: m, or 0 when m is not finite
};

// ---- a whole row per workgroup ------------------------------------------------------
template <typename T, int NT, int V, bool ALIGNED>
__global__ __launch_bounds__(NT) void softmax_row_kernel(const T *in, T *out, uint32_t n, int nan_where,
                                                         float nan_value) {
    constexpr int VEC = Vec128<T>::N;
    constexpr int NW = NT / kWave;
    __shared__ float fscratch[NW];
    __shared__ double dscratch[NW];
    const uint32_t tid = threadIdx.x;
    const size_t row0 = static_cast<size_t>(blockIdx.x) * n;
    const T *rowp = in + row0;
    Vec128<T> q[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = (static_cast<uint32_t>(i) * NT + tid) * VEC;
        q[i].v = make_uint4(0, 0, 0, 0);
        if constexpr (ALIGNED) {
            q[i].load(rowp + (e0 < n ? e0 : 0u));
        } else {
#pragma unroll
            for (int c = 0; c < VEC; c++) q[i].set(c, load_elem(rowp, e0 + c < n ? e0 + c : 0u));
        }
    }
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = (static_cast<uint32_t>(i) * NT + tid) * VEC;
#pragma unroll
        for (int c = 0; c < VEC; c++)
            if (e0 + c < n) m = fmaxf(m, q[i].get(c));
    }
    m = block_max<NT>(m, fscratch);
    // the terms replace the inputs in the registers (a term is a float; for half
    // tensors it is kept in a float array instead)
    float e[V][VEC];
    double acc = 0.0;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = (static_cast<uint32_t>(i) * NT + tid) * VEC;
#pragma unroll
        for (int c = 0; c < VEC; c++) {
            e[i][c] = e0 + c < n ? softmax_term(q[i].get(c), m) : 0.f;
            acc += static_cast<double>(e[i][c]);
        }
    }
    const double rinv = 1.0 / block_sum<NT>(acc, dscratch);
    T *orow = out + row0;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = (static_cast<uint32_t>(i) * NT + tid) * VEC;
        Vec128<T> r;
        r.v = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int c = 0; c < VEC; c++) {
            float p = round_to_storage<T>(static_cast<float>(static_cast<double>(e[i][c]) * rinv));
            if (nan_where && p != p) p = nan_value;
            if constexpr (ALIGNED) r.set(c, p);
            else if (e0 + c < n) store_elem(orow, e0 + c, p);
        }
        if constexpr (ALIGNED)
            if (e0 < n) *reinterpret_cast<uint4 *>(orow + e0) = r.v;
    }
}

// ---- chunked rows: statistics ---------------------------------------------------------
// Launch: rows * G workgroups; per = elements per chunk (multiple of the vector
// width, <= NT * V * vector width).
template <typename T, int NT, int V, bool ALIGNED>
__global__ __launch_bounds__(NT) void softmax_stats_kernel(const T *__restrict__ in, ChunkStat *__restrict__ stats,
                                                           uint32_t n, uint32_t G, uint32_t per) {
    constexpr int VEC = Vec128<T>::N;
    constexpr int NW = NT / kWave;
    __shared__ float fscratch[NW];
    __shared__ double dscratch[NW];
    const uint32_t tid = threadIdx.x;
    const uint32_t row = blockIdx.x / G, chunk = blockIdx.x - row * G;
    const uint32_t c0 = min(chunk * per, n), c1 = min(c0 + per, n);
    const T *rowp = in + static_cast<size_t>(row) * n;
    Vec128<T> q[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * NT + tid) * VEC;
        q[i].v = make_uint4(0, 0, 0, 0);
        if constexpr (ALIGNED) {
            q[i].load(rowp + (e0 < c1 ? e0 : 0u));
        } else {
#pragma unroll
            for (int c = 0; c < VEC; c++) q[i].set(c, load_elem(rowp, e0 + c < c1 ? e0 + c : 0u));
        }
    }
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * NT + tid) * VEC;
#pragma unroll
        for (int c = 0; c < VEC; c++)
            if (e0 + c < c1) m = fmaxf(m, q[i].get(c));
    }
    m = block_max<NT>(m, fscratch);
    // reference of the chunk's sum: its maximum, or 0 when that is not finite
    // (then every term is 0, inf or NaN, and NaN / inf must reach the sum)
    const float ref = (m > -INFINITY && m < INFINITY) ? m : 0.f;
    double acc = 0.0;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * NT + tid) * VEC;
#pragma unroll
        for (int c = 0; c < VEC; c++)
            if (e0 + c < c1) acc += static_cast<double>(fast_term_unbiased(q[i].get(c), ref));
    }
    const double s = block_sum<NT>(acc, dscratch);
    if (tid == 0) stats[blockIdx.x] = ChunkStat{s, m, ref};
}

// ---- chunked rows: exp(x - M) / S -----------------------------------------------------
template <typename T, int NT, int V, bool ALIGNED>
__global__ __launch_bounds__(NT) void softmax_scale_kernel(const T *in, T *out, const ChunkStat *__restrict__ stats,
                                                           uint32_t n, uint32_t G, uint32_t per, int nan_where,
                                                           float nan_value) {
    constexpr int VEC = Vec128<T>::N;
    constexpr int NW = NT / kWave;
    __shared__ float fscratch[NW];
    __shared__ double dscratch[NW];
    const uint32_t tid = threadIdx.x;
    const uint32_t row = blockIdx.x / G, chunk = blockIdx.x - row * G;
    const uint32_t c0 = min(chunk * per, n), c1 = min(c0 + per, n);
    const size_t row0 = static_cast<size_t>(row) * n;
    const T *rowp = in + row0;
    Vec128<T> q[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * NT + tid) * VEC;
        q[i].v = make_uint4(0, 0, 0, 0);
        if constexpr (ALIGNED) {
            q[i].load(rowp + (e0 < c1 ? e0 : 0u));
        } else {
#pragma unroll
            for (int c = 0; c < VEC; c++) q[i].set(c, load_elem(rowp, e0 + c < c1 ? e0 + c : 0u));
        }
    }
    // the row's maximum and sum from its G chunk results (G <= NT)
    ChunkStat st{0.0, -INFINITY, 0.f};
    if (tid < G) st = stats[static_cast<size_t>(row) * G + tid];
    const float M = block_max<NT>(st.m, fscratch);
    double part = 0.0;
    if (tid < G && st.s != 0.0) part = st.s * exp(static_cast<double>(st.ref) - static_cast<double>(M));
    const LineStats ls{M, 0.f, 1.0 / block_sum<NT>(part, dscratch)};
    T *orow = out + row0;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * NT + tid) * VEC;
        Vec128<T> r;
        r.v = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int c = 0; c < VEC; c++) {
            float p = round_to_storage<T>(softmax_prob(q[i].get(c), ls));
            if (nan_where && p != p) p = nan_value;
            if constexpr (ALIGNED) r.set(c, p);
            else if (e0 + c < c1) store_elem(orow, e0 + c, p);
        }
        if constexpr (ALIGNED)
            if (e0 < c1) *reinterpret_cast<uint4 *>(orow + e0) = r.v;
    }
}

// ---- short strided lines, staged in LDS --------------------------------------------------
// One thread per line; n <= kStridedMaxN.  Dynamic LDS: n * NT floats.
constexpr int kStridedThreads = 128;
constexpr int kStridedMaxN = 128;

// MAX_ONLY: instead of the softmax tensor write, per line, its largest entry --
// the probability of the line's maximum, (float)(exp_accurate(0) / S) -- to
// out[line]: softmax followed by a max over the same axis, in one read.
template <typename T, bool MAX_ONLY>
__global__ __launch_bounds__(kStridedThreads) void softmax_strided_lds_kernel(const T *in, T *out, LineGeom g,
                                                                              int nan_where, float nan_value) {
    constexpr int NT = kStridedThreads;
    extern __shared__ float stage[];  // [n][NT]
    const uint32_t tid = threadIdx.x;
    const uint32_t line = blockIdx.x * NT + tid;
    const bool live = line < g.outer * g.inner;
    const size_t base = live ? g.base(line) : 0;
    // loads in batches of sixteen, all in flight before the first use
    float m = -INFINITY;
    for (uint32_t j0 = 0; j0 < g.n; j0 += 16) {
        float x[16];
#pragma unroll
        for (int u = 0; u < 16; u++) {
            const uint32_t j = j0 + u < g.n ? j0 + u : 0u;
            x[u] = load_elem(in, base + static_cast<size_t>(j) * g.inner);
        }
#pragma unroll
        for (int u = 0; u < 16; u++) {
            if (j0 + u < g.n) {
                stage[(j0 + u) * NT + tid] = x[u];
                m = fmaxf(m, x[u]);
            }
        }
    }
    // four independent exponentials in flight per thread (few waves fit beside
    // this much LDS, so the instruction-level parallelism has to come from here);
    // the sum itself stays in index order
    double s = 0.0;
    uint32_t j4 = 0;
    for (; j4 + 4 <= g.n; j4 += 4) {
        float e[4];
#pragma unroll
        for (int u = 0; u < 4; u++) e[u] = softmax_term(stage[(j4 + u) * NT + tid], m);
#pragma unroll
        for (int u = 0; u < 4; u++) {
            stage[(j4 + u) * NT + tid] = e[u];
            s += static_cast<double>(e[u]);
        }
    }
    for (uint32_t j = j4; j < g.n; j++) {
        const float e = softmax_term(stage[j * NT + tid], m);
        stage[j * NT + tid] = e;
        s += static_cast<double>(e);
    }
    const double rinv = 1.0 / s;
    if (!live) return;
    if constexpr (MAX_ONLY) {
        // the largest term is exp_accurate(0) = 1 unless the line holds no finite maximum
        float top = 0.f;
        for (uint32_t j = 0; j < g.n; j++) {
            const float e = stage[j * NT + tid];
            top = (e != e) ? e : ((top != top) ? top : fmaxf(top, e));  // NaN propagates
        }
        float p = round_to_storage<T>(static_cast<float>(static_cast<double>(top) * rinv));
        if (nan_where && p != p) p = nan_value;
        store_elem(out, line, p);
        return;
    }
    for (uint32_t j = 0; j < g.n; j++) {
        float p = round_to_storage<T>(static_cast<float>(static_cast<double>(stage[j * NT + tid]) * rinv));
        if (nan_where && p != p) p = nan_value;
        store_elem(out, base + static_cast<size_t>(j) * g.inner, p);
    }
}

}  // namespace vkop
