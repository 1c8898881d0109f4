// Exact top-k of long contiguous rows for any k <= kMaxK, by all workgroups of
// the chip: the route for what the streaming kernels of kernels_rows.hpp do not
// take (k > 255, smallest-first, rows too long for their merge).
//
// A radix select over the 32-bit order key, 11 + 11 + 10 bits, with the
// histograms in global memory:
//   bigk_hist_kernel<PASS>   every chunk of a row adds its histogram of the next
//                            digit (of the elements matching the digits found so
//                            far) to the row's histogram;
//   the next kernel's workgroups each locate the digit holding the k-th element
//   from that histogram (all get the same answer; the first chunk records it);
//   bigk_count_kernel        after the third digit the key T of the k-th element
//                            is known, and how many elements equal to T are
//                            wanted; counts per chunk the elements above T and
//                            equal to T;
//   bigk_gather_kernel       writes every element above T, and the wanted number
//                            of elements equal to T in index order (lowest
//                            indices first, found with prefix sums over chunks
//                            and threads), as 64-bit composites;
//   bigk_sort_kernel         one workgroup per row sorts the k composites
//                            (bitonic, LDS) and writes values and indices.
// Ties are therefore resolved exactly as everywhere else: equal keys, lower
// index first.  The row is read five times; after the first pass it comes from
// the L2 / Infinity Cache for rows sets that fit there.
// KEYS selects what is ranked: the input itself, or the probability the softmax
// of the row gives it (from the row's statistics), rounded to the tensor type.
#pragma once

#include "device_utils.hpp"
#include "kernels_general.hpp"
#include "kernels_rows.hpp"
#include "kernels_softmax.hpp"
#include "select.hpp"

namespace vkop {

constexpr int kBigThreads = 256;
constexpr int kBigSortThreads = 1024;
constexpr int kBigBins = 2048;  // digits of 11, 11 and 10 bits

struct BigKWorkspace {
    uint32_t *hist;           // [3][rows][kBigBins], zero when the first kernel starts
    uint32_t *state;          // [rows][8]: digit and remaining need after each pass
    uint32_t *counts;         // [rows][G][2]: elements above T, equal to T
    uint64_t *sel;            // [rows][kpad]
    const LineStats *stats;   // per row, for probability keys
    uint32_t kpad;
};

template <typename T, bool SOFTMAX>
__device__ __forceinline__ uint32_t bigk_key(float x, const LineStats &st, uint32_t flip) {
    if constexpr (SOFTMAX) return order_key(round_to_storage<T>(softmax_prob(x, st))) ^ flip;
    else return order_key(x) ^ flip;
}

// Inclusive suffix sums over the workgroup's threads (thread t gets the sum of
// v over threads >= t); scratch: kBigThreads words.  Ends with a barrier.
__device__ __forceinline__ uint32_t block_suffix_sum(uint32_t v, uint32_t *scratch) {
    const uint32_t tid = threadIdx.x;
    scratch[tid] = v;
    __syncthreads();
    for (uint32_t o = 1; o < kBigThreads; o <<= 1) {
        const uint32_t add = tid + o < kBigThreads ? scratch[tid + o] : 0u;
        __syncthreads();
        scratch[tid] += add;
        __syncthreads();
    }
    const uint32_t r = scratch[tid];
    __syncthreads();
    return r;
}
// Exclusive prefix sums (thread t gets the sum over threads < t).
__device__ __forceinline__ uint32_t block_prefix_sum(uint32_t v, uint32_t *scratch, uint32_t *total) {
    const uint32_t tid = threadIdx.x;
    scratch[tid] = v;
    __syncthreads();
    for (uint32_t o = 1; o < kBigThreads; o <<= 1) {
        const uint32_t add = tid >= o ? scratch[tid - o] : 0u;
        __syncthreads();
        scratch[tid] += add;
        __syncthreads();
    }
    const uint32_t incl = scratch[tid];
    *total = scratch[kBigThreads - 1];
    __syncthreads();
    return incl - v;
}

// The digit d with  #(digit > d) < need <= #(digit >= d)  in a histogram of BINS
// bins, and need - #(digit > d).  All threads call; all get the answer.
template <int BINS>
__device__ __forceinline__ void resolve_digit(const uint32_t *hist, uint32_t need, uint32_t *scratch, uint32_t *answer,
                                              uint32_t &digit, uint32_t &need_in) {
    constexpr int PER = BINS / kBigThreads;
    const uint32_t tid = threadIdx.x;
    uint32_t h[PER];
    uint32_t mine = 0;
#pragma unroll
    for (int i = 0; i < PER; i++) {
        h[i] = hist[tid * PER + i];
        mine += h[i];
    }
    const uint32_t incl = block_suffix_sum(mine, scratch);
    uint32_t above = incl - mine;  // population of the digits held by higher threads
    if (above < need && need <= incl) {
#pragma unroll
        for (int i = PER - 1; i >= 0; i--) {
            if (above < need && need <= above + h[i]) {
                answer[0] = tid * PER + static_cast<uint32_t>(i);
                answer[1] = need - above;
            }
            above += h[i];
        }
    }
    __syncthreads();
    digit = answer[0];
    need_in = answer[1];
    __syncthreads();
}

// Striped chunk: vector i of thread t starts at c0 + (i * NT + t) * VEC.
template <typename T, int V, bool ALIGNED>
__device__ __forceinline__ void bigk_load_striped(Vec128<T> (&q)[V], const T *rowp, uint32_t c0, uint32_t c1) {
    constexpr int VEC = Vec128<T>::N;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * kBigThreads + threadIdx.x) * VEC;
        q[i].v = make_uint4(0, 0, 0, 0);
        if constexpr (ALIGNED) {
            q[i].load(rowp + (e0 < c1 ? e0 : 0u));
        } else {
#pragma unroll
            for (int c = 0; c < VEC; c++) q[i].set(c, load_elem(rowp, e0 + c < c1 ? e0 + c : 0u));
        }
    }
}

// PASS 0: histogram of key >> 21.  PASS 1: of (key >> 10) & 2047 among keys whose
// top 11 bits are the first digit.  PASS 2: of key & 1023 among keys whose top 22
// bits are the first two digits.
template <typename T, int V, bool SOFTMAX, bool ALIGNED, int PASS>
__global__ __launch_bounds__(kBigThreads) void bigk_hist_kernel(const T *__restrict__ in, uint32_t n, uint32_t k,
                                                                uint32_t G, uint32_t per, uint32_t flip,
                                                                BigKWorkspace ws) {
    constexpr int VEC = Vec128<T>::N;
    constexpr int BINS = PASS == 2 ? 1024 : kBigBins;
    __shared__ uint32_t lh[kBigBins];
    __shared__ uint32_t scratch[kBigThreads];
    __shared__ uint32_t answer[2];
    const uint32_t tid = threadIdx.x;
    const uint32_t rows = gridDim.x / G;
    const uint32_t row = blockIdx.x / G, chunk = blockIdx.x - row * G;
    const uint32_t c0 = min(chunk * per, n), c1 = min(c0 + per, n);
    const T *rowp = in + static_cast<size_t>(row) * n;
    Vec128<T> q[V];
    bigk_load_striped<T, V, ALIGNED>(q, rowp, c0, c1);
    for (uint32_t b = tid; b < BINS; b += kBigThreads) lh[b] = 0;

    uint32_t *state = ws.state + static_cast<size_t>(row) * 8;
    uint32_t want_hi = 0;  // the digits found so far, as the high bits of a key
    if constexpr (PASS == 1) {
        uint32_t d, need;
        resolve_digit<kBigBins>(ws.hist + (static_cast<size_t>(0) * rows + row) * kBigBins, k, scratch, answer, d, need);
        if (chunk == 0 && tid == 0) {
            state[0] = d;
            state[1] = need;
        }
        want_hi = d;
    } else if constexpr (PASS == 2) {
        const uint32_t d0 = state[0], need0 = state[1];
        uint32_t d, need;
        resolve_digit<kBigBins>(ws.hist + (static_cast<size_t>(1) * rows + row) * kBigBins, need0, scratch, answer, d, need);
        if (chunk == 0 && tid == 0) {
            state[2] = d;
            state[3] = need;
        }
        want_hi = (d0 << 11) | d;
    }
    __syncthreads();  // lh is cleared
    LineStats st{0.f, 0.f, 0.0};
    if constexpr (SOFTMAX) st = ws.stats[row];
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * kBigThreads + tid) * VEC;
#pragma unroll
        for (int c = 0; c < VEC; c++) {
            if (e0 + c < c1) {
                const uint32_t key = bigk_key<T, SOFTMAX>(q[i].get(c), st, flip);
                // (lanes that share a digit add once between them: rows of equal values)
                if constexpr (PASS == 0) hist_add_grouped(lh, key >> 21);
                else if constexpr (PASS == 1) {
                    if ((key >> 21) == want_hi) hist_add_grouped(lh, (key >> 10) & 2047u);
                } else {
                    if ((key >> 10) == want_hi) hist_add_grouped(lh, key & 1023u);
                }
            }
        }
    }
    __syncthreads();
    uint32_t *gh = ws.hist + (static_cast<size_t>(PASS) * rows + row) * kBigBins;
    for (uint32_t b = tid; b < BINS; b += kBigThreads) {
        const uint32_t c = lh[b];
        if (c) atomicAdd(&gh[b], c);
    }
}

template <typename T, int V, bool SOFTMAX, bool ALIGNED>
__global__ __launch_bounds__(kBigThreads) void bigk_count_kernel(const T *__restrict__ in, uint32_t n, uint32_t G,
                                                                 uint32_t per, uint32_t flip, BigKWorkspace ws) {
    constexpr int VEC = Vec128<T>::N;
    __shared__ uint32_t scratch[kBigThreads];
    __shared__ uint32_t answer[2];
    const uint32_t tid = threadIdx.x;
    const uint32_t rows = gridDim.x / G;
    const uint32_t row = blockIdx.x / G, chunk = blockIdx.x - row * G;
    const uint32_t c0 = min(chunk * per, n), c1 = min(c0 + per, n);
    const T *rowp = in + static_cast<size_t>(row) * n;
    Vec128<T> q[V];
    bigk_load_striped<T, V, ALIGNED>(q, rowp, c0, c1);
    uint32_t *state = ws.state + static_cast<size_t>(row) * 8;
    const uint32_t d0 = state[0], d1 = state[2], need1 = state[3];
    uint32_t d2, need_eq;
    resolve_digit<1024>(ws.hist + (static_cast<size_t>(2) * rows + row) * kBigBins, need1, scratch, answer, d2, need_eq);
    const uint32_t thr = (d0 << 21) | (d1 << 10) | d2;  // the key of the k-th element
    if (chunk == 0 && tid == 0) {
        state[4] = thr;
        state[5] = need_eq;  // elements equal to thr that belong to the result
    }
    LineStats st{0.f, 0.f, 0.0};
    if constexpr (SOFTMAX) st = ws.stats[row];
    uint32_t gt = 0, eq = 0;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * kBigThreads + tid) * VEC;
#pragma unroll
        for (int c = 0; c < VEC; c++) {
            if (e0 + c < c1) {
                const uint32_t key = bigk_key<T, SOFTMAX>(q[i].get(c), st, flip);
                gt += key > thr ? 1u : 0u;
                eq += key == thr ? 1u : 0u;
            }
        }
    }
    uint32_t tot_gt, tot_eq;
    block_prefix_sum(gt, scratch, &tot_gt);
    block_prefix_sum(eq, scratch, &tot_eq);
    if (tid == 0) {
        ws.counts[(row * G + chunk) * 2 + 0] = tot_gt;
        ws.counts[(row * G + chunk) * 2 + 1] = tot_eq;
    }
}

// Blocked chunk: thread t owns the V * VEC consecutive elements starting at
// c0 + t * V * VEC, so thread order is index order.  G <= kBigThreads.
template <typename T, int V, bool SOFTMAX, bool ALIGNED>
__global__ __launch_bounds__(kBigThreads) void bigk_gather_kernel(const T *__restrict__ in, uint32_t n, uint32_t k,
                                                                  uint32_t G, uint32_t per, uint32_t flip,
                                                                  BigKWorkspace ws) {
    constexpr int VEC = Vec128<T>::N;
    __shared__ uint32_t scratch[kBigThreads];
    const uint32_t tid = threadIdx.x;
    const uint32_t row = blockIdx.x / G, chunk = blockIdx.x - row * G;
    const uint32_t c0 = min(chunk * per, n), c1 = min(c0 + per, n);
    const T *rowp = in + static_cast<size_t>(row) * n;
    const uint32_t t0 = c0 + tid * V * VEC;
    Vec128<T> q[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = t0 + static_cast<uint32_t>(i) * VEC;
        q[i].v = make_uint4(0, 0, 0, 0);
        if constexpr (ALIGNED) {
            q[i].load(rowp + (e0 < c1 ? e0 : 0u));
        } else {
#pragma unroll
            for (int c = 0; c < VEC; c++) q[i].set(c, load_elem(rowp, e0 + c < c1 ? e0 + c : 0u));
        }
    }
    const uint32_t *state = ws.state + static_cast<size_t>(row) * 8;
    const uint32_t thr = state[4], need_eq = state[5];
    // elements above / equal to the threshold in earlier chunks of the row
    uint32_t cg = 0, ce = 0;
    if (tid < G) {
        cg = ws.counts[(row * G + tid) * 2 + 0];
        ce = ws.counts[(row * G + tid) * 2 + 1];
    }
    uint32_t total_gt, total_eq;
    const uint32_t pg = block_prefix_sum(cg, scratch, &total_gt);
    const uint32_t pe = block_prefix_sum(ce, scratch, &total_eq);
    __shared__ uint32_t before[2];
    if (tid == chunk) {
        before[0] = pg;
        before[1] = pe;
    }
    __syncthreads();
    const uint32_t gt_before = before[0], eq_before = before[1];
    (void)total_eq;

    LineStats st{0.f, 0.f, 0.0};
    if constexpr (SOFTMAX) st = ws.stats[row];
    uint32_t keys[V * VEC];
    uint32_t gt = 0, eq = 0;
#pragma unroll
    for (int i = 0; i < V; i++) {
#pragma unroll
        for (int c = 0; c < VEC; c++) {
            const uint32_t idx = t0 + static_cast<uint32_t>(i) * VEC + c;
            const uint32_t key = idx < c1 ? bigk_key<T, SOFTMAX>(q[i].get(c), st, flip) : 0u;
            keys[i * VEC + c] = key;
            if (idx < c1) {
                gt += key > thr ? 1u : 0u;
                eq += key == thr ? 1u : 0u;
            }
        }
    }
    uint32_t dummy;
    uint32_t my_gt = gt_before + block_prefix_sum(gt, scratch, &dummy);
    uint32_t my_eq = eq_before + block_prefix_sum(eq, scratch, &dummy);
    uint64_t *sel = ws.sel + static_cast<size_t>(row) * ws.kpad;
    const uint32_t eq_base = k - need_eq;  // = elements above the threshold in the whole row
    (void)total_gt;
#pragma unroll
    for (int e = 0; e < V * VEC; e++) {
        const uint32_t idx = t0 + static_cast<uint32_t>(e);
        if (idx < c1) {
            const uint32_t key = keys[e];
            if (key > thr) {
                if (my_gt < k) sel[my_gt] = composite(key, idx);
                my_gt++;
            } else if (key == thr) {
                if (my_eq < need_eq) sel[eq_base + my_eq] = composite(key, idx);
                my_eq++;
            }
        }
    }
}

// Orders the k composites of a row and writes the result.  The composites are
// distinct, so an element's place is the number of larger ones.  A workgroup
// takes a slice of kBigSortSlice elements of one row; four threads share an
// element, each counting over a quarter of the row's list held in LDS (all lanes
// read the same word at a time, a broadcast).  No sorting network, no barrier
// stages.  Launch: rows * ceil(k / kBigSortSlice) workgroups of kBigSortThreads.
constexpr int kBigSortSlice = kBigSortThreads / 4;

template <typename T, bool SOFTMAX>
__global__ __launch_bounds__(kBigSortThreads) void bigk_sort_kernel(const T *__restrict__ in, T *__restrict__ values,
                                                                    int32_t *__restrict__ indices, uint32_t n,
                                                                    uint32_t k, uint32_t slices, BigKWorkspace ws,
                                                                    uint32_t in_order) {
    __shared__ uint64_t sel[kMaxK];
    __shared__ uint32_t rank[kBigSortSlice];
    const uint32_t tid = threadIdx.x;
    const uint32_t row = blockIdx.x / slices, slice = blockIdx.x - row * slices;
    const uint64_t *src = ws.sel + static_cast<size_t>(row) * ws.kpad;
    if (in_order == 0u) {
        // the caller did not ask for an order (sorted = 0): the k elements as the select listed them -- those
        // above the k-th element's value, then those equal to it, each group by position in the row -- without
        // the ranking
        const uint32_t t = slice * kBigSortSlice + tid;
        if (tid < static_cast<uint32_t>(kBigSortSlice) && t < k) {
            const uint32_t idx = composite_index(src[t]);
            const T *rowp = in + static_cast<size_t>(row) * n;
            if constexpr (SOFTMAX) {
                const LineStats st = ws.stats[row];
                store_elem(values, static_cast<size_t>(row) * k + t, softmax_prob(load_elem(rowp, idx), st));
            } else {
                values[static_cast<size_t>(row) * k + t] = rowp[idx];  // bit copy
            }
            indices[static_cast<size_t>(row) * k + t] = static_cast<int32_t>(idx);
        }
        return;
    }
    const uint32_t k16 = (k + 15u) & ~15u;  // four quarters of whole groups of four
    for (uint32_t t = tid; t < k16; t += kBigSortThreads) sel[t] = t < k ? src[t] : 0ull;  // 0: below every composite
    if (tid < kBigSortSlice) rank[tid] = 0;
    __syncthreads();
    const uint32_t local = tid % kBigSortSlice, quarter = tid / kBigSortSlice;
    const uint32_t t = slice * kBigSortSlice + local;
    if (t < k) {
        const uint64_t mine = sel[t];
        const uint32_t q4 = k16 / 4, j0 = quarter * q4;
        uint32_t r = 0;
        for (uint32_t j = j0; j < j0 + q4; j += 4) {
            const uint64_t a = sel[j], b = sel[j + 1], c = sel[j + 2], d = sel[j + 3];
            r += (a > mine ? 1u : 0u) + (b > mine ? 1u : 0u) + (c > mine ? 1u : 0u) + (d > mine ? 1u : 0u);
        }
        if (r) atomicAdd(&rank[local], r);
    }
    __syncthreads();
    if (quarter == 0 && t < k) {
        const uint32_t r = rank[local];
        const uint32_t idx = composite_index(sel[t]);
        const T *rowp = in + static_cast<size_t>(row) * n;
        if constexpr (SOFTMAX) {
            const LineStats st = ws.stats[row];
            store_elem(values, static_cast<size_t>(row) * k + r, softmax_prob(load_elem(rowp, idx), st));
        } else {
            values[static_cast<size_t>(row) * k + r] = rowp[idx];  // bit copy
        }
        indices[static_cast<size_t>(row) * k + r] = static_cast<int32_t>(idx);
    }
}

// Per-row softmax statistics from the chunk statistics softmax_stats_kernel
// leaves: one wave per row, fixed combination order.  Launch: rows workgroups of 64.
__global__ __launch_bounds__(kWave) void bigk_row_stats_kernel(const ChunkStat *__restrict__ chunks,
                                                               LineStats *__restrict__ stats, uint32_t G) {
    const uint32_t row = blockIdx.x, lane = threadIdx.x;
    const ChunkStat *c = chunks + static_cast<size_t>(row) * G;
    float m = -INFINITY;
    for (uint32_t g = lane; g < G; g += kWave) m = fmaxf(m, c[g].m);
    m = wave_max(m);
    double s = 0.0;
    for (uint32_t g = lane; g < G; g += kWave) {
        if (c[g].s != 0.0) s += c[g].s * sum_rescale(c[g].s, c[g].ref, m);
        // (the copies of the chunk's minimum, which its sum leaves out)
        if (c[g].nmin != 0u) s += static_cast<double>(c[g].nmin) * static_cast<double>(softmax_term(c[g].vmin, m));
    }
    s = wave_sum(s);
    if (lane == 0) stats[row] = LineStats{m, 0.f, 1.0 / s};
}

}  // namespace vkop
