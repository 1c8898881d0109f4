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
//   softmax_wave_kernel     rows of up to 512 elements: one wave per row, four rows a
//                           workgroup, no LDS.
// Strided lines (another axis, long lines):
//   softmax_strided_tile_kernel  a tile of up to 64 neighbouring lines per workgroup of 16 waves,
//                           rows dealt to the waves, three passes over the tile; with few
//                           tiles, the tile's rows split over several workgroups (two launches).
// Strided lines (another axis, short lines):
//   softmax_strided_reg_kernel  one thread per line, threads along the
//                           contiguous inner axis; the line's elements stay in
//                           registers, so the input is read once.
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
    double s;       // sum of exp(x - ref) over the chunk (softmax_stats_kernel: without the copies of its minimum)
    float m;        // maximum of the chunk (NaN ignored; -inf for an empty chunk)
    float ref;      // reference of the sum: m, or 0 when m is not finite
    float vmin;     // the value whose copies the sum leaves out (softmax_stats_kernel: the chunk's minimum; the
                    // strided tiles: the line's first element in the chunk) ...
    uint32_t nmin;  // ... and how many elements equal it (0: none set apart)
};

// ---- a whole row per workgroup ------------------------------------------------------
// A workgroup takes the rows blockIdx.x, blockIdx.x + gridDim.x, ... (the launch caps the grid:
// half a million workgroups of one short row each are handed out at about 2 ns apiece, which
// bounded [16,32,1024,1024] in both precisions); the next row's loads are issued before the
// current row's arithmetic.
constexpr uint32_t kSoftmaxRowGridMax = 16384;
template <typename T, int NT, int V, bool ALIGNED>
__global__ __launch_bounds__(NT) void softmax_row_kernel(const T *in, T *out, uint32_t rows, uint32_t n, int nan_where,
                                                         float nan_value) {
    constexpr int VEC = Vec128<T>::N;
    constexpr int NW = NT / kWave;
    __shared__ float fscratch[NW];
    __shared__ double dscratch[NW];
    const uint32_t tid = threadIdx.x;
    auto load_row = [&](Vec128<T> (&q)[V], uint32_t row) __attribute__((always_inline)) {
        const T *rowp = in + static_cast<size_t>(row) * n;
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
    };
    Vec128<T> q[V], qn[V];
    load_row(q, blockIdx.x);
    for (uint32_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const uint32_t next = row + gridDim.x;
        if (next < rows) load_row(qn, next);  // (the same in every thread)
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
        TermSum<T> acc = 0;
#pragma unroll
        for (int i = 0; i < V; i++) {
            const uint32_t e0 = (static_cast<uint32_t>(i) * NT + tid) * VEC;
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                e[i][c] = e0 + c < n ? softmax_term_as<T>(q[i].get(c), m) : 0.f;
                acc += static_cast<TermSum<T>>(e[i][c]);
            }
        }
        const double rinv = 1.0 / block_sum<NT>(static_cast<double>(acc), dscratch);
        T *orow = out + static_cast<size_t>(row) * n;
#pragma unroll
        for (int i = 0; i < V; i++) {
            const uint32_t e0 = (static_cast<uint32_t>(i) * NT + tid) * VEC;
            Vec128<T> r;
            r.v = make_uint4(0, 0, 0, 0);
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                float p = round_to_storage<T>(scale_term<T>(e[i][c], rinv));
                if (nan_where && p != p) p = nan_value;
                if constexpr (ALIGNED) r.set(c, p);
                else if (e0 + c < n) store_elem(orow, e0 + c, p);
            }
            if constexpr (ALIGNED)
                if (e0 < n) *reinterpret_cast<uint4 *>(orow + e0) = r.v;
        }
#pragma unroll
        for (int i = 0; i < V; i++) q[i] = qn[i];
    }
}

// ---- rows of a few hundred to two thousand elements, many of them: a wave per row, 128-bit loads ----
// Rows of up to 64 * V vectors that start on 16 bytes (n a multiple of the vector width): lane l
// holds vectors l, l + 64, ...; maximum and sum cross the lanes without LDS or a barrier (a
// workgroup per row pays four barriers a row for two waves' work), four rows a workgroup, each
// wave on to its next row (grid-stride) with that row's loads issued before this row's arithmetic.
constexpr int kSoftmaxVecRows = 4;  // rows (waves) per workgroup
template <typename T, int V>
__global__ __launch_bounds__(kSoftmaxVecRows *kWave) void softmax_wave_vec_kernel(const T *__restrict__ in, T *__restrict__ out,
                                                                                  uint32_t rows, uint32_t n, int nan_where,
                                                                                  float nan_value) {
    constexpr int VEC = Vec128<T>::N;
    const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const uint32_t step = gridDim.x * kSoftmaxVecRows;
    auto load_row = [&](Vec128<T> (&q)[V], uint32_t row) __attribute__((always_inline)) {
        const T *rowp = in + static_cast<size_t>(row) * n;
#pragma unroll
        for (int i = 0; i < V; i++) {
            const uint32_t e0 = (static_cast<uint32_t>(i) * kWave + lane) * VEC;
            q[i].load(rowp + (e0 < n ? e0 : 0u));
        }
    };
    uint32_t row = blockIdx.x * kSoftmaxVecRows + wave;
    if (row >= rows) return;  // (a whole wave)
    Vec128<T> q[V], qn[V];
    load_row(q, row);
    for (; row < rows; row += step) {
        if (row + step < rows) load_row(qn, row + step);  // (wave-uniform)
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < V; i++) {
            const bool live = (static_cast<uint32_t>(i) * kWave + lane) * VEC < n;
#pragma unroll
            for (int c = 0; c < VEC; c++)
                if (live) m = fmaxf(m, q[i].get(c));
        }
        m = wave_max_f32_uniform(m);
        float e[V][VEC];
        TermSum<T> acc = 0;
#pragma unroll
        for (int i = 0; i < V; i++) {
            const bool live = (static_cast<uint32_t>(i) * kWave + lane) * VEC < n;
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                e[i][c] = live ? softmax_term_as<T>(q[i].get(c), m) : 0.f;
                acc += static_cast<TermSum<T>>(e[i][c]);
            }
        }
        const double rinv = 1.0 / wave_sum_f64_uniform(static_cast<double>(acc));
        T *orow = out + static_cast<size_t>(row) * n;
#pragma unroll
        for (int i = 0; i < V; i++) {
            const uint32_t e0 = (static_cast<uint32_t>(i) * kWave + lane) * VEC;
            Vec128<T> r;
            r.v = make_uint4(0, 0, 0, 0);
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                float p = round_to_storage<T>(scale_term<T>(e[i][c], rinv));
                if (nan_where && p != p) p = nan_value;
                r.set(c, p);
            }
            if (e0 < n) *reinterpret_cast<uint4 *>(orow + e0) = r.v;
        }
#pragma unroll
        for (int i = 0; i < V; i++) q[i] = qn[i];
    }
}

// ---- short rows: one wave per row ---------------------------------------------------------
// Rows of up to 64 * E elements (E <= 8): lane l holds elements l, l + 64, ...; every
// load and store instruction of a wave covers 64 neighbouring elements whatever the row's
// alignment; maximum and sum cross the lanes without LDS or a barrier.  Four rows a
// workgroup.  (A workgroup of 256 threads per row leaves three quarters of them idle on a
// 64-element row and takes two barriers: [65536,64] took 68 us.)
constexpr int kSoftmaxWaveRows = 4;  // rows (waves) per workgroup
template <typename T, int E>
__global__ __launch_bounds__(kSoftmaxWaveRows *kWave) void softmax_wave_kernel(const T *__restrict__ in, T *__restrict__ out,
                                                                                uint32_t rows, uint32_t n, int nan_where,
                                                                                float nan_value) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t row = blockIdx.x * kSoftmaxWaveRows + threadIdx.x / kWave;
    if (row >= rows) return;  // (the whole wave)
    const T *rowp = in + static_cast<size_t>(row) * n;
    T *orow = out + static_cast<size_t>(row) * n;
    float x[E];
#pragma unroll
    for (int j = 0; j < E; j++) {
        const uint32_t e = static_cast<uint32_t>(j) * kWave + lane;
        x[j] = load_elem(rowp, e < n ? e : 0u);
    }
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < E; j++)
        if (static_cast<uint32_t>(j) * kWave + lane < n) m = fmaxf(m, x[j]);  // (drops NaN)
    m = wave_max_f32_uniform(m);
    float t[E];
    TermSum<T> acc = 0;
#pragma unroll
    for (int j = 0; j < E; j++) {
        t[j] = static_cast<uint32_t>(j) * kWave + lane < n ? softmax_term_as<T>(x[j], m) : 0.f;
        acc += static_cast<TermSum<T>>(t[j]);
    }
    const double rinv = 1.0 / wave_sum_f64_uniform(static_cast<double>(acc));
#pragma unroll
    for (int j = 0; j < E; j++) {
        const uint32_t e = static_cast<uint32_t>(j) * kWave + lane;
        float p = round_to_storage<T>(scale_term<T>(t[j], rinv));
        if (nan_where && p != p) p = nan_value;
        if (e < n) store_elem(orow, e, p);
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
    __shared__ float fscratch2[NW];
    __shared__ uint32_t uscratch[NW];
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
    // The copies of the chunk's smallest value are set apart and counted: a value that fills most
    // of a row (padding, a floor, zeros) is usually its smallest, every copy of it has the same
    // term, and that term's error would go into the sum thousands of times over -- the row's sum
    // is DEFINED with exp_accurate(fl(x - M)) for each, which only the kernel that knows M can
    // count (4 ulp on rows of one value and a few peaks otherwise).  Maximum and minimum in one
    // pass and one reduction.
    float m = -INFINITY, mn = INFINITY;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * NT + tid) * VEC;
#pragma unroll
        for (int c = 0; c < VEC; c++) {
            if (e0 + c < c1) {
                m = fmaxf(m, q[i].get(c));   // (drops NaN)
                mn = fminf(mn, q[i].get(c));
            }
        }
    }
    m = wave_max(m);
    mn = -wave_max(-mn);
    if constexpr (NW > 1) {
        if ((tid & (kWave - 1)) == 0) {
            fscratch[tid / kWave] = m;
            fscratch2[tid / kWave] = mn;
        }
        __syncthreads();
#pragma unroll
        for (int w = 0; w < NW; w++) {
            m = fmaxf(m, fscratch[w]);
            mn = fminf(mn, fscratch2[w]);
        }
    }
    // reference of the chunk's sum: its maximum, or 0 when that is not finite
    // (then every term is 0, inf or NaN, and NaN / inf must reach the sum)
    const float ref = (m > -INFINITY && m < INFINITY) ? m : 0.f;
    const bool apart = mn > -INFINITY && mn < INFINITY;  // (copies of -inf count for nothing either way)
    double acc = 0.0;
    uint32_t copies = 0;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * NT + tid) * VEC;
#pragma unroll
        for (int c = 0; c < VEC; c++) {
            if (e0 + c < c1) {
                const float x = q[i].get(c);
                copies += (x == mn) ? 1u : 0u;
                acc += static_cast<double>(fast_term_unbiased(x, ref));
            }
        }
    }
    // (every copy added the same float: taking them out again is exact to the sum's own rounding)
    if (apart) acc -= static_cast<double>(copies) * static_cast<double>(fast_term_unbiased(mn, ref));
    else copies = 0;
    acc = wave_sum(acc);
    copies = wave_sum(copies);
    if constexpr (NW > 1) {
        if ((tid & (kWave - 1)) == 0) {
            dscratch[tid / kWave] = acc;
            uscratch[tid / kWave] = copies;
        }
        __syncthreads();
        acc = dscratch[0];
        copies = uscratch[0];
#pragma unroll
        for (int w = 1; w < NW; w++) {  // fixed order: run-to-run stable
            acc += dscratch[w];
            copies += uscratch[w];
        }
    }
    if (tid == 0) stats[blockIdx.x] = ChunkStat{acc, m, ref, mn, copies};
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
    ChunkStat st{0.0, -INFINITY, 0.f, 0.f, 0u};
    if (tid < G) st = stats[static_cast<size_t>(row) * G + tid];
    const float M = block_max<NT>(st.m, fscratch);
    double part = 0.0;
    if (tid < G && st.s != 0.0) part = st.s * sum_rescale(st.s, st.ref, M);
    if (tid < G && st.nmin != 0u) part += static_cast<double>(st.nmin) * static_cast<double>(softmax_term_as<T>(st.vmin, M));
    const LineStats ls{M, 0.f, 1.0 / block_sum<NT>(part, dscratch)};
    T *orow = out + row0;
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * NT + tid) * VEC;
        Vec128<T> r;
        r.v = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int c = 0; c < VEC; c++) {
            float p = round_to_storage<T>(softmax_prob_as<T>(q[i].get(c), ls));
            if (nan_where && p != p) p = nan_value;
            if constexpr (ALIGNED) r.set(c, p);
            else if (e0 + c < c1) store_elem(orow, e0 + c, p);
        }
        if constexpr (ALIGNED)
            if (e0 < c1) *reinterpret_cast<uint4 *>(orow + e0) = r.v;
    }
}

// ---- long strided lines: a tile of neighbouring lines per workgroup -----------------------------
// Lines along a non-last axis that the register kernel below does not hold (n above
// kStridedMaxN).  A workgroup takes TI neighbouring lines (TI = the power of two at or
// above min(inner, 64)); lane l of a wave looks at line l % TI of the tile and, with 64 / TI
// rows per instruction, at row l / TI of the instruction's rows, so every load and store
// covers contiguous pieces of TI elements; the workgroup's waves take the rows in turn.
// Three passes over the tile (maximum, sum of terms, output; the second and third come
// from the cache for tiles of a few hundred kilobytes), each reduced across a wave's row
// groups by shuffles and across the waves through LDS.  One thread per line -- what this
// replaces -- had 2048 threads on a [32,1000,64] tensor: 741 us for 16 MB.
constexpr int kStridedTileThreads = 1024;
// What a launch of the tile kernel does: the whole softmax of its tiles, or -- when the tensor
// has too few tiles to fill the chip -- one of the two halves of a split over G row chunks a
// tile: every chunk's maximum and sum (hardware-exp terms against the chunk's own maximum, as
// in the chunked row kernels) into stats[(tile * G + chunk) * TI + line], then the
// probabilities from the line's G results.  G * TI <= 1024.
// The ...Max modes write, instead of the tensor, each line's largest probability to out[line]
// (softmax followed by a max over the same axis): from the same statistics, so bit-equal to
// the maximum of what the other modes write.
enum { kTileWhole = 0, kTileStats = 1, kTileScale = 2, kTileWholeMax = 3, kTileFoldMax = 4 };
template <typename T, int MODE>
__global__ __launch_bounds__(kStridedTileThreads) void softmax_strided_tile_kernel(const T *__restrict__ in, T *__restrict__ out,
                                                                                    ChunkStat *__restrict__ stats, LineGeom g,
                                                                                    uint32_t ti_shift, uint32_t G, uint32_t per,
                                                                                    int nan_where, float nan_value) {
    constexpr int NT = kStridedTileThreads, NW = NT / kWave;
    constexpr int U = 16;  // rows a lane has in flight (a pass is a chain of n / (16 waves * U) round trips)
    __shared__ float fmax_lds[NW * kWave];
    __shared__ double dsum_lds[NW * kWave];
    __shared__ uint32_t ucnt_lds[MODE == kTileStats ? NW * kWave : 1];
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t TI = 1u << ti_shift, RPW = kWave >> ti_shift;  // lines a tile, rows per wave instruction
    const uint32_t tiles = (g.inner + TI - 1) >> ti_shift;
    const uint32_t tileid = blockIdx.x / G, chunk = blockIdx.x - tileid * G;
    const uint32_t o = tileid / tiles, tile = tileid - o * tiles;
    const uint32_t c0 = min(chunk * per, g.n), c1 = min(c0 + per, g.n);  // this workgroup's rows
    const uint32_t mine = lane & (TI - 1);                               // this lane's line of the tile
    const uint32_t col = (tile << ti_shift) + mine, r = lane >> ti_shift;
    const bool col_ok = col < g.inner;
    const size_t base = static_cast<size_t>(o) * g.n * g.inner + (col_ok ? col : 0u);
    const uint32_t step = NW * RPW;  // rows the workgroup covers per turn
    // element of row j of this lane's line
    auto at = [&](uint32_t j) { return base + static_cast<size_t>(j) * g.inner; };
    // combine v over the lanes of a wave that look at the same line, then over the waves; all threads call
    auto reduce_max = [&](float v) -> float {
        for (uint32_t off = TI; off < static_cast<uint32_t>(kWave); off <<= 1) v = fmaxf(v, __shfl_xor(v, static_cast<int>(off), kWave));
        fmax_lds[tid] = v;
        __syncthreads();
        float m = fmax_lds[mine];
#pragma unroll
        for (int w = 1; w < NW; w++) m = fmaxf(m, fmax_lds[w * kWave + mine]);
        return m;
    };
    auto reduce_sum = [&](double v) -> double {
        for (uint32_t off = TI; off < static_cast<uint32_t>(kWave); off <<= 1) v += __shfl_xor(v, static_cast<int>(off), kWave);
        dsum_lds[tid] = v;
        __syncthreads();
        double sum = dsum_lds[mine];
#pragma unroll
        for (int w = 1; w < NW; w++) sum += dsum_lds[w * kWave + mine];  // fixed order: run-to-run stable
        return sum;
    };
    // one pass over the workgroup's rows: use(x, j) for every element of this lane's line
    auto pass = [&](auto use) {
        for (uint32_t j0 = c0 + wave * RPW + r; j0 < c1; j0 += step * U) {
            float x[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const uint32_t j = j0 + static_cast<uint32_t>(u) * step;
                x[u] = load_elem(in, at(j < c1 ? j : c0));
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const uint32_t j = j0 + static_cast<uint32_t>(u) * step;
                if (j < c1) use(x[u], j);
            }
        }
    };
    constexpr bool kFold = MODE == kTileScale || MODE == kTileFoldMax;
    constexpr bool kMaxOnly = MODE == kTileWholeMax || MODE == kTileFoldMax;
    if (MODE == kTileFoldMax && chunk != 0) return;  // (the whole workgroup: one writer a tile)
    LineStats st{0.f, 0.f, 0.0};
    if constexpr (!kFold) {
        // ---- 1. the lines' maxima
        float m = -INFINITY;
        pass([&](float x, uint32_t) { m = fmaxf(m, x); });  // (drops NaN)
        m = reduce_max(m);
        // ---- 2. the sums of the terms
        double acc = 0.0;
        if constexpr (MODE != kTileStats) {
            pass([&](float x, uint32_t) { acc += static_cast<double>(softmax_term_as<T>(x, m)); });
            st = LineStats{m, 0.f, 1.0 / reduce_sum(acc)};
        } else {
            // reference of the chunk's sum: its maximum, or 0 when that is not finite (then
            // every term is 0, inf or NaN, and NaN / inf must reach the sum)
            const float ref = (m > -INFINITY && m < INFINITY) ? m : 0.f;
            // The copies of ONE value are counted apart (as in softmax_stats_kernel: the kernel that knows
            // the line's maximum adds the accurate term for each): the line's first element in this chunk,
            // where the second equals it -- a value that fills a line turns up at once, every lane of the
            // line reads the same two elements (from the cache) and decides alike, and a line of spread-out
            // values pays a comparison per element and nothing else.
            const float x0 = load_elem(in, at(c0 < c1 ? c0 : 0u)), x1 = load_elem(in, at(c0 + 1u < c1 ? c0 + 1u : 0u));
            const bool apart = c0 + 1u < c1 && x0 == x1 && x0 > -INFINITY && x0 < INFINITY;
            uint32_t copies = 0;
            pass([&](float x, uint32_t) {
                if (apart && x == x0) copies += 1u;
                else acc += static_cast<double>(fast_term_unbiased(x, ref));
            });
            // (both sums in one round: over the lanes of a wave that look at the same line, then over the waves)
            for (uint32_t off = TI; off < static_cast<uint32_t>(kWave); off <<= 1) {
                acc += __shfl_xor(acc, static_cast<int>(off), kWave);
                copies += __shfl_xor(copies, static_cast<int>(off), kWave);
            }
            dsum_lds[tid] = acc;
            ucnt_lds[tid] = copies;
            __syncthreads();
            if (tid < TI) {
                double sum = dsum_lds[tid];
                uint32_t nx0 = ucnt_lds[tid];
#pragma unroll
                for (int w = 1; w < NW; w++) {  // fixed order: run-to-run stable
                    sum += dsum_lds[w * kWave + tid];
                    nx0 += ucnt_lds[w * kWave + tid];
                }
                stats[(static_cast<size_t>(tileid) * G + chunk) * TI + tid] = ChunkStat{sum, m, ref, x0, nx0};
            }
            return;
        }
    } else {
        // thread c * TI + l fetches chunk c's result for line l; every lane then folds its line's G
        const bool holds = tid < G * TI;
        ChunkStat cs{0.0, -INFINITY, 0.f, 0.f, 0u};
        if (holds) cs = stats[(static_cast<size_t>(tileid) * G + (tid >> ti_shift)) * TI + mine];
        fmax_lds[tid] = cs.m;
        __syncthreads();
        float M = fmax_lds[mine];
        for (uint32_t c = 1; c < G; c++) M = fmaxf(M, fmax_lds[c * TI + mine]);
        dsum_lds[tid] = ((holds && cs.s != 0.0) ? cs.s * sum_rescale(cs.s, cs.ref, M) : 0.0) +
                        ((holds && cs.nmin != 0u) ? static_cast<double>(cs.nmin) * static_cast<double>(softmax_term_as<T>(cs.vmin, M)) : 0.0);
        __syncthreads();
        double sum = dsum_lds[mine];
        for (uint32_t c = 1; c < G; c++) sum += dsum_lds[c * TI + mine];
        st = LineStats{M, 0.f, 1.0 / sum};
    }
    if constexpr (kMaxOnly) {
        // the line's maximum has the term exp_accurate(0) = 1 (NaN statistics give NaN, as the tensor would)
        if (tid < TI && col_ok) store_elem(out, static_cast<size_t>(o) * g.inner + col, softmax_prob_as<T>(st.m, st));
        return;
    }
    // ---- 3. the probabilities
    pass([&](float x, uint32_t j) {
        float p = round_to_storage<T>(softmax_prob_as<T>(x, st));
        if (nan_where && p != p) p = nan_value;
        if (col_ok) store_elem(out, at(j), p);
    });
}

// ---- short strided lines held in registers -------------------------------------------------
// Lines along a non-last axis with n <= kStridedMaxN elements (scores laid out
// [batch, classes, anchors]: softmax over the classes).  Lanes run along the
// contiguous inner axis, so every load is a coalesced piece of a row of the slab.
// P lanes of a wave share a line (lane l and l + 64/P, ...: element j belongs to
// part j mod P), each keeps its part in registers: one read of the input, no LDS,
// and enough waves to hide the loads and the exponentials even when the lines
// are few (one thread per line left two waves per SIMD on [16,80,8400]; staging
// the lines in LDS, the first version, no more).  NMAX: compile-time bound of n,
// a multiple of 16 and of P (the loops are unrolled over NMAX / P and masked).
constexpr int kStridedThreads = 128;
constexpr int kStridedMaxN = 128;

// MAX_ONLY: instead of the softmax tensor write, per line, its largest entry --
// the probability of the line's maximum, (float)(exp_accurate(0) / S) -- to
// out[line]: softmax followed by a max over the same axis, in one read.
template <typename T, int NMAX, int P, bool MAX_ONLY>
__global__ __launch_bounds__(kStridedThreads) void softmax_strided_reg_kernel(const T *in, T *out, LineGeom g,
                                                                              int nan_where, float nan_value) {
    constexpr int LPW = kWave / P;  // lines per wave
    constexpr int NPER = NMAX / P;  // elements per lane
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t part = lane / LPW;
    // (neighbouring groups of lines share cache lines where rows of the slab start off a line boundary)
    const uint32_t wave_id = (xcd_grouped_block() * kStridedThreads + threadIdx.x) / kWave;
    const uint32_t lines = g.outer * g.inner;
    const uint32_t line_raw = wave_id * LPW + (lane % LPW);
    const bool live = line_raw < lines;
    const uint32_t line = live ? line_raw : 0u;  // (idle lanes shadow line 0 and store nothing)
    const size_t base = g.base(line);
    const uint32_t n = g.n;
    float x[NPER];
    // every load in flight before the first use (slots past the line re-read element 0)
#pragma unroll
    for (int i = 0; i < NPER; i++) {
        const uint32_t j = static_cast<uint32_t>(i) * P + part;
        x[i] = load_elem(in, base + static_cast<size_t>(j < n ? j : 0u) * g.inner);
    }
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < NPER; i++)
        if (static_cast<uint32_t>(i) * P + part < n) m = fmaxf(m, x[i]);
#pragma unroll
    for (int o = LPW; o < kWave; o <<= 1) m = fmaxf(m, __shfl_xor(m, o, kWave));
    // terms replace the elements; the parts' sums are added in a fixed order
    TermSum<T> s_own = 0;
#pragma unroll
    for (int i = 0; i < NPER; i++) {
        if (static_cast<uint32_t>(i) * P + part < n) {
            x[i] = softmax_term_as<T>(x[i], m);
            s_own += static_cast<TermSum<T>>(x[i]);
        }
    }
    double s = static_cast<double>(s_own);
#pragma unroll
    for (int o = LPW; o < kWave; o <<= 1) s += __shfl_xor(s, o, kWave);
    const double rinv = 1.0 / s;
    if constexpr (MAX_ONLY) {
        // the largest term is exp_accurate(0) = 1 unless the line holds no finite maximum
        float top = 0.f;
#pragma unroll
        for (int i = 0; i < NPER; i++) {
            if (static_cast<uint32_t>(i) * P + part < n) {
                const float e = x[i];
                top = (e != e) ? e : ((top != top) ? top : fmaxf(top, e));  // NaN propagates
            }
        }
#pragma unroll
        for (int o = LPW; o < kWave; o <<= 1) {
            const float other = __shfl_xor(top, o, kWave);
            top = (other != other) ? other : ((top != top) ? top : fmaxf(top, other));
        }
        float p = round_to_storage<T>(scale_term<T>(top, rinv));
        if (nan_where && p != p) p = nan_value;
        if (live && part == 0) store_elem(out, line, p);
        return;
    }
#pragma unroll
    for (int i = 0; i < NPER; i++) {
        const uint32_t j = static_cast<uint32_t>(i) * P + part;
        if (live && j < n) {
            float p = round_to_storage<T>(scale_term<T>(x[i], rinv));
            if (nan_where && p != p) p = nan_value;
            store_elem(out, base + static_cast<size_t>(j) * g.inner, p);
        }
    }
}

}  // namespace vkop
