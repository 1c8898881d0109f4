// Streaming kernels for contiguous rows (the reduced axis is the last one).
//
// rows_chunk_kernel makes the one pass over the input.  A row is split into G
// chunks, one workgroup per chunk, so a few long rows still fill the chip.
// Each workgroup
//   1. pulls its chunk into registers with 128-bit loads (V per thread),
//   2. reduces max and sum of exp(x - max) (wave DPP + one LDS hop),
//   3. finds a threshold that at least k+1 of its elements reach -- per wave the
//      c-th largest per-lane maximum, then the minimum over the waves -- and
//      appends the few elements above it to an LDS list,
//   4. ranks that list exactly (key, then lower index) and writes its k+1 best,
//      in order, plus (max, sum) to the workspace.
// rows_merge_kernel (one workgroup per row; run inside the chunk kernel when
// G == 1) merges the G partial results the same way, computes the
// probabilities of the winners only, orders equal probabilities by index and
// writes the row's result.  There are no atomics or fences between workgroups:
// the kernel boundary publishes the partial results, and the outcome does not
// depend on scheduling.
// Whatever the shortcut cannot prove exact (too many elements at a threshold,
// a probability tie across the k-th place, NaN/inf rows) is redone by the
// merging workgroup with the exact radix select of select.hpp, so the result
// is always top-k (probability, then lower index) of the row's softmax.
#pragma once

#include "device_utils.hpp"
#include "kernels_general.hpp"
#include "select.hpp"

namespace vkop {

constexpr int kFastCap = 1024;     // LDS slots for elements above a threshold
constexpr int kFastMaxK = 255;     // k + 1 <= 256 ranks are kept in LDS
constexpr int kMergeThreads = 1024;
constexpr int kMergeSlots = 4096;  // G * (k + 1) the merge takes in registers

// ---- wave-level helpers (all 64 lanes must be active) -----------------------

// max over the wave, returned wave-uniform: four DPP-fused steps inside each
// row of 16 lanes, then the four row results through scalar registers.
#define VKOP_DPP_U32(a, ctrl) \
    static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(a), ctrl, 0xF, 0xF, true))
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = max(v, VKOP_DPP_U32(v, 0xB1));   // quad_perm 1,0,3,2
    v = max(v, VKOP_DPP_U32(v, 0x4E));   // quad_perm 2,3,0,1
    v = max(v, VKOP_DPP_U32(v, 0x141));  // row_half_mirror
    v = max(v, VKOP_DPP_U32(v, 0x140));  // row_mirror
    const uint32_t r0 = __builtin_amdgcn_readlane(static_cast<int>(v), 0);
    const uint32_t r1 = __builtin_amdgcn_readlane(static_cast<int>(v), 16);
    const uint32_t r2 = __builtin_amdgcn_readlane(static_cast<int>(v), 32);
    const uint32_t r3 = __builtin_amdgcn_readlane(static_cast<int>(v), 48);
    return max(max(r0, r1), max(r2, r3));
}
#undef VKOP_DPP_U32

// Bijective order-preserving float <-> uint32 (no NaN / -0 canonicalisation).
__device__ __forceinline__ uint32_t float_to_ordered(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float ordered_to_float(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k);
}
__device__ __forceinline__ float wave_max_f32_uniform(float v) {
    return ordered_to_float(wave_max_u32(float_to_ordered(v)));
}

// A lower bound, wave-uniform, of the c-th largest (1 <= c <= 64) of the 64 lane
// values that at least c lanes reach: bitwise descent over the top `bits` bits
// with ballots (the low bits stay zero, which only lowers the bound).  Returns
// 0 when fewer than c lanes are non-zero.
__device__ __forceinline__ uint32_t wave_cth_largest_floor(uint32_t v, uint32_t c, int bits) {
    uint32_t prefix = 0;
    for (int bit = 31; bit > 31 - bits; bit--) {
        const uint32_t trial = prefix | (1u << bit);
        if (static_cast<uint32_t>(__popcll(__ballot(v >= trial))) >= c) prefix = trial;
    }
    return prefix;
}

// ---- workspace ---------------------------------------------------------------

struct ChunkPartial {
    double s;        // sum of exp(x - m) over the chunk
    float m;         // chunk max
    uint32_t count;  // candidates written (<= k + 1), in rank order
    uint32_t flags;  // bit 0: the chunk could not bound its candidates -> exact path
    uint32_t pad[3];
};

struct RowsWorkspace {
    ChunkPartial *partials;  // [rows][G]
    uint64_t *cands;         // [rows][G][kc]
    uint32_t kc;             // slots per chunk (k + 1)
};

struct RowsShared {
    uint64_t cand[kFastCap];
    uint32_t rank[kFastCap];
    float prob[kFastMaxK + 1];
    uint32_t pidx[kFastMaxK + 1];
    uint32_t wave_key[16];
    uint32_t wave_valid[16];
    float wave_m[16];
    double wave_s[16];
    uint32_t count;
    // row statistics published by wave 0 of the merging workgroup
    float row_m;
    uint32_t row_total, row_slow;
    double row_rinv;
};

union RowsSharedUnion {
    RowsShared fast;
    SelectShared exact;
    __device__ RowsSharedUnion() {}
};

// Fast term for the running sum: exp2((x - m) * log2 e) on the hardware
// exponential unit.  Only ever summed; every probability that is output uses
// exp_accurate, and the terms of a chunk's largest elements are replaced by
// accurate ones before the sum leaves the workgroup.
__device__ __forceinline__ float fast_term(float x, float m) {
    return __builtin_amdgcn_exp2f((x - m) * 1.44269504088896341f);
}

// Exact ranking of sh.cand[0..C): sh.rank[i] = number of larger composites.
// All NT threads call with the same C; ends with a barrier.
template <int NT> __device__ __forceinline__ void block_rank(RowsShared &sh, uint32_t C) {
    const uint32_t tid = threadIdx.x;
    if (C == 0) return;
    for (uint32_t t = tid; t < C; t += NT) sh.rank[t] = 0;
    __syncthreads();
    if (C <= NT) {
        const uint32_t parts = NT / C;                  // >= 1
        const uint32_t span = (C + parts - 1) / parts;  // entries per part
        const uint32_t part = tid / C, i = tid - part * C;
        if (part < parts) {
            const uint64_t mine = sh.cand[i];
            const uint32_t j0 = part * span, j1 = min(j0 + span, C);
            uint32_t cnt = 0;
            for (uint32_t j = j0; j < j1; j++) cnt += (sh.cand[j] > mine) ? 1u : 0u;
            if (cnt) atomicAdd(&sh.rank[i], cnt);
        }
    } else {
        for (uint32_t i = tid; i < C; i += NT) {
            const uint64_t mine = sh.cand[i];
            uint32_t cnt = 0;
            for (uint32_t j = 0; j < C; j++) cnt += (sh.cand[j] > mine) ? 1u : 0u;
            sh.rank[i] = cnt;
        }
    }
    __syncthreads();
}

// Threshold + gather.  Every thread holds E elements; key_at(e) is the order
// key of its e-th element (0 = no element), lane_max_key the largest of them.
// On return sh.cand[0..sh.count) holds the composite of every element whose key
// reaches the block threshold -- at least min(want, elements in the block) of
// them -- unless sh.count > kFastCap (too many; the list is truncated).
template <int NT, int E, typename KeyAt, typename IdxAt>
__device__ __forceinline__ void block_threshold_gather(RowsShared &sh, uint32_t lane_max_key, uint32_t want,
                                                       KeyAt key_at, IdxAt idx_at) {
    constexpr int NW = NT / kWave;
    const uint32_t tid = threadIdx.x, wave = tid / kWave, lane = tid & (kWave - 1);
    const uint32_t valid = static_cast<uint32_t>(__popcll(__ballot(lane_max_key != 0u)));
    if (lane == 0) sh.wave_valid[wave] = valid;
    if (tid == 0) sh.count = 0;
    __syncthreads();
    // smallest c such that taking min(c, valid lanes) lanes from every wave
    // reaches `want`; none (c = 0) means: take everything
    uint32_t c = 0;
    for (uint32_t t = (want + NW - 1) / NW; t <= kWave; t++) {
        uint32_t got = 0;
#pragma unroll
        for (int w = 0; w < NW; w++) got += min(t, sh.wave_valid[w]);
        if (got >= want) {
            c = t;
            break;
        }
    }
    const uint32_t cw = min(c, valid);
    const uint32_t tw = (c == 0) ? 0u : (cw == 0 ? 0xFFFFFFFFu : wave_cth_largest_floor(lane_max_key, cw, 24));
    if (lane == 0) sh.wave_key[wave] = tw;
    __syncthreads();
    uint32_t thr = sh.wave_key[0];
#pragma unroll
    for (int w = 1; w < NW; w++) thr = min(thr, sh.wave_key[w]);
    thr = max(thr, 1u);  // key 0 is "no element"
    if (lane_max_key >= thr) {
#pragma unroll
        for (int e = 0; e < E; e++) {
            const uint32_t key = key_at(e);
            if (key >= thr) {
                const uint32_t pos = atomicAdd(&sh.count, 1u);
                if (pos < kFastCap) sh.cand[pos] = composite(key, idx_at(e));
            }
        }
    }
    __syncthreads();
}

template <typename T> struct Vec128;
template <> struct Vec128<float> {
    static constexpr int N = 4;
    float4 v;
    __device__ __forceinline__ void load(const float *p) { v = *reinterpret_cast<const float4 *>(p); }
    __device__ __forceinline__ float get(int c) const { return c == 0 ? v.x : c == 1 ? v.y : c == 2 ? v.z : v.w; }
};
template <> struct Vec128<uint16_t> {
    static constexpr int N = 8;
    uint4 v;
    __device__ __forceinline__ void load(const uint16_t *p) { v = *reinterpret_cast<const uint4 *>(p); }
    __device__ __forceinline__ float get(int c) const {
        const uint32_t w = (c >> 1) == 0 ? v.x : (c >> 1) == 1 ? v.y : (c >> 1) == 2 ? v.z : v.w;
        return __half2float(__ushort_as_half(static_cast<uint16_t>((c & 1) ? (w >> 16) : (w & 0xFFFFu))));
    }
};

// ---- merge of one row's chunk results (all NT threads of a workgroup) --------
// EM = candidate slots each thread takes (EM * NT >= G * ws.kc).
template <typename T, int NT, int EM, bool SOFTMAX>
__device__ __forceinline__ void merge_row(RowsSharedUnion &smem, float *fscratch, double *dscratch, const T *rowp,
                                          T *ov, int32_t *oi, uint32_t n, uint32_t k, uint32_t G,
                                          const ChunkPartial *pp, const uint64_t *rc, uint32_t kc) {
    RowsShared &sh = smem.fast;
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t want = k + 1;
    const uint32_t kk = min(k, n);
    const uint32_t slots = G * kc;

    // candidates first: their loads do not depend on the row statistics
    uint64_t mc[EM];
    uint32_t lmk = 0;
#pragma unroll
    for (int e = 0; e < EM; e++) {
        const uint32_t t = static_cast<uint32_t>(e) * NT + tid;
        uint64_t c = 0;
        if (t < slots) {
            const uint32_t g = t / kc, j = t - g * kc;
            if (j < pp[g].count) c = rc[t];
        }
        mc[e] = c;
        lmk = max(lmk, static_cast<uint32_t>(c >> 32));
    }

    // row statistics: lane g of wave 0 takes chunk g (G <= 64), fixed reduction tree
    if (wave == 0) {
        float mg = -INFINITY;
        double sg = 0.0;
        uint32_t cnt = 0, flg = 0;
        if (lane < G) {
            mg = pp[lane].m;
            sg = pp[lane].s;
            cnt = pp[lane].count;
            flg = pp[lane].flags;
        }
        const float M = wave_max_f32_uniform(mg);
        double term = 0.0;
        if (SOFTMAX && sg != 0.0) term = sg * exp(static_cast<double>(mg) - static_cast<double>(M));
        const double S = wave_sum(term);
        const uint32_t tot = wave_sum(cnt);
        bool bad = __ballot(flg != 0u) != 0ull;
        if (SOFTMAX && !(S > 0.0 && S < 1e300)) bad = true;  // NaN / inf rows
        if (SOFTMAX && !(M > -INFINITY && M < INFINITY)) bad = true;
        if (slots > static_cast<uint32_t>(EM) * NT) bad = true;
        if (lane == 0) {
            sh.row_m = M;
            sh.row_rinv = 1.0 / S;
            sh.row_total = tot;
            sh.row_slow = bad ? 1u : 0u;
        }
    }
    __syncthreads();
    LineStats st{sh.row_m, 0.f, sh.row_rinv};
    bool slow = sh.row_slow != 0u;
    const uint32_t total = sh.row_total;

    if (!slow) {
        block_threshold_gather<NT, EM>(
            sh, lmk, min(want, total), [&](int e) -> uint32_t { return static_cast<uint32_t>(mc[e] >> 32); },
            [&](int e) -> uint32_t { return composite_index(mc[e]); });
        const uint32_t C2 = sh.count;
        if (C2 > kFastCap) {
            slow = true;
        } else {
            block_rank<NT>(sh, C2);
            for (uint32_t t = tid; t < C2; t += NT) {
                const uint32_t r = sh.rank[t];
                if (r <= kk && r <= static_cast<uint32_t>(kFastMaxK)) {
                    const uint32_t idx = composite_index(sh.cand[t]);
                    sh.pidx[r] = idx;
                    if constexpr (SOFTMAX) sh.prob[r] = round_to_storage<T>(softmax_prob(load_elem(rowp, idx), st));
                }
            }
            __syncthreads();
            if constexpr (SOFTMAX) {
                // Probabilities are non-increasing along the rank order, so equal
                // ones are neighbours.  A tie that reaches past the k-th place
                // cannot be settled from the candidates.
                if (C2 > kk && sh.prob[kk - 1] == sh.prob[kk]) slow = true;
            }
        }
    }

    if (!slow) {
        for (uint32_t r = tid; r < kk; r += NT) {
            const uint32_t idx = sh.pidx[r];
            if constexpr (SOFTMAX) {
                const float p = sh.prob[r];
                // final place inside a run of equal probabilities: by index
                uint32_t lo = r, hi = r, pos = r;
                while (lo > 0 && sh.prob[lo - 1] == p) lo--;
                while (hi + 1 < kk && sh.prob[hi + 1] == p) hi++;
                if (hi > lo) {
                    pos = lo;
                    for (uint32_t q = lo; q <= hi; q++) pos += (sh.pidx[q] < idx) ? 1u : 0u;
                }
                store_elem(ov, pos, p);
                oi[pos] = static_cast<int32_t>(idx);
            } else {
                ov[r] = rowp[idx];
                oi[r] = static_cast<int32_t>(idx);
            }
        }
        return;
    }

    // ---- exact path: radix select over the whole row ----------------------------
    __syncthreads();  // smem changes owner
    if constexpr (SOFTMAX) {
        // redo the statistics the way the general kernels define them
        st = line_stats<T, NT>(rowp, 0, n, 1, fscratch, dscratch);
        select_topk_line<NT>(smem.exact, n, kk, [&](uint32_t j) {
            return order_key(round_to_storage<T>(softmax_prob(load_elem(rowp, j), st)));
        });
        for (uint32_t r = tid; r < kk; r += NT) {
            const uint32_t idx = composite_index(smem.exact.sel[r]);
            store_elem(ov, r, softmax_prob(load_elem(rowp, idx), st));
            oi[r] = static_cast<int32_t>(idx);
        }
    } else {
        select_topk_line<NT>(smem.exact, n, kk, [&](uint32_t j) { return order_key(load_elem(rowp, j)); });
        for (uint32_t r = tid; r < kk; r += NT) {
            const uint32_t idx = composite_index(smem.exact.sel[r]);
            ov[r] = rowp[idx];
            oi[r] = static_cast<int32_t>(idx);
        }
    }
}

// SOFTMAX = true : fused softmax -> top-k (values are probabilities)
// SOFTMAX = false: plain top-k, largest first (values are copies of the input)
// ALIGNED: every row start is 16-byte aligned and n is a multiple of the vector
// width, so chunks are read with 128-bit loads.
// Launch: rows * G workgroups of NT threads; per = elements per chunk
// (a multiple of the vector width, per <= NT * V * vector width, G * per >= n).
// With G == 1 the workgroup also merges (no second kernel).
template <typename T, int NT, int V, bool SOFTMAX, bool ALIGNED>
__global__ __launch_bounds__(NT) void rows_chunk_kernel(const T *__restrict__ in, T *__restrict__ values,
                                                        int32_t *__restrict__ indices, uint32_t n, uint32_t k,
                                                        uint32_t G, uint32_t per, RowsWorkspace ws) {
    constexpr int VEC = Vec128<T>::N;
    constexpr int E = V * VEC;
    constexpr int NW = NT / kWave;
    __shared__ RowsSharedUnion smem;
    __shared__ float fscratch[NW];
    __shared__ double dscratch[NW];
    RowsShared &sh = smem.fast;

    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t row = blockIdx.x / G, chunk = blockIdx.x - row * G;
    const uint32_t c0 = min(chunk * per, n), c1 = min(c0 + per, n);
    const T *rowp = in + static_cast<size_t>(row) * n;
    const uint32_t want = k + 1;  // one extra: the merge needs the (k+1)-th to prove the cut

    // ---- 1. chunk -> registers ------------------------------------------------
    float x[E];
    if constexpr (ALIGNED) {
        Vec128<T> q[V];
#pragma unroll
        for (int i = 0; i < V; i++) {
            const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * NT + tid) * VEC;
            if (e0 < c1) q[i].load(rowp + e0);
        }
#pragma unroll
        for (int i = 0; i < V; i++) {
            const uint32_t e0 = c0 + (static_cast<uint32_t>(i) * NT + tid) * VEC;
#pragma unroll
            for (int c = 0; c < VEC; c++) x[i * VEC + c] = (e0 < c1) ? q[i].get(c) : -INFINITY;
        }
    } else {
#pragma unroll
        for (int i = 0; i < V; i++) {
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                const uint32_t e = c0 + (static_cast<uint32_t>(i) * NT + tid) * VEC + c;
                x[i * VEC + c] = (e < c1) ? load_elem(rowp, e) : -INFINITY;
            }
        }
    }
    auto index_of = [&](int e) -> uint32_t {
        return c0 + (static_cast<uint32_t>(e / VEC) * NT + tid) * VEC + static_cast<uint32_t>(e % VEC);
    };

    // ---- 2. max and sum of exp ------------------------------------------------
    float lmax = -INFINITY;
#pragma unroll
    for (int e = 0; e < E; e++) lmax = fmaxf(lmax, x[e]);
    float m_g = -INFINITY, ref = 0.f;
    if constexpr (SOFTMAX) {
        const float wm = wave_max_f32_uniform(lmax);
        if (lane == 0) sh.wave_m[wave] = wm;
        __syncthreads();
        m_g = sh.wave_m[0];
#pragma unroll
        for (int w = 1; w < NW; w++) m_g = fmaxf(m_g, sh.wave_m[w]);
        // a chunk without a finite element sums against 0: its terms are all 0
        // (or NaN, which must survive), never -inf - -inf
        ref = (m_g > -INFINITY) ? m_g : 0.f;
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int e = 0; e < E; e += 2) {
            a0 += fast_term(x[e], ref);
            a1 += fast_term(x[e + 1], ref);
        }
        const double wsum = wave_sum(static_cast<double>(a0) + static_cast<double>(a1));
        if (lane == 0) sh.wave_s[wave] = wsum;
    }

    // ---- 3. threshold and gather ------------------------------------------------
    const bool any_valid = (c0 + tid * VEC) < c1;
    uint32_t lkey = any_valid ? order_key(lmax) : 0u;
    if constexpr (!SOFTMAX) {
        // fmaxf drops NaN, but NaN ranks first in a plain top-k: take the max of
        // the keys instead (a softmax row with a NaN goes to the exact path anyway)
        lkey = 0u;
#pragma unroll
        for (int e = 0; e < E; e++) lkey = max(lkey, index_of(e) < c1 ? order_key(x[e]) : 0u);
    }
    block_threshold_gather<NT, E>(
        sh, lkey, want, [&](int e) -> uint32_t { return index_of(e) < c1 ? order_key(x[e]) : 0u; },
        [&](int e) -> uint32_t { return index_of(e); });
    const uint32_t C = sh.count;
    const bool overflow = C > kFastCap;

    // ---- 4. exact ranking of the gathered elements, emit the best `want` -------
    uint64_t *out_c = ws.cands + (static_cast<size_t>(row) * G + chunk) * ws.kc;
    uint32_t emitted = 0;
    if (!overflow) {
        block_rank<NT>(sh, C);
        emitted = min(C, want);
        for (uint32_t t = tid; t < C; t += NT) {
            const uint32_t r = sh.rank[t];
            if (r < emitted) {
                const uint64_t cmp = sh.cand[t];
                out_c[r] = cmp;
                if constexpr (SOFTMAX) {
                    // replace this element's fast term by the accurate one (the
                    // difference of two nearby floats is exact)
                    const float xv = ordered_to_float(static_cast<uint32_t>(cmp >> 32));
                    sh.prob[r] = exp_accurate(xv - ref) - fast_term(xv, ref);
                }
            }
        }
    }
    __syncthreads();
    if (wave == 0) {
        double acc = 0.0;
        if constexpr (SOFTMAX) {
            if (lane < NW) acc = sh.wave_s[lane];
            for (uint32_t r = lane; r < emitted; r += kWave) acc += static_cast<double>(sh.prob[r]);
            acc = wave_sum(acc);  // same tree every time: run-to-run stable
        }
        if (lane == 0) {
            ChunkPartial p;
            p.s = acc;
            p.m = m_g;
            p.count = emitted;
            p.flags = overflow ? 1u : 0u;
            p.pad[0] = p.pad[1] = p.pad[2] = 0;
            ws.partials[static_cast<size_t>(row) * G + chunk] = p;
        }
    }
    if (G != 1) return;

    // ---- single-chunk rows: merge right here --------------------------------------
    __syncthreads();  // this workgroup's own global writes, and sh is free again
    constexpr int EM1 = (kFastMaxK + 1 + NT - 1) / NT;
    merge_row<T, NT, EM1, SOFTMAX>(smem, fscratch, dscratch, rowp, values + static_cast<size_t>(row) * k,
                                   indices + static_cast<size_t>(row) * k, n, k, 1u, ws.partials + row,
                                   ws.cands + static_cast<size_t>(row) * ws.kc, ws.kc);
}

// One workgroup of kMergeThreads per row.
template <typename T, bool SOFTMAX>
__global__ __launch_bounds__(kMergeThreads) void rows_merge_kernel(const T *__restrict__ in, T *__restrict__ values,
                                                                   int32_t *__restrict__ indices, uint32_t n,
                                                                   uint32_t k, uint32_t G, RowsWorkspace ws) {
    __shared__ RowsSharedUnion smem;
    __shared__ float fscratch[kMergeThreads / kWave];
    __shared__ double dscratch[kMergeThreads / kWave];
    const uint32_t row = blockIdx.x;
    merge_row<T, kMergeThreads, kMergeSlots / kMergeThreads, SOFTMAX>(
        smem, fscratch, dscratch, in + static_cast<size_t>(row) * n, values + static_cast<size_t>(row) * k,
        indices + static_cast<size_t>(row) * k, n, k, G, ws.partials + static_cast<size_t>(row) * G,
        ws.cands + static_cast<size_t>(row) * G * ws.kc, ws.kc);
}

}  // namespace vkop
