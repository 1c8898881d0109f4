// Short last-axis rows and small k (a classifier head: [batch, 1000], k = 5): one
// wave per row, the row in its registers, nothing but cross-lane operations between
// the load and the store -- a latency path: what a call costs here is the launch and
// one chain of dependent instructions, so the chain is kept short.
//
//   1. V 128-bit loads per lane (the row striped over the lanes);
//   2. the row's maximum; (softmax) the sum of fast terms exp2((x - M) log2 e);
//   3. the (k+1)-th largest of the 64 lane maxima, by a ballot descent: at least k+1
//      elements reach it (a probability tie that runs off the end of the candidates:
//      again with 2 (k+1) + 2 lane maxima, and once more);
//   4. the elements that reach it -- the candidates, at most 64 -- one per lane;
//   5. (softmax) their accurate terms replace the fast ones in the sum; each gets its
//      probability, float(term / sum) rounded to the tensor's type;
//   6. every candidate counts the candidates that rank before it (larger probability,
//      or key for a plain top-k; then lower index) and stores itself at that place if
//      it is below k.
// More than 64 candidates or fewer than k+1 (equal values en masse at the k-th place,
// rows of mostly -inf): the elements above the tie value and the first elements equal to
// it, in index order, and a tie in probability across the k-th place filled from every
// element of the row that has that probability.  What is left -- a sum that is not a
// positive finite number, more than k distinct larger values crowded into few lanes --
// goes to the exact single-workgroup select over the row (select.hpp) in the same kernel.
// The plain top-k also runs smallest first: the same steps on order keys turned round.
#pragma once

#include "kernels_general.hpp"
#include "kernels_rows.hpp"
#include "kernels_softmax.hpp"
#include "select.hpp"

namespace vkop {

constexpr int kTinyMaxK = 32;  // (k + 1 candidates, one per lane, and room for a few more)

// SAMPLING (softmax variant): every element counts times `scale` (one single-precision multiplication where it is
// read), and counts, if not null, receives each row's nucleus cut for top_p (the stored values walked in order).
union TinyShared {
    uint64_t cand[kWave];
    SelectShared exact;
    __device__ TinyShared() {}
};

// One row by the 64 lanes of the workgroup's only wave (the body of both kernels below).
template <typename T, int V, bool SOFTMAX, bool ALIGNED, bool SAMPLING>
__device__ __forceinline__ void tiny_row(TinyShared &smem, float *fscratch, double *dscratch, const T *__restrict__ in,
                                         T *__restrict__ values, int32_t *__restrict__ indices, uint32_t n, uint32_t k,
                                         uint32_t smallest, float scale) {
    static_assert(!SAMPLING || SOFTMAX, "the scaled form belongs to the softmax variant");
    auto elem_of = [&](float x) __attribute__((always_inline)) {
        if constexpr (SAMPLING) x = scaled(x, scale);
        return x;
    };
    constexpr int VEC = Vec128<T>::N;
    constexpr int ELEMS = V * VEC;
    // smallest (plain top-k only): the k smallest, in increasing order.  Everything below works
    // on order keys, so the keys are turned round where they are made: the complement for a
    // number or an infinity (+inf takes -inf's key, the floor that never becomes a candidate),
    // 1 for a NaN -- still the largest value, hence last, below every other element's key; a
    // row whose k smallest reach into its NaNs ends in the exact select like any row the
    // candidates do not settle.
    auto key_of_value = [&](float x) -> uint32_t {
        const uint32_t kx = order_key(x);
        if constexpr (!SOFTMAX) {
            if (smallest) return (x != x) ? 1u : ~kx;
        }
        return kx;
    };
    const uint32_t lane = threadIdx.x;
    const uint32_t row = blockIdx.x;
    const T *rowp = in + static_cast<size_t>(row) * n;
    T *ov = values + static_cast<size_t>(row) * k;
    int32_t *oi = indices + static_cast<size_t>(row) * k;
    const uint32_t want = k + 1, kk = min(k, n);

    BPS(20);
    // ---- 1. the row: element c of vector i of this lane is element (i * 64 + lane) * VEC + c
    Vec128<T> q[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = (static_cast<uint32_t>(i) * kWave + lane) * VEC;
        q[i].v = make_uint4(0, 0, 0, 0);
        if constexpr (ALIGNED) {
            q[i].load(rowp + (e0 < n ? e0 : 0u));
        } else {
#pragma unroll
            for (int c = 0; c < VEC; c++) q[i].set(c, load_elem(rowp, e0 + c < n ? e0 + c : 0u));
        }
    }
    // ---- 2. keys, maximum, sum of fast terms
    uint32_t key[ELEMS];  // 0: not an element (past the row, or a NaN of the softmax variant)
    uint32_t lmk = 0;
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < V; i++) {
#pragma unroll
        for (int c = 0; c < VEC; c++) {
            const uint32_t e = (static_cast<uint32_t>(i) * kWave + lane) * VEC + static_cast<uint32_t>(c);
            const float x = elem_of(q[i].get(c));
            const bool live = e < n && !(SOFTMAX && x != x);
            key[i * VEC + c] = live ? key_of_value(x) : 0u;
            lmk = max(lmk, key[i * VEC + c]);
            if (e < n) m = fmaxf(m, x);  // (drops NaN)
        }
    }
    float M = 0.f, ref = 0.f;
    double s_fast = 0.0;
    bool bad = false;
    BPS(29);
    if constexpr (SOFTMAX) {
        M = wave_max_f32_uniform(m);
        ref = (M > -INFINITY && M < INFINITY) ? M : 0.f;
        double acc = 0.0;
#pragma unroll
        for (int i = 0; i < V; i++) {
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                const uint32_t e = (static_cast<uint32_t>(i) * kWave + lane) * VEC + static_cast<uint32_t>(c);
                if (e < n) acc += static_cast<double>(fast_term_reduced(elem_of(q[i].get(c)), ref));  // (a NaN element makes the sum NaN)
            }
        }
        s_fast = wave_sum_f64_uniform(acc);
        bad = !(s_fast > 0.0 && s_fast < static_cast<double>(INFINITY)) || !(M > -INFINITY && M < INFINITY);
        if (bad) {
            // a NaN or +inf element, or nothing above -inf: every probability of the row is
            // NaN, all of them tie, the lowest indices win
            for (uint32_t r = lane; r < kk; r += kWave) {
                store_elem(ov, r, __uint_as_float(0x7FC00000u));
                oi[r] = static_cast<int32_t>(r);
            }
            return;
        }
    }
    // How many of the C composites that the lanes 0 .. C-1 hold (0 in the other lanes) rank before
    // this lane's: the composites go through LDS, where every lane reads all of them -- one
    // address per load for the whole wave, eight loads in flight (lane-to-lane reads through
    // scalar registers took 36 ns a candidate).  All lanes call; the list in LDS is overwritten.
    auto rank_among = [&](uint64_t own, uint32_t C) -> uint32_t {
        __syncthreads();  // (one wave: whoever still reads the list is done)
        smem.cand[lane] = own;
        __syncthreads();
        uint32_t ahead = 0;
        for (uint32_t c0 = 0; c0 < C; c0 += 8) {
            uint64_t other[8];
#pragma unroll
            for (int j = 0; j < 8; j++) other[j] = smem.cand[c0 + static_cast<uint32_t>(j)];  // (C <= 64 entries; past C: 0, never ahead)
#pragma unroll
            for (int j = 0; j < 8; j++) ahead += (other[j] > own) ? 1u : 0u;
        }
        return ahead;
    };
    // Places g0 .. k-1 of the result go to the first elements, in index order, whose keys lie in
    // [lo_key, hi_key] -- a group of equal probability pc; all of the row is in this wave's registers.
    auto fill_group = [&](uint32_t g0, uint32_t lo_key, uint32_t hi_key, float pc) {
        const uint32_t places = kk - g0;
        uint32_t filled = 0;  // wave-uniform
#pragma unroll
        for (int i = 0; i < V; i++) {
            if (filled < places) {
                uint32_t mine_in = 0;
#pragma unroll
                for (int c = 0; c < VEC; c++) mine_in += (key[i * VEC + c] >= lo_key && key[i * VEC + c] <= hi_key) ? 1u : 0u;
                uint32_t incl = mine_in;
#pragma unroll
                for (int o = 1; o < kWave; o <<= 1) {
                    const uint32_t t = __shfl_up(incl, o, kWave);
                    if (lane >= static_cast<uint32_t>(o)) incl += t;
                }
                uint32_t pos = filled + incl - mine_in;
#pragma unroll
                for (int c = 0; c < VEC; c++) {
                    if (key[i * VEC + c] >= lo_key && key[i * VEC + c] <= hi_key) {
                        if (pos < places) {
                            store_elem(ov, g0 + pos, pc);
                            oi[g0 + pos] = static_cast<int32_t>((static_cast<uint32_t>(i) * kWave + lane) * VEC + static_cast<uint32_t>(c));
                        }
                        pos++;
                    }
                }
                filled += static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(incl), kWave - 1));
            }
        }
    };
    // Steps 3 to 6, at most three times: with k+1 lane maxima, then with twice and four
    // times as many when a probability tie runs off the end of the candidates.
    BPS(21);
    bool exact = bad;
    for (uint32_t lanes_wanted = want; !exact; lanes_wanted = 2u * lanes_wanted + 2u) {
        // ---- 3. the lanes_wanted-th largest lane maximum, to 16 bits (-inf never becomes a candidate)
        uint32_t thr = 0;
        for (int bit = 31; bit >= 16; bit--) {
            const uint32_t trial = thr | (1u << bit);
            if (static_cast<uint32_t>(__popcll(__ballot(lmk >= trial))) >= lanes_wanted) thr = trial;
        }
        thr = max(thr, kKeyNegInf + 1u);
        // ---- 4. the candidates, in LDS one after the other, then one per lane
        uint32_t C = 0;  // wave-uniform
#pragma unroll
        for (int i = 0; i < V; i++) {
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                const bool pass = key[i * VEC + c] >= thr;
                const uint64_t mask = __ballot(pass);
                if (mask != 0ull) {  // (wave-uniform)
                    const uint32_t at = C + lanes_below(mask);
                    const uint32_t e = (static_cast<uint32_t>(i) * kWave + lane) * VEC + static_cast<uint32_t>(c);
                    if (pass && at < static_cast<uint32_t>(kWave)) smem.cand[at] = composite(key[i * VEC + c], e);
                    C += static_cast<uint32_t>(__popcll(mask));
                }
            }
        }
        __syncthreads();  // (one wave: the list is written)
        if (C > static_cast<uint32_t>(kWave) || C < min(want, n)) break;
        const bool have = lane < C;
        uint64_t mine = have ? smem.cand[lane] : 0ull;
        const uint32_t xkey = static_cast<uint32_t>(mine >> 32);  // the candidate's logit
        __syncthreads();  // (the list may be written again)
        double rinv = 0.0;  // 1 / the corrected sum
        if constexpr (SOFTMAX) {
            // ---- 5. accurate terms for the candidates, the corrected sum, probabilities
            const float xv = ordered_to_float(static_cast<uint32_t>(mine >> 32));
            const float term = have ? softmax_term(xv, M) : 0.f;
            const double cr = have ? static_cast<double>(term) - static_cast<double>(fast_term_reduced(xv, ref)) : 0.0;
            const double total = s_fast + wave_sum_f64_uniform(cr);
            rinv = 1.0 / total;
            const float p = round_to_storage<T>(static_cast<float>(static_cast<double>(term) * rinv));
            mine = have ? ((static_cast<uint64_t>(order_key(p)) << 32) | (mine & 0xFFFFFFFFull)) : 0ull;
        }
        BPS(28);
        // ---- 6. ranks among the candidates
        const uint32_t mine_hi = static_cast<uint32_t>(mine >> 32);
        const uint32_t before = rank_among(mine, C);
        if constexpr (SOFTMAX) {
            // a probability shared by the k-th place and the last candidate may go on below the candidates
            if (C < n && C > kk) {
                const uint64_t at_cut = __ballot(have && before == kk - 1u), at_end = __ballot(have && before == C - 1u);
                const uint32_t p_cut = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(mine_hi), __builtin_ctzll(at_cut)));
                const uint32_t p_end = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(mine_hi), __builtin_ctzll(at_end)));
                if (p_cut == p_end) {
                    if (p_cut == order_key(0.f)) {
                        // A tie at probability 0: the underflowed tail of the row, which runs to the
                        // row's end -- the candidates of probability 0 and everything below the
                        // candidates.  Its places go to its first elements in index order.
                        const uint32_t g0 = static_cast<uint32_t>(__popcll(__ballot(have && mine_hi > p_cut)));
                        uint32_t hi_key = (have && mine_hi == p_cut) ? xkey : 0u;
#pragma unroll
                        for (int o = 32; o > 0; o >>= 1) hi_key = max(hi_key, static_cast<uint32_t>(__shfl_xor(static_cast<int>(hi_key), o, kWave)));
                        fill_group(g0, 1u, hi_key, 0.f);
                        if (have && before < g0) {
                            store_elem(ov, before, ordered_to_float(mine_hi));
                            oi[before] = static_cast<int32_t>(composite_index(mine));
                        }
                        return;
                    }
                    // The tie reaches the last candidate; whether it goes on below the candidates is a
                    // question about ONE element, the largest that is not a candidate (every element from thr up
                    // is one): with a probability below p_cut the group ends inside the candidates, and the
                    // ranking just made stands.  Equal half-precision logits at the cut -- a few rows in a
                    // hundred on a classifier's output -- are this case; going round again for them cost the
                    // whole call the slowest wave's second turn.
                    uint32_t below = 0;
#pragma unroll
                    for (int e = 0; e < ELEMS; e++) below = max(below, key[e] < thr ? key[e] : 0u);
                    below = wave_max_u32(below);
                    bool ends_inside = below == 0u;  // (the candidates are all there is)
                    if (!ends_inside) {
                        const float pb = round_to_storage<T>(static_cast<float>(static_cast<double>(softmax_term(ordered_to_float(below), M)) * rinv));
                        ends_inside = order_key(pb) < p_cut;
                    }
                    if (!ends_inside) {
                    if (lanes_wanted >= static_cast<uint32_t>(kWave)) break;
#ifdef VKOP_STAMPS
                    if (threadIdx.x == 0) atomicAdd(&g_bp_stamps[31], 1ull);
#endif
                    continue;  // more candidates
                    }
                }
            }
        }
        if (have && before < kk) {
            const uint32_t idx = composite_index(mine);
            if constexpr (SOFTMAX) store_elem(ov, before, ordered_to_float(mine_hi));
            else ov[before] = rowp[idx];  // bit copy (keeps the sign of a zero)
            oi[before] = static_cast<int32_t>(idx);
        }
        BPS(27);
        return;
    }
    // ---- equal values en masse at the k-th place, or a row of mostly -inf ---------------------------
    // The row's k+1 largest are then the elements above the tie value T -- the exact
    // (k+1)-th largest lane maximum; -inf when fewer than k+1 lanes hold anything -- and the
    // first elements equal to T in index order.  A probability that the k-th place shares
    // with the place behind it (equal values do, and different values can) is settled over
    // every element of the row that has it.
    BPS(22);
    if (!bad) {
        uint32_t tie = 0;
        for (int bit = 31; bit >= 0; bit--) {
            const uint32_t trial = tie | (1u << bit);
            if (static_cast<uint32_t>(__popcll(__ballot(lmk >= trial))) >= want) tie = trial;
        }
        tie = max(tie, kKeyNegInf);
        // the elements above T, as in step 4 (all threads call; returns their number)
        auto gather_above = [&](uint32_t t) __attribute__((always_inline)) -> uint32_t {
            uint32_t count = 0;  // wave-uniform
#pragma unroll
            for (int i = 0; i < V; i++) {
#pragma unroll
                for (int c = 0; c < VEC; c++) {
                    const bool pass = key[i * VEC + c] > t;
                    const uint64_t mask = __ballot(pass);
                    if (mask != 0ull) {
                        const uint32_t at = count + lanes_below(mask);
                        const uint32_t e = (static_cast<uint32_t>(i) * kWave + lane) * VEC + static_cast<uint32_t>(c);
                        if (pass && at < static_cast<uint32_t>(kWave)) smem.cand[at] = composite(key[i * VEC + c], e);
                        count += static_cast<uint32_t>(__popcll(mask));
                    }
                }
            }
            return count;
        };
        BPS(23);
        uint32_t above = gather_above(tie);
        BPS(24);
#ifdef VKOP_STAMPS
        if (threadIdx.x == 0 && blockIdx.x == 0) g_bp_stamps[29] = above;
#endif
        if (above >= want) {
            // More than k elements above the (k+1)-th largest LANE maximum: the top of the row
            // sits in few lanes (a sorted row: a lane's elements are neighbours).  The exact
            // (k+1)-th largest ELEMENT then, by a descent over all of them; fewer than k+1
            // elements lie above that.
            uint32_t t2 = 0;
            if (above <= static_cast<uint32_t>(kWave)) {
                // (up to 64 of them: each is in the list, a lane each, and the descent is over one key a lane)
                __syncthreads();  // (one wave: the list is written)
                const uint32_t own = lane < above ? static_cast<uint32_t>(smem.cand[lane] >> 32) : 0u;
                for (int bit = 31; bit >= 0; bit--) {
                    const uint32_t trial = t2 | (1u << bit);
                    if (static_cast<uint32_t>(__popcll(__ballot(own >= trial))) >= want) t2 = trial;
                }
            } else {
                for (int bit = 31; bit >= 0; bit--) {
                    const uint32_t trial = t2 | (1u << bit);
                    uint32_t c = 0;
#pragma unroll
                    for (int e = 0; e < ELEMS; e++) c += static_cast<uint32_t>(__popcll(__ballot(key[e] >= trial)));
                    if (c >= want) t2 = trial;
                }
            }
            tie = max(t2, kKeyNegInf);
            BPS(25);
            __syncthreads();  // (one wave: the list is written again)
            above = gather_above(tie);
            BPS(26);
        }
        if (above < want) {
            // the first want - above elements equal to T: vector by vector, lane by lane, element by element
            const uint32_t need = want - above;
            uint32_t taken = 0;  // wave-uniform
#pragma unroll
            for (int i = 0; i < V; i++) {
                if (taken < need) {
                    uint32_t mine_eq = 0;
#pragma unroll
                    for (int c = 0; c < VEC; c++) mine_eq += (key[i * VEC + c] == tie) ? 1u : 0u;
                    uint32_t incl = mine_eq;  // over the lanes up to this one
#pragma unroll
                    for (int o = 1; o < kWave; o <<= 1) {
                        const uint32_t t = __shfl_up(incl, o, kWave);
                        if (lane >= static_cast<uint32_t>(o)) incl += t;
                    }
                    uint32_t pos = taken + incl - mine_eq;
#pragma unroll
                    for (int c = 0; c < VEC; c++) {
                        if (key[i * VEC + c] == tie) {
                            const uint32_t e = (static_cast<uint32_t>(i) * kWave + lane) * VEC + static_cast<uint32_t>(c);
                            if (pos < need) smem.cand[above + pos] = composite(tie, e);
                            pos++;
                        }
                    }
                    taken += static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(incl), kWave - 1));
                }
            }
            __syncthreads();
            // (a row shorter than k+1 has them all)
            const uint32_t C = above + min(taken, need);
            if (C >= min(want, n)) {
                const bool have = lane < C;
                uint64_t mine = have ? smem.cand[lane] : 0ull;
                const uint32_t xkey = static_cast<uint32_t>(mine >> 32);
                double rinv = 0.0;
                auto prob_of_key = [&](uint32_t kx) {
                    return round_to_storage<T>(static_cast<float>(static_cast<double>(softmax_term(ordered_to_float(kx), M)) * rinv));
                };
                if constexpr (SOFTMAX) {
                    const float xv = ordered_to_float(xkey);
                    const float term = have ? softmax_term(xv, M) : 0.f;
                    const double cr = have ? static_cast<double>(term) - static_cast<double>(fast_term_reduced(xv, ref)) : 0.0;
                    rinv = 1.0 / (s_fast + wave_sum_f64_uniform(cr));
                    const float p = round_to_storage<T>(static_cast<float>(static_cast<double>(term) * rinv));
                    mine = have ? ((static_cast<uint64_t>(order_key(p)) << 32) | (mine & 0xFFFFFFFFull)) : 0ull;
                }
                const uint32_t mine_hi = static_cast<uint32_t>(mine >> 32);
                const uint32_t before = rank_among(mine, C);
                uint32_t g0 = kk;  // ranks from here on are filled as one group of equal probability
                if constexpr (SOFTMAX) {
                    if (C > kk) {
                        const uint64_t at_cut = __ballot(have && before == kk - 1u), at_next = __ballot(have && before == kk);
                        const uint32_t p_cut = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(mine_hi), __builtin_ctzll(at_cut)));
                        const uint32_t p_next = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(mine_hi), __builtin_ctzll(at_next)));
                        if (p_cut == p_next) {
                            // The probability at the k-th place goes on behind it.  It belongs to an
                            // interval of values [lo, hi]: hi is the largest candidate that has it
                            // (everything above the tie value is a candidate), lo is searched for; the
                            // places from the group's first rank on go to the interval's first
                            // elements in index order -- all of them are in this wave's registers.
                            const float pc = ordered_to_float(p_cut);
                            g0 = static_cast<uint32_t>(__popcll(__ballot(have && mine_hi > p_cut)));
                            uint32_t hi_key = (have && mine_hi == p_cut) ? xkey : 0u;
#pragma unroll
                            for (int o = 32; o > 0; o >>= 1) hi_key = max(hi_key, static_cast<uint32_t>(__shfl_xor(static_cast<int>(hi_key), o, kWave)));
                            const uint32_t lo_key = pc > 0.f ? lowest_key_of_probability(hi_key, pc, prob_of_key) : 1u;
                            fill_group(g0, lo_key, hi_key, pc);
                        }
                    }
                }
                if (have && before < min(kk, g0)) {
                    const uint32_t idx = composite_index(mine);
                    if constexpr (SOFTMAX) store_elem(ov, before, ordered_to_float(mine_hi));
                    else ov[before] = rowp[idx];  // bit copy (keeps the sign of a zero)
                    oi[before] = static_cast<int32_t>(idx);
                }
                return;
            }
        }
    }
    // ---- the exact select over the whole row -----------------------------------------------
#ifdef VKOP_STAMPS
    if (threadIdx.x == 0) atomicAdd(&g_bp_stamps[30], 1ull);
#endif
    BPS(26);
    __syncthreads();  // LDS changes owner
    SelectShared &ex = smem.exact;
    if constexpr (SOFTMAX) {
        const LineStats st = line_stats<T, kWave>(rowp, 0, n, 1, fscratch, dscratch, SAMPLING ? scale : 1.f);
        select_topk_line<kWave>(ex, n, kk, [&](uint32_t j) {
            return order_key(round_to_storage<T>(softmax_prob(elem_of(load_elem(rowp, j)), st)));
        });
        for (uint32_t r = lane; r < kk; r += kWave) {
            const uint32_t idx = composite_index(ex.sel[r]);
            store_elem(ov, r, softmax_prob(elem_of(load_elem(rowp, idx)), st));
            oi[r] = static_cast<int32_t>(idx);
        }
    } else {
        select_topk_line<kWave>(ex, n, kk, [&](uint32_t j) { return key_of_value(load_elem(rowp, j)); });
        for (uint32_t r = lane; r < kk; r += kWave) {
            const uint32_t idx = composite_index(ex.sel[r]);
            ov[r] = rowp[idx];
            oi[r] = static_cast<int32_t>(idx);
        }
    }
}

// Launch: one workgroup of 64 threads per row.
template <typename T, int V, bool SOFTMAX, bool ALIGNED>
__global__ __launch_bounds__(kWave) void rows_tiny_kernel(const T *__restrict__ in, T *__restrict__ values,
                                                          int32_t *__restrict__ indices, uint32_t n, uint32_t k,
                                                          uint32_t smallest = 0) {
    __shared__ TinyShared smem;
    __shared__ float fscratch[1];
    __shared__ double dscratch[1];
    tiny_row<T, V, SOFTMAX, ALIGNED, false>(smem, fscratch, dscratch, in, values, indices, n, k, smallest, 1.f);
}

// The softmax variant with every element times `scale`, and, if counts is not null, each row's nucleus cut for top_p.
template <typename T, int V, bool ALIGNED>
__global__ __launch_bounds__(kWave) void rows_tiny_sampling_kernel(const T *__restrict__ in, T *__restrict__ values,
                                                                   int32_t *__restrict__ indices, uint32_t n, uint32_t k,
                                                                   float scale, int32_t *__restrict__ counts, float top_p) {
    __shared__ TinyShared smem;
    __shared__ float fscratch[1];
    __shared__ double dscratch[1];
    tiny_row<T, V, true, ALIGNED, true>(smem, fscratch, dscratch, in, values, indices, n, k, 0u, scale);
    if (counts != nullptr) {
        // the nucleus cut of what was just stored (whichever way the row went): the wave reads its own result
        // back -- the barrier makes the workgroup's stores visible to it -- and walks it in order
        __syncthreads();
        const uint32_t kk = min(k, n);
        const T *ov = values + static_cast<size_t>(blockIdx.x) * k;
        const uint32_t count = nucleus_count_wave(kk, top_p, [&](uint32_t r) { return load_elem(ov, r); });
        if (threadIdx.x == 0) counts[blockIdx.x] = static_cast<int32_t>(count);
    }
}

}  // namespace vkop
