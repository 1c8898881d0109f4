// Long contiguous rows, k beyond what one workgroup's candidate list holds
// (kFastMaxK < k <= kMaxK), largest first: the two kernels that follow
// rows_scan_kernel there.  Few rows are long enough for this (a row needs a few
// thousand 256-byte blocks), so each row's work is spread over many workgroups:
//
//   bigpick_gather_kernel   rows * G2 workgroups.  Every workgroup finds, from the
//                           row's block maxima, a value that at least k+1 of them
//                           reach (a 2048-bin LDS histogram of every fourth key over
//                           the range the keys span, then a count over all of them;
//                           after coarse bins a second round inside one bin),
//                           lowers it by a margin
//                           that keeps probability ties above it (softmax variant),
//                           reads again those of ITS share of the blocks that reach
//                           it and appends their elements to the row's candidate
//                           lists in global memory: everything above the value, and
//                           up to a quota of what lies at or just below it -- for the
//                           softmax variant with the element's accurate term
//                           exp(x - M), whose difference to the fast term the scan
//                           added goes into the row's correction (an integer sum, so
//                           that the order of arrival does not show in it);
//   bigpick_rank_kernel     rows * 256 workgroups, 32 candidates each.  Every
//                           workgroup takes the whole list into registers, a quarter
//                           per wave (softmax: as probabilities, term / corrected
//                           sum), counts for each of its own 32 how many of the list
//                           rank before it -- larger key first, then lower index; one
//                           vector compare and a population count per 64 pairs --
//                           and stores those that rank below k at their place.
//
// Rows whose cut falls into a crowd -- one value in thousands of places, rows of mostly
// -inf, probabilities that underflow to 0 and tie -- exceed the quota: the lists then
// hold everything that ranks ABOVE the threshold's own rank group, and the row's last
// rank workgroup takes that group's first members from a walk over the row in index
// order (first_members_by_vectors).  Rows of NaN probabilities are written directly.
// What is left -- more elements above the threshold than the lists hold, a group too
// small to fill the places -- goes to the first workgroup of the row, which runs the
// exact single-workgroup select over the whole row (select.hpp); every workgroup of the
// row reaches the same verdict from the same numbers.
#pragma once

#include "kernels_stream.hpp"

namespace vkop {

// In-kernel time stamps of the first workgroup's phases, for tuning: compiled in only
// with -DVKOP_STAMPS=<name of the C function that reads them out> (rows_inst.hip).

constexpr int kBigPickThreads = 256;
constexpr int kBigPickWaves = kBigPickThreads / kWave;
constexpr int kBigPickCap = 8192;       // candidates of a row that are ranked (block-clustered rows have about 2 (k+1))
constexpr int kBigPickLists = 8;        // lists a row's candidates are appended to (gather workgroup p uses list p % 8:
                                        // eight counters instead of one that every workgroup of the row queues for)
constexpr int kBigPickListCap = 2048;   // entries per list
constexpr int kBigPickLocalCap = 4096;  // candidates one gather workgroup can hold (a sorted row's are all in one or two shares)
constexpr int kBigPickSpread = 512;     // a gather workgroup with more candidates than this deals them over all the lists
constexpr int kBigPickZoneQuota = 32;   // elements at or below the threshold (down to the margin) one gather workgroup
                                        // passes on at most (fewer for a large k: bigpick_zone_quota); with more the
                                        // threshold's own rank group comes from a walk over the row (below)
constexpr int kBigPickMine = 32;        // candidates one rank workgroup places
constexpr int kBigPickRecsMax = 1024;   // wave records of a row (chunks * kScanWaves)
constexpr int kBigPickHeadWords = 16 * kBigPickLists + 16;  // per row: 16 words per list, then 16 for the row
constexpr double kBigPickFixUnit = 1152921504606846976.0;  // 2^60: corrections are added in units of 2^-60

struct BigPickWorkspace {
    uint64_t *cand;  // [rows][kBigPickLists][kBigPickListCap] composites (order key of the element, index)
    float *term;     // same shape, softmax variant: exp(x - M) of the same elements
    uint32_t *head;  // [rows][kBigPickHeadWords].  List j of a row: word 16 j = entries appended (more than the
                     // capacity = incomplete), words 16 j + 2, 3 = its part of the row's correction (64-bit integer);
                     // word 128 = the threshold the gather kernel found, before the margin; word 129 != 0: some
                     // workgroup left out its elements at or below the threshold (more than its quota).  All
                     // zero when the gather kernel starts (the scan kernel clears them).
    double *stat;    // [rows][2] softmax variant: the row's sum of fast terms, scaled to its maximum; that maximum
};

// The margin below the threshold, in the elements' own unit: two elements further
// apart than HALF of this have probabilities whose storage values differ (single
// precision: exp(5e-6) is 40 ulp above 1, and the float subtraction x - M in front of
// it moves an argument by at most 2^-20 for |x - M| < 16; half precision: exp(2e-3) is
// 4 ulp above 1).  Twice the needed distance, so that the rounding of thr - margin
// (at most half an ulp of thr, and then adjacent floats are further apart than the
// margin anyway) cannot eat it.
template <typename T> __device__ __forceinline__ float bigpick_margin() { return sizeof(T) == 2 ? 4e-3f : 1e-5f; }

// What one of a row's G2 gather workgroups passes on of elements at or below the
// threshold: so that these and 1.5 (k+1) elements above it (the usual excess is 1.2 to
// 1.5) stay within what the rank kernel holds.
__device__ __forceinline__ uint32_t bigpick_zone_quota(uint32_t want, uint32_t G2) {
    const uint32_t room = static_cast<uint32_t>(kBigPickCap) > want + want / 2u ? static_cast<uint32_t>(kBigPickCap) - want - want / 2u : 0u;
    return min(static_cast<uint32_t>(kBigPickZoneQuota), max(4u, room / G2));
}

// thr: key of a finite number or +inf (never below kKeyNegInf + 1)
template <typename T, bool SOFTMAX> __device__ __forceinline__ uint32_t bigpick_lowered(uint32_t thr) {
    if constexpr (!SOFTMAX) return thr;
    const float t = ordered_to_float(thr) - bigpick_margin<T>();
    return (t > -INFINITY) ? max(order_key(t), kKeyNegInf + 1u) : kKeyNegInf + 1u;
}

// hist[d] += 1 for every lane with `on` (hist_add_grouped: lanes that share a digit add once).
__device__ __forceinline__ void bigpick_hist_add(uint32_t *hist, bool on, uint32_t d) {
    if (on) hist_add_grouped(hist, d);
}

// The digit d of hist[0..2048) with #(digits above d) < need <= #(digits >= d); all
// 256 threads call, all can read answer[0] afterwards (ends with a barrier).  need
// must not exceed the histogram's total.  wtot: kBigPickWaves words of scratch.
__device__ __forceinline__ void bigpick_resolve(const uint32_t *hist, uint32_t need, uint32_t *answer, uint32_t *wtot) {
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    // thread t owns bins 8 t .. 8 t + 7
    const uint4 *hp = reinterpret_cast<const uint4 *>(hist + tid * 8u);
    const uint4 lo4 = hp[0], hi4 = hp[1];
    const uint32_t h[8] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
    const uint32_t s = ((h[0] + h[1]) + (h[2] + h[3])) + ((h[4] + h[5]) + (h[6] + h[7]));
    uint32_t incl = s;  // sum over the wave's lanes >= this one
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const uint32_t t = __shfl_down(incl, o, kWave);
        if (lane + static_cast<uint32_t>(o) < static_cast<uint32_t>(kWave)) incl += t;
    }
    if (lane == 0) wtot[wave] = incl;
    __syncthreads();
    uint32_t above = incl - s;
#pragma unroll
    for (int w = 1; w < kBigPickWaves; w++) above += (static_cast<uint32_t>(w) > wave) ? wtot[w] : 0u;
    if (above < need && need <= above + s) {
#pragma unroll
        for (int j = 7; j >= 0; j--) {
            if (above < need && need <= above + h[j]) answer[0] = tid * 8u + static_cast<uint32_t>(j);
            above += h[j];
        }
    }
    __syncthreads();
}

// Workgroup-wide sum of a wave-uniform count (every wave passes its own); ends with a
// barrier.  slots: kBigPickWaves words that nothing else uses until the next call.
__device__ __forceinline__ uint32_t bigpick_count_sum(uint32_t wave_count, uint32_t *slots) {
    const uint32_t tid = threadIdx.x;
    if ((tid & (kWave - 1)) == 0) slots[tid / kWave] = wave_count;
    __syncthreads();
    uint32_t total = 0;
#pragma unroll
    for (int w = 0; w < kBigPickWaves; w++) total += slots[w];
    return total;
}

// GE: block keys a thread takes in (a multiple of 4; GE * 256 >= blocks per row).  G2
// workgroups a row; workgroup `part` reads again blocks part * share .. (part + 1) *
// share - 1, share = ceil(blocks / G2) <= 256.  G, per: chunks per row and elements
// per chunk of the scan kernel (which wave summed which element).
template <typename T, bool SOFTMAX, bool ALIGNED, int GE>
__global__ __launch_bounds__(kBigPickThreads) void bigpick_gather_kernel(const T *__restrict__ in, uint32_t n, uint32_t k,
                                                                          uint32_t G2, uint32_t G, uint32_t per,
                                                                          ScanWorkspace ws, BigPickWorkspace bw) {
    constexpr int NT = kBigPickThreads, NW = kBigPickWaves;
    constexpr int VEC = Vec128<T>::N;
    constexpr int U = 4;  // loads per thread in flight while blocks are read again
    constexpr uint32_t BE = kBlockLanes * VEC;
    static_assert(GE % 4 == 0, "every fourth key is sampled");
    __shared__ __align__(16) uint32_t hist[2048];
    __shared__ uint32_t answer[1];
    __shared__ uint32_t hits[NT];
    __shared__ uint32_t wred[NW][3];
    __shared__ uint32_t wave_hits[NW];
    __shared__ uint32_t wtot[NW];
    __shared__ uint32_t cslots[2][NW];
    __shared__ uint32_t lcount, zcount, lbase[kBigPickLists];
    __shared__ uint64_t lcand[kBigPickLocalCap];
    __shared__ uint64_t zcand[kBigPickZoneQuota];
    __shared__ float lterm[SOFTMAX ? kBigPickLocalCap : 1];
    __shared__ float fscratch[NW];
    __shared__ double dscratch[NW];
    __shared__ long long iscratch[NW];
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t row = blockIdx.x / G2, part = blockIdx.x - row * G2;
    const T *rowp = in + static_cast<size_t>(row) * n;
    const uint32_t blocks = ws.blocks;
    const uint32_t *bmax = ws.bmax + static_cast<size_t>(row) * blocks;
    const uint32_t want = k + 1;
    const uint32_t waves = G * kScanWaves;
    const uint64_t *recs = ws.recs + 2 * static_cast<size_t>(row) * waves;
    uint32_t *head = bw.head + static_cast<size_t>(row) * kBigPickHeadWords;
    BPS(0);
    // ---- everything read first, in one round trip -------------------------------------
    uint32_t gk[GE];
#pragma unroll
    for (int e = 0; e < GE; e++) {
        const uint32_t b = static_cast<uint32_t>(e) * NT + tid;
        gk[e] = bmax[b < blocks ? b : 0u];
    }
    const uint32_t *bmin = ws.bmin + static_cast<size_t>(row) * blocks;
    uint32_t gn[GE];  // the same blocks' minima
#pragma unroll
    for (int e = 0; e < GE; e++) {
        const uint32_t b = static_cast<uint32_t>(e) * NT + tid;
        gn[e] = bmin[b < blocks ? b : 0u];
    }
    const uint32_t share = (blocks + G2 - 1) / G2;
    const uint32_t myb = part * share + tid;  // this thread's block of the workgroup's share
    const bool mine_live = tid < share && myb < blocks;
    const uint32_t mykey = bmax[mine_live ? myb : 0u];
    float M = 0.f;
    if constexpr (SOFTMAX) {
        float m = -INFINITY;
        for (uint32_t w = tid; w < waves; w += NT) m = fmaxf(m, __uint_as_float(static_cast<uint32_t>(recs[2 * w + 1] >> 32)));
        M = block_max_fast<NT>(m, fscratch);
    }

    // ---- a value that at least k+1 block maxima reach ---------------------------------------
    // The keys above that of -inf (a block of nothing else never counts), their range,
    // their number: one reduction.
    uint32_t kmax = 0, kmin = 0xFFFFFFFFu, nlive = 0;
#pragma unroll
    for (int e = 0; e < GE; e++) {
        const bool live = static_cast<uint32_t>(e) * NT + tid < blocks && gk[e] > kKeyNegInf;
        if (!live) gk[e] = 0;  // (0: not a key)
        if (!live) gn[e] = 0;
        kmax = max(kmax, gk[e]);
        kmin = live ? min(kmin, gk[e]) : kmin;
        nlive += static_cast<uint32_t>(__popcll(__ballot(live)));  // wave-uniform
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        kmax = max(kmax, static_cast<uint32_t>(__shfl_xor(static_cast<int>(kmax), o, kWave)));
        kmin = min(kmin, static_cast<uint32_t>(__shfl_xor(static_cast<int>(kmin), o, kWave)));
    }
    if (lane == 0) {
        wred[wave][0] = kmax;
        wred[wave][1] = kmin;
        wred[wave][2] = nlive;
    }
    if (tid == 0) {
        lcount = 0;
        zcount = 0;
    }
    __syncthreads();
    kmax = wred[0][0];
    kmin = wred[0][1];
    nlive = wred[0][2];
#pragma unroll
    for (int w = 1; w < NW; w++) {
        kmax = max(kmax, wred[w][0]);
        kmin = min(kmin, wred[w][1]);
        nlive += wred[w][2];
    }
    BPS(1);
    // how many of all the keys reach t (every thread gets the answer; a barrier inside)
    uint32_t flip = 0;
    auto reach = [&](uint32_t t) __attribute__((always_inline)) -> uint32_t {
        uint32_t c = 0;
#pragma unroll
        for (int e = 0; e < GE; e++) c += static_cast<uint32_t>(__popcll(__ballot(gk[e] >= t)));
        flip ^= 1u;
        return bigpick_count_sum(c, cslots[flip]);
    };
    uint32_t thr;
    if (nlive < want) {
        // fewer than k+1 blocks hold anything above -inf: every element above -inf is a
        // candidate, and the -inf elements (the threshold's own) follow in index order
        thr = kKeyNegInf;
    } else if (kmax == kmin) {
        thr = kmin;
    } else {
        // Every fourth key (block b = 256 e + t with e = t mod 4: one of every four
        // neighbouring blocks) goes into 2048 bins over [floor, kmax]; the bin that holds the
        // sample's (k+1)/4-th largest, and a few more for the sampling error, gives a value,
        // and the count over ALL keys says whether k+1 reach it -- if not, lower bins are
        // tried (1, 2, 4 .. further down; the floor itself is reached by enough).  A value
        // that clearly more than k+1 reach (coarse bins: keys of both signs, an outlier, a NaN
        // stretch the range) is followed by a second round over one bin alone, with all of
        // its keys and the exact number still wanted there.
        const uint32_t quarter = (want + 3u) / 4u;
        const uint32_t need_s = quarter + 2u * static_cast<uint32_t>(sqrtf(static_cast<float>(quarter))) + 8u;
        uint32_t floor_key = kmin, ceil_key = kmax, need_all = want;
        bool all_keys = false;  // the second round after coarse bins: every key of one bin, the exact number wanted there
        thr = kmin;
        for (int round = 0; round < 2; round++) {  // (every condition below is the same for every thread)
            const uint32_t range = ceil_key - floor_key;
            const uint32_t s = range < 2048u ? 0u : (32u - static_cast<uint32_t>(__clz(range))) - 11u;
            __syncthreads();
            reinterpret_cast<uint4 *>(hist)[2 * tid] = make_uint4(0, 0, 0, 0);
            reinterpret_cast<uint4 *>(hist)[2 * tid + 1] = make_uint4(0, 0, 0, 0);
            __syncthreads();
            uint32_t ns = 0;  // keys that went in (wave-uniform)
            if (!all_keys) {
#pragma unroll
                for (int i = 0; i < GE / 4; i++) {
                    const uint32_t sel = tid & 3u;
                    const uint32_t key = sel == 0u ? gk[4 * i] : sel == 1u ? gk[4 * i + 1] : sel == 2u ? gk[4 * i + 2] : gk[4 * i + 3];
                    const bool on = key != 0u && key >= floor_key;
                    ns += static_cast<uint32_t>(__popcll(__ballot(on)));
                    bigpick_hist_add(hist, on, (key - floor_key) >> s);
                }
            } else {
#pragma unroll
                for (int e = 0; e < GE; e++) {
                    const bool on = gk[e] >= floor_key && gk[e] <= ceil_key;  // (floor_key > 0: never "not a key")
                    ns += static_cast<uint32_t>(__popcll(__ballot(on)));
                    bigpick_hist_add(hist, on, (gk[e] - floor_key) >> s);
                }
            }
            const uint32_t went_in = bigpick_count_sum(ns, cslots[0]);  // (barrier: the histogram is complete)
            const uint32_t need = all_keys ? need_all : need_s;
            uint32_t d = 0;
            if (went_in >= need) {
                bigpick_resolve(hist, need, answer, wtot);
                d = answer[0];
            }
            uint32_t cand_thr = floor_key + (d << s), got = 0;
            for (uint32_t step = 1;; step <<= 1) {
                got = d == 0u ? 0xFFFFFFFFu : reach(cand_thr);  // (bin 0 starts at the floor)
                if (got >= want) break;
                d = d > step ? d - step : 0u;
                cand_thr = floor_key + (d << s);
            }
            thr = cand_thr;
            // (bins of 2^16 keys and more are coarse -- 1 % of a float's value; finer ones
            // are rarely worth a second round: tied keys stay tied)
            const uint32_t tight = s >= 16u ? want + want / 8u + 32u : 2u * want + 64u;
            if (round == 1 || s == 0u || got <= tight) break;
            // The bin [cand_thr, cand_thr + 2^s) alone -- or a bin further up: the sample's
            // allowance makes the choice err downwards, and where k+1 keys still reach a
            // higher bin's lower end, that is the better value.  The highest such bin: the
            // next one first (the usual answer: not that one either), then in doubling
            // steps and by bisection (keys of few distinct values leave most bins empty).
            const uint32_t nbins = (range >> s) + 1u;
            uint32_t dlo = d, dhi = nbins, above = 0;  // reach(bin dlo) >= k+1 > reach(bin dhi) = above (bin nbins: nothing)
            // (fine bins: one bin too low is harmless, the second round starts from here)
            for (uint32_t step = 1; s >= 16u && dlo + step < nbins; step <<= 1) {
                const uint32_t c = reach(floor_key + ((dlo + step) << s));
                if (c < want) {
                    dhi = dlo + step;
                    above = c;
                    break;
                }
                dlo += step;
                got = c;
            }
            while (s >= 16u && dhi - dlo > 1u) {
                const uint32_t mid = dlo + (dhi - dlo) / 2u;
                const uint32_t c = reach(floor_key + (mid << s));
                if (c < want) {
                    dhi = mid;
                    above = c;
                } else {
                    dlo = mid;
                    got = c;
                }
            }
            cand_thr = floor_key + (dlo << s);
            thr = cand_thr;
            if (got <= tight) break;
            const uint32_t c1 = dhi < nbins ? floor_key + (dhi << s) - 1u : ceil_key;
            floor_key = cand_thr;
            ceil_key = c1;
            need_all = want - above;
            all_keys = s >= 16u;
        }
    }
    // (thr == kKeyNegInf: the -inf elements are the threshold's own)
    uint32_t lo = thr > kKeyNegInf ? bigpick_lowered<T, SOFTMAX>(thr) : thr;
    // ---- clustered rows -------------------------------------------------------------------------
    // Blocks whose MINIMUM reaches thr hold 16 * VEC elements that do.  When the blocks that
    // reach lo are known to hold more candidates than a row's lists (a sorted row: k+1 blocks
    // reach thr and all but one are such blocks; a row of one value: every block is), two
    // facts about the block minima make the candidates few again without a look at the
    // elements:
    //  * a block whose minimum reaches a value holds 16 * VEC elements that do, a block whose
    //    maximum does holds one: the largest value for which these known elements come to k+1 is
    //    a threshold as valid as thr and, on such rows, far higher;
    //  * in index order, let B be the first block at which the count "all of a block whose
    //    minimum reaches thr, one of a block whose maximum does" comes to k+1: k+1 elements
    //    at or above thr lie in blocks up to B, so an element at or below thr in a later
    //    block has k+1 elements in front of it that rank no lower and come first -- it is
    //    not part of the result, nor of any tie that decides it, and is left out.
    uint32_t last_block_for_equals = 0xFFFFFFFFu;
    {
        uint32_t c2 = 0;  // (wave-uniform) blocks whose minimum reaches thr, high half; blocks whose maximum reaches lo, low half
#pragma unroll
        for (int e = 0; e < GE; e++)
            c2 += (static_cast<uint32_t>(__popcll(__ballot(gn[e] >= thr && gk[e] != 0u))) << 16) +
                  static_cast<uint32_t>(__popcll(__ballot(gk[e] >= lo)));
        flip ^= 1u;
        const uint32_t both = bigpick_count_sum(c2, cslots[flip]);
        const uint32_t nfull = both >> 16, nhit = both & 0xFFFFu;
        if (nfull * BE + (nhit - nfull) > static_cast<uint32_t>(kBigPickCap)) {  // (the same for every thread of every workgroup of the row)
            // the largest value (its low ten bits aside) that k+1 elements are KNOWN to reach
            uint32_t tmin = 0;
            for (int bit = 31; bit >= 10; bit--) {
                const uint32_t trial = tmin | (1u << bit);
                uint32_t c = 0;
#pragma unroll
                for (int e = 0; e < GE; e++)
                    c += (static_cast<uint32_t>(__popcll(__ballot(gn[e] >= trial && gk[e] != 0u))) << 16) +
                         static_cast<uint32_t>(__popcll(__ballot(gk[e] >= trial)));
                flip ^= 1u;
                const uint32_t packed = bigpick_count_sum(c, cslots[flip]);
                const uint32_t full = packed >> 16, reached = packed & 0xFFFFu;
                if (full * BE + (reached - full) >= want) tmin = trial;
            }
            if (tmin > thr) {
                thr = tmin;
                lo = thr > kKeyNegInf ? bigpick_lowered<T, SOFTMAX>(thr) : thr;
            }
            // per block, in index order, how many elements at or above thr it is KNOWN to hold
            uint16_t *known = reinterpret_cast<uint16_t *>(lcand);  // (8192 entries; the list is not in use yet)
            __syncthreads();
#pragma unroll
            for (int e = 0; e < GE; e++) {
                const uint32_t b = static_cast<uint32_t>(e) * NT + tid;
                if (b < 8192u) known[b] = static_cast<uint16_t>(gk[e] == 0u ? 0u : gn[e] >= thr ? BE : gk[e] >= thr ? 1u : 0u);
            }
            for (uint32_t b = static_cast<uint32_t>(GE) * NT + tid; b < 8192u; b += NT) known[b] = 0;
            if (tid == 0) answer[0] = 0xFFFFFFFFu;
            __syncthreads();
            if (tid < static_cast<uint32_t>(kWave)) {
                // lane L owns blocks 128 L .. 128 L + 127 (summed in rotated order: lanes on different banks)
                uint32_t sum = 0;
                for (uint32_t j = 0; j < 128u; j++) sum += known[lane * 128u + ((j + 2u * lane) & 127u)];
                uint32_t incl = sum;  // sum over lanes <= this one
#pragma unroll
                for (int o = 1; o < kWave; o <<= 1) {
                    const uint32_t t = __shfl_up(incl, o, kWave);
                    if (lane >= static_cast<uint32_t>(o)) incl += t;
                }
                uint32_t before = incl - sum;
                if (before < want && want <= incl) {
                    for (uint32_t j = 0; j < 128u; j++) {
                        before += known[lane * 128u + j];
                        if (before >= want) {
                            answer[0] = lane * 128u + j;
                            break;
                        }
                    }
                }
            }
            __syncthreads();
            last_block_for_equals = answer[0];
            __syncthreads();  // (the list's LDS is free again)
        }
    }
    if (part == 0 && tid == 0) head[16 * kBigPickLists] = thr;
    BPS(3);

    // ---- the blocks of this workgroup's share that reach lo --------------------------------
    const bool pass = mine_live && mykey >= lo && (myb <= last_block_for_equals || mykey > thr);
    const uint64_t mask = __ballot(pass);
    if (lane == 0) wave_hits[wave] = static_cast<uint32_t>(__popcll(mask));
    __syncthreads();
    uint32_t H = 0, pos = 0;
#pragma unroll
    for (int w = 0; w < NW; w++) {
        const uint32_t c = wave_hits[w];
        pos += (static_cast<uint32_t>(w) < wave) ? c : 0u;
        H += c;
    }
    if (pass) hits[pos + lanes_below(mask)] = myb;
    __syncthreads();
    BPS(4);

    // ---- their elements at or above lo -> lcand ---------------------------------------------
    const float lo_f = ordered_to_float(lo);
    const uint32_t items = H * kBlockLanes;
    for (uint32_t j0 = 0; j0 < items; j0 += NT * U) {
        Vec128<T> r[U];
        uint32_t e0[U], cend[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t j = j0 + static_cast<uint32_t>(u) * NT + tid;
            const uint32_t b = hits[j < items ? j / kBlockLanes : 0u];
            e0[u] = b * BE + (j % kBlockLanes) * VEC;
            cend[u] = j < items ? n : 0u;
            r[u].v = make_uint4(0, 0, 0, 0);
            if constexpr (ALIGNED) {
                r[u].load(rowp + (e0[u] < cend[u] ? e0[u] : 0u));
            } else {
#pragma unroll
                for (int c = 0; c < VEC; c++) r[u].set(c, load_elem(rowp, e0[u] + c < cend[u] ? e0[u] + c : 0u));
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            float vm = -INFINITY;
            bool any_nan = false;
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                const float x = r[u].get(c);
                vm = fmaxf(vm, x);
                if constexpr (!SOFTMAX) any_nan = any_nan || x != x;
            }
            if (!(vm < lo_f) || any_nan) {
#pragma unroll
                for (int c = 0; c < VEC; c++) {
                    const float x = r[u].get(c);
                    const uint32_t idx = e0[u] + static_cast<uint32_t>(c);
                    const uint32_t key = (SOFTMAX && x != x) ? 0u : order_key(x);
                    if (idx < cend[u] && key >= lo && (key > thr || idx / BE <= last_block_for_equals)) {
                        // above the threshold: wanted whatever else happens; at or below it: up to the quota
                        if (key > thr) {
                            const uint32_t at = atomicAdd(&lcount, 1u);
                            if (at < static_cast<uint32_t>(kBigPickLocalCap)) lcand[at] = composite(key, idx);
                        } else {
                            const uint32_t at = atomicAdd(&zcount, 1u);
                            if (at < static_cast<uint32_t>(kBigPickZoneQuota)) zcand[at] = composite(key, idx);
                        }
                    }
                }
            }
        }
    }
    __syncthreads();
    BPS(5);
    // Elements at or below the threshold: within the quota they join the candidates; beyond
    // it (equal values en masse, rows of mostly -inf) none of this workgroup's do, the row
    // is marked, and the rank kernel takes the threshold's own rank group from a walk over
    // the row in index order -- everything ABOVE the threshold is in the lists either way.
    const uint32_t cnt_a = lcount, cnt_z = zcount;  // (the same for every thread)
    const bool trimmed = cnt_z > bigpick_zone_quota(want, G2);
    if (!trimmed && tid < cnt_z && cnt_a + tid < static_cast<uint32_t>(kBigPickLocalCap)) lcand[cnt_a + tid] = zcand[tid];
    if (trimmed && tid == 0) atomicOr(&head[16 * kBigPickLists + 1], 1u);
    __syncthreads();
    const uint32_t cnt = cnt_a + (trimmed ? 0u : cnt_z);
    const uint32_t held = min(cnt, static_cast<uint32_t>(kBigPickLocalCap));

    // ---- softmax: the candidates' accurate terms; what they add to the row's sum ------------
    long long fix = 0;
    if constexpr (SOFTMAX) {
        for (uint32_t t = tid; t < held; t += NT) {
            const uint64_t c = lcand[t];
            const uint32_t idx = composite_index(c);
            const float xv = ordered_to_float(static_cast<uint32_t>(c >> 32));
            const uint32_t b = idx / per, off = idx - b * per;
            const uint32_t sp = b * kScanWaves + ((off / VEC) % kScanThreads) / kWave;  // the scan wave that summed it
            const float ref = __uint_as_float(static_cast<uint32_t>(recs[2 * sp + 1]));
            const uint64_t apart = ws.recs2[static_cast<size_t>(row) * waves + sp];  // the value that wave counted apart
            const bool copy = static_cast<uint32_t>(apart) != 0u && xv == __uint_as_float(static_cast<uint32_t>(apart >> 32));
            const float term = softmax_term(xv, M);
            // what the element should contribute, exp(fl(x - M)), minus what its wave
            // added for it, fast_term(x, ref) * exp(ref - M) (a copy went in with this very term)
            const double cr = copy ? 0.0
                                   : static_cast<double>(term) -
                                         static_cast<double>(fast_term(xv, ref)) *
                                             sum_rescale(__longlong_as_double(static_cast<long long>(recs[2 * sp])), ref, M);
            if (cr > -1.0 && cr < 1.0) fix += static_cast<long long>(cr * kBigPickFixUnit);  // (anything else: the row's sum is not finite)
            lterm[t] = term;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) fix += __shfl_xor(fix, o, kWave);
        if (lane == 0) iscratch[wave] = fix;
    }
    if (cnt != 0) {
        // Few candidates (the rule): all to list part % 8.  Many (a sorted row's candidates lie
        // in one or two shares): candidate t to list t % 8, so that no list carries them alone.
        const bool spread = cnt > static_cast<uint32_t>(kBigPickSpread) && cnt <= static_cast<uint32_t>(kBigPickLocalCap);
        const uint32_t list0 = part % kBigPickLists;
        __syncthreads();
        if (tid < static_cast<uint32_t>(kBigPickLists)) {
            if (spread) {
                lbase[tid] = atomicAdd(&head[16 * tid], (cnt + (kBigPickLists - 1u) - tid) / kBigPickLists);
            } else if (tid == list0) {
                // more than the workgroup can hold: the list's count is pushed past its capacity
                lbase[tid] = atomicAdd(&head[16 * tid], cnt <= static_cast<uint32_t>(kBigPickLocalCap) ? cnt : kBigPickListCap + 1u);
            }
            if constexpr (SOFTMAX) {
                if (tid == list0) {
                    long long total = 0;
#pragma unroll
                    for (int w = 0; w < NW; w++) total += iscratch[w];
                    atomicAdd(reinterpret_cast<unsigned long long *>(head + 16 * tid + 2), static_cast<unsigned long long>(total));
                }
            }
        }
        __syncthreads();
        BPS(6);
        if (cnt <= static_cast<uint32_t>(kBigPickLocalCap)) {
            const size_t row_at = static_cast<size_t>(row) * kBigPickLists * kBigPickListCap;
            for (uint32_t t = tid; t < cnt; t += NT) {
                const uint32_t list = spread ? t % kBigPickLists : list0;
                const uint32_t slot = lbase[list] + (spread ? t / kBigPickLists : t);
                if (slot < static_cast<uint32_t>(kBigPickListCap)) {  // (a list past its capacity: the rank kernel sees its count)
                    const size_t at = row_at + static_cast<size_t>(list) * kBigPickListCap + slot;
                    bw.cand[at] = lcand[t];
                    if constexpr (SOFTMAX) bw.term[at] = lterm[t];
                }
            }
        }
    }
    BPS(7);
    // ---- softmax: the row's maximum and sum of fast terms, once per row ------------------------
    if constexpr (SOFTMAX) {
        if (part == 0) {  // (the same for every thread)
            double acc = 0.0;
            for (uint32_t w = tid; w < waves; w += NT) {
                const double sv = __longlong_as_double(static_cast<long long>(recs[2 * w]));
                const float ref = __uint_as_float(static_cast<uint32_t>(recs[2 * w + 1]));
                if (sv != 0.0) acc += sv * sum_rescale(sv, ref, M);
                const uint64_t apart = ws.recs2[static_cast<size_t>(row) * waves + w];
                if (static_cast<uint32_t>(apart) != 0u)
                    acc += static_cast<double>(static_cast<uint32_t>(apart)) *
                           static_cast<double>(softmax_term(__uint_as_float(static_cast<uint32_t>(apart >> 32)), M));
            }
            const double s_base = block_sum_fast<NT>(acc, dscratch);
            if (tid == 0) {
                bw.stat[2 * static_cast<size_t>(row)] = s_base;
                bw.stat[2 * static_cast<size_t>(row) + 1] = static_cast<double>(M);
            }
        }
    }
}

// The exact single-workgroup select over a whole row (select.hpp): what the lists could
// not hold or decide.  All threads of the workgroup call.
template <typename T, bool SOFTMAX>
__device__ __forceinline__ void bigpick_exact_row(SelectShared &ex, const T *rowp, T *ov, int32_t *oi, uint32_t n, uint32_t kk,
                                                  float *fscratch, double *dscratch) {
    constexpr int NT = kBigPickThreads;
    const uint32_t tid = threadIdx.x;
    if constexpr (SOFTMAX) {
        const LineStats st = line_stats<T, NT>(rowp, 0, n, 1, fscratch, dscratch, 1.f);
        select_topk_line<NT>(ex, n, kk, [&](uint32_t j) {
            return order_key(round_to_storage<T>(softmax_prob(load_elem(rowp, j), st)));
        });
        for (uint32_t r = tid; r < kk; r += NT) {
            const uint32_t idx = composite_index(ex.sel[r]);
            store_elem(ov, r, softmax_prob(load_elem(rowp, idx), st));
            oi[r] = static_cast<int32_t>(idx);
        }
    } else {
        select_topk_line<NT>(ex, n, kk, [&](uint32_t j) { return order_key(load_elem(rowp, j)); });
        for (uint32_t r = tid; r < kk; r += NT) {
            const uint32_t idx = composite_index(ex.sel[r]);
            ov[r] = rowp[idx];
            oi[r] = static_cast<int32_t>(idx);
        }
    }
}

constexpr int kBigRankPerLane = kBigPickCap / kBigPickThreads;  // list entries a lane holds: a wave takes a quarter of the list

// kBigPickCap / kBigPickMine workgroups a row; workgroup g places candidates
// 32 g .. 32 g + 31 of the row's lists (taken one after the other).
template <typename T, bool SOFTMAX>
__global__ __launch_bounds__(kBigPickThreads) void bigpick_rank_kernel(const T *__restrict__ in, T *__restrict__ values,
                                                                        int32_t *__restrict__ indices, uint32_t n, uint32_t k,
                                                                        BigPickWorkspace bw) {
    constexpr int NT = kBigPickThreads, NW = kBigPickWaves;
    constexpr uint32_t G3 = kBigPickCap / kBigPickMine;
    static_assert(kBigPickMine == 32, "a candidate per lane of half a wave");
    __shared__ union U {
        uint32_t part[NW][kBigPickMine];
        SelectShared exact;
        __device__ U() {}
    } smem;
    __shared__ float fscratch[NW];
    __shared__ double dscratch[NW];
    __shared__ uint32_t walk_slots[NW], walk_counts[2 * NW], walk_keys[2];
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    // (workgroup g of every row before workgroup g + 1 of any: the few that have candidates are dispatched first)
    const uint32_t rows = gridDim.x / G3;
    const uint32_t g = blockIdx.x / rows, row = blockIdx.x - g * rows;
    const T *rowp = in + static_cast<size_t>(row) * n;
    T *ov = values + static_cast<size_t>(row) * k;
    int32_t *oi = indices + static_cast<size_t>(row) * k;
    const uint32_t want = k + 1, kk = min(k, n);
    const uint32_t *head = bw.head + static_cast<size_t>(row) * kBigPickHeadWords;
    BPS(16);
    // the lists' lengths and where each starts in the row's one sequence of candidates
    uint32_t len[kBigPickLists], start[kBigPickLists + 1];
    bool exact = false;  // (the same in every workgroup of the row)
    start[0] = 0;
#pragma unroll
    for (int j = 0; j < kBigPickLists; j++) len[j] = head[16 * j];
#pragma unroll
    for (int j = 0; j < kBigPickLists; j++) {
        exact = exact || len[j] > static_cast<uint32_t>(kBigPickListCap);
        len[j] = min(len[j], static_cast<uint32_t>(kBigPickListCap));
        start[j + 1] = start[j] + len[j];
    }
    const uint32_t C = start[kBigPickLists];
    const uint32_t thr = head[16 * kBigPickLists];
    exact = exact || C > static_cast<uint32_t>(kBigPickCap);
    // Walk mode: the lists hold every element above the threshold, but of the elements at
    // or below it not all that the result may need (a gather workgroup met more than its
    // quota of them; fewer than k+1 candidates; a margin that does not separate
    // probabilities).  Then everything that ranks with the threshold forms ONE group of equal
    // rank, taken in index order: the ranking below places what ranks above that group, and
    // the row's last workgroup fills the remaining places with the group's first members
    // from a walk over the row.
    bool walk = !exact && (head[16 * kBigPickLists + 1] != 0u || C < want);
    uint32_t star = thr;  // what ranks with the threshold: this key (softmax: this probability's key)
    double rinv = 0.0;
    float M = 0.f;
    if constexpr (SOFTMAX) {
        if (!exact) {
            const double s_base = bw.stat[2 * static_cast<size_t>(row)];
            M = static_cast<float>(bw.stat[2 * static_cast<size_t>(row) + 1]);
            if (!(s_base > 0.0 && s_base < static_cast<double>(INFINITY)) || !(M > -INFINITY && M < INFINITY)) {
                // a NaN or +inf element, or nothing above -inf: every probability of the row is
                // NaN, all of them tie, the lowest indices win
                if (g == 0)
                    for (uint32_t r = tid; r < kk; r += NT) {
                        store_elem(ov, r, __uint_as_float(0x7FC00000u));
                        oi[r] = static_cast<int32_t>(r);
                    }
                return;
            }
            long long fix = 0;
#pragma unroll
            for (int j = 0; j < kBigPickLists; j++)
                fix += static_cast<long long>(*reinterpret_cast<const unsigned long long *>(head + 16 * j + 2));
            const double total = s_base + static_cast<double>(fix) * (1.0 / kBigPickFixUnit);
            exact = !(total > 0.0 && total < static_cast<double>(INFINITY));
            if (!exact) {
                rinv = 1.0 / total;
                auto prob = [&](float xv) {
                    return round_to_storage<T>(static_cast<float>(static_cast<double>(softmax_term(xv, M)) * rinv));
                };
                const float p_star = prob(ordered_to_float(thr));
                star = order_key(p_star);
                // the margin has to separate what is below it from the k+1 at or above the threshold
                if (thr > kKeyNegInf) walk = walk || !(p_star > prob(ordered_to_float(bigpick_lowered<T, true>(thr))));
            }
        }
    }
    const bool walker = walk && !exact && g == G3 - 1;
    if (!exact && !walker && g * kBigPickMine >= C) return;  // nothing of the sequence is this workgroup's
    if (exact) {
        if (g != 0) return;
        bigpick_exact_row<T, SOFTMAX>(smem.exact, rowp, ov, oi, n, kk, fscratch, dscratch);
        return;
    }
    BPS(17);
    // ---- candidate f of the sequence (0 past its end: ranks before nothing), softmax: keyed by probability
    const size_t row0 = static_cast<size_t>(row) * kBigPickLists * kBigPickListCap;
    auto where = [&](uint32_t f) {  // (f < C)
        uint32_t j = 0;
#pragma unroll
        for (int q = 1; q < kBigPickLists; q++) j += (f >= start[q]) ? 1u : 0u;
        uint32_t s0 = start[0];
#pragma unroll
        for (int q = 1; q < kBigPickLists; q++) s0 = (j == static_cast<uint32_t>(q)) ? start[q] : s0;
        return row0 + static_cast<size_t>(j) * kBigPickListCap + (f - s0);
    };
    auto keyed = [&](uint64_t c, float term, bool live) -> uint64_t {
        if constexpr (SOFTMAX) {
            const float p = round_to_storage<T>(static_cast<float>(static_cast<double>(term) * rinv));
            c = (static_cast<uint64_t>(order_key(p)) << 32) | (c & 0xFFFFFFFFull);
        }
        return live ? c : 0ull;
    };
    if (g * kBigPickMine < C) {  // (the same for every thread; false only for a walker without candidates of its own)
        // this wave's quarter of the sequence, entry e of lane L = candidate w Q + 64 e + L; all loads first
        const uint32_t Q = (C + NW - 1) / NW;
        const uint32_t steps = (Q + kWave - 1) / kWave;  // (<= kBigRankPerLane)
        uint64_t ent[kBigRankPerLane];
        float eterm[kBigRankPerLane];
#pragma unroll
        for (int e = 0; e < kBigRankPerLane; e++) {
            const uint32_t o = static_cast<uint32_t>(e) * kWave + lane;
            const uint32_t f = wave * Q + o;
            const bool live = o < Q && f < C;
            ent[e] = 0;
            eterm[e] = 0.f;
            if (static_cast<uint32_t>(e) < steps) {  // (wave-uniform)
                const size_t at = where(live ? f : 0u);
                ent[e] = bw.cand[at];
                if constexpr (SOFTMAX) eterm[e] = bw.term[at];
            }
        }
        // this workgroup's own candidates: lane L < 32 of every wave holds candidate 32 g + L
        const uint32_t my_at = g * kBigPickMine + (lane & 31u);
        const bool my_live = my_at < C;
        const size_t mat = where(my_live ? my_at : 0u);
        uint64_t mine = bw.cand[mat];
        float mterm = 0.f;
        if constexpr (SOFTMAX) mterm = bw.term[mat];
        mine = keyed(mine, mterm, my_live);
#pragma unroll
        for (int e = 0; e < kBigRankPerLane; e++) {
            const uint32_t o = static_cast<uint32_t>(e) * kWave + lane;
            ent[e] = keyed(ent[e], eterm[e], static_cast<uint32_t>(e) < steps && o < Q && wave * Q + o < C);
        }
        BPS(18);
        // ---- how many of this wave's entries rank before each of the 32: one compare of the
        // wave's 64 entries against the candidate (a scalar), and the population count of the result
        const uint32_t mine_lo = static_cast<uint32_t>(mine), mine_hi = static_cast<uint32_t>(mine >> 32);
        uint32_t before = 0;  // lane j: the count for candidate j
        // (entries past the wave's share are 0 and count for nothing: the loop over them is
        // compiled for 4, 8, 12, 16, 24 and 32 entries a lane, without a branch inside)
        auto count_all = [&](auto steps_tag) __attribute__((always_inline)) {
            constexpr int STEPS = decltype(steps_tag)::value;
            for (int j = 0; j < kBigPickMine; j++) {
                const uint64_t m = (static_cast<uint64_t>(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(mine_hi), j))) << 32) |
                                   static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(mine_lo), j));
                uint32_t c = 0;
#pragma unroll
                for (int e = 0; e < STEPS; e++) c += static_cast<uint32_t>(__popcll(__ballot(ent[e] > m)));
                before = (lane == static_cast<uint32_t>(j)) ? c : before;
            }
        };
        if (steps <= 4u) count_all(std::integral_constant<int, 4>{});
        else if (steps <= 8u) count_all(std::integral_constant<int, 8>{});
        else if (steps <= 12u) count_all(std::integral_constant<int, 12>{});
        else if (steps <= 16u) count_all(std::integral_constant<int, 16>{});
        else if (steps <= 24u) count_all(std::integral_constant<int, 24>{});
        else count_all(std::integral_constant<int, kBigRankPerLane>{});
        if (lane < static_cast<uint32_t>(kBigPickMine)) smem.part[wave][lane] = before;
        __syncthreads();
        BPS(19);
        // (walk mode: only what ranks above the threshold's group is placed here)
        if (tid < static_cast<uint32_t>(kBigPickMine) && my_live && (!walk || mine_hi > star)) {
            uint32_t rank = 0;
#pragma unroll
            for (int w = 0; w < NW; w++) rank += smem.part[w][tid];
            if (rank < kk) {
                const uint32_t idx = composite_index(mine);
                if constexpr (SOFTMAX) store_elem(ov, rank, ordered_to_float(mine_hi));
                else ov[rank] = rowp[idx];  // bit copy (keeps the sign of a zero)
                oi[rank] = static_cast<int32_t>(idx);
            }
        }
        BPS(20);
    }
    if (!walker) return;  // (the same for every thread)

    // ---- walk mode, the row's last workgroup: the group that ranks with the threshold ---------
    // n_above entries of the lists rank above it and are placed by the ranking; its members
    // (an interval of order keys: probability does not decrease with the logit) take the
    // places behind them in index order.
    __syncthreads();
    uint32_t c_above = 0;  // (wave-uniform)
    for (uint32_t f0 = 0; f0 < C; f0 += NT) {
        const uint32_t f = f0 + tid;
        const bool live = f < C;
        const size_t at = where(live ? f : 0u);
        float term = 0.f;
        if constexpr (SOFTMAX) term = bw.term[at];
        const uint64_t c = keyed(bw.cand[at], term, live);
        c_above += static_cast<uint32_t>(__popcll(__ballot(static_cast<uint32_t>(c >> 32) > star)));
    }
    const uint32_t n_above = bigpick_count_sum(c_above, walk_slots);
    if (n_above >= kk) return;
    uint32_t xlo = thr, xhi = thr;
    float p_star = 0.f;
    if constexpr (SOFTMAX) {
        p_star = ordered_to_float(star);
        if (wave == 0) {
            auto prob_of_key = [&](uint32_t key) {
                return round_to_storage<T>(static_cast<float>(static_cast<double>(softmax_term(ordered_to_float(key), M)) * rinv));
            };
            // down to the smallest key of that probability (probability 0: everything below as well) ...
            const uint32_t lo_key = (p_star > 0.f && thr > kKeyNegInf) ? lowest_key_of_probability(thr, p_star, prob_of_key) : 0u;
            // ... and up to the largest: one below the smallest key of a larger probability
            const float p_next = __uint_as_float(__float_as_uint(p_star) + 1u);
            const uint32_t top = order_key(M);
            const uint32_t hi_key = prob_of_key(top) >= p_next ? lowest_key_of_probability(top, p_next, prob_of_key) - 1u : top;
            if (lane == 0) {
                walk_keys[0] = lo_key;
                walk_keys[1] = hi_key;
            }
        }
        __syncthreads();
        xlo = walk_keys[0];
        xhi = walk_keys[1];
    }
    const uint32_t places = kk - n_above;
    auto place = [&](uint32_t pos, uint32_t j, float x) {
        if constexpr (SOFTMAX) store_elem(ov, n_above + pos, p_star);
        else store_elem(ov, n_above + pos, x);  // (the element's own bits: a half widened to float narrows back exactly)
        oi[n_above + pos] = static_cast<int32_t>(j);
    };
    const bool row_aligned = (reinterpret_cast<uintptr_t>(rowp) & 15u) == 0;  // (the same for every thread)
#ifdef VKOP_STAMPS
    const unsigned long long walk_t0 = wall_clock64();
#endif
    const uint32_t found = (row_aligned && xhi != 0xFFFFFFFFu) ? first_members_by_vectors<T, NT>(walk_counts, rowp, n, places, xlo, xhi, place)
                                       : first_members_by_scan<T, NT>(walk_counts, rowp, n, places, xlo, xhi, 1.f,
                                                                      [&](uint32_t pos, uint32_t j) { place(pos, j, load_elem(rowp, j)); });
#ifdef VKOP_STAMPS
    if (tid == 0 && row < 8) {  // per row: (found << 40 | places << 20 | n_above), nanoseconds
        g_bp_stamps[32 + 2 * row] = (static_cast<unsigned long long>(found) << 40) | (static_cast<unsigned long long>(places) << 20) | n_above;
        g_bp_stamps[33 + 2 * row] = (wall_clock64() - walk_t0) * 10;
    }
#endif
    if (found < places) {
        // the group does not fill the places: elements that rank below it are part of the
        // result, and of those the lists say nothing
        __syncthreads();
        bigpick_exact_row<T, SOFTMAX>(smem.exact, rowp, ov, oi, n, kk, fscratch, dscratch);
    }
}

}  // namespace vkop
