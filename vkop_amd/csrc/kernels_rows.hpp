// Streaming kernels for contiguous rows (the reduced axis is the last one).
//
// rows_chunk_kernel makes the one pass over the input.  A row is split into G
// chunks, one workgroup per chunk, so a few long rows still fill the chip.
// Each workgroup
//   1. issues all of its 128-bit loads (V per thread) at once,
//   2. consumes the vectors in the order they arrive: per vector its maximum and
//      the sum of exp(x - ref), where ref is taken from the wave's FIRST vector
//      (any reference is valid for a partial sum; taking it from the first
//      vector lets the exponentials overlap the rest of the stream; a wave that
//      later meets an element well above it sums again against its maximum),
//   3. publishes per-lane maxima to LDS; the waves find, by ballot descents over
//      them, a threshold that at least k+1 elements of the chunk reach,
//   4. compacts the elements at or above the threshold: the few vectors holding
//      one go to a per-wave stage in LDS (ballot + popcount), are unpacked one
//      element per lane, and the survivors are written as (order key, ~index)
//      composites into the chunk's candidate list; a list that overflows (values
//      in order or in clusters, many equal values) is made again with the
//      chunk's exact (k+1)-th largest element as the threshold and only the
//      first k+1 elements equal to it,
//   5. writes one record per wave: partial sum, reference, maximum, threshold
//      and the candidates it contributed.
// The merge (rows_merge_kernel, or in the one-kernel variant the workgroup that
// finishes a row's last chunk, found with one counter per row) combines the
// partial sums, finds the (k+1)-th largest candidate, ranks the candidates
// above it exactly (key, then lower index), replaces the summed fast terms of
// the ranked elements by accurate ones, computes the probabilities of the
// winners only, orders equal probabilities by index and writes the row's
// result.  Every order of summation is fixed and the ranking does not depend on
// the order candidates were stored in, so results are bit-identical from run to
// run.  The merge also settles by itself: a probability tie across the k-th
// place (the tied logit interval is searched, its members fetched or, if they
// are many, taken from the start of the row), rows of NaN, rows with fewer than
// k+1 elements above -inf, ties at probability 0, and more candidates than its
// LDS array holds (exact cut over the candidates in registers).  What is left
// for the exact radix select of select.hpp over the whole row -- a candidate
// list that overflows even after the second attempt -- needs an adversarial
// layout of equal values; the result is always top-k (probability, then lower
// index) of the row's softmax.
#pragma once

#include <type_traits>

#include "device_utils.hpp"
#include "kernels_general.hpp"
#include "select.hpp"

namespace vkop {

// Debug builds only (-DVKOP_STAMPS=<name of the C function that reads them out>, rows_inst.hip):
// clock stamps of one workgroup's first thread (workgroup 0 unless g_bp_block is set).
#ifdef VKOP_STAMPS
static __device__ unsigned long long g_bp_stamps[64];
static __device__ unsigned int g_bp_block;
#define BPS(i) do { if (threadIdx.x == 0 && blockIdx.x == g_bp_block) g_bp_stamps[i] = wall_clock64(); } while (0)
#else
#define BPS(i) do { } while (0)
#endif

constexpr int kFastCap = 1024;       // LDS slots for elements above the merge threshold
constexpr int kFastMaxK = 511;       // k + 1 <= 512 ranks are kept in LDS (the merging workgroup has a thread per rank:
                                     // k <= 255 for rows_merge_kernel, more only where one larger workgroup holds the row)
constexpr int kMergeThreads = 256;    // rows_merge_kernel workgroup
constexpr int kMergeRecsMax = 4096;   // candidate slots per row the merge takes in registers
constexpr int kMergeWavesMax = 256;   // chunk-kernel waves per row the merge can combine
constexpr int kMergeChunksMax = 64;   // chunks per row
constexpr int kLocalCap = 1024;       // candidate slots of the LDS-resident list of a one-workgroup row (cap for k = 255)

// f(std::integral_constant<int, I>) for I = B .. E-1, unrolled at compile time
template <int B, int E, typename F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

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

// Sum of a double over the wave, returned wave-uniform.  Same four in-row steps
// (every lane of a row ends with the same bits, because each step adds the same
// two partial sums in either order), then the four rows in a fixed order.
__device__ __forceinline__ double wave_sum_f64_uniform(double v) {
    auto step = [](double a, auto tag) {
        constexpr int ctrl = decltype(tag)::value;
        const uint64_t u = static_cast<uint64_t>(__double_as_longlong(a));
        const uint32_t lo = VKOP_DPP_U32(static_cast<uint32_t>(u), ctrl);
        const uint32_t hi = VKOP_DPP_U32(static_cast<uint32_t>(u >> 32), ctrl);
        return a + __longlong_as_double(static_cast<long long>((static_cast<uint64_t>(hi) << 32) | lo));
    };
    v = step(v, std::integral_constant<int, 0xB1>{});
    v = step(v, std::integral_constant<int, 0x4E>{});
    v = step(v, std::integral_constant<int, 0x141>{});
    v = step(v, std::integral_constant<int, 0x140>{});
    const uint64_t u = static_cast<uint64_t>(__double_as_longlong(v));
    auto row = [&](int l) {
        const uint32_t lo = __builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(u)), l);
        const uint32_t hi = __builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(u >> 32)), l);
        return __longlong_as_double(static_cast<long long>((static_cast<uint64_t>(hi) << 32) | lo));
    };
    return (row(0) + row(16)) + (row(32) + row(48));
}
// Inclusive prefix sum over the wave's lanes: four shifts inside each row of 16 lanes, then the
// last lane of row 0 (rows 0 and 1) broadcast into the rows above (lanes without a source add 0).
__device__ __forceinline__ uint32_t wave_inclusive_sum_u32(uint32_t v) {
#define VKOP_DPP_ADD(ctrl, rows) \
    v += static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), ctrl, rows, 0xF, false))
    VKOP_DPP_ADD(0x111, 0xF);  // row_shr:1
    VKOP_DPP_ADD(0x112, 0xF);  // row_shr:2
    VKOP_DPP_ADD(0x114, 0xF);  // row_shr:4
    VKOP_DPP_ADD(0x118, 0xF);  // row_shr:8
    VKOP_DPP_ADD(0x142, 0xA);  // row_bcast:15 into rows 1 and 3
    VKOP_DPP_ADD(0x143, 0xC);  // row_bcast:31 into rows 2 and 3
#undef VKOP_DPP_ADD
    return v;
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

constexpr uint32_t kKeyNegInf = 0x007FFFFFu;  // order key of -inf, the smallest key of a real element

// Float threshold equivalent to an order-key threshold: x passes iff
// !(x < thr_f).  Keys at or below the key of -inf mean "everything passes".
__device__ __forceinline__ float key_threshold_to_float(uint32_t thr) {
    return thr <= kKeyNegInf ? -INFINITY : ordered_to_float(thr);
}

// One wave finds a lower bound of the `want`-th largest of NW * 64 keys held in
// LDS (key 0 = no element): bitwise descent over the top `bits` bits, counting
// with ballots; the untouched low bits stay zero, which only lowers the bound.
// Returns 0 (= take everything) when fewer than `want` keys are non-zero in
// those bits.  Called by all 64 lanes of one wave.
template <int NW>
__device__ __forceinline__ uint32_t block_kth_largest_floor(const uint32_t *keys, uint32_t want, int bits) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    uint32_t kv[NW];
#pragma unroll
    for (int w = 0; w < NW; w++) kv[w] = keys[w * kWave + lane];
    uint32_t prefix = 0;
    for (int bit = 31; bit > 31 - bits; bit--) {
        const uint32_t trial = prefix | (1u << bit);
        uint32_t cnt = 0;
#pragma unroll
        for (int w = 0; w < NW; w++) cnt += static_cast<uint32_t>(__popcll(__ballot(kv[w] >= trial)));
        if (cnt >= want) prefix = trial;
    }
    return prefix;
}

// Block-wide max / sum with the wave step done by DPP moves (no trips through
// LDS inside a wave: the merge is a chain of dependent steps, and each of those
// trips is one of them).  Same contract as block_max / block_sum.
template <int NT> __device__ __forceinline__ float block_max_fast(float v, float *scratch) {
    constexpr int NW = NT / kWave;
    v = wave_max_f32_uniform(v);
    if constexpr (NW == 1) return v;
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    float r = scratch[0];
#pragma unroll
    for (int w = 1; w < NW; w++) r = fmaxf(r, scratch[w]);
    return r;
}
template <int NT> __device__ __forceinline__ double block_sum_fast(double v, double *scratch) {
    constexpr int NW = NT / kWave;
    v = wave_sum_f64_uniform(v);
    if constexpr (NW == 1) return v;
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    double r = scratch[0];
#pragma unroll
    for (int w = 1; w < NW; w++) r += scratch[w];  // fixed order: run-to-run stable
    return r;
}

// exp(x) in double to a relative error below 1e-13, for rescaling partial sums
// (x = a reference minus the row maximum, so x <= 0 in practice).
__device__ __forceinline__ double exp_rescale(double x) {
    if (!(x == x)) return x;
    if (x < -745.0) return 0.0;
    if (x > 709.0) return static_cast<double>(INFINITY);
    const double n = rint(x * 1.4426950408889634074);
    const double r = fma(-n, 1.9082149292705877000e-10, fma(-n, 0.693147180369123816490, x));  // ln 2 in two parts
    double p = 1.0 / 39916800.0;
    p = fma(p, r, 1.0 / 3628800.0);
    p = fma(p, r, 1.0 / 362880.0);
    p = fma(p, r, 1.0 / 40320.0);
    p = fma(p, r, 1.0 / 5040.0);
    p = fma(p, r, 1.0 / 720.0);
    p = fma(p, r, 1.0 / 120.0);
    p = fma(p, r, 1.0 / 24.0);
    p = fma(p, r, 1.0 / 6.0);
    p = fma(p, r, 0.5);
    p = fma(p, r, 1.0);
    p = fma(p, r, 1.0);
    return ldexp(p, static_cast<int>(n));
}

// The factor that carries a partial sum of terms exp(x - ref) over to the row's maximum M.
// A sum that is a whole number comes from terms that were all exactly 1 (or 0): a flat stretch
// of the row, every element equal to the reference (or -inf).  Each of them counts
// exp_accurate(fl(ref - M)) in the sum as defined (kernels_general.hpp) -- a float, off the exact
// exponential of the exact difference by up to 3e-7 relative, the same for every copy -- so that
// is the factor then: rows that are one repeated value and a few peaks stay within the bar.
__device__ __forceinline__ double sum_rescale(double s, float ref, float M) {
    if (s != 0.0 && s == rint(s)) return static_cast<double>(softmax_term(ref, M));  // (0: an idle lane's, or nothing to carry)
    return exp_rescale(static_cast<double>(ref) - static_cast<double>(M));
}

// ---- memory shared between workgroups ------------------------------------------
// Everything one workgroup writes for another to read goes through device-scope
// atomic stores and loads (relaxed): such a store is written through to memory
// and such a load never takes a stale line from a cache, whichever XCD either
// workgroup runs on.  No release fence is used: it would write back the whole L2.

__device__ __forceinline__ void publish(uint64_t *p, uint64_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t fetch(const uint64_t *p) {
    return __hip_atomic_load(const_cast<uint64_t *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Returns once every store this thread has issued has been performed (for a
// published value: is visible device-wide).
__device__ __forceinline__ void drain_stores() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // the compiler keeps earlier stores above this point
    __builtin_amdgcn_s_waitcnt(0);                          // vmcnt(0) expcnt(0) lgkmcnt(0)
}

constexpr int kRecWords = 4;  // 64-bit words of a chunk-kernel wave's record
struct RowsWorkspace {
    uint32_t *tickets;  // [rows]: chunks of the row that have published; 0 between calls
    uint64_t *sums;     // [rows][G * waves per chunk][kRecWords]: the wave's sum of exp(x - ref) as double bits; ref (low
                        // half) and the wave's maximum (high half) as float bits; the candidates the wave
                        // contributed to its chunk's list (low half; all ones: it could not stage them all)
                        // and the chunk's threshold as an order key (high half); the value whose copies the
                        // wave counted apart (float bits, high half) and how many it found (low half; 0: none):
                        // its sum leaves them out
    uint64_t *cand;     // [rows][G][cap]: composites (order key, ~index) of the elements at or above the chunk threshold
    uint32_t cap;       // candidate slots per chunk (power of two)
    uint32_t cap_shift;
};

struct SumPartial {
    double s;   // sum of exp(x - ref) over the wave's elements
    float ref;  // reference of that sum: the maximum of the wave's first vectors, or 0 if that is -inf
    float m;    // the maximum of the wave's elements
};

template <int NT> struct ChunkShared {  // chunk phase
    uint32_t lane_key[NT];
    uint4 stage_v[NT];     // per wave: up to 64 vectors holding an element at or above the threshold ...
    uint32_t stage_e[NT];  // ... and the index of their first element
    uint32_t wave_thr[16];
    uint32_t refine[40];  // element counts per bit of the exact threshold search; [32], [33]: smallest key at or above a bound / elements
                          // above that key, and the same in [34] ... [39] for the next two distinct values up
    uint32_t thr, total, over;
};

struct RowsShared {  // merge phase
    uint64_t cand[kFastCap];
    uint32_t rank[kFastCap];
    float prob[kFastMaxK + 1];
    uint32_t pidx[kFastMaxK + 1];
    double corr[kFastMaxK + 1];
    double scale[kMergeWavesMax];  // exp(ref - M) per wave partial
    float ref[kMergeWavesMax];
    float x0[kMergeWavesMax];        // the value whose copies the wave's sum leaves out (counted apart); NaN: none
    uint32_t cnt[kMergeChunksMax];   // live candidates per chunk
    uint32_t cthr[kMergeChunksMax];  // threshold per chunk: the chunk's elements at or above it are candidates
    uint32_t pkey[kFastMaxK + 1];    // order key of the logit, by rank
    uint32_t g0, xlo;                // tie at the cut: first rank of the tied group, smallest key in it
    uint32_t members;                // ... and how many of its members are in lane_key[] (their indices)
    float row_max;                   // the row's maximum; its sum of terms is `total`
    uint32_t scan_counts[2 * 16];    // fill_group_by_scan: members per wave, double-buffered
    uint32_t wave_thr[16];           // merge threshold: each wave's bound
    uint32_t lane_key[1024];
    uint32_t thr;
    uint32_t count;
    uint32_t flag;
    uint32_t wave_overflow;          // pick kernel: a wave found more blocks to read again than its share of the list holds
    double total;
};

template <int NT> union RowsSharedUnion {
    ChunkShared<NT> chunk;
    RowsShared fast;
    SelectShared exact;
    __device__ RowsSharedUnion() {}
};

// Fast term for the running sum: exp2((x - m) * log2 e) on the hardware
// exponential unit.  Only ever summed; every probability that is output uses
// exp_accurate, and the merge replaces the fast terms of the row's largest
// elements (the ones it ranks) by accurate ones.  Its relative error grows with
// |x - m| (the float argument of exp2 carries an absolute rounding error of
// about |x - m| * 2^-24), which is harmless below m, where the term shrinks
// faster than the error grows, and not above it.
__device__ __forceinline__ float fast_term(float x, float m) {
    return __builtin_amdgcn_exp2f((x - m) * 1.44269504088896341f);
}

// The same term with the argument's rounding taken back out: a = fl(d log2 e) goes to
// the hardware unit, and what the rounding dropped (from a fused multiply-add, plus the
// low part of log2 e) comes back as a first-order factor: 2^(a + l) = 2^a (1 + l ln 2),
// |l| < 1e-6.  The hardware unit's one ulp is then all the error there is (fast_term's
// argument alone is good to about |d| 2^-24 absolute: 1.4 ulp of the term at d = -3).
// For rows that few waves sum: one repeated value that carries most of a row's sum and
// is not among the ranked elements puts its term's error, the same every time, into
// every probability of the row -- a flat row with a few peaks came out 4 ulp off with
// fast_term, against a bar of 2; on long rows hundreds of waves with references of their
// own spread that error.  Four instructions more per element.
__device__ __forceinline__ float fast_term_reduced(float x, float m) {
    const float d = x - m;
    constexpr float kHi = 1.44269502162933349609375f;  // float(log2 e)
    constexpr float kLo = 1.925963033500011e-8f;       // log2 e - kHi
    const float a = d * kHi;
    const float l = fmaf(d, kLo, fmaf(d, kHi, -a));  // (d = -inf: NaN, and so is the product below -- see the select)
    const float e = __builtin_amdgcn_exp2f(a);
    const float t = fmaf(e, l * 0.693147180559945309f, e);
    return e > 0.f && e < INFINITY ? t : e;  // (0, inf and NaN as the hardware unit gives them)
}
template <bool REDUCED> __device__ __forceinline__ float fast_term_as(float x, float m) {
    if constexpr (REDUCED) return fast_term_reduced(x, m);
    else return fast_term(x, m);
}

// A wave sums its terms against a reference taken from the first vectors it
// receives, so that the exponentials overlap the loads still in flight: kRefLift
// above the maximum of those vectors.  Should a later element lie more than
// kTermSwitch above that reference (rare on any data with a spread of a few
// units), the wave sums again against its true maximum once everything has
// arrived.  Either way no element is far above the reference its term was taken
// against, the record the wave publishes names that reference, and
// fast_term(x, reference) is what the wave added for x: the merge calls it to
// take back the fast terms of the elements it ranks.
constexpr float kRefLift = 2.0f;
constexpr float kTermSwitch = 1.0f;

// Exact ranking of sh.cand[0..C): sh.rank[i] = number of larger composites.
// All NT threads call with the same C; sh.rank[0..C) must be zero on entry (and a
// barrier must lie between that zeroing and the call); ends with a barrier.
template <int NT> __device__ __forceinline__ void block_rank(RowsShared &sh, uint32_t C) {
    const uint32_t tid = threadIdx.x;
    if (C == 0) return;
    if (C <= NT) {
        // Every candidate has a thread in each of `parts` groups, and a group takes one part of the list.
        // Short lists: groups of P threads, P the power of two at or above C -- shifts only, since a division by
        // a number known at run time is three dozen dependent instructions, as much as the counting itself.
        // Longer lists: groups of exactly C threads (NT = 1024, C = 300: three parts of 100 instead of two of 150).
        uint32_t parts, span, part, i;
        bool live;
        if (C <= 128u) {
            const uint32_t pshift = C > 1u ? 32u - static_cast<uint32_t>(__clz(C - 1u)) : 0u;
            parts = static_cast<uint32_t>(NT) >> pshift;                               // >= 1, a power of two
            span = (C + parts - 1u) >> (31u - static_cast<uint32_t>(__clz(parts)));  // entries per part
            part = tid >> pshift;
            i = tid & ((1u << pshift) - 1u);
            live = i < C;
        } else {
            parts = static_cast<uint32_t>(NT) / C;
            span = (C + parts - 1u) / parts;
            part = tid / C;
            i = tid - part * C;
            live = part < parts;
        }
        if (live) {
            const uint64_t mine = sh.cand[i];
            const uint32_t j0 = part * span, j1 = min(j0 + span, C);
            uint32_t cnt = 0;
            uint32_t j = j0;
            for (; j + 8 <= j1; j += 8) {  // eight independent reads in flight
                uint64_t o[8];
#pragma unroll
                for (int u = 0; u < 8; u++) o[u] = sh.cand[j + u];
#pragma unroll
                for (int u = 0; u < 8; u++) cnt += (o[u] > mine) ? 1u : 0u;
            }
            if (j < j1) {  // the last few, again all at once (past the part's end: entry 0, not counted)
                uint64_t o[8];
#pragma unroll
                for (int u = 0; u < 8; u++) o[u] = sh.cand[j + u < j1 ? j + u : 0u];
#pragma unroll
                for (int u = 0; u < 8; u++) cnt += (j + u < j1 && o[u] > mine) ? 1u : 0u;
            }
            if (parts > 1) {
                if (cnt) atomicAdd(&sh.rank[i], cnt);
            } else {
                sh.rank[i] = cnt;
            }
        }
    } else {
        for (uint32_t i = tid; i < C; i += NT) {
            const uint64_t mine = sh.cand[i];
            uint32_t cnt = 0;
            uint32_t j = 0;
            for (; j + 8 <= C; j += 8) {  // eight independent reads in flight
                uint64_t o[8];
#pragma unroll
                for (int u = 0; u < 8; u++) o[u] = sh.cand[j + u];
#pragma unroll
                for (int u = 0; u < 8; u++) cnt += (o[u] > mine) ? 1u : 0u;
            }
            for (; j < C; j++) cnt += (sh.cand[j] > mine) ? 1u : 0u;
            sh.rank[i] = cnt;
        }
    }
    __syncthreads();
}

// The same for a long list (hundreds of candidates: k of 100 and more), where counting all pairs is LDS bandwidth --
// 1024 threads reading 180 entries each is 4 us on one CU: the candidates are dealt into 256 bins by key
// (equal steps from the smallest key to the largest), and a candidate's rank is the number of candidates in the
// bins above its own -- a suffix sum over the bin counts, by one wave -- plus the larger ones in its own bin, which
// it finds through the bin's list of members (a handful on spread-out data).  A bin with more than kBinnedMax
// members (values equal en masse; a NaN stretching the range) sends the whole list to block_rank instead.
// Uses sh.pidx (bin counts, then the bins' fill marks), sh.pkey (where a bin's members start), sh.lane_key (the
// members, bin by bin from the top), sh.scan_counts: all free until the ranks are known.  Same contract as block_rank.
constexpr uint32_t kBinnedMin = 64;  // lists up to this long are counted pair by pair
constexpr uint32_t kBinnedMax = 48;
template <int NT> __device__ __forceinline__ void block_rank_binned(RowsShared &sh, uint32_t C) {
    constexpr int NW = NT / kWave;
    static_assert(kFastMaxK + 1 >= 512 && kFastCap <= 1024, "bin tables in pidx / pkey, members in lane_key");
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    if (C <= kBinnedMin) {
        block_rank<NT>(sh, C);
        return;
    }
    uint32_t *count = sh.pidx, *mark = sh.pidx + 256, *start = sh.pkey, *member = sh.lane_key;
    // the range of the keys
    uint32_t kmax = 0, kmin = 0xFFFFFFFFu;
    for (uint32_t t = tid; t < C; t += NT) {
        const uint32_t key = static_cast<uint32_t>(sh.cand[t] >> 32);
        kmax = max(kmax, key);
        kmin = min(kmin, key);
    }
    kmax = wave_max_u32(kmax);
    kmin = ~wave_max_u32(~kmin);
    if (lane == 0) {
        sh.scan_counts[wave] = kmax;
        sh.scan_counts[16 + wave] = kmin;
    }
    for (uint32_t t = tid; t < 256u; t += NT) count[t] = 0;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < NW; w++) {
        kmax = max(kmax, sh.scan_counts[w]);
        kmin = min(kmin, sh.scan_counts[16 + w]);
    }
    const uint32_t range = kmax - kmin;
    const uint32_t shift = range < 256u ? 0u : 24u - static_cast<uint32_t>(__clz(range));  // (range >> shift) <= 255
    for (uint32_t t = tid; t < C; t += NT) atomicAdd(&count[(static_cast<uint32_t>(sh.cand[t] >> 32) - kmin) >> shift], 1u);
    __syncthreads();
    if (wave == 0) {
        // lane l takes bins 4 l .. 4 l + 3; start[b] = candidates in the bins above b
        const uint32_t c0 = count[4 * lane], c1 = count[4 * lane + 1], c2 = count[4 * lane + 2], c3 = count[4 * lane + 3];
        const uint32_t mine = c0 + c1 + c2 + c3;
        const uint32_t incl = wave_inclusive_sum_u32(mine);
        const uint32_t total = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(incl), kWave - 1));
        const uint32_t above = total - incl;  // in the lanes above this one
        start[4 * lane + 3] = above;
        start[4 * lane + 2] = above + c3;
        start[4 * lane + 1] = above + c3 + c2;
        start[4 * lane] = above + c3 + c2 + c1;
        mark[4 * lane + 3] = above;
        mark[4 * lane + 2] = above + c3;
        mark[4 * lane + 1] = above + c3 + c2;
        mark[4 * lane] = above + c3 + c2 + c1;
        const uint32_t crowd = wave_max_u32(max(max(c0, c1), max(c2, c3)));
        if (lane == 0) sh.scan_counts[0] = crowd;
    }
    __syncthreads();
    if (sh.scan_counts[0] > kBinnedMax) {  // (the same for every thread)
        __syncthreads();  // (sh.scan_counts is free again)
        block_rank<NT>(sh, C);
        return;
    }
    for (uint32_t t = tid; t < C; t += NT) {
        const uint32_t b = (static_cast<uint32_t>(sh.cand[t] >> 32) - kmin) >> shift;
        member[atomicAdd(&mark[b], 1u)] = t;
    }
    __syncthreads();
    for (uint32_t t = tid; t < C; t += NT) {
        const uint64_t mine = sh.cand[t];
        const uint32_t b = (static_cast<uint32_t>(mine >> 32) - kmin) >> shift;
        const uint32_t j0 = start[b], j1 = j0 + count[b];
        uint32_t r = j0;
        for (uint32_t j = j0; j < j1; j += 4) {  // four members in flight (past the bin's end: the candidate itself, not counted)
            uint32_t m[4];
            uint64_t o[4];
#pragma unroll
            for (int u = 0; u < 4; u++) m[u] = j + u < j1 ? member[j + u] : t;
#pragma unroll
            for (int u = 0; u < 4; u++) o[u] = sh.cand[m[u]];
#pragma unroll
            for (int u = 0; u < 4; u++) r += (o[u] > mine) ? 1u : 0u;
        }
        sh.rank[t] = r;
    }
    __syncthreads();
}

// The same for a list that is followed by zeros up to the power of two P at or above C (a
// zero ranks behind every candidate), 64 <= P <= NT, sh.rank[0..P) zero: every thread takes
// P * P / NT entries, two per LDS read, without a test per entry.  Ends with a barrier.
template <int NT> __device__ __forceinline__ void block_rank_padded(RowsShared &sh, uint32_t C) {
    const uint32_t tid = threadIdx.x;
    const uint32_t pshift = 32u - static_cast<uint32_t>(__clz(C - 1u));  // (C > 32)
    const uint32_t span = (1u << pshift << pshift) / static_cast<uint32_t>(NT);  // entries per thread: 8, 32, 128, 512
    const uint32_t i = tid & ((1u << pshift) - 1u);
    const uint64_t mine = sh.cand[i];
    const uint4 *src = reinterpret_cast<const uint4 *>(sh.cand + (tid >> pshift) * span);
    uint32_t cnt = 0;
    for (uint32_t j = 0; j < span / 2; j += 4) {  // four reads of two entries in flight
        uint4 o[4];
#pragma unroll
        for (int u = 0; u < 4; u++) o[u] = src[j + u];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            cnt += (((static_cast<uint64_t>(o[u].y) << 32) | o[u].x) > mine) ? 1u : 0u;
            cnt += (((static_cast<uint64_t>(o[u].w) << 32) | o[u].z) > mine) ? 1u : 0u;
        }
    }
    if (cnt) atomicAdd(&sh.rank[i], cnt);
    __syncthreads();
}

template <typename T> struct Vec128;
template <> struct Vec128<float> {
    static constexpr int N = 4;
    uint4 v;
    __device__ __forceinline__ void load(const float *p) { v = *reinterpret_cast<const uint4 *>(p); }
    __device__ __forceinline__ float get(int c) const {
        return __uint_as_float(c == 0 ? v.x : c == 1 ? v.y : c == 2 ? v.z : v.w);
    }
    __device__ __forceinline__ void set(int c, float f) {
        const uint32_t u = __float_as_uint(f);
        if (c == 0) v.x = u;
        else if (c == 1) v.y = u;
        else if (c == 2) v.z = u;
        else v.w = u;
    }
};
template <> struct Vec128<uint16_t> {
    static constexpr int N = 8;
    uint4 v;
    __device__ __forceinline__ void load(const uint16_t *p) { v = *reinterpret_cast<const uint4 *>(p); }
    __device__ __forceinline__ float get(int c) const {
        const uint32_t w = (c >> 1) == 0 ? v.x : (c >> 1) == 1 ? v.y : (c >> 1) == 2 ? v.z : v.w;
        return __half2float(__ushort_as_half(static_cast<uint16_t>((c & 1) ? (w >> 16) : (w & 0xFFFFu))));
    }
    __device__ __forceinline__ void set(int c, float f) {  // f is a widened half: exact
        const uint32_t h = __half_as_ushort(__float2half_rn(f));
        uint32_t &w = (c >> 1) == 0 ? v.x : (c >> 1) == 1 ? v.y : (c >> 1) == 2 ? v.z : v.w;
        w = (c & 1) ? ((w & 0x0000FFFFu) | (h << 16)) : ((w & 0xFFFF0000u) | h);
    }
};

// The first `places` elements of a row, in index order, whose order key lies in
// [xlo, xhi]: the row is read from its start, NT * 4 elements at a time, until enough
// are found -- soon, when they are many, which is when this is used.  emit(pos, j) is
// called by the thread that read element j, the pos-th such element (pos < places).
// counts: 2 * NT / 64 words of LDS.  scale: the keys are those of the elements times
// scale (1: as they are).  All NT threads call; returns how many were found (the same
// in every thread; at least `places` unless the row has fewer).
template <typename T, int NT, typename Emit>
__device__ __forceinline__ uint32_t first_members_by_scan(uint32_t *counts, const T *rowp, uint32_t n, uint32_t places,
                                                          uint32_t xlo, uint32_t xhi, float scale, Emit emit) {
    constexpr int NW = NT / kWave;
    constexpr int U = 4;
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    uint32_t found = 0;  // the same in every thread
    uint32_t round = 0;
    for (uint32_t base = 0; base < n && found < places; base += NT * U, round++) {
        const uint32_t j0 = base + tid * U;
        bool member[U];
        uint32_t below = 0, in_wave = 0;
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t j = j0 + u;
            const uint32_t key = order_key(scaled(load_elem(rowp, j < n ? j : 0u), scale));
            member[u] = j < n && key >= xlo && key <= xhi;
            const uint64_t mask = __ballot(member[u]);
            below += lanes_below(mask);
            in_wave += static_cast<uint32_t>(__popcll(mask));
        }
        uint32_t *wc = counts + (round & 1u) * NW;
        if (lane == 0) wc[wave] = in_wave;
        __syncthreads();
        // index order inside the tile: thread, then u
        uint32_t pos = found + below, in_tile = 0;
#pragma unroll
        for (int w = 0; w < NW; w++) {
            const uint32_t c = wc[w];
            pos += (static_cast<uint32_t>(w) < wave) ? c : 0u;
            in_tile += c;
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (member[u]) {
                if (pos < places) emit(pos, j0 + static_cast<uint32_t>(u));
                pos++;
            }
        }
        found += in_tile;
    }
    return found;
}

// The digit d of hist[0..256) with #(entries of digits above d) < need <= #(entries of digits
// >= d), and that first count; one whole wave calls (hist is complete and visible to it).
// d = 256 when the histogram holds fewer than need entries.
__device__ __forceinline__ uint2 hist256_resolve(const uint32_t *hist, uint32_t need) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint4 h4 = reinterpret_cast<const uint4 *>(hist)[lane];  // lane l owns digits 4 l .. 4 l + 3
    const uint32_t h[4] = {h4.x, h4.y, h4.z, h4.w};
    const uint32_t s = (h[0] + h[1]) + (h[2] + h[3]);
    uint32_t incl = s;  // entries of this lane's digits and of the lanes above
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const uint32_t t = __shfl_down(incl, o, kWave);
        if (lane + static_cast<uint32_t>(o) < static_cast<uint32_t>(kWave)) incl += t;
    }
    uint32_t above = incl - s, d = 256u;
    if (above < need && need <= incl) {
#pragma unroll
        for (int j = 3; j >= 0; j--) {
            if (d == 256u) {
                if (need <= above + h[j]) d = lane * 4u + static_cast<uint32_t>(j);
                else above += h[j];
            }
        }
    }
    const uint64_t holder = __ballot(d != 256u);
    const int src = holder != 0ull ? __ffsll(static_cast<unsigned long long>(holder)) - 1 : 0;
    return make_uint2(static_cast<uint32_t>(__shfl(static_cast<int>(d), src, kWave)),
                      static_cast<uint32_t>(__shfl(static_cast<int>(above), src, kWave)));
}

// The same for a row that starts on a 16-byte boundary and is walked far (members
// may be sparse): a thread takes 16 consecutive elements a round (128-bit loads), the
// next round's loads in flight while the current tile is counted, membership by
// two-sided float comparison (a median instruction), one prefix sum over the wave's
// lanes a round.  emit(pos, j, x) also gets the element.  counts: 2 * NT / 64 words of
// LDS.  Keys of the elements as they are (no scale); xhi must not be a NaN's key.
template <typename T, int NT, typename Emit>
__device__ __forceinline__ uint32_t first_members_by_vectors(uint32_t *counts, const T *rowp, uint32_t n, uint32_t places,
                                                             uint32_t xlo, uint32_t xhi, Emit emit) {
    constexpr int NW = NT / kWave, VEC = Vec128<T>::N, U = 16 / VEC;
    constexpr uint32_t per_thread = 16, tile = static_cast<uint32_t>(NT) * per_thread;  // (more a round was measured slower)
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t nv = n - n % VEC;  // the elements that lie in whole vectors
    // x is a member iff flo <= x <= fhi (keys at or below that of -inf: no lower bound); -0 == +0 as in the keys
    const float flo = xlo <= kKeyNegInf ? -INFINITY : ordered_to_float(xlo), fhi = ordered_to_float(xhi);
    Vec128<T> cur[U], nxt[U];
    auto load_tile = [&](Vec128<T>(&q)[U], uint32_t base) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t e0 = base + tid * per_thread + static_cast<uint32_t>(u) * VEC;
            q[u].v = make_uint4(0, 0, 0, 0);
            q[u].load(rowp + (e0 < nv ? e0 : 0u));
        }
    };
    load_tile(cur, 0);
    uint32_t found = 0, round = 0;  // (found: the same in every thread)
    for (uint32_t base = 0; base < nv && found < places; base += tile, round++) {
        const bool more = base + tile < nv;
        if (more) load_tile(nxt, base + tile);
        // index order inside the tile: thread, then its elements
        const uint32_t e_first = base + tid * per_thread;
        uint32_t bits = 0;
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                const float x = cur[u].get(c);
                const bool member = __builtin_amdgcn_fmed3f(x, flo, fhi) == x;  // (false for NaN)
                bits |= member ? (1u << (u * VEC + c)) : 0u;
            }
        }
        // (vectors past the row's end were read from its start)
#pragma unroll
        for (int u = 0; u < U; u++)
            if (e_first + static_cast<uint32_t>(u) * VEC >= nv) bits &= ~(((1u << VEC) - 1u) << (u * VEC));  // (VEC <= 8)
        const uint32_t mine = static_cast<uint32_t>(__popc(bits));
        uint32_t incl = mine;  // members in this lane and the lanes below it
#pragma unroll
        for (int o = 1; o < kWave; o <<= 1) {
            const uint32_t t = __shfl_up(incl, o, kWave);
            if (lane >= static_cast<uint32_t>(o)) incl += t;
        }
        uint32_t *wc = counts + (round & 1u) * NW;
        if (lane == kWave - 1) wc[wave] = incl;
        __syncthreads();
        uint32_t pos = found + incl - mine, in_tile = 0;
#pragma unroll
        for (int w = 0; w < NW; w++) {
            const uint32_t c = wc[w];
            pos += (static_cast<uint32_t>(w) < wave) ? c : 0u;
            in_tile += c;
        }
        if (bits != 0u && pos < places) {
#pragma unroll
            for (int u = 0; u < U; u++) {
#pragma unroll
                for (int c = 0; c < VEC; c++) {
                    if ((bits >> (u * VEC + c)) & 1u) {
                        if (pos < places) emit(pos, e_first + static_cast<uint32_t>(u * VEC + c), cur[u].get(c));
                        pos++;
                    }
                }
            }
        }
        found += in_tile;
        if (more) {
#pragma unroll
            for (int u = 0; u < U; u++) cur[u] = nxt[u];
        }
    }
    if (found < places && nv < n) {
        // the row's last elements, fewer than a vector: every wave counts them, the first one places them
        const uint32_t j = nv + lane;
        const float x = load_elem(rowp, j < n ? j : 0u);
        const bool member = j < n && __builtin_amdgcn_fmed3f(x, flo, fhi) == x;
        const uint64_t mask = __ballot(member);
        const uint32_t pos = found + lanes_below(mask);
        if (member && wave == 0 && pos < places) emit(pos, j, x);
        found += static_cast<uint32_t>(__popcll(mask));
    }
    return found;
}

// Places g0 .. kk-1 of a row's result go to the lowest-index elements whose order
// key lies in [xlo, xhi] (a group of equal rank too large to collect).  SOFTMAX:
// every member's value is tie_value (the group's probability); otherwise the element
// itself.  All NT threads call.
template <typename T, int NT, bool SOFTMAX>
__device__ __forceinline__ void fill_group_by_scan(uint32_t *counts, const T *rowp, T *ov, int32_t *oi, uint32_t n,
                                                   uint32_t g0, uint32_t kk, uint32_t xlo, uint32_t xhi, float tie_value,
                                                   float scale = 1.f) {
    first_members_by_scan<T, NT>(counts, rowp, n, kk - g0, xlo, xhi, scale, [&](uint32_t pos, uint32_t j) {
        if constexpr (SOFTMAX) store_elem(ov, g0 + pos, tie_value);
        else ov[g0 + pos] = rowp[j];
        oi[g0 + pos] = static_cast<int32_t>(j);
    });
}

// The smallest order key whose probability (prob_of_key, non-decreasing in the key) is
// still p_cut, given one key `member` that has it: a 64-way search, one evaluation per
// lane and round.  Called by all 64 lanes of one wave; the same answer in every lane.
template <typename ProbOfKey>
__device__ __forceinline__ uint32_t lowest_key_of_probability(uint32_t member, float p_cut, ProbOfKey prob_of_key) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    // invariant: probability(b) == p_cut, probability(a) < p_cut (a = 0 stands for "below everything")
    uint64_t a = 0, b = member;
    {
        // First the keys b - 1, b - 2, b - 4, ...: the interval is usually a few keys
        // wide (one, for float logits away from 0), and this finds its size class at once.
        const uint32_t off = lane < 32 ? (1u << lane) : 0xFFFFFFFFu;
        const uint64_t probe = b > off ? b - off : 0;
        const bool in = probe != 0 && prob_of_key(static_cast<uint32_t>(probe)) >= p_cut;  // true ... true false ... false
        const int f = __ffsll(static_cast<long long>(~__ballot(in))) - 1;                   // lanes 32.. are false: f >= 0
        a = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(probe)), f));
        if (f > 0) b = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(probe)), f > 0 ? f - 1 : 0));
    }
    while (b - a > 1) {
        const uint64_t step = (b - a + 63) / 64;
        uint64_t probe = a + step * (lane + 1);
        probe = probe < b ? probe : b;
        const bool in = prob_of_key(static_cast<uint32_t>(probe)) >= p_cut;  // false ... false true ... true
        const int f = __ffsll(static_cast<long long>(__ballot(in))) - 1;      // lane 63 probes b: f >= 0
        const uint32_t blo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(probe)), f));
        const uint32_t alo = f > 0 ? static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(probe)), f > 0 ? f - 1 : 0))
                                   : static_cast<uint32_t>(a);
        b = blo;
        a = alo;
    }
    return static_cast<uint32_t>(b);
}

// A probability tie across the k-th place.  Probability is monotone in the logit,
// so the tied group is an interval of logits [x_lo, x_hi]: x_hi is the logit at
// the group's first rank g0, x_lo is found by a 64-way search over order keys (six
// rounds of one exponential per lane).  Elements of that interval that are not
// among the candidates yet (below the merge threshold or their chunk's) are
// fetched from the row, then the k - g0 members with the lowest indices take the
// places g0 .. k-1.  A group that does not fit the candidate array, and the
// group of probability 0 (the underflowed tail of the row and its -inf
// elements), is filled by fill_group_by_scan instead.  Writes those places and
// returns g0.  All NT threads call.
// add_missing(xlo): all threads call it; it appends to sh.cand / sh.count (atomicAdd;
// entries past kFastCap are dropped but counted) every element of the row whose key is
// at least xlo and that is not among the candidates yet, and returns whether it
// touched them (the same value in every thread).
template <typename T, int NT, typename AddMissing>
__device__ __forceinline__ uint32_t settle_tie(RowsShared &sh, AddMissing add_missing, const T *rowp, T *ov, int32_t *oi,
                                               uint32_t n, uint32_t kk, float p_cut, float M, double rinv, float scale = 1.f) {
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    auto prob_of_key = [&](uint32_t key) {
        return round_to_storage<T>(static_cast<float>(static_cast<double>(softmax_term(ordered_to_float(key), M)) * rinv));
    };
    if (tid < kk && sh.prob[tid] == p_cut && (tid == 0 || sh.prob[tid - 1] != p_cut)) sh.g0 = tid;
    if (!(p_cut > 0.f)) {
        // probability 0: every element from the group's largest logit down
        __syncthreads();
        const uint32_t g0 = sh.g0;
        fill_group_by_scan<T, NT, true>(sh.scan_counts, rowp, ov, oi, n, g0, kk, 0u, sh.pkey[g0], p_cut, scale);
        return g0;
    }
    if (tid == 0) sh.members = 0;
    if (wave == 0) {
        const uint32_t b = lowest_key_of_probability(sh.pkey[kk], p_cut, prob_of_key);
        if (lane == 0) sh.xlo = static_cast<uint32_t>(b);
    }
    __syncthreads();
    const uint32_t g0 = sh.g0, xlo = sh.xlo, xhi = sh.pkey[g0];
    // members of the group that are not in the candidate array yet
    if (add_missing(xlo)) __syncthreads();
    const uint32_t C3 = sh.count;
    if (C3 > kFastCap) {
        fill_group_by_scan<T, NT, true>(sh.scan_counts, rowp, ov, oi, n, g0, kk, xlo, xhi, p_cut, scale);
        return g0;
    }
    // the group's members (their indices) side by side, then each counts the members before it
    const uint32_t places = kk - g0;
    for (uint32_t t = tid; t < C3; t += NT) {
        const uint64_t mine = sh.cand[t];
        const uint32_t key = static_cast<uint32_t>(mine >> 32);
        if (key >= xlo && key <= xhi) sh.lane_key[atomicAdd(&sh.members, 1u)] = composite_index(mine);
    }
    __syncthreads();
    const uint32_t members = sh.members;
    for (uint32_t t = tid; t < members; t += NT) {
        const uint32_t idx = sh.lane_key[t];
        uint32_t before = 0;  // members of the group with a lower index
        for (uint32_t u = 0; u < members; u++) before += (sh.lane_key[u] < idx) ? 1u : 0u;
        if (before < places) {
            store_elem(ov, g0 + before, p_cut);
            oi[g0 + before] = static_cast<int32_t>(idx);
        }
    }
    return g0;
}

// ---- from the candidates above the threshold to the row's result ------------------
// sh.cand[0..C2) holds every element of the row at or above some threshold (C2 <=
// kFastCap; `partial`: fewer than k+1 of them, the rest of the row is -inf);
// sh.rank[0..kFastCap) is zero and a barrier lies behind both; M, s_base: the row's
// maximum and its sum of fast terms; sh.ref / sh.scale: per summing wave, its reference
// and exp(ref - M); wave_of(idx): the wave that summed element idx.  Exact ranks (key,
// then lower index); the fast terms of the k+1 ranked elements are replaced by accurate
// ones; probabilities for those only; a probability tie across the k-th place is
// settled over every element of the row with that probability (settle_tie with
// add_missing); ordered store.  scale: the row's elements count times scale (the keys
// of the candidates are those of the scaled elements already).  count_out (softmax
// variant, may be null): receives the nucleus cut of the row's result for top_p -- the
// smallest m >= 1 whose first m probabilities, added in float front to back, reach
// top_p, else kk -- the number topp_count_kernel gives on the stored values.
// All NT threads call.
// REDUCED: the waves summed fast_term_reduced (else fast_term).
template <typename T, int NT, bool SOFTMAX, bool REDUCED = false, typename WaveOf, typename AddMissing>
__device__ __forceinline__ void finish_row(RowsShared &sh, uint32_t C2, bool partial, float M, double s_base, const T *rowp,
                                           T *ov, int32_t *oi, uint32_t n, uint32_t kk, uint32_t want, WaveOf wave_of,
                                           AddMissing add_missing, float scale = 1.f, int32_t *count_out = nullptr,
                                           float top_p = 0.f) {
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1);
    uint32_t tie_g0 = 0xFFFFFFFFu;  // first rank of a group filled on its own (a tie across the k-th place), if any
    // ---- E. exact ranks; accurate terms for the ranked elements ----------------
    BPS(30);
    block_rank_binned<NT>(sh, C2);
    BPS(31);
    // only the k+1 largest are used from here on: which other candidates
    // passed the threshold depends on the order the chunks stored theirs in,
    // and nothing that reaches the output may
    const uint32_t ranked = min(C2, want);
    for (uint32_t t = tid; t < C2; t += NT) {
        const uint32_t r = sh.rank[t];
        if (r < ranked) {
            const uint64_t cmp = sh.cand[t];
            const uint32_t key = static_cast<uint32_t>(cmp >> 32);
            const uint32_t idx = composite_index(cmp);
            sh.pidx[r] = idx;
            sh.pkey[r] = key;
            double cr = 0.0;
            float term = 0.f;  // the element's softmax term, exp(fl(x - M))
            if (SOFTMAX && key != 0xFFFFFFFFu) {
                const uint32_t sp = wave_of(idx);
                const float xv = ordered_to_float(key);
                // what the element should contribute, exp(fl(x - M)), minus what
                // its wave added for it, fast_term(x, ref) * exp(ref - M)
                // (a copy of the value its wave counted apart went in with this very term)
                term = softmax_term(xv, M);
                cr = (xv == sh.x0[sp]) ? 0.0
                                       : static_cast<double>(term) - static_cast<double>(fast_term_as<REDUCED>(xv, sh.ref[sp])) * sh.scale[sp];
            }
            sh.prob[r] = term;  // scaled to a probability below
            sh.corr[r] = cr;
        }
    }
    __syncthreads();
    BPS(32);
    // every wave adds up the corrections itself (same values, same tree, same
    // result, run after run), which saves a trip through LDS and a barrier
    double csum = 0.0;
    for (uint32_t r = lane; r < ranked; r += kWave) csum += sh.corr[r];
    const double total = s_base + wave_sum_f64_uniform(csum);
    if constexpr (SOFTMAX) {
        // the formula of softmax_prob(): the float term scaled in double, rounded once
        const double rinv = 1.0 / total;
        if (tid <= kk && tid < ranked)
            sh.prob[tid] = round_to_storage<T>(static_cast<float>(static_cast<double>(sh.prob[tid]) * rinv));
        __syncthreads();
        BPS(33);
        // Probabilities are non-increasing along the rank order, so equal
        // ones are neighbours.  A tie that reaches past the k-th place is
        // settled by index over every element of the row with that
        // probability, candidates or not.
        if (partial) {
            // the candidates of probability 0, if any, and the -inf elements form one
            // group behind every positive probability: lowest indices first
            if (tid == 0) sh.g0 = C2;
            __syncthreads();
            if (tid < C2 && sh.prob[tid] == 0.f && (tid == 0 || sh.prob[tid - 1] != 0.f)) sh.g0 = tid;
            __syncthreads();
            tie_g0 = sh.g0;
            fill_group_by_scan<T, NT, true>(sh.scan_counts, rowp, ov, oi, n, tie_g0, kk, 0u,
                                            tie_g0 < C2 ? sh.pkey[tie_g0] : kKeyNegInf, 0.f, scale);
        } else if (C2 > kk && sh.prob[kk - 1] == sh.prob[kk]) {
            tie_g0 = settle_tie<T, NT>(sh, add_missing, rowp, ov, oi, n, kk, sh.prob[kk], M, rinv, scale);
        }
    } else if (partial) {
        // the -inf elements follow the candidates, lowest indices first
        tie_g0 = C2;
        fill_group_by_scan<T, NT, false>(sh.scan_counts, rowp, ov, oi, n, C2, kk, kKeyNegInf, kKeyNegInf, 0.f);
    }

    BPS(34);
    const uint32_t plain = min(kk, tie_g0);  // ranks at or after tie_g0 were written by settle_tie
    for (uint32_t r = tid; r < plain; r += NT) {
        const uint32_t idx = sh.pidx[r];
        if constexpr (SOFTMAX) {
            const float p = sh.prob[r];
            // final place inside a run of equal probabilities: by index
            // (rows of few distinct values have runs of hundreds: the run's ends are looked for eight
            // entries a step, not one dependent LDS read after the other; equal logits are in index order
            // already, so a run of one logit -- the usual kind -- needs no count)
            uint32_t lo = r, hi = r, pos = r;
            if (lo > 0 && sh.prob[lo - 1] == p) {
                bool more = true;
                while (more && lo > 0) {
                    float v[8];
#pragma unroll
                    for (int u = 0; u < 8; u++) v[u] = sh.prob[lo > static_cast<uint32_t>(u) ? lo - 1u - u : 0u];
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        const bool same = more && lo > 0 && v[u] == p;  // (v[u] was read for the lo of the step's start)
                        more = same;
                        lo -= same ? 1u : 0u;
                    }
                }
            }
            if (hi + 1 < plain && sh.prob[hi + 1] == p) {
                bool more = true;
                while (more && hi + 1 < plain) {
                    float v[8];
#pragma unroll
                    for (int u = 0; u < 8; u++) v[u] = sh.prob[hi + 1u + u < plain ? hi + 1u + u : plain - 1u];
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        const bool same = more && hi + 1 < plain && v[u] == p;
                        more = same;
                        hi += same ? 1u : 0u;
                    }
                }
            }
            if (hi > lo && (sh.pkey[lo] != sh.pkey[hi])) {
                pos = lo;
                uint32_t q = lo;
                for (; q + 8 <= hi + 1; q += 8) {
                    uint32_t o[8];
#pragma unroll
                    for (int u = 0; u < 8; u++) o[u] = sh.pidx[q + u];
#pragma unroll
                    for (int u = 0; u < 8; u++) pos += (o[u] < idx) ? 1u : 0u;
                }
                for (; q <= hi; q++) pos += (sh.pidx[q] < idx) ? 1u : 0u;
            }
            store_elem(ov, pos, p);
            oi[pos] = static_cast<int32_t>(idx);
        } else {
            ov[r] = rowp[idx];  // bit copy (keeps the sign of a zero)
            oi[r] = static_cast<int32_t>(idx);
        }
    }
    if constexpr (SOFTMAX) {
        if (count_out != nullptr && tid < static_cast<uint32_t>(kWave)) {
            // The stored values in output order: equal probabilities only change places
            // among themselves, so rank order gives the same sequence; from tie_g0 on every
            // place holds the tied group's probability (0 when the row ran out of elements
            // above -inf).  Walked through the lanes in order, as topp_count_kernel does.
            const float tail = (!partial && kk < C2) ? sh.prob[kk] : 0.f;
            const uint32_t count = nucleus_count_wave(kk, top_p, [&](uint32_t r) { return r < plain ? sh.prob[r] : tail; });
            if (lane == 0) *count_out = static_cast<int32_t>(count);
        }
    }
}

// ---- merge of one row's chunk results (all NT threads of a workgroup) --------
// G chunks of `per` elements, each summed and scanned by a workgroup of src_nt
// threads; G << cap_shift <= kMergeRecsMax, G <= kMergeChunksMax,
// G * src_nt / 64 <= kMergeWavesMax (the host checks all three).
// RECS: candidate slots the merge can take in (a multiple of NT).
template <typename T, int NT, bool SOFTMAX, int RECS = kMergeRecsMax, bool REDUCED = false>
__device__ __forceinline__ void merge_row(RowsShared &sh, SelectShared &exact, float *fscratch, double *dscratch,
                                          const T *rowp, T *ov, int32_t *oi, uint32_t n, uint32_t k, uint32_t G,
                                          uint32_t per, uint32_t src_nt, const uint64_t *sums,
                                          const uint64_t *cand, uint32_t cap_shift, float scale = 1.f,
                                          int32_t *count_out = nullptr, float top_p = 0.f) {
    // (scale: the row's elements count times scale -- the candidates' keys are those of the scaled elements
    // already; count_out, top_p: the nucleus cut of the row's result, finish_row)
    constexpr int NW = NT / kWave;
    constexpr int VEC = Vec128<T>::N;
    constexpr int ES = RECS / NT;  // candidate slots per thread
    // (the caller sees to it that there is a thread per wave record and per chunk:
    // G * src_nt / 64 <= NT and G <= NT)
    static_assert(RECS % NT == 0, "whole slots per thread");
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t want = k + 1;
    const uint32_t kk = min(k, n);
    const uint32_t cap = 1u << cap_shift;
    const uint32_t slots = G << cap_shift;
    const uint32_t src_nw = src_nt / kWave;
    const uint32_t waves = G * src_nw;

    // ---- A. everything the merge reads, in one round trip ---------------------------
    // (never a branch around a load: out-of-range threads re-read entry 0)
    const uint32_t wq = tid < waves ? tid : 0u;
    const uint64_t s_bits = fetch(sums + kRecWords * wq);
    const uint64_t rm_bits = fetch(sums + kRecWords * wq + 1);
    const uint64_t c_bits = fetch(sums + kRecWords * wq + 3);
    // thread b < G adds up the candidate counts of chunk b's waves
    // (four loads in flight at a time; a chunk workgroup has 4, 8 or 16 waves)
    uint64_t cm = 0;       // the chunk's candidates, all ones if any of its waves overflowed
    uint32_t cthr = 0;     // the chunk's threshold
    for (uint32_t w0 = 0; w0 < src_nw; w0 += 4) {
        uint64_t c[4];
#pragma unroll
        for (int u = 0; u < 4; u++)  // (a one-wave workgroup has a single record: it is read four times, counted once)
            c[u] = fetch(sums + kRecWords * ((tid < G ? tid : 0u) * src_nw + (w0 + u < src_nw ? w0 + u : 0u)) + 2);
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint32_t cnt = w0 + u < src_nw ? static_cast<uint32_t>(c[u]) : 0u;
            cm = (cnt == 0xFFFFFFFFu || cm == ~0ull) ? ~0ull : cm + cnt;
            cthr = static_cast<uint32_t>(c[u] >> 32);
        }
    }
    // Slot s of the row's lists = entry (s mod cap) + 37 * chunk (mod cap) of chunk s / cap.
    // A chunk fills its list from entry 0, so without the rotation the threads with a
    // small (s mod cap) would hold every live candidate and the others none; with
    // it each thread's slots spread over the positions, every thread holds a few
    // live candidates, and the per-thread maxima below bound the row's (k+1)-th
    // largest much more tightly (fewer candidates left to rank).
    auto slot_pos = [&](uint32_t s) { return ((s & (cap - 1)) + 37u * (s >> cap_shift)) & (cap - 1); };
    uint64_t cv[ES];
#pragma unroll
    for (int e = 0; e < ES; e++) {
        const uint32_t s = static_cast<uint32_t>(e) * NT + tid;
        cv[e] = fetch(cand + (s < slots ? (s & ~(cap - 1)) + slot_pos(s) : 0u));
    }

    // ---- B. the row's maximum and sum from the wave partials --------------------------
    for (uint32_t t = tid; t < static_cast<uint32_t>(kFastCap); t += NT) sh.rank[t] = 0;  // for block_rank, barriers away
    if (tid == 0) {
        sh.count = 0;
        sh.flag = 0;
    }
    bool bad = false;
    SumPartial p0{0.0, 0.f, -INFINITY};
    if (tid < waves) {
        p0.s = __longlong_as_double(static_cast<long long>(s_bits));
        p0.ref = __uint_as_float(static_cast<uint32_t>(rm_bits));
        p0.m = __uint_as_float(static_cast<uint32_t>(rm_bits >> 32));
        sh.ref[tid] = p0.ref;
        sh.x0[tid] = static_cast<uint32_t>(c_bits) != 0u ? __uint_as_float(static_cast<uint32_t>(c_bits >> 32)) : __uint_as_float(0x7FC00000u);
    }
    if (tid < G) {
        sh.cnt[tid] = static_cast<uint32_t>(cm < cap ? cm : cap);
        sh.cthr[tid] = cthr;
        bad = cm > cap;
    }
    // the copies the wave counted apart: each counts exp_accurate(fl(x0 - M)), as the sum is defined
    auto copies_term = [&](float m) -> double {
        const uint32_t cn = (SOFTMAX && tid < waves) ? static_cast<uint32_t>(c_bits) : 0u;
        return cn != 0u ? static_cast<double>(cn) * static_cast<double>(softmax_term(__uint_as_float(static_cast<uint32_t>(c_bits >> 32)), m)) : 0.0;
    };
    // With at most 64 wave records (one per lane of wave 0) that wave alone combines
    // them, by cross-lane steps, while the others go on to the threshold; the
    // results are published by the barrier there.
    if (waves <= static_cast<uint32_t>(kWave)) {
        if (wave == 0) {
            const float m = wave_max_f32_uniform(p0.m);
            double acc = 0.0;
            if (tid < waves) {
                const double sc = sum_rescale(p0.s, p0.ref, m);
                sh.scale[tid] = sc;
                if (SOFTMAX && p0.s != 0.0) acc = p0.s * sc;
            }
            acc += copies_term(m);
            const double total = wave_sum_f64_uniform(acc);
            if (lane == 0) {
                sh.row_max = m;
                sh.total = total;
            }
        }
    } else {
        const float m = block_max_fast<NT>(p0.m, fscratch);  // (barrier: sh.ref is published)
        double acc = 0.0;
        if (tid < waves) {
            const double sc = sum_rescale(p0.s, p0.ref, m);
            sh.scale[tid] = sc;
            if (SOFTMAX && p0.s != 0.0) acc = p0.s * sc;
        }
        acc += copies_term(m);
        const double total = block_sum_fast<NT>(acc, dscratch);  // (barrier: sh.scale is published)
        if (tid == 0) {
            sh.row_max = m;
            sh.total = total;
        }
    }

    // ---- C. threshold: the (k+1)-th largest per-thread maximum -------------------------
    uint32_t lmk = 0;
#pragma unroll
    for (int e = 0; e < ES; e++) {
        // (the unused entries of a list are 0, the chunk kernel sees to that; slots past
        // the row's lists were read from entry 0)
        if (static_cast<uint32_t>(e) * NT + tid >= slots) cv[e] = 0;
        lmk = max(lmk, static_cast<uint32_t>(cv[e] >> 32));
    }
    // Every wave takes, by a ballot descent over its own 64 thread maxima (18 bits),
    // the largest value that its share of k+1 of them reach: the smallest of
    // these bounds is reached by k+1 thread maxima in all, hence by k+1
    // candidates.  (The rotation above keeps the waves alike, so little is lost
    // against the exact (k+1)-th largest.)  A share of more than half a wave, or a
    // wave without enough live threads, leaves it to one wave and all the maxima.
    const uint32_t quota = (want + NW - 1) / NW;
    uint32_t mine_q = 0;
    if (G > 1 && quota <= 32u) {
        for (int bit = 31; bit > 13; bit--) {
            const uint32_t trial = mine_q | (1u << bit);
            if (static_cast<uint32_t>(__popcll(__ballot(lmk >= trial))) >= quota) mine_q = trial;
        }
    }
    sh.lane_key[tid] = lmk;
    if (lane == 0) sh.wave_thr[wave] = mine_q;
    if (bad) sh.flag = 1;  // every writer stores the same value (cleared before the barriers of B)
    __syncthreads();
    const float M = sh.row_max;
    const double s_base = sh.total;
    uint32_t thr = sh.wave_thr[0];
#pragma unroll
    for (int w = 1; w < NW; w++) thr = min(thr, sh.wave_thr[w]);
    // (a single chunk's list is already cut at that chunk's threshold: everything in it is taken)
    if (G > 1 && thr <= 1u) {  // (the same for every thread)
        if (wave == 0) {
            const uint32_t t = block_kth_largest_floor<NW>(sh.lane_key, want, 20);
            if (lane == 0) sh.thr = t > 1u ? t : 1u;  // key 0 is "no element"
        }
        __syncthreads();
        thr = sh.thr;
    }
    if (G == 1) {
        // One chunk: its list is cut at its own threshold, and as a rule everything in it is taken.  Where the
        // list is half as long again as k+1 and more (values equal en masse just below the cut: the chunk's
        // threshold comes from lane maxima), ranking all of it costs more than a threshold among the
        // candidates themselves: the (k+1)-th largest thread maximum, by one wave.
        thr = 1u;
        if (sh.cnt[0] > want + (want >> 1) + 32u) {  // (the same for every thread)
            if (wave == 0) {
                const uint32_t t = block_kth_largest_floor<NW>(sh.lane_key, want, 20);
                if (lane == 0) sh.thr = t > 1u ? t : 1u;
            }
            __syncthreads();
            thr = sh.thr;
        }
    }
    uint32_t merge_thr = thr;  // candidates with keys at or above it are in sh.cand (of equal keys maybe only the first)
    const bool slow = sh.flag != 0u;
    if constexpr (SOFTMAX) {
        if (!(s_base > 0.0 && s_base < static_cast<double>(INFINITY)) || !(M > -INFINITY && M < INFINITY)) {
            // a NaN or +inf element, or nothing above -inf: every probability of the
            // row is NaN, all of them tie, the lowest indices win
            for (uint32_t r = tid; r < kk; r += NT) {
                store_elem(ov, r, __uint_as_float(0x7FC00000u));
                oi[r] = static_cast<int32_t>(r);
            }
            if (count_out != nullptr && tid == 0) *count_out = static_cast<int32_t>(kk);  // (a sum of NaN reaches nothing)
            return;
        }
    }

    if (!slow) {
        // ---- D. the candidates reaching the threshold go to LDS ------------------------
        // (counted per wave with ballots first, so that every one has its place
        // without an atomic and its wait)
        uint32_t wave_n = 0;  // wave-uniform
#pragma unroll
        for (int e = 0; e < ES; e++)
            wave_n += static_cast<uint32_t>(__popcll(__ballot(static_cast<uint32_t>(cv[e] >> 32) >= thr)));
        if (lane == 0) sh.scan_counts[wave] = wave_n;
        __syncthreads();
        uint32_t C2 = 0, pos = 0;
#pragma unroll
        for (int w = 0; w < NW; w++) {
            const uint32_t c = sh.scan_counts[w];
            pos += (static_cast<uint32_t>(w) < wave) ? c : 0u;
            C2 += c;
        }
        if (tid == 0) sh.count = C2;
#pragma unroll
        for (int e = 0; e < ES; e++) {
            const bool pass = static_cast<uint32_t>(cv[e] >> 32) >= thr;
            const uint64_t mask = __ballot(pass);
            if (mask != 0ull) {
                const uint32_t p = pos + lanes_below(mask);
                if (pass && p < kFastCap) sh.cand[p] = cv[e];
                pos += static_cast<uint32_t>(__popcll(mask));
            }
        }
        __syncthreads();
        if (C2 > kFastCap) {
            // Too many reach the threshold (it comes from per-thread maxima and is
            // rounded down; rows full of equal values).  Take the exact cut over all
            // candidates instead: the (k+1)-th largest key, then among the
            // candidates equal to it the ones with the lowest indices -- k+1 of them
            // for the softmax variant (a tie across the k-th place is settled among
            // equal probabilities by index), else as many as make k+1 in all.
            uint32_t round = 0;
            auto count_if = [&](auto pred) -> uint32_t {  // over every candidate of the row; all threads call
                uint32_t c = 0;
#pragma unroll
                for (int e = 0; e < ES; e++) c += static_cast<uint32_t>(__popcll(__ballot(pred(cv[e]))));
                uint32_t *wc = sh.scan_counts + (round & 1u) * NW;
                round++;
                if (lane == 0) wc[wave] = c;
                __syncthreads();
                uint32_t total = 0;
#pragma unroll
                for (int w = 0; w < NW; w++) total += wc[w];
                return total;
            };
            // the key lies in [thr, all ones]: those share the leading ones of thr
            uint32_t cutkey = thr;
            if (thr != 0xFFFFFFFFu) {
                const int d = 31 - __clz(static_cast<int>(~thr));  // highest zero bit of thr
                cutkey = thr & ~((2u << d) - 1u);
                for (int bit = d; bit >= 0; bit--) {
                    const uint32_t trial = cutkey | (1u << bit);
                    if (count_if([&](uint64_t c) { return static_cast<uint32_t>(c >> 32) >= trial; }) >= want) cutkey = trial;
                }
                cutkey = max(cutkey, thr);
            }
            const uint32_t reach = count_if([&](uint64_t c) { return static_cast<uint32_t>(c >> 32) >= cutkey; });
            const uint32_t exceed = count_if([&](uint64_t c) { return static_cast<uint32_t>(c >> 32) > cutkey; });
            const uint32_t keep = SOFTMAX ? exceed + want : want;
            uint64_t cut = static_cast<uint64_t>(cutkey) << 32;
            if (reach > keep) {
                // the keep-th largest composite: descent over the index half
                for (int bit = 31; bit >= 0; bit--) {
                    const uint64_t trial = cut | (1ull << bit);
                    if (count_if([&](uint64_t c) { return c >= trial; }) >= keep) cut = trial;
                }
            }
            __syncthreads();
            if (tid == 0) sh.count = 0;
            __syncthreads();
#pragma unroll
            for (int e = 0; e < ES; e++) {
                if (cv[e] >= cut && cv[e] != 0) {
                    const uint32_t pos = atomicAdd(&sh.count, 1u);
                    if (pos < kFastCap) sh.cand[pos] = cv[e];
                }
            }
            __syncthreads();
            C2 = sh.count;
            merge_thr = cutkey;
        }
        if (C2 <= kFastCap) {
            // Fewer than k+1 candidates: no chunk had k+1 elements above -inf, so every
            // chunk listed all it has and the rest of the row is -inf (probability 0).
            const bool partial = C2 < min(want, n);
            // Members of a tie across the k-th place that are not candidates yet:
            // candidates this workgroup loaded but left below the merge threshold (still
            // in registers), and elements their chunk never listed (below the chunk's
            // threshold: those chunks are read again, which a chunk threshold far below
            // the k-th place never needs).
            auto add_missing = [&](uint32_t xlo) -> bool {
                bool added = false;
                if (xlo < merge_thr) {
#pragma unroll
                    for (int e = 0; e < ES; e++) {
                        const uint32_t key = static_cast<uint32_t>(cv[e] >> 32);
                        if (key >= xlo && key < merge_thr) {
                            const uint32_t pos = atomicAdd(&sh.count, 1u);
                            if (pos < kFastCap) sh.cand[pos] = cv[e];
                        }
                    }
                    added = true;
                }
                for (uint32_t b = 0; b < G; b++) {
                    const uint32_t ct = sh.cthr[b];
                    if (ct <= xlo) continue;  // (same for every thread)
                    const uint32_t c0 = min(b * per, n), c1 = min(c0 + per, n);
                    for (uint32_t j = c0 + tid; j < c1; j += NT) {
                        const uint32_t key = order_key(scaled(load_elem(rowp, j), scale));
                        if (key >= xlo && key < ct) {
                            const uint32_t pos = atomicAdd(&sh.count, 1u);
                            if (pos < kFastCap) sh.cand[pos] = composite(key, j);
                        }
                    }
                    added = true;
                }
                return added;
            };
            // the chunk-kernel wave that summed element idx
            auto wave_of = [&](uint32_t idx) {
                const uint32_t b = idx / per, off = idx - b * per;
                return b * src_nw + ((off / VEC) % src_nt) / kWave;
            };
            finish_row<T, NT, SOFTMAX, REDUCED>(sh, C2, partial, M, s_base, rowp, ov, oi, n, kk, want, wave_of, add_missing, scale,
                                                count_out, top_p);
            return;
        }
    }

    // ---- exact path: radix select over the whole row ----------------------------
#ifdef VKOP_STAMPS
    if (threadIdx.x == 0) atomicAdd(&g_bp_stamps[61], 1ull);
#endif
    __syncthreads();  // LDS changes owner
    if constexpr (SOFTMAX) {
        // redo the statistics the way the general kernels define them
        const LineStats st = line_stats<T, NT>(rowp, 0, n, 1, fscratch, dscratch, scale);
        select_topk_line<NT>(exact, n, kk, [&](uint32_t j) {
            return order_key(round_to_storage<T>(softmax_prob(scaled(load_elem(rowp, j), scale), st)));
        });
        for (uint32_t r = tid; r < kk; r += NT) {
            const uint32_t idx = composite_index(exact.sel[r]);
            store_elem(ov, r, softmax_prob(scaled(load_elem(rowp, idx), scale), st));
            oi[r] = static_cast<int32_t>(idx);
        }
        if (count_out != nullptr) {
            // (rare path: the stored values walked in order by the first wave)
            __syncthreads();
            if (tid < static_cast<uint32_t>(kWave)) {
                const uint32_t count = nucleus_count_wave(kk, top_p, [&](uint32_t r) {
                    return round_to_storage<T>(softmax_prob(scaled(load_elem(rowp, composite_index(exact.sel[r])), scale), st));
                });
                if (tid == 0) *count_out = static_cast<int32_t>(count);
            }
        }
    } else {
        select_topk_line<NT>(exact, n, kk, [&](uint32_t j) { return order_key(load_elem(rowp, j)); });
        for (uint32_t r = tid; r < kk; r += NT) {
            const uint32_t idx = composite_index(exact.sel[r]);
            ov[r] = rowp[idx];
            oi[r] = static_cast<int32_t>(idx);
        }
    }
}

// SOFTMAX = true : fused softmax -> top-k (values are probabilities)
// SOFTMAX = false: plain top-k, largest first (values are copies of the input)
// ALIGNED: every row start is 16-byte aligned and n is a multiple of the vector
// width, so chunks are read with 128-bit loads.
// MERGE: kMergeSplit    -- rows_merge_kernel must follow on the same stream;
//        kMergeByTicket -- the workgroup that publishes a row's last chunk (found
//                          with one counter per row) merges the row before it exits;
//        kMergeLocal    -- one workgroup holds the whole row (G = 1): what the chunk
//                          phase hands to the merge stays in LDS instead of making
//                          the trip through memory.
// Launch: rows * G workgroups of NT threads; per = elements per chunk
// (a multiple of the vector width, per <= NT * V * vector width, G * per >= n).
constexpr int kMergeSplit = 0, kMergeByTicket = 1, kMergeLocal = 2;

// SAMPLING (a row in one workgroup, softmax variant): every element counts times `scale` (one single-precision
// multiplication where it is read), and counts, if not null, receives each row's nucleus cut for top_p.
template <typename T, int NT, int V, bool SOFTMAX, bool ALIGNED, int MERGE, bool SAMPLING = false>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(sizeof(T) == 4 && ALIGNED && NT == 256 && MERGE == kMergeSplit ? 5 : 1))) void rows_chunk_kernel(const T *__restrict__ in, T *__restrict__ values,
                                                        int32_t *__restrict__ indices, uint32_t n, uint32_t k,
                                                        uint32_t G, uint32_t per, RowsWorkspace ws, float scale = 1.f,
                                                        int32_t *__restrict__ counts = nullptr, float top_p = 0.f) {
    static_assert(!SAMPLING || (SOFTMAX && MERGE == kMergeLocal), "the scaled form exists for rows one workgroup holds");
    // an element of a loaded vector, as the row counts it
    auto getq = [&](const Vec128<T> &vec, int c) __attribute__((always_inline)) {
        float x = vec.get(c);
        if constexpr (SAMPLING) x = scaled(x, scale);
        return x;
    };
    constexpr int VEC = Vec128<T>::N;
    constexpr int NW = NT / kWave;
    constexpr int VPP = kWave / VEC;    // staged vectors a wave unpacks per pass (one element per lane)
    constexpr int PASSES = kWave / VPP;  // passes over a full stage of 64 vectors
    constexpr bool FUSED = MERGE != kMergeSplit;
    constexpr bool LOCAL = MERGE == kMergeLocal;
    __shared__ std::conditional_t<FUSED, RowsSharedUnion<NT>, ChunkShared<NT>> smem;
    __shared__ float fscratch[FUSED ? NW : 1];
    __shared__ double dscratch[FUSED ? NW : 1];
    __shared__ uint64_t local_ws[LOCAL ? kLocalCap + kRecWords * NW : 1];  // candidate list, then the wave records
#ifdef VKOP_STAMPS
    const unsigned long long dbg_t0 = wall_clock64();
#endif
    __shared__ uint32_t s_last;
    ChunkShared<NT> *csp;
    if constexpr (FUSED) csp = &smem.chunk;
    else csp = &smem;
    ChunkShared<NT> &cs = *csp;

    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t row = blockIdx.x / G, chunk = blockIdx.x - row * G;
    const uint32_t c0 = min(chunk * per, n), c1 = min(c0 + per, n);
    const T *rowp = in + static_cast<size_t>(row) * n;
    const uint32_t want = k + 1;  // one extra: the merge needs the (k+1)-th to prove the cut
    const uint32_t e_first = c0 + tid * VEC;  // this lane's first element; vector i starts NT * VEC * i later
    const uint32_t went = (row * G + chunk) * NW + wave;  // this wave's slot in the row-major wave list
    if (tid == 0) {
        cs.total = 0;
        cs.over = 0;
    }

    // ---- 1. all loads in flight -----------------------------------------------------
    Vec128<T> q[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        const uint32_t e0 = e_first + static_cast<uint32_t>(i) * NT * VEC;
        // never a branch around a load (the compiler would wait for each one in
        // turn): out-of-chunk lanes read the row's first element(s) instead and
        // are masked wherever the data is used
        q[i].v = make_uint4(0, 0, 0, 0);
        if constexpr (ALIGNED) {
            q[i].load(rowp + (e0 < c1 ? e0 : 0u));
        } else {
#pragma unroll
            for (int c = 0; c < VEC; c++) q[i].set(c, load_elem(rowp, e0 + c < c1 ? e0 + c : 0u));
        }
    }

    // The rest of the chunk phase exists twice: for a chunk that fills every lane
    // of every vector (no masking anywhere) and for a ragged one.
    auto body = [&](auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;
        auto in_range = [&](uint32_t e) { return FULL || e < c1; };

        // ---- 2. per vector, in arrival order: maximum and sum of exp(x - ref) -----------
        // vmax[i]: float max of vector i (NaN dropped) for the softmax variant; for the
        // plain top-k the max of the order keys, so that NaN (which ranks first) counts.
        float vmax[V];
        uint32_t vkey[V];
        // Every term is added in double (fp64 adds run at the fp32 rate here): a
        // dominant term must not swallow the low bits of what the lane adds after it.
        float lmax = -INFINITY, ref = 0.f;
        double acc = 0.0;
        uint32_t lkey = 0u;
        float x0 = __uint_as_float(0x7FC00000u);  // the value whose copies the wave counts apart (NaN: equal to nothing)
        bool counting = false;
        uint32_t counted = 0;  // this lane's copies
        if constexpr (SOFTMAX && LOCAL) {
            // A row in one workgroup is summed by a few waves, and against the ROW's maximum:
            // fl(x - ref) is then the subtraction the softmax definition itself rounds.  (Against
            // a reference of the wave's own, that rounding -- up to 2 ulp of the term at
            // x - ref = -5 -- is an error, the same for every element of one value; where
            // hundreds of waves share a row their references differ and it averages out, here
            // it would not.)  The row is short: waiting for all of it costs little.
            float pm = -INFINITY;
#pragma unroll
            for (int i = 0; i < V; i++) {
                const uint32_t e0 = e_first + static_cast<uint32_t>(i) * NT * VEC;
#pragma unroll
                for (int c = 0; c < VEC; c++) pm = fmaxf(pm, in_range(ALIGNED ? e0 : e0 + c) ? getq(q[i], c) : -INFINITY);
            }
            const float row_max = block_max_fast<NT>(pm, fscratch);
            ref = (row_max > -INFINITY && row_max < INFINITY) ? row_max : 0.f;
        }
#pragma unroll
        for (int i = 0; i < V; i++) {
            const uint32_t e0 = e_first + static_cast<uint32_t>(i) * NT * VEC;
            float xv[VEC];
            float vm = -INFINITY;
            uint32_t vk = 0u;
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                xv[c] = in_range(ALIGNED ? e0 : e0 + c) ? getq(q[i], c) : -INFINITY;
                vm = fmaxf(vm, xv[c]);
                if constexpr (!SOFTMAX) vk = max(vk, in_range(ALIGNED ? e0 : e0 + c) ? order_key(xv[c]) : 0u);
            }
            vmax[i] = vm;
            vkey[i] = vk;
            lmax = fmaxf(lmax, vm);
            lkey = max(lkey, vk);
            if constexpr (SOFTMAX) {
                if (i == 0 && !LOCAL) {
                    // reference of the wave's partial sum: the maximum of its first
                    // vectors; 0 if they hold no finite element (terms are then 0, or
                    // NaN, which must survive -- never -inf - -inf)
                    const float wm0 = wave_max_f32_uniform(vm);
                    ref = (wm0 > -INFINITY) ? wm0 + kRefLift : 0.f;
                    // The copies of one value -- the wave's first element, where half of the lanes' first
                    // elements equal it: a value that fills a row turns up at once -- are counted after the
                    // loop and left out of the sum: every copy has the same term, so its error would enter
                    // the sum once per copy; the merge, which knows the row's maximum, adds
                    // exp_accurate(fl(x0 - M)) for each of them instead.
                    const float first = __uint_as_float(static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(__float_as_uint(xv[0])))));
                    const bool mine = xv[0] == first && first > -INFINITY && first < INFINITY;
                    x0 = first;
                    counting = __popcll(__ballot(mine)) >= kWave / 2;
                }
#pragma unroll
                for (int c = 0; c < VEC; c++) acc += static_cast<double>(fast_term_as<LOCAL>(xv[c], ref));  // (a row in one workgroup: few waves)
            }
        }
        if constexpr (SOFTMAX) lkey = in_range(e_first) ? order_key(lmax) : 0u;
        uint32_t thr_block;

        // ---- 3. the chunk threshold: at least k+1 elements of the chunk reach it -----------
        const float wm = wave_max_f32_uniform(lmax);
        double wsum = 0.0;
        if constexpr (SOFTMAX) wsum = wave_sum_f64_uniform(acc);
        {
            // Every wave finds the q-th largest of its own 64 lane maxima, q = its share
            // of k+1.  The (k+1)-th largest lane maximum of the whole workgroup lies
            // between the smallest and the largest of these, so every wave then
            // settles the few bits in which the two differ over all lane maxima
            // (all waves compute the same value: no broadcast).  A wave short of lane
            // maxima (a ragged chunk) reports 0, which only widens that search.
            const uint32_t quota = (want + NW - 1) / NW;
            uint32_t mine_q = 0;
            if (quota <= static_cast<uint32_t>(kWave)) {
                for (int bit = 31; bit > 15; bit--) {
                    const uint32_t trial = mine_q | (1u << bit);
                    if (static_cast<uint32_t>(__popcll(__ballot(lkey >= trial))) >= quota) mine_q = trial;
                }
            }
            cs.lane_key[tid] = lkey;
            if (lane == 0) cs.wave_thr[wave] = mine_q;
            __syncthreads();
            uint32_t lo = cs.wave_thr[0], hi = lo;
#pragma unroll
            for (int w = 1; w < NW; w++) {
                lo = min(lo, cs.wave_thr[w]);
                hi = max(hi, cs.wave_thr[w]);
            }
            uint32_t t = lo;
            if (lo != hi) {
                uint32_t kv[NW];
#pragma unroll
                for (int w = 0; w < NW; w++) kv[w] = cs.lane_key[w * kWave + lane];
                const int d = 31 - __clz(static_cast<int>(lo ^ hi));  // highest bit in which they differ
                t = hi & ~((2u << d) - 1u);                            // their common prefix
                for (int bit = d; bit > 15; bit--) {
                    const uint32_t trial = t | (1u << bit);
                    uint32_t cnt = 0;
#pragma unroll
                    for (int w = 0; w < NW; w++) cnt += static_cast<uint32_t>(__popcll(__ballot(kv[w] >= trial)));
                    if (cnt >= want) t = trial;
                }
            }
            thr_block = t;
        }
        // -inf never becomes a candidate: a row with k+1 larger elements does not
        // need it, and any other row is left to the exact path
        uint32_t thr = max(thr_block, kKeyNegInf + 1u);

        // ---- 4. the elements at or above the threshold go to the chunk's candidate list --------
        // Returns the wave's count (all ones if the wave had more than 64 vectors to stage;
        // staged_vectors = how many it staged).
        uint64_t *cand_out;
        if constexpr (LOCAL) cand_out = local_ws;
        else cand_out = ws.cand + (static_cast<size_t>(row * G + chunk) << ws.cap_shift);
        uint64_t *record;  // this wave's
        if constexpr (LOCAL) record = local_ws + kLocalCap + kRecWords * wave;
        else record = ws.sums + kRecWords * static_cast<size_t>(went);
        uint4 *stv = cs.stage_v + wave * kWave;
        uint32_t *ste = cs.stage_e + wave * kWave;
        auto compact = [&](uint32_t thr_key, uint32_t &staged_vectors) -> uint32_t {
            const float thr_f = ordered_to_float(thr_key);
            // 4a. the wave's vectors holding such an element -> LDS
            uint32_t nv = 0;  // wave-uniform
#pragma unroll
            for (int i = 0; i < V; i++) {
                const uint32_t e0 = e_first + static_cast<uint32_t>(i) * NT * VEC;
                bool hit;
                if constexpr (SOFTMAX) hit = !(vmax[i] < thr_f) && in_range(e0);
                else hit = vkey[i] >= thr_key && in_range(e0);
                const uint64_t mask = __ballot(hit);
                if (mask != 0ull) {
                    if (hit) {
                        const uint32_t pos = nv + lanes_below(mask);
                        if (pos < kWave) {
                            stv[pos] = q[i].v;
                            ste[pos] = e0;
                        }
                    }
                    nv += static_cast<uint32_t>(__popcll(mask));
                }
            }
            const bool over = nv > kWave;
            nv = min(nv, static_cast<uint32_t>(kWave));
            staged_vectors = nv;
            __builtin_amdgcn_wave_barrier();  // the stage is read by other lanes of the same wave

            // 4b. one element per lane: keep those at or above the threshold
            uint64_t mine[PASSES];
            uint32_t mpos[PASSES];
            uint32_t wcount = 0;  // wave-uniform
#pragma unroll
            for (int p = 0; p < PASSES; p++) {
                mine[p] = 0;  // 0 = nothing to write
                mpos[p] = 0;
                if (static_cast<uint32_t>(p) * VPP < nv) {
                    const uint32_t sv = static_cast<uint32_t>(p) * VPP + lane / VEC;
                    const bool live = sv < nv;
                    Vec128<T> r;
                    r.v = stv[live ? sv : 0u];
                    const uint32_t idx = ste[live ? sv : 0u] + (lane % VEC);
                    const float x = getq(r, static_cast<int>(lane % VEC));
                    const uint32_t key = order_key(x);
                    const bool pass = live && idx < c1 && key >= thr_key;
                    const uint64_t mask = __ballot(pass);
                    if (pass) {
                        mine[p] = composite(key, idx);
                        mpos[p] = wcount + lanes_below(mask);
                    }
                    wcount += static_cast<uint32_t>(__popcll(mask));
                }
            }
            // room in the chunk's candidate list, reserved once per wave
            uint32_t base = 0;
            if (lane == 0) {
                base = atomicAdd(&cs.total, wcount);
                if (over) cs.over = 1;
            }
            base = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(base)));
#pragma unroll
            for (int p = 0; p < PASSES; p++) {
                const uint32_t pos = base + mpos[p];
                if (mine[p] != 0 && pos < ws.cap) publish(cand_out + pos, mine[p]);
            }
            return over ? 0xFFFFFFFFu : wcount;
        };
        uint32_t staged = 0;
        BPS(48);
        uint32_t wave_candidates = compact(thr, staged);
        BPS(49);

        // ---- the wave's partial sum (here, so that none of it is live across what follows) ------
        uint32_t copies = 0;  // wave-uniform: the copies of x0 the sum leaves out
        if constexpr (SOFTMAX && !LOCAL) {
            if (counting) {  // (wave-uniform; everything is still in registers)
                uint32_t ncopy = 0;
#pragma unroll
                for (int i = 0; i < V; i++) {
                    const uint32_t e0 = e_first + static_cast<uint32_t>(i) * NT * VEC;
#pragma unroll
                    for (int c = 0; c < VEC; c++) ncopy += (in_range(ALIGNED ? e0 : e0 + c) && getq(q[i], c) == x0) ? 1u : 0u;
                }
                // (every copy added the same float: taking them out again is exact to the sum's own rounding)
                if (ncopy != 0u) acc -= static_cast<double>(ncopy) * static_cast<double>(fast_term(x0, ref));
                wsum = wave_sum_f64_uniform(acc);
                copies = static_cast<uint32_t>(wave_sum_f64_uniform(static_cast<double>(ncopy)));
                counted = ncopy;
            }
        }
        if constexpr (SOFTMAX) {
            if (wm - ref > kTermSwitch) {  // wave-uniform
                // an element well above the reference: its fast term is poor (or has
                // overflowed); everything is in registers, so sum again against the maximum
                ref = (wm < INFINITY) ? wm : ref;
                acc = 0.0;
#pragma unroll
                for (int i = 0; i < V; i++) {
                    const uint32_t e0 = e_first + static_cast<uint32_t>(i) * NT * VEC;
#pragma unroll
                    for (int c = 0; c < VEC; c++) {
                        const float x = in_range(ALIGNED ? e0 : e0 + c) ? getq(q[i], c) : -INFINITY;
                        acc += static_cast<double>(fast_term_as<LOCAL>(x, ref));
                    }
                }
                if (counted != 0u) acc -= static_cast<double>(counted) * static_cast<double>(fast_term(x0, ref));
                wsum = wave_sum_f64_uniform(acc);
            }
        }
        if (lane == 0) {
            publish(record, static_cast<uint64_t>(__double_as_longlong(wsum)));
            publish(record + 1, (static_cast<uint64_t>(__float_as_uint(wm)) << 32) | __float_as_uint(ref));
            publish(record + 3, (static_cast<uint64_t>(__float_as_uint(x0)) << 32) | copies);
        }
        __syncthreads();
        const bool too_many = cs.total > ws.cap || cs.over != 0u;  // (the same in every thread)
        if (__builtin_expect(too_many, 0)) {
            // Too many.  The lane maxima give a loose bound when values in order or in
            // clusters put many large elements into few lanes, or when many are equal.
            // The list is made once more, with the exact (k+1)-th largest element of
            // the chunk as the threshold.  It lies between the bound just used and the
            // chunk's maximum: a descent over the bits in which the two differ, counting
            // over the staged elements (everything at or above the old bound is among
            // them) or, if a wave's stage was too small, over every element held in
            // registers.  Of the elements equal to that value only the first k+1 (by
            // index) are listed, so that no number of equal values overflows the list:
            // the others cannot reach the row's result, k+1 elements of this chunk come
            // before each.
            // (Keys are derived from the loaded vectors at every use: the empty asm keeps
            // the compiler from holding them all in registers, which would cost the whole
            // kernel waves per SIMD for the sake of this path.)
            auto key_of = [&](int i, int c) {
                const uint32_t e0 = e_first + static_cast<uint32_t>(i) * NT * VEC;
                float x = getq(q[i], c);
                asm volatile("" : "+v"(x));
                return in_range(ALIGNED ? e0 : e0 + c) ? order_key(x) : 0u;
            };
            const bool from_stage = cs.over == 0u;
            // (a short row in a workgroup shaped for longer ones -- 8400 elements, 1024 threads, V = 8 -- has
            // vectors no thread holds anything of: the passes below leave them out, the same in every thread)
            const int v_used = static_cast<int>(min(static_cast<uint32_t>(V), (c1 - c0 + NT * VEC - 1u) / (NT * VEC)));
            // Values in order (a sorted row, a row sorted in runs) put many large elements into few lanes, and
            // the bound from the lane maxima is then far too low.  On such a row the elements of a VECTOR are
            // alike, and every element of a vector reaches the vector's minimum: with q = ceil((k+1) / width)
            // lanes that hold a vector whose minimum reaches T, k+1 elements reach T.  The q-th largest of the
            // lanes' largest vector minima is such a T (its leading 24 bits: lower, so still reached) -- close
            // under the cut on a row in order, useless, and then not used, on any other.  Where it beats the
            // bound, everything at or above it is listed straight away if that fits (first turn of the loop
            // below), and only otherwise the exact cut is looked for (second turn).
            bool tight = false;
            if (tid < 40) cs.refine[tid] = (tid >= 32 && (tid & 1u) == 0u) ? 0xFFFFFFFFu : 0u;
            {
                uint32_t a = 0;
#pragma unroll
                for (int i = 0; i < V; i++) {
                    if (i >= v_used) continue;
                    const uint32_t e0 = e_first + static_cast<uint32_t>(i) * NT * VEC;
                    float vm = INFINITY;  // (a NaN is dropped: it ranks above everything, the others' minimum still holds)
#pragma unroll
                    for (int c = 0; c < VEC; c++) {
                        float x = getq(q[i], c);
                        asm volatile("" : "+v"(x));
                        vm = fminf(vm, in_range(ALIGNED ? e0 : e0 + c) ? x : -INFINITY);
                    }
                    a = max(a, vm == vm ? order_key(vm) : 0u);
                }
                cs.lane_key[tid] = a;
                const uint32_t qn = (want + VEC - 1u) / VEC;
                __syncthreads();
                // (q lanes must beat the bound for T to: counted first, which is all a row not in order pays)
                const uint32_t beat = static_cast<uint32_t>(__popcll(__ballot(a > thr)));
                if (lane == 0 && beat) atomicAdd(&cs.refine[39], beat);
                __syncthreads();
                if (cs.refine[39] >= qn) {  // (the same in every thread)
                    if (wave == 0) {
                        const uint32_t t = block_kth_largest_floor<NW>(cs.lane_key, qn, 24);
                        if (lane == 0) cs.thr = t;
                    }
                    __syncthreads();
                    const uint32_t tmin = cs.thr;
                    tight = tmin > thr;
                    if (tight) thr = tmin;
                    __syncthreads();  // (cs.thr and cs.lane_key are free again)
                }
            }
#pragma unroll 1
            for (int turn = tight ? 0 : 1; turn < 2; turn++) {
            const bool exact = turn == 1;
            if (exact) {
            uint32_t wk = 0;
#pragma unroll
            for (int i = 0; i < V; i++) {
                if (i >= v_used) continue;
#pragma unroll
                for (int c = 0; c < VEC; c++) wk = max(wk, key_of(i, c));
            }
            wk = wave_max_u32(wk);
            if (lane == 0) cs.wave_thr[wave] = wk;
            __syncthreads();
            uint32_t hi = cs.wave_thr[0];
#pragma unroll
            for (int w = 1; w < NW; w++) hi = max(hi, cs.wave_thr[w]);
            // count(trial): elements of this wave at or above trial (wave-uniform)
            // floor_at(t): the smallest key at or above t among this lane's elements (all ones if none)
            auto exact_threshold = [&](auto count, auto floor_at) -> uint32_t {
                if (thr >= hi) return thr;
                // Equal values en masse first (a row of few distinct values): the smallest key at or
                // above the bound is then the answer -- k+1 elements reach it, fewer exceed it -- and
                // costs two passes over the elements instead of one per bit.
                uint32_t lb = thr;
                const uint32_t wmin = ~wave_max_u32(~floor_at(thr));
                if (lane == 0) atomicMin(&cs.refine[32], wmin);
                __syncthreads();
                const uint32_t t0 = cs.refine[32];
                if (t0 < hi) {  // (the same in every thread; t0 >= thr)
                    const uint32_t c = count(t0 + 1u);
                    if (lane == 0 && c) atomicAdd(&cs.refine[33], c);
                    __syncthreads();
                    if (cs.refine[33] < want) return t0;
                    lb = t0 + 1u;  // k+1 elements reach it
                }
                if (lb >= hi) return lb;
                const int d = 31 - __clz(static_cast<int>(lb ^ hi));  // highest bit in which they differ
                uint32_t t = hi & ~((2u << d) - 1u);                   // their common prefix
                for (int bit = d; bit >= 0; bit--) {
                    const uint32_t trial = t | (1u << bit);
                    const uint32_t c = count(trial);
                    if (lane == 0 && c) atomicAdd(&cs.refine[bit], c);
                    __syncthreads();
                    if (cs.refine[bit] >= want) t = trial;
                }
                return max(t, lb);
            };
            BPS(55);
            if (from_stage) {
                uint32_t keys[PASSES];
#pragma unroll
                for (int p = 0; p < PASSES; p++) {
                    const uint32_t sv = static_cast<uint32_t>(p) * VPP + lane / VEC;
                    const bool live = sv < staged;
                    Vec128<T> r;
                    r.v = stv[live ? sv : 0u];
                    const uint32_t idx = ste[live ? sv : 0u] + (lane % VEC);
                    keys[p] = (live && idx < c1) ? order_key(getq(r, static_cast<int>(lane % VEC))) : 0u;
                }
                thr = exact_threshold([&](uint32_t trial) {
                    uint32_t c = 0;
#pragma unroll
                    for (int p = 0; p < PASSES; p++) c += static_cast<uint32_t>(__popcll(__ballot(keys[p] >= trial)));
                    return c;
                }, [&](uint32_t t) {
                    uint32_t f = 0xFFFFFFFFu;
#pragma unroll
                    for (int p = 0; p < PASSES; p++) f = keys[p] >= t ? min(f, keys[p]) : f;
                    return f;
                });
            } else if (thr < hi) {
                // Every element held in registers: a radix select over the keys, eight bits a
                // pass, counted in LDS (lanes that share a digit add once) -- four passes whatever
                // the values, where a descent over the bits in which bound and maximum differ
                // takes up to two dozen (a pass costs the same either way: the keys are derived
                // from the loaded vectors again).  Rows of few distinct values first: the
                // smallest key at or above the bound is their answer -- k+1 elements reach it,
                // fewer exceed it.
                static_assert(sizeof(cs.stage_v) >= 256 * sizeof(uint32_t), "the digit counts take 256 words");
                uint32_t *hist = reinterpret_cast<uint32_t *>(cs.stage_v);  // (the stage is filled anew afterwards)
                // (up to three distinct values from the bound up: the lane maxima of a row of a dozen levels
                // put the bound a level or two under the cut, and a step costs two passes where the radix
                // select costs eight)
                uint32_t lb = thr;
                bool settled = false, levels = true;
                uint32_t reach = cs.total;  // elements at or above lb (at least: a wave whose stage overflowed counted short)
#pragma unroll 1
                for (uint32_t step = 0; step < 3u && !settled && levels; step++) {
                    uint32_t f = 0xFFFFFFFFu, above = 0;
#pragma unroll
                    for (int i = 0; i < V; i++) {
                        if (i >= v_used) continue;
#pragma unroll
                        for (int cc = 0; cc < VEC; cc++) {
                            const uint32_t kx = key_of(i, cc);
                            f = kx >= lb ? min(f, kx) : f;
                        }
                    }
                    f = ~wave_max_u32(~f);
                    if (lane == 0) atomicMin(&cs.refine[32 + 2 * step], f);
                    __syncthreads();
                    const uint32_t t0 = cs.refine[32 + 2 * step];  // (>= lb: the same in every thread)
#pragma unroll
                    for (int i = 0; i < V; i++) {
                        if (i >= v_used) continue;
#pragma unroll
                        for (int cc = 0; cc < VEC; cc++) above += static_cast<uint32_t>(__popcll(__ballot(key_of(i, cc) > t0)));
                    }
                    if (lane == 0 && above) atomicAdd(&cs.refine[33 + 2 * step], above);
                    __syncthreads();
                    if (cs.refine[33 + 2 * step] < want) {
                        thr = t0;  // k+1 elements reach it, fewer exceed it
                        settled = true;
                    } else {
                        lb = t0 + 1u;  // (t0 < the row's maximum: k+1 elements exceed it)
                        // a value that few elements have: not a row of levels, the next value up will not be the cut either
                        const uint32_t exceed = cs.refine[33 + 2 * step];
                        levels = reach >= exceed + 8u;
                        reach = exceed;
                    }
                }
                if (!settled) {
                    thr = lb;  // k+1 elements reach it
                    uint32_t prefix = 0, need = want;
                    for (int shift = 24; shift >= 0; shift -= 8) {
                        __syncthreads();  // (the last pass's answer has been read)
                        if (tid < 256u) hist[tid] = 0;
                        __syncthreads();
#pragma unroll
                        for (int i = 0; i < V; i++) {
                            if (i >= v_used) continue;
#pragma unroll
                            for (int cc = 0; cc < VEC; cc++) {
                                const uint32_t kx = key_of(i, cc);  // (0 past the chunk's end: the lowest digit, below every element)
                                if ((static_cast<uint64_t>(kx ^ prefix) >> (shift + 8)) == 0ull) hist_add_grouped(hist, (kx >> shift) & 255u);
                            }
                        }
                        __syncthreads();
                        if (wave == 0) {
                            const uint2 r = hist256_resolve(hist, need);
                            if (lane == 0) {
                                cs.refine[32] = r.x;
                                cs.refine[33] = r.y;
                            }
                        }
                        __syncthreads();
                        prefix |= (cs.refine[32] & 255u) << shift;  // (a digit is always found: the chunk holds k+1 elements at or above thr)
                        need -= cs.refine[33];
                    }
                    thr = max(thr, prefix);
                }
            }
            BPS(50);
            BPS(51);
            }
            drain_stores();  // the first attempt's stores have landed before the same slots are written again
            __syncthreads();  // (and every wave is done with its stage)
            // The list, straight from the registers -- not through the waves' stages of 64 vectors, which a sorted
            // row, whose candidates all sit in one wave's elements, would overflow again: everything above thr and,
            // of the elements equal to it, the first k+1 in index order (the exact turn; at most 2 k + 1 entries) or
            // all of them (the other turn).  Elements are in index order by (vector, wave, lane, position in the
            // vector), so three tables with an entry per (vector, wave) say it all: the entry's elements above thr,
            // its elements equal to thr, and -- from a prefix over those -- how many of the equal ones are still
            // wanted when the entry begins.  One pass over the registers fills the tables, a second writes; only the
            // ONE entry that holds the last wanted equal element looks at positions inside itself.
            {
                static_assert(3 * V * NW <= NT, "three tables of an entry per (vector, wave)");
                static_assert(V * NW <= 2 * kWave, "a table takes at most two waves");
                constexpr uint32_t VN = static_cast<uint32_t>(V * NW);
                uint32_t *tie_tab = cs.lane_key, *lst_tab = cs.lane_key + VN, *abv_tab = cs.lane_key + 2 * VN;
                const uint32_t want_ties = exact ? want : 0xFFFFFFFFu;
#pragma unroll
                for (int i = 0; i < V; i++) {
                    uint32_t ties = 0, abv = 0;
                    if (i < v_used) {
#pragma unroll
                        for (int c = 0; c < VEC; c++) {
                            const uint32_t kx = key_of(i, c);
                            ties += static_cast<uint32_t>(__popcll(__ballot(kx == thr)));
                            abv += static_cast<uint32_t>(__popcll(__ballot(kx > thr)));
                        }
                    }
                    if (lane == 0) {
                        tie_tab[i * NW + wave] = ties;
                        abv_tab[i * NW + wave] = abv;
                    }
                }
                __syncthreads();
                // prefix over the equal ones (a scan over the lanes of each of the table's waves, the second adding
                // the first one's total), then over what each entry lists
                const uint32_t mine_ties = tid < VN ? tie_tab[tid] : 0u;
                const uint32_t mine_abv = tid < VN ? abv_tab[tid] : 0u;
                const uint32_t incl_t = wave_inclusive_sum_u32(mine_ties);
                uint32_t ties_before = incl_t - mine_ties;
                if (tid == static_cast<uint32_t>(kWave) - 1u) cs.refine[32] = incl_t;
                __syncthreads();
                if (tid >= static_cast<uint32_t>(kWave)) ties_before += cs.refine[32];
                const uint32_t room = want_ties > ties_before ? want_ties - ties_before : 0u;
                const uint32_t mine_lst = min(mine_ties, room);
                const uint32_t mine_cnt = tid < VN ? mine_abv + mine_lst : 0u;
                const uint32_t incl_c = wave_inclusive_sum_u32(mine_cnt);
                uint32_t before_mine = incl_c - mine_cnt;
                if (tid == static_cast<uint32_t>(kWave) - 1u) cs.refine[33] = incl_c;
                __syncthreads();
                if (tid >= static_cast<uint32_t>(kWave)) before_mine += cs.refine[33];
                if (tid < VN) {
                    if (tid == VN - 1u) cs.total = before_mine + mine_cnt;
                    lst_tab[tid] = mine_lst;
                    abv_tab[tid] = before_mine;  // (from here on: the entry's first place in the list)
                }
                if (tid == 0) cs.over = 0;
                __syncthreads();
                if (!exact && cs.total > ws.cap) {  // (the same in every thread: on to the exact cut)
                    __syncthreads();
                    continue;
                }
                uint32_t wave_total = 0;  // wave-uniform
#pragma unroll
                for (int i = 0; i < V; i++) {
                    if (i >= v_used) continue;
                    const uint32_t e0 = e_first + static_cast<uint32_t>(i) * NT * VEC;
                    const uint32_t n_ties = tie_tab[i * NW + wave], n_lst = lst_tab[i * NW + wave];
                    uint32_t pos = abv_tab[i * NW + wave];
                    uint32_t kxs[VEC];
                    uint32_t tie_at = 0;  // this lane's first equal element's place among the entry's equal ones
#pragma unroll
                    for (int c = 0; c < VEC; c++) kxs[c] = key_of(i, c);
                    const bool partly = n_lst != 0u && n_lst < n_ties;  // (wave-uniform; one entry of a row at most)
                    if (partly) {
#pragma unroll
                        for (int c = 0; c < VEC; c++) tie_at += lanes_below(__ballot(kxs[c] == thr));
                    }
#pragma unroll
                    for (int c = 0; c < VEC; c++) {
                        const bool tie = kxs[c] == thr;
                        const bool pass = kxs[c] > thr || (tie && (partly ? tie_at < n_lst : n_lst != 0u));
                        if (partly && tie) tie_at++;
                        const uint64_t mask = __ballot(pass);
                        if (mask != 0ull) {
                            const uint32_t at = pos + lanes_below(mask);
                            if (pass && at < ws.cap) publish(cand_out + at, composite(kxs[c], e0 + c));
                            pos += static_cast<uint32_t>(__popcll(mask));
                            wave_total += static_cast<uint32_t>(__popcll(mask));
                        }
                    }
                }
                wave_candidates = wave_total;
            }
            break;
            }
            __syncthreads();  // (cs.total is final)
            BPS(52);
        }
        // the unused entries of the list read as "no element": the merge tells live
        // candidates from stale ones by that alone
        for (uint32_t p = min(cs.total, ws.cap) + tid; p < ws.cap; p += NT) publish(cand_out + p, 0ull);

        // ---- 5. the chunk's threshold and the wave's candidate count -------------------------------
        if (lane == 0) {
            publish(record + 2, (static_cast<uint64_t>(thr) << 32) | static_cast<uint64_t>(wave_candidates));
        }
    };
    if (c1 - c0 == static_cast<uint32_t>(NT) * V * VEC) body(std::true_type{});
    else body(std::false_type{});

    // ---- 6. one-kernel variant: the row's last chunk merges ------------------------------------
    // (otherwise the workgroup is done: the merge kernel adds up the waves' counts itself)
    if constexpr (MERGE == kMergeByTicket) {
        drain_stores();
        __syncthreads();  // every thread's published values are visible device-wide
        if (tid == 0) {
            uint32_t last = 1;
            if (G > 1) {
                const uint32_t done = __hip_atomic_fetch_add(ws.tickets + row, 1u, __ATOMIC_RELAXED,
                                                             __HIP_MEMORY_SCOPE_AGENT);
                last = (done == G - 1) ? 1u : 0u;
                // ready for the next call (nobody else touches this row's counter any more)
                if (last) __hip_atomic_store(ws.tickets + row, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            s_last = last;
        }
    }
    if constexpr (LOCAL) {
        __syncthreads();  // the list and the records are in LDS; so is what the merge builds, in other arrays
        BPS(53);
        merge_row<T, NT, SOFTMAX, kLocalCap, true>(smem.fast, smem.exact, fscratch, dscratch, rowp,
                                             values + static_cast<size_t>(row) * k, indices + static_cast<size_t>(row) * k, n, k,
                                             1u, per, NT, local_ws + kLocalCap, local_ws, ws.cap_shift, SAMPLING ? scale : 1.f,
                                             (SAMPLING && counts != nullptr) ? counts + row : nullptr, top_p);
        BPS(54);
#ifdef VKOP_STAMPS
        if (threadIdx.x == 0) {
            atomicMax(&g_bp_stamps[60], wall_clock64() - dbg_t0);
            atomicAdd(&g_bp_stamps[62], 1ull);
        }
#endif
        (void)s_last;
    } else if constexpr (FUSED) {
        __syncthreads();
        if (s_last == 0u) return;
        merge_row<T, NT, SOFTMAX>(smem.fast, smem.exact, fscratch, dscratch, rowp, values + static_cast<size_t>(row) * k,
                                  indices + static_cast<size_t>(row) * k, n, k, G, per, NT,
                                  ws.sums + kRecWords * static_cast<size_t>(row) * G * NW,
                                  ws.cand + (static_cast<size_t>(row) * G << ws.cap_shift), ws.cap_shift);
    } else {
        (void)values;
        (void)indices;
        (void)fscratch;
        (void)dscratch;
    }
}

union MergeShared {
    RowsShared fast;
    SelectShared exact;
    __device__ MergeShared() {}
};

// Second kernel of the unfused variant: one workgroup of kMergeThreads per row.
// RECS: candidate slots it takes in, at least G * cap (1024, 2048 or kMergeRecsMax:
// the smallest that holds the row's lists keeps the per-thread loops short).
template <typename T, bool SOFTMAX, int RECS>
__global__ __launch_bounds__(kMergeThreads) void rows_merge_kernel(const T *__restrict__ in, T *__restrict__ values,
                                                                   int32_t *__restrict__ indices, uint32_t n,
                                                                   uint32_t k, uint32_t G, uint32_t per,
                                                                   uint32_t src_nt, RowsWorkspace ws) {
    __shared__ MergeShared smem;
    __shared__ float fscratch[kMergeThreads / kWave];
    __shared__ double dscratch[kMergeThreads / kWave];
    const uint32_t row = blockIdx.x;
    merge_row<T, kMergeThreads, SOFTMAX, RECS>(smem.fast, smem.exact, fscratch, dscratch, in + static_cast<size_t>(row) * n,
                                         values + static_cast<size_t>(row) * k, indices + static_cast<size_t>(row) * k,
                                         n, k, G, per, src_nt,
                                         ws.sums + kRecWords * static_cast<size_t>(row) * G * (src_nt / kWave),
                                         ws.cand + (static_cast<size_t>(row) * G << ws.cap_shift), ws.cap_shift);
}

}  // namespace vkop
