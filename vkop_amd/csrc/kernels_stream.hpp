// Long contiguous rows split over several workgroups: the streaming pass.
//
// rows_scan_kernel reads the input once and does nothing with an element but what
// every element needs: it goes into the maximum of its BLOCK -- 16 consecutive
// 128-bit vectors of the row, 256 bytes, what 16 neighbouring lanes read with one
// load -- and, for the softmax variant, into the wave's sum of exp(x - ref).  It
// writes one order key per block and one record per wave.  No threshold, no
// compaction, no barrier: the pass is issue-bound on this chip (every instruction of
// every wave costs four cycles of its SIMD), so whatever only a few elements need is
// left to the kernel that follows.
//
// rows_pick_kernel (one workgroup per row) finds a value that k+1 block maxima
// reach, reads again the few blocks that reach it (k+1 of them plus ties, 256
// contiguous bytes each), and ranks their elements at or above that value exactly
// (kernels_rows.hpp: finish_row).
#pragma once

#include "kernels_rows.hpp"

namespace vkop {

// Debug builds only (-DVKOP_STAMPS): a log of (kernel, workspace, workgroup, entry and exit clock) records,
// appended by some workgroups as they leave, for a timeline of calls that overlap.
#ifdef VKOP_STAMPS
struct TimelineRec {
    unsigned long long tag, t0, t1;
};
constexpr unsigned kTimelineCap = 1u << 20;
static __device__ TimelineRec g_timeline[kTimelineCap];
static __device__ unsigned g_timeline_n;
#define VKOP_TL_BEGIN() const unsigned long long tl_t0 = wall_clock64()
#define VKOP_TL_END(kind, wsptr, logged)                                                                            \
    do {                                                                                                            \
        if (threadIdx.x == 0 && (logged)) {                                                                         \
            const unsigned long long tl_t1 = wall_clock64();                                                        \
            const unsigned tl_i = atomicAdd(&g_timeline_n, 1u);                                                     \
            if (tl_i < kTimelineCap)                                                                                \
                g_timeline[tl_i] = TimelineRec{(static_cast<unsigned long long>(kind) << 63) |                      \
                                                   (static_cast<unsigned long long>(blockIdx.x & 0xFFFFu) << 40) |   \
                                                   ((reinterpret_cast<unsigned long long>(wsptr) >> 8) & 0xFFFFFFFFFFull), \
                                               tl_t0, tl_t1};                                                       \
        }                                                                                                           \
    } while (0)
#else
#define VKOP_TL_BEGIN() do { } while (0)
#define VKOP_TL_END(kind, wsptr, logged) do { } while (0)
#endif

constexpr int kScanThreads = 256;
constexpr int kScanWaves = kScanThreads / kWave;
constexpr int kBlockLanes = 16;  // lanes (vectors) per block: one row of a wave's cross-lane network

struct ScanWorkspace {
    uint32_t *bmax;    // [rows][blocks]: order key of the block's maximum (softmax: NaN dropped; plain top-k: all
                       // ones if the block holds a NaN); block b = elements b * 16 * vector width ... of the row
    uint64_t *recs;    // [rows][G][kScanWaves][2]: sum of exp(x - ref) over the wave's elements (double bits); ref
                       // (low half) and the wave's maximum (high half) as float bits
    uint64_t *recs2;   // [rows][G][kScanWaves]: the value whose copies the wave counted apart (float bits, high half)
                       // and how many it found (low half; 0: none): its sum leaves them out
    uint32_t blocks;   // blocks per row: ceil(n / (16 * vector width))
    uint32_t *bmin;    // null, or (WITH_MIN) [rows][blocks]: order key of the block's minimum (NaN dropped; the key
                       // of -inf for a block that reaches past the row's end or holds -inf)
    uint32_t *zero;    // null, or [rows][zero_words] words the scan kernel clears for the kernels behind it
    uint32_t zero_words;  // (at most 256)
};

// Launch: rows * G workgroups of kScanThreads; a chunk is exactly 256 * V vectors
// (G = ceil(n / that)), so that blocks never straddle chunks.
// SCALED: every element counts times `scale` (a temperature; > 0), one multiplication
// in single precision before anything else sees it.
// WITH_MIN: the blocks' minima as well (for the large-k kernels behind it: a block whose
// minimum reaches a value holds 16 * vector width elements that do).
// One chunk of one row by kScanThreads threads (tid: 0 .. kScanThreads - 1; block: row * G + chunk).
// No barrier inside, so several chunks can share a workgroup.  vm_lds: [kScanWaves][V][kWave] floats
// (per wave: the maximum of every lane's vector i), vmin_lds the same for WITH_MIN.  Lane l of vector i
// writes to place l ^ 4 (i mod 4): the lane that later reads a block's 16 maxima as four 128-bit words
// finds them in another order (a maximum does not care), and lanes 64 bytes apart no longer meet in the
// same banks -- half of the LDS cycles of this kernel were bank conflicts of those reads.
template <typename T, int V, bool SOFTMAX, bool ALIGNED, bool SCALED, bool WITH_MIN>
__device__ __forceinline__ void scan_chunk(const T *__restrict__ in, uint32_t n, uint32_t G, const ScanWorkspace &ws,
                                           float scale, uint32_t block, uint32_t tid, float (*vm_lds)[V][kWave],
                                           float (*vmin_lds)[V][kWave]) {
    constexpr int NT = kScanThreads, NW = kScanWaves;
    constexpr int VEC = Vec128<T>::N;
    constexpr uint32_t per = static_cast<uint32_t>(NT) * V * VEC;
    constexpr int WB = V * (kWave / kBlockLanes);  // blocks a wave covers: V vectors x 4 rows of 16 lanes
    static_assert(WB <= kWave, "a lane per block of the wave");
    const uint32_t lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t row = block / G, chunk = block - row * G;
    const uint32_t c0 = min(chunk * per, n), c1 = min(c0 + per, n);
    const T *rowp = in + static_cast<size_t>(row) * n;
    const uint32_t e_first = c0 + tid * VEC;  // this lane's first element; vector i starts NT * VEC * i later
    if (ws.zero != nullptr && chunk == 0 && tid < ws.zero_words) ws.zero[static_cast<size_t>(row) * ws.zero_words + tid] = 0;

    // all loads in flight (never a branch around a load: out-of-chunk lanes read the
    // row's first element(s) instead and are masked where the data is used)
    Vec128<T> q[V];
    auto issue_load = [&](auto i_tag) __attribute__((always_inline)) {
        constexpr int i = decltype(i_tag)::value;
        const uint32_t e0 = e_first + static_cast<uint32_t>(i) * NT * VEC;
        q[i].v = make_uint4(0, 0, 0, 0);
        if constexpr (ALIGNED) {
            q[i].load(rowp + (e0 < c1 ? e0 : 0u));
        } else {
#pragma unroll
            for (int c = 0; c < VEC; c++) q[i].set(c, load_elem(rowp, e0 + c < c1 ? e0 + c : 0u));
        }
    };
    static_for<0, V>(issue_load);

    // The rest exists twice: for a chunk that fills every lane of every vector (no
    // masking anywhere) and for a ragged one.
    auto body = [&](auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;
        auto in_range = [&](uint32_t e) { return FULL || e < c1; };
        auto elem = [&](auto i_tag, int c) {
            constexpr int i = decltype(i_tag)::value;
            const uint32_t e0 = e_first + static_cast<uint32_t>(i) * NT * VEC;
            float x = q[i].get(c);
            if constexpr (SCALED) x = scaled(x, scale);
            return in_range(ALIGNED ? e0 : e0 + static_cast<uint32_t>(c)) ? x : -INFINITY;
        };
        float ref = 0.f;
        float wm0 = -INFINITY;  // the maximum of the wave's first vectors
        // The copies of one value -- the wave's first element, where half of the lanes' first
        // elements equal it: a value that fills a row turns up at once -- are counted and left
        // out of the sum: every copy has the same term, so its error (the hardware exponential's, and
        // the rounding of x - M that the definition asks for and a pass that does not know M cannot
        // make) would enter the sum once per copy; the kernel that knows M adds
        // exp_accurate(fl(x0 - M)) for each of them instead.
        float x0 = __uint_as_float(0x7FC00000u);  // (NaN: equal to nothing)
        uint32_t ncopy = 0;
        bool counting = false;
        double acc = 0.0;  // every term is added in double: a dominant term must not swallow what follows it
        static_for<0, V>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            float xv[VEC];
            float vm = -INFINITY;
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                xv[c] = elem(i_tag, c);
                vm = fmaxf(vm, xv[c]);  // (drops NaN)
            }
            if constexpr (WITH_MIN) {
                float vn = INFINITY;
#pragma unroll
                for (int c = 0; c < VEC; c++) vn = fminf(vn, xv[c]);  // (an element past the chunk's end counts as -inf)
                vmin_lds[wave][i][lane ^ ((i & 3) << 2)] = vn;
            }
            if constexpr (SOFTMAX) {
                if constexpr (i == 0) {
                    // reference of the wave's partial sum: kRefLift above the maximum of its
                    // first vectors; 0 if they hold no finite element (terms are then 0, or
                    // NaN, which must survive -- never -inf - -inf)
                    wm0 = wave_max_f32_uniform(vm);
                    ref = (wm0 > -INFINITY) ? wm0 + kRefLift : 0.f;
                    // (the wave's very first element, if most lanes' first elements equal it: on
                    // spread-out rows none does, and nothing below is done for it)
                    const float first = __uint_as_float(static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(__float_as_uint(xv[0])))));
                    const bool mine = xv[0] == first && first > -INFINITY && first < INFINITY;
                    x0 = first;
                    counting = __popcll(__ballot(mine)) >= kWave / 2;
                }
#pragma unroll
                for (int c = 0; c < VEC; c++) acc += static_cast<double>(fast_term(xv[c], ref));
                // the sum so far exists HERE, under the loads still in flight (or the
                // compiler moves all of it behind the last load)
                asm volatile("" : "+v"(acc));
            } else {
                // NaN ranks first in a plain top-k: the vector's maximum is then NaN
                bool has_nan = false;
#pragma unroll
                for (int c = 0; c < VEC; c += 2) has_nan = has_nan || __builtin_isunordered(xv[c], xv[c + 1]);
                vm = has_nan ? __uint_as_float(0x7FC00000u) : vm;
            }
            vm_lds[wave][i][lane ^ ((i & 3) << 2)] = vm;
        });
        // ---- block maxima: lane L of the wave takes block L of the wave's WB blocks -----
        // (block (vector i, lanes 16 r .. 16 r + 15) is the wave's block 4 i + r, and its 16
        // lane values lie side by side; the wave's blocks are read by the wave that wrote them)
        __builtin_amdgcn_wave_barrier();
        float bm = -INFINITY;
        bool b_nan = false;
        if (lane < static_cast<uint32_t>(WB)) {
            const float4 *src = reinterpret_cast<const float4 *>(&vm_lds[wave][0][0] + lane * kBlockLanes);
#pragma unroll
            for (int j = 0; j < kBlockLanes / 4; j++) {
                const float4 v4 = src[j ^ ((lane >> 2) & 3)];  // (the block of vector lane / 4: its words are in the order 0..3 ^ that vector's number mod 4)
                bm = fmaxf(fmaxf(bm, fmaxf(v4.x, v4.y)), fmaxf(v4.z, v4.w));
                if constexpr (!SOFTMAX) b_nan = b_nan || __builtin_isunordered(v4.x, v4.y) || __builtin_isunordered(v4.z, v4.w);
            }
            // the wave's block L = vector L / 4, lane row L % 4 starts at element
            // c0 + ((L / 4) * NT + wave * 64 + (L % 4) * 16) * VEC of the row
            const uint32_t e_block = c0 + ((lane / 4u) * NT + wave * kWave + (lane % 4u) * kBlockLanes) * VEC;
            if (FULL || e_block < c1) {
                const uint32_t key = b_nan ? 0xFFFFFFFFu : order_key(bm);
                ws.bmax[static_cast<size_t>(row) * ws.blocks + e_block / (kBlockLanes * VEC)] = key;
                if constexpr (WITH_MIN) {
                    const float4 *srcn = reinterpret_cast<const float4 *>(&vmin_lds[wave][0][0] + lane * kBlockLanes);
                    float bn = INFINITY;
#pragma unroll
                    for (int j = 0; j < kBlockLanes / 4; j++) {
                        const float4 v4 = srcn[j ^ ((lane >> 2) & 3)];
                        bn = fminf(fminf(bn, fminf(v4.x, v4.y)), fminf(v4.z, v4.w));
                    }
                    ws.bmin[static_cast<size_t>(row) * ws.blocks + e_block / (kBlockLanes * VEC)] = order_key(bn);
                }
            }
        }
        // ---- the wave's record ---------------------------------------------------------------
        if constexpr (SOFTMAX) {
            const float wm = wave_max_f32_uniform(bm);
            if (counting) {  // (wave-uniform; everything is still in registers)
                static_for<0, V>([&](auto i_tag) {
#pragma unroll
                    for (int c = 0; c < VEC; c++) ncopy += (elem(i_tag, c) == x0) ? 1u : 0u;
                });
            }
            // (every copy added the same float: taking them out again is exact to the sum's own rounding)
            if (ncopy != 0u) acc -= static_cast<double>(ncopy) * static_cast<double>(fast_term(x0, ref));
            double wsum = wave_sum_f64_uniform(acc);
            if (wm - ref > kTermSwitch) {  // wave-uniform
                // an element well above the reference: its fast term is poor (or has
                // overflowed); everything is in registers, so sum again against the maximum
                ref = (wm < INFINITY) ? wm : ref;
                acc = 0.0;
                static_for<0, V>([&](auto i_tag) {
#pragma unroll
                    for (int c = 0; c < VEC; c++) acc += static_cast<double>(fast_term(elem(i_tag, c), ref));
                });
                if (ncopy != 0u) acc -= static_cast<double>(ncopy) * static_cast<double>(fast_term(x0, ref));
                wsum = wave_sum_f64_uniform(acc);
            }
            const uint32_t copies = counting ? static_cast<uint32_t>(wave_sum_f64_uniform(static_cast<double>(ncopy))) : 0u;
            if (lane == 0) {
                ws.recs2[static_cast<size_t>(row * G + chunk) * NW + wave] = (static_cast<uint64_t>(__float_as_uint(x0)) << 32) | copies;
                uint64_t *record = ws.recs + 2 * (static_cast<size_t>(row * G + chunk) * NW + wave);
                record[0] = static_cast<uint64_t>(__double_as_longlong(wsum));
                record[1] = (static_cast<uint64_t>(__float_as_uint(wm)) << 32) | __float_as_uint(ref);
            }
        }
    };
    if (c1 - c0 == per) body(std::true_type{});
    else body(std::false_type{});
}

// Launch: rows * G workgroups of kScanThreads, a chunk each.
template <typename T, int V, bool SOFTMAX, bool ALIGNED, bool SCALED = false, bool WITH_MIN = false>
__global__ __launch_bounds__(kScanThreads) void rows_scan_kernel(const T *__restrict__ in, uint32_t n, uint32_t G,
                                                                 ScanWorkspace ws, float scale = 1.f) {
    VKOP_TL_BEGIN();
    __shared__ float vm_lds[kScanWaves][V][kWave];
    if constexpr (WITH_MIN) {
        __shared__ float vmin_lds[kScanWaves][V][kWave];
        scan_chunk<T, V, SOFTMAX, ALIGNED, SCALED, true>(in, n, G, ws, scale, blockIdx.x, threadIdx.x, vm_lds, vmin_lds);
    } else {
        scan_chunk<T, V, SOFTMAX, ALIGNED, SCALED, false>(in, n, G, ws, scale, blockIdx.x, threadIdx.x, vm_lds, nullptr);
    }
    VKOP_TL_END(0, ws.bmax, blockIdx.x % 16u == 0u || blockIdx.x + 48u >= gridDim.x);
}

constexpr int kPickHitCap = 1024;  // blocks one gather reads again

constexpr int kPickThreads = 512;
struct PickShared {
    RowsShared fast;
    uint32_t hits[kPickHitCap];  // the blocks to read again (the first gather: a part per wave)
    uint4 stage_v[kPickThreads / kWave][kWave];     // per wave: the vectors that hold an element at or above the threshold ...
    uint32_t stage_e[kPickThreads / kWave][kWave];  // ... and the index of their first element
    uint32_t trial_cnt[kPickThreads / kWave][kPickThreads / kWave];  // [wave][trial]: the wave's thread maxima that reach another wave's bound
};
union PickSharedUnion {
    PickShared pick;
    SelectShared exact;
    __device__ PickSharedUnion() {}
};

// One workgroup of NT threads per row, after rows_scan_kernel on the same stream.
// GE: block keys a thread takes in (GE * NT >= blocks per row); G, per: chunks per
// row and elements per chunk of the scan kernel (which wave summed which element).
//   A. one round trip: the wave records and the row's block keys (GE per thread);
//   B. the row's maximum and sum of terms from the wave records;
//   C. a value that at least k+1 block maxima reach: ballot descents over the
//      per-thread maxima of the keys (every block maximum is an element);
//   D. the blocks that reach it -- k+1 and a few -- are read again, 16 lanes a block,
//      several loads per thread in flight; their elements at or above the value are
//      the candidates (everything else in the row is below k+1 elements);
//   E. finish_row: exact ranks, accurate terms, probabilities, ties, ordered store.
// More candidates than the list holds: a second threshold a level down (the largest
// element every thread saw), then -- if that left fewer but still too many: rows sorted
// in runs -- the exact (k+1)-th largest of those blocks' elements by a radix select over
// them, or -- if it left as many: equal values en masse -- the first elements equal to the
// exact threshold from the row's start.
// A probability tie across the k-th place that reaches below the value gathers again
// with the tied interval's lower end (settle_tie); what that cannot hold (rows full of
// equal values) goes to the scan from the row's start or, from D, to the exact radix
// select over the whole row.
// scale: as in the scan kernel (1 when that ran unscaled); counts (softmax variant,
// may be null): per row the nucleus cut of its result for top_p (finish_row).
// SCALED false: scale is 1, and the common case does without the multiplications.
// pick_row: one row by all NT threads of a workgroup (smem, fscratch, dscratch: its LDS).
template <typename T, bool SOFTMAX, bool ALIGNED, int GE, bool SCALED, int NT>
__device__ __forceinline__ void pick_row(PickSharedUnion &smem, float *fscratch, double *dscratch, uint32_t row,
                                         const T *__restrict__ in, T *__restrict__ values, int32_t *__restrict__ indices,
                                         uint32_t n, uint32_t k, uint32_t G, uint32_t per, const ScanWorkspace &ws,
                                         float scale, int32_t *__restrict__ counts, float top_p) {
    constexpr int NW = NT / kWave;
    constexpr int VEC = Vec128<T>::N;
    constexpr int U = NT >= 1024 ? 2 : NT >= 512 ? 4 : 8;  // loads per thread in flight while blocks are read again (128 blocks a round)
    constexpr uint32_t BE = kBlockLanes * VEC;  // elements per block
    RowsShared &sh = smem.pick.fast;
    uint32_t *hits = smem.pick.hits;
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const T *rowp = in + static_cast<size_t>(row) * n;
    T *ov = values + static_cast<size_t>(row) * k;
    int32_t *oi = indices + static_cast<size_t>(row) * k;
    const uint32_t want = k + 1;
    const uint32_t kk = min(k, n);
    const uint32_t waves = G * kScanWaves;
    // (a short chain of dependent steps per row, often beside the streaming kernel of another call on the same
    // CU, whose waves issue all the time: this kernel's waves go first)
    __builtin_amdgcn_s_setprio(3);
    BPS(14);
#ifdef VKOP_STAMPS
    if (threadIdx.x == 0 && blockIdx.x == 0) g_bp_stamps[60] = clock64();
#endif
    // ---- A. everything the kernel reads first, in one round trip --------------------
    // (never a branch around a load: out-of-range threads re-read entry 0)
    const uint64_t *recs = ws.recs + 2 * static_cast<size_t>(row) * waves;
    const uint32_t wq = tid < waves ? tid : 0u;
    uint64_t s_bits = 0, rm_bits = 0, c_bits = 0;
    if constexpr (SOFTMAX) {
        s_bits = recs[2 * wq];
        rm_bits = recs[2 * wq + 1];
        c_bits = ws.recs2[static_cast<size_t>(row) * waves + wq];
    }
    const uint32_t blocks = ws.blocks;
    const uint32_t *bmax = ws.bmax + static_cast<size_t>(row) * blocks;
    uint32_t gk[GE];
#pragma unroll
    for (int e = 0; e < GE; e++) {
        const uint32_t b = static_cast<uint32_t>(e) * NT + tid;
        gk[e] = bmax[b < blocks ? b : 0u];
    }

    // ---- B. the row's maximum and sum from the wave partials --------------------------
    // (runs while the blocks that are read again are on their way: nothing before the ranking needs it)
    BPS(8);
    for (uint32_t t = tid; t < static_cast<uint32_t>(kFastCap); t += NT) sh.rank[t] = 0;  // for block_rank, barriers away
    sh.cand[tid] = 0;  // (the list the waves make below ends in zeros: block_rank_padded)
    auto times_scale = [&](float x) {
        if constexpr (SCALED) return scaled(x, scale);
        else return x;
    };
    if (tid == 0) {
        sh.count = 0;
        sh.wave_overflow = 0;
    }
    auto combine_records = [&]() __attribute__((always_inline)) {
      if constexpr (SOFTMAX) {
        SumPartial p0{0.0, 0.f, -INFINITY};
        if (tid < waves) {
            p0.s = __longlong_as_double(static_cast<long long>(s_bits));
            p0.ref = __uint_as_float(static_cast<uint32_t>(rm_bits));
            p0.m = __uint_as_float(static_cast<uint32_t>(rm_bits >> 32));
            sh.ref[tid] = p0.ref;
            sh.x0[tid] = static_cast<uint32_t>(c_bits) != 0u ? __uint_as_float(static_cast<uint32_t>(c_bits >> 32)) : __uint_as_float(0x7FC00000u);
        }
        // the copies the wave counted apart: each counts exp_accurate(fl(x0 - M)), as the sum is defined
        auto copies_term = [&](float m) -> double {
            const uint32_t cn = tid < waves ? static_cast<uint32_t>(c_bits) : 0u;
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
                    if (p0.s != 0.0) acc = p0.s * sc;
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
                if (p0.s != 0.0) acc = p0.s * sc;
            }
            acc += copies_term(m);
            const double total = block_sum_fast<NT>(acc, dscratch);  // (barrier: sh.scale is published)
            if (tid == 0) {
                sh.row_max = m;
                sh.total = total;
            }
        }
      }
    };

    // ---- C. a value that k+1 block maxima reach ---------------------------------------------
    BPS(9);
    uint32_t lmk = 0;
#pragma unroll
    for (int e = 0; e < GE; e++) {
        if (static_cast<uint32_t>(e) * NT + tid >= blocks) gk[e] = 0;  // (block 0 was read instead)
        lmk = max(lmk, gk[e]);
    }
    // Every wave takes, by a ballot descent over its own 64 thread maxima (18 bits),
    // the largest value that its share of k+1 of them reach: the smallest of these
    // bounds is reached by k+1 thread maxima in all, hence by k+1 blocks.  A share of
    // more than half a wave, or a wave without enough live threads, leaves it to one
    // wave and all the maxima.
    // (all threads call, each with its own maximum; the first barrier inside also
    // publishes the row's maximum and sum of phase B)
    // by_quota false: one wave and all the maxima at once (waves that are not alike -- a
    // sorted row -- make the smallest of the waves' bounds far too low).
    // bits: how many leading bits of the answer are worked out when one wave does it (32:
    // the exact (k+1)-th largest, the key of an element).
    auto threshold_of_thread_maxima = [&](uint32_t mine_max, bool by_quota, int bits = 20) -> uint32_t {
        const uint32_t quota = (want + NW - 1) / NW;
        uint32_t mine_q = 0;
        if (by_quota && quota <= 32u) {
            // two bits a step (three trial values counted side by side): the steps depend on each other
            for (int bit = 30; bit > 13; bit -= 2) {
                const uint32_t t1 = mine_q | (1u << bit), t2 = mine_q | (2u << bit), t3 = mine_q | (3u << bit);
                const uint32_t c1 = static_cast<uint32_t>(__popcll(__ballot(mine_max >= t1)));
                const uint32_t c2 = static_cast<uint32_t>(__popcll(__ballot(mine_max >= t2)));
                const uint32_t c3 = static_cast<uint32_t>(__popcll(__ballot(mine_max >= t3)));
                mine_q = c3 >= quota ? t3 : c2 >= quota ? t2 : c1 >= quota ? t1 : mine_q;
            }
        }
        sh.lane_key[tid] = mine_max;
        if (lane == 0) sh.wave_thr[wave] = mine_q;
        __syncthreads();
        uint32_t bound[NW];
        uint32_t t = 0xFFFFFFFFu;
#pragma unroll
        for (int w = 0; w < NW; w++) {
            bound[w] = sh.wave_thr[w];
            t = min(t, bound[w]);
        }
        if (by_quota && t > 1u) {
            // The smallest of the waves' bounds is reached by k+1 thread maxima but is lower than it need be
            // (about 1.8 (k+1) blocks reach it at k = 50).  Every wave counts its thread maxima that reach
            // each of the NW bounds; the largest bound that k+1 maxima in all reach is the threshold (1.15 (k+1)
            // blocks): a barrier more, fewer blocks to read again, half as many candidates to rank.
            uint32_t mine_c = 0;
#pragma unroll
            for (int w = 0; w < NW; w++) {
                const uint32_t c = static_cast<uint32_t>(__popcll(__ballot(mine_max >= bound[w])));
                mine_c = lane == static_cast<uint32_t>(w) ? c : mine_c;
            }
            if (lane < static_cast<uint32_t>(NW)) smem.pick.trial_cnt[wave][lane] = mine_c;
            __syncthreads();
            uint32_t reach = 0, mine_b = 0;
            if (lane < static_cast<uint32_t>(NW)) {
#pragma unroll
                for (int w = 0; w < NW; w++) reach += smem.pick.trial_cnt[w][lane];
                mine_b = sh.wave_thr[lane];
            }
            return wave_max_u32(reach >= want ? mine_b : t);  // (the smallest bound always qualifies)
        }
        if (t <= 1u) {  // (the same for every thread)
            if (wave == 0) {
                const uint32_t f = block_kth_largest_floor<NW>(sh.lane_key, want, bits);
                if (lane == 0) sh.thr = f;
            }
            __syncthreads();
            t = sh.thr;
        }
        return t;
    };
    uint32_t thr = threshold_of_thread_maxima(lmk, true);
    BPS(10);
    // -inf never becomes a candidate: a row with k+1 larger elements does not need it,
    // and finish_row fills any other row's last places from the row itself
    thr = max(thr, kKeyNegInf + 1u);

    // ---- D1. the first gather, wave by wave ------------------------------------------------
    // Every wave reads again ITS threads' blocks that reach thr (a list of its own in LDS: no
    // workgroup barrier between the threshold and the loads), 16 lanes a block, 2 U loads per
    // lane in flight (the second U only in a wave with more than 16 such blocks); phase B runs
    // under them.  A vector that holds an element at or above thr (one in 16 of those read) goes
    // to the wave's stage in LDS, and one lane per staged vector lists its elements in sh.cand:
    // a prefix sum over the lanes and one LDS atomic per wave give the places.
    // A wave with more blocks or vectors than its lists hold only raises sh.wave_overflow: the
    // workgroup then gathers the general way (below).
    constexpr uint32_t kWaveHitCap = 2 * U * (kWave / kBlockLanes);  // blocks a wave reads again in one go
    static_assert(NW * kWaveHitCap <= kPickHitCap, "every wave's list of blocks fits");
    static_assert(NW <= kPickThreads / kWave, "a stage per wave");
    // About 1.15 (k+1) blocks reach thr, a wave's share of them has to fit its list, and the shares are not alike:
    // from five eighths of the lists' total on, some wave of most rows has too many, and what the waves did is
    // thrown away (an unaligned row pays a load per element for it).  Such rows go the general way at once.
    const bool wave_lists = want <= NW * kWaveHitCap * 5u / 8u;
    if (wave_lists) {
        uint32_t wave_n = 0;  // wave-uniform
#pragma unroll
        for (int e = 0; e < GE; e++) wave_n += static_cast<uint32_t>(__popcll(__ballot(gk[e] >= thr)));
        const bool wave_ok = wave_n <= kWaveHitCap;
        uint32_t *whits = hits + wave * kWaveHitCap;
        if (wave_ok) {
            uint32_t pos = 0;
#pragma unroll
            for (int e = 0; e < GE; e++) {
                const bool pass = gk[e] >= thr;
                const uint64_t mask = __ballot(pass);
                if (pass) whits[pos + lanes_below(mask)] = static_cast<uint32_t>(e) * NT + tid;
                pos += static_cast<uint32_t>(__popcll(mask));
            }
        }
        __builtin_amdgcn_wave_barrier();  // (the wave reads its own list: LDS keeps a wave's accesses in order)
        const uint32_t items = wave_ok ? wave_n * kBlockLanes : 0u;  // one per vector of a block that is read again
        const float lo_f = ordered_to_float(thr);
        Vec128<T> r[2 * U];
        uint32_t e0[2 * U];
        auto issue = [&](auto u_tag) __attribute__((always_inline)) {
            constexpr int u = decltype(u_tag)::value;
            const uint32_t j = static_cast<uint32_t>(u) * kWave + lane;
            const uint32_t b = whits[j < items ? j / kBlockLanes : 0u];
            // (a slot past the wave's items reads the row's start and is marked by an index past the row's end)
            e0[u] = j < items ? b * BE + (j % kBlockLanes) * VEC : 0xFFFFFFFFu;
            r[u].v = make_uint4(0, 0, 0, 0);
            if constexpr (ALIGNED) {
                r[u].load(rowp + (e0[u] < n ? e0[u] : 0u));
            } else {
#pragma unroll
                for (int c = 0; c < VEC; c++) r[u].set(c, load_elem(rowp, e0[u] < n && e0[u] + c < n ? e0[u] + c : 0u));
            }
        };
        static_for<0, U>(issue);
        const bool second_half = items > static_cast<uint32_t>(U) * kWave;  // wave-uniform
        if (second_half) static_for<U, 2 * U>(issue);
        combine_records();
        // vectors with an element at or above thr -> the wave's stage
        uint4 *stage_v = smem.pick.stage_v[wave];
        uint32_t *stage_e = smem.pick.stage_e[wave];
        uint32_t nv = 0;  // wave-uniform
        auto sift = [&](auto u_tag) __attribute__((always_inline)) {
            constexpr int u = decltype(u_tag)::value;
            float vm = -INFINITY;
            bool any_nan = false;
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                const float x = times_scale(r[u].get(c));
                vm = fmaxf(vm, x);
                if constexpr (!SOFTMAX) any_nan = any_nan || x != x;
            }
            const bool pv = e0[u] < n && (!(vm < lo_f) || any_nan);
            const uint64_t mask = __ballot(pv);
            if (mask != 0ull) {
                const uint32_t slot = nv + lanes_below(mask);
                if (pv && slot < static_cast<uint32_t>(kWave)) {
                    stage_v[slot] = r[u].v;
                    stage_e[slot] = e0[u];
                }
                nv += static_cast<uint32_t>(__popcll(mask));
            }
        };
        static_for<0, U>(sift);
        if (second_half) static_for<U, 2 * U>(sift);
        __builtin_amdgcn_wave_barrier();
        if (!wave_ok || nv > static_cast<uint32_t>(kWave)) {
            if (lane == 0) sh.wave_overflow = 1;
        } else if (nv != 0u) {
            // lane l lists the elements of staged vector l
            Vec128<T> sv;
            sv.v = stage_v[lane < nv ? lane : 0u];
            const uint32_t eb = stage_e[lane < nv ? lane : 0u];
            uint32_t pbits = 0;
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                const float x = times_scale(sv.get(c));
                // (softmax: a NaN never passes, and thr is the key of a number, so the floats compare as the keys do)
                bool pass;
                if constexpr (SOFTMAX) pass = x >= lo_f;
                else pass = order_key(x) >= thr;
                pass = pass && lane < nv && (ALIGNED || eb + static_cast<uint32_t>(c) < n);
                pbits |= pass ? (1u << c) : 0u;
            }
            const uint32_t mine_n = static_cast<uint32_t>(__popc(pbits));
            const uint32_t incl = wave_inclusive_sum_u32(mine_n);
            const uint32_t wave_total = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(incl), kWave - 1));
            uint32_t base = 0;
            if (lane == 0) base = atomicAdd(&sh.count, wave_total);
            base = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(base)));
            uint32_t at = base + incl - mine_n;
#pragma unroll
            for (int c = 0; c < VEC; c++) {
                if (pbits & (1u << c)) {
                    const float x = times_scale(sv.get(c));
                    if (at < static_cast<uint32_t>(kFastCap)) sh.cand[at] = composite(order_key(x), eb + static_cast<uint32_t>(c));
                    at++;
                }
            }
        }
    } else {
        combine_records();
    }
    BPS(44);
    __syncthreads();  // the candidates and phase B's results
    BPS(11);
    float M = 0.f;
    double s_base = 0.0;
    if constexpr (SOFTMAX) {
        M = sh.row_max;
        s_base = sh.total;
    }
    const uint32_t per_shift = 31u - static_cast<uint32_t>(__clz(per));
    // the scan-kernel wave that summed element idx (per = 256 * V vectors: a power of two)
    auto wave_of = [&](uint32_t idx) {
        const uint32_t b = idx >> per_shift, off = idx & (per - 1u);
        return b * kScanWaves + ((off / VEC) % kScanThreads) / kWave;
    };

    bool have_list = false;
    // ---- E1. the common case to its end ---------------------------------------------------------
    // Every wave listed its candidates, they are at least k+1 and a thread can take one each, and
    // the row's sum is a positive number: ranks, accurate terms for the k+1 first, probabilities.
    // Equal probabilities of DIFFERENT logits among the k+1 (to be put in order by index; across the k-th
    // place a matter of the whole row) leave it to the general code below, as does everything else.  Equal
    // logits are no such case -- the ranking has them in index order already, and every element with the
    // logit of rank k is in the list -- which is what logits that went through bfloat16 or int8 are full of.
    {
        const uint32_t C2 = sh.count;
        bool common = wave_lists && sh.wave_overflow == 0u && C2 >= want && C2 <= static_cast<uint32_t>(NT) && kk == k;
        if constexpr (SOFTMAX) common = common && s_base > 0.0 && s_base < static_cast<double>(INFINITY) && M > -INFINITY && M < INFINITY;
        if (__builtin_expect(common, 1)) {
            // A candidate's own part (its wave's record, its accurate term) and the ranking are two chains of
            // a hundred instructions and more: where the candidates fill at most half of the workgroup's waves
            // (P, the power of two at or above their number, up to NT / 2), those waves take the terms and the
            // others the ranking -- NT / P - 1 groups of P threads, a group a part of the list, which ends in zeros.
            static_assert(NT == 512, "the table of parts below");
            const uint32_t pshift = C2 > 64u ? 32u - static_cast<uint32_t>(__clz(C2 - 1u)) : 6u;  // P >= 64
            const bool apart = pshift <= 8u;
            uint64_t mine = 0;
            float term = 0.f;
            double cr = 0.0;
            if (tid < C2) {
                mine = sh.cand[tid];
                if constexpr (SOFTMAX) {
                    const uint32_t key = static_cast<uint32_t>(mine >> 32);
                    const uint32_t sp = wave_of(composite_index(mine));
                    const float xv = ordered_to_float(key);
                    // what the element should contribute, exp(fl(x - M)), minus what its wave added for it,
                    // fast_term(x, ref) * exp(ref - M) (a copy of the value its wave counted apart went in with this very term)
                    term = softmax_term(xv, M);
                    cr = (xv == sh.x0[sp]) ? 0.0 : static_cast<double>(term) - static_cast<double>(fast_term(xv, sh.ref[sp])) * sh.scale[sp];
                }
            }
            BPS(30);
            if (apart) {
                if (tid >= (1u << pshift)) {
                    // 7 groups of 64 take 10 entries each, 3 groups of 128 take 44, 1 group of 256 all of them (even numbers: two per read)
                    const uint32_t span = pshift == 6u ? 10u : pshift == 7u ? 44u : 256u;
                    const uint32_t i = tid & ((1u << pshift) - 1u);
                    const uint64_t cmp = sh.cand[i];
                    const uint4 *src = reinterpret_cast<const uint4 *>(sh.cand + ((tid >> pshift) - 1u) * span);
                    uint32_t cnt = 0;
                    for (uint32_t j = 0; j < span / 2; j += 4) {  // four reads of two entries in flight (past the span: counted by the next group too -- never: zeros or skipped)
                        uint4 o[4];
#pragma unroll
                        for (int u = 0; u < 4; u++) o[u] = src[j + u < span / 2 ? j + u : 0u];
#pragma unroll
                        for (int u = 0; u < 4; u++) {
                            const bool in = j + u < span / 2;
                            cnt += (in && ((static_cast<uint64_t>(o[u].y) << 32) | o[u].x) > cmp) ? 1u : 0u;
                            cnt += (in && ((static_cast<uint64_t>(o[u].w) << 32) | o[u].z) > cmp) ? 1u : 0u;
                        }
                    }
                    if (cnt) atomicAdd(&sh.rank[i], cnt);
                }
                __syncthreads();
            } else {
                block_rank_padded<NT>(sh, C2);  // (ends with a barrier)
            }
            BPS(31);
            if (tid < C2) {
                const uint32_t rk = sh.rank[tid];
                if (rk < want) {
                    sh.pidx[rk] = composite_index(mine);
                    sh.pkey[rk] = static_cast<uint32_t>(mine >> 32);
                    sh.prob[rk] = term;
                    sh.corr[rk] = cr;
                }
            }
            __syncthreads();
            BPS(32);
            // every wave works the rest out for itself: the same values in the same order, so every
            // wave decides alike whether the row is done, and no barrier is needed for that
            bool tie = false;
            if constexpr (SOFTMAX) {
                double csum = 0.0;
                for (uint32_t r = lane; r < want; r += kWave) csum += sh.corr[r];
                const double rinv = 1.0 / (s_base + wave_sum_f64_uniform(csum));
                float p_first = 0.f;  // lane l of the first 64 ranks: its probability
                for (uint32_t base = 0; base < k; base += kWave) {
                    const uint32_t r = base + lane;  // ranks r and r + 1 <= k
                    const float p0 = round_to_storage<T>(static_cast<float>(static_cast<double>(sh.prob[r < k ? r : 0u]) * rinv));
                    const float p1 = round_to_storage<T>(static_cast<float>(static_cast<double>(sh.prob[r < k ? r + 1u : 0u]) * rinv));
                    tie = tie || (r < k && p0 == p1 && sh.pkey[r] != sh.pkey[r < k ? r + 1u : 0u]);
                    if (base == 0) p_first = p0;
                }
                tie = __ballot(tie) != 0ull;
                if (!tie) {
                    // (the waves take the ranks 64 at a time, in turn)
                    for (uint32_t base = wave * kWave; base < k; base += NW * kWave) {
                        const uint32_t r = base + lane;
                        const float p0 = base == 0 ? p_first
                                                   : round_to_storage<T>(static_cast<float>(static_cast<double>(sh.prob[r < k ? r : 0u]) * rinv));
                        if (r < k) {
                            store_elem(ov, r, p0);
                            oi[r] = static_cast<int32_t>(sh.pidx[r]);
                        }
                    }
                }
                if (!tie && counts != nullptr && wave == 0) {
                    // the nucleus cut: the stored values walked in order through the lanes, as topp_count_kernel does
                    const uint32_t count = nucleus_count_wave(k, top_p, [&](uint32_t r) {
                        return r < static_cast<uint32_t>(kWave) ? p_first : round_to_storage<T>(static_cast<float>(static_cast<double>(sh.prob[r]) * rinv));
                    });
                    if (lane == 0) counts[row] = static_cast<int32_t>(count);
                }
            } else {
                // values are bit copies of the elements: the key gives the bits back, except for a zero (either sign) and a NaN
                for (uint32_t r = tid; r < k; r += NT) {
                    const uint32_t key = sh.pkey[r], idx = sh.pidx[r];
                    if (key == 0x80000000u || key == 0xFFFFFFFFu) ov[r] = rowp[idx];
                    else store_elem(ov, r, ordered_to_float(key));
                    oi[r] = static_cast<int32_t>(idx);
                }
            }
            BPS(13);
#ifdef VKOP_STAMPS
            if (threadIdx.x == 0 && blockIdx.x == 0) g_bp_stamps[61] = clock64();
#endif
            if (__builtin_expect(!tie, 1)) return;
            // (equal probabilities: what was stored is written again below, in its final order)
        }
        // The general code: with the list the waves made, if every wave could list all of its blocks
        // (the list may still hold fewer than k+1 entries, or have dropped what came after its capacity:
        // sh.count says how many there were), else from an empty one.
        have_list = wave_lists && sh.wave_overflow == 0u;
        __syncthreads();
        for (uint32_t t = tid; t < static_cast<uint32_t>(kFastCap); t += NT) sh.rank[t] = 0;
        if (!have_list && tid == 0) sh.count = 0;
        __syncthreads();
    }
    if constexpr (SOFTMAX) {
        if (!(s_base > 0.0 && s_base < static_cast<double>(INFINITY)) || !(M > -INFINITY && M < INFINITY)) {
            // a NaN or +inf element, or nothing above -inf: every probability of the
            // row is NaN, all of them tie, the lowest indices win
            for (uint32_t r = tid; r < kk; r += NT) {
                store_elem(ov, r, __uint_as_float(0x7FC00000u));
                oi[r] = static_cast<int32_t>(r);
            }
            if (counts != nullptr && tid == 0) counts[row] = static_cast<int32_t>(kk);  // (a sum of NaN reaches nothing)
            return;
        }
    }

    // ---- D. the elements with keys in [lo, hi) of the blocks whose maximum reaches lo -> sh.cand ----
    // All threads call; ends with a barrier.  Returns true (in every thread) when more
    // than hit_cap blocks reach lo: nothing was gathered then.
    uint32_t round = 0;
    // (always inlined: a call would put the block keys, captured by reference, into scratch memory)
    // dry_tag true: nothing is appended; dry_max becomes the largest key this thread saw in [lo, hi).
    // dry_tag 2: nothing is appended; the keys in [lo, hi) that agree with digit_prefix above bit
    // digit_shift + 8 are counted by their eight bits from digit_shift up, into digit_hist.
    uint32_t dry_max = 0;
    uint32_t hit_cap = kPickHitCap;  // more blocks than this are not read: gather returns true
    uint32_t *digit_hist = reinterpret_cast<uint32_t *>(sh.cand);  // (the list is gathered anew afterwards)
    uint32_t digit_prefix = 0;
    int digit_shift = 24;
    auto gather = [&](uint32_t lo, uint64_t hi, auto dry_tag) __attribute__((always_inline)) -> bool {
        constexpr int MODE = static_cast<int>(decltype(dry_tag)::value);
        constexpr bool DRY = MODE == 1;
        uint32_t wave_n = 0;  // wave-uniform
#pragma unroll
        for (int e = 0; e < GE; e++) wave_n += static_cast<uint32_t>(__popcll(__ballot(gk[e] >= lo)));
        uint32_t *wc = sh.scan_counts + (round & 1u) * NW;
        round++;
        if (lane == 0) wc[wave] = wave_n;
        __syncthreads();
        uint32_t H = 0, pos = 0;
#pragma unroll
        for (int w = 0; w < NW; w++) {
            const uint32_t c = wc[w];
            pos += (static_cast<uint32_t>(w) < wave) ? c : 0u;
            H += c;
        }
        if (H > hit_cap) return true;
#pragma unroll
        for (int e = 0; e < GE; e++) {
            const bool pass = gk[e] >= lo;
            const uint64_t mask = __ballot(pass);
            if (mask != 0ull) {
                if (pass) hits[pos + lanes_below(mask)] = static_cast<uint32_t>(e) * NT + tid;
                pos += static_cast<uint32_t>(__popcll(mask));
            }
        }
        __syncthreads();
        const uint32_t items = H * kBlockLanes;  // one per vector of a block that is read again
        for (uint32_t j0 = 0; j0 < items; j0 += NT * U) {
            Vec128<T> r[U];
            uint32_t e0[U], cend[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const uint32_t j = j0 + static_cast<uint32_t>(u) * NT + tid;
                const uint32_t b = hits[j < items ? j / kBlockLanes : 0u];
                e0[u] = b * BE + (j % kBlockLanes) * VEC;
                cend[u] = j < items ? n : 0u;  // (0: nothing of this slot counts)
                r[u].v = make_uint4(0, 0, 0, 0);
                if constexpr (ALIGNED) {
                    r[u].load(rowp + (e0[u] < cend[u] ? e0[u] : 0u));
                } else {
#pragma unroll
                    for (int c = 0; c < VEC; c++) r[u].set(c, load_elem(rowp, e0[u] + c < cend[u] ? e0[u] + c : 0u));
                }
            }
            const float lo_f = ordered_to_float(lo);  // (lo > key of -inf: a number or +inf)
#pragma unroll
            for (int u = 0; u < U; u++) {
                // a vector without an element at or above lo (15 of a block's 16) costs one test
                float vm = -INFINITY;
                bool any_nan = false;
#pragma unroll
                for (int c = 0; c < VEC; c++) {
                    const float x = scaled(r[u].get(c), scale);
                    vm = fmaxf(vm, x);
                    if constexpr (!SOFTMAX) any_nan = any_nan || x != x;
                }
                if (!(vm < lo_f) || any_nan) {
#pragma unroll
                    for (int c = 0; c < VEC; c++) {
                        const float x = scaled(r[u].get(c), scale);
                        const uint32_t idx = e0[u] + static_cast<uint32_t>(c);
                        const uint32_t key = (SOFTMAX && x != x) ? 0u : order_key(x);
                        if (idx < cend[u] && key >= lo && static_cast<uint64_t>(key) < hi) {
                            if constexpr (DRY) {
                                dry_max = max(dry_max, key);
                            } else if constexpr (MODE == 2) {
                                if ((static_cast<uint64_t>(key ^ digit_prefix) >> (digit_shift + 8)) == 0ull)
                                    hist_add_grouped(digit_hist, (key >> digit_shift) & 255u);
                            } else {
                                const uint32_t at = atomicAdd(&sh.count, 1u);
                                if (at < static_cast<uint32_t>(kFastCap)) sh.cand[at] = composite(key, idx);
                            }
                        }
                    }
                }
            }
        }
        __syncthreads();
        return false;
    };
    // The first value is reached by k+1 blocks and a few (about 2.5 (k+1) on spread-out rows at
    // k = 50, fewer at larger k).  Three times k+1 and more are a row whose block maxima are equal en
    // masse (a constant row, a few levels) or whose threads' shares are not alike (below): reading
    // all of them again -- the whole row, for a constant one -- settles nothing.
    // (The same when EVERY block reaches it and the row has a quarter more blocks than places.)
    hit_cap = min(static_cast<uint32_t>(kPickHitCap), 3u * want + 64u);
    if (blocks > want + want / 4u) hit_cap = min(hit_cap, blocks - 1u);
    bool many_groups = have_list ? false : gather(thr, 1ull << 32, std::false_type{});
    if (many_groups) {
        // More than kPickHitCap blocks reach thr: the threads' shares of the block maxima are
        // not alike (rows sorted in runs as long as the stride between a thread's blocks put
        // every run's top block into the same few threads, and the (k+1)-th largest THREAD
        // maximum is then far below the (k+1)-th largest block maximum).  That one exactly,
        // by a descent over all the keys, a barrier a bit: a dozen microseconds, on such rows.
        uint32_t exact_thr = 0;
        for (int bit = 31; bit >= 0; bit--) {
            const uint32_t trial = exact_thr | (1u << bit);
            uint32_t c = 0;  // wave-uniform
#pragma unroll
            for (int e = 0; e < GE; e++) c += static_cast<uint32_t>(__popcll(__ballot(gk[e] >= trial)));
            uint32_t *wc = sh.scan_counts + (round & 1u) * NW;
            round++;
            if (lane == 0) wc[wave] = c;
            __syncthreads();
            uint32_t total = 0;
#pragma unroll
            for (int w = 0; w < NW; w++) total += wc[w];
            if (total >= want) exact_thr = trial;
        }
        if (exact_thr > thr) {
            thr = exact_thr;
            many_groups = gather(thr, 1ull << 32, std::false_type{});
        }
    }
    hit_cap = kPickHitCap;  // (from here on: whatever the list of blocks holds)
    uint32_t C2 = sh.count;
    uint32_t level_max = lmk;  // the thread maxima the current threshold was taken from
    bool fewer = false;        // the step below left fewer candidates than it found
    if (!many_groups && C2 > static_cast<uint32_t>(kFastCap)) {
        // More elements at or above thr than the list holds although only k+1 and a few
        // blocks reach it: those blocks' maxima are alike and so are their other elements
        // (a sorted row; the waves' shares of the block maxima are then not alike either, and
        // thr is lower than it need be).  The same step once more, a level down: every
        // thread takes the largest of the elements it reads from those blocks, and the
        // (k+1)-th largest of these thread maxima is a threshold as good as thr -- k+1
        // elements reach it, and whatever reaches it lies in a block whose maximum does --
        // and far tighter.
        const uint32_t before = C2;
        dry_max = 0;
        gather(thr, 1ull << 32, std::true_type{});
        level_max = dry_max;
        const uint32_t tight = threshold_of_thread_maxima(dry_max, false);  // (the barrier at the end of gather lies between this and the last use of its LDS)
        if (tid == 0) sh.count = 0;
        __syncthreads();
        thr = max(thr, tight);
        many_groups = gather(thr, 1ull << 32, std::false_type{});
        C2 = sh.count;
        fewer = C2 < before;
    }
    bool thr_is_exact = false;  // thr is the key of the row's (k+1)-th largest element
    if (!many_groups && C2 > static_cast<uint32_t>(kFastCap) && fewer) {
        // Still more than the list holds, but fewer than before: the blocks that reach thr are
        // full of elements that do (a row sorted in runs: k+1 blocks of 16 vectors whose every
        // element lies above the next block's maximum; the step above ends at one element per
        // vector at best -- 4 (k+1) of them, 8 (k+1) in half precision).  The (k+1)-th largest
        // of those blocks' elements is the row's, and a radix select finds it whatever the
        // values: four passes over the same blocks, eight bits of the key each, counted in LDS.
        // (As many as before means equal values en masse: the step below, without these passes.)
        uint32_t need = want;
        digit_prefix = 0;
        bool found = true;
        for (digit_shift = 24; digit_shift >= 0 && found; digit_shift -= 8) {
            __syncthreads();
            if (tid < 256u) digit_hist[tid] = 0;
            __syncthreads();
            gather(thr, 1ull << 32, std::integral_constant<int, 2>{});  // (ends with a barrier)
            if (wave == 0) {
                const uint2 r = hist256_resolve(digit_hist, need);
                if (lane == 0) {
                    sh.wave_thr[0] = r.x;
                    sh.wave_thr[1] = r.y;
                }
            }
            __syncthreads();
            const uint32_t d = sh.wave_thr[0];
            found = d < 256u;  // (k+1 elements reach thr, so a digit is always found)
            if (found) {
                digit_prefix |= d << digit_shift;
                need -= sh.wave_thr[1];
            }
        }
        __syncthreads();
        if (tid == 0) sh.count = 0;
        __syncthreads();
        if (found) {
            thr = max(thr, digit_prefix);
            thr_is_exact = true;
            many_groups = gather(thr, 1ull << 32, std::false_type{});
            C2 = sh.count;
        } else {
            many_groups = true;
        }
    }
    // Still too many: equal values en masse AT the threshold (rows of few distinct
    // values, constant rows).  k+1 elements reach thr, so the row's k+1 largest are the
    // elements above it -- fewer than k+1, or thr + 1 is the threshold to use -- and then
    // the first elements equal to it, in index order: those are found by reading the row
    // from its start, where a value this frequent turns up at once.
    bool first_equals_only = false;  // the candidates hold only some of the elements equal to thr
    if ((many_groups || C2 > static_cast<uint32_t>(kFastCap)) && !thr_is_exact) {
        // (thr so far is a value rounded down; this needs the key of an element: the exact
        // (k+1)-th largest of the thread maxima it came from)
        __syncthreads();
        thr = max(thr, threshold_of_thread_maxima(level_max, false, 32));
    }
    if ((many_groups || C2 > static_cast<uint32_t>(kFastCap)) && thr < 0xFFFFFFFFu) {
        __syncthreads();
        if (tid == 0) sh.count = 0;
        __syncthreads();
        const bool many_above = gather(thr + 1u, 1ull << 32, std::false_type{});
        const uint32_t above = sh.count;
        many_groups = true;  // (the exact select, unless one of the two cases below applies)
        if (!many_above && above <= static_cast<uint32_t>(kFastCap)) {
            if (above >= want) {
                thr += 1u;
                C2 = above;
                many_groups = false;
            } else {
                const uint32_t need = want - above, at = thr;
                const uint32_t found = first_members_by_scan<T, NT>(sh.scan_counts, rowp, n, need, at, at, scale,
                                                                    [&](uint32_t pos, uint32_t j) { sh.cand[above + pos] = composite(at, j); });
                __syncthreads();
                if (found >= need) {
                    if (tid == 0) sh.count = want;
                    __syncthreads();
                    C2 = want;
                    first_equals_only = true;
                    many_groups = false;
                }
            }
        }
    }
    if (!many_groups && C2 <= static_cast<uint32_t>(kFastCap)) {
        // Fewer than k+1 candidates: fewer than k+1 blocks hold an element above -inf,
        // every one of them was read again, and the rest of the row is -inf.
        const bool partial = C2 < min(want, n);
        // members of a tie across the k-th place below the value used above
        auto add_missing = [&](uint32_t xlo) -> bool {
            if (first_equals_only) {
                // the tied group reaches into values the candidates hold only in part: its
                // places are filled from the row's start, whatever the list holds
                __syncthreads();
                if (tid == 0) sh.count = kFastCap + 1;
                __syncthreads();
                return true;
            }
            if (xlo >= thr) return false;
            if (gather(xlo, thr, std::false_type{})) {
                if (tid == 0) sh.count = kFastCap + 1;  // too many to collect: the scan from the row's start
                __syncthreads();
            }
            return true;
        };
        BPS(12);
        finish_row<T, NT, SOFTMAX>(sh, C2, partial, M, s_base, rowp, ov, oi, n, kk, want, wave_of, add_missing, scale,
                                   counts != nullptr ? counts + row : nullptr, top_p);
        BPS(13);
#ifdef VKOP_STAMPS
        if (threadIdx.x == 0 && blockIdx.x == 0) g_bp_stamps[61] = clock64();
#endif
        return;
    }

    // ---- exact path: radix select over the whole row ----------------------------
    __syncthreads();  // LDS changes owner
    SelectShared &exact = smem.exact;
    if constexpr (SOFTMAX) {
        // the statistics the way the general kernels define them
        const LineStats st = line_stats<T, NT>(rowp, 0, n, 1, fscratch, dscratch, scale);
        select_topk_line<NT>(exact, n, kk, [&](uint32_t j) {
            return order_key(round_to_storage<T>(softmax_prob(scaled(load_elem(rowp, j), scale), st)));
        });
        for (uint32_t r = tid; r < kk; r += NT) {
            const uint32_t idx = composite_index(exact.sel[r]);
            store_elem(ov, r, softmax_prob(scaled(load_elem(rowp, idx), scale), st));
            oi[r] = static_cast<int32_t>(idx);
        }
        if (counts != nullptr) {
            // (rare path: the stored values are read back by the first wave, walked in order)
            __syncthreads();
            if (tid < static_cast<uint32_t>(kWave)) {
                const uint32_t count = nucleus_count_wave(kk, top_p, [&](uint32_t r) {
                    return round_to_storage<T>(softmax_prob(scaled(load_elem(rowp, composite_index(exact.sel[r])), scale), st));
                });
                if (lane == 0) counts[row] = static_cast<int32_t>(count);
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

// Launch: one workgroup of NT threads per row, after rows_scan_kernel on the same stream.
template <typename T, bool SOFTMAX, bool ALIGNED, int GE, bool SCALED = true, int NT = kPickThreads>
__global__ __launch_bounds__(NT) void rows_pick_kernel(const T *__restrict__ in, T *__restrict__ values,
                                                       int32_t *__restrict__ indices, uint32_t n, uint32_t k, uint32_t G,
                                                       uint32_t per, ScanWorkspace ws, float scale = 1.f,
                                                       int32_t *__restrict__ counts = nullptr, float top_p = 0.f) {
    __shared__ PickSharedUnion smem;
    __shared__ float fscratch[NT / kWave];
    __shared__ double dscratch[NT / kWave];
    VKOP_TL_BEGIN();
    pick_row<T, SOFTMAX, ALIGNED, GE, SCALED, NT>(smem, fscratch, dscratch, blockIdx.x, in, values, indices, n, k, G, per,
                                                         ws, scale, counts, top_p);
    VKOP_TL_END(1, ws.bmax, true);
}

}  // namespace vkop
