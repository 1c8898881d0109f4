// Non-maximum suppression: the operator behind the detection chain's top-k.
//
// boxes [B][N][4], scores [B][C][N].  One workgroup per (batch, class), as in the
// reference (ops/Nms.hpp:115, shaders/nms.comp:74-82), but every phase is done by
// the whole workgroup instead of its first thread:
//   1. the boxes whose score is greater than the threshold are collected in box
//      order (ballot prefix per tile of 1024 boxes), at most kNmsMaxCandidates;
//   2. they are sorted by (score, then lower box index) as 64-bit composites in LDS
//      (counting sort for few, bitonic network for many), and every thread loads the
//      corner coordinates of its own sorted positions into registers;
//   3. the sorted list is walked in blocks of 64: all waves compute, for every
//      candidate of the block, which earlier ones of the block would suppress it
//      (IoU as in shaders/nms.comp:61-72, every operation rounded on its own so
//      that the comparison with the threshold is the same bit for bit on the
//      host); the first wave finds the kept set with a few ballots (a fixed-point
//      iteration instead of one step per kept box); then every thread tests its
//      own later candidates against the block's survivors and clears their bits
//      in the active mask; two barriers per block of 64 instead of one per
//      selection;
//   4. the selected box indices go to the pair's segment of the workspace.
// nms_pack_kernel then writes the (batch, class, box) records of all pairs one
// after the other, in order of batch and class: the result does not depend on
// scheduling (the reference appends through a global atomic counter).
#pragma once

#include "device_utils.hpp"
#include "kernels_rows.hpp"
#include "select.hpp"

namespace vkop {

constexpr int kNmsThreadsWide = 1024;   // few (batch, class) pairs
constexpr int kNmsThreadsNarrow = 256;  // many
constexpr int kNmsNarrowMinPairs = 1024;
constexpr int kNmsMaxCandidates = 2048;  // per (batch, class); the reference's shader holds 1024
constexpr int kNmsRankSortMax = 512;     // up to here a counting sort beats the bitonic network's barriers

__device__ __forceinline__ uint32_t uniform_u32(uint32_t x) {
    return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(x)));
}

// Four consecutive scores starting at element i (i a multiple of four, the row 16-byte aligned).
__device__ __forceinline__ float4 nms_load4(const float *p, uint32_t i) { return *reinterpret_cast<const float4 *>(p + i); }
__device__ __forceinline__ float4 nms_load4(const uint16_t *p, uint32_t i) {
    const uint2 w = *reinterpret_cast<const uint2 *>(p + i);
    return make_float4(__half2float(__ushort_as_half(static_cast<unsigned short>(w.x & 0xFFFFu))),
                       __half2float(__ushort_as_half(static_cast<unsigned short>(w.x >> 16))),
                       __half2float(__ushort_as_half(static_cast<unsigned short>(w.y & 0xFFFFu))),
                       __half2float(__ushort_as_half(static_cast<unsigned short>(w.y >> 16))));
}

__device__ __forceinline__ float nms_iou(const float4 &a, const float4 &b) {
    const float x1 = fmaxf(a.x, b.x), y1 = fmaxf(a.y, b.y), x2 = fminf(a.z, b.z), y2 = fminf(a.w, b.w);
    if (x2 <= x1 || y2 <= y1) return 0.f;
    const float inter = __fmul_rn(__fsub_rn(x2, x1), __fsub_rn(y2, y1));
    const float area_a = __fmul_rn(__fsub_rn(a.z, a.x), __fsub_rn(a.w, a.y));
    const float area_b = __fmul_rn(__fsub_rn(b.z, b.x), __fsub_rn(b.w, b.y));
    const float uni = __fsub_rn(__fadd_rn(area_a, area_b), inter);
    return uni > 0.f ? __fdiv_rn(inter, uni) : 0.f;
}

// counts[pair] = boxes selected; counts[pairs + pair] = 1 if more than
// kNmsMaxCandidates boxes passed the score threshold (the later ones were left out).
// selected: [pairs][max_sel] box indices.  Launch: B * C workgroups of NT threads:
// 1024 when there are few pairs (one pair's work spread wide), 256 when there are
// enough pairs to put many workgroups on a CU, so that one's score loads overlap
// another's sort and walk.  Each thread keeps the boxes of its own kNmsMaxCandidates / NT
// sorted candidates in registers; LDS holds the composites and two blocks of 64 boxes.
template <typename T, int NT, bool VEC>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(NT >= 1024 ? 8 : 6))) void nms_kernel(
    const T *__restrict__ boxes, const T *__restrict__ scores, int32_t *__restrict__ selected, uint32_t *__restrict__ counts,
    uint32_t pairs, uint32_t C, uint32_t N, int center_point_box, uint32_t max_out, float iou_threshold, float score_threshold,
    uint32_t max_sel) {
    static_assert(NT % kWave == 0 && kNmsMaxCandidates % NT == 0 && (kNmsRankSortMax % NT == 0 || NT % kNmsRankSortMax == 0), "workgroup size");
    constexpr int NW = NT / kWave;
    constexpr int PER = kNmsMaxCandidates / NT;      // sorted candidates per thread
    constexpr int SMALL = NT >= kNmsRankSortMax ? 1 : kNmsRankSortMax / NT;  // of them, when the counting sort applies
    constexpr int JP = kWave / NW;                   // candidates of a block each wave tests the block against
    constexpr int TILES = NT >= 1024 ? 12 : 36;      // scores per thread and round
    __shared__ uint64_t comp[kNmsMaxCandidates];
    __shared__ float4 block_box[2][kWave];
    __shared__ unsigned long long active[kNmsMaxCandidates / 64];
    __shared__ unsigned long long block_cols[kWave];
    __shared__ unsigned long long block_keep;
    __shared__ uint32_t wave_n[2][NW];
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = uniform_u32(tid) / kWave;  // (scalar)
    const uint32_t pair = blockIdx.x, batch = pair / C;
    const T *srow = scores + static_cast<size_t>(pair) * N;
    const T *brow = boxes + static_cast<size_t>(batch) * N * 4;
    if (tid < static_cast<uint32_t>(kNmsMaxCandidates / 64)) active[tid] = ~0ull;  // positions at or after K are masked where read
    if (tid >= NT - kWave) block_cols[lane] = 0;

    // ---- 1. candidates, in box order ----------------------------------------------
    // A round covers NT * TILES boxes, each wave a contiguous run of them (tiles of 64), so that all of a thread's
    // scores are in flight together; one barrier per round.  Candidates are rare in a detection head, and every
    // wave instruction here is paid NT / 64 times per workgroup: per tile the vector unit sees the load, its
    // address and one comparison per pass; tile bounds, counts and places are scalar, and a tile without a
    // candidate is left with one scalar branch.
    uint32_t found = 0, round = 0;  // the same in every thread
    if constexpr (VEC) {
        // Rows that start on a 16-byte boundary and hold a multiple of four scores: a lane takes four consecutive
        // scores with one load, a quarter of the loads, addresses and bounds checks of the form below.  Places stay
        // in box order: lanes below, then the lane's own components below.
        constexpr int VT = TILES / 4;
        for (uint32_t base = 0; base < N; base += NT * TILES, round++) {
            const uint32_t tiles = min(static_cast<uint32_t>(VT), (N - base + NT * 4 - 1) / (NT * 4));  // per wave, this round
            const uint32_t wave_first = base + wave * tiles * (kWave * 4);
            float4 s[VT];
#pragma unroll
            for (int u = 0; u < VT; u++)  // (past the end of the row: its last four again, masked out below)
                s[u] = nms_load4(srow, min(wave_first + static_cast<uint32_t>(u) * (kWave * 4) + lane * 4, N - 4));
            const int32_t reach = static_cast<int32_t>(min(N - min(N, wave_first), tiles * (kWave * 4))) - static_cast<int32_t>(lane * 4);
            uint32_t in_wave = 0;
#pragma unroll
            for (int u = 0; u < VT; u++) {
                const bool here = reach > u * (kWave * 4);
                in_wave += static_cast<uint32_t>(__popcll(__ballot(here && s[u].x > score_threshold)) + __popcll(__ballot(here && s[u].y > score_threshold)) +
                                                 __popcll(__ballot(here && s[u].z > score_threshold)) + __popcll(__ballot(here && s[u].w > score_threshold)));
            }
            if (lane == 0) wave_n[round & 1u][wave] = in_wave;
            __syncthreads();
            uint32_t pos = found;
#pragma unroll
            for (int w = 0; w < NW; w++) {
                const uint32_t c = wave_n[round & 1u][w];
                pos += (static_cast<uint32_t>(w) < wave) ? c : 0u;
                found += c;
            }
            if (in_wave != 0) {
#pragma unroll
                for (int u = 0; u < VT; u++) {
                    asm volatile("" : "+v"(s[u].x), "+v"(s[u].y), "+v"(s[u].z), "+v"(s[u].w));  // (masks again, not kept: see below)
                    const bool here = reach > u * (kWave * 4);
                    const float v[4] = {s[u].x, s[u].y, s[u].z, s[u].w};
                    uint64_t mask[4];
#pragma unroll
                    for (int c = 0; c < 4; c++) mask[c] = __ballot(here && v[c] > score_threshold);
                    if ((mask[0] | mask[1] | mask[2] | mask[3]) != 0) {
                        asm volatile("; four tiles with candidates");  // (a real branch)
                        uint32_t at = pos + lanes_below(mask[0]) + lanes_below(mask[1]) + lanes_below(mask[2]) + lanes_below(mask[3]);
#pragma unroll
                        for (int c = 0; c < 4; c++) {
                            if ((mask[c] >> lane) & 1ull) {
                                if (at < static_cast<uint32_t>(kNmsMaxCandidates))
                                    comp[at] = composite(order_key(v[c]), wave_first + static_cast<uint32_t>(u) * (kWave * 4) + lane * 4 + static_cast<uint32_t>(c));
                                at++;
                            }
                            pos += static_cast<uint32_t>(__popcll(mask[c]));
                        }
                    }
                }
            }
        }
    } else
    for (uint32_t base = 0; base < N; base += NT * TILES, round++) {  // (to the end: the count tells whether boxes were left out)
        const uint32_t tiles = min(static_cast<uint32_t>(TILES), (N - base + NT - 1) / NT);  // per wave, this round
        const uint32_t wave_first = base + wave * tiles * kWave;
        float s[TILES];
#pragma unroll
        for (int u = 0; u < TILES; u++)  // (past the end of the row: its last score again, masked out below)
            s[u] = load_elem(srow, min(wave_first + static_cast<uint32_t>(u) * kWave + lane, N - 1));
        // lane l's score of tile u exists iff u * 64 < reach: inside the row and inside this wave's run
        const int32_t reach = static_cast<int32_t>(min(N - min(N, wave_first), tiles * kWave)) - static_cast<int32_t>(lane);
        auto candidates = [&](int u) -> uint64_t { return __ballot(s[u] > score_threshold && reach > u * kWave); };
        uint32_t in_wave = 0;
#pragma unroll
        for (int u = 0; u < TILES; u++) in_wave += static_cast<uint32_t>(__popcll(candidates(u)));
        if (lane == 0) wave_n[round & 1u][wave] = in_wave;
        __syncthreads();
        uint32_t pos = found;
#pragma unroll
        for (int w = 0; w < NW; w++) {
            const uint32_t c = wave_n[round & 1u][w];
            pos += (static_cast<uint32_t>(w) < wave) ? c : 0u;
            found += c;
        }
        if (in_wave != 0) {
#pragma unroll
            for (int u = 0; u < TILES; u++) {
                // (again rather than kept: dozens of masks crowd the scalar registers and get spilled; the empty
                //  statement keeps the compiler from reusing the first pass's)
                asm volatile("" : "+v"(s[u]));
                const uint64_t mask = candidates(u);
                if (mask != 0) {
                    asm volatile("; a tile with candidates");  // (a real branch: as straight-line code all tiles pay for the few)
                    const uint32_t at = pos + lanes_below(mask);
                    if (((mask >> lane) & 1ull) && at < static_cast<uint32_t>(kNmsMaxCandidates))
                        comp[at] = composite(order_key(s[u]), wave_first + static_cast<uint32_t>(u) * kWave + lane);
                    pos += static_cast<uint32_t>(__popcll(mask));
                }
            }
        }
    }
    const uint32_t K = min(found, static_cast<uint32_t>(kNmsMaxCandidates));
    __syncthreads();

    // ---- 2. by score, largest first; equal scores: lower box index first --------------
    if (K > static_cast<uint32_t>(kNmsRankSortMax)) {
        uint32_t p2 = 1;
        while (p2 < K) p2 <<= 1;
        for (uint32_t t = K + tid; t < p2; t += NT) comp[t] = 0;  // below every real composite
        __syncthreads();
        bitonic_sort_desc<NT>(comp, p2);
    } else if (K > 1) {
        // few candidates: each counts the composites above its own (all distinct) and moves there; two barriers
        // instead of one per step of the network
        uint64_t c[SMALL];
        uint32_t rank[SMALL];
#pragma unroll
        for (int e = 0; e < SMALL; e++) {
            const uint32_t p = static_cast<uint32_t>(e) * NT + tid;
            c[e] = p < K ? comp[p] : 0;
            rank[e] = 0;
        }
        if (tid < K) {
#pragma unroll 16
            for (uint32_t q = 0; q < K; q++) {
                const uint64_t other = comp[q];
                rank[0] += other > c[0] ? 1u : 0u;
            }
#pragma unroll
            for (int e = 1; e < SMALL; e++) {
                if (K > static_cast<uint32_t>(e) * NT) {  // (the same for the whole workgroup)
#pragma unroll 16
                    for (uint32_t q = 0; q < K; q++) rank[e] += comp[q] > c[e] ? 1u : 0u;
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < SMALL; e++)
            if (static_cast<uint32_t>(e) * NT + tid < K) comp[rank[e]] = c[e];
        __syncthreads();
    }
    float4 mine[PER];  // corners of this thread's candidates: sorted positions e * NT + tid
#pragma unroll
    for (int e = 0; e < PER; e++) {
        const uint32_t p = static_cast<uint32_t>(e) * NT + tid;
        mine[e] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (p < K) {
            const T *r = brow + static_cast<size_t>(composite_index(comp[p])) * 4;
            float4 b = make_float4(load_elem(r, 0), load_elem(r, 1), load_elem(r, 2), load_elem(r, 3));
            if (center_point_box) {  // (x_center, y_center, width, height), shaders/nms.comp:55-58
                const float hw = b.z * 0.5f, hh = b.w * 0.5f;
                b = make_float4(__fsub_rn(b.x, hw), __fsub_rn(b.y, hh), __fadd_rn(b.x, hw), __fadd_rn(b.y, hh));
            }
            mine[e] = b;
        }
    }

    // ---- 3. walk the list, 64 candidates at a time ------------------------------------
    const uint32_t limit = max_out > 0 ? min(max_out, K) : K;
    uint32_t chosen = 0;
    for (uint32_t base = 0; base < K && chosen < limit; base += kWave) {
        // the block's boxes go to LDS: its 64 positions belong to the lanes of one wave (two buffers in turn:
        // the block before may still be read by slower waves in step c)
        float4(&box)[kWave] = block_box[(base / kWave) & 1u];
        if (wave == (base % NT) / kWave) {
            float4 b = mine[0];
#pragma unroll
            for (int e = 1; e < PER; e++)
                if (static_cast<uint32_t>(e) == base / NT) b = mine[e];
            box[lane] = b;
        }
        __syncthreads();
        // a. for candidate i of the block (one per lane, in every wave) the earlier candidates of the block that
        //    would suppress it: each wave tests JP of them and adds its bits to the lane's word
        //    (positions at or after K hold zeros: they are never active below)
        const float4 bi = box[lane];
        uint32_t bits = 0;
#pragma unroll
        for (int r = 0; r < JP; r++) {
            const uint32_t j = wave * JP + static_cast<uint32_t>(r);
            if (lane > j && nms_iou(bi, box[j]) > iou_threshold) bits |= 1u << r;
        }
        if (bits != 0) atomicOr(&block_cols[lane], static_cast<unsigned long long>(bits) << (wave * JP));
        __syncthreads();  // (also: the bits cleared by the block before are in place)
        // b. the first wave resolves the block.  Kept = active and suppressed by nobody kept before it: that set is
        //    the only fixed point of  S -> { i active : no member of S suppresses i },  and iterating from any S
        //    reaches it, one more leading position settled per step at worst, a handful of steps as a rule.
        if (wave == 0) {
            const unsigned long long col = block_cols[lane];
            block_cols[lane] = 0;  // for the next block (its additions come after the next barrier)
            const bool alive = base + lane < K && ((active[base / kWave] >> lane) & 1ull);
            uint64_t keep = __ballot(alive);
            for (int step = 0; step < kWave; step++) {
                const uint64_t next = __ballot(alive && (col & keep) == 0);
                if (next == keep) break;
                keep = next;
            }
            const uint32_t room = limit - chosen;  // > 0 here
            if (static_cast<uint32_t>(__popcll(keep)) > room) keep = __ballot(((keep >> lane) & 1ull) && lanes_below(keep) < room);
            if (lane == 0) block_keep = keep;
            if ((keep >> lane) & 1u) {
                const uint32_t slot = chosen + lanes_below(keep);
                if (slot < max_sel)
                    selected[static_cast<size_t>(pair) * max_sel + slot] = static_cast<int32_t>(composite_index(comp[base + lane]));
            }
        }
        __syncthreads();
        const unsigned long long kept = block_keep;
        const uint64_t keep = (static_cast<uint64_t>(uniform_u32(static_cast<uint32_t>(kept >> 32))) << 32) |
                              uniform_u32(static_cast<uint32_t>(kept));
        chosen += static_cast<uint32_t>(__popcll(keep));
        if (chosen >= limit) break;
        // c. every later candidate still active against the block's survivors
#pragma unroll
        for (int e = 0; e < PER; e++) {
            const uint32_t p = static_cast<uint32_t>(e) * NT + tid;
            if (p >= base + kWave && p < K && ((active[p / 64] >> (p % 64)) & 1ull)) {
                bool dead = false;
                for (uint64_t kk = keep; kk != 0 && !dead; kk &= kk - 1)
                    dead = nms_iou(mine[e], box[static_cast<uint32_t>(__builtin_ctzll(kk))]) > iou_threshold;
                if (dead) atomicAnd(&active[p / 64], ~(1ull << (p % 64)));
            }
        }
        // (no barrier here: the next block writes the other box buffer, and its barriers order the rest)
    }
    if (tid == 0) {
        counts[pair] = min(chosen, max_sel);
        counts[pairs + pair] = found > static_cast<uint32_t>(kNmsMaxCandidates) ? 1u : 0u;
    }
}

// The records of all pairs one after the other.  out: [capacity][3]; out_count[0] =
// records in all (also when capacity holds fewer), out_count[1] = 1 if some pair
// had more candidates than kNmsMaxCandidates; a (-1,-1,-1) record follows the last
// one when capacity allows.  Launch: B * C workgroups of 256.
__global__ __launch_bounds__(256) void nms_pack_kernel(const int32_t *__restrict__ selected,
                                                              const uint32_t *__restrict__ counts, int32_t *__restrict__ out,
                                                              int32_t *__restrict__ out_count, uint32_t pairs, uint32_t C,
                                                              uint32_t max_sel, uint32_t capacity) {
    __shared__ uint32_t scratch[256 / kWave];
    const uint32_t tid = threadIdx.x, pair = blockIdx.x;
    uint32_t before = 0, over = 0;
    for (uint32_t q = tid; q < pairs; q += 256) {
        if (q < pair) before += counts[q];
        over |= counts[pairs + q];
    }
    before = wave_sum(before);
    over = wave_sum(over);
    if ((tid & (kWave - 1)) == 0) scratch[tid / kWave] = before;
    __syncthreads();
    uint32_t offset = 0;
    for (int w = 0; w < 256 / kWave; w++) offset += scratch[w];
    __syncthreads();
    if ((tid & (kWave - 1)) == 0) scratch[tid / kWave] = over;
    __syncthreads();
    const uint32_t n = counts[pair];
    for (uint32_t r = tid; r < n; r += 256) {
        const uint32_t o = offset + r;
        if (o < capacity) {
            out[static_cast<size_t>(o) * 3 + 0] = static_cast<int32_t>(pair / C);
            out[static_cast<size_t>(o) * 3 + 1] = static_cast<int32_t>(pair % C);
            out[static_cast<size_t>(o) * 3 + 2] = selected[static_cast<size_t>(pair) * max_sel + r];
        }
    }
    if (pair == pairs - 1 && tid == 0) {
        uint32_t any = 0;
        for (int w = 0; w < 256 / kWave; w++) any |= scratch[w];
        const uint32_t total = offset + n;
        out_count[0] = static_cast<int32_t>(total);
        out_count[1] = any ? 1 : 0;
        if (total < capacity) {  // end of the list for a reader of the tensor alone (the reference writes such a record too)
            out[static_cast<size_t>(total) * 3 + 0] = -1;
            out[static_cast<size_t>(total) * 3 + 1] = -1;
            out[static_cast<size_t>(total) * 3 + 2] = -1;
        }
    }
}

}  // namespace vkop
