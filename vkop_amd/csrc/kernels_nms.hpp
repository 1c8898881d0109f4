// Non-maximum suppression: the operator behind the detection chain's top-k.
//
// boxes [B][N][4], scores [B][C][N].  One workgroup per (batch, class), as in the
// reference (ops/Nms.hpp:115, shaders/nms.comp:74-82), but every phase is done by
// the whole workgroup instead of its first thread:
//   1. the boxes whose score is greater than the threshold are collected in box
//      order (ballot prefix per tile of 1024 boxes), at most kNmsMaxCandidates;
//   2. they are sorted by (score, then lower box index) with a bitonic network over
//      64-bit composites in LDS, and their corner coordinates are staged in LDS in
//      that order;
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

constexpr int kNmsThreads = 1024;
constexpr int kNmsMaxCandidates = 2048;  // per (batch, class); the reference's shader holds 1024
constexpr int kNmsRankSortMax = 512;     // up to here a counting sort beats the bitonic network's barriers

__device__ __forceinline__ uint32_t uniform_u32(uint32_t x) {
    return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(x)));
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
// selected: [pairs][max_sel] box indices.  Launch: B * C workgroups of kNmsThreads.
template <typename T>
__global__ __launch_bounds__(kNmsThreads) __attribute__((amdgpu_waves_per_eu(8))) void nms_kernel(const T *__restrict__ boxes, const T *__restrict__ scores,
                                                          int32_t *__restrict__ selected, uint32_t *__restrict__ counts,
                                                          uint32_t pairs, uint32_t C, uint32_t N, int center_point_box,
                                                          uint32_t max_out, float iou_threshold, float score_threshold,
                                                          uint32_t max_sel) {
    constexpr int NT = kNmsThreads;
    constexpr int NW = NT / kWave;
    constexpr int PER = kNmsMaxCandidates / NT;  // sorted candidates per thread
    __shared__ uint64_t comp[kNmsMaxCandidates];
    __shared__ float4 sbox[kNmsMaxCandidates];
    __shared__ unsigned long long active[kNmsMaxCandidates / 64];
    __shared__ unsigned long long block_cols[kWave];
    __shared__ unsigned long long block_keep;
    constexpr int TILES = 12;  // scores per thread and round
    __shared__ uint32_t wave_n[2][NW];
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t pair = blockIdx.x, batch = pair / C;
    const T *srow = scores + static_cast<size_t>(pair) * N;
    const T *brow = boxes + static_cast<size_t>(batch) * N * 4;

    // ---- 1. candidates, in box order ----------------------------------------------
    // A round covers NT * TILES boxes, each wave a contiguous run of them, so that all of a thread's scores are
    // in flight together and the places inside a wave follow from scalar counts; one barrier per round.
    uint32_t found = 0, round = 0;  // the same in every thread
    for (uint32_t base = 0; base < N; base += NT * TILES, round++) {  // (to the end: the count tells whether boxes were left out)
        const uint32_t tiles = min(static_cast<uint32_t>(TILES), (N - base + NT - 1) / NT);  // per wave, this round
        const uint32_t first = base + wave * tiles * kWave + lane;
        float s[TILES];
#pragma unroll
        for (int u = 0; u < TILES; u++) {
            const uint32_t i = first + static_cast<uint32_t>(u) * kWave;
            s[u] = load_elem(srow, (static_cast<uint32_t>(u) < tiles && i < N) ? i : 0u);
        }
        uint32_t in_wave = 0;
#pragma unroll
        for (int u = 0; u < TILES; u++) {
            const uint32_t i = first + static_cast<uint32_t>(u) * kWave;
            in_wave += static_cast<uint32_t>(__popcll(__ballot(static_cast<uint32_t>(u) < tiles && i < N && s[u] > score_threshold)));
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
#pragma unroll
        for (int u = 0; u < TILES; u++) {
            const uint32_t i = first + static_cast<uint32_t>(u) * kWave;
            const bool pass = static_cast<uint32_t>(u) < tiles && i < N && s[u] > score_threshold;
            const uint64_t mask = __ballot(pass);  // (again rather than kept: a dozen masks crowd the scalar registers)
            const uint32_t at = pos + lanes_below(mask);
            if (pass && at < static_cast<uint32_t>(kNmsMaxCandidates)) comp[at] = composite(order_key(s[u]), i);
            pos += static_cast<uint32_t>(__popcll(mask));
        }
    }
    const uint32_t K = min(found, static_cast<uint32_t>(kNmsMaxCandidates));
    uint32_t p2 = 1;
    while (p2 < K) p2 <<= 1;
    __syncthreads();
    for (uint32_t t = K + tid; t < p2; t += NT) comp[t] = 0;  // below every real composite
    if (tid >= NT - kWave) block_cols[lane] = 0;
    if (tid < static_cast<uint32_t>(kNmsMaxCandidates / 64)) {
        const uint32_t first = tid * 64;
        active[tid] = first + 64 <= K ? ~0ull : (first < K ? ((1ull << (K - first)) - 1ull) : 0ull);
    }
    __syncthreads();

    // ---- 2. by score, largest first; equal scores: lower box index first --------------
    if (K > static_cast<uint32_t>(kNmsRankSortMax)) {
        bitonic_sort_desc<NT>(comp, p2);
    } else if (K > 1) {
        // few candidates: each counts the composites above its own (all distinct) and moves there; two barriers
        // instead of one per step of the network
        const uint64_t c = tid < K ? comp[tid] : 0;
        uint32_t rank = 0;
        if (tid < K) {
#pragma unroll 8
            for (uint32_t q = 0; q < K; q++) rank += comp[q] > c ? 1u : 0u;
        }
        __syncthreads();
        if (tid < K) comp[rank] = c;
        __syncthreads();
    }
    float4 mine[PER];
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
            sbox[p] = b;
        }
    }
    __syncthreads();

    // ---- 3. walk the list, 64 candidates at a time ------------------------------------
    const uint32_t limit = max_out > 0 ? min(max_out, K) : K;
    uint32_t chosen = 0;
    for (uint32_t base = 0; base < K && chosen < limit; base += kWave) {
        // a. for candidate i of the block (one per lane, in every wave) the earlier candidates of the block that
        //    would suppress it: each wave tests four of them and adds its four bits to the lane's word
        //    (positions at or after K hold nothing: they are never active below)
        const float4 bi = sbox[base + lane];
        uint32_t bits = 0;
#pragma unroll
        for (int r = 0; r < kWave / NW; r++) {
            const uint32_t j = wave * (kWave / NW) + static_cast<uint32_t>(r);
            if (lane > j && nms_iou(bi, sbox[base + j]) > iou_threshold) bits |= 1u << r;
        }
        if (bits != 0) atomicOr(&block_cols[lane], static_cast<unsigned long long>(bits) << (wave * (kWave / NW)));
        __syncthreads();  // (also: the bits cleared by the block before are in place)
        // b. the first wave resolves the block.  Kept = active and suppressed by nobody kept before it: that set is
        //    the only fixed point of  S -> { i active : no member of S suppresses i },  and iterating from any S
        //    reaches it, one more leading position settled per step at worst, a handful of steps as a rule.
        if (wave == 0) {
            const unsigned long long col = block_cols[lane];
            block_cols[lane] = 0;  // for the next block (its additions come after the next barrier)
            const bool alive = (active[base / kWave] >> lane) & 1ull;
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
                    dead = nms_iou(mine[e], sbox[base + static_cast<uint32_t>(__builtin_ctzll(kk))]) > iou_threshold;
                if (dead) atomicAnd(&active[p / 64], ~(1ull << (p % 64)));
            }
        }
        // (no barrier here: a. of the next block touches neither the mask nor block_keep, and its barrier orders the rest)
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
