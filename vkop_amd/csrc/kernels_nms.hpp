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
//   3. the sorted list is walked: the first box still active is selected, every
//      thread tests its own later candidates against it (IoU as in
//      shaders/nms.comp:61-72, every operation rounded on its own so that the
//      comparison with the threshold is the same bit for bit on the host) and
//      clears their bits in the active mask; one barrier per selected box;
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
__global__ __launch_bounds__(kNmsThreads) void nms_kernel(const T *__restrict__ boxes, const T *__restrict__ scores,
                                                          int32_t *__restrict__ selected, uint32_t *__restrict__ counts,
                                                          uint32_t pairs, uint32_t C, uint32_t N, int center_point_box,
                                                          uint32_t max_out, float iou_threshold, float score_threshold,
                                                          uint32_t max_sel) {
    constexpr int NT = kNmsThreads;
    constexpr int NW = NT / kWave;
    constexpr int PER = kNmsMaxCandidates / NT;  // sorted candidates per thread
    __shared__ uint64_t comp[kNmsMaxCandidates];
    __shared__ float4 sbox[kNmsMaxCandidates];
    __shared__ uint32_t active[kNmsMaxCandidates / 32];
    __shared__ uint32_t wave_n[2][NW];
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t pair = blockIdx.x, batch = pair / C;
    const T *srow = scores + static_cast<size_t>(pair) * N;
    const T *brow = boxes + static_cast<size_t>(batch) * N * 4;

    // ---- 1. candidates, in box order ----------------------------------------------
    uint32_t found = 0, round = 0;  // the same in every thread
    for (uint32_t base = 0; base < N; base += NT, round++) {  // (to the end: the count tells whether boxes were left out)
        const uint32_t i = base + tid;
        const float s = load_elem(srow, i < N ? i : 0u);
        const bool pass = i < N && s > score_threshold;
        const uint64_t mask = __ballot(pass);
        uint32_t *wn = wave_n[round & 1u];
        if (lane == 0) wn[wave] = static_cast<uint32_t>(__popcll(mask));
        __syncthreads();
        uint32_t pos = found + lanes_below(mask), in_tile = 0;
#pragma unroll
        for (int w = 0; w < NW; w++) {
            const uint32_t c = wn[w];
            pos += (static_cast<uint32_t>(w) < wave) ? c : 0u;
            in_tile += c;
        }
        if (pass && pos < static_cast<uint32_t>(kNmsMaxCandidates)) comp[pos] = composite(order_key(s), i);
        found += in_tile;
    }
    const uint32_t K = min(found, static_cast<uint32_t>(kNmsMaxCandidates));
    uint32_t p2 = 1;
    while (p2 < K) p2 <<= 1;
    __syncthreads();
    for (uint32_t t = K + tid; t < p2; t += NT) comp[t] = 0;  // below every real composite
    for (uint32_t t = tid; t < static_cast<uint32_t>(kNmsMaxCandidates / 32); t += NT) {
        const uint32_t first = t * 32;
        active[t] = first + 32 <= K ? 0xFFFFFFFFu : (first < K ? ((1u << (K - first)) - 1u) : 0u);
    }
    __syncthreads();

    // ---- 2. by score, largest first; equal scores: lower box index first --------------
    if (K > 1) bitonic_sort_desc<NT>(comp, p2);
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

    // ---- 3. walk the list ---------------------------------------------------------
    const uint32_t limit = max_out > 0 ? min(max_out, K) : K;
    uint32_t chosen = 0, cur = 0;
    while (chosen < limit) {
        // first active position at or after cur (every thread finds the same one)
        uint32_t pos = K;
        for (uint32_t w = cur / 32; w * 32 < K; w++) {
            uint32_t bits = active[w];
            if (w == cur / 32) bits &= 0xFFFFFFFFu << (cur % 32);
            if (bits) {
                pos = w * 32 + static_cast<uint32_t>(__ffs(static_cast<int>(bits))) - 1u;
                break;
            }
        }
        if (pos >= K) break;
        if (tid == 0 && chosen < max_sel)
            selected[static_cast<size_t>(pair) * max_sel + chosen] = static_cast<int32_t>(composite_index(comp[pos]));
        chosen++;
        const float4 best = sbox[pos];
#pragma unroll
        for (int e = 0; e < PER; e++) {
            const uint32_t p = static_cast<uint32_t>(e) * NT + tid;
            if (p > pos && p < K && ((active[p / 32] >> (p % 32)) & 1u) && nms_iou(mine[e], best) > iou_threshold)
                atomicAnd(&active[p / 32], ~(1u << (p % 32)));
        }
        __syncthreads();
        cur = pos + 1;
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
