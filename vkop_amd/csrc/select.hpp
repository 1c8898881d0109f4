// Exact top-k of one line by a single workgroup: radix select over the 64-bit
// composite (order key, ~index), then an LDS bitonic sort of the k winners.
//
// This is the general routine: any line length, any k <= kMaxK, any key
// function, any amount of ties (the composite is unique per element, so ties
// are resolved by position inside the select itself).  It makes one pass over
// the line per 8 bits it has to resolve -- typically 2-3 passes, 8 at most --
// plus one gathering pass, so it is used where a line is short, where the data
// is pathological for the streaming kernels, and as their exact fallback.
#pragma once

#include "device_utils.hpp"

namespace vkop {

constexpr int kMaxK = 2048;  // == VKOP_HIP_MAX_K

struct SelectShared {
    uint64_t sel[kMaxK];  // gathered winners, then sorted in place
    uint32_t hist[256];
    uint32_t wave_tot[16];
    uint32_t count;       // gather cursor
    uint32_t digit;       // chosen digit of the current pass
    uint32_t need;        // winners still to take inside the chosen bucket
    uint32_t bucket;      // population of the chosen bucket
};

// Bitonic sort of sel[0..p2) (p2 a power of two) into descending order by all
// NT threads of the workgroup; sel lives in LDS.  Ends with a barrier.
template <int NT> __device__ __forceinline__ void bitonic_sort_desc(uint64_t *sel, uint32_t p2) {
    const uint32_t tid = threadIdx.x;
    for (uint32_t size = 2; size <= p2; size <<= 1) {
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            for (uint32_t t = tid; t < (p2 >> 1); t += NT) {
                const uint32_t i = ((t & ~(stride - 1)) << 1) | (t & (stride - 1));
                const uint32_t j = i | stride;
                const uint64_t a = sel[i], b = sel[j];
                const bool desc = ((i & size) == 0);
                if (desc ? (a < b) : (a > b)) {
                    sel[i] = b;
                    sel[j] = a;
                }
            }
            __syncthreads();
        }
    }
}

// KeyFn: uint32_t operator()(uint32_t j) -> order key of element j of the line.
// On return sh.sel[0..k) holds the k largest composites in descending order
// (rank order) and all threads have passed a barrier.
template <int NT, typename KeyFn>
__device__ __forceinline__ void select_topk_line(SelectShared &sh, uint32_t n, uint32_t k, KeyFn keyfn) {
    static_assert(NT % kWave == 0 && NT >= kWave && NT <= 1024, "block size");
    const uint32_t tid = threadIdx.x;
    uint64_t prefix = 0;  // the top `bits` bits every winner-or-better shares or exceeds
    int bits = 0;
    uint32_t need = k;

    for (int pass = 0; pass < 8; pass++) {
        for (uint32_t t = tid; t < 256; t += NT) sh.hist[t] = 0;
        __syncthreads();
        const int shift = 64 - bits - 8;
        for (uint32_t j = tid; j < n; j += NT) {
            const uint64_t c = composite(keyfn(j), j);
            if (bits == 0 || (c >> (64 - bits)) == prefix)
                hist_add_grouped(sh.hist, static_cast<uint32_t>(c >> shift) & 0xFFu);
        }
        __syncthreads();
        // Wave 0 locates the digit d with  #(digit > d) < need <= #(digit >= d).
        if (tid < kWave) {
            const uint32_t h0 = sh.hist[tid * 4 + 0], h1 = sh.hist[tid * 4 + 1];
            const uint32_t h2 = sh.hist[tid * 4 + 2], h3 = sh.hist[tid * 4 + 3];
            const uint32_t mine = h0 + h1 + h2 + h3;
            // inclusive suffix sum over lanes: lanes above hold the higher digits
            uint32_t suf = mine;
#pragma unroll
            for (int o = 1; o < kWave; o <<= 1) {
                const uint32_t up = __shfl_down(suf, o, kWave);
                if (tid + o < kWave) suf += up;
            }
            uint32_t above = suf - mine;  // population of digits in higher lanes
            // walk this lane's four digits from the top
            const uint32_t hh[4] = {h3, h2, h1, h0};
#pragma unroll
            for (int q = 0; q < 4; q++) {
                if (above < need && need <= above + hh[q]) {
                    sh.digit = tid * 4 + (3 - q);
                    sh.need = need - above;
                    sh.bucket = hh[q];
                }
                above += hh[q];
            }
        }
        __syncthreads();
        prefix = (prefix << 8) | sh.digit;
        need = sh.need;
        bits += 8;
        const bool done = (need == sh.bucket);
        __syncthreads();  // sh.digit / sh.need are rewritten next pass
        if (done) break;
    }

    // Gather: everything whose top `bits` bits are >= prefix (exactly k elements).
    if (tid == 0) sh.count = 0;
    __syncthreads();
    for (uint32_t j = tid; j < n; j += NT) {
        const uint64_t c = composite(keyfn(j), j);
        const uint64_t top = (bits == 64) ? c : (c >> (64 - bits));
        if (top >= prefix) {
            const uint32_t pos = atomicAdd(&sh.count, 1u);
            if (pos < kMaxK) sh.sel[pos] = c;
        }
    }
    uint32_t p2 = 1;
    while (p2 < k) p2 <<= 1;
    for (uint32_t t = k + tid; t < p2; t += NT) sh.sel[t] = 0;  // below every real composite
    __syncthreads();

    bitonic_sort_desc<NT>(sh.sel, p2);
}

}  // namespace vkop
