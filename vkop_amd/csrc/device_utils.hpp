// Device-side building blocks shared by the softmax / top-k kernels (gfx950,
// wave64).  Header only; every function is __device__ __forceinline__.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace vkop {

constexpr int kWave = 64;

// ---------------------------------------------------------------- loads ----

// Element of a float or half (uint16_t bits) tensor, widened to float.
template <typename T> __device__ __forceinline__ float load_elem(const T *p, size_t i);
template <> __device__ __forceinline__ float load_elem<float>(const float *p, size_t i) { return p[i]; }
template <> __device__ __forceinline__ float load_elem<uint16_t>(const uint16_t *p, size_t i) {
    return __half2float(__ushort_as_half(p[i]));
}

// Round-to-nearest-even store of a float into a float or half tensor.
template <typename T> __device__ __forceinline__ void store_elem(T *p, size_t i, float v);
template <> __device__ __forceinline__ void store_elem<float>(float *p, size_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void store_elem<uint16_t>(uint16_t *p, size_t i, float v) {
    p[i] = __half_as_ushort(__float2half_rn(v));
}

// Value as the tensor type would hold it (float stays, half is rounded to
// binary16 and widened again).
template <typename T> __device__ __forceinline__ float round_to_storage(float v);
template <> __device__ __forceinline__ float round_to_storage<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_to_storage<uint16_t>(float v) {
    return __half2float(__float2half_rn(v));
}

// x * scale rounded to float on its own: never contracted into a fused multiply-add
// with what follows, so that a kernel given a scale computes on exactly the values
// a tensor scaled beforehand would hold.
// (the empty asm hides the product from the optimizer; `__fmul_rn` alone is a plain
// multiplication to this compiler and does get contracted)
__device__ __forceinline__ float scaled(float x, float scale) {
#pragma clang fp contract(off)
    float p = x * scale;
    asm volatile("" : "+v"(p));
    return p;
}

// ------------------------------------------------------------ ordering ----

// Maps a float to a uint32 whose unsigned order is the ranking top-k uses:
// NaN (either sign) above +inf, -0 == +0, otherwise the numeric order.
__device__ __forceinline__ uint32_t order_key(float v) {
    if (v != v) return 0xFFFFFFFFu;
    uint32_t u = __float_as_uint(v + 0.0f);  // -0 + +0 = +0
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Composite of key and position: larger composite = ranks earlier; among equal
// keys the lower index is the larger composite.  Never 0 for idx < 2^32-1.
__device__ __forceinline__ uint64_t composite(uint32_t key, uint32_t idx) {
    return (static_cast<uint64_t>(key) << 32) | static_cast<uint64_t>(0xFFFFFFFFu - idx);
}
__device__ __forceinline__ uint32_t composite_index(uint64_t c) {
    return 0xFFFFFFFFu - static_cast<uint32_t>(c);
}

// Number of lanes below the caller among those set in `mask`.
__device__ __forceinline__ uint32_t lanes_below(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

// hist[d] += 1 for every lane that calls (lanes may call under divergence).  The lanes that
// share the first such lane's digit add once between them: keys repeat (tied data, a dominant
// value, the leading bits of a sorted row), and same-address LDS atomics of one instruction
// are carried out one after the other.
__device__ __forceinline__ void hist_add_grouped(uint32_t *hist, uint32_t d) {
    const uint32_t lead = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(d)));
    const uint64_t same = __ballot(d == lead);
    if (d == lead) {
        if (lanes_below(same) == 0) atomicAdd(&hist[lead], static_cast<uint32_t>(__popcll(same)));
    } else {
        atomicAdd(&hist[d], 1u);
    }
}

// ------------------------------------------------------- block order ----
// Workgroups are handed to the chip's 8 XCDs in turn (workgroup b runs on XCD b mod 8),
// and each XCD has an L2 of its own: two workgroups with neighbouring blockIdx never
// share one.  For kernels whose neighbouring pieces of work touch the same cache lines
// (rows of a slab that do not start on a line boundary), this gives the position in
// the work's own order that workgroup blockIdx.x should take so that neighbouring
// pieces run on one XCD: XCD x takes the x-th eighth of the pieces.  A bijection on
// [0, gridDim.x).
constexpr uint32_t kXcds = 8;
__device__ __forceinline__ uint32_t xcd_grouped_block() {
    const uint32_t nb = gridDim.x, b = blockIdx.x;
    const uint32_t xcd = b % kXcds, local = b / kXcds;
    const uint32_t each = nb / kXcds, rem = nb % kXcds;  // the first `rem` XCDs get one piece more
    return xcd * each + min(xcd, rem) + local;
}

// ---------------------------------------------------------- reductions ----

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ __forceinline__ uint32_t wave_sum(uint32_t v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

// Block-wide max / sum through a small LDS array (one slot per wave).  Every
// thread of the block must call; the result is returned to all of them.
// `scratch` needs NT / 64 slots and is reusable after the call returns.
template <int NT> __device__ __forceinline__ float block_max(float v, float *scratch) {
    constexpr int NW = NT / kWave;
    v = wave_max(v);
    if constexpr (NW == 1) return v;
    __syncthreads();  // scratch may still be read from a previous call
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    float r = scratch[0];
#pragma unroll
    for (int w = 1; w < NW; w++) r = fmaxf(r, scratch[w]);
    return r;
}
template <int NT> __device__ __forceinline__ double block_sum(double v, double *scratch) {
    constexpr int NW = NT / kWave;
    v = wave_sum(v);
    if constexpr (NW == 1) return v;
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    double r = scratch[0];
#pragma unroll
    for (int w = 1; w < NW; w++) r += scratch[w];  // fixed order: run-to-run stable
    return r;
}

// --------------------------------------------------------------- softmax ----

// exp(d) rounded to float, evaluated in double (fp64 FMA runs at the same rate
// as scalar fp32 FMA on this chip): the relative error before the final
// rounding is below 2^-36, so the result is the correctly rounded float except
// within that distance of a rounding midpoint, where it is the other
// neighbour.  d <= -104 (including -inf) gives 0; NaN gives NaN.
__device__ __forceinline__ float exp_accurate(float d) {
    if (d <= -104.0f) return 0.0f;
    if (d > 89.0f) return __uint_as_float(0x7F800000u);
    const double x = static_cast<double>(d);
    const double n = rint(x * 1.4426950408889634074);
    const double r = fma(-n, 0.69314718055994530942, x);  // |r| <= 0.3466
    double p = 1.0 / 362880.0;
    p = fma(p, r, 1.0 / 40320.0);
    p = fma(p, r, 1.0 / 5040.0);
    p = fma(p, r, 1.0 / 720.0);
    p = fma(p, r, 1.0 / 120.0);
    p = fma(p, r, 1.0 / 24.0);
    p = fma(p, r, 1.0 / 6.0);
    p = fma(p, r, 0.5);
    p = fma(p, r, 1.0);
    p = fma(p, r, 1.0);
    return static_cast<float>(ldexp(p, static_cast<int>(n)));
}

// One softmax term: exp of the single-precision difference x - m.
__device__ __forceinline__ float softmax_term(float x, float m) { return exp_accurate(x - m); }

// exp(d) in single precision throughout, good to about two units in the last place of a float: the
// hardware exponential of a = fl(d log2 e), and what that rounding and the low part of log2 e left
// out as a first-order factor (2^(a + l) = 2^a (1 + l ln 2), |l| < 1e-6).  For results that are
// stored in half precision: 2^-22 relative before a rounding to 11 bits moves one result in two
// thousand by one unit of a half, and costs a third of exp_accurate.  Results below 2^-126 are 0.
__device__ __forceinline__ float exp_half_grade(float d) {
    constexpr float kHi = 1.44269502162933349609375f;  // float(log2 e)
    constexpr float kLo = 1.925963033500011e-8f;       // log2 e - kHi
    const float a = d * kHi;
    const float l = fmaf(d, kLo, fmaf(d, kHi, -a));  // (d = -inf: NaN, and so is the product below)
    const float e = __builtin_amdgcn_exp2f(a);
    const float t = fmaf(e, l * 0.693147180559945309f, e);
    return e > 0.f && e < INFINITY ? t : e;  // (0, inf and NaN as the hardware unit gives them)
}

// The term as the element type asks for it: float tensors get the correctly rounded exponential,
// half tensors (uint16_t) the single-precision one.  Every kernel that writes a softmax TENSOR
// takes its terms from here, so the results of one element type agree between them.
template <typename T> __device__ __forceinline__ float softmax_term_as(float x, float m) {
    if constexpr (sizeof(T) == 2) return exp_half_grade(x - m);
    else return exp_accurate(x - m);
}

// What a thread adds its own few terms up in, and how a term becomes a probability, in the same
// kernels: double for float tensors (the sum and the quotient as the definition rounds them), float
// for half tensors (a few dozen terms a thread: 2^-19 relative at worst, against 2^-11 of a half;
// the threads' sums are then added in double like everyone's).  Conversions to and from double are
// a quarter-rate instruction each, four of them an element: half tensors ran at the speed of float
// tensors of the same shape, for half the bytes.
template <typename T> using TermSum = std::conditional_t<sizeof(T) == 2, float, double>;
template <typename T> __device__ __forceinline__ float scale_term(float e, double rinv) {
    if constexpr (sizeof(T) == 2) return e * static_cast<float>(rinv);
    else return static_cast<float>(static_cast<double>(e) * rinv);
}

// The nucleus cut of a sorted result, by all 64 lanes of one wave: the number of leading values whose
// running sum -- added in order, in float, sum = fl(sum + v) -- first reaches p, or k if it never does
// (a NaN reaches nothing).  value(r) gives rank r < k.  The running sums move through the lanes: every lane
// keeps adding its own value to what its left neighbour holds (one instruction across the wave; lane 0
// holds fl(carry + v0) and adds 0 to itself), and after t steps lanes 0..t hold their final sums -- the
// additions of the walk one value at a time, in the same order, each a wave-wide instruction instead of
// a read of one lane, an addition, a comparison and a branch.
template <typename F> __device__ __forceinline__ uint32_t nucleus_count_wave(uint32_t k, float p, F &&value) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    float carry = 0.f;
    for (uint32_t base = 0; base < k; base += kWave) {
        const uint32_t m = min(static_cast<uint32_t>(kWave), k - base);
        const float v = base + lane < k ? value(base + lane) : 0.f;
        float s = lane == 0 ? __fadd_rn(carry, v) : v;
        const float own = lane == 0 ? 0.f : v;
        for (uint32_t t = 1; t < m; t += 4) {  // (steps past m - 1 change nothing below lane m)
#pragma unroll
            for (int u = 0; u < 4; u++) {
                // wave_shr:1 -- lane l reads lane l - 1, lane 0 (no source) keeps its own
                const float left = __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(s), __float_as_int(s), 0x138, 0xF, 0xF, false));
                s = __fadd_rn(own, left);
            }
        }
        const unsigned long long reached = __ballot(lane < m && s >= p);
        if (reached != 0ull) return base + static_cast<uint32_t>(__builtin_ctzll(reached)) + 1u;
        carry = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s), static_cast<int>(m - 1u)));
    }
    return k;
}

}  // namespace vkop
