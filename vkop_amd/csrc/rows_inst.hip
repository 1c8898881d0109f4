// One (element type, variant) slice of the one-pass row kernels (chunk, merge, one wave per row):
//   hipcc -DVKOP_ROWS_T=float|uint16_t -DVKOP_ROWS_SOFTMAX=true|false -c rows_inst.hip
// (the scan / pick / large-k kernels of the same slice: stream_inst.hip)
#include "rows_launch.hpp"

#ifndef VKOP_ROWS_T
#error "define VKOP_ROWS_T (float or uint16_t) and VKOP_ROWS_SOFTMAX (true or false)"
#endif

namespace vkop {

template <typename T, bool SOFTMAX> bool launch_rows_chunk(const RowsLaunch &a) {
    const T *in = static_cast<const T *>(a.in);
    T *values = static_cast<T *>(a.values);
    const uint32_t blocks = a.rows * a.g;
#define VKOP_ROWS_LAUNCH(NT, V, AL, MERGE)                       \
    rows_chunk_kernel<T, NT, V, SOFTMAX, AL, MERGE>              \
        <<<blocks, NT, 0, a.stream>>>(in, values, a.indices, a.n, a.k, a.g, a.per, a.ws)
#define VKOP_ROWS_CASE(NT, V)                                                                  \
    if (a.nt == NT && a.v == V) {                                                              \
        if (a.aligned && a.merge == kMergeLocal) VKOP_ROWS_LAUNCH(NT, V, true, kMergeLocal);   \
        else if (a.aligned && a.merge == kMergeByTicket) VKOP_ROWS_LAUNCH(NT, V, true, kMergeByTicket); \
        else if (a.aligned) VKOP_ROWS_LAUNCH(NT, V, true, kMergeSplit);                        \
        else if (a.merge == kMergeLocal) VKOP_ROWS_LAUNCH(NT, V, false, kMergeLocal);          \
        else if (a.merge == kMergeByTicket) VKOP_ROWS_LAUNCH(NT, V, false, kMergeByTicket);    \
        else VKOP_ROWS_LAUNCH(NT, V, false, kMergeSplit);                                      \
        return true;                                                                           \
    }
    if constexpr (SOFTMAX) {
        if (a.sampling) {
            // a row in one workgroup, every logit times a.scale, the nucleus count beside the result
            if (a.merge != kMergeLocal) return false;
#define VKOP_ROWS_SAMPLING(NT, V)                                                                                              \
    if (a.nt == NT && a.v == V) {                                                                                              \
        if (a.aligned)                                                                                                         \
            rows_chunk_kernel<T, NT, V, true, true, kMergeLocal, true>                                                         \
                <<<blocks, NT, 0, a.stream>>>(in, values, a.indices, a.n, a.k, a.g, a.per, a.ws, a.scale, a.counts, a.top_p);  \
        else                                                                                                                   \
            rows_chunk_kernel<T, NT, V, true, false, kMergeLocal, true>                                                        \
                <<<blocks, NT, 0, a.stream>>>(in, values, a.indices, a.n, a.k, a.g, a.per, a.ws, a.scale, a.counts, a.top_p);  \
        return true;                                                                                                           \
    }
            VKOP_ROWS_SAMPLING(64, 1)
            VKOP_ROWS_SAMPLING(64, 2)
            VKOP_ROWS_SAMPLING(64, 4)
            VKOP_ROWS_SAMPLING(256, 1)
            VKOP_ROWS_SAMPLING(256, 2)
            VKOP_ROWS_SAMPLING(256, 4)
            VKOP_ROWS_SAMPLING(512, 4)
            VKOP_ROWS_SAMPLING(1024, 4)
            if constexpr (sizeof(T) == 4) {
                VKOP_ROWS_SAMPLING(64, 8)
                VKOP_ROWS_SAMPLING(256, 8)
                VKOP_ROWS_SAMPLING(512, 8)
                VKOP_ROWS_SAMPLING(1024, 8)
            }
#undef VKOP_ROWS_SAMPLING
            return false;
        }
    }
    // one wave per row (short rows, small k): no barrier costs anything, nothing leaves the wave
#define VKOP_ROWS_CASE_WAVE(V)                                                 \
    if (a.nt == 64 && a.v == V && a.merge == kMergeLocal) {                    \
        if (a.aligned) VKOP_ROWS_LAUNCH(64, V, true, kMergeLocal);             \
        else VKOP_ROWS_LAUNCH(64, V, false, kMergeLocal);                      \
        return true;                                                           \
    }
    VKOP_ROWS_CASE_WAVE(1)
    VKOP_ROWS_CASE_WAVE(2)
    VKOP_ROWS_CASE_WAVE(4)
    if constexpr (sizeof(T) == 4) {
        VKOP_ROWS_CASE_WAVE(8)
    }
#undef VKOP_ROWS_CASE_WAVE
    VKOP_ROWS_CASE(256, 1)
    VKOP_ROWS_CASE(256, 2)
    VKOP_ROWS_CASE(256, 4)
    VKOP_ROWS_CASE(512, 4)
    VKOP_ROWS_CASE(1024, 4)
    if constexpr (sizeof(T) == 4) {
        VKOP_ROWS_CASE(256, 8)
        VKOP_ROWS_CASE(512, 8)
        VKOP_ROWS_CASE(1024, 8)
    }
#undef VKOP_ROWS_CASE
#undef VKOP_ROWS_LAUNCH
    return false;
}

template <typename T, bool SOFTMAX> void launch_rows_merge(const RowsLaunch &a) {
    const uint32_t slots = a.g << a.ws.cap_shift;
#define VKOP_MERGE_LAUNCH(RECS)                                               \
    rows_merge_kernel<T, SOFTMAX, RECS><<<a.rows, kMergeThreads, 0, a.stream>>>( \
        static_cast<const T *>(a.in), static_cast<T *>(a.values), a.indices, a.n, a.k, a.g, a.per, a.nt, a.ws)
    if (slots <= 1024) VKOP_MERGE_LAUNCH(1024);
    else if (slots <= 2048) VKOP_MERGE_LAUNCH(2048);
    else VKOP_MERGE_LAUNCH(kMergeRecsMax);
#undef VKOP_MERGE_LAUNCH
}

template <typename T, bool SOFTMAX> bool launch_rows_tiny(const TinyLaunch &a) {
    if constexpr (SOFTMAX) {
        if (a.sampling) {
#define VKOP_TINY_SAMPLING(V)                                                                          \
    if (a.v == V) {                                                                                    \
        if (a.aligned)                                                                                 \
            rows_tiny_sampling_kernel<T, V, true><<<a.rows, kWave, 0, a.stream>>>(                     \
                static_cast<const T *>(a.in), static_cast<T *>(a.values), a.indices, a.n, a.k,         \
                a.scale, a.counts, a.top_p);                                                           \
        else                                                                                           \
            rows_tiny_sampling_kernel<T, V, false><<<a.rows, kWave, 0, a.stream>>>(                    \
                static_cast<const T *>(a.in), static_cast<T *>(a.values), a.indices, a.n, a.k,         \
                a.scale, a.counts, a.top_p);                                                           \
        return true;                                                                                   \
    }
            VKOP_TINY_SAMPLING(1)
            VKOP_TINY_SAMPLING(2)
            VKOP_TINY_SAMPLING(4)
            if constexpr (sizeof(T) == 4) {
                VKOP_TINY_SAMPLING(8)
            }
#undef VKOP_TINY_SAMPLING
            return false;
        }
    }
#define VKOP_TINY_CASE(V)                                                                              \
    if (a.v == V) {                                                                                    \
        if (a.aligned)                                                                                 \
            rows_tiny_kernel<T, V, SOFTMAX, true><<<a.rows, kWave, 0, a.stream>>>(                     \
                static_cast<const T *>(a.in), static_cast<T *>(a.values), a.indices, a.n, a.k,         \
                a.smallest ? 1u : 0u);                                                                 \
        else                                                                                           \
            rows_tiny_kernel<T, V, SOFTMAX, false><<<a.rows, kWave, 0, a.stream>>>(                    \
                static_cast<const T *>(a.in), static_cast<T *>(a.values), a.indices, a.n, a.k,         \
                a.smallest ? 1u : 0u);                                                                 \
        return true;                                                                                   \
    }
    VKOP_TINY_CASE(1)
    VKOP_TINY_CASE(2)
    VKOP_TINY_CASE(4)
    if constexpr (sizeof(T) == 4) {
        VKOP_TINY_CASE(8)
    }
#undef VKOP_TINY_CASE
    return false;
}

template bool launch_rows_tiny<VKOP_ROWS_T, VKOP_ROWS_SOFTMAX>(const TinyLaunch &);
template bool launch_rows_chunk<VKOP_ROWS_T, VKOP_ROWS_SOFTMAX>(const RowsLaunch &);
template void launch_rows_merge<VKOP_ROWS_T, VKOP_ROWS_SOFTMAX>(const RowsLaunch &);

}  // namespace vkop

#ifdef VKOP_STAMPS
extern "C" int VKOP_STAMPS(unsigned long long *out) {
    const int rc = static_cast<int>(hipMemcpyFromSymbol(out, HIP_SYMBOL(vkop::g_bp_stamps), 64 * sizeof(unsigned long long)));
    static const unsigned long long zeros[64] = {};
    (void)hipMemcpyToSymbol(HIP_SYMBOL(vkop::g_bp_stamps), zeros, sizeof(zeros));  // (each readout starts the next interval)
    return rc;
}
#define VKOP_STAMPS_CAT2(a, b) a##b
#define VKOP_STAMPS_CAT(a, b) VKOP_STAMPS_CAT2(a, b)
extern "C" int VKOP_STAMPS_CAT(VKOP_STAMPS, _block)(unsigned int block) {
    return static_cast<int>(hipMemcpyToSymbol(HIP_SYMBOL(vkop::g_bp_block), &block, sizeof(block)));
}
#endif
