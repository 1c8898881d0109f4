// One (element type, variant) slice of the scan kernels and what runs behind them (pick; gather + rank):
//   hipcc -DVKOP_ROWS_T=float|uint16_t -DVKOP_ROWS_SOFTMAX=true|false -c stream_inst.hip
#include "rows_launch.hpp"

#ifndef VKOP_ROWS_T
#error "define VKOP_ROWS_T (float or uint16_t) and VKOP_ROWS_SOFTMAX (true or false)"
#endif

namespace vkop {

template <typename T, bool SOFTMAX> bool launch_rows_scan(const ScanLaunch &a) {
    const T *in = static_cast<const T *>(a.in);
    constexpr uint32_t VEC = 16 / sizeof(T);
    const uint32_t per = kScanThreads * a.v * VEC;
    const uint32_t ge = (a.ws.blocks + kPickThreads - 1) / kPickThreads;
    const uint32_t ge_big = (a.ws.blocks + kBigPickThreads - 1) / kBigPickThreads;
    if (a.g2 == 0 ? ge > 32 : ge_big > 32) return false;
    bool scanned = (a.stages & 1) == 0;
    const bool scaled = SOFTMAX && a.scale != 1.f;
#define VKOP_SCAN_LAUNCH(V, AL, SC) \
    rows_scan_kernel<T, V, SOFTMAX, AL, SC><<<a.rows * a.g, kScanThreads, 0, a.stream>>>(in, a.n, a.g, a.ws, a.scale)
#define VKOP_SCAN_MIN_LAUNCH(V, AL) \
    rows_scan_kernel<T, V, SOFTMAX, AL, false, true><<<a.rows * a.g, kScanThreads, 0, a.stream>>>(in, a.n, a.g, a.ws, 1.f)
#define VKOP_SCAN_CASE(V)                                             \
    if (!scanned && a.v == V && a.g2 != 0) {                          \
        if (a.aligned) VKOP_SCAN_MIN_LAUNCH(V, true);                 \
        else VKOP_SCAN_MIN_LAUNCH(V, false);                          \
        scanned = true;                                               \
    }                                                                 \
    if (!scanned && a.v == V) {                                       \
        if constexpr (SOFTMAX) {                                      \
            if (scaled && a.aligned) VKOP_SCAN_LAUNCH(V, true, true); \
            else if (scaled) VKOP_SCAN_LAUNCH(V, false, true);        \
        }                                                             \
        if (!scaled && a.aligned) VKOP_SCAN_LAUNCH(V, true, false);   \
        else if (!scaled) VKOP_SCAN_LAUNCH(V, false, false);          \
        scanned = true;                                               \
    }
    VKOP_SCAN_CASE(2)
    VKOP_SCAN_CASE(4)
    VKOP_SCAN_CASE(8)
    if constexpr (sizeof(T) == 4) {
        VKOP_SCAN_CASE(16)
    }
#undef VKOP_SCAN_CASE
#undef VKOP_SCAN_MIN_LAUNCH
#undef VKOP_SCAN_LAUNCH
    if (!scanned) return false;
    if ((a.stages & 2) == 0) return true;
    if (a.g2 != 0) {
#define VKOP_BIG_LAUNCH(GE, AL)                                                                  \
    bigpick_gather_kernel<T, SOFTMAX, AL, GE><<<a.rows * a.g2, kBigPickThreads, 0, a.stream>>>( \
        in, a.n, a.k, a.g2, a.g, per, a.ws, a.bw)
#define VKOP_BIG_CASE(GE)                         \
    if (!gathered && ge_big <= GE) {              \
        if (a.aligned) VKOP_BIG_LAUNCH(GE, true); \
        else VKOP_BIG_LAUNCH(GE, false);          \
        gathered = true;                          \
    }
        bool gathered = false;
        VKOP_BIG_CASE(4)
        VKOP_BIG_CASE(8)
        VKOP_BIG_CASE(16)
        VKOP_BIG_CASE(32)
#undef VKOP_BIG_CASE
#undef VKOP_BIG_LAUNCH
        bigpick_rank_kernel<T, SOFTMAX><<<a.rows * (kBigPickCap / kBigPickMine), kBigPickThreads, 0, a.stream>>>(
            in, static_cast<T *>(a.values), a.indices, a.n, a.k, a.bw);
        return true;
    }
#define VKOP_PICK_LAUNCH(GE, AL, SC)                                                  \
    rows_pick_kernel<T, SOFTMAX, AL, GE, SC><<<a.rows, kPickThreads, 0, a.stream>>>(  \
        in, static_cast<T *>(a.values), a.indices, a.n, a.k, a.g, per, a.ws, SOFTMAX ? a.scale : 1.f, a.counts, a.top_p)
#define VKOP_PICK_CASE(GE)                                            \
    if (ge <= GE) {                                                   \
        if constexpr (SOFTMAX) {                                      \
            if (scaled && a.aligned) VKOP_PICK_LAUNCH(GE, true, true); \
            else if (scaled) VKOP_PICK_LAUNCH(GE, false, true);       \
        }                                                             \
        if (!scaled && a.aligned) VKOP_PICK_LAUNCH(GE, true, false);  \
        else if (!scaled) VKOP_PICK_LAUNCH(GE, false, false);         \
        return true;                                                  \
    }
    VKOP_PICK_CASE(2)
    VKOP_PICK_CASE(4)
    VKOP_PICK_CASE(8)
    VKOP_PICK_CASE(16)
    VKOP_PICK_CASE(32)
#undef VKOP_PICK_CASE
#undef VKOP_PICK_LAUNCH
    return false;
}

template bool launch_rows_scan<VKOP_ROWS_T, VKOP_ROWS_SOFTMAX>(const ScanLaunch &);

}  // namespace vkop

#ifdef VKOP_STAMPS
// (debug builds: the clock stamps of this translation unit's kernels; <name>_stream reads them out)
#define VKOP_STAMPS_CAT2(a, b) a##b
#define VKOP_STAMPS_CAT(a, b) VKOP_STAMPS_CAT2(a, b)
extern "C" int VKOP_STAMPS_CAT(VKOP_STAMPS, _stream)(unsigned long long *out) {
    const int rc = static_cast<int>(hipMemcpyFromSymbol(out, HIP_SYMBOL(vkop::g_bp_stamps), 64 * sizeof(unsigned long long)));
    static const unsigned long long zeros[64] = {};
    (void)hipMemcpyToSymbol(HIP_SYMBOL(vkop::g_bp_stamps), zeros, sizeof(zeros));  // (each readout starts the next interval)
    return rc;
}
// (the timeline log: the number of records, then up to `cap` of them; the log starts again)
extern "C" int VKOP_STAMPS_CAT(VKOP_STAMPS, _timeline)(unsigned long long *out, unsigned cap) {
    unsigned n = 0;
    int rc = static_cast<int>(hipMemcpyFromSymbol(&n, HIP_SYMBOL(vkop::g_timeline_n), sizeof(n)));
    const unsigned take = n < cap ? n : cap;
    if (rc == 0 && take > 0)
        rc = static_cast<int>(hipMemcpyFromSymbol(out, HIP_SYMBOL(vkop::g_timeline), static_cast<size_t>(take) * sizeof(vkop::TimelineRec)));
    const unsigned zero = 0;
    (void)hipMemcpyToSymbol(HIP_SYMBOL(vkop::g_timeline_n), &zero, sizeof(zero));
    return rc == 0 ? static_cast<int>(take) : -1;
}
#endif
