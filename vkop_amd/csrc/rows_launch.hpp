// Host-side launch of the streaming row kernels (kernels_rows.hpp).  Their many
// instantiations (threads x loads x aligned x merge mode) are compiled one
// translation unit per (element type, softmax or plain top-k), rows_inst.hip
// built four times, so that the library builds in parallel; the C ABI source
// only sees these declarations.
#pragma once

#include <hip/hip_runtime.h>

#include "kernels_rows.hpp"
#include "kernels_bigpick.hpp"
#include "kernels_stream.hpp"
#include "kernels_tiny.hpp"

namespace vkop {

struct RowsLaunch {
    const void *in;
    void *values;
    int32_t *indices;
    uint32_t rows, n, k;
    uint32_t nt, v;    // threads per workgroup, 128-bit loads per thread
    uint32_t g, per;   // chunks per row, elements per chunk
    bool aligned;      // rows start on 16 bytes and n is a multiple of the vector width
    int merge;         // kMergeSplit / kMergeByTicket / kMergeLocal
    RowsWorkspace ws;
    hipStream_t stream;
    // sampling form (softmax variant, merge == kMergeLocal only): every logit times scale; counts: per-row nucleus cut for top_p, or null
    bool sampling = false;
    float scale = 1.f;
    int32_t *counts = nullptr;
    float top_p = 0.f;
};

// Launch of the streaming pair rows_scan_kernel + rows_pick_kernel (kernels_stream.hpp).
struct ScanLaunch {
    const void *in;
    void *values;
    int32_t *indices;
    uint32_t rows, n, k;
    uint32_t v;        // 128-bit loads per thread of the scan kernel (a chunk is 256 * v vectors)
    uint32_t g;        // chunks per row
    bool aligned;      // rows start on 16 bytes and n is a multiple of the vector width
    int stages;        // 1 = scan only, 2 = pick only, 3 = both (1 and 2: measurements)
    float scale;       // softmax variant: every logit times this (1 = the unscaled kernels)
    int32_t *counts;   // softmax variant: per-row nucleus cut for top_p, or null
    float top_p;
    ScanWorkspace ws;
    uint32_t g2;          // 0, or (k beyond the pick kernel's list) workgroups a row of bigpick_gather_kernel
    BigPickWorkspace bw;  // ... and its candidate lists
    hipStream_t stream;
};
// Enqueues rows_scan_kernel and rows_pick_kernel (or, with g2 set, the bigpick pair
// behind the scan); false if no kernel is built for the shape.
template <typename T, bool SOFTMAX> bool launch_rows_scan(const ScanLaunch &a);
extern template bool launch_rows_scan<float, true>(const ScanLaunch &);
extern template bool launch_rows_scan<float, false>(const ScanLaunch &);
extern template bool launch_rows_scan<uint16_t, true>(const ScanLaunch &);
extern template bool launch_rows_scan<uint16_t, false>(const ScanLaunch &);

// Enqueues rows_tiny_kernel (one wave per row, v 128-bit loads per lane); false if no kernel is built for v.
struct TinyLaunch {
    const void *in;
    void *values;
    int32_t *indices;
    uint32_t rows, n, k, v;
    bool aligned;
    bool smallest = false;  // plain top-k: the k smallest, increasing
    hipStream_t stream;
    // sampling form (softmax variant): every logit times scale; counts: per-row nucleus cut for top_p, or null
    bool sampling = false;
    float scale = 1.f;
    int32_t *counts = nullptr;
    float top_p = 0.f;
};
template <typename T, bool SOFTMAX> bool launch_rows_tiny(const TinyLaunch &a);
extern template bool launch_rows_tiny<float, true>(const TinyLaunch &);
extern template bool launch_rows_tiny<float, false>(const TinyLaunch &);
extern template bool launch_rows_tiny<uint16_t, true>(const TinyLaunch &);
extern template bool launch_rows_tiny<uint16_t, false>(const TinyLaunch &);

// Enqueues rows_chunk_kernel; false if no kernel is built for (nt, v).
template <typename T, bool SOFTMAX> bool launch_rows_chunk(const RowsLaunch &a);
// Enqueues rows_merge_kernel (after a chunk kernel launched with kMergeSplit).
template <typename T, bool SOFTMAX> void launch_rows_merge(const RowsLaunch &a);

extern template bool launch_rows_chunk<float, true>(const RowsLaunch &);
extern template bool launch_rows_chunk<float, false>(const RowsLaunch &);
extern template bool launch_rows_chunk<uint16_t, true>(const RowsLaunch &);
extern template bool launch_rows_chunk<uint16_t, false>(const RowsLaunch &);
extern template void launch_rows_merge<float, true>(const RowsLaunch &);
extern template void launch_rows_merge<float, false>(const RowsLaunch &);
extern template void launch_rows_merge<uint16_t, true>(const RowsLaunch &);
extern template void launch_rows_merge<uint16_t, false>(const RowsLaunch &);

}  // namespace vkop
