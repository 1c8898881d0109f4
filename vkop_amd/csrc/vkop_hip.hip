// C ABI of the softmax / top-k library (declared in include/vkop_hip.h):
// argument checking, kernel selection and launches (the only kernel here clears a workspace).
#include "../../include/vkop_hip.h"
#include "vkop_hip_internal.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "kernels_general.hpp"
#include "kernels_rows.hpp"
#include "rows_launch.hpp"
#include "kernels_softmax.hpp"
#include "kernels_bigk.hpp"
#include "kernels_nms.hpp"

namespace vkop {

// workspace clear (a kernel, not a memset: safe inside a captured graph)
__global__ void fill_zero_kernel(uint32_t *p, size_t words) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < words) p[i] = 0u;
}

}  // namespace vkop

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

#define VKOP_HIP_TRY(expr)                                                                        \
    do {                                                                                          \
        hipError_t e_ = (expr);                                                                   \
        if (e_ != hipSuccess) return fail(VKOP_HIP_ERR_DEVICE, "%s: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

inline hipStream_t as_stream(void *s) { return static_cast<hipStream_t>(s); }

// (outer, n, inner) view of a dense tensor around `axis`.
struct View {
    vkop::LineGeom g;
    uint64_t elems;
};

int make_view(const int *shape, int ndim, int axis, View *v) {
    if (shape == nullptr) return fail(VKOP_HIP_ERR_INVALID, "shape is null");
    if (ndim < 1 || ndim > 4) return fail(VKOP_HIP_ERR_INVALID, "rank %d outside 1..4", ndim);
    if (axis < 0) axis += ndim;
    if (axis < 0 || axis >= ndim) return fail(VKOP_HIP_ERR_INVALID, "axis outside the tensor's rank %d", ndim);
    uint64_t outer = 1, inner = 1;
    for (int d = 0; d < ndim; d++) {
        if (shape[d] < 0) return fail(VKOP_HIP_ERR_INVALID, "negative extent %d at dim %d", shape[d], d);
        if (d < axis) outer *= static_cast<uint64_t>(shape[d]);
        if (d > axis) inner *= static_cast<uint64_t>(shape[d]);
    }
    const uint64_t n = static_cast<uint64_t>(shape[axis]);
    const uint64_t elems = outer * n * inner;
    if (outer * inner >= (1ull << 31) || elems >= (1ull << 40))
        return fail(VKOP_HIP_ERR_UNSUPPORTED, "tensor too large (%llu elements)", static_cast<unsigned long long>(elems));
    v->g.outer = static_cast<uint32_t>(outer);
    v->g.n = static_cast<uint32_t>(n);
    v->g.inner = static_cast<uint32_t>(inner);
    v->elems = elems;
    return VKOP_HIP_OK;
}

int check_dtype(int dtype) {
    if (dtype != VKOP_HIP_F32 && dtype != VKOP_HIP_F16) return fail(VKOP_HIP_ERR_INVALID, "unknown dtype %d", dtype);
    return VKOP_HIP_OK;
}

int check_k(const View &v, int k) {
    if (k < 1) return fail(VKOP_HIP_ERR_INVALID, "k = %d must be at least 1", k);
    if (static_cast<uint64_t>(k) > v.g.n)
        return fail(VKOP_HIP_ERR_INVALID, "k = %d exceeds the axis extent %u", k, v.g.n);
    if (k > VKOP_HIP_MAX_K) return fail(VKOP_HIP_ERR_UNSUPPORTED, "k = %d exceeds VKOP_HIP_MAX_K = %d", k, VKOP_HIP_MAX_K);
    return VKOP_HIP_OK;
}

int launched(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(VKOP_HIP_ERR_DEVICE, "launch of %s failed: %s", what, hipGetErrorString(e));
    return VKOP_HIP_OK;
}

// ---- scratch of the entry point that allocates nothing ------------------------
// One array per GPU, created when the library's code is loaded on that GPU and
// held until the process ends.  In host code the array's name is only a handle:
// its device address is looked up once per device (resolve_static_scratch) and
// that address is what kernels, fills and copies are given.
static __device__ __align__(256) unsigned char scratch[VKOP_HIP_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];
// set when a call on the static scratch may have left a row's arrival counter
// non-zero (a launch failed half way): the next call clears the counters first
std::atomic<int> g_scratch_dirty[kMaxDevices];

// Device address of `scratch` on the current device (looked up on the first call
// per device, with that device current), and the device's ordinal.
int resolve_static_scratch(void **ptr, int *device) {
    int dev = 0;
    VKOP_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(VKOP_HIP_ERR_UNSUPPORTED, "device ordinal %d beyond %d", dev, kMaxDevices);
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        VKOP_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (p == nullptr) return fail(VKOP_HIP_ERR_DEVICE, "hipGetSymbolAddress gave no address for the static scratch");
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *ptr = p;
    *device = dev;
    return VKOP_HIP_OK;
}

// vkop_hip_tune state
std::atomic<int> g_rows_threads{0}, g_rows_loads{0}, g_rows_chunks{0}, g_rows_fused{0}, g_rows_path{0},
    g_nms_threads{0};
// Which kernels of a two-kernel streaming call are launched: both, except in the benchmark build of the
// library (-DVKOP_BENCH_HOOKS, libvkop_hip_bench.so), where vkop_hip_measure_stages can leave one out.
#ifdef VKOP_BENCH_HOOKS
std::atomic<int> g_rows_stages{3};
inline int measured_stages() { return g_rows_stages.load(); }
#else
inline int measured_stages() { return 3; }
#endif

// The per-row arrival counters of the one-kernel top-k variant sit at a fixed
// place, the first kTicketRows words of every workspace, whatever the operator
// and tensor: each call leaves them at zero, so a workspace cleared once can
// serve calls of different kinds and shapes in turn.  Nothing else is ever
// stored there.
constexpr size_t kTicketRows = 16384;
constexpr size_t kTicketBytes = kTicketRows * sizeof(uint32_t);  // a multiple of the workspace alignment

constexpr int kLineThreads = 256;
constexpr size_t kAlign = 256;
inline size_t align_up(size_t b) { return (b + kAlign - 1) / kAlign * kAlign; }

// ---------------------------------------------------------------- softmax ----
// Launch shapes shared by the row kernels: threads per workgroup and 128-bit
// loads per thread, smallest first.
struct RowShape {
    int nt, v;
};
const RowShape kShapesF32[] = {{256, 1}, {256, 2}, {256, 4}, {256, 8}, {512, 8}, {1024, 8}};
const RowShape kShapesF16[] = {{128, 1}, {256, 1}, {256, 2}, {256, 4}, {512, 4}, {1024, 4}};

struct SoftmaxPlan {
    enum Kind { kGeneralLines, kGeneralStrided, kRow, kWaveRow, kChunked, kStridedRegs, kStridedTile } kind = kGeneralLines;
    RowShape shape{0, 0};
    uint32_t g = 1, per = 0;
    uint32_t ti_shift = 0;  // kStridedTile: log2 of the lines a tile
    size_t workspace = 0;
};

// Lines of up to kStridedMaxN elements along a non-last axis, held in registers: the
// kernel is compiled for a few bounds of n and the smallest that fits is launched;
// longer lines are shared by two or four lanes.
template <typename T, bool MAX_ONLY>
void launch_strided_reg(const T *in, T *out, const View &v, int nan_where, float nan_value, hipStream_t st) {
    const uint32_t lines = v.g.outer * v.g.inner;
#define VKOP_STRIDED_CASE(NMAX, P)                                                          \
    if (v.g.n <= NMAX) {                                                                    \
        const uint32_t per_block = vkop::kStridedThreads / P;                               \
        vkop::softmax_strided_reg_kernel<T, NMAX, P, MAX_ONLY>                              \
            <<<(lines + per_block - 1) / per_block, vkop::kStridedThreads, 0, st>>>(in, out, v.g, nan_where, nan_value); \
        return;                                                                             \
    }
    VKOP_STRIDED_CASE(16, 1)
    VKOP_STRIDED_CASE(32, 2)
    VKOP_STRIDED_CASE(48, 4)
    VKOP_STRIDED_CASE(64, 4)
    VKOP_STRIDED_CASE(80, 4)
    VKOP_STRIDED_CASE(96, 4)
    VKOP_STRIDED_CASE(128, 4)
#undef VKOP_STRIDED_CASE
}

SoftmaxPlan plan_softmax(const View &v, int dtype) {
    SoftmaxPlan p;
    const uint32_t vec = dtype == VKOP_HIP_F32 ? 4u : 8u;
    const RowShape *shapes = dtype == VKOP_HIP_F32 ? kShapesF32 : kShapesF16;
    const uint32_t n = v.g.n, rows = v.g.outer;
    if (v.g.inner != 1) {
        if (n <= static_cast<uint32_t>(vkop::kStridedMaxN)) p.kind = SoftmaxPlan::kStridedRegs;
        else {
            // a tile of TI lines (the power of two at or above min(inner, 64)) per workgroup; with too
            // few tiles to fill the chip, every tile's rows are split over G workgroups (two launches)
            p.kind = SoftmaxPlan::kStridedTile;
            while (p.ti_shift < 6 && (1u << p.ti_shift) < v.g.inner) p.ti_shift++;
            const uint32_t ti = 1u << p.ti_shift;
            const uint64_t tiles = static_cast<uint64_t>(rows) * ((v.g.inner + ti - 1) >> p.ti_shift);
            const uint32_t turn = (vkop::kStridedTileThreads / vkop::kWave) * (vkop::kWave >> p.ti_shift);  // rows per turn
            p.g = 1;
            p.per = n;
            if (tiles < 256 && n >= 8 * turn) {
                uint32_t want = static_cast<uint32_t>((512 + tiles - 1) / tiles);
                want = std::min(want, static_cast<uint32_t>(vkop::kStridedTileThreads) >> p.ti_shift);
                uint32_t per = (n + want - 1) / want;
                per = std::max((per + turn - 1) / turn * turn, 4 * turn);
                p.g = (n + per - 1) / per;
                p.per = per;
                if (p.g > 1)
                    p.workspace = kTicketBytes + align_up(static_cast<size_t>(tiles) * p.g * ti * sizeof(vkop::ChunkStat));
                else p.per = n;
            }
        }
        return p;
    }
    if (n <= 8u * vkop::kWave) {  // short rows: a wave each
        p.kind = SoftmaxPlan::kWaveRow;
        return p;
    }
    const uint32_t biggest = static_cast<uint32_t>(shapes[5].nt) * shapes[5].v * vec;
    // a whole row per workgroup when rows are short or there are enough of them
    if (n <= 8192 || (n <= biggest && rows >= 512)) {
        for (int i = 0; i < 6; i++) {
            if (static_cast<uint32_t>(shapes[i].nt) * shapes[i].v * vec >= n) {
                p.kind = SoftmaxPlan::kRow;
                p.shape = shapes[i];
                return p;
            }
        }
    }
    // chunked: the largest chunk that still leaves >= 1024 workgroups, else the smallest
    int pick = -1;
    for (int i = 0; i < 6; i++) {
        const uint32_t span = static_cast<uint32_t>(shapes[i].nt) * shapes[i].v * vec;
        const uint32_t g = (n + span - 1) / span;
        if (g > static_cast<uint32_t>(shapes[i].nt) || static_cast<uint64_t>(rows) * g >= (1ull << 31)) continue;
        if (pick < 0) pick = i;
        if (static_cast<uint64_t>(rows) * g >= 1024) pick = i;
    }
    if (pick < 0) return p;  // (rows of more than 2^25 elements: the general kernel)
    p.kind = SoftmaxPlan::kChunked;
    p.shape = shapes[pick];
    p.per = static_cast<uint32_t>(p.shape.nt) * p.shape.v * vec;
    p.g = (n + p.per - 1) / p.per;
    p.workspace = kTicketBytes + align_up(static_cast<size_t>(rows) * p.g * sizeof(vkop::ChunkStat));
    return p;
}

#define VKOP_FOR_EACH_ROW_SHAPE(X, T) \
    X(256, 1) X(256, 2) X(256, 4) X(512, 4) X(1024, 4)                          \
    if constexpr (sizeof(T) == 4) { X(256, 8) X(512, 8) X(1024, 8) }          \
    if constexpr (sizeof(T) == 2) { X(128, 1) }

template <typename T>
int softmax_impl(const T *in, T *out, const View &v, int dtype, int nan_where, float nan_value, void *ws,
                 size_t ws_bytes, hipStream_t st) {
    const SoftmaxPlan p = plan_softmax(v, dtype);
    const uint32_t lines = v.g.outer * v.g.inner;
    const uint32_t vec = 16 / sizeof(T);
    const bool aligned = reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                         v.g.n % vec == 0;
    switch (p.kind) {
    case SoftmaxPlan::kRow: {
        bool done = false;
        const uint32_t row_grid = std::min(lines, vkop::kSoftmaxRowGridMax);
        // thousands of rows that a wave holds in a few 128-bit loads a lane: a wave per row, no barrier
        const uint32_t vectors = (v.g.n + vec - 1) / vec;
        if (aligned && lines >= 4096 && vectors <= 4 * vkop::kWave) {
            const uint32_t wgs = std::min((lines + vkop::kSoftmaxVecRows - 1) / vkop::kSoftmaxVecRows, 8192u);
#define VKOP_VEC_ROW(V)                                                                                                          \
    vkop::softmax_wave_vec_kernel<T, V><<<wgs, vkop::kSoftmaxVecRows * vkop::kWave, 0, st>>>(in, out, lines, v.g.n, nan_where, nan_value)
            if (vectors <= vkop::kWave) VKOP_VEC_ROW(1);
            else if (vectors <= 2 * vkop::kWave) VKOP_VEC_ROW(2);
            else VKOP_VEC_ROW(4);
#undef VKOP_VEC_ROW
            return launched("softmax_wave_vec_kernel");
        }
#define VKOP_ROW(NT, V)                                                                                        \
    if (!done && p.shape.nt == NT && p.shape.v == V) {                                                         \
        if (aligned) vkop::softmax_row_kernel<T, NT, V, true><<<row_grid, NT, 0, st>>>(in, out, lines, v.g.n, nan_where, nan_value); \
        else vkop::softmax_row_kernel<T, NT, V, false><<<row_grid, NT, 0, st>>>(in, out, lines, v.g.n, nan_where, nan_value);        \
        done = true;                                                                                           \
    }
        VKOP_FOR_EACH_ROW_SHAPE(VKOP_ROW, T)
#undef VKOP_ROW
        if (!done) return fail(VKOP_HIP_ERR_UNSUPPORTED, "no softmax_row_kernel for %d x %d", p.shape.nt, p.shape.v);
        return launched("softmax_row_kernel");
    }
    case SoftmaxPlan::kWaveRow: {
        const uint32_t blocks = (lines + vkop::kSoftmaxWaveRows - 1) / vkop::kSoftmaxWaveRows;
        const uint32_t per_lane = (v.g.n + vkop::kWave - 1) / vkop::kWave;
#define VKOP_WAVE_ROW(E)                                                                                    \
    vkop::softmax_wave_kernel<T, E><<<blocks, vkop::kSoftmaxWaveRows * vkop::kWave, 0, st>>>(in, out, lines, v.g.n, \
                                                                                              nan_where, nan_value)
        if (per_lane <= 1) VKOP_WAVE_ROW(1);
        else if (per_lane <= 2) VKOP_WAVE_ROW(2);
        else if (per_lane <= 4) VKOP_WAVE_ROW(4);
        else VKOP_WAVE_ROW(8);
#undef VKOP_WAVE_ROW
        return launched("softmax_wave_kernel");
    }
    case SoftmaxPlan::kChunked: {
        if (ws == nullptr || ws_bytes < p.workspace)
            return fail(VKOP_HIP_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", ws_bytes, p.workspace);
        auto *stats = reinterpret_cast<vkop::ChunkStat *>(static_cast<unsigned char *>(ws) + kTicketBytes);
        const uint32_t blocks = v.g.outer * p.g;
        bool done = false;
#define VKOP_CHUNKED(NT, V)                                                                                    \
    if (!done && p.shape.nt == NT && p.shape.v == V) {                                                         \
        if (aligned) {                                                                                         \
            vkop::softmax_stats_kernel<T, NT, V, true><<<blocks, NT, 0, st>>>(in, stats, v.g.n, p.g, p.per);   \
            vkop::softmax_scale_kernel<T, NT, V, true>                                                         \
                <<<blocks, NT, 0, st>>>(in, out, stats, v.g.n, p.g, p.per, nan_where, nan_value);              \
        } else {                                                                                               \
            vkop::softmax_stats_kernel<T, NT, V, false><<<blocks, NT, 0, st>>>(in, stats, v.g.n, p.g, p.per);  \
            vkop::softmax_scale_kernel<T, NT, V, false>                                                        \
                <<<blocks, NT, 0, st>>>(in, out, stats, v.g.n, p.g, p.per, nan_where, nan_value);              \
        }                                                                                                      \
        done = true;                                                                                           \
    }
        VKOP_FOR_EACH_ROW_SHAPE(VKOP_CHUNKED, T)
#undef VKOP_CHUNKED
        if (!done) return fail(VKOP_HIP_ERR_UNSUPPORTED, "no chunked softmax for %d x %d", p.shape.nt, p.shape.v);
        return launched("softmax_stats_kernel / softmax_scale_kernel");
    }
    case SoftmaxPlan::kStridedRegs: {
        launch_strided_reg<T, false>(in, out, v, nan_where, nan_value, st);
        return launched("softmax_strided_reg_kernel");
    }
    case SoftmaxPlan::kStridedTile: {
        const uint32_t tiles = v.g.outer * ((v.g.inner + (1u << p.ti_shift) - 1) >> p.ti_shift);
        if (p.g == 1) {
            vkop::softmax_strided_tile_kernel<T, vkop::kTileWhole>
                <<<tiles, vkop::kStridedTileThreads, 0, st>>>(in, out, nullptr, v.g, p.ti_shift, 1, v.g.n, nan_where, nan_value);
            return launched("softmax_strided_tile_kernel");
        }
        if (ws == nullptr || ws_bytes < p.workspace)
            return fail(VKOP_HIP_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", ws_bytes, p.workspace);
        auto *stats = reinterpret_cast<vkop::ChunkStat *>(static_cast<unsigned char *>(ws) + kTicketBytes);
        vkop::softmax_strided_tile_kernel<T, vkop::kTileStats>
            <<<tiles * p.g, vkop::kStridedTileThreads, 0, st>>>(in, out, stats, v.g, p.ti_shift, p.g, p.per, nan_where, nan_value);
        vkop::softmax_strided_tile_kernel<T, vkop::kTileScale>
            <<<tiles * p.g, vkop::kStridedTileThreads, 0, st>>>(in, out, stats, v.g, p.ti_shift, p.g, p.per, nan_where, nan_value);
        return launched("softmax_strided_tile_kernel (split)");
    }
    case SoftmaxPlan::kGeneralLines:
        vkop::softmax_lines_kernel<T, kLineThreads>
            <<<lines, kLineThreads, 0, st>>>(in, out, v.g, nan_where, nan_value, nullptr);
        return launched("softmax_lines_kernel");
    case SoftmaxPlan::kGeneralStrided:
    default: {
        const uint32_t blocks = (lines + kLineThreads - 1) / kLineThreads;
        vkop::softmax_strided_kernel<T, kLineThreads><<<blocks, kLineThreads, 0, st>>>(in, out, v.g, nan_where, nan_value);
        return launched("softmax_strided_kernel");
    }
    }
}

// ------------------------------------------------- streaming rows kernel ----
// Launch shape of rows_chunk_kernel: NT threads, V 128-bit loads per thread,
// G chunks per row of `per` elements each, `cap` candidate slots per chunk.
struct RowsCfg {
    bool ok = false;
    int nt = 0, v = 0;
    uint32_t g = 0, per = 0;
    uint32_t cap = 0, cap_shift = 0;
};

// Candidate slots per chunk: 2.5 times the k+1 wanted elements (a chunk of
// identically distributed data has about 1.2 times k+1 at or above its
// threshold), at least 64, power of two.
uint32_t rows_cap(int k) {
    const uint32_t want = static_cast<uint32_t>(k) + 1u;
    uint32_t cap = 64;
    while (2u * cap < 5u * want) cap <<= 1;
    return cap;
}

constexpr int kWaveRowMaxK = 32;  // largest k served by the one-wave-per-row launch
constexpr int kWideRowMinK = 64;  // above it a row that fits one workgroup is given to one (of enough threads)

// (for_size: what a call could use whatever rows.path says at that time)
RowsCfg choose_rows_cfg(const View &v, int k, int dtype, bool for_size = false) {
    RowsCfg c;
    if (v.g.inner != 1 || k > vkop::kFastMaxK || v.g.n == 0 || v.g.outer == 0) return c;
    const uint32_t vec = dtype == VKOP_HIP_F32 ? 4u : 8u;
    const uint32_t n = v.g.n, rows = v.g.outer;
    static const int shapes_f32[][2] = {{256, 1}, {256, 2}, {256, 4}, {256, 8}, {512, 8}, {1024, 8}};
    static const int shapes_f16[][2] = {{256, 1}, {256, 2}, {256, 4}, {512, 4}, {1024, 4}, {1024, 4}};
    const auto *shapes = dtype == VKOP_HIP_F32 ? shapes_f32 : shapes_f16;
    int forced_nt = g_rows_threads.load(), forced_v = g_rows_loads.load(), forced_g = g_rows_chunks.load();
    if (forced_nt <= 0 || forced_v <= 0 || forced_g <= 0) forced_nt = 0;
    const uint32_t nvec = (n + vec - 1) / vec;
    const uint32_t cap = rows_cap(k);
    auto fits = [&](int nt, int vv, uint32_t g) {
        const uint32_t nw = static_cast<uint32_t>(nt) / 64u;
        if (g < 1 || g > static_cast<uint32_t>(vkop::kMergeChunksMax)) return false;
        if (static_cast<uint64_t>(g) * nw > static_cast<uint64_t>(vkop::kMergeWavesMax)) return false;
        if (static_cast<uint64_t>(g) * cap > static_cast<uint64_t>(vkop::kMergeRecsMax)) return false;
        const uint64_t span = static_cast<uint64_t>(nt) * vv * vec;
        return span * g >= n && static_cast<uint64_t>(rows) * g < (1ull << 31);
    };
    // short rows and a small k: one wave per row (64 threads, up to 8 loads each)
    const uint32_t wave_loads = (nvec + 63) / 64;
    // A large k on a row that one workgroup can hold: that workgroup takes the whole
    // row, list in LDS, if it has at least 2 (k + 1) threads (its waves share the
    // staging of the candidates, 64 vectors each, and the ranking; several chunks of
    // 256 threads would hand a merge of 256 threads more candidates than it ranks
    // quickly).  Beyond 255 ranks it is the only way: the merge kernel has a thread
    // per rank.
    int wide = -1;
    if (cap <= static_cast<uint32_t>(vkop::kLocalCap)) {
        for (int i = 0; i < 6 && wide < 0; i++) {
            const uint64_t span = static_cast<uint64_t>(shapes[i][0]) * shapes[i][1] * vec;
            if (span >= n && shapes[i][0] >= 2 * (k + 1)) wide = i;
        }
    }
    if (k > vkop::kMergeThreads - 1 && wide < 0) return c;
    if (wide >= 0 && (k > vkop::kMergeThreads - 1 || (k > kWideRowMinK && !forced_nt))) {
        c.nt = shapes[wide][0], c.v = shapes[wide][1], c.g = 1;
    } else if (forced_nt) {
        if (!fits(forced_nt, forced_v, static_cast<uint32_t>(forced_g))) return c;
        c.nt = forced_nt, c.v = forced_v, c.g = static_cast<uint32_t>(forced_g);
    } else if (k <= kWaveRowMaxK && wave_loads <= (dtype == VKOP_HIP_F32 ? 8u : 4u)) {
        c.nt = 64, c.g = 1;
        c.v = wave_loads <= 1 ? 1 : wave_loads <= 2 ? 2 : wave_loads <= 4 ? 4 : 8;
    } else {
        // Several chunks a row.  With a k above 64 (only rows the scan kernels do not take
        // get here: half-precision rows of 32K to 64K elements, rows beyond 8192 blocks) the
        // chunks' lists overflow on anything but well-spread data and are made again from an
        // exact select, 70 to 700 us measured; the multi-pass radix select takes 50 us
        // whatever the data.  (rows.path = 1 keeps these kernels on every shape they can do.)
        if (!for_size && k > kWideRowMinK && g_rows_path.load() != 1) return c;
        // a row that one workgroup of 256 threads can hold: the smallest such shape (many short rows
        // would otherwise get the largest workgroup, most of its threads without an element); else the
        // largest per-workgroup chunk that still leaves >= 1024 workgroups; if the
        // tensor is too small for that, the smallest shape that covers a row
        int pick = -1;
        for (int i = 0; i < 4 && pick < 0; i++) {
            const uint64_t span = static_cast<uint64_t>(shapes[i][0]) * shapes[i][1] * vec;
            if (shapes[i][0] == 256 && span >= n && fits(shapes[i][0], shapes[i][1], 1)) pick = i;
        }
        // a row just past those shapes that has too few blocks for the scan kernels (8193 to 8320 elements at
        // k = 64): the wider workgroup that holds it, rather than several chunks and a merge
        const uint32_t blocks = (n + vkop::kBlockLanes * vec - 1) / (vkop::kBlockLanes * vec);
        if (pick < 0 && wide >= 0 && !forced_nt && g_rows_path.load() != 1 &&
            4ull * blocks < (rows <= 16 ? 8ull : 7ull) * (static_cast<uint64_t>(k) + 1u))
            pick = wide;
        const bool one_workgroup = pick >= 0;
        for (int i = 0; i < 6 && !one_workgroup; i++) {
            const uint32_t span = static_cast<uint32_t>(shapes[i][0]) * shapes[i][1] * vec;
            const uint32_t g = (n + span - 1) / span;
            if (!fits(shapes[i][0], shapes[i][1], g)) continue;
            if (pick < 0) pick = i;
            if (static_cast<uint64_t>(rows) * g >= 1024) pick = i;
        }
        if (pick < 0) return c;
        c.nt = shapes[pick][0], c.v = shapes[pick][1];
        const uint32_t span = static_cast<uint32_t>(c.nt) * c.v * vec;
        c.g = (n + span - 1) / span;
    }
    // chunks are whole multiples of the workgroup's capacity wherever the row allows
    // it, so that all but the last chunk of a row run the unmasked code
    c.per = static_cast<uint32_t>(c.nt) * c.v * vec;
    if (static_cast<uint64_t>(c.per) * (c.g - 1) >= n) c.per = (nvec + c.g - 1) / c.g * vec;
    c.cap = cap;
    while ((1u << c.cap_shift) < c.cap) c.cap_shift++;
    c.ok = true;
    return c;
}

// Short last-axis rows, largest first, k up to kTinyMaxK: one wave per row
// (kernels_tiny.hpp); v = 128-bit loads per lane, 0 = not for this tensor.
int choose_tiny_loads(const View &v, int k, int dtype) {
    if (v.g.inner != 1 || k < 1 || k > vkop::kTinyMaxK || v.g.n == 0 || v.g.outer == 0) return 0;
    if (g_rows_path.load() == 1) return 0;
    if (g_rows_threads.load() > 0 && g_rows_loads.load() > 0 && g_rows_chunks.load() > 0) return 0;
    const uint32_t vec = dtype == VKOP_HIP_F32 ? 4u : 8u;
    const int vmax = dtype == VKOP_HIP_F32 ? 8 : 4;
    for (int vv = 1; vv <= vmax; vv *= 2)
        if (static_cast<uint32_t>(vkop::kWave) * vv * vec >= v.g.n) return vv;
    return 0;
}

template <typename T, bool SOFTMAX>
int launch_tiny(const T *in, T *values, int32_t *indices, const View &v, int k, int loads, hipStream_t st,
                bool smallest = false, bool sampling = false, float scale = 1.f, int32_t *counts = nullptr, float top_p = 0.f) {
    vkop::TinyLaunch a;
    a.in = in;
    a.values = values;
    a.indices = indices;
    a.rows = v.g.outer;
    a.n = v.g.n;
    a.k = static_cast<uint32_t>(k);
    a.v = static_cast<uint32_t>(loads);
    a.aligned = (reinterpret_cast<uintptr_t>(in) % 16 == 0) && (v.g.n % (16 / sizeof(T)) == 0);
    a.smallest = smallest;
    a.stream = st;
    a.sampling = sampling;
    a.scale = scale;
    a.counts = counts;
    a.top_p = top_p;
    if (!vkop::launch_rows_tiny<T, SOFTMAX>(a)) return fail(VKOP_HIP_ERR_UNSUPPORTED, "no rows_tiny_kernel for %d loads", loads);
    return launched("rows_tiny_kernel");
}

// Launch shape of the streaming pair rows_scan_kernel + rows_pick_kernel: 256 threads,
// V 128-bit loads per thread, G chunks per row; blocks = 256-byte blocks per row.
struct ScanCfg {
    bool ok = false;
    int v = 0;
    uint32_t g = 0, blocks = 0;
    uint32_t g2 = 0;  // k beyond the pick kernel's list: workgroups a row of the gather kernel (kernels_bigpick.hpp)
};

// Long last-axis rows, largest first: the scan kernel followed by the pick kernel (k up to
// kFastMaxK) or by the large-k pair (g2 != 0: beyond that k, and on up to 16 rows from k = 256,
// or from k = 160 where the pick kernel has too few blocks).  The largest chunk that still
// leaves 512 workgroups (else the smallest); rows too short to be split, or with too few
// blocks per wanted place (below), or with more blocks than the kernel behind the scan takes
// in, are left to the other kernels.
// (for_size: what a call could use whatever the tuning knobs say at that time)
ScanCfg choose_scan_cfg(const View &v, int k, int dtype, bool for_size = false) {
    ScanCfg c;
    if (v.g.inner != 1 || k > vkop::kMaxK || v.g.n == 0 || v.g.outer == 0) return c;
    const uint32_t vec = dtype == VKOP_HIP_F32 ? 4u : 8u;
    const uint32_t n = v.g.n, rows = v.g.outer;
    // The pick kernel ranks a row in one workgroup, the large-k pair spreads it over many: on up to 16
    // rows that pair is the faster one from k = 256 on ([8,262144] k = 256: 17.7 against 23.1 us;
    // [4,100000] k = 500: 15.6 against 44 us), with more rows the pick kernel stays ahead up to its
    // limit ([64,128256] k = 500 fused: 50 against 52 us; [128,65536] k = 256: 24 against 39 us).
    const bool few_rows = rows <= 16;
    bool big = k > vkop::kFastMaxK || (few_rows && k >= 256);
    if (!for_size) {
        if (g_rows_path.load() == 1) return c;
        // a forced shape of the other streaming kernels
        if (g_rows_threads.load() > 0 && g_rows_loads.load() > 0 && g_rows_chunks.load() > 0) return c;
    }
    const uint32_t blocks = (n + vkop::kBlockLanes * vec - 1) / (vkop::kBlockLanes * vec);
    // Blocks per wanted place, in quarters.  The pick kernel's threshold is the (k+1)-th largest of its
    // 512 threads' maxima: at or above their median -- k + 1 <= 256, twice as many blocks -- few blocks
    // and elements reach it; closer to the smallest of them, more blocks have to stand behind every
    // thread -- which costs one workgroup per row less when other rows keep the chip busy: with more
    // than 16 rows, 1.75 blocks a place are enough at every k ([64,128256] f16 k = 300, 3.3 a place:
    // 28.9 us, fused 34.5, against 49 / 132 us of the radix select; [32,50257] f16 k = 200, 1.95 a
    // place: 24.4 against 46.8 us).  The large-k kernels get by with 1.25 a place on a few rows (they
    // read most of the row again then, and still beat the radix select: [8,262144] f16 k = 1024, 2048
    // blocks: 21.7 against 42.8 us; [2,65536] k = 512: 16.0 against 37.8 us); with many rows their
    // ranking is what the time goes into ([64,100000] k = 1240: 125 against 64 us).
    const uint64_t places = static_cast<uint64_t>(k) + 1u;
    uint32_t quarters = big ? (few_rows ? 5u : 8u) : (!few_rows ? 7u : (places <= 256 ? 8u : 16u));
    if (!big && few_rows && k >= 160 && 4ull * blocks < quarters * places) {
        // too few blocks for the pick kernel on a few rows: the large-k pair again, from k = 160 on (below,
        // rows sorted in runs cost it several times the radix select: [16,128256] k = 128: 422 us)
        // ([8,50257] f16 k = 200: 16.8 against 44.5 us of the radix select; [16,100000] f16 k = 400: 21.0 against 38.9)
        big = true;
        quarters = 5u;
    }
    if (4ull * blocks < quarters * places) return c;
    if (k <= vkop::kFastMaxK && !for_size) {
        // a row that ONE workgroup of the chunk kernel holds (up to 8192 elements for k <= 64, up to
        // 32768 beyond): one launch instead of two, measured 1.4 to 1.6 times faster on spread-out
        // rows ([1024,4096] k = 16: 9.0 against 14.5 us; [64,32768] k = 200: 12.5 against 20.3 us)
        const RowsCfg one = choose_rows_cfg(v, k, dtype);
        if (one.ok && one.g == 1 && one.nt >= 256) return c;
    }
    if (!big && (blocks + vkop::kPickThreads - 1) / vkop::kPickThreads > 32u) return c;
    if (big && (blocks + vkop::kBigPickThreads - 1) / vkop::kBigPickThreads > 32u) return c;
    if (big && static_cast<uint64_t>(rows) * (vkop::kBigPickCap / vkop::kBigPickMine) >= (1ull << 31)) return c;
    const uint32_t waves_max = big ? static_cast<uint32_t>(vkop::kBigPickRecsMax) : static_cast<uint32_t>(vkop::kMergeWavesMax);
    const int vmax = dtype == VKOP_HIP_F32 ? 16 : 8;
    int pick = 0;
    for (int vv = 2; vv <= vmax; vv *= 2) {
        const uint32_t per = static_cast<uint32_t>(vkop::kScanThreads) * vv * vec;
        const uint32_t g = (n + per - 1) / per;
        if (g < 2 || g * vkop::kScanWaves > waves_max) continue;
        if (static_cast<uint64_t>(rows) * g >= (1ull << 31)) continue;
        if (pick == 0) pick = vv;
        if (static_cast<uint64_t>(rows) * g >= 512) pick = vv;
    }
    if (pick == 0) return c;
    c.v = pick;
    const uint32_t per = static_cast<uint32_t>(vkop::kScanThreads) * pick * vec;
    c.g = (n + per - 1) / per;
    c.blocks = blocks;
    if (big) {
        // a share of at most 256 blocks (a thread each) and, rows permitting, of at least 32;
        // about 512 workgroups in all
        const uint32_t least = (blocks + 255u) / 256u, most = (blocks + 31u) / 32u;
        const uint32_t fill = (512u + rows - 1u) / rows;
        c.g2 = std::max(least, std::min(fill, most));
        if (static_cast<uint64_t>(rows) * c.g2 >= (1ull << 31)) return c;
    }
    c.ok = true;
    return c;
}

struct RowsLayout {
    size_t tickets = 0, sums = 0, cand = 0, stats = 0, total = 0;
    // scan + pick pair (kernels_stream.hpp)
    size_t bmax = 0, recs = 0, bmin = 0, bcand = 0, bterm = 0, bhead = 0, bstat = 0;
    // multi-workgroup radix select (kernels_bigk.hpp)
    size_t hist = 0, hist_bytes = 0, state = 0, counts = 0, sel = 0, chunkstats = 0;
};

// Launch shape of the multi-workgroup radix select: chunks of 8192 elements.
struct BigKCfg {
    bool ok = false;
    int v = 0;
    uint32_t g = 0, per = 0, kpad = 0;
};

BigKCfg choose_bigk_cfg(const View &v, int k, int dtype) {
    BigKCfg c;
    if (v.g.inner != 1 || v.g.n < 16384 || k < 1 || k > vkop::kMaxK || v.g.outer == 0) return c;
    c.v = dtype == VKOP_HIP_F32 ? 8 : 4;
    c.per = static_cast<uint32_t>(vkop::kBigThreads) * c.v * (dtype == VKOP_HIP_F32 ? 4u : 8u);
    c.g = (v.g.n + c.per - 1) / c.per;
    if (c.g > static_cast<uint32_t>(vkop::kBigThreads) || static_cast<uint64_t>(v.g.outer) * c.g >= (1ull << 31)) return c;
    c.kpad = (static_cast<uint32_t>(k) + 31u) / 32u * 32u;
    c.ok = true;
    return c;
}

// One layout serves the streaming kernel and the general two-kernel path, so
// the size does not depend on which of them a call ends up taking.
// (the arrival counters come first, see kTicketRows)

RowsLayout rows_layout(const View &v, const RowsCfg &c, const BigKCfg &b = BigKCfg{}, const ScanCfg &sc = ScanCfg{}) {
    RowsLayout l;
    const size_t lines = static_cast<size_t>(v.g.outer) * v.g.inner;
    size_t off = 0;
    l.tickets = off;
    off += kTicketBytes;
    l.stats = off;
    off += align_up(lines * sizeof(vkop::LineStats));
    if (sc.ok) {
        l.bmax = off;
        off += align_up(lines * sc.blocks * sizeof(uint32_t));
        l.recs = off;
        off += align_up(lines * sc.g * vkop::kScanWaves * 3 * sizeof(uint64_t));  // (two words a wave, then the waves' third words)
        if (sc.g2 != 0) {
            l.bmin = off;
            off += align_up(lines * sc.blocks * sizeof(uint32_t));
            l.bcand = off;
            off += align_up(lines * vkop::kBigPickLists * vkop::kBigPickListCap * sizeof(uint64_t));
            l.bterm = off;
            off += align_up(lines * vkop::kBigPickLists * vkop::kBigPickListCap * sizeof(float));
            l.bhead = off;
            off += align_up(lines * vkop::kBigPickHeadWords * sizeof(uint32_t));
            l.bstat = off;
            off += align_up(2 * lines * sizeof(double));
        }
    } else if (c.ok) {
        const size_t chunks = lines * c.g;
        l.sums = off;
        off += align_up(chunks * (static_cast<size_t>(c.nt) / 64) * vkop::kRecWords * sizeof(uint64_t));
        l.cand = off;
        off += align_up(chunks * c.cap * sizeof(uint64_t));
    } else if (b.ok) {
        const size_t chunks = lines * b.g;
        l.hist = off;
        l.hist_bytes = align_up(3 * lines * vkop::kBigBins * sizeof(uint32_t));
        off += l.hist_bytes;
        l.state = off;
        off += align_up(lines * 8 * sizeof(uint32_t));
        l.counts = off;
        off += align_up(chunks * 2 * sizeof(uint32_t));
        l.sel = off;
        off += align_up(lines * b.kpad * sizeof(uint64_t));
        l.chunkstats = off;
        off += align_up(chunks * sizeof(vkop::ChunkStat));
    }
    l.total = off;
    return l;
}

template <typename T, bool SOFTMAX>
int launch_bigk(const T *in, T *values, int32_t *indices, const View &v, int k, int largest, const BigKCfg &c, void *ws,
                const RowsLayout &l, hipStream_t st, bool in_order = true) {
    auto *base = static_cast<unsigned char *>(ws);
    vkop::BigKWorkspace w;
    w.hist = reinterpret_cast<uint32_t *>(base + l.hist);
    w.state = reinterpret_cast<uint32_t *>(base + l.state);
    w.counts = reinterpret_cast<uint32_t *>(base + l.counts);
    w.sel = reinterpret_cast<uint64_t *>(base + l.sel);
    auto *stats = reinterpret_cast<vkop::LineStats *>(base + l.stats);
    w.stats = stats;
    w.kpad = c.kpad;
    const uint32_t rows = v.g.outer, n = v.g.n, blocks = rows * c.g;
    const uint32_t flip = largest ? 0u : 0xFFFFFFFFu;
    const uint32_t uk = static_cast<uint32_t>(k);
    const uint32_t vec = 16 / sizeof(T);
    const bool aligned = (reinterpret_cast<uintptr_t>(in) % 16 == 0) && (n % vec == 0);
    constexpr int V = sizeof(T) == 4 ? 8 : 4;
    constexpr int NT = vkop::kBigThreads;
    const size_t words = l.hist_bytes / 4;
    vkop::fill_zero_kernel<<<static_cast<unsigned>((words + 255) / 256), 256, 0, st>>>(w.hist, words);
    auto run = [&](auto al) {
        constexpr bool AL = decltype(al)::value;
        if constexpr (SOFTMAX) {
            auto *cs = reinterpret_cast<vkop::ChunkStat *>(base + l.chunkstats);
            vkop::softmax_stats_kernel<T, NT, V, AL><<<blocks, NT, 0, st>>>(in, cs, n, c.g, c.per);
            vkop::bigk_row_stats_kernel<<<rows, vkop::kWave, 0, st>>>(cs, stats, c.g);
        }
        vkop::bigk_hist_kernel<T, V, SOFTMAX, AL, 0><<<blocks, NT, 0, st>>>(in, n, uk, c.g, c.per, flip, w);
        vkop::bigk_hist_kernel<T, V, SOFTMAX, AL, 1><<<blocks, NT, 0, st>>>(in, n, uk, c.g, c.per, flip, w);
        vkop::bigk_hist_kernel<T, V, SOFTMAX, AL, 2><<<blocks, NT, 0, st>>>(in, n, uk, c.g, c.per, flip, w);
        vkop::bigk_count_kernel<T, V, SOFTMAX, AL><<<blocks, NT, 0, st>>>(in, n, c.g, c.per, flip, w);
        vkop::bigk_gather_kernel<T, V, SOFTMAX, AL><<<blocks, NT, 0, st>>>(in, n, uk, c.g, c.per, flip, w);
    };
    if (aligned) run(std::true_type{});
    else run(std::false_type{});
    const uint32_t slices = (uk + vkop::kBigSortSlice - 1) / vkop::kBigSortSlice;
    vkop::bigk_sort_kernel<T, SOFTMAX>
        <<<rows * slices, vkop::kBigSortThreads, 0, st>>>(in, values, indices, n, uk, slices, w, in_order ? 1u : 0u);
    return launched("multi-workgroup radix select");
}

template <typename T, bool SOFTMAX>
int launch_scan(const T *in, T *values, int32_t *indices, const View &v, int k, const ScanCfg &c, void *ws,
                const RowsLayout &l, hipStream_t st, float scale = 1.f, int32_t *counts = nullptr, float top_p = 0.f) {
    auto *base = static_cast<unsigned char *>(ws);
    const uint32_t vec = 16 / sizeof(T);
    vkop::ScanLaunch a;
    a.in = in;
    a.values = values;
    a.indices = indices;
    a.rows = v.g.outer;
    a.n = v.g.n;
    a.k = static_cast<uint32_t>(k);
    a.v = static_cast<uint32_t>(c.v);
    a.g = c.g;
    a.aligned = (reinterpret_cast<uintptr_t>(in) % 16 == 0) && (v.g.n % vec == 0);
    a.stages = measured_stages();
    a.scale = scale;
    a.counts = counts;
    a.top_p = top_p;
    a.ws.bmax = reinterpret_cast<uint32_t *>(base + l.bmax);
    a.ws.recs = reinterpret_cast<uint64_t *>(base + l.recs);
    a.ws.recs2 = a.ws.recs + 2 * static_cast<size_t>(v.g.outer) * c.g * vkop::kScanWaves;
    a.ws.blocks = c.blocks;
    a.ws.bmin = nullptr;
    a.ws.zero = nullptr;
    a.ws.zero_words = 0;
    a.g2 = c.g2;
    a.bw = vkop::BigPickWorkspace{nullptr, nullptr, nullptr, nullptr};
    if (c.g2 != 0) {
        a.bw.cand = reinterpret_cast<uint64_t *>(base + l.bcand);
        a.bw.term = reinterpret_cast<float *>(base + l.bterm);
        a.bw.head = reinterpret_cast<uint32_t *>(base + l.bhead);
        a.bw.stat = reinterpret_cast<double *>(base + l.bstat);
        a.ws.bmin = reinterpret_cast<uint32_t *>(base + l.bmin);
        a.ws.zero = a.bw.head;
        a.ws.zero_words = vkop::kBigPickHeadWords;
    }
    a.stream = st;
    if (!vkop::launch_rows_scan<T, SOFTMAX>(a))
        return fail(VKOP_HIP_ERR_UNSUPPORTED, "no rows_scan_kernel / rows_pick_kernel for %d loads, %u blocks", c.v, c.blocks);
    return launched("rows_scan_kernel / rows_pick_kernel");
}

template <typename T, bool SOFTMAX>
int launch_rows(const T *in, T *values, int32_t *indices, const View &v, int k, const RowsCfg &c, void *ws,
                const RowsLayout &l, hipStream_t st, bool sampling = false, float scale = 1.f, int32_t *counts = nullptr,
                float top_p = 0.f) {
    vkop::RowsWorkspace w;
    auto *base = static_cast<unsigned char *>(ws);
    w.tickets = reinterpret_cast<uint32_t *>(base + l.tickets);
    w.sums = reinterpret_cast<uint64_t *>(base + l.sums);
    w.cand = reinterpret_cast<uint64_t *>(base + l.cand);
    w.cap = c.cap;
    w.cap_shift = c.cap_shift;
    const uint32_t vec = 16 / sizeof(T);
    // more rows than arrival counters: the merge runs as a kernel of its own
    const bool by_ticket = g_rows_fused.load() != 0 && v.g.outer <= kTicketRows;
    vkop::RowsLaunch a;
    a.in = in;
    a.values = values;
    a.indices = indices;
    a.rows = v.g.outer;
    a.n = v.g.n;
    a.k = static_cast<uint32_t>(k);
    a.nt = static_cast<uint32_t>(c.nt);
    a.v = static_cast<uint32_t>(c.v);
    a.g = c.g;
    a.per = c.per;
    a.aligned = (reinterpret_cast<uintptr_t>(in) % 16 == 0) && (v.g.n % vec == 0);
    // a row that one workgroup holds never leaves it: list and records stay in LDS
    a.merge = (c.g == 1 && c.cap <= static_cast<uint32_t>(vkop::kLocalCap)) ? vkop::kMergeLocal
              : (c.g == 1 || by_ticket)                                         ? vkop::kMergeByTicket
                                                                                : vkop::kMergeSplit;
    if (a.merge == vkop::kMergeLocal) {
        // the list is in LDS, where the kernel reserves kLocalCap entries whatever k is: all of them are the
        // list (an overflow -- values equal en masse at the cut -- makes the workgroup list a second time)
        w.cap = static_cast<uint32_t>(vkop::kLocalCap);
        w.cap_shift = 0;
        while ((1u << w.cap_shift) < w.cap) w.cap_shift++;
    }
    a.ws = w;
    a.stream = st;
    a.sampling = sampling;
    a.scale = scale;
    a.counts = counts;
    a.top_p = top_p;
    if (sampling && a.merge != vkop::kMergeLocal) return fail(VKOP_HIP_ERR_UNSUPPORTED, "no scaled form of these kernels for this shape");
    const int stages = a.merge != vkop::kMergeSplit ? 1 : measured_stages();
    if (stages & 1) {
        if (!vkop::launch_rows_chunk<T, SOFTMAX>(a))
            return fail(VKOP_HIP_ERR_UNSUPPORTED, "no rows_chunk_kernel for %d threads x %d loads", c.nt, c.v);
        if (int rc = launched("rows_chunk_kernel")) return rc;
    }
    if (a.merge == vkop::kMergeSplit && (stages & 2)) {
        vkop::launch_rows_merge<T, SOFTMAX>(a);
        return launched("rows_merge_kernel");
    }
    return VKOP_HIP_OK;
}

// ------------------------------------------------------------------ top-k ----
template <typename T>
int topk_impl(const T *in, T *values, int32_t *indices, const View &v, int k, int largest, int sorted, int dtype, void *ws,
              size_t ws_bytes, hipStream_t st) {
    // (the one-wave kernel serves both directions: it turns its order keys round)
    if (const int tiny = choose_tiny_loads(v, k, dtype)) return launch_tiny<T, false>(in, values, indices, v, k, tiny, st, !largest);
    const ScanCfg sc = largest ? choose_scan_cfg(v, k, dtype) : ScanCfg{};
    const RowsCfg c = (largest && !sc.ok) ? choose_rows_cfg(v, k, dtype) : RowsCfg{};
    const BigKCfg b = (c.ok || sc.ok) ? BigKCfg{} : choose_bigk_cfg(v, k, dtype);
    if (sc.ok || c.ok || b.ok) {
        const RowsLayout l = rows_layout(v, c, b, sc);
        if (ws == nullptr || ws_bytes < l.total)
            return fail(VKOP_HIP_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", ws_bytes, l.total);
        if ((reinterpret_cast<uintptr_t>(ws) & (kAlign - 1)) != 0)
            return fail(VKOP_HIP_ERR_WORKSPACE, "workspace must be %zu-byte aligned", kAlign);
        if (sc.ok) return launch_scan<T, false>(in, values, indices, v, k, sc, ws, l, st);
        if (c.ok) return launch_rows<T, false>(in, values, indices, v, k, c, ws, l, st);
        // (sorted == 0: the one route where an order costs a step of its own leaves it out; every other route's
        // result is in order by construction, which satisfies "any order" too)
        return launch_bigk<T, false>(in, values, indices, v, k, largest, b, ws, l, st, sorted != 0);
    }
    const uint32_t lines = v.g.outer * v.g.inner;
    // one workgroup per line: a big one when the line is long and lines are few
    if (v.g.n >= 4096 && lines <= 1024)
        vkop::topk_lines_kernel<T, 1024><<<lines, 1024, 0, st>>>(in, values, indices, v.g, static_cast<uint32_t>(k), largest);
    else
        vkop::topk_lines_kernel<T, kLineThreads>
            <<<lines, kLineThreads, 0, st>>>(in, values, indices, v.g, static_cast<uint32_t>(k), largest);
    return launched("topk_lines_kernel");
}

// ------------------------------------------------------------------ fused ----
// Which route a fused call takes; the workspace size follows from it.
struct FusedPlan {
    ScanCfg scan;
    RowsCfg rows;
    BigKCfg big;
};
FusedPlan plan_fused(const View &v, int k, int dtype, int largest, bool want_probs) {
    FusedPlan p;
    if (want_probs) return p;  // the softmax tensor is written by the general kernels
    if (largest) p.scan = choose_scan_cfg(v, k, dtype);
    if (largest && !p.scan.ok) p.rows = choose_rows_cfg(v, k, dtype);
    if (!p.scan.ok && !p.rows.ok) p.big = choose_bigk_cfg(v, k, dtype);
    return p;
}

template <typename T>
int fused_impl(const T *in, T *probs, T *values, int32_t *indices, const View &v, int k, int largest, int dtype,
               void *ws, hipStream_t st, size_t ws_limit = ~static_cast<size_t>(0)) {
    if (const int tiny = (largest && probs == nullptr) ? choose_tiny_loads(v, k, dtype) : 0)
        return launch_tiny<T, true>(in, values, indices, v, k, tiny, st);
    const FusedPlan p = plan_fused(v, k, dtype, largest, probs != nullptr);
    const RowsLayout l = rows_layout(v, p.rows, p.big, p.scan);
    // (the layout the kernels are given is the one checked here: a tuning change between a caller's
    // size query and this call cannot put it past the end of what the caller holds)
    if (l.total > ws_limit)
        return fail(VKOP_HIP_ERR_WORKSPACE, "this call's scratch layout takes %zu bytes, %zu are there", l.total, ws_limit);
    if (p.scan.ok) return launch_scan<T, true>(in, values, indices, v, k, p.scan, ws, l, st);
    if (p.rows.ok) return launch_rows<T, true>(in, values, indices, v, k, p.rows, ws, l, st);
    if (p.big.ok) return launch_bigk<T, true>(in, values, indices, v, k, largest, p.big, ws, l, st);
    // general path: line statistics (and the softmax tensor when asked for), then
    // an exact select keyed by the probabilities those statistics define
    const uint32_t lines = v.g.outer * v.g.inner;
    auto *stats = reinterpret_cast<vkop::LineStats *>(static_cast<unsigned char *>(ws) + l.stats);
    vkop::softmax_lines_kernel<T, kLineThreads><<<lines, kLineThreads, 0, st>>>(in, probs, v.g, 0, 0.f, stats);
    if (int rc = launched("softmax_lines_kernel")) return rc;
    vkop::softmax_topk_lines_kernel<T, kLineThreads>
        <<<lines, kLineThreads, 0, st>>>(in, stats, values, indices, v.g, static_cast<uint32_t>(k), largest);
    return launched("softmax_topk_lines_kernel");
}

// Workspace that serves whichever route a top-k or fused call on this tensor can
// take (largest or smallest, with or without the softmax tensor).
size_t selection_workspace(const View &v, int k, int dtype) {
    const size_t a = rows_layout(v, choose_rows_cfg(v, k, dtype, true)).total;
    const size_t b = rows_layout(v, RowsCfg{}, choose_bigk_cfg(v, k, dtype)).total;
    const size_t c = rows_layout(v, RowsCfg{}, BigKCfg{}, choose_scan_cfg(v, k, dtype, true)).total;
    return a > b ? (a > c ? a : c) : (b > c ? b : c);
}

// max over `axis` of the softmax along `axis`, without the softmax tensor
template <typename T>
int softmax_reduce_max_impl(const T *in, T *out, const View &v, void *ws, size_t ws_bytes, hipStream_t st) {
    const uint32_t lines = v.g.outer * v.g.inner;
    if (v.g.n <= static_cast<uint32_t>(vkop::kStridedMaxN)) {
        launch_strided_reg<T, true>(in, out, v, 0, 0.f, st);
        return launched("softmax_strided_reg_kernel");
    }
    if (v.g.inner != 1) {
        // long lines along a non-last axis: the statistics of the tile kernel, as the softmax itself takes them
        const SoftmaxPlan p = plan_softmax(v, sizeof(T) == 4 ? VKOP_HIP_F32 : VKOP_HIP_F16);
        const uint32_t tiles = v.g.outer * ((v.g.inner + (1u << p.ti_shift) - 1) >> p.ti_shift);
        if (p.g == 1) {
            vkop::softmax_strided_tile_kernel<T, vkop::kTileWholeMax>
                <<<tiles, vkop::kStridedTileThreads, 0, st>>>(in, out, nullptr, v.g, p.ti_shift, 1, v.g.n, 0, 0.f);
            return launched("softmax_strided_tile_kernel (max)");
        }
        if (ws == nullptr || ws_bytes < p.workspace)
            return fail(VKOP_HIP_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", ws_bytes, p.workspace);
        auto *cstats = reinterpret_cast<vkop::ChunkStat *>(static_cast<unsigned char *>(ws) + kTicketBytes);
        vkop::softmax_strided_tile_kernel<T, vkop::kTileStats>
            <<<tiles * p.g, vkop::kStridedTileThreads, 0, st>>>(in, out, cstats, v.g, p.ti_shift, p.g, p.per, 0, 0.f);
        vkop::softmax_strided_tile_kernel<T, vkop::kTileFoldMax>
            <<<tiles * p.g, vkop::kStridedTileThreads, 0, st>>>(in, out, cstats, v.g, p.ti_shift, p.g, p.per, 0, 0.f);
        return launched("softmax_strided_tile_kernel (split, max)");
    }
    // long rows: the line statistics, then exp_accurate(0) / S per line
    const size_t need = kTicketBytes + align_up(static_cast<size_t>(lines) * sizeof(vkop::LineStats));
    if (ws == nullptr || ws_bytes < need)
        return fail(VKOP_HIP_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", ws_bytes, need);
    auto *stats = reinterpret_cast<vkop::LineStats *>(static_cast<unsigned char *>(ws) + kTicketBytes);
    vkop::softmax_lines_kernel<T, kLineThreads>
        <<<lines, kLineThreads, 0, st>>>(in, static_cast<T *>(nullptr), v.g, 0, 0.f, stats);
    vkop::stats_to_max_kernel<T><<<(lines + 255) / 256, 256, 0, st>>>(stats, out, lines);
    return launched("softmax_lines_kernel / stats_to_max_kernel");
}

template <typename T> int reduce_max_impl(const T *in, T *out, const View &v, hipStream_t st) {
    const uint32_t lines = v.g.outer * v.g.inner;
    if (v.g.inner == 1) {
        vkop::reduce_max_lines_kernel<T, kLineThreads><<<lines, kLineThreads, 0, st>>>(in, out, v.g);
        return launched("reduce_max_lines_kernel");
    }
    const uint32_t per_block = kLineThreads / 4;  // four lanes per line
    const uint32_t blocks = (lines + per_block - 1) / per_block;
    vkop::reduce_max_strided_kernel<T, kLineThreads><<<blocks, kLineThreads, 0, st>>>(in, out, v.g);
    return launched("reduce_max_strided_kernel");
}

// ---------------------------------------------------------------- nms ----
uint32_t nms_max_sel(int N, int max_per_class) {
    uint32_t m = static_cast<uint32_t>(N) < static_cast<uint32_t>(vkop::kNmsMaxCandidates)
                     ? static_cast<uint32_t>(N) : static_cast<uint32_t>(vkop::kNmsMaxCandidates);
    if (max_per_class > 0 && static_cast<uint32_t>(max_per_class) < m) m = static_cast<uint32_t>(max_per_class);
    return m < 1 ? 1 : m;
}
size_t nms_workspace(int B, int C, int N, int max_per_class) {
    const size_t pairs = static_cast<size_t>(B) * C;
    return kTicketBytes + align_up(2 * pairs * sizeof(uint32_t)) + align_up(pairs * nms_max_sel(N, max_per_class) * sizeof(int32_t));
}

template <typename T>
int nms_impl(const T *boxes, const T *scores, int32_t *out, int out_capacity, int32_t *out_count, int B, int C, int N,
             int center_point_box, int max_per_class, float iou_threshold, float score_threshold, void *ws, hipStream_t st) {
    const uint32_t pairs = static_cast<uint32_t>(B) * static_cast<uint32_t>(C);
    auto *base = static_cast<unsigned char *>(ws) + kTicketBytes;
    auto *counts = reinterpret_cast<uint32_t *>(base);
    auto *selected = reinterpret_cast<int32_t *>(base + align_up(2 * static_cast<size_t>(pairs) * sizeof(uint32_t)));
    const uint32_t max_sel = nms_max_sel(N, max_per_class);
    const uint32_t per = max_per_class > 0 ? static_cast<uint32_t>(max_per_class) : 0u;
    const int knob = g_nms_threads;  // 0: by the number of pairs
    const bool narrow = knob > 0 ? knob == vkop::kNmsThreadsNarrow : pairs >= static_cast<uint32_t>(vkop::kNmsNarrowMinPairs);
    // rows that start on 16-byte boundaries and hold a multiple of four scores are read four scores per load
    const bool vec = N % 4 == 0 && N >= 4 && (reinterpret_cast<uintptr_t>(scores) & 15u) == 0;
#define VKOP_NMS_LAUNCH(NT, VEC)                                                                                          \
    vkop::nms_kernel<T, NT, VEC><<<pairs, NT, 0, st>>>(boxes, scores, selected, counts, pairs, static_cast<uint32_t>(C),  \
                                                       static_cast<uint32_t>(N), center_point_box, per, iou_threshold,   \
                                                       score_threshold, max_sel)
    if (narrow && vec) VKOP_NMS_LAUNCH(vkop::kNmsThreadsNarrow, true);
    else if (narrow) VKOP_NMS_LAUNCH(vkop::kNmsThreadsNarrow, false);
    else if (vec) VKOP_NMS_LAUNCH(vkop::kNmsThreadsWide, true);
    else VKOP_NMS_LAUNCH(vkop::kNmsThreadsWide, false);
#undef VKOP_NMS_LAUNCH
    if (int rc = launched("nms_kernel")) return rc;
    vkop::nms_pack_kernel<<<pairs, 256, 0, st>>>(selected, counts, out, out_count, pairs, static_cast<uint32_t>(C), max_sel,
                                                 static_cast<uint32_t>(out_capacity));
    return launched("nms_pack_kernel");
}

}  // namespace

extern "C" {

const char *vkop_hip_last_error(void) { return g_err; }

int vkop_hip_init(int device) {
    int count = 0;
    VKOP_HIP_TRY(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return fail(VKOP_HIP_ERR_INVALID, "device %d of %d", device, count);
    VKOP_HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    VKOP_HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(VKOP_HIP_ERR_UNSUPPORTED, "device %d is %s; this library is built for gfx950 only", device,
                    prop.gcnArchName);
    VKOP_HIP_TRY(hipFree(nullptr));  // force context creation here, not inside the first timed call
    // the address of this device's static scratch, for vkop_hip_softmax_topk_static
    void *sp = nullptr;
    int dev = 0;
    if (int rc = resolve_static_scratch(&sp, &dev)) return rc;
    return VKOP_HIP_OK;
}

int vkop_hip_shutdown(void) {
    VKOP_HIP_TRY(hipDeviceSynchronize());
    return VKOP_HIP_OK;
}

int vkop_hip_device_info(char *name, size_t name_len, int *compute_units, size_t *memory_bytes) {
    int dev = 0;
    VKOP_HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    VKOP_HIP_TRY(hipGetDeviceProperties(&prop, dev));
    if (name != nullptr && name_len > 0) std::snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
    if (compute_units != nullptr) *compute_units = prop.multiProcessorCount;
    if (memory_bytes != nullptr) *memory_bytes = prop.totalGlobalMem;
    return VKOP_HIP_OK;
}

int vkop_hip_malloc(void **ptr, size_t bytes) {
    if (ptr == nullptr) return fail(VKOP_HIP_ERR_INVALID, "ptr is null");
    *ptr = nullptr;
    if (bytes == 0) return VKOP_HIP_OK;
    VKOP_HIP_TRY(hipMalloc(ptr, bytes));
    return VKOP_HIP_OK;
}

int vkop_hip_free(void *ptr) {
    if (ptr == nullptr) return VKOP_HIP_OK;
    VKOP_HIP_TRY(hipFree(ptr));
    return VKOP_HIP_OK;
}

int vkop_hip_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return VKOP_HIP_OK;
    if (dst == nullptr || src == nullptr) return fail(VKOP_HIP_ERR_INVALID, "null pointer in h2d copy");
    VKOP_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    VKOP_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return VKOP_HIP_OK;
}

int vkop_hip_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return VKOP_HIP_OK;
    if (dst == nullptr || src == nullptr) return fail(VKOP_HIP_ERR_INVALID, "null pointer in d2h copy");
    VKOP_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    VKOP_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return VKOP_HIP_OK;
}

int vkop_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return VKOP_HIP_OK;
    if (dst == nullptr || src == nullptr) return fail(VKOP_HIP_ERR_INVALID, "null pointer in d2d copy");
    VKOP_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return VKOP_HIP_OK;
}

int vkop_hip_stream_create(void **stream) {
    if (stream == nullptr) return fail(VKOP_HIP_ERR_INVALID, "stream is null");
    hipStream_t s;
    VKOP_HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
    *stream = s;
    return VKOP_HIP_OK;
}

int vkop_hip_stream_destroy(void *stream) {
    if (stream == nullptr) return VKOP_HIP_OK;
    VKOP_HIP_TRY(hipStreamDestroy(as_stream(stream)));
    return VKOP_HIP_OK;
}

int vkop_hip_stream_sync(void *stream) {
    VKOP_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return VKOP_HIP_OK;
}

int vkop_hip_event_create(void **event) {
    if (event == nullptr) return fail(VKOP_HIP_ERR_INVALID, "event is null");
    hipEvent_t e;
    VKOP_HIP_TRY(hipEventCreate(&e));
    *event = e;
    return VKOP_HIP_OK;
}

int vkop_hip_event_destroy(void *event) {
    if (event == nullptr) return VKOP_HIP_OK;
    VKOP_HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return VKOP_HIP_OK;
}

int vkop_hip_event_record(void *event, void *stream) {
    if (event == nullptr) return fail(VKOP_HIP_ERR_INVALID, "event is null");
    VKOP_HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)));
    return VKOP_HIP_OK;
}

int vkop_hip_event_sync(void *event) {
    if (event == nullptr) return fail(VKOP_HIP_ERR_INVALID, "event is null");
    VKOP_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(event)));
    return VKOP_HIP_OK;
}

int vkop_hip_stream_wait_event(void *stream, void *event) {
    if (event == nullptr) return fail(VKOP_HIP_ERR_INVALID, "event is null");
    VKOP_HIP_TRY(hipStreamWaitEvent(as_stream(stream), static_cast<hipEvent_t>(event), 0));
    return VKOP_HIP_OK;
}

int vkop_hip_event_elapsed_ms(void *start, void *stop, float *ms) {
    if (start == nullptr || stop == nullptr || ms == nullptr) return fail(VKOP_HIP_ERR_INVALID, "null argument");
    VKOP_HIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return VKOP_HIP_OK;
}

int vkop_hip_graph_begin(void *stream) {
    if (stream == nullptr) return fail(VKOP_HIP_ERR_INVALID, "recording needs a stream created by vkop_hip_stream_create");
    VKOP_HIP_TRY(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
    return VKOP_HIP_OK;
}

int vkop_hip_graph_end(void *stream, void **graph) {
    if (stream == nullptr || graph == nullptr) return fail(VKOP_HIP_ERR_INVALID, "null argument");
    *graph = nullptr;
    hipGraph_t g = nullptr;
    VKOP_HIP_TRY(hipStreamEndCapture(as_stream(stream), &g));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) return fail(VKOP_HIP_ERR_DEVICE, "hipGraphInstantiate: %s", hipGetErrorString(e));
    *graph = exec;
    return VKOP_HIP_OK;
}

int vkop_hip_graph_launch(void *graph, void *stream) {
    if (graph == nullptr) return fail(VKOP_HIP_ERR_INVALID, "graph is null");
    VKOP_HIP_TRY(hipGraphLaunch(static_cast<hipGraphExec_t>(graph), as_stream(stream)));
    return VKOP_HIP_OK;
}

int vkop_hip_graph_destroy(void *graph) {
    if (graph == nullptr) return VKOP_HIP_OK;
    VKOP_HIP_TRY(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph)));
    return VKOP_HIP_OK;
}

int vkop_hip_workspace_init(void *workspace, size_t bytes, void *stream) {
    if (bytes == 0) return VKOP_HIP_OK;
    if (workspace == nullptr) return fail(VKOP_HIP_ERR_INVALID, "workspace is null");
    if ((reinterpret_cast<uintptr_t>(workspace) & 3u) != 0 || (bytes & 3u) != 0)
        return fail(VKOP_HIP_ERR_INVALID, "workspace address and size must be multiples of 4");
    const size_t words = bytes / 4;
    const unsigned blocks = static_cast<unsigned>((words + 255) / 256);
    vkop::fill_zero_kernel<<<blocks, 256, 0, as_stream(stream)>>>(static_cast<uint32_t *>(workspace), words);
    return launched("fill_zero_kernel");
}

size_t vkop_hip_softmax_workspace_bytes(int dtype, const int *shape, int ndim, int axis) {
    View v;
    if (check_dtype(dtype) || make_view(shape, ndim, axis, &v)) return 0;
    return plan_softmax(v, dtype).workspace;
}

int vkop_hip_softmax(const void *in, void *out, int dtype, const int *shape, int ndim, int axis, int nan_where,
                     float nan_value, void *workspace, size_t workspace_bytes, void *stream) {
    View v;
    if (int rc = check_dtype(dtype)) return rc;
    if (int rc = make_view(shape, ndim, axis, &v)) return rc;
    if (v.elems == 0) return VKOP_HIP_OK;
    if (in == nullptr || out == nullptr) return fail(VKOP_HIP_ERR_INVALID, "null tensor pointer");
    if (dtype == VKOP_HIP_F32)
        return softmax_impl(static_cast<const float *>(in), static_cast<float *>(out), v, dtype, nan_where, nan_value,
                            workspace, workspace_bytes, as_stream(stream));
    return softmax_impl(static_cast<const uint16_t *>(in), static_cast<uint16_t *>(out), v, dtype, nan_where,
                        nan_value, workspace, workspace_bytes, as_stream(stream));
}

size_t vkop_hip_topk_workspace_bytes(int dtype, const int *shape, int ndim, int axis, int k) {
    View v;
    if (check_dtype(dtype) || make_view(shape, ndim, axis, &v) || k < 1) return 0;
    return selection_workspace(v, k, dtype);
}

int vkop_hip_topk(const void *in, void *out_values, int32_t *out_indices, int dtype, const int *shape, int ndim,
                  int axis, int k, int largest, int sorted, void *workspace, size_t workspace_bytes, void *stream) {
    View v;
    if (int rc = check_dtype(dtype)) return rc;
    if (int rc = make_view(shape, ndim, axis, &v)) return rc;
    if (v.elems == 0 && k == 0) return VKOP_HIP_OK;
    if (int rc = check_k(v, k)) return rc;
    if (v.g.outer == 0 || v.g.inner == 0) return VKOP_HIP_OK;
    if (in == nullptr || out_values == nullptr || out_indices == nullptr)
        return fail(VKOP_HIP_ERR_INVALID, "null tensor pointer");
    if (dtype == VKOP_HIP_F32)
        return topk_impl(static_cast<const float *>(in), static_cast<float *>(out_values), out_indices, v, k, largest,
                         sorted, dtype, workspace, workspace_bytes, as_stream(stream));
    return topk_impl(static_cast<const uint16_t *>(in), static_cast<uint16_t *>(out_values), out_indices, v, k,
                     largest, sorted, dtype, workspace, workspace_bytes, as_stream(stream));
}

size_t vkop_hip_softmax_topk_workspace_bytes(int dtype, const int *shape, int ndim, int axis, int k) {
    View v;
    if (check_dtype(dtype) || make_view(shape, ndim, axis, &v) || k < 1) return 0;
    return selection_workspace(v, k, dtype);
}

int vkop_hip_softmax_topk(const void *in, void *out_probs, void *out_values, int32_t *out_indices, int dtype,
                          const int *shape, int ndim, int axis, int k, int largest, void *workspace,
                          size_t workspace_bytes, void *stream) {
    View v;
    if (int rc = check_dtype(dtype)) return rc;
    if (int rc = make_view(shape, ndim, axis, &v)) return rc;
    if (v.elems == 0 && k == 0) return VKOP_HIP_OK;
    if (int rc = check_k(v, k)) return rc;
    if (v.g.outer == 0 || v.g.inner == 0) return VKOP_HIP_OK;
    if (in == nullptr || out_values == nullptr || out_indices == nullptr)
        return fail(VKOP_HIP_ERR_INVALID, "null tensor pointer");
    const FusedPlan plan = plan_fused(v, k, dtype, largest, out_probs != nullptr);
    const size_t need = rows_layout(v, plan.rows, plan.big, plan.scan).total;
    if (workspace == nullptr || workspace_bytes < need)
        return fail(VKOP_HIP_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    if ((reinterpret_cast<uintptr_t>(workspace) & (kAlign - 1)) != 0)
        return fail(VKOP_HIP_ERR_WORKSPACE, "workspace must be %zu-byte aligned", kAlign);
    if (dtype == VKOP_HIP_F32)
        return fused_impl(static_cast<const float *>(in), static_cast<float *>(out_probs),
                          static_cast<float *>(out_values), out_indices, v, k, largest, dtype, workspace,
                          as_stream(stream), workspace_bytes);
    return fused_impl(static_cast<const uint16_t *>(in), static_cast<uint16_t *>(out_probs),
                      static_cast<uint16_t *>(out_values), out_indices, v, k, largest, dtype, workspace,
                      as_stream(stream), workspace_bytes);
}

int vkop_hip_softmax_topk_sampling(const void *in, void *out_values, int32_t *out_indices, int32_t *out_counts, int dtype,
                                   const int *shape, int ndim, int axis, int k, float scale, float top_p, void *workspace,
                                   size_t workspace_bytes, void *stream) {
    View v;
    if (int rc = check_dtype(dtype)) return rc;
    if (int rc = make_view(shape, ndim, axis, &v)) return rc;
    if (!(scale > 0.f) || !(scale < INFINITY)) return fail(VKOP_HIP_ERR_INVALID, "scale must be positive and finite");
    if (v.elems == 0 && k == 0) return VKOP_HIP_OK;
    if (int rc = check_k(v, k)) return rc;
    if (v.g.outer == 0 || v.g.inner == 0) return VKOP_HIP_OK;
    if (in == nullptr || out_values == nullptr || out_indices == nullptr)
        return fail(VKOP_HIP_ERR_INVALID, "null tensor pointer");
    if (out_counts != nullptr && v.g.inner != 1)
        return fail(VKOP_HIP_ERR_UNSUPPORTED, "the nucleus count is defined along the last axis only");
    const size_t need = selection_workspace(v, k, dtype);
    if (workspace == nullptr || workspace_bytes < need)
        return fail(VKOP_HIP_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    if ((reinterpret_cast<uintptr_t>(workspace) & (kAlign - 1)) != 0)
        return fail(VKOP_HIP_ERR_WORKSPACE, "workspace must be %zu-byte aligned", kAlign);
    const hipStream_t st = as_stream(stream);
    const ScanCfg sc = choose_scan_cfg(v, k, dtype);
    auto run = [&](auto tag) -> int {
        using T = decltype(tag);
        const T *x = static_cast<const T *>(in);
        T *values = static_cast<T *>(out_values);
        if (sc.ok && sc.g2 == 0) {
            const RowsLayout l = rows_layout(v, RowsCfg{}, BigKCfg{}, sc);
            return launch_scan<T, true>(x, values, out_indices, v, k, sc, workspace, l, st, scale, out_counts, top_p);
        }
        // short rows and a small k: one wave per row, in the scaled form
        if (const int tiny = choose_tiny_loads(v, k, dtype))
            return launch_tiny<T, true>(x, values, out_indices, v, k, tiny, st, false, true, scale, out_counts, top_p);
        // a row that one workgroup holds: its kernel in the scaled form
        if (!sc.ok) {
            const RowsCfg rc = choose_rows_cfg(v, k, dtype);
            if (rc.ok && rc.g == 1 && rows_cap(k) <= static_cast<uint32_t>(vkop::kLocalCap) && g_rows_fused.load() == 0) {
                const RowsLayout lr = rows_layout(v, rc);
                return launch_rows<T, true>(x, values, out_indices, v, k, rc, workspace, lr, st, true, scale, out_counts, top_p);
            }
        }
        // every other shape: the line kernels on the scaled elements, then the count on their sorted result
        const RowsLayout l = rows_layout(v, RowsCfg{}, BigKCfg{});
        const uint32_t lines = v.g.outer * v.g.inner;
        auto *stats = reinterpret_cast<vkop::LineStats *>(static_cast<unsigned char *>(workspace) + l.stats);
        vkop::softmax_lines_kernel<T, kLineThreads>
            <<<lines, kLineThreads, 0, st>>>(x, static_cast<T *>(nullptr), v.g, 0, 0.f, stats, scale);
        vkop::softmax_topk_lines_kernel<T, kLineThreads>
            <<<lines, kLineThreads, 0, st>>>(x, stats, values, out_indices, v.g, static_cast<uint32_t>(k), 1, scale);
        if (out_counts != nullptr)
            vkop::topp_count_kernel<T><<<lines, vkop::kWave, 0, st>>>(values, out_counts, static_cast<uint32_t>(k),
                                                                      static_cast<size_t>(k), top_p);
        return launched("softmax_lines_kernel / softmax_topk_lines_kernel / topp_count_kernel");
    };
    if (dtype == VKOP_HIP_F32) return run(float{});
    return run(uint16_t{});
}

int vkop_hip_softmax_topk_static(const void *in, void *out_values, int32_t *out_indices, int dtype, const int *shape,
                                 int ndim, int axis, int k, int largest, void *stream) {
    View v;
    if (int rc = check_dtype(dtype)) return rc;
    if (int rc = make_view(shape, ndim, axis, &v)) return rc;
    if (v.elems == 0 && k == 0) return VKOP_HIP_OK;
    if (int rc = check_k(v, k)) return rc;
    if (v.g.outer == 0 || v.g.inner == 0) return VKOP_HIP_OK;
    if (in == nullptr || out_values == nullptr || out_indices == nullptr)
        return fail(VKOP_HIP_ERR_INVALID, "null tensor pointer");
    const FusedPlan plan = plan_fused(v, k, dtype, largest, false);
    const size_t need = rows_layout(v, plan.rows, plan.big, plan.scan).total;
    if (need > static_cast<size_t>(VKOP_HIP_STATIC_SCRATCH_BYTES))
        return fail(VKOP_HIP_ERR_WORKSPACE,
                    "this tensor needs %zu bytes of scratch, the static array holds %zu: use vkop_hip_softmax_topk with a workspace",
                    need, static_cast<size_t>(VKOP_HIP_STATIC_SCRATCH_BYTES));
    void *sp = nullptr;
    int dev = 0;
    {
        // the stream belongs to the current device (each device has its own copy of the array), and the
        // array's address is looked up outside a recording (vkop_hip_init does it)
        int cur = 0;
        VKOP_HIP_TRY(hipGetDevice(&cur));
        if (stream != nullptr) {
            int sdev = cur;
            VKOP_HIP_TRY(hipStreamGetDevice(as_stream(stream), &sdev));
            if (sdev != cur)
                return fail(VKOP_HIP_ERR_INVALID, "the stream belongs to device %d, the current device is %d", sdev, cur);
        }
        if (cur >= 0 && cur < kMaxDevices && g_scratch_ptr[cur].load(std::memory_order_acquire) == nullptr) {
            hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
            VKOP_HIP_TRY(hipStreamIsCapturing(as_stream(stream), &cs));
            if (cs != hipStreamCaptureStatusNone)
                return fail(VKOP_HIP_ERR_INVALID, "the static scratch of device %d is not resolved yet and the stream is recording: "
                                                  "call vkop_hip_init(%d) before recording", cur, cur);
        }
    }
    if (int rc = resolve_static_scratch(&sp, &dev)) return rc;
    // The array keeps what the last call left.  All a call needs to find at zero
    // are the per-row arrival counters, which every call that completes returns
    // to zero; after a call that failed half way they are cleared here (a fill
    // kernel, not a memset, so that the call may be recorded).
    if (g_scratch_dirty[dev].exchange(0) != 0) {
        const size_t words = kTicketBytes / 4;
        vkop::fill_zero_kernel<<<static_cast<unsigned>((words + 255) / 256), 256, 0, as_stream(stream)>>>(
            static_cast<uint32_t *>(sp), words);
        if (int rc = launched("fill_zero_kernel")) {
            g_scratch_dirty[dev].store(1);
            return rc;
        }
    }
    int rc;
    if (dtype == VKOP_HIP_F32)
        rc = fused_impl(static_cast<const float *>(in), static_cast<float *>(nullptr), static_cast<float *>(out_values),
                        out_indices, v, k, largest, dtype, sp, as_stream(stream), static_cast<size_t>(VKOP_HIP_STATIC_SCRATCH_BYTES));
    else
        rc = fused_impl(static_cast<const uint16_t *>(in), static_cast<uint16_t *>(nullptr),
                        static_cast<uint16_t *>(out_values), out_indices, v, k, largest, dtype, sp, as_stream(stream),
                        static_cast<size_t>(VKOP_HIP_STATIC_SCRATCH_BYTES));
    if (rc != VKOP_HIP_OK) g_scratch_dirty[dev].store(1);
    return rc;
}

int vkop_hip_reduce_max(const void *in, void *out, int dtype, const int *shape, int ndim, int axis, void *stream) {
    View v;
    if (int rc = check_dtype(dtype)) return rc;
    if (int rc = make_view(shape, ndim, axis, &v)) return rc;
    if (v.g.outer == 0 || v.g.inner == 0) return VKOP_HIP_OK;
    if (v.g.n == 0) return fail(VKOP_HIP_ERR_INVALID, "max over an empty axis");
    if (in == nullptr || out == nullptr) return fail(VKOP_HIP_ERR_INVALID, "null tensor pointer");
    if (dtype == VKOP_HIP_F32)
        return reduce_max_impl(static_cast<const float *>(in), static_cast<float *>(out), v, as_stream(stream));
    return reduce_max_impl(static_cast<const uint16_t *>(in), static_cast<uint16_t *>(out), v, as_stream(stream));
}

int vkop_hip_topp_count(const void *values, int32_t *counts, int dtype, int rows, int k, int row_stride, float p, void *stream) {
    if (int rc = check_dtype(dtype)) return rc;
    if (rows < 0 || k < 1 || row_stride < k) return fail(VKOP_HIP_ERR_INVALID, "rows %d, k %d, row stride %d", rows, k, row_stride);
    if (rows == 0) return VKOP_HIP_OK;
    if (values == nullptr || counts == nullptr) return fail(VKOP_HIP_ERR_INVALID, "null tensor pointer");
    if (dtype == VKOP_HIP_F32)
        vkop::topp_count_kernel<float><<<rows, vkop::kWave, 0, as_stream(stream)>>>(static_cast<const float *>(values), counts,
                                                                                static_cast<uint32_t>(k), static_cast<size_t>(row_stride), p);
    else
        vkop::topp_count_kernel<uint16_t><<<rows, vkop::kWave, 0, as_stream(stream)>>>(static_cast<const uint16_t *>(values), counts,
                                                                                   static_cast<uint32_t>(k), static_cast<size_t>(row_stride), p);
    return launched("topp_count_kernel");
}

int vkop_hip_tune(const char *name, int value) {
    if (name == nullptr) return fail(VKOP_HIP_ERR_INVALID, "name is null");
    if (std::strcmp(name, "rows.threads") == 0) g_rows_threads = value;
    else if (std::strcmp(name, "rows.loads") == 0) g_rows_loads = value;
    else if (std::strcmp(name, "rows.chunks") == 0) g_rows_chunks = value;
    else if (std::strcmp(name, "rows.fused") == 0) g_rows_fused = value != 0;
    else if (std::strcmp(name, "rows.path") == 0) {
        if (value != 0 && value != 1) return fail(VKOP_HIP_ERR_INVALID, "rows.path must be 0 or 1");
        g_rows_path = value;
    }
    else if (std::strcmp(name, "nms.threads") == 0) {
        if (value != 0 && value != vkop::kNmsThreadsNarrow && value != vkop::kNmsThreadsWide)
            return fail(VKOP_HIP_ERR_INVALID, "nms.threads must be 0, %d or %d", vkop::kNmsThreadsNarrow, vkop::kNmsThreadsWide);
        g_nms_threads = value;
    }
    else return fail(VKOP_HIP_ERR_INVALID, "unknown tuning name '%s'", name);
    return VKOP_HIP_OK;
}

int vkop_hip_measure_path(int dtype, const int *shape, int ndim, int axis, int k) {
    View v;
    if (check_dtype(dtype) || make_view(shape, ndim, axis, &v) || k < 1) return -1;
    if (choose_tiny_loads(v, k, dtype) != 0) return 4;
    const ScanCfg sc = choose_scan_cfg(v, k, dtype);
    if (sc.ok) return sc.g2 != 0 ? 3 : 2;
    if (choose_rows_cfg(v, k, dtype).ok) return 1;
    return 0;
}

#ifdef VKOP_BENCH_HOOKS
int vkop_hip_measure_stages(int stages) {
    if (stages < 1 || stages > 3) return fail(VKOP_HIP_ERR_INVALID, "stages must be 1, 2 or 3");
    g_rows_stages = stages;
    return VKOP_HIP_OK;
}
#endif

int vkop_hip_rows_plan(int dtype, const int *shape, int ndim, int axis, int k, int *threads, int *loads,
                       int *chunks) {
    View v;
    if (int rc = check_dtype(dtype)) return rc;
    if (int rc = make_view(shape, ndim, axis, &v)) return rc;
    if (const int tiny = choose_tiny_loads(v, k, dtype)) {
        if (threads != nullptr) *threads = vkop::kWave;
        if (loads != nullptr) *loads = tiny;
        if (chunks != nullptr) *chunks = 1;
        return VKOP_HIP_OK;
    }
    const ScanCfg sc = k >= 1 ? choose_scan_cfg(v, k, dtype) : ScanCfg{};
    if (sc.ok) {
        if (threads != nullptr) *threads = vkop::kScanThreads;
        if (loads != nullptr) *loads = sc.v;
        if (chunks != nullptr) *chunks = static_cast<int>(sc.g);
        return VKOP_HIP_OK;
    }
    const RowsCfg c = k >= 1 ? choose_rows_cfg(v, k, dtype) : RowsCfg{};
    if (threads != nullptr) *threads = c.ok ? c.nt : 0;
    if (loads != nullptr) *loads = c.ok ? c.v : 0;
    if (chunks != nullptr) *chunks = c.ok ? static_cast<int>(c.g) : 0;
    return VKOP_HIP_OK;
}

size_t vkop_hip_softmax_reduce_max_workspace_bytes(int dtype, const int *shape, int ndim, int axis) {
    View v;
    if (check_dtype(dtype) || make_view(shape, ndim, axis, &v)) return 0;
    if (v.g.n <= static_cast<uint32_t>(vkop::kStridedMaxN)) return 0;
    if (v.g.inner != 1) return plan_softmax(v, dtype).workspace;
    return kTicketBytes + align_up(static_cast<size_t>(v.g.outer) * v.g.inner * sizeof(vkop::LineStats));
}

int vkop_hip_softmax_reduce_max(const void *in, void *out, int dtype, const int *shape, int ndim, int axis,
                                void *workspace, size_t workspace_bytes, void *stream) {
    View v;
    if (int rc = check_dtype(dtype)) return rc;
    if (int rc = make_view(shape, ndim, axis, &v)) return rc;
    if (v.g.outer == 0 || v.g.inner == 0) return VKOP_HIP_OK;
    if (v.g.n == 0) return fail(VKOP_HIP_ERR_INVALID, "max over an empty axis");
    if (in == nullptr || out == nullptr) return fail(VKOP_HIP_ERR_INVALID, "null tensor pointer");
    if (dtype == VKOP_HIP_F32)
        return softmax_reduce_max_impl(static_cast<const float *>(in), static_cast<float *>(out), v, workspace,
                                       workspace_bytes, as_stream(stream));
    return softmax_reduce_max_impl(static_cast<const uint16_t *>(in), static_cast<uint16_t *>(out), v, workspace,
                                   workspace_bytes, as_stream(stream));
}

size_t vkop_hip_nms_workspace_bytes(int B, int C, int N, int max_output_boxes_per_class) {
    if (B < 0 || C < 0 || N < 0) return 0;
    return nms_workspace(B, C, N, max_output_boxes_per_class);
}

int vkop_hip_nms(const void *boxes, const void *scores, int32_t *out, int out_capacity, int32_t *out_count, int dtype, int B,
                 int C, int N, int center_point_box, int max_output_boxes_per_class, float iou_threshold,
                 float score_threshold, void *workspace, size_t workspace_bytes, void *stream) {
    if (int rc = check_dtype(dtype)) return rc;
    if (B < 0 || C < 0 || N < 0 || out_capacity < 0) return fail(VKOP_HIP_ERR_INVALID, "negative extent");
    if (static_cast<uint64_t>(B) * static_cast<uint64_t>(C) >= (1ull << 31) || static_cast<uint64_t>(N) >= (1ull << 31) / 4)
        return fail(VKOP_HIP_ERR_UNSUPPORTED, "too many (batch, class) pairs or boxes");
    if (out_count == nullptr) return fail(VKOP_HIP_ERR_INVALID, "out_count is null");
    if (B == 0 || C == 0) {
        vkop::fill_zero_kernel<<<1, 64, 0, as_stream(stream)>>>(reinterpret_cast<uint32_t *>(out_count), 2);  // (no memset: capture-safe)
        return launched("fill_zero_kernel");
    }
    if (boxes == nullptr || scores == nullptr || (out == nullptr && out_capacity > 0))
        return fail(VKOP_HIP_ERR_INVALID, "null tensor pointer");
    const size_t need = nms_workspace(B, C, N, max_output_boxes_per_class);
    if (workspace == nullptr || workspace_bytes < need)
        return fail(VKOP_HIP_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    if ((reinterpret_cast<uintptr_t>(workspace) & (kAlign - 1)) != 0)
        return fail(VKOP_HIP_ERR_WORKSPACE, "workspace must be %zu-byte aligned", kAlign);
    if (dtype == VKOP_HIP_F32)
        return nms_impl(static_cast<const float *>(boxes), static_cast<const float *>(scores), out, out_capacity, out_count,
                        B, C, N, center_point_box, max_output_boxes_per_class, iou_threshold, score_threshold, workspace,
                        as_stream(stream));
    return nms_impl(static_cast<const uint16_t *>(boxes), static_cast<const uint16_t *>(scores), out, out_capacity, out_count,
                    B, C, N, center_point_box, max_output_boxes_per_class, iou_threshold, score_threshold, workspace,
                    as_stream(stream));
}

}  // extern "C"
