// Device-wide exclusive sum, degree histogram, and the library's error plumbing.
//
// exclusive sum: three launches, no spin-waits -- (1) per-tile sums, (2) one workgroup
// turns the tile sums into tile prefixes, (3) per-tile local scan + prefix.  A tile is
// 256 threads x 8 consecutive items (32 contiguous bytes per lane, 2 KiB per wave).
#include <stdarg.h>

#include <chrono>

#include "fgl_common.hpp"
#include "fgl_kernels.hpp"

namespace fgl {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

constexpr int kScanItems = 8;
constexpr int kScanTile = kBlock * kScanItems;

__global__ __launch_bounds__(kBlock) void scan_tile_sums_kernel(const int32_t* __restrict__ in, int64_t n_max,
                                                                const int32_t* __restrict__ d_n,
                                                                int32_t* __restrict__ tile_sums)
{
    __shared__ int smem[kBlock / kWave + 1];
    const int64_t n = actual_count(n_max, d_n);
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
    int s = 0;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j)
        if (base + j < n) s += in[base + j];
    int total;
    (void)block_exclusive_scan<kBlock>(s, smem, &total);
    if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// One workgroup: tile_prefix[t] = sum of tile_sums[0..t).  The grand total goes to
// *total_a and *total_b and to at_count_base[actual count] (each optional).  With
// tile_items > 0 only the tiles that the actual count occupies are read.
__global__ __launch_bounds__(1024) void scan_tile_prefix_kernel(const int32_t* __restrict__ tile_sums, int n_tiles,
                                                                int32_t* __restrict__ tile_prefix,
                                                                int32_t* __restrict__ total_a,
                                                                int32_t* __restrict__ total_b,
                                                                int32_t* __restrict__ at_count_base, int64_t n_max,
                                                                const int32_t* __restrict__ d_n, int tile_items,
                                                                int32_t* __restrict__ readback,
                                                                const uint32_t* __restrict__ d_status)
{
    __shared__ int smem[1024 / kWave + 1];
    if (tile_items > 0) {
        const int64_t used = (actual_count(n_max, d_n) + tile_items - 1) / tile_items;
        if (used < n_tiles) n_tiles = (int)used;
    }
    int carry = 0;
    for (int start = 0; start < n_tiles; start += 1024) {
        const int t = start + (int)threadIdx.x;
        const int v = t < n_tiles ? tile_sums[t] : 0;
        int total;
        const int ex = block_exclusive_scan<1024>(v, smem, &total);
        if (t < n_tiles) tile_prefix[t] = carry + ex;
        carry += total;
    }
    if (threadIdx.x == 0) {
        if (total_a) *total_a = carry;
        if (total_b) *total_b = carry;
        if (at_count_base) at_count_base[actual_count(n_max, d_n)] = carry;
        if (readback) {  // {total, status word as it stands}: see fgl_sample_node's d_readback
            readback[0] = carry;
            readback[1] = d_status ? (int32_t)*d_status : 0;
        }
    }
}

int launch_tile_prefix(const int32_t* tile_sums, int n_tiles, int32_t* tile_prefix, int32_t* total_a,
                       int32_t* total_b, int32_t* at_count_base, int64_t n_max, const int32_t* d_n, int tile_items,
                       hipStream_t stream, int32_t* readback, const uint32_t* d_status)
{
    hipLaunchKernelGGL(scan_tile_prefix_kernel, dim3(1), dim3(1024), 0, stream, tile_sums, n_tiles, tile_prefix,
                       total_a, total_b, at_count_base, n_max, d_n, tile_items, readback, d_status);
    FGL_CHECK_LAUNCH("scan_tile_prefix_kernel");
    return FGL_OK;
}

// `in` and `out` may be the same buffer: every lane reads its items before the barrier and
// writes only its own positions after it (hence no __restrict__ on them).
// tile_prefix == nullptr: no prefix launch ran; the workgroup sums the earlier tiles' sums itself
// (tile 0 needs none), and the lane that holds index n also stores the grand total in *total_extra.
__global__ __launch_bounds__(kBlock) void scan_apply_kernel(const int32_t* in, int64_t n_max,
                                                            const int32_t* __restrict__ d_n,
                                                            const int32_t* __restrict__ tile_sums,
                                                            const int32_t* __restrict__ tile_prefix, int32_t* out,
                                                            int32_t* __restrict__ total_extra)
{
    __shared__ int smem[kBlock / kWave + 1];
    const int64_t n = actual_count(n_max, d_n);
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
    int v[kScanItems];
    int s = 0;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
        v[j] = (base + j < n) ? in[base + j] : 0;
        s += v[j];
    }
    const int before = tile_prefix ? tile_prefix[blockIdx.x] : block_sum_before<kBlock>(tile_sums, blockIdx.x, smem);
    int total;
    int run = block_exclusive_scan<kBlock>(s, smem, &total) + before;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
        if (base + j <= n) out[base + j] = run;  // index n receives the grand total
        if (base + j == n && tile_prefix == nullptr && total_extra) *total_extra = run;
        run += v[j];
    }
}

// Up to this many tiles the apply pass derives its tile offsets itself (no prefix launch).
constexpr int64_t kScanSelfPrefixTiles = 4096;

size_t scan_workspace_bytes(int64_t n_max)
{
    const int64_t tiles = ceil_div(n_max + 1, kScanTile);
    Carver c(nullptr);
    c.take<int32_t>((size_t)tiles);
    c.take<int32_t>((size_t)tiles);
    return c.used();
}

int launch_exclusive_sum(const int32_t* d_in, int64_t n_max, const int32_t* d_n, int32_t* d_out,
                         int32_t* d_total_extra, void* d_ws, size_t ws_bytes, hipStream_t stream)
{
    // n_max + 1 outputs: the tile holding index n must exist even when n is a multiple of the tile.
    const int64_t tiles = ceil_div(n_max + 1, kScanTile);
    if (tiles > 0x7FFFFFFF) {
        set_error("exclusive_sum: too many items (%lld)", (long long)n_max);
        return FGL_ERR_UNSUPPORTED;
    }
    if (ws_bytes < scan_workspace_bytes(n_max) || d_ws == nullptr) {
        set_error("exclusive_sum: workspace too small (%zu < %zu)", ws_bytes, scan_workspace_bytes(n_max));
        return FGL_ERR_WORKSPACE;
    }
    Carver c(d_ws);
    int32_t* sums = c.take<int32_t>((size_t)tiles);
    int32_t* prefix = c.take<int32_t>((size_t)tiles);
    // one tile: its offset is zero, the apply pass alone does the job; few tiles: the apply pass sums the
    // tile sums before its own; many: a single-workgroup launch turns the sums into offsets first
    if (tiles > 1) {
        hipLaunchKernelGGL(scan_tile_sums_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream, d_in, n_max, d_n, sums);
        FGL_CHECK_LAUNCH("scan_tile_sums_kernel");
    }
    if (tiles > kScanSelfPrefixTiles) {
        int rc = launch_tile_prefix(sums, (int)tiles, prefix, d_total_extra, nullptr, nullptr, 0, nullptr, 0, stream);
        if (rc != FGL_OK) return rc;
    } else {
        prefix = nullptr;
    }
    hipLaunchKernelGGL(scan_apply_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream, d_in, n_max, d_n, sums, prefix,
                       d_out, d_total_extra);
    FGL_CHECK_LAUNCH("scan_apply_kernel");
    return FGL_OK;
}

// ---- fill / histogram -----------------------------------------------------------
__global__ __launch_bounds__(kBlock) void fill_u32_kernel(uint32_t* __restrict__ p, int64_t n, uint32_t value)
{
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) p[i] = value;
}

int launch_fill_u32(uint32_t* p, int64_t n, uint32_t value, hipStream_t stream)
{
    if (n <= 0) return FGL_OK;
    int64_t blocks = ceil_div(n, (int64_t)kBlock * 4);
    if (blocks > 65536) blocks = 65536;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, p, n, value);
    FGL_CHECK_LAUNCH("fill_u32_kernel");
    return FGL_OK;
}

__global__ __launch_bounds__(kBlock) void cal_deg_kernel(const int32_t* __restrict__ ids, int64_t n_max,
                                                         const int32_t* __restrict__ d_n, int32_t* __restrict__ deg,
                                                         int64_t n_nodes)
{
    const int64_t n = actual_count(n_max, d_n);
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int32_t id = ids[i];
    if (id >= 0 && (int64_t)id < n_nodes) atomicAdd(&deg[id], 1);
}

}  // namespace fgl

using namespace fgl;

FGL_EXPORT int fgl_abi_version(void) { return FGL_ABI_VERSION; }
FGL_EXPORT const char* fgl_last_error(void) { return g_err; }

// Host side of a d_readback: the caller stored `pending` into every word before it enqueued the call; the launch
// that knows the sizes overwrites them.  Looking at the words themselves returns as soon as they have landed --
// which is before that launch has finished, and without the wake-up of a stream wait.  Bounded: past spin_limit_us
// the stream is waited for instead, and words that are still pending then are an error.
FGL_EXPORT int fgl_wait_words(const int32_t* h_words, int n_words, int32_t pending, void* stream, int64_t spin_limit_us)
{
    FGL_REQUIRE(h_words != nullptr && n_words >= 1, "wait_words: nothing to wait for");
    const volatile int32_t* w = h_words;
    auto all_there = [&]() {
        for (int i = 0; i < n_words; ++i)
            if (w[i] == pending) return false;
        return true;
    };
    if (spin_limit_us > 0) {
        const auto t0 = std::chrono::steady_clock::now();
        for (;;) {
            for (int k = 0; k < 256; ++k) {
                if (all_there()) return FGL_OK;
                __builtin_ia32_pause();
            }
            if (std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - t0).count() > spin_limit_us) break;
        }
    }
    FGL_REQUIRE(hipStreamSynchronize(as_stream(stream)) == hipSuccess, "wait_words: waiting for the stream failed");
    FGL_REQUIRE(all_there(), "wait_words: the stream is idle and the words were not written");
    return FGL_OK;
}

FGL_EXPORT size_t fgl_exclusive_sum_workspace_bytes(int64_t n_max) { return scan_workspace_bytes(n_max < 0 ? 0 : n_max); }

FGL_EXPORT int fgl_exclusive_sum_i32(const int32_t* d_in, int64_t n_max, const int32_t* d_n, int32_t* d_out,
                                     void* d_ws, size_t ws_bytes, void* stream)
{
    FGL_REQUIRE(n_max >= 0, "exclusive_sum: negative length");
    FGL_REQUIRE(d_out != nullptr, "exclusive_sum: null output");
    FGL_REQUIRE(d_in != nullptr || n_max == 0, "exclusive_sum: null input");
    return launch_exclusive_sum(d_in, n_max, d_n, d_out, nullptr, d_ws, ws_bytes, as_stream(stream));
}

FGL_EXPORT int fgl_cal_deg(const int32_t* d_ids, int64_t n_ids_max, const int32_t* d_n_ids, int32_t* d_deg,
                           int64_t n_nodes, void* stream)
{
    FGL_REQUIRE(n_ids_max >= 0 && n_nodes >= 0, "cal_deg: negative size");
    FGL_REQUIRE(d_deg != nullptr || n_nodes == 0, "cal_deg: null output");
    FGL_REQUIRE(d_ids != nullptr || n_ids_max == 0, "cal_deg: null input");
    int rc = launch_fill_u32(reinterpret_cast<uint32_t*>(d_deg), n_nodes, 0u, as_stream(stream));
    if (rc != FGL_OK) return rc;
    if (n_ids_max == 0) return FGL_OK;
    const int64_t blocks = ceil_div(n_ids_max, kBlock);
    FGL_REQUIRE(blocks <= 0x7FFFFFFF, "cal_deg: too many ids");
    hipLaunchKernelGGL(cal_deg_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, as_stream(stream), d_ids, n_ids_max,
                       d_n_ids, d_deg, n_nodes);
    FGL_CHECK_LAUNCH("cal_deg_kernel");
    return FGL_OK;
}
