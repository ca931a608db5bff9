// Transposes of several blocks at once.  The blocks of a mini-batch that a backward pass needs in transposed
// form are small (all but the outermost hop), and each transpose is five launches -- clear, count, two for the
// scan, fill -- of a few microseconds apiece, far below what fills the chip: here the same five launches serve
// every block of the batch, each workgroup finding its block from a short table of workgroup ranges.
// (Stands in, like fgl_block_transpose, for what lets the reference's atomic scatter backward kernels,
// aggregate_acc_kernel.cu:467-517,554-596, run as gathers.)  Exact sizes only, unordered lists within a
// transposed row, blocks below 2^20 entries and 8 M columns; the caller falls back to fgl_block_transpose otherwise.
#include "fgl_common.hpp"
#include "fgl_kernels.hpp"

namespace fgl {

struct TBlock {
    const int32_t* indptr;
    const int32_t* indices;
    int64_t n_rows, n_cols, n_edges;
    int32_t* t_indptr;
    int32_t* t_indices;
    int32_t* t_edge;   // may be null
    int32_t* longest;  // may be null
    int32_t* rank;
    int32_t* tile_sums;
};

struct TBatch {
    int n;
    TBlock b[FGL_TRANSPOSE_BATCH_MAX];
    unsigned first_wg[FGL_TRANSPOSE_BATCH_MAX + 1];  // of the launch at hand: block i owns workgroups [first_wg[i], first_wg[i+1])
};

__device__ __forceinline__ int which_block(const TBatch& t, unsigned wg, unsigned* local)
{
    int i = 0;
#pragma unroll
    for (int k = 1; k < FGL_TRANSPOSE_BATCH_MAX; ++k)
        if (k < t.n && wg >= t.first_wg[k]) i = k;
    *local = wg - t.first_wg[i];
    return i;
}

constexpr int kTbScanItems = 8;
constexpr int kTbScanTile = kBlock * kTbScanItems;

__global__ __launch_bounds__(kBlock) void tbatch_clear_kernel(const TBatch t)
{
    unsigned local;
    const TBlock& b = t.b[which_block(t, blockIdx.x, &local)];
    const int64_t i = (int64_t)local * kBlock + threadIdx.x;
    if (i <= b.n_cols) b.t_indptr[i] = 0;
    if (i == 0 && b.longest) *b.longest = 0;
}

__global__ __launch_bounds__(kBlock) void tbatch_count_kernel(const TBatch t)
{
    unsigned local;
    const TBlock& b = t.b[which_block(t, blockIdx.x, &local)];
    const int64_t e = (int64_t)local * kBlock + threadIdx.x;
    if (e >= b.n_edges) return;
    const int32_t c = b.indices[e];
    int32_t k = -1;
    if (c >= 0 && (int64_t)c < b.n_cols) k = atomicAdd(&b.t_indptr[c], 1);
    b.rank[e] = k;
    // only the few entries that land far down a long column report its length
    if (b.longest != nullptr && k >= FGL_SHORT_ROW_ENTRIES) atomicMax(b.longest, k + 1);
}

__global__ __launch_bounds__(kBlock) void tbatch_tile_sums_kernel(const TBatch t)
{
    __shared__ int smem[kBlock / kWave + 1];
    unsigned local;
    const TBlock& b = t.b[which_block(t, blockIdx.x, &local)];
    const int64_t base = (int64_t)local * kTbScanTile + (int64_t)threadIdx.x * kTbScanItems;
    int s = 0;
#pragma unroll
    for (int j = 0; j < kTbScanItems; ++j)
        if (base + j < b.n_cols) s += b.t_indptr[base + j];
    int total;
    (void)block_exclusive_scan<kBlock>(s, smem, &total);
    if (threadIdx.x == 0) b.tile_sums[local] = total;
}

// in place: t_indptr[0..n_cols] = exclusive sums of the counts (entry n_cols = the total)
__global__ __launch_bounds__(kBlock) void tbatch_scan_apply_kernel(const TBatch t)
{
    __shared__ int smem[kBlock / kWave + 1];
    unsigned local;
    const TBlock& b = t.b[which_block(t, blockIdx.x, &local)];
    const int64_t base = (int64_t)local * kTbScanTile + (int64_t)threadIdx.x * kTbScanItems;
    int v[kTbScanItems];
    int s = 0;
#pragma unroll
    for (int j = 0; j < kTbScanItems; ++j) {
        v[j] = (base + j < b.n_cols) ? b.t_indptr[base + j] : 0;
        s += v[j];
    }
    const int before = block_sum_before<kBlock>(b.tile_sums, local, smem);
    int total;
    int run = block_exclusive_scan<kBlock>(s, smem, &total) + before;
#pragma unroll
    for (int j = 0; j < kTbScanItems; ++j) {
        if (base + j <= b.n_cols) b.t_indptr[base + j] = run;
        run += v[j];
    }
}

// sixteen lanes per row: the row's entries are read coalesced and scattered in parallel
__global__ __launch_bounds__(kBlock) void tbatch_fill_kernel(const TBatch t)
{
    constexpr int kLanes = 16;
    unsigned local;
    const TBlock& b = t.b[which_block(t, blockIdx.x, &local)];
    const int64_t r = (int64_t)local * (kBlock / kLanes) + (int)threadIdx.x / kLanes;
    if (r >= b.n_rows) return;
    const int lane = (int)threadIdx.x % kLanes;
    const int64_t first = b.indptr[r];
    int64_t last = b.indptr[r + 1];
    if (last > b.n_edges) last = b.n_edges;
    for (int64_t e = first + lane; e < last; e += kLanes) {
        const int32_t k = b.rank[e];
        if (k >= 0) {
            const int64_t pos = (int64_t)b.t_indptr[b.indices[e]] + k;
            b.t_indices[pos] = (int32_t)r;
            if (b.t_edge) b.t_edge[pos] = (int32_t)e;
        }
    }
}

static size_t tbatch_workspace_bytes(int n_blocks, const int64_t* n_cols, const int64_t* n_edges, TBatch* t, void* ws)
{
    Carver c(ws);
    for (int i = 0; i < n_blocks; ++i) {
        int32_t* rank = c.take<int32_t>((size_t)n_edges[i]);
        int32_t* sums = c.take<int32_t>((size_t)ceil_div(n_cols[i] + 1, kTbScanTile));
        if (t) {
            t->b[i].rank = rank;
            t->b[i].tile_sums = sums;
        }
    }
    return c.used();
}

}  // namespace fgl

using namespace fgl;

FGL_EXPORT size_t fgl_block_transpose_batch_workspace_bytes(int n_blocks, const int64_t* n_cols, const int64_t* n_edges)
{
    if (n_blocks < 1 || n_blocks > FGL_TRANSPOSE_BATCH_MAX || !n_cols || !n_edges) return 0;
    for (int i = 0; i < n_blocks; ++i)
        if (n_cols[i] < 0 || n_edges[i] < 0) return 0;
    return tbatch_workspace_bytes(n_blocks, n_cols, n_edges, nullptr, nullptr);
}

FGL_EXPORT int fgl_block_transpose_batch(int n_blocks, const int32_t* const* d_indptr, const int32_t* const* d_indices,
                                         const int64_t* n_rows, const int64_t* n_cols, const int64_t* n_edges,
                                         int32_t* const* d_t_indptr, int32_t* const* d_t_indices, int32_t* const* d_t_edge,
                                         int32_t* const* d_t_longest_row, void* d_ws, size_t ws_bytes, void* stream)
{
    FGL_REQUIRE(n_blocks >= 1 && n_blocks <= FGL_TRANSPOSE_BATCH_MAX, "block_transpose_batch: %d blocks outside [1, %d]", n_blocks,
                FGL_TRANSPOSE_BATCH_MAX);
    FGL_REQUIRE(d_indptr && d_indices && n_rows && n_cols && n_edges && d_t_indptr && d_t_indices, "block_transpose_batch: null argument");
    TBatch t;
    memset(&t, 0, sizeof(t));
    t.n = n_blocks;
    for (int i = 0; i < n_blocks; ++i) {
        FGL_REQUIRE(n_rows[i] >= 0 && n_cols[i] >= 0 && n_edges[i] >= 0, "block_transpose_batch: negative size (block %d)", i);
        FGL_REQUIRE(n_edges[i] < FGL_TRANSPOSE_BATCH_MAX_EDGES && n_cols[i] < FGL_TRANSPOSE_BATCH_MAX_COLS,
                    "block_transpose_batch: block %d (%lld entries, %lld columns) is too large: use fgl_block_transpose", i,
                    (long long)n_edges[i], (long long)n_cols[i]);
        FGL_REQUIRE(d_t_indptr[i] != nullptr, "block_transpose_batch: null output (block %d)", i);
        FGL_REQUIRE(n_edges[i] == 0 || (d_indptr[i] && d_indices[i] && d_t_indices[i]), "block_transpose_batch: null pointer (block %d)", i);
        t.b[i] = TBlock{d_indptr[i], d_indices[i], n_rows[i], n_cols[i], n_rows[i] > 0 ? n_edges[i] : 0, d_t_indptr[i], d_t_indices[i],
                        d_t_edge ? d_t_edge[i] : nullptr, d_t_longest_row ? d_t_longest_row[i] : nullptr, nullptr, nullptr};
    }
    const size_t need = tbatch_workspace_bytes(n_blocks, n_cols, n_edges, nullptr, nullptr);
    if (d_ws == nullptr || ws_bytes < need) {
        set_error("block_transpose_batch: workspace too small (%zu < %zu)", ws_bytes, need);
        return FGL_ERR_WORKSPACE;
    }
    tbatch_workspace_bytes(n_blocks, n_cols, n_edges, &t, d_ws);
    hipStream_t s = as_stream(stream);
    // workgroups per block of each launch; a launch is skipped when no block has work for it
    auto ranges = [&](auto wgs_of) -> unsigned {
        unsigned total = 0;
        for (int i = 0; i < n_blocks; ++i) {
            t.first_wg[i] = total;
            total += (unsigned)wgs_of(t.b[i]);
        }
        for (int i = n_blocks; i <= FGL_TRANSPOSE_BATCH_MAX; ++i) t.first_wg[i] = total;
        return total;
    };
    unsigned grid = ranges([](const TBlock& b) { return ceil_div(b.n_cols + 1, kBlock); });
    hipLaunchKernelGGL(tbatch_clear_kernel, dim3(grid), dim3(kBlock), 0, s, t);
    FGL_CHECK_LAUNCH("tbatch_clear_kernel");
    grid = ranges([](const TBlock& b) { return ceil_div(b.n_edges, kBlock); });
    if (grid > 0) {
        hipLaunchKernelGGL(tbatch_count_kernel, dim3(grid), dim3(kBlock), 0, s, t);
        FGL_CHECK_LAUNCH("tbatch_count_kernel");
    }
    grid = ranges([](const TBlock& b) { return ceil_div(b.n_cols + 1, kTbScanTile); });
    hipLaunchKernelGGL(tbatch_tile_sums_kernel, dim3(grid), dim3(kBlock), 0, s, t);
    FGL_CHECK_LAUNCH("tbatch_tile_sums_kernel");
    hipLaunchKernelGGL(tbatch_scan_apply_kernel, dim3(grid), dim3(kBlock), 0, s, t);
    FGL_CHECK_LAUNCH("tbatch_scan_apply_kernel");
    grid = ranges([](const TBlock& b) { return b.n_edges > 0 ? ceil_div(b.n_rows, kBlock / 16) : 0; });
    if (grid > 0) {
        hipLaunchKernelGGL(tbatch_fill_kernel, dim3(grid), dim3(kBlock), 0, s, t);
        FGL_CHECK_LAUNCH("tbatch_fill_kernel");
    }
    return FGL_OK;
}
