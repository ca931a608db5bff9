// The transposed form of a sampled block, built inside the all-hops sampling call (fgl_sample_blocks) without a
// launch of its own wherever another launch of the call can carry the work.  (It is what turns the reference's
// atomic-scatter backward kernels, aggregate_acc_kernel.cu:467-517,554-596, into gathers; the reference builds
// nothing of the kind and the per-hop loop it runs instead is FusedMapSampler.py:72-107.)
//
// A counting sort by source node in five steps, each a grid-stride device function that any kernel of the
// right stream position can call on entry, before its own work:
//   zero        the per-column counters                                  (hop h's sampling kernel)
//   rank        k = counter[col]++ for every edge, as its local source id becomes known
//                                                                         (hop h's id-map passes: take_rank)
//   tile sums   per 2048 counters                                        (hop h+1's sampling kernel)
//   scan        counters -> offsets in place, the transposed row pointer, the longest row
//                                                                         (hop h+1's first id-map pass)
//   fill        t_dst[offset[col] + k] = row, t_edge[...] = edge         (hop h+1's second id-map pass)
// The last hop of a call has no hop after it: its three closing steps are launches of their own.
// A carried step runs in workgroups of its own, appended to the carrying launch's grid (side_blocks of them,
// the last of the grid, see side_block): in front of the launch's own work it would lengthen the chain of
// memory latencies that a small hop's launch is (measured: 20 us per mini-batch, what the separate launches cost).
// Sizes that exist only on the device are read from the call's count array; every array is sized by the
// host-side bound.  `split` > 1 gives every column that many counters (entry e uses number e % split): returning
// atomics on one address complete one after the other, and a hub column of a large hop is mentioned thousands
// of times.
#pragma once
#include "fgl_common.hpp"
#include "fgl_kernels.hpp"

namespace fgl {

constexpr int kTjobTile = 2048;  // counters per scan tile

#if defined(__HIPCC__)

// rank of edge e within the transposed row of its local source id (-1: the edge has none)
__device__ __forceinline__ void take_rank(const TransposeRank& r, int64_t e, int32_t local)
{
    if (r.rank == nullptr) return;
    int32_t k = -1;
    if (local >= 0 && (int64_t)local < r.cols_max) k = atomicAdd(&r.cnt[(int64_t)local * r.split + (int)(e & (r.split - 1))], 1);
    r.rank[e] = k;
}

// This workgroup's index among the job's side workgroups -- the last side_blocks of the grid but side_first --
// or -1 if it is none of them.
__device__ __forceinline__ int side_block(const TransposeJob& j)
{
    const int64_t sb = (int64_t)gridDim.x - 1 - (int64_t)blockIdx.x - j.side_first;
    return (sb >= 0 && sb < j.side_blocks) ? (int)sb : -1;
}

__device__ __forceinline__ int64_t tjob_entries(const TransposeJob& j)
{
    return actual_count(j.cols_max, j.d_n_cols) * j.split + 1;  // one more: the total
}

template <int NT>
__device__ __forceinline__ void tjob_zero(const TransposeJob& j)
{
    if (j.cnt == nullptr) return;
    const int sb = side_block(j);
    if (sb < 0) return;
    const int64_t n = j.cols_max * j.split + 1;
    const int64_t stride = (int64_t)j.side_blocks * NT;
    for (int64_t i = (int64_t)sb * NT + threadIdx.x; i < n; i += stride) j.cnt[i] = 0;
}

template <int NT>
__device__ __forceinline__ void tjob_tile_sums(const TransposeJob& j)
{
    if (j.cnt == nullptr) return;
    __shared__ int smem[NT / kWave + 1];
    const int sb = side_block(j);
    if (sb < 0) return;  // (uniform over the workgroup: barriers below)
    const int64_t n = tjob_entries(j);
    const int64_t n_tiles = (n + kTjobTile - 1) / kTjobTile;
    for (int64_t tile = sb; tile < n_tiles; tile += j.side_blocks) {
        int v[kTjobTile / NT];
#pragma unroll
        for (int q = 0; q < kTjobTile / NT; ++q) {  // (all of the lane's loads in flight together)
            const int64_t i = tile * kTjobTile + (int64_t)q * NT + threadIdx.x;
            v[q] = (i < n - 1) ? j.cnt[i] : 0;  // (the last entry is the slot of the total: not a counter)
        }
        int s = 0;
#pragma unroll
        for (int q = 0; q < kTjobTile / NT; ++q) s += v[q];
        const int total = block_sum_of_lanes<NT>(s, smem);
        if (threadIdx.x == 0) j.tile_sums[tile] = total;
    }
}

// counters -> exclusive prefix sums in place; t_ptr[c] = the prefix of column c's first counter; the longest
// row (if it holds more than FGL_SHORT_ROW_ENTRIES entries) into *longest, which starts at zero.
// A lane scans kItems consecutive counters: with split counters those are exactly one column's.
template <int NT>
__device__ __forceinline__ void tjob_scan(const TransposeJob& j)
{
    if (j.cnt == nullptr) return;
    constexpr int kItems = kTjobTile / NT;
    static_assert(kItems == 8 || kItems == 32, "tiles are dealt 8 (256 lanes) or 32 (64 lanes) counters per lane");
    __shared__ int smem[NT / kWave + 1];
    const int sb = side_block(j);
    if (sb < 0) return;  // (uniform over the workgroup: barriers below)
    const int64_t n = tjob_entries(j);
    const int64_t n_tiles = (n + kTjobTile - 1) / kTjobTile;
    const int split = j.split;
    for (int64_t tile = sb; tile < n_tiles; tile += j.side_blocks) {
        const int64_t base = tile * kTjobTile + (int64_t)threadIdx.x * kItems;
        int v[kItems];
        int s = 0;
#pragma unroll
        for (int q = 0; q < kItems; ++q) {
            v[q] = (base + q < n - 1) ? j.cnt[base + q] : 0;
            s += v[q];
        }
        const int before = block_sum_before<NT>(j.tile_sums, tile, smem);
        int total;
        int run = block_exclusive_scan<NT>(s, smem, &total) + before;
        int longest = 0, len = 0;
#pragma unroll
        for (int q = 0; q < kItems; ++q) {
            const int64_t i = base + q;
            if (i < n) {
                if (split > 1 || j.cnt != j.t_ptr) j.cnt[i] = run;
                if (split == 1) {
                    j.t_ptr[i] = run;
                    longest = v[q] > longest ? v[q] : longest;
                } else {
                    // (split is a power of two that divides kItems: a column's counters never straddle lanes)
                    if ((i & (split - 1)) == 0) {
                        j.t_ptr[i / split] = run;
                        len = 0;
                    }
                    len += v[q];
                    longest = len > longest ? len : longest;
                }
            }
            run += v[q];
        }
        if (j.longest != nullptr && longest > FGL_SHORT_ROW_ENTRIES) atomicMax(j.longest, longest);
    }
}

// sixteen lanes per row of the block: its entries are read coalesced and scattered in parallel
template <int NT>
__device__ __forceinline__ void tjob_fill(const TransposeJob& j)
{
    if (j.cnt == nullptr) return;
    constexpr int kLanes = 16;
    const int sb = side_block(j);
    if (sb < 0) return;
    const int64_t n_rows = actual_count(j.rows_max, j.d_n_rows);
    const int64_t n_edges = actual_count(j.edges_max, j.d_n_edges);
    const int lane = (int)threadIdx.x % kLanes;
    const int split = j.split;
    const int64_t stride = (int64_t)j.side_blocks * (NT / kLanes);
    for (int64_t r = (int64_t)sb * (NT / kLanes) + (int)threadIdx.x / kLanes; r < n_rows; r += stride) {
        const int64_t a = j.block_ptr[r];
        int64_t b = j.block_ptr[r + 1];
        if (b > n_edges) b = n_edges;
        for (int64_t e = a + lane; e < b; e += kLanes) {
            const int32_t k = j.rank[e];
            if (k >= 0) {
                const int64_t pos = (int64_t)j.cnt[(int64_t)j.src_local[e] * split + (int)(e & (split - 1))] + k;
                if (pos < j.edges_max) {
                    j.t_dst[pos] = (int32_t)r;
                    if (j.t_edge) j.t_edge[pos] = (int32_t)e;
                }
            }
        }
    }
}

#endif  // __HIPCC__

}  // namespace fgl
