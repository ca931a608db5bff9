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

// ---- rows in a fixed order ------------------------------------------------------------------------------------
// The fill step leaves the entries of a transposed row in the order in which their atomics landed.  Sorting every
// row by the position of its entries in the block (t_edge; ascending positions = ascending destination rows,
// the order a stable counting sort gives) makes the transposed block, and with it the fp32 sums of every gather
// over it, the same from run to run.  Rows are short with few exceptions, so the work is dealt by length:
//   up to 8 entries     the row's lane sorts it in registers;
//   up to 64            the row's wave, one entry per lane, by shuffles;
//   longer rows         are listed by that pass and dealt out, one workgroup per row, by a second launch (hubs sit
//                       next to each other in the numbering: left to the workgroup that finds them they would queue
//                       up behind each other): up to kSortLds entries in LDS, beyond that kSortLds / 2 entries at a
//                       time and then odd-even rounds of merging neighbouring pieces (as many rounds as pieces: a
//                       hub of a whole graph taken as one block).
// Keys are distinct (positions), or -- without t_edge -- destination rows, whose ties are interchangeable.
constexpr int kSortLds = 4096;
constexpr int kSortMax = 0x7FFFFFFF;

struct SortJobs {
    TransposeJob job[8];
    int32_t* long_rows;   // pairs (job, row) of the rows left to the second launch
    int32_t* n_long;      // how many (zero when the first launch starts; may exceed long_max: then rows were dropped
    int64_t long_max;     //   from the list -- which its size, one per 65 entries, rules out)
};

__device__ __forceinline__ void sort_exchange(int& ka, int& va, int& kb, int& vb)
{
    if (kb < ka) {
        const int k = ka, v = va;
        ka = kb;
        va = vb;
        kb = k;
        vb = v;
    }
}

// bitonic sort of n (a power of two, <= kSortLds) pairs in LDS by the whole workgroup; `merge_only`: the two
// halves are sorted already (ascending), only the last merge is needed
template <int NT>
__device__ __forceinline__ void sort_lds(int* s_key, int* s_val, int n, bool merge_only)
{
    if (merge_only) {  // (a bitonic merge wants the second half descending)
        for (int i = threadIdx.x; i < n / 4; i += NT) {
            const int a = n / 2 + i, b = n - 1 - i;
            const int k = s_key[a], v = s_val[a];
            s_key[a] = s_key[b];
            s_val[a] = s_val[b];
            s_key[b] = k;
            s_val[b] = v;
        }
        __syncthreads();
    }
    for (int k = merge_only ? n : 2; k <= n; k <<= 1) {
        for (int jj = k >> 1; jj > 0; jj >>= 1) {
            for (int t = threadIdx.x; t < n / 2; t += NT) {
                const int i = 2 * t - (t & (jj - 1));  // the lower index of the t-th pair at distance jj
                const int o = i + jj;
                const bool up = (i & k) == 0 || k == n;  // (the last merge is ascending throughout)
                int ka = s_key[i], va = s_val[i], kb = s_key[o], vb = s_val[o];
                if (up ? kb < ka : ka < kb) {
                    s_key[i] = kb;
                    s_val[i] = vb;
                    s_key[o] = ka;
                    s_val[o] = va;
                }
            }
            __syncthreads();
        }
    }
}

template <int NT>
__device__ __forceinline__ void sort_load(int* s_key, int* s_val, int at, const int32_t* key, const int32_t* val, int64_t a,
                                          int64_t first, int64_t len, int n)
{
    for (int i = threadIdx.x; i < n; i += NT) {
        const int64_t e = first + i;
        s_key[at + i] = e < len ? key[a + e] : kSortMax;
        s_val[at + i] = (val != nullptr && e < len) ? val[a + e] : 0;
    }
}

template <int NT>
__device__ __forceinline__ void sort_store(const int* s_key, const int* s_val, int at, int32_t* key, int32_t* val, int64_t a,
                                           int64_t first, int64_t len, int n)
{
    for (int i = threadIdx.x; i < n; i += NT) {
        const int64_t e = first + i;
        if (e < len) {
            key[a + e] = s_key[at + i];
            if (val != nullptr) val[a + e] = s_val[at + i];
        }
    }
}

// one row of more than 64 entries, by the whole workgroup
template <int NT>
__device__ __forceinline__ void sort_row_block(int* s_key, int* s_val, int32_t* key, int32_t* val, int64_t a, int64_t len)
{
    if (len <= kSortLds) {
        int n = 128;
        while (n < len) n <<= 1;
        sort_load<NT>(s_key, s_val, 0, key, val, a, 0, len, n);
        __syncthreads();
        sort_lds<NT>(s_key, s_val, n, false);
        sort_store<NT>(s_key, s_val, 0, key, val, a, 0, len, n);
        __syncthreads();
        return;
    }
    constexpr int kPiece = kSortLds / 2;
    const int64_t pieces = (len + kPiece - 1) / kPiece;
    for (int64_t p = 0; p < pieces; ++p) {
        sort_load<NT>(s_key, s_val, 0, key, val, a, p * kPiece, len, kPiece);
        __syncthreads();
        sort_lds<NT>(s_key, s_val, kPiece, false);
        sort_store<NT>(s_key, s_val, 0, key, val, a, p * kPiece, len, kPiece);
        __syncthreads();
    }
    // odd-even rounds: neighbouring pieces are merged and split again, smaller half first; the padding of the last
    // piece sorts to its end, which is never stored
    for (int64_t round = 0; round < pieces; ++round) {
        for (int64_t p = round & 1; p + 1 < pieces; p += 2) {
            sort_load<NT>(s_key, s_val, 0, key, val, a, p * kPiece, len, kSortLds);
            __syncthreads();
            sort_lds<NT>(s_key, s_val, kSortLds, true);
            sort_store<NT>(s_key, s_val, 0, key, val, a, p * kPiece, len, kSortLds);
            __syncthreads();
        }
    }
}

template <int NT>
__device__ __forceinline__ void tjob_sort_rows(const SortJobs& jobs, int job_index)
{
    const TransposeJob& j = jobs.job[job_index];
    if (j.t_ptr == nullptr) return;
    int32_t* key = j.t_edge ? j.t_edge : j.t_dst;
    int32_t* val = j.t_edge ? j.t_dst : nullptr;
    const int64_t n_cols = actual_count(j.cols_max, j.d_n_cols);
    const int64_t n_edges = actual_count(j.edges_max, j.d_n_edges);
    const int lane = lane_id();
    // Neighbouring rows go to different waves (row r to wave r mod the number of waves): the long rows of a block
    // sit next to each other -- hubs are met early and numbered early -- and a wave takes its rows of 9..64 entries
    // one after the other.
    const int64_t n_waves = (int64_t)gridDim.x * (NT / kWave);
    const int64_t wave = (int64_t)blockIdx.x * (NT / kWave) + threadIdx.x / kWave;
    for (int64_t first = 0; first < n_cols; first += n_waves * kWave) {  // (uniform over the launch)
        const int64_t c = first + wave + n_waves * lane;
        int64_t a = 0, b = 0;
        if (c < n_cols) {
            a = j.t_ptr[c];
            b = j.t_ptr[c + 1];
            if (b > n_edges) b = n_edges;
            if (a > b) a = b;
        }
        const int64_t len = b - a;
        if (len >= 2 && len <= 8) {  // in registers: a sorting network for eight
            int k[8], v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                k[i] = i < len ? key[a + i] : kSortMax;
                v[i] = (val != nullptr && i < len) ? val[a + i] : 0;
            }
#define FGL_CX(x, y) sort_exchange(k[x], v[x], k[y], v[y])
            FGL_CX(0, 1); FGL_CX(2, 3); FGL_CX(4, 5); FGL_CX(6, 7);
            FGL_CX(0, 2); FGL_CX(1, 3); FGL_CX(4, 6); FGL_CX(5, 7);
            FGL_CX(1, 2); FGL_CX(5, 6); FGL_CX(0, 4); FGL_CX(3, 7);
            FGL_CX(1, 5); FGL_CX(2, 6);
            FGL_CX(1, 4); FGL_CX(3, 6);
            FGL_CX(2, 4); FGL_CX(3, 5);
            FGL_CX(3, 4);
#undef FGL_CX
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (i < len) {
                    key[a + i] = k[i];
                    if (val != nullptr) val[a + i] = v[i];
                }
        }
        // rows of 9..64 entries: the wave takes them one after the other, an entry per lane
        unsigned long long todo = __ballot(len > 8 && len <= kWave);
        while (todo != 0) {
            const int r = __ffsll((long long)todo) - 1;
            todo &= todo - 1;
            const int64_t ra = __shfl(a, r, kWave);
            const int rl = (int)__shfl(len, r, kWave);
            int kk = lane < rl ? key[ra + lane] : kSortMax;
            int vv = (val != nullptr && lane < rl) ? val[ra + lane] : 0;
#pragma unroll
            for (int k2 = 2; k2 <= kWave; k2 <<= 1) {
#pragma unroll
                for (int jj = k2 >> 1; jj > 0; jj >>= 1) {
                    const int ok = __shfl_xor(kk, jj, kWave);
                    const int ov = __shfl_xor(vv, jj, kWave);
                    const bool up = (lane & k2) == 0;
                    const bool lower = (lane & jj) == 0;
                    const bool take = (lower == up) ? (ok < kk) : (ok > kk);
                    if (take) {
                        kk = ok;
                        vv = ov;
                    }
                }
            }
            if (lane < rl) {
                key[ra + lane] = kk;
                if (val != nullptr) val[ra + lane] = vv;
            }
        }
        // longer rows: listed for the second launch
        if (len > kWave) {
            const int64_t at = atomicAdd(jobs.n_long, 1);
            if (at < jobs.long_max) {
                jobs.long_rows[2 * at] = job_index;
                jobs.long_rows[2 * at + 1] = (int32_t)c;
            }
        }
    }
}

template <int NT>
__device__ __forceinline__ void tjob_sort_long_rows(const SortJobs& jobs, int* s_key, int* s_val)
{
    int64_t n = *jobs.n_long;
    if (n > jobs.long_max) n = jobs.long_max;
    for (int64_t q = blockIdx.x; q < n; q += gridDim.x) {
        const TransposeJob& j = jobs.job[jobs.long_rows[2 * q] & 7];
        const int64_t c = jobs.long_rows[2 * q + 1];
        const int64_t n_edges = actual_count(j.edges_max, j.d_n_edges);
        int64_t a = j.t_ptr[c], b = j.t_ptr[c + 1];
        if (b > n_edges) b = n_edges;
        if (a > b) a = b;
        sort_row_block<NT>(s_key, s_val, j.t_edge ? j.t_edge : j.t_dst, j.t_edge ? j.t_dst : nullptr, a, b - a);
    }
}

#endif  // __HIPCC__

}  // namespace fgl
