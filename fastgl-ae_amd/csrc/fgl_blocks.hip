// All hops of one mini-batch in a single enqueue (stands in for the layer loop of the
// reference's FusedMapSampler.sample_blocks, FusedMapSampler.py:63-109, which synchronises
// with the host at least four times per hop and rebuilds its hash table per hop,
// id_map.cu:408-409,454).  Here the table and the numbering persist across hops -- hop h's
// unique list is hop h+1's seed list with the same local ids -- node and edge counts stay on
// the device, and each launch is sized by a host-side bound and reads the actual count.
//
// Also: the seeded R-MAT key generator used to build the synthetic benchmark graphs.
#include "fgl_common.hpp"
#include "fgl_kernels.hpp"
#include "fgl_table.hpp"
#include "fgl_transpose_job.hpp"

namespace fgl {

// Start of a mini-batch in one launch (the table is empty -- left so by the call before, or by a fill launch):
//   - counts: node count of hop 0 = the seed count, the other counts and the status word zero;
//   - the per-tile edge counts of the later hops zero (they are accumulated with atomics as hops run);
//   - every seed: its id into the unique list and the table (local id = position), the start and length of
//     its row in the graph for the first hop's sampling kernel, and the first hop's per-tile edge counts.
// The status word is being initialised by this launch, so nothing here reports through it: a seed outside the
// graph or one that found the table full gets a negative row start, which the first hop's sampling kernel
// (the next launch) reports.
template <int TS>
__global__ __launch_bounds__(TS) void blocks_prepare_kernel(TableRef t, const void* __restrict__ indptr, int is64,
                                                            int64_t n_nodes, const int32_t* __restrict__ seeds,
                                                            int64_t n_seeds, int fanout, int32_t* __restrict__ uniq,
                                                            int64_t* __restrict__ row_start, int32_t* __restrict__ deg_out,
                                                            int32_t* __restrict__ tile_sums, int32_t* __restrict__ later_sums,
                                                            int64_t n_later_sums, int32_t* __restrict__ counts, int n_counts,
                                                            int32_t* __restrict__ sort_n_long)
{
    __shared__ int smem[TS / kWave + 1];
    const int64_t first = (int64_t)blockIdx.x * TS + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * TS;
    for (int64_t i = first; i < n_counts; i += stride) counts[i] = (i == 0) ? (int32_t)n_seeds : 0;
    if (first < 4) sort_n_long[first] = 0;  // (the counters of the row sort that may close the call)
    for (int64_t i = first; i < n_later_sums; i += stride) later_sums[i] = 0;
    const int64_t n_tiles = (n_seeds + TS - 1) / TS;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t i = tile * TS + threadIdx.x;
        int k = 0;
        if (i < n_seeds) {
            const int32_t s = seeds[i];
            if (uniq != seeds) uniq[i] = s;
            int64_t a = kRowBadId, deg = 0;
            if (s >= 0 && (int64_t)s < n_nodes) {
                int64_t b;
                if (is64) {
                    const int64_t* p = static_cast<const int64_t*>(indptr);
                    a = p[s];
                    b = p[s + 1];
                } else {
                    const int32_t* p = static_cast<const int32_t*>(indptr);
                    a = p[s];
                    b = p[s + 1];
                }
                // (the table probe goes out before the two offsets are looked at: one wait for both)
                uint32_t seen;
                const bool full = find_or_insert(t, (uint32_t)s, (uint32_t)i, &seen) == kEmpty;  // a repeated seed keeps its first position
                deg = b - a;
                if (deg < 0) deg = 0;
                if (deg > 0x7FFFFFFF) deg = 0x7FFFFFFF;
                if (full) {
                    a = kRowTableFull;
                    deg = 0;
                }
            }
            row_start[i] = a;
            deg_out[i] = (int32_t)deg;
            k = deg < fanout ? (int)deg : fanout;
        }
        int total;
        (void)block_exclusive_scan<TS>(k, smem, &total);
        if (threadIdx.x == 0) tile_sums[tile] = total;
    }
}

struct BlocksPlan {
    int64_t cap_dst[32];
    int64_t cap_edges[32];
    int64_t cap_uniq;
    int64_t table_slots;
    size_t ws_bytes;
    // layout of the workspace: what persists over the hops of a mini-batch, then the id-map's per-hop scratch
    int64_t n_positions;       // row start / degree entries: one per node that is a seed of some hop
    int64_t tile_first[33];    // per-tile edge counts of hop h start at entry tile_first[h]; [n_hops] = their total
    int64_t max_tiles;
    int64_t max_edges;
    size_t idmap_bytes;
    // transposed blocks built inside the call (bit h of transpose_hops: hop h's)
    uint32_t transpose_hops;
    int64_t cap_src[32];  // max source nodes (= columns) of hop h
    int split[32];        // counters per column while hop h's transposed rows are being counted
    int64_t sort_long_max;  // rows of more than 64 entries that the transposed blocks can hold between them
};

struct BlocksScratch {
    int64_t* row_start;
    int32_t* deg;
    int32_t* tile_sums;
    int32_t* tile_prefix;
    uint8_t* lowered;  // one byte per edge of a hop: cleared by the hop's sampling kernel, used by its id-map passes
    char* idmap_ws;
    // per hop whose transposed block is wanted (null otherwise)
    int32_t* t_rank[32];
    int32_t* t_tile_sums[32];
    int32_t* t_split_cnt[32];  // split counters (hops that count with several counters per column)
    int32_t* sort_long_rows;   // rows left to the second launch of the row sort: pairs (job, row)
    int32_t* sort_n_long;      // their number, one counter per group of eight transposed blocks (zeroed by the first launch of a call)
};

static size_t carve_scratch(const BlocksPlan& p, void* ws, BlocksScratch* out)
{
    Carver c(ws);
    int64_t* row_start = c.take<int64_t>((size_t)p.n_positions);
    int32_t* deg = c.take<int32_t>((size_t)p.n_positions);
    int32_t* tile_sums = c.take<int32_t>((size_t)p.tile_first[32]);
    int32_t* tile_prefix = c.take<int32_t>((size_t)p.max_tiles);
    uint8_t* lowered = c.take<uint8_t>((size_t)p.max_edges);
    char* idmap_ws = c.take<char>(p.idmap_bytes);
    int32_t* sort_long_rows = c.take<int32_t>((size_t)(2 * p.sort_long_max));
    int32_t* sort_n_long = c.take<int32_t>(4);
    if (out) {
        memset(out, 0, sizeof(*out));
        out->sort_long_rows = sort_long_rows;
        out->sort_n_long = sort_n_long;
        out->row_start = row_start;
        out->deg = deg;
        out->tile_sums = tile_sums;
        out->tile_prefix = tile_prefix;
        out->lowered = lowered;
        out->idmap_ws = idmap_ws;
    }
    for (int h = 0; h < 32; ++h) {
        if (!((p.transpose_hops >> h) & 1u)) continue;
        const int64_t counters = p.cap_src[h] * p.split[h] + 1;
        int32_t* rank = c.take<int32_t>((size_t)p.cap_edges[h]);
        int32_t* sums = c.take<int32_t>((size_t)ceil_div(counters, kTjobTile));
        int32_t* cnt = p.split[h] > 1 ? c.take<int32_t>((size_t)counters) : nullptr;
        if (out) {
            out->t_rank[h] = rank;
            out->t_tile_sums[h] = sums;
            out->t_split_cnt[h] = cnt;
        }
    }
    return c.used();
}

// node_capacity (optional, n_hops+1 entries): the caller's own limit on the number of nodes before
// hop h (entry n_hops: after the last hop).  The plan is the worst case clipped to it.
// Hops of at least this many edges (by the plan's bound) count their transposed rows with kTransposeSplit
// counters per column: a hub column of such a hop is mentioned thousands of times.
#ifndef FGL_TRANSPOSE_SPLIT_MIN_EDGES
#define FGL_TRANSPOSE_SPLIT_MIN_EDGES (1 << 20)
#endif
constexpr int64_t kTransposeSplitMinEdges = FGL_TRANSPOSE_SPLIT_MIN_EDGES;
constexpr int kTransposeSplit = 8;

static int make_plan(int64_t n_nodes, int64_t n_seeds, const int32_t* fanouts, int n_hops, const int64_t* node_capacity,
                     uint32_t transpose_hops, BlocksPlan* p)
{
    FGL_REQUIRE(n_hops >= 1 && n_hops <= 32, "sample_blocks: %d hops outside [1, 32]", n_hops);
    FGL_REQUIRE(n_nodes >= 0 && n_seeds >= 0 && fanouts != nullptr, "sample_blocks: bad sizes");
    int64_t cur = n_seeds;
    size_t idmap_ws = 0;
    int64_t tiles_total = 0, max_tiles = 1, max_edges = 1;
    for (int h = 0; h < n_hops; ++h) {
        FGL_REQUIRE(fanouts[h] >= 1 && fanouts[h] <= FGL_MAX_FANOUT, "sample_blocks: fanout %d outside [1, %d]", fanouts[h], FGL_MAX_FANOUT);
        if (node_capacity) {
            FGL_REQUIRE(node_capacity[h] >= n_seeds, "sample_blocks: node_capacity[%d] = %lld is below the seed count", h, (long long)node_capacity[h]);
            // (a hop's nodes are a prefix of the next hop's: the bounds must not shrink, the workspace layout relies on it)
            FGL_REQUIRE(h == 0 || node_capacity[h] >= p->cap_dst[h - 1], "sample_blocks: node_capacity[%d] is below an earlier entry", h);
            if (cur > node_capacity[h]) cur = node_capacity[h];
        }
        p->cap_dst[h] = cur;
        p->cap_edges[h] = cur * fanouts[h];
        FGL_REQUIRE(p->cap_edges[h] <= 0x7FFFFFFF, "sample_blocks: hop %d may produce %lld edges, beyond int32 offsets", h, (long long)p->cap_edges[h]);
        if (p->cap_edges[h] > max_edges) max_edges = p->cap_edges[h];
        const size_t w = idmap_map_src_workspace_bytes(p->cap_edges[h]);
        if (w > idmap_ws) idmap_ws = w;
        const int64_t tiles = sample_tile_count(p->cap_dst[h], fanouts[h]);
        p->tile_first[h] = tiles_total;
        tiles_total += tiles;
        if (tiles > max_tiles) max_tiles = tiles;
        // every node is numbered once; repeated seeds are the only way past n_nodes
        int64_t next = cur + p->cap_edges[h];
        if (next > n_nodes + n_seeds) next = n_nodes + n_seeds;
        cur = next;
    }
    for (int h = n_hops; h <= 32; ++h) p->tile_first[h] = tiles_total;
    if (node_capacity) {
        FGL_REQUIRE(node_capacity[n_hops] >= p->cap_dst[n_hops - 1], "sample_blocks: node_capacity[%d] is below an earlier entry", n_hops);
        if (cur > node_capacity[n_hops]) cur = node_capacity[n_hops];
    }
    p->cap_uniq = cur;
    FGL_REQUIRE(n_hops == 32 || (transpose_hops >> n_hops) == 0, "sample_blocks: transpose_hops names a hop beyond the %d of the call", n_hops);
    p->transpose_hops = transpose_hops;
    for (int h = 0; h < 32; ++h) {
        p->cap_src[h] = h < n_hops ? (h + 1 < n_hops ? p->cap_dst[h + 1] : cur) : 0;
        p->split[h] = (h < n_hops && p->cap_edges[h] >= kTransposeSplitMinEdges) ? kTransposeSplit : 1;
        if (h < n_hops && ((transpose_hops >> h) & 1u))
            FGL_REQUIRE(p->cap_src[h] * p->split[h] + 1 <= 0x7FFFFFFF, "sample_blocks: hop %d has too many columns to transpose", h);
    }
    p->sort_long_max = 0;
    for (int h = 0; h < n_hops; ++h)
        if ((transpose_hops >> h) & 1u) p->sort_long_max += p->cap_edges[h] / (kWave + 1) + 1;
    p->table_slots = fgl_idmap_slots(cur);
    FGL_REQUIRE(p->table_slots <= ((int64_t)1 << 31), "sample_blocks: table too large");
    p->n_positions = p->cap_dst[n_hops - 1] > 0 ? p->cap_dst[n_hops - 1] : 1;
    p->max_tiles = max_tiles;
    p->max_edges = max_edges;
    p->idmap_bytes = idmap_ws;
    p->ws_bytes = carve_scratch(*p, nullptr, nullptr);
    return FGL_OK;
}

// The three closing steps of a transposed block as launches of their own: for the last hop of a call, which has no
// later hop whose launches could carry them.
// The last of them also hands the call's counts to the host, if asked: everything in them is final by then.
template <int STEP>
__global__ __launch_bounds__(kBlock) void transpose_step_kernel(const TransposeJob j, int32_t* __restrict__ readback,
                                                                const int32_t* __restrict__ counts, int n_counts)
{
    if (STEP == 0) tjob_tile_sums<kBlock>(j);
    if (STEP == 1) tjob_scan<kBlock>(j);
    if (STEP == 2) {
        if (readback != nullptr && blockIdx.x == 0 && (int)threadIdx.x < n_counts) readback[threadIdx.x] = counts[threadIdx.x];
        tjob_fill<kBlock>(j);
    }
}

// Every row of the call's transposed blocks into ascending order of its entries' positions in the block (one launch
// for all of them: blockIdx.y names the block).
__global__ __launch_bounds__(kBlock) void transpose_sort_rows_kernel(const SortJobs jobs)
{
    tjob_sort_rows<kBlock>(jobs, (int)blockIdx.y);
}

// ... and the rows of more than 64 entries that it listed, a workgroup per row
__global__ __launch_bounds__(kBlock) void transpose_sort_long_rows_kernel(const SortJobs jobs)
{
    __shared__ int s_key[kSortLds];
    __shared__ int s_val[kSortLds];
    tjob_sort_long_rows<kBlock>(jobs, s_key, s_val);
}

// ---- R-MAT -------------------------------------------------------------------------
constexpr uint32_t kCutA = 0x91EB851Eu;  // floor(0.57 * 2^32)
constexpr uint32_t kCutB = 0xC28F5C28u;  // floor(0.76 * 2^32)
constexpr uint32_t kCutC = 0xF3333333u;  // floor(0.95 * 2^32)

__global__ __launch_bounds__(kBlock) void rmat_keys_kernel(int64_t first_edge, int64_t n_edges, int scale, int64_t n_nodes,
                                                           uint32_t seed_lo, uint32_t seed_hi, int64_t* __restrict__ keys)
{
    const int64_t x = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (x >= n_edges) return;
    const uint64_t e = (uint64_t)(first_edge + x);
    uint64_t u = 0, v = 0;
    uint32_t o[4] = {0u, 0u, 0u, 0u};
    for (int lvl = 0; lvl < scale; ++lvl) {
        if ((lvl & 3) == 0) philox4x32_10((uint32_t)e, (uint32_t)(e >> 32), (uint32_t)(lvl >> 2), 0x524D4154u, seed_lo, seed_hi, o);
        const uint32_t r = o[lvl & 3];
        const uint32_t ub = r >= kCutB;
        const uint32_t vb = (r >= kCutA && r < kCutB) || r >= kCutC;
        u = (u << 1) | ub;
        v = (v << 1) | vb;
    }
    int64_t k0 = INT64_MAX, k1 = INT64_MAX;
    if (u != v && u < (uint64_t)n_nodes && v < (uint64_t)n_nodes) {
        k0 = (int64_t)((v << 32) | u);
        k1 = (int64_t)((u << 32) | v);
    }
    keys[2 * x] = k0;
    keys[2 * x + 1] = k1;
}

}  // namespace fgl

using namespace fgl;

FGL_EXPORT int fgl_sample_blocks_plan(int64_t n_nodes, int64_t n_seeds, const int32_t* fanouts, int n_hops,
                                      const int64_t* node_capacity, uint32_t transpose_hops, int64_t* cap_dst,
                                      int64_t* cap_edges, int64_t* cap_uniq, int64_t* table_slots, size_t* ws_bytes)
{
    BlocksPlan p;
    int rc = make_plan(n_nodes, n_seeds, fanouts, n_hops, node_capacity, transpose_hops, &p);
    if (rc != FGL_OK) return rc;
    for (int h = 0; h < n_hops; ++h) {
        if (cap_dst) cap_dst[h] = p.cap_dst[h];
        if (cap_edges) cap_edges[h] = p.cap_edges[h];
    }
    if (cap_uniq) *cap_uniq = p.cap_uniq;
    if (table_slots) *table_slots = p.table_slots;
    if (ws_bytes) *ws_bytes = p.ws_bytes;
    return FGL_OK;
}

FGL_EXPORT int fgl_sample_blocks(const void* d_indptr, int indptr_is64, const int32_t* d_indices, int64_t n_nodes,
                                 const int32_t* d_seeds, int64_t n_seeds, const int32_t* fanouts, int n_hops,
                                 const int64_t* node_capacity, uint64_t rng_seed, uint32_t stream_base,
                                 const uint32_t* d_stream_offset, int idmap_flags, void* d_table,
                                 int64_t table_slots,
                                 int32_t* d_uniq, int64_t uniq_capacity, int32_t* const* block_ptr,
                                 int32_t* const* src_local, int32_t* const* src_global, int32_t* const* t_ptr,
                                 int32_t* const* t_dst, int32_t* const* t_edge, int32_t* d_counts, int32_t* d_readback,
                                 void* d_ws, size_t ws_bytes, void* stream)
{
    // the hops whose transposed block is wanted: those with a row-pointer output
    uint32_t transpose_hops = 0;
    if (t_ptr != nullptr && n_hops >= 1 && n_hops <= 32)
        for (int h = 0; h < n_hops; ++h)
            if (t_ptr[h] != nullptr) transpose_hops |= 1u << h;
    BlocksPlan p;
    int rc = make_plan(n_nodes, n_seeds, fanouts, n_hops, node_capacity, transpose_hops, &p);
    if (rc != FGL_OK) return rc;
    for (int h = 0; h < n_hops; ++h)
        if ((transpose_hops >> h) & 1u)
            FGL_REQUIRE(t_dst != nullptr && t_dst[h] != nullptr, "sample_blocks: hop %d has a transposed row pointer but no entry array", h);
    const int order = idmap_flags & FGL_IDMAP_ARRIVAL;
    const bool table_is_empty = (idmap_flags & FGL_BLOCKS_TABLE_EMPTY) != 0;
    const bool leave_empty = (idmap_flags & FGL_BLOCKS_LEAVE_TABLE_EMPTY) != 0;
    const bool sort_rows = (idmap_flags & FGL_BLOCKS_SORT_TRANSPOSED) != 0;
    FGL_REQUIRE((idmap_flags & ~(FGL_IDMAP_ARRIVAL | FGL_BLOCKS_TABLE_EMPTY | FGL_BLOCKS_LEAVE_TABLE_EMPTY | FGL_BLOCKS_SORT_TRANSPOSED)) == 0,
                "sample_blocks: unknown flags %d", idmap_flags);
    FGL_REQUIRE(d_indptr && d_indices && d_table && d_uniq && block_ptr && src_local && d_counts, "sample_blocks: null pointer");
    FGL_REQUIRE(n_seeds == 0 || d_seeds != nullptr, "sample_blocks: null seeds");
    // A table smaller than the plan's worst case is accepted (batches are usually far below the
    // bound and a small table stays cache-resident): the seeds must fit, and a batch that
    // outgrows the table is reported through FGL_STATUS_TABLE_FULL, never by a fault.
    FGL_REQUIRE(table_slots >= fgl_idmap_slots(n_seeds), "sample_blocks: table has %lld slots, the seeds alone need %lld", (long long)table_slots, (long long)fgl_idmap_slots(n_seeds));
    FGL_REQUIRE(uniq_capacity >= p.cap_uniq, "sample_blocks: unique list holds %lld, plan needs %lld", (long long)uniq_capacity, (long long)p.cap_uniq);
    if (d_ws == nullptr || ws_bytes < p.ws_bytes) {
        set_error("sample_blocks: workspace too small (%zu < %zu)", ws_bytes, p.ws_bytes);
        return FGL_ERR_WORKSPACE;
    }
    for (int h = 0; h < n_hops; ++h) FGL_REQUIRE(block_ptr[h] && src_local[h], "sample_blocks: null output for hop %d", h);

    hipStream_t s = as_stream(stream);
    const int n_counts = 3 * n_hops + 2;
    uint32_t* d_status = reinterpret_cast<uint32_t*>(d_counts + 2 * n_hops + 1);
    FGL_REQUIRE(valid_slots(table_slots), "sample_blocks: slot count %lld is not a power of two in [64, 2^31]", (long long)table_slots);
    FGL_REQUIRE(((uintptr_t)d_table & 15) == 0 && ((uintptr_t)d_ws & 15) == 0, "sample_blocks: table and workspace must be 16-byte aligned");
    BlocksScratch ws;
    carve_scratch(p, d_ws, &ws);
    const TableRef t = make_ref(d_table, table_slots);

    // launch 1 (only if the caller does not vouch for an empty table): every slot to empty
    if (!table_is_empty) {
        rc = launch_fill_u32(t.words, table_slots * 2, kEmpty, s);
        if (rc != FGL_OK) return rc;
    }
    TransposeJob job_before;
    memset(&job_before, 0, sizeof(job_before));
    auto make_job = [&](int h) {
        TransposeJob j;
        memset(&j, 0, sizeof(j));
        if (!((transpose_hops >> h) & 1u)) return j;
        j.split = p.split[h];
        j.cnt = j.split > 1 ? ws.t_split_cnt[h] : t_ptr[h];
        j.tile_sums = ws.t_tile_sums[h];
        j.rank = ws.t_rank[h];
        j.t_ptr = t_ptr[h];
        j.t_dst = t_dst[h];
        j.t_edge = t_edge ? t_edge[h] : nullptr;
        j.longest = d_counts + 2 * n_hops + 2 + h;
        j.block_ptr = block_ptr[h];
        j.src_local = src_local[h];
        j.d_n_rows = d_counts + h;
        j.d_n_cols = d_counts + h + 1;
        j.d_n_edges = d_counts + n_hops + 1 + h;
        j.rows_max = p.cap_dst[h];
        j.cols_max = p.cap_src[h];
        j.edges_max = p.cap_edges[h];
        return j;
    };
    // launch 2: counts, the later hops' tile sums, the seeds into the table, the first hop's rows and tile sums
    {
        const int ts0 = sample_tile_seeds(fanouts[0], n_seeds);
        const int64_t tiles0 = sample_tile_count(n_seeds, fanouts[0]);
        const int64_t n_later = p.tile_first[n_hops] - p.tile_first[1];
        int64_t blocks = tiles0;
        if (blocks < ceil_div(n_later, ts0)) blocks = ceil_div(n_later, ts0);
        if (blocks > 8192) blocks = 8192;
        if (blocks < 1) blocks = 1;
        if (ts0 == 256)
            hipLaunchKernelGGL(blocks_prepare_kernel<256>, dim3((unsigned)blocks), dim3(256), 0, s, t, d_indptr, indptr_is64, n_nodes,
                               d_seeds, n_seeds, fanouts[0], d_uniq, ws.row_start, ws.deg, ws.tile_sums,
                               ws.tile_sums + p.tile_first[1], n_later, d_counts, n_counts, ws.sort_n_long);
        else
            hipLaunchKernelGGL(blocks_prepare_kernel<64>, dim3((unsigned)blocks), dim3(64), 0, s, t, d_indptr, indptr_is64, n_nodes,
                               d_seeds, n_seeds, fanouts[0], d_uniq, ws.row_start, ws.deg, ws.tile_sums,
                               ws.tile_sums + p.tile_first[1], n_later, d_counts, n_counts, ws.sort_n_long);
        FGL_CHECK_LAUNCH("blocks_prepare_kernel");
    }

    for (int h = 0; h < n_hops; ++h) {
        const bool last = h == n_hops - 1;
        const int32_t* hop_seeds = (h == 0) ? d_seeds : d_uniq;
        int32_t* d_n_dst = d_counts + h;
        int32_t* d_n_edges = d_counts + n_hops + 1 + h;
        int32_t* sampled = (src_global && src_global[h]) ? src_global[h] : src_local[h];
        // what this hop's passes prepare for the next hop's sampling: the hop's seeds are the next hop's first
        // seeds (their row starts and degrees are in place already; the sampling kernel adds their share of the
        // next tile sums), the nodes it numbers are the rest (the id-map's numbering pass fills in theirs)
        NextHop next{};
        if (!last) {
            next.indptr = d_indptr;
            next.is64 = indptr_is64;
            next.n_nodes = n_nodes;
            next.row_start = ws.row_start;
            next.deg = ws.deg;
            next.tile_sums = ws.tile_sums + p.tile_first[h + 1];
            next.fanout = fanouts[h + 1];
            next.tile_seeds = sample_tile_seeds(fanouts[h + 1], p.cap_dst[h + 1]);
        }
        // transposed blocks: this hop's (if wanted) has its counters cleared by the sampling launch and its ranks
        // taken by the id-map passes; the one of the hop before is closed by this hop's first three launches
        TransposeSteps steps;
        steps.before = job_before;
        steps.zero = make_job(h);
        rc = launch_sample_edges(d_indices, hop_seeds, p.cap_dst[h], d_n_dst, fanouts[h], ws.row_start, ws.deg,
                                 ws.tile_sums + p.tile_first[h], ws.tile_prefix, rng_seed, stream_base + (uint32_t)h, sampled,
                                 nullptr, block_ptr[h], d_n_edges, d_status, s, d_stream_offset, last ? nullptr : &next,
                                 ws.lowered, &steps);
        if (rc != FGL_OK) return rc;
        // the node count this hop may grow to: what the next hop's buffers (or the unique list) hold;
        // growing past it is reported as FGL_STATUS_UNIQ_OVERFLOW and the count is clamped
        const int64_t grow_to = (!last && p.cap_dst[h + 1] < p.cap_uniq) ? p.cap_dst[h + 1] : p.cap_uniq;
        // the host's copy of the counts: written by whichever launch makes the last of them final -- the last hop's
        // node total, or (if the last hop's transposed block is wanted) its longest row, below
        const bool counts_final_here = last && steps.zero.cnt == nullptr;
        rc = launch_idmap_map_src(d_table, table_slots, sampled, src_local[h], p.cap_edges[h], d_n_edges, 0, d_n_dst,
                                  d_counts + h + 1, d_uniq, grow_to, order | (last ? FGL_IDMAP_FINAL : 0), d_status,
                                  ws.idmap_ws, p.idmap_bytes, s, /*counter_is_zeroed=*/true, last ? nullptr : &next,
                                  /*leave_table_empty=*/last && leave_empty, ws.lowered, &steps.zero, &job_before, nullptr,
                                  counts_final_here ? d_readback : nullptr, d_counts, n_counts);
        if (rc != FGL_OK) return rc;
        job_before = steps.zero;
    }
    if (job_before.cnt != nullptr) {  // the last hop's transposed block: no later launch to carry its closing steps
        job_before.side_first = 0;
        job_before.side_blocks = side_blocks_for(job_before.cols_max * job_before.split + 1, kTjobTile, 8192);
        hipLaunchKernelGGL(transpose_step_kernel<0>, dim3((unsigned)job_before.side_blocks), dim3(kBlock), 0, s, job_before,
                           nullptr, nullptr, 0);
        hipLaunchKernelGGL(transpose_step_kernel<1>, dim3((unsigned)job_before.side_blocks), dim3(kBlock), 0, s, job_before,
                           nullptr, nullptr, 0);
        job_before.side_blocks = side_blocks_for(job_before.rows_max, kBlock / 16, 16384);
        hipLaunchKernelGGL(transpose_step_kernel<2>, dim3((unsigned)job_before.side_blocks), dim3(kBlock), 0, s, job_before,
                           d_readback, d_counts, n_counts);
        FGL_CHECK_LAUNCH("transpose_step_kernel");
    }
    if (sort_rows && transpose_hops != 0) {
        // rows of the transposed blocks in a fixed order: two more launches per eight blocks -- every row of up to
        // 64 entries, then the longer ones that the first launch has listed
        SortJobs jobs;
        memset(&jobs, 0, sizeof(jobs));
        jobs.long_rows = ws.sort_long_rows;
        jobs.long_max = p.sort_long_max;
        int n_jobs = 0, round = 0;
        int64_t most_cols = 1;
        for (int h = 0; h <= n_hops; ++h) {
            if (h < n_hops && ((transpose_hops >> h) & 1u)) {
                jobs.job[n_jobs++] = make_job(h);
                if (p.cap_src[h] > most_cols) most_cols = p.cap_src[h];
            }
            if (n_jobs == 8 || (h == n_hops && n_jobs > 0)) {
                jobs.n_long = ws.sort_n_long + round++;
                const int64_t gx = ceil_div(most_cols, kBlock) < 4096 ? ceil_div(most_cols, kBlock) : 4096;
                hipLaunchKernelGGL(transpose_sort_rows_kernel, dim3((unsigned)gx, (unsigned)n_jobs), dim3(kBlock), 0, s, jobs);
                const int64_t gl = p.sort_long_max < 2048 ? p.sort_long_max : 2048;
                hipLaunchKernelGGL(transpose_sort_long_rows_kernel, dim3((unsigned)(gl > 0 ? gl : 1)), dim3(kBlock), 0, s, jobs);
                FGL_CHECK_LAUNCH("transpose_sort_rows_kernel");
                n_jobs = 0;
                most_cols = 1;
                memset(jobs.job, 0, sizeof(jobs.job));
            }
        }
    }
    return FGL_OK;
}

FGL_EXPORT int fgl_rmat_keys(int64_t first_edge, int64_t n_edges, int scale, int64_t n_nodes, uint64_t seed,
                             int64_t* d_keys, void* stream)
{
    FGL_REQUIRE(first_edge >= 0 && n_edges >= 0 && n_nodes >= 0, "rmat_keys: negative size");
    FGL_REQUIRE(scale >= 1 && scale <= 31, "rmat_keys: scale %d outside [1, 31]", scale);
    if (n_edges == 0) return FGL_OK;
    FGL_REQUIRE(d_keys != nullptr, "rmat_keys: null output");
    const int64_t blocks = ceil_div(n_edges, kBlock);
    FGL_REQUIRE(blocks <= 0x7FFFFFFF, "rmat_keys: too many edges in one call");
    hipLaunchKernelGGL(rmat_keys_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, as_stream(stream), first_edge, n_edges,
                       scale, n_nodes, (uint32_t)seed, (uint32_t)(seed >> 32), d_keys);
    FGL_CHECK_LAUNCH("rmat_keys_kernel");
    return FGL_OK;
}
