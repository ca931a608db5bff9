// Internal launchers shared between the translation units of libfastgl_hip.
#pragma once
#include "fgl_common.hpp"

namespace fgl {

// exclusive sum (fgl_scan.hip).  d_out gets n+1 entries; d_total_extra (optional) the total.
size_t scan_workspace_bytes(int64_t n_max);
int launch_exclusive_sum(const int32_t* d_in, int64_t n_max, const int32_t* d_n, int32_t* d_out,
                         int32_t* d_total_extra, void* d_ws, size_t ws_bytes, hipStream_t stream);
// single-workgroup scan of per-tile sums; the total is written to *total_a, *total_b and
// at_count_base[actual count of (n_max, d_n)] (each optional); tile_items > 0 restricts the
// scan to the tiles the actual count occupies
int launch_tile_prefix(const int32_t* tile_sums, int n_tiles, int32_t* tile_prefix, int32_t* total_a,
                       int32_t* total_b, int32_t* at_count_base, int64_t n_max, const int32_t* d_n, int tile_items,
                       hipStream_t stream, int32_t* readback = nullptr, const uint32_t* d_status = nullptr);
int launch_fill_u32(uint32_t* p, int64_t n, uint32_t value, hipStream_t stream);

// Row start of a node whose id lies outside the graph / whose insert found the table full: how a launch that
// must not touch the status word hands the error to the next one that reads the entry.
constexpr int64_t kRowBadId = -1;
constexpr int64_t kRowTableFull = -2;

// What a pass over a hop's nodes prepares for the sampling of the next hop: row start and degree of every node
// at its position in the unique list, and the per-tile sums of min(fanout, degree) that place the tiles' output.
struct NextHop {
    const void* indptr;
    int is64;
    int64_t n_nodes;
    int64_t* row_start;
    int32_t* deg;
    int32_t* tile_sums;  // zeroed by the caller; [position / tile_seeds] += min(fanout, degree)
    int fanout;
    int tile_seeds;
};

// A block's transposed form under construction inside the all-hops call (fgl_transpose_job.hpp).  cnt == nullptr:
// no such work.
struct TransposeJob {
    int32_t* cnt;        // split * cols_max + 1 counters, then their prefix sums; split == 1: the same array as t_ptr
    int32_t* tile_sums;  // one per 2048 counters
    int32_t* rank;       // per edge: its position within its transposed row
    int32_t* t_ptr;      // cols_max + 1
    int32_t* t_dst;      // edges_max
    int32_t* t_edge;     // edges_max, or null
    int32_t* longest;    // one int, zero before the scan step: the longest transposed row if beyond FGL_SHORT_ROW_ENTRIES
    const int32_t* block_ptr;
    const int32_t* src_local;
    const int32_t* d_n_rows;
    const int32_t* d_n_cols;
    const int32_t* d_n_edges;
    int64_t rows_max, cols_max, edges_max;
    int split;
    // which workgroups of the launch at hand work on the step it carries: side_blocks of them, the last of the
    // grid but side_first (set per launch by the launcher, which appends them to the grid)
    int side_blocks, side_first;
};
// Side workgroups for a step over n_items, items_per_block at a time: never more than the work needs, and few
// enough that they are an appendix to the launch that carries them.
inline int side_blocks_for(int64_t n_items, int64_t items_per_block, int cap = 8192)
{
    int64_t b = (n_items + items_per_block - 1) / items_per_block;
    if (b < 1) b = 1;
    return (int)(b < cap ? b : cap);
}
// what the id-map passes need of it: where an edge takes its rank
struct TransposeRank {
    int32_t* cnt;
    int32_t* rank;  // null: no transposed block is being built
    int64_t cols_max;
    int split;
};
__host__ __device__ inline TransposeRank rank_of(const TransposeJob* j)
{
    return j && j->cnt ? TransposeRank{j->cnt, j->rank, j->cols_max, j->split} : TransposeRank{nullptr, nullptr, 0, 1};
}
// what one launch carries along for the transposed blocks: steps of the hop before (tile sums / scan / fill, by the
// launch's place in the hop) and the zeroing of this hop's counters (sampling launch only)
struct TransposeSteps {
    TransposeJob before;
    TransposeJob zero;
};

// neighbour sampling (fgl_sample.hip)
int sample_tile_seeds(int fanout, int64_t n_seeds_max);
int64_t sample_tile_count(int64_t n_seeds_max, int fanout);
size_t sample_workspace_bytes(int64_t n_seeds_max, int fanout);
// the second half of launch_sample, for callers that hold row starts, degrees and tile sums already
int launch_sample_edges(const int32_t* d_indices, const int32_t* d_seeds, int64_t n_seeds_max, const int32_t* d_n_seeds,
                        int fanout, const int64_t* row_start, const int32_t* deg, const int32_t* tile_sums,
                        int32_t* tile_prefix, uint64_t rng_seed, uint32_t stream_id, int32_t* d_src_out,
                        int32_t* d_dst_out, int32_t* d_block_ptr, int32_t* d_n_edges_out, uint32_t* d_status,
                        hipStream_t stream, const uint32_t* d_stream_add, const NextHop* next,
                        uint8_t* d_zero_per_edge = nullptr,   // (optional) one byte per output edge, cleared along with the writes
                        const TransposeSteps* steps = nullptr,   // (optional) zero this hop's counters, tile sums of the hop before
                        int32_t* d_readback = nullptr);          // (optional) {edge count, status word} once both are final; may be host memory
int launch_sample(const void* d_indptr, int indptr_is64, const int32_t* d_indices, int64_t n_nodes,
                  const int32_t* d_seeds, int64_t n_seeds_max, const int32_t* d_n_seeds, int fanout,
                  uint64_t rng_seed, uint32_t stream_id, int32_t* d_src_out, int32_t* d_dst_out,
                  int32_t* d_block_ptr, int32_t* d_n_edges_out, uint32_t* d_status, void* d_ws, size_t ws_bytes,
                  hipStream_t stream, const uint32_t* d_stream_add = nullptr, int32_t* d_readback = nullptr);

// id-map (fgl_idmap.hip)
size_t idmap_map_src_workspace_bytes(int64_t n_edges_max);
int launch_idmap_reset(void* d_table, int64_t slots, hipStream_t stream);
int launch_idmap_insert_dst(void* d_table, int64_t slots, const int32_t* d_dst_ids, int64_t n_max,
                            const int32_t* d_n, int32_t* d_uniq, uint32_t* d_status, hipStream_t stream,
                            uint32_t* d_zero_words, int64_t n_zero_words);  // (optional) scratch words to clear on the way
int launch_idmap_map_src(void* d_table, int64_t slots, const int32_t* d_src_in, int32_t* d_src_out,
                         int64_t n_edges_max, const int32_t* d_n_edges, int64_t n_base, const int32_t* d_n_base,
                         int32_t* d_n_total_out, int32_t* d_uniq, int64_t uniq_capacity, int flags,
                         uint32_t* d_status, void* d_ws, size_t ws_bytes, hipStream_t stream,
                         bool counter_is_zeroed,          // arrival order: *d_n_total_out holds zero and may count the new ids
                         const NextHop* next_hop,         // (may be null) the new nodes are seeds of a next hop: prepare its sampling
                         bool leave_table_empty,          // final calls only: every slot of the table is empty when the call's work is done
                         uint8_t* d_lowered,              // (may be null) n_edges_max bytes, zero on entry: lets the mark pass skip most table reads
                         const TransposeJob* rank_job = nullptr,     // (may be null) the edges take their ranks in this block's transposed rows
                         const TransposeJob* before_job = nullptr,   // (may be null) scan and fill steps of the hop before, carried by the first two passes
                         int32_t* d_dst_inout = nullptr,             // (may be null) n_edges_max ids that are in the table already: relabelled in place by the first pass
                         int32_t* d_readback = nullptr,              // (may be null) {node total, status word} once both are final; may be host memory
                         const int32_t* d_readback_counts = nullptr, // (may be null) instead of those two words: a copy of this array, which holds
                         int n_readback_counts = 0);                 //   *d_n_total_out and the status word, taken when the node total is final

// deterministic block transpose (fgl_transpose_sort.hip): fills t_indices / t_edge given the offsets
size_t sorted_transpose_workspace_bytes(int64_t n_cols, int64_t n_edges);
int launch_sorted_transpose_fill(const int32_t* d_indptr, const int32_t* d_indices, int64_t n_rows, int64_t n_cols,
                                 int64_t n_edges, int32_t* d_t_indices, int32_t* d_t_edge, void* d_ws, size_t ws_bytes,
                                 hipStream_t stream);

}  // namespace fgl
