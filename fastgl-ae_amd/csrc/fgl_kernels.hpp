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
                       hipStream_t stream);
int launch_fill_u32(uint32_t* p, int64_t n, uint32_t value, hipStream_t stream);

// neighbour sampling (fgl_sample.hip)
size_t sample_workspace_bytes(int64_t n_seeds_max, int fanout);
int launch_sample(const void* d_indptr, int indptr_is64, const int32_t* d_indices, int64_t n_nodes,
                  const int32_t* d_seeds, int64_t n_seeds_max, const int32_t* d_n_seeds, int fanout,
                  uint64_t rng_seed, uint32_t stream_id, int32_t* d_src_out, int32_t* d_dst_out,
                  int32_t* d_block_ptr, int32_t* d_n_edges_out, uint32_t* d_status, void* d_ws, size_t ws_bytes,
                  hipStream_t stream, const uint32_t* d_stream_add = nullptr);

// id-map (fgl_idmap.hip)
size_t idmap_map_src_workspace_bytes(int64_t n_edges_max);
int launch_idmap_reset(void* d_table, int64_t slots, hipStream_t stream);
int launch_idmap_insert_dst(void* d_table, int64_t slots, const int32_t* d_dst_ids, int64_t n_max,
                            const int32_t* d_n, int32_t* d_uniq, uint32_t* d_status, hipStream_t stream);
int launch_idmap_map_src(void* d_table, int64_t slots, const int32_t* d_src_in, int32_t* d_src_out,
                         int64_t n_edges_max, const int32_t* d_n_edges, int64_t n_base, const int32_t* d_n_base,
                         int32_t* d_n_total_out, int32_t* d_uniq, int64_t uniq_capacity, int flags,
                         uint32_t* d_status, void* d_ws, size_t ws_bytes, hipStream_t stream,
                         bool counter_is_zeroed = false);  // arrival order: *d_n_total_out holds zero and may count the new ids

// deterministic block transpose (fgl_transpose_sort.hip): fills t_indices / t_edge given the offsets
size_t sorted_transpose_workspace_bytes(int64_t n_cols, int64_t n_edges);
int launch_sorted_transpose_fill(const int32_t* d_indptr, const int32_t* d_indices, int64_t n_rows, int64_t n_cols,
                                 int64_t n_edges, int32_t* d_t_indices, int32_t* d_t_edge, void* d_ws, size_t ws_bytes,
                                 hipStream_t stream);

}  // namespace fgl
