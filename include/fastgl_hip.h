/*
 * fastgl_hip.h -- C ABI of libfastgl_hip.so, the MI355X (gfx950) implementation of
 * FastGL's hot path: CSR neighbour sampling, the fused id-map, block-CSR helpers and
 * memory-aware aggregation (forward and backward).
 *
 * Conventions
 *   - every pointer named d_* or documented "device" is a device pointer; everything
 *     else is a host value.  The library never allocates or frees device memory and
 *     never synchronises: all work is enqueued on `stream` (a hipStream_t passed as
 *     void*, NULL = the null stream) and scratch comes from a caller workspace whose
 *     size the matching *_workspace_bytes() function returns.
 *   - "max/count pairs": a size that is only known on the device is passed as a host
 *     upper bound (n_max) plus a device pointer to the actual int32 count (d_n, may be
 *     NULL meaning "exactly n_max").  Grids are sized for the bound, kernels read the
 *     count.  This is what lets a whole mini-batch be sampled without a host sync.
 *   - return value: FGL_OK or an FGL_ERR_* code; fgl_last_error() gives the message of
 *     the last failing call on the calling thread.  Argument errors are detected on the
 *     host before anything is launched.  Conditions only a kernel can see (hash table
 *     full, output capacity exceeded, id missing from the map) set bits in a device
 *     status word (FGL_STATUS_*), never fault, and never spin.
 *   - index arrays are int32; graph offsets (indptr of the full graph) int32 or int64.
 *
 * Each entry point names the reference interface (a1bc2def6g/fastgl-ae) it stands in for.
 */
#ifndef FASTGL_HIP_H
#define FASTGL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FGL_ABI_VERSION 11

enum fgl_error {
    FGL_OK = 0,
    FGL_ERR_ARG = 1,         /* bad argument (null pointer, negative size, unsupported value) */
    FGL_ERR_WORKSPACE = 2,   /* workspace too small or misaligned */
    FGL_ERR_HIP = 3,         /* a HIP runtime call or kernel launch failed */
    FGL_ERR_UNSUPPORTED = 4  /* valid request outside what the kernels implement */
};

enum fgl_dtype { FGL_F32 = 0, FGL_BF16 = 1 };

/* per-edge weight of fgl_aggregate (row = output row, col = gathered row) */
enum fgl_agg_mode {
    FGL_AGG_SUM = 0,     /* w = 1                                             (GIN)  */
    FGL_AGG_MEAN = 1,    /* w = 1 / deg(row)                                  (SAGE) */
    FGL_AGG_GCN = 2,     /* w = (1/sqrt(row_norm[row])) * (1/sqrt(col_norm[col]))    */
    FGL_AGG_COLMEAN = 3, /* w = 1 / max(col_norm[col], 1)   (backward of MEAN)        */
    FGL_AGG_EDGE = 4,    /* w = edge_w[entry_id * n_heads + column / (D / n_heads)]  (GAT) */
    FGL_AGG_COLMEAN_PTR = 5 /* FGL_AGG_COLMEAN with the columns' entry counts given as an offsets array:
                               col_norm[col+1] - col_norm[col] -- the row pointer of the block whose transpose is
                               being gathered, so the backward of MEAN needs no degree array */
};

/* what an output row with no entries gets */
enum fgl_zero_policy {
    FGL_ZERO_COPY_SELF = 0, /* X[row]  (reference forward kernels)   */
    FGL_ZERO_ZEROS = 1      /* zeros   (backward; DGL-style mean)    */
};

/* bits of the device status word */
#define FGL_STATUS_TABLE_FULL 1u   /* an insert found no free slot          */
#define FGL_STATUS_UNIQ_OVERFLOW 2u /* more unique ids than uniq_capacity   */
#define FGL_STATUS_MISSING_KEY 4u  /* a looked-up id is not in the table    */
#define FGL_STATUS_BAD_SEED 8u     /* a seed id outside [0, n_nodes)        */
#define FGL_STATUS_BAD_ID 16u      /* a negative id handed to the id-map    */

#define FGL_IDMAP_ORDERED 0 /* new ids numbered by first occurrence (deterministic) */
#define FGL_IDMAP_ARRIVAL 1 /* new ids numbered as their inserts land (the reference's rule,
                               id_map.cu:314-321): two passes instead of three or four and about a
                               tenth faster; the order of the new ids depends on scheduling */
#define FGL_IDMAP_FINAL 2   /* (or'ed in) the table is not consulted after this call: the local ids of the
                               new ids go to the edges and the unique list, not back into the table */
#define FGL_IDMAP_LEAVE_TABLE_EMPTY 8 /* (or'ed in, with FGL_IDMAP_FINAL only) the call's last pass, which no longer reads
                               the table, stores the empty marker over all `slots` of it: the next call on the same slots
                               needs no fgl_idmap_reset (same value and meaning as FGL_BLOCKS_LEAVE_TABLE_EMPTY) */
/* fgl_sample_blocks only, or'ed into idmap_flags: */
#define FGL_BLOCKS_TABLE_EMPTY 4       /* the caller vouches that every slot of the table is empty (as fgl_idmap_reset
                                          leaves it, or an earlier fgl_sample_blocks call with FGL_BLOCKS_LEAVE_TABLE_EMPTY
                                          on the same slots): the call's fill launch is skipped */
#define FGL_BLOCKS_LEAVE_TABLE_EMPTY 8 /* the last pass of the call also empties the table again (it no longer reads
                                          it), so that the next call may say FGL_BLOCKS_TABLE_EMPTY */
#define FGL_BLOCKS_SORT_TRANSPOSED 16  /* the rows of the transposed blocks that the call builds come out sorted by the
                                          position of their entries in the block (= by destination row), instead of in the
                                          order in which the entries' atomics landed: the same arrays from run to run, and
                                          with them the same fp32 sums in every gather over them; one more launch per call */
#define FGL_MAX_FANOUT 192

int fgl_abi_version(void);
const char* fgl_last_error(void);

/* Host side of the d_readback arguments below (where the reference copies a count back with cudaMemcpy and waits:
 * sample.cu:202, id_map.cu:454,491).  The caller stores `pending` -- a value that no size or status word can
 * take, e.g. -1 -- into each of the n_words host words, enqueues the call, and waits here: the function returns
 * when every word has been overwritten, which the device does as soon as the sizes are final -- before the
 * call's last launch has finished, and without the wake-up latency of a stream wait.  It looks at the words for
 * at most spin_limit_us microseconds (0: not at all), then waits for `stream` (the one the call went to) and
 * reports words that are still pending as an error.  What the call wrote besides is ordered by the stream, as
 * always: only the sizes are on the host early. */
int fgl_wait_words(const int32_t* h_words, int n_words, int32_t pending, void* stream, int64_t spin_limit_us);

/* ---------------------------------------------------------------------------------
 * exclusive_sum  -- replaces fastgl.exclusive_sum (cuda_operators/aggregate_acc.cpp:514-520,
 * utilis.cu:17-41): out[0..n] = exclusive prefix sums of in[0..n-1], out[n] = total.
 * `out` may alias `in` if it has room for n+1 entries.
 * ------------------------------------------------------------------------------- */
size_t fgl_exclusive_sum_workspace_bytes(int64_t n_max);
int fgl_exclusive_sum_i32(const int32_t* d_in, int64_t n_max, const int32_t* d_n, int32_t* d_out,
                          void* d_ws, size_t ws_bytes, void* stream);

/* cal_deg -- replaces fastgl.cal_deg (aggregate_acc.cpp:522-529, utilis.cu:43-79):
 * d_deg[0..n_nodes) = histogram of d_ids[0..n_ids).  d_deg is cleared by the call. */
int fgl_cal_deg(const int32_t* d_ids, int64_t n_ids_max, const int32_t* d_n_ids, int32_t* d_deg,
                int64_t n_nodes, void* stream);

/* ---------------------------------------------------------------------------------
 * sample_node -- replaces fastgl.sample_node (aggregate_acc.cpp:491-512, sample.cu:102-203).
 * For seed position i (node s = d_seeds[i]): k_i = min(fanout, deg(s)); d_block_ptr =
 * exclusive scan of k (n+1 entries; this IS the indptr of the sampled block's CSR);
 * d_src_out[block_ptr[i] + j] = j-th chosen in-neighbour (global id);
 * d_dst_out (optional, may be NULL) = s for each of those edges.
 * deg <= fanout copies the row in CSR order; otherwise a uniform random k-subset WITHOUT
 * replacement (Floyd) from Philox4x32-10 keyed by (rng_seed, stream_id, s): what a node
 * draws does not depend on its position in the seed list.
 * d_n_edges_out (optional) receives the edge count as int32.
 * d_readback (optional): two int32 that the call writes once both are final -- {edge count, status word} -- for a
 * caller that must know the size at once (as the reference's operator does, sample.cu:202).  It may point to
 * pinned host memory that the device can write (hipHostMalloc): the caller then only waits for the stream and reads
 * the two words, with no copy to enqueue behind the kernels.
 * d_src_out / d_dst_out need room for n_seeds_max * fanout entries.
 * ------------------------------------------------------------------------------- */
size_t fgl_sample_workspace_bytes(int64_t n_seeds_max, int fanout);
int fgl_sample_node(const void* d_indptr, int indptr_is64, const int32_t* d_indices, int64_t n_nodes,
                    const int32_t* d_seeds, int64_t n_seeds_max, const int32_t* d_n_seeds, int fanout,
                    uint64_t rng_seed, uint32_t stream_id,
                    int32_t* d_src_out, int32_t* d_dst_out, int32_t* d_block_ptr, int32_t* d_n_edges_out,
                    uint32_t* d_status, int32_t* d_readback, void* d_ws, size_t ws_bytes, void* stream);

/* sample_node without a workspace argument.  Has no counterpart in the reference; it is for callers
 * that cannot allocate device memory at the point of the call (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc) and therefore have no workspace to pass.  Same
 * arguments, kernels and results as fgl_sample_node; the scratch is a 16 MiB device array that the
 * library itself holds on every GPU it runs on until the process ends.  Limits: n_seeds_max <=
 * 1 048 576 (FGL_ERR_ARG beyond).  The call allocates and frees nothing.  All calls on one GPU share
 * that GPU's array: calls that overlap in time on one GPU (different streams) race -- serialise them.
 * The first call on a device looks the array's address up (hipGetSymbolAddress); make that call
 * outside stream capture. */
#define FGL_STATIC_MAX_SEEDS 1048576
int fgl_sample_node_static(const void* d_indptr, int indptr_is64, const int32_t* d_indices, int64_t n_nodes,
                           const int32_t* d_seeds, int64_t n_seeds_max, const int32_t* d_n_seeds, int fanout,
                           uint64_t rng_seed, uint32_t stream_id,
                           int32_t* d_src_out, int32_t* d_dst_out, int32_t* d_block_ptr, int32_t* d_n_edges_out,
                           uint32_t* d_status, void* stream);

/* TableSize -- the reference's sizing rule (cuda_hashtable.cuh:27-30), evaluated in 64 bits:
 * (largest power of two <= num) << scale.  Kept for callers that size by it. */
int64_t fgl_table_size(int64_t num, int scale);

/* ---------------------------------------------------------------------------------
 * id-map hash table -- replaces MutableDeviceOrderedHashTable and the free functions
 * Hash/Insert/InsertSrc/Search (id_map.cu:26-59,179-255).  8-byte slots {key, local id},
 * power-of-two slot count, multiplicative hash, linear probing bounded by the slot count.
 * fgl_idmap_slots(n) = slot count for at most n distinct ids (load factor <= 1/2).
 * ------------------------------------------------------------------------------- */
int64_t fgl_idmap_slots(int64_t max_unique);
size_t fgl_idmap_table_bytes(int64_t slots);
int fgl_idmap_reset(void* d_table, int64_t slots, void* stream);

/* insert the destination ids: local id of d_dst_ids[i] is i (id_map.cu:259-287); the ids
 * are also copied to d_uniq[0..n) when d_uniq != d_dst_ids.  If an id repeats, lookups
 * return its first position. */
int fgl_idmap_insert_dst(void* d_table, int64_t slots, const int32_t* d_dst_ids, int64_t n_max,
                         const int32_t* d_n, int32_t* d_uniq, uint32_t* d_status, void* stream);

/* number the new source ids and relabel the edges (id_map.cu:290-383 for the src half).
 * n_base ids are already numbered (host value n_base, or *d_n_base when non-NULL).
 * New ids get n_base, n_base+1, ... and are appended to d_uniq -- in order of first
 * occurrence in d_src_in (flags = FGL_IDMAP_ORDERED) or of arrival (FGL_IDMAP_ARRIVAL), either
 * optionally or'ed with FGL_IDMAP_FINAL when no later call will look these ids up in the table (and then also
 * with FGL_IDMAP_LEAVE_TABLE_EMPTY);
 * d_src_out[e] = local id of d_src_in[e] (may alias d_src_in);
 * *d_n_total_out = n_base + number of new ids (must not alias d_n_base).
 * n_base + n_edges_max must stay below 2^31 - 2. */
size_t fgl_idmap_map_src_workspace_bytes(int64_t n_edges_max);
int fgl_idmap_map_src(void* d_table, int64_t slots, const int32_t* d_src_in, int32_t* d_src_out,
                      int64_t n_edges_max, const int32_t* d_n_edges,
                      int64_t n_base, const int32_t* d_n_base, int32_t* d_n_total_out,
                      int32_t* d_uniq, int64_t uniq_capacity, int flags,
                      uint32_t* d_status, void* d_ws, size_t ws_bytes, void* stream);

/* transfer_edge_id -- the whole device part of fastgl.transfer_edge_id (aggregate_acc.cpp:467-489,
 * id_map.cu:386-493) on a table that holds nothing: the destination ids get the local ids 0..n_dst-1 and go to
 * d_uniq[0..n_dst); d_src_edges and d_dst_edges (n_edges global ids each, distinct arrays) are relabelled in place;
 * new source ids are numbered from n_dst on and appended to d_uniq; *d_n_total_out = n_dst + their number.
 * A destination id of an edge that is not in d_dst_unique becomes -1 and sets FGL_STATUS_MISSING_KEY.
 * Four launches with first-occurrence numbering (the destination half rides on the first pass over the
 * edges), against the reference's table allocation, fill and four kernels per call.  flags and workspace
 * (fgl_idmap_map_src_workspace_bytes(n_edges)) as for fgl_idmap_map_src; a caller that keeps the table between
 * calls passes FGL_IDMAP_FINAL | FGL_IDMAP_LEAVE_TABLE_EMPTY and never fills it again.
 * d_readback (optional): {node total, status word}, written once both are final; may be device-writable pinned host
 * memory, as for fgl_sample_node (the reference reads the same size back at id_map.cu:454,491). */
int fgl_idmap_transfer(void* d_table, int64_t slots, const int32_t* d_dst_unique, int64_t n_dst,
                       int32_t* d_src_edges, int32_t* d_dst_edges, int64_t n_edges, int32_t* d_uniq,
                       int64_t uniq_capacity, int flags, int32_t* d_n_total_out, uint32_t* d_status,
                       int32_t* d_readback, void* d_ws, size_t ws_bytes, void* stream);

/* relabel ids that are already in the table, in place (the dst half of
 * transfer_edge_id_kernel, id_map.cu:377-381).  A missing id becomes -1 and sets
 * FGL_STATUS_MISSING_KEY (the reference's Search would loop forever, id_map.cu:242-255). */
int fgl_idmap_lookup(const void* d_table, int64_t slots, int32_t* d_ids, int64_t n_max, const int32_t* d_n,
                     uint32_t* d_status, void* stream);

/* ---------------------------------------------------------------------------------
 * sample_blocks -- all hops of FusedMapSampler.sample_blocks (FusedMapSampler.py:63-109)
 * in one call with no host synchronisation: per hop sample_node -> id-map, the table and
 * the numbering persisting across hops (hop h's unique list is hop h+1's seed list).
 * Hops are indexed in sampling order: hop 0 expands the raw seeds with fanouts[0];
 * idmap_flags is FGL_IDMAP_ORDERED or FGL_IDMAP_ARRIVAL (the last hop adds FGL_IDMAP_FINAL by itself), optionally
 * or'ed with FGL_BLOCKS_TABLE_EMPTY, FGL_BLOCKS_LEAVE_TABLE_EMPTY and / or FGL_BLOCKS_SORT_TRANSPOSED.
 * Launches for H hops, first-occurrence numbering: one that starts the batch (counts, seeds into the table, the
 * first hop's row offsets) and four per hop (sample, insert, mark, number) = 4H + 1, plus a table fill unless the
 * caller vouches for an empty table, plus one scan per hop beyond a million seeds or four million edges, plus three
 * if the last hop's transposed block is wanted, plus two with FGL_BLOCKS_SORT_TRANSPOSED.  Each
 * hop's passes also prepare the next hop's sampling (row starts, degrees and per-tile edge counts of the nodes
 * they touch), so no hop after the first reads the graph's offsets in a pass of its own.
 * (The reference lists fanouts the other way round and iterates reversed(); the caller
 * passes them already reversed.)
 *
 * node_capacity (optional, n_hops+1 host entries, NULL = none): the caller's own limit on the
 * number of nodes before hop h (last entry: after the last hop); every entry at least the seed
 * count and none below the one before it.  Worst-case bounds assume
 * that no neighbour ever repeats; for deep fanouts they reach the size of the graph, so a
 * caller that knows its batches may size its buffers by experience instead.  A batch that
 * grows past a limit sets FGL_STATUS_UNIQ_OVERFLOW (its outputs are then invalid, nothing is
 * written out of bounds) and is repeated with larger limits.
 *
 * fgl_sample_blocks_plan fills, for the given bounds, cap_dst[h] (max seeds of hop h),
 * cap_edges[h] (max edges of hop h), *cap_uniq (max unique ids overall), *table_slots
 * (the slot count that can never overflow) and *ws_bytes.  fgl_sample_blocks also accepts a
 * smaller power-of-two table (at least fgl_idmap_slots(n_seeds)), which stays cache-resident
 * when batches are far below the bound; a batch that outgrows it sets FGL_STATUS_TABLE_FULL
 * in the status word, its outputs are then invalid and the caller repeats it with more slots.
 *
 * The call only enqueues kernels (no memset, no copy, no allocation, no synchronisation), so
 * a caller may capture it in a HIP graph and replay it: seeds, outputs, table and workspace
 * are then fixed buffers, and d_stream_offset (may be NULL) points to one device uint32 that
 * is added to stream_base when the kernels run -- the caller advances it between replays so
 * that every mini-batch draws from its own random stream.
 *
 * Outputs (device): block_ptr[h] int32[cap_dst[h]+1], src_local[h] int32[cap_edges[h]],
 * src_global[h] int32[cap_edges[h]] or NULL; d_uniq int32[cap_uniq];
 * d_counts int32[3*n_hops+2]: [0..n_hops] node count before hop h / after the last hop,
 * [n_hops+1 .. 2*n_hops] edges of hop h, [2*n_hops+1] the status word, [2*n_hops+2+h] the entry count of the
 * longest row of hop h's transposed block if that exceeds FGL_SHORT_ROW_ENTRIES, else some value not above it
 * (zero for hops whose transposed block is not built) -- read back with the sizes, it is the host bound that
 * fgl_aggregate's longest_row_max wants.
 * d_readback (may be NULL): 3*n_hops+2 int32 words of host memory that the device can write (hipHostMalloc); the
 * launch that makes the last of the counts final stores a copy of d_counts there, so the host's one read per
 * mini-batch is a wait for the stream (or for an event recorded behind the call) and a load, with no copy to enqueue.
 *
 * Transposed blocks (the column-major companions that the backward kernels gather over, see fgl_block_transpose):
 * t_ptr / t_dst / t_edge are NULL, or arrays of n_hops pointers of which any may be NULL.  Where t_ptr[h] is given
 * (int32[cap_src[h]+1], cap_src[h] = cap_dst[h+1], or cap_uniq for the last hop) the call also builds hop h's
 * transposed block: t_ptr[h] = row pointer over the hop's source nodes, t_dst[h] int32[cap_edges[h]] (required
 * then) = the destination rows each source node feeds (unordered within a row unless FGL_BLOCKS_SORT_TRANSPOSED is
 * given), t_edge[h] (optional) = the
 * position in src_local[h] of every transposed entry.  Sizes are the call's own device-side counts, so nothing
 * waits for the host.  The work rides on launches the call makes anyway -- a hop's edges take their place in their
 * transposed rows as the id-map numbers them, and the next hop's launches turn the counts into offsets and
 * fill the rows -- except for the last hop, whose transposed block costs three short launches of its own.
 * fgl_sample_blocks_plan takes the same choice as a bit mask (bit h: hop h), since the workspace depends on it.
 * The table is scratch: after the call it holds the local ids of the nodes of every hop but the
 * last (whose new nodes keep a transient value there) -- or nothing, with FGL_BLOCKS_LEAVE_TABLE_EMPTY;
 * d_uniq is the complete map local -> global.
 * ------------------------------------------------------------------------------- */
int fgl_sample_blocks_plan(int64_t n_nodes, int64_t n_seeds, const int32_t* fanouts, int n_hops,
                           const int64_t* node_capacity, uint32_t transpose_hops, int64_t* cap_dst, int64_t* cap_edges,
                           int64_t* cap_uniq, int64_t* table_slots, size_t* ws_bytes);
int fgl_sample_blocks(const void* d_indptr, int indptr_is64, const int32_t* d_indices, int64_t n_nodes,
                      const int32_t* d_seeds, int64_t n_seeds, const int32_t* fanouts, int n_hops,
                      const int64_t* node_capacity, uint64_t rng_seed, uint32_t stream_base,
                      const uint32_t* d_stream_offset, int idmap_flags,
                      void* d_table, int64_t table_slots, int32_t* d_uniq, int64_t uniq_capacity,
                      int32_t* const* block_ptr, int32_t* const* src_local, int32_t* const* src_global,
                      int32_t* const* t_ptr, int32_t* const* t_dst, int32_t* const* t_edge,
                      int32_t* d_counts, int32_t* d_readback, void* d_ws, size_t ws_bytes, void* stream);

/* ---------------------------------------------------------------------------------
 * block transpose -- the column-major companion of a block CSR, which turns the
 * reference's atomic scatter in the backward kernels (aggregate_acc_kernel.cu:467-517,
 * 554-596) into an atomic-free gather.  d_t_indptr int32[n_cols_max+1],
 * d_t_indices int32[n_edges_max] (row ids, unordered within a column); d_t_edge (optional,
 * may be NULL) int32[n_edges_max]: the position in d_indices each transposed entry came from
 * (what per-edge data, e.g. attention weights, is indexed by).  sorted = 1 orders every column
 * by ascending row (deterministic output, needs exact sizes: d_n_rows = d_n_cols = NULL, and
 * n_edges_max = the number of entries); sorted = 0 is faster and leaves the order within a
 * column to scheduling.
 * d_t_longest_row (may be NULL) receives one int32 for fgl_aggregate's d_longest_row: the
 * entry count of the transposed block's longest row if that exceeds FGL_SHORT_ROW_ENTRIES,
 * else some value not above it.
 * ------------------------------------------------------------------------------- */
#define FGL_SHORT_ROW_ENTRIES 32
size_t fgl_block_transpose_workspace_bytes(int64_t n_cols_max, int64_t n_edges_max, int sorted);
int fgl_block_transpose(const int32_t* d_indptr, const int32_t* d_indices,
                        int64_t n_rows_max, const int32_t* d_n_rows,
                        int64_t n_cols_max, const int32_t* d_n_cols, int64_t n_edges_max,
                        int32_t* d_t_indptr, int32_t* d_t_indices, int32_t* d_t_edge,
                        int32_t* d_t_longest_row, int sorted,
                        void* d_ws, size_t ws_bytes, void* stream);

/* The same for up to FGL_TRANSPOSE_BATCH_MAX blocks in the five launches that one block takes: the inner blocks of a
 * mini-batch are small, and their transposes are launch-bound one by one.  Host arrays of n_blocks entries each;
 * exact sizes only (n_edges[i] = the number of entries of block i), lists unordered within a transposed row,
 * blocks below FGL_TRANSPOSE_BATCH_MAX_EDGES entries and FGL_TRANSPOSE_BATCH_MAX_COLS columns (FGL_ERR_ARG
 * beyond: such a block fills the chip on its own, use fgl_block_transpose).  d_t_edge and d_t_longest_row may be
 * NULL, or hold NULL for some blocks. */
#define FGL_TRANSPOSE_BATCH_MAX 8
#define FGL_TRANSPOSE_BATCH_MAX_EDGES (1 << 20)
#define FGL_TRANSPOSE_BATCH_MAX_COLS (1 << 23)
size_t fgl_block_transpose_batch_workspace_bytes(int n_blocks, const int64_t* n_cols, const int64_t* n_edges);
int fgl_block_transpose_batch(int n_blocks, const int32_t* const* d_indptr, const int32_t* const* d_indices,
                              const int64_t* n_rows, const int64_t* n_cols, const int64_t* n_edges,
                              int32_t* const* d_t_indptr, int32_t* const* d_t_indices, int32_t* const* d_t_edge,
                              int32_t* const* d_t_longest_row, void* d_ws, size_t ws_bytes, void* stream);

/* ---------------------------------------------------------------------------------
 * aggregate -- the memory-aware aggregation kernels: replaces the device part of
 * fastgl.forward_gcn / forwaed_gin / forward_gat (aggregate_acc_kernel.cu:270-331, 375-427,
 * 835-886) and, on the transposed block, of backward_gcn / backward_gin / backward_gat
 * (:467-517, :554-596, :924-979); adds mean.
 *   out[r, :] = sum over e in [indptr[r], indptr[r+1]) of w(r, indices[e]) * X[indices[e], :]
 * X: [*, D] with row stride ldx elements; out: [n_rows, D] with row stride ldo; both of
 * `dtype` (fp32, or bf16 with fp32 accumulation).  d_row_norm / d_col_norm: int32 degree
 * arrays as required by `mode` (else NULL).  FGL_AGG_EDGE: d_edge_w float[n_entries, n_heads],
 * n_heads divides D, d_edge_index (optional) maps a position in d_indices to its row of
 * d_edge_w (NULL: the position itself; the d_t_edge of a transposed block otherwise).
 * (longest_row_max, d_longest_row): what the caller knows about the entry count of the
 * longest row, in the library's usual (host bound, device value) form -- host: no row holds
 * more entries than longest_row_max (the fanout for a sampled block; < 0: unknown); device:
 * NULL, or one int32 as fgl_block_transpose writes it.  Rows of several hundred entries and
 * more (hubs of a transposed block) are summed by a second launch in which a whole
 * workgroup shares each such row; a host bound that rules them out saves that launch, a
 * device value that does lets it end at once.  Speed only: wrong values still give correct sums.
 * n_entries_max: what the caller knows about the number of entries (indptr[n_rows]): an upper bound, or
 * < 0 for "unknown".  Together with n_rows_max and longest_row_max it picks the lane mapping -- several
 * lane groups per row for a few thousand rows of long lists (a small sampled block), several rows per lane
 * group for many rows of one entry on average (a transposed block), one group per row otherwise.  Speed
 * only as well; the order of the fp32 additions within a row depends on the mapping, not on the run.
 * ------------------------------------------------------------------------------- */
int fgl_aggregate(const int32_t* d_indptr, const int32_t* d_indices,
                  int64_t n_rows_max, const int32_t* d_n_rows,
                  const void* d_x, int64_t ldx, int D, int dtype, int mode, int zero_policy,
                  const int32_t* d_row_norm, const int32_t* d_col_norm,
                  const float* d_edge_w, int n_heads, const int32_t* d_edge_index,
                  int64_t longest_row_max, const int32_t* d_longest_row, int64_t n_entries_max,
                  void* d_out, int64_t ldo, void* stream);
/* Which kernel and lane mapping the calling thread's last fgl_aggregate call launched, as text ("aggregate_kernel
 * lanes/row=32", "aggregate_bundle_kernel lanes/row=64 (rows bundled by 4) + long_rows", ...): for benchmark
 * records and bug reports.  No counterpart in the reference, whose kernels have one fixed mapping
 * (aggregate_acc_kernel.cu:238-247). */
const char* fgl_aggregate_last_mapping(void);

/* ---------------------------------------------------------------------------------
 * Attention coefficients of a GAT layer over a block CSR -- replaces the three DGL calls of
 * the reference's GATConv.forward (GraphConv.py:265-272: apply_edges(u_add_v('el','er')),
 * leaky_relu, edge_softmax).  d_el float[n_cols, n_heads] (per source node), d_er
 * float[n_rows, n_heads] (per destination row); for entry e of row r and head h
 *   s = leaky_relu(el[indices[e], h] + er[r, h]),  alpha[e, h] = softmax of s over the row's entries.
 * d_alpha float[n_entries, n_heads] is what fgl_aggregate(FGL_AGG_EDGE) takes as d_edge_w.
 * A row without entries writes nothing.
 * ------------------------------------------------------------------------------- */
int fgl_edge_softmax(const int32_t* d_indptr, const int32_t* d_indices, int64_t n_rows_max,
                     const int32_t* d_n_rows, const float* d_el, const float* d_er, int n_heads,
                     float negative_slope, float* d_alpha, void* stream);

/* ---------------------------------------------------------------------------------
 * Seeded R-MAT key generator for the synthetic graphs (a=.57 b=.19 c=.19 d=.05).
 * For draw e in [first_edge, first_edge+n_edges): writes the two symmetrised keys
 * (row<<32 | col) of the in-neighbour CSR, or INT64_MAX twice for a self loop / an
 * endpoint >= n_nodes.  Has no counterpart in the reference (which downloads its datasets
 * with shell scripts); it exists so benchmark graphs are reproducible on CPU and GPU.
 * ------------------------------------------------------------------------------- */
int fgl_rmat_keys(int64_t first_edge, int64_t n_edges, int scale, int64_t n_nodes, uint64_t seed,
                  int64_t* d_keys, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FASTGL_HIP_H */
