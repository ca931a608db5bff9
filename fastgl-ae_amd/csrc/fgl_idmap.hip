// Fused id-map: open-addressing hash table over global node ids (stands in for the
// reference's Entry table and its four kernels, cuda_operators/id_map.cu:26-59,179-383).
//
// Slot = 8 bytes {uint32 key, uint32 val}, empty = all ones.  Slot count is a power of two,
// hash = (id * 0x9E3779B1) >> (32 - log2 slots), linear probing (8 slots per 64-byte line),
// every probe loop bounded by the slot count.  `val` is the node's local id once the id is
// numbered; while a batch of new ids is being numbered it transiently holds
// kPending | (index of the first edge that mentions the id), maintained with atomicMin, so that
// new ids are numbered in first-occurrence order -- deterministic, and the order DGL's
// to_block gives -- instead of the reference's race on one global counter (id_map.cu:317-320).
//
// map_src = four launches (three for small inputs):
//   1. insert     per edge: probe (one 8-byte load per slot), install {key, pending first-edge index}
//                 with one 64-bit CAS if new, else atomicMin the first-edge index; remember the slot.
//                 An id that was numbered before this call is relabelled on the spot from the val
//                 the probe has loaded anyway, and the edge takes no further part.
//   2. mark       per edge: "am I the first edge of a new id?" -> one flag bit per edge
//                 (8 edges per lane, one byte), the count of flags before each byte within its tile
//                 of 2048 edges, and per-tile counts
//   3. prefix     single workgroup over the tile counts; publishes the new node total
//                 (the edge-parallel launches are grid-stride loops over the actual count,
//                 so a bound much larger than the batch costs nothing).  Skipped while the bound
//                 is at most 2048 tiles (4 M edges): the number pass then scans the tile counts
//                 itself in every workgroup, and its first workgroup publishes the total
//   4. number     per edge, coalesced: the local id follows from the first-edge index that the mark
//                 pass left for the edge and the three counts (cache-resident arrays): no table read.
//                 The first edge of a new id appends the id to the unique list and stores the local id
//                 in the id's slot for later calls -- skipped with FGL_IDMAP_FINAL, when the caller
//                 will not consult the table again (the last hop of a mini-batch: most of its edges).
#include "fgl_common.hpp"
#include "fgl_kernels.hpp"
#include "fgl_table.hpp"
#include "fgl_transpose_job.hpp"
#include "fgl_idmap_device.hpp"

namespace fgl {

constexpr int kItems = 8;
constexpr int kTile = kBlock * kItems;

__global__ __launch_bounds__(kBlock) void idmap_insert_dst_kernel(TableRef t, const int32_t* __restrict__ ids,
                                                                  int64_t n_max, const int32_t* __restrict__ d_n,
                                                                  int32_t* __restrict__ uniq, uint32_t* __restrict__ d_status,
                                                                  uint32_t* __restrict__ zero_words, int64_t n_zero_words)
{
    const int64_t n = actual_count(n_max, d_n);
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    // (scratch of the passes that follow in the same call, cleared on the way)
    for (int64_t w = i; w < n_zero_words; w += (int64_t)gridDim.x * kBlock) zero_words[w] = 0u;
    if (i >= n) return;
    const int32_t id = ids[i];
    if (uniq != nullptr && uniq != ids) uniq[i] = id;
    if (id < 0) {  // not a node id (and -1 would read as the empty marker): reported, never inserted
        if (d_status) atomicOr(d_status, FGL_STATUS_BAD_ID);
        return;
    }
    uint32_t seen;
    const uint32_t p = find_or_insert(t, (uint32_t)id, (uint32_t)i, &seen);  // a repeated id keeps its first position
    if (p == kEmpty && d_status) atomicOr(d_status, FGL_STATUS_TABLE_FULL);
}

// Edges per lane of the insert pass: the lane's first slot loads go out together, then the compare-and-swaps of
// the edges that found their slot empty, then each sequence is finished (most are, by then).  Measured on the
// 1.5 M-edge outer hop of a 111 M-node graph: 1 edge per lane 56 us, 2 -> 62 us, 4 -> 70 us -- the pass is bound
// by the rate at which the chip retires atomics, and fewer, longer-lived waves only take parallelism away.
#ifndef FGL_INSERT_ITEMS
#define FGL_INSERT_ITEMS 1
#endif

// `src` and `out` may be the same array (relabelling in place): neither is __restrict__.
// lowered (may be null; one byte per edge, zero on entry): lowered[e] is set when a later-running insert takes the
// place of edge e as its id's first known mention.  Together with the holder bit in slot_of[] it tells the mark pass
// which edges are first mentions without a look at the table.
template <int ITEMS>
__global__ __launch_bounds__(kBlock) void idmap_insert_src_kernel(TableRef t, const int32_t* src,
                                                                  int64_t e_max, const int32_t* __restrict__ d_e,
                                                                  uint32_t* __restrict__ slot_of, int32_t* out,
                                                                  uint8_t* __restrict__ lowered,
                                                                  uint32_t* __restrict__ d_status, const TransposeRank tr,
                                                                  const TransposeJob before, int32_t* dst_inout)
{
    tjob_scan<kBlock>(before);  // (the hop before, if its transposed block is being built: counters -> offsets)
    unsigned long long* slots = reinterpret_cast<unsigned long long*>(t.words);
    const int64_t n_e = actual_count(e_max, d_e);
    constexpr int kEdges = kBlock * ITEMS;
    const int64_t n_tiles = (n_e + kEdges - 1) / kEdges;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t first = tile * kEdges + threadIdx.x;
        int32_t id[ITEMS];
        uint32_t p[ITEMS];
        unsigned long long s[ITEMS];
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            const int64_t e = first + (int64_t)j * kBlock;
            id[j] = e < n_e ? src[e] : -1;
        }
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            p[j] = ((uint32_t)id[j] * kHashMul) >> t.shift;
            s[j] = id[j] >= 0 ? slots[p[j]] : 0ull;
        }
        // The destination half of transfer_edge_id (id_map.cu:377-381) rides on this pass when the caller asks: the
        // edge's destination id -- numbered by an earlier launch -- is looked up and relabelled in place, its first
        // probe travelling together with the source id's.
        if (dst_inout != nullptr) {
#pragma unroll
            for (int j = 0; j < ITEMS; ++j) {
                const int64_t e = first + (int64_t)j * kBlock;
                if (e >= n_e) continue;
                const uint32_t d = (uint32_t)dst_inout[e];
                int32_t local = -1;
                if ((int32_t)d >= 0) {
                    uint32_t q = (d * kHashMul) >> t.shift;
                    const uint32_t limit = t.mask < kMaxProbes ? t.mask + 1 : kMaxProbes;
                    for (uint32_t n = 0; n < limit; ++n) {
                        const unsigned long long v = slots[q];
                        if ((uint32_t)v == d) {
                            // (a destination id holds its number; one that only an edge of this call has mentioned
                            // so far -- pending -- is not a destination: missing)
                            if (!((uint32_t)(v >> 32) & kPending)) local = (int32_t)(v >> 32);
                            break;
                        }
                        if ((uint32_t)v == kEmpty) break;
                        q = (q + 1) & t.mask;
                    }
                }
                if (local < 0 && d_status) atomicOr(d_status, FGL_STATUS_MISSING_KEY);
                dst_inout[e] = local;
            }
        }
        // (the compare-and-swaps of the edges whose first slot is empty -- most edges of an outer hop -- are issued
        // before any of their results is looked at)
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            const int64_t e = first + (int64_t)j * kBlock;
            if (id[j] >= 0 && (uint32_t)s[j] == kEmpty) {
                const unsigned long long fresh = (unsigned long long)(uint32_t)id[j] | ((unsigned long long)(kPending | (uint32_t)e) << 32);
                const unsigned long long seen = atomicCAS(&slots[p[j]], ~0ull, fresh);
                // what the slot held: still empty = this edge's key went in; (an installed slot is never empty again,
                // so "our own key with our own pending index" tells the continuation below that the install is done)
                s[j] = seen == ~0ull ? fresh : seen;
            }
        }
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            const int64_t e = first + (int64_t)j * kBlock;
            if (e >= n_e) continue;
            // ids numbered earlier hold a local id (no pending bit) and stay as they are; a new id keeps
            // the smallest pending edge index among the edges that mention it
            const uint32_t mine = kPending | (uint32_t)e;
            uint32_t seen = 0, displaced = kEmpty, q = kEmpty;
            bool holder = false;
            if (id[j] >= 0) {
                if (s[j] == ((unsigned long long)(uint32_t)id[j] | ((unsigned long long)mine << 32))) {
                    // installed by the compare-and-swap above (no other edge carries this pending index)
                    q = p[j];
                    seen = mine;
                    holder = true;
                } else {
                    q = insert_mention_from(t, (uint32_t)id[j], mine, p[j], s[j], &seen, &holder, &displaced);
                }
            }
            if (q == kEmpty) {
                // table full, or not a node id: reported; the edge's local id becomes -1 (written by the number pass)
                if (d_status) atomicOr(d_status, id[j] >= 0 ? FGL_STATUS_TABLE_FULL : FGL_STATUS_BAD_ID);
            } else if (!(seen & kPending)) {
                // numbered in an earlier hop (or a destination node): the edge is relabelled right here and
                // takes no further part (`out` may be `src`: this lane is the only one that touches entry e)
                out[e] = (int32_t)seen;
                take_rank(tr, e, (int32_t)seen);
                q = kDone;
            } else if (lowered != nullptr) {
                if (holder) q |= kHolderBit;
                // (a pending value left over from an earlier call's overflow may name an edge beyond this call's)
                if ((displaced & kPending) && displaced != kEmpty && (int64_t)(displaced & ~kPending) < n_e) lowered[displaced & ~kPending] = 1;
            }
            slot_of[e] = q;
        }
    }
}

__device__ __forceinline__ int64_t tiles_of(int64_t n) { return (n + kTile - 1) / kTile; }

// flags8[tile*256 + lane] bit j  <=>  edge (tile*2048 + lane*8 + j) is the first edge of a new id;
// before8[tile*256 + lane] = number of flagged edges of the tile before edge tile*2048 + lane*8;
// first_of[e] = pending | index of the first edge that mentions e's id (edges that take part only)
__global__ __launch_bounds__(kBlock) void idmap_mark_kernel(TableRef t, int64_t e_max, const int32_t* __restrict__ d_e,
                                                            const uint32_t* __restrict__ slot_of,
                                                            const uint8_t* __restrict__ lowered,
                                                            uint32_t* __restrict__ first_of,
                                                            uint8_t* __restrict__ flags8, uint16_t* __restrict__ before8,
                                                            int32_t* __restrict__ tile_sums, const TransposeJob before)
{
    __shared__ int smem[kBlock / kWave + 1];
    tjob_fill<kBlock>(before);  // (the hop before, if its transposed block is being built: entries into their rows)
    const int64_t n_e = actual_count(e_max, d_e);
    const int64_t n_tiles = tiles_of(n_e);
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t first = tile * kTile + (int64_t)threadIdx.x * kItems;
        const bool whole = first + kItems <= n_e;  // the lane's eight edges all exist: 32-byte vector accesses
        uint32_t p[kItems];
        if (whole) {
            const uint4 lo = *reinterpret_cast<const uint4*>(slot_of + first);
            const uint4 hi = *reinterpret_cast<const uint4*>(slot_of + first + 4);
            p[0] = lo.x; p[1] = lo.y; p[2] = lo.z; p[3] = lo.w;
            p[4] = hi.x; p[5] = hi.y; p[6] = hi.z; p[7] = hi.w;
        } else {
#pragma unroll
            for (int j = 0; j < kItems; ++j) p[j] = (first + j < n_e) ? slot_of[first + j] : kEmpty;
        }
        // An edge that became its id's first known mention when it was inserted and was not displaced afterwards
        // is the first mention: nothing to read.  The others (an eighth of the edges of a large hop, where the
        // inserts run nearly in edge order) read what the slot holds now.
        uint32_t low[kItems];
#pragma unroll
        for (int j = 0; j < kItems; ++j) low[j] = 1u;  // without the bookkeeping: every edge reads its slot
        if (lowered != nullptr) {
            if (whole) {
                const uint2 b = *reinterpret_cast<const uint2*>(lowered + first);
#pragma unroll
                for (int j = 0; j < kItems; ++j) low[j] = ((j < 4 ? b.x : b.y) >> (8 * (j & 3))) & 0xFFu;
            } else {
#pragma unroll
                for (int j = 0; j < kItems; ++j) low[j] = (first + j < n_e) ? lowered[first + j] : 1u;
            }
        }
        uint32_t v[kItems];
#pragma unroll
        for (int j = 0; j < kItems; ++j) {
            v[j] = 0u;
            if (p[j] < kDone) {
                if ((p[j] & kHolderBit) && low[j] == 0u) v[j] = kPending | (uint32_t)(first + j);
                else v[j] = t.words[2 * (size_t)(p[j] & ~kHolderBit) + 1];
            }
        }
        uint32_t bits = 0;
#pragma unroll
        for (int j = 0; j < kItems; ++j)
            if (p[j] < kDone && v[j] == (kPending | (uint32_t)(first + j))) bits |= 1u << j;
        // what the slot holds now -- pending | index of the id's first edge -- is all the number pass
        // needs to know about the edge: it never goes back to the table for it
        if (whole) {
            *reinterpret_cast<uint4*>(first_of + first) = make_uint4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<uint4*>(first_of + first + 4) = make_uint4(v[4], v[5], v[6], v[7]);
        } else {
#pragma unroll
            for (int j = 0; j < kItems; ++j)
                if (first + j < n_e) first_of[first + j] = v[j];
        }
        flags8[tile * kBlock + threadIdx.x] = (uint8_t)bits;
        int total;
        const int before = block_exclusive_scan<kBlock>(__popc(bits), smem, &total);
        before8[tile * kBlock + threadIdx.x] = (uint16_t)before;
        if (threadIdx.x == 0) tile_sums[tile] = total;
    }
}

// n_total = n_base + (number of new ids), clamped to the capacity of the unique list.
// readback (optional, may be host memory that the device can write): where the host reads the call's sizes.
// Without rb_counts: two words, {node total, status word}.  With rb_counts (the all-hops call's count array, which
// holds both d_n_total_out and the status word): a copy of its rb_n words as they stand now -- the other entries
// were final before this launch began.
__device__ __forceinline__ void publish_node_total(int64_t n_base, int n_new, int64_t capacity,
                                                   int32_t* __restrict__ d_n_total_out, uint32_t* __restrict__ d_status,
                                                   int32_t* __restrict__ readback = nullptr,
                                                   const int32_t* __restrict__ rb_counts = nullptr, int rb_n = 0)
{
    int64_t total = n_base + (int64_t)n_new;
    uint32_t overflow = 0u;
    if (total > capacity) {
        overflow = FGL_STATUS_UNIQ_OVERFLOW;
        if (d_status) atomicOr(d_status, FGL_STATUS_UNIQ_OVERFLOW);
        total = capacity;
    }
    if (d_n_total_out) *d_n_total_out = (int32_t)total;
    if (readback == nullptr) return;
    // (every other bit of the status word was set by an earlier launch of the call)
    const int32_t status = (int32_t)((d_status ? *d_status : 0u) | overflow);
    if (rb_counts == nullptr) {
        readback[0] = (int32_t)total;
        readback[1] = status;
        return;
    }
    for (int i = 0; i < rb_n; ++i) {
        int32_t v = rb_counts[i];
        if (rb_counts + i == d_n_total_out) v = (int32_t)total;
        if (rb_counts + i == reinterpret_cast<const int32_t*>(d_status)) v = status;
        readback[i] = v;
    }
}

// One workgroup: exclusive scan of the per-tile counts of new ids, then
// n_total = n_base + (number of new ids), clamped to the capacity of the unique list.
__global__ __launch_bounds__(1024) void idmap_prefix_publish_kernel(const int32_t* __restrict__ tile_sums,
                                                                    int32_t* __restrict__ tile_prefix, int64_t e_max,
                                                                    const int32_t* __restrict__ d_e, int64_t n_base_h,
                                                                    const int32_t* __restrict__ d_n_base, int64_t capacity,
                                                                    int32_t* __restrict__ d_n_total_out,
                                                                    uint32_t* __restrict__ d_status, int32_t* __restrict__ readback,
                                                                    const int32_t* __restrict__ rb_counts, int rb_n)
{
    __shared__ int smem[1024 / kWave + 1];
    const int n_tiles = (int)tiles_of(actual_count(e_max, d_e));
    int carry = 0;
    for (int start = 0; start < n_tiles; start += 1024) {
        const int i = start + (int)threadIdx.x;
        const int v = i < n_tiles ? tile_sums[i] : 0;
        int total;
        const int ex = block_exclusive_scan<1024>(v, smem, &total);
        if (i < n_tiles) tile_prefix[i] = carry + ex;
        carry += total;
    }
    if (threadIdx.x == 0)
        publish_node_total(d_n_base ? (int64_t)(*d_n_base) : n_base_h, carry, capacity, d_n_total_out, d_status, readback, rb_counts, rb_n);
}

// Up to this many tiles the number pass scans the tile counts itself (every workgroup, into LDS) and
// its first workgroup publishes the node total: one launch less per call where launches, not
// edges, set the time.  Above it the single-workgroup prefix launch prepares the array once.
constexpr int kSelfTilesPerLane = 8;
#ifndef FGL_NUMBER_SELF_MAX_BLOCKS
#define FGL_NUMBER_SELF_MAX_BLOCKS 1024
#endif
constexpr int kIdmapSelfPrefixTiles = kBlock * kSelfTilesPerLane;

// The new nodes that the lanes of a wave number in one step have consecutive positions (a position is a count of
// earlier new nodes, and the lanes hold consecutive edges), so their tiles of the next hop are at most two:
// one atomic per tile and wave instead of one per node -- updates of one address run one after the other, and a
// tile's 256 nodes would otherwise queue up on it.  k = 0 for lanes without a new node.  Every lane of the wave
// must call this.
__device__ __forceinline__ void add_next_tile_sums(const NextHop& next, int k, int tile)
{
    if (__ballot(k != 0) == 0) return;  // uniform
    int tmin = k != 0 ? tile : 0x7FFFFFFF;
#pragma unroll
    for (int d = kWave / 2; d >= 1; d >>= 1) {
        const int o = __shfl_xor(tmin, d, kWave);
        tmin = o < tmin ? o : tmin;
    }
    int s0 = (k != 0 && tile == tmin) ? k : 0;
    int s1 = (k != 0 && tile != tmin) ? k : 0;
#pragma unroll
    for (int d = kWave / 2; d >= 1; d >>= 1) {
        s0 += __shfl_xor(s0, d, kWave);
        s1 += __shfl_xor(s1, d, kWave);
    }
    if (lane_id() == 0) {
        atomicAdd(&next.tile_sums[tmin], s0);
        if (s1 != 0) atomicAdd(&next.tile_sums[tmin + 1], s1);
    }
}

// Lane per edge, coalesced.  `src` and `out` may be the same array: an entry is read and written by one lane only.
// (Edges whose id was numbered before this call were relabelled by the insert pass.)  The local id of an
// edge's node follows from the index of the node's first edge (first_of, from the mark pass) and the three
// counts -- small arrays that stay in cache -- so no lane reads the table; the first edge of a new id also
// appends the id to the unique list and, unless the caller has said that the table will not be consulted
// again (WRITE_BACK = false), stores the local id in the id's slot.
// SELF: no prefix launch ran; tile_prefix is unused, the tile counts are scanned here.
template <bool SELF, bool WRITE_BACK>
__global__ __launch_bounds__(kBlock) void idmap_number_kernel(TableRef t, const int32_t* src, int64_t e_max,
                                                              const int32_t* __restrict__ d_e, int64_t n_base_h,
                                                              const int32_t* __restrict__ d_n_base,
                                                              const uint32_t* __restrict__ slot_of,
                                                              const uint32_t* __restrict__ first_of,
                                                              const uint8_t* __restrict__ flags8,
                                                              const uint16_t* __restrict__ before8,
                                                              const int32_t* __restrict__ tile_sums,
                                                              const int32_t* __restrict__ tile_prefix,
                                                              int32_t* __restrict__ uniq, int64_t capacity, int32_t* out,
                                                              int32_t* __restrict__ d_n_total_out,
                                                              uint32_t* __restrict__ d_status, const NextHop next,
                                                              uint32_t* __restrict__ clear_words, int64_t n_clear_words,
                                                              const TransposeRank tr, int32_t* __restrict__ readback,
                                                              const int32_t* __restrict__ rb_counts, int rb_n)
{
    __shared__ int s_prefix[SELF ? kIdmapSelfPrefixTiles : 1];
    __shared__ int smem[kBlock / kWave + 1];
    const int64_t n_e = actual_count(e_max, d_e);
    const int64_t n_base = d_n_base ? (int64_t)(*d_n_base) : n_base_h;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    // What the first trip of the loop below reads about its edge is fetched now, so that it travels together with
    // the tile counts that the scan waits for (a small hop is one trip per workgroup: a chain of memory latencies).
    uint32_t p_ahead = kDone, first_ahead = 0;
    int32_t id_ahead = 0;
    {
        const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
        if (e < n_e) {
            p_ahead = slot_of[e];
            first_ahead = first_of[e];
            id_ahead = src[e];
        }
    }
    if constexpr (SELF) {
        const int n_tiles = (int)tiles_of(n_e);  // <= kIdmapSelfPrefixTiles: the launcher checks the bound
        int v[kSelfTilesPerLane];
        int s = 0;
#pragma unroll
        for (int j = 0; j < kSelfTilesPerLane; ++j) {
            const int i = (int)threadIdx.x * kSelfTilesPerLane + j;
            v[j] = i < n_tiles ? tile_sums[i] : 0;
            s += v[j];
        }
        int total;
        int run = block_exclusive_scan<kBlock>(s, smem, &total);
#pragma unroll
        for (int j = 0; j < kSelfTilesPerLane; ++j) {
            s_prefix[(int)threadIdx.x * kSelfTilesPerLane + j] = run;
            run += v[j];
        }
        __syncthreads();
        if (blockIdx.x == 0 && threadIdx.x == 0) publish_node_total(n_base, total, capacity, d_n_total_out, d_status, readback, rb_counts, rb_n);
    }
    // the last pass of a mini-batch, which no longer reads the table, can leave it empty for the next one
    // (first, so that the stores drain while the edges are being numbered)
    if (!WRITE_BACK && clear_words != nullptr) {
        uint4* v = reinterpret_cast<uint4*>(clear_words);  // (a table is 8-byte slots, a power of two of them, 16-byte aligned)
        const uint4 empty = make_uint4(kEmpty, kEmpty, kEmpty, kEmpty);
        for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n_clear_words / 4; i += stride) v[i] = empty;
    }
    // (the trip count is the same for all lanes of a wave: they add up their next-hop tile sums together)
    for (int64_t base = (int64_t)blockIdx.x * kBlock; base < n_e; base += stride) {
        const int64_t e = base + threadIdx.x;
        int next_k = 0, next_tile = 0;
        const bool first_trip = base == (int64_t)blockIdx.x * kBlock;
        const uint32_t p = first_trip ? p_ahead : (e < n_e ? slot_of[e] : kDone);
        int32_t id = first_trip ? id_ahead : 0;
        int64_t row_a = kRowBadId, row_deg = 0;
        if (next.row_start != nullptr && p < kDone) {  // most such edges are first mentions: fetch their node's row now
            if (!first_trip) id = src[e];
            load_row_of(next, id, &row_a, &row_deg);
        }
        if (p != kDone) {
            int64_t local = -1;
            if (p != kEmpty) {
                const int64_t ef = (int64_t)((first_trip ? first_ahead : first_of[e]) & ~kPending);  // first edge of this edge's id (ef <= e)
                if (ef < n_e) {
                    const int64_t tile = ef / kTile;
                    const int before_tile = SELF ? s_prefix[tile] : tile_prefix[tile];
                    local = n_base + before_tile + before8[ef >> 3] + __popc((uint32_t)flags8[ef >> 3] & ((1u << (ef & 7)) - 1u));
                }
                if (local >= capacity) local = -1;  // the unique list is full (reported with the node total)
                if (ef == e && local >= 0) {
                    if (next.row_start == nullptr && !first_trip) id = src[e];
                    uniq[local] = id;
                    if (WRITE_BACK) t.words[2 * (size_t)(p & ~kHolderBit) + 1] = (uint32_t)local;
                    if (next.row_start != nullptr) {
                        next_k = store_next_hop(next, local, row_a, row_deg);
                        next_tile = (int)(local / next.tile_seeds);
                    }
                }
            }
            out[e] = (int32_t)local;
            take_rank(tr, e, (int32_t)local);
        }
        if (next.row_start != nullptr) add_next_tile_sums(next, next_k, next_tile);
    }
}

__global__ __launch_bounds__(kBlock) void idmap_lookup_kernel(TableRef t, int32_t* __restrict__ ids, int64_t n_max,
                                                              const int32_t* __restrict__ d_n, uint32_t* __restrict__ d_status)
{
    const int64_t n = actual_count(n_max, d_n);
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        const uint32_t p = find_only(t.words, t.mask, t.shift, (uint32_t)ids[i]);
        if (p == kEmpty) {
            if (d_status) atomicOr(d_status, FGL_STATUS_MISSING_KEY);
            ids[i] = -1;
        } else {
            ids[i] = (int32_t)t.words[2 * (size_t)p + 1];
        }
    }
}

// ---- arrival-order numbering (FGL_IDMAP_ARRIVAL) ---------------------------------------
// The lane whose CAS installs a key numbers it at once from a global counter, as the
// reference does (id_map.cu:314-321) -- but with one counter update per workgroup instead
// of one per new id -- and relabels its edge on the spot; so does every lane that finds its id
// already numbered (a destination, an id of an earlier hop, or a new id whose number has landed).
// Only the lanes that meet a key between its install and its number (val still all ones) leave
// their edge to the second, short pass.  Two passes over the edges, one table access per edge in
// most cases; the numbering of new ids depends on scheduling (any run is a valid map, and equal
// to every other after sorting the new ids).  `src` and `out` may be the same array.
template <int ITEMS>
__global__ __launch_bounds__(kBlock) void idmap_insert_arrival_kernel(TableRef t, const int32_t* src,
                                                                      int64_t e_max, const int32_t* __restrict__ d_e,
                                                                      int64_t n_base_h, const int32_t* __restrict__ d_n_base,
                                                                      uint32_t* __restrict__ slot_of, int32_t* __restrict__ counter,
                                                                      int32_t* __restrict__ uniq, int64_t capacity, int32_t* out,
                                                                      uint32_t* __restrict__ d_status, const NextHop next,
                                                                      const TransposeRank tr, const TransposeJob before)
{
    __shared__ int smem[kBlock / kWave + 1];
    __shared__ int s_base;
    tjob_scan<kBlock>(before);  // (the hop before, if its transposed block is being built: counters -> offsets)
    constexpr int kNextTiles = kBlock * ITEMS / kWave + 2;  // next-hop tiles (64 seeds or more each) that a tile's new nodes can touch
    __shared__ int s_next[kNextTiles];
    unsigned long long* slots = reinterpret_cast<unsigned long long*>(t.words);
    const int64_t n_e = actual_count(e_max, d_e);
    const int64_t n_base = d_n_base ? (int64_t)(*d_n_base) : n_base_h;
    constexpr int kEdges = kBlock * ITEMS;
    const int64_t n_tiles = (n_e + kEdges - 1) / kEdges;
    const uint32_t limit = t.mask < kMaxProbes ? t.mask + 1 : kMaxProbes;
    // A workgroup takes a tile of 256 * ITEMS edges at a time, ITEMS per lane (edge = tile start + j * 256 + lane).
    // Several edges per lane for large inputs: one update of the global counter per tile -- updates of one address
    // run one after the other, and one per 256 edges costs more than the probing -- against the length of a
    // lane's chain of probes; one edge per lane for small inputs, which need the workgroups.
    // (The trip count is the same for every lane of the workgroup: the loop holds barriers.)
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t first = tile * kEdges + threadIdx.x;
        // p: kDone = the edge is relabelled; a slot = its id is being numbered, see the second pass; kEmpty = table full
        uint32_t p[ITEMS], id[ITEMS];
        uint32_t won = 0;
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            const int64_t e = first + (int64_t)j * kBlock;
            p[j] = kDone;
            id[j] = 0;
            if (e < n_e) {
                id[j] = (uint32_t)src[e];
                p[j] = kEmpty;
                uint32_t q = (id[j] * kHashMul) >> t.shift;
                // (a negative id is not a node id -- and -1 would read as the empty marker: no probe, reported below)
                for (uint32_t n = 0; n < ((int32_t)id[j] >= 0 ? limit : 0u); ++n) {
                    unsigned long long slot = slots[q];
                    if ((uint32_t)slot == kEmpty) {
                        // the key goes in with val still all ones = "not numbered yet"
                        const unsigned long long seen = atomicCAS(&slots[q], ~0ull, (unsigned long long)id[j] | 0xFFFFFFFF00000000ull);
                        if (seen == ~0ull) {
                            won |= 1u << j;
                            p[j] = q;
                            break;
                        }
                        slot = seen;
                    }
                    if ((uint32_t)slot == id[j]) {
                        const uint32_t v = (uint32_t)(slot >> 32);
                        if (v & 0x80000000u) {
                            p[j] = q;
                        } else {
                            out[e] = (int32_t)v;
                            take_rank(tr, e, (int32_t)v);
                            p[j] = kDone;
                        }
                        break;
                    }
                    q = (q + 1) & t.mask;
                }
                if (p[j] == kEmpty) {
                    out[e] = -1;
                    take_rank(tr, e, -1);
                    if (d_status) atomicOr(d_status, (int32_t)id[j] >= 0 ? FGL_STATUS_TABLE_FULL : FGL_STATUS_BAD_ID);
                }
            }
        }
        // the new nodes' rows in the graph (for the next hop) are fetched while the workgroup takes its numbers
        int64_t row_a[ITEMS], row_deg[ITEMS];
        if (next.row_start != nullptr) {
#pragma unroll
            for (int j = 0; j < ITEMS; ++j)
                if ((won >> j) & 1u) load_row_of(next, (int32_t)id[j], &row_a[j], &row_deg[j]);
        }
        int total;
        int rank = block_exclusive_scan<kBlock>(__popc(won), smem, &total);
        if (threadIdx.x == 0) s_base = total ? atomicAdd(counter, total) : 0;
        if (next.row_start != nullptr)
            for (int i = threadIdx.x; i < kNextTiles; i += kBlock) s_next[i] = 0;
        __syncthreads();
        const int64_t base = n_base + s_base;
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            const int64_t e = first + (int64_t)j * kBlock;
            if ((won >> j) & 1u) {
                const int64_t local = base + rank++;
                if (local < capacity) {
                    t.words[2 * (size_t)p[j] + 1] = (uint32_t)local;
                    uniq[local] = (int32_t)id[j];
                    out[e] = (int32_t)local;
                    take_rank(tr, e, (int32_t)local);
                    if (next.row_start != nullptr) {
                        // (the tile's new nodes have consecutive positions: few next-hop tiles, summed in LDS first)
                        const int k = store_next_hop(next, local, row_a[j], row_deg[j]);
                        if (k != 0) atomicAdd(&s_next[(int)(local / next.tile_seeds - base / next.tile_seeds)], k);
                    }
                } else {
                    out[e] = -1;  // the unique list is full (reported by the second pass); val stays "not numbered"
                    take_rank(tr, e, -1);
                }
                p[j] = kDone;
            }
            if (e < n_e) slot_of[e] = p[j];
        }
        __syncthreads();
        if (next.row_start != nullptr) {
            for (int i = threadIdx.x; i < kNextTiles; i += kBlock)
                if (s_next[i] != 0) atomicAdd(&next.tile_sums[base / next.tile_seeds + i], s_next[i]);
            __syncthreads();  // s_next is cleared again at the top of the next tile
        }
    }
}

// Second pass of the arrival-order numbering: the edges whose id was between install and number when
// their lane met it read the number now; also publishes the node total.
__global__ __launch_bounds__(kBlock) void idmap_relabel_publish_kernel(TableRef t, int64_t e_max, const int32_t* __restrict__ d_e,
                                                                       const uint32_t* __restrict__ slot_of,
                                                                       int32_t* __restrict__ out, const int32_t* __restrict__ counter,
                                                                       int64_t n_base_h, const int32_t* __restrict__ d_n_base,
                                                                       int64_t capacity, int32_t* __restrict__ d_n_total_out,
                                                                       uint32_t* __restrict__ d_status, const TransposeRank tr,
                                                                       const TransposeJob before, int32_t* __restrict__ readback,
                                                                       const int32_t* __restrict__ rb_counts, int rb_n)
{
    tjob_fill<kBlock>(before);  // (the hop before, if its transposed block is being built: entries into their rows)
    const int64_t n_e = actual_count(e_max, d_e);
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < n_e; e += stride) {
        const uint32_t p = slot_of[e];
        if (p >= kDone) continue;  // relabelled by the first pass (kDone) or reported there (kEmpty)
        const uint32_t v = t.words[2 * (size_t)p + 1];
        const int32_t local = (v & 0x80000000u) ? -1 : (int32_t)v;  // (still unnumbered: the unique list was full)
        out[e] = local;
        take_rank(tr, e, local);
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        const int64_t n_base = d_n_base ? (int64_t)(*d_n_base) : n_base_h;
        publish_node_total(n_base, *counter, capacity, d_n_total_out, d_status, readback, rb_counts, rb_n);
    }
}

// Inputs up to this many edges number their new ids one edge per lane (see idmap_insert_arrival_kernel).
constexpr int64_t kArrivalSmallEdges = 1 << 18;
constexpr int kArrivalItems = 4;  // edges per lane for large inputs (measured on a 1.5 M-edge hop: 8 -> 69 us, 4 -> 62 us, 2 -> 66 us, 1 -> 100 us)

// Workgroups for a grid-stride pass over n items: enough to fill every CU several times
// over, never more than the work needs.
static inline unsigned stride_grid(int64_t n_items, int items_per_block)
{
    int64_t blocks = ceil_div(n_items > 0 ? n_items : 1, items_per_block);
    if (blocks > 8192) blocks = 8192;
    return (unsigned)blocks;
}

// ---- launchers ------------------------------------------------------------------
int launch_idmap_reset(void* d_table, int64_t slots, hipStream_t stream)
{
    FGL_REQUIRE(d_table != nullptr && valid_slots(slots), "idmap: slot count %lld is not a power of two in [64, 2^31]", (long long)slots);
    return launch_fill_u32(static_cast<uint32_t*>(d_table), slots * 2, kEmpty, stream);
}

int launch_idmap_insert_dst(void* d_table, int64_t slots, const int32_t* d_dst_ids, int64_t n_max, const int32_t* d_n,
                            int32_t* d_uniq, uint32_t* d_status, hipStream_t stream, uint32_t* d_zero_words, int64_t n_zero_words)
{
    FGL_REQUIRE(d_table != nullptr && valid_slots(slots), "idmap: slot count %lld is not a power of two in [64, 2^31]", (long long)slots);
    FGL_REQUIRE(n_max >= 0 && n_max <= slots / 2, "idmap_insert_dst: %lld ids do not fit %lld slots at load 1/2", (long long)n_max, (long long)slots);
    FGL_REQUIRE(n_max <= 0x7FFFFFFF, "idmap_insert_dst: too many ids");
    if (d_zero_words == nullptr) n_zero_words = 0;
    if (n_max == 0 && n_zero_words == 0) return FGL_OK;
    FGL_REQUIRE(n_max == 0 || d_dst_ids != nullptr, "idmap_insert_dst: null ids");
    int64_t blocks = ceil_div(n_max, kBlock);
    const int64_t zero_blocks = ceil_div(n_zero_words, (int64_t)kBlock * 16) < 2048 ? ceil_div(n_zero_words, (int64_t)kBlock * 16) : 2048;
    if (blocks < zero_blocks) blocks = zero_blocks;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(idmap_insert_dst_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, make_ref(d_table, slots),
                       d_dst_ids, n_max, d_n, d_uniq, d_status, d_zero_words, n_zero_words);
    FGL_CHECK_LAUNCH("idmap_insert_dst_kernel");
    return FGL_OK;
}

size_t idmap_map_src_workspace_bytes(int64_t n_edges_max)
{
    const int64_t tiles = ceil_div(n_edges_max > 0 ? n_edges_max : 1, kTile);
    Carver c(nullptr);
    c.take<uint32_t>((size_t)n_edges_max);      // slot_of
    c.take<uint32_t>((size_t)n_edges_max);      // first_of
    c.take<uint8_t>((size_t)tiles * kBlock);    // flags8
    c.take<uint16_t>((size_t)tiles * kBlock);   // before8
    c.take<int32_t>((size_t)tiles);             // tile sums
    c.take<int32_t>((size_t)tiles);             // tile prefix
    c.take<uint32_t>((size_t)(n_edges_max + 3) / 4);  // one byte per edge ("displaced as first mention"), used by fgl_idmap_transfer
    return c.used();
}

int launch_idmap_map_src(void* d_table, int64_t slots, const int32_t* d_src_in, int32_t* d_src_out, int64_t n_edges_max,
                         const int32_t* d_n_edges, int64_t n_base, const int32_t* d_n_base, int32_t* d_n_total_out,
                         int32_t* d_uniq, int64_t uniq_capacity, int flags, uint32_t* d_status, void* d_ws,
                         size_t ws_bytes, hipStream_t stream, bool counter_is_zeroed, const NextHop* next_hop,
                         bool leave_table_empty, uint8_t* d_lowered, const TransposeJob* rank_job,
                         const TransposeJob* before_job, int32_t* d_dst_inout, int32_t* d_readback,
                         const int32_t* d_readback_counts, int n_readback_counts)
{
    FGL_REQUIRE(d_table != nullptr && valid_slots(slots), "idmap: slot count %lld is not a power of two in [64, 2^31]", (long long)slots);
    FGL_REQUIRE((flags & ~(FGL_IDMAP_ARRIVAL | FGL_IDMAP_FINAL)) == 0, "idmap_map_src: unknown flags %d", flags);
    const bool final_call = (flags & FGL_IDMAP_FINAL) != 0;
    FGL_REQUIRE(n_edges_max >= 0 && n_base >= 0 && uniq_capacity >= 0, "idmap_map_src: negative size");
    FGL_REQUIRE(n_base + n_edges_max <= 0x7FFFFFFDll, "idmap_map_src: n_base + n_edges exceeds 31 bits");
    FGL_REQUIRE(n_edges_max == 0 || (d_src_in && d_src_out && d_uniq), "idmap_map_src: null pointer");
    FGL_REQUIRE(d_n_total_out == nullptr || d_n_total_out != d_n_base, "idmap_map_src: n_total_out must not alias n_base");
    if (d_ws == nullptr || ws_bytes < idmap_map_src_workspace_bytes(n_edges_max)) {
        set_error("idmap_map_src: workspace too small (%zu < %zu)", ws_bytes, idmap_map_src_workspace_bytes(n_edges_max));
        return FGL_ERR_WORKSPACE;
    }
    FGL_REQUIRE(((uintptr_t)d_ws & 15) == 0, "idmap_map_src: the workspace must be 16-byte aligned");
    const int64_t tiles = ceil_div(n_edges_max > 0 ? n_edges_max : 1, kTile);
    Carver c(d_ws);
    uint32_t* slot_of = c.take<uint32_t>((size_t)n_edges_max);
    uint32_t* first_of = c.take<uint32_t>((size_t)n_edges_max);
    uint8_t* flags8 = c.take<uint8_t>((size_t)tiles * kBlock);
    uint16_t* before8 = c.take<uint16_t>((size_t)tiles * kBlock);
    int32_t* sums = c.take<int32_t>((size_t)tiles);
    int32_t* prefix = c.take<int32_t>((size_t)tiles);
    const TableRef t = make_ref(d_table, slots);
    unsigned edge_blocks = stride_grid(n_edges_max, kBlock);
    const unsigned tile_blocks = stride_grid(n_edges_max, kTile);
    NextHop next{};  // all null: nothing to prepare
    if (next_hop != nullptr) next = *next_hop;
    const TransposeRank tr = rank_of(rank_job);
    TransposeJob before;
    memset(&before, 0, sizeof(before));
    if (before_job != nullptr) before = *before_job;
    // the two passes that carry the hop before's scan and fill steps get workgroups of their own for those,
    // behind the pass's own
    TransposeJob scan_job = before, fill_job = before;
    unsigned scan_blocks = 0, fill_blocks_t = 0;
    if (before.cnt != nullptr) {
        scan_job.side_first = fill_job.side_first = 0;
        scan_blocks = scan_job.side_blocks = side_blocks_for(before.cols_max * before.split + 1, kTjobTile);
        fill_blocks_t = fill_job.side_blocks = side_blocks_for(before.rows_max, kBlock / 16, 16384);
    }
    FGL_REQUIRE(!leave_table_empty || final_call, "idmap_map_src: only a final call can leave the table empty");

    if (flags & FGL_IDMAP_ARRIVAL) {
        if (d_dst_inout != nullptr && n_edges_max > 0) {  // (this numbering's passes do not carry the destination half: a launch of its own)
            hipLaunchKernelGGL(idmap_lookup_kernel, dim3(edge_blocks), dim3(kBlock), 0, stream, t, d_dst_inout, n_edges_max, d_n_edges, d_status);
            FGL_CHECK_LAUNCH("idmap_lookup_kernel");
        }
        // the counter of new ids: *d_n_total_out itself when the caller vouches that it holds zero (the all-hops
        // entry point zeroes its counts when it resets the table), else one int of the (otherwise unused)
        // tile-sum array, zeroed by a launch of its own
        int32_t* counter = (counter_is_zeroed && d_n_total_out) ? d_n_total_out : sums;
        if (counter == sums) {
            int rc0 = launch_fill_u32(reinterpret_cast<uint32_t*>(counter), 1, 0u, stream);
            if (rc0 != FGL_OK) return rc0;
        }
        if (n_edges_max > kArrivalSmallEdges)
            hipLaunchKernelGGL(idmap_insert_arrival_kernel<kArrivalItems>,
                               dim3(stride_grid(n_edges_max, kBlock * kArrivalItems) + scan_blocks),
                               dim3(kBlock), 0, stream, t, d_src_in,
                               n_edges_max, d_n_edges, n_base, d_n_base, slot_of, counter, d_uniq, uniq_capacity, d_src_out,
                               d_status, next, tr, scan_job);
        else
            hipLaunchKernelGGL(idmap_insert_arrival_kernel<1>, dim3(edge_blocks + scan_blocks), dim3(kBlock), 0, stream, t, d_src_in,
                               n_edges_max, d_n_edges, n_base, d_n_base, slot_of, counter, d_uniq, uniq_capacity, d_src_out,
                               d_status, next, tr, scan_job);
        FGL_CHECK_LAUNCH("idmap_insert_arrival_kernel");
        hipLaunchKernelGGL(idmap_relabel_publish_kernel, dim3(edge_blocks + fill_blocks_t), dim3(kBlock), 0, stream, t, n_edges_max, d_n_edges,
                           slot_of, d_src_out, counter, n_base, d_n_base, uniq_capacity, d_n_total_out, d_status, tr, fill_job, d_readback,
                           d_readback_counts, n_readback_counts);
        FGL_CHECK_LAUNCH("idmap_relabel_publish_kernel");
        // (the second pass reads the table, so emptying it takes a launch of its own here)
        if (leave_table_empty) return launch_fill_u32(t.words, slots * 2, kEmpty, stream);
        return FGL_OK;
    }

    // (the holder bit shares a word with the slot index: tables of 2^31 slots go without the bookkeeping)
    uint8_t* lowered = slots <= ((int64_t)1 << 30) ? d_lowered : nullptr;
    // (small inputs need the workgroups more than the edges in flight per lane)
    if (n_edges_max > kArrivalSmallEdges)
        hipLaunchKernelGGL(idmap_insert_src_kernel<FGL_INSERT_ITEMS>, dim3(stride_grid(n_edges_max, kBlock * FGL_INSERT_ITEMS) + scan_blocks),
                           dim3(kBlock), 0, stream, t, d_src_in, n_edges_max, d_n_edges, slot_of, d_src_out, lowered, d_status, tr, scan_job,
                           d_dst_inout);
    else
        hipLaunchKernelGGL(idmap_insert_src_kernel<1>, dim3(edge_blocks + scan_blocks), dim3(kBlock), 0, stream, t, d_src_in,
                           n_edges_max, d_n_edges, slot_of, d_src_out, lowered, d_status, tr, scan_job, d_dst_inout);
    FGL_CHECK_LAUNCH("idmap_insert_src_kernel");
    hipLaunchKernelGGL(idmap_mark_kernel, dim3(tile_blocks + fill_blocks_t), dim3(kBlock), 0, stream, t, n_edges_max, d_n_edges,
                       slot_of, lowered, first_of, flags8, before8, sums, fill_job);
    FGL_CHECK_LAUNCH("idmap_mark_kernel");
#define FGL_LAUNCH_NUMBER(SELF, WB, PREFIX, TOTAL, STATUS, READBACK)                                                              \
    hipLaunchKernelGGL((idmap_number_kernel<SELF, WB>), dim3(edge_blocks), dim3(kBlock), 0, stream, t, d_src_in,        \
                       n_edges_max, d_n_edges, n_base, d_n_base, slot_of, first_of, flags8, before8, sums, PREFIX, d_uniq, \
                       uniq_capacity, d_src_out, TOTAL, STATUS, next, clear_words, n_clear_words, tr, READBACK, d_readback_counts,   \
                       n_readback_counts)
    // emptying the table rides on the last pass: enough workgroups for a fill of that size
    uint32_t* clear_words = leave_table_empty ? t.words : nullptr;
    const int64_t n_clear_words = leave_table_empty ? slots * 2 : 0;
    if (leave_table_empty) {
        const unsigned fill_blocks = stride_grid(n_clear_words, kBlock * 8);
        if (fill_blocks > edge_blocks) edge_blocks = fill_blocks;
    }
    // every workgroup of a pass that scans the tile counts itself pays for that scan once: a few workgroups per
    // compute unit, each looping over several tiles of edges, instead of one per 256 edges
    if (tiles <= kIdmapSelfPrefixTiles && edge_blocks > FGL_NUMBER_SELF_MAX_BLOCKS) edge_blocks = FGL_NUMBER_SELF_MAX_BLOCKS;
    if (tiles <= kIdmapSelfPrefixTiles) {
        if (final_call) FGL_LAUNCH_NUMBER(true, false, nullptr, d_n_total_out, d_status, d_readback);
        else FGL_LAUNCH_NUMBER(true, true, nullptr, d_n_total_out, d_status, d_readback);
    } else {
        hipLaunchKernelGGL(idmap_prefix_publish_kernel, dim3(1), dim3(1024), 0, stream, sums, prefix, n_edges_max,
                           d_n_edges, n_base, d_n_base, uniq_capacity, d_n_total_out, d_status, d_readback, d_readback_counts,
                           n_readback_counts);
        FGL_CHECK_LAUNCH("idmap_prefix_publish_kernel");
        if (final_call) FGL_LAUNCH_NUMBER(false, false, prefix, nullptr, nullptr, nullptr);
        else FGL_LAUNCH_NUMBER(false, true, prefix, nullptr, nullptr, nullptr);
    }
#undef FGL_LAUNCH_NUMBER
    FGL_CHECK_LAUNCH("idmap_number_kernel");
    return FGL_OK;
}

}  // namespace fgl

using namespace fgl;

FGL_EXPORT int64_t fgl_table_size(int64_t num, int scale)
{
    // (largest power of two <= num) << scale, as cuda_hashtable.cuh:27-30 computes for num >= 2
    int64_t half = num >> 1, p = 1;
    if (half >= 1) {
        int lg = 0;
        while ((half >> (lg + 1)) != 0) ++lg;
        p = (int64_t)1 << (1 + lg);
    }
    return p << scale;
}

FGL_EXPORT int64_t fgl_idmap_slots(int64_t max_unique)
{
    int64_t want = 2 * (max_unique > 0 ? max_unique : 0);
    int64_t s = 64;
    while (s < want) s <<= 1;
    return s;
}

FGL_EXPORT size_t fgl_idmap_table_bytes(int64_t slots) { return slots > 0 ? (size_t)slots * 8 : 0; }

FGL_EXPORT int fgl_idmap_reset(void* d_table, int64_t slots, void* stream) { return launch_idmap_reset(d_table, slots, as_stream(stream)); }

FGL_EXPORT int fgl_idmap_insert_dst(void* d_table, int64_t slots, const int32_t* d_dst_ids, int64_t n_max,
                                    const int32_t* d_n, int32_t* d_uniq, uint32_t* d_status, void* stream)
{
    return launch_idmap_insert_dst(d_table, slots, d_dst_ids, n_max, d_n, d_uniq, d_status, as_stream(stream), nullptr, 0);
}

FGL_EXPORT size_t fgl_idmap_map_src_workspace_bytes(int64_t n_edges_max) { return idmap_map_src_workspace_bytes(n_edges_max < 0 ? 0 : n_edges_max); }

FGL_EXPORT int fgl_idmap_map_src(void* d_table, int64_t slots, const int32_t* d_src_in, int32_t* d_src_out,
                                 int64_t n_edges_max, const int32_t* d_n_edges, int64_t n_base, const int32_t* d_n_base,
                                 int32_t* d_n_total_out, int32_t* d_uniq, int64_t uniq_capacity, int flags,
                                 uint32_t* d_status, void* d_ws, size_t ws_bytes, void* stream)
{
    const bool leave_empty = (flags & FGL_IDMAP_LEAVE_TABLE_EMPTY) != 0;
    FGL_REQUIRE(!leave_empty || (flags & FGL_IDMAP_FINAL), "idmap_map_src: FGL_IDMAP_LEAVE_TABLE_EMPTY needs FGL_IDMAP_FINAL");
    return launch_idmap_map_src(d_table, slots, d_src_in, d_src_out, n_edges_max, d_n_edges, n_base, d_n_base,
                                d_n_total_out, d_uniq, uniq_capacity, flags & ~FGL_IDMAP_LEAVE_TABLE_EMPTY, d_status, d_ws, ws_bytes,
                                as_stream(stream), false, nullptr, leave_empty, nullptr, nullptr, nullptr, nullptr);
}

FGL_EXPORT int fgl_idmap_transfer(void* d_table, int64_t slots, const int32_t* d_dst_unique, int64_t n_dst,
                                  int32_t* d_src_edges, int32_t* d_dst_edges, int64_t n_edges, int32_t* d_uniq,
                                  int64_t uniq_capacity, int flags, int32_t* d_n_total_out, uint32_t* d_status,
                                  int32_t* d_readback, void* d_ws, size_t ws_bytes, void* stream)
{
    FGL_REQUIRE(n_dst >= 0 && n_edges >= 0, "idmap_transfer: negative size");
    FGL_REQUIRE(n_edges == 0 || (d_src_edges && d_dst_edges), "idmap_transfer: null edge array");
    FGL_REQUIRE(d_src_edges == nullptr || d_src_edges != d_dst_edges, "idmap_transfer: the two edge arrays must be distinct");
    FGL_REQUIRE(d_uniq != nullptr && uniq_capacity >= n_dst, "idmap_transfer: the unique list cannot hold the destination ids");
    const bool leave_empty = (flags & FGL_IDMAP_LEAVE_TABLE_EMPTY) != 0;
    FGL_REQUIRE(!leave_empty || (flags & FGL_IDMAP_FINAL), "idmap_transfer: FGL_IDMAP_LEAVE_TABLE_EMPTY needs FGL_IDMAP_FINAL");
    if (d_ws == nullptr || ws_bytes < idmap_map_src_workspace_bytes(n_edges)) {
        set_error("idmap_transfer: workspace too small (%zu < %zu)", ws_bytes, idmap_map_src_workspace_bytes(n_edges));
        return FGL_ERR_WORKSPACE;
    }
    // the last piece of the workspace: one byte per edge that lets the mark pass skip most of its table reads;
    // cleared by the launch that inserts the destination ids
    const int64_t tiles = ceil_div(n_edges > 0 ? n_edges : 1, kTile);
    Carver c(d_ws);
    c.take<uint32_t>((size_t)n_edges);
    c.take<uint32_t>((size_t)n_edges);
    c.take<uint8_t>((size_t)tiles * kBlock);
    c.take<uint16_t>((size_t)tiles * kBlock);
    c.take<int32_t>((size_t)tiles);
    c.take<int32_t>((size_t)tiles);
    uint32_t* lowered_words = c.take<uint32_t>((size_t)(n_edges + 3) / 4);
    int rc = launch_idmap_insert_dst(d_table, slots, d_dst_unique, n_dst, nullptr, d_uniq, d_status, as_stream(stream), lowered_words,
                                     (n_edges + 3) / 4);
    if (rc != FGL_OK) return rc;
    return launch_idmap_map_src(d_table, slots, d_src_edges, d_src_edges, n_edges, nullptr, n_dst, nullptr, d_n_total_out, d_uniq,
                                uniq_capacity, flags & ~FGL_IDMAP_LEAVE_TABLE_EMPTY, d_status, d_ws, ws_bytes, as_stream(stream), false,
                                nullptr, leave_empty, reinterpret_cast<uint8_t*>(lowered_words), nullptr, nullptr, d_dst_edges, d_readback);
}

FGL_EXPORT int fgl_idmap_lookup(const void* d_table, int64_t slots, int32_t* d_ids, int64_t n_max, const int32_t* d_n,
                                uint32_t* d_status, void* stream)
{
    FGL_REQUIRE(d_table != nullptr && valid_slots(slots), "idmap: slot count %lld is not a power of two in [64, 2^31]", (long long)slots);
    FGL_REQUIRE(n_max >= 0, "idmap_lookup: negative size");
    if (n_max == 0) return FGL_OK;
    FGL_REQUIRE(d_ids != nullptr, "idmap_lookup: null ids");
    hipLaunchKernelGGL(idmap_lookup_kernel, dim3(stride_grid(n_max, kBlock)), dim3(kBlock), 0, as_stream(stream),
                       make_ref(const_cast<void*>(d_table), slots), d_ids, n_max, d_n, d_status);
    FGL_CHECK_LAUNCH("idmap_lookup_kernel");
    return FGL_OK;
}
