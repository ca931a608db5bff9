// Fused id-map: open-addressing hash table over global node ids (stands in for the
// reference's Entry table and its four kernels, cuda_operators/id_map.cu:26-59,179-383).
//
// Slot = 8 bytes {uint32 key, uint32 val}, empty = all ones.  Slot count is a power of two,
// hash = (id * 0x9E3779B1) >> (32 - log2 slots), linear probing (8 slots per 64-byte line),
// every probe loop bounded by the slot count.  `val` is the node's local id once the id is
// numbered; while a batch of new ids is being numbered it transiently holds
// n_base + (index of the first edge that mentions the id), maintained with atomicMin, so that
// new ids are numbered in first-occurrence order -- deterministic, and the order DGL's
// to_block gives -- instead of the reference's race on one global counter (id_map.cu:317-320).
//
// map_src = five launches:
//   1. insert     per edge: probe, CAS the key in if new, atomicMin the first-edge index,
//                 remember the slot
//   2. mark       per edge: "am I the first edge of a new id?" -> one flag bit per edge
//                 (8 edges per lane, one byte) + per-tile counts
//   3. prefix     single workgroup over the tile counts; publishes the new node total
//   4. assign     per tile: scan of the flags -> local ids for the first edges; writes the
//                 slot's val and appends the id to the unique list
//   5. relabel    per edge: src_out[e] = val of the remembered slot
#include "fgl_common.hpp"
#include "fgl_kernels.hpp"

namespace fgl {

constexpr uint32_t kEmpty = 0xFFFFFFFFu;
constexpr uint32_t kHashMul = 0x9E3779B1u;
constexpr int kItems = 8;
constexpr int kTile = kBlock * kItems;

struct TableRef {
    uint32_t* words;  // 2 per slot: key, val
    uint32_t mask;
    int shift;
};

static inline int log2_slots(int64_t slots)
{
    int lg = 0;
    while (((int64_t)1 << lg) < slots) ++lg;
    return lg;
}

static inline bool valid_slots(int64_t slots) { return slots >= 64 && slots <= ((int64_t)1 << 31) && (slots & (slots - 1)) == 0; }

static inline TableRef make_ref(void* d_table, int64_t slots)
{
    TableRef t;
    t.words = static_cast<uint32_t*>(d_table);
    t.mask = (uint32_t)(slots - 1);
    t.shift = 32 - log2_slots(slots);
    return t;
}

__device__ __forceinline__ uint32_t load_key(const uint32_t* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Finds the slot of `id`, inserting the key if absent.  Returns kEmpty if the table is full.
__device__ __forceinline__ uint32_t find_or_insert(const TableRef t, uint32_t id)
{
    uint32_t p = (id * kHashMul) >> t.shift;
    for (uint32_t n = 0; n <= t.mask; ++n) {
        uint32_t k = load_key(&t.words[2 * (size_t)p]);
        if (k == kEmpty) {
            // a stale or racing view of an empty slot is settled by the CAS
            const uint32_t seen = atomicCAS(&t.words[2 * (size_t)p], kEmpty, id);
            k = (seen == kEmpty) ? id : seen;
        }
        if (k == id) return p;
        p = (p + 1) & t.mask;
    }
    return kEmpty;
}

// Finds the slot of `id` without inserting.  kEmpty if absent.
__device__ __forceinline__ uint32_t find_only(const uint32_t* __restrict__ words, uint32_t mask, int shift, uint32_t id)
{
    uint32_t p = (id * kHashMul) >> shift;
    for (uint32_t n = 0; n <= mask; ++n) {
        const uint32_t k = words[2 * (size_t)p];
        if (k == id) return p;
        if (k == kEmpty) return kEmpty;
        p = (p + 1) & mask;
    }
    return kEmpty;
}

__global__ __launch_bounds__(kBlock) void idmap_insert_dst_kernel(TableRef t, const int32_t* __restrict__ ids,
                                                                  int64_t n_max, const int32_t* __restrict__ d_n,
                                                                  int32_t* __restrict__ uniq, uint32_t* __restrict__ d_status)
{
    const int64_t n = actual_count(n_max, d_n);
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int32_t id = ids[i];
    if (uniq != nullptr && uniq != ids) uniq[i] = id;
    const uint32_t p = find_or_insert(t, (uint32_t)id);
    if (p == kEmpty) {
        if (d_status) atomicOr(d_status, FGL_STATUS_TABLE_FULL);
        return;
    }
    atomicMin(&t.words[2 * (size_t)p + 1], (uint32_t)i);
}

__global__ __launch_bounds__(kBlock) void idmap_insert_src_kernel(TableRef t, const int32_t* __restrict__ src,
                                                                  int64_t e_max, const int32_t* __restrict__ d_e,
                                                                  int64_t n_base_h, const int32_t* __restrict__ d_n_base,
                                                                  uint32_t* __restrict__ slot_of, uint32_t* __restrict__ d_status)
{
    const int64_t n_e = actual_count(e_max, d_e);
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_e) return;
    const uint32_t n_base = d_n_base ? (uint32_t)(*d_n_base) : (uint32_t)n_base_h;
    const uint32_t id = (uint32_t)src[e];
    const uint32_t p = find_or_insert(t, id);
    slot_of[e] = p;
    if (p == kEmpty) {
        if (d_status) atomicOr(d_status, FGL_STATUS_TABLE_FULL);
        return;
    }
    uint32_t* val = &t.words[2 * (size_t)p + 1];
    const uint32_t mine = n_base + (uint32_t)e;
    // ids numbered earlier (val < n_base) are final; otherwise keep the smallest edge index
    if (__hip_atomic_load(val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) > mine) atomicMin(val, mine);
}

// flags8[tile*256 + lane] bit j  <=>  edge (tile*2048 + lane*8 + j) is the first edge of a new id
__global__ __launch_bounds__(kBlock) void idmap_mark_kernel(TableRef t, int64_t e_max, const int32_t* __restrict__ d_e,
                                                            int64_t n_base_h, const int32_t* __restrict__ d_n_base,
                                                            const uint32_t* __restrict__ slot_of,
                                                            uint8_t* __restrict__ flags8, int32_t* __restrict__ tile_sums)
{
    __shared__ int smem[kBlock / kWave + 1];
    const int64_t n_e = actual_count(e_max, d_e);
    const uint32_t n_base = d_n_base ? (uint32_t)(*d_n_base) : (uint32_t)n_base_h;
    const int64_t first = (int64_t)blockIdx.x * kTile + (int64_t)threadIdx.x * kItems;
    uint32_t bits = 0;
#pragma unroll
    for (int j = 0; j < kItems; ++j) {
        const int64_t e = first + j;
        if (e < n_e) {
            const uint32_t p = slot_of[e];
            if (p != kEmpty && t.words[2 * (size_t)p + 1] == n_base + (uint32_t)e) bits |= 1u << j;
        }
    }
    flags8[(int64_t)blockIdx.x * kBlock + threadIdx.x] = (uint8_t)bits;
    int total;
    (void)block_exclusive_scan<kBlock>(__popc(bits), smem, &total);
    if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// n_total = n_base + (number of new ids), clamped to the capacity of the unique list
__global__ void idmap_publish_total_kernel(const int32_t* __restrict__ new_count, int64_t n_base_h,
                                           const int32_t* __restrict__ d_n_base, int64_t capacity,
                                           int32_t* __restrict__ d_n_total_out, uint32_t* __restrict__ d_status)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const int64_t n_base = d_n_base ? (int64_t)(*d_n_base) : n_base_h;
    int64_t total = n_base + (int64_t)(*new_count);
    if (total > capacity) {
        if (d_status) atomicOr(d_status, FGL_STATUS_UNIQ_OVERFLOW);
        total = capacity;
    }
    if (d_n_total_out) *d_n_total_out = (int32_t)total;
}

__global__ __launch_bounds__(kBlock) void idmap_assign_kernel(TableRef t, const int32_t* __restrict__ src, int64_t e_max,
                                                              const int32_t* __restrict__ d_e, int64_t n_base_h,
                                                              const int32_t* __restrict__ d_n_base,
                                                              const uint32_t* __restrict__ slot_of,
                                                              const uint8_t* __restrict__ flags8,
                                                              const int32_t* __restrict__ tile_prefix,
                                                              int32_t* __restrict__ uniq, int64_t capacity)
{
    __shared__ int smem[kBlock / kWave + 1];
    const int64_t n_e = actual_count(e_max, d_e);
    const int64_t n_base = d_n_base ? (int64_t)(*d_n_base) : n_base_h;
    const int64_t first = (int64_t)blockIdx.x * kTile + (int64_t)threadIdx.x * kItems;
    const uint32_t bits = first < n_e ? flags8[(int64_t)blockIdx.x * kBlock + threadIdx.x] : 0u;
    int total;
    int64_t local = n_base + tile_prefix[blockIdx.x] + block_exclusive_scan<kBlock>(__popc(bits), smem, &total);
#pragma unroll
    for (int j = 0; j < kItems; ++j) {
        if (bits & (1u << j)) {
            const int64_t e = first + j;
            if (local < capacity) {
                t.words[2 * (size_t)slot_of[e] + 1] = (uint32_t)local;
                uniq[local] = src[e];
            }
            ++local;
        }
    }
}

__global__ __launch_bounds__(kBlock) void idmap_relabel_kernel(TableRef t, int64_t e_max, const int32_t* __restrict__ d_e,
                                                               const uint32_t* __restrict__ slot_of,
                                                               int32_t* __restrict__ out)
{
    const int64_t n_e = actual_count(e_max, d_e);
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_e) return;
    const uint32_t p = slot_of[e];
    out[e] = p == kEmpty ? -1 : (int32_t)t.words[2 * (size_t)p + 1];
}

__global__ __launch_bounds__(kBlock) void idmap_lookup_kernel(TableRef t, int32_t* __restrict__ ids, int64_t n_max,
                                                              const int32_t* __restrict__ d_n, uint32_t* __restrict__ d_status)
{
    const int64_t n = actual_count(n_max, d_n);
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const uint32_t p = find_only(t.words, t.mask, t.shift, (uint32_t)ids[i]);
    if (p == kEmpty) {
        if (d_status) atomicOr(d_status, FGL_STATUS_MISSING_KEY);
        ids[i] = -1;
    } else {
        ids[i] = (int32_t)t.words[2 * (size_t)p + 1];
    }
}

// ---- launchers ------------------------------------------------------------------
int launch_idmap_reset(void* d_table, int64_t slots, hipStream_t stream)
{
    FGL_REQUIRE(d_table != nullptr && valid_slots(slots), "idmap: slot count %lld is not a power of two in [64, 2^31]", (long long)slots);
    return launch_fill_u32(static_cast<uint32_t*>(d_table), slots * 2, kEmpty, stream);
}

int launch_idmap_insert_dst(void* d_table, int64_t slots, const int32_t* d_dst_ids, int64_t n_max, const int32_t* d_n,
                            int32_t* d_uniq, uint32_t* d_status, hipStream_t stream)
{
    FGL_REQUIRE(d_table != nullptr && valid_slots(slots), "idmap: slot count %lld is not a power of two in [64, 2^31]", (long long)slots);
    FGL_REQUIRE(n_max >= 0 && n_max <= slots / 2, "idmap_insert_dst: %lld ids do not fit %lld slots at load 1/2", (long long)n_max, (long long)slots);
    if (n_max == 0) return FGL_OK;
    FGL_REQUIRE(d_dst_ids != nullptr, "idmap_insert_dst: null ids");
    const int64_t blocks = ceil_div(n_max, kBlock);
    hipLaunchKernelGGL(idmap_insert_dst_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, make_ref(d_table, slots),
                       d_dst_ids, n_max, d_n, d_uniq, d_status);
    FGL_CHECK_LAUNCH("idmap_insert_dst_kernel");
    return FGL_OK;
}

size_t idmap_map_src_workspace_bytes(int64_t n_edges_max)
{
    const int64_t tiles = ceil_div(n_edges_max > 0 ? n_edges_max : 1, kTile);
    Carver c(nullptr);
    c.take<uint32_t>((size_t)n_edges_max);      // slot_of
    c.take<uint8_t>((size_t)tiles * kBlock);    // flags8
    c.take<int32_t>((size_t)tiles);             // tile sums
    c.take<int32_t>((size_t)tiles);             // tile prefix
    c.take<int32_t>(1);                         // new id count
    return c.used();
}

int launch_idmap_map_src(void* d_table, int64_t slots, const int32_t* d_src_in, int32_t* d_src_out, int64_t n_edges_max,
                         const int32_t* d_n_edges, int64_t n_base, const int32_t* d_n_base, int32_t* d_n_total_out,
                         int32_t* d_uniq, int64_t uniq_capacity, int flags, uint32_t* d_status, void* d_ws,
                         size_t ws_bytes, hipStream_t stream)
{
    FGL_REQUIRE(d_table != nullptr && valid_slots(slots), "idmap: slot count %lld is not a power of two in [64, 2^31]", (long long)slots);
    FGL_REQUIRE(flags == FGL_IDMAP_ORDERED, "idmap_map_src: unknown flags %d", flags);
    FGL_REQUIRE(n_edges_max >= 0 && n_base >= 0 && uniq_capacity >= 0, "idmap_map_src: negative size");
    FGL_REQUIRE(n_base + n_edges_max <= 0xFFFFFFFEll, "idmap_map_src: n_base + n_edges exceeds 32 bits");
    FGL_REQUIRE(uniq_capacity <= slots / 2, "idmap_map_src: %lld unique ids do not fit %lld slots at load 1/2", (long long)uniq_capacity, (long long)slots);
    FGL_REQUIRE(n_edges_max == 0 || (d_src_in && d_src_out && d_uniq), "idmap_map_src: null pointer");
    FGL_REQUIRE(d_n_total_out == nullptr || d_n_total_out != d_n_base, "idmap_map_src: n_total_out must not alias n_base");
    if (d_ws == nullptr || ws_bytes < idmap_map_src_workspace_bytes(n_edges_max)) {
        set_error("idmap_map_src: workspace too small (%zu < %zu)", ws_bytes, idmap_map_src_workspace_bytes(n_edges_max));
        return FGL_ERR_WORKSPACE;
    }
    const int64_t tiles = ceil_div(n_edges_max > 0 ? n_edges_max : 1, kTile);
    Carver c(d_ws);
    uint32_t* slot_of = c.take<uint32_t>((size_t)n_edges_max);
    uint8_t* flags8 = c.take<uint8_t>((size_t)tiles * kBlock);
    int32_t* sums = c.take<int32_t>((size_t)tiles);
    int32_t* prefix = c.take<int32_t>((size_t)tiles);
    int32_t* new_count = c.take<int32_t>(1);
    const TableRef t = make_ref(d_table, slots);
    const int64_t edge_blocks = ceil_div(n_edges_max > 0 ? n_edges_max : 1, kBlock);

    hipLaunchKernelGGL(idmap_insert_src_kernel, dim3((unsigned)edge_blocks), dim3(kBlock), 0, stream, t, d_src_in,
                       n_edges_max, d_n_edges, n_base, d_n_base, slot_of, d_status);
    FGL_CHECK_LAUNCH("idmap_insert_src_kernel");
    hipLaunchKernelGGL(idmap_mark_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream, t, n_edges_max, d_n_edges, n_base,
                       d_n_base, slot_of, flags8, sums);
    FGL_CHECK_LAUNCH("idmap_mark_kernel");
    int rc = launch_tile_prefix(sums, (int)tiles, prefix, new_count, nullptr, nullptr, 0, nullptr, stream);
    if (rc != FGL_OK) return rc;
    hipLaunchKernelGGL(idmap_publish_total_kernel, dim3(1), dim3(64), 0, stream, new_count, n_base, d_n_base, uniq_capacity,
                       d_n_total_out, d_status);
    FGL_CHECK_LAUNCH("idmap_publish_total_kernel");
    hipLaunchKernelGGL(idmap_assign_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream, t, d_src_in, n_edges_max,
                       d_n_edges, n_base, d_n_base, slot_of, flags8, prefix, d_uniq, uniq_capacity);
    FGL_CHECK_LAUNCH("idmap_assign_kernel");
    hipLaunchKernelGGL(idmap_relabel_kernel, dim3((unsigned)edge_blocks), dim3(kBlock), 0, stream, t, n_edges_max,
                       d_n_edges, slot_of, d_src_out);
    FGL_CHECK_LAUNCH("idmap_relabel_kernel");
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
    return launch_idmap_insert_dst(d_table, slots, d_dst_ids, n_max, d_n, d_uniq, d_status, as_stream(stream));
}

FGL_EXPORT size_t fgl_idmap_map_src_workspace_bytes(int64_t n_edges_max) { return idmap_map_src_workspace_bytes(n_edges_max < 0 ? 0 : n_edges_max); }

FGL_EXPORT int fgl_idmap_map_src(void* d_table, int64_t slots, const int32_t* d_src_in, int32_t* d_src_out,
                                 int64_t n_edges_max, const int32_t* d_n_edges, int64_t n_base, const int32_t* d_n_base,
                                 int32_t* d_n_total_out, int32_t* d_uniq, int64_t uniq_capacity, int flags,
                                 uint32_t* d_status, void* d_ws, size_t ws_bytes, void* stream)
{
    return launch_idmap_map_src(d_table, slots, d_src_in, d_src_out, n_edges_max, d_n_edges, n_base, d_n_base,
                                d_n_total_out, d_uniq, uniq_capacity, flags, d_status, d_ws, ws_bytes, as_stream(stream));
}

FGL_EXPORT int fgl_idmap_lookup(const void* d_table, int64_t slots, int32_t* d_ids, int64_t n_max, const int32_t* d_n,
                                uint32_t* d_status, void* stream)
{
    FGL_REQUIRE(d_table != nullptr && valid_slots(slots), "idmap: slot count %lld is not a power of two in [64, 2^31]", (long long)slots);
    FGL_REQUIRE(n_max >= 0, "idmap_lookup: negative size");
    if (n_max == 0) return FGL_OK;
    FGL_REQUIRE(d_ids != nullptr, "idmap_lookup: null ids");
    const int64_t blocks = ceil_div(n_max, kBlock);
    hipLaunchKernelGGL(idmap_lookup_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, as_stream(stream),
                       make_ref(const_cast<void*>(d_table), slots), d_ids, n_max, d_n, d_status);
    FGL_CHECK_LAUNCH("idmap_lookup_kernel");
    return FGL_OK;
}
