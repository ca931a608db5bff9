// CSR neighbour sampling without replacement (stands in for the reference's
// sample_node_cuda, cuda_operators/sample.cu:102-203).
//
// Three launches, no host synchronisation:
//   1. sample_degree_kernel   one lane per seed: two offsets of the row, k = min(fanout, deg),
//                             staged row start / degree, per-tile sum of k
//   2. tile prefix            single workgroup; also writes block_ptr[n] and the edge count
//   3. sample_edges_reg_kernel (fanout <= 32) / sample_edges_kernel (larger fanouts)
//                             per tile of TS seeds: wave64 scan of k -> output offsets,
//                             Floyd subset selection for rows longer than the fanout (one lane
//                             per seed, Philox stream keyed by the node id, picks kept in LDS in a
//                             conflict-free [pick][seed] layout),
//                             then a flat pass over the tile's output edges so that the
//                             src/dst writes are fully coalesced and the copy-all rows read
//                             `indices` contiguously.
// Launches 1 and 3 are grid-stride loops over the tiles the actual seed count occupies, so
// a host-side bound far above the actual count costs nothing.
#include <mutex>

#include "fgl_common.hpp"
#include "fgl_kernels.hpp"
#include "fgl_transpose_job.hpp"

// Scratch of fgl_sample_node_static: device memory that belongs to the library, one copy per GPU, held
// until the process ends.  In host code this name is only a handle for hipGetSymbolAddress -- it is
// not a device address and is never passed to a kernel or a memset; static_scratch() below resolves
// it once per device and everything else uses the pointer it returns.
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace fgl {

constexpr int64_t kStaticMaxSeeds = FGL_STATIC_MAX_SEEDS;  // 12.2 bytes of scratch per seed at most: fits 16 MiB
constexpr int kStaticMaxDevices = 64;

// The calling thread's current device's copy of `scratch` (each GPU holds its own at its own address).
static int static_scratch(void** out)
{
    static std::mutex mu;
    static void* ptr_of_device[kStaticMaxDevices] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kStaticMaxDevices) {
        set_error("sample_node_static: cannot name the current device (%s)", e != hipSuccess ? hipGetErrorString(e) : "index out of range");
        return FGL_ERR_HIP;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (ptr_of_device[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr) {
            set_error("sample_node_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return FGL_ERR_HIP;
        }
        ptr_of_device[dev] = p;
    }
    *out = ptr_of_device[dev];
    return FGL_OK;
}

template <int TS>
__global__ __launch_bounds__(TS) void sample_degree_kernel(const void* __restrict__ indptr, int is64, int64_t n_nodes,
                                                           const int32_t* __restrict__ seeds, int64_t n_max,
                                                           const int32_t* __restrict__ d_n, int fanout,
                                                           int64_t* __restrict__ row_start, int32_t* __restrict__ deg_out,
                                                           int32_t* __restrict__ tile_sums, uint32_t* __restrict__ d_status)
{
    __shared__ int smem[TS / kWave + 1];
    const int64_t n = actual_count(n_max, d_n);
    const int64_t n_tiles = (n + TS - 1) / TS;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t i = tile * TS + threadIdx.x;
        int k = 0;
        if (i < n) {
            const int64_t s = seeds[i];
            int64_t a = 0, deg = 0;
            if (s >= 0 && s < n_nodes) {
                if (is64) {
                    const int64_t* p = static_cast<const int64_t*>(indptr);
                    a = p[s];
                    deg = p[s + 1] - a;
                } else {
                    const int32_t* p = static_cast<const int32_t*>(indptr);
                    a = p[s];
                    deg = (int64_t)p[s + 1] - a;
                }
                if (deg < 0) deg = 0;
                if (deg > 0x7FFFFFFF) deg = 0x7FFFFFFF;
            } else if (d_status) {
                atomicOr(d_status, FGL_STATUS_BAD_SEED);
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

// Output offset of a tile of seeds.  With a prefix array (from the single-workgroup scan launch) it
// is one load.  Without one (tile_prefix == nullptr: the launcher skips that launch while the tile
// count is small) the workgroup sums the earlier tiles' sums itself, and the workgroup of the last
// tile also publishes the edge total: block_ptr[n] and *n_edges_out.
template <int TS>
__device__ __forceinline__ int tile_base(int lane_sum_of_earlier_tiles, const int32_t* __restrict__ tile_prefix, int64_t tile,
                                         int64_t n_tiles, int64_t n, int tile_total, int* smem,
                                         int32_t* __restrict__ block_ptr, int32_t* __restrict__ n_edges_out,
                                         int32_t* __restrict__ readback, const uint32_t* __restrict__ d_status)
{
    if (tile_prefix) return tile_prefix[tile];
    const int base = block_sum_of_lanes<TS>(lane_sum_of_earlier_tiles, smem);
    if (tile == n_tiles - 1 && threadIdx.x == 0) {
        block_ptr[n] = base + tile_total;
        if (n_edges_out) *n_edges_out = base + tile_total;
        if (readback) {  // (nothing in a launch that is handed a read-back pointer sets status bits: they are final)
            readback[0] = base + tile_total;
            readback[1] = d_status ? (int32_t)*d_status : 0;
        }
    }
    return base;
}

// The launch for zero seeds still has to publish the (empty) totals when no scan launch does.
__device__ __forceinline__ void publish_empty(const int32_t* __restrict__ tile_prefix, int64_t n_tiles,
                                              int32_t* __restrict__ block_ptr, int32_t* __restrict__ n_edges_out,
                                              int32_t* __restrict__ readback, const uint32_t* __restrict__ d_status)
{
    if (tile_prefix == nullptr && n_tiles == 0 && blockIdx.x == 0 && threadIdx.x == 0) {
        block_ptr[0] = 0;
        if (n_edges_out) *n_edges_out = 0;
        if (readback) {
            readback[0] = 0;
            readback[1] = d_status ? (int32_t)*d_status : 0;
        }
    }
}

// Two things the edges kernels do for every seed besides sampling it.
// (1) A negative row start is how the launch that prepared the seed's row start and degree (the first launch
// of a mini-batch, or the id-map pass that numbered the node) says that something was wrong with it; it
// is reported here, where the status word is no longer being initialised, and the seed gets no edges.
// (2) The seeds of this hop are also the first seeds of the next one (a hop's nodes are a prefix of the next
// hop's): their share of the next hop's per-tile edge counts, sum of min(next fanout, degree), is added
// here -- one integer atomic per wave, order-independent -- so that the next hop needs no pass of its own
// over degrees.  Call from uniform control flow (all lanes of the workgroup).
template <int TS>
__device__ __forceinline__ void seed_checks_and_next_hop(bool valid, int64_t tile, int64_t& row, int& deg,
                                                         uint32_t* __restrict__ d_status, int next_fanout,
                                                         int next_tile_seeds, int32_t* __restrict__ next_tile_sums)
{
    if (valid && row < 0) {
        if (d_status) atomicOr(d_status, row == kRowBadId ? FGL_STATUS_BAD_SEED : FGL_STATUS_TABLE_FULL);
        row = 0;
        deg = 0;
    }
    if (next_tile_sums != nullptr) {
        int kn = valid ? (deg < next_fanout ? deg : next_fanout) : 0;
#pragma unroll
        for (int d = kWave / 2; d >= 1; d >>= 1) kn += __shfl_xor(kn, d, kWave);
        // (tiles are multiples of the wave size: a wave's seeds lie in one tile of the next hop)
        if (lane_id() == 0 && kn != 0)
            atomicAdd(&next_tile_sums[(tile * TS + (int64_t)(threadIdx.x / kWave) * kWave) / next_tile_seeds], kn);
    }
}

template <int TS, int U>
__global__ __launch_bounds__(TS) void sample_edges_kernel(const int32_t* __restrict__ indices,
                                                          const int32_t* __restrict__ seeds, int64_t n_max,
                                                          const int32_t* __restrict__ d_n, int fanout,
                                                          const int64_t* __restrict__ row_start,
                                                          const int32_t* __restrict__ deg_arr,
                                                          const int32_t* __restrict__ tile_sums,
                                                          const int32_t* __restrict__ tile_prefix, uint32_t seed_lo,
                                                          uint32_t seed_hi, uint32_t stream_id,
                                                          const uint32_t* __restrict__ d_stream_add,
                                                          int32_t* __restrict__ src_out, int32_t* __restrict__ dst_out,
                                                          int32_t* __restrict__ block_ptr, int32_t* __restrict__ n_edges_out,
                                                          uint32_t* __restrict__ d_status, int next_fanout, int next_tile_seeds,
                                                          int32_t* __restrict__ next_tile_sums, uint8_t* __restrict__ zero_per_edge,
                                                          const TransposeSteps steps, int32_t* __restrict__ readback)
{
    extern __shared__ uint32_t s_sel[];  // [fanout][TS] picked positions
    __shared__ int s_scan[TS / kWave + 1];
    __shared__ int s_off[TS + 1];
    __shared__ int64_t s_row[TS];
    __shared__ int s_deg[TS];
    __shared__ int s_seed[TS];

    const int tid = (int)threadIdx.x;
    if (d_stream_add) stream_id += *d_stream_add;  // lets a captured launch sequence advance its random stream
    // work for the transposed blocks that this launch carries along (nothing in the per-hop operator)
    tjob_zero<TS>(steps.zero);
    tjob_tile_sums<TS>(steps.before);
    const int64_t n = actual_count(n_max, d_n);
    const int64_t n_tiles = (n + TS - 1) / TS;
    publish_empty(tile_prefix, n_tiles, block_ptr, n_edges_out, readback, d_status);
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t i = tile * TS + tid;
        int deg = 0, seed = 0;
        int64_t row = 0;
        if (i < n) {
            deg = deg_arr[i];
            row = row_start[i];
            seed = seeds[i];
        }
        // (the earlier tiles' sums are fetched while the seed's own three loads are still under way)
        const int sum_before = tile_prefix ? 0 : lane_sum_before<TS>(tile_sums, tile);
        seed_checks_and_next_hop<TS>(i < n, tile, row, deg, d_status, next_fanout, next_tile_seeds, next_tile_sums);
        const int k = deg < fanout ? deg : fanout;
        int total;
        const int ex = block_exclusive_scan<TS>(k, s_scan, &total);
        const int base = tile_base<TS>(sum_before, tile_prefix, tile, n_tiles, n, total, s_scan, block_ptr, n_edges_out, readback, d_status);
        s_off[tid] = ex;
        if (tid == 0) s_off[TS] = total;
        s_row[tid] = row;
        s_deg[tid] = deg;
        s_seed[tid] = seed;
        if (i < n) block_ptr[i] = base + ex;

        if (deg > fanout) {
            // Floyd: for j = deg-k .. deg-1 draw t in [0, j]; take t unless already taken, else j.
            uint32_t o[4];
            for (int m = 0; m < fanout; ++m) {
                if ((m & 1) == 0) philox4x32_10((uint32_t)seed, 0u, stream_id, (uint32_t)(m >> 1), seed_lo, seed_hi, o);
                const uint64_t r = (m & 1) ? ((uint64_t)o[2] | ((uint64_t)o[3] << 32)) : ((uint64_t)o[0] | ((uint64_t)o[1] << 32));
                const uint32_t j = (uint32_t)(deg - fanout + m);
                const uint32_t t = (uint32_t)__umul64hi(r, (uint64_t)j + 1u);
                bool dup = false;
                for (int q = 0; q < m; ++q) dup |= (s_sel[q * TS + tid] == t);
                s_sel[m * TS + tid] = dup ? j : t;
            }
        }
        __syncthreads();

        // flat pass over the tile's output edges, U independent gathers in flight per lane
        // (U * TS covers a whole tile for the common fanouts, so the pass is one round trip)
        for (int x0 = tid; x0 < total; x0 += U * TS) {
            int seed_of[U];
            int32_t got[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int x = x0 + u * TS;
                got[u] = 0;
                seed_of[u] = 0;
                if (x < total) {
                    int lo = 0, hi = TS;  // s_off[lo] <= x < s_off[hi]
                    while (hi - lo > 1) {
                        const int mid = (lo + hi) >> 1;
                        if (s_off[mid] <= x) lo = mid; else hi = mid;
                    }
                    const int j = x - s_off[lo];
                    const int64_t pos = s_deg[lo] <= fanout ? (int64_t)j : (int64_t)s_sel[j * TS + lo];
                    got[u] = indices[s_row[lo] + pos];
                    seed_of[u] = s_seed[lo];
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int x = x0 + u * TS;
                if (x < total) {
                    src_out[(int64_t)base + x] = got[u];
                    if (dst_out) dst_out[(int64_t)base + x] = seed_of[u];
                    if (zero_per_edge) zero_per_edge[(int64_t)base + x] = 0;
                }
            }
        }
        __syncthreads();  // the tile's LDS is reused by the next iteration
    }
}

// Variant for fanout <= F (F = 8, 16, 32): the picks live in registers (both Floyd loops are
// fully unrolled, so the membership test costs no LDS traffic), every lane issues all of its
// row reads at once (one memory round trip per tile), and the values are staged through LDS at
// their output offsets so that the global writes are one coalesced pass.
template <int TS, int F>
__global__ __launch_bounds__(TS) void sample_edges_reg_kernel(const int32_t* __restrict__ indices,
                                                              const int32_t* __restrict__ seeds, int64_t n_max,
                                                              const int32_t* __restrict__ d_n, int fanout,
                                                              const int64_t* __restrict__ row_start,
                                                              const int32_t* __restrict__ deg_arr,
                                                              const int32_t* __restrict__ tile_sums,
                                                              const int32_t* __restrict__ tile_prefix, uint32_t seed_lo,
                                                              uint32_t seed_hi, uint32_t stream_id,
                                                              const uint32_t* __restrict__ d_stream_add,
                                                              int32_t* __restrict__ src_out, int32_t* __restrict__ dst_out,
                                                              int32_t* __restrict__ block_ptr, int32_t* __restrict__ n_edges_out,
                                                              uint32_t* __restrict__ d_status, int next_fanout, int next_tile_seeds,
                                                              int32_t* __restrict__ next_tile_sums, uint8_t* __restrict__ zero_per_edge,
                                                              const TransposeSteps steps, int32_t* __restrict__ readback)
{
    extern __shared__ int32_t s_stage[];  // [TS*fanout] sampled ids (+ [TS*fanout] seed ids when dst_out is wanted)
    __shared__ int s_scan[TS / kWave + 1];
    int32_t* s_val = s_stage;
    int32_t* s_dst = s_stage + TS * fanout;

    const int tid = (int)threadIdx.x;
    if (d_stream_add) stream_id += *d_stream_add;  // lets a captured launch sequence advance its random stream
    // work for the transposed blocks that this launch carries along (nothing in the per-hop operator)
    tjob_zero<TS>(steps.zero);
    tjob_tile_sums<TS>(steps.before);
    const int64_t n = actual_count(n_max, d_n);
    const int64_t n_tiles = (n + TS - 1) / TS;
    publish_empty(tile_prefix, n_tiles, block_ptr, n_edges_out, readback, d_status);
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t i = tile * TS + tid;
        int deg = 0, seed = 0;
        int64_t row = 0;
        if (i < n) {
            deg = deg_arr[i];
            row = row_start[i];
            seed = seeds[i];
        }
        // (the earlier tiles' sums are fetched while the seed's own three loads are still under way)
        const int sum_before = tile_prefix ? 0 : lane_sum_before<TS>(tile_sums, tile);
        seed_checks_and_next_hop<TS>(i < n, tile, row, deg, d_status, next_fanout, next_tile_seeds, next_tile_sums);
        const int k = deg < fanout ? deg : fanout;
        int total;
        const int ex = block_exclusive_scan<TS>(k, s_scan, &total);
        const int base = tile_base<TS>(sum_before, tile_prefix, tile, n_tiles, n, total, s_scan, block_ptr, n_edges_out, readback, d_status);
        if (i < n) block_ptr[i] = base + ex;

        uint32_t sel[F];
#pragma unroll
        for (int m = 0; m < F; ++m) sel[m] = (uint32_t)m;  // deg <= fanout: the whole row, in CSR order
        if (deg > fanout) {
            // Floyd: for j = deg-k .. deg-1 draw t in [0, j]; take t unless already taken, else j.
            uint32_t o[4] = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int m = 0; m < F; ++m) {
                if (m < fanout) {
                    if ((m & 1) == 0) philox4x32_10((uint32_t)seed, 0u, stream_id, (uint32_t)(m >> 1), seed_lo, seed_hi, o);
                    const uint64_t r = (m & 1) ? ((uint64_t)o[2] | ((uint64_t)o[3] << 32)) : ((uint64_t)o[0] | ((uint64_t)o[1] << 32));
                    const uint32_t j = (uint32_t)(deg - fanout + m);
                    const uint32_t t = (uint32_t)__umul64hi(r, (uint64_t)j + 1u);
                    bool dup = false;
#pragma unroll
                    for (int q = 0; q < m; ++q) dup |= (sel[q] == t);
                    sel[m] = dup ? j : t;
                }
            }
        }
        int32_t v[F];
#pragma unroll
        for (int m = 0; m < F; ++m) v[m] = (m < k) ? indices[row + (int64_t)sel[m]] : 0;
#pragma unroll
        for (int m = 0; m < F; ++m)
            if (m < k) {
                s_val[ex + m] = v[m];
                if (dst_out) s_dst[ex + m] = seed;
            }
        __syncthreads();
        for (int x = tid; x < total; x += TS) {
            src_out[(int64_t)base + x] = s_val[x];
            if (dst_out) dst_out[(int64_t)base + x] = s_dst[x];
            if (zero_per_edge) zero_per_edge[(int64_t)base + x] = 0;
        }
        __syncthreads();  // the staging area is reused by the next tile
    }
}

// Seeds per workgroup of the sampling kernels.  Small hops take one wave per tile: a hop of a few ten thousand
// seeds is a chain of latencies, and 64-seed tiles spread it over four times the compute units.
#ifndef FGL_SMALL_HOP_SEEDS
#define FGL_SMALL_HOP_SEEDS 65536
#endif
int sample_tile_seeds(int fanout, int64_t n_seeds_max) { return (fanout <= 48 && n_seeds_max > FGL_SMALL_HOP_SEEDS) ? 256 : 64; }

int64_t sample_tile_count(int64_t n_seeds_max, int fanout)
{
    return ceil_div(n_seeds_max > 0 ? n_seeds_max : 1, sample_tile_seeds(fanout, n_seeds_max));
}

// Up to this many tiles of seeds the edges kernel derives its tile offsets itself (at most 16 KiB of
// tile sums per workgroup, read from L2); above it a scan launch prepares them.
constexpr int64_t kSampleSelfPrefixTiles = 4096;

size_t sample_workspace_bytes(int64_t n_seeds_max, int fanout)
{
    const int64_t tiles = sample_tile_count(n_seeds_max, fanout);
    Carver c(nullptr);
    c.take<int64_t>((size_t)n_seeds_max);
    c.take<int32_t>((size_t)n_seeds_max);
    c.take<int32_t>((size_t)tiles);
    c.take<int32_t>((size_t)tiles);
    return c.used();
}

template <int TS>
static int launch_edges_ts(const int32_t* d_indices, const int32_t* d_seeds, int64_t n_seeds_max, const int32_t* d_n_seeds,
                           int fanout, const int64_t* row_start, const int32_t* deg, const int32_t* sums, int32_t* prefix,
                           uint64_t rng_seed, uint32_t stream_id, int32_t* d_src_out, int32_t* d_dst_out,
                           int32_t* d_block_ptr, int32_t* d_n_edges_out, uint32_t* d_status, hipStream_t stream,
                           const uint32_t* d_stream_add, const NextHop* next, uint8_t* d_zero_per_edge,
                           const TransposeSteps* steps_in, int32_t* d_readback)
{
    const int64_t tiles = ceil_div(n_seeds_max > 0 ? n_seeds_max : 1, TS);
    unsigned grid = (unsigned)(tiles < 8192 ? tiles : 8192);
    TransposeSteps steps;
    memset(&steps, 0, sizeof(steps));
    if (steps_in) {
        steps = *steps_in;
        // the carried steps get workgroups of their own behind the sampling ones: clearing this hop's counters
        // (16 per lane), then the tile sums of the hop before
        if (steps.zero.cnt != nullptr) {
            steps.zero.side_first = 0;
            steps.zero.side_blocks = side_blocks_for(steps.zero.cols_max * steps.zero.split + 1, (int64_t)TS * 16);
            grid += (unsigned)steps.zero.side_blocks;
        }
        if (steps.before.cnt != nullptr) {
            steps.before.side_first = steps.zero.cnt != nullptr ? steps.zero.side_blocks : 0;
            steps.before.side_blocks = side_blocks_for(steps.before.cols_max * steps.before.split + 1, kTjobTile);
            grid += (unsigned)steps.before.side_blocks;
        }
    }
    // few tiles: each workgroup of the edges kernel sums the earlier tile sums itself (the last one
    // publishes the totals), which saves the scan launch in between
    if (tiles > kSampleSelfPrefixTiles) {
        int rc = launch_tile_prefix(sums, (int)tiles, prefix, d_n_edges_out, nullptr, d_block_ptr, n_seeds_max, d_n_seeds,
                                    TS, stream, d_readback, d_status);
        if (rc != FGL_OK) return rc;
    } else {
        prefix = nullptr;
    }
    const int next_fanout = next ? next->fanout : 0;
    const int next_ts = next ? next->tile_seeds : TS;
    int32_t* next_sums = next ? next->tile_sums : nullptr;
    // the register variant stages the tile's output (and, if wanted, the seed ids) in LDS: it is used
    // while that fits comfortably in the 64 KiB a workgroup may take
    const size_t lds_reg = (size_t)fanout * TS * sizeof(int32_t) * (d_dst_out ? 2 : 1);
    if (fanout <= 32 && lds_reg <= 60 * 1024) {
#define FGL_LAUNCH_REG(F)                                                                                           \
    hipLaunchKernelGGL((sample_edges_reg_kernel<TS, F>), dim3(grid), dim3(TS), lds_reg, stream, d_indices, d_seeds,   \
                       n_seeds_max, d_n_seeds, fanout, row_start, deg, sums, prefix, (uint32_t)rng_seed,                   \
                       (uint32_t)(rng_seed >> 32), stream_id, d_stream_add, d_src_out, d_dst_out, d_block_ptr, d_n_edges_out, \
                       d_status, next_fanout, next_ts, next_sums, d_zero_per_edge, steps, d_readback)
        if (fanout <= 8) FGL_LAUNCH_REG(8);
        else if (fanout <= 16) FGL_LAUNCH_REG(16);
        else FGL_LAUNCH_REG(32);
#undef FGL_LAUNCH_REG
        FGL_CHECK_LAUNCH("sample_edges_reg_kernel");
        return FGL_OK;
    }
    const size_t lds = (size_t)fanout * TS * sizeof(uint32_t);
    hipLaunchKernelGGL((sample_edges_kernel<TS, 16>), dim3(grid), dim3(TS), lds, stream, d_indices, d_seeds,
                       n_seeds_max, d_n_seeds, fanout, row_start, deg, sums, prefix, (uint32_t)rng_seed,
                       (uint32_t)(rng_seed >> 32), stream_id, d_stream_add, d_src_out, d_dst_out, d_block_ptr, d_n_edges_out,
                       d_status, next_fanout, next_ts, next_sums, d_zero_per_edge, steps, d_readback);
    FGL_CHECK_LAUNCH("sample_edges_kernel");
    return FGL_OK;
}

int launch_sample_edges(const int32_t* d_indices, const int32_t* d_seeds, int64_t n_seeds_max, const int32_t* d_n_seeds,
                        int fanout, const int64_t* row_start, const int32_t* deg, const int32_t* tile_sums,
                        int32_t* tile_prefix, uint64_t rng_seed, uint32_t stream_id, int32_t* d_src_out,
                        int32_t* d_dst_out, int32_t* d_block_ptr, int32_t* d_n_edges_out, uint32_t* d_status,
                        hipStream_t stream, const uint32_t* d_stream_add, const NextHop* next, uint8_t* d_zero_per_edge,
                        const TransposeSteps* steps, int32_t* d_readback)
{
    if (sample_tile_seeds(fanout, n_seeds_max) == 256)
        return launch_edges_ts<256>(d_indices, d_seeds, n_seeds_max, d_n_seeds, fanout, row_start, deg, tile_sums, tile_prefix,
                                    rng_seed, stream_id, d_src_out, d_dst_out, d_block_ptr, d_n_edges_out, d_status, stream,
                                    d_stream_add, next, d_zero_per_edge, steps, d_readback);
    return launch_edges_ts<64>(d_indices, d_seeds, n_seeds_max, d_n_seeds, fanout, row_start, deg, tile_sums, tile_prefix,
                               rng_seed, stream_id, d_src_out, d_dst_out, d_block_ptr, d_n_edges_out, d_status, stream,
                               d_stream_add, next, d_zero_per_edge, steps, d_readback);
}

int launch_sample(const void* d_indptr, int indptr_is64, const int32_t* d_indices, int64_t n_nodes,
                  const int32_t* d_seeds, int64_t n_seeds_max, const int32_t* d_n_seeds, int fanout,
                  uint64_t rng_seed, uint32_t stream_id, int32_t* d_src_out, int32_t* d_dst_out,
                  int32_t* d_block_ptr, int32_t* d_n_edges_out, uint32_t* d_status, void* d_ws, size_t ws_bytes,
                  hipStream_t stream, const uint32_t* d_stream_add, int32_t* d_readback)
{
    FGL_REQUIRE(n_seeds_max >= 0 && n_nodes >= 0, "sample_node: negative size");
    FGL_REQUIRE(fanout >= 1 && fanout <= FGL_MAX_FANOUT, "sample_node: fanout %d outside [1, %d]", fanout, FGL_MAX_FANOUT);
    FGL_REQUIRE(n_seeds_max * (int64_t)fanout <= 0x7FFFFFFF, "sample_node: %lld seeds x fanout %d overflows int32 edge offsets",
                (long long)n_seeds_max, fanout);
    FGL_REQUIRE(d_block_ptr != nullptr, "sample_node: null block_ptr");
    FGL_REQUIRE(n_seeds_max == 0 || (d_indptr && d_indices && d_seeds && d_src_out), "sample_node: null pointer");
    if (d_ws == nullptr || ws_bytes < sample_workspace_bytes(n_seeds_max, fanout)) {
        set_error("sample_node: workspace too small (%zu < %zu)", ws_bytes, sample_workspace_bytes(n_seeds_max, fanout));
        return FGL_ERR_WORKSPACE;
    }
    const int ts = sample_tile_seeds(fanout, n_seeds_max);
    const int64_t tiles = sample_tile_count(n_seeds_max, fanout);
    Carver c(d_ws);
    int64_t* row_start = c.take<int64_t>((size_t)n_seeds_max);
    int32_t* deg = c.take<int32_t>((size_t)n_seeds_max);
    int32_t* sums = c.take<int32_t>((size_t)tiles);
    int32_t* prefix = c.take<int32_t>((size_t)tiles);
    const unsigned grid = (unsigned)(tiles < 8192 ? tiles : 8192);
    if (ts == 256)
        hipLaunchKernelGGL(sample_degree_kernel<256>, dim3(grid), dim3(256), 0, stream, d_indptr, indptr_is64, n_nodes, d_seeds,
                           n_seeds_max, d_n_seeds, fanout, row_start, deg, sums, d_status);
    else
        hipLaunchKernelGGL(sample_degree_kernel<64>, dim3(grid), dim3(64), 0, stream, d_indptr, indptr_is64, n_nodes, d_seeds,
                           n_seeds_max, d_n_seeds, fanout, row_start, deg, sums, d_status);
    FGL_CHECK_LAUNCH("sample_degree_kernel");
    return launch_sample_edges(d_indices, d_seeds, n_seeds_max, d_n_seeds, fanout, row_start, deg, sums, prefix, rng_seed,
                               stream_id, d_src_out, d_dst_out, d_block_ptr, d_n_edges_out, d_status, stream, d_stream_add,
                               nullptr, nullptr, nullptr, d_readback);
}

}  // namespace fgl

using namespace fgl;

FGL_EXPORT size_t fgl_sample_workspace_bytes(int64_t n_seeds_max, int fanout)
{
    if (n_seeds_max < 0 || fanout < 1) return 0;
    return sample_workspace_bytes(n_seeds_max, fanout);
}

FGL_EXPORT int fgl_sample_node(const void* d_indptr, int indptr_is64, const int32_t* d_indices, int64_t n_nodes,
                               const int32_t* d_seeds, int64_t n_seeds_max, const int32_t* d_n_seeds, int fanout,
                               uint64_t rng_seed, uint32_t stream_id, int32_t* d_src_out, int32_t* d_dst_out,
                               int32_t* d_block_ptr, int32_t* d_n_edges_out, uint32_t* d_status, int32_t* d_readback,
                               void* d_ws, size_t ws_bytes, void* stream)
{
    return launch_sample(d_indptr, indptr_is64, d_indices, n_nodes, d_seeds, n_seeds_max, d_n_seeds, fanout, rng_seed,
                         stream_id, d_src_out, d_dst_out, d_block_ptr, d_n_edges_out, d_status, d_ws, ws_bytes,
                         as_stream(stream), nullptr, d_readback);
}

FGL_EXPORT int fgl_sample_node_static(const void* d_indptr, int indptr_is64, const int32_t* d_indices, int64_t n_nodes,
                                      const int32_t* d_seeds, int64_t n_seeds_max, const int32_t* d_n_seeds, int fanout,
                                      uint64_t rng_seed, uint32_t stream_id, int32_t* d_src_out, int32_t* d_dst_out,
                                      int32_t* d_block_ptr, int32_t* d_n_edges_out, uint32_t* d_status, void* stream)
{
    FGL_REQUIRE(n_seeds_max >= 0 && n_seeds_max <= kStaticMaxSeeds,
                "sample_node_static: %lld seeds outside [0, %lld] (the library's own scratch holds no more; "
                "use fgl_sample_node with a caller workspace)", (long long)n_seeds_max, (long long)kStaticMaxSeeds);
    FGL_REQUIRE(fanout >= 1 && fanout <= FGL_MAX_FANOUT, "sample_node_static: fanout %d outside [1, %d]", fanout, FGL_MAX_FANOUT);
    const size_t need = sample_workspace_bytes(n_seeds_max, fanout);
    FGL_REQUIRE(need <= kStaticScratchBytes, "sample_node_static: needs %zu bytes of scratch, the library holds %zu", need,
                kStaticScratchBytes);
    void* ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc != FGL_OK) return rc;
    // (nothing in the scratch has to start at zero: the degree pass writes every entry the edges pass reads)
    return launch_sample(d_indptr, indptr_is64, d_indices, n_nodes, d_seeds, n_seeds_max, d_n_seeds, fanout, rng_seed,
                         stream_id, d_src_out, d_dst_out, d_block_ptr, d_n_edges_out, d_status, ws, kStaticScratchBytes,
                         as_stream(stream));
}
