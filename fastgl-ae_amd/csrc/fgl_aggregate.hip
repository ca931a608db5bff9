// Memory-aware row aggregation over a block CSR, and the block transpose that lets the
// backward pass run as the same gather (stands in for the reference's forward kernels,
// cuda_operators/aggregate_acc_kernel.cu:270-331,375-427, and -- on the transposed block --
// for its atomic-scatter backward kernels, :467-517,554-596).
//
// Mapping: one LPR-lane group per (output row, column slice); LPR in {8,16,32,64} is the
// smallest power of two that covers the row with one 16-byte (or narrower, if the row
// length or stride forbids it) vector load per lane, so a 128-float row is one
// global_load_dwordx4 from each of 32 lanes and a wave streams two rows at a time.  The
// group's lanes first load up to LPR neighbour ids (and their per-edge weights) in one
// coalesced read, then broadcast them lane by lane; the row loads are issued four at a
// time before the first FMA so that each lane keeps several 16-byte loads in flight.
// Accumulation is fp32, in CSR order, in registers: no shared-memory read-modify-write
// and no redundant staging of the id list as in the reference kernel.
//
// Rows of more than 128 entries (hubs of a transposed block; none in a sampled block) are left to a
// second launch, aggregate_long_rows_kernel, in which a whole 512-lane workgroup sums one row; the
// caller's knowledge of the longest row decides whether that launch is enqueued at all.
#include "fgl_common.hpp"
#include "fgl_kernels.hpp"

namespace fgl {


// ---- vector load / store of VEC elements as fp32 -----------------------------------
// Rows are moved with one 16-byte access per lane.  The vector types are declared with
// 4-byte alignment: rows whose length is not a multiple of the vector (602 floats = 2408
// bytes) start on 8- or 4-byte boundaries, and gfx950 global loads/stores of any width only
// need dword alignment.  The last lane of a row whose length is not a multiple of VEC uses
// the element-wise partial forms.
template <typename T, int VEC>
struct RowIO;

template <>
struct RowIO<float, 4> {
    typedef float Raw __attribute__((ext_vector_type(4), aligned(4)));
    static __device__ __forceinline__ Raw load(const float* p) { return *reinterpret_cast<const Raw*>(p); }
    static __device__ __forceinline__ Raw load_partial(const float* p, int n)
    {
        Raw r = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < 3; ++i)
            if (i < n) r[i] = p[i];
        return r;
    }
    static __device__ __forceinline__ void fma(float (&acc)[4], float w, Raw r)
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += w * r[i];
    }
    static __device__ __forceinline__ void store(float* p, const float (&acc)[4])
    {
        Raw r = {acc[0], acc[1], acc[2], acc[3]};
        *reinterpret_cast<Raw*>(p) = r;
    }
    static __device__ __forceinline__ void store_partial(float* p, const float (&acc)[4], int n)
    {
#pragma unroll
        for (int i = 0; i < 3; ++i)
            if (i < n) p[i] = acc[i];
    }
};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
// Two floats to two bf16 in one 32-bit word (round to nearest even; low half = a): gfx950 has an instruction
// for it, v_cvt_pk_bf16_f32, which the compiler emits for this vector conversion.  A wave64 ALU instruction
// occupies its SIMD for four cycles, so the dozen integer operations of a hand-written rounding per element
// were what bounded the bf16 kernels on short rows, not memory.
typedef __bf16 Bf16x2 __attribute__((ext_vector_type(2)));
typedef float Float2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float a, float b)
{
    const Float2 f = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, Bf16x2));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return f32x2_to_bf16x2_bits(f, 0.0f) & 0xFFFFu; }

// bf16: eight elements per lane as four 32-bit words (rows must start on 4-byte boundaries)
template <>
struct RowIO<uint16_t, 8> {
    typedef uint32_t Raw __attribute__((ext_vector_type(4), aligned(4)));
    static __device__ __forceinline__ Raw load(const uint16_t* p) { return *reinterpret_cast<const Raw*>(p); }
    static __device__ __forceinline__ Raw load_partial(const uint16_t* p, int n)
    {
        Raw r = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < 7; ++i)
            if (i < n) r[i >> 1] |= (uint32_t)p[i] << ((i & 1) * 16);
        return r;
    }
    static __device__ __forceinline__ void fma(float (&acc)[8], float w, Raw r)
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] += w * __uint_as_float(r[i] << 16);
            acc[2 * i + 1] += w * __uint_as_float(r[i] & 0xFFFF0000u);
        }
    }
    static __device__ __forceinline__ void store(uint16_t* p, const float (&acc)[8])
    {
        Raw r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = f32x2_to_bf16x2_bits(acc[2 * i], acc[2 * i + 1]);
        *reinterpret_cast<Raw*>(p) = r;
    }
    static __device__ __forceinline__ void store_partial(uint16_t* p, const float (&acc)[8], int n)
    {
#pragma unroll
        for (int i = 0; i < 7; ++i)
            if (i < n) p[i] = (uint16_t)f32_to_bf16_bits(acc[i]);
    }
};
// bf16 rows that start on odd element boundaries: one element per lane
template <>
struct RowIO<uint16_t, 1> {
    using Raw = uint16_t;
    static __device__ __forceinline__ Raw load(const uint16_t* p) { return *p; }
    static __device__ __forceinline__ Raw load_partial(const uint16_t* p, int) { return *p; }
    static __device__ __forceinline__ void fma(float (&acc)[1], float w, Raw r) { acc[0] += w * bf16_bits_to_f32(r); }
    static __device__ __forceinline__ void store(uint16_t* p, const float (&acc)[1]) { *p = (uint16_t)f32_to_bf16_bits(acc[0]); }
    static __device__ __forceinline__ void store_partial(uint16_t* p, const float (&acc)[1], int) { store(p, acc); }
};

// Everything one launch needs.  T-typed pointers are kept as void* so that one struct serves
// both element types.
struct AggArgs {
    const int32_t* indptr;
    const int32_t* indices;
    int64_t n_rows_max;
    const int32_t* d_n_rows;
    const void* x;
    int64_t ldx;
    int D;
    int zero_policy;
    const int32_t* row_norm;
    const int32_t* col_norm;
    void* out;
    int64_t ldo;
    // FGL_AGG_EDGE only: per-entry, per-head weights w[entry_id * n_heads + head(column)]
    const float* edge_w;
    const int32_t* edge_index;  // entry -> entry_id (NULL: the entry's own position)
    const int32_t* longest_row; // device: entry count of the longest row, if the caller has it (NULL: unknown)
    int skip_rows_longer_than;  // aggregate_kernel leaves rows with more entries to aggregate_long_rows_kernel
    int n_heads;
    int unit_dim;               // D / n_heads
    int col_norm_is_ptr;        // FGL_AGG_COLMEAN: col_norm is an offsets array, the counts are its differences
};

// per-edge weight, evaluated by the lane that loaded the neighbour id
template <int MODE>
__device__ __forceinline__ float edge_weight(int col, float row_factor, const int32_t* __restrict__ col_norm, int col_norm_is_ptr)
{
    if (MODE == FGL_AGG_GCN) return row_factor * (1.0f / sqrtf((float)col_norm[col]));
    if (MODE == FGL_AGG_COLMEAN) {
        // (the columns' entry counts, or the offsets array they are the differences of)
        const int c = col_norm_is_ptr ? col_norm[col + 1] - col_norm[col] : col_norm[col];
        return 1.0f / (float)(c > 1 ? c : 1);
    }
    return row_factor;  // SUM: 1, MEAN: 1/deg(row)
}

// The last lane of a row whose length is not a multiple of VEC can move the row's last VEC columns
// instead of a cut-off vector when that address is dword-aligned: it overlaps its neighbour, both
// compute the same sums for the shared columns (same entries, same order) and store the same bits.
// Then no lane of the launch needs the element-wise path, which otherwise every wave that holds a
// row's last lane pays for on every load (602 bf16 columns: 59.6 -> 44.5 us on 8192 x 25 rows).
template <typename T, int VEC>
__host__ __device__ __forceinline__ bool tail_overlaps(int D)
{
    return D % VEC != 0 && D >= VEC && ((D - VEC) * (int)sizeof(T)) % 4 == 0;
}
// every live lane moves whole vectors
template <typename T, int VEC>
__host__ __device__ __forceinline__ bool all_lanes_full(int D)
{
    return D % VEC == 0 || tail_overlaps<T, VEC>(D);
}

// A lane's share of a row: VEC consecutive columns starting at col0 (possibly cut off by the row's end,
// or moved back to end with the row, see tail_overlaps).
template <typename T, int VEC>
struct LaneSlice {
    using IO = RowIO<T, VEC>;
    int col0;
    int nvalid;  // elements of this lane's vector that exist in the row
    bool live;
    bool full;   // false only for the last lane of a row with D % VEC != 0
    __device__ __forceinline__ LaneSlice(int slice, int lanes, int gl, int D)
    {
        col0 = (slice * lanes + gl) * VEC;
        nvalid = D - col0;
        live = nvalid > 0;
        full = nvalid >= VEC;
        if (live && !full && tail_overlaps<T, VEC>(D)) {
            col0 = D - VEC;
            nvalid = VEC;
            full = true;
        }
    }
    __device__ __forceinline__ typename IO::Raw load(const T* p) const { return full ? IO::load(p) : IO::load_partial(p, nvalid); }
    // ALL_FULL: the row length is a multiple of VEC, so every live lane moves a whole vector -- the caller
    // has tested that once for the launch, and the loads carry no per-lane branch
    template <bool ALL_FULL>
    __device__ __forceinline__ typename IO::Raw load_row(const T* p) const
    {
        if (ALL_FULL) return IO::load(p);
        return load(p);
    }
    __device__ __forceinline__ void store(T* p, const float (&a)[VEC]) const
    {
        if (full) IO::store(p, a);
        else IO::store_partial(p, a, nvalid);
    }
};

// part += the weighted rows of one chunk of at most LPR entries, whose ids and weights the group's lanes hold
// (lane t: entry t).  Four row loads are issued before the first FMA; the tail of the list goes together as well
// (measured: longer or predicated unrolls gain nothing on long lists and lose up to 2x on the one- and two-entry
// lists of a transposed block).
template <typename T, int VEC, int LPR, bool ALL_FULL>
__device__ __forceinline__ void accumulate_chunk(const LaneSlice<T, VEC>& ls, const T* __restrict__ X, int64_t ldx, int my_col,
                                                 float my_w, int cnt, float (&part)[VEC])
{
    using IO = RowIO<T, VEC>;
    const int col0 = ls.col0;
    const bool live = ls.live;
    int t = 0;
    for (; t + 4 <= cnt; t += 4) {
        const int c0 = __shfl(my_col, t, LPR), c1 = __shfl(my_col, t + 1, LPR);
        const int c2 = __shfl(my_col, t + 2, LPR), c3 = __shfl(my_col, t + 3, LPR);
        const float w0 = __shfl(my_w, t, LPR), w1 = __shfl(my_w, t + 1, LPR);
        const float w2 = __shfl(my_w, t + 2, LPR), w3 = __shfl(my_w, t + 3, LPR);
        if (live) {
            const typename IO::Raw r0 = ls.template load_row<ALL_FULL>(X + (int64_t)c0 * ldx + col0);
            const typename IO::Raw r1 = ls.template load_row<ALL_FULL>(X + (int64_t)c1 * ldx + col0);
            const typename IO::Raw r2 = ls.template load_row<ALL_FULL>(X + (int64_t)c2 * ldx + col0);
            const typename IO::Raw r3 = ls.template load_row<ALL_FULL>(X + (int64_t)c3 * ldx + col0);
            IO::fma(part, w0, r0);
            IO::fma(part, w1, r1);
            IO::fma(part, w2, r2);
            IO::fma(part, w3, r3);
        }
    }
    // the last one to three entries: their loads are issued together as well (most lists of a
    // transposed block have only this tail)
    const int rem = cnt - t;
    if (rem > 0) {
        const int c0 = __shfl(my_col, t, LPR);
        const int c1 = __shfl(my_col, rem > 1 ? t + 1 : t, LPR);
        const int c2 = __shfl(my_col, rem > 2 ? t + 2 : t, LPR);
        const float w0 = __shfl(my_w, t, LPR);
        const float w1 = __shfl(my_w, rem > 1 ? t + 1 : t, LPR);
        const float w2 = __shfl(my_w, rem > 2 ? t + 2 : t, LPR);
        if (live) {
            const typename IO::Raw r0 = ls.template load_row<ALL_FULL>(X + (int64_t)c0 * ldx + col0);
            typename IO::Raw r1 = r0, r2 = r0;
            if (rem > 1) r1 = ls.template load_row<ALL_FULL>(X + (int64_t)c1 * ldx + col0);
            if (rem > 2) r2 = ls.template load_row<ALL_FULL>(X + (int64_t)c2 * ldx + col0);
            IO::fma(part, w0, r0);
            if (rem > 1) IO::fma(part, w1, r1);
            if (rem > 2) IO::fma(part, w2, r2);
        }
    }
}

// acc += sum over the entries [a, b) of one row (a < b), all modes except FGL_AGG_EDGE.
// first_col (optional): the ids of the row's first chunk, already loaded (lane t: entry a + t).
template <typename T, int VEC, int LPR, int MODE, bool ALL_FULL>
__device__ __forceinline__ void gather_row(const AggArgs& g, const LaneSlice<T, VEC>& ls, int gl, int64_t row, int a, int b,
                                           float (&acc)[VEC], const int* first_col = nullptr)
{
    const int32_t* __restrict__ indices = g.indices;
    const T* __restrict__ X = static_cast<const T*>(g.x);
    float row_factor = 1.0f;
    if (MODE == FGL_AGG_MEAN) row_factor = 1.0f / (float)(b - a);
    if (MODE == FGL_AGG_GCN) row_factor = 1.0f / sqrtf((float)g.row_norm[row]);

    for (int base = a; base < b; base += LPR) {
        const int cnt = (b - base) < LPR ? (b - base) : LPR;
        int my_col = 0;
        float my_w = 0.0f;
        if (gl < cnt) {
            my_col = (first_col != nullptr && base == a) ? *first_col : indices[base + gl];
            my_w = edge_weight<MODE>(my_col, row_factor, g.col_norm, g.col_norm_is_ptr);
        }
        // Two-level summation: each chunk of LPR entries is summed on its own and then added to
        // the row total, so the rounding error of a row with thousands of entries (a hub in a
        // transposed block) grows like LPR + n/LPR instead of n.  Rows of at most LPR entries --
        // every sampled block -- are summed in plain CSR order.
        float part[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) part[i] = 0.0f;
        accumulate_chunk<T, VEC, LPR, ALL_FULL>(ls, X, g.ldx, my_col, my_w, cnt, part);
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] += part[i];
    }
}

// acc += sum over the entries [a, b) of one row (a < b) with per-entry, per-head weights (FGL_AGG_EDGE).
template <typename T, int VEC, int LPR>
__device__ __forceinline__ void gather_row_edge(const AggArgs& g, const LaneSlice<T, VEC>& ls, int gl, int a, int b,
                                                float (&acc)[VEC])
{
    using IO = RowIO<T, VEC>;
    const int32_t* __restrict__ indices = g.indices;
    const T* __restrict__ X = static_cast<const T*>(g.x);
    const int64_t ldx = g.ldx;
    const int D = g.D;
    const int col0 = ls.col0;
    const bool live = ls.live;
    // attention-style weights: one float per (entry, head); a lane's VEC columns lie in one
    // head when unit_dim is a multiple of VEC, else each column looks its head up
    const float* __restrict__ ew = g.edge_w;
    const int H = g.n_heads, unit = g.unit_dim;
    const bool one_head = (unit % VEC) == 0;
    int head[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        const int c = col0 + i < D ? col0 + i : D - 1;
        head[i] = c / unit;
    }
    for (int base = a; base < b; base += LPR) {
        const int cnt = (b - base) < LPR ? (b - base) : LPR;
        int my_col = 0, my_eid = 0;
        if (gl < cnt) {
            my_col = indices[base + gl];
            my_eid = g.edge_index ? g.edge_index[base + gl] : base + gl;
        }
        float part[VEC];  // this chunk's sum (see the note on two-level summation in gather_row)
#pragma unroll
        for (int i = 0; i < VEC; ++i) part[i] = 0.0f;
        int t = 0;
        if (one_head) {
            // as in gather_row: four row loads -- and the four weights that go with them -- are issued
            // before the first FMA
            for (; t + 4 <= cnt; t += 4) {
                const int c0 = __shfl(my_col, t, LPR), c1 = __shfl(my_col, t + 1, LPR);
                const int c2 = __shfl(my_col, t + 2, LPR), c3 = __shfl(my_col, t + 3, LPR);
                const int64_t e0 = __shfl(my_eid, t, LPR), e1 = __shfl(my_eid, t + 1, LPR);
                const int64_t e2 = __shfl(my_eid, t + 2, LPR), e3 = __shfl(my_eid, t + 3, LPR);
                if (live) {
                    const typename IO::Raw r0 = ls.load(X + (int64_t)c0 * ldx + col0);
                    const typename IO::Raw r1 = ls.load(X + (int64_t)c1 * ldx + col0);
                    const typename IO::Raw r2 = ls.load(X + (int64_t)c2 * ldx + col0);
                    const typename IO::Raw r3 = ls.load(X + (int64_t)c3 * ldx + col0);
                    const float w0 = ew[e0 * H + head[0]], w1 = ew[e1 * H + head[0]];
                    const float w2 = ew[e2 * H + head[0]], w3 = ew[e3 * H + head[0]];
                    IO::fma(part, w0, r0);
                    IO::fma(part, w1, r1);
                    IO::fma(part, w2, r2);
                    IO::fma(part, w3, r3);
                }
            }
        }
        for (; t < cnt; ++t) {
            const int c0 = __shfl(my_col, t, LPR);
            const int64_t e0 = __shfl(my_eid, t, LPR);
            if (live) {
                const typename IO::Raw r0 = ls.load(X + (int64_t)c0 * ldx + col0);
                if (one_head) {
                    IO::fma(part, ew[e0 * H + head[0]], r0);
                } else {
                    float x[VEC];
#pragma unroll
                    for (int i = 0; i < VEC; ++i) x[i] = 0.0f;
                    IO::fma(x, 1.0f, r0);
#pragma unroll
                    for (int i = 0; i < VEC; ++i) part[i] += ew[e0 * H + head[i]] * x[i];
                }
            }
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] += part[i];
    }
}

// A list with more entries than this is left to aggregate_long_rows_kernel when the caller cannot rule
// such lists out: a hub of a transposed block can hold thousands of entries, the one lane group that
// walks a list here would outlast the rest of the launch, and hubs sit next to each other.  (Measured on
// the transposed outer block of a 2.4 M-node graph, 256 floats per row: 432 us with every list walked
// here, 250 us with lists beyond 256 entries handed over, less with 128.)  Sampled blocks stay below it
// for fanouts up to 128.
constexpr int kLongRowEntries = 128;

template <typename T, int VEC, int LPR, int MODE>
__global__ __launch_bounds__(kBlock) void aggregate_kernel(const AggArgs g)
{
    using IO = RowIO<T, VEC>;
    constexpr int kGroups = kBlock / LPR;
    const int32_t* __restrict__ indptr = g.indptr;
    const T* __restrict__ X = static_cast<const T*>(g.x);
    T* __restrict__ out = static_cast<T*>(g.out);
    const int64_t ldx = g.ldx, ldo = g.ldo;
    const int D = g.D;

    const int64_t n_rows = actual_count(g.n_rows_max, g.d_n_rows);
    const int gl = (int)threadIdx.x % LPR;  // lane within the group
    const int64_t row = (int64_t)blockIdx.x * kGroups + (int)threadIdx.x / LPR;
    if (row >= n_rows) return;  // uniform per group: the cross-lane reads below stay inside the group
    const LaneSlice<T, VEC> ls((int)blockIdx.y, LPR, gl, D);
    const int col0 = ls.col0;
    const bool live = ls.live;

    const int a = indptr[row], b = indptr[row + 1];
    {
        // rows left to aggregate_long_rows_kernel -- unless the caller's device-side count rules long
        // rows out, in which case that kernel ends at once and every row is summed here
        int skip = g.skip_rows_longer_than;
        if (g.longest_row != nullptr && *g.longest_row <= skip) skip = 0x7FFFFFFF;
        if (b - a > skip) return;
    }
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;

    if (a == b) {
        if (live && g.zero_policy == FGL_ZERO_COPY_SELF) IO::fma(acc, 1.0f, ls.load(X + row * ldx + col0));
    } else if constexpr (MODE == FGL_AGG_EDGE) {
        gather_row_edge<T, VEC, LPR>(g, ls, gl, a, b, acc);
    } else {
        // one test per launch instead of one per load: is every live lane's vector whole?
        if (all_lanes_full<T, VEC>(D)) gather_row<T, VEC, LPR, MODE, true>(g, ls, gl, row, a, b, acc);
        else gather_row<T, VEC, LPR, MODE, false>(g, ls, gl, row, a, b, acc);
    }
    if (live) ls.store(out + row * ldo + col0, acc);
}

// The same mapping as a loop: a fixed number of lane groups, each taking rows g, g + G, g + 2G, ... and fetching the
// row after next's two offsets and the next row's neighbour ids while the current row's data is in flight, so that
// a row's chain offsets -> ids -> data is not walked from its start for every row.  Same sums in the same order.
// An experiment, not built by default (make HIPFLAGS_EXTRA="-DFGL_AGG_PIPE=1 -DFGL_AGG_PIPE_BLOCKS=8192" builds it in):
// measured on the outermost block of a 111 M-node graph's mini-batches (1.5 M gathered rows of 512 B, and of 256 B
// in bf16) it runs 0-3 % slower than one lane group per row with 2048-8192 persistent workgroups -- the gather is
// bound by the rate at which the memory system serves random rows, and the thousands of resident waves of the
// plain mapping already hide a single row's chain.
#ifndef FGL_AGG_PIPE
#define FGL_AGG_PIPE 0
#endif
#ifndef FGL_AGG_PIPE_BLOCKS
#define FGL_AGG_PIPE_BLOCKS 4096
#endif
template <typename T, int VEC, int LPR, int MODE>
__global__ __launch_bounds__(kBlock) void aggregate_pipe_kernel(const AggArgs g)
{
    using IO = RowIO<T, VEC>;
    constexpr int kGroups = kBlock / LPR;
    const int32_t* __restrict__ indptr = g.indptr;
    const int32_t* __restrict__ indices = g.indices;
    const T* __restrict__ X = static_cast<const T*>(g.x);
    T* __restrict__ out = static_cast<T*>(g.out);
    const int64_t ldx = g.ldx, ldo = g.ldo;
    const int64_t n_rows = actual_count(g.n_rows_max, g.d_n_rows);
    const int gl = (int)threadIdx.x % LPR;
    const int64_t stride = (int64_t)gridDim.x * kGroups;
    const LaneSlice<T, VEC> ls((int)blockIdx.y, LPR, gl, g.D);
    const bool all_full = all_lanes_full<T, VEC>(g.D);
    int64_t row = (int64_t)blockIdx.x * kGroups + (int)threadIdx.x / LPR;
    int64_t nrow = row + stride;
    int a = 0, b = 0, na = 0, nb = 0;
    if (row < n_rows) {
        a = indptr[row];
        b = indptr[row + 1];
    }
    if (nrow < n_rows) {
        na = indptr[nrow];
        nb = indptr[nrow + 1];
    }
    int my_col = (row < n_rows && gl < b - a) ? indices[a + gl] : 0;
    while (row < n_rows) {  // (uniform over a lane group; a wave's groups may leave at different times)
        const int64_t nnrow = nrow + stride;
        int nna = 0, nnb = 0;
        if (nnrow < n_rows) {
            nna = indptr[nnrow];
            nnb = indptr[nnrow + 1];
        }
        const int n_col = (nrow < n_rows && gl < nb - na) ? indices[na + gl] : 0;
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
        if (a == b) {
            if (ls.live && g.zero_policy == FGL_ZERO_COPY_SELF) IO::fma(acc, 1.0f, ls.load(X + row * ldx + ls.col0));
        } else if (all_full) {
            gather_row<T, VEC, LPR, MODE, true>(g, ls, gl, row, a, b, acc, &my_col);
        } else {
            gather_row<T, VEC, LPR, MODE, false>(g, ls, gl, row, a, b, acc, &my_col);
        }
        if (ls.live) ls.store(out + row * ldo + ls.col0, acc);
        row = nrow;
        a = na;
        b = nb;
        nrow = nnrow;
        na = nna;
        nb = nnb;
        my_col = n_col;
    }
}

// ---- few rows, long lists: several lane groups share a row -----------------------------------------
// A block of a few thousand rows (8192 destination rows of 25 entries, say) gives aggregate_kernel one
// lane group per row: 8192 rows of 64 bf16 columns are 1024 waves, four per CU, each lane with four
// 16-byte loads in flight -- a few MB in flight on the whole chip, which at the latency of a memory
// access is a fraction of what HBM delivers.  Here S lane groups of the same wave share a row: all S * LPR
// lanes load the row's neighbour ids in one coalesced read, group p sums the entries p, p + S, p + 2S, ...
// (four row loads in flight per lane, all groups at once), and the S partial sums are added with a
// fixed-order __shfl_xor tree -- no LDS, no atomics, the same bits on every run.  S times the waves, S times
// the bytes in flight.  Not for FGL_AGG_EDGE.
template <typename T, int VEC, int LPR, int S, int MODE>
__global__ __launch_bounds__(kBlock) void aggregate_split_kernel(const AggArgs g)
{
    using IO = RowIO<T, VEC>;
    constexpr int W = S * LPR;  // lanes per row: a divisor of the wave size
    static_assert(W <= kWave && kWave % W == 0, "a row's lanes must lie within one wave");
    constexpr int kRowsPerBlock = kBlock / W;
    const int32_t* __restrict__ indptr = g.indptr;
    const int32_t* __restrict__ indices = g.indices;
    const T* __restrict__ X = static_cast<const T*>(g.x);
    T* __restrict__ out = static_cast<T*>(g.out);
    const int64_t ldx = g.ldx;
    const int64_t n_rows = actual_count(g.n_rows_max, g.d_n_rows);
    const int q = (int)threadIdx.x % W;  // lane within the row's lanes
    const int part = q / LPR, gl = q % LPR;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (int)threadIdx.x / W;
    if (row >= n_rows) return;  // uniform over the row's lanes: the cross-lane reads below stay among live lanes
    const LaneSlice<T, VEC> ls((int)blockIdx.y, LPR, gl, g.D);
    const int col0 = ls.col0;
    const bool live = ls.live;
    const bool all_full = all_lanes_full<T, VEC>(g.D);

    const int a = indptr[row], b = indptr[row + 1];
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
    if (a == b) {
        if (part == 0 && live && g.zero_policy == FGL_ZERO_COPY_SELF) IO::fma(acc, 1.0f, ls.load(X + row * ldx + col0));
    } else {
        float row_factor = 1.0f;
        if (MODE == FGL_AGG_MEAN) row_factor = 1.0f / (float)(b - a);
        if (MODE == FGL_AGG_GCN) row_factor = 1.0f / sqrtf((float)g.row_norm[row]);
        for (int base = a; base < b; base += W) {
            const int cnt = (b - base) < W ? (b - base) : W;
            int my_col = 0;
            float my_w = 0.0f;
            if (q < cnt) {
                my_col = indices[base + q];
                my_w = edge_weight<MODE>(my_col, row_factor, g.col_norm, g.col_norm_is_ptr);
            }
            float sum[VEC];  // this chunk's share of the row (two-level summation, as in gather_row)
#pragma unroll
            for (int i = 0; i < VEC; ++i) sum[i] = 0.0f;
            // every group runs the same number of rounds (the cross-lane reads need all of the row's lanes);
            // entries past the end are read from lane 0 and neither loaded nor added
            for (int t = part; t - part < cnt; t += 4 * S) {
                int c[4];
                float w[4];
                typename IO::Raw x[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int src = t + j * S < cnt ? t + j * S : 0;
                    c[j] = __shfl(my_col, src, W);
                    w[j] = __shfl(my_w, src, W);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    x[j] = typename IO::Raw{};
                    if (live && t + j * S < cnt)
                        x[j] = all_full ? IO::load(X + (int64_t)c[j] * ldx + col0) : ls.load(X + (int64_t)c[j] * ldx + col0);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (t + j * S < cnt) IO::fma(sum, w[j], x[j]);
            }
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] += sum[i];
        }
    }
    // the groups' partial sums: pairwise, in an order that does not depend on scheduling
#pragma unroll
    for (int d = LPR; d < W; d <<= 1) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] += __shfl_xor(acc[i], d, W);
    }
    if (part == 0 && live) ls.store(out + row * g.ldo + col0, acc);
}

// ---- many rows, short lists: a lane group takes several rows at once -------------------------------
// The rows of a transposed block hold one entry on average (a third of them none): with one row per lane
// group, a group's life is three dependent memory accesses -- its two offsets, its one neighbour id, one row
// of data -- for 16 bytes per lane, and the chip spends its time waiting.  Here a group takes kBundleRows
// consecutive rows: their offsets are one read, their entries are consecutive in `indices` and are read
// (with their weights and the row each belongs to) in one coalesced chunk, and the data rows of all of
// them are in flight together, four at a time; the running sum is stored and cleared whenever an entry is
// the last of its row.  A bundle that holds a hub (more than 128 entries in all) falls back to one row
// after the other.  Sums are in CSR order, as in aggregate_kernel.
#ifndef FGL_BUNDLE_ROWS
#define FGL_BUNDLE_ROWS 4
#endif
constexpr int kBundleRows = FGL_BUNDLE_ROWS;

template <typename T, int VEC, int LPR, int MODE>
__global__ __launch_bounds__(kBlock) void aggregate_bundle_kernel(const AggArgs g)
{
    using IO = RowIO<T, VEC>;
    constexpr int R = kBundleRows;
    static_assert(R + 1 <= LPR, "a group reads the offsets of its rows with one lane each");
    constexpr int kGroups = kBlock / LPR;
    const int32_t* __restrict__ indptr = g.indptr;
    const int32_t* __restrict__ indices = g.indices;
    const T* __restrict__ X = static_cast<const T*>(g.x);
    T* __restrict__ out = static_cast<T*>(g.out);
    const int64_t ldx = g.ldx, ldo = g.ldo;
    const int64_t n_rows = actual_count(g.n_rows_max, g.d_n_rows);
    const int gl = (int)threadIdx.x % LPR;
    const int64_t r0 = ((int64_t)blockIdx.x * kGroups + (int)threadIdx.x / LPR) * R;
    if (r0 >= n_rows) return;  // uniform per group
    const int nr = n_rows - r0 < R ? (int)(n_rows - r0) : R;
    const LaneSlice<T, VEC> ls((int)blockIdx.y, LPR, gl, g.D);
    const int col0 = ls.col0;
    const bool live = ls.live;

    const int my_off = indptr[r0 + (gl < nr ? gl : nr)];
    int off[R + 1];  // off[j] = start of row j's entries; rows past the bundle's end are empty
#pragma unroll
    for (int j = 0; j <= R; ++j) off[j] = __shfl(my_off, j < nr ? j : nr, LPR);
    int skip = g.skip_rows_longer_than;  // as in aggregate_kernel
    if (g.longest_row != nullptr && *g.longest_row <= skip) skip = 0x7FFFFFFF;
    const int total = off[R] - off[0];

    if (total <= kLongRowEntries) {
        // (no row of the bundle is long enough to be left to the long-row launch)
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
        // cnt entries from the bundle's entry number cb on: ids, weights and row ends in one coalesced read,
        // then the data rows four at a time
        // FGL_AGG_EDGE (only where a lane's columns lie in one head, which the launcher checks): a lane looks up the
        // weight of (entry, its head) itself, next to the row load
        const int head = MODE == FGL_AGG_EDGE ? col0 / g.unit_dim : 0;
        auto chunk = [&](int cb, int cnt) {
            int my_col = 0, my_tag = 0;  // tag: row within the bundle, + 256 if the entry is the last of its row
            int my_eid = 0;
            float my_w = 0.0f;
            if (gl < cnt) {
                const int e = off[0] + cb + gl;
                my_col = indices[e];
                if (MODE == FGL_AGG_EDGE) my_eid = g.edge_index ? g.edge_index[e] : e;
                int j = 0;  // the rows that start at or before e: the last of them, row j, holds e
                int begin_j = off[0], end_j = off[1];
#pragma unroll
                for (int k = 1; k < R; ++k) {
                    if (off[k] <= e) {
                        j = k;
                        begin_j = off[k];
                        end_j = off[k + 1];
                    }
                }
                float row_factor = 1.0f;
                if (MODE == FGL_AGG_MEAN) row_factor = 1.0f / (float)(end_j - begin_j);
                if (MODE == FGL_AGG_GCN) row_factor = 1.0f / sqrtf((float)g.row_norm[r0 + j]);
                if (MODE != FGL_AGG_EDGE) my_w = edge_weight<MODE>(my_col, row_factor, g.col_norm, g.col_norm_is_ptr);
                my_tag = j | (e + 1 == end_j ? 256 : 0);
            }
            for (int t = 0; t < cnt; t += 4) {
                int c[4], tag[4];
                float w[4];
                typename IO::Raw x[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int src = t + j < cnt ? t + j : t;
                    c[j] = __shfl(my_col, src, LPR);
                    if (MODE == FGL_AGG_EDGE) w[j] = __int_as_float(__shfl(my_eid, src, LPR));  // (the entry's id, for now)
                    else w[j] = __shfl(my_w, src, LPR);
                    tag[j] = __shfl(my_tag, src, LPR);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    x[j] = typename IO::Raw{};
                    if (live && t + j < cnt) {
                        x[j] = ls.load(X + (int64_t)c[j] * ldx + col0);
                        if (MODE == FGL_AGG_EDGE) w[j] = g.edge_w[(int64_t)__float_as_int(w[j]) * g.n_heads + head];
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (t + j < cnt) {
                        IO::fma(acc, w[j], x[j]);
                        if (tag[j] & 256) {
                            if (live) ls.store(out + (r0 + (tag[j] & 255)) * ldo + col0, acc);
#pragma unroll
                            for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
                        }
                    }
                }
            }
        };
        if (total <= LPR) {  // the usual case, without the loop around it
            chunk(0, total);
        } else {
            for (int cb = 0; cb < total; cb += LPR) chunk(cb, total - cb < LPR ? total - cb : LPR);
        }
        // the rows without entries
#pragma unroll
        for (int j = 0; j < R; ++j) {
            if (j < nr && off[j + 1] == off[j] && live) {
                float z[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) z[i] = 0.0f;
                if (g.zero_policy == FGL_ZERO_COPY_SELF) IO::fma(z, 1.0f, ls.load(X + (r0 + j) * ldx + col0));
                ls.store(out + (r0 + j) * ldo + col0, z);
            }
        }
        return;
    }
    // a bundle with a longer list: one row after the other, as aggregate_kernel does
    for (int j = 0; j < nr; ++j) {
        const int a = off[j], b = off[j + 1];
        if (b - a > skip) continue;  // left to aggregate_long_rows_kernel
        const int64_t row = r0 + j;
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
        if (a == b) {
            if (live && g.zero_policy == FGL_ZERO_COPY_SELF) IO::fma(acc, 1.0f, ls.load(X + row * ldx + col0));
        } else if constexpr (MODE == FGL_AGG_EDGE) {
            gather_row_edge<T, VEC, LPR>(g, ls, gl, a, b, acc);
        } else {
            gather_row<T, VEC, LPR, MODE, false>(g, ls, gl, row, a, b, acc);
        }
        if (live) ls.store(out + row * ldo + col0, acc);
    }
}

// Rows whose length fills a power-of-two lane group badly (602 floats = 151 vector lanes: 79 % of three
// 64-lane groups; 602 bf16 = 76 lanes: 59 % of two) are mapped flat instead: lane t of the launch owns
// vector t % lanes of row t / lanes, rows packed back to back, so every lane of every wave moves data and
// the lanes of a row cover it contiguously.  There are no lane groups, hence no cross-lane broadcast:
// each lane reads the neighbour id (and its weight) itself -- the same address in all lanes of a row, one
// request per wave.  Four row loads are in flight before the first FMA, as in aggregate_kernel; sums are
// two-level with chunks of 32 entries.  Not for FGL_AGG_EDGE.
constexpr int kFlatChunk = 32;

template <typename T, int VEC, int MODE>
__global__ __launch_bounds__(kBlock) void aggregate_flat_kernel(const AggArgs g, int lanes)
{
    using IO = RowIO<T, VEC>;
    const int32_t* __restrict__ indptr = g.indptr;
    const int32_t* __restrict__ indices = g.indices;
    const T* __restrict__ X = static_cast<const T*>(g.x);
    T* __restrict__ out = static_cast<T*>(g.out);
    const int64_t ldx = g.ldx;
    const int64_t n_rows = actual_count(g.n_rows_max, g.d_n_rows);
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t row = t / lanes;
    if (row >= n_rows) return;
    int col0 = (int)(t - row * lanes) * VEC;
    // (the last lane of a row moves the row's last VEC columns where it can, see tail_overlaps)
    if (col0 + VEC > g.D && tail_overlaps<T, VEC>(g.D)) col0 = g.D - VEC;
    const int nvalid = g.D - col0;  // >= 1: lanes = ceil(D / VEC)
    const bool full = nvalid >= VEC;
    auto load = [&](const T* p) -> typename IO::Raw { return full ? IO::load(p) : IO::load_partial(p, nvalid); };

    const int a = indptr[row], b = indptr[row + 1];
    {
        int skip = g.skip_rows_longer_than;  // as in aggregate_kernel
        if (g.longest_row != nullptr && *g.longest_row <= skip) skip = 0x7FFFFFFF;
        if (b - a > skip) return;
    }
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
    if (a == b) {
        if (g.zero_policy == FGL_ZERO_COPY_SELF) IO::fma(acc, 1.0f, load(X + row * ldx + col0));
    } else {
        float row_factor = 1.0f;
        if (MODE == FGL_AGG_MEAN) row_factor = 1.0f / (float)(b - a);
        if (MODE == FGL_AGG_GCN) row_factor = 1.0f / sqrtf((float)g.row_norm[row]);
        for (int base = a; base < b; base += kFlatChunk) {
            const int end = b - base < kFlatChunk ? b : base + kFlatChunk;
            float part[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) part[i] = 0.0f;
            int e = base;
            for (; e + 4 <= end; e += 4) {
                const int c0 = indices[e], c1 = indices[e + 1], c2 = indices[e + 2], c3 = indices[e + 3];
                const float w0 = edge_weight<MODE>(c0, row_factor, g.col_norm, g.col_norm_is_ptr), w1 = edge_weight<MODE>(c1, row_factor, g.col_norm, g.col_norm_is_ptr);
                const float w2 = edge_weight<MODE>(c2, row_factor, g.col_norm, g.col_norm_is_ptr), w3 = edge_weight<MODE>(c3, row_factor, g.col_norm, g.col_norm_is_ptr);
                const typename IO::Raw r0 = load(X + (int64_t)c0 * ldx + col0);
                const typename IO::Raw r1 = load(X + (int64_t)c1 * ldx + col0);
                const typename IO::Raw r2 = load(X + (int64_t)c2 * ldx + col0);
                const typename IO::Raw r3 = load(X + (int64_t)c3 * ldx + col0);
                IO::fma(part, w0, r0);
                IO::fma(part, w1, r1);
                IO::fma(part, w2, r2);
                IO::fma(part, w3, r3);
            }
            const int rem = end - e;  // the last one to three entries, their loads issued together
            if (rem > 0) {
                const int c0 = indices[e];
                const int c1 = indices[rem > 1 ? e + 1 : e];
                const int c2 = indices[rem > 2 ? e + 2 : e];
                const float w0 = edge_weight<MODE>(c0, row_factor, g.col_norm, g.col_norm_is_ptr);
                const float w1 = edge_weight<MODE>(c1, row_factor, g.col_norm, g.col_norm_is_ptr);
                const float w2 = edge_weight<MODE>(c2, row_factor, g.col_norm, g.col_norm_is_ptr);
                const typename IO::Raw r0 = load(X + (int64_t)c0 * ldx + col0);
                typename IO::Raw r1 = r0, r2 = r0;
                if (rem > 1) r1 = load(X + (int64_t)c1 * ldx + col0);
                if (rem > 2) r2 = load(X + (int64_t)c2 * ldx + col0);
                IO::fma(part, w0, r0);
                if (rem > 1) IO::fma(part, w1, r1);
                if (rem > 2) IO::fma(part, w2, r2);
            }
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] += part[i];
        }
    }
    if (full) IO::store(out + row * g.ldo + col0, acc);
    else IO::store_partial(out + row * g.ldo + col0, acc, nvalid);
}

// The flat mapping for many rows of short lists (wide rows of a transposed block): lane t owns vector
// t % lanes of the kBundleRows consecutive rows of bundle t / lanes.  As in aggregate_bundle_kernel the rows'
// entries are walked as one list, four data rows in flight, the running sum stored at the end of each row;
// as in aggregate_flat_kernel every lane reads offsets and neighbour ids itself (the same addresses in all
// lanes of a bundle).
template <typename T, int VEC, int MODE>
__global__ __launch_bounds__(kBlock) void aggregate_flat_bundle_kernel(const AggArgs g, int lanes)
{
    using IO = RowIO<T, VEC>;
    constexpr int R = kBundleRows;
    const int32_t* __restrict__ indptr = g.indptr;
    const int32_t* __restrict__ indices = g.indices;
    const T* __restrict__ X = static_cast<const T*>(g.x);
    T* __restrict__ out = static_cast<T*>(g.out);
    const int64_t ldx = g.ldx, ldo = g.ldo;
    const int64_t n_rows = actual_count(g.n_rows_max, g.d_n_rows);
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t r0 = (t / lanes) * R;
    if (r0 >= n_rows) return;
    const int nr = n_rows - r0 < R ? (int)(n_rows - r0) : R;
    int col0 = (int)(t % lanes) * VEC;
    if (col0 + VEC > g.D && tail_overlaps<T, VEC>(g.D)) col0 = g.D - VEC;
    const int nvalid = g.D - col0;
    const bool full = nvalid >= VEC;
    auto load = [&](const T* p) -> typename IO::Raw { return full ? IO::load(p) : IO::load_partial(p, nvalid); };
    auto store = [&](T* p, const float (&a)[VEC]) {
        if (full) IO::store(p, a);
        else IO::store_partial(p, a, nvalid);
    };
    int off[R + 1];
#pragma unroll
    for (int j = 0; j <= R; ++j) off[j] = indptr[r0 + (j < nr ? j : nr)];
    int skip = g.skip_rows_longer_than;  // as in aggregate_kernel
    if (g.longest_row != nullptr && *g.longest_row <= skip) skip = 0x7FFFFFFF;
    const int total = off[R] - off[0];

    if (total <= kLongRowEntries) {
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
        for (int cb = 0; cb < total; cb += 4) {
            int c[4], tag[4];
            float w[4];
            typename IO::Raw x[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) c[j] = indices[off[0] + (cb + j < total ? cb + j : cb)];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                x[j] = typename IO::Raw{};
                if (cb + j < total) x[j] = load(X + (int64_t)c[j] * ldx + col0);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int e = off[0] + cb + j;
                int row_j = 0, begin_j = off[0], end_j = off[1];  // the row that holds e
#pragma unroll
                for (int k = 1; k < R; ++k) {
                    if (off[k] <= e) {
                        row_j = k;
                        begin_j = off[k];
                        end_j = off[k + 1];
                    }
                }
                float row_factor = 1.0f;
                if (MODE == FGL_AGG_MEAN) row_factor = 1.0f / (float)(end_j - begin_j);
                if (MODE == FGL_AGG_GCN && cb + j < total) row_factor = 1.0f / sqrtf((float)g.row_norm[r0 + row_j]);
                w[j] = cb + j < total ? edge_weight<MODE>(c[j], row_factor, g.col_norm, g.col_norm_is_ptr) : 0.0f;
                tag[j] = row_j | (e + 1 == end_j ? 256 : 0);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (cb + j < total) {
                    IO::fma(acc, w[j], x[j]);
                    if (tag[j] & 256) {
                        store(out + (r0 + (tag[j] & 255)) * ldo + col0, acc);
#pragma unroll
                        for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < R; ++j) {
            if (j < nr && off[j + 1] == off[j]) {
                float z[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) z[i] = 0.0f;
                if (g.zero_policy == FGL_ZERO_COPY_SELF) IO::fma(z, 1.0f, load(X + (r0 + j) * ldx + col0));
                store(out + (r0 + j) * ldo + col0, z);
            }
        }
        return;
    }
    // a bundle that holds a hub: one row after the other, two-level sums as in aggregate_flat_kernel
    for (int j = 0; j < nr; ++j) {
        const int a = off[j], b = off[j + 1];
        if (b - a > skip) continue;  // left to aggregate_long_rows_kernel
        const int64_t row = r0 + j;
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
        if (a == b) {
            if (g.zero_policy == FGL_ZERO_COPY_SELF) IO::fma(acc, 1.0f, load(X + row * ldx + col0));
        } else {
            float row_factor = 1.0f;
            if (MODE == FGL_AGG_MEAN) row_factor = 1.0f / (float)(b - a);
            if (MODE == FGL_AGG_GCN) row_factor = 1.0f / sqrtf((float)g.row_norm[row]);
            for (int base = a; base < b; base += kFlatChunk) {
                const int end = b - base < kFlatChunk ? b : base + kFlatChunk;
                float part[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) part[i] = 0.0f;
                for (int e = base; e < end; ++e) {
                    const int c0 = indices[e];
                    IO::fma(part, edge_weight<MODE>(c0, row_factor, g.col_norm, g.col_norm_is_ptr), load(X + (int64_t)c0 * ldx + col0));
                }
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[i] += part[i];
            }
        }
        store(out + row * ldo + col0, acc);
    }
}

// The rows that aggregate_kernel skipped.  Every workgroup (512 lanes) looks through its share of the
// row offsets and sums each long list it finds with all of its lane groups: group k takes the chunks
// k, k + groups, ... into a partial row, sixteen row loads in flight per lane, and the partials are added up
// through LDS in group order -- a fixed order, so the result does not depend on scheduling -- by the
// first group, which writes the row.  Few workgroups find anything, so this kernel is built for the
// latency of one long list, not for occupancy.  When the caller supplies the longest row's entry count
// on the device and it rules long lists out, every workgroup leaves after one scalar load.
constexpr int kLongBlock = 512;

template <typename T, int VEC, int LPR, int MODE>
__global__ __launch_bounds__(kLongBlock) void aggregate_long_rows_kernel(const AggArgs g)
{
    using IO = RowIO<T, VEC>;
    constexpr int kGroups = kLongBlock / LPR;
    constexpr int kInFlight = 16;
    const int threshold = g.skip_rows_longer_than;
    if (g.longest_row != nullptr && *g.longest_row <= threshold) return;
    const int32_t* __restrict__ indptr = g.indptr;
    const int32_t* __restrict__ indices = g.indices;
    const T* __restrict__ X = static_cast<const T*>(g.x);
    T* __restrict__ out = static_cast<T*>(g.out);
    const int64_t ldx = g.ldx;
    const int64_t n_rows = actual_count(g.n_rows_max, g.d_n_rows);
    const int gl = (int)threadIdx.x % LPR;
    const int grp = (int)threadIdx.x / LPR;
    const LaneSlice<T, VEC> ls((int)blockIdx.y, LPR, gl, g.D);
    const int col0 = ls.col0;
    const bool all_full = all_lanes_full<T, VEC>(g.D);  // every live lane moves a whole vector: loads without a per-lane branch

    __shared__ int found[kLongBlock];  // the lanes that met a long row in the current pass
    __shared__ int n_found;
    __shared__ float partial[kLongBlock * VEC];
    // Rows are dealt out one by one, round robin over the workgroups: hubs tend to sit next to each other
    // (the lowest local ids of a sampled block), and this gives neighbouring hubs to different workgroups.
    // (The offset reads are strided by that; they are a small part of the launch.)
    const int64_t per_pass = (int64_t)gridDim.x * kLongBlock;
    const int64_t passes = (n_rows + per_pass - 1) / per_pass;
    for (int64_t pass = 0; pass < passes; ++pass) {  // trip count uniform over the workgroup
        const int64_t r = (pass * kLongBlock + (int)threadIdx.x) * gridDim.x + blockIdx.x;
        const bool is_long = r < n_rows && indptr[r + 1] - indptr[r] > threshold;
        if (threadIdx.x == 0) n_found = 0;
        __syncthreads();
        if (is_long) found[atomicAdd(&n_found, 1)] = (int)threadIdx.x;
        __syncthreads();
        const int n = n_found;
        for (int i = 0; i < n; ++i) {
            // the order in which the long rows of a pass are taken does not matter: each is summed on its own
            const int64_t row = (pass * kLongBlock + found[i]) * gridDim.x + blockIdx.x;
            const int a = indptr[row], b = indptr[row + 1];
            float row_factor = 1.0f;
            if (MODE == FGL_AGG_MEAN) row_factor = 1.0f / (float)(b - a);
            if (MODE == FGL_AGG_GCN) row_factor = 1.0f / sqrtf((float)g.row_norm[row]);
            float acc[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
            for (int64_t base = (int64_t)a + (int64_t)grp * LPR; base < b; base += (int64_t)kGroups * LPR) {
                const int cnt = (b - base) < LPR ? (int)(b - base) : LPR;
                int my_col = 0;
                int my_eid = 0;     // FGL_AGG_EDGE: which row of edge_w the entry uses
                float my_w = 0.0f;  // the other modes: the entry's weight
                if (gl < cnt) {
                    my_col = indices[base + gl];
                    if (MODE == FGL_AGG_EDGE) my_eid = g.edge_index ? g.edge_index[base + gl] : (int)(base + gl);
                    else my_w = edge_weight<MODE>(my_col, row_factor, g.col_norm, g.col_norm_is_ptr);
                }
                float part[VEC];  // two-level summation, as in gather_row
#pragma unroll
                for (int k = 0; k < VEC; ++k) part[k] = 0.0f;
                for (int t = 0; t < cnt; t += kInFlight) {
                    int c[kInFlight];
                    int eid[kInFlight];
                    float w[kInFlight];
                    typename IO::Raw x[kInFlight];
#pragma unroll
                    for (int j = 0; j < kInFlight; ++j) {
                        const int src = t + j < cnt ? t + j : t;  // lanes past the end repeat entry t and are not added
                        c[j] = __shfl(my_col, src, LPR);
                        if (MODE == FGL_AGG_EDGE) eid[j] = __shfl(my_eid, src, LPR);
                        else w[j] = __shfl(my_w, src, LPR);
                    }
                    if (ls.live) {
                        if (all_full) {
#pragma unroll
                            for (int j = 0; j < kInFlight; ++j) x[j] = IO::load(X + (int64_t)c[j] * ldx + col0);
                        } else {
#pragma unroll
                            for (int j = 0; j < kInFlight; ++j) x[j] = ls.load(X + (int64_t)c[j] * ldx + col0);
                        }
                        if constexpr (MODE == FGL_AGG_EDGE) {
                            // one float per (entry, head); this lane's columns lie in one head when the head
                            // width is a multiple of VEC, else each column looks its head up
                            const float* __restrict__ ew = g.edge_w;
                            const int H = g.n_heads, unit = g.unit_dim;
                            if (unit % VEC == 0) {
                                const int head = col0 / unit;
#pragma unroll
                                for (int j = 0; j < kInFlight; ++j) w[j] = ew[(int64_t)eid[j] * H + head];
#pragma unroll
                                for (int j = 0; j < kInFlight; ++j)
                                    if (t + j < cnt) IO::fma(part, w[j], x[j]);
                            } else {
#pragma unroll
                                for (int j = 0; j < kInFlight; ++j) {
                                    if (t + j < cnt) {
                                        float xf[VEC];
#pragma unroll
                                        for (int k = 0; k < VEC; ++k) xf[k] = 0.0f;
                                        IO::fma(xf, 1.0f, x[j]);
#pragma unroll
                                        for (int k = 0; k < VEC; ++k) {
                                            const int col = col0 + k < g.D ? col0 + k : g.D - 1;
                                            part[k] += ew[(int64_t)eid[j] * H + col / unit] * xf[k];
                                        }
                                    }
                                }
                            }
                        } else {
#pragma unroll
                            for (int j = 0; j < kInFlight; ++j)
                                if (t + j < cnt) IO::fma(part, w[j], x[j]);
                        }
                    }
                }
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[k] += part[k];
            }
#pragma unroll
            for (int k = 0; k < VEC; ++k) partial[(int)threadIdx.x * VEC + k] = acc[k];
            __syncthreads();
            if (grp == 0 && ls.live) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
                for (int q = 0; q < kGroups; ++q)
#pragma unroll
                    for (int k = 0; k < VEC; ++k) acc[k] += partial[(q * LPR + gl) * VEC + k];
                ls.store(out + row * g.ldo + col0, acc);
            }
            __syncthreads();  // partial[] and found[] are reused
        }
    }
}

// ---- block transpose ---------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void transpose_count_kernel(const int32_t* __restrict__ indptr,
                                                                 const int32_t* __restrict__ indices, int64_t n_rows_max,
                                                                 const int32_t* __restrict__ d_n_rows, int64_t n_edges_max,
                                                                 int64_t n_cols_max, int32_t* __restrict__ counts,
                                                                 int split, int32_t* __restrict__ rank,
                                                                 int32_t* __restrict__ longest)
{
    const int64_t n_rows = actual_count(n_rows_max, d_n_rows);
    int64_t n_e = n_rows > 0 ? (int64_t)indptr[n_rows] : 0;
    if (n_e > n_edges_max) n_e = n_edges_max;
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_e) return;
    const int32_t c = indices[e];
    int32_t k = -1;
    // split > 1: every column has `split` counters and entry e uses number e % split -- a returning atomic
    // on one address completes before the next one starts, and a hub column is mentioned thousands of times
    if (c >= 0 && (int64_t)c < n_cols_max) k = atomicAdd(&counts[(int64_t)c * split + (int)(e & (split - 1))], 1);
    rank[e] = k;
    // only the few entries that land far down a long column report its length (split counters: see
    // transpose_offsets_kernel)
    if (split == 1 && longest != nullptr && k >= FGL_SHORT_ROW_ENTRIES) atomicMax(longest, k + 1);
}

// split counters, after their scan: the column offsets are every split-th prefix
__global__ __launch_bounds__(kBlock) void transpose_offsets_kernel(const int32_t* __restrict__ scanned, int split,
                                                                   int64_t n_cols_max, int32_t* __restrict__ t_indptr,
                                                                   int32_t* __restrict__ longest)
{
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x; c <= n_cols_max; c += stride) {
        const int32_t begin = scanned[c * split];
        t_indptr[c] = begin;
        if (longest != nullptr && c < n_cols_max) {
            const int32_t len = scanned[(c + 1) * split] - begin;
            if (len > FGL_SHORT_ROW_ENTRIES) atomicMax(longest, len);
        }
    }
}

__global__ __launch_bounds__(kBlock) void transpose_init_kernel(int32_t* __restrict__ counts, int64_t n, int32_t* __restrict__ longest)
{
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) counts[i] = 0;
    if (longest != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *longest = 0;
}

// sixteen lanes per row: the row's entries are read coalesced and scattered in parallel
__global__ __launch_bounds__(kBlock) void transpose_fill_kernel(const int32_t* __restrict__ indptr,
                                                                const int32_t* __restrict__ indices, int64_t n_rows_max,
                                                                const int32_t* __restrict__ d_n_rows, int64_t n_edges_max,
                                                                const int32_t* __restrict__ t_indptr, int split,
                                                                const int32_t* __restrict__ rank,
                                                                int32_t* __restrict__ t_indices,
                                                                int32_t* __restrict__ t_edge)
{
    constexpr int kLanes = 16;
    const int64_t n_rows = actual_count(n_rows_max, d_n_rows);
    const int lane = (int)threadIdx.x % kLanes;
    const int64_t stride = (int64_t)gridDim.x * (kBlock / kLanes);
    for (int64_t r = (int64_t)blockIdx.x * (kBlock / kLanes) + (int)threadIdx.x / kLanes; r < n_rows; r += stride) {
        const int64_t a = indptr[r];
        int64_t b = indptr[r + 1];
        if (b > n_edges_max) b = n_edges_max;
        for (int64_t e = a + lane; e < b; e += kLanes) {
            const int32_t k = rank[e];
            if (k >= 0) {
                // t_indptr: the column offsets, or (split > 1) the scanned split counters
                const int64_t pos = (int64_t)t_indptr[(int64_t)indices[e] * split + (int)(e & (split - 1))] + k;
                t_indices[pos] = (int32_t)r;
                if (t_edge) t_edge[pos] = (int32_t)e;
            }
        }
    }
}

// Blocks of at least this many entries count with kCountSplit counters per column (the extra scan and the
// offsets pass cost a few microseconds; below, the contention they remove costs less than that).
constexpr int64_t kCountSplitMinEdges = (int64_t)1 << 20;
constexpr int kCountSplit = 8;
static inline int count_split(int64_t n_edges_max, int sorted) { return (!sorted && n_edges_max >= kCountSplitMinEdges) ? kCountSplit : 1; }

size_t transpose_workspace_bytes(int64_t n_cols_max, int64_t n_edges_max, int sorted)
{
    const int split = count_split(n_edges_max, sorted);
    Carver c(nullptr);
    c.take<int32_t>((size_t)n_edges_max);
    c.take<char>(scan_workspace_bytes(n_cols_max * split));
    if (split > 1) c.take<int32_t>((size_t)(n_cols_max * split + 1));
    if (sorted) c.take<char>(sorted_transpose_workspace_bytes(n_cols_max, n_edges_max));
    return c.used();
}

// ---- dispatch ----------------------------------------------------------------------
// Which lane mapping the calling thread's last fgl_aggregate call chose (for benchmarks and bug reports).
static thread_local char g_mapping[96] = "";
static void note_mapping(const char* kernel, int lpr, int extra, bool second_pass)
{
    snprintf(g_mapping, sizeof(g_mapping), "%s lanes/row=%d%s%s", kernel, lpr,
             extra > 1 ? (extra >= 100 ? " (rows bundled by 4)" : " (groups/row>1)") : "", second_pass ? " + long_rows" : "");
}

// Workgroups of the long-row pass: each looks through an equal share of the row offsets.
constexpr int kLongRowBlocks = 1021;  // a prime: rows are dealt round robin, and ids that agree in their low bits are
                                       // alike in synthetic (R-MAT) graphs -- a power of two would hand all hubs to a few workgroups

template <typename T, int VEC, int LPR>
static int launch_agg_mode(int mode, bool long_rows_possible, dim3 grid, hipStream_t stream, AggArgs g)
{
    const bool second_pass = long_rows_possible;
    g.skip_rows_longer_than = second_pass ? kLongRowEntries : 0x7FFFFFFF;
    if constexpr (FGL_AGG_PIPE != 0) {
      if (!second_pass && mode != FGL_AGG_EDGE && (int64_t)grid.x > FGL_AGG_PIPE_BLOCKS) {
        note_mapping("aggregate_pipe_kernel", LPR, 1, false);
        const dim3 pgrid(FGL_AGG_PIPE_BLOCKS, grid.y);
#define FGL_LAUNCH_PIPE(M) hipLaunchKernelGGL((aggregate_pipe_kernel<T, VEC, LPR, M>), pgrid, dim3(kBlock), 0, stream, g)
        switch (mode) {
            case FGL_AGG_SUM: FGL_LAUNCH_PIPE(FGL_AGG_SUM); break;
            case FGL_AGG_MEAN: FGL_LAUNCH_PIPE(FGL_AGG_MEAN); break;
            case FGL_AGG_GCN: FGL_LAUNCH_PIPE(FGL_AGG_GCN); break;
            default: FGL_LAUNCH_PIPE(FGL_AGG_COLMEAN); break;
        }
#undef FGL_LAUNCH_PIPE
        FGL_CHECK_LAUNCH("aggregate_pipe_kernel");
        return FGL_OK;
      }
    }
    note_mapping("aggregate_kernel", LPR, 1, second_pass);
#define FGL_LAUNCH_MODE(M)                                                                                         \
    do {                                                                                                           \
        hipLaunchKernelGGL((aggregate_kernel<T, VEC, LPR, M>), grid, dim3(kBlock), 0, stream, g);                  \
        if (second_pass) {                                                                                         \
            int64_t blocks = ceil_div(g.n_rows_max, kLongBlock);                                                   \
            if (blocks > kLongRowBlocks) blocks = kLongRowBlocks;                                                  \
            hipLaunchKernelGGL((aggregate_long_rows_kernel<T, VEC, LPR, M>), dim3((unsigned)blocks, grid.y),       \
                               dim3(kLongBlock), 0, stream, g);                                                    \
        }                                                                                                          \
    } while (0)
    switch (mode) {
        case FGL_AGG_SUM: FGL_LAUNCH_MODE(FGL_AGG_SUM); break;
        case FGL_AGG_MEAN: FGL_LAUNCH_MODE(FGL_AGG_MEAN); break;
        case FGL_AGG_GCN: FGL_LAUNCH_MODE(FGL_AGG_GCN); break;
        case FGL_AGG_COLMEAN: FGL_LAUNCH_MODE(FGL_AGG_COLMEAN); break;
        default: FGL_LAUNCH_MODE(FGL_AGG_EDGE); break;
    }
#undef FGL_LAUNCH_MODE
    FGL_CHECK_LAUNCH("aggregate_kernel");
    return FGL_OK;
}

// Flat mapping (aggregate_flat_kernel) for the short rows, the usual second launch for the long ones.
template <typename T, int VEC>
static int launch_agg_flat(int mode, bool long_rows_possible, int lanes, bool bundle, hipStream_t stream, AggArgs g)
{
    g.skip_rows_longer_than = long_rows_possible ? kLongRowEntries : 0x7FFFFFFF;
    note_mapping(bundle ? "aggregate_flat_bundle_kernel" : "aggregate_flat_kernel", lanes, bundle ? 100 : 1, long_rows_possible);
    const int64_t blocks = ceil_div((bundle ? ceil_div(g.n_rows_max, kBundleRows) : g.n_rows_max) * lanes, kBlock);
    if (blocks > 0x7FFFFFFF) {
        set_error("aggregate: grid too large (%lld workgroups)", (long long)blocks);
        return FGL_ERR_UNSUPPORTED;
    }
#define FGL_LAUNCH_FLAT(M)                                                                                          \
    do {                                                                                                            \
        if (bundle)                                                                                                 \
            hipLaunchKernelGGL((aggregate_flat_bundle_kernel<T, VEC, M>), dim3((unsigned)blocks), dim3(kBlock), 0,   \
                               stream, g, lanes);                                                                   \
        else                                                                                                        \
            hipLaunchKernelGGL((aggregate_flat_kernel<T, VEC, M>), dim3((unsigned)blocks), dim3(kBlock), 0, stream,  \
                               g, lanes);                                                                           \
        if (long_rows_possible) {                                                                                   \
            int64_t lb = ceil_div(g.n_rows_max, kLongBlock);                                                        \
            if (lb > kLongRowBlocks) lb = kLongRowBlocks;                                                           \
            hipLaunchKernelGGL((aggregate_long_rows_kernel<T, VEC, 64, M>),                                          \
                               dim3((unsigned)lb, (unsigned)ceil_div(lanes, 64)), dim3(kLongBlock), 0, stream, g);   \
        }                                                                                                           \
    } while (0)
    switch (mode) {
        case FGL_AGG_SUM: FGL_LAUNCH_FLAT(FGL_AGG_SUM); break;
        case FGL_AGG_MEAN: FGL_LAUNCH_FLAT(FGL_AGG_MEAN); break;
        case FGL_AGG_GCN: FGL_LAUNCH_FLAT(FGL_AGG_GCN); break;
        default: FGL_LAUNCH_FLAT(FGL_AGG_COLMEAN); break;
    }
#undef FGL_LAUNCH_FLAT
    FGL_CHECK_LAUNCH("aggregate_flat_kernel");
    return FGL_OK;
}

// Launches of the two special mappings.  (Only for rows that fit one lane group; never for FGL_AGG_EDGE.)
#define FGL_FOR_ANY_MODE(mode, LAUNCH)                    \
    switch (mode) {                                       \
        case FGL_AGG_SUM: LAUNCH(FGL_AGG_SUM); break;     \
        case FGL_AGG_MEAN: LAUNCH(FGL_AGG_MEAN); break;   \
        case FGL_AGG_GCN: LAUNCH(FGL_AGG_GCN); break;     \
        case FGL_AGG_COLMEAN: LAUNCH(FGL_AGG_COLMEAN); break; \
        default: LAUNCH(FGL_AGG_EDGE); break;             \
    }
#define FGL_FOR_PLAIN_MODE(mode, LAUNCH)                  \
    switch (mode) {                                       \
        case FGL_AGG_SUM: LAUNCH(FGL_AGG_SUM); break;     \
        case FGL_AGG_MEAN: LAUNCH(FGL_AGG_MEAN); break;   \
        case FGL_AGG_GCN: LAUNCH(FGL_AGG_GCN); break;     \
        default: LAUNCH(FGL_AGG_COLMEAN); break;          \
    }

template <typename T, int VEC, int LPR, int S>
static int launch_agg_split(int mode, unsigned gy, hipStream_t stream, AggArgs g)
{
    g.skip_rows_longer_than = 0x7FFFFFFF;
    note_mapping("aggregate_split_kernel", LPR, S, false);
    const int64_t gx = ceil_div(g.n_rows_max, kBlock / (S * LPR));
#define FGL_LAUNCH_SPLIT(M) \
    hipLaunchKernelGGL((aggregate_split_kernel<T, VEC, LPR, S, M>), dim3((unsigned)gx, gy), dim3(kBlock), 0, stream, g)
    FGL_FOR_PLAIN_MODE(mode, FGL_LAUNCH_SPLIT)
#undef FGL_LAUNCH_SPLIT
    FGL_CHECK_LAUNCH("aggregate_split_kernel");
    return FGL_OK;
}

template <typename T, int VEC, int LPR>
static int launch_agg_bundle(int mode, bool long_rows_possible, unsigned gy, hipStream_t stream, AggArgs g)
{
    g.skip_rows_longer_than = long_rows_possible ? kLongRowEntries : 0x7FFFFFFF;
    note_mapping("aggregate_bundle_kernel", LPR, 100, long_rows_possible);
    const int64_t gx = ceil_div(ceil_div(g.n_rows_max, kBundleRows), kBlock / LPR);
#define FGL_LAUNCH_BUNDLE(M)                                                                                          \
    do {                                                                                                              \
        hipLaunchKernelGGL((aggregate_bundle_kernel<T, VEC, LPR, M>), dim3((unsigned)gx, gy), dim3(kBlock), 0, stream, g); \
        if (long_rows_possible) {                                                                                     \
            int64_t lb = ceil_div(g.n_rows_max, kLongBlock);                                                          \
            if (lb > kLongRowBlocks) lb = kLongRowBlocks;                                                             \
            hipLaunchKernelGGL((aggregate_long_rows_kernel<T, VEC, LPR, M>), dim3((unsigned)lb, gy), dim3(kLongBlock), \
                               0, stream, g);                                                                         \
        }                                                                                                             \
    } while (0)
    FGL_FOR_ANY_MODE(mode, FGL_LAUNCH_BUNDLE)
#undef FGL_LAUNCH_BUNDLE
    FGL_CHECK_LAUNCH("aggregate_bundle_kernel");
    return FGL_OK;
}

// A launch of fewer waves than this leaves the chip waiting on memory latency (one lane group per row): rows
// whose lists are known to be long enough are then shared by several groups (aggregate_split_kernel).
#ifndef FGL_SPLIT_BELOW_WAVES
#define FGL_SPLIT_BELOW_WAVES 2048
#endif
#ifndef FGL_SPLIT_TARGET_WAVES
#define FGL_SPLIT_TARGET_WAVES 4096  // groups per row are doubled until the launch has this many waves
#endif
// Lists of at most this many entries on average (per row, from the caller's entry count) are taken several
// rows at a time (aggregate_bundle_kernel).  Launches of a million rows and more bundle up to longer averages:
// there the one-group-per-row kernel falls behind (2 M rows of 2.1 entries, 256 bf16 columns: 614 us against
// 436 us bundled; 1 M rows: 255 against 217; at 3 entries per row 656 against 552 and 272 against 276), while
// below half a million rows bundling lists of more than two entries costs a few per cent.
#ifndef FGL_BUNDLE_MAX_AVG_ENTRIES
#define FGL_BUNDLE_MAX_AVG_ENTRIES 2
#endif
static inline bool lists_are_short(int64_t n_entries, int64_t n_rows)
{
    if (n_entries < 0 || n_rows < 1024) return false;
    // twice the largest average that is bundled, so that 2.5 can be said
    const int64_t twice = n_rows >= ((int64_t)1 << 21) ? 8 : n_rows >= ((int64_t)1 << 20) ? 5 : 2 * FGL_BUNDLE_MAX_AVG_ENTRIES;
    return 2 * n_entries <= twice * n_rows;
}

template <typename T, int VEC>
static int launch_agg_vec(int mode, int64_t longest_row_max, int64_t n_entries_max, hipStream_t stream, const AggArgs& g)
{
    const int lanes_needed = (g.D + VEC - 1) / VEC;
    int lpr = 8;
    while (lpr < 64 && lpr < lanes_needed) lpr <<= 1;
    // many rows of short lists (a transposed block): several rows per lane group
    const bool short_lists = lists_are_short(n_entries_max, g.n_rows_max) &&
                             (mode != FGL_AGG_EDGE || (g.unit_dim % VEC == 0 && lanes_needed <= 64));
    // rows wider than one 64-lane group that fill their groups to less than 90 %: flat mapping
    // (602 fp32 columns: 100 -> 80 us; 602 bf16: 59 -> 44 us forward, 135 -> 84 us on the transposed block)
    if (lanes_needed > 64 && mode != FGL_AGG_EDGE && lanes_needed * 10 < ceil_div(lanes_needed, 64) * 64 * 9)
        return launch_agg_flat<T, VEC>(mode, longest_row_max < 0 || longest_row_max > kLongRowEntries, lanes_needed,
                                       short_lists, stream, g);
    const int64_t groups = kBlock / lpr;
    const int64_t gx = ceil_div(g.n_rows_max, groups);
    const int64_t gy = ceil_div(lanes_needed, lpr);
    if (gx > 0x7FFFFFFF || gy > 65535) {
        set_error("aggregate: grid too large (%lld x %lld)", (long long)gx, (long long)gy);
        return FGL_ERR_UNSUPPORTED;
    }
    const dim3 grid((unsigned)gx, (unsigned)gy);
    // a host-side bound that rules long rows out makes this exactly one launch of the plain kernel
    const bool long_rows_possible = longest_row_max < 0 || longest_row_max > kLongRowEntries;
    if constexpr (VEC > 1) {
        // few rows, lists known to be long: S lane groups per row, chosen so that each group still gets
        // three entries or more and the launch reaches FGL_SPLIT_BELOW_WAVES waves
        const int64_t waves = ceil_div(g.n_rows_max * lpr, kWave);
        if (mode != FGL_AGG_EDGE && lpr < 64 && !long_rows_possible && waves < FGL_SPLIT_BELOW_WAVES) {
            int s = 64 / lpr;
            while (s > 1 && ((int64_t)s * 3 > longest_row_max || waves * (s / 2) >= FGL_SPLIT_TARGET_WAVES)) s >>= 1;
#define FGL_SPLIT_CASE(L, S_) if (lpr == L && s == S_) return launch_agg_split<T, VEC, L, S_>(mode, grid.y, stream, g)
            FGL_SPLIT_CASE(8, 8);
            FGL_SPLIT_CASE(8, 4);
            FGL_SPLIT_CASE(8, 2);
            FGL_SPLIT_CASE(16, 4);
            FGL_SPLIT_CASE(16, 2);
            FGL_SPLIT_CASE(32, 2);
#undef FGL_SPLIT_CASE
        }
        // (not for rows of eight lanes -- 128 bytes, one cache line: there the bundle's bookkeeping costs what it saves)
        if (short_lists && lpr >= 16) {
            switch (lpr) {
                case 16: return launch_agg_bundle<T, VEC, 16>(mode, long_rows_possible, grid.y, stream, g);
                case 32: return launch_agg_bundle<T, VEC, 32>(mode, long_rows_possible, grid.y, stream, g);
                default: return launch_agg_bundle<T, VEC, 64>(mode, long_rows_possible, grid.y, stream, g);
            }
        }
    }
    switch (lpr) {
        case 8: return launch_agg_mode<T, VEC, 8>(mode, long_rows_possible, grid, stream, g);
        case 16: return launch_agg_mode<T, VEC, 16>(mode, long_rows_possible, grid, stream, g);
        case 32: return launch_agg_mode<T, VEC, 32>(mode, long_rows_possible, grid, stream, g);
        default: return launch_agg_mode<T, VEC, 64>(mode, long_rows_possible, grid, stream, g);
    }
}

// bf16 rows can be moved eight elements at a time when every row starts on a 4-byte boundary
static bool bf16_rows_dword_aligned(int64_t ldx, int64_t ldo, const void* x, const void* out)
{
    return ldx % 2 == 0 && ldo % 2 == 0 && ((uintptr_t)x % 4) == 0 && ((uintptr_t)out % 4) == 0;
}

}  // namespace fgl

using namespace fgl;

FGL_EXPORT int fgl_aggregate(const int32_t* d_indptr, const int32_t* d_indices, int64_t n_rows_max,
                             const int32_t* d_n_rows, const void* d_x, int64_t ldx, int D, int dtype, int mode,
                             int zero_policy, const int32_t* d_row_norm, const int32_t* d_col_norm,
                             const float* d_edge_w, int n_heads, const int32_t* d_edge_index,
                             int64_t longest_row_max, const int32_t* d_longest_row, int64_t n_entries_max,
                             void* d_out, int64_t ldo, void* stream)
{
    FGL_REQUIRE(n_rows_max >= 0, "aggregate: negative row count");
    FGL_REQUIRE(D >= 1, "aggregate: feature length %d < 1", D);
    FGL_REQUIRE(ldx >= D && ldo >= D, "aggregate: row stride smaller than the row length");
    FGL_REQUIRE(dtype == FGL_F32 || dtype == FGL_BF16, "aggregate: unknown dtype %d", dtype);
    FGL_REQUIRE(mode >= FGL_AGG_SUM && mode <= FGL_AGG_COLMEAN_PTR, "aggregate: unknown mode %d", mode);
    const int col_norm_is_ptr = mode == FGL_AGG_COLMEAN_PTR;
    if (col_norm_is_ptr) mode = FGL_AGG_COLMEAN;
    FGL_REQUIRE(zero_policy == FGL_ZERO_COPY_SELF || zero_policy == FGL_ZERO_ZEROS, "aggregate: unknown zero policy %d", zero_policy);
    FGL_REQUIRE(mode != FGL_AGG_GCN || (d_row_norm && d_col_norm), "aggregate: gcn mode needs row_norm and col_norm");
    FGL_REQUIRE(mode != FGL_AGG_COLMEAN || d_col_norm, "aggregate: colmean mode needs col_norm");
    FGL_REQUIRE(mode != FGL_AGG_EDGE || (d_edge_w && n_heads >= 1 && D % n_heads == 0),
                "aggregate: edge mode needs edge weights and a head count that divides the row length");
    if (n_rows_max == 0) return FGL_OK;
    FGL_REQUIRE(d_indptr && d_indices && d_x && d_out, "aggregate: null pointer");
    FGL_REQUIRE(d_x != d_out, "aggregate: output aliases the input");
    AggArgs g;
    g.indptr = d_indptr; g.indices = d_indices; g.n_rows_max = n_rows_max; g.d_n_rows = d_n_rows;
    g.x = d_x; g.ldx = ldx; g.D = D; g.zero_policy = zero_policy; g.row_norm = d_row_norm; g.col_norm = d_col_norm;
    g.out = d_out; g.ldo = ldo; g.edge_w = d_edge_w; g.edge_index = d_edge_index; g.longest_row = d_longest_row;
    g.n_heads = n_heads > 0 ? n_heads : 1; g.unit_dim = D / g.n_heads; g.col_norm_is_ptr = col_norm_is_ptr;
    hipStream_t s = as_stream(stream);
    if (dtype == FGL_F32) return launch_agg_vec<float, 4>(mode, longest_row_max, n_entries_max, s, g);
    if (bf16_rows_dword_aligned(ldx, ldo, d_x, d_out)) return launch_agg_vec<uint16_t, 8>(mode, longest_row_max, n_entries_max, s, g);
    return launch_agg_vec<uint16_t, 1>(mode, longest_row_max, n_entries_max, s, g);
}

FGL_EXPORT const char* fgl_aggregate_last_mapping(void) { return g_mapping; }

FGL_EXPORT size_t fgl_block_transpose_workspace_bytes(int64_t n_cols_max, int64_t n_edges_max, int sorted)
{
    if (n_cols_max < 0 || n_edges_max < 0) return 0;
    return transpose_workspace_bytes(n_cols_max, n_edges_max, sorted);
}

FGL_EXPORT int fgl_block_transpose(const int32_t* d_indptr, const int32_t* d_indices, int64_t n_rows_max,
                                   const int32_t* d_n_rows, int64_t n_cols_max, const int32_t* d_n_cols,
                                   int64_t n_edges_max, int32_t* d_t_indptr, int32_t* d_t_indices,
                                   int32_t* d_t_edge, int32_t* d_t_longest_row, int sorted, void* d_ws, size_t ws_bytes,
                                   void* stream)
{
    FGL_REQUIRE(sorted == 0 || (d_n_rows == nullptr && d_n_cols == nullptr),
                "block_transpose: the sorted variant needs exact sizes (no device-side counts)");
    FGL_REQUIRE(n_rows_max >= 0 && n_cols_max >= 0 && n_edges_max >= 0, "block_transpose: negative size");
    FGL_REQUIRE(n_edges_max <= 0x7FFFFFFF, "block_transpose: edge count exceeds int32 offsets");
    FGL_REQUIRE(d_t_indptr != nullptr, "block_transpose: null output");
    FGL_REQUIRE(n_edges_max == 0 || (d_indptr && d_indices && d_t_indices), "block_transpose: null pointer");
    if (d_ws == nullptr || ws_bytes < transpose_workspace_bytes(n_cols_max, n_edges_max, sorted)) {
        set_error("block_transpose: workspace too small (%zu < %zu)", ws_bytes, transpose_workspace_bytes(n_cols_max, n_edges_max, sorted));
        return FGL_ERR_WORKSPACE;
    }
    hipStream_t s = as_stream(stream);
    const int split = count_split(n_edges_max, sorted);
    Carver c(d_ws);
    int32_t* rank = c.take<int32_t>((size_t)n_edges_max);
    char* scan_ws = c.take<char>(scan_workspace_bytes(n_cols_max * split));
    // the counts live in t_indptr and are scanned in place; with split counters they live in the workspace
    int32_t* counts = split > 1 ? c.take<int32_t>((size_t)(n_cols_max * split + 1)) : d_t_indptr;
    const int64_t n_counts = n_cols_max * split;
    {
        int64_t blocks = ceil_div(n_counts + 1, kBlock);
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(transpose_init_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, counts, n_counts + 1,
                           d_t_longest_row);
        FGL_CHECK_LAUNCH("transpose_init_kernel");
    }
    if (n_edges_max > 0 && n_rows_max > 0) {
        hipLaunchKernelGGL(transpose_count_kernel, dim3((unsigned)ceil_div(n_edges_max, kBlock)), dim3(kBlock), 0, s,
                           d_indptr, d_indices, n_rows_max, d_n_rows, n_edges_max, n_cols_max, counts, split, rank,
                           d_t_longest_row);
        FGL_CHECK_LAUNCH("transpose_count_kernel");
    }
    // (split counters are scanned up to the host bound: counters of columns past a device-side count are zero)
    int rc = launch_exclusive_sum(counts, n_counts, split > 1 ? nullptr : d_n_cols, counts, nullptr, scan_ws,
                                  scan_workspace_bytes(n_counts), s);
    if (rc != FGL_OK) return rc;
    if (split > 1) {
        int64_t blocks = ceil_div(n_cols_max + 1, kBlock);
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(transpose_offsets_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, counts, split, n_cols_max,
                           d_t_indptr, d_t_longest_row);
        FGL_CHECK_LAUNCH("transpose_offsets_kernel");
    }
    if (sorted) {
        const size_t sort_bytes = sorted_transpose_workspace_bytes(n_cols_max, n_edges_max);
        char* sort_ws = c.take<char>(sort_bytes);
        return launch_sorted_transpose_fill(d_indptr, d_indices, n_rows_max, n_cols_max, n_rows_max > 0 ? n_edges_max : 0,
                                            d_t_indices, d_t_edge, sort_ws, sort_bytes, s);
    }
    if (n_edges_max > 0 && n_rows_max > 0) {
        int64_t fill_blocks = ceil_div(n_rows_max, kBlock / 16);
        if (fill_blocks > 16384) fill_blocks = 16384;
        hipLaunchKernelGGL(transpose_fill_kernel, dim3((unsigned)fill_blocks), dim3(kBlock), 0, s, d_indptr,
                           d_indices, n_rows_max, d_n_rows, n_edges_max, counts, split, rank, d_t_indices, d_t_edge);
        FGL_CHECK_LAUNCH("transpose_fill_kernel");
    }
    return FGL_OK;
}
