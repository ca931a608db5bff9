/*
 * CPU oracle for the FastGL hot path (sample -> fused id-map -> aggregate).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in plain C, what the
 * reference's CUDA operators compute, so that the HIP kernels can be checked against
 * it.  Only the test-suite, the smoke check and the CPU-baseline leg of the benchmark
 * may load it; the product library never links or calls anything in this file.
 *
 * Reference files followed (paths relative to the reference checkout):
 *   cuda_operators/sample.cu:17-38,76-95      degree clamp, exclusive scan, copy-all / pick
 *   cuda_operators/cuda_hashtable.cuh:27-30   TableSize
 *   cuda_operators/id_map.cu:259-383,386-493  local-id rule, in-place relabel, return layout
 *   cuda_operators/utilis.cu:17-79            cal_deg (histogram), exclusive_sum (padded scan)
 *   cuda_operators/aggregate_acc_kernel.cu:270-331,375-427,467-517,554-596
 *                                             GCN / GIN forward and backward, zero-degree rule
 *   cuda_operators/aggregate_acc_kernel.cu:835-886,924-979   GAT forward and backward
 *   GraphConv.py:265-272                      GAT attention coefficients (DGL u_add_v, leaky_relu,
 *                                             edge_softmax: third-party, restated from their definitions)
 *
 * Deliberate departures from the reference (each one is also what the HIP library does):
 *   - random picks are WITHOUT replacement (Floyd's subset algorithm) from a
 *     Philox4x32-10 stream keyed by (rng_seed, stream_id, node id); the reference
 *     draws curand()%deg with replacement from a per-launch-constant stream
 *     (sample.cu:70,91), which its own caller labels replace=False;
 *   - new source ids get local ids in first-occurrence order (one legal outcome of the
 *     reference's race at id_map.cu:317-320, and the order DGL's to_block produces);
 *   - 64-bit offsets are accepted for the graph's indptr.
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   orc_philox4x32_10   Random123 known-answer vectors
 *   orc_sample_node     closed form when fanout >= degree; validity invariants and a
 *                       chi-square uniformity test otherwise; exhaustive subset
 *                       enumeration for tiny degrees
 *   orc_table_size      closed form / hand-evaluated values of the reference expression
 *   orc_idmap           numpy/python dict restatement, order-free invariants, hand cases
 *   orc_idmap_parallel  (timing variant only) identical output to orc_idmap
 *   orc_cal_deg, orc_exclusive_sum   numpy.bincount / numpy.cumsum
 *   orc_aggregate_f64   scipy.sparse products, all-ones / one-hot closed forms
 *   orc_aggregate_edge_f64  scipy.sparse products per head; reduces to orc_aggregate_f64 for unit weights
 *   orc_edge_softmax_f64  scipy.special.softmax per row and head; rows sum to one; invariance to a
 *                       shift of er; uniform 1/deg for equal scores; the leaky-relu slope by hand values
 *   orc_transpose       scipy.sparse transpose (stable order)
 *   orc_rmat_keys       quadrant frequencies against (a,b,c,d); symmetry; determinism
 *   orc_aggregate_f32   (timing variant only) compared with orc_aggregate_f64
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------
 * Philox4x32-10 (Salmon, Moraes, Dror, Shaw, SC'11; the generator the reference uses via
 * cuRAND at sample.cu:69-70).  Published algorithm, restated.
 * ---------------------------------------------------------------------------------- */
ORC_API void orc_philox4x32_10(const uint32_t ctr_in[4], const uint32_t key_in[2], uint32_t out[4])
{
    uint32_t c0 = ctr_in[0], c1 = ctr_in[1], c2 = ctr_in[2], c3 = ctr_in[3];
    uint32_t k0 = key_in[0], k1 = key_in[1];
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

static inline uint64_t mulhi64(uint64_t a, uint64_t b)
{
    return (uint64_t)(((unsigned __int128)a * b) >> 64);
}

/* The m-th 64-bit draw for node `pos` in sampling stream `stream_id` (the picks of a node
 * depend on the node, the stream and the seed only -- not on where it sits in the seed list).
 * Counter = {node_lo, node_hi, stream_id, m/2}, key = {seed_lo, seed_hi}; even m takes words
 * 0..1 of the block, odd m words 2..3. */
static inline uint64_t sample_draw(uint64_t rng_seed, uint32_t stream_id, uint64_t pos, uint32_t m)
{
    uint32_t ctr[4] = {(uint32_t)pos, (uint32_t)(pos >> 32), stream_id, m >> 1};
    uint32_t key[2] = {(uint32_t)rng_seed, (uint32_t)(rng_seed >> 32)};
    uint32_t o[4];
    orc_philox4x32_10(ctr, key, o);
    return (m & 1u) ? ((uint64_t)o[2] | ((uint64_t)o[3] << 32)) : ((uint64_t)o[0] | ((uint64_t)o[1] << 32));
}

/* Floyd's algorithm: a uniformly random k-subset of {0..deg-1}, in insertion order. */
ORC_API void orc_floyd_subset(int64_t deg, int k, uint64_t rng_seed, uint32_t stream_id, uint64_t pos, int64_t* sel)
{
    for (int m = 0; m < k; ++m) {
        int64_t j = deg - k + m;
        uint64_t r = sample_draw(rng_seed, stream_id, pos, (uint32_t)m);
        int64_t t = (int64_t)mulhi64(r, (uint64_t)(j + 1));
        int dup = 0;
        for (int q = 0; q < m; ++q) dup |= (sel[q] == t);
        sel[m] = dup ? j : t;
    }
}

static inline int64_t ptr_at(const void* indptr, int is64, int64_t i)
{
    return is64 ? ((const int64_t*)indptr)[i] : (int64_t)((const int32_t*)indptr)[i];
}

/* ------------------------------------------------------------------------------------
 * sample_node  (reference: sample.cu:17-38 clamp, :155-159 scan, :76-95 copy-all / pick)
 * For seed position i with node s: k = min(fanout, deg(s)); block_ptr = exclusive scan of k;
 * src_out[block_ptr[i] + j] = j-th chosen in-neighbour (global id), dst_out[...] = s.
 * deg <= fanout: all neighbours in CSR order.  Returns the number of sampled edges.
 * ---------------------------------------------------------------------------------- */
ORC_API int64_t orc_sample_node(const void* indptr, int indptr_is64, const int32_t* indices,
                                const int32_t* seeds, int64_t n_seeds, int fanout,
                                uint64_t rng_seed, uint32_t stream_id,
                                int32_t* src_out, int32_t* dst_out, int32_t* block_ptr)
{
    int64_t run = 0;
    for (int64_t i = 0; i < n_seeds; ++i) {
        int64_t s = seeds[i];
        int64_t deg = ptr_at(indptr, indptr_is64, s + 1) - ptr_at(indptr, indptr_is64, s);
        block_ptr[i] = (int32_t)run;
        run += deg < fanout ? deg : fanout;
    }
    block_ptr[n_seeds] = (int32_t)run;

#pragma omp parallel
    {
        int64_t* sel = (int64_t*)malloc(sizeof(int64_t) * (size_t)(fanout > 0 ? fanout : 1));
#pragma omp for schedule(dynamic, 256)
        for (int64_t i = 0; i < n_seeds; ++i) {
            int64_t s = seeds[i];
            int64_t a = ptr_at(indptr, indptr_is64, s);
            int64_t deg = ptr_at(indptr, indptr_is64, s + 1) - a;
            int64_t off = block_ptr[i];
            if (deg <= fanout) {
                for (int64_t j = 0; j < deg; ++j) {
                    src_out[off + j] = indices[a + j];
                    if (dst_out) dst_out[off + j] = (int32_t)s;
                }
            } else {
                orc_floyd_subset(deg, fanout, rng_seed, stream_id, (uint64_t)s, sel);
                for (int j = 0; j < fanout; ++j) {
                    src_out[off + j] = indices[a + sel[j]];
                    if (dst_out) dst_out[off + j] = (int32_t)s;
                }
            }
        }
        free(sel);
    }
    return run;
}

/* ------------------------------------------------------------------------------------
 * TableSize  (reference: cuda_hashtable.cuh:27-30)
 *   next_pow2 = 1 << (size_t)(1 + log2(num >> 1));  return next_pow2 << scale;
 * i.e. (largest power of two <= num) << scale for num >= 2; evaluated in 64 bits here
 * (the reference's `1 <<` is a 32-bit shift).
 * ---------------------------------------------------------------------------------- */
ORC_API int64_t orc_table_size(int64_t num, int scale)
{
    int64_t half = num >> 1;
    int64_t p = 1;
    if (half >= 1) {
        int lg = 0;
        while ((half >> (lg + 1)) != 0) ++lg; /* floor(log2(half)) */
        p = (int64_t)1 << (1 + lg);
    }
    return p << scale;
}

/* ------------------------------------------------------------------------------------
 * Fused id-map (reference: id_map.cu:259-287 dst insert with local = position,
 * :290-347 new source ids numbered from n_dst upwards, :351-383 in-place relabel of both
 * edge arrays, :491 return cat(dst_unique, new ids in local order)).
 * New ids are numbered in order of first occurrence in src[].  A dst id that occurs more
 * than once in dst_unique keeps the local id of its first position.
 * src/dst are rewritten in place (dst may be NULL).  Returns n_dst + number of new ids,
 * or -1 if an id in dst[] is not in the map, or -2 if uniq_capacity is too small.
 * ---------------------------------------------------------------------------------- */
typedef struct { int32_t key; int32_t val; } orc_slot;

static inline uint64_t orc_hash(uint32_t id, int shift) { return ((uint64_t)(id * 0x9E3779B1u)) >> shift; }

ORC_API int64_t orc_idmap(int32_t* src, int32_t* dst, int64_t n_edges,
                          const int32_t* dst_unique, int64_t n_dst,
                          int32_t* uniq, int64_t uniq_capacity)
{
    int64_t want = 2 * (n_dst + n_edges) + 2;
    int lg = 1;
    while (((int64_t)1 << lg) < want) ++lg;
    if (lg > 31) return -2;
    int64_t slots = (int64_t)1 << lg;
    int shift = 32 - lg;
    orc_slot* tab = (orc_slot*)malloc(sizeof(orc_slot) * (size_t)slots);
    memset(tab, 0xFF, sizeof(orc_slot) * (size_t)slots);
    int64_t mask = slots - 1;
    int64_t n = n_dst;
    int64_t rc = 0;
    if (n_dst > uniq_capacity) { free(tab); return -2; }
    for (int64_t i = 0; i < n_dst; ++i) {
        int32_t id = dst_unique[i];
        uniq[i] = id;
        int64_t p = (int64_t)orc_hash((uint32_t)id, shift);
        while (tab[p].key != -1 && tab[p].key != id) p = (p + 1) & mask;
        if (tab[p].key == -1) { tab[p].key = id; tab[p].val = (int32_t)i; }
    }
    for (int64_t e = 0; e < n_edges; ++e) {
        int32_t id = src[e];
        int64_t p = (int64_t)orc_hash((uint32_t)id, shift);
        while (tab[p].key != -1 && tab[p].key != id) p = (p + 1) & mask;
        if (tab[p].key == -1) {
            if (n >= uniq_capacity) { rc = -2; break; }
            tab[p].key = id; tab[p].val = (int32_t)n; uniq[n] = id; ++n;
        }
        src[e] = tab[p].val;
    }
    if (rc == 0 && dst) {
        for (int64_t e = 0; e < n_edges; ++e) {
            int32_t id = dst[e];
            int64_t p = (int64_t)orc_hash((uint32_t)id, shift);
            while (tab[p].key != -1 && tab[p].key != id) p = (p + 1) & mask;
            if (tab[p].key == -1) { rc = -1; break; }
            dst[e] = tab[p].val;
        }
    }
    free(tab);
    return rc ? rc : n;
}

/* The same map built by all host threads (timing variant for the CPU baseline; its output is
 * checked to be identical to orc_idmap's).  Keys are claimed with a compare-and-swap; a key that is new
 * in this call carries, until it is numbered, the smallest index of an edge that mentions it (kept with
 * an atomic minimum), so that new ids are numbered in first-occurrence order whatever the thread
 * interleaving: flag the first mentions, prefix-sum the flags, number, relabel. */
#define ORC_PENDING 0x80000000u

static inline int64_t orc_claim(orc_slot* tab, int64_t mask, int shift, int32_t id)
{
    int64_t p = (int64_t)orc_hash((uint32_t)id, shift);
    for (;;) {
        int32_t k = __atomic_load_n(&tab[p].key, __ATOMIC_RELAXED);
        if (k == -1) {
            int32_t expected = -1;
            if (__atomic_compare_exchange_n(&tab[p].key, &expected, id, 0, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) return p;
            k = expected;
        }
        if (k == id) return p;
        p = (p + 1) & mask;
    }
}

static inline void orc_atomic_min_u32(uint32_t* addr, uint32_t v)
{
    uint32_t cur = __atomic_load_n(addr, __ATOMIC_RELAXED);
    while (v < cur && !__atomic_compare_exchange_n(addr, &cur, v, 0, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) {}
}

ORC_API int64_t orc_idmap_parallel(int32_t* src, int64_t n_edges, const int32_t* dst_unique, int64_t n_dst,
                                   int32_t* uniq, int64_t uniq_capacity)
{
    int64_t want = 2 * (n_dst + n_edges) + 2;
    int lg = 1;
    while (((int64_t)1 << lg) < want) ++lg;
    if (lg > 31 || n_edges >= (int64_t)ORC_PENDING || n_dst > uniq_capacity) return -2;
    int64_t slots = (int64_t)1 << lg, mask = slots - 1;
    int shift = 32 - lg;
    orc_slot* tab = (orc_slot*)malloc(sizeof(orc_slot) * (size_t)slots);
    int64_t* slot_of = (int64_t*)malloc(sizeof(int64_t) * (size_t)(n_edges > 0 ? n_edges : 1));
    int nt = 1;
#ifdef _OPENMP
    nt = omp_get_max_threads();
#endif
    int64_t* part = (int64_t*)calloc((size_t)nt + 1, sizeof(int64_t));
    int64_t n_new = 0;
#pragma omp parallel num_threads(nt)
    {
        int t = 0;
#ifdef _OPENMP
        t = omp_get_thread_num();
#endif
#pragma omp for schedule(static)
        for (int64_t i = 0; i < slots; ++i) { tab[i].key = -1; tab[i].val = -1; }  /* val: all ones = larger than any index */
#pragma omp for schedule(static)
        for (int64_t i = 0; i < n_dst; ++i) {
            uniq[i] = dst_unique[i];
            int64_t p = orc_claim(tab, mask, shift, dst_unique[i]);
            orc_atomic_min_u32((uint32_t*)&tab[p].val, (uint32_t)i);  /* a repeated id keeps its first position */
        }
#pragma omp for schedule(static)
        for (int64_t e = 0; e < n_edges; ++e) {
            int64_t p = orc_claim(tab, mask, shift, src[e]);
            slot_of[e] = p;
            orc_atomic_min_u32((uint32_t*)&tab[p].val, ORC_PENDING | (uint32_t)e);  /* no effect on numbered ids */
        }
        /* first mentions of new ids: count per thread (static schedule = contiguous, ordered ranges) */
        int64_t lo = n_edges * t / nt, hi = n_edges * (t + 1) / nt, cnt = 0;
        for (int64_t e = lo; e < hi; ++e) cnt += ((uint32_t)tab[slot_of[e]].val == (ORC_PENDING | (uint32_t)e));
        part[t + 1] = cnt;
#pragma omp barrier
#pragma omp single
        {
            for (int i = 0; i < nt; ++i) part[i + 1] += part[i];
            n_new = part[nt];
        }
        if (n_dst + n_new <= uniq_capacity) {
            int64_t next = n_dst + part[t];
            for (int64_t e = lo; e < hi; ++e) {
                if ((uint32_t)tab[slot_of[e]].val == (ORC_PENDING | (uint32_t)e)) {
                    uniq[next] = src[e];
                    slot_of[e] = -1 - next;  /* the slot's val is replaced after the barrier: others still compare against it */
                    ++next;
                }
            }
#pragma omp barrier
            for (int64_t e = lo; e < hi; ++e)
                if (slot_of[e] < 0) {
                    int64_t p = orc_claim(tab, mask, shift, src[e]);
                    tab[p].val = (int32_t)(-1 - slot_of[e]);
                    slot_of[e] = p;
                }
#pragma omp barrier
            for (int64_t e = lo; e < hi; ++e) src[e] = tab[slot_of[e]].val;
        }
    }
    int64_t rc = (n_dst + n_new <= uniq_capacity) ? n_dst + n_new : -2;
    free(part);
    free(slot_of);
    free(tab);
    return rc;
}

/* cal_deg (reference: utilis.cu:43-79): deg[ids[e]] += 1 over a zeroed array. */
ORC_API void orc_cal_deg(const int32_t* ids, int64_t n_ids, int32_t* deg, int64_t n_nodes)
{
    memset(deg, 0, sizeof(int32_t) * (size_t)n_nodes);
    for (int64_t e = 0; e < n_ids; ++e) deg[ids[e]] += 1;
}

/* exclusive_sum (reference: utilis.cu:17-41): pad one 0, exclusive scan -> n+1 entries. */
ORC_API void orc_exclusive_sum(const int32_t* deg, int64_t n, int32_t* out)
{
    int32_t run = 0;
    for (int64_t i = 0; i < n; ++i) { out[i] = run; run += deg[i]; }
    out[n] = run;
}

/* Stable transpose of a block CSR: row r of the result lists, in increasing order, the
 * rows of the input that contain column r.  (The backward kernels of the reference,
 * aggregate_acc_kernel.cu:467-517,554-596, scatter along exactly these lists.) */
ORC_API void orc_transpose(const int32_t* indptr, const int32_t* indices, int64_t n_rows, int64_t n_cols,
                           int32_t* t_indptr, int32_t* t_indices)
{
    int64_t nnz = indptr[n_rows];
    memset(t_indptr, 0, sizeof(int32_t) * (size_t)(n_cols + 1));
    for (int64_t e = 0; e < nnz; ++e) t_indptr[indices[e] + 1] += 1;
    for (int64_t c = 0; c < n_cols; ++c) t_indptr[c + 1] += t_indptr[c];
    int32_t* cur = (int32_t*)malloc(sizeof(int32_t) * (size_t)(n_cols > 0 ? n_cols : 1));
    memcpy(cur, t_indptr, sizeof(int32_t) * (size_t)n_cols);
    for (int64_t r = 0; r < n_rows; ++r)
        for (int64_t e = indptr[r]; e < indptr[r + 1]; ++e) t_indices[cur[indices[e]]++] = (int32_t)r;
    free(cur);
}

/* ------------------------------------------------------------------------------------
 * Aggregation (reference: aggregate_acc_kernel.cu:270-331 GCN forward, :375-427 GIN
 * forward; the backward kernels :467-517,:554-596 are the same sums over the transposed
 * lists with the same per-edge weight).
 *   mode 0  sum      w = 1
 *   mode 1  mean     w = 1 / deg(row)                 (not in the reference; sum / deg)
 *   mode 2  gcn      w = (1/sqrt(row_norm[row])) * (1/sqrt(col_norm[col]))
 *   mode 3  colmean  w = 1 / max(col_norm[col], 1)    (transpose of mode 1)
 * Rows with no entries: zero_policy 0 copies X[row] (reference :307-309,:405-407),
 * zero_policy 1 writes zeros.  Accumulation in double; X is fp32, row stride ldx.
 * ---------------------------------------------------------------------------------- */
ORC_API void orc_aggregate_f64(const int32_t* indptr, const int32_t* indices, int64_t n_rows,
                               const float* X, int64_t ldx, int D, int mode, int zero_policy,
                               const int32_t* row_norm, const int32_t* col_norm, double* out)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t r = 0; r < n_rows; ++r) {
        double* o = out + r * (int64_t)D;
        int64_t a = indptr[r], b = indptr[r + 1];
        if (a == b) {
            for (int f = 0; f < D; ++f) o[f] = zero_policy == 0 ? (double)X[r * ldx + f] : 0.0;
            continue;
        }
        for (int f = 0; f < D; ++f) o[f] = 0.0;
        for (int64_t e = a; e < b; ++e) {
            int64_t c = indices[e];
            double w = 1.0;
            if (mode == 1) w = 1.0 / (double)(b - a);
            else if (mode == 2) w = (1.0 / sqrt((double)row_norm[r])) * (1.0 / sqrt((double)col_norm[c]));
            else if (mode == 3) w = 1.0 / (double)(col_norm[c] > 1 ? col_norm[c] : 1);
            const float* x = X + c * ldx;
            for (int f = 0; f < D; ++f) o[f] += w * (double)x[f];
        }
    }
}

/* Attention-weighted aggregation (reference: aggregate_acc_kernel.cu:835-886 forward,
 * :924-979 backward on the transposed lists):
 *   out[r, f] = sum_e edge_w[id(e) * n_heads + f / (D / n_heads)] * X[indices[e], f]
 * with id(e) = edge_index ? edge_index[e] : e.  Rows without entries as in orc_aggregate_f64. */
ORC_API void orc_aggregate_edge_f64(const int32_t* indptr, const int32_t* indices, int64_t n_rows,
                                    const float* X, int64_t ldx, int D, int zero_policy, const float* edge_w,
                                    int n_heads, const int32_t* edge_index, double* out)
{
    const int unit = D / n_heads;
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t r = 0; r < n_rows; ++r) {
        double* o = out + r * (int64_t)D;
        int64_t a = indptr[r], b = indptr[r + 1];
        if (a == b) {
            for (int f = 0; f < D; ++f) o[f] = zero_policy == 0 ? (double)X[r * ldx + f] : 0.0;
            continue;
        }
        for (int f = 0; f < D; ++f) o[f] = 0.0;
        for (int64_t e = a; e < b; ++e) {
            const float* x = X + (int64_t)indices[e] * ldx;
            const float* w = edge_w + (int64_t)(edge_index ? edge_index[e] : e) * n_heads;
            for (int f = 0; f < D; ++f) o[f] += (double)w[f / unit] * (double)x[f];
        }
    }
}

/* GAT attention coefficients (reference: GraphConv.py:265-272, which calls DGL 1.0's
 * apply_edges(fn.u_add_v), torch's LeakyReLU and dgl.nn.functional.edge_softmax; DGL is not
 * part of the reference checkout, so their published definitions are restated):
 *   s(e, h)     = leaky_relu(el[indices[e], h] + er[r, h])   for entry e of destination row r
 *   alpha(e, h) = exp(s(e, h)) / sum over the entries e' of row r of exp(s(e', h))
 * computed in fp64 with the row maximum subtracted. */
ORC_API void orc_edge_softmax_f64(const int32_t* indptr, const int32_t* indices, int64_t n_rows, const float* el,
                                  const float* er, int n_heads, double negative_slope, double* alpha)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t r = 0; r < n_rows; ++r) {
        for (int h = 0; h < n_heads; ++h) {
            double top = -INFINITY, sum = 0.0;
            for (int64_t e = indptr[r]; e < indptr[r + 1]; ++e) {
                double s = (double)el[(int64_t)indices[e] * n_heads + h] + (double)er[r * n_heads + h];
                if (s < 0.0) s *= negative_slope;
                alpha[e * n_heads + h] = s;
                if (s > top) top = s;
            }
            for (int64_t e = indptr[r]; e < indptr[r + 1]; ++e) {
                alpha[e * n_heads + h] = exp(alpha[e * n_heads + h] - top);
                sum += alpha[e * n_heads + h];
            }
            for (int64_t e = indptr[r]; e < indptr[r + 1]; ++e) alpha[e * n_heads + h] /= sum;
        }
    }
}

/* fp32 variant used only to TIME a CPU aggregation next to the GPU kernel. */
ORC_API void orc_aggregate_f32(const int32_t* indptr, const int32_t* indices, int64_t n_rows,
                               const float* X, int64_t ldx, int D, int mode, int zero_policy,
                               const int32_t* row_norm, const int32_t* col_norm, float* out)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t r = 0; r < n_rows; ++r) {
        float* o = out + r * (int64_t)D;
        int64_t a = indptr[r], b = indptr[r + 1];
        if (a == b) {
            for (int f = 0; f < D; ++f) o[f] = zero_policy == 0 ? X[r * ldx + f] : 0.0f;
            continue;
        }
        for (int f = 0; f < D; ++f) o[f] = 0.0f;
        for (int64_t e = a; e < b; ++e) {
            int64_t c = indices[e];
            float w = 1.0f;
            if (mode == 1) w = 1.0f / (float)(b - a);
            else if (mode == 2) w = (1.0f / sqrtf((float)row_norm[r])) * (1.0f / sqrtf((float)col_norm[c]));
            else if (mode == 3) w = 1.0f / (float)(col_norm[c] > 1 ? col_norm[c] : 1);
            const float* x = X + c * ldx;
            for (int f = 0; f < D; ++f) o[f] += w * x[f];
        }
    }
}

/* ------------------------------------------------------------------------------------
 * Seeded R-MAT edge generator (the synthetic graphs the benchmark configurations name:
 * a=.57 b=.19 c=.19 d=.05).  Edge number e draws one quadrant per level from
 * Philox4x32-10 with counter {e_lo, e_hi, level/4, 0x524D4154} and key = seed; word
 * (level%4) of the block is compared with integer cut points, so CPU and GPU agree bit
 * for bit.  Emits, per drawn edge (u,v), the two keys (v<<32|u) and (u<<32|v)
 * (symmetrised; key = row<<32 | column of the in-neighbour CSR).  Self loops and
 * endpoints >= n_nodes give INT64_MAX twice (sorted to the end, dropped by the caller).
 * ---------------------------------------------------------------------------------- */
#define ORC_RMAT_CUT_A 0x91EB851Eu /* floor(0.57 * 2^32) */
#define ORC_RMAT_CUT_B 0xC28F5C28u /* floor(0.76 * 2^32) */
#define ORC_RMAT_CUT_C 0xF3333333u /* floor(0.95 * 2^32) */

ORC_API void orc_rmat_keys(int64_t first_edge, int64_t n_edges, int scale, int64_t n_nodes, uint64_t seed, int64_t* keys)
{
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
#pragma omp parallel for schedule(static)
    for (int64_t x = 0; x < n_edges; ++x) {
        uint64_t e = (uint64_t)(first_edge + x);
        uint64_t u = 0, v = 0;
        uint32_t o[4] = {0, 0, 0, 0};
        for (int lvl = 0; lvl < scale; ++lvl) {
            if ((lvl & 3) == 0) {
                uint32_t ctr[4] = {(uint32_t)e, (uint32_t)(e >> 32), (uint32_t)(lvl >> 2), 0x524D4154u};
                orc_philox4x32_10(ctr, key, o);
            }
            uint32_t r = o[lvl & 3];
            uint32_t ub = r >= ORC_RMAT_CUT_B;                               /* quadrants c,d: row bit 1 */
            uint32_t vb = (r >= ORC_RMAT_CUT_A && r < ORC_RMAT_CUT_B) || r >= ORC_RMAT_CUT_C; /* b,d: col bit 1 */
            u = (u << 1) | ub;
            v = (v << 1) | vb;
        }
        if (u == v || u >= (uint64_t)n_nodes || v >= (uint64_t)n_nodes) {
            keys[2 * x] = INT64_MAX; keys[2 * x + 1] = INT64_MAX;
        } else {
            keys[2 * x] = (int64_t)((v << 32) | u);
            keys[2 * x + 1] = (int64_t)((u << 32) | v);
        }
    }
}

ORC_API int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
