// Attention coefficients of a GAT layer over a block CSR: for every destination row r and head h
//   s(e)     = leaky_relu(el[indices[e], h] + er[r, h])          e in [indptr[r], indptr[r+1])
//   alpha(e) = exp(s(e) - max_e' s(e')) / sum_e' exp(s(e') - max)
// -- what the reference gets from three DGL calls (apply_edges(u_add_v), leaky_relu,
// edge_softmax; GraphConv.py:265-272) and what a torch restatement spends ten launches over
// [n_entries, n_heads] on.  The result feeds FGL_AGG_EDGE as its per-entry weights.
//
// One lane per (row, head), the heads of a row in neighbouring lanes (they read the same
// neighbour id and 4 * n_heads contiguous bytes of el).  Two passes over the row's entries: a
// running maximum with a rescaled running sum, then the normalised values; the scores are
// recomputed in the second pass (the reads hit in cache) rather than kept.  Sampled blocks hold at
// most `fanout` entries per row; a hub row of an unsampled block is walked by its one lane.
#include "fgl_common.hpp"
#include "fgl_kernels.hpp"

namespace fgl {

__global__ __launch_bounds__(kBlock) void edge_softmax_kernel(const int32_t* __restrict__ indptr,
                                                              const int32_t* __restrict__ indices, int64_t n_rows_max,
                                                              const int32_t* __restrict__ d_n_rows,
                                                              const float* __restrict__ el, const float* __restrict__ er,
                                                              int n_heads, float negative_slope, float* __restrict__ alpha)
{
    const int64_t n_rows = actual_count(n_rows_max, d_n_rows);
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t row = t / n_heads;
    if (row >= n_rows) return;
    const int h = (int)(t - row * n_heads);
    const int a = indptr[row], b = indptr[row + 1];
    const float r = er[row * n_heads + h];
    float top = -INFINITY, sum = 0.0f;
    for (int e = a; e < b; ++e) {
        float s = el[(int64_t)indices[e] * n_heads + h] + r;
        s = s > 0.0f ? s : negative_slope * s;
        if (s > top) {
            sum = sum * expf(top - s) + 1.0f;  // (first entry: 0 * exp(-inf) + 1)
            top = s;
        } else {
            sum += expf(s - top);
        }
    }
    const float inv = 1.0f / sum;
    for (int e = a; e < b; ++e) {
        float s = el[(int64_t)indices[e] * n_heads + h] + r;
        s = s > 0.0f ? s : negative_slope * s;
        alpha[(int64_t)e * n_heads + h] = expf(s - top) * inv;
    }
}

}  // namespace fgl

using namespace fgl;

FGL_EXPORT int fgl_edge_softmax(const int32_t* d_indptr, const int32_t* d_indices, int64_t n_rows_max,
                                const int32_t* d_n_rows, const float* d_el, const float* d_er, int n_heads,
                                float negative_slope, float* d_alpha, void* stream)
{
    FGL_REQUIRE(n_rows_max >= 0, "edge_softmax: negative row count");
    FGL_REQUIRE(n_heads >= 1 && n_heads <= 1024, "edge_softmax: head count %d outside [1, 1024]", n_heads);
    if (n_rows_max == 0) return FGL_OK;
    FGL_REQUIRE(d_indptr && d_indices && d_el && d_er && d_alpha, "edge_softmax: null pointer");
    const int64_t blocks = ceil_div(n_rows_max * n_heads, kBlock);
    FGL_REQUIRE(blocks <= 0x7FFFFFFF, "edge_softmax: grid too large");
    hipLaunchKernelGGL(edge_softmax_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, as_stream(stream), d_indptr, d_indices,
                       n_rows_max, d_n_rows, d_el, d_er, n_heads, negative_slope, d_alpha);
    FGL_CHECK_LAUNCH("edge_softmax_kernel");
    return FGL_OK;
}
