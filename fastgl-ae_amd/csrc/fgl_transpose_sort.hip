// Deterministic variant of the block transpose: the entries of every column in ascending row
// order (which is ascending edge order), independent of scheduling.  A stable device-wide radix
// sort of (column -> edge index) pairs by rocPRIM (the library primitive, as the reference takes
// its scans from CUB, sample.cu:155-159) followed by one pass that names each edge's row.  Long
// columns (hub nodes) cost nothing extra, unlike a per-column sort.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

#include "fgl_common.hpp"
#include "fgl_kernels.hpp"

namespace fgl {

__global__ __launch_bounds__(kBlock) void transpose_rows_of_edges_kernel(const int32_t* __restrict__ indptr, int64_t n_rows,
                                                                         const int32_t* __restrict__ sorted_edge,
                                                                         int64_t n_edges, int32_t* __restrict__ t_indices)
{
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n_edges; i += stride) {
        const int32_t e = sorted_edge[i];
        int64_t lo = 0, hi = n_rows;  // indptr[lo] <= e < indptr[hi]
        while (hi - lo > 1) {
            const int64_t mid = (lo + hi) >> 1;
            if (indptr[mid] <= e) lo = mid; else hi = mid;
        }
        t_indices[i] = (int32_t)lo;
    }
}

static unsigned bits_for(int64_t n)
{
    unsigned b = 1;
    while (b < 32 && ((int64_t)1 << b) < n) ++b;
    return b;
}

size_t sorted_transpose_workspace_bytes(int64_t n_cols, int64_t n_edges)
{
    size_t temp = 0;
    (void)rocprim::radix_sort_pairs(nullptr, temp, (const int32_t*)nullptr, (int32_t*)nullptr,
                                    rocprim::counting_iterator<int32_t>(0), (int32_t*)nullptr, (size_t)n_edges, 0u,
                                    bits_for(n_cols), (hipStream_t)0);
    Carver c(nullptr);
    c.take<int32_t>((size_t)n_edges);  // sorted keys (discarded)
    c.take<int32_t>((size_t)n_edges);  // sorted edge ids when the caller does not want them
    c.take<char>(temp);
    return c.used();
}

// d_t_indptr must already hold the column offsets.
int launch_sorted_transpose_fill(const int32_t* d_indptr, const int32_t* d_indices, int64_t n_rows, int64_t n_cols,
                                 int64_t n_edges, int32_t* d_t_indices, int32_t* d_t_edge, void* d_ws, size_t ws_bytes,
                                 hipStream_t stream)
{
    if (n_edges == 0) return FGL_OK;
    if (d_ws == nullptr || ws_bytes < sorted_transpose_workspace_bytes(n_cols, n_edges)) {
        set_error("block_transpose: workspace too small for the sorted variant");
        return FGL_ERR_WORKSPACE;
    }
    size_t temp = 0;
    const unsigned end_bit = bits_for(n_cols);
    (void)rocprim::radix_sort_pairs(nullptr, temp, d_indices, (int32_t*)nullptr, rocprim::counting_iterator<int32_t>(0),
                                    (int32_t*)nullptr, (size_t)n_edges, 0u, end_bit, stream);
    Carver c(d_ws);
    int32_t* keys_out = c.take<int32_t>((size_t)n_edges);
    int32_t* edge_scratch = c.take<int32_t>((size_t)n_edges);
    char* temp_storage = c.take<char>(temp);
    int32_t* sorted_edge = d_t_edge ? d_t_edge : edge_scratch;
    hipError_t err = rocprim::radix_sort_pairs(temp_storage, temp, d_indices, keys_out, rocprim::counting_iterator<int32_t>(0),
                                               sorted_edge, (size_t)n_edges, 0u, end_bit, stream);
    if (err != hipSuccess) {
        set_error("block_transpose: radix sort failed: %s", hipGetErrorString(err));
        return FGL_ERR_HIP;
    }
    int64_t blocks = ceil_div(n_edges, kBlock);
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(transpose_rows_of_edges_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, d_indptr, n_rows,
                       sorted_edge, n_edges, d_t_indices);
    FGL_CHECK_LAUNCH("transpose_rows_of_edges_kernel");
    return FGL_OK;
}

}  // namespace fgl
