// The torch extension module `fastgl`: the operators that the reference's Python code calls
// (cuda_operators/aggregate_acc.cpp:601-621 registers them; FusedMapSampler.py:76,98 and
// GraphConv.py:26,37,93-96,109,132,204,224 call them), with the reference's names, positional
// arguments and return lists, forwarding to the C ABI of libfastgl_hip.so.
//
// Host code only: compiled with g++ against the torch headers and linked with libfastgl_hip.so; torch
// owns the device memory and names the stream, every kernel lives behind include/fastgl_hip.h.
// Errors surface as c10::Error (a Python RuntimeError), as the reference's CHECK_INPUT does
// (aggregate_acc.cpp:4-6); the device status word of the id-map and the sampler is read back with the
// sizes (the reference reads its sizes back at the same points: sample.cu:202, id_map.cu:454,491).
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <c10/hip/HIPGuard.h>

#include <atomic>
#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "fastgl_hip.h"

namespace {

#define CHECK_CUDA(x) TORCH_CHECK((x).is_cuda(), #x " must be a CUDA tensor")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define CHECK_INPUT(x) \
    CHECK_CUDA(x);     \
    CHECK_CONTIGUOUS(x)
#define CHECK_I32(x) \
    CHECK_INPUT(x);  \
    TORCH_CHECK((x).scalar_type() == torch::kInt32, #x " must be int32")
#define CHECK_FEAT(x)                                                                                   \
    CHECK_INPUT(x);                                                                                     \
    TORCH_CHECK((x).scalar_type() == torch::kFloat32 || (x).scalar_type() == torch::kBFloat16, #x " must be float32 or bfloat16")

void ok(int rc)
{
    TORCH_CHECK(rc == FGL_OK, "fastgl: ", fgl_last_error(), " (error ", rc, ")");
}

void* stream_of(const torch::Tensor& t) { return c10::hip::getCurrentHIPStream(t.get_device()).stream(); }

torch::Tensor scratch(size_t bytes, const torch::Tensor& like)
{
    return torch::empty({(int64_t)(bytes > 0 ? bytes : 1)}, like.options().dtype(torch::kUInt8));
}

void raise_status(uint32_t bits, const char* where)
{
    if (bits == 0) return;
    std::string what;
    auto add = [&](const char* s) { what += (what.empty() ? "" : ", "); what += s; };
    if (bits & FGL_STATUS_TABLE_FULL) add("hash table full");
    if (bits & FGL_STATUS_UNIQ_OVERFLOW) add("more unique ids than the output holds");
    if (bits & FGL_STATUS_MISSING_KEY) add("an id to relabel is not in the map");
    if (bits & FGL_STATUS_BAD_SEED) add("a seed id lies outside the graph");
    if (bits & FGL_STATUS_BAD_ID) add("a negative id was handed to the id-map");
    TORCH_CHECK(false, "fastgl.", where, ": ", what);
}

// Philox streams of sample_node: one seed for the process, one stream per call (the reference draws every
// call from the same constant stream, sample.cu:70)
std::atomic<uint64_t> g_rng_seed{0};
std::atomic<uint32_t> g_rng_calls{0};

void manual_seed(uint64_t seed)
{
    g_rng_seed = seed;
    g_rng_calls = 0;
}

// What sample_node and transfer_edge_id keep between calls, per (device, stream): the reference allocates, fills and
// frees its hash table and scratch on every call (id_map.cu:45-59,408-409; sample.cu:118,151,157) and reads its sizes
// back through pageable memory.  Here the table persists and is left empty by each call's last pass (so no call pays
// for a fill once the largest table has been seen), the scratch persists, and the two words that the host needs --
// a size and the status -- come back through one pinned buffer.
struct CallState {
    torch::Tensor table;      // int64 slots; grows to the largest table asked for
    int64_t empty_slots = 0;  // slots [0, empty_slots) hold the empty marker (0: nothing is known)
    torch::Tensor ws;         // uint8 scratch, grows on demand
    torch::Tensor meta;       // device int32[2]: {size, status}; the status word is zero between calls
    torch::Tensor host;       // pinned int32[2] that the kernels write themselves: {size, status} of the call at hand
};

CallState& call_state(const torch::Tensor& like)
{
    static std::mutex mu;
    static std::map<std::pair<int, void*>, CallState> states;
    const int dev = like.get_device();
    void* stream = c10::hip::getCurrentHIPStream(dev).stream();
    std::lock_guard<std::mutex> lock(mu);
    CallState& st = states[{dev, stream}];
    if (!st.meta.defined()) {
        st.meta = torch::zeros({2}, like.options().dtype(torch::kInt32));
        st.host = torch::empty({2}, torch::TensorOptions().dtype(torch::kInt32).pinned_memory(true));
    }
    return st;
}

void* grown(torch::Tensor& buf, size_t bytes, const torch::Tensor& like)
{
    if (!buf.defined() || (size_t)buf.numel() < bytes)
        buf = torch::empty({(int64_t)std::max<size_t>(bytes, (size_t)1 << 20)}, like.options().dtype(torch::kUInt8));
    return buf.data_ptr();
}

// {size, status} of a call.  The call's own launches write both words into the pinned buffer (device-writable host
// memory), so there is no copy to enqueue: expect() marks the words as pending before the call is enqueued, and
// read_back() looks at them until they have been overwritten -- which the launch that knows the size does when it
// starts, so the host is back at work while the call's last kernel is still running (and falls back to a stream
// wait after a few milliseconds).  A non-zero status word is cleared on the device again (the kernels only ever
// or into it).
// (Polling hipStreamQuery instead was measured: 0.34 -> 0.40 ms per three-hop mini-batch.)
constexpr int32_t kPendingWord = -1;  // no size and no status word is all ones

int32_t* expect(CallState& st)
{
    int32_t* h = st.host.data_ptr<int32_t>();
    h[0] = h[1] = kPendingWord;
    return h;
}

std::pair<int64_t, uint32_t> read_back(CallState& st, void* stream)
{
    ok(fgl_wait_words(st.host.data_ptr<int32_t>(), 2, kPendingWord, stream, 5000));
    const volatile int32_t* h = st.host.data_ptr<int32_t>();
    const std::pair<int64_t, uint32_t> out{h[0], (uint32_t)h[1]};
    if (out.second != 0) st.meta.zero_();
    return out;
}

int dtype_of(const torch::Tensor& t) { return t.scalar_type() == torch::kFloat32 ? FGL_F32 : FGL_BF16; }

// out[r] = sum_e w * feat[indices[e]] through fgl_aggregate; longest_row < 0: nothing known about the rows
torch::Tensor aggregate(const torch::Tensor& indptr, const torch::Tensor& indices, const torch::Tensor& feat, int64_t n_rows,
                        int mode, int zero_policy, const torch::Tensor* row_norm, const torch::Tensor* col_norm,
                        const torch::Tensor* edge_w, int n_heads, const torch::Tensor* edge_index, int64_t longest_row,
                        const torch::Tensor* longest_dev)
{
    TORCH_CHECK(feat.dim() == 2, "features must be 2-D");
    TORCH_CHECK(n_rows >= 0 && n_rows <= indptr.numel() - 1, "row count ", n_rows, " does not match the offsets (", indptr.numel(), " entries)");
    TORCH_CHECK(zero_policy != FGL_ZERO_COPY_SELF || n_rows <= feat.size(0), "features must have a row for every output row");
    const int64_t D = feat.size(1);
    auto out = torch::empty({n_rows, D}, feat.options());
    if (n_rows == 0) return out;
    const void* idx = indices.numel() ? indices.data_ptr() : indptr.data_ptr();  // a block without entries: never read
    ok(fgl_aggregate(indptr.data_ptr<int32_t>(), static_cast<const int32_t*>(idx), n_rows, nullptr, feat.data_ptr(), feat.stride(0),
                     (int)D, dtype_of(feat), mode, zero_policy, row_norm ? row_norm->data_ptr<int32_t>() : nullptr,
                     col_norm ? col_norm->data_ptr<int32_t>() : nullptr, edge_w ? edge_w->data_ptr<float>() : nullptr, n_heads,
                     edge_index ? edge_index->data_ptr<int32_t>() : nullptr, longest_row,
                     longest_dev ? longest_dev->data_ptr<int32_t>() : nullptr, indices.numel(), out.data_ptr(), out.stride(0),
                     stream_of(feat)));
    return out;
}

struct Transposed {
    torch::Tensor ptr, idx, edge, longest;
};

Transposed transpose(const torch::Tensor& indptr, const torch::Tensor& indices, int64_t n_rows, int64_t n_cols, bool edge_ids)
{
    const int64_t nnz = indices.numel();
    TORCH_CHECK(n_rows >= 0 && n_rows <= indptr.numel() - 1, "row count ", n_rows, " does not match the offsets (", indptr.numel(), " entries)");
    TORCH_CHECK(n_cols >= 0, "negative node count");
    auto opt = indptr.options();
    Transposed t;
    t.ptr = torch::empty({n_cols + 1}, opt);
    t.idx = torch::empty({nnz > 0 ? nnz : 1}, opt).slice(0, 0, nnz);
    if (edge_ids) t.edge = torch::empty({nnz > 0 ? nnz : 1}, opt).slice(0, 0, nnz);
    t.longest = torch::empty({1}, opt);
    auto ws = scratch(fgl_block_transpose_workspace_bytes(n_cols, nnz, 0), indptr);
    ok(fgl_block_transpose(indptr.data_ptr<int32_t>(), nnz ? indices.data_ptr<int32_t>() : nullptr, n_rows, nullptr, n_cols, nullptr,
                           nnz, t.ptr.data_ptr<int32_t>(), nnz ? t.idx.data_ptr<int32_t>() : nullptr,
                           (edge_ids && nnz) ? t.edge.data_ptr<int32_t>() : nullptr, t.longest.data_ptr<int32_t>(), 0,
                           ws.data_ptr(), (size_t)ws.numel(), stream_of(indptr)));
    return t;
}

// ---- the reference's operators ---------------------------------------------------------------------

// aggregate_acc.cpp:491-512 (sample.cu:102-203).  dst_edges is accepted and, as in the reference's kernels, never read.
std::vector<torch::Tensor> sample_node(torch::Tensor src_edges, torch::Tensor dst_edges, torch::Tensor edge_ptr,
                                       torch::Tensor seed_nodes, int dst_nodes, int neighbor_num)
{
    CHECK_I32(src_edges);
    CHECK_INPUT(dst_edges);
    CHECK_INPUT(edge_ptr);
    TORCH_CHECK(edge_ptr.scalar_type() == torch::kInt32 || edge_ptr.scalar_type() == torch::kInt64, "edge_ptr must be int32 or int64");
    CHECK_I32(seed_nodes);
    const int64_t n_seeds = seed_nodes.size(0);
    TORCH_CHECK(dst_nodes >= n_seeds, "dst_nodes (", dst_nodes, ") is smaller than the number of seeds (", n_seeds, ")");
    TORCH_CHECK(neighbor_num >= 1 && neighbor_num <= FGL_MAX_FANOUT, "neighbor_num outside [1, ", FGL_MAX_FANOUT, "]");
    c10::hip::HIPGuard guard(seed_nodes.get_device());
    auto opt = seed_nodes.options();
    const int64_t cap = std::max<int64_t>((int64_t)dst_nodes * neighbor_num, 1);
    auto src_out = torch::empty({cap}, opt), dst_out = torch::empty({cap}, opt);
    auto block_ptr = torch::empty({n_seeds + 1}, opt);
    CallState& st = call_state(seed_nodes);
    const size_t ws_bytes = fgl_sample_workspace_bytes(n_seeds, neighbor_num);
    void* ws = grown(st.ws, ws_bytes, seed_nodes);
    void* stream = stream_of(seed_nodes);
    int32_t* meta = st.meta.data_ptr<int32_t>();
    ok(fgl_sample_node(edge_ptr.data_ptr(), edge_ptr.scalar_type() == torch::kInt64, src_edges.data_ptr<int32_t>(),
                       edge_ptr.size(0) - 1, seed_nodes.data_ptr<int32_t>(), n_seeds, nullptr, neighbor_num, g_rng_seed.load(),
                       g_rng_calls.fetch_add(1), src_out.data_ptr<int32_t>(), dst_out.data_ptr<int32_t>(), block_ptr.data_ptr<int32_t>(),
                       meta, reinterpret_cast<uint32_t*>(meta) + 1, expect(st), ws, (size_t)st.ws.numel(), stream));
    const auto back = read_back(st, stream);  // the read-back of sample.cu:202
    raise_status(back.second, "sample_node");
    // (the edge count as a device tensor, as the reference returns it: the last entry of the block's row pointer)
    return {src_out.slice(0, 0, back.first), dst_out.slice(0, 0, back.first), block_ptr.slice(0, n_seeds, n_seeds + 1)};
}

// aggregate_acc.cpp:467-489 (id_map.cu:386-493): in-place relabelling; uniq = cat(dst_edges_unique, new source ids
// in first-occurrence order).
std::vector<torch::Tensor> transfer_edge_id(torch::Tensor src_edges, torch::Tensor dst_edges, torch::Tensor dst_edges_unique,
                                            int dst_nodes, int total_items, int unique_num, long int edge_nums)
{
    CHECK_I32(src_edges);
    CHECK_I32(dst_edges);
    CHECK_I32(dst_edges_unique);
    const int64_t n_dst = dst_nodes, n_edges = edge_nums;
    TORCH_CHECK(n_dst >= 0 && n_dst <= dst_edges_unique.size(0), "dst_nodes (", n_dst, ") exceeds len(dst_edges_unique)");
    TORCH_CHECK(n_edges >= 0 && n_edges <= src_edges.size(0) && n_edges <= dst_edges.size(0), "edge_nums (", n_edges, ") exceeds the edge arrays");
    TORCH_CHECK((int64_t)total_items - n_dst == n_edges, "total_items - dst_nodes must equal edge_nums (id_map.cu:308)");
    c10::hip::HIPGuard guard(src_edges.get_device());
    const int64_t max_new = std::max<int64_t>(0, std::min<int64_t>(unique_num, n_edges));
    const int64_t capacity = n_dst + max_new;
    const int64_t slots = fgl_idmap_slots(capacity);
    auto opt = src_edges.options();
    auto uniq = torch::empty({std::max<int64_t>(capacity, 1)}, opt);
    CallState& st = call_state(src_edges);
    void* stream = stream_of(src_edges);
    if (!st.table.defined() || st.table.numel() < slots) {
        st.table = torch::empty({slots}, opt.dtype(torch::kInt64));
        st.empty_slots = 0;
    }
    void* table = st.table.data_ptr();
    // the table is a prefix of the persistent buffer; whatever part of it is not known to be empty is filled now
    // (in the steady state of a training loop: never)
    if (st.empty_slots < slots) ok(fgl_idmap_reset(table, slots, stream));
    const int64_t known_empty = std::max(st.empty_slots, slots);
    st.empty_slots = 0;  // (until the call's last pass has been enqueued)
    const size_t ws_bytes = fgl_idmap_map_src_workspace_bytes(n_edges);
    void* ws = grown(st.ws, ws_bytes, src_edges);
    int32_t* meta = st.meta.data_ptr<int32_t>();
    uint32_t* status = reinterpret_cast<uint32_t*>(meta) + 1;
    TORCH_CHECK(n_edges == 0 || src_edges.data_ptr() != dst_edges.data_ptr(), "src_edges and dst_edges must be distinct tensors");
    // destination ids in, then three passes over the edges (the destination half rides on the first); the last pass
    // neither writes the new ids' numbers back into the table (nobody will look them up: the next call brings its
    // own destination list) nor leaves anything in it
    ok(fgl_idmap_transfer(table, slots, dst_edges_unique.data_ptr<int32_t>(), n_dst, src_edges.data_ptr<int32_t>(),
                          dst_edges.data_ptr<int32_t>(), n_edges, uniq.data_ptr<int32_t>(), capacity,
                          FGL_IDMAP_ORDERED | FGL_IDMAP_FINAL | FGL_IDMAP_LEAVE_TABLE_EMPTY, meta, status, expect(st), ws,
                          (size_t)st.ws.numel(), stream));
    st.empty_slots = known_empty;
    const auto back = read_back(st, stream);  // the read-back of id_map.cu:454,491
    raise_status(back.second, "transfer_edge_id");
    return {src_edges, dst_edges, uniq.slice(0, 0, back.first)};
}

// aggregate_acc.cpp:522-529 (utilis.cu:43-79)
torch::Tensor cal_deg(torch::Tensor edges, int nodes_num)
{
    CHECK_I32(edges);
    TORCH_CHECK(nodes_num >= 0, "negative node count");
    c10::hip::HIPGuard guard(edges.get_device());
    auto deg = torch::empty({std::max(nodes_num, 1)}, edges.options()).slice(0, 0, nodes_num);
    ok(fgl_cal_deg(edges.data_ptr<int32_t>(), edges.numel(), nullptr, deg.data_ptr<int32_t>(), nodes_num, stream_of(edges)));
    return deg;
}

// aggregate_acc.cpp:514-520 (utilis.cu:17-41)
torch::Tensor exclusive_sum(torch::Tensor in_degs)
{
    CHECK_I32(in_degs);
    c10::hip::HIPGuard guard(in_degs.get_device());
    const int64_t n = in_degs.numel();
    auto out = torch::empty({n + 1}, in_degs.options());
    auto ws = scratch(fgl_exclusive_sum_workspace_bytes(n), in_degs);
    ok(fgl_exclusive_sum_i32(in_degs.data_ptr<int32_t>(), n, nullptr, out.data_ptr<int32_t>(), ws.data_ptr(), (size_t)ws.numel(),
                             stream_of(in_degs)));
    return out;
}

// aggregate_acc.cpp:133-160 (kernel aggregate_acc_kernel.cu:270-331): [A_norm (X W)]
std::vector<torch::Tensor> forward_gcn(torch::Tensor edge_ptr, torch::Tensor src_edges, torch::Tensor src_norm_degs,
                                       torch::Tensor dst_norm_degs, torch::Tensor input_feat, torch::Tensor weight,
                                       int neighbor_num, int dst_nodes)
{
    CHECK_I32(edge_ptr);
    CHECK_I32(src_edges);
    CHECK_I32(src_norm_degs);
    CHECK_I32(dst_norm_degs);
    CHECK_FEAT(input_feat);
    CHECK_FEAT(weight);
    c10::hip::HIPGuard guard(input_feat.get_device());
    auto tmp = torch::mm(input_feat, weight);
    return {aggregate(edge_ptr, src_edges, tmp, dst_nodes, FGL_AGG_GCN, FGL_ZERO_COPY_SELF, &dst_norm_degs, &src_norm_degs, nullptr, 1,
                      nullptr, neighbor_num > 0 ? neighbor_num : -1, nullptr)};
}

// aggregate_acc.cpp:349-376 (kernel :467-517).  As in the reference's kernel the third argument is indexed by
// destination and the fourth by source (:494,509); the caller passes (dst_norm, src_norm) there (GraphConv.py:37).
std::vector<torch::Tensor> backward_gcn(torch::Tensor edge_ptr, torch::Tensor src_edges, torch::Tensor src_norm_degs,
                                        torch::Tensor dst_norm_degs, torch::Tensor d_input, torch::Tensor weight,
                                        torch::Tensor input_feat)
{
    CHECK_I32(edge_ptr);
    CHECK_I32(src_edges);
    CHECK_I32(src_norm_degs);
    CHECK_I32(dst_norm_degs);
    CHECK_FEAT(d_input);
    CHECK_FEAT(weight);
    CHECK_FEAT(input_feat);
    c10::hip::HIPGuard guard(d_input.get_device());
    const torch::Tensor &by_dst = src_norm_degs, &by_src = dst_norm_degs;
    const int64_t n_src = input_feat.size(0), n_dst = d_input.size(0);
    auto t = transpose(edge_ptr, src_edges, n_dst, n_src, false);
    auto g = aggregate(t.ptr, t.idx, d_input, n_src, FGL_AGG_GCN, FGL_ZERO_ZEROS, &by_src, &by_dst, nullptr, 1, nullptr, -1, &t.longest);
    return {torch::mm(g, weight.transpose(0, 1)), torch::mm(input_feat.transpose(0, 1), g)};
}

// aggregate_acc.cpp:173-199, exported under this spelling at :613 (kernel :375-427): [tmp W, tmp]
std::vector<torch::Tensor> forwaed_gin(torch::Tensor edge_ptr, torch::Tensor src_edges, torch::Tensor input_feat, torch::Tensor weight,
                                       int neighbor_num, int dst_nodes)
{
    CHECK_I32(edge_ptr);
    CHECK_I32(src_edges);
    CHECK_FEAT(input_feat);
    CHECK_FEAT(weight);
    c10::hip::HIPGuard guard(input_feat.get_device());
    auto tmp = aggregate(edge_ptr, src_edges, input_feat, dst_nodes, FGL_AGG_SUM, FGL_ZERO_COPY_SELF, nullptr, nullptr, nullptr, 1, nullptr,
                         neighbor_num > 0 ? neighbor_num : -1, nullptr);
    return {torch::mm(tmp, weight), tmp};
}

// aggregate_acc.cpp:387-409 (kernel :554-596); input_feat is the tmp that forwaed_gin returned
std::vector<torch::Tensor> backward_gin(torch::Tensor edge_ptr, torch::Tensor src_edges, torch::Tensor d_input, torch::Tensor weight,
                                        torch::Tensor input_feat, int src_nodes)
{
    CHECK_I32(edge_ptr);
    CHECK_I32(src_edges);
    CHECK_FEAT(d_input);
    CHECK_FEAT(weight);
    CHECK_FEAT(input_feat);
    c10::hip::HIPGuard guard(d_input.get_device());
    auto d_tmp = torch::mm(d_input, weight.transpose(0, 1));
    auto d_w = torch::mm(input_feat.transpose(0, 1), d_input);
    auto t = transpose(edge_ptr, src_edges, d_input.size(0), src_nodes, false);
    auto d_x = aggregate(t.ptr, t.idx, d_tmp, src_nodes, FGL_AGG_SUM, FGL_ZERO_ZEROS, nullptr, nullptr, nullptr, 1, nullptr, -1, &t.longest);
    return {d_x, d_w};
}

// aggregate_acc.cpp:211-236 (kernel aggregate_acc_kernel.cu:835-886): out[d, f] = sum_e edge_data[e, head(f)] * X[src[e], f]
std::vector<torch::Tensor> forward_gat(torch::Tensor edge_ptr, torch::Tensor edge_data, torch::Tensor src_edges,
                                       torch::Tensor input_feat, int neighbor_num, int dst_nodes, int num_heads)
{
    CHECK_I32(edge_ptr);
    CHECK_I32(src_edges);
    CHECK_INPUT(edge_data);
    TORCH_CHECK(edge_data.scalar_type() == torch::kFloat32, "edge_data must be float32");
    CHECK_FEAT(input_feat);
    TORCH_CHECK(num_heads >= 1 && input_feat.size(1) % num_heads == 0, "num_heads must divide the feature length");
    TORCH_CHECK(edge_data.numel() >= src_edges.numel() * num_heads, "edge_data has fewer rows than there are edges");
    c10::hip::HIPGuard guard(input_feat.get_device());
    auto w = edge_data.view({-1, num_heads});
    return {aggregate(edge_ptr, src_edges, input_feat, dst_nodes, FGL_AGG_EDGE, FGL_ZERO_COPY_SELF, nullptr, nullptr, &w, num_heads, nullptr,
                      -1, nullptr)};
}

// kernel aggregate_acc_kernel.cu:924-979: d_x[s, f] = sum over the edges (s -> d) of edge_data[e, head(f)] * d_input[d, f]
std::vector<torch::Tensor> backward_gat(torch::Tensor edge_ptr, torch::Tensor edge_data, torch::Tensor src_edges, torch::Tensor d_input,
                                        int src_nodes, int num_heads)
{
    CHECK_I32(edge_ptr);
    CHECK_I32(src_edges);
    CHECK_INPUT(edge_data);
    TORCH_CHECK(edge_data.scalar_type() == torch::kFloat32, "edge_data must be float32");
    CHECK_FEAT(d_input);
    TORCH_CHECK(num_heads >= 1 && d_input.size(1) % num_heads == 0, "num_heads must divide the feature length");
    c10::hip::HIPGuard guard(d_input.get_device());
    auto w = edge_data.view({-1, num_heads});
    auto t = transpose(edge_ptr, src_edges, d_input.size(0), src_nodes, true);
    return {aggregate(t.ptr, t.idx, d_input, src_nodes, FGL_AGG_EDGE, FGL_ZERO_ZEROS, nullptr, nullptr, &w, num_heads, &t.edge, -1, &t.longest)};
}

}  // namespace

PYBIND11_MODULE(fastgl, m)
{
    m.doc() = "FastGL operators on MI355X (libfastgl_hip.so behind the reference's operator names)";
    m.def("cal_deg", &cal_deg, "cal_deg (HIP)");
    m.def("exclusive_sum", &exclusive_sum, "exclusive_sum (HIP)");
    m.def("transfer_edge_id", &transfer_edge_id, "transfer_edge_id (HIP)");
    m.def("sample_node", &sample_node, "sample_node (HIP)");
    m.def("forward_gcn", &forward_gcn, "computation_aware_forward_gcn (HIP)");
    m.def("forwaed_gin", &forwaed_gin, "computation_aware_forward_gin (HIP)");
    m.def("forward_gat", &forward_gat, "computation_aware_forward_gat (HIP)");
    m.def("backward_gcn", &backward_gcn, "computation_aware_backward_gcn (HIP)");
    m.def("backward_gin", &backward_gin, "computation_aware_backward_gin (HIP)");
    m.def("backward_gat", &backward_gat, "computation_aware_backward_gat (HIP)");
    m.def("manual_seed", &manual_seed, "seed of sample_node's Philox streams (also restarts the per-call stream counter)");
    m.def("abi_version", []() { return fgl_abi_version(); });
}
