"""The compiled torch extension module `fastgl` (fastgl-ae_amd/csrc/fastgl_module.cpp, built by
`make -C fastgl-ae_amd/csrc module`): the reference's own call sequences -- the sampler's layer loop
(FusedMapSampler.py:72-107) and a GCN / GIN layer's operator calls (GraphConv.py:91-98, 26, 37, 109, 132) --
driven through it, checked against the oracle.  The module is loaded from its file under a private name: in this
test process the name `fastgl` belongs to the Python package."""
import glob
import importlib.util
import os

import numpy as np
import pytest
import torch

from conftest import ROOT

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ext():
    paths = glob.glob(os.path.join(ROOT, "fastgl-ae_amd", "fastgl_ext", "fastgl*.so"))
    if not paths:
        pytest.fail("the compiled module is not built: make -C fastgl-ae_amd/csrc module")
    spec = importlib.util.spec_from_file_location("fastgl", paths[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def rel_err(got, want):
    want = np.asarray(want, dtype=np.float64)
    return np.abs(got.double().cpu().numpy() - want).max() / max(np.abs(want).max(), 1e-30)


def reference_layer_loop(ext, edge_src, edge_dst, edge_ptr, nodes_num, seed_nodes, fanouts):
    """FusedMapSampler.sample_blocks of the reference, statement for statement, with a (src, dst, n_src, n_dst)
    tuple where it builds a DGL block."""
    raw_seed_nodes = seed_nodes.int().clone()
    seed_nodes_acc = seed_nodes.clone()
    blocks = []
    dst_nodes = seed_nodes.size(0)
    for block_index, fanout in enumerate(reversed(fanouts)):
        src_edges_out, dst_edges_out, edge_num = ext.sample_node(edge_src, edge_dst, edge_ptr, seed_nodes_acc.int(), dst_nodes, fanout)
        edge_nums = src_edges_out.size(0)
        assert int(edge_num.item()) == edge_nums
        if block_index == 0:
            dst_edges_unique = raw_seed_nodes
        else:
            dst_edges_unique = seed_nodes_acc
        if block_index == 0:
            output_nodes = raw_seed_nodes
        max_src_num = nodes_num if (fanout * dst_edges_unique.size(0) > nodes_num) else (fanout * dst_edges_unique.size(0))
        src_global = src_edges_out.clone()
        src_edges, dst_edges, seed_nodes_acc = ext.transfer_edge_id(src_edges_out, dst_edges_out, dst_edges_unique,
                                                                    dst_nodes, dst_nodes + edge_nums, max_src_num, edge_nums)
        assert src_edges.data_ptr() == src_edges_out.data_ptr() and dst_edges.data_ptr() == dst_edges_out.data_ptr()  # in place
        blocks.insert(0, (src_edges, dst_edges, seed_nodes_acc.size(0), dst_edges_unique.size(0), src_global))
        dst_nodes = seed_nodes_acc.size(0)
    return seed_nodes_acc, output_nodes, blocks


def test_sampler_loop_and_layers_through_the_compiled_module(cuda, oracle, small_graph, ext):
    print("compiled module: sampler loop + layer operators", flush=True)
    import fastgl
    assert ext.abi_version() == fastgl.lib().fgl_abi_version()
    indptr, indices = small_graph
    n = indptr.size - 1
    # the trainer's CSR: int32 offsets (train_fastgl.py:228-230) -- and int64, which this build also takes
    for ptr_dtype in (np.int32, np.int64):
        edge_ptr = torch.from_numpy(indptr.astype(ptr_dtype)).to(cuda)
        edge_src = torch.from_numpy(indices).to(cuda)
        edge_dst = torch.repeat_interleave(torch.arange(n, device=cuda, dtype=torch.int32), torch.from_numpy(np.diff(indptr)).to(cuda))
        seeds_h = np.random.default_rng(3).permutation(n)[:1024].astype(np.int32)
        seeds = torch.from_numpy(seeds_h).to(cuda)
        fanouts = [15, 10, 5]
        ext.manual_seed(21)
        input_nodes, output_nodes, blocks = reference_layer_loop(ext, edge_src, edge_dst, edge_ptr, n, seeds, fanouts)
        # the oracle's loop draws hop h from stream h, as the module's per-call counter does after manual_seed
        w_inp, w_blocks = oracle.sample_blocks(indptr.astype(ptr_dtype), indices, seeds_h, fanouts, 21, 0)
        assert torch.equal(output_nodes, seeds)
        assert np.array_equal(input_nodes.cpu().numpy(), w_inp)
        for (src, dst, n_src, n_dst, src_g), w in zip(blocks, w_blocks):
            assert (n_src, n_dst) == (w["n_src"], w["n_dst"])
            assert np.array_equal(src.cpu().numpy(), w["src_local"])
            assert np.array_equal(src_g.cpu().numpy(), w["src_global"])
            assert np.array_equal(dst.cpu().numpy(), np.repeat(np.arange(n_dst), np.diff(w["indptr"])))

    # one GCN layer and one GIN layer on the outermost block, as GraphConv.py drives them
    src, dst, n_src, n_dst, _ = blocks[0]
    w0 = w_blocks[0]
    raw_dst_norm_degs = ext.cal_deg(dst.int(), n_dst)
    edge_ptr_b = ext.exclusive_sum(raw_dst_norm_degs)
    assert np.array_equal(edge_ptr_b.cpu().numpy(), w0["indptr"])
    src_norm_degs = ext.cal_deg(src.int(), n_src).clamp(min=1)
    dst_norm_degs = raw_dst_norm_degs.clamp(min=1)
    sn_h, dn_h = src_norm_degs.cpu().numpy(), dst_norm_degs.cpu().numpy()
    rng = np.random.default_rng(8)
    X = torch.from_numpy(rng.standard_normal((n_src, 32)).astype(np.float32)).to(cuda)
    W = torch.from_numpy(rng.standard_normal((32, 16)).astype(np.float32)).to(cuda)
    d_out = torch.from_numpy(rng.standard_normal((n_dst, 16)).astype(np.float32)).to(cuda)
    on_gpu = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(cuda)
    ptr_h, src_h = w0["indptr"], w0["src_local"]
    t_ptr, t_idx = oracle.transpose(ptr_h, src_h, n_src)
    # (products formed with the same library call on both sides: what is compared is the aggregation, at 1e-5)
    (out,) = ext.forward_gcn(edge_ptr_b, src.int(), src_norm_degs, dst_norm_degs, X, W, fanouts[0], n_dst)
    assert rel_err(out, oracle.aggregate(ptr_h, src_h, torch.mm(X, W).cpu().numpy(), "gcn", 0, dn_h, sn_h)) <= 1e-5
    d_x, d_w = ext.backward_gcn(edge_ptr_b, src.int(), dst_norm_degs, src_norm_degs, d_out, W, X)  # (dst, src): GraphConv.py:37
    G = oracle.aggregate(t_ptr, t_idx, d_out.cpu().numpy(), "gcn", 1, sn_h, dn_h)
    assert rel_err(d_x, torch.mm(on_gpu(G), W.t()).cpu().numpy()) <= 1e-5
    assert rel_err(d_w, torch.mm(X.t(), on_gpu(G)).cpu().numpy()) <= 1e-5
    out, tmp = ext.forwaed_gin(edge_ptr_b, src.int(), X, W, fanouts[0], n_dst)
    want_tmp = oracle.aggregate(ptr_h, src_h, X.cpu().numpy(), "sum", 0)
    assert rel_err(tmp, want_tmp) <= 1e-5
    assert rel_err(out, torch.mm(on_gpu(want_tmp), W).cpu().numpy()) <= 1e-5
    d_x, d_w = ext.backward_gin(edge_ptr_b, src.int(), d_out, W, tmp, n_src)
    assert rel_err(d_x, oracle.aggregate(t_ptr, t_idx, torch.mm(d_out, W.t()).cpu().numpy(), "sum", 1)) <= 1e-5
    assert rel_err(d_w, torch.mm(on_gpu(want_tmp).t(), d_out).cpu().numpy()) <= 1e-5
    # GAT aggregation with per-edge, per-head weights
    H = 4
    alpha = torch.from_numpy(rng.random((src.numel(), H, 1)).astype(np.float32)).to(cuda)
    (xg,) = ext.forward_gat(edge_ptr_b, alpha, src.int(), X, fanouts[0], n_dst, H)
    assert rel_err(xg, oracle.aggregate_edge(ptr_h, src_h, X.cpu().numpy(), alpha.view(-1, H).cpu().numpy(), zero_policy=0)) <= 1e-5
    (dxg,) = ext.backward_gat(edge_ptr_b, alpha, src.int(), d_out, n_src, H)
    tp, ti, te = oracle.transpose_with_edges(ptr_h, src_h, n_src)
    assert rel_err(dxg, oracle.aggregate_edge(tp, ti, d_out.cpu().numpy(), alpha.view(-1, H).cpu().numpy(), 1, edge_index=te)) <= 1e-5


def test_compiled_module_errors_are_runtime_errors(cuda, ext):
    cpu = torch.zeros(4, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ext.cal_deg(cpu, 4)
    d = torch.zeros(8, dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError, match="contiguous"):
        ext.cal_deg(d[::2], 4)
    with pytest.raises(RuntimeError, match="int32"):
        ext.exclusive_sum(d.long())
    ptr = torch.tensor([0, 2, 4], dtype=torch.int32, device=cuda)
    idx = torch.tensor([1, 0, 0, 1], dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError, match="outside the graph"):
        ext.sample_node(idx, idx, ptr, torch.tensor([0, 5], dtype=torch.int32, device=cuda), 2, 2)
    with pytest.raises(RuntimeError, match="negative id"):
        ext.transfer_edge_id(torch.tensor([1, -1], dtype=torch.int32, device=cuda), torch.tensor([0, 0], dtype=torch.int32, device=cuda),
                             torch.tensor([0], dtype=torch.int32, device=cuda), 1, 3, 2, 2)
