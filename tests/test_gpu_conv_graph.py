"""Layer-level parity (forward and autograd backward) against dense fp64 torch on the CPU,
the drop-in operator signatures, and the device R-MAT generator against the oracle."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def dev_i32(a, cuda):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(cuda)


def small_blocks(cuda, oracle, small_graph, fanouts=(4, 3), batch=200):
    import fastgl
    indptr, indices = small_graph
    sampler = fastgl.FusedMapSampler(list(fanouts), rng_seed=3).set_graph(torch.from_numpy(indptr).to(cuda), dev_i32(indices, cuda))
    seeds = np.random.default_rng(0).permutation(indptr.size - 1)[:batch].astype(np.int32)
    return sampler.sample_blocks(None, dev_i32(seeds, cuda))


def dense_adj(block, kind):
    """fp64 dense operator of a block as the reference kernels define it"""
    n_dst, n_src = block.num_dst_nodes(), block.num_src_nodes()
    src, dst = (t.cpu().long() for t in block.edges())
    A = torch.zeros(n_dst, n_src, dtype=torch.float64)
    A.index_put_((dst, src), torch.ones(src.numel(), dtype=torch.float64), accumulate=True)
    deg = A.sum(1)
    if kind == "gcn":
        dn = deg.clamp(min=1)
        sn = torch.bincount(src, minlength=n_src).double().clamp(min=1)
        A = dn.rsqrt()[:, None] * A * sn.rsqrt()[None, :]
    if kind == "mean":
        A = A / deg.clamp(min=1)[:, None]
    passthrough = (deg == 0)
    return A, passthrough


@pytest.mark.parametrize("input_grad", [True, False])
@pytest.mark.parametrize("model_name", ["gcn", "gcn:product_first", "gcn:gather_first", "gin"])
def test_gcn_gin_forward_backward(cuda, oracle, small_graph, model_name, input_grad):
    """input_grad=False is the training case (raw features): the first layer then computes only the weight
    gradient, without ever building the outermost block's transpose.  GCN in both orders of product and
    gather (the reference's, and gather first) and with the layer's own choice."""
    import fastgl
    print("conv %s input_grad=%s" % (model_name, input_grad), flush=True)
    input_nodes, _, blocks = small_blocks(cuda, oracle, small_graph)
    torch.manual_seed(0)
    model_name, _, order = model_name.partition(":")
    cls = fastgl.GCN if model_name == "gcn" else fastgl.GIN
    model = cls(20, 16, 5, 2, None, True, 0.0).to(cuda)
    for layer in model.layers:
        if order:
            layer.order = order
    x = torch.randn(input_nodes.numel(), 20, device=cuda, requires_grad=input_grad)
    out = model(blocks, x, neighbor_list=[4, 3])
    gout = torch.randn_like(out)
    out.backward(gout)

    h = x.detach().cpu().double().requires_grad_(True)
    ws = [l.weights.detach().cpu().double().requires_grad_(True) for l in model.layers]
    cur = h
    for block, w in zip(blocks, ws):
        A, passthrough = dense_adj(block, "gcn" if model_name == "gcn" else "sum")
        n_dst = block.num_dst_nodes()
        if model_name == "gcn":
            t = cur @ w
            # rows without edges pass (X W)[d] through, and no gradient flows back through that copy
            cur = A @ t + passthrough[:, None] * t[:n_dst].detach()
        else:
            cur = (A @ cur + passthrough[:, None] * cur[:n_dst].detach()) @ w
    cur.backward(gout.cpu().double())
    assert torch.allclose(out.detach().cpu().double(), cur.detach(), rtol=1e-4, atol=1e-5)
    if input_grad:
        assert torch.allclose(x.grad.cpu().double(), h.grad, rtol=1e-4, atol=1e-5)
    else:
        assert x.grad is None and blocks[0]._transposed is None and blocks[1]._transposed is not None
    for l, w in zip(model.layers, ws):
        assert torch.allclose(l.weights.grad.cpu().double(), w.grad, rtol=1e-4, atol=1e-5)


def test_sage_mean_with_fused_input_gather(cuda, oracle, small_graph):
    import fastgl
    print("conv sage", flush=True)
    indptr, _ = small_graph
    input_nodes, _, blocks = small_blocks(cuda, oracle, small_graph)
    torch.manual_seed(1)
    feat = torch.randn(indptr.size - 1, 24, device=cuda)
    model = fastgl.SAGE(24, 16, 5, 2, dropout=0.0).to(cuda)
    out_fused = model(blocks, feat, input_nodes=input_nodes)          # first layer reads the full table
    x = feat.index_select(0, input_nodes.long()).requires_grad_(True)  # the explicit gather the reference does
    out = model(blocks, x)
    assert torch.allclose(out, out_fused, rtol=1e-5, atol=1e-6)
    gout = torch.randn_like(out)
    out.backward(gout)

    h = x.detach().cpu().double().requires_grad_(True)
    cur = h
    params = []
    for i, (layer, block) in enumerate(zip(model.layers, blocks)):
        A, _ = dense_adj(block, "mean")
        ws = layer.fc_self.weight.detach().cpu().double().requires_grad_(True)
        wn = layer.fc_neigh.weight.detach().cpu().double().requires_grad_(True)
        b = layer.fc_neigh.bias.detach().cpu().double().requires_grad_(True)
        params.append((layer, ws, wn, b))
        cur = cur[:block.num_dst_nodes()] @ ws.T + (A @ cur) @ wn.T + b
        if i == 0:
            cur = torch.relu(cur)
    cur.backward(gout.cpu().double())
    assert torch.allclose(out.detach().cpu().double(), cur.detach(), rtol=1e-4, atol=1e-5)
    assert torch.allclose(x.grad.cpu().double(), h.grad, rtol=1e-4, atol=1e-5)
    for layer, ws, wn, b in params:
        assert torch.allclose(layer.fc_self.weight.grad.cpu().double(), ws.grad, rtol=1e-4, atol=1e-5)
        assert torch.allclose(layer.fc_neigh.weight.grad.cpu().double(), wn.grad, rtol=1e-4, atol=1e-5)


def test_drop_in_operator_flow(cuda, oracle, small_graph):
    """The reference's own call sequence (GraphConv.py:91-98 on COO edges): cal_deg -> exclusive_sum ->
    forward_gcn / backward_gcn and forwaed_gin / backward_gin, checked against the oracle."""
    import fastgl
    print("drop-in operator flow", flush=True)
    _, _, blocks = small_blocks(cuda, oracle, small_graph)
    block = blocks[0]
    src, dst = block.edges()
    n_dst, n_src = block.num_dst_nodes(), block.num_src_nodes()
    raw = fastgl.cal_deg(dst, n_dst)
    edge_ptr = fastgl.exclusive_sum(raw)
    assert torch.equal(edge_ptr, block.edge_ptr)
    src_norm = fastgl.cal_deg(src, n_src).clamp(min=1)
    dst_norm = raw.clamp(min=1)
    rng = np.random.default_rng(4)
    X = torch.from_numpy(rng.standard_normal((n_src, 12)).astype(np.float32)).to(cuda)
    W = torch.from_numpy(rng.standard_normal((12, 8)).astype(np.float32)).to(cuda)
    ptr_h, src_h = edge_ptr.cpu().numpy(), src.cpu().numpy()
    sn_h, dn_h = src_norm.cpu().numpy(), dst_norm.cpu().numpy()
    # The operators multiply with the library GEMM (as the reference does with torch::mm); the products are
    # formed here with the same call on both sides, so that what is compared is the aggregation, at the
    # acceptance tolerance: 1e-5 relative to the largest magnitude of the fp64 result.
    def close(got, want, what):
        want = np.asarray(want, dtype=np.float64)
        err = np.abs(got.double().cpu().numpy() - want).max() / max(np.abs(want).max(), 1e-30)
        assert err <= 1e-5, (what, err)

    def on_gpu(a):
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(cuda)

    T = torch.mm(X, W)
    (out,) = fastgl.forward_gcn(edge_ptr, src, src_norm, dst_norm, X, W, 4, n_dst)
    close(out, oracle.aggregate(ptr_h, src_h, T.cpu().numpy(), "gcn", 0, dn_h, sn_h), "forward_gcn")

    d_out = torch.from_numpy(rng.standard_normal((n_dst, 8)).astype(np.float32)).to(cuda)
    d_x, d_w = fastgl.backward_gcn(edge_ptr, src, dst_norm, src_norm, d_out, W, X)  # (dst, src) order: GraphConv.py:37
    t_ptr, t_idx = oracle.transpose(ptr_h, src_h, n_src)
    G = oracle.aggregate(t_ptr, t_idx, d_out.cpu().numpy(), "gcn", 1, sn_h, dn_h)
    close(d_x, torch.mm(on_gpu(G), W.t()).cpu().numpy(), "backward_gcn d_x")
    close(d_w, torch.mm(X.t(), on_gpu(G)).cpu().numpy(), "backward_gcn d_w")
    close(d_x, G @ W.cpu().numpy().T.astype(np.float64), "backward_gcn d_x vs fp64")

    out, tmp = fastgl.forwaed_gin(edge_ptr, src, X, W, 4, n_dst)
    want_tmp = oracle.aggregate(ptr_h, src_h, X.cpu().numpy(), "sum", 0)
    close(tmp, want_tmp, "forwaed_gin tmp")
    close(out, torch.mm(on_gpu(want_tmp), W).cpu().numpy(), "forwaed_gin out")
    d_x, d_w = fastgl.backward_gin(edge_ptr, src, d_out, W, tmp, n_src)
    d_tmp = torch.mm(d_out, W.t())
    close(d_x, oracle.aggregate(t_ptr, t_idx, d_tmp.cpu().numpy(), "sum", 1), "backward_gin d_x")
    close(d_w, torch.mm(on_gpu(want_tmp).t(), d_out).cpu().numpy(), "backward_gin d_w")


def test_rmat_keys_match_oracle(cuda, oracle):
    import fastgl
    print("rmat keys", flush=True)
    for n_nodes, n, first, seed in ((1000, 5000, 0, 0), (100_000, 200_000, 12345, 7), (3, 100, 0, 1)):
        scale = fastgl.graph.rmat_scale(n_nodes)
        got = fastgl.rmat_keys(first, n, scale, n_nodes, seed, cuda).cpu().numpy()
        assert np.array_equal(got, oracle.rmat_keys(first, n, scale, n_nodes, seed))


def test_rmat_csr_matches_oracle(cuda, oracle, small_graph):
    import fastgl
    print("rmat csr", flush=True)
    indptr, indices = small_graph
    ptr, src = fastgl.graph.rmat_csr(100_000, 1_500_000, seed=0, device=cuda, chunk_draws=400_000)
    assert np.array_equal(ptr.cpu().numpy(), indptr) and np.array_equal(src.cpu().numpy(), indices)


def test_merge_of_sorted_parts_by_key_range(cuda):
    """the large-graph path of the CSR builder (union assembled per key range) equals a plain unique"""
    import fastgl
    print("graph merge by range", flush=True)
    g = torch.Generator(device=cuda).manual_seed(0)
    parts = [torch.unique(torch.randint(0, 1 << 40, (n,), generator=g, device=cuda)) for n in (50_000, 1, 120_000, 70_000)]
    want = torch.unique(torch.cat(parts))
    got = fastgl.graph._merge_sorted_unique(parts, cuda, max_items=40_000)
    assert torch.equal(got, want)


def test_gat_forward_backward(cuda, oracle, small_graph):
    """GAT model against dense fp64 torch; as in the reference the attention weights are constants
    for the backward pass (MA_Function_GAT returns no gradient for them, GraphConv.py:227)."""
    import fastgl
    print("conv gat", flush=True)
    input_nodes, _, blocks = small_blocks(cuda, oracle, small_graph)
    torch.manual_seed(2)
    model = fastgl.GAT(20, 8, 5, 2, None, 0.0, heads=4).to(cuda)
    x = torch.randn(input_nodes.numel(), 20, device=cuda, requires_grad=True)
    out = model(blocks, x, neighbor_list=[4, 3])
    assert tuple(out.shape) == (blocks[-1].num_dst_nodes(), 5)
    gout = torch.randn_like(out)
    out.backward(gout)

    h = x.detach().cpu().double().requires_grad_(True)
    cur = h
    weights = []
    for layer, block in zip(model.layers, blocks):
        H, F = layer.num_heads, layer.out_feats
        W = layer.fc.weight.detach().cpu().double().requires_grad_(True)
        weights.append((layer, W))
        al, ar = layer.attn_l.detach().cpu().double(), layer.attn_r.detach().cpu().double()
        n_dst, n_src = block.num_dst_nodes(), block.num_src_nodes()
        src, dst = (t.cpu().long() for t in block.edges())
        z = (cur @ W.T).view(n_src, H, F)
        el, er = (z * al).sum(-1), (z[:n_dst] * ar).sum(-1)
        e = torch.nn.functional.leaky_relu(el[src] + er[dst], 0.2).detach()   # constants in the backward pass
        alpha = torch.zeros_like(e)
        for d in range(n_dst):
            m = dst == d
            if m.any():
                alpha[m] = torch.softmax(e[m], 0)
        msg = alpha[:, :, None] * z[src]                                        # [E, H, F]
        agg = torch.zeros(n_dst, H, F, dtype=torch.float64).index_add_(0, dst, msg)
        deg = torch.bincount(dst, minlength=n_dst)
        agg = torch.where((deg == 0)[:, None, None], z[:n_dst].detach(), agg)   # pass-through, no gradient
        cur = agg.reshape(n_dst, H * F)
    cur.backward(gout.cpu().double())
    assert torch.allclose(out.detach().cpu().double(), cur.detach(), rtol=1e-4, atol=1e-5)
    assert torch.allclose(x.grad.cpu().double(), h.grad, rtol=1e-4, atol=1e-5)
    for layer, W in weights:
        assert torch.allclose(layer.fc.weight.grad.cpu().double(), W.grad, rtol=1e-4, atol=1e-5)


def test_sage_bf16_features(cuda, oracle, small_graph):
    """bf16 feature table and activations (fp32 accumulation inside the kernels): forward and the
    gradient of the inner layer stay within the bf16 tolerance of an fp32 run"""
    import fastgl
    print("conv sage bf16", flush=True)
    indptr, _ = small_graph
    input_nodes, _, blocks = small_blocks(cuda, oracle, small_graph)
    torch.manual_seed(3)
    feat = torch.randn(indptr.size - 1, 32, device=cuda)
    model = fastgl.SAGE(32, 16, 4, 2, dropout=0.0).to(cuda)
    ref = model(blocks, feat, input_nodes=input_nodes)
    ref.sum().backward()
    g_ref = [p.grad.clone() for p in model.parameters()]
    model.zero_grad()
    model_bf = model.to(torch.bfloat16)
    out = model_bf(blocks, feat.to(torch.bfloat16), input_nodes=input_nodes)
    assert out.dtype == torch.bfloat16
    assert (out.float() - ref).norm() <= 0.02 * ref.norm()
    out.float().sum().backward()
    for p, g in zip(model_bf.parameters(), g_ref):  # norm-wise and loose: the weights themselves are rounded to bf16 and ReLUs flip
        assert (p.grad.float() - g).norm() <= 0.15 * g.norm() + 1e-3
