"""Size-independent properties at a full benchmark shape: the 2.4M-node / ~62M-edge R-MAT
graph, batch 8192, fanout [15,10,5] (the oracle is not run at this size)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_mid_shape_properties(cuda):
    import fastgl
    print("full-size: building 2.4M-node graph", flush=True)
    n = 2_400_000
    ptr, src = fastgl.graph.rmat_csr(n, 36_000_000, seed=0, device=cuda)
    n_edges = int(src.numel())
    print("edges:", n_edges, "max degree:", int((ptr[1:] - ptr[:-1]).max()), flush=True)
    assert 50_000_000 < n_edges < 75_000_000
    row_of_edge = torch.repeat_interleave(torch.arange(n, device=cuda), ptr[1:] - ptr[:-1])
    graph_keys = (row_of_edge << 32) | src.long()
    del row_of_edge

    fanouts = [15, 10, 5]
    sampler = fastgl.FusedMapSampler(fanouts, rng_seed=11).set_graph(ptr, src)
    seeds = torch.randperm(n, device=cuda)[:8192].int()
    input_nodes, out_nodes, blocks = sampler.sample_blocks(None, seeds)
    print("blocks:", blocks, flush=True)
    assert torch.equal(out_nodes, seeds)
    assert input_nodes.unique().numel() == input_nodes.numel()           # unique ids
    assert torch.equal(input_nodes[:8192], seeds)                        # seeds keep their positions
    deg_all = (ptr[1:] - ptr[:-1])
    cur_dst = seeds
    for block, fanout in zip(reversed(blocks), reversed(fanouts)):
        n_dst, n_src = block.num_dst_nodes(), block.num_src_nodes()
        assert n_dst == cur_dst.numel()
        src_l, dst_l = block.edges()
        uniq = input_nodes[:n_src]
        # exactly min(fanout, deg) edges per destination
        want_k = torch.clamp(deg_all[cur_dst.long()], max=fanout).int()
        assert torch.equal(block.in_degrees(), want_k)
        # every sampled edge exists in the graph
        g_src, g_dst = uniq[src_l.long()].long(), uniq[dst_l.long()].long()
        keys = (g_dst << 32) | g_src
        pos = torch.searchsorted(graph_keys, keys).clamp(max=n_edges - 1)
        assert torch.equal(graph_keys[pos], keys)
        # no neighbour twice for one destination
        pair = (dst_l.long() << 32) | src_l.long()
        assert pair.unique().numel() == pair.numel()
        # the id-map: every local id in range, all source nodes referenced or inherited
        assert int(src_l.max()) < n_src and int(src_l.min()) >= 0
        if block.src_global is not None:
            assert torch.equal(uniq[src_l.long()], block.src_global)
        new_ids = torch.unique(src_l[src_l >= n_dst])
        assert new_ids.numel() == n_src - n_dst                          # every new id is used by some edge
        cur_dst = uniq
    # aggregation at this shape: linearity and the all-ones closed form on the outermost block
    b0 = blocks[0]
    ones = torch.ones(b0.num_src_nodes(), 128, device=cuda)
    deg0 = b0.in_degrees().float()
    s = fastgl.aggregate(b0.edge_ptr, b0.src_local, ones, mode="sum", zero_policy="zeros")
    assert torch.equal(s, deg0[:, None].expand(-1, 128))
    x = torch.randn(b0.num_src_nodes(), 128, device=cuda)
    y = torch.randn(b0.num_src_nodes(), 128, device=cuda)
    lhs = fastgl.aggregate(b0.edge_ptr, b0.src_local, x + 2 * y, mode="mean", zero_policy="zeros")
    rhs = fastgl.aggregate(b0.edge_ptr, b0.src_local, x, mode="mean", zero_policy="zeros") + \
        2 * fastgl.aggregate(b0.edge_ptr, b0.src_local, y, mode="mean", zero_policy="zeros")
    assert torch.allclose(lhs, rhs, rtol=1e-4, atol=1e-4)
    # adjointness <A x, g> == <x, A^T g> ties the backward gather to the forward one
    t_ptr, t_idx = b0.transposed()
    g = torch.randn(b0.num_dst_nodes(), 128, device=cuda)
    ax = fastgl.aggregate(b0.edge_ptr, b0.src_local, x, mode="sum", zero_policy="zeros")
    atg = fastgl.aggregate(t_ptr, t_idx, g, mode="sum", zero_policy="zeros")
    a, b = (ax.double() * g.double()).sum().item(), (x.double() * atg.double()).sum().item()
    scale = (ax.double().abs() * g.double().abs()).sum().item()  # the inner products cancel heavily: compare on this scale
    assert abs(a - b) <= 1e-6 * scale


def test_whole_graph_as_one_block(cuda):
    """Aggregation over the whole 2.4M-node graph as one block: tens of thousands of rows beyond 128 entries
    (the longest holds ~85 K), so the long-row launch carries most of the work.  Closed forms (exact in fp32:
    sums of ones stay below 2^24), the same result whatever the caller says about the longest row, and
    linearity."""
    import fastgl
    print("full-size: whole graph as one block", flush=True)
    n = 2_400_000
    ptr, src = fastgl.graph.rmat_csr(n, 36_000_000, seed=0, device=cuda)
    ptr32 = ptr.int()
    deg = ptr32[1:] - ptr32[:-1]
    assert int((deg > 128).sum()) > 10_000 and int(deg.max()) > 50_000
    ones = torch.ones(n, 8, device=cuda)
    total = fastgl.aggregate(ptr32, src, ones, mode="sum", zero_policy="zeros")
    assert torch.equal(total, deg.float()[:, None].expand(-1, 8))
    mean = fastgl.aggregate(ptr32, src, ones, mode="mean", zero_policy="zeros")
    # n terms of fl(1/n), summed in fp32 per chunk and then across chunks: not exactly 1 for the longest rows
    mean_err = float((mean - (deg > 0).float()[:, None]).abs().max())
    print("mean of ones: max deviation %.2e" % mean_err, flush=True)
    assert mean_err <= 2e-5
    gen = torch.Generator(device=cuda).manual_seed(3)
    x = torch.randn(n, 32, device=cuda, generator=gen)
    y = torch.randn(n, 32, device=cuda, generator=gen)
    two = fastgl.aggregate(ptr32, src, x, mode="mean", zero_policy="zeros")                  # nothing known: two launches
    one = fastgl.aggregate(ptr32, src, x, mode="mean", zero_policy="zeros", longest_row=1)    # (wrong) bound: one launch
    scale = float(two.abs().max())
    assert float((two - one).abs().max()) <= 1e-5 * scale
    both = fastgl.aggregate(ptr32, src, 2.0 * x - y, mode="mean", zero_policy="zeros")
    ay = fastgl.aggregate(ptr32, src, y, mode="mean", zero_policy="zeros")
    assert float((both - (2.0 * two - ay)).abs().max()) <= 1e-5 * max(scale, float(ay.abs().max())) * 3


def test_offsets_beyond_int32(cuda):
    """A CSR with more than 2^31 edges (int64 row offsets): rows at the far end are sampled from the
    right place.  Closed form: indices[e] = e mod 2^20, so a full-neighbourhood row is a known range."""
    import fastgl
    print("full-size: >2^31-edge CSR", flush=True)
    n_nodes, deg = 1 << 22, 520                      # 2.18e9 edges
    n_edges = n_nodes * deg
    assert n_edges > (1 << 31)
    ptr = torch.arange(n_nodes + 1, dtype=torch.int64, device=cuda) * deg
    idx = torch.empty(n_edges, dtype=torch.int32, device=cuda)
    step = 1 << 28
    for lo in range(0, n_edges, step):
        hi = min(n_edges, lo + step)
        idx[lo:hi] = (torch.arange(lo, hi, dtype=torch.int64, device=cuda) & ((1 << 20) - 1)).int()
    seeds = torch.tensor([n_nodes - 1, n_nodes - 2, (1 << 22) - 4096, 5, 0], dtype=torch.int32, device=cuda)
    # fanout >= degree is impossible here (520 > 192), so check picks against the row's value range instead:
    # row v holds the consecutive values (v*deg + j) mod 2^20, j < deg; every pick must be one of them, without repeats
    src, dst, num = fastgl.sample_node(idx, idx, ptr, seeds, seeds.numel(), 192)
    assert int(num.item()) == 192 * seeds.numel()
    src = src.view(seeds.numel(), 192).long()
    assert torch.equal(dst.view(seeds.numel(), 192), seeds[:, None].expand(-1, 192))
    first = (seeds.long() * deg) & ((1 << 20) - 1)
    off = (src - first[:, None]) & ((1 << 20) - 1)
    assert int(off.max()) < deg and int(off.min()) >= 0
    assert all(off[i].unique().numel() == 192 for i in range(seeds.numel()))


# ---- the two largest benchmark shapes, checked against the oracle at full size ------------------------
def _rel_err(got, want):
    return np.abs(got.astype(np.float64) - want).max() / max(np.abs(want).max(), 1e-30)


def _resident_features(n, dim, dtype, cuda, seed):
    gen = torch.Generator(device=cuda).manual_seed(seed)
    feat = torch.empty((n, dim), dtype=dtype, device=cuda)
    for lo in range(0, n, 1 << 22):
        hi = min(n, lo + (1 << 22))
        feat[lo:hi] = torch.randn((hi - lo, dim), generator=gen, device=cuda, dtype=torch.float32).to(dtype)
    return feat


def _check_batch_against_oracle(cuda, oracle, ptr, src, h_ptr, h_src, feat, fanouts, rng_seed, tol, id_orders=("first", "arrival"),
                                steady_batches=None, graph_replay=False):
    """One mini-batch of 8192 seeds: unique list, every block's offsets and local ids bit-exact against the
    oracle (first-occurrence numbering; the arrival rule after sorting the new ids per hop), then the outermost
    block's mean aggregation from the resident table against the fp64 oracle on the rows it gathers."""
    import fastgl
    n = int(ptr.numel()) - 1
    seeds = torch.randperm(n, device=cuda, generator=torch.Generator(device=cuda).manual_seed(rng_seed))[:8192].int()
    h_seeds = seeds.cpu().numpy()
    w_inp, w_blocks = oracle.sample_blocks(h_ptr, h_src, h_seeds, fanouts, rng_seed, 0)
    print("oracle blocks:", [(b["n_src"], b["n_dst"], int(b["src_local"].size)) for b in w_blocks], flush=True)

    from test_gpu_idmap_blocks import check_transposed

    def same_as_oracle(got, want, want_seeds):
        g_inp, g_out, g_blocks = got
        w_inp_, w_blocks_ = want
        assert torch.equal(g_out, want_seeds)
        assert np.array_equal(g_inp.cpu().numpy(), w_inp_)
        for b, w in zip(g_blocks, w_blocks_):
            assert (b.num_src_nodes(), b.num_dst_nodes(), b.num_edges()) == (w["n_src"], w["n_dst"], int(w["src_local"].size))
            assert np.array_equal(b.edge_ptr.cpu().numpy(), w["indptr"])
            assert np.array_equal(b.src_local.cpu().numpy(), w["src_local"])
            if b._transposed is not None:  # the inner blocks come with their transposed form
                check_transposed(oracle, b, w)
        assert np.array_equal(g_blocks[0].src_global.cpu().numpy(), w_blocks_[0]["src_global"])
        assert [b._transposed is not None for b in g_blocks] == [False] + [True] * (len(g_blocks) - 1)

    sampler = fastgl.FusedMapSampler(fanouts, rng_seed=rng_seed).set_graph(ptr, src)
    input_nodes, out_nodes, blocks = sampler.sample_blocks(None, seeds)
    same_as_oracle((input_nodes, out_nodes, blocks), (w_inp, w_blocks), seeds)

    # The steady state, which is what a training loop and the benchmark run: the same sampler's next mini-batches use
    # buffers and a hash table sized from the batches before (a fraction of the worst case), skip the table fill
    # (the batch before left the table empty), and may be enqueued ahead of their read-back (begin_sample / finish)
    # or replayed from a captured graph.  Each form, on fresh seeds, bit for bit against the oracle.
    pool = torch.randperm(n, device=cuda, generator=torch.Generator(device=cuda).manual_seed(rng_seed + 100))
    n_extra = 3 if steady_batches is None else steady_batches
    first_state = sampler._state_for(seeds)
    assert first_state.nodes_seen is not None
    for i in range(1, 1 + n_extra):
        s_i = pool[i * 8192:(i + 1) * 8192].int()
        want = oracle.sample_blocks(h_ptr, h_src, s_i.cpu().numpy(), fanouts, rng_seed, 64 * i)
        if i == n_extra:  # the last of them through the two-phase form
            pend = sampler.begin_sample(s_i)
            got = pend.finish()
            assert not pend.redone
        else:
            got = sampler.sample_blocks(None, s_i)
        (plan,) = [v for k, v in first_state.plans.items() if k is not None]  # the plan sized by experience
        worst = first_state.plans[None]
        assert plan.cap_uniq < worst.cap_uniq and sum(plan.cap_edges) < sum(worst.cap_edges)
        assert plan.empty_slots is not None and plan.empty_slots < worst.slots  # a small table, left empty by the batch
        same_as_oracle(got, want, s_i)
        print("steady-state batch %d ok (%d edges)" % (i, sum(b.num_edges() for b in got[2])), flush=True)
    # ... and as the prefetching iterator runs them: two mini-batches in flight, each on a stream of its own with its
    # own table and scratch, the main stream busy with a consumer meanwhile
    first = sampler.batches
    seed_sets = [pool[(first + j) * 8192:(first + j + 1) * 8192].int() for j in range(4)]
    for j, got in enumerate(sampler.iter_batches(iter(seed_sets), prefetch=2)):
        want = oracle.sample_blocks(h_ptr, h_src, seed_sets[j].cpu().numpy(), fanouts, rng_seed, 64 * (first + j))
        same_as_oracle(got, want, seed_sets[j])
        fastgl.aggregate(got[2][0].edge_ptr, got[2][0].src_global, feat, mode="mean", zero_policy="zeros")
    print("prefetching iterator ok", flush=True)
    del got
    if graph_replay:
        gs = fastgl.FusedMapSampler(fanouts, rng_seed=rng_seed, graph_slots=2).set_graph(ptr, src)
        for i in range(4):  # batch 0 eager (worst-case plan); 1 and 2 capture the two slots; 3 replays slot 0
            s_i = pool[i * 8192:(i + 1) * 8192].int() if i else seeds
            want = oracle.sample_blocks(h_ptr, h_src, s_i.cpu().numpy(), fanouts, rng_seed, 64 * i)
            got = gs.sample_blocks(None, s_i)
            same_as_oracle(got, want, s_i)
        st = gs._state_for(seeds)
        assert st.graphs is not None and all(slot is not None for slot in st.graphs[2])
        print("graph replay ok", flush=True)
        del gs, got

    if "arrival" in id_orders:
        # the reference's numbering rule: any run is a valid map -- per hop the same set of new ids (the rows of
        # the next hop are then a permutation of the oracle's), and the same set of edges in graph ids (what a
        # node draws depends on its id, not on its position)
        alt = fastgl.FusedMapSampler(fanouts, rng_seed=rng_seed, id_order="arrival").set_graph(ptr, src)
        a_inp, _, a_blocks = alt.sample_blocks(None, seeds)
        a_inp_h = a_inp.cpu().numpy().astype(np.int64)
        assert a_inp_h.size == w_inp.size and np.array_equal(a_inp_h[:8192], h_seeds)
        for b, w in zip(a_blocks, w_blocks):
            nd, ns = w["n_dst"], w["n_src"]
            assert (b.num_src_nodes(), b.num_dst_nodes(), b.num_edges()) == (ns, nd, int(w["src_local"].size))
            assert np.array_equal(np.sort(a_inp_h[nd:ns]), np.sort(w_inp[nd:ns]))
            a_src, a_dst = (t.cpu().numpy() for t in b.edges())
            got_keys = np.sort((a_inp_h[a_dst] << 32) | a_inp_h[a_src])
            w_dst = np.repeat(np.arange(nd), np.diff(w["indptr"]))
            want_keys = np.sort((w_inp[w_dst].astype(np.int64) << 32) | w["src_global"].astype(np.int64))
            assert np.array_equal(got_keys, want_keys)
        del alt, a_blocks, a_inp

    # aggregation of the outermost block straight from the resident table: the first rows of the block (all of
    # them unless the block is huge) against the fp64 oracle on exactly the values the kernel reads
    b0, w0 = blocks[0], w_blocks[0]
    out = fastgl.aggregate(b0.edge_ptr, b0.src_global, feat, mode="mean", zero_policy="zeros")
    assert tuple(out.shape) == (w0["n_dst"], feat.size(1))
    m = min(w0["n_dst"], 1 << 18)
    e_m = int(w0["indptr"][m])
    ids, inv = np.unique(w0["src_global"][:e_m], return_inverse=True)
    x_sub = feat.index_select(0, torch.from_numpy(ids).to(cuda).long()).float().cpu().numpy()
    want = oracle.aggregate(w0["indptr"][:m + 1], inv.astype(np.int32), x_sub, "mean", 1)
    err = _rel_err(out[:m].float().cpu().numpy(), want)
    print("outermost mean aggregation: %d rows, %d entries, rel err %.2e" % (m, e_m, err), flush=True)
    assert err < tol
    # rows without neighbours give zeros (DGL's mean), the others are finite
    deg0 = np.diff(w0["indptr"])
    zero_rows = torch.from_numpy(np.flatnonzero(deg0 == 0)).to(cuda)
    assert float(out.index_select(0, zero_rows).float().abs().max()) == 0.0 if zero_rows.numel() else True
    assert bool(torch.isfinite(out.float()).all())
    # and the layer-wise (reference call pattern) path gives the same blocks as the fused one
    lw = fastgl.FusedMapSampler(fanouts, rng_seed=rng_seed, fused=False).set_graph(ptr, src)
    l_inp, _, l_blocks = lw.sample_blocks(None, seeds)
    assert torch.equal(l_inp, input_nodes)
    for a, b in zip(l_blocks, blocks):
        assert torch.equal(a.edge_ptr, b.edge_ptr) and torch.equal(a.src_local, b.src_local)


def test_large_resident_shape_vs_oracle(cuda, oracle):
    """111 M nodes / ~1.7 B edges (int64 offsets), features 111 M x 128 fp32 resident, batch 8192, fanout
    [15,10,5]: the configuration the headline figures are quoted on."""
    import fastgl
    print("full-size: 111M-node graph", flush=True)
    torch.cuda.empty_cache()
    n = 111_000_000
    ptr, src = fastgl.graph.rmat_csr(n, 900_000_000, seed=0, device=cuda)
    assert ptr.dtype == torch.int64 and 1_500_000_000 < int(src.numel()) < 1_900_000_000
    torch.cuda.empty_cache()
    h_ptr, h_src = ptr.cpu().numpy(), src.cpu().numpy()
    print("graph on the host: %d edges" % h_src.size, flush=True)
    feat = _resident_features(n, 128, torch.float32, cuda, seed=1)
    _check_batch_against_oracle(cuda, oracle, ptr, src, h_ptr, h_src, feat, [15, 10, 5], rng_seed=5, tol=1e-5, graph_replay=True)
    del feat, ptr, src
    torch.cuda.empty_cache()


def test_very_large_shape_vs_oracle(cuda, oracle):
    """269 M nodes / ~4.0 B edges (row offsets beyond 2^31), features 269 M x 128 bf16 resident, batch 8192,
    fanouts [15,10,5] and [10,10,10,10,10]."""
    import fastgl
    print("full-size: 269M-node graph", flush=True)
    torch.cuda.empty_cache()
    n = 269_000_000
    ptr, src = fastgl.graph.rmat_csr(n, 3_320_000_000, seed=0, device=cuda)
    assert ptr.dtype == torch.int64 and int(src.numel()) > (1 << 31) and int(ptr[-1]) == int(src.numel())
    torch.cuda.empty_cache()
    h_ptr, h_src = ptr.cpu().numpy(), src.cpu().numpy()
    print("graph on the host: %d edges" % h_src.size, flush=True)
    feat = _resident_features(n, 128, torch.bfloat16, cuda, seed=2)
    _check_batch_against_oracle(cuda, oracle, ptr, src, h_ptr, h_src, feat, [15, 10, 5], rng_seed=6, tol=1e-2)
    print("full-size: deep fanout", flush=True)
    _check_batch_against_oracle(cuda, oracle, ptr, src, h_ptr, h_src, feat, [10, 10, 10, 10, 10], rng_seed=7, tol=1e-2, steady_batches=2)
    del feat, ptr, src
    torch.cuda.empty_cache()
