"""HIP fused id-map and the all-hops sampler against the oracle, through the C ABI."""
import os

import numpy as np
import pytest
import torch

from conftest import GOLDEN_DIR

pytestmark = pytest.mark.gpu


def dev_i32(a, cuda):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(cuda)


def canonical(src_local, uniq, n_dst, block_ptr=None):
    """Order-free form of an id-map result: new ids renumbered by ascending graph id, each
    destination row's edge list sorted."""
    tail = uniq[n_dst:]
    order = np.argsort(tail, kind="stable")
    remap = np.concatenate([np.arange(n_dst), n_dst + np.argsort(order, kind="stable")])
    s = remap[src_local]
    if block_ptr is not None:
        s = np.concatenate([np.sort(s[block_ptr[i]:block_ptr[i + 1]]) for i in range(len(block_ptr) - 1)] or [s[:0]])
    return s, np.concatenate([uniq[:n_dst], tail[order]])


def run_transfer(cuda, src, dst, dst_unique, n_nodes):
    import fastgl
    s, d = dev_i32(src, cuda), dev_i32(dst, cuda)
    n_dst, e = len(dst_unique), len(src)
    out = fastgl.transfer_edge_id(s, d, dev_i32(dst_unique, cuda), n_dst, n_dst + e, min(n_nodes, max(e, 1)), e)
    assert out[0].data_ptr() == s.data_ptr() and out[1].data_ptr() == d.data_ptr()  # in place, like the reference
    return out[0].cpu().numpy(), out[1].cpu().numpy(), out[2].cpu().numpy()


def test_hand_fixture(cuda):
    print("idmap hand fixture", flush=True)
    g = np.load(os.path.join(GOLDEN_DIR, "idmap_hand.npz"))
    s, d, u = run_transfer(cuda, g["src"], g["dst"], g["dst_unique"], 10)
    assert np.array_equal(s, g["src_local"]) and np.array_equal(d, g["dst_local"]) and np.array_equal(u, g["uniq"])


@pytest.mark.parametrize("n_ids,n_dst,n_edges", [(50, 10, 4000), (100_000, 1000, 15_000), (2**31 - 1, 64, 50_000),
                                                 (3_000_000, 8192, 1_000_000), (7, 7, 0), (1000, 1, 2049),
                                                 # 2048 tiles of 2048 edges: up to there the numbering pass scans the
                                                 # tile counts itself, beyond a scan launch does
                                                 (5_000_000, 4096, 2_097_153), (5_000_000, 4096, 4_194_304), (5_000_000, 4096, 4_194_305),
                                                 (40_000_000, 100, 2_500_000)])
def test_transfer_edge_id_vs_oracle(cuda, oracle, n_ids, n_dst, n_edges):
    print("idmap %d %d %d" % (n_ids, n_dst, n_edges), flush=True)
    rng = np.random.default_rng(n_edges + n_dst)
    dst_unique = rng.choice(min(n_ids, 10**7), size=n_dst, replace=False).astype(np.int32)
    # power-law-ish sources so that hot ids collide heavily
    src = (rng.pareto(1.2, size=n_edges) * 50).astype(np.int64) % n_ids
    src[::7] = rng.integers(0, n_ids, size=src[::7].size)
    src = src.astype(np.int32)
    dst = np.sort(rng.integers(0, n_dst, size=n_edges))
    dst_g = dst_unique[dst] if n_edges else np.zeros(0, np.int32)
    s, d, u = run_transfer(cuda, src, dst_g, dst_unique, n_ids)
    ws, wd, wu = oracle.idmap(src, dst_g, dst_unique)
    # bit-exact, order included (first-occurrence numbering) ...
    assert np.array_equal(u, wu) and np.array_equal(s, ws) and np.array_equal(d, wd)
    # ... and after the canonical sort that the acceptance criterion names
    bptr = np.concatenate([[0], np.cumsum(np.bincount(dst, minlength=n_dst))])
    cs, cu = canonical(s, u, n_dst, bptr)
    cws, cwu = canonical(ws, wu, n_dst, bptr)
    assert np.array_equal(cs, cws) and np.array_equal(cu, cwu)


def test_transfer_edge_id_reports_missing_dst(cuda):
    print("idmap missing key", flush=True)
    with pytest.raises(RuntimeError, match="not in the map"):
        run_transfer(cuda, np.array([1, 2], np.int32), np.array([5, 77], np.int32), np.array([5], np.int32), 100)


def load_graph(cuda, indptr, indices):
    return torch.from_numpy(indptr).to(cuda), dev_i32(indices, cuda)


def check_blocks(oracle, indptr, indices, seeds, fanouts, got, rng_seed, stream_base):
    inp, out_nodes, blocks = got
    w_inp, w_blocks = oracle.sample_blocks(indptr, indices, seeds, fanouts, rng_seed, stream_base)
    assert np.array_equal(inp.cpu().numpy(), w_inp)
    assert np.array_equal(out_nodes.cpu().numpy(), seeds)
    assert len(blocks) == len(w_blocks)
    for b, w in zip(blocks, w_blocks):
        assert (b.num_src_nodes(), b.num_dst_nodes()) == (w["n_src"], w["n_dst"])
        assert np.array_equal(b.edge_ptr.cpu().numpy(), w["indptr"])
        assert np.array_equal(b.src_local.cpu().numpy(), w["src_local"])
        if b.src_global is not None:
            assert np.array_equal(b.src_global.cpu().numpy(), w["src_global"])
        src, dst = b.edges()
        assert np.array_equal(dst.cpu().numpy(), np.repeat(np.arange(w["n_dst"]), np.diff(w["indptr"])))
        if b._transposed is not None:
            check_transposed(oracle, b, w)


def check_transposed(oracle, b, w):
    """The transposed block that came with a sampled block: offsets equal to the oracle's transpose, the same set of
    destination rows per source node (their order within a row is left to scheduling), every entry pointing back at
    the edge it came from, and the longest row as it was read back with the sizes."""
    t_ptr, t_dst, t_edge = (t.cpu().numpy() for t in b.transposed(edge_ids=True))
    n_src, n_dst = w["n_src"], w["n_dst"]
    w_ptr, w_idx = oracle.transpose(w["indptr"], w["src_local"], n_src)
    assert t_ptr.size == n_src + 1 and np.array_equal(t_ptr, w_ptr)
    assert t_dst.size == w_idx.size == t_edge.size
    row_of = np.repeat(np.arange(n_src, dtype=np.int64), np.diff(w_ptr))
    assert np.array_equal(np.sort(row_of * (n_dst + 1) + t_dst), np.sort(row_of * (n_dst + 1) + w_idx))
    assert np.array_equal(np.sort(t_edge), np.arange(w["src_local"].size))
    assert np.array_equal(w["src_local"][t_edge], row_of)
    assert np.array_equal(np.repeat(np.arange(n_dst), np.diff(w["indptr"]))[t_edge], t_dst)
    longest = int(np.diff(w_ptr).max()) if n_src else 0
    reported = b.transposed()[0].fgl_longest_row
    assert isinstance(reported, int) and reported == max(longest, 32)
    assert np.array_equal(b.out_degrees().cpu().numpy(), np.diff(w_ptr))


@pytest.mark.parametrize("fused", [True, False])
def test_sample_blocks_golden(cuda, oracle, fused):
    import fastgl
    print("sample_blocks golden fused=%s" % fused, flush=True)
    g = np.load(os.path.join(GOLDEN_DIR, "sample_blocks_small.npz"))
    ptr, idx = load_graph(cuda, g["indptr"], g["indices"])
    s = fastgl.FusedMapSampler(g["fanouts"].tolist(), fused=fused, rng_seed=int(g["rng_seed"])).set_graph(ptr, idx)
    inp, out_nodes, blocks = s.sample_blocks(None, dev_i32(g["seeds"], cuda))
    assert np.array_equal(inp.cpu().numpy(), g["input_nodes"])
    for i, b in enumerate(blocks):
        assert np.array_equal(b.edge_ptr.cpu().numpy(), g["b%d_ptr" % i])
        assert np.array_equal(b.src_local.cpu().numpy(), g["b%d_src_local" % i])
        assert [b.num_src_nodes(), b.num_dst_nodes()] == g["b%d_shape" % i].tolist()
    assert np.array_equal(blocks[0].src_global.cpu().numpy(), g["b0_src_global"])


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("fanouts,batch", [([15, 10, 5], 1024), ([10, 10, 10, 10, 10], 64), ([3], 1), ([64, 2], 300),
                                           # batches of 8192 and more seeds with small and mid fanouts, a single hop of fanout 16; a third
                                           # mini-batch is all hubs
                                           ([3, 16], 8192), ([3, 17], 500), ([2, 8], 8192), ([2, 5], 8193), ([4, 1], 1), ([16], 700)])
def test_sample_blocks_vs_oracle(cuda, oracle, small_graph, fused, fanouts, batch):
    import fastgl
    print("sample_blocks %s batch=%d fused=%s" % (fanouts, batch, fused), flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    sampler = fastgl.FusedMapSampler(fanouts, fused=fused, rng_seed=5).set_graph(ptr, idx)
    rng = np.random.default_rng(batch)
    hubs = np.argsort(-np.diff(indptr))
    for it in range(3):  # the later mini-batches use the next Philox streams and a reused table; the last is all hubs
        seeds = (rng.permutation(indptr.size - 1)[:batch] if it < 2 else hubs[:batch]).astype(np.int32)
        got = sampler.sample_blocks(None, dev_i32(seeds, cuda))
        check_blocks(oracle, indptr, indices, seeds, fanouts, got, 5, it * 64)


@pytest.mark.parametrize("id_order", ["first", "arrival"])
@pytest.mark.parametrize("which", ["inner", "all", "none"])
def test_transposed_blocks_come_with_the_sample(cuda, oracle, small_graph, which, id_order):
    """The fused call builds the transposed blocks itself (all, all but the outermost, or none): their offsets equal
    the oracle's transpose, rows hold the same entries, edge ids point back, the longest row is right -- on a first
    batch (worst-case bounds: the outermost hop counts with several counters per column), on batches sized by
    experience, on hub seeds (rows of hundreds of entries), and for a single hop."""
    import fastgl
    print("sample_blocks transposed=%s id_order=%s" % (which, id_order), flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    n = indptr.size - 1
    rng = np.random.default_rng(77)
    hubs = np.argsort(-np.diff(indptr))[:1100].astype(np.int32)
    for fanouts, batches in (([15, 10, 5], [rng.permutation(n)[:1100].astype(np.int32), rng.permutation(n)[:1100].astype(np.int32), hubs]),
                             ([7], [rng.permutation(n)[:300].astype(np.int32)]),
                             ([4, 4, 4, 4], [hubs[:64], hubs[64:128]])):
        sampler = fastgl.FusedMapSampler(fanouts, rng_seed=3, transposed=which, id_order=id_order).set_graph(ptr, idx)
        for it, seeds in enumerate(batches):
            got = sampler.sample_blocks(None, dev_i32(seeds, cuda))
            blocks = got[2]
            have = [b._transposed is not None for b in blocks]
            want = {"inner": [False] + [True] * (len(blocks) - 1), "all": [True] * len(blocks), "none": [False] * len(blocks)}[which]
            assert have == want
            if id_order == "first":
                check_blocks(oracle, indptr, indices, seeds, fanouts, got, 3, it * 64)
            else:  # arrival order: local ids differ from the oracle's, so the transposed blocks are checked against their own blocks
                for b in blocks:
                    if b._transposed is not None:
                        check_transposed(oracle, b, dict(n_src=b.num_src_nodes(), n_dst=b.num_dst_nodes(),
                                                         indptr=b.edge_ptr.cpu().numpy(), src_local=b.src_local.cpu().numpy()))
            fastgl.transpose_blocks(blocks)  # builds only what is missing
            assert all(b._transposed is not None for b in blocks)


@pytest.mark.parametrize("id_order", ["first", "arrival"])
@pytest.mark.parametrize("hops", [(), (0, 1), (0, 1, 2)])
def test_counts_written_where_the_host_reads_them(cuda, small_graph, hops, id_order):
    """`readback` of the all-hops call: pinned host words that the call's own kernels fill with a copy of its count
    array once the last count is final (the last hop's node total, or the longest row of the last hop's transposed
    block when that is built) -- equal to the device array after a wait for the stream, batch after batch; stale
    contents of the words never survive."""
    import torch
    from fastgl import ops
    print("sample_blocks readback hops=%s %s" % (hops, id_order), flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    n = indptr.size - 1
    rng = np.random.default_rng(5)
    plan = ops.BlocksPlan(n, 700, [5, 10, 15], cuda, transpose_hops=hops)
    host = torch.empty(3 * 3 + 2, dtype=torch.int32, pin_memory=True)
    for it in range(3):
        host.fill_(-7)
        seeds = dev_i32(rng.permutation(n)[:700].astype(np.int32), cuda)
        out = ops.sample_blocks_fused(plan, ptr, idx, seeds, 9, 64 * it, id_order=id_order, readback=host)
        torch.cuda.current_stream(cuda).synchronize()
        got, want = host.tolist(), out[4].cpu().tolist()
        assert got == want and want[2 * 3 + 1] == 0 and want[0] == 700 and want[3] > want[0]
        for h in range(3):
            assert h in hops or want[2 * 3 + 2 + h] == 0
    with pytest.raises(RuntimeError, match="pinned"):
        ops.sample_blocks_fused(plan, ptr, idx, seeds, 9, 0, readback=torch.empty(11, dtype=torch.int32))


def test_waiting_for_the_words_and_dropped_batches(cuda, oracle, small_graph):
    """The host side of the read-back: `fgl_wait_words` returns once the kernels have overwritten every pending
    word (also with no spinning at all: the stream wait), and a batch that was begun and dropped unread never
    hands its sizes to the batch that gets its host words next."""
    import gc
    import torch
    import fastgl
    from fastgl import ops
    print("wait_words / dropped pending batches", flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    n = indptr.size - 1
    rng = np.random.default_rng(6)
    plan = ops.BlocksPlan(n, 500, [5, 10, 15], cuda, transpose_hops=(0, 1))
    host = torch.empty(11, dtype=torch.int32, pin_memory=True)
    lib = fastgl.lib()
    stream = torch.cuda.current_stream(cuda).cuda_stream
    for spin_us in (5000, 0):
        host.fill_(-1)
        seeds = dev_i32(rng.permutation(n)[:500].astype(np.int32), cuda)
        out = ops.sample_blocks_fused(plan, ptr, idx, seeds, 9, 0, readback=host)
        assert lib.fgl_wait_words(host.data_ptr(), 11, -1, stream, spin_us) == 0
        got = host.tolist()
        assert -1 not in got and got == out[4].cpu().tolist()
    torch.cuda.synchronize()
    host.fill_(-1)  # nothing enqueued that would write them: reported after the stream wait, not waited for for ever
    assert lib.fgl_wait_words(host.data_ptr(), 11, -1, stream, 100) != 0
    sampler = fastgl.FusedMapSampler([15, 10, 5], rng_seed=3).set_graph(ptr, idx)
    batches = [rng.permutation(n)[:600].astype(np.int32) for _ in range(6)]
    for it, seeds in enumerate(batches):
        if it % 2 == 0:
            sampler.begin_sample(dev_i32(seeds, cuda))  # dropped at once, unread
            gc.collect()
        else:
            got = sampler.sample_blocks(None, dev_i32(seeds, cuda))
            check_blocks(oracle, indptr, indices, seeds, [15, 10, 5], got, 3, it * 64)
    assert len(sampler._host_counts[11]) <= 2


def test_sorted_transposed_blocks_equal_the_stable_transpose(cuda, oracle):
    """FGL_BLOCKS_SORT_TRANSPOSED (a deterministic sampler): every row of the transposed blocks that the call builds is in
    ascending order of its entries' positions -- the arrays equal the oracle's stable counting sort entry for entry, run
    after run.  A hand-built graph gives rows of every length class of the sort: 1, 2..8, 9..64, 65..4096 and beyond
    (merged in pieces), and one node that nobody samples."""
    import fastgl
    print("sample_blocks sorted transposed rows", flush=True)
    rng = np.random.default_rng(3)
    n = 30_000
    # node v < 24 000 has the single neighbour hub(v): hubs 0..5 are mentioned 9 000, 5 000, 3 000, 700, 40 and 6 times,
    # the other nodes point at random targets (rows of one or two entries)
    counts = [9000, 5000, 3000, 700, 40, 6]
    target = np.concatenate([np.full(c, h) for h, c in enumerate(counts)] + [rng.integers(100, n, 24_000 - sum(counts))]).astype(np.int32)
    rows = [[int(t)] for t in target] + [[] for _ in range(n - 24_000)]
    indptr, indices = _csr_from_rows(rows)
    ptr, idx = load_graph(cuda, indptr, indices)
    seeds = rng.permutation(24_000)[:20_000].astype(np.int32)
    for which in ("inner", "all"):
        first = None
        for run in range(2):
            sampler = fastgl.FusedMapSampler([3, 2], rng_seed=4, deterministic=True, transposed=which).set_graph(ptr, idx)
            inp, _, blocks = sampler.sample_blocks(None, dev_i32(seeds, cuda))
            w_inp, w_blocks = oracle.sample_blocks(indptr, indices, seeds, [3, 2], 4, 0)
            assert np.array_equal(inp.cpu().numpy(), w_inp)
            got = []
            for b, w in zip(blocks, w_blocks):
                if b._transposed is None:
                    continue
                t_ptr, t_dst, t_edge = (t.cpu().numpy() for t in b.transposed(edge_ids=True))
                w_ptr, w_idx = oracle.transpose(w["indptr"], w["src_local"], w["n_src"])
                assert np.array_equal(t_ptr, w_ptr) and np.array_equal(t_dst, w_idx)
                row_of = np.repeat(np.arange(w["n_src"]), np.diff(w_ptr))
                order = np.lexsort((t_edge, row_of))
                assert np.array_equal(order, np.arange(t_edge.size))  # positions ascend within every row
                assert np.array_equal(w["src_local"][t_edge], row_of)
                got.append((t_dst, t_edge))
            assert len(got) == (1 if which == "inner" else 2)
            longest = max(int(np.diff(oracle.transpose(w["indptr"], w["src_local"], w["n_src"])[0]).max()) for w in w_blocks[1:])
            assert longest > 4096  # the piecewise merge ran
            if first is None:
                first = got
            else:
                assert all(np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]) for a, b in zip(first, got))


def test_dataloader_with_the_trainers_constructor(cuda, oracle, small_graph):
    """fastgl.DataLoader, constructed and iterated as the reference's trainer does with DGL's (train_fastgl.py:248-258,346):
    every seed once per epoch, a different order every epoch, a short last batch unless drop_last, each mini-batch equal
    to the oracle's for its seeds and its place in the sampler's sequence of random streams."""
    import fastgl
    print("DataLoader", flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    train = dev_i32(np.random.default_rng(8).permutation(indptr.size - 1)[:2500].astype(np.int32), cuda)
    sampler = fastgl.FusedMapSampler([15, 10, 5], replace=False, rng_seed=6).set_graph(ptr, idx)
    loader = fastgl.DataLoader(None, train, sampler, use_ddp=False, batch_size=600, shuffle=True, drop_last=False,
                               prefetch_factor=2, num_workers=0)
    assert len(loader) == 5
    orders = []
    n_batch = 0
    for epoch in range(2):
        seen = []
        for step, (input_nodes, output_nodes, blocks) in enumerate(loader):
            seeds = output_nodes.cpu().numpy()
            assert seeds.size == (600 if step < 4 else 100)
            check_blocks(oracle, indptr, indices, seeds, [15, 10, 5], (input_nodes, output_nodes, blocks), 6, 64 * n_batch)
            seen.append(seeds)
            n_batch += 1
        assert step == 4
        order = np.concatenate(seen)
        assert np.array_equal(np.sort(order), np.sort(train.cpu().numpy()))
        orders.append(order)
    assert not np.array_equal(orders[0], orders[1])
    assert len(fastgl.DataLoader(None, train, sampler, batch_size=600, drop_last=True)) == 4
    plain = fastgl.DataLoader(None, train, sampler, batch_size=1000, prefetch_factor=0)
    assert [int(o.numel()) for _, o, _ in plain] == [1000, 1000, 500]
    with pytest.raises(NotImplementedError):
        fastgl.DataLoader(None, train, sampler, use_ddp=True)


def test_sample_blocks_int32_ptr_and_long_seeds(cuda, oracle, small_graph):
    import fastgl
    print("sample_blocks int32 ptr", flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr.astype(np.int32), indices)
    sampler = fastgl.FusedMapSampler([4, 4], rng_seed=1).set_graph(ptr, idx)
    seeds = np.arange(100, 612, dtype=np.int32)
    got = sampler.sample_blocks(None, torch.from_numpy(seeds.astype(np.int64)).to(cuda))  # DataLoader seeds are int64
    check_blocks(oracle, indptr, indices, seeds, [4, 4], got, 1, 0)


def test_begin_sample_then_finish(cuda, oracle, small_graph):
    """The two-phase form of sample_blocks: the outermost block is usable (bound-sized, row count on the
    device) before the sizes are read back; finish() then returns exactly what sample_blocks returns.  A batch
    that outgrows its buffers is redone inside finish() and says so."""
    import fastgl
    print("begin_sample / finish", flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    n = indptr.size - 1
    feat = torch.randn(n, 24, device=cuda)
    sampler = fastgl.FusedMapSampler([15, 10, 5], rng_seed=4).set_graph(ptr, idx)
    rng = np.random.default_rng(2)
    for batch in range(3):  # first batch: worst-case buffers; then sized by experience
        seeds = rng.permutation(n)[:700].astype(np.int32)
        pend = sampler.begin_sample(dev_i32(seeds, cuda))
        early = fastgl.aggregate(pend.outer_edge_ptr, pend.outer_src_global, feat, mode="mean", zero_policy="zeros",
                                 n_rows=pend.outer_n_dst_bound, n_rows_dev=pend.outer_n_dst, longest_row=pend.outer_fanout)
        got = pend.finish()
        assert not pend.redone
        check_blocks(oracle, indptr, indices, seeds, [15, 10, 5], got, 4, 64 * batch)
        b0 = got[2][0]
        late = fastgl.aggregate(b0.edge_ptr, b0.src_global, feat, mode="mean", zero_policy="zeros")
        # (the two launches may map lanes to rows differently -- the bound-sized one has many more rows -- and the
        # order of the fp32 additions within a row follows the mapping: equal up to rounding, not bit for bit)
        assert torch.allclose(early[:b0.num_dst_nodes()], late, rtol=1e-5, atol=1e-6)
    hubs = np.argsort(-np.diff(indptr))[:700].astype(np.int32)
    sampler._state_for(dev_i32(hubs, cuda)).nodes_seen = [700, 800, 900, 1000]  # (pretend the batches stayed tiny)
    pend = sampler.begin_sample(dev_i32(hubs, cuda))
    fastgl.aggregate(pend.outer_edge_ptr, pend.outer_src_global, feat, mode="mean", zero_policy="zeros",
                     n_rows=pend.outer_n_dst_bound, n_rows_dev=pend.outer_n_dst)  # on an overflowed batch: stays in bounds
    got = pend.finish()
    assert pend.redone
    check_blocks(oracle, indptr, indices, hubs, [15, 10, 5], got, 4, 64 * 3)


def test_undersized_buffers_are_detected_and_redone(cuda, oracle, small_graph):
    """The sampler sizes its hash table and output buffers from earlier batches; a batch that outgrows
    them must be caught by the kernels (status word) and repeated with the worst-case plan, same result."""
    import fastgl
    print("sample_blocks undersized buffers", flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    sampler = fastgl.FusedMapSampler([15, 10, 5], rng_seed=9).set_graph(ptr, idx)
    low = np.flatnonzero(np.diff(indptr) <= 1)[:512].astype(np.int32)       # a batch that hardly grows ...
    got = sampler.sample_blocks(None, dev_i32(low, cuda))
    check_blocks(oracle, indptr, indices, low, [15, 10, 5], got, 9, 0)
    state = sampler._state_for(dev_i32(low, cuda))
    state.nodes_seen = [512, 600, 700, 800]                                 # (pretend it stayed tiny)
    hubs = np.argsort(-np.diff(indptr))[:512].astype(np.int32)              # ... followed by one that explodes
    got = sampler.sample_blocks(None, dev_i32(hubs, cuda))
    check_blocks(oracle, indptr, indices, hubs, [15, 10, 5], got, 9, 64)
    assert state.nodes_seen[-1] == got[0].numel() > 4096                    # outgrew the 4096-node buffers, was redone
    got = sampler.sample_blocks(None, dev_i32(low, cuda))                   # and sized-by-experience again
    check_blocks(oracle, indptr, indices, low, [15, 10, 5], got, 9, 128)
    # the raw entry point reports both kinds of overflow instead of faulting or spinning
    seeds = dev_i32(hubs, cuda)
    plan = fastgl.BlocksPlan(indptr.size - 1, 512, [5, 10, 15], cuda)
    out = fastgl.sample_blocks_fused(plan, ptr, idx, seeds, 9, 0, table_slots=1024)
    assert out[4].tolist()[2 * 3 + 1] & 1  # FGL_STATUS_TABLE_FULL (the status word follows the 2 x 3 + 1 sizes)
    tight = fastgl.BlocksPlan(indptr.size - 1, 512, [5, 10, 15], cuda, node_capacity=[512, 600, 700, 800])
    assert tight.cap_dst == [512, 600, 700] and tight.cap_uniq == 800
    out = fastgl.sample_blocks_fused(tight, ptr, idx, seeds, 9, 0)
    c = out[4].tolist()
    assert c[2 * 3 + 1] & 2 and c[1] <= 600 and c[2] <= 700 and c[3] <= 800  # FGL_STATUS_UNIQ_OVERFLOW, counts clamped


@pytest.mark.parametrize("fanouts,batch", [([15, 10, 5], 1024), ([10, 10, 10, 10, 10], 64)])
def test_arrival_order_equals_oracle_after_canonical_sort(cuda, oracle, small_graph, fanouts, batch):
    """id_order="arrival" numbers new ids in scheduling order (the reference's rule), so local ids
    differ from run to run; in graph ids -- the canonical form -- every hop must hold exactly the
    oracle's edges, because what a node draws depends only on (seed, stream, node id)."""
    import fastgl
    print("sample_blocks arrival order %s" % fanouts, flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    sampler = fastgl.FusedMapSampler(fanouts, rng_seed=17, id_order="arrival").set_graph(ptr, idx)
    seeds = np.random.default_rng(batch + 1).permutation(indptr.size - 1)[:batch].astype(np.int32)
    for it in range(2):
        inp, _, blocks = sampler.sample_blocks(None, dev_i32(seeds, cuda))
        w_inp, w_blocks = oracle.sample_blocks(indptr, indices, seeds, fanouts, 17, it * 64)
        uniq = inp.cpu().numpy()
        assert np.array_equal(uniq[:batch], seeds)
        assert np.unique(uniq).size == uniq.size
        assert np.array_equal(np.sort(uniq), np.sort(w_inp))
        for b, w in zip(blocks, w_blocks):
            assert (b.num_src_nodes(), b.num_dst_nodes(), b.num_edges()) == (w["n_src"], w["n_dst"], w["src_local"].size)
            src_l, dst_l = (t.cpu().numpy() for t in b.edges())
            got = np.stack([uniq[dst_l], uniq[src_l]], 1)
            w_dst = np.repeat(np.arange(w["n_dst"]), np.diff(w["indptr"]))
            want = np.stack([w_inp[w_dst], w_inp[w["src_local"]]], 1)
            assert np.array_equal(got[np.lexsort((got[:, 1], got[:, 0]))], want[np.lexsort((want[:, 1], want[:, 0]))])
            # the block's node numbering is a prefix of the batch's: dst nodes first, in place
            assert set(uniq[:b.num_src_nodes()].tolist()) == set(w_inp[:w["n_src"]].tolist())
            if b.src_global is not None:
                assert np.array_equal(uniq[src_l], b.src_global.cpu().numpy())


@pytest.mark.parametrize("prefetch", [1, 2, 3])
def test_pipelined_iterator_equals_batch_by_batch(cuda, oracle, small_graph, prefetch):
    """iter_batches samples up to `prefetch` mini-batches ahead, each on a stream of its own with its own table and
    scratch; every batch must equal the oracle's (and hence sample_blocks'), also while the consumer keeps the main
    stream busy, for more batches than lanes and fewer."""
    import fastgl
    print("sample_blocks pipelined iterator, %d in flight" % prefetch, flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    rng = np.random.default_rng(77)
    batches = [rng.permutation(indptr.size - 1)[:700].astype(np.int32) for _ in range(11)]
    batches[3] = np.argsort(-np.diff(indptr))[:700].astype(np.int32)  # outgrows the buffers sized by experience
    sampler = fastgl.FusedMapSampler([15, 10, 5], rng_seed=21).set_graph(ptr, idx)
    assert len(list(sampler.iter_batches([dev_i32(batches[0], cuda)], prefetch=prefetch))) == 1
    sampler = fastgl.FusedMapSampler([15, 10, 5], rng_seed=21).set_graph(ptr, idx)
    feat = torch.randn(indptr.size - 1, 64, device=cuda)
    n = 0
    for i, got in enumerate(sampler.iter_batches((dev_i32(b, cuda) for b in batches), prefetch=prefetch)):
        check_blocks(oracle, indptr, indices, batches[i], [15, 10, 5], got, 21, i * 64)
        b0 = got[2][0]
        out = fastgl.aggregate(b0.edge_ptr, b0.src_global, feat, mode="mean", zero_policy="zeros")  # main-stream consumer
        want = oracle.aggregate(b0.edge_ptr.cpu().numpy(), b0.src_global.cpu().numpy(), feat.cpu().numpy(), "mean", 1)
        assert np.abs(out.cpu().numpy() - want).max() < 1e-5
        n += 1
    assert n == len(batches)
    assert list(sampler.iter_batches([])) == []


@pytest.mark.parametrize("pipelined", [False, True])
def test_graph_replay_equals_the_oracle_batch_after_batch(cuda, oracle, small_graph, pipelined):
    """graph_slots=2: the launch sequence is captured per slot and replayed.  Twelve mini-batches -- so every
    graph is replayed several times, with eager work of this test and of the consumer between the replays --
    each checked against the oracle (seeds and random stream change from replay to replay); one batch outgrows
    the buffers sized by experience and is redone eagerly, after which the plan changes and the graphs are
    captured anew."""
    import fastgl
    print("sample_blocks graph replay pipelined=%s" % pipelined, flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    rng = np.random.default_rng(5)
    batches = [rng.permutation(indptr.size - 1)[:700].astype(np.int32) for _ in range(12)]
    batches[7] = np.argsort(-np.diff(indptr))[:700].astype(np.int32)
    sampler = fastgl.FusedMapSampler([15, 10, 5], rng_seed=33, graph_slots=2).set_graph(ptr, idx)
    feat = torch.randn(indptr.size - 1, 32, device=cuda)
    seeds_dev = [dev_i32(b, cuda) for b in batches]
    results = sampler.iter_batches(iter(seeds_dev)) if pipelined else (sampler.sample_blocks(None, s) for s in seeds_dev)
    captures = set()
    for i, got in enumerate(results):
        check_blocks(oracle, indptr, indices, batches[i], [15, 10, 5], got, 33, i * 64)
        b0 = got[2][0]
        out = fastgl.aggregate(b0.edge_ptr, b0.src_global, feat, mode="mean", zero_policy="zeros")  # eager work between replays
        want = oracle.aggregate(b0.edge_ptr.cpu().numpy(), b0.src_global.cpu().numpy(), feat.cpu().numpy(), "mean", 1)
        assert np.abs(out.cpu().numpy() - want).max() < 1e-5
        for lane, state in enumerate(sampler._states.values()):  # (one state per mini-batch in flight when pipelined)
            if state.graphs is not None:
                captures.add((lane, state.graphs[0]))
    states = list(sampler._states.values())
    assert len(states) == (2 if pipelined else 1)
    assert all(st.graphs is not None and any(slot is not None for slot in st.graphs[2]) for st in states)  # graphs were used
    assert len(captures) >= len(states) + 1  # ... and captured anew after a plan changed


@pytest.mark.parametrize("fused", [True, False])
def test_sample_blocks_degenerate_batches(cuda, oracle, small_graph, fused):
    """no seeds, repeated seeds, seeds without neighbours: same answers as the oracle"""
    import fastgl
    print("sample_blocks degenerate fused=%s" % fused, flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    iso = np.flatnonzero(np.diff(indptr) == 0)[:40].astype(np.int32)
    hub = np.argsort(-np.diff(indptr))[:3].astype(np.int32)
    cases = [np.zeros(0, np.int32), iso, np.concatenate([hub, hub, iso[:2], hub[:1]]), np.repeat(hub[:1], 100)]
    for k, seeds in enumerate(cases):
        sampler = fastgl.FusedMapSampler([6, 4], fused=fused, rng_seed=4).set_graph(ptr, idx)
        got = sampler.sample_blocks(None, dev_i32(seeds, cuda))
        check_blocks(oracle, indptr, indices, seeds, [6, 4], got, 4, 0)
        if k == 1:
            assert all(b.num_edges() == 0 for b in got[2]) and got[0].numel() == iso.size


def _colliding_ids(n, lg_slots):
    """n distinct non-negative ids whose multiplicative hash lands in ONE home slot of a 2^lg table"""
    inv = pow(0x9E3779B1, -1, 1 << 32)
    ids, j = [], 0
    while len(ids) < n:
        v = (inv * ((0x5A << (32 - 8)) + j)) % (1 << 32)  # id * M mod 2^32 == fixed top bits | j
        j += 1
        if v < (1 << 31):
            ids.append(v)
    ids = np.array(ids, dtype=np.int64)
    home = ((ids * 0x9E3779B1) % (1 << 32)) >> (32 - lg_slots)
    assert np.unique(home).size == 1 and np.unique(ids).size == n
    return ids.astype(np.int32)


def test_hash_collisions_and_probe_limit(cuda, oracle):
    """2000 ids that all hash to one slot: long probe chains, same answer as the oracle.  5000 of them
    exceed the probe limit: reported through the status word, not by an endless loop."""
    import fastgl
    print("idmap collisions", flush=True)
    rng = np.random.default_rng(0)
    for n_ids, ok in ((2000, True), (5000, False)):
        n_edges = 20000
        lg = int(np.log2(fastgl.lib().fgl_idmap_slots(16 + n_edges)))
        ids = _colliding_ids(n_ids, lg)
        dst_unique = ids[:16].copy()
        src = ids[rng.integers(0, n_ids, size=n_edges)]
        dst = dst_unique[np.sort(rng.integers(0, 16, size=n_edges))]
        if ok:
            s, d, u = run_transfer(cuda, src, dst, dst_unique, 1 << 31)
            ws, wd, wu = oracle.idmap(src, dst, dst_unique)
            assert np.array_equal(s, ws) and np.array_equal(d, wd) and np.array_equal(u, wu)
        else:
            with pytest.raises(RuntimeError, match="hash table full"):
                run_transfer(cuda, src, dst, dst_unique, 1 << 31)


def test_random_configurations_against_the_oracle(cuda, oracle):
    """Thirty seeded random configurations -- graph size and density, 1 to 4 hops, fanouts 1 to 192 (all three
    sampling kernels), int32 and int64 offsets, repeated seeds, plain launches and graph replay, three
    mini-batches each -- every output bit for bit against the oracle."""
    import fastgl
    rng = np.random.default_rng(123)
    for case in range(30):
        n = int(rng.integers(50, 20000))
        indptr, indices = oracle.rmat_csr(n, int(n * rng.uniform(0.5, 20)), seed=int(rng.integers(0, 1000)),
                                          indptr_dtype=np.int64 if case % 2 else np.int32)
        hops = int(rng.integers(1, 5))
        fanouts = [int(rng.integers(1, 41)) if rng.random() < 0.8 else int(rng.integers(41, 193)) for _ in range(hops)]
        n_seeds = int(rng.integers(1, min(n, 2000) + 1))
        seeds = rng.permutation(n)[:n_seeds].astype(np.int32)
        if case % 7 == 0:
            seeds[rng.integers(0, n_seeds)] = seeds[0]
        rng_seed = int(rng.integers(0, 2 ** 40))
        print("random configuration %d: n=%d fanouts=%s seeds=%d" % (case, n, fanouts, n_seeds), flush=True)
        ptr, idx = load_graph(cuda, indptr, indices)
        sampler = fastgl.FusedMapSampler(fanouts, rng_seed=rng_seed, graph_slots=2 if case % 3 == 0 else 0).set_graph(ptr, idx)
        for batch in range(3):
            got = sampler.sample_blocks(None, dev_i32(seeds, cuda))
            check_blocks(oracle, indptr, indices, seeds, fanouts, got, rng_seed, batch * 64)


@pytest.mark.parametrize("n_edges", [5000, 2_200_000])
def test_final_call_leaves_the_table_alone_and_the_results_unchanged(cuda, oracle, n_edges):
    """FGL_IDMAP_FINAL (the caller will not consult the table again): same relabelled edges, same unique list,
    same count as without it -- on both sides of the tile count where the number pass changes form -- and the new
    ids' slots keep their transient value, so a later lookup of a new id reports it (top bit set = not a local id)."""
    import ctypes as C
    import fastgl
    from fastgl import _lib as L
    print("idmap final n_edges=%d" % n_edges, flush=True)
    rng = np.random.default_rng(n_edges)
    n_dst = 300
    dst_unique = rng.choice(10**6, size=n_dst, replace=False).astype(np.int32)
    src = rng.integers(0, 3 * 10**6, size=n_edges).astype(np.int32)
    src[::5] = dst_unique[rng.integers(0, n_dst, size=src[::5].size)]     # ids that are numbered already
    lib = fastgl.lib()
    capacity = n_dst + n_edges
    slots = lib.fgl_idmap_slots(capacity)
    results = []
    for flags in (L.IDMAP_ORDERED, L.IDMAP_ORDERED | L.IDMAP_FINAL):
        table = torch.empty(slots, dtype=torch.int64, device=cuda)
        uniq = torch.empty(capacity, dtype=torch.int32, device=cuda)
        meta = torch.zeros(2, dtype=torch.int32, device=cuda)
        d_src, d_out = dev_i32(src, cuda), torch.empty(n_edges, dtype=torch.int32, device=cuda)
        ws = torch.empty(lib.fgl_idmap_map_src_workspace_bytes(n_edges), dtype=torch.uint8, device=cuda)
        st = L.stream_handle()
        L.check(lib.fgl_idmap_reset(L.ptr(table), slots, st))
        L.check(lib.fgl_idmap_insert_dst(L.ptr(table), slots, L.ptr(dev_i32(dst_unique, cuda)), n_dst, None, L.ptr(uniq),
                                         meta.data_ptr() + 4, st))
        L.check(lib.fgl_idmap_map_src(L.ptr(table), slots, L.ptr(d_src), L.ptr(d_out), n_edges, None, n_dst, None,
                                      meta.data_ptr(), L.ptr(uniq), capacity, flags, meta.data_ptr() + 4, L.ptr(ws), ws.numel(), st))
        n_total, status = meta.tolist()
        assert status == 0
        probe = d_src.clone()
        L.check(lib.fgl_idmap_lookup(L.ptr(table), slots, L.ptr(probe), n_edges, None, meta.data_ptr() + 4, st))
        results.append((d_out.cpu().numpy(), uniq[:n_total].cpu().numpy(), probe.cpu().numpy()))
    (out_a, uniq_a, look_a), (out_b, uniq_b, look_b) = results
    ws_, _, wu = oracle.idmap(src, np.zeros(n_edges, np.int32) + dst_unique[0], dst_unique)
    assert np.array_equal(out_a, ws_) and np.array_equal(uniq_a, wu)
    assert np.array_equal(out_b, out_a) and np.array_equal(uniq_b, uniq_a)
    assert np.array_equal(look_a, out_a)                      # written back: the table answers for every id
    new = out_a >= n_dst
    assert np.array_equal(look_b[~new], out_a[~new])          # ids numbered before the call: unchanged
    assert (look_b[new] < 0).all()                            # new ids: still the transient value (top bit set)


@pytest.mark.parametrize("n_edges", [5000, 262_144, 262_145, 900_000])
def test_arrival_order_through_the_c_abi(cuda, oracle, n_edges):
    """FGL_IDMAP_ARRIVAL (the reference's numbering rule) on both sides of the size where its insert pass changes
    from one edge per lane to eight: the order-free characterisation of a correct map -- destinations keep their
    positions, no id twice, the new ids are exactly the sources that are not destinations, every edge points at
    its own id -- and equality with the oracle after sorting the new ids.  In place (src_out = src_in)."""
    import fastgl
    from fastgl import _lib as L
    print("idmap arrival n_edges=%d" % n_edges, flush=True)
    rng = np.random.default_rng(n_edges + 1)
    n_dst = 500
    dst_unique = rng.choice(10**6, size=n_dst, replace=False).astype(np.int32)
    src = ((rng.pareto(1.1, size=n_edges) * 40).astype(np.int64) % (2 * 10**6)).astype(np.int32)   # hot ids repeat a lot
    src[::6] = dst_unique[rng.integers(0, n_dst, size=src[::6].size)]
    lib = fastgl.lib()
    capacity = n_dst + n_edges
    slots = lib.fgl_idmap_slots(capacity)
    table = torch.empty(slots, dtype=torch.int64, device=cuda)
    uniq = torch.empty(capacity, dtype=torch.int32, device=cuda)
    meta = torch.zeros(2, dtype=torch.int32, device=cuda)
    d_src = dev_i32(src, cuda)
    ws = torch.empty(lib.fgl_idmap_map_src_workspace_bytes(n_edges), dtype=torch.uint8, device=cuda)
    st = L.stream_handle()
    L.check(lib.fgl_idmap_reset(L.ptr(table), slots, st))
    L.check(lib.fgl_idmap_insert_dst(L.ptr(table), slots, L.ptr(dev_i32(dst_unique, cuda)), n_dst, None, L.ptr(uniq),
                                     meta.data_ptr() + 4, st))
    L.check(lib.fgl_idmap_map_src(L.ptr(table), slots, L.ptr(d_src), L.ptr(d_src), n_edges, None, n_dst, None,
                                  meta.data_ptr(), L.ptr(uniq), capacity, L.IDMAP_ARRIVAL, meta.data_ptr() + 4, L.ptr(ws),
                                  ws.numel(), st))
    n_total, status = meta.tolist()
    assert status == 0
    out, u = d_src.cpu().numpy(), uniq[:n_total].cpu().numpy()
    assert np.array_equal(u[:n_dst], dst_unique)
    assert np.unique(u).size == u.size
    assert set(u[n_dst:].tolist()) == set(src.tolist()) - set(dst_unique.tolist())
    assert out.min() >= 0 and out.max() < n_total and np.array_equal(u[out], src)
    ws_, _, wu = oracle.idmap(src, np.zeros(n_edges, np.int32) + dst_unique[0], dst_unique)
    cs, cu = canonical(out, u, n_dst, None)
    cws, cwu = canonical(ws_, wu, n_dst, None)
    assert np.array_equal(cs, cws) and np.array_equal(cu, cwu)
    # the table answers for every id afterwards (arrival order always writes the numbers back)
    probe = dev_i32(src, cuda)
    L.check(lib.fgl_idmap_lookup(L.ptr(table), slots, L.ptr(probe), n_edges, None, meta.data_ptr() + 4, st))
    assert np.array_equal(probe.cpu().numpy(), out)


def test_negative_ids_are_reported_not_inserted(cuda):
    """An id of -1 has the bit pattern of the table's empty marker, any negative id is no node id: the id-map
    reports them (status bit, RuntimeError from the operator), gives their edges the local id -1 and leaves the
    table intact -- lookups of the good ids still work."""
    import fastgl
    from fastgl import _lib as L
    print("id-map: negative ids", flush=True)
    lib = L.lib()
    for flags in (L.IDMAP_ORDERED, L.IDMAP_ARRIVAL):
        slots = lib.fgl_idmap_slots(64)
        table = torch.empty(slots, dtype=torch.int64, device=cuda)
        dst = torch.tensor([7, 3, 9], dtype=torch.int32, device=cuda)
        src = torch.tensor([3, -1, 11, 7, -5, 11, 12], dtype=torch.int32, device=cuda)
        uniq = torch.full((16,), -9, dtype=torch.int32, device=cuda)
        meta = torch.zeros(2, dtype=torch.int32, device=cuda)
        ws = torch.empty(lib.fgl_idmap_map_src_workspace_bytes(src.numel()), dtype=torch.uint8, device=cuda)
        st = L.stream_handle()
        L.check(lib.fgl_idmap_reset(L.ptr(table), slots, st))
        L.check(lib.fgl_idmap_insert_dst(L.ptr(table), slots, L.ptr(dst), 3, None, L.ptr(uniq), meta.data_ptr() + 4, st))
        L.check(lib.fgl_idmap_map_src(L.ptr(table), slots, L.ptr(src), L.ptr(src), src.numel(), None, 3, None, meta.data_ptr(),
                                      L.ptr(uniq), 16, flags, meta.data_ptr() + 4, L.ptr(ws), ws.numel(), st))
        n_total, status = meta.tolist()
        assert status == L.STATUS_BAD_ID and n_total == 5
        got = src.tolist()
        assert got[0] == 1 and got[3] == 0 and got[1] == -1 and got[4] == -1
        assert got[2] == got[5] and sorted({got[2], got[6]}) == [3, 4]
        assert sorted(uniq[3:5].tolist()) == [11, 12] and uniq[:3].tolist() == [7, 3, 9]
        probe = torch.tensor([12, 9, 11, 3], dtype=torch.int32, device=cuda)
        meta.zero_()
        L.check(lib.fgl_idmap_lookup(L.ptr(table), slots, L.ptr(probe), 4, None, meta.data_ptr() + 4, st))
        assert meta.tolist()[1] == 0 and probe.tolist() == [got[6], 2, got[2], 1]
    # through the drop-in operator: a RuntimeError that names the cause
    src = torch.tensor([3, -1, 11], dtype=torch.int32, device=cuda)
    d = torch.tensor([7, 7, 3], dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError, match="negative id"):
        fastgl.transfer_edge_id(src, d, torch.tensor([7, 3], dtype=torch.int32, device=cuda), 2, 5, 3, 3)
    # a negative destination id
    meta = torch.zeros(2, dtype=torch.int32, device=cuda)
    slots = lib.fgl_idmap_slots(8)
    table = torch.empty(slots, dtype=torch.int64, device=cuda)
    L.check(lib.fgl_idmap_reset(L.ptr(table), slots, L.stream_handle()))
    bad = torch.tensor([4, -1, 6], dtype=torch.int32, device=cuda)
    L.check(lib.fgl_idmap_insert_dst(L.ptr(table), slots, L.ptr(bad), 3, None, None, meta.data_ptr() + 4, L.stream_handle()))
    assert meta.tolist()[1] == L.STATUS_BAD_ID
    probe = torch.tensor([6, 4], dtype=torch.int32, device=cuda)
    meta.zero_()
    L.check(lib.fgl_idmap_lookup(L.ptr(table), slots, L.ptr(probe), 2, None, meta.data_ptr() + 4, L.stream_handle()))
    assert probe.tolist() == [2, 0] and meta.tolist()[1] == 0


def test_a_short_last_batch_keeps_what_the_full_batches_learned(cuda, oracle, small_graph):
    """An epoch ends with a batch of fewer seeds; the next epoch starts with full batches again.  Plans, learned
    buffer sizes and captured graphs are kept per batch shape, so neither change of shape starts from the
    worst-case plan again -- also with the next batch launched before the current one is finished."""
    import fastgl
    print("sample_blocks: short last batch", flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    rng = np.random.default_rng(17)
    sizes = [600, 600, 600, 150, 600, 600, 150, 600]
    batches = [rng.permutation(indptr.size - 1)[:n].astype(np.int32) for n in sizes]
    for pipelined in (False, True):
        sampler = fastgl.FusedMapSampler([15, 10, 5], rng_seed=2).set_graph(ptr, idx)
        seeds_dev = [dev_i32(b, cuda) for b in batches]
        results = sampler.iter_batches(iter(seeds_dev)) if pipelined else (sampler.sample_blocks(None, s) for s in seeds_dev)
        plans_full = []
        for i, got in enumerate(results):
            check_blocks(oracle, indptr, indices, batches[i], [15, 10, 5], got, 2, i * 64)
            full = sampler._state_for(seeds_dev[0])
            plans_full.append({k: id(v) for k, v in full.plans.items()})
        assert len({key[:-1] for key in sampler._states}) == 2  # (two shapes; when pipelined, each on both lanes)
        full, short = sampler._state_for(seeds_dev[0]), sampler._state_for(seeds_dev[3])
        assert full.nodes_seen is not None and short.nodes_seen is not None and full.nodes_seen[0] == 600 and short.nodes_seen[0] == 150
        # the full-size shape's sized-by-experience plan of batch 2 is still the one in use at the end
        sized = [k for k in plans_full[2] if k is not None]
        assert sized and all(plans_full[j].get(sized[0]) == plans_full[2][sized[0]] for j in range(3, len(sizes)))


@pytest.mark.parametrize("id_order", ["first", "arrival"])
@pytest.mark.parametrize("fanouts,n_seeds", [([64, 3], 3000), ([2, 50], 3000), ([33, 20], 700), ([192, 1], 2000), ([3, 3, 3, 3, 3], 4000),
                                             ([4, 2], 70_000), ([49, 2], 70_000), ([15, 10, 5], 1), ([1], 5000)])
def test_hops_of_mixed_shapes_chain_correctly(cuda, oracle, small_graph, id_order, fanouts, n_seeds):
    """Each hop's passes prepare the next hop's sampling (row starts, degrees, per-tile edge counts): fanouts on both sides
    of the tile-size rules (256-seed tiles only beyond 65 536 seeds and up to fanout 48), of the register-held picks (32)
    and of the small-hop threshold, so that consecutive hops use different tile sizes and kernels; one to five hops."""
    import fastgl
    print("sample_blocks hops %s seeds %d %s" % (fanouts, n_seeds, id_order), flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    rng = np.random.default_rng(len(fanouts) * 1000 + n_seeds)
    sampler = fastgl.FusedMapSampler(fanouts, rng_seed=12, id_order=id_order).set_graph(ptr, idx)
    for batch in range(2):  # worst-case buffers first, then sized by experience (and the table left empty by the first)
        seeds = rng.permutation(indptr.size - 1)[:n_seeds].astype(np.int32)
        got = sampler.sample_blocks(None, dev_i32(seeds, cuda))
        if id_order == "first":
            check_blocks(oracle, indptr, indices, seeds, fanouts, got, 12, 64 * batch)
            continue
        inp, _, blocks = got
        w_inp, w_blocks = oracle.sample_blocks(indptr, indices, seeds, fanouts, 12, 64 * batch)
        inp_h = inp.cpu().numpy().astype(np.int64)
        assert inp_h.size == w_inp.size and np.array_equal(inp_h[:n_seeds], seeds)
        for b, w in zip(blocks, w_blocks):
            nd, ns = w["n_dst"], w["n_src"]
            assert (b.num_src_nodes(), b.num_dst_nodes(), b.num_edges()) == (ns, nd, int(w["src_local"].size))
            assert np.array_equal(np.sort(inp_h[nd:ns]), np.sort(w_inp[nd:ns]))
            a_src, a_dst = (t.cpu().numpy() for t in b.edges())
            w_dst = np.repeat(np.arange(nd), np.diff(w["indptr"]))
            assert np.array_equal(np.sort((inp_h[a_dst] << 32) | inp_h[a_src]),
                                  np.sort((w_inp[w_dst].astype(np.int64) << 32) | w["src_global"].astype(np.int64)))


def _csr_from_rows(rows, ptr_dtype=np.int64):
    indptr = np.zeros(len(rows) + 1, dtype=ptr_dtype)
    indptr[1:] = np.cumsum([len(r) for r in rows])
    return indptr, np.asarray([v for r in rows for v in r], dtype=np.int32)


@pytest.mark.parametrize("id_order", ["first", "arrival"])
def test_hand_built_graphs_with_repeated_neighbours_self_loops_and_a_hub(cuda, oracle, id_order):
    """Graphs that an R-MAT generator never makes: rows that list a neighbour several times and themselves (the
    sampler draws positions, so such rows give repeated sources within one seed), rows of exactly fanout - 1,
    fanout and fanout + 1 entries, isolated nodes -- and a star: every node lists the hub, so the hub's row of the
    transposed block holds one entry per seed (far beyond the 128 entries that the backward gather leaves to its
    hub-row launch).  Sampling, id-map, forward and backward gathers against the oracle."""
    import fastgl
    print("hand-built graphs, id_order=%s" % id_order, flush=True)
    rng = np.random.default_rng(17)
    n = 3000
    rows = []
    for v in range(n):
        kind = v % 6
        if kind == 0:
            row = []                                             # isolated
        elif kind == 1:
            row = [v, v, (v + 1) % n]                            # self loops, one of them twice
        elif kind == 2:
            row = [(v + 7) % n] * 9                              # one neighbour nine times
        else:
            row = rng.integers(0, n, size=(3, 4, 5)[kind - 3]).tolist()  # fanout - 1, fanout, fanout + 1 entries
        rows.append([0] + row if v != 0 else row)                # the star: everyone lists node 0 first
    indptr, indices = _csr_from_rows(rows)
    ptr, idx = load_graph(cuda, indptr, indices)
    fanouts = [4, 4]
    seeds = rng.permutation(n)[:2000].astype(np.int32)
    sampler = fastgl.FusedMapSampler(fanouts, rng_seed=9, id_order=id_order).set_graph(ptr, idx)
    for batch in range(2):
        got = sampler.sample_blocks(None, dev_i32(seeds, cuda))
        inp, _, blocks = got
        w_inp, w_blocks = oracle.sample_blocks(indptr, indices, seeds, fanouts, 9, batch * 64)
        if id_order == "first":
            check_blocks(oracle, indptr, indices, seeds, fanouts, got, 9, batch * 64)
        else:  # any numbering of the new ids is a valid map: compare the edges in graph ids, hop by hop
            uniq = inp.cpu().numpy()
            for b, w in zip(blocks, w_blocks):
                assert (b.num_src_nodes(), b.num_dst_nodes()) == (w["n_src"], w["n_dst"])
                src, dst = b.edges()
                got_keys = np.sort(uniq[dst.cpu().numpy()].astype(np.int64) << 32 | uniq[src.cpu().numpy()])
                want_keys = np.sort(w_inp[np.repeat(np.arange(w["n_dst"]), np.diff(w["indptr"]))].astype(np.int64) << 32 | w["src_global"])
                assert np.array_equal(got_keys, want_keys)
            assert np.array_equal(np.sort(uniq), np.sort(w_inp))
    # the outermost block: forward mean, then the backward gather over its transpose, whose hub row is long
    b = blocks[0]
    n_src, n_dst = b.num_src_nodes(), b.num_dst_nodes()
    ptr_h, src_h = b.edge_ptr.cpu().numpy(), b.src_local.cpu().numpy()
    hub_local = int(np.flatnonzero(inp.cpu().numpy() == 0)[0])
    assert int((src_h == hub_local).sum()) > 1000
    X = torch.from_numpy(rng.standard_normal((n_src, 48)).astype(np.float32)).to(cuda)
    out = fastgl.aggregate(b.edge_ptr, b.src_local, X, mode="mean", zero_policy="zeros", n_rows=n_dst)
    want = oracle.aggregate(ptr_h, src_h, X.cpu().numpy(), "mean", 1)
    assert np.abs(out.cpu().numpy() - want).max() <= 1e-5 * max(np.abs(want).max(), 1.0)
    t_ptr, t_idx = b.transposed()[:2]
    assert int(torch.diff(t_ptr).max()) > 1000  # the hub
    d_out = torch.from_numpy(rng.standard_normal((n_dst, 48)).astype(np.float32)).to(cuda)
    d_x = fastgl.aggregate(t_ptr, t_idx, d_out, mode="colmean", zero_policy="zeros", col_norm=b.in_degrees().contiguous(), n_rows=n_src)
    tp, ti = oracle.transpose(ptr_h, src_h, n_src)
    deg = np.maximum(np.diff(ptr_h), 1).astype(np.int32)
    want = oracle.aggregate(tp, ti, d_out.cpu().numpy(), "colmean", 1, None, deg)
    assert np.abs(d_x.cpu().numpy() - want).max() <= 1e-5 * max(np.abs(want).max(), 1.0)


def test_block_degrees_with_and_without_the_transpose(cuda, oracle, small_graph):
    """``Block.out_degrees()`` counts with a histogram pass, or reads the transposed block's row lengths if the
    transpose is already there: the same numbers either way."""
    import fastgl
    print("Block.in_degrees / out_degrees", flush=True)
    indptr, indices = small_graph
    ptr, idx = load_graph(cuda, indptr, indices)
    seeds = np.random.default_rng(2).permutation(indptr.size - 1)[:2048].astype(np.int32)
    sampler = fastgl.FusedMapSampler([15, 10, 5], rng_seed=1).set_graph(ptr, idx)
    for transposed_first in (False, True):
        _, _, blocks = sampler.sample_blocks(None, dev_i32(seeds, cuda))
        if transposed_first:
            fastgl.transpose_blocks(blocks)
        for b in blocks:
            src = b.src_local.cpu().numpy()
            assert np.array_equal(b.out_degrees().cpu().numpy(), np.bincount(src, minlength=b.num_src_nodes()))
            assert np.array_equal(b.in_degrees().cpu().numpy(), np.diff(b.edge_ptr.cpu().numpy()))
