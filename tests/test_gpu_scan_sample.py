"""HIP scan / histogram / sampling against the oracle (bit-exact), through the C ABI."""
import numpy as np
import pytest
import torch
from scipy import stats

pytestmark = pytest.mark.gpu


def dev_i32(a, cuda):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(cuda)


# one tile (a single launch), a few tiles (offsets summed by each workgroup), beyond 4096 tiles (scan launch in between)
@pytest.mark.parametrize("n", [0, 1, 63, 2047, 2048, 2049, 100_000, 3_000_001, 8_388_607, 8_388_608, 9_000_001])
def test_exclusive_sum(cuda, oracle, n):
    import fastgl
    print("exclusive_sum n=%d" % n, flush=True)
    v = np.random.default_rng(n).integers(0, 16, size=n).astype(np.int32)
    got = fastgl.exclusive_sum(dev_i32(v, cuda)).cpu().numpy()
    assert np.array_equal(got, oracle.exclusive_sum(v))


@pytest.mark.parametrize("n_ids,n_nodes", [(0, 5), (1000, 10), (500_000, 70_000), (300_000, 1)])
def test_cal_deg(cuda, oracle, n_ids, n_nodes):
    import fastgl
    print("cal_deg %d %d" % (n_ids, n_nodes), flush=True)
    ids = np.random.default_rng(1).integers(0, n_nodes, size=n_ids).astype(np.int32)
    got = fastgl.cal_deg(dev_i32(ids, cuda), n_nodes).cpu().numpy()
    assert np.array_equal(got, oracle.cal_deg(ids, n_nodes))


def _sample(cuda, indptr, indices, seeds, fanout, seed, stream):
    import fastgl
    fastgl.manual_seed(seed)
    fastgl.ops._rng_state["calls"] = stream
    ptr = torch.from_numpy(indptr).to(cuda)
    idx = dev_i32(indices, cuda)
    src, dst, num = fastgl.sample_node(idx, idx, ptr, dev_i32(seeds, cuda), len(seeds), fanout)
    bptr = fastgl.sample_node.last_block_ptr
    assert int(num.item()) == src.numel() == dst.numel()
    return src.cpu().numpy(), dst.cpu().numpy(), bptr.cpu().numpy()


@pytest.mark.parametrize("ptr_dtype", [np.int32, np.int64])
@pytest.mark.parametrize("fanout", [1, 5, 8, 9, 15, 16, 17, 20, 29, 30, 32, 33, 48, 49, 64, 192])
def test_sample_bit_exact_vs_oracle(cuda, oracle, small_graph, ptr_dtype, fanout):
    print("sample fanout=%d ptr=%s" % (fanout, ptr_dtype.__name__), flush=True)
    indptr, indices = small_graph
    indptr = indptr.astype(ptr_dtype)
    seeds = np.random.default_rng(fanout).permutation(indptr.size - 1)[:5000].astype(np.int32)
    src, dst, bptr = _sample(cuda, indptr, indices, seeds, fanout, seed=77, stream=fanout)
    wsrc, wdst, wptr = oracle.sample_node(indptr, indices, seeds, fanout, rng_seed=77, stream_id=fanout)
    assert np.array_equal(bptr, wptr)
    assert np.array_equal(dst, wdst)
    assert np.array_equal(src, wsrc)


@pytest.mark.parametrize("n_seeds", [1_048_576, 1_048_577, 1_300_000])
def test_sample_many_seeds_vs_oracle(cuda, oracle, small_graph, n_seeds):
    """Around 4096 tiles of 256 seeds the way the tile offsets are derived changes (summed by each
    workgroup below, a scan launch above): same bits either way."""
    print("sample %d seeds" % n_seeds, flush=True)
    indptr, indices = small_graph
    seeds = np.random.default_rng(n_seeds).integers(0, indptr.size - 1, size=n_seeds).astype(np.int32)
    src, dst, bptr = _sample(cuda, indptr, indices, seeds, 5, seed=3, stream=1)
    wsrc, wdst, wptr = oracle.sample_node(indptr, indices, seeds, 5, rng_seed=3, stream_id=1)
    assert np.array_equal(bptr, wptr) and np.array_equal(dst, wdst) and np.array_equal(src, wsrc)


def test_sample_full_neighbourhood_closed_form(cuda, small_graph):
    print("sample full neighbourhood", flush=True)
    indptr, indices = small_graph
    deg_all = np.diff(indptr)
    cand = np.flatnonzero(deg_all <= 192)
    seeds = np.random.default_rng(5).choice(cand, size=3000, replace=False).astype(np.int32)
    src, dst, bptr = _sample(cuda, indptr, indices, seeds, 192, seed=1, stream=0)
    deg = deg_all[seeds]
    assert np.array_equal(bptr, np.concatenate([[0], np.cumsum(deg)]))
    assert np.array_equal(src, np.concatenate([indices[indptr[s]:indptr[s + 1]] for s in seeds]))
    assert np.array_equal(dst, np.repeat(seeds, deg))


def test_sample_edge_cases(cuda, oracle, small_graph):
    import fastgl
    print("sample edge cases", flush=True)
    indptr, indices = small_graph
    # no seeds
    src, dst, bptr = _sample(cuda, indptr, indices, np.zeros(0, np.int32), 5, 0, 0)
    assert src.size == 0 and bptr.tolist() == [0]
    # isolated nodes only, repeated seeds, a single seed of maximal degree
    iso = np.flatnonzero(np.diff(indptr) == 0)[:7].astype(np.int32)
    hub = np.array([np.argmax(np.diff(indptr))], np.int32)
    for seeds in (iso, np.repeat(hub, 300), hub, np.concatenate([iso, hub, iso])):
        got = _sample(cuda, indptr, indices, seeds, 15, 9, 4)
        want = oracle.sample_node(indptr, indices, seeds, 15, rng_seed=9, stream_id=4)
        for g, w in zip(got, want):
            assert np.array_equal(g, w)
    # a seed outside the graph is reported, never dereferenced
    with pytest.raises(RuntimeError, match="outside the graph"):
        _sample(cuda, indptr, indices, np.array([indptr.size + 5], np.int32), 5, 0, 0)
    with pytest.raises(RuntimeError, match="fanout"):
        _sample(cuda, indptr, indices, hub, 193, 0, 0)


def test_sample_chi_square_on_device(cuda):
    """uniformity of the HIP sampler itself: ring graph of degree 40, fanout 15"""
    print("sample chi-square", flush=True)
    n, deg, fanout = 30000, 40, 15
    indptr = np.arange(0, (n + 1) * deg, deg, dtype=np.int64)
    indices = ((np.arange(n)[:, None] + np.arange(1, deg + 1)[None, :]) % n).astype(np.int32).ravel()
    src, dst, bptr = _sample(cuda, indptr, indices, np.arange(n, dtype=np.int32), fanout, seed=31337, stream=2)
    assert np.array_equal(np.diff(bptr), np.full(n, fanout))
    offs = (src.astype(np.int64) - dst - 1) % n
    per_seed = offs.reshape(n, fanout)
    assert (np.sort(per_seed, 1)[:, 1:] != np.sort(per_seed, 1)[:, :-1]).all()  # no duplicates
    counts = np.bincount(offs, minlength=deg)
    expect = n * fanout / deg
    stat = ((counts - expect) ** 2 / expect).sum() * (deg - 1) / (deg - fanout)
    assert stats.chi2.sf(stat, deg - 1) > 1e-4


@pytest.mark.parametrize("where", ["pinned_host", "device"])
def test_sizes_written_where_the_caller_reads_them(cuda, small_graph, where):
    """d_readback of fgl_sample_node / fgl_idmap_transfer: {size, status word}, written by the call's own launches --
    into pinned host memory (no copy to enqueue: wait, read) or into device memory.  With and without a status bit;
    zero seeds; more than a million seeds (the size then comes from the scan launch)."""
    from fastgl import _lib as L
    lib = L.lib()
    print("read-back pair in %s memory" % where, flush=True)
    indptr, indices = small_graph
    ptr, idx = torch.from_numpy(indptr).to(cuda), dev_i32(indices, cuda)
    n_nodes = indptr.size - 1
    rb = torch.full((2,), -7, dtype=torch.int32, pin_memory=True) if where == "pinned_host" else torch.full((2,), -7, dtype=torch.int32, device=cuda)
    st = L.stream_handle()
    rng = np.random.default_rng(9)
    for n_seeds, fanout, bad in ((3000, 7, False), (3000, 7, True), (0, 5, False), (1_100_000, 2, False)):
        seeds = rng.integers(0, n_nodes, size=n_seeds).astype(np.int32)
        if bad:
            seeds[17] = n_nodes + 5
        d_seeds = dev_i32(seeds, cuda)
        cap = max(n_seeds * fanout, 1)
        src, bptr = torch.empty(cap, dtype=torch.int32, device=cuda), torch.empty(n_seeds + 1, dtype=torch.int32, device=cuda)
        meta = torch.zeros(2, dtype=torch.int32, device=cuda)
        ws = torch.empty(max(lib.fgl_sample_workspace_bytes(n_seeds, fanout), 256), dtype=torch.uint8, device=cuda)
        rb.fill_(-7)
        torch.cuda.synchronize()
        L.check(lib.fgl_sample_node(L.ptr(ptr), 1, L.ptr(idx), n_nodes, L.ptr(d_seeds), n_seeds, None, fanout, 3, 1, L.ptr(src), None,
                                    L.ptr(bptr), meta.data_ptr(), meta.data_ptr() + 4, rb.data_ptr(), L.ptr(ws), ws.numel(), st))
        torch.cuda.synchronize()
        assert rb.tolist() == meta.tolist() == [int(bptr[-1]), 8 if bad else 0]
    # the fused id-map: node total and status
    for missing in (False, True):
        dst_unique = np.arange(100, 164, dtype=np.int32)
        src_e = rng.integers(0, 500, size=1000).astype(np.int32)
        dst_e = np.sort(rng.integers(100, 164, size=1000)).astype(np.int32)
        if missing:
            dst_e[5] = 99
        slots = lib.fgl_idmap_slots(64 + 1000)
        table = torch.full((slots,), -1, dtype=torch.int64, device=cuda)
        uniq = torch.empty(64 + 1000, dtype=torch.int32, device=cuda)
        meta = torch.zeros(2, dtype=torch.int32, device=cuda)
        ws = torch.empty(max(lib.fgl_idmap_map_src_workspace_bytes(1000), 256), dtype=torch.uint8, device=cuda)
        d_src, d_dst = dev_i32(src_e, cuda), dev_i32(dst_e, cuda)
        rb.fill_(-7)
        torch.cuda.synchronize()
        L.check(lib.fgl_idmap_transfer(L.ptr(table), slots, L.ptr(dev_i32(dst_unique, cuda)), 64, L.ptr(d_src), L.ptr(d_dst), 1000,
                                       L.ptr(uniq), 64 + 1000, L.IDMAP_ORDERED | L.IDMAP_FINAL | L.IDMAP_LEAVE_TABLE_EMPTY,
                                       meta.data_ptr(), meta.data_ptr() + 4, rb.data_ptr(), L.ptr(ws), ws.numel(), st))
        torch.cuda.synchronize()
        n_total = 64 + np.setdiff1d(src_e, dst_unique).size
        assert rb.tolist() == meta.tolist() == [n_total, 4 if missing else 0]
        assert bool((table == -1).all())  # left empty for the next call
        assert np.array_equal(uniq[:n_total].cpu().numpy()[d_src.cpu().numpy()], src_e)
