"""HIP aggregation (forward, and backward as a gather over the transposed block) against the
fp64 oracle, through the C ABI.  Tolerances are the acceptance criterion's: 1e-5 relative
for fp32 and 1e-2 for bf16, relative to the largest magnitude of the fp64 result row-block."""
import os

import numpy as np
import pytest
import torch

from conftest import GOLDEN_DIR

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2}


def dev_i32(a, cuda):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(cuda)


def rel_err(got, want):
    scale = max(np.abs(want).max(), 1e-30)
    return np.abs(got.astype(np.float64) - want).max() / scale


def make_block(rng, n_dst, n_src, max_deg, hubs=()):
    deg = rng.integers(0, max_deg + 1, size=n_dst)
    for r, d in hubs:
        deg[r] = d
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    idx = rng.integers(0, n_src, size=ptr[-1]).astype(np.int32)
    return ptr, idx, deg


def run_modes(cuda, oracle, ptr, idx, deg, X_t, n_src, tol):
    import fastgl
    X_ref = X_t.float().cpu().numpy()  # the exact values the kernel reads (bf16 widened)
    rn = np.maximum(deg, 1).astype(np.int32)
    cn = np.maximum(np.bincount(idx, minlength=n_src), 1).astype(np.int32)
    d_ptr, d_idx, d_rn, d_cn = dev_i32(ptr, cuda), dev_i32(idx, cuda), dev_i32(rn, cuda), dev_i32(cn, cuda)
    for mode in ("sum", "mean", "gcn", "colmean"):
        for pol_name, pol in (("self", 0), ("zeros", 1)):
            want = oracle.aggregate(ptr, idx, X_ref, mode, pol, rn, cn)
            got = fastgl.aggregate(d_ptr, d_idx, X_t, mode=mode, zero_policy=pol_name, row_norm=d_rn, col_norm=d_cn)
            assert got.dtype == X_t.dtype and tuple(got.shape) == want.shape
            err = rel_err(got.float().cpu().numpy(), want)
            assert err < tol, (mode, pol_name, err)
            if mode == "colmean":
                # the same weights from an offsets array whose differences are the (unclamped) column counts
                cptr = np.concatenate([[0], np.cumsum(np.bincount(idx, minlength=n_src))]).astype(np.int32)
                again = fastgl.aggregate(d_ptr, d_idx, X_t, mode="colmean_ptr", zero_policy=pol_name, col_norm=dev_i32(cptr, cuda))
                assert torch.equal(again, got)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
# 602, 1030, 300 (and 514 in bf16): rows that fill 64-lane groups badly take the flat-mapped kernel; 7, 30, 50, 130:
# the last lane of a row overlaps its neighbour instead of moving a cut-off vector
@pytest.mark.parametrize("D", [1, 3, 7, 30, 50, 64, 100, 128, 130, 256, 300, 514, 602, 1030])
def test_aggregate_vs_oracle(cuda, oracle, dtype, D):
    print("aggregate D=%d %s" % (D, dtype), flush=True)
    rng = np.random.default_rng(D)
    n_dst, n_src = 517, 2000
    ptr, idx, deg = make_block(rng, n_dst, n_src, 12, hubs=[(3, 64), (4, 65), (100, 300)])
    X = torch.from_numpy(rng.standard_normal((n_src, D)).astype(np.float32)).to(cuda).to(dtype)
    run_modes(cuda, oracle, ptr, idx, deg, X, n_src, TOL[dtype])


@pytest.mark.parametrize("n_dst", [1, 2, 3, 4, 5, 1023, 4096])
@pytest.mark.parametrize("max_deg", [1, 2, 3, 9])
def test_short_row_blocks(cuda, oracle, n_dst, max_deg):
    """Blocks whose rows hold zero to a few entries (what a transposed block looks like; a block can also
    have no entries at all), with a few longer lists in between and at the very end."""
    print("short rows n_dst=%d max_deg=%d" % (n_dst, max_deg), flush=True)
    rng = np.random.default_rng(n_dst * 16 + max_deg)
    n_src = 300
    hubs = [(n_dst - 1, 40)] if n_dst >= 1023 else []
    if n_dst == 4096:
        hubs += [(8, 7), (9, 1), (10, 0), (11, 1), (2001, 33), (2002, 31)]
    ptr, idx, deg = make_block(rng, n_dst, max(n_src, n_dst), max_deg, hubs=hubs)
    for dtype, D in ((torch.float32, 128), (torch.float32, 50), (torch.bfloat16, 256), (torch.bfloat16, 602)):
        X = torch.from_numpy(rng.standard_normal((max(n_src, n_dst), D)).astype(np.float32)).to(cuda).to(dtype)
        run_modes(cuda, oracle, ptr, idx, deg, X, max(n_src, n_dst), TOL[dtype])


def test_long_rows_and_what_the_caller_knows_about_them(cuda, oracle):
    """Rows beyond 128 entries are summed by a second launch (a workgroup per row).  Rows right at that
    limit, hubs of thousands of entries next to each other and at the very end; and every form of the
    caller's knowledge about the longest row -- none, a host bound, the device value that block_transpose
    writes, and deliberately wrong values of both -- gives the same sums (the knowledge is for speed only)."""
    import fastgl
    rng = np.random.default_rng(77)
    n_dst, n_src = 3001, 5000
    hubs = [(0, 5000), (1, 129), (2, 128), (3, 127), (4, 2500), (5, 131), (1500, 640), (1501, 1), (1502, 0), (3000, 900)]
    ptr, idx, deg = make_block(rng, n_dst, n_src, 6, hubs=hubs)
    rn = np.maximum(deg, 1).astype(np.int32)
    cn = np.maximum(np.bincount(idx, minlength=n_src), 1).astype(np.int32)
    d_ptr, d_idx, d_rn, d_cn = dev_i32(ptr, cuda), dev_i32(idx, cuda), dev_i32(rn, cuda), dev_i32(cn, cuda)
    true_max = int(deg.max())
    knowledge = [None, true_max, 4, 10 ** 9, dev_i32([true_max], cuda), dev_i32([7], cuda), dev_i32([0], cuda)]
    for dtype, D in ((torch.float32, 128), (torch.float32, 20), (torch.float32, 602), (torch.bfloat16, 256), (torch.bfloat16, 31)):
        print("long rows D=%d %s" % (D, dtype), flush=True)
        X = torch.from_numpy(rng.standard_normal((n_src, D)).astype(np.float32)).to(cuda).to(dtype)
        X_ref = X.float().cpu().numpy()
        for mode in ("sum", "mean", "gcn", "colmean"):
            want = oracle.aggregate(ptr, idx, X_ref, mode, 1, rn, cn)
            for know in knowledge:
                got = fastgl.aggregate(d_ptr, d_idx, X, mode=mode, zero_policy="zeros", row_norm=d_rn, col_norm=d_cn,
                                       longest_row=know)
                err = rel_err(got.float().cpu().numpy(), want)
                assert err < TOL[dtype], (D, dtype, mode, know if not isinstance(know, torch.Tensor) else int(know), err)


def test_block_transpose_reports_its_longest_row(cuda):
    import fastgl
    rng = np.random.default_rng(5)
    for n_dst, n_src, hub_count in ((400, 50, 0), (4000, 300, 700), (2000, 2000, 33), (2000, 2000, 32)):
        deg = rng.integers(0, 3, size=n_dst)
        ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
        idx = rng.integers(1, n_src, size=ptr[-1]).astype(np.int32)  # column 0 is filled below
        rows = rng.choice(np.nonzero(deg)[0], size=hub_count, replace=False) if hub_count else []
        for r in rows:
            idx[ptr[r]] = 0  # hub_count rows mention column 0 once
        counts = np.bincount(idx, minlength=n_src)
        t_ptr, _ = fastgl.block_transpose(dev_i32(ptr, cuda), dev_i32(idx, cuda), n_dst, n_src)
        reported = int(t_ptr.fgl_longest_row)
        longest = int(counts.max())
        print("transpose n_dst=%d longest=%d reported=%d" % (n_dst, longest, reported), flush=True)
        # exact beyond 32 entries; below that only "not above 32" is promised
        assert (reported == longest) if longest > 32 else (reported <= 32)


def test_transpose_of_a_large_block(cuda):
    """Blocks of 2M+ entries count with several counters per column: offsets, the permutation of the entries
    and the reported longest row against device-side recomputation (the transposition is the same multiset of
    (row, column) pairs, t_edge names the entry each one came from)."""
    import fastgl
    gen = torch.Generator(device=cuda).manual_seed(9)
    n_dst, n_src, k = 150_000, 400_000, 15
    ptr = (torch.arange(n_dst + 1, device=cuda, dtype=torch.int32) * k)
    idx = torch.randint(0, n_src, (n_dst * k,), generator=gen, device=cuda, dtype=torch.int32)
    hub = torch.randint(0, n_dst * k, (60_000,), generator=gen, device=cuda)
    idx[hub[:40_000]] = 7          # one column mentioned ~40 K times
    idx[hub[40_000:]] = 123_456    # another ~20 K times
    print("large transpose: %d entries" % idx.numel(), flush=True)
    t_ptr, t_idx, t_edge = fastgl.block_transpose(ptr, idx, n_dst, n_src, edge_ids=True)
    counts = torch.bincount(idx.long(), minlength=n_src)
    want_ptr = torch.cat([torch.zeros(1, dtype=torch.long, device=cuda), counts.cumsum(0)])
    assert torch.equal(t_ptr.long(), want_ptr)
    assert int(t_ptr.fgl_longest_row) == int(counts.max())
    assert torch.equal(torch.sort(t_edge.long()).values, torch.arange(idx.numel(), device=cuda))   # a permutation
    col_of_t = torch.repeat_interleave(torch.arange(n_src, device=cuda), counts)
    assert torch.equal(idx.long()[t_edge.long()], col_of_t)                    # every entry sits in its column's list
    assert torch.equal((t_edge // k).int(), t_idx)                             # and names the row it came from


def test_aggregate_golden(cuda):
    import fastgl
    print("aggregate golden", flush=True)
    g = np.load(os.path.join(GOLDEN_DIR, "aggregate_small.npz"))
    d = lambda k: dev_i32(g[k], cuda)
    X = torch.from_numpy(g["X"]).to(cuda)
    for mode in ("sum", "mean", "gcn", "colmean"):
        for pol_name, pol in (("self", 0), ("zeros", 1)):
            got = fastgl.aggregate(d("ptr"), d("idx"), X, mode=mode, zero_policy=pol_name, row_norm=d("row_norm"), col_norm=d("col_norm"))
            assert rel_err(got.cpu().numpy(), g["%s_%d" % (mode, pol)]) < 1e-5


def test_strided_rows_and_narrow_vectors(cuda, oracle):
    """a column slice of a wider table: row stride != row length, base not 16-byte aligned"""
    import fastgl
    print("aggregate strided", flush=True)
    rng = np.random.default_rng(8)
    n_dst, n_src = 200, 900
    ptr, idx, deg = make_block(rng, n_dst, n_src, 10)
    wide = torch.from_numpy(rng.standard_normal((n_src, 70)).astype(np.float32)).to(cuda)
    for lo, hi in ((0, 64), (1, 65), (2, 66), (3, 35)):
        X = wide[:, lo:hi]
        got = fastgl.aggregate(dev_i32(ptr, cuda), dev_i32(idx, cuda), X, mode="mean", zero_policy="zeros")
        want = oracle.aggregate(ptr, idx, X.cpu().numpy(), "mean", 1)
        assert rel_err(got.cpu().numpy(), want) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_strided_wide_rows(cuda, oracle, dtype):
    """Column slices of a 700-column table: wide rows (flat-mapped kernel) whose stride differs from their
    length, even and odd lengths, bases that are only 4-byte (fp32) or 2-byte (bf16) aligned; one block with
    rows of several hundred entries, so that the long-row launch sees the same layouts."""
    import fastgl
    print("aggregate strided wide %s" % dtype, flush=True)
    rng = np.random.default_rng(9)
    n_dst, n_src = 150, 700
    ptr, idx, deg = make_block(rng, n_dst, n_src, 10, hubs=[(5, 200), (6, 129)])
    wide = torch.from_numpy(rng.standard_normal((n_src, 700)).astype(np.float32)).to(cuda).to(dtype)
    for lo, hi in ((0, 602), (1, 603), (2, 603), (3, 700), (0, 301), (5, 38), (4, 37)):
        X = wide[:, lo:hi]
        for mode in ("sum", "mean"):
            got = fastgl.aggregate(dev_i32(ptr, cuda), dev_i32(idx, cuda), X, mode=mode, zero_policy="self")
            want = oracle.aggregate(ptr, idx, X.float().cpu().numpy(), mode, 0)
            assert rel_err(got.float().cpu().numpy(), want) < TOL[dtype], (lo, hi, mode)


def test_closed_forms_on_device(cuda):
    import fastgl
    print("aggregate closed forms", flush=True)
    rng = np.random.default_rng(2)
    ptr, idx, deg = make_block(rng, 300, 300, 20)
    ones = torch.ones(300, 128, device=cuda)
    s = fastgl.aggregate(dev_i32(ptr, cuda), dev_i32(idx, cuda), ones, mode="sum", zero_policy="zeros").cpu().numpy()
    assert np.array_equal(s, np.repeat(deg[:, None], 128, 1).astype(np.float32))  # small integers: exact in fp32
    m = fastgl.aggregate(dev_i32(ptr, cuda), dev_i32(idx, cuda), ones, mode="mean", zero_policy="zeros").cpu().numpy()
    assert np.allclose(m[deg > 0], 1.0, rtol=1e-6) and (m[deg == 0] == 0).all()


def test_block_transpose_and_backward(cuda, oracle):
    """d_x = A^T d_out computed by gathering over the transposed block == oracle on the oracle's
    (stable) transpose; the device transpose holds the same lists up to order within a column."""
    import fastgl
    print("transpose + backward", flush=True)
    rng = np.random.default_rng(21)
    n_dst, n_src, D = 3000, 9000, 128
    ptr, idx, deg = make_block(rng, n_dst, n_src, 15, hubs=[(0, 500)])
    idx[: 2500] = 17  # a hub column
    t_ptr, t_idx = fastgl.block_transpose(dev_i32(ptr, cuda), dev_i32(idx, cuda), n_dst, n_src)
    w_ptr, w_idx = oracle.transpose(ptr, idx, n_src)
    g_ptr, g_idx = t_ptr.cpu().numpy(), t_idx.cpu().numpy()
    assert np.array_equal(g_ptr, w_ptr)
    seg = np.repeat(np.arange(n_src), np.diff(w_ptr))
    assert np.array_equal(g_idx[np.lexsort((g_idx, seg))], w_idx)             # same lists, sorted within columns
    rn = np.maximum(deg, 1).astype(np.int32)
    cn = np.maximum(np.bincount(idx, minlength=n_src), 1).astype(np.int32)
    d_out = rng.standard_normal((n_dst, D)).astype(np.float32)
    for mode, row_norm, col_norm in (("sum", None, None), ("colmean", None, rn), ("gcn", cn, rn)):
        got = fastgl.aggregate(t_ptr, t_idx, torch.from_numpy(d_out).to(cuda), mode=mode, zero_policy="zeros",
                               row_norm=None if row_norm is None else dev_i32(row_norm, cuda),
                               col_norm=None if col_norm is None else dev_i32(col_norm, cuda))
        want = oracle.aggregate(w_ptr, w_idx, d_out, mode, 1, row_norm, col_norm)
        assert rel_err(got.cpu().numpy(), want) < 1e-5, mode


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128, 256, 602])
def test_microbench_shape(cuda, oracle, dtype, D):
    """8192 destination rows x exactly 25 neighbours out of 200K source rows, sum and mean,
    forward and backward"""
    import fastgl
    print("microbench shape D=%d %s" % (D, dtype), flush=True)
    g = torch.Generator().manual_seed(0)
    n_dst, n_src, k = 8192, 200_000, 25
    ptr = (torch.arange(n_dst + 1, dtype=torch.int32) * k)
    idx = torch.randint(0, n_src, (n_dst * k,), generator=g, dtype=torch.int32)
    X = torch.randn(n_src, D, generator=g).to(dtype)
    dO = torch.randn(n_dst, D, generator=g).to(dtype)
    d_ptr, d_idx, Xd, dOd = ptr.to(cuda), idx.to(cuda), X.to(cuda), dO.to(cuda)
    t_ptr, t_idx = fastgl.block_transpose(d_ptr, d_idx, n_dst, n_src)
    w_tptr, w_tidx = oracle.transpose(ptr.numpy(), idx.numpy(), n_src)
    deg = np.full(n_dst, k, np.int32)
    for mode, bmode in (("sum", "sum"), ("mean", "colmean")):
        fwd = fastgl.aggregate(d_ptr, d_idx, Xd, mode=mode, zero_policy="zeros")
        want = oracle.aggregate(ptr.numpy(), idx.numpy(), X.float().numpy(), mode, 1)
        assert rel_err(fwd.float().cpu().numpy(), want) < TOL[dtype]
        bwd = fastgl.aggregate(t_ptr, t_idx, dOd, mode=bmode, zero_policy="zeros", col_norm=dev_i32(deg, cuda))
        wantb = oracle.aggregate(w_tptr, w_tidx, dO.float().numpy(), bmode, 1, None, deg)
        assert rel_err(bwd.float().cpu().numpy(), wantb) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,unit", [(1, 64), (8, 8), (4, 32), (3, 5), (2, 301)])
def test_edge_weighted_forward_backward(cuda, oracle, dtype, H, unit):
    """GAT aggregation (per-edge, per-head weights) forward, and backward over the transposed block"""
    import fastgl
    print("aggregate edge mode H=%d unit=%d %s" % (H, unit, dtype), flush=True)
    rng = np.random.default_rng(H * 100 + unit)
    n_dst, n_src, D = 400, 1500, H * unit
    ptr, idx, deg = make_block(rng, n_dst, n_src, 10, hubs=[(7, 130), (8, 400)])
    idx[rng.choice(idx.size, size=350, replace=False)] = 3  # a hub column: a long row of the transposed block
    X = torch.from_numpy(rng.standard_normal((n_src, D)).astype(np.float32)).to(cuda).to(dtype)
    alpha = rng.random((ptr[-1], H)).astype(np.float32)
    d_ptr, d_idx, d_alpha = dev_i32(ptr, cuda), dev_i32(idx, cuda), torch.from_numpy(alpha).to(cuda)
    (out,) = fastgl.forward_gat(d_ptr, d_alpha, d_idx, X, 10, n_dst, H)  # (a bound that the hubs exceed: speed only)
    want = oracle.aggregate_edge(ptr, idx, X.float().cpu().numpy(), alpha, zero_policy=0)
    assert rel_err(out.float().cpu().numpy(), want) < TOL[dtype]
    # nothing known about the rows: the two hub rows go through the long-row launch
    out2 = fastgl.aggregate(d_ptr, d_idx, X, mode="edge", zero_policy="self", edge_weight=d_alpha, n_heads=H)
    assert rel_err(out2.float().cpu().numpy(), want) < TOL[dtype]
    dO = torch.from_numpy(rng.standard_normal((n_dst, D)).astype(np.float32)).to(cuda).to(dtype)
    (d_x,) = fastgl.backward_gat(d_ptr, d_alpha, d_idx, dO, n_src, H)
    t_ptr, t_idx, t_edge = oracle.transpose_with_edges(ptr, idx, n_src)
    wantb = oracle.aggregate_edge(t_ptr, t_idx, dO.float().cpu().numpy(), alpha, 1, edge_index=t_edge)
    assert rel_err(d_x.float().cpu().numpy(), wantb) < TOL[dtype]
    # the device transpose names the right edge for every transposed entry
    g_ptr, g_idx, g_edge = fastgl.block_transpose(d_ptr, d_idx, n_dst, n_src, edge_ids=True)
    g_edge = g_edge.cpu().numpy()
    assert np.array_equal(np.sort(g_edge), np.arange(ptr[-1]))
    assert np.array_equal(idx[g_edge], np.repeat(np.arange(n_src), np.diff(g_ptr.cpu().numpy())))
    row_of_edge = np.repeat(np.arange(n_dst), deg)
    assert np.array_equal(row_of_edge[g_edge], g_idx.cpu().numpy())


@pytest.mark.parametrize("n_dst,n_src,max_deg", [(3000, 9000, 15), (1, 5, 3), (50, 1, 4), (200, 70000, 2)])
def test_sorted_transpose_is_the_stable_transpose(cuda, oracle, n_dst, n_src, max_deg):
    """sorted_rows=True: offsets, row lists and edge ids equal the oracle's stable counting sort exactly,
    run after run (the default variant matches only up to the order inside a column)."""
    import fastgl
    print("sorted transpose %d %d" % (n_dst, n_src), flush=True)
    rng = np.random.default_rng(n_dst + n_src)
    ptr, idx, deg = make_block(rng, n_dst, n_src, max_deg, hubs=[(0, 700)] if n_dst > 100 else ())
    if n_dst > 100:
        idx[:2000] = 3  # a hub column
    w_ptr, w_idx, w_edge = oracle.transpose_with_edges(ptr, idx, n_src)
    for _ in range(2):
        t_ptr, t_idx, t_edge = fastgl.block_transpose(dev_i32(ptr, cuda), dev_i32(idx, cuda), n_dst, n_src, edge_ids=True,
                                                      sorted_rows=True)
        assert np.array_equal(t_ptr.cpu().numpy(), w_ptr)
        assert np.array_equal(t_idx.cpu().numpy(), w_idx)
        assert np.array_equal(t_edge.cpu().numpy(), w_edge)
    t_ptr, t_idx = fastgl.block_transpose(dev_i32(ptr, cuda), dev_i32(idx, cuda), n_dst, n_src, sorted_rows=True)
    assert np.array_equal(t_idx.cpu().numpy(), w_idx)


def test_deterministic_sampler_gives_bitwise_reproducible_gradients(cuda, oracle, small_graph):
    import fastgl
    print("deterministic backward", flush=True)
    indptr, indices = small_graph
    ptr, idx = torch.from_numpy(indptr).to(cuda), dev_i32(indices, cuda)
    seeds = dev_i32(np.argsort(-np.diff(indptr))[:2048], cuda)  # hub seeds: long transposed lists
    grads = []
    for _ in range(2):
        sampler = fastgl.FusedMapSampler([10, 10], rng_seed=1, deterministic=True).set_graph(ptr, idx)
        _, _, blocks = sampler.sample_blocks(None, seeds)
        b = blocks[0]
        g = torch.randn(b.num_dst_nodes(), 64, device=cuda, generator=torch.Generator(device=cuda).manual_seed(5))
        t_ptr, t_idx = b.transposed()
        grads.append(fastgl.aggregate(t_ptr, t_idx, g, mode="sum", zero_policy="zeros"))
    assert torch.equal(grads[0], grads[1])


def test_random_blocks_all_modes_against_the_oracle(cuda, oracle):
    """Thirty seeded random blocks -- row counts, row lengths from empty to beyond the long-row limit, feature
    lengths from 1 to 700 (whole and partial vectors, one to several column slices), both element types, all
    modes and both policies for empty rows, forward and over the transposed block."""
    import fastgl
    rng = np.random.default_rng(2024)
    for case in range(30):
        n_dst = int(rng.integers(1, 3000))
        n_src = max(n_dst, int(rng.integers(1, 6000)))
        max_deg = int(rng.choice([0, 1, 2, 5, 20, 70]))
        hubs = [(int(rng.integers(0, n_dst)), int(rng.integers(100, 900))) for _ in range(int(rng.integers(0, 4)))]
        ptr, idx, deg = make_block(rng, n_dst, n_src, max_deg, hubs=hubs)
        D = int(rng.choice([1, 2, 5, 8, 31, 32, 64, 100, 128, 200, 256, 602, 700]))
        dtype = torch.float32 if case % 3 else torch.bfloat16
        print("random block %d: %d x %d, %d entries, D=%d %s" % (case, n_dst, n_src, idx.size, D, dtype), flush=True)
        X = torch.from_numpy(rng.standard_normal((n_src, D)).astype(np.float32)).to(cuda).to(dtype)
        run_modes(cuda, oracle, ptr, idx, deg, X, n_src, TOL[dtype])
        # the transposed block: every source row sums the destination rows it feeds
        G = torch.from_numpy(rng.standard_normal((n_dst, D)).astype(np.float32)).to(cuda).to(dtype)
        t_ptr, t_idx = fastgl.block_transpose(dev_i32(ptr, cuda), dev_i32(idx, cuda), n_dst, n_src)
        got = fastgl.aggregate(t_ptr, t_idx, G, mode="sum", zero_policy="zeros")
        want_ptr, want_idx = oracle.transpose(ptr, idx, n_src)
        want = oracle.aggregate(want_ptr, want_idx, G.float().cpu().numpy(), "sum", 1)
        assert np.array_equal(t_ptr.cpu().numpy(), want_ptr)
        assert rel_err(got.float().cpu().numpy(), want) < TOL[dtype], case


@pytest.mark.parametrize("H", [1, 3, 4, 8])
def test_edge_softmax_vs_oracle_and_torch(cuda, oracle, H):
    """GAT attention coefficients in one launch against the fp64 oracle and against the plain torch fp32
    restatement (gather, leaky_relu, scatter-max, exp, scatter-add, divide); tolerance 1e-5 relative to the
    largest coefficient (fp32 exp and division).  Rows without entries, one-entry rows (coefficient 1), a row
    of several hundred entries, scores large enough that exp would overflow without the maximum subtracted."""
    import fastgl
    print("edge_softmax H=%d" % H, flush=True)
    rng = np.random.default_rng(40 + H)
    n_dst, n_src = 700, 2500
    ptr, idx, deg = make_block(rng, n_dst, n_src, 12, hubs=[(5, 300), (6, 1), (7, 0)])
    el = (rng.standard_normal((n_src, H)) * 3).astype(np.float32)
    er = (rng.standard_normal((n_dst, H)) * 3).astype(np.float32)
    el[:10] += 95.0  # exp(95) overflows fp32
    d_ptr, d_idx = dev_i32(ptr, cuda), dev_i32(idx, cuda)
    d_el, d_er = torch.from_numpy(el).to(cuda), torch.from_numpy(er).to(cuda)
    got = fastgl.edge_softmax(d_ptr, d_idx, d_el, d_er, 0.2)
    want = oracle.edge_softmax(ptr, idx, el, er, 0.2)
    assert tuple(got.shape) == want.shape and got.dtype == torch.float32
    assert rel_err(got.cpu().numpy(), want) < 1e-5
    assert torch.isfinite(got).all()
    one = ptr[6]
    assert np.array_equal(got[one].cpu().numpy(), np.ones(H, np.float32))
    dst = torch.repeat_interleave(torch.arange(n_dst, device=cuda), torch.from_numpy(deg).to(cuda)).int()
    e = torch.nn.functional.leaky_relu(d_el.index_select(0, d_idx.long()) + d_er.index_select(0, dst.long()), 0.2)
    ref = fastgl.edge_softmax_torch(d_ptr, dst, e, n_dst)
    assert rel_err(got.cpu().numpy(), ref.double().cpu().numpy()) < 1e-5
    # an empty block
    empty = fastgl.edge_softmax(dev_i32(np.zeros(4, np.int32), cuda), dev_i32(np.zeros(0, np.int32), cuda), d_el, d_er[:3], 0.2)
    assert tuple(empty.shape) == (0, H)


@pytest.mark.parametrize("dtype,D", [(torch.float32, 24), (torch.float32, 64), (torch.float32, 100), (torch.bfloat16, 64),
                                     (torch.bfloat16, 50), (torch.bfloat16, 128), (torch.bfloat16, 256)])
@pytest.mark.parametrize("bound", [6, 12, 25, 64, 100])
def test_few_rows_of_long_lists(cuda, oracle, dtype, D, bound):
    """A block of a few rows whose lists are known to be long (the caller names a bound, as the sampler names its
    fanout): several lane groups share a row and their partial sums are added across lanes.  Rows of every
    length from none to the bound, row counts that do not fill a workgroup, all modes and both policies."""
    import fastgl
    print("few long rows D=%d %s bound=%d" % (D, dtype, bound), flush=True)
    rng = np.random.default_rng(D * 1000 + bound)
    for n_dst in (1, 7, 333, 4000):
        n_src = 5000
        deg = rng.integers(0, bound + 1, size=n_dst)
        deg[rng.integers(0, n_dst)] = bound
        ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
        idx = rng.integers(0, n_src, size=ptr[-1]).astype(np.int32)
        X = torch.from_numpy(rng.standard_normal((n_src, D)).astype(np.float32)).to(cuda).to(dtype)
        X_ref = X.float().cpu().numpy()
        rn = np.maximum(deg, 1).astype(np.int32)
        cn = np.maximum(np.bincount(idx, minlength=n_src), 1).astype(np.int32)
        d_ptr, d_idx, d_rn, d_cn = dev_i32(ptr, cuda), dev_i32(idx, cuda), dev_i32(rn, cuda), dev_i32(cn, cuda)
        for mode in ("sum", "mean", "gcn", "colmean"):
            for pol_name, pol in (("self", 0), ("zeros", 1)):
                want = oracle.aggregate(ptr, idx, X_ref, mode, pol, rn, cn)
                got = fastgl.aggregate(d_ptr, d_idx, X, mode=mode, zero_policy=pol_name, row_norm=d_rn, col_norm=d_cn,
                                       longest_row=bound)
                err = rel_err(got.float().cpu().numpy(), want)
                assert err < TOL[dtype], (n_dst, mode, pol_name, err)
                # the same sums bit for bit on a second run (the cross-lane additions have a fixed order)
                again = fastgl.aggregate(d_ptr, d_idx, X, mode=mode, zero_policy=pol_name, row_norm=d_rn, col_norm=d_cn,
                                         longest_row=bound)
                assert torch.equal(got, again)


@pytest.mark.parametrize("dtype,D", [(torch.float32, 64), (torch.float32, 128), (torch.float32, 256), (torch.float32, 602),
                                     (torch.bfloat16, 64), (torch.bfloat16, 128), (torch.bfloat16, 602), (torch.bfloat16, 31)])
def test_many_rows_of_short_lists(cuda, oracle, dtype, D):
    """What a transposed block looks like: thousands of rows with one entry on average (many with none), which a lane
    group takes several at a time; with a few lists long enough to span the group's chunks, hubs that go to the
    long-row launch, and row counts that leave the last bundle incomplete."""
    import fastgl
    print("many short rows D=%d %s" % (D, dtype), flush=True)
    rng = np.random.default_rng(D)
    for n_dst, hubs in ((1024, []), (4099, [(5, 70), (6, 9), (7, 140), (2000, 33), (4098, 600)]), (6001, [(6000, 17), (0, 129)])):
        n_src = 3000
        deg = rng.poisson(1.0, size=n_dst)
        for r, d in hubs:
            deg[r] = d
        deg[0] = 0 if not hubs else deg[0]
        assert deg.sum() <= 2 * n_dst
        ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
        idx = rng.integers(0, n_src, size=ptr[-1]).astype(np.int32)
        X = torch.from_numpy(rng.standard_normal((max(n_src, n_dst), D)).astype(np.float32)).to(cuda).to(dtype)
        run_modes(cuda, oracle, ptr, idx, deg, X, max(n_src, n_dst), TOL[dtype])


def test_batched_transpose_matches_the_single_one(cuda, oracle):
    """Several blocks transposed by one batched call: offsets equal the oracle's, every transposed row holds the same set of
    entries (lists are unordered), edge ids name the right entries, the longest row is reported; blocks without entries or
    columns, and more blocks than one batch takes."""
    import fastgl
    print("batched transpose", flush=True)
    rng = np.random.default_rng(31)
    shapes = [(300, 900, 6), (1, 1, 3), (50, 7, 0), (2500, 40000, 12), (4000, 500, 3), (0, 10, 0), (700, 700, 40), (33, 5000, 2),
              (1200, 10, 5), (9, 9, 9)]
    host, dev_blocks = [], []
    for n_dst, n_src, max_deg in shapes:
        deg = rng.integers(0, max_deg + 1, size=n_dst)
        ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
        idx = rng.integers(0, n_src, size=ptr[-1]).astype(np.int32)
        host.append((ptr, idx, n_dst, n_src))
        dev_blocks.append((dev_i32(ptr, cuda), dev_i32(idx, cuda), n_dst, n_src))
    got = fastgl.block_transpose_batch(dev_blocks, edge_ids=True)
    assert len(got) == len(shapes)
    for (ptr, idx, n_dst, n_src), (t_ptr, t_idx, t_edge) in zip(host, got):
        w_ptr, w_idx = oracle.transpose(ptr, idx, n_src)
        g_ptr, g_idx, g_edge = t_ptr.cpu().numpy(), t_idx.cpu().numpy(), t_edge.cpu().numpy()
        assert np.array_equal(g_ptr, w_ptr)
        # same entries per transposed row, in any order
        row_of = np.repeat(np.arange(n_src), np.diff(w_ptr))
        assert g_idx.size == w_idx.size
        assert np.array_equal(np.sort(row_of * (n_dst + 1) + g_idx), np.sort(row_of * (n_dst + 1) + w_idx))
        assert np.array_equal(np.sort(g_edge), np.arange(ptr[-1]))
        assert np.array_equal(idx[g_edge], row_of)
        assert np.array_equal(np.repeat(np.arange(n_dst), np.diff(ptr))[g_edge], g_idx)
        longest = int(np.diff(w_ptr).max()) if n_src else 0
        reported = int(t_ptr.fgl_longest_row)
        assert (reported == longest) if longest > 32 else (reported <= 32)
    # through Block objects: transposed() afterwards returns what the batch call built
    blocks = [fastgl.Block(p, i, n_src, n_dst) for p, i, n_dst, n_src in dev_blocks[:4]]
    fastgl.transpose_blocks(blocks)
    for b, (ptr, idx, n_dst, n_src) in zip(blocks, host):
        assert b._transposed is not None
        t_ptr, t_idx = b.transposed()
        assert np.array_equal(t_ptr.cpu().numpy(), oracle.transpose(ptr, idx, n_src)[0])
