"""Pins the oracle's generator and sampler (CPU only)."""
import itertools

import numpy as np
import pytest
from scipy import stats

# Random123 known-answer vectors for philox4x32-10 (counter, key) -> output
KAT = [
    ([0x00000000] * 4, [0x00000000] * 2, [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
    ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
    ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
     [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
]


@pytest.mark.parametrize("ctr,key,want", KAT)
def test_philox_known_answers(oracle, ctr, key, want):
    assert [int(x) for x in oracle.philox4x32_10(ctr, key)] == want


def _ring_graph(n, deg):
    """node v has in-neighbours v+1 .. v+deg (mod n), listed in that order"""
    indptr = np.arange(0, (n + 1) * deg, deg, dtype=np.int64)
    indices = ((np.arange(n)[:, None] + np.arange(1, deg + 1)[None, :]) % n).astype(np.int32).ravel()
    return indptr, indices


@pytest.mark.parametrize("ptr_dtype", [np.int32, np.int64])
def test_full_neighbourhood_is_the_csr_row(oracle, small_graph, ptr_dtype):
    indptr, indices = small_graph
    indptr = indptr.astype(ptr_dtype)
    rng = np.random.default_rng(1)
    seeds = rng.permutation(indptr.size - 1)[:2000].astype(np.int32)
    fanout = int(np.diff(indptr)[seeds].max())  # fanout >= every degree: closed form
    src, dst, ptr = oracle.sample_node(indptr, indices, seeds, fanout)
    deg = np.diff(indptr)[seeds]
    assert np.array_equal(ptr, np.concatenate([[0], np.cumsum(deg)]).astype(np.int32))
    want_src = np.concatenate([indices[indptr[s]:indptr[s + 1]] for s in seeds])
    assert np.array_equal(src, want_src)
    assert np.array_equal(dst, np.repeat(seeds, deg))


def test_random_case_validity(oracle, small_graph):
    indptr, indices = small_graph
    rng = np.random.default_rng(2)
    seeds = rng.permutation(indptr.size - 1)[:4096].astype(np.int32)
    for fanout in (1, 5, 15, 64):
        src, dst, ptr = oracle.sample_node(indptr, indices, seeds, fanout, rng_seed=7, stream_id=3)
        deg = np.diff(indptr)[seeds]
        k = np.minimum(deg, fanout)
        assert np.array_equal(np.diff(ptr), k)           # exactly min(fanout, deg) per seed
        assert np.array_equal(dst, np.repeat(seeds, k))  # contiguous, in seed order
        for i, s in enumerate(seeds[:512]):
            row = indices[indptr[s]:indptr[s + 1]]
            got = src[ptr[i]:ptr[i + 1]]
            assert np.isin(got, row).all()               # every edge exists
            assert np.unique(got).size == got.size       # without replacement (rows are duplicate-free)


def test_streams_differ_and_repeat(oracle, small_graph):
    indptr, indices = small_graph
    seeds = np.arange(0, 3000, dtype=np.int32)
    a = oracle.sample_node(indptr, indices, seeds, 5, rng_seed=1, stream_id=0)[0]
    b = oracle.sample_node(indptr, indices, seeds, 5, rng_seed=1, stream_id=0)[0]
    c = oracle.sample_node(indptr, indices, seeds, 5, rng_seed=1, stream_id=1)[0]
    d = oracle.sample_node(indptr, indices, seeds, 5, rng_seed=2, stream_id=0)[0]
    assert np.array_equal(a, b)
    assert not np.array_equal(a, c) and not np.array_equal(a, d)


@pytest.mark.parametrize("deg,fanout", [(16, 5), (1000, 15), (17, 16), (40, 1)])
def test_uniform_inclusion_chi_square(oracle, deg, fanout):
    """Every neighbour must be picked with probability fanout/deg.  Inclusion counts over
    n seeds are NOT independent multinomial cells (each seed contributes exactly `fanout`
    picks), so the Pearson statistic is rescaled by (deg-1)/(deg-fanout)... for sampling
    without replacement sum((O-E)^2/E) * (deg-1)/(deg-fanout) ~ chi2(deg-1)."""
    n = 20000
    indptr, indices = _ring_graph(n, deg)
    seeds = np.random.default_rng(deg).permutation(n).astype(np.int32)
    src, dst, ptr = oracle.sample_node(indptr, indices, seeds, fanout, rng_seed=123, stream_id=9)
    offs = (src.astype(np.int64) - dst - 1) % n          # position of the pick inside the row
    counts = np.bincount(offs, minlength=deg)
    assert counts.sum() == n * fanout
    expect = n * fanout / deg
    stat = ((counts - expect) ** 2 / expect).sum() * (deg - 1) / (deg - fanout)
    p = stats.chi2.sf(stat, deg - 1)
    assert p > 1e-4, (stat, p)


def test_uniform_over_subsets_exhaustive(oracle):
    """deg 6, fanout 3: all 20 subsets must be equally likely (chi-square over subsets)."""
    deg, k, n = 6, 3, 40000
    subsets = {s: i for i, s in enumerate(itertools.combinations(range(deg), k))}
    counts = np.zeros(len(subsets))
    for pos in range(n):
        sel = oracle.floyd_subset(deg, k, 99, 0, pos)
        assert len(set(sel.tolist())) == k and sel.min() >= 0 and sel.max() < deg
        counts[subsets[tuple(sorted(sel.tolist()))]] += 1
    stat = ((counts - n / 20) ** 2 / (n / 20)).sum()
    assert stats.chi2.sf(stat, 19) > 1e-4


def test_pair_inclusion_is_uniform(oracle):
    """second-order check: every unordered pair is co-selected with probability k(k-1)/(d(d-1))."""
    deg, k, n = 12, 4, 30000
    pair = np.zeros((deg, deg))
    for pos in range(n):
        sel = sorted(oracle.floyd_subset(deg, k, 5, 2, pos).tolist())
        for a, b in itertools.combinations(sel, 2):
            pair[a, b] += 1
    got = pair[np.triu_indices(deg, 1)]
    expect = n * k * (k - 1) / (deg * (deg - 1))
    assert np.abs(got / expect - 1).max() < 0.08
