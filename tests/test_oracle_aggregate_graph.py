"""Pins the oracle's aggregation and R-MAT restatements (CPU only)."""
import numpy as np
import pytest
import scipy.sparse as sp


def _block(rng, n_dst, n_src, max_deg, zero_rows=True):
    deg = rng.integers(0 if zero_rows else 1, max_deg + 1, size=n_dst)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    indices = rng.integers(0, n_src, size=indptr[-1]).astype(np.int32)
    return indptr, indices, deg


@pytest.mark.parametrize("mode", ["sum", "mean", "gcn", "colmean"])
def test_against_scipy(oracle, mode):
    rng = np.random.default_rng(11)
    n_dst, n_src, D = 200, 700, 33
    indptr, indices, deg = _block(rng, n_dst, n_src, 9)
    X = rng.standard_normal((n_src, D)).astype(np.float32)
    A = sp.csr_matrix((np.ones(indptr[-1]), indices, indptr), shape=(n_dst, n_src))  # duplicates add up
    rn = np.maximum(deg, 1).astype(np.int32)
    cn = np.maximum(np.bincount(indices, minlength=n_src), 1).astype(np.int32)
    if mode == "sum":
        want = A @ X.astype(np.float64)
    elif mode == "mean":
        want = sp.diags(1.0 / rn) @ A @ X.astype(np.float64)
    elif mode == "gcn":
        want = sp.diags(rn ** -0.5) @ A @ sp.diags(cn ** -0.5) @ X.astype(np.float64)
    else:
        want = A @ sp.diags(1.0 / cn) @ X.astype(np.float64)
    for policy in (0, 1):
        got = oracle.aggregate(indptr, indices, X, mode, policy, rn, cn)
        w = want.copy()
        if policy == 0:
            w[deg == 0] = X[:n_dst][deg == 0]
        assert np.allclose(got, w, rtol=1e-12, atol=1e-12)
    f32 = oracle.aggregate(indptr, indices, X, mode, 1, rn, cn, out_dtype=np.float32)
    assert np.allclose(f32, want, rtol=1e-4, atol=1e-4)


def test_closed_forms(oracle):
    rng = np.random.default_rng(5)
    n_dst, n_src = 64, 64
    indptr, indices, deg = _block(rng, n_dst, n_src, 7, zero_rows=False)
    ones = np.ones((n_src, 4), np.float32)
    assert np.array_equal(oracle.aggregate(indptr, indices, ones, "sum"), np.repeat(deg[:, None], 4, 1).astype(float))
    assert np.allclose(oracle.aggregate(indptr, indices, ones, "mean"), 1.0)
    eye = np.eye(n_src, dtype=np.float32)  # one-hot features: output row = neighbour histogram
    hist = np.zeros((n_dst, n_src))
    for r in range(n_dst):
        np.add.at(hist[r], indices[indptr[r]:indptr[r + 1]], 1)
    assert np.array_equal(oracle.aggregate(indptr, indices, eye, "sum"), hist)


def test_backward_is_the_transpose(oracle):
    """<A x, y> == <x, A^T y> with A^T applied as the forward kernel on the transposed block."""
    rng = np.random.default_rng(9)
    n_dst, n_src, D = 150, 400, 16
    indptr, indices, deg = _block(rng, n_dst, n_src, 11)
    rn = np.maximum(deg, 1).astype(np.int32)
    cn = np.maximum(np.bincount(indices, minlength=n_src), 1).astype(np.int32)
    t_ptr, t_idx = oracle.transpose(indptr, indices, n_src)
    x = rng.standard_normal((n_src, D)).astype(np.float32)
    y = rng.standard_normal((n_dst, D)).astype(np.float32)
    for fwd, bwd, brn, bcn in (("sum", "sum", None, None), ("mean", "colmean", None, rn), ("gcn", "gcn", cn, rn)):
        ax = oracle.aggregate(indptr, indices, x, fwd, 1, rn, cn)
        aty = oracle.aggregate(t_ptr, t_idx, y, bwd, 1, brn, bcn)
        assert np.isclose((ax * y).sum(), (x * aty).sum(), rtol=1e-10)


def test_rmat_quadrants_and_symmetry(oracle):
    n, scale, seed = 200000, 18, 4
    keys = oracle.rmat_keys(0, n, scale, 1 << scale, seed)
    ok = keys != np.iinfo(np.int64).max
    k0 = keys[0::2][ok[0::2]]
    k1 = keys[1::2][ok[1::2]]
    v, u = k0 >> 32, k0 & 0xFFFFFFFF
    assert np.array_equal(k1 >> 32, u) and np.array_equal(k1 & 0xFFFFFFFF, v)  # the mirrored edge
    assert (u != v).all()
    # top-level quadrant of (u, v): probabilities a, b, c, d = .57 .19 .19 .05
    ub, vb = u >> (scale - 1), v >> (scale - 1)
    freq = np.array([np.mean((ub == 0) & (vb == 0)), np.mean((ub == 0) & (vb == 1)),
                     np.mean((ub == 1) & (vb == 0)), np.mean((ub == 1) & (vb == 1))])
    assert np.abs(freq - [0.57, 0.19, 0.19, 0.05]).max() < 0.01
    # levels are independent draws: second bit has the same marginals
    u2 = (u >> (scale - 2)) & 1
    assert abs(np.mean(u2) - 0.24) < 0.01
    # chunked generation equals one-shot generation
    again = np.concatenate([oracle.rmat_keys(0, 1000, scale, 1 << scale, seed), oracle.rmat_keys(1000, n - 1000, scale, 1 << scale, seed)])
    assert np.array_equal(keys, again)


def test_rmat_csr_shape(oracle, small_graph):
    indptr, indices = small_graph
    n = indptr.size - 1
    assert n == 100_000 and indptr[0] == 0 and indptr[-1] == indices.size
    assert 2_300_000 < indices.size < 2_700_000       # the ~2.5M directed edges of the small configuration
    rows = np.repeat(np.arange(n), np.diff(indptr))
    assert (rows != indices).all()                      # no self loops
    key = rows.astype(np.int64) << 32 | indices
    assert (np.diff(key) > 0).all()                     # sorted rows, no duplicate edges
    rev = indices.astype(np.int64) << 32 | rows
    assert np.array_equal(np.sort(rev), key)            # symmetric
    assert np.diff(indptr).max() > 2000                 # power-law tail


def test_edge_weighted_aggregation(oracle):
    """GAT aggregation: per head h, out[:, head-h columns] = (A o alpha_h) @ X[:, head-h columns]"""
    rng = np.random.default_rng(13)
    n_dst, n_src, H, unit = 120, 300, 3, 5
    D = H * unit
    indptr, indices, deg = _block(rng, n_dst, n_src, 8)
    X = rng.standard_normal((n_src, D)).astype(np.float32)
    alpha = rng.random((indptr[-1], H)).astype(np.float32)
    got = oracle.aggregate_edge(indptr, indices, X, alpha, zero_policy=1)
    want = np.zeros((n_dst, D))
    for h in range(H):
        A = sp.csr_matrix((alpha[:, h].astype(np.float64), indices, indptr), shape=(n_dst, n_src))
        want[:, h * unit:(h + 1) * unit] = A @ X[:, h * unit:(h + 1) * unit].astype(np.float64)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    passthrough = oracle.aggregate_edge(indptr, indices, X, alpha, zero_policy=0)
    assert np.array_equal(passthrough[deg == 0], X[:n_dst][deg == 0].astype(np.float64))
    # unit weights reduce it to the plain sum
    ones = np.ones_like(alpha)
    assert np.allclose(oracle.aggregate_edge(indptr, indices, X, ones, 1), oracle.aggregate(indptr, indices, X, "sum", 1))
    # backward = the same sum over the transposed lists, weights looked up through the edge ids
    t_ptr, t_idx, t_edge = oracle.transpose_with_edges(indptr, indices, n_src)
    assert np.array_equal(indices[t_edge], np.repeat(np.arange(n_src), np.diff(t_ptr)))
    y = rng.standard_normal((n_dst, D)).astype(np.float32)
    aty = oracle.aggregate_edge(t_ptr, t_idx, y, alpha, 1, edge_index=t_edge)
    assert np.isclose((want * y).sum(), (X * aty).sum(), rtol=1e-9)


def test_edge_softmax_pins(oracle):
    """The attention coefficients against scipy's softmax row by row and head by head, plus what the
    mathematics fixes: rows sum to one, a shift of er changes nothing where no score changes sign, equal
    scores give 1/deg, and hand values for the leaky-relu slope."""
    from scipy.special import softmax
    rng = np.random.default_rng(21)
    n_dst, n_src, H = 150, 400, 3
    indptr, indices, deg = _block(rng, n_dst, n_src, 11)
    el = rng.standard_normal((n_src, H)).astype(np.float32)
    er = rng.standard_normal((n_dst, H)).astype(np.float32)
    got = oracle.edge_softmax(indptr, indices, el, er, 0.2)
    assert got.shape == (indptr[-1], H)
    for r in range(n_dst):
        a, b = indptr[r], indptr[r + 1]
        if a == b:
            continue
        s = el[indices[a:b]].astype(np.float64) + er[r].astype(np.float64)
        s = np.where(s > 0, s, 0.2 * s)
        assert np.allclose(got[a:b], softmax(s, axis=0), rtol=1e-12, atol=1e-15)
        assert np.allclose(got[a:b].sum(0), 1.0, rtol=1e-12)
    # all scores positive: leaky_relu is the identity and a shift of er cancels in the softmax
    el_pos = np.abs(el) + 1.0
    a1 = oracle.edge_softmax(indptr, indices, el_pos, np.full((n_dst, H), 0.5, np.float32), 0.2)
    a2 = oracle.edge_softmax(indptr, indices, el_pos, np.full((n_dst, H), 3.0, np.float32), 0.2)
    assert np.allclose(a1, a2, rtol=1e-6)
    # equal scores: 1/deg
    a3 = oracle.edge_softmax(indptr, indices, np.zeros((n_src, H), np.float32), er, 0.2)
    assert np.allclose(a3, np.repeat(1.0 / np.maximum(deg, 1), deg)[:, None], rtol=1e-12)
    # by hand: one row, two entries, scores +1 and -1 with slope 0.5 -> exp(1), exp(-0.5)
    a4 = oracle.edge_softmax(np.array([0, 2], np.int32), np.array([0, 1], np.int32),
                             np.array([[1.0], [-1.0]], np.float32), np.zeros((1, 1), np.float32), 0.5)
    want = np.exp([1.0, -0.5]) / np.exp([1.0, -0.5]).sum()
    assert np.allclose(a4[:, 0], want, rtol=1e-12)
