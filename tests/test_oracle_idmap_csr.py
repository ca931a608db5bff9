"""Pins the oracle's id-map, TableSize, degree / scan and transpose restatements (CPU only)."""
import numpy as np
import pytest
import scipy.sparse as sp


def py_idmap(src, dst_unique):
    """Independent restatement with a python dict: dst ids first, new ids by first occurrence."""
    local = {}
    uniq = []
    for i, v in enumerate(dst_unique.tolist()):
        uniq.append(v)
        local.setdefault(v, i)
    out = []
    for v in src.tolist():
        if v not in local:
            local[v] = len(uniq)
            uniq.append(v)
        out.append(local[v])
    return np.array(out, dtype=np.int32), np.array(uniq, dtype=np.int32)


def test_hand_case(oracle):
    # seeds 7,3 ; edges (src->dst): 9->7, 3->7, 9->3, 5->3, 7->3
    src = np.array([9, 3, 9, 5, 7], dtype=np.int32)
    dst = np.array([7, 7, 3, 3, 3], dtype=np.int32)
    s, d, u = oracle.idmap(src, dst, np.array([7, 3], dtype=np.int32))
    assert u.tolist() == [7, 3, 9, 5]
    assert s.tolist() == [2, 1, 2, 3, 0]
    assert d.tolist() == [0, 0, 1, 1, 1]


@pytest.mark.parametrize("n_ids,n_dst,n_edges", [(50, 10, 400), (100000, 1000, 15000), (2**31 - 1, 64, 5000), (5, 5, 0)])
def test_against_dict(oracle, n_ids, n_dst, n_edges):
    rng = np.random.default_rng(n_edges)
    dst_unique = rng.choice(min(n_ids, 10**7), size=n_dst, replace=False).astype(np.int32)
    if n_ids > 10**7:
        dst_unique[0] = n_ids - 1  # largest representable id
    src = rng.integers(0, n_ids, size=n_edges).astype(np.int32)
    dst = dst_unique[rng.integers(0, n_dst, size=n_edges)] if n_edges else np.zeros(0, np.int32)
    s, d, u = oracle.idmap(src, dst, dst_unique)
    ws, wu = py_idmap(src, dst_unique)
    assert np.array_equal(s, ws) and np.array_equal(u, wu)
    # order-free invariants that characterise a correct map
    assert np.array_equal(u[:n_dst], dst_unique)
    assert np.unique(u).size == u.size
    assert set(u[n_dst:].tolist()) == set(src.tolist()) - set(dst_unique.tolist())
    assert np.array_equal(u[s], src)
    if n_edges:
        assert np.array_equal(u[d], dst)


def test_missing_dst_is_an_error(oracle):
    with pytest.raises(KeyError):
        oracle.idmap(np.array([1], np.int32), np.array([99], np.int32), np.array([0], np.int32))


def test_table_size_closed_form(oracle):
    # hand evaluation of (1 << (size_t)(1 + log2(num >> 1))) << scale
    assert oracle.table_size(40960, 2) == 131072      # log2(20480)=14.32 -> 1<<15 -> <<2
    assert oracle.table_size(491520, 2) == 1048576
    assert oracle.table_size(8110080, 2) == 16777216
    for num in [2, 3, 4, 5, 7, 8, 9, 1000, 1024, 1025, 2**20 - 1, 2**20, 2**33 + 5]:
        for scale in (0, 1, 2):
            assert oracle.table_size(num, scale) == (1 << (num.bit_length() - 1)) << scale


def test_cal_deg_and_exclusive_sum(oracle):
    rng = np.random.default_rng(0)
    ids = rng.integers(0, 1000, size=20000).astype(np.int32)
    deg = oracle.cal_deg(ids, 1000)
    assert np.array_equal(deg, np.bincount(ids, minlength=1000))
    ex = oracle.exclusive_sum(deg)
    assert np.array_equal(ex, np.concatenate([[0], np.cumsum(deg)]))
    assert oracle.exclusive_sum(np.zeros(0, np.int32)).tolist() == [0]


def test_transpose_matches_scipy(oracle):
    rng = np.random.default_rng(3)
    n_rows, n_cols = 300, 500
    deg = rng.integers(0, 12, size=n_rows)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    indices = rng.integers(0, n_cols, size=indptr[-1]).astype(np.int32)
    t_ptr, t_idx = oracle.transpose(indptr, indices, n_cols)
    # scipy keeps duplicates when converting csr -> csc and orders rows ascending within a column
    m = sp.csr_matrix((np.arange(1, indptr[-1] + 1), indices, indptr), shape=(n_rows, n_cols)).tocsc()
    assert np.array_equal(t_ptr, m.indptr)
    assert np.array_equal(t_idx, m.indices)


def test_parallel_idmap_equals_the_sequential_one(oracle):
    """The multi-threaded variant that the benchmark's CPU baseline times gives exactly the output of the
    sequential oracle (which the python-dict restatement and the invariants above pin)."""
    rng = np.random.default_rng(21)
    for trial in range(25):
        n_dst = int(rng.integers(0, 400))
        n_edges = int(rng.integers(0, 30000))
        pool = int(rng.integers(1, 5000))
        dst_unique = rng.permutation(50000)[:n_dst].astype(np.int32)
        if trial % 4 == 0 and n_dst > 5:
            dst_unique[5] = dst_unique[1]  # a repeated destination keeps its first position
        src = rng.integers(0, pool, size=n_edges).astype(np.int32)
        want_src, _, want_uniq = oracle.idmap(src, None, dst_unique)
        got_src, got_uniq = oracle.idmap_parallel(src, dst_unique)
        assert np.array_equal(got_src, want_src), trial
        assert np.array_equal(got_uniq, want_uniq), trial
