"""The oracle reproduces the committed fixtures (CPU only)."""
import os

import numpy as np

from conftest import GOLDEN_DIR


def test_sample_blocks_fixture(oracle):
    g = np.load(os.path.join(GOLDEN_DIR, "sample_blocks_small.npz"))
    inp, blocks = oracle.sample_blocks(g["indptr"], g["indices"], g["seeds"], g["fanouts"].tolist(), int(g["rng_seed"]), 0)
    assert np.array_equal(inp, g["input_nodes"])
    for i, b in enumerate(blocks):
        assert np.array_equal(b["indptr"], g["b%d_ptr" % i])
        assert np.array_equal(b["src_local"], g["b%d_src_local" % i])
        assert np.array_equal(b["src_global"], g["b%d_src_global" % i])
        assert [b["n_src"], b["n_dst"]] == g["b%d_shape" % i].tolist()
    # chain property of the layer loop: block i's dst nodes are block i+1's src nodes
    for i in range(len(blocks) - 1):
        assert blocks[i]["n_dst"] == blocks[i + 1]["n_src"]


def test_aggregate_fixture(oracle):
    g = np.load(os.path.join(GOLDEN_DIR, "aggregate_small.npz"))
    for mode in ("sum", "mean", "gcn", "colmean"):
        for policy in (0, 1):
            got = oracle.aggregate(g["ptr"], g["idx"], g["X"], mode, policy, g["row_norm"], g["col_norm"])
            assert np.allclose(got, g["%s_%d" % (mode, policy)], rtol=1e-13, atol=0)


def test_idmap_hand_fixture(oracle):
    g = np.load(os.path.join(GOLDEN_DIR, "idmap_hand.npz"))
    s, d, u = oracle.idmap(g["src"], g["dst"], g["dst_unique"])
    assert np.array_equal(s, g["src_local"]) and np.array_equal(d, g["dst_local"]) and np.array_equal(u, g["uniq"])
