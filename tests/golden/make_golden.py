"""Writes the committed fixtures of this directory from the CPU oracle.

The reference ships no tests, golden vectors or fixtures for this path, so these are the
build's own: small seeded inputs with the outputs the (separately pinned) oracle gives,
kept so that both the oracle and the HIP kernels can be regression-checked without
regenerating anything.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as O  # noqa: E402


def main():
    # --- sampling + id-map over three hops -------------------------------------------
    indptr, indices = O.rmat_csr(2000, 24000, seed=3)
    seeds = np.random.default_rng(0).permutation(2000)[:200].astype(np.int32)
    fanouts = [4, 3, 2]  # reference order: the seeds are expanded with fanouts[-1] first
    input_nodes, blocks = O.sample_blocks(indptr, indices, seeds, fanouts, rng_seed=2024, stream_base=0)
    out = dict(indptr=indptr, indices=indices, seeds=seeds, fanouts=np.array(fanouts, np.int32),
               rng_seed=np.array(2024, np.int64), input_nodes=input_nodes)
    for i, b in enumerate(blocks):
        out["b%d_ptr" % i] = b["indptr"]
        out["b%d_src_local" % i] = b["src_local"]
        out["b%d_src_global" % i] = b["src_global"]
        out["b%d_shape" % i] = np.array([b["n_src"], b["n_dst"]], np.int64)
    np.savez_compressed(os.path.join(HERE, "sample_blocks_small.npz"), **out)

    # --- aggregation -------------------------------------------------------------------
    rng = np.random.default_rng(1)
    n_dst, n_src, D = 96, 300, 20
    deg = rng.integers(0, 9, size=n_dst)
    deg[5] = 70  # one row longer than a wave
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    idx = rng.integers(0, n_src, size=ptr[-1]).astype(np.int32)
    X = rng.standard_normal((n_src, D)).astype(np.float32)
    rn = np.maximum(deg, 1).astype(np.int32)
    cn = np.maximum(np.bincount(idx, minlength=n_src), 1).astype(np.int32)
    agg = dict(ptr=ptr, idx=idx, X=X, row_norm=rn, col_norm=cn)
    for mode in ("sum", "mean", "gcn", "colmean"):
        for policy in (0, 1):
            agg["%s_%d" % (mode, policy)] = O.aggregate(ptr, idx, X, mode, policy, rn, cn)
    t_ptr, t_idx = O.transpose(ptr, idx, n_src)
    agg["t_ptr"], agg["t_idx"] = t_ptr, t_idx
    np.savez_compressed(os.path.join(HERE, "aggregate_small.npz"), **agg)

    # --- hand-enumerated id-map case (written out by hand, not by the oracle) ----------
    np.savez(os.path.join(HERE, "idmap_hand.npz"),
             src=np.array([9, 3, 9, 5, 7], np.int32), dst=np.array([7, 7, 3, 3, 3], np.int32),
             dst_unique=np.array([7, 3], np.int32), uniq=np.array([7, 3, 9, 5], np.int32),
             src_local=np.array([2, 1, 2, 3, 0], np.int32), dst_local=np.array([0, 0, 1, 1, 1], np.int32))


if __name__ == "__main__":
    main()
