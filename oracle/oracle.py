"""ctypes front-end of the CPU oracle (``libfgl_oracle.so``, built from ``fgl_oracle.c``).

TEST INFRASTRUCTURE ONLY.  The product package never imports this module: it is loaded
by the test-suite, by the smoke check and by the benchmark's CPU-baseline leg, as the
checker.  All arrays are numpy, C-contiguous; index arrays are int32 (graph ``indptr``
may be int32 or int64).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfgl_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a couple of seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libfgl_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        i64, i32, u64, u32, vp = C.c_int64, C.c_int, C.c_uint64, C.c_uint32, C.c_void_p
        L.orc_philox4x32_10.argtypes = [vp, vp, vp]
        L.orc_philox4x32_10.restype = None
        L.orc_floyd_subset.argtypes = [i64, i32, u64, u32, u64, vp]
        L.orc_floyd_subset.restype = None
        L.orc_sample_node.argtypes = [vp, i32, vp, vp, i64, i32, u64, u32, vp, vp, vp]
        L.orc_sample_node.restype = i64
        L.orc_table_size.argtypes = [i64, i32]
        L.orc_table_size.restype = i64
        L.orc_idmap.argtypes = [vp, vp, i64, vp, i64, vp, i64]
        L.orc_idmap.restype = i64
        L.orc_idmap_parallel.argtypes = [vp, i64, vp, i64, vp, i64]
        L.orc_idmap_parallel.restype = i64
        L.orc_cal_deg.argtypes = [vp, i64, vp, i64]
        L.orc_cal_deg.restype = None
        L.orc_exclusive_sum.argtypes = [vp, i64, vp]
        L.orc_exclusive_sum.restype = None
        L.orc_transpose.argtypes = [vp, vp, i64, i64, vp, vp]
        L.orc_transpose.restype = None
        for f in (L.orc_aggregate_f64, L.orc_aggregate_f32):
            f.argtypes = [vp, vp, i64, vp, i64, i32, i32, i32, vp, vp, vp]
            f.restype = None
        L.orc_aggregate_edge_f64.argtypes = [vp, vp, i64, vp, i64, i32, i32, vp, i32, vp, vp]
        L.orc_aggregate_edge_f64.restype = None
        L.orc_edge_softmax_f64.argtypes = [vp, vp, i64, vp, vp, i32, C.c_double, vp]
        L.orc_edge_softmax_f64.restype = None
        L.orc_rmat_keys.argtypes = [i64, i64, i32, i64, u64, vp]
        L.orc_rmat_keys.restype = None
        L.orc_num_threads.argtypes = []
        L.orc_num_threads.restype = i32
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _i32(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a


def num_threads() -> int:
    return int(lib().orc_num_threads())


# ---------------------------------------------------------------------------------------
def philox4x32_10(ctr, key):
    ctr = np.ascontiguousarray(ctr, dtype=np.uint32)
    key = np.ascontiguousarray(key, dtype=np.uint32)
    out = np.zeros(4, dtype=np.uint32)
    lib().orc_philox4x32_10(_p(ctr), _p(key), _p(out))
    return out


def floyd_subset(deg: int, k: int, rng_seed: int, stream_id: int, pos: int):
    sel = np.zeros(max(k, 1), dtype=np.int64)
    lib().orc_floyd_subset(deg, k, rng_seed, stream_id, pos, _p(sel))
    return sel[:k]


def sample_node(indptr, indices, seeds, fanout: int, rng_seed: int = 0, stream_id: int = 0):
    """-> (src_out[E], dst_out[E], block_ptr[S+1]) with global ids."""
    indptr = np.ascontiguousarray(indptr)
    assert indptr.dtype in (np.int32, np.int64)
    indices = _i32(indices)
    seeds = _i32(seeds)
    n = seeds.shape[0]
    src = np.zeros(max(n * fanout, 1), dtype=np.int32)
    dst = np.zeros(max(n * fanout, 1), dtype=np.int32)
    ptr = np.zeros(n + 1, dtype=np.int32)
    e = lib().orc_sample_node(_p(indptr), int(indptr.dtype == np.int64), _p(indices), _p(seeds), n, fanout,
                              rng_seed, stream_id, _p(src), _p(dst), _p(ptr))
    return src[:e].copy(), dst[:e].copy(), ptr


def table_size(num: int, scale: int) -> int:
    return int(lib().orc_table_size(num, scale))


def idmap(src_global, dst_global, dst_unique):
    """-> (src_local, dst_local or None, uniq).  First-occurrence numbering of new ids."""
    src = _i32(src_global).copy()
    dst = None if dst_global is None else _i32(dst_global).copy()
    du = _i32(dst_unique)
    cap = du.shape[0] + src.shape[0]
    uniq = np.zeros(max(cap, 1), dtype=np.int32)
    n = lib().orc_idmap(_p(src), _p(dst), src.shape[0], _p(du), du.shape[0], _p(uniq), cap)
    if n == -1:
        raise KeyError("an id of dst_global is not in dst_unique/src_global")
    if n < 0:
        raise RuntimeError("orc_idmap failed: %d" % n)
    return src, dst, uniq[:n].copy()


def idmap_parallel(src_global, dst_unique):
    """``idmap`` on all host threads (the CPU baseline's timing variant): -> (src_local, uniq)."""
    src = _i32(src_global).copy()
    du = _i32(dst_unique)
    cap = du.shape[0] + src.shape[0]
    uniq = np.empty(max(cap, 1), dtype=np.int32)
    n = lib().orc_idmap_parallel(_p(src), src.shape[0], _p(du), du.shape[0], _p(uniq), cap)
    if n < 0:
        raise RuntimeError("orc_idmap_parallel failed: %d" % n)
    return src, uniq[:n].copy()


def cal_deg(ids, n_nodes: int):
    ids = _i32(ids)
    deg = np.zeros(max(n_nodes, 1), dtype=np.int32)
    lib().orc_cal_deg(_p(ids), ids.shape[0], _p(deg), n_nodes)
    return deg[:n_nodes]


def exclusive_sum(deg):
    deg = _i32(deg)
    out = np.zeros(deg.shape[0] + 1, dtype=np.int32)
    lib().orc_exclusive_sum(_p(deg), deg.shape[0], _p(out))
    return out


def transpose(indptr, indices, n_cols: int):
    indptr = _i32(indptr)
    indices = _i32(indices)
    n_rows = indptr.shape[0] - 1
    t_ptr = np.zeros(n_cols + 1, dtype=np.int32)
    t_idx = np.zeros(max(int(indptr[-1]), 1), dtype=np.int32)
    lib().orc_transpose(_p(indptr), _p(indices), n_rows, n_cols, _p(t_ptr), _p(t_idx))
    return t_ptr, t_idx[: int(indptr[-1])]


MODES = {"sum": 0, "mean": 1, "gcn": 2, "colmean": 3}


def aggregate(indptr, indices, X, mode="sum", zero_policy=0, row_norm=None, col_norm=None, out_dtype=np.float64):
    """fp64-accumulated (or fp32 for timing) row aggregation of fp32 X over a CSR."""
    indptr = _i32(indptr)
    indices = _i32(indices)
    X = np.ascontiguousarray(X, dtype=np.float32)
    n_rows = indptr.shape[0] - 1
    D = X.shape[1]
    m = MODES[mode] if isinstance(mode, str) else int(mode)
    rn = None if row_norm is None else _i32(row_norm)
    cn = None if col_norm is None else _i32(col_norm)
    if m == 2:
        assert rn is not None and cn is not None
    if m == 3:
        assert cn is not None
    out = np.zeros((n_rows, D), dtype=out_dtype)
    fn = lib().orc_aggregate_f64 if out_dtype == np.float64 else lib().orc_aggregate_f32
    fn(_p(indptr), _p(indices), n_rows, _p(X), X.shape[1], D, m, zero_policy, _p(rn), _p(cn), _p(out))
    return out


def aggregate_edge(indptr, indices, X, edge_w, zero_policy=0, edge_index=None):
    """fp64 attention-weighted aggregation: edge_w is float32 [n_entries, n_heads]."""
    indptr = _i32(indptr)
    indices = _i32(indices)
    X = np.ascontiguousarray(X, dtype=np.float32)
    edge_w = np.ascontiguousarray(edge_w, dtype=np.float32)
    ei = None if edge_index is None else _i32(edge_index)
    n_rows = indptr.shape[0] - 1
    D = X.shape[1]
    assert D % edge_w.shape[1] == 0
    out = np.zeros((n_rows, D), dtype=np.float64)
    lib().orc_aggregate_edge_f64(_p(indptr), _p(indices), n_rows, _p(X), X.shape[1], D, zero_policy, _p(edge_w),
                                 edge_w.shape[1], _p(ei), _p(out))
    return out


def edge_softmax(indptr, indices, el, er, negative_slope=0.2):
    """fp64 GAT attention coefficients [n_entries, n_heads]; el float32 [n_cols, H], er float32 [n_rows, H]."""
    indptr = _i32(indptr)
    indices = _i32(indices)
    el = np.ascontiguousarray(el, dtype=np.float32)
    er = np.ascontiguousarray(er, dtype=np.float32)
    n_rows = indptr.shape[0] - 1
    H = el.shape[1]
    assert er.shape == (n_rows, H)
    alpha = np.zeros((indices.shape[0], H), dtype=np.float64)
    lib().orc_edge_softmax_f64(_p(indptr), _p(indices), n_rows, _p(el), _p(er), H, float(negative_slope), _p(alpha))
    return alpha


def transpose_with_edges(indptr, indices, n_cols: int):
    """(t_ptr, t_idx, t_edge): the stable transpose plus, per transposed entry, its position in `indices`."""
    indptr = _i32(indptr)
    indices = _i32(indices)
    order = np.argsort(indices, kind="stable").astype(np.int32)
    t_ptr, t_idx = transpose(indptr, indices, n_cols)
    return t_ptr, t_idx, order


def rmat_keys(first_edge: int, n_edges: int, scale: int, n_nodes: int, seed: int):
    keys = np.zeros(2 * n_edges, dtype=np.int64)
    lib().orc_rmat_keys(first_edge, n_edges, scale, n_nodes, seed, _p(keys))
    return keys


def rmat_csr(n_nodes: int, n_draws: int, seed: int = 0, indptr_dtype=np.int64):
    """Symmetrised, de-duplicated, self-loop-free R-MAT graph as an in-neighbour CSR
    (indptr, int32 indices sorted within each row)."""
    scale = max(1, int(np.ceil(np.log2(max(n_nodes, 2)))))
    keys = rmat_keys(0, n_draws, scale, n_nodes, seed)
    keys = np.unique(keys)
    if keys.size and keys[-1] == np.iinfo(np.int64).max:
        keys = keys[:-1]
    rows = (keys >> 32).astype(np.int64)
    cols = (keys & 0xFFFFFFFF).astype(np.int32)
    indptr = np.zeros(n_nodes + 1, dtype=np.int64)
    np.cumsum(np.bincount(rows, minlength=n_nodes), out=indptr[1:])
    return indptr.astype(indptr_dtype), cols


def sample_blocks(indptr, indices, seeds, fanouts, rng_seed=0, stream_base=0, parallel_idmap=False):
    """Layer loop of the reference's sampler (FusedMapSampler.py:63-109): seeds are expanded
    with fanouts[-1] first; layer k's unique list is layer k+1's seed list.
    -> (input_nodes, blocks) where blocks[i] = dict(indptr, src_local, src_global, n_dst, n_src),
    blocks[0] being the outermost hop."""
    cur = _i32(seeds).copy()
    blocks = []
    for li, fanout in enumerate(reversed(list(fanouts))):
        src_g, _dst_g, bptr = sample_node(indptr, indices, cur, fanout, rng_seed, stream_base + li)
        if parallel_idmap:
            src_l, uniq = idmap_parallel(src_g, cur)
        else:
            src_l, _, uniq = idmap(src_g, None, cur)
        blocks.insert(0, dict(indptr=bptr, src_local=src_l, src_global=src_g, n_dst=cur.shape[0], n_src=uniq.shape[0]))
        cur = uniq
    return cur, blocks
