"""The operator functions of the reference's ``fastgl`` extension module, with the same
names, positional arguments, return lists and error type (cuda_operators/aggregate_acc.cpp:
601-621 lists them; only the ones its Python code calls are provided), implemented over
the HIP C ABI.  Extensions that the reference does not have (mean aggregation, the
transposed block, the all-hops sampler) follow at the end.

Index tensors are int32 and must be contiguous device tensors (``RuntimeError`` otherwise,
as the reference's CHECK_INPUT, aggregate_acc.cpp:4-6); ``edge_ptr`` of the full graph may
also be int64.  Features are fp32 or bf16.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib as L

_rng_state = {"seed": 0, "calls": 0}


def manual_seed(seed: int) -> None:
    """Seed of the sampler's Philox streams; also resets the per-call stream counter.
    (The reference's picks come from one constant stream, sample.cu:70.)"""
    _rng_state["seed"] = int(seed) & 0xFFFFFFFFFFFFFFFF
    _rng_state["calls"] = 0


def _check_input(t, name, dtypes=None):
    if not isinstance(t, torch.Tensor):
        raise RuntimeError("%s must be a tensor" % name)
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    if dtypes is not None and t.dtype not in dtypes:
        raise RuntimeError("%s must have dtype in %s, got %s" % (name, [str(d) for d in dtypes], t.dtype))


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(dev):
    """Context that makes ``dev`` the current device -- nothing at all when it already is (the usual case: entering
    and leaving ``torch.cuda.device`` costs several microseconds per call)."""
    index = dev.index
    if index is None or index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(dev)


def _same_device(*tensors):
    dev = tensors[0].device
    for t in tensors[1:]:
        if t is not None and t.device != dev:
            raise RuntimeError("all tensors must live on the same device")
    return dev


_I32 = (torch.int32,)
_PTR = (torch.int32, torch.int64)
_FEAT = (torch.float32, torch.bfloat16)


def _raise_status(bits: int, where: str):
    if bits:
        raise RuntimeError("fastgl.%s: %s" % (where, L.status_message(bits)))


# ---------------------------------------------------------------------------------------
# drop-in operators
# ---------------------------------------------------------------------------------------
_host_words = {}


def _expect_sizes(dev, stream):
    """Two pinned host words per (device, stream) for a call's ``{size, status}``, marked pending: the call's kernels
    store both there themselves (no copy to enqueue), ``_sizes`` waits for them."""
    key = (torch.device(dev).index, stream)
    h = _host_words.get(key)
    if h is None:
        h = _host_words[key] = torch.empty(2, dtype=torch.int32, pin_memory=True)
    h.fill_(-1)  # (no size and no status word is all ones)
    return h


def _sizes(h, stream):
    L.check(L.lib().fgl_wait_words(h.data_ptr(), 2, -1, stream, 5000))
    return h.tolist()


def sample_node(src_edges, dst_edges, edge_ptr, seed_nodes, dst_nodes, neighbor_num):
    """fastgl.sample_node (aggregate_acc.cpp:491-512): ``-> [src_out, dst_out, edges_num]``.

    ``src_edges`` is the CSR ``indices`` of the in-neighbour graph, ``edge_ptr`` its
    ``indptr``; ``dst_edges`` is accepted and, as in the reference kernels, never read.
    Outputs hold global ids, each seed's edges contiguous, seeds in order.
    """
    _check_input(src_edges, "src_edges", _I32)
    _check_input(dst_edges, "dst_edges")
    _check_input(edge_ptr, "edge_ptr", _PTR)
    _check_input(seed_nodes, "seed_nodes", _I32)
    dev = _same_device(src_edges, edge_ptr, seed_nodes)
    n_seeds = int(seed_nodes.size(0))
    dst_nodes = int(dst_nodes)
    fanout = int(neighbor_num)
    if dst_nodes < n_seeds:
        raise RuntimeError("dst_nodes (%d) is smaller than the number of seeds (%d)" % (dst_nodes, n_seeds))
    lib = L.lib()
    with _on_device(dev):
        src_out = torch.empty(max(dst_nodes * fanout, 1), dtype=torch.int32, device=dev)
        dst_out = torch.empty(max(dst_nodes * fanout, 1), dtype=torch.int32, device=dev)
        block_ptr = torch.empty(n_seeds + 1, dtype=torch.int32, device=dev)
        meta = torch.zeros(2, dtype=torch.int32, device=dev)  # [edge count, status]
        ws_bytes = lib.fgl_sample_workspace_bytes(n_seeds, fanout)
        ws = L.workspace(ws_bytes, dev)
        stream_id = _rng_state["calls"] & 0xFFFFFFFF
        _rng_state["calls"] += 1
        st = L.stream_handle()
        host = _expect_sizes(dev, st)
        L.check(lib.fgl_sample_node(L.ptr(edge_ptr), int(edge_ptr.dtype == torch.int64), L.ptr(src_edges),
                                    int(edge_ptr.size(0)) - 1, L.ptr(seed_nodes), n_seeds, None, fanout,
                                    _rng_state["seed"], stream_id, L.ptr(src_out), L.ptr(dst_out), L.ptr(block_ptr),
                                    meta.data_ptr(), meta.data_ptr() + 4, host.data_ptr(), L.ptr(ws), ws.numel(), st))
        n_edges, status = _sizes(host, st)  # the host read-back the reference also does (sample.cu:202)
    _raise_status(status, "sample_node")
    edges_num = meta[:1]
    out = [src_out[:n_edges], dst_out[:n_edges], edges_num]
    sample_node.last_block_ptr = block_ptr  # CSR offsets of the block just sampled
    return out


sample_node.last_block_ptr = None


def transfer_edge_id(src_edges, dst_edges, dst_edges_unique, dst_nodes, total_items, unique_num, edge_nums):
    """fastgl.transfer_edge_id (aggregate_acc.cpp:467-489, id_map.cu:386-493): the fused
    id-map.  Rewrites ``src_edges`` / ``dst_edges`` in place to local ids and returns
    ``[src_edges, dst_edges, uniq]`` with ``uniq = cat(dst_edges_unique, new source ids)``.
    New ids are numbered in first-occurrence order."""
    _check_input(src_edges, "src_edges", _I32)
    _check_input(dst_edges, "dst_edges", _I32)
    _check_input(dst_edges_unique, "dst_edges_unique", _I32)
    dev = _same_device(src_edges, dst_edges, dst_edges_unique)
    n_dst = int(dst_nodes)
    n_edges = int(edge_nums)
    if n_dst > dst_edges_unique.size(0):
        raise RuntimeError("dst_nodes (%d) exceeds len(dst_edges_unique) (%d)" % (n_dst, dst_edges_unique.size(0)))
    if n_edges > src_edges.size(0) or n_edges > dst_edges.size(0):
        raise RuntimeError("edge_nums (%d) exceeds the edge arrays" % n_edges)
    if int(total_items) - n_dst != n_edges:
        raise RuntimeError("total_items - dst_nodes must equal edge_nums (id_map.cu:308)")
    lib = L.lib()
    max_new = max(0, min(int(unique_num), n_edges))
    capacity = n_dst + max_new
    slots = lib.fgl_idmap_slots(capacity)
    with _on_device(dev):
        st = L.stream_handle()
        key = (torch.device(dev).index, st)
        table, known_empty = _table(slots, dev)
        uniq = torch.empty(max(capacity, 1), dtype=torch.int32, device=dev)
        meta = torch.zeros(2, dtype=torch.int32, device=dev)  # [n_total, status]
        ws_bytes = lib.fgl_idmap_map_src_workspace_bytes(n_edges)
        ws = L.workspace(ws_bytes, dev)
        status_ptr = meta.data_ptr() + 4
        # the table is a prefix of a persistent buffer that every call leaves empty: only slots that no call has
        # emptied yet are filled here (in the steady state of a training loop: none)
        if known_empty < slots:
            L.check(lib.fgl_idmap_reset(L.ptr(table), slots, st))
        _tables[key] = (table, 0)
        host = _expect_sizes(dev, st)
        # destination ids in, then three passes over the edges (the destination half rides on the first); the last
        # writes nothing back into the table (no later call looks these ids up) and empties it
        L.check(lib.fgl_idmap_transfer(L.ptr(table), slots, L.ptr(dst_edges_unique), n_dst, L.ptr(src_edges), L.ptr(dst_edges),
                                       n_edges, L.ptr(uniq), capacity,
                                       L.IDMAP_ORDERED | L.IDMAP_FINAL | L.IDMAP_LEAVE_TABLE_EMPTY, meta.data_ptr(), status_ptr,
                                       host.data_ptr(), L.ptr(ws), ws.numel(), st))
        _tables[key] = (table, max(known_empty, slots))
        n_total, status = _sizes(host, st)  # host read-back, as id_map.cu:454,491
    _raise_status(status, "transfer_edge_id")
    return [src_edges, dst_edges, uniq[:n_total]]


_tables = {}


def _table(slots: int, dev):
    """Hash-table storage, cached per (device, stream) and grown on demand (the reference
    cudaMallocs, memsets and cudaFrees one per call, id_map.cu:45-59), with the number of its leading slots
    that are known to hold the empty marker."""
    key = (torch.device(dev).index, L.stream_handle())
    t, known_empty = _tables.get(key, (None, 0))
    if t is None or t.numel() < slots:
        t, known_empty = torch.empty(int(slots), dtype=torch.int64, device=dev), 0
        _tables[key] = (t, 0)
    return t, known_empty


def cal_deg(edges, nodes_num):
    """fastgl.cal_deg (aggregate_acc.cpp:522-529): int32 histogram of ``edges`` over ``nodes_num`` bins."""
    _check_input(edges, "edges", _I32)
    n = int(nodes_num)
    dev = edges.device
    with _on_device(dev):
        deg = torch.empty(max(n, 1), dtype=torch.int32, device=dev)[:n]
        L.check(L.lib().fgl_cal_deg(L.ptr(edges), int(edges.numel()), None, L.ptr(deg), n, L.stream_handle()))
    return deg


def exclusive_sum(in_degs):
    """fastgl.exclusive_sum (aggregate_acc.cpp:514-520): ``len+1`` exclusive prefix sums (int32)."""
    _check_input(in_degs, "in_degs", _I32)
    n = int(in_degs.numel())
    dev = in_degs.device
    lib = L.lib()
    with _on_device(dev):
        out = torch.empty(n + 1, dtype=torch.int32, device=dev)
        ws = L.workspace(lib.fgl_exclusive_sum_workspace_bytes(n), dev)
        L.check(lib.fgl_exclusive_sum_i32(L.ptr(in_degs), n, None, L.ptr(out), L.ptr(ws), ws.numel(), L.stream_handle()))
    return out


def _fanout_bound(edge_ptr, neighbor_num):
    """``neighbor_num`` bounds the entries per row of a sampled block (the reference sizes its shared
    staging by it, aggregate_acc_kernel.cu:238-247)."""
    bound = getattr(edge_ptr, "fgl_longest_row", None)
    if bound is None and int(neighbor_num) > 0:
        bound = int(neighbor_num)
    return bound


def forward_gcn(edge_ptr, src_edges, src_norm_degs, dst_norm_degs, input_feat, weight, neighbor_num, dst_nodes):
    """fastgl.forward_gcn (aggregate_acc.cpp:133-160): ``[A_norm (X W)]`` with
    ``A_norm[d, s] = 1/sqrt(dst_norm[d]) * 1/sqrt(src_norm[s])``; a dst row without edges
    passes ``(X W)[d]`` through (aggregate_acc_kernel.cu:307-309)."""
    for t, n in ((edge_ptr, "edge_ptr"), (src_edges, "src_edges"), (src_norm_degs, "src_norm_degs"),
                 (dst_norm_degs, "dst_norm_degs")):
        _check_input(t, n, _I32)
    _check_input(input_feat, "input_feat", _FEAT)
    _check_input(weight, "weight", _FEAT)
    tmp = torch.mm(input_feat, weight)
    out = aggregate(edge_ptr, src_edges, tmp, mode="gcn", zero_policy="self", row_norm=dst_norm_degs,
                    col_norm=src_norm_degs, n_rows=int(dst_nodes), longest_row=_fanout_bound(edge_ptr, neighbor_num))
    return [out]


def backward_gcn(edge_ptr, src_edges, src_norm_degs, dst_norm_degs, d_input, weight, input_feat):
    """fastgl.backward_gcn (aggregate_acc.cpp:349-376): ``[d_x, d_w]``.

    Positional meaning as in the reference kernel (aggregate_acc_kernel.cu:494,509): the
    third argument is indexed by destination id and the fourth by source id -- the caller
    passes ``(dst_norm, src_norm)`` there (GraphConv.py:37)."""
    by_dst, by_src = src_norm_degs, dst_norm_degs
    for t, n in ((edge_ptr, "edge_ptr"), (src_edges, "src_edges"), (by_dst, "src_norm_degs"), (by_src, "dst_norm_degs")):
        _check_input(t, n, _I32)
    _check_input(d_input, "d_input", _FEAT)
    _check_input(weight, "weight", _FEAT)
    _check_input(input_feat, "input_feat", _FEAT)
    n_src = int(input_feat.size(0))
    n_dst = int(d_input.size(0))
    t_ptr, t_idx = block_transpose(edge_ptr, src_edges, n_dst, n_src)
    g = aggregate(t_ptr, t_idx, d_input, mode="gcn", zero_policy="zeros", row_norm=by_src, col_norm=by_dst, n_rows=n_src)
    d_x = torch.mm(g, weight.transpose(0, 1))
    d_w = torch.mm(input_feat.transpose(0, 1), g)
    return [d_x, d_w]


def forwaed_gin(edge_ptr, src_edges, input_feat, weight, neighbor_num, dst_nodes):
    """fastgl.forwaed_gin (sic; aggregate_acc.cpp:173-199, exported at :613): ``[tmp W, tmp]``
    with ``tmp[d] = sum of X[s] over the edges into d`` (``X[d]`` if there are none)."""
    _check_input(edge_ptr, "edge_ptr", _I32)
    _check_input(src_edges, "src_edges", _I32)
    _check_input(input_feat, "input_feat", _FEAT)
    _check_input(weight, "weight", _FEAT)
    tmp = aggregate(edge_ptr, src_edges, input_feat, mode="sum", zero_policy="self", n_rows=int(dst_nodes),
                    longest_row=_fanout_bound(edge_ptr, neighbor_num))
    return [torch.mm(tmp, weight), tmp]


def backward_gin(edge_ptr, src_edges, d_input, weight, input_feat, src_nodes):
    """fastgl.backward_gin (aggregate_acc.cpp:387-409): ``[d_x, d_w]``; ``input_feat`` is the
    ``tmp`` that forwaed_gin returned."""
    _check_input(edge_ptr, "edge_ptr", _I32)
    _check_input(src_edges, "src_edges", _I32)
    _check_input(d_input, "d_input", _FEAT)
    _check_input(weight, "weight", _FEAT)
    _check_input(input_feat, "input_feat", _FEAT)
    d_tmp = torch.mm(d_input, weight.transpose(0, 1))
    d_w = torch.mm(input_feat.transpose(0, 1), d_input)
    n_dst = int(d_input.size(0))
    t_ptr, t_idx = block_transpose(edge_ptr, src_edges, n_dst, int(src_nodes))
    d_x = aggregate(t_ptr, t_idx, d_tmp, mode="sum", zero_policy="zeros", n_rows=int(src_nodes))
    return [d_x, d_w]


def forward_gat(edge_ptr, edge_data, src_edges, input_feat, neighbor_num, dst_nodes, num_heads):
    """fastgl.forward_gat (aggregate_acc.cpp, kernel aggregate_acc_kernel.cu:835-886):
    ``[out]`` with ``out[d, f] = sum_e edge_data[e, f // (D / num_heads)] * input_feat[src[e], f]``
    (``input_feat[d]`` if d has no edges)."""
    _check_input(edge_ptr, "edge_ptr", _I32)
    _check_input(src_edges, "src_edges", _I32)
    _check_input(edge_data, "edge_data", (torch.float32,))
    _check_input(input_feat, "input_feat", _FEAT)
    return [aggregate(edge_ptr, src_edges, input_feat, mode="edge", zero_policy="self", n_rows=int(dst_nodes),
                      edge_weight=edge_data.view(edge_data.size(0), -1), n_heads=int(num_heads))]


def backward_gat(edge_ptr, edge_data, src_edges, d_input, src_nodes, num_heads):
    """fastgl.backward_gat (kernel aggregate_acc_kernel.cu:924-979): ``[d_x]`` with
    ``d_x[s, f] = sum over the edges (s -> d) of edge_data[e, head(f)] * d_input[d, f]`` -- as a gather
    over the transposed block instead of float atomics."""
    _check_input(edge_ptr, "edge_ptr", _I32)
    _check_input(src_edges, "src_edges", _I32)
    _check_input(edge_data, "edge_data", (torch.float32,))
    _check_input(d_input, "d_input", _FEAT)
    n_dst = int(d_input.size(0))
    t_ptr, t_idx, t_edge = block_transpose(edge_ptr, src_edges, n_dst, int(src_nodes), edge_ids=True)
    return [aggregate(t_ptr, t_idx, d_input, mode="edge", zero_policy="zeros", n_rows=int(src_nodes),
                      edge_weight=edge_data.view(edge_data.size(0), -1), n_heads=int(num_heads), edge_index=t_edge)]


# ---------------------------------------------------------------------------------------
# extensions
# ---------------------------------------------------------------------------------------
_MODES = {"sum": L.AGG_SUM, "mean": L.AGG_MEAN, "gcn": L.AGG_GCN, "colmean": L.AGG_COLMEAN, "edge": L.AGG_EDGE,
          "colmean_ptr": L.AGG_COLMEAN_PTR}
_ZERO = {"self": L.ZERO_COPY_SELF, "zeros": L.ZERO_ZEROS}


def aggregate(indptr, indices, feat, mode="sum", zero_policy="self", row_norm=None, col_norm=None, n_rows=None,
              out=None, edge_weight=None, n_heads=1, edge_index=None, longest_row=None, n_rows_dev=None, mapping="auto"):
    """``out[r] = sum_e w(r, indices[e]) * feat[indices[e]]`` over the CSR rows (fp32
    accumulation; fp32 or bf16 storage).  ``mode``: sum | mean | gcn | colmean | edge | colmean_ptr (colmean with
    ``col_norm`` holding the offsets array whose differences are the counts: a block's ``edge_ptr``);
    ``zero_policy``: what a row without entries gets -- ``self`` (``feat[r]``) or ``zeros``.
    ``longest_row``: what is known about the longest row's entry count -- an ``int`` bound (the fanout of a
    sampled block) or a one-element int32 device tensor (as ``block_transpose`` makes).  Speed only: hub rows
    of hundreds of entries get a second launch that a bound can save.  When not given it is taken from the
    ``fgl_longest_row`` attribute that ``block_transpose`` and the sampler attach to their ``indptr`` tensors.
    ``mode="edge"``: ``edge_weight`` float32 [n_entries, n_heads], weight of entry e for column f is
    ``edge_weight[edge_index[e] if edge_index is not None else e, f // (D // n_heads)]``.
    ``n_rows_dev``: one-element int32 device tensor with the actual row count when the host only knows the
    bound ``n_rows`` (a block whose sizes have not been read back yet): rows past it are left unwritten.
    ``mapping``: ``"auto"`` lets the library pick how lanes are dealt to rows from the row count, the entry count
    and ``longest_row`` (several lane groups per row for few long rows, several rows per group for many short
    ones); ``"row"`` asks for one lane group per row whatever the shape (what measurements of that kernel use)."""
    _check_input(indptr, "indptr", _I32)
    _check_input(indices, "indices", _I32)
    if not isinstance(feat, torch.Tensor) or not feat.is_cuda:
        raise RuntimeError("feat must be a CUDA tensor")
    if feat.dim() != 2 or feat.stride(1) != 1 or feat.dtype not in _FEAT:
        raise RuntimeError("feat must be a 2-D fp32/bf16 tensor with unit column stride")
    if row_norm is not None:
        _check_input(row_norm, "row_norm", _I32)
    if col_norm is not None:
        _check_input(col_norm, "col_norm", _I32)
    if edge_weight is not None:
        _check_input(edge_weight, "edge_weight", (torch.float32,))
        if edge_weight.dim() != 2 or edge_weight.size(1) != int(n_heads):
            raise RuntimeError("edge_weight must be [n_entries, n_heads]")
        if edge_index is None and edge_weight.size(0) < indices.numel():
            raise RuntimeError("edge_weight has fewer rows than there are entries")
    if edge_index is not None:
        _check_input(edge_index, "edge_index", _I32)
        if edge_index.numel() < indices.numel():
            raise RuntimeError("edge_index has fewer entries than indices")
    if mode == "edge" and (edge_weight is None or feat.size(1) % int(n_heads) != 0):
        raise RuntimeError("mode 'edge' needs edge_weight and a head count that divides the row length")
    if longest_row is None:
        longest_row = getattr(indptr, "fgl_longest_row", None)
    longest_host, longest_dev = -1, None
    if isinstance(longest_row, torch.Tensor):
        _check_input(longest_row, "longest_row", _I32)
        if longest_row.numel() != 1:
            raise RuntimeError("longest_row must hold one int32")
        longest_dev = longest_row
    elif longest_row is not None:
        longest_host = int(longest_row)
    if n_rows_dev is not None:
        _check_input(n_rows_dev, "n_rows_dev", _I32)
        if n_rows_dev.numel() != 1:
            raise RuntimeError("n_rows_dev must hold one int32")
    dev = _same_device(indptr, indices, feat, row_norm, col_norm, edge_weight, edge_index, longest_dev, n_rows_dev)
    n = int(indptr.numel()) - 1 if n_rows is None else int(n_rows)
    if n < 0 or n > indptr.numel() - 1:
        raise RuntimeError("n_rows (%d) does not match indptr (%d entries)" % (n, indptr.numel()))
    if mapping not in ("auto", "row"):
        raise RuntimeError("mapping must be 'auto' or 'row'")
    m = _MODES[mode]
    z = _ZERO[zero_policy]
    if z == L.ZERO_COPY_SELF and n > feat.size(0):
        raise RuntimeError("zero_policy 'self' needs feat to have a row for every output row")
    D = int(feat.size(1))
    with _on_device(dev):
        if out is None:
            out = torch.empty((n, D), dtype=feat.dtype, device=dev)
        elif out.shape != (n, D) or out.dtype != feat.dtype or out.stride(1) != 1 or not out.is_cuda:
            raise RuntimeError("out has the wrong shape, dtype or layout")
        if n > 0:
            # a block without entries has no index array to point at; the kernel then reads none
            idx_ptr = L.ptr(indices) if indices.numel() else L.ptr(indptr)
            L.check(L.lib().fgl_aggregate(L.ptr(indptr), idx_ptr, n, L.ptr(n_rows_dev), L.ptr(feat), int(feat.stride(0)), D,
                                          L.F32 if feat.dtype == torch.float32 else L.BF16, m, z, L.ptr(row_norm),
                                          L.ptr(col_norm), L.ptr(edge_weight), int(n_heads), L.ptr(edge_index),
                                          longest_host if mapping == "auto" else -1, L.ptr(longest_dev),
                                          int(indices.numel()) if mapping == "auto" else -1, L.ptr(out),
                                          int(out.stride(0)), L.stream_handle()))
    return out


def edge_softmax(indptr, indices, el, er, negative_slope=0.2, n_rows=None):
    """Attention coefficients of a GAT layer over a block CSR, ``float32 [n_entries, n_heads]``:
    ``softmax`` over the entries of each row of ``leaky_relu(el[indices[e]] + er[row])`` -- the reference's
    ``u_add_v`` + ``leaky_relu`` + ``edge_softmax`` (GraphConv.py:265-272) in one launch.  ``el``: float32
    [n_cols, n_heads], ``er``: float32 [n_rows, n_heads]."""
    _check_input(indptr, "indptr", _I32)
    _check_input(indices, "indices", _I32)
    _check_input(el, "el", (torch.float32,))
    _check_input(er, "er", (torch.float32,))
    if el.dim() != 2 or er.dim() != 2 or el.size(1) != er.size(1):
        raise RuntimeError("el and er must be [n, n_heads] with the same head count")
    dev = _same_device(indptr, indices, el, er)
    n = int(indptr.numel()) - 1 if n_rows is None else int(n_rows)
    if n < 0 or n > indptr.numel() - 1 or n > er.size(0):
        raise RuntimeError("n_rows (%d) does not match indptr (%d entries) / er (%d rows)" % (n, indptr.numel(), er.size(0)))
    H = int(el.size(1))
    with _on_device(dev):
        alpha = torch.empty((int(indices.numel()), H), dtype=torch.float32, device=dev)
        if n > 0 and indices.numel() > 0:
            L.check(L.lib().fgl_edge_softmax(L.ptr(indptr), L.ptr(indices), n, None, L.ptr(el), L.ptr(er), H,
                                             float(negative_slope), L.ptr(alpha), L.stream_handle()))
    return alpha


def block_transpose(indptr, indices, n_rows, n_cols, edge_ids=False, sorted_rows=False):
    """Column-major companion ``(t_indptr[n_cols+1], t_indices[nnz])`` of a block CSR; with
    ``edge_ids=True`` also ``t_edge[nnz]``, the position in ``indices`` of every transposed entry.
    ``sorted_rows=True`` lists every column's rows in ascending order (deterministic; the default
    leaves the order within a column to scheduling and is faster)."""
    _check_input(indptr, "indptr", _I32)
    _check_input(indices, "indices", _I32)
    dev = _same_device(indptr, indices)
    n_rows, n_cols = int(n_rows), int(n_cols)
    nnz = int(indices.numel())
    lib = L.lib()
    with _on_device(dev):
        t_ptr = torch.empty(n_cols + 1, dtype=torch.int32, device=dev)
        t_idx = torch.empty(max(nnz, 1), dtype=torch.int32, device=dev)[:nnz]
        t_edge = torch.empty(max(nnz, 1), dtype=torch.int32, device=dev)[:nnz] if edge_ids else None
        longest = torch.empty(1, dtype=torch.int32, device=dev)
        ws = L.workspace(lib.fgl_block_transpose_workspace_bytes(n_cols, nnz, int(sorted_rows)), dev)
        L.check(lib.fgl_block_transpose(L.ptr(indptr), L.ptr(indices), n_rows, None, n_cols, None, nnz, L.ptr(t_ptr),
                                        L.ptr(t_idx), L.ptr(t_edge), L.ptr(longest), int(sorted_rows), L.ptr(ws), ws.numel(),
                                        L.stream_handle()))
    t_ptr.fgl_longest_row = longest  # read by aggregate()
    return (t_ptr, t_idx, t_edge) if edge_ids else (t_ptr, t_idx)


def block_transpose_batch(blocks, edge_ids=False):
    """``block_transpose`` (unordered lists) for several blocks in the launches that one takes.  ``blocks``: list of
    ``(indptr, indices, n_rows, n_cols)``; returns a list of ``(t_indptr, t_indices, t_edge or None)`` in the same order.
    Blocks too large for the batched entry point (2^20 entries, 2^23 columns: they fill the chip on their own) are
    transposed one by one."""
    lib = L.lib()
    out = [None] * len(blocks)
    small = []
    for i, (indptr, indices, n_rows, n_cols) in enumerate(blocks):
        _check_input(indptr, "indptr", _I32)
        _check_input(indices, "indices", _I32)
        if int(indices.numel()) < L.TRANSPOSE_BATCH_MAX_EDGES and int(n_cols) < L.TRANSPOSE_BATCH_MAX_COLS:
            small.append(i)
        else:
            r = block_transpose(indptr, indices, n_rows, n_cols, edge_ids=edge_ids)
            out[i] = (r[0], r[1], r[2] if edge_ids else None)
    for g in range(0, len(small), L.TRANSPOSE_BATCH_MAX):
        group = small[g:g + L.TRANSPOSE_BATCH_MAX]
        n = len(group)
        dev = _same_device(*[blocks[i][0] for i in group], *[blocks[i][1] for i in group])
        with _on_device(dev):
            res = []
            for i in group:
                indptr, indices, n_rows, n_cols = blocks[i]
                nnz = int(indices.numel())
                t_ptr = torch.empty(int(n_cols) + 1, dtype=torch.int32, device=dev)
                t_idx = torch.empty(max(nnz, 1), dtype=torch.int32, device=dev)[:nnz]
                t_edge = torch.empty(max(nnz, 1), dtype=torch.int32, device=dev)[:nnz] if edge_ids else None
                longest = torch.empty(1, dtype=torch.int32, device=dev)
                t_ptr.fgl_longest_row = longest
                res.append((t_ptr, t_idx, t_edge, longest))
            i64 = lambda vals: (C.c_int64 * n)(*[int(v) for v in vals])
            ptrs = lambda ts: (C.c_void_p * n)(*[L.ptr(t) for t in ts])
            n_rows_a, n_cols_a = i64(blocks[i][2] for i in group), i64(blocks[i][3] for i in group)
            n_edges_a = i64(blocks[i][1].numel() for i in group)
            ws = L.workspace(lib.fgl_block_transpose_batch_workspace_bytes(n, n_cols_a, n_edges_a), dev)
            L.check(lib.fgl_block_transpose_batch(n, ptrs(blocks[i][0] for i in group), ptrs(blocks[i][1] for i in group), n_rows_a,
                                                  n_cols_a, n_edges_a, ptrs(r[0] for r in res), ptrs(r[1] for r in res),
                                                  ptrs(r[2] for r in res) if edge_ids else None, ptrs(r[3] for r in res),
                                                  L.ptr(ws), ws.numel(), L.stream_handle()))
        for i, r in zip(group, res):
            out[i] = r[:3]
    return out


def table_size(num: int, scale: int) -> int:
    """The reference's TableSize (cuda_hashtable.cuh:27-30)."""
    return int(L.lib().fgl_table_size(int(num), int(scale)))


class BlocksPlan:
    """Bounds and persistent scratch for sampling mini-batches of one shape."""

    def __init__(self, n_nodes: int, n_seeds: int, hop_fanouts, device, node_capacity=None, transpose_hops=()):
        """``node_capacity`` (optional, ``n_hops + 1`` ints): the caller's own limit on the node count
        before each hop / after the last; the worst-case bounds are clipped to it.
        ``transpose_hops``: the hops (sampling order, negative = from the end) whose transposed block
        ``sample_blocks_fused`` is to build along the way."""
        lib = L.lib()
        self.n_nodes, self.n_seeds = int(n_nodes), int(n_seeds)
        self.hop_fanouts = [int(f) for f in hop_fanouts]
        self.n_hops = len(self.hop_fanouts)
        self.device = torch.device(device)
        self._fan = (C.c_int32 * self.n_hops)(*self.hop_fanouts)
        self._node_cap = None if node_capacity is None else (C.c_int64 * (self.n_hops + 1))(*[int(c) for c in node_capacity])
        cap_dst = (C.c_int64 * self.n_hops)()
        cap_edges = (C.c_int64 * self.n_hops)()
        cap_uniq, slots, ws_bytes = C.c_int64(), C.c_int64(), C.c_size_t()
        self.transpose_hops = sorted({(int(h) + self.n_hops) % self.n_hops for h in transpose_hops})
        self.transpose_mask = sum(1 << h for h in self.transpose_hops)
        L.check(lib.fgl_sample_blocks_plan(self.n_nodes, self.n_seeds, self._fan, self.n_hops, self._node_cap, self.transpose_mask,
                                           cap_dst, cap_edges, C.byref(cap_uniq), C.byref(slots), C.byref(ws_bytes)))
        self.cap_dst = list(cap_dst)
        self.cap_edges = list(cap_edges)
        self.cap_uniq, self.slots, self.ws_bytes = cap_uniq.value, slots.value, ws_bytes.value
        self.cap_src = self.cap_dst[1:] + [self.cap_uniq]  # source nodes (columns) of each hop's block
        self.table = torch.empty(self.slots, dtype=torch.int64, device=self.device)
        self.ws = torch.empty(max(self.ws_bytes, 256), dtype=torch.uint8, device=self.device)
        # the slot count that the last call on this plan's table left empty (None: unknown contents)
        self.empty_slots = None


def sample_blocks_fused(plan: BlocksPlan, edge_ptr, indices, seeds, rng_seed: int, stream_base: int,
                        keep_global=(0,), table_slots=None, id_order="first", stream_offset=None, readback=None,
                        launch_stream=None, sort_transposed=False):
    """All hops of one mini-batch in one enqueue (no host synchronisation inside).

    Returns device tensors sized by the plan's bounds: ``(uniq, block_ptr[h], src_local[h],
    src_global[h] or None, counts, transposed[h])``; hop 0 expands the raw seeds.  ``counts`` (int32,
    ``3*n_hops + 2``) holds the node count before each hop and after the last, then the
    edge count of each hop, then the status word, then per hop the longest row of its transposed block
    (zero where none was built); the caller reads it once per batch.
    For the hops in ``plan.transpose_hops`` the call also builds the transposed block:
    ``transposed[h] = (t_ptr, t_dst, t_edge)`` (bound-sized; ``None`` for the other hops).
    ``keep_global`` lists the hops (negative = from the end) whose pre-relabel source ids are kept.
    ``table_slots`` (a power of two, default the plan's worst case) uses only that much of the
    hash table; a batch that outgrows it is reported in the status word (FGL_STATUS_TABLE_FULL).
    ``id_order``: ``"first"`` numbers new ids by first occurrence (deterministic), ``"arrival"`` as
    their inserts land (the reference's rule, and about a tenth faster; any run is a valid map, equal to every other after
    sorting the new ids).
    ``stream_offset``: one-element int32 device tensor added to ``stream_base`` when the kernels run (for
    callers that capture this call in a graph and advance the random stream between replays).
    ``readback``: a pinned int32 host tensor of ``3*n_hops + 2`` elements; the kernels store a copy of
    ``counts`` there when the last of them is final, so the caller's read-back is a wait for the stream and a
    look at that tensor, with no copy to enqueue.
    ``sort_transposed``: the rows of the transposed blocks come out in ascending order of their entries' positions in
    the block (run-to-run identical arrays and, with them, fp32 sums of the backward gathers; one more launch).
    ``launch_stream``: a ``torch.cuda.Stream`` to enqueue the kernels on instead of the current one (the outputs are
    still allocated on the current stream, where their consumer runs; the caller orders the two streams)."""
    _check_input(edge_ptr, "edge_ptr", _PTR)
    _check_input(indices, "indices", _I32)
    _check_input(seeds, "seeds", _I32)
    if stream_offset is not None:
        _check_input(stream_offset, "stream_offset", _I32)
    dev = _same_device(edge_ptr, indices, seeds, stream_offset)
    if int(seeds.numel()) != plan.n_seeds:
        raise RuntimeError("plan was made for %d seeds, got %d" % (plan.n_seeds, seeds.numel()))
    H = plan.n_hops
    if readback is not None and not (readback.dtype == torch.int32 and readback.is_pinned() and readback.is_contiguous()
                                     and readback.numel() >= 3 * H + 2):
        raise RuntimeError("readback must be a contiguous pinned int32 host tensor of at least %d elements" % (3 * H + 2))
    keep = {(h + H) % H for h in keep_global}
    slots = plan.slots if table_slots is None else min(int(table_slots), plan.slots)
    lib = L.lib()
    with _on_device(dev):
        uniq = torch.empty(max(plan.cap_uniq, 1), dtype=torch.int32, device=dev)
        block_ptr = [torch.empty(plan.cap_dst[h] + 1, dtype=torch.int32, device=dev) for h in range(H)]
        src_local = [torch.empty(max(plan.cap_edges[h], 1), dtype=torch.int32, device=dev) for h in range(H)]
        src_global = [torch.empty(max(plan.cap_edges[h], 1), dtype=torch.int32, device=dev) if h in keep else None
                      for h in range(H)]
        counts = torch.empty(3 * H + 2, dtype=torch.int32, device=dev)
        arr = lambda ts: (C.c_void_p * H)(*[L.ptr(t) for t in ts])
        transposed = [None] * H
        for h in plan.transpose_hops:
            transposed[h] = (torch.empty(plan.cap_src[h] + 1, dtype=torch.int32, device=dev),
                             torch.empty(max(plan.cap_edges[h], 1), dtype=torch.int32, device=dev),
                             torch.empty(max(plan.cap_edges[h], 1), dtype=torch.int32, device=dev))
        t_arr = lambda k: arr([None if t is None else t[k] for t in transposed]) if plan.transpose_hops else None
        # every call leaves the table empty for the next one (its last pass no longer reads it), so only a
        # plan's first call -- or the first after a failed one, or with another slot count -- pays for a fill
        flags = {"first": L.IDMAP_ORDERED, "arrival": L.IDMAP_ARRIVAL}[id_order] | L.BLOCKS_LEAVE_TABLE_EMPTY
        if plan.empty_slots == slots:
            flags |= L.BLOCKS_TABLE_EMPTY
        if sort_transposed:
            flags |= L.BLOCKS_SORT_TRANSPOSED
        plan.empty_slots = None
        L.check(lib.fgl_sample_blocks(L.ptr(edge_ptr), int(edge_ptr.dtype == torch.int64), L.ptr(indices),
                                      int(edge_ptr.numel()) - 1, L.ptr(seeds), plan.n_seeds, plan._fan, H, plan._node_cap,
                                      int(rng_seed) & 0xFFFFFFFFFFFFFFFF, int(stream_base) & 0xFFFFFFFF, L.ptr(stream_offset),
                                      flags, L.ptr(plan.table), slots, L.ptr(uniq), plan.cap_uniq, arr(block_ptr),
                                      arr(src_local), arr(src_global), t_arr(0), t_arr(1), t_arr(2), L.ptr(counts),
                                      None if readback is None else readback.data_ptr(), L.ptr(plan.ws),
                                      plan.ws.numel(), L.stream_handle() if launch_stream is None else launch_stream.cuda_stream))
        plan.empty_slots = slots
    return uniq, block_ptr, src_local, src_global, counts, transposed


def rmat_keys(first_edge: int, n_edges: int, scale: int, n_nodes: int, seed: int, device) -> torch.Tensor:
    """2*n_edges symmetrised int64 keys ``row<<32 | col`` of seeded R-MAT draws (INT64_MAX = dropped)."""
    with torch.cuda.device(device):
        keys = torch.empty(2 * int(n_edges), dtype=torch.int64, device=device)
        L.check(L.lib().fgl_rmat_keys(int(first_edge), int(n_edges), int(scale), int(n_nodes),
                                      int(seed) & 0xFFFFFFFFFFFFFFFF, L.ptr(keys), L.stream_handle()))
    return keys

