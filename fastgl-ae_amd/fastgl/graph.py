"""Synthetic graphs and the CSR layout the sampler consumes.

The layout is the one the reference's trainer builds (train_fastgl.py:218-230): edges sorted
by destination, ``edge_ptr = [0, cumsum(in_degree)]``, ``edge_src`` = source id of every edge.
Here ``edge_ptr`` is int64 (graphs with more than 2^31 edges) unless asked otherwise, and
``edge_src`` is int32.
"""
from __future__ import annotations

import math

import torch

from . import ops

_I64_MAX = (1 << 63) - 1


def rmat_scale(n_nodes: int) -> int:
    return max(1, int(math.ceil(math.log2(max(int(n_nodes), 2)))))


def rmat_csr(n_nodes: int, n_draws: int, seed: int = 0, device="cuda", ptr_dtype=torch.int64, chunk_draws=1 << 28):
    """Seeded R-MAT graph (a=.57, b=.19, c=.19, d=.05), symmetrised, without self loops or
    duplicate edges, as an in-neighbour CSR ``(edge_ptr, edge_src)`` with sorted rows."""
    scale = rmat_scale(n_nodes)
    parts = []
    for first in range(0, int(n_draws), int(chunk_draws)):
        n = min(int(chunk_draws), int(n_draws) - first)
        k = torch.unique(ops.rmat_keys(first, n, scale, n_nodes, seed, device))
        if k.numel() and int(k[-1]) == _I64_MAX:
            k = k[:-1]
        parts.append(k)
    keys = _merge_sorted_unique(parts, device)
    del parts
    return csr_from_keys(keys, n_nodes, ptr_dtype)


def _merge_sorted_unique(parts, device, max_items=1 << 30):
    """Union of sorted duplicate-free int64 lists, sorted.  torch's sort/unique take fewer than
    2^31 items per call, so a large union is assembled from disjoint key ranges (each range is a
    contiguous slice of every sorted part)."""
    if not parts:
        return torch.empty(0, dtype=torch.int64, device=device)
    if len(parts) == 1:
        return parts[0]
    total = sum(int(p.numel()) for p in parts)
    if total <= max_items:
        return torch.unique(torch.cat(parts))
    n_ranges = 2 * ((total + max_items - 1) // max_items)
    ref = max(parts, key=lambda p: p.numel())
    cuts = ref[torch.linspace(0, ref.numel() - 1, n_ranges + 1, device=device).long()[1:-1]]  # quantiles of one part
    cut_pos = [torch.searchsorted(p, cuts).tolist() for p in parts]
    out = []
    for r in range(n_ranges):
        segs = []
        for p, pos in zip(parts, cut_pos):
            lo = 0 if r == 0 else pos[r - 1]
            hi = p.numel() if r == n_ranges - 1 else pos[r]
            segs.append(p[lo:hi])
        seg = torch.cat(segs)
        if seg.numel() >= (1 << 31) - 1:
            raise RuntimeError("rmat_csr: a key range holds %d items; use smaller chunks" % seg.numel())
        out.append(torch.unique(seg))
        del segs, seg
    return torch.cat(out)


def csr_from_keys(keys, n_nodes: int, ptr_dtype=torch.int64, chunk=1 << 26):
    """Sorted unique keys ``row<<32 | col`` -> ``(edge_ptr[n_nodes+1], edge_src int32)``."""
    dev = keys.device
    edge_src = (keys & 0xFFFFFFFF).to(torch.int32)
    edge_ptr = torch.empty(n_nodes + 1, dtype=ptr_dtype, device=dev)
    for first in range(0, n_nodes + 1, chunk):
        last = min(first + chunk, n_nodes + 1)
        bounds = torch.arange(first, last, dtype=torch.int64, device=dev) << 32
        edge_ptr[first:last] = torch.searchsorted(keys, bounds).to(ptr_dtype)
    return edge_ptr, edge_src


def csr_from_coo(src, dst, n_nodes: int, ptr_dtype=torch.int64):
    """The reference trainer's CSR construction (train_fastgl.py:218-230) for an arbitrary
    edge list: stable sort by destination, offsets from the in-degrees."""
    dst_sorted, order = torch.sort(dst.long(), stable=True)
    edge_src = src[order].to(torch.int32).contiguous()
    deg = torch.bincount(dst_sorted, minlength=n_nodes)
    edge_ptr = torch.zeros(n_nodes + 1, dtype=ptr_dtype, device=src.device)
    edge_ptr[1:] = torch.cumsum(deg, 0).to(ptr_dtype)
    return edge_ptr, edge_src
