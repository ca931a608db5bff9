"""fgl_sample_node_static -- the entry point that allocates nothing (its scratch is a device array the
library itself holds) -- against fgl_sample_node with a caller workspace: same bits, on two calls in a
row, the second with a smaller input (the scratch keeps the first call's contents)."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(cuda, ptr, idx, seeds, fanout, rng_seed, stream_id):
    from fastgl import _lib as L
    lib = L.lib()
    n = int(seeds.numel())
    st = L.stream_handle()
    outs = []
    for static in (False, True):
        src = torch.full((max(n * fanout, 1),), -7, dtype=torch.int32, device=cuda)
        dst = torch.full((max(n * fanout, 1),), -7, dtype=torch.int32, device=cuda)
        bptr = torch.full((n + 1,), -7, dtype=torch.int32, device=cuda)
        meta = torch.zeros(2, dtype=torch.int32, device=cuda)  # [edge count, status]
        head = (L.ptr(ptr), int(ptr.dtype == torch.int64), L.ptr(idx), int(ptr.numel()) - 1, L.ptr(seeds), n, None, fanout,
                rng_seed, stream_id, L.ptr(src), L.ptr(dst), L.ptr(bptr), meta.data_ptr(), meta.data_ptr() + 4)
        if static:
            L.check(lib.fgl_sample_node_static(*head, st))
        else:
            ws = torch.empty(max(lib.fgl_sample_workspace_bytes(n, fanout), 256), dtype=torch.uint8, device=cuda)
            L.check(lib.fgl_sample_node(*head, None, L.ptr(ws), ws.numel(), st))
        torch.cuda.synchronize()
        outs.append((src.cpu().numpy(), dst.cpu().numpy(), bptr.cpu().numpy(), meta.cpu().numpy()))
    return outs


@pytest.mark.parametrize("ptr_dtype", [np.int64, np.int32])
def test_static_scratch_matches_workspace_variant(cuda, oracle, small_graph, ptr_dtype):
    indptr, indices = small_graph
    ptr = torch.from_numpy(indptr.astype(ptr_dtype)).to(cuda)
    idx = torch.from_numpy(indices).to(cuda)
    rng = np.random.default_rng(12)
    # a large call first, then smaller ones: what the first leaves in the scratch must not show
    for n_seeds, fanout, stream_id in ((300_000, 15, 3), (5_000, 15, 4), (777, 64, 5), (0, 5, 6)):
        print("static sample: %d seeds, fanout %d, %s offsets" % (n_seeds, fanout, ptr_dtype.__name__), flush=True)
        seeds_h = rng.integers(0, indptr.size - 1, size=n_seeds).astype(np.int32)
        seeds = torch.from_numpy(seeds_h).to(cuda)
        (src_a, dst_a, ptr_a, meta_a), (src_b, dst_b, ptr_b, meta_b) = _both(cuda, ptr, idx, seeds, fanout, 99, stream_id)
        assert meta_a[1] == 0 and meta_b[1] == 0
        assert np.array_equal(meta_a, meta_b)
        assert np.array_equal(ptr_a, ptr_b)
        assert np.array_equal(src_a, src_b) and np.array_equal(dst_a, dst_b)
        if 0 < n_seeds <= 5_000:  # and both equal the oracle
            wsrc, wdst, wptr = oracle.sample_node(indptr.astype(ptr_dtype), indices, seeds_h, fanout, rng_seed=99, stream_id=stream_id)
            e = int(meta_b[0])
            assert np.array_equal(ptr_b, wptr) and np.array_equal(src_b[:e], wsrc) and np.array_equal(dst_b[:e], wdst)


def test_static_scratch_rejects_what_it_cannot_hold(cuda):
    from fastgl import _lib as L
    lib = L.lib()
    rc = lib.fgl_sample_node_static(None, 1, None, 10, None, (1 << 20) + 1, None, 5, 0, 0, None, None, None, None, None, None)
    assert rc == 1 and b"1048576" in lib.fgl_last_error()
