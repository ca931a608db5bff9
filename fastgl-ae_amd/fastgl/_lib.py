"""ctypes binding of ``libfastgl_hip.so`` (the C ABI declared in ``include/fastgl_hip.h``).

There is no fallback: if the shared library is missing or a call fails, a ``RuntimeError``
is raised.  torch is used only to own device memory and to name the current HIP stream.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libfastgl_hip.so")
CSRC_DIR = os.path.normpath(os.path.join(_PKG_DIR, "..", "csrc"))

# enum values of include/fastgl_hip.h
F32, BF16 = 0, 1
AGG_SUM, AGG_MEAN, AGG_GCN, AGG_COLMEAN, AGG_EDGE, AGG_COLMEAN_PTR = 0, 1, 2, 3, 4, 5
ZERO_COPY_SELF, ZERO_ZEROS = 0, 1
ABI_VERSION = 11  # FGL_ABI_VERSION of include/fastgl_hip.h that the signatures below follow
STATUS_TABLE_FULL, STATUS_UNIQ_OVERFLOW, STATUS_MISSING_KEY, STATUS_BAD_SEED, STATUS_BAD_ID = 1, 2, 4, 8, 16
IDMAP_ORDERED, IDMAP_ARRIVAL, IDMAP_FINAL, IDMAP_LEAVE_TABLE_EMPTY = 0, 1, 2, 8
BLOCKS_TABLE_EMPTY, BLOCKS_LEAVE_TABLE_EMPTY, BLOCKS_SORT_TRANSPOSED = 4, 8, 16
MAX_FANOUT = 192
SHORT_ROW_ENTRIES = 32
TRANSPOSE_BATCH_MAX, TRANSPOSE_BATCH_MAX_EDGES, TRANSPOSE_BATCH_MAX_COLS = 8, 1 << 20, 1 << 23

_i64, _i32, _u64, _u32, _vp, _sz = C.c_int64, C.c_int, C.c_uint64, C.c_uint32, C.c_void_p, C.c_size_t

# name -> (restype, argtypes): every symbol the header declares
SIGNATURES = {
    "fgl_abi_version": (_i32, []),
    "fgl_last_error": (C.c_char_p, []),
    "fgl_exclusive_sum_workspace_bytes": (_sz, [_i64]),
    "fgl_exclusive_sum_i32": (_i32, [_vp, _i64, _vp, _vp, _vp, _sz, _vp]),
    "fgl_cal_deg": (_i32, [_vp, _i64, _vp, _vp, _i64, _vp]),
    "fgl_sample_workspace_bytes": (_sz, [_i64, _i32]),
    "fgl_sample_node": (_i32, [_vp, _i32, _vp, _i64, _vp, _i64, _vp, _i32, _u64, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fgl_sample_node_static": (_i32, [_vp, _i32, _vp, _i64, _vp, _i64, _vp, _i32, _u64, _u32, _vp, _vp, _vp, _vp, _vp, _vp]),
    "fgl_table_size": (_i64, [_i64, _i32]),
    "fgl_idmap_slots": (_i64, [_i64]),
    "fgl_idmap_table_bytes": (_sz, [_i64]),
    "fgl_idmap_reset": (_i32, [_vp, _i64, _vp]),
    "fgl_idmap_insert_dst": (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp]),
    "fgl_idmap_map_src_workspace_bytes": (_sz, [_i64]),
    "fgl_idmap_map_src": (_i32, [_vp, _i64, _vp, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _i64, _i32, _vp, _vp, _sz, _vp]),
    "fgl_idmap_transfer": (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _i64, _vp, _i64, _i32, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fgl_idmap_lookup": (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _vp]),
    "fgl_wait_words": (_i32, [_vp, _i32, _i32, _vp, _i64]),
    "fgl_sample_blocks_plan": (_i32, [_i64, _i64, _vp, _i32, _vp, _u32, _vp, _vp, _vp, _vp, _vp]),
    "fgl_sample_blocks": (_i32, [_vp, _i32, _vp, _i64, _vp, _i64, _vp, _i32, _vp, _u64, _u32, _vp, _i32, _vp, _i64, _vp, _i64, _vp, _vp, _vp,
                                 _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fgl_block_transpose_workspace_bytes": (_sz, [_i64, _i64, _i32]),
    "fgl_block_transpose": (_i32, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i32, _vp, _sz, _vp]),
    "fgl_block_transpose_batch_workspace_bytes": (_sz, [_i32, _vp, _vp]),
    "fgl_block_transpose_batch": (_i32, [_i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fgl_aggregate": (_i32, [_vp, _vp, _i64, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _i32, _vp, _i64, _vp, _i64,
                             _vp, _i64, _vp]),
    "fgl_aggregate_last_mapping": (C.c_char_p, []),
    "fgl_edge_softmax": (_i32, [_vp, _vp, _i64, _vp, _vp, _vp, _i32, C.c_float, _vp, _vp]),
    "fgl_rmat_keys": (_i32, [_i64, _i64, _i32, _i64, _u64, _vp, _vp]),
}

_lib = None


def build(force: bool = True) -> str:
    """Compile the HIP sources for gfx950 into ``libfastgl_hip.so`` (hipcc cross-compiles
    without a GPU)."""
    args = ["make", "-C", CSRC_DIR, "-j8"]
    if force:
        args.append("-B")
    subprocess.check_call(args)
    return LIB_PATH


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "fastgl: %s is missing -- build it with `make -C %s` (there is no CPU fallback)" % (LIB_PATH, CSRC_DIR))
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        if L.fgl_abi_version() != ABI_VERSION:
            raise RuntimeError("fastgl: ABI version mismatch")
        _lib = L
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise RuntimeError("fastgl: %s (error %d)" % (lib().fgl_last_error().decode(), rc))


def ptr(t):
    """Device pointer of a tensor (or None)."""
    return None if t is None else t.data_ptr()


def stream_handle() -> int:
    return torch.cuda.current_stream().cuda_stream


_workspaces = {}


def workspace(nbytes: int, device) -> torch.Tensor:
    """A scratch buffer of at least nbytes for (device, current stream).  Kernels are
    stream-ordered, so consecutive calls on one stream may share it."""
    key = (torch.device(device).index, stream_handle())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def status_message(bits: int) -> str:
    names = []
    if bits & STATUS_TABLE_FULL:
        names.append("hash table full")
    if bits & STATUS_UNIQ_OVERFLOW:
        names.append("more unique ids than the output holds")
    if bits & STATUS_MISSING_KEY:
        names.append("an id to relabel is not in the map")
    if bits & STATUS_BAD_SEED:
        names.append("a seed id lies outside the graph")
    if bits & STATUS_BAD_ID:
        names.append("a negative id was handed to the id-map")
    return ", ".join(names) or "ok"
