"""``fastgl`` -- MI355X (gfx950) implementation of FastGL's hot path, importable under the
name of the reference's extension module so that ``import fastgl`` in the reference's
sampler and layer code resolves to it.

Operators with the reference's signatures: ``sample_node``, ``transfer_edge_id``, ``cal_deg``,
``exclusive_sum``, ``forward_gcn``, ``backward_gcn``, ``forwaed_gin`` (sic), ``backward_gin``,
``forward_gat``, ``backward_gat``.
Everything runs in hand-written HIP kernels behind ``libfastgl_hip.so``; there is no CPU path.
"""
from ._lib import LIB_PATH, build, lib  # noqa: F401
from .ops import (  # noqa: F401
    BlocksPlan,
    aggregate,
    backward_gat,
    backward_gcn,
    backward_gin,
    block_transpose,
    block_transpose_batch,
    cal_deg,
    edge_softmax,
    exclusive_sum,
    forwaed_gin,
    forward_gat,
    forward_gcn,
    manual_seed,
    rmat_keys,
    sample_blocks_fused,
    sample_node,
    table_size,
    transfer_edge_id,
)
from .sampler import Block, DataLoader, FusedMapSampler, PendingBatch, transpose_blocks  # noqa: F401
from .conv import (  # noqa: F401
    GAT,
    GCN,
    GIN,
    SAGE,
    GATConv,
    GCNConv,
    GINConv,
    MA_Function,
    MA_Function_GAT,
    MA_Function_GIN,
    MA_Function_Mean,
    SAGEConv,
    edge_softmax_torch,
)
from . import graph  # noqa: F401
