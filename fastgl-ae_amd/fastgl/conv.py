"""GNN layers over the memory-aware aggregation operators, with the class names, call
signatures and autograd wiring of the reference's GraphConv.py (MA_Function, GCNConv, GCN,
MA_Function_GIN, GINConv, GIN, MA_Function_GAT, GATConv, GAT; GraphConv.py:19-312), plus a mean
aggregator (GraphSAGE), which the reference's benchmark configurations name but its kernels do
not provide.

The reference's quirks are kept where they define results: weights are drawn from
U(-1/sqrt(out), 1/sqrt(out)) (GraphConv.py:52-55), dropout sits between layers, no activation
is applied by GCN / GIN (the ``activation`` argument is ignored, GraphConv.py:69,86-99), the
backward of GCN receives (dst_norm, src_norm) in the slots the extension calls
(src_norm_degs, dst_norm_degs) (GraphConv.py:37), and destination rows without edges pass
their input through in the forward pass and receive no gradient from it.
"""
from __future__ import annotations

import math

import torch
from torch import nn

from . import ops
from .sampler import Block


def _transposed(t, edge_ids=False):
    """The transposed block behind the ``transposed`` argument of the autograd functions: either the tuple
    itself or a ``Block``, whose transpose is built here, on first use in a backward pass."""
    if isinstance(t, Block):
        return t.transposed(edge_ids=True) if edge_ids else t.transposed()
    return t


def _block_csr(graph):
    """(edge_ptr, src_edges, raw_dst_degs) of a block.  A ``Block`` carries its CSR; any other
    object with ``edges()`` goes through cal_deg + exclusive_sum like GraphConv.py:93-98."""
    dst_nodes = graph.num_dst_nodes()
    if isinstance(graph, Block):
        return graph.edge_ptr, graph.src_local, graph.in_degrees()
    raw = ops.cal_deg(graph.edges()[1].int(), dst_nodes)
    return ops.exclusive_sum(raw), graph.edges()[0].int(), raw


def _aggregate_first_is_cheaper(n_src, n_dst, n_edges, d_in, d_out):
    """(A X) W against A (X W): the product runs over n_dst rows instead of n_src, the gather moves rows of
    d_in instead of d_out columns.  Priced with round figures for this GPU (fp32 matrix product ~50 TFLOP/s,
    random row gather ~5 TB/s); the two orders agree up to fp32 rounding."""
    flop_s, byte_s = 50e12, 5e12
    product_first = 2.0 * n_src * d_in * d_out / flop_s + 4.0 * n_edges * d_out / byte_s
    gather_first = 2.0 * n_dst * d_in * d_out / flop_s + 4.0 * n_edges * d_in / byte_s
    return gather_first < product_first


class MA_Function(torch.autograd.Function):
    """GCN layer ``A_norm X W``.  The reference multiplies first and gathers rows of ``X W``
    (aggregate_acc.cpp:133-160); a sampled block has several times more source than destination rows, so
    for most layers it is cheaper to gather rows of ``X`` and multiply the (fewer) gathered rows --
    ``order="auto"`` (default) prices both and picks; ``"product_first"`` is the reference's order.  Either
    way a destination row without edges passes ``(X W)[d]`` through and sends no gradient back
    (aggregate_acc_kernel.cu:307-309,498-500)."""

    @staticmethod
    def forward(ctx, edge_ptr, src_edges, src_norm_degs, dst_norm_degs, dst_nodes, input_feat, weight, neighbor_num,
                transposed=None, order="auto"):
        ctx.transposed = transposed
        n_dst = int(dst_nodes)
        gather_first = order == "gather_first" or (order == "auto" and _aggregate_first_is_cheaper(
            input_feat.size(0), n_dst, src_edges.numel(), weight.size(0), weight.size(1)))
        ctx.gather_first = gather_first
        if not gather_first:
            ctx.save_for_backward(edge_ptr, src_edges, src_norm_degs, dst_norm_degs, weight, input_feat)
            return ops.forward_gcn(edge_ptr, src_edges, src_norm_degs, dst_norm_degs, input_feat, weight, neighbor_num,
                                   dst_nodes)[0]
        ax = ops.aggregate(edge_ptr, src_edges, input_feat, mode="gcn", zero_policy="self", row_norm=dst_norm_degs,
                           col_norm=src_norm_degs, n_rows=n_dst, longest_row=ops._fanout_bound(edge_ptr, neighbor_num))
        ctx.n_src = int(input_feat.size(0))
        ctx.save_for_backward(edge_ptr, src_edges, src_norm_degs, dst_norm_degs, weight, ax)
        return torch.mm(ax, weight)

    @staticmethod
    def backward(ctx, d_input):
        d_input = d_input.contiguous()
        if ctx.gather_first:
            edge_ptr, src_edges, src_norm_degs, dst_norm_degs, weight, ax = ctx.saved_tensors
            # rows without edges took no part in the sum: no gradient through them (as in the reference)
            has_edges = (edge_ptr[1:] != edge_ptr[:-1]).to(d_input.dtype)[:, None]
            d_out = d_input * has_edges
            d_w = torch.mm(ax.transpose(0, 1), d_out)
            d_x = None
            if ctx.needs_input_grad[5]:
                d_ax = torch.mm(d_out, weight.transpose(0, 1))
                if ctx.transposed is None:
                    t_ptr, t_idx = ops.block_transpose(edge_ptr, src_edges, int(d_input.size(0)), ctx.n_src)
                else:
                    t_ptr, t_idx = _transposed(ctx.transposed)
                d_x = ops.aggregate(t_ptr, t_idx, d_ax, mode="gcn", zero_policy="zeros", row_norm=src_norm_degs,
                                    col_norm=dst_norm_degs, n_rows=ctx.n_src)
            return None, None, None, None, None, d_x, d_w, None, None, None
        edge_ptr, src_edges, src_norm_degs, dst_norm_degs, weight, input_feat = ctx.saved_tensors
        if ctx.transposed is None:
            d_x, d_w = ops.backward_gcn(edge_ptr, src_edges, dst_norm_degs, src_norm_degs, d_input, weight, input_feat)
        elif not ctx.needs_input_grad[5]:
            # the first layer: nobody wants d_x, and d_w = X^T (A^T d_out) = (A X)^T d_out needs no transposed
            # block -- one more forward-direction gather (rows without edges contribute nothing, as in the
            # reference's backward kernel, aggregate_acc_kernel.cu:498-500)
            ax = ops.aggregate(edge_ptr, src_edges, input_feat, mode="gcn", zero_policy="zeros", row_norm=dst_norm_degs,
                               col_norm=src_norm_degs, n_rows=int(d_input.size(0)))
            d_x, d_w = None, torch.mm(ax.transpose(0, 1), d_input)
        else:  # same arithmetic as backward_gcn, with the block's cached transpose
            t_ptr, t_idx = _transposed(ctx.transposed)
            g = ops.aggregate(t_ptr, t_idx, d_input, mode="gcn", zero_policy="zeros", row_norm=src_norm_degs,
                              col_norm=dst_norm_degs, n_rows=int(input_feat.size(0)))
            d_x = torch.mm(g, weight.transpose(0, 1))
            d_w = torch.mm(input_feat.transpose(0, 1), g)
        return None, None, None, None, None, d_x, d_w, None, None, None


class _Conv(nn.Module):
    def __init__(self, input_dim, output_dim, weight=False):
        super().__init__()
        if weight:
            self.weights = nn.Parameter(torch.randn(input_dim, output_dim))
        else:
            self.weights = self.register_parameter('weight', None)
        self.reset_parameters()

    def reset_parameters(self):
        if self.weights is not None:
            stdv = 1. / math.sqrt(self.weights.size(1))
            self.weights.data.uniform_(-stdv, stdv)

    def _weight(self):
        if self.weights is None:
            raise RuntimeError("layer was built with weight=False")
        return self.weights


class GCNConv(_Conv):
    order = "auto"  # "product_first": the reference's order of product and gather in every layer (see MA_Function)

    def forward(self, edge_ptr, src_edges, src_norm_degs, dst_norm_degs, dst_nodes, input_feat, neighbor_num,
                transposed=None):
        return MA_Function.apply(edge_ptr, src_edges, src_norm_degs, dst_norm_degs, dst_nodes, input_feat,
                                 self._weight(), neighbor_num, transposed, self.order)


def _stack(conv, in_feats, n_hidden, n_classes, n_layers, weight):
    layers = nn.ModuleList()
    layers.append(conv(in_feats, n_hidden, weight=weight))
    for _ in range(1, n_layers - 1):
        layers.append(conv(n_hidden, n_hidden, weight=weight))
    layers.append(conv(n_hidden, n_classes, weight=weight))
    return layers


class GCN(nn.Module):
    def __init__(self, in_feats, n_hidden, n_classes, n_layers, activation, weight, dropout):
        super().__init__()
        self.layers = _stack(GCNConv, in_feats, n_hidden, n_classes, n_layers, weight)
        self.dropout = nn.Dropout(p=dropout)

    def forward(self, blocks, features, neighbor_list=[5, 10, 15]):
        h = features
        for i, layer in enumerate(self.layers):
            if i != 0:
                h = self.dropout(h)
            graph = blocks[i]
            dst_nodes = graph.num_dst_nodes()
            edge_ptr, src_edges, raw_dst_norm_degs = _block_csr(graph)
            if isinstance(graph, Block):
                src_norm_degs = graph.out_degrees().clamp(min=1)
                transposed = graph if torch.is_grad_enabled() else None  # transposed on demand, in backward
            else:
                src_norm_degs = ops.cal_deg(src_edges, graph.num_src_nodes()).clamp(min=1)
                transposed = None
            dst_norm_degs = raw_dst_norm_degs.clamp(min=1)
            h = layer(edge_ptr, src_edges, src_norm_degs, dst_norm_degs, dst_nodes, h, neighbor_list[i], transposed)
        return h


class MA_Function_GIN(torch.autograd.Function):
    @staticmethod
    def forward(ctx, edge_ptr, src_edges, dst_nodes, input_feat, weight, neighbor_num, transposed=None):
        X_prime, tmp = ops.forwaed_gin(edge_ptr, src_edges, input_feat, weight, neighbor_num, dst_nodes)
        ctx.src_nodes = input_feat.size(0)
        ctx.neighbor_num = neighbor_num
        ctx.transposed = transposed
        ctx.save_for_backward(edge_ptr, src_edges, weight, tmp)
        return X_prime

    @staticmethod
    def backward(ctx, d_input):
        edge_ptr, src_edges, weight, tmp = ctx.saved_tensors
        d_input = d_input.contiguous()
        if ctx.transposed is None:
            d_x, d_w = ops.backward_gin(edge_ptr, src_edges, d_input, weight, tmp, ctx.src_nodes)
        else:
            d_w = torch.mm(tmp.transpose(0, 1), d_input)
            d_x = None
            if ctx.needs_input_grad[3]:  # not for the first layer: its transposed block is never built
                t_ptr, t_idx = _transposed(ctx.transposed)
                d_tmp = torch.mm(d_input, weight.transpose(0, 1))
                d_x = ops.aggregate(t_ptr, t_idx, d_tmp, mode="sum", zero_policy="zeros", n_rows=int(ctx.src_nodes))
        return None, None, None, d_x, d_w, None, None


class GINConv(_Conv):
    def forward(self, edge_ptr, src_edges, dst_nodes, input_feat, neighbor_num, transposed=None):
        return MA_Function_GIN.apply(edge_ptr, src_edges, dst_nodes, input_feat, self._weight(), neighbor_num, transposed)


class GIN(nn.Module):
    def __init__(self, in_feats, n_hidden, n_classes, n_layers, activation, weight, dropout):
        super().__init__()
        self.layers = _stack(GINConv, in_feats, n_hidden, n_classes, n_layers, weight)
        self.dropout = nn.Dropout(p=dropout)

    def forward(self, blocks, features, neighbor_list=[5, 10, 15]):
        h = features
        for i, layer in enumerate(self.layers):
            if i != 0:
                h = self.dropout(h)
            graph = blocks[i]
            dst_nodes = graph.num_dst_nodes()
            edge_ptr, src_edges, _ = _block_csr(graph)
            transposed = graph if isinstance(graph, Block) and torch.is_grad_enabled() else None
            h = layer(edge_ptr, src_edges, dst_nodes, h, neighbor_list[i], transposed)
        return h


# ---------------------------------------------------------------------------------------
# attention-weighted aggregation (GAT; GraphConv.py:198-312)
# ---------------------------------------------------------------------------------------
class MA_Function_GAT(torch.autograd.Function):
    @staticmethod
    def forward(ctx, edge_ptr, edge_data, src_edges, dst_edges, dst_nodes, input_feat, num_heads, neighbor_num,
                transposed=None):
        X_prime = ops.forward_gat(edge_ptr, edge_data, src_edges, input_feat, neighbor_num, dst_nodes, num_heads)[0]
        ctx.src_nodes = input_feat.size(0)
        ctx.num_heads = num_heads
        ctx.neighbor_num = neighbor_num
        ctx.transposed = transposed
        ctx.save_for_backward(edge_ptr, edge_data, src_edges, dst_edges, input_feat)
        return X_prime

    @staticmethod
    def backward(ctx, d_input):
        edge_ptr, edge_data, src_edges, dst_edges, input_feat = ctx.saved_tensors
        d_input = d_input.contiguous()
        if ctx.transposed is None:
            d_x = ops.backward_gat(edge_ptr, edge_data, src_edges, d_input, ctx.src_nodes, ctx.num_heads)[0]
        elif not ctx.needs_input_grad[5]:
            d_x = None
        else:
            t_ptr, t_idx, t_edge = _transposed(ctx.transposed, edge_ids=True)
            d_x = ops.aggregate(t_ptr, t_idx, d_input, mode="edge", zero_policy="zeros", n_rows=int(ctx.src_nodes),
                                edge_weight=edge_data, n_heads=int(ctx.num_heads), edge_index=t_edge)
        # as in the reference (GraphConv.py:227) the attention weights receive no gradient from here
        return None, None, None, None, None, d_x, None, None, None


def edge_softmax_torch(edge_ptr, dst_edges, e, n_dst):
    """softmax of the edge scores ``e`` [E, H] over the edges of each destination (what the reference
    takes from dgl.nn.functional.edge_softmax, GraphConv.py:272), written with torch operators: the plain
    fp32 restatement that ``ops.edge_softmax`` (one HIP launch, used by ``GATConv``) is tested against."""
    idx = dst_edges.long()
    top = torch.full((n_dst, e.size(1)), float("-inf"), dtype=e.dtype, device=e.device)
    top = top.scatter_reduce(0, idx[:, None].expand(-1, e.size(1)), e, reduce="amax", include_self=True)
    ex = torch.exp(e - top.index_select(0, idx))
    den = torch.zeros_like(top).index_add_(0, idx, ex)
    return ex / den.index_select(0, idx)


class GATConv(nn.Module):
    def __init__(self, input_dim, output_dim, num_heads, feat_drop=0, attn_drop=0, negative_slope=0.2):
        super().__init__()
        self.out_feats = output_dim
        self.num_heads = num_heads
        self.fc = nn.Linear(input_dim, output_dim * num_heads, bias=False)
        self.attn_l = nn.Parameter(torch.empty(1, num_heads, output_dim))
        self.attn_r = nn.Parameter(torch.empty(1, num_heads, output_dim))
        self.feat_drop = nn.Dropout(feat_drop)
        self.attn_drop = nn.Dropout(attn_drop)
        self.leaky_relu = nn.LeakyReLU(negative_slope)
        self.reset_parameters()

    def reset_parameters(self):
        gain = nn.init.calculate_gain('relu')
        nn.init.xavier_normal_(self.fc.weight, gain=gain)
        nn.init.xavier_normal_(self.attn_l, gain=gain)
        nn.init.xavier_normal_(self.attn_r, gain=gain)

    def forward(self, graph, input_feat, neighbor_num):
        dst_nodes = graph.num_dst_nodes()
        feat_src = self.fc(input_feat).view(-1, self.num_heads, self.out_feats)
        feat_dst = feat_src[:dst_nodes]
        el = (feat_src * self.attn_l).sum(dim=-1)  # [n_src, H]
        er = (feat_dst * self.attn_r).sum(dim=-1)  # [n_dst, H]
        edge_ptr, src_edges, _ = _block_csr(graph)
        # u_add_v + leaky_relu + edge_softmax (DGL calls in the reference, GraphConv.py:265-272) in one launch.
        # No gradient reaches the coefficients (the aggregation's backward returns none for them, as in the
        # reference, GraphConv.py:227), so they are computed outside the autograd graph.
        with torch.no_grad():
            alpha = ops.edge_softmax(edge_ptr, src_edges, el.detach().contiguous(), er.detach().contiguous(),
                                     self.leaky_relu.negative_slope, n_rows=dst_nodes)
            edge_data = self.attn_drop(alpha).contiguous()
        feat_src = feat_src.reshape(-1, self.out_feats * self.num_heads)
        transposed = graph if isinstance(graph, Block) and torch.is_grad_enabled() else None
        return MA_Function_GAT.apply(edge_ptr, edge_data, src_edges, None, dst_nodes, feat_src, self.num_heads,
                                     neighbor_num, transposed)


class GAT(nn.Module):
    def __init__(self, in_feats, n_hidden, n_classes, n_layers, activation, dropout, heads=8):
        super().__init__()
        self.layers = nn.ModuleList()
        self.layers.append(GATConv(in_feats, n_hidden, num_heads=heads))
        for _ in range(1, n_layers - 1):
            self.layers.append(GATConv(n_hidden * heads, n_hidden, num_heads=heads, feat_drop=dropout))
        self.layers.append(GATConv(n_hidden * heads, n_classes, num_heads=1, feat_drop=dropout))
        self.dropout = nn.Dropout(p=dropout)

    def forward(self, blocks, features, neighbor_list=[5, 10, 15]):
        h = features
        for i, layer in enumerate(self.layers):
            h = layer(blocks[i], h, neighbor_list[i])
        return h


# ---------------------------------------------------------------------------------------
# mean aggregation (GraphSAGE-mean)
# ---------------------------------------------------------------------------------------
class MA_Function_Mean(torch.autograd.Function):
    """``out[d] = mean of feat[src] over the edges into d`` (zeros if there are none).
    ``indices`` may hold block-local ids (``feat`` = the block's source rows) or graph ids
    (``feat`` = the whole resident feature table: the input-row gather fused into the first
    layer).  The gradient w.r.t. ``feat`` is produced only in the block-local form."""

    @staticmethod
    def forward(ctx, block, feat, use_global):
        indices = block.src_global if use_global else block.src_local
        ctx.block = block
        ctx.use_global = use_global
        ctx.n_src = block.num_src_nodes()
        return ops.aggregate(block.edge_ptr, indices, feat, mode="mean", zero_policy="zeros", n_rows=block.num_dst_nodes())

    @staticmethod
    def backward(ctx, d_out):
        if ctx.use_global or not ctx.needs_input_grad[1]:
            return None, None, None
        block = ctx.block
        t_ptr, t_idx = block.transposed()
        # (the destination rows' entry counts are the differences of the block's own row pointer: no degree array)
        d_feat = ops.aggregate(t_ptr, t_idx, d_out.contiguous(), mode="colmean_ptr", zero_policy="zeros",
                               col_norm=block.edge_ptr, n_rows=ctx.n_src)
        return None, d_feat, None


class SAGEConv(nn.Module):
    """``h_dst W_self + mean(h_src) W_neigh + b`` (the mean aggregator of GraphSAGE)."""

    def __init__(self, input_dim, output_dim, bias=True):
        super().__init__()
        self.fc_self = nn.Linear(input_dim, output_dim, bias=False)
        self.fc_neigh = nn.Linear(input_dim, output_dim, bias=bias)

    def forward(self, block, feat_src, feat_dst=None, use_global=False):
        h_neigh = MA_Function_Mean.apply(block, feat_src, use_global)
        if feat_dst is None:
            feat_dst = feat_src[:block.num_dst_nodes()]
        return self.fc_self(feat_dst) + self.fc_neigh(h_neigh)


class SAGE(nn.Module):
    def __init__(self, in_feats, n_hidden, n_classes, n_layers, activation=torch.relu, dropout=0.0):
        super().__init__()
        dims = [in_feats] + [n_hidden] * (n_layers - 1) + [n_classes]
        self.layers = nn.ModuleList(SAGEConv(dims[i], dims[i + 1]) for i in range(n_layers))
        self.activation = activation
        self.dropout = nn.Dropout(p=dropout)

    def forward(self, blocks, features, input_nodes=None):
        """``features``: the rows of the input nodes, or -- with ``input_nodes`` given -- the
        whole feature table, in which case the first layer gathers straight from it."""
        h = features
        for i, (layer, block) in enumerate(zip(self.layers, blocks)):
            if i == 0 and input_nodes is not None:
                if block.src_global is None:
                    raise RuntimeError("the outermost block does not carry graph ids")
                dst_ids = input_nodes[:block.num_dst_nodes()].long()
                h = layer(block, features, feat_dst=features.index_select(0, dst_ids), use_global=True)
            else:
                h = layer(block, h)
            if i != len(self.layers) - 1:
                if self.activation is not None:
                    h = self.activation(h)
                h = self.dropout(h)
        return h
