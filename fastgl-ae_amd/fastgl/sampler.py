"""Mini-batch block sampler with the interface of the reference's ``FusedMapSampler``
(FusedMapSampler.py:27-109) -- same constructor arguments, same attributes the trainer
fills in (``edge_src``, ``edge_dst``, ``edge_ptr``, ``nodes_num``; train_fastgl.py:240-244),
same ``sample_blocks(g, seed_nodes) -> (input_nodes, output_nodes, blocks)`` -- without DGL:
a block is the light ``Block`` below instead of a ``DGLBlock``.

Two paths produce identical blocks:
  * ``fused=True`` (default): all hops in one enqueue of the C ABI's ``fgl_sample_blocks``;
    one host read-back per mini-batch;
  * ``fused=False``: the reference's per-hop loop, call for call, through the drop-in
    operators ``sample_node`` and ``transfer_edge_id``.
"""
from __future__ import annotations

import collections
import itertools

import torch

from . import ops


class Block:
    """One hop of a sampled mini-batch: a bipartite graph from ``n_src`` source nodes to
    ``n_dst`` destination nodes (the first ``n_dst`` source nodes *are* the destination
    nodes), stored as a CSR over destination rows: ``edge_ptr`` int32[n_dst+1],
    ``src_local`` int32[E].  ``src_global`` (optional) holds the same edges with graph ids."""

    def __init__(self, edge_ptr, src_local, n_src, n_dst, src_global=None, sorted_transpose=False):
        self.sorted_transpose = bool(sorted_transpose)  # deterministic order inside the transposed lists
        self.edge_ptr = edge_ptr
        self.src_local = src_local
        self._n_src = int(n_src)
        self._n_dst = int(n_dst)
        self.src_global = src_global
        self._dst_local = None
        self._transposed = None
        self._src_deg = None
        self._in_deg = None

    # -- the part of the DGLBlock interface that the reference's model code uses -------------
    def num_src_nodes(self):
        return self._n_src

    def num_dst_nodes(self):
        return self._n_dst

    def num_edges(self):
        return int(self.src_local.numel())

    def edges(self):
        """``(src_local, dst_local)`` as COO, grouped by destination in row order."""
        if self._dst_local is None:
            deg = (self.edge_ptr[1:] - self.edge_ptr[:-1]).long()
            rows = torch.arange(self._n_dst, device=self.edge_ptr.device, dtype=torch.int32)
            self._dst_local = torch.repeat_interleave(rows, deg, output_size=self.num_edges())
        return self.src_local, self._dst_local

    def int(self):
        return self

    def to(self, device):
        # a device without an index ("cuda") means the current device of that type
        want, have = torch.device(device), self.edge_ptr.device
        same = want.type == have.type
        if same and have.type == "cuda":
            same = (torch.cuda.current_device() if want.index is None else want.index) == have.index
        if not same:
            raise RuntimeError("Block.to: blocks live on the device they were sampled on")
        return self

    # -- what this library adds ---------------------------------------------------------
    def in_degrees(self):
        if self._in_deg is None:
            self._in_deg = self.edge_ptr[1:] - self.edge_ptr[:-1]
        return self._in_deg

    def out_degrees(self):
        if self._src_deg is None:
            if self._transposed is not None:  # the transposed block's row lengths: no histogram pass
                t_ptr = self._transposed[0]
                self._src_deg = t_ptr[1:] - t_ptr[:-1]
            else:
                self._src_deg = ops.cal_deg(self.src_local, self._n_src)
        return self._src_deg

    def transposed(self, edge_ids=False):
        """``(t_ptr int32[n_src+1], t_dst int32[E])``: for each source node the destination
        rows it feeds (built on first use, kept for the backward pass); with ``edge_ids=True``
        also ``t_edge int32[E]``, the position of every transposed entry in ``src_local``."""
        if self._transposed is None:
            self._transposed = ops.block_transpose(self.edge_ptr, self.src_local, self._n_dst, self._n_src, edge_ids=True,
                                                   sorted_rows=self.sorted_transpose)
        return self._transposed if edge_ids else self._transposed[:2]

    def clone(self):
        """A copy that owns its memory (a block of a graph-replaying sampler lives in a slot that a later
        mini-batch overwrites)."""
        edge_ptr = self.edge_ptr.clone()
        if hasattr(self.edge_ptr, "fgl_longest_row"):
            edge_ptr.fgl_longest_row = self.edge_ptr.fgl_longest_row
        return Block(edge_ptr, self.src_local.clone(), self._n_src, self._n_dst,
                     None if self.src_global is None else self.src_global.clone(), sorted_transpose=self.sorted_transpose)

    def __repr__(self):
        return "Block(num_src_nodes=%d, num_dst_nodes=%d, num_edges=%d)" % (self._n_src, self._n_dst, self.num_edges())


def transpose_blocks(blocks):
    """Builds the transposed form (``Block.transposed()``) of every block of the list that does not have it yet, all
    in the five launches that one block takes: the inner blocks of a mini-batch are small and their transposes are
    launch-bound one by one.  Call it before a backward pass that will want them (every layer but the first).
    Blocks of a ``deterministic=True`` sampler are transposed one by one (ordered lists)."""
    todo = [b for b in blocks if b._transposed is None and not b.sorted_transpose]
    for b in blocks:
        if b._transposed is None and b.sorted_transpose:
            b.transposed()
    if todo:
        res = ops.block_transpose_batch([(b.edge_ptr, b.src_local, b._n_dst, b._n_src) for b in todo], edge_ids=True)
        for b, r in zip(todo, res):
            b._transposed = r


class _ShapeState:
    """What the sampler has learned about mini-batches of one shape (seed count, fanouts, graph size, device)."""

    def __init__(self):
        self.plans = {}         # node-capacity tuple (None = worst case) -> BlocksPlan
        self.nodes_seen = None  # per hop: the node counts that the buffer sizes are derived from
        self.graphs = None      # (plan, table slots) -> captured launch sequences, see FusedMapSampler._replay
        self.graph_turn = 0     # which of them is next


class _HostCounts:
    """Pinned host words that the kernels of a mini-batch write its sizes into (``readback`` of
    ``ops.sample_blocks_fused``).  A sampler keeps a few and hands them out in turn; one that is still waiting to be
    read is never handed out again."""
    PENDING = -1  # no count and no status word is all ones

    def __init__(self, n_words):
        self.words = torch.empty(n_words, dtype=torch.int32, pin_memory=True)
        self.busy = False
        self.abandoned = False  # handed out, never read: its kernels may still be about to write
        self.stream = None

    def expect(self, stream):
        """Before the call is enqueued on ``stream``: every word pending."""
        self.words.fill_(self.PENDING)
        self.stream = stream
        return self.words

    def read(self):
        """Waits until the kernels have overwritten every word -- the launch that makes the last count final does so
        when it starts, so this returns while that launch is still running, without the wake-up of a stream wait
        (bounded: after a few milliseconds the stream is waited for instead) -- and returns them as a list."""
        ops.L.check(ops.L.lib().fgl_wait_words(self.words.data_ptr(), int(self.words.numel()), self.PENDING,
                                               self.stream.cuda_stream, 5000))
        values = self.words.tolist()
        self.busy = False
        return values


class PendingBatch:
    """A mini-batch whose kernels are enqueued and whose sizes are still on the device
    (``FusedMapSampler.begin_sample``).  The sampling kernels store the sizes into pinned host memory themselves as
    soon as the last of them is final; ``finish`` waits for those words, whatever the caller enqueues in the meantime."""

    def __init__(self, sampler, pending):
        self._sampler, self._pending = sampler, pending
        _, bptr, _, src_g, counts, _ = pending["out"]
        H = len(sampler.fanouts)
        self.outer_edge_ptr = bptr[H - 1]        # int32[bound + 1]: row offsets of the outermost block
        self.outer_src_global = src_g[H - 1]     # int32[edge bound]: its neighbour lists in graph ids
        self.outer_n_dst = counts[H - 1:H]       # int32[1] on the device: its actual row count
        self.outer_n_dst_bound = int(bptr[H - 1].numel()) - 1
        self.outer_fanout = int(sampler.fanouts[0])
        self.redone = False

    def __del__(self):
        # a batch that was begun and dropped: its kernels may still be about to write its host words, so the sampler
        # waits for them before it hands the words out again
        try:
            host = self._pending["host"]
            if host.busy:
                host.abandoned = True
        except Exception:  # noqa: BLE001 -- interpreter shutdown
            pass

    def finish(self):
        """The second half: wait for the sizes, then ``(input_nodes, output_nodes, blocks)`` as ``sample_blocks``
        returns them.  ``redone`` is set if the batch outgrew its buffers and was sampled again with larger
        ones -- anything computed from the ``outer_*`` arrays before is then void (it read valid memory, the
        kernels never leave their bounds)."""
        outer_ptr = self.outer_edge_ptr.data_ptr()
        result = self._sampler._finish_fused(self._pending, self._pending["host"].read())
        self.redone = result[2][0].edge_ptr.data_ptr() != outer_ptr
        return result


class FusedMapSampler:
    def __init__(self, fanouts, edge_dir='in', prob=None, mask=None, replace=False, prefetch_node_feats=None,
                 prefetch_labels=None, prefetch_edge_feats=None, output_device=None, fused=True, rng_seed=0,
                 id_order="first", deterministic=False, graph_slots=0, transposed="inner"):
        if mask is not None and prob is not None:
            raise ValueError('Mask and probability arguments are mutually exclusive. '
                             'Consider multiplying the probability with the mask to achieve the same goal.')
        if prob is not None or mask is not None:
            raise NotImplementedError("weighted / masked sampling is not part of this library")
        if edge_dir != 'in':
            raise NotImplementedError("only in-neighbour sampling (edge_dir='in'), as in the reference")
        if replace:
            raise NotImplementedError("sampling is without replacement")
        self.fanouts = list(fanouts)
        self.edge_dir = edge_dir
        self.replace = replace
        self.output_device = output_device
        self.fused = fused
        if id_order not in ("first", "arrival"):
            raise ValueError("id_order must be 'first' or 'arrival'")
        self.id_order = id_order  # numbering of new node ids (fused path): see ops.sample_blocks_fused
        # deterministic=True also fixes the order inside each block's transposed lists, so that the
        # fp32 sums of the backward pass are reproducible bit for bit (one more launch per mini-batch for the transposed
        # blocks that the sampling call builds, a stable sort for those built on demand)
        self.deterministic = bool(deterministic)
        if self.deterministic and id_order != "first":
            raise ValueError("deterministic=True needs id_order='first'")
        # graph_slots = R > 0: the fused path's launch sequence (26 kernels for three hops) is captured once in a
        # HIP graph per output slot and replayed, which takes the host's launch cost out of the small hops.  It
        # pays off where the GPU would otherwise wait for the host -- one mini-batch at a time from an idle GPU:
        # -11 % at batch 8192, -26 % at batch 1024 -- and not in a loop that keeps the GPU busy, where the launches
        # are hidden behind the previous step's kernels anyway.  The price: outputs live in R fixed slots used in
        # turn, so the tensors of a mini-batch are overwritten when the R-th mini-batch after it is sampled (with
        # iter_batches: the R-th after it on the same lane, i.e. R * prefetch mini-batches later) -- consume (or
        # clone) them before that.
        # transposed: which blocks come with their transposed form (what the backward pass of a layer gathers over),
        # built inside the fused sampling call at next to no cost: "inner" = every block but the outermost (the first
        # layer's input needs no gradient), "all", or "none" (built on demand, Block.transposed()).  A deterministic
        # sampler has the call sort their rows as well (one more launch); blocks whose transposed form is built on
        # demand get theirs from a stable sort.
        if transposed not in ("inner", "all", "none"):
            raise ValueError("transposed must be 'inner', 'all' or 'none'")
        self.transposed = transposed
        self.graph_slots = int(graph_slots)
        if self.graph_slots < 0 or self.graph_slots == 1:
            raise ValueError("graph_slots must be 0 (off) or at least 2")
        self.rng_seed = int(rng_seed)
        self.batches = 0
        self.nodes_num = 0
        self.edge_src = None  # CSR indices (source id of every edge, edges sorted by destination)
        self.edge_dst = None  # unused by the kernels; kept because the reference's trainer sets it
        self.edge_ptr = None  # CSR indptr (int32 or int64)
        self.output_nodes = None
        self._states = {}       # shape of a mini-batch -> _ShapeState
        self._lanes = []         # streams of iter_batches, one per mini-batch in flight
        self._lane_events = []   # per lane: recorded behind the lane's latest mini-batch
        self._host_counts = {}   # word count -> pinned words for the per-batch size read-back, handed out in turn (_HostCounts)
        self._host_turn = 0

    def set_graph(self, edge_ptr, edge_src, nodes_num=None, edge_dst=None):
        self.edge_ptr, self.edge_src, self.edge_dst = edge_ptr, edge_src, edge_dst
        self.nodes_num = int(edge_ptr.numel()) - 1 if nodes_num is None else int(nodes_num)
        return self

    # -------------------------------------------------------------------------------------
    def sample_blocks(self, g, seed_nodes, exclude_eids=None):
        """``-> (input_nodes, output_nodes, blocks)``; ``blocks[0]`` is the outermost hop and
        was sampled with ``fanouts[0]`` (seeds are expanded with ``fanouts[-1]`` first,
        FusedMapSampler.py:72).  ``g`` is ignored, as in the reference (train_fastgl.py:245-246)."""
        if self.edge_ptr is None or self.edge_src is None:
            raise RuntimeError("FusedMapSampler: edge_ptr / edge_src are not set")
        self.output_nodes = seed_nodes
        seeds = seed_nodes.to(device=self.edge_src.device, dtype=torch.int32).contiguous()
        stream_base = (self.batches * 64) & 0xFFFFFFFF
        self.batches += 1
        if self.fused:
            return self._sample_fused(seeds, stream_base)
        return self._sample_layerwise(seeds, stream_base)

    # -- fused path: enqueue (no host synchronisation) / finish (one read-back) -----------------
    @staticmethod
    def _caps(state, n_seeds):
        # Worst-case bounds assume that no neighbour ever repeats: 8.6 M nodes for 8192 seeds and
        # fanouts 5/10/15 where real batches hold ~1 M, and the whole graph for deep fanouts.  A hash
        # table that fits the caches is much faster and output buffers sized by the bound cost GBs,
        # so after the first batch both are sized from the largest batch seen (x1.5, table load <=
        # 1/4).  A batch that outgrows them is detected by the kernels (status word) and simply
        # redone with the worst-case plan; results do not depend on the sizes.
        if state.nodes_seen is None:
            return None
        return tuple(max(n_seeds, -(-int(1.5 * n) // 4096) * 4096) for n in state.nodes_seen)

    def _state_for(self, seeds, lane=0):
        # Plans, learned buffer sizes and captured graphs are kept per shape: the short last batch of an epoch gets
        # an entry of its own and does not throw away what the full-size batches have learned.  Mini-batches that are
        # in flight together (iter_batches: one lane per stream) each need a table and scratch of their own: the
        # lane is part of the key.
        shape = (int(seeds.numel()), tuple(reversed(self.fanouts)), self.nodes_num, seeds.device, lane)
        state = self._states.get(shape)
        if state is None:
            if sum(1 for k in self._states if k[-1] == lane) >= 4:  # (ever-changing batch sizes: forget the lane's oldest shape)
                self._states.pop(next(k for k in self._states if k[-1] == lane))
            state = self._states[shape] = _ShapeState()
            first = self._states.get(shape[:-1] + (0,))
            if first is not None and first.nodes_seen is not None:  # (what the first lane has learned about this shape)
                state.nodes_seen = list(first.nodes_seen)
        return state

    def _launch_fused(self, seeds, stream_base, worst_case=False, state=None, lane=0, stream=None):
        """stream: enqueue on this stream instead of the current one (eager path only); the outputs are allocated on
        the current stream all the same."""
        hop_fanouts = list(reversed(self.fanouts))
        lib = ops.L.lib()
        n_seeds = int(seeds.numel())
        if state is None:
            state = self._state_for(seeds, lane)
        caps = None if worst_case else self._caps(state, n_seeds)
        plan = state.plans.get(caps)
        if plan is None:
            n_hops = len(hop_fanouts)
            hops = {"inner": range(n_hops - 1), "all": range(n_hops), "none": ()}[self.transposed]
            # (table and scratch belong to the stream that the kernels run on: when a plan is dropped, its memory
            # must not reach allocations of another stream while that one may still be using it)
            with torch.cuda.stream(stream if stream is not None else torch.cuda.current_stream(seeds.device)):
                plan = ops.BlocksPlan(self.nodes_num, n_seeds, hop_fanouts, seeds.device, node_capacity=caps, transpose_hops=hops)
            state.plans = {k: v for k, v in state.plans.items() if k is None}  # keep the worst-case plan only
            state.plans[caps] = plan
        slots = plan.slots
        if caps is not None:
            slots = min(slots, max(lib.fgl_idmap_slots(2 * state.nodes_seen[-1]), lib.fgl_idmap_slots(n_seeds)))
        if self.graph_slots and caps is not None:  # steady state only: the worst-case plan (first batch, redo) runs eagerly
            out, host = self._replay(state, plan, slots, seeds, stream_base)
        else:
            host = self._take_host_counts(3 * len(hop_fanouts) + 2)
            run_on = stream if stream is not None else torch.cuda.current_stream(seeds.device)
            out = ops.sample_blocks_fused(plan, self.edge_ptr, self.edge_src, seeds, self.rng_seed, stream_base,
                                          keep_global=(len(hop_fanouts) - 1,), table_slots=slots, id_order=self.id_order,
                                          readback=host.expect(run_on), launch_stream=stream, sort_transposed=self.deterministic)
        return dict(seeds=seeds, stream_base=stream_base, caps=caps, out=out, state=state, host=host)

    def _take_host_counts(self, n_words):
        """Pinned words for one mini-batch's sizes: one of the sampler's that is not waiting to be read (a batch begun
        and not finished keeps its own), a new one if all are.  They live as long as the sampler: kernels in flight
        write into them."""
        rows = self._host_counts.setdefault(n_words, [])
        for _ in range(len(rows)):
            h = rows[self._host_turn % len(rows)]
            self._host_turn += 1
            if h.abandoned:  # (its batch was dropped unread: once its kernels have written, it is free again)
                h.abandoned = False
                h.read()
            if not h.busy:
                h.busy = True
                return h
        h = _HostCounts(n_words)
        h.busy = True
        rows.append(h)
        return h

    def _replay(self, state, plan, slots, seeds, stream_base):
        """Graph mode: copy the seeds and the random-stream offset into the turn's slot, replay its graph."""
        key = (id(plan), slots)
        if state.graphs is None or state.graphs[0] != key:
            state.graphs = (key, plan, [None] * self.graph_slots)  # graphs of an outgrown plan are dropped
        ring = state.graphs[2]
        turn = state.graph_turn % self.graph_slots  # (per lane: a lane's next mini-batch never lands in the slot of its last)
        state.graph_turn += 1
        if ring[turn] is None:
            ring[turn] = self._capture(plan, slots, seeds.device)
        slot = ring[turn]
        slot["seeds"].copy_(seeds)
        slot["offset"].fill_(stream_base - (1 << 32) if stream_base >= (1 << 31) else stream_base)  # uint32 bits in an int32
        # A captured sequence holds no table fill: it was recorded behind a call that left the table empty, and
        # leaves it empty itself.  If anything since then may have left entries behind (a call on this plan that
        # failed half-way), the table is emptied here, eagerly, before the replay.
        if plan.empty_slots != slots:
            ops.L.check(ops.L.lib().fgl_idmap_reset(ops.L.ptr(plan.table), slots, ops.L.stream_handle()))
        plan.empty_slots = None
        slot["host"].expect(torch.cuda.current_stream(seeds.device))
        slot["graph"].replay()
        plan.empty_slots = slots
        return slot["out"], slot["host"]

    def _capture(self, plan, slots, dev):
        hop_fanouts = list(reversed(self.fanouts))
        slot = dict(seeds=torch.zeros(plan.n_seeds, dtype=torch.int32, device=dev),
                    offset=torch.zeros(1, dtype=torch.int32, device=dev),
                    host=_HostCounts(3 * len(hop_fanouts) + 2))  # (the slot's own: rewritten by every replay, like its outputs)

        def enqueue():
            # stream_base 0: the slot's offset carries the mini-batch's stream number
            return ops.sample_blocks_fused(plan, self.edge_ptr, self.edge_src, slot["seeds"], self.rng_seed, 0,
                                           keep_global=(len(hop_fanouts) - 1,), table_slots=slots, id_order=self.id_order,
                                           stream_offset=slot["offset"], readback=slot["host"].words,
                                           sort_transposed=self.deterministic)

        cur = torch.cuda.current_stream(dev)
        warm = torch.cuda.Stream(device=dev)  # default priority
        warm.wait_stream(cur)
        with torch.cuda.stream(warm):  # one eager run off the capturing stream first
            enqueue()
        cur.wait_stream(warm)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):  # kernels only: the library enqueues no memset, copy or allocation
            slot["out"] = enqueue()
        slot["graph"] = graph
        return slot

    def _finish_fused(self, pending, counts_host):
        """counts_host: the batch's counts as a python list (already read back)."""
        H = len(self.fanouts)
        c = counts_host
        status = c[2 * H + 1]
        state = pending["state"]
        if status & (ops.L.STATUS_TABLE_FULL | ops.L.STATUS_UNIQ_OVERFLOW) and pending["caps"] is not None:
            state.nodes_seen = None
            pending = self._launch_fused(pending["seeds"], pending["stream_base"], worst_case=True, state=state)
            c = self._read_counts(pending)
            status = c[2 * H + 1]
        if status:
            ops._raise_status(status, "sample_blocks")
        seen = c[:H + 1]
        # the sizes are kept while batches stay within 1.25 x what they were derived from (the buffers hold 1.5 x):
        # every change means a new plan, new buffers and, in graph mode, new captures
        if state.nodes_seen is None:
            state.nodes_seen = seen
        elif any(a > 1.25 * b for a, b in zip(seen, state.nodes_seen)):
            state.nodes_seen = [max(a, b) for a, b in zip(seen, state.nodes_seen)]
        uniq, bptr, src_l, src_g, _, transposed = pending["out"]
        blocks = []
        for h in range(H):
            n_dst, n_src, n_e = c[h], c[h + 1], c[H + 1 + h]
            block_ptr = bptr[h][:n_dst + 1]
            block_ptr.fgl_longest_row = int(self.fanouts[H - 1 - h])  # no row exceeds the fanout (read by ops.aggregate)
            block = Block(block_ptr, src_l[h][:n_e], n_src, n_dst, None if src_g[h] is None else src_g[h][:n_e],
                          sorted_transpose=self.deterministic)
            if transposed[h] is not None:
                # built by the same call; its longest row came back with the sizes, so the backward gather knows
                # on the host whether any row needs the hub-row launch
                t_ptr = transposed[h][0][:n_src + 1]
                t_ptr.fgl_longest_row = max(int(c[2 * H + 2 + h]), ops.L.SHORT_ROW_ENTRIES)
                block._transposed = (t_ptr, transposed[h][1][:n_e], transposed[h][2][:n_e])
            blocks.insert(0, block)
        return uniq[:c[H]], pending["seeds"], blocks

    def begin_sample(self, seed_nodes):
        """First half of ``sample_blocks`` (fused path): enqueue every hop and return at once, without the host
        read-back.  The ``PendingBatch`` exposes the outermost block with bound-sized arrays and its row count on
        the device, so that the first layer's aggregation -- the largest kernel of a step -- can be enqueued
        before ``finish()`` waits for the sizes; the host's wake-up then hides behind that kernel."""
        if not self.fused:
            raise RuntimeError("begin_sample needs the fused path")
        if self.edge_ptr is None or self.edge_src is None:
            raise RuntimeError("FusedMapSampler: edge_ptr / edge_src are not set")
        self.output_nodes = seed_nodes
        seeds = seed_nodes.to(device=self.edge_src.device, dtype=torch.int32).contiguous()
        stream_base = (self.batches * 64) & 0xFFFFFFFF
        self.batches += 1
        return PendingBatch(self, self._launch_fused(seeds, stream_base))

    def _read_counts(self, pending):
        """The batch's sizes on the host: the kernels store them into pinned memory, the host waits for the words."""
        return pending["host"].read()

    def _sample_fused(self, seeds, stream_base):
        pending = self._launch_fused(seeds, stream_base)
        return self._finish_fused(pending, self._read_counts(pending))  # the one host synchronisation of the mini-batch

    def _lane_stream(self, dev, lane):
        while len(self._lanes) <= lane:
            self._lanes.append(torch.cuda.Stream(device=dev))  # default priority
        return self._lanes[lane]

    def iter_batches(self, seed_batches, prefetch=2):
        """Yields ``(input_nodes, output_nodes, blocks)`` for every seed batch, with up to ``prefetch`` mini-batches
        being sampled ahead of the one the caller works on, each on a HIP stream of its own (the role of the
        prefetching ``DataLoader`` that the reference plugs its sampler into, train_fastgl.py:109-122,248-258,
        ``prefetch_factor`` 2).  Mini-batches in flight together overlap on the GPU: the small hops of one -- chains
        of launch and memory latencies that leave most of the chip idle -- run under the large kernels of another
        and under the caller's aggregation (sampling alone, 111 M-node graph, batch 8192: 6.2 G sampled edges/s one
        at a time, 10.2 G with two in flight, 11.0 G with three).  Each lane has its own hash table and scratch.
        Results are identical to calling ``sample_blocks`` batch by batch."""
        if not self.fused:
            for seeds in seed_batches:
                yield self.sample_blocks(None, seeds)
            return
        prefetch = max(1, int(prefetch))
        dev = self.edge_src.device
        main = torch.cuda.current_stream(dev)

        def launch(seed_nodes, lane):
            seeds = seed_nodes.to(device=dev, dtype=torch.int32).contiguous()
            stream_base = (self.batches * 64) & 0xFFFFFFFF
            self.batches += 1
            side = self._lane_stream(dev, lane)
            side.wait_stream(main)  # the seeds (and anything else the caller produced) are ready
            if self.graph_slots:  # (a graph replays on the current stream)
                with torch.cuda.stream(side):
                    pending = self._launch_fused(seeds, stream_base, lane=lane)
                pending["on_lane"] = True
            else:
                # kernels on the lane's stream, outputs allocated on the caller's (where they are consumed and,
                # in stream order behind that, freed)
                pending = self._launch_fused(seeds, stream_base, lane=lane, stream=side)
            done = self._lane_events[lane]
            done.record(side)
            return pending, side, done

        def finish(item):
            pending, side, done = item
            counts = pending["host"].read()
            main.wait_event(done)  # whatever the caller enqueues from here on runs behind the mini-batch's kernels
            if not pending.get("on_lane"):
                return self._finish_fused(pending, counts)  # (a batch that outgrew its buffers is redone here, on the caller's stream)
            with torch.cuda.stream(side):
                result = self._finish_fused(pending, counts)
                redone = torch.cuda.Event()
                redone.record(side)
            main.wait_event(redone)
            for t in (result[0],) + tuple(x for b in result[2]
                                          for x in (b.edge_ptr, b.src_local, b.src_global) + tuple(b._transposed or ())
                                          if x is not None):
                t.record_stream(main)  # (possibly allocated on the lane's stream; consumed on the caller's)
            return result

        while len(self._lane_events) < prefetch:
            self._lane_events.append(torch.cuda.Event())
        it = iter(seed_batches)
        in_flight = collections.deque()
        n_launched = 0
        try:
            for seeds in itertools.islice(it, prefetch):
                in_flight.append(launch(seeds, n_launched % prefetch))
                n_launched += 1
            while in_flight:
                result = finish(in_flight.popleft())
                for seeds in itertools.islice(it, 1):  # (its lane is the one that has just become free)
                    in_flight.append(launch(seeds, n_launched % prefetch))
                    n_launched += 1
                yield result
        finally:
            # a consumer that stops early: the mini-batches still in flight write into memory that is about to be
            # freed on the caller's stream, so that stream waits for them first
            for _, _, done in in_flight:
                main.wait_event(done)

    def _sample_layerwise(self, seeds, stream_base):
        # the reference loop (FusedMapSampler.py:72-107), one drop-in call per step
        raw_seed_nodes = seeds.clone()
        seed_nodes_acc = seeds
        blocks = []
        dst_nodes = int(seeds.size(0))
        saved = dict(ops._rng_state)
        ops._rng_state["seed"] = self.rng_seed
        try:
            for block_index, fanout in enumerate(reversed(self.fanouts)):
                ops._rng_state["calls"] = stream_base + block_index
                src_out, dst_out, _ = ops.sample_node(self.edge_src, self.edge_dst if self.edge_dst is not None else self.edge_src,
                                                      self.edge_ptr, seed_nodes_acc, dst_nodes, fanout)
                block_ptr = ops.sample_node.last_block_ptr
                edge_nums = int(src_out.size(0))
                dst_unique = raw_seed_nodes if block_index == 0 else seed_nodes_acc
                n_dst = int(dst_unique.size(0))
                max_src_num = min(self.nodes_num, fanout * n_dst)
                src_global = src_out.clone() if block_index == len(self.fanouts) - 1 else None
                src_edges, _dst_edges, seed_nodes_acc = ops.transfer_edge_id(src_out, dst_out, dst_unique, dst_nodes,
                                                                             dst_nodes + edge_nums, max_src_num, edge_nums)
                block_ptr.fgl_longest_row = int(fanout)
                blocks.insert(0, Block(block_ptr, src_edges, int(seed_nodes_acc.size(0)), n_dst, src_global,
                                       sorted_transpose=self.deterministic))
                dst_nodes = int(seed_nodes_acc.size(0))
        finally:
            ops._rng_state.update(saved)
        return seed_nodes_acc, raw_seed_nodes, blocks


class DataLoader:
    """Mini-batch iterator with the constructor that the reference's trainer uses for DGL's ``DataLoader``
    (train_fastgl.py:248-258: ``DataLoader(g, train_nids, sampler, use_ddp=..., batch_size=..., shuffle=True,
    drop_last=False, prefetch_factor=..., num_workers=...)``) and the same iteration protocol
    (``for step, (input_nodes, output_nodes, blocks) in enumerate(dataloader)``, train_fastgl.py:346), without DGL.
    Every epoch it cuts the (optionally shuffled) seed ids into batches and hands them to
    ``sampler.iter_batches(..., prefetch=prefetch_factor)``: ``prefetch_factor`` mini-batches are sampled ahead on the
    GPU, each on a stream of its own, where DGL would run CPU workers.  ``g`` is ignored, as the reference's sampler
    ignores it (train_fastgl.py:245-246); ``num_workers`` is accepted and unused (sampling runs on the GPU);
    ``use_ddp`` must be false (one GPU)."""

    def __init__(self, g, nids, sampler, use_ddp=False, batch_size=1, shuffle=False, drop_last=False, prefetch_factor=2,
                 num_workers=0, seed=0, **unused):
        if use_ddp:
            raise NotImplementedError("one GPU: seed shards per rank are the trainer's business")
        if int(batch_size) < 1:
            raise ValueError("batch_size must be positive")
        self.nids = nids
        self.sampler = sampler
        self.batch_size = int(batch_size)
        self.shuffle = bool(shuffle)
        self.drop_last = bool(drop_last)
        self.prefetch_factor = max(0, int(prefetch_factor if prefetch_factor is not None else 0))
        self.seed = int(seed)
        self.epoch = 0

    def __len__(self):
        n = int(self.nids.numel())
        return n // self.batch_size if self.drop_last else -(-n // self.batch_size)

    def __iter__(self):
        ids = self.nids
        if self.shuffle:  # a fresh, seeded permutation per epoch
            gen = torch.Generator(device=ids.device).manual_seed(self.seed + self.epoch)
            ids = ids[torch.randperm(int(ids.numel()), generator=gen, device=ids.device)]
        self.epoch += 1
        B = self.batch_size
        batches = (ids[i * B:(i + 1) * B] for i in range(len(self)))
        if self.prefetch_factor > 0 and getattr(self.sampler, "fused", False):
            return self.sampler.iter_batches(batches, prefetch=self.prefetch_factor)
        return (self.sampler.sample_blocks(None, b) for b in batches)

