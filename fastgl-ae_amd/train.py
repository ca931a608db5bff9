#!/usr/bin/env python3
"""Mini-batch GNN training on one MI355X with the `fastgl` hot path -- the counterpart of the
reference's train_fastgl.py without DGL, datasets or multi-process set-up: a seeded synthetic
graph stays resident in HBM, seeds are shuffled and batched on the device, every step is
sample_blocks -> model forward -> loss -> backward -> Adam.

The timing protocol and the result lines follow the reference (train_fastgl.py:346-440): the
first epoch warms up and is not counted, phases are fenced by device synchronisation, and the
run ends with `test_result:{sample,copy,forward,backward,epoch}_time=...` lines that are also
written to `<log_path>/<model>_<dataset>_<layers>_<hidden>_<batch>_1.txt`.  `copy_time` is the
feature/label gather; with a resident feature table and the SAGE model it is fused into the
first layer's aggregation and only the label lookup remains.
"""
import argparse
import os
import sys
import time

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import fastgl  # noqa: E402


def make_dataset(n_nodes, n_draws, feat_dim, n_classes, train_frac, seed, device):
    """R-MAT graph + N(0,1) features + labels that depend on the one-hop mean of the features
    (so that aggregation is what makes them learnable)."""
    edge_ptr, edge_src = fastgl.graph.rmat_csr(n_nodes, n_draws, seed=seed, device=device)
    gen = torch.Generator(device=device).manual_seed(seed)
    feat = torch.randn((n_nodes, feat_dim), generator=gen, device=device)
    if edge_src.numel() >= 2 ** 31:
        raise RuntimeError("the label construction needs int32 row offsets (< 2^31 edges)")
    hop = fastgl.aggregate(edge_ptr.int(), edge_src, feat, mode="mean", zero_policy="zeros")
    proj = torch.randn((feat_dim, n_classes), generator=gen, device=device)
    label = ((hop + 0.5 * feat) @ proj).argmax(1)
    perm = torch.randperm(n_nodes, generator=gen, device=device)
    train_nids = perm[: max(1, int(n_nodes * train_frac))].int()
    return edge_ptr, edge_src, feat, label, train_nids


def build_model(name, in_feats, n_hidden, n_classes, n_layers, dropout):
    if name == "gcn":
        return fastgl.GCN(in_feats, n_hidden, n_classes, n_layers, None, True, dropout)
    if name == "gin":
        return fastgl.GIN(in_feats, n_hidden, n_classes, n_layers, None, True, dropout)
    if name == "gat":
        return fastgl.GAT(in_feats, n_hidden, n_classes, n_layers, None, dropout, heads=4)
    if name == "sage":
        return fastgl.SAGE(in_feats, n_hidden, n_classes, n_layers, dropout=dropout)
    raise ValueError("unknown model %r" % name)


def run(args):
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    torch.manual_seed(args.seed)
    edge_ptr, edge_src, feat, label, train_nids = make_dataset(args.nodes, args.draws, args.feat_dim, args.classes,
                                                               args.train_frac, args.seed, device)
    print("config:dataset=rmat_%d nodes=%d edges=%d train=%d" % (args.nodes, args.nodes, edge_src.numel(), train_nids.numel()))
    for k, v in sorted(vars(args).items()):
        print("config:{:}={:}".format(k, v))
    sampler = fastgl.FusedMapSampler(args.fanout, rng_seed=args.seed, id_order=args.id_order,
                                     deterministic=bool(args.deterministic)).set_graph(edge_ptr, edge_src)
    model = build_model(args.model, args.feat_dim, args.num_hidden, args.classes, len(args.fanout), args.dropout).to(device)
    loss_fcn = torch.nn.CrossEntropyLoss()
    optimizer = torch.optim.Adam(model.parameters(), lr=args.lr, weight_decay=args.weight_decay)
    sync = torch.cuda.synchronize

    # the reference wraps its sampler in DGL's DataLoader (train_fastgl.py:248-258); here the library's own, with the same
    # arguments: a seeded shuffle per epoch, prefetch_factor mini-batches sampled ahead on streams of their own
    dataloader = fastgl.DataLoader(None, train_nids, sampler, use_ddp=False, batch_size=args.batch_size, shuffle=True,
                                   drop_last=False, prefetch_factor=args.prefetch, num_workers=0, seed=args.seed + 1000)
    steps = len(dataloader)
    epochs = []
    losses = []
    for epoch in range(args.num_epoch + 1):  # the first epoch is the warm-up (train_fastgl.py:96-97)
        t = dict(sample=0.0, copy=0.0, forward=0.0, backward=0.0)
        n_edges = n_inputs = 0
        sync()
        tic = time.time()
        batches = iter(dataloader)
        for step in range(steps):
            t0 = time.time()
            input_nodes, output_nodes, blocks = next(batches)
            if not args.prefetch:
                sync()
            t1 = time.time()
            fastgl.transpose_blocks(blocks[1:])  # the backward pass of every layer but the first gathers over the transposed block
            batch_labels = label.index_select(0, output_nodes.long())
            if args.model == "sage":
                batch_inputs = None  # the first layer gathers straight from the resident table
            else:
                batch_inputs = feat.index_select(0, input_nodes.long())
            sync()
            t2 = time.time()
            if args.model == "sage":
                batch_pred = model(blocks, feat, input_nodes=input_nodes)
            else:
                batch_pred = model(blocks, batch_inputs, neighbor_list=args.fanout)
            loss = loss_fcn(batch_pred, batch_labels)
            sync()
            t3 = time.time()
            optimizer.zero_grad()
            loss.backward()
            optimizer.step()
            sync()
            t4 = time.time()
            t["sample"] += t1 - t0
            t["copy"] += t2 - t1
            t["forward"] += t3 - t2
            t["backward"] += t4 - t3
            n_edges += sum(b.num_edges() for b in blocks)
            n_inputs += blocks[0].num_src_nodes()
            losses.append(float(loss.detach()))
            if step % args.log_every == 0:
                print("Epoch {:05d} | Step {:05d} | Nodes {:.0f} | Samples {:.0f} | Sample Time {:.4f} | Copy Time {:.4f} | "
                      "Train time {:.4f} | Loss {:.4f}".format(epoch, step, blocks[0].num_src_nodes(),
                                                               sum(b.num_edges() for b in blocks), t1 - t0, t2 - t1,
                                                               t4 - t2, float(loss.detach())))
        sync()
        t["total"] = time.time() - tic
        t["edges"], t["inputs"] = n_edges, n_inputs
        epochs.append(t)

    timed = epochs[1:] if len(epochs) > 1 else epochs
    mean = lambda k: sum(e[k] for e in timed) / len(timed)
    print("[Worker 0({:s})] Avg Epoch Time {:.4f} | Avg Nodes {:.0f} | Avg Samples {:.0f} | Sample Time {:.4f} | "
          "Copy Time {:.4f} | Train Time {:.4f}".format(torch.cuda.get_device_name(device), mean("total"), mean("inputs"),
                                                        mean("edges"), mean("sample"), mean("copy"), mean("forward")))
    test_result = {
        "sample_time": mean("sample"), "copy_time": mean("copy"), "forward_time": mean("forward"),
        "backward_time": mean("backward"),
    }
    test_result["epoch_time"] = sum(test_result.values())
    for k, v in test_result.items():
        print("test_result:{:}={:.5f}".format(k, v))
    print("finish")
    if args.log_path:
        os.makedirs(args.log_path, exist_ok=True)
        name = "%s_rmat%d_%d_%d_%d_1.txt" % (args.model, args.nodes, len(args.fanout), args.num_hidden, args.batch_size)
        with open(os.path.join(args.log_path, name), "w") as f:
            for k, v in test_result.items():
                f.write("%s:%s\n" % (k, v))
    return test_result, losses


def parse_args(argv=None):
    ap = argparse.ArgumentParser("fastgl synthetic training")
    ap.add_argument("--model", default="sage", choices=["gcn", "gin", "gat", "sage"])
    ap.add_argument("--fanout", nargs="+", type=int, default=[15, 10, 5])
    ap.add_argument("--num_epoch", type=int, default=3)
    ap.add_argument("--num_hidden", type=int, default=256)
    ap.add_argument("--batch_size", type=int, default=8192)
    ap.add_argument("--nodes", type=int, default=2_400_000)
    ap.add_argument("--draws", type=int, default=36_000_000)
    ap.add_argument("--feat_dim", type=int, default=100)
    ap.add_argument("--classes", type=int, default=16)
    ap.add_argument("--train_frac", type=float, default=0.1)
    ap.add_argument("--lr", type=float, default=0.01)
    ap.add_argument("--dropout", type=float, default=0.5)
    ap.add_argument("--weight_decay", type=float, default=0.0005)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--id_order", default="first", choices=["first", "arrival"])
    ap.add_argument("--deterministic", type=int, default=0,
                    help="1: order the transposed blocks' lists too, so that the fp32 sums of the backward pass -- and with them "
                         "the whole run -- are reproducible bit for bit (two more launches per mini-batch; needs --id_order first)")
    ap.add_argument("--prefetch", type=int, default=2,
                    help="mini-batches sampled ahead of the one that trains, each on a stream of its own (the reference's "
                         "prefetch_factor, train_fastgl.py:109-122); 0: sample and train in turn")
    ap.add_argument("--log_every", type=int, default=10)
    ap.add_argument("--log_path", default="")
    return ap.parse_args(argv)


if __name__ == "__main__":
    run(parse_args())
