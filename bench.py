#!/usr/bin/env python3
"""Benchmark of the FastGL hot path on one MI355X:  sample -> fused id-map -> aggregate.

One step = one mini-batch of the workload through the hot path with everything resident in
HBM: all hops of neighbour sampling + id-map (one enqueue, one count read-back), then the
aggregation kernels of a GraphSAGE-mean model over the sampled blocks -- forward for every
block (the outermost one gathers straight from the full feature table), and, for the blocks
whose input needs a gradient, the block transpose and the backward gather.  The dense
layers between aggregations are library GEMMs outside this path and are not run.

Prints ONE JSON line.  `value` is sampled edges per second of the sampling + id-map stage;
`roofline` describes the dominant kernel (the outermost block's forward aggregation) against
the 8 TB/s HBM peak; `cpu_baseline` is the CPU oracle timed on a bounded sample of the same
workload on this machine's host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "fastgl-ae_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0
# HBM traffic per launch of the dominant kernel comes from the tracked summary of two `rocprofv3 --pmc` runs
# (FETCH_SIZE, WRITE_SIZE, each scaled by what the same counter reads for this kernel run as a plain copy of
# known size).  The summary carries a record line with the kernel source's hash and the algorithmic bytes
# per launch that it was taken at; `traffic` is reported only while both still match this run.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "aggregate_kernel_c3_pmc.md")
AGGREGATE_SOURCE = os.path.join(ROOT, "fastgl-ae_amd", "csrc", "fgl_aggregate.hip")


def source_hash(path=AGGREGATE_SOURCE):
    import hashlib
    with open(path, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def traffic_from_profile(workload, bytes_per_launch):
    """HBM bytes per launch of the dominant kernel from the tracked counter summary, or None (with a note on
    stderr) when the summary is missing, covers another workload, or was taken with another kernel source or
    at another problem size."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        log("roofline.traffic: %s is missing -> null" % TRAFFIC_PROFILE)
        return None
    rec = None
    for line in text.splitlines():
        if line.startswith("traffic_record:"):
            rec = json.loads(line[len("traffic_record:"):])
    if rec is None:
        log("roofline.traffic: no traffic_record line in %s -> null" % TRAFFIC_PROFILE)
        return None
    if rec.get("workload") != workload:
        log("roofline.traffic: the counter summary covers workload %s, not %s -> null" % (rec.get("workload"), workload))
        return None
    if rec.get("source_sha16") != source_hash():
        log("roofline.traffic: fgl_aggregate.hip has changed since the counter runs (%s -> %s): profile again -> null"
            % (rec.get("source_sha16"), source_hash()))
        return None
    if abs(rec["algorithmic_bytes_per_launch"] - bytes_per_launch) > 0.03 * bytes_per_launch:
        log("roofline.traffic: the counter runs moved %.1f MB per launch, this run %.1f MB -> null"
            % (rec["algorithmic_bytes_per_launch"] / 1e6, bytes_per_launch / 1e6))
        return None
    return rec["traffic_bytes_per_launch"]


WORKLOADS = {
    # name: nodes, R-MAT draws, feature dim, feature dtype, hidden, batch, training seeds, fanouts (reference order)
    "c1": dict(nodes=100_000, draws=1_500_000, dim=128, dtype="f32", hidden=256, batch=1024, train=100_000, fanouts=[15, 10, 5]),
    "c2": dict(nodes=2_400_000, draws=36_000_000, dim=100, dtype="f32", hidden=256, batch=8192, train=240_000, fanouts=[15, 10, 5]),
    "c3": dict(nodes=111_000_000, draws=900_000_000, dim=128, dtype="f32", hidden=256, batch=8192, train=1_200_000, fanouts=[15, 10, 5]),
    "c5": dict(nodes=269_000_000, draws=3_320_000_000, dim=128, dtype="bf16", hidden=256, batch=8192, train=1_200_000, fanouts=[15, 10, 5]),
    "c5deep": dict(nodes=269_000_000, draws=3_320_000_000, dim=128, dtype="bf16", hidden=256, batch=8192, train=1_200_000,
                   fanouts=[10, 10, 10, 10, 10]),
    "c4": None,  # aggregation-only microbench, see run_c4
    "ceiling": None,  # random row gathers from a 48 GB table, see run_ceiling
    "reuse_ab": None,  # outermost block in one launch vs two passes by source id, see run_reuse_ab
    "idmap_stats": None,  # intra-tile repeats and probes per lookup on real mini-batches, see run_idmap_stats
}
DESCRIPTIONS = {
    "c1": "R-MAT 100K nodes / ~2.5M edges, feat 128 fp32, batch 1024, fanout [15,10,5]",
    "c2": "R-MAT 2.4M nodes / ~62M edges, feat 100 fp32, hidden 256, batch 8192, fanout [15,10,5]",
    "c3": "R-MAT 111M nodes / ~1.6B edges (int64 indptr, int32 indices), feat 111Mx128 fp32 resident, hidden 256, "
          "batch 8192 of 1.2M training seeds, fanout [15,10,5]",
    "c5": "R-MAT 269M nodes / ~4.0B edges (int64 indptr, int32 indices), feat 269Mx128 bf16 resident, hidden 256, "
          "batch 8192, fanout [15,10,5]",
    "c5deep": "R-MAT 269M nodes / ~4.0B edges (int64 indptr, int32 indices), feat 269Mx128 bf16 resident, hidden 256, "
              "batch 8192, fanout [10,10,10,10,10]",
    "ceiling": "random row gathers from a 48 GB table: 2^20 output rows x 1 or 13 uniformly random source rows of 256 B - 2 KB, "
               "fp32 and bf16, through the aggregation kernel and through torch.index_select; streaming copy and add",
    "reuse_ab": "outermost block of c3 mini-batches (1.5 M gathered rows of 512 B, 1.0 M distinct, 57 GB table): one launch vs "
                "two launches cut by a source-id threshold",
    "idmap_stats": "c3 mini-batches: ids repeated within a 2048-edge tile per hop; slots probed per lookup in the id-map's table",
    "c4": "aggregation microbench: 8192 dst x exactly 25 src out of 200K rows (int32 CSR), D in {64,128,256,602}, fp32 and bf16, "
          "sum and mean, forward and backward",
}


def run_c4(args, edge_weighted=True):
    """Aggregation-only microbench.  Forward = gather over the block, backward = gather over the
    transposed block; every case is 50 back-to-back launches between two HIP events ("cold" = the
    same launches rotating over copies of the tables -- the gathered one and, for the backward pass, the written
    one as well -- that do not fit the Infinity Cache together, so that the figures are HBM figures).  Returns the
    record; `launch_floor_us` is a launch of the library that moves a few hundred bytes, timed the same way."""
    import torch

    import fastgl

    last_mapping = lambda: fastgl.lib().fgl_aggregate_last_mapping().decode()

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    n_dst, n_src, k = 8192, 200_000, 25
    ptr = (torch.arange(n_dst + 1, dtype=torch.int32) * k).to(dev)
    idx = torch.randint(0, n_src, (n_dst * k,), generator=g, dtype=torch.int32).to(dev)
    t_ptr, t_idx = fastgl.block_transpose(ptr, idx, n_dst, n_src)
    # The transposed block's longest row: the transpose leaves it on the device (the backward launches below find it there
    # and pay a second, empty launch that looks for hub rows); a caller that has read it back -- a block that is
    # transposed once and used many times, or one whose sizes travel to the host anyway -- passes it as a bound.
    t_longest = max(int(t_ptr.fgl_longest_row.item()), 32)  # (the transpose reports lengths beyond 32 entries only)
    deg = torch.full((n_dst,), k, dtype=torch.int32, device=dev)
    E = n_dst * k
    ev = lambda: torch.cuda.Event(enable_timing=True)

    def timed(fn, reps=50):
        """us per launch of `reps` launches between two HIP events.  The launches are replayed from a captured
        HIP graph: a launch through the Python binding costs the host about 10 us, more than the smaller
        kernels run, so launched one by one the interval would measure the host (`--c4-eager` does that)."""
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        a, b = ev(), ev()
        if args.c4_eager:
            a.record()
            for _ in range(reps):
                fn()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / reps * 1e3
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):  # kernels only: the library enqueues no memset, copy or allocation
            for _ in range(reps):
                fn()
        graph.replay()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            a.record()
            graph.replay()
            b.record()
            torch.cuda.synchronize()
            t = a.elapsed_time(b) / reps * 1e3
            best = t if best is None or t < best else best
        del graph
        return best  # us

    # what a launch costs in this harness when there is next to nothing to move: one row of one entry
    tiny_ptr = torch.tensor([0, 1], dtype=torch.int32, device=dev)
    tiny_idx = torch.zeros(1, dtype=torch.int32, device=dev)
    tiny_x = torch.zeros((1, 64), device=dev)
    tiny_o = torch.empty((1, 64), device=dev)
    launch_floor_us = timed(lambda: fastgl.aggregate(tiny_ptr, tiny_idx, tiny_x, mode="sum", zero_policy="zeros", out=tiny_o, longest_row=1))
    log("launch floor (one row of one entry, same harness): %.2f us" % launch_floor_us)

    rows = []
    for dt, name, esz in ((torch.float32, "f32", 4), (torch.bfloat16, "bf16", 2)):
        for D in (64, 128, 256, 602):
            X = torch.randn(n_src, D, generator=g).to(dt).to(dev)
            dO = torch.randn(n_dst, D, generator=g).to(dt).to(dev)
            of = torch.empty((n_dst, D), dtype=dt, device=dev)
            ob = torch.empty((n_src, D), dtype=dt, device=dev)
            bf = E * D * esz + n_dst * D * esz + 4 * E + 4 * (n_dst + 1)
            bb = E * D * esz + n_src * D * esz + 4 * E + 4 * (n_src + 1)
            # cold-cache variant: rotate among copies of the table that together exceed the 256 MB
            # Infinity Cache several times, so that no launch finds its rows cached by the one before
            n_copies = max(2, -(-(1 << 30) // (n_src * D * esz)))
            Xs = [X] + [X.clone() for _ in range(n_copies - 1)]
            turn = [0]

            def fwd_cold(mode):
                turn[0] = (turn[0] + 1) % n_copies
                fastgl.aggregate(ptr, idx, Xs[turn[0]], mode=mode, zero_policy="zeros", out=of, longest_row=k)

            # cold backward: the gathered table (upstream gradients, 8192 rows) is small, the written one
            # (200 K rows) is what would otherwise sit in the cache from one launch to the next: rotate both
            dOs = [dO] + [dO.clone() for _ in range(n_copies - 1)]
            obs = [ob] + [torch.empty_like(ob) for _ in range(n_copies - 1)]

            def bwd_cold(bmode):
                turn[0] = (turn[0] + 1) % n_copies
                fastgl.aggregate(t_ptr, t_idx, dOs[turn[0]], mode=bmode, zero_policy="zeros", col_norm=deg, out=obs[turn[0]],
                                 longest_row=t_longest)

            for mode, bmode in (("sum", "sum"), ("mean", "colmean")):
                # longest_row: every row holds exactly k entries (a sampler knows its fanout the same way)
                uf = timed(lambda: fastgl.aggregate(ptr, idx, X, mode=mode, zero_policy="zeros", out=of, longest_row=k))
                kf = last_mapping()
                uc = timed(lambda: fwd_cold(mode), reps=5 * n_copies)
                ubc = timed(lambda: bwd_cold(bmode), reps=5 * n_copies)
                ub = timed(lambda: fastgl.aggregate(t_ptr, t_idx, dO, mode=bmode, zero_policy="zeros", col_norm=deg, out=ob))
                uk = timed(lambda: fastgl.aggregate(t_ptr, t_idx, dO, mode=bmode, zero_policy="zeros", col_norm=deg, out=ob,
                                                    longest_row=t_longest))
                kb = last_mapping()
                rows.append({"dtype": name, "D": D, "mode": mode, "fwd_kernel": kf, "bwd_kernel": kb,
                             "bwd_cold_us": ubc, "bwd_cold_GBps": bb / ubc / 1e3, "bwd_cold_frac_peak": bb / ubc / 1e3 / HBM_PEAK_GBPS,
                             "fwd_us": uf, "fwd_GBps": bf / uf / 1e3,
                             "bwd_known_longest_us": uk, "bwd_known_longest_GBps": bb / uk / 1e3,
                             "bwd_known_longest_frac_peak": bb / uk / 1e3 / HBM_PEAK_GBPS,
                             "fwd_frac_peak": bf / uf / 1e3 / HBM_PEAK_GBPS, "fwd_cold_us": uc,
                             "fwd_cold_GBps": bf / uc / 1e3, "fwd_cold_frac_peak": bf / uc / 1e3 / HBM_PEAK_GBPS, "bwd_us": ub, "bwd_GBps": bb / ub / 1e3,
                             "bwd_frac_peak": bb / ub / 1e3 / HBM_PEAK_GBPS})
                log("%-4s D=%-3d %-4s fwd %6.1f us %5.0f GB/s (%4.1f%%) | cold fwd %6.1f us %5.0f GB/s (%4.1f%%) | "
                    "bwd %6.1f us %5.0f GB/s (%4.1f%%) | bwd, longest row (%d) known to the host %6.1f us (%4.1f%%) | cold %6.1f us (%4.1f%%)"
                    % (name, D, mode, uf, bf / uf / 1e3, bf / uf / 1e3 / HBM_PEAK_GBPS * 100, uc, bf / uc / 1e3,
                       bf / uc / 1e3 / HBM_PEAK_GBPS * 100, ub, bb / ub / 1e3, bb / ub / 1e3 / HBM_PEAK_GBPS * 100, t_longest, uk,
                       bb / uk / 1e3 / HBM_PEAK_GBPS * 100, ubc, bb / ubc / 1e3 / HBM_PEAK_GBPS * 100))
            del Xs, dOs, obs
    # attention-weighted aggregation (GAT): one float per (entry, head) on top of the row gather
    gat_rows = []
    n_heads = 4
    alpha = torch.rand((E, n_heads), generator=g).to(dev)
    t_ptr3, t_idx3, t_edge3 = fastgl.block_transpose(ptr, idx, n_dst, n_src, edge_ids=True)
    for dt, name, esz in ((torch.float32, "f32", 4), (torch.bfloat16, "bf16", 2)):
        for D in (128, 256) if edge_weighted else ():
            X = torch.randn(n_src, D, generator=g).to(dt).to(dev)
            dO = torch.randn(n_dst, D, generator=g).to(dt).to(dev)
            of = torch.empty((n_dst, D), dtype=dt, device=dev)
            ob = torch.empty((n_src, D), dtype=dt, device=dev)
            bf = E * D * esz + n_dst * D * esz + 4 * E + 4 * (n_dst + 1) + 4 * n_heads * E
            bb = E * D * esz + n_src * D * esz + 4 * E + 4 * (n_src + 1) + 4 * n_heads * E + 4 * E  # + edge ids of the transposed entries
            us = timed(lambda: fastgl.aggregate(ptr, idx, X, mode="sum", zero_policy="zeros", out=of, longest_row=k))
            uf = timed(lambda: fastgl.aggregate(ptr, idx, X, mode="edge", zero_policy="zeros", out=of, longest_row=k,
                                                edge_weight=alpha, n_heads=n_heads))
            ub = timed(lambda: fastgl.aggregate(t_ptr3, t_idx3, dO, mode="edge", zero_policy="zeros", out=ob, edge_weight=alpha,
                                                n_heads=n_heads, edge_index=t_edge3))
            bs = bf - 4 * n_heads * E
            gat_rows.append({"dtype": name, "D": D, "heads": n_heads, "fwd_us": uf, "fwd_GBps": bf / uf / 1e3,
                             "fwd_frac_peak": bf / uf / 1e3 / HBM_PEAK_GBPS, "sum_fwd_us": us, "sum_fwd_GBps": bs / us / 1e3,
                             "bwd_us": ub, "bwd_GBps": bb / ub / 1e3, "bwd_frac_peak": bb / ub / 1e3 / HBM_PEAK_GBPS})
            log("%-4s D=%-3d edge weights x%d: fwd %6.1f us %5.0f GB/s (%4.1f%%; plain sum %6.1f us %5.0f GB/s) | bwd %6.1f us %5.0f GB/s (%4.1f%%)"
                % (name, D, n_heads, uf, bf / uf / 1e3, bf / uf / 1e3 / HBM_PEAK_GBPS * 100, us, bs / us / 1e3, ub, bb / ub / 1e3,
                   bb / ub / 1e3 / HBM_PEAK_GBPS * 100))
    head = [r for r in rows if r["dtype"] == "f32" and r["D"] == 128 and r["mode"] == "mean"][0]
    return {
        "metric": "aggregation HBM GB/s (% peak), 1 MI355X", "value": head["fwd_GBps"], "unit": "GB/s", "n_gpus": 1,
        "steps": 50, "warmup": 5, "ms_per_step": head["fwd_us"] / 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic", "config": {"workload": DESCRIPTIONS["c4"]},
        "roofline": {"bound": "hbm", "achieved": head["fwd_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": head["fwd_frac_peak"], "traffic": None, "kernel": "aggregate_kernel (D=128 fp32 mean forward)"},
        "cpu_baseline": None, "launch_floor_us": launch_floor_us, "transposed_longest_row": t_longest, "cases": rows,
        "edge_weighted_cases": gat_rows}


def c4_compact(rec):
    """The microbench's record cut down to what rides on the default benchmark line: per case the time and
    fraction of the HBM peak of the forward gather, the backward gather (longest transposed row known to the
    host, as the sampler hands it over) and their cold-cache forms, with the kernel that ran; the worst
    forward and the worst backward case named."""
    cases = []
    for r in rec["cases"]:
        cases.append({"case": "%s D=%d %s" % (r["dtype"], r["D"], r["mode"]),
                      "fwd_us": round(r["fwd_us"], 2), "fwd_frac": round(r["fwd_frac_peak"], 3),
                      "fwd_cold_us": round(r["fwd_cold_us"], 2), "fwd_cold_frac": round(r["fwd_cold_frac_peak"], 3),
                      "bwd_us": round(r["bwd_known_longest_us"], 2), "bwd_frac": round(r["bwd_known_longest_frac_peak"], 3),
                      "bwd_cold_us": round(r["bwd_cold_us"], 2), "bwd_cold_frac": round(r["bwd_cold_frac_peak"], 3),
                      "fwd_kernel": r["fwd_kernel"], "bwd_kernel": r["bwd_kernel"]})
    worst = lambda key: min(cases, key=lambda c: c[key])
    return {"workload": DESCRIPTIONS["c4"],
            "timing": "50 launches replayed from a captured HIP graph between two HIP events, best of 3; frac = algorithmic bytes / time / 8 TB/s; "
                      "warm = the same tables every launch (a 200K-row table of <= 481 MB partly stays in the 256 MB Infinity Cache; the backward "
                      "pass gathers from an 8192-row table that always does, so its warm figures are not HBM figures); cold = rotating over "
                      "copies that exceed the cache several times",
            "launch_floor_us": round(rec["launch_floor_us"], 2), "transposed_longest_row": rec["transposed_longest_row"],
            "worst_fwd": {k: worst("fwd_frac")[k] for k in ("case", "fwd_us", "fwd_frac", "fwd_kernel")},
            "worst_fwd_cold": {k: worst("fwd_cold_frac")[k] for k in ("case", "fwd_cold_us", "fwd_cold_frac", "fwd_kernel")},
            "worst_bwd": {k: worst("bwd_frac")[k] for k in ("case", "bwd_us", "bwd_frac", "bwd_kernel")},
            "worst_bwd_cold": {k: worst("bwd_cold_frac")[k] for k in ("case", "bwd_cold_us", "bwd_cold_frac", "bwd_kernel")},
            "cases": cases}



def run_ceiling(args):
    """What the box gives to row gathers, whatever kernel asks: the aggregation kernel as a pure random
    gather (one random source row per output row: no reuse, no arithmetic to speak of) and with 13 random
    rows per output row (the outer block's shape), for several row sizes, from a table far larger than the
    caches; next to it torch's own row gather, a streaming add and a device-to-device copy."""
    import torch

    import fastgl

    dev = torch.device("cuda:0")
    ev = lambda: torch.cuda.Event(enable_timing=True)

    def timed(fn, reps=20):
        for _ in range(3):
            fn()
        a, b = ev(), ev()
        torch.cuda.synchronize()
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps * 1e-3  # seconds

    gen = torch.Generator(device=dev).manual_seed(0)
    table_bytes = 48 << 30
    n_out = 1 << 20
    rows_out = []
    for dtype, esz in ((torch.float32, 4), (torch.bfloat16, 2)):
        for row_bytes in (256, 512, 1024, 2048):
            D = row_bytes // esz
            n_rows = table_bytes // row_bytes
            table = torch.empty((n_rows, D), dtype=dtype, device=dev)
            table.view(torch.int32).fill_(0)  # the values do not matter (zeros in either format), the addresses do
            out = torch.empty((n_out, D), dtype=dtype, device=dev)
            case = {"dtype": "f32" if esz == 4 else "bf16", "row_bytes": row_bytes, "table_GB": table_bytes / 2 ** 30}
            for k in (1, 13):
                ptr = torch.arange(n_out + 1, dtype=torch.int32, device=dev) * k
                idx = torch.randint(0, n_rows, (n_out * k,), generator=gen, device=dev, dtype=torch.int32)
                t = timed(lambda: fastgl.aggregate(ptr, idx, table, mode="sum", zero_policy="zeros", out=out, longest_row=k))
                moved = n_out * k * row_bytes + n_out * row_bytes + 4 * n_out * k + 4 * (n_out + 1)
                case["k%d_GBps" % k] = moved / t / 1e9
                case["k%d_Grows_per_s" % k] = n_out * k / t / 1e9
                if k == 1:
                    idx64 = idx.long()
                    t = timed(lambda: torch.index_select(table, 0, idx64, out=out))
                    case["torch_index_select_GBps"] = 2 * n_out * row_bytes / t / 1e9
                else:
                    # the same gather-and-sum by a kernel that is not this library's: torch's embedding_bag
                    # (same bytes counted; it also writes a bag index per entry, which is not)
                    try:
                        idx64 = idx.long()
                        off64 = ptr[:-1].long()
                        bag = lambda: torch.nn.functional.embedding_bag(idx64, table, off64, mode="sum")
                        t = timed(bag)
                        case["torch_embedding_bag_k13_GBps"] = moved / t / 1e9
                        del bag
                    except Exception as e:  # (a dtype the library kernel does not take)
                        case["torch_embedding_bag_k13_GBps"] = None
                        log("embedding_bag: %s" % str(e).splitlines()[0])
            rows_out.append(case)
            log("%-4s rows of %4d B: 1 source per row %5.0f GB/s (%.1f G rows/s; torch.index_select %5.0f GB/s) | "
                "13 sources per row %5.0f GB/s (%.1f G rows/s; torch embedding_bag %5.0f GB/s)"
                % (case["dtype"], row_bytes, case["k1_GBps"], case["k1_Grows_per_s"], case["torch_index_select_GBps"],
                   case["k13_GBps"], case["k13_Grows_per_s"], case["torch_embedding_bag_k13_GBps"] or 0.0))
            del table, out
            torch.cuda.empty_cache()
    a = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    b = torch.empty_like(a)
    t = timed(lambda: b.copy_(a))
    copy_gbps = 2 * (1 << 30) / t / 1e9
    x = a.view(torch.float32)
    y = b.view(torch.float32)
    t = timed(lambda: torch.add(x, 1.0, out=y))
    add_gbps = 2 * (1 << 30) / t / 1e9
    log("streaming: device copy %.0f GB/s, elementwise add %.0f GB/s (read + write)" % (copy_gbps, add_gbps))
    head = [r for r in rows_out if r["dtype"] == "f32" and r["row_bytes"] == 512][0]
    print(json.dumps({
        "metric": "random row gather GB/s (context for the aggregation roofline), 1 MI355X", "value": head["k13_GBps"],
        "unit": "GB/s", "n_gpus": 1, "steps": 20, "warmup": 3, "ms_per_step": None, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": DESCRIPTIONS["ceiling"]},
        "roofline": {"bound": "hbm", "achieved": head["k13_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": head["k13_GBps"] / HBM_PEAK_GBPS, "traffic": None,
                     "kernel": "aggregate_kernel<float,4,32,SUM> (13 random 512-byte rows per output row, 48 GB table)"},
        "cpu_baseline": None, "stream_copy_GBps": copy_gbps, "stream_add_GBps": add_gbps, "cases": rows_out}), flush=True)


def _c3_inputs(torch, fastgl, dev, need_features=True):
    w = WORKLOADS["c3"]
    edge_ptr, edge_src = fastgl.graph.rmat_csr(w["nodes"], w["draws"], seed=0, device=dev)
    torch.cuda.empty_cache()
    gen = torch.Generator(device=dev).manual_seed(0)
    feat = None
    if need_features:
        feat = torch.empty((w["nodes"], w["dim"]), dtype=torch.float32, device=dev)
        for lo in range(0, w["nodes"], 1 << 22):
            hi = min(w["nodes"], lo + (1 << 22))
            feat[lo:hi] = torch.randn((hi - lo, w["dim"]), generator=gen, device=dev, dtype=torch.float32)
    train = torch.randperm(w["nodes"], generator=gen, device=dev)[:w["train"]].to(torch.int32)
    return w, edge_ptr, edge_src, feat, train


def run_reuse_ab(args):
    """Does it pay to gather the outermost block in two passes by source id, so that each pass's distinct rows fit the
    256 MB Infinity Cache?  (A mini-batch's outermost block gathers 1.5 M rows of which 1.0 M are distinct.)  Times
    the whole block in one launch against the same block cut in two by a source-id threshold -- the launches of the
    two halves only; the pass that would add the two partial outputs is not even counted -- for the threshold that
    halves the ids and the one that halves the gathered rows."""
    import torch

    import fastgl

    dev = torch.device("cuda:0")
    w, edge_ptr, edge_src, feat, train = _c3_inputs(torch, fastgl, dev)
    B, D = w["batch"], w["dim"]
    sampler = fastgl.FusedMapSampler(w["fanouts"], rng_seed=0).set_graph(edge_ptr, edge_src)
    ev = lambda: torch.cuda.Event(enable_timing=True)

    def timed(fn, reps=10):
        for _ in range(3):
            fn()
        a, b = ev(), ev()
        torch.cuda.synchronize()
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps * 1e3

    cases = []
    for batch in range(3):
        _, _, blocks = sampler.sample_blocks(None, train[batch * B:(batch + 1) * B])
        b0 = blocks[0]
        n_dst, E = b0.num_dst_nodes(), b0.num_edges()
        src = b0.src_global.long()
        rows = torch.repeat_interleave(torch.arange(n_dst, device=dev), b0.in_degrees().long())
        distinct = int(torch.unique(src).numel())
        out = torch.empty((n_dst, D), device=dev)
        t_full = timed(lambda: fastgl.aggregate(b0.edge_ptr, b0.src_global, feat, mode="sum", zero_policy="zeros", out=out,
                                                longest_row=w["fanouts"][0]))
        case = {"edges": E, "distinct_rows": distinct, "rows": n_dst, "one_launch_us": t_full,
                "one_launch_GBps": (E * D * 4 + n_dst * D * 4 + 4 * E + 4 * n_dst) / t_full / 1e3}
        for name, thr in (("half_of_the_ids", w["nodes"] // 2), ("half_of_the_gathered_rows", int(torch.median(src)))):
            halves = []
            for keep in (src < thr, src >= thr):
                sub_src = b0.src_global[keep].contiguous()
                counts = torch.bincount(rows[keep], minlength=n_dst)
                sub_ptr = torch.zeros(n_dst + 1, dtype=torch.int32, device=dev)
                sub_ptr[1:] = torch.cumsum(counts, 0).int()
                halves.append((sub_ptr, sub_src, int(torch.unique(sub_src).numel())))
            outs = [torch.empty((n_dst, D), device=dev) for _ in halves]

            def two():
                for (p_, s_, _), o_ in zip(halves, outs):
                    fastgl.aggregate(p_, s_, feat, mode="sum", zero_policy="zeros", out=o_, longest_row=w["fanouts"][0])

            t_two = timed(two)
            case[name] = {"threshold": thr, "edges": [int(h[1].numel()) for h in halves], "distinct_rows": [h[2] for h in halves],
                          "two_launches_us": t_two}
            log("batch %d: %d edges, %d distinct rows: one launch %.1f us | cut at %s (%d): halves of %s edges / %s distinct rows, "
                "two launches %.1f us" % (batch, E, distinct, t_full, name, thr, case[name]["edges"], case[name]["distinct_rows"], t_two))
        cases.append(case)
    print(json.dumps({"metric": "outermost-block gather in one launch vs two passes by source id (us), 1 MI355X",
                      "value": cases[-1]["one_launch_us"], "unit": "us", "n_gpus": 1, "steps": 10, "warmup": 3, "ms_per_step": None,
                      "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                      "config": {"workload": DESCRIPTIONS["reuse_ab"]}, "roofline": None, "cpu_baseline": None, "cases": cases}), flush=True)


def run_idmap_stats(args):
    """The numbers behind two design decisions of the id-map, on real mini-batches of workload c3: how many edges of a
    2048-edge tile repeat an id already seen in the same tile (what a per-tile LDS dedup before the global table could
    save), and how many slots a lookup probes in the table at the load factor the sampler runs it at (what probing with
    several lanes per key could save)."""
    import numpy as np
    import torch

    import fastgl

    dev = torch.device("cuda:0")
    w, edge_ptr, edge_src, _, train = _c3_inputs(torch, fastgl, dev, need_features=False)
    B = w["batch"]
    sampler = fastgl.FusedMapSampler(w["fanouts"], rng_seed=0).set_graph(edge_ptr, edge_src)
    hops = []
    for batch in range(3):
        input_nodes, _, blocks = sampler.sample_blocks(None, train[batch * B:(batch + 1) * B])
        uniq = input_nodes.long()
        for h, block in enumerate(reversed(blocks)):
            src_l = block.src_local.long()
            src_g = uniq[src_l]
            E = int(src_g.numel())
            tile = torch.arange(E, device=dev) // 2048
            pair = tile * (1 << 32) + src_g
            repeats_in_tile = E - int(torch.unique(pair).numel())
            new_edges = int((src_l >= block.num_dst_nodes()).sum())
            new_ids = block.num_src_nodes() - block.num_dst_nodes()
            hops.append({"batch": batch, "hop": h, "edges": E, "repeat_an_id_of_the_same_tile": repeats_in_tile,
                         "frac": repeats_in_tile / max(E, 1), "edges_of_new_ids": new_edges, "new_ids": new_ids})
            log("batch %d hop %d: %d edges, %d (%.2f %%) repeat an id of their own 2048-edge tile; %d edges mention %d new ids"
                % (batch, h, E, repeats_in_tile, 100 * repeats_in_tile / max(E, 1), new_edges, new_ids))
    # probes per lookup: the table as the sampler sizes it (a power of two of at least 4 x the ids), filled with the
    # last batch's ids by the library's hash and linear probing, replayed on the host
    ids = input_nodes.cpu().numpy().astype(np.uint64)
    slots = 64
    while slots < 4 * ids.size:
        slots *= 2
    shift = 32 - int(np.log2(slots))
    home = ((ids * np.uint64(0x9E3779B1)) & np.uint64(0xFFFFFFFF)) >> np.uint64(shift)
    occupied = bytearray(slots)
    lookups = np.empty(ids.size, dtype=np.int64)  # slots a lookup of the id reads = 1 + its distance from its home slot
    mask = slots - 1
    for i, h in enumerate(home.tolist()):
        p, c = h, 1
        while occupied[p]:
            p = (p + 1) & mask
            c += 1
        occupied[p] = 1
        lookups[i] = c
    stats = {"ids": int(ids.size), "slots": int(slots), "load": ids.size / slots, "mean_probes": float(lookups.mean()),
             "p99_probes": int(np.percentile(lookups, 99)), "max_probes": int(lookups.max()),
             "within_first_64B_line": float(np.mean((home.astype(np.int64) % 8) + lookups <= 8))}
    log("table of %d slots for %d ids (load %.2f): %.2f slots probed per lookup on average, 99 %% within %d, max %d; %.1f %% of the "
        "lookups end in the 64-byte line of their first slot" % (slots, ids.size, stats["load"], stats["mean_probes"], stats["p99_probes"],
                                                               stats["max_probes"], 100 * stats["within_first_64B_line"]))
    print(json.dumps({"metric": "id-map design statistics (intra-tile repeats, probes per lookup), workload c3", "value": stats["mean_probes"],
                      "unit": "slots probed per lookup", "n_gpus": 1, "steps": 3, "warmup": 0, "ms_per_step": None, "higher_is_better": False,
                      "scaling": "weak", "vs_baseline": None, "dtype": "int32", "data": "synthetic",
                      "config": {"workload": DESCRIPTIONS["idmap_stats"]}, "roofline": None, "cpu_baseline": None,
                      "hops": hops, "probing": stats}), flush=True)


def time_dgl_cpu_path(h_ptr, h_src, train, B, fanouts, n_batches):
    """The reference's own CPU sampling path -- DGL's `sample_neighbors` + `to_block` per hop, as its
    DGLNeighborSampler drives them (FusedMapSampler.py:130-148) -- timed on the same mini-batches, if a DGL
    happens to be importable on this box.  It is not part of the image this library is built and tested in, so
    this leg normally reports that it was skipped; nothing is ever installed or downloaded for it."""
    try:
        import dgl  # noqa: F401
        import torch
    except Exception as exc:  # not installed: the usual case
        return {"timed": False, "why": "dgl is not importable here (%s)" % type(exc).__name__}
    try:
        n = int(h_ptr.shape[0]) - 1
        g = dgl.graph(("csc", (torch.from_numpy(h_ptr.astype("int64")), torch.from_numpy(h_src.astype("int64")), torch.tensor([], dtype=torch.int64))),
                      num_nodes=n)
        edges, t = 0, 0.0
        for i in range(n_batches):
            seeds = train[i * B:(i + 1) * B].cpu().long()
            t0 = time.perf_counter()
            for fanout in reversed(fanouts):
                frontier = g.sample_neighbors(seeds, fanout, edge_dir="in", replace=False)
                block = dgl.to_block(frontier, seeds)
                seeds = block.srcdata[dgl.NID]
                edges += int(block.num_edges())
            t += time.perf_counter() - t0
        log("DGL %s on the host: %.3g sampled edges/s" % (dgl.__version__, edges / t))
        return {"timed": True, "version": dgl.__version__, "value": edges / t, "unit": "sampled edges/s",
                "threads": torch.get_num_threads(), "sample": "%d mini-batches of %d seeds" % (n_batches, B)}
    except Exception as exc:
        return {"timed": False, "why": "dgl is importable but the run failed: %r" % (exc,)}


def compare_with_oracle(O, np, g_inp, g_blocks, w_inp, w_blocks, exact_order=True):
    """None if the sampler's output equals the oracle's, else a short description of the first difference."""
    g_inp = g_inp.cpu().numpy()
    if exact_order:
        if not np.array_equal(g_inp, w_inp):
            return "unique list differs (%d vs %d ids)" % (g_inp.size, w_inp.size)
    elif not np.array_equal(np.sort(g_inp), np.sort(w_inp)):
        return "unique ids differ as a set"
    if len(g_blocks) != len(w_blocks):
        return "block count"
    for k, (b, w) in enumerate(zip(g_blocks, w_blocks)):
        if (b.num_src_nodes(), b.num_dst_nodes(), b.num_edges()) != (w["n_src"], w["n_dst"], int(w["src_local"].size)):
            return "block %d: sizes %s vs %s" % (k, (b.num_src_nodes(), b.num_dst_nodes(), b.num_edges()),
                                                  (w["n_src"], w["n_dst"], int(w["src_local"].size)))
        ptr_h, src_h = b.edge_ptr.cpu().numpy(), b.src_local.cpu().numpy()
        if exact_order:
            if not np.array_equal(ptr_h, w["indptr"]):
                return "block %d: row offsets" % k
            if not np.array_equal(src_h, w["src_local"]):
                return "block %d: local ids" % k
            if b.src_global is not None and not np.array_equal(b.src_global.cpu().numpy(), w["src_global"]):
                return "block %d: graph ids" % k
        else:
            # arrival order: any run is a valid map -- the hop's new ids as a set, and its edges in graph ids as a set
            # (rows and local ids are a permutation of the oracle's)
            nd, ns = w["n_dst"], w["n_src"]
            if not np.array_equal(np.sort(g_inp[nd:ns]), np.sort(w_inp[nd:ns])):
                return "block %d: new ids differ as a set" % k
            g64, w64 = g_inp.astype(np.int64), w_inp.astype(np.int64)
            g_dst = np.repeat(np.arange(nd), np.diff(ptr_h))
            w_dst = np.repeat(np.arange(nd), np.diff(w["indptr"]))
            if not np.array_equal(np.sort((g64[g_dst] << 32) | g64[src_h]),
                                  np.sort((w64[w_dst] << 32) | w["src_global"].astype(np.int64))):
                return "block %d: edges in graph ids differ as a set" % k
            if b.src_global is not None and not np.array_equal(b.src_global.cpu().numpy(), g_inp[src_h]):
                return "block %d: graph ids do not match the local ids" % k
        if b._transposed is not None:
            t_ptr, t_dst = (t.cpu().numpy() for t in b.transposed())
            w_ptr, w_dst = O.transpose(ptr_h, src_h, b.num_src_nodes())
            if not np.array_equal(t_ptr, w_ptr):
                return "block %d: transposed row offsets" % k
            row_of = np.repeat(np.arange(b.num_src_nodes(), dtype=np.int64), np.diff(w_ptr))
            if not np.array_equal(np.sort(row_of * (b.num_dst_nodes() + 1) + t_dst), np.sort(row_of * (b.num_dst_nodes() + 1) + w_dst)):
                return "block %d: transposed entries" % k
    return None


def sampling_stage_bytes(blocks, ptr_bytes):
    """Algorithmic bytes of sampling + id-map for one mini-batch: per hop with S seeds, E sampled edges and U new ids,
    sampling reads a seed id and two row offsets per seed and one graph entry per edge and writes the edge's source and the
    block's row offsets, the id-map reads the source, touches one 8-byte slot and writes the local id per edge, and per new
    id fills a slot and writes the unique list."""
    total = 0
    for b in blocks:
        S, E, U = b.num_dst_nodes(), b.num_edges(), b.num_src_nodes() - b.num_dst_nodes()
        total += S * (4 + 2 * ptr_bytes) + (S + 1) * 4 + E * (4 + 4) + E * (4 + 8 + 4) + U * (8 + 4)
    return total


def log(*a):
    print("[bench]", *a, file=sys.stderr, flush=True)


def load_compiled_module():
    """The compiled torch extension module `fastgl` (fastgl-ae_amd/csrc/fastgl_module.cpp), loaded from its file
    under a private name: in this process the name `fastgl` belongs to the Python package."""
    import glob
    import importlib.util
    paths = glob.glob(os.path.join(ROOT, "fastgl-ae_amd", "fastgl_ext", "fastgl*.so"))
    if not paths:
        raise RuntimeError("not built: make -C fastgl-ae_amd/csrc module")
    spec = importlib.util.spec_from_file_location("fastgl", paths[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--sampler", choices=["graph", "eager"], default="eager",
                    help="eager: launch the fused sampler's kernels (default); graph: replay them from a captured HIP graph "
                         "(pays off when the GPU would wait for the host: small batches, one batch at a time)")
    ap.add_argument("--cpu-batches", type=int, default=128, help="mini-batches timed on the CPU oracle (0 = skip)")
    ap.add_argument("--id-order", default="first", choices=["first", "arrival"],
                    help="numbering of new node ids: first occurrence (deterministic, default) or arrival (the reference's rule)")
    ap.add_argument("--readback", choices=["hidden", "first"], default="hidden",
                    help="hidden: enqueue the outermost aggregation before waiting for the batch's sizes (default); "
                         "first: read the sizes back right after sampling, as sample_blocks() does")
    ap.add_argument("--other-order", choices=["on", "off"], default="on",
                    help="also time the steps with the other numbering rule of the id-map (value_other_id_order)")
    ap.add_argument("--other-forms", choices=["on", "off"], default="on",
                    help="also time sample_blocks() with its read-back (value_sample_blocks) and the reference's per-hop call "
                         "pattern through the compiled extension module (value_drop_in_api)")
    ap.add_argument("--extras", choices=["on", "off"], default="on",
                    help="workload c3 only: also run the aggregation microbench (key c4) and the very large shape (key c5) and "
                         "attach their compact records to the line")
    ap.add_argument("--prefetch", type=int, default=2,
                    help="mini-batches that the sampler keeps in flight ahead of the one being aggregated "
                         "(FusedMapSampler.iter_batches; 0: one mini-batch at a time only)")
    ap.add_argument("--c4-eager", action="store_true",
                    help="workload c4: time launches made one by one through the Python binding instead of replaying them "
                         "from a captured graph (the interval then includes the host's cost per call)")
    ap.add_argument("--pmc-copy-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB (a kernel of known traffic, to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures the single-GPU hot path only; run with --gpus 1 "
              "(mini-batches shard over GPUs by seed partition with no exchange between them)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import fastgl

    fastgl.lib()  # fail here, loudly, if the HIP library is not built
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload == "c4":
        print(json.dumps(run_c4(args)), flush=True)
        return
    if args.workload == "ceiling":
        return run_ceiling(args)
    if args.workload == "reuse_ab":
        return run_reuse_ab(args)
    if args.workload == "idmap_stats":
        return run_idmap_stats(args)
    out = run_graph_workload(args, args.workload)
    if args.workload == "c3" and args.extras == "on":
        # Two more configurations ride on the default line, each a compact object: the aggregation microbench
        # (seconds) and, now that this workload's tensors are freed, the very large shape with bf16 features.
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        try:
            out["c4"] = c4_compact(run_c4(args, edge_weighted=False))
        except Exception as exc:  # noqa: BLE001 -- context figures: reported, never fatal to the headline line
            out["c4"] = {"error": repr(exc)}
        gc.collect()
        torch.cuda.empty_cache()
        try:
            out["c5"] = light_summary(run_graph_workload(args, "c5", light=True))
        except Exception as exc:  # noqa: BLE001
            out["c5"] = {"error": repr(exc)}
    print(json.dumps(out), flush=True)
    parity = out.get("parity_checked")
    if parity is not None and not parity["ok"]:
        print("bench.py: the timed mini-batches differ from the oracle's: %s" % parity.get("first_difference"), file=sys.stderr)
        sys.exit(1)


def light_summary(rec):
    """A workload's record cut down to what rides on another workload's line."""
    r = rec["roofline"]
    return {"workload": rec["config"]["workload"], "value": rec["value"], "value_one_at_a_time": rec["value_one_at_a_time"],
            "unit": rec["unit"], "dtype": rec["dtype"],
            "steps": rec["steps"], "warmup": rec["warmup"], "ms_per_step": rec["ms_per_step"],
            "ms_per_step_one_at_a_time": rec["ms_per_step_one_at_a_time"], "stages_ms": rec["stages_ms"],
            "sampled_edges_per_step": rec["config"]["sampled_edges_per_step"], "graph_edges": rec["config"]["graph_edges"],
            "roofline": {k: r[k] for k in ("bound", "achieved", "peak", "unit", "frac", "kernel", "bytes_per_launch", "us_per_launch")},
            "random_read_Gps": rec["random_read_Gps"]}


def run_graph_workload(args, workload, light=False):
    """One of the graph workloads (c1, c2, c3, c5, c5deep): builds the synthetic inputs on the device, times the steps and
    returns the record.  light: the steps and the dominant kernel only (no other forms of the sampler, no CPU leg)."""
    import numpy as np
    import torch

    import fastgl

    dev = torch.device("cuda:0")
    other_order_on = args.other_order == "on" and not light
    other_forms_on = args.other_forms == "on" and not light
    cpu_batches = 0 if light else args.cpu_batches
    w = WORKLOADS[workload]
    N, D, H, B = w["nodes"], w["dim"], w["hidden"], w["batch"]
    fdtype = torch.float32 if w["dtype"] == "f32" else torch.bfloat16
    esz = 4 if fdtype == torch.float32 else 2

    # ---- synthetic inputs, generated on the device ------------------------------------
    t0 = time.time()
    edge_ptr, edge_src = fastgl.graph.rmat_csr(N, w["draws"], seed=0, device=dev)
    torch.cuda.synchronize()
    n_graph_edges = int(edge_src.numel())
    log("graph: %d nodes, %d directed edges, built in %.1fs" % (N, n_graph_edges, time.time() - t0))
    torch.cuda.empty_cache()
    t0 = time.time()
    gen = torch.Generator(device=dev).manual_seed(0)
    feat = torch.empty((N, D), dtype=fdtype, device=dev)
    for lo in range(0, N, 1 << 22):
        hi = min(N, lo + (1 << 22))
        feat[lo:hi] = torch.randn((hi - lo, D), generator=gen, device=dev, dtype=torch.float32).to(fdtype)
    train = torch.randperm(N, generator=gen, device=dev)[:w["train"]].to(torch.int32)
    n_batches = max(1, w["train"] // B)
    torch.cuda.synchronize()
    log("features %s x %d %s and %d training seeds in %.1fs" % (N, D, w["dtype"], w["train"], time.time() - t0))

    def make_sampler(graph_slots):
        return fastgl.FusedMapSampler(w["fanouts"], rng_seed=0, id_order=args.id_order,
                                      graph_slots=graph_slots).set_graph(edge_ptr, edge_src)

    # --sampler graph: the fused path's launch sequence is replayed from a captured HIP graph.  The mode is
    # checked here against the eager path on a few mini-batches and abandoned, loudly, if capture fails or
    # any result differs.
    sampler_mode = args.sampler
    sampler = make_sampler(2 if sampler_mode == "graph" else 0)
    if sampler_mode == "graph":
        try:
            check = make_sampler(0)
            for i in range(4):
                got, want = sampler.sample_blocks(None, train[i * B:i * B + B]), check.sample_blocks(None, train[i * B:i * B + B])
                same = torch.equal(got[0], want[0]) and all(torch.equal(a.edge_ptr, b.edge_ptr) and torch.equal(a.src_local, b.src_local)
                                                            for a, b in zip(got[2], want[2]))
                if not same:
                    raise RuntimeError("graph replay differs from the eager path on mini-batch %d" % i)
            del check, got, want
        except Exception as exc:  # noqa: BLE001 -- any failure of the optional mode falls back to the eager path
            log("graph-replay sampler abandoned: %s" % exc)
            sampler_mode = "eager (graph replay abandoned: %s)" % exc
            sampler = make_sampler(0)
    main_sampler = sampler
    L = len(w["fanouts"])
    # hidden activations / upstream gradients of the inner layers: synthetic; sized from a probe
    # batch with head-room (the worst-case bound would be tens of GB for deep fanouts) and grown on demand
    _, _, probe = sampler.sample_blocks(None, train[:B])
    inner = {"rows": 0}

    def inner_buffers(rows):
        if rows > inner["rows"]:
            inner["rows"] = int(rows * 1.5) + 1
            inner["hid"] = torch.randn((inner["rows"], H), generator=gen, device=dev, dtype=torch.float32).to(fdtype)
            inner["grad"] = torch.randn((inner["rows"], H), generator=gen, device=dev, dtype=torch.float32).to(fdtype)
        return inner["hid"], inner["grad"]

    inner_buffers(max(b.num_src_nodes() for b in probe[1:]) if L > 1 else 1)
    del probe

    ev = lambda: torch.cuda.Event(enable_timing=True)

    parity_keep = []  # (seed batch, random stream, outputs) of the first timed steps, compared with the oracle in the CPU leg
    N_PARITY = 4

    stage_bytes = []  # algorithmic bytes of the sampling stage, per recorded step (of every sampler that ran the steps)

    def step(i, rec=None, sampler=sampler):
        seeds = train[(i % n_batches) * B:(i % n_batches) * B + B]
        stream_base = (sampler.batches * 64) & 0xFFFFFFFF  # the Philox streams this mini-batch draws from
        e0, e1, e2, e3, e4 = ev(), ev(), ev(), ev(), ev()
        e0.record()
        if args.readback == "hidden":
            # the outermost aggregation is enqueued on the bound-sized block with its row count on the device,
            # and the host's wait for the batch's sizes hides behind it
            pend = sampler.begin_sample(seeds)
            e1.record()
            out0 = fastgl.aggregate(pend.outer_edge_ptr, pend.outer_src_global, feat, mode="mean", zero_policy="zeros",
                                    n_rows=pend.outer_n_dst_bound, n_rows_dev=pend.outer_n_dst, longest_row=pend.outer_fanout)
            e2.record()
            input_nodes, _, blocks = pend.finish()
            b0 = blocks[0]
            if pend.redone:  # the batch outgrew its buffers and was sampled again: aggregate again
                out0 = fastgl.aggregate(b0.edge_ptr, b0.src_global, feat, mode="mean", zero_policy="zeros")
            out0 = out0[:b0.num_dst_nodes()]
        else:
            input_nodes, _, blocks = sampler.sample_blocks(None, seeds)  # includes the one count read-back
            e1.record()
            b0 = blocks[0]
            out0 = fastgl.aggregate(b0.edge_ptr, b0.src_global, feat, mode="mean", zero_policy="zeros")
            e2.record()
        outs = [out0]
        hid, grad = inner_buffers(max([b.num_src_nodes() for b in blocks[1:]] + [1]))
        for b in blocks[1:]:
            outs.append(fastgl.aggregate(b.edge_ptr, b.src_local, hid[:b.num_src_nodes()], mode="mean", zero_policy="zeros"))
        e3.record()
        fastgl.transpose_blocks(blocks[1:])  # all inner blocks in the launches that one transpose takes
        for b in blocks[1:]:
            t_ptr, t_idx = b.transposed()
            outs.append(fastgl.aggregate(t_ptr, t_idx, grad[:b.num_dst_nodes()], mode="colmean_ptr", zero_policy="zeros",
                                         col_norm=b.edge_ptr))
        e4.record()
        if rec is not None:
            rec.append(((sum(b.num_edges() for b in blocks), b0.num_edges(), b0.num_dst_nodes()), (e0, e1, e2, e3, e4)))
            stage_bytes.append(sampling_stage_bytes(blocks, 8 if edge_ptr.dtype == torch.int64 else 4))
            keep.append(b0.clone() if sampler.graph_slots else b0)  # (a graph-replay slot is overwritten two batches on)
            del keep[:-4]  # a few outermost blocks are kept for the kernel-time replay below
            if sampler is main_sampler and len(parity_keep) < N_PARITY and cpu_batches > 0:
                # what this timed step produced, kept as it is (references, or copies where a replay slot would be
                # overwritten) for the comparison with the oracle after the timing
                if sampler.graph_slots:
                    parity_keep.append((i % n_batches, stream_base, input_nodes.clone(), [b.clone() for b in blocks]))
                else:
                    parity_keep.append((i % n_batches, stream_base, input_nodes, blocks))
        return blocks

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    rec, keep = [], []
    t_start = time.perf_counter()
    last_blocks = None
    for i in range(args.steps):
        last_blocks = step(args.warmup + i, rec)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t_start

    # ---- the same steps with the other numbering rule of the id-map (context for `value`) ----------------
    other_order = "arrival" if args.id_order == "first" else "first"
    value_other = None
    if sampler_mode == "eager" and other_order_on:
        keep_main = list(keep)
        alt = fastgl.FusedMapSampler(w["fanouts"], rng_seed=0, id_order=other_order).set_graph(edge_ptr, edge_src)
        for i in range(args.warmup):
            step(i, None, alt)
        torch.cuda.synchronize()
        rec_alt = []
        for i in range(args.steps):
            step(args.warmup + i, rec_alt, alt)
        torch.cuda.synchronize()
        keep[:] = keep_main  # (the replay below uses the main run's blocks)
        alt_edges = sum(r[0][0] for r in rec_alt)
        alt_ms = sum(r[1][0].elapsed_time(r[1][1]) for r in rec_alt)
        value_other = alt_edges / (alt_ms * 1e-3)
        log("id order %s: %.3g sampled edges/s (sample+idmap %.3f ms)" % (other_order, value_other, alt_ms / args.steps))
        del alt, rec_alt

    # ---- the same steps with a sampler that hands over the blocks only (transposed="none"): the transposed inner
    # blocks are then built by the batch transpose behind the forward pass, five launches, as a caller without
    # the all-in-one call would; shows what carrying them inside the sampling call costs that stage and saves the step
    blocks_only = None
    if sampler_mode == "eager" and other_order_on and L > 1:
        keep_main = list(keep)
        alt = fastgl.FusedMapSampler(w["fanouts"], rng_seed=0, id_order=args.id_order, transposed="none").set_graph(edge_ptr, edge_src)
        for i in range(args.warmup):
            step(i, None, alt)
        torch.cuda.synchronize()
        rec_alt = []
        for i in range(args.steps):
            step(args.warmup + i, rec_alt, alt)
        torch.cuda.synchronize()
        keep[:] = keep_main
        alt_edges = sum(r[0][0] for r in rec_alt)
        t01 = sum(r[1][0].elapsed_time(r[1][1]) for r in rec_alt)
        t34 = sum(r[1][3].elapsed_time(r[1][4]) for r in rec_alt)
        t04 = sum(r[1][0].elapsed_time(r[1][4]) for r in rec_alt)
        blocks_only = {"value": alt_edges / (t01 * 1e-3), "sample_idmap_ms": t01 / args.steps,
                       "default_gpu_ms_per_step": sum(r[1][0].elapsed_time(r[1][4]) for r in rec) / args.steps,
                       "transpose_agg_bwd_inner_ms": t34 / args.steps, "gpu_ms_per_step": t04 / args.steps,
                       "what": "the sampler hands over the blocks without their transposed form "
                               "(FusedMapSampler(transposed='none')); the inner blocks are transposed by "
                               "fgl_block_transpose_batch in front of the backward gathers"}
        log("blocks only: %.3g sampled edges/s (sample+idmap %.3f ms, transpose+bwd %.3f ms, GPU time of a step %.3f ms)"
            % (blocks_only["value"], blocks_only["sample_idmap_ms"], blocks_only["transpose_agg_bwd_inner_ms"],
               blocks_only["gpu_ms_per_step"]))
        del alt, rec_alt

    # ---- the same mini-batches through the two other forms of the sampler (context for `value`) -------------
    # value_sample_blocks: FusedMapSampler.sample_blocks(), i.e. the fused call followed at once by the one
    # read-back of the batch's sizes (the host's wait is inside the interval).
    # value_drop_in_api: the reference's own call pattern -- sample_node + transfer_edge_id per hop, each returning
    # exact-size tensors (FusedMapSampler.py:72-107) -- through the compiled extension module.
    def time_sampler(fn):
        for i in range(args.warmup):
            fn(train[(i % n_batches) * B:(i % n_batches) * B + B])
        torch.cuda.synchronize()
        edges, ms = 0, 0.0
        for i in range(args.steps):
            seeds = train[((args.warmup + i) % n_batches) * B:((args.warmup + i) % n_batches) * B + B]
            a, b = ev(), ev()
            a.record()
            n_e = fn(seeds)
            b.record()
            torch.cuda.synchronize()
            edges += n_e
            ms += a.elapsed_time(b)
        return edges / (ms * 1e-3), ms / args.steps

    value_sample_blocks = value_drop_in = None
    if other_forms_on:
        plain = fastgl.FusedMapSampler(w["fanouts"], rng_seed=0, id_order=args.id_order).set_graph(edge_ptr, edge_src)
        value_sample_blocks, ms_sb = time_sampler(lambda seeds: sum(b.num_edges() for b in plain.sample_blocks(None, seeds)[2]))
        log("sample_blocks() with its read-back: %.3g sampled edges/s (%.3f ms per mini-batch)" % (value_sample_blocks, ms_sb))
        del plain
        try:
            ext = load_compiled_module()
        except Exception as exc:  # noqa: BLE001 -- reported, not fatal: the figure is context
            log("compiled module unavailable (%s): value_drop_in_api -> null" % exc)
            ext = None
        if ext is not None:
            nodes_num = int(edge_ptr.numel()) - 1

            def reference_loop(seeds):  # FusedMapSampler.py:63-109 without the DGL block objects
                seed_nodes_acc, dst_nodes, total = seeds, int(seeds.size(0)), 0
                for block_index, fanout in enumerate(reversed(w["fanouts"])):
                    src_out, dst_out, _ = ext.sample_node(edge_src, edge_src, edge_ptr, seed_nodes_acc.int(), dst_nodes, fanout)
                    edge_nums = src_out.size(0)
                    dst_unique = seeds if block_index == 0 else seed_nodes_acc
                    max_src = nodes_num if fanout * dst_unique.size(0) > nodes_num else fanout * dst_unique.size(0)
                    _, _, seed_nodes_acc = ext.transfer_edge_id(src_out, dst_out, dst_unique, dst_nodes, dst_nodes + edge_nums,
                                                                max_src, edge_nums)
                    dst_nodes = int(seed_nodes_acc.size(0))
                    total += edge_nums
                return total

            value_drop_in, ms_di = time_sampler(reference_loop)
            log("reference call pattern through the compiled module: %.3g sampled edges/s (%.3f ms per mini-batch)"
                % (value_drop_in, ms_di))

    # ---- the sampler as a prefetching iterator (FusedMapSampler.iter_batches, the role of the DataLoader that the
    # reference plugs its sampler into: train_fastgl.py:109-122,248-258, prefetch_factor 2): `prefetch` mini-batches are
    # sampled ahead, each on a stream of its own, so that the small hops of one -- latency chains on a mostly idle
    # chip -- run under the large kernels of another and under the aggregation.  Two timings, each a pass of its own
    # (pipeline fill and drain inside the interval), wall clock between two device synchronisations:
    #   the sampling stage alone (nothing else on the GPU, every mini-batch's read-back included) -> edges per second;
    #   whole steps (sampling + the aggregation of every block, forward and backward)             -> ms per step.
    pipelined = None
    K = args.steps
    if args.prefetch > 0:
        def aggregate_only(blocks):
            b0 = blocks[0]
            fastgl.aggregate(b0.edge_ptr, b0.src_global, feat, mode="mean", zero_policy="zeros")
            hid, grad = inner_buffers(max([b.num_src_nodes() for b in blocks[1:]] + [1]))
            for b in blocks[1:]:
                fastgl.aggregate(b.edge_ptr, b.src_local, hid[:b.num_src_nodes()], mode="mean", zero_policy="zeros")
            fastgl.transpose_blocks(blocks[1:])
            for b in blocks[1:]:
                t_ptr, t_idx = b.transposed()
                fastgl.aggregate(t_ptr, t_idx, grad[:b.num_dst_nodes()], mode="colmean_ptr", zero_policy="zeros",
                                 col_norm=b.edge_ptr)

        pipe = fastgl.FusedMapSampler(w["fanouts"], rng_seed=0, id_order=args.id_order).set_graph(edge_ptr, edge_src)
        batch_of = lambda i: train[(i % n_batches) * B:(i % n_batches) * B + B]
        for _, _, blocks in pipe.iter_batches([batch_of(i) for i in range(max(args.warmup, 2 * args.prefetch))], prefetch=args.prefetch):
            aggregate_only(blocks)  # warm-up: every lane has learned its buffer sizes
        first = pipe.batches
        n_sampling = max(K, 100 if not light else K)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        pipe_edges = 0
        for j, (inp, _, blocks) in enumerate(pipe.iter_batches([batch_of(first + i) for i in range(n_sampling)], prefetch=args.prefetch)):
            pipe_edges += sum(b.num_edges() for b in blocks)
            if j < 2 and cpu_batches > 0 and not pipe.graph_slots:  # (also held against the oracle below)
                parity_keep.append(((first + j) % n_batches, ((first + j) * 64) & 0xFFFFFFFF, inp, blocks))
        torch.cuda.synchronize()
        t_sampling = time.perf_counter() - t0
        first = pipe.batches
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _, _, blocks in pipe.iter_batches([batch_of(first + i) for i in range(K)], prefetch=args.prefetch):
            aggregate_only(blocks)
        torch.cuda.synchronize()
        t_steps = time.perf_counter() - t0
        pipelined = {"prefetch": args.prefetch, "value": pipe_edges / t_sampling, "sampling_batches": n_sampling,
                     "ms_per_batch_sampling": t_sampling / n_sampling * 1e3, "ms_per_step": t_steps / K * 1e3}
        log("prefetching sampler, %d mini-batches in flight: sampling alone %.3g sampled edges/s (%.3f ms per mini-batch over %d), "
            "whole steps %.3f ms per step" % (args.prefetch, pipelined["value"], pipelined["ms_per_batch_sampling"], n_sampling,
                                              pipelined["ms_per_step"]))
        del pipe

    # ---- duration of the dominant kernel -------------------------------------------------
    # The stage interval above starts right after the sampler's host read-back, when the queue
    # is empty, so it contains the host's launch latency.  For the roofline the same launches
    # (same kernel, same blocks as the timed steps) are replayed back to back between two HIP
    # events on the stream they run on: the queue stays full and the interval is kernel time.
    out_buf = torch.empty((max(b.num_dst_nodes() for b in keep), D), dtype=fdtype, device=dev)
    ra, rb = ev(), ev()
    torch.cuda.synchronize()
    ra.record()
    replay_bytes = 0
    for r in range(args.steps):
        b0 = keep[r % len(keep)]
        fastgl.aggregate(b0.edge_ptr, b0.src_global, feat, mode="mean", zero_policy="zeros", out=out_buf[:b0.num_dst_nodes()])
        replay_bytes += b0.num_edges() * D * esz + b0.num_dst_nodes() * D * esz + 4 * b0.num_edges() + 4 * (b0.num_dst_nodes() + 1)
    rb.record()
    torch.cuda.synchronize()
    t_kernel0 = ra.elapsed_time(rb)

    # ---- the same sampling without graph replay (context for `value`) -----------------------
    value_eager = None
    if sampler.graph_slots:
        eager = make_sampler(0)
        for i in range(3):
            eager.sample_blocks(None, train[i * B:i * B + B])
        ea, eb = ev(), ev()
        eager_edges, eager_ms = 0, 0.0
        for i in range(args.steps):
            seeds = train[((args.warmup + i) % n_batches) * B:((args.warmup + i) % n_batches) * B + B]
            torch.cuda.synchronize()
            ea.record()
            _, _, blocks = eager.sample_blocks(None, seeds)
            eb.record()
            torch.cuda.synchronize()
            eager_ms += ea.elapsed_time(eb)
            eager_edges += sum(b.num_edges() for b in blocks)
        value_eager = eager_edges / (eager_ms * 1e-3)
        del eager, blocks
        log("sampling without graph replay: %.3g edges/s" % value_eager)

    # ---- context: what a plain streaming copy reaches on this box ---------------------------
    cp_src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    cp_dst = torch.empty_like(cp_src)
    cp_dst.copy_(cp_src)
    ca, cb = ev(), ev()
    torch.cuda.synchronize()
    ca.record()
    for _ in range(10):
        cp_dst.copy_(cp_src)
    cb.record()
    torch.cuda.synchronize()
    stream_gbps = 10 * 2 * (1 << 30) / (ca.elapsed_time(cb) * 1e-3) / 1e9  # bytes read + bytes written
    del cp_src, cp_dst
    log("1 GiB device copy: %.0f GB/s (read + write)" % stream_gbps)
    # ---- context: the rate of independent random 4-byte reads from the graph's edge array (what
    # bounds the sampling kernels), measured with a library gather of 16 M random positions
    ra_idx = torch.randint(0, edge_src.numel(), (1 << 24,), device=dev, dtype=torch.int64)
    ra_out = torch.empty(1 << 24, dtype=edge_src.dtype, device=dev)
    torch.index_select(edge_src, 0, ra_idx, out=ra_out)
    ca, cb = ev(), ev()
    torch.cuda.synchronize()
    ca.record()
    for _ in range(5):
        torch.index_select(edge_src, 0, ra_idx, out=ra_out)
    cb.record()
    torch.cuda.synchronize()
    random_read_gps = 5 * (1 << 24) / (ca.elapsed_time(cb) * 1e-3) / 1e9
    del ra_idx, ra_out
    log("random 4-byte reads from the edge array: %.1f G/s" % random_read_gps)

    if args.pmc_copy_mib > 0:
        a = torch.zeros(args.pmc_copy_mib << 20, dtype=torch.uint8, device=dev)
        b = torch.empty_like(a)
        torch.cuda.synchronize()
        b.copy_(a)  # __amd_rocclr_copyBuffer: reads and writes exactly pmc_copy_mib MiB
        torch.cuda.synchronize()
        c = a.view(torch.float32) * 1.0  # an ordinary elementwise kernel: reads and writes the same amount
        torch.cuda.synchronize()
        # the aggregation kernel itself as a plain copy: every row has exactly one neighbour, itself
        # (sum mode, D=128 fp32): reads and writes pmc_copy_mib MiB of rows with the same instructions
        rows = (args.pmc_copy_mib << 20) // (128 * 4)
        x = a.view(torch.float32)[:rows * 128].view(rows, 128)
        ident_ptr = torch.arange(rows + 1, dtype=torch.int32, device=dev)
        ident_idx = torch.arange(rows, dtype=torch.int32, device=dev)
        y = fastgl.aggregate(ident_ptr, ident_idx, x, mode="sum", zero_policy="zeros", mapping="row")
        torch.cuda.synchronize()
        del a, b, c, x, y

    # ---- reduce -------------------------------------------------------------------------
    tot_edges = 0
    t_sample = t_agg0 = t_fwd_in = t_bwd = 0.0
    bytes_agg0 = 0
    for (n_e_all, e_, nd), (e0, e1, e2, e3, e4) in rec:
        tot_edges += n_e_all
        t_sample += e0.elapsed_time(e1)
        t_agg0 += e1.elapsed_time(e2)
        t_fwd_in += e2.elapsed_time(e3)
        t_bwd += e3.elapsed_time(e4)
        bytes_agg0 += e_ * D * esz + nd * D * esz + 4 * e_ + 4 * (nd + 1)  # gathered rows + output + indices + offsets
    K = args.steps
    edges_per_s = tot_edges / (t_sample * 1e-3)
    stage_bytes_per_batch = sum(stage_bytes[:len(rec)]) / max(1, len(rec))  # (the main sampler's steps come first)
    agg_gbps = replay_bytes / (t_kernel0 * 1e-3) / 1e9
    bytes_agg0 = replay_bytes
    log("last batch blocks:", last_blocks)
    log("per step: sample+idmap %.3f ms, agg fwd outer %.3f ms, agg fwd inner %.3f ms, transpose+bwd %.3f ms, wall %.3f ms"
        % (t_sample / K, t_agg0 / K, t_fwd_in / K, t_bwd / K, wall / K * 1e3))

    # ---- CPU baseline: the oracle on a bounded sample of the same workload ------------
    cpu = None
    parity = None
    if cpu_batches > 0:
        from oracle import oracle as O
        t0 = time.time()
        h_ptr, h_src = edge_ptr.cpu().numpy(), edge_src.cpu().numpy()
        log("graph copied to the host in %.1fs; oracle threads: %d" % (time.time() - t0, O.num_threads()))
        cpu_edges, cpu_t, cpu_t_seq, agg_t, agg_bytes = 0, 0.0, 0.0, 0.0, 0
        for i in range(cpu_batches):
            seeds = train[i * B:(i + 1) * B].cpu().numpy()
            t0 = time.perf_counter()
            inp, oblocks = O.sample_blocks(h_ptr, h_src, seeds, w["fanouts"], 0, i * 64, parallel_idmap=True)
            cpu_t += time.perf_counter() - t0
            t0 = time.perf_counter()
            O.sample_blocks(h_ptr, h_src, seeds, w["fanouts"], 0, i * 64, parallel_idmap=False)
            cpu_t_seq += time.perf_counter() - t0
            cpu_edges += sum(int(b["src_local"].size) for b in oblocks)
            ob = oblocks[0]
            xb = feat.index_select(0, torch.from_numpy(inp).to(dev).long()).float().cpu().numpy()  # rows of the input nodes
            t0 = time.perf_counter()
            O.aggregate(ob["indptr"], ob["src_local"], xb, "mean", 1, out_dtype=np.float32)
            agg_t += time.perf_counter() - t0
            e_, nd = int(ob["src_local"].size), int(ob["n_dst"])
            agg_bytes += e_ * D * 4 + nd * D * 4 + 4 * e_ + 4 * (nd + 1)
        cpu = {"value": cpu_edges / cpu_t, "unit": "sampled edges/s", "cores": O.num_threads(), "kind": "port",
               "sample": "%d mini-batches of %d seeds of the same workload through the CPU oracle "
                         "(OpenMP sampling + OpenMP id-map: CAS insert, first-occurrence numbering by prefix sum; "
                         "value_sequential_idmap = the same with a single-threaded hash-map id-map); "
                         "aggregation = fp32 OpenMP row gather of the outermost block" % (cpu_batches, B),
               "value_sequential_idmap": cpu_edges / cpu_t_seq,
               "aggregation_GBps": agg_bytes / agg_t / 1e9, "host_cpus": os.cpu_count()}
        log("cpu baseline: %.3g edges/s (%d threads), aggregation %.1f GB/s" % (cpu["value"], cpu["cores"], cpu["aggregation_GBps"]))
        # ---- parity of the timed path: the first timed steps' own outputs against the oracle on the same seeds and
        # random streams -- unique list, every block's offsets and local ids, the outermost block's graph ids, and the
        # transposed inner blocks (offsets, and each row's entries as a set) -- bit for bit
        t0 = time.time()
        first_difference = None
        for bi, sb, g_inp, g_blocks in parity_keep:
            seeds = train[bi * B:(bi + 1) * B].cpu().numpy()
            w_inp, w_blocks = O.sample_blocks(h_ptr, h_src, seeds, w["fanouts"], 0, sb)
            first_difference = compare_with_oracle(O, np, g_inp, g_blocks, w_inp, w_blocks, exact_order=args.id_order == "first")
            if first_difference is not None:
                first_difference = "seed batch %d, stream %d: %s" % (bi, sb, first_difference)
                break
        parity = {"batches": len(parity_keep), "ok": first_difference is None,
                  "what": "the first timed sequential steps' outputs (the steady-state path: learned buffer sizes, small table, no "
                          "fill, begin_sample/finish) and the first two mini-batches of the timed prefetching run (two in flight on "
                          "two streams) vs the CPU oracle on the same seeds and Philox streams: unique list, block offsets, "
                          "local ids, outermost graph ids, transposed inner blocks; bit-exact"
                          + ("" if args.id_order == "first" else " after sorting the new ids (arrival order)")}
        if first_difference is not None:
            parity["first_difference"] = first_difference
        log("parity of %d timed mini-batches against the oracle: %s (%.1fs)"
            % (len(parity_keep), "ok" if first_difference is None else "MISMATCH " + first_difference, time.time() - t0))
        cpu["dgl"] = time_dgl_cpu_path(h_ptr, h_src, train, B, w["fanouts"], min(cpu_batches, 16))

    out = {
        "metric": "sampled edges/s (sample+id_map) + aggregation HBM GB/s (% peak), 1 MI355X",
        "value": pipelined["value"] if pipelined else edges_per_s,
        "unit": "sampled edges/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": args.warmup,
        "ms_per_step": pipelined["ms_per_step"] if pipelined else wall / K * 1e3,
        "value_is": ("throughput of the sampling stage (all hops, id-map, transposed inner blocks, one host read-back per "
                     "mini-batch) run as FusedMapSampler.iter_batches runs it in training: %d mini-batches in flight, each on a "
                     "stream of its own; %d mini-batches, wall clock between two device synchronisations, nothing else on the "
                     "GPU.  value_one_at_a_time is the same stage with one mini-batch in flight (HIP events around the stage "
                     "inside sequential steps); ms_per_step is K whole steps with the prefetching sampler, "
                     "ms_per_step_one_at_a_time the sequential steps that stages_ms is taken from"
                     % (pipelined["prefetch"], pipelined["sampling_batches"])) if pipelined else
                    "the sampling stage with one mini-batch in flight (HIP events around the stage inside sequential steps)",
        "value_one_at_a_time": edges_per_s,
        "ms_per_step_one_at_a_time": wall / K * 1e3,
        "pipelined": pipelined,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w["dtype"],
        "data": "synthetic",
        "config": {"workload": DESCRIPTIONS[workload], "graph_edges": n_graph_edges,
                   "sampled_edges_per_step": tot_edges / K,
                   "note": "seeds are drawn uniformly from an R-MAT graph without degree noise, so most of them have degree 0-1 "
                           "(the first hop expands 8192 seeds to ~10 K edges): a mini-batch samples ~1.6 M edges, not the "
                           "8.6 M that the fanouts would allow",
                   "sampler": sampler_mode, "id_order": "first-occurrence (deterministic)" if args.id_order == "first" else "arrival (run-dependent)",
                   "step": "sample+id-map all hops (the transposed inner blocks come out of the same call); mean aggregation fwd on "
                           "every block (outermost gathers from the full feature table); bwd gather over the transposed inner "
                           "blocks; no dense layers",
                   "readback": ("the batch's sizes are stored into pinned host memory by the sampling kernels; the host waits for them while the outermost aggregation runs "
                                "(sample_idmap = the sampling kernels' own time)") if args.readback == "hidden" else
                               "the batch's sizes are read back before anything else is enqueued (inside sample_idmap)"},
        "stages_ms_are": "per stage of the sequential steps (one mini-batch at a time), HIP events on the launch stream",
        "stages_ms": {"sample_idmap": t_sample / K, "agg_fwd_outer": t_agg0 / K, "agg_fwd_inner": t_fwd_in / K,
                      "transpose_agg_bwd_inner": t_bwd / K},
        "sampling": {"algorithmic_bytes_per_mini_batch": stage_bytes_per_batch,
                     "algorithmic_bytes_per_edge": stage_bytes_per_batch / (tot_edges / K),
                     "GBps_one_at_a_time": stage_bytes_per_batch / (t_sample / K * 1e-3) / 1e9,
                     "GBps": (stage_bytes_per_batch / (pipelined["ms_per_batch_sampling"] * 1e-3) / 1e9) if pipelined else None,
                     "frac_peak": (stage_bytes_per_batch / (pipelined["ms_per_batch_sampling"] * 1e-3) / 1e9 / HBM_PEAK_GBPS)
                                  if pipelined else stage_bytes_per_batch / (t_sample / K * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                     "bound": "not bytes: the rate of random accesses (one 4-byte graph read per edge, ~38 G/s here: random_read_Gps) "
                              "and of atomics (one 64-bit compare-and-swap per new id, 23-25 G/s on this chip); the byte rate is "
                              "reported because the stage is priced per edge in bytes elsewhere"},
        "aggregation": {"GBps": agg_gbps, "frac_peak": agg_gbps / HBM_PEAK_GBPS,
                        "stream_copy_GBps": stream_gbps, "frac_of_stream_copy": agg_gbps / stream_gbps},
        "random_read_Gps": random_read_gps,
        "value_eager_launch": value_eager,
        "value_sample_blocks": value_sample_blocks,
        "value_drop_in_api": value_drop_in,
        "value_other_id_order": {"id_order": other_order, "value": value_other},
        "value_blocks_only": blocks_only,
        "speedup_vs_cpu": None if cpu is None else (pipelined["value"] if pipelined else edges_per_s) / cpu["value"],
        "speedup_vs_cpu_one_at_a_time": None if cpu is None else edges_per_s / cpu["value"],
        "roofline": {"bound": "hbm", "achieved": agg_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": agg_gbps / HBM_PEAK_GBPS,
                     "traffic": traffic_from_profile(workload, bytes_agg0 / K),
                     "achieved_is": "an effective rate: algorithmic bytes (every sampled edge counted as one row fetch) / kernel time; "
                                    "frac_of_peak_by_traffic = the counter-derived bytes / the same time / peak; "
                                    "traffic = bytes per launch that the L2s fetch and write (rocprofv3 FETCH_SIZE / WRITE_SIZE, scaled): "
                                    "repeated rows that hit in L2 are not in it, hits in the memory-side Infinity Cache still are",
                     "kernel": ("aggregate_kernel<float,4,32,MEAN>" if w["dtype"] == "f32" and D == 128 else
                                "aggregate_kernel, %s rows of %d columns, MEAN" % (w["dtype"], D)) + " (outermost block, forward)",
                     "bytes_per_launch": bytes_agg0 / K, "us_per_launch": t_kernel0 / K * 1e3},
        "cpu_baseline": cpu,
        "parity_checked": parity,
    }
    r = out["roofline"]
    # the same launch priced by what the counters saw move instead of by the algorithmic bytes
    r["frac_of_peak_by_traffic"] = None if r["traffic"] is None else r["traffic"] / (r["us_per_launch"] * 1e-6) / 1e9 / HBM_PEAK_GBPS
    return out


if __name__ == "__main__":
    main()
