#!/usr/bin/env python3
"""Benchmark of the per-GPU hot path on one MI355X: multi-layer row-wise
neighbour sampling + unique/relabel + ChunkTensor feature gather.

A step = one batch: ChunkTensorSampler.sample_blocks over fanouts [15,10,5]
(hops run over the reversed list) followed by one _CAPI_index of the final
frontier.  Inputs (graph, features, seed batches) are resident in HBM before the
timed region.  Prints ONE JSON line.

  python bench.py --gpus 1 --steps 50 --warmup 5
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
# HBM bytes per gathered 400-byte row of workload c1, from rocprofv3 FETCH_SIZE (x2.0 after
# calibration against a plain copy) and WRITE_SIZE (x1.0): 378.3 MB + 288.2 MB per 719,002 rows
C1_GATHER_TRAFFIC_BYTES_PER_ROW = (378.3e6 + 288.2e6) / 719002.0

WORKLOADS = {
    # BASELINE.json configs[1]: the configuration the metric is quoted on
    "c1": dict(nodes=2_449_029, edges=123_718_280, max_deg=17_000, deg1_frac=0.05, feat_dim=100,
               feat_dtype="float32", batch=1024, fanouts=[15, 10, 5], replace=False, graph_seed=20240602),
    # BASELINE.json configs[0] (CPU-runnable plumbing case), used by --workload c0
    "c0": dict(nodes=10_000, edges=200_000, max_deg=1_000, deg1_frac=0.0, feat_dim=128,
               feat_dtype="float32", batch=1024, fanouts=[10, 5], replace=False, graph_seed=20240601),
}


def make_degrees(rng, n, e, max_deg, deg1_frac):
    """Power-law in-degrees in [1, max_deg] with sum exactly e and about deg1_frac ones."""
    raw = (rng.pareto(1.25, size=n) + 1.0)
    ones = rng.random(n) < deg1_frac
    lo, hi = 0.1, 1000.0
    for _ in range(60):  # bisect the scale so the clipped sum matches e
        mid = 0.5 * (lo + hi)
        deg = np.clip(np.floor(raw * mid), 2, max_deg)
        deg[ones] = 1
        if deg.sum() > e:
            hi = mid
        else:
            lo = mid
    deg = np.clip(np.floor(raw * lo), 2, max_deg)
    deg[ones] = 1
    deg = deg.astype(np.int64)
    rest = int(e - deg.sum())
    if rest > 0:
        cand = np.flatnonzero((deg > 1) & (deg < max_deg - 1))
        pick = rng.choice(cand, size=rest, replace=rest > cand.size)
        np.add.at(deg, pick, 1)
    assert deg.sum() == e, (deg.sum(), e)
    return deg


def make_graph(cfg):
    rng = np.random.default_rng(cfg["graph_seed"])
    n, e = cfg["nodes"], cfg["edges"]
    deg = make_degrees(rng, n, e, cfg["max_deg"], cfg["deg1_frac"])
    indptr = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(deg, out=indptr[1:])
    g = torch.Generator().manual_seed(cfg["graph_seed"])
    indices = torch.randint(0, n, (e,), generator=g, dtype=torch.int64)  # sources uniform
    g = torch.Generator().manual_seed(cfg["graph_seed"] + 1)
    feats = torch.randn((n, cfg["feat_dim"]), generator=g, dtype=getattr(torch, cfg["feat_dtype"]))
    return torch.from_numpy(indptr), indices, feats, deg


def make_batches(cfg, count):
    g = torch.Generator().manual_seed(cfg["graph_seed"] + 2)
    return [torch.randint(0, cfg["nodes"], (cfg["batch"],), generator=g, dtype=torch.int64) for _ in range(count)]


def algorithmic_bytes(stats, feat_dim, feat_bytes, w_id=8, w_ptr=8):
    """Bytes the path must move per batch: sampling B_s, relabel B_u per hop, gather B_g."""
    b_s = b_u = 0
    for s, nnz, u in stats["hops"]:
        b_s += s * w_id + 2 * s * w_ptr + nnz * w_id + nnz * 2 * w_id
        b_u += (s + nnz) * w_id + u * w_id + 4 * nnz * w_id
    f = stats["frontier"]
    b_g = f * (2 * feat_dim * feat_bytes + w_id)
    return b_s, b_u, b_g


def cpu_baseline(cfg, indptr, indices, feats, batches, budget_s=12.0):
    """The CPU oracle (a port of the reference algorithm, OpenMP over seed rows) plus
    torch.index_select, timed on this machine's host cores on a bounded sample of the
    same batches."""
    from oracle import oracle
    oracle.build()
    threads = min(16, os.cpu_count() or 1)
    os.environ["OMP_NUM_THREADS"] = str(threads)
    torch.set_num_threads(threads)
    ip, ix = indptr.numpy(), indices.numpy()
    edges = rows = 0
    t_sample = t_gather = 0.0
    done = 0
    t_begin = time.perf_counter()
    extra = torch.Generator().manual_seed(cfg["graph_seed"] + 3)
    def more():  # the timed GPU batches first, then fresh ones until the budget is used
        yield from batches
        while True:
            yield torch.randint(0, cfg["nodes"], (cfg["batch"],), generator=extra, dtype=torch.int64)
    for b in more():
        t0 = time.perf_counter()
        frontier, _, blocks = oracle.sample_blocks(b.numpy(), ip, ix, cfg["fanouts"], cfg["replace"], 1, 0)
        t1 = time.perf_counter()
        x = torch.index_select(feats, 0, torch.from_numpy(frontier))
        t2 = time.perf_counter()
        edges += sum(blk[0].size for blk in blocks)
        rows += frontier.size
        t_sample += t1 - t0
        t_gather += t2 - t1
        done += 1
        del x
        if time.perf_counter() - t_begin > budget_s and done >= 3:
            break
        if done >= 2000:
            break
    total = t_sample + t_gather
    gather_bytes = rows * (2 * feats.shape[1] * feats.element_size() + 8)
    return {"value": edges / total, "unit": "edges/s", "cores": threads, "kind": "port",
            "sample": f"{done} batches of {cfg['batch']} seeds, fanouts {cfg['fanouts']}, same graph/features "
                      f"({total:.1f} s of CPU work): oracle sampling+relabel, torch.index_select gather",
            "sample_edges_per_s": edges / t_sample, "gather_GBps": gather_bytes / t_gather / 1e9,
            "ms_per_batch": 1e3 * total / done, "ms_sample_relabel": 1e3 * t_sample / done,
            "ms_gather": 1e3 * t_gather / done}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c1", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-budget-s", type=float, default=12.0)
    ap.add_argument("--calibrate-copy-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB (a known-size kernel to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings against)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build measures ONE GPU (world size 1); --gpus N with N > 1 is not supported")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")

    dgs = importlib.import_module("dist-gpu-sampling_amd")
    cfg = WORKLOADS[args.workload]
    torch.cuda.set_device(0)
    t0 = time.perf_counter()
    indptr, indices, feats, _ = make_graph(cfg)
    t_gen = time.perf_counter() - t0

    # everything in HBM: capacity = the whole tensor
    big = 1 << 62
    ct_indptr = dgs.create_chunktensor(indptr, 1, big)
    ct_indices = dgs.create_chunktensor(indices, 1, big)
    ct_feats = dgs.create_chunktensor(feats, 1, big)
    sampler = dgs.ChunkTensorSampler(cfg["fanouts"], ct_indptr, ct_indices, replace=cfg["replace"])

    n_batches = args.steps + args.warmup
    batches_cpu = make_batches(cfg, n_batches)
    batches = [b.cuda() for b in batches_cpu]
    feat_bytes = feats.element_size()
    dgs.set_rng_state(20240602, 0)

    def step(seeds):
        # sampler loop + feature gather, one blocking length read at the very end
        frontier, _, blocks, x = sampler.sample_blocks_and_index(None, seeds, ct_feats)
        return frontier, blocks, x

    for i in range(args.warmup):
        step(batches[i])
    torch.cuda.synchronize()
    if args.calibrate_copy_mib > 0:
        src = torch.empty(args.calibrate_copy_mib << 18, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads and writes calibrate_copy_mib MiB each
        torch.cuda.synchronize()
        del src, dst

    stats = []
    frontiers = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        frontier, blocks, x = step(batches[args.warmup + i])
        stats.append({"frontier": frontier.numel(),
                      "hops": [(b.num_dst, b.src_local.numel(), b.num_src) for b in reversed(blocks)]})
        frontiers.append(frontier)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    # Stage split and the dominant kernel's duration, on the same batches: events on torch's
    # current stream (the one the C ABI launches on) around the sampler call and around the
    # gather launch of each batch's frontier.
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    dgs.set_rng_state(20240602, 0)
    for i in range(args.warmup):
        sampler.sample_blocks(None, batches[i])
    torch.cuda.synchronize()
    for i in range(args.steps):
        events[i][0].record()
        sampler.sample_blocks(None, batches[args.warmup + i])
        events[i][1].record()
    torch.cuda.synchronize()
    gather_ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(args.steps)]
    for i in range(args.steps):  # queued back to back: the GPU never waits for the host
        gather_ev[i][0].record()
        x = ct_feats._CAPI_index(frontiers[i])
        gather_ev[i][1].record()
    torch.cuda.synchronize()

    ms_step = 1e3 * elapsed / args.steps
    ms_sample = float(np.mean([e[0].elapsed_time(e[1]) for e in events]))
    ms_gather = float(np.mean([e[0].elapsed_time(e[1]) for e in gather_ev]))
    edges = sum(sum(h[1] for h in s["hops"]) for s in stats)
    rows = sum(s["frontier"] for s in stats)
    bs = bu = bg = 0
    for s in stats:
        a, b, c = algorithmic_bytes(s, cfg["feat_dim"], feat_bytes)
        bs, bu, bg = bs + a, bu + b, bg + c
    gather_gbps = bg / args.steps / (ms_gather * 1e-3) / 1e9
    step_gbps = (bs + bu + bg) / elapsed / 1e9

    out = {
        "metric": "sampled edges/s (sampling + relabel + feature gather per batch), 1 MI355X",
        "value": edges / elapsed,
        "unit": "edges/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int64",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: {cfg['nodes']} nodes / {cfg['edges']} edges CSC int64, "
                               f"features {cfg['feat_dtype']} x{cfg['feat_dim']}, all in HBM, batch {cfg['batch']} "
                               f"uniform seeds, fanouts {cfg['fanouts']} without replacement, then gather",
                   "fanouts": cfg["fanouts"], "batch": cfg["batch"]},
        "sample_edges_per_s": edges / args.steps / (ms_sample * 1e-3),
        "gather_GBps": gather_gbps,
        "ms_sample_relabel": ms_sample,
        "ms_gather": ms_gather,
        "avg_edges_per_batch": edges / args.steps,
        "avg_frontier_rows": rows / args.steps,
        "step_algorithmic_GBps": step_gbps,
        "step_hbm_frac": step_gbps / HBM_PEAK_GBPS,
        "roofline": {"bound": "hbm", "kernel": "gather_flat_kernel (ChunkTensor._CAPI_index)",
                     "achieved": gather_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": gather_gbps / HBM_PEAK_GBPS,
                     "traffic": (C1_GATHER_TRAFFIC_BYTES_PER_ROW * rows / args.steps) if args.workload == "c1" else None,
                     "algorithmic_bytes": bg / args.steps, "avg_launch_us": 1e3 * ms_gather},
        "graph_gen_s": t_gen,
    }
    if not args.no_cpu_baseline:
        cb = cpu_baseline(cfg, indptr, indices, feats, batches_cpu[args.warmup:], args.cpu_budget_s)
        out["cpu_baseline"] = cb
        out["gpu_over_cpu"] = out["value"] / cb["value"]
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
