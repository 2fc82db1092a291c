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
PCIE_PEAK_GBPS = 64.0   # PCIe Gen5 x16, one direction
GATHER_SOURCE = os.path.join(ROOT, "dist-gpu-sampling_amd", "csrc", "gather.hip")
GATHER_TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "gather_flat_kernel_c1_pmc.txt")


def measured_gather_traffic():
    """HBM bytes per gathered 400-byte row of workload c1, as the committed counter summary holds
    them (rocprofv3 FETCH_SIZE and WRITE_SIZE, scaled by a plain copy of known size), together
    with where they come from.  The summary names the version of the gather source it was taken
    on; for any other version the reading says nothing and (None, why) is returned."""
    import hashlib
    import re
    try:
        text = open(GATHER_TRAFFIC_SUMMARY).read()
        source_hash = hashlib.sha256(open(GATHER_SOURCE, "rb").read()).hexdigest()[:16]
    except OSError as err:
        return None, f"no counter summary to read ({err.filename})"
    per_row = re.search(r"^traffic_bytes_per_row\s*=\s*([0-9.]+)", text, re.M)
    taken_on = re.search(r"^gather_source_sha256_16\s*=\s*([0-9a-f]{16})", text, re.M)
    name = os.path.relpath(GATHER_TRAFFIC_SUMMARY, ROOT)
    if not per_row or not taken_on:
        return None, f"{name} holds no traffic_bytes_per_row / gather_source_sha256_16 lines"
    if taken_on.group(1) != source_hash:
        return None, (f"{name} was taken on gather.hip {taken_on.group(1)}, this run has {source_hash}: "
                      "counters not re-taken for this kernel")
    return float(per_row.group(1)), (f"{name} (gather.hip {source_hash}): counter bytes per gathered row "
                                     "x this run's rows; not a counter reading of this run")


WORKLOADS = {
    # benchmark configuration 1: the one the headline metric is quoted on
    "c1": dict(nodes=2_449_029, edges=123_718_280, max_deg=17_000, deg1_frac=0.05, feat_dim=100,
               feat_dtype="float32", batch=1024, fanouts=[15, 10, 5], replace=False, graph_seed=20240602),
    # c1 with a float32 weight per edge: every hop uses the weighted operator
    # (upstream ChunkTensorSampler with chunk_probs), per-hop path, then the same gather
    "c1w": dict(nodes=2_449_029, edges=123_718_280, max_deg=17_000, deg1_frac=0.05, feat_dim=100,
                feat_dtype="float32", batch=1024, fanouts=[15, 10, 5], replace=False, graph_seed=20240602,
                weighted=True),
    # benchmark configuration 0 (CPU-runnable plumbing case), used by --workload c0
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


def make_weights(cfg, n_edges):
    """Edge weights of the weighted workload: uniform in (0.01, 1.01)."""
    g = torch.Generator().manual_seed(cfg["graph_seed"] + 4)
    return torch.rand(n_edges, generator=g, dtype=torch.float32) + 0.01


def cpu_baseline(cfg, indptr, indices, feats, batches, budget_s=12.0, probs=None):
    """The CPU oracle (a port of the reference algorithm, OpenMP over seed rows) plus
    torch.index_select, timed on this machine's host cores on a bounded sample of the
    same batches."""
    from oracle import oracle
    oracle.build()
    threads = min(16, os.cpu_count() or 1)
    os.environ["OMP_NUM_THREADS"] = str(threads)
    torch.set_num_threads(threads)
    ip, ix = indptr.numpy(), indices.numpy()
    pr = None if probs is None else probs.numpy()
    edges = rows = 0
    t_sample = t_gather = 0.0
    done = 0
    t_begin = time.perf_counter()
    extra = torch.Generator().manual_seed(cfg["graph_seed"] + 3)
    def more():  # the timed GPU batches first, then fresh ones until the budget is used
        yield from batches
        while True:
            yield torch.randint(0, cfg["nodes"], (cfg["batch"],), generator=extra, dtype=torch.int64)
    # the checker's unique/relabel is sequential (upstream's algorithm in a fixed order); the timed
    # leg uses the all-threads variant, held against the sequential one on the first batch, once
    # for the result and once for what it costs
    first = batches[0].numpy()
    t0 = time.perf_counter()
    want = oracle.sample_blocks(first, ip, ix, cfg["fanouts"], cfg["replace"], 1, 0, probs=pr)
    t_sequential = time.perf_counter() - t0
    got = oracle.sample_blocks(first, ip, ix, cfg["fanouts"], cfg["replace"], 1, 0, probs=pr, parallel_relabel=True)
    same = np.array_equal(want[0], got[0]) and all(
        all(np.array_equal(x, y) for x, y in zip(a, b)) for a, b in zip(want[2], got[2]))
    if not same:
        raise RuntimeError("cpu baseline: the all-threads relabel differs from the sequential one")
    del want, got
    for b in more():
        t0 = time.perf_counter()
        frontier, _, blocks = oracle.sample_blocks(b.numpy(), ip, ix, cfg["fanouts"], cfg["replace"], 1, 0, probs=pr,
                                                   parallel_relabel=True)
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
            "host_cpus": os.cpu_count(), "omp_threads": threads, "torch_threads": torch.get_num_threads(),
            "threads_per_leg": {"sampling": f"{threads} (OpenMP over the seed rows)",
                                "unique/relabel": f"{threads} (tables sharded by id, one per thread; the sequential "
                                                  "restatement of upstream's table is the checker, and this one "
                                                  "was held against it on the first batch)",
                                "gather": f"{torch.get_num_threads()} (torch.index_select)"},
            "sample": f"{done} batches of {cfg['batch']} seeds, fanouts {cfg['fanouts']}, same graph/features "
                      f"({total:.1f} s of CPU work): oracle sampling+relabel, torch.index_select gather",
            "sample_edges_per_s": edges / t_sample, "gather_GBps": gather_bytes / t_gather / 1e9,
            "ms_per_batch": 1e3 * total / done, "ms_sample_relabel": 1e3 * t_sample / done,
            "ms_gather": 1e3 * t_gather / done,
            "ms_sample_relabel_with_sequential_relabel": 1e3 * t_sequential}


def device_powerlaw_csc(n, e, max_deg, one_frac, id_dtype, gen, sort_by_degree, sources="uniform"):
    """Power-law CSC built on the device (the large workloads never exist on the host).
    sources="uniform": every edge's source is a uniform node (the benchmark configurations);
    "by_degree": a node is a source in proportion to its in-degree, as in the symmetric graphs
    that citation and co-purchase data are (the source of an edge is the row that holds a
    uniformly drawn edge slot)."""
    u = torch.rand(n, generator=gen, device="cuda", dtype=torch.float64)
    raw = (1.0 - u).pow(-1.0 / 1.25)
    ones = torch.rand(n, generator=gen, device="cuda") < one_frac
    lo, hi = 0.01, 1000.0
    for _ in range(50):
        mid = 0.5 * (lo + hi)
        deg = (raw * mid).floor().clamp_(2, max_deg)
        deg[ones] = 1
        if deg.sum().item() > e:
            hi = mid
        else:
            lo = mid
    deg = (raw * lo).floor().clamp_(2, max_deg)
    deg[ones] = 1
    deg = deg.long()
    rest = int(e - deg.sum().item())
    deg[torch.nonzero((deg > 1) & (deg < max_deg - 1)).flatten()[:rest]] += 1
    if sort_by_degree:  # node ids in decreasing in-degree: the hottest rows land in the HBM slice
        deg = torch.sort(deg, descending=True).values
    indptr = torch.zeros(n + 1, dtype=torch.int64, device="cuda")
    torch.cumsum(deg, 0, out=indptr[1:])
    e = int(indptr[-1].item())
    indices = torch.empty(e, dtype=id_dtype, device="cuda")
    step = 1 << 28 if sources == "uniform" else 1 << 26
    for a in range(0, e, step):
        b = min(e, a + step)
        if sources == "uniform":
            indices[a:b] = torch.randint(0, n, (b - a,), generator=gen, device="cuda", dtype=id_dtype)
        else:
            slot = torch.randint(0, e, (b - a,), generator=gen, device="cuda")
            indices[a:b] = (torch.searchsorted(indptr, slot, right=True) - 1).to(id_dtype)
    return indptr, indices


def store_from_device(dgs, t, capacity_bytes):
    """ChunkTensor filled through its slice views from a device tensor."""
    ct = dgs.ChunkTensor(list(t.shape), t.dtype, capacity_bytes)
    flat = t.reshape(-1)
    dev = ct._CAPI_get_sub_device_tensor()
    dev.copy_(flat[: dev.numel()])
    host = ct._CAPI_get_host_tensor()
    for a in range(0, host.numel(), 1 << 28):
        b = min(host.numel(), a + (1 << 28))
        host[a:b].copy_(flat[dev.numel() + a: dev.numel() + b])
    torch.cuda.synchronize()
    return ct


def run_batches(sampler, seed_batches, features, inflight, consume=lambda r: None, hand_over=False):
    """The timed loop: the package's BatchPipeline submits every batch on one of `inflight` streams
    in turn and hands each one out once `inflight` batches are queued, so that many batches share
    the GPU at any time.  `consume` turns each result into what the caller keeps (the big buffers
    are dropped at once so the allocator can hand them to the next batch).  The caller brackets
    the call with synchronisations.  Nothing here touches a batch on another stream than its own,
    so by default the pipeline does not hand batches over to the calling stream."""
    if features is None:  # sampling + relabel only
        return [consume(sampler.sample_blocks(None, b)) for b in seed_batches]
    if inflight <= 1 or not sampler.fused:
        return [consume(sampler.sample_blocks_and_index(None, b, features)) for b in seed_batches]
    # (a pipeline is made once and iterated many times, as a training loop would per epoch)
    key = (id(sampler), id(features), inflight, hand_over)
    if key not in _pipelines:
        _pipelines[key] = (sys.modules[type(sampler).__module__].BatchPipeline(sampler, features, inflight,
                                                                              hand_over=hand_over), sampler, features)
    return [consume(r) for r in _pipelines[key][0](seed_batches)]


_pipelines = {}


def table_access_rates(dgs, slots, n_ops, reps=50):
    """Random 8-byte accesses per second this GPU serves on a table of `slots` slots, by kind:
    the library's probe kernel (one access per thread, nothing else), timed with events on the
    stream it is launched on.  The fused sampler does one atomicMin with return per pick on a
    table of one slot per node, so these are the rates that bound it."""
    capi = dgs.capi
    table = torch.full((slots,), -1, dtype=torch.int64, device="cuda")
    sink = torch.zeros(1, dtype=torch.int64, device="cuda")
    out = {"slots": slots, "table_bytes": 8 * slots, "accesses_per_launch": n_ops, "unit": "G accesses/s"}
    for name, op in (("load", capi.PROBE_LOAD), ("store", capi.PROBE_STORE),
                     ("atomic_min_with_return", capi.PROBE_ATOMIC_MIN),
                     ("atomic_min_no_return", capi.PROBE_ATOMIC_MIN_NO_RETURN)):
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        capi.probe_table(op, table, n_ops, 0, sink)
        torch.cuda.synchronize()
        begin.record()
        for rep in range(reps):  # back to back, so that the gaps around a single short launch do not count
            capi.probe_table(op, table, n_ops, 1 + rep, sink)
        end.record()
        torch.cuda.synchronize()
        t = begin.elapsed_time(end) * 1e-3 / reps
        out[name] = n_ops / t / 1e9
        out[name + "_us"] = 1e6 * t
    return out


def time_call(fn, reps):
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(reps)]
    fn()
    torch.cuda.synchronize()
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return float(np.mean([a.elapsed_time(b) for a, b in ev])) * 1e-3


def device_rmat_csc(scale_bits, e, gen):
    """R-MAT (a, b, c, d) = (.57, .19, .19, .05) grouped by destination without sorting: the
    destination bits are independent with P(bit = 1) = b + d, so in-degrees follow from the
    per-node probability, and every source bit is drawn given the destination's bit."""
    a, b, c, d = 0.57, 0.19, 0.19, 0.05
    n = 1 << scale_bits
    ids = torch.arange(n, device="cuda")
    ones = torch.zeros(n, device="cuda", dtype=torch.float64)
    for bit in range(scale_bits):
        ones += ((ids >> bit) & 1).double()
    lam = torch.exp(ones * np.log(b + d) + (scale_bits - ones) * np.log(a + c) + np.log(e))
    deg = torch.poisson(lam.float(), generator=gen).long()
    diff = int(e - deg.sum().item())
    top = torch.argsort(lam, descending=True)[: abs(diff)]
    deg[top] += 1 if diff > 0 else -1
    deg.clamp_(min=0)
    deg[0] += e - int(deg.sum().item())
    indptr = torch.zeros(n + 1, dtype=torch.int64, device="cuda")
    torch.cumsum(deg, 0, out=indptr[1:])
    indices = torch.empty(e, dtype=torch.int32, device="cuda")
    for lo in range(0, e, 1 << 26):
        hi = min(e, lo + (1 << 26))
        dst = torch.searchsorted(indptr, torch.arange(lo, hi, device="cuda"), right=True) - 1
        src = torch.zeros(hi - lo, dtype=torch.int32, device="cuda")
        for bit in range(scale_bits):
            p1 = torch.where(((dst >> bit) & 1) == 1, d / (b + d), c / (a + c)).float()
            src |= (torch.rand(hi - lo, generator=gen, device="cuda") < p1).int() << bit
        indices[lo:hi] = src
    return indptr, indices


LARGE = {
    # benchmark configuration 2: large graph, all in HBM, bf16 x128, 4096 seeds from a 1% train subset
    "c2": dict(graph="powerlaw", nodes=111_059_956, edges=1_615_685_872, dim=128, feat_dtype=torch.bfloat16,
               hbm_rows=1.0, batch=4096, fanouts=[15, 10, 5], replace=False, train_frac=0.01, seed=20240603),
    # configuration 3: same graph, f32 x256, top 40% of rows by in-degree in HBM, rest in pinned host memory
    "c3": dict(graph="powerlaw", nodes=111_059_956, edges=1_615_685_872, dim=256, feat_dtype=torch.float32,
               hbm_rows=0.4, batch=8192, fanouts=[20, 15, 10], replace=False, train_frac=1.0, seed=20240604),
    # configuration 4: R-MAT scale 26, 2^30 edges, with replacement, fanouts [50, 50], 16384 seeds, f32 x64
    "c4": dict(graph="rmat", nodes=1 << 26, edges=1 << 30, dim=64, feat_dtype=torch.float32,
               hbm_rows=1.0, batch=16384, fanouts=[50, 50], replace=True, train_frac=1.0, seed=20240605),
}
# batches in flight by default: the best of 2..5 measured on each (c2: 0.176-0.187 ms per step with four against
# 0.189-0.194 with three; c4: three and four are level and three hold less memory; a two-tier c3 batch runs alone)
LARGE_INFLIGHT = {"c2": 4, "c3": 3, "c4": 3}


def measure_large(name, dgs, steps, warmup, inflight, scale=1.0, stage_batches=8):
    """Benchmark configurations 2 to 4, built on the device; returns the result record.  For the
    two-tier case (c3) the tiers are also timed separately: device tier against HBM, host tier
    against PCIe Gen5 x16."""
    cfg = LARGE[name]
    n, e = int(cfg["nodes"] * scale), int(cfg["edges"] * scale)
    dim, fanouts, batch = cfg["dim"], cfg["fanouts"], cfg["batch"]
    gen = torch.Generator(device="cuda").manual_seed(cfg["seed"])
    t0 = time.perf_counter()
    if cfg["graph"] == "rmat":
        bits = int(round(np.log2(n)))
        n = 1 << bits
        indptr, indices = device_rmat_csc(bits, e, gen)
    else:
        indptr, indices = device_powerlaw_csc(n, e, 30_000, 0.05, torch.int32, gen,
                                              sort_by_degree=cfg["hbm_rows"] < 1.0)
    ct_ip = store_from_device(dgs, indptr, 1 << 62)
    ct_ix = store_from_device(dgs, indices, 1 << 62)
    del indptr, indices
    hot_rows = int(n * cfg["hbm_rows"])
    eb = torch.empty(0, dtype=cfg["feat_dtype"]).element_size()
    ct_x = dgs.ChunkTensor([n, dim], cfg["feat_dtype"], hot_rows * dim * eb)
    dev, host = ct_x._CAPI_get_sub_device_tensor(), ct_x._CAPI_get_host_tensor()
    chunk = 1 << 26
    for a in range(0, dev.numel(), chunk):
        dev[a: a + chunk].normal_(generator=gen)
    stage = torch.empty(chunk, device="cuda", dtype=cfg["feat_dtype"])
    for a in range(0, host.numel(), chunk):
        m = min(chunk, host.numel() - a)
        stage[:m].normal_(generator=gen)
        host[a: a + m].copy_(stage[:m])
    del stage, dev, host
    torch.cuda.synchronize()
    t_gen = time.perf_counter() - t0
    sampler = dgs.ChunkTensorSampler(fanouts, ct_ip, ct_ix, replace=cfg["replace"])
    pool = None
    if cfg["train_frac"] < 1.0:  # seeds come from a fixed uniform subset of the nodes
        pool = torch.randperm(n, generator=gen, device="cuda")[: int(n * cfg["train_frac"])].to(torch.int32)
    seeds = []
    for _ in range(steps + warmup):
        r = torch.randint(0, n if pool is None else pool.numel(), (batch,), generator=gen, device="cuda")
        seeds.append(r.to(torch.int32) if pool is None else pool[r])
    dgs.set_rng_state(cfg["seed"], 0)
    # the two-tier case gathers tens of GB per batch: one batch at a time
    two_tier = cfg["hbm_rows"] < 1.0
    inflight = inflight if not two_tier else 1
    run_batches(sampler, seeds[:warmup], ct_x, inflight)
    if inflight > 1:  # the allocator's per-stream pools see every buffer size before anything is timed
        run_batches(sampler, (seeds * 4)[:4 * inflight + warmup], ct_x, inflight)
    torch.cuda.synchronize()
    def keep(r):  # of a timed batch only the lengths are kept: every buffer goes back to its stream's pool at once
        return {"frontier": r[0].numel(),
                "hops": [(b.num_dst, b.src_local.numel(), b.num_src) for b in reversed(r[2])]}
    resident = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    t0 = time.perf_counter()
    results = run_batches(sampler, seeds[warmup:], ct_x, inflight, keep)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    peak_batch_bytes = torch.cuda.max_memory_allocated() - resident
    rows = sum(r["frontier"] for r in results)
    edges = sum(sum(h[1] for h in r["hops"]) for r in results)
    row_bytes = dim * eb

    def total_bytes(all_stats):
        bs = bu = bg = 0
        for st in all_stats:
            a, b, c = algorithmic_bytes(st, dim, eb, w_id=4, w_ptr=8)
            bs, bu, bg = bs + a, bu + b, bg + c
        return bs, bu, bg
    bs, bu, bg = total_bytes(results)
    # one batch at a time on one stream, call to result (what upstream's own loop, num_workers=0, sees)
    ms_alone = None
    if inflight > 1:
        n_alone = min(steps, 10)
        run_batches(sampler, seeds[:2], ct_x, 1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_batches(sampler, seeds[warmup:warmup + n_alone], ct_x, 1, keep)
        torch.cuda.synchronize()
        ms_alone = 1e3 * (time.perf_counter() - t0) / n_alone
    # stage split: the sampler alone (events on the launching stream around the fused call), then
    # the gather alone, once per kept frontier (a repeat of the same rows would be served by the
    # 256 MB last-level cache), queued back to back
    n_stage = min(steps, stage_batches)
    sample_ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(n_stage)]
    stage_stats = []
    frontiers = []
    sampler.sample_blocks(None, seeds[0])
    torch.cuda.synchronize()
    for i in range(n_stage):
        sample_ev[i][0].record()
        r = sampler.sample_blocks(None, seeds[warmup + i])
        sample_ev[i][1].record()
        stage_stats.append({"frontier": r[0].numel(),
                            "hops": [(b.num_dst, b.src_local.numel(), b.num_src) for b in reversed(r[2])]})
        frontiers.append(r[0].clone())  # for the gather leg below (a copy: the batch's own block goes back to the pool)
        del r
    torch.cuda.synchronize()
    ms_sample = float(np.mean([a.elapsed_time(b) for a, b in sample_ev]))
    sbs, sbu, _ = total_bytes(stage_stats)
    sampler_gbps = (sbs + sbu) / n_stage / (ms_sample * 1e-3) / 1e9
    frontier = frontiers[-1]
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in frontiers]
    ct_x._CAPI_index(frontiers[-1][:1024])
    torch.cuda.synchronize()
    for f, (a, b) in zip(frontiers, ev):
        a.record()
        x = ct_x._CAPI_index(f)
        b.record()
        del x
    torch.cuda.synchronize()
    t_mixed = sum(a.elapsed_time(b) for a, b in ev) * 1e-3
    gather_bytes = sum(f.numel() for f in frontiers) * (2 * row_bytes + 4)
    gather_gbps = gather_bytes / t_mixed / 1e9
    t_mixed /= len(frontiers)
    step_gbps = (bs + bu + bg) / elapsed / 1e9
    out = {
        "metric": "sampled edges/s (sampling + relabel + feature gather per batch), 1 MI355X",
        "value": edges / elapsed, "unit": "edges/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": 1e3 * elapsed / steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int32", "data": "synthetic",
        "config": {"workload": f"{name}: {cfg['graph']} graph, {n} nodes / {e} edges CSC int64+int32, "
                               f"features {str(cfg['feat_dtype']).split('.')[-1]} x{dim} ({n * row_bytes / 1e9:.1f} GB), "
                               f"{int(100 * cfg['hbm_rows'])}% of rows in HBM, batch {batch}, fanouts {fanouts}, "
                               f"{'with' if cfg['replace'] else 'without'} replacement", "scale": scale,
                   "batches_in_flight": inflight},
        "ms_per_batch_alone": ms_alone,
        "edges_per_s": edges / elapsed,
        "avg_frontier_rows": rows / steps, "avg_edges_per_batch": edges / steps,
        # per hop, in hop order: seeds, sampled edges, frontier size afterwards (averages over the timed batches)
        "avg_hops": [[float(np.mean([r["hops"][h][j] for r in results])) for j in range(3)]
                     for h in range(len(fanouts))],
        "ms_sample_relabel": ms_sample,
        "gather_ms": 1e3 * t_mixed, "gather_GBps": gather_gbps, "graph_gen_s": t_gen,
        "step_algorithmic_GBps": step_gbps, "step_hbm_frac": step_gbps / HBM_PEAK_GBPS,
        "stages": [
            {"stage": "sampling + relabel of every hop (fused sampler kernels, one batch alone on one stream)",
             "bound": "hbm", "achieved": sampler_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
             "frac": sampler_gbps / HBM_PEAK_GBPS, "algorithmic_bytes": (sbs + sbu) / n_stage, "avg_us": 1e3 * ms_sample},
            {"stage": "feature gather of the last frontier (gather_flat_kernel), both tiers as the store holds them",
             "bound": "hbm", "achieved": gather_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
             "frac": gather_gbps / HBM_PEAK_GBPS, "algorithmic_bytes": gather_bytes / len(frontiers),
             "avg_us": 1e6 * t_mixed},
            {"stage": "whole step as timed", "bound": "hbm", "achieved": step_gbps, "peak": HBM_PEAK_GBPS,
             "unit": "GB/s", "frac": step_gbps / HBM_PEAK_GBPS, "algorithmic_bytes": (bs + bu + bg) / steps,
             "avg_us": 1e6 * elapsed / steps},
        ],
        # torch allocations of the batches in flight at their peak (outputs, workspaces),
        # beyond what was resident before the timed loop; the stores themselves are not torch memory
        "peak_batch_bytes": peak_batch_bytes,
        "gather_buffer_cap_bytes": int(torch.ops.dgs_ops._CAPI_get_gather_buffer_cap()),
    }
    if two_tier:
        local, _, host_ids = ct_x._CAPI_split_index(frontier)
        t_local = time_call(lambda: ct_x._CAPI_local_index(local), 5)
        t_host = time_call(lambda: ct_x._CAPI_host_index(host_ids), 3)
        dev_gbps = local.numel() * (2 * row_bytes + 4) / t_local / 1e9
        host_gbps = host_ids.numel() * row_bytes / t_host / 1e9
        out.update({
            "frontier_rows_device_tier": local.numel(), "frontier_rows_host_tier": host_ids.numel(),
            "device_tier_gather_GBps": dev_gbps, "device_tier_ms": 1e3 * t_local,
            "device_tier_hbm_frac": dev_gbps / HBM_PEAK_GBPS,
            "host_tier_gather_GBps": host_gbps, "host_tier_ms": 1e3 * t_host,
            "host_tier_peak_GBps": PCIE_PEAK_GBPS, "host_tier_pcie_frac": host_gbps / PCIE_PEAK_GBPS,
            "roofline": {"bound": "hbm", "kernel": "gather_flat_kernel (_CAPI_local_index, device tier)",
                         "achieved": dev_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": dev_gbps / HBM_PEAK_GBPS, "traffic": None},
        })
    else:
        out["roofline"] = {"bound": "hbm", "kernel": "gather_flat_kernel (_CAPI_index)", "achieved": gather_gbps,
                           "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gather_gbps / HBM_PEAK_GBPS,
                           "traffic": None}
    return out


def measure_placement(dgs, scale=1.0, steps=4, hbm_rows=0.4, seed=20240606):
    """What "hottest rows first" is worth on a two-tier store: the c3 shapes (111 M nodes, 1.6 G
    edges, f32 x256 rows, 40 % of the rows in HBM, 8192 seeds, fanouts [20,15,10]) on a graph whose
    sources follow the in-degrees, once with the nodes in the arbitrary order they were generated
    in and once renumbered by decreasing in-degree (placement.degree_order + renumber_csc; the
    feature rows are random either way, so the placed store is filled afresh instead of
    permuted).  Per variant: the share of sampled edges whose source row lies in the HBM slice
    beside placement.expected_hit_rate, the frontier's rows per tier, host-tier bytes, step time."""
    cfg = LARGE["c3"]
    n, e = int(cfg["nodes"] * scale), int(cfg["edges"] * scale)
    dim, fanouts, batch = cfg["dim"], cfg["fanouts"], cfg["batch"]
    pl = dgs.placement
    gen = torch.Generator(device="cuda").manual_seed(seed)
    indptr, indices = device_powerlaw_csc(n, e, 30_000, 0.05, torch.int32, gen, sort_by_degree=False,
                                          sources="by_degree")
    hot_rows = int(n * hbm_rows)
    row_bytes = dim * 4
    seeds = [torch.randint(0, n, (batch,), generator=gen, device="cuda").to(torch.int32) for _ in range(steps + 1)]
    out = {"config": {"workload": f"c3 shapes, sources drawn in proportion to in-degree: {n} nodes / {e} edges, "
                                  f"f32 x{dim} rows, {int(100 * hbm_rows)}% of rows in HBM, batch {batch}, fanouts {fanouts}",
                      "scale": scale, "steps": steps}}

    def variant(ip, ix, seed_batches):
        deg = ip[1:] - ip[:-1]
        expected = pl.expected_hit_rate(deg, hot_rows)
        ct_ip = store_from_device(dgs, ip, 1 << 62)
        ct_ix = store_from_device(dgs, ix, 1 << 62)
        ct_x = dgs.ChunkTensor([n, dim], torch.float32, hot_rows * row_bytes)
        dev, host = ct_x._CAPI_get_sub_device_tensor(), ct_x._CAPI_get_host_tensor()
        chunk = 1 << 26
        for a in range(0, dev.numel(), chunk):
            dev[a: a + chunk].normal_(generator=gen)
        stage = torch.empty(chunk, device="cuda", dtype=torch.float32)
        for a in range(0, host.numel(), chunk):
            m = min(chunk, host.numel() - a)
            stage[:m].normal_(generator=gen)
            host[a: a + m].copy_(stage[:m])
        del stage, dev, host
        sampler = dgs.ChunkTensorSampler(fanouts, ct_ip, ct_ix, replace=False)
        dgs.set_rng_state(seed, 0)
        sampler.sample_blocks_and_index(None, seed_batches[0], ct_x)
        torch.cuda.synchronize()
        picks = hot_picks = rows = rows_hbm = 0
        t0 = time.perf_counter()
        results = [sampler.sample_blocks_and_index(None, sb, ct_x) for sb in seed_batches[1:]]
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        for frontier, _, blocks, x in results:
            for b in blocks:
                src = b.src_ids[b.src_local.long()]
                picks += src.numel()
                hot_picks += int((src < hot_rows).sum().item())
            rows += frontier.numel()
            rows_hbm += int((frontier < hot_rows).sum().item())
        k = len(results)
        return {"expected_hit_rate": expected, "measured_hit_rate_of_sampled_edges": hot_picks / max(picks, 1),
                "frontier_rows": rows / k, "frontier_rows_in_hbm": rows_hbm / k,
                "frontier_rows_in_host_memory": (rows - rows_hbm) / k,
                "frontier_share_in_hbm": rows_hbm / max(rows, 1),
                "host_tier_bytes_per_batch": (rows - rows_hbm) / k * row_bytes,
                "ms_per_step": 1e3 * elapsed / k,
                "host_tier_GBps_if_it_bounds_the_step": (rows - rows_hbm) * row_bytes / elapsed / 1e9}

    out["unplaced"] = variant(indptr, indices, seeds)
    release_everything()
    order = pl.degree_order(indptr)
    new_ip, new_ix, rank = pl.renumber_csc(indptr, indices, order)
    del indptr, indices, order
    out["placed_by_in_degree"] = variant(new_ip, new_ix, [rank[sb.long()] for sb in seeds])
    out["step_time_ratio_unplaced_over_placed"] = out["unplaced"]["ms_per_step"] / out["placed_by_in_degree"]["ms_per_step"]
    return out


def release_everything():
    """Between workloads: pipelines (and their samplers' worker threads), cached blocks."""
    import gc
    _pipelines.clear()
    gc.collect()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c1", choices=sorted(WORKLOADS) + sorted(LARGE) + ["c3_placement"])
    ap.add_argument("--scale", type=float, default=1.0, help="size factor of the c2/c3/c4 workloads (1.0 = full)")
    ap.add_argument("--inflight", type=int, default=None,
                    help="batches in flight on as many streams (1 = one blocking call per batch); default 4 for "
                         "c0/c1/c1w/c2 and 3 for c3/c4 (measured best of 2..5 on each; c3 always runs one)")
    ap.add_argument("--gather-buffer-cap-gib", type=float, default=None,
                    help="largest feature buffer the fused operator allocates ahead of a batch's sizes "
                         "(the library's default when not given)")
    ap.add_argument("--node-table-max-nodes", type=int, default=None,
                    help="graphs above this many nodes sample on a per-call hash table instead of persistent "
                         "node tables (the library's default when not given)")
    ap.add_argument("--last-hop", type=int, default=0,
                    help="how the fused sampler's last hop finds first occurrences (the library's test hook "
                         "DGS_DEBUG_SAMPLER_BUCKETED): 0 by size, 1 always on the node table, 2 always the bucketed pass, "
                         "3 / 4 its hashed form for graphs of any node count (16384- / 256-slot LDS tables)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="with --workload c1: do not also run c1w, c2, c4 and c3 after the headline")
    ap.add_argument("--other-steps", type=int, default=40, help="timed batches of each other workload")
    ap.add_argument("--other-budget-s", type=float, default=300.0,
                    help="no further workload is started once this much time has gone into them")
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
    torch.cuda.set_device(0)
    if args.inflight is None:
        args.inflight = LARGE_INFLIGHT.get(args.workload, 4)
    if args.gather_buffer_cap_gib is not None:
        dgs.set_gather_buffer_cap(int(args.gather_buffer_cap_gib * (1 << 30)))
    if args.last_hop:
        dgs.capi.check(dgs.capi.lib.dgs_debug_set(dgs.capi.DEBUG_SAMPLER_BUCKETED, args.last_hop))
    if args.node_table_max_nodes is not None:
        torch.ops.dgs_ops._CAPI_set_node_table_max_nodes(args.node_table_max_nodes)
    if args.workload == "c3_placement":
        print(json.dumps(measure_placement(dgs, args.scale, min(args.steps, 8))), flush=True)
        return
    if args.workload in LARGE:
        print(json.dumps(measure_large(args.workload, dgs, args.steps, args.warmup, args.inflight, args.scale)),
              flush=True)
        return
    cfg = WORKLOADS[args.workload]
    t0 = time.perf_counter()
    indptr, indices, feats, _ = make_graph(cfg)
    t_gen = time.perf_counter() - t0

    # everything in HBM: capacity = the whole tensor
    big = 1 << 62
    ct_indptr = dgs.create_chunktensor(indptr, 1, big)
    ct_indices = dgs.create_chunktensor(indices, 1, big)
    ct_feats = dgs.create_chunktensor(feats, 1, big)
    probs = ct_probs = None
    if cfg.get("weighted"):
        probs = make_weights(cfg, indices.numel())
        ct_probs = dgs.create_chunktensor(probs, 1, big)
    sampler = dgs.ChunkTensorSampler(cfg["fanouts"], ct_indptr, ct_indices, ct_probs, replace=cfg["replace"])

    n_batches = args.steps + args.warmup
    batches_cpu = make_batches(cfg, n_batches)
    batches = [b.cuda() for b in batches_cpu]
    feat_bytes = feats.element_size()
    dgs.set_rng_state(20240602, 0)

    inflight = args.inflight if sampler.fused else 1
    if args.calibrate_copy_mib > 0:
        src = torch.empty(args.calibrate_copy_mib << 18, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads and writes calibrate_copy_mib MiB each
        torch.cuda.synchronize()
        del src, dst

    def sizes(r):  # what the timed loops keep of a batch: its lengths; every buffer is dropped at once
        return {"frontier": r[0].numel(),
                "hops": [(b.num_dst, b.src_local.numel(), b.num_src) for b in reversed(r[2])]}

    def timed_steps(smp, seed_batches, n_inflight, hand_over=False, features=ct_feats):
        """W untimed warm-up batches, then exactly K batches between two synchronisations."""
        run_batches(smp, seed_batches[:args.warmup], features, n_inflight, sizes, hand_over)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        res = run_batches(smp, seed_batches[args.warmup:], features, n_inflight, sizes, hand_over)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, res

    # Set-up, not a step: enough batches that torch's caching allocator, which keeps a pool per
    # stream, has seen every buffer size on every stream, and that the GPU has left its idle
    # clocks, before anything is timed (the W warm-up batches alone are fewer than two per stream
    # and over in a millisecond).
    setup_batches = 256
    run_batches(sampler, (batches * (1 + setup_batches // len(batches)))[:setup_batches], ct_feats, inflight, sizes)
    torch.cuda.synchronize()
    # the headline: `inflight` batches on the GPU at any time, seeds already in HBM, each batch
    # left on the stream it ran on
    elapsed, stats = timed_steps(sampler, batches, inflight)
    repeats = [1e3 * timed_steps(sampler, batches, inflight)[0] / args.steps for _ in range(3)]
    # one batch at a time on one stream: what a single batch takes from call to result
    ms_latency = 1e3 * timed_steps(sampler, batches, 1)[0] / args.steps
    # batches in flight again, each handed over to the calling stream (made to wait for the batch,
    # buffers recorded there): what a consumer on another stream than the batch's own sees
    # (the calling stream is one more stream: with it, at most four share the GPU's hardware queues)
    handed_inflight = min(inflight, 3)
    ms_handed_over = (1e3 * timed_steps(sampler, batches, handed_inflight, True)[0] / args.steps
                      if inflight > 1 else None)
    # seeds as upstream's DataLoader passes them: pageable host tensors, uploaded by the operator
    ms_host_seeds = 1e3 * timed_steps(sampler, batches_cpu, inflight)[0] / args.steps
    # both: host seeds in, every batch handed to the calling stream -- what upstream's training loop
    # would see (its DataLoader passes host seeds, its model runs on the current stream)
    ms_handed_over_host_seeds = (1e3 * timed_steps(sampler, batches_cpu, handed_inflight, True)[0] / args.steps
                                 if inflight > 1 else None)
    # the training loop's own shape: SeedLoader in the place of upstream's DataLoader (host ids in, as
    # train_idx; batches cut by the loader, each handed to the calling stream with its feature rows)
    loader_ids = torch.cat(batches_cpu[args.warmup:])
    loader = dgs.SeedLoader(None, loader_ids, sampler, batch_size=cfg["batch"], chunk_features=ct_feats,
                            inflight=handed_inflight)
    ms_seed_loader = None
    if len(loader) == args.steps:
        for out in loader:  # untimed: the loader's first iteration
            sizes(out)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for out in loader:
            sizes(out)
        torch.cuda.synchronize()
        ms_seed_loader = 1e3 * (time.perf_counter() - t0) / len(loader)
    # what an unmodified upstream harness runs: per hop one sampling operator and one relabel
    # operator (each returns tensors of exact length, so each waits for its lengths), then _CAPI_index
    # -- called through torch.ops.dgs_ops with torch as it is, which is what such a harness does
    per_hop = dgs.ChunkTensorSampler(cfg["fanouts"], ct_indptr, ct_indices, ct_probs, replace=cfg["replace"],
                                     fused=False)
    per_hop.ops = torch.ops.dgs_ops
    ms_per_hop_ops = 1e3 * timed_steps(per_hop, batches, 1)[0] / args.steps
    # the same loop without its last line: the sampling and relabel operators alone
    ms_per_hop_ops_no_gather = 1e3 * timed_steps(per_hop, batches, 1, features=None)[0] / args.steps
    # the same loop again with the package's two opt-in shortcuts through torch's Python front end
    # (lighten_torch_dispatch, and the operators' C++ entries instead of their packets)
    per_hop.ops = dgs.fast_ops
    dgs.lighten_torch_dispatch(True)
    ms_per_hop_ops_light = 1e3 * timed_steps(per_hop, batches, 1)[0] / args.steps
    dgs.lighten_torch_dispatch(False)

    # Stage split and the dominant kernel's duration, on the same batches: events on torch's
    # current stream (the one the C ABI launches on) around the sampler call and around the
    # gather launch of each batch's frontier.
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    dgs.set_rng_state(20240602, 0)
    for i in range(args.warmup):
        sampler.sample_blocks(None, batches[i])
    torch.cuda.synchronize()
    frontiers = []
    stage_stats = []
    for i in range(args.steps):
        events[i][0].record()
        r = sampler.sample_blocks(None, batches[args.warmup + i])
        events[i][1].record()
        frontiers.append(r[0].clone())  # a copy, outside the events: the batch's own block goes back to the pool
        stage_stats.append(sizes(r))
        widest_hop_seeds = r[2][0].dst_ids
    del r
    torch.cuda.synchronize()
    gather_ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(args.steps)]
    for i in range(args.steps):  # queued back to back: the GPU never waits for the host
        gather_ev[i][0].record()
        x = ct_feats._CAPI_index(frontiers[i])
        gather_ev[i][1].record()
    torch.cuda.synchronize()
    del x, frontiers

    def total_bytes(all_stats):
        bs = bu = bg = 0
        for s in all_stats:
            a, b, c = algorithmic_bytes(s, cfg["feat_dim"], feat_bytes)
            bs, bu, bg = bs + a, bu + b, bg + c
        return bs, bu, bg

    ms_step = 1e3 * elapsed / args.steps
    ms_sample = float(np.mean([e[0].elapsed_time(e[1]) for e in events]))
    ms_gather = float(np.mean([e[0].elapsed_time(e[1]) for e in gather_ev]))
    edges = sum(sum(h[1] for h in s["hops"]) for s in stats)
    rows = sum(s["frontier"] for s in stats)
    bs, bu, bg = total_bytes(stats)
    stage_edges = sum(sum(h[1] for h in s["hops"]) for s in stage_stats)
    stage_rows = sum(s["frontier"] for s in stage_stats)
    sbs, sbu, sbg = total_bytes(stage_stats)  # the batches of the stage-split runs (same seeds, their own picks)
    gather_gbps = sbg / args.steps / (ms_gather * 1e-3) / 1e9
    sampler_gbps = (sbs + sbu) / args.steps / (ms_sample * 1e-3) / 1e9
    step_gbps = (bs + bu + bg) / elapsed / 1e9
    traffic_per_row, traffic_source = measured_gather_traffic() if args.workload in ("c1", "c1w") else (None, None)

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
                               f"uniform seeds, fanouts {cfg['fanouts']} without replacement"
                               f"{', weighted by a float32 weight per edge' if cfg.get('weighted') else ''}, then gather",
                   "fanouts": cfg["fanouts"], "batch": cfg["batch"], "batches_in_flight": inflight,
                   "setup_batches": setup_batches,
                   "timed": "value / ms_per_step: the fused operator (_CAPI_sample_blocks_submit, sampling + "
                            "relabel of every hop + gather per batch), seeds resident in HBM, "
                            f"{inflight} batches in flight on as many streams, each batch left on its own stream"},
        "ms_per_step_repeats": repeats,
        "ms_per_batch_alone": ms_latency,
        "ms_per_step_handed_over": ms_handed_over,
        "ms_per_step_host_seeds": ms_host_seeds,
        "ms_per_step_handed_over_host_seeds": ms_handed_over_host_seeds,
        "ms_per_step_seed_loader": ms_seed_loader,
        "ms_per_step_per_hop_ops": ms_per_hop_ops,
        "ms_per_step_per_hop_ops_no_gather": ms_per_hop_ops_no_gather,
        "ms_per_step_per_hop_ops_light_dispatch": ms_per_hop_ops_light,
        "timings": {"ms_per_step_repeats": "the timed region run three more times (spread)",
                    "ms_per_batch_alone": "one batch at a time, one stream, call to result",
                    "ms_per_step_handed_over": "as the headline, each batch handed to the calling stream "
                                               "(at most three batches in flight: the calling stream is a stream too)",
                    "ms_per_step_host_seeds": "as the headline, seeds passed as pageable host tensors",
                    "ms_per_step_handed_over_host_seeds": "host seeds in, each batch handed to the calling stream",
                    "ms_per_step_seed_loader": "the training loop's own shape: SeedLoader where upstream builds the DGL "
                                               "DataLoader (host ids in, batches cut by the loader, each handed to the "
                                               "calling stream with its feature rows)",
                    "ms_per_step_per_hop_ops": "upstream's own loop: _CAPI_sample_neighbors_with_chunk_tensor + "
                                               "_CAPI_tensor_relabel per hop, then _CAPI_index, one batch at a time",
                    "ms_per_step_per_hop_ops_no_gather": "that loop without _CAPI_index: the six operator calls alone",
                    "ms_per_step_per_hop_ops_light_dispatch": "that loop (with _CAPI_index) after "
                                                              "lighten_torch_dispatch(), operators called by their C++ entries",
                    "what_an_unmodified_harness_sees": "ms_per_step_per_hop_ops (one batch at a time through the "
                                                       "upstream operator names); with this package's ChunkTensorSampler "
                                                       "in the place of upstream's class: ms_per_batch_alone; with "
                                                       "SeedLoader in the place of the DataLoader as well: "
                                                       "ms_per_step_seed_loader; the headline leaves each batch on "
                                                       "its own stream"},
        "sample_edges_per_s": stage_edges / args.steps / (ms_sample * 1e-3),
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
                     "traffic": None if traffic_per_row is None else traffic_per_row * stage_rows / args.steps,
                     "traffic_source": traffic_source,
                     "algorithmic_bytes": sbg / args.steps, "avg_launch_us": 1e3 * ms_gather},
        "stages": [
            {"stage": "sampling + relabel of every hop (fused sampler kernels, one batch alone on one stream)",
             "bound": "hbm", "achieved": sampler_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
             "frac": sampler_gbps / HBM_PEAK_GBPS, "algorithmic_bytes": (sbs + sbu) / args.steps,
             "avg_us": 1e3 * ms_sample},
            {"stage": "feature gather of the last frontier (gather_flat_kernel)",
             "bound": "hbm", "achieved": gather_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
             "frac": gather_gbps / HBM_PEAK_GBPS, "algorithmic_bytes": sbg / args.steps,
             "avg_us": 1e3 * ms_gather},
            {"stage": "whole step as timed for the headline", "bound": "hbm", "achieved": step_gbps,
             "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": step_gbps / HBM_PEAK_GBPS,
             "algorithmic_bytes": (bs + bu + bg) / args.steps, "avg_us": 1e3 * ms_step},
        ],
        "graph_gen_s": t_gen,
    }
    if args.workload != "c0":
        # on a table the size of the sampler's node table; eight times the picks of the widest hop per
        # launch, so that a launch lasts long enough for the host's launch rate not to show
        out["table_access_rates"] = table_access_rates(dgs, cfg["nodes"], 8 * int(max(h[1] for h in stats[0]["hops"])))
    if cfg.get("weighted"):
        # the weighted fill of the widest hop alone: its input is every weight of every sampled row
        ops = torch.ops.dgs_ops
        seeds = widest_hop_seeds
        k = cfg["fanouts"][0]
        ip_dev = ct_indptr._CAPI_get_sub_device_tensor()
        degs = ip_dev[seeds + 1] - ip_dev[seeds]
        scanned = int(degs[degs > k].sum().item())
        t = time_call(lambda: ops._CAPI_sample_neighbors_with_probs_with_chunk_tensor(
            seeds, ct_indptr, ct_indices, ct_probs, k, cfg["replace"]), 10)
        out["weighted_hop"] = {"seeds": seeds.numel(), "num_picks": k, "weights_scanned": scanned,
                               "us_per_call": 1e6 * t, "weights_per_s": scanned / t,
                               "weights_GBps": 4 * scanned / t / 1e9,
                               "hbm_frac_of_weight_bytes": 4 * scanned / t / 1e9 / HBM_PEAK_GBPS}
    if not args.no_cpu_baseline:
        cb = cpu_baseline(cfg, indptr, indices, feats, batches_cpu[args.warmup:], args.cpu_budget_s, probs)
        out["cpu_baseline"] = cb
        out["gpu_over_cpu"] = out["value"] / cb["value"]
        # leg by leg, each GPU stage alone on one stream against the same stage of the CPU run
        out["gpu_over_cpu_per_leg"] = {
            "sampling_relabel": out["sample_edges_per_s"] / cb["sample_edges_per_s"],
            "gather": out["gather_GBps"] / cb["gather_GBps"],
            "note": "stage alone on the GPU (events around it) over the same stage on the CPU"}
    if args.workload == "c1" and not args.no_other_workloads:
        # The other benchmark configurations, after the headline and never at its cost: a leg that
        # fails becomes {"error": ...}.  c1w reuses this graph (c1 + a float32 weight per edge).
        others = {}
        t_others = time.perf_counter()
        k_other, w_other = args.other_steps, min(args.warmup, 3)

        def guarded(name, fn):
            if time.perf_counter() - t_others > args.other_budget_s:
                others[name] = {"skipped": f"the {args.other_budget_s:.0f} s for the other workloads were used up"}
                return
            t0 = time.perf_counter()
            try:
                others[name] = fn()
                others[name]["leg_wall_s"] = time.perf_counter() - t0
            except Exception as err:  # noqa: BLE001 (whatever it is, the headline stands)
                others[name] = {"error": f"{type(err).__name__}: {err}"[:500]}
            release_everything()

        def c1w_leg():
            w = make_weights(cfg, indices.numel())
            ct_w = dgs.create_chunktensor(w, 1, big)
            smp = dgs.ChunkTensorSampler(cfg["fanouts"], ct_indptr, ct_indices, ct_w, replace=cfg["replace"])
            some = batches[:k_other + args.warmup]
            run_batches(smp, (some * 4)[:64], ct_feats, inflight, sizes)
            torch.cuda.synchronize()
            el, st = timed_steps(smp, some, inflight)
            el_alone, _ = timed_steps(smp, some, 1)
            ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(k_other)]
            st_stats = []
            for i in range(k_other):
                ev[i][0].record()
                r = smp.sample_blocks(None, some[args.warmup + i])
                ev[i][1].record()
                st_stats.append(sizes(r))
                del r
            torch.cuda.synchronize()
            ms_s = float(np.mean([a.elapsed_time(b) for a, b in ev]))
            wbs, wbu, wbg = total_bytes(st)
            tbs, tbu, _ = total_bytes(st_stats)
            w_edges = sum(sum(h[1] for h in x["hops"]) for x in st)
            weight_bytes = 0  # every weight of every sampled row is read: not counted, as for the uniform picks
            return {"config": {"workload": "c1w: c1 with a float32 weight per edge, weighted picks in every hop "
                                           "(dgs_sample_blocks_weighted), then the same gather",
                               "batches_in_flight": inflight},
                    "steps": k_other, "ms_per_step": 1e3 * el / k_other, "ms_per_batch_alone": 1e3 * el_alone / k_other,
                    "edges_per_s": w_edges / el, "gather_GBps": gather_gbps,
                    "step_algorithmic_GBps": (wbs + wbu + wbg + weight_bytes) / el / 1e9,
                    "step_hbm_frac": (wbs + wbu + wbg + weight_bytes) / el / 1e9 / HBM_PEAK_GBPS,
                    "ms_sample_relabel": ms_s,
                    "stages": [{"stage": "weighted sampling + relabel of every hop, one batch alone on one stream",
                                "bound": "valu (the races), priced against hbm", "achieved": (tbs + tbu) / k_other / (ms_s * 1e-3) / 1e9,
                                "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                "frac": (tbs + tbu) / k_other / (ms_s * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                "algorithmic_bytes": (tbs + tbu) / k_other, "avg_us": 1e3 * ms_s}]}

        guarded("c1w", c1w_leg)
        for name in ("c2", "c4", "c3"):
            guarded(name, lambda name=name: measure_large(name, dgs, k_other, w_other, LARGE_INFLIGHT[name]))
        # what the hottest-rows-first placement buys where a node's popularity follows its degree
        # (the benchmark's own c3 draws sources uniformly: there the hot prefix catches its row share)
        guarded("c3_placement", lambda: measure_placement(dgs))
        if "error" not in others.get("c3", {"error": 1}) and "error" not in others["c3_placement"]:
            others["c3"]["placement"] = others.pop("c3_placement")
        out["other_workloads"] = others
        out["other_workloads_wall_s"] = time.perf_counter() - t_others
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
