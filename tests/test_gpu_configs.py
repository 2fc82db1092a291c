"""The benchmark configurations at their real shapes and dtypes (GPU).

Each case builds its synthetic graph on the device, runs the fused sampler and the gather,
and checks (a) bit-exact parity with the CPU oracle on the same seeds, and (b) properties that
do not depend on size: per-row pick counts, full-fanout rows equal to the CSC rows, picked ids
are neighbours, distinct frontier with the seeds first, ranks that map back to the ids, the
per-hop operators giving the same answer as the fused one, gathered rows equal to the stored
rows.  Graph arrays reach the stores through the device/host slice views, never through a
host copy of the whole tensor.
"""
import gc

import numpy as np
import pytest
import torch

from helpers import load_pkg

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pkg():
    return load_pkg()


def _free():
    gc.collect()
    torch.cuda.empty_cache()


def _powerlaw_degrees(n, e, max_deg, one_frac, gen):
    """Power-law in-degrees on the device with sum exactly e."""
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
    assert 0 <= rest < n
    cand = torch.nonzero((deg > 1) & (deg < max_deg - 1)).flatten()[:rest]
    deg[cand] += 1
    assert deg.sum().item() == e
    return deg


def _csc_uniform_sources(n, deg, id_dtype, gen):
    indptr = torch.zeros(n + 1, dtype=torch.int64, device="cuda")
    torch.cumsum(deg, 0, out=indptr[1:])
    e = int(indptr[-1].item())
    indices = torch.empty(e, dtype=id_dtype, device="cuda")
    step = 1 << 28
    for a in range(0, e, step):
        b = min(e, a + step)
        indices[a:b] = torch.randint(0, n, (b - a,), generator=gen, device="cuda", dtype=id_dtype)
    return indptr, indices


def _store_from_device(pkg, t, capacity_bytes):
    """A ChunkTensor holding device tensor `t`, filled through its slice views."""
    ct = pkg.ChunkTensor(list(t.shape), t.dtype, capacity_bytes)
    flat = t.reshape(-1)
    dev = ct._CAPI_get_sub_device_tensor()
    dev.copy_(flat[: dev.numel()])
    host = ct._CAPI_get_host_tensor()
    if host.numel():
        step = 1 << 28
        for a in range(0, host.numel(), step):
            b = min(host.numel(), a + step)
            host[a:b].copy_(flat[dev.numel() + a: dev.numel() + b])
    torch.cuda.synchronize()
    return ct


def _check_properties(pkg, indptr, indices, seeds, fanouts, replace, frontier, blocks):
    """Size-independent properties of one sample_blocks result (all on the device)."""
    cur = seeds
    for k, b in zip(reversed(fanouts), reversed(blocks)):
        assert torch.equal(b.dst_ids, cur) and b.num_dst == cur.numel() and b.num_src == b.src_ids.numel()
        deg = indptr[cur.long() + 1] - indptr[cur.long()]
        want = torch.where(deg == 0, 0, k) if replace else torch.clamp(deg, max=k)
        dst = b.dst_local.long()
        distinct_seeds = torch.unique(cur).numel() == cur.numel()  # the caller's seeds may repeat
        if distinct_seeds:
            assert torch.equal(torch.bincount(dst, minlength=cur.numel()), want)
            assert torch.equal(b.src_ids[: cur.numel()], cur)
            assert (dst[1:] >= dst[:-1]).all()  # edges grouped by seed row, rows in order
        assert b.src_local.numel() == int(want.sum().item())
        assert torch.unique(b.src_ids).numel() == b.src_ids.numel()
        assert int(b.src_local.max().item()) < b.num_src and int(dst.max().item()) < b.num_dst
        src_ids = b.src_ids[b.src_local.long()]
        # a repeated seed is relabelled to its first occurrence, which names the same node
        dst_ids = b.src_ids[dst]
        assert torch.equal(dst_ids, torch.repeat_interleave(cur, want))
        if not replace:
            # rows with deg <= k come back whole, in CSC order
            full = deg <= k
            rows = torch.nonzero(full).flatten()
            if rows.numel():
                edge_full = torch.repeat_interleave(full, want)
                starts = indptr[cur[rows].long()]
                lens = deg[rows]
                off = torch.repeat_interleave(starts - (torch.cumsum(lens, 0) - lens), lens)
                pos = off + torch.arange(int(lens.sum().item()), device="cuda")
                assert torch.equal(src_ids[edge_full], indices[pos])
        # every picked id is a neighbour of its row (spot check on the host)
        pick = torch.randint(0, src_ids.numel(), (300,), device="cuda")
        for s, d in zip(src_ids[pick].tolist(), dst_ids[pick].tolist()):
            lo, hi = int(indptr[d].item()), int(indptr[d + 1].item())
            assert (indices[lo:hi] == s).any()
        cur = b.src_ids
    assert torch.equal(cur, frontier)


def _run_case(pkg, oracle, indptr, indices, feats, feat_capacity, seeds, fanouts, replace, oracle_parity=True,
              graph_capacity=1 << 62, ct_x=None):
    ct_ip = _store_from_device(pkg, indptr, graph_capacity)
    ct_ix = _store_from_device(pkg, indices, graph_capacity)
    if ct_x is None:
        ct_x = _store_from_device(pkg, feats, feat_capacity)
    sampler = pkg.ChunkTensorSampler(fanouts, ct_ip, ct_ix, replace=replace)
    pkg.set_rng_state(20240601, 0)
    frontier, _, blocks, x = sampler.sample_blocks_and_index(None, seeds, ct_x)
    torch.cuda.synchronize()
    _check_properties(pkg, indptr, indices, seeds, fanouts, replace, frontier, blocks)
    # gathered rows are the stored rows, bit for bit (integer view: NaN-safe, dtype-agnostic)
    as_int = {2: torch.int16, 4: torch.int32}[feats.element_size()]
    for a in range(0, frontier.numel(), 1 << 20):
        idx = frontier[a: a + (1 << 20)].long()
        assert torch.equal(x[a: a + (1 << 20)].view(as_int), feats[idx].view(as_int))
    # the per-hop operators (separate kernels, exact-size outputs) agree with the fused path
    if max(fanouts) <= 64:
        pkg.set_rng_state(20240601, 0)
        per_hop = pkg.ChunkTensorSampler(fanouts, ct_ip, ct_ix, replace=replace, fused=False)
        f2, _, blocks2 = per_hop.sample_blocks(None, seeds)
        assert torch.equal(f2, frontier)
        for a, b in zip(blocks, blocks2):
            assert torch.equal(a.src_local, b.src_local) and torch.equal(a.dst_local, b.dst_local)
        del f2, blocks2
    if oracle_parity:
        o_frontier, _, o_blocks = oracle.sample_blocks(seeds.cpu().numpy(), indptr.cpu().numpy(),
                                                       indices.cpu().numpy(), fanouts, replace, 20240601, 0)
        assert np.array_equal(frontier.cpu().numpy(), o_frontier)
        for b, ob in zip(blocks, o_blocks):
            assert np.array_equal(b.src_local.cpu().numpy(), ob[0])
            assert np.array_equal(b.dst_local.cpu().numpy(), ob[1])
    return frontier.numel(), sum(b.src_local.numel() for b in blocks)


def test_config0_host_resident_features(pkg, oracle):
    # 10,000 nodes, Zipf(2.1) in-degrees clipped to [1, 1000], features f32 x128 entirely in host memory
    gen = torch.Generator(device="cuda").manual_seed(20240601)
    rng = np.random.default_rng(20240601)
    n = 10_000
    deg = torch.from_numpy(np.clip(rng.zipf(2.1, size=n), 1, 1000)).cuda()
    indptr, indices = _csc_uniform_sources(n, deg, torch.int64, gen)
    feats = torch.randn((n, 128), generator=gen, device="cuda")
    seeds = torch.randint(0, n, (1024,), generator=gen, device="cuda")
    rows, edges = _run_case(pkg, oracle, indptr, indices, feats, 0, seeds, [10, 5], False)
    assert rows > 1024 and edges > 1024


def test_config1_mid_size_all_in_hbm(pkg, oracle):
    # 2,449,029 nodes / 123,718,280 edges, int64 CSC, f32 x100, 1024 seeds, [15, 10, 5]
    gen = torch.Generator(device="cuda").manual_seed(20240602)
    n, e = 2_449_029, 123_718_280
    deg = _powerlaw_degrees(n, e, 17_000, 0.05, gen)
    indptr, indices = _csc_uniform_sources(n, deg, torch.int64, gen)
    feats = torch.randn((n, 100), generator=gen, device="cuda")
    seeds = torch.randint(0, n, (1024,), generator=gen, device="cuda")
    rows, edges = _run_case(pkg, oracle, indptr, indices, feats, 1 << 62, seeds, [15, 10, 5], False)
    assert 300_000 < rows <= 1_081_344 and edges <= 1_080_320
    del indptr, indices, feats
    _free()


def test_config2_large_graph_int32_ids_bf16(pkg, oracle):
    # 111,059,956 nodes / 1,615,685,872 edges, int64 indptr + int32 indices, bf16 x128,
    # 4096 seeds from a fixed 1% subset, [15, 10, 5]
    gen = torch.Generator(device="cuda").manual_seed(20240603)
    n, e = 111_059_956, 1_615_685_872
    deg = _powerlaw_degrees(n, e, 30_000, 0.05, gen)
    indptr, indices = _csc_uniform_sources(n, deg, torch.int32, gen)
    del deg
    feats = torch.empty((n, 128), dtype=torch.bfloat16, device="cuda")
    for a in range(0, n, 1 << 24):
        feats[a: a + (1 << 24)].normal_(generator=gen)
    train = torch.randperm(n, generator=gen, device="cuda")[: n // 100]
    seeds = train[torch.randint(0, train.numel(), (4096,), generator=gen, device="cuda")].to(torch.int32)
    rows, edges = _run_case(pkg, oracle, indptr, indices, feats, 1 << 62, seeds, [15, 10, 5], False)
    assert rows > 100_000 and edges > rows - 4096
    del indptr, indices, feats, train
    _free()


def _config3(pkg, oracle, n, e):
    """The large graph's shape with f32 x256 features: the top 40% of rows (ids are assigned in
    decreasing in-degree) in HBM, the rest in pinned host memory; int32 ids, 8192 seeds, [20, 15, 10]."""
    gen = torch.Generator(device="cuda").manual_seed(20240604)
    deg = _powerlaw_degrees(n, e, 30_000, 0.05, gen)
    deg = torch.sort(deg, descending=True).values  # hottest rows first
    indptr, indices = _csc_uniform_sources(n, deg, torch.int32, gen)
    del deg
    feats = torch.empty((n, 256), dtype=torch.float32, device="cuda")
    for a in range(0, n, 1 << 22):
        feats[a: a + (1 << 22)].normal_(generator=gen)
    hot_rows = int(n * 0.4)
    capacity = hot_rows * 256 * 4 + 4 * 100  # the boundary falls inside a row
    host_bytes = n * 256 * 4 - capacity
    try:
        ct_x = _store_from_device(pkg, feats, capacity)
    except RuntimeError as err:  # the one thing that depends on the machine: pinning the host slice
        del indptr, indices, feats
        _free()
        pytest.skip(f"the {host_bytes / 1e9:.1f} GB host slice could not be allocated as pinned memory: {err}")
    seeds = torch.randint(0, n, (8192,), generator=gen, device="cuda", dtype=torch.int32)
    rows, edges = _run_case(pkg, oracle, indptr, indices, feats, capacity, seeds, [20, 15, 10], False, ct_x=ct_x)
    assert rows > 1_000_000
    # tier-specific gathers on the partitioned frontier give the same rows (the straddling row
    # hot_rows counts as a host row)
    idx = torch.randint(0, n, (200_000,), generator=gen, device="cuda")
    idx[:3] = torch.tensor([hot_rows - 1, hot_rows, hot_rows + 1], device="cuda")
    local, remote, host = ct_x._CAPI_split_index(idx)
    assert remote.numel() == 0 and local.numel() + host.numel() == idx.numel()
    assert torch.equal(local, idx[idx < hot_rows]) and torch.equal(host, idx[idx >= hot_rows])
    assert torch.equal(ct_x._CAPI_local_index(local), feats[local])
    assert torch.equal(ct_x._CAPI_host_index(host), feats[host])
    del indptr, indices, feats, ct_x
    _free()
    return rows, edges


def test_config3_two_tier_features(pkg, oracle):
    # 1/8 of the full size: 5.7 GB in HBM, 8.5 GB pinned
    _config3(pkg, oracle, 13_882_494, 201_960_734)


@pytest.mark.timeout(900)
def test_config3_two_tier_features_full_size(pkg, oracle):
    # 111,059,956 nodes / 1,615,685,872 edges, 113.7 GB of features: 45.5 GB in HBM, 68.2 GB pinned
    rows, edges = _config3(pkg, oracle, 111_059_956, 1_615_685_872)
    assert rows > 2_000_000 and edges > rows - 8192


def _rmat_csc(scale, e, gen):
    """R-MAT (a, b, c, d) = (.57, .19, .19, .05) grouped by destination without sorting: the
    destination bits are independent with P(bit = 1) = b + d, so in-degrees follow from the
    per-node probability, and each source bit is drawn given the destination's bit."""
    a, b, c, d = 0.57, 0.19, 0.19, 0.05
    n = 1 << scale
    ids = torch.arange(n, device="cuda")
    ones = torch.zeros(n, device="cuda", dtype=torch.float64)
    for bit in range(scale):
        ones += ((ids >> bit) & 1).double()
    logp = ones * np.log(b + d) + (scale - ones) * np.log(a + c)
    lam = torch.exp(logp + np.log(e))
    deg = torch.poisson(lam.float(), generator=gen).long()
    diff = int(e - deg.sum().item())  # push the total to exactly e on the heaviest rows
    top = torch.argsort(lam, descending=True)[: abs(diff)]
    deg[top] += 1 if diff > 0 else -1
    deg.clamp_(min=0)
    deg[0] += e - int(deg.sum().item())
    indptr = torch.zeros(n + 1, dtype=torch.int64, device="cuda")
    torch.cumsum(deg, 0, out=indptr[1:])
    indices = torch.empty(e, dtype=torch.int32, device="cuda")
    step = 1 << 26
    for lo in range(0, e, step):
        hi = min(e, lo + step)
        pos = torch.arange(lo, hi, device="cuda")
        dst = torch.searchsorted(indptr, pos, right=True) - 1
        src = torch.zeros(hi - lo, dtype=torch.int32, device="cuda")
        for bit in range(scale):
            dbit = (dst >> bit) & 1
            p1 = torch.where(dbit == 1, d / (b + d), c / (a + c)).float()  # P(source bit = 1 | destination bit)
            src |= (torch.rand(hi - lo, generator=gen, device="cuda") < p1).int() << bit
        indices[lo:hi] = src
    return indptr, indices


def test_config4_replacement_high_fanout_rmat(pkg, oracle):
    # R-MAT scale 26 with 2^30 edges, int32 indices, with replacement, fanouts [50, 50],
    # 16384 seeds, f32 x64 features: frontiers of tens of millions of ids
    gen = torch.Generator(device="cuda").manual_seed(20240605)
    scale, e = 26, 1 << 30
    indptr, indices = _rmat_csc(scale, e, gen)
    n = 1 << scale
    feats = torch.empty((n, 64), dtype=torch.float32, device="cuda")
    for a in range(0, n, 1 << 23):
        feats[a: a + (1 << 23)].normal_(generator=gen)
    seeds = torch.randint(0, n, (16384,), generator=gen, device="cuda", dtype=torch.int32)
    rows, edges = _run_case(pkg, oracle, indptr, indices, feats, 1 << 62, seeds, [50, 50], True)
    assert edges > 1_000_000
    del indptr, indices, feats
    _free()
