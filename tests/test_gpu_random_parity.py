"""Randomised parity sweep (GPU): random graphs, id widths, tier splits, fanouts, seed lists and
generator states; the fused driver, the per-hop operators and the weighted driver against the
CPU oracle, the gathered rows against the stored rows.  Seeds are fixed: a failure names its case."""
import numpy as np
import pytest
import torch

from helpers import load_pkg, powerlaw_graph, LAST_HOP_MODES, set_last_hop_mode

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pkg():
    return load_pkg()


@pytest.fixture(params=LAST_HOP_MODES)
def last_hop(request, pkg):
    set_last_hop_mode(pkg, request.param)
    yield request.param
    set_last_hop_mode(pkg, LAST_HOP_MODES[0])


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _np(t):
    return t.cpu().numpy()


def _same_blocks(got, want):
    return all(np.array_equal(_np(g.src_local), w[0]) and np.array_equal(_np(g.dst_local), w[1])
               for g, w in zip(got, want)) and len(got) == len(want)


@pytest.mark.parametrize("sweep", [2024, 7])
def test_random_cases_match_the_oracle(pkg, oracle, sweep, last_hop):
    rng = np.random.default_rng(sweep)
    big = 1 << 40
    for case in range(40):
        n = int(rng.integers(1, 6000))
        idt = rng.choice([np.int32, np.int64])
        pdt = rng.choice([np.int32, np.int64])
        indptr, indices = powerlaw_graph(rng, n, int(rng.integers(1, 40)), int(rng.integers(1, 3000)),
                                         zero_frac=float(rng.random() * 0.3), id_dtype=idt, ptr_dtype=pdt)
        probs = (rng.random(indices.size) ** 4).astype(np.float32)
        probs[rng.random(indices.size) < 0.1] = 0
        fan = [int(rng.integers(0, 20)) for _ in range(int(rng.integers(1, 4)))]
        if rng.random() < 0.2:
            fan[0] = int(rng.integers(30, 65))
        replace = bool(rng.random() < 0.4)
        seeds = rng.integers(0, n, size=int(rng.integers(0, 700))).astype(idt)
        what = (sweep, case, n, idt.__name__, pdt.__name__, fan, replace, seeds.size)

        def store(a):  # nothing, a part or all of the tensor in HBM
            return pkg.create_chunktensor(torch.from_numpy(a), 1, big, cache_rate=float(rng.choice([0.0, 0.3, 1.0])))

        ip_ct, ix_ct, pr_ct = store(indptr), store(indices), store(probs)
        feats = rng.integers(0, 1 << 30, size=(n, int(rng.integers(1, 70)))).astype(np.int32)
        x_ct = store(feats)
        seed, stream = int(rng.integers(0, 2 ** 62)), int(rng.integers(0, 1000))
        want_f, _, want_b = oracle.sample_blocks(seeds, indptr, indices, fan, replace, seed, stream)
        for fused in (True, False):
            pkg.set_rng_state(seed, stream)
            sampler = pkg.ChunkTensorSampler(fan, ip_ct, ix_ct, replace=replace, fused=fused)
            f, _, blocks, x = sampler.sample_blocks_and_index(None, _dev(seeds), x_ct)
            assert np.array_equal(_np(f), want_f), ("frontier", fused) + what
            assert np.array_equal(_np(x), feats[want_f]), ("features", fused) + what
            assert _same_blocks(blocks, want_b), ("blocks", fused) + what
        fan_w = fan if replace else [min(k, 64) for k in fan]
        want_f, _, want_b = oracle.sample_blocks(seeds, indptr, indices, fan_w, replace, seed, stream, probs=probs)
        pkg.set_rng_state(seed, stream)
        f, _, blocks = pkg.ChunkTensorSampler(fan_w, ip_ct, ix_ct, pr_ct, replace).sample_blocks(None, _dev(seeds))
        assert np.array_equal(_np(f), want_f), ("weighted frontier",) + what
        assert _same_blocks(blocks, want_b), ("weighted blocks",) + what


def test_random_larger_cases_match_the_oracle(pkg, oracle, last_hop):
    # fewer, larger cases: up to 300 k nodes, up to five hops, several thousand seeds, so that
    # frontiers span many tiles and the last hop's units many pieces per bucket; worst-case sizes
    # (seeds x product of (1 + fanout)) are kept below 2 * 10^7 ids
    rng = np.random.default_rng(99)
    big = 1 << 40
    for case in range(8):
        n = int(rng.integers(50_000, 300_000))
        idt = rng.choice([np.int32, np.int64])
        indptr, indices = powerlaw_graph(rng, n, int(rng.integers(4, 24)), int(rng.integers(50, 5000)),
                                         zero_frac=float(rng.random() * 0.2), id_dtype=idt, ptr_dtype=np.int64)
        while True:
            fan = [int(rng.integers(1, 13)) for _ in range(int(rng.integers(2, 6)))]
            n_seeds = int(rng.integers(500, 5000))
            if n_seeds * np.prod([1 + k for k in fan]) <= 2e7:
                break
        replace = bool(rng.random() < 0.3)
        seeds = rng.integers(0, n, size=n_seeds).astype(idt)
        what = (case, n, idt.__name__, fan, replace, n_seeds)
        ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, big)
        ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, big)
        seed, stream = int(rng.integers(0, 2 ** 62)), int(rng.integers(0, 1000))
        want_f, _, want_b = oracle.sample_blocks(seeds, indptr, indices, fan, replace, seed, stream)
        pkg.set_rng_state(seed, stream)
        f, _, blocks = pkg.ChunkTensorSampler(fan, ip_ct, ix_ct, replace=replace).sample_blocks(None, _dev(seeds))
        assert np.array_equal(_np(f), want_f), ("frontier",) + what
        assert _same_blocks(blocks, want_b), ("blocks",) + what
