"""The committed fixtures: oracle (CPU, always) and kernels (GPU) must reproduce them."""
import json
import os

import numpy as np
import pytest

from helpers import load_pkg

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = [(5, False), (20, False), (70, False), (6, True), (80, True)]


@pytest.fixture(scope="module")
def gold():
    return np.load(os.path.join(GOLD, "sample_small.npz"))


def test_oracle_reproduces_readme_demo(oracle):
    d = json.load(open(os.path.join(GOLD, "readme_demo.json")))
    s = oracle.store_split(d["shape"], 8, d["capacity_per_gpu"])
    full = np.arange(100)
    assert list(full[: s["threshold"]]) == d["device_tensor"]
    assert list(full[s["threshold"]:]) == d["host_tensor"]


def test_oracle_reproduces_draws(oracle):
    d = json.load(open(os.path.join(GOLD, "philox_draws.json")))
    for seed, stream, row, j, n, value in d["draws"]:
        assert oracle.draw(seed, stream, row, j, n) == value


def test_oracle_reproduces_samples(oracle, gold):
    seed, stream = int(gold["rng_seed"][0]), int(gold["rng_stream"][0])
    for k, replace in CASES:
        tag = f"k{k}_{'rep' if replace else 'norep'}"
        r, c = oracle.sample_neighbors(gold["seeds"], gold["indptr"], gold["indices"], k, replace, seed, stream)
        assert np.array_equal(r, gold[f"rows_{tag}"]) and np.array_equal(c, gold[f"cols_{tag}"])
    u, (rl, cl) = oracle.unique_relabel([gold["seeds"], gold["cols_k5_norep"]],
                                        [gold["rows_k5_norep"], gold["cols_k5_norep"]])
    assert np.array_equal(u, gold["unique"]) and np.array_equal(rl, gold["rows_local"])
    assert np.array_equal(cl, gold["cols_local"])


@pytest.mark.gpu
def test_kernels_reproduce_samples(gold):
    import torch
    pkg = load_pkg()
    capi = pkg.capi
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    seed, stream = int(gold["rng_seed"][0]), int(gold["rng_stream"][0])
    ip, ix, seeds = dev(gold["indptr"]), dev(gold["indices"]), dev(gold["seeds"])
    for k, replace in CASES:
        tag = f"k{k}_{'rep' if replace else 'norep'}"
        r, c, flags = capi.sample_neighbors(seeds, capi.tensor_view(ip), capi.tensor_view(ix), k, replace, seed, stream)
        assert flags == 0
        assert np.array_equal(r.cpu().numpy(), gold[f"rows_{tag}"])
        assert np.array_equal(c.cpu().numpy(), gold[f"cols_{tag}"])
    u, (rl, cl) = capi.unique_relabel([seeds, dev(gold["cols_k5_norep"])],
                                      [dev(gold["rows_k5_norep"]), dev(gold["cols_k5_norep"])])
    assert np.array_equal(u.cpu().numpy(), gold["unique"])
    assert np.array_equal(rl.cpu().numpy(), gold["rows_local"]) and np.array_equal(cl.cpu().numpy(), gold["cols_local"])
    # the multi-layer driver through the operator layer
    ct_ip = pkg.create_chunktensor(torch.from_numpy(gold["indptr"]), 1, 1 << 40)
    ct_ix = pkg.create_chunktensor(torch.from_numpy(gold["indices"]), 1, 1 << 40, cache_rate=0.5)
    pkg.set_rng_state(seed, 100)
    frontier, _, blocks = pkg.ChunkTensorSampler([4, 3, 2], ct_ip, ct_ix).sample_blocks(None, torch.from_numpy(gold["seeds"]))
    assert np.array_equal(frontier.cpu().numpy(), gold["blocks_frontier"])
    for i, b in enumerate(blocks):
        assert np.array_equal(b.src_local.cpu().numpy(), gold[f"block{i}_src"])
        assert np.array_equal(b.dst_local.cpu().numpy(), gold[f"block{i}_dst"])


WEIGHTED_CASES = [(5, False), (20, False), (64, False), (6, True), (80, True)]


def test_oracle_reproduces_weighted_samples(oracle, gold):
    wg = np.load(os.path.join(GOLD, "weighted_small.npz"))
    seed = int(gold["rng_seed"][0])
    for x, bits in zip(wg["neg_log_x"], wg["neg_log_bits"]):
        assert np.float64(oracle.neg_log_u32(int(x))).view(np.uint64) == bits
    for k, replace in WEIGHTED_CASES:
        tag = f"k{k}_{'rep' if replace else 'norep'}"
        r, c = oracle.sample_neighbors_weighted(gold["seeds"], gold["indptr"], gold["indices"], wg["probs"], k,
                                                replace, seed, 23)
        assert np.array_equal(r, wg[f"rows_{tag}"]) and np.array_equal(c, wg[f"cols_{tag}"])


@pytest.mark.gpu
def test_kernels_reproduce_weighted_samples(gold):
    import torch
    pkg = load_pkg()
    capi = pkg.capi
    wg = np.load(os.path.join(GOLD, "weighted_small.npz"))
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    seed = int(gold["rng_seed"][0])
    ip, ix, pr, seeds = dev(gold["indptr"]), dev(gold["indices"]), dev(wg["probs"]), dev(gold["seeds"])
    for k, replace in WEIGHTED_CASES:
        tag = f"k{k}_{'rep' if replace else 'norep'}"
        r, c, flags = capi.sample_neighbors_weighted(seeds, capi.tensor_view(ip), capi.tensor_view(ix),
                                                     capi.tensor_view(pr), k, replace, seed, 23)
        assert flags == 0
        assert np.array_equal(r.cpu().numpy(), wg[f"rows_{tag}"])
        assert np.array_equal(c.cpu().numpy(), wg[f"cols_{tag}"])


@pytest.mark.gpu
def test_kernels_reproduce_readme_demo():
    import torch
    pkg = load_pkg()
    d = json.load(open(os.path.join(GOLD, "readme_demo.json")))
    c = pkg.ChunkTensor(d["shape"], torch.int64, d["capacity_per_gpu"])
    c._CAPI_load_from_tensor(torch.arange(100))
    assert c._CAPI_get_host_tensor().tolist() == d["host_tensor"]
    assert c._CAPI_get_sub_device_tensor().cpu().tolist() == d["device_tensor"]
