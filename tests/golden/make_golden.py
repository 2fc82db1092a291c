"""Writes the committed fixtures in this directory.

The upstream repository has no tests and holds one known answer (the README demo
of the ChunkTensor split); that one is written to readme_demo.json by hand below.
Everything else here is produced by the CPU oracle once its pins pass
(tests/test_oracle.py) and freezes the "dgs-philox-1" random-pick contract, so a
later change to oracle or kernels that alters results is caught.

Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle  # noqa: E402


def main():
    # upstream README.md:51-62 / example/demo.py:24-36
    json.dump({"shape": [100], "dtype": "int64", "capacity_per_gpu": 200,
               "device_tensor": list(range(0, 25)), "host_tensor": list(range(25, 100))},
              open(os.path.join(HERE, "readme_demo.json"), "w"))

    rng = np.random.default_rng(7)
    n = 400
    deg = np.minimum(np.floor(rng.pareto(1.2, size=n) * 4).astype(np.int64), 120)
    indptr = np.zeros(n + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n, size=int(indptr[-1])).astype(np.int64)
    seeds = rng.permutation(n)[:48].astype(np.int64)
    out = {"indptr": indptr, "indices": indices, "seeds": seeds,
           "rng_seed": np.array([0x5EED1234ABCD], dtype=np.uint64), "rng_stream": np.array([17], dtype=np.uint32)}
    for k, replace in [(5, False), (20, False), (70, False), (6, True), (80, True)]:
        r, c = oracle.sample_neighbors(seeds, indptr, indices, k, replace, 0x5EED1234ABCD, 17)
        tag = f"k{k}_{'rep' if replace else 'norep'}"
        out[f"rows_{tag}"] = r
        out[f"cols_{tag}"] = c
    r, c = out["rows_k5_norep"], out["cols_k5_norep"]
    u, (rl, cl) = oracle.unique_relabel([seeds, c], [r, c])
    out.update(unique=u, rows_local=rl, cols_local=cl)
    frontier, _, blocks = oracle.sample_blocks(seeds, indptr, indices, [4, 3, 2], False, 0x5EED1234ABCD, 100)
    out["blocks_frontier"] = frontier
    for i, b in enumerate(blocks):
        out[f"block{i}_src"] = b[0]
        out[f"block{i}_dst"] = b[1]
    np.savez_compressed(os.path.join(HERE, "sample_small.npz"), **out)
    # weighted sampling on the same graph: weights over many binades with zeros, a negative, ties
    w = (rng.random(indices.size) ** 5 * 50.0).astype(np.float32)
    w[rng.random(indices.size) < 0.08] = 0.0
    w[rng.random(indices.size) < 0.15] = np.float32(0.25)
    w[3] = -1.0
    wout = {"probs": w}
    for k, replace in [(5, False), (20, False), (64, False), (6, True), (80, True)]:
        r, c = oracle.sample_neighbors_weighted(seeds, indptr, indices, w, k, replace, 0x5EED1234ABCD, 23)
        tag = f"k{k}_{'rep' if replace else 'norep'}"
        wout[f"rows_{tag}"] = r
        wout[f"cols_{tag}"] = c
    xs = np.array([0, 1, 2, 1000, 2 ** 31 - 1, 2 ** 31, 3037000499, 3037000500, 2 ** 32 - 2, 2 ** 32 - 1], dtype=np.uint64)
    wout["neg_log_x"] = xs
    wout["neg_log_bits"] = np.array([np.float64(oracle.neg_log_u32(int(x))).view(np.uint64) for x in xs], dtype=np.uint64)
    np.savez_compressed(os.path.join(HERE, "weighted_small.npz"), **wout)
    draws = [[s, st, row, j, nn, oracle.draw(s, st, row, j, nn)]
             for s, st, row, j, nn in [(0, 0, 0, 0, 10), (1, 2, 3, 4, 5), (2 ** 63 + 5, 7, 2 ** 40 + 3, 63, 1000003),
                                       (7777, 0, 2449028, 14, 17000), (42, 4294967295, 1, 0, 4294967295)]]
    json.dump({"columns": ["seed", "stream", "row", "draw", "n", "value"], "draws": draws},
              open(os.path.join(HERE, "philox_draws.json"), "w"))


if __name__ == "__main__":
    main()
