"""Pins of the CPU oracle: each oracle function is checked against something it
was not derived from (published known-answer vectors, the reference's README
demo, a numpy library routine, brute force on tiny inputs)."""
import itertools
import math

import numpy as np
import pytest


# ---- Philox4x32-10: Random123 known-answer vectors ------------------------
KAT = [
    ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
     (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


@pytest.mark.parametrize("ctr,key,want", KAT)
def test_philox_known_answers(oracle, ctr, key, want):
    assert tuple(int(x) for x in oracle.philox(ctr, key)) == want


def test_draw_counter_layout(oracle):
    # draw(seed, stream, row, j, n) must be bounded(philox(ctr=(j, stream, row_lo, row_hi),
    # key=(seed_lo, seed_hi)), n): a transposed counter word fails here.
    seed, stream, row, j, n = 0x0123456789abcdef, 7, (5 << 32) | 9, 3, 1000
    w = oracle.philox((j, stream, row & 0xffffffff, row >> 32), (seed & 0xffffffff, seed >> 32))
    assert oracle.draw(seed, stream, row, j, n) == oracle.bounded(w, n)
    # with n = 2^32-1 nearly every word is accepted at the first try: result = floor(w0*n/2^32)
    n = 0xffffffff
    assert oracle.draw(seed, stream, row, j, n) == (int(w[0]) * n) >> 32


def test_bounded_rejection_rule(oracle):
    # brute force the rule on a 2^32 grid is too big; check the rule's definition on
    # hand-built words: a word whose low product half falls under 2^32 mod n is skipped.
    n = 6
    t = (1 << 32) % n  # 4
    # w*n low half < t  <=> rejected.  w = 0 gives low half 0 -> rejected.
    assert oracle.bounded([0, 0x80000001, 1, 1], n) == (0x80000001 * n) >> 32 == 3
    # low half 0..3 is the rejection zone: 0x80000000*6 = 3*2^32 has low half 0 -> skipped too
    assert oracle.bounded([0x80000000, 0x2aaaaaac, 9, 9], n) == (0x2aaaaaac * n) >> 32 == 1
    # 0x2aaaaaab*6 = 2^32 + 2: low half 2 < 4 -> rejected, third word (9*6 = 54) accepted
    assert oracle.bounded([0x80000000, 0x2aaaaaab, 9, 0xffffffff], n) == 0
    # accepted first word
    assert oracle.bounded([0x40000000, 0, 0, 0], n) == (0x40000000 * n) >> 32
    # all four rejected -> last accepted unconditionally
    assert oracle.bounded([0, 0, 0, 0], n) == 0
    assert t == 4
    # n = 1 always 0
    assert oracle.bounded([0xdeadbeef, 1, 2, 3], 1) == 0


def test_bounded_uniform(oracle):
    n = 7
    counts = np.zeros(n)
    for j in range(7000):
        counts[oracle.draw(1, 0, 0, j, n)] += 1
    chi2 = ((counts - 1000) ** 2 / 1000).sum()
    assert chi2 < 22.46  # chi-square 6 dof, p = 0.001


# ---- store split: README demo + invariants ---------------------------------
def test_store_split_readme_demo(oracle):
    # README.md:51-62 / example/demo.py:24: [100] int64 with 200 B -> 25 device, 75 host
    s = oracle.store_split([100], 8, 200)
    assert (s["device_elems"], s["host_elems"], s["threshold"], s["elem_stride"]) == (25, 75, 25, 1)


def test_store_split_invariants(oracle):
    for shape, eb, cap in [([10, 7], 4, 0), ([10, 7], 4, 10 ** 9), ([10, 7], 4, 101), ([3], 8, 23)]:
        s = oracle.store_split(shape, eb, cap)
        assert s["device_elems"] + s["host_elems"] == s["total"] or cap >= s["total"] * eb
        assert s["threshold"] + s["host_elems"] == s["total"]
        if cap == 0:
            assert s["host_elems"] == s["total"]
        if cap >= s["total"] * eb:
            assert s["host_elems"] == 0 and s["device_elems"] == s["total"]
    assert oracle.store_split([10, 7], 4, 101)["device_elems"] == 25  # floor(101 / 4)
    assert oracle.store_split([10, 7], 4, 101)["elem_stride"] == 7


# ---- gather == numpy fancy indexing for every split point -------------------
@pytest.mark.parametrize("dtype", [np.float32, np.int64, np.int32])
def test_gather_matches_numpy(oracle, dtype):
    rng = np.random.default_rng(0)
    full = rng.integers(-1000, 1000, size=(13, 5)).astype(dtype)
    idx = rng.integers(0, 13, size=40).astype(np.int64)
    for thr in range(0, full.size + 1):
        assert np.array_equal(oracle.gather(full, idx, thr), full[idx])
    one_d = full.reshape(-1)
    idx1 = rng.integers(0, one_d.size, size=17).astype(np.int32)
    got = oracle.gather(one_d, idx1, 11)
    assert got.shape == (17, 1) and np.array_equal(got[:, 0], one_d[idx1])


def test_gather_tier_variants(oracle):
    full = np.arange(60, dtype=np.int64).reshape(12, 5)
    thr = 30  # rows 0..5 device, 6..11 host
    assert np.array_equal(oracle.gather(full, np.array([0, 5, 3]), thr, tier=1), full[[0, 5, 3]])
    assert np.array_equal(oracle.gather(full, np.array([6, 11, 7]), thr, tier=2), full[[6, 11, 7]])


def test_split_index_closed_form(oracle):
    rng = np.random.default_rng(1)
    idx = rng.integers(0, 20, size=100).astype(np.int64)
    thr, stride = 53, 5  # threshold/stride = 10 ; device_elems/stride = 10
    loc, rem, host = oracle.split_index(idx, thr, thr, stride)
    assert np.array_equal(host, idx[idx >= 10])
    assert np.array_equal(loc, idx[idx < 10])
    assert rem.size == 0


# ---- sampling ----------------------------------------------------------------
def _toy_graph(rng, n, max_deg):
    deg = rng.integers(0, max_deg + 1, size=n)
    indptr = np.zeros(n + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n, size=indptr[-1]).astype(np.int64)
    return indptr, indices


def test_counts_closed_form(oracle):
    rng = np.random.default_rng(2)
    indptr, _ = _toy_graph(rng, 50, 12)
    seeds = rng.integers(0, 50, size=30).astype(np.int64)
    deg = indptr[seeds + 1] - indptr[seeds]
    for k in (1, 5, 20):
        sub = oracle.sample_counts(seeds, indptr, k, False)
        assert np.array_equal(np.diff(sub), np.minimum(deg, k)) and sub[0] == 0
        sub = oracle.sample_counts(seeds, indptr, k, True)
        assert np.array_equal(np.diff(sub), np.where(deg == 0, 0, k))


def test_full_fanout_is_the_csc_row(oracle):
    rng = np.random.default_rng(3)
    indptr, indices = _toy_graph(rng, 40, 9)
    seeds = rng.permutation(40).astype(np.int64)
    rows, cols = oracle.sample_neighbors(seeds, indptr, indices, 9, False, 123, 0)
    want_r = np.concatenate([np.full(indptr[s + 1] - indptr[s], s) for s in seeds])
    want_c = np.concatenate([indices[indptr[s]:indptr[s + 1]] for s in seeds])
    assert np.array_equal(rows, want_r) and np.array_equal(cols, want_c)


def test_floyd_every_subset_equally_often(oracle):
    # one row of degree 6 with distinct neighbour ids; k = 3: 20 subsets.
    deg, k, trials = 6, 3, 20000
    indptr = np.arange(0, (trials + 1) * deg, deg, dtype=np.int64)
    indices = np.tile(np.arange(deg, dtype=np.int64), trials)
    seeds = np.arange(trials, dtype=np.int64)
    rows, cols = oracle.sample_neighbors(seeds, indptr, indices, k, False, 99, 5)
    assert np.array_equal(rows, np.repeat(seeds, k))
    picks = np.sort(cols.reshape(trials, k), axis=1)
    assert (picks[:, 1:] != picks[:, :-1]).all()  # distinct positions
    codes = picks[:, 0] * 36 + picks[:, 1] * 6 + picks[:, 2]
    subsets = {a * 36 + b * 6 + c: 0 for a, b, c in itertools.combinations(range(deg), k)}
    for c in codes:
        subsets[int(c)] += 1
    cnt = np.array(list(subsets.values()), dtype=float)
    exp = trials / len(cnt)
    chi2 = ((cnt - exp) ** 2 / exp).sum()
    assert len(cnt) == math.comb(deg, k)
    assert chi2 < 43.82  # chi-square 19 dof, p = 0.001


def test_floyd_definition_by_hand(oracle):
    # restate Floyd from the textbook with the oracle's draw() and compare picks
    deg, k, seed, stream, row = 37, 10, 4242, 3, 0
    indptr = np.array([0, deg], dtype=np.int64)
    indices = np.arange(1000, 1000 + deg, dtype=np.int64)
    _, cols = oracle.sample_neighbors(np.array([row]), indptr, indices, k, False, seed, stream)
    chosen = []
    for i in range(k):
        j = deg - k + i
        t = oracle.draw(seed, stream, row, i, j + 1)
        chosen.append(j if t in chosen else t)
    assert list(cols - 1000) == chosen and len(set(chosen)) == k


def test_replace_draws(oracle):
    deg, k = 11, 25
    indptr = np.array([0, 0, deg], dtype=np.int64)  # row 0 empty, row 1 has 11
    indices = np.arange(500, 500 + deg, dtype=np.int64)
    rows, cols = oracle.sample_neighbors(np.array([0, 1, 1]), indptr, indices, k, True, 8, 1)
    assert rows.size == 2 * k and (rows == 1).all()
    want = [500 + oracle.draw(8, 1, 1, j, deg) for j in range(k)]
    assert list(cols[:k]) == want and list(cols[k:]) == want  # keyed by row id, not slot


def test_sampling_mixed_widths(oracle):
    rng = np.random.default_rng(4)
    indptr, indices = _toy_graph(rng, 64, 30)
    seeds = rng.integers(0, 64, size=50)
    r64, c64 = oracle.sample_neighbors(seeds.astype(np.int64), indptr, indices, 7, False, 5, 2)
    r32, c32 = oracle.sample_neighbors(seeds.astype(np.int32), indptr.astype(np.int32),
                                       indices.astype(np.int32), 7, False, 5, 2)
    assert r32.dtype == np.int32 and np.array_equal(r64, r32) and np.array_equal(c64, c32)
    # tiered graph arrays give the same answer as flat ones
    r, c = oracle.sample_neighbors(seeds.astype(np.int64), indptr, indices, 7, False, 5, 2,
                                   indptr_threshold=20, indices_threshold=333)
    assert np.array_equal(r, r64) and np.array_equal(c, c64)


# ---- unique / relabel ---------------------------------------------------------
def _np_unique_first(x):
    u, first = np.unique(x, return_index=True)
    return u[np.argsort(first, kind="stable")]


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_unique_relabel_vs_numpy(oracle, dtype):
    rng = np.random.default_rng(5)
    for n, hi in [(1, 5), (100, 20), (1000, 100000), (4096, 4096), (777, 3)]:
        seeds = rng.permutation(hi)[: min(hi, 10)].astype(dtype)
        cols = rng.integers(0, hi, size=n).astype(dtype)
        rows = rng.choice(seeds, size=n).astype(dtype)
        uniq, (rl, cl) = oracle.unique_relabel([seeds, cols], [rows, cols])
        want = _np_unique_first(np.concatenate([seeds, cols]))
        assert np.array_equal(uniq, want)
        assert np.array_equal(uniq[: seeds.size], seeds)
        assert np.array_equal(uniq[rl], rows) and np.array_equal(uniq[cl], cols)
        assert uniq.dtype == dtype and rl.dtype == dtype


def test_relabel_absent_key(oracle):
    uniq, (r,) = oracle.unique_relabel([np.array([5, 3, 5], dtype=np.int64)],
                                       [np.array([3, 9, 5], dtype=np.int64)])
    assert list(uniq) == [5, 3] and list(r) == [1, -1, 0]


def test_unique_colliding_keys(oracle):
    # keys equal modulo the table size stress the triangular probe
    keys = (np.arange(50, dtype=np.int64) * 64) % 1024 + 1024 * np.arange(50)
    keys = np.concatenate([keys, keys[::-1]])
    uniq, (r,) = oracle.unique_relabel([keys], [keys])
    assert np.array_equal(uniq, keys[:50]) and np.array_equal(uniq[r], keys)


def test_unique_empty(oracle):
    e = np.empty(0, dtype=np.int64)
    uniq, (r,) = oracle.unique_relabel([e], [e])
    assert uniq.size == 0 and r.size == 0


# ---- multi-layer driver ---------------------------------------------------------
def test_sample_blocks_structure(oracle):
    rng = np.random.default_rng(6)
    indptr, indices = _toy_graph(rng, 300, 25)
    seeds = rng.permutation(300)[:16].astype(np.int64)
    fanouts = [7, 4, 2]
    frontier, out_seeds, blocks = oracle.sample_blocks(seeds, indptr, indices, fanouts, False, 77)
    assert np.array_equal(out_seeds, seeds) and len(blocks) == 3
    # the block nearest the seeds is last and was sampled with fanouts[-1]
    src_l, dst_l, n_src, n_dst, src_ids, dst_ids = blocks[-1]
    assert np.array_equal(dst_ids, seeds) and n_dst == 16
    deg = indptr[seeds + 1] - indptr[seeds]
    assert src_l.size == np.minimum(deg, 2).sum()
    # chaining: each block's destination ids are the next block's frontier
    for outer, inner in zip(blocks[:-1], blocks[1:]):
        assert np.array_equal(outer[5], inner[4])
    assert np.array_equal(blocks[0][4], frontier)
    for src_l, dst_l, n_src, n_dst, src_ids, dst_ids in blocks:
        assert np.array_equal(src_ids[:n_dst], dst_ids)  # seeds come first in the frontier
        assert src_l.max(initial=-1) < n_src and dst_l.max(initial=-1) < n_dst
        # every edge (src -> dst) is an edge of the graph
        for s, d in zip(src_ids[src_l][:200], dst_ids[dst_l][:200]):
            assert s in indices[indptr[d]:indptr[d + 1]]
