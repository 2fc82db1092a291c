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


def _subset_picks(oracle, deg, k, trials, replace=False):
    """[trials, k] picked positions of independent rows of degree `deg` (neighbour id = position).
    Small cases are one call over `trials` rows (draws are keyed by the row id); rows too long for
    that many copies are drawn one call at a time from a single row under `trials` different seeds."""
    if deg * trials <= 30_000_000:
        indptr = np.arange(0, (trials + 1) * deg, deg, dtype=np.int64)
        indices = np.tile(np.arange(deg, dtype=np.int32), trials)
        _, cols = oracle.sample_neighbors(np.arange(trials, dtype=np.int32), indptr, indices, k, replace, 777, 2)
        return cols.reshape(trials, k).astype(np.int64)
    indptr = np.array([0, deg], dtype=np.int64)
    indices = np.arange(deg, dtype=np.int32)
    row = np.zeros(1, dtype=np.int32)
    out = np.empty((trials, k), dtype=np.int64)
    for t in range(trials):
        _, cols = oracle.sample_neighbors(row, indptr, indices, k, replace, 1000 + t, 2)
        out[t] = cols
    return out


@pytest.mark.parametrize("deg,k,trials", [(1000, 15, 20000), (17000, 15, 15000), (30000, 20, 12000), (5000, 3000, 600)])
def test_floyd_is_a_uniform_subset_on_long_rows(oracle, deg, k, trials):
    # The degrees of the benchmark graphs' tails (17 k, 30 k), where the bounded draw works on
    # large ranges, and a fanout in the thousands.  A uniform k-subset includes every position with
    # probability p = k / deg and every pair with k (k - 1) / (deg (deg - 1)).  A wrong range of a
    # step's draw, a wrong replacement position, or a biased reduction shows in one of:
    picks = _subset_picks(oracle, deg, k, trials)
    assert picks.min() >= 0 and picks.max() < deg
    srt = np.sort(picks, axis=1)
    assert (srt[:, 1:] != srt[:, :-1]).all()  # distinct positions in every row
    p = k / deg
    # (1) inclusion counts per position: trials Bernoulli(p) each, negatively correlated across
    # positions; sum (c - E)^2 / (E (1 - p)) * (deg - 1) / deg is chi-square with deg - 1 dof
    counts = np.bincount(picks.ravel(), minlength=deg).astype(float)
    exp = trials * p
    stat = ((counts - exp) ** 2).sum() / (exp * (1 - p)) * (deg - 1) / deg
    dof = deg - 1
    assert abs(stat - dof) < 5 * math.sqrt(2 * dof), (stat, dof)
    # (2) Floyd treats the last k positions differently (they are what a repeated draw is replaced
    # by) and the first deg - k are only ever drawn: both blocks must be included at the common rate
    for lo, hi in ((deg - k, deg), (0, k), (deg - 2 * k, deg - k) if deg >= 3 * k else (0, deg - k)):
        got = counts[lo:hi].sum()
        want = trials * p * (hi - lo)
        sd = math.sqrt(want * (1 - p))  # an upper bound: the counts are negatively correlated
        assert abs(got - want) < 5 * sd, (lo, hi, got, want)
    # (3) pairs: neighbouring positions, mirrored positions, and (first, last) k positions
    member = np.zeros((trials, deg), dtype=bool) if deg * trials <= 40_000_000 else None
    p2 = k * (k - 1) / (deg * (deg - 1))
    if member is not None:
        member[np.arange(trials)[:, None], picks] = True
        both_adjacent = (member[:, 1:] & member[:, :-1]).sum()
        both_mirrored = (member[:, : deg // 2] & member[:, ::-1][:, : deg // 2]).sum()
        for got, pairs in ((both_adjacent, deg - 1), (both_mirrored, deg // 2)):
            want = trials * pairs * p2
            assert abs(got - want) < 5 * math.sqrt(want) + 1, (got, want)
    else:
        # without the membership matrix: count adjacent pairs from the sorted picks
        both_adjacent = (srt[:, 1:] - srt[:, :-1] == 1).sum()
        want = trials * (deg - 1) * p2
        assert abs(both_adjacent - want) < 5 * math.sqrt(want) + 1, (both_adjacent, want)
    # (4) the order of the output slots: slot j holds a draw from [0, deg - k + j] (or that top
    # position itself), so it never exceeds deg - k + j, and it is that top position exactly when the
    # draw repeated an earlier slot or hit the top by itself: probability (j + 1) / (deg - k + j + 1)
    tops = deg - k + np.arange(k)
    assert (picks <= tops[None, :]).all()
    at_top = (picks == tops[None, :]).sum(axis=0).astype(float)
    want_top = trials * (np.arange(k) + 1) / (tops + 1)
    z = (at_top.sum() - want_top.sum()) / math.sqrt(want_top.sum())
    assert abs(z) < 5, (at_top.sum(), want_top.sum())


def test_replace_draws_are_uniform_on_a_long_row(oracle):
    # with replacement on a row of degree 30 000: 3 M independent draws, 100 expected per position
    deg, k = 30000, 3_000_000
    picks = _subset_picks(oracle, deg, k, 1, replace=True).ravel()
    counts = np.bincount(picks, minlength=deg).astype(float)
    exp = k / deg
    stat = ((counts - exp) ** 2 / exp).sum()
    assert abs(stat - (deg - 1)) < 5 * math.sqrt(2 * (deg - 1)), stat
    # consecutive draws are independent: how often draw j + 1 lands in the same hundredth of the row as draw j
    same = (picks[1:] // 300 == picks[:-1] // 300).sum()
    assert abs(same - (k - 1) / 100) < 5 * math.sqrt((k - 1) / 100)


@pytest.mark.parametrize("n", [65537, 65535, 2 ** 16 + 2 ** 15 + 1, 2 ** 31 - 1, 2 ** 31 + 12345, 3 * 2 ** 30, 2 ** 32 - 5])
def test_bounded_accepts_the_same_number_of_words_for_every_value(oracle, n):
    # Lemire's reduction maps word w to v = floor(w n / 2^32) and must accept, for EVERY v, exactly
    # floor(2^32 / n) of the words that map to it (that is what makes it unbiased); the words that
    # map to v are the integers of [v 2^32 / n, (v + 1) 2^32 / n).  Counted by brute force over all
    # of them, for values at both ends and in the middle of the range, with n on either side of
    # 2^16 and 2^31, where the rejection zone 2^32 mod n is small, large, or nearly all of n.
    import ctypes
    lib = oracle.lib()
    per_value = 2 ** 32 // n
    words = np.zeros(4, dtype=np.uint32)
    ptr = ctypes.c_void_p(words.ctypes.data)
    # a word that is accepted whatever happens and maps to a value no tested word maps to
    marker_value = n // 3 + 7
    marker = next(w for w in range(-(-(marker_value << 32) // n), -(-((marker_value + 1) << 32) // n))
                  if (w * n) % 2 ** 32 >= 2 ** 32 % n)
    values = [0, 1, 2, n // 2, n - 2, n - 1] + [int(x) for x in np.random.default_rng(n % 1000).integers(0, n, size=6)]
    zone = 2 ** 32 % n
    for v in values:
        if v == marker_value:
            continue
        lo = -(-(v << 32) // n)          # ceil(v 2^32 / n)
        hi = -(-((v + 1) << 32) // n)    # ceil((v + 1) 2^32 / n)
        assert hi - lo in (per_value, per_value + 1)
        accepted = 0
        for w in range(lo, hi):
            words[:] = (w, marker, marker, marker)
            got = lib.oracle_bounded(ptr, ctypes.c_uint32(n))
            assert got in (v, marker_value)
            accepted += got == v
        assert accepted == per_value, (n, v, accepted, per_value)
        # (the rejected word, when there is one, is the one whose product falls in the zone)
        assert (hi - lo == per_value + 1) == any((w * n) % 2 ** 32 < zone for w in range(lo, hi))


@pytest.mark.parametrize("n", [65537, 2 ** 31 + 12345, 3 * 2 ** 30])
def test_bounded_draws_follow_the_contract_near_the_powers_of_two(oracle, n):
    # The draws themselves (Philox words, not hand-made ones), 400 k of them.  The contract accepts
    # the fourth word of a block unconditionally, so a value v comes up with probability
    #   (1 - q^3) / n + q^3 * (words that map to v) / 2^32,   q = (2^32 mod n) / 2^32:
    # uniform but for q^3, which is 2e-15 at n = 65537 (and less on any real row), 1/8 just above
    # 2^31 (where nearly every value has two words, so the skew stays invisible) and 1/64 at
    # n = 3 * 2^30, where every third value has two words and the other two one: that residue class
    # must come up 1/3 + (1/64)(1/2 - 1/3) of the time, no more (a dropped rejection would give
    # 1/2) and no less (a fifth word, or none, would give 1/3).
    import ctypes
    lib = oracle.lib()
    draws = np.array([lib.oracle_draw(ctypes.c_uint64(31337), ctypes.c_uint32(9), ctypes.c_int64(j >> 10),
                                      ctypes.c_uint32(j & 1023), ctypes.c_uint32(n)) for j in range(400_000)],
                     dtype=np.int64)
    assert draws.min() >= 0 and draws.max() < n
    q3 = (2 ** 32 % n / 2 ** 32) ** 3
    cells = 64
    edges = [c * n // cells for c in range(cells + 1)]
    words_into = np.array([-(-(edges[c + 1] << 32) // n) - -(-(edges[c] << 32) // n) for c in range(cells)], dtype=float)
    sizes = np.diff(np.array(edges, dtype=float))
    exp = draws.size * ((1 - q3) * sizes / n + q3 * words_into / 2 ** 32)
    counts = np.bincount(np.searchsorted(np.array(edges[1:]), draws, side="right"), minlength=cells).astype(float)
    stat = ((counts - exp) ** 2 / exp).sum()
    assert stat < cells - 1 + 5 * math.sqrt(2 * (cells - 1)), (n, stat)
    if n == 3 * 2 ** 30:
        counts = np.bincount(draws % 3, minlength=3).astype(float)
        share = np.array([0.5, 0.25, 0.25])  # words per value: 2, 1, 1, repeating
        exp = draws.size * ((1 - q3) / 3 + q3 * share)
        stat = ((counts - exp) ** 2 / exp).sum()
        assert stat < 2 + 5 * math.sqrt(4), (counts, exp, stat)
        uniform = draws.size / 3
        assert ((counts - uniform) ** 2 / uniform).sum() > 10  # the contract's skew is there, and it is this one


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


@pytest.mark.parametrize("dtype", [np.int64, np.int32])
def test_parallel_unique_relabel_is_the_sequential_one(oracle, dtype):
    # the all-threads variant that the benchmark's CPU baseline times gives the sequential
    # restatement's results, bit for bit: sizes around the shard and thread counts, many repeats, few
    # repeats, absent and negative ids to look up, nothing at all
    rng = np.random.default_rng(17)
    for n, hi in [(0, 10), (1, 10), (7, 3), (100, 1000), (5000, 300), (200000, 50000), (200000, 2 ** 30), (1 << 20, 1 << 21)]:
        mapping = [rng.integers(0, hi, size=n // 3).astype(dtype), rng.integers(0, hi, size=n - n // 3).astype(dtype)]
        requiring = [rng.integers(-3, hi + 5, size=n // 2 + 3).astype(dtype), mapping[1]]
        want_u, want_r = oracle.unique_relabel(mapping, requiring)
        got_u, got_r = oracle.unique_relabel(mapping, requiring, parallel=True)
        assert np.array_equal(got_u, want_u)
        for a, b in zip(got_r, want_r):
            assert np.array_equal(a, b)
    # and through the multi-layer driver
    indptr, indices = _toy_graph(rng, 3000, 40)
    seeds = rng.integers(0, 3000, size=500).astype(np.int64)
    a = oracle.sample_blocks(seeds, indptr, indices, [5, 4, 3], False, 3, 1)
    b = oracle.sample_blocks(seeds, indptr, indices, [5, 4, 3], False, 3, 1, parallel_relabel=True)
    assert np.array_equal(a[0], b[0])
    for x, y in zip(a[2], b[2]):
        assert all(np.array_equal(p, q) for p, q in zip(x, y))


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


# ---- weighted sampling ----------------------------------------------------
def _tiled_rows(weights, trials):
    """`trials` rows that all have the same weights; neighbour ids = positions."""
    deg = len(weights)
    indptr = np.arange(0, (trials + 1) * deg, deg, dtype=np.int64)
    indices = np.tile(np.arange(deg, dtype=np.int64), trials)
    probs = np.tile(np.asarray(weights, dtype=np.float32), trials)
    return indptr, indices, probs, np.arange(trials, dtype=np.int64)


def test_neg_log_matches_libm(oracle):
    rng = np.random.default_rng(5)
    fold = int(2 ** 32 / math.sqrt(2))  # where the mantissa is folded from above sqrt(2) to below 1
    xs = [0, 1, 2, 3, 2 ** 31 - 1, 2 ** 31, 2 ** 32 - 2, 2 ** 32 - 1] + list(range(fold - 50, fold + 50))
    xs += [int(x) for x in rng.integers(0, 2 ** 32, size=20000)]
    xs += [int(x) for x in 2 ** 32 - 1 - rng.integers(0, 4096, size=2000)]  # u close to 1: heavy cancellation
    for x in xs:
        got = oracle.neg_log_u32(x)
        want = -math.log((x + 0.5) / 4294967296.0)  # the argument is exact in float64
        assert abs(got - want) <= 2 * np.spacing(want), (x, got, want)
    # monotone where neighbouring arguments straddle a power of two or the fold
    for x0 in (fold - 200, 2 ** 31 - 200, 2 ** 30 - 200):
        vals = [oracle.neg_log_u32(x) for x in range(x0, x0 + 400)]
        assert all(a >= b for a, b in zip(vals, vals[1:]))


def test_weighted_key_layout(oracle):
    seed, stream, row = 0xfeedface12345678, 11, (3 << 32) | 77
    for p, wgt in [(0, 1.0), (1, 0.25), (2, 3.5), (3, 1e-3), (4, 2.0), (1022, 7.0), (1023, 0.5)]:
        w = oracle.philox((0x80000000 | (p >> 2), stream, row & 0xffffffff, row >> 32),
                          (seed & 0xffffffff, seed >> 32))
        want = -math.log((int(w[p & 3]) + 0.5) / 4294967296.0) / float(np.float32(wgt))
        got = oracle.weighted_key(seed, stream, row, p, wgt)
        assert abs(got - want) <= 4 * np.spacing(want), (p, got, want)
    for bad in (0.0, -1.0, float("nan"), -float("inf")):
        assert oracle.weighted_key(seed, stream, row, 5, bad) == float("inf")
    assert oracle.weighted_key(seed, stream, row, 5, float("inf")) == 0.0


def test_weighted_matches_successive_sampling(oracle):
    # order of the race = order of successive draws without replacement:
    # P(a then b) = w_a / W * w_b / (W - w_a)
    weights, k, trials = [1.0, 2.0, 3.0, 4.0], 2, 120000
    indptr, indices, probs, seeds = _tiled_rows(weights, trials)
    rows, cols = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, k, False, 2024, 3)
    assert np.array_equal(rows, np.repeat(seeds, k))
    pairs = cols.reshape(trials, k)
    assert (pairs[:, 0] != pairs[:, 1]).all()
    total = sum(weights)
    chi2 = 0.0
    for a, b in itertools.permutations(range(4), 2):
        exp = trials * weights[a] / total * weights[b] / (total - weights[a])
        cnt = int(((pairs[:, 0] == a) & (pairs[:, 1] == b)).sum())
        chi2 += (cnt - exp) ** 2 / exp
    assert chi2 < 31.26  # chi-square 11 dof, p = 0.001


def test_weighted_equal_weights_give_uniform_subsets(oracle):
    deg, k, trials = 5, 3, 50000
    indptr, indices, probs, seeds = _tiled_rows([0.7] * deg, trials)
    _, cols = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, k, False, 7, 0)
    picks = np.sort(cols.reshape(trials, k), axis=1)
    assert (picks[:, 1:] != picks[:, :-1]).all()
    codes = picks[:, 0] * 25 + picks[:, 1] * 5 + picks[:, 2]
    cnt = np.array([(codes == a * 25 + b * 5 + c).sum() for a, b, c in itertools.combinations(range(deg), k)], float)
    assert cnt.sum() == trials
    exp = trials / len(cnt)
    assert ((cnt - exp) ** 2 / exp).sum() < 27.88  # chi-square 9 dof, p = 0.001


def test_weighted_non_positive_weights_lose(oracle):
    weights = [0.0, 1.0, 0.0, 2.0, -1.0, float("nan"), 0.0]
    indptr, indices, probs, seeds = _tiled_rows(weights, 500)
    _, cols = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, 2, False, 1, 1)
    assert (np.sort(cols.reshape(500, 2), axis=1) == [1, 3]).all()
    # more picks than positive weights: still num_picks picks (as upstream), the rest by position
    _, cols = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, 4, False, 1, 1)
    got = cols.reshape(500, 4)
    assert (np.sort(got[:, :2], axis=1) == [1, 3]).all() and (got[:, 2:] == [0, 2]).all()


def test_weighted_full_row_and_counts(oracle):
    rng = np.random.default_rng(8)
    deg = rng.integers(0, 9, size=60)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = rng.integers(0, 60, size=int(indptr[-1])).astype(np.int64)
    probs = rng.random(indices.size).astype(np.float32)
    seeds = rng.permutation(60).astype(np.int64)
    rows, cols = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, 8, False, 5, 5)
    assert np.array_equal(rows, np.concatenate([np.full(deg[s], s) for s in seeds]))
    assert np.array_equal(cols, np.concatenate([indices[indptr[s]:indptr[s + 1]] for s in seeds]))
    rows, _ = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, 3, True, 5, 5)
    assert np.array_equal(rows, np.concatenate([np.full(3 if deg[s] else 0, s) for s in seeds]))


def test_weighted_replace_frequencies(oracle):
    weights, k, trials = [1.0, 2.0, 0.0, 3.0, 4.0], 8, 40000
    indptr, indices, probs, seeds = _tiled_rows(weights, trials)
    _, cols = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, k, True, 99, 2)
    cnt = np.bincount(cols, minlength=5).astype(float)
    assert cnt[2] == 0
    exp = np.array(weights) / sum(weights) * trials * k
    keep = exp > 0
    assert ((cnt[keep] - exp[keep]) ** 2 / exp[keep]).sum() < 16.27  # chi-square 3 dof, p = 0.001
    # slots are independent draws: the pair (slot 0, slot 1) has product probabilities
    two = cols.reshape(trials, k)[:, :2]
    chi2 = 0.0
    for a in (0, 1, 3, 4):
        for b in (0, 1, 3, 4):
            e = trials * weights[a] * weights[b] / 100.0
            chi2 += (int(((two[:, 0] == a) & (two[:, 1] == b)).sum()) - e) ** 2 / e
    assert chi2 < 37.70  # chi-square 15 dof, p = 0.001
    # no positive weight at all: the last neighbour, as upstream's clamped search returns
    indptr, indices, probs, seeds = _tiled_rows([0.0, -2.0, 0.0], 10)
    _, cols = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, 4, True, 99, 2)
    assert (cols == 2).all()


def test_weighted_infinite_weights(oracle):
    weights = [1.0, float("inf"), 5.0, float("inf"), 2.0, float("inf")]
    indptr, indices, probs, seeds = _tiled_rows(weights, 3000)
    # without replacement: keys 0 for the infinite weights, taken first and in position order
    _, cols = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, 4, False, 6, 0)
    got = cols.reshape(3000, 4)
    assert (got[:, :3] == [1, 3, 5]).all() and np.isin(got[:, 3], [0, 2, 4]).all()
    # with replacement: only they hold a share, equally
    _, cols = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, 6, True, 6, 0)
    cnt = np.bincount(cols, minlength=6).astype(float)
    assert cnt[[0, 2, 4]].sum() == 0
    assert ((cnt[[1, 3, 5]] - 6000) ** 2 / 6000).sum() < 13.82  # chi-square 2 dof, p = 0.001


def test_weighted_replace_against_numpy_cdf(oracle):
    # quanta, inclusive sums and the upper-bound search recomputed with numpy and Python integers
    rng = np.random.default_rng(21)
    deg, k, seed, stream = 300, 70, 0x1122334455, 4
    w = (rng.random(deg) ** 4).astype(np.float32)
    w[rng.integers(0, deg, 20)] = 0.0
    shift = 32 - math.frexp(float(w.max()))[1]  # 2^(E-1) <= max w < 2^E, shares = floor(w * 2^(32-E))
    q = np.floor(np.ldexp(w.astype(np.float64), shift)).astype(np.uint64)
    assert 2 ** 31 <= int(q.max()) < 2 ** 32
    assert [oracle.weight_quantum(float(x), float(w.max())) for x in w[:50]] == [int(x) for x in q[:50]]
    cdf = np.cumsum(q)
    total = int(cdf[-1])
    indptr = np.array([0, 0, 0, deg], dtype=np.int64)  # the sampled row is id 2
    _, cols = oracle.sample_neighbors_weighted(np.array([2]), indptr, np.arange(deg, dtype=np.int64), w, k,
                                               True, seed, stream)
    want = []
    for j in range(k):
        wd = [int(x) for x in oracle.philox((0x40000000 | j, stream, 2, 0), (seed & 0xffffffff, seed >> 32))]
        x = wd[0] | (wd[1] << 32)
        lo = (x * total) & (2 ** 64 - 1)
        if lo < total and lo < (2 ** 64 - total) % total:
            x = wd[2] | (wd[3] << 32)
        r = (x * total) >> 64
        want.append(int(np.searchsorted(cdf, np.uint64(r), side="right")))
    assert list(cols) == want


def test_bounded64_rejection_rule(oracle):
    n = 2 ** 63 + 1  # 2^64 mod n = 2^63 - 1: x = 2 gives lo = 2 < threshold -> rejected
    assert oracle.bounded64((2, 0, 0, 0x80000000), n) == ((0x80000000 << 32) * n) >> 64
    assert oracle.bounded64((1, 0, 9, 9), n) == 0          # lo = n >= n: accepted at once
    assert oracle.bounded64((0, 0x80000000, 9, 9), 3) == 1  # x = 2^63: lo = 2^63 >= 3
    assert oracle.bounded64((0, 0, 5, 0), 3) == 0           # x = 0: lo = 0 < 2^64 mod 3 = 1 -> second pair
    rng = np.random.default_rng(2)
    cnt = np.zeros(7)
    for _ in range(7000):
        cnt[oracle.bounded64([int(x) for x in rng.integers(0, 2 ** 32, 4)], 7)] += 1
    assert ((cnt - 1000) ** 2 / 1000).sum() < 22.46  # chi-square 6 dof, p = 0.001


# ---- placement ------------------------------------------------------------
def test_renumber_is_an_isomorphism(oracle):
    rng = np.random.default_rng(12)
    deg = rng.integers(0, 12, size=200)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = rng.integers(0, 200, size=int(indptr[-1])).astype(np.int64)
    order = oracle.degree_order(indptr)
    new_deg = deg[order]
    assert (new_deg[:-1] >= new_deg[1:]).all()                       # hottest first
    same = new_deg[:-1] == new_deg[1:]
    assert (order[:-1][same] < order[1:][same]).all()                # ties keep the old order
    new_indptr, new_indices, rank = oracle.renumber_csc(indptr, indices, order)
    assert np.array_equal(rank[order], np.arange(200)) and np.array_equal(np.diff(new_indptr), new_deg)
    # edge (u -> v) exists, at the same place in v's list, iff (rank[u] -> rank[v]) does
    for v in range(200):
        r = rank[v]
        assert np.array_equal(order[new_indices[new_indptr[r]:new_indptr[r + 1]]],
                              indices[indptr[v]:indptr[v + 1]])
    # renumbering back with the inverse permutation restores the graph
    back_indptr, back_indices, _ = oracle.renumber_csc(new_indptr, new_indices, rank.astype(np.int64))
    assert np.array_equal(back_indptr, indptr) and np.array_equal(back_indices, indices)
