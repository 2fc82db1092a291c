"""GPU parity of weighted row-wise sampling against the CPU oracle.  The picks are bit-exact:
race keys are float64 values built from exactly rounded operations on both sides, and the
with-replacement rule works on integer quanta."""
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


def _weights(rng, n):
    """Spread over many binades, with zeros, negatives, NaN and exact ties."""
    w = (rng.random(n) ** 6 * 100.0).astype(np.float32)
    w[rng.random(n) < 0.05] = 0.0
    w[rng.random(n) < 0.01] = -1.0
    w[rng.random(n) < 0.005] = np.nan
    ties = rng.random(n) < 0.2
    w[ties] = np.float32(0.5)
    return w


@pytest.fixture(scope="module")
def graph():
    rng = np.random.default_rng(17)
    indptr, indices = powerlaw_graph(rng, 20000, 20, 6000)
    return indptr, indices, _weights(rng, indices.size)


@pytest.mark.parametrize("k,replace", [(1, False), (5, False), (15, False), (32, False), (33, False), (63, False),
                                       (64, False), (1, True), (10, True), (64, True), (65, True), (150, True)])
def test_weighted_parity_c_abi(pkg, oracle, graph, k, replace):
    capi = pkg.capi
    indptr, indices, probs = graph
    rng = np.random.default_rng(100 + k)
    seeds = rng.integers(0, 20000, size=3001).astype(np.int64)
    want_r, want_c = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, k, replace, 0x5eed5eed77, 6)
    ip, ix, pr = _dev(indptr), _dev(indices), _dev(probs)
    for two_step in (False, True):
        r, c, flags = capi.sample_neighbors_weighted(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix),
                                                     capi.tensor_view(pr), k, replace, 0x5eed5eed77, 6,
                                                     two_step=two_step)
        assert flags == 0
        assert np.array_equal(_np(r), want_r), (k, replace, two_step)
        assert np.array_equal(_np(c), want_c), (k, replace, two_step)


def test_weighted_row_lengths_around_the_wave_width(pkg, oracle):
    # degrees 0..200 and a few long rows: every residue of the 64-wide passes, the first-chunk
    # sort with padding lanes, the insertion path, and rows shorter than num_picks
    capi = pkg.capi
    rng = np.random.default_rng(4)
    deg = np.concatenate([np.arange(0, 201), [255, 256, 257, 1023, 1024, 1025, 5000, 20000]])
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = rng.integers(0, deg.size, size=int(indptr[-1])).astype(np.int64)
    probs = rng.random(indices.size).astype(np.float32)
    probs[indptr[150]:indptr[151]] = 0.0   # a row without any positive weight
    probs[indptr[160]:indptr[161]] = 2.0   # a row of ties: positions decide
    probs[indptr[-2]:indptr[-2] + 19000] = 0.0  # a long row with few positive weights
    for row in (170, 190, 205, 207):                # infinite weights: race keys tie at 0, positions decide;
        probs[indptr[row]:indptr[row + 1]:3] = np.inf  # with replacement only they hold a share
    seeds = np.arange(deg.size, dtype=np.int64)
    ip, ix, pr = _dev(indptr), _dev(indices), _dev(probs)
    for k, replace in [(7, False), (64, False), (7, True), (100, True)]:
        want_r, want_c = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, k, replace, 31, 1)
        r, c, _ = capi.sample_neighbors_weighted(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix),
                                                 capi.tensor_view(pr), k, replace, 31, 1)
        assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c), (k, replace)


@pytest.mark.parametrize("group", ["16", "32", "64"])
def test_weighted_every_group_width(pkg, oracle, graph, group, request):
    # the library picks the lanes-per-row from num_picks; the hook forces each width (and with it
    # each long-row threshold) over the same inputs
    capi = pkg.capi
    capi.check(capi.lib.dgs_debug_set(capi.DEBUG_WEIGHTED_GROUP, int(group)))
    request.addfinalizer(lambda: capi.lib.dgs_debug_set(capi.DEBUG_WEIGHTED_GROUP, 0))
    indptr, indices, probs = graph
    rng = np.random.default_rng(int(group))
    seeds = rng.integers(0, 20000, size=4000).astype(np.int64)
    ip, ix, pr = _dev(indptr), _dev(indices), _dev(probs)
    for k, replace in [(3, False), (12, False), (16, False), (5, True), (40, True)]:
        want_r, want_c = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, k, replace, 77, 9)
        r, c, _ = capi.sample_neighbors_weighted(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix),
                                                 capi.tensor_view(pr), k, replace, 77, 9)
        assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c), (group, k, replace)


@pytest.mark.parametrize("id_dtype,ptr_dtype", [(np.int32, np.int32), (np.int32, np.int64), (np.int64, np.int32)])
def test_weighted_mixed_widths(pkg, oracle, id_dtype, ptr_dtype):
    capi = pkg.capi
    rng = np.random.default_rng(3)
    indptr, indices = powerlaw_graph(rng, 5000, 15, 500, id_dtype=id_dtype, ptr_dtype=ptr_dtype)
    probs = _weights(rng, indices.size)
    seeds = rng.integers(0, 5000, size=1500).astype(id_dtype)
    ip, ix, pr = _dev(indptr), _dev(indices), _dev(probs)
    for k, replace in [(10, False), (7, True)]:
        want_r, want_c = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, k, replace, 42, 1)
        r, c, _ = capi.sample_neighbors_weighted(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix),
                                                 capi.tensor_view(pr), k, replace, 42, 1)
        assert r.dtype == _dev(seeds).dtype
        assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c)


def test_weighted_operators_and_tiers(pkg, oracle, graph):
    indptr, indices, probs = graph
    rng = np.random.default_rng(8)
    seeds = rng.permutation(20000)[:2048].astype(np.int64)
    # all three arrays split across HBM and host memory
    ip_ct = pkg.ChunkTensor([indptr.size], torch.int64, 8 * 7001)
    ip_ct._CAPI_load_from_tensor(torch.from_numpy(indptr))
    ix_ct = pkg.ChunkTensor([indices.size], torch.int64, 8 * (indices.size // 3))
    ix_ct._CAPI_load_from_tensor(torch.from_numpy(indices))
    pr_ct = pkg.ChunkTensor([probs.size], torch.float32, 4 * (probs.size // 2))
    pr_ct._CAPI_load_from_tensor(torch.from_numpy(probs))
    for k, replace in [(10, False), (10, True)]:
        pkg.set_rng_state(777, 2)
        r, c = pkg.ops._CAPI_sample_neighbors_with_probs_with_chunk_tensor(_dev(seeds), ip_ct, ix_ct, pr_ct, k,
                                                                           replace)
        want_r, want_c = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, k, replace, 777, 2)
        assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c)
        assert pkg.ops._CAPI_get_rng_state() == [777, 3]
        pkg.set_rng_state(777, 2)
        r, c = pkg.ops._CAPI_sample_neighbors_with_probs(_dev(seeds), _dev(indptr), _dev(indices), _dev(probs), k,
                                                         replace)
        assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c)


def test_weighted_argument_errors(pkg, graph):
    indptr, indices, probs = graph
    seeds = _dev(np.arange(10, dtype=np.int64))
    ops = pkg.ops
    with pytest.raises(RuntimeError, match="num_picks <= 64"):
        ops._CAPI_sample_neighbors_with_probs(seeds, _dev(indptr), _dev(indices), _dev(probs), 65, False)
    with pytest.raises(RuntimeError, match="float32"):
        ops._CAPI_sample_neighbors_with_probs(seeds, _dev(indptr), _dev(indices), _dev(probs.astype(np.float64)), 5,
                                              False)
    with pytest.raises(RuntimeError, match="weights for"):
        ops._CAPI_sample_neighbors_with_probs(seeds, _dev(indptr), _dev(indices), _dev(probs[:-1]), 5, False)
    r, c = ops._CAPI_sample_neighbors_with_probs(seeds[:0], _dev(indptr), _dev(indices), _dev(probs), 5, False)
    assert r.numel() == 0 and c.numel() == 0


def test_weighted_inclusion_frequencies(pkg):
    # 20000 rows with the same 40 weights, k = 1: P(position i) = w_i / W exactly
    rng = np.random.default_rng(9)
    deg, trials = 80, 20000
    w = (rng.random(deg) + 0.05).astype(np.float32)
    indptr = np.arange(0, (trials + 1) * deg, deg, dtype=np.int64)
    indices = np.tile(np.arange(deg, dtype=np.int64), trials)
    probs = np.tile(w, trials)
    seeds = _dev(np.arange(trials, dtype=np.int64))
    exp = w.astype(np.float64) / w.astype(np.float64).sum() * trials
    for replace in (False, True):
        pkg.set_rng_state(12, 0)
        _, c = pkg.ops._CAPI_sample_neighbors_with_probs(seeds, _dev(indptr), _dev(indices), _dev(probs), 1, replace)
        cnt = np.bincount(_np(c), minlength=deg).astype(float)
        assert ((cnt - exp) ** 2 / exp).sum() < 124.8  # chi-square 79 dof, p = 0.001


@pytest.mark.parametrize("replace", [False, True])
def test_weighted_sampler_loop(pkg, oracle, graph, replace, last_hop):
    # ChunkTensorSampler with chunk_probs: the upstream loop with weighted picks in every hop, through
    # the fused driver (default), the per-hop operators, and with batches in flight on two streams
    indptr, indices, probs = graph
    rng = np.random.default_rng(2)
    big = 1 << 40
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, big)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, big, cache_rate=0.5)
    pr_ct = pkg.create_chunktensor(torch.from_numpy(probs), 1, big, cache_rate=0.3)
    feats = rng.standard_normal((20000, 12)).astype(np.float32)
    x_ct = pkg.create_chunktensor(torch.from_numpy(feats), 1, big)
    fanouts = [6, 4, 3]
    batches = [rng.permutation(20000)[:512].astype(np.int64) for _ in range(4)]
    batches.append(np.array([5, 5, 7, 5], dtype=np.int64))      # repeated seeds
    batches.append(np.empty(0, dtype=np.int64))

    def check(got, want_f, want_blocks):
        assert np.array_equal(_np(got[0]), want_f)
        assert len(got[2]) == 3
        for g, w in zip(got[2], want_blocks):
            assert np.array_equal(_np(g.src_local), w[0]) and np.array_equal(_np(g.dst_local), w[1])
            assert (g.num_src, g.num_dst) == (w[2], w[3])

    for fused in (True, False):
        sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, pr_ct, replace, fused=fused)
        assert sampler.fused == fused
        pkg.set_rng_state(31337, 10)
        for i, b in enumerate(batches):
            want_f, _, want_blocks = oracle.sample_blocks(b, indptr, indices, fanouts, replace, 31337, 10 + 3 * i,
                                                          probs=probs)
            got = sampler.sample_blocks_and_index(None, torch.from_numpy(b), x_ct)
            check(got, want_f, want_blocks)
            assert np.array_equal(_np(got[3]), feats[want_f])
    # in flight
    sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, pr_ct, replace)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    pkg.set_rng_state(31337, 10)
    pending = []
    for i, b in enumerate(batches):
        with torch.cuda.stream(streams[i % 2]):
            pending.append(sampler.submit(None, _dev(b)))
    for i in reversed(range(len(batches))):
        want_f, _, want_blocks = oracle.sample_blocks(batches[i], indptr, indices, fanouts, replace, 31337, 10 + 3 * i,
                                                      probs=probs)
        check(pending[i].result(), want_f, want_blocks)
    torch.cuda.synchronize()


def test_weighted_fused_long_rows_and_wide_fanout(pkg, oracle, last_hop):
    # rows longer than a wave's share (block-per-row launch inside the fused driver), fanout 64,
    # rows without positive weights, int32 ids with int64 offsets
    rng = np.random.default_rng(6)
    deg = np.concatenate([rng.integers(0, 90, size=3000), [2049, 4100, 9000, 30000, 2048, 0, 1]])
    rng.shuffle(deg)
    n = deg.size
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = rng.integers(0, n, size=int(indptr[-1])).astype(np.int32)
    probs = (rng.random(indices.size) ** 3).astype(np.float32)
    probs[indptr[10]:indptr[11]] = 0.0
    big = 1 << 40
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, big)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, big)
    pr_ct = pkg.create_chunktensor(torch.from_numpy(probs), 1, big)
    long_rows = np.flatnonzero(deg > 2000).astype(np.int32)
    seeds = np.concatenate([long_rows, rng.integers(0, n, size=400).astype(np.int32)])
    for fanouts, replace in [([64, 5], False), ([3, 64], True), ([20], False), ([20], True)]:
        pkg.set_rng_state(99, 0)
        sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, pr_ct, replace)
        assert sampler.fused
        f, _, blocks = sampler.sample_blocks(None, torch.from_numpy(seeds))
        want_f, _, want_blocks = oracle.sample_blocks(seeds, indptr, indices, fanouts, replace, 99, 0, probs=probs)
        assert np.array_equal(_np(f), want_f), (fanouts, replace)
        for g, w in zip(blocks, want_blocks):
            assert np.array_equal(_np(g.src_local), w[0]) and np.array_equal(_np(g.dst_local), w[1])


def test_weighted_rows_that_the_key_halves_leave_open(pkg, oracle, last_hop):
    # the race first compares the upper 32 bits of the keys and repeats a row on full keys when
    # those tie where it matters: infinite weights (all keys 0), fewer usable weights than picks
    # (the unusable ones tie), on rows served by a lane group, by a wave and by a whole block;
    # plus ordinary rows sharing their waves with such rows
    rng = np.random.default_rng(12)
    deg = np.array([40, 300, 1500, 2500, 6000, 18000] * 3 + [30, 50, 64, 65, 200, 33, 17, 90])
    n = deg.size
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = rng.integers(0, n, size=int(indptr[-1])).astype(np.int64)
    probs = (rng.random(indices.size) + 0.01).astype(np.float32)
    for row in range(0, 6):          # every third weight infinite
        probs[indptr[row]:indptr[row + 1]:3] = np.inf
    for row in range(6, 12):         # three usable weights near the end of the row
        probs[indptr[row]:indptr[row + 1]] = 0.0
        probs[indptr[row + 1] - 9:indptr[row + 1]:3] = 1.5
    for row in range(12, 18):        # usable weights only in the first 64 positions, fewer than some fanouts
        probs[indptr[row] + 20:indptr[row + 1]] = np.nan
    seeds = rng.permutation(n).astype(np.int64)
    capi = pkg.capi
    ip, ix, pr = _dev(indptr), _dev(indices), _dev(probs)
    for k in (2, 7, 16, 31, 64):
        want_r, want_c = oracle.sample_neighbors_weighted(seeds, indptr, indices, probs, k, False, 5, 2)
        r, c, _ = capi.sample_neighbors_weighted(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix),
                                                 capi.tensor_view(pr), k, False, 5, 2)
        assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c), k
    big = 1 << 40
    cts = [pkg.create_chunktensor(torch.from_numpy(a), 1, big) for a in (indptr, indices, probs)]
    for fanouts in ([7, 3], [33], [16, 2]):
        pkg.set_rng_state(1234, 3)
        sampler = pkg.ChunkTensorSampler(fanouts, cts[0], cts[1], cts[2], False)
        f, _, blocks = sampler.sample_blocks(None, torch.from_numpy(seeds))
        want_f, _, want_blocks = oracle.sample_blocks(seeds, indptr, indices, fanouts, False, 1234, 3, probs=probs)
        assert np.array_equal(_np(f), want_f), fanouts
        for g, w in zip(blocks, want_blocks):
            assert np.array_equal(_np(g.src_local), w[0]) and np.array_equal(_np(g.dst_local), w[1])


def test_weighted_fused_on_more_streams_than_node_tables(pkg, oracle, graph, last_hop):
    # a graph keeps at most four node tables, one per stream; a fifth and sixth stream take over a
    # table whose stream is idle, or run on a hash table in their workspace: same batches either way
    indptr, indices, probs = graph
    big = 1 << 40
    cts = [pkg.create_chunktensor(torch.from_numpy(a), 1, big) for a in (indptr, indices, probs)]
    sampler = pkg.ChunkTensorSampler([5, 3], *cts)
    rng = np.random.default_rng(9)
    streams = [torch.cuda.Stream() for _ in range(6)]
    batches = [rng.integers(0, 20000, size=400).astype(np.int64) for _ in range(14)]
    pkg.set_rng_state(555, 0)
    pending = []
    for i, b in enumerate(batches):
        with torch.cuda.stream(streams[(i * 5) % 6]):
            pending.append(sampler.submit(None, _dev(b)))
    for i, b in enumerate(batches):
        want_f, _, want_blocks = oracle.sample_blocks(b, indptr, indices, [5, 3], False, 555, 2 * i, probs=probs)
        f, _, blocks = pending[i].result()
        assert np.array_equal(_np(f), want_f), i
        for g, w in zip(blocks, want_blocks):
            assert np.array_equal(_np(g.src_local), w[0]) and np.array_equal(_np(g.dst_local), w[1])
    torch.cuda.synchronize()


@pytest.mark.parametrize("id_dtype", [np.int64, np.int32])
def test_weighted_fused_c_abi_on_every_table_kind(pkg, oracle, graph, id_dtype, last_hop):
    # the weighted multi-hop driver through the C ABI: hash table in the workspace (packed slots,
    # then id + value arrays), then the persistent node table; every hop picks by weight
    capi = pkg.capi
    indptr, indices, probs = graph
    ix = indices.astype(id_dtype)
    ip_t, ix_t, pr_t = _dev(indptr), _dev(ix), _dev(probs)
    rng = np.random.default_rng(21)
    seeds = rng.integers(0, 20000, size=700).astype(id_dtype)
    n_nodes = indptr.size - 1
    node_table = torch.full((capi.lib.dgs_node_table_bytes(n_nodes) // 8,), -1, dtype=torch.int64, device="cuda")
    epoch = 0  # grows by one per call for as long as the table lives
    for fanouts, replace in (([6, 4], False), ([9, 3], True)):
        want_f, _, want_blocks = oracle.sample_blocks(seeds, indptr, ix, fanouts, replace, 77, 3, probs=probs)
        hop_fanouts = list(reversed(fanouts))
        for mode in ("packed", "split", "direct", "direct"):
            capi.check(capi.lib.dgs_debug_set(capi.DEBUG_FORCE_SPLIT_TABLE, int(mode == "split")))
            kw = {}
            if mode == "direct":
                epoch += 1
                kw = dict(node_table=node_table, epoch=epoch)
            try:
                hops, _, flags = capi.sample_blocks(_dev(seeds), capi.tensor_view(ip_t), capi.tensor_view(ix_t),
                                                    hop_fanouts, replace, 77, 3, probs_view=capi.tensor_view(pr_t), **kw)
            finally:
                capi.check(capi.lib.dgs_debug_set(capi.DEBUG_FORCE_SPLIT_TABLE, 0))
            assert list(flags) == [0] * len(fanouts)
            assert np.array_equal(_np(hops[-1][0]), want_f), mode
            for (f, s, d), w in zip(hops, reversed(want_blocks)):
                assert np.array_equal(_np(s), w[0]) and np.array_equal(_np(d), w[1]), mode
