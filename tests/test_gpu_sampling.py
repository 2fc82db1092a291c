"""GPU parity of row-wise sampling and unique/relabel against the CPU oracle.
Everything is bit-exact: full-fanout rows by construction, fanout < degree rows
because kernel and oracle implement the same Philox/Floyd contract."""
import numpy as np
import pytest
import torch

from helpers import load_pkg, np_unique_first, powerlaw_graph, LAST_HOP_MODES, set_last_hop_mode

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


@pytest.fixture(scope="module")
def graph():
    rng = np.random.default_rng(11)
    return powerlaw_graph(rng, 20000, 20, 3000)


@pytest.mark.parametrize("k,replace", [(1, False), (5, False), (8, False), (10, False), (15, False), (16, False),
                                       (25, False), (50, False), (64, False), (65, False), (200, False),
                                       (3, True), (15, True), (50, True), (64, True), (100, True)])
def test_sample_parity_c_abi(pkg, oracle, graph, k, replace):
    capi = pkg.capi
    indptr, indices = graph
    rng = np.random.default_rng(k * 7 + int(replace))
    seeds = rng.integers(0, 20000, size=3001).astype(np.int64)
    want_r, want_c = oracle.sample_neighbors(seeds, indptr, indices, k, replace, 0xABCDEF0123, 9)
    ip, ix = _dev(indptr), _dev(indices)
    for two_step in (False, True, "mirrored"):  # "mirrored": the length through polled pinned words
        r, c, flags = capi.sample_neighbors(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix), k, replace,
                                            0xABCDEF0123, 9, two_step=two_step)
        assert flags == 0
        assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c), (k, replace, two_step)


@pytest.mark.parametrize("id_dtype,ptr_dtype", [(np.int32, np.int32), (np.int32, np.int64), (np.int64, np.int32)])
def test_sample_mixed_widths(pkg, oracle, id_dtype, ptr_dtype):
    capi = pkg.capi
    rng = np.random.default_rng(3)
    indptr, indices = powerlaw_graph(rng, 5000, 15, 500, id_dtype=id_dtype, ptr_dtype=ptr_dtype)
    seeds = rng.integers(0, 5000, size=1500).astype(id_dtype)
    ip, ix = _dev(indptr), _dev(indices)
    for k, replace in [(10, False), (7, True), (70, False)]:
        want_r, want_c = oracle.sample_neighbors(seeds, indptr, indices, k, replace, 42, 1)
        r, c, _ = capi.sample_neighbors(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix), k, replace, 42, 1)
        assert r.dtype == _dev(seeds).dtype
        assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c)


def test_sample_edge_cases(pkg, oracle):
    capi = pkg.capi
    # rows: empty, degree 1, degree == k, degree k+1, large
    deg = np.array([0, 1, 5, 6, 0, 300, 5, 0], dtype=np.int64)
    indptr = np.zeros(9, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    indices = np.arange(indptr[-1], dtype=np.int64) * 3 + 1
    ip, ix = _dev(indptr), _dev(indices)
    seeds = np.array([7, 0, 3, 3, 5, 2, 1, 4, 6], dtype=np.int64)  # duplicates allowed
    for k, replace in [(5, False), (5, True), (0, False), (1000, False)]:
        want_r, want_c = oracle.sample_neighbors(seeds, indptr, indices, k, replace, 1, 2)
        r, c, flags = capi.sample_neighbors(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix), k, replace, 1, 2)
        assert flags == 0 and np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c)
    # no seeds at all
    r, c, flags = capi.sample_neighbors(_dev(seeds[:0]), capi.tensor_view(ip), capi.tensor_view(ix), 5, False, 1, 2)
    assert r.numel() == 0 and c.numel() == 0 and flags == 0
    r, c, flags = capi.sample_neighbors(_dev(np.array([5], dtype=np.int64)), capi.tensor_view(ip),
                                        capi.tensor_view(ix), 3000, False, 1, 2, two_step=True)
    assert flags == 0 and r.numel() == 300  # deg 300 <= k: plain copy


@pytest.mark.parametrize("id_dtype", [np.int64, np.int32])
def test_sample_any_fanout_without_replacement(pkg, oracle, id_dtype):
    # fanouts above what fits the on-chip kept set, on rows that need sampling (upstream's
    # reservoir kernel takes any num_picks, src/cuda/rowwise_sampling.cu:42-99)
    capi = pkg.capi
    deg = np.array([5000, 10, 3001, 3000, 0, 2999, 9000, 2050], dtype=np.int64)
    indptr = np.zeros(deg.size + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    rng = np.random.default_rng(12)
    indices = rng.integers(0, 10 ** 6, size=int(indptr[-1])).astype(id_dtype)
    ip, ix = _dev(indptr), _dev(indices)
    seeds = np.array([0, 2, 1, 6, 3, 4, 5, 7, 0], dtype=id_dtype)
    for k in (3000, 2049, 4500):
        want_r, want_c = oracle.sample_neighbors(seeds, indptr, indices, k, False, 0xC0FFEE, 3)
        for two_step in (False, True):
            r, c, flags = capi.sample_neighbors(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix), k, False,
                                                0xC0FFEE, 3, two_step=two_step)
            assert flags == 0
            assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c), (k, two_step)
        # picks of a sampled row are distinct positions: the row's ids are distinct with high probability,
        # so check through positions recovered from a row whose neighbour ids are its positions
    ix2 = _dev(np.concatenate([np.arange(d) for d in deg]).astype(id_dtype))
    r, c, _ = capi.sample_neighbors(_dev(seeds[:1]), capi.tensor_view(ip), capi.tensor_view(ix2), 3000, False, 9, 9)
    got = _np(c)
    assert got.size == 3000 and np.unique(got).size == 3000 and got.min() >= 0 and got.max() < 5000
    r, c = pkg.ops._CAPI_sample_neighbors(_dev(seeds), ip, _dev(indices), 3000, False)
    assert r.numel() == sum(min(int(deg[s]), 3000) for s in seeds)


def test_seed_ids_outside_the_graph_are_refused(pkg, oracle, graph, last_hop):
    # a seed id is checked before it addresses indptr: its row emits nothing, the call is flagged,
    # the operators raise
    capi = pkg.capi
    indptr, indices = graph
    n = indptr.size - 1
    ip, ix = _dev(indptr), _dev(indices)
    good = np.array([5, 17, n - 1, 0], dtype=np.int64)
    for bad_id in (-1, n, n + 12345, 2 ** 40, -2 ** 50):
        seeds = np.concatenate([good[:2], [bad_id], good[2:]]).astype(np.int64)
        want_r, want_c = oracle.sample_neighbors(good, indptr, indices, 6, False, 3, 1)
        r, c, flags = capi.sample_neighbors(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix), 6, False, 3, 1)
        assert flags == 2
        assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c)  # the other rows are as ever
        with pytest.raises(RuntimeError, match="seed id"):
            pkg.ops._CAPI_sample_neighbors(_dev(seeds), ip, ix, 6, False)
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, 1 << 40)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
    probs = pkg.create_chunktensor(torch.rand(indices.size) + 0.1, 1, 1 << 40)
    for sampler in (pkg.ChunkTensorSampler([4, 3], ip_ct, ix_ct), pkg.ChunkTensorSampler([4, 3], ip_ct, ix_ct, fused=False),
                    pkg.ChunkTensorSampler([4, 3], ip_ct, ix_ct, probs)):
        for bad_id in (-1, n, 2 ** 33):
            seeds = torch.tensor([3, bad_id, 9])
            with pytest.raises(RuntimeError, match="seed id"):
                sampler.sample_blocks(None, seeds)
        f, _, _ = sampler.sample_blocks(None, torch.tensor([3, 9]))  # and the sampler still works
        assert f[:2].tolist() == [3, 9]
    # int32 ids; hash-table path of the C ABI (no node table)
    seeds32 = _dev(np.array([1, -5, 2], dtype=np.int32))
    ix32 = _dev(indices.astype(np.int32))
    hops, _, flags = capi.sample_blocks(seeds32, capi.tensor_view(ip), capi.tensor_view(ix32), [3, 2], False, 1, 0)
    assert flags[0] == 2 and flags[1] == 0


def test_neighbour_ids_outside_the_graph_are_refused(pkg, last_hop):
    # a graph whose edge array holds an id that is no node: with the direct node table the id would
    # address the table, so it is checked first and the call raises
    n = 1000
    rng = np.random.default_rng(4)
    deg = rng.integers(1, 9, size=n)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    for bad_id in (n, -1, 2 ** 35, -7):
        indices = rng.integers(0, n, size=int(indptr[-1])).astype(np.int64)
        indices[indptr[10]] = bad_id  # first neighbour of node 10
        ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, 1 << 40)
        ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
        sampler = pkg.ChunkTensorSampler([8, 8], ip_ct, ix_ct)
        with pytest.raises(RuntimeError, match="neighbour id"):
            sampler.sample_blocks(None, torch.tensor([10, 11]))
    # degree and offset checks: an indptr entry pointing past the edge array
    bad_ptr = indptr.copy()
    bad_ptr[21:] += 10 ** 9
    ip_ct = pkg.create_chunktensor(torch.from_numpy(bad_ptr), 1, 1 << 40)
    with pytest.raises(RuntimeError, match="offsets outside"):
        pkg.ChunkTensorSampler([8], ip_ct, ix_ct).sample_blocks(None, torch.tensor([30]))
    # the per-hop operators refuse such a row as well, before their fill reads through the offsets:
    # stores, plain tensors, weighted picks, any fanout (group, wave and global fills)
    seeds = torch.tensor([5, 30, 7]).cuda()
    d_ptr, d_ix = torch.from_numpy(bad_ptr).cuda(), torch.from_numpy(indices).cuda()
    d_w = torch.rand(indices.size, device="cuda")
    for k in (8, 100, 3000):
        for replace in (False, True):
            with pytest.raises(RuntimeError, match="offsets outside"):
                pkg.ChunkTensorSampler([k], ip_ct, ix_ct, replace=replace, fused=False).sample_blocks(None, seeds)
            with pytest.raises(RuntimeError, match="offsets outside"):
                pkg.ops._CAPI_sample_neighbors(seeds, d_ptr, d_ix, k, replace)
    with pytest.raises(RuntimeError, match="offsets outside"):
        pkg.ops._CAPI_sample_neighbors_with_probs(seeds, d_ptr, d_ix, d_w, 8, False)
    # a row that ends exactly at the end of the edge array is fine
    last = torch.tensor([n - 1]).cuda()
    rows, cols = pkg.ops._CAPI_sample_neighbors(last, torch.from_numpy(indptr).cuda(), d_ix, 100, False)
    assert cols.cpu().numpy().tolist() == indices[indptr[n - 1]:].tolist()
    torch.cuda.synchronize()


def test_capped_feature_buffer_gives_the_same_batch(pkg, oracle, graph, last_hop):
    # when the worst-case feature buffer exceeds the cap the gather goes into the largest buffer the
    # cap allows, and a frontier that does not fit even that is gathered once its size is known,
    # into exactly that many rows
    indptr, indices = graph
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, 1 << 40)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
    feats = torch.randn((20000, 48))
    ft = pkg.create_chunktensor(feats, 1, 1 << 40, cache_rate=0.4)
    rng = np.random.default_rng(19)
    seeds = torch.from_numpy(rng.integers(0, 20000, size=600))
    sampler = pkg.ChunkTensorSampler([9, 6], ip_ct, ix_ct)
    default_cap = pkg.ops._CAPI_get_gather_buffer_cap()
    assert default_cap == 2 << 30
    results = []
    try:
        for cap in (default_cap, 0, 600 * 7 * 10 * 48 * 4 - 1, 600 * 7 * 10 * 48 * 4, 1000 * 48 * 4):
            pkg.set_gather_buffer_cap(cap)
            pkg.set_rng_state(8, 8)
            torch.cuda.reset_peak_memory_stats()
            before = torch.cuda.memory_allocated()
            f, _, blocks, x = sampler.sample_blocks_and_index(None, seeds, ft)
            peak = torch.cuda.max_memory_allocated() - before
            results.append((f.cpu(), x.cpu(), peak, x.untyped_storage().nbytes()))
            streams = [torch.cuda.Stream(), torch.cuda.Stream()]
            got = list(pkg.BatchPipeline(sampler, ft, 2, streams=streams)([seeds, seeds.cuda(), seeds]))
            assert all(torch.equal(g[3].cpu(), feats[g[0].cpu()]) for g in got)
    finally:
        pkg.set_gather_buffer_cap(default_cap)
    o_frontier, _, _ = oracle.sample_blocks(seeds.numpy(), indptr, indices, [9, 6], False, 8, 8)
    for f, x, _, _ in results:
        assert np.array_equal(f.numpy(), o_frontier) and torch.equal(x, feats[f])
    worst = 600 * 7 * 10 * 48 * 4
    assert results[0][3] == worst and results[3][3] == worst            # ahead of the sizes: worst case
    rows = results[1][0].numel()
    assert 1000 < rows < 600 * 7 * 10 - 1
    assert results[1][3] == rows * 48 * 4 == results[4][3]  # nothing fits the cap: exactly the frontier, afterwards
    assert results[2][3] == (600 * 7 * 10 - 1) * 48 * 4      # the frontier fits what the cap allows
    assert results[1][2] < results[0][2]


def test_samplers_with_their_own_generator(pkg, oracle, graph, last_hop):
    # a sampler made with seed= draws batch b from its own streams whatever other threads do
    import threading
    indptr, indices = graph
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, 1 << 40)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
    rng = np.random.default_rng(2)
    fanouts = [5, 4]
    batches = [rng.integers(0, 20000, size=400).astype(np.int64) for _ in range(12)]
    samplers = [pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, seed=1000 + t) for t in range(3)]
    samplers.append(pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, seed=2000, fused=False))
    results = [dict() for _ in samplers]
    errors = []
    pkg.set_rng_state(555, 5)

    def work(t):
        try:
            with torch.cuda.stream(torch.cuda.Stream()):
                for i, b in enumerate(batches):
                    results[t][i] = samplers[t].sample_blocks(None, torch.from_numpy(b))
        except Exception as e:
            errors.append(e)

    threads = [threading.Thread(target=work, args=(t,)) for t in range(len(samplers))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for t, sampler in enumerate(samplers):
        for i, b in enumerate(batches):
            want_f, _, want_blocks = oracle.sample_blocks(b, indptr, indices, fanouts, False, sampler.seed, 2 * i)
            assert np.array_equal(_np(results[t][i][0]), want_f), (t, i)
            _check_blocks(results[t][i][2], want_blocks)
    assert pkg.ops._CAPI_get_rng_state() == [555, 5]  # the process-wide generator was left as it was
    # an explicit batch number names the streams
    f, _, _ = samplers[0].sample_blocks(None, torch.from_numpy(batches[3]), batch=7)
    want_f, _, _ = oracle.sample_blocks(batches[3], indptr, indices, fanouts, False, 1000, 14)
    assert np.array_equal(_np(f), want_f)


def test_node_tables_move_to_new_streams(pkg, oracle, graph):
    # streams that come and go (one per epoch, say): once four streams have sampled from a graph,
    # a new stream takes over the table of a stream that has nothing left to run
    indptr, indices = graph
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, 1 << 40)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
    sampler = pkg.ChunkTensorSampler([6, 5, 4], ip_ct, ix_ct, seed=77)
    rng = np.random.default_rng(6)
    seeds = rng.integers(0, 20000, size=500).astype(np.int64)
    want = [oracle.sample_blocks(seeds, indptr, indices, [6, 5, 4], False, 77, 3 * b)[0] for b in range(4)]
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    for epoch in range(9):
        st = torch.cuda.Stream()
        with torch.cuda.stream(st):
            for b in range(4):
                f, _, _ = sampler.sample_blocks(None, torch.from_numpy(seeds), batch=b)
                assert np.array_equal(_np(f), want[b]), (epoch, b)
        st.synchronize()
    # busy streams are left alone: batches in flight on six streams at once
    streams = [torch.cuda.Stream() for _ in range(6)]
    pending = []
    for i, st in enumerate(streams * 2):
        with torch.cuda.stream(st):
            pending.append(sampler.submit(None, _dev(seeds), batch=i % 4))
    for i, p in enumerate(pending):
        assert np.array_equal(_np(p.result()[0]), want[i % 4])
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() - base <= 4 * 8 * (indptr.size - 1) + (64 << 20)
    # a stream's owner can give its table up (before destroying the stream, say): the memory goes
    # back, and a stream that comes later gets a table of its own again
    assert ip_ct._CAPI_node_table_count() == 4
    released = 0
    for st in streams:
        released += int(ip_ct._CAPI_release_node_table(st.cuda_stream))
    assert released >= 1 and ip_ct._CAPI_node_table_count() == 4 - released
    assert not ip_ct._CAPI_release_node_table(streams[0].cuda_stream)  # gone already, or never had one
    with torch.cuda.stream(streams[0]):
        f, _, _ = sampler.sample_blocks(None, torch.from_numpy(seeds), batch=2)
        assert np.array_equal(_np(f), want[2])
        assert ip_ct._CAPI_release_node_table(0)  # 0: the current stream
    torch.cuda.synchronize()


def test_sample_with_chunk_tensor_tiers(pkg, oracle, graph):
    indptr, indices = graph
    rng = np.random.default_rng(8)
    seeds = rng.permutation(20000)[:2048].astype(np.int64)
    # both graph arrays split across HBM and host memory
    ip_ct = pkg.ChunkTensor([indptr.size], torch.int64, 8 * 7001)
    ip_ct._CAPI_load_from_tensor(torch.from_numpy(indptr))
    ix_ct = pkg.ChunkTensor([indices.size], torch.int64, 8 * (indices.size // 3))
    ix_ct._CAPI_load_from_tensor(torch.from_numpy(indices))
    for k, replace in [(10, False), (10, True)]:
        pkg.set_rng_state(555, 3)
        r, c = pkg.ops._CAPI_sample_neighbors_with_chunk_tensor(_dev(seeds), ip_ct, ix_ct, k, replace)
        want_r, want_c = oracle.sample_neighbors(seeds, indptr, indices, k, replace, 555, 3)
        assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c)
        assert pkg.ops._CAPI_get_rng_state() == [555, 4]  # one stream per call
    # plain-tensor operator
    pkg.set_rng_state(555, 3)
    r, c = pkg.ops._CAPI_sample_neighbors(_dev(seeds), _dev(indptr), _dev(indices), 10, False)
    want_r, want_c = oracle.sample_neighbors(seeds, indptr, indices, 10, False, 555, 3)
    assert np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c)


def test_sample_chi_square_uniform(pkg):
    # 4000 copies of one row of degree 40, k = 10 without replacement: each position is
    # included with probability 1/4.  Rows are keyed by their id, so copies differ.
    capi = pkg.capi
    deg, k, copies = 40, 10, 4000
    indptr = np.arange(0, (copies + 1) * deg, deg, dtype=np.int64)
    indices = np.tile(np.arange(deg, dtype=np.int64), copies)
    seeds = np.arange(copies, dtype=np.int64)
    ip, ix = _dev(indptr), _dev(indices)
    r, c, _ = capi.sample_neighbors(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix), k, False, 2024, 0)
    picks = _np(c).reshape(copies, k)
    assert all(len(set(row)) == k for row in picks[:500])
    counts = np.bincount(picks.ravel(), minlength=deg).astype(float)
    exp = copies * k / deg
    # inclusion indicators are negatively correlated; variance per cell = n p (1-p)
    z2 = ((counts - exp) ** 2 / (exp * (1 - k / deg))).sum()
    assert z2 < 72.05  # chi-square 39 dof, p = 0.001
    # with replacement: plain multinomial
    r, c, _ = capi.sample_neighbors(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix), k, True, 2024, 1)
    counts = np.bincount(_np(c), minlength=deg).astype(float)
    assert ((counts - exp) ** 2 / exp).sum() < 72.05


def _inclusion_statistic(picks, deg, k, rows):
    """Chi-square statistic of the per-position inclusion counts of `rows` uniform k-subsets of
    [0, deg) (cells are negatively correlated Bernoulli sums: scaled to deg - 1 dof)."""
    counts = np.bincount(picks.ravel(), minlength=deg).astype(float)
    p = k / deg
    exp = rows * p
    return ((counts - exp) ** 2).sum() / (exp * (1 - p)) * (deg - 1) / deg


@pytest.mark.parametrize("deg,k,rows", [(400, 100, 3000), (6000, 3000, 60), (17000, 15, 20000)])
def test_wave_and_global_fills_pick_uniform_subsets(pkg, deg, k, rows):
    # the fills for fanouts above 64 (a wave per row, Floyd's set in LDS) and above 2048 (the set in
    # the row's own output slots), and the group fill on a row of the benchmark graph's longest degree:
    # distinct positions, every position included at rate k / deg
    capi = pkg.capi
    indptr = torch.arange(0, (rows + 1) * deg, deg, dtype=torch.int64, device="cuda")
    indices = torch.arange(deg, dtype=torch.int64, device="cuda").repeat(rows)
    seeds = torch.arange(rows, dtype=torch.int64, device="cuda")
    r, c, flags = capi.sample_neighbors(seeds, capi.tensor_view(indptr), capi.tensor_view(indices), k, False, 4711, 6)
    assert flags == 0 and c.numel() == rows * k
    picks = _np(c).reshape(rows, k)
    srt = np.sort(picks, axis=1)
    assert (srt[:, 1:] != srt[:, :-1]).all() and picks.min() >= 0 and picks.max() < deg
    stat = _inclusion_statistic(picks, deg, k, rows)
    assert abs(stat - (deg - 1)) < 5 * np.sqrt(2 * (deg - 1)), stat
    # with replacement through the same fills: independent uniform draws
    r, c, flags = capi.sample_neighbors(seeds, capi.tensor_view(indptr), capi.tensor_view(indices), k, True, 4711, 7)
    counts = np.bincount(_np(c), minlength=deg).astype(float)
    exp = rows * k / deg
    stat = ((counts - exp) ** 2 / exp).sum()
    assert abs(stat - (deg - 1)) < 5 * np.sqrt(2 * (deg - 1)), stat


@pytest.mark.parametrize("replace", [False, True])
def test_fused_path_picks_uniform_subsets(pkg, last_hop, replace):
    # the fused sampler (both ways its last hop can take) on 6000 rows of degree 40 with fanout 10,
    # then one of degree 17 000 with fanout 15: what comes out as picked ids (neighbour id = position)
    # is a uniform subset, or with replacement independent draws whose repeats were folded inside
    # the wave without changing a single pick
    for deg, k, rows in ((40, 10, 6000), (17000, 15, 3000)):
        n_nodes = max(rows, deg)
        ptr = np.zeros(n_nodes + 1, dtype=np.int64)
        ptr[1: rows + 1] = np.arange(1, rows + 1) * deg
        ptr[rows + 1:] = rows * deg
        indices = np.tile(np.arange(deg, dtype=np.int64), rows)
        ip_ct = pkg.create_chunktensor(torch.from_numpy(ptr), 1, 1 << 40)
        ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
        sampler = pkg.ChunkTensorSampler([k], ip_ct, ix_ct, replace=replace, seed=99)
        frontier, _, blocks = sampler.sample_blocks(None, torch.arange(rows, dtype=torch.int64), batch=3)
        blk = blocks[0]
        picked = _np(blk.src_ids[blk.src_local])
        owner = _np(blk.dst_ids[blk.dst_local])
        assert picked.size == rows * k and np.array_equal(owner, np.repeat(np.arange(rows), k))
        picks = picked.reshape(rows, k)
        if replace:
            counts = np.bincount(picked, minlength=deg).astype(float)
            exp = rows * k / deg
            stat = ((counts - exp) ** 2 / exp).sum()
        else:
            srt = np.sort(picks, axis=1)
            assert (srt[:, 1:] != srt[:, :-1]).all()
            stat = _inclusion_statistic(picks, deg, k, rows)
        assert abs(stat - (deg - 1)) < 5 * np.sqrt(2 * (deg - 1)), (deg, k, replace, stat)


@pytest.mark.parametrize("dtype", [np.int64, np.int32])
@pytest.mark.parametrize("n,hi", [(0, 10), (1, 10), (1000, 50), (5000, 10 ** 6), (100000, 3000), (300000, 10 ** 9)])
def test_unique_relabel_parity(pkg, oracle, dtype, n, hi):
    rng = np.random.default_rng(n + hi)
    seeds = rng.permutation(min(hi, 10 ** 6))[: min(hi, 37)].astype(dtype)
    cols = rng.integers(0, hi, size=n).astype(dtype)
    rows = rng.choice(seeds, size=n).astype(dtype)
    want_u, (want_r, want_c) = oracle.unique_relabel([seeds, cols], [rows, cols])
    assert np.array_equal(want_u, np_unique_first(np.concatenate([seeds, cols])))
    for polled in (False, True):  # the counts by a copy, and through pinned words the host polls
        u, (r, c) = pkg.capi.unique_relabel([_dev(seeds), _dev(cols)], [_dev(rows), _dev(cols)], polled=polled)
        assert np.array_equal(_np(u), want_u) and np.array_equal(_np(r), want_r) and np.array_equal(_np(c), want_c)
    # operator layer, including an id that is absent from the mapping
    extra = np.array([hi + 5], dtype=dtype)
    u2, outs = pkg.ops._CAPI_tensor_relabel([_dev(seeds), _dev(cols)], [_dev(rows), _dev(cols), _dev(extra)])
    assert np.array_equal(_np(u2), want_u) and np.array_equal(_np(outs[1]), want_c)
    assert _np(outs[2]).tolist() == [-1] and outs[0].dtype == _dev(rows).dtype
    # the same device tensor on both sides, as the upstream loop passes its picked neighbours
    # (their slots are reused instead of probed again), next to a shorter view of it
    d_seeds, d_cols = _dev(seeds), _dev(cols)
    u3, outs3 = pkg.ops._CAPI_tensor_relabel([d_seeds, d_cols], [d_cols, _dev(rows), d_cols[: n // 2], d_seeds])
    assert np.array_equal(_np(u3), want_u) and np.array_equal(_np(outs3[0]), want_c)
    assert np.array_equal(_np(outs3[1]), want_r) and np.array_equal(_np(outs3[2]), want_c[: n // 2])
    assert np.array_equal(_np(outs3[3]), np.arange(seeds.size))


def test_unique_many_segments(pkg, oracle):
    rng = np.random.default_rng(12)
    parts = [rng.integers(0, 500, size=s).astype(np.int64) for s in (5, 0, 300, 1, 77, 0, 1024, 3, 9, 200)]
    want_u, want_outs = oracle.unique_relabel(parts, parts)
    u, outs = pkg.ops._CAPI_tensor_relabel([_dev(p) for p in parts], [_dev(p) for p in parts])
    assert np.array_equal(_np(u), want_u)
    for a, b in zip(outs, want_outs):
        assert np.array_equal(_np(a), b)
    u8, outs8 = pkg.capi.unique_relabel([_dev(p) for p in parts[:8]], [_dev(p) for p in parts[:8]])
    want_u8, _ = oracle.unique_relabel(parts[:8], parts[:8])
    assert np.array_equal(_np(u8), want_u8)


def test_sample_blocks_driver(pkg, oracle, graph):
    indptr, indices = graph
    ip_ct = pkg.ChunkTensor([indptr.size], torch.int64, 8 * indptr.size)
    ip_ct._CAPI_load_from_tensor(torch.from_numpy(indptr))
    ix_ct = pkg.ChunkTensor([indices.size], torch.int64, 8 * indices.size)
    ix_ct._CAPI_load_from_tensor(torch.from_numpy(indices))
    rng = np.random.default_rng(21)
    seeds = rng.permutation(20000)[:512].astype(np.int64)
    for fanouts, replace in [([15, 10, 5], False), ([4, 4], True)]:
        sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, replace=replace)
        pkg.set_rng_state(31337, 0)
        frontier, out_seeds, blocks = sampler.sample_blocks(None, torch.from_numpy(seeds))
        o_frontier, _, o_blocks = oracle.sample_blocks(seeds, indptr, indices, fanouts, replace, 31337, 0)
        assert np.array_equal(_np(frontier), o_frontier) and len(blocks) == len(o_blocks)
        for b, ob in zip(blocks, o_blocks):
            assert np.array_equal(_np(b.src_local), ob[0]) and np.array_equal(_np(b.dst_local), ob[1])
            assert (b.num_src, b.num_dst) == (ob[2], ob[3])
            assert np.array_equal(_np(b.src_ids), ob[4]) and np.array_equal(_np(b.dst_ids), ob[5])
        # then the feature gather of the final frontier
        feats = torch.randn((20000, 100))
        ft = pkg.create_chunktensor(feats, 1, 10 ** 12, cache_rate=0.5)
        x = ft._CAPI_index(frontier)
        assert torch.equal(x.cpu(), feats[frontier.cpu()])


def _check_blocks(blocks_gpu, o_blocks):
    assert len(blocks_gpu) == len(o_blocks)
    for b, ob in zip(blocks_gpu, o_blocks):
        assert np.array_equal(_np(b.src_local), ob[0]) and np.array_equal(_np(b.dst_local), ob[1])
        assert (b.num_src, b.num_dst) == (ob[2], ob[3])
        assert np.array_equal(_np(b.src_ids), ob[4]) and np.array_equal(_np(b.dst_ids), ob[5])


@pytest.mark.parametrize("id_dtype,ptr_dtype", [(np.int64, np.int64), (np.int32, np.int64), (np.int32, np.int32)])
@pytest.mark.parametrize("fanouts,replace", [([15, 10, 5], False), ([5], False), ([3, 0, 4], False), ([64, 2], False),
                                             ([7, 9], True), ([20, 15, 10], False)])
def test_fused_sample_blocks_parity(pkg, oracle, id_dtype, ptr_dtype, fanouts, replace, last_hop):
    rng = np.random.default_rng(len(fanouts) * 31 + fanouts[0])
    indptr, indices = powerlaw_graph(rng, 30000, 12, 2000, id_dtype=id_dtype, ptr_dtype=ptr_dtype)
    t_ip, t_ix = torch.from_numpy(indptr), torch.from_numpy(indices)
    ip_ct = pkg.create_chunktensor(t_ip, 1, 1 << 40)
    ix_ct = pkg.create_chunktensor(t_ix, 1, 1 << 40, cache_rate=0.6)  # part of the edges in host memory
    feats = torch.randn((30000, 36))
    ft = pkg.create_chunktensor(feats, 1, 1 << 40, cache_rate=0.3)
    seeds = rng.integers(0, 30000, size=700).astype(id_dtype)  # may hold duplicates
    fused = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, replace=replace)
    per_hop = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, replace=replace, fused=False)
    assert fused.fused and not per_hop.fused
    o_frontier, _, o_blocks = oracle.sample_blocks(seeds, indptr, indices, fanouts, replace, 2718, 40)
    for sampler in (fused, per_hop):
        pkg.set_rng_state(2718, 40)
        frontier, out_seeds, blocks = sampler.sample_blocks(None, torch.from_numpy(seeds))
        assert pkg.ops._CAPI_get_rng_state() == [2718, 40 + len(fanouts)]
        assert np.array_equal(_np(frontier), o_frontier)
        _check_blocks(blocks, o_blocks)
        pkg.set_rng_state(2718, 40)
        frontier, _, blocks, x = sampler.sample_blocks_and_index(None, torch.from_numpy(seeds), ft)
        assert np.array_equal(_np(frontier), o_frontier)
        _check_blocks(blocks, o_blocks)
        assert torch.equal(x.cpu(), feats[torch.from_numpy(o_frontier).long()])


def test_fused_sample_blocks_c_abi_and_split_table(pkg, oracle, graph, last_hop):
    capi = pkg.capi
    indptr, indices = graph
    ip, ix = _dev(indptr), _dev(indices)
    rng = np.random.default_rng(77)
    seeds = rng.permutation(20000)[:1024].astype(np.int64)
    o_frontier, _, o_blocks = oracle.sample_blocks(seeds, indptr, indices, [15, 10, 5], False, 99, 7)
    feats = torch.randn((20000, 100), device="cuda")
    n_nodes = indptr.size - 1
    node_table = torch.full((capi.lib.dgs_node_table_bytes(n_nodes) // 8,), -1, dtype=torch.int64, device="cuda")
    epoch = 0
    # hash table in the workspace (packed, then split slots), then the persistent node table twice
    for mode in ("packed", "split", "direct", "direct"):
        capi.check(capi.lib.dgs_debug_set(capi.DEBUG_FORCE_SPLIT_TABLE, int(mode == "split")))
        kw = {}
        if mode == "direct":
            epoch += 1
            kw = dict(node_table=node_table, epoch=epoch)
        hops, x, flags = capi.sample_blocks(_dev(seeds), capi.tensor_view(ip), capi.tensor_view(ix), [5, 10, 15],
                                            False, 99, 7, capi.tensor_view(feats), 100, torch.float32, **kw)
        assert flags == [0, 0, 0] and len(hops) == 3
        assert np.array_equal(_np(hops[-1][0]), o_frontier)
        for (f, s, d), ob in zip(hops, reversed(o_blocks)):
            assert np.array_equal(_np(f), ob[4]) and np.array_equal(_np(s), ob[0]) and np.array_equal(_np(d), ob[1])
        assert torch.equal(x, feats[hops[-1][0]])
    # no seeds: everything empty
    hops, x, flags = capi.sample_blocks(_dev(seeds[:0]), capi.tensor_view(ip), capi.tensor_view(ix), [5, 10], False,
                                        1, 0)
    assert all(f.numel() == 0 and s.numel() == 0 for f, s, d in hops) and flags == [0, 0]
    # fanouts above 64 are refused by the fused entry point
    fan = (capi.c_i64 * 1)(65)
    out = (capi.c_i64 * 2)()
    assert capi.lib.dgs_sample_blocks_plan(10, fan, 1, out, out) == capi.DGS_ERR_UNSUPPORTED


def test_fused_long_tile_lists(pkg, oracle, last_hop):
    # > 2048 position tiles and > 2048 row tiles in the last hop: the separate scan launches
    rng = np.random.default_rng(5)
    indptr, indices = powerlaw_graph(rng, 1_000_000, 6, 200, zero_frac=0.1)
    seeds = rng.permutation(1_000_000)[:60_000].astype(np.int64)
    fanouts = [9, 40]  # hop order: 40 first, then 9 over ~1.5M rows
    o_frontier, _, o_blocks = oracle.sample_blocks(seeds, indptr, indices, fanouts, True, 11, 0)
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, 1 << 40)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
    sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, replace=True)
    pkg.set_rng_state(11, 0)
    frontier, _, blocks = sampler.sample_blocks(None, torch.from_numpy(seeds))
    assert np.array_equal(_np(frontier), o_frontier)
    _check_blocks(blocks, o_blocks)
    # the launch plan is sized by the worst case: 60000 * 41 rows and 9 times as many positions
    assert 60_000 * 41 > 2048 * 256 and blocks[0].num_dst > 200_000


def test_host_seeds_are_accepted(pkg, oracle, graph, last_hop):
    # upstream's sampler receives host-side seed_nodes and uploads them itself
    indptr, indices = graph
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, 1 << 40)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
    feats = torch.randn((20000, 16))
    ft = pkg.create_chunktensor(feats, 1, 1 << 40)
    seeds = torch.arange(100, 612)
    sampler = pkg.ChunkTensorSampler([6, 3], ip_ct, ix_ct)
    o_frontier, _, o_blocks = oracle.sample_blocks(seeds.numpy(), indptr, indices, [6, 3], False, 5, 9)
    for s in (seeds, seeds.pin_memory(), seeds.cuda()):
        pkg.set_rng_state(5, 9)
        frontier, out_seeds, blocks, x = sampler.sample_blocks_and_index(None, s, ft)
        assert out_seeds is s and np.array_equal(_np(frontier), o_frontier)
        _check_blocks(blocks, o_blocks)
        assert blocks[-1].dst_ids.is_cuda and torch.equal(x.cpu(), feats[frontier.cpu()])


def test_batches_in_flight_on_two_streams(pkg, oracle, graph):
    # submit() on alternating streams, results collected later and out of order: every batch must
    # equal the oracle's for its own rng stream, and the synchronous call must still interleave
    indptr, indices = graph
    big = 1 << 40
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, big)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, big)
    rng = np.random.default_rng(77)
    feats = rng.standard_normal((20000, 20)).astype(np.float32)
    x_ct = pkg.create_chunktensor(torch.from_numpy(feats), 1, big, cache_rate=0.5)
    fanouts = [7, 5, 3]
    sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct)
    streams = [torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.current_stream()]
    batches = [rng.integers(0, 20000, size=700).astype(np.int64) for _ in range(9)]
    pkg.set_rng_state(4321, 50)
    pending = []
    for i, b in enumerate(batches):
        with torch.cuda.stream(streams[i % 3]):
            pending.append(sampler.submit(None, _dev(b), x_ct if i % 2 == 0 else None))
        if i == 4:  # a blocking call in the middle takes its own three rng streams
            f_sync, _, _ = sampler.sample_blocks(None, _dev(batches[0]))
    order = [8, 0, 3, 1, 7, 2, 6, 5, 4]
    results = {i: pending[i].result() for i in order}
    torch.cuda.synchronize()
    first_stream = 50
    for i, b in enumerate(batches):
        want_f, _, want_blocks = oracle.sample_blocks(b, indptr, indices, fanouts, False, 4321, first_stream)
        first_stream += 3
        got = results[i]
        assert np.array_equal(_np(got[0]), want_f), i
        for gb, wb in zip(got[2], want_blocks):
            assert np.array_equal(_np(gb.src_local), wb[0]) and np.array_equal(_np(gb.dst_local), wb[1])
        if i % 2 == 0:
            assert np.array_equal(_np(got[3]), feats[want_f])
        if i == 4:
            want_sync, _, _ = oracle.sample_blocks(batches[0], indptr, indices, fanouts, False, 4321, first_stream)
            assert np.array_equal(_np(f_sync), want_sync)
            first_stream += 3
    with pytest.raises(RuntimeError, match="already finished"):
        pending[0]._handle._CAPI_finish()
    # a fifth stream finds the table pool full and runs on the hash table: same results
    extra = [torch.cuda.Stream() for _ in range(3)]
    pkg.set_rng_state(4321, 50)
    for s_ in extra:
        with torch.cuda.stream(s_):
            f, _, _ = sampler.submit(None, _dev(batches[0])).result()
        s_.synchronize()
        want_f, _, _ = oracle.sample_blocks(batches[0], indptr, indices, fanouts, False, 4321, 50)
        assert np.array_equal(_np(f), want_f)
        pkg.set_rng_state(4321, 50)


def test_host_threads_sampling_from_one_graph_on_one_stream(pkg, oracle):
    # two host threads submit batches on the same stream: their calls share that stream's node
    # table, so the launches of one call must not be interleaved with another's.  Full
    # neighbourhoods (fanout >= every degree) make the result independent of which rng stream a
    # call happened to draw.
    import threading
    rng = np.random.default_rng(5)
    n = 4000
    deg = rng.integers(0, 7, size=n)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = rng.integers(0, n, size=int(indptr[-1])).astype(np.int64)
    big = 1 << 40
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, big)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, big)
    fanouts = [6, 6, 6]
    sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct)
    batches = [rng.integers(0, n, size=300).astype(np.int64) for _ in range(40)]
    dev_batches = [_dev(b) for b in batches]
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    results, errors = {}, []

    def work(ids):
        try:
            with torch.cuda.stream(stream):
                for i in ids:
                    results[i] = sampler.submit(None, dev_batches[i]).result()
        except Exception as e:  # surfaced below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(range(t, 40, 2),)) for t in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for i, b in enumerate(batches):
        want_f, _, want_blocks = oracle.sample_blocks(b, indptr, indices, fanouts, False, 1, 0)
        assert np.array_equal(_np(results[i][0]), want_f), i
        for gb, wb in zip(results[i][2], want_blocks):
            assert np.array_equal(_np(gb.src_local), wb[0]) and np.array_equal(_np(gb.dst_local), wb[1])


@pytest.mark.parametrize("native_loop", [True, False])
def test_batch_pipeline_hands_out_usable_batches(pkg, oracle, graph, native_loop, last_hop):
    # BatchPipeline: batches in flight on its own streams, results in submission order, usable on
    # the caller's stream at once (reduced there right away, buffers dropped while later batches
    # are still running), host and device seeds, uniform and weighted samplers; with the
    # extension's worker thread beginning the batches, and with the Python loop
    indptr, indices = graph
    big = 1 << 40
    rng = np.random.default_rng(8)
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, big)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, big)
    probs = (rng.random(indices.size) + 0.1).astype(np.float32)
    pr_ct = pkg.create_chunktensor(torch.from_numpy(probs), 1, big)
    feats = rng.standard_normal((20000, 24)).astype(np.float32)
    x_ct = pkg.create_chunktensor(torch.from_numpy(feats), 1, big, cache_rate=0.6)
    fanouts = [6, 4]
    batches = [rng.integers(0, 20000, size=900).astype(np.int64) for _ in range(11)]
    for weights, inflight in ((None, 2), (None, 3), (pr_ct, 2), (None, 1)):
        sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, weights)
        pipe = pkg.BatchPipeline(sampler, x_ct, inflight, native_loop=native_loop)
        feeds = [torch.from_numpy(b) if i % 2 else _dev(b) for i, b in enumerate(batches)]
        # an iteration that is left early leaves nothing behind, and one that starts inside another
        # gets its own batches
        for i, out in enumerate(pipe(feeds)):
            if i == 0:
                inner = [o[0].clone() for o in pipe(feeds[:3])]
                assert len(inner) == 3
            if i == 1:
                break
        pkg.set_rng_state(99, 7)
        sums, kept = [], []
        for i, (f, seeds, blocks, x) in enumerate(pipe(feeds)):
            sums.append(x.double().sum(dim=0))           # on the caller's stream, no extra wait
            kept.append((f.clone(), [(b.src_local.clone(), b.dst_local.clone()) for b in blocks]))
            assert seeds is feeds[i]
            del f, blocks, x
        torch.cuda.synchronize()
        assert len(kept) == len(batches)
        for i, b in enumerate(batches):
            want_f, _, want_blocks = oracle.sample_blocks(b, indptr, indices, fanouts, False, 99, 7 + 2 * i,
                                                          probs=None if weights is None else probs)
            assert np.array_equal(_np(kept[i][0]), want_f), (inflight, i)
            for (src, dst), wb in zip(kept[i][1], want_blocks):
                assert np.array_equal(_np(src), wb[0]) and np.array_equal(_np(dst), wb[1])
            assert np.allclose(_np(sums[i]), feats[want_f].astype(np.float64).sum(axis=0), rtol=0, atol=1e-9)
    with pytest.raises(ValueError):
        pkg.BatchPipeline(sampler, x_ct, 0)
    with pytest.raises(RuntimeError):
        list(pkg.BatchPipeline(pkg.ChunkTensorSampler([100], ip_ct, ix_ct), x_ct,
                               native_loop=native_loop)([_dev(batches[0])]))


@pytest.mark.parametrize("cap", [1, 7, 300])
def test_fused_sampler_under_a_small_grid_cap(pkg, oracle, graph, cap, request, last_hop):
    # every launch of the fused sampler loops over its blocks when there are more than the cap:
    # the results do not depend on the cap
    capi = pkg.capi
    indptr, indices = graph
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, 1 << 40)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
    probs = (np.random.default_rng(1).random(indices.size) + 0.05).astype(np.float32)
    pr_ct = pkg.create_chunktensor(torch.from_numpy(probs), 1, 1 << 40)
    feats = torch.randn((20000, 12))
    ft = pkg.create_chunktensor(feats, 1, 1 << 40)
    rng = np.random.default_rng(cap)
    seeds = rng.integers(0, 20000, size=1500).astype(np.int64)
    capi.check(capi.lib.dgs_debug_set(capi.DEBUG_SAMPLER_GRID_CAP, cap))
    request.addfinalizer(lambda: capi.lib.dgs_debug_set(capi.DEBUG_SAMPLER_GRID_CAP, 0))
    for weights, fanouts, replace in ((None, [12, 6, 3], False), (None, [20, 9], True), (probs, [5, 4], False)):
        sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, None if weights is None else pr_ct, replace=replace, seed=5)
        f, _, blocks, x = sampler.sample_blocks_and_index(None, torch.from_numpy(seeds), ft)
        want_f, _, want_blocks = oracle.sample_blocks(seeds, indptr, indices, fanouts, replace, 5, 0, probs=weights)
        assert np.array_equal(_np(f), want_f)
        _check_blocks(blocks, want_blocks)
        assert torch.equal(x.cpu(), feats[f.cpu()])


def test_unique_relabel_ids_beyond_32_bits(pkg, oracle):
    # 8-byte ids are first tried in one-word table slots; an id of 2^32 - 1 or more sends the call
    # to the two-array table.  Ids that only differ above bit 31 must not be confused, present or not.
    rng = np.random.default_rng(40)
    small = rng.integers(0, 5000, size=4000).astype(np.int64)
    for big in (2 ** 32 - 1, 2 ** 32 + 7, 2 ** 40 + 3):
        mapping = [small[:1000].copy(), np.concatenate([small[1000:], [big, 7, big + 2 ** 32]]).astype(np.int64)]
        requiring = [np.array([7, 7 + 2 ** 32, big, -1, -5, 2 ** 62, 4999, big - 2 ** 32], dtype=np.int64), mapping[1]]
        want_u, want_outs = oracle.unique_relabel(mapping, requiring)
        want_first = want_outs[0].copy()
        in_map = np.isin(requiring[0], np.concatenate(mapping))
        assert (want_first[~in_map] == -1).all()
        u, outs = pkg.capi.unique_relabel([_dev(p) for p in mapping], [_dev(p) for p in requiring])
        assert np.array_equal(_np(u), want_u)
        for a, b in zip(outs, want_outs):
            assert np.array_equal(_np(a), b)
        u, outs = pkg.ops._CAPI_tensor_relabel([_dev(p) for p in mapping], [_dev(p) for p in requiring])
        assert np.array_equal(_np(u), want_u)
        for a, b in zip(outs, want_outs):
            assert np.array_equal(_np(a), b)
    # ids that all fit: the packed attempt stands, and an id absent from the mapping that aliases a
    # present one in its low 32 bits is still absent
    mapping = [small]
    requiring = [np.array([small[0], small[0] + 2 ** 32, -1], dtype=np.int64)]
    u, outs = pkg.capi.unique_relabel([_dev(p) for p in mapping], [_dev(p) for p in requiring])
    assert _np(outs[0]).tolist() == [0, -1, -1]


@pytest.mark.parametrize("n", [3000, 70000])
def test_unique_relabel_of_a_tensor_on_both_sides_with_ids_the_table_cannot_hold(pkg, oracle, n):
    # The upstream loop passes its picked neighbours as a mapping AND as a requiring tensor (the same
    # device memory), and such a tensor is relabelled through the slot words its ids were given on
    # insertion.  An id the table in use cannot hold gets no slot: the attempt on one-word slots
    # (ids below 2^32 - 1) is void and repeated on the two-array table, and a negative id, which no
    # table holds, makes the call fail cleanly.  Above 2048 ids, so that the table lives in HBM.
    rng = np.random.default_rng(n)
    seeds = rng.permutation(5000)[:64].astype(np.int64)
    cols = rng.integers(0, 40000, size=n).astype(np.int64)
    cols[::97] += 2 ** 33                      # ids beyond the one-word slots, spread over the list
    cols[5] = cols[n - 1] = 2 ** 32 - 1        # the smallest such id, twice
    rows = rng.choice(seeds, size=n).astype(np.int64)
    want_u, (want_r, want_c) = oracle.unique_relabel([seeds, cols], [rows, cols])
    d_seeds, d_cols, d_rows = _dev(seeds), _dev(cols), _dev(rows)
    u, outs = pkg.ops._CAPI_tensor_relabel([d_seeds, d_cols], [d_rows, d_cols])
    assert np.array_equal(_np(u), want_u) and np.array_equal(_np(outs[0]), want_r) and np.array_equal(_np(outs[1]), want_c)
    u, outs = pkg.capi.unique_relabel([d_seeds, d_cols], [d_rows, d_cols])
    assert np.array_equal(_np(u), want_u) and np.array_equal(_np(outs[0]), want_r) and np.array_equal(_np(outs[1]), want_c)
    # the void attempt alone (what runs before the host has seen the overflow word): every output is
    # a rank of the list or -1, nothing else was read
    u, outs = pkg.capi.unique_relabel([d_seeds, d_cols], [d_rows, d_cols], packed_table=True, retry=False)
    got = _np(outs[1])
    assert ((got >= -1) & (got < n + 64)).all()
    # a negative id among the mapped ones: no table holds it
    bad = cols.copy()
    bad[n // 2] = -7
    d_bad = _dev(bad)
    with pytest.raises(RuntimeError, match="rejected an id"):
        pkg.ops._CAPI_tensor_relabel([d_seeds, d_bad], [d_rows, d_bad])
    torch.cuda.synchronize()
    # and the store is fine afterwards
    u, outs = pkg.ops._CAPI_tensor_relabel([d_seeds, d_cols], [d_rows, d_cols])
    assert np.array_equal(_np(u), want_u) and np.array_equal(_np(outs[1]), want_c)


def test_pipeline_streams_do_not_share_a_hardware_queue(pkg):
    # a process that has made streams before (here: six of them) still gets pipeline streams that
    # run side by side; streams that share a hardware queue would run their batches one after the other
    others = [torch.cuda.Stream() for _ in range(6)]
    chosen = pkg.pipeline_streams(3)
    assert len(chosen) == 3 and len({s.cuda_stream for s in chosen}) == 3
    assert pkg.pipeline_streams(2) == chosen[:2] and pkg.pipeline_streams(3) == chosen   # shared by all pipelines
    for i in range(3):
        for j in range(3):
            if i != j:
                assert pkg.streams_overlap(chosen[i], chosen[j])
    assert not pkg.streams_overlap(chosen[0], chosen[0])  # one stream runs in order
    del others


def test_batch_loop_of_the_extension_directly(pkg, oracle, graph):
    # torch.classes.dgs_classes.BatchLoop without the Python pipeline around it: batches come back in
    # the order they were pushed, whatever mix of host and device seeds; nothing is pending after
    # the last pop; a closed loop refuses more
    indptr, indices = graph
    big = 1 << 40
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, big)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, big)
    feats = torch.randn((20000, 16))
    x_ct = pkg.create_chunktensor(feats, 1, big)
    streams = pkg.pipeline_streams(2)
    triples = []
    for st in streams:
        triples += [st.stream_id, st.device_index, st.device_type]
    loop = torch.classes.dgs_classes.BatchLoop(ip_ct, ix_ct, None, [4, 6], False, x_ct, triples, True, True, [])
    rng = np.random.default_rng(3)
    batches = [rng.integers(0, 20000, size=300).astype(np.int64) for _ in range(5)]
    pkg.set_rng_state(5, 100)
    for i, b in enumerate(batches):
        loop._CAPI_push(torch.from_numpy(b) if i % 2 else _dev(b), i < 2, -1)
    assert loop._CAPI_pending() == 5
    for i, b in enumerate(batches):
        frontiers, srcs, dsts, x, seeds_dev = loop._CAPI_pop()
        want_f, _, want_blocks = oracle.sample_blocks(b, indptr, indices, [6, 4], False, 5, 100 + 2 * i)
        assert np.array_equal(_np(frontiers[-1]), want_f) and np.array_equal(_np(seeds_dev), b)
        for h, wb in enumerate(reversed(want_blocks)):
            assert np.array_equal(_np(srcs[h]), wb[0]) and np.array_equal(_np(dsts[h]), wb[1])
        assert torch.equal(x.cpu(), feats[torch.from_numpy(want_f)])
    assert loop._CAPI_pending() == 0
    with pytest.raises(RuntimeError, match="nothing to pop"):
        loop._CAPI_pop()
    loop._CAPI_close()
    loop._CAPI_close()  # closing twice is fine
    with pytest.raises(RuntimeError, match="closed"):
        loop._CAPI_push(_dev(batches[0]), False, -1)


def test_batch_loop_closed_with_batches_pending(pkg, graph):
    # closing a loop gives up what was pushed and not popped: nothing is pending afterwards, a pop
    # raises instead of waiting for a batch that will never come, and so does a push
    indptr, indices = graph
    big = 1 << 40
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, big)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, big)
    streams = pkg.pipeline_streams(2)
    triples = []
    for st in streams:
        triples += [st.stream_id, st.device_index, st.device_type]
    loop = torch.classes.dgs_classes.BatchLoop(ip_ct, ix_ct, None, [4, 6], False, None, triples, False, False, [])
    rng = np.random.default_rng(4)
    for i in range(6):  # more than the two streams take: some are begun, some still queued
        loop._CAPI_push(_dev(rng.integers(0, 20000, size=200).astype(np.int64)), i < 2, -1)
    frontiers, _, _, _, _ = loop._CAPI_pop()
    assert frontiers[-1].numel() > 0 and loop._CAPI_pending() == 5
    loop._CAPI_close()
    assert loop._CAPI_pending() == 0
    with pytest.raises(RuntimeError, match="closed"):
        loop._CAPI_pop()
    with pytest.raises(RuntimeError, match="closed"):
        loop._CAPI_push(_dev(np.arange(10, dtype=np.int64)), True, -1)
    torch.cuda.synchronize()
    # a pipeline whose iteration is abandoned while its loop gets closed underneath ends, too
    sampler = pkg.ChunkTensorSampler([6, 4], ip_ct, ix_ct)
    pipe = pkg.BatchPipeline(sampler, None, inflight=2)
    it = pipe([_dev(rng.integers(0, 20000, size=200).astype(np.int64)) for _ in range(5)])
    next(it)
    for entry in sampler._loops.values():
        entry["loop"]._CAPI_close()
    with pytest.raises(RuntimeError, match="closed"):
        next(it)
    it.close()
    torch.cuda.synchronize()


@pytest.mark.parametrize("native_loop", [True, False])
def test_batch_pipeline_with_a_sampler_that_has_its_own_generator(pkg, oracle, graph, native_loop):
    # batch b of such a sampler draws from streams b * hops ... of its seed, in submission order,
    # whichever loop begins the batches, and leaves the process-wide generator alone
    indptr, indices = graph
    big = 1 << 40
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, big)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, big)
    fanouts = [5, 3]
    rng = np.random.default_rng(21)
    batches = [rng.integers(0, 20000, size=500).astype(np.int64) for _ in range(7)]
    sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, seed=4242)
    pkg.set_rng_state(9, 9)
    pipe = pkg.BatchPipeline(sampler, None, 3, native_loop=native_loop)
    got = [(f.clone(), [(b.src_local.clone(), b.dst_local.clone()) for b in blocks])
           for f, _, blocks in pipe([_dev(b) for b in batches[:4]])]
    got += [(f.clone(), [(b.src_local.clone(), b.dst_local.clone()) for b in blocks])
            for f, _, blocks in pipe([torch.from_numpy(b) for b in batches[4:]])]  # the count goes on
    torch.cuda.synchronize()
    for i, b in enumerate(batches):
        want_f, _, want_blocks = oracle.sample_blocks(b, indptr, indices, fanouts, False, 4242, 2 * i)
        assert np.array_equal(_np(got[i][0]), want_f), i
        for (src, dst), wb in zip(got[i][1], want_blocks):
            assert np.array_equal(_np(src), wb[0]) and np.array_equal(_np(dst), wb[1])
    assert pkg.ops._CAPI_get_rng_state() == [9, 9]


@pytest.mark.parametrize("n_nodes", [1 << 24, (1 << 24) + 1])
def test_bucketed_last_hop_at_its_largest_graph(pkg, oracle, n_nodes):
    # 2^24 nodes is the most the bucketed pass takes (2048 buckets x 8192 ids in LDS); one node
    # more and the hop stays on the table.  Ids from the very top of the range are picked and
    # seeded, so the last LDS entries of the last buckets are in use.
    rng = np.random.default_rng(n_nodes & 0xff)
    deg = np.zeros(n_nodes, dtype=np.int64)
    busy = np.concatenate([rng.integers(0, n_nodes, size=40000), np.arange(n_nodes - 3000, n_nodes)])
    deg[busy] = rng.integers(1, 30, size=busy.size)
    indptr = np.zeros(n_nodes + 1, dtype=np.int64)
    np.cumsum(deg, out=indptr[1:])
    pool = np.concatenate([busy, np.arange(n_nodes - 64, n_nodes), np.arange(64)])
    indices = pool[rng.integers(0, pool.size, size=int(indptr[-1]))].astype(np.int64)
    seeds = np.concatenate([busy[rng.integers(0, busy.size, size=1500)], np.arange(n_nodes - 20, n_nodes)]).astype(np.int64)
    fanouts = [6, 5]
    want_f, _, want_blocks = oracle.sample_blocks(seeds, indptr, indices, fanouts, False, 31, 4)
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, 1 << 40)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
    sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct)
    set_last_hop_mode(pkg, LAST_HOP_MODES[1])
    try:
        pkg.set_rng_state(31, 4)
        frontier, _, blocks = sampler.sample_blocks(None, _dev(seeds))
    finally:
        set_last_hop_mode(pkg, LAST_HOP_MODES[0])
    assert np.array_equal(_np(frontier), want_f)
    _check_blocks(blocks, want_blocks)
    assert want_f.max() >= n_nodes - 20
    del ip_ct, ix_ct, sampler
    torch.cuda.empty_cache()


def test_bucketed_last_hop_near_its_largest_worst_case(pkg, oracle, graph):
    # 1024 seeds x [7, 30, 31] (hop order): the last hop's worst case is 8.1 M units, just inside what
    # the bucketed pass has room for (1985 of its 2048 tiles; most of them stay empty on this graph,
    # whose 20,000 nodes the frontier soon exhausts), and the pass is chosen by size
    indptr, indices = graph
    rng = np.random.default_rng(17)
    seeds = rng.permutation(20000)[:1024].astype(np.int64)
    fanouts = [31, 30, 7]
    want_f, _, want_blocks = oracle.sample_blocks(seeds, indptr, indices, fanouts, False, 77, 3)
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, 1 << 40)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
    sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct)
    for mode in LAST_HOP_MODES:
        set_last_hop_mode(pkg, mode)
        try:
            pkg.set_rng_state(77, 3)
            frontier, _, blocks = sampler.sample_blocks(None, _dev(seeds))
        finally:
            set_last_hop_mode(pkg, LAST_HOP_MODES[0])
        assert np.array_equal(_np(frontier), want_f), mode
        _check_blocks(blocks, want_blocks)


def test_seed_loader_stands_in_for_the_dataloader(pkg, oracle, graph):
    # SeedLoader where upstream's loop has the DGL DataLoader (single_node/chunktensor.py:123-151): batches of
    # the training ids in order or shuffled, the short last batch kept or dropped, every batch what the
    # sampler returns for it (held against the oracle), with and without the feature gather, one batch at a
    # time and in flight, and with a sampler that cannot run fused
    indptr, indices = graph
    big = 1 << 40
    rng = np.random.default_rng(21)
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, big)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, big)
    feats = rng.standard_normal((20000, 12)).astype(np.float32)
    x_ct = pkg.create_chunktensor(torch.from_numpy(feats), 1, big, cache_rate=0.5)
    train = rng.permutation(20000)[:1050].astype(np.int64)

    def check(loader, fanouts, seed, want_batches, with_x):
        got = list(loader)
        assert len(got) == len(loader) == len(want_batches)
        for i, (out, want_seeds) in enumerate(zip(got, want_batches)):
            assert np.array_equal(_np(out[1]), want_seeds)
            want_f, _, want_blocks = oracle.sample_blocks(want_seeds, indptr, indices, fanouts, False, seed,
                                                          len(fanouts) * i)
            assert np.array_equal(_np(out[0]), want_f)
            for b, w in zip(out[2], want_blocks):
                assert np.array_equal(_np(b.src_local), w[0]) and np.array_equal(_np(b.dst_local), w[1])
            assert len(out) == (4 if with_x else 3)
            if with_x:
                assert np.array_equal(_np(out[3]), feats[want_f])

    in_order = [train[i:i + 100] for i in range(0, 1050, 100)]
    for inflight, fanouts, device in ((3, [5, 4], None), (1, [5, 4], "cuda"), (3, [70, 3], None)):
        sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct, seed=77)
        assert sampler.fused == (max(fanouts) <= 64)
        check(pkg.SeedLoader(None, torch.from_numpy(train), sampler, device=device, batch_size=100, chunk_features=x_ct,
                             inflight=inflight, use_ddp=True, use_uva=True), fanouts, 77, in_order, True)
    sampler = pkg.ChunkTensorSampler([5, 4], ip_ct, ix_ct, seed=78)
    check(pkg.SeedLoader(None, torch.from_numpy(train), sampler, batch_size=100, drop_last=True), [5, 4], 78, in_order[:10], False)
    # shuffled: every id once per iteration (the tail of 50 dropped), a new order every iteration, the order
    # that the generator gives
    sampler = pkg.ChunkTensorSampler([3], ip_ct, ix_ct, seed=79)
    loader = pkg.SeedLoader(None, torch.from_numpy(train), sampler, device="cuda", batch_size=100, shuffle=True,
                            drop_last=True, generator=torch.Generator().manual_seed(5))
    first = torch.cat([out[1] for out in loader]).cpu()
    second = torch.cat([out[1] for out in loader]).cpu()
    g = torch.Generator().manual_seed(5)
    assert torch.equal(first, torch.from_numpy(train)[torch.randperm(1050, generator=g)][:1000])
    assert torch.equal(second, torch.from_numpy(train)[torch.randperm(1050, generator=g)][:1000])
    assert not torch.equal(first, second) and first.unique().numel() == 1000


def test_hashed_pass_reports_a_bucket_its_table_cannot_hold(pkg, oracle):
    # The hashed form of the bucketed pass tells a bucket's ids apart in an on-chip table and goes over a
    # crowded bucket in parts; ids that share bucket AND part beyond the table's slots cannot happen by
    # chance, but they can be made: 400 distinct neighbour ids whose hash (the library's, restated here)
    # agrees in the bits that choose the bucket (256 of them for an input this small) and the part (4 for
    # 400 units and tables of 256 slots).  Every kernel runs to its end, the hop's flag word says so, the
    # operator raises, and the same call on the node table gives the oracle's answer.  (The pass serves the
    # last of at least two hops: the first hop here has fanout 0 and leaves the seeds as they are.)
    def hash_id(ids):
        h = ids.astype(np.uint32)
        h ^= h >> np.uint32(16); h *= np.uint32(0x85EBCA6B)
        h ^= h >> np.uint32(13); h *= np.uint32(0xC2B2AE35)
        h ^= h >> np.uint32(16)
        return h

    n = 1 << 21
    h = hash_id(np.arange(n, dtype=np.int64))
    crowd = np.flatnonzero(((h & 255) == 0) & ((h >> 23) % 4 == 0))[:400]
    assert crowd.size == 400
    seeds = np.flatnonzero((h & 255) != 0)[:40].astype(np.int64)
    deg = np.zeros(n, dtype=np.int64)
    deg[seeds] = 10
    indptr = np.concatenate([[0], np.cumsum(deg)])
    indices = crowd.astype(np.int64)  # row of seed j = crowd[10 j : 10 j + 10], copied whole at fanout 10
    ip_ct = pkg.create_chunktensor(torch.from_numpy(indptr), 1, 1 << 40)
    ix_ct = pkg.create_chunktensor(torch.from_numpy(indices), 1, 1 << 40)
    fanouts = [10, 0]  # model order: hop order is 0, then 10
    sampler = pkg.ChunkTensorSampler(fanouts, ip_ct, ix_ct)
    try:
        set_last_hop_mode(pkg, LAST_HOP_MODES[3])
        with pytest.raises(RuntimeError, match="crowd"):
            sampler.sample_blocks(None, _dev(seeds))
        torch.cuda.synchronize()
        # half of the crowd fits the tables: the same mode then answers, and answers right
        want_f, _, want_b = oracle.sample_blocks(seeds[:20], indptr, indices, fanouts, False, 3, 0)
        pkg.set_rng_state(3, 0)
        f, _, blocks = sampler.sample_blocks(None, _dev(seeds[:20]))
        assert np.array_equal(_np(f), want_f) and np.array_equal(_np(blocks[0].src_local), want_b[0][0])
    finally:
        set_last_hop_mode(pkg, LAST_HOP_MODES[0])
    want_f, _, want_b = oracle.sample_blocks(seeds, indptr, indices, fanouts, False, 3, 0)
    pkg.set_rng_state(3, 0)
    f, _, blocks = sampler.sample_blocks(None, _dev(seeds))
    assert np.array_equal(_np(f), want_f) and np.array_equal(_np(blocks[0].src_local), want_b[0][0])
    assert np.array_equal(_np(blocks[0].dst_local), want_b[0][1])
