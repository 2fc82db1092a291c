"""GPU parity of the two-tier store and its gathers against the CPU oracle and
torch.index_select, through the C ABI and through the torch operator layer."""
import numpy as np
import pytest
import torch

from helpers import load_pkg

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pkg():
    return load_pkg()


def _bits(t):
    """Reinterpret any tensor as integers for bit-exact comparison."""
    t = t.contiguous()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])


def test_readme_demo(pkg):
    # upstream README.md:51-62: [100] int64 with 200 bytes per GPU
    before = pkg.ops._CAPI_get_current_allocated()
    c = pkg.ChunkTensor([100], torch.int64, 200)
    assert pkg.ops._CAPI_get_current_allocated() - before == 200
    assert (c._CAPI_get_sub_device_tensor() == -1).all()  # slice is pre-filled with 0xFF bytes
    c._CAPI_load_from_tensor(torch.arange(100))
    assert c._CAPI_get_host_tensor().tolist() == list(range(25, 100))
    dev = c._CAPI_get_sub_device_tensor()
    assert dev.is_cuda and dev.cpu().tolist() == list(range(25))
    out = c._CAPI_index(torch.tensor([99, 0, 24, 25], device="cuda"))
    assert out.shape == (4, 1) and out[:, 0].cpu().tolist() == [99, 0, 24, 25]
    del c, dev
    assert pkg.ops._CAPI_get_current_allocated() == before


def test_create_chunktensor_capacity(pkg):
    # chunktensor_sampler.py:40-42 + chunk_tensor.cc:57-73 on real stores: the device slice holds
    # int(min(total_bytes * cache_rate // 1, available_mem)) // element size elements (at most all),
    # the host slice the rest; numbers worked out by hand for a [1000, 25] float32 tensor (100 000 B)
    t = torch.arange(25000, dtype=torch.float32).reshape(1000, 25)
    for rate, avail, want_dev in [(1.0, 1 << 40, 25000), (0.5, 1 << 40, 12500), (0.25, 1 << 40, 6250), (0.0, 1 << 40, 0),
                                  (0.333, 1 << 40, 8325), (1.0, 30001, 7500), (0.1, 5000, 1250), (2.0, 1 << 40, 25000)]:
        before = pkg.ops._CAPI_get_current_allocated()
        ct = pkg.create_chunktensor(t, 1, avail, cache_rate=rate)
        dev, host = ct._CAPI_get_sub_device_tensor(), ct._CAPI_get_host_tensor()
        assert (dev.numel(), host.numel()) == (want_dev, 25000 - want_dev), (rate, avail)
        assert pkg.ops._CAPI_get_current_allocated() - before == 4 * want_dev
        assert torch.equal(dev.cpu(), t.reshape(-1)[:want_dev]) and torch.equal(host, t.reshape(-1)[want_dev:])
        idx = torch.tensor([0, 999, 333, 332, 334, 500], device="cuda")  # rows around every boundary above
        assert torch.equal(ct._CAPI_index(idx).cpu(), t[idx.cpu()])
        del ct, dev, host
    # an int64 store, as the harness makes for indptr / indices
    t8 = torch.arange(1001, dtype=torch.int64)
    ct = pkg.create_chunktensor(t8, 1, 1 << 40, cache_rate=0.4)
    assert ct._CAPI_get_sub_device_tensor().numel() == 400  # 8008 * 0.4 // 1 = 3203 bytes -> 400 elements


@pytest.mark.parametrize("dtype", [torch.float32, torch.int64, torch.int32, torch.bfloat16, torch.uint8,
                                   torch.float64, torch.bool])
@pytest.mark.parametrize("rows,dim", [(257, 100), (64, 128), (1000, 1), (33, 7), (50, 256)])
def test_index_every_split(pkg, oracle, dtype, rows, dim):
    g = torch.Generator().manual_seed(rows * 1000 + dim)
    if dtype == torch.bool:
        full = torch.rand((rows, dim), generator=g) > 0.5
    elif dtype.is_floating_point:
        full = torch.randn((rows, dim), generator=g).to(dtype)
    else:
        full = torch.randint(0, 200, (rows, dim), generator=g).to(dtype)
    eb = full.element_size()
    total_bytes = full.numel() * eb
    # none, all, a row boundary, a split inside a row, an odd byte count
    caps = [0, total_bytes, total_bytes + 999, (rows // 2) * dim * eb, (rows // 3) * dim * eb + 3 * eb,
            (rows // 2) * dim * eb + 1]
    for idx_dtype in (torch.int64, torch.int32):
        idx = torch.randint(0, rows, (513,), generator=g).to(idx_dtype)
        want = full[idx.long()]
        for cap in caps:
            ct = pkg.ChunkTensor([rows, dim], dtype, cap)
            ct._CAPI_load_from_tensor(full)
            got = ct._CAPI_index(idx.cuda())
            assert got.dtype == dtype and got.shape == (513, dim)
            assert torch.equal(_bits(got.cpu()), _bits(want)), (dtype, rows, dim, cap)
            # the oracle (restating chunk_tensor_wrapper::At) agrees for the same split
            if dtype not in (torch.bfloat16, torch.bool):
                thr = oracle.store_split([rows, dim], eb, cap)["threshold"]
                o = oracle.gather(full.numpy(), idx.numpy(), thr)
                assert np.array_equal(o, got.cpu().numpy())


def test_index_1d_and_empty(pkg):
    full = torch.arange(1000, dtype=torch.int32)
    ct = pkg.ChunkTensor([1000], torch.int32, 1234)
    ct._CAPI_load_from_tensor(full)
    idx = torch.tensor([999, 0, 308, 309, 500], device="cuda")
    assert ct._CAPI_index(idx)[:, 0].cpu().tolist() == [999, 0, 308, 309, 500]
    e = ct._CAPI_index(torch.empty(0, dtype=torch.int64, device="cuda"))
    assert e.shape == (0, 1)
    assert ct._CAPI_remote_index(torch.empty(0, dtype=torch.int64, device="cuda")).shape == (0, 1)


def test_wide_rows(pkg):
    # 600000-byte rows take the segment-per-block kernel
    full = torch.randn((6, 150000))
    ct = pkg.ChunkTensor([6, 150000], torch.float32, 2 * 150000 * 4 + 4 * 100)
    ct._CAPI_load_from_tensor(full)
    idx = torch.tensor([5, 2, 0, 2, 1], device="cuda")
    assert torch.equal(ct._CAPI_index(idx).cpu(), full[idx.cpu()])


def test_split_local_host_index(pkg, oracle):
    rows, dim = 400, 12
    full = torch.randn((rows, dim))
    cap = 150 * dim * 4 + 5 * 4  # row 150 straddles the boundary
    ct = pkg.ChunkTensor([rows, dim], torch.float32, cap)
    ct._CAPI_load_from_tensor(full)
    g = torch.Generator().manual_seed(5)
    for n in (0, 1, 1023, 1024, 1025, 5000):
        idx = torch.randint(0, rows, (n,), generator=g)
        loc, rem, host = ct._CAPI_split_index(idx.cuda())
        s = oracle.store_split([rows, dim], 4, cap)
        o_loc, o_rem, o_host = oracle.split_index(idx.numpy(), s["threshold"], s["device_elems"], dim)
        assert np.array_equal(loc.cpu().numpy(), o_loc) and np.array_equal(host.cpu().numpy(), o_host)
        assert rem.numel() == 0 and o_rem.size == 0
    # tier-specific gathers on the lists split_index made: the host list holds row 150, which
    # straddles the boundary (its first five elements are in the device slice)
    assert (host == 150).any() and not (loc >= 150).any()
    assert torch.equal(ct._CAPI_local_index(loc).cpu(), full[loc.cpu()])
    assert torch.equal(ct._CAPI_host_index(host).cpu(), full[host.cpu()])
    ct._CAPI_synchronize_and_check()
    # int32 ids
    idx32 = torch.randint(0, rows, (777,), generator=g, dtype=torch.int32)
    loc, _, host = ct._CAPI_split_index(idx32.cuda())
    assert loc.dtype == torch.int32
    assert torch.equal(loc.cpu(), idx32[idx32 < 150]) and torch.equal(host.cpu(), idx32[idx32 >= 150])


def test_gather_through_c_abi(pkg, oracle):
    capi = pkg.capi
    rows, dim = 300, 100
    full = torch.randn((rows, dim))
    cap = 100 * dim * 4 + 8
    st = capi.Store(rows * dim, 4, cap)
    st.load(full)
    assert (st.view.threshold, st.view.total, st.view.elem_bytes) == (100 * dim + 2, rows * dim, 4)
    idx = torch.randint(0, rows, (999,), device="cuda")
    out = capi.gather_rows(st.view, dim, idx, torch.float32)
    assert np.array_equal(out.cpu().numpy(), oracle.gather(full.numpy(), idx.cpu().numpy(), st.view.threshold))
    loc, host = capi.split_index(st.view, dim, idx)
    assert torch.equal(loc, idx[idx < 100]) and torch.equal(host, idx[idx >= 100])
    # plain device tensor as a single-tier view
    dev = full.cuda()
    out2 = capi.gather_rows(capi.tensor_view(dev), dim, idx, torch.float32)
    assert torch.equal(out2, dev[idx])
    st.close()


def test_errors_raise_instead_of_aborting(pkg):
    with pytest.raises(RuntimeError):
        pkg.ChunkTensor([2, 2, 2], torch.float32, 0)
    with pytest.raises(RuntimeError):
        pkg.ChunkTensor([10], torch.float32, -1)
    ct = pkg.ChunkTensor([10, 4], torch.float32, 64)
    with pytest.raises(RuntimeError):
        ct._CAPI_load_from_tensor(torch.zeros(10, 4, dtype=torch.float64))
    with pytest.raises(RuntimeError):
        ct._CAPI_load_from_tensor(torch.zeros(10, 5))
    with pytest.raises(RuntimeError):
        ct._CAPI_load_from_tensor(torch.zeros(4, 10).t())
    with pytest.raises(RuntimeError):
        ct._CAPI_load_from_tensor(torch.zeros(10, 4, device="cuda"))
    with pytest.raises(RuntimeError):
        ct._CAPI_index(torch.zeros(3, dtype=torch.int64))  # CPU index
    with pytest.raises(RuntimeError):
        ct._CAPI_index(torch.zeros(3, device="cuda"))  # float index
    capi = pkg.capi
    v = capi.tensor_view(torch.zeros(8, device="cuda"))
    assert capi.lib.dgs_gather_rows(v, 1, None, 3, 1, None, 0, None, None) == capi.DGS_ERR_INVALID
    assert b"index width" in capi.lib.dgs_last_error()


def test_gather_refuses_row_ids_outside_the_store(pkg):
    # ids are checked before they address anything: bad rows come back as zeros, the flag word is
    # set, good rows are untouched by it
    capi = pkg.capi
    rows, dim = 300, 25
    full = torch.randn((rows, dim))
    cap = 100 * dim * 4  # rows 0..99 in HBM, 100..299 in host memory, no straddling row
    st = capi.Store(rows * dim, 4, cap)
    st.load(full)
    flag = torch.zeros(1, dtype=torch.int64, device="cuda")
    good = torch.tensor([0, 299, 100, 99, 150], device="cuda")
    out = capi.gather_rows(st.view, dim, good, torch.float32, bad_index=flag)
    assert flag.item() == 0 and torch.equal(out.cpu(), full[good.cpu()])
    for dtype in (torch.int64, torch.int32):
        idx = torch.tensor([5, -1, 299, 300, 2 ** 31 - 1, 120, -2 ** 31], dtype=dtype, device="cuda")
        ok = torch.tensor([True, False, True, False, False, True, False])
        flag.zero_()
        out = capi.gather_rows(st.view, dim, idx, torch.float32, bad_index=flag).cpu()
        assert flag.item() == 1
        assert torch.equal(out[ok], full[idx.cpu().long()[ok]]) and (out[~ok] == 0).all()
    idx = torch.tensor([2 ** 40, 7, -2 ** 62], device="cuda")
    out = capi.gather_rows(st.view, dim, idx, torch.float32).cpu()  # no flag word: rows are just zero-filled
    assert torch.equal(out[1], full[7]) and (out[0] == 0).all() and (out[2] == 0).all()
    # a tier-specific gather refuses rows of the other tier
    for tier, idx, ok in ((capi.TIER_DEVICE, [3, 100, 99, 299], [True, False, True, False]),
                          (capi.TIER_HOST, [100, 99, 299, 0], [True, False, True, False])):
        flag.zero_()
        ids = torch.tensor(idx, device="cuda")
        out = capi.gather_rows(st.view, dim, ids, torch.float32, tier=tier, bad_index=flag).cpu()
        ok = torch.tensor(ok)
        assert flag.item() == 1 and torch.equal(out[ok], full[ids.cpu()[ok]]) and (out[~ok] == 0).all()
    st.close()
    # the operator: the store remembers, and says so at its next call
    ct = pkg.ChunkTensor([rows, dim], torch.float32, cap)
    ct._CAPI_load_from_tensor(full)
    x = ct._CAPI_index(torch.tensor([1, rows, 2], device="cuda"))
    assert (x[1] == 0).all().item() and torch.equal(x[2].cpu(), full[2])
    with pytest.raises(RuntimeError, match="outside the store"):
        ct._CAPI_synchronize_and_check()
    ct._CAPI_synchronize_and_check()  # reported once
    ct._CAPI_local_index(torch.tensor([100], device="cuda"))
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="outside the store"):
        ct._CAPI_index(torch.tensor([1], device="cuda"))
    assert torch.equal(ct._CAPI_index(torch.tensor([1], device="cuda")).cpu(), full[1:2])


def test_probe_table_touches_only_its_table(pkg):
    # the measurement aid behind bench.py's table_access_rates: every kind of access stays inside
    # the table, loads change nothing, stores and atomics leave thread indices behind
    capi = pkg.capi
    slots, n_ops = 1000, 5000
    guard = torch.full((slots + 2,), -7, dtype=torch.int64, device="cuda")
    table = guard[1:-1]
    sink = torch.zeros(1, dtype=torch.int64, device="cuda")
    table.fill_(torch.iinfo(torch.int64).max)
    capi.probe_table(capi.PROBE_LOAD, table, n_ops, 3, sink)
    assert (table == torch.iinfo(torch.int64).max).all()
    capi.probe_table(capi.PROBE_ATOMIC_MIN, table, n_ops, 0, sink)
    touched = table[table != torch.iinfo(torch.int64).max]
    assert 900 < touched.numel() <= slots and int(touched.max()) < n_ops and int(touched.min()) >= 0
    before = table.clone()
    capi.probe_table(capi.PROBE_ATOMIC_MIN_NO_RETURN, table, n_ops, 0, sink)  # the same values again: no change
    assert torch.equal(table, before)
    table.fill_(-1)
    capi.probe_table(capi.PROBE_STORE, table, n_ops, 1, sink)
    stored = table[table != -1]
    assert 900 < stored.numel() <= slots and int(stored.max()) < n_ops and int(stored.min()) >= 0
    assert int(guard[0]) == -7 and int(guard[-1]) == -7
    with pytest.raises(RuntimeError):
        capi.probe_table(9, table, n_ops, 0, sink)


def test_gather_of_a_tier_that_holds_no_whole_row(pkg):
    # a device slice shorter than one row holds no row whole: a device-tier gather refuses every
    # id (and reads nothing), the per-chunk gather still serves the straddling row exactly
    capi = pkg.capi
    rows, dim = 50, 24
    full = torch.randn((rows, dim))
    st = capi.Store(rows * dim, 4, 10 * 4)  # 10 of row 0's 24 elements in HBM
    st.load(full)
    flag = torch.zeros(1, dtype=torch.int64, device="cuda")
    idx = torch.tensor([0, 1, 49, 7], device="cuda")
    out = capi.gather_rows(st.view, dim, idx, torch.float32, tier=capi.TIER_DEVICE, bad_index=flag)
    assert flag.item() == 1 and (out == 0).all().item()
    flag.zero_()
    out = capi.gather_rows(st.view, dim, idx, torch.float32, bad_index=flag)
    assert flag.item() == 0 and torch.equal(out.cpu(), full[idx.cpu()])
    out = capi.gather_rows(st.view, dim, idx, torch.float32, tier=capi.TIER_HOST, bad_index=flag)  # row 0 straddles
    assert flag.item() == 0 and torch.equal(out.cpu(), full[idx.cpu()])
    st.close()


@pytest.mark.parametrize("dim", [25, 40000 * 4])  # the flattened kernel and the one for very wide rows
def test_gather_dyn_leaves_a_buffer_alone_that_is_too_small(pkg, dim):
    # dgs_gather_rows_dyn with a device-side row count above the rows the output holds writes
    # nothing; with a count that fits it gathers exactly that many rows
    capi = pkg.capi
    rows = 64 if dim > 1000 else 4000
    full = torch.randn((rows, dim))
    st = capi.Store(rows * dim, 4, 1 << 40)
    st.load(full)
    n_max = 40
    idx = torch.randint(0, rows, (100,), device="cuda")
    out = torch.full((n_max + 1, dim), -3.0, device="cuda")
    for count, written in ((41, 0), (100, 0), (-1, 0), (40, 40), (7, 7), (0, 0)):
        for expected in (0, 1, 7, 40, 1000):  # how many rows the launch is sized for: a hint, never a limit
            out.fill_(-3.0)
            n_dev = torch.tensor([count], dtype=torch.int64, device="cuda")
            capi.check(capi.lib.dgs_gather_rows_dyn(st.view, dim, idx.data_ptr(), 8, n_max, n_dev.data_ptr(), expected,
                                                    out.data_ptr(), capi.TIER_ANY, None, capi.stream_ptr()))
            assert torch.equal(out[:written].cpu(), full[idx[:written].cpu()]), (count, expected)
            assert (out[written:] == -3.0).all().item(), (count, expected)
    st.close()


@pytest.mark.parametrize("dtype,dim", [(torch.float32, 100), (torch.bfloat16, 128), (torch.float32, 3)])
def test_gather_dyn_with_more_rows_than_expected(pkg, dtype, dim):
    # a launch sized for far fewer rows than turn up (its blocks loop), for about as many, and for
    # more: the same rows come out; the ids behind the count are readable but never used (they
    # name no row of the store here), and a bad id inside the count is still refused
    capi = pkg.capi
    rows = 30000
    full = torch.randn((rows, dim)).to(dtype)
    st = capi.Store(rows * dim, full.element_size(), rows * dim * full.element_size() // 3)  # both tiers
    st.load(full)
    view = st.view
    n_max = 50000
    idx = torch.randint(0, rows, (n_max,), device="cuda", dtype=torch.int32)
    bad = torch.zeros(1, dtype=torch.int64, device="cuda")
    out = torch.empty((n_max, dim), dtype=dtype, device="cuda")
    for count in (0, 1, 999, 20011, n_max):
        tail = idx.clone()
        tail[count:] = 2 ** 31 - 1  # what lies behind the count is no row id at all
        for expected in (0, 1, 300, count, count + count // 4 + 1024, 10 ** 9):
            out.fill_(-3.0)
            bad.zero_()
            n_dev = torch.tensor([count], dtype=torch.int64, device="cuda")
            capi.check(capi.lib.dgs_gather_rows_dyn(view, dim, tail.data_ptr(), 4, n_max, n_dev.data_ptr(), expected,
                                                    out.data_ptr(), capi.TIER_ANY, bad.data_ptr(), capi.stream_ptr()))
            assert torch.equal(out[:count].cpu(), full[idx[:count].cpu().long()]), (count, expected)
            assert (out[count:] == -3.0).all().item() and bad.item() == 0, (count, expected)
        # the same gather with fewer of its blocks on a CU at a time (for callers that share the GPU with
        # compute-bound kernels): the same rows, whatever the limit
        for blocks_per_cu in (0, 1, 3, 4, 7, 8, 1000):
            out.fill_(-3.0)
            capi.check(capi.lib.dgs_gather_rows_dyn_shared(view, dim, tail.data_ptr(), 4, n_max, n_dev.data_ptr(), count,
                                                           out.data_ptr(), capi.TIER_ANY, blocks_per_cu, bad.data_ptr(),
                                                           capi.stream_ptr()))
            assert torch.equal(out[:count].cpu(), full[idx[:count].cpu().long()]), (count, blocks_per_cu)
            assert (out[count:] == -3.0).all().item() and bad.item() == 0, (count, blocks_per_cu)
    assert capi.lib.dgs_gather_rows_dyn_shared(view, dim, idx.data_ptr(), 4, n_max, n_dev.data_ptr(), 0, out.data_ptr(),
                                               capi.TIER_ANY, -1, None, capi.stream_ptr()) == capi.DGS_ERR_INVALID
    tail = idx.clone()
    tail[17] = rows  # one past the last row, inside the count
    n_dev = torch.tensor([100], dtype=torch.int64, device="cuda")
    capi.check(capi.lib.dgs_gather_rows_dyn(view, dim, tail.data_ptr(), 4, n_max, n_dev.data_ptr(), 50, out.data_ptr(),
                                            capi.TIER_ANY, bad.data_ptr(), capi.stream_ptr()))
    assert bad.item() == 1 and (out[17] == 0).all().item()
    assert torch.equal(out[18:100].cpu(), full[idx[18:100].cpu().long()])
    st.close()


def test_waiting_for_words_that_nobody_writes_ends_with_the_ticket(pkg):
    # dgs_ticket_wait_words / dgs_stream_wait_words poll pinned words that the kernels turn
    # non-negative; a ticket whose point is reached, or a stream that has drained, ends the wait
    # all the same (here: nothing was launched that would write the words), and words that were
    # written before the call end it at once
    import ctypes
    import time
    capi = pkg.capi
    words = torch.full((3,), -1, dtype=torch.int64).pin_memory()
    torch.cuda.synchronize()
    ticket = ctypes.c_void_p()
    capi.check(capi.lib.dgs_ticket_record(capi.stream_ptr(), ctypes.byref(ticket)))
    t0 = time.perf_counter()
    capi.check(capi.lib.dgs_ticket_wait_words(ticket, words.data_ptr(), 3))
    assert time.perf_counter() - t0 < 0.5 and words.tolist() == [-1, -1, -1]
    t0 = time.perf_counter()
    capi.check(capi.lib.dgs_stream_wait_words(capi.stream_ptr(), words.data_ptr(), 3))
    assert time.perf_counter() - t0 < 0.5
    words[:] = torch.tensor([0, 7, 1 << 40])
    capi.check(capi.lib.dgs_ticket_record(capi.stream_ptr(), ctypes.byref(ticket)))
    capi.check(capi.lib.dgs_ticket_wait_words(ticket, words.data_ptr(), 3))
    capi.check(capi.lib.dgs_stream_wait_words(capi.stream_ptr(), words.data_ptr(), 3))
    with pytest.raises(capi.DgsError):
        capi.check(capi.lib.dgs_stream_wait_words(capi.stream_ptr(), None, 3))
