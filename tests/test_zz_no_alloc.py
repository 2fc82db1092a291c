"""The entry point that allocates nothing (dgs_sample_neighbors_static) against the entry point it is
a variant of (dgs_sample_neighbors with a caller workspace) and against the CPU oracle: bit-exact
rows, columns, edge count and flags, on calls that follow each other on one GPU and share the
library's static scratch; and that such a call leaves every allocation count where it was."""
import numpy as np
import pytest
import torch

from helpers import load_pkg, powerlaw_graph

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _static_call(capi, seeds, ipv, ixv, k, replace, rng_seed, rng_stream):
    # outputs are the caller's; poisoned so that a slot the call leaves unwritten shows
    n = seeds.numel()
    rows = torch.full((max(n * k, 1),), -7, dtype=seeds.dtype, device="cuda")
    cols = torch.full((max(n * k, 1),), -7, dtype=seeds.dtype, device="cuda")
    nnz = torch.full((2,), -7, dtype=torch.int64, device="cuda")
    return capi.sample_neighbors_static(seeds, ipv, ixv, k, replace, rng_seed, rng_stream, rows, cols, nnz)


@pytest.mark.parametrize("id_dtype,ptr_dtype", [(np.int64, np.int64), (np.int32, np.int64)])
def test_static_entry_point_matches_the_workspace_one(oracle, id_dtype, ptr_dtype):
    capi = load_pkg().capi
    rng = np.random.default_rng(77)
    indptr, indices = powerlaw_graph(rng, 30000, 20, 4000, id_dtype=id_dtype, ptr_dtype=ptr_dtype)
    ip, ix = _dev(indptr), _dev(indices)
    ipv, ixv = capi.tensor_view(ip), capi.tensor_view(ix)
    # two calls in a row, the second with a smaller input: what the first left in the scratch
    # (per-seed offsets, tile sums of 8 tiles more) must not leak into the second; then a larger
    # one again, with replacement, and a fanout that takes the wave-per-row fill
    for n_seeds, k, replace in [(20011, 15, False), (1500, 15, False), (40000, 7, True), (300, 100, False), (0, 5, False)]:
        seeds = _dev(rng.integers(0, 30000, size=n_seeds).astype(id_dtype))
        want_r, want_c, want_flags = capi.sample_neighbors(seeds, ipv, ixv, k, replace, 0xFEED5EED, 4)
        got_r, got_c, got_flags = _static_call(capi, seeds, ipv, ixv, k, replace, 0xFEED5EED, 4)
        assert got_flags == want_flags == 0
        assert got_r.numel() == want_r.numel() and got_c.numel() == want_c.numel()
        assert torch.equal(got_r, want_r) and torch.equal(got_c, want_c), (n_seeds, k, replace)
        o_r, o_c = oracle.sample_neighbors(seeds.cpu().numpy(), indptr, indices, k, replace, 0xFEED5EED, 4)
        assert np.array_equal(got_r.cpu().numpy(), o_r) and np.array_equal(got_c.cpu().numpy(), o_c)


def test_static_entry_point_allocates_nothing(oracle):
    # after a first call (which looks the scratch symbol's address up), calls through the C ABI with
    # the caller's own output buffers leave the library's, torch's and the device's allocation
    # counts where they were, whatever the input size
    pkg = load_pkg()
    capi = pkg.capi
    rng = np.random.default_rng(78)
    indptr, indices = powerlaw_graph(rng, 20000, 20, 2000)
    ip, ix = _dev(indptr), _dev(indices)
    ipv, ixv = capi.tensor_view(ip), capi.tensor_view(ix)
    k, n_max = 12, 30000
    rows = torch.empty(n_max * k, dtype=torch.int64, device="cuda")
    cols = torch.empty(n_max * k, dtype=torch.int64, device="cuda")
    nnz = torch.empty(2, dtype=torch.int64, device="cuda")
    all_seeds = _dev(rng.integers(0, 20000, size=n_max))
    stream = capi.stream_ptr()

    def call(n):
        capi.check(capi.lib.dgs_sample_neighbors_static(all_seeds.data_ptr(), 8, n, ipv, ixv, k, 0, 21, 3,
                                                        rows.data_ptr(), cols.data_ptr(), nnz.data_ptr(), stream))
    for n in (100, n_max):  # warm-up: resolves the symbol on this device, loads the kernels
        call(n)
    torch.cuda.synchronize()
    before = (capi.lib.dgs_current_allocated(), torch.cuda.memory_allocated(), torch.cuda.memory_reserved(),
              torch.cuda.mem_get_info()[0])
    for n in (n_max, 17, 4097):
        call(n)
        torch.cuda.synchronize()
        after = (capi.lib.dgs_current_allocated(), torch.cuda.memory_allocated(), torch.cuda.memory_reserved(),
                 torch.cuda.mem_get_info()[0])
        assert after == before, (n, before, after)
    cnt = int(nnz[0].item())
    o_r, o_c = oracle.sample_neighbors(all_seeds[:4097].cpu().numpy(), indptr, indices, k, False, 21, 3)
    assert cnt == o_r.size and np.array_equal(rows[:cnt].cpu().numpy(), o_r) and np.array_equal(cols[:cnt].cpu().numpy(), o_c)


def test_static_entry_point_rejects_what_does_not_fit():
    capi = load_pkg().capi
    ip = _dev(np.arange(0, 11, dtype=np.int64))
    ix = _dev(np.arange(10, dtype=np.int64))
    n = capi.STATIC_MAX_SEEDS + 1
    seeds = torch.zeros(n, dtype=torch.int64, device="cuda")
    buf = torch.empty(n, dtype=torch.int64, device="cuda")
    nnz = torch.empty(2, dtype=torch.int64, device="cuda")
    st = capi.lib.dgs_sample_neighbors_static(seeds.data_ptr(), 8, n, capi.tensor_view(ip), capi.tensor_view(ix), 1, 0,
                                              1, 0, buf.data_ptr(), buf.data_ptr(), nnz.data_ptr(), capi.stream_ptr())
    assert st == capi.DGS_ERR_UNSUPPORTED and b"65536" in capi.lib.dgs_last_error()
    # the largest size that fits runs, and agrees with the workspace entry point
    seeds = _dev(np.random.default_rng(5).integers(0, 10, size=capi.STATIC_MAX_SEEDS))
    want = capi.sample_neighbors(seeds, capi.tensor_view(ip), capi.tensor_view(ix), 1, False, 1, 0)
    got = _static_call(capi, seeds, capi.tensor_view(ip), capi.tensor_view(ix), 1, False, 1, 0)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]) and got[2] == want[2] == 0
