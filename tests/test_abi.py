"""CPU-side checks of the boundary: the C ABI library loads, exports every symbol
the header declares, and its host-only entry points behave; the operator layer
registers the upstream names.  No GPU work is launched here."""
import ctypes
import os
import re

import pytest

from helpers import load_pkg

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "dgs_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dgs_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    pkg = load_pkg()
    names = _declared_functions()
    assert len(names) >= 18
    lib = ctypes.CDLL(pkg.HIP_LIB)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/dgs_hip.h but not exported"
    # the ctypes binding covers exactly the declared functions
    assert sorted(pkg.capi.SIGNATURES) == names


def test_struct_layouts_match_the_header():
    pkg = load_pkg()
    assert ctypes.sizeof(pkg.capi.View) == 40      # 2 pointers + 2 int64 + 2 int32
    assert ctypes.sizeof(pkg.capi.Segments) == 8 * 8 + 8 * 8 + 8
    # header, library and binding name one version; the binding and the operator layer refuse a library of another
    header = open(os.path.join(ROOT, "include", "dgs_hip.h")).read()
    declared = int(re.search(r"#define DGS_ABI_VERSION (\d+)", header).group(1))
    assert pkg.capi.lib.dgs_abi_version() == declared == pkg.capi.ABI_VERSION == 3


def test_store_split_matches_oracle(oracle):
    pkg = load_pkg()
    lib = pkg.capi.lib
    d, h = ctypes.c_int64(), ctypes.c_int64()
    for total, eb, cap in [(100, 8, 200), (100, 8, 0), (100, 8, 10 ** 6), (70, 4, 101), (0, 4, 16), (7, 1, 3),
                           (10 ** 12, 2, 10 ** 11 + 1)]:
        assert lib.dgs_store_split(total, eb, cap, ctypes.byref(d), ctypes.byref(h)) == 0
        o = oracle.store_split([total], eb, cap)
        assert (d.value, h.value) == (o["threshold"], o["host_elems"])
    assert lib.dgs_store_split(100, 8, -1, ctypes.byref(d), ctypes.byref(h)) == pkg.capi.DGS_ERR_INVALID
    assert b"capacity_per_gpu" in lib.dgs_last_error()
    assert lib.dgs_store_split(100, 3, 8, ctypes.byref(d), ctypes.byref(h)) == pkg.capi.DGS_ERR_INVALID
    assert lib.dgs_status_name(5) == b"DGS_ERR_RANGE"


def test_workspace_queries_are_monotone():
    lib = load_pkg().capi.lib
    prev = 0
    for n in (0, 1, 255, 256, 257, 10 ** 4, 10 ** 6):
        cur = lib.dgs_sample_workspace_bytes(n)
        assert cur >= prev and cur >= 12 * n
        prev = cur
    assert lib.dgs_unique_relabel_workspace_bytes(1000, 8) >= 2048 * 12 + 4000
    assert lib.dgs_unique_relabel_workspace_bytes(10 ** 6, 4) < lib.dgs_unique_relabel_workspace_bytes(10 ** 6, 8)
    assert lib.dgs_split_index_workspace_bytes(0) > 0


def test_operator_surface_is_registered():
    import torch
    load_pkg()
    for name in ("_CAPI_tensor_relabel", "_CAPI_sample_neighbors", "_CAPI_sample_neighbors_with_chunk_tensor",
                 "_CAPI_get_current_allocated", "_CAPI_get_unique_id", "_CAPI_set_nccl"):
        assert hasattr(torch.ops.dgs_ops, name)
    cls = torch.classes.dgs_classes.ChunkTensor
    assert cls is not None
    schema = str(torch.ops.dgs_ops._CAPI_sample_neighbors.default._schema)
    assert "Tensor seeds" in schema or "Tensor _0" in schema
    assert torch.ops.dgs_ops._CAPI_get_current_allocated() == 0
    assert len(torch.ops.dgs_ops._CAPI_get_unique_id()) == 16
    torch.ops.dgs_ops._CAPI_set_nccl(1, [0] * 16, 0)
    with pytest.raises(RuntimeError):
        torch.ops.dgs_ops._CAPI_set_nccl(2, [0] * 16, 1)


def test_torch_dispatch_is_left_alone_unless_asked():
    # importing the package changes nothing of torch: torch.ScriptObject has no __torch_function__
    # entry and every torch.ops.dgs_ops name is the packet torch made (schemas reachable);
    # lighten_torch_dispatch() opts torch.ScriptObject out of the lookup (a miss costs two C++
    # exceptions per ChunkTensor argument per call), lighten_torch_dispatch(False) takes that back;
    # the package's own calls go to the packets' C++ entries without touching the packets
    import subprocess
    import sys
    code = ("import importlib, os, sys, torch; sys.path.insert(0, %r);"
            "had = '__torch_function__' in vars(torch.ScriptObject);"
            "dgs = importlib.import_module('dist-gpu-sampling_amd');"
            "name = '_CAPI_sample_neighbors_with_chunk_tensor';"
            "print(had, '__torch_function__' in vars(torch.ScriptObject), type(getattr(torch.ops.dgs_ops, name)).__name__,"
            " 'ChunkTensor' in str(getattr(torch.ops.dgs_ops, name).default._schema));"
            "print(dgs.lighten_torch_dispatch(), vars(torch.ScriptObject).get('__torch_function__') is torch._C._disabled_torch_function_impl);"
            "print(dgs.lighten_torch_dispatch(False), type(getattr(torch.ops.dgs_ops, name)).__name__);"
            "print(type(getattr(dgs.fast_ops, name)).__name__, callable(dgs.fast_ops._CAPI_tensor_relabel))"
            % os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    env = {k: v for k, v in os.environ.items() if k != "DGS_LIGHT_TORCH_DISPATCH"}
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    lines = [line.split() for line in out.stdout.strip().splitlines()]
    assert lines[0] == ["False", "False", "OpOverloadPacket", "True"]
    assert lines[1] == ["True", "True"]
    assert lines[2] == ["False", "OpOverloadPacket"]
    assert lines[3] == ["builtin_function_or_method", "True"]
    # asked for through the environment: in place after the import
    code = ("import importlib, sys, torch; sys.path.insert(0, %r); importlib.import_module('dist-gpu-sampling_amd');"
            "print('__torch_function__' in vars(torch.ScriptObject))"
            % os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    out = subprocess.run([sys.executable, "-c", code], env=dict(env, DGS_LIGHT_TORCH_DISPATCH="1"),
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert out.stdout.split() == ["True"]


def test_no_gpu_means_a_loud_error_not_a_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    pkg = load_pkg()
    with pytest.raises(RuntimeError, match="DGS_ERR_HIP"):
        pkg.ChunkTensor([10], torch.float32, 16)


def test_sampler_cache_size_formula():
    # chunktensor_sampler.py:40-42: int(min(total_bytes * cache_rate // num_gpus, available_mem)), then
    # chunk_tensor.cc:57-68: that many bytes / element size elements in HBM, at most all of them.
    # Values worked out by hand, not by the formula's own text; the GPU suite checks the same numbers
    # on real stores (test_gpu_store_gather.py::test_create_chunktensor_capacity).
    import ctypes
    import torch
    pkg = load_pkg()
    for total, rate, avail, want_bytes in [(4000, 1.0, 10 ** 9, 4000), (4000, 0.5, 10 ** 9, 2000), (4000, 0.3, 10 ** 9, 1200),
                                           (4000, 0.333, 10 ** 9, 1332), (4000, 0.0, 10 ** 9, 0), (4000, 1.0, 1001, 1001),
                                           (4001, 0.5, 10 ** 9, 2000), (979_611_600, 0.4, 1 << 40, 391_844_640)]:
        got = pkg.cached_bytes_per_gpu(total, 1, avail, rate)
        assert got == want_bytes and isinstance(got, int), (total, rate, avail, got)
        for elem_bytes in (4, 8):
            dev, host = ctypes.c_int64(), ctypes.c_int64()
            pkg.capi.check(pkg.capi.lib.dgs_store_split(total // elem_bytes, elem_bytes, got, ctypes.byref(dev),
                                                        ctypes.byref(host)))
            assert dev.value == min(want_bytes // elem_bytes, total // elem_bytes)
            assert dev.value + host.value == total // elem_bytes
    with pytest.raises(ValueError):
        pkg.create_chunktensor(torch.zeros(4), 2, 100)


def test_query_entry_points_check_their_arguments():
    # no GPU needed: null arguments are refused before any runtime call
    import ctypes
    capi = load_pkg().capi
    flag = ctypes.c_int32(7)
    assert capi.lib.dgs_stream_query(None, None) == capi.DGS_ERR_INVALID
    assert capi.lib.dgs_ticket_query(None, ctypes.byref(flag)) == capi.DGS_ERR_INVALID
    assert b"ticket_query" in capi.lib.dgs_last_error()


def test_fused_plan_arithmetic_and_limits():
    # host-only parts of the fused sampler's entry points: worst-case sizes by hand (hop h adds seeds * k picks
    # to a frontier that already holds the seeds), and the limits stated beside dgs_sample_blocks
    import ctypes
    capi = load_pkg().capi
    lib, c_i64 = capi.lib, capi.c_i64

    def plan(n, fanouts):
        fan = (c_i64 * max(len(fanouts), 1))(*fanouts)
        smax, emax = (c_i64 * (len(fanouts) + 1))(), (c_i64 * max(len(fanouts), 1))()
        return lib.dgs_sample_blocks_plan(n, fan, len(fanouts), smax, emax), list(smax), list(emax)

    # benchmark configuration 1 in hop order: 1024 seeds, fanouts 5, 10, 15
    assert plan(1024, [5, 10, 15]) == (0, [1024, 6144, 67584, 1081344], [5120, 61440, 1013760])
    assert plan(0, [7]) == (0, [0, 0], [0])
    assert plan(3, [0, 64]) == (0, [3, 3, 195], [0, 192])
    st, _, _ = plan(10, [65])
    assert st == capi.DGS_ERR_UNSUPPORTED and b"per-hop" in lib.dgs_last_error()
    assert plan(10, [-1])[0] == capi.DGS_ERR_UNSUPPORTED
    # 2^30 ids is the largest worst-case frontier: 2^24 seeds x (1 + 63) fits exactly, one seed more does not
    assert plan(1 << 24, [63])[0] == 0
    st, _, _ = plan((1 << 24) + 1, [63])
    assert st == capi.DGS_ERR_UNSUPPORTED and b"2^30" in lib.dgs_last_error()
    assert plan(16384, [50, 50, 50])[0] == capi.DGS_ERR_UNSUPPORTED
    assert plan(10, [])[0] == capi.DGS_ERR_INVALID and plan(10, [1] * 9)[0] == capi.DGS_ERR_INVALID  # 1..8 hops
    assert plan(-1, [3])[0] == capi.DGS_ERR_INVALID
    fan = (c_i64 * 1)(3)
    assert lib.dgs_sample_blocks_plan(10, fan, 1, None, None) == capi.DGS_ERR_INVALID
    # the node table: 8 bytes per node below 2^31 - 1 nodes, none otherwise
    assert lib.dgs_node_table_bytes(2449029) == 8 * 2449029 and lib.dgs_node_table_bytes(0) == 0
    assert lib.dgs_node_table_bytes((1 << 31) - 2) == 8 * ((1 << 31) - 2) and lib.dgs_node_table_bytes((1 << 31) - 1) == 0
    # workspaces: grow with the input, smaller for 4-byte ids, nothing for a plan that is refused
    fan3 = (c_i64 * 3)(5, 10, 15)
    small, large = (lib.dgs_sample_blocks_workspace_bytes(n, fan3, 3, 8) for n in (256, 1024))
    assert 0 < small < large and lib.dgs_sample_blocks_workspace_bytes(1024, fan3, 3, 4) < large
    assert lib.dgs_sample_blocks_weighted_workspace_bytes(1024, fan3, 3, 8) >= large
    assert lib.dgs_sample_blocks_workspace_bytes(1024, (c_i64 * 1)(65), 1, 8) == 0
    assert lib.dgs_sample_blocks_workspace_bytes(1024, fan3, 3, 2) == 0


def test_seed_loader_host_side():
    # what SeedLoader does before any GPU work: batch counts, the options it takes from upstream's
    # DataLoader call (single_node/chunktensor.py:123-132) and the ones it refuses
    import torch
    pkg = load_pkg()

    class NoSampler:
        fused = True

    ids = torch.arange(1050)
    loader = pkg.SeedLoader(None, ids, NoSampler(), device=None, batch_size=100, shuffle=True, drop_last=False,
                            num_workers=0, use_ddp=True, use_uva=True)
    assert len(loader) == 11 and sorted(b.numel() for b in loader._batches()) == [50] + [100] * 10
    assert len(pkg.SeedLoader(None, ids, NoSampler(), batch_size=100, drop_last=True)) == 10
    assert len(pkg.SeedLoader(None, ids[:0], NoSampler(), batch_size=100)) == 0
    assert len(pkg.SeedLoader(None, ids[:100], NoSampler(), batch_size=100)) == 1
    with pytest.raises(TypeError, match="collate"):
        pkg.SeedLoader(None, ids, NoSampler(), collate_fn=None)
    with pytest.raises(ValueError, match="num_workers"):
        pkg.SeedLoader(None, ids, NoSampler(), num_workers=2)
    with pytest.raises(ValueError):
        pkg.SeedLoader(None, ids.float(), NoSampler())
    with pytest.raises(ValueError):
        pkg.SeedLoader(None, ids, NoSampler(), batch_size=0)


def test_placement_host_arithmetic(oracle):
    # the parts of the placement helpers that need no GPU: degree order, capacity <-> rows, hit rate
    import numpy as np
    import torch
    pl = load_pkg().placement
    rng = np.random.default_rng(3)
    deg = rng.integers(0, 9, size=500)
    indptr = torch.from_numpy(np.concatenate([[0], np.cumsum(deg)]).astype(np.int64))
    order = pl.degree_order(indptr)
    assert np.array_equal(order.numpy(), oracle.degree_order(indptr.numpy()))
    indices = torch.from_numpy(rng.integers(0, 500, size=int(indptr[-1])).astype(np.int64))
    by_out = pl.degree_order(indptr, indices, by="out")
    out_deg = np.bincount(indices.numpy(), minlength=500)
    assert (np.diff(out_deg[by_out.numpy()]) <= 0).all()
    feats = torch.arange(500 * 6, dtype=torch.float32).reshape(500, 6)
    assert torch.equal(pl.permute_rows(feats, order, chunk_rows=64), feats[order])
    # capacity for a prefix of rows and back; upstream's split is in elements, a partial row counts for neither tier
    cap = pl.capacity_for_rows(feats, rows=123)
    assert cap == 123 * 6 * 4 and pl.rows_in_hbm(feats, feats.dtype, cap) == 123
    assert pl.rows_in_hbm(feats, feats.dtype, cap + 5) == 123 and pl.rows_in_hbm(feats, feats.dtype, 10 ** 9) == 500
    assert pl.capacity_for_rows([500, 6], torch.float32, fraction=0.4) == 200 * 24
    d = torch.tensor([5.0, 3.0, 1.0, 1.0])
    assert pl.expected_hit_rate(d, 2) == 0.8 and pl.expected_hit_rate(torch.zeros(3), 1) == 0.0
    with pytest.raises(ValueError):
        pl.degree_order(indptr, by="sideways")


def test_bench_refuses_more_than_one_gpu():
    # the benchmark measures one GPU; asking for more ends with a message, before any GPU work
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for argv, env in ((["--gpus", "2"], {}), ([], {"WORLD_SIZE": "4"})):
        p = subprocess.run([sys.executable, os.path.join(root, "bench.py")] + argv, capture_output=True, text=True,
                           env={**os.environ, **env}, timeout=120)
        assert p.returncode != 0 and "ONE GPU" in p.stderr and p.stdout.strip() == ""
