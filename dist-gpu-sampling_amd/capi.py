"""ctypes binding of the C ABI in include/dgs_hip.h (libdgs_hip.so).

Thin by design: arguments are raw addresses and sizes.  The helpers at the
bottom accept torch tensors only to take their data_ptr(); torch supplies the
device memory and the stream, nothing else.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdgs_hip.so")

DGS_OK, DGS_ERR_INVALID, DGS_ERR_HIP, DGS_ERR_WORKSPACE, DGS_ERR_UNSUPPORTED, DGS_ERR_RANGE = range(6)
TIER_ANY, TIER_DEVICE, TIER_HOST = 0, 1, 2
DEBUG_FORCE_SPLIT_TABLE, DEBUG_WEIGHTED_GROUP, DEBUG_GATHER_LDS_BYTES, DEBUG_SAMPLER_GRID_CAP = 0, 1, 2, 3
DEBUG_SAMPLER_BUCKETED = 4
PROBE_LOAD, PROBE_STORE, PROBE_ATOMIC_MIN, PROBE_ATOMIC_MIN_NO_RETURN = 0, 1, 2, 3
MAX_SEGMENTS = 8

c_i64, c_i32, c_u64, c_u32, c_vp, c_sz = (ctypes.c_int64, ctypes.c_int32, ctypes.c_uint64, ctypes.c_uint32,
                                          ctypes.c_void_p, ctypes.c_size_t)


class View(ctypes.Structure):
    """dgs_view"""
    _fields_ = [("dev", c_vp), ("host", c_vp), ("threshold", c_i64), ("total", c_i64),
                ("elem_bytes", c_i32), ("reserved_", c_i32)]


class BlockOut(ctypes.Structure):
    """dgs_block_out"""
    _fields_ = [("src_local", c_vp), ("dst_local", c_vp)]


class Segments(ctypes.Structure):
    """dgs_segments"""
    _fields_ = [("ptr", c_vp * MAX_SEGMENTS), ("len", c_i64 * MAX_SEGMENTS), ("count", c_i32),
                ("reserved_", c_i32)]


# name -> (restype, argtypes); must list every function include/dgs_hip.h declares
SIGNATURES = {
    "dgs_last_error": (ctypes.c_char_p, []),
    "dgs_status_name": (ctypes.c_char_p, [ctypes.c_int]),
    "dgs_abi_version": (ctypes.c_int, []),
    "dgs_debug_set": (ctypes.c_int, [c_i32, c_i64]),
    "dgs_debug_probe_table": (ctypes.c_int, [c_i32, c_vp, c_i64, c_i64, c_u64, c_vp, c_vp]),
    "dgs_store_split": (ctypes.c_int, [c_i64, c_i32, c_i64, ctypes.POINTER(c_i64), ctypes.POINTER(c_i64)]),
    "dgs_store_create": (ctypes.c_int, [c_i64, c_i32, c_i64, ctypes.POINTER(c_vp)]),
    "dgs_store_destroy": (ctypes.c_int, [c_vp]),
    "dgs_store_load": (ctypes.c_int, [c_vp, c_vp, c_i64]),
    "dgs_store_view": (ctypes.c_int, [c_vp, ctypes.POINTER(View)]),
    "dgs_store_slices": (ctypes.c_int, [c_vp, ctypes.POINTER(c_vp), ctypes.POINTER(c_i64),
                                        ctypes.POINTER(c_vp), ctypes.POINTER(c_i64)]),
    "dgs_current_allocated": (c_i64, []),
    "dgs_gather_rows": (ctypes.c_int, [View, c_i64, c_vp, c_i32, c_i64, c_vp, c_i32, c_vp, c_vp]),
    "dgs_gather_rows_dyn": (ctypes.c_int, [View, c_i64, c_vp, c_i32, c_i64, c_vp, c_i64, c_vp, c_i32, c_vp, c_vp]),
    "dgs_gather_rows_dyn_shared": (ctypes.c_int, [View, c_i64, c_vp, c_i32, c_i64, c_vp, c_i64, c_vp, c_i32, c_i32, c_vp,
                                                  c_vp]),
    "dgs_split_index_workspace_bytes": (c_sz, [c_i64]),
    "dgs_split_index": (ctypes.c_int, [View, c_i64, c_vp, c_i32, c_i64, c_vp, c_vp, c_vp, c_vp, c_sz, c_vp]),
    "dgs_sample_workspace_bytes": (c_sz, [c_i64]),
    "dgs_sample_count": (ctypes.c_int, [c_vp, c_i32, c_i64, View, c_i64, c_i64, c_i32, c_vp, c_vp, c_vp, c_sz, c_vp]),
    "dgs_sample_fill": (ctypes.c_int, [c_vp, c_i32, c_i64, View, c_i64, c_i32, c_u64, c_u32, c_vp, c_vp,
                                       c_vp, c_sz, c_vp]),
    "dgs_sample_neighbors": (ctypes.c_int, [c_vp, c_i32, c_i64, View, View, c_i64, c_i32, c_u64, c_u32,
                                            c_vp, c_vp, c_vp, c_vp, c_sz, c_vp]),
    "dgs_sample_neighbors_static": (ctypes.c_int, [c_vp, c_i32, c_i64, View, View, c_i64, c_i32, c_u64, c_u32,
                                                   c_vp, c_vp, c_vp, c_vp]),
    "dgs_sample_fill_weighted": (ctypes.c_int, [c_vp, c_i32, c_i64, View, View, c_i64, c_i32, c_u64, c_u32, c_vp,
                                                c_vp, c_vp, c_sz, c_vp]),
    "dgs_sample_neighbors_weighted": (ctypes.c_int, [c_vp, c_i32, c_i64, View, View, View, c_i64, c_i32, c_u64,
                                                     c_u32, c_vp, c_vp, c_vp, c_vp, c_sz, c_vp]),
    "dgs_unique_relabel_workspace_bytes": (c_sz, [c_i64, c_i32]),
    "dgs_unique_relabel": (ctypes.c_int, [Segments, Segments, c_i32, c_i32, c_vp, c_vp, c_vp, ctypes.POINTER(c_vp),
                                          Segments, c_vp, c_sz, c_vp]),
    "dgs_sample_blocks_plan": (ctypes.c_int, [c_i64, ctypes.POINTER(c_i64), c_i32, ctypes.POINTER(c_i64),
                                              ctypes.POINTER(c_i64)]),
    "dgs_sample_blocks_workspace_bytes": (c_sz, [c_i64, ctypes.POINTER(c_i64), c_i32, c_i32]),
    "dgs_node_table_bytes": (c_sz, [c_i64]),
    "dgs_sample_blocks": (ctypes.c_int, [c_vp, c_i32, c_i64, View, View, ctypes.POINTER(c_i64), c_i32, c_i32,
                                         c_u64, c_u32, c_vp, c_u32, c_vp, ctypes.POINTER(BlockOut), c_vp, c_vp,
                                         ctypes.POINTER(c_vp), c_vp, c_sz, c_vp]),
    "dgs_sample_blocks_weighted_workspace_bytes": (c_sz, [c_i64, ctypes.POINTER(c_i64), c_i32, c_i32]),
    "dgs_sample_blocks_weighted": (ctypes.c_int, [c_vp, c_i32, c_i64, View, View, View, ctypes.POINTER(c_i64), c_i32,
                                                  c_i32, c_u64, c_u32, c_vp, c_u32, c_vp, ctypes.POINTER(BlockOut),
                                                  c_vp, c_vp, ctypes.POINTER(c_vp), c_vp, c_sz, c_vp]),
    "dgs_renumber_csc": (ctypes.c_int, [c_vp, c_i32, c_vp, c_i32, c_vp, c_vp, c_vp, c_i64, c_i64, c_vp, c_vp]),
    "dgs_read_back": (ctypes.c_int, [c_vp, c_vp, c_sz, c_vp]),
    "dgs_read_back_begin": (ctypes.c_int, [c_vp, c_vp, c_sz, c_vp, ctypes.POINTER(c_vp)]),
    "dgs_read_back_wait": (ctypes.c_int, [c_vp]),
    "dgs_ticket_record": (ctypes.c_int, [c_vp, ctypes.POINTER(c_vp)]),
    "dgs_ticket_stream_wait": (ctypes.c_int, [c_vp, c_vp]),
    "dgs_ticket_wait": (ctypes.c_int, [c_vp]),
    "dgs_ticket_wait_words": (ctypes.c_int, [c_vp, c_vp, c_i32]),
    "dgs_ticket_sync": (ctypes.c_int, [c_vp]),
    "dgs_ticket_sync_words": (ctypes.c_int, [c_vp, c_vp, c_i32]),
    "dgs_stream_wait_words": (ctypes.c_int, [c_vp, c_vp, c_i32]),
    "dgs_ticket_release": (ctypes.c_int, [c_vp]),
    "dgs_stream_query": (ctypes.c_int, [c_vp, ctypes.POINTER(c_i32)]),
    "dgs_ticket_query": (ctypes.c_int, [c_vp, ctypes.POINTER(c_i32)]),
}

if not os.path.exists(LIB_PATH):
    raise ImportError(f"{LIB_PATH} is missing; build it with dist-gpu-sampling_amd/build.py")
lib = ctypes.CDLL(LIB_PATH)
# the signatures above are those of one version of include/dgs_hip.h; a library of another version
# would take its arguments from the wrong places
ABI_VERSION = 3
lib.dgs_abi_version.restype = ctypes.c_int
if lib.dgs_abi_version() != ABI_VERSION:
    raise ImportError(f"{LIB_PATH} reports C ABI version {lib.dgs_abi_version()}, this binding is written for "
                      f"{ABI_VERSION}; rebuild it with dist-gpu-sampling_amd/build.py")
for _name, (_res, _args) in SIGNATURES.items():
    _f = getattr(lib, _name)
    _f.restype = _res
    _f.argtypes = _args


class DgsError(RuntimeError):
    def __init__(self, status):
        self.status = status
        super().__init__(f"{lib.dgs_status_name(status).decode()}: {lib.dgs_last_error().decode()}")


def check(status):
    if status != DGS_OK:
        raise DgsError(status)


# ---- helpers over torch tensors (addresses only) --------------------------------
def stream_ptr():
    return c_vp(torch.cuda.current_stream().cuda_stream)


def tensor_view(t):
    """A plain device array as a single-tier view."""
    assert t.is_contiguous()
    return View(t.data_ptr(), None, t.numel(), t.numel(), t.element_size(), 0)


def segments(tensors):
    s = Segments()
    s.count = len(tensors)
    for i, t in enumerate(tensors):
        assert t.is_contiguous()
        s.ptr[i] = t.data_ptr()
        s.len[i] = t.numel()
    return s


class Store:
    """Owner of a dgs_store (two-tier ChunkTensor storage)."""

    def __init__(self, total_elems, elem_bytes, capacity_bytes):
        h = c_vp()
        check(lib.dgs_store_create(total_elems, elem_bytes, capacity_bytes, ctypes.byref(h)))
        self.handle = h
        self.view = View()
        check(lib.dgs_store_view(self.handle, ctypes.byref(self.view)))

    def load(self, cpu_tensor):
        assert cpu_tensor.device.type == "cpu" and cpu_tensor.is_contiguous()
        check(lib.dgs_store_load(self.handle, cpu_tensor.data_ptr(), cpu_tensor.numel()))

    def close(self):
        if self.handle is not None:
            check(lib.dgs_store_destroy(self.handle))
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _ws(nbytes, device):
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def read_i64(dev_tensor, count):
    host = torch.empty(count, dtype=torch.int64).pin_memory()
    check(lib.dgs_read_back(host.data_ptr(), dev_tensor.data_ptr(), 8 * count, stream_ptr()))
    return host.tolist()


def probe_table(op, table, n_ops, salt, sink):
    """dgs_debug_probe_table on torch's current stream: n_ops random 8-byte accesses of kind `op`
    to `table` (an int64 device tensor); `sink` is an int64 device tensor of one element."""
    check(lib.dgs_debug_probe_table(op, table.data_ptr(), table.numel(), n_ops, salt, sink.data_ptr(), stream_ptr()))


def gather_rows(view, row_elems, index, dtype, tier=TIER_ANY, bad_index=None):
    """`bad_index`: optional int64[1] device tensor that the kernel sets to 1 on an index outside
    the rows the tier holds (the caller clears it)."""
    n = index.numel()
    out = torch.empty((n, row_elems), dtype=dtype, device=index.device)
    check(lib.dgs_gather_rows(view, row_elems, index.data_ptr(), index.element_size(), n, out.data_ptr(), tier,
                              bad_index.data_ptr() if bad_index is not None else None, stream_ptr()))
    return out


def split_index(view, row_elems, index):
    n = index.numel()
    local = torch.empty_like(index)
    host = torch.empty_like(index)
    counts = torch.empty(2, dtype=torch.int64, device=index.device)
    nb = lib.dgs_split_index_workspace_bytes(n)
    ws = _ws(nb, index.device)
    check(lib.dgs_split_index(view, row_elems, index.data_ptr(), index.element_size(), n, local.data_ptr(),
                              host.data_ptr(), counts.data_ptr(), ws.data_ptr(), nb, stream_ptr()))
    c = read_i64(counts, 2)
    return local[:c[0]], host[:c[1]]


def sample_neighbors(seeds, indptr_view, indices_view, num_picks, replace, rng_seed, rng_stream, two_step=False):
    """Returns (coo_row, coo_col, flags)."""
    n = seeds.numel()
    nb = lib.dgs_sample_workspace_bytes(n)
    ws = _ws(nb, seeds.device)
    nnz = torch.empty(2, dtype=torch.int64, device=seeds.device)
    w = seeds.element_size()
    if two_step:
        if two_step == "mirrored":
            # the lengths through pinned words that the count kernel writes and the host polls
            pinned = torch.full((2,), -1, dtype=torch.int64).pin_memory()
            check(lib.dgs_sample_count(seeds.data_ptr(), w, n, indptr_view, indices_view.total, num_picks, int(replace), nnz.data_ptr(),
                                       pinned.data_ptr(), ws.data_ptr(), nb, stream_ptr()))
            ticket = ctypes.c_void_p()
            check(lib.dgs_ticket_record(stream_ptr(), ctypes.byref(ticket)))
            check(lib.dgs_ticket_wait_words(ticket, pinned.data_ptr(), 2))
            cnt, flags = pinned.tolist()
        else:
            check(lib.dgs_sample_count(seeds.data_ptr(), w, n, indptr_view, indices_view.total, num_picks, int(replace),
                                       nnz.data_ptr(), None, ws.data_ptr(), nb, stream_ptr()))
            cnt, flags = read_i64(nnz, 2)
        rows = torch.empty(cnt, dtype=seeds.dtype, device=seeds.device)
        cols = torch.empty(cnt, dtype=seeds.dtype, device=seeds.device)
        check(lib.dgs_sample_fill(seeds.data_ptr(), w, n, indices_view, num_picks, int(replace), rng_seed,
                                  rng_stream, rows.data_ptr(), cols.data_ptr(), ws.data_ptr(), nb, stream_ptr()))
        return rows, cols, flags
    rows = torch.empty(n * num_picks, dtype=seeds.dtype, device=seeds.device)
    cols = torch.empty(n * num_picks, dtype=seeds.dtype, device=seeds.device)
    check(lib.dgs_sample_neighbors(seeds.data_ptr(), w, n, indptr_view, indices_view, num_picks, int(replace),
                                   rng_seed, rng_stream, rows.data_ptr(), cols.data_ptr(), nnz.data_ptr(),
                                   ws.data_ptr(), nb, stream_ptr()))
    cnt, flags = read_i64(nnz, 2)
    return rows[:cnt], cols[:cnt], flags


STATIC_MAX_SEEDS = 65536  # DGS_STATIC_MAX_SEEDS


def sample_neighbors_static(seeds, indptr_view, indices_view, num_picks, replace, rng_seed, rng_stream,
                            rows, cols, nnz):
    """dgs_sample_neighbors_static into caller-provided buffers (rows / cols: n * num_picks ids,
    nnz: int64[2]); nothing is allocated here or in the library.  Returns (coo_row, coo_col, flags)."""
    n = seeds.numel()
    check(lib.dgs_sample_neighbors_static(seeds.data_ptr(), seeds.element_size(), n, indptr_view, indices_view,
                                          num_picks, int(replace), rng_seed, rng_stream, rows.data_ptr(),
                                          cols.data_ptr(), nnz.data_ptr(), stream_ptr()))
    cnt, flags = read_i64(nnz, 2)
    return rows[:cnt], cols[:cnt], flags


def sample_neighbors_weighted(seeds, indptr_view, indices_view, probs_view, num_picks, replace, rng_seed,
                              rng_stream, two_step=False):
    """Returns (coo_row, coo_col, flags)."""
    n = seeds.numel()
    nb = lib.dgs_sample_workspace_bytes(n)
    ws = _ws(nb, seeds.device)
    nnz = torch.empty(2, dtype=torch.int64, device=seeds.device)
    w = seeds.element_size()
    if two_step:
        check(lib.dgs_sample_count(seeds.data_ptr(), w, n, indptr_view, indices_view.total, num_picks, int(replace), nnz.data_ptr(),
                                   None, ws.data_ptr(), nb, stream_ptr()))
        cnt, flags = read_i64(nnz, 2)
        rows = torch.empty(cnt, dtype=seeds.dtype, device=seeds.device)
        cols = torch.empty(cnt, dtype=seeds.dtype, device=seeds.device)
        check(lib.dgs_sample_fill_weighted(seeds.data_ptr(), w, n, indices_view, probs_view, num_picks,
                                           int(replace), rng_seed, rng_stream, rows.data_ptr(), cols.data_ptr(),
                                           ws.data_ptr(), nb, stream_ptr()))
        return rows, cols, flags
    rows = torch.empty(n * num_picks, dtype=seeds.dtype, device=seeds.device)
    cols = torch.empty(n * num_picks, dtype=seeds.dtype, device=seeds.device)
    check(lib.dgs_sample_neighbors_weighted(seeds.data_ptr(), w, n, indptr_view, indices_view, probs_view,
                                            num_picks, int(replace), rng_seed, rng_stream, rows.data_ptr(),
                                            cols.data_ptr(), nnz.data_ptr(), ws.data_ptr(), nb, stream_ptr()))
    cnt, flags = read_i64(nnz, 2)
    return rows[:cnt], cols[:cnt], flags


def renumber_csc(indptr, indices, order, rank, new_indptr):
    """New edge array of the graph renumbered by order[new] = old / rank[old] = new."""
    out = torch.empty_like(indices)
    check(lib.dgs_renumber_csc(indptr.data_ptr(), indptr.element_size(), indices.data_ptr(), indices.element_size(),
                               order.data_ptr(), rank.data_ptr(), new_indptr.data_ptr(), indptr.numel() - 1,
                               indices.numel(), out.data_ptr(), stream_ptr()))
    return out


def unique_relabel(mapping, requiring, packed_table=True, polled=False, retry=True):
    """Returns (unique, [relabelled ...]).  With `packed_table` 8-byte ids are tried in the one-word
    slots first and the call is repeated with the two-array table if an id does not fit
    (`retry=False`: it is not, and the void results of the first attempt are returned as they are).
    With `polled` the counts come through pinned words that the host polls instead of a copy."""
    dev = mapping[0].device
    dt = mapping[0].dtype
    n = sum(t.numel() for t in mapping)
    unique = torch.empty(n, dtype=dt, device=dev)
    outs = [torch.empty_like(t) for t in requiring]
    num = torch.empty(2, dtype=torch.int64, device=dev)
    w = mapping[0].element_size()
    nb = lib.dgs_unique_relabel_workspace_bytes(n, w)
    ws = _ws(nb, dev)
    for packed in ((1, 0) if packed_table and retry else (1,) if packed_table else (0,)):
        if polled:
            pinned = torch.full((2,), -1, dtype=torch.int64).pin_memory()
            check(lib.dgs_unique_relabel(segments(mapping), segments(requiring), w, packed, unique.data_ptr(),
                                         num.data_ptr(), pinned.data_ptr(), None, segments(outs), ws.data_ptr(), nb,
                                         stream_ptr()))
            check(lib.dgs_stream_wait_words(stream_ptr(), pinned.data_ptr(), 2))
            u, overflow = pinned.tolist()
        else:
            check(lib.dgs_unique_relabel(segments(mapping), segments(requiring), w, packed, unique.data_ptr(),
                                         num.data_ptr(), None, None, segments(outs), ws.data_ptr(), nb, stream_ptr()))
            u, overflow = read_i64(num, 2)
        if not overflow:
            break
    return unique[:u], outs


def sample_blocks(seeds, indptr_view, indices_view, hop_fanouts, replace, rng_seed, first_stream,
                  feature_view=None, feature_row_elems=None, feature_dtype=None, node_table=None, epoch=0,
                  probs_view=None, gather_expected=0):
    """All hops in one call (picks by the edge weights `probs_view` when given).  Returns [(frontier, src_local, dst_local) per hop], the gathered
    rows of the last frontier when a feature view is given, and the per-hop error flags.
    `node_table` is an int64 device tensor of dgs_node_table_bytes(n_nodes) bytes filled with -1."""
    hops = len(hop_fanouts)
    n = seeds.numel()
    fan = (c_i64 * hops)(*hop_fanouts)
    smax = (c_i64 * (hops + 1))()
    emax = (c_i64 * hops)()
    check(lib.dgs_sample_blocks_plan(n, fan, hops, smax, emax))
    w = seeds.element_size()
    frontier = torch.empty(smax[hops], dtype=seeds.dtype, device=seeds.device)
    bufs = []
    outs = (BlockOut * hops)()
    for h in range(hops):
        s = torch.empty(emax[h], dtype=seeds.dtype, device=seeds.device)
        d = torch.empty(emax[h], dtype=seeds.dtype, device=seeds.device)
        bufs.append((s, d))
        outs[h] = BlockOut(s.data_ptr(), d.data_ptr())
    sizes = torch.empty(3 * hops + 1, dtype=torch.int64, device=seeds.device)
    table_ptr = node_table.data_ptr() if node_table is not None else None
    if probs_view is None:
        nb = lib.dgs_sample_blocks_workspace_bytes(n, fan, hops, w)
        ws = _ws(nb, seeds.device)
        check(lib.dgs_sample_blocks(seeds.data_ptr(), w, n, indptr_view, indices_view, fan, hops, int(replace),
                                    rng_seed, first_stream, table_ptr, epoch, frontier.data_ptr(), outs,
                                    sizes.data_ptr(), None, None, ws.data_ptr(), nb, stream_ptr()))
    else:
        nb = lib.dgs_sample_blocks_weighted_workspace_bytes(n, fan, hops, w)
        ws = _ws(nb, seeds.device)
        check(lib.dgs_sample_blocks_weighted(seeds.data_ptr(), w, n, indptr_view, indices_view, probs_view, fan, hops,
                                             int(replace), rng_seed, first_stream, table_ptr, epoch,
                                             frontier.data_ptr(), outs, sizes.data_ptr(), None, None, ws.data_ptr(),
                                             nb, stream_ptr()))
    x = None
    if feature_view is not None:
        x = torch.empty((smax[hops], feature_row_elems), dtype=feature_dtype, device=seeds.device)
        check(lib.dgs_gather_rows_dyn(feature_view, feature_row_elems, frontier.data_ptr(), w, smax[hops],
                                      sizes.data_ptr() + 8 * hops, gather_expected, x.data_ptr(), TIER_ANY, None,
                                      stream_ptr()))
    sz = read_i64(sizes, 3 * hops + 1)
    result = [(frontier[:sz[h + 1]], s[:sz[hops + 1 + h]], d[:sz[hops + 1 + h]]) for h, (s, d) in enumerate(bufs)]
    if x is not None:
        x = x[:sz[hops]]
    return result, x, sz[2 * hops + 1:]
