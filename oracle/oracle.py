"""numpy front end of the CPU oracle (oracle/dgs_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of the benchmark.  The shipped package never imports it.

Every function here is a thin wrapper; the algorithms (and their citations of
the upstream sources) are in dgs_oracle.c.  `sample_blocks` restates the
multi-layer driver of oppo_bench/single_node/utils/chunktensor_sampler.py:93-118.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    stale = not os.path.exists(_LIB_PATH) or any(
        os.path.getmtime(os.path.join(_HERE, f)) > os.path.getmtime(_LIB_PATH) for f in ("dgs_oracle.c", "Makefile"))
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B", "-s", "liboracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_bounded.restype = ctypes.c_uint32
        _lib.oracle_draw.restype = ctypes.c_uint32
        _lib.oracle_sample_counts.restype = ctypes.c_int64
        _lib.oracle_unique_relabel.restype = ctypes.c_int64
        _lib.oracle_unique_relabel_parallel.restype = ctypes.c_int64
        _lib.oracle_neg_log_u32.restype = ctypes.c_double
        _lib.oracle_weighted_key.restype = ctypes.c_double
        _lib.oracle_weight_quantum.restype = ctypes.c_uint64
        _lib.oracle_bounded64.restype = ctypes.c_uint64
    return _lib


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _i64(x):
    return ctypes.c_int64(int(x))


def _ids(a):
    a = np.ascontiguousarray(a)
    assert a.dtype in (np.int32, np.int64), a.dtype
    return a


# ---------------------------------------------------------------- Philox ----
def philox(ctr, key):
    c = np.asarray(ctr, dtype=np.uint32)
    k = np.asarray(key, dtype=np.uint32)
    out = np.zeros(4, dtype=np.uint32)
    lib().oracle_philox4x32_10(_p(c), _p(k), _p(out))
    return out


def bounded(words, n):
    w = np.asarray(words, dtype=np.uint32)
    return int(lib().oracle_bounded(_p(w), ctypes.c_uint32(n)))


def draw(seed, stream, row, j, n):
    return int(lib().oracle_draw(ctypes.c_uint64(seed), ctypes.c_uint32(stream), _i64(row),
                                 ctypes.c_uint32(j), ctypes.c_uint32(n)))


# ----------------------------------------------------------------- store ----
def store_split(shape, elem_bytes, capacity_bytes, world=1):
    """Split arithmetic of the ChunkTensor constructor (src/chunk_tensor.cc:44-73)."""
    shape = list(shape)
    assert len(shape) in (1, 2)
    strides = [1] * len(shape)
    total = 1
    for i in range(len(shape) - 1, -1, -1):
        strides[i] = total
        total *= shape[i]
    dev = ctypes.c_int64()
    host = ctypes.c_int64()
    thr = ctypes.c_int64()
    lib().oracle_store_split(_i64(total), _i64(elem_bytes), _i64(capacity_bytes), _i64(world),
                             ctypes.byref(dev), ctypes.byref(host), ctypes.byref(thr))
    return {"total": total, "elem_stride": strides[0], "device_elems": dev.value,
            "host_elems": host.value, "threshold": thr.value}


def _tiers(full_flat, threshold):
    dev = np.ascontiguousarray(full_flat[:threshold])
    host = np.ascontiguousarray(full_flat[threshold:])
    return dev, host


def gather(full, index, threshold=None, tier=0):
    """Row gather through the two-tier accessor.  `full` is the whole logical
    tensor (1-D or 2-D); the first `threshold` ELEMENTS form the device slice."""
    full = np.ascontiguousarray(full)
    row_elems = 1 if full.ndim == 1 else full.shape[1]
    flat = full.reshape(-1)
    if threshold is None:
        threshold = flat.size
    dev, host = _tiers(flat, threshold)
    index = _ids(index)
    n = index.size
    out = np.empty((n, row_elems), dtype=full.dtype)
    lib().oracle_gather(_p(dev), _p(host), _i64(threshold), _i64(full.dtype.itemsize),
                        _i64(row_elems), _p(index), ctypes.c_int(index.dtype.itemsize), _i64(n),
                        _p(out), ctypes.c_int(tier))
    return out


def split_index(index, threshold, device_elems, stride):
    index = _ids(index)
    n = index.size
    outs = [np.empty(n, dtype=index.dtype) for _ in range(3)]
    counts = np.zeros(3, dtype=np.int64)
    lib().oracle_split_index(_i64(threshold), _i64(device_elems), _i64(stride), _p(index),
                             ctypes.c_int(index.dtype.itemsize), _i64(n), _p(outs[0]),
                             _p(outs[1]), _p(outs[2]), _p(counts))
    return tuple(o[:c] for o, c in zip(outs, counts))


# -------------------------------------------------------------- sampling ----
def sample_neighbors(seeds, indptr, indices, num_picks, replace, rng_seed=0, rng_stream=0,
                     indptr_threshold=None, indices_threshold=None):
    """One hop; returns (coo_row, coo_col) like _CAPI_sample_neighbors."""
    seeds = _ids(seeds)
    indptr = _ids(indptr)
    indices = _ids(indices)
    assert seeds.dtype == indices.dtype
    ipt = indptr.size if indptr_threshold is None else indptr_threshold
    ixt = indices.size if indices_threshold is None else indices_threshold
    ipd, iph = _tiers(indptr, ipt)
    ixd, ixh = _tiers(indices, ixt)
    n = seeds.size
    sub = np.zeros(n + 1, dtype=np.int64)
    idb = ctypes.c_int(seeds.dtype.itemsize)
    pb = ctypes.c_int(indptr.dtype.itemsize)
    nnz = lib().oracle_sample_counts(_p(seeds), idb, _i64(n), _p(ipd), _p(iph), _i64(ipt), pb,
                                     _i64(num_picks), ctypes.c_int(int(replace)), _p(sub))
    rows = np.empty(nnz, dtype=seeds.dtype)
    cols = np.empty(nnz, dtype=indices.dtype)
    lib().oracle_sample_fill(_p(seeds), idb, _i64(n), _p(ipd), _p(iph), _i64(ipt), pb, _p(ixd),
                             _p(ixh), _i64(ixt), _i64(num_picks), ctypes.c_int(int(replace)),
                             ctypes.c_uint64(rng_seed), ctypes.c_uint32(rng_stream), _p(sub),
                             _p(rows), _p(cols))
    return rows, cols


def neg_log_u32(x):
    """-ln((x + 0.5) / 2^32) as the weighted sampler computes it."""
    return lib().oracle_neg_log_u32(ctypes.c_uint32(x))


def weighted_key(seed, stream, row, p, weight):
    return lib().oracle_weighted_key(ctypes.c_uint64(seed), ctypes.c_uint32(stream), _i64(row),
                                     ctypes.c_uint32(p), ctypes.c_float(weight))


def weight_quantum(weight, row_max):
    return lib().oracle_weight_quantum(ctypes.c_float(weight), ctypes.c_float(row_max))


def bounded64(words, n):
    w = (ctypes.c_uint32 * 4)(*words)
    return lib().oracle_bounded64(w, ctypes.c_uint64(n))


def sample_neighbors_weighted(seeds, indptr, indices, probs, num_picks, replace, rng_seed=0,
                              rng_stream=0, indptr_threshold=None, indices_threshold=None,
                              probs_threshold=None):
    """One weighted hop; returns (coo_row, coo_col) like _CAPI_sample_neighbors_with_probs."""
    seeds = _ids(seeds)
    indptr = _ids(indptr)
    indices = _ids(indices)
    probs = np.ascontiguousarray(probs, dtype=np.float32)
    assert seeds.dtype == indices.dtype and probs.size == indices.size
    ipt = indptr.size if indptr_threshold is None else indptr_threshold
    ixt = indices.size if indices_threshold is None else indices_threshold
    prt = probs.size if probs_threshold is None else probs_threshold
    ipd, iph = _tiers(indptr, ipt)
    ixd, ixh = _tiers(indices, ixt)
    prd, prh = _tiers(probs, prt)
    n = seeds.size
    sub = np.zeros(n + 1, dtype=np.int64)
    idb = ctypes.c_int(seeds.dtype.itemsize)
    pb = ctypes.c_int(indptr.dtype.itemsize)
    nnz = lib().oracle_sample_counts(_p(seeds), idb, _i64(n), _p(ipd), _p(iph), _i64(ipt), pb,
                                     _i64(num_picks), ctypes.c_int(int(replace)), _p(sub))
    rows = np.empty(nnz, dtype=seeds.dtype)
    cols = np.empty(nnz, dtype=indices.dtype)
    lib().oracle_sample_fill_weighted(_p(seeds), idb, _i64(n), _p(ipd), _p(iph), _i64(ipt), pb,
                                      _p(ixd), _p(ixh), _i64(ixt), _p(prd), _p(prh), _i64(prt),
                                      _i64(num_picks), ctypes.c_int(int(replace)),
                                      ctypes.c_uint64(rng_seed), ctypes.c_uint32(rng_stream),
                                      _p(sub), _p(rows), _p(cols))
    return rows, cols


def sample_counts(seeds, indptr, num_picks, replace):
    seeds = _ids(seeds)
    indptr = _ids(indptr)
    sub = np.zeros(seeds.size + 1, dtype=np.int64)
    lib().oracle_sample_counts(_p(seeds), ctypes.c_int(seeds.dtype.itemsize), _i64(seeds.size),
                               _p(indptr), _p(indptr[:0]), _i64(indptr.size),
                               ctypes.c_int(indptr.dtype.itemsize), _i64(num_picks),
                               ctypes.c_int(int(replace)), _p(sub))
    return sub


# -------------------------------------------------------- unique/relabel ----
def unique_relabel(mapping, requiring, parallel=False):
    """_CAPI_tensor_relabel(mapping_tensors, requiring_relabel_tensors).  `parallel`: the same
    result computed on all host threads (sharded tables), for the timed CPU baseline."""
    mapping = [_ids(m) for m in mapping]
    requiring = [_ids(r) for r in requiring]
    dt = mapping[0].dtype if mapping else requiring[0].dtype
    m = np.concatenate(mapping) if mapping else np.empty(0, dt)
    r = np.concatenate(requiring) if requiring else np.empty(0, dt)
    assert m.dtype == dt and r.dtype == dt
    uniq = np.empty(m.size, dtype=dt)
    rel = np.empty(r.size, dtype=dt)
    fn = lib().oracle_unique_relabel_parallel if parallel else lib().oracle_unique_relabel
    tot = fn(_p(m), _i64(m.size), _p(r), _i64(r.size), ctypes.c_int(dt.itemsize), _p(uniq), _p(rel))
    assert tot >= 0
    sizes = np.cumsum([x.size for x in requiring])[:-1]
    return uniq[:tot].copy(), [x.copy() for x in np.split(rel, sizes)]


# --------------------------------------------------- multi-layer driver -----
def sample_blocks(seed_nodes, indptr, indices, fanouts, replace=False, rng_seed=0,
                  first_stream=0, probs=None, parallel_relabel=False):
    """ChunkTensorSampler.sample_blocks
    (oppo_bench/single_node/utils/chunktensor_sampler.py:93-118) with the DGL
    block replaced by the tuple (src_local, dst_local, n_src, n_dst, src_ids,
    dst_ids).  Hops run over reversed(fanouts); hop h uses rng stream
    first_stream + h.  Returns (frontier, seed_nodes, blocks) with blocks in
    input-to-output order (each new block is inserted at the front)."""
    seeds = _ids(seed_nodes)
    blocks = []
    frontier = seeds
    for hop, fan_out in enumerate(reversed(list(fanouts))):
        if probs is not None:  # chunktensor_sampler.py:97-100
            coo_row, coo_col = sample_neighbors_weighted(seeds, indptr, indices, probs, fan_out,
                                                         replace, rng_seed, first_stream + hop)
        else:
            coo_row, coo_col = sample_neighbors(seeds, indptr, indices, fan_out, replace, rng_seed,
                                                first_stream + hop)
        frontier, (row_l, col_l) = unique_relabel([seeds, coo_col], [coo_row, coo_col], parallel=parallel_relabel)
        blocks.insert(0, (col_l, row_l, frontier.size, seeds.size, frontier, seeds))
        seeds = frontier
    return frontier, _ids(seed_nodes), blocks


# ------------------------------------------------------------ placement -----
def degree_order(indptr):
    """order[new] = old by decreasing in-degree, ties by increasing old id."""
    deg = np.diff(_ids(indptr))
    return np.argsort(-deg, kind="stable").astype(np.int64)


def renumber_csc(indptr, indices, order):
    """The graph with node order[r] renamed r, row by row (plain Python loop over rows:
    the definition itself).  Returns (new_indptr, new_indices, rank), rank[old] = new."""
    indptr, indices = _ids(indptr), _ids(indices)
    order = np.asarray(order, dtype=np.int64)
    n = order.size
    rank = np.empty(n, dtype=indices.dtype)
    rank[order] = np.arange(n, dtype=indices.dtype)
    new_indptr = np.zeros(n + 1, dtype=indptr.dtype)
    new_indices = np.empty_like(indices)
    at = 0
    for r in range(n):
        o = order[r]
        seg = indices[indptr[o]:indptr[o + 1]]
        new_indices[at:at + seg.size] = rank[seg]
        at += seg.size
        new_indptr[r + 1] = at
    return new_indptr, new_indices, rank
