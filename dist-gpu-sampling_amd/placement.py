"""Hottest-rows-first placement for the positional two-tier stores.

A ChunkTensor keeps its first `capacity_per_gpu` bytes in HBM and the rest in pinned host
memory (src/chunk_tensor.cc:57-73); upstream's harness sizes that prefix
(oppo_bench/single_node/utils/chunktensor_sampler.py:32-60) and leaves the order of the rows to
the caller.  This module orders them: nodes are renumbered by decreasing degree, the CSC arrays
and the feature rows are rewritten for the new ids, and the capacity that puts a wanted share of
rows (or whatever fits a memory budget) into HBM is computed with upstream's own formula.
"""
import torch


def degree_order(indptr, indices=None, by="in"):
    """order[new] = old, sorted by decreasing degree, ties by increasing old id.
    by="in": in-degree of the CSC rows (indptr differences); by="out": how often a node
    occurs in `indices`, i.e. how often sampling can pick it as a neighbour."""
    if by == "in":
        deg = indptr[1:] - indptr[:-1]
    elif by == "out":
        if indices is None:
            raise ValueError('degree_order(by="out") needs the indices array')
        deg = torch.bincount(indices.long(), minlength=indptr.numel() - 1)
    else:
        raise ValueError(f'by must be "in" or "out", got {by!r}')
    return torch.sort(deg, descending=True, stable=True).indices


def renumber_csc(indptr, indices, order):
    """The graph with node `order[r]` renamed r.  Device tensors in, (new_indptr, new_indices,
    rank) out, rank[old] = new; the edges of a row keep their order."""
    return torch.ops.dgs_ops._CAPI_renumber_csc(indptr, indices, order.to(indptr.device))


def permute_rows(tensor, order, chunk_rows=1 << 22):
    """tensor[order] for a node-indexed tensor, on the tensor's own device, a slab at a time
    (a feature matrix that does not fit HBM is permuted where it lives)."""
    order = order.to(tensor.device)
    out = torch.empty_like(tensor)
    for a in range(0, order.numel(), chunk_rows):
        b = min(order.numel(), a + chunk_rows)
        torch.index_select(tensor, 0, order[a:b], out=out[a:b])
    return out


def capacity_for_rows(tensor_or_shape, dtype=None, rows=None, fraction=None):
    """capacity_per_gpu in bytes that keeps the first `rows` rows (or that `fraction` of the
    rows) of a [n, ...] tensor in HBM."""
    if isinstance(tensor_or_shape, torch.Tensor):
        shape, dtype = tuple(tensor_or_shape.shape), tensor_or_shape.dtype
    else:
        shape = tuple(tensor_or_shape)
    row_elems = 1
    for d in shape[1:]:
        row_elems *= d
    if rows is None:
        rows = int(shape[0] * fraction)
    rows = max(0, min(int(rows), shape[0]))
    return rows * row_elems * torch.empty(0, dtype=dtype).element_size()


def rows_in_hbm(tensor_or_shape, dtype, capacity_bytes):
    """Whole rows of a [n, ...] store that a capacity keeps in HBM (a row straddling the
    boundary belongs to neither tier, index_with_chunk_tensor.cu:68-76)."""
    shape = tuple(tensor_or_shape.shape) if isinstance(tensor_or_shape, torch.Tensor) else tuple(tensor_or_shape)
    row_elems = 1
    for d in shape[1:]:
        row_elems *= d
    elems = min(capacity_bytes // torch.empty(0, dtype=dtype).element_size(), shape[0] * row_elems)
    return int(elems // row_elems)


def expected_hit_rate(degrees_in_new_order, hot_rows):
    """Share of neighbour picks that land on the first `hot_rows` rows when a node is picked in
    proportion to the given degree (its number of occurrences as a neighbour)."""
    d = degrees_in_new_order.double()
    total = d.sum()
    return float(d[:hot_rows].sum() / total) if total > 0 else 0.0
