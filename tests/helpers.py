import importlib

import numpy as np


def load_pkg():
    """The package directory name is not a Python identifier; import it by string."""
    return importlib.import_module("dist-gpu-sampling_amd")


def powerlaw_graph(rng, n, mean_deg, max_deg, zero_frac=0.02, id_dtype=np.int64, ptr_dtype=np.int64):
    """CSC arrays with Pareto-like in-degrees (some zero) and uniform sources."""
    deg = np.floor(rng.pareto(1.3, size=n) * mean_deg * 0.35 + 1).astype(np.int64)
    deg = np.minimum(deg, max_deg)
    deg[rng.random(n) < zero_frac] = 0
    indptr = np.zeros(n + 1, dtype=ptr_dtype)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n, size=int(indptr[-1])).astype(id_dtype)
    return indptr, indices


def np_unique_first(x):
    u, first = np.unique(x, return_index=True)
    return u[np.argsort(first, kind="stable")]


LAST_HOP_MODES = ["last hop by size", "last hop bucketed", "last hop bucketed by hash", "last hop bucketed by hash in parts"]


def set_last_hop_mode(pkg, mode):
    """How the fused sampler's last hop finds its first occurrences in this test: by size (small
    test inputs then take the node table's atomics), always through the bucketed LDS pass, or
    always through the form of that pass for graphs of any node count (buckets by a hash of the id),
    or through that form with on-chip tables so small that buckets are gone over in parts."""
    capi = pkg.capi
    capi.check(capi.lib.dgs_debug_set(capi.DEBUG_SAMPLER_BUCKETED, {LAST_HOP_MODES[0]: 0, LAST_HOP_MODES[1]: 2,
                                                                    LAST_HOP_MODES[2]: 3, LAST_HOP_MODES[3]: 4}[mode]))
