"""Penalty factor of the store's tiers: measured gather time over the time the same bytes
would take at a stated bandwidth (upstream python/compute_loading_factor.py:11-101, options
'local' and 'host'; 'remote' needs a second GPU).  Upstream quotes A100 figures (1300 GB/s HBM,
31 GB/s PCIe Gen4); the defaults here are MI355X's: 8000 GB/s HBM3E, 64 GB/s PCIe Gen5 x16.

  python -c "import importlib; importlib.import_module('dist-gpu-sampling_amd.loading_factor').main()"
"""
import time

import torch

HBM_GBPS = 8000.0
PCIE_GBPS = 64.0


def compute_loading_factor(chunk_features, num_rows, row_elems, elem_bytes, option, bandwidth_gbps,
                           valid_time_threshold_ms=1.0, start_size=2000, valid_needed=10, seed=0, log=print):
    """Same procedure as upstream: batches of distinct random row ids, growing tenfold until a
    gather takes longer than the threshold, then ten measured sizes growing by 1.2; each size is
    timed ten times and the first three are dropped.  Returns the mean of measured / ideal time,
    ideal = gathered bytes / bandwidth (upstream counts the row bytes once, :82-84).
    option 'local': ids below the HBM row count, _CAPI_local_index; 'host': any id of a store
    created with capacity 0, _CAPI_host_index."""
    if option not in ("local", "host"):
        raise ValueError("option must be 'local' or 'host' at world size 1")
    gen = torch.Generator(device="cuda").manual_seed(seed)
    nids_size = start_size
    factors = []
    while len(factors) < valid_needed and nids_size <= num_rows:
        times = []
        for _ in range(10):
            total = torch.randint(0, num_rows, (nids_size,), generator=gen, device="cuda").unique().long()
            if option == "local":
                nids, _, _ = chunk_features._CAPI_split_index(total)
            else:
                nids = total
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            if option == "local":
                chunk_features._CAPI_local_index(nids)
            else:
                chunk_features._CAPI_host_index(nids)
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        fact_ms = 1e3 * sum(times[3:]) / len(times[3:])
        if fact_ms > valid_time_threshold_ms:
            ideal_ms = nids.numel() * row_elems * elem_bytes / 1e9 / bandwidth_gbps * 1e3
            factors.append(fact_ms / ideal_ms)
            log(f"{option}: {nids.numel()} rows, ideal {ideal_ms:.3f} ms, measured {fact_ms:.3f} ms, "
                f"{nids.numel() * row_elems * elem_bytes / fact_ms / 1e6:.1f} GB/s")
            nids_size = int(nids_size * 1.2)
        else:
            nids_size *= 10
    return sum(factors) / len(factors) if factors else float("nan")


def main(feature_size=20_000_000, feature_dim=128):
    """Upstream's __main__ (:104-125) at world size 1: [20M x 128] float32 rows."""
    ChunkTensor = torch.classes.dgs_classes.ChunkTensor
    for option, capacity, bw, thr in (("local", feature_size * feature_dim * 4, HBM_GBPS, 1.0),
                                      ("host", 0, PCIE_GBPS, 5.0)):
        ct = ChunkTensor([feature_size, feature_dim], torch.float32, capacity)
        dev, host = ct._CAPI_get_sub_device_tensor(), ct._CAPI_get_host_tensor()
        if dev.numel():
            dev.fill_(1.0)
        if host.numel():
            host.fill_(1.0)
        f = compute_loading_factor(ct, feature_size, feature_dim, 4, option, bw, thr)
        print(f"#GPU = 1, the penalty factor of {option} loading time = {f:.3f} (against {bw:.0f} GB/s)")
        del ct, dev, host


if __name__ == "__main__":
    import importlib
    importlib.import_module("dist-gpu-sampling_amd")
    main()
