"""MI355X-native implementation of the per-GPU hot path of Dist-GPU-sampling:
row-wise neighbour sampling over CSC (uniform or weighted), first-occurrence
unique/relabel, the two-tier ChunkTensor row gather, and the hottest-rows-first
placement that feeds it.

Importing the package loads the two in-tree shared libraries:
  libdgs_hip.so  HIP kernels behind a C ABI (include/dgs_hip.h), bound in `capi`;
  libdgs.so      torch.classes.dgs_classes.ChunkTensor and torch.ops.dgs_ops.*,
                 the operator surface of the upstream library.
There is no CPU implementation: a missing library is an ImportError.
"""
import os

import torch  # noqa: F401  (must come first: it brings the HIP runtime the kernels share)

_HERE = os.path.dirname(os.path.abspath(__file__))
HIP_LIB = os.path.join(_HERE, "libdgs_hip.so")
TORCH_LIB = os.path.join(_HERE, "libdgs.so")

for _p in (HIP_LIB, TORCH_LIB):
    if not os.path.exists(_p):
        raise ImportError(
            f"{_p} is missing: build it with `python {os.path.join(_HERE, 'build.py')}` "
            "(there is no fallback implementation)")

from . import capi  # noqa: E402

torch.ops.load_library(TORCH_LIB)


_script_object_had_opt_out = "__torch_function__" in vars(torch.ScriptObject)


def lighten_torch_dispatch(enable=True):
    """Opt-in, process-wide: takes a per-argument cost of torch's Python front end off operators
    that run for 30 us.  Returns whether the shortcut is in place afterwards.

    For every operator argument that is not a tensor, torch asks
    `hasattr(arg, "__torch_function__")`.  On a custom-class object (torch.ScriptObject: every
    ChunkTensor, and every object of any other extension's custom classes) the miss goes through
    the class's `__getattr__` and two C++ exceptions: 5.4 us per argument per call, 11 us of a
    34 us `_CAPI_sample_neighbors_with_chunk_tensor`.  torch's own opt-out value for that
    protocol, set on the class, makes the lookup a hit that means "no override" (0.03 us).
    Because torch.ScriptObject is shared by all custom classes of the process, nothing here does
    this on import: a program calls lighten_torch_dispatch() if it wants it (bench.py does, and
    reports the per-hop operators both ways), lighten_torch_dispatch(False) takes it back, and
    DGS_LIGHT_TORCH_DISPATCH=1 in the environment asks for it at import.

    The package's own calls also skip `OpOverloadPacket.__call__` (a walk over the arguments in
    Python, 4 us a call) by calling the packets' C++ entries (sampler.fast_ops); that touches
    nothing of torch: `torch.ops.dgs_ops.<name>` stay the packets torch made, with their
    `.default` overloads and schemas."""
    if enable:
        if "__torch_function__" not in vars(torch.ScriptObject):
            torch.ScriptObject.__torch_function__ = torch._C._disabled_torch_function_impl
    elif not _script_object_had_opt_out and "__torch_function__" in vars(torch.ScriptObject):
        del torch.ScriptObject.__torch_function__
    return "__torch_function__" in vars(torch.ScriptObject)


if os.environ.get("DGS_LIGHT_TORCH_DISPATCH", "0") not in ("", "0"):
    lighten_torch_dispatch()

from .sampler import (  # noqa: E402
    BatchPipeline,
    ChunkTensorSampler,
    Block,
    PendingBatch,
    SeedLoader,
    cached_bytes_per_gpu,
    create_chunktensor,
    create_dgs_communicator,
    fast_ops,
    get_available_memory,
    pipeline_streams,
    set_gather_buffer_cap,
    set_rng_state,
    streams_overlap,
)

from . import placement  # noqa: E402
from . import loading_factor  # noqa: E402

ChunkTensor = torch.classes.dgs_classes.ChunkTensor
ops = torch.ops.dgs_ops

__all__ = ["capi", "placement", "loading_factor", "ops", "ChunkTensor", "ChunkTensorSampler", "BatchPipeline", "Block", "PendingBatch", "SeedLoader", "cached_bytes_per_gpu", "create_chunktensor",
           "create_dgs_communicator", "get_available_memory", "set_rng_state", "set_gather_buffer_cap", "pipeline_streams", "streams_overlap", "lighten_torch_dispatch", "fast_ops", "HIP_LIB", "TORCH_LIB"]
