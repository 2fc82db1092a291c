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


def _lighten_torch_dispatch():
    """Takes two per-call costs of torch's Python front end off operators that run for 30 us.

    1. For every argument that is not a tensor, torch asks `hasattr(arg, "__torch_function__")`.
       On a custom-class object (torch.ScriptObject: every ChunkTensor) the miss goes through
       the class's `__getattr__` and two C++ exceptions: 5.4 us per argument per call, 11 us of a
       34 us `_CAPI_sample_neighbors_with_chunk_tensor`.  torch's own opt-out value for that
       protocol, set on the class, makes the lookup a hit that means "no override" (0.03 us).
    2. For operators with custom-class arguments, `OpOverloadPacket.__call__` first walks the
       arguments in Python looking for FakeScriptObjects (export/compile tracing; 4 us a call)
       and then calls the C++ entry `packet._op`.  The names in `torch.ops.dgs_ops` that take
       ChunkTensors are bound to that entry directly.  They remain callables with the same
       arguments, results and errors; what they lose is the tracing support, which these
       operators (blocking reads of data-dependent sizes) do not have anyway.

    Set DGS_PLAIN_TORCH_DISPATCH=1 to leave torch as it is."""
    if os.environ.get("DGS_PLAIN_TORCH_DISPATCH", "0") not in ("", "0"):
        return
    if "__torch_function__" not in vars(torch.ScriptObject):
        torch.ScriptObject.__torch_function__ = torch._C._disabled_torch_function_impl
    for name in ("_CAPI_sample_neighbors_with_chunk_tensor", "_CAPI_sample_neighbors_with_probs_with_chunk_tensor",
                 "_CAPI_sample_blocks", "_CAPI_sample_blocks_and_index", "_CAPI_sample_blocks_begin",
                 "_CAPI_sample_blocks_and_index_begin", "_CAPI_sample_blocks_weighted_begin",
                 "_CAPI_sample_blocks_submit"):
        entry = getattr(getattr(torch.ops.dgs_ops, name), "_op", None)
        if callable(entry):
            setattr(torch.ops.dgs_ops, name, entry)


_lighten_torch_dispatch()

from .sampler import (  # noqa: E402
    BatchPipeline,
    ChunkTensorSampler,
    Block,
    PendingBatch,
    create_chunktensor,
    create_dgs_communicator,
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

__all__ = ["capi", "placement", "loading_factor", "ops", "ChunkTensor", "ChunkTensorSampler", "BatchPipeline", "Block", "PendingBatch", "create_chunktensor",
           "create_dgs_communicator", "get_available_memory", "set_rng_state", "set_gather_buffer_cap", "pipeline_streams", "streams_overlap", "HIP_LIB", "TORCH_LIB"]
