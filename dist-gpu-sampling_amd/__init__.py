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
