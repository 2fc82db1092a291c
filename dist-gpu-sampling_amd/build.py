"""Builds the two shared libraries of the package, in-tree, for gfx950.

libdgs_hip.so : the HIP kernels and their C ABI (include/dgs_hip.h); hipcc only.
libdgs.so     : the torch operator layer (torch.classes.dgs_classes /
                torch.ops.dgs_ops); plain g++ against the torch headers, linked
                to libdgs_hip.so.  No hipify pass is involved.

Run `python build.py` (or call build_all()) on a machine with hipcc; no GPU is
needed to compile.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
HIP_LIB = os.path.join(HERE, "libdgs_hip.so")
TORCH_LIB = os.path.join(HERE, "libdgs.so")
OBJ_DIR = os.path.join(HERE, "build")  # objects of the HIP sources (not tracked)

HIP_SOURCES = ["store.hip", "gather.hip", "sample.hip", "weighted.hip", "placement.hip", "unique.hip", "pipeline.hip"]
HIP_HEADERS = ["common.h", "table.h", "picks.h", "weights.h", "race.h", "sample_workspace.h"]
ARCH = "gfx950"


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def _stale(target, sources):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in sources)


def build_hip(force=True):
    """One object per source (compiled side by side: the sources are independent), then one link.
    Without `force` only the objects older than their source or a header are compiled again."""
    from concurrent.futures import ThreadPoolExecutor
    headers = [os.path.join(CSRC, h) for h in HIP_HEADERS] + [os.path.join(INCLUDE, "dgs_hip.h")]
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ_DIR, exist_ok=True)
    flags = ["-O3", "--offload-arch=" + ARCH, "-std=c++17", "-fPIC", "-fvisibility=hidden",
             # packed-FP32 instruction selection is switched off for every kernel in this library
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wall", "-Wextra", "-Wno-unused-command-line-argument", "-I" + INCLUDE]
    jobs = []
    objects = []
    for name in HIP_SOURCES:
        src = os.path.join(CSRC, name)
        obj = os.path.join(OBJ_DIR, name.replace(".hip", ".o"))
        objects.append(obj)
        if force or _stale(obj, [src] + headers):
            jobs.append([hipcc] + flags + ["-c", src, "-o", obj])
    if jobs:
        with ThreadPoolExecutor(max_workers=min(len(jobs), int(os.environ.get("MAX_JOBS", "8")))) as pool:
            list(pool.map(_run, jobs))
    if jobs or _stale(HIP_LIB, objects):
        _run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", HIP_LIB] + objects)
    return HIP_LIB


def build_torch(force=True):
    src = os.path.join(CSRC, "dgs_torch.cpp")
    if not force and not _stale(TORCH_LIB, [src, HIP_LIB, os.path.join(INCLUDE, "dgs_hip.h")]):
        return TORCH_LIB
    import torch
    tdir = os.path.dirname(torch.__file__)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    abi = "1" if torch._C._GLIBCXX_USE_CXX11_ABI else "0"
    _run([os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
          "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-D_GLIBCXX_USE_CXX11_ABI=" + abi,
          "-I" + INCLUDE, "-I" + os.path.join(tdir, "include"),
          "-I" + os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
          "-I" + os.path.join(rocm, "include"),
          "-o", TORCH_LIB, src,
          "-L" + HERE, "-ldgs_hip", "-L" + os.path.join(tdir, "lib"),
          "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch",
          "-Wl,-rpath,$ORIGIN", "-Wl,--no-undefined"])
    return TORCH_LIB


def build_all(force=True):
    build_hip(force)
    build_torch(force)
    return HIP_LIB, TORCH_LIB


if __name__ == "__main__":
    build_all(force="--if-stale" not in sys.argv)
