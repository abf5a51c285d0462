"""Builds libapcost.so (the C-ABI HIP library) in-tree for gfx950."""

from __future__ import annotations

import os
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG)
# APCOST_LIBRARY names another build of the same sources (a debug or instrumented one)
LIB_PATH = os.environ.get("APCOST_LIBRARY") or os.path.join(_PKG, "libapcost.so")
SOURCES = [os.path.join(_PKG, "csrc", "apcost.hip")]
INCLUDE = os.path.join(_ROOT, "include")

# -ffp-contract=off: one IEEE rounding per fp64 operation (bit-identical to the
#   Python reference arithmetic).
# packed-fp32-ops off: keep the compiler from emitting packed fp32 instructions.
# amdgpu-kernarg-preload-count: see below (Llama-3-8B table pass 13.15 -> 12.6 us per launch).
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-ffp-contract=off",
    "-fPIC",
    "-shared",
    # (the torch layer names the library by this soname: whichever build of it is in the process
    # first, APCOST_LIBRARY's included, serves both bindings)
    "-Wl,-soname,libapcost.so",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first kernel arguments (a tile kernel's: tile records, counts) arrive in registers with
    # the wavefront instead of through a load that its first dependent load has to wait for
    "-mllvm", "-amdgpu-kernarg-preload-count=8",
]


def build_library(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, f"-I{INCLUDE}", "-o", LIB_PATH, *SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; harmless.
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err)
    return LIB_PATH


TORCH_EXT_SOURCE = os.path.join(_PKG, "csrc", "apcost_torch.cpp")
TORCH_EXT_PATH = os.path.join(_PKG, "libapcost_torch.so")


def build_torch_extension(verbose: bool = False) -> str:
    """The torch layer over the C ABI (operators of the ``apcost`` namespace), compiled against
    the installed torch and linked to libapcost.so beside it.  Host code only."""
    import torch
    from torch.utils import cpp_extension

    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    includes = [f"-I{d}" for d in cpp_extension.include_paths("cuda")]
    cmd = [hipcc, "-x", "c++", "-std=c++17", "-O2", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", *includes, f"-I{INCLUDE}",
           "-o", TORCH_EXT_PATH, TORCH_EXT_SOURCE, f"-L{_PKG}", "-lapcost", f"-L{torch_lib}", "-lc10", "-lc10_hip",
           "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{proc.stderr}")
    return TORCH_EXT_PATH


ABI_CONSUMER_SOURCE = os.path.join(_ROOT, "tests", "abi_consumer.cpp")
ABI_CONSUMER_PATH = os.path.join(_ROOT, "tests", "abi_consumer")


def build_abi_consumer(verbose: bool = False) -> str:
    """The C++ program that uses the library through include/apcost.h alone (no Python, no
    torch): proof that the boundary is a plain C ABI.  A GPU test runs it."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "--offload-arch=gfx950", "-O1", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           f"-I{INCLUDE}", "-o", ABI_CONSUMER_PATH,
           ABI_CONSUMER_SOURCE, f"-L{_PKG}", "-lapcost", "-Wl,-rpath,$ORIGIN/../autoparallel_amd"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    return ABI_CONSUMER_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_torch_extension(verbose=True))
    print(build_abi_consumer(verbose=True))
