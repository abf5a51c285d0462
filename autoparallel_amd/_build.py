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
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-ffp-contract=off",
    "-fPIC",
    "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
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
    print(build_abi_consumer(verbose=True))
