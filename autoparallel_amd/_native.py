"""ctypes binding of libapcost.so (see include/apcost.h for the contract).

There is no CPU fallback: if the library has not been built, or a launch fails,
a RuntimeError is raised.
"""

from __future__ import annotations

import ctypes
import os

from ._build import LIB_PATH, TORCH_EXT_PATH

APC_ABI_VERSION = 3  # include/apcost.h: the interface this binding's structs and limits mirror
APC_MAX_RANK = 8
APC_MAX_MESH = 4
APC_MAX_DTYPES = 8
APC_TILE_MAX_COLS = 64
APC_TILE_MAX_ROWS = 64
APC_TILE_MAX_DUPS = 32
APC_PACKED_MAX_DUPS = 16

EDGE_GRAD_RESCALE = 1
EDGE_NO_PRODUCER = 2


class ApcParams(ctypes.Structure):
    _fields_ = [
        ("mesh_ndim", ctypes.c_int32),
        ("mesh_size", ctypes.c_int32 * APC_MAX_MESH),
        ("bw", ctypes.c_double * APC_MAX_MESH),
        ("lat", ctypes.c_double * APC_MAX_MESH),
        ("base_latency", ctypes.c_double),
        ("a2a_scale", ctypes.c_double),
        ("hbm_bw", ctypes.c_double),
        ("rw_eff", ctypes.c_double),
        ("launch_floor", ctypes.c_double),
        ("compute_eff", ctypes.c_double),
        ("rescale", ctypes.c_double),
        ("gpu_flops", ctypes.c_double * APC_MAX_DTYPES),
        ("transition_scale", ctypes.c_int32),
        ("inv_bw", ctypes.c_double * APC_MAX_MESH),
        ("inv_mesh", ctypes.c_double * APC_MAX_MESH),
        ("inv_hbm_bw", ctypes.c_double),
        ("inv_rw_eff", ctypes.c_double),
        ("inv_compute_eff", ctypes.c_double),
        ("inv_gpu_flops", ctypes.c_double * APC_MAX_DTYPES),
    ]


class ApcTile(ctypes.Structure):
    _fields_ = [
        ("edge", ctypes.c_int32), ("row_begin", ctypes.c_int32), ("col_begin", ctypes.c_int32),
        ("counts", ctypes.c_int32),
        ("src_begin", ctypes.c_int32), ("n_src", ctypes.c_int32), ("tgt_begin", ctypes.c_int32),
        ("flags", ctypes.c_int32), ("strat_begin", ctypes.c_int32), ("tensor", ctypes.c_int32),
        ("entry_begin", ctypes.c_int64), ("pt_begin", ctypes.c_int64),
        ("dup_begin", ctypes.c_int32), ("dup_count", ctypes.c_int32),
    ]


class ApcRowMinima(ctypes.Structure):
    _fields_ = [
        ("edge_row_begin", ctypes.c_void_p), ("dup_row_begin", ctypes.c_void_p),
        ("row_min", ctypes.c_void_p), ("row_argmin", ctypes.c_void_p),
    ]


EXPORTS = (
    "apc_version",
    "apc_last_error",
    "apc_validate_tables_host",
    "apc_tensor_tables",
    "apc_spec_tables",
    "apc_compute_costs",
    "apc_input_tables",
    "apc_redistribute_tables",
    "apc_build_tables",
    "apc_redistribute_tables_row_min",
    "apc_build_tables_row_min",
    "apc_segmented_min",
    "apc_segmented_min_copies",
    "apc_strategy_bounds",
    "apc_cost_objective",
    "apc_validate_row_minima_host",
    "apc_diffusion_sweeps",
    "apc_redistribute_tables_static",
    "apc_strategy_inputs",
    "apc_validate_packed_tiles_host",
    "apc_build_tables_packed",
    "apc_calibrate_launch",
    "apc_calibrate_fill",
)

_lib = None


def library_path() -> str:
    return LIB_PATH


def lib() -> ctypes.CDLL:
    """Loads the built library; raises if it is missing (build it with
    ``python -m autoparallel_amd._build`` or ``__graft_entry__.build()``)."""
    global _lib
    if _lib is None:
        # torch ships its own HIP runtime; it must be in the process before this library
        # is mapped so that both resolve to the same runtime (streams and device pointers
        # are shared between them).
        import torch  # noqa: F401

        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP library has not been built "
                "(run `python -m autoparallel_amd._build`). There is no CPU fallback."
            )
        l = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        for name in EXPORTS:
            if not hasattr(l, name):
                raise RuntimeError(f"{LIB_PATH} does not export {name}")
        l.apc_last_error.restype = ctypes.c_char_p
        l.apc_version.restype = ctypes.c_int
        if int(l.apc_version()) != APC_ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH} implements interface version {int(l.apc_version())}, this binding "
                               f"mirrors version {APC_ABI_VERSION} of include/apcost.h: rebuild the library")
        for name in EXPORTS:
            if name != "apc_last_error":
                getattr(l, name).restype = ctypes.c_int
        _lib = l
    return _lib


_ops = None


def torch_ops():
    """The ``apcost`` operator namespace of the torch layer (csrc/apcost_torch.cpp): operators
    over torch tensors on the HIP device, bound to the same library.  Raises if it has not
    been built."""
    global _ops
    if _ops is None:
        import torch

        lib()  # the C-ABI library first: the extension resolves its symbols against it
        if not os.path.exists(TORCH_EXT_PATH):
            raise RuntimeError(
                f"{TORCH_EXT_PATH} is missing: the torch layer has not been built "
                "(run `python -m autoparallel_amd._build`). There is no CPU fallback."
            )
        torch.ops.load_library(TORCH_EXT_PATH)
        _ops = torch.ops.apcost
        if int(_ops.abi_version()) != APC_ABI_VERSION or int(_ops.library_abi_version()) != APC_ABI_VERSION:
            raise RuntimeError(f"the torch layer was compiled against interface version {int(_ops.abi_version())} and "
                               f"sees a library of version {int(_ops.library_abi_version())}; this binding mirrors "
                               f"version {APC_ABI_VERSION}: rebuild both")
    return _ops


def params_tensor(c_params: "ApcParams"):
    """``struct apc_params`` as the CPU uint8 tensor the operators take."""
    import torch

    return torch.frombuffer(bytearray(bytes(c_params)), dtype=torch.uint8)


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().apc_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed ({rc}): {msg}")


def vp(ptr) -> ctypes.c_void_p:
    """int / None -> void*"""
    return ctypes.c_void_p(ptr if ptr else None)
