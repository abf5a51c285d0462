"""ctypes front-end of the plain-C oracle (oracle/cost_oracle.c).

TEST INFRASTRUCTURE: used by tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg only.  Takes the flattened tables as a dict of numpy arrays
(plain data) and the oracle's own CostParams.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

from .cost_oracle import CostParams

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcost_oracle.so")
_lib = None


class _Params(ctypes.Structure):
    _fields_ = [
        ("ndim", ctypes.c_int32),
        ("mesh", ctypes.c_int32 * 4),
        ("bw", ctypes.c_double * 4),
        ("lat", ctypes.c_double * 4),
        ("base_latency", ctypes.c_double),
        ("a2a_scale", ctypes.c_double),
        ("hbm_bw", ctypes.c_double),
        ("rw_eff", ctypes.c_double),
        ("launch_floor", ctypes.c_double),
        ("compute_eff", ctypes.c_double),
        ("rescale", ctypes.c_double),
        ("gpu_flops", ctypes.c_double * 8),
        ("transition_scale", ctypes.c_int32),
    ]


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "cost_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libcost_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_compute_costs.restype = ctypes.c_int
    return _lib


def _cparams(p: CostParams) -> _Params:
    cp = _Params()
    cp.ndim = p.ndim
    for i in range(p.ndim):
        cp.mesh[i] = p.mesh_sizes[i]
        cp.bw[i] = p.bw[i]
        cp.lat[i] = p.lat[i]
    cp.base_latency = p.base_latency
    cp.a2a_scale = p.a2a_scale
    cp.hbm_bw = p.hbm_bw
    cp.rw_eff = p.rw_eff
    cp.launch_floor = p.launch_floor
    cp.compute_eff = p.compute_eff
    cp.rescale = p.rescale
    for i, g in enumerate(p.gpu_flops):
        cp.gpu_flops[i] = g
    cp.transition_scale = p.transition_scale
    return cp


def _ptr(a: np.ndarray, dtype):
    assert a.dtype == np.dtype(dtype) and a.flags["C_CONTIGUOUS"], (a.dtype, dtype)
    return a.ctypes.data_as(ctypes.c_void_p)


def _arr(enc, key, dtype):
    return np.ascontiguousarray(np.asarray(enc[key], dtype=dtype))


def compute_costs(enc: dict, p: CostParams):
    n = len(enc["strat_flops"])
    flops = _arr(enc, "strat_flops", np.int64)
    rw = _arr(enc, "strat_rw_bytes", np.int64)
    dt = _arr(enc, "strat_dtype", np.int8)
    zc = _arr(enc, "strat_zero_cost", np.uint8)
    na = _arr(enc, "strat_num_args", np.int32)
    compute = np.empty(n, np.float64)
    per_arg = np.empty(n, np.float64)
    cp = _cparams(p)
    rc = lib().orc_compute_costs(ctypes.byref(cp), ctypes.c_int64(n), _ptr(flops, np.int64), _ptr(rw, np.int64),
                                 _ptr(dt, np.int8), _ptr(zc, np.uint8), _ptr(na, np.int32),
                                 _ptr(compute, np.float64), _ptr(per_arg, np.float64))
    if rc != 0:
        raise ValueError("dtype not supported on this device row")
    return compute, per_arg


def build_tables(enc: dict, p: CostParams, edge_range=None, per_arg=None):
    if per_arg is None:
        _, per_arg = compute_costs(enc, p)
    eb = _arr(enc, "edge_entry_begin", np.int64)
    n_edges = len(enc["edge_n_src"])
    lo, hi = (0, n_edges) if edge_range is None else edge_range
    n_entries = int(eb[hi] - eb[lo])
    comm = np.empty(n_entries, np.float64)
    trans = np.empty(n_entries, np.uint8)
    cost = np.empty(n_entries, np.float64)
    cp = _cparams(p)
    a = {
        "t_rank": _arr(enc, "tensor_rank", np.int32),
        "t_item": _arr(enc, "tensor_itemsize", np.int32),
        "t_shape": _arr(enc, "tensor_shape", np.int64),
        "t_stride": _arr(enc, "tensor_stride", np.int64),
        "s_codes": _arr(enc, "spec_codes", np.uint32),
        "s_tensor": _arr(enc, "spec_tensor", np.int32),
        "e_sb": _arr(enc, "edge_src_begin", np.int32),
        "e_ns": _arr(enc, "edge_n_src", np.int32),
        "e_tb": _arr(enc, "edge_tgt_begin", np.int32),
        "e_nt": _arr(enc, "edge_n_tgt", np.int32),
        "e_fl": _arr(enc, "edge_flags", np.int32),
        "e_pt": _arr(enc, "edge_pt_begin", np.int64),
        "e_st": _arr(enc, "edge_strat_begin", np.int32),
        "pt": _arr(enc, "pt_values", np.float64),
    }
    per_arg = np.ascontiguousarray(per_arg, dtype=np.float64)
    lib().orc_build_tables(
        ctypes.byref(cp), _ptr(a["t_rank"], np.int32), _ptr(a["t_item"], np.int32),
        _ptr(a["t_shape"], np.int64), _ptr(a["t_stride"], np.int64), _ptr(a["s_codes"], np.uint32),
        _ptr(a["s_tensor"], np.int32), _ptr(a["e_sb"], np.int32), _ptr(a["e_ns"], np.int32),
        _ptr(a["e_tb"], np.int32), _ptr(a["e_nt"], np.int32), _ptr(a["e_fl"], np.int32),
        _ptr(a["e_pt"], np.int64), _ptr(eb, np.int64), _ptr(a["e_st"], np.int32),
        _ptr(a["pt"], np.float64), _ptr(per_arg, np.float64), ctypes.c_int64(lo), ctypes.c_int64(hi),
        _ptr(comm, np.float64), _ptr(trans, np.uint8), _ptr(cost, np.float64))
    return {"comm": comm, "transition": trans, "cost": cost}


def tensor_tables(enc: dict):
    n = len(enc["tensor_rank"])
    out_b = np.empty(n, np.int64)
    out_c = np.empty(n, np.uint8)
    lib().orc_tensor_tables(ctypes.c_int64(n), _ptr(_arr(enc, "tensor_rank", np.int32), np.int32),
                            _ptr(_arr(enc, "tensor_itemsize", np.int32), np.int32),
                            _ptr(_arr(enc, "tensor_shape", np.int64), np.int64),
                            _ptr(_arr(enc, "tensor_stride", np.int64), np.int64),
                            _ptr(out_b, np.int64), _ptr(out_c, np.uint8))
    return out_b, out_c


def spec_tables(enc: dict, mesh_sizes):
    n = len(enc["spec_codes"])
    mesh = np.asarray(mesh_sizes, np.int32)
    shards = np.empty(n, np.int64)
    lshape = np.empty((n, 8), np.int64)
    lstride = np.empty((n, 8), np.int64)
    lnumel = np.empty(n, np.int64)
    lbytes = np.empty(n, np.int64)
    lib().orc_spec_tables(ctypes.c_int(len(mesh)), _ptr(mesh, np.int32), ctypes.c_int64(n),
                          _ptr(_arr(enc, "spec_codes", np.uint32), np.uint32),
                          _ptr(_arr(enc, "spec_tensor", np.int32), np.int32),
                          _ptr(_arr(enc, "tensor_rank", np.int32), np.int32),
                          _ptr(_arr(enc, "tensor_itemsize", np.int32), np.int32),
                          _ptr(_arr(enc, "tensor_shape", np.int64), np.int64),
                          _ptr(_arr(enc, "tensor_stride", np.int64), np.int64),
                          _ptr(shards, np.int64), _ptr(lshape, np.int64), _ptr(lstride, np.int64),
                          _ptr(lnumel, np.int64), _ptr(lbytes, np.int64))
    return shards, lshape, lstride, lnumel, lbytes


def segmented_min(values, seg_ptr):
    values = np.ascontiguousarray(values, np.float64)
    seg_ptr = np.ascontiguousarray(seg_ptr, np.int64)
    n = len(seg_ptr) - 1
    mins = np.empty(n, np.float64)
    args = np.empty(n, np.int32)
    lib().orc_segmented_min(_ptr(values, np.float64), _ptr(seg_ptr, np.int64), ctypes.c_int64(n),
                            _ptr(mins, np.float64), _ptr(args, np.int32))
    return mins, args
