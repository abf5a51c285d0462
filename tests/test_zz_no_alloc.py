"""The entry point that allocates nothing (apc_redistribute_tables_static: staging tables in a
device array inside the library) against apc_input_tables + apc_redistribute_tables with
caller-allocated staging, through the C ABI: bit-identical outputs on two calls in a row, the
second on a smaller table (the array keeps the first call's contents).  Around the second call
the device's free memory is read from the HIP runtime itself (hipMemGetInfo sees a hipMalloc made
anywhere in the process, torch's counters only torch's own): it must not move."""

import ctypes

import numpy as np
import pytest
import torch

from autoparallel_amd import CostModelParams, _native
from autoparallel_amd.device_tables import DeviceCostTables
from autoparallel_amd.synthetic import stress_dag

pytestmark = pytest.mark.gpu


def _hip_runtime():
    """The HIP runtime this process has loaded (the one torch brought in), by its mapped path."""
    with open("/proc/self/maps") as f:
        paths = {line.split()[-1] for line in f if "libamdhip64" in line}
    assert len(paths) == 1, paths
    return ctypes.CDLL(paths.pop())


def _free_device_memory(hip):
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def _static_call(d, outputs, hip=None):
    tb = d.tables
    n = tb.n_entries
    out = {"comm": torch.full((n,), -1.0, dtype=torch.float64, device=d.device) if "comm" in outputs else None,
           "transition": torch.full((n,), 9, dtype=torch.uint8, device=d.device) if "transition" in outputs else None,
           "cost": torch.full((n,), -1.0, dtype=torch.float64, device=d.device) if "cost" in outputs else None}
    P = d._p
    with torch.cuda.device(d.device):
        torch.cuda.synchronize()
        free_before = _free_device_memory(hip) if hip is not None else None
        rc = d.lib.apc_redistribute_tables_static(
            ctypes.byref(d.c_params), ctypes.c_int64(tb.n_tensors), P("tensor_rank"), P("tensor_itemsize"),
            P("tensor_shape"), P("tensor_stride"), ctypes.c_int64(tb.n_strategies), P("strat_flops"), P("strat_rw_bytes"),
            P("strat_dtype"), P("strat_zero_cost"), P("strat_num_args"), P("spec_codes"), P("spec_tensor"), P("pt_values"),
            ctypes.c_int64(tb.n_tiles), P("tile_records"), P("dup_entry_begin"), ctypes.c_int64(n), P(out["comm"]),
            P(out["transition"]), P(out["cost"]), d._stream())
        if hip is not None:
            torch.cuda.synchronize()
            assert _free_device_memory(hip) == free_before, "the entry point changed the device's free memory"
    _native.check(rc, "apc_redistribute_tables_static")
    return out


def test_static_staging_matches_caller_allocated_staging(gpu_device):
    mesh = (16, 8, 4)
    p = CostModelParams.from_mesh(mesh, rescale=2.2)
    cases = [(stress_dag(seed=11, n_nodes=3000, mesh_sizes=mesh, frac_nonspec_nodes=0.03, frac_noncontiguous=0.2),
              ("comm", "transition", "cost")),
             (stress_dag(seed=12, n_nodes=400, mesh_sizes=mesh, frac_nonspec_nodes=0.03, frac_noncontiguous=0.3), ("cost",))]
    assert cases[1][0].n_strategies < cases[0][0].n_strategies and cases[1][0].n_tensors < cases[0][0].n_tensors
    hip = _hip_runtime()
    for i, (tb, outputs) in enumerate(cases):  # two calls in a row on the same device, the second on a smaller table
        d = DeviceCostTables(tb, p, device=gpu_device)
        step = d.prepare_step(row_min=False, fused_inputs=True, one_launch=False, outputs=outputs, spec_table=False)
        assert list(step) == ["input_tables", "redistribute_tables"]
        for launch in step.values():
            launch()
        torch.cuda.synchronize()
        want = {k: getattr(d, k) for k in outputs}
        got = _static_call(d, outputs, hip if i else None)  # (the first call loads the code object and looks the array up)
        torch.cuda.synchronize()
        for k in outputs:
            assert torch.equal(got[k], want[k]), k
        assert (want["cost"] > 0).any()
    # tables beyond the static staging are refused with a clear error, before anything is launched
    rc = d.lib.apc_redistribute_tables_static(
        ctypes.byref(d.c_params), ctypes.c_int64(1 << 17), *([None] * 4), ctypes.c_int64(10), *([None] * 5), None, None, None,
        ctypes.c_int64(0), None, None, ctypes.c_int64(0), None, None, None, None)
    assert rc != 0 and "static staging holds" in d.lib.apc_last_error().decode()
