"""The helper thread the planner's device work runs on: no dispatch mode of the caller is
active there, nested calls run in place, exceptions and results come back unchanged, the
caller's current stream is carried over."""

import threading

import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensor, FakeTensorMode

from autoparallel_amd import _device_thread
from autoparallel_amd._device_thread import call, on_device_thread


def test_caller_modes_are_not_active_on_the_device_thread():
    def make():
        t = torch.arange(4.0)
        return t, threading.current_thread().name

    with FakeTensorMode():
        assert isinstance(torch.arange(4.0), FakeTensor)
        t, name = call(make)
    assert not isinstance(t, FakeTensor) and t.sum().item() == 6.0
    assert name.startswith("apcost-device")


def test_nested_calls_run_in_place_and_one_thread_serves_all():
    seen = []

    @on_device_thread
    def inner():
        seen.append(threading.get_ident())
        return 7

    @on_device_thread
    def outer():
        seen.append(threading.get_ident())
        return inner() + 1  # would deadlock a one-worker pool if it were queued

    assert outer() == 8 and inner() == 7
    assert len(set(seen)) == 1 and seen[0] != threading.get_ident()
    assert seen[0] == _device_thread._worker_ident


def test_exceptions_come_back_to_the_caller():
    class Marker(Exception):
        pass

    def fail():
        raise Marker("from the device thread")

    with pytest.raises(Marker, match="from the device thread"):
        call(fail)
    assert call(lambda: 3) == 3  # the thread survives


def test_device_tables_fail_loudly_without_a_device():
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    from autoparallel_amd import CostModelParams
    from autoparallel_amd.device_tables import DeviceCostTables
    from autoparallel_amd.synthetic import stress_dag

    tables = stress_dag(seed=1, n_nodes=20, mesh_sizes=(2, 2))
    with pytest.raises(RuntimeError, match="no CPU path"):
        DeviceCostTables(tables, CostModelParams.from_mesh((2, 2)))


@pytest.mark.gpu
def test_real_tables_under_a_fake_tensor_mode_and_the_callers_stream():
    from autoparallel_amd import CostModelParams
    from autoparallel_amd.device_tables import DeviceCostTables
    from autoparallel_amd.synthetic import stress_dag

    tables = stress_dag(seed=5, n_nodes=300, mesh_sizes=(4, 2))
    params = CostModelParams.from_mesh((4, 2))
    plain = DeviceCostTables(tables, params)
    plain.build_all()
    want = plain.cost.cpu()
    side = torch.cuda.Stream()  # default priority
    with FakeTensorMode():
        dev = DeviceCostTables(tables, params)
        with torch.cuda.stream(side):
            dev.build_all()
            seen = call(lambda: torch.cuda.current_stream().cuda_stream)
        assert seen == side.cuda_stream
        assert not isinstance(dev.cost, FakeTensor)
    side.synchronize()
    assert torch.equal(dev.cost.cpu(), want)


def test_warm_up_returns_at_once_and_never_raises():
    """The planner starts the device's first-use costs before it captures the graph; without a
    device (or with one) the future completes with None and construction reports any problem."""
    from autoparallel_amd.optimize_sharding import DeviceBackend

    assert DeviceBackend.warm_up().result(timeout=120) is None


@pytest.mark.gpu
def test_tables_after_a_warm_up():
    from autoparallel_amd import CostModelParams
    from autoparallel_amd.device_tables import DeviceCostTables
    from autoparallel_amd.optimize_sharding import DeviceBackend
    from autoparallel_amd.synthetic import stress_dag

    DeviceBackend.warm_up()  # (not waited for: the construction below queues behind it)
    tables = stress_dag(seed=6, n_nodes=200, mesh_sizes=(4, 2))
    dev = DeviceCostTables(tables, CostModelParams.from_mesh((4, 2)))
    dev.build_all()
    assert torch.isfinite(dev.compute_cost).all()


def test_a_forked_child_starts_its_own_thread():
    """Covers a parent that has not initialised the GPU (every CPU run, and a GPU process that
    forks before its first device call): the child gets a worker of its own.  A parent that has
    initialised the GPU cannot have children that use it; that case is the next test."""
    import os

    import torch

    if torch.cuda.is_initialized():
        pytest.skip("this process has initialised the GPU: its forked children cannot use the device")
    assert call(lambda: 1) == 1  # the parent's thread exists
    r, w = os.pipe()
    pid = os.fork()
    if pid == 0:  # child: the parent's worker did not come along
        try:
            ok = call(lambda: threading.current_thread().name).startswith("apcost-device")
            os.write(w, b"1" if ok else b"0")
        finally:
            os._exit(0)
    os.close(w)
    import select

    ready, _, _ = select.select([r], [], [], 30)
    got = os.read(r, 1) if ready else b"timeout"
    os.close(r)
    if not ready:
        os.kill(pid, 9)
    os.waitpid(pid, 0)
    assert got == b"1"


def test_a_child_of_a_gpu_parent_is_told_so(monkeypatch):
    """torch refuses to initialise the GPU in a child forked after the parent did: the caller
    gets an error that names the situation and the way out."""
    import torch

    from autoparallel_amd import _device_thread

    def refuse():
        raise RuntimeError("Cannot re-initialize CUDA in forked subprocess. To use CUDA with multiprocessing, "
                           "you must use the 'spawn' start method")

    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    monkeypatch.setattr(torch.cuda, "current_stream", refuse)
    with pytest.raises(RuntimeError, match="forked from one that had initialised the GPU"):
        _device_thread._callers_stream()
    monkeypatch.setattr(torch.cuda, "current_stream", lambda: (_ for _ in ()).throw(RuntimeError("something else")))
    with pytest.raises(RuntimeError, match="something else"):
        _device_thread._callers_stream()
