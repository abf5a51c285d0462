import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")
    # load what is built; build only if nothing is
    from autoparallel_amd import _build

    if not os.path.exists(_build.LIB_PATH):
        _build.build_library()
    from oracle import c_oracle

    c_oracle.build()


@pytest.fixture(scope="session")
def fake_pg():
    """A 512-rank "fake" process group, as the reference's planner tests use
    (tests/test_optimize_placement.py:20-28): no devices, no communication."""
    import torch.distributed as dist
    from torch.testing._internal.distributed.fake_pg import FakeStore

    if not dist.is_initialized():
        dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=512)
    yield
    # left initialised for the whole session


@pytest.fixture(scope="session")
def torch_topo(fake_pg):
    """Builds torch's own MeshTopoInfo for a logical mesh with 8 devices per host."""
    from unittest.mock import patch

    from torch.distributed.device_mesh import _mesh_resources, init_device_mesh
    from torch.distributed.tensor._collective_utils import MeshTopoInfo

    cache = {}

    def make(mesh_sizes):
        mesh_sizes = tuple(mesh_sizes)
        if mesh_sizes not in cache:
            import warnings

            with warnings.catch_warnings():
                warnings.simplefilter("ignore")
                mesh = init_device_mesh("cpu", mesh_sizes)
            MeshTopoInfo.build_from_mesh.cache_clear()
            with patch.object(type(_mesh_resources), "num_devices_per_host", lambda self, device_type: 8):
                topo = MeshTopoInfo.build_from_mesh(mesh)
            MeshTopoInfo.build_from_mesh.cache_clear()
            cache[mesh_sizes] = (mesh, topo)
        return cache[mesh_sizes]

    return make


@pytest.fixture(scope="session")
def gpu_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    return torch.device("cuda:0")
