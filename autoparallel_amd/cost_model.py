"""Cost-model parameters: what the reference reads implicitly from its environment
(torch ``MeshTopoInfo``, the ``DEVICE_LIMITS`` row selected by the CUDA device name,
module-level constants), collected into one explicit object that is handed to the
kernels by value.

Reference:
  torch/distributed/tensor/_collective_utils.py:246-278   (mesh bandwidth / latency)
  autoparallel/compute_estimation.py:63-203               (device rows and lookup)
  autoparallel/compute_estimation.py:307-309, 361         (0.70 efficiency, 7 us floor)
  autoparallel/collective_runtime_estimation.py:30-31     (all-to-all x5)
  autoparallel/optimize_sharding.py:298                   (transition scale 1)
"""

from __future__ import annotations

from dataclasses import dataclass, field

from ._native import APC_MAX_DTYPES, APC_MAX_MESH, ApcParams

# dtype name -> code used by the per-strategy compute-cost table
DTYPE_CODES = {"float64": 0, "float32": 1, "float16": 2, "bfloat16": 3, "int8": 4}


@dataclass(frozen=True)
class DeviceLimit:
    name: str
    gmem_bandwidth: float  # bytes / s
    gemm_tflops: dict  # dtype name -> TFLOP/s


# Datasheet rows of the reference's table (compute_estimation.py:63-166); the order is
# the lookup order (first row whose name is a substring of the device name wins).
DEVICE_LIMITS = (
    DeviceLimit("H100", 3.35 * (1024**4),
                {"float64": 67, "float32": 989 // 2, "float16": 1979 // 2, "bfloat16": 1979 // 2, "int8": 3958 // 2}),
    DeviceLimit("B200", 7.7 * (1024**4),
                {"float64": 37, "float32": 2200 // 2, "float16": 4500 // 2, "bfloat16": 4500 // 2, "int8": 9000 // 2}),
    DeviceLimit("A100", 2 * (1024**4),
                {"float64": 19.5, "float32": 156, "float16": 312, "bfloat16": 312, "int8": 624}),
    DeviceLimit("A30", 933 * (1024**3),
                {"float64": 10.3, "float32": 82, "float16": 165, "bfloat16": 165, "int8": 330}),
    DeviceLimit("A10G", 933 * (1024**3), {"float32": 31.2, "float16": 125, "bfloat16": 125, "int8": 250}),
    DeviceLimit("T4", 300 * (1024**3), {"float32": 8.1, "float16": 65, "int8": 130}),
    DeviceLimit("V100", 900 * (1024**3), {"float64": 7.8, "float32": 15.7, "float16": 125}),
    DeviceLimit("P100", 732 * (1024**3), {"float64": 5.3, "float32": 10.6, "float16": 21.2}),
)

# Not a reference row: lets the planner model the machine it runs on.  Dense peaks
# (no sparsity); HBM3E 8 TB/s.  Never used for parity.
MI355X_LIMIT = DeviceLimit(
    "MI355X", 8.0e12,
    {"float64": 78.6, "float32": 157.3, "float16": 2500, "bfloat16": 2500, "int8": 5000})


def get_device_limit(device_name: str, extra_rows=()) -> DeviceLimit:
    """compute_estimation.py:169-186: substring match in table order, ValueError otherwise."""
    for limit in tuple(extra_rows) + DEVICE_LIMITS:
        if limit.name in device_name or (limit.name == "A100" and "PG509" in device_name):
            return limit
    raise ValueError(
        f"Unsupported device: {device_name}. Supported devices: {[limit.name for limit in DEVICE_LIMITS]}"
    )


def mesh_topology(mesh_sizes, devices_per_host=8, base_bw=87.7, inter_host_factor=0.22,
                  intra_latency=0.6, inter_latency=2.7):
    """Per-mesh-dim bandwidth (GB/s) and hop latency (us).

    torch _collective_utils.py:246-278: dims are visited innermost first; once the
    running device product exceeds one host the dim is inter-host.
    """
    ndim = len(mesh_sizes)
    bw = [base_bw] * ndim
    lat = [intra_latency] * ndim
    total = 1
    for d in reversed(range(ndim)):
        total *= int(mesh_sizes[d])
        if total > devices_per_host:
            bw[d] *= inter_host_factor
            lat[d] = inter_latency
    return tuple(bw), tuple(lat)


@dataclass
class CostModelParams:
    mesh_sizes: tuple
    bw: tuple
    lat: tuple
    hbm_bw: float
    gpu_flops: tuple  # per dtype code, tflops * 10**12; 0.0 = dtype unsupported
    device_name: str = "H100"
    base_latency: float = 6.6
    a2a_scale: float = 5.0
    rw_eff: float = 0.70
    launch_floor: float = 7.0
    compute_eff: float = 0.70
    rescale: float = 1.0
    transition_scale: int = 1
    inf_replacement_cost: float = 10000.0  # optimize_sharding.py:531-533
    extras: dict = field(default_factory=dict)

    @property
    def ndim(self) -> int:
        return len(self.mesh_sizes)

    @classmethod
    def from_mesh(cls, mesh_sizes, device_name="H100", devices_per_host=8, rescale=1.0, extra_rows=()):
        """The parity preset is the reference tests' environment: 8 devices per host
        and the "H100" device row (tests/test_optimize_placement.py:141-142)."""
        mesh_sizes = tuple(int(x) for x in mesh_sizes)
        if not 1 <= len(mesh_sizes) <= APC_MAX_MESH:
            raise ValueError(f"mesh ndim {len(mesh_sizes)} outside [1, {APC_MAX_MESH}]")
        bw, lat = mesh_topology(mesh_sizes, devices_per_host)
        limit = get_device_limit(device_name, extra_rows)
        gf = [0.0] * APC_MAX_DTYPES
        for name, code in DTYPE_CODES.items():
            if name in limit.gemm_tflops:
                gf[code] = float(limit.gemm_tflops[name] * 10**12)  # compute_estimation.py:356
        return cls(mesh_sizes, bw, lat, float(limit.gmem_bandwidth), tuple(gf), device_name=limit.name,
                   rescale=float(rescale))

    def to_c(self) -> ApcParams:
        c = ApcParams()
        c.mesh_ndim = self.ndim
        for i in range(self.ndim):
            c.mesh_size[i] = self.mesh_sizes[i]
            c.bw[i] = self.bw[i]
            c.lat[i] = self.lat[i]
        c.base_latency = self.base_latency
        c.a2a_scale = self.a2a_scale
        c.hbm_bw = self.hbm_bw
        c.rw_eff = self.rw_eff
        c.launch_floor = self.launch_floor
        c.compute_eff = self.compute_eff
        c.rescale = self.rescale
        for i, g in enumerate(self.gpu_flops):
            c.gpu_flops[i] = g
        c.transition_scale = self.transition_scale
        # reciprocals the kernels divide through (the library checks them)
        for i in range(self.ndim):
            c.inv_bw[i] = 1.0 / self.bw[i]
            c.inv_mesh[i] = 1.0 / float(self.mesh_sizes[i])
        c.inv_hbm_bw = 1.0 / self.hbm_bw
        c.inv_rw_eff = 1.0 / self.rw_eff
        c.inv_compute_eff = 1.0 / self.compute_eff
        for i, g in enumerate(self.gpu_flops):
            c.inv_gpu_flops[i] = 1.0 / g if g else 0.0
        return c
