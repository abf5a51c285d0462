"""MI355X-native sharding-cost evaluation for AutoParallel-style planners.

Public pieces:
  CostModelParams      explicit cost-model parameters (mesh topology, device row)
  CostTables           flattened strategy / placement encoding (numpy, host)
  DeviceCostTables     the encoding resident in HBM + the HIP kernels over it
  stress_dag           seeded synthetic strategy graph
"""

from .cost_model import CostModelParams, DEVICE_LIMITS, DeviceLimit, get_device_limit, mesh_topology
from .encoding import CostTables

__all__ = [
    "CostModelParams", "CostTables", "DEVICE_LIMITS", "DeviceLimit", "get_device_limit", "mesh_topology",
]
