"""Planning front-end: the part of the reference's ``AutoParallel`` context manager that
leads up to and includes ``optimize_placement`` (autoparallel/api.py:195-291, 385-445).
Applying the plan (re-tracing with collectives, compilation) is outside this package.

    with AutoParallelPlanner(model, input_fn, mesh, param_dtype=torch.bfloat16,
                             reduce_dtype=torch.float32) as autop:
        autop.add_parameter_memory_constraint(low=None, high=None)
        autop.add_input_constraints([...]); autop.add_output_constraints([...])
        placement = autop.optimize_placement()
"""

from __future__ import annotations

import logging
import time

from .graphs.capture import capture_joint_graph
from .optimize_sharding import ShardingOptimizer

logger = logging.getLogger(__name__)


class AutoParallelPlanner:
    optimizer_cls = ShardingOptimizer

    def __init__(self, model, input_fn, mesh, param_dtype=None, reduce_dtype=None, repeated_subgraphs=False,
                 device="cpu", dynamo=False):
        self.model = model
        self.input_fn = input_fn
        self.mesh = mesh
        self.param_dtype = param_dtype
        self.reduce_dtype = reduce_dtype
        self.repeated_subgraphs = repeated_subgraphs
        self.trace_device = device
        self.dynamo = dynamo  # capture the forward with Dynamo first: needed for local_map regions
        self.timings = {}
        self._ctx = None
        self.input_constraints = None
        self.output_constraints = None

    def __enter__(self):
        t0 = time.perf_counter()
        self._ctx = capture_joint_graph(self.model, self.input_fn, param_dtype=self.param_dtype,
                                        device=self.trace_device, dynamo=self.dynamo)
        self.gm, self.joint_with_descriptors = self._ctx.__enter__()
        self.timings["capture_s"] = time.perf_counter() - t0
        logger.info("%s %.3f s", "capture_s", self.timings["capture_s"])
        # api.py:264-272: gradients reduced in a wider dtype than the parameters cost more to
        # communicate; x1.1 breaks the tie towards reducing in the wider dtype
        rescale = 1.0
        if self.param_dtype is not None and self.reduce_dtype is not None:
            p, r = self.param_dtype.itemsize, self.reduce_dtype.itemsize
            if p != r:
                rescale = r / p * 1.1
        t0 = time.perf_counter()
        self.sharding_optimizer = self.optimizer_cls(self.gm, self.mesh, rescale,
                                                     repeated_subgraphs=self.repeated_subgraphs)
        self.sharding_optimizer.add_grad_param_constraints()
        self.timings["optimizer_s"] = time.perf_counter() - t0
        logger.info("%s %.3f s", "optimizer_s", self.timings["optimizer_s"])
        self.timings.update({f"optimizer_{k}": v for k, v in self.sharding_optimizer.timings.items()})
        return self

    def __exit__(self, *exc):
        return self._ctx.__exit__(*exc)

    def add_parameter_memory_constraint(self, low=None, high=None):
        if low is None:
            low = 0.0
        if high is None:
            high = 1.0 / self.mesh.size()
        assert low <= high, f"low should be <= high, got low{low}, high={high}"
        self.sharding_optimizer.add_parameter_memory_constraint(low, high)

    def add_input_constraints(self, constraints):
        assert self.input_constraints is None, "Input constraints have already been set"
        self.sharding_optimizer.add_sharded_input_constraint(constraints)
        self.input_constraints = constraints if constraints is not None else ()

    def add_output_constraints(self, constraints):
        assert self.output_constraints is None, "Output constraints have already been set"
        self.sharding_optimizer.add_sharded_output_constraint(constraints)
        self.output_constraints = constraints if constraints is not None else ()

    def optimize_placement(self, verbose=False):
        if self.input_constraints is None:
            self.add_input_constraints(None)
        if self.output_constraints is None:
            self.add_output_constraints(None)
        t0 = time.perf_counter()
        self.sharding_placement = self.sharding_optimizer.get_solution(verbose=False)
        self.timings["solve_s"] = time.perf_counter() - t0
        logger.info("%s %.3f s", "solve_s", self.timings["solve_s"])
        if verbose:
            print(self.sharding_optimizer.get_log())
        if self.sharding_optimizer.prob.status == -1:
            raise RuntimeError("Didn't find solution")
        return self.sharding_placement
