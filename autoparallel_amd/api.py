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

import torch

from .graphs.capture import capture_joint_graph
from .ilp import preload_solver
from .optimize_sharding import ShardingOptimizer

logger = logging.getLogger(__name__)


class AutoParallelPlanner:
    optimizer_cls = ShardingOptimizer
    active = False  # api.py:251-308: False before the with block, True inside, None after

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

    def _assert_entered(self):
        # api.py:300-308
        if self.active is False:
            raise RuntimeError("You must use AutoParallel as a context manager: with AutoParallel() as p: ...")
        if self.active is None:
            raise RuntimeError("AutoParallel is not reentrant, please file a bug report if you need this functionality")

    def __enter__(self):
        assert self.active is False
        # Capture and construction allocate millions of long-lived objects (graph nodes,
        # strategies, specs): the cyclic collector's passes over them find nothing worth the
        # time (5 % of the capture, and a pass over everything when it is switched on again).
        # It is paused here, and what exists when construction ends is moved out of its sight
        # (gc.freeze) until __exit__, so the solve's own collections stay short too.
        import gc

        collector_was_on = gc.isenabled()
        # An application that froze its own objects (a server after start-up) keeps its frozen
        # set: this planner then neither freezes nor, on exit, thaws.
        host_has_frozen = gc.get_freeze_count() != 0
        gc.disable()
        try:
            out = self._enter()
        except BaseException:
            # `with` does not call __exit__ after a failing __enter__: nothing may stay frozen,
            # and the capture context that was entered is left here
            if collector_was_on:
                gc.enable()
            ctx, self._ctx = self._ctx, None
            if ctx is not None and getattr(self, "gm", None) is not None:
                import sys

                try:
                    ctx.__exit__(*sys.exc_info())
                except Exception:  # (the failure being reported is the one that matters)
                    logger.debug("closing the capture context after a failed construction raised", exc_info=True)
            raise
        if not host_has_frozen:
            gc.freeze()
            self._frozen = True
        if collector_was_on:
            gc.enable()
        return out

    def _enter(self):
        # the device's first-use costs (a fifth of a second) overlap the capture
        warm_up = getattr(getattr(self.optimizer_cls, "backend_cls", None), "warm_up", None)
        if warm_up is not None:
            warm_up()
        preload_solver()  # likewise scipy's libraries, which the solve reads in otherwise
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
        self.active = True
        return self

    def __exit__(self, *exc):
        self.active = None
        if getattr(self, "_frozen", False):
            import gc

            self._frozen = False
            gc.unfreeze()  # (the collector sees everything again; cycles left by planning go at its next pass)
        ctx, self._ctx = self._ctx, None
        return ctx.__exit__(*exc) if ctx is not None else None

    def add_parameter_memory_constraint(self, low=None, high=None):
        self._assert_entered()
        if low is None:
            low = 0.0
        if high is None:
            high = 1.0 / self.mesh.size()
        assert low <= high, f"low should be <= high, got low{low}, high={high}"
        self.sharding_optimizer.add_parameter_memory_constraint(low, high)

    def add_input_constraints(self, constraints):
        self._assert_entered()
        assert self.input_constraints is None, "Input constraints have already been set"
        self.sharding_optimizer.add_sharded_input_constraint(constraints)
        self.input_constraints = constraints if constraints is not None else ()

    def add_output_constraints(self, constraints):
        self._assert_entered()
        assert self.output_constraints is None, "Output constraints have already been set"
        self.sharding_optimizer.add_sharded_output_constraint(constraints)
        self.output_constraints = constraints if constraints is not None else ()

    def optimize_placement(self, verbose=False):
        self._assert_entered()
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


class _ModelWithLoss(torch.nn.Module):
    """forward(*model_inputs, target) -> loss_fn(model(*model_inputs), target) (api.py:329-332)."""

    def __init__(self, model, loss_fn):
        super().__init__()
        self.model = model
        self.loss_fn = loss_fn

    def forward(self, *args):
        *model_inputs, target = args
        return self.loss_fn(self.model(*model_inputs), target)


class AutoParallel(AutoParallelPlanner):
    """The reference's entry point with its constructor (api.py:195-253), for the planning
    half of its life cycle: ``with AutoParallel(model, input_fn, mesh, mp_policy) as autop:``
    then the constraint methods and ``optimize_placement()``.  ``mp_policy`` is torch's
    ``MixedPrecisionPolicy`` (``reduce_dtype`` defaults to ``param_dtype`` as in
    cast_parametrization.py:116-125); ``repeated_subgraphs`` travels in ``**kwargs`` as in the
    reference.  The arguments that only matter once a plan is applied (``compile``,
    ``enable_ac``, ``ac_stage_size_in_GiB``, ``reshard_after_forward``) are kept as
    attributes; applying a plan is outside this package and ``apply_placement`` says so."""

    def __init__(self, model, input_fn, mesh, mp_policy=None, compile: bool = False, enable_ac: bool = True,
                 ac_stage_size_in_GiB="auto", reshard_after_forward: bool = True, dynamic: bool = False,
                 loss_fn=None, **kwargs):
        if dynamic:
            raise NotImplementedError("dynamic shapes are not planned by this package")
        param_dtype = reduce_dtype = None
        if mp_policy is not None:
            param_dtype = mp_policy.param_dtype
            reduce_dtype = mp_policy.reduce_dtype or param_dtype
        self.mp_policy = mp_policy
        self.kwargs = kwargs
        self.compile = compile
        self.enable_ac = enable_ac
        self.ac_stage_size_in_GiB = ac_stage_size_in_GiB
        self.reshard_after_forward = reshard_after_forward
        self.loss_fn = loss_fn
        if loss_fn is not None:
            user_input_fn = input_fn

            def input_fn():
                raw = user_input_fn()
                if not (isinstance(raw, tuple) and len(raw) == 2):
                    raise ValueError("When loss_fn is provided, input_fn must return (inputs, target) "
                                     "where inputs can be a single tensor or tuple of tensors")
                model_inputs, target = raw
                if not isinstance(model_inputs, tuple):
                    model_inputs = (model_inputs,)
                return (*model_inputs, target)

            model = _ModelWithLoss(model, loss_fn)
        super().__init__(model, input_fn, mesh, param_dtype=param_dtype, reduce_dtype=reduce_dtype,
                         repeated_subgraphs=kwargs.get("repeated_subgraphs", False),
                         dynamo=kwargs.get("dynamo", False))

    def optimize_placement(self, verbose=True):
        return super().optimize_placement(verbose=verbose)

    def apply_placement(self, sharding_placement=None):
        raise NotImplementedError("applying a plan (re-tracing with collectives, api.py:447-602) is outside this package: "
                                  "hand optimize_placement()'s result to the reference's apply_placement")
