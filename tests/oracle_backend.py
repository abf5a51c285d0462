"""Test-only table backend: the CPU oracle behind the planner's backend interface, so the
host logic (encoding, ILP) can be exercised without a GPU and so GPU-built tables can be
compared with oracle-built ones through the same solver.  Never used by the product."""


from oracle import c_oracle
from oracle import cost_oracle as po


class OracleBackend:
    def __init__(self, tables, params, device=None):
        self.tables = tables
        self.product_params = params
        self.params = po.make_params(params.mesh_sizes, device_name=params.device_name, rescale=params.rescale)
        assert self.params.bw == params.bw and self.params.lat == params.lat
        self.timings = {}

    def local_shapes(self):
        _, lshape, lstride, _, _ = c_oracle.spec_tables(self.tables.as_dict(), self.tables.mesh_sizes)
        return lshape, lstride

    def upload_strategy_inputs(self, tables, tile_entries=None, dedupe=True, max_copies=8):
        # host-side tiling / de-duplication runs as in the product (the oracle ignores the tiles)
        tables.build_tiles(tile_entries, dedupe=dedupe, max_copies=max_copies)
        tables.validate(self.product_params)

    def build(self):
        enc = self.tables.as_dict()
        compute, per_arg = c_oracle.compute_costs(enc, self.params)
        out = c_oracle.build_tables(enc, self.params, per_arg=per_arg)
        out["compute"] = compute
        out["compute_per_arg"] = per_arg
        self.cost = out["cost"]
        return out

    def row_min(self, row_ptr):
        return c_oracle.segmented_min(self.cost, row_ptr)

    def greedy(self, row_ptr):
        import numpy as np

        mins, _ = c_oracle.segmented_min(self.cost, row_ptr)
        bound, node_min, node_arg, _ = po.greedy_strategies(self.tables.as_dict(), mins)
        return np.asarray(bound), np.asarray(node_min), np.asarray(node_arg)
