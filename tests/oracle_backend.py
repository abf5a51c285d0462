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

    def upload_strategy_inputs(self, tables, tile_entries=None, dedupe=True, max_copies=16):
        # host-side tiling / de-duplication runs as in the product (the oracle ignores the tiles)
        tables.build_tiles(tile_entries, dedupe=dedupe, max_copies=max_copies)
        tables.validate(self.product_params)

    def launch_tables(self):
        enc = self.tables.as_dict()
        compute, per_arg = c_oracle.compute_costs(enc, self.params)
        self.out = c_oracle.build_tables(enc, self.params, per_arg=per_arg)
        self.out["compute"] = compute
        self.out["compute_per_arg"] = per_arg
        self.cost = self.out["cost"]
        self.launches = ("oracle",)

    def finish(self, n_vars, group_var_begin, group_member_begin, member_entry_begin):
        import numpy as np

        # variable of every entry from the group arrays, then the reference's accumulation
        # (numpy.bincount adds the weights one by one in input order, like the oracle's loop)
        sizes = np.diff(group_var_begin)
        var = np.full(len(self.cost), -1, np.int64)
        for g in range(len(sizes)):
            for m in range(int(group_member_begin[g]), int(group_member_begin[g + 1])):
                b = int(member_entry_begin[m])
                var[b:b + sizes[g]] = group_var_begin[g] + np.arange(sizes[g])
        assert (var >= 0).all()
        bad = ~np.isfinite(self.cost)
        obj = np.bincount(var, weights=np.where(bad, 10000.0, self.cost), minlength=n_vars)
        forced = np.bincount(var, weights=bad, minlength=n_vars) > 0
        return {"objective": obj, "forced_zero": forced, "compute": self.out["compute"],
                "compute_per_arg": self.out["compute_per_arg"]}

    def diffusion_sweeps(self, graph, theta, unary, n_sweeps):
        theta, unary = theta.copy(), unary.copy()
        po.diffusion_sweeps(n_sweeps, graph.label_begin, graph.inc_begin, graph.inc_edge, graph.inc_side,
                            graph.edge_begin, graph.edge_i, graph.edge_j, graph.color_begin, graph.color_nodes,
                            theta, unary)
        return theta, unary

    def host_array(self, name):
        return self.out[name]

    def gather(self, name, entries):
        return self.out[name][entries]

    def row_min(self, row_ptr):
        return c_oracle.segmented_min(self.cost, row_ptr)

    def greedy(self, row_ptr):
        import numpy as np

        mins, _ = c_oracle.segmented_min(self.cost, row_ptr)
        bound, node_min, node_arg, _ = po.greedy_strategies(self.tables.as_dict(), mins)
        return np.asarray(bound), np.asarray(node_min), np.asarray(node_arg)
