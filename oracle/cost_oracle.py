"""Scalar pure-Python restatement of the reference's sharding-cost formulas.

TEST INFRASTRUCTURE (see oracle/__init__.py): imported only by tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg.

Every function names the reference lines it follows.  ``ref:`` paths are
relative to the reference checkout, ``torch:`` paths relative to the installed
torch package (the third-party dependency that holds part of the arithmetic).

All floating point is CPython ``float`` (IEEE binary64), evaluated in the same
operation order as the reference so results are bit-identical to it.

Placement codes (one unsigned byte per mesh dim; the same contract the device
tables use):
    0x00            Replicate
    0x40 | op       Partial(op)      op 0 = "sum"; other reduce ops 1..63
    0x80 | v<<4 | d Shard(d)         d = tensor dim 0..15, v = variant id
                                      (0 = plain Shard; >0 = interned
                                      _StridedShard flavours, equal only to
                                      themselves)
A spec's placements are packed little-endian into a uint32 (byte i = mesh dim i).
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Sequence

REPLICATE = 0x00
PARTIAL_SUM = 0x40
KIND_R, KIND_P, KIND_S = 0, 1, 2
MAX_RANK = 8
MAX_MESH = 4

# edge flags
EDGE_GRAD_RESCALE = 1  # consumer is a parameter-gradient node
EDGE_NO_PRODUCER = 2  # placeholder / factory pseudo-argument: rule-provided costs kept


def shard(dim: int, variant: int = 0) -> int:
    return 0x80 | (variant << 4) | dim


def partial(op: int = 0) -> int:
    return 0x40 | op


def kind(code: int) -> int:
    return code >> 6


def shard_dim(code: int) -> int:
    return code & 0x0F


def pack_codes(codes: Sequence[int]) -> int:
    out = 0
    for i, c in enumerate(codes):
        out |= (c & 0xFF) << (8 * i)
    return out


def unpack_codes(packed: int, ndim: int) -> tuple[int, ...]:
    return tuple((packed >> (8 * i)) & 0xFF for i in range(ndim))


# --------------------------------------------------------------------------------------
# device rows  (ref: autoparallel/compute_estimation.py:63-166)
# name -> (hbm bytes/s, {dtype name: tflops}); order matters for substring matching.
# --------------------------------------------------------------------------------------
DEVICE_LIMITS = (
    ("H100", 3.35 * (1024**4), {"float64": 67, "float32": 989 // 2, "float16": 1979 // 2, "bfloat16": 1979 // 2, "int8": 3958 // 2}),
    ("B200", 7.7 * (1024**4), {"float64": 37, "float32": 2200 // 2, "float16": 4500 // 2, "bfloat16": 4500 // 2, "int8": 9000 // 2}),
    ("A100", 2 * (1024**4), {"float64": 19.5, "float32": 156, "float16": 312, "bfloat16": 312, "int8": 624}),
    ("A30", 933 * (1024**3), {"float64": 10.3, "float32": 82, "float16": 165, "bfloat16": 165, "int8": 330}),
    ("A10G", 933 * (1024**3), {"float32": 31.2, "float16": 125, "bfloat16": 125, "int8": 250}),
    ("T4", 300 * (1024**3), {"float32": 8.1, "float16": 65, "int8": 130}),
    ("V100", 900 * (1024**3), {"float64": 7.8, "float32": 15.7, "float16": 125}),
    ("P100", 732 * (1024**3), {"float64": 5.3, "float32": 10.6, "float16": 21.2}),
)

# dtype codes used by the per-strategy compute-cost table
DTYPE_CODES = {"float64": 0, "float32": 1, "float16": 2, "bfloat16": 3, "int8": 4}
NUM_DTYPE_CODES = 5


def device_limit(device_name: str):
    """ref: compute_estimation.py:169-186 (first row whose name is a substring)."""
    for name, bw, tflops in DEVICE_LIMITS:
        if name in device_name or (name == "A100" and "PG509" in device_name):
            return name, bw, tflops
    raise ValueError(
        f"Unsupported device: {device_name}. Supported devices: {[r[0] for r in DEVICE_LIMITS]}"
    )


def device_tflops(device_name: str, dtype_name: str):
    """ref: compute_estimation.py:189-203."""
    name, _, tflops = device_limit(device_name)
    if dtype_name not in tflops:
        raise ValueError(
            f"Dtype {dtype_name} not supported on {name}. Supported dtypes: {list(tflops.keys())}"
        )
    return tflops[dtype_name]


@dataclass
class CostParams:
    """Everything the reference reads implicitly from its environment, made explicit."""

    mesh_sizes: tuple[int, ...]
    bw: tuple[float, ...]
    lat: tuple[float, ...]
    hbm_bw: float
    # gpu_flops[dtype code] = tflops * 10**12 (0.0 = dtype unsupported on this row)
    gpu_flops: tuple[float, ...]
    base_latency: float = 6.6
    a2a_scale: float = 5
    rw_eff: float = 0.70
    launch_floor: float = 7
    compute_eff: float = 0.70
    rescale: float = 1.0
    transition_scale: int = 1
    extras: dict = field(default_factory=dict)

    @property
    def ndim(self) -> int:
        return len(self.mesh_sizes)


def mesh_topology(mesh_sizes, devices_per_host=8, base_bw=87.7, inter_factor=0.22,
                  intra_lat=0.6, inter_lat=2.7):
    """torch: distributed/tensor/_collective_utils.py:246-278 (MeshTopoInfo.build_from_mesh).

    Walks mesh dims innermost-first; a dim whose cumulative device product exceeds the
    devices of one host is inter-host: bandwidth scaled by 0.22, latency 2.7 us.
    """
    ndim = len(mesh_sizes)
    bw = [base_bw] * ndim
    lat = [intra_lat] * ndim
    total = 1
    for d in reversed(range(ndim)):
        total *= mesh_sizes[d]
        if total > devices_per_host:
            bw[d] *= inter_factor
            lat[d] = inter_lat
    return tuple(int(x) for x in mesh_sizes), tuple(bw), tuple(lat)


def make_params(mesh_sizes, device_name="H100", devices_per_host=8, rescale=1.0) -> CostParams:
    n, bw, lat = mesh_topology(mesh_sizes, devices_per_host)
    _, hbm, tflops = device_limit(device_name)
    gf = [0.0] * 8
    for name, code in DTYPE_CODES.items():
        if name in tflops:
            # ref: compute_estimation.py:356  gpu_flops = tflops * 10**12
            gf[code] = float(tflops[name] * 10**12)
    return CostParams(n, bw, lat, hbm, tuple(gf), rescale=rescale)


# --------------------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------------------
def read_write_time(read_write_bytes, p: CostParams) -> float:
    """ref: compute_estimation.py:302-314 (compute_read_write_time)."""
    t = read_write_bytes / p.hbm_bw * 1e6
    return max(t / p.rw_eff, p.launch_floor)


def _ring(bytes_gb: float, p: CostParams, mesh_dim: int, num_hops: int) -> float:
    n = p.mesh_sizes[mesh_dim]
    latency = p.base_latency + num_hops * p.lat[mesh_dim]
    bw = (bytes_gb * num_hops / n) / p.bw[mesh_dim]
    return latency + bw * 1e6


def allgather_cost(bytes_gb, p, mesh_dim) -> float:
    """torch: distributed/tensor/_collective_utils.py:281-288."""
    return _ring(bytes_gb, p, mesh_dim, p.mesh_sizes[mesh_dim] - 1)


def allreduce_cost(bytes_gb, p, mesh_dim) -> float:
    """torch: distributed/tensor/_collective_utils.py:291-299."""
    return _ring(bytes_gb, p, mesh_dim, 2 * (p.mesh_sizes[mesh_dim] - 1))


def reduce_scatter_cost(bytes_gb, p, mesh_dim) -> float:
    """torch: distributed/tensor/_collective_utils.py:302-313."""
    return _ring(bytes_gb, p, mesh_dim, p.mesh_sizes[mesh_dim] - 1)


def all_to_all_cost(bytes_gb, p, mesh_dim) -> float:
    """ref: collective_runtime_estimation.py:22-32."""
    total_time = _ring(bytes_gb, p, mesh_dim, p.mesh_sizes[mesh_dim] - 1)
    total_time *= p.a2a_scale
    return total_time


def is_contiguous(shape, stride) -> bool:
    """torch: _prims_common/__init__.py:252-292 (check_contiguous_sizes_strides), concrete ints."""
    expected = 1
    expected_max = 1
    for x, y in reversed(tuple(zip(shape, stride))):
        if x == 1:
            continue
        if y != expected and y != expected_max:
            return False
        expected_max *= max(x, 1)
        expected *= x
    return True


def tensor_bytes(itemsize: int, shape) -> int:
    """torch: distributed/tensor/_collective_utils.py:230-232 (spec_to_bytes)."""
    return itemsize * math.prod(shape)


def num_shards(codes, mesh_sizes) -> int:
    """torch: distributed/tensor/_dtensor_spec.py:555-561 (Partial does not count)."""
    out = 1
    for c, n in zip(codes, mesh_sizes):
        if kind(c) == KIND_S:
            out *= n
    return out


def sharded_shape_stride(shape, stride, codes, mesh_sizes):
    """ref: compute_estimation.py:211-229 (_get_sharded_shape_stride).

    Ceil-div of the sharded dim; the stride of dim-1 is ceil-divided only when
    dim-1 > 0 (the reference's own quirk, kept).
    """
    new_shape = list(shape)
    new_stride = list(stride)
    for n, c in zip(mesh_sizes, codes):
        if kind(c) == KIND_S:
            d = shard_dim(c)
            new_shape[d] = (new_shape[d] + n - 1) // n
            if d - 1 > 0:
                new_stride[d - 1] = (new_stride[d - 1] + n - 1) // n
    return new_shape, new_stride


# --------------------------------------------------------------------------------------
# one redistribution-cost entry
# --------------------------------------------------------------------------------------
def redistribute_cost(src, tgt, shape, stride, itemsize, p: CostParams, order) -> float:
    """ref: collective_runtime_estimation.py:37-143 (single mesh: the mesh-mismatch
    branch :51-54 cannot occur in this encoding)."""
    if all(c == REPLICATE for c in src):  # :56-62
        if any(kind(t) == KIND_P for t in tgt):
            return math.inf
        return 0.0

    cost = 0.0
    comm_bytes_gb = tensor_bytes(itemsize, shape) / num_shards(src, p.mesh_sizes) / 1024 / 1024 / 1024
    contiguous = is_contiguous(shape, stride)  # :74-76, GLOBAL shape/stride
    for i in order:
        current, target = src[i], tgt[i]
        if current == target:
            continue
        n = p.mesh_sizes[i]
        if not contiguous:
            cost += read_write_time(comm_bytes_gb * 2 * 1024**3, p)
        ck, tk = kind(current), kind(target)
        if ck == KIND_S and tk == KIND_R:  # :83-96
            comm_bytes_gb *= n
            cost += allgather_cost(comm_bytes_gb, p, i)
            if shard_dim(current) != 0:
                cost += read_write_time(comm_bytes_gb * 2 * 1024**3, p)
        elif ck == KIND_S and tk == KIND_S:  # :97-113
            cost += all_to_all_cost(comm_bytes_gb, p, i)
            num_copies = 0
            if shard_dim(current) != 0:
                num_copies += 1
            if shard_dim(target) != 0:
                num_copies += 1
            cost += num_copies * read_write_time(comm_bytes_gb * 2 * 1024**3, p)
        elif ck == KIND_P and tk == KIND_R:  # :115-117
            cost += allreduce_cost(comm_bytes_gb, p, i)
        elif ck == KIND_P and tk == KIND_S:  # :118-130
            cost += reduce_scatter_cost(comm_bytes_gb, p, i)
            if shard_dim(target) != 0:
                cost += read_write_time(comm_bytes_gb * 2 * 1024**3, p)
            comm_bytes_gb /= n
        elif ck == KIND_S and tk == KIND_P:  # :131-134
            return math.inf
        elif ck == KIND_R and tk == KIND_P:  # :135-138
            return math.inf
        contiguous = True  # :141
    return cost


def comms_order(src, tgt, ndim):
    """ref: collective_runtime_estimation.py:146-151: mesh dims are walked in
    natural order, except (Partial(sum), Partial(sum)) -> all-Shard on a 2-D mesh."""
    if tuple(src) == (PARTIAL_SUM, PARTIAL_SUM) and all(kind(t) == KIND_S for t in tgt):
        return [1, 0]
    return list(range(ndim))


def estimate_strategy_comms_cost(src, tgt, shape, stride, itemsize, p: CostParams) -> float:
    """ref: collective_runtime_estimation.py:146-153."""
    return redistribute_cost(src, tgt, shape, stride, itemsize, p, comms_order(src, tgt, p.ndim))


# --------------------------------------------------------------------------------------
# per-strategy compute cost
# --------------------------------------------------------------------------------------
def mm_flop(m, k, n):
    """torch: utils/flop_counter.py:58-66."""
    return m * n * 2 * k


def bmm_flop(b, m, k, n):
    """torch: utils/flop_counter.py:74-85."""
    return b * m * n * 2 * k


def sdpa_flop(b, h, s_q, s_k, d_q, d_v):
    """torch: utils/flop_counter.py:267-292 (sdpa_flop_count)."""
    return bmm_flop(b * h, s_q, d_q, s_k) + bmm_flop(b * h, s_q, s_k, d_v)


def sdpa_backward_flop(b, h, s_q, s_k, d_q, d_v):
    """torch: utils/flop_counter.py:478-512 (sdpa_backward_flop_count): five bmm terms."""
    total = 0
    total += bmm_flop(b * h, s_q, d_q, s_k)  # recompute scores
    total += bmm_flop(b * h, s_q, d_v, s_k)  # gradOut @ v^T -> gradScores
    total += bmm_flop(b * h, s_k, s_q, d_v)  # scores^T @ gradOut -> gradV
    total += bmm_flop(b * h, s_q, s_k, d_q)  # gradScores @ k -> gradQ
    total += bmm_flop(b * h, d_q, s_q, s_k)  # q^T @ gradScores -> gradK^T
    return total


NODE_ZERO_COST, NODE_BYTES_ONLY, NODE_MM, NODE_BMM, NODE_SDPA, NODE_SDPA_BACKWARD = range(6)


def strategy_inputs(strat_node, node_strat_begin, node_kind, node_dtype, node_const_bytes, node_row_begin, byte_rows,
                    node_flop_rows, local_shape, local_bytes):
    """ref: compute_estimation.py:232-299, 334-349 per (node, strategy), on the encoded form:
    the bytes of every tensor argument and output on its local shard (rows of the spec table)
    plus the node's constant bytes, and the flops torch's counter gives the operator on the
    local shapes (mm / bmm / attention formulas above; zero for operators outside its registry;
    zero-cost nodes :279-291 get nothing).
    -> (flops, rw_bytes, dtype_code, zero_cost), one row per strategy."""
    n = len(strat_node)
    flops, rw, dtype, zero = [0] * n, [0] * n, [0] * n, [0] * n
    for i in range(n):
        node = int(strat_node[i])
        ss = i - int(node_strat_begin[node])
        kind = int(node_kind[node])
        dtype[i] = int(node_dtype[node])
        zero[i] = 1 if kind == NODE_ZERO_COST else 0
        if kind == NODE_ZERO_COST:
            continue
        total = int(node_const_bytes[node])
        for r in range(int(node_row_begin[node]), int(node_row_begin[node + 1])):
            total += int(local_bytes[int(byte_rows[r]) + ss])
        rw[i] = total

        def shape(t):
            return [int(x) for x in local_shape[int(node_flop_rows[node][t]) + ss]]

        if kind == NODE_MM:
            (m, k), (_, nn) = shape(0)[:2], shape(1)[:2]
            flops[i] = mm_flop(m, k, nn)
        elif kind == NODE_BMM:
            (b, m, k), (_, _, nn) = shape(0)[:3], shape(1)[:3]
            flops[i] = bmm_flop(b, m, k, nn)
        elif kind in (NODE_SDPA, NODE_SDPA_BACKWARD):
            (b, h, s_q, d_q), s_k, d_v = shape(0)[:4], shape(1)[2], shape(2)[3]
            flops[i] = (sdpa_flop if kind == NODE_SDPA else sdpa_backward_flop)(b, h, s_q, s_k, d_q, d_v)
    return flops, rw, dtype, zero


def compute_cost(zero_cost: bool, flops: int, rw_bytes: int, dtype_code: int, p: CostParams):
    """ref: compute_estimation.py:334-365 tail (after flops / bytes are known)."""
    if zero_cost:
        return 0
    read_write_time_ = read_write_time(rw_bytes, p)
    if flops == 0:
        return read_write_time_
    gpu_flops = p.gpu_flops[dtype_code]
    if gpu_flops == 0.0:
        raise ValueError(f"Dtype code {dtype_code} not supported on this device row")
    compute_time = flops / gpu_flops * 1e6
    compute_time = compute_time / p.compute_eff
    return max(compute_time, read_write_time_)


# --------------------------------------------------------------------------------------
# table build over the flattened encoding  (ref: optimize_sharding.py:270-380)
# --------------------------------------------------------------------------------------
def build_tables(enc: dict, p: CostParams, edge_range=None):
    """Walks every (edge, consumer strategy, producer strategy) entry like
    ShardingOptimizer.build_ds and returns python lists
    comm[], transition[], cost[] in edge-major, consumer-row-major order, plus the
    per-strategy compute_cost[] and compute_cost/num_args[].

    ``enc`` is a dict of numpy arrays / lists with the keys documented in
    autoparallel_amd/encoding.py (plain data, no product code is called).
    """
    M = p.ndim
    n_strat = len(enc["strat_flops"])
    compute = [0.0] * n_strat
    compute_per_arg = [0.0] * n_strat
    for s in range(n_strat):
        c = compute_cost(bool(enc["strat_zero_cost"][s]), int(enc["strat_flops"][s]),
                         int(enc["strat_rw_bytes"][s]), int(enc["strat_dtype"][s]), p)
        compute[s] = c
        compute_per_arg[s] = c / int(enc["strat_num_args"][s])  # optimize_sharding.py:371-373

    t_rank = enc["tensor_rank"]
    t_shape = enc["tensor_shape"]
    t_stride = enc["tensor_stride"]
    t_item = enc["tensor_itemsize"]
    s_codes = enc["spec_codes"]
    s_tensor = enc["spec_tensor"]
    pt = enc["pt_values"]
    n_edges = len(enc["edge_n_src"])
    lo, hi = (0, n_edges) if edge_range is None else edge_range
    comm_out, trans_out, cost_out = [], [], []
    for e in range(lo, hi):
        sb, ns = int(enc["edge_src_begin"][e]), int(enc["edge_n_src"][e])
        tb, nt = int(enc["edge_tgt_begin"][e]), int(enc["edge_n_tgt"][e])
        flags = int(enc["edge_flags"][e])
        ptb = int(enc["edge_pt_begin"][e])
        stb = int(enc["edge_strat_begin"][e])
        for ss in range(nt):
            tgt_spec = tb + ss
            for ii in range(ns):
                src_spec = sb + ii
                passthrough = (flags & EDGE_NO_PRODUCER) or s_tensor[src_spec] < 0 or s_tensor[tgt_spec] < 0
                if passthrough:
                    comm = float(pt[ptb + ss * ns + ii])
                    trans = 0
                else:
                    t = int(s_tensor[src_spec])
                    r = int(t_rank[t])
                    src = unpack_codes(int(s_codes[src_spec]), M)
                    tgt = unpack_codes(int(s_codes[tgt_spec]), M)
                    comm = estimate_strategy_comms_cost(
                        src, tgt, [int(x) for x in t_shape[t][:r]], [int(x) for x in t_stride[t][:r]],
                        int(t_item[t]), p)
                    trans = int(src != tgt) * p.transition_scale  # :345-351
                if flags & EDGE_GRAD_RESCALE:
                    comm = comm / p.rescale  # :358-359
                comm_out.append(comm)
                trans_out.append(trans)
                cost_out.append(comm + compute_per_arg[stb + ss] + trans)  # :368-372
    return {"comm": comm_out, "transition": trans_out, "cost": cost_out,
            "compute": compute, "compute_per_arg": compute_per_arg}


# --------------------------------------------------------------------------------------
# integer tables  (a7 / a8)
# --------------------------------------------------------------------------------------
def tensor_tables(enc: dict):
    """bytes and contiguity flag per tensor row."""
    out_bytes, out_cont = [], []
    for t in range(len(enc["tensor_rank"])):
        r = int(enc["tensor_rank"][t])
        shape = [int(x) for x in enc["tensor_shape"][t][:r]]
        stride = [int(x) for x in enc["tensor_stride"][t][:r]]
        out_bytes.append(tensor_bytes(int(enc["tensor_itemsize"][t]), shape))
        out_cont.append(int(is_contiguous(shape, stride)))
    return out_bytes, out_cont


def spec_tables(enc: dict, mesh_sizes):
    """num_shards, local shape/stride, local numel and local bytes per spec row.
    Rows with tensor < 0 (not a DTensorSpec) yield zeros."""
    M = len(mesh_sizes)
    shards, lshape, lstride, lnumel, lbytes = [], [], [], [], []
    for s in range(len(enc["spec_codes"])):
        t = int(enc["spec_tensor"][s])
        if t < 0:
            shards.append(0); lshape.append([0] * MAX_RANK); lstride.append([0] * MAX_RANK)
            lnumel.append(0); lbytes.append(0)
            continue
        r = int(enc["tensor_rank"][t])
        codes = unpack_codes(int(enc["spec_codes"][s]), M)
        shape = [int(x) for x in enc["tensor_shape"][t][:r]]
        stride = [int(x) for x in enc["tensor_stride"][t][:r]]
        ns, nst = sharded_shape_stride(shape, stride, codes, mesh_sizes)
        shards.append(num_shards(codes, mesh_sizes))
        lshape.append(ns + [0] * (MAX_RANK - r))
        lstride.append(nst + [0] * (MAX_RANK - r))
        ne = math.prod(ns)
        lnumel.append(ne)
        lbytes.append(ne * int(enc["tensor_itemsize"][t]))
    return shards, lshape, lstride, lnumel, lbytes


# --------------------------------------------------------------------------------------
# segmented min (a14; no reference counterpart: defined by this build, checked by brute force)
# --------------------------------------------------------------------------------------
def segmented_min(values, seg_ptr):
    """min and first argmin (index relative to the segment start) of each
    [seg_ptr[k], seg_ptr[k+1]) slice; empty segments give (+inf, -1)."""
    mins, args = [], []
    for k in range(len(seg_ptr) - 1):
        lo, hi = int(seg_ptr[k]), int(seg_ptr[k + 1])
        best, arg = math.inf, -1
        for j in range(lo, hi):
            v = values[j]
            if arg < 0 or v < best:
                best, arg = v, j - lo
        mins.append(best)
        args.append(arg)
    return mins, args


def cost_objective(cost, var_of_entry, n_vars: int, inf_replacement: float = 10000.0):
    """Objective coefficient and forced-to-zero flag of every ILP variable.
    ref: autoparallel/optimize_sharding.py:650-655 (``opt_target = defaultdict(int)``;
    ``opt_target[x["va"]] += x["cost"]`` over ``ds.values()``: entries that share a variable
    add up one by one, in entry order, starting from the int 0) after :522-536 (a cost that is
    not finite has been replaced by 10000.0 and its variable forced to 0).
    Pinned by ``numpy.bincount`` (a sequential accumulation in input order) and by hand cases."""
    obj = [0] * n_vars
    forced = [False] * n_vars
    for c, v in zip(cost, var_of_entry):
        c, v = float(c), int(v)
        if not math.isfinite(c):
            c = inf_replacement
            forced[v] = True
        obj[v] += c
    return [float(x) for x in obj], forced


def diffusion_sweeps(n_sweeps, label_begin, inc_begin, inc_edge, inc_side, edge_begin, edge_i, edge_j, color_begin,
                     color_nodes, theta, unary):
    """Min-sum diffusion over a pairwise labelling problem, in place on ``theta`` / ``unary``
    (numpy fp64 arrays).  No reference counterpart (the reference does no pruning,
    ref: autoparallel/optimize_sharding.py:648-659); defined by this build and pinned by its
    invariants: every update leaves the cost of every labelling unchanged (brute force on tiny
    problems), the bound never decreases and never exceeds the brute-force optimum.
    One sweep updates the classes colour by colour, in ``color_nodes`` order.  A node update:
      tot = unary of the class; for every incident edge, in incidence order: d = row minima
      (the class labels the rows) or column minima of the edge matrix; rows / columns with a
      finite minimum have it subtracted; tot += d.  Then share = tot / degree; labels with a
      finite share get unary 0 and share added back to their row / column of every incident
      matrix; the others (no finite pair left on some edge) get unary +inf and +inf rows."""
    import numpy as np

    def mat(k):
        ni = int(label_begin[edge_i[k] + 1] - label_begin[edge_i[k]])
        nj = int(label_begin[edge_j[k] + 1] - label_begin[edge_j[k]])
        return theta[int(edge_begin[k]):int(edge_begin[k + 1])].reshape(ni, nj)

    for _ in range(int(n_sweeps)):
        for c in color_nodes:
            c = int(c)
            lo, hi = int(inc_begin[c]), int(inc_begin[c + 1])
            if hi == lo:
                continue
            u = unary[int(label_begin[c]):int(label_begin[c + 1])]
            tot = u.copy()
            for t in range(lo, hi):
                m = mat(int(inc_edge[t]))
                if inc_side[t] == 1:
                    m = m.T
                d = m.min(axis=1)
                fin = np.isfinite(d)
                m[fin, :] -= d[fin, None]
                tot = tot + d
            share = tot / float(hi - lo)
            fin = np.isfinite(tot)
            for t in range(lo, hi):
                m = mat(int(inc_edge[t]))
                if inc_side[t] == 1:
                    m = m.T
                m[fin, :] += share[fin, None]
                m[~fin, :] = np.inf
            u[:] = np.where(fin, 0.0, np.inf)


def strategy_bounds(enc: dict, row_min):
    """Optimistic cost of every (node, strategy): the sum, over the node's edges in edge
    order, of that consumer strategy's row minimum (``row_min`` ordered by edge, then consumer
    strategy).  No reference counterpart (a14); pinned by brute force over all plans of tiny
    graphs: min over a node's strategies, summed over nodes, never exceeds the best plan."""
    nsb = [int(x) for x in enc["node_strat_begin"]]
    bound = [0.0] * nsb[-1]
    row = 0
    for e in range(len(enc["edge_node"])):
        n, nt = int(enc["edge_node"][e]), int(enc["edge_n_tgt"][e])
        assert nt == nsb[n + 1] - nsb[n], "an edge has one row per strategy of its consumer"
        for k in range(nt):
            bound[nsb[n] + k] += float(row_min[row + k])
        row += nt
    return bound


def greedy_strategies(enc: dict, row_min):
    """-> (bound per strategy, min per node, first argmin per node, lower bound of any plan's
    cost); a node without strategies (the graph's output node) has argmin -1 and adds nothing."""
    bound = strategy_bounds(enc, row_min)
    mins, args = segmented_min(bound, enc["node_strat_begin"])
    return bound, mins, args, math.fsum(m for m, a in zip(mins, args) if a >= 0)
