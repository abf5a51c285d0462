"""Pins the CPU oracle (oracle/cost_oracle.py and its C twin) against sources that do
not share its text: the torch library routines it restates, hand-derived known-answer
values, special cases and brute-force properties.  The reference holds no numeric cost
fixtures (its tests only pin ILP outcomes), so these are the anchors of cost parity.
"""

import itertools
import math
import random

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import cost_oracle as po

R, P = po.REPLICATE, po.PARTIAL_SUM
S0, S1, S2 = po.shard(0), po.shard(1), po.shard(2)


# ---------------------------------------------------------------------------------------
# topology and the three ring collectives vs torch's own routines
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("mesh_sizes", [(64,), (8,), (32, 8), (8, 8, 8), (64, 4), (16, 8, 4), (2, 2, 2), (3, 5)])
def test_mesh_topology_matches_torch(torch_topo, mesh_sizes):
    _, topo = torch_topo(mesh_sizes)
    n, bw, lat = po.mesh_topology(mesh_sizes, devices_per_host=8)
    assert list(n) == topo.mesh_dim_devices
    assert list(bw) == topo.mesh_dim_bandwidth  # exact fp64 equality
    assert list(lat) == topo.mesh_dim_latency


def test_inter_host_bandwidth_value():
    _, bw, lat = po.mesh_topology((32, 8))
    assert bw == (87.7 * 0.22, 87.7) and bw[0] == 19.294
    assert lat == (2.7, 0.6)


@pytest.mark.parametrize("mesh_sizes", [(32, 8), (16, 8, 4), (3, 5)])
def test_ring_collectives_match_torch(torch_topo, mesh_sizes):
    from torch.distributed.tensor._collective_utils import allgather_cost, allreduce_cost, reduce_scatter_cost

    _, topo = torch_topo(mesh_sizes)
    p = po.make_params(mesh_sizes)
    rng = random.Random(0)
    for _ in range(200):
        gb = rng.random() * 10 ** rng.randint(-6, 2)
        for d in range(len(mesh_sizes)):
            assert po.allgather_cost(gb, p, d) == allgather_cost(gb, topo, d)
            assert po.allreduce_cost(gb, p, d) == allreduce_cost(gb, topo, d)
            assert po.reduce_scatter_cost(gb, p, d) == reduce_scatter_cost(gb, topo, d)
            # all-to-all = 5 x the all-gather shaped ring (reference's own formula)
            assert po.all_to_all_cost(gb, p, d) == allgather_cost(gb, topo, d) * 5


# ---------------------------------------------------------------------------------------
# contiguity / bytes / shard counts vs torch
# ---------------------------------------------------------------------------------------
def test_contiguity_matches_torch():
    from torch._prims_common import check_contiguous_sizes_strides

    rng = random.Random(1)
    cases = [((4, 4), (4, 1)), ((4, 4), (1, 4)), ((1, 4), (99, 1)), ((4, 1), (1, 77)), ((), ()), ((0, 3), (3, 1)),
             ((2, 0, 3), (0, 3, 1)), ((2, 0, 3), (3, 3, 1)), ((2, 3, 4), (12, 4, 1)), ((2, 3, 4), (12, 1, 3))]
    for _ in range(500):
        r = rng.randint(1, 5)
        shape = tuple(rng.choice([1, 1, 2, 3, 4, 8]) for _ in range(r))
        t = torch.empty(shape)
        perm = list(range(r))
        if rng.random() < 0.5:
            rng.shuffle(perm)
        v = t.permute(perm)
        cases.append((tuple(v.shape), tuple(v.stride())))
        if rng.random() < 0.3:
            cases.append((tuple(v.shape), tuple(rng.choice([1, 2, 4, 8]) for _ in range(r))))
    for shape, stride in cases:
        assert po.is_contiguous(shape, stride) == check_contiguous_sizes_strides(shape, stride), (shape, stride)


def test_num_shards_and_bytes_match_dtensor_spec(torch_topo):
    from torch.distributed.tensor._collective_utils import spec_to_bytes
    from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

    mesh, _ = torch_topo((16, 8, 4))
    tm = TensorMeta(torch.Size([64, 128, 32]), (4096, 32, 1), torch.bfloat16)
    opts = [(Replicate(), R), (Partial(), P), (Shard(0), S0), (Shard(2), S2)]
    for combo in itertools.product(opts, repeat=3):
        spec = DTensorSpec(mesh, tuple(c[0] for c in combo), tensor_meta=tm)
        codes = tuple(c[1] for c in combo)
        assert po.num_shards(codes, (16, 8, 4)) == spec.num_shards
        assert po.tensor_bytes(2, (64, 128, 32)) == spec_to_bytes(spec)


# ---------------------------------------------------------------------------------------
# redistribute_cost: known answers, torch's own redistribute_cost where both coincide,
# special cases, invariants
# ---------------------------------------------------------------------------------------
KAT_SHAPE, KAT_STRIDE = [4096, 4096], [4096, 1]


def _cost(src, tgt, shape=KAT_SHAPE, stride=KAT_STRIDE, itemsize=2, mesh=(32, 8)):
    return po.estimate_strategy_comms_cost(src, tgt, shape, stride, itemsize, po.make_params(mesh))


def _golden():
    import json
    import os

    with open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")) as f:
        return json.load(f)


_NAMED = {"R": R, "P": P, "S0": S0, "S1": S1, "S2": S2}


def test_known_answers_2d_mesh():
    # hand-derived from the published formulas, mesh (32, 8), 8 devices/host, H100 row
    g = _golden()
    mesh = tuple(g["environment"]["mesh"])
    for case in g["redistribute_cost_us"]:
        src, tgt = tuple(_NAMED[x] for x in case["src"]), tuple(_NAMED[x] for x in case["tgt"])
        assert _cost(src, tgt, case["shape"], case["stride"], case["itemsize"], mesh) == case["value"], case["note"]
    u = g["unflipped_order_us"]
    p = po.make_params(mesh)
    assert po.redistribute_cost(tuple(_NAMED[x] for x in u["src"]), tuple(_NAMED[x] for x in u["tgt"]), u["shape"],
                                u["stride"], u["itemsize"], p, u["order"]) == u["value"]
    assert p.bw[0] == g["inter_host_bandwidth_GBps"]


def test_known_answers_3d_mesh():
    """Mesh (8, 8, 8), 8 devices per host: dims 0 and 1 inter-host, dim 2 intra-host.  The running
    bytes carried across three mesh dims, a reduce-scatter onto a non-dim-0 shard, an all-to-all
    between two non-dim-0 shards and the non-contiguity charge, from the golden file and written
    out here term by term (plain arithmetic, none of the oracle's helpers)."""
    g = _golden()["mesh_8x8x8"]
    mesh = tuple(g["environment"]["mesh"])
    p = po.make_params(mesh)
    assert list(p.bw) == g["environment"]["bandwidth_GBps"] and list(p.lat) == g["environment"]["hop_latency_us"]
    for case in g["redistribute_cost_us"]:
        src, tgt = tuple(_NAMED[x] for x in case["src"]), tuple(_NAMED[x] for x in case["tgt"])
        assert _cost(src, tgt, case["shape"], case["stride"], case["itemsize"], mesh) == case["value"], case["note"]
    inter, intra = 87.7 * 0.22, 87.7

    def rw(nbytes):
        return max(nbytes / (3.35 * 1024**4) * 1e6 / 0.70, 7)

    # (S0, P, S1) -> (R, S0, R): gather over dim 0, reduce-scatter on the gathered bytes over dim 1,
    # gather of a dim-1 shard over dim 2 with its reshuffle
    gb = 2 * 4096 * 4096 / 64 / 1024 / 1024 / 1024  # Partial does not count as a shard
    gb *= 8
    expect = (6.6 + 7 * 2.7) + ((gb * 7 / 8) / inter) * 1e6
    expect += (6.6 + 7 * 2.7) + ((gb * 7 / 8) / inter) * 1e6
    gb /= 8
    gb *= 8
    expect += (6.6 + 7 * 0.6) + ((gb * 7 / 8) / intra) * 1e6
    expect += rw(gb * 2 * 1024**3)
    assert g["redistribute_cost_us"][0]["value"] == expect == _cost((S0, P, S1), (R, S0, R), mesh=mesh)
    # Partial -> Shard(1): the reshuffle is charged on the bytes before the scatter
    gb = 4 * 8192 * 4096 / 1024 / 1024 / 1024
    expect = (6.6 + 7 * 2.7) + ((gb * 7 / 8) / inter) * 1e6
    expect += rw(gb * 2 * 1024**3)
    assert g["redistribute_cost_us"][1]["value"] == expect
    # Shard(1) -> Shard(2): five times the ring term, two reshuffles
    gb = 2 * 64 * 2048 * 4096 / 8 / 1024 / 1024 / 1024
    expect = ((6.6 + 7 * 2.7) + ((gb * 7 / 8) / inter) * 1e6) * 5
    expect += 2 * rw(gb * 2 * 1024**3)
    assert g["redistribute_cost_us"][2]["value"] == expect
    # dropping the reshuffle of the dim-1 gather, or charging the reduce-scatter after the division, is seen
    assert _cost((S0, P, S0), (R, S0, R), mesh=mesh) < g["redistribute_cost_us"][0]["value"]
    assert _cost((S0, P, S1), (R, S0, R), mesh=mesh) != _cost((S0, R, S1), (R, S0, R), mesh=mesh)


def test_hand_expanded_allgather_value():
    # (S0, S0) -> (R, S0) written out term by term, independent of the oracle's helpers
    gb = 4096 * 4096 * 2 / 256 / 1024 / 1024 / 1024
    gb *= 32
    expect = (6.6 + 31 * 2.7) + ((gb * 31 / 32) / (87.7 * 0.22)) * 1e6
    assert _cost((S0, S0), (R, S0)) == expect
    # S(1) -> R on the intra-host dim adds the reshuffle read+write
    gb1 = 4096 * 4096 * 2 / 8 / 1024 / 1024 / 1024 * 8
    rw = max(gb1 * 2 * 1024**3 / (3.35 * 1024**4) * 1e6 / 0.70, 7)
    expect = (6.6 + 7 * 0.6) + ((gb1 * 7 / 8) / 87.7) * 1e6 + rw
    assert _cost((R, S1), (R, R)) == expect


def test_matches_torch_redistribute_cost_where_definitions_coincide(torch_topo):
    """torch's redistribute_cost (the function the reference's is derived from) has no
    non-contiguity / non-dim-0 penalties and no all-to-all; for contiguous tensors,
    dim-0 shards and single-step S->R, P->R, P->S transitions both must agree bit for bit."""
    from unittest.mock import patch

    from torch.distributed.device_mesh import _mesh_resources
    from torch.distributed.tensor._collective_utils import MeshTopoInfo, redistribute_cost
    from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

    mesh_sizes = (32, 8)
    mesh, _ = torch_topo(mesh_sizes)
    tm = TensorMeta(torch.Size([8192, 4096]), (4096, 1), torch.float32)
    tp = {R: Replicate(), P: Partial(), S0: Shard(0)}
    pairs = [((S0, R), (R, R)), ((R, S0), (R, R)), ((P, R), (R, R)), ((R, P), (R, R)), ((P, R), (S0, R)),
             ((R, P), (R, S0)), ((R, R), (S0, S0)), ((R, R), (R, R)), ((S0, R), (S0, R)), ((P, S0), (R, S0)),
             ((S0, P), (S0, R)), ((S0, P), (S0, S0))]
    MeshTopoInfo.build_from_mesh.cache_clear()
    with patch.object(type(_mesh_resources), "num_devices_per_host", lambda self, device_type: 8):
        for src, tgt in pairs:
            a = DTensorSpec(mesh, tuple(tp[c] for c in src), tensor_meta=tm)
            b = DTensorSpec(mesh, tuple(tp[c] for c in tgt), tensor_meta=tm)
            assert _cost(src, tgt, [8192, 4096], [4096, 1], 4) == redistribute_cost(a, b), (src, tgt)
    MeshTopoInfo.build_from_mesh.cache_clear()


def test_special_cases():
    inf = math.inf
    assert _cost((R, R), (S0, S1)) == 0.0  # replicated source: free
    assert _cost((R, R), (P, R)) == inf  # ... unless the target is Partial
    assert _cost((S0, R), (P, R)) == inf  # Shard -> Partial banned
    assert _cost((R, S0), (P, S0)) == inf  # Replicate -> Partial banned
    assert _cost((R, S0), (S1, S0)) == 0.0  # Replicate -> Shard is a local slice
    for src in itertools.product((R, P, S0, S1), repeat=2):
        assert _cost(src, src) == 0.0
    # non-contiguous: exactly one read+write on the first mismatching dim, none afterwards
    p = po.make_params((32, 8))
    nc = [1, 4096]
    gb = 4096 * 4096 * 2 / 256 / 1024**3
    extra = po.read_write_time(gb * 2 * 1024**3, p)
    assert _cost((S0, S0), (R, R), stride=nc) == extra + _cost((S0, S0), (R, R))
    assert _cost((R, S0), (S1, S0), stride=nc) == po.read_write_time(4096 * 4096 * 2 / 8 / 1024**3 * 2 * 1024**3, p)
    # Partial(sum) -> Partial(avg): no collective is charged
    assert _cost((P, R), (po.partial(1), R)) == 0.0
    # a different Partial pair does not trigger the order flip
    assert _cost((po.partial(1), po.partial(1)), (S0, S0)) == po.redistribute_cost(
        (po.partial(1), po.partial(1)), (S0, S0), KAT_SHAPE, KAT_STRIDE, 2, p, [0, 1])


def test_order_flip_only_for_partial_partial_to_all_shard():
    assert po.comms_order((P, P), (S0, S1), 2) == [1, 0]
    assert po.comms_order((P, P), (S0, R), 2) == [0, 1]
    assert po.comms_order((P, S0), (S0, S0), 2) == [0, 1]
    assert po.comms_order((P,), (S0,), 1) == [0]
    assert po.comms_order((P, P, P), (S0, S0, S0), 3) == [0, 1, 2]


def test_invariants_brute_force():
    """All placement pairs on a tiny tensor: cost >= 0, monotone in bytes, finite unless
    a -> Partial transition from a non-Partial occurs."""
    p = po.make_params((4, 2))
    opts = (R, P, S0, S1)
    for src in itertools.product(opts, repeat=2):
        for tgt in itertools.product(opts, repeat=2):
            c1 = po.estimate_strategy_comms_cost(src, tgt, [8, 8], [8, 1], 2, p)
            c2 = po.estimate_strategy_comms_cost(src, tgt, [64, 64], [64, 1], 4, p)
            assert c1 >= 0 and c2 >= c1
            if all(s == R for s in src):
                banned = any(po.kind(t) == 1 for t in tgt)
            else:
                # the walk returns inf at the first banned dim it reaches
                banned = any(po.kind(t) == 1 and po.kind(s) != 1 for s, t in zip(src, tgt))
            assert math.isinf(c1) == banned, (src, tgt)


# ---------------------------------------------------------------------------------------
# sharded shapes
# ---------------------------------------------------------------------------------------
def test_sharded_shape_matches_torch_chunk():
    for size, n in [(4096, 8), (4096, 32), (10, 4), (7, 8), (128, 3)]:
        t = torch.empty(size, 3)
        local, _ = po.sharded_shape_stride([size, 3], [3, 1], (po.shard(0),), (n,))
        assert local[0] == torch.chunk(t, n, dim=0)[0].shape[0]
    # two mesh dims on the same tensor dim: sequential ceil-div
    local, _ = po.sharded_shape_stride([100, 6], [6, 1], (S0, S0), (8, 4))
    assert local == [math.ceil(math.ceil(100 / 8) / 4), 6]


def test_sharded_stride_quirk():
    # stride of dim-1 is divided only when dim-1 > 0 (i.e. shard dim >= 2)
    shape, stride = [8, 16, 32], [512, 32, 1]
    assert po.sharded_shape_stride(shape, stride, (S2,), (4,)) == ([8, 16, 8], [512, 8, 1])
    assert po.sharded_shape_stride(shape, stride, (S1,), (4,)) == ([8, 4, 32], [512, 32, 1])
    assert po.sharded_shape_stride(shape, stride, (S0,), (4,)) == ([2, 16, 32], [512, 32, 1])


# ---------------------------------------------------------------------------------------
# compute cost
# ---------------------------------------------------------------------------------------
def test_compute_cost_known_answer():
    p = po.make_params((32, 8))
    flops, rw = po.mm_flop(2048, 4096, 4096), 2 * (2048 * 4096 + 4096 * 4096 + 2048 * 4096)
    assert flops == 68719476736 and rw == 67108864
    assert po.read_write_time(rw, p) == 26.027785181236673
    assert po.compute_cost(False, flops, rw, po.DTYPE_CODES["bfloat16"], p) == 99.26256931388127
    assert po.compute_cost(True, flops, rw, 3, p) == 0
    assert po.compute_cost(False, 0, 1024, 3, p) == 7  # launch floor
    with pytest.raises(ValueError):
        po.compute_cost(False, 1, 1, 7, p)


def test_flop_formulas_match_torch_flop_counter():
    from torch.utils.flop_counter import FlopCounterMode

    def count(fn):
        with FlopCounterMode(display=False) as fc:
            fn()
        return fc.get_total_flops()

    a, b = torch.empty(48, 80, device="meta"), torch.empty(80, 24, device="meta")
    assert count(lambda: a @ b) == po.mm_flop(48, 80, 24)
    x, y = torch.empty(5, 48, 80, device="meta"), torch.empty(5, 80, 24, device="meta")
    assert count(lambda: torch.bmm(x, y)) == po.bmm_flop(5, 48, 80, 24)
    q = torch.empty(2, 4, 64, 16, device="meta", requires_grad=True)
    k = torch.empty(2, 4, 96, 16, device="meta", requires_grad=True)
    v = torch.empty(2, 4, 96, 32, device="meta", requires_grad=True)
    from torch.utils.flop_counter import sdpa_backward_flop_count, sdpa_flop_count

    assert sdpa_flop_count(q.shape, k.shape, v.shape) == po.sdpa_flop(2, 4, 64, 96, 16, 32)
    assert sdpa_backward_flop_count((2, 4, 64, 32), q.shape, k.shape, v.shape) == po.sdpa_backward_flop(2, 4, 64, 96, 16, 32)


def test_device_rows():
    assert po.device_limit("NVIDIA H100 80GB HBM3")[0] == "H100"
    assert po.device_limit("NVIDIA A100-SXM4")[0] == "A100"
    assert po.device_limit("PG509-210")[0] == "A100"
    with pytest.raises(ValueError):
        po.device_limit("AMD Instinct MI355X")
    with pytest.raises(ValueError):
        po.device_tflops("Tesla T4", "bfloat16")
    assert po.device_tflops("H100", "float32") == 494 and po.device_tflops("H100", "bfloat16") == 989


# ---------------------------------------------------------------------------------------
# C oracle == Python oracle, bit for bit
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("mesh_sizes", [(64,), (32, 8), (16, 8, 4), (6, 3), (2, 3, 2, 2)])
def test_c_oracle_equals_python_oracle(mesh_sizes):
    from autoparallel_amd.synthetic import stress_dag

    tb = stress_dag(seed=7, n_nodes=60, mesh_sizes=mesh_sizes, min_strategies=2, max_strategies=12,
                    frac_nonspec_nodes=0.1, frac_noncontiguous=0.3, min_log2_dim=2, max_log2_dim=9)
    enc = tb.as_dict()
    p = po.make_params(mesh_sizes, rescale=2.2)
    py = po.build_tables(enc, p)
    c = c_oracle.build_tables(enc, p)
    assert np.array_equal(np.asarray(py["comm"]), c["comm"])
    assert np.array_equal(np.asarray(py["cost"]), c["cost"])
    assert np.array_equal(np.asarray(py["transition"], dtype=np.uint8), c["transition"])
    cc, pa = c_oracle.compute_costs(enc, p)
    assert np.array_equal(np.asarray(py["compute"], dtype=np.float64), cc)
    assert np.array_equal(np.asarray(py["compute_per_arg"]), pa)
    tb_bytes, tb_cont = po.tensor_tables(enc)
    cb, ccont = c_oracle.tensor_tables(enc)
    assert np.array_equal(np.asarray(tb_bytes), cb) and np.array_equal(np.asarray(tb_cont, dtype=np.uint8), ccont)
    for a, b in zip(po.spec_tables(enc, mesh_sizes), c_oracle.spec_tables(enc, mesh_sizes)):
        assert np.array_equal(np.asarray(a, dtype=np.int64), b)


def test_segmented_min_matches_numpy():
    rng = np.random.default_rng(3)
    lens = rng.integers(1, 40, size=300)
    ptr = np.zeros(len(lens) + 1, np.int64)
    np.cumsum(lens, out=ptr[1:])
    vals = rng.choice([0.0, 1.5, 7.0, 12.25, np.inf], size=int(ptr[-1]))
    mins, args = po.segmented_min(vals, ptr)
    assert np.array_equal(np.asarray(mins), np.minimum.reduceat(vals, ptr[:-1]))
    for k in range(len(lens)):
        assert args[k] == int(np.argmin(vals[ptr[k]:ptr[k + 1]]))  # numpy argmin is first-min too
    cm, ca = c_oracle.segmented_min(vals, ptr)
    assert np.array_equal(cm, np.asarray(mins)) and np.array_equal(ca, np.asarray(args, dtype=np.int32))
    # empty segments
    m, a = po.segmented_min([3.0, 1.0], [0, 0, 2, 2])
    assert m == [math.inf, 1.0, math.inf] and a == [-1, 1, -1]
    cm, ca = c_oracle.segmented_min([3.0, 1.0], [0, 0, 2, 2])
    assert list(cm) == m and list(ca) == a
