"""CPU oracle for the sharding-cost evaluation path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory: it is the checker used by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``; it is never the thing that is
measured as the product or that serves a product call.

Contents
--------
``cost_oracle.py``   scalar pure-Python restatement of the reference formulas
                     (one function per reference function, each citing the
                     file:line it follows).  This is the timed CPU baseline:
                     the reference itself is interpreted Python.
``cost_oracle.c``    the same arithmetic in plain C (IEEE binary64, FMA
                     contraction off) so parity tests can cover tables of
                     10^6..10^8 entries in seconds.  Built by ``Makefile`` into
                     ``libcost_oracle.so``; loaded through ``c_oracle.py``.

Parity pins (what each function is checked against, see tests/test_oracle_*):
  * alpha-beta collectives, mesh topology, contiguity, byte counts, shard
    counts: the torch library routines they restate
    (torch.distributed.tensor._collective_utils, torch._prims_common,
    DTensorSpec.num_shards) on the same inputs;
  * redistribute_cost: torch's own redistribute_cost for the transitions where
    the two definitions coincide, hand-derived known-answer values, special
    cases (inf bans, zero cost, order flip), brute-force invariants;
  * sharded shape: torch.chunk sizes for even splits, explicit stride quirk case;
  * compute-cost tail and flop formulas: torch.utils.flop_counter on real
    (meta) tensors and a hand-derived mm value;
  * segmented min: numpy.minimum.reduceat / brute force.
No function here is "parity unpinned"; the reference holds no numeric cost
fixtures, so cost values are pinned by the closed forms above and plan-level
expectations from the reference's tests.
"""
