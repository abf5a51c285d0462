/*
 * apcost — C ABI of the MI355X sharding-cost evaluation library (libapcost.so).
 *
 * The reference (pure Python) has no FFI layer; the seam these entry points sit
 * behind is the pair of per-entry Python calls made by
 * ShardingOptimizer.build_ds (autoparallel/optimize_sharding.py:270-380):
 *   estimate_strategy_comms_cost   autoparallel/collective_runtime_estimation.py:146-153
 *   estimate_strategy_runtime_cost autoparallel/compute_estimation.py:334-365
 * plus _get_sharded_shape_stride   autoparallel/compute_estimation.py:211-229.
 * Each entry point below names the reference function(s) it replaces, batched
 * over the whole graph.
 *
 * Conventions
 *   - Every array pointer is a DEVICE pointer unless the name ends in _host.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Calls
 *     enqueue work and return; they never synchronise and never allocate.
 *   - Return value 0 = success; negative = error, text via apc_last_error().
 *   - The library owns no memory.  Outputs are caller-allocated.
 *   - Device arrays come from hipMalloc (or an allocator built on it): a byte array may be
 *     read as aligned 4-byte words, i.e. up to its end rounded up to a multiple of 4, which
 *     such allocations always cover (tensor_contiguous is read this way).
 *   - No CPU fallback exists: without a HIP device every launch entry fails.
 *
 * Flattened graph tables ("encoding")
 *   placement code, one byte per mesh dim:
 *       0x00            Replicate
 *       0x40 | op       Partial(op), op 0 = sum
 *       0x80 | v<<4 | d Shard(tensor dim d), v = variant (0 plain)
 *   spec_codes[s]   uint32, byte i = code of mesh dim i (mesh ndim <= 4)
 *   spec_tensor[s]  int32 row of the tensor table, -1 = "not a DTensorSpec"
 *   tensor table    rank int32, itemsize int32, shape/stride int64[APC_MAX_RANK]
 *   edge e = (consumer node, argument):
 *       producer output specs  spec rows [edge_src_begin, +edge_n_src)
 *       consumer input specs   spec rows [edge_tgt_begin, +edge_n_tgt)
 *       matrix entries         [edge_entry_begin[e], +n_tgt*n_src), row = consumer
 *                              strategy, column = producer strategy
 *       edge_strat_begin[e]    row of the consumer's first strategy in the
 *                              per-strategy tables
 *       edge_pt_begin[e]       offset into pt_values of the rule-provided costs
 *                              kept where either spec is not a DTensorSpec
 *       edge_flags             APC_EDGE_*
 *   tile t = a rectangle of one edge's matrix handled by one workgroup (apc_tile)
 */
#ifndef APCOST_H
#define APCOST_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Version of this interface: the value apc_version() of a matching library returns.  It changes
 * whenever a struct layout, a limit below or the meaning of an argument changes (2: at most 32
 * identical edges per tile instead of 127; the row-minimum entry points write the minima of the
 * assembled cost whichever arrays are stored; 3: packed tiles).  A binding compares the two before its
 * first call. */
#define APC_ABI_VERSION 3

#define APC_MAX_RANK 8
#define APC_MAX_MESH 4
#define APC_MAX_DTYPES 8
#define APC_TILE_MAX_COLS 64 /* producer specs staged in LDS per tile */
#define APC_TILE_MAX_ROWS 64 /* consumer specs staged in LDS per tile */
#define APC_TILE_MAX_DUPS 32 /* identical edges served by one tile (offsets staged in LDS); a larger group of
                              identical edges is served by several tiled edges.  apc_validate_tables_host
                              rejects a tile with more; the kernels leave such a tile unwritten */
#define APC_MAX_STRATEGIES (1 << 22) /* strategies of one node: a tile's rows span < 4 GiB of fp64 */

#define APC_EDGE_GRAD_RESCALE 1 /* consumer is a parameter-gradient node (optimize_sharding.py:358-359) */
#define APC_EDGE_NO_PRODUCER 2  /* placeholder / factory pseudo-argument (optimize_sharding.py:312-355) */

/* One tile: a rows x cols rectangle of one edge's matrix, handled by one workgroup.
 * The record repeats the fields of its edge so that the kernel reaches everything it
 * needs with one load; apc_validate_tables_host checks it against the edge arrays.
 * Edges whose matrices are provably identical (same spec lists, tensor, flags, consumer
 * compute costs: the layers of a transformer) may be tiled once: the tile then lists the
 * entry offsets of the other copies (dup_entry_begin[dup_begin .. dup_begin + dup_count))
 * and every value is stored to all of them. */
typedef struct apc_tile {
  int32_t edge;
  int32_t row_begin;   /* first consumer strategy */
  int32_t col_begin;   /* first producer strategy */
  int32_t counts;      /* row_count | col_count << 16 */
  int32_t src_begin;   /* = edge_src_begin[edge] */
  int32_t n_src;       /* = edge_n_src[edge] */
  int32_t tgt_begin;   /* = edge_tgt_begin[edge] */
  int32_t flags;       /* = edge_flags[edge] */
  int32_t strat_begin; /* = edge_strat_begin[edge] */
  int32_t tensor;      /* = spec_tensor[src_begin + col_begin] */
  int64_t entry_begin; /* = edge_entry_begin[edge] */
  int64_t pt_begin;    /* = edge_pt_begin[edge] */
  int32_t dup_begin;   /* first row of dup_entry_begin for this tile's edge */
  int32_t dup_count;   /* number of identical edges that receive the same values */
} apc_tile;

/* Cost-model parameters: everything the reference reads from its environment
 * (torch MeshTopoInfo, DEVICE_LIMITS row, module constants), made explicit. */
typedef struct apc_params {
  int32_t mesh_ndim;
  int32_t mesh_size[APC_MAX_MESH];
  double bw[APC_MAX_MESH];  /* GB/s per mesh dim   torch _collective_utils.py:256-274 */
  double lat[APC_MAX_MESH]; /* us per hop          torch _collective_utils.py:258-274 */
  double base_latency;      /* 6.6 us              torch _collective_utils.py:286 */
  double a2a_scale;         /* 5                   collective_runtime_estimation.py:30-31 */
  double hbm_bw;            /* bytes/s             compute_estimation.py:63-166 */
  double rw_eff;            /* 0.70                compute_estimation.py:307 */
  double launch_floor;      /* 7 us                compute_estimation.py:309 */
  double compute_eff;       /* 0.70                compute_estimation.py:361 */
  double rescale;           /* grad comm rescale   optimize_sharding.py:358-359 */
  double gpu_flops[APC_MAX_DTYPES]; /* tflops*10^12 per dtype code; 0 = unsupported */
  int32_t transition_scale; /* 1                   optimize_sharding.py:298 */
  /* Derived values, checked by the library: the kernels divide by constants through their
   * correctly rounded reciprocals (same bits as a division, a sixth of the instructions). */
  double inv_bw[APC_MAX_MESH];   /* 1.0 / bw[i] */
  double inv_mesh[APC_MAX_MESH]; /* 1.0 / mesh_size[i] */
  double inv_hbm_bw;             /* 1.0 / hbm_bw */
  double inv_rw_eff;             /* 1.0 / rw_eff */
  double inv_compute_eff;        /* 1.0 / compute_eff */
  double inv_gpu_flops[APC_MAX_DTYPES]; /* 1.0 / gpu_flops[i]; 0 where gpu_flops[i] is 0 */
} apc_params;

int apc_version(void);
const char *apc_last_error(void);

/* Host-side structural check of the tables (HOST pointers).  Replaces the
 * reference's assertions in ShardingOptimizer.validate
 * (optimize_sharding.py:908-958) for the flattened form: monotone entry
 * offsets, spec/tensor/strategy indices in range, rank <= APC_MAX_RANK, shard
 * dims < rank, tiles inside their edge and within the LDS staging limits, duplicate
 * offsets naming edges of the same shape. */
int apc_validate_tables_host(const apc_params *params, int64_t n_tensors, const int32_t *tensor_rank_host,
                             int64_t n_specs, const uint32_t *spec_codes_host, const int32_t *spec_tensor_host,
                             int64_t n_edges, const int32_t *edge_src_begin_host, const int32_t *edge_n_src_host,
                             const int32_t *edge_tgt_begin_host, const int32_t *edge_n_tgt_host,
                             const int32_t *edge_flags_host, const int64_t *edge_pt_begin_host,
                             const int64_t *edge_entry_begin_host, const int32_t *edge_strat_begin_host,
                             int64_t n_pt, int64_t n_strategies, int64_t n_tiles, const apc_tile *tiles_host,
                             int64_t n_dups, const int64_t *dup_entry_begin_host);

/* Bytes and contiguity of every tensor row.
 * Replaces torch spec_to_bytes (distributed/tensor/_collective_utils.py:230-232) and
 * check_contiguous_sizes_strides (_prims_common/__init__.py:252-292) as called from
 * collective_runtime_estimation.py:66-76. */
int apc_tensor_tables(int64_t n_tensors, const int32_t *tensor_rank, const int32_t *tensor_itemsize,
                      const int64_t *tensor_shape, const int64_t *tensor_stride, int64_t *tensor_bytes,
                      uint8_t *tensor_contiguous, void *stream);

/* Local shard shape / stride / element and byte counts and shard count per spec.
 * Replaces _get_sharded_shape_stride (compute_estimation.py:211-229) and
 * DTensorSpec.num_shards (torch distributed/tensor/_dtensor_spec.py:555-561).
 * local_shape / local_stride are [n_specs][shape_width], zero padded: shape_width is even, at
 * most APC_MAX_RANK and at least the largest tensor rank (the caller's choice: rows of rank-4
 * tables padded to 8 would double the bytes this table writes). */
int apc_spec_tables(const apc_params *params, int64_t n_specs, const uint32_t *spec_codes,
                    const int32_t *spec_tensor, const int32_t *tensor_rank, const int32_t *tensor_itemsize,
                    const int64_t *tensor_shape, const int64_t *tensor_stride, int64_t *num_shards,
                    int64_t *local_shape, int64_t *local_stride, int32_t shape_width, int64_t *local_numel,
                    int64_t *local_bytes, void *stream);

/* Per-(node, strategy) compute cost and compute cost / num_args.
 * Replaces the arithmetic tail of estimate_strategy_runtime_cost
 * (compute_estimation.py:334-365) with compute_read_write_time (:302-314), and the
 * division at optimize_sharding.py:371-373.  A strategy with flops != 0 whose dtype
 * has no throughput on the device row sets *error_flag (device int32) to 1. */
int apc_compute_costs(const apc_params *params, int64_t n_strategies, const int64_t *flops,
                      const int64_t *rw_bytes, const int8_t *dtype_code, const uint8_t *zero_cost,
                      const int32_t *num_args, double *compute_cost, double *compute_cost_per_arg,
                      int32_t *error_flag, void *stream);

/* a9, integer part: flop and byte counts of every (node, strategy) from the local shard shapes
 * (replaces the fake-tensor run of compute_estimation.py:232-299, 334-349 for the operators whose
 * flop count torch/utils/flop_counter.py gives in closed form).  One recipe per node:
 *   node_kind         what the flop formula is (APC_NODE_*); APC_NODE_ZERO_COST rows get
 *                     flops = rw_bytes = 0 and zero_cost = 1 (compute_estimation.py:279-291)
 *   node_dtype        dtype code of the node's first tensor argument (written to every strategy)
 *   node_const_bytes  bytes that do not depend on the strategy (factory outputs, tensor constants)
 *   node_row_begin / byte_rows   CSR: first spec rows of the node's tensor arguments and output
 *                     slots; strategy ss adds local_bytes[row + ss] of each
 *   node_flop_rows    [n_nodes, 4] first spec rows of the tensors the formula reads (mm: mat1,
 *                     mat2; bmm: batch1, batch2; attention: query, key, value), unused slots 0
 * local_shape [n_specs, shape_width] / local_bytes [n_specs] are outputs of apc_spec_tables.
 * The caller guarantees that every row + ss lies inside the spec table and that the tensors a
 * formula reads have the rank it expects (2 / 3 / 4).  Outputs: one row per strategy. */
#define APC_NODE_ZERO_COST 0
#define APC_NODE_BYTES_ONLY 1 /* not counted by torch's flop counter: flops = 0 */
#define APC_NODE_MM 2         /* aten.mm, aten.addmm:    m * n * 2 * k */
#define APC_NODE_BMM 3        /* aten.bmm, aten.baddbmm: b * m * n * 2 * k */
#define APC_NODE_SDPA 4       /* _scaled_dot_product_{flash,efficient,cudnn}_attention */
#define APC_NODE_SDPA_BACKWARD 5
int apc_strategy_inputs(int64_t n_strategies, const int32_t *strat_node, int64_t n_nodes,
                        const int64_t *node_strat_begin, const int32_t *node_kind, const int8_t *node_dtype,
                        const int64_t *node_const_bytes, const int64_t *node_row_begin, const int32_t *byte_rows,
                        const int32_t *node_flop_rows, const int64_t *local_shape, int32_t shape_width,
                        const int64_t *local_bytes, int64_t *flops, int64_t *rw_bytes, int8_t *dtype_code,
                        uint8_t *zero_cost, void *stream);

/* apc_tensor_tables + apc_spec_tables + apc_compute_costs in ONE launch (none of the three
 * reads another's output): same arguments, same results, two launches fewer.  For a caller that
 * already holds the per-strategy flop / byte counts, e.g. when the tables of a graph are
 * rebuilt under another cost model.  (A planner that still has to infer those counts from the
 * local shard shapes calls apc_spec_tables and apc_strategy_inputs first.)
 * The five spec-table outputs may all be NULL: the spec table is then skipped. */
int apc_input_tables(const apc_params *params, int64_t n_tensors, const int32_t *tensor_rank,
                     const int32_t *tensor_itemsize, const int64_t *tensor_shape, const int64_t *tensor_stride,
                     int64_t *tensor_bytes, uint8_t *tensor_contiguous, int64_t n_specs, const uint32_t *spec_codes,
                     const int32_t *spec_tensor, int64_t *num_shards, int64_t *local_shape, int64_t *local_stride,
                     int32_t shape_width, int64_t *local_numel, int64_t *local_bytes, int64_t n_strategies,
                     const int64_t *flops, const int64_t *rw_bytes, const int8_t *dtype_code,
                     const uint8_t *zero_cost, const int32_t *num_args, double *compute_cost,
                     double *compute_cost_per_arg, int32_t *error_flag, void *stream);

/* The redistribution-cost matrices of every edge, plus the assembled ILP cost.
 * Replaces the two inner loops of ShardingOptimizer.build_ds
 * (optimize_sharding.py:306-379): estimate_strategy_comms_cost /
 * redistribute_cost / all_to_all_cost (collective_runtime_estimation.py:22-153),
 * torch allgather_cost / allreduce_cost / reduce_scatter_cost
 * (distributed/tensor/_collective_utils.py:281-313), the transition tie-break
 * (:345-351), the grad rescale (:358-359) and cost assembly (:368-372).
 * comm_out / transition_out / cost_out are [n_entries]; any may be NULL (an array that is not
 * wanted costs nothing: "all three" and "cost_out alone", the array the ILP objective is summed
 * from, are separate instantiations of the kernel on 2-D and 3-D meshes).
 * tensor_contiguous: see "Device arrays" above. */
int apc_redistribute_tables(const apc_params *params, const int64_t *tensor_bytes,
                            const uint8_t *tensor_contiguous, const uint32_t *spec_codes,
                            const int32_t *spec_tensor, const double *pt_values,
                            const double *compute_cost_per_arg, int64_t n_tiles, const apc_tile *tiles,
                            const int64_t *dup_entry_begin, int64_t n_entries, double *comm_out,
                            uint8_t *transition_out, double *cost_out, void *stream);

/* Every table of a pass in ONE launch: apc_input_tables + apc_redistribute_tables (same
 * arguments, same results: the union of the reference lines those replace).  The workgroups
 * that tile the cost matrices do not read tensor_bytes / tensor_contiguous /
 * compute_cost_per_arg, which other workgroups of the same launch are writing: they derive the
 * values they need from the tensor and strategy tables with the same device functions.  A
 * table of a few tens of MB (one transformer graph on a 2-D mesh) spends a third of each
 * launch ramping the chip up and draining it; this saves one of each.  The five spec-table
 * outputs may all be NULL (the spec table is then skipped: a planner computes it first and
 * alone, because the flop / byte counts passed here depend on it). */
int apc_build_tables(const apc_params *params, int64_t n_tensors, const int32_t *tensor_rank,
                     const int32_t *tensor_itemsize, const int64_t *tensor_shape, const int64_t *tensor_stride,
                     int64_t *tensor_bytes, uint8_t *tensor_contiguous, int64_t n_specs, const uint32_t *spec_codes,
                     const int32_t *spec_tensor, int64_t *num_shards, int64_t *local_shape, int64_t *local_stride,
                     int32_t shape_width, int64_t *local_numel, int64_t *local_bytes, int64_t n_strategies,
                     const int64_t *flops, const int64_t *rw_bytes, const int8_t *dtype_code,
                     const uint8_t *zero_cost, const int32_t *num_args, double *compute_cost,
                     double *compute_cost_per_arg, int32_t *error_flag, const double *pt_values, int64_t n_tiles,
                     const apc_tile *tiles,
                     const int64_t *dup_entry_begin, int64_t n_entries, double *comm_out, uint8_t *transition_out,
                     double *cost_out, void *stream);

/* Row minima taken by the launch that writes the cost matrices: for every matrix row (edge,
 * consumer strategy) the minimum of cost_out over the producer strategies and the first
 * column that has it, i.e. what apc_segmented_min gives over the rows of cost_out, without
 * reading the matrices again (and once per tiled edge, not once per identical copy).
 * Rows are numbered edge by edge: row = edge_row_begin[edge] + consumer strategy.
 * dup_row_begin[k] is the first row of the identical edge whose first entry is
 * dup_entry_begin[k] (NULL when dup_entry_begin is).
 * Precondition (apc_validate_row_minima_host checks it): every edge with rows has between 1
 * and APC_TILE_MAX_COLS producer strategies and every tile holds whole rows (col_begin = 0,
 * col_count = n_src); rows of tiles that do not are left unwritten.
 * The minima are those of the assembled cost whether or not cost_out is written.
 * No counterpart in the reference (see apc_segmented_min). */
typedef struct apc_row_minima {
  const int64_t *edge_row_begin; /* [n_edges] */
  const int64_t *dup_row_begin;  /* parallel to dup_entry_begin */
  double *row_min;               /* [n_rows] */
  int32_t *row_argmin;           /* [n_rows] */
} apc_row_minima;

/* Host-side check of the precondition above (HOST pointers); 0 when the row minima can be
 * taken by the table launch. */
int apc_validate_row_minima_host(int64_t n_edges, const int32_t *edge_n_src_host, const int32_t *edge_n_tgt_host,
                                 int64_t n_tiles, const apc_tile *tiles_host);

/* apc_redistribute_tables with the row minima; any of the three outputs may be NULL. */
int apc_redistribute_tables_row_min(const apc_params *params, const int64_t *tensor_bytes,
                                    const uint8_t *tensor_contiguous, const uint32_t *spec_codes,
                                    const int32_t *spec_tensor, const double *pt_values,
                                    const double *compute_cost_per_arg, int64_t n_tiles, const apc_tile *tiles,
                                    const int64_t *dup_entry_begin, int64_t n_entries, double *comm_out,
                                    uint8_t *transition_out, double *cost_out, const apc_row_minima *rows,
                                    void *stream);

/* apc_build_tables with the row minima; any of the three outputs may be NULL. */
int apc_build_tables_row_min(const apc_params *params, int64_t n_tensors, const int32_t *tensor_rank,
                             const int32_t *tensor_itemsize, const int64_t *tensor_shape,
                             const int64_t *tensor_stride, int64_t *tensor_bytes, uint8_t *tensor_contiguous,
                             int64_t n_specs, const uint32_t *spec_codes, const int32_t *spec_tensor,
                             int64_t *num_shards, int64_t *local_shape, int64_t *local_stride, int32_t shape_width,
                             int64_t *local_numel, int64_t *local_bytes, int64_t n_strategies, const int64_t *flops,
                             const int64_t *rw_bytes, const int8_t *dtype_code, const uint8_t *zero_cost,
                             const int32_t *num_args, double *compute_cost, double *compute_cost_per_arg,
                             int32_t *error_flag, const double *pt_values, int64_t n_tiles, const apc_tile *tiles,
                             const int64_t *dup_entry_begin, int64_t n_entries, double *comm_out,
                             uint8_t *transition_out, double *cost_out, const apc_row_minima *rows, void *stream);

/* Segmented minimum with first-argmin (relative to the segment start); empty
 * segments give (+inf, -1).  No counterpart in the reference (which hands the full
 * table to the ILP solver, optimize_sharding.py:648-659): used for pruning and
 * warm start.  n_values = seg_ptr[n_segments] (the host knows it; it selects how many lanes
 * share a segment). */
int apc_segmented_min(const double *values, const int64_t *seg_ptr, int64_t n_segments, int64_t n_values,
                      double *seg_min, int32_t *seg_argmin, void *stream);

/* apc_segmented_min over selected segments only, for value arrays in which whole segments
 * repeat (the rows of identical edges, which the table kernels fill with the same values):
 * segment selected[i] is reduced (seg_ptr indexed by segment id, as above) and its result is
 * stored at seg_min / seg_argmin [selected[i]] and at [copy_segments[k]] for k in
 * [copy_ptr[i], copy_ptr[i + 1]).  The caller vouches that those segments hold the same
 * values; segments that are neither selected nor a copy are left unwritten.
 * n_values_selected = total length of the selected segments.  No counterpart in the reference. */
int apc_segmented_min_copies(const double *values, const int64_t *seg_ptr, int64_t n_selected, const int64_t *selected,
                             const int64_t *copy_ptr, const int64_t *copy_segments, int64_t n_values_selected,
                             double *seg_min, int32_t *seg_argmin, void *stream);

/* Optimistic cost of every (node, strategy): bound[s] = sum, over the edges e of the node that
 * owns strategy s (edges_by_node[node_edge_begin[n] .. node_edge_begin[n + 1]), added in that
 * order), of row_min[edge_row_begin[e] + (s - node_strat_begin[n])], where row_min holds the
 * row minima of the cost matrices (apc_segmented_min over the rows) and edge_row_begin[e] is
 * the first row of edge e.  Every plan pays at least the row minimum of its consumer's
 * strategy on every edge, so apc_segmented_min of bound over node_strat_begin gives a lower
 * bound of the ILP objective (the sum of the minima) and a greedy strategy per node (the
 * argmin).  No counterpart in the reference (optimize_sharding.py:648-659 goes straight to
 * the solver): used for pruning and warm start.  The caller checks the index arrays. */
int apc_strategy_bounds(int64_t n_strategies, const int32_t *strat_node, const int64_t *node_strat_begin,
                        const int64_t *node_edge_begin, const int32_t *edges_by_node, const int64_t *edge_row_begin,
                        const double *row_min, double *bound, void *stream);

/* The ILP objective vector, summed on the device so that only one number per variable (not
 * three arrays per entry) has to leave it.
 * Replaces the accumulation at optimize_sharding.py:650-655 (opt_target[va] += cost over
 * ds.values(): entries that share a variable, optimize_sharding.py:211-231, add up in entry
 * order starting from 0) and the substitution of add_inf_cost_constraint (:522-536: a cost
 * that is not finite counts as inf_replacement, 10000.0 in the reference, and its variable is
 * forced to 0).
 * Variables are numbered group by group.  Group g owns variables [group_var_begin[g],
 * group_var_begin[g + 1]) and has members [group_member_begin[g], group_member_begin[g + 1]):
 * edges whose matrices have group_var_begin[g + 1] - group_var_begin[g] entries each and share
 * variables position by position; member_entry_begin[m] is the member's first entry, members
 * of a group in ascending order.  group_var_begin[0] is 0, group_var_begin[n_groups] is n_vars,
 * and no group is empty (group_var_begin ascends strictly); the arrays are device memory and
 * the caller checks them.  objective[v] / forced_zero[v] are [n_vars]. */
int apc_cost_objective(int64_t n_vars, int64_t n_groups, const int64_t *group_var_begin,
                       const int64_t *group_member_begin, const int64_t *member_entry_begin, const double *cost,
                       double inf_replacement, double *objective, uint8_t *forced_zero, void *stream);

/* Min-sum diffusion sweeps over the planning program written as a pairwise labelling problem
 * (no counterpart in the reference, which hands the whole program to the solver,
 * optimize_sharding.py:648-659): the row / column minima of the (reparametrised) cost matrices
 * are moved into the classes and handed back in equal shares, which raises the lower bound
 * sum_classes min unary + sum_edges min matrix  without changing the cost of any labelling.
 * The planner rounds an incumbent from the result and fixes to zero every variable whose bound
 * exceeds it (ILP pruning and warm start).
 *   class c        labels [label_begin[c], label_begin[c + 1]) of unary (f64, +inf = not allowed)
 *   edge k         matrix theta[edge_begin[k] ..], rows = labels of class edge_i[k], columns =
 *                  labels of class edge_j[k], row-major, +inf = forbidden pair
 *   incidence      edges of class c: inc_edge / inc_side [inc_begin[c], inc_begin[c + 1]),
 *                  side 0 = c labels the rows, 1 = the columns
 *   colours        color_nodes holds the classes grouped by colour, color_begin_host (HOST array,
 *                  n_colors + 1) the groups; two classes of one colour share no edge.
 * One sweep = one launch per colour, in order; theta and unary are updated in place.
 * max_labels = the largest label count of a class (at most 2048). */
int apc_diffusion_sweeps(int32_t n_sweeps, int32_t n_colors, const int64_t *color_begin_host,
                         const int32_t *color_nodes, int64_t n_classes, const int64_t *label_begin,
                         const int64_t *inc_begin, const int32_t *inc_edge, const uint8_t *inc_side,
                         const int64_t *edge_begin, const int32_t *edge_i, const int32_t *edge_j, int32_t max_labels,
                         double *theta, double *unary, void *stream);

/* apc_redistribute_tables for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  It takes the tensor and strategy tables themselves instead of the staging tables
 * apc_input_tables would write from them (tensor_bytes, tensor_contiguous,
 * compute_cost_per_arg): those are staged in a fixed device array inside the library (17.1 MB
 * that every GPU the library runs on holds until the process ends), at most 65 536 tensors and
 * 2 097 152 strategies; larger tables are rejected with an error.  Two launches on `stream`
 * (staging, then the tiles); no hipMalloc / hipFree, no synchronisation.  Results equal those of
 * apc_input_tables followed by apc_redistribute_tables.  All calls on one GPU share the array:
 * calls that overlap on a GPU (two streams, two threads) race: a call on another stream must be
 * ordered (an event, a synchronisation) after the previous call's tile launch has finished, not
 * merely after it was enqueued.  A strategy with flops whose
 * dtype has no throughput on the device row yields NaN costs (there is no error flag). */
int apc_redistribute_tables_static(const apc_params *params, int64_t n_tensors, const int32_t *tensor_rank,
                                   const int32_t *tensor_itemsize, const int64_t *tensor_shape,
                                   const int64_t *tensor_stride, int64_t n_strategies, const int64_t *flops,
                                   const int64_t *rw_bytes, const int8_t *dtype_code, const uint8_t *zero_cost,
                                   const int32_t *num_args, const uint32_t *spec_codes, const int32_t *spec_tensor,
                                   const double *pt_values, int64_t n_tiles, const apc_tile *tiles,
                                   const int64_t *dup_entry_begin, int64_t n_entries, double *comm_out,
                                   uint8_t *transition_out, double *cost_out, void *stream);

/* ---- packed tiles: the table pass of a small graph in one round of loads ----------------------
 * A table of a few million entries is bound by the latency of one workgroup, not by bytes: the
 * chain "tile record -> spec rows, strategy rows, tensor row, identical edges' offsets -> compute"
 * costs more than the stores.  A packed tile holds everything one tile reads, copied out of the
 * tables above by the host into one fixed-size record, so that a workgroup's loads depend on
 * nothing but its own index.  It describes whole rows of one edge's matrix (cols = the edge's
 * producer count <= APC_TILE_MAX_COLS, rows <= APC_TILE_MAX_ROWS) and at most APC_PACKED_MAX_DUPS
 * identical edges.  apc_validate_packed_tiles_host checks every record against the tables it
 * was copied from.  The values computed from it are those of apc_build_tables_row_min. */
#define APC_PACKED_MAX_DUPS 16
#define APC_PACKED_MIXED 0x100 /* flags: some spec of the tile is not a DTensorSpec, or a producer spec names
                                  another tensor than `tensor`: entries are evaluated one by one */
typedef struct apc_packed_tile {
  int32_t rows, cols;      /* consumer / producer strategies of the tile (cols = edge_n_src[edge]) */
  int32_t flags;           /* edge_flags[edge] | APC_PACKED_MIXED */
  int32_t dup_count;       /* identical edges that receive the same values */
  int32_t tensor;          /* spec_tensor of the first producer spec, -1: none */
  int32_t tensor_rank;     /* rank / itemsize / shape / stride rows of that tensor (zeros when none) */
  int32_t tensor_itemsize;
  int32_t edge;
  int64_t entry_begin;     /* first entry of the tile: edge_entry_begin[edge] + row_begin * cols */
  int64_t row_begin;       /* its first matrix row: edge_row_begin[edge] + row_begin (rows numbered edge by edge) */
  int64_t pt_begin;        /* pt_values offset of its first entry (edge_pt_begin[edge] + row_begin * cols), -1: none */
  int64_t reserved;
  int64_t tensor_shape[APC_MAX_RANK];
  int64_t tensor_stride[APC_MAX_RANK];
  int64_t dup_entry_begin[APC_PACKED_MAX_DUPS]; /* the tile's first entry in every identical edge */
  int64_t dup_row_begin[APC_PACKED_MAX_DUPS];   /* its first matrix row there */
  uint32_t col_codes[APC_TILE_MAX_COLS];        /* producer specs: placement codes, tensor rows */
  int32_t col_tensor[APC_TILE_MAX_COLS];
  uint32_t row_codes[APC_TILE_MAX_ROWS];        /* consumer specs */
  int32_t row_tensor[APC_TILE_MAX_ROWS];
  int64_t row_flops[APC_TILE_MAX_ROWS];         /* the consumer strategies' rows of the strategy table */
  int64_t row_rw_bytes[APC_TILE_MAX_ROWS];
  int32_t row_meta[APC_TILE_MAX_ROWS];          /* dtype code (low byte, signed) | zero_cost << 8 | num_args << 16 */
} apc_packed_tile;

/* Host-side check (HOST pointers) that packed[t] repeats, field by field, what tiles[t] and the
 * tables say; tiles must hold whole rows (apc_validate_row_minima_host) and at most
 * APC_PACKED_MAX_DUPS identical edges each.  edge_row_begin[e] = first matrix row of edge e. */
int apc_validate_packed_tiles_host(int64_t n_tensors, const int32_t *tensor_rank_host, const int32_t *tensor_itemsize_host,
                                   const int64_t *tensor_shape_host, const int64_t *tensor_stride_host, int64_t n_specs,
                                   const uint32_t *spec_codes_host, const int32_t *spec_tensor_host, int64_t n_strategies,
                                   const int64_t *flops_host, const int64_t *rw_bytes_host, const int8_t *dtype_code_host,
                                   const uint8_t *zero_cost_host, const int32_t *num_args_host, int64_t n_edges,
                                   const int64_t *edge_row_begin_host, int64_t n_tiles, const apc_tile *tiles_host,
                                   int64_t n_dups, const int64_t *dup_entry_begin_host, const int64_t *dup_row_begin_host,
                                   const apc_packed_tile *packed_host);

/* The table pass of a planner over packed tiles, ONE launch: the tensor table, the compute costs,
 * the assembled cost of every entry and the row minima (what apc_build_tables_row_min writes with
 * cost_out alone and no spec table; same reference lines, same values).  Every wavefront works
 * on its own: it reads the tile's record, evaluates whole matrix rows entry by entry in
 * registers (collective_runtime_estimation.py:37-153 directly, no staging in LDS, no barrier),
 * takes their minima and stores values and minima to the tile's edge and to every identical
 * edge.  tensor_* / strategy arrays as in apc_build_tables (a tile whose producer specs name
 * several tensors reads the tensor table).  cost_out [n_entries], row_min / row_argmin [n_rows].
 * The cost entries and the table rows are written through to memory (a launch of this size would
 * otherwise wait, after its last wavefront, for the L2 to write them back). */
int apc_build_tables_packed(const apc_params *params, int64_t n_tensors, const int32_t *tensor_rank,
                            const int32_t *tensor_itemsize, const int64_t *tensor_shape, const int64_t *tensor_stride,
                            int64_t *tensor_bytes, uint8_t *tensor_contiguous, int64_t n_strategies, const int64_t *flops,
                            const int64_t *rw_bytes, const int8_t *dtype_code, const uint8_t *zero_cost,
                            const int32_t *num_args, double *compute_cost, double *compute_cost_per_arg,
                            int32_t *error_flag, const double *pt_values, int64_t n_tiles, const apc_packed_tile *packed,
                            int64_t n_entries, double *cost_out, double *row_min, int32_t *row_argmin, void *stream);

/* Measurement aids, no counterpart in the reference.  apc_calibrate_launch enqueues a kernel that
 * does nothing (n_workgroups workgroups of `threads` threads): launched back to back it shows what
 * a launch costs on the system before any work.  apc_calibrate_fill enqueues a kernel that only
 * writes: out[0 .. n) = value, workgroup b taking doubles [b * per_workgroup, (b + 1) *
 * per_workgroup) (even, >= 2; 256 threads, 16-byte stores; out 16-byte aligned): the ceiling of
 * the store path for a launch that moves the same bytes as a table build.  write_through != 0:
 * the stores are written through to memory instead of being left in the L2 until the kernel ends
 * (what apc_build_tables_packed does with its own stores; the faster of the two on a launch of a
 * few tens of MB, the slower on one that streams through the L2). */
int apc_calibrate_launch(int64_t n_workgroups, int32_t threads, void *stream);
int apc_calibrate_fill(double *out, int64_t n, int64_t per_workgroup, double value, int32_t write_through, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* APCOST_H */
