// Torch layer over the C ABI of libapcost.so (include/apcost.h): operators of the `apcost`
// namespace that take and return torch tensors on the HIP device, check their arguments with
// TORCH_CHECK (dtype, device, contiguity, lengths that must agree), run on the current HIP
// stream of the tensors' device under a device guard, and turn the library's error codes into
// RuntimeError.  No computation happens here and nothing falls back to the CPU: every operator
// is one launch of the library.
//
//   apcost::tensor_tables, apcost::shard_shapes_bytes   local shard shapes / byte counts
//       (torch _dtensor_spec.py:555-561, _utils.py compute_local_shape; compute_estimation.py:211-231)
//   apcost::compute_cost                                per-strategy roofline estimate
//       (compute_estimation.py:334-365)
//   apcost::redistribute_cost_tables                    per-edge producer x consumer matrices
//       (collective_runtime_estimation.py:37-153 assembled as optimize_sharding.py:300-372)
//   apcost::segmented_min                               row minima + first argmin
//   apcost::cost_objective                              ILP objective coefficients
//       (optimize_sharding.py:650-655)
//   apcost::bind_*  ->  apcost.BoundLaunch              a launch with its arguments checked and
//       bound once, for callers that repeat it (the planner's table pass): run() only looks up
//       the current stream and enqueues.
//
// Built against the installed torch: autoparallel_amd/_build.py (build_torch_extension).

#include <ATen/ATen.h>
#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/custom_class.h>
#include <torch/library.h>

#include <cstring>
#include <functional>
#include <optional>
#include <string>
#include <tuple>
#include <vector>

#include "apcost.h"

namespace {

using at::Tensor;
using OptTensor = std::optional<Tensor>;

void check_device_tensor(const Tensor &t, at::ScalarType dtype, const char *name) {
  TORCH_CHECK(t.defined(), "apcost: ", name, " is undefined");
  TORCH_CHECK(t.is_cuda(), "apcost: ", name, " must be on the HIP device (got ", t.device(), ")");
  TORCH_CHECK(t.scalar_type() == dtype, "apcost: ", name, " must be ", dtype, " (got ", t.scalar_type(), ")");
  TORCH_CHECK(t.is_contiguous(), "apcost: ", name, " must be contiguous");
}

// Pointer of a checked device tensor (NULL for an empty one: the library accepts NULL for
// arrays of no rows).
template <typename T>
T *dev(const Tensor &t, at::ScalarType dtype, const char *name) {
  check_device_tensor(t, dtype, name);
  return t.numel() ? static_cast<T *>(t.data_ptr()) : nullptr;
}
template <typename T>
T *dev_opt(const OptTensor &t, at::ScalarType dtype, const char *name) {
  if (!t.has_value() || !t->defined()) return nullptr;
  return dev<T>(*t, dtype, name);
}
// Placement codes and tile records travel as int32 words (torch's uint32 support is partial).
const uint32_t *codes_of(const Tensor &t) { return reinterpret_cast<const uint32_t *>(dev<int32_t>(t, at::kInt, "spec_codes")); }

void same_device(const Tensor &a, const Tensor &b, const char *what) {
  TORCH_CHECK(a.device() == b.device(), "apcost: ", what, " is on ", b.device(), ", expected ", a.device());
}

// apc_params as the bytes of the C struct in a CPU uint8 tensor.
apc_params params_of(const Tensor &p) {
  TORCH_CHECK(p.defined() && p.device().is_cpu() && p.scalar_type() == at::kByte && p.is_contiguous(),
              "apcost: params must be a contiguous CPU uint8 tensor holding struct apc_params");
  TORCH_CHECK(p.numel() == (int64_t)sizeof(apc_params), "apcost: params holds ", p.numel(), " bytes, struct apc_params has ",
              sizeof(apc_params));
  apc_params out;
  std::memcpy(&out, p.data_ptr(), sizeof(out));
  TORCH_CHECK(out.mesh_ndim >= 1 && out.mesh_ndim <= APC_MAX_MESH, "apcost: mesh_ndim ", out.mesh_ndim, " outside [1, ",
              APC_MAX_MESH, "]");
  return out;
}

void check_rc(int rc, const char *what) { TORCH_CHECK(rc == 0, what, ": ", apc_last_error(), " (code ", rc, ")"); }

// Runs `launch(stream)` on the current stream of `device` with that device current.
template <typename F>
void on_current_stream(const at::Device &device, const char *what, F &&launch) {
  c10::hip::HIPGuard guard(device.index());
  void *stream = c10::hip::getCurrentHIPStream(device.index()).stream();
  check_rc(launch(stream), what);
}

Tensor empty_like_device(const Tensor &ref, at::IntArrayRef shape, at::ScalarType dtype) {
  return at::empty(shape, ref.options().dtype(dtype));
}

struct TensorTable {  // rank / itemsize / shape / stride of the global tensors
  const int32_t *rank, *itemsize;
  const int64_t *shape, *stride;
  int64_t n;
};
TensorTable tensor_table(const Tensor &rank, const Tensor &itemsize, const Tensor &shape, const Tensor &stride) {
  TensorTable t{dev<int32_t>(rank, at::kInt, "tensor_rank"), dev<int32_t>(itemsize, at::kInt, "tensor_itemsize"),
                dev<int64_t>(shape, at::kLong, "tensor_shape"), dev<int64_t>(stride, at::kLong, "tensor_stride"), rank.numel()};
  TORCH_CHECK(itemsize.numel() == t.n, "apcost: tensor_itemsize has ", itemsize.numel(), " rows, tensor_rank ", t.n);
  TORCH_CHECK(shape.numel() == t.n * APC_MAX_RANK && stride.numel() == t.n * APC_MAX_RANK,
              "apcost: tensor_shape / tensor_stride must be [n_tensors, ", APC_MAX_RANK, "]");
  same_device(rank, itemsize, "tensor_itemsize");
  same_device(rank, shape, "tensor_shape");
  same_device(rank, stride, "tensor_stride");
  return t;
}

struct StrategyTable {
  const int64_t *flops, *rw_bytes;
  const int8_t *dtype;
  const uint8_t *zero_cost;
  const int32_t *num_args;
  int64_t n;
};
StrategyTable strategy_table(const Tensor &flops, const Tensor &rw_bytes, const Tensor &dtype, const Tensor &zero_cost,
                             const Tensor &num_args) {
  StrategyTable s{dev<int64_t>(flops, at::kLong, "flops"), dev<int64_t>(rw_bytes, at::kLong, "rw_bytes"),
                  dev<int8_t>(dtype, at::kChar, "dtype_code"), dev<uint8_t>(zero_cost, at::kByte, "zero_cost"),
                  dev<int32_t>(num_args, at::kInt, "num_args"), flops.numel()};
  TORCH_CHECK(rw_bytes.numel() == s.n && dtype.numel() == s.n && zero_cost.numel() == s.n && num_args.numel() == s.n,
              "apcost: the strategy arrays must have one row per strategy (", s.n, ")");
  return s;
}

// ---- functional operators --------------------------------------------------------------------

std::tuple<Tensor, Tensor> tensor_tables(const Tensor &rank, const Tensor &itemsize, const Tensor &shape, const Tensor &stride) {
  const TensorTable t = tensor_table(rank, itemsize, shape, stride);
  Tensor bytes = empty_like_device(rank, {t.n}, at::kLong), contiguous = empty_like_device(rank, {t.n}, at::kByte);
  on_current_stream(rank.device(), "apc_tensor_tables", [&](void *s) {
    return apc_tensor_tables(t.n, t.rank, t.itemsize, t.shape, t.stride, t.n ? bytes.data_ptr<int64_t>() : nullptr,
                             t.n ? contiguous.data_ptr<uint8_t>() : nullptr, s);
  });
  return {bytes, contiguous};
}

std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor> shard_shapes_bytes(const Tensor &params, const Tensor &spec_codes,
                                                                      const Tensor &spec_tensor, const Tensor &rank,
                                                                      const Tensor &itemsize, const Tensor &shape,
                                                                      const Tensor &stride, int64_t shape_width) {
  const apc_params p = params_of(params);
  const TensorTable t = tensor_table(rank, itemsize, shape, stride);
  const int64_t n = spec_codes.numel();
  const uint32_t *codes = codes_of(spec_codes);
  const int32_t *owner = dev<int32_t>(spec_tensor, at::kInt, "spec_tensor");
  TORCH_CHECK(spec_tensor.numel() == n, "apcost: spec_tensor has ", spec_tensor.numel(), " rows, spec_codes ", n);
  TORCH_CHECK(shape_width >= 1 && shape_width <= APC_MAX_RANK, "apcost: shape_width ", shape_width, " outside [1, ", APC_MAX_RANK, "]");
  same_device(spec_codes, rank, "tensor_rank");
  Tensor num_shards = empty_like_device(spec_codes, {n}, at::kLong), local_shape = empty_like_device(spec_codes, {n, shape_width}, at::kLong),
         local_stride = empty_like_device(spec_codes, {n, shape_width}, at::kLong), local_numel = empty_like_device(spec_codes, {n}, at::kLong),
         local_bytes = empty_like_device(spec_codes, {n}, at::kLong);
  on_current_stream(spec_codes.device(), "apc_spec_tables", [&](void *s) {
    return apc_spec_tables(&p, n, codes, owner, t.rank, t.itemsize, t.shape, t.stride, static_cast<int64_t *>(num_shards.data_ptr()),
                           static_cast<int64_t *>(local_shape.data_ptr()), static_cast<int64_t *>(local_stride.data_ptr()),
                           (int32_t)shape_width, static_cast<int64_t *>(local_numel.data_ptr()),
                           static_cast<int64_t *>(local_bytes.data_ptr()), s);
  });
  return {num_shards, local_shape, local_stride, local_numel, local_bytes};
}

std::tuple<Tensor, Tensor, Tensor> compute_cost(const Tensor &params, const Tensor &flops, const Tensor &rw_bytes,
                                                const Tensor &dtype, const Tensor &zero_cost, const Tensor &num_args) {
  const apc_params p = params_of(params);
  const StrategyTable st = strategy_table(flops, rw_bytes, dtype, zero_cost, num_args);
  Tensor compute = empty_like_device(flops, {st.n}, at::kDouble), per_arg = empty_like_device(flops, {st.n}, at::kDouble),
         error_flag = at::zeros({1}, flops.options().dtype(at::kInt));
  on_current_stream(flops.device(), "apc_compute_costs", [&](void *s) {
    return apc_compute_costs(&p, st.n, st.flops, st.rw_bytes, st.dtype, st.zero_cost, st.num_args,
                             static_cast<double *>(compute.data_ptr()), static_cast<double *>(per_arg.data_ptr()),
                             error_flag.data_ptr<int32_t>(), s);
  });
  return {compute, per_arg, error_flag};
}

std::tuple<Tensor, Tensor> segmented_min(const Tensor &values, const Tensor &seg_ptr) {
  const double *v = dev<double>(values, at::kDouble, "values");
  const int64_t *ptr = dev<int64_t>(seg_ptr, at::kLong, "seg_ptr");
  TORCH_CHECK(seg_ptr.numel() >= 1, "apcost: seg_ptr needs n_segments + 1 rows");
  same_device(values, seg_ptr, "seg_ptr");
  const int64_t n_seg = seg_ptr.numel() - 1;
  Tensor mins = empty_like_device(values, {n_seg}, at::kDouble), args = empty_like_device(values, {n_seg}, at::kInt);
  on_current_stream(values.device(), "apc_segmented_min", [&](void *s) {
    return apc_segmented_min(v, ptr, n_seg, values.numel(), static_cast<double *>(mins.data_ptr()), args.data_ptr<int32_t>(), s);
  });
  return {mins, args};
}

std::tuple<Tensor, Tensor> cost_objective(int64_t n_vars, const Tensor &group_var_begin, const Tensor &group_member_begin,
                                          const Tensor &member_entry_begin, const Tensor &cost, double inf_replacement) {
  const int64_t *gvb = dev<int64_t>(group_var_begin, at::kLong, "group_var_begin");
  const int64_t *gmb = dev<int64_t>(group_member_begin, at::kLong, "group_member_begin");
  const int64_t *meb = dev<int64_t>(member_entry_begin, at::kLong, "member_entry_begin");
  const double *c = dev<double>(cost, at::kDouble, "cost");
  TORCH_CHECK(n_vars >= 0 && group_var_begin.numel() >= 1 && group_member_begin.numel() == group_var_begin.numel(),
              "apcost: group_var_begin / group_member_begin need n_groups + 1 rows each");
  same_device(cost, group_var_begin, "group_var_begin");
  same_device(cost, group_member_begin, "group_member_begin");
  same_device(cost, member_entry_begin, "member_entry_begin");
  Tensor objective = empty_like_device(cost, {n_vars}, at::kDouble), forced = empty_like_device(cost, {n_vars}, at::kByte);
  on_current_stream(cost.device(), "apc_cost_objective", [&](void *s) {
    return apc_cost_objective(n_vars, group_var_begin.numel() - 1, gvb, gmb, meb, c, inf_replacement,
                              static_cast<double *>(objective.data_ptr()), forced.data_ptr<uint8_t>(), s);
  });
  return {objective, forced};
}

// ---- launches bound once ---------------------------------------------------------------------

struct BoundLaunch : torch::CustomClassHolder {
  std::string what;
  at::Device device{at::kCPU};
  std::function<int(void *)> launch;
  std::vector<Tensor> keep;  // every tensor whose memory the launch reads or writes

  void run() {
    c10::hip::HIPGuard guard(device.index());
    check_rc(launch(c10::hip::getCurrentHIPStream(device.index()).stream()), what.c_str());
  }
  // The launch on a stream given by its handle (torch.cuda.Stream.cuda_stream).
  void run_on(int64_t stream) {
    c10::hip::HIPGuard guard(device.index());
    check_rc(launch(reinterpret_cast<void *>(stream)), what.c_str());
  }
  std::string name() const { return what; }
};

struct Outputs {  // per-entry arrays a table launch writes (each optional) and the row minima
  double *comm = nullptr;
  uint8_t *transition = nullptr;
  double *cost = nullptr;
  bool rows = false;
  apc_row_minima row_minima{};
};

Outputs outputs_of(int64_t n_entries, const OptTensor &comm, const OptTensor &transition, const OptTensor &cost,
                   const OptTensor &edge_row_begin, const OptTensor &dup_row_begin, const OptTensor &row_min,
                   const OptTensor &row_argmin, std::vector<Tensor> &keep) {
  Outputs o;
  o.comm = dev_opt<double>(comm, at::kDouble, "comm");
  o.transition = dev_opt<uint8_t>(transition, at::kByte, "transition");
  o.cost = dev_opt<double>(cost, at::kDouble, "cost");
  for (const OptTensor *t : {&comm, &transition, &cost})
    if (t->has_value() && (*t)->defined()) {
      TORCH_CHECK((*t)->numel() == n_entries, "apcost: a per-entry output has ", (*t)->numel(), " rows, the table ", n_entries, " entries");
      keep.push_back(**t);
    }
  const bool any_rows = row_min.has_value() || row_argmin.has_value() || edge_row_begin.has_value();
  if (any_rows) {
    TORCH_CHECK(row_min.has_value() && row_argmin.has_value() && edge_row_begin.has_value(),
                "apcost: row minima need edge_row_begin, row_min and row_argmin together");
    o.rows = true;
    o.row_minima.edge_row_begin = dev<int64_t>(*edge_row_begin, at::kLong, "edge_row_begin");
    o.row_minima.dup_row_begin = dev_opt<int64_t>(dup_row_begin, at::kLong, "dup_row_begin");
    o.row_minima.row_min = dev<double>(*row_min, at::kDouble, "row_min");
    o.row_minima.row_argmin = dev<int32_t>(*row_argmin, at::kInt, "row_argmin");
    TORCH_CHECK(row_min->numel() == row_argmin->numel(), "apcost: row_min and row_argmin differ in length");
    keep.push_back(*edge_row_begin);
    keep.push_back(*row_min);
    keep.push_back(*row_argmin);
    if (dup_row_begin.has_value()) keep.push_back(*dup_row_begin);
  }
  return o;
}

const apc_tile *tiles_of(const Tensor &tiles, int64_t &n_tiles) {
  const int32_t *words = dev<int32_t>(tiles, at::kInt, "tiles");
  constexpr int64_t kWords = sizeof(apc_tile) / 4;
  TORCH_CHECK(tiles.numel() % kWords == 0, "apcost: tiles must be [n_tiles, ", kWords, "] int32 words (struct apc_tile)");
  n_tiles = tiles.numel() / kWords;
  return reinterpret_cast<const apc_tile *>(words);
}

// apc_redistribute_tables[_row_min] over tables the caller has built.
c10::intrusive_ptr<BoundLaunch> bind_redistribute_tables(
    const Tensor &params, const Tensor &tensor_bytes, const Tensor &tensor_contiguous, const Tensor &spec_codes,
    const Tensor &spec_tensor, const Tensor &pt_values, const OptTensor &per_arg, const Tensor &tiles,
    const Tensor &dup_entry_begin, int64_t n_entries, const OptTensor &comm, const OptTensor &transition,
    const OptTensor &cost, const OptTensor &edge_row_begin, const OptTensor &dup_row_begin, const OptTensor &row_min,
    const OptTensor &row_argmin) {
  auto b = c10::make_intrusive<BoundLaunch>();
  const apc_params p = params_of(params);
  const int64_t *bytes = dev<int64_t>(tensor_bytes, at::kLong, "tensor_bytes");
  const uint8_t *contiguous = dev<uint8_t>(tensor_contiguous, at::kByte, "tensor_contiguous");
  TORCH_CHECK(tensor_bytes.numel() == tensor_contiguous.numel(), "apcost: tensor_bytes and tensor_contiguous differ in length");
  const uint32_t *codes = codes_of(spec_codes);
  const int32_t *owner = dev<int32_t>(spec_tensor, at::kInt, "spec_tensor");
  TORCH_CHECK(spec_tensor.numel() == spec_codes.numel(), "apcost: spec_tensor and spec_codes differ in length");
  const double *pt = dev<double>(pt_values, at::kDouble, "pt_values");
  const double *cpa = dev_opt<double>(per_arg, at::kDouble, "compute_cost_per_arg");
  int64_t n_tiles = 0;
  const apc_tile *tile_records = tiles_of(tiles, n_tiles);
  const int64_t *dups = dev<int64_t>(dup_entry_begin, at::kLong, "dup_entry_begin");
  for (const Tensor *t : {&tensor_contiguous, &spec_codes, &spec_tensor, &pt_values, &tiles, &dup_entry_begin}) {
    same_device(tensor_bytes, *t, "a table");
    b->keep.push_back(*t);
  }
  b->keep.push_back(tensor_bytes);
  if (per_arg.has_value()) b->keep.push_back(*per_arg);
  const Outputs o = outputs_of(n_entries, comm, transition, cost, edge_row_begin, dup_row_begin, row_min, row_argmin, b->keep);
  TORCH_CHECK(comm.has_value() || transition.has_value() || cost.has_value(), "apcost: no per-entry output given");
  b->what = o.rows ? "apc_redistribute_tables_row_min" : "apc_redistribute_tables";
  b->device = tensor_bytes.device();
  b->launch = [=](void *s) {
    if (o.rows)
      return apc_redistribute_tables_row_min(&p, bytes, contiguous, codes, owner, pt, cpa, n_tiles, tile_records, dups, n_entries,
                                             o.comm, o.transition, o.cost, &o.row_minima, s);
    return apc_redistribute_tables(&p, bytes, contiguous, codes, owner, pt, cpa, n_tiles, tile_records, dups, n_entries, o.comm,
                                   o.transition, o.cost, s);
  };
  return b;
}

struct InputTables {  // arguments shared by apc_input_tables and apc_build_tables
  apc_params p;
  TensorTable t;
  int64_t *tensor_bytes;
  uint8_t *tensor_contiguous;
  int64_t n_specs;
  const uint32_t *codes;
  const int32_t *owner;
  int64_t *num_shards = nullptr, *local_shape = nullptr, *local_stride = nullptr, *local_numel = nullptr, *local_bytes = nullptr;
  int32_t shape_width = APC_MAX_RANK;
  StrategyTable st;
  double *compute, *per_arg;
  int32_t *error_flag;
};

InputTables input_tables_of(const Tensor &params, const Tensor &rank, const Tensor &itemsize, const Tensor &shape,
                            const Tensor &stride, const Tensor &tensor_bytes, const Tensor &tensor_contiguous,
                            const Tensor &spec_codes, const Tensor &spec_tensor, const std::vector<Tensor> &spec_outputs,
                            int64_t shape_width, const Tensor &flops, const Tensor &rw_bytes, const Tensor &dtype,
                            const Tensor &zero_cost, const Tensor &num_args, const Tensor &compute, const Tensor &per_arg,
                            const Tensor &error_flag, std::vector<Tensor> &keep) {
  InputTables in;
  in.p = params_of(params);
  in.t = tensor_table(rank, itemsize, shape, stride);
  in.tensor_bytes = dev<int64_t>(tensor_bytes, at::kLong, "tensor_bytes");
  in.tensor_contiguous = dev<uint8_t>(tensor_contiguous, at::kByte, "tensor_contiguous");
  TORCH_CHECK(tensor_bytes.numel() == in.t.n && tensor_contiguous.numel() == in.t.n, "apcost: tensor_bytes / tensor_contiguous need one row per tensor");
  in.n_specs = spec_codes.numel();
  in.codes = codes_of(spec_codes);
  in.owner = dev<int32_t>(spec_tensor, at::kInt, "spec_tensor");
  TORCH_CHECK(spec_tensor.numel() == in.n_specs, "apcost: spec_tensor and spec_codes differ in length");
  TORCH_CHECK(spec_outputs.empty() || spec_outputs.size() == 5,
              "apcost: the spec table has five outputs (num_shards, local_shape, local_stride, local_numel, local_bytes) or none");
  if (!spec_outputs.empty()) {
    TORCH_CHECK(shape_width >= 1 && shape_width <= APC_MAX_RANK, "apcost: shape_width ", shape_width, " outside [1, ", APC_MAX_RANK, "]");
    in.shape_width = (int32_t)shape_width;
    in.num_shards = dev<int64_t>(spec_outputs[0], at::kLong, "num_shards");
    in.local_shape = dev<int64_t>(spec_outputs[1], at::kLong, "local_shape");
    in.local_stride = dev<int64_t>(spec_outputs[2], at::kLong, "local_stride");
    in.local_numel = dev<int64_t>(spec_outputs[3], at::kLong, "local_numel");
    in.local_bytes = dev<int64_t>(spec_outputs[4], at::kLong, "local_bytes");
    TORCH_CHECK(spec_outputs[0].numel() == in.n_specs && spec_outputs[3].numel() == in.n_specs && spec_outputs[4].numel() == in.n_specs &&
                    spec_outputs[1].numel() == in.n_specs * shape_width && spec_outputs[2].numel() == in.n_specs * shape_width,
                "apcost: the spec table's outputs need one row per spec (local shape / stride rows shape_width wide)");
    for (const Tensor &t : spec_outputs) keep.push_back(t);
  }
  in.st = strategy_table(flops, rw_bytes, dtype, zero_cost, num_args);
  in.compute = dev<double>(compute, at::kDouble, "compute_cost");
  in.per_arg = dev<double>(per_arg, at::kDouble, "compute_cost_per_arg");
  TORCH_CHECK(compute.numel() == in.st.n && per_arg.numel() == in.st.n, "apcost: compute_cost / compute_cost_per_arg need one row per strategy");
  in.error_flag = dev<int32_t>(error_flag, at::kInt, "error_flag");
  TORCH_CHECK(error_flag.numel() >= 1, "apcost: error_flag needs one element");
  for (const Tensor *t : {&rank, &itemsize, &shape, &stride, &tensor_bytes, &tensor_contiguous, &spec_codes, &spec_tensor, &flops,
                          &rw_bytes, &dtype, &zero_cost, &num_args, &compute, &per_arg, &error_flag}) {
    same_device(rank, *t, "a table");
    keep.push_back(*t);
  }
  return in;
}

#define APCOST_INPUT_TABLE_PARAMS                                                                                          \
  const Tensor &params, const Tensor &rank, const Tensor &itemsize, const Tensor &shape, const Tensor &stride,             \
      const Tensor &tensor_bytes, const Tensor &tensor_contiguous, const Tensor &spec_codes, const Tensor &spec_tensor,    \
      std::vector<Tensor> spec_outputs, int64_t shape_width, const Tensor &flops, const Tensor &rw_bytes,                  \
      const Tensor &dtype, const Tensor &zero_cost, const Tensor &num_args, const Tensor &compute, const Tensor &per_arg,  \
      const Tensor &error_flag
#define APCOST_INPUT_TABLE_ARGS                                                                                            \
  params, rank, itemsize, shape, stride, tensor_bytes, tensor_contiguous, spec_codes, spec_tensor, spec_outputs,           \
      shape_width, flops, rw_bytes, dtype, zero_cost, num_args, compute, per_arg, error_flag

// apc_input_tables: tensor table, compute costs and (with spec_outputs) the spec table in one launch.
c10::intrusive_ptr<BoundLaunch> bind_input_tables(APCOST_INPUT_TABLE_PARAMS) {
  auto b = c10::make_intrusive<BoundLaunch>();
  const InputTables in = input_tables_of(APCOST_INPUT_TABLE_ARGS, b->keep);
  b->what = "apc_input_tables";
  b->device = rank.device();
  b->launch = [=](void *s) {
    return apc_input_tables(&in.p, in.t.n, in.t.rank, in.t.itemsize, in.t.shape, in.t.stride, in.tensor_bytes, in.tensor_contiguous,
                            in.n_specs, in.codes, in.owner, in.num_shards, in.local_shape, in.local_stride, in.shape_width,
                            in.local_numel, in.local_bytes, in.st.n, in.st.flops, in.st.rw_bytes, in.st.dtype, in.st.zero_cost,
                            in.st.num_args, in.compute, in.per_arg, in.error_flag, s);
  };
  return b;
}

// apc_build_tables[_row_min]: every table of a pass in one launch.
c10::intrusive_ptr<BoundLaunch> bind_cost_tables(APCOST_INPUT_TABLE_PARAMS, const Tensor &pt_values, const Tensor &tiles,
                                                 const Tensor &dup_entry_begin, int64_t n_entries, const OptTensor &comm,
                                                 const OptTensor &transition, const OptTensor &cost,
                                                 const OptTensor &edge_row_begin, const OptTensor &dup_row_begin,
                                                 const OptTensor &row_min, const OptTensor &row_argmin) {
  auto b = c10::make_intrusive<BoundLaunch>();
  const InputTables in = input_tables_of(APCOST_INPUT_TABLE_ARGS, b->keep);
  const double *pt = dev<double>(pt_values, at::kDouble, "pt_values");
  int64_t n_tiles = 0;
  const apc_tile *tile_records = tiles_of(tiles, n_tiles);
  const int64_t *dups = dev<int64_t>(dup_entry_begin, at::kLong, "dup_entry_begin");
  for (const Tensor *t : {&pt_values, &tiles, &dup_entry_begin}) {
    same_device(rank, *t, "a table");
    b->keep.push_back(*t);
  }
  const Outputs o = outputs_of(n_entries, comm, transition, cost, edge_row_begin, dup_row_begin, row_min, row_argmin, b->keep);
  b->what = o.rows ? "apc_build_tables_row_min" : "apc_build_tables";
  b->device = rank.device();
  b->launch = [=](void *s) {
#define APCOST_BUILD_ARGS                                                                                                  \
  &in.p, in.t.n, in.t.rank, in.t.itemsize, in.t.shape, in.t.stride, in.tensor_bytes, in.tensor_contiguous, in.n_specs,     \
      in.codes, in.owner, in.num_shards, in.local_shape, in.local_stride, in.shape_width, in.local_numel, in.local_bytes,  \
      in.st.n, in.st.flops, in.st.rw_bytes, in.st.dtype, in.st.zero_cost, in.st.num_args, in.compute, in.per_arg,          \
      in.error_flag, pt, n_tiles, tile_records, dups, n_entries, o.comm, o.transition, o.cost
    if (o.rows) return apc_build_tables_row_min(APCOST_BUILD_ARGS, &o.row_minima, s);
    return apc_build_tables(APCOST_BUILD_ARGS, s);
#undef APCOST_BUILD_ARGS
  };
  return b;
}

// apc_build_tables_packed: the planner's pass over packed tiles (one record of int32 words per tile).
c10::intrusive_ptr<BoundLaunch> bind_cost_tables_packed(const Tensor &params, const Tensor &rank, const Tensor &itemsize,
                                                        const Tensor &shape, const Tensor &stride, const Tensor &tensor_bytes,
                                                        const Tensor &tensor_contiguous, const Tensor &flops,
                                                        const Tensor &rw_bytes, const Tensor &dtype, const Tensor &zero_cost,
                                                        const Tensor &num_args, const Tensor &compute, const Tensor &per_arg,
                                                        const Tensor &error_flag, const Tensor &pt_values, const Tensor &packed,
                                                        int64_t n_entries, int64_t n_rows, const Tensor &cost,
                                                        const Tensor &row_min, const Tensor &row_argmin) {
  auto b = c10::make_intrusive<BoundLaunch>();
  const apc_params p = params_of(params);
  const TensorTable t = tensor_table(rank, itemsize, shape, stride);
  int64_t *bytes = dev<int64_t>(tensor_bytes, at::kLong, "tensor_bytes");
  uint8_t *contiguous = dev<uint8_t>(tensor_contiguous, at::kByte, "tensor_contiguous");
  TORCH_CHECK(tensor_bytes.numel() == t.n && tensor_contiguous.numel() == t.n, "apcost: tensor_bytes / tensor_contiguous need one row per tensor");
  const StrategyTable st = strategy_table(flops, rw_bytes, dtype, zero_cost, num_args);
  double *cc = dev<double>(compute, at::kDouble, "compute_cost"), *cpa = dev<double>(per_arg, at::kDouble, "compute_cost_per_arg");
  TORCH_CHECK(compute.numel() == st.n && per_arg.numel() == st.n, "apcost: compute_cost / compute_cost_per_arg need one row per strategy");
  int32_t *err = dev<int32_t>(error_flag, at::kInt, "error_flag");
  TORCH_CHECK(error_flag.numel() >= 1, "apcost: error_flag needs one element");
  const double *pt = dev<double>(pt_values, at::kDouble, "pt_values");
  constexpr int64_t kWords = (int64_t)(sizeof(apc_packed_tile) / sizeof(int32_t));
  TORCH_CHECK(packed.dim() == 2 && packed.size(1) == kWords, "apcost: packed tiles must be [n_tiles, ", kWords, "] int32 words (struct apc_packed_tile)");
  const apc_packed_tile *tiles = reinterpret_cast<const apc_packed_tile *>(dev<int32_t>(packed, at::kInt, "packed"));
  const int64_t n_tiles = packed.size(0);
  TORCH_CHECK(n_entries >= 0 && n_rows >= 0, "apcost: negative count");
  double *cost_out = dev<double>(cost, at::kDouble, "cost");
  double *mins = dev<double>(row_min, at::kDouble, "row_min");
  int32_t *args = dev<int32_t>(row_argmin, at::kInt, "row_argmin");
  TORCH_CHECK(cost.numel() == n_entries, "apcost: cost needs one value per entry");
  TORCH_CHECK(row_min.numel() == n_rows && row_argmin.numel() == n_rows, "apcost: row_min / row_argmin need one value per matrix row");
  for (const Tensor *x : {&rank, &itemsize, &shape, &stride, &tensor_bytes, &tensor_contiguous, &flops, &rw_bytes, &dtype, &zero_cost,
                          &num_args, &compute, &per_arg, &error_flag, &pt_values, &packed, &cost, &row_min, &row_argmin}) {
    same_device(rank, *x, "a table");
    b->keep.push_back(*x);
  }
  b->what = "apc_build_tables_packed";
  b->device = rank.device();
  b->launch = [=](void *s) {
    return apc_build_tables_packed(&p, t.n, t.rank, t.itemsize, t.shape, t.stride, bytes, contiguous, st.n, st.flops, st.rw_bytes,
                                   st.dtype, st.zero_cost, st.num_args, cc, cpa, err, pt, n_tiles, tiles, n_entries, cost_out, mins,
                                   args, s);
  };
  return b;
}

// The matrices as fresh tensors: (comm, transition, cost) of apc_redistribute_tables.
std::tuple<Tensor, Tensor, Tensor> redistribute_cost_tables(const Tensor &params, const Tensor &tensor_bytes,
                                                            const Tensor &tensor_contiguous, const Tensor &spec_codes,
                                                            const Tensor &spec_tensor, const Tensor &pt_values,
                                                            const Tensor &per_arg, const Tensor &tiles,
                                                            const Tensor &dup_entry_begin, int64_t n_entries) {
  TORCH_CHECK(n_entries >= 0, "apcost: n_entries < 0");
  Tensor comm = empty_like_device(tensor_bytes, {n_entries}, at::kDouble), transition = empty_like_device(tensor_bytes, {n_entries}, at::kByte),
         cost = empty_like_device(tensor_bytes, {n_entries}, at::kDouble);
  bind_redistribute_tables(params, tensor_bytes, tensor_contiguous, spec_codes, spec_tensor, pt_values, per_arg, tiles, dup_entry_begin,
                           n_entries, comm, transition, cost, std::nullopt, std::nullopt, std::nullopt, std::nullopt)
      ->run();
  return {comm, transition, cost};
}

// ---- more launches bound once: the three input tables one by one, the row minima --------------

c10::intrusive_ptr<BoundLaunch> bind_tensor_tables(const Tensor &rank, const Tensor &itemsize, const Tensor &shape,
                                                   const Tensor &stride, const Tensor &tensor_bytes,
                                                   const Tensor &tensor_contiguous) {
  auto b = c10::make_intrusive<BoundLaunch>();
  const TensorTable t = tensor_table(rank, itemsize, shape, stride);
  int64_t *bytes = dev<int64_t>(tensor_bytes, at::kLong, "tensor_bytes");
  uint8_t *contiguous = dev<uint8_t>(tensor_contiguous, at::kByte, "tensor_contiguous");
  TORCH_CHECK(tensor_bytes.numel() == t.n && tensor_contiguous.numel() == t.n, "apcost: tensor_bytes / tensor_contiguous need one row per tensor");
  b->keep = {rank, itemsize, shape, stride, tensor_bytes, tensor_contiguous};
  b->what = "apc_tensor_tables";
  b->device = rank.device();
  b->launch = [=](void *s) { return apc_tensor_tables(t.n, t.rank, t.itemsize, t.shape, t.stride, bytes, contiguous, s); };
  return b;
}

c10::intrusive_ptr<BoundLaunch> bind_spec_tables(const Tensor &params, const Tensor &spec_codes, const Tensor &spec_tensor,
                                                 const Tensor &rank, const Tensor &itemsize, const Tensor &shape,
                                                 const Tensor &stride, std::vector<Tensor> spec_outputs, int64_t shape_width) {
  auto b = c10::make_intrusive<BoundLaunch>();
  const apc_params p = params_of(params);
  const TensorTable t = tensor_table(rank, itemsize, shape, stride);
  const int64_t n = spec_codes.numel();
  const uint32_t *codes = codes_of(spec_codes);
  const int32_t *owner = dev<int32_t>(spec_tensor, at::kInt, "spec_tensor");
  TORCH_CHECK(spec_tensor.numel() == n, "apcost: spec_tensor and spec_codes differ in length");
  TORCH_CHECK(spec_outputs.size() == 5, "apcost: the spec table has five outputs (num_shards, local_shape, local_stride, local_numel, local_bytes)");
  TORCH_CHECK(shape_width >= 1 && shape_width <= APC_MAX_RANK, "apcost: shape_width ", shape_width, " outside [1, ", APC_MAX_RANK, "]");
  int64_t *out[5];
  static const char *names[5] = {"num_shards", "local_shape", "local_stride", "local_numel", "local_bytes"};
  for (int i = 0; i < 5; ++i) {
    out[i] = dev<int64_t>(spec_outputs[i], at::kLong, names[i]);
    TORCH_CHECK(spec_outputs[i].numel() == n * ((i == 1 || i == 2) ? shape_width : 1), "apcost: ", names[i], " has the wrong length");
    b->keep.push_back(spec_outputs[i]);
  }
  for (const Tensor *x : {&spec_codes, &spec_tensor, &rank, &itemsize, &shape, &stride}) b->keep.push_back(*x);
  int64_t *o0 = out[0], *o1 = out[1], *o2 = out[2], *o3 = out[3], *o4 = out[4];
  const int32_t width = (int32_t)shape_width;
  b->what = "apc_spec_tables";
  b->device = spec_codes.device();
  b->launch = [=](void *s) {
    return apc_spec_tables(&p, n, codes, owner, t.rank, t.itemsize, t.shape, t.stride, o0, o1, o2, width, o3, o4, s);
  };
  return b;
}

c10::intrusive_ptr<BoundLaunch> bind_compute_costs(const Tensor &params, const Tensor &flops, const Tensor &rw_bytes,
                                                   const Tensor &dtype, const Tensor &zero_cost, const Tensor &num_args,
                                                   const Tensor &compute, const Tensor &per_arg, const Tensor &error_flag) {
  auto b = c10::make_intrusive<BoundLaunch>();
  const apc_params p = params_of(params);
  const StrategyTable st = strategy_table(flops, rw_bytes, dtype, zero_cost, num_args);
  double *c = dev<double>(compute, at::kDouble, "compute_cost"), *cpa = dev<double>(per_arg, at::kDouble, "compute_cost_per_arg");
  TORCH_CHECK(compute.numel() == st.n && per_arg.numel() == st.n, "apcost: compute_cost / compute_cost_per_arg need one row per strategy");
  int32_t *err = dev<int32_t>(error_flag, at::kInt, "error_flag");
  TORCH_CHECK(error_flag.numel() >= 1, "apcost: error_flag needs one element");
  b->keep = {flops, rw_bytes, dtype, zero_cost, num_args, compute, per_arg, error_flag};
  b->what = "apc_compute_costs";
  b->device = flops.device();
  b->launch = [=](void *s) {
    return apc_compute_costs(&p, st.n, st.flops, st.rw_bytes, st.dtype, st.zero_cost, st.num_args, c, cpa, err, s);
  };
  return b;
}

// Row minima into given outputs; with `selected` (and the two copy arrays) only the selected
// segments are read and each result goes to its copies too (apc_segmented_min_copies).
c10::intrusive_ptr<BoundLaunch> bind_segmented_min(const Tensor &values, const Tensor &seg_ptr, const OptTensor &selected,
                                                   const OptTensor &copy_ptr, const OptTensor &copy_segments,
                                                   int64_t n_values_selected, const Tensor &seg_min, const Tensor &seg_argmin) {
  auto b = c10::make_intrusive<BoundLaunch>();
  const double *v = dev<double>(values, at::kDouble, "values");
  const int64_t *ptr = dev<int64_t>(seg_ptr, at::kLong, "seg_ptr");
  TORCH_CHECK(seg_ptr.numel() >= 1, "apcost: seg_ptr needs n_segments + 1 rows");
  const int64_t n_seg = seg_ptr.numel() - 1, n_values = values.numel();
  double *mins = dev<double>(seg_min, at::kDouble, "seg_min");
  int32_t *args = dev<int32_t>(seg_argmin, at::kInt, "seg_argmin");
  TORCH_CHECK(seg_min.numel() == n_seg && seg_argmin.numel() == n_seg, "apcost: seg_min / seg_argmin need one row per segment");
  same_device(values, seg_ptr, "seg_ptr");
  same_device(values, seg_min, "seg_min");
  b->keep = {values, seg_ptr, seg_min, seg_argmin};
  b->device = values.device();
  if (selected.has_value()) {
    TORCH_CHECK(copy_ptr.has_value() && copy_segments.has_value(), "apcost: selected segments need copy_ptr and copy_segments");
    const int64_t *sel = dev<int64_t>(*selected, at::kLong, "selected"), *cp = dev<int64_t>(*copy_ptr, at::kLong, "copy_ptr"),
                  *cs = dev<int64_t>(*copy_segments, at::kLong, "copy_segments");
    const int64_t n_sel = selected->numel();
    TORCH_CHECK(copy_ptr->numel() == n_sel + 1, "apcost: copy_ptr needs one row per selected segment + 1");
    b->keep.insert(b->keep.end(), {*selected, *copy_ptr, *copy_segments});
    b->what = "apc_segmented_min_copies";
    b->launch = [=](void *s) { return apc_segmented_min_copies(v, ptr, n_sel, sel, cp, cs, n_values_selected, mins, args, s); };
  } else {
    b->what = "apc_segmented_min";
    b->launch = [=](void *s) { return apc_segmented_min(v, ptr, n_seg, n_values, mins, args, s); };
  }
  return b;
}

Tensor strategy_bounds(const Tensor &strat_node, const Tensor &node_strat_begin, const Tensor &node_edge_begin,
                       const Tensor &edges_by_node, const Tensor &edge_row_begin, const Tensor &row_min) {
  const int32_t *sn = dev<int32_t>(strat_node, at::kInt, "strat_node");
  const int64_t *nsb = dev<int64_t>(node_strat_begin, at::kLong, "node_strat_begin"), *neb = dev<int64_t>(node_edge_begin, at::kLong, "node_edge_begin");
  const int32_t *ebn = dev<int32_t>(edges_by_node, at::kInt, "edges_by_node");
  const int64_t *erb = dev<int64_t>(edge_row_begin, at::kLong, "edge_row_begin");
  const double *rm = dev<double>(row_min, at::kDouble, "row_min");
  TORCH_CHECK(node_strat_begin.numel() == node_edge_begin.numel(), "apcost: node_strat_begin and node_edge_begin need n_nodes + 1 rows each");
  TORCH_CHECK(edges_by_node.numel() == edge_row_begin.numel(), "apcost: edges_by_node and edge_row_begin need one row per edge");
  for (const Tensor *t : {&node_strat_begin, &node_edge_begin, &edges_by_node, &edge_row_begin, &row_min}) same_device(strat_node, *t, "an index array");
  const int64_t n = strat_node.numel();
  Tensor bound = empty_like_device(row_min, {n}, at::kDouble);
  on_current_stream(row_min.device(), "apc_strategy_bounds", [&](void *s) {
    return apc_strategy_bounds(n, sn, nsb, neb, ebn, erb, rm, n ? static_cast<double *>(bound.data_ptr()) : nullptr, s);
  });
  return bound;
}

// Sweeps of min-sum diffusion over a labelling problem, in place on theta / unary.
void diffusion_sweeps_(int64_t n_sweeps, const Tensor &color_begin, const Tensor &color_nodes, const Tensor &label_begin,
                       const Tensor &inc_begin, const Tensor &inc_edge, const Tensor &inc_side, const Tensor &edge_begin,
                       const Tensor &edge_i, const Tensor &edge_j, int64_t max_labels, int64_t n_labels_total, int64_t n_elements,
                       const Tensor &theta, const Tensor &unary) {
  TORCH_CHECK(color_begin.device().is_cpu() && color_begin.scalar_type() == at::kLong && color_begin.is_contiguous() && color_begin.numel() >= 1,
              "apcost: color_begin must be a contiguous CPU int64 tensor of n_colors + 1 rows");
  const int32_t *cn = dev<int32_t>(color_nodes, at::kInt, "color_nodes");
  const int64_t *lb = dev<int64_t>(label_begin, at::kLong, "label_begin"), *ib = dev<int64_t>(inc_begin, at::kLong, "inc_begin");
  const int32_t *ie = dev<int32_t>(inc_edge, at::kInt, "inc_edge");
  const uint8_t *is = dev<uint8_t>(inc_side, at::kByte, "inc_side");
  const int64_t *eb = dev<int64_t>(edge_begin, at::kLong, "edge_begin");
  const int32_t *ei = dev<int32_t>(edge_i, at::kInt, "edge_i"), *ej = dev<int32_t>(edge_j, at::kInt, "edge_j");
  double *th = dev<double>(theta, at::kDouble, "theta"), *un = dev<double>(unary, at::kDouble, "unary");
  TORCH_CHECK(label_begin.numel() >= 1 && inc_begin.numel() == label_begin.numel(), "apcost: label_begin / inc_begin need n_classes + 1 rows each");
  TORCH_CHECK(edge_i.numel() == edge_j.numel() && edge_begin.numel() == edge_i.numel() + 1, "apcost: edge_begin needs n_edges + 1 rows, edge_i / edge_j n_edges");
  TORCH_CHECK(inc_edge.numel() == inc_side.numel(), "apcost: inc_edge and inc_side differ in length");
  // the ends of the pointer arrays as the host knows them: the kernels index unary by label_begin and theta by edge_begin
  TORCH_CHECK(unary.numel() == n_labels_total, "apcost: unary has ", unary.numel(), " values, label_begin ends at ", n_labels_total);
  TORCH_CHECK(theta.numel() == n_elements, "apcost: theta has ", theta.numel(), " values, edge_begin ends at ", n_elements);
  TORCH_CHECK(color_nodes.numel() == label_begin.numel() - 1, "apcost: color_nodes needs one row per class");
  for (const Tensor *t : {&color_nodes, &label_begin, &inc_begin, &inc_edge, &inc_side, &edge_begin, &edge_i, &edge_j, &unary}) same_device(theta, *t, "an index array");
  const int64_t n_classes = label_begin.numel() - 1;
  on_current_stream(theta.device(), "apc_diffusion_sweeps", [&](void *s) {
    return apc_diffusion_sweeps((int32_t)n_sweeps, (int32_t)(color_begin.numel() - 1), color_begin.data_ptr<int64_t>(), cn, n_classes, lb, ib, ie,
                                is, eb, ei, ej, (int32_t)max_labels, th, un, s);
  });
}

// Flop and byte counts of every (node, strategy) from the spec table's local shapes and the
// per-node recipes (compute_estimation.py:232-299, 334-349; apc_strategy_inputs).
std::tuple<Tensor, Tensor, Tensor, Tensor> strategy_inputs(const Tensor &strat_node, const Tensor &node_strat_begin,
                                                           const Tensor &node_kind, const Tensor &node_dtype,
                                                           const Tensor &node_const_bytes, const Tensor &node_row_begin,
                                                           const Tensor &byte_rows, const Tensor &node_flop_rows,
                                                           const Tensor &local_shape, const Tensor &local_bytes) {
  const int32_t *sn = dev<int32_t>(strat_node, at::kInt, "strat_node");
  const int64_t *nsb = dev<int64_t>(node_strat_begin, at::kLong, "node_strat_begin");
  const int32_t *kind = dev<int32_t>(node_kind, at::kInt, "node_kind");
  const int8_t *dt = dev<int8_t>(node_dtype, at::kChar, "node_dtype");
  const int64_t *cb = dev<int64_t>(node_const_bytes, at::kLong, "node_const_bytes");
  const int64_t *rb = dev<int64_t>(node_row_begin, at::kLong, "node_row_begin");
  const int32_t *rows = dev<int32_t>(byte_rows, at::kInt, "byte_rows");
  const int32_t *fr = dev<int32_t>(node_flop_rows, at::kInt, "node_flop_rows");
  const int64_t *ls = dev<int64_t>(local_shape, at::kLong, "local_shape");
  const int64_t *lb = dev<int64_t>(local_bytes, at::kLong, "local_bytes");
  const int64_t n = strat_node.numel(), n_nodes = node_kind.numel();
  TORCH_CHECK(node_strat_begin.numel() == n_nodes + 1 && node_row_begin.numel() == n_nodes + 1,
              "apcost: node_strat_begin / node_row_begin need n_nodes + 1 rows");
  TORCH_CHECK(node_dtype.numel() == n_nodes && node_const_bytes.numel() == n_nodes && node_flop_rows.numel() == 4 * n_nodes,
              "apcost: the recipe arrays need one row per node (node_flop_rows four values per node)");
  TORCH_CHECK(local_shape.dim() == 2 && local_shape.size(0) == local_bytes.numel(),
              "apcost: local_shape must be [n_specs, shape_width] with one row per row of local_bytes");
  for (const Tensor *t : {&node_strat_begin, &node_kind, &node_dtype, &node_const_bytes, &node_row_begin, &byte_rows, &node_flop_rows,
                          &local_shape, &local_bytes})
    same_device(strat_node, *t, "a recipe array");
  Tensor flops = empty_like_device(strat_node, {n}, at::kLong), rw_bytes = empty_like_device(strat_node, {n}, at::kLong),
         dtype = empty_like_device(strat_node, {n}, at::kChar), zero_cost = empty_like_device(strat_node, {n}, at::kByte);
  on_current_stream(strat_node.device(), "apc_strategy_inputs", [&](void *s) {
    return apc_strategy_inputs(n, sn, n_nodes, nsb, kind, dt, cb, rb, rows, fr, ls, (int32_t)local_shape.size(1), lb,
                               n ? static_cast<int64_t *>(flops.data_ptr()) : nullptr, n ? static_cast<int64_t *>(rw_bytes.data_ptr()) : nullptr,
                               n ? static_cast<int8_t *>(dtype.data_ptr()) : nullptr, n ? zero_cost.data_ptr<uint8_t>() : nullptr, s);
  });
  return {flops, rw_bytes, dtype, zero_cost};
}

// Structural check of the flattened tables on the host (apc_validate_tables_host; the kernels
// trust their indices): CPU tensors, RuntimeError naming the first malformed row
// (non-monotone pointers, placement codes out of range, rank above the maximum, tiles that
// leave their edge, ...).
template <typename T>
const T *host(const Tensor &t, at::ScalarType dtype, const char *name) {
  TORCH_CHECK(t.defined() && t.device().is_cpu(), "apcost: ", name, " must be a CPU tensor (host-side validation)");
  TORCH_CHECK(t.scalar_type() == dtype, "apcost: ", name, " must be ", dtype, " (got ", t.scalar_type(), ")");
  TORCH_CHECK(t.is_contiguous(), "apcost: ", name, " must be contiguous");
  return t.numel() ? static_cast<const T *>(t.data_ptr()) : nullptr;
}

void validate_tables(const Tensor &params, const Tensor &tensor_rank, const Tensor &spec_codes, const Tensor &spec_tensor,
                     const Tensor &edge_src_begin, const Tensor &edge_n_src, const Tensor &edge_tgt_begin,
                     const Tensor &edge_n_tgt, const Tensor &edge_flags, const Tensor &edge_pt_begin,
                     const Tensor &edge_entry_begin, const Tensor &edge_strat_begin, int64_t n_pt, int64_t n_strategies,
                     const Tensor &tiles, const Tensor &dup_entry_begin) {
  const apc_params p = params_of(params);
  const int64_t n_edges = edge_src_begin.numel();
  for (const Tensor *t : {&edge_n_src, &edge_tgt_begin, &edge_n_tgt, &edge_flags, &edge_pt_begin, &edge_strat_begin})
    TORCH_CHECK(t->numel() == n_edges, "apcost: the edge arrays must have one row per edge (", n_edges, ")");
  TORCH_CHECK(edge_entry_begin.numel() == n_edges + 1, "apcost: edge_entry_begin needs n_edges + 1 rows");
  TORCH_CHECK(spec_tensor.numel() == spec_codes.numel(), "apcost: spec_tensor and spec_codes differ in length");
  constexpr int64_t kWords = sizeof(apc_tile) / 4;
  TORCH_CHECK(tiles.numel() % kWords == 0, "apcost: tiles must be [n_tiles, ", kWords, "] int32 words (struct apc_tile)");
  const int rc = apc_validate_tables_host(
      &p, tensor_rank.numel(), host<int32_t>(tensor_rank, at::kInt, "tensor_rank"), spec_codes.numel(),
      reinterpret_cast<const uint32_t *>(host<int32_t>(spec_codes, at::kInt, "spec_codes")), host<int32_t>(spec_tensor, at::kInt, "spec_tensor"),
      n_edges, host<int32_t>(edge_src_begin, at::kInt, "edge_src_begin"), host<int32_t>(edge_n_src, at::kInt, "edge_n_src"),
      host<int32_t>(edge_tgt_begin, at::kInt, "edge_tgt_begin"), host<int32_t>(edge_n_tgt, at::kInt, "edge_n_tgt"),
      host<int32_t>(edge_flags, at::kInt, "edge_flags"), host<int64_t>(edge_pt_begin, at::kLong, "edge_pt_begin"),
      host<int64_t>(edge_entry_begin, at::kLong, "edge_entry_begin"), host<int32_t>(edge_strat_begin, at::kInt, "edge_strat_begin"), n_pt,
      n_strategies, tiles.numel() / kWords, reinterpret_cast<const apc_tile *>(host<int32_t>(tiles, at::kInt, "tiles")),
      dup_entry_begin.numel(), host<int64_t>(dup_entry_begin, at::kLong, "dup_entry_begin"));
  check_rc(rc, "apc_validate_tables_host");
}

// The interface version this layer was compiled against; the binding compares it with what the
// loaded library reports (apc_version) before the first call.
int64_t abi_version() { return APC_ABI_VERSION; }
int64_t library_abi_version() { return apc_version(); }

}  // namespace

TORCH_LIBRARY(apcost, m) {
  m.class_<BoundLaunch>("BoundLaunch").def("run", &BoundLaunch::run).def("run_on", &BoundLaunch::run_on).def("name", &BoundLaunch::name);
#define APCOST_TENSOR_TABLE "Tensor tensor_rank, Tensor tensor_itemsize, Tensor tensor_shape, Tensor tensor_stride"
#define APCOST_STRATEGY_TABLE "Tensor flops, Tensor rw_bytes, Tensor dtype_code, Tensor zero_cost, Tensor num_args"
#define APCOST_INPUT_TABLES                                                                                          \
  "Tensor params, " APCOST_TENSOR_TABLE ", Tensor tensor_bytes, Tensor tensor_contiguous, Tensor spec_codes, "       \
  "Tensor spec_tensor, Tensor[] spec_outputs, int shape_width, " APCOST_STRATEGY_TABLE                               \
  ", Tensor compute_cost, Tensor compute_cost_per_arg, Tensor error_flag"
#define APCOST_TABLE_OUTPUTS                                                                                         \
  "Tensor? comm, Tensor? transition, Tensor? cost, Tensor? edge_row_begin, Tensor? dup_row_begin, Tensor? row_min, " \
  "Tensor? row_argmin"
  m.def("abi_version() -> int", &abi_version);
  m.def("library_abi_version() -> int", &library_abi_version);
  m.def("validate_tables(Tensor params, Tensor tensor_rank, Tensor spec_codes, Tensor spec_tensor, Tensor edge_src_begin, "
        "Tensor edge_n_src, Tensor edge_tgt_begin, Tensor edge_n_tgt, Tensor edge_flags, Tensor edge_pt_begin, "
        "Tensor edge_entry_begin, Tensor edge_strat_begin, int n_pt, int n_strategies, Tensor tiles, Tensor dup_entry_begin) -> ()",
        &validate_tables);
  m.def("tensor_tables(" APCOST_TENSOR_TABLE ") -> (Tensor tensor_bytes, Tensor tensor_contiguous)", &tensor_tables);
  m.def("shard_shapes_bytes(Tensor params, Tensor spec_codes, Tensor spec_tensor, " APCOST_TENSOR_TABLE
        ", int shape_width) -> (Tensor num_shards, Tensor local_shape, Tensor local_stride, Tensor local_numel, Tensor local_bytes)",
        &shard_shapes_bytes);
  m.def("compute_cost(Tensor params, " APCOST_STRATEGY_TABLE
        ") -> (Tensor compute_cost, Tensor compute_cost_per_arg, Tensor error_flag)",
        &compute_cost);
  m.def("strategy_inputs(Tensor strat_node, Tensor node_strat_begin, Tensor node_kind, Tensor node_dtype, Tensor node_const_bytes, "
        "Tensor node_row_begin, Tensor byte_rows, Tensor node_flop_rows, Tensor local_shape, Tensor local_bytes) "
        "-> (Tensor flops, Tensor rw_bytes, Tensor dtype_code, Tensor zero_cost)",
        &strategy_inputs);
  m.def("segmented_min(Tensor values, Tensor seg_ptr) -> (Tensor seg_min, Tensor seg_argmin)", &segmented_min);
  m.def("cost_objective(int n_vars, Tensor group_var_begin, Tensor group_member_begin, Tensor member_entry_begin, Tensor cost, "
        "float inf_replacement) -> (Tensor objective, Tensor forced_zero)",
        &cost_objective);
  m.def("redistribute_cost_tables(Tensor params, Tensor tensor_bytes, Tensor tensor_contiguous, Tensor spec_codes, "
        "Tensor spec_tensor, Tensor pt_values, Tensor compute_cost_per_arg, Tensor tiles, Tensor dup_entry_begin, int n_entries) "
        "-> (Tensor comm, Tensor transition, Tensor cost)",
        &redistribute_cost_tables);
  m.def("strategy_bounds(Tensor strat_node, Tensor node_strat_begin, Tensor node_edge_begin, Tensor edges_by_node, "
        "Tensor edge_row_begin, Tensor row_min) -> Tensor",
        &strategy_bounds);
  m.def("diffusion_sweeps_(int n_sweeps, Tensor color_begin, Tensor color_nodes, Tensor label_begin, Tensor inc_begin, "
        "Tensor inc_edge, Tensor inc_side, Tensor edge_begin, Tensor edge_i, Tensor edge_j, int max_labels, int n_labels_total, int n_elements, Tensor(a!) theta, "
        "Tensor(b!) unary) -> ()",
        &diffusion_sweeps_);
  m.def("bind_tensor_tables(" APCOST_TENSOR_TABLE ", Tensor tensor_bytes, Tensor tensor_contiguous) -> __torch__.torch.classes.apcost.BoundLaunch",
        &bind_tensor_tables);
  m.def("bind_spec_tables(Tensor params, Tensor spec_codes, Tensor spec_tensor, " APCOST_TENSOR_TABLE
        ", Tensor[] spec_outputs, int shape_width) -> __torch__.torch.classes.apcost.BoundLaunch",
        &bind_spec_tables);
  m.def("bind_compute_costs(Tensor params, " APCOST_STRATEGY_TABLE
        ", Tensor compute_cost, Tensor compute_cost_per_arg, Tensor error_flag) -> __torch__.torch.classes.apcost.BoundLaunch",
        &bind_compute_costs);
  m.def("bind_segmented_min(Tensor values, Tensor seg_ptr, Tensor? selected, Tensor? copy_ptr, Tensor? copy_segments, "
        "int n_values_selected, Tensor seg_min, Tensor seg_argmin) -> __torch__.torch.classes.apcost.BoundLaunch",
        &bind_segmented_min);
  m.def("bind_redistribute_tables(Tensor params, Tensor tensor_bytes, Tensor tensor_contiguous, Tensor spec_codes, "
        "Tensor spec_tensor, Tensor pt_values, Tensor? compute_cost_per_arg, Tensor tiles, Tensor dup_entry_begin, int n_entries, "
        APCOST_TABLE_OUTPUTS ") -> __torch__.torch.classes.apcost.BoundLaunch",
        &bind_redistribute_tables);
  m.def("bind_input_tables(" APCOST_INPUT_TABLES ") -> __torch__.torch.classes.apcost.BoundLaunch", &bind_input_tables);
  m.def("bind_cost_tables(" APCOST_INPUT_TABLES ", Tensor pt_values, Tensor tiles, Tensor dup_entry_begin, int n_entries, "
        APCOST_TABLE_OUTPUTS ") -> __torch__.torch.classes.apcost.BoundLaunch",
        &bind_cost_tables);
  m.def("bind_cost_tables_packed(Tensor params, " APCOST_TENSOR_TABLE ", Tensor tensor_bytes, Tensor tensor_contiguous, "
        APCOST_STRATEGY_TABLE ", Tensor compute_cost, Tensor compute_cost_per_arg, Tensor error_flag, Tensor pt_values, "
        "Tensor packed, int n_entries, int n_rows, Tensor cost, Tensor row_min, Tensor row_argmin) "
        "-> __torch__.torch.classes.apcost.BoundLaunch",
        &bind_cost_tables_packed);
}
