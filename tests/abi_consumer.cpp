// A consumer of the C ABI that is not Python: fills the flat tables of a two-node graph by
// hand (one producer strategy, three consumer strategies, mesh (32, 8), 8 devices per host,
// H100 row), calls the library on the default stream and compares the redistribution costs
// with the hand-derived known answers (tests/golden/known_answers.json), bit for bit.
// Built by autoparallel_amd/_build.py; run by tests/test_gpu_parity.py.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <vector>

#include "apcost.h"

#define HIP_OK(x)                                                                     \
  do {                                                                                \
    hipError_t e_ = (x);                                                              \
    if (e_ != hipSuccess) {                                                           \
      std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
      return 2;                                                                       \
    }                                                                                 \
  } while (0)
#define APC_OK(x)                                                                     \
  do {                                                                                \
    int rc_ = (x);                                                                    \
    if (rc_ != 0) {                                                                   \
      std::printf("apcost error %d at line %d: %s\n", rc_, __LINE__, apc_last_error()); \
      return 3;                                                                       \
    }                                                                                 \
  } while (0)

template <typename T>
static T *to_device(const std::vector<T> &v) {
  T *d = nullptr;
  if (hipMalloc(&d, v.size() * sizeof(T) + 16) != hipSuccess) return nullptr;
  if (!v.empty() && hipMemcpy(d, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  return d;
}

int main() {
  apc_params p;
  std::memset(&p, 0, sizeof(p));
  p.mesh_ndim = 2;
  p.mesh_size[0] = 32;
  p.mesh_size[1] = 8;
  // torch _collective_utils.py:246-278 with 8 devices per host: dim 1 stays inside a host
  p.bw[0] = 87.7 * 0.22;
  p.lat[0] = 2.7;
  p.bw[1] = 87.7;
  p.lat[1] = 0.6;
  p.base_latency = 6.6;
  p.a2a_scale = 5.0;
  p.hbm_bw = 3.35 * 1024.0 * 1024.0 * 1024.0 * 1024.0;  // H100 row, compute_estimation.py:63-166
  p.rw_eff = 0.70;
  p.launch_floor = 7.0;
  p.compute_eff = 0.70;
  p.rescale = 1.0;
  p.gpu_flops[3] = 989.0 * 1e12;
  p.transition_scale = 1;
  for (int i = 0; i < 2; ++i) {
    p.inv_bw[i] = 1.0 / p.bw[i];
    p.inv_mesh[i] = 1.0 / (double)p.mesh_size[i];
  }
  p.inv_hbm_bw = 1.0 / p.hbm_bw;
  p.inv_rw_eff = 1.0 / p.rw_eff;
  p.inv_compute_eff = 1.0 / p.compute_eff;
  for (int i = 0; i < APC_MAX_DTYPES; ++i) p.inv_gpu_flops[i] = p.gpu_flops[i] != 0.0 ? 1.0 / p.gpu_flops[i] : 0.0;

  // one tensor: [4096, 4096] bf16, contiguous
  const std::vector<int32_t> rank{2}, itemsize{2};
  std::vector<int64_t> shape(APC_MAX_RANK, 0), stride(APC_MAX_RANK, 0);
  shape[0] = shape[1] = 4096;
  stride[0] = 4096;
  stride[1] = 1;
  // specs: the producer's (Shard(0), Shard(0)); the consumer's (R, S0), (R, R), (S0, S1)
  const uint32_t S0 = 0x80, S1 = 0x81, R = 0x00;
  const std::vector<uint32_t> codes{S0 | (S0 << 8), R | (S0 << 8), R | (R << 8), S0 | (S1 << 8)};
  const std::vector<int32_t> spec_tensor{0, 0, 0, 0};
  // strategies: 1 of the producer node, 3 of the consumer node, all free of compute cost
  const std::vector<int64_t> flops(4, 0), rw_bytes(4, 0);
  const std::vector<int8_t> dtype(4, 3);
  const std::vector<uint8_t> zero_cost(4, 1);
  const std::vector<int32_t> num_args(4, 1);
  // one edge (consumer node 1, argument 0), one tile covering its 3 x 1 matrix
  const std::vector<int32_t> e_src_begin{0}, e_n_src{1}, e_tgt_begin{1}, e_n_tgt{3}, e_flags{0}, e_strat_begin{1};
  const std::vector<int64_t> e_pt_begin{-1}, e_entry_begin{0, 3};
  apc_tile tile;
  std::memset(&tile, 0, sizeof(tile));
  tile.counts = 3 | (1 << 16);
  tile.n_src = 1;
  tile.tgt_begin = 1;
  tile.strat_begin = 1;
  tile.pt_begin = -1;
  const std::vector<apc_tile> tiles{tile};

  APC_OK(apc_validate_tables_host(&p, 1, rank.data(), 4, codes.data(), spec_tensor.data(), 1, e_src_begin.data(),
                                  e_n_src.data(), e_tgt_begin.data(), e_n_tgt.data(), e_flags.data(), e_pt_begin.data(),
                                  e_entry_begin.data(), e_strat_begin.data(), 0, 4, 1, tiles.data(), 0, nullptr));

  int n_dev = 0;
  HIP_OK(hipGetDeviceCount(&n_dev));
  if (n_dev < 1) {
    std::printf("no HIP device\n");
    return 2;
  }
  auto *d_rank = to_device(rank);
  auto *d_item = to_device(itemsize);
  auto *d_shape = to_device(shape);
  auto *d_stride = to_device(stride);
  auto *d_codes = to_device(codes);
  auto *d_spec_tensor = to_device(spec_tensor);
  auto *d_flops = to_device(flops);
  auto *d_rw = to_device(rw_bytes);
  auto *d_dtype = to_device(dtype);
  auto *d_zero = to_device(zero_cost);
  auto *d_args = to_device(num_args);
  auto *d_tiles = to_device(tiles);
  int64_t *d_bytes = nullptr, *d_shards = nullptr, *d_lshape = nullptr, *d_lstride = nullptr, *d_lnumel = nullptr,
          *d_lbytes = nullptr;
  uint8_t *d_cont = nullptr, *d_trans = nullptr;
  double *d_compute = nullptr, *d_per_arg = nullptr, *d_comm = nullptr, *d_cost = nullptr, *d_min = nullptr;
  int32_t *d_err = nullptr, *d_arg = nullptr;
  int64_t *d_seg = nullptr;
  HIP_OK(hipMalloc(&d_bytes, 8));
  HIP_OK(hipMalloc(&d_cont, 16));
  HIP_OK(hipMalloc(&d_shards, 4 * 8));
  const int width = 2;  // values per row of the local shape / stride tables: the tensor's rank
  HIP_OK(hipMalloc(&d_lshape, 4 * width * 8));
  HIP_OK(hipMalloc(&d_lstride, 4 * width * 8));
  HIP_OK(hipMalloc(&d_lnumel, 4 * 8));
  HIP_OK(hipMalloc(&d_lbytes, 4 * 8));
  HIP_OK(hipMalloc(&d_compute, 4 * 8));
  HIP_OK(hipMalloc(&d_per_arg, 4 * 8));
  HIP_OK(hipMalloc(&d_err, 4));
  HIP_OK(hipMemset(d_err, 0, 4));
  HIP_OK(hipMalloc(&d_comm, 3 * 8));
  HIP_OK(hipMalloc(&d_cost, 3 * 8));
  HIP_OK(hipMalloc(&d_trans, 16));
  HIP_OK(hipMalloc(&d_min, 8));
  HIP_OK(hipMalloc(&d_arg, 4));
  const std::vector<int64_t> seg{0, 3};
  d_seg = to_device(seg);
  if (!d_rank || !d_item || !d_shape || !d_stride || !d_codes || !d_spec_tensor || !d_flops || !d_rw || !d_dtype ||
      !d_zero || !d_args || !d_tiles || !d_seg) {
    std::printf("device allocation failed\n");
    return 2;
  }

  // every table of the pass in one launch, then the minimum of the whole matrix
  APC_OK(apc_build_tables(&p, 1, d_rank, d_item, d_shape, d_stride, d_bytes, d_cont, 4, d_codes, d_spec_tensor, d_shards,
                          d_lshape, d_lstride, width, d_lnumel, d_lbytes, 4, d_flops, d_rw, d_dtype, d_zero, d_args, d_compute,
                          d_per_arg, d_err, nullptr, 1, d_tiles, nullptr, 3, d_comm, d_trans, d_cost, nullptr));
  APC_OK(apc_segmented_min(d_cost, d_seg, 1, 3, d_min, d_arg, nullptr));
  // the same pass with the minimum of every matrix row (three rows of one column) taken by the launch itself
  const std::vector<int64_t> edge_row_begin{0};
  double *d_row_min = nullptr;
  int32_t *d_row_arg = nullptr;
  HIP_OK(hipMalloc(&d_row_min, 3 * 8));
  HIP_OK(hipMalloc(&d_row_arg, 3 * 4));
  const apc_row_minima rows{to_device(edge_row_begin), nullptr, d_row_min, d_row_arg};
  if (!rows.edge_row_begin) {
    std::printf("device allocation failed\n");
    return 2;
  }
  APC_OK(apc_build_tables_row_min(&p, 1, d_rank, d_item, d_shape, d_stride, d_bytes, d_cont, 4, d_codes, d_spec_tensor,
                                  d_shards, d_lshape, d_lstride, width, d_lnumel, d_lbytes, 4, d_flops, d_rw, d_dtype,
                                  d_zero, d_args, d_compute, d_per_arg, d_err, nullptr, 1, d_tiles, nullptr, 3, d_comm,
                                  d_trans, d_cost, &rows, nullptr));
  HIP_OK(hipDeviceSynchronize());
  double row_min[3];
  int32_t row_arg[3];
  HIP_OK(hipMemcpy(row_min, d_row_min, sizeof(row_min), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(row_arg, d_row_arg, sizeof(row_arg), hipMemcpyDeviceToHost));

  double comm[3], cost[3], seg_min = 0.0;
  uint8_t trans[3];
  int64_t bytes = 0, lshape[4 * 2];
  int32_t seg_arg = -1;
  HIP_OK(hipMemcpy(comm, d_comm, sizeof(comm), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(cost, d_cost, sizeof(cost), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(trans, d_trans, sizeof(trans), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(&bytes, d_bytes, 8, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(lshape, d_lshape, sizeof(lshape), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(&seg_min, d_min, 8, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(&seg_arg, d_arg, 4, hipMemcpyDeviceToHost));

  // hand-derived: all-gather over the inter-host dim; two all-gathers; all-to-all x 5 + one reshuffle
  const double want[3] = {286.43246022079404, 609.0198034363015, 67.08959654717788};
  int bad = 0;
  for (int i = 0; i < 3; ++i) {
    std::printf("entry %d: comm %.17g (want %.17g) transition %d cost %.17g\n", i, comm[i], want[i], (int)trans[i], cost[i]);
    bad += comm[i] != want[i];
    bad += trans[i] != 1;
    bad += cost[i] != want[i] + 0.0 + 1.0;  // comm + compute / num_args + transition (optimize_sharding.py:368-372)
  }
  bad += bytes != 4096LL * 4096 * 2;
  bad += lshape[0] != 4096 / 32 / 8 || lshape[1] != 4096;                        // (S0, S0): dim 0 split twice
  bad += lshape[3 * width] != 4096 / 32 || lshape[3 * width + 1] != 4096 / 8;  // (S0, S1)
  bad += seg_min != want[2] + 1.0 || seg_arg != 2;
  for (int i = 0; i < 3; ++i) bad += row_min[i] != want[i] + 1.0 || row_arg[i] != 0;
  std::printf(bad ? "abi consumer: %d MISMATCHES\n" : "abi consumer ok\n", bad);
  return bad ? 1 : 0;
}
