// apcost — sharding-cost evaluation kernels for MI355X (gfx950) and their C ABI.
//
// Built with -ffp-contract=off: every fp64 operation below is a single IEEE
// rounding in the order the reference's Python evaluates it, so results are
// bit-identical to CPython's floats rather than merely close.
//
// Reference functions restated here (batched over the whole graph):
//   autoparallel/collective_runtime_estimation.py:22-153
//   autoparallel/compute_estimation.py:211-229, 302-365
//   autoparallel/optimize_sharding.py:306-379
//   torch/distributed/tensor/_collective_utils.py:230-313
//   torch/_prims_common/__init__.py:252-292
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "apcost.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(-3, "%s: %s", what, hipGetErrorString(e));
  return 0;
}

constexpr int kBlock = 256;

// ------------------------------------------------------------------------------------------
// placement codes
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ int kind_of(uint32_t c) { return (int)(c >> 6); }  // 0 R, 1 P, 2 S
__device__ __forceinline__ int dim_of(uint32_t c) { return (int)(c & 0x0F); }

// A load from a wave-uniform address of a table that no kernel of this library writes while it
// reads it (the uploaded encoding): through the constant address space, i.e. the scalar cache,
// into scalar registers.  (Left as a plain load the compiler takes such an address through vector
// memory, where the load queues behind the wavefront's other vector loads.)
#define APC_CONSTANT __attribute__((address_space(4)))
template <typename T>
__device__ __forceinline__ T uniform_load(const T *p) {
  return *(const APC_CONSTANT T *)p;
}
// A plain store that is written through to memory (system scope, no ordering).  What a launch of
// a few tens of MB leaves in the L2 is written back when the kernel ends, after its last
// wavefront, and the launch lasts until that is done; written through, the lines leave while the
// wavefronts still work.  For the tables of a small pass only: a large table streams through the
// L2 anyway, and its tile kernels lose what the L2 does for them when neighbouring wavefronts fill
// a line together (write-through there: Llama-3-70B 126 -> 221 us, the stress table 1.19 -> 1.24 ms).
template <typename T>
__device__ __forceinline__ void store_through(T *p, T value) {
  __hip_atomic_store(p, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
typedef int32_t i32x16 __attribute__((ext_vector_type(16)));
typedef int64_t i64x8 __attribute__((ext_vector_type(8)));

// The value lane `lane` (wave-uniform) holds.
__device__ __forceinline__ int64_t value_of_lane(int64_t x, int lane) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)x, lane);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)((uint64_t)x >> 32), lane);
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

// Kernel arguments a wavefront will need, fetched now: the compiler loads an argument where it
// is first used, each behind the wait of whatever came before it, and a chain of such loads in
// front of a tile's own loads cost more than the loads themselves.  Naming the values as scalar
// operands of an (empty) asm statement puts their loads here, together, under one wait.
// One statement for all of them: a load may be moved past an asm statement that does not name it.
template <typename T0>
__device__ __forceinline__ void fetch_arguments_now(T0 v0) {
  __asm__ volatile("" ::"s"(v0));
}
template <typename T0, typename T1>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1) {
  __asm__ volatile("" ::"s"(v0), "s"(v1));
}
template <typename T0, typename T1, typename T2>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2));
}
template <typename T0, typename T1, typename T2, typename T3>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12, typename T13>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12, T13 v13) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12), "s"(v13));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12, typename T13, typename T14>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12, T13 v13, T14 v14) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12), "s"(v13), "s"(v14));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12, typename T13, typename T14, typename T15>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12, T13 v13, T14 v14, T15 v15) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12), "s"(v13), "s"(v14), "s"(v15));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12, typename T13, typename T14, typename T15, typename T16>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12, T13 v13, T14 v14, T15 v15, T16 v16) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12), "s"(v13), "s"(v14), "s"(v15), "s"(v16));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12, typename T13, typename T14, typename T15, typename T16, typename T17>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12, T13 v13, T14 v14, T15 v15, T16 v16, T17 v17) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12), "s"(v13), "s"(v14), "s"(v15), "s"(v16), "s"(v17));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12, typename T13, typename T14, typename T15, typename T16, typename T17, typename T18>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12, T13 v13, T14 v14, T15 v15, T16 v16, T17 v17, T18 v18) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12), "s"(v13), "s"(v14), "s"(v15), "s"(v16), "s"(v17), "s"(v18));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12, typename T13, typename T14, typename T15, typename T16, typename T17, typename T18, typename T19>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12, T13 v13, T14 v14, T15 v15, T16 v16, T17 v17, T18 v18, T19 v19) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12), "s"(v13), "s"(v14), "s"(v15), "s"(v16), "s"(v17), "s"(v18), "s"(v19));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12, typename T13, typename T14, typename T15, typename T16, typename T17, typename T18, typename T19, typename T20>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12, T13 v13, T14 v14, T15 v15, T16 v16, T17 v17, T18 v18, T19 v19, T20 v20) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12), "s"(v13), "s"(v14), "s"(v15), "s"(v16), "s"(v17), "s"(v18), "s"(v19), "s"(v20));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12, typename T13, typename T14, typename T15, typename T16, typename T17, typename T18, typename T19, typename T20, typename T21>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12, T13 v13, T14 v14, T15 v15, T16 v16, T17 v17, T18 v18, T19 v19, T20 v20, T21 v21) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12), "s"(v13), "s"(v14), "s"(v15), "s"(v16), "s"(v17), "s"(v18), "s"(v19), "s"(v20), "s"(v21));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12, typename T13, typename T14, typename T15, typename T16, typename T17, typename T18, typename T19, typename T20, typename T21, typename T22>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12, T13 v13, T14 v14, T15 v15, T16 v16, T17 v17, T18 v18, T19 v19, T20 v20, T21 v21, T22 v22) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12), "s"(v13), "s"(v14), "s"(v15), "s"(v16), "s"(v17), "s"(v18), "s"(v19), "s"(v20), "s"(v21), "s"(v22));
}
template <typename T0, typename T1, typename T2, typename T3, typename T4, typename T5, typename T6, typename T7, typename T8, typename T9, typename T10, typename T11, typename T12, typename T13, typename T14, typename T15, typename T16, typename T17, typename T18, typename T19, typename T20, typename T21, typename T22, typename T23>
__device__ __forceinline__ void fetch_arguments_now(T0 v0, T1 v1, T2 v2, T3 v3, T4 v4, T5 v5, T6 v6, T7 v7, T8 v8, T9 v9, T10 v10, T11 v11, T12 v12, T13 v13, T14 v14, T15 v15, T16 v16, T17 v17, T18 v18, T19 v19, T20 v20, T21 v21, T22 v22, T23 v23) {
  __asm__ volatile("" ::"s"(v0), "s"(v1), "s"(v2), "s"(v3), "s"(v4), "s"(v5), "s"(v6), "s"(v7), "s"(v8), "s"(v9), "s"(v10), "s"(v11), "s"(v12), "s"(v13), "s"(v14), "s"(v15), "s"(v16), "s"(v17), "s"(v18), "s"(v19), "s"(v20), "s"(v21), "s"(v22), "s"(v23));
}

// compute_estimation.py:302-314
__device__ __forceinline__ double rw_time(double bytes, const apc_params &p) {
  double t = bytes / p.hbm_bw * 1e6;
  t = t / p.rw_eff;
  return t > p.launch_floor ? t : p.launch_floor;
}

// torch _collective_utils.py:281-313: latency + bandwidth term of a ring collective
__device__ __forceinline__ double ring(double gb, const apc_params &p, int d, int hops) {
  double latency = p.base_latency + (double)hops * p.lat[d];
  double bw = (gb * (double)hops / (double)p.mesh_size[d]) / p.bw[d];
  return latency + bw * 1e6;
}

// a / b for a divisor whose correctly rounded reciprocal y = RN(1 / b) is known: one
// multiply and two Newton corrections, each residual computed exactly by an FMA.  With y
// correctly rounded the second correction returns the correctly rounded quotient (Markstein),
// i.e. the same bits as the division instruction sequence, at a sixth of its cost.  The
// reciprocals travel in apc_params and are checked against 1.0 / b on the host.
__device__ __forceinline__ double div_by(double a, double b, double y) {
  double q = a * y;
  double r = __builtin_fma(-b, q, a);
  q = __builtin_fma(r, y, q);
  r = __builtin_fma(-b, q, a);
  return __builtin_fma(r, y, q);
}

__device__ __forceinline__ double rw_time_r(double bytes, const apc_params &p) {
  double t = div_by(bytes, p.hbm_bw, p.inv_hbm_bw) * 1e6;
  t = div_by(t, p.rw_eff, p.inv_rw_eff);
  return t > p.launch_floor ? t : p.launch_floor;
}

__device__ __forceinline__ double ring_r(double gb, const apc_params &p, int d, int hops) {
  const double latency = p.base_latency + (double)hops * p.lat[d];
  const double bw = div_by(div_by(gb * (double)hops, (double)p.mesh_size[d], p.inv_mesh[d]), p.bw[d], p.inv_bw[d]);
  return latency + bw * 1e6;
}

// collective_runtime_estimation.py:37-153 for one (producer spec, consumer spec) pair.
// gb = bytes / num_shards / 1024^3 of the producer spec, cont = global contiguity.
template <int M>
__device__ __forceinline__ double entry_cost(uint32_t srcp, uint32_t tgtp, double gb, bool cont,
                                             const apc_params &p) {
  if (srcp == 0u) {  // fully replicated producer (:56-62)
    bool tgt_partial = false;
#pragma unroll
    for (int i = 0; i < M; ++i) tgt_partial |= kind_of((tgtp >> (8 * i)) & 0xFF) == 1;
    return tgt_partial ? INFINITY : 0.0;
  }
  bool flip = false;
  if (M == 2) {  // :146-151
    flip = srcp == 0x4040u && kind_of(tgtp & 0xFF) == 2 && kind_of((tgtp >> 8) & 0xFF) == 2;
  }
  double cost = 0.0;
#pragma unroll
  for (int k = 0; k < M; ++k) {
    const int i = (M == 2 && flip) ? 1 - k : k;
    const uint32_t c = (srcp >> (8 * i)) & 0xFF, t = (tgtp >> (8 * i)) & 0xFF;
    if (c == t) continue;
    const double n = (double)p.mesh_size[i];
    if (!cont) cost += rw_time(gb * 2 * 1073741824.0, p);
    const int ck = kind_of(c), tk = kind_of(t);
    if (ck == 2 && tk == 0) {  // all-gather (:83-96)
      gb *= n;
      cost += ring(gb, p, i, p.mesh_size[i] - 1);
      if (dim_of(c) != 0) cost += rw_time(gb * 2 * 1073741824.0, p);
    } else if (ck == 2 && tk == 2) {  // all-to-all (:97-113)
      double a2a = ring(gb, p, i, p.mesh_size[i] - 1);
      a2a *= p.a2a_scale;
      cost += a2a;
      const int copies = (dim_of(c) != 0) + (dim_of(t) != 0);
      cost += (double)copies * rw_time(gb * 2 * 1073741824.0, p);
    } else if (ck == 1 && tk == 0) {  // all-reduce (:115-117)
      cost += ring(gb, p, i, 2 * (p.mesh_size[i] - 1));
    } else if (ck == 1 && tk == 2) {  // reduce-scatter (:118-130)
      cost += ring(gb, p, i, p.mesh_size[i] - 1);
      if (dim_of(t) != 0) cost += rw_time(gb * 2 * 1073741824.0, p);
      gb /= n;
    } else if (tk == 1 && ck != 1) {  // Shard->Partial, Replicate->Partial banned (:131-138)
      return INFINITY;
    }
    cont = true;  // :141
  }
  return cost;
}

// ------------------------------------------------------------------------------------------
// Running-bytes states.  The redistribution cost of an entry is a sum of per-mesh-dim terms,
// and every term is an expensive expression (fp64 divisions) of ONE quantity only: the
// running comm_bytes_gb at that dim.  For a given tensor that quantity takes few distinct
// values: it starts from bytes / num_shards (decided by WHICH mesh dims the producer
// shards: a mask of M bits) and every earlier dim either left it alone or applied its
// single possible update (x n after an all-gather when the producer shards that dim, / n
// after a reduce-scatter when it does not).  State (level L, mask, history) indexes every
// value that can occur; level L in [0, M] has 2^M masks x 2^L histories.
// ------------------------------------------------------------------------------------------
template <int M>
struct States {
  static constexpr int kCount = (1 << M) * ((1 << (M + 1)) - 1);
  __device__ static __forceinline__ int index(int level, int mask, int hist) {
    return (((1 << level) - 1) << M) + (mask << level) + hist;
  }
};
// ------------------------------------------------------------------------------------------
// XCD-aware work order.  The dispatcher deals workgroups to the chip's 8 XCDs round-robin by
// workgroup id, and every XCD has its own L2.  With the plain order, neighbouring units of
// work (which write neighbouring memory and share the cache lines at their boundaries) sit
// in eight different L2s and those lines are written back in parts.  The launchers round the
// grid up to a multiple of 2^shift and the kernel takes unit (id mod 2^shift) * per + id /
// 2^shift, so each XCD walks one contiguous share of the units.  (Measured: helps the tile
// kernel, whose units end at arbitrary byte offsets; the kernels whose workgroups write
// whole aligned blocks are faster in the plain order.)
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ int64_t xcd_chunked_unit(int shift) {
  const int64_t per = gridDim.x >> shift;
  return (int64_t)(blockIdx.x & ((1u << shift) - 1)) * per + (blockIdx.x >> shift);
}

// Element `i` (a per-lane index below M) of one of the arrays of the kernel parameters, as a select chain over scalar registers.  (Indexing the array by a lane value
// makes the compiler read the kernel arguments through vector memory, and a vector load
// waits behind every store the compute unit has in flight.)
template <int M, typename T, int N>
__device__ __forceinline__ T pick(const T (&v)[N], int i) {
  static_assert(M <= N, "array shorter than the mesh");
  T e[M];  // every element is read (scalar loads) before the selects, so they stay selects
#pragma unroll
  for (int k = 0; k < M; ++k) e[k] = v[k];
  T r = e[0];
#pragma unroll
  for (int k = 1; k < M; ++k) r = i == k ? e[k] : r;
  return r;
}

// ------------------------------------------------------------------------------------------
// a7: bytes + contiguity per tensor
// ------------------------------------------------------------------------------------------
struct TensorTableArgs {
  int64_t n;
  const int32_t *rank, *itemsize;
  const int64_t *shape, *stride;
  int64_t *bytes;
  uint8_t *cont;
};

// Bytes and contiguity of one tensor (torch _collective_utils.py:230-232,
// _prims_common/__init__.py:252-292) from its zero-padded shape and stride rows, held in registers.
template <typename Row>
__device__ __forceinline__ void tensor_bytes_and_contiguity_of(int r, int64_t itemsize, const Row &x, const Row &y,
                                                               int64_t &nbytes, bool &contiguous) {
  nbytes = itemsize;
  int64_t expected = 1, expected_max = 1;
  bool ok = true;
#pragma unroll
  for (int i = APC_MAX_RANK - 1; i >= 0; --i) {
    if (i >= r) continue;
    nbytes *= x[i];
    if (x[i] == 1) continue;
    if (y[i] != expected && y[i] != expected_max) ok = false;
    expected_max *= (x[i] > 1 ? x[i] : 1);
    expected *= x[i];
  }
  contiguous = ok;
}

__device__ __forceinline__ void tensor_bytes_and_contiguity(int r, int64_t itemsize, const int64_t *sh, const int64_t *st,
                                                            int64_t &nbytes, bool &contiguous) {
  // the whole (zero-padded) rows are read at once, before the scan: one round of loads
  // instead of one per dim
  int64_t x[APC_MAX_RANK], y[APC_MAX_RANK];
#pragma unroll
  for (int i = 0; i < APC_MAX_RANK; ++i) {
    x[i] = sh[i];
    y[i] = st[i];
  }
  tensor_bytes_and_contiguity_of(r, itemsize, x, y, nbytes, contiguous);
}

// THROUGH: the rows are written through to memory (the packed pass: see store_through)
template <int BS, bool THROUGH = false>
__device__ __forceinline__ void tensor_tables_block(int64_t block, const TensorTableArgs &a) {
  const int64_t t = block * BS + threadIdx.x;
  if (t >= a.n) return;
  int64_t nbytes;
  bool ok;
  tensor_bytes_and_contiguity(a.rank[t], a.itemsize[t], a.shape + t * APC_MAX_RANK, a.stride + t * APC_MAX_RANK, nbytes, ok);
  if (THROUGH) {
    store_through(a.bytes + t, nbytes);
    store_through(a.cont + t, (uint8_t)(ok ? 1 : 0));
  } else {
    a.bytes[t] = nbytes;
    a.cont[t] = ok ? 1 : 0;
  }
}

__global__ __launch_bounds__(kBlock) void tensor_tables_kernel(TensorTableArgs a) {
  tensor_tables_block<kBlock>(blockIdx.x, a);
}

// ceil(x / m) for x >= 0 and a mesh size m whose correctly rounded reciprocal y is known.
// Below 2^52 the quotient is taken in fp64 (both operands exact, div_by rounds once, so the
// truncated value is off by at most one) and corrected by the exact integer remainder: a
// dozen instructions against the ~120 of a 64-bit integer division, which made this kernel
// VALU-bound.  Larger values take the integer division.
__device__ __forceinline__ int64_t ceil_div_by(int64_t x, int32_t m, double y) {
  const int64_t num = x + m - 1;
  if (num >> 52) return num / m;
  int64_t q = (int64_t)div_by((double)num, (double)m, y);
  int64_t rem = num - q * m;
  if (rem < 0) {
    q -= 1;
    rem += m;
  }
  if (rem >= m) q += 1;
  return q;
}

// ------------------------------------------------------------------------------------------
// a8: local shard shape / stride / counts per spec
// ------------------------------------------------------------------------------------------
struct SpecTableArgs {
  int64_t n;
  const uint32_t *codes;
  const int32_t *tensor, *rank, *itemsize;
  const int64_t *shape, *stride;
  int64_t *shards, *lshape, *lstride, *lnumel, *lbytes;
  int width;  // values per row of lshape / lstride: even, 2 .. APC_MAX_RANK, >= every tensor's rank
};

// s_rows: kBlock * (APC_MAX_RANK + 1) values of LDS
// Writes the staged rows of the workgroup (APC_MAX_RANK + 1 slots per row in LDS) to `out`, the
// first `width` values of each row, `live` values in all (rows x width), as one contiguous run,
// two values (one 16-byte store) per lane: width is even, so a pair never straddles rows.
template <int BS>
__device__ __forceinline__ void write_rows(int64_t *__restrict__ out, const int64_t *s_rows, int live, int width) {
  typedef int64_t pair_t __attribute__((ext_vector_type(2)));
  for (int k = 2 * threadIdx.x; k < live; k += 2 * BS) {
    const int r = k / width, c = k - r * width;
    const int64_t *src = s_rows + r * (APC_MAX_RANK + 1) + c;
    pair_t v = {src[0], src[1]};
    *reinterpret_cast<pair_t *>(out + k) = v;
  }
}

template <int BS>
__device__ __forceinline__ void spec_tables_block(int64_t block, const apc_params &p, const SpecTableArgs &a,
                                                  int64_t *s_rows) {
  const int64_t n = a.n;
  const uint32_t *__restrict__ codes = a.codes;
  const int32_t *__restrict__ tensor = a.tensor, *__restrict__ rank = a.rank, *__restrict__ itemsize = a.itemsize;
  const int64_t *__restrict__ shape = a.shape, *__restrict__ stride = a.stride;
  int64_t *__restrict__ shards = a.shards, *__restrict__ lshape = a.lshape, *__restrict__ lstride = a.lstride;
  int64_t *__restrict__ lnumel = a.lnumel, *__restrict__ lbytes = a.lbytes;
  // Each thread derives one spec in its own row of an LDS buffer (the Shard dim indexes the
  // row, so no register array is indexed by a lane value), first the shape and then, in the
  // same buffer, the stride; the workgroup (BS threads) writes each [BS][8] result block out
  // as one contiguous run.
  const int64_t base = block * BS;
  const int64_t s = base + threadIdx.x;
  int64_t *row = s_rows + threadIdx.x * (APC_MAX_RANK + 1);
  const int width = a.width;
  const int live = (int)(n - base < BS ? n - base : BS) * width;
  int t = -1, r = 0;
  uint32_t pc = 0;
  if (s < n) {
    t = tensor[s];
    if (t >= 0) {
      r = rank[t];
      pc = codes[s];
    }
  }
  // (every load is issued before the first store: a load behind stores waits for them)
  int64_t st[APC_MAX_RANK];
#pragma unroll
  for (int i = 0; i < APC_MAX_RANK; ++i) {
    row[i] = i < r ? shape[(int64_t)t * APC_MAX_RANK + i] : 0;
    st[i] = i < r ? stride[(int64_t)t * APC_MAX_RANK + i] : 0;
  }
  const int64_t item = t >= 0 ? itemsize[t] : 0;
  int64_t nsh = t >= 0 ? 1 : 0;
  for (int i = 0; i < p.mesh_ndim; ++i) {
    const uint32_t c = (pc >> (8 * i)) & 0xFF;
    if (kind_of(c) == 2) {
      const int d = dim_of(c);
      nsh *= p.mesh_size[i];
      if (d < APC_MAX_RANK) row[d] = ceil_div_by(row[d], p.mesh_size[i], p.inv_mesh[i]);
    }
  }
  if (s < n) {
    int64_t ne = 0, nb = 0;
    if (t >= 0) {
      ne = 1;
#pragma unroll
      for (int i = 0; i < APC_MAX_RANK; ++i)
        if (i < r) ne *= row[i];
      nb = ne * item;
    }
    shards[s] = nsh;
    lnumel[s] = ne;
    lbytes[s] = nb;
  }
  __syncthreads();
  write_rows<BS>(lshape + base * width, s_rows, live, width);
  __syncthreads();
#pragma unroll
  for (int i = 0; i < APC_MAX_RANK; ++i) row[i] = st[i];
  for (int i = 0; i < p.mesh_ndim; ++i) {
    const uint32_t c = (pc >> (8 * i)) & 0xFF;
    if (kind_of(c) == 2) {
      const int d = dim_of(c);
      if (d - 1 > 0 && d - 1 < APC_MAX_RANK)  // compute_estimation.py:225-228
        row[d - 1] = ceil_div_by(row[d - 1], p.mesh_size[i], p.inv_mesh[i]);
    }
  }
  __syncthreads();
  write_rows<BS>(lstride + base * width, s_rows, live, width);
}

__global__ __launch_bounds__(kBlock) void spec_tables_kernel(apc_params p, SpecTableArgs a) {
  __shared__ int64_t s_rows[kBlock * (APC_MAX_RANK + 1)];
  spec_tables_block<kBlock>(blockIdx.x, p, a, s_rows);
}

// ------------------------------------------------------------------------------------------
// a9/a10: compute-cost tail per (node, strategy)
// ------------------------------------------------------------------------------------------
struct ComputeCostArgs {
  int64_t n;
  const int64_t *flops, *rw_bytes;
  const int8_t *dtype;
  const uint8_t *zero_cost;
  const int32_t *num_args;
  double *compute, *per_arg;
  int32_t *error_flag;
};

// Compute cost of one strategy (compute_estimation.py:334-365); `unsupported` is set when the
// strategy has flops and its dtype has no throughput on the device row (the result is NaN).
__device__ __forceinline__ double compute_cost_of(const apc_params &p, bool zero_cost, int64_t rw_bytes, int64_t flops,
                                                  int dt, bool &unsupported) {
  unsupported = false;
  if (zero_cost) return 0.0;
  const double rw = rw_time((double)rw_bytes, p);
  if (flops == 0) return rw;
  const double gf = (dt >= 0 && dt < APC_MAX_DTYPES) ? pick<APC_MAX_DTYPES>(p.gpu_flops, dt) : 0.0;
  if (gf == 0.0) {
    unsupported = true;  // compute_estimation.py:198-201 raises ValueError
    return NAN;
  }
  double t = (double)flops / gf * 1e6;
  t = t / p.compute_eff;
  return t > rw ? t : rw;
}

// The same value with the divisions taken through the checked reciprocals (div_by): gf / inv_gf =
// the device row's throughput for the strategy's dtype and its reciprocal, 0 when unsupported.
__device__ __forceinline__ double compute_cost_through_reciprocals(const apc_params &p, bool zero_cost, int64_t rw_bytes,
                                                                   int64_t flops, double gf, double inv_gf) {
  if (zero_cost) return 0.0;
  const double rw = rw_time_r((double)rw_bytes, p);
  if (flops == 0) return rw;
  if (gf == 0.0) return NAN;  // compute_estimation.py:198-201 raises ValueError (flagged by compute_costs_block)
  double t = div_by((double)flops, gf, inv_gf) * 1e6;
  t = div_by(t, p.compute_eff, p.inv_compute_eff);
  return t > rw ? t : rw;
}

template <int BS, bool THROUGH = false>
__device__ __forceinline__ void compute_costs_block(int64_t block, const apc_params &p, const ComputeCostArgs &a) {
  const int64_t s = block * BS + threadIdx.x;
  if (s >= a.n) return;
  // (the divisions through the checked reciprocals: the same bits as compute_cost_of, a third of
  // its instructions; these workgroups share the chip with the ones that write the matrices)
  const int dt = a.dtype[s];
  const bool zero = a.zero_cost[s] != 0;
  const int64_t flops = a.flops[s];
  const bool known = dt >= 0 && dt < APC_MAX_DTYPES;
  const double gf = known ? pick<APC_MAX_DTYPES>(p.gpu_flops, dt) : 0.0, inv_gf = known ? pick<APC_MAX_DTYPES>(p.inv_gpu_flops, dt) : 0.0;
  const double c = compute_cost_through_reciprocals(p, zero, a.rw_bytes[s], flops, gf, inv_gf);
  const bool unsupported = !zero && flops != 0 && gf == 0.0;
  if (unsupported && a.error_flag) *a.error_flag = 1;
  const double per_arg = c / (double)a.num_args[s];
  if (THROUGH) {
    if (a.compute) store_through(a.compute + s, c);
    if (a.per_arg) store_through(a.per_arg + s, per_arg);
  } else {
    if (a.compute) a.compute[s] = c;
    if (a.per_arg) a.per_arg[s] = per_arg;
  }
}

__global__ __launch_bounds__(kBlock) void compute_costs_kernel(apc_params p, ComputeCostArgs a) {
  compute_costs_block<kBlock>(blockIdx.x, p, a);
}

// ------------------------------------------------------------------------------------------
// a9, integer part: flop and byte counts per (node, strategy) from the local shard shapes.
// The reference runs every operator on fake tensors of the local shard shapes under torch's
// FlopCounterMode and adds the bytes of all tensor arguments and outputs
// (compute_estimation.py:232-299, 334-349).  For the operators torch's counter knows in the
// planned graphs the count is a closed form of the local shapes (torch/utils/flop_counter.py:
// mm_flop, bmm_flop, sdpa_flop_count, sdpa_backward_flop_count), and the bytes are the local
// bytes of the strategy's input and output specs (the rows of the spec table) plus a per-node
// constant (outputs of factories, tensor constants).  One recipe per node, written by the
// host; one thread per strategy.
// ------------------------------------------------------------------------------------------
struct StrategyInputArgs {
  int64_t n;
  const int32_t *strat_node;
  const int64_t *node_strat_begin;
  const int32_t *node_kind;        // APC_NODE_*
  const int8_t *node_dtype;
  const int64_t *node_const_bytes;
  const int64_t *node_row_begin;   // CSR over byte_rows
  const int32_t *byte_rows;        // first spec rows of the node's argument and output slots (strategy ss reads row + ss)
  const int32_t *node_flop_rows;   // [n_nodes, 4]: first spec rows of the tensors the flop formula reads
  const int64_t *local_shape;      // [n_specs, width]
  int32_t width;
  const int64_t *local_bytes;      // [n_specs]
  int64_t *flops, *rw_bytes;
  int8_t *dtype;
  uint8_t *zero_cost;
};

// b * m * n * 2 * k, in torch's order of multiplications (exact in int64 below 2^63)
__device__ __forceinline__ int64_t bmm_flops(int64_t b, int64_t m, int64_t k, int64_t n) { return b * m * n * 2 * k; }

__global__ __launch_bounds__(kBlock) void strategy_inputs_kernel(StrategyInputArgs a) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= a.n) return;
  const int node = a.strat_node[i];
  const int64_t ss = i - a.node_strat_begin[node];
  const int kind = a.node_kind[node];
  int64_t flops = 0, bytes = 0;
  if (kind != APC_NODE_ZERO_COST) {
    bytes = a.node_const_bytes[node];
    for (int64_t r = a.node_row_begin[node]; r < a.node_row_begin[node + 1]; ++r) bytes += a.local_bytes[a.byte_rows[r] + ss];
    const int32_t *rows = a.node_flop_rows + (int64_t)node * 4;
    const int w = a.width;
    // (a dim past the row's width reads as 1: the host checks ranks, this keeps the load inside the table)
    auto dim = [&](int t, int d) { return d < w ? a.local_shape[(rows[t] + ss) * w + d] : (int64_t)1; };
    if (kind == APC_NODE_MM) {  // [m, k] x [k, n]
      flops = dim(0, 0) * dim(1, 1) * 2 * dim(0, 1);
    } else if (kind == APC_NODE_BMM) {  // [b, m, k] x [b, k, n]
      flops = bmm_flops(dim(0, 0), dim(0, 1), dim(0, 2), dim(1, 2));
    } else if (kind == APC_NODE_SDPA || kind == APC_NODE_SDPA_BACKWARD) {
      // rows: query [b, h, s_q, d_q], key [b, h, s_k, d_q], value [b, h, s_k, d_v]
      const int64_t bh = dim(0, 0) * dim(0, 1), s_q = dim(0, 2), d_q = dim(0, 3), s_k = dim(1, 2), d_v = dim(2, 3);
      if (kind == APC_NODE_SDPA) {
        flops = bmm_flops(bh, s_q, d_q, s_k) + bmm_flops(bh, s_q, s_k, d_v);
      } else {  // recomputed scores, gradScores, gradV, gradQ, gradK
        flops = bmm_flops(bh, s_q, d_q, s_k) + bmm_flops(bh, s_q, d_v, s_k) + bmm_flops(bh, s_k, s_q, d_v) +
                bmm_flops(bh, s_q, s_k, d_q) + bmm_flops(bh, d_q, s_q, s_k);
      }
    }
  }
  a.flops[i] = flops;
  a.rw_bytes[i] = bytes;
  a.dtype[i] = a.node_dtype[node];
  a.zero_cost[i] = kind == APC_NODE_ZERO_COST ? 1 : 0;
}

// The three tables above in one launch: workgroups [0, spec_blocks) take the spec table (the
// largest), the next tensor_blocks the tensor table, the rest the compute costs.  None of the
// three reads another's output.
__global__ __launch_bounds__(kBlock) void input_tables_kernel(apc_params p, TensorTableArgs t, SpecTableArgs sp,
                                                              ComputeCostArgs c, int64_t spec_blocks,
                                                              int64_t tensor_blocks) {
  __shared__ int64_t s_rows[kBlock * (APC_MAX_RANK + 1)];
  const int64_t b = blockIdx.x;
  if (b < spec_blocks) spec_tables_block<kBlock>(b, p, sp, s_rows);
  else if (b < spec_blocks + tensor_blocks) tensor_tables_block<kBlock>(b - spec_blocks, t);
  else compute_costs_block<kBlock>(b - spec_blocks - tensor_blocks, p, c);
}

// ------------------------------------------------------------------------------------------
// a1-a6: redistribution-cost matrices.  The unit of work is a tile: a rectangle of one edge's
// matrix.  A tile's producer and consumer specs and the per-state terms of the edge's tensor
// are staged in LDS (TileStage); the per-entry loop walks the mesh dims, looks the terms of
// the current state up and adds them in the reference's order, so results are bit-identical
// to evaluating every entry directly (entry_cost).  The direct evaluation remains the path
// for the rare cases the states do not cover: producer specs of one edge that point at
// different tensors, and the 2-D (Partial, Partial) -> all-Shard order flip.
//
// One workgroup per tile.  (A variant in which a workgroup walked a run of tiles, one
// wavefront staging tile t+1 into a second LDS stage while the others computed and stored
// tile t, was measured 35 - 60 % slower on both large tables, also with the one-round
// staging below: fewer, longer-lived workgroups keep fewer stores in flight.)
// ------------------------------------------------------------------------------------------

// What is the same for every tile of a launch (see "Term arrays" and "Lookup words" below):
// the layout of the term arrays, the part of the lookup words that does not depend on the
// producer spec (by dim x 16 + producer class x 4 + consumer class; the producer spec's state
// or exponent index is added when a tile is staged) and, for the power-of-two layout, the
// constants of every computed array.
constexpr int kMaxTermArrays = 16;
struct TermArrayConstants {  // value at exponent index j = max(lat + ldexp(B, j + shift), floor) x scale,
  double hops;               // B = RN(RN(RN(RN(bytes x hops) / div1) x 1e6) / div2)
  double div1, inv_div1;
  double div2, inv_div2;
  double lat;
  double floor;
  double scale;
  int32_t shift;
  int32_t pad_;
};
struct TermLayout {
  uint32_t pair[APC_MAX_MESH * 16];
  int32_t exponents;         // 0: general layout; else E, the number of exponents
  int32_t lg[APC_MAX_MESH];  // log2 of the mesh sizes (power-of-two layout)
  int32_t lg_total;          // L
  int32_t state_stride;      // bytes between the entries of two consecutive states / exponents
  uint32_t exponent_magic;   // ceil(65536 / E): t / E = (t * magic) >> 16 for t < 512
  double inv_rescale;        // 1.0 / params.rescale
  TermArrayConstants arrays[kMaxTermArrays - 2];  // of arrays 2 .. (power-of-two layout)
};

struct TableArgs {
  const int64_t *tensor_bytes;
  const uint8_t *tensor_contiguous;
  const uint32_t *spec_codes;
  const int32_t *spec_tensor;
  const double *pt_values;
  const double *per_arg;
  const apc_tile *tiles;
  const int64_t *dup_entry_begin;
  double *comm_out;
  uint8_t *trans_out;
  double *cost_out;
  // When the tensor and compute-cost tables are produced by the same launch (build_tables_kernel)
  // a tile cannot read them: tensor_bytes / tensor_contiguous / per_arg are NULL and the tile
  // derives the few values it needs from the tables those are computed from.
  const int32_t *rank, *itemsize;
  const int64_t *shape, *stride;
  const int64_t *flops, *rw_bytes;
  const int8_t *dtype;
  const uint8_t *zero_cost;
  const int32_t *num_args;
  // Row minima written by the tiles themselves (NULL: not wanted).  Matrix rows are numbered
  // edge by edge (edge_row_begin[e] + consumer strategy); dup_row_begin[k] is the first row of
  // the identical edge whose first entry is dup_entry_begin[k].
  const int64_t *edge_row_begin;
  const int64_t *dup_row_begin;
  double *row_min_out;
  int32_t *row_arg_out;
  TermLayout lay;  // the launch's term-array layout and lookup-word bases
};

// Bytes and contiguity of tensor t: read from the tensor table, or (DERIVE) derived from its
// shape row.  A compile-time choice: as a run-time one it cost the tile kernel a third of
// its registers.
template <bool DERIVE>
__device__ __forceinline__ void tensor_info(const TableArgs &a, int t, int64_t &nbytes, bool &contiguous) {
  if (!DERIVE) {
    nbytes = a.tensor_bytes[t];
    contiguous = a.tensor_contiguous[t] != 0;
  } else {
    tensor_bytes_and_contiguity(a.rank[t], a.itemsize[t], a.shape + (int64_t)t * APC_MAX_RANK,
                                a.stride + (int64_t)t * APC_MAX_RANK, nbytes, contiguous);
  }
}


// What one mesh dim contributes, by (producer class, consumer class) with classes
// 0 Replicate, 1 Partial, 2 Shard(0), 3 Shard(d != 0); only consulted when the two placement
// codes differ.  One byte per pair:
//   bits 0-2  term array: 0 none, 1 all-gather, 2 reduce-scatter, 3 all-reduce, 4 all-to-all
//   bits 3-4  number of read+write reshuffles added after the collective
//   bit  5    banned transition (-> Partial from Replicate / Shard): cost is inf
//   bit  6    the running bytes change after this dim (x n after all-gather, / n after
//             reduce-scatter)
// collective_runtime_estimation.py:83-138.
__host__ __device__ constexpr uint32_t pair_action(int c, int t) {
  constexpr uint32_t AG = 1, RS = 2, AR = 3, A2A = 4, BAN = 1u << 5, UPD = 1u << 6;
  const uint32_t cn = c == 3, tn = t == 3;
  if (t == 1) return c == 1 ? 0u : BAN;            // -> Partial
  if (c == 0) return 0u;                           // Replicate -> Replicate / Shard: local
  if (c == 1) return t == 0 ? AR : (RS | (tn << 3) | UPD);
  return t == 0 ? (AG | (cn << 3) | UPD) : (A2A | ((cn + tn) << 3));
}
__device__ __forceinline__ int placement_class(uint32_t code) {
  const int k = kind_of(code);
  return k == 2 ? 2 + (dim_of(code) != 0 ? 1 : 0) : k;
}

// Term arrays staged per tile, interleaved: the entry of (state s, array a) sits at byte
// s x state_stride + 8 a, state_stride = 8 x (arrays + 1): an odd number of doubles, so that
// lanes reading one array at different states hit different LDS banks.  Two layouts, chosen per
// launch by the host (TermLayout):
//
// General (any mesh): one value per running-bytes state, 8 arrays: [0] zeros, [1] +inf (banned
// transitions), [2] one read+write, [3] two read+writes (2.0 x [2]: the same bits as
// (double)2 * rw), [4] all-gather, [5] reduce-scatter, [6] all-reduce, [7] all-to-all (=
// reduce-scatter shaped term x a2a_scale, :22-32).  An entry's running index is the history of
// the earlier dims.
//
// Power-of-two meshes (every mesh size a power of two, world size at most 2^31): the running
// bytes are the tensor's bytes times a power of two, bytes x 2^e with e in [-30 - L, -30],
// L = log2(world size): dividing by the shards, x n after an all-gather and / n after a
// reduce-scatter are exact.  Every term is then a rounding-free rescaling of ONE chain of
// operations on the tensor's bytes: RN(2^e x) = 2^e RN(x) for the multiplications and divisions
// of the ring and read+write formulas (no underflow: bytes < 2^53, e >= -61), so
//   ring term of dim d at exponent e = latency_d + ldexp(B_d, e - log2 n_d),
//       B_d = RN(RN(RN(bytes x hops_d) / bw_d) x 1e6)      (two hops per step: B doubles)
//   read+write at exponent e = max(ldexp(R, e + 31), launch floor),
//       R = RN(RN(RN(bytes / hbm_bw) x 1e6) / rw_eff)
// and one value per (array, exponent) replaces one per (array, state); 16 arrays: [0] zeros,
// [1] +inf, [2] one read+write, [3] two, then per mesh dim d [4 + 3d] one-hop ring (all-gather
// and reduce-scatter), [5 + 3d] two-hop ring (all-reduce), [6 + 3d] all-to-all; E = L + 1
// exponents.  An entry's running index is e + 30 + L.  Every computed array is one formula,
// max(lat + ldexp(B, j + shift), floor) x scale with B from one chain bytes x hops / div1 x 1e6
// / div2 (division by 1.0, x 1.0, 0.0 + x and max(x, -inf) return x), with constants the host
// works out per launch (TermArrayConstants): a lane per array takes B, then a lane per (array,
// exponent) the value.  (3-D mesh of 512 devices: 11 chains and 110 values of five operations,
// against 120 states x 6 terms of two divisions each.)
constexpr int kMaxExponents = 32;
constexpr int kGeneralStride = 8 * (8 + 1), kPow2Stride = 8 * (kMaxTermArrays + 1);  // bytes per state / exponent
template <int M>
struct TermTable {
  static constexpr int kGeneral = kGeneralStride / 8 * States<M>::kCount;
  static constexpr int kPow2 = kPow2Stride / 8 * kMaxExponents;
  static constexpr int kEntries = kGeneral > kPow2 ? kGeneral : kPow2;
};
static_assert(4 + 3 * APC_MAX_MESH <= kMaxTermArrays, "arrays of the power-of-two layout");

// Lookup words.  What a mesh dim adds to an entry depends on the producer spec (its class at
// that dim and which dims it shards), on the consumer's class at that dim and on the running
// index left by the earlier dims; everything but the running index is known per (producer
// spec, dim, consumer class) when the tile is staged.  One 32-bit word per such triple, in
// fields an instruction can take as a half or a byte of a register:
//   bits  0-15  byte offset of the collective's term for running index 0 (general: array of
//               pair_action's term, state of the bytes the collective moves: after the update
//               for an all-gather, before it else; the +inf array for a banned transition)
//   bits 16-23  signed: bytes from there to the read+write term of the same state (zeros / one
//               / two reshuffles)
//   bits 24-31  signed step of the running index after this dim (general: the dim's history
//               bit; power-of-two meshes: + log2 n after an all-gather, - log2 n after a
//               reduce-scatter)
// Slot 4 of a (spec, dim) is the word of "same placement": zeros, no step; slot 5 is the byte
// offset of one read+write at the state BEFORE the dim, charged once to a non-contiguous tensor.
constexpr int kWordsPerDim = 6;
constexpr uint32_t kZerosArray = 0, kInfArray = 1, kRw1Array = 2;
static_assert(TermTable<APC_MAX_MESH>::kEntries * 8 <= 0xFFFF + 1, "term offsets fit their 16 bits");

static TermLayout term_layout(const apc_params &p) {
  TermLayout lay{};
  const int M = p.mesh_ndim;
  bool pow2 = getenv("APC_GENERAL_TERMS") == nullptr;  // (testing override: the general layout on any mesh)
  int total = 0;
  for (int i = 0; i < M; ++i) {
    const int n = p.mesh_size[i];
    if (n < 1 || (n & (n - 1)) != 0) {
      pow2 = false;
      break;
    }
    int lg = 0;
    while ((1 << lg) < n) ++lg;
    lay.lg[i] = lg;
    total += lg;
  }
  if (total + 1 > kMaxExponents) pow2 = false;
  const int E = pow2 ? total + 1 : 0;
  lay.exponents = E;
  lay.lg_total = pow2 ? total : 0;
  lay.state_stride = pow2 ? kPow2Stride : kGeneralStride;
  lay.exponent_magic = pow2 ? (uint32_t)((65536 + E - 1) / E) : 0u;
  lay.inv_rescale = 1.0 / p.rescale;
  for (int i = 0; i < M; ++i)
    for (int c = 0; c < 4; ++c)
      for (int t = 0; t < 4; ++t) {
        const uint32_t e = pair_action(c, t);
        const uint32_t sel = e & 7u, copies = (e >> 3) & 3u;
        const bool ban = (e & 32u) != 0, upd = (e & 64u) != 0;
        const uint32_t rw_array = copies == 0u ? kZerosArray : kRw1Array + copies - 1u;
        uint32_t term_array, state = 0;
        int step;
        if (!pow2) {
          term_array = ban ? kInfArray : sel == 0u ? kZerosArray : 3u + sel;
          step = upd ? (1 << i) : 0;
        } else {
          if (sel == 1u) state = (uint32_t)lay.lg[i];  // an all-gather is charged on the gathered bytes
          term_array = ban ? kInfArray : sel == 0u ? kZerosArray : sel <= 2u ? 4u + 3u * i : sel == 3u ? 5u + 3u * i : 6u + 3u * i;
          step = !upd ? 0 : sel == 1u ? lay.lg[i] : -lay.lg[i];
        }
        const int to_rw = ((int)rw_array - (int)term_array) * 8;
        lay.pair[i * 16 + c * 4 + t] = (state * (uint32_t)lay.state_stride + term_array * 8u) | ((uint32_t)(to_rw & 0xFF) << 16) |
                                       ((uint32_t)(step & 0xFF) << 24);
      }
  if (pow2) {
    const double ninf = -INFINITY;
    // one read+write, two (compute_estimation.py:302-314 on bytes x 2^(e + 31))
    lay.arrays[0] = {1.0, p.hbm_bw, p.inv_hbm_bw, p.rw_eff, p.inv_rw_eff, 0.0, p.launch_floor, 1.0, -total - 30 + 31, 0};
    lay.arrays[1] = lay.arrays[0];
    lay.arrays[1].scale = 2.0;
    for (int d = 0; d < M; ++d) {  // torch _collective_utils.py:281-313 on bytes x 2^e
      const double h = (double)(p.mesh_size[d] - 1);
      const double lat1 = p.base_latency + h * p.lat[d];
      const double lat2 = p.base_latency + (2.0 * h) * p.lat[d];
      const int shift = -total - 30 - lay.lg[d];
      lay.arrays[2 + 3 * d] = {h, p.bw[d], p.inv_bw[d], 1.0, 1.0, lat1, ninf, 1.0, shift, 0};
      lay.arrays[3 + 3 * d] = {h, p.bw[d], p.inv_bw[d], 1.0, 1.0, lat2, ninf, 1.0, shift + 1, 0};
      lay.arrays[4 + 3 * d] = {h, p.bw[d], p.inv_bw[d], 1.0, 1.0, lat1, ninf, p.a2a_scale, shift, 0};
    }
  }
  return lay;
}

// Everything the entry loops need about one tile, in LDS.
// What a tile that also takes its row minima keeps in LDS beside the rest (a launch that does
// not want them is a different instantiation and does not pay for the space).
struct RowMinStage {
  // A row of at most 64 entries meets at most two of the 64-entry chunks the wavefronts
  // walk.  Slot 0 takes the part that holds the row's first column, slot 1 the part that
  // starts a chunk: one writer per slot, no atomics.
  double rmin[2][APC_TILE_MAX_ROWS];
  int rarg[2][APC_TILE_MAX_ROWS];
};
struct NoRowMinStage {};

// A consumer spec of a tile: its placement codes; per mesh dim i, in byte i of `slots`, the
// byte offset of its class's lookup word within a producer spec's words ((6 i + class) x 4;
// byte 0 = 0xFF: not a DTensorSpec; on a 2-D mesh bit 24 = every dim is a Shard); the compute
// cost / num_args of its strategy.  One 16-byte LDS read per entry.
struct alignas(16) RowRecord {
  uint32_t codes, slots;
  double cpa;
};
constexpr uint32_t kRowNotASpec = 0xFFu, kRowAllShard = 1u << 24;

// The part of TermArrayConstants a value needs after its array's chain.
struct alignas(16) TermValueConstants {
  double lat, floor, scale;
  int32_t shift, pad_;
};

template <int M, bool RM>
struct TileStage : std::conditional_t<RM, RowMinStage, NoRowMinStage> {
  RowRecord row[APC_TILE_MAX_ROWS];  // consumer specs
  uint2 colh[APC_TILE_MAX_COLS];  // producer specs: x = codes, y = info
  uint32_t col_codes[APC_TILE_MAX_COLS];  // their codes again, packed (one LDS bank per lane)
  // lookup words per (producer spec, dim, consumer class); an odd number of words per spec, so
  // that the lanes of consecutive producer specs hit different banks
  uint32_t words[APC_TILE_MAX_COLS * (M * kWordsPerDim + 1)];
  alignas(16) uint32_t pair_base[M * 16];  // TermLayout::pair of the launch
  double gb_unsharded;  // bytes / 1024^3 of the tile's tensor
  int mixed[4];         // per staging wavefront: some spec is not a DTensorSpec on the tile's tensor (generic loop)
  int cont;             // the tile's tensor is contiguous
  // Last: the tile kernels size their LDS per launch for the entries the layout in use needs
  // (stage_lds_bytes), so that the small power-of-two layout leaves room for more workgroups.
  // In front of the entries, one StagingScratch per wavefront of the workgroup (a compile-time
  // number in every kernel, so the entries still sit at a fixed offset): term_base.
  alignas(16) double terms[TermTable<M>::kEntries];
};

// What one wavefront keeps while it stages the term arrays of the power-of-two layout.
struct alignas(16) StagingScratch {
  double chain[kMaxTermArrays];
  TermValueConstants value_of[kMaxTermArrays];
};
// Where the term arrays of a stage start, for a workgroup of `nthreads` threads.
template <typename Stage>
__device__ __forceinline__ char *term_base(Stage &st, int nthreads) {
  return const_cast<char *>(reinterpret_cast<const char *>(st.terms)) + sizeof(StagingScratch) * (size_t)(nthreads >> 6);
}

// LDS bytes of a tile stage whose term arrays hold what the launch's layout needs.
template <int M, bool RM>
static size_t stage_lds_bytes(const TermLayout &lay, int threads) {
  const size_t entries = lay.exponents ? (size_t)(kPow2Stride / 8) * lay.exponents : (size_t)TermTable<M>::kGeneral;
  return sizeof(TileStage<M, RM>) - sizeof(double) * TermTable<M>::kEntries + sizeof(StagingScratch) * (size_t)(threads / 64) +
         sizeof(double) * entries;
}

// Where the copies of a tile's values go: lane k of EVERY wavefront holds the first entry and the
// first matrix row of the k-th identical edge (k < dup_count <= APC_TILE_MAX_DUPS <= 64), read
// back one by one as scalars (value_of_lane) when a value is stored to all copies: no LDS, no
// load in the store loop.  row_out (the same in every lane) is the first matrix row of the tile's own edge.
struct TileCopies {
  int64_t entry0, row0;
  int64_t row_out;
};
static_assert(APC_TILE_MAX_DUPS <= 64, "one lane per identical edge");

// Waits for the loads of `copies` now.  On this hardware loads and stores share one counter of
// outstanding vector-memory operations, and a wait for a load behind which stores were issued
// can only be a wait for all of them: offsets first touched inside the store loop would make
// every wavefront sit out the full round trip of its first store.  Called before the stores begin.
__device__ __forceinline__ void settle(TileCopies &copies) {
  __asm__ volatile("" : "+v"(copies.entry0), "+v"(copies.row0), "+v"(copies.row_out));
}

// The fields of a tile record the entry loops use.
struct TileView {
  int rows, cols, row_begin, col_begin, n_src, flags, dup_count, src_begin;
  int64_t entry_begin, pt_begin;
};

__device__ __forceinline__ int uniform_i32(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int64_t uniform_i64(int64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ TileView view_of(const apc_tile &tile) {
  return TileView{tile.counts & 0xFFFF, tile.counts >> 16, tile.row_begin, tile.col_begin, tile.n_src,
                  tile.flags,           tile.dup_count,    tile.src_begin, tile.entry_begin, tile.pt_begin};
}

// ring_r on a per-lane mesh dim d, with hops = hop_scale * (mesh_size[d] - 1).
template <int M>
__device__ __forceinline__ double ring_at(double gb, const apc_params &p, int d, int hop_scale) {
  const int n = pick<M>(p.mesh_size, d);
  const double hops = (double)(hop_scale * (n - 1));
  const double latency = p.base_latency + hops * pick<M>(p.lat, d);
  const double bw = div_by(div_by(gb * hops, (double)n, pick<M>(p.inv_mesh, d)), pick<M>(p.bw, d), pick<M>(p.inv_bw, d));
  return latency + bw * 1e6;
}

// Stages tile `tile` with `nthreads` (>= 64) cooperating threads (this thread is `tid`).  The
// caller synchronises before the stage is read.  Only global loads and LDS writes: no stores.
// Every vector load of the tile is issued first, in one round, and the state terms are
// computed from scalar operands while the loads are in flight: under a store-bound kernel
// each dependent round of vector loads queues behind the stores of the other workgroups of
// the compute unit, so the number of rounds, not of loads, is what staging costs.
template <int M, bool DERIVE, bool RM>
__device__ __forceinline__ void stage_tile(const apc_params &p, const TableArgs &a, const apc_tile &tile,
                                           TileStage<M, RM> &st, int tid, int nthreads, TileCopies &copies) {
  constexpr int NS = States<M>::kCount;
  const int rows = tile.counts & 0xFFFF, cols = tile.counts >> 16;
  const int t0 = tile.tensor;  // spec_tensor of the tile's first producer spec (checked by the host)
  const bool no_producer = (tile.flags & APC_EDGE_NO_PRODUCER) != 0;
  const bool terms_wanted = t0 >= 0 && !no_producer;
  bool mixed = !terms_wanted;
  const TermLayout &lay = a.lay;
  const int E = lay.exponents;  // wave-uniform; 0: general layout
  const int lane = tid & 63, wave = tid >> 6;
  // (written and read by the first wavefront only, which stages the producer specs: in order.
  // A kernel argument indexed by the lane: one vector load, part of the round below.)
  uint32_t pair_word = 0;
  if (tid < 16 * M) pair_word = lay.pair[tid];
  // power-of-two layout: the constants of array 2 + lane (whose chain this lane computes) and of
  // the array of the first value this thread computes, also read by lane
  constexpr int kComputed = 3 * M + 2;
  TermArrayConstants chain_of{};
  if (E != 0 && lane < kComputed) chain_of = lay.arrays[lane];
  // ---- the round of vector loads ------------------------------------------------------------
  // producer spec tid, consumer spec nthreads - 1 - tid (taken from the far end: with two
  // wavefronts one loads the producer specs while the other loads the consumer specs).
  // Threads past the tile's specs load its first spec again: unconditional loads, whose
  // values are first touched after the state terms.
  const int jc = tid, jr = nthreads - 1 - tid;
  const bool has_col = jc < cols, has_row = jr < rows;
  const int sp = tile.src_begin + tile.col_begin + (has_col ? jc : 0);
  const int ts = tile.tgt_begin + tile.row_begin + (has_row ? jr : 0);
  const int col_tensor = a.spec_tensor[sp];
  const uint32_t col_codes = a.spec_codes[sp];
  const uint32_t row_codes = a.spec_codes[ts];
  const int row_tensor = a.spec_tensor[ts];
  const int sr = tile.strat_begin + tile.row_begin + (has_row ? jr : 0);
  double row_cpa = 0.0;
  int64_t row_flops = 0, row_rw = 0;
  int row_dtype = 0, row_zero = 1, row_args = 1;
  if (!DERIVE) {
    if (a.per_arg) row_cpa = a.per_arg[sr];
  } else {
    row_flops = a.flops[sr];
    row_rw = a.rw_bytes[sr];
    row_dtype = a.dtype[sr];
    row_zero = a.zero_cost[sr];
    row_args = a.num_args[sr];
  }
  // (every wavefront its own copy of the identical edges' offsets, in lanes 0 .. dup_count - 1)
  const bool has_dup0 = lane < tile.dup_count;
  copies.entry0 = copies.row0 = copies.row_out = 0;
  if (has_dup0) copies.entry0 = a.dup_entry_begin[tile.dup_begin + lane];
  if constexpr (RM) {
    if (has_dup0) copies.row0 = a.dup_row_begin[tile.dup_begin + lane];
    // (wave-uniform, but needed last: with the vector loads of the round, so that the scalar
    // loads the term arrays wait for are one round and not two)
    copies.row_out = a.edge_row_begin[tile.edge];
  }
  // ---- the scalar loads of the round (wave-uniform addresses), issued together ---------------------
  // The tile's tensor (row 0 when the tile has none: unconditional loads, the values are not
  // used then) and the first matrix row of its edge.  The contiguity byte is read as the aligned
  // word around it (which lies in the byte's own page).
  const int t0c = t0 >= 0 ? t0 : 0;
  uint32_t contiguous = 1;
  int64_t tensor_nbytes = 0;
  if constexpr (!DERIVE) {
    const uint8_t *flag = a.tensor_contiguous + t0c;
    const uint32_t byte = (uint32_t)(reinterpret_cast<uintptr_t>(flag) & 3);
    const uint32_t word = uniform_load(reinterpret_cast<const uint32_t *>(flag - byte));
    tensor_nbytes = uniform_load(a.tensor_bytes + t0c);
    fetch_arguments_now(word, tensor_nbytes);
    contiguous = (word >> (8 * byte)) & 0xFFu;
  } else {
    const int t_rank = uniform_load(a.rank + t0c), t_item = uniform_load(a.itemsize + t0c);
    const i64x8 t_shape = uniform_load(reinterpret_cast<const i64x8 *>(a.shape + (int64_t)t0c * APC_MAX_RANK));
    const i64x8 t_stride = uniform_load(reinterpret_cast<const i64x8 *>(a.stride + (int64_t)t0c * APC_MAX_RANK));
    fetch_arguments_now(t_rank, t_item, t_shape[0], t_stride[0]);
    bool ok;
    tensor_bytes_and_contiguity_of(t_rank, t_item, t_shape, t_stride, tensor_nbytes, ok);
    contiguous = ok ? 1u : 0u;
  }
  // ---- term arrays (scalar operands only) ---------------------------------------------------
  if (terms_wanted && E != 0) {
    // power-of-two mesh.  A lane per computed array takes the array's chain on the tensor's
    // bytes (every wavefront its own copy: no barrier), then a lane per (array, exponent) the
    // value.
    const double fbytes = (double)tensor_nbytes;
    StagingScratch &mine = reinterpret_cast<StagingScratch *>(st.terms)[wave];
    if (lane < kComputed) {
      mine.chain[lane] = div_by(div_by(fbytes * chain_of.hops, chain_of.div1, chain_of.inv_div1) * 1e6, chain_of.div2,
                                chain_of.inv_div2);
      mine.value_of[lane] = TermValueConstants{chain_of.lat, chain_of.floor, chain_of.scale, chain_of.shift, 0};
    }
    __builtin_amdgcn_wave_barrier();  // (LDS operations of one wavefront complete in order)
    // (The value constants go through LDS as well.  Read from the kernel arguments by a per-lane
    // index inside the loop below, `lat + ldexp(..)` was compiled to `x + x` in the 4-D
    // instantiations by hipcc 7.2: the placement-pair tests on 4-D power-of-two meshes show it.)
    char *terms = term_base(st, nthreads);
    for (int t = tid; t < kComputed * E; t += nthreads) {
      const int arr = (int)(((uint32_t)t * lay.exponent_magic) >> 16);  // t / E
      const int j = t - arr * E;  // the running bytes are bytes x 2^(j - L - 30)
      const TermValueConstants k = mine.value_of[arr];
      double v = k.lat + __builtin_ldexp(mine.chain[arr], j + k.shift);
      v = v > k.floor ? v : k.floor;
      v = v * k.scale;
      *reinterpret_cast<double *>(terms + j * kPow2Stride + (arr + 2) * 8) = v;
    }
    if (tid < 2 * E) {
      const int j = tid < E ? tid : tid - E;
      *reinterpret_cast<double *>(terms + j * kPow2Stride + (tid < E ? 0 : 8)) = tid < E ? 0.0 : __builtin_inf();
    }
    if (tid == 0) st.gb_unsharded = fbytes / 1024 / 1024 / 1024;
  } else if (terms_wanted) {
    // every collective / read-write term the tile can need, once per running-bytes state, in
    // the reference's operation order (collective_runtime_estimation.py:66-68, :86, :128;
    // torch _collective_utils.py:281-313; compute_estimation.py:302-314)
    const double fbytes = (double)tensor_nbytes;
    for (int k = tid; k < NS; k += nthreads) {
      const int level = 31 - __clz((k >> M) + 1);
      const int rem = k - (((1 << level) - 1) << M);
      const int mask = rem >> level, hist = rem & ((1 << level) - 1);
      double shards = 1.0;  // exact: a product of mesh sizes (torch _dtensor_spec.py:555-561)
#pragma unroll
      for (int i = 0; i < M; ++i)
        if ((mask >> i) & 1) shards *= (double)p.mesh_size[i];
      double gb = fbytes / shards * 0x1p-30;  // / 1024 / 1024 / 1024
#pragma unroll
      for (int i = 0; i < M; ++i) {
        if (i < level && ((hist >> i) & 1)) {
          const double m = (double)p.mesh_size[i];
          gb = ((mask >> i) & 1) ? gb * m : div_by(gb, m, p.inv_mesh[i]);
        }
      }
      double ag = 0.0, rs = 0.0, ar = 0.0;
      if (level >= 1) ag = ring_at<M>(gb, p, level - 1, 1);
      if (level < M) {
        rs = ring_at<M>(gb, p, level, 1);
        ar = ring_at<M>(gb, p, level, 2);
      }
      double a2a = rs;
      a2a *= p.a2a_scale;
      const double rw = rw_time_r(gb * 2 * 1073741824.0, p);
      double *e = reinterpret_cast<double *>(term_base(st, nthreads)) + k * (kGeneralStride / 8);
      e[kZerosArray] = 0.0;
      e[kInfArray] = __builtin_inf();
      e[kRw1Array] = rw;
      e[kRw1Array + 1] = 2.0 * rw;
      e[4] = ag;
      e[5] = rs;
      e[6] = ar;
      e[7] = a2a;
    }
    if (tid == 0) st.gb_unsharded = fbytes / 1024 / 1024 / 1024;
  } else if (tid == 0) {
    st.gb_unsharded = 0.0;
  }
  // ---- what the loads brought, to LDS ---------------------------------------------------------
  if (tid == 0) st.cont = contiguous != 0;
  if (tid < 16 * M) st.pair_base[tid] = pair_word;
  if constexpr (RM) {
    if (tid < APC_TILE_MAX_ROWS) st.rmin[1][tid] = __builtin_inf();  // (slot 0 of every row is always written)
  }
  if (has_col) {
    // info: bit0 valid spec, bit1 fully replicated, bits 4.. mask of sharded mesh dims
    uint32_t info = (col_tensor >= 0 ? 1u : 0u) | (col_codes == 0u ? 2u : 0u);
    uint32_t mask = 0;
#pragma unroll
    for (int i = 0; i < M; ++i) mask |= (kind_of((col_codes >> (8 * i)) & 0xFF) == 2 ? 1u : 0u) << i;
    info |= mask << 4;
    st.colh[jc] = make_uint2(col_codes, info);
    st.col_codes[jc] = col_codes;
    // power-of-two mesh: the producer spec's exponent index, L - log2(its shards)
    uint32_t j0 = (uint32_t)lay.lg_total;
#pragma unroll
    for (int i = 0; i < M; ++i) j0 -= ((mask >> i) & 1u) ? (uint32_t)lay.lg[i] : 0u;
#pragma unroll
    for (int i = 0; i < M; ++i) {
      const int cls = placement_class((col_codes >> (8 * i)) & 0xFF);
      const uint4 base = reinterpret_cast<const uint4 *>(st.pair_base)[i * 4 + cls];
      // general layout: states of this dim for history 0, before the dim and after an update at
      // it; the all-gather (a sharding producer, a replicating consumer: class 0) is charged on
      // the gathered bytes.  (Power-of-two layout: that shift is part of the word's base.)
      const uint32_t k = (uint32_t)States<M>::index(i, 0, 0) + (mask << i);
      const uint32_t k2 = (uint32_t)States<M>::index(i + 1, 0, 0) + (mask << (i + 1)) + (1u << i);
      const uint32_t at = __umul24(E != 0 ? j0 : k, (uint32_t)lay.state_stride);
      const uint32_t at0 = __umul24(E != 0 ? j0 : cls >= 2 ? k2 : k, (uint32_t)lay.state_stride);
      uint32_t *w = st.words + jc * (M * kWordsPerDim + 1) + i * kWordsPerDim;
      w[0] = base.x + at0;
      w[1] = base.y + at;
      w[2] = base.z + at;
      w[3] = base.w + at;
      w[4] = at;  // the zeros array, no read+write, no step
      w[5] = at + kRw1Array * 8u;
    }
    if (col_tensor != t0 || col_tensor < 0) mixed = true;
  }
  if (has_row) {
    uint32_t slots = 0;
    bool all_shard = true;
#pragma unroll
    for (int i = 0; i < M; ++i) {
      const uint32_t t = (row_codes >> (8 * i)) & 0xFF;
      slots |= (uint32_t)((kWordsPerDim * i + placement_class(t)) * 4) << (8 * i);
      all_shard &= kind_of(t) == 2;
    }
    if (M == 2 && all_shard) slots |= kRowAllShard;
    if (row_tensor < 0) {  // a consumer spec that is not a DTensorSpec
      slots |= kRowNotASpec;
      mixed = true;
    }
    if (DERIVE) {  // the value compute_costs_block writes for this strategy
      bool unsupported;
      row_cpa = compute_cost_of(p, row_zero != 0, row_rw, row_flops, row_dtype, unsupported) / (double)row_args;
    }
    st.row[jr] = RowRecord{row_codes, slots, row_cpa};
  }
  // one flag per wavefront, written unconditionally: nothing to clear beforehand
  const bool wave_mixed = __ballot(mixed) != 0;
  if ((tid & 63) == 0) st.mixed[tid >> 6] = wave_mixed ? 1 : 0;
}

// One entry of a tile whose producer specs all name one tensor (column c, row r of the tile).
// Straight-line code: all lookups of an entry are independent of its fp additions, so they
// are issued together; no vector memory loads.
template <int M, bool CONT, bool RESCALE, bool RM>
__device__ __forceinline__ void uniform_entry(const apc_params &p, const TermLayout &lay, const TileStage<M, RM> &st,
                                              const char *terms, int r, int c, double &comm_o, double &total_o,
                                              int &trans_o) {
  const uint32_t src = st.col_codes[c];
  const RowRecord row = st.row[r];
  const uint32_t tgt = row.codes;
  const uint32_t x = src ^ tgt;
  const char *words = reinterpret_cast<const char *>(st.words) + __umul24((uint32_t)c, (M * kWordsPerDim + 1) * 4);
  // ---- integer part: which term at which running index each mesh dim adds -------------------
  uint32_t at = 0;  // byte offset of the running index (history of the earlier dims / exponent steps), mod 2^32
  uint32_t term_at[M], rw_at[M], nc_at[M];
  bool neq[M];
#pragma unroll
  for (int i = 0; i < M; ++i) {
    neq[i] = ((x >> (8 * i)) & 0xFF) != 0;
    // (slot 4: same placement, nothing to add)
    const uint32_t slot = neq[i] ? (row.slots >> (8 * i)) & 0xFFu : (uint32_t)((kWordsPerDim * i + 4) * 4);
    const uint32_t w = *reinterpret_cast<const uint32_t *>(words + slot);
    term_at[i] = (w & 0xFFFFu) + at;
    rw_at[i] = term_at[i] + (uint32_t)(int32_t)(int8_t)(w >> 16);
    if (!CONT) nc_at[i] = *reinterpret_cast<const uint32_t *>(words + (kWordsPerDim * i + 5) * 4) + at;
    at += (uint32_t)__mul24((int32_t)w >> 24, lay.state_stride);  // (24-bit multiplies issue at full rate)
  }
  // ---- lookups ------------------------------------------------------------------------------
  double term[M], rw[M], nc[M];
#pragma unroll
  for (int i = 0; i < M; ++i) {
    term[i] = *reinterpret_cast<const double *>(terms + term_at[i]);
    rw[i] = *reinterpret_cast<const double *>(terms + rw_at[i]);
    if (!CONT) nc[i] = *reinterpret_cast<const double *>(terms + nc_at[i]);
  }
  // ---- additions in the reference's order (0.0 + t == t for these non-negative terms) ------------
  double cost = 0.0;
  // a fully replicated producer returns before the non-contiguity term (:56-62)
  bool cont = CONT || src == 0u;
#pragma unroll
  for (int i = 0; i < M; ++i) {
    if (!CONT) {
      cost += (neq[i] && !cont) ? nc[i] : 0.0;
      cont = cont || neq[i];
    }
    if (CONT && i == 0) cost = term[0];
    else cost += term[i];
    cost += rw[i];  // 0, 1 or 2 read+writes: (double)copies * rw, picked from the staged multiples
  }
  double comm = cost;  // (a banned transition added the +inf term)
  const int trans = x != 0u ? p.transition_scale : 0;  // optimize_sharding.py:345-351
  if (M == 2 && src == 0x4040u && (row.slots & kRowAllShard)) {  // (Partial, Partial) -> all Shard walks dim 1 first
    comm = entry_cost<M>(src, tgt, st.gb_unsharded, CONT, p);
  }
  // :358-359; the quotient through the reciprocal is the division's (div_by), +inf stays +inf
  if (RESCALE) comm = comm < __builtin_inf() ? div_by(comm, p.rescale, lay.inv_rescale) : comm;
  comm_o = comm;
  total_o = comm + row.cpa + (double)trans;  // :368-372
  trans_o = trans;
}

// The three output streams of one tile: wave-uniform bases, so an entry's addresses are a
// scalar base plus a 32-bit lane offset (the host checks that a tile spans < 4 GiB).
struct TileOut {
  double *comm;
  uint8_t *trans;
  double *cost;
  int64_t entry_begin;  // first entry of the tile's edge (an identical edge's values sit at its own first entry)
};

// Which of the three per-entry output arrays a launch writes, as a compile-time choice of the
// kernel (no per-store checks, and the registers of streams that are not written are free):
// the planner's table build wants the assembled cost alone (what the ILP objective is summed
// from, optimize_sharding.py:650-655; comm and transition are fetched by a later launch only
// if a report asks for them), a caller that wants every array gets all three, any other subset
// is checked per store.
enum : int { kOutAny = 0, kOutAll = 1, kOutCost = 2 };

// Stores one entry's values to its edge and to every identical edge.  Called by every lane of
// the wavefront (`active`: this lane holds an entry), so that the copies' offsets are read from
// their lanes under uniform control flow.
template <int OUT>
__device__ __forceinline__ void store_entry(const TileOut &o, int dup_count, const TileCopies &copies, bool active,
                                            uint32_t local, double comm, double total, int trans) {
  constexpr bool ALL = OUT == kOutAll, COST = OUT == kOutCost;
  const uint32_t off8 = local * 8u;
  if (active) {
    if (ALL || (!COST && o.comm)) *reinterpret_cast<double *>(reinterpret_cast<char *>(o.comm) + off8) = comm;
    if (ALL || (!COST && o.trans)) o.trans[local] = (uint8_t)trans;
    if (ALL || COST || o.cost) *reinterpret_cast<double *>(reinterpret_cast<char *>(o.cost) + off8) = total;
  }
  for (int d = 0; d < dup_count; ++d) {
    const int64_t delta = value_of_lane(copies.entry0, d) - o.entry_begin;
    if (active) {
      if (ALL || (!COST && o.comm)) *reinterpret_cast<double *>(reinterpret_cast<char *>(o.comm + delta) + off8) = comm;
      if (ALL || (!COST && o.trans)) (o.trans + delta)[local] = (uint8_t)trans;
      if (ALL || COST || o.cost) *reinterpret_cast<double *>(reinterpret_cast<char *>(o.cost + delta) + off8) = total;
    }
  }
}

// A 32-bit value from the lane `N` further on within the lane's row of 16 (DPP row_shl:N); a
// lane whose source lies outside its row keeps its own value.
template <int N>
__device__ __forceinline__ int from_lane_ahead(int x) {
  return __builtin_amdgcn_update_dpp(x, x, 0x100 + N, 0xF, 0xF, false);
}
template <int N>
__device__ __forceinline__ double from_lane_ahead(double x) {
  const int lo = from_lane_ahead<N>(__double2loint(x)), hi = from_lane_ahead<N>(__double2hiint(x));
  return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double value_of_lane(double x, int lane) {  // lane: a constant
  const int lo = __builtin_amdgcn_readlane(__double2loint(x), lane), hi = __builtin_amdgcn_readlane(__double2hiint(x), lane);
  return __hiloint2double(hi, lo);
}

// Row minima inside the tile kernel.  The 64 lanes of a wavefront hold 64 consecutive entries
// of the tile (inactive lanes: +inf), row after row.  `c` is the lane's column, `cols` the row
// length.  First a segmented minimum by doubling inside every 16 lanes (data-parallel
// primitives: vector ALU only, the LDS pipe stays free for the entry loop's lookups): a lane
// then holds the minimum, and the first column that has it, of its row's entries from itself to
// the end of its 16 lanes.  Lanes 16, 32 and 48 hold such a part for a row that came in from the
// lanes before them: their values are read as scalars and joined, in lane order, by the lanes
// whose row reaches them.  The first lane of every run of one row writes the row's slot.
// row_min_in_wave: the reduction itself; on return a lane holds minimum and first argmin of its
// row's entries from itself to the row's end within the wavefront (the whole row for c == 0).
__device__ __forceinline__ void row_min_in_wave(bool active, double value, int c, int cols, int lane, double &m, int &mc) {
  m = active ? value : __builtin_inf();
  mc = c;
  const int in_row16 = lane & 15;
#define APC_ROW_MIN_STEP(N_)                                                            \
  if (N_ < cols) { /* (cols is wave-uniform) */                                         \
    const double om = from_lane_ahead<N_>(m);                                           \
    const int oc = from_lane_ahead<N_>(mc);                                             \
    /* that lane holds an entry of the same row; strict <: ties keep the lower column */ \
    if (in_row16 + N_ < 16 && c + N_ < cols && om < m) {                                \
      m = om;                                                                           \
      mc = oc;                                                                          \
    }                                                                                   \
  }
  APC_ROW_MIN_STEP(1)
  APC_ROW_MIN_STEP(2)
  APC_ROW_MIN_STEP(4)
  APC_ROW_MIN_STEP(8)
#undef APC_ROW_MIN_STEP
#define APC_ROW_MIN_JOIN(LANE_)                                              \
  {                                                                          \
    const double pm = value_of_lane(m, LANE_);                               \
    const int pc = __builtin_amdgcn_readlane(mc, LANE_);                     \
    if (LANE_ > lane && c + (LANE_ - lane) < cols && pm < m) {               \
      m = pm;                                                                \
      mc = pc;                                                               \
    }                                                                        \
  }
  if (cols > 1) {
    APC_ROW_MIN_JOIN(16)
    APC_ROW_MIN_JOIN(32)
    APC_ROW_MIN_JOIN(48)
  }
#undef APC_ROW_MIN_JOIN
}

__device__ __forceinline__ void row_min_chunk(double (&rmin)[2][APC_TILE_MAX_ROWS], int (&rarg)[2][APC_TILE_MAX_ROWS],
                                              bool active, double value, int r, int c, int cols, int lane) {
  double m;
  int mc;
  row_min_in_wave(active, value, c, cols, lane, m, mc);
  if (active && (c == 0 || lane == 0)) {
    const int slot = c == 0 ? 0 : 1;
    rmin[slot][r] = m;
    rarg[slot][r] = mc;
  }
}

// After every wavefront of the tile has written its slots: one thread per row joins the two
// parts and stores minimum and first argmin to the row of the tile's edge and of every
// identical edge.  (Called by every thread of the workgroup.)
template <int M>
__device__ __forceinline__ void row_min_finish(const TableArgs &a, TileStage<M, true> &st, const TileView &v,
                                               const TileCopies &copies, int tid, int nthreads) {
  __syncthreads();
  // lane = row, wavefront w takes the copies w, w + waves, ...: copy 0 is the tile's own edge, copy
  // d > 0 the d-th identical edge (a tile of many copies ends with a short store phase in every
  // wavefront instead of a long one in the first)
  const int row = tid & 63;
  const bool live = row < v.rows;
  double m = __builtin_inf();
  int mc = 0;
  if (live) {
    m = st.rmin[0][row];
    mc = st.rarg[0][row];
    const double m1 = st.rmin[1][row];
    if (m1 < m) {  // the later part wins only if strictly smaller
      m = m1;
      mc = st.rarg[1][row];
    }
  }
  const int waves = nthreads >> 6;
  for (int d = uniform_i32(tid >> 6); d <= v.dup_count; d += waves) {
    const int64_t first = d == 0 ? uniform_i64(copies.row_out) : value_of_lane(copies.row0, d - 1);  // (uniform control flow)
    if (live) {
      const int64_t out = first + v.row_begin + row;
      a.row_min_out[out] = m;
      a.row_arg_out[out] = v.col_begin + mc;
    }
  }
}

// The entry loop of a tile that holds whole rows, with the row minima: the walk of
// uniform_tile_entries, except that every lane of a wavefront makes the same number of
// passes (a lane in front of the tile's first entry idles in the first pass instead of
// wrapping round), so that the lanes of one pass hold consecutive entries.
template <int M, bool CONT, bool RESCALE, int OUT>
__device__ __forceinline__ void uniform_tile_entries_row_min(const apc_params &p, const TableArgs &a, TileStage<M, true> &st,
                                                             const TileView &v, const TileCopies &copies, int tid,
                                                             int nthreads) {
  const int n = v.rows * v.cols;
  const int dr = nthreads / v.cols, dc = nthreads - dr * v.cols;
  const int64_t tile_base = v.entry_begin + (int64_t)v.row_begin * v.n_src + v.col_begin;
  const int shift = (int)(tile_base & 63);
  const int lane = tid & 63;
  int idx = tid - shift;
  const int first = idx < 0 ? idx + nthreads : idx;
  int r = first / v.cols, c = first - r * v.cols;
  const TileOut out{a.comm_out ? a.comm_out + tile_base : nullptr, a.trans_out ? a.trans_out + tile_base : nullptr,
                    a.cost_out ? a.cost_out + tile_base : nullptr, v.entry_begin};
  for (int wave_first = tid - lane - shift; wave_first < n; wave_first += nthreads, idx += nthreads) {
    const bool active = idx >= 0 && idx < n;
    double comm = 0.0, total = 0.0;
    int trans = 0;
    if (active) uniform_entry<M, CONT, RESCALE>(p, a.lay, st, term_base(st, nthreads), r, c, comm, total, trans);
    store_entry<OUT>(out, v.dup_count, copies, active, __umul24((uint32_t)r, (uint32_t)v.n_src) + (uint32_t)c, comm, total,
                     trans);
    row_min_chunk(st.rmin, st.rarg, active, total, r, c, v.cols, lane);
    if (active) {
      c += dc;
      r += dr;
      if (c >= v.cols) {
        c -= v.cols;
        r += 1;
      }
    }
  }
  row_min_finish<M>(a, st, v, copies, tid, nthreads);
}

// The per-entry loop of such a tile for `nthreads` threads (this one is `tid`): a flattened
// (row, column) walk, so a wavefront writes 64 consecutive entries.
template <int M, bool CONT, bool RESCALE, int OUT, bool RM>
__device__ __forceinline__ void uniform_tile_entries(const apc_params &p, const TableArgs &a, const TileStage<M, RM> &st,
                                                     const TileView &v, const TileCopies &copies, int tid, int nthreads) {
  const int n = v.rows * v.cols;
  const int dr = nthreads / v.cols, dc = nthreads - dr * v.cols;
  const int64_t tile_base = v.entry_begin + (int64_t)v.row_begin * v.n_src + v.col_begin;
  // A full-width tile is one contiguous run of entries: lanes are shifted so that every
  // wavefront store starts on a 64-entry boundary of the output arrays (whole 128-byte lines
  // of the fp64 streams) instead of straddling one more line than it fills.  Every lane of a
  // wavefront makes the same number of passes (a lane in front of the tile's first entry idles
  // in the first one), so the copies' offsets are read under uniform control flow.
  const int shift = v.cols == v.n_src ? (int)(tile_base & 63) : 0;
  const int lane = tid & 63;
  int idx = tid - shift;
  const int first = idx < 0 ? idx + nthreads : idx;
  int r = first / v.cols, c = first - r * v.cols;
  const TileOut out{a.comm_out ? a.comm_out + tile_base : nullptr, a.trans_out ? a.trans_out + tile_base : nullptr,
                    a.cost_out ? a.cost_out + tile_base : nullptr, v.entry_begin};
  for (int wave_first = tid - lane - shift; wave_first < n; wave_first += nthreads, idx += nthreads) {
    const bool active = idx >= 0 && idx < n;
    double comm = 0.0, total = 0.0;
    int trans = 0;
    if (active) uniform_entry<M, CONT, RESCALE>(p, a.lay, st, term_base(st, nthreads), r, c, comm, total, trans);
    store_entry<OUT>(out, v.dup_count, copies, active, __umul24((uint32_t)r, (uint32_t)v.n_src) + (uint32_t)c, comm, total,
                     trans);
    if (active) {
      c += dc;
      r += dr;
      if (c >= v.cols) {
        c -= v.cols;
        r += 1;
      }
    }
  }
}

// Generic loop: pass-through edges and edges whose producer specs name different tensors.
// Every lane of a wavefront makes the same number of passes; ROW_MIN (tiles of whole rows only):
// the row minima are taken on the way.
template <int M, bool DERIVE, bool ROW_MIN, bool RM>
__device__ __forceinline__ void generic_tile_entries(const apc_params &p, const TableArgs &a, TileStage<M, RM> &st,
                                                     const TileView &v, const TileCopies &copies, int tid, int nthreads) {
  const int n = v.rows * v.cols;
  const int lane = tid & 63;
  int r = tid / v.cols, c = tid - r * v.cols;
  const int dr = nthreads / v.cols, dc = nthreads - dr * v.cols;
  const bool no_producer = (v.flags & APC_EDGE_NO_PRODUCER) != 0;
  for (int idx = tid; idx - lane < n; idx += nthreads) {
    const bool active = idx < n;
    double total = 0.0, comm = 0.0;
    int trans = 0;
    int64_t o = 0;
    if (active) {
      const int64_t local = (int64_t)(v.row_begin + r) * v.n_src + (v.col_begin + c);
      const uint32_t src = st.colh[c].x, cinfo = st.colh[c].y;
      const RowRecord row = st.row[r];
      const uint32_t tgt = row.codes;
      if (no_producer || !(cinfo & 1u) || (row.slots & 0xFFu) == kRowNotASpec) {
        comm = a.pt_values[v.pt_begin + local];
      } else {
        trans = (src != tgt) ? p.transition_scale : 0;
        const int sten = a.spec_tensor[v.src_begin + v.col_begin + c];
        int64_t shards = 1;
#pragma unroll
        for (int i = 0; i < M; ++i)
          if (kind_of((src >> (8 * i)) & 0xFF) == 2) shards *= p.mesh_size[i];
        int64_t sten_bytes;
        bool sten_contiguous;
        tensor_info<DERIVE>(a, sten, sten_bytes, sten_contiguous);
        const double gb = (double)sten_bytes / (double)shards / 1024 / 1024 / 1024;
        comm = entry_cost<M>(src, tgt, gb, sten_contiguous, p);
      }
      if (v.flags & APC_EDGE_GRAD_RESCALE) comm = comm / p.rescale;
      o = v.entry_begin + local;
      total = comm + row.cpa + (double)trans;
      if (a.comm_out) a.comm_out[o] = comm;
      if (a.trans_out) a.trans_out[o] = (uint8_t)trans;
      if (a.cost_out) a.cost_out[o] = total;
    }
    for (int d = 0; d < v.dup_count; ++d) {
      const int64_t delta = value_of_lane(copies.entry0, d) - v.entry_begin;  // (uniform control flow)
      if (active) {
        if (a.comm_out) a.comm_out[o + delta] = comm;
        if (a.trans_out) a.trans_out[o + delta] = (uint8_t)trans;
        if (a.cost_out) a.cost_out[o + delta] = total;
      }
    }
    if constexpr (ROW_MIN && RM) row_min_chunk(st.rmin, st.rarg, active, total, r, c, v.cols, lane);
    if (active) {
      c += dc;
      r += dr;
      if (c >= v.cols) {
        c -= v.cols;
        r += 1;
      }
    }
  }
  if constexpr (ROW_MIN && RM) row_min_finish<M>(a, st, v, copies, tid, nthreads);
}

// All entries of a staged tile.  Row minima are taken when the caller wants them and the tile
// holds whole rows (which the host arranges for every tile of a table before asking).
template <int M, bool DERIVE, bool RM, int OUT>
__device__ __forceinline__ void tile_entries(const apc_params &p, const TableArgs &a, TileStage<M, RM> &st,
                                             const TileView &v, const TileCopies &copies, int tid, int nthreads) {
  int mixed = st.mixed[0];
  for (int w = 1; w < nthreads / 64; ++w) mixed |= st.mixed[w];
  const bool row_minima = RM && v.cols == v.n_src;
  if (uniform_i32(mixed)) {
    if constexpr (RM) {
      if (row_minima) {
        generic_tile_entries<M, DERIVE, true>(p, a, st, v, copies, tid, nthreads);
        return;
      }
    }
    generic_tile_entries<M, DERIVE, false>(p, a, st, v, copies, tid, nthreads);
    return;
  }
  const bool rescale = (v.flags & APC_EDGE_GRAD_RESCALE) != 0;
#define APC_TILE_LOOP(CONT_, RESCALE_)                                                            \
  do {                                                                                            \
    if constexpr (RM) {                                                                           \
      if (row_minima) {                                                                           \
        uniform_tile_entries_row_min<M, CONT_, RESCALE_, OUT>(p, a, st, v, copies, tid, nthreads); \
        break;                                                                                    \
      }                                                                                           \
    }                                                                                             \
    uniform_tile_entries<M, CONT_, RESCALE_, OUT>(p, a, st, v, copies, tid, nthreads);            \
  } while (0)
  if (uniform_i32(st.cont)) {
    if (rescale) { APC_TILE_LOOP(true, true); } else { APC_TILE_LOOP(true, false); }
  } else {
    if (rescale) { APC_TILE_LOOP(false, true); } else { APC_TILE_LOOP(false, false); }
  }
#undef APC_TILE_LOOP
}

// A tile record (64 bytes, wave-uniform) as one scalar load.
__device__ __forceinline__ apc_tile load_tile_record(const apc_tile *tiles, int64_t tile_id) {
  static_assert(sizeof(apc_tile) == sizeof(i32x16), "one 64-byte scalar load per record");
  const i32x16 raw = uniform_load(reinterpret_cast<const i32x16 *>(tiles + tile_id));
  apc_tile tile;
  __builtin_memcpy(&tile, &raw, sizeof(tile));
  return tile;
}

// A tile's record and the table addresses its wavefronts use, all fetched on entry under one wait
// (fetch_arguments_now): the record's address needs only arguments that arrive in registers.
template <bool DERIVE, bool RM, int OUT>
__device__ __forceinline__ apc_tile fetch_tile(const apc_tile *tiles, int64_t tile_id, const TableArgs &a) {
  const apc_tile tile = load_tile_record(tiles, tile_id);
  if constexpr (DERIVE && RM && OUT == kOutCost)
    fetch_arguments_now(tile.counts, a.lay.exponents, a.spec_codes, a.spec_tensor, a.dup_entry_begin, a.cost_out, a.rank, a.itemsize, a.shape,
                        a.stride, a.flops, a.rw_bytes, a.dtype, a.zero_cost, a.num_args, a.edge_row_begin, a.dup_row_begin,
                        a.row_min_out, a.row_arg_out);
  else if constexpr (DERIVE)
    fetch_arguments_now(tile.counts, a.lay.exponents, a.spec_codes, a.spec_tensor, a.dup_entry_begin, a.rank, a.itemsize, a.shape, a.stride,
                        a.flops, a.rw_bytes, a.dtype, a.zero_cost, a.num_args);
  else if constexpr (RM)
    fetch_arguments_now(tile.counts, a.lay.exponents, a.spec_codes, a.spec_tensor, a.dup_entry_begin, a.tensor_bytes, a.tensor_contiguous,
                        a.per_arg, a.edge_row_begin, a.dup_row_begin);
  else
    fetch_arguments_now(tile.counts, a.lay.exponents, a.spec_codes, a.spec_tensor, a.dup_entry_begin, a.tensor_bytes, a.tensor_contiguous,
                        a.per_arg);
  return tile;
}

template <int M, int kTileThreads, bool RM, int OUT>
__device__ __forceinline__ void redistribute_tile(const apc_params &p, const TableArgs &a, const apc_tile *tiles, int n_tiles,
                                                  int xcd_shift, TileStage<M, RM> &stage) {
  const int64_t tile_id = xcd_chunked_unit(xcd_shift);
  if (tile_id >= n_tiles) return;
  static_assert(kTileThreads == 64 || kTileThreads == 128 || kTileThreads == 256, "wavefronts per tile: 1, 2 or 4");
  static_assert(kTileThreads >= APC_TILE_MAX_COLS && kTileThreads >= APC_TILE_MAX_ROWS &&
                kTileThreads >= APC_TILE_MAX_DUPS, "one staging round covers a tile");
  const apc_tile tile = fetch_tile<false, RM, OUT>(tiles, tile_id, a);
  // a record the host validator would have rejected (more identical edges than lanes hold): skipped
  if ((unsigned)tile.dup_count > (unsigned)APC_TILE_MAX_DUPS) return;
  TileCopies copies;
  stage_tile<M, false, RM>(p, a, tile, stage, threadIdx.x, kTileThreads, copies);
  settle(copies);
  __syncthreads();
  tile_entries<M, false, RM, OUT>(p, a, stage, view_of(tile), copies, threadIdx.x, kTileThreads);
}

// Wavefronts per SIMD the tile kernels ask for: what the LDS of their larger, row-minimum
// instantiation leaves room for (one-wavefront workgroups and 4-D meshes hold more LDS per
// wavefront).  Asked for explicitly because the compiler sizes its register budget by the LDS
// use otherwise: the row-minimum kernel got 97 registers and 4 wavefronts on a 3-D mesh where 67
// registers do without spilling (stress table 2.94 -> 2.58 ms); the kernel without the minima
// gains 1 - 2 % (same box: stress 1.93 -> 1.88 ms, Llama-3-70B 251 -> 248 us).
constexpr int tile_waves_per_simd(int mesh_ndim, int threads, bool row_min) {
  if (mesh_ndim >= 4) return threads >= 256 ? 4 : threads >= 128 ? 3 : 2;
  if (threads < 128) return mesh_ndim <= 1 ? 7 : mesh_ndim == 2 ? 6 : 4;
  // two-wavefront tiles without the minima fit sixteen to a compute unit (under 10 KB of LDS
  // each on a power-of-two mesh): all eight wavefront slots of a SIMD, 64 registers
  return threads == 128 && !row_min ? 8 : 7;
}

template <int M, int kTileThreads, int OUT>
__global__ __launch_bounds__(kTileThreads) __attribute__((amdgpu_waves_per_eu(tile_waves_per_simd(M, kTileThreads, false), 8)))
void redistribute_tiles_kernel(const apc_tile *tiles, int n_tiles, int xcd_shift, apc_params p, TableArgs a) {
  extern __shared__ __align__(16) unsigned char s_stage_bytes[];  // stage_lds_bytes<M, false>
  redistribute_tile<M, kTileThreads, false, OUT>(p, a, tiles, n_tiles, xcd_shift,
                                                 *reinterpret_cast<TileStage<M, false> *>(s_stage_bytes));
}

// The same with the row minima.
template <int M, int kTileThreads, int OUT>
__global__ __launch_bounds__(kTileThreads)
__attribute__((amdgpu_waves_per_eu(tile_waves_per_simd(M, kTileThreads, true), 8)))
void redistribute_tiles_row_min_kernel(const apc_tile *tiles, int n_tiles, int xcd_shift, apc_params p, TableArgs a) {
  extern __shared__ __align__(16) unsigned char s_stage_bytes[];  // stage_lds_bytes<M, true>
  redistribute_tile<M, kTileThreads, true, OUT>(p, a, tiles, n_tiles, xcd_shift,
                                                *reinterpret_cast<TileStage<M, true> *>(s_stage_bytes));
}

// Every table of a pass in one launch: workgroups [0, tile_blocks) take the tiles of the
// redistribution-cost matrices (tile_blocks = n_tiles rounded up to the XCD chunking), the
// next spec_blocks the spec table, then the tensor table, then the compute costs, kThreads rows
// per workgroup.  No workgroup reads what another writes: a tile derives its tensor's byte
// count and contiguity and its consumer strategies' compute costs with the functions the
// table workgroups use (TableArgs), so the values are the same bits.  One launch instead of
// two spares a table of a few tens of MB one ramp-up and one drain of the chip, which at that
// size are a third of each kernel.
// (Wavefronts per SIMD are capped at 5 on 1-D and 2-D meshes: with more resident, the launch's
// many store streams hinder each other a little.  Llama-3-8B table, each pair on one box:
// 18.5 us against 18.9 us uncapped, 18.7 us against 18.8 us on another box; capped at 6 as
// uncapped; 20.3 us capped at 3 or when asked for 8.  The mixture-of-experts table: no change.)
template <int M, int kThreads, bool RM, int OUT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(M <= 2 ? 5 : 1, M <= 2 ? 5 : 8)))
void build_tables_kernel(const apc_tile *tiles, int n_tiles, int xcd_shift, int64_t tile_blocks, apc_params p, TableArgs a,
                         TensorTableArgs t, SpecTableArgs sp, ComputeCostArgs c, int64_t spec_blocks,
                         int64_t tensor_blocks) {
  constexpr size_t kRowBytes = (size_t)kThreads * (APC_MAX_RANK + 1) * sizeof(int64_t);
  constexpr size_t kStage = sizeof(TileStage<M, RM>) + sizeof(StagingScratch) * (kThreads / 64);
  constexpr size_t kLds = kStage > kRowBytes ? kStage : kRowBytes;
  __shared__ __align__(16) unsigned char s_raw[kLds];
  static_assert(kThreads == 64 || kThreads == 128 || kThreads == 256, "wavefronts per workgroup: 1, 2 or 4");
  const int64_t b = blockIdx.x;
  if (b < tile_blocks) {
    const int64_t per = tile_blocks >> xcd_shift;
    const int64_t tile_id = (b & ((1 << xcd_shift) - 1)) * per + (b >> xcd_shift);
    if (tile_id >= n_tiles) return;
    TileStage<M, RM> &stage = *reinterpret_cast<TileStage<M, RM> *>(s_raw);
    const apc_tile tile = fetch_tile<true, RM, OUT>(tiles, tile_id, a);
    if ((unsigned)tile.dup_count > (unsigned)APC_TILE_MAX_DUPS) return;  // (see redistribute_tile)
    TileCopies copies;
    stage_tile<M, true, RM>(p, a, tile, stage, threadIdx.x, kThreads, copies);
    settle(copies);
    __syncthreads();
    tile_entries<M, true, RM, OUT>(p, a, stage, view_of(tile), copies, threadIdx.x, kThreads);
    return;
  }
  const int64_t tb = b - tile_blocks;
  if (tb < spec_blocks) spec_tables_block<kThreads>(tb, p, sp, reinterpret_cast<int64_t *>(s_raw));
  else if (tb < spec_blocks + tensor_blocks) tensor_tables_block<kThreads>(tb - spec_blocks, t);
  else compute_costs_block<kThreads>(tb - spec_blocks - tensor_blocks, p, c);
}

// ------------------------------------------------------------------------------------------
// Packed tiles: the planner's pass over a small table, every wavefront on its own.
//
// A table of a few million entries is bound by the latency of one workgroup: all workgroups are
// resident at once, stage and then store in step, and the chain of dependent loads in front of
// the first store decides the launch.  Here a workgroup's loads depend on nothing but its index
// (one fixed-size record per tile, copied out of the tables by the host: apc_packed_tile), and
// nothing is staged in LDS: lane j of every wavefront holds producer spec j, consumer spec j and
// the compute cost / num_args of consumer strategy j; a wavefront walks whole matrix rows,
// fetches an entry's two specs from their lanes, evaluates the entry directly
// (collective_runtime_estimation.py:37-153 in the reference's operation order, divisions through
// the checked reciprocals), reduces the row minima across its lanes and stores values and minima to
// the tile's edge and to every identical edge.  No barrier, no second pass over the rows.
// ------------------------------------------------------------------------------------------
struct DimConstants {  // of one mesh dim, wave-uniform
  double n, inv_n, bw, inv_bw;
  double hops1, lat1;  // all-gather, reduce-scatter, all-to-all: n - 1 hops (torch _collective_utils.py:281-301)
  double hops2, lat2;  // all-reduce: 2 (n - 1) hops (:304-313)
};
template <int M>
struct FlatConstants {
  DimConstants dim[M];
};

template <int M>
__device__ __forceinline__ FlatConstants<M> flat_constants(const apc_params &p) {
  FlatConstants<M> k;
#pragma unroll
  for (int i = 0; i < M; ++i) {
    DimConstants &d = k.dim[i];
    d.n = (double)p.mesh_size[i];
    d.inv_n = p.inv_mesh[i];
    d.bw = p.bw[i];
    d.inv_bw = p.inv_bw[i];
    d.hops1 = (double)(p.mesh_size[i] - 1);
    d.hops2 = (double)(2 * (p.mesh_size[i] - 1));
    d.lat1 = p.base_latency + d.hops1 * p.lat[i];
    d.lat2 = p.base_latency + d.hops2 * p.lat[i];
  }
  return k;
}

// entry_cost without branches: every lane of a wavefront evaluates its own (producer spec,
// consumer spec) pair, whatever collectives the pair needs.  What a mesh dim adds is selected,
// not branched on: the ring term of the one collective the dim can need (none: + 0.0, which
// leaves a non-negative sum unchanged), 0, 1 or 2 read+write reshuffles ((double)copies x rw:
// 0.0, rw, 2.0 x rw).  FIRST = 1 (2-D meshes): dim 1 before dim 0 (:146-151).  CONT: the tensor
// is contiguous (no lane ever adds the non-contiguity term).  gb = bytes / num_shards / 1024^3.
template <int M, int FIRST, bool CONT>
__device__ __forceinline__ double entry_cost_flat(uint32_t srcp, uint32_t tgtp, double gb, const apc_params &p,
                                                  const FlatConstants<M> &k) {
  double cost = 0.0;
  bool banned = false, cont = CONT;
  bool tgt_partial = false;
#pragma unroll
  for (int s = 0; s < M; ++s) {
    const int i = (M == 2 && FIRST == 1) ? 1 - s : s;
    const DimConstants &d = k.dim[i];
    const uint32_t c = (srcp >> (8 * i)) & 0xFF, t = (tgtp >> (8 * i)) & 0xFF;
    const bool neq = c != t;
    const uint32_t ck = c >> 6, tk = t >> 6;
    tgt_partial |= tk == 1;
    const bool from_shard = neq && ck == 2, from_partial = neq && ck == 1;
    const bool is_ag = from_shard && tk == 0, is_a2a = from_shard && tk == 2;  // :83-113
    const bool is_ar = from_partial && tk == 0, is_rs = from_partial && tk == 2;  // :115-130
    banned |= neq && tk == 1 && ck != 1;  // :131-138
    if (!CONT) {  // :81-82: charged once, on the bytes before this dim
      const double rw_before = rw_time_r(gb * 2 * 1073741824.0, p);
      cost += (neq && !cont) ? rw_before : 0.0;
      cont = cont || neq;  // :141
    }
    const double x = is_ag ? gb * d.n : gb;  // an all-gather is charged on the gathered bytes (:86)
    const double hops = is_ar ? d.hops2 : d.hops1;
    const double ring0 = (is_ar ? d.lat2 : d.lat1) + div_by(div_by(x * hops, d.n, d.inv_n), d.bw, d.inv_bw) * 1e6;
    const double ring = is_a2a ? ring0 * p.a2a_scale : ring0;  // :22-32
    cost += (from_shard || from_partial) && tk != 1 ? ring : 0.0;
    const double rw = rw_time_r(x * 2 * 1073741824.0, p);
    const uint32_t cn = (c & 0x0F) != 0 ? 1u : 0u, tn = (t & 0x0F) != 0 ? 1u : 0u;
    const uint32_t copies = is_ag ? cn : is_a2a ? cn + tn : is_rs ? tn : 0u;
    cost += copies == 0u ? 0.0 : copies == 1u ? rw : 2.0 * rw;
    gb = is_ag ? x : is_rs ? div_by(gb, d.n, d.inv_n) : gb;  // :86, :128
  }
  if (srcp == 0u) return tgt_partial ? __builtin_inf() : 0.0;  // :56-62
  return banned ? __builtin_inf() : cost;
}

// The same entry on a mesh whose sizes are all powers of two (TermLayout::exponents != 0; "Term
// arrays" above): the running bytes are the tensor's bytes x 2^(j - L - 30) for an integer j a lane
// carries from dim to dim, and every term is one ldexp of a wave-uniform chain value: no division
// per entry.  R / B[d]: the chains of the read+write and of dim d's one-hop ring on the tensor's
// bytes (TermArrayConstants of arrays 2 and 4 + 3 d).
template <int M>
struct Pow2Constants {
  double R, B[M];
  double lat1[M], lat2[M];
  int lg[M], shift[M];  // log2 n_d; -L - 30 - log2 n_d
  int rw_shift;         // -L - 30 + 31
  double floor;         // launch floor of a read+write
};

template <int M, int FIRST, bool CONT>
__device__ __forceinline__ double entry_cost_pow2(uint32_t srcp, uint32_t tgtp, int j, double a2a_scale, const Pow2Constants<M> &k) {
  double cost = 0.0;
  bool banned = false, cont = CONT, tgt_partial = false;
#pragma unroll
  for (int s = 0; s < M; ++s) {
    const int i = (M == 2 && FIRST == 1) ? 1 - s : s;
    const uint32_t c = (srcp >> (8 * i)) & 0xFF, t = (tgtp >> (8 * i)) & 0xFF;
    const bool neq = c != t;
    const uint32_t ck = c >> 6, tk = t >> 6;
    tgt_partial |= tk == 1;
    const bool from_shard = neq && ck == 2, from_partial = neq && ck == 1;
    const bool is_ag = from_shard && tk == 0, is_a2a = from_shard && tk == 2;
    const bool is_ar = from_partial && tk == 0, is_rs = from_partial && tk == 2;
    banned |= neq && tk == 1 && ck != 1;
    if (!CONT) {
      const double before = __builtin_ldexp(k.R, j + k.rw_shift);
      cost += (neq && !cont) ? (before > k.floor ? before : k.floor) : 0.0;
      cont = cont || neq;
    }
    const int jx = is_ag ? j + k.lg[i] : j;  // an all-gather is charged on the gathered bytes
    const double ring0 = (is_ar ? k.lat2[i] : k.lat1[i]) + __builtin_ldexp(k.B[i], jx + k.shift[i] + (is_ar ? 1 : 0));
    const double ring = is_a2a ? ring0 * a2a_scale : ring0;
    cost += (from_shard || from_partial) && tk != 1 ? ring : 0.0;
    const double rw0 = __builtin_ldexp(k.R, jx + k.rw_shift);
    const double rw = rw0 > k.floor ? rw0 : k.floor;
    const uint32_t cn = (c & 0x0F) != 0 ? 1u : 0u, tn = (t & 0x0F) != 0 ? 1u : 0u;
    const uint32_t copies = is_ag ? cn : is_a2a ? cn + tn : is_rs ? tn : 0u;
    cost += copies == 0u ? 0.0 : copies == 1u ? rw : 2.0 * rw;
    j = is_ag ? jx : is_rs ? j - k.lg[i] : j;
  }
  if (srcp == 0u) return tgt_partial ? __builtin_inf() : 0.0;
  return banned ? __builtin_inf() : cost;
}

__device__ __forceinline__ int from_lane(int v, int lane) { return __builtin_amdgcn_ds_bpermute(lane << 2, v); }
__device__ __forceinline__ double from_lane(double v, int lane) {
  return __hiloint2double(from_lane(__double2hiint(v), lane), from_lane(__double2loint(v), lane));
}
__device__ __forceinline__ int64_t from_lane_i64(int64_t v, int lane) {
  const uint32_t lo = (uint32_t)from_lane((int)(uint32_t)v, lane), hi = (uint32_t)from_lane((int)(uint32_t)((uint64_t)v >> 32), lane);
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

// value -> *(double *)((char *)base + byte_offset) for a wave-uniform base: the address stays a
// scalar register pair plus a 32-bit lane offset (left to the compiler, the sum is re-associated
// into per-lane 64-bit arithmetic inside a loop over bases).  A store needs no wait before the
// wavefront ends, and a wait by count for an older load stays correct with younger stores in
// flight (loads return in order among themselves).
// (sc0 sc1: the store is written through to memory.  Left in the L2 until the kernel ends, the
// table's lines are written back after the last wavefront has finished, and a launch of this
// size waits for that: 10.0 -> 8.6 us on the Llama-3-8B table.)
// (s_nop 4: a vector-memory instruction may read a scalar register a vector instruction wrote,
// such as a value fetched from a lane, only five cycles later; the compiler inserts that wait
// for its own instructions and does not look inside an asm statement.)
__device__ __forceinline__ void store_at(double *base, uint32_t byte_offset, double value) {
  __asm__ volatile("s_nop 4\n\tglobal_store_dwordx2 %0, %1, %2 sc0 sc1" ::"v"(byte_offset), "v"(value), "s"(base) : "memory");
}

struct PackedArgs {
  // the wavefronts of the tiles read their own copy of the parameters: a value both kinds of
  // workgroup load from one place is loaded on entry, for all of them, before the first branch
  apc_params p;
  double *row_min_out;
  int32_t *row_arg_out;
  const double *pt_values;
  // the tensor table: a tile whose producer specs name several tensors reads it entry by entry
  const int32_t *rank, *itemsize;
  const int64_t *shape, *stride;
  double inv_rescale;  // 1.0 / params.rescale
  // every mesh size a power of two (term_layout): log2 of the sizes and of their product; else exponents = 0
  int32_t exponents, lg_total, lg[APC_MAX_MESH];
};

template <int M, bool POW2>
__device__ __forceinline__ void packed_tile(const apc_packed_tile *T, double *cost_out, const PackedArgs &a) {
  const apc_params &p = a.p;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
  // ---- the one round of loads: nothing here depends on another load ---------------------------
  const i32x16 h = uniform_load(reinterpret_cast<const i32x16 *>(T));
  const i64x8 t_shape = uniform_load(reinterpret_cast<const i64x8 *>(T->tensor_shape));
  const i64x8 t_stride = uniform_load(reinterpret_cast<const i64x8 *>(T->tensor_stride));
  TileCopies copies;
  copies.entry0 = T->dup_entry_begin[lane & (APC_PACKED_MAX_DUPS - 1)];
  copies.row0 = T->dup_row_begin[lane & (APC_PACKED_MAX_DUPS - 1)];
  copies.row_out = 0;
  const uint32_t col_code = T->col_codes[lane], row_code = T->row_codes[lane];
  const int col_tensor = T->col_tensor[lane], row_tensor = T->row_tensor[lane];
  const int64_t row_flops = T->row_flops[lane], row_rw = T->row_rw_bytes[lane];
  const int row_meta = T->row_meta[lane];
  // (lane j holds the throughput of dtype code j & 7: fetched by the lanes that need it, below)
  const double gf_of_lane = a.p.gpu_flops[lane & (APC_MAX_DTYPES - 1)], inv_gf_of_lane = a.p.inv_gpu_flops[lane & (APC_MAX_DTYPES - 1)];
  // (kernel arguments the wavefront needs first or in its store loops, under the same wait)
  fetch_arguments_now(h[0], t_shape[0], t_stride[0], a.row_min_out, a.row_arg_out, p.hbm_bw, p.inv_hbm_bw, p.rw_eff, p.inv_rw_eff,
                      p.launch_floor, p.compute_eff, p.inv_compute_eff, a.inv_rescale, p.rescale, p.a2a_scale, p.base_latency);
  const int rows = h[0], cols = h[1], flags = h[2], dup_count = h[3], t0 = h[4];
  if ((unsigned)rows > (unsigned)APC_TILE_MAX_ROWS || (unsigned)(cols - 1) >= (unsigned)APC_TILE_MAX_COLS ||
      (unsigned)dup_count > (unsigned)APC_PACKED_MAX_DUPS)
    return;  // a record the host validator would have rejected
  const int64_t entry_begin = ((int64_t)h[9] << 32) | (uint32_t)h[8], row_begin = ((int64_t)h[11] << 32) | (uint32_t)h[10];
  const int64_t pt_begin = ((int64_t)h[13] << 32) | (uint32_t)h[12];
  const uint32_t magic = (65536u + (uint32_t)cols - 1u) / (uint32_t)cols;  // x / cols = (x magic) >> 16 for x <= 64
  const int rows_per_pass = (int)((64u * magic) >> 16);
  if (wave * rows_per_pass >= rows) return;  // a wavefront without rows (a tile of fewer rows than the workgroup walks at once)
  // ---- per wavefront: the tensor's bytes, the rows' compute costs -------------------------------
  int64_t nbytes;
  bool contiguous;
  tensor_bytes_and_contiguity_of(h[5], h[6], t_shape, t_stride, nbytes, contiguous);
  const double fbytes = (double)nbytes;
  const int dt = (int)(int8_t)(row_meta & 0xFF);
  const bool known_dtype = dt >= 0 && dt < APC_MAX_DTYPES;
  const double gf = from_lane(gf_of_lane, dt & (APC_MAX_DTYPES - 1)), inv_gf = from_lane(inv_gf_of_lane, dt & (APC_MAX_DTYPES - 1));
  const double cpa = compute_cost_through_reciprocals(p, ((row_meta >> 8) & 0xFF) != 0, row_rw, row_flops, known_dtype ? gf : 0.0,
                                                      known_dtype ? inv_gf : 0.0) /
                     (double)(row_meta >> 16);  // (lanes past the tile's rows: never read)
  settle(copies);
  FlatConstants<M> k;
  constexpr bool pow2 = POW2;
  Pow2Constants<M> k2;
  if constexpr (!POW2) k = flat_constants<M>(p);
  if constexpr (POW2) {  // the chains of TermArrayConstants arrays 2 (read+write) and 4 + 3 d (one-hop ring of dim d)
    k2.R = div_by(div_by(fbytes, p.hbm_bw, p.inv_hbm_bw) * 1e6, p.rw_eff, p.inv_rw_eff);
    k2.rw_shift = 1 - a.lg_total;
    k2.floor = p.launch_floor;
#pragma unroll
    for (int i = 0; i < M; ++i) {
      const double hops1 = (double)(p.mesh_size[i] - 1), hops2 = (double)(2 * (p.mesh_size[i] - 1));
      k2.B[i] = div_by(fbytes * hops1, p.bw[i], p.inv_bw[i]) * 1e6;
      k2.lat1[i] = p.base_latency + hops1 * p.lat[i];
      k2.lat2[i] = p.base_latency + hops2 * p.lat[i];
      k2.lg[i] = a.lg[i];
      k2.shift[i] = -a.lg_total - 30 - a.lg[i];
    }
  }
  // ---- whole rows: cols lanes per row, 64 / cols rows per pass, wavefront w the passes w, w + waves, ...
  const int r_local = (int)(((uint32_t)lane * magic) >> 16), c = lane - r_local * cols;
  const bool in_pass = r_local < rows_per_pass;
  // (for the stores of the row minima: lane -> (row of the pass, copy))
  const uint32_t magic_rows = (65536u + (uint32_t)rows_per_pass - 1u) / (uint32_t)rows_per_pass;
  const int copies_per_store = (int)((64u * magic_rows) >> 16);
  const int copy_slot = (int)(((uint32_t)lane * magic_rows) >> 16), q = lane - copy_slot * rows_per_pass;
  const int q_first_lane = q * cols;
  const bool rescale = (flags & APC_EDGE_GRAD_RESCALE) != 0, no_producer = (flags & APC_EDGE_NO_PRODUCER) != 0;
  const bool entry_by_entry = (flags & APC_PACKED_MIXED) != 0 || no_producer || t0 < 0;
  double *const cost_base = cost_out + entry_begin;
  for (int row0 = wave * rows_per_pass; row0 < rows; row0 += waves * rows_per_pass) {
    const int r = row0 + r_local;
    const bool active = in_pass && r < rows;
    const uint32_t src = (uint32_t)from_lane((int)col_code, c), tgt = (uint32_t)from_lane((int)row_code, r);
    const double row_cpa = from_lane(cpa, r);
    const uint32_t local = (uint32_t)(r * cols + c);
    double comm = 0.0;
    int trans = 0;
    if (!entry_by_entry) {
      const bool flip = M == 2 && src == 0x4040u && ((tgt >> 6) & 3u) == 2u && ((tgt >> 14) & 3u) == 2u;
      const bool some_flip = M == 2 && __ballot(flip && active) != 0;  // (Partial, Partial) -> all Shard walks dim 1 first (:146-151)
      if constexpr (pow2) {
        int j = a.lg_total;  // bytes / num_shards = bytes x 2^(j - L): exact on such a mesh
#pragma unroll
        for (int i = 0; i < M; ++i) j -= ((src >> (8 * i + 6)) & 3u) == 2u ? k2.lg[i] : 0;
        comm = contiguous ? entry_cost_pow2<M, 0, true>(src, tgt, j, p.a2a_scale, k2) : entry_cost_pow2<M, 0, false>(src, tgt, j, p.a2a_scale, k2);
        if (some_flip) {
          const double other = contiguous ? entry_cost_pow2<M, 1, true>(src, tgt, j, p.a2a_scale, k2)
                                          : entry_cost_pow2<M, 1, false>(src, tgt, j, p.a2a_scale, k2);
          comm = flip ? other : comm;
        }
      } else {
        double shards = 1.0;  // exact: a product of mesh sizes (torch _dtensor_spec.py:555-561)
#pragma unroll
        for (int i = 0; i < M; ++i) shards *= ((src >> (8 * i + 6)) & 3u) == 2u ? (double)p.mesh_size[i] : 1.0;
        const double gb = fbytes / shards * 0x1p-30;  // / 1024 / 1024 / 1024 (:66-68)
        comm = contiguous ? entry_cost_flat<M, 0, true>(src, tgt, gb, p, k) : entry_cost_flat<M, 0, false>(src, tgt, gb, p, k);
        if (some_flip) {
          const double other = contiguous ? entry_cost_flat<M, 1, true>(src, tgt, gb, p, k)
                                          : entry_cost_flat<M, 1, false>(src, tgt, gb, p, k);
          comm = flip ? other : comm;
        }
      }
      trans = src != tgt ? p.transition_scale : 0;  // optimize_sharding.py:345-351
      // :358-359; the quotient through the reciprocal is the division's (div_by), +inf stays +inf
      if (rescale) comm = comm < __builtin_inf() ? div_by(comm, p.rescale, a.inv_rescale) : comm;
    } else {
      // pass-through edges and tiles whose specs are not all DTensorSpecs on one tensor: the
      // rule-provided value, or the direct evaluation on the entry's own tensor
      const int sten = from_lane(col_tensor, c), tten = from_lane(row_tensor, r);
      if (active) {
        if (no_producer || sten < 0 || tten < 0) {
          comm = a.pt_values[pt_begin + local];
        } else {
          trans = src != tgt ? p.transition_scale : 0;
          int64_t shards = 1;
#pragma unroll
          for (int i = 0; i < M; ++i)
            if (kind_of((src >> (8 * i)) & 0xFF) == 2) shards *= p.mesh_size[i];
          int64_t sten_bytes;
          bool sten_contiguous;
          tensor_bytes_and_contiguity(a.rank[sten], a.itemsize[sten], a.shape + (int64_t)sten * APC_MAX_RANK,
                                      a.stride + (int64_t)sten * APC_MAX_RANK, sten_bytes, sten_contiguous);
          const double gb = (double)sten_bytes / (double)shards / 1024 / 1024 / 1024;
          comm = entry_cost<M>(src, tgt, gb, sten_contiguous, p);
        }
        if (rescale) comm = comm / p.rescale;
      }
    }
    const double total = comm + row_cpa + (double)trans;  // optimize_sharding.py:368-372
    // ---- the entry, to the tile's edge and to every identical edge ----------------------------------
    const uint32_t off8 = local * 8u;
    if (active) store_at(cost_base, off8, total);
    for (int d = 0; d < dup_count; ++d) {  // per copy: the offset out of its lane, scalar address arithmetic, the store
      double *const base = cost_out + value_of_lane(copies.entry0, d);
      if (active) store_at(base, off8, total);
    }
    // ---- the rows' minima ----------------------------------------------------------------------------
    double m;
    int mc;
    row_min_in_wave(active, total, c, cols, lane, m, mc);
    // A row's minimum sits in the row's first lane.  Stored to all copies at once: lane (q, copy) =
    // (lane mod rows per pass, lane / rows per pass) fetches row q's result and writes it to its
    // copy (copy 0 = the tile's own edge), 64 / rows-per-pass copies per store instruction.
    const double m_q = from_lane(m, q_first_lane);
    const int mc_q = from_lane(mc, q_first_lane);
    const bool row_live = row0 + q < rows;
    for (int copy0 = 0; copy0 <= dup_count; copy0 += copies_per_store) {
      const int copy = copy0 + copy_slot;
      const int64_t first_row = from_lane_i64(copies.row0, copy - 1);  // (every lane takes part)
      if (row_live && copy_slot < copies_per_store && copy <= dup_count) {
        const int64_t out = (copy == 0 ? row_begin : first_row) + row0 + q;
        // (plain stores: written through, these 8- and 4-byte pieces cost whole sectors of HBM
        // writes, 21.0 instead of 19.2 MB per launch, for 0.15 us)
        a.row_min_out[out] = m_q;
        a.row_arg_out[out] = mc_q;
      }
    }
  }
}

template <int M, bool POW2>
__global__ __launch_bounds__(kBlock) void build_tables_packed_kernel(const apc_packed_tile *tiles, int n_tiles, int xcd_shift,
                                                                     int64_t tile_blocks, double *cost_out, PackedArgs a,
                                                                     apc_params p, TensorTableArgs t, ComputeCostArgs c,
                                                                     int64_t tensor_blocks) {
  const int64_t b = blockIdx.x;
  if (b < tile_blocks) {
    const int64_t per = tile_blocks >> xcd_shift;
    const int64_t tile_id = (b & ((1 << xcd_shift) - 1)) * per + (b >> xcd_shift);
    if (tile_id >= n_tiles) return;
    packed_tile<M, POW2>(tiles + tile_id, cost_out, a);
    return;
  }
  const int64_t tb = b - tile_blocks;
  if (tb < tensor_blocks) tensor_tables_block<kBlock, true>(tb, t);
  else compute_costs_block<kBlock, true>(tb - tensor_blocks, p, c);
}

// ------------------------------------------------------------------------------------------
// a14: segmented min + first argmin.  G consecutive lanes share one segment (G = 4 .. 64,
// chosen by the host from the mean segment length), so short segments do not leave most of
// a wavefront idle.
// ------------------------------------------------------------------------------------------
// Which segments to reduce and where else each result goes (SELECTED instantiation): segment
// selected[i] is reduced and its result stored to itself and to copy_segments[copy_ptr[i] ..
// copy_ptr[i + 1]), segments the caller knows to hold the same values.
struct SegmentCopies {
  const int64_t *selected;
  const int64_t *copy_ptr;
  const int64_t *copy_segments;
};

template <int G, bool SELECTED>
__global__ __launch_bounds__(kBlock) void segmented_min_kernel(const double *__restrict__ values,
                                                               const int64_t *__restrict__ seg_ptr,
                                                               int64_t n_seg, double *__restrict__ mins,
                                                               int32_t *__restrict__ args, SegmentCopies copies) {
  const int sub = threadIdx.x & (G - 1);
  const int64_t slot = (int64_t)blockIdx.x * (kBlock / G) + (threadIdx.x / G);
  const bool live = slot < n_seg;  // (n_seg counts the selected segments when SELECTED)
  const int64_t seg = SELECTED ? (live ? copies.selected[slot] : 0) : slot;
  const int64_t lo = live ? seg_ptr[seg] : 0, hi = live ? seg_ptr[seg + 1] : 0;
  double best = INFINITY;
  int64_t arg = INT64_MAX;  // absolute index; INT64_MAX = none seen
  auto take = [&](double v, int64_t j) {
    if (arg == INT64_MAX || v < best) {
      best = v;
      arg = j;
    }
  };
  // A lane reads pairs of consecutive values (one 16-byte load; segments start at any 8-byte
  // offset, which global loads allow), four such loads in flight (two on a short remainder), taken in index order (first
  // minimum wins); the G lanes of a group sweep 2 G consecutive values per load.
  struct __attribute__((packed, aligned(8))) Pair {
    double x, y;
  };
  int64_t j = lo + 2 * sub;
  for (; j + 6 * G + 1 < hi; j += 8 * G) {
    const Pair a = *reinterpret_cast<const Pair *>(values + j);
    const Pair b = *reinterpret_cast<const Pair *>(values + j + 2 * G);
    const Pair c = *reinterpret_cast<const Pair *>(values + j + 4 * G);
    const Pair d = *reinterpret_cast<const Pair *>(values + j + 6 * G);
    take(a.x, j);
    take(a.y, j + 1);
    take(b.x, j + 2 * G);
    take(b.y, j + 2 * G + 1);
    take(c.x, j + 4 * G);
    take(c.y, j + 4 * G + 1);
    take(d.x, j + 6 * G);
    take(d.y, j + 6 * G + 1);
  }
  for (; j + 2 * G + 1 < hi; j += 4 * G) {
    const Pair a = *reinterpret_cast<const Pair *>(values + j);
    const Pair b = *reinterpret_cast<const Pair *>(values + j + 2 * G);
    take(a.x, j);
    take(a.y, j + 1);
    take(b.x, j + 2 * G);
    take(b.y, j + 2 * G + 1);
  }
  for (; j + 1 < hi; j += 2 * G) {
    const Pair a = *reinterpret_cast<const Pair *>(values + j);
    take(a.x, j);
    take(a.y, j + 1);
  }
  if (j < hi) take(values[j], j);
  // lexicographic (value, index) min inside the group; lanes that saw nothing lose
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) {
    const double ob = __shfl_xor(best, off, 64);
    const int64_t oa = __shfl_xor(arg, off, 64);
    const bool take = (oa != INT64_MAX) && (arg == INT64_MAX || ob < best || (ob == best && oa < arg));
    if (take) {
      best = ob;
      arg = oa;
    }
  }
  if (live && sub == 0) {
    const int32_t rel = arg == INT64_MAX ? -1 : (int32_t)(arg - lo);
    mins[seg] = best;
    args[seg] = rel;
    if (SELECTED) {
      for (int64_t k = copies.copy_ptr[slot], end = copies.copy_ptr[slot + 1]; k < end; ++k) {
        const int64_t to = copies.copy_segments[k];
        mins[to] = best;
        args[to] = rel;
      }
    }
  }
}

// 8 XCDs; APC_XCD_SHIFT=0 restores the plain work order (tuning)
int xcd_shift() {
  static const int shift = [] {
    const char *env = getenv("APC_XCD_SHIFT");
    const int v = env ? atoi(env) : 3;
    return v < 0 ? 0 : v > 5 ? 5 : v;
  }();
  return shift;
}

// ------------------------------------------------------------------------------------------
// a14: optimistic cost of every (node, strategy): the sum over the node's edges of that
// consumer strategy's row minimum.  A plan pays, on every edge, at least the minimum of the
// row of the strategy its consumer takes, so min over a node's strategies, summed over the
// nodes, bounds the ILP objective from below, and the per-node argmin is the greedy choice a
// warm start begins from.  One thread per strategy; a node's edges are added in the order of
// edges_by_node (deterministic sum).
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void strategy_bounds_kernel(int64_t n_strategies,
                                                                 const int32_t *__restrict__ strat_node,
                                                                 const int64_t *__restrict__ node_strat_begin,
                                                                 const int64_t *__restrict__ node_edge_begin,
                                                                 const int32_t *__restrict__ edges_by_node,
                                                                 const int64_t *__restrict__ edge_row_begin,
                                                                 const double *__restrict__ row_min,
                                                                 double *__restrict__ bound) {
  const int64_t s = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (s >= n_strategies) return;
  const int n = strat_node[s];
  const int64_t k = s - node_strat_begin[n];
  double sum = 0.0;
  for (int64_t j = node_edge_begin[n]; j < node_edge_begin[n + 1]; ++j) sum += row_min[edge_row_begin[edges_by_node[j]] + k];
  bound[s] = sum;
}

// ------------------------------------------------------------------------------------------
// The ILP objective, summed on the device.  Entries of linked nodes share an ILP variable
// (optimize_sharding.py:211-231) and the objective coefficient of a variable is the sum of the
// costs of its entries, added one by one in entry order starting from 0
// (optimize_sharding.py:650-655: opt_target[va] += cost over ds.values()); a cost that is not
// finite counts as inf_replacement and forces the variable to 0 (:522-536).  Variables are
// numbered group by group: a group is a set of edges with matrices of the same shape whose
// entries share variables position by position (one edge when nothing is linked); variable
// group_var_begin[g] + k sums entry k of every member edge, members in ascending entry order.
// One workgroup per group (gridDim.y workgroups share a group, each taking every gridDim.y-th
// run of kBlock variables): which group a variable belongs to is never searched for, what a
// group needs (its first variable, its size, its member list) is the same for every lane and is
// fetched once, and neighbouring lanes read neighbouring entries of each member.  The member
// list goes through LDS, so the loads a thread has in flight are costs and nothing else:
// kObjectiveMembersAhead members of one variable, or kObjectiveAhead variables of a group with a
// single member; the additions of a variable stay in member order.
// ------------------------------------------------------------------------------------------
constexpr int kObjectiveAhead = 8;          // variables of a single-member group a thread has in flight
constexpr int kObjectiveMembersAhead = 8;   // members of a variable a thread has in flight

__global__ __launch_bounds__(kBlock) void cost_objective_kernel(const int64_t *__restrict__ group_var_begin,
                                                                const int64_t *__restrict__ group_member_begin,
                                                                const int64_t *__restrict__ member_entry_begin,
                                                                const double *__restrict__ cost, double inf_replacement,
                                                                double *__restrict__ objective,
                                                                uint8_t *__restrict__ forced_zero) {
  __shared__ int64_t s_first_entry[kBlock];
  const int tid = threadIdx.x;
  const int64_t g = blockIdx.x;
  const int64_t var0 = uniform_load(group_var_begin + g), size = uniform_load(group_var_begin + g + 1) - var0;
  const int64_t member0 = uniform_load(group_member_begin + g), n_members = uniform_load(group_member_begin + g + 1) - member0;
  const int64_t begin = (int64_t)blockIdx.y * kBlock, stride = (int64_t)gridDim.y * kBlock;
  if (begin >= size) return;
  const double inf = __builtin_inf();
  auto put = [&](int64_t k, double sum, bool forced) {
    objective[var0 + k] = sum;
    forced_zero[var0 + k] = forced ? 1 : 0;
  };
  if (n_members == 1) {  // nothing is linked: one entry per variable, kObjectiveAhead variables of a thread in flight
    const int64_t first = uniform_load(member_entry_begin + member0);
    for (int64_t base = begin; base < size; base += kObjectiveAhead * stride) {
      double c[kObjectiveAhead];
#pragma unroll
      for (int i = 0; i < kObjectiveAhead; ++i) {
        const int64_t k = base + i * stride + tid;
        c[i] = k < size ? cost[first + k] : 0.0;
      }
#pragma unroll
      for (int i = 0; i < kObjectiveAhead; ++i) {
        const int64_t k = base + i * stride + tid;
        if (k >= size) continue;
        const bool bad = !(__builtin_fabs(c[i]) < inf);  // inf or nan: math.isfinite is false
        put(k, 0.0 + (bad ? inf_replacement : c[i]), bad);
      }
    }
    return;
  }
  for (int64_t base = begin; base < size; base += stride) {  // (the same trips for every thread of the workgroup)
    const int64_t k = base + tid;
    const bool active = k < size;
    double sum = 0.0;
    bool forced = false;
    for (int64_t chunk = 0; chunk < n_members; chunk += kBlock) {
      const int in_chunk = (int)(n_members - chunk < kBlock ? n_members - chunk : kBlock);
      if (n_members > kBlock || base == begin) {  // (a list of at most kBlock members is staged once)
        __syncthreads();
        if (tid < in_chunk) s_first_entry[tid] = member_entry_begin[member0 + chunk + tid];
        __syncthreads();
      }
      for (int at = 0; at < in_chunk; at += kObjectiveMembersAhead) {
        double c[kObjectiveMembersAhead];
#pragma unroll
        for (int i = 0; i < kObjectiveMembersAhead; ++i) c[i] = active && at + i < in_chunk ? cost[s_first_entry[at + i] + k] : 0.0;
#pragma unroll
        for (int i = 0; i < kObjectiveMembersAhead; ++i) {
          if (at + i < in_chunk) {
            const bool bad = !(__builtin_fabs(c[i]) < inf);
            forced |= bad;
            sum += bad ? inf_replacement : c[i];
          }
        }
      }
    }
    if (active) put(k, sum, forced);
  }
}

// ------------------------------------------------------------------------------------------
// a14 put to work: min-sum diffusion over the planning program's labelling form.  A class
// (linked nodes) has a unary cost vector; an edge between two classes has a cost matrix
// (rows = labels of class edge_i, columns = labels of class edge_j, +inf = forbidden pair).
// A node update takes, for every incident matrix, the minima of the rows (or columns) the
// class labels out of the matrix and into the class, then hands their sum back to the
// incident matrices in equal shares.  Every update leaves the cost of every labelling unchanged
// and never lowers  sum_classes min unary + sum_edges min matrix,  a lower bound of the
// program's optimum; min-marginals read off the reparametrised costs prune the program.
// One workgroup per class of one colour (classes of a colour share no edge, so they update
// together); the sweep is the sequence of colours.  Arithmetic in a fixed order (the sum over
// incident edges in incidence order, one division, one subtraction and one addition per
// matrix element): the same bits as the CPU restatement.
// ------------------------------------------------------------------------------------------
constexpr int kDiffusionMaxLabels = 2048;

struct DiffusionArgs {
  const int32_t *nodes;  // the classes of this launch
  const int64_t *label_begin, *inc_begin;
  const int32_t *inc_edge;
  const uint8_t *inc_side;
  const int64_t *edge_begin;
  const int32_t *edge_i, *edge_j;
  double *theta, *unary;
};

__device__ __forceinline__ double wave_min(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const double o = __shfl_xor(v, off, 64);
    v = o < v ? o : v;
  }
  return v;
}

// The update of one class against the matrices where they lie: one pass over every incident
// matrix for the minima, one for the shares, the matrices taken one after the other.  The path
// of a class whose matrices do not fit the staging arrays of the kernel below.
__device__ void diffusion_update_in_memory(const DiffusionArgs &a, double *s_tot, int64_t l0, int n_labels, int64_t t0,
                                           int64_t t1) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int kWaves = kBlock / 64;
  const double inf = __builtin_inf();
  for (int x = tid; x < n_labels; x += kBlock) s_tot[x] = a.unary[l0 + x];
  __syncthreads();
  // pull: the minimum of every row / column of the class out of each incident matrix
  for (int64_t t = t0; t < t1; ++t) {
    const int k = a.inc_edge[t];
    double *m = a.theta + a.edge_begin[k];
    const int ej = a.edge_j[k];
    const int nj = (int)(a.label_begin[ej + 1] - a.label_begin[ej]);
    if (a.inc_side[t] == 0) {  // the class labels the rows: one wavefront per row
      for (int x = wave; x < n_labels; x += kWaves) {
        double *row = m + (int64_t)x * nj;
        double d = inf;
        for (int y = lane; y < nj; y += 64) {
          const double v = row[y];
          d = v < d ? v : d;
        }
        d = wave_min(d);
        if (d < inf)
          for (int y = lane; y < nj; y += 64) row[y] -= d;
        if (lane == 0) s_tot[x] += d;
      }
    } else {  // the class labels the columns: one thread per column
      const int ei = a.edge_i[k];
      const int ni = (int)(a.label_begin[ei + 1] - a.label_begin[ei]);
      for (int y = tid; y < n_labels; y += kBlock) {
        double d = inf;
        for (int x = 0; x < ni; ++x) {
          const double v = m[(int64_t)x * n_labels + y];
          d = v < d ? v : d;
        }
        if (d < inf)
          for (int x = 0; x < ni; ++x) m[(int64_t)x * n_labels + y] -= d;
        s_tot[y] += d;
      }
    }
    __syncthreads();
  }
  // share: an equal part of the total for every incident matrix; a label without a finite
  // pair on some edge can never be taken: +inf everywhere
  const double degree = (double)(t1 - t0);
  for (int x = tid; x < n_labels; x += kBlock) {
    const double tot = s_tot[x];
    const bool finite = tot < inf;
    s_tot[x] = finite ? tot / degree : inf;
    a.unary[l0 + x] = finite ? 0.0 : inf;
  }
  __syncthreads();
  for (int64_t t = t0; t < t1; ++t) {
    const int k = a.inc_edge[t];
    double *m = a.theta + a.edge_begin[k];
    if (a.inc_side[t] == 0) {
      const int ej = a.edge_j[k];
      const int nj = (int)(a.label_begin[ej + 1] - a.label_begin[ej]);
      for (int x = wave; x < n_labels; x += kWaves) {
        double *row = m + (int64_t)x * nj;
        const double share = s_tot[x];
        for (int y = lane; y < nj; y += 64) row[y] = share < inf ? row[y] + share : inf;
      }
    } else {
      const int ei = a.edge_i[k];
      const int ni = (int)(a.label_begin[ei + 1] - a.label_begin[ei]);
      for (int y = tid; y < n_labels; y += kBlock) {
        const double share = s_tot[y];
        for (int x = 0; x < ni; ++x) {
          double *p = m + (int64_t)x * n_labels + y;
          *p = share < inf ? *p + share : inf;
        }
      }
    }
  }
}

// One workgroup per class.  A planning program's classes are small (tens of labels, a handful
// of incident matrices of a few hundred elements), so an update is a chain of dependent memory
// round trips and nothing else; the kernel keeps that chain as short as the data allows: the
// incidence list in one round, every incident matrix into LDS in one round of independent
// loads (the elements of all matrices numbered through, a thread finds the matrix of an
// element by bisecting the staged offsets), minima, totals and shares out of LDS, and every
// element stored once.  Element by element the arithmetic is that of the path above, in the
// same order: (v - d) where the row has a finite minimum, then + share or +inf.
// (48 KB of LDS in all, so that a compute unit holds three classes: the largest class of the planning programs
// measured has 3 856 elements and 256 pairs)
constexpr int kDiffusionStagedElements = 4096;  // doubles of LDS for the incident matrices of a class
constexpr int kDiffusionStagedDegree = 64;      // incident matrices of a class
constexpr int kDiffusionStagedPairs = 1024;     // (incident matrix, label) pairs of a class
static_assert(kDiffusionStagedElements >= kDiffusionMaxLabels, "the update in memory keeps its totals where the matrices are staged");

__global__ __launch_bounds__(kBlock) void diffusion_node_update_kernel(DiffusionArgs a) {
  __shared__ double s_m[kDiffusionStagedElements];
  __shared__ double s_d[kDiffusionStagedPairs];
  __shared__ double s_share[kDiffusionStagedPairs];  // (a staged class has at most kDiffusionStagedPairs labels)
  double *s_tot = s_m;                               // the update in memory stages no matrix: its totals lie there
  __shared__ int64_t s_base[kDiffusionStagedDegree];
  __shared__ int s_off[kDiffusionStagedDegree + 1];
  __shared__ int s_other[kDiffusionStagedDegree];
  __shared__ int s_side[kDiffusionStagedDegree];
  const int c = a.nodes[blockIdx.x];
  const int64_t l0 = a.label_begin[c];
  const int n_labels = (int)(a.label_begin[c + 1] - l0);
  const int64_t t0 = a.inc_begin[c], t1 = a.inc_begin[c + 1];
  if (t1 == t0) return;
  if (n_labels > kDiffusionMaxLabels || n_labels < 0) return;  // (the host entry point refuses such a class)
  const int tid = threadIdx.x;
  const int64_t degree64 = t1 - t0;
  if (degree64 > kDiffusionStagedDegree || degree64 * n_labels > kDiffusionStagedPairs) {
    diffusion_update_in_memory(a, s_tot, l0, n_labels, t0, t1);
    return;
  }
  const int degree = (int)degree64;
  const double inf = __builtin_inf();
  // the incidence list: edge, side, where its matrix starts and how many labels the class at
  // its other end has; the unary vector rides along in the same round
  double unary = 0.0;
  if (tid < n_labels) unary = a.unary[l0 + tid];  // (n_labels <= kStagedPairs / degree; labels beyond kBlock below)
  int size = 0;
  if (tid < degree) {
    const int k = a.inc_edge[t0 + tid];
    const int side = a.inc_side[t0 + tid];
    const int other_class = side == 0 ? a.edge_j[k] : a.edge_i[k];
    const int other = (int)(a.label_begin[other_class + 1] - a.label_begin[other_class]);
    s_base[tid] = a.edge_begin[k];
    s_other[tid] = other;
    s_side[tid] = side;
    size = other * n_labels;
  }
  if (tid < 64) {  // degree <= 64: the offsets of the matrices in LDS, a scan within the first wavefront
    int incl = size;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int o = __shfl_up(incl, off, 64);
      if (tid >= off) incl += o;
    }
    if (tid < degree) s_off[tid + 1] = incl;
    if (tid == 0) s_off[0] = 0;
  }
  __syncthreads();
  const int total = s_off[degree];
  if (total > kDiffusionStagedElements || total < 0) {  // uniform: every thread reads the same word
    diffusion_update_in_memory(a, s_tot, l0, n_labels, t0, t1);
    return;
  }
  auto matrix_of = [&](int g) {  // the incident matrix that holds staged element g: the last t with s_off[t] <= g
    int lo = 0, hi = degree - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (s_off[mid] <= g) lo = mid; else hi = mid - 1;
    }
    return lo;
  };
  constexpr int kAhead = 4;  // loads a thread issues before it waits for the first
  for (int base = 0; base < total; base += kAhead * kBlock) {
    double v[kAhead];
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int g = base + u * kBlock + tid;
      v[u] = 0.0;
      if (g < total) {
        const int t = matrix_of(g);
        v[u] = a.theta[s_base[t] + (g - s_off[t])];
      }
    }
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int g = base + u * kBlock + tid;
      if (g < total) s_m[g] = v[u];
    }
  }
  __syncthreads();
  // pull: one thread per (incident matrix, label of the class)
  const int pairs = degree * n_labels;
  for (int q = tid; q < pairs; q += kBlock) {
    const int t = q / n_labels, x = q - t * n_labels;
    const int other = s_other[t];
    // rows of the class are contiguous runs of `other` elements; its columns are strided by n_labels
    const int first = s_off[t] + (s_side[t] == 0 ? x * other : x);
    const int step = s_side[t] == 0 ? 1 : n_labels;
    double d = inf;
    for (int y = 0; y < other; ++y) {
      const double v = s_m[first + y * step];
      d = v < d ? v : d;
    }
    if (d < inf)
      for (int y = 0; y < other; ++y) s_m[first + y * step] -= d;
    s_d[q] = d;
  }
  __syncthreads();
  // totals in incidence order, one division: the share every incident matrix gets back
  for (int x = tid; x < n_labels; x += kBlock) {
    double tot = x == tid && tid < n_labels ? unary : a.unary[l0 + x];
    for (int t = 0; t < degree; ++t) tot += s_d[t * n_labels + x];
    const bool finite = tot < inf;
    s_share[x] = finite ? tot / (double)degree : inf;
    a.unary[l0 + x] = finite ? 0.0 : inf;
  }
  __syncthreads();
  for (int g = tid; g < total; g += kBlock) {
    const int t = matrix_of(g);
    const int e = g - s_off[t];
    const int x = s_side[t] == 0 ? e / s_other[t] : e % n_labels;
    const double share = s_share[x];
    a.theta[s_base[t] + e] = share < inf ? s_m[g] + share : inf;
  }
}

inline unsigned blocks_for(int64_t n, int per_block) { return (unsigned)((n + per_block - 1) / per_block); }

template <int G>
void launch_segmented_min(const double *values, const int64_t *seg_ptr, int64_t n_seg, double *mins, int32_t *args,
                          const SegmentCopies *copies, hipStream_t stream) {
  if (copies)
    hipLaunchKernelGGL((segmented_min_kernel<G, true>), dim3(blocks_for(n_seg, kBlock / G)), dim3(kBlock), 0, stream,
                       values, seg_ptr, n_seg, mins, args, *copies);
  else
    hipLaunchKernelGGL((segmented_min_kernel<G, false>), dim3(blocks_for(n_seg, kBlock / G)), dim3(kBlock), 0, stream,
                       values, seg_ptr, n_seg, mins, args, SegmentCopies{nullptr, nullptr, nullptr});
}

int check_width(int width) {
  if (width < 2 || width > APC_MAX_RANK || (width & 1))
    return fail(-1, "shape_width %d must be even and in [2, %d]", width, APC_MAX_RANK);
  return 0;
}

int check_params(const apc_params *p) {
  if (!p) return fail(-1, "params is NULL");
  if (p->mesh_ndim < 1 || p->mesh_ndim > APC_MAX_MESH)
    return fail(-1, "mesh_ndim %d outside [1, %d]", p->mesh_ndim, APC_MAX_MESH);
  for (int i = 0; i < p->mesh_ndim; ++i) {
    if (p->mesh_size[i] < 1) return fail(-1, "mesh_size[%d] = %d must be >= 1", i, p->mesh_size[i]);
    // the kernels divide through these reciprocals: they must be the correctly rounded ones
    if (p->inv_mesh[i] != 1.0 / (double)p->mesh_size[i] || p->inv_bw[i] != 1.0 / p->bw[i])
      return fail(-1, "inv_mesh[%d] / inv_bw[%d] are not 1.0 / mesh_size, 1.0 / bw", i, i);
  }
  if (p->inv_hbm_bw != 1.0 / p->hbm_bw || p->inv_rw_eff != 1.0 / p->rw_eff || p->inv_compute_eff != 1.0 / p->compute_eff)
    return fail(-1, "inv_hbm_bw / inv_rw_eff / inv_compute_eff are not 1.0 / hbm_bw, 1.0 / rw_eff, 1.0 / compute_eff");
  for (int i = 0; i < APC_MAX_DTYPES; ++i)
    if (p->inv_gpu_flops[i] != (p->gpu_flops[i] != 0.0 ? 1.0 / p->gpu_flops[i] : 0.0))
      return fail(-1, "inv_gpu_flops[%d] is not 1.0 / gpu_flops[%d] (0 for an unsupported dtype)", i, i);
  return 0;
}

}  // namespace

extern "C" {

int apc_version(void) { return APC_ABI_VERSION; }

const char *apc_last_error(void) { return g_err; }

int apc_validate_tables_host(const apc_params *params, int64_t n_tensors, const int32_t *tensor_rank,
                             int64_t n_specs, const uint32_t *spec_codes, const int32_t *spec_tensor,
                             int64_t n_edges, const int32_t *edge_src_begin, const int32_t *edge_n_src,
                             const int32_t *edge_tgt_begin, const int32_t *edge_n_tgt,
                             const int32_t *edge_flags, const int64_t *edge_pt_begin,
                             const int64_t *edge_entry_begin, const int32_t *edge_strat_begin, int64_t n_pt,
                             int64_t n_strategies, int64_t n_tiles, const apc_tile *tiles, int64_t n_dups,
                             const int64_t *dup_entry_begin) {
  if (int rc = check_params(params)) return rc;
  const int M = params->mesh_ndim;
  for (int64_t t = 0; t < n_tensors; ++t)
    if (tensor_rank[t] < 0 || tensor_rank[t] > APC_MAX_RANK)
      return fail(-2, "tensor %lld: rank %d outside [0, %d]", (long long)t, tensor_rank[t], APC_MAX_RANK);
  for (int64_t s = 0; s < n_specs; ++s) {
    const int t = spec_tensor[s];
    if (t < -1 || t >= n_tensors)
      return fail(-2, "spec %lld: tensor row %d out of range [-1, %lld)", (long long)s, t, (long long)n_tensors);
    if (M < 4 && (spec_codes[s] >> (8 * M)) != 0)
      return fail(-2, "spec %lld: placement bytes beyond mesh ndim %d are set (0x%08x)", (long long)s, M,
                  spec_codes[s]);
    for (int i = 0; i < M; ++i) {
      const uint32_t c = (spec_codes[s] >> (8 * i)) & 0xFF;
      if ((c >> 6) == 3) return fail(-2, "spec %lld: placement code 0x%02x has no meaning", (long long)s, c);
      if ((c >> 6) == 0 && c != 0) return fail(-2, "spec %lld: placement code 0x%02x has no meaning", (long long)s, c);
      if ((c >> 6) == 2 && t >= 0 && (int)(c & 0x0F) >= tensor_rank[t])
        return fail(-2, "spec %lld: Shard(%d) on a rank-%d tensor", (long long)s, (int)(c & 0x0F), tensor_rank[t]);
    }
  }
  int64_t expect = 0;
  for (int64_t e = 0; e < n_edges; ++e) {
    if (edge_entry_begin[e] != expect)
      return fail(-2, "edge %lld: entry_begin %lld, expected %lld (offsets must be the running sum of n_tgt*n_src)",
                  (long long)e, (long long)edge_entry_begin[e], (long long)expect);
    const int64_t ns = edge_n_src[e], nt = edge_n_tgt[e];
    if (ns < 0 || nt < 0) return fail(-2, "edge %lld: negative strategy count", (long long)e);
    if (ns > APC_MAX_STRATEGIES || nt > APC_MAX_STRATEGIES)
      return fail(-2, "edge %lld: %lld x %lld strategies, at most %d a side", (long long)e, (long long)nt,
                  (long long)ns, APC_MAX_STRATEGIES);
    if (edge_src_begin[e] < 0 || edge_src_begin[e] + ns > n_specs)
      return fail(-2, "edge %lld: producer spec range [%d, +%lld) outside the spec table", (long long)e,
                  edge_src_begin[e], (long long)ns);
    if (edge_tgt_begin[e] < 0 || edge_tgt_begin[e] + nt > n_specs)
      return fail(-2, "edge %lld: consumer spec range [%d, +%lld) outside the spec table", (long long)e,
                  edge_tgt_begin[e], (long long)nt);
    if (edge_strat_begin[e] < 0 || edge_strat_begin[e] + nt > n_strategies)
      return fail(-2, "edge %lld: strategy rows [%d, +%lld) outside the strategy table", (long long)e,
                  edge_strat_begin[e], (long long)nt);
    bool needs_pt = (edge_flags[e] & APC_EDGE_NO_PRODUCER) != 0;
    if (!needs_pt) {
      for (int64_t j = 0; j < ns && !needs_pt; ++j) needs_pt = spec_tensor[edge_src_begin[e] + j] < 0;
      for (int64_t j = 0; j < nt && !needs_pt; ++j) needs_pt = spec_tensor[edge_tgt_begin[e] + j] < 0;
    }
    if (needs_pt && (edge_pt_begin[e] < 0 || edge_pt_begin[e] + ns * nt > n_pt))
      return fail(-2, "edge %lld: pass-through values [%lld, +%lld) outside pt_values", (long long)e,
                  (long long)edge_pt_begin[e], (long long)(ns * nt));
    expect += ns * nt;
  }
  if (edge_entry_begin[n_edges] != expect)
    return fail(-2, "entry_begin[n_edges] = %lld, expected %lld", (long long)edge_entry_begin[n_edges],
                (long long)expect);
  for (int64_t t = 0; t < n_tiles; ++t) {
    const apc_tile &tl = tiles[t];
    const int e = tl.edge;
    const int row_count = tl.counts & 0xFFFF, col_count = tl.counts >> 16;
    if (e < 0 || e >= n_edges) return fail(-2, "tile %lld: edge %d out of range", (long long)t, e);
    if (row_count < 1 || row_count > APC_TILE_MAX_ROWS || tl.row_begin < 0 ||
        tl.row_begin + row_count > edge_n_tgt[e])
      return fail(-2, "tile %lld: rows [%d, +%d) outside edge %d (n_tgt %d, max %d per tile)", (long long)t,
                  tl.row_begin, row_count, e, edge_n_tgt[e], APC_TILE_MAX_ROWS);
    if (col_count < 1 || col_count > APC_TILE_MAX_COLS || tl.col_begin < 0 ||
        tl.col_begin + col_count > edge_n_src[e])
      return fail(-2, "tile %lld: cols [%d, +%d) outside edge %d (n_src %d, max %d per tile)", (long long)t,
                  tl.col_begin, col_count, e, edge_n_src[e], APC_TILE_MAX_COLS);
    if (tl.src_begin != edge_src_begin[e] || tl.n_src != edge_n_src[e] || tl.tgt_begin != edge_tgt_begin[e] ||
        tl.flags != edge_flags[e] || tl.strat_begin != edge_strat_begin[e] ||
        tl.entry_begin != edge_entry_begin[e] || tl.pt_begin != edge_pt_begin[e])
      return fail(-2, "tile %lld: record does not repeat the fields of edge %d", (long long)t, e);
    if (tl.tensor != spec_tensor[edge_src_begin[e] + tl.col_begin])
      return fail(-2, "tile %lld: tensor %d is not the tensor of its first producer spec", (long long)t, tl.tensor);
    if (tl.dup_count < 0 || tl.dup_count > APC_TILE_MAX_DUPS || tl.dup_begin < 0 ||
        (int64_t)tl.dup_begin + tl.dup_count > n_dups)
      return fail(-2, "tile %lld: duplicate list [%d, +%d) outside dup_entry_begin", (long long)t, tl.dup_begin,
                  tl.dup_count);
    for (int d = 0; d < tl.dup_count; ++d) {
      // the offset must be the start of another edge with the same matrix shape
      const int64_t off = dup_entry_begin[tl.dup_begin + d];
      int64_t lo = 0, hi = n_edges;  // first edge whose entry_begin >= off, then skip empty edges
      while (lo < hi) {
        const int64_t mid = (lo + hi) / 2;
        if (edge_entry_begin[mid] < off) lo = mid + 1; else hi = mid;
      }
      while (lo < n_edges && (int64_t)edge_n_src[lo] * edge_n_tgt[lo] == 0) ++lo;
      if (lo >= n_edges || edge_entry_begin[lo] != off || lo == e || edge_n_src[lo] != edge_n_src[e] ||
          edge_n_tgt[lo] != edge_n_tgt[e])
        return fail(-2, "tile %lld: duplicate offset %lld is not the start of an edge shaped like edge %d",
                    (long long)t, (long long)off, e);
    }
  }
  return 0;
}

int apc_tensor_tables(int64_t n, const int32_t *rank, const int32_t *itemsize, const int64_t *shape,
                      const int64_t *stride, int64_t *bytes, uint8_t *cont, void *stream) {
  if (n < 0) return fail(-1, "n_tensors < 0");
  if (n == 0) return 0;
  if (!rank || !itemsize || !shape || !stride || !bytes || !cont) return fail(-1, "apc_tensor_tables: NULL array");
  hipLaunchKernelGGL(tensor_tables_kernel, dim3(blocks_for(n, kBlock)), dim3(kBlock), 0, (hipStream_t)stream,
                     TensorTableArgs{n, rank, itemsize, shape, stride, bytes, cont});
  return check_launch("apc_tensor_tables");
}

int apc_spec_tables(const apc_params *params, int64_t n, const uint32_t *codes, const int32_t *tensor,
                    const int32_t *rank, const int32_t *itemsize, const int64_t *shape, const int64_t *stride,
                    int64_t *shards, int64_t *lshape, int64_t *lstride, int32_t shape_width, int64_t *lnumel,
                    int64_t *lbytes, void *stream) {
  if (int rc = check_params(params)) return rc;
  if (int rc = check_width(shape_width)) return rc;
  if (n < 0) return fail(-1, "n_specs < 0");
  if (n == 0) return 0;
  if (!codes || !tensor || !rank || !itemsize || !shape || !stride || !shards || !lshape || !lstride || !lnumel ||
      !lbytes)
    return fail(-1, "apc_spec_tables: NULL array");
  hipLaunchKernelGGL(spec_tables_kernel, dim3(blocks_for(n, kBlock)), dim3(kBlock), 0, (hipStream_t)stream, *params,
                     SpecTableArgs{n, codes, tensor, rank, itemsize, shape, stride, shards, lshape, lstride, lnumel,
                                   lbytes, shape_width});
  return check_launch("apc_spec_tables");
}

int apc_compute_costs(const apc_params *params, int64_t n, const int64_t *flops, const int64_t *rw_bytes,
                      const int8_t *dtype, const uint8_t *zero_cost, const int32_t *num_args, double *compute,
                      double *per_arg, int32_t *error_flag, void *stream) {
  if (int rc = check_params(params)) return rc;
  if (n < 0) return fail(-1, "n_strategies < 0");
  if (n == 0) return 0;
  if (!flops || !rw_bytes || !dtype || !zero_cost || !num_args) return fail(-1, "apc_compute_costs: NULL input");
  hipLaunchKernelGGL(compute_costs_kernel, dim3(blocks_for(n, kBlock)), dim3(kBlock), 0, (hipStream_t)stream,
                     *params,
                     ComputeCostArgs{n, flops, rw_bytes, dtype, zero_cost, num_args, compute, per_arg, error_flag});
  return check_launch("apc_compute_costs");
}

int apc_strategy_inputs(int64_t n_strategies, const int32_t *strat_node, int64_t n_nodes, const int64_t *node_strat_begin,
                        const int32_t *node_kind, const int8_t *node_dtype, const int64_t *node_const_bytes,
                        const int64_t *node_row_begin, const int32_t *byte_rows, const int32_t *node_flop_rows,
                        const int64_t *local_shape, int32_t shape_width, const int64_t *local_bytes, int64_t *flops,
                        int64_t *rw_bytes, int8_t *dtype_code, uint8_t *zero_cost, void *stream) {
  if (n_strategies < 0 || n_nodes < 0) return fail(-1, "apc_strategy_inputs: negative count");
  if (n_strategies == 0) return 0;
  if (int rc = check_width(shape_width)) return rc;
  if (!strat_node || !node_strat_begin || !node_kind || !node_dtype || !node_const_bytes || !node_row_begin ||
      !node_flop_rows || !local_shape || !local_bytes || !flops || !rw_bytes || !dtype_code || !zero_cost)
    return fail(-1, "apc_strategy_inputs: NULL array");
  hipLaunchKernelGGL(strategy_inputs_kernel, dim3(blocks_for(n_strategies, kBlock)), dim3(kBlock), 0, (hipStream_t)stream,
                     StrategyInputArgs{n_strategies, strat_node, node_strat_begin, node_kind, node_dtype, node_const_bytes,
                                       node_row_begin, byte_rows, node_flop_rows, local_shape, shape_width, local_bytes, flops,
                                       rw_bytes, dtype_code, zero_cost});
  return check_launch("apc_strategy_inputs");
}

int apc_input_tables(const apc_params *params, int64_t n_tensors, const int32_t *rank, const int32_t *itemsize,
                     const int64_t *shape, const int64_t *stride, int64_t *tensor_bytes, uint8_t *tensor_contiguous,
                     int64_t n_specs, const uint32_t *spec_codes, const int32_t *spec_tensor, int64_t *num_shards,
                     int64_t *local_shape, int64_t *local_stride, int32_t shape_width, int64_t *local_numel,
                     int64_t *local_bytes, int64_t n_strategies, const int64_t *flops, const int64_t *rw_bytes,
                     const int8_t *dtype, const uint8_t *zero_cost, const int32_t *num_args, double *compute,
                     double *per_arg, int32_t *error_flag, void *stream) {
  if (int rc = check_params(params)) return rc;
  if (n_tensors < 0 || n_specs < 0 || n_strategies < 0) return fail(-1, "apc_input_tables: negative count");
  if (n_tensors > 0 && (!rank || !itemsize || !shape || !stride || !tensor_bytes || !tensor_contiguous))
    return fail(-1, "apc_input_tables: NULL tensor array");
  // the five spec-table outputs may all be NULL: the spec table is then skipped
  const bool spec_table = num_shards || local_shape || local_stride || local_numel || local_bytes;
  if (spec_table)
    if (int rc = check_width(shape_width)) return rc;
  if (spec_table && n_specs > 0 && (!spec_codes || !spec_tensor || !rank || !itemsize || !shape || !stride ||
                                    !num_shards || !local_shape || !local_stride || !local_numel || !local_bytes))
    return fail(-1, "apc_input_tables: the spec table needs all five of its outputs");
  if (n_strategies > 0 && (!flops || !rw_bytes || !dtype || !zero_cost || !num_args))
    return fail(-1, "apc_input_tables: NULL strategy array");
  const int64_t sb = spec_table ? blocks_for(n_specs, kBlock) : 0, tb = blocks_for(n_tensors, kBlock),
                cb = blocks_for(n_strategies, kBlock);
  if (sb + tb + cb == 0) return 0;
  if (sb + tb + cb > INT32_MAX) return fail(-1, "apc_input_tables: too many rows for one launch");
  hipLaunchKernelGGL(input_tables_kernel, dim3((unsigned)(sb + tb + cb)), dim3(kBlock), 0, (hipStream_t)stream, *params,
                     TensorTableArgs{n_tensors, rank, itemsize, shape, stride, tensor_bytes, tensor_contiguous},
                     SpecTableArgs{n_specs, spec_codes, spec_tensor, rank, itemsize, shape, stride, num_shards,
                                   local_shape, local_stride, local_numel, local_bytes, shape_width},
                     ComputeCostArgs{n_strategies, flops, rw_bytes, dtype, zero_cost, num_args, compute, per_arg,
                                     error_flag},
                     sb, tb);
  return check_launch("apc_input_tables");
}

}  // extern "C"

// Row minima need their index arrays and, when some tile serves identical edges, those edges' rows.
static int check_row_minima(const apc_row_minima *rows, const int64_t *dup_entry_begin, const char *who) {
  if (!rows) return 0;
  if (!rows->edge_row_begin || !rows->row_min || !rows->row_argmin) return fail(-1, "%s: NULL row-minimum array", who);
  if (dup_entry_begin && !rows->dup_row_begin) return fail(-1, "%s: identical edges need dup_row_begin", who);
  return 0;
}

// The compile-time output mode of a launch (kOut*).  The specialised modes exist for 2-D and
// 3-D meshes (the planned graphs); other mesh ranks check their output pointers per store.
static int out_mode(int mesh_ndim, const double *comm_out, const uint8_t *trans_out, const double *cost_out) {
  if (mesh_ndim != 2 && mesh_ndim != 3) return kOutAny;
  if (comm_out && trans_out && cost_out) return kOutAll;
  if (cost_out && !comm_out && !trans_out) return kOutCost;
  return kOutAny;
}

static int redistribute_tables_impl(const apc_params *params, const int64_t *tensor_bytes,
                                    const uint8_t *tensor_contiguous, const uint32_t *spec_codes,
                                    const int32_t *spec_tensor, const double *pt_values, const double *per_arg,
                                    int64_t n_tiles, const apc_tile *tiles, const int64_t *dup_entry_begin,
                                    int64_t n_entries, double *comm_out, uint8_t *trans_out, double *cost_out,
                                    const apc_row_minima *rows, void *stream) {
  if (int rc = check_params(params)) return rc;
  if (n_tiles < 0 || n_tiles > (1 << 30)) return fail(-1, "n_tiles %lld out of range", (long long)n_tiles);
  if (n_tiles == 0) return 0;
  if (int rc = check_row_minima(rows, dup_entry_begin, "apc_redistribute_tables_row_min")) return rc;
  if (n_entries < 0) return fail(-1, "n_entries < 0");
  if (!tensor_bytes || !tensor_contiguous || !spec_codes || !spec_tensor || !tiles)
    return fail(-1, "apc_redistribute_tables: NULL table");
  if (cost_out && !per_arg) return fail(-1, "cost_out needs compute_cost_per_arg");
  TableArgs a{tensor_bytes, tensor_contiguous, spec_codes, spec_tensor, pt_values, per_arg,
              tiles,        dup_entry_begin,   comm_out,   trans_out,   cost_out,
              nullptr,      nullptr,           nullptr,    nullptr,     nullptr, nullptr, nullptr, nullptr, nullptr,
              rows ? rows->edge_row_begin : nullptr, rows ? rows->dup_row_begin : nullptr,
              rows ? rows->row_min : nullptr, rows ? rows->row_argmin : nullptr, term_layout(*params)};
  const int nt = (int)n_tiles, xs = xcd_shift();
  hipStream_t s = (hipStream_t)stream;
  // Wavefronts per tile by the mean number of values a tile stores (n_entries counts the
  // copies written for de-duplicated edges too: work per tile either way): one below 512,
  // two up to 4096, four above.  Measured on tables of 290 .. 1800 values per tile: more
  // wavefronts drain a long tile sooner, fewer leave more tiles resident per compute unit
  // (1800 values per tile, Llama-3-70B: 169 / 154 / 179 us with one / two / four).
  const dim3 grid((unsigned)(((n_tiles + (1 << xs) - 1) >> xs) << xs));  // rounded up for xcd_chunked_unit
  const int64_t per_tile = n_entries / n_tiles;
  int threads = per_tile >= 4096 ? 256 : per_tile >= 512 ? 128 : 64;
  if (const char *env = getenv("APC_TILE_THREADS")) threads = atoi(env);  // tuning override
  const int om = out_mode(params->mesh_ndim, comm_out, trans_out, cost_out);
#define APC_LAUNCH_T(KERNEL_, M_, OUT_)                                                                               \
  const int wg = threads >= 256 ? 256 : threads >= 128 ? 128 : 64;                                                     \
  const size_t lds = rows ? stage_lds_bytes<M_, true>(a.lay, wg) : stage_lds_bytes<M_, false>(a.lay, wg);              \
  if (threads >= 256) hipLaunchKernelGGL((KERNEL_<M_, 256, OUT_>), grid, dim3(256), lds, s, a.tiles, nt, xs, *params, a);      \
  else if (threads >= 128) hipLaunchKernelGGL((KERNEL_<M_, 128, OUT_>), grid, dim3(128), lds, s, a.tiles, nt, xs, *params, a); \
  else hipLaunchKernelGGL((KERNEL_<M_, 64, OUT_>), grid, dim3(64), lds, s, a.tiles, nt, xs, *params, a)
#define APC_LAUNCH_K(KERNEL_, M_)                                   \
  if (om == kOutAll) { APC_LAUNCH_T(KERNEL_, M_, kOutAll); }        \
  else if (om == kOutCost) { APC_LAUNCH_T(KERNEL_, M_, kOutCost); } \
  else { APC_LAUNCH_T(KERNEL_, M_, kOutAny); }
#define APC_LAUNCH_ANY(KERNEL_, M_) { APC_LAUNCH_T(KERNEL_, M_, kOutAny); }
  if (rows) {
    switch (params->mesh_ndim) {
      case 1: APC_LAUNCH_ANY(redistribute_tiles_row_min_kernel, 1); break;
      case 2: APC_LAUNCH_K(redistribute_tiles_row_min_kernel, 2); break;
      case 3: APC_LAUNCH_K(redistribute_tiles_row_min_kernel, 3); break;
      default: APC_LAUNCH_ANY(redistribute_tiles_row_min_kernel, 4); break;
    }
  } else {
    switch (params->mesh_ndim) {
      case 1: APC_LAUNCH_ANY(redistribute_tiles_kernel, 1); break;
      case 2: APC_LAUNCH_K(redistribute_tiles_kernel, 2); break;
      case 3: APC_LAUNCH_K(redistribute_tiles_kernel, 3); break;
      default: APC_LAUNCH_ANY(redistribute_tiles_kernel, 4); break;
    }
  }
#undef APC_LAUNCH_T
#undef APC_LAUNCH_K
#undef APC_LAUNCH_ANY
  return check_launch("apc_redistribute_tables");
}

static int build_tables_impl(const apc_params *params, int64_t n_tensors, const int32_t *rank, const int32_t *itemsize,
                     const int64_t *shape, const int64_t *stride, int64_t *tensor_bytes, uint8_t *tensor_contiguous,
                     int64_t n_specs, const uint32_t *spec_codes, const int32_t *spec_tensor, int64_t *num_shards,
                     int64_t *local_shape, int64_t *local_stride, int32_t shape_width, int64_t *local_numel,
                     int64_t *local_bytes, int64_t n_strategies, const int64_t *flops, const int64_t *rw_bytes,
                     const int8_t *dtype, const uint8_t *zero_cost, const int32_t *num_args, double *compute,
                     double *per_arg, int32_t *error_flag, const double *pt_values, int64_t n_tiles, const apc_tile *tiles,
                     const int64_t *dup_entry_begin, int64_t n_entries, double *comm_out, uint8_t *trans_out,
                     double *cost_out, const apc_row_minima *rows, void *stream) {
  if (int rc = check_params(params)) return rc;
  if (n_tiles > 0)
    if (int rc = check_row_minima(rows, dup_entry_begin, "apc_build_tables_row_min")) return rc;
  if (n_tensors < 0 || n_specs < 0 || n_strategies < 0 || n_entries < 0) return fail(-1, "apc_build_tables: negative count");
  if (n_tiles < 0 || n_tiles > (1 << 30)) return fail(-1, "n_tiles %lld out of range", (long long)n_tiles);
  if (n_tensors > 0 && (!rank || !itemsize || !shape || !stride || !tensor_bytes || !tensor_contiguous))
    return fail(-1, "apc_build_tables: NULL tensor array");
  const bool spec_table = num_shards || local_shape || local_stride || local_numel || local_bytes;
  if (spec_table)
    if (int rc = check_width(shape_width)) return rc;
  if (spec_table && n_specs > 0 && (!spec_codes || !spec_tensor || !num_shards || !local_shape || !local_stride ||
                                    !local_numel || !local_bytes))
    return fail(-1, "apc_build_tables: the spec table needs all five of its outputs");
  if (n_strategies > 0 && (!flops || !rw_bytes || !dtype || !zero_cost || !num_args))
    return fail(-1, "apc_build_tables: NULL strategy array");
  if (n_tiles > 0 && (!spec_codes || !spec_tensor || !tiles || !rank || !itemsize || !shape || !stride))
    return fail(-1, "apc_build_tables: NULL table");
  // (a tile without a tensor still loads row 0 of the tensor table: unconditional loads)
  if (n_tiles > 0 && n_tensors == 0) return fail(-1, "apc_build_tables: tiles need a tensor table with at least one row");
  const int xs = xcd_shift();
  int threads = 256;
  if (n_tiles > 0) {
    const int64_t per_tile = n_entries / n_tiles;
    threads = per_tile >= 1536 ? 256 : per_tile >= 512 ? 128 : 64;
  }
  if (const char *env = getenv("APC_TILE_THREADS")) threads = atoi(env);  // tuning override
  threads = threads >= 256 ? 256 : threads >= 128 ? 128 : 64;
  const int64_t tile_blocks = ((n_tiles + (1 << xs) - 1) >> xs) << xs;
  const int64_t sb = spec_table ? blocks_for(n_specs, threads) : 0, tb = blocks_for(n_tensors, threads),
                cb = blocks_for(n_strategies, threads);
  const int64_t blocks = tile_blocks + sb + tb + cb;
  if (blocks == 0) return 0;
  if (blocks > INT32_MAX) return fail(-1, "apc_build_tables: too many rows for one launch");
  // the tiles read neither the tensor table nor the compute costs (written by this launch)
  TableArgs a{nullptr, nullptr, spec_codes, spec_tensor, pt_values, nullptr, tiles, dup_entry_begin,
              comm_out, trans_out, cost_out, rank, itemsize, shape, stride, flops, rw_bytes, dtype, zero_cost, num_args,
              rows ? rows->edge_row_begin : nullptr, rows ? rows->dup_row_begin : nullptr,
              rows ? rows->row_min : nullptr, rows ? rows->row_argmin : nullptr, term_layout(*params)};
  const TensorTableArgs ta{n_tensors, rank, itemsize, shape, stride, tensor_bytes, tensor_contiguous};
  const SpecTableArgs sa{n_specs, spec_codes, spec_tensor, rank, itemsize, shape, stride, num_shards,
                         local_shape, local_stride, local_numel, local_bytes, shape_width};
  const ComputeCostArgs ca{n_strategies, flops, rw_bytes, dtype, zero_cost, num_args, compute, per_arg, error_flag};
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)blocks);
  const int nt = (int)n_tiles;
  const int om = out_mode(params->mesh_ndim, comm_out, trans_out, cost_out);
#define APC_LAUNCH_ALL_T(M_, RM_, OUT_)                                                                                 \
  if (threads == 256) hipLaunchKernelGGL((build_tables_kernel<M_, 256, RM_, OUT_>), grid, dim3(256), 0, s, a.tiles, nt, xs, tile_blocks, *params, a, ta, sa, ca, sb, tb); \
  else if (threads == 128) hipLaunchKernelGGL((build_tables_kernel<M_, 128, RM_, OUT_>), grid, dim3(128), 0, s, a.tiles, nt, xs, tile_blocks, *params, a, ta, sa, ca, sb, tb); \
  else hipLaunchKernelGGL((build_tables_kernel<M_, 64, RM_, OUT_>), grid, dim3(64), 0, s, a.tiles, nt, xs, tile_blocks, *params, a, ta, sa, ca, sb, tb)
#define APC_LAUNCH_ALL_RM(M_, RM_)                                   \
  if (om == kOutAll) { APC_LAUNCH_ALL_T(M_, RM_, kOutAll); }         \
  else if (om == kOutCost) { APC_LAUNCH_ALL_T(M_, RM_, kOutCost); }  \
  else { APC_LAUNCH_ALL_T(M_, RM_, kOutAny); }
#define APC_LAUNCH_ALL(M_)                    \
  if (rows) { APC_LAUNCH_ALL_RM(M_, true); } else { APC_LAUNCH_ALL_RM(M_, false); }
#define APC_LAUNCH_ALL_ANY(M_)                \
  if (rows) { APC_LAUNCH_ALL_T(M_, true, kOutAny); } else { APC_LAUNCH_ALL_T(M_, false, kOutAny); }
  switch (params->mesh_ndim) {
    case 1: APC_LAUNCH_ALL_ANY(1); break;
    case 2: APC_LAUNCH_ALL(2); break;
    case 3: APC_LAUNCH_ALL(3); break;
    default: APC_LAUNCH_ALL_ANY(4); break;
  }
#undef APC_LAUNCH_ALL_T
#undef APC_LAUNCH_ALL_RM
#undef APC_LAUNCH_ALL
#undef APC_LAUNCH_ALL_ANY
  return check_launch("apc_build_tables");
}

extern "C" {

int apc_redistribute_tables(const apc_params *params, const int64_t *tensor_bytes, const uint8_t *tensor_contiguous,
                            const uint32_t *spec_codes, const int32_t *spec_tensor, const double *pt_values,
                            const double *per_arg, int64_t n_tiles, const apc_tile *tiles,
                            const int64_t *dup_entry_begin, int64_t n_entries, double *comm_out, uint8_t *trans_out,
                            double *cost_out, void *stream) {
  return redistribute_tables_impl(params, tensor_bytes, tensor_contiguous, spec_codes, spec_tensor, pt_values, per_arg,
                                  n_tiles, tiles, dup_entry_begin, n_entries, comm_out, trans_out, cost_out, nullptr,
                                  stream);
}

int apc_redistribute_tables_row_min(const apc_params *params, const int64_t *tensor_bytes,
                                    const uint8_t *tensor_contiguous, const uint32_t *spec_codes,
                                    const int32_t *spec_tensor, const double *pt_values, const double *per_arg,
                                    int64_t n_tiles, const apc_tile *tiles, const int64_t *dup_entry_begin,
                                    int64_t n_entries, double *comm_out, uint8_t *trans_out, double *cost_out,
                                    const apc_row_minima *rows, void *stream) {
  if (!rows) return fail(-1, "apc_redistribute_tables_row_min: NULL rows");
  return redistribute_tables_impl(params, tensor_bytes, tensor_contiguous, spec_codes, spec_tensor, pt_values, per_arg,
                                  n_tiles, tiles, dup_entry_begin, n_entries, comm_out, trans_out, cost_out, rows, stream);
}

#define APC_BUILD_TABLES_PARAMS                                                                                         \
  const apc_params *params, int64_t n_tensors, const int32_t *rank, const int32_t *itemsize, const int64_t *shape,      \
      const int64_t *stride, int64_t *tensor_bytes, uint8_t *tensor_contiguous, int64_t n_specs,                        \
      const uint32_t *spec_codes, const int32_t *spec_tensor, int64_t *num_shards, int64_t *local_shape,                \
      int64_t *local_stride, int32_t shape_width, int64_t *local_numel, int64_t *local_bytes, int64_t n_strategies,     \
      const int64_t *flops, const int64_t *rw_bytes, const int8_t *dtype, const uint8_t *zero_cost,                     \
      const int32_t *num_args, double *compute, double *per_arg, int32_t *error_flag, const double *pt_values,          \
      int64_t n_tiles, const apc_tile *tiles, const int64_t *dup_entry_begin, int64_t n_entries, double *comm_out,      \
      uint8_t *trans_out, double *cost_out
#define APC_BUILD_TABLES_ARGS                                                                                           \
  params, n_tensors, rank, itemsize, shape, stride, tensor_bytes, tensor_contiguous, n_specs, spec_codes, spec_tensor,  \
      num_shards, local_shape, local_stride, shape_width, local_numel, local_bytes, n_strategies, flops, rw_bytes,      \
      dtype, zero_cost, num_args, compute, per_arg, error_flag, pt_values, n_tiles, tiles, dup_entry_begin, n_entries,  \
      comm_out, trans_out, cost_out

int apc_build_tables(APC_BUILD_TABLES_PARAMS, void *stream) {
  return build_tables_impl(APC_BUILD_TABLES_ARGS, nullptr, stream);
}

int apc_build_tables_row_min(APC_BUILD_TABLES_PARAMS, const apc_row_minima *rows, void *stream) {
  if (!rows) return fail(-1, "apc_build_tables_row_min: NULL rows");
  return build_tables_impl(APC_BUILD_TABLES_ARGS, rows, stream);
}
#undef APC_BUILD_TABLES_PARAMS
#undef APC_BUILD_TABLES_ARGS

}  // extern "C"

static int segmented_min_impl(const double *values, const int64_t *seg_ptr, int64_t n_seg, int64_t n_values, double *mins,
                              int32_t *args, const SegmentCopies *copies, const char *who, void *stream) {
  if (n_seg < 0 || n_values < 0) return fail(-1, "negative count");
  if (n_seg == 0) return 0;
  if (!seg_ptr || !mins || !args || (!values && n_values > 0)) return fail(-1, "%s: NULL array", who);
  if (n_seg > (int64_t)INT32_MAX * 4) return fail(-1, "n_segments %lld too large", (long long)n_seg);
  hipStream_t s = (hipStream_t)stream;
  // lanes per segment: about a tenth of the mean length, so that a lane has several
  // independent loads in flight (measured best on both benchmark tables; APC_SEGMIN_GROUP
  // overrides, for tuning)
  const double mean = (double)n_values / (double)n_seg;
  int g = 2;
  while (g < 64 && g * 12 <= mean) g *= 2;
  if (const char *env = getenv("APC_SEGMIN_GROUP")) g = atoi(env);
  switch (g) {
    case 1: launch_segmented_min<1>(values, seg_ptr, n_seg, mins, args, copies, s); break;
    case 2: launch_segmented_min<2>(values, seg_ptr, n_seg, mins, args, copies, s); break;
    case 4: launch_segmented_min<4>(values, seg_ptr, n_seg, mins, args, copies, s); break;
    case 8: launch_segmented_min<8>(values, seg_ptr, n_seg, mins, args, copies, s); break;
    case 16: launch_segmented_min<16>(values, seg_ptr, n_seg, mins, args, copies, s); break;
    case 32: launch_segmented_min<32>(values, seg_ptr, n_seg, mins, args, copies, s); break;
    case 64: launch_segmented_min<64>(values, seg_ptr, n_seg, mins, args, copies, s); break;
    default: return fail(-1, "segment group width %d is not a power of two up to 64", g);
  }
  return check_launch(who);
}

extern "C" {

int apc_segmented_min(const double *values, const int64_t *seg_ptr, int64_t n_seg, int64_t n_values, double *mins,
                      int32_t *args, void *stream) {
  return segmented_min_impl(values, seg_ptr, n_seg, n_values, mins, args, nullptr, "apc_segmented_min", stream);
}

int apc_segmented_min_copies(const double *values, const int64_t *seg_ptr, int64_t n_selected, const int64_t *selected,
                             const int64_t *copy_ptr, const int64_t *copy_segments, int64_t n_values_selected,
                             double *mins, int32_t *args, void *stream) {
  if (n_selected > 0 && (!selected || !copy_ptr)) return fail(-1, "apc_segmented_min_copies: NULL selection");
  const SegmentCopies copies{selected, copy_ptr, copy_segments};
  return segmented_min_impl(values, seg_ptr, n_selected, n_values_selected, mins, args, &copies,
                            "apc_segmented_min_copies", stream);
}

int apc_strategy_bounds(int64_t n_strategies, const int32_t *strat_node, const int64_t *node_strat_begin,
                        const int64_t *node_edge_begin, const int32_t *edges_by_node, const int64_t *edge_row_begin,
                        const double *row_min, double *bound, void *stream) {
  if (n_strategies < 0) return fail(-1, "negative count");
  if (n_strategies == 0) return 0;
  if (!strat_node || !node_strat_begin || !node_edge_begin || !edge_row_begin || !row_min || !bound)
    return fail(-1, "apc_strategy_bounds: NULL array");  // (edges_by_node may be NULL when no node has an edge)
  if ((n_strategies + kBlock - 1) / kBlock > INT32_MAX) return fail(-1, "n_strategies %lld too large", (long long)n_strategies);
  hipLaunchKernelGGL(strategy_bounds_kernel, dim3(blocks_for(n_strategies, kBlock)), dim3(kBlock), 0, (hipStream_t)stream,
                     n_strategies, strat_node, node_strat_begin, node_edge_begin, edges_by_node, edge_row_begin, row_min,
                     bound);
  return check_launch("apc_strategy_bounds");
}

int apc_cost_objective(int64_t n_vars, int64_t n_groups, const int64_t *group_var_begin, const int64_t *group_member_begin,
                       const int64_t *member_entry_begin, const double *cost, double inf_replacement, double *objective,
                       uint8_t *forced_zero, void *stream) {
  if (n_vars < 0 || n_groups < 0) return fail(-1, "apc_cost_objective: negative count");
  if (n_vars == 0) return 0;
  if (n_groups == 0) return fail(-1, "apc_cost_objective: %lld variables and no group", (long long)n_vars);
  if (!group_var_begin || !group_member_begin || !member_entry_begin || !cost || !objective || !forced_zero)
    return fail(-1, "apc_cost_objective: NULL array");
  if (n_groups > INT32_MAX) return fail(-1, "apc_cost_objective: %lld groups, at most %d are launched", (long long)n_groups, INT32_MAX);
  // a program of few groups spreads each over several workgroups (those beyond a group's size
  // leave at once); with thousands of groups the device is full as it is
  // (and no more shares than twice what a group of average size fills)
  const int64_t average_runs = (n_vars / n_groups + kBlock - 1) / kBlock;
  const int64_t shares = n_groups >= 4096 ? 1 : std::min<int64_t>({64, (4096 + n_groups - 1) / n_groups, 2 * std::max<int64_t>(1, average_runs)});
  hipLaunchKernelGGL(cost_objective_kernel, dim3((unsigned)n_groups, (unsigned)shares), dim3(kBlock), 0, (hipStream_t)stream,
                     group_var_begin, group_member_begin, member_entry_begin, cost, inf_replacement, objective, forced_zero);
  return check_launch("apc_cost_objective");
}

int apc_validate_row_minima_host(int64_t n_edges, const int32_t *edge_n_src, const int32_t *edge_n_tgt, int64_t n_tiles,
                                 const apc_tile *tiles) {
  if (n_edges < 0 || n_tiles < 0) return fail(-1, "apc_validate_row_minima_host: negative count");
  if ((n_edges > 0 && (!edge_n_src || !edge_n_tgt)) || (n_tiles > 0 && !tiles))
    return fail(-1, "apc_validate_row_minima_host: NULL array");
  for (int64_t e = 0; e < n_edges; ++e)
    if (edge_n_tgt[e] > 0 && (edge_n_src[e] < 1 || edge_n_src[e] > APC_TILE_MAX_COLS))
      return fail(-2, "edge %lld: %d producer strategies; row minima inside the table launch need 1 .. %d", (long long)e,
                  edge_n_src[e], APC_TILE_MAX_COLS);
  for (int64_t t = 0; t < n_tiles; ++t) {
    const apc_tile &tl = tiles[t];
    if (tl.edge < 0 || tl.edge >= n_edges) return fail(-2, "tile %lld: edge %d out of range", (long long)t, tl.edge);
    if (tl.col_begin != 0 || (tl.counts >> 16) != edge_n_src[tl.edge])
      return fail(-2, "tile %lld: columns [%d, +%d) are not the whole rows of edge %d (%d columns)", (long long)t,
                  tl.col_begin, tl.counts >> 16, tl.edge, edge_n_src[tl.edge]);
  }
  return 0;
}

int apc_diffusion_sweeps(int32_t n_sweeps, int32_t n_colors, const int64_t *color_begin_host, const int32_t *color_nodes,
                         int64_t n_classes, const int64_t *label_begin, const int64_t *inc_begin, const int32_t *inc_edge,
                         const uint8_t *inc_side, const int64_t *edge_begin, const int32_t *edge_i, const int32_t *edge_j,
                         int32_t max_labels, double *theta, double *unary, void *stream) {
  if (n_sweeps < 0 || n_colors < 0 || n_classes < 0) return fail(-1, "apc_diffusion_sweeps: negative count");
  if (n_sweeps == 0 || n_colors == 0 || n_classes == 0) return 0;
  if (max_labels > kDiffusionMaxLabels)
    return fail(-1, "apc_diffusion_sweeps: a class has %d labels, at most %d are staged", max_labels, kDiffusionMaxLabels);
  if (!color_begin_host || !color_nodes || !label_begin || !inc_begin || !edge_begin || !theta || !unary)
    return fail(-1, "apc_diffusion_sweeps: NULL array");
  if (color_begin_host[0] != 0 || color_begin_host[n_colors] != n_classes)
    return fail(-1, "apc_diffusion_sweeps: the colours must partition the classes");
  for (int32_t s = 0; s < n_sweeps; ++s) {
    for (int32_t c = 0; c < n_colors; ++c) {
      const int64_t n = color_begin_host[c + 1] - color_begin_host[c];
      if (n < 0 || n > INT32_MAX) return fail(-1, "apc_diffusion_sweeps: colour %d has %lld classes", c, (long long)n);
      if (n == 0) continue;
      hipLaunchKernelGGL(diffusion_node_update_kernel, dim3((unsigned)n), dim3(kBlock), 0, (hipStream_t)stream,
                         DiffusionArgs{color_nodes + color_begin_host[c], label_begin, inc_begin, inc_edge, inc_side,
                                       edge_begin, edge_i, edge_j, theta, unary});
    }
    if (int rc = check_launch("apc_diffusion_sweeps")) return rc;
  }
  return 0;
}

}  // extern "C"

// ------------------------------------------------------------------------------------------
// An entry point that allocates nothing and needs no caller-provided staging: the cost
// matrices straight from the tensor and strategy tables.  The staging tables the tile kernel
// reads (bytes and contiguity per tensor, compute cost / num_args per strategy; what
// apc_input_tables writes into caller arrays for apc_redistribute_tables) live in a file-scope
// device array of fixed size.  Every device holds its own copy of the array at its own address,
// looked up once per device; calls on one device share it, so calls that overlap on a device race.
// ------------------------------------------------------------------------------------------
constexpr int64_t kStaticMaxTensors = 1 << 16;     // 8 B + 1 B each
constexpr int64_t kStaticMaxStrategies = 1 << 21;  // 8 B each (compute cost / num_args)
constexpr size_t kStaticBytesOff = 0;
constexpr size_t kStaticPerArgOff = kStaticBytesOff + (size_t)kStaticMaxTensors * sizeof(int64_t);
constexpr size_t kStaticContigOff = kStaticPerArgOff + (size_t)kStaticMaxStrategies * sizeof(double);
constexpr size_t kStaticScratchBytes = kStaticContigOff + (size_t)kStaticMaxTensors;  // 17.1 MB
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void *g_scratch_of_device[kMaxDevices];  // the array's device address, per device (0 = not looked up yet)

// The address of this device's copy of `scratch` (the array's name is only a host-side handle).
static int scratch_of_current_device(unsigned char **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(-3, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(-1, "device %d outside [0, %d)", dev, kMaxDevices);
  void *p = __atomic_load_n(&g_scratch_of_device[dev], __ATOMIC_ACQUIRE);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return fail(-3, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    __atomic_store_n(&g_scratch_of_device[dev], p, __ATOMIC_RELEASE);  // (every thread finds the same address)
  }
  *out = static_cast<unsigned char *>(p);
  return 0;
}

extern "C" {

int apc_redistribute_tables_static(const apc_params *params, int64_t n_tensors, const int32_t *rank, const int32_t *itemsize,
                                   const int64_t *shape, const int64_t *stride, int64_t n_strategies, const int64_t *flops,
                                   const int64_t *rw_bytes, const int8_t *dtype, const uint8_t *zero_cost,
                                   const int32_t *num_args, const uint32_t *spec_codes, const int32_t *spec_tensor,
                                   const double *pt_values, int64_t n_tiles, const apc_tile *tiles,
                                   const int64_t *dup_entry_begin, int64_t n_entries, double *comm_out, uint8_t *trans_out,
                                   double *cost_out, void *stream) {
  if (n_tensors < 0 || n_strategies < 0) return fail(-1, "apc_redistribute_tables_static: negative count");
  if (n_tensors > kStaticMaxTensors)
    return fail(-1, "apc_redistribute_tables_static: %lld tensors, the static staging holds %lld (use apc_input_tables + "
                "apc_redistribute_tables with caller-allocated staging)", (long long)n_tensors, (long long)kStaticMaxTensors);
  if (n_strategies > kStaticMaxStrategies)
    return fail(-1, "apc_redistribute_tables_static: %lld strategies, the static staging holds %lld (use apc_input_tables + "
                "apc_redistribute_tables with caller-allocated staging)", (long long)n_strategies,
                (long long)kStaticMaxStrategies);
  unsigned char *base = nullptr;
  if (int rc = scratch_of_current_device(&base)) return rc;
  int64_t *tensor_bytes = reinterpret_cast<int64_t *>(base + kStaticBytesOff);
  double *per_arg = reinterpret_cast<double *>(base + kStaticPerArgOff);
  uint8_t *tensor_contiguous = base + kStaticContigOff;
  // staging tables into the static array (no spec table, no per-strategy compute cost, no error
  // flag: a strategy with flops and an unsupported dtype shows as NaN costs), then the tiles;
  // both launches on the caller's stream, so the second sees what the first wrote
  if (int rc = apc_input_tables(params, n_tensors, rank, itemsize, shape, stride, tensor_bytes, tensor_contiguous, 0, nullptr,
                                nullptr, nullptr, nullptr, nullptr, 2, nullptr, nullptr, n_strategies, flops, rw_bytes, dtype,
                                zero_cost, num_args, nullptr, per_arg, nullptr, stream))
    return rc;
  return redistribute_tables_impl(params, tensor_bytes, tensor_contiguous, spec_codes, spec_tensor, pt_values, per_arg, n_tiles,
                                  tiles, dup_entry_begin, n_entries, comm_out, trans_out, cost_out, nullptr, stream);
}

}  // extern "C"

// ------------------------------------------------------------------------------------------
// Packed tiles: host-side check and launch.
// ------------------------------------------------------------------------------------------
static_assert(sizeof(apc_packed_tile) == 2752 && sizeof(apc_packed_tile) % 64 == 0, "apc_packed_tile layout");
static_assert(offsetof(apc_packed_tile, entry_begin) == 32 && offsetof(apc_packed_tile, tensor_shape) == 64,
              "the header is the record's first 64 bytes");

extern "C" {

int apc_validate_packed_tiles_host(int64_t n_tensors, const int32_t *tensor_rank, const int32_t *tensor_itemsize,
                                   const int64_t *tensor_shape, const int64_t *tensor_stride, int64_t n_specs,
                                   const uint32_t *spec_codes, const int32_t *spec_tensor, int64_t n_strategies,
                                   const int64_t *flops, const int64_t *rw_bytes, const int8_t *dtype_code,
                                   const uint8_t *zero_cost, const int32_t *num_args, int64_t n_edges,
                                   const int64_t *edge_row_begin, int64_t n_tiles, const apc_tile *tiles, int64_t n_dups,
                                   const int64_t *dup_entry_begin, const int64_t *dup_row_begin,
                                   const apc_packed_tile *packed) {
  if (n_tiles < 0 || n_tensors < 0 || n_specs < 0 || n_strategies < 0 || n_edges < 0 || n_dups < 0)
    return fail(-1, "apc_validate_packed_tiles_host: negative count");
  if (n_tiles == 0) return 0;
  if (!tiles || !packed || !spec_codes || !spec_tensor || !edge_row_begin || !flops || !rw_bytes || !dtype_code || !zero_cost ||
      !num_args || (n_dups > 0 && (!dup_entry_begin || !dup_row_begin)) ||
      (n_tensors > 0 && (!tensor_rank || !tensor_itemsize || !tensor_shape || !tensor_stride)))
    return fail(-1, "apc_validate_packed_tiles_host: NULL array");
  for (int64_t t = 0; t < n_tiles; ++t) {
    const apc_tile &tl = tiles[t];
    const apc_packed_tile &pk = packed[t];
    const int rows = tl.counts & 0xFFFF, cols = tl.counts >> 16;
    if (tl.edge < 0 || tl.edge >= n_edges) return fail(-2, "tile %lld: edge %d out of range", (long long)t, tl.edge);
    if (tl.col_begin != 0 || cols != tl.n_src || cols < 1 || cols > APC_TILE_MAX_COLS || rows < 1 || rows > APC_TILE_MAX_ROWS)
      return fail(-2, "tile %lld: a packed tile holds 1 .. %d whole rows of at most %d columns (%d rows, columns [%d, +%d) of %d)",
                  (long long)t, APC_TILE_MAX_ROWS, APC_TILE_MAX_COLS, rows, tl.col_begin, cols, tl.n_src);
    if (tl.dup_count < 0 || tl.dup_count > APC_PACKED_MAX_DUPS || tl.dup_begin < 0 || (int64_t)tl.dup_begin + tl.dup_count > n_dups)
      return fail(-2, "tile %lld: %d identical edges, a packed tile serves at most %d", (long long)t, tl.dup_count,
                  APC_PACKED_MAX_DUPS);
    if (tl.src_begin < 0 || (int64_t)tl.src_begin + cols > n_specs || tl.tgt_begin < 0 ||
        (int64_t)tl.tgt_begin + tl.row_begin + rows > n_specs || tl.strat_begin < 0 ||
        (int64_t)tl.strat_begin + tl.row_begin + rows > n_strategies)
      return fail(-2, "tile %lld: spec or strategy rows outside their tables", (long long)t);
    const int64_t first = (int64_t)tl.row_begin * cols;
    bool mixed = false;
    for (int j = 0; j < cols; ++j) {
      const int64_t sp = (int64_t)tl.src_begin + j;
      if (pk.col_codes[j] != spec_codes[sp] || pk.col_tensor[j] != spec_tensor[sp])
        return fail(-2, "packed tile %lld: producer spec %d differs from the spec table", (long long)t, j);
      mixed |= spec_tensor[sp] < 0 || spec_tensor[sp] != tl.tensor;
    }
    for (int j = 0; j < rows; ++j) {
      const int64_t ts = (int64_t)tl.tgt_begin + tl.row_begin + j, sr = (int64_t)tl.strat_begin + tl.row_begin + j;
      if (pk.row_codes[j] != spec_codes[ts] || pk.row_tensor[j] != spec_tensor[ts])
        return fail(-2, "packed tile %lld: consumer spec %d differs from the spec table", (long long)t, j);
      mixed |= spec_tensor[ts] < 0;
      if (num_args[sr] < 1 || num_args[sr] > 0x7FFF)
        return fail(-2, "packed tile %lld: num_args %d of consumer strategy %d does not fit its 15 bits", (long long)t,
                    num_args[sr], j);
      const int32_t meta = (int32_t)(uint8_t)dtype_code[sr] | ((int32_t)(zero_cost[sr] != 0) << 8) | (num_args[sr] << 16);
      if (pk.row_flops[j] != flops[sr] || pk.row_rw_bytes[j] != rw_bytes[sr] || pk.row_meta[j] != meta)
        return fail(-2, "packed tile %lld: consumer strategy %d differs from the strategy table", (long long)t, j);
    }
    if (pk.rows != rows || pk.cols != cols || pk.dup_count != tl.dup_count || pk.tensor != tl.tensor || pk.edge != tl.edge ||
        pk.flags != (tl.flags | (mixed ? APC_PACKED_MIXED : 0)) || pk.entry_begin != tl.entry_begin + first ||
        pk.row_begin != edge_row_begin[tl.edge] + tl.row_begin || pk.pt_begin != (tl.pt_begin < 0 ? -1 : tl.pt_begin + first))
      return fail(-2, "packed tile %lld: header does not repeat the fields of tile record %lld", (long long)t, (long long)t);
    if (tl.tensor >= 0) {
      if (tl.tensor >= n_tensors) return fail(-2, "tile %lld: tensor %d out of range", (long long)t, tl.tensor);
      if (pk.tensor_rank != tensor_rank[tl.tensor] || pk.tensor_itemsize != tensor_itemsize[tl.tensor] ||
          memcmp(pk.tensor_shape, tensor_shape + (int64_t)tl.tensor * APC_MAX_RANK, sizeof(pk.tensor_shape)) != 0 ||
          memcmp(pk.tensor_stride, tensor_stride + (int64_t)tl.tensor * APC_MAX_RANK, sizeof(pk.tensor_stride)) != 0)
        return fail(-2, "packed tile %lld: tensor row differs from the tensor table", (long long)t);
    }
    for (int d = 0; d < tl.dup_count; ++d)
      if (pk.dup_entry_begin[d] != dup_entry_begin[tl.dup_begin + d] + first ||
          pk.dup_row_begin[d] != dup_row_begin[tl.dup_begin + d] + tl.row_begin)
        return fail(-2, "packed tile %lld: identical edge %d differs from the duplicate lists", (long long)t, d);
  }
  return 0;
}

int apc_build_tables_packed(const apc_params *params, int64_t n_tensors, const int32_t *rank, const int32_t *itemsize,
                            const int64_t *shape, const int64_t *stride, int64_t *tensor_bytes, uint8_t *tensor_contiguous,
                            int64_t n_strategies, const int64_t *flops, const int64_t *rw_bytes, const int8_t *dtype,
                            const uint8_t *zero_cost, const int32_t *num_args, double *compute, double *per_arg,
                            int32_t *error_flag, const double *pt_values, int64_t n_tiles, const apc_packed_tile *packed,
                            int64_t n_entries, double *cost_out, double *row_min, int32_t *row_argmin, void *stream) {
  if (int rc = check_params(params)) return rc;
  if (n_tensors < 0 || n_strategies < 0 || n_entries < 0) return fail(-1, "apc_build_tables_packed: negative count");
  if (n_tiles < 0 || n_tiles > (1 << 30)) return fail(-1, "n_tiles %lld out of range", (long long)n_tiles);
  if (n_tensors > 0 && (!rank || !itemsize || !shape || !stride || !tensor_bytes || !tensor_contiguous))
    return fail(-1, "apc_build_tables_packed: NULL tensor array");
  if (n_strategies > 0 && (!flops || !rw_bytes || !dtype || !zero_cost || !num_args))
    return fail(-1, "apc_build_tables_packed: NULL strategy array");
  if (n_tiles > 0 && (!packed || !cost_out || !row_min || !row_argmin))
    return fail(-1, "apc_build_tables_packed: NULL tile records or outputs");
  if ((reinterpret_cast<uintptr_t>(packed) & 63) != 0) return fail(-1, "apc_build_tables_packed: packed tiles must be 64-byte aligned");
  const int xs = xcd_shift();
  const int64_t tile_blocks = ((n_tiles + (1 << xs) - 1) >> xs) << xs;
  const int64_t tb = blocks_for(n_tensors, kBlock), cb = blocks_for(n_strategies, kBlock);
  const int64_t blocks = tile_blocks + tb + cb;
  if (blocks == 0) return 0;
  if (blocks > INT32_MAX) return fail(-1, "apc_build_tables_packed: too many rows for one launch");
  const TermLayout lay = term_layout(*params);
  PackedArgs a{*params, row_min, row_argmin, pt_values, rank, itemsize, shape, stride, 1.0 / params->rescale, lay.exponents,
               lay.lg_total, {0, 0, 0, 0}};
  for (int i = 0; i < APC_MAX_MESH; ++i) a.lg[i] = lay.lg[i];
  const TensorTableArgs ta{n_tensors, rank, itemsize, shape, stride, tensor_bytes, tensor_contiguous};
  const ComputeCostArgs ca{n_strategies, flops, rw_bytes, dtype, zero_cost, num_args, compute, per_arg, error_flag};
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)blocks);
  const int nt = (int)n_tiles;
#define APC_LAUNCH_PACKED(M_)                                                                                                    \
  if (lay.exponents)                                                                                                           \
    hipLaunchKernelGGL((build_tables_packed_kernel<M_, true>), grid, dim3(kBlock), 0, s, packed, nt, xs, tile_blocks, cost_out, a, \
                       *params, ta, ca, tb);                                                                                   \
  else                                                                                                                         \
    hipLaunchKernelGGL((build_tables_packed_kernel<M_, false>), grid, dim3(kBlock), 0, s, packed, nt, xs, tile_blocks, cost_out, a, \
                       *params, ta, ca, tb)
  switch (params->mesh_ndim) {
    case 1: APC_LAUNCH_PACKED(1); break;
    case 2: APC_LAUNCH_PACKED(2); break;
    case 3: APC_LAUNCH_PACKED(3); break;
    default: APC_LAUNCH_PACKED(4); break;
  }
#undef APC_LAUNCH_PACKED
  return check_launch("apc_build_tables_packed");
}

}  // extern "C"

// ------------------------------------------------------------------------------------------
// Measurement aids (no counterpart in the reference): what a launch costs on this system
// before it does any work, and what the store path gives a kernel that does nothing but write.
// A benchmark prices the table launches against both.
// ------------------------------------------------------------------------------------------
namespace {

__global__ void calibrate_empty_kernel() {}

// Workgroup b writes doubles [b * per_workgroup, (b + 1) * per_workgroup) of out (clipped to n),
// 16 bytes per lane and store instruction, consecutive lanes consecutive addresses.
// THROUGH: the stores are written through to memory (store_through), as the packed pass writes.
template <bool THROUGH>
__global__ __launch_bounds__(kBlock) void calibrate_fill_kernel(double *__restrict__ out, int64_t n, int64_t per_workgroup,
                                                                double value) {
  typedef double pair_t __attribute__((ext_vector_type(2)));
  const int64_t begin = (int64_t)blockIdx.x * per_workgroup;
  const int64_t end = begin + per_workgroup < n ? begin + per_workgroup : n;
  const pair_t v = {value, value};
  int64_t i = begin + 2 * (int64_t)threadIdx.x;
  for (; i + 1 < end; i += 2 * kBlock) {
    if (THROUGH) {
      __asm__ volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(out + i), "v"(v) : "memory");
    } else {
      *reinterpret_cast<pair_t *>(out + i) = v;
    }
  }
  if (i < end) {
    if (THROUGH) store_through(out + i, value);
    else out[i] = value;
  }
}

}  // namespace

extern "C" {

int apc_calibrate_launch(int64_t n_workgroups, int32_t threads, void *stream) {
  if (n_workgroups < 1 || n_workgroups > INT32_MAX || threads < 1 || threads > 1024)
    return fail(-1, "apc_calibrate_launch: %lld workgroups of %d threads", (long long)n_workgroups, threads);
  hipLaunchKernelGGL(calibrate_empty_kernel, dim3((unsigned)n_workgroups), dim3((unsigned)threads), 0, (hipStream_t)stream);
  return check_launch("apc_calibrate_launch");
}

int apc_calibrate_fill(double *out, int64_t n, int64_t per_workgroup, double value, int32_t write_through, void *stream) {
  if (n < 0 || per_workgroup < 2 || (per_workgroup & 1)) return fail(-1, "apc_calibrate_fill: n >= 0, per_workgroup even and >= 2");
  if (n == 0) return 0;
  if (!out) return fail(-1, "apc_calibrate_fill: NULL array");
  if ((reinterpret_cast<uintptr_t>(out) & 15) != 0) return fail(-1, "apc_calibrate_fill: out must be 16-byte aligned");
  const int64_t blocks = (n + per_workgroup - 1) / per_workgroup;
  if (blocks > INT32_MAX) return fail(-1, "apc_calibrate_fill: too many workgroups");
  if (write_through)
    hipLaunchKernelGGL(calibrate_fill_kernel<true>, dim3((unsigned)blocks), dim3(kBlock), 0, (hipStream_t)stream, out, n,
                       per_workgroup, value);
  else
    hipLaunchKernelGGL(calibrate_fill_kernel<false>, dim3((unsigned)blocks), dim3(kBlock), 0, (hipStream_t)stream, out, n,
                       per_workgroup, value);
  return check_launch("apc_calibrate_fill");
}

}  // extern "C"
