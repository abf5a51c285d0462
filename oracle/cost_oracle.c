/*
 * Plain-C restatement of the reference's sharding-cost arithmetic.
 *
 * TEST INFRASTRUCTURE: linked or loaded only by tests/, __graft_entry__.smoke()
 * and bench.py's cpu_baseline leg.  It mirrors oracle/cost_oracle.py function by
 * function (which in turn cites the reference file:line for each formula) and is
 * checked against it bit for bit; it exists so that parity tests can cover
 * tables of 10^6..10^8 entries in seconds.
 *
 * Build with FMA contraction off (see Makefile) so every operation is a single
 * IEEE binary64 rounding, as in CPython.
 *
 * Integer -> double conversions are exact for the value ranges the encoders
 * accept (byte counts and flop counts below 2^53).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define ORC_MAX_RANK 8
#define ORC_MAX_MESH 4

typedef struct {
  int32_t ndim;
  int32_t mesh[ORC_MAX_MESH];
  double bw[ORC_MAX_MESH];
  double lat[ORC_MAX_MESH];
  double base_latency; /* 6.6  torch: _collective_utils.py:286 */
  double a2a_scale;    /* 5    ref: collective_runtime_estimation.py:30-31 */
  double hbm_bw;       /* device row, bytes/s */
  double rw_eff;       /* 0.70 ref: compute_estimation.py:307 */
  double launch_floor; /* 7    ref: compute_estimation.py:309 */
  double compute_eff;  /* 0.70 ref: compute_estimation.py:361 */
  double rescale;      /* ref: optimize_sharding.py:358-359 */
  double gpu_flops[8]; /* tflops * 10**12 per dtype code, 0 = unsupported */
  int32_t transition_scale;
} orc_params;

static inline int kind_of(unsigned c) { return (int)(c >> 6); }
static inline int dim_of(unsigned c) { return (int)(c & 0x0F); }

/* ref: compute_estimation.py:302-314 */
static double rw_time(double bytes, const orc_params *p) {
  double t = bytes / p->hbm_bw * 1e6;
  t = t / p->rw_eff;
  return t > p->launch_floor ? t : p->launch_floor;
}

/* torch: _collective_utils.py:281-313 */
static double ring(double gb, const orc_params *p, int d, int hops) {
  double latency = p->base_latency + (double)hops * p->lat[d];
  double bw = (gb * (double)hops / (double)p->mesh[d]) / p->bw[d];
  return latency + bw * 1e6;
}

/* torch: _prims_common/__init__.py:252-292 */
static int contiguous(int rank, const int64_t *shape, const int64_t *stride) {
  int64_t expected = 1, expected_max = 1;
  for (int i = rank - 1; i >= 0; --i) {
    int64_t x = shape[i], y = stride[i];
    if (x == 1) continue;
    if (y != expected && y != expected_max) return 0;
    expected_max *= (x > 1 ? x : 1);
    expected *= x;
  }
  return 1;
}

static int64_t tensor_bytes(int itemsize, int rank, const int64_t *shape) {
  int64_t n = itemsize;
  for (int i = 0; i < rank; ++i) n *= shape[i];
  return n;
}

/* ref: collective_runtime_estimation.py:37-153 */
static double entry_cost(uint32_t srcp, uint32_t tgtp, int64_t bytes, int cont, const orc_params *p) {
  const int M = p->ndim;
  unsigned src[ORC_MAX_MESH], tgt[ORC_MAX_MESH];
  int all_rep = 1, tgt_partial = 0, tgt_all_shard = 1;
  int64_t shards = 1;
  for (int i = 0; i < M; ++i) {
    src[i] = (srcp >> (8 * i)) & 0xFF;
    tgt[i] = (tgtp >> (8 * i)) & 0xFF;
    if (src[i] != 0) all_rep = 0;
    if (kind_of(tgt[i]) == 1) tgt_partial = 1;
    if (kind_of(tgt[i]) != 2) tgt_all_shard = 0;
    if (kind_of(src[i]) == 2) shards *= p->mesh[i];
  }
  if (all_rep) return tgt_partial ? INFINITY : 0.0;
  int order[ORC_MAX_MESH];
  for (int i = 0; i < M; ++i) order[i] = i;
  if (M == 2 && src[0] == 0x40 && src[1] == 0x40 && tgt_all_shard) {
    order[0] = 1;
    order[1] = 0;
  }
  double cost = 0.0;
  double gb = (double)bytes / (double)shards / 1024 / 1024 / 1024;
  for (int k = 0; k < M; ++k) {
    int i = order[k];
    unsigned c = src[i], t = tgt[i];
    if (c == t) continue;
    double n = (double)p->mesh[i];
    if (!cont) cost += rw_time(gb * 2 * 1073741824.0, p);
    int ck = kind_of(c), tk = kind_of(t);
    if (ck == 2 && tk == 0) {
      gb *= n;
      cost += ring(gb, p, i, p->mesh[i] - 1);
      if (dim_of(c) != 0) cost += rw_time(gb * 2 * 1073741824.0, p);
    } else if (ck == 2 && tk == 2) {
      double t5 = ring(gb, p, i, p->mesh[i] - 1);
      t5 *= p->a2a_scale;
      cost += t5;
      int copies = (dim_of(c) != 0) + (dim_of(t) != 0);
      cost += (double)copies * rw_time(gb * 2 * 1073741824.0, p);
    } else if (ck == 1 && tk == 0) {
      cost += ring(gb, p, i, 2 * (p->mesh[i] - 1));
    } else if (ck == 1 && tk == 2) {
      cost += ring(gb, p, i, p->mesh[i] - 1);
      if (dim_of(t) != 0) cost += rw_time(gb * 2 * 1073741824.0, p);
      gb /= n;
    } else if (tk == 1 && (ck == 2 || ck == 0)) {
      return INFINITY;
    }
    cont = 1;
  }
  return cost;
}

/* ref: compute_estimation.py:334-365 (tail) and optimize_sharding.py:371-373 */
int orc_compute_costs(const orc_params *p, int64_t n, const int64_t *flops, const int64_t *rw_bytes,
                      const int8_t *dtype, const uint8_t *zero_cost, const int32_t *num_args,
                      double *compute, double *per_arg) {
  for (int64_t s = 0; s < n; ++s) {
    double c;
    if (zero_cost[s]) {
      c = 0.0;
    } else {
      double rw = rw_time((double)rw_bytes[s], p);
      if (flops[s] == 0) {
        c = rw;
      } else {
        double gf = p->gpu_flops[dtype[s]];
        if (gf == 0.0) return -1;
        double t = (double)flops[s] / gf * 1e6;
        t = t / p->compute_eff;
        c = t > rw ? t : rw;
      }
    }
    compute[s] = c;
    per_arg[s] = c / (double)num_args[s];
  }
  return 0;
}

/* ref: optimize_sharding.py:270-380 over the flattened encoding */
void orc_build_tables(const orc_params *p, const int32_t *t_rank, const int32_t *t_item,
                      const int64_t *t_shape, const int64_t *t_stride, const uint32_t *s_codes,
                      const int32_t *s_tensor, const int32_t *e_src_begin, const int32_t *e_n_src,
                      const int32_t *e_tgt_begin, const int32_t *e_n_tgt, const int32_t *e_flags,
                      const int64_t *e_pt_begin, const int64_t *e_entry_begin,
                      const int32_t *e_strat_begin, const double *pt, const double *per_arg,
                      int64_t edge_lo, int64_t edge_hi, double *comm_out, uint8_t *trans_out,
                      double *cost_out) {
  const int64_t base = e_entry_begin[edge_lo];
  for (int64_t e = edge_lo; e < edge_hi; ++e) {
    const int ns = e_n_src[e], nt = e_n_tgt[e];
    const int flags = e_flags[e];
    int64_t o = e_entry_begin[e] - base;
    for (int ss = 0; ss < nt; ++ss) {
      const int ts = e_tgt_begin[e] + ss;
      for (int ii = 0; ii < ns; ++ii, ++o) {
        const int sp = e_src_begin[e] + ii;
        double comm;
        int trans;
        if ((flags & 2) || s_tensor[sp] < 0 || s_tensor[ts] < 0) {
          comm = pt[e_pt_begin[e] + (int64_t)ss * ns + ii];
          trans = 0;
        } else {
          const int t = s_tensor[sp];
          const int r = t_rank[t];
          const int64_t *shape = t_shape + (int64_t)t * ORC_MAX_RANK;
          const int64_t *stride = t_stride + (int64_t)t * ORC_MAX_RANK;
          comm = entry_cost(s_codes[sp], s_codes[ts], tensor_bytes(t_item[t], r, shape),
                            contiguous(r, shape, stride), p);
          trans = (s_codes[sp] != s_codes[ts]) * p->transition_scale;
        }
        if (flags & 1) comm = comm / p->rescale;
        if (comm_out) comm_out[o] = comm;
        if (trans_out) trans_out[o] = (uint8_t)trans;
        if (cost_out) cost_out[o] = comm + per_arg[e_strat_begin[e] + ss] + (double)trans;
      }
    }
  }
}

/* a7: bytes + contiguity per tensor row */
void orc_tensor_tables(int64_t n, const int32_t *t_rank, const int32_t *t_item, const int64_t *t_shape,
                       const int64_t *t_stride, int64_t *bytes, uint8_t *cont) {
  for (int64_t t = 0; t < n; ++t) {
    bytes[t] = tensor_bytes(t_item[t], t_rank[t], t_shape + t * ORC_MAX_RANK);
    cont[t] = (uint8_t)contiguous(t_rank[t], t_shape + t * ORC_MAX_RANK, t_stride + t * ORC_MAX_RANK);
  }
}

/* a8 + num_shards: ref compute_estimation.py:211-229, torch _dtensor_spec.py:555-561 */
void orc_spec_tables(int ndim, const int32_t *mesh, int64_t n, const uint32_t *s_codes,
                     const int32_t *s_tensor, const int32_t *t_rank, const int32_t *t_item,
                     const int64_t *t_shape, const int64_t *t_stride, int64_t *shards,
                     int64_t *lshape, int64_t *lstride, int64_t *lnumel, int64_t *lbytes) {
  for (int64_t s = 0; s < n; ++s) {
    int64_t *osh = lshape + s * ORC_MAX_RANK, *ost = lstride + s * ORC_MAX_RANK;
    memset(osh, 0, sizeof(int64_t) * ORC_MAX_RANK);
    memset(ost, 0, sizeof(int64_t) * ORC_MAX_RANK);
    int t = s_tensor[s];
    if (t < 0) {
      shards[s] = 0;
      lnumel[s] = 0;
      lbytes[s] = 0;
      continue;
    }
    int r = t_rank[t];
    for (int i = 0; i < r; ++i) {
      osh[i] = t_shape[(int64_t)t * ORC_MAX_RANK + i];
      ost[i] = t_stride[(int64_t)t * ORC_MAX_RANK + i];
    }
    int64_t nsh = 1;
    for (int i = 0; i < ndim; ++i) {
      unsigned c = (s_codes[s] >> (8 * i)) & 0xFF;
      if (kind_of(c) == 2) {
        int d = dim_of(c);
        int64_t m = mesh[i];
        nsh *= m;
        osh[d] = (osh[d] + m - 1) / m;
        if (d - 1 > 0) ost[d - 1] = (ost[d - 1] + m - 1) / m;
      }
    }
    shards[s] = nsh;
    int64_t ne = 1;
    for (int i = 0; i < r; ++i) ne *= osh[i];
    lnumel[s] = ne;
    lbytes[s] = ne * t_item[t];
  }
}

/* a14: first-argmin per segment; empty segment -> (+inf, -1) */
void orc_segmented_min(const double *values, const int64_t *seg_ptr, int64_t n_seg, double *mins,
                       int32_t *args) {
  for (int64_t k = 0; k < n_seg; ++k) {
    double best = INFINITY;
    int32_t arg = -1;
    for (int64_t j = seg_ptr[k]; j < seg_ptr[k + 1]; ++j) {
      if (arg < 0 || values[j] < best) {
        best = values[j];
        arg = (int32_t)(j - seg_ptr[k]);
      }
    }
    mins[k] = best;
    args[k] = arg;
  }
}
