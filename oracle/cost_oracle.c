/*
 * CPU oracle in C.  TEST INFRASTRUCTURE ONLY: nothing under autoparallel_amd/
 * links or loads this file; it is the checker (tests) and the compiled CPU
 * baseline beside the GPU figure (bench.py, cpu_baseline leg).
 *
 * Plain-C restatement, per entry and without memo caches, of the reference's
 * default cost path on the packed arrays:
 *   topology              torch/distributed/tensor/_collective_utils.py:246-278
 *   collectives           same file :281-313;
 *                         autoparallel/cost_models/collective_runtime_estimation.py:65-110
 *   redistribute_cost     collective_runtime_estimation.py:115-229, order rule :253-258
 *   contiguity            torch/_prims_common/__init__.py:252-293
 *   read/write time       autoparallel/cost_models/compute_estimation.py:391-403
 *   sharded shapes        compute_estimation.py:300-318
 *   roofline estimate     compute_estimation.py:438-493 (on compute programs)
 *   entry assembly        autoparallel/optimize_sharding.py:446-552
 * Every operation is a separately rounded binary64 operation in the Python's
 * order (build with -ffp-contract=off).
 *
 * Pinning: bit-identical to oracle/cost_oracle.py (itself pinned by the
 * reference's golden vectors) on every test graph: tests/test_oracle_c.py.
 * The NCCL collective model is not restated here (oracle/nccl_oracle.py).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define MAX_MESH 4
#define MAX_RANK 8
#define SPEC_NONE 0xFFFFFFFFu
#define KIND 0xC0
#define SHARD 0x40
#define PARTIAL 0x80
#define ARG 0x3F

typedef struct {
  int32_t ndim;
  int32_t mesh[MAX_MESH];
  double bw[MAX_MESH], lat[MAX_MESH];
  double gmem_bw;
  double tflops[8]; /* by dtype code, <= 0: none */
} oc_model;

typedef struct {
  oc_model m;
  /* metas */
  const int32_t* meta_rank;
  const int64_t* meta_shape;  /* [M][8] */
  const int64_t* meta_stride; /* [M][8] */
  const int32_t* meta_itemsize;
  const int32_t* meta_dtype;
  const uint8_t* tuple_plc; /* [NT][4] */
  const uint32_t* lists;
  /* nodes */
  int32_t n_node;
  const int32_t* node_nstrat;
  const int32_t* node_nargs;
  const int32_t* node_op;
  const int64_t* node_comp_off;
  const int32_t* node_edge_off;
  const int64_t* node_prog_off;
  const int64_t* prog;
  const int64_t* explicit_flops;
  const int64_t* explicit_bytes;
  /* edges */
  const int32_t* edge_src_node;
  const int32_t* edge_ssrc;
  const int32_t* edge_sdst;
  const int64_t* edge_dst_list;
  const int64_t* edge_src_list;
  const int64_t* edge_off;
  const int32_t* edge_flags;
  const int64_t* edge_default_off;
  const double* default_vals;
} oc_graph;

void oc_topology(const int32_t* mesh, int32_t ndim, int32_t devices_per_host, double* bw, double* lat) {
  int64_t total = 1;
  for (int d = 0; d < ndim; ++d) {
    bw[d] = 87.7;
    lat[d] = 0.6;
  }
  for (int d = ndim - 1; d >= 0; --d) {
    total *= mesh[d];
    if (total > devices_per_host) {
      bw[d] *= 0.22;
      lat[d] = 2.7;
    }
  }
}

static double rw_time(double nbytes, double gmem_bw) {
  double t = nbytes / gmem_bw * 1e6;
  t = t / 0.70;
  return t >= 7.0 ? t : 7.0;
}

/* kind: 0 allgather, 1 all_to_all, 2 allreduce, 3 reduce_scatter */
static double collective(const oc_model* m, int kind, int64_t nbytes, int i) {
  double g = (double)nbytes / 1073741824.0;
  int n = m->mesh[i];
  int hops = kind == 2 ? 2 * (n - 1) : n - 1;
  double latency = 6.6 + (double)hops * m->lat[i];
  double bw = (g * (double)hops / (double)n) / m->bw[i];
  double t = latency + bw * 1e6;
  if (kind == 1) t *= 5;
  return t;
}

static int contiguous(const int64_t* shape, const int64_t* stride, int rank) {
  int64_t expected = 1, expected_max = 1;
  for (int d = rank - 1; d >= 0; --d) {
    int64_t x = shape[d], y = stride[d];
    if (x == 1) continue;
    if (y != expected && y != expected_max) return 0;
    expected_max *= x > 1 ? x : 1;
    expected *= x;
  }
  return 1;
}

double oc_redistribute(const oc_model* m, const uint8_t* src, const uint8_t* tgt, const int64_t* shape,
                       const int64_t* stride, int rank, int itemsize, int order_mode) {
  const int nd = m->ndim;
  int all_rep = 1, any_partial_tgt = 0, tgt_all_shard = 1, src_pp = nd == 2;
  for (int i = 0; i < nd; ++i) {
    if (src[i] != 0) all_rep = 0;
    if ((tgt[i] & KIND) == PARTIAL) any_partial_tgt = 1;
    if ((tgt[i] & KIND) != SHARD) tgt_all_shard = 0;
    if (src[i] != PARTIAL) src_pp = 0; /* Partial("sum") on every dim */
  }
  if (all_rep) return any_partial_tgt ? INFINITY : 0.0;
  int64_t numel = 1, shards = 1;
  for (int d = 0; d < rank; ++d) numel *= shape[d];
  for (int i = 0; i < nd; ++i)
    if ((src[i] & KIND) == SHARD) shards *= m->mesh[i];
  double gb = (double)(itemsize * numel) / (double)shards / 1024 / 1024 / 1024;
  int contig = contiguous(shape, stride, rank);
  int reversed = order_mode == 0 ? (src_pp && tgt_all_shard) : order_mode == 2;
  double cost = 0.0;
  for (int s = 0; s < nd; ++s) {
    int i = reversed ? nd - 1 - s : s;
    int cur = src[i], tg = tgt[i];
    if (cur == tg) continue;
    int n = m->mesh[i];
    if (!contig) cost += rw_time(gb * 2 * 1073741824.0, m->gmem_bw);
    int ck = cur & KIND, tk = tg & KIND;
    if (ck == SHARD && tg == 0) {
      gb *= n;
      cost += collective(m, 0, (int64_t)(gb * 1073741824.0), i);
      if ((cur & ARG) != 0) cost += rw_time(gb * 2 * 1073741824.0, m->gmem_bw);
    } else if (ck == SHARD && tk == SHARD) {
      cost += collective(m, 1, (int64_t)(gb * 1073741824.0), i);
      int copies = ((cur & ARG) != 0) + ((tg & ARG) != 0);
      cost += copies * rw_time(gb * 2 * 1073741824.0, m->gmem_bw);
    } else if (ck == PARTIAL && tg == 0) {
      cost += collective(m, 2, (int64_t)(gb * 1073741824.0), i);
    } else if (ck == PARTIAL && tk == SHARD) {
      cost += collective(m, 3, (int64_t)(gb * 1073741824.0), i);
      if ((tg & ARG) != 0) cost += rw_time(gb * 2 * 1073741824.0, m->gmem_bw);
      gb /= n;
    } else if ((ck == SHARD || cur == 0) && tk == PARTIAL) {
      return INFINITY;
    }
    contig = 1;
  }
  return cost;
}

static void local_shape(const oc_graph* g, uint32_t w, int64_t* out, int* rank) {
  uint32_t mid = w >> 12;
  const uint8_t* plc = g->tuple_plc + (size_t)(w & 0xFFF) * 4;
  int r = g->meta_rank[mid];
  for (int d = 0; d < r; ++d) out[d] = g->meta_shape[(size_t)mid * 8 + d];
  for (int i = 0; i < g->m.ndim; ++i)
    if ((plc[i] & KIND) == SHARD) {
      int d = plc[i] & ARG;
      out[d] = (out[d] + g->m.mesh[i] - 1) / g->m.mesh[i];
    }
  *rank = r;
}

/* estimate_strategy_runtime_cost for (node v, strategy o); *bad set if a flop
 * count meets a dtype without a tflops entry */
static double node_compute(const oc_graph* g, int v, int o, int* bad) {
  int op = g->node_op[v];
  if (op == 0) return 0.0;
  int e0 = g->node_edge_off[v], na = g->node_edge_off[v + 1] - e0;
  int64_t shp[64][MAX_RANK];
  int rk[64], isz[64];
  int dtype = 1;
  int have = 0;
  if (na > 64) abort();
  for (int a = 0; a < na; ++a) {
    uint32_t w = g->lists[g->edge_dst_list[e0 + a] + o];
    if (w == SPEC_NONE) {
      rk[a] = -1;
      continue;
    }
    local_shape(g, w, shp[a], &rk[a]);
    isz[a] = g->meta_itemsize[w >> 12];
    if (!have) {
      dtype = g->meta_dtype[w >> 12];
      have = 1;
    }
  }
  int64_t flops = 0, nbytes = 0;
  if (op == 2) {
    flops = g->explicit_flops[g->node_comp_off[v] + o];
    nbytes = g->explicit_bytes[g->node_comp_off[v] + o];
  } else {
    const int64_t* p = g->prog + g->node_prog_off[v];
    int n_terms = (int)p[0], n_outs = (int)p[1];
    p += 2;
    for (int t = 0; t < n_terms; ++t) {
      int64_t term = p[0];
      int nfac = (int)p[1];
      p += 2;
      for (int f = 0; f < nfac; ++f, p += 2) term *= shp[p[0]][p[1]];
      flops += term;
    }
    for (int a = 0; a < na; ++a) {
      if (rk[a] < 0) continue;
      int64_t numel = 1;
      for (int d = 0; d < rk[a]; ++d) numel *= shp[a][d];
      nbytes += numel * isz[a];
    }
    for (int k = 0; k < n_outs; ++k) {
      int64_t osz = p[0];
      int rank = (int)p[1];
      p += 2;
      int64_t numel = 1;
      for (int d = 0; d < rank; ++d, p += 3) {
        int64_t size;
        if (p[0] == 0) {
          size = p[1];
        } else if (p[0] == 1) {
          size = shp[p[1]][p[2]];
        } else if (p[0] == 3) { /* all local sizes of an argument */
          size = 1;
          for (int q = 0; q < rk[p[1]]; ++q) size *= shp[p[1]][q];
        } else {
          size = 1;
          for (int a = 0; a < na; ++a) {
            if (rk[a] < 0 || p[1] >= rk[a]) continue;
            int64_t s = shp[a][rk[a] - 1 - p[1]];
            if (s != 1) size = s;
          }
        }
        numel *= size;
      }
      nbytes += numel * osz;
    }
  }
  double rw = rw_time((double)nbytes, g->m.gmem_bw);
  if (flops == 0) return rw;
  if (dtype < 0 || dtype >= 8 || !(g->m.tflops[dtype] > 0)) {
    *bad = 1;
    return NAN;
  }
  double t = (double)flops / (g->m.tflops[dtype] * 1e12) * 1e6;
  t = t / 0.70;
  return t >= rw ? t : rw;
}

/* All coefficients of nodes [v0, v1): comm, cost (before the inf rewrite) and
 * transition per slot, compute per (node, out_idx).  Returns 0, or 1 if a node
 * needed a dtype without a tflops entry. */
int oc_build(const oc_graph* g, int v0, int v1, int n_threads, double* comm, double* cost, uint8_t* trans,
             double* compute) {
  int bad = 0;
#ifdef _OPENMP
  if (n_threads > 0) omp_set_num_threads(n_threads);
#pragma omp parallel for schedule(dynamic, 4) reduction(| : bad)
#endif
  for (int v = v0; v < v1; ++v) {
    int S = g->node_nstrat[v], nargs = g->node_nargs[v];
    int e0 = g->node_edge_off[v], e1 = g->node_edge_off[v + 1];
    for (int o = 0; o < S; ++o) {
      double cc = node_compute(g, v, o, &bad);
      compute[g->node_comp_off[v] + o] = cc;
      double per_arg = cc / (double)nargs;
      for (int e = e0; e < e1; ++e) {
        int ssrc = g->edge_ssrc[e];
        int64_t base = g->edge_off[e] + (int64_t)o * ssrc;
        uint32_t tw = g->lists[g->edge_dst_list[e] + o];
        for (int j = 0; j < ssrc; ++j) {
          uint32_t sw = (g->edge_flags[e] & 1) ? g->lists[g->edge_src_list[e] + j] : SPEC_NONE;
          double c;
          int t = 0;
          if (sw != SPEC_NONE && tw != SPEC_NONE) {
            uint32_t sm = sw >> 12;
            const uint8_t* sp = g->tuple_plc + (size_t)(sw & 0xFFF) * 4;
            const uint8_t* tp = g->tuple_plc + (size_t)(tw & 0xFFF) * 4;
            c = oc_redistribute(&g->m, sp, tp, g->meta_shape + (size_t)sm * 8, g->meta_stride + (size_t)sm * 8,
                                g->meta_rank[sm], g->meta_itemsize[sm], 0);
            t = memcmp(sp, tp, (size_t)g->m.ndim) != 0;
          } else {
            c = g->default_vals[g->edge_default_off[e] + (int64_t)o * ssrc + j];
          }
          comm[base + j] = c;
          trans[base + j] = (uint8_t)t;
          cost[base + j] = c + per_arg + t;
        }
      }
    }
  }
  return bad;
}
