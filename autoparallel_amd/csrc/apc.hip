// HIP kernels and C ABI of the sharding-search cost engine (gfx950 / CDNA4).
//
// Everything here is HBM-bound integer/fp64 scalar work: no matrix cores.  The
// entry kernel is a flat scan over the E cost entries in work items of 256
// entries of one edge block: a wavefront owns an item, lane L the entries
// L + 64 k, so every load and store instruction covers 64 consecutive entries.
// All floating-point code is compiled with -ffp-contract=off: the reference is
// a chain of separately rounded binary64 operations, and the results here are
// bit-identical to it.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "apc.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, const char* detail = "") {
  snprintf(g_err, sizeof(g_err), fmt, detail);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
    return APC_ERR_LAUNCH;
  }
  return 0;
}

constexpr uint32_t kTupleMask = (1u << APC_TUPLE_BITS) - 1u;
constexpr int kKindMask = 0xC0, kShard = 0x40, kPartial = 0x80, kArgMask = 0x3F;
constexpr int kPartialSum = 0x80;
constexpr int kBlock = 256;

typedef double double2_t __attribute__((ext_vector_type(2)));
typedef long long ll2_t __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------------------
// Cost model, scalar device functions (order of operations is the contract)
// ---------------------------------------------------------------------------

// compute_read_write_time (compute_estimation.py:391-403)
__device__ __forceinline__ double rw_time(double nbytes, double gmem_bw) {
  double t = nbytes / gmem_bw * 1e6;
  t = t / 0.70;
  return t >= 7.0 ? t : 7.0;  // max(t, 7): keeps t on ties, as Python's max
}

// allgather / reduce_scatter / allreduce / all_to_all cost for `nbytes` on
// mesh dim i (torch _collective_utils.py:281-313;
// collective_runtime_estimation.py:100-110).  kind: 0 AG, 1 A2A, 2 AR, 3 RS.
__device__ __forceinline__ int log2i64(int64_t n) {  // _log2i (nccl_cost_model.py:287-291)
  return n <= 0 ? 0 : 63 - __clzll((unsigned long long)n);
}

// _interp_correction (nccl_cost_model.py:294-315): linear interpolation of a
// 24-entry table indexed by log2(nbytes >> 6).  The integer part of the
// logarithm comes from the bit position, the fraction from log2 of the
// mantissa in [1, 2); their sum is rounded once, as the host's log2 result is.
__device__ __forceinline__ double interp_correction(const double* __restrict__ table, int64_t nbytes) {
  const int64_t shifted = nbytes >> 6;
  if (shifted <= 0) return table[0];
  const int lo = log2i64(shifted);
  if (lo + 1 >= APC_NCCL_TABLE_LEN) return table[APC_NCCL_TABLE_LEN - 1];
  const double mant = (double)shifted / (double)(1ll << lo);
  const double lv = (double)lo + log2(mant);
  const double frac = lv - (double)lo;
  return table[lo] * (1.0 - frac) + table[lo + 1] * frac;
}

// nccl_collective_time / nccl_all_to_all_cost (nccl_cost_model.py:1163-1313):
// minimum over the candidates the host resolved for (mesh dim, collective),
// each with its message-size corrections (_nccl_algo_time :577-613,
// _table_algo_time :1035-1075).
__device__ double nccl_collective_cost(int kind, int64_t nbytes, int i,
                                       const apc_nccl_plan* __restrict__ plan) {
  const apc_nccl_dim& d = plan->dim[i];
  const int nc = d.n_cand[kind];
  double best = INFINITY;
  for (int c = 0; c < nc; ++c) {
    const apc_nccl_cand& k = d.cand[kind][c];
    double bw = k.bw, lat = k.lat, t;
    const int f = k.flags;
    if (f & APC_NC_NIC) {
      const int lg = log2i64((nbytes / d.n_ranks) >> 6);
      double corr = lg < APC_NCCL_TABLE_LEN ? plan->a2a_nic_ramp[lg] : 1.0;
      if (d.a2a_log_nodes > 1 && corr < 1.0) corr = 1.0 - (1.0 - corr) / (double)d.a2a_log_nodes;
      t = lat + (double)nbytes * d.a2a_remote / (1000.0 * bw * corr);
    } else {
      if (f & (APC_NC_TREE_CORR | APC_NC_TREE_CORR24)) {
        const int ls = log2i64(nbytes >> 6);
        if (ls < ((f & APC_NC_TREE_CORR24) ? 24 : 23)) bw *= plan->tree_corr[k.proto][ls];
      }
      if (f & (APC_NC_RING_CORR | APC_NC_NVLS_RAMP | APC_NC_FULL_MESH_RAMP)) {
        const int64_t per_rank = nbytes / d.n_ranks;
        if (f & APC_NC_RING_CORR) bw *= interp_correction(d.ring_corr, per_rank);
        if (f & APC_NC_NVLS_RAMP) bw *= interp_correction(plan->nvls_tree_ramp, per_rank);
        if ((f & APC_NC_FULL_MESH_RAMP) && log2i64(per_rank >> 6) < APC_NCCL_TABLE_LEN)
          bw *= interp_correction(plan->full_mesh_ramp, per_rank);
      }
      if ((f & APC_NC_PLATEAU) && (double)nbytes / (double)(d.n_channels * d.n_ranks) >= 64.0) lat *= 1.4;
      t = lat + (double)nbytes / (1000.0 * bw);
    }
    best = t < best ? t : best;
  }
  return best;
}

__device__ __forceinline__ double collective_cost(int kind, int64_t nbytes, int i,
                                                  const apc_model& m) {
  if (m.nccl_plan != nullptr) return nccl_collective_cost(kind, nbytes, i, m.nccl_plan);
  double g = (double)nbytes / 1073741824.0;
  int n = m.mesh_shape[i];
  int hops = (kind == 2) ? 2 * (n - 1) : (n - 1);
  double latency = 6.6 + (double)hops * m.mesh_lat[i];
  double bw = (g * (double)hops / (double)n) / m.mesh_bw[i];
  double t = latency + bw * 1e6;
  if (kind == 1) t = t * 5.0;
  return t;
}

// redistribute_cost with estimate_strategy_comms_cost's order rule
// (collective_runtime_estimation.py:115-229, 253-258).  src/tgt: placement
// bytes packed little-endian, one per mesh dim.
__device__ double redistribute_cost(uint32_t src, uint32_t tgt, int64_t tensor_bytes,
                                    bool contiguous, const apc_model& m) {
  const int ndim = m.ndim;
  if (src == 0u) {  // source fully replicated
    bool any_partial = false;
    for (int i = 0; i < ndim; ++i)
      any_partial |= (((tgt >> (8 * i)) & kKindMask) == kPartial);
    return any_partial ? INFINITY : 0.0;
  }
  int64_t num_shards = 1;
  bool tgt_all_shard = true;
  for (int i = 0; i < ndim; ++i) {
    if (((src >> (8 * i)) & kKindMask) == kShard) num_shards *= m.mesh_shape[i];
    tgt_all_shard &= (((tgt >> (8 * i)) & kKindMask) == kShard);
  }
  double gb = (double)tensor_bytes / (double)num_shards / 1024.0 / 1024.0 / 1024.0;
  // order rule of estimate_strategy_comms_cost (:253-258), or an order forced by
  // the caller of redistribute_cost (order_mode 1: 0..ndim-1, 2: ndim-1..0)
  const bool reversed =
      m.order_mode == 0
          ? ((ndim == 2) && (src == (uint32_t)(kPartialSum | (kPartialSum << 8))) && tgt_all_shard)
          : (m.order_mode == 2);
  double cost = 0.0;
  for (int step = 0; step < ndim; ++step) {
    const int i = reversed ? (ndim - 1 - step) : step;
    const int cur = (src >> (8 * i)) & 0xFF, tg = (tgt >> (8 * i)) & 0xFF;
    if (cur == tg) continue;
    const int n = m.mesh_shape[i];
    if (!contiguous) cost += rw_time(gb * 2.0 * 1073741824.0, m.gmem_bw);
    const int ck = cur & kKindMask, tk = tg & kKindMask;
    if (ck == kShard && tg == 0) {
      gb = gb * (double)n;
      cost += collective_cost(0, (int64_t)(gb * 1073741824.0), i, m);
      if ((cur & kArgMask) != 0) cost += rw_time(gb * 2.0 * 1073741824.0, m.gmem_bw);
    } else if (ck == kShard && tk == kShard) {
      cost += collective_cost(1, (int64_t)(gb * 1073741824.0), i, m);
      int copies = ((cur & kArgMask) != 0) + ((tg & kArgMask) != 0);
      cost += (double)copies * rw_time(gb * 2.0 * 1073741824.0, m.gmem_bw);
    } else if (ck == kPartial && tg == 0) {
      cost += collective_cost(2, (int64_t)(gb * 1073741824.0), i, m);
    } else if (ck == kPartial && tk == kShard) {
      cost += collective_cost(3, (int64_t)(gb * 1073741824.0), i, m);
      if ((tg & kArgMask) != 0) cost += rw_time(gb * 2.0 * 1073741824.0, m.gmem_bw);
      gb = gb / (double)n;
    } else if (ck == kShard && tk == kPartial) {
      return INFINITY;
    } else if (cur == 0 && tk == kPartial) {
      return INFINITY;
    }
    contiguous = true;
  }
  return cost;
}

__device__ __forceinline__ uint32_t load_tuple(const uint8_t* tuple_plc, uint32_t t) {
  return *reinterpret_cast<const uint32_t*>(tuple_plc + (size_t)t * APC_MAX_MESH_DIMS);
}

// itemsize * prod(shape) and contiguity of tensor meta `mid`.  Both rows are
// fetched with unconditional 16-byte loads before any element is used, so the
// lane pays one memory latency, not one per dimension.
__device__ __forceinline__ void meta_bytes_contig(const apc_problem& p, uint32_t mid,
                                                  int64_t& nbytes, bool& contiguous) {
  const int rank = p.meta_rank[mid];
  const int64_t isz = p.meta_itemsize[mid];
  const ll2_t* sh = reinterpret_cast<const ll2_t*>(p.meta_shape + (size_t)mid * APC_MAX_RANK);
  const ll2_t* st = reinterpret_cast<const ll2_t*>(p.meta_stride + (size_t)mid * APC_MAX_RANK);
  ll2_t shape[APC_MAX_RANK / 2], stride[APC_MAX_RANK / 2];
#pragma unroll
  for (int q = 0; q < APC_MAX_RANK / 2; ++q) { shape[q] = sh[q]; stride[q] = st[q]; }
  int64_t b = isz, expected = 1, expected_max = 1;
  bool ok = true;
#pragma unroll
  for (int d = APC_MAX_RANK - 1; d >= 0; --d) {
    if (d >= rank) continue;
    const int64_t x = (d & 1) ? shape[d >> 1].y : shape[d >> 1].x;
    const int64_t y = (d & 1) ? stride[d >> 1].y : stride[d >> 1].x;
    b *= x;
    // check_contiguous_sizes_strides (torch _prims_common/__init__.py:252-293)
    if (x != 1) {
      if (y != expected && y != expected_max) ok = false;
      expected_max *= (x > 1 ? x : 1);
      expected *= x;
    }
  }
  nbytes = b;
  contiguous = ok;
}

__device__ __forceinline__ int64_t ceil_div_pos(int64_t s, int64_t n) {
  // sizes are almost always below 2^31: a 32-bit divide is several times cheaper
  if (s <= 0x7FFFFFFF && n <= 0x7FFFFFFF)
    return (int64_t)(((uint32_t)s + (uint32_t)n - 1u) / (uint32_t)n);
  return (s + n - 1) / n;
}

// ---------------------------------------------------------------------------
// Kernel: pair table T[m][src tuple][tgt tuple] and node compute estimate
// ---------------------------------------------------------------------------
// Local size of dim d of the tensor behind spec word w: the global size, ceil-
// divided by each mesh dim that shards d, in mesh-dim order
// (_get_sharded_shape_stride, compute_estimation.py:300-318).
__device__ __forceinline__ int64_t local_size(const apc_problem& p, uint32_t w, int d) {
  if (w == APC_SPEC_NONE) return 1;  // a program never names a non-tensor arg
  const uint32_t mid = w >> APC_TUPLE_BITS;
  int64_t s = p.meta_shape[(size_t)mid * APC_MAX_RANK + d];
  const uint32_t plc = load_tuple(p.tuple_plc, w & kTupleMask);
  for (int i = 0; i < p.model.ndim; ++i) {
    const int c = (plc >> (8 * i)) & 0xFF;
    if ((c & kKindMask) == kShard && (c & kArgMask) == d)
      s = ceil_div_pos(s, p.model.mesh_shape[i]);
  }
  return s;
}

// Roofline tail of estimate_strategy_runtime_cost (compute_estimation.py:474-489).
__device__ __forceinline__ double roofline(const apc_problem& p, int64_t flops, int64_t nbytes,
                                           int dtype, int32_t* __restrict__ status) {
  const double rw = rw_time((double)nbytes, p.model.gmem_bw);
  if (flops == 0) return rw;
  const double tf = (dtype >= 0 && dtype < APC_NUM_DTYPES) ? p.model.tflops[dtype] : 0.0;
  if (!(tf > 0.0)) {
    atomicExch(status, 1);
    return NAN;
  }
  const double gpu_flops = tf * 1e12;
  double ct = (double)flops / gpu_flops * 1e6;
  ct = ct / 0.70;
  return ct >= rw ? ct : rw;  // max(ct, rw): keeps ct on ties
}

constexpr int kNodesPerBlock = 2;  // one wavefront each; the other wavefronts of a node block exit at once:
                                   // the block table's blocks share the launch and its LDS size per block,
                                   // which decides how many of them a CU holds
constexpr int kFusedTableBlocks = 2048;  // larger tables are built by a launch of their own
constexpr int kProgCache = 128;    // int64 words of program staged per wave
constexpr int kRecWords = 8;       // int64 words of LDS for the record's argument runs
static_assert(kRecWords * 2 >= APC_REC_ARGS && sizeof(apc_comp_rec) == 96, "record layout");

// One wavefront per 64 strategies of an evaluated node.  Phase 1: the lanes split the node's
// (strategy, argument) pairs and write each argument's local (sharded) sizes
// to LDS as local[arg][dim][strategy-slot]; all loads of a pair are issued
// together.  Phase 2: one lane per strategy interprets the node's compute
// program out of LDS.  A wavefront handles the 64 strategies from o0; a node
// with more strategies is split over several wavefronts.  `slow` (the LDS
// layout does not fit) reads sizes from memory on demand instead.
// The record of evaluated node i: read as it is, or gathered from the node
// arrays when the caller keeps none.
__device__ __forceinline__ apc_comp_rec load_comp_rec(const apc_problem& p, int i) {
  if (p.comp_recs) return p.comp_recs[i];
  apc_comp_rec r;
  const int v = __builtin_amdgcn_readfirstlane(p.comp_nodes[i]);
  r.node = v;
  r.nstrat = p.node_nstrat[v];
  r.nargs = p.node_nargs[v];
  r.op = p.node_op[v];
  r.comp_off = p.node_comp_off[v];
  r.prog_off = p.node_prog_off[v];
  r.prog_len = p.node_prog_len[v];
  const int e0 = p.node_edge_off[v];
  r.n_edge = p.node_edge_off[v + 1] - e0;
#pragma unroll
  for (int a = 0; a < APC_REC_ARGS; ++a) r.dst_list[a] = a < r.n_edge ? p.edges[e0 + a].dst_list : 0u;
  return r;
}

__device__ __forceinline__ void node_compute_wave(const apc_problem& p, const apc_comp_rec& rec,
                                                  int o0, int lane, int64_t* __restrict__ s_prog,
                                                  uint32_t* __restrict__ s_dst,
                                                  int64_t* __restrict__ s_local, bool slow,
                                                  double* __restrict__ compute,
                                                  double* __restrict__ per_arg,
                                                  int32_t* __restrict__ status) {
  const int S = rec.nstrat;
  const int64_t base = rec.comp_off;
  const int nargs = rec.nargs;
  const int op = rec.op;
  if (o0 >= S) return;  // wave-uniform
  if (op == APC_OP_ZERO) {
    const int o = o0 + lane;
    if (o < S) {
      compute[base + o] = 0.0;
      per_arg[base + o] = 0.0 / (double)nargs;
    }
    return;
  }
  const int na = rec.n_edge;
  // lanes look the run of an argument up by a lane-varying index: through LDS
  if (lane == 0) {  // constant indices: the record stays in scalar registers
#pragma unroll
    for (int a = 0; a < APC_REC_ARGS; ++a) s_dst[a] = rec.dst_list[a];
  }
  const int e0 = na > APC_REC_ARGS ? p.node_edge_off[rec.node] : 0;  // only for the arguments past the record
  auto dst_of = [&](int a) -> uint32_t {
    return a < APC_REC_ARGS ? s_dst[a] : p.edges[e0 + a].dst_list;
  };
  const int max_rank = p.max_rank;
  const int slots = max_rank + 2;  // per argument: max_rank sizes, an info word, its local bytes
  // program words: loaded now, parked in LDS after the argument loads below are
  // on their way
  const int64_t* prog = nullptr;
  int64_t pw0 = 0, pw1 = 0;
  bool cached = false;
  if (op == APC_OP_PROGRAM) {
    prog = p.prog + rec.prog_off;
    cached = rec.prog_len <= kProgCache;
    if (cached) {
      if (lane < rec.prog_len) pw0 = prog[lane];
      if (lane + 64 < rec.prog_len) pw1 = prog[lane + 64];
    }
  }
  {
    const int chunk = (S - o0 < 64) ? (S - o0) : 64;
    if (!slow && op == APC_OP_PROGRAM) {
      for (int t = lane; t < chunk * na; t += 64) {
        const int a = t / chunk, oo = t - a * chunk;
        const uint32_t w = p.lists[(size_t)dst_of(a) + o0 + oo];
        const bool none = (w == APC_SPEC_NONE);
        const uint32_t mid = none ? 0u : (w >> APC_TUPLE_BITS);
        const int rank = none ? 0 : p.meta_rank[mid];
        const uint32_t plc = load_tuple(p.tuple_plc, none ? 0u : (w & kTupleMask));
        const ll2_t* r = reinterpret_cast<const ll2_t*>(p.meta_shape + (size_t)mid * APC_MAX_RANK);
        ll2_t row[APC_MAX_RANK / 2];
#pragma unroll
        for (int q = 0; q < APC_MAX_RANK / 2; ++q) row[q] = r[q];
        int64_t numel = 1;
#pragma unroll
        for (int d = 0; d < APC_MAX_RANK; ++d) {
          if (d >= max_rank) break;  // wave-uniform
          int64_t sz = (d & 1) ? row[d >> 1].y : row[d >> 1].x;
          if (d >= rank) {
            sz = 1;
          } else {
            for (int i = 0; i < p.model.ndim; ++i) {
              const int c = (plc >> (8 * i)) & 0xFF;
              if ((c & kKindMask) == kShard && (c & kArgMask) == d)
                sz = ceil_div_pos(sz, p.model.mesh_shape[i]);
            }
          }
          s_local[(a * slots + d) * 64 + oo] = sz;
          numel *= sz;  // sizes past the rank are 1
        }
        // info word: rank | itemsize << 8 | dtype << 40, or -1 for a missing spec
        const int64_t isz = p.meta_itemsize[mid];
        s_local[(a * slots + max_rank) * 64 + oo] =
            none ? -1 : ((int64_t)rank | (isz << 8) | ((int64_t)p.meta_dtype[mid] << 40));
        // numel * itemsize of the local tensor, formed here where the sizes are
        // in registers: phase 2 adds one word per argument
        s_local[(a * slots + max_rank + 1) * 64 + oo] = numel * isz;
      }
    }
    if (cached) {  // LDS operations of one wave execute in order
      if (lane < rec.prog_len) s_prog[lane] = pw0;
      if (lane + 64 < rec.prog_len) s_prog[lane + 64] = pw1;
      prog = s_prog;
    }
    const int o = o0 + lane;
    if (lane >= chunk) return;
    const int64_t idx = base + o;
    int64_t flops = 0, nbytes = 0;
    int dtype = 1;  // float32 when the node has no tensor argument
    bool have_dtype = false;
    const bool staged = !slow && op == APC_OP_PROGRAM;
    auto size_of = [&](int a, int d) -> int64_t {
      if (staged) return s_local[(a * slots + d) * 64 + lane];
      return local_size(p, p.lists[(size_t)dst_of(a) + o], d);
    };
    // rank of argument a, or -1 if it has no spec
    auto rank_of = [&](int a) -> int {
      if (staged) {
        const int64_t info = s_local[(a * slots + max_rank) * 64 + lane];
        return info < 0 ? -1 : (int)(info & 0xFF);
      }
      const uint32_t w = p.lists[(size_t)dst_of(a) + o];
      return w == APC_SPEC_NONE ? -1 : p.meta_rank[w >> APC_TUPLE_BITS];
    };
    for (int a = 0; a < na; ++a) {
      int rank, isz, dt;
      if (staged) {
        const int64_t info = s_local[(a * slots + max_rank) * 64 + lane];
        if (info < 0) continue;
        if (!have_dtype) { dtype = (int)(info >> 40); have_dtype = true; }
        nbytes += s_local[(a * slots + max_rank + 1) * 64 + lane];
        continue;
      } else {
        const uint32_t w = p.lists[(size_t)dst_of(a) + o];
        if (w == APC_SPEC_NONE) continue;
        const uint32_t mid = w >> APC_TUPLE_BITS;
        rank = p.meta_rank[mid];
        isz = p.meta_itemsize[mid];
        dt = p.meta_dtype[mid];
      }
      if (!have_dtype) { dtype = dt; have_dtype = true; }
      if (op != APC_OP_PROGRAM) continue;
      int64_t numel = 1;
      for (int d = 0; d < rank; ++d) numel *= size_of(a, d);
      nbytes += numel * (int64_t)isz;
    }
    if (op == APC_OP_EXPLICIT) {
      flops = p.explicit_flops[idx];
      nbytes = p.explicit_bytes[idx];
    } else {
      const int64_t* pr = prog;
      const int n_terms = (int)pr[0], n_outs = (int)pr[1];
      pr += 2;
      for (int t = 0; t < n_terms; ++t) {
        int64_t term = pr[0];
        const int nfac = (int)pr[1];
        pr += 2;
        for (int f = 0; f < nfac; ++f) {
          term *= size_of((int)pr[0], (int)pr[1]);
          pr += 2;
        }
        flops += term;
      }
      for (int k = 0; k < n_outs; ++k) {
        const int64_t isz = pr[0];
        const int rank = (int)pr[1];
        pr += 2;
        int64_t numel = 1;
        for (int d = 0; d < rank; ++d) {
          const int kind = (int)pr[0];
          int64_t size;
          if (kind == 0) {
            size = pr[1];
          } else if (kind == 1) {
            size = size_of((int)pr[1], (int)pr[2]);
          } else {  // broadcast of all tensor args at a right-aligned position
            size = 1;
            const int pos = (int)pr[1];
            for (int a = 0; a < na; ++a) {
              const int r = rank_of(a);
              if (pos >= r) continue;
              const int64_t sz = size_of(a, r - 1 - pos);
              if (sz != 1) size = sz;
            }
          }
          numel *= size;
          pr += 3;
        }
        nbytes += numel * isz;
      }
    }
    const double result = roofline(p, flops, nbytes, dtype, status);
    compute[idx] = result;
    per_arg[idx] = result / (double)nargs;
  }
}

// Touch `bytes` of an array (capped) so that the dependent loads that follow
// find it in L2: the entry arrays stream through L2 between two builds and evict
// the small tables.  One 4-byte load per 128-byte line per lane, results kept
// alive but unused.
__device__ __forceinline__ uint32_t warm_lines(const void* base, int64_t bytes, int lane,
                                               int lanes) {
  const int64_t cap = bytes < (1 << 16) ? bytes : (1 << 16);
  uint32_t acc = 0;
  for (int64_t off = (int64_t)lane * 128; off + 4 <= cap; off += (int64_t)lanes * 128)
    acc ^= *reinterpret_cast<const uint32_t*>(reinterpret_cast<const char*>(base) + off);
  return acc;
}

__device__ __forceinline__ uint32_t warm_problem(const apc_problem& p, int lane, int lanes) {
  uint32_t acc = 0;
  if (p.n_list) acc ^= warm_lines(p.lists, p.n_list * 4, lane, lanes);
  if (p.n_meta) {
    acc ^= warm_lines(p.meta_shape, (int64_t)p.n_meta * APC_MAX_RANK * 8, lane, lanes);
    acc ^= warm_lines(p.meta_stride, (int64_t)p.n_meta * APC_MAX_RANK * 8, lane, lanes);
    acc ^= warm_lines(p.meta_rank, (int64_t)p.n_meta * 4, lane, lanes);
    acc ^= warm_lines(p.meta_itemsize, (int64_t)p.n_meta * 4, lane, lanes);
    acc ^= warm_lines(p.meta_dtype, (int64_t)p.n_meta * 4, lane, lanes);
  }
  if (p.n_tuple) acc ^= warm_lines(p.tuple_plc, (int64_t)p.n_tuple * APC_MAX_MESH_DIMS, lane, lanes);
  return acc;
}

// Block table.  Edges whose producer run and consumer run are the same spec
// words have the same S_dst x S_src matrix of redistribution costs; one copy of
// each distinct matrix is kept, in the edge block's own [out_idx][inp_idx]
// order, padded to a multiple of 256 elements so that a workgroup works on one
// matrix.  An edge with a producer and a missing spec has a matrix of its own
// (the missing positions hold its default values).  An element is the cost
// with its sign bit set when the two placements differ (costs are never
// negative, so the sign is free to carry the transition flag): the entry kernel
// reads comm and transition with one coalesced load and no spec words.
template <bool kWarm>
__device__ __forceinline__ void pair_table_block(const apc_problem& p, double* __restrict__ table,
                                                 int unit) {
  const uint32_t keep = kWarm ? warm_problem(p, threadIdx.x, blockDim.x) : 0u;
  const int b = p.table_unit_block[unit];
  const int64_t base = p.block_off[b];
  const apc_edge ed = p.edges[p.block_edge[b]];  // any edge with this matrix
  // a compressed matrix has one column / row per distinct word of the two runs
  const bool squeezed = (ed.flags & APC_EDGE_COMPRESSED) != 0;
  const uint32_t ncol = squeezed ? (uint32_t)ed.flags >> APC_EDGE_USRC_SHIFT : (uint32_t)ed.ssrc;
  const uint32_t nrow = squeezed ? (uint32_t)p.block_udst[b] : (uint32_t)ed.sdst;
  const int64_t l64 = (int64_t)unit * 256 - base + threadIdx.x;
  if (l64 < (int64_t)ncol * nrow) {
    const uint32_t l = (uint32_t)l64;
    uint32_t o = l / ncol, j = l - o * ncol;
    if (squeezed) {  // position in its run of an occurrence of that word
      o = (uint32_t)p.list_ufirst[(size_t)ed.dst_list + o];
      j = (uint32_t)p.list_ufirst[(size_t)ed.src_list + j];
    }
    const uint32_t sw = p.lists[(size_t)ed.src_list + j];
    const uint32_t tw = p.lists[(size_t)ed.dst_list + o];
    if (sw != APC_SPEC_NONE && tw != APC_SPEC_NONE) {
      const uint32_t st = sw & kTupleMask, tt = tw & kTupleMask;
      int64_t nbytes;
      bool contig;
      meta_bytes_contig(p, sw >> APC_TUPLE_BITS, nbytes, contig);
      const double c = redistribute_cost(load_tuple(p.tuple_plc, st), load_tuple(p.tuple_plc, tt),
                                         nbytes, contig, p.model);
      table[base + l] = (st != tt) ? -c : c;
    } else {  // a missing spec keeps the default row's value and is no transition
      table[base + l] = p.default_vals[ed.default_off + (int64_t)l];  // never squeezed
    }
  }
  asm volatile("" ::"v"(keep));
}

// Blocks [0, table_blocks) fill the pair table, the rest price the nodes of
// comp_nodes: the two are independent, and one launch saves a dispatch on a
// problem this small.  Dynamic LDS: per wave kProgCache words of program, then
// (unless slow) max_node_args * (max_rank + 2) * 64 words of local sizes, local bytes and
// argument info.
__global__ void __launch_bounds__(256)
prepare_kernel(apc_problem p, double* __restrict__ table, int table_blocks, int slow,
               double* __restrict__ compute, double* __restrict__ per_arg,
               int32_t* __restrict__ status) {
  extern __shared__ int64_t s_dyn[];
  if ((int)blockIdx.x < table_blocks) {
    pair_table_block<true>(p, table, blockIdx.x);
    return;
  }
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (wave >= kNodesPerBlock) return;
  const int unit = ((int)blockIdx.x - table_blocks) * kNodesPerBlock + wave;
  const int chunks = (p.max_nstrat + 63) >> 6;  // wavefronts per node
  const int i = unit / chunks;
  if (i >= p.n_comp_node) return;
  const apc_comp_rec rec = load_comp_rec(p, i);
  const int per_wave = kProgCache + kRecWords + (slow ? 0 : p.max_node_args * (p.max_rank + 2) * 64);
  int64_t* s_prog = s_dyn + (size_t)wave * per_wave;
  node_compute_wave(p, rec, (unit - i * chunks) * 64, threadIdx.x & 63, s_prog,
                    reinterpret_cast<uint32_t*>(s_prog + kProgCache), s_prog + kProgCache + kRecWords,
                    slow != 0, compute, per_arg, status);
}

// The block table alone, for tables of many units: no dynamic LDS (which in
// prepare_kernel limits the blocks per CU to what the node wavefronts need) and
// no cache warming (thousands of blocks keep the descriptor arrays in L2 by
// themselves).
__global__ void __launch_bounds__(256)
pair_table_kernel(apc_problem p, double* __restrict__ table) {
  pair_table_block<false>(p, table, blockIdx.x);
}

// ---------------------------------------------------------------------------
// Kernel: cost entries
// ---------------------------------------------------------------------------
constexpr int kPerLane = 4;  // entries per lane of a work item of APC_ITEM_ENTRIES entries
static_assert(sizeof(apc_edge) == 64, "edge record layout");
static_assert(64 * kPerLane == APC_ITEM_ENTRIES, "work items are built for this kernel");

// Edge that owns slot idx.  Edge blocks start on multiples of 16 slots, so each
// 16-slot chunk belongs to exactly one edge.
__device__ __forceinline__ apc_edge find_edge(const apc_problem& p, int64_t idx) {
  return p.edges[p.chunk_edge[idx >> APC_CHUNK_SHIFT]];
}

// comm / transition of one entry, general path (direct evaluation, missing
// specs, default rows).
__device__ __forceinline__ void eval_entry(const apc_problem& p, const apc_edge& ed, uint32_t o,
                                           uint32_t j, double& comm, int& trans) {
  const uint32_t tw = p.lists[(size_t)ed.dst_list + o];
  const uint32_t sw =
      (ed.flags & APC_EDGE_HAS_PRODUCER) ? p.lists[(size_t)ed.src_list + j] : APC_SPEC_NONE;
  if (sw != APC_SPEC_NONE && tw != APC_SPEC_NONE) {
    const uint32_t st = sw & kTupleMask, tt = tw & kTupleMask, sm = sw >> APC_TUPLE_BITS;
    trans = (st != tt);
    int64_t nbytes;
    bool contig;
    meta_bytes_contig(p, sm, nbytes, contig);
    comm = redistribute_cost(load_tuple(p.tuple_plc, st), load_tuple(p.tuple_plc, tt), nbytes,
                             contig, p.model);
  } else {
    comm = p.default_vals[ed.default_off + (int64_t)o * ed.ssrc + j];
    trans = 0;
  }
}

// Entries [local0, local0 + 256) of one edge block: lane L owns entries
// local0 + L + 64 k, k < 4, so that every load and store instruction of the
// wavefront touches 64 consecutive entries (512 contiguous bytes of fp64):
// measured on MI355X, stores whose 64 lanes cover one contiguous span stream
// about 20% faster than lanes owning 32 contiguous bytes each.  The item record
// is a copy of the edge record (plus local0), wave-uniform, so it lives in
// scalar registers.  Without a block table every entry is evaluated directly
// from its two spec words.
__device__ __forceinline__ void process_item(const apc_problem& p, const apc_edge& ed, int lane,
                                             const double* __restrict__ per_arg,
                                             double* __restrict__ comm, double* __restrict__ cost,
                                             uint8_t* __restrict__ flags, int clamp_inf) {
  const uint32_t ssrc = (uint32_t)ed.ssrc;
  const uint32_t size = ssrc * (uint32_t)ed.sdst;

  uint32_t lk[kPerLane], ok[kPerLane], jk[kPerLane];
  bool live[kPerLane];
#pragma unroll
  for (int k = 0; k < kPerLane; ++k) {
    lk[k] = ed.local0 + (uint32_t)(k * 64 + lane);
    live[k] = lk[k] < size;
    const uint32_t l = live[k] ? lk[k] : 0u;
    ok[k] = ed.magic ? __umulhi(l, ed.magic) : l / ssrc;
    jk[k] = l - ok[k] * ssrc;
  }
  double v_comm[kPerLane], v_pa[kPerLane];
  int v_trans[kPerLane];
#pragma unroll
  for (int k = 0; k < kPerLane; ++k) {
    v_comm[k] = 0.0; v_pa[k] = 0.0; v_trans[k] = 0;
    if (live[k]) {
      eval_entry(p, ed, ok[k], jk[k], v_comm[k], v_trans[k]);
      v_pa[k] = per_arg[ed.comp_base + ok[k]];
    }
  }
  // ---- assemble (optimize_sharding.py:544) and store
#pragma unroll
  for (int k = 0; k < kPerLane; ++k) {
    double c = (v_comm[k] + v_pa[k]) + (double)v_trans[k];
    const bool finite = isfinite(c);
    if (clamp_inf && !finite) c = 10000.0;
    if (live[k]) {
      const int64_t idx = ed.off + lk[k];
      if (comm) comm[idx] = v_comm[k];
      if (cost) cost[idx] = c;
      if (flags) flags[idx] = (uint8_t)(v_trans[k] | (finite ? 0 : APC_ENTRY_NONFINITE));
    }
  }
}

// Table path.  A lane loads, per entry, one element of the edge's matrix (cost
// and transition flag of the entry's position: same order as the output, so
// the reads coalesce exactly like the stores) and the per-arg compute term of
// its row, adds and stores; no spec word is read.  The matrix of an edge with a
// producer is in the block table; an edge without one has no specs to compare,
// and its matrix is its rows of default_vals as they are.  Split in two so that
// the loads of a wave's next item are in flight while the current item is
// stored.  The kernel needs a third of the registers of the direct one, which
// is why the two do not share a body: eight waves per SIMD instead of three.
// Work items of the table path hold 256 or 512 entries (apc_problem.item_entries):
// measured on MI355X, 256 is faster while the whole launch is a few tens of
// microseconds (more wavefronts to spread), 512 from some tens of millions of
// entries on (half the wavefronts, twice the bytes in flight per wavefront:
// 1.44 ms against 1.67 ms at 418 M entries).
template <int kN>
struct ItemLoads {
  double raw[kN];
  double pa[kN];
  uint32_t lk[kN];
  uint32_t live;  // bit k: entry k of this lane exists
};

template <bool kSqueezed, int kN>
__device__ __forceinline__ void item_load(const apc_edge& ed, int lane, const double* __restrict__ table,
                                          const double* __restrict__ default_vals,
                                          const int32_t* __restrict__ list_uidx,
                                          const double* __restrict__ per_arg, ItemLoads<kN>& r) {
  const uint32_t ssrc = (uint32_t)ed.ssrc;
  const uint32_t size = ssrc * (uint32_t)ed.sdst;
  const double* __restrict__ matrix =  // wave-uniform
      ed.table_off >= 0 ? table + ed.table_off : default_vals + ed.default_off;
  r.live = 0;
  uint32_t lv[kN], ov[kN];
#pragma unroll
  for (int k = 0; k < kN; ++k) {
    r.lk[k] = ed.local0 + (uint32_t)(k * 64 + lane);
    const bool live = r.lk[k] < size;
    r.live |= (uint32_t)live << k;
    lv[k] = live ? r.lk[k] : 0u;
    ov[k] = ed.magic ? __umulhi(lv[k], ed.magic) : lv[k] / ssrc;
    r.pa[k] = per_arg[ed.comp_base + ov[k]];
  }
  if (kSqueezed && (ed.flags & APC_EDGE_COMPRESSED)) {  // wave-uniform
    // the matrix has one row / column per distinct spec word of the two runs:
    // two index loads, then a gather inside the (cache-resident) matrix
    const uint32_t usrc = (uint32_t)ed.flags >> APC_EDGE_USRC_SHIFT;
    uint32_t at[kN];
#pragma unroll
    for (int k = 0; k < kN; ++k) {
      const uint32_t uo = (uint32_t)list_uidx[(size_t)ed.dst_list + ov[k]];
      const uint32_t uj = (uint32_t)list_uidx[(size_t)ed.src_list + (lv[k] - ov[k] * ssrc)];
      at[k] = uo * usrc + uj;
    }
#pragma unroll
    for (int k = 0; k < kN; ++k) r.raw[k] = matrix[at[k]];
  } else {
#pragma unroll
    for (int k = 0; k < kN; ++k) r.raw[k] = matrix[lv[k]];
  }
}

template <int kN>
__device__ __forceinline__ void item_store(const apc_edge& ed, const ItemLoads<kN>& r,
                                           double* __restrict__ comm, double* __restrict__ cost,
                                           uint8_t* __restrict__ flags, int clamp_inf) {
#pragma unroll
  for (int k = 0; k < kN; ++k) {
    const int trans = (int)((uint64_t)__double_as_longlong(r.raw[k]) >> 63);
    const double cm = fabs(r.raw[k]);
    double c = (cm + r.pa[k]) + (double)trans;  // optimize_sharding.py:544
    const bool finite = isfinite(c);
    if (clamp_inf && !finite) c = 10000.0;
    if ((r.live >> k) & 1) {
      const int64_t idx = ed.off + r.lk[k];
      if (comm) comm[idx] = cm;
      if (cost) cost[idx] = c;
      // byte stores: gathering a lane's four flags into one 4-byte store through
      // cross-lane exchanges measured slower
      if (flags) flags[idx] = (uint8_t)(trans | (finite ? 0 : APC_ENTRY_NONFINITE));
    }
  }
}

// Wave w takes items w, w + W, w + 2W, ... (W = waves in the grid, which the
// launcher caps).
// kMode 0: direct evaluation; 1: block table; 2: block table with compressed matrices.
// kN: entries per lane of a work item (table modes; the direct path has 4).
template <int kMode, int kN>
__global__ void __launch_bounds__(kBlock)
edge_cost_kernel(apc_problem p, const double* __restrict__ table,
                 const double* __restrict__ per_arg, double* __restrict__ comm,
                 double* __restrict__ cost, uint8_t* __restrict__ flags, int clamp_inf) {
  const int n_waves = gridDim.x * (kBlock / 64);
  const int w = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6)));
  const int lane = threadIdx.x & 63;
  if (kMode == 0) {
    for (int i = w; i < p.n_item; i += n_waves) {
      const apc_edge item = p.items[i];
      process_item(p, item, lane, per_arg, comm, cost, flags, clamp_inf);
    }
    return;
  }
  // pipelined: the loads of the next item are issued before the current one is stored
  const apc_edge* __restrict__ items = p.items;
  const double* __restrict__ default_vals = p.default_vals;
  const int32_t* __restrict__ list_uidx = p.list_uidx;
  const int n_item = p.n_item;
  bool have = false;
  apc_edge cur;
  ItemLoads<kN> cur_r;
  apc_edge nxt;
  if (w < n_item) nxt = items[w];
  for (int i = w; i < n_item; i += n_waves) {
    const apc_edge item = nxt;
    if (i + n_waves < n_item) nxt = items[i + n_waves];  // record of the item after this one
    ItemLoads<kN> r;
    item_load<kMode == 2, kN>(item, lane, table, default_vals, list_uidx, per_arg, r);
    if (have) item_store(cur, cur_r, comm, cost, flags, clamp_inf);
    cur = item;
    cur_r = r;
    have = true;
  }
  if (have) item_store(cur, cur_r, comm, cost, flags, clamp_inf);
}

// Plain copy kernel of known size: the reference point against which the
// hardware traffic counters are scaled when a profile is taken.
__global__ void __launch_bounds__(kBlock)
calibration_copy_kernel(const double2_t* __restrict__ src, double2_t* __restrict__ dst, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

// ---------------------------------------------------------------------------
// Kernels: post-passes over the entry arrays (one entry per lane)
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock)
prefetch_discount_kernel(apc_problem p, const double* __restrict__ per_arg, double scale,
                         double* __restrict__ comm, double* __restrict__ cost,
                         const uint8_t* __restrict__ flags, unsigned long long* n_modified) {
  const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  unsigned int mine = 0;
  if (idx < p.n_slot) {
    const apc_edge ed = find_edge(p, idx);
    const int64_t local = idx - ed.off;
    if (local < (int64_t)ed.ssrc * ed.sdst && (ed.flags & APC_EDGE_PREFETCHABLE) &&
        ed.src_node >= 0) {
      double c = comm[idx];
      if (c > 0.0 && isfinite(c)) {
        const uint32_t o = (uint32_t)local / (uint32_t)ed.ssrc;
        c = c * scale;
        comm[idx] = c;
        cost[idx] = (c + per_arg[ed.comp_base + o]) + (double)(flags[idx] & APC_ENTRY_TRANSITION);
        mine = 1;
      }
    }
  }
  // wavefront reduction, one atomic per wave
  for (int off = 32; off > 0; off >>= 1) mine += __shfl_down(mine, off, 64);
  if ((threadIdx.x & 63) == 0 && mine) atomicAdd(n_modified, (unsigned long long)mine);
}

__global__ void __launch_bounds__(kBlock)
objective_kernel(apc_problem p, const double* __restrict__ cost, double* __restrict__ obj) {
  const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= p.n_slot) return;
  const apc_edge ed = find_edge(p, idx);
  if (idx - ed.off < (int64_t)ed.ssrc * ed.sdst)
    obj[idx] = cost[idx] * (double)p.node_multiplier[ed.node];
}

// ---------------------------------------------------------------------------
// Kernel: structural hash of every node, the key under which repeated layers
// are clustered.  It covers what the reference's node key covers
// (graph_passes/graph_clustering.py:68-82: the op, the forward/backward tag, the
// node's own strategies and its producers' strategies), read from the packed
// arrays: op class, program, strategy counts, output/input/producer spec runs,
// default rows.  H = mix(sum over (section, position) of mix(word ^ salt)): a
// position-salted sum, so the lanes of a wavefront hash disjoint positions and
// add.
// ---------------------------------------------------------------------------
__host__ __device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ uint64_t hash_term(uint64_t section, uint64_t pos, uint64_t w) {
  return mix64(w ^ mix64((section << 40) + pos + 0x9E3779B97F4A7C15ull));
}

__global__ void __launch_bounds__(kBlock)
node_hash_kernel(apc_problem p, const int64_t* __restrict__ node_out_list,
                 const int32_t* __restrict__ node_phase, uint64_t* __restrict__ out) {
  const int v = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (v >= p.n_node) return;  // wave-uniform
  const int lane = threadIdx.x & 63;
  const int S = p.node_nstrat[v];
  const int e0 = p.node_edge_off[v], e1 = p.node_edge_off[v + 1];
  const int op = p.node_op[v];
  uint64_t acc = 0;
  if (lane == 0) {
    acc += hash_term(0, 0, (uint64_t)op);
    acc += hash_term(0, 1, (uint64_t)p.node_nargs[v]);
    acc += hash_term(0, 2, (uint64_t)S);
    acc += hash_term(0, 3, (uint64_t)(node_phase ? node_phase[v] : 0));
    acc += hash_term(0, 4, (uint64_t)(e1 - e0));
  }
  const int plen = p.node_prog_len[v];
  for (int i = lane; i < plen; i += 64) acc += hash_term(1, i, (uint64_t)p.prog[p.node_prog_off[v] + i]);
  for (int k = lane; k < S; k += 64) acc += hash_term(2, k, p.lists[(size_t)node_out_list[v] + k]);
  if (op == APC_OP_EXPLICIT) {
    const int64_t b = p.node_comp_off[v];
    for (int k = lane; k < S; k += 64) {
      acc += hash_term(3, k, (uint64_t)p.explicit_flops[b + k]);
      acc += hash_term(4, k, (uint64_t)p.explicit_bytes[b + k]);
    }
  }
  for (int e = e0; e < e1; ++e) {
    const apc_edge ed = p.edges[e];
    const uint64_t sec = 16 + 4 * (uint64_t)(e - e0);
    if (lane == 0) {
      acc += hash_term(sec, 0, (uint64_t)ed.ssrc);
      acc += hash_term(sec, 1, (uint64_t)ed.sdst);
      acc += hash_term(sec, 2, (uint64_t)(ed.flags & (APC_EDGE_HAS_PRODUCER | APC_EDGE_SCORE_TRANSITION)));
      acc += hash_term(sec, 3, (uint64_t)(ed.default_off >= 0));
    }
    for (int k = lane; k < ed.sdst; k += 64) acc += hash_term(sec + 1, k, p.lists[(size_t)ed.dst_list + k]);
    if (ed.src_node >= 0)
      for (int j = lane; j < ed.ssrc; j += 64) acc += hash_term(sec + 2, j, p.lists[(size_t)ed.src_list + j]);
    if (ed.default_off >= 0) {
      const int64_t n = (int64_t)ed.ssrc * ed.sdst;
      for (int64_t i = lane; i < n; i += 64)
        acc += hash_term(sec + 3, (uint64_t)i, (uint64_t)__double_as_longlong(p.default_vals[ed.default_off + i]));
    }
  }
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor((unsigned long long)acc, off);
  if (lane == 0) out[v] = mix64(acc);
}

// ---------------------------------------------------------------------------
// Kernel: packed twin of the decision variables, in the reference's insertion
// order (node, out_idx, argi, inp_idx): row of entry (e, o, j) is
// row_base[e] + o * row_stride[e] + j, where row_stride is the node's sum of
// S_src over its arguments.  One lane per slot; the lanes of a run of inp_idx
// write consecutive rows.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock)
export_kernel(apc_problem p, const double* __restrict__ per_arg, const double* __restrict__ comm,
              const uint8_t* __restrict__ flags, const int64_t* __restrict__ row_base,
              const int32_t* __restrict__ row_stride, int32_t* __restrict__ keys,
              double* __restrict__ vals) {
  const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= p.n_slot) return;
  const int e = p.chunk_edge[idx >> APC_CHUNK_SHIFT];
  const apc_edge ed = p.edges[e];
  const int64_t local = idx - ed.off;
  if (local >= (int64_t)ed.ssrc * ed.sdst) return;
  const uint32_t o = (uint32_t)local / (uint32_t)ed.ssrc;
  const uint32_t j = (uint32_t)local - o * (uint32_t)ed.ssrc;
  const int64_t row = row_base[e] + (int64_t)o * row_stride[e] + j;
  int4 k;
  k.x = ed.node;
  k.y = e - p.node_edge_off[ed.node];
  k.z = (int)o;
  k.w = (int)j;
  *reinterpret_cast<int4*>(keys + row * 4) = k;
  double* v = vals + row * 3;
  v[0] = per_arg[ed.comp_base + o];
  v[1] = comm[idx];
  v[2] = (double)(flags[idx] & APC_ENTRY_TRANSITION);
}

// The selected entry of every edge under one assignment (out_idx per node):
// terms[e] = (per-arg compute, comm, transition, cost) of entry
// (e, assign[node], assign[producer] or 0) and slot[e] = its slot.
__global__ void __launch_bounds__(kBlock)
solution_terms_kernel(apc_problem p, const double* __restrict__ per_arg,
                      const double* __restrict__ comm, const double* __restrict__ cost,
                      const uint8_t* __restrict__ flags, const uint16_t* __restrict__ assign,
                      double* __restrict__ terms, int64_t* __restrict__ slot) {
  const int e = blockIdx.x * kBlock + threadIdx.x;
  if (e >= p.n_edge) return;
  const apc_edge ed = p.edges[e];
  const uint32_t o = assign[ed.node];
  const uint32_t j = ed.src_node >= 0 ? assign[ed.src_node] : 0u;
  double* t = terms + (size_t)e * 4;
  if (o >= (uint32_t)ed.sdst || j >= (uint32_t)ed.ssrc) {  // not a strategy index of this edge
    t[0] = t[1] = t[2] = t[3] = NAN;
    slot[e] = -1;
    return;
  }
  const int64_t idx = ed.off + (int64_t)o * ed.ssrc + j;
  t[0] = per_arg[ed.comp_base + o];
  t[1] = comm[idx];
  t[2] = (double)(flags[idx] & APC_ENTRY_TRANSITION);
  t[3] = cost[idx];
  slot[e] = idx;
}

// ---------------------------------------------------------------------------
// Kernel: batch scoring.  One lane per assignment; the lane walks the graph in
// node order then argument order, so every sum has the reference's order.
// ---------------------------------------------------------------------------
__host__ __device__ __forceinline__ uint32_t mix_assignment(uint64_t seed, int64_t a, int32_t node,
                                                            int32_t nstrat) {
  // counter-based draw: a 32-bit mix of (seed, assignment, node) through
  // murmur3's finaliser, scaled to [0, nstrat) by a multiply-high.  The part
  // that does not depend on the node is loop-invariant in the scorers; the
  // walk is instruction-bound, and the 64-bit mix with a modulo that was
  // here before took a quarter of it.
  uint32_t h = (uint32_t)seed ^ ((uint32_t)(seed >> 32) * 0x27D4EB2Fu);
  h ^= (uint32_t)(uint64_t)a * 0x9E3779B1u;
  h ^= (uint32_t)((uint64_t)a >> 32) * 0x85EBCA77u;
  h ^= (uint32_t)(node + 1) * 0xC2B2AE3Du;
  h ^= h >> 16;
  h *= 0x85EBCA6Bu;
  h ^= h >> 13;
  h *= 0xC2B2AE35u;
  h ^= h >> 16;
  return (uint32_t)(((uint64_t)h * (uint64_t)(uint32_t)nstrat) >> 32);
}

// An edge record through one 64-byte load.  In the scorers the index is
// wave-uniform, so this is a single scalar load instead of one per field with a
// wait after each, and the record of the next edge is requested before the
// current one is used.
typedef uint32_t u32x16_t __attribute__((ext_vector_type(16)));
__device__ __forceinline__ apc_edge load_edge(const apc_edge* __restrict__ e) {
  union { u32x16_t raw; apc_edge ed; } u;
  u.raw = *reinterpret_cast<const u32x16_t*>(e);
  return u.ed;
}

template <bool kRandom>
__global__ void __launch_bounds__(kBlock)
score_kernel(apc_problem p, const double* __restrict__ per_arg, const double* __restrict__ comm,
             const double* __restrict__ cost, const uint8_t* __restrict__ flags,
             const uint16_t* __restrict__ assign, int64_t stride, uint64_t seed, int64_t first,
             int64_t n_assign, double* __restrict__ out) {
  const int64_t a = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (a >= n_assign) return;
  double t_compute = 0.0, t_comm = 0.0, t_trans = 0.0, obj = 0.0, forbidden = 0.0;
  apc_edge nxt;  // edges are visited in index order
  if (p.n_edge > 0) nxt = load_edge(p.edges);
  for (int v = 0; v < p.n_node; ++v) {
    const uint32_t o = kRandom ? mix_assignment(seed, first + a, v, p.node_nstrat[v])
                               : (uint32_t)assign[(size_t)v * stride + a];
    const int nargs = p.node_nargs[v];
    const double pa = per_arg[p.node_comp_off[v] + o];
    t_compute += pa * (double)(nargs > 1 ? nargs : 1);
    const double mult = (double)p.node_multiplier[v];
    for (int e = p.node_edge_off[v]; e < p.node_edge_off[v + 1]; ++e) {
      const apc_edge ed = nxt;
      if (e + 1 < p.n_edge) nxt = load_edge(p.edges + e + 1);
      uint32_t j = 0;
      if (ed.src_node >= 0)  // ssrc is the producer's strategy count
        j = kRandom ? mix_assignment(seed, first + a, ed.src_node, ed.ssrc)
                    : (uint32_t)assign[(size_t)ed.src_node * stride + a];
      const int64_t idx = ed.off + (int64_t)o * ed.ssrc + j;
      const uint8_t f = flags[idx];
      obj += cost[idx] * mult;
      forbidden += (double)((f & APC_ENTRY_NONFINITE) != 0);
      if (ed.src_node >= 0) {
        const double c = comm[idx];
        if (isfinite(c)) t_comm += c;
        if ((ed.flags & APC_EDGE_SCORE_TRANSITION) && (f & APC_ENTRY_TRANSITION)) t_trans += 1.0;
      }
    }
  }
  double* r = out + a * 6;
  r[0] = (t_compute + t_comm) + t_trans;
  r[1] = t_compute;
  r[2] = t_comm;
  r[3] = t_trans;
  r[4] = obj;
  r[5] = forbidden;
}

// In-order fold of one value per lane into acc: acc = (..((acc + v0) + v1)..) + v63,
// the association a sequential loop over 64 items has.
__device__ __forceinline__ double fold_in_order(double acc, double v) {
  const int lo = __double2loint(v), hi = __double2hiint(v);
#pragma unroll
  for (int i = 0; i < 64; ++i)
    acc += __hiloint2double(__builtin_amdgcn_readlane(hi, i), __builtin_amdgcn_readlane(lo, i));
  return acc;
}

// Small batches: one wavefront per assignment.  Lanes take 64 consecutive
// nodes (then 64 consecutive edges) at a time, gather their terms in parallel,
// and the terms are folded lane by lane in order, so the sums keep the
// reference's sequential association (bit-identical to score_kernel) while the
// gathers of a tile overlap.
// score_kernel<true> over a window of a larger graph: global node ids for the
// draw, sums continued from the previous window's.
__global__ void __launch_bounds__(kBlock)
score_window_kernel(apc_problem p, const double* __restrict__ per_arg,
                    const double* __restrict__ comm, const double* __restrict__ cost,
                    const uint8_t* __restrict__ flags, uint64_t seed, int64_t first,
                    int64_t n_assign, const int32_t* __restrict__ node_gid, int first_node,
                    const double* __restrict__ init, double* __restrict__ out) {
  const int64_t a = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (a >= n_assign) return;
  double t_compute = 0.0, t_comm = 0.0, t_trans = 0.0, obj = 0.0, forbidden = 0.0;
  if (init) {
    const double* r = init + a * 6;
    t_compute = r[1]; t_comm = r[2]; t_trans = r[3]; obj = r[4]; forbidden = r[5];
  }
  apc_edge nxt;
  if (first_node < p.n_node && p.node_edge_off[first_node] < p.n_edge)
    nxt = load_edge(p.edges + p.node_edge_off[first_node]);
  for (int v = first_node; v < p.n_node; ++v) {
    const uint32_t o = mix_assignment(seed, first + a, node_gid[v], p.node_nstrat[v]);
    const int nargs = p.node_nargs[v];
    const double pa = per_arg[p.node_comp_off[v] + o];
    t_compute += pa * (double)(nargs > 1 ? nargs : 1);
    const double mult = (double)p.node_multiplier[v];
    for (int e = p.node_edge_off[v]; e < p.node_edge_off[v + 1]; ++e) {
      const apc_edge ed = nxt;
      if (e + 1 < p.n_edge) nxt = load_edge(p.edges + e + 1);
      uint32_t j = 0;
      if (ed.src_node >= 0)
        j = mix_assignment(seed, first + a, node_gid[ed.src_node], ed.ssrc);
      const int64_t idx = ed.off + (int64_t)o * ed.ssrc + j;
      const uint8_t f = flags[idx];
      obj += cost[idx] * mult;
      forbidden += (double)((f & APC_ENTRY_NONFINITE) != 0);
      if (ed.src_node >= 0) {
        const double c = comm[idx];
        if (isfinite(c)) t_comm += c;
        if ((ed.flags & APC_EDGE_SCORE_TRANSITION) && (f & APC_ENTRY_TRANSITION)) t_trans += 1.0;
      }
    }
  }
  double* r = out + a * 6;
  r[0] = (t_compute + t_comm) + t_trans;
  r[1] = t_compute;
  r[2] = t_comm;
  r[3] = t_trans;
  r[4] = obj;
  r[5] = forbidden;
}

// The lane-per-assignment walk over interleaved records (apc_score_rec): one
// gather per drawn entry.  Covers explicit assignments, drawn ones, and windows
// of a larger graph (global ids for the draw, sums continued from init).
__global__ void __launch_bounds__(kBlock)
score_pack_kernel(int64_t n, const double* __restrict__ comm, const double* __restrict__ cost,
                  const uint8_t* __restrict__ flags, apc_score_rec* __restrict__ recs) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  apc_score_rec r;
  r.comm = comm[i];
  r.cost = cost[i];
  r.flags = flags[i];
  r.reserved = 0;
  recs[i] = r;
}

template <bool kRandom>
__global__ void __launch_bounds__(kBlock)
score_packed_kernel(apc_problem p, const double* __restrict__ per_arg,
                    const apc_score_rec* __restrict__ recs, const uint16_t* __restrict__ assign,
                    int64_t stride, uint64_t seed, int64_t first, int64_t n_assign,
                    const int32_t* __restrict__ node_gid, int first_node,
                    const double* __restrict__ init, double* __restrict__ out) {
  const int64_t a = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (a >= n_assign) return;
  double t_compute = 0.0, t_comm = 0.0, t_trans = 0.0, obj = 0.0, forbidden = 0.0;
  if (init) {
    const double* r = init + a * 6;
    t_compute = r[1]; t_comm = r[2]; t_trans = r[3]; obj = r[4]; forbidden = r[5];
  }
  auto choice = [&](int v, int nstrat) -> uint32_t {
    return kRandom ? mix_assignment(seed, first + a, node_gid ? node_gid[v] : v, nstrat)
                   : (uint32_t)assign[(size_t)v * stride + a];
  };
  apc_edge nxt;
  if (first_node < p.n_node && p.node_edge_off[first_node] < p.n_edge)
    nxt = load_edge(p.edges + p.node_edge_off[first_node]);
  for (int v = first_node; v < p.n_node; ++v) {
    const uint32_t o = choice(v, p.node_nstrat[v]);
    const int nargs = p.node_nargs[v];
    const double pa = per_arg[p.node_comp_off[v] + o];
    t_compute += pa * (double)(nargs > 1 ? nargs : 1);
    const double mult = (double)p.node_multiplier[v];
    for (int e = p.node_edge_off[v]; e < p.node_edge_off[v + 1]; ++e) {
      const apc_edge ed = nxt;
      if (e + 1 < p.n_edge) nxt = load_edge(p.edges + e + 1);
      const uint32_t j = ed.src_node >= 0 ? choice(ed.src_node, ed.ssrc) : 0u;  // ssrc: the producer's count
      const apc_score_rec r = recs[ed.off + (int64_t)o * ed.ssrc + j];
      const uint32_t f = (uint32_t)r.flags;
      obj += r.cost * mult;
      forbidden += (double)((f & APC_ENTRY_NONFINITE) != 0);
      if (ed.src_node >= 0) {
        if (isfinite(r.comm)) t_comm += r.comm;
        if ((ed.flags & APC_EDGE_SCORE_TRANSITION) && (f & APC_ENTRY_TRANSITION)) t_trans += 1.0;
      }
    }
  }
  double* r = out + a * 6;
  r[0] = (t_compute + t_comm) + t_trans;
  r[1] = t_compute;
  r[2] = t_comm;
  r[3] = t_trans;
  r[4] = obj;
  r[5] = forbidden;
}

template <bool kRandom>
__global__ void __launch_bounds__(kBlock)
score_wave_kernel(apc_problem p, const double* __restrict__ per_arg,
                  const double* __restrict__ comm, const double* __restrict__ cost,
                  const uint8_t* __restrict__ flags, const uint16_t* __restrict__ assign,
                  int64_t stride, uint64_t seed, int64_t first, int64_t n_assign,
                  double* __restrict__ out) {
  const int64_t a = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (a >= n_assign) return;  // wave-uniform
  const int lane = threadIdx.x & 63;
  auto choice = [&](int v) -> uint32_t {
    return kRandom ? mix_assignment(seed, first + a, v, p.node_nstrat[v])
                   : (uint32_t)assign[(size_t)v * stride + a];
  };
  double t_compute = 0.0, t_comm = 0.0, t_trans = 0.0, obj = 0.0, forbidden = 0.0;
  for (int v0 = 0; v0 < p.n_node; v0 += 64) {
    const int v = v0 + lane;
    double term = 0.0;
    if (v < p.n_node) {
      const int nargs = p.node_nargs[v];
      term = per_arg[p.node_comp_off[v] + choice(v)] * (double)(nargs > 1 ? nargs : 1);
    }
    t_compute = fold_in_order(t_compute, term);  // + 0.0 for the lanes past the end
  }
  for (int e0 = 0; e0 < p.n_edge; e0 += 64) {
    const int e = e0 + lane;
    double c_term = 0.0, o_term = 0.0, tr = 0.0, fb = 0.0;
    if (e < p.n_edge) {
      const apc_edge ed = p.edges[e];
      const uint32_t o = choice(ed.node);
      const uint32_t j = ed.src_node >= 0 ? choice(ed.src_node) : 0u;
      const int64_t idx = ed.off + (int64_t)o * ed.ssrc + j;
      const uint8_t f = flags[idx];
      o_term = cost[idx] * (double)p.node_multiplier[ed.node];
      fb = (double)((f & APC_ENTRY_NONFINITE) != 0);
      if (ed.src_node >= 0) {
        const double c = comm[idx];
        if (isfinite(c)) c_term = c;
        if ((ed.flags & APC_EDGE_SCORE_TRANSITION) && (f & APC_ENTRY_TRANSITION)) tr = 1.0;
      }
    }
    t_comm = fold_in_order(t_comm, c_term);
    obj = fold_in_order(obj, o_term);
    // small integers: any order is exact
    for (int off = 32; off > 0; off >>= 1) {
      tr += __shfl_xor(tr, off, 64);
      fb += __shfl_xor(fb, off, 64);
    }
    t_trans += tr;
    forbidden += fb;
  }
  if (lane == 0) {
    double* r = out + a * 6;
    r[0] = (t_compute + t_comm) + t_trans;
    r[1] = t_compute;
    r[2] = t_comm;
    r[3] = t_trans;
    r[4] = obj;
    r[5] = forbidden;
  }
}

// ---------------------------------------------------------------------------
// Kernel: input/parameter placement options
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock)
enumerate_kernel(apc_model m, int32_t n, const int32_t* __restrict__ rank,
                 const int64_t* __restrict__ shape, const int64_t* __restrict__ cand_off,
                 uint8_t* __restrict__ valid, uint8_t* __restrict__ plc) {
  const int64_t total = cand_off[n];
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    int lo = 0, hi = n;
    while (hi - lo > 1) {
      int mid = (lo + hi) >> 1;
      if (cand_off[mid] <= idx) lo = mid; else hi = mid;
    }
    const int t = lo;
    const int r = rank[t];
    int64_t c = idx - cand_off[t];
    // itertools.product order: the last mesh dim varies fastest
    int code[APC_MAX_MESH_DIMS] = {0, 0, 0, 0};
    for (int i = m.ndim - 1; i >= 0; --i) {
      const int opt = (int)(c % (r + 1));
      c /= (r + 1);
      code[i] = opt == 0 ? 0 : (kShard | (opt - 1));
    }
    int64_t sh[APC_MAX_RANK];
    for (int d = 0; d < APC_MAX_RANK; ++d) sh[d] = shape[(size_t)t * APC_MAX_RANK + d];
    bool ok = true;
    for (int i = 0; i < m.ndim && ok; ++i) {
      if ((code[i] & kKindMask) == kShard) {
        const int d = code[i] & kArgMask;
        const int64_t ms = m.mesh_shape[i];
        // dynamic index kept in a loop so sh[] stays in registers
        for (int dd = 0; dd < APC_MAX_RANK; ++dd) {
          if (dd == d) {
            if (sh[dd] >= ms) sh[dd] = (sh[dd] + ms - 1) / ms; else ok = false;
          }
        }
      }
    }
    valid[idx] = ok ? 1 : 0;
    for (int i = 0; i < APC_MAX_MESH_DIMS; ++i) plc[idx * APC_MAX_MESH_DIMS + i] = (uint8_t)code[i];
  }
}

// ---------------------------------------------------------------------------
// Kernels: scalar cost-model functions in batch form
// ---------------------------------------------------------------------------
// _get_sharded_shape_stride (compute_estimation.py:300-318), including its
// stride rule: the stride of dim d-1 is divided only when d-1 > 0.
__global__ void __launch_bounds__(kBlock)
local_shape_kernel(apc_model m, int32_t n, const int32_t* __restrict__ rank,
                   const int64_t* __restrict__ shape, const int64_t* __restrict__ stride,
                   const uint8_t* __restrict__ plc, int64_t* __restrict__ out_shape,
                   int64_t* __restrict__ out_stride) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  const int r = rank[t];
  for (int d = 0; d < APC_MAX_RANK; ++d) {
    out_shape[(size_t)t * APC_MAX_RANK + d] = shape[(size_t)t * APC_MAX_RANK + d];
    out_stride[(size_t)t * APC_MAX_RANK + d] = stride[(size_t)t * APC_MAX_RANK + d];
  }
  for (int i = 0; i < m.ndim; ++i) {
    const int c = plc[(size_t)t * APC_MAX_MESH_DIMS + i];
    if ((c & kKindMask) != kShard) continue;
    const int d = c & kArgMask;
    if (d >= r) continue;
    const int64_t ms = m.mesh_shape[i];
    int64_t* s = out_shape + (size_t)t * APC_MAX_RANK;
    int64_t* st = out_stride + (size_t)t * APC_MAX_RANK;
    s[d] = (s[d] + ms - 1) / ms;
    if (d - 1 > 0) st[d - 1] = (st[d - 1] + ms - 1) / ms;
  }
}

// collective_comm_cost, default model (collective_runtime_estimation.py:65-97):
// kind 0 allgather, 1 all_to_all, 2 allreduce, 3 reduce_scatter, else 0.0
__global__ void __launch_bounds__(kBlock)
collective_kernel(apc_model m, int32_t n, const int32_t* __restrict__ kind,
                  const int64_t* __restrict__ nbytes, const int32_t* __restrict__ dim,
                  double* __restrict__ out) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  const int k = kind[t], d = dim[t];
  out[t] = (k >= 0 && k <= 3 && d >= 0 && d < m.ndim) ? collective_cost(k, nbytes[t], d, m) : 0.0;
}

// compute_read_write_time (compute_estimation.py:391-403)
__global__ void __launch_bounds__(kBlock)
rw_time_kernel(apc_model m, int32_t n, const double* __restrict__ nbytes, double* __restrict__ out) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) out[t] = rw_time(nbytes[t], m.gmem_bw);
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
// below this many assignments one wavefront per assignment is faster than one lane
constexpr int64_t kScoreWaveBelow = 32768;

int validate_problem(const apc_problem* p) {
  if (!p) return fail(APC_ERR_INVALID, "null problem%s");
  if (p->model.ndim < 1 || p->model.ndim > APC_MAX_MESH_DIMS)
    return fail(APC_ERR_INVALID, "mesh ndim out of range%s");
  for (int i = 0; i < p->model.ndim; ++i)
    if (p->model.mesh_shape[i] < 1) return fail(APC_ERR_INVALID, "mesh size < 1%s");
  if (p->model.order_mode < 0 || p->model.order_mode > 2)
    return fail(APC_ERR_INVALID, "order_mode must be 0, 1 or 2%s");
  if (p->n_meta < 0 || p->n_tuple < 0 || p->n_tuple > (1 << APC_TUPLE_BITS))
    return fail(APC_ERR_INVALID, "bad meta/tuple counts%s");
  if (p->n_node < 0 || p->n_edge < 0 || p->n_entry < 0 || p->n_comp_node < 0 ||
      p->n_comp_node > p->n_node || p->n_compute < 0)
    return fail(APC_ERR_INVALID, "bad sizes%s");
  if (p->n_slot < p->n_entry || (p->n_slot & ((1 << APC_CHUNK_SHIFT) - 1)) ||
      p->n_chunk != (p->n_slot >> APC_CHUNK_SHIFT) || p->n_item < 0)
    return fail(APC_ERR_INVALID, "n_slot / n_chunk / n_item inconsistent%s");
  if (p->n_entry > 0 && (!p->edges || !p->chunk_edge || !p->lists || !p->items))
    return fail(APC_ERR_INVALID, "null edge/list/item arrays%s");
  if (p->n_comp_node > 0 && !p->comp_nodes) return fail(APC_ERR_INVALID, "null comp_nodes%s");
  if (p->n_block < 0 || p->table_size < 0 || (p->table_size & 255) ||
      p->n_table_unit != p->table_size / 256 ||
      (p->table_size > 0 && (!p->block_edge || !p->block_off || !p->table_unit_block)))
    return fail(APC_ERR_INVALID, "bad block table description%s");
  if (p->item_entries != 0 && p->item_entries != APC_ITEM_ENTRIES &&
      p->item_entries != 2 * APC_ITEM_ENTRIES)
    return fail(APC_ERR_INVALID, "item_entries must be 0, 256 or 512%s");
  if ((p->list_uidx != nullptr) != (p->list_ufirst != nullptr) ||
      (p->list_uidx != nullptr) != (p->block_udst != nullptr))
    return fail(APC_ERR_INVALID, "compressed block table: list_uidx, list_ufirst and block_udst go together%s");
  if (p->max_rank < 0 || p->max_rank > APC_MAX_RANK || p->max_node_args < 0)
    return fail(APC_ERR_INVALID, "max_rank / max_node_args out of range%s");
  return 0;
}

int grid_for(int64_t total, int block) {
  int64_t g = (total + block - 1) / block;
  const int64_t cap = 256 * 32;  // grid-stride kernels: a few waves per CU
  if (g > cap) g = cap;
  if (g < 1) g = 1;
  return (int)g;
}

int slot_grid(const apc_problem* p, int per_block, unsigned* grid) {
  const int64_t g = (p->n_slot + per_block - 1) / per_block;
  if (g > 0x7FFFFFFF) return fail(APC_ERR_INVALID, "too many entries for one launch%s");
  *grid = (unsigned)g;
  return 0;
}

int launch_prepare(const apc_problem* p, double* table, bool do_nodes, double* compute,
                   double* per_arg, int32_t* status, hipStream_t stream) {
  int table_blocks = (table && p->table_size > 0) ? p->n_table_unit : 0;
  if (table_blocks > kFusedTableBlocks) {  // a launch of its own: see pair_table_kernel
    hipLaunchKernelGGL(pair_table_kernel, dim3(table_blocks), dim3(256), 0, stream, *p, table);
    if (int rc = check_launch("pair_table_kernel")) return rc;
    table_blocks = 0;
  }
  const int64_t chunks = (p->max_nstrat + 63) >> 6;
  const int64_t units = (int64_t)p->n_comp_node * chunks;  // one wavefront per 64 strategies of a node
  if (do_nodes && (chunks < 1 || units > (1ll << 30)))
    return fail(APC_ERR_INVALID, "launch_prepare: max_nstrat must be >= 1 and n_comp_node * chunks < 2^30%s");
  const int node_blocks = do_nodes ? (int)((units + kNodesPerBlock - 1) / kNodesPerBlock) : 0;
  if (table_blocks + node_blocks == 0) return 0;
  // LDS for the local-size staging (a CU has 160 KB); beyond 96 KB per block,
  // sizes are read on demand instead
  const int64_t words = (int64_t)p->max_node_args * (p->max_rank + 2) * 64;
  const int slow = ((kProgCache + kRecWords + words) * kNodesPerBlock * 8 > 96 * 1024 ||
                    p->n_meta == 0 || p->n_tuple == 0) ? 1 : 0;
  const size_t lds =
      do_nodes ? (size_t)kNodesPerBlock * (kProgCache + kRecWords + (slow ? 0 : words)) * 8 : 0;
  static bool attr_set = false;  // raise the 64 KB default limit of dynamic LDS once
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(prepare_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
    if (e != hipSuccess) {
      snprintf(g_err, sizeof(g_err), "hipFuncSetAttribute: %s", hipGetErrorString(e));
      return APC_ERR_LAUNCH;
    }
    attr_set = true;
  }
  hipLaunchKernelGGL(prepare_kernel, dim3(table_blocks + node_blocks), dim3(256), lds, stream, *p,
                     table, table_blocks, slow, compute, per_arg, status);
  return check_launch("prepare_kernel");
}

}  // namespace

extern "C" {

int apc_version(void) { return 2; }

const char* apc_last_error(void) { return g_err; }

__attribute__((visibility("hidden"))) void apc_internal_set_error(const char* msg) {
  snprintf(g_err, sizeof(g_err), "%s", msg);
}

int apc_mesh_topology(const int32_t* mesh_shape, int32_t ndim, int32_t devices_per_host,
                      double* bw, double* lat) {
  if (!mesh_shape || !bw || !lat || ndim < 1 || ndim > APC_MAX_MESH_DIMS)
    return fail(APC_ERR_INVALID, "apc_mesh_topology: bad arguments%s");
  const double base_bw = 87.7;
  int64_t total = 1;
  for (int i = 0; i < ndim; ++i) { bw[i] = base_bw; lat[i] = 0.6; }
  for (int i = ndim - 1; i >= 0; --i) {
    total *= mesh_shape[i];
    if (total > devices_per_host) {
      bw[i] = bw[i] * 0.22;
      lat[i] = 2.7;
    }
  }
  return 0;
}

int apc_device_limits(const char* device_name, apc_model* model) {
  if (!device_name || !model) return fail(APC_ERR_INVALID, "apc_device_limits: null argument%s");
  for (int i = 0; i < APC_NUM_DTYPES; ++i) model->tflops[i] = 0.0;
  // dtype codes: 0 f64, 1 f32, 2 f16, 3 bf16, 4 int8
  if (strstr(device_name, "AMD Instinct MI355X")) {
    model->gmem_bw = 8.0 * (1024.0 * 1024.0 * 1024.0 * 1024.0);
    model->tflops[0] = 78.6; model->tflops[1] = 157.3; model->tflops[2] = 2516.6;
    model->tflops[3] = 2516.6; model->tflops[4] = 5033.2;
    return 0;
  }
  if (strstr(device_name, "AMD Instinct MI300X")) {
    model->gmem_bw = 5.3 * (1024.0 * 1024.0 * 1024.0 * 1024.0);
    model->tflops[0] = 81.7; model->tflops[1] = 163.4; model->tflops[2] = 1307.4;
    model->tflops[3] = 1307.4; model->tflops[4] = 2614.9;
    return 0;
  }
  return fail(APC_ERR_UNSUPPORTED, "Unsupported device: %s", device_name);
}

int64_t apc_pair_table_size(const apc_problem* p) {
  if (!p) return 0;
  return p->table_size;
}

int apc_build_pair_table(const apc_problem* p, double* table, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (apc_pair_table_size(p) == 0) return 0;
  if (!table) return fail(APC_ERR_INVALID, "apc_build_pair_table: null table%s");
  return launch_prepare(p, table, false, nullptr, nullptr, nullptr, (hipStream_t)stream);
}

int apc_node_compute_costs(const apc_problem* p, double* compute, double* per_arg,
                           int32_t* status, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_comp_node == 0) return 0;
  if (!compute || !per_arg || !status)
    return fail(APC_ERR_INVALID, "apc_node_compute_costs: null output%s");
  return launch_prepare(p, nullptr, true, compute, per_arg, status, (hipStream_t)stream);
}

int apc_prepare(const apc_problem* p, double* table, double* compute, double* per_arg,
                int32_t* status, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (!compute || !per_arg || !status) return fail(APC_ERR_INVALID, "apc_prepare: null output%s");
  return launch_prepare(p, table, p->n_comp_node > 0, compute, per_arg, status,
                        (hipStream_t)stream);
}

// start / stop: events recorded at the kernel's own begin and end (NULL: none)
static int launch_edge_costs(const apc_problem* p, const double* table, const double* per_arg,
                             double* comm, double* cost, uint8_t* flags, int32_t clamp_inf,
                             hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_entry == 0) return 0;
  if (!per_arg) return fail(APC_ERR_INVALID, "apc_edge_costs: null per_arg%s");
  unsigned grid = (unsigned)((p->n_item + (kBlock / 64) - 1) / (kBlock / 64));
  // Measured on MI355X: the table kernel (8 waves per SIMD) is fastest with one
  // wave per item, the direct kernel (4 per SIMD, long-lived waves) with a few
  // items per wave; the caps only bound the grid of very large problems.
  const unsigned cap = table ? (1u << 22) : (1u << 14);
  if (grid > cap) grid = cap;
  const bool wide = p->item_entries == 2 * APC_ITEM_ENTRIES;
  if (wide && !table)
    return fail(APC_ERR_INVALID, "apc_edge_costs: work items of 512 entries need a block table%s");
#define APC_LAUNCH_EDGE(MODE, N)                                                                   \
  hipExtLaunchKernelGGL((edge_cost_kernel<MODE, N>), dim3(grid), dim3(kBlock), 0, stream, start,   \
                        stop, 0, *p, table, per_arg, comm, cost, flags, clamp_inf)
  if (table && p->list_uidx) {
    if (wide) APC_LAUNCH_EDGE(2, 2 * kPerLane); else APC_LAUNCH_EDGE(2, kPerLane);
  } else if (table) {
    if (wide) APC_LAUNCH_EDGE(1, 2 * kPerLane); else APC_LAUNCH_EDGE(1, kPerLane);
  } else {
    APC_LAUNCH_EDGE(0, kPerLane);
  }
#undef APC_LAUNCH_EDGE
  return check_launch("edge_cost_kernel");
}

int apc_edge_costs(const apc_problem* p, const double* table, const double* per_arg, double* comm,
                   double* cost, uint8_t* flags, int32_t clamp_inf, void* stream) {
  return launch_edge_costs(p, table, per_arg, comm, cost, flags, clamp_inf, (hipStream_t)stream,
                           nullptr, nullptr);
}

struct apc_timer {
  int32_t n;
  hipEvent_t* ev;  // 2 n events: start and stop of each slot
};

int apc_timer_create(int32_t n_slots, void** timer) {
  if (n_slots <= 0 || !timer) return fail(APC_ERR_INVALID, "apc_timer_create: need n_slots > 0 and a result pointer%s");
  apc_timer* t = new apc_timer{n_slots, new hipEvent_t[2 * (size_t)n_slots]};
  for (int i = 0; i < 2 * n_slots; ++i) {
    if (hipEventCreate(&t->ev[i]) != hipSuccess) {
      for (int j = 0; j < i; ++j) (void)hipEventDestroy(t->ev[j]);
      delete[] t->ev;
      delete t;
      return fail(APC_ERR_LAUNCH, "apc_timer_create: hipEventCreate failed%s");
    }
  }
  *timer = t;
  return 0;
}

int apc_timer_destroy(void* timer) {
  apc_timer* t = static_cast<apc_timer*>(timer);
  if (!t) return 0;
  for (int i = 0; i < 2 * t->n; ++i) (void)hipEventDestroy(t->ev[i]);
  delete[] t->ev;
  delete t;
  return 0;
}

int apc_timer_elapsed_ms(void* timer, int32_t slot, float* ms) {
  apc_timer* t = static_cast<apc_timer*>(timer);
  if (!t || slot < 0 || slot >= t->n || !ms) return fail(APC_ERR_INVALID, "apc_timer_elapsed_ms: bad timer or slot%s");
  hipError_t e = hipEventElapsedTime(ms, t->ev[2 * slot], t->ev[2 * slot + 1]);
  if (e != hipSuccess) {
    snprintf(g_err, sizeof(g_err), "apc_timer_elapsed_ms: %s", hipGetErrorString(e));
    return APC_ERR_LAUNCH;
  }
  return 0;
}

int apc_edge_costs_timed(const apc_problem* p, const double* table, const double* per_arg,
                         double* comm, double* cost, uint8_t* flags, int32_t clamp_inf, void* timer,
                         int32_t slot, void* stream) {
  apc_timer* t = static_cast<apc_timer*>(timer);
  if (!t || slot < 0 || slot >= t->n) return fail(APC_ERR_INVALID, "apc_edge_costs_timed: bad timer or slot%s");
  return launch_edge_costs(p, table, per_arg, comm, cost, flags, clamp_inf, (hipStream_t)stream,
                           t->ev[2 * slot], t->ev[2 * slot + 1]);
}

int apc_build_all(const apc_problem* p, double* table, double* compute, double* per_arg,
                  int32_t* status, double* comm, double* cost, uint8_t* flags, int32_t clamp_inf,
                  void* stream) {
  if (int rc = apc_prepare(p, table, compute, per_arg, status, stream)) return rc;
  return apc_edge_costs(p, table, per_arg, comm, cost, flags, clamp_inf, stream);
}

int apc_build_all_timed(const apc_problem* p, double* table, double* compute, double* per_arg,
                        int32_t* status, double* comm, double* cost, uint8_t* flags,
                        int32_t clamp_inf, void* timer, int32_t slot, void* stream) {
  if (int rc = apc_prepare(p, table, compute, per_arg, status, stream)) return rc;
  return apc_edge_costs_timed(p, table, per_arg, comm, cost, flags, clamp_inf, timer, slot, stream);
}

int apc_calibration_copy(const void* src, void* dst, int64_t nbytes, void* stream) {
  if (!src || !dst || nbytes <= 0 || (nbytes & 15))
    return fail(APC_ERR_INVALID, "apc_calibration_copy: need non-null buffers, nbytes %% 16 == 0%s");
  hipLaunchKernelGGL(calibration_copy_kernel, dim3(256 * 16), dim3(kBlock), 0, (hipStream_t)stream,
                     (const double2_t*)src, (double2_t*)dst, nbytes / 16);
  return check_launch("calibration_copy_kernel");
}

int apc_apply_prefetch_discount(const apc_problem* p, const double* per_arg, double scale,
                                double* comm, double* cost, const uint8_t* flags,
                                unsigned long long* n_modified, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_entry == 0) return 0;
  if (!per_arg || !comm || !cost || !flags || !n_modified)
    return fail(APC_ERR_INVALID, "apc_apply_prefetch_discount: null argument%s");
  unsigned grid;
  if (int rc = slot_grid(p, kBlock, &grid)) return rc;
  hipLaunchKernelGGL(prefetch_discount_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream,
                     *p, per_arg, scale, comm, cost, flags, n_modified);
  return check_launch("prefetch_discount_kernel");
}

int apc_objective_coeffs(const apc_problem* p, const double* cost, double* obj, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_entry == 0) return 0;
  if (!cost || !obj || !p->node_multiplier)
    return fail(APC_ERR_INVALID, "apc_objective_coeffs: null argument%s");
  unsigned grid;
  if (int rc = slot_grid(p, kBlock, &grid)) return rc;
  hipLaunchKernelGGL(objective_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *p, cost,
                     obj);
  return check_launch("objective_kernel");
}

int apc_node_hashes(const apc_problem* p, const int64_t* node_out_list, const int32_t* node_phase,
                    uint64_t* out, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_node == 0) return 0;
  if (!node_out_list || !out) return fail(APC_ERR_INVALID, "apc_node_hashes: null argument%s");
  hipLaunchKernelGGL(node_hash_kernel, dim3((p->n_node + (kBlock / 64) - 1) / (kBlock / 64)), dim3(kBlock),
                     0, (hipStream_t)stream, *p, node_out_list, node_phase, out);
  return check_launch("node_hash_kernel");
}

int apc_export_decision_vars(const apc_problem* p, const double* per_arg, const double* comm,
                             const uint8_t* flags, const int64_t* row_base,
                             const int32_t* row_stride, int32_t* keys, double* vals, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_slot == 0) return 0;
  if (!per_arg || !comm || !flags || !row_base || !row_stride || !keys || !vals)
    return fail(APC_ERR_INVALID, "apc_export_decision_vars: null argument%s");
  unsigned grid;
  if (int rc = slot_grid(p, kBlock, &grid)) return rc;
  hipLaunchKernelGGL(export_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *p, per_arg,
                     comm, flags, row_base, row_stride, keys, vals);
  return check_launch("export_kernel");
}

int apc_solution_terms(const apc_problem* p, const double* per_arg, const double* comm,
                       const double* cost, const uint8_t* flags, const uint16_t* assign,
                       double* terms, int64_t* slot, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_edge == 0) return 0;
  if (!per_arg || !comm || !cost || !flags || !assign || !terms || !slot)
    return fail(APC_ERR_INVALID, "apc_solution_terms: null argument%s");
  hipLaunchKernelGGL(solution_terms_kernel, dim3((p->n_edge + kBlock - 1) / kBlock), dim3(kBlock), 0,
                     (hipStream_t)stream, *p, per_arg, comm, cost, flags, assign, terms, slot);
  return check_launch("solution_terms_kernel");
}

// Launches in chunks: beyond a few hundred thousand lanes walking the graph at
// once, the lanes drift apart and stop sharing cache lines of the entry arrays.
static int launch_score(const apc_problem* p, const double* per_arg, const double* comm,
                        const double* cost, const uint8_t* flags, const uint16_t* assign,
                        bool random, uint64_t seed, int64_t first, int64_t n_assign, double* out,
                        hipStream_t stream) {
  const int64_t kChunk = 262144;
  for (int64_t a0 = 0; a0 < n_assign; a0 += kChunk) {
    const int64_t n = (n_assign - a0 < kChunk) ? (n_assign - a0) : kChunk;
    const uint16_t* asg = assign ? assign + a0 : nullptr;
    double* o = out + a0 * 6;
    if (n_assign < kScoreWaveBelow) {
      const unsigned grid = (unsigned)((n + (kBlock / 64) - 1) / (kBlock / 64));
      if (random)
        hipLaunchKernelGGL(score_wave_kernel<true>, dim3(grid), dim3(kBlock), 0, stream, *p, per_arg,
                           comm, cost, flags, asg, n_assign, seed, first + a0, n, o);
      else
        hipLaunchKernelGGL(score_wave_kernel<false>, dim3(grid), dim3(kBlock), 0, stream, *p,
                           per_arg, comm, cost, flags, asg, n_assign, seed, first + a0, n, o);
    } else {
      const unsigned grid = (unsigned)((n + kBlock - 1) / kBlock);
      if (random)
        hipLaunchKernelGGL(score_kernel<true>, dim3(grid), dim3(kBlock), 0, stream, *p, per_arg, comm,
                           cost, flags, asg, n_assign, seed, first + a0, n, o);
      else
        hipLaunchKernelGGL(score_kernel<false>, dim3(grid), dim3(kBlock), 0, stream, *p, per_arg,
                           comm, cost, flags, asg, n_assign, seed, first + a0, n, o);
    }
    if (int rc = check_launch("score kernel")) return rc;
  }
  return 0;
}

int apc_score_assignments(const apc_problem* p, const double* per_arg, const double* comm,
                          const double* cost, const uint8_t* flags, const uint16_t* assign,
                          int64_t n_assign, double* out, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (n_assign <= 0) return 0;
  if (!per_arg || !comm || !cost || !flags || !assign || !out || !p->node_multiplier)
    return fail(APC_ERR_INVALID, "apc_score_assignments: null argument%s");
  return launch_score(p, per_arg, comm, cost, flags, assign, false, 0, 0, n_assign, out,
                      (hipStream_t)stream);
}

int apc_score_random_assignments(const apc_problem* p, const double* per_arg, const double* comm,
                                 const double* cost, const uint8_t* flags, uint64_t seed,
                                 int64_t first, int64_t n_assign, double* out, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (n_assign <= 0) return 0;
  if (!per_arg || !comm || !cost || !flags || !out || !p->node_multiplier)
    return fail(APC_ERR_INVALID, "apc_score_random_assignments: null argument%s");
  return launch_score(p, per_arg, comm, cost, flags, nullptr, true, seed, first, n_assign, out,
                      (hipStream_t)stream);
}

int apc_score_random_window(const apc_problem* p, const double* per_arg, const double* comm,
                            const double* cost, const uint8_t* flags, uint64_t seed,
                            int64_t first, int64_t n_assign, const int32_t* node_gid,
                            int32_t first_node, const double* init, double* out, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (n_assign <= 0) return 0;
  if (!per_arg || !comm || !cost || !flags || !out || !node_gid || !p->node_multiplier)
    return fail(APC_ERR_INVALID, "apc_score_random_window: null argument%s");
  if (first_node < 0 || first_node > p->n_node)
    return fail(APC_ERR_INVALID, "apc_score_random_window: first_node out of range%s");
  const int64_t kChunk = 262144;  // as launch_score
  for (int64_t a0 = 0; a0 < n_assign; a0 += kChunk) {
    const int64_t n = (n_assign - a0 < kChunk) ? (n_assign - a0) : kChunk;
    hipLaunchKernelGGL(score_window_kernel, dim3((unsigned)((n + kBlock - 1) / kBlock)), dim3(kBlock),
                       0, (hipStream_t)stream, *p, per_arg, comm, cost, flags, seed, first + a0, n,
                       node_gid, first_node, init ? init + a0 * 6 : nullptr, out + a0 * 6);
    if (int rc = check_launch("score_window_kernel")) return rc;
  }
  return 0;
}

int apc_pack_score_records(const apc_problem* p, const double* comm, const double* cost,
                           const uint8_t* flags, apc_score_rec* recs, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_slot == 0) return 0;
  if (!comm || !cost || !flags || !recs)
    return fail(APC_ERR_INVALID, "apc_pack_score_records: null argument%s");
  unsigned grid;
  if (int rc = slot_grid(p, kBlock, &grid)) return rc;
  hipLaunchKernelGGL(score_pack_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, p->n_slot,
                     comm, cost, flags, recs);
  return check_launch("score_pack_kernel");
}

int apc_score_packed(const apc_problem* p, const double* per_arg, const apc_score_rec* recs,
                     const uint16_t* assign, uint64_t seed, int64_t first, int64_t n_assign,
                     const int32_t* node_gid, int32_t first_node, const double* init,
                     double* out, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (n_assign <= 0) return 0;
  if (!per_arg || !recs || !out || !p->node_multiplier)
    return fail(APC_ERR_INVALID, "apc_score_packed: null argument%s");
  if (first_node < 0 || first_node > p->n_node)
    return fail(APC_ERR_INVALID, "apc_score_packed: first_node out of range%s");
  const int64_t kChunk = 262144;  // as launch_score
  for (int64_t a0 = 0; a0 < n_assign; a0 += kChunk) {
    const int64_t n = (n_assign - a0 < kChunk) ? (n_assign - a0) : kChunk;
    const dim3 grid((unsigned)((n + kBlock - 1) / kBlock));
    const double* in = init ? init + a0 * 6 : nullptr;
    if (assign)
      hipLaunchKernelGGL(score_packed_kernel<false>, grid, dim3(kBlock), 0, (hipStream_t)stream, *p,
                         per_arg, recs, assign + a0, n_assign, seed, first + a0, n, node_gid,
                         first_node, in, out + a0 * 6);
    else
      hipLaunchKernelGGL(score_packed_kernel<true>, grid, dim3(kBlock), 0, (hipStream_t)stream, *p,
                         per_arg, recs, assign, n_assign, seed, first + a0, n, node_gid, first_node,
                         in, out + a0 * 6);
    if (int rc = check_launch("score_packed_kernel")) return rc;
  }
  return 0;
}

uint32_t apc_random_assignment(uint64_t seed, int64_t a, int32_t node, int32_t nstrat) {
  return mix_assignment(seed, a, node, nstrat);
}

int apc_local_shapes(const apc_model* model, int32_t n, const int32_t* rank, const int64_t* shape,
                     const int64_t* stride, const uint8_t* plc, int64_t* out_shape,
                     int64_t* out_stride, void* stream) {
  if (!model || model->ndim < 1 || model->ndim > APC_MAX_MESH_DIMS)
    return fail(APC_ERR_INVALID, "apc_local_shapes: bad model%s");
  if (n <= 0) return 0;
  if (!rank || !shape || !stride || !plc || !out_shape || !out_stride)
    return fail(APC_ERR_INVALID, "apc_local_shapes: null argument%s");
  hipLaunchKernelGGL(local_shape_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0,
                     (hipStream_t)stream, *model, n, rank, shape, stride, plc, out_shape, out_stride);
  return check_launch("local_shape_kernel");
}

int apc_collective_costs(const apc_model* model, int32_t n, const int32_t* kind,
                         const int64_t* nbytes, const int32_t* dim, double* out, void* stream) {
  if (!model || model->ndim < 1 || model->ndim > APC_MAX_MESH_DIMS)
    return fail(APC_ERR_INVALID, "apc_collective_costs: bad model%s");
  if (n <= 0) return 0;
  if (!kind || !nbytes || !dim || !out)
    return fail(APC_ERR_INVALID, "apc_collective_costs: null argument%s");
  hipLaunchKernelGGL(collective_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0,
                     (hipStream_t)stream, *model, n, kind, nbytes, dim, out);
  return check_launch("collective_kernel");
}

int apc_rw_times(const apc_model* model, int32_t n, const double* nbytes, double* out,
                 void* stream) {
  if (!model) return fail(APC_ERR_INVALID, "apc_rw_times: null model%s");
  if (n <= 0) return 0;
  if (!nbytes || !out) return fail(APC_ERR_INVALID, "apc_rw_times: null argument%s");
  hipLaunchKernelGGL(rw_time_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0,
                     (hipStream_t)stream, *model, n, nbytes, out);
  return check_launch("rw_time_kernel");
}

int apc_enumerate_input_options(const apc_model* model, int32_t n, const int32_t* rank,
                                const int64_t* shape, const int64_t* cand_off, uint8_t* valid,
                                uint8_t* plc, void* stream) {
  if (!model || model->ndim < 1 || model->ndim > APC_MAX_MESH_DIMS)
    return fail(APC_ERR_INVALID, "apc_enumerate_input_options: bad model%s");
  if (n <= 0) return 0;
  if (!rank || !shape || !cand_off || !valid || !plc)
    return fail(APC_ERR_INVALID, "apc_enumerate_input_options: null argument%s");
  hipLaunchKernelGGL(enumerate_kernel, dim3(grid_for((int64_t)n * 64, kBlock)), dim3(kBlock), 0,
                     (hipStream_t)stream, *model, n, rank, shape, cand_off, valid, plc);
  return check_launch("enumerate_kernel");
}

}  // extern "C"
