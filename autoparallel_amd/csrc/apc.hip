// HIP kernels and C ABI of the sharding-search cost engine (gfx950 / CDNA4).
//
// Everything here is HBM-bound integer/fp64 scalar work: no matrix cores.  The
// entry kernel is a flat scan over the E cost entries: consecutive lanes own
// consecutive entries, so every store instruction writes 512 contiguous bytes
// (fp64) or 64 bytes (flag bytes).  All floating-point code is compiled with
// -ffp-contract=off: the reference is a chain of separately rounded binary64
// operations, and the results here are bit-identical to it.
#include <hip/hip_runtime.h>
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
__device__ __forceinline__ double collective_cost(int kind, int64_t nbytes, int i,
                                                  const apc_model& m) {
  double g = (double)nbytes / 1073741824.0;
  int n = m.mesh_shape[i];
  int hops = (kind == 2) ? 2 * (n - 1) : (n - 1);
  double latency = 6.6 + (double)hops * m.mesh_lat[i];
  double bw = (g * (double)hops / (double)n) / m.mesh_bw[i];
  double t = latency + bw * 1e6;
  if (kind == 1) t = t * 5.0;
  return t;
}

// check_contiguous_sizes_strides (torch _prims_common/__init__.py:252-293)
__device__ __forceinline__ bool is_contiguous(const int64_t* shape, const int64_t* stride,
                                              int rank) {
  int64_t expected = 1, expected_max = 1;
  for (int d = rank - 1; d >= 0; --d) {
    int64_t x = shape[d], y = stride[d];
    if (x == 1) continue;
    if (y != expected && y != expected_max) return false;
    expected_max *= (x > 1 ? x : 1);
    expected *= x;
  }
  return true;
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
  const bool reversed =
      (ndim == 2) && (src == (uint32_t)(kPartialSum | (kPartialSum << 8))) && tgt_all_shard;
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

__device__ __forceinline__ int64_t meta_bytes(const apc_problem& p, uint32_t mid) {
  int rank = p.meta_rank[mid];
  int64_t b = p.meta_itemsize[mid];
  const int64_t* sh = p.meta_shape + (size_t)mid * APC_MAX_RANK;
  for (int d = 0; d < rank; ++d) b *= sh[d];
  return b;
}

__device__ __forceinline__ bool meta_contiguous(const apc_problem& p, uint32_t mid) {
  return is_contiguous(p.meta_shape + (size_t)mid * APC_MAX_RANK,
                       p.meta_stride + (size_t)mid * APC_MAX_RANK, p.meta_rank[mid]);
}

// ---------------------------------------------------------------------------
// Kernel: pair table  T[m][src tuple][tgt tuple]
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) pair_table_kernel(apc_problem p, double* __restrict__ table) {
  const int64_t nt = p.n_tuple;
  const int64_t per_meta = nt * nt;
  const int64_t total = per_meta * p.n_meta;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const uint32_t mid = (uint32_t)(idx / per_meta);
    const int64_t r = idx - (int64_t)mid * per_meta;
    const uint32_t s = (uint32_t)(r / nt), t = (uint32_t)(r - (int64_t)s * nt);
    table[idx] = redistribute_cost(load_tuple(p.tuple_plc, s), load_tuple(p.tuple_plc, t),
                                   meta_bytes(p, mid), meta_contiguous(p, mid), p.model);
  }
}

// ---------------------------------------------------------------------------
// Kernel: node compute estimate
// ---------------------------------------------------------------------------
// Local size of dim d of the tensor behind spec word w: the global size, ceil-
// divided by each mesh dim that shards d, in mesh-dim order
// (_get_sharded_shape_stride, compute_estimation.py:300-318).
__device__ __forceinline__ int64_t local_size(const apc_problem& p, uint32_t w, int d) {
  const uint32_t mid = w >> APC_TUPLE_BITS;
  int64_t s = p.meta_shape[(size_t)mid * APC_MAX_RANK + d];
  const uint32_t plc = load_tuple(p.tuple_plc, w & kTupleMask);
  for (int i = 0; i < p.model.ndim; ++i) {
    const int c = (plc >> (8 * i)) & 0xFF;
    if ((c & kKindMask) == kShard && (c & kArgMask) == d) {
      const int64_t n = p.model.mesh_shape[i];
      s = (s + n - 1) / n;
    }
  }
  return s;
}

__device__ __forceinline__ int64_t local_numel(const apc_problem& p, uint32_t w) {
  const int rank = p.meta_rank[w >> APC_TUPLE_BITS];
  int64_t n = 1;
  for (int d = 0; d < rank; ++d) n *= local_size(p, w, d);
  return n;
}

__global__ void __launch_bounds__(256)
node_compute_kernel(apc_problem p, double* __restrict__ compute, double* __restrict__ per_arg,
                    int32_t* __restrict__ status) {
  const int64_t total = p.node_comp_off[p.n_node];
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    // node owning idx: last v with node_comp_off[v] <= idx
    int lo = 0, hi = p.n_node;
    while (hi - lo > 1) {
      int mid = (lo + hi) >> 1;
      if (p.node_comp_off[mid] <= idx) lo = mid; else hi = mid;
    }
    const int v = lo;
    const int o = (int)(idx - p.node_comp_off[v]);
    const int nargs = p.node_nargs[v];
    const int op = p.node_op[v];
    if (op == APC_OP_ZERO) {
      compute[idx] = 0.0;
      per_arg[idx] = 0.0 / (double)nargs;
      continue;
    }
    const int e0 = p.node_edge_off[v], e1 = p.node_edge_off[v + 1];
    int64_t flops = 0, nbytes = 0;
    int dtype = 1;  // float32 when the node has no tensor argument
    bool have_dtype = false;
    for (int e = e0; e < e1; ++e) {
      const uint32_t w = p.lists[(size_t)p.edges[e].dst_list + o];
      if (w == APC_SPEC_NONE) continue;
      if (!have_dtype) { dtype = p.meta_dtype[w >> APC_TUPLE_BITS]; have_dtype = true; }
    }
    if (op == APC_OP_EXPLICIT) {
      flops = p.explicit_flops[idx];
      nbytes = p.explicit_bytes[idx];
    } else {
      for (int e = e0; e < e1; ++e) {
        const uint32_t w = p.lists[(size_t)p.edges[e].dst_list + o];
        if (w == APC_SPEC_NONE) continue;
        nbytes += local_numel(p, w) * (int64_t)p.meta_itemsize[w >> APC_TUPLE_BITS];
      }
      const int64_t* pr = p.prog + p.node_prog_off[v];
      const int n_terms = (int)pr[0], n_outs = (int)pr[1];
      pr += 2;
      for (int t = 0; t < n_terms; ++t) {
        int64_t term = pr[0];
        const int nfac = (int)pr[1];
        pr += 2;
        for (int f = 0; f < nfac; ++f) {
          const uint32_t w = p.lists[(size_t)p.edges[e0 + (int)pr[0]].dst_list + o];
          term *= local_size(p, w, (int)pr[1]);
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
            const uint32_t w = p.lists[(size_t)p.edges[e0 + (int)pr[1]].dst_list + o];
            size = local_size(p, w, (int)pr[2]);
          } else {  // broadcast of all tensor args at a right-aligned position
            size = 1;
            const int pos = (int)pr[1];
            for (int e = e0; e < e1; ++e) {
              const uint32_t w = p.lists[(size_t)p.edges[e].dst_list + o];
              if (w == APC_SPEC_NONE) continue;
              const int r = p.meta_rank[w >> APC_TUPLE_BITS];
              if (pos >= r) continue;
              const int64_t s = local_size(p, w, r - 1 - pos);
              if (s != 1) size = s;
            }
          }
          numel *= size;
          pr += 3;
        }
        nbytes += numel * isz;
      }
    }
    // roofline (compute_estimation.py:474-489)
    const double rw = rw_time((double)nbytes, p.model.gmem_bw);
    double result;
    if (flops == 0) {
      result = rw;
    } else {
      const double tf = (dtype >= 0 && dtype < APC_NUM_DTYPES) ? p.model.tflops[dtype] : 0.0;
      if (!(tf > 0.0)) {
        atomicExch(status, 1);
        result = NAN;
      } else {
        const double gpu_flops = tf * 1e12;
        double ct = (double)flops / gpu_flops * 1e6;
        ct = ct / 0.70;
        result = ct >= rw ? ct : rw;  // max(ct, rw): keeps ct on ties
      }
    }
    compute[idx] = result;
    per_arg[idx] = result / (double)nargs;
  }
}

// ---------------------------------------------------------------------------
// Kernel: cost entries
// ---------------------------------------------------------------------------
constexpr int kTile = 1 << APC_TILE_SHIFT;  // entries per workgroup
constexpr int kBlock = 256;

struct EntryOut {
  double comm;
  double pa;
  int trans;
};

// Evaluate entry `local` of edge `ed`.
template <bool kUseTable>
__device__ __forceinline__ EntryOut eval_entry(const apc_problem& p, const apc_edge& ed,
                                               uint32_t local, const double* __restrict__ table,
                                               const double* __restrict__ per_arg) {
  const uint32_t ssrc = (uint32_t)ed.ssrc;
  const uint32_t o = local / ssrc;
  const uint32_t j = local - o * ssrc;
  const uint32_t tw = p.lists[(size_t)ed.dst_list + o];
  const uint32_t sw =
      (ed.flags & APC_EDGE_HAS_PRODUCER) ? p.lists[(size_t)ed.src_list + j] : APC_SPEC_NONE;
  EntryOut r;
  r.pa = per_arg[ed.comp_base + o];
  if (sw != APC_SPEC_NONE && tw != APC_SPEC_NONE) {
    const uint32_t st = sw & kTupleMask, tt = tw & kTupleMask, sm = sw >> APC_TUPLE_BITS;
    r.trans = (st != tt);
    if (kUseTable) {
      r.comm = table[((size_t)sm * p.n_tuple + st) * p.n_tuple + tt];
    } else {
      r.comm = redistribute_cost(load_tuple(p.tuple_plc, st), load_tuple(p.tuple_plc, tt),
                                 meta_bytes(p, sm), meta_contiguous(p, sm), p.model);
    }
  } else {
    r.comm = p.default_vals[ed.default_off + local];
    r.trans = 0;
  }
  return r;
}

// Advance (e, ed) so that edge e contains entry idx.  Entries only move
// forward, so this is a short walk from the tile's first edge.
__device__ __forceinline__ void seek_edge(const apc_problem& p, int64_t idx, int& e, apc_edge& ed) {
  while (idx >= ed.off + (int64_t)ed.ssrc * ed.sdst) {
    ++e;
    ed = p.edges[e];
  }
}

template <bool kUseTable>
__global__ void __launch_bounds__(kBlock)
edge_cost_kernel(apc_problem p, const double* __restrict__ table,
                 const double* __restrict__ per_arg, double* __restrict__ comm,
                 double* __restrict__ cost, uint8_t* __restrict__ flags, int clamp_inf) {
  const int64_t tile0 = (int64_t)blockIdx.x << APC_TILE_SHIFT;
  int e = p.tile_edge[blockIdx.x];
  apc_edge ed = p.edges[e];
#pragma unroll
  for (int u = 0; u < kTile / kBlock; ++u) {
    const int64_t idx = tile0 + u * kBlock + threadIdx.x;
    if (idx >= p.n_entry) break;
    seek_edge(p, idx, e, ed);
    const EntryOut r = eval_entry<kUseTable>(p, ed, (uint32_t)(idx - ed.off), table, per_arg);
    double c = (r.comm + r.pa) + (double)r.trans;
    const bool finite = isfinite(c);
    if (clamp_inf && !finite) c = 10000.0;
    if (comm) comm[idx] = r.comm;
    if (cost) cost[idx] = c;
    if (flags) flags[idx] = (uint8_t)(r.trans | (finite ? 0 : APC_ENTRY_NONFINITE));
  }
}

// ---------------------------------------------------------------------------
// Kernel: prefetch discount
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock)
prefetch_discount_kernel(apc_problem p, const double* __restrict__ per_arg, double scale,
                         double* __restrict__ comm, double* __restrict__ cost,
                         const uint8_t* __restrict__ flags, unsigned long long* n_modified) {
  const int64_t tile0 = (int64_t)blockIdx.x << APC_TILE_SHIFT;
  int e = p.tile_edge[blockIdx.x];
  apc_edge ed = p.edges[e];
  unsigned int mine = 0;
  for (int u = 0; u < kTile / kBlock; ++u) {
    const int64_t idx = tile0 + u * kBlock + threadIdx.x;
    if (idx >= p.n_entry) break;
    seek_edge(p, idx, e, ed);
    if (!(ed.flags & APC_EDGE_PREFETCHABLE) || ed.src_node < 0) continue;
    double c = comm[idx];
    if (c > 0.0 && isfinite(c)) {
      const uint32_t o = (uint32_t)(idx - ed.off) / (uint32_t)ed.ssrc;
      c = c * scale;
      comm[idx] = c;
      cost[idx] = (c + per_arg[ed.comp_base + o]) + (double)(flags[idx] & APC_ENTRY_TRANSITION);
      ++mine;
    }
  }
  // wavefront reduction, one atomic per wave
  for (int off = 32; off > 0; off >>= 1) mine += __shfl_down(mine, off, 64);
  if ((threadIdx.x & 63) == 0 && mine) atomicAdd(n_modified, (unsigned long long)mine);
}

__global__ void __launch_bounds__(kBlock)
objective_kernel(apc_problem p, const double* __restrict__ cost, double* __restrict__ obj) {
  const int64_t tile0 = (int64_t)blockIdx.x << APC_TILE_SHIFT;
  int e = p.tile_edge[blockIdx.x];
  apc_edge ed = p.edges[e];
  for (int u = 0; u < kTile / kBlock; ++u) {
    const int64_t idx = tile0 + u * kBlock + threadIdx.x;
    if (idx >= p.n_entry) break;
    seek_edge(p, idx, e, ed);
    obj[idx] = cost[idx] * (double)p.node_multiplier[ed.node];
  }
}

// ---------------------------------------------------------------------------
// Kernel: batch scoring.  One lane per assignment; the lane walks the graph in
// node order then argument order, so every sum has the reference's order.
// ---------------------------------------------------------------------------
__host__ __device__ __forceinline__ uint32_t mix_assignment(uint64_t seed, int64_t a, int32_t node,
                                                            int32_t nstrat) {
  // splitmix64 finaliser over (seed, assignment, node)
  uint64_t z = seed + 0x9E3779B97F4A7C15ull * (uint64_t)(a + 1) + 0xBF58476D1CE4E5B9ull * (uint64_t)(node + 1);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z = z ^ (z >> 31);
  return (uint32_t)((z >> 32) % (uint64_t)nstrat);
}

template <bool kRandom>
__global__ void __launch_bounds__(kBlock)
score_kernel(apc_problem p, const double* __restrict__ per_arg, const double* __restrict__ comm,
             const double* __restrict__ cost, const uint8_t* __restrict__ flags,
             const uint16_t* __restrict__ assign, uint64_t seed, int64_t first, int64_t n_assign,
             double* __restrict__ out) {
  const int64_t a = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (a >= n_assign) return;
  double t_compute = 0.0, t_comm = 0.0, t_trans = 0.0, obj = 0.0, forbidden = 0.0;
  for (int v = 0; v < p.n_node; ++v) {
    const uint32_t o = kRandom ? mix_assignment(seed, first + a, v, p.node_nstrat[v])
                               : (uint32_t)assign[(size_t)v * n_assign + a];
    const int nargs = p.node_nargs[v];
    const double pa = per_arg[p.node_comp_off[v] + o];
    t_compute += pa * (double)(nargs > 1 ? nargs : 1);
    const double mult = (double)p.node_multiplier[v];
    for (int e = p.node_edge_off[v]; e < p.node_edge_off[v + 1]; ++e) {
      const apc_edge ed = p.edges[e];
      uint32_t j = 0;
      if (ed.src_node >= 0)
        j = kRandom ? mix_assignment(seed, first + a, ed.src_node, p.node_nstrat[ed.src_node])
                    : (uint32_t)assign[(size_t)ed.src_node * n_assign + a];
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

int validate_problem(const apc_problem* p) {
  if (!p) return fail(APC_ERR_INVALID, "null problem%s");
  if (p->model.ndim < 1 || p->model.ndim > APC_MAX_MESH_DIMS)
    return fail(APC_ERR_INVALID, "mesh ndim out of range%s");
  for (int i = 0; i < p->model.ndim; ++i)
    if (p->model.mesh_shape[i] < 1) return fail(APC_ERR_INVALID, "mesh size < 1%s");
  if (p->n_meta < 0 || p->n_tuple < 0 || p->n_tuple > (1 << APC_TUPLE_BITS))
    return fail(APC_ERR_INVALID, "bad meta/tuple counts%s");
  if (p->n_node < 0 || p->n_edge < 0 || p->n_entry < 0)
    return fail(APC_ERR_INVALID, "negative sizes%s");
  if (p->n_tile != (int32_t)((p->n_entry + kTile - 1) >> APC_TILE_SHIFT))
    return fail(APC_ERR_INVALID, "n_tile does not match n_entry%s");
  if (p->n_entry > 0 && (!p->edges || !p->tile_edge || !p->lists))
    return fail(APC_ERR_INVALID, "null edge/list arrays%s");
  return 0;
}

int grid_for(int64_t total, int block) {
  int64_t g = (total + block - 1) / block;
  const int64_t cap = 256 * 32;  // grid-stride kernels: a few waves per CU
  if (g > cap) g = cap;
  if (g < 1) g = 1;
  return (int)g;
}

}  // namespace

extern "C" {

int apc_version(void) { return 1; }

const char* apc_last_error(void) { return g_err; }

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
  return (int64_t)p->n_meta * p->n_tuple * p->n_tuple;
}

int apc_build_pair_table(const apc_problem* p, double* table, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  const int64_t total = apc_pair_table_size(p);
  if (total == 0) return 0;
  if (!table) return fail(APC_ERR_INVALID, "apc_build_pair_table: null table%s");
  hipLaunchKernelGGL(pair_table_kernel, dim3(grid_for(total, 256)), dim3(256), 0,
                     (hipStream_t)stream, *p, table);
  return check_launch("pair_table_kernel");
}

int apc_node_compute_costs(const apc_problem* p, double* compute, double* per_arg,
                           int32_t* status, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_node == 0) return 0;
  if (!compute || !per_arg || !status)
    return fail(APC_ERR_INVALID, "apc_node_compute_costs: null output%s");
  // total strategies is not known on the host side of this ABI without a
  // copy; size the grid from n_node (grid-stride loop covers the rest)
  hipLaunchKernelGGL(node_compute_kernel, dim3(grid_for((int64_t)p->n_node * 16, 256)), dim3(256),
                     0, (hipStream_t)stream, *p, compute, per_arg, status);
  return check_launch("node_compute_kernel");
}

int apc_edge_costs(const apc_problem* p, const double* table, const double* per_arg, double* comm,
                   double* cost, uint8_t* flags, int32_t clamp_inf, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_entry == 0) return 0;
  if (!per_arg) return fail(APC_ERR_INVALID, "apc_edge_costs: null per_arg%s");
  if (table)
    hipLaunchKernelGGL(edge_cost_kernel<true>, dim3(p->n_tile), dim3(kBlock), 0,
                       (hipStream_t)stream, *p, table, per_arg, comm, cost, flags, clamp_inf);
  else
    hipLaunchKernelGGL(edge_cost_kernel<false>, dim3(p->n_tile), dim3(kBlock), 0,
                       (hipStream_t)stream, *p, table, per_arg, comm, cost, flags, clamp_inf);
  return check_launch("edge_cost_kernel");
}

int apc_apply_prefetch_discount(const apc_problem* p, const double* per_arg, double scale,
                                double* comm, double* cost, const uint8_t* flags,
                                unsigned long long* n_modified, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_entry == 0) return 0;
  if (!per_arg || !comm || !cost || !flags || !n_modified)
    return fail(APC_ERR_INVALID, "apc_apply_prefetch_discount: null argument%s");
  hipLaunchKernelGGL(prefetch_discount_kernel, dim3(p->n_tile), dim3(kBlock), 0,
                     (hipStream_t)stream, *p, per_arg, scale, comm, cost, flags, n_modified);
  return check_launch("prefetch_discount_kernel");
}

int apc_objective_coeffs(const apc_problem* p, const double* cost, double* obj, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_entry == 0) return 0;
  if (!cost || !obj || !p->node_multiplier)
    return fail(APC_ERR_INVALID, "apc_objective_coeffs: null argument%s");
  hipLaunchKernelGGL(objective_kernel, dim3(p->n_tile), dim3(kBlock), 0, (hipStream_t)stream, *p,
                     cost, obj);
  return check_launch("objective_kernel");
}

int apc_score_assignments(const apc_problem* p, const double* per_arg, const double* comm,
                          const double* cost, const uint8_t* flags, const uint16_t* assign,
                          int64_t n_assign, double* out, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (n_assign <= 0) return 0;
  if (!per_arg || !comm || !cost || !flags || !assign || !out || !p->node_multiplier)
    return fail(APC_ERR_INVALID, "apc_score_assignments: null argument%s");
  const int64_t grid = (n_assign + kBlock - 1) / kBlock;
  hipLaunchKernelGGL(score_kernel<false>, dim3((unsigned)grid), dim3(kBlock), 0,
                     (hipStream_t)stream, *p, per_arg, comm, cost, flags, assign, 0ull, 0ll,
                     n_assign, out);
  return check_launch("score_kernel");
}

int apc_score_random_assignments(const apc_problem* p, const double* per_arg, const double* comm,
                                 const double* cost, const uint8_t* flags, uint64_t seed,
                                 int64_t first, int64_t n_assign, double* out, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (n_assign <= 0) return 0;
  if (!per_arg || !comm || !cost || !flags || !out || !p->node_multiplier)
    return fail(APC_ERR_INVALID, "apc_score_random_assignments: null argument%s");
  const int64_t grid = (n_assign + kBlock - 1) / kBlock;
  hipLaunchKernelGGL(score_kernel<true>, dim3((unsigned)grid), dim3(kBlock), 0,
                     (hipStream_t)stream, *p, per_arg, comm, cost, flags, (const uint16_t*)nullptr,
                     seed, first, n_assign, out);
  return check_launch("score_kernel<random>");
}

uint32_t apc_random_assignment(uint64_t seed, int64_t a, int32_t node, int32_t nstrat) {
  return mix_assignment(seed, a, node, nstrat);
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
