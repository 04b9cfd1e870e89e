// Device functions and host helpers shared by the translation units of
// libapc_hip.so (internal: the C ABI is include/apc.h).
//
// The cost model lives here as scalar device functions whose order of
// operations is the contract: all floating-point code is compiled with
// -ffp-contract=off, the reference is a chain of separately rounded binary64
// operations, and the results are bit-identical to it.
#ifndef APC_DEVICE_H_
#define APC_DEVICE_H_
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "apc.h"

// Host helpers, defined once (apc.hip).
namespace apc_impl {
#define APC_HIDDEN __attribute__((visibility("hidden")))
extern APC_HIDDEN thread_local char g_err[512];  // text behind apc_last_error()
APC_HIDDEN int fail(int code, const char* fmt, const char* detail = "");
APC_HIDDEN int check_launch(const char* what);
APC_HIDDEN int validate_problem(const apc_problem* p);
APC_HIDDEN int grid_for(int64_t total, int block);
APC_HIDDEN int slot_grid(const apc_problem* p, int per_block, unsigned* grid);
// The two events of a timer's slot (apc_timer_create); false for a bad timer or slot.
APC_HIDDEN bool timer_events(void* timer, int slot, hipEvent_t* start, hipEvent_t* stop);
// The lookup-table kernels over the problem's own tile lists (lut.hip).
APC_HIDDEN int launch_lut_table(const apc_problem* p, double* table, hipStream_t stream);
APC_HIDDEN int launch_lut_entries(const apc_problem* p, const double* per_arg, double* comm, double* cost,
                                  uint8_t* flags, int clamp_inf, hipStream_t stream, hipEvent_t start,
                                  hipEvent_t stop);
}  // namespace apc_impl

namespace {

using apc_impl::check_launch;
using apc_impl::fail;
using apc_impl::grid_for;
using apc_impl::slot_grid;
using apc_impl::validate_problem;

constexpr uint32_t kTupleMask = (1u << APC_TUPLE_BITS) - 1u;
constexpr int kKindMask = 0xC0, kShard = 0x40, kPartial = 0x80, kArgMask = 0x3F;
constexpr int kPartialSum = 0x80;
constexpr int kBlock = 256;

typedef double double2_t __attribute__((ext_vector_type(2)));
typedef long long ll2_t __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------------------
// Cost model, scalar device functions (order of operations is the contract)
// ---------------------------------------------------------------------------

// x / d, correctly rounded.  A quotient by a power of two is the product with
// its reciprocal, bit for bit (both are the one correctly rounded value of the
// same real number), and costs one instruction instead of a division sequence:
// mesh sizes, shard counts and the MI355X memory bandwidth (8 * 1024^4 B/s) are
// powers of two.  The branch is on the divisor, which is the same for every
// lane of a wavefront wherever this is called with a model constant.
__device__ __forceinline__ double div_exact(double x, double d) {
  const uint64_t bits = (uint64_t)__double_as_longlong(d);
  const uint64_t exp = (bits >> 52) & 0x7FF;
  // a normal power of two whose reciprocal is normal too
  if ((bits & 0x800FFFFFFFFFFFFFull) == 0 && exp >= 2 && exp <= 2044)
    return x * __longlong_as_double((long long)((2046 - exp) << 52));
  return x / d;
}

// x / n for a positive integer n
__device__ __forceinline__ double div_int(double x, int64_t n) {
  if ((n & (n - 1)) == 0 && n > 0 && n < (1ll << 62))
    return x * __longlong_as_double((long long)((uint64_t)(1023 - (63 - __clzll((unsigned long long)n))) << 52));
  return x / (double)n;
}

// compute_read_write_time (compute_estimation.py:391-403)
__device__ __forceinline__ double rw_time(double nbytes, double gmem_bw) {
  double t = div_exact(nbytes, gmem_bw) * 1e6;
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
  // an all_to_all may see another bandwidth than the ring collectives (direct links)
  const double dim_bw = (kind == 1 && m.mesh_a2a_bw[i] > 0.0) ? m.mesh_a2a_bw[i] : m.mesh_bw[i];
  double bw = div_int(g * (double)hops, n) / dim_bw;
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
  double gb = div_int((double)tensor_bytes, num_shards) / 1024.0 / 1024.0 / 1024.0;
  // order rule of estimate_strategy_comms_cost (:253-258), or an order forced by
  // the caller of redistribute_cost (order_mode 1: 0..ndim-1, 2: ndim-1..0)
  const bool reversed =
      m.order_mode == 0
          ? ((ndim == 2) && (src == (uint32_t)(kPartialSum | (kPartialSum << 8))) && tgt_all_shard)
          : (m.order_mode == 2);
  // The lanes of a wavefront hold unrelated (source, target) pairs, so a branch
  // per transition kind would make every wavefront walk all of them, each with
  // its own divisions.  Instead a step selects the operands of the one
  // collective and the one read/write time it may need and evaluates those
  // once; which of the reference's additions happen is decided by predicates.
  // An addition that the reference does not make is skipped, not made with
  // zero, except `copies * rw` of Shard -> Shard, which the reference also adds
  // when copies is 0.
  double cost = 0.0;
  bool forbidden = false;
  for (int step = 0; step < ndim; ++step) {
    const int i = reversed ? (ndim - 1 - step) : step;
    const int cur = (src >> (8 * i)) & 0xFF, tg = (tgt >> (8 * i)) & 0xFF;
    if (cur == tg) continue;
    const int n = m.mesh_shape[i];
    const int ck = cur & kKindMask, tk = tg & kKindMask;
    const bool s_r = ck == kShard && tg == 0;      // allgather, on gb * n
    const bool s_s = ck == kShard && tk == kShard;  // all_to_all
    const bool p_r = ck == kPartial && tg == 0;     // allreduce
    const bool p_s = ck == kPartial && tk == kShard;  // reduce_scatter, then gb / n
    forbidden |= (ck == kShard && tk == kPartial) || (cur == 0 && tk == kPartial);
    if (!contiguous) cost += rw_time(gb * 2.0 * 1073741824.0, m.gmem_bw);
    if (s_r | s_s | p_r | p_s) {
      if (s_r) gb = gb * (double)n;
      const int kind = s_r ? 0 : s_s ? 1 : p_r ? 2 : 3;
      cost += collective_cost(kind, (int64_t)(gb * 1073741824.0), i, m);
      // reshuffle penalties: S(d != 0) -> R on the gathered bytes, each side of
      // S(d) -> S(d') that is not dim 0, P -> S(d' != 0)
      const int copies = s_r ? ((cur & kArgMask) != 0)
                             : s_s ? ((cur & kArgMask) != 0) + ((tg & kArgMask) != 0)
                                   : p_s ? ((tg & kArgMask) != 0) : 0;
      if (s_s | (copies != 0)) {
        const double rw = rw_time(gb * 2.0 * 1073741824.0, m.gmem_bw);
        cost += s_s ? (double)copies * rw : rw;
      }
      if (p_s) gb = div_int(gb, n);
    }
    contiguous = true;
  }
  return forbidden ? INFINITY : cost;
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
// Edge that owns slot idx.  Edge blocks start on multiples of 16 slots, so each
// 16-slot chunk belongs to exactly one edge.
__device__ __forceinline__ apc_edge find_edge(const apc_problem& p, int64_t idx) {
  return p.edges[p.chunk_edge[idx >> APC_CHUNK_SHIFT]];
}

}  // namespace
#endif  // APC_DEVICE_H_
