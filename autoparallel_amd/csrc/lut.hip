// Redistribution costs of whole matrices through a per-source lookup table in
// LDS: the block table of large problems, and the direct evaluation of entries
// when no block table applies (gfx950 / CDNA4).
//
// A redistribution cost is a walk over the mesh dims that adds, per dim whose
// placement changes, one collective and up to two read/write times, all of them
// functions of the bytes in flight at that step.  For a fixed source spec the
// bytes at step s take at most 2^s values: every earlier step either left them
// alone or, if the source is sharded (partial) there and the target replicated
// (sharded), multiplied (divided) them by that dim's size.  So the terms depend
// on the source spec, the step and which earlier steps changed the bytes, not on
// the target: a workgroup owns a tile of one matrix (up to 64 source columns, a
// chunk of target rows), computes those terms once per source column into LDS
// with the cost model's own functions, and an element is then the reference's
// additions in the reference's order over looked-up terms: bit-identical to the
// per-element fold, at a fraction of its arithmetic.
#include "apc_device.h"

namespace {

constexpr int kLutCols = 64;                     // source columns per tile
constexpr int kLutBlock = 512;                   // lanes per tile: eight waves share the tile's lookup tables
constexpr int kLutRows = 1024;                   // target rows per tile
static_assert(sizeof(apc_lut_tile) == 64, "tile record layout");

struct Terms {  // of one (source column, step, mask)
  double coll_a;  // Shard -> Replicate: allgather of the gathered bytes; Partial -> Replicate: allreduce
  double rw_a;    // read/write time of the gathered bytes (S(d != 0) -> R)
  double coll_b;  // Shard -> Shard: all_to_all; Partial -> Shard: reduce_scatter
  double rw_b;    // read/write time of the bytes as they are (non-contiguous source, reshuffles)
};

__device__ __forceinline__ int step_dim(const apc_model& m, int step) {
  return m.order_mode == 2 ? m.ndim - 1 - step : step;
}

// The walk of redistribute_cost (apc_device.h) over looked-up terms.  `lut`: the
// source column's terms, 4 doubles per state, state (step, mask) at
// (1 << step) - 1 + mask.  Branch-free: every step reads its four terms and adds
// three values, each either the term the reference adds at that point or +0.0
// (which leaves a non-negative sum as it is, bit for bit); the lanes of a
// wavefront hold unrelated pairs, so branches would only serialise them.
template <int kNdim>
__device__ __forceinline__ double walk_lut(const double* __restrict__ lut, uint32_t src, uint32_t tgt,
                                           bool contiguous, bool reversed) {
  double cost = 0.0;
  bool forbidden = false;
  uint32_t mask = 0;
#pragma unroll
  for (int step = 0; step < kNdim; ++step) {
    const int i = reversed ? kNdim - 1 - step : step;
    const int cur = (src >> (8 * i)) & 0xFF, tg = (tgt >> (8 * i)) & 0xFF;
    const bool active = cur != tg;
    const double2_t* q = reinterpret_cast<const double2_t*>(lut + (((1u << step) - 1u + mask) << 2));
    const double2_t qa = q[0], qb = q[1];  // coll_a, rw_a | coll_b, rw_b
    const int ck = cur & kKindMask, tk = tg & kKindMask;
    const bool s_r = active && ck == kShard && tg == 0;
    const bool s_s = active && ck == kShard && tk == kShard;
    const bool p_r = active && ck == kPartial && tg == 0;
    const bool p_s = active && ck == kPartial && tk == kShard;
    forbidden |= active && ((ck == kShard && tk == kPartial) || (cur == 0 && tk == kPartial));
    const double pre = (active && !contiguous) ? qb.y : 0.0;
    const double coll = (s_r | p_r) ? qa.x : ((s_s | p_s) ? qb.x : 0.0);
    const bool cur_off0 = (cur & kArgMask) != 0, tg_off0 = (tg & kArgMask) != 0;
    const double copies = (double)((int)cur_off0 + (int)tg_off0);
    const double rw = s_r ? (cur_off0 ? qa.y : 0.0) : s_s ? copies * qb.y : ((p_s && tg_off0) ? qb.y : 0.0);
    cost = ((cost + pre) + coll) + rw;
    if (s_r | p_s) mask |= 1u << step;
    contiguous |= active;
  }
  return forbidden ? INFINITY : cost;
}

// For up to three mesh dims the terms of a (column, state) are laid out by what the
// target asks for at that step, so that a step of an element is one 16-byte read
// chosen by the target's class, three additions and two flag bits, instead of a
// dozen selects among the four raw terms:
//   [0] the read/write time a non-contiguous source pays at its first transition
//   [2 + 2 c], [3 + 2 c]  collective and read/write time if the target's placement at
//       this step is of class c: Replicate, Shard(0), Shard(d > 0), Partial, other
// and per column one word of flags, two bits per (step, class): the transition
// changes the bytes in flight (Shard -> Replicate, Partial -> Shard); it is forbidden
// (-> Partial from Shard or Replicate).  Measured on the 3 000-node stress graph with
// eight waves per tile: 1.70 ms for all entries against 1.94 ms with the raw terms.
constexpr int kClassDoubles = 12;
constexpr int kClasses = 5;
template <int kNdim>
struct LutLayout {
  static constexpr bool by_class = kNdim <= 3;  // four dims: 93 KB by class, more than the static LDS limit
  static constexpr int per_state = by_class ? kClassDoubles : 4;
  static constexpr int stride = ((1 << kNdim) - 1) * per_state + 2;  // 16-byte aligned, off the bank period
};

__device__ __forceinline__ int target_class(int tg) {
  const int k = tg & kKindMask;
  return tg == 0 ? 0 : k == kShard ? ((tg & kArgMask) == 0 ? 1 : 2) : k == kPartial ? 3 : 4;
}

// The same walk over the class layout.  Every value added is the one walk_lut adds
// at that point, or +0.0.
template <int kNdim>
__device__ __forceinline__ double walk_classes(const double* __restrict__ lut, uint32_t col_flags, uint32_t src,
                                               uint32_t tgt, bool contiguous, bool reversed) {
  double cost = 0.0;
  bool forbidden = false;
  uint32_t mask = 0;
#pragma unroll
  for (int step = 0; step < kNdim; ++step) {
    const int i = reversed ? kNdim - 1 - step : step;
    const int cur = (src >> (8 * i)) & 0xFF, tg = (tgt >> (8 * i)) & 0xFF;
    const int cls = target_class(tg);  // the same for a whole row of a matrix
    const bool active = cur != tg;
    const double* q = lut + ((1u << step) - 1u + mask) * kClassDoubles;
    const double pre_term = q[0];
    const double2_t cr = *reinterpret_cast<const double2_t*>(q + 2 + 2 * cls);  // collective, read/write
    const uint32_t fl = (col_flags >> (2 * (step * kClasses + cls))) & 3u;
    const double pre = (active && !contiguous) ? pre_term : 0.0;
    const double coll = active ? cr.x : 0.0;
    const double rw = active ? cr.y : 0.0;
    cost = ((cost + pre) + coll) + rw;
    forbidden |= active && (fl & 2u);
    if (active && (fl & 1u)) mask |= 1u << step;
    contiguous |= active;
  }
  return forbidden ? INFINITY : cost;
}

template <bool kEntries, int kNdim>
__global__ void __launch_bounds__(kLutBlock)
lut_kernel(apc_problem p, const apc_lut_tile* __restrict__ tiles, double* __restrict__ table,
           const double* __restrict__ per_arg, double* __restrict__ comm, double* __restrict__ cost,
           uint8_t* __restrict__ flags, int clamp_inf) {
  using Layout = LutLayout<kNdim>;
  __shared__ __align__(16) double s_lut[kLutCols * Layout::stride];
  __shared__ uint32_t s_flags[kLutCols];  // per column: two bits per (step, class), class layout only
  __shared__ apc_spec_rec s_src[kLutCols];
  __shared__ uint2 s_tgt[kLutRows];  // per target row of the tile: spec word, placement bytes
  const apc_lut_tile t = tiles[blockIdx.x];  // the same for the whole workgroup: scalar registers
  const int tid = threadIdx.x;
  const apc_model& m = p.model;
  constexpr int ndim = kNdim;  // == m.ndim: the launcher picks the instance
  constexpr int nstate = (1 << ndim) - 1;
  const bool reversed = m.order_mode == 2;
  const bool has_producer = (t.flags & APC_EDGE_HAS_PRODUCER) != 0;
  const bool squeezed = (t.flags & APC_EDGE_COMPRESSED) != 0;
  // 1. the tile's source columns
  if (tid < (int)t.ncols) {
    apc_spec_rec r = {APC_SPEC_NONE, 0u, 0};
    if (has_producer) {
      uint32_t j = t.col0 + (uint32_t)tid;
      if (squeezed) j = (uint32_t)p.list_ufirst[(size_t)t.src_list + j];
      r = p.spec_recs[(size_t)t.src_list + j];
    }
    s_src[tid] = r;
  }
  // ... and its target rows
  for (uint32_t rr = tid; rr < t.nrows; rr += kLutBlock) {
    uint2 w = make_uint2(APC_SPEC_NONE, 0u);
    if (has_producer) {
      uint32_t o = t.row0 + rr;
      if (squeezed) o = (uint32_t)p.list_ufirst[(size_t)t.dst_list + o];
      const apc_spec_rec rt = p.spec_recs[(size_t)t.dst_list + o];
      w = make_uint2(rt.word, rt.plc);
    }
    s_tgt[rr] = w;
  }
  __syncthreads();
  // 2. their terms: one task per (column, step, mask)
  if (has_producer) {
    for (int task = tid; task < (int)t.ncols * nstate; task += kLutBlock) {
      const int c = task / nstate, st = task - c * nstate;
      const apc_spec_rec r = s_src[c];
      const uint32_t src = r.plc;
      if (r.word == APC_SPEC_NONE || src == 0u) continue;  // no walk from a missing or fully replicated source
      const int step = 31 - __clz(st + 1);
      const uint32_t mask = (uint32_t)(st + 1) - (1u << step);
      int64_t num_shards = 1;
      for (int i = 0; i < ndim; ++i)
        if (((src >> (8 * i)) & kKindMask) == kShard) num_shards *= m.mesh_shape[i];
      double gb = div_int((double)(r.nbytes2 >> 1), num_shards) / 1024.0 / 1024.0 / 1024.0;
      bool reachable = true;  // a step changes the bytes only from a Shard or a Partial
      for (int k = 0; k < step; ++k) {
        if (!((mask >> k) & 1)) continue;
        const int i = step_dim(m, k);
        const int ck = (src >> (8 * i)) & kKindMask;
        if (ck == kShard) gb = gb * (double)m.mesh_shape[i];
        else if (ck == kPartial) gb = div_int(gb, m.mesh_shape[i]);
        else reachable = false;
      }
      if (!reachable) continue;
      const int i = step_dim(m, step);
      const int ck = (src >> (8 * i)) & kKindMask;
      Terms q = {0.0, 0.0, 0.0, 0.0};
      q.rw_b = rw_time(gb * 2.0 * 1073741824.0, m.gmem_bw);
      if (ck == kShard) {
        const double gathered = gb * (double)m.mesh_shape[i];
        q.coll_a = collective_cost(0, (int64_t)(gathered * 1073741824.0), i, m);
        q.rw_a = rw_time(gathered * 2.0 * 1073741824.0, m.gmem_bw);
        q.coll_b = collective_cost(1, (int64_t)(gb * 1073741824.0), i, m);
      } else if (ck == kPartial) {
        q.coll_a = collective_cost(2, (int64_t)(gb * 1073741824.0), i, m);
        q.coll_b = collective_cost(3, (int64_t)(gb * 1073741824.0), i, m);
      }
      double* out = s_lut + c * Layout::stride + st * Layout::per_state;
      if (!Layout::by_class) {
        out[0] = q.coll_a; out[1] = q.rw_a; out[2] = q.coll_b; out[3] = q.rw_b;
      } else {
        // what walk_lut would pick from the four terms for each class of target
        const bool from_shard = ck == kShard, from_partial = ck == kPartial;
        const bool moves = from_shard || from_partial;
        const bool cur_off0 = (((src >> (8 * i)) & kArgMask) != 0);
        out[0] = q.rw_b;
        out[1] = 0.0;
        out[2] = moves ? q.coll_a : 0.0;                                         // -> Replicate
        out[3] = (from_shard && cur_off0) ? q.rw_a : 0.0;
        out[4] = moves ? q.coll_b : 0.0;                                         // -> Shard(0)
        out[5] = from_shard ? (double)(int)cur_off0 * q.rw_b : 0.0;
        out[6] = moves ? q.coll_b : 0.0;                                         // -> Shard(d > 0)
        out[7] = from_shard ? (double)((int)cur_off0 + 1) * q.rw_b : from_partial ? q.rw_b : 0.0;
        out[8] = 0.0; out[9] = 0.0;                                              // -> Partial
        out[10] = 0.0; out[11] = 0.0;                                            // -> other
      }
    }
    if (Layout::by_class && tid < (int)t.ncols) {
      const uint32_t src = s_src[tid].plc;
      uint32_t fl = 0;
      for (int step = 0; step < ndim; ++step) {
        const int cur = (src >> (8 * step_dim(m, step))) & 0xFF, ck = cur & kKindMask;
        uint32_t bits = 0;
        if (ck == kShard) bits |= 1u << (2 * 0);                                 // Shard -> Replicate gathers
        if (ck == kPartial) bits |= (1u << (2 * 1)) | (1u << (2 * 2));           // Partial -> Shard scatters
        if (ck == kShard || cur == 0) bits |= 2u << (2 * 3);                     // -> Partial is forbidden
        fl |= bits << (2 * kClasses * step);
      }
      s_flags[tid] = fl;
    }
  }
  __syncthreads();
  // 3. the tile's elements, row-major: consecutive lanes write consecutive elements
  const uint32_t total = t.nrows * t.ncols;
  const bool pp_rule = m.order_mode == 0 && ndim == 2;  // (Partial, Partial) -> all-Shard walks the dims backwards
  // One element: its value and transition flag from the two specs, then the store.
  auto element = [&](uint32_t rr, uint32_t c, const apc_spec_rec& rs, uint32_t tgt_word, uint32_t tgt) {
    const uint32_t o = t.row0 + rr, j = t.col0 + c;
    const int64_t at = (int64_t)o * t.ncol + j;  // element of the matrix
    double value;
    int trans = 0;
    bool from_specs = false;
    if (has_producer && rs.word != APC_SPEC_NONE && tgt_word != APC_SPEC_NONE) {
      from_specs = true;
      trans = (rs.word & kTupleMask) != (tgt_word & kTupleMask);
      const uint32_t src = rs.plc;
      const bool contig = (rs.nbytes2 & 1) != 0;
      if (src == 0u) {
        bool any_partial = false;
        for (int i = 0; i < ndim; ++i) any_partial |= (((tgt >> (8 * i)) & kKindMask) == kPartial);
        value = any_partial ? INFINITY : 0.0;
      } else if (pp_rule && src == (uint32_t)(kPartialSum | (kPartialSum << 8)) &&
                 (tgt & kKindMask) == kShard && ((tgt >> 8) & kKindMask) == kShard) {
        value = redistribute_cost(src, tgt, rs.nbytes2 >> 1, contig, m);  // the one pair with its own order
      } else {
        value = Layout::by_class ? walk_classes<kNdim>(s_lut + c * Layout::stride, s_flags[c], src, tgt, contig, reversed)
                                 : walk_lut<kNdim>(s_lut + c * Layout::stride, src, tgt, contig, reversed);
      }
    }
    if (!from_specs) value = p.default_vals[t.default_off + at];  // a missing spec keeps the default row's value
    if (kEntries) {
      const double pa = per_arg[t.comp_base + (int64_t)o];
      double total_cost = (value + pa) + (double)trans;  // optimize_sharding.py:544
      const bool finite = isfinite(total_cost);
      if (clamp_inf && !finite) total_cost = 10000.0;
      const int64_t slot = t.out + at;
      if (comm) comm[slot] = value;
      if (cost) cost[slot] = total_cost;
      if (flags) flags[slot] = (uint8_t)(trans | (finite ? 0 : APC_ENTRY_NONFINITE));
    } else {
      table[t.out + at] = trans ? -value : value;
    }
  };
  if (t.ncols == kLutCols) {
    // A full tile: a wave takes whole rows, lane = column.  The lane keeps its source
    // spec for all of its rows, and what depends on the target alone is the same for the
    // whole wave: it is held in scalar registers, and most of the walk's decisions are
    // made once per row instead of once per element.
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const apc_spec_rec rs = s_src[lane];
    for (uint32_t rr = wave; rr < t.nrows; rr += kLutBlock / 64) {
      const uint2 rt = s_tgt[rr];  // x: word, y: placement bytes
      element(rr, lane, rs, __builtin_amdgcn_readfirstlane(rt.x), __builtin_amdgcn_readfirstlane(rt.y));
    }
  } else {
    for (uint32_t idx = tid; idx < total; idx += kLutBlock) {
      const uint32_t rr = t.magic ? __umulhi(idx, t.magic) : idx, c = idx - rr * t.ncols;
      const uint2 rt = s_tgt[rr];
      element(rr, c, s_src[c], rt.x, rt.y);
    }
  }
}

template <bool kEntries>
void launch_lut(const apc_problem* p, const apc_lut_tile* tiles, int64_t n_tile, double* table, const double* per_arg,
                double* comm, double* cost, uint8_t* flags, int clamp_inf, hipStream_t stream,
                hipEvent_t start = nullptr, hipEvent_t stop = nullptr) {
#define APC_LAUNCH_LUT(N)                                                                                   \
  hipExtLaunchKernelGGL((lut_kernel<kEntries, N>), dim3((unsigned)n_tile), dim3(kLutBlock), 0, stream, start, stop, \
                        0, *p, tiles, table, per_arg, comm, cost, flags, clamp_inf)
  switch (p->model.ndim) {  // validate_problem has checked the range
    case 1: APC_LAUNCH_LUT(1); break;
    case 2: APC_LAUNCH_LUT(2); break;
    case 3: APC_LAUNCH_LUT(3); break;
    default: APC_LAUNCH_LUT(4); break;
  }
#undef APC_LAUNCH_LUT
}

int check_tiles(const apc_problem* p, const apc_lut_tile* tiles, int64_t n_tile, const char* what) {
  if (int rc = validate_problem(p)) return rc;
  if (n_tile < 0 || n_tile > 0x7FFFFFFF || (n_tile > 0 && !tiles)) return fail(APC_ERR_INVALID, "%s: bad tile list", what);
  if (n_tile > 0 && !p->spec_recs) return fail(APC_ERR_INVALID, "%s: needs apc_problem.spec_recs", what);
  // (a tile has at most 64 columns and 1024 rows: the host that made the list guarantees it)
  return 0;
}

}  // namespace

namespace apc_impl {
// The problem's own tile lists, for the entry points that take no list (apc.hip).
int launch_lut_table(const apc_problem* p, double* table, hipStream_t stream) {
  launch_lut<false>(p, p->lut_table_tiles, p->n_lut_table_tile, table, nullptr, nullptr, nullptr, nullptr, 0, stream);
  return check_launch("lut_kernel<table>");
}

int launch_lut_entries(const apc_problem* p, const double* per_arg, double* comm, double* cost, uint8_t* flags,
                       int clamp_inf, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
  launch_lut<true>(p, p->lut_entry_tiles, p->n_lut_entry_tile, nullptr, per_arg, comm, cost, flags, clamp_inf, stream,
                   start, stop);
  return check_launch("lut_kernel<entries>");
}
}  // namespace apc_impl

extern "C" {

int apc_build_pair_table_lut(const apc_problem* p, const apc_lut_tile* tiles, int64_t n_tile, double* table,
                             void* stream) {
  if (int rc = check_tiles(p, tiles, n_tile, "apc_build_pair_table_lut")) return rc;
  if (n_tile == 0) return 0;
  if (!table) return fail(APC_ERR_INVALID, "apc_build_pair_table_lut: null table%s");
  launch_lut<false>(p, tiles, n_tile, table, nullptr, nullptr, nullptr, nullptr, 0, (hipStream_t)stream);
  return check_launch("lut_kernel<table>");
}

int apc_edge_costs_lut(const apc_problem* p, const apc_lut_tile* tiles, int64_t n_tile, const double* per_arg,
                       double* comm, double* cost, uint8_t* flags, int32_t clamp_inf, void* stream) {
  if (int rc = check_tiles(p, tiles, n_tile, "apc_edge_costs_lut")) return rc;
  if (n_tile == 0) return 0;
  if (!per_arg) return fail(APC_ERR_INVALID, "apc_edge_costs_lut: null per_arg%s");
  launch_lut<true>(p, tiles, n_tile, nullptr, per_arg, comm, cost, flags, clamp_inf, (hipStream_t)stream);
  return check_launch("lut_kernel<entries>");
}

/* apc_edge_costs_lut with the timer's events of `slot` at the kernel's begin and end. */
int apc_edge_costs_lut_timed(const apc_problem* p, const apc_lut_tile* tiles, int64_t n_tile, const double* per_arg,
                             double* comm, double* cost, uint8_t* flags, int32_t clamp_inf, void* timer,
                             int32_t slot, void* stream) {
  if (int rc = check_tiles(p, tiles, n_tile, "apc_edge_costs_lut_timed")) return rc;
  hipEvent_t start, stop;
  if (!apc_impl::timer_events(timer, slot, &start, &stop))
    return fail(APC_ERR_INVALID, "apc_edge_costs_lut_timed: bad timer or slot%s");
  if (n_tile == 0) return 0;
  if (!per_arg) return fail(APC_ERR_INVALID, "apc_edge_costs_lut_timed: null per_arg%s");
  launch_lut<true>(p, tiles, n_tile, nullptr, per_arg, comm, cost, flags, clamp_inf, (hipStream_t)stream, start, stop);
  return check_launch("lut_kernel<entries>");
}

}  // extern "C"
