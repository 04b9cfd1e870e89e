// Batch scoring of candidate assignments against the objective and the
// constraints (gfx950), and its C ABI.
#include "apc_device.h"

namespace {

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

typedef int32_t i32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ apc_score_edge_aux load_aux(const apc_score_edge_aux* __restrict__ a) {
  union { i32x4_t raw; apc_score_edge_aux aux; } u;
  u.raw = *reinterpret_cast<const i32x4_t*>(a);
  return u.aux;
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

// x + 1.0 n times over.  While x is a whole number below 2^52 every step is exact, and so
// is x + n in one step (what the carried sums are in practice: counts); anything else is
// added one by one, as a sequential walk does.
__device__ __forceinline__ double add_ones(double x, uint32_t n) {
  if (x == floor(x) && fabs(x) < 4503599627370496.0 - 4294967296.0) return x + (double)n;
  for (uint32_t i = 0; i < n; ++i) x += 1.0;
  return x;
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
template <bool kRandom>
__global__ void __launch_bounds__(kBlock)
score_window_kernel(apc_problem p, const double* __restrict__ per_arg,
                    const double* __restrict__ comm, const double* __restrict__ cost,
                    const uint8_t* __restrict__ flags, const uint16_t* __restrict__ assign, int64_t stride,
                    uint64_t seed, int64_t first,
                    int64_t n_assign, const int32_t* __restrict__ node_gid, int first_node,
                    const double* __restrict__ init, double* __restrict__ out) {
  const int64_t a = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (a >= n_assign) return;
  // the choice at node v: drawn from its id in the whole graph, or read from the matrix
  auto choice = [&](int v, int nstrat) -> uint32_t {
    return kRandom ? mix_assignment(seed, first + a, node_gid ? node_gid[v] : v, nstrat)
                   : (uint32_t)assign[(size_t)v * stride + a];
  };
  double t_compute = 0.0, t_comm = 0.0, t_trans = 0.0, obj = 0.0, forbidden = 0.0;
  if (init) {
    const double* r = init + a * 6;
    t_compute = r[1]; t_comm = r[2]; t_trans = r[3]; obj = r[4]; forbidden = r[5];
  }
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
      uint32_t j = 0;
      if (ed.src_node >= 0) j = choice(ed.src_node, ed.ssrc);
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

// ---------------------------------------------------------------------------
// Compact records and the walk over them: what scoring falls back to on a graph
// with large blocks when it cannot read the block table (no table, or entry
// arrays that something changed after the build).
//
// A drawn entry is one random read inside its edge's block, and the walk runs at
// the rate at which a CU has cache misses served, wherever the line comes from
// (measured: with the blocks kept in L2, 93% hits instead of 27%, the same time).
// What helps is fewer and better used requests:
//   - the record is {comm, flags}, 16 bytes: the cost of an entry is (comm +
//     per_arg) + transition, clamped or not, and the lane holds per_arg of its
//     node's choice already, so cost need not be stored;
//   - a lane carries kPer assignments, whose reads of an edge are independent and
//     issued back to back, and the whole batch walks the graph once.
// Measured on a 3000-node window of the stress DAG, 2^20 assignments: 99 ms from
// 32-byte records in launches of 2^18 lanes, 70-80 ms here with kPer = 8.
// The sums of an assignment run in node order, then argument order, as in
// score_kernel: same results, bit for bit.
// ---------------------------------------------------------------------------

// One lane per slot.  mismatch[0] is set if some cost is neither (comm + per_arg)
// + transition nor that sum's clamp: then the compact records cannot stand for
// the arrays and the caller must not use them.
__global__ void __launch_bounds__(kBlock)
score_pack16_kernel(apc_problem p, const double* __restrict__ per_arg, const double* __restrict__ comm,
                    const double* __restrict__ cost, const uint8_t* __restrict__ flags,
                    apc_score_rec16* __restrict__ recs, int32_t* __restrict__ mismatch) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= p.n_slot) return;
  const apc_edge* ed = p.edges + p.chunk_edge[i >> 4];
  const int64_t l = i - ed->off;
  const int ssrc = ed->ssrc;
  apc_score_rec16 r;
  r.comm = 0.0;
  r.flags = 0;
  if (l < (int64_t)ssrc * ed->sdst) {  // else padding behind the block
    const uint32_t o = (uint32_t)l / (uint32_t)ssrc;
    const double cm = comm[i], c = cost[i];
    const uint32_t f = flags[i];
    const double want = (cm + per_arg[ed->comp_base + o]) + (double)(int)(f & APC_ENTRY_TRANSITION);
    bool bad = ((f & APC_ENTRY_NONFINITE) != 0) != !isfinite(want);
    uint64_t extra = 0;
    if (__double_as_longlong(c) != __double_as_longlong(want)) {
      if (c == 10000.0 && !isfinite(want)) extra = APC_SCORE_CLAMPED;
      else bad = true;
    }
    if (bad) atomicOr(mismatch, 1);
    r.comm = cm;
    r.flags = (uint64_t)f | extra;
  }
  recs[i] = r;
}

__global__ void clear_flag_kernel(int32_t* flag) { *flag = 0; }

template <bool kRandom, int kPer>
__global__ void __launch_bounds__(kBlock)
score_compact_kernel(apc_problem p, const double* __restrict__ per_arg,
                     const apc_score_rec16* __restrict__ recs, const uint16_t* __restrict__ assign,
                     int64_t stride, uint64_t seed, int64_t first, int64_t n_assign,
                     const int32_t* __restrict__ node_gid, int first_node, int end_node,
                     const double* __restrict__ init, double* __restrict__ out) {
  const int64_t lanes = (int64_t)gridDim.x * blockDim.x;
  const int64_t t_raw = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t_raw >= n_assign) return;
  const int64_t t = t_raw;
  // assignment k of this lane; a lane past the end repeats another one and stores nothing
  auto asg = [&](int k) -> int64_t {
    const int64_t ak = t_raw + k * lanes;
    return ak < n_assign ? ak : t;
  };
  double t_compute[kPer], t_comm[kPer], t_trans[kPer], obj[kPer], forbidden[kPer];
  uint32_t h0[kPer];
#pragma unroll
  for (int k = 0; k < kPer; ++k) {
    t_compute[k] = 0.0; t_comm[k] = 0.0; t_trans[k] = 0.0; obj[k] = 0.0; forbidden[k] = 0.0;
    if (init) {
      const double* r = init + asg(k) * 6;
      t_compute[k] = r[1]; t_comm[k] = r[2]; t_trans[k] = r[3]; obj[k] = r[4]; forbidden[k] = r[5];
    }
    // the part of mix_assignment that does not depend on the node
    const uint64_t ua = (uint64_t)(first + asg(k));
    uint32_t h = (uint32_t)seed ^ ((uint32_t)(seed >> 32) * 0x27D4EB2Fu);
    h ^= (uint32_t)ua * 0x9E3779B1u;
    h ^= (uint32_t)(ua >> 32) * 0x85EBCA77u;
    h0[k] = h;
  }
  auto choice = [&](int k, int v, int nstrat) -> uint32_t {
    if (!kRandom) return (uint32_t)assign[(size_t)v * stride + asg(k)];
    uint32_t h = h0[k] ^ ((uint32_t)((node_gid ? node_gid[v] : v) + 1) * 0xC2B2AE3Du);
    h ^= h >> 16;
    h *= 0x85EBCA6Bu;
    h ^= h >> 13;
    h *= 0xC2B2AE35u;
    h ^= h >> 16;
    return (uint32_t)(((uint64_t)h * (uint64_t)(uint32_t)nstrat) >> 32);
  };
  apc_edge nxt;
  if (first_node < p.n_node && p.node_edge_off[first_node] < p.n_edge)
    nxt = load_edge(p.edges + p.node_edge_off[first_node]);
  for (int v = first_node; v < end_node; ++v) {
    const int nstrat = p.node_nstrat[v];
    const int nargs = p.node_nargs[v];
    const double fargs = (double)(nargs > 1 ? nargs : 1);
    const double mult = (double)p.node_multiplier[v];
    const int64_t comp_off = p.node_comp_off[v];
    uint32_t o[kPer];
    double pa[kPer];
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
      o[k] = choice(k, v, nstrat);
      pa[k] = per_arg[comp_off + o[k]];
    }
#pragma unroll
    for (int k = 0; k < kPer; ++k) t_compute[k] += pa[k] * fargs;
    for (int e = p.node_edge_off[v]; e < p.node_edge_off[v + 1]; ++e) {
      const apc_edge ed = nxt;
      if (e + 1 < p.n_edge) nxt = load_edge(p.edges + e + 1);
      const bool has_src = ed.src_node >= 0;
      apc_score_rec16 r[kPer];
#pragma unroll
      for (int k = 0; k < kPer; ++k) {
        const uint32_t j = has_src ? choice(k, ed.src_node, ed.ssrc) : 0u;  // ssrc: the producer's count
        r[k] = recs[ed.off + (int64_t)o[k] * ed.ssrc + j];
      }
      const bool count_trans = has_src && (ed.flags & APC_EDGE_SCORE_TRANSITION);
#pragma unroll
      for (int k = 0; k < kPer; ++k) {
        const uint32_t f = (uint32_t)r[k].flags;
        double c = (r[k].comm + pa[k]) + (double)(int)(f & APC_ENTRY_TRANSITION);
        if (f & (uint32_t)APC_SCORE_CLAMPED) c = 10000.0;
        obj[k] += c * mult;
        forbidden[k] += (double)((f & APC_ENTRY_NONFINITE) != 0);
        if (has_src && isfinite(r[k].comm)) t_comm[k] += r[k].comm;
        if (count_trans && (f & APC_ENTRY_TRANSITION)) t_trans[k] += 1.0;
      }
    }
  }
#pragma unroll
  for (int k = 0; k < kPer; ++k) {
    if (t_raw + k * lanes >= n_assign) continue;
    double* r = out + asg(k) * 6;
    r[0] = (t_compute[k] + t_comm[k]) + t_trans[k];
    r[1] = t_compute[k];
    r[2] = t_comm[k];
    r[3] = t_trans[k];
    r[4] = obj[k];
    r[5] = forbidden[k];
  }
}

// ---------------------------------------------------------------------------
// Scoring from the block table, for graphs whose blocks are large.
//
// A drawn entry of a block of 10^5 entries is a random read that misses the
// CU's cache, and the walk over such records runs at the rate at which a CU
// can have misses served (measured: one per 8 cycles per CU whether the line
// comes from L2 or from memory; 7e10 draws/s on the whole chip).  The block
// table holds the same numbers in far less room: an edge's matrix has one row
// per distinct consumer spec word and one column per distinct producer spec
// word (8 times fewer elements than the blocks on the stress DAG, 63 KB a
// matrix on average), and an entry is (|m| + per_arg) + transition with the
// transition flag in m's sign, clamped or not: what the build makes of it
// (item_store in apc.hip).  So one workgroup per CU, 1024 lanes with kPer
// assignments each, has the matrix of the current edge in LDS and draws from
// there.  The matrix comes in by loads that write LDS directly
// (global_load_lds: no registers in between), into one of two buffers: the
// loads of the next edge's matrix are issued before the draws of the current
// one.  Matrices larger than a buffer are taken in several tiles; very large
// ones and the default rows of edges without a producer are read in place.
// The sums of an assignment run in node order, then argument order, as in
// score_kernel: same results, bit for bit, as scoring the entry arrays that a
// build with the same clamp_inf wrote.
// ---------------------------------------------------------------------------
constexpr int kTileDoubles = 8192;  // 64 KB: a tile of a matrix
constexpr int kListInts = 1024;     // an index list that goes through LDS
constexpr int kLanes = 1024;        // one workgroup per CU
constexpr int kBufs = 2;            // tile buffers: the next edge's matrix arrives while the lanes draw from this one
constexpr int kTableLds = kBufs * kTileDoubles * 8 + kBufs * 2 * kListInts * 4;  // 144 KB
// Measured on a 3 000-node window of the stress DAG, 2^20 assignments, where this shape
// takes 18.3 ms: two workgroups of 512 lanes per CU with one buffer each, which overlap
// each other instead of prefetching, 24.4 ms; a quarter of the waves (by turns) issuing
// the whole copy while the others go on to their draws, 25.0 ms.

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// Lane i's 16 (4) bytes src[i] -> LDS, for the lanes with i < n.  lds_wave is the LDS
// byte address of the element of the wave's first lane; the hardware adds lane * 16
// (lane * 4).  The load is written out by hand because the compiler, which cannot
// tell these LDS writes from the LDS reads of the draws, would wait for it before the
// next LDS read, and the point is that it stays in flight while the lanes draw from
// the other buffer.  So the compiler does not count it either: the code that needs
// the data waits for the vector-memory counter itself.  (Loads complete in order, so the
// compiler's own counts for its own loads only ever wait longer than they must.)
// m0 holds the LDS address for the load; the compiler keeps m0 for its own uses
// (it is a reserved register, which a clobber list cannot name), so the statement
// puts back what it found there.
__device__ __forceinline__ void copy16_to_lds(const double2_t* __restrict__ src, uint32_t lds_wave, int i, int n) {
  if (i < n) {
    const uint32_t m = __builtin_amdgcn_readfirstlane(lds_wave);
    const double2_t* g = src + i;
    uint32_t saved;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved) : "s"(m), "v"(g) : "memory");
  }
}
__device__ __forceinline__ void copy4_to_lds(const int32_t* __restrict__ src, uint32_t lds_wave, int i, int n) {
  if (i < n) {
    const uint32_t m = __builtin_amdgcn_readfirstlane(lds_wave);
    const int32_t* g = src + i;
    uint32_t saved;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 3\n\tglobal_load_lds_dword %2, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved) : "s"(m), "v"(g) : "memory");
  }
}

// Every vector-memory operation of this wave has completed (the copies into LDS
// among them); scalar loads requested ahead (the next edge's and node's records)
// stay in flight.  s_waitcnt fields of gfx9: vmcnt [3:0] and [15:14], expcnt [6:4],
// lgkmcnt [11:8].
__device__ __forceinline__ void wait_vector_memory() { __builtin_amdgcn_s_waitcnt(0x0F70); }

template <bool kRandom, int kPer>
__global__ void __launch_bounds__(kLanes)
score_table_kernel(apc_problem p, const double* __restrict__ per_arg, const double* __restrict__ table,
                   const apc_score_edge_aux* __restrict__ edge_aux,
                   const uint16_t* __restrict__ assign, int64_t stride, uint64_t seed, int64_t first,
                   int64_t n_assign, const int32_t* __restrict__ node_gid, int first_node, int end_node,
                   int clamp_inf, const double* __restrict__ init, double* __restrict__ out) {
  extern __shared__ __align__(16) double s_all[];
  // [kBufs][kTileDoubles] doubles, then [kBufs][2][kListInts] ints
  int32_t* const s_lists = reinterpret_cast<int32_t*>(s_all + kBufs * kTileDoubles);
  const int tid = threadIdx.x;
  const int wave0 = tid & ~63;
  const uint32_t lds_mat = (uint32_t)(uintptr_t)(lds_ptr_t)s_all;  // byte addresses inside LDS
  const uint32_t lds_lists = lds_mat + kBufs * kTileDoubles * 8;
  const int64_t lanes = (int64_t)gridDim.x * kLanes;
  const int64_t t_raw = (int64_t)blockIdx.x * kLanes + tid;
  const int64_t t = t_raw < n_assign ? t_raw : 0;  // no lane leaves early: the workgroup meets at barriers
  // assignment k of this lane; a lane past the end repeats another one and stores nothing
  auto asg = [&](int k) -> int64_t {
    const int64_t ak = t_raw + k * lanes;
    return ak < n_assign ? ak : t;
  };
  // t_trans and forbidden only ever grow by ones: counted in integers and added to the
  // carried sums at the end, exactly as the ones would have been (see below)
  double t_compute[kPer], t_comm[kPer], obj[kPer];
  uint32_t n_trans[kPer], n_forbidden[kPer], h0[kPer];
#pragma unroll
  for (int k = 0; k < kPer; ++k) {
    t_compute[k] = 0.0; t_comm[k] = 0.0; obj[k] = 0.0; n_trans[k] = 0; n_forbidden[k] = 0;
    if (init) {
      const double* r = init + asg(k) * 6;
      t_compute[k] = r[1]; t_comm[k] = r[2]; obj[k] = r[4];
    }
    // the part of mix_assignment that does not depend on the node
    const uint64_t ua = (uint64_t)(first + asg(k));
    uint32_t h = (uint32_t)seed ^ ((uint32_t)(seed >> 32) * 0x27D4EB2Fu);
    h ^= (uint32_t)ua * 0x9E3779B1u;
    h ^= (uint32_t)(ua >> 32) * 0x85EBCA77u;
    h0[k] = h;
  }
  // the choice of assignment k at node v, whose id for the draw is gid
  auto choice = [&](int k, int v, int gid, int nstrat) -> uint32_t {
    if (!kRandom) return (uint32_t)assign[(size_t)v * stride + asg(k)];
    uint32_t h = h0[k] ^ ((uint32_t)(gid + 1) * 0xC2B2AE3Du);
    h ^= h >> 16;
    h *= 0x85EBCA6Bu;
    h ^= h >> 13;
    h *= 0xC2B2AE35u;
    h ^= h >> 16;
    return (uint32_t)(((uint64_t)h * (uint64_t)(uint32_t)nstrat) >> 32);
  };
  // Whether the two index lists of a compressed matrix go through LDS too.
  auto lists_staged = [](const apc_edge& x) {
    return (x.flags & APC_EDGE_COMPRESSED) && x.sdst <= kListInts && x.ssrc <= kListInts;
  };
  // The loads of tile `base` of edge x's matrix (and, with its first tile, of its index
  // lists) into buffer b.  Nothing waits here.
  auto issue = [&](const apc_edge& x, int msize, int base, int b) {
    const int n = msize - base < kTileDoubles ? msize - base : kTileDoubles;
    const double2_t* __restrict__ src2 = reinterpret_cast<const double2_t*>(table + x.table_off + base);
#pragma unroll
    for (int r = 0; r < kTileDoubles / 2 / kLanes; ++r)
      copy16_to_lds(src2, lds_mat + (uint32_t)(b * kTileDoubles + 2 * (r * kLanes + wave0)) * 8u,
                    r * kLanes + tid, n >> 1);
    if (base == 0 && lists_staged(x)) {
#pragma unroll
      for (int r = 0; r < kListInts / kLanes; ++r) {
        copy4_to_lds(p.list_uidx + x.dst_list, lds_lists + (uint32_t)((b * 2 + 0) * kListInts + r * kLanes + wave0) * 4u,
                     r * kLanes + tid, x.sdst);
        copy4_to_lds(p.list_uidx + x.src_list, lds_lists + (uint32_t)((b * 2 + 1) * kListInts + r * kLanes + wave0) * 4u,
                     r * kLanes + tid, x.ssrc);
      }
    }
  };
  const int e_begin = first_node < end_node ? p.node_edge_off[first_node] : 0;
  const int e_end = first_node < end_node ? p.node_edge_off[end_node] : 0;
  // The record of an edge and what else the walk needs to know about it (apc_score_edge_aux)
  // are requested one edge ahead, and what it needs to know about a node one node ahead, so
  // that an edge and a node start with everything in scalar registers.
  struct NodeInfo { int nstrat, nargs, mult, gid, e_end; int64_t comp_off; };
  auto load_node = [&](int v) -> NodeInfo {
    NodeInfo n;
    n.nstrat = p.node_nstrat[v]; n.nargs = p.node_nargs[v]; n.mult = p.node_multiplier[v];
    n.gid = node_gid ? node_gid[v] : v; n.e_end = p.node_edge_off[v + 1]; n.comp_off = p.node_comp_off[v];
    return n;
  };
  NodeInfo node_nxt = {1, 1, 1, 0, 0, 0};
  if (first_node < end_node) node_nxt = load_node(first_node);
  apc_edge nxt;
  apc_score_edge_aux aux_nxt = {0, -1, 0, 0};
  if (e_begin < e_end) {
    nxt = load_edge(p.edges + e_begin);
    aux_nxt = load_aux(edge_aux + e_begin);
  }
  int buf = 0;
  {
    const int s0 = aux_nxt.next_staged;  // the first edge that goes through LDS
    if (s0 >= 0 && s0 < e_end)
      issue(s0 == e_begin ? nxt : load_edge(p.edges + s0), s0 == e_begin ? aux_nxt.msize : edge_aux[s0].msize, 0, buf);
  }
  int e = e_begin;
  for (int v = first_node; v < end_node; ++v) {
    const NodeInfo node = node_nxt;
    if (v + 1 < end_node) node_nxt = load_node(v + 1);
    const double fargs = (double)(node.nargs > 1 ? node.nargs : 1);
    const double mult = (double)node.mult;
    uint32_t o[kPer];
    double pa[kPer];
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
      o[k] = choice(k, v, node.gid, node.nstrat);
      pa[k] = per_arg[node.comp_off + o[k]];  // first needed when the node's first edge has drawn
    }
    for (; e < node.e_end; ++e) {
      const apc_edge ed = nxt;
      const apc_score_edge_aux aux = aux_nxt;
      if (e + 1 < e_end) nxt = load_edge(p.edges + e + 1);
      aux_nxt = load_aux(edge_aux + e + 1);  // the list ends with a record of its own
      const int msize = aux.msize;  // elements that go through LDS; 0: read the matrix in place
      const bool has_src = ed.src_node >= 0;
      const bool squeezed = (ed.flags & APC_EDGE_COMPRESSED) != 0;
      const uint32_t usrc = (uint32_t)ed.flags >> APC_EDGE_USRC_SHIFT;
      uint32_t j[kPer], at[kPer];
#pragma unroll
      for (int k = 0; k < kPer; ++k) j[k] = has_src ? choice(k, ed.src_node, aux.src_gid, ed.ssrc) : 0u;
      double raw[kPer];
      if (msize > 0) {  // uniform over the workgroup, as everything that decides a barrier below
        const double* const mat = s_all + buf * kTileDoubles;
        wait_vector_memory();  // this lane's part of the first tile has arrived,
        __syncthreads();       // and everyone's; and the draws of the edge before are done,
        {                      // so its buffer can take the next matrix
          const int s1 = aux_nxt.next_staged;
          if (s1 >= 0 && s1 < e_end)
            issue(s1 == e + 1 ? nxt : load_edge(p.edges + s1), s1 == e + 1 ? aux_nxt.msize : edge_aux[s1].msize, 0,
                  buf ^ 1);
        }
        if (squeezed && lists_staged(ed)) {
          const int32_t* const ud = s_lists + (buf * 2 + 0) * kListInts;
          const int32_t* const us = s_lists + (buf * 2 + 1) * kListInts;
#pragma unroll
          for (int k = 0; k < kPer; ++k) at[k] = (uint32_t)ud[o[k]] * usrc + (uint32_t)us[j[k]];
        } else if (squeezed) {
#pragma unroll
          for (int k = 0; k < kPer; ++k)
            at[k] = (uint32_t)p.list_uidx[(size_t)ed.dst_list + o[k]] * usrc +
                    (uint32_t)p.list_uidx[(size_t)ed.src_list + j[k]];
        } else {
#pragma unroll
          for (int k = 0; k < kPer; ++k) at[k] = o[k] * (uint32_t)ed.ssrc + j[k];
        }
        for (int base = 0;;) {
          const int n = msize - base < kTileDoubles ? msize - base : kTileDoubles;
#pragma unroll
          for (int k = 0; k < kPer; ++k) {
            const uint32_t local = at[k] - (uint32_t)base;
            if (local < (uint32_t)n) raw[k] = mat[local];
          }
          base += kTileDoubles;
          if (base >= msize) break;
          __syncthreads();  // the draws from this tile are done
          issue(ed, msize, base, buf);
          wait_vector_memory();
          __syncthreads();
        }
        buf ^= 1;
      } else {
        const double* __restrict__ matrix =
            ed.table_off >= 0 ? table + ed.table_off : p.default_vals + ed.default_off;
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
          if (squeezed)
            at[k] = (uint32_t)p.list_uidx[(size_t)ed.dst_list + o[k]] * usrc +
                    (uint32_t)p.list_uidx[(size_t)ed.src_list + j[k]];
          else at[k] = o[k] * (uint32_t)ed.ssrc + j[k];
        }
#pragma unroll
        for (int k = 0; k < kPer; ++k) raw[k] = matrix[at[k]];
      }
      const bool count_trans = has_src && (ed.flags & APC_EDGE_SCORE_TRANSITION);
#pragma unroll
      for (int k = 0; k < kPer; ++k) {
        // as item_store makes an entry from its matrix element
        const uint32_t trans = (uint32_t)((uint64_t)__double_as_longlong(raw[k]) >> 63);
        const double cm = fabs(raw[k]);
        double c = (cm + pa[k]) + (double)(int)trans;
        const bool finite = isfinite(c);
        if (clamp_inf && !finite) c = 10000.0;
        obj[k] += c * mult;
        n_forbidden[k] += finite ? 0u : 1u;
        if (has_src && isfinite(cm)) t_comm[k] += cm;
        n_trans[k] += count_trans ? trans : 0u;
      }
    }
    // the node's own term, added where its compute terms have long arrived (nothing else
    // is added to this sum in between, so its order is the walk's)
#pragma unroll
    for (int k = 0; k < kPer; ++k) t_compute[k] += pa[k] * fargs;
  }
  __builtin_amdgcn_s_waitcnt(0);  // nothing is in flight towards LDS when the workgroup ends
#pragma unroll
  for (int k = 0; k < kPer; ++k) {
    if (t_raw + k * lanes >= n_assign) continue;
    const double t_trans = add_ones(init ? init[asg(k) * 6 + 3] : 0.0, n_trans[k]);
    // the other scorers add 0.0 or 1.0 for every edge: what an edge without a forbidden
    // entry adds changes nothing, except the sign of a carried -0.0
    double forbidden = init ? init[asg(k) * 6 + 5] : 0.0;
    if (e_end > e_begin) forbidden += 0.0;
    forbidden = add_ones(forbidden, n_forbidden[k]);
    double* r = out + asg(k) * 6;
    r[0] = (t_compute[k] + t_comm[k]) + t_trans;
    r[1] = t_compute[k];
    r[2] = t_comm[k];
    r[3] = t_trans;
    r[4] = obj[k];
    r[5] = forbidden;
  }
}

template <bool kRandom, int kPer>
int launch_table_k(int64_t lanes, hipStream_t stream, const apc_problem& p, const double* per_arg, const double* table,
                   const apc_score_edge_aux* edge_aux, const uint16_t* assign, int64_t stride,
                   uint64_t seed, int64_t first, int64_t n_assign, const int32_t* node_gid, int first_node,
                   int end_node, int clamp_inf, const double* init, double* out) {
  // dynamic LDS beyond 64 KB needs the limit raised, per kernel and device; cheap enough to do per launch
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(score_table_kernel<kRandom, kPer>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kTableLds);
  if (e != hipSuccess) return fail(APC_ERR_LAUNCH, "hipFuncSetAttribute(score_table_kernel): %s", hipGetErrorString(e));
  const dim3 grid((unsigned)((lanes + kLanes - 1) / kLanes));
  hipLaunchKernelGGL((score_table_kernel<kRandom, kPer>), grid, dim3(kLanes), kTableLds, stream, p, per_arg,
                     table, edge_aux, assign, stride, seed, first, n_assign, node_gid, first_node,
                     end_node, clamp_inf, init, out);
  return check_launch("score_table_kernel");
}

template <bool kRandom, typename... Args>
int launch_table(int per, Args... args) {
  switch (per) {
    case 1: return launch_table_k<kRandom, 1>(args...);
    case 2: return launch_table_k<kRandom, 2>(args...);
    default: return launch_table_k<kRandom, 4>(args...);
  }
}

template <bool kRandom>
__global__ void __launch_bounds__(kBlock)
score_wave_kernel(apc_problem p, const double* __restrict__ per_arg,
                  const double* __restrict__ comm, const double* __restrict__ cost,
                  const uint8_t* __restrict__ flags, const uint16_t* __restrict__ assign,
                  int64_t stride, uint64_t seed, int64_t first, int64_t n_assign,
                  const int32_t* __restrict__ node_gid, int first_node, const double* __restrict__ init,
                  double* __restrict__ out) {
  const int64_t a = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (a >= n_assign) return;  // wave-uniform
  const int lane = threadIdx.x & 63;
  auto choice = [&](int v) -> uint32_t {
    return kRandom ? mix_assignment(seed, first + a, node_gid ? node_gid[v] : v, p.node_nstrat[v])
                   : (uint32_t)assign[(size_t)v * stride + a];
  };
  // a window of a larger graph: the nodes below first_node (stand-ins) contribute nothing,
  // and the sums continue from init
  double t_compute = 0.0, t_comm = 0.0, t_trans = 0.0, obj = 0.0, forbidden = 0.0;
  if (init) {
    const double* r = init + a * 6;
    t_compute = r[1]; t_comm = r[2]; t_trans = r[3]; obj = r[4]; forbidden = r[5];
  }
  const int e_first = first_node < p.n_node ? p.node_edge_off[first_node] : p.n_edge;
  for (int v0 = first_node; v0 < p.n_node; v0 += 64) {
    const int v = v0 + lane;
    double term = 0.0;
    if (v < p.n_node) {
      const int nargs = p.node_nargs[v];
      term = per_arg[p.node_comp_off[v] + choice(v)] * (double)(nargs > 1 ? nargs : 1);
    }
    t_compute = fold_in_order(t_compute, term);  // + 0.0 for the lanes past the end
  }
  for (int e0 = e_first; e0 < p.n_edge; e0 += 64) {
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
    // small integers: any order is exact; onto the carried sums as so many ones
    for (int off = 32; off > 0; off >>= 1) {
      tr += __shfl_xor(tr, off, 64);
      fb += __shfl_xor(fb, off, 64);
    }
    t_trans = add_ones(t_trans, (uint32_t)tr);
    forbidden = add_ones(forbidden + 0.0, (uint32_t)fb);  // a walk adds 0.0 or 1.0 per edge: a carried -0.0 loses its sign
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

// below this many assignments one wavefront per assignment is faster than one lane
constexpr int64_t kScoreWaveBelow = 32768;

template <bool kRandom>
int launch_compact(int per, dim3 grid, hipStream_t stream, const apc_problem& p, const double* per_arg,
                          const apc_score_rec16* recs, const uint16_t* assign, int64_t stride, uint64_t seed,
                          int64_t first, int64_t n_assign, const int32_t* node_gid, int first_node, int end_node,
                          const double* init, double* out) {
#define APC_COMPACT(K)                                                                                     \
  hipLaunchKernelGGL((score_compact_kernel<kRandom, K>), grid, dim3(kBlock), 0, stream, p, per_arg, recs, \
                     assign, stride, seed, first, n_assign, node_gid, first_node, end_node, init, out)
  switch (per) {
    case 1: APC_COMPACT(1); break;
    case 2: APC_COMPACT(2); break;
    case 4: APC_COMPACT(4); break;
    default: APC_COMPACT(8); break;
  }
#undef APC_COMPACT
  return check_launch("score_compact_kernel");
}

}  // namespace

extern "C" {

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
                           comm, cost, flags, asg, n_assign, seed, first + a0, n, nullptr, 0, nullptr, o);
      else
        hipLaunchKernelGGL(score_wave_kernel<false>, dim3(grid), dim3(kBlock), 0, stream, *p,
                           per_arg, comm, cost, flags, asg, n_assign, seed, first + a0, n, nullptr, 0, nullptr, o);
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
  if (n_assign < kScoreWaveBelow) {  // a wavefront per assignment
    hipLaunchKernelGGL(score_wave_kernel<true>, dim3((unsigned)((n_assign + (kBlock / 64) - 1) / (kBlock / 64))),
                       dim3(kBlock), 0, (hipStream_t)stream, *p, per_arg, comm, cost, flags, nullptr, n_assign, seed,
                       first, n_assign, node_gid, (int)first_node, init, out);
    return check_launch("score_wave_kernel");
  }
  const int64_t kChunk = 262144;  // as launch_score
  for (int64_t a0 = 0; a0 < n_assign; a0 += kChunk) {
    const int64_t n = (n_assign - a0 < kChunk) ? (n_assign - a0) : kChunk;
    hipLaunchKernelGGL(score_window_kernel<true>, dim3((unsigned)((n + kBlock - 1) / kBlock)), dim3(kBlock),
                       0, (hipStream_t)stream, *p, per_arg, comm, cost, flags, nullptr, 0, seed, first + a0, n,
                       node_gid, first_node, init ? init + a0 * 6 : nullptr, out + a0 * 6);
    if (int rc = check_launch("score_window_kernel")) return rc;
  }
  return 0;
}

int apc_score_assignments_window(const apc_problem* p, const double* per_arg, const double* comm,
                                 const double* cost, const uint8_t* flags, const uint16_t* assign,
                                 int64_t n_assign, int32_t first_node, const double* init, double* out,
                                 void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (n_assign <= 0) return 0;
  if (!per_arg || !comm || !cost || !flags || !out || !assign || !p->node_multiplier)
    return fail(APC_ERR_INVALID, "apc_score_assignments_window: null argument%s");
  if (first_node < 0 || first_node > p->n_node)
    return fail(APC_ERR_INVALID, "apc_score_assignments_window: first_node out of range%s");
  if (n_assign < kScoreWaveBelow) {  // a wavefront per assignment
    hipLaunchKernelGGL(score_wave_kernel<false>, dim3((unsigned)((n_assign + (kBlock / 64) - 1) / (kBlock / 64))),
                       dim3(kBlock), 0, (hipStream_t)stream, *p, per_arg, comm, cost, flags, assign, n_assign, 0, 0,
                       n_assign, nullptr, (int)first_node, init, out);
    return check_launch("score_wave_kernel");
  }
  const int64_t kChunk = 262144;  // as launch_score
  for (int64_t a0 = 0; a0 < n_assign; a0 += kChunk) {
    const int64_t n = (n_assign - a0 < kChunk) ? (n_assign - a0) : kChunk;
    hipLaunchKernelGGL(score_window_kernel<false>, dim3((unsigned)((n + kBlock - 1) / kBlock)), dim3(kBlock),
                       0, (hipStream_t)stream, *p, per_arg, comm, cost, flags, assign + a0, n_assign, 0, 0, n,
                       nullptr, first_node, init ? init + a0 * 6 : nullptr, out + a0 * 6);
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

int apc_pack_score_records16(const apc_problem* p, const double* per_arg, const double* comm,
                             const double* cost, const uint8_t* flags, apc_score_rec16* recs,
                             int32_t* mismatch, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (!per_arg || !comm || !cost || !flags || !recs || !mismatch)
    return fail(APC_ERR_INVALID, "apc_pack_score_records16: null argument%s");
  hipLaunchKernelGGL(clear_flag_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, mismatch);
  if (p->n_slot == 0) return check_launch("clear_flag_kernel");
  if (!p->chunk_edge) return fail(APC_ERR_INVALID, "apc_pack_score_records16: the problem has no chunk_edge%s");
  unsigned grid;
  if (int rc = slot_grid(p, kBlock, &grid)) return rc;
  hipLaunchKernelGGL(score_pack16_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *p, per_arg, comm,
                     cost, flags, recs, mismatch);
  return check_launch("score_pack16_kernel");
}

int apc_score_compact(const apc_problem* p, const double* per_arg, const apc_score_rec16* recs,
                      const uint16_t* assign, uint64_t seed, int64_t first, int64_t n_assign,
                      const int32_t* node_gid, int32_t first_node, int32_t end_node, int32_t per_lane,
                      const double* init, double* out, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (n_assign <= 0) return 0;
  if (!per_arg || !recs || !out || !p->node_multiplier)
    return fail(APC_ERR_INVALID, "apc_score_compact: null argument%s");
  if (first_node < 0 || first_node > end_node || end_node > p->n_node)
    return fail(APC_ERR_INVALID, "apc_score_compact: need 0 <= first_node <= end_node <= n_node%s");
  // Batches of up to kResident * 8 assignments per launch: kResident lanes are what the
  // 256 CUs hold at once with this kernel's registers, so that no workgroup waits for
  // another to finish and all of them walk the graph together.
  const int64_t kResident = 262144;
  for (int64_t a0 = 0; a0 < n_assign; a0 += kResident * 8) {
    const int64_t n = (n_assign - a0 < kResident * 8) ? (n_assign - a0) : kResident * 8;
    int per = per_lane;
    if (per <= 0) per = n <= kResident ? 1 : n <= 2 * kResident ? 2 : n <= 4 * kResident ? 4 : 8;
    if (per != 1 && per != 2 && per != 4 && per != 8)
      return fail(APC_ERR_INVALID, "apc_score_compact: per_lane must be 0 (choose), 1, 2, 4 or 8%s");
    const int64_t lanes = (n + per - 1) / per;
    const dim3 grid((unsigned)((lanes + kBlock - 1) / kBlock));
    const double* in = init ? init + a0 * 6 : nullptr;
    int rc = assign ? launch_compact<false>(per, grid, (hipStream_t)stream, *p, per_arg, recs, assign + a0, n_assign,
                                            seed, first + a0, n, node_gid, first_node, end_node, in, out + a0 * 6)
                    : launch_compact<true>(per, grid, (hipStream_t)stream, *p, per_arg, recs, assign, n_assign,
                                           seed, first + a0, n, node_gid, first_node, end_node, in, out + a0 * 6);
    if (rc) return rc;
  }
  return 0;
}

int apc_score_table_tile(void) { return kTileDoubles; }

int apc_score_table(const apc_problem* p, const double* per_arg, const double* table,
                    const apc_score_edge_aux* edge_aux, const uint16_t* assign,
                    uint64_t seed, int64_t first, int64_t n_assign, const int32_t* node_gid,
                    int32_t first_node, int32_t end_node, int32_t clamp_inf, int32_t per_lane,
                    const double* init, double* out, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (n_assign <= 0) return 0;
  if (!per_arg || !edge_aux || !out || !p->node_multiplier || (p->table_size > 0 && !table))
    return fail(APC_ERR_INVALID, "apc_score_table: null argument%s");
  if (first_node < 0 || first_node > end_node || end_node > p->n_node)
    return fail(APC_ERR_INVALID, "apc_score_table: need 0 <= first_node <= end_node <= n_node%s");
  if (per_lane != 0 && per_lane != 1 && per_lane != 2 && per_lane != 4)
    return fail(APC_ERR_INVALID, "apc_score_table: per_lane must be 0 (choose), 1, 2 or 4%s");
  // 262144 lanes are one workgroup of 1024 on each of the 256 CUs; four
  // assignments a lane is what the registers of that many waves allow.
  const int64_t kResident = 262144;
  for (int64_t a0 = 0; a0 < n_assign; a0 += kResident * 4) {
    const int64_t n = (n_assign - a0 < kResident * 4) ? (n_assign - a0) : kResident * 4;
    const int per = per_lane ? per_lane : n <= kResident ? 1 : n <= 2 * kResident ? 2 : 4;
    const int64_t lanes = (n + per - 1) / per;
    const double* in = init ? init + a0 * 6 : nullptr;
    int rc = assign ? launch_table<false>(per, lanes, (hipStream_t)stream, *p, per_arg, table, edge_aux,
                                          assign + a0, n_assign, seed, first + a0, n, node_gid, (int)first_node,
                                          (int)end_node, (int)clamp_inf, in, out + a0 * 6)
                    : launch_table<true>(per, lanes, (hipStream_t)stream, *p, per_arg, table, edge_aux,
                                         assign, n_assign, seed, first + a0, n, node_gid, (int)first_node,
                                         (int)end_node, (int)clamp_inf, in, out + a0 * 6);
    if (rc) return rc;
  }
  return 0;
}

uint32_t apc_random_assignment(uint64_t seed, int64_t a, int32_t node, int32_t nstrat) {
  return mix_assignment(seed, a, node, nstrat);
}
}  // extern "C"
