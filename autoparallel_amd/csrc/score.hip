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

// below this many assignments one wavefront per assignment is faster than one lane
constexpr int64_t kScoreWaveBelow = 32768;

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
}  // extern "C"
