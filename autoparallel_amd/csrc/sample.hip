// Candidate assignments without a forbidden entry, drawn on the device (gfx950),
// and the C ABI of the sampler.
//
// The ILP forbids every decision variable whose cost is not finite
// (add_inf_cost_constraint, autoparallel/optimize_sharding.py:803-812).  An
// assignment made of independent uniform draws per node nearly always selects
// one, so it scores an objective no feasible plan has.  This sampler walks the
// nodes in graph order and gives node v, uniformly, one of the strategies whose
// entries against the choices already made for its producers are all finite;
// a node that has none takes the plain draw and is counted.  Consistency of the
// flow rows holds by construction, as for the plain draws: an edge's inp_idx is
// its producer's choice.
//
// Large batches: one lane per assignment.  Lanes of a wave read the flags of the same edge
// block and the same row, at the columns their producers' choices name: one or
// two cache lines per load, out of L2.  The choice among the allowed strategies
// is a reservoir walk (the k-th allowed one replaces the pick when a hash of
// (seed, assignment, node, k) scaled to [0, k) is zero), so the flags are read
// once and the draw is a function of counters alone: a host can repeat it.
#include "apc_device.h"

namespace {

constexpr int kSampleArgs = 6;  // argument rows of a node whose bases a lane keeps in registers

__host__ __device__ __forceinline__ uint32_t finalise32(uint32_t h) {
  h ^= h >> 16;
  h *= 0x85EBCA6Bu;
  h ^= h >> 13;
  h *= 0xC2B2AE35u;
  h ^= h >> 16;
  return h;
}

// the part of every draw of assignment a that does not depend on the node
__host__ __device__ __forceinline__ uint32_t assignment_hash(uint64_t seed, int64_t a) {
  uint32_t h = (uint32_t)seed ^ ((uint32_t)(seed >> 32) * 0x27D4EB2Fu);
  h ^= (uint32_t)(uint64_t)a * 0x9E3779B1u;
  h ^= (uint32_t)((uint64_t)a >> 32) * 0x85EBCA77u;
  return h;
}

// The plain draw of the scorers (apc_random_assignment): uniform in [0, nstrat).
__host__ __device__ __forceinline__ uint32_t plain_draw(uint32_t h0, int32_t gid, int32_t nstrat) {
  const uint32_t h = finalise32(h0 ^ ((uint32_t)(gid + 1) * 0xC2B2AE3Du));
  return (uint32_t)(((uint64_t)h * (uint64_t)(uint32_t)nstrat) >> 32);
}

// Whether the k-th allowed strategy (k >= 1) replaces the pick: probability 1 / k.
__host__ __device__ __forceinline__ bool reservoir_takes(uint32_t h0, int32_t gid, uint32_t k) {
  const uint32_t h = finalise32(h0 ^ ((uint32_t)(gid + 1) * 0xC2B2AE3Du) ^ (k * 0x9E3779B1u) ^ 0x68E31DA4u);
  return (uint32_t)(((uint64_t)h * (uint64_t)k) >> 32) == 0u;
}

__global__ void __launch_bounds__(kBlock)
sample_feasible_kernel(apc_problem p, const uint8_t* __restrict__ flags, uint64_t seed, int64_t first,
                       int64_t n_assign, const int32_t* __restrict__ node_gid, int first_node,
                       uint16_t* __restrict__ assign, int32_t* __restrict__ n_fallback) {
  const int64_t a = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (a >= n_assign) return;
  const uint32_t h0 = assignment_hash(seed, first + a);
  int fallbacks = 0;
  for (int v = first_node; v < p.n_node; ++v) {
    const int S = p.node_nstrat[v];
    const int gid = node_gid ? node_gid[v] : v;
    const int e0 = p.node_edge_off[v], e1 = p.node_edge_off[v + 1];
    // slot of (row 0, the producer's choice) in every argument's block, and the row length
    int64_t base[kSampleArgs];
    int32_t ssrc[kSampleArgs];
#pragma unroll
    for (int i = 0; i < kSampleArgs; ++i) {
      base[i] = 0;
      ssrc[i] = 0;
      if (e0 + i < e1) {
        const apc_edge* ed = p.edges + (e0 + i);
        const int u = ed->src_node;
        const uint32_t j = u >= 0 ? (uint32_t)assign[(size_t)u * n_assign + a] : 0u;
        base[i] = ed->off + j;
        ssrc[i] = ed->ssrc;
      }
    }
    uint32_t count = 0, pick = 0;
    for (int o = 0; o < S; ++o) {
      uint32_t bad = 0;
#pragma unroll
      for (int i = 0; i < kSampleArgs; ++i)
        if (e0 + i < e1) bad |= flags[base[i] + (int64_t)o * ssrc[i]];
      for (int e = e0 + kSampleArgs; e < e1; ++e) {  // a node with more argument rows than the registers hold
        const apc_edge* ed = p.edges + e;
        const int u = ed->src_node;
        const uint32_t j = u >= 0 ? (uint32_t)assign[(size_t)u * n_assign + a] : 0u;
        bad |= flags[ed->off + (int64_t)o * ed->ssrc + j];
      }
      if (!(bad & APC_ENTRY_NONFINITE)) {
        ++count;
        if (reservoir_takes(h0, gid, count)) pick = (uint32_t)o;
      }
    }
    if (count == 0) {
      pick = plain_draw(h0, gid, S);
      ++fallbacks;
    }
    assign[(size_t)v * n_assign + a] = (uint16_t)pick;
  }
  n_fallback[a] = fallbacks;
}

// Small batches: one wavefront per assignment, lanes over the strategies of the
// node.  A lane finds out whether its strategy is allowed, the ballot of the wave
// gives every allowed strategy its rank k in out_idx order, each lane evaluates the
// reservoir's test for its own k, and the pick is the last strategy whose test
// says "take": what the sequential walk ends with.  Same choices as the kernel
// above, bit for bit; the lanes of a wave read one column of a block (a cache line
// each) instead of sharing a row, which is the better trade while there are
// fewer assignments than lanes on the chip.
__global__ void __launch_bounds__(kBlock)
sample_feasible_wave_kernel(apc_problem p, const uint8_t* __restrict__ flags, uint64_t seed, int64_t first,
                            int64_t n_assign, const int32_t* __restrict__ node_gid, int first_node,
                            uint16_t* __restrict__ assign, int32_t* __restrict__ n_fallback) {
  const int64_t a = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (a >= n_assign) return;  // wave-uniform
  const int lane = threadIdx.x & 63;
  const uint32_t h0 = assignment_hash(seed, first + a);
  int fallbacks = 0;
  for (int v = first_node; v < p.n_node; ++v) {
    const int S = p.node_nstrat[v];
    const int gid = node_gid ? node_gid[v] : v;
    const int e0 = p.node_edge_off[v], e1 = p.node_edge_off[v + 1];
    uint32_t count = 0;
    int pick = -1;
    // The producers' choices (written by this wave's lane 0, or by the caller): lane i reads
    // that of argument row i, and the wave takes them from there.  One load whose 64 lanes
    // all read the same address costs as much as a 64-way gather on this chip.
    int j_of = 0;
    if (e0 + lane < e1) {
      const int u = p.edges[e0 + lane].src_node;
      j_of = u >= 0 ? (int)assign[(size_t)u * n_assign + a] : 0;
    }
    for (int o0 = 0; o0 < S; o0 += 64) {
      const int o = o0 + lane;
      uint32_t bad = o < S ? 0u : (uint32_t)APC_ENTRY_NONFINITE;
      for (int e = e0; e < e1; ++e) {
        const apc_edge* ed = p.edges + e;  // wave-uniform: scalar loads
        uint32_t j;
        if (e - e0 < 64) {
          j = (uint32_t)__builtin_amdgcn_readlane(j_of, e - e0);
        } else {  // more argument rows than lanes
          const int u = ed->src_node;
          j = u >= 0 ? (uint32_t)assign[(size_t)u * n_assign + a] : 0u;
        }
        if (o < S) bad |= flags[ed->off + (int64_t)o * ed->ssrc + j];
      }
      const bool allowed = !(bad & APC_ENTRY_NONFINITE);
      const uint64_t mask = __ballot(allowed);
      const uint32_t rank = count + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull)) + 1u;
      const uint64_t takes = __ballot(allowed && reservoir_takes(h0, gid, rank));
      if (takes) pick = o0 + 63 - __clzll(takes);
      count += (uint32_t)__popcll(mask);
    }
    if (count == 0) {
      pick = (int)plain_draw(h0, gid, S);
      ++fallbacks;
    }
    if (lane == 0) assign[(size_t)v * n_assign + a] = (uint16_t)pick;
    // the next node may read this choice through the vector memory path of other lanes
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  if (lane == 0) n_fallback[a] = fallbacks;
}

constexpr int64_t kSampleWaveBelow = 65536;  // assignments: below, a wavefront each

}  // namespace

extern "C" {

int apc_sample_feasible(const apc_problem* p, const uint8_t* flags, uint64_t seed, int64_t first,
                        int64_t n_assign, const int32_t* node_gid, int32_t first_node, uint16_t* assign,
                        int32_t* n_fallback, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (n_assign <= 0) return 0;
  if (!assign || !n_fallback || (p->n_entry > 0 && !flags))
    return fail(APC_ERR_INVALID, "apc_sample_feasible: null argument%s");
  if (first_node < 0 || first_node > p->n_node)
    return fail(APC_ERR_INVALID, "apc_sample_feasible: first_node out of range%s");
  if (n_assign < kSampleWaveBelow) {
    const int64_t per = kBlock / 64;
    hipLaunchKernelGGL(sample_feasible_wave_kernel, dim3((unsigned)((n_assign + per - 1) / per)), dim3(kBlock), 0,
                       (hipStream_t)stream, *p, flags, seed, first, n_assign, node_gid, (int)first_node, assign,
                       n_fallback);
    return check_launch("sample_feasible_wave_kernel");
  }
  hipLaunchKernelGGL(sample_feasible_kernel, dim3((unsigned)((n_assign + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                     (hipStream_t)stream, *p, flags, seed, first, n_assign, node_gid, (int)first_node, assign,
                     n_fallback);
  return check_launch("sample_feasible_kernel");
}

int32_t apc_sample_takes(uint64_t seed, int64_t a, int32_t node, uint32_t k) {
  return reservoir_takes(assignment_hash(seed, a), node, k) ? 1 : 0;
}

}  // extern "C"
