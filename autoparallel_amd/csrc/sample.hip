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
// Two steps.  apc_pack_allowed_columns turns the flags of a build into bit
// columns: for an argument row (edge) and a choice j of its producer, one bit per
// strategy of the consumer, set where the entry is finite.  The strategies a node
// may take are then the AND of one column per argument row, a few 64-bit words,
// instead of a walk over the flag bytes of every strategy; their number is a
// population count, and the draw is the r-th set bit with r one hash of (seed,
// assignment, node) scaled to the count: a function of counters alone, which a
// host can repeat.  (When a lane walked the flag bytes and hashed once per allowed
// strategy, a reservoir walk, 2^20 assignments of the 5.5 M-entry Llama-3-8B graph
// took 136 ms on MI355X.)
#include "apc_device.h"

namespace {

constexpr int kSampleArgs = 6;   // argument rows of a node whose columns a lane keeps in registers
constexpr int kSampleWords = 8;  // words of a node's strategies a lane keeps in registers (512 strategies)
typedef uint64_t u64x2_t __attribute__((ext_vector_type(2)));

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

// Which of the count allowed strategies of a node is taken, counted in out_idx order:
// uniform in [0, count), from a hash of its own (not the plain draw's).
__host__ __device__ __forceinline__ uint32_t rank_draw(uint32_t h0, int32_t gid, uint32_t count) {
  const uint32_t h = finalise32(h0 ^ ((uint32_t)(gid + 1) * 0xC2B2AE3Du) ^ 0x68E31DA4u);
  return (uint32_t)(((uint64_t)h * (uint64_t)count) >> 32);
}

// position of the r-th set bit of m (r < popcount(m)): six halvings
__device__ __forceinline__ int select_bit(uint64_t m, uint32_t r) {
  int base = 0;
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) {
    const uint64_t low = m & ((1ull << s) - 1ull);
    const uint32_t c = (uint32_t)__popcll(low);
    if (r >= c) {
      r -= c;
      m >>= s;
      base += s;
    } else {
      m = low;
    }
  }
  return base;
}

// the strategies of word w of a node with S strategies
__device__ __forceinline__ uint64_t word_mask(int S, int w) {
  const int left = S - 64 * w;
  return left >= 64 ? ~0ull : (left <= 0 ? 0ull : ((1ull << left) - 1ull));
}

// One wavefront per (argument row e, 64 strategies of the consumer).  lane = choice j of the
// producer, so a load reads 64 consecutive flag bytes of one row of the block; a walk over the
// 64 strategies o fills, one bit a step, the word every lane keeps of its own column.
__global__ void __launch_bounds__(kBlock)
pack_allowed_columns_kernel(apc_problem p, const uint8_t* __restrict__ flags,
                            const int64_t* __restrict__ col_off, int max_words,
                            uint64_t* __restrict__ colbits) {
  const int64_t unit = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  const int e = __builtin_amdgcn_readfirstlane((int)(unit / max_words));
  const int w = __builtin_amdgcn_readfirstlane((int)(unit % max_words));
  if (e >= p.n_edge) return;
  const apc_edge* ed = p.edges + e;  // wave-uniform: scalar loads
  const int sdst = ed->sdst, ssrc = ed->ssrc;
  const int W = (sdst + 63) >> 6;
  if (w >= W) return;
  const int Wc = (W + 1) & ~1;  // words from one column to the next: whole pairs
  const int lane = threadIdx.x & 63;
  const int rows = min(64, sdst - 64 * w);
  const uint8_t* __restrict__ tile = flags + ed->off + (int64_t)(64 * w) * ssrc;
  uint64_t* __restrict__ out = colbits + col_off[e] + w;
  for (int j0 = 0; j0 < ssrc; j0 += 64) {
    const int j = j0 + lane;
    const bool mine = j < ssrc;
    const uint8_t* __restrict__ col = tile + (mine ? j : 0);
    uint64_t m = 0;
#pragma unroll 8
    for (int k = 0; k < rows; ++k)
      m |= (uint64_t)((col[(int64_t)k * ssrc] & APC_ENTRY_NONFINITE) == 0) << k;
    if (mine) out[(int64_t)j * Wc] = m;
  }
}

// One lane per assignment.  The lanes of a wave read, per argument row and word, the column
// their producer's choice names: 8-byte gathers inside one block of columns.
// kAhead: for launches of few wavefronts (see below).
template <bool kAhead>
__global__ void __launch_bounds__(kBlock)
sample_feasible_kernel(apc_problem p, const uint64_t* __restrict__ colbits,
                       const int64_t* __restrict__ col_off, uint64_t seed, int64_t first,
                       int64_t n_assign, const int32_t* __restrict__ node_gid, int first_node,
                       const uint64_t* __restrict__ row_filter, const int64_t* __restrict__ filter_off,
                       uint16_t* __restrict__ assign, int32_t* __restrict__ n_fallback) {
  const int64_t a = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (a >= n_assign) return;
  const uint32_t h0 = assignment_hash(seed, first + a);
  int fallbacks = 0;
  // What the walk needs to know about a node is the same for every lane.  With few
  // assignments a launch is a handful of wavefronts and lasts as long as its chain of
  // dependent loads; kAhead requests this part one node ahead, which takes two links out of
  // the chain (16 384 assignments of a 5 000-node window: 11.0 -> 9.8 ms).  A launch that
  // fills the chip hides the chain by itself and only pays for the registers (2^20
  // assignments of the same window: 62 -> 72 ms), so it runs without.
  struct Head {
    int S, gid, e0, e1;
    int64_t keep;  // first word of the node's filter, or -1
    int src[kSampleArgs];
    int64_t off[kSampleArgs];
  };
  auto load_head = [&](int v) -> Head {
    Head h;
    h.S = p.node_nstrat[v];
    h.gid = node_gid ? node_gid[v] : v;
    h.e0 = p.node_edge_off[v];
    h.e1 = p.node_edge_off[v + 1];
    h.keep = filter_off ? filter_off[v] : -1;
    if (kAhead) {
#pragma unroll
      for (int i = 0; i < kSampleArgs; ++i) {
        h.src[i] = -1;
        h.off[i] = 0;
        if (h.e0 + i < h.e1) {
          h.src[i] = p.edges[h.e0 + i].src_node;
          h.off[i] = col_off[h.e0 + i];
        }
      }
    }
    return h;
  };
  Head next = {};
  if (kAhead && first_node < p.n_node) next = load_head(first_node);
  for (int v = first_node; v < p.n_node; ++v) {
    const Head head = kAhead ? next : load_head(v);
    if (kAhead && v + 1 < p.n_node) next = load_head(v + 1);
    const int S = head.S, gid = head.gid, e0 = head.e0, e1 = head.e1;
    const int W = (S + 63) >> 6;
    const int Wc = (W + 1) & ~1;  // words from one column to the next: whole pairs, 16-byte aligned
    // the column of every argument row: that of the producer's choice
    const u64x2_t* col[kSampleArgs];
#pragma unroll
    for (int i = 0; i < kSampleArgs; ++i) {
      col[i] = reinterpret_cast<const u64x2_t*>(colbits);
      if (e0 + i < e1) {
        const int u = kAhead ? head.src[i] : p.edges[e0 + i].src_node;
        const int64_t j = u >= 0 ? (int64_t)assign[(size_t)u * n_assign + a] : 0;
        col[i] = reinterpret_cast<const u64x2_t*>(colbits + (kAhead ? head.off[i] : col_off[e0 + i]) + j * Wc);
      }
    }
    // words 2 q and 2 q + 1 of the node's allowed strategies: a lane reads its columns 16 bytes at
    // a time (the lanes of a wave read different columns, and such a load costs the same for 8
    // bytes as for 16)
    auto allowed_pair = [&](int q) -> u64x2_t {
      u64x2_t m = {word_mask(S, 2 * q), word_mask(S, 2 * q + 1)};
      if (head.keep >= 0) {  // the strategies the node may take at all
        m.x &= row_filter[head.keep + 2 * q];
        if (2 * q + 1 < W) m.y &= row_filter[head.keep + 2 * q + 1];
      }
#pragma unroll
      for (int i = 0; i < kSampleArgs; ++i)
        if (e0 + i < e1) m &= col[i][q];
      for (int e = e0 + kSampleArgs; e < e1; ++e) {  // a node with more argument rows than the registers hold
        const int u = p.edges[e].src_node;
        const int64_t j = u >= 0 ? (int64_t)assign[(size_t)u * n_assign + a] : 0;
        m &= reinterpret_cast<const u64x2_t*>(colbits + col_off[e] + j * Wc)[q];
      }
      return m;
    };
    uint32_t count = 0;
    int pick = 0;
    if (W == 1) {  // up to 64 strategies (most nodes of a traced model): one word, read by itself
      uint64_t m = word_mask(S, 0);
      if (head.keep >= 0) m &= row_filter[head.keep];
#pragma unroll
      for (int i = 0; i < kSampleArgs; ++i)
        if (e0 + i < e1) m &= reinterpret_cast<const uint64_t*>(col[i])[0];
      for (int e = e0 + kSampleArgs; e < e1; ++e) {
        const int u = p.edges[e].src_node;
        const int64_t j = u >= 0 ? (int64_t)assign[(size_t)u * n_assign + a] : 0;
        m &= colbits[col_off[e] + j * Wc];
      }
      count = (uint32_t)__popcll(m);
      if (count > 0) pick = select_bit(m, rank_draw(h0, gid, count));
    } else if (W <= kSampleWords) {  // wave-uniform: the words stay in registers
      uint64_t m[kSampleWords];
#pragma unroll
      for (int q = 0; q < kSampleWords / 2; ++q) {
        const u64x2_t mm = 2 * q < W ? allowed_pair(q) : u64x2_t{0ull, 0ull};
        m[2 * q] = mm.x;
        m[2 * q + 1] = mm.y;
        count += (uint32_t)__popcll(mm.x) + (uint32_t)__popcll(mm.y);
      }
      if (count > 0) {
        uint32_t r = rank_draw(h0, gid, count);
        bool found = false;
#pragma unroll
        for (int w = 0; w < kSampleWords; ++w) {
          const uint32_t c = (uint32_t)__popcll(m[w]);
          if (!found && r < c) {
            pick = 64 * w + select_bit(m[w], r);
            found = true;
          }
          if (!found) r -= c;
        }
      }
    } else {  // more than 512 strategies: the words are formed twice
      for (int q = 0; 2 * q < W; ++q) {
        const u64x2_t mm = allowed_pair(q);
        count += (uint32_t)__popcll(mm.x) + (uint32_t)__popcll(mm.y);
      }
      if (count > 0) {
        uint32_t r = rank_draw(h0, gid, count);
        for (int q = 0; 2 * q < W; ++q) {
          const u64x2_t mm = allowed_pair(q);
          const uint32_t cx = (uint32_t)__popcll(mm.x), cy = (uint32_t)__popcll(mm.y);
          if (r < cx) {
            pick = 128 * q + select_bit(mm.x, r);
            break;
          }
          r -= cx;
          if (r < cy) {
            pick = 128 * q + 64 + select_bit(mm.y, r);
            break;
          }
          r -= cy;
        }
      }
    }
    if (count == 0) {
      pick = (int)plain_draw(h0, gid, S);
      ++fallbacks;
    }
    assign[(size_t)v * n_assign + a] = (uint16_t)pick;
  }
  n_fallback[a] = fallbacks;
}

}  // namespace

extern "C" {

int apc_pack_allowed_columns(const apc_problem* p, const uint8_t* flags, const int64_t* col_off,
                             int32_t max_words, uint64_t* colbits, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_edge == 0 || p->n_entry == 0) return 0;
  if (!flags || !col_off || !colbits || max_words <= 0)
    return fail(APC_ERR_INVALID, "apc_pack_allowed_columns: null argument or max_words <= 0%s");
  const int64_t units = (int64_t)p->n_edge * max_words;
  const int64_t grid = (units + (kBlock / 64) - 1) / (kBlock / 64);
  if (grid > 0x7FFFFFFF)
    return fail(APC_ERR_INVALID, "apc_pack_allowed_columns: too many argument rows for one launch%s");
  hipLaunchKernelGGL(pack_allowed_columns_kernel, dim3((unsigned)grid), dim3(kBlock), 0, (hipStream_t)stream, *p,
                     flags, col_off, (int)max_words, colbits);
  return check_launch("pack_allowed_columns_kernel");
}

int apc_sample_feasible(const apc_problem* p, const uint64_t* colbits, const int64_t* col_off, uint64_t seed,
                        int64_t first, int64_t n_assign, const int32_t* node_gid, int32_t first_node,
                        const uint64_t* row_filter, const int64_t* filter_off, uint16_t* assign,
                        int32_t* n_fallback, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (n_assign <= 0) return 0;
  if (!assign || !n_fallback || (p->n_entry > 0 && (!colbits || !col_off)))
    return fail(APC_ERR_INVALID, "apc_sample_feasible: null argument%s");
  if (first_node < 0 || first_node > p->n_node)
    return fail(APC_ERR_INVALID, "apc_sample_feasible: first_node out of range%s");
  if ((row_filter == nullptr) != (filter_off == nullptr))
    return fail(APC_ERR_INVALID, "apc_sample_feasible: row_filter and filter_off come together%s");
  const dim3 grid((unsigned)((n_assign + kBlock - 1) / kBlock));
  if (n_assign < 65536)  // fewer wavefronts than SIMDs
    hipLaunchKernelGGL(sample_feasible_kernel<true>, grid, dim3(kBlock), 0, (hipStream_t)stream, *p, colbits, col_off,
                       seed, first, n_assign, node_gid, (int)first_node, row_filter, filter_off, assign, n_fallback);
  else
    hipLaunchKernelGGL(sample_feasible_kernel<false>, grid, dim3(kBlock), 0, (hipStream_t)stream, *p, colbits, col_off,
                       seed, first, n_assign, node_gid, (int)first_node, row_filter, filter_off, assign, n_fallback);
  return check_launch("sample_feasible_kernel");
}

uint32_t apc_sample_rank(uint64_t seed, int64_t a, int32_t node, uint32_t count) {
  return count ? rank_draw(assignment_hash(seed, a), node, count) : 0u;
}

}  // extern "C"
