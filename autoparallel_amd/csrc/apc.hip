// The coefficient build of the sharding-search cost engine (gfx950 / CDNA4):
// block table, node compute estimate and the entry kernel, their C ABI, and the
// host helpers the other translation units share (score.hip: batch scoring;
// passes.hip: passes over the results and batch forms of the scalar functions;
// schedule.hip: the lowered-graph estimator; nccl_plan.cpp: the NCCL model's
// host half).
//
// Everything here is HBM-bound integer/fp64 scalar work: no matrix cores.  The
// entry kernel is a flat scan over the E cost entries in work items of 256 (or
// 512) entries of one edge block: a wavefront owns an item, lane L the entries
// L + 64 k, so every load and store instruction covers 64 consecutive entries.
#include "apc_device.h"

#include <mutex>

namespace apc_impl {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, const char* detail) {
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
  if (p->n_prog_term < 0 || (p->n_prog_term > 0 && !p->prog_terms))
    return fail(APC_ERR_INVALID, "n_prog_term without prog_terms%s");
  if (p->n_lut_table_tile < 0 || p->n_lut_table_tile > 0x7FFFFFFF || p->n_lut_entry_tile < 0 ||
      p->n_lut_entry_tile > 0x7FFFFFFF || (p->n_lut_table_tile > 0 && !p->lut_table_tiles) ||
      (p->n_lut_entry_tile > 0 && !p->lut_entry_tiles))
    return fail(APC_ERR_INVALID, "bad lookup-table tile lists%s");
  if ((p->n_lut_table_tile > 0 || p->n_lut_entry_tile > 0) && !p->spec_recs)
    return fail(APC_ERR_INVALID, "lookup-table tiles need apc_problem.spec_recs%s");
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
}  // namespace apc_impl

namespace {

using apc_impl::g_err;

// What the library remembers per device (a kernel attribute that is set once,
// the address of the static scratch array): looked up by the current device of
// the calling thread, guarded by a mutex of its own.
struct DeviceState {
  std::mutex mu;
  bool lds_limit_raised = false;
  double* scratch = nullptr;  // device address of `scratch` on this device
};
constexpr int kMaxDevices = 64;
DeviceState g_devices[kMaxDevices];

DeviceState* current_device_state() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    snprintf(g_err, sizeof(g_err), "hipGetDevice: %s (device %d)", hipGetErrorString(e), dev);
    return nullptr;
  }
  return &g_devices[dev];
}

// Scratch of apc_build_all_noalloc: the block table of one build.  Every GPU
// the library runs on holds its own copy (8 MiB) until the process ends.  The
// name is a host-side stand-in, not a device address: host code uses the
// address hipGetSymbolAddress returns for the current device (resolve_scratch).
__device__ __align__(256) static double scratch[APC_NOALLOC_MAX_TABLE];

// Device address of `scratch` on the calling thread's current device, resolved
// on the first call there.
double* resolve_scratch() {
  DeviceState* dev = current_device_state();
  if (!dev) return nullptr;
  std::lock_guard<std::mutex> lock(dev->mu);
  if (!dev->scratch) {
    void* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      snprintf(g_err, sizeof(g_err), "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
      return nullptr;
    }
    dev->scratch = static_cast<double*>(ptr);
  }
  return dev->scratch;
}

// ---------------------------------------------------------------------------
// Kernel: block table and node compute estimate
// ---------------------------------------------------------------------------
constexpr int kFusedTableBlocks = 2048;  // larger tables are built by a launch of their own
constexpr int kProgCache = 128;    // int64 words of program (or 64 product terms) staged per node block
constexpr int kRecWords = 8;       // int64 words of LDS for the record's argument runs
constexpr int kHintWords = 4;      // and for its 16 meta hints
constexpr int kPartWords = 4 * 3 * 64;  // per wavefront and lane: partial flops, bytes, first argument with a spec
constexpr int kNodeHeader = kProgCache + kRecWords + kHintWords + kPartWords;  // words before the value table
static_assert(kRecWords * 2 >= APC_REC_ARGS && sizeof(apc_comp_rec) == 160, "record layout");
static_assert(sizeof(apc_prog_term) == 16 && 2 * APC_TERMS_MAX <= kProgCache, "term layout");
static_assert(sizeof(apc_spec_rec) == 16 && sizeof(apc_table_unit) == 32, "record layout");

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
  r.term_off = 0; r.n_term = 0; r.term_flags = 0;
#pragma unroll
  for (int a = 0; a < 16; ++a) r.arg_meta[a] = 0xFFFF;
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
  const int slots = max_rank + 2;  // per argument: max_rank sizes, an info word, its local element count
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
        // element count of the local tensor, formed here where the sizes are in
        // registers: phase 2 reads one word per argument
        s_local[(a * slots + max_rank + 1) * 64 + oo] = numel;
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
        nbytes += s_local[(a * slots + max_rank + 1) * 64 + lane] * (int64_t)((info >> 8) & 0xFFFFFFFF);
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
          } else if (kind == 3) {  // all local sizes of an argument
            const int a = (int)pr[1];
            if (staged) {
              size = s_local[(a * slots + max_rank + 1) * 64 + lane];
            } else {
              size = 1;
              const int r = rank_of(a);
              for (int d = 0; d < r; ++d) size *= size_of(a, d);
            }
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

// One workgroup (four wavefronts) per 64 strategies of an evaluated node whose
// program has the product-term form.  Phase 1: the 256 lanes split the node's
// (strategy, argument) pairs and write each argument's local sizes, an info
// word and its local element count into the value table in LDS (row layout:
// apc_prog_term in include/apc.h).  Phase 1b, only for programs that read a
// broadcast size: one lane per (position, strategy).  Phase 2: lane = strategy,
// the wavefronts share the terms (term t goes to wavefront t mod 4); each term
// is one 16-byte LDS read, then independent reads of its factors.  Integer
// sums do not depend on their order, so the partial sums per wavefront add up
// to the interpreter's flops and bytes exactly.  Wavefront 0 folds them and
// writes the estimate.  Nodes without that form (or when the table does not fit
// in LDS) are interpreted by wavefront 0 alone.
__device__ __forceinline__ void node_compute_block(const apc_problem& p, const apc_comp_rec& rec,
                                                   int o0, int tid, int64_t* __restrict__ s_dyn,
                                                   bool slow, double* __restrict__ compute,
                                                   double* __restrict__ per_arg,
                                                   int32_t* __restrict__ status) {
  const int S = rec.nstrat;
  if (o0 >= S) return;  // uniform over the workgroup
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  int64_t* s_prog = s_dyn;
  uint32_t* s_dst = reinterpret_cast<uint32_t*>(s_dyn + kProgCache);
  uint16_t* s_hint = reinterpret_cast<uint16_t*>(s_dyn + kProgCache + kRecWords);
  int64_t* s_part = s_dyn + kProgCache + kRecWords + kHintWords;
  int64_t* s_val = s_dyn + kNodeHeader;
  const bool fast = !slow && rec.op == APC_OP_PROGRAM && rec.n_term > 0 && p.prog_terms != nullptr;
  if (!fast) {
    if (wave == 0)
      node_compute_wave(p, rec, o0, lane, s_prog, s_dst, s_val, slow, compute, per_arg, status);
    return;
  }
  const int na = rec.n_edge;  // at most APC_REC_ARGS on this path
  const int R = p.max_rank, slots = R + 2;
  const int chunk = (S - o0 < 64) ? (S - o0) : 64;
  const int n_words = 2 * rec.n_term;
  int64_t term_word = 0;
  if (tid < n_words) term_word = reinterpret_cast<const int64_t*>(p.prog_terms + rec.term_off)[tid];
  if (tid == 0) {  // constant indices: the record stays in scalar registers
#pragma unroll
    for (int a = 0; a < APC_REC_ARGS; ++a) {
      s_dst[a] = rec.dst_list[a];
      s_hint[a] = rec.arg_meta[a];
    }
  }
  __syncthreads();
  for (int t = tid; t < chunk * na; t += 256) {
    const int a = t / chunk, oo = t - a * chunk;
    const size_t pos = (size_t)s_dst[a] + o0 + oo;
    // The rows of the hinted meta are fetched together with the spec word, not
    // after it; a word that names another meta fetches its own.
    uint32_t mid = s_hint[a];
    const bool hinted = mid != 0xFFFFu;
    if (!hinted) mid = 0;
    uint32_t w, plc = 0;
    if (p.spec_recs) {
      const apc_spec_rec sr = p.spec_recs[pos];
      w = sr.word;
      plc = sr.plc;
    } else {
      w = p.lists[pos];
    }
    int rank = p.meta_rank[mid];
    int64_t isz = p.meta_itemsize[mid];
    int64_t dt = p.meta_dtype[mid];
    const ll2_t* r = reinterpret_cast<const ll2_t*>(p.meta_shape + (size_t)mid * APC_MAX_RANK);
    ll2_t row[APC_MAX_RANK / 2];
#pragma unroll
    for (int q = 0; q < APC_MAX_RANK / 2; ++q) row[q] = r[q];
    const bool none = (w == APC_SPEC_NONE);
    if (!none && (!hinted || (w >> APC_TUPLE_BITS) != mid)) {
      mid = w >> APC_TUPLE_BITS;
      rank = p.meta_rank[mid];
      isz = p.meta_itemsize[mid];
      dt = p.meta_dtype[mid];
      r = reinterpret_cast<const ll2_t*>(p.meta_shape + (size_t)mid * APC_MAX_RANK);
#pragma unroll
      for (int q = 0; q < APC_MAX_RANK / 2; ++q) row[q] = r[q];
    }
    if (!p.spec_recs) plc = load_tuple(p.tuple_plc, none ? 0u : (w & kTupleMask));
    if (none) rank = 0;
    int64_t numel = 1;
    int64_t* col = s_val + (size_t)(R + a * slots) * 64 + oo;
#pragma unroll
    for (int d = 0; d < APC_MAX_RANK; ++d) {
      if (d >= R) break;  // uniform
      int64_t sz = (d & 1) ? row[d >> 1].y : row[d >> 1].x;
      if (d >= rank) {
        sz = 1;
      } else {
        for (int i = 0; i < p.model.ndim; ++i) {
          const int c = (plc >> (8 * i)) & 0xFF;
          if ((c & kKindMask) == kShard && (c & kArgMask) == d) sz = ceil_div_pos(sz, p.model.mesh_shape[i]);
        }
      }
      col[d * 64] = sz;
      numel *= sz;  // sizes past the rank are 1
    }
    // info word: rank | itemsize << 8 | dtype << 40, or -1 for a missing spec
    col[R * 64] = none ? -1 : ((int64_t)rank | (isz << 8) | (dt << 40));
    col[(R + 1) * 64] = numel;
  }
  if (tid < n_words) s_prog[tid] = term_word;
  __syncthreads();
  if (rec.term_flags & APC_TERMS_BCAST) {
    // broadcast of all arguments at a right-aligned position: the size of the last
    // argument that reaches the position with a size other than 1
    for (int t = tid; t < chunk * R; t += 256) {
      const int pos = t / chunk, oo = t - pos * chunk;
      int64_t size = 1;
      for (int a = 0; a < na; ++a) {
        const int64_t* col = s_val + (size_t)(R + a * slots) * 64 + oo;
        const int64_t info = col[R * 64];
        const int r = info < 0 ? -1 : (int)(info & 0xFF);
        if (pos >= r) continue;
        const int64_t sz = col[(r - 1 - pos) * 64];
        if (sz != 1) size = sz;
      }
      s_val[pos * 64 + oo] = size;
    }
    __syncthreads();
  }
  // Phase 2.  Wavefront w takes the terms and the arguments congruent to w mod 4;
  // `first` is its lowest argument that has a spec (the node's dtype is that of
  // the lowest over all wavefronts) or 255.
  int64_t flops = 0, nbytes = 0;
  int first = 255, dtype = 1;  // float32 when the node has no tensor argument
  if (lane < chunk) {
    for (int t = wave; t < rec.n_term; t += 4) {
      const ll2_t tw = *reinterpret_cast<const ll2_t*>(s_prog + 2 * t);
      int64_t term = tw.x;
      // the term is the same for every lane: its factor list goes to scalar registers
      const uint32_t ilo = __builtin_amdgcn_readfirstlane((uint32_t)tw.y);
      const uint32_t ihi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)tw.y >> 32));
      int64_t v[7];
#pragma unroll
      for (int f = 0; f < 7; ++f) {
        const uint32_t i = ((f < 4 ? ilo >> (8 * f) : ihi >> (8 * (f - 4))) & 0xFF);
        v[f] = (i != 0xFF) ? s_val[i * 64 + lane] : 1;
      }
#pragma unroll
      for (int f = 0; f < 7; ++f) term *= v[f];
      if (ihi >> 24) nbytes += term; else flops += term;
    }
    for (int a = wave; a < na; a += 4) {
      const int64_t* col = s_val + (size_t)(R + a * slots) * 64 + lane;
      const int64_t info = col[R * 64];
      const int64_t numel = col[(R + 1) * 64];
      if (info < 0) continue;
      if (first == 255) { first = a; dtype = (int)(info >> 40); }
      nbytes += numel * (int64_t)((info >> 8) & 0xFFFFFFFF);
    }
  }
  if (wave != 0) {
    s_part[(wave * 3 + 0) * 64 + lane] = flops;
    s_part[(wave * 3 + 1) * 64 + lane] = nbytes;
    s_part[(wave * 3 + 2) * 64 + lane] = (int64_t)first | ((int64_t)dtype << 8);
  }
  __syncthreads();
  if (wave == 0 && lane < chunk) {
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      flops += s_part[(w * 3 + 0) * 64 + lane];
      nbytes += s_part[(w * 3 + 1) * 64 + lane];
      const int64_t fd = s_part[(w * 3 + 2) * 64 + lane];
      if ((int)(fd & 0xFF) < first) { first = (int)(fd & 0xFF); dtype = (int)(fd >> 8); }
    }
    const int64_t idx = rec.comp_off + o0 + lane;
    const double result = roofline(p, flops, nbytes, dtype, status);
    compute[idx] = result;
    per_arg[idx] = result / (double)rec.nargs;
  }
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
__device__ __forceinline__ void pair_table_block(const apc_problem& p, double* __restrict__ table,
                                                 int unit) {
  const int tid = threadIdx.x;
  apc_table_unit u;
  if (p.table_units) {
    u = p.table_units[unit];
  } else {  // the same fields through the block and edge arrays
    const int b = p.table_unit_block[unit];
    const apc_edge ed = p.edges[p.block_edge[b]];  // any edge with this matrix
    const bool squeezed = (ed.flags & APC_EDGE_COMPRESSED) != 0;
    u.default_off = ed.default_off;
    u.src_list = ed.src_list;
    u.dst_list = ed.dst_list;
    u.ncol = squeezed ? (uint32_t)ed.flags >> APC_EDGE_USRC_SHIFT : (uint32_t)ed.ssrc;
    u.nrow = squeezed ? (uint32_t)p.block_udst[b] : (uint32_t)ed.sdst;
    u.first = (uint32_t)((int64_t)unit * 256 - p.block_off[b]);
    u.flags = squeezed ? APC_EDGE_COMPRESSED : 0;
  }
  const uint32_t l = u.first + (uint32_t)tid;
  if (l >= u.ncol * u.nrow) return;  // a matrix has fewer than 2^31 elements
  uint32_t o = l / u.ncol, j = l - o * u.ncol;
  if (u.flags & APC_EDGE_COMPRESSED) {  // position in its run of an occurrence of that word
    o = (uint32_t)p.list_ufirst[(size_t)u.dst_list + o];
    j = (uint32_t)p.list_ufirst[(size_t)u.src_list + j];
  }
  // the two specs: a record per side when the caller made them, else the word,
  // then its tuple row and its tensor's shape and stride rows
  uint32_t sw, tw, src_plc, tgt_plc;
  int64_t nbytes;
  bool contig;
  if (p.spec_recs) {
    const apc_spec_rec rs = p.spec_recs[(size_t)u.src_list + j];
    const apc_spec_rec rt = p.spec_recs[(size_t)u.dst_list + o];
    sw = rs.word; tw = rt.word;
    src_plc = rs.plc; tgt_plc = rt.plc;
    nbytes = rs.nbytes2 >> 1;
    contig = (rs.nbytes2 & 1) != 0;
  } else {
    sw = p.lists[(size_t)u.src_list + j];
    tw = p.lists[(size_t)u.dst_list + o];
    if (sw != APC_SPEC_NONE && tw != APC_SPEC_NONE) {
      src_plc = load_tuple(p.tuple_plc, sw & kTupleMask);
      tgt_plc = load_tuple(p.tuple_plc, tw & kTupleMask);
      meta_bytes_contig(p, sw >> APC_TUPLE_BITS, nbytes, contig);
    }
  }
  double* out = table + (int64_t)unit * 256 + tid;
  if (sw != APC_SPEC_NONE && tw != APC_SPEC_NONE) {
    const double c = redistribute_cost(src_plc, tgt_plc, nbytes, contig, p.model);
    *out = ((sw & kTupleMask) != (tw & kTupleMask)) ? -c : c;
  } else {  // a missing spec keeps the default row's value and is no transition
    *out = p.default_vals[u.default_off + (int64_t)l];  // never a compressed matrix
  }
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
    pair_table_block(p, table, blockIdx.x);
    return;
  }
  const int unit = (int)blockIdx.x - table_blocks;
  const int chunks = (p.max_nstrat + 63) >> 6;  // workgroups per node
  const int i = unit / chunks;
  if (i >= p.n_comp_node) return;
  const apc_comp_rec rec = load_comp_rec(p, i);
  node_compute_block(p, rec, (unit - i * chunks) * 64, threadIdx.x, s_dyn, slow != 0, compute, per_arg,
                     status);
}

// The block table alone, for tables of many units: no dynamic LDS (which in
// prepare_kernel limits the blocks per CU to what the node wavefronts need) and
// no cache warming (thousands of blocks keep the descriptor arrays in L2 by
// themselves).
__global__ void __launch_bounds__(256)
pair_table_kernel(apc_problem p, double* __restrict__ table) {
  pair_table_block(p, table, blockIdx.x);
}

// ---------------------------------------------------------------------------
// Kernel: cost entries
// ---------------------------------------------------------------------------
constexpr int kPerLane = 4;  // entries per lane of a work item of APC_ITEM_ENTRIES entries
constexpr unsigned kXcdRun = 64;  // consecutive workgroups of wide items that share an XCD
static_assert(sizeof(apc_edge) == 64, "edge record layout");
static_assert(64 * kPerLane == APC_ITEM_ENTRIES, "work items are built for this kernel");

// comm / transition of one entry, general path (direct evaluation, missing
// specs, default rows).
__device__ __forceinline__ void eval_entry(const apc_problem& p, const apc_edge& ed, uint32_t o,
                                           uint32_t j, double& comm, int& trans) {
  const bool has_producer = (ed.flags & APC_EDGE_HAS_PRODUCER) != 0;  // wave-uniform
  uint32_t sw = APC_SPEC_NONE, tw, src_plc = 0, tgt_plc = 0;
  int64_t nbytes = 0;
  bool contig = true;
  if (p.spec_recs) {  // one record per side
    const apc_spec_rec rt = p.spec_recs[(size_t)ed.dst_list + o];
    tw = rt.word;
    tgt_plc = rt.plc;
    if (has_producer) {
      const apc_spec_rec rs = p.spec_recs[(size_t)ed.src_list + j];
      sw = rs.word;
      src_plc = rs.plc;
      nbytes = rs.nbytes2 >> 1;
      contig = (rs.nbytes2 & 1) != 0;
    }
  } else {
    tw = p.lists[(size_t)ed.dst_list + o];
    if (has_producer) sw = p.lists[(size_t)ed.src_list + j];
    if (sw != APC_SPEC_NONE && tw != APC_SPEC_NONE) {
      src_plc = load_tuple(p.tuple_plc, sw & kTupleMask);
      tgt_plc = load_tuple(p.tuple_plc, tw & kTupleMask);
      meta_bytes_contig(p, sw >> APC_TUPLE_BITS, nbytes, contig);
    }
  }
  if (sw != APC_SPEC_NONE && tw != APC_SPEC_NONE) {
    trans = ((sw & kTupleMask) != (tw & kTupleMask));
    comm = redistribute_cost(src_plc, tgt_plc, nbytes, contig, p.model);
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
      const uint8_t f = (uint8_t)(trans | (finite ? 0 : APC_ENTRY_NONFINITE));
      if (kN > kPerLane) {
        // Wide items are for outputs that stream past every cache: stored as such they
        // leave the block table in L2 (measured at 418 M entries: 1.39 -> 1.33 ms, with
        // the workgroup order below 1.21 ms; on the 5.5 M entries of the headline graph
        // the same stores cost 2 us of 19, which is why narrow items keep plain ones).
        if (comm) __builtin_nontemporal_store(cm, comm + idx);
        if (cost) __builtin_nontemporal_store(c, cost + idx);
        if (flags) __builtin_nontemporal_store(f, flags + idx);
      } else {
        if (comm) comm[idx] = cm;
        if (cost) cost[idx] = c;
        // byte stores: gathering a lane's four flags into one 4-byte store through
        // cross-lane exchanges measured slower
        if (flags) flags[idx] = f;
      }
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
  // Workgroup b runs on XCD b mod 8, each with an L2 of its own.  With wide items
  // (large problems) a run of kXcdRun consecutive workgroups' worth of items goes to
  // one XCD, so that the items of an edge block, which read one matrix of the block
  // table, mostly share an L2 instead of fetching it into all eight; the eight XCDs
  // still write neighbouring runs (1 MB of costs each), which keeps the store stream
  // compact.  The launcher rounds the grid up to whole groups of 8 runs.
  unsigned wg = blockIdx.x;
  if (kN > kPerLane) {
    const unsigned k = wg >> 3, xcd = wg & 7;
    wg = ((k / kXcdRun) * 8 + xcd) * kXcdRun + (k % kXcdRun);
  }
  const int w = __builtin_amdgcn_readfirstlane((int)(wg * (kBlock / 64) + (threadIdx.x >> 6)));
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

// One wavefront per work item, nothing predicated: the form the launcher takes
// whenever all three outputs are asked for and the grid can hold a wave per item
// (it always can below 8.6e9 entries).  A wave's life is a chain of dependent
// accesses (item record, index loads of a compressed matrix, matrix and per-arg
// loads, stores) and the chip hides it with the waves it holds, so the body is
// written for few registers: no loop state, and lanes outside the block (before
// its first entry in the block's first item, past its last in the last one) repeat
// the nearest entry of the block (same loads, same values stored to the same
// place) instead of being switched off, which keeps every access of the wave
// unconditional.
//
// What depends on an entry's row alone (the per-arg compute term, the row's index
// in a compressed matrix) is not loaded per entry with one vector load whose lanes
// all read the same address: such a load costs about as much as a 64-way gather
// on this chip.  Measured on MI355X (264 M entries of compressed matrices): with
// eight such loads of the row index per lane the kernel took 1.11 ms, without them
// 0.86 ms.  Rows of 64 entries and more: 64 consecutive entries lie in two rows
// at most, the same two for the whole wave, so their values come through the
// scalar cache and a lane picks one of the two (0.86 ms).  Shorter rows: lane r of
// the wave loads the values of the item's r-th row, one coalesced load each, and an
// entry takes its row's values from that lane through the cross-lane network
// (0.95 ms when rows of every length go this way); only an item of more than 64 rows
// (rows shorter than 9 entries) loads per entry.
template <bool kSqueezed, int kN>
__global__ void __launch_bounds__(kBlock)
edge_cost_item_kernel(apc_problem p, const double* __restrict__ table,
                      const double* __restrict__ per_arg, double* __restrict__ comm,
                      double* __restrict__ cost, uint8_t* __restrict__ flags, int clamp_inf) {
  // runs of kXcdRun consecutive workgroups per XCD, as in edge_cost_kernel; here for narrow
  // items too (headline graph, event-timed A/B on one box: 18.7 us against 19.2 us)
  unsigned wg = blockIdx.x;
  {
    const unsigned k = wg >> 3, xcd = wg & 7;
    wg = ((k / kXcdRun) * 8 + xcd) * kXcdRun + (k % kXcdRun);
  }
  const int i = __builtin_amdgcn_readfirstlane((int)(wg * (kBlock / 64) + (threadIdx.x >> 6)));
  if (i >= p.n_item) return;
  const int lane = threadIdx.x & 63;
  const apc_edge ed = p.items[i];
  const uint32_t ssrc = (uint32_t)ed.ssrc;
  const uint32_t last = ssrc * (uint32_t)ed.sdst - 1u;
  const uint32_t last_row = (uint32_t)ed.sdst - 1u;
  const bool compressed = kSqueezed && (ed.flags & APC_EDGE_COMPRESSED);  // wave-uniform
  const uint32_t usrc = (uint32_t)ed.flags >> APC_EDGE_USRC_SHIFT;
  const int32_t* __restrict__ list_uidx = p.list_uidx;
  const double* __restrict__ matrix =  // wave-uniform
      ed.table_off >= 0 ? table + ed.table_off : p.default_vals + ed.default_off;
  uint32_t l[kN], o[kN], urow[kN];
  double pa[kN];
#pragma unroll
  for (int k = 0; k < kN; ++k) {
    // the first item of a block may start up to 48 slots before it (local0 negative
    // modulo 2^32): those lanes repeat the block's first entry, the ones past its end the last
    const int32_t lk = (int32_t)ed.local0 + (k * 64 + lane);
    l[k] = (uint32_t)(lk < 0 ? 0 : (lk > (int32_t)last ? (int32_t)last : lk));
    o[k] = ed.magic ? __umulhi(l[k], ed.magic) : l[k] / ssrc;
    urow[k] = 0;
  }
  // rows of the item: from the row of its first entry (lane 0) to that of its last (lane 63)
  const uint32_t o_first = (uint32_t)__builtin_amdgcn_readfirstlane((int)o[0]);
  const uint32_t o_last = (uint32_t)__builtin_amdgcn_readlane((int)o[kN - 1], 63);
  if (ssrc >= 64) {
    // 64 consecutive entries of rows this long lie in two rows at most, that of lane 0's
    // entry and the next: the same two addresses for the whole wave, read through the
    // scalar cache, and a lane picks one of the two values
#pragma unroll
    for (int k = 0; k < kN; ++k) {
      const uint32_t oa = (uint32_t)__builtin_amdgcn_readfirstlane((int)o[k]);
      const uint32_t ob = oa < last_row ? oa + 1u : last_row;
      const double pa_a = per_arg[ed.comp_base + oa], pa_b = per_arg[ed.comp_base + ob];
      pa[k] = o[k] == oa ? pa_a : pa_b;
      if (compressed) {
        const uint32_t u_a = (uint32_t)list_uidx[(size_t)ed.dst_list + oa];
        const uint32_t u_b = (uint32_t)list_uidx[(size_t)ed.dst_list + ob];
        urow[k] = o[k] == oa ? u_a : u_b;
      }
    }
  } else if (o_last - o_first < 64u) {
    // lane r loads the values of the item's r-th row; an entry takes its row's from there
    const uint32_t row = o_first + (uint32_t)lane < last_row ? o_first + (uint32_t)lane : last_row;
    const double pa_row = per_arg[ed.comp_base + row];
    const int pa_lo = (int)(uint32_t)__double_as_longlong(pa_row);
    const int pa_hi = (int)(uint32_t)((uint64_t)__double_as_longlong(pa_row) >> 32);
    const int u_row = compressed ? list_uidx[(size_t)ed.dst_list + row] : 0;
#pragma unroll
    for (int k = 0; k < kN; ++k) {
      const int from = (int)((o[k] - o_first) << 2);  // byte address of the lane that holds the row
      const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute(from, pa_lo);
      const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute(from, pa_hi);
      pa[k] = __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
      if (compressed) urow[k] = (uint32_t)__builtin_amdgcn_ds_bpermute(from, u_row);
    }
  } else {
#pragma unroll
    for (int k = 0; k < kN; ++k) {
      pa[k] = per_arg[ed.comp_base + o[k]];
      if (compressed) urow[k] = (uint32_t)list_uidx[(size_t)ed.dst_list + o[k]];
    }
  }
  uint32_t at[kN];
  if (compressed) {
    // the matrix has one row / column per distinct spec word of the two runs
#pragma unroll
    for (int k = 0; k < kN; ++k)
      at[k] = urow[k] * usrc + (uint32_t)list_uidx[(size_t)ed.src_list + (l[k] - o[k] * ssrc)];
  } else {
#pragma unroll
    for (int k = 0; k < kN; ++k) at[k] = l[k];
  }
  double raw[kN];
#pragma unroll
  for (int k = 0; k < kN; ++k) raw[k] = matrix[at[k]];
#pragma unroll
  for (int k = 0; k < kN; ++k) {
    const int trans = (int)((uint64_t)__double_as_longlong(raw[k]) >> 63);
    const double cm = fabs(raw[k]);
    double c = (cm + pa[k]) + (double)trans;  // optimize_sharding.py:544
    const bool finite = isfinite(c);
    if (clamp_inf && !finite) c = 10000.0;
    const int64_t idx = ed.off + l[k];
    const uint8_t f = (uint8_t)(trans | (finite ? 0 : APC_ENTRY_NONFINITE));
    if (kN > kPerLane) {  // outputs that stream past every cache: see item_store
      __builtin_nontemporal_store(cm, comm + idx);
      __builtin_nontemporal_store(c, cost + idx);
      __builtin_nontemporal_store(f, flags + idx);
    } else {
      comm[idx] = cm;
      cost[idx] = c;
      flags[idx] = f;
    }
  }
}

// Plain copy kernel of known size: the reference point against which the
// hardware traffic counters are scaled when a profile is taken.
__global__ void __launch_bounds__(kBlock)
calibration_copy_kernel(const double2_t* __restrict__ src, double2_t* __restrict__ dst, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

int launch_prepare(const apc_problem* p, double* table, bool do_nodes, double* compute,
                   double* per_arg, int32_t* status, hipStream_t stream) {
  int table_blocks = (table && p->table_size > 0) ? p->n_table_unit : 0;
  if (table_blocks > 0 && p->n_lut_table_tile > 0) {  // tile by tile, per-source terms in LDS (lut.hip)
    if (int rc = apc_impl::launch_lut_table(p, table, stream)) return rc;
    table_blocks = 0;
  }
  if (table_blocks > kFusedTableBlocks) {  // a launch of its own: see pair_table_kernel
    hipLaunchKernelGGL(pair_table_kernel, dim3(table_blocks), dim3(256), 0, stream, *p, table);
    if (int rc = check_launch("pair_table_kernel")) return rc;
    table_blocks = 0;
  }
  const int64_t chunks = (p->max_nstrat + 63) >> 6;
  const int64_t units = (int64_t)p->n_comp_node * chunks;  // one workgroup per 64 strategies of a node
  if (do_nodes && (chunks < 1 || units > (1ll << 30)))
    return fail(APC_ERR_INVALID, "launch_prepare: max_nstrat must be >= 1 and n_comp_node * chunks < 2^30%s");
  const int node_blocks = do_nodes ? (int)units : 0;
  if (table_blocks + node_blocks == 0) return 0;
  // LDS for the value table of a node workgroup (a CU has 160 KB); beyond 96 KB
  // per workgroup, sizes are read on demand instead
  const int64_t words = ((int64_t)p->max_rank + (int64_t)p->max_node_args * (p->max_rank + 2)) * 64;
  const int slow = ((kNodeHeader + words) * 8 > 96 * 1024 || p->n_meta == 0 || p->n_tuple == 0) ? 1 : 0;
  const size_t lds = do_nodes ? (size_t)(kNodeHeader + (slow ? 0 : words)) * 8 : 0;
  if (lds > 0) {  // dynamic LDS beyond the 64 KB default needs the limit raised: once per device
    DeviceState* dev = current_device_state();
    if (!dev) return APC_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(dev->mu);
    if (!dev->lds_limit_raised) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(prepare_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
      if (e != hipSuccess) {
        snprintf(g_err, sizeof(g_err), "hipFuncSetAttribute: %s", hipGetErrorString(e));
        return APC_ERR_LAUNCH;
      }
      dev->lds_limit_raised = true;
    }
  }
  hipLaunchKernelGGL(prepare_kernel, dim3(table_blocks + node_blocks), dim3(256), lds, stream, *p,
                     table, table_blocks, slow, compute, per_arg, status);
  return check_launch("prepare_kernel");
}

}  // namespace

extern "C" {

int apc_version(void) { return 5; }

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

int apc_xgmi_topology(const apc_xgmi_config* cfg, const int32_t* mesh_shape, int32_t ndim, double* bw,
                      double* lat, double* a2a_bw) {
  if (!cfg || !mesh_shape || !bw || !lat || !a2a_bw || ndim < 1 || ndim > APC_MAX_MESH_DIMS)
    return fail(APC_ERR_INVALID, "apc_xgmi_topology: bad arguments%s");
  if (cfg->gpus_per_node < 1 || cfg->links_per_gpu < 1 || !(cfg->link_gbps > 0.0) || !(cfg->nic_gbps > 0.0))
    return fail(APC_ERR_INVALID, "apc_xgmi_topology: gpus_per_node, links_per_gpu, link_gbps, nic_gbps must be positive%s");
  const double one_way = cfg->link_gbps / 2.0;
  int64_t total = 1;
  for (int i = ndim - 1; i >= 0; --i) {
    const int n = mesh_shape[i];
    if (n < 1) return fail(APC_ERR_INVALID, "apc_xgmi_topology: mesh size < 1%s");
    total *= n;
    if (total <= cfg->gpus_per_node) {
      const int links = n - 1 < cfg->links_per_gpu ? n - 1 : cfg->links_per_gpu;
      bw[i] = one_way;
      a2a_bw[i] = one_way * (double)(links > 1 ? links : 1);
      lat[i] = cfg->lat_intra_us;
    } else {
      bw[i] = cfg->nic_gbps;
      a2a_bw[i] = cfg->nic_gbps;
      lat[i] = cfg->lat_inter_us;
    }
  }
  return 0;
}

namespace {
// Device table of autoparallel/cost_models/compute_estimation.py:66-255, in its
// order (the first entry whose name occurs in the device name wins): memory
// bandwidth in bytes/s and dense GEMM TFLOP/s for f64, f32 (tf32 where the
// device has it), f16, bf16, int8; 0 = the reference lists no figure.
struct DeviceRow { const char* name; double gmem_bw; double tflops[APC_NUM_DTYPES]; };
constexpr double kGiB = 1024.0 * 1024.0 * 1024.0, kTiB = 1024.0 * kGiB;
const DeviceRow kDevices[] = {
    {"H100", 3.35 * kTiB, {67, 989 / 2, 1979 / 2, 1979 / 2, 3958 / 2}},  // integer halves, as written there
    {"B200", 7.7 * kTiB, {37, 2200 / 2, 4500 / 2, 4500 / 2, 9000 / 2}},
    {"A100", 2 * kTiB, {19.5, 156, 312, 312, 624}},
    {"A30", 933 * kGiB, {10.3, 82, 165, 165, 330}},
    {"A10G", 933 * kGiB, {0, 31.2, 125, 125, 250}},
    {"T4", 300 * kGiB, {0, 8.1, 65, 0, 130}},
    {"V100", 900 * kGiB, {7.8, 15.7, 125, 0, 0}},
    {"P100", 732 * kGiB, {5.3, 10.6, 21.2, 0, 0}},
    {"AMD Instinct MI200X", 1.6 * kTiB, {45.3, 45.3, 181.0, 181.0, 181.0}},
    {"AMD Instinct MI300X", 5.3 * kTiB, {163.4, 653.7, 1307.4, 1307.4, 2614.9}},
    {"AMD Instinct MI325X", 6.0 * kTiB, {163.4, 653.7, 1307.4, 1307.4, 2614.9}},
    {"AMD Instinct MI350X", 8.0 * kTiB, {72.1, 144.2, 2309.6, 2309.6, 4614.0}},
    {"AMD Instinct MI355X", 8.0 * kTiB, {78.6, 157.3, 2516.6, 2516.6, 5033.2}},
    {"Max 1550", 3.3 * kTiB, {46, 46, 367, 367, 734}},
};
}  // namespace

int apc_device_limits(const char* device_name, apc_model* model) {
  if (!device_name || !model) return fail(APC_ERR_INVALID, "apc_device_limits: null argument%s");
  for (int i = 0; i < APC_NUM_DTYPES; ++i) model->tflops[i] = 0.0;
  // dtype codes: 0 f64, 1 f32, 2 f16, 3 bf16, 4 int8
  for (const DeviceRow& d : kDevices) {
    // compute_estimation.py:262-266: substring match, and PG509 boards are A100s
    if (strstr(device_name, d.name) || (!strcmp(d.name, "A100") && strstr(device_name, "PG509"))) {
      model->gmem_bw = d.gmem_bw;
      for (int i = 0; i < APC_NUM_DTYPES; ++i) model->tflops[i] = d.tflops[i];
      return 0;
    }
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
  if (!table && p->n_lut_entry_tile > 0)  // direct evaluation by tiles (lut.hip), same bits
    return apc_impl::launch_lut_entries(p, per_arg, comm, cost, flags, clamp_inf, stream, start, stop);
  unsigned grid = (unsigned)((p->n_item + (kBlock / 64) - 1) / (kBlock / 64));
  // Measured on MI355X: the table kernel (8 waves per SIMD) is fastest with one
  // wave per item, the direct kernel (4 per SIMD, long-lived waves) with a few
  // items per wave; the caps only bound the grid of very large problems.
  const unsigned cap = table ? (1u << 22) : (1u << 14);
  if (grid > cap) grid = cap;
  const bool wide = p->item_entries == 2 * APC_ITEM_ENTRIES;
  const bool wave_per_item = table && comm && cost && flags && (unsigned)((p->n_item + 3) / 4) <= cap;
  if (wide || wave_per_item)
    grid = (grid + 8 * kXcdRun - 1) / (8 * kXcdRun) * (8 * kXcdRun);  // whole groups of runs: see the kernels
  if (wide && !table)
    return fail(APC_ERR_INVALID, "apc_edge_costs: work items of 512 entries need a block table%s");
#define APC_LAUNCH_EDGE(MODE, N)                                                                   \
  hipExtLaunchKernelGGL((edge_cost_kernel<MODE, N>), dim3(grid), dim3(kBlock), 0, stream, start,   \
                        stop, 0, *p, table, per_arg, comm, cost, flags, clamp_inf)
#define APC_LAUNCH_ITEMS(SQ, N)                                                                    \
  hipExtLaunchKernelGGL((edge_cost_item_kernel<SQ, N>), dim3(grid), dim3(kBlock), lds, stream,    \
                        start, stop, 0, *p, table, per_arg, comm, cost, flags, clamp_inf)
  // Waves per SIMD of the wave-per-item kernel.  It fits eight, and a problem whose block
  // table is far larger than the caches wants them all (264 M entries over a table of
  // 100 MB and more: 0.95 ms with eight, 1.13 ms with four).  A large problem whose table
  // the L2s can hold is bound by its stores alone and runs best with four (418 M entries,
  // table of 15 MB: 1.19 ms against 1.27 ms with eight; a plain fill of the same bytes takes
  // 1.18 ms).  The kernel uses no LDS, so a workgroup that asks for a quarter of a CU's
  // 160 KB limits a CU to four workgroups: one wave per SIMD each.
  const size_t lds = wide && (size_t)p->table_size * sizeof(double) <= ((size_t)32 << 20) ? (size_t)40 << 10 : 0;
  if (wave_per_item) {
    if (p->list_uidx) {
      if (wide) APC_LAUNCH_ITEMS(true, 2 * kPerLane); else APC_LAUNCH_ITEMS(true, kPerLane);
    } else {
      if (wide) APC_LAUNCH_ITEMS(false, 2 * kPerLane); else APC_LAUNCH_ITEMS(false, kPerLane);
    }
  } else if (table && p->list_uidx) {
    if (wide) APC_LAUNCH_EDGE(2, 2 * kPerLane); else APC_LAUNCH_EDGE(2, kPerLane);
  } else if (table) {
    if (wide) APC_LAUNCH_EDGE(1, 2 * kPerLane); else APC_LAUNCH_EDGE(1, kPerLane);
  } else {
    APC_LAUNCH_EDGE(0, kPerLane);
  }
#undef APC_LAUNCH_EDGE
#undef APC_LAUNCH_ITEMS
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

}  // extern "C"
namespace apc_impl {
bool timer_events(void* timer, int slot, hipEvent_t* start, hipEvent_t* stop) {
  apc_timer* t = static_cast<apc_timer*>(timer);
  if (!t || slot < 0 || slot >= t->n) return false;
  *start = t->ev[2 * slot];
  *stop = t->ev[2 * slot + 1];
  return true;
}
}  // namespace apc_impl
extern "C" {

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

int apc_build_all_noalloc(const apc_problem* p, double* compute, double* per_arg, int32_t* status,
                          double* comm, double* cost, uint8_t* flags, int32_t clamp_inf,
                          void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->table_size > APC_NOALLOC_MAX_TABLE) {
    snprintf(g_err, sizeof(g_err),
             "apc_build_all_noalloc: the block table has %lld doubles, the static scratch holds %lld; "
             "use apc_build_all with a table of the caller's",
             (long long)p->table_size, (long long)APC_NOALLOC_MAX_TABLE);
    return APC_ERR_INVALID;
  }
  // without a block table (table_size 0) every edge is evaluated directly, as
  // apc_build_all does with table == NULL
  double* table = nullptr;
  if (p->table_size > 0) {
    table = resolve_scratch();
    if (!table) return APC_ERR_LAUNCH;
  }
  return apc_build_all(p, table, compute, per_arg, status, comm, cost, flags, clamp_inf, stream);
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
}  // extern "C"
