// Schedule estimator (gfx950): timeline and peak memory of a lowered graph under
// many candidate orders, one lane per order.
//
// The walk over the nodes of one order is a chain of dependent max/add steps
// (estimate_graph_metrics, autoparallel/graph_passes/estimate_graph_metrics.py:
// 30-89), so the parallelism is across orders: lane b of the grid walks order b.
// Node attributes are read through the order (a gather of a few bytes per
// step, the same address for every lane when the orders agree); the two pieces
// of per-order state that do not fit registers, the end time of every
// collective and the unscheduled-reader count of every storage, live in
// caller-provided scratch laid out [index][order] so that the lanes of a
// wavefront touch consecutive addresses.  Floating-point sums are formed in the
// reference's order, one rounding per operation (-ffp-contract=off).
//
// A step is a chain of dependent accesses (order -> node attributes -> storages
// -> reader counts, and the counts again after the node's allocations), and with
// a wavefront per CU nothing hides their latency.  When the graph is small enough
// (48 bytes per node and 264 per storage within the 160 KB of a CU's LDS) the
// wavefront first builds one record per node in LDS and keeps the reader counts
// there too, [storage][lane]; a step then reads global memory only for the order
// (requested eight steps ahead) and for the end times of collectives; and not for
// those either when the caller has numbered the nodes that have one (comm_slot)
// and 512 bytes for each of them fit as well.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "apc.h"

extern "C" __attribute__((visibility("hidden"))) void apc_internal_set_error(const char* msg);

namespace {

constexpr int kBlock = 64;  // one wavefront: a block's lanes finish together

__device__ __forceinline__ double pymax(double a, double b) {  // Python's max(a, b)
  return b > a ? b : a;
}

// kIdentity: every lane walks the graph's own order (n_sched == 1 in practice).
template <bool kIdentity>
__global__ void __launch_bounds__(kBlock)
schedule_metrics_kernel(apc_schedule s, const int32_t* __restrict__ order, int64_t n_sched,
                        double* __restrict__ end_time, int32_t* __restrict__ remaining,
                        double* __restrict__ times, int64_t* __restrict__ peak_out) {
  const int64_t b = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (b >= n_sched) return;
  const int N = s.n_node, S = s.n_storage;
  // absent from global_time: a negative end time (times are never negative)
  for (int i = 0; i < N; ++i) end_time[(int64_t)i * n_sched + b] = -1.0;
  for (int k = 0; k < S; ++k) remaining[(int64_t)k * n_sched + b] = s.st_users[k];

  double cur[APC_SCHED_MAX_STREAMS];
  bool seen[APC_SCHED_MAX_STREAMS];
#pragma unroll
  for (int t = 0; t < APC_SCHED_MAX_STREAMS; ++t) { cur[t] = 0.0; seen[t] = (t == 0); }
  double compute_time = 0.0, comm_time = 0.0, exposed = 0.0;
  int64_t live = s.initial_bytes, peak = s.initial_bytes;
  const int32_t* ord = kIdentity ? nullptr : order + b * N;

  // What a step needs to know about its node is requested one step ahead, before the
  // step's own stores to the scratch arrays (which the compiler must assume to alias
  // the schedule's arrays): a step is a chain of dependent gathers (order -> node
  // attributes -> storages -> scratch), and with one wavefront per CU nothing else hides
  // them.
  struct NodeAttr { int v; double dur; int tid, fl, u0, u1, a0, a1, wait_src; };
  auto load_attr = [&](int v) -> NodeAttr {
    NodeAttr n;
    n.v = v; n.dur = s.dur[v]; n.tid = s.stream[v]; n.fl = s.flags[v];
    n.u0 = s.use_off[v]; n.u1 = s.use_off[v + 1];
    n.a0 = s.alloc_off[v]; n.a1 = s.alloc_off[v + 1];
    n.wait_src = s.wait_src[v];
    return n;
  };
  NodeAttr nxt = {};
  int v_after = 0;  // the node of step t + 2
  if (N > 0) nxt = load_attr(kIdentity ? 0 : ord[0]);
  if (N > 1) v_after = kIdentity ? 1 : ord[1];
  for (int t = 0; t < N; ++t) {
    const NodeAttr cur_n = nxt;
    if (t + 1 < N) nxt = load_attr(v_after);
    if (t + 2 < N) v_after = kIdentity ? t + 2 : ord[t + 2];
    const int v = cur_n.v;
    const double dur = cur_n.dur;
    const int tid = cur_n.tid;
    const int fl = cur_n.fl;

    // ---- memory (MemoryTracker.schedule_node)
    const int u0 = cur_n.u0, u1 = cur_n.u1;
    for (int q = u0; q < u1; ++q) {  // this reader is now scheduled
      const int64_t at = (int64_t)s.use_st[q] * n_sched + b;
      remaining[at] = remaining[at] - 1;
    }
    if (!(fl & APC_SCHED_NO_MEM)) {
      for (int q = cur_n.a0; q < cur_n.a1; ++q) live += s.st_bytes[s.alloc_st[q]];
      peak = live > peak ? live : peak;
      for (int q = u0; q < u1; ++q) {
        const int k = s.use_st[q];
        if (s.st_freeable[k] && remaining[(int64_t)k * n_sched + b] == 0) live -= s.st_bytes[k];
      }
    }

    // ---- timeline; cur[tid] with tid a lane-varying index: select, not index
    double c0 = cur[0], ct = c0;
    bool known = false;
#pragma unroll
    for (int k = 0; k < APC_SCHED_MAX_STREAMS; ++k)
      if (k == tid) { ct = cur[k]; known = seen[k]; }
    if (!known) ct = c0;  // a stream starts at the compute stream's present time
    if (fl & APC_SCHED_COMM) {
      if (tid == 0 && (fl & APC_SCHED_WAIT)) {
        const int src = cur_n.wait_src;
        double end = c0;
        if (src >= 0) {
          const double e = end_time[(int64_t)src * n_sched + b];
          if (e >= 0.0) {
            end = e;
            end_time[(int64_t)src * n_sched + b] = -1.0;  // global_time.pop
          }
        }
        const double stall = end - c0;
        exposed += stall > 0.0 ? stall : 0.0;
        ct = pymax(ct, end);
      } else {
        ct = pymax(c0, ct);
        comm_time += dur;
      }
    } else {
      compute_time += dur;
    }
    ct += dur + 1.0;
    if (tid == 0) {
      c0 = ct;
    } else {
      c0 += 1.0;
      end_time[(int64_t)v * n_sched + b] = ct;
      if (fl & APC_SCHED_SYNC) {
        const double stall = ct - c0;
        exposed += stall > 0.0 ? stall : 0.0;
        c0 = pymax(c0, ct);
      }
    }
    cur[0] = c0;
#pragma unroll
    for (int k = 1; k < APC_SCHED_MAX_STREAMS; ++k)
      if (k == tid) { cur[k] = ct; seen[k] = true; }
  }
  double total = cur[0];
#pragma unroll
  for (int k = 1; k < APC_SCHED_MAX_STREAMS; ++k)
    if (seen[k]) total = pymax(total, cur[k]);
  times[b * 4 + 0] = total;
  times[b * 4 + 1] = compute_time;
  times[b * 4 + 2] = comm_time;
  times[b * 4 + 3] = exposed;
  peak_out[b] = peak;
}

// ---- the same walk with the schedule and the reader counts in LDS
//
// One wavefront issues an instruction every few cycles at best and a CU holds one to four of
// these workgroups, so the time of a launch is the time of one walk: instructions per step
// times steps.  The step is therefore written without branches: a record names four storages
// (unused places name a spare row that absorbs their updates), the counts are lowered by LDS
// atomics that return nothing, and the timeline's cases are selects.
constexpr int kRecDwords = 12;  // 48 bytes a node
constexpr int kRecUses = 4;     // storages a record names itself; further ones are read from use_st
constexpr int kAhead = 8;       // steps between the request of an order's entry and its use
constexpr int kLdsLimit = 160 * 1024;

// NodeRec.bits: the stream in the low byte, the number of storages read from bit 16 on, and
enum : int32_t {
  kRecWait = 1 << 8,     // a wait on the compute stream
  kRecComm = 1 << 9,     // any other communication node
  kRecCompute = 1 << 10, // not a communication node
  kRecSync = 1 << 11,    // on a stream of its own, and the compute stream waits for it
  kRecMem = 1 << 12,     // counts for memory
};

struct alignas(16) NodeRec {
  double dur;
  int32_t bits;
  int32_t rd_row;  // row of the end times a wait reads (a row that is always empty for the other nodes)
  int64_t alloc;   // bytes the node allocates (0 if it does not count for memory)
  int32_t wr_row;  // row of the end times the node writes: a wait its collective's, a node on a stream of its own
                   // its own, the others a row nobody reads
  int32_t u0;      // its readers' list in use_st
  int32_t use[kRecUses];  // the first storages of that list; the spare row n_storage in unused places
};
static_assert(sizeof(NodeRec) == kRecDwords * 4, "record layout");

// records, bytes a storage gives back and reader counts [storage][order], each with a spare
// row; the end times [slot][order], if they are kept in LDS too, have two (one always empty,
// one nobody reads)
__host__ __device__ inline int64_t schedule_lds_bytes(int n_node, int n_storage) {
  return (int64_t)n_node * sizeof(NodeRec) + (int64_t)(n_storage + 1) * (8 + kBlock * 4);
}
__host__ __device__ inline int64_t schedule_end_lds_bytes(int n_comm) { return (int64_t)(n_comm + 2) * kBlock * 8; }

// A workgroup walks 64 orders whatever its shape: kWaves wavefronts with 64 / kWaves working
// lanes each, so that the 64 walks are spread over the CU's SIMDs when the LDS a workgroup
// needs leaves room for only one or two of them per CU.
// kEndLds: the end times are rows [slot][order] of LDS, slot = comm_slot of the node; otherwise
// rows [node][order] of end_scratch (row -1: none).
template <bool kIdentity, int kWaves, bool kEndLds>
__global__ void __launch_bounds__(kBlock * kWaves)
schedule_metrics_lds_kernel(apc_schedule s, const int32_t* __restrict__ order, int64_t n_sched,
                            double* __restrict__ end_scratch, double* __restrict__ times,
                            int64_t* __restrict__ peak_out) {
  constexpr int kThreads = kBlock * kWaves, kWork = kBlock / kWaves;
  extern __shared__ __align__(16) unsigned char s_raw[];
  const int N = s.n_node, S = s.n_storage;
  NodeRec* const recs = reinterpret_cast<NodeRec*>(s_raw);
  int64_t* const freed = reinterpret_cast<int64_t*>(s_raw + (size_t)N * sizeof(NodeRec));  // bytes a storage gives back
  int32_t* const remaining = reinterpret_cast<int32_t*>(freed + (S + 1));
  double* const end_lds = reinterpret_cast<double*>(s_raw + schedule_lds_bytes(N, S));
  const int row_empty = s.n_comm, row_unread = s.n_comm + 1;  // kEndLds
  const int thread = threadIdx.x;
  for (int v = thread; v < N; v += kThreads) {
    NodeRec r;
    const int tid = s.stream[v], fl = s.flags[v];
    const bool comm = (fl & APC_SCHED_COMM) != 0;
    const bool wait = comm && tid == 0 && (fl & APC_SCHED_WAIT);
    const bool mem = !(fl & APC_SCHED_NO_MEM);
    r.dur = s.dur[v];
    r.u0 = s.use_off[v];
    const int n_use = s.use_off[v + 1] - r.u0;
    r.bits = tid | (wait ? kRecWait : (comm ? kRecComm : kRecCompute)) |
             (tid != 0 && (fl & APC_SCHED_SYNC) ? kRecSync : 0) | (mem ? kRecMem : 0) | (n_use << 16);
    const int src = wait ? s.wait_src[v] : -1;
    if (kEndLds) {
      const int src_slot = src >= 0 ? s.comm_slot[src] : -1;
      const int own_slot = tid != 0 ? s.comm_slot[v] : -1;
      r.rd_row = src_slot >= 0 && src_slot < s.n_comm ? src_slot : row_empty;
      r.wr_row = wait ? r.rd_row : (own_slot >= 0 && own_slot < s.n_comm ? own_slot : row_unread);
    } else {
      r.rd_row = src;
      r.wr_row = tid != 0 ? v : -1;
    }
    r.alloc = 0;
    if (mem)
      for (int q = s.alloc_off[v]; q < s.alloc_off[v + 1]; ++q) r.alloc += s.st_bytes[s.alloc_st[q]];
#pragma unroll
    for (int i = 0; i < kRecUses; ++i) r.use[i] = i < n_use ? s.use_st[r.u0 + i] : S;
    recs[v] = r;
  }
  for (int k = thread; k <= S; k += kThreads) freed[k] = (k < S && s.st_freeable[k]) ? s.st_bytes[k] : 0;
  for (int i = thread; i < (S + 1) * kBlock; i += kThreads) remaining[i] = i < S * kBlock ? s.st_users[i / kBlock] : 0;
  if (kEndLds)  // absent from global_time: a negative end time (times are never negative)
    for (int i = thread; i < (s.n_comm + 2) * kBlock; i += kThreads) end_lds[i] = -1.0;
  __syncthreads();

  // order `lane` of the workgroup's 64: the first kWork lanes of every wavefront work
  const int lane = (thread >> 6) * kWork + (thread & 63);
  const int64_t b = (int64_t)blockIdx.x * kBlock + lane;
  if ((thread & 63) >= kWork || b >= n_sched) return;  // no barrier follows
  double* const end_time = kEndLds ? end_lds + lane : end_scratch + b;  // this order's column
  const int64_t end_stride = kEndLds ? kBlock : n_sched;
  if (!kEndLds)
    for (int i = 0; i < N; ++i) end_time[i * end_stride] = -1.0;
  int32_t* const my_remaining = remaining + lane;

  double cur[APC_SCHED_MAX_STREAMS];
  bool seen[APC_SCHED_MAX_STREAMS];
#pragma unroll
  for (int t = 0; t < APC_SCHED_MAX_STREAMS; ++t) { cur[t] = 0.0; seen[t] = (t == 0); }
  double compute_time = 0.0, comm_time = 0.0, exposed = 0.0;
  int64_t live = s.initial_bytes, peak = s.initial_bytes;
  const int32_t* ord = kIdentity ? nullptr : order + b * N;

  auto step = [&](int v) {
    const NodeRec r = recs[v];
    const int tid = r.bits & 0xFF;
    const int n_use = (int)((uint32_t)r.bits >> 16);
    const bool is_wait = r.bits & kRecWait, is_comm = r.bits & kRecComm, is_compute = r.bits & kRecCompute;
    const bool is_sync = r.bits & kRecSync, mem = r.bits & kRecMem;
    const double dur = r.dur;
    // ---- memory (MemoryTracker.schedule_node): this reader is now scheduled
#pragma unroll
    for (int i = 0; i < kRecUses; ++i)
      __hip_atomic_fetch_sub(my_remaining + r.use[i] * kBlock, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (n_use > kRecUses)
      for (int q = r.u0 + kRecUses; q < r.u0 + n_use; ++q) my_remaining[s.use_st[q] * kBlock] -= 1;
    live += r.alloc;
    peak = live > peak ? live : peak;
#pragma unroll
    for (int i = 0; i < kRecUses; ++i) {
      const int left = my_remaining[r.use[i] * kBlock];
      const int64_t bytes = freed[r.use[i]];
      live -= (mem && left == 0) ? bytes : 0;
    }
    if (n_use > kRecUses && mem)
      for (int q = r.u0 + kRecUses; q < r.u0 + n_use; ++q) {
        const int k = s.use_st[q];
        if (my_remaining[k * kBlock] == 0) live -= freed[k];
      }
    // ---- timeline; cur[tid] with tid a lane-varying index: select, not index
    double c0 = cur[0], ct = c0;
    bool known = false;
#pragma unroll
    for (int k = 0; k < APC_SCHED_MAX_STREAMS; ++k)
      if (k == tid) { ct = cur[k]; known = seen[k]; }
    if (!known) ct = c0;  // a stream starts at the compute stream's present time
    if (kEndLds) {
      // every node reads a row and writes a row: a wait its collective's (the pop of
      // global_time), a node on a stream of its own its own, the others the spare ones
      const double e = end_time[r.rd_row * kBlock];
      const bool got = e >= 0.0;  // only a wait reads a row that can hold a time
      const double end = got ? e : c0;
      const double stall_w = end - c0;
      exposed += (got && stall_w > 0.0) ? stall_w : 0.0;
      ct = is_wait ? pymax(ct, end) : (is_comm ? pymax(c0, ct) : ct);
      comm_time += is_comm ? dur : 0.0;
      compute_time += is_compute ? dur : 0.0;
      ct += dur + 1.0;
      end_time[r.wr_row * kBlock] = is_wait ? -1.0 : ct;
      const double c0n = c0 + 1.0;
      const double stall_s = ct - c0n;
      exposed += (is_sync && stall_s > 0.0) ? stall_s : 0.0;
      c0 = tid == 0 ? ct : (is_sync ? pymax(c0n, ct) : c0n);
    } else {
      if (is_wait) {
        double end = c0;
        if (r.rd_row >= 0) {
          const double e = end_time[r.rd_row * end_stride];
          if (e >= 0.0) {
            end = e;
            end_time[r.rd_row * end_stride] = -1.0;  // global_time.pop
          }
        }
        const double stall = end - c0;
        exposed += stall > 0.0 ? stall : 0.0;
        ct = pymax(ct, end);
      } else if (is_comm) {
        ct = pymax(c0, ct);
        comm_time += dur;
      } else {
        compute_time += dur;
      }
      ct += dur + 1.0;
      if (tid == 0) {
        c0 = ct;
      } else {
        c0 += 1.0;
        end_time[r.wr_row * end_stride] = ct;
        if (is_sync) {
          const double stall = ct - c0;
          exposed += stall > 0.0 ? stall : 0.0;
          c0 = pymax(c0, ct);
        }
      }
    }
    cur[0] = c0;
#pragma unroll
    for (int k = 1; k < APC_SCHED_MAX_STREAMS; ++k)
      if (k == tid) { cur[k] = ct; seen[k] = true; }
  };

  // The order's entries are requested kAhead steps before their use, every time the same
  // number of loads (past the end the last entry again), so that the wait before a block of
  // steps is for the loads of the block before and not for the ones just issued.
  auto entry = [&](int t) -> int {
    const int tc = t < N ? t : N - 1;
    return (kIdentity || N == 0) ? tc : ord[tc];  // (an empty graph has no entries to read)
  };
  int nxt[kAhead];
#pragma unroll
  for (int i = 0; i < kAhead; ++i) nxt[i] = entry(i);
  for (int t0 = 0; t0 < N; t0 += kAhead) {
    int now[kAhead];
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      now[i] = nxt[i];
      nxt[i] = entry(t0 + kAhead + i);
    }
#pragma unroll
    for (int i = 0; i < kAhead; ++i)
      if (t0 + i < N) step(now[i]);
  }
  double total = cur[0];
#pragma unroll
  for (int k = 1; k < APC_SCHED_MAX_STREAMS; ++k)
    if (seen[k]) total = pymax(total, cur[k]);
  times[b * 4 + 0] = total;
  times[b * 4 + 1] = compute_time;
  times[b * 4 + 2] = comm_time;
  times[b * 4 + 3] = exposed;
  peak_out[b] = peak;
}

int fail(const char* msg) {
  apc_internal_set_error(msg);
  return APC_ERR_INVALID;
}

}  // namespace

extern "C" int apc_schedule_metrics(const apc_schedule* s, const int32_t* order, int64_t n_sched,
                                    double* end_scratch, int32_t* remaining_scratch,
                                    double* times, int64_t* peak, void* stream) {
  if (!s || n_sched < 0) return fail("apc_schedule_metrics: null schedule or negative count");
  if (n_sched == 0) return 0;
  if (s->n_node < 0 || s->n_storage < 0 || s->n_stream < 1 || s->n_stream > APC_SCHED_MAX_STREAMS)
    return fail("apc_schedule_metrics: n_stream must be 1..APC_SCHED_MAX_STREAMS, sizes >= 0");
  if (!times || !peak) return fail("apc_schedule_metrics: null output");
  if (s->n_node > 0 && (!s->dur || !s->stream || !s->flags || !s->wait_src || !s->alloc_off ||
                        !s->use_off || !end_scratch))
    return fail("apc_schedule_metrics: null node array or end_scratch");
  if (s->n_storage > 0 && (!s->st_bytes || !s->st_freeable || !s->st_users || !remaining_scratch))
    return fail("apc_schedule_metrics: null storage array or remaining_scratch");
  if (!order && n_sched != 1)
    return fail("apc_schedule_metrics: the graph's own order (order == NULL) is one schedule");
  const int64_t grid = (n_sched + kBlock - 1) / kBlock;
  if (grid > 0x7FFFFFFF) return fail("apc_schedule_metrics: too many schedules for one launch");
  // Small graphs are walked from LDS; the scratch of the reader counts is then left alone.
  int64_t lds = schedule_lds_bytes(s->n_node, s->n_storage);
  if (lds <= kLdsLimit) {
    if (s->comm_slot && (s->n_comm < 0 || s->n_comm > s->n_node))
      return fail("apc_schedule_metrics: n_comm must be 0..n_node");
    const bool end_lds = s->comm_slot && lds + schedule_end_lds_bytes(s->n_comm) <= kLdsLimit;
    if (end_lds) lds += schedule_end_lds_bytes(s->n_comm);
    // workgroups a CU holds at once: by their LDS, and no more than the launch has for it
    int64_t resident = kLdsLimit / (lds > 0 ? lds : 1);
    const int64_t share = (grid + 255) / 256;
    if (share < resident) resident = share;
    const int waves = resident >= 4 ? 1 : (resident >= 2 ? 2 : 4);
#define APC_SCHED_LAUNCH_(IDENT, WAVES, END)                                                                        \
  do {                                                                                                          \
    if (lds > 64 * 1024) { /* above the default limit of a launch: ask for it (cheap, so asked every time) */   \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(schedule_metrics_lds_kernel<IDENT, WAVES, END>), \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit);                \
      if (e != hipSuccess) return fail("apc_schedule_metrics: hipFuncSetAttribute failed");                     \
    }                                                                                                           \
    hipLaunchKernelGGL((schedule_metrics_lds_kernel<IDENT, WAVES, END>), dim3((unsigned)grid), dim3(kBlock * WAVES), \
                       (size_t)lds, (hipStream_t)stream, *s, order, n_sched, end_scratch, times, peak);         \
  } while (0)
#define APC_SCHED_LAUNCH(IDENT, WAVES)                         \
  do {                                                         \
    if (end_lds) APC_SCHED_LAUNCH_(IDENT, WAVES, true);        \
    else APC_SCHED_LAUNCH_(IDENT, WAVES, false);               \
  } while (0)
    if (!order) APC_SCHED_LAUNCH(true, 4);
    else if (waves == 1) APC_SCHED_LAUNCH(false, 1);
    else if (waves == 2) APC_SCHED_LAUNCH(false, 2);
    else APC_SCHED_LAUNCH(false, 4);
#undef APC_SCHED_LAUNCH
#undef APC_SCHED_LAUNCH_
  } else if (order)
    hipLaunchKernelGGL(schedule_metrics_kernel<false>, dim3((unsigned)grid), dim3(kBlock), 0,
                       (hipStream_t)stream, *s, order, n_sched, end_scratch, remaining_scratch,
                       times, peak);
  else
    hipLaunchKernelGGL(schedule_metrics_kernel<true>, dim3((unsigned)grid), dim3(kBlock), 0,
                       (hipStream_t)stream, *s, order, n_sched, end_scratch, remaining_scratch,
                       times, peak);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    char buf[256];
    snprintf(buf, sizeof(buf), "schedule_metrics_kernel: %s", hipGetErrorString(e));
    apc_internal_set_error(buf);
    return APC_ERR_LAUNCH;
  }
  return 0;
}
