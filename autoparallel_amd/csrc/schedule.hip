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
  if (order)
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
