// Host side of the NCCL-tuning collective model: resolves, per mesh dim and
// collective, the (latency, bandwidth) candidates whose minimum the device
// evaluates per entry.  Follows autoparallel/cost_models/nccl_cost_model.py;
// every product, quotient and sum is a separately rounded binary64 operation in
// the order the Python performs it (the file is built with -ffp-contract=off),
// and pow() is the same libm call CPython's float ** makes.
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "apc.h"

// defined beside apc_last_error: records the text it returns
extern "C" __attribute__((visibility("hidden"))) void apc_internal_set_error(const char* msg);

namespace {

enum Func { kAG = 0, kRS = 1, kAR = 2 };
enum Algo { kTree = 0, kRing, kCollnetDirect, kCollnetChain, kNvls, kNvlsTree, kNumAlgo };
enum Proto { kLL = 0, kLL128, kSimple };
enum Arch { kAmpere = 0, kHopper, kBlackwell };

// collective codes of the C ABI (apc_collective_costs): 0 AG, 1 A2A, 2 AR, 3 RS
constexpr int kAbiSlot[3] = {0, 3, 2};

constexpr int kDefaultChannels[3] = {12, 16, 16};

// [algo][proto]  (nccl_cost_model.py:112-146)
constexpr double kBaseLat[kNumAlgo][3] = {{6.8, 14.0, 8.4}, {6.6, 14.0, 8.4}, {0, 0, 0}, {0, 0, 0}, {0, 0, 0}, {0, 0, 0}};
constexpr double kHwLatNvlink[kNumAlgo][3] = {{0.6, 1.25, 4.0}, {0.6, 1.9, 3.4}, {0, 0, 3.7}, {0, 0, 2.8}, {0, 0, 25.0}, {0, 0, 25.0}};
constexpr double kHwLatNet[kNumAlgo][3] = {{5.0, 8.5, 14.0}, {2.7, 4.0, 14.0}, {0, 0, 31.0}, {0, 0, 30.0}, {0, 0, 18.0}, {0, 0, 20.9}};

// [arch][node bucket]  (:148-190)
constexpr double kMaxTreeBw[3][3] = {{24.0, 23.6, 17.8}, {38.7, 41.4, 36.0}, {70.0, 42.8, 24.0}};
constexpr double kMaxNvlsTreeBw[3][3] = {{24.0, 23.6, 17.8}, {0.0, 57.7, 45.5}, {0.0, 96.0, 43.8}};
constexpr double kLLMaxBw[3][3] = {{87.7, 39.0, 20.4}, {141.0, 39.0, 20.4}, {282.0, 39.0, 20.4}};
constexpr double kMaxRingLL128Bw[3][3] = {{20.0, 20.0, 20.0}, {36.7, 36.7, 36.7}, {40.0, 40.0, 40.0}};
constexpr double kMaxTreeLL128Bw[3][3] = {{20.0, 20.0, 20.0}, {36.7, 36.7, 29.0}, {55.6, 31.67, 20.0}};
constexpr double kNvlsEff[3] = {0.0, 0.85, 0.74};

// treeCorrectionFactor[proto][24]  (:192-272)
constexpr double kTreeCorr[3][APC_NCCL_TABLE_LEN] = {
    {1.0, 1.0, 1.0, 1.0, 0.9, 0.8, 0.7, 0.7, 0.7, 0.7, 0.6, 0.5, 0.4, 0.4, 0.5, 0.6, 0.7, 0.8, 0.9, 1.0, 1.0, 1.0, 1.0, 1.0},
    {1.0, 1.0, 1.0, 1.0, 1.0, 0.9, 0.8, 0.8, 0.8, 0.7, 0.6, 0.6, 0.6, 0.6, 0.6, 0.6, 0.8, 0.9, 0.9, 0.9, 0.9, 1.0, 1.0, 1.0},
    {0.9, 0.9, 0.9, 0.9, 0.9, 0.9, 0.9, 0.8, 0.7, 0.6, 0.6, 0.5, 0.5, 0.5, 0.5, 0.6, 0.7, 0.8, 0.7, 0.7, 0.8, 0.9, 0.9, 0.9}};
// fitted ramps, index log2(bytes per rank >> 6)  (:669-697, :862-890, :900-907, :947-975)
constexpr double kRingCorr[APC_NCCL_TABLE_LEN] = {1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 0.10, 0.18, 0.30, 0.43, 0.63, 0.55, 0.78, 0.93, 1, 1, 1, 1, 1};
constexpr double kNvlsTreeRamp[APC_NCCL_TABLE_LEN] = {1, 1, 1, 1, 1, 1, 1, 1, 0.10, 0.10, 0.15, 0.28, 0.41, 0.55, 0.72, 0.88, 1, 1, 1, 1, 1, 1, 1, 1};
constexpr double kFullMeshRamp[APC_NCCL_TABLE_LEN] = {0.01, 0.02, 0.03, 0.06, 0.10, 0.16, 0.25, 0.36, 0.68, 0.68, 0.68, 0.68, 0.68, 0.68, 0.68, 0.68, 0.68, 0.68, 0.79, 0.87, 0.87, 0.87, 0.87, 0.87};
constexpr double kA2aNicRamp[APC_NCCL_TABLE_LEN] = {1, 1, 1, 1, 1, 1, 1, 1, 0.28, 0.28, 0.35, 0.43, 0.62, 0.71, 0.82, 0.89, 0.92, 0.95, 1, 1, 1, 1, 1, 1};

constexpr double kNetOverhead = 1.0;       // :275
constexpr double kRingSyncPerNode = 4.7;   // :727
constexpr double kBlackwellScale = 640.0 / 320.0;  // :747
constexpr double kA2aCeLat = 50.0;         // :921
constexpr double kA2aSmCorr = 0.7;         // :926
constexpr double kA2aNicOverhead = 0.44;   // :938

struct Point { int x; double y; };
// intra-node NVSwitch measurements (:737-746): [func] -> (ranks, value)
constexpr Point kSwitchBw[3][3] = {{{2, 537.0}, {4, 434.0}, {8, 394.0}}, {{2, 537.0}, {4, 434.0}, {8, 394.0}}, {{2, 324.0}, {4, 236.0}, {8, 267.0}}};
constexpr Point kSwitchLat[3][3] = {{{2, 8.0}, {4, 17.0}, {8, 30.0}}, {{2, 8.0}, {4, 17.0}, {8, 30.0}}, {{2, 10.0}, {4, 15.0}, {8, 31.0}}};
constexpr Point kA2aNodeLat[5] = {{2, 37.0}, {4, 42.0}, {8, 60.0}, {16, 98.0}, {32, 290.0}};  // :932

// multi-node H100 NVSwitch tuning tables (:764-853): rows ordered by
// nodes (2,4,8,16,32) x ranks per node (1,2,4,8); columns LL, LL128, Simple
struct LatBw { double lat, bw; };
constexpr LatBw kAgRsRing[20][3] = {
    {{11.6, 48.0}, {22.5, 88.3}, {22.4, 96.0}},     {{11.3, 52.0}, {21.8, 117.8}, {29.2, 128.0}},
    {{15.3, 44.6}, {29.4, 201.9}, {42.8, 219.4}},   {{23.3, 41.6}, {44.6, 313.2}, {70.0, 409.6}},
    {{21.6, 27.2}, {39.5, 58.9}, {50.4, 64.0}},     {{18.7, 23.3}, {33.6, 100.9}, {64.0, 109.7}},
    {{26.7, 21.8}, {48.8, 188.4}, {91.2, 204.8}},   {{42.7, 21.1}, {79.2, 303.1}, {145.6, 396.4}},
    {{41.6, 23.3}, {73.5, 50.5}, {106.4, 54.9}},    {{33.5, 21.8}, {57.2, 94.2}, {133.6, 102.4}},
    {{49.5, 21.1}, {87.6, 182.3}, {188.0, 198.2}},  {{81.5, 20.7}, {148.4, 298.3}, {296.8, 390.1}},
    {{81.6, 21.8}, {141.5, 47.1}, {218.4, 51.2}},   {{63.1, 21.1}, {104.4, 91.2}, {272.8, 99.1}},
    {{95.1, 20.7}, {165.2, 179.4}, {381.6, 195.0}}, {{159.1, 20.6}, {286.8, 295.9}, {599.2, 387.0}},
    {{161.6, 21.1}, {277.5, 45.6}, {442.4, 49.5}},  {{122.3, 20.7}, {198.8, 89.7}, {551.2, 97.5}},
    {{186.3, 20.6}, {320.4, 178.0}, {768.8, 193.5}}, {{314.3, 20.5}, {563.6, 294.8}, {1204.0, 385.5}}};
constexpr LatBw kArTree[20][3] = {
    {{16.8, 9.3}, {31.0, 31.2}, {36.4, 35.2}},    {{18.0, 16.6}, {33.5, 62.4}, {44.4, 70.4}},
    {{20.4, 16.6}, {38.5, 124.8}, {60.4, 140.8}}, {{25.2, 16.6}, {48.5, 124.8}, {92.4, 140.8}},
    {{26.8, 4.9}, {48.0, 17.6}, {64.4, 18.8}},    {{28.0, 8.7}, {50.5, 35.2}, {72.4, 37.5}},
    {{30.4, 8.7}, {55.5, 70.4}, {88.4, 75.1}},    {{35.2, 8.7}, {65.5, 98.6}, {120.4, 122.4}},
    {{36.8, 4.9}, {65.0, 17.6}, {92.4, 18.8}},    {{38.0, 8.7}, {67.5, 35.2}, {100.4, 37.5}},
    {{40.4, 8.7}, {72.5, 70.4}, {116.4, 75.1}},   {{45.2, 8.7}, {82.5, 98.6}, {148.4, 122.4}},
    {{46.8, 4.9}, {82.0, 17.6}, {120.4, 18.8}},   {{48.0, 8.7}, {84.5, 35.2}, {128.4, 37.5}},
    {{50.4, 8.7}, {89.5, 70.4}, {144.4, 75.1}},   {{55.2, 8.7}, {99.5, 98.6}, {176.4, 122.4}},
    {{56.8, 4.9}, {99.0, 17.6}, {148.4, 18.8}},   {{58.0, 8.7}, {101.5, 35.2}, {156.4, 37.5}},
    {{60.4, 8.7}, {106.5, 70.4}, {172.4, 75.1}},  {{65.2, 8.7}, {116.5, 98.6}, {204.4, 122.4}}};
// NVLS tree, Simple only, ranks per node 4 and 8: [node index][ppn == 8]
constexpr LatBw kArNvlsTree[5][2] = {{{53.0, 160.0}, {53.0, 266.7}},
                                     {{81.0, 80.0}, {81.0, 160.0}},
                                     {{109.0, 80.0}, {109.0, 160.0}},
                                     {{137.0, 80.0}, {137.0, 160.0}},
                                     {{165.0, 80.0}, {165.0, 160.0}}};

inline double pymin(double a, double b) { return b < a ? b : a; }
inline double pymax(double a, double b) { return b > a ? b : a; }

int log2i(int64_t n) {
  int k = 0;
  if (n <= 0) return 0;
  while (n >>= 1) ++k;
  return k;
}

int node_index(int n_nodes) {
  switch (n_nodes) {
    case 2: return 0;
    case 4: return 1;
    case 8: return 2;
    case 16: return 3;
    case 32: return 4;
  }
  return -1;
}
int ppn_index(int ppn) {
  switch (ppn) {
    case 1: return 0;
    case 2: return 1;
    case 4: return 2;
    case 8: return 3;
  }
  return -1;
}

template <int N>
double interp_clamped(const Point (&pts)[N], int x) {  // :980-992
  if (x <= pts[0].x) return pts[0].y;
  if (x >= pts[N - 1].x) return pts[N - 1].y;
  for (int i = 0; i + 1 < N; ++i) {
    if (x <= pts[i + 1].x) {
      double t = (double)(x - pts[i].x) / (double)(pts[i + 1].x - pts[i].x);
      return pts[i].y + t * (pts[i + 1].y - pts[i].y);
    }
  }
  return pts[N - 1].y;
}

struct Topo {
  int n_ranks, n_nodes, ppn, nch;
  double bw_intra, bw_inter;
};

// _compute_algo_bw (:323-465)
double algo_bw(int func, int algo, int proto, const Topo& t, const apc_nccl_config& c) {
  const int nsteps = func == kAR ? 2 * (t.n_ranks - 1) : t.n_ranks - 1;
  const int nb = t.n_nodes <= 1 ? 0 : (t.n_nodes <= 2 ? 1 : 2);
  const int nch = t.nch, ppn = t.ppn, arch = c.arch;
  const bool agrs = func == kAG || func == kRS;
  if (proto != kSimple && algo != kRing && algo != kTree) return 0.0;
  const double inter_agg =
      (c.has_nvswitch && t.n_nodes > 1) ? pymin(t.bw_intra, t.bw_inter * (double)ppn) : t.bw_inter;
  const double link = t.n_nodes <= 2 ? t.bw_intra : inter_agg;
  double bus;
  if (algo == kRing) {
    bus = (double)nch * link;
  } else if (algo == kTree) {
    if (func != kAR) return 0.0;
    bus = (double)nch * link;
  } else if (algo == kNvls) {
    if (nch < 2) return 0.0;
    if (agrs && t.n_nodes > 1 && !c.has_collnet) return 0.0;
    double intra = t.bw_intra * kNvlsEff[arch] * (double)(nch - 1) / (double)nch;
    if (func == kAR)
      intra *= 2.0;
    else
      intra *= (double)(ppn - 1) / (double)ppn;
    bus = (double)nch * (t.n_nodes > 1 ? pymin(intra, t.bw_inter) : intra);
  } else if (algo == kNvlsTree) {
    if (func != kAR) return 0.0;
    if (nch < 2) return 0.0;
    double intra = t.bw_intra * kNvlsEff[arch] * (double)(nch - 1) / (double)nch;
    intra *= 2.0;
    double inter = inter_agg * (double)(t.n_nodes <= 2 ? 2 : 1);
    bus = (double)nch * pymin(pymin(intra, inter), kMaxNvlsTreeBw[arch][nb]);
  } else if (algo == kCollnetDirect) {
    if (agrs) return (double)ppn * pymin(t.bw_intra * (double)nch, t.bw_inter * (double)nch * 0.9);
    bus = (double)nch * link;
    double factor = (double)ppn / (double)nch;
    factor -= (factor - 1.0) / 2.0;
    bus /= factor;
    if (arch == kHopper || arch == kBlackwell) bus *= 0.85;
  } else if (algo == kCollnetChain) {
    if (func != kAR) return 0.0;
    bus = (double)nch * link;
  } else {
    return 0.0;
  }
  const double ll_max = kLLMaxBw[arch][nb];
  if (algo == kRing && proto == kLL) bus = pymin(ll_max, bus * 0.5);
  if (algo == kRing && proto == kLL128) bus = pymin(bus * 0.92, (double)nch * kMaxRingLL128Bw[arch][nb]);
  if (algo == kTree && func == kAR) bus = pymin(bus * 0.92, (double)nch * kMaxTreeBw[arch][nb]);
  if (algo == kTree && proto == kLL) bus = pymin(bus / 3.8, ll_max);
  if (algo == kTree && proto == kLL128)
    bus = pymin(bus * (t.n_nodes == 1 ? 7.0 / 9.0 : 120.0 / 128.0), (double)nch * kMaxTreeLL128Bw[arch][nb]);
  if (algo == kRing || !agrs) {
    if (algo == kRing || algo == kNvls || algo == kNvlsTree)
      bus *= (double)t.n_ranks / (double)nsteps;
    else
      bus *= 0.5;
  }
  return bus;
}

double inter_latency(int algo, int proto, const Topo& t, const apc_nccl_config& c) {
  double inter = kHwLatNet[t.ppn == 1 ? kTree : algo][proto] + c.net_latency;
  if (proto == kSimple) inter += c.net_latency;
  return inter;
}

// ring latency for `nsteps` steps of which `n_inter` cross nodes (:505-521, :1295-1311)
double ring_steps_latency(int proto, int nsteps, int n_inter, const Topo& t, const apc_nccl_config& c) {
  double overhead = 0.0;
  if (t.n_nodes > 1) {
    overhead = kNetOverhead;
    if (proto == kSimple) overhead *= 3.0;
  }
  const double intra = pymax(kHwLatNvlink[kRing][proto], overhead);
  const double inter = inter_latency(kRing, proto, t, c);
  return kBaseLat[kRing][proto] + (double)(nsteps - n_inter) * intra + (double)n_inter * inter;
}

// _compute_algo_latency (:473-551)
double algo_latency(int func, int algo, int proto, const Topo& t, const apc_nccl_config& c) {
  const double base = kBaseLat[algo][proto];
  const double intra = kHwLatNvlink[algo][proto];
  const double inter = inter_latency(algo, proto, t, c);
  const int nsteps = func == kAR ? 2 * (t.n_ranks - 1) : t.n_ranks - 1;
  switch (algo) {
    case kRing: {
      const int n_inter = t.n_nodes == 1 ? 0 : (func == kAR ? 2 * (t.n_nodes - 1) : t.n_nodes - 1);
      double lat = ring_steps_latency(proto, nsteps, n_inter, t, c);
      if (t.n_nodes > 1) {
        double sync = kRingSyncPerNode * (double)t.n_nodes;
        if (t.n_nodes > 4) sync *= pow((double)t.n_nodes / 4.0, 0.65);
        lat += sync;
      }
      return lat;
    }
    case kTree:
      return base + 2.0 * ((double)(t.n_ranks / t.n_nodes - 1) * intra + (double)log2i(t.n_nodes) * inter);
    case kCollnetDirect:
      return base + 2.0 * ((double)(t.ppn - 1 < 1 ? t.ppn - 1 : 1) * intra + (double)(t.ppn - 1) * 0.4) + inter;
    case kCollnetChain:
      return base + (double)(2 * (t.ppn - 1)) * intra + inter;
    case kNvls:
      return intra + (t.n_nodes > 1 ? inter : 0.0);
    case kNvlsTree:
      return base + intra + (double)(2 * log2i(t.n_nodes)) * inter;
  }
  return 0.0;
}

void push(apc_nccl_dim& d, int slot, double lat, double bw, int flags, int proto) {
  if (!(bw > 0.0)) return;  // disabled candidate: costs +inf, never the minimum
  apc_nccl_cand& k = d.cand[slot][d.n_cand[slot]++];
  k.lat = lat;
  k.bw = bw;
  k.flags = flags;
  k.proto = proto;
}

// one candidate of the algorithm loop (_nccl_algo_time, :559-613)
void push_algo(apc_nccl_dim& d, int func, int algo, int proto, const Topo& t, const apc_nccl_config& c) {
  int flags = 0;
  if (algo == kTree && func == kAR) flags |= APC_NC_TREE_CORR;
  if (algo == kNvlsTree && func == kAR && c.arch == kBlackwell) flags |= APC_NC_TREE_CORR24;
  if (algo == kRing && t.n_nodes > 1) flags |= APC_NC_RING_CORR;
  if (algo == kRing && proto == kSimple && t.n_nodes > 1 && func == kAR) flags |= APC_NC_PLATEAU;
  push(d, kAbiSlot[func], algo_latency(func, algo, proto, t, c), algo_bw(func, algo, proto, t, c), flags, proto);
}

// nccl_collective_time (:1163-1212) with _table_collective_time (:1081-1160)
void plan_collective(apc_nccl_dim& d, int func, const Topo& t, const apc_nccl_config& c) {
  const int slot = kAbiSlot[func];
  const bool sw = (c.arch == kHopper || c.arch == kBlackwell) && c.has_nvswitch;
  if (sw && t.n_nodes == 1) {
    double bw = interp_clamped(kSwitchBw[func], t.n_ranks);
    if (c.arch == kBlackwell) bw *= kBlackwellScale;
    push(d, slot, interp_clamped(kSwitchLat[func], t.n_ranks), bw, 0, kSimple);
    return;
  }
  if (sw && t.n_nodes > 1) {
    const int ni = node_index(t.n_nodes), pi = ppn_index(t.ppn);
    const double scale = c.arch == kBlackwell ? kBlackwellScale : 1.0;
    if (ni >= 0 && pi >= 0) {  // every (nodes, ppn) row exists for ring and tree
      const int row = ni * 4 + pi;
      if (func != kAR) {
        const int fm = t.ppn == c.gpus_per_node ? APC_NC_FULL_MESH_RAMP : 0;
        for (int p = 0; p < 3; ++p) push(d, slot, kAgRsRing[row][p].lat, kAgRsRing[row][p].bw * scale, fm, p);
        return;
      }
      for (int p = 0; p < 3; ++p)
        push(d, slot, kArTree[row][p].lat, kArTree[row][p].bw * scale, APC_NC_TREE_CORR, p);
      if (t.ppn >= 4) {
        const LatBw& nv = kArNvlsTree[ni][t.ppn == 8];
        push(d, slot, nv.lat, nv.bw * scale, APC_NC_NVLS_RAMP, kSimple);
      }
      for (int p = 0; p < 3; ++p) push_algo(d, func, kRing, p, t, c);
      return;
    }
  }
  // _eligible_algos / _eligible_protos (:616-649)
  const bool nvls_ok = c.has_nvswitch && (c.arch == kHopper || c.arch == kBlackwell);
  int algos[6], na = 0;
  algos[na++] = kRing;
  if (func != kAR) {
    if (nvls_ok) algos[na++] = kNvls;
    if (c.has_collnet) algos[na++] = kCollnetDirect;
  } else {
    algos[na++] = kTree;
    if (c.has_collnet) {
      algos[na++] = kCollnetDirect;
      algos[na++] = kCollnetChain;
    }
    if (nvls_ok) {
      algos[na++] = kNvls;
      if (t.n_nodes > 1) algos[na++] = kNvlsTree;
    }
  }
  for (int a = 0; a < na; ++a) {
    if (algos[a] == kRing || algos[a] == kTree) {
      for (int p = 0; p < 3; ++p) push_algo(d, func, algos[a], p, t, c);
    } else {
      push_algo(d, func, algos[a], kSimple, t, c);
    }
  }
}

// nccl_all_to_all_cost (:1215-1313)
void plan_all_to_all(apc_nccl_dim& d, const Topo& t, const apc_nccl_config& c) {
  const int slot = 1;
  const bool hopper = c.arch == kHopper || c.arch == kBlackwell;
  if (hopper && c.has_nvswitch && t.n_nodes == 1) {
    push(d, slot, kA2aCeLat, c.arch == kHopper ? 380.0 : 675.0, 0, kSimple);
    return;
  }
  if (t.n_nodes > 1 && c.has_nvswitch) {
    d.a2a_remote = (double)(t.n_ranks - t.ppn) / (double)t.n_ranks;
    d.a2a_log_nodes = log2i(t.n_nodes);
    const double nic = c.bw_inter * (1.0 - kA2aNicOverhead / (double)t.n_nodes);
    push(d, slot, interp_clamped(kA2aNodeLat, t.n_nodes), nic, APC_NC_NIC, kSimple);
    return;
  }
  const double bw = t.n_nodes <= 2 ? t.bw_intra : t.bw_inter;
  const double bus = (double)t.nch * bw * kA2aSmCorr;
  const int n_inter = t.n_nodes == 1 ? 0 : t.n_nodes - 1;
  push(d, slot, ring_steps_latency(kSimple, t.n_ranks, n_inter, t, c), bus, 0, kSimple);
}

bool config_ok(const apc_nccl_config* cfg, const char* who) {
  if (cfg && cfg->arch >= 0 && cfg->arch <= 2 && cfg->gpus_per_node >= 1 && cfg->num_channels >= 0) return true;
  char msg[160];
  snprintf(msg, sizeof(msg), "%s: config must have arch 0..2, gpus_per_node >= 1, num_channels >= 0", who);
  apc_internal_set_error(msg);
  return false;
}

void init_plan(apc_nccl_plan* plan, int ndim) {
  memset(plan, 0, sizeof(*plan));
  plan->ndim = ndim;
  memcpy(plan->tree_corr, kTreeCorr, sizeof(kTreeCorr));
  memcpy(plan->nvls_tree_ramp, kNvlsTreeRamp, sizeof(kNvlsTreeRamp));
  memcpy(plan->full_mesh_ramp, kFullMeshRamp, sizeof(kFullMeshRamp));
  memcpy(plan->a2a_nic_ramp, kA2aNicRamp, sizeof(kA2aNicRamp));
}

// candidates and tables of one communicator
void plan_dim(apc_nccl_dim& d, const Topo& t, const apc_nccl_config& cfg) {
  d.n_ranks = t.n_ranks;
  d.n_nodes = t.n_nodes;
  d.ppn = t.ppn;
  d.n_channels = t.nch;
  d.bw_intra = t.bw_intra;
  d.bw_inter = t.bw_inter;
  // ring correction table of this communicator (:596-599, :700-719)
  const double e = 1.0 + 0.2 * (double)(log2i(t.n_nodes) - 2);
  for (int k = 0; k < APC_NCCL_TABLE_LEN; ++k) {
    double corr = kRingCorr[k];
    if (t.n_nodes > 4) {
      if (corr < 1.0) corr = pow(corr, e);
      if (k > 0) corr = pymin(corr, 2.0 * d.ring_corr[k - 1]);
    }
    d.ring_corr[k] = corr;
  }
  // One rank means zero ring steps: the reference's algorithm loop divides by
  // them (ZeroDivisionError); only its measured-point paths are defined there.
  // Undefined combinations keep zero candidates (cost +inf).
  const bool measured = (cfg.arch == kHopper || cfg.arch == kBlackwell) && cfg.has_nvswitch && t.n_nodes == 1;
  if (t.n_ranks >= 2 || measured)
    for (int f = 0; f < 3; ++f) plan_collective(d, f, t, cfg);
  plan_all_to_all(d, t, cfg);
}

}  // namespace

extern "C" int apc_nccl_plan_build(const apc_nccl_config* cfg, const int32_t* mesh_shape, int32_t ndim,
                                   apc_nccl_plan* plan) {
  if (!mesh_shape || !plan || ndim < 1 || ndim > APC_MAX_MESH_DIMS) {
    apc_internal_set_error("apc_nccl_plan_build: null argument or mesh rank outside 1..4");
    return APC_ERR_INVALID;
  }
  if (!config_ok(cfg, "apc_nccl_plan_build")) return APC_ERR_INVALID;
  init_plan(plan, ndim);
  for (int i = 0; i < ndim; ++i) {
    if (mesh_shape[i] < 1) {
      apc_internal_set_error("apc_nccl_plan_build: mesh dim size < 1");
      return APC_ERR_INVALID;
    }
    // derive_mesh_dim_topo (:1001-1021)
    int64_t inner = 1;
    for (int j = i + 1; j < ndim; ++j) inner *= mesh_shape[j];
    Topo t;
    t.n_ranks = mesh_shape[i];
    int64_t q = cfg->gpus_per_node / inner;
    if (q > t.n_ranks) q = t.n_ranks;
    t.ppn = q < 1 ? 1 : (int)q;
    t.n_nodes = t.n_ranks / t.ppn;
    t.nch = cfg->num_channels > 0 ? cfg->num_channels : kDefaultChannels[cfg->arch];
    t.bw_intra = cfg->bw_intra / (double)t.nch;
    t.bw_inter = cfg->bw_inter / (double)t.nch;
    plan_dim(plan->dim[i], t, *cfg);
  }
  return 0;
}

extern "C" int apc_nccl_plan_for_topo(const apc_nccl_config* cfg, int32_t n_ranks, int32_t n_nodes, int32_t ppn,
                                      int32_t n_channels, double bw_intra, double bw_inter,
                                      apc_nccl_plan* plan) {
  if (!plan || n_ranks < 1 || n_nodes < 1 || ppn < 1 || n_channels < 1) {
    apc_internal_set_error("apc_nccl_plan_for_topo: null plan or non-positive topology field");
    return APC_ERR_INVALID;
  }
  if (!config_ok(cfg, "apc_nccl_plan_for_topo")) return APC_ERR_INVALID;
  init_plan(plan, 1);
  Topo t;
  t.n_ranks = n_ranks;
  t.n_nodes = n_nodes;
  t.ppn = ppn;
  t.nch = n_channels;
  t.bw_intra = bw_intra;
  t.bw_inter = bw_inter;
  plan_dim(plan->dim[0], t, *cfg);
  return 0;
}
