// Passes over the resident results and the batch forms of the scalar cost-model
// functions (gfx950), and their C ABI: prefetch discount, objective
// coefficients, node hashes, the decision-variable twin, a plan's terms,
// placement enumeration, local shapes, collective and read/write times.
#include "apc_device.h"

namespace {

// ---------------------------------------------------------------------------
// Kernels: post-passes over the entry arrays (one entry per lane)
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock)
prefetch_discount_kernel(apc_problem p, const double* __restrict__ per_arg, double scale,
                         double* __restrict__ comm, double* __restrict__ cost,
                         const uint8_t* __restrict__ flags, unsigned long long* n_modified) {
  const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  unsigned int mine = 0;
  if (idx < p.n_slot) {
    const apc_edge ed = find_edge(p, idx);
    const int64_t local = idx - ed.off;
    if (local < (int64_t)ed.ssrc * ed.sdst && (ed.flags & APC_EDGE_PREFETCHABLE) &&
        ed.src_node >= 0) {
      double c = comm[idx];
      if (c > 0.0 && isfinite(c)) {
        const uint32_t o = (uint32_t)local / (uint32_t)ed.ssrc;
        c = c * scale;
        comm[idx] = c;
        cost[idx] = (c + per_arg[ed.comp_base + o]) + (double)(flags[idx] & APC_ENTRY_TRANSITION);
        mine = 1;
      }
    }
  }
  // wavefront reduction, one atomic per wave
  for (int off = 32; off > 0; off >>= 1) mine += __shfl_down(mine, off, 64);
  if ((threadIdx.x & 63) == 0 && mine) atomicAdd(n_modified, (unsigned long long)mine);
}

__global__ void __launch_bounds__(kBlock)
objective_kernel(apc_problem p, const double* __restrict__ cost, double* __restrict__ obj) {
  const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= p.n_slot) return;
  const apc_edge ed = find_edge(p, idx);
  if (idx - ed.off < (int64_t)ed.ssrc * ed.sdst)
    obj[idx] = cost[idx] * (double)p.node_multiplier[ed.node];
}

// ---------------------------------------------------------------------------
// Kernel: structural hash of every node, the key under which repeated layers
// are clustered.  It covers what the reference's node key covers
// (graph_passes/graph_clustering.py:68-82: the op, the forward/backward tag, the
// node's own strategies and its producers' strategies), read from the packed
// arrays: op class, program, strategy counts, output/input/producer spec runs,
// default rows.  H = mix(sum over (section, position) of mix(word ^ salt)): a
// position-salted sum, so the lanes of a wavefront hash disjoint positions and
// add.
// ---------------------------------------------------------------------------
__host__ __device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ uint64_t hash_term(uint64_t section, uint64_t pos, uint64_t w) {
  return mix64(w ^ mix64((section << 40) + pos + 0x9E3779B97F4A7C15ull));
}

__global__ void __launch_bounds__(kBlock)
node_hash_kernel(apc_problem p, const int64_t* __restrict__ node_out_list,
                 const int32_t* __restrict__ node_phase, uint64_t* __restrict__ out) {
  const int v = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (v >= p.n_node) return;  // wave-uniform
  const int lane = threadIdx.x & 63;
  const int S = p.node_nstrat[v];
  const int e0 = p.node_edge_off[v], e1 = p.node_edge_off[v + 1];
  const int op = p.node_op[v];
  uint64_t acc = 0;
  if (lane == 0) {
    acc += hash_term(0, 0, (uint64_t)op);
    acc += hash_term(0, 1, (uint64_t)p.node_nargs[v]);
    acc += hash_term(0, 2, (uint64_t)S);
    acc += hash_term(0, 3, (uint64_t)(node_phase ? node_phase[v] : 0));
    acc += hash_term(0, 4, (uint64_t)(e1 - e0));
  }
  const int plen = p.node_prog_len[v];
  for (int i = lane; i < plen; i += 64) acc += hash_term(1, i, (uint64_t)p.prog[p.node_prog_off[v] + i]);
  for (int k = lane; k < S; k += 64) acc += hash_term(2, k, p.lists[(size_t)node_out_list[v] + k]);
  if (op == APC_OP_EXPLICIT) {
    const int64_t b = p.node_comp_off[v];
    for (int k = lane; k < S; k += 64) {
      acc += hash_term(3, k, (uint64_t)p.explicit_flops[b + k]);
      acc += hash_term(4, k, (uint64_t)p.explicit_bytes[b + k]);
    }
  }
  for (int e = e0; e < e1; ++e) {
    const apc_edge ed = p.edges[e];
    const uint64_t sec = 16 + 4 * (uint64_t)(e - e0);
    if (lane == 0) {
      acc += hash_term(sec, 0, (uint64_t)ed.ssrc);
      acc += hash_term(sec, 1, (uint64_t)ed.sdst);
      acc += hash_term(sec, 2, (uint64_t)(ed.flags & (APC_EDGE_HAS_PRODUCER | APC_EDGE_SCORE_TRANSITION)));
      acc += hash_term(sec, 3, (uint64_t)(ed.default_off >= 0));
    }
    for (int k = lane; k < ed.sdst; k += 64) acc += hash_term(sec + 1, k, p.lists[(size_t)ed.dst_list + k]);
    if (ed.src_node >= 0)
      for (int j = lane; j < ed.ssrc; j += 64) acc += hash_term(sec + 2, j, p.lists[(size_t)ed.src_list + j]);
    if (ed.default_off >= 0) {
      const int64_t n = (int64_t)ed.ssrc * ed.sdst;
      for (int64_t i = lane; i < n; i += 64)
        acc += hash_term(sec + 3, (uint64_t)i, (uint64_t)__double_as_longlong(p.default_vals[ed.default_off + i]));
    }
  }
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor((unsigned long long)acc, off);
  if (lane == 0) out[v] = mix64(acc);
}

// Entry arrays without their padding: slot -> decision variable.  Blocks start on
// multiples of 16 slots, variables are numbered through the real entries only;
// var_start[e] is the first variable of edge e's block.  One lane per slot, so the
// reads are coalesced and the writes are the same stream shifted by the padding
// before them.
__global__ void __launch_bounds__(kBlock)
compact_kernel(apc_problem p, const int64_t* __restrict__ var_start, const double* __restrict__ comm,
               const double* __restrict__ cost, const uint8_t* __restrict__ flags,
               double* __restrict__ out_comm, double* __restrict__ out_cost,
               uint8_t* __restrict__ out_flags) {
  const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= p.n_slot) return;
  const int e = p.chunk_edge[idx >> APC_CHUNK_SHIFT];
  const apc_edge* ed = p.edges + e;
  const int64_t local = idx - ed->off;
  if (local >= (int64_t)ed->ssrc * ed->sdst) return;
  const int64_t v = var_start[e] + local;
  out_comm[v] = comm[idx];
  out_cost[v] = cost[idx];
  out_flags[v] = flags[idx];
}

// ---------------------------------------------------------------------------
// Kernel: packed twin of the decision variables, in the reference's insertion
// order (node, out_idx, argi, inp_idx): row of entry (e, o, j) is
// row_base[e] + o * row_stride[e] + j, where row_stride is the node's sum of
// S_src over its arguments.  One lane per slot; the lanes of a run of inp_idx
// write consecutive rows.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock)
export_kernel(apc_problem p, const double* __restrict__ per_arg, const double* __restrict__ comm,
              const uint8_t* __restrict__ flags, const int64_t* __restrict__ row_base,
              const int32_t* __restrict__ row_stride, int32_t* __restrict__ keys,
              double* __restrict__ vals) {
  const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= p.n_slot) return;
  const int e = p.chunk_edge[idx >> APC_CHUNK_SHIFT];
  const apc_edge ed = p.edges[e];
  const int64_t local = idx - ed.off;
  if (local >= (int64_t)ed.ssrc * ed.sdst) return;
  const uint32_t o = (uint32_t)local / (uint32_t)ed.ssrc;
  const uint32_t j = (uint32_t)local - o * (uint32_t)ed.ssrc;
  const int64_t row = row_base[e] + (int64_t)o * row_stride[e] + j;
  int4 k;
  k.x = ed.node;
  k.y = e - p.node_edge_off[ed.node];
  k.z = (int)o;
  k.w = (int)j;
  *reinterpret_cast<int4*>(keys + row * 4) = k;
  double* v = vals + row * 3;
  v[0] = per_arg[ed.comp_base + o];
  v[1] = comm[idx];
  v[2] = (double)(flags[idx] & APC_ENTRY_TRANSITION);
}

// The selected entry of every edge under one assignment (out_idx per node):
// terms[e] = (per-arg compute, comm, transition, cost) of entry
// (e, assign[node], assign[producer] or 0) and slot[e] = its slot.
__global__ void __launch_bounds__(kBlock)
solution_terms_kernel(apc_problem p, const double* __restrict__ per_arg,
                      const double* __restrict__ comm, const double* __restrict__ cost,
                      const uint8_t* __restrict__ flags, const uint16_t* __restrict__ assign,
                      double* __restrict__ terms, int64_t* __restrict__ slot) {
  const int e = blockIdx.x * kBlock + threadIdx.x;
  if (e >= p.n_edge) return;
  const apc_edge ed = p.edges[e];
  const uint32_t o = assign[ed.node];
  const uint32_t j = ed.src_node >= 0 ? assign[ed.src_node] : 0u;
  double* t = terms + (size_t)e * 4;
  if (o >= (uint32_t)ed.sdst || j >= (uint32_t)ed.ssrc) {  // not a strategy index of this edge
    t[0] = t[1] = t[2] = t[3] = NAN;
    slot[e] = -1;
    return;
  }
  const int64_t idx = ed.off + (int64_t)o * ed.ssrc + j;
  t[0] = per_arg[ed.comp_base + o];
  t[1] = comm[idx];
  t[2] = (double)(flags[idx] & APC_ENTRY_TRANSITION);
  t[3] = cost[idx];
  slot[e] = idx;
}

// ---------------------------------------------------------------------------
// Kernel: input/parameter placement options
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock)
enumerate_kernel(apc_model m, int32_t n, const int32_t* __restrict__ rank,
                 const int64_t* __restrict__ shape, const int64_t* __restrict__ cand_off,
                 uint8_t* __restrict__ valid, uint8_t* __restrict__ plc) {
  const int64_t total = cand_off[n];
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    int lo = 0, hi = n;
    while (hi - lo > 1) {
      int mid = (lo + hi) >> 1;
      if (cand_off[mid] <= idx) lo = mid; else hi = mid;
    }
    const int t = lo;
    const int r = rank[t];
    int64_t c = idx - cand_off[t];
    // itertools.product order: the last mesh dim varies fastest
    int code[APC_MAX_MESH_DIMS] = {0, 0, 0, 0};
    for (int i = m.ndim - 1; i >= 0; --i) {
      const int opt = (int)(c % (r + 1));
      c /= (r + 1);
      code[i] = opt == 0 ? 0 : (kShard | (opt - 1));
    }
    int64_t sh[APC_MAX_RANK];
    for (int d = 0; d < APC_MAX_RANK; ++d) sh[d] = shape[(size_t)t * APC_MAX_RANK + d];
    bool ok = true;
    for (int i = 0; i < m.ndim && ok; ++i) {
      if ((code[i] & kKindMask) == kShard) {
        const int d = code[i] & kArgMask;
        const int64_t ms = m.mesh_shape[i];
        // dynamic index kept in a loop so sh[] stays in registers
        for (int dd = 0; dd < APC_MAX_RANK; ++dd) {
          if (dd == d) {
            if (sh[dd] >= ms) sh[dd] = (sh[dd] + ms - 1) / ms; else ok = false;
          }
        }
      }
    }
    valid[idx] = ok ? 1 : 0;
    for (int i = 0; i < APC_MAX_MESH_DIMS; ++i) plc[idx * APC_MAX_MESH_DIMS + i] = (uint8_t)code[i];
  }
}

// ---------------------------------------------------------------------------
// Kernel: validity filter and de-duplication of operator strategies.  A set is the
// candidate strategies of one node, a row of spec words per strategy (its input
// specs, then its output specs; APC_SPEC_NONE where there is none).  A row is
// valid when every spec passes the rule of enumerate_kernel: walking the mesh dims
// in order, a Shard(d) needs the (already divided) size of dim d to be at least
// the mesh size and divides it, rounding up.  Among the valid rows of a set, one
// that repeats the words of an earlier valid row is dropped.  One workgroup per
// set: a lane per row for the rule and a 64-bit hash of the row (LDS), then a
// lane per row against the rows before it, hashes first.
// ---------------------------------------------------------------------------
constexpr int kFilterRows = 4096;  // rows of a set whose hashes fit the workgroup's LDS

__device__ __forceinline__ uint64_t mix_word(uint64_t h, uint32_t w, int pos) {
  uint64_t z = h ^ (((uint64_t)w << 8) + (uint64_t)(pos + 1)) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__global__ void __launch_bounds__(kBlock)
filter_strategies_kernel(apc_model m, const int32_t* __restrict__ meta_rank, const int64_t* __restrict__ meta_shape,
                         const uint8_t* __restrict__ tuple_plc, const int64_t* __restrict__ set_row,
                         const int32_t* __restrict__ set_width, const int64_t* __restrict__ set_word,
                         const uint32_t* __restrict__ words, uint8_t* __restrict__ valid,
                         uint8_t* __restrict__ keep) {
  __shared__ uint64_t s_hash[kFilterRows];
  __shared__ uint8_t s_valid[kFilterRows];
  const int set = blockIdx.x;
  const int64_t row0 = set_row[set];
  const int n_rows = (int)(set_row[set + 1] - row0);
  const int width = set_width[set];
  const uint32_t* __restrict__ w0 = words + set_word[set];
  for (int r = threadIdx.x; r < n_rows; r += kBlock) {
    const uint32_t* __restrict__ row = w0 + (size_t)r * width;
    bool ok = true;
    uint64_t h = 0x243F6A8885A308D3ull;
    for (int c = 0; c < width; ++c) {
      const uint32_t w = row[c];
      h = mix_word(h, w, c);
      if (w == APC_SPEC_NONE) continue;
      const uint32_t mid = w >> APC_TUPLE_BITS;
      const uint32_t plc = load_tuple(tuple_plc, w & kTupleMask);
      const int rank = meta_rank[mid];
      int64_t sh[APC_MAX_RANK];
#pragma unroll
      for (int d = 0; d < APC_MAX_RANK; ++d) sh[d] = meta_shape[(size_t)mid * APC_MAX_RANK + d];
      for (int i = 0; i < m.ndim; ++i) {
        const int code = (plc >> (8 * i)) & 0xFF;
        if ((code & kKindMask) != kShard) continue;
        const int d = code & kArgMask;
        const int64_t ms = m.mesh_shape[i];
        if (d >= rank) { ok = false; continue; }  // a dim the tensor does not have (the packer refuses such a spec)
#pragma unroll
        for (int dd = 0; dd < APC_MAX_RANK; ++dd) {  // dynamic index kept in a loop so sh[] stays in registers
          if (dd == d) {
            if (sh[dd] >= ms) sh[dd] = (sh[dd] + ms - 1) / ms; else ok = false;
          }
        }
      }
    }
    s_hash[r] = h;
    s_valid[r] = ok ? 1 : 0;
    valid[row0 + r] = ok ? 1 : 0;
  }
  __syncthreads();
  for (int r = threadIdx.x; r < n_rows; r += kBlock) {
    bool kept = s_valid[r] != 0;
    if (kept) {
      const uint64_t h = s_hash[r];
      const uint32_t* __restrict__ row = w0 + (size_t)r * width;
      for (int q = 0; q < r; ++q) {
        if (!s_valid[q] || s_hash[q] != h) continue;
        const uint32_t* __restrict__ other = w0 + (size_t)q * width;
        bool same = true;
        for (int c = 0; c < width && same; ++c) same = row[c] == other[c];
        if (same) { kept = false; break; }
      }
    }
    keep[row0 + r] = kept ? 1 : 0;
  }
}

// ---------------------------------------------------------------------------
// Kernels: scalar cost-model functions in batch form
// ---------------------------------------------------------------------------
// _get_sharded_shape_stride (compute_estimation.py:300-318), including its
// stride rule: the stride of dim d-1 is divided only when d-1 > 0.
__global__ void __launch_bounds__(kBlock)
local_shape_kernel(apc_model m, int32_t n, const int32_t* __restrict__ rank,
                   const int64_t* __restrict__ shape, const int64_t* __restrict__ stride,
                   const uint8_t* __restrict__ plc, int64_t* __restrict__ out_shape,
                   int64_t* __restrict__ out_stride) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  const int r = rank[t];
  for (int d = 0; d < APC_MAX_RANK; ++d) {
    out_shape[(size_t)t * APC_MAX_RANK + d] = shape[(size_t)t * APC_MAX_RANK + d];
    out_stride[(size_t)t * APC_MAX_RANK + d] = stride[(size_t)t * APC_MAX_RANK + d];
  }
  for (int i = 0; i < m.ndim; ++i) {
    const int c = plc[(size_t)t * APC_MAX_MESH_DIMS + i];
    if ((c & kKindMask) != kShard) continue;
    const int d = c & kArgMask;
    if (d >= r) continue;
    const int64_t ms = m.mesh_shape[i];
    int64_t* s = out_shape + (size_t)t * APC_MAX_RANK;
    int64_t* st = out_stride + (size_t)t * APC_MAX_RANK;
    s[d] = (s[d] + ms - 1) / ms;
    if (d - 1 > 0) st[d - 1] = (st[d - 1] + ms - 1) / ms;
  }
}

// collective_comm_cost, default model (collective_runtime_estimation.py:65-97):
// kind 0 allgather, 1 all_to_all, 2 allreduce, 3 reduce_scatter, else 0.0
__global__ void __launch_bounds__(kBlock)
collective_kernel(apc_model m, int32_t n, const int32_t* __restrict__ kind,
                  const int64_t* __restrict__ nbytes, const int32_t* __restrict__ dim,
                  double* __restrict__ out) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  const int k = kind[t], d = dim[t];
  out[t] = (k >= 0 && k <= 3 && d >= 0 && d < m.ndim) ? collective_cost(k, nbytes[t], d, m) : 0.0;
}

// compute_read_write_time (compute_estimation.py:391-403)
__global__ void __launch_bounds__(kBlock)
rw_time_kernel(apc_model m, int32_t n, const double* __restrict__ nbytes, double* __restrict__ out) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) out[t] = rw_time(nbytes[t], m.gmem_bw);
}

}  // namespace

extern "C" {

int apc_apply_prefetch_discount(const apc_problem* p, const double* per_arg, double scale,
                                double* comm, double* cost, const uint8_t* flags,
                                unsigned long long* n_modified, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_entry == 0) return 0;
  if (!per_arg || !comm || !cost || !flags || !n_modified)
    return fail(APC_ERR_INVALID, "apc_apply_prefetch_discount: null argument%s");
  unsigned grid;
  if (int rc = slot_grid(p, kBlock, &grid)) return rc;
  hipLaunchKernelGGL(prefetch_discount_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream,
                     *p, per_arg, scale, comm, cost, flags, n_modified);
  return check_launch("prefetch_discount_kernel");
}

int apc_objective_coeffs(const apc_problem* p, const double* cost, double* obj, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_entry == 0) return 0;
  if (!cost || !obj || !p->node_multiplier)
    return fail(APC_ERR_INVALID, "apc_objective_coeffs: null argument%s");
  unsigned grid;
  if (int rc = slot_grid(p, kBlock, &grid)) return rc;
  hipLaunchKernelGGL(objective_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *p, cost,
                     obj);
  return check_launch("objective_kernel");
}

int apc_node_hashes(const apc_problem* p, const int64_t* node_out_list, const int32_t* node_phase,
                    uint64_t* out, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_node == 0) return 0;
  if (!node_out_list || !out) return fail(APC_ERR_INVALID, "apc_node_hashes: null argument%s");
  hipLaunchKernelGGL(node_hash_kernel, dim3((p->n_node + (kBlock / 64) - 1) / (kBlock / 64)), dim3(kBlock),
                     0, (hipStream_t)stream, *p, node_out_list, node_phase, out);
  return check_launch("node_hash_kernel");
}

int apc_export_decision_vars(const apc_problem* p, const double* per_arg, const double* comm,
                             const uint8_t* flags, const int64_t* row_base,
                             const int32_t* row_stride, int32_t* keys, double* vals, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_slot == 0) return 0;
  if (!per_arg || !comm || !flags || !row_base || !row_stride || !keys || !vals)
    return fail(APC_ERR_INVALID, "apc_export_decision_vars: null argument%s");
  unsigned grid;
  if (int rc = slot_grid(p, kBlock, &grid)) return rc;
  hipLaunchKernelGGL(export_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *p, per_arg,
                     comm, flags, row_base, row_stride, keys, vals);
  return check_launch("export_kernel");
}

int apc_compact_entries(const apc_problem* p, const int64_t* var_start, const double* comm,
                        const double* cost, const uint8_t* flags, double* out_comm, double* out_cost,
                        uint8_t* out_flags, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_slot == 0) return 0;
  if (!var_start || !comm || !cost || !flags || !out_comm || !out_cost || !out_flags)
    return fail(APC_ERR_INVALID, "apc_compact_entries: null argument%s");
  unsigned grid;
  if (int rc = slot_grid(p, kBlock, &grid)) return rc;
  hipLaunchKernelGGL(compact_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *p, var_start,
                     comm, cost, flags, out_comm, out_cost, out_flags);
  return check_launch("compact_kernel");
}

int apc_solution_terms(const apc_problem* p, const double* per_arg, const double* comm,
                       const double* cost, const uint8_t* flags, const uint16_t* assign,
                       double* terms, int64_t* slot, void* stream) {
  if (int rc = validate_problem(p)) return rc;
  if (p->n_edge == 0) return 0;
  if (!per_arg || !comm || !cost || !flags || !assign || !terms || !slot)
    return fail(APC_ERR_INVALID, "apc_solution_terms: null argument%s");
  hipLaunchKernelGGL(solution_terms_kernel, dim3((p->n_edge + kBlock - 1) / kBlock), dim3(kBlock), 0,
                     (hipStream_t)stream, *p, per_arg, comm, cost, flags, assign, terms, slot);
  return check_launch("solution_terms_kernel");
}

int apc_local_shapes(const apc_model* model, int32_t n, const int32_t* rank, const int64_t* shape,
                     const int64_t* stride, const uint8_t* plc, int64_t* out_shape,
                     int64_t* out_stride, void* stream) {
  if (!model || model->ndim < 1 || model->ndim > APC_MAX_MESH_DIMS)
    return fail(APC_ERR_INVALID, "apc_local_shapes: bad model%s");
  if (n <= 0) return 0;
  if (!rank || !shape || !stride || !plc || !out_shape || !out_stride)
    return fail(APC_ERR_INVALID, "apc_local_shapes: null argument%s");
  hipLaunchKernelGGL(local_shape_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0,
                     (hipStream_t)stream, *model, n, rank, shape, stride, plc, out_shape, out_stride);
  return check_launch("local_shape_kernel");
}

int apc_collective_costs(const apc_model* model, int32_t n, const int32_t* kind,
                         const int64_t* nbytes, const int32_t* dim, double* out, void* stream) {
  if (!model || model->ndim < 1 || model->ndim > APC_MAX_MESH_DIMS)
    return fail(APC_ERR_INVALID, "apc_collective_costs: bad model%s");
  if (n <= 0) return 0;
  if (!kind || !nbytes || !dim || !out)
    return fail(APC_ERR_INVALID, "apc_collective_costs: null argument%s");
  hipLaunchKernelGGL(collective_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0,
                     (hipStream_t)stream, *model, n, kind, nbytes, dim, out);
  return check_launch("collective_kernel");
}

int apc_rw_times(const apc_model* model, int32_t n, const double* nbytes, double* out,
                 void* stream) {
  if (!model) return fail(APC_ERR_INVALID, "apc_rw_times: null model%s");
  if (n <= 0) return 0;
  if (!nbytes || !out) return fail(APC_ERR_INVALID, "apc_rw_times: null argument%s");
  hipLaunchKernelGGL(rw_time_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0,
                     (hipStream_t)stream, *model, n, nbytes, out);
  return check_launch("rw_time_kernel");
}

int apc_enumerate_input_options(const apc_model* model, int32_t n, const int32_t* rank,
                                const int64_t* shape, const int64_t* cand_off, uint8_t* valid,
                                uint8_t* plc, void* stream) {
  if (!model || model->ndim < 1 || model->ndim > APC_MAX_MESH_DIMS)
    return fail(APC_ERR_INVALID, "apc_enumerate_input_options: bad model%s");
  if (n <= 0) return 0;
  if (!rank || !shape || !cand_off || !valid || !plc)
    return fail(APC_ERR_INVALID, "apc_enumerate_input_options: null argument%s");
  hipLaunchKernelGGL(enumerate_kernel, dim3(grid_for((int64_t)n * 64, kBlock)), dim3(kBlock), 0,
                     (hipStream_t)stream, *model, n, rank, shape, cand_off, valid, plc);
  return check_launch("enumerate_kernel");
}

int apc_filter_strategies(const apc_model* model, int32_t n_meta, const int32_t* meta_rank,
                          const int64_t* meta_shape, int32_t n_tuple, const uint8_t* tuple_plc, int32_t n_set,
                          const int64_t* set_row, const int32_t* set_width, const int64_t* set_word,
                          const uint32_t* words, int32_t max_rows, uint8_t* valid, uint8_t* keep, void* stream) {
  if (!model || model->ndim < 1 || model->ndim > APC_MAX_MESH_DIMS)
    return fail(APC_ERR_INVALID, "apc_filter_strategies: bad model%s");
  if (n_set <= 0) return 0;
  if (n_meta <= 0 || n_tuple <= 0 || !meta_rank || !meta_shape || !tuple_plc || !set_row || !set_width || !set_word ||
      !words || !valid || !keep)
    return fail(APC_ERR_INVALID, "apc_filter_strategies: null argument%s");
  if (max_rows < 0 || max_rows > kFilterRows)
    return fail(APC_ERR_INVALID, "apc_filter_strategies: a set has more than 4096 rows%s");
  hipLaunchKernelGGL(filter_strategies_kernel, dim3((unsigned)n_set), dim3(kBlock), 0, (hipStream_t)stream, *model,
                     meta_rank, meta_shape, tuple_plc, set_row, set_width, set_word, words, valid, keep);
  return check_launch("filter_strategies_kernel");
}

}  // extern "C"
