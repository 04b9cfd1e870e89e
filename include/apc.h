/*
 * apc.h -- C ABI of the MI355X sharding-search cost engine (libapc_hip.so).
 *
 * The reference (meta-pytorch/autoparallel) is pure Python and has no FFI: each
 * entry point below replaces a Python function of the reference's cost path,
 * cited per declaration (paths relative to the reference tree, or "torch:" for
 * the installed torch it calls into).  All array arguments are DEVICE pointers
 * unless marked "host"; the caller owns every buffer; calls are asynchronous on
 * the given HIP stream (pass the raw hipStream_t, NULL = default stream).
 * Return value: 0 on success, negative on error (apc_last_error() gives text).
 * No entry point allocates device memory.
 */
#ifndef APC_H_
#define APC_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define APC_MAX_MESH_DIMS 4
#define APC_MAX_RANK 8
#define APC_TUPLE_BITS 12
#define APC_SPEC_NONE 0xFFFFFFFFu
#define APC_CHUNK_SHIFT 4    /* edge blocks start on multiples of 16 slots */
#define APC_ITEM_ENTRIES 256 /* entries of one edge per work item (one wavefront);
                                apc_problem.item_entries may double it */
#define APC_NUM_DTYPES 8

/* edge flags */
#define APC_EDGE_HAS_PRODUCER 1
#define APC_EDGE_SCORE_TRANSITION 2
#define APC_EDGE_PREFETCHABLE 4
/* the edge's matrix in the block table is stored by distinct spec word (see
 * apc_problem.list_uidx); its row length is flags >> APC_EDGE_USRC_SHIFT */
#define APC_EDGE_COMPRESSED 8
#define APC_EDGE_USRC_SHIFT 8

/* node op classes */
#define APC_OP_ZERO 0
#define APC_OP_PROGRAM 1
#define APC_OP_EXPLICIT 2

/* entry flag bits written by apc_edge_costs */
#define APC_ENTRY_TRANSITION 1 /* src placements != tgt placements        */
#define APC_ENTRY_NONFINITE 2  /* cost was inf: variable must be pinned 0  */

#define APC_ERR_INVALID (-1)
#define APC_ERR_LAUNCH (-2)
#define APC_ERR_UNSUPPORTED (-3)

/* One (consumer node, argument) pair: an S_dst x S_src block of entries,
 * row-major [out_idx][inp_idx], starting at slot `off` (a multiple of 16; the
 * slots between one block's end and the next block's start are padding that
 * no kernel reads or writes). */
typedef struct apc_edge {
  int64_t off;         /* slot of entry (out_idx 0, inp_idx 0)                 */
  int64_t default_off; /* into default_vals, or -1                             */
  uint32_t src_list;   /* into lists: S_src producer output spec words         */
  uint32_t dst_list;   /* into lists: S_dst consumer input spec words          */
  int32_t ssrc;
  int32_t sdst;
  int32_t comp_base; /* index of (node, out_idx 0) in the compute vector     */
  int32_t flags;
  int32_t node;
  int32_t src_node;  /* producer node or -1                                   */
  int64_t table_off; /* first element of the edge's matrix in the block table;
                        -1 for an edge without a producer (its matrix is its
                        rows of default_vals)                                   */
  uint32_t magic;    /* floor(2^32 / ssrc) + 1 if ssrc > 1 and ssrc * ssrc * sdst
                        < 2^32 (then local / ssrc == umulhi(local, magic)), else 0 */
  uint32_t local0;   /* 0 in the edge table; in a work item, its first entry
                        (modulo 2^32: see apc_problem.items)                 */
} apc_edge; /* 64 bytes */

/* Everything the node estimate reads about one evaluated node, in one record,
 * so that a workgroup starts with one load instead of a chain through the
 * node, edge-offset and edge arrays. */
#define APC_REC_ARGS 14
typedef struct apc_comp_rec {
  int32_t node;      /* the evaluated node                                    */
  int32_t nstrat;
  int32_t nargs;     /* len(input_specs): the divisor of per_arg              */
  int32_t op;        /* APC_OP_*                                              */
  int64_t comp_off;  /* slot of (node, out_idx 0) in the compute vector       */
  int64_t prog_off;  /* into prog, -1 if none                                 */
  int32_t prog_len;
  int32_t n_edge;    /* arguments with an edge                                */
  uint32_t dst_list[APC_REC_ARGS]; /* dst_list of the node's first edges      */
  int32_t term_off;  /* into prog_terms: the node's program as product terms  */
  int32_t n_term;    /* 0: none, the kernel interprets prog                   */
  int32_t term_flags; /* APC_TERMS_*                                          */
  /* the tensor meta behind argument a's specs (all strategies of a node see the
   * same tensor per argument), so that its rows are fetched together with the
   * spec words instead of after them; 0xFFFF: none or not uniform.  A hint: a
   * spec whose meta differs is looked up by its own. */
  uint16_t arg_meta[16];
  int32_t reserved[5];
} apc_comp_rec; /* 160 bytes */

/* A compute program as independent product terms, so that the wavefronts of a
 * workgroup can share them: value = coeff * product of the per-strategy values
 * idx[k] names (0xFF: no factor), added to the node's flops, or to its bytes
 * when `to_bytes` is set.  The per-strategy values are rows of the workgroup's
 * table of local sizes: rows [0, max_rank) the broadcast of all arguments'
 * sizes at a right-aligned position (row = position from the right), then per
 * argument a the rows max_rank + a * (max_rank + 2) + d: d < max_rank the local
 * size of dim d, d == max_rank + 1 the local element count.  Constant dims of
 * an output are folded into coeff.  Made from `prog` by the host
 * (PackedGraph.program_terms); same integers as the interpreted program. */
typedef struct apc_prog_term {
  int64_t coeff;
  uint8_t idx[7];
  uint8_t to_bytes;
} apc_prog_term; /* 16 bytes */
#define APC_TERMS_BCAST 1 /* some term reads a broadcast row */
#define APC_TERMS_MAX 64  /* terms per program                 */

/* A spec word of `lists` with what the redistribution cost reads behind it:
 * the placement bytes of its tuple, and itemsize * prod(shape) and the
 * contiguity of its tensor meta (spec_to_bytes,
 * torch:distributed/tensor/_collective_utils.py:230-232, and
 * check_contiguous_sizes_strides, torch:_prims_common/__init__.py:252-293).
 * One 16-byte load per side of a table element instead of the word, then its
 * tuple row, then two shape/stride rows.  Made per position of `lists` by the
 * host (PackedGraph.spec_records). */
typedef struct apc_spec_rec {
  uint32_t word;   /* lists[k]                                              */
  uint32_t plc;    /* tuple_plc row of the word, one byte per mesh dim      */
  int64_t nbytes2; /* nbytes << 1 | contiguous; 0 for APC_SPEC_NONE          */
} apc_spec_rec; /* 16 bytes */

/* What a workgroup of the block-table build reads about its 256 elements, in
 * one record instead of a chain through table_unit_block, block_off,
 * block_edge and the edge array. */
typedef struct apc_table_unit {
  int64_t default_off; /* default rows of the matrix's edge, or -1            */
  uint32_t src_list;   /* the two runs of spec words                          */
  uint32_t dst_list;
  uint32_t ncol;       /* columns / rows of the stored matrix (of distinct    */
  uint32_t nrow;       /* words when compressed)                              */
  uint32_t first;      /* element of the matrix that the unit starts at       */
  uint32_t flags;      /* APC_EDGE_COMPRESSED or 0                            */
} apc_table_unit; /* 32 bytes */

/* Cost-model constants (host values, passed by value into the kernels). */
typedef struct apc_model {
  int32_t ndim;
  int32_t mesh_shape[APC_MAX_MESH_DIMS];
  double mesh_bw[APC_MAX_MESH_DIMS];  /* GB/s per mesh dim                  */
  double mesh_lat[APC_MAX_MESH_DIMS]; /* us per hop per mesh dim            */
  double gmem_bw;                     /* bytes/s                            */
  double tflops[APC_NUM_DTYPES];      /* by dtype code; <= 0: unsupported   */
  /* mesh-dim order of the redistribution fold: 0 = the rule of
   * estimate_strategy_comms_cost (collective_runtime_estimation.py:253-258:
   * [1,0] for (Partial,Partial) -> all-Shard on a 2-D mesh, else 0..ndim-1);
   * 1 = always 0..ndim-1; 2 = always ndim-1..0 (an explicit `order` argument
   * of redistribute_cost, :115-119) */
  int32_t order_mode;
  int32_t reserved;
  /* NULL: alpha-beta collectives from mesh_bw / mesh_lat.  Otherwise a DEVICE
   * copy of the plan that apc_nccl_plan_build fills: collectives are priced by
   * the NCCL-tuning model (collective_runtime_estimation.py:44-62, 85-86). */
  const struct apc_nccl_plan* nccl_plan;
  /* GB/s that all_to_all sees on each mesh dim, where it differs from mesh_bw
   * (a fabric of direct links, on which an all-to-all drives every link at once
   * while a ring drives one); 0 = mesh_bw, the reference's model.  Filled by
   * apc_xgmi_topology. */
  double mesh_a2a_bw[APC_MAX_MESH_DIMS];
} apc_model;

/* ---- NCCL-tuning collective model (autoparallel/cost_models/nccl_cost_model.py) ----
 * The model is min over (algorithm, protocol) candidates of
 *     latency + n_bytes / (1000 * bandwidth)
 * where latency and bandwidth depend on the topology only, apart from a few
 * message-size corrections.  apc_nccl_plan_build resolves, on the host, the
 * size-independent part for every (mesh dim, collective); the kernels apply
 * the size-dependent corrections per entry. */
#define APC_NCCL_MAX_CAND 10
#define APC_NCCL_TABLE_LEN 24
/* candidate flags: size-dependent corrections applied on the device */
#define APC_NC_TREE_CORR 1       /* bw *= tree_corr[proto][log2i(n >> 6)] if that index < 23 (:577-580, :1038-1041) */
#define APC_NC_TREE_CORR24 2     /* same with index < 24 (:582-589)                                */
#define APC_NC_RING_CORR 4       /* bw *= interp(dim's ring table, n / n_ranks) (:594-601)          */
#define APC_NC_NVLS_RAMP 8       /* bw *= interp(nvls_tree_ramp, n / n_ranks) (:1046-1048)          */
#define APC_NC_FULL_MESH_RAMP 16 /* bw *= interp(full_mesh_ramp, n / n_ranks) below 2^30 B/rank (:1053-1061) */
#define APC_NC_PLATEAU 32        /* lat *= 1.4 if n / (n_channels * n_ranks) >= 64 (:603-611, :1064-1071) */
#define APC_NC_NIC 64            /* all-to-all NIC path: lat + n * remote / (1000 * bw * corr) (:1260-1285) */

typedef struct apc_nccl_config { /* NCCLTopoConfig (:67-82) */
  int32_t arch; /* 0 Ampere, 1 Hopper, 2 Blackwell */
  int32_t num_nodes;
  int32_t gpus_per_node;
  int32_t num_channels; /* 0 = architecture default */
  int32_t has_nvswitch;
  int32_t has_collnet;
  double bw_intra; /* GB/s per GPU inside a node */
  double bw_inter; /* GB/s per GPU between nodes */
  double net_latency;
} apc_nccl_config;

typedef struct apc_nccl_cand {
  double lat;    /* us */
  double bw;     /* GB/s */
  int32_t flags; /* APC_NC_* */
  int32_t proto; /* 0 LL, 1 LL128, 2 Simple: row of tree_corr */
} apc_nccl_cand;

typedef struct apc_nccl_dim { /* MeshDimTopo (:85-92) + resolved candidates */
  int32_t n_ranks, n_nodes, ppn, n_channels;
  double bw_intra, bw_inter; /* per channel */
  int32_t n_cand[4];         /* by collective: 0 allgather, 1 all_to_all, 2 allreduce, 3 reduce_scatter */
  apc_nccl_cand cand[4][APC_NCCL_MAX_CAND];
  double ring_corr[APC_NCCL_TABLE_LEN]; /* depth-scaled when n_nodes > 4 (:700-719) */
  double a2a_remote;                    /* (n_ranks - ppn) / n_ranks            */
  int32_t a2a_log_nodes;
  int32_t reserved;
} apc_nccl_dim;

typedef struct apc_nccl_plan {
  int32_t ndim;
  int32_t reserved;
  apc_nccl_dim dim[APC_MAX_MESH_DIMS];
  double tree_corr[3][APC_NCCL_TABLE_LEN];
  double nvls_tree_ramp[APC_NCCL_TABLE_LEN];
  double full_mesh_ramp[APC_NCCL_TABLE_LEN];
  double a2a_nic_ramp[APC_NCCL_TABLE_LEN];
} apc_nccl_plan;

/* The packed problem (see autoparallel_amd/packed.py for the layout). */
typedef struct apc_problem {
  apc_model model;
  /* tensor metas */
  int32_t n_meta;
  const int32_t* meta_rank;
  const int64_t* meta_shape;  /* [n_meta][APC_MAX_RANK] */
  const int64_t* meta_stride; /* [n_meta][APC_MAX_RANK] */
  const int32_t* meta_itemsize;
  const int32_t* meta_dtype;
  /* interned placement tuples, one byte per mesh dim */
  int32_t n_tuple;
  const uint8_t* tuple_plc; /* [n_tuple][APC_MAX_MESH_DIMS] */
  /* runs of spec words: meta_id << 12 | tuple_id, or APC_SPEC_NONE */
  int64_t n_list;
  const uint32_t* lists;
  /* nodes */
  int32_t n_node;
  const int32_t* node_nstrat;
  const int32_t* node_nargs;
  const int32_t* node_op;
  const int64_t* node_comp_off; /* [n_node] slot of (v, out_idx 0) in the compute
                                   vector; nodes with identical program and
                                   input specs may share a slot */
  const int32_t* node_edge_off; /* [n_node+1] */
  const int64_t* node_prog_off; /* -1 = none */
  const int32_t* node_prog_len; /* words of the node's program, 0 = none */
  int32_t max_node_args;        /* max over nodes of edges per node */
  int32_t max_rank;             /* max tensor rank over all metas */
  int64_t n_compute;            /* length of the compute / per_arg vectors */
  int32_t n_comp_node;          /* nodes to evaluate: one per distinct slot */
  int32_t max_nstrat;           /* max of node_nstrat over comp_nodes (>= 1)  */
  const int32_t* comp_nodes;    /* [n_comp_node] */
  const int32_t* node_multiplier;
  int64_t n_prog;
  const int64_t* prog;
  const int64_t* explicit_flops; /* may be NULL */
  const int64_t* explicit_bytes; /* may be NULL */
  /* edges */
  int32_t n_edge;
  const apc_edge* edges;
  int64_t n_entry;           /* real entries: sum of sdst * ssrc               */
  int64_t n_slot;            /* length of the entry arrays (with padding)      */
  int64_t n_chunk;           /* n_slot / 16                                    */
  const int32_t* chunk_edge; /* [n_chunk] edge owning slots [16c, 16c + 16)    */
  /* work items of the entry kernel: copies of the edge record, slot order, each
   * covering 256 (or item_entries) slots from entry local0 of its block on.  An
   * item may start before its block (local0 negative modulo 2^32, so that it
   * starts at a multiple of 64 slots of the entry arrays) and end after it:
   * lanes whose entry local0 + i is not below sdst * ssrc (unsigned) are idle */
  int32_t n_item;
  const apc_edge* items;     /* [n_item] */
  int64_t n_default;
  const double* default_vals;
  /* block table: one S_dst x S_src matrix per distinct (producer run, consumer
   * run) pair among the edges that have a producer and no missing spec, and one
   * of its own for each edge with a producer and a missing spec, in the edge
   * block's [out_idx][inp_idx] order: table[block_off[b] + out_idx * S_src +
   * inp_idx] = comm cost, with the sign bit set when the two placements differ.
   * Each matrix is padded to a multiple of 256 elements; apc_edge.table_off is
   * the matrix of the edge.  A caller that passes a table to apc_edge_costs
   * gives every edge with a producer a matrix, and keeps every default value's
   * sign bit clear (the table path reads default rows with the same decoding). */
  int32_t n_block;
  const int32_t* block_edge;       /* [n_block] an edge that owns matrix b          */
  const int64_t* block_off;        /* [n_block+1], multiples of 256                  */
  int64_t table_size;              /* doubles: block_off[n_block]                    */
  int32_t n_table_unit;            /* table_size / 256                               */
  const int32_t* table_unit_block; /* [n_table_unit] matrix owning elements [256 u, 256 u + 256) */
  /* compressed block table (all three NULL otherwise).  Strategies of a node
   * that differ in other arguments or outputs repeat spec words, and a cost
   * depends on the two words only (the key of the reference's own memo,
   * autoparallel/cost_models/collective_runtime_estimation.py:232-246): the
   * matrix of an edge flagged APC_EDGE_COMPRESSED has one row per distinct
   * word of the consumer run and one column per distinct word of the producer
   * run, table[table_off + list_uidx[dst_list + out_idx] * usrc +
   * list_uidx[src_list + inp_idx]].  Runs are disjoint ranges of lists. */
  const int32_t* list_uidx;   /* [n_list] rank of the word among its run's distinct words */
  const int32_t* list_ufirst; /* [n_list] at run + k: position in the run of its k-th distinct word */
  const int32_t* block_udst;  /* [n_block] rows of matrix b */
  /* optional: one record per entry of comp_nodes (NULL: the kernel gathers the
   * same fields from the arrays above) */
  const apc_comp_rec* comp_recs;
  /* entries per work item: 0 or APC_ITEM_ENTRIES, or 2 * APC_ITEM_ENTRIES (block
   * table only), as the items array was built */
  int32_t item_entries;
  /* optional accelerators of the prepare launch, each derived from the arrays
   * above by the host (NULL: the kernels walk those arrays instead) */
  const apc_table_unit* table_units; /* [n_table_unit]                          */
  const apc_spec_rec* spec_recs;     /* [n_list]                                */
  int64_t n_prog_term;
  const apc_prog_term* prog_terms;   /* named by apc_comp_rec.term_off / n_term */
  /* optional: tile lists for the lookup-table kernels (both need spec_recs).
   * With lut_table_tiles (every matrix of the block table covered exactly once)
   * apc_prepare / apc_build_pair_table / apc_build_all build the table tile by
   * tile (lut_kernel<table>) instead of element by element; worth it from a few
   * thousand table units on.  With lut_entry_tiles (every edge block that owns
   * entries covered exactly once, edges without a producer included)
   * apc_edge_costs / apc_build_all called with table == NULL evaluate the
   * entries tile by tile (lut_kernel<entries>, three times the rate of the
   * per-entry fold).  NULL: the element-by-element kernels, same bits. */
  const struct apc_lut_tile* lut_table_tiles;
  int64_t n_lut_table_tile;
  const struct apc_lut_tile* lut_entry_tiles;
  int64_t n_lut_entry_tile;
} apc_problem;

/* What is checked, and what is the caller's to check.  Every entry point that
 * takes an apc_problem checks sizes, counts and null pointers on the host and
 * refuses what is inconsistent (APC_ERR_INVALID).  The CONTENTS of the index
 * arrays are not read on the host (they live in device memory): chunk_edge,
 * edges[].off / src_list / dst_list / default_off / table_off / comp_base, items,
 * node_edge_off, node_comp_off, block_off, list_uidx / list_ufirst, the tile
 * lists and the program words must name positions inside the arrays they index,
 * or a kernel reads or writes outside them.  The Python packer validates all of
 * them before it uploads (PackedGraph.validate); a C caller that fills the
 * arrays itself owns that check.
 *
 * Which kernel an entry point launches (all on `stream`, asynchronously):
 *   apc_prepare             prepare_kernel: table blocks + node blocks in one launch;
 *                           tables of more than 2 048 units get pair_table_kernel of
 *                           their own first; with lut_table_tiles the table is built
 *                           by lut_kernel<table> instead (then prepare_kernel prices
 *                           the nodes only)
 *   apc_build_pair_table    the table part of the above alone
 *   apc_node_compute_costs  the node part of the above alone
 *   apc_edge_costs          with a table and all three outputs: edge_cost_item_kernel
 *                           <compressed,n>, one wavefront per work item (compressed:
 *                           list_uidx set; n = 4 or 8 entries per lane by
 *                           item_entries); with an output left out (or more than
 *                           16.7 M work items): edge_cost_kernel<1,n> / <2,n>, the same
 *                           arithmetic in a loop of predicated accesses;
 *                           table == NULL: lut_kernel<entries>
 *                           when the problem carries lut_entry_tiles, else
 *                           edge_cost_kernel<0,4>, the per-entry fold (the fallback
 *                           for problems without spec_recs; a third of the rate)
 *   apc_build_all           apc_prepare, then apc_edge_costs
 *   apc_build_pair_table_lut / apc_edge_costs_lut   lut_kernel over a list passed as
 *                           an argument instead of the problem's own
 *
 * Version of the ABI (struct layouts and signatures of this header): 5. */
int apc_version(void);
const char* apc_last_error(void);

/* Host helper.  Replaces MeshTopoInfo.build_from_mesh
 * (torch:distributed/tensor/_collective_utils.py:246-278): per-mesh-dim
 * bandwidth (GB/s) and latency (us) from the mesh shape and the number of
 * devices per host.  bw/lat: host arrays of ndim doubles. */
int apc_mesh_topology(const int32_t* mesh_shape, int32_t ndim, int32_t devices_per_host,
                      double* bw, double* lat);

/* Host helper, no counterpart in the reference, which has topology presets for
 * NVLink/NVSwitch systems only (nccl_cost_model.py:1413-1470) and detects none
 * on an MI355X (:1341-1410), leaving that user with NVLink constants.  Per-dim
 * constants of the alpha-beta model for nodes whose GPUs are joined pairwise
 * by xGMI links: walking the mesh dims from the innermost out, a dim lies inside
 * a node while the product of the sizes so far is at most gpus_per_node.
 * Inside a node a ring collective (allgather, reduce_scatter, allreduce) moves
 * every byte over one link per rank and direction: bw = link_gbps / 2 (a link's
 * figure counts both directions); an all_to_all among the n ranks of the dim
 * drives min(n - 1, links_per_gpu) links of every rank at once: a2a_bw = that
 * many times bw.  Between nodes both are nic_gbps (per GPU).  lat: lat_intra_us
 * / lat_inter_us per hop.  bw, lat, a2a_bw: host arrays of ndim doubles, to be
 * copied into apc_model.mesh_bw / mesh_lat / mesh_a2a_bw. */
typedef struct apc_xgmi_config {
  int32_t gpus_per_node; /* 8 */
  int32_t links_per_gpu; /* 7: one direct link to every peer of the node */
  double link_gbps;      /* one link, both directions together: 153.6 on MI355X */
  double nic_gbps;       /* per GPU between nodes */
  double lat_intra_us;   /* per hop inside a node */
  double lat_inter_us;   /* per hop between nodes */
} apc_xgmi_config;
int apc_xgmi_topology(const apc_xgmi_config* cfg, const int32_t* mesh_shape, int32_t ndim, double* bw,
                      double* lat, double* a2a_bw);

/* Host helper.  Replaces _get_device_limit / _get_device_tflops /
 * _get_device_gmem_bandwidth (autoparallel/cost_models/compute_estimation.py:258-297)
 * for the devices this library knows: fills gmem_bw and tflops[] of *model.
 * Returns APC_ERR_UNSUPPORTED for an unknown device name (the reference raises
 * ValueError there). */
int apc_device_limits(const char* device_name, apc_model* model);

/* Host helper.  Replaces derive_mesh_dim_topo (nccl_cost_model.py:1001-1021),
 * _compute_algo_bw (:323-465), _compute_algo_latency (:473-551), the candidate
 * selection of nccl_collective_time (:1163-1212, :1081-1160), _eligible_algos /
 * _eligible_protos (:616-649), _depth_scaled_ring_correction (:700-719) and the
 * size-independent part of nccl_all_to_all_cost (:1215-1313).  plan: host
 * memory; copy it to the device and point apc_model.nccl_plan at the copy. */
int apc_nccl_plan_build(const apc_nccl_config* cfg, const int32_t* mesh_shape, int32_t ndim,
                        struct apc_nccl_plan* plan);

/* Host helper.  As apc_nccl_plan_build for ONE communicator whose topology the
 * caller states (the MeshDimTopo argument of nccl_allgather_cost /
 * nccl_allreduce_cost / nccl_reduce_scatter_cost / nccl_all_to_all_cost,
 * nccl_cost_model.py:1215-1336): fills plan->dim[0], plan->ndim = 1.
 * bw_intra / bw_inter are per channel, as MeshDimTopo holds them. */
int apc_nccl_plan_for_topo(const apc_nccl_config* cfg, int32_t n_ranks, int32_t n_nodes, int32_t ppn,
                           int32_t n_channels, double bw_intra, double bw_inter,
                           struct apc_nccl_plan* plan);

/* Number of doubles of the block table apc_build_pair_table fills
 * (= p->table_size). */
int64_t apc_pair_table_size(const apc_problem* p);

/* Replaces estimate_strategy_comms_cost + redistribute_cost + collective_comm_cost
 * + all_to_all_cost (autoparallel/cost_models/collective_runtime_estimation.py:65-110,
 * 115-229, 239-262), torch's allgather/allreduce/reduce_scatter_cost
 * (torch:distributed/tensor/_collective_utils.py:281-313) and
 * compute_read_write_time (autoparallel/cost_models/compute_estimation.py:391-403),
 * evaluated once per distinct (producer strategies, consumer strategies) matrix:
 * table[block_off[b] + out_idx * S_src + inp_idx], microseconds, +inf for
 * forbidden transitions, sign bit = the transition flag of
 * _compute_edge_costs (autoparallel/optimize_sharding.py:474-478). */
int apc_build_pair_table(const apc_problem* p, double* table, void* stream);

/* A tile of one cost matrix for the lookup-table kernels below: columns
 * [col0, col0 + ncols) (ncols <= 64) and rows [row0, row0 + nrows) (nrows <= 1024) of an
 * S_dst x S_src matrix (nrow x ncol; of distinct words when APC_EDGE_COMPRESSED),
 * whose element (o, j) goes to out + o * ncol + j. */
typedef struct apc_lut_tile {
  int64_t out;         /* table: first element of the matrix; entries: slot of entry (0, 0) */
  int64_t default_off; /* default rows of the edge, or -1                       */
  uint32_t src_list;
  uint32_t dst_list;
  uint32_t ncol;
  uint32_t nrow;
  uint32_t col0;
  uint32_t ncols;
  uint32_t row0;
  uint32_t nrows;
  uint32_t flags;      /* APC_EDGE_HAS_PRODUCER | APC_EDGE_COMPRESSED            */
  int32_t comp_base;   /* entries: index of (node, out_idx 0) in per_arg         */
  uint32_t magic;      /* floor(2^32 / ncols) + 1: idx / ncols == umulhi(idx, magic) for idx < 2^20;
                          0 for ncols == 1 */
  uint32_t reserved;
} apc_lut_tile; /* 64 bytes */

/* apc_build_pair_table for large tables: the same table, bit for bit, built
 * tile by tile with the terms of each source spec computed once per tile into
 * LDS (replaces the same reference functions as apc_build_pair_table).  tiles:
 * device array covering every matrix of the block table exactly once
 * (PackedGraph.lut_tiles).  Needs apc_problem.spec_recs. */
int apc_build_pair_table_lut(const apc_problem* p, const apc_lut_tile* tiles, int64_t n_tile, double* table,
                             void* stream);

/* apc_edge_costs with table == NULL (direct evaluation), bit for bit, tile by
 * tile the same way: tiles cover every edge block exactly once, edges without
 * a producer included (their entries are their default rows). */
int apc_edge_costs_lut(const apc_problem* p, const apc_lut_tile* tiles, int64_t n_tile, const double* per_arg,
                       double* comm, double* cost, uint8_t* flags, int32_t clamp_inf, void* stream);

/* Replaces estimate_strategy_runtime_cost
 * (autoparallel/cost_models/compute_estimation.py:438-493, with
 * _get_sharded_shape_stride :300-318 and compute_memory_cost :321-331) for
 * every (node, out_idx) of the nodes in comp_nodes: compute[node_comp_off[v] + o]
 * in microseconds, and
 * per_arg = compute / num_args (autoparallel/optimize_sharding.py:516).
 * status (device int32[1], zeroed by the caller) is set non-zero if a node
 * with flops has an input dtype without a tflops entry (ValueError in the
 * reference, compute_estimation.py:287-291). */
int apc_node_compute_costs(const apc_problem* p, double* compute, double* per_arg,
                           int32_t* status, void* stream);

/* Replaces the entry loop of ShardingOptimizer._build_decision_vars and
 * _compute_edge_costs (autoparallel/optimize_sharding.py:446-479, 511-552):
 * for every entry (node, argi, out_idx, inp_idx)
 *     comm  = table lookup / direct evaluation / default row value
 *     flags = APC_ENTRY_TRANSITION | APC_ENTRY_NONFINITE
 *     cost  = comm + per_arg + transition
 * and, if clamp_inf != 0, add_inf_cost_constraint's rewrite of non-finite cost
 * to 10000.0 (:803-812).  table may be NULL: every entry is then evaluated
 * directly (same arithmetic, no table memory, any default values).  comm /
 * cost / flags may each be NULL to skip that output. */
int apc_edge_costs(const apc_problem* p, const double* table, const double* per_arg,
                   double* comm, double* cost, uint8_t* flags, int32_t clamp_inf, void* stream);

/* apc_build_pair_table (skipped if table is NULL) and apc_node_compute_costs in
 * one launch: the two are independent of each other. */
int apc_prepare(const apc_problem* p, double* table, double* compute, double* per_arg,
                int32_t* status, void* stream);

/* The three steps above in two launches (pair table and node estimates share
 * one; three when the table is built by tiles): the whole of
 * ShardingOptimizer._build_decision_vars' arithmetic
 * (autoparallel/optimize_sharding.py:481-552) in one call.  table may be NULL
 * (direct evaluation: by tiles if the problem carries lut_entry_tiles). */
int apc_build_all(const apc_problem* p, double* table, double* compute, double* per_arg,
                  int32_t* status, double* comm, double* cost, uint8_t* flags, int32_t clamp_inf,
                  void* stream);

/* apc_build_all for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): no
 * counterpart in the reference.  The block table, the one buffer of the build
 * that is neither input nor output, lives in a static device array of
 * APC_NOALLOC_MAX_TABLE doubles (8 MiB per GPU, held until the process ends)
 * instead of a buffer of the caller's; everything else is passed as for
 * apc_build_all, and the results are the same bit for bit.  Returns
 * APC_ERR_INVALID when p->table_size exceeds APC_NOALLOC_MAX_TABLE; with
 * table_size == 0 every entry is evaluated directly.  The call allocates
 * nothing.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress) and sets a kernel attribute once: make one eager call
 * per device before capturing calls into a HIP graph, where those two host
 * calls may be refused.  Every
 * call on a GPU shares that GPU's array: calls that overlap on one GPU (two
 * streams, two threads) race; a build reads only the table elements it wrote
 * itself, so nothing needs clearing between calls. */
#define APC_NOALLOC_MAX_TABLE (1 << 20)
int apc_build_all_noalloc(const apc_problem* p, double* compute, double* per_arg, int32_t* status,
                          double* comm, double* cost, uint8_t* flags, int32_t clamp_inf,
                          void* stream);

/* Measurement aids, no counterpart in the reference.  A timer owns n_slots
 * pairs of HIP events (host objects, no device memory).  apc_edge_costs_timed
 * is apc_edge_costs with the pair of `slot` recorded at the kernel's own begin
 * and end on the launch stream (hipExtLaunchKernelGGL's start/stop events), so
 * the elapsed time is the kernel's duration without dispatch latency; read it
 * with apc_timer_elapsed_ms after synchronising the stream. */
int apc_timer_create(int32_t n_slots, void** timer);
int apc_timer_destroy(void* timer);
int apc_timer_elapsed_ms(void* timer, int32_t slot, float* ms);
int apc_edge_costs_timed(const apc_problem* p, const double* table, const double* per_arg,
                         double* comm, double* cost, uint8_t* flags, int32_t clamp_inf, void* timer,
                         int32_t slot, void* stream);
/* apc_edge_costs_lut with the events at the begin and end of its kernel. */
int apc_edge_costs_lut_timed(const apc_problem* p, const apc_lut_tile* tiles, int64_t n_tile,
                             const double* per_arg, double* comm, double* cost, uint8_t* flags,
                             int32_t clamp_inf, void* timer, int32_t slot, void* stream);
/* apc_build_all with the entry kernel timed as apc_edge_costs_timed does. */
int apc_build_all_timed(const apc_problem* p, double* table, double* compute, double* per_arg,
                        int32_t* status, double* comm, double* cost, uint8_t* flags,
                        int32_t clamp_inf, void* timer, int32_t slot, void* stream);

/* Measurement aid, no counterpart in the reference: a plain device copy of
 * nbytes (multiple of 16) whose HBM traffic is known (nbytes read + nbytes
 * written), used to scale hardware traffic counters in profiles. */
int apc_calibration_copy(const void* src, void* dst, int64_t nbytes, void* stream);

/* Replaces apply_prefetch_discount (autoparallel/optimize_sharding.py:824-875)
 * on the entry arrays, for edges flagged APC_EDGE_PREFETCHABLE: comm *= scale
 * and cost = comm + per_arg + transition where 0 < comm < inf.  n_modified:
 * device uint64[1], zeroed by the caller, receives the number of entries changed. */
int apc_apply_prefetch_discount(const apc_problem* p, const double* per_arg, double scale,
                                double* comm, double* cost, const uint8_t* flags,
                                unsigned long long* n_modified, void* stream);

/* Replaces the coefficient rule of _set_objective
 * (autoparallel/optimize_sharding.py:879-885): obj = cost * node_multiplier. */
int apc_objective_coeffs(const apc_problem* p, const double* cost, double* obj, void* stream);

/* Replaces _hash_node (autoparallel/graph_passes/graph_clustering.py:68-82),
 * the key under which get_identical_regions groups repeated nodes: a 64-bit
 * structural hash per node over its op class, program, forward/backward tag
 * (node_phase int32[n_node], may be NULL; a caller that knows more of the
 * reference's key than the problem holds, such as the operator's name, source
 * position and non-tensor arguments of a traced node, passes one id per
 * distinct combination of those and the tag here), strategy counts, output spec run
 * (node_out_list int64[n_node]: offset of the node's output run in lists),
 * input and producer spec runs and default rows.  Equal keys in the reference
 * imply equal hashes here; out: uint64[n_node]. */
int apc_node_hashes(const apc_problem* p, const int64_t* node_out_list, const int32_t* node_phase,
                    uint64_t* out, void* stream);

/* Replaces the per-variable loop of save_optimizer
 * (autoparallel/serialization.py:145-161): the packed twin of decision_vars,
 * keys int32[E][4] = (node_idx, argi, out_idx, inp_idx) and vals double[E][3] =
 * (compute_cost, comm_cost, sharding_transition_cost), rows in decision_vars'
 * insertion order (node, out_idx, argi, inp_idx;
 * autoparallel/optimize_sharding.py:511-520).  row_base[e] (int64) is the row of
 * entry (e, 0, 0) and row_stride[e] (int32) the number of rows per out_idx of
 * e's node (sum of S_src over the node's arguments). */
int apc_export_decision_vars(const apc_problem* p, const double* per_arg, const double* comm,
                             const uint8_t* flags, const int64_t* row_base,
                             const int32_t* row_stride, int32_t* keys, double* vals, void* stream);

/* The three entry arrays with the padding between edge blocks taken out: element
 * var_start[e] + out_idx * S_src + inp_idx of the outputs is entry (e, out_idx,
 * inp_idx), i.e. the arrays are indexed by decision variable, in
 * walk_over_options order (autoparallel/optimize_sharding.py:400-410), which is
 * the column order of the ILP.  var_start: int64[n_edge], running sum of the
 * entries of the edges that own a block.  Outputs hold n_entry elements.  This is
 * what a host reads back (17 B per variable) instead of the padded arrays. */
int apc_compact_entries(const apc_problem* p, const int64_t* var_start, const double* comm,
                        const double* cost, const uint8_t* flags, double* out_comm, double* out_cost,
                        uint8_t* out_flags, void* stream);

/* Replaces the selected-variable gathers of export_sharding_json
 * (autoparallel/export_json.py:314-361) and get_log
 * (autoparallel/log_formatting.py:118-130) for one assignment (assign:
 * uint16[n_node], out_idx per node): terms double[n_edge][4] = (compute_cost,
 * comm_cost, sharding_transition_cost, cost) of the selected entry of every
 * (node, arg) edge, slot int64[n_edge] its slot (NaN / -1 where the assignment
 * is not a strategy index of the edge). */
int apc_solution_terms(const apc_problem* p, const double* per_arg, const double* comm,
                       const double* cost, const uint8_t* flags, const uint16_t* assign,
                       double* terms, int64_t* slot, void* stream);

/* Replaces _compute_solution_cost (autoparallel/optimize_sharding.py:1056-1111)
 * and evaluates the ILP objective (:879-885) with its inf-cost rows (:803-812)
 * for a batch of assignments.  assign: uint16 [n_node][n_assign] (node-major),
 * the chosen out_idx per node.  out: double [n_assign][6] =
 * (total, compute, comm, transition, ilp_objective, n_forbidden_selected).
 * Sums run in graph node order then argument order, as the reference's loop. */
int apc_score_assignments(const apc_problem* p, const double* per_arg, const double* comm,
                          const double* cost, const uint8_t* flags, const uint16_t* assign,
                          int64_t n_assign, double* out, void* stream);

/* As apc_score_assignments, with assignment a drawn on the fly: out_idx of node
 * v = mix32(seed, a, v) * node_nstrat[v] >> 32 (counter-based, nothing materialised).
 * apc_random_assignment (host) gives the same draw for checking. */
int apc_score_random_assignments(const apc_problem* p, const double* per_arg, const double* comm,
                                 const double* cost, const uint8_t* flags, uint64_t seed,
                                 int64_t first, int64_t n_assign, double* out, void* stream);
uint32_t apc_random_assignment(uint64_t seed, int64_t a, int32_t node, int32_t nstrat);

/* Candidate assignments that select no forbidden variable, where the graph allows
 * it.  No function of the reference does this; "forbidden" is the reference's own
 * notion: a decision variable whose cost is not finite, which
 * add_inf_cost_constraint pins to zero (autoparallel/optimize_sharding.py:803-812;
 * the APC_ENTRY_NONFINITE bit of flags).  Two calls.
 *
 * apc_pack_allowed_columns writes, for every argument row (edge) e and every
 * choice j of its producer, the bit column of the consumer's strategies whose entry
 * (e, out_idx, j) is finite: words colbits[col_off[e] + j * Wc + w], w < W =
 * ceil(S_dst / 64), bit (out_idx mod 64) of word out_idx / 64; bits past S_dst are
 * zero.  Wc = W rounded up to an even number: a column is whole pairs of words, and
 * with colbits 16-byte aligned and every col_off even the sampler reads it 16 bytes
 * at a time (the odd word of a column with an odd W is never written and may hold
 * anything).  col_off: int64[n_edge], the caller's layout (S_src * Wc words per edge;
 * edges that share a block may share their columns); max_words: the largest W.
 * To be called again after anything that rewrites flags.
 *
 * apc_sample_feasible: for assignment a (counter first + a) the nodes from
 * first_node on are walked in order and node v gets, uniformly, one of the
 * strategies out_idx whose entries (v, arg, out_idx, choice of the producer of arg)
 * are all finite: the AND of one column per argument row; with `count` of them
 * it is the one of rank apc_sample_rank(seed, first + a, id of v, count) in out_idx
 * order.  A node without such a strategy takes the plain draw of
 * apc_random_assignment and is counted in n_fallback[a].
 * assign: uint16[n_node][n_assign], written for v >= first_node; the rows below
 * first_node are read (choices made earlier, e.g. for the stand-in nodes of a
 * window of a larger graph).  node_gid: id of every node for the hashes (NULL:
 * its index).  row_filter / filter_off (both or neither): strategies a node may
 * take at all, whatever its producers chose; filter_off[v] is the first of the W
 * words of node v's filter in row_filter (bit out_idx mod 64 of word out_idx / 64),
 * or -1 for a node without one.  With filters that confine the producers of the
 * nodes that would otherwise run out of strategies (autoparallel_amd/feasible_plan.py
 * makes them on the host), no node of the planner stress DAG falls back.  The
 * plain draw of a node that does fall back ignores its filter.
 * Score the result with apc_score_assignments or the batch scorers
 * that take explicit assignments: element 5 of a row is 0 where n_fallback is.
 * One lane per assignment. */
int apc_pack_allowed_columns(const apc_problem* p, const uint8_t* flags, const int64_t* col_off,
                             int32_t max_words, uint64_t* colbits, void* stream);
int apc_sample_feasible(const apc_problem* p, const uint64_t* colbits, const int64_t* col_off, uint64_t seed,
                        int64_t first, int64_t n_assign, const int32_t* node_gid, int32_t first_node,
                        const uint64_t* row_filter, const int64_t* filter_off, uint16_t* assign,
                        int32_t* n_fallback, void* stream);
uint32_t apc_sample_rank(uint64_t seed, int64_t a, int32_t node, uint32_t count);

/* apc_score_random_assignments for a graph too large to keep its coefficients
 * resident: the problem holds a window of the graph's nodes (preceded by
 * first_node stand-ins for producers outside the window, which are not scored),
 * node_gid[v] is the node's index in the whole graph (the draw uses it, so a
 * node gets the same out_idx in every window), and the sums continue from
 * init (the out of the previous window; NULL = start at zero): scoring the
 * windows in node order forms every sum in the order of one pass over the whole
 * graph, bit for bit.  One lane per assignment. */
int apc_score_random_window(const apc_problem* p, const double* per_arg, const double* comm,
                            const double* cost, const uint8_t* flags, uint64_t seed,
                            int64_t first, int64_t n_assign, const int32_t* node_gid,
                            int32_t first_node, const double* init, double* out, void* stream);

/* apc_score_assignments for a window of a larger graph: the first first_node
 * nodes (stand-ins for producers outside the window, whose rows of assign carry
 * the choices made for them) contribute nothing, and the sums continue from init
 * (double[n_assign][6], or NULL to start from zero).  assign: uint16[n_node][n_assign]. */
int apc_score_assignments_window(const apc_problem* p, const double* per_arg, const double* comm,
                                 const double* cost, const uint8_t* flags, const uint16_t* assign,
                                 int64_t n_assign, int32_t first_node, const double* init, double* out,
                                 void* stream);

/* The three entry arrays interleaved, for scoring graphs whose edge blocks are
 * large: a drawn entry then costs one 32-byte gather instead of three gathers in
 * three arrays (measured 2x on blocks of 65 k entries, nothing on blocks of
 * 650). */
typedef struct apc_score_rec {
  double comm;
  double cost;
  uint64_t flags; /* APC_ENTRY_* */
  uint64_t reserved;
} apc_score_rec; /* 32 bytes */

/* recs[slot] = {comm[slot], cost[slot], flags[slot]} for the n_slot slots. */
int apc_pack_score_records(const apc_problem* p, const double* comm, const double* cost,
                           const uint8_t* flags, apc_score_rec* recs, void* stream);

/* apc_score_assignments (assign != NULL) or apc_score_random_assignments /
 * apc_score_random_window (assign == NULL; node_gid, init may be NULL: local
 * node ids, sums from zero) reading the interleaved records; same sums, bit
 * for bit.  One lane per assignment. */
int apc_score_packed(const apc_problem* p, const double* per_arg, const apc_score_rec* recs,
                     const uint16_t* assign, uint64_t seed, int64_t first, int64_t n_assign,
                     const int32_t* node_gid, int32_t first_node, const double* init,
                     double* out, void* stream);

/* Compact records for graphs with large blocks: cost is not stored, because
 * the cost of an entry is (comm + per_arg[comp_base + out_idx]) + transition
 * (autoparallel/optimize_sharding.py:544), or the clamp 10000 where that sum
 * is not finite, and the scorer holds per_arg of its node's choice already. */
#define APC_SCORE_CLAMPED 4 /* in apc_score_rec16.flags beside APC_ENTRY_*: cost is the clamp */
typedef struct apc_score_rec16 {
  double comm;
  uint64_t flags;
} apc_score_rec16; /* 16 bytes */

/* recs[slot] = {comm[slot], flags[slot] | clamped}; mismatch[0] (device) = 0,
 * or 1 if some cost[slot] is neither that sum nor its clamp (arrays changed
 * after the build): then the records must not be used.  p needs chunk_edge. */
int apc_pack_score_records16(const apc_problem* p, const double* per_arg, const double* comm,
                             const double* cost, const uint8_t* flags, apc_score_rec16* recs,
                             int32_t* mismatch, void* stream);

/* apc_score_packed over the compact records, for the nodes [first_node,
 * end_node), per_lane assignments per lane (1, 2, 4, 8; 0: chosen so that a
 * batch of up to 2^21 walks the graph once, larger batches in launches of
 * 2^21).  Same sums, bit for bit. */
int apc_score_compact(const apc_problem* p, const double* per_arg, const apc_score_rec16* recs,
                      const uint16_t* assign, uint64_t seed, int64_t first, int64_t n_assign,
                      const int32_t* node_gid, int32_t first_node, int32_t end_node, int32_t per_lane,
                      const double* init, double* out, void* stream);

/* What the table scorer needs to know about an edge beside its apc_edge record,
 * in one 16-byte load. */
typedef struct apc_score_edge_aux {
  int32_t msize;       /* elements of the edge's matrix to take through LDS, tile by tile
                          (apc_score_table_tile() elements a tile): even, and only for an
                          edge with table_off >= 0 (the matrix's padded size in the table
                          will do); 0: read the matrix in place (no matrix: default rows;
                          or too large to be worth it)                                   */
  int32_t next_staged; /* the first edge >= this one with msize > 0, or -1            */
  int32_t src_gid;     /* id of the producer node for the draw: node_gid[src_node], or
                          src_node itself when the draw uses local ids; unused without
                          a producer                                                  */
  int32_t reserved;
} apc_score_edge_aux; /* 16 bytes */

/* The same sums from the block table instead of the entry arrays, for graphs
 * with large blocks: an entry is (|m| + per_arg) + transition with the flag in
 * the sign of its matrix element m, clamped to 10000 if clamp_inf and not finite
 * (what apc_edge_costs writes from the table), so the result equals, bit for
 * bit, that of apc_score_packed on the arrays of a build with this clamp_inf.
 * One workgroup of 1024 lanes per CU, per_lane assignments each (1, 2, 4; 0:
 * chosen), has the current edge's matrix in LDS and draws from there.
 * edge_aux (device): n_edge + 1 records, the last one {0, -1, 0, 0}.  table as
 * for apc_edge_costs; p carries list_uidx if it has compressed matrices. */
int apc_score_table(const apc_problem* p, const double* per_arg, const double* table,
                    const apc_score_edge_aux* edge_aux, const uint16_t* assign,
                    uint64_t seed, int64_t first, int64_t n_assign, const int32_t* node_gid,
                    int32_t first_node, int32_t end_node, int32_t clamp_inf, int32_t per_lane,
                    const double* init, double* out, void* stream);
int apc_score_table_tile(void);

/* Replaces remove_invalid_configs (autoparallel/shardings/propagation_rules.py:127-158)
 * and keep_unique_configs (autoparallel/shardings/placement_options.py:151-170) for the
 * candidate strategies of n_set nodes in packed form.  Set s has rows
 * [set_row[s], set_row[s + 1]), each of set_width[s] spec words (the strategy's
 * input specs, then its output specs; APC_SPEC_NONE for a missing one) starting at
 * words[set_word[s]], row-major.  valid[row] = 1 if every spec of the row keeps
 * every sharded dim non-empty (walking the mesh dims in order, Shard(d) needs the
 * size of dim d, already divided by the earlier mesh dims that shard it, to be at
 * least the mesh size); keep[row] = valid and no earlier valid row of the set has
 * the same words (equal words stand for equal specs when the words were interned
 * by value).  max_rows: the largest set's row count, at most 4096.  Word layout
 * and tables are those of an apc_problem; meta_shape is [n_meta][APC_MAX_RANK]. */
int apc_filter_strategies(const apc_model* model, int32_t n_meta, const int32_t* meta_rank,
                          const int64_t* meta_shape, int32_t n_tuple, const uint8_t* tuple_plc, int32_t n_set,
                          const int64_t* set_row, const int32_t* set_width, const int64_t* set_word,
                          const uint32_t* words, int32_t max_rows, uint8_t* valid, uint8_t* keep, void* stream);

/* Replaces _get_sharded_shape_stride
 * (autoparallel/cost_models/compute_estimation.py:300-318) for n specs:
 * rank[i], shape/stride[i][APC_MAX_RANK], plc[i][APC_MAX_MESH_DIMS] ->
 * out_shape / out_stride[i][APC_MAX_RANK]. */
int apc_local_shapes(const apc_model* model, int32_t n, const int32_t* rank, const int64_t* shape,
                     const int64_t* stride, const uint8_t* plc, int64_t* out_shape,
                     int64_t* out_stride, void* stream);

/* Replaces collective_comm_cost
 * (autoparallel/cost_models/collective_runtime_estimation.py:65-110), default
 * model or, with model->nccl_plan set, _nccl_comm_cost (:44-62) and
 * nccl_collective_time / nccl_all_to_all_cost (nccl_cost_model.py:1163-1313), for n
 * queries: kind[i] 0 allgather, 1 all_to_all, 2 allreduce, 3 reduce_scatter
 * (anything else costs 0.0), nbytes[i], mesh dim[i] -> out[i] microseconds. */
int apc_collective_costs(const apc_model* model, int32_t n, const int32_t* kind,
                         const int64_t* nbytes, const int32_t* dim, double* out, void* stream);

/* Replaces compute_read_write_time
 * (autoparallel/cost_models/compute_estimation.py:391-403) for n byte counts. */
int apc_rw_times(const apc_model* model, int32_t n, const double* nbytes, double* out,
                 void* stream);

/* Replaces _create_all_options + remove_invalid_configs for input/parameter
 * nodes (autoparallel/shardings/propagation_rules.py:127-158, 184-201): for
 * each of n tensors (rank[i], shape[i][APC_MAX_RANK]) writes, for every
 * candidate c in itertools.product order over {R, S(0..rank-1)}^ndim,
 * valid[cand_off[i] + c] (uint8) and its placement bytes
 * plc[(cand_off[i] + c) * APC_MAX_MESH_DIMS ..]. */
int apc_enumerate_input_options(const apc_model* model, int32_t n, const int32_t* rank,
                                const int64_t* shape, const int64_t* cand_off, uint8_t* valid,
                                uint8_t* plc, void* stream);

/* ---------------------------------------------------------------------------
 * Schedule estimator: timeline and peak memory of a lowered graph (collectives
 * as nodes) under many candidate orders.
 * ------------------------------------------------------------------------- */
#define APC_SCHED_MAX_STREAMS 8
/* node flags */
#define APC_SCHED_COMM 1    /* a communication node (collective or wait_tensor)      */
#define APC_SCHED_WAIT 2    /* wait_tensor on the compute stream whose argument is
                               not a graph input: stalls until wait_src has ended  */
#define APC_SCHED_SYNC 4    /* blocking collective: the compute stream waits for it */
#define APC_SCHED_NO_MEM 8  /* placeholder / get_attr / output: allocates and frees
                               nothing when scheduled                               */

typedef struct apc_schedule {
  int32_t n_node;
  int32_t n_stream;        /* streams in use, <= APC_SCHED_MAX_STREAMS; 0 = compute   */
  const double* dur;       /* [n_node] runtime estimate of the node, microseconds    */
  const int32_t* stream;   /* [n_node] stream the node runs on                        */
  const uint8_t* flags;    /* [n_node] APC_SCHED_*                                    */
  const int32_t* wait_src; /* [n_node] for APC_SCHED_WAIT: the collective waited for, or -1 */
  /* storages (liveness as torch's MemoryTracker keeps it) */
  int32_t n_storage;
  const int64_t* st_bytes;    /* [n_storage]                                          */
  const uint8_t* st_freeable; /* [n_storage] on a tracked device and releasable       */
  const int32_t* st_users;    /* [n_storage] number of nodes that read the storage    */
  const int32_t* alloc_off;   /* [n_node+1] into alloc_st: storages the node allocates */
  const int32_t* alloc_st;
  const int32_t* use_off;     /* [n_node+1] into use_st: storages the node reads       */
  const int32_t* use_st;
  int64_t initial_bytes;      /* live before the first node (graph inputs, attributes) */
  /* optional accelerator, derived from `stream` by the host (NULL: end times stay
   * in end_scratch): comm_slot[v] numbers the nodes that run on a stream other
   * than 0, the only ones whose end time is kept, 0 .. n_comm-1 in any order; -1
   * for the others.  With it, and when 48 B per node, 264 B per storage (plus
   * one) and 512 B per such node (plus two) fit in the 160 KB of a CU's LDS, the
   * walk touches global memory for the orders alone. */
  const int32_t* comm_slot;   /* [n_node] or NULL                                     */
  int32_t n_comm;
} apc_schedule;

/* Replaces estimate_graph_metrics
 * (autoparallel/graph_passes/estimate_graph_metrics.py:30-89; the same timeline
 * as create_execution_trace, graph_passes/debug_helpers.py:336-420) for n_sched
 * orders of the same nodes at once: order[b * n_node + t] is the node scheduled
 * t-th in order b (NULL: the graph's own order, n_sched must be 1).  A compute
 * stream (0) and one stream per communication group advance by dur + 1 us of
 * launch overhead per node; a wait_tensor stalls the compute stream until its
 * collective has ended; peak memory follows torch's MemoryTracker
 * (torch/_inductor/fx_passes/memory_estimator.py: a storage is allocated when
 * its allocator is scheduled and freed at the last scheduled of its readers).
 * times[b * 4 ..] = total_time, compute_time, communication_time,
 * exposed_comm_time; peak[b] = peak_memory.  Scratch, device memory the caller
 * provides and the call may overwrite: end_scratch double[n_sched * n_node],
 * remaining_scratch int32[n_sched * n_storage] (a graph small enough for a
 * CU's LDS is walked from there by schedule_metrics_lds_kernel and leaves one
 * or both untouched; schedule_metrics_kernel uses both).  Every order must be a
 * permutation that schedules a storage's allocator before its readers. */
int apc_schedule_metrics(const apc_schedule* s, const int32_t* order, int64_t n_sched,
                         double* end_scratch, int32_t* remaining_scratch, double* times,
                         int64_t* peak, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* APC_H_ */
