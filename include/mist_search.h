/*
 * C ABI of the MI355X configuration-search library (libmist_search.so).
 *
 * Plain pointers and sizes only.  Every pointer named `d_*` is DEVICE memory owned by the
 * caller (the python host side allocates it with torch); `problem` and `tables` are small HOST
 * structs that are copied into the kernel arguments.  Nothing here allocates or frees device
 * memory.  All work is enqueued on the `stream` argument (a hipStream_t passed as
 * void*) and is asynchronous with respect to the host.  Return value: 0 on success, a
 * negative MIST_E_* code otherwise; mist_last_error() gives the message of the calling
 * thread's last failure.
 *
 * The reference implements this path in python/numpy/numba; the reference interface each
 * entry point replaces is cited per function (paths relative to the reference repository).
 */
#ifndef MIST_SEARCH_H
#define MIST_SEARCH_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MIST_MAX_PAR 64     /* parallelism rows (b, dp, tp, ZeRO flags) per group */
#define MIST_MAX_RATIOS 32  /* values per offload-ratio list */
#define MIST_MAX_PAIRS (MIST_MAX_RATIOS * MIST_MAX_RATIOS)
#define MIST_PAR_FIELDS 20
#define MIST_ROW_TERMS 34   /* doubles per candidate row produced by mist_row_terms */
#define MIST_KEY_TERMS 28   /* doubles per (parallelism row, activation ratio, offload pair) of the
                             * key-term workspace of mist_row_terms */
#define MIST_LC_TILE 64     /* (layers, ckpt) pairs per workgroup (one wavefront) of the reduce kernel */
#ifndef MIST_P_TILE
#define MIST_P_TILE 16      /* pre-saved micro-batch values per thread of the reduce kernel */
#endif
#define MIST_MAX_MESH 16    /* device-mesh candidates of the inter-stage DP */
#define MIST_MAX_SCOUT_PAIRS 8 /* offload pairs whose rows the scout pass of a group gathers */
#define MIST_MAX_SAMPLE_BATCH 16 /* alpha samples per mist_eval_reduce_samples call */

#define MIST_E_INVALID (-1) /* argument / shape check failed, nothing was launched */
#define MIST_E_HIP (-2)     /* a HIP runtime call failed */

/* Indices into MistGroupDesc.par[i][...] (all float64). */
enum {
  MIST_PAR_B = 0, MIST_PAR_DP, MIST_PAR_TP, MIST_PAR_WRE, MIST_PAR_GRE, MIST_PAR_ORE,
  MIST_PAR_W,        /* full weights of one block layer at this tp, MB */
  MIST_PAR_G,        /* full grads, MB */
  MIST_PAR_O,        /* full optimizer states, MB */
  MIST_PAR_RAW_CK,   /* saved activations of a checkpointed layer, MB */
  MIST_PAR_RAW_NOCK, /* saved activations without checkpointing, MB */
  MIST_PAR_FWD_PEAK, /* forward peak without checkpointing, MB */
  MIST_PAR_BWD_PEAK, /* backward peak, MB */
  MIST_PAR_OUT,      /* layer output, MB */
  MIST_PAR_GCB,      /* attention score buffer when flash attention is off, MB (else 0) */
  MIST_PAR_EXEC_FWD, MIST_PAR_EXEC_BWD, MIST_PAR_EXTRA_FWD, MIST_PAR_EXTRA_BWD, /* seconds */
  MIST_PAR_RESERVED
};

/* Indices into one candidate row of the row-term workspace (all float64). */
enum {
  MIST_T_S_LAYER_CK = 0, MIST_T_S_LAYER_NOCK, MIST_T_S_FIRST_CK, MIST_T_S_FIRST_NOCK,
  MIST_T_S_LAST_CK, MIST_T_S_LAST_NOCK,
  MIST_T_D_LAYER_CK, MIST_T_D_LAYER_NOCK, MIST_T_D_FIRST_CK, MIST_T_D_FIRST_NOCK,
  MIST_T_D_LAST_CK, MIST_T_D_LAST_NOCK,
  MIST_T_FWD_STATES0, /* 2*(Wbuf+Gbuf) + O // ore_size */
  MIST_T_BWD_STATES0, /* 2*(Wbuf+Gbuf) */
  MIST_T_PWG,         /* partial weights + partial grads */
  MIST_T_PO,          /* partial optimizer states */
  MIST_T_PWGO,        /* (pW + pG) + pO */
  MIST_T_S_CK, MIST_T_S_NOCK, MIST_T_D_CK, MIST_T_D_NOCK,
  MIST_T_MF_BASE,     /* memory_factor_for_pp + 0.01 */
  MIST_T_MF_PP,       /* memory_factor + 0.025 */
  MIST_T_MF,          /* memory_factor */
  MIST_T_FWD_PEAK, MIST_T_BWD_PEAK, MIST_T_OUT, MIST_T_GCB,
  MIST_T_NAG_CK, MIST_T_NAG_NOCK, MIST_T_NRS_CK, MIST_T_NRS_NOCK,
  MIST_T_OPB,         /* max(post_bwd - extra_pre_bwd_not_last_ck, 0) */
  MIST_T_RD           /* raw_saved_nock - saved_nock */
};

/* Problem-wide constants (one tuner call = one tp candidate over all (G, mesh) groups). */
typedef struct MistProblem {
  double gpu_gpu[32];      /* hardware.gpu_gpu_comm_params: [inter 1,2,4,8][intra 1,2,4,8](k GB/s, b s) */
  double cpu_gpu[2];       /* hardware.cpu_gpu_comm_params (k, b): CPU -> GPU */
  double gpu_cpu[2];       /* hardware.gpu_cpu_comm_params (k, b): GPU -> CPU */
  double interf_factor[11][4]; /* per mask (4-way, 4x 3-way, 6x 2-way): factor per resource, 1 outside the mask */
  double mem_cap_mb;       /* hardware.memory_capacity(*0.88) * GB / MB */
  double frag_factor;      /* fragmentation term of the memory factor */
  int32_t num_layers;      /* L: layer candidates 1..L, ckpt candidates 0..L */
  int32_t p_dim;           /* P+1: extent of the pre-saved-micro-batch axis of the tables */
  int32_t sample_size;     /* S: extent of the trailing sample axis of the tables */
  int32_t num_grad_accum;  /* extent of the g axis */
  int32_t num_mesh;        /* extent of the q axis */
  int32_t adv_first_block; /* enable_advanced_opt_in_first_block */
  int32_t max_scout_rows;  /* largest n_par * n_oo * n_ao * scout_stride of the call's groups with a
                            * scout pass; 0 = unknown (mist_intra_stage_eval then runs the row
                            * terms and the scout pass one after the other) */
  int32_t max_group_keys;  /* largest n_par * n_ao * n_pair of the call's groups; 0 = unknown
                            * (mist_row_terms then evaluates every row on its own) */
  /* Optional (NULL = none; sample_size 1 only, where a cell's objective is its stage cost): one
   * double in device memory, an estimate of the cost of the best pipeline the caller's
   * inter-stage search returns (+inf before the first call).  The scout pass lowers it to the
   * cost of the best partition into equal stages on equal meshes that its seeds allow; the main
   * launch (and the scout pass itself, with the value it finds) then does not look for stage
   * costs above
   *     bound(G) = incumbent / G * (1 + mist_incumbent_slack()).
   * A cell whose minimum is not above bound(G) holds its minimum and row as always; any other
   * cell holds some value above it (a seed, or +inf / -1), not necessarily its minimum.
   * The reference's scan tries thresholds t with t * G < best (inter_tuning.py:196-197), so
   * below limit(G) = incumbent * (1 + slack) * (1 - 1e-5) / G it reads the same values, in the
   * same order, as from the full tables; what it does above that limit on the full tables these
   * tables cannot tell.  mist_inter_stage_search_bounded (mist_inter.h) is the search for them:
   * it stays below the limit and reports when that leaves the result uncertain, in which case
   * (or when the result is not below incumbent * (1 + slack) * (1 - 1e-5)) the caller
   * evaluates again without the incumbent. */
  double *stage_cost_incumbent;
  int32_t incumbent_num_devices; /* devices of the cluster: stages = this / (n * m of the group) */
  int32_t incumbent_ckpt_rule;   /* ckpt counts the search admits for a stage that ends at layer
                                  * i with l layers: 0 = 0..min(l, L - i) (inter_tuning.py:315),
                                  * 1 = 0..l, 2 = l only (inter_tuning_uniform_device.py:400-404) */
  int32_t incumbent_first_estimate; /* != 0: before its scout pass the call forms a first estimate
                                  * of the same pipeline cost from about a thousand rows per
                                  * group, and the scout pass, too, leaves out stage costs above
                                  * bound(G) of the estimate it finds in place.  For the first call
                                  * after the incumbent was set to +inf; later calls of the same
                                  * search (further groups) read what the earlier ones left. */
  int32_t reserved0;
} MistProblem;

/* One (gradient-accumulation steps, device mesh) group = one call of the reference's
 * batched_tune_best_latency_for_stage (mist/analyzer/batched_module_analyzer.py:581-684).
 * Candidate rows are never materialised: row r decodes as
 *   par = r / n_off,  off = r % n_off,  pair = off / (n_oo*n_ao),
 *   oo  = (off / n_ao) % n_oo,  ao = off % n_ao,  (wo, go) = (pair_wo[pair], pair_go[pair]),
 * i.e. itertools.product(wo, go, oo, ao) minus (wo > 0 and go == 0), parallelism-major
 * (batched_module_analyzer.py:490-534). */
typedef struct MistGroupDesc {
  int32_t g_index, q_index;     /* position in the (g, q) axes of the output tables */
  int32_t num_nodes, num_gpus_per_node; /* stage mesh (n, m) */
  int32_t grad_accum;           /* G */
  int32_t num_p;                /* pre-saved micro-batch candidates 0..num_p-1 */
  int32_t n_par, n_pair, n_oo, n_ao, n_off;
  int32_t pp_wre, pp_gre;       /* ZeRO flags of the pre/post layer strategy */
  int32_t rows_per_chunk, n_chunks, n_lc_tiles, n_p_tiles; /* decomposition of the reduce kernel */
  int32_t lc_tile_begin;        /* the group's n_lc_tiles tiles of 64 (layers, ckpt) pairs start at
                                 * this tile of the pair list: 0 with all tiles for the whole
                                 * tables; a caller that reads a range of layer counts only (the
                                 * stage assignment of inter_tuning_mip.py:282-290) evaluates the
                                 * tiles that hold it, the cells of the other tiles keep their
                                 * pre-filled +inf / -1 */
  int32_t scout_stride;         /* reduce kernel: 0 = no scout pass for this group; m >= 1 = the
                                 * scout pass reduces the rows of the m (weight, gradient) offload
                                 * pairs scout_pair[0 .. m-1] (n_par * n_oo * n_ao rows each) */
  int16_t scout_pair[MIST_MAX_SCOUT_PAIRS]; /* indices into the pair list, distinct */
  int64_t n_rows;               /* n_par * n_off */
  int64_t row_offset;           /* first row of this group in the row-term workspace */
  int64_t key_offset;           /* first key of this group in the key-term workspace: keys are
                                 * (par * n_ao + ao) * n_pair + pair, n_par * n_ao * n_pair per group */
  double par[MIST_MAX_PAR][MIST_PAR_FIELDS];
  double wo[MIST_MAX_RATIOS], go[MIST_MAX_RATIOS], oo[MIST_MAX_RATIOS], ao[MIST_MAX_RATIOS];
  uint8_t pair_wo[MIST_MAX_PAIRS], pair_go[MIST_MAX_PAIRS];
  /* pre / post layer scalars (batched_module_analyzer.py:777-1138) */
  double pre_full_w, pre_full_g, post_full_w, post_full_g;      /* MB */
  double pre_states, pre_saved, pre_states_and_saved;            /* MB */
  double post_states, post_fwd_peak, post_bwd_peak, post_output; /* MB */
  double pre_fwd, pre_bwd, post_fwd, post_bwd;                   /* s */
  double pre_ag, pre_rs, post_ag, post_rs;                       /* s, 0 when the pre/post dp size is 1 */
} MistGroupDesc;

/* Output tables of one tuner call, float64 costs and int32 row indices, laid out like the
 * reference's IntraStageTuner tables (mist/analyzer/intra_tuning.py:127-166):
 *   base, with_pre : [g][q][p_dim][L][L+1][S]
 *   with_post      : [g][q][L][L+1][S]
 *   no_pp          : [g][q][L+1][S]
 * The caller pre-fills costs with +inf and indices with -1; only the cells the reference
 * writes are written. */
typedef struct MistOutTables {
  double *stable[4], *delta[4];
  int32_t *index[4];
} MistOutTables;

/* Library identification and error text. */
const char *mist_version(void);
const char *mist_last_error(void);
int mist_sizeof_problem(void);
double mist_incumbent_slack(void); /* see MistProblem.stage_cost_incumbent */
int mist_sizeof_group(void);
int mist_reduce_p_tile(void); /* MIST_P_TILE the library was built with */
int mist_reduce_lc_tile(void); /* MIST_LC_TILE the library was built with */
int mist_reduce_scout_split(void); /* scout workgroups per (group, (l, c) tile, p tile) */
int mist_workspace_oo_tile(void);  /* optimizer-ratio tile T of the workspace order (mist_row_terms) */
int mist_terms_block_rows(void); /* candidate rows per workgroup of mist_row_terms */
int mist_reduce_stage_rows(void); /* rows per LDS stage; rows_per_chunk must be a multiple */
int mist_max_sample_batch(void); /* MIST_MAX_SAMPLE_BATCH the library was built with */
int mist_key_terms_per_key(void); /* MIST_KEY_TERMS the library was built with */
int mist_max_scout_pairs(void);  /* MIST_MAX_SCOUT_PAIRS the library was built with */
/* doubles of the stage-summary workspace for `total_rows` workspace rows in `n_groups` groups */
int64_t mist_stage_floor_doubles(int64_t total_rows, int n_groups);
/* doubles of the key-term workspace for `total_keys` keys (sum of n_par * n_ao * n_pair) */
int64_t mist_key_terms_doubles(int64_t total_keys);

/* Row-invariant terms of every candidate row: decodes the row index, evaluates the alpha-beta
 * communication terms, the 36 interference evaluations and the memory pieces that do not
 * depend on (layers, ckpt, pre-saved micro-batches).
 * Replaces batched_stage_analyze lines 1144-2162 of mist/analyzer/batched_module_analyzer.py
 * (with predict_gpu_gpu_comm_latency / predict_cpu_gpu_comm_latency /
 * interference_estimate_for_one_group of mist/tools/optimize.py:201-303,459-470,1012-1122).
 * d_block_prefix[n_groups+1]: first workgroup of each group, mist_terms_block_rows() rows per
 * workgroup.
 * d_row_terms: [total_rows][MIST_ROW_TERMS] float64.  Within a group the workspace is ordered
 *   position = (par * n_ao + ao) * n_oo * n_pair + t * T * n_pair + pair * w + oo % T
 * with T = mist_workspace_oo_tile(), t = oo / T and w = min(T, n_oo - t * T): per (par, ao) the
 * optimizer ratios in tiles of T, pair by pair inside a tile (rows of similar latency and memory
 * footprint next to each other, which the reduce kernel's per-stage bound relies on for speed,
 * not for correctness); all results carry reference row numbers.
 * d_stage_floor: mist_stage_floor_doubles() float64, written here and read by mist_eval_reduce:
 * per stage of mist_reduce_stage_rows() workspace rows the term-wise minimum of the latency and
 * memory terms (the pseudo row that bounds every row of the stage from below).
 * d_key_terms: mist_key_terms_doubles() float64 or NULL.  28 of a row's 36 interference
 * evaluations do not depend on its optimizer-offload ratio; with this workspace (and
 * MistProblem.max_group_keys, MistGroupDesc.key_offset set) a first kernel evaluates them once
 * per (parallelism row, activation ratio, offload pair) and the rows read them; without it every
 * row evaluates all 36.  Same operations on the same operands either way: identical row terms.
 * Fails with MIST_E_INVALID when an interference factor of `problem` is not positive and finite
 * (the kernel peels two overlapping resources with one division and takes 0 / f == +0 for the
 * other one). */
int mist_row_terms(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                   const int32_t *d_block_prefix, int n_blocks, double *d_row_terms,
                   double *d_stage_floor, double *d_key_terms, void *stream);

/* Per (group, row chunk, (l, c) tile, p tile): evaluates latency and memory per cell, applies
 * the memory mask and keeps the running lexicographic (cost, row) minimum per bucket.
 * Replaces the two hot loops of batched_stage_analyze (batched_module_analyzer.py:2218-3106)
 * and compute_indices (mist/utils/pareto.py:124-144) for one ratio r = alpha/(1-alpha).
 * d_block_prefix[n_groups+1]: first workgroup of each group; a group owns
 * n_lc_tiles*n_p_tiles*n_chunks workgroups ordered (chunk, lc_tile, p_tile), p_tile fastest.
 * Optional scout pass (n_scout_blocks > 0): d_scout_prefix[n_groups+1] gives each group
 * n_lc_tiles*n_p_tiles*mist_reduce_scout_split() workgroups that first reduce the rows of the
 * group's scout pairs (MistGroupDesc.scout_stride; the search's winners sit almost exclusively
 * on rows without weight / gradient offloading; a small kernel then combines the slabs of a
 * tile's scout workgroups into the first of them); every chunk then starts from those minima (they
 * belong to real rows of the group, so the result is unchanged) and lets far fewer rows through
 * to the memory model.
 * d_partial_cost / d_partial_index: [n_blocks + n_scout_blocks][2*MIST_P_TILE+2][MIST_LC_TILE];
 * the first n_blocks slabs are the per-chunk results mist_finalize reads.  A chunk other than
 * the first of its tile whose minima are still its seeds does not write its slab: it stores -2
 * as the slab's first row index (rows are >= -1) and mist_finalize skips the slab; the first
 * chunk always writes and carries the seeds. */
int mist_eval_reduce(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                     const int32_t *d_block_prefix, int n_blocks,
                     const int32_t *d_scout_prefix, int n_scout_blocks,
                     const double *d_row_terms, const double *d_stage_floor, double ratio,
                     double *d_partial_cost, int32_t *d_partial_index, void *stream);

/* First estimate of MistProblem.stage_cost_incumbent, the step mist_eval_reduce takes before its
 * scout pass when problem->incumbent_first_estimate is set: for every group with a scout pass
 * whose mesh divides the cluster into S equal stages of L / S layers, about a thousand of its
 * scout rows (every parallelism row of every scout pair, activation / optimizer ratios from the
 * first on) are evaluated at that layer count for every ckpt count the caller's search admits
 * (same cells, latencies and memory tests as the tables: batched_module_analyzer.py:2165-2216,
 * 2755-2834, 2866-2923, 2946-3106), the cheapest feasible cost of each stage is kept, and
 * sum + (G - 1) * largest (inter_tuning.py:342) lowers *stage_cost_incumbent.  Needs the row terms
 * of the scout rows (mist_row_terms).  Scratch: the first 4096 doubles of each such group's scout
 * slabs, d_partial_cost + (n_blocks + d_scout_prefix[group]) slabs, which a later scout pass
 * overwrites. */
int mist_stage_cost_first_estimate(const MistProblem *problem, const MistGroupDesc *d_groups,
                                   int n_groups, const int32_t *d_scout_prefix, int n_blocks,
                                   const double *d_row_terms, double ratio, double *d_partial_cost,
                                   void *stream);

/* mist_eval_reduce + mist_finalize for n_samples <= MIST_MAX_SAMPLE_BATCH ratios of the same
 * row terms (reference: the S samples of one compute_indices call, mist/utils/pareto.py:124-144):
 * the scout passes of all samples run as ONE launch (a single one fills a tenth of the GPU), then
 * the main launches, each seeded from its sample's scout slabs, and the finalize launches into
 * sample position sample_index[i], `main_batch` samples per launch (1 <= main_batch <= n_samples;
 * the wavefronts of one sample's tail then run beside the next sample's).  `ratios` and
 * `sample_index` are HOST arrays.
 * d_partial_cost / d_partial_index: [main_batch * n_blocks + n_samples * n_scout_blocks] slabs. */
int mist_eval_reduce_samples(const MistProblem *problem, const MistGroupDesc *d_groups,
                             int n_groups, const int32_t *d_block_prefix, int n_blocks,
                             const int32_t *d_scout_prefix, int n_scout_blocks,
                             const double *d_row_terms, const double *d_stage_floor,
                             const double *ratios, const int32_t *sample_index, int n_samples,
                             int main_batch, double *d_partial_cost, int32_t *d_partial_index,
                             const MistOutTables *tables, void *stream);

/* mist_row_terms + mist_eval_reduce_samples for ALL n_samples ratios of a tuner call (any
 * number; batches of `sample_batch` <= MIST_MAX_SAMPLE_BATCH, main launches of `main_batch` <=
 * sample_batch samples), with the small launches moved out of the way of the large ones: the
 * scout pass of the first batch runs on the library's second stream beside the row terms of the
 * rows it does not gather (as in mist_intra_stage_eval), and the scout pass of batch b + 1 beside
 * the main launches of batch b, into the other of two scout regions.  Same tables as the calls
 * it replaces (reference: the S samples of one compute_indices call per group,
 * mist/utils/pareto.py:124-144).  `ratios` and `sample_index` are HOST arrays of n_samples.
 * d_partial_cost / d_partial_index: [main_batch * n_reduce_blocks + 2 * sample_batch *
 * n_scout_blocks] slabs.  Without a scout pass (n_scout_blocks == 0 or
 * problem->max_scout_rows == 0) the calls it replaces run one after the other on `stream`. */
int mist_intra_stage_eval_samples(const MistProblem *problem, const MistGroupDesc *d_groups,
                                  int n_groups, const int32_t *d_terms_block_prefix,
                                  int n_terms_blocks, const int32_t *d_reduce_block_prefix,
                                  int n_reduce_blocks, const int32_t *d_scout_prefix,
                                  int n_scout_blocks, double *d_row_terms, double *d_stage_floor,
                                  double *d_key_terms, double *d_partial_cost,
                                  int32_t *d_partial_index, const double *ratios,
                                  const int32_t *sample_index, int n_samples, int sample_batch,
                                  int main_batch, const MistOutTables *tables, void *stream);

/* mist_eval_reduce with every cell evaluated: each (row, layers, ckpt) through the latency and
 * memory model and each pre-saved micro-batch value through the reference's feasibility test
 * (batched_module_analyzer.py:2218-3106, pareto.py:124-144 as written, cell by cell), no scout
 * pass, no sieves.  Same workgroup decomposition (d_block_prefix, n_blocks) and slab layout as
 * the main launch of mist_eval_reduce; every slab is written.  The reference point the pruned
 * search is tested and measured against: identical tables, ~20x the time. */
int mist_eval_reduce_exhaustive(const MistProblem *problem, const MistGroupDesc *d_groups,
                                int n_groups, const int32_t *d_block_prefix, int n_blocks,
                                const double *d_row_terms, double ratio, double *d_partial_cost,
                                int32_t *d_partial_index, void *stream);

/* Combines the per-chunk partial minima (smallest cost, lowest row among equals),
 * recomputes stable / delta of the winning row and scatters into the output tables at sample
 * position `sample_index`, reproducing which cells the reference leaves unwritten
 * (batched_module_analyzer.py:2819-2834, 2915-2923, 3021-3033, 3103-3106). */
int mist_finalize(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                  const int32_t *d_block_prefix, const double *d_row_terms,
                  const double *d_partial_cost, const int32_t *d_partial_index,
                  int sample_index, const MistOutTables *tables, void *stream);

/* mist_row_terms (when `compute_terms` != 0) + mist_eval_reduce + mist_finalize for one ratio:
 * the device side of IntraStageTuner.tune (mist/analyzer/intra_tuning.py:169-282) for one tp
 * candidate and one sample.  d_key_terms: as for mist_row_terms, may be NULL. */
int mist_intra_stage_eval(const MistProblem *problem, const MistGroupDesc *d_groups,
                          int n_groups, const int32_t *d_terms_block_prefix, int n_terms_blocks,
                          const int32_t *d_reduce_block_prefix, int n_reduce_blocks,
                          const int32_t *d_scout_prefix, int n_scout_blocks, double *d_row_terms,
                          double *d_stage_floor, double *d_key_terms, double *d_partial_cost,
                          int32_t *d_partial_index, double ratio, int sample_index,
                          int compute_terms, const MistOutTables *tables, void *stream);

/* Analysis path: what batched_stage_analyze(get_best_solution=False) reports
 * (mist/analyzer/batched_module_analyzer.py:2788-2803, 2876-2892, 2980-2996, 3063-3079) for given
 * strategy rows, without the memory mask.  d_requests: [n_requests][5] int32 = (group, workspace
 * position of the row within the group, layers l, ckpt layers c <= l, pre-saved micro-batches p);
 * d_row_terms as written by mist_row_terms.  d_out: [n_requests][MIST_ANALYZE_FIELDS] float64 =
 * for the variants middle stage, first stage (with_pre), last stage (with_post) and single stage
 * (pre_and_post), five values each: stable latency, delta latency, stable + delta / G, forward
 * peak MB, backward peak MB; then the module-level memory of the cell that get_extra_info
 * reports (:2401-2749): forward states, backward states, saved activations of one micro-batch.
 * The last two variants are evaluated with the peaks at the request's p; the reference reports
 * them for p == 0 only.  An invalid request yields NaN. */
#define MIST_ANALYZE_REQUEST_FIELDS 5
#define MIST_ANALYZE_FIELDS 23
int mist_stage_analyze(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                       const double *d_row_terms, const int32_t *d_requests, int n_requests,
                       double *d_out, void *stream);

/* What the row terms fold together, for the debugging entries of the reference's per-cell
 * dictionaries (get_extra_info, mist/analyzer/batched_module_analyzer.py:2401-2749): swap and
 * collective latencies (:1310-1408), the communication operands of the four phases without the
 * activation swaps (:1432-1452, 1646-1670), the full weight / gradient buffers (:2120-2141),
 * the partial weights / gradients, and the five members (layer, first layer, last layer, extra
 * before, extra after) of the eight latency families (:1453-1902).
 * d_requests: [n_requests][2] int32 = (group, workspace position of the row within the group);
 * d_out: [n_requests][MIST_DIAG_FIELDS] float64, NaN for an invalid request. */
enum MistDiagField {
  MIST_DG_SO_W, MIST_DG_SI_W, MIST_DG_SO_G, MIST_DG_SI_G, MIST_DG_SO_O, MIST_DG_SI_O,
  MIST_DG_SO_A_CK, MIST_DG_SI_A_CK, MIST_DG_SO_A_NOCK, MIST_DG_SI_A_NOCK, /* swap out / in, s */
  MIST_DG_AG_W, MIST_DG_RS_G, MIST_DG_AR_G, /* all-gather weights, reduce-scatter / all-reduce grads */
  MIST_DG_WBUF, MIST_DG_GBUF, MIST_DG_PW, MIST_DG_PG, /* MB */
  /* gpu->cpu, cpu->gpu, gpu<->gpu operands: forward first / later micro-batch, backward (the
   * first two are the same for the last and the other micro-batches) last / not last */
  MIST_DG_G2C_F0, MIST_DG_C2G_F0, MIST_DG_G2G_F0, MIST_DG_G2C_F1, MIST_DG_C2G_F1, MIST_DG_G2G_F1,
  MIST_DG_G2C_B, MIST_DG_C2G_B, MIST_DG_G2G_B0, MIST_DG_G2G_B1,
  /* 8 families x (layer, first, last, extra_pre, extra_post): forward first micro-batch without /
   * with ckpt, forward later, backward last micro-batch, backward not last */
  MIST_DG_FAMILIES
};
#define MIST_DIAG_FIELDS (MIST_DG_FAMILIES + 40)
int mist_row_diagnostics(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                         const int32_t *d_requests, int n_requests, double *d_out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MIST_SEARCH_H */
