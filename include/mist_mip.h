/*
 * C ABI of the stage-assignment search of the `uniform-device-pp-mip` granularity (part of
 * libmist_search.so).  Conventions as in mist_search.h: `d_*` pointers are caller-owned DEVICE
 * memory, structs and the other pointers are HOST memory, `stream` is a hipStream_t passed as
 * void*, return >= 0 / negative MIST_E_* with mist_last_error().
 *
 * Reference: mist/analyzer/inter_tuning_mip.py.  For one gradient-accumulation count G, one
 * stage count S and the uniform mesh of that S, stage i takes j layers (j in layers_min ..
 * layers_max) and one sampled policy k; with stable time T_i and delta time D_i of that choice
 * the reference minimises
 *     (G - 1) * max_i T_i + sum_i T_i + max(0, max_i (D_i - sum_{i' < i} T_i'))
 * subject to sum_i j_i == L with an external MILP solver (PuLP / CBC, :317-400).
 */
#ifndef MIST_MIP_H
#define MIST_MIP_H

#include <stdint.h>

#include "mist_search.h"

#ifdef __cplusplus
extern "C" {
#endif

#define MIST_MIP_CKPT_TUNED 0 /* every ckpt count 0..L is a candidate (inter_tuning_mip.py:471-473) */
#define MIST_MIP_CKPT_FIXED 1 /* only ckpt == fixed_ckpt (:474-481) */
#define MIST_MIP_CKPT_FULL 2  /* only ckpt == layer count of the stage (:482-489) */

#define MIST_MIP_MAX_SAMPLES 64 /* sample_size limit: one wavefront lane per sample */
#define MIST_MIP_MAX_VALUE 1000000.0f /* stands for "infeasible" in the assignment (:39, :527-530) */

typedef struct MistMipShape {
  int32_t num_layers;  /* L */
  int32_t p_dim;       /* extent of the pre-saved-micro-batch axis of the intra-stage tables */
  int32_t sample_size; /* P: policies sampled per table cell (last axis of the tables) */
  int32_t num_stages;  /* S */
  int32_t layers_min, layers_max; /* layer counts a stage may take (:282-290) */
  int32_t ckpt_mode;   /* MIST_MIP_CKPT_* */
  int32_t fixed_ckpt;  /* used by MIST_MIP_CKPT_FIXED */
} MistMipShape;

/* The float64 tables of the intra-stage search for ONE (gradient-accumulation, mesh) pair:
 * variant 0 (middle stages) and 1 (first stage): [p_dim][L][L+1][P]; 2 (last stage): [L][L+1][P];
 * 3 (single stage): [L+1][P].  Device pointers. */
typedef struct MistMipTables {
  const double *stable[4], *delta[4];
} MistMipTables;

int mist_sizeof_mip_shape(void);

/* Device side of preprocess_stable_and_delta_costs (inter_tuning_mip.py:427-535) restricted to
 * the layer counts the assignment can use.  For stage i and layer count j (row r = i * nl +
 * (j - layers_min), nl = layers_max - layers_min + 1) and sample a < P:
 *   - candidates n = (ckpt, policy) of the stage's table row, values rounded to float32
 *     (stage 0 with L layers reads variant 3, the last stage variant 2, stage 0 variant 1 at
 *     p = S - 1, stage i variant 0 at p = S - i - 1; p >= p_dim reads +inf);
 *   - d_index[r][a] = first n minimising d_ratios[a] * x[n] + y[n] in float64, -1 if none is
 *     finite (sample_pareto_frontier / compute_indices, mist/utils/pareto.py:8-85, :124-144);
 *   - d_keep[r][a] = 1 when no a' < a selected the same (x, y) pair (fill_redundant_samples,
 *     pareto.py:158-214);
 *   - d_t_stable / d_t_delta [r][a]: the selected pair with negatives raised to 0 and +inf (or a
 *     slot not kept) replaced by MIST_MIP_MAX_VALUE.
 * One launch; outputs are [S][nl][P]. */
int mist_mip_stage_samples(const MistMipShape *shape, const MistMipTables *tables,
                           const double *d_ratios, float *d_t_stable, float *d_t_delta,
                           int32_t *d_index, uint8_t *d_keep, void *stream);

/* mist_mip_stage_samples for every problem of a search (all G, all stage counts) in ONE launch.
 * items[n_items] (HOST) and d_items (the same array in DEVICE memory, uploaded by the caller):
 * problem i owns workgroups first_block .. first_block + S_i * nl_i - 1 and writes its
 * [S_i][nl_i][P] outputs from element out_offset on; both must continue the list (first_block
 * and out_offset of problem 0 are 0, of problem i + 1 those of i plus its counts); problems
 * without a layer count to sample are left out by the caller. */
typedef struct MistMipBatchItem {
  MistMipShape shape;
  MistMipTables tables;
  int64_t out_offset;
  int32_t first_block, reserved;
} MistMipBatchItem;
int mist_sizeof_mip_batch_item(void);
int mist_mip_stage_samples_batch(const MistMipBatchItem *items, const MistMipBatchItem *d_items,
                                 int n_items, const double *d_ratios, float *d_t_stable,
                                 float *d_t_delta, int32_t *d_index, uint8_t *d_keep,
                                 void *stream);

/* Exact solver for the assignment problem, on the host (replaces the PuLP / CBC call,
 * inter_tuning_mip.py:317-400).  `t_stable`, `t_delta`, `keep` are HOST copies of the arrays
 * above.  Writes the optimal objective and, per stage, the layer count and the sample slot.
 * Entries with (G - 1) * T > best_cost are excluded (:358).  Among equal optima: the smallest
 * max T first, then per state the first minimum in (layer count, slot) order.
 * Returns 1 when an assignment exists, 0 when none does, negative on invalid arguments. */
int mist_mip_solve(const MistMipShape *shape, int grad_accum, double best_cost,
                   const float *t_stable, const float *t_delta, const uint8_t *keep,
                   double *out_cost, int32_t *out_layers, int32_t *out_slot);

/* Pre-fill of the intra-stage tables for a caller that reads the cells of the stage assignment
 * only (the reference allocates whole tables of +inf, mist/analyzer/intra_tuning.py:127-166; an
 * assignment with 30 samples per cell reads a sixth of them): costs +inf and row indices -1 in
 * the table rows of n_regions regions, every other cell is left as it is.
 * regions[n_regions][6] (HOST, and the same array in DEVICE memory as d_regions) =
 *   (table row g, mesh q, smallest layer count, largest layer count, number of pre-saved
 *    micro-batch values p = 0.., first workgroup of the region);
 * a region covers, for its layer counts l, all ckpt counts and samples of variants 0 and 1 at
 * every p below its count (at most p_dim), of variant 2, and of variant 3 when its largest layer
 * count is num_layers; region i + 1 starts at the first workgroup of region i plus its rows
 * (2 * p values * layer counts + layer counts [+ 1]).  Table extents as in MistOutTables:
 * [num_table_rows][num_mesh][p_dim][L][L+1][sample_size] etc. */
int mist_mip_prefill_cells(int num_layers, int p_dim, int sample_size, int num_mesh,
                           int num_table_rows, const int32_t *regions, const int32_t *d_regions,
                           int n_regions, const MistOutTables *tables, void *stream);

/* mist_mip_solve over the problems of whole searches (inter_stage_tune, inter_tuning_mip.py:
 * 131-214: for every G, for every stage count, one assignment bounded by the best cost so far,
 * which starts at MIST_MIP_MAX_VALUE; a strictly smaller cost replaces it).  `n_chains`
 * searches (one per tensor-parallel candidate) of `items_per_chain` problems each, chain c's
 * problems at items[c * items_per_chain ...] in the reference's order; problem i of every chain
 * runs with grad_accum[i]; each problem's samples lie at its out_offset in the three HOST
 * arrays (the layout mist_mip_stage_samples_batch writes).  Chains are solved on a thread each.
 * Per chain: out_cost (MIST_MIP_MAX_VALUE when no problem has an assignment below it), out_item
 * (index of the winning problem inside the chain, -1 = none), out_layers / out_slot
 * [chain][num_layers], the winner's first num_stages entries. */
int mist_mip_solve_chains(const MistMipBatchItem *items, const int32_t *grad_accum,
                          int items_per_chain, int n_chains, const float *t_stable,
                          const float *t_delta, const uint8_t *keep, double *out_cost,
                          int32_t *out_item, int32_t *out_layers, int32_t *out_slot);

#ifdef __cplusplus
}
#endif
#endif /* MIST_MIP_H */
