/*
 * C ABI of the inter-stage pipeline-partition DP (part of libmist_search.so).
 * Conventions as in mist_search.h: `d_*` pointers are caller-owned DEVICE memory, small structs
 * are HOST memory copied into kernel arguments, `stream` is a hipStream_t passed as void*,
 * return 0 / negative MIST_E_* with mist_last_error().
 */
#ifndef MIST_DP_H
#define MIST_DP_H

#include <stdint.h>

#include "mist_search.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Shape of one DP instance family (reference: inter_stage_tune_dp_impl,
 * mist/analyzer/inter_tuning.py:220-355). */
typedef struct MistDpShape {
  int32_t num_layers;   /* L */
  int32_t num_devices;  /* D */
  int32_t num_mesh;     /* Q <= MIST_MAX_MESH, in candidate-list order */
  int32_t p_dim;        /* P+1: extent of the pre-saved-micro-batch axis of the cost tables */
  int32_t max_stages;   /* stage counts 1..max_stages are searched (<= p_dim, <= L) */
  int32_t ckpt_rule;    /* ckpt candidates j of a stage of l layers ending at layer i:
                         * MIST_DP_CKPT_TAIL 0..L-i (inter_tuning.py:315),
                         * MIST_DP_CKPT_STAGE 0..l, MIST_DP_CKPT_ALL only l
                         * (inter_tuning_uniform_device.py:400-404) */
  int32_t free_devices; /* != 0: stages do not consume devices (every stage runs on mesh 0 and the
                         * stage count alone decides feasibility; inter_tuning_uniform_device.py);
                         * num_devices must then be 0 and num_mesh 1 */
  int32_t reserved;
  int32_t mesh_n[MIST_MAX_MESH], mesh_m[MIST_MAX_MESH];
} MistDpShape;

/* float32 stage-cost tables of all gradient-accumulation candidates, C-contiguous per g:
 *   costs, costs_pre : [g][Q][p_dim][L][L+1]   costs_post : [g][Q][L][L+1]   costs_nopp : [g][Q][L+1]
 * g_stride[v] = elements between consecutive g of table v (costs, pre, post, nopp). */
typedef struct MistDpCosts {
  const float *costs, *costs_pre, *costs_post, *costs_nopp;
  /* running minima along the ckpt axis, same layouts: pmin[..][j] = min(costs[..][0..j]) */
  const float *pmin, *pmin_pre, *pmin_post, *pmin_nopp;
  int64_t g_stride[4];
  /* Optional (NULL = absent): the running minima the recurrence reads, re-laid by
   * mist_dp_stage_minima() as [g][p = stage count - 1][Q][triangle over (k, i >= k)], with
   * stage_min_g_stride elements between consecutive g.  With it mist_dp_run() may keep a whole
   * instance in one workgroup's LDS (one launch instead of one per stage count); the results
   * are the same either way. */
  const float *stage_min;
  int64_t stage_min_g_stride;
} MistDpCosts;

#define MIST_DP_CKPT_TAIL 0
#define MIST_DP_CKPT_STAGE 1
#define MIST_DP_CKPT_ALL 2

#define MIST_DP_THRESHOLD 0  /* sum of stage costs subject to cost <= t_max */
#define MIST_DP_BOTTLENECK 1 /* smallest achievable maximum stage cost; t_max is ignored */

int mist_sizeof_dp_shape(void);

/* Builds the float32 DP cost tables of every gradient-accumulation candidate from the float64
 * stable / delta tables of the intra-stage search at sample position `slot`:
 *   cost = (float)stable + (float)delta / (float)G          (float32 arithmetic)
 * This is the combination the reference's uniform search applies (mist/analyzer/
 * inter_tuning_uniform.py:300-316); the reference's DP expects it precomputed in fields its
 * intra tuner no longer emits (mist/analyzer/inter_tuning.py:75-92).
 * d_grad_accum[num_grad_accum]: G per g index.  d_out[v]: variant v table for all g, i.e. the
 * layouts of MistOutTables without the trailing sample axis; d_out_pmin[v]: its running minimum
 * along the ckpt axis (what MistDpCosts.pmin* expects).  tables->index[v], when not NULL, must
 * be the row-index table that belongs to the costs (-1 exactly where they are +inf, as the
 * intra-stage search leaves them): the costs of such cells are then not read. */
int mist_dp_cost_tables(const MistProblem *problem, const MistOutTables *tables,
                        const int32_t *d_grad_accum, int slot, float *const d_out[4],
                        float *const d_out_pmin[4], void *stream);

/* Fills MistDpCosts.stage_min for a DP family: d_out[num_grad_accum][mist_dp_stage_minima_floats()]
 * (max_stages * Q * L(L+1)/2 floats per g).  Entry (g, p, q, k, i) is the smallest cost over the
 * ckpt candidates shape->ckpt_rule admits of the stage k..i on mesh q followed by p stages, i.e.
 * what inter_tuning.py:312-322 compares with t_max first; entries no stage count reaches are
 * +inf.  `costs` needs its eight table pointers and g_stride only. */
int64_t mist_dp_stage_minima_floats(const MistDpShape *shape);
int mist_dp_stage_minima(const MistDpShape *shape, const MistDpCosts *costs, int num_grad_accum,
                         float *d_out, void *stream);

/* Host helper: applies the reference's gap rule (inter_tuning.py:198: skip t when
 * t - last_run < 1e-6, float32 difference compared in float64) to an ascending list of
 * candidate t_max values; writes the kept values to out and returns their count. */
int mist_dp_filter_tmax(const float *sorted_unique, int n, double gap, float *out);

/* Host helper for a walk that does not start at the bottom of the candidate list.  `ascending`
 * holds the candidates in (lo, hi] of one table row (all candidates up to hi when `open_below`).
 * Whether the reference's walk keeps a candidate only depends on the last kept one, and a
 * candidate whose predecessor is at least the gap below it is kept in any case: the walk is
 * restarted at the last such candidate that is <= start_value (the smallest feasible threshold;
 * everything below is infeasible and leaves the scan of inter_tuning.py:189-217 unchanged), or at
 * the first fetched candidate when that lies above start_value and is certain itself.  Writes
 * the kept values from there on and returns their count, or MIST_DP_NO_START when the fetched
 * part holds no certain start (the caller fetches from further below). */
#define MIST_DP_NO_START (-3)
int mist_dp_window_begin(const float *ascending, int n, float lo, int open_below,
                         float start_value, double gap, float *out);

/* mist_dp_window_begin for n_windows walks in one call: window w owns
 * ascending[offsets[w] .. offsets[w + 1]) and writes its kept values to the same range of out;
 * out_count[w] = number kept, or MIST_DP_NO_START. */
int mist_dp_window_begin_many(const float *ascending, const int64_t *offsets, int n_windows,
                              const float *lo, const uint8_t *open_below,
                              const float *start_value, double gap, float *out,
                              int32_t *out_count);

/* t_max candidates of value windows (reference: the sort + scan over every finite stage cost,
 * inter_tuning.py:180-199, restricted to where the scan can get).  Request r selects the finite
 * values v of the costs / with_pre / with_post tables of table row d_rows[r] with
 * d_lo[r] < v <= d_hi[r] (-inf / +inf for open ends).  Selected values are appended unordered to
 * d_out_values with their request number in d_out_request (capacity entries each).
 * d_counts[1 + n_requests], zeroed by the caller: [0] = values selected in total (if larger than
 * capacity the lists are incomplete: call again with larger lists), [1 + r] = finite values of
 * request r above d_hi[r]. */
int mist_dp_select_candidates(const MistDpCosts *costs, int n_requests, const int32_t *d_rows,
                              const float *d_lo, const float *d_hi, float *d_out_values,
                              int32_t *d_out_request, int capacity, int32_t *d_counts,
                              void *stream);

/* The threshold windows of a search and its first scan batch, decided on the device (no
 * counterpart in the reference: its sort + gap walk of inter_tuning.py:180-199 runs on the host
 * over every finite stage cost).  Request r selects the candidates of table row d_rows[r] with
 * d_lo[r] < v <= d_hi[r] as mist_dp_select_candidates does, into a list of its own; a workgroup
 * per request sorts them, finds the start of the walk as mist_dp_window_begin does (the fetch is
 * never open below) for the smallest feasible threshold d_start[r] (+inf: nothing feasible, the
 * request is skipped), walks them with the gap rule and appends the kept thresholds, ascending,
 * to d_kept; of the n_avail kept thresholds at or above d_start[r], min(first_chunk, n_avail)
 * become DP instances, instance k at the mist_dp_first_batch_index(k, ...)-th of them: all if
 * they fit, else the first `first_lead` ones and the rest of the batch spread evenly up to the
 * last one.  The instances are appended to d_inst_tmax / d_inst_row[n_requests * first_chunk]
 * (row -1 in the unused tail: mist_dp_run skips such instances and reports them infeasible).
 *   window_capacity : candidates a request may select (a power of two in [128, 8192])
 *   d_values[n_requests][window_capacity], d_counts[2 + 2 n_requests] : work space
 *   d_meta[n_requests][8] : selected, candidates above d_hi[r], status, kept, offset of the
 *                   kept thresholds in d_kept, kept thresholds below d_start[r], instances,
 *                   offset of the instances
 * status 0 = done; 1 = skipped (d_start[r] = +inf); 2 = more than window_capacity candidates;
 * 3 = no certain start in the window (MIST_DP_NO_START); 4 = nothing kept at or above d_start[r];
 * 5 = d_kept too small.  A caller that meets a status above 1 decides that window on the host
 * (mist_dp_select_candidates + mist_dp_window_begin). */
int mist_dp_windows_first_batch(const MistDpCosts *costs, int n_requests, const int32_t *d_rows,
                                const float *d_lo, const float *d_hi, const float *d_start,
                                double gap, int window_capacity, int first_chunk, int first_lead,
                                float *d_values, int32_t *d_counts, float *d_kept,
                                int kept_capacity, int32_t *d_meta, float *d_inst_tmax,
                                int32_t *d_inst_row, void *stream);
/* Host function: index (among the n_avail kept thresholds of a window from its first feasible
 * one on) of instance k of that window's first scan batch; -1 for k outside the batch. */
int mist_dp_first_batch_index(int k, int n_avail, int first_chunk, int first_lead);

/* Runs n_tmax DP instances at once: one launch per stage count with a thread (or a team of
 * lanes) per (instance, start layer, devices) state, or, for large batches whose state planes fit
 * the LDS of a compute unit and whose costs->stage_min is set, one workgroup per instance.
 * Instance t uses the cost tables of g = d_g_index[t]; g < 0 marks an empty slot of the batch,
 * reported as infeasible (d_best_s -1).
 * MIST_DP_THRESHOLD (reference: inter_stage_tune_dp_impl, inter_tuning.py:220-355):
 *   F(s,k,d) = min over mesh q (n*m <= d), end layer i >= k, ckpt j (shape->ckpt_rule) of
 *              cost(s,k,i,q,j) + F(s-1,i+1,d-n*m)   subject to cost <= d_tmax[t],
 *   float32 adds, strict "<" in the reference's (q, i, j) order.  Outputs per instance:
 *   d_best_s (-1 = infeasible), d_best_sum = F(best_s,0,D), d_stage_max = running max of the
 *   chosen stage costs.
 * MIST_DP_BOTTLENECK: same recurrence with max() in place of "+" and no threshold; d_best_sum
 *   is the smallest threshold for which the instance is feasible (+inf if none) and d_stage_max
 *   the float32 sum of the stage costs of the partition that attains it (so the threshold DP at
 *   that threshold returns a sum no larger).  The reference
 *   finds that point by running the threshold DP for every smaller candidate, all of which
 *   return "infeasible" and change nothing.
 * d_argmin (may be NULL): [n_tmax][max_stages+1][L+1][D+1][4] int32 =
 *   (end layer, n, m, ckpt), pre-filled with -1 by the caller.
 * d_scratch: mist_dp_scratch_floats() floats (four (L+1)(D+1) state planes per instance plus the
 * reachable row range of every device column).
 * For tests the environment variable MIST_DP_FORCE_SCHEDULE (step | fused | plane) overrides the
 * choice of schedule; a shape the forced schedule does not support fails with MIST_E_INVALID. */
int64_t mist_dp_scratch_floats(const MistDpShape *shape, int n_tmax);
int mist_dp_run(const MistDpShape *shape, const MistDpCosts *costs, const float *d_tmax,
                const int32_t *d_g_index, int n_tmax, int mode, int32_t *d_best_s,
                float *d_best_sum, float *d_stage_max, int32_t *d_argmin, float *d_scratch,
                void *stream);

/* mist_dp_run() for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments, results and argument checks as mist_dp_run() without d_scratch: the state planes
 * live in an array built into the library, mist_dp_static_scratch_floats() floats (16 MiB) per
 * GPU, held until the process ends.  Always runs the one-launch-per-stage-count schedule (the
 * one that uses the scratch).  Calls no hipMalloc / hipFree or any other allocating routine.
 * Fails with MIST_E_INVALID when mist_dp_scratch_floats(shape, n_tmax) exceeds the built-in
 * array.  All calls on one GPU share that array: calls that overlap in time on one GPU (two
 * streams, two threads) race and must be serialised by the caller. */
int64_t mist_dp_static_scratch_floats(void);
int mist_dp_run_static(const MistDpShape *shape, const MistDpCosts *costs, const float *d_tmax,
                       const int32_t *d_g_index, int n_tmax, int mode, int32_t *d_best_s,
                       float *d_best_sum, float *d_stage_max, int32_t *d_argmin, void *stream);

/* Partition of every instance of a mist_dp_run() call that recorded back-pointers
 * (reference: the walk of inter_tuning.py:341-355, here on the GPU so that only the partitions
 * travel to the host).  d_path[n_tmax][max_stages][4] int32: stage i of instance t in pipeline
 * order as (end layer, n, m, ckpt), -1 in the unused tail (all -1 if d_best_s[t] < 0).  The
 * stages start at layer 0 and each starts after the previous one's end; a walk that meets an
 * entry the DP did not write stops early, which the caller can tell from the last end layer.
 * d_argmin needs no pre-fill for this. */
int mist_dp_backtrack(const MistDpShape *shape, const int32_t *d_argmin, const int32_t *d_best_s,
                      int n_tmax, int32_t *d_path, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MIST_DP_H */
