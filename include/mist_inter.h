/*
 * C ABI of the inter-stage search driver (part of libmist_search.so): the whole search of
 * inter_stage_tune (mist/analyzer/inter_tuning.py:95-217; with several DP families the one of
 * mist/analyzer/inter_tuning_uniform_device.py:312-367) in one call.  Conventions as in
 * mist_search.h; these entry points allocate their own device and pinned host buffers (kept per
 * device for the life of the process) and synchronise `stream` between their dependent batches.
 */
#ifndef MIST_INTER_H
#define MIST_INTER_H

#include <stdint.h>

#include "mist_dp.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Row-index tables of the intra-stage search (MistOutTables.index of the launch that covers
 * every table row the search uses) and how to address them: what
 * get_solution_from_intra_stage_tuner_output (inter_tuning.py:38-60) reads for a stage. */
typedef struct MistStrategyIndex {
  const int32_t *index[4]; /* DEVICE: [g][Q][p_dim][L][L+1][S] x2, [g][Q][L][L+1][S], [g][Q][L+1][S] */
  int32_t num_layers, p_dim, num_mesh, sample_size;
  int32_t slot;            /* position on the sample axis */
  int32_t mesh_n[MIST_MAX_MESH], mesh_m[MIST_MAX_MESH]; /* the q axis, in candidate-list order */
} MistStrategyIndex;
int mist_sizeof_strategy_index(void);

/* Searches n_instances independent instances (the tensor-parallel candidates of one tune call)
 * over the same n_grad_accum gradient-accumulation candidates, each exactly as the reference does
 * alone: G after G in the given order, the kept thresholds of a G ascending
 * (inter_tuning.py:180-199), "t * G >= best -> next G" (:196-197), strict "<" (:206), the DP of
 * :220-355 per threshold.  Thresholds are evaluated ahead in batches; the sequential rules are
 * replayed on the results, so batching changes the work done, never the outcome.
 *   shape, costs : the DP family (free_devices == 0) and its tables (HOST structs, device
 *                  pointers inside; costs->stage_min set enables the one-workgroup-per-instance
 *                  schedule of mist_dp_run)
 *   rows[n_instances][n_grad_accum] (HOST): table row (index into the g axis of the cost tables)
 *                  of every (instance, G); grad_accum[n_grad_accum] (HOST): the G values
 *   only_best_path != 0: only the instance with the smallest cost (the first of equals) gets
 *                  its partition
 * Outputs (HOST): out_cost[n_instances] (+inf if nothing is feasible), out_g[n_instances] (index
 * of the winning G, -1 if none), out_tmax[n_instances] (its threshold), out_stages[n_instances]
 * (stages of the partition, 0 if not walked), out_path[n_instances][max_stages][4] (stage i as
 * (end layer, n, m, ckpt), -1 beyond), out_stats[4] (may be NULL): DP batches, candidate
 * fetches, candidates fetched, DP instances run. */
int mist_inter_stage_search(const MistDpShape *shape, const MistDpCosts *costs, int n_instances,
                            int n_grad_accum, const int32_t *rows, const int32_t *grad_accum,
                            int only_best_path, double *out_cost, int32_t *out_g, float *out_tmax,
                            int32_t *out_stages, int32_t *out_path, int64_t *out_stats,
                            void *stream);

/* The same search over n_families DP families (shapes[f], costs[f]; HOST arrays): the cost of a
 * (G, threshold) pair is the smallest family total, the first family winning ties, as the
 * reference's loop over stage counts with its strict "<" does
 * (inter_tuning_uniform_device.py:360-367 around the DP of :370-470; one family with
 * free_devices != 0 per admissible stage count).  One family with free_devices == 0 is the
 * search of mist_inter_stage_search.
 *   select_costs : the tables whose costs / with_pre / with_post entries of a table row are the
 *                  threshold candidates of that row (inter_tuning.py:180-186); for the per-mesh
 *                  recurrence the family's own tables
 *   strategy     : may be NULL; with it the strategy rows of the winners' stages are read on the
 *                  GPU in the same round trip as their partitions
 * Additional outputs (HOST): out_family[n_instances] (family of the winning partition, -1 if not
 * walked), out_path[n_instances][S][4] and out_rows[n_instances][S] with S = the largest
 * max_stages of the families (out_rows: row index of stage i's strategy in its group's search
 * space, -1 beyond the partition; may be NULL without `strategy`), out_stats[6] (may be NULL): as
 * above, then the number of stream synchronisations the search waited for and the number of
 * threshold windows the device left to the host (those join the scan one batch later, which
 * changes the batches, not the results). */
int mist_inter_stage_search_families(int n_families, const MistDpShape *shapes,
                                     const MistDpCosts *costs, const MistDpCosts *select_costs,
                                     const MistStrategyIndex *strategy, int n_instances,
                                     int n_grad_accum, const int32_t *rows,
                                     const int32_t *grad_accum, int only_best_path, double *out_cost,
                                     int32_t *out_g, float *out_tmax, int32_t *out_family,
                                     int32_t *out_stages, int32_t *out_path, int32_t *out_rows,
                                     int64_t *out_stats, void *stream);

/* mist_inter_stage_search_families over tables that hold their values only up to a limit per G
 * (the tables an intra-stage call with MistProblem.stage_cost_incumbent leaves: a cell whose
 * minimum is not above estimate / G * (1 + mist_incumbent_slack()) holds it, any other cell
 * holds something above).  No counterpart in the reference: it is the reference's scan
 * (inter_tuning.py:163-217) made safe for such tables.
 *   host_estimate : one double in (pinned) HOST memory that holds the estimate once the work
 *                   queued on `stream` before this call has run (the search reads it after its
 *                   first synchronisation); +inf = the tables are complete, plain search
 *   limit_factor  : limit(G) = *host_estimate * limit_factor / G, at or below which every cell
 *                   the DP reads holds its value ((1 + slack) shortened by a few float32 ulps)
 *   out_unresolved: HOST.  The scan tries no threshold at or above limit(G), and one DP run per
 *                   (instance, G) at limit(G) itself travels with its first batch of requests:
 *                   the number of (instance, G) pairs for which that run finds a partition
 *                   cheaper than the running best the scan of G ended with.  Zero, and a
 *                   returned cost below estimate * limit_factor, means the result is what the
 *                   scan over the complete tables returns: thresholds above limit(G) can then
 *                   only produce partitions with a stage above limit(G), which cost more than
 *                   estimate * limit_factor, or partitions the scan already has.  Otherwise the
 *                   reference's scan may find such a partition at a threshold above limit(G)
 *                   (its threshold candidates leave out single-stage costs and those its gap
 *                   rule drops), which these tables cannot tell: evaluate again on complete
 *                   tables. */
int mist_inter_stage_search_bounded(int n_families, const MistDpShape *shapes,
                                    const MistDpCosts *costs, const MistDpCosts *select_costs,
                                    const MistStrategyIndex *strategy, int n_instances,
                                    int n_grad_accum, const int32_t *rows,
                                    const int32_t *grad_accum, int only_best_path, double *out_cost,
                                    int32_t *out_g, float *out_tmax, int32_t *out_family,
                                    int32_t *out_stages, int32_t *out_path, int32_t *out_rows,
                                    int64_t *out_stats, void *stream, const double *host_estimate,
                                    double limit_factor, int32_t *out_unresolved);

#ifdef __cplusplus
}
#endif
#endif /* MIST_INTER_H */
