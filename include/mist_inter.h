/*
 * C ABI of the inter-stage search driver (part of libmist_search.so): the whole search of
 * inter_stage_tune (mist/analyzer/inter_tuning.py:95-217) for the per-mesh recurrence in one
 * call.  Conventions as in mist_search.h; this entry point allocates its own device and pinned
 * host buffers (kept per device for the life of the process) and synchronises `stream` between
 * its dependent batches.
 */
#ifndef MIST_INTER_H
#define MIST_INTER_H

#include <stdint.h>

#include "mist_dp.h"

#ifdef __cplusplus
extern "C" {
#endif

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

#ifdef __cplusplus
}
#endif
#endif /* MIST_INTER_H */
