/*
 * C ABI of the host-side plan builder of libmist_search.so: the group descriptors of one tuner
 * call (MistGroupDesc, mist_search.h) and the launch decomposition of the kernels, from the
 * configuration alone.  HOST code only: no device memory, no stream, nothing is launched.
 *
 * The reference does this work in python for every (tensor-parallel size, G, mesh) group:
 *   - create_search_space_for_a_block_layer   mist/analyzer/batched_module_analyzer.py:417-536
 *   - the group loop of IntraStageTuner.tune  mist/analyzer/intra_tuning.py:169-213
 *   - the table look-ups at (b, tp)           mist/analyzer/batched_module_analyzer.py:1216-1297
 *   - the op-latency aggregation              mist/analyzer/batched_module_analyzer.py:324-414
 *   - the pre / post layer scalars            mist/analyzer/batched_module_analyzer.py:777-1138
 *   - the alpha-beta collective model         mist/tools/optimize.py:201-303
 * All arithmetic is float64 in the operation order of the python host side of this package
 * (mist_amd/stage_inputs.py, layer_tables.py, search_space.py, intra_tuning.py), whose
 * descriptors this builder reproduces byte for byte.
 *
 * The layer quantities come from closed forms of the model shape (MistLayerShapes); a plan
 * whose latencies come from an operator database is built by the python host side instead.
 */
#ifndef MIST_PLAN_H
#define MIST_PLAN_H

#include <stdint.h>

#include "mist_search.h"

#ifdef __cplusplus
extern "C" {
#endif

#define MIST_PLAN_MAX_LIST 32    /* tensor-parallel sizes, G candidates, ZeRO flag choices */
#define MIST_PLAN_MAX_BATCH_SIZES 64
#define MIST_PLAN_OP_CLASSES 12

#define MIST_E_PLAN_UNSUPPORTED (-3) /* the request is outside what this builder covers or fails
                                      * one of its checks: the caller builds the plan (and words
                                      * the error, if it is one) on its python path */

/* Efficiency classes of the closed-form operator latencies, in the order of
 * MistLayerShapes.efficiency. */
enum {
  MIST_OP_QKV_GEMM = 0, MIST_OP_ATTN_CORE, MIST_OP_ATTN_SOFTMAX, MIST_OP_OUT_GEMM,
  MIST_OP_FC1_GEMM, MIST_OP_FC2_GEMM, MIST_OP_ACTIVATION, MIST_OP_NORM, MIST_OP_EMBEDDING,
  MIST_OP_LM_HEAD_GEMM, MIST_OP_XENTROPY, MIST_OP_GRAD_ACCUM
};

/* How the pre / post layers are parallelised (tuning.pre_post_strategy,
 * batched_module_analyzer.py:777-845). */
enum {
  MIST_PP_DP = 0,               /* data parallel over the stage's devices, optimizer states sharded */
  MIST_PP_INTRA_NODE_TP_ORE,    /* tp inside a node, dp across nodes, grads + optimizer sharded */
  MIST_PP_INTRA_NODE_TP,        /* ... grads sharded only */
  MIST_PP_PRESET                /* pp_preset = strategy.pre_post_strategy_array */
};

/* Model shape behind the closed-form layer quantities (the stand-in for the reference's three
 * traced LayerInfo objects, mist/analyzer/info.py:120-222). */
typedef struct MistLayerShapes {
  double hidden, heads, kv_heads, ffn, vocab, seq_len;
  double norm_params;      /* parameters of one normalisation layer */
  double opt_mult;         /* optimizer-state bytes per weight byte (info.py:199-212) */
  double bytes_per_param;
  double peak_flops, hbm_bw;
  double efficiency[MIST_PLAN_OP_CLASSES][2]; /* (forward, backward) per op class */
  int32_t flash, gated, abs_pos, tied;
} MistLayerShapes;

typedef struct MistPlanRequest {
  MistLayerShapes layers;
  double gpu_gpu[32];            /* hardware.gpu_gpu_comm_params */
  double memory_capacity_gb;     /* hardware.memory_capacity */
  double wo[MIST_MAX_RATIOS], go[MIST_MAX_RATIOS], oo[MIST_MAX_RATIOS], ao[MIST_MAX_RATIOS];
  double pp_preset[10];
  double scout_tight_fraction;
  int64_t global_batch_size;
  int64_t workspace_rows;        /* rows of the row-term workspace: bound of a batch of groups */
  /* model.num_attention_heads, training.max_sequence_length, model.use_flash_attn as the
   * attention score buffer reads them (batched_module_analyzer.py:1203-1213) */
  int32_t model_heads, model_seq_len, model_flash;
  int32_t num_layers;            /* L */
  int32_t max_pre_saved;         /* P: largest number of pre-saved micro-batches (intra_tuning.py:117-126) */
  int32_t evaluate_all_p;        /* every p of 0..P for every G */
  int32_t exhaustive;            /* the evaluate-every-cell kernel: no scout pass */
  int32_t n_tp, tp_size[MIST_PLAN_MAX_LIST]; /* 0 = none given: the first feasible batch size decides */
  int32_t n_grad_accum, grad_accum[MIST_PLAN_MAX_LIST];
  int32_t n_mesh, mesh_n[MIST_MAX_MESH], mesh_m[MIST_MAX_MESH];
  int32_t n_batch_sizes, batch_size[MIST_PLAN_MAX_BATCH_SIZES];
  int32_t zero_2_and_3, n_flag_choices, flag_choice[MIST_PLAN_MAX_LIST][3];
  int32_t disable_tp;
  int32_t check_shapes;          /* heads, kv heads, ffn and hidden size must split evenly over tp
                                  * (batched_module_analyzer.py:563-578) */
  int32_t n_wo, n_go, n_oo, n_ao, n_pair;
  uint8_t pair_wo[MIST_MAX_PAIRS], pair_go[MIST_MAX_PAIRS];
  int32_t pp_mode;
  /* sizing of the reduce launches and of the scout pass */
  int32_t target_reduce_waves, scout_min_stages, scout_min_pairs, scout_pairs, scout_pair_span,
      scout_tight_pairs;
  /* optional [n_grad_accum][n_mesh][3] = (smallest layer count, largest layer count, number of
   * pre-saved micro-batch values) a caller reads of a (G, mesh); a first entry < 0 = none of it */
  const int32_t *cells_wanted;
} MistPlanRequest;

typedef struct MistPlanResult {
  int32_t n_groups;
  int32_t n_batches;        /* runs of consecutive groups under the workspace bound */
  int32_t max_scout_rows;   /* MistProblem.max_scout_rows */
  int32_t max_group_keys;   /* MistProblem.max_group_keys */
  int64_t total_rows;
  int64_t n_space_rows;     /* rows written to space_rows */
} MistPlanResult;

int mist_sizeof_plan_request(void);

/* Builds every group of a tuner call: entries (t, g, q) = tensor-parallel size x G x mesh in
 * that order; an entry without candidate rows (or outside cells_wanted) has no group.
 *   groups[group_capacity]   zero-filled by the caller; group_capacity >= n_tp * n_grad_accum * n_mesh
 *   space_offset[entries+1], space_rows[entries * MIST_MAX_PAR][6]: the parallelism rows
 *     (b, dp, tp, wre, gre, ore) of every entry, also of those without a group
 *   group_of_entry[entries]: index into groups, -1 = none
 *   terms_prefix, reduce_prefix, scout_prefix [group_capacity+1]: first workgroup of each group
 *     in the row-term, reduce and scout launches
 *   batch_bounds[group_capacity+1]: first group of each batch, then n_groups
 * Returns 0, MIST_E_INVALID (bad sizes) or MIST_E_PLAN_UNSUPPORTED. */
int mist_plan_groups(const MistPlanRequest *request, MistGroupDesc *groups, int32_t group_capacity,
                     int64_t *space_offset, double *space_rows, int32_t *group_of_entry,
                     int32_t *terms_prefix, int32_t *reduce_prefix, int32_t *scout_prefix,
                     int32_t *batch_bounds, MistPlanResult *result);

#ifdef __cplusplus
}
#endif
#endif /* MIST_PLAN_H */
