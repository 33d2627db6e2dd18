// Host-side plan builder: group descriptors and launch decomposition of one tuner call from the
// configuration (see mist_plan.h).  No device code.  Every float64 expression keeps the operand
// order of the python host side it mirrors (left to right, no contraction: the library is built
// with -ffp-contract=off), so that the descriptors are equal byte for byte.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

#include "mist_plan.h"
#include "mist_common.h"

namespace {

constexpr double kMB = 1048576.0;
constexpr double kGB = 1073741824.0;

enum Kind { kPre = 0, kBlock = 1, kPost = 2 };

struct Unsupported {
  const char *why;
};

// ---------------------------------------------------------------------------------------------
// Alpha-beta model of a collective (mist/tools/optimize.py:201-303): sizes 1, 2, 4, >= 8 index a
// 4 x 4 table of (bandwidth GB/s, latency s).
int table_index(double size) {
  if (size == 1) return 0;
  if (size == 2) return 1;
  if (size == 4) return 2;
  if (size >= 8) return 3;
  throw Unsupported{"communication group size is not one of 1, 2, 4, >= 8"};
}

double collective_latency(double factor, double gbytes, double inter, double intra, const double *params) {
  const double ngpu = intra * inter;
  double lat;
  if (gbytes < 1e-5 || ngpu == 1) {
    lat = 0.0;
  } else {
    const int cell = (table_index(inter) * 4 + table_index(intra)) * 2;
    const double k = params[cell], b = params[cell + 1];
    lat = gbytes / k * (ngpu - 1) / ngpu + b;
  }
  return lat * factor;
}
constexpr double kAllReduce = 2.1, kAllGather = 1.0, kReduceScatter = 1.1;

// ---------------------------------------------------------------------------------------------
// Closed-form layer quantities (memory in MB, latencies in seconds).
struct Layers {
  const MistLayerShapes &m;
  const double *gpu_gpu;

  double params(Kind kind, double tp) const {
    const double h = m.hidden;
    if (kind == kBlock) {
      const double kvh = h * m.kv_heads / m.heads;
      const double attn = h * (h + 2.0 * kvh) + h * h;
      const double mlp = (m.gated ? 3.0 : 2.0) * h * m.ffn;
      return (attn + mlp) / tp + 2.0 * m.norm_params;
    }
    if (kind == kPre) {
      double p = m.vocab * h / tp;
      if (m.abs_pos) p = p + m.seq_len * h;
      return p;
    }
    double p = m.norm_params + 0.0 * tp;
    if (!m.tied) p = p + m.vocab * h / tp;
    return p;
  }
  double weights_mb(Kind kind, double tp) const { return params(kind, tp) * m.bytes_per_param / kMB; }
  double opts_mb(Kind kind, double tp) const { return weights_mb(kind, tp) * m.opt_mult; }

  // (saved without checkpointing, transient forward, transient backward) in bytes
  void act_bytes(Kind kind, double b, double tp, double *saved, double *tmp_f, double *tmp_b) const {
    const double s = m.seq_len, h = m.hidden;
    const double bsh = b * s * h;
    if (kind == kBlock) {
      const double kvh = h * m.kv_heads / m.heads;
      double attn = 2.0 * bsh + 2.0 * b * s * (h + 2.0 * kvh) / tp + 2.0 * bsh / tp;
      double attn_tmp;
      if (m.flash) {
        attn = attn + 4.0 * b * m.heads / tp * s;
        attn_tmp = 0.0 * b;
      } else {
        attn = attn + 5.0 * b * m.heads / tp * s * s;
        attn_tmp = 4.0 * b * m.heads / tp * s * s;
      }
      const double n_fc1 = m.gated ? 3.0 : 2.0;
      const double mlp = 2.0 * bsh + 2.0 * n_fc1 * b * s * m.ffn / tp;
      *saved = attn + mlp + 2.0 * bsh;
      *tmp_f = attn_tmp + 2.0 * b * s * m.ffn / tp;
      *tmp_b = attn_tmp + 4.0 * b * s * m.ffn / tp + 4.0 * bsh;
    } else if (kind == kPre) {
      *saved = 8.0 * b * s + 0.0 * tp;
      *tmp_f = 2.0 * bsh;
      *tmp_b = 2.0 * bsh;
    } else {
      const double logits = b * s * m.vocab / tp;
      *saved = 2.0 * bsh + 6.0 * logits;
      *tmp_f = 4.0 * logits;
      *tmp_b = 6.0 * logits;
    }
  }
  double saved_mb(Kind kind, bool ckpt, double b, double tp) const {
    if (ckpt) return 2.0 * b * m.seq_len * m.hidden / kMB + 0.0 * tp;
    double saved, f, bw;
    act_bytes(kind, b, tp, &saved, &f, &bw);
    return saved / kMB;
  }
  double fwd_peak_mb(Kind kind, double b, double tp) const {
    double saved, f, bw;
    act_bytes(kind, b, tp, &saved, &f, &bw);
    return (saved + f) / kMB;
  }
  double bwd_peak_mb(Kind kind, double b, double tp) const {
    double saved, f, bw;
    act_bytes(kind, b, tp, &saved, &f, &bw);
    return (saved + bw) / kMB;
  }
  double output_mb(Kind kind, double b, double tp) const {
    if (kind == kPost) return 4.0 * b * m.seq_len / kMB + 0.0 * tp;
    return 2.0 * b * m.seq_len * m.hidden / kMB + 0.0 * tp;
  }

  // ---- operator latencies: flops / (efficiency * peak), bytes / (efficiency * bandwidth) ----
  struct Op {
    double fwd, bwd, extra_fwd, extra_bwd;
  };
  Op gemm(int cls, double flops, double extra_fwd, double extra_bwd) const {
    const double ef = m.efficiency[cls][0], eb = m.efficiency[cls][1];
    return {flops / (ef * m.peak_flops), 2.0 * flops / (eb * m.peak_flops), extra_fwd, extra_bwd};
  }
  Op membound(int cls, double nbytes, double extra_fwd, double extra_bwd) const {
    const double ef = m.efficiency[cls][0], eb = m.efficiency[cls][1];
    return {nbytes / (ef * m.hbm_bw), 2.0 * nbytes / (eb * m.hbm_bw), extra_fwd, extra_bwd};
  }
  double tp_all_reduce(double nbytes, double inter, double intra) const {
    return collective_latency(kAllReduce, nbytes / kGB, inter, intra, gpu_gpu);
  }
  int op_profiles(Kind kind, double b, double tp, double inter, double intra, Op *ops) const {
    const double s = m.seq_len, h = m.hidden;
    const double act = 2.0 * b * s * h;
    const double ar = tp > 1 ? tp_all_reduce(act, inter, intra) : 0.0;
    int n = 0;
    if (kind == kBlock) {
      const double kvh = h * m.kv_heads / m.heads;
      ops[n++] = membound(MIST_OP_NORM, 2.0 * act, 0.0, 0.0);
      ops[n++] = gemm(MIST_OP_QKV_GEMM, 2.0 * b * s * h * (h + 2.0 * kvh) / tp, 0.0, ar);
      if (m.flash) {
        ops[n++] = gemm(MIST_OP_ATTN_CORE, 4.0 * b * s * s * h / tp, 0.0, 0.0);
      } else {
        ops[n++] = gemm(MIST_OP_ATTN_CORE, 2.0 * b * s * s * h / tp, 0.0, 0.0);
        ops[n++] = membound(MIST_OP_ATTN_SOFTMAX, 6.0 * b * m.heads / tp * s * s, 0.0, 0.0);
        ops[n++] = gemm(MIST_OP_ATTN_CORE, 2.0 * b * s * s * h / tp, 0.0, 0.0);
      }
      ops[n++] = gemm(MIST_OP_OUT_GEMM, 2.0 * b * s * h * h / tp, ar, 0.0);
      ops[n++] = membound(MIST_OP_NORM, 2.0 * act, 0.0, 0.0);
      const double n_fc1 = m.gated ? 2.0 : 1.0;
      ops[n++] = gemm(MIST_OP_FC1_GEMM, 2.0 * n_fc1 * b * s * h * m.ffn / tp, 0.0, ar);
      ops[n++] = membound(MIST_OP_ACTIVATION, (2.0 + n_fc1) * 2.0 * b * s * m.ffn / tp, 0.0, 0.0);
      ops[n++] = gemm(MIST_OP_FC2_GEMM, 2.0 * b * s * m.ffn * h / tp, ar, 0.0);
    } else if (kind == kPre) {
      ops[n++] = membound(MIST_OP_EMBEDDING, 3.0 * act, ar, 0.0);
    } else {
      ops[n++] = membound(MIST_OP_NORM, 2.0 * act, 0.0, 0.0);
      ops[n++] = gemm(MIST_OP_LM_HEAD_GEMM, 2.0 * b * s * h * m.vocab / tp, 0.0, ar);
      const double xe = tp > 1 ? tp_all_reduce(3.0 * 4.0 * b * s, inter, intra) : 0.0;
      ops[n++] = membound(MIST_OP_XENTROPY, 10.0 * b * s * m.vocab / tp, xe, 0.0);
    }
    return n;
  }
  double grad_accum_latency(Kind kind, double tp) const {
    const double nbytes = 3.0 * params(kind, tp) * m.bytes_per_param;
    return nbytes / (m.efficiency[MIST_OP_GRAD_ACCUM][0] * m.hbm_bw);
  }

  // Op-latency aggregation of one layer (batched_module_analyzer.py:324-414): backward clamp,
  // drop of the very short ops, gradient-accumulation term.
  void latency_exec(Kind kind, int64_t b, int64_t tp, double inter, double intra, int64_t G,
                    double out[4]) const {
    Op ops[16];
    const int n = op_profiles(kind, (double)b, (double)tp, inter, intra, ops);
    double fwd_sum = 0, bwd_sum = 0, efwd_sum = 0, ebwd_sum = 0;
    for (int i = 0; i < n; ++i) {
      double fwd = ops[i].fwd, bwd = ops[i].bwd;
      if (bwd != 0 && bwd > 2.3 * fwd) bwd = fwd * 2;
      fwd += ops[i].extra_fwd;
      bwd += ops[i].extra_bwd;
      if (fwd < 5e-5 || bwd < 1e-4) continue;
      fwd_sum += fwd;
      bwd_sum += bwd;
      efwd_sum += ops[i].extra_fwd;
      ebwd_sum += ops[i].extra_bwd;
    }
    bwd_sum += grad_accum_latency(kind, (double)tp) * (double)(G - 1) / (double)G;
    out[0] = fwd_sum, out[1] = bwd_sum, out[2] = efwd_sum, out[3] = ebwd_sum;
  }
};

// get_concrete_mem_partial_states (batched_module_analyzer.py:143-153)
double partial(double full, double shard, double ratio) { return full / shard * (1.0 - ratio); }

bool tame(double v) { return std::isfinite(v) && v >= 0.0; }

struct Builder {
  const MistPlanRequest &r;
  Layers layers;

  explicit Builder(const MistPlanRequest &request) : r(request), layers{request.layers, request.gpu_gpu} {}

  bool shapes_split(int64_t tp) const {
    if (!r.check_shapes) return true;
    const double v[4] = {r.layers.heads, r.layers.kv_heads, r.layers.ffn, r.layers.hidden};
    for (double x : v)
      if ((int64_t)x % tp != 0) return false;
    return true;
  }

  // create_search_space_for_a_block_layer (batched_module_analyzer.py:417-536): the parallelism
  // rows of a (mesh, G) for a tensor-parallel size (0 = the first feasible batch size decides).
  int parallelism_rows(int n, int m, int64_t G, int64_t tp_size, double rows[][6]) const {
    const int64_t num_gpus = (int64_t)n * m;
    const int64_t per_micro_batch = r.global_batch_size / G;
    int count = 0;
    for (int i = 0; i < r.n_batch_sizes; ++i) {
      const int64_t batch = r.batch_size[i];
      if (batch <= 0) throw Unsupported{"batch size candidate <= 0"};
      if (batch > per_micro_batch || per_micro_batch % batch != 0) continue;
      const int64_t dp = per_micro_batch / batch;
      if (dp > num_gpus || num_gpus % dp != 0) continue;
      const int64_t tp = num_gpus / dp;
      if (!shapes_split(tp)) continue;
      if (tp_size == 0) tp_size = tp;
      if (tp_size != tp) continue;
      if (tp_size > m) continue;
      if (r.disable_tp && tp_size > 1) continue;
      const bool one = dp == 1 || !r.zero_2_and_3;
      const int n_flags = one ? 1 : r.n_flag_choices;
      for (int f = 0; f < n_flags; ++f) {
        if (count >= MIST_MAX_PAR) throw Unsupported{"more parallelism rows than a group holds"};
        double *row = rows[count++];
        row[0] = (double)batch, row[1] = (double)dp, row[2] = (double)tp_size;
        row[3] = one ? 0.0 : (double)r.flag_choice[f][0];
        row[4] = one ? 0.0 : (double)r.flag_choice[f][1];
        row[5] = one ? 1.0 : (double)r.flag_choice[f][2];
      }
    }
    return count;
  }

  // MIST_PAR_* fields of one parallelism row from W on: the table look-ups at (b, tp).
  void par_fields(int64_t b, int64_t tp, int m, int64_t G, double *v) const {
    const double fb = (double)b, ftp = (double)tp;
    v[MIST_PAR_W] = layers.weights_mb(kBlock, ftp);
    v[MIST_PAR_G] = layers.weights_mb(kBlock, ftp);
    v[MIST_PAR_O] = layers.opts_mb(kBlock, ftp);
    v[MIST_PAR_RAW_CK] = layers.saved_mb(kBlock, true, fb, ftp);
    v[MIST_PAR_RAW_NOCK] = layers.saved_mb(kBlock, false, fb, ftp);
    v[MIST_PAR_FWD_PEAK] = layers.fwd_peak_mb(kBlock, fb, ftp);
    v[MIST_PAR_BWD_PEAK] = layers.bwd_peak_mb(kBlock, fb, ftp);
    v[MIST_PAR_OUT] = layers.output_mb(kBlock, fb, ftp);
    double gcb = 0.0;
    if (!r.model_flash)  // batched_module_analyzer.py:1203-1213
      gcb = 2 * fb * (double)r.model_heads / ftp * (double)((int64_t)r.model_seq_len * r.model_seq_len) /
            (double)(1024 * 1024);
    v[MIST_PAR_GCB] = gcb;
    const double inter = tp > m ? (double)(tp / m) : 1.0;
    const double intra = tp > m ? (double)m : (double)tp;
    layers.latency_exec(kBlock, b, tp, inter, intra, G, &v[MIST_PAR_EXEC_FWD]);
  }

  double dp_collective(double factor, double mbytes, int64_t dp, int n) const {
    const double inter = dp > n ? (double)n : (double)dp;
    const double intra = dp > n ? (double)(dp / n) : 1.0;
    return collective_latency(factor, mbytes / 1024, inter, intra, r.gpu_gpu);
  }

  // Pre / post layer scalars of a (mesh, G) (batched_module_analyzer.py:777-1138).
  void pre_post(int n, int m, int64_t G, MistGroupDesc *g) const {
    int64_t pp_dp, pp_tp;
    bool wre, gre, ore;
    double pp_wo = 0.0, pp_go = 0.0, pp_oo = 0.0;
    switch (r.pp_mode) {
      case MIST_PP_DP:
        pp_dp = (int64_t)n * m, pp_tp = 1, wre = false, gre = false, ore = true;
        break;
      case MIST_PP_INTRA_NODE_TP_ORE:
      case MIST_PP_INTRA_NODE_TP:
        pp_dp = n, pp_tp = m, wre = false, gre = true, ore = r.pp_mode == MIST_PP_INTRA_NODE_TP_ORE;
        break;
      case MIST_PP_PRESET: {
        const double *a = r.pp_preset;
        pp_dp = (int64_t)a[1], pp_tp = (int64_t)a[2];
        wre = a[3] != 0, gre = a[4] != 0, ore = a[5] != 0;
        pp_wo = a[6], pp_go = a[7], pp_oo = a[8];
        break;
      }
      default:
        throw Unsupported{"pre / post strategy"};
    }
    if (pp_dp <= 0 || pp_tp <= 0) throw Unsupported{"pre / post parallelism <= 0"};
    // floor division of non-negative integers, as python's //
    const int64_t pp_b = r.global_batch_size / G / pp_dp;
    const double fb = (double)pp_b, ftp = (double)pp_tp, fdp = (double)pp_dp;
    const double pre_W = layers.weights_mb(kPre, ftp), pre_G = pre_W, pre_O = layers.opts_mb(kPre, ftp);
    const double pre_states = partial(pre_W, wre ? fdp : 1.0, pp_wo) + partial(pre_G, gre ? fdp : 1.0, pp_go) +
                              partial(pre_O, ore ? fdp : 1.0, pp_oo);
    const double pre_saved = layers.saved_mb(kPre, false, fb, ftp);
    const double post_W = layers.weights_mb(kPost, ftp), post_G = post_W, post_O = layers.opts_mb(kPost, ftp);
    const double post_pO = partial(post_O, ore ? fdp : 1.0, pp_oo);
    g->pp_wre = wre, g->pp_gre = gre;
    g->pre_full_w = pre_W, g->pre_full_g = pre_G;
    g->post_full_w = post_W, g->post_full_g = post_G;
    g->pre_states = pre_states;
    g->pre_saved = pre_saved;
    g->pre_states_and_saved = pre_states + pre_saved;
    g->post_states = post_W + post_G + post_pO;
    g->post_fwd_peak = layers.fwd_peak_mb(kPost, fb, ftp);
    g->post_bwd_peak = layers.bwd_peak_mb(kPost, fb, ftp);
    g->post_output = layers.output_mb(kPost, fb, ftp);
    const double inter = pp_tp > m ? (double)(pp_tp / m) : 1.0;
    const double intra = pp_tp > m ? (double)m : (double)pp_tp;
    double lat[4];
    layers.latency_exec(kPre, pp_b, pp_tp, inter, intra, G, lat);
    g->pre_fwd = lat[0], g->pre_bwd = lat[1];
    layers.latency_exec(kPost, pp_b, pp_tp, inter, intra, G, lat);
    g->post_fwd = lat[0], g->post_bwd = lat[1];
    if (pp_dp == 1) {
      g->pre_ag = g->post_ag = g->pre_rs = g->post_rs = 0.0;
    } else {
      g->pre_ag = dp_collective(kAllGather, pre_W, pp_dp, n);
      g->post_ag = dp_collective(kAllGather, post_W, pp_dp, n);
      g->pre_rs = dp_collective(kReduceScatter, pre_G, pp_dp, n);
      g->post_rs = dp_collective(kReduceScatter, post_G, pp_dp, n);
    }
    const double checked[] = {g->pre_full_w, g->pre_full_g, g->post_full_w, g->post_full_g, g->pre_states,
                              g->pre_saved, g->pre_states_and_saved, g->post_states, g->post_fwd_peak,
                              g->post_bwd_peak, g->post_output, g->pre_fwd, g->pre_bwd, g->post_fwd,
                              g->post_bwd, g->pre_ag, g->pre_rs, g->post_ag, g->post_rs};
    for (double v : checked)
      if (!tame(v)) throw Unsupported{"pre / post layer input not finite and non-negative"};
  }
};

void check_request(const MistPlanRequest &r) {
  auto within = [](int v, int lo, int hi) { return v >= lo && v <= hi; };
  if (!within(r.n_tp, 1, MIST_PLAN_MAX_LIST) || !within(r.n_grad_accum, 1, MIST_PLAN_MAX_LIST) ||
      !within(r.n_mesh, 1, MIST_MAX_MESH) || !within(r.n_batch_sizes, 0, MIST_PLAN_MAX_BATCH_SIZES) ||
      !within(r.n_flag_choices, 0, MIST_PLAN_MAX_LIST))
    throw Unsupported{"list lengths"};
  if (!within(r.n_wo, 1, MIST_MAX_RATIOS) || !within(r.n_go, 1, MIST_MAX_RATIOS) ||
      !within(r.n_oo, 1, MIST_MAX_RATIOS) || !within(r.n_ao, 1, MIST_MAX_RATIOS) ||
      !within(r.n_pair, 0, MIST_MAX_PAIRS))
    throw Unsupported{"ratio list lengths"};
  const double *lists[4] = {r.wo, r.go, r.oo, r.ao};
  const int counts[4] = {r.n_wo, r.n_go, r.n_oo, r.n_ao};
  for (int k = 0; k < 4; ++k)
    for (int i = 0; i < counts[k]; ++i)
      if (!(lists[k][i] >= 0 && lists[k][i] <= 1)) throw Unsupported{"offload ratio outside [0, 1]"};
  for (int i = 0; i < r.n_pair; ++i)
    if (r.pair_wo[i] >= r.n_wo || r.pair_go[i] >= r.n_go) throw Unsupported{"offload pair index"};
  for (int i = 0; i < r.n_grad_accum; ++i)
    if (r.grad_accum[i] <= 0) throw Unsupported{"gradient accumulation count <= 0"};
  for (int i = 0; i < r.n_mesh; ++i)
    if (r.mesh_n[i] <= 0 || r.mesh_m[i] <= 0) throw Unsupported{"mesh extent <= 0"};
  for (int i = 0; i < r.n_tp; ++i)
    if (r.tp_size[i] < 0) throw Unsupported{"tensor-parallel size < 0"};
  if (r.num_layers < 1 || r.max_pre_saved < 0 || r.global_batch_size < 1 || r.workspace_rows < 1 ||
      r.target_reduce_waves < 1 || r.scout_pair_span < 1)
    throw Unsupported{"sizes"};
  const MistLayerShapes &m = r.layers;
  if (!(m.heads > 0) || !(m.hidden > 0)) throw Unsupported{"model shape"};
}

}  // namespace

extern "C" int mist_sizeof_plan_request(void) { return (int)sizeof(MistPlanRequest); }

extern "C" int mist_plan_groups(const MistPlanRequest *request, MistGroupDesc *groups, int32_t group_capacity,
                                int64_t *space_offset, double *space_rows, int32_t *group_of_entry,
                                int32_t *terms_prefix, int32_t *reduce_prefix, int32_t *scout_prefix,
                                int32_t *batch_bounds, MistPlanResult *result) {
  if (!request || !groups || !space_offset || !space_rows || !group_of_entry || !terms_prefix ||
      !reduce_prefix || !scout_prefix || !batch_bounds || !result)
    return mist::fail(MIST_E_INVALID, "mist_plan_groups: null argument");
  const MistPlanRequest &r = *request;
  try {
    check_request(r);
    const int64_t entries = (int64_t)r.n_tp * r.n_grad_accum * r.n_mesh;
    if (group_capacity < entries)
      return mist::fail(MIST_E_INVALID, "mist_plan_groups: %d group slots for %lld entries", group_capacity,
                        (long long)entries);
    const Builder builder(r);
    // tile sizes of the kernels this library was built with
    const int64_t kLcTile = mist_reduce_lc_tile(), kPTile = mist_reduce_p_tile();
    const int64_t kStageRows = mist_reduce_stage_rows(), kTermsBlock = mist_terms_block_rows();
    const int64_t kScoutSplit = mist_reduce_scout_split(), kMaxScoutPairs = mist_max_scout_pairs();
    const int L = r.num_layers, P = r.max_pre_saved;
    const int64_t n_pairs = (int64_t)L * (L + 1) / 2 + L;
    const int lc_tiles_all = (int)((n_pairs + kLcTile - 1) / kLcTile);
    const int n_off = r.n_pair * r.n_oo * r.n_ao;
    int n_groups = 0;
    int64_t space_cursor = 0;
    std::vector<int> n_lc_tiles;
    // ---- the groups: search space, table look-ups, pre / post scalars ----
    for (int t = 0; t < r.n_tp; ++t)
      for (int g = 0; g < r.n_grad_accum; ++g)
        for (int q = 0; q < r.n_mesh; ++q) {
          const int64_t entry = ((int64_t)t * r.n_grad_accum + g) * r.n_mesh + q;
          const int n = r.mesh_n[q], m = r.mesh_m[q];
          const int64_t G = r.grad_accum[g];
          double(*rows)[6] = reinterpret_cast<double(*)[6]>(space_rows + 6 * space_cursor);
          const int n_par = builder.parallelism_rows(n, m, G, r.tp_size[t], rows);
          space_offset[entry] = space_cursor;
          space_cursor += n_par;
          group_of_entry[entry] = -1;
          const int64_t n_rows = (int64_t)n_par * n_off;
          if (n_rows == 0) continue;
          if (n_rows >= (int64_t)1 << 31) throw Unsupported{"a group with 2^31 rows or more"};
          int num_p = (int)std::min<int64_t>(std::min<int64_t>(G, L), P + 1);  // intra_tuning.py:185-193
          if (r.evaluate_all_p) num_p = P + 1;
          int tile_begin = 0, tile_count = lc_tiles_all;
          if (r.cells_wanted) {
            const int32_t *w = r.cells_wanted + 3 * ((int64_t)g * r.n_mesh + q);
            if (w[0] < 0) continue;
            const int64_t l_min = std::max<int64_t>(w[0], 1), l_max = std::min<int64_t>(w[1], L);
            if (l_min > l_max || w[2] < 1) continue;
            num_p = std::min(num_p, (int)w[2]);
            // pairs are numbered l-major: index(l, c) = l (l + 1) / 2 - 1 + c
            const int64_t first = (l_min * (l_min + 1) / 2 - 1) / kLcTile;
            const int64_t last = (l_max * (l_max + 1) / 2 - 1 + l_max) / kLcTile;
            tile_begin = (int)first, tile_count = (int)(last - first + 1);
          }
          MistGroupDesc *d = &groups[n_groups];
          group_of_entry[entry] = n_groups++;
          n_lc_tiles.push_back(tile_count);
          d->g_index = t * r.n_grad_accum + g, d->q_index = q;
          d->num_nodes = n, d->num_gpus_per_node = m;
          d->grad_accum = (int32_t)G, d->num_p = num_p;
          d->n_par = n_par, d->n_pair = r.n_pair, d->n_oo = r.n_oo, d->n_ao = r.n_ao, d->n_off = n_off;
          d->n_rows = n_rows;
          d->lc_tile_begin = tile_begin;
          std::memcpy(d->wo, r.wo, sizeof(double) * r.n_wo);
          std::memcpy(d->go, r.go, sizeof(double) * r.n_go);
          std::memcpy(d->oo, r.oo, sizeof(double) * r.n_oo);
          std::memcpy(d->ao, r.ao, sizeof(double) * r.n_ao);
          std::memcpy(d->pair_wo, r.pair_wo, r.n_pair);
          std::memcpy(d->pair_go, r.pair_go, r.n_pair);
          for (int i = 0; i < n_par; ++i) {
            double *v = d->par[i];
            std::memcpy(v, rows[i], sizeof(double) * 6);
            builder.par_fields((int64_t)rows[i][0], (int64_t)rows[i][2], m, G, v);
            for (int k = 0; k < MIST_PAR_FIELDS; ++k)
              if (!tame(v[k])) throw Unsupported{"layer table value not finite and non-negative"};
          }
          builder.pre_post(n, m, G, d);
        }
    space_offset[entries] = space_cursor;

    // ---- batches of consecutive groups under the workspace bound; rows per chunk per batch ----
    int n_batches = 0;
    for (int first = 0; first < n_groups;) {
      int last = first;
      int64_t rows = 0;
      while (last < n_groups && (last == first || rows + groups[last].n_rows <= r.workspace_rows))
        rows += groups[last++].n_rows;
      batch_bounds[n_batches++] = first;
      int64_t tile_rows = 0;
      for (int i = first; i < last; ++i) {
        const int64_t p_tiles = (groups[i].num_p + kPTile - 1) / kPTile;
        tile_rows += groups[i].n_rows * n_lc_tiles[i] * p_tiles;
      }
      const int64_t waves = std::max<int64_t>((int64_t)r.target_reduce_waves * 64 / kLcTile, 1);
      int64_t rows_per_chunk = (tile_rows + waves - 1) / waves;
      rows_per_chunk = (rows_per_chunk + kStageRows - 1) / kStageRows * kStageRows;
      rows_per_chunk = std::max<int64_t>(256, std::min<int64_t>(16384, rows_per_chunk));
      for (int i = first; i < last; ++i) groups[i].rows_per_chunk = (int32_t)rows_per_chunk;
      first = last;
    }
    batch_bounds[n_batches] = n_groups;

    // ---- decomposition of the launches, scout pass ----
    const double capacity_mb = r.memory_capacity_gb * 1024.0;
    int64_t row_offset = 0, key_offset = 0, terms = 0, reduce = 0, scout_blocks = 0;
    int64_t max_scout_rows = 0, max_group_keys = 0;
    bool any_scout = false;
    for (int i = 0; i < n_groups; ++i) {
      MistGroupDesc *d = &groups[i];
      const int64_t p_tiles = (d->num_p + kPTile - 1) / kPTile;
      d->n_chunks = (int32_t)((d->n_rows + d->rows_per_chunk - 1) / d->rows_per_chunk);
      d->n_lc_tiles = n_lc_tiles[i];
      d->n_p_tiles = (int32_t)p_tiles;
      d->row_offset = row_offset;
      d->key_offset = key_offset;
      row_offset += d->n_rows;
      const int64_t n_keys = (int64_t)d->n_par * d->n_ao * d->n_pair;
      key_offset += n_keys;
      max_group_keys = std::max(max_group_keys, n_keys);
      terms_prefix[i] = (int32_t)terms;
      reduce_prefix[i] = (int32_t)reduce;
      terms += (d->n_rows + kTermsBlock - 1) / kTermsBlock;
      reduce += (int64_t)d->n_chunks * n_lc_tiles[i] * p_tiles;
      // Scout pass: the rows of a few (weight, gradient) offload pairs seed the group's chunks;
      // groups that are small or have few offload pairs go without.
      const int64_t n_stages = (d->n_rows + kStageRows - 1) / kStageRows;
      const bool scout = n_stages >= r.scout_min_stages && d->n_pair >= r.scout_min_pairs &&
                         r.scout_min_stages > 0 && !r.exhaustive;
      int64_t pairs = r.scout_pairs + d->n_pair / r.scout_pair_span;
      double layer_states = INFINITY;
      for (int k = 0; k < d->n_par; ++k)
        layer_states = std::min(layer_states, d->par[k][MIST_PAR_W] + d->par[k][MIST_PAR_G] + d->par[k][MIST_PAR_O]);
      if (capacity_mb < r.scout_tight_fraction * L * layer_states) pairs = std::max<int64_t>(pairs, r.scout_tight_pairs);
      pairs = std::min<int64_t>(std::min<int64_t>(pairs, d->n_pair), kMaxScoutPairs);
      int count = scout ? (int)pairs : 0;
      // the first pair, (0, 0), then evenly spread ones up to the last; distinct
      int picked = 0;
      if (count == 1) {
        d->scout_pair[picked++] = 0;
      } else if (count > 1) {
        for (int k = 0; k < count; ++k) {
          const int16_t pair = (int16_t)((int64_t)k * (d->n_pair - 1) / (count - 1));
          if (picked == 0 || d->scout_pair[picked - 1] != pair) d->scout_pair[picked++] = pair;
        }
      }
      d->scout_stride = picked;
      if (picked > 0) {
        any_scout = true;
        max_scout_rows = std::max(max_scout_rows, (int64_t)d->n_par * d->n_oo * d->n_ao * picked);
      }
    }
    terms_prefix[n_groups] = (int32_t)terms;
    reduce_prefix[n_groups] = (int32_t)reduce;
    for (int i = 0; i < n_groups; ++i) {
      scout_prefix[i] = (int32_t)scout_blocks;
      if (any_scout) scout_blocks += (int64_t)n_lc_tiles[i] * kScoutSplit * groups[i].n_p_tiles;
    }
    scout_prefix[n_groups] = (int32_t)scout_blocks;
    if (terms >= (int64_t)1 << 31 || reduce + scout_blocks >= (int64_t)1 << 31)
      throw Unsupported{"launch decomposition beyond 2^31 workgroups"};
    if (max_scout_rows >= (int64_t)1 << 31 || max_group_keys >= (int64_t)1 << 31)
      throw Unsupported{"scout rows or keys beyond 2^31"};
    result->n_groups = n_groups;
    result->n_batches = n_batches;
    result->max_scout_rows = (int32_t)max_scout_rows;
    result->max_group_keys = (int32_t)max_group_keys;
    result->total_rows = row_offset;
    result->n_space_rows = space_cursor;
    return 0;
  } catch (const Unsupported &u) {
    return mist::fail(MIST_E_PLAN_UNSUPPORTED, "mist_plan_groups: %s", u.why);
  }
}
