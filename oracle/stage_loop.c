/* Oracle (test infrastructure): plain-C form of the loops over (ckpt layers c, pre-saved
 * micro-batches p) of the reference's `batched_stage_analyze` with `get_best_solution=True`
 * (mist/analyzer/batched_module_analyzer.py:2165-2216 get_latencies, :2233-2355 pre / post
 * additions, :2358-2385 saved activations, :2755-3106 peaks, masks, reduction and the writes)
 * together with the argmin scan `compute_indices` (mist/utils/pareto.py:124-144).
 *
 * The numpy oracle (oracle/stage.py) evaluates whole (layers, rows) arrays per (c, p); one group
 * of the largest benchmark plans keeps a core busy for up to an hour that way.  This file
 * evaluates the same expressions cell by cell - every sum in the operand order numpy applies,
 * float32 rounding where the reference rounds (:2212-2213), float64 elsewhere, no contraction
 * (-ffp-contract=off) - so that its tables equal the numpy oracle's bit for bit.  It is held to
 * that by tests/test_oracle_stage_c.py (randomised small plans, all four variants, several
 * samples) and by the digests of whole benchmark groups that the numpy oracle wrote into
 * tests/golden/search_tables_plan*.json.
 *
 * Everything that does not depend on (l, c, p) - the row-invariant latency families and memory
 * terms - is computed by oracle/stage.py in numpy and handed over as float64 arrays of n_rows.
 *
 * Build: gcc -O3 -mavx2 -ffp-contract=off -fopenmp -shared -fPIC (oracle/stage_c.py).
 * One task = one (l, c) pair; tasks are spread over OpenMP threads.
 *
 * -DMIST_ORACLE_FUSED (a second library, oracle/stage_c.py `fused=True`) evaluates the objective
 * `r * x + y` of the argmin scan as ONE fused multiply-add: the reference compiles that scan with
 * numba `fastmath=True`, which permits the contraction, and no reference-held value says which
 * form its binary takes.  tests/test_oracle_stage_c.py compares the two forms' winners.  */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef __AVX2__
#include <immintrin.h>
#endif

#define BLOCK 512

typedef struct {
  int64_t n_rows;
  int32_t L;        /* num_layers_candidates = 1..L */
  int32_t C;        /* num_ckpt_layers_candidates = 0..C */
  int32_t n_p;      /* pre_saved_micro_batches_candidates = 0..n_p-1 */
  int32_t S;        /* samples */
  int32_t G;        /* gradient accumulation steps */
  int32_t pp_wre;   /* pre / post layer strategy shards weights ... */
  int32_t pp_gre;   /* ... gradients */
  int32_t pad_;
  const double *ratios; /* [S] alpha / (1 - alpha) */
  /* per row, [0] = without ckpt, [1] = with ckpt (stage.py `lat`) */
  const double *s_layer[2], *s_first[2], *s_last[2];
  const double *d_layer[2], *d_first[2], *d_last[2];
  /* per row memory terms (MB) */
  const double *T0;    /* 2 (Wbuf + Gbuf) + O // ore_size */
  const double *T1;    /* 2 (Wbuf + Gbuf) */
  const double *pWG;   /* pW + pG */
  const double *pO;
  const double *pWGO;  /* pW + pG + pO */
  const double *S_sav[2], *D_sav[2]; /* saved activations kept / offloaded, [nock, ck] */
  const double *fwd_peak, *bwd_peak, *out, *gcb, *mf, *RD;
  /* per row post-layer terms */
  const double *nAG[2], *nRS[2], *opb;
  /* scalars of the pre / post layers */
  double pre_fwd, pre_bwd, W1, W2, W1d, W2d, post_fwd;
  double pre_saved, pre_states, pre_states_and_saved;
  double post_states, post_fwd_peak, post_bwd_peak, post_output;
  double cap;
} StageLoopIn;

typedef struct {
  /* base, with_pre: [n_p][L][C+1][S]; with_post: [L][C+1][S]; no_pp: [C+1][S];
   * pre-filled by the caller with -1 / inf */
  int64_t *idx[4];
  double *stable[4];
  double *delta[4];
} StageLoopOut;

/* get_latencies (:2165-2216): float64 sums, then float32. */
static inline void row_latency(const StageLoopIn *in, int64_t i, int l, int c, float *stable32,
                               float *delta32) {
  const int lm2 = l - 2 > 0 ? l - 2 : 0;
  int n_ck = c - 1;
  if (n_ck < 0) n_ck = 0;
  if (n_ck > lm2) n_ck = lm2;
  const int n_nock = lm2 - n_ck;
  const int all_ck = c == l, no_ck = c == 0;
  const double st = (((double)n_ck * in->s_layer[1][i] + (double)n_nock * in->s_layer[0][i]) +
                     in->s_first[all_ck][i]) + in->s_last[!no_ck][i];
  const double de = (((double)n_ck * in->d_layer[1][i] + (double)n_nock * in->d_layer[0][i]) +
                     in->d_first[all_ck][i]) + in->d_last[!no_ck][i];
  *stable32 = (float)st;
  *delta32 = (float)de;
}

/* x / y_num of the four variants for one row (:2233-2355); y = y_num / G (:2813-2818).  The base
 * variant stays float32 (float32 array / python int), the others are float64 sums. */
static inline void variant_xy(const StageLoopIn *in, int64_t i, int c, float s32, float d32,
                              int variant, double *x, double *y_num, double *y) {
  const int k = c > 0;
  const double s = (double)s32, d = (double)d32;
  if (variant == 0) {
    *x = s;
    *y_num = d;
    *y = (double)(d32 / (float)in->G);
    return;
  }
  const double PS1 = in->pp_wre ? in->nAG[k][i] : 0.0, PD1 = in->pp_wre ? 0.0 : in->nAG[k][i];
  const double PS2 = in->pp_gre ? in->nRS[k][i] : 0.0, PD2 = in->pp_gre ? 0.0 : in->nRS[k][i];
  if (variant == 1) {
    *x = (((s + in->pre_fwd) + in->pre_bwd) + in->W1) + in->W2;
    *y_num = (d + in->W1d) + in->W2d;
  } else if (variant == 2) {
    *x = (((s + in->post_fwd) + in->opb[i]) + PS1) + PS2;
    *y_num = (d + PD1) + PD2;
  } else {
    *x = (((((((s + in->pre_fwd) + in->pre_bwd) + in->post_fwd) + in->opb[i]) + in->W1) + in->W2) + PS1) + PS2;
    *y_num = (((d + in->W1d) + in->W2d) + PD1) + PD2;
  }
  *y = *y_num / (double)in->G;
}

static inline double block_min(const double *v, int n) {
  double m = INFINITY;
  int i = 0;
#ifdef __AVX2__
  if (n >= 8) {
    __m256d a = _mm256_loadu_pd(v), b = _mm256_loadu_pd(v + 4);
    for (i = 8; i + 8 <= n; i += 8) {
      a = _mm256_min_pd(a, _mm256_loadu_pd(v + i));
      b = _mm256_min_pd(b, _mm256_loadu_pd(v + i + 4));
    }
    a = _mm256_min_pd(a, b);
    double t[4];
    _mm256_storeu_pd(t, a);
    for (int j = 0; j < 4; ++j)
      if (t[j] < m) m = t[j];
  }
#endif
  for (; i < n; ++i)
    if (v[i] < m) m = v[i];
  return m;
}

/* compute_indices (pareto.py:124-144) over one block: cost = r x + y where the mask holds, strict
 * "<" against the running minimum, so the first index of the smallest cost wins. */
static inline void scan_block(const double *restrict x, const double *restrict y,
                              const double *restrict ok, int n, int64_t first_row,
                              const double *ratios, int S, double *best, int64_t *best_row,
                              double *restrict cost) {
  for (int s = 0; s < S; ++s) {
    const double r = ratios[s];
    for (int i = 0; i < n; ++i) {
#ifdef MIST_ORACLE_FUSED
      /* what numba's fastmath=True may turn `r * x + y` into (pareto.py:124,138): one rounding */
      const double v = fma(r, x[i], y[i]);
#else
      const double v = r * x[i] + y[i];
#endif
      cost[i] = ok[i] != 0.0 ? v : INFINITY;
    }
    const double m = block_min(cost, n);
    if (m < best[s]) {
      int i = 0;
      while (cost[i] != m) ++i;
      best[s] = m;
      best_row[s] = first_row + i;
    }
  }
}

#define MAX2(a, b) ((a) > (b) ? (a) : (b)) /* np.maximum on NaN-free operands */

static void run_pair(const StageLoopIn *in, const StageLoopOut *o, int l, int c) {
  const int S = in->S, n_p = in->n_p, L = in->L, C1 = in->C + 1;
  const int64_t N = in->n_rows;
  /* running minima: [variant 0, 1][p][s], then with_post [s], no_pp [s] */
  const size_t n_best = (size_t)(2 * n_p + 2) * S;
  double *best = (double *)malloc(sizeof(double) * n_best);
  int64_t *best_row = (int64_t *)malloc(sizeof(int64_t) * n_best);
  for (size_t i = 0; i < n_best; ++i) { best[i] = INFINITY; best_row[i] = -1; }
  double x0[BLOCK], y0[BLOCK], x1[BLOCK], y1[BLOCK], x2[BLOCK], y2[BLOCK], x3[BLOCK], y3[BLOCK];
  double fs[BLOCK], bs[BLOCK], mod[BLOCK], cur[BLOCK], ckd[BLOCK], cost[BLOCK];
  double pfb[BLOCK], pbb[BLOCK], ok0[BLOCK], ok1[BLOCK], ok2[BLOCK], ok3[BLOCK];
  float s32[BLOCK], d32[BLOCK];
  const int c_eq_l = c == l, c_eq_0 = c == 0, ge = c >= l - 1, k = c > 0;
  const double dl = (double)l, dlm1 = (double)(l - 1 > 0 ? l - 1 : 0), dc = (double)c;
  const double f_eq = (double)c_eq_l, f_ne = (double)(1 - c_eq_l), f_ge = (double)ge,
               f_lt = (double)(1 - ge), f_c0 = (double)c_eq_0;
  const double dlm1s = (double)(l - 1), dlc1 = (double)(l - c - 1), dlc = (double)(l - c);
  const int lm2 = l - 2 > 0 ? l - 2 : 0;
  int n_ck_i = c - 1;
  if (n_ck_i < 0) n_ck_i = 0;
  if (n_ck_i > lm2) n_ck_i = lm2;
  const double n_ck = (double)n_ck_i, n_nock = (double)(lm2 - n_ck_i);
  const double dG = (double)in->G;
  const float fG = (float)in->G;
  const double pre_fwd = in->pre_fwd, pre_bwd = in->pre_bwd, W1 = in->W1, W2 = in->W2,
               W1d = in->W1d, W2d = in->W2d, post_fwd = in->post_fwd, cap = in->cap,
               pre_saved = in->pre_saved, pre_states = in->pre_states,
               pre_ss = in->pre_states_and_saved, post_states = in->post_states,
               post_fwd_peak = in->post_fwd_peak, post_bwd_peak = in->post_bwd_peak,
               post_output = in->post_output;
  const int pp_wre = in->pp_wre, pp_gre = in->pp_gre;
  for (int64_t r0 = 0; r0 < N; r0 += BLOCK) {
    const int n = (int)(N - r0 < BLOCK ? N - r0 : BLOCK);
    const double *restrict sl_ck = in->s_layer[1] + r0, *restrict sl_no = in->s_layer[0] + r0;
    const double *restrict dl_ck = in->d_layer[1] + r0, *restrict dl_no = in->d_layer[0] + r0;
    const double *restrict sf = in->s_first[c_eq_l] + r0, *restrict sla = in->s_last[!c_eq_0] + r0;
    const double *restrict df = in->d_first[c_eq_l] + r0, *restrict dla = in->d_last[!c_eq_0] + r0;
    const double *restrict T0 = in->T0 + r0, *restrict T1 = in->T1 + r0, *restrict pWG = in->pWG + r0,
                 *restrict pO = in->pO + r0, *restrict pWGO = in->pWGO + r0;
    const double *restrict S_ck = in->S_sav[1] + r0, *restrict S_no = in->S_sav[0] + r0;
    const double *restrict D_ck = in->D_sav[1] + r0, *restrict D_no = in->D_sav[0] + r0;
    const double *restrict fpk = in->fwd_peak + r0, *restrict bpk = in->bwd_peak + r0;
    const double *restrict outp = in->out + r0, *restrict gcbp = in->gcb + r0, *restrict mfp = in->mf + r0;
    const double *restrict RD = in->RD + r0, *restrict nAG = in->nAG[k] + r0, *restrict nRS = in->nRS[k] + r0;
    const double *restrict opb = in->opb + r0;
    /* get_latencies (:2165-2216): float64 sums, then float32 */
    for (int j = 0; j < n; ++j) {
      const double st = ((n_ck * sl_ck[j] + n_nock * sl_no[j]) + sf[j]) + sla[j];
      const double de = ((n_ck * dl_ck[j] + n_nock * dl_no[j]) + df[j]) + dla[j];
      s32[j] = (float)st;
      d32[j] = (float)de;
    }
    /* x, y = y_num / G of the four variants (:2233-2355, 2813-2818): the base variant stays
     * float32 (float32 array / python int), the others are float64 sums */
    for (int j = 0; j < n; ++j) {
      const double s = (double)s32[j], d = (double)d32[j];
      const double PS1 = pp_wre ? nAG[j] : 0.0, PD1 = pp_wre ? 0.0 : nAG[j];
      const double PS2 = pp_gre ? nRS[j] : 0.0, PD2 = pp_gre ? 0.0 : nRS[j];
      x0[j] = s;
      y0[j] = (double)(d32[j] / fG);
      x1[j] = (((s + pre_fwd) + pre_bwd) + W1) + W2;
      y1[j] = ((d + W1d) + W2d) / dG;
      x2[j] = (((s + post_fwd) + opb[j]) + PS1) + PS2;
      y2[j] = ((d + PD1) + PD2) / dG;
      x3[j] = (((((((s + pre_fwd) + pre_bwd) + post_fwd) + opb[j]) + W1) + W2) + PS1) + PS2;
      y3[j] = ((((d + W1d) + W2d) + PD1) + PD2) / dG;
    }
    for (int j = 0; j < n; ++j) {
      /* module states (:2150-2162) */
      fs[j] = (T0[j] + dl * pWG[j]) + dlm1 * pO[j];
      bs[j] = T1[j] + dl * pWGO[j];
      /* saved activations (:2358-2385); c <= l here, so the MEM_INF branch is not taken */
      const double cur_if_eq = dlm1s * S_ck[j];
      const double cur_if_not = dc * S_ck[j] + dlc1 * S_no[j];
      cur[j] = cur_if_eq * f_eq + cur_if_not * f_ne;
      mod[j] = S_ck[j] * dc + S_no[j] * dlc;
      ckd[j] = D_ck[j] * f_ge + D_no[j] * f_lt;
    }
    for (int p = 0; p < n_p; ++p) {
      const double dp = (double)p;
      const double p_pre = dp * pre_saved;
      for (int j = 0; j < n; ++j) { /* :2755-2812, 2866-2897 */
        const double outi = outp[j], gcb = gcbp[j], mf_pp = mfp[j] + 0.025;
        const double pipe = dp * mod[j] + cur[j];
        const double out2p = outi * dp * 2;
        const double pf = ((((fs[j] + pipe) + ckd[j]) + fpk[j]) + out2p) + gcb;
        const double pb = (((((bs[j] + pipe) + ckd[j]) + bpk[j]) + out2p) + outi * 2) + gcb;
        pfb[j] = pf;
        pbb[j] = pb;
        ok0[j] = MAX2(pf, pb) * (mf_pp + 0.01) <= cap ? 1.0 : 0.0;
        const double pf1 = (p_pre + pf) + pre_ss;
        const double pb1 = (p_pre + pb) + pre_ss;
        ok1[j] = MAX2(pf1, pb1) * mf_pp <= cap ? 1.0 : 0.0;
      }
      scan_block(x0, y0, ok0, n, r0, in->ratios, S, best + (size_t)p * S, best_row + (size_t)p * S, cost);
      scan_block(x1, y1, ok1, n, r0, in->ratios, S, best + (size_t)(n_p + p) * S,
                 best_row + (size_t)(n_p + p) * S, cost);
      if (p == 0) {
        for (int j = 0; j < n; ++j) { /* :2946-3001, 3057-3083 */
          const double outi = outp[j], gcb = gcbp[j], mf = mfp[j], mf_pp = mf + 0.025;
          const double f_in = (((fs[j] + post_states) + mod[j]) + post_fwd_peak) + gcb;
          const double b_in = ((((bs[j] + post_states) + mod[j]) + post_bwd_peak) + RD[j] * f_c0) + gcb;
          const double a2 = pfb[j] + post_states, b2 = (pbb[j] - outi) + post_states;
          const double pf2 = MAX2(f_in, a2);
          const double pb2 = MAX2(b_in, b2) + post_output;
          ok2[j] = MAX2(pf2, pb2) * mf_pp <= cap ? 1.0 : 0.0;
          const double pf3 = (pf2 + pre_states) + pre_saved;
          const double pb3 = (pb2 + pre_states) + pre_saved;
          ok3[j] = MAX2(pf3, pb3) * mf <= cap ? 1.0 : 0.0;
        }
        scan_block(x2, y2, ok2, n, r0, in->ratios, S, best + (size_t)(2 * n_p) * S,
                   best_row + (size_t)(2 * n_p) * S, cost);
        scan_block(x3, y3, ok3, n, r0, in->ratios, S, best + (size_t)(2 * n_p + 1) * S,
                   best_row + (size_t)(2 * n_p + 1) * S, cost);
      }
    }
  }
  /* The writes.  base / with_pre: every p for c <= l, except that the layer mask is narrowed by
   * `c != l - 1` when the last-stage variant is written at p == 0 (:3021-3023) and stays narrowed
   * for the later p of the same c.  with_post: c != l - 1.  no_pp: l == L and c != C - 1 (:3103). */
  for (int v = 0; v < 4; ++v) {
    if (v == 2 && c == l - 1) continue;
    if (v == 3 && (l != L || c == in->C - 1)) continue;
    for (int p = 0; p < (v < 2 ? n_p : 1); ++p) {
      if (v < 2 && p >= 1 && c == l - 1) continue;
      for (int s = 0; s < S; ++s) {
        const size_t at = v < 2    ? (((size_t)p * L + (l - 1)) * C1 + c) * S + s
                          : v == 2 ? ((size_t)(l - 1) * C1 + c) * S + s
                                   : (size_t)c * S + s;
        const int64_t row = best_row[(size_t)(v < 2 ? v * n_p + p : 2 * n_p + (v - 2)) * S + s];
        o->idx[v][at] = row;
        if (row >= 0) {
          float rs32, rd32;
          double x, ynum, y;
          row_latency(in, row, l, c, &rs32, &rd32);
          variant_xy(in, row, c, rs32, rd32, v, &x, &ynum, &y);
          o->stable[v][at] = x;
          o->delta[v][at] = ynum;
        }
      }
    }
  }
  free(best);
  free(best_row);
}

/* Returns 0.  `n_threads` <= 0 leaves the OpenMP default. */
int mist_oracle_stage_loop(const StageLoopIn *in, const StageLoopOut *out, int n_threads) {
  const int L = in->L, C = in->C;
  /* (l, c) pairs with c <= l, long ones (small c: most layers... all cost the same) in order */
  int n_pairs = 0;
  int *pl = (int *)malloc(sizeof(int) * (size_t)L * (C + 1));
  int *pc = (int *)malloc(sizeof(int) * (size_t)L * (C + 1));
  for (int l = 1; l <= L; ++l)
    for (int c = 0; c <= C && c <= l; ++c) { pl[n_pairs] = l; pc[n_pairs] = c; ++n_pairs; }
#ifdef _OPENMP
  if (n_threads > 0) {
#pragma omp parallel for schedule(dynamic, 1) num_threads(n_threads)
    for (int t = 0; t < n_pairs; ++t) run_pair(in, out, pl[t], pc[t]);
  } else {
#pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < n_pairs; ++t) run_pair(in, out, pl[t], pc[t]);
  }
#else
  for (int t = 0; t < n_pairs; ++t) run_pair(in, out, pl[t], pc[t]);
#endif
  free(pl);
  free(pc);
  return 0;
}

int mist_oracle_stage_loop_struct_bytes(void) { return (int)sizeof(StageLoopIn); }
