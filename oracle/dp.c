/* Oracle (test infrastructure): plain-C restatement of the reference's inter-stage DP kernel
 * `inter_stage_tune_dp_impl` (mist/analyzer/inter_tuning.py:220-355), which the reference
 * compiles with numba.  Same loop nest (s, k, d, mesh, i, j), float32 tables, strict "<"
 * updates.  Build: gcc -O2 -ffp-contract=off -shared -fPIC (see oracle/dp_c.py).
 * Checked against the python-loop form in oracle/inter_dp.py and, through it, against a
 * brute-force enumeration of all partitions (tests/test_oracle_dp.py). */
#include <math.h>
#include <stdlib.h>

/* Tables for one gradient-accumulation candidate, C-contiguous float32:
 *   costs, costs_pre: [Q][P1][L][L+1]   costs_post: [Q][L][L+1]   costs_nopp: [Q][L+1]
 * Outputs: *best_s (-1 if infeasible), *best_sum = f[best_s][0][D], *stage_max = f_stage_max[...],
 * argmin[(S+1)*(L+1)*(D+1)*4] = (end layer, n, m, ckpt) per state (may be NULL). */
int mist_oracle_dp(float t_max, int L, int D, int Q, const int *mesh_n, const int *mesh_m, int P1,
                   const float *costs, const float *costs_pre, const float *costs_post,
                   const float *costs_nopp, int *best_s, float *best_sum, float *stage_max,
                   int *argmin) {
  int max_nm = 0;
  for (int q = 0; q < Q; ++q)
    if (mesh_n[q] * mesh_m[q] > max_nm) max_nm = mesh_n[q] * mesh_m[q];
  const int S = (max_nm < L ? max_nm : L) / 2;
  const size_t plane = (size_t)(L + 1) * (D + 1);
  float *f = (float *)malloc(sizeof(float) * (S + 1) * plane);
  float *fm = (float *)malloc(sizeof(float) * (S + 1) * plane);
  if (!f || !fm) { free(f); free(fm); return -1; }
  for (size_t i = 0; i < (S + 1) * plane; ++i) { f[i] = INFINITY; fm[i] = 0.0f; }
  if (argmin)
    for (size_t i = 0; i < (S + 1) * plane * 4; ++i) argmin[i] = -1;
  f[(size_t)0 * plane + (size_t)L * (D + 1) + 0] = 0.0f;
  const int C = L + 1;
  for (int s = 1; s <= S; ++s) {
    const int p = s - 1;
    for (int k = L - s; k >= 0; --k) {
      for (int d = 1; d <= D; ++d) {
        const size_t at = (size_t)s * plane + (size_t)k * (D + 1) + d;
        for (int q = 0; q < Q; ++q) {
          const int nm = mesh_n[q] * mesh_m[q];
          if (nm > d) continue;
          for (int i = k; i < L; ++i) {
            const size_t from = (size_t)(s - 1) * plane + (size_t)(i + 1) * (D + 1) + (d - nm);
            const float prev = f[from];
            const int l = i - k + 1;
            const float *row;
            if (k == 0 && i == L - 1) row = costs_nopp + (size_t)q * C;
            else if (k == 0) row = costs_pre + (((size_t)q * P1 + p) * L + (l - 1)) * C;
            else if (i == L - 1) row = costs_post + ((size_t)q * L + (l - 1)) * C;
            else row = costs + (((size_t)q * P1 + p) * L + (l - 1)) * C;
            for (int j = 0; j <= L - i; ++j) {
              const float stage_cost = row[j];
              const float new_cost = stage_cost + prev;
              if (stage_cost <= t_max && new_cost < f[at]) {
                f[at] = new_cost;
                fm[at] = fm[from] > stage_cost ? fm[from] : stage_cost;
                if (argmin) {
                  argmin[at * 4 + 0] = i;
                  argmin[at * 4 + 1] = mesh_n[q];
                  argmin[at * 4 + 2] = mesh_m[q];
                  argmin[at * 4 + 3] = j;
                }
              }
            }
          }
        }
      }
    }
  }
  *best_s = -1;
  float best = INFINITY;
  for (int s = 1; s <= S; ++s) {
    const float v = f[(size_t)s * plane + D];
    if (v < best) { best = v; *best_s = s; }
  }
  *best_sum = best;
  *stage_max = *best_s > 0 ? fm[(size_t)(*best_s) * plane + D] : 0.0f;
  free(f);
  free(fm);
  return 0;
}
