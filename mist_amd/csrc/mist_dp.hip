// Inter-stage pipeline-partition DP on MI355X (gfx950).
//
// One workgroup per t_max threshold.  The stage index s is the sequential (wavefront) axis;
// the (start layer k, devices d) states of one s are independent and are spread over the
// threads.  F(s-1, ., .) / F(s, ., .) and the running stage maxima live in LDS when they fit
// (4 * (L+1) * (D+1) floats), otherwise in a caller-provided global scratch slab that stays in
// L2.  Each thread walks its state's (mesh, end layer, ckpt) candidates in the reference's
// order with float32 adds and strict "<", so ties resolve exactly as in the reference loop
// nest (mist/analyzer/inter_tuning.py:298-333).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>

#include "mist_common.h"
#include "mist_dp.h"

namespace {

using mist::fail;

constexpr int kDpThreads = 512;
constexpr int kLdsStateFloats = 12 * 1024;  // 48 KB of float32 state per workgroup

// ------------------------------------------------------------------------------------------
// Adapter: float64 (stable, delta) tables -> float32 DP cost tables for every g.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void cost_table_kernel(const double *__restrict__ stable,
                                                         const double *__restrict__ delta,
                                                         const int32_t *__restrict__ grad_accum,
                                                         int64_t n_cells, int64_t cells_per_g,
                                                         int sample_size, int slot,
                                                         float *__restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_cells) return;
  const float G = (float)grad_accum[i / cells_per_g];
  const float s = (float)stable[i * sample_size + slot];
  const float d = (float)delta[i * sample_size + slot];
  out[i] = s + d / G;
}

// ------------------------------------------------------------------------------------------
// DP kernel.
// ------------------------------------------------------------------------------------------
template <bool kUseLds>
__global__ __launch_bounds__(kDpThreads) void dp_kernel(
    const MistDpShape shape, const MistDpCosts tabs, const float *__restrict__ tmax_list,
    int32_t *__restrict__ best_s_out, float *__restrict__ best_sum_out,
    float *__restrict__ stage_max_out, int32_t *__restrict__ argmin, float *__restrict__ scratch) {
  extern __shared__ float lds_state[];
  const int L = shape.num_layers, D = shape.num_devices, Q = shape.num_mesh;
  const int P1 = shape.p_dim, S = shape.max_stages;
  const int W = D + 1;            // row pitch of a state plane
  const int plane = (L + 1) * W;  // states per s
  const int C = L + 1;            // ckpt extent of the cost tables
  float *state = kUseLds ? lds_state : scratch + (int64_t)blockIdx.x * 4 * plane;
  float *f_prev = state, *f_cur = state + plane;
  float *m_prev = state + 2 * plane, *m_cur = state + 3 * plane;
  const float t_max = tmax_list[blockIdx.x];

  for (int i = threadIdx.x; i < plane; i += kDpThreads) {
    f_prev[i] = INFINITY;
    m_prev[i] = 0.0f;
  }
  __syncthreads();
  if (threadIdx.x == 0) f_prev[L * W + 0] = 0.0f;  // F(0, L, 0) = 0
  int best_s = -1;
  float best_sum = INFINITY, best_max = 0.0f;
  __syncthreads();

  for (int s = 1; s <= S; ++s) {
    const int p = s - 1;
    // States of this step: k = 0..L-s, d = 1..D; everything else stays (inf, 0).
    for (int i = threadIdx.x; i < plane; i += kDpThreads) {
      f_cur[i] = INFINITY;
      m_cur[i] = 0.0f;
    }
    __syncthreads();
    const int n_states = (L - s + 1) * D;
    for (int st = threadIdx.x; st < n_states; st += kDpThreads) {
      // Largest loops (small k) first so that long states start early.
      const int k = st / D, d = st % D + 1;
      float best = INFINITY, best_m = 0.0f;
      int arg_i = -1, arg_q = -1, arg_j = -1;
      for (int q = 0; q < Q; ++q) {
        const int nm = shape.mesh_n[q] * shape.mesh_m[q];
        if (nm > d) continue;
        for (int i = k; i < L; ++i) {
          const int from = (i + 1) * W + (d - nm);
          const float prev = f_prev[from];
          const int l = i - k + 1;
          const float *__restrict__ row;
          if (k == 0 && i == L - 1) row = tabs.costs_nopp + (int64_t)q * C;
          else if (k == 0) row = tabs.costs_pre + (((int64_t)q * P1 + p) * L + (l - 1)) * C;
          else if (i == L - 1) row = tabs.costs_post + ((int64_t)q * L + (l - 1)) * C;
          else row = tabs.costs + (((int64_t)q * P1 + p) * L + (l - 1)) * C;
          // A state reachable only through an unreachable successor cannot improve: inf + c is
          // never < best.  Skipping it changes nothing and saves the inner loop.
          if (prev == INFINITY) continue;
          const float prev_m = m_prev[from];
          const int j_end = L - i;
          for (int j = 0; j <= j_end; ++j) {
            const float stage_cost = row[j];
            const float new_cost = stage_cost + prev;
            if (stage_cost <= t_max && new_cost < best) {
              best = new_cost;
              best_m = fmaxf(prev_m, stage_cost);
              arg_i = i;
              arg_q = q;
              arg_j = j;
            }
          }
        }
      }
      f_cur[k * W + d] = best;
      m_cur[k * W + d] = best_m;
      if (argmin != nullptr && arg_i >= 0) {
        int32_t *a = argmin + ((int64_t)s * plane + k * W + d) * 4;
        a[0] = arg_i;
        a[1] = shape.mesh_n[arg_q];
        a[2] = shape.mesh_m[arg_q];
        a[3] = arg_j;
      }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      const float v = f_cur[0 * W + D];
      if (v < best_sum) {  // first s wins ties (inter_tuning.py:335-340)
        best_sum = v;
        best_s = s;
        best_max = m_cur[0 * W + D];
      }
    }
    float *t0 = f_prev; f_prev = f_cur; f_cur = t0;
    float *t1 = m_prev; m_prev = m_cur; m_cur = t1;
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    best_s_out[blockIdx.x] = best_s;
    best_sum_out[blockIdx.x] = best_sum;
    stage_max_out[blockIdx.x] = best_max;
  }
}

int check_shape(const MistDpShape *shape) {
  if (!shape) return fail(MIST_E_INVALID, "null DP shape");
  if (shape->num_layers <= 0 || shape->num_devices <= 0 || shape->p_dim <= 0)
    return fail(MIST_E_INVALID, "bad DP extents L=%d D=%d P+1=%d", shape->num_layers,
                shape->num_devices, shape->p_dim);
  if (shape->num_mesh <= 0 || shape->num_mesh > MIST_MAX_MESH)
    return fail(MIST_E_INVALID, "num_mesh %d outside [1, %d]", shape->num_mesh, MIST_MAX_MESH);
  if (shape->max_stages < 0 || shape->max_stages > shape->p_dim)
    return fail(MIST_E_INVALID, "max_stages %d exceeds the p axis (%d) of the cost tables",
                shape->max_stages, shape->p_dim);
  if (shape->max_stages > shape->num_layers)
    return fail(MIST_E_INVALID, "max_stages %d exceeds num_layers %d", shape->max_stages,
                shape->num_layers);
  for (int q = 0; q < shape->num_mesh; ++q)
    if (shape->mesh_n[q] <= 0 || shape->mesh_m[q] <= 0)
      return fail(MIST_E_INVALID, "mesh %d is (%d, %d)", q, shape->mesh_n[q], shape->mesh_m[q]);
  return 0;
}

bool fits_lds(const MistDpShape *shape) {
  const int64_t plane = (int64_t)(shape->num_layers + 1) * (shape->num_devices + 1);
  return 4 * plane <= kLdsStateFloats;
}

}  // namespace

extern "C" {

int mist_sizeof_dp_shape(void) { return (int)sizeof(MistDpShape); }

int mist_dp_cost_tables(const MistProblem *problem, const MistOutTables *tables,
                        const int32_t *d_grad_accum, int slot, float *const d_out[4],
                        void *stream) {
  if (!problem || !tables || !d_grad_accum || !d_out)
    return fail(MIST_E_INVALID, "null pointer argument");
  const int64_t L = problem->num_layers, P1 = problem->p_dim, S = problem->sample_size;
  const int64_t Gn = problem->num_grad_accum, Q = problem->num_mesh;
  if (L <= 0 || P1 <= 0 || S <= 0 || Gn <= 0 || Q <= 0)
    return fail(MIST_E_INVALID, "bad problem extents");
  if (slot < 0 || slot >= S) return fail(MIST_E_INVALID, "slot %d outside [0, %d)", slot, (int)S);
  const int64_t per_g[4] = {Q * P1 * L * (L + 1), Q * P1 * L * (L + 1), Q * L * (L + 1), Q * (L + 1)};
  for (int v = 0; v < 4; ++v) {
    if (!tables->stable[v] || !tables->delta[v] || !d_out[v])
      return fail(MIST_E_INVALID, "table %d is null", v);
    const int64_t n = Gn * per_g[v];
    hipLaunchKernelGGL(cost_table_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, tables->stable[v], tables->delta[v], d_grad_accum, n,
                       per_g[v], (int)S, slot, d_out[v]);
    MIST_HIP_CHECK(hipGetLastError());
  }
  return 0;
}

int mist_dp_filter_tmax(const float *sorted_unique, int n, double gap, float *out) {
  if (n < 0 || (n > 0 && (!sorted_unique || !out))) return fail(MIST_E_INVALID, "bad t_max list");
  int kept = 0;
  float last = 0.0f;
  for (int i = 0; i < n; ++i) {
    const float t = sorted_unique[i];
    const float diff = t - last;  // float32 difference ...
    if ((double)diff < gap) continue;  // ... compared in float64
    out[kept++] = t;
    last = t;
  }
  return kept;
}

int64_t mist_dp_scratch_floats(const MistDpShape *shape, int n_tmax) {
  if (check_shape(shape) != 0 || n_tmax <= 0) return -1;
  if (fits_lds(shape)) return 0;
  return (int64_t)4 * n_tmax * (shape->num_layers + 1) * (shape->num_devices + 1);
}

int mist_dp_run(const MistDpShape *shape, const MistDpCosts *costs, const float *d_tmax,
                int n_tmax, int32_t *d_best_s, float *d_best_sum, float *d_stage_max,
                int32_t *d_argmin, float *d_scratch, void *stream) {
  if (int rc = check_shape(shape)) return rc;
  if (!costs || !costs->costs || !costs->costs_pre || !costs->costs_post || !costs->costs_nopp)
    return fail(MIST_E_INVALID, "null cost table");
  if (!d_tmax || !d_best_s || !d_best_sum || !d_stage_max)
    return fail(MIST_E_INVALID, "null threshold / output pointer");
  if (n_tmax <= 0) return fail(MIST_E_INVALID, "n_tmax must be positive, got %d", n_tmax);
  if (d_argmin && n_tmax != 1)
    return fail(MIST_E_INVALID, "argmin output needs n_tmax == 1, got %d", n_tmax);
  const int plane = (shape->num_layers + 1) * (shape->num_devices + 1);
  if (fits_lds(shape)) {
    hipLaunchKernelGGL(dp_kernel<true>, dim3(n_tmax), dim3(kDpThreads),
                       4 * plane * sizeof(float), (hipStream_t)stream, *shape, *costs, d_tmax,
                       d_best_s, d_best_sum, d_stage_max, d_argmin, (float *)nullptr);
  } else {
    if (!d_scratch) return fail(MIST_E_INVALID, "state does not fit in LDS: scratch is required");
    hipLaunchKernelGGL(dp_kernel<false>, dim3(n_tmax), dim3(kDpThreads), 0, (hipStream_t)stream,
                       *shape, *costs, d_tmax, d_best_s, d_best_sum, d_stage_max, d_argmin,
                       d_scratch);
  }
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // extern "C"
