// Stage-assignment search of the `uniform-device-pp-mip` granularity
// (reference: mist/analyzer/inter_tuning_mip.py).
//
//   stage_samples_kernel  one workgroup (one wavefront) per (stage, layer count): stages the
//                         candidate row in LDS as float32 pairs, lane a scans it for sample a,
//                         then the lanes compare their picks to drop repeated pairs.
//   mist_mip_solve        host: exact optimum of the assignment the reference gives to CBC.
//
// Why the host solver is exact.  For fixed stage choices let Z_0 = 0, Z_{i+1} = T_i + max(Z_i,
// D_i).  By induction Z_i = sum_{i'<i} T_i' + max(0, max_{i'<i} (D_i' - sum_{i''<i'} T_i'')), so
// Z_S is the objective without its (G - 1) * max T term.  Z_{i+1} grows with Z_i, hence the
// smallest Z per (stages done, layers used) is all a recurrence over the stages has to keep.
// The optimum's max T equals one of the entry values: for every such value tau (ascending) the
// recurrence runs over the entries with T <= tau and (G - 1) * tau + Z_S is a candidate total.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <limits>
#include <thread>
#include <vector>

#include "mist_common.h"
#include "mist_mip.h"

using mist::fail;

namespace {

constexpr int kSampleLanes = 64;

struct StageRow {
  const double *stable, *delta;  // first candidate of the row, nullptr = every candidate +inf
};

// Table row of stage `stage` holding `layers` layers (inter_tuning_mip.py:453-468; later
// assignments there overwrite earlier ones, which fixes the order of the tests below).
__device__ StageRow stage_row(const MistMipShape &s, const MistMipTables &t, int stage,
                              int layers) {
  const int64_t L = s.num_layers, P = s.sample_size;
  const int64_t row = (L + 1) * P;  // one (ckpt, policy) plane
  if (stage == 0 && layers == L) return {t.stable[3], t.delta[3]};
  if (stage == s.num_stages - 1) {
    const int64_t off = (int64_t)(layers - 1) * row;
    return {t.stable[2] + off, t.delta[2] + off};
  }
  const int p = s.num_stages - stage - 1;  // pre-saved micro-batches of this stage
  if (p >= s.p_dim) return {nullptr, nullptr};
  const int64_t off = ((int64_t)p * L + (layers - 1)) * row;
  const int v = stage == 0 ? 1 : 0;
  return {t.stable[v] + off, t.delta[v] + off};
}

// One (stage, layer count) row of one problem: `block` = stage * nl + (layers - layers_min).
__device__ __forceinline__ void stage_samples_row(
    const MistMipShape &shape, const MistMipTables &tables, int block, float *lds,
    const double *__restrict__ ratios, float *__restrict__ out_stable,
    float *__restrict__ out_delta, int32_t *__restrict__ out_index,
    uint8_t *__restrict__ out_keep) {
  const int P = shape.sample_size, L = shape.num_layers;
  const int nl = shape.layers_max - shape.layers_min + 1;
  const int stage = block / nl, layers = shape.layers_min + block % nl;
  const int lane = threadIdx.x;

  int n_cand = P, first = 0;  // candidates of the row: all planes, or one ckpt plane
  if (shape.ckpt_mode == MIST_MIP_CKPT_TUNED) n_cand = (L + 1) * P;
  else if (shape.ckpt_mode == MIST_MIP_CKPT_FIXED) first = shape.fixed_ckpt * P;
  else first = layers * P;

  float *x = lds, *y = lds + n_cand;
  float *pick_x = y + n_cand, *pick_y = pick_x + kSampleLanes;
  const StageRow row = stage_row(shape, tables, stage, layers);
  for (int n = lane; n < n_cand; n += kSampleLanes) {
    x[n] = row.stable ? (float)row.stable[first + n] : INFINITY;
    y[n] = row.delta ? (float)row.delta[first + n] : INFINITY;
  }
  __syncthreads();

  int best = -1;
  float sx = 0.0f, sy = 0.0f;
  if (lane < P) {
    const double r = ratios[lane];
    double best_cost = INFINITY;
    for (int n = 0; n < n_cand; ++n) {
      const double cost = r * (double)x[n] + (double)y[n];
      if (cost < best_cost) {
        best_cost = cost;
        best = n;
      }
    }
    // numpy reads index -1 as the last candidate (pareto.py:76-77)
    sx = x[best >= 0 ? best : n_cand - 1];
    sy = y[best >= 0 ? best : n_cand - 1];
    pick_x[lane] = sx;
    pick_y[lane] = sy;
  }
  __syncthreads();
  if (lane >= P) return;
  bool keep = true;
  for (int a = 0; a < lane; ++a) keep = keep && !(pick_x[a] == sx && pick_y[a] == sy);
  if (!keep) sx = sy = INFINITY;
  if (sx < 0.0f) sx = 0.0f;
  if (sy < 0.0f) sy = 0.0f;
  if (sx == INFINITY) sx = MIST_MIP_MAX_VALUE;
  if (sy == INFINITY) sy = MIST_MIP_MAX_VALUE;
  const int64_t o = (int64_t)block * P + lane;
  out_stable[o] = sx;
  out_delta[o] = sy;
  out_index[o] = best;
  out_keep[o] = keep ? 1 : 0;
}

__global__ __launch_bounds__(kSampleLanes) void stage_samples_kernel(
    MistMipShape shape, MistMipTables tables, const double *__restrict__ ratios,
    float *__restrict__ out_stable, float *__restrict__ out_delta, int32_t *__restrict__ out_index,
    uint8_t *__restrict__ out_keep) {
  extern __shared__ float lds[];
  stage_samples_row(shape, tables, blockIdx.x, lds, ratios, out_stable, out_delta, out_index,
                    out_keep);
}

// Every problem of a search in one launch: workgroup -> (problem, row) through the problems'
// first workgroups (ascending); outputs of problem i start at its out_offset.
__global__ __launch_bounds__(kSampleLanes) void stage_samples_batch_kernel(
    const MistMipBatchItem *__restrict__ items, int n_items, const double *__restrict__ ratios,
    float *__restrict__ out_stable, float *__restrict__ out_delta, int32_t *__restrict__ out_index,
    uint8_t *__restrict__ out_keep) {
  extern __shared__ float lds[];
  int lo = 0, hi = n_items;  // items[lo].first_block <= blockIdx.x < items[hi].first_block
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (items[mid].first_block <= (int)blockIdx.x) lo = mid; else hi = mid;
  }
  const MistMipBatchItem &it = items[lo];
  const int64_t o = it.out_offset;
  stage_samples_row(it.shape, it.tables, (int)blockIdx.x - it.first_block, lds, ratios,
                    out_stable + o, out_delta + o, out_index + o, out_keep + o);
}

// One workgroup per table row (a (variant, pre-saved micro-batches, layer count) of a region, all
// its ckpt counts and samples): costs +inf, row indices -1.
__global__ __launch_bounds__(256) void prefill_cells_kernel(const int32_t *__restrict__ regions,
                                                            int n_regions, int L, int P1, int S,
                                                            int Q, const MistOutTables tables) {
  int lo = 0, hi = n_regions - 1;
  const int block = blockIdx.x;
  while (lo < hi) {  // last region whose first row is <= block
    const int mid = (lo + hi + 1) >> 1;
    if (regions[6 * mid + 5] <= block) lo = mid;
    else hi = mid - 1;
  }
  const int32_t *r = regions + 6 * lo;
  const int64_t g = r[0], q = r[1];
  const int l_min = r[2], nl = r[3] - r[2] + 1, pc = min(r[4], P1);
  int row = block - r[5];
  const int64_t cells = (int64_t)(L + 1) * S;
  int v;
  int64_t at;
  if (row < 2 * pc * nl) {
    v = row / (pc * nl);
    row -= v * pc * nl;
    const int p = row / nl, l = l_min + row % nl;
    at = (((g * Q + q) * P1 + p) * L + (l - 1)) * cells;
  } else if (row < 2 * pc * nl + nl) {
    v = 2;
    at = ((g * Q + q) * L + (l_min + row - 2 * pc * nl - 1)) * cells;
  } else {
    v = 3;
    at = (g * Q + q) * cells;
  }
  double *__restrict__ stable = tables.stable[v] + at, *__restrict__ delta = tables.delta[v] + at;
  int32_t *__restrict__ index = tables.index[v] + at;
  for (int64_t e = threadIdx.x; e < cells; e += blockDim.x) {
    stable[e] = INFINITY;
    delta[e] = INFINITY;
    index[e] = -1;
  }
}

int check_mip_shape(const MistMipShape *s) {
  if (!s) return fail(MIST_E_INVALID, "null MistMipShape");
  if (s->num_layers < 1 || s->num_stages < 1 || s->num_stages > s->num_layers)
    return fail(MIST_E_INVALID, "num_stages %d outside [1, num_layers %d]", s->num_stages,
                s->num_layers);
  if (s->sample_size < 1 || s->sample_size > MIST_MIP_MAX_SAMPLES)
    return fail(MIST_E_INVALID, "sample_size %d outside [1, %d]", s->sample_size,
                MIST_MIP_MAX_SAMPLES);
  if (s->layers_min < 1 || s->layers_max > s->num_layers)
    return fail(MIST_E_INVALID, "layer counts %d..%d outside [1, %d]", s->layers_min,
                s->layers_max, s->num_layers);
  if (s->p_dim < 1) return fail(MIST_E_INVALID, "p_dim %d < 1", s->p_dim);
  if (s->ckpt_mode < MIST_MIP_CKPT_TUNED || s->ckpt_mode > MIST_MIP_CKPT_FULL)
    return fail(MIST_E_INVALID, "unknown ckpt_mode %d", s->ckpt_mode);
  if (s->ckpt_mode == MIST_MIP_CKPT_FIXED && (s->fixed_ckpt < 0 || s->fixed_ckpt > s->num_layers))
    return fail(MIST_E_INVALID, "fixed_ckpt %d outside [0, %d]", s->fixed_ckpt, s->num_layers);
  return 0;
}

}  // namespace

extern "C" {

int mist_sizeof_mip_shape(void) { return (int)sizeof(MistMipShape); }

int mist_mip_stage_samples(const MistMipShape *shape, const MistMipTables *tables,
                           const double *d_ratios, float *d_t_stable, float *d_t_delta,
                           int32_t *d_index, uint8_t *d_keep, void *stream) {
  if (int rc = check_mip_shape(shape)) return rc;
  if (shape->layers_min > shape->layers_max) return 0;  // no layer count to sample
  if (!tables || !d_ratios || !d_t_stable || !d_t_delta || !d_index || !d_keep)
    return fail(MIST_E_INVALID, "null pointer");
  for (int v = 0; v < 4; ++v)
    if (!tables->stable[v] || !tables->delta[v])
      return fail(MIST_E_INVALID, "null table of variant %d", v);
  const int64_t n_cand = shape->ckpt_mode == MIST_MIP_CKPT_TUNED
                             ? (int64_t)(shape->num_layers + 1) * shape->sample_size
                             : shape->sample_size;
  const int64_t lds_bytes = (2 * n_cand + 2 * kSampleLanes) * (int64_t)sizeof(float);
  if (lds_bytes > 64 * 1024)
    return fail(MIST_E_INVALID, "%lld candidates per table row exceed the LDS staging buffer",
                (long long)n_cand);
  const int nl = shape->layers_max - shape->layers_min + 1;
  hipLaunchKernelGGL(stage_samples_kernel, dim3((unsigned)(shape->num_stages * nl)),
                     dim3(kSampleLanes), (size_t)lds_bytes, (hipStream_t)stream, *shape, *tables,
                     d_ratios, d_t_stable, d_t_delta, d_index, d_keep);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int mist_sizeof_mip_batch_item(void) { return (int)sizeof(MistMipBatchItem); }

int mist_mip_stage_samples_batch(const MistMipBatchItem *items, const MistMipBatchItem *d_items,
                                 int n_items, const double *d_ratios, float *d_t_stable,
                                 float *d_t_delta, int32_t *d_index, uint8_t *d_keep,
                                 void *stream) {
  if (!items || !d_items || n_items <= 0)
    return fail(MIST_E_INVALID, "null / empty problem list (n_items=%d)", n_items);
  if (!d_ratios || !d_t_stable || !d_t_delta || !d_index || !d_keep)
    return fail(MIST_E_INVALID, "null pointer");
  int64_t blocks = 0, lds_bytes = 0, out = 0;
  for (int i = 0; i < n_items; ++i) {
    const MistMipShape *s = &items[i].shape;
    if (int rc = check_mip_shape(s)) return rc;
    const int nl = s->layers_max - s->layers_min + 1;
    if (nl <= 0) return fail(MIST_E_INVALID, "problem %d has no layer count to sample", i);
    for (int v = 0; v < 4; ++v)
      if (!items[i].tables.stable[v] || !items[i].tables.delta[v])
        return fail(MIST_E_INVALID, "problem %d: null table of variant %d", i, v);
    if (items[i].first_block != blocks || items[i].out_offset != out)
      return fail(MIST_E_INVALID, "problem %d: first_block / out_offset do not continue the list", i);
    blocks += (int64_t)s->num_stages * nl;
    out += (int64_t)s->num_stages * nl * s->sample_size;
    const int64_t n_cand = s->ckpt_mode == MIST_MIP_CKPT_TUNED
                               ? (int64_t)(s->num_layers + 1) * s->sample_size : s->sample_size;
    lds_bytes = std::max<int64_t>(lds_bytes, (2 * n_cand + 2 * kSampleLanes) * (int64_t)sizeof(float));
  }
  if (lds_bytes > 64 * 1024)
    return fail(MIST_E_INVALID, "candidates per table row exceed the LDS staging buffer");
  if (blocks >= (int64_t)1 << 31) return fail(MIST_E_INVALID, "too many rows for one launch");
  hipLaunchKernelGGL(stage_samples_batch_kernel, dim3((unsigned)blocks), dim3(kSampleLanes),
                     (size_t)lds_bytes, (hipStream_t)stream, d_items, n_items, d_ratios,
                     d_t_stable, d_t_delta, d_index, d_keep);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int mist_mip_solve(const MistMipShape *shape, int grad_accum, double best_cost,
                   const float *t_stable, const float *t_delta, const uint8_t *keep,
                   double *out_cost, int32_t *out_layers, int32_t *out_slot) {
  if (int rc = check_mip_shape(shape)) return rc;
  if (grad_accum < 1) return fail(MIST_E_INVALID, "grad_accum %d < 1", grad_accum);
  if (!out_cost || !out_layers || !out_slot) return fail(MIST_E_INVALID, "null output");
  const double inf = std::numeric_limits<double>::infinity();
  *out_cost = inf;
  if (shape->layers_min > shape->layers_max) return 0;
  if (!t_stable || !t_delta || !keep) return fail(MIST_E_INVALID, "null pointer");
  const int S = shape->num_stages, L = shape->num_layers, P = shape->sample_size;
  const int lo = shape->layers_min, nl = shape->layers_max - lo + 1;
  const int per_stage = nl * P;

  std::vector<double> z((size_t)(S + 1) * (L + 1));
  std::vector<int32_t> back((size_t)S * (L + 1));
  std::vector<int32_t> picks((size_t)S);
  // Smallest Z_S[L] over kept entries with T <= tau; fills `picks` (entry index per stage).
  auto chain = [&](double tau) -> double {
    std::fill(z.begin(), z.end(), inf);
    z[0] = 0.0;
    for (int i = 0; i < S; ++i) {
      const double *prev = &z[(size_t)i * (L + 1)];
      double *cur = &z[(size_t)(i + 1) * (L + 1)];
      const int64_t base = (int64_t)i * per_stage;
      for (int m = 0; m <= L; ++m) {
        double best = inf;
        int32_t arg = -1;
        for (int a = 0; a < nl; ++a) {
          const int from = m - (lo + a);
          if (from < 0) break;
          const double zp = prev[from];
          if (!(zp < inf)) continue;
          for (int k = 0; k < P; ++k) {
            const int64_t e = base + (int64_t)a * P + k;
            const double t = (double)t_stable[e];
            if (!keep[e] || !(t <= tau)) continue;
            const double cand = t + std::max(zp, (double)t_delta[e]);
            if (cand < best) {
              best = cand;
              arg = (int32_t)(a * P + k);
            }
          }
        }
        cur[m] = best;
        back[(size_t)i * (L + 1) + m] = arg;
      }
    }
    const double total = z[(size_t)S * (L + 1) + L];
    if (!(total < inf)) return inf;
    int m = L;
    for (int i = S - 1; i >= 0; --i) {
      const int32_t arg = back[(size_t)i * (L + 1) + m];
      picks[i] = arg;
      m -= lo + arg / P;
    }
    return total;
  };
  auto emit = [&](double cost) {
    *out_cost = cost;
    for (int i = 0; i < S; ++i) {
      out_layers[i] = lo + picks[i] / P;
      out_slot[i] = picks[i] % P;
    }
  };

  const double z_free = chain(inf);
  if (!(z_free < inf)) return 0;
  if (grad_accum == 1) {
    emit(z_free);
    return 1;
  }
  std::vector<double> taus;
  for (int64_t e = 0; e < (int64_t)S * per_stage; ++e)
    if (keep[e] && std::isfinite(t_stable[e])) taus.push_back((double)t_stable[e]);
  std::sort(taus.begin(), taus.end());
  taus.erase(std::unique(taus.begin(), taus.end()), taus.end());
  double best = inf;
  for (double tau : taus) {
    const double weight = (double)(grad_accum - 1) * tau;
    if (weight > best_cost || weight + z_free >= best) break;
    const double zs = chain(tau);
    if (zs < inf && weight + zs < best) {
      best = weight + zs;
      emit(best);
    }
  }
  return best < inf ? 1 : 0;
}

int mist_mip_prefill_cells(int num_layers, int p_dim, int sample_size, int num_mesh,
                           int num_table_rows, const int32_t *regions, const int32_t *d_regions,
                           int n_regions, const MistOutTables *tables, void *stream) {
  if (!regions || !d_regions || !tables) return fail(MIST_E_INVALID, "null pointer");
  if (n_regions < 1) return fail(MIST_E_INVALID, "n_regions %d < 1", n_regions);
  if (num_layers < 1 || p_dim < 1 || sample_size < 1 || num_mesh < 1 || num_table_rows < 1)
    return fail(MIST_E_INVALID, "table extents must be positive");
  for (int v = 0; v < 4; ++v)
    if (!tables->stable[v] || !tables->delta[v] || !tables->index[v])
      return fail(MIST_E_INVALID, "null table of variant %d", v);
  int64_t rows = 0;
  for (int i = 0; i < n_regions; ++i) {
    const int32_t *r = regions + 6 * i;
    if (r[0] < 0 || r[0] >= num_table_rows || r[1] < 0 || r[1] >= num_mesh)
      return fail(MIST_E_INVALID, "region %d: table row %d / mesh %d outside the tables", i, r[0], r[1]);
    if (r[2] < 1 || r[3] > num_layers || r[2] > r[3] || r[4] < 1)
      return fail(MIST_E_INVALID, "region %d: layer counts %d..%d, %d pre-saved micro-batch values", i,
                  r[2], r[3], r[4]);
    if (r[5] != rows) return fail(MIST_E_INVALID, "region %d: first row does not continue the list", i);
    const int64_t nl = r[3] - r[2] + 1, pc = std::min(r[4], p_dim);
    rows += 2 * pc * nl + nl + (r[3] == num_layers ? 1 : 0);
  }
  if (rows >= (int64_t)1 << 31) return fail(MIST_E_INVALID, "too many rows for one launch");
  hipLaunchKernelGGL(prefill_cells_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream,
                     d_regions, n_regions, num_layers, p_dim, sample_size, num_mesh, *tables);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int mist_mip_solve_chains(const MistMipBatchItem *items, const int32_t *grad_accum,
                          int items_per_chain, int n_chains, const float *t_stable,
                          const float *t_delta, const uint8_t *keep, double *out_cost,
                          int32_t *out_item, int32_t *out_layers, int32_t *out_slot) {
  if (!items || !grad_accum || !t_stable || !t_delta || !keep || !out_cost || !out_item || !out_layers ||
      !out_slot)
    return fail(MIST_E_INVALID, "null pointer");
  if (items_per_chain < 1 || n_chains < 1)
    return fail(MIST_E_INVALID, "%d chains of %d problems", n_chains, items_per_chain);
  int L = 0;
  for (int64_t i = 0; i < (int64_t)items_per_chain * n_chains; ++i) {
    if (int rc = check_mip_shape(&items[i].shape)) return rc;
    if (grad_accum[i % items_per_chain] < 1)
      return fail(MIST_E_INVALID, "grad_accum %d < 1", grad_accum[i % items_per_chain]);
    if (i > 0 && items[i].shape.num_layers != L)
      return fail(MIST_E_INVALID, "problem %lld has %d layers, problem 0 has %d", (long long)i,
                  items[i].shape.num_layers, L);
    L = items[i].shape.num_layers;
  }
  // One chain = the problems of one search in the reference's order: the bound of a problem is
  // the best cost of those before it (inter_tuning_mip.py:131-214).  Chains do not depend on
  // each other: a thread each.
  std::vector<int> status((size_t)n_chains, 0);
  auto run_chain = [&](int c) {
    double best_cost = (double)MIST_MIP_MAX_VALUE;
    int best_item = -1;
    std::vector<int32_t> layers((size_t)L), slots((size_t)L);
    for (int i = 0; i < items_per_chain; ++i) {
      const MistMipBatchItem &item = items[(int64_t)c * items_per_chain + i];
      double cost = 0.0;
      const int rc = mist_mip_solve(&item.shape, grad_accum[i], best_cost, t_stable + item.out_offset,
                                    t_delta + item.out_offset, keep + item.out_offset, &cost,
                                    layers.data(), slots.data());
      if (rc < 0) {
        status[c] = rc;
        return;
      }
      if (rc == 1 && cost < best_cost) {
        best_cost = cost;
        best_item = i;
        std::copy(layers.begin(), layers.begin() + item.shape.num_stages, out_layers + (int64_t)c * L);
        std::copy(slots.begin(), slots.begin() + item.shape.num_stages, out_slot + (int64_t)c * L);
      }
    }
    out_cost[c] = best_cost;
    out_item[c] = best_item;
  };
  if (n_chains == 1) {
    run_chain(0);
  } else {
    std::vector<std::thread> workers;
    for (int c = 0; c < n_chains; ++c) workers.emplace_back(run_chain, c);
    for (std::thread &w : workers) w.join();
  }
  for (int c = 0; c < n_chains; ++c)
    if (status[c] < 0)  // (every argument the solver checks was checked above)
      return fail(status[c], "the solver of chain %d rejected its arguments", c);
  return 0;
}

}  // extern "C"
