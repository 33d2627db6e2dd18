// Host orchestration of the inter-stage search (reference: inter_stage_tune /
// inter_stage_tune_with_fixed_grad_accumu, mist/analyzer/inter_tuning.py:95-217, and the
// uniform-device variant, mist/analyzer/inter_tuning_uniform_device.py:312-367): bottleneck DP,
// threshold windows, speculative scan batches with the sequential replay of the reference's
// rules, back-pointers of the winner, strategy rows of its stages.  Same steps as the Python
// driver (mist_amd/inter_tuning.py); here they run without an interpreter between the batches,
// and the first three of them (bottleneck DP, windows, first scan batch) without the host: a
// search waits for the GPU three times (that batch, the second scan batch, the back-pointers).
//
// A search runs over one or more DP families (shape + tables): the per-mesh recurrence is one
// family, the uniform-device recurrence one family per admissible stage count.  The cost of a
// (G, threshold) instance is the smallest family total, the first family winning ties; all
// families of a batch run back to back on the stream and come back with one synchronisation.
//
// Everything that decides a result is shared with the Python driver through the C ABI:
// mist_dp_run, mist_dp_select_candidates, mist_dp_window_begin, mist_dp_filter_tmax,
// mist_dp_backtrack (mist_dp_windows_first_batch walks the windows with the code of
// mist_dp_window_begin, and a window it cannot decide sends the search down the host route).
// How far a window is fetched or how many thresholds a batch speculates on
// only changes the work done, never the outcome: the replay consumes DP results in the
// reference's order with its stop rule and its strict "<", and passes without a DP run only
// the thresholds at which the reference's run provably changes nothing (struct Scan).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <map>
#include <mutex>
#include <vector>

#include "mist_common.h"
#include "mist_dp.h"
#include "mist_inter.h"

using mist::fail;

namespace {

constexpr int kFirstChunk = 48;   // thresholds per G in the first speculative batch ...
constexpr int kFirstLead = 16;    // ... of a window longer than that: the first ones, the rest spread
constexpr int kProbes = 16;       // thresholds spread over what a later request does not reach
constexpr double kFloorSlack = 1e-6;  // relative slack of the bound that lets the scan pass thresholds
constexpr int kMaxChunk = 4096;   // most thresholds per G in one batch
constexpr double kGap = 1e-6;     // inter_tuning.py:177
constexpr int kSelectHead = 1 << 16;  // selected candidates that travel with the counts of a fetch
constexpr int kWindowCapacity = 8192;  // candidates of a window that is walked on the device
constexpr int kKeptCapacity = 1 << 18;  // kept thresholds of all windows of a search, on the device
constexpr int kKeptHead = 1 << 15;      // of which this many travel with the first round trip
const double kInf = std::numeric_limits<double>::infinity();

// ---- buffers that live as long as the process: device and pinned host memory per device ----
struct Buffer {
  void *ptr = nullptr;
  size_t bytes = 0;
  bool pinned = false;
  int reserve(size_t want) {
    if (want <= bytes) return 0;
    size_t grown = std::max(want, bytes * 2);
    if (ptr) {
      if (pinned) MIST_HIP_CHECK(hipHostFree(ptr));
      else MIST_HIP_CHECK(hipFree(ptr));
      ptr = nullptr;
      bytes = 0;
    }
    if (pinned) MIST_HIP_CHECK(hipHostMalloc(&ptr, grown, hipHostMallocDefault));
    else MIST_HIP_CHECK(hipMalloc(&ptr, grown));
    bytes = grown;
    return 0;
  }
  template <typename T>
  T *as() const { return static_cast<T *>(ptr); }
};

struct Workspace {
  Buffer d_in, d_out, d_scratch, d_req, d_counts, d_values, d_request, d_argmin, d_grad;
  Buffer h_in, h_out, h_req, h_counts, h_values, h_request, h_grad;
  // windows and first scan batch decided on the device
  // (requests, window descriptions, DP outputs and kept thresholds in one buffer: one copy back)
  Buffer d_win_values, d_win_counts, d_inst_t, d_inst_row, d_first;
  Buffer h_first;
  int select_capacity = 1 << 18;
  Workspace() {
    h_in.pinned = h_out.pinned = h_req.pinned = h_counts.pinned = h_values.pinned =
        h_request.pinned = h_grad.pinned = h_first.pinned = true;
  }
};

std::mutex g_lock;  // one search at a time per process: the workspaces are shared
std::map<int, Workspace> g_workspaces;

struct Window {
  bool exists = false;
  int row = 0, G = 1;
  float start_value = 0.0f;
  double start_sum = 0.0, bound = kInf;
  std::vector<float> kept;
  std::vector<double> scaled;
  float hi = 0.0f;
  bool complete = false;

  float lower_margin(int widen) const {
    const double step = (1e-4 + 1e-5 * std::fabs((double)start_value)) * std::pow(4.0, widen);
    return start_value - (float)step;
  }
  void append(const float *values, size_t n) {
    for (size_t i = 0; i < n; ++i) {
      kept.push_back(values[i]);
      scaled.push_back((double)values[i] * (double)G);
    }
    if (!(bound < kInf)) {
      const auto at = std::lower_bound(kept.begin(), kept.end(), start_value);
      if (at != kept.end()) bound = start_sum + (double)(G - 1) * (double)*at;
    }
  }
  // every kept candidate the scan can reach under the running best is materialised
  bool covers(double best_cost) const {
    const double need = std::min(best_cost, bound);
    return complete || (double)hi * (double)G >= need;
  }
  float extension_target(double best_cost) const {
    const float a = 16.0f * (std::fabs(hi) * 1e-4f + 1e-4f);
    const double b = 2.0 * std::fabs((double)hi - (double)start_value);
    float want = hi + (float)std::max((double)a, b);
    const double need = std::min(best_cost, bound);
    if (need < kInf)
      want = std::max(want, std::nextafter((float)(need / (double)G),
                                           std::numeric_limits<float>::infinity()));
    return want;
  }
};

struct Fetched {  // one request of a candidate fetch: ascending values and how many lie above
  std::vector<float> values;
  int above = 0;
};

// ---- two small kernels that keep dependent steps on the GPU ----

// Window request of every (instance, G) right after the bottleneck DP of all families
// (out[f][3][n], rows 1 and 2 = smallest feasible threshold and the stage-cost sum there): the
// family with the smallest threshold (the first of equals) gives the start of the window;
// req[0][i] = table row, req[1][i] = lo, req[2][i] = hi of the candidates to fetch, req[3][i] =
// the smallest feasible threshold itself; an empty window (lo = hi = +inf) when no family is
// feasible.  The bounds only size the fetch; what the scan does with the candidates follows the
// reference's rules on the values that lie inside.
__global__ void window_request_kernel(const float *__restrict__ out, int n_families, int n,
                                      const int32_t *__restrict__ rows,
                                      const int32_t *__restrict__ grad_accum, int n_grad_accum,
                                      double gap, float *__restrict__ req) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float bott = INFINITY, sum = INFINITY;
  for (int f = 0; f < n_families; ++f) {
    const float b = out[(size_t)f * 3 * n + n + i];
    if (b < bott) {
      bott = b;
      sum = out[(size_t)f * 3 * n + 2 * n + i];
    }
  }
  reinterpret_cast<int32_t *>(req)[i] = rows[i];
  req[3 * n + i] = bott;
  if (!(bott < INFINITY)) {
    req[n + i] = INFINITY;
    req[2 * n + i] = INFINITY;
    return;
  }
  const double G = (double)grad_accum[i % n_grad_accum];
  // the min-max partition is admissible at the bottleneck: its total bounds the scan's best;
  // the first KEPT candidate may lie a few gaps above, and when the bottleneck is a single-stage
  // cost (no candidate itself) a little further up
  const double cost0 = (double)sum + (G - 1.0) * (double)bott;
  const double room = (G - 1.0) * (4.0 * gap);
  float hi = nextafterf((float)((cost0 + room) * (1.0 + 1e-5) / G), INFINITY);
  hi = fmaxf(hi, (float)((double)bott * (1.0 + 2e-3) + 2e-4));
  req[n + i] = bott - (float)(1e-4 + 1e-5 * fabs((double)bott));
  req[2 * n + i] = hi;
}

// Strategy row of every stage of the walked partitions: stage i of partition k (path[k][i] =
// (end layer, n, m, ckpt), stages[k] of them) reads the row-index table of its variant
// (inter_tuning.py:38-60: whole model / first stage / last stage / inner stage) at table row
// g_rows[k], mesh (n, m), pre-saved micro-batches = stages after it.
__global__ void strategy_rows_kernel(const MistStrategyIndex tabs, const int32_t *__restrict__ path,
                                     const int32_t *__restrict__ best_s,
                                     const int32_t *__restrict__ g_rows, int n, int max_stages,
                                     int32_t *__restrict__ out) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n * max_stages) return;
  const int k = e / max_stages, i = e % max_stages;
  const int n_stages = best_s[k];
  int32_t row = -1;
  if (i < n_stages) {
    const int32_t *st = path + (size_t)e * 4;
    const int start = i == 0 ? 0 : path[(size_t)(e - 1) * 4] + 1;
    const int end = st[0], c = st[3];
    int q = -1;
    for (int m = 0; m < tabs.num_mesh; ++m)
      if (tabs.mesh_n[m] == st[1] && tabs.mesh_m[m] == st[2]) q = m;
    const int64_t L = tabs.num_layers, C = L + 1, S = tabs.sample_size, Q = tabs.num_mesh;
    const int64_t g = g_rows[k], l = end - start + 1, p = n_stages - i - 1;
    if (q >= 0 && end >= start && end < L && c >= 0 && c <= L && p < tabs.p_dim) {
      if (start == 0 && end == L - 1)
        row = tabs.index[3][((g * Q + q) * C + c) * S + tabs.slot];
      else if (end == L - 1)
        row = tabs.index[2][(((g * Q + q) * L + (l - 1)) * C + c) * S + tabs.slot];
      else
        row = tabs.index[start == 0 ? 1 : 0]
                        [((((g * Q + q) * tabs.p_dim + p) * L + (l - 1)) * C + c) * S + tabs.slot];
    }
  }
  out[e] = row;
}

struct Search {
  int n_families;
  const MistDpShape *shapes;  // [n_families]
  const MistDpCosts *costs;   // [n_families]
  const MistDpCosts *select_costs;  // tables the threshold candidates are taken from
  const MistStrategyIndex *strategy;  // may be null
  hipStream_t stream;
  Workspace *ws;
  int64_t launches = 0, fetches = 0, selected = 0, thresholds_run = 0, round_trips = 0,
          left_to_host = 0;

  // Stage counts the next run of a single family goes up to (0 = all of the shape's).  The
  // back-pointer run of a winner whose scan result has s stages stops there: the recurrence of
  // the stage counts 1..s is the same, no smaller count reaches its sum (the first count wins
  // ties), so the result and the back-pointers on its path are those of the full run.
  int stage_limit = 0;
  MistDpShape shape_of(int f) const {
    MistDpShape shape = shapes[f];
    if (n_families == 1 && stage_limit > 0) shape.max_stages = std::min(shape.max_stages, stage_limit);
    return shape;
  }
  size_t path_ints(int f) const { return (size_t)shape_of(f).max_stages * 4; }
  // ints in front of family f's partitions in the path buffers of a batch of n instances
  size_t path_offset(int f, int n) const {
    size_t at = 0;
    for (int k = 0; k < f; ++k) at += path_ints(k) * n;
    return at;
  }

  // DP instances (g_index[i], tmax[i]) of every family -> ws->h_out as [family][3][n] (best_s
  // bits, best_sum, stage_max); with `want_path` also the partitions (h_path, family after
  // family) and, when strategy tables were given, the strategy rows of their stages
  // (h_rows, same order without the factor 4).  `sync` false leaves the copies of the
  // outputs queued on the stream for the caller to wait for.
  int run(const std::vector<int32_t> &g_index, const std::vector<float> &tmax, int mode,
          bool want_path, bool sync = true) {
    const int n = (int)tmax.size();
    if (n == 0) return 0;
    const size_t n_out = (size_t)3 * n * n_families;
    // the partitions and their strategy rows lie behind the outputs: one copy back
    const size_t n_path = path_offset(n_families, n);
    const size_t n_back = n_out + (want_path ? n_path + n_path / 4 : 0);
    if (int rc = ws->h_in.reserve(sizeof(float) * 2 * n)) return rc;
    if (int rc = ws->d_in.reserve(sizeof(float) * 2 * n)) return rc;
    if (int rc = ws->d_out.reserve(sizeof(float) * n_back)) return rc;
    if (int rc = ws->h_out.reserve(sizeof(float) * n_back)) return rc;
    int32_t *d_paths = reinterpret_cast<int32_t *>(ws->d_out.as<float>() + n_out);
    int32_t *d_strategy_rows = d_paths + n_path;
    h_path = reinterpret_cast<const int32_t *>(ws->h_out.as<float>() + n_out);
    h_rows = h_path + n_path;
    int64_t n_scratch = 1;
    size_t slab = 0;
    for (int f = 0; f < n_families; ++f) {
      const int64_t want = mist_dp_scratch_floats(&shapes[f], n);
      if (want < 0) return MIST_E_INVALID;
      n_scratch = std::max(n_scratch, want);
      slab = std::max(slab, (size_t)(shapes[f].max_stages + 1) * (shapes[f].num_layers + 1) *
                                (shapes[f].num_devices + 1) * 4);
    }
    if (int rc = ws->d_scratch.reserve(sizeof(float) * (size_t)n_scratch)) return rc;
    if (want_path)
      if (int rc = ws->d_argmin.reserve(sizeof(int32_t) * slab * n)) return rc;
    float *h_in = ws->h_in.as<float>();
    std::memcpy(h_in, tmax.data(), sizeof(float) * n);
    std::memcpy(h_in + n, g_index.data(), sizeof(int32_t) * n);
    MIST_HIP_CHECK(hipMemcpyAsync(ws->d_in.ptr, h_in, sizeof(float) * 2 * n, hipMemcpyHostToDevice,
                                  stream));
    float *d_in = ws->d_in.as<float>();
    const int32_t *d_g = reinterpret_cast<int32_t *>(d_in + n);
    // the families share the state planes and the back-pointer slab: they run one after the
    // other on the stream
    for (int f = 0; f < n_families; ++f) {
      float *d_out = ws->d_out.as<float>() + (size_t)f * 3 * n;
      int32_t *d_argmin = want_path ? ws->d_argmin.as<int32_t>() : nullptr;  // no fill: the
                                                     // walk reads what the DP wrote
      const MistDpShape shape = shape_of(f);
      if (int rc = mist_dp_run(&shape, &costs[f], d_in, d_g, n, mode,
                               reinterpret_cast<int32_t *>(d_out), d_out + n, d_out + 2 * n,
                               d_argmin, ws->d_scratch.as<float>(), stream))
        return rc;
      if (want_path) {
        int32_t *d_path = d_paths + path_offset(f, n);
        if (int rc = mist_dp_backtrack(&shape, d_argmin, reinterpret_cast<int32_t *>(d_out), n,
                                       d_path, stream))
          return rc;
        if (strategy) {
          const int cells = n * shape.max_stages;
          hipLaunchKernelGGL(strategy_rows_kernel, dim3((cells + 63) / 64), dim3(64), 0, stream,
                             *strategy, d_path, reinterpret_cast<int32_t *>(d_out), d_g, n,
                             shape.max_stages, d_strategy_rows + path_offset(f, n) / 4);
          MIST_HIP_CHECK(hipGetLastError());
        }
      }
    }
    MIST_HIP_CHECK(hipMemcpyAsync(ws->h_out.ptr, ws->d_out.ptr, sizeof(float) * n_back,
                                  hipMemcpyDeviceToHost, stream));
    launches += n_families;
    thresholds_run += (int64_t)n * n_families;
    if (sync) {
      MIST_HIP_CHECK(hipStreamSynchronize(stream));
      ++round_trips;
    }
    return 0;
  }

  // best + (g - 1) * f_stage_max in float64 (inter_tuning.py:342) of family f, inf if infeasible
  double total_of(int f, int i, int n, int G, const float *out = nullptr) const {
    const float *h = (out ? out : ws->h_out.as<float>()) + (size_t)f * 3 * n;
    int32_t best_s;
    std::memcpy(&best_s, h + i, sizeof(best_s));
    if (best_s < 0) return kInf;
    return (double)h[n + i] + ((double)G - 1.0) * (double)h[2 * n + i];
  }
  // smallest family total (the first family wins ties); *family = the one that attains it
  double total(int i, int n, int G, int *family = nullptr, const float *out = nullptr,
               int *stages = nullptr, double *min_sum = nullptr) const {
    double best = kInf;
    if (min_sum) *min_sum = kInf;
    for (int f = 0; f < n_families; ++f) {
      const double c = total_of(f, i, n, G, out);
      if (min_sum && c < kInf)  // smallest stage-cost sum of any family that is feasible here
        *min_sum = std::min(*min_sum,
                            (double)((out ? out : ws->h_out.as<float>()) + (size_t)f * 3 * n)[n + i]);
      if (c < best) {
        best = c;
        if (family) *family = f;
        if (stages)
          std::memcpy(stages, (out ? out : ws->h_out.as<float>()) + (size_t)f * 3 * n + i, sizeof(int));
      }
    }
    return best;
  }

  // ascending candidates v of table row rows[r] with lo[r] < v <= hi[r], and how many lie above
  int fetch(const std::vector<int32_t> &rows, const std::vector<float> &lo,
            const std::vector<float> &hi, std::vector<Fetched> *out) {
    const int n = (int)rows.size();
    out->assign(n, Fetched());
    if (n == 0) return 0;
    if (int rc = ws->h_req.reserve(sizeof(float) * 3 * n)) return rc;
    if (int rc = ws->d_req.reserve(sizeof(float) * 3 * n)) return rc;
    float *h_req = ws->h_req.as<float>();
    std::memcpy(h_req, rows.data(), sizeof(int32_t) * n);
    std::memcpy(h_req + n, lo.data(), sizeof(float) * n);
    std::memcpy(h_req + 2 * n, hi.data(), sizeof(float) * n);
    MIST_HIP_CHECK(hipMemcpyAsync(ws->d_req.ptr, h_req, sizeof(float) * 3 * n,
                                  hipMemcpyHostToDevice, stream));
    return collect(n, out);
  }

  // The bottleneck DP of every (instance, G) and the first fetch of their windows in one round
  // trip: the requests are made on the GPU from the DP's outputs.  ws->h_out holds the DP
  // outputs afterwards, ws->h_req the requests as they were made ([3][n]: row, lo, hi).
  int bottleneck_and_fetch(const std::vector<int32_t> &rows, const int32_t *grad_accum,
                           int n_grad_accum, std::vector<Fetched> *out) {
    const int n = (int)rows.size();
    if (int rc = ws->h_grad.reserve(sizeof(int32_t) * n_grad_accum)) return rc;
    if (int rc = ws->d_grad.reserve(sizeof(int32_t) * n_grad_accum)) return rc;
    if (int rc = ws->h_req.reserve(sizeof(float) * 4 * n)) return rc;
    if (int rc = ws->d_req.reserve(sizeof(float) * 4 * n)) return rc;
    std::memcpy(ws->h_grad.ptr, grad_accum, sizeof(int32_t) * n_grad_accum);
    MIST_HIP_CHECK(hipMemcpyAsync(ws->d_grad.ptr, ws->h_grad.ptr, sizeof(int32_t) * n_grad_accum,
                                  hipMemcpyHostToDevice, stream));
    const std::vector<float> zeros(n, 0.0f);
    if (int rc = run(rows, zeros, MIST_DP_BOTTLENECK, false, /*sync=*/false)) return rc;
    hipLaunchKernelGGL(window_request_kernel, dim3((n + 63) / 64), dim3(64), 0, stream,
                       ws->d_out.as<float>(), n_families, n,
                       reinterpret_cast<const int32_t *>(ws->d_in.as<float>() + n),
                       ws->d_grad.as<int32_t>(), n_grad_accum, kGap, ws->d_req.as<float>());
    MIST_HIP_CHECK(hipGetLastError());
    MIST_HIP_CHECK(hipMemcpyAsync(ws->h_req.ptr, ws->d_req.ptr, sizeof(float) * 4 * n,
                                  hipMemcpyDeviceToHost, stream));
    out->assign(n, Fetched());
    return collect(n, out);
  }

  // The same, and the windows and the first scan batch with it (mist_dp_windows_first_batch +
  // the threshold DP of its instances for every family): one round trip.  Afterwards
  // ws->h_out holds the bottleneck DP's outputs; first_req the requests ([4][n]: row, lo, hi,
  // smallest feasible threshold), first_meta the windows' descriptions ([n][8]), first_kept
  // their kept thresholds and first_out the DP outputs of the batch
  // ([family][3][n * first_chunk]; the instances of window r start at first_meta[r][7]).
  const float *first_req = nullptr, *first_kept = nullptr, *first_out = nullptr;
  const int32_t *first_meta = nullptr;
  // partitions and strategy rows of the last run with `want_path` (behind its outputs in ws->h_out)
  const int32_t *h_path = nullptr, *h_rows = nullptr;
  int bottleneck_windows_first_batch(const std::vector<int32_t> &rows, const int32_t *grad_accum,
                                     int n_grad_accum, int window_capacity, int first_chunk) {
    const int n = (int)rows.size(), n_inst = n * first_chunk;
    if (int rc = ws->h_grad.reserve(sizeof(int32_t) * n_grad_accum)) return rc;
    if (int rc = ws->d_grad.reserve(sizeof(int32_t) * n_grad_accum)) return rc;
    if (int rc = ws->d_win_values.reserve(sizeof(float) * (size_t)n * window_capacity)) return rc;
    if (int rc = ws->d_win_counts.reserve(sizeof(int32_t) * (2 + 2 * (size_t)n))) return rc;
    if (int rc = ws->d_inst_t.reserve(sizeof(float) * n_inst)) return rc;
    if (int rc = ws->d_inst_row.reserve(sizeof(int32_t) * n_inst)) return rc;
    const size_t n_out = (size_t)3 * n_inst * n_families;
    // one buffer of 4-byte words: [requests 4 n][descriptions 8 n][outputs n_out][kept thresholds]
    const size_t at_meta = (size_t)4 * n, at_out = at_meta + (size_t)8 * n, at_kept = at_out + n_out;
    const size_t words = at_kept + kKeptCapacity;
    if (int rc = ws->d_first.reserve(sizeof(float) * words)) return rc;
    if (int rc = ws->h_first.reserve(sizeof(float) * words)) return rc;
    float *d_first = ws->d_first.as<float>(), *h_first = ws->h_first.as<float>();
    first_req = h_first;
    first_meta = reinterpret_cast<const int32_t *>(h_first + at_meta);
    first_out = h_first + at_out;
    first_kept = h_first + at_kept;
    // the state planes of the batch are the larger need: sized before anything is queued
    int64_t n_scratch = 1;
    for (int f = 0; f < n_families; ++f) {
      const int64_t want = mist_dp_scratch_floats(&shapes[f], n_inst);
      if (want < 0) return MIST_E_INVALID;
      n_scratch = std::max(n_scratch, want);
    }
    if (int rc = ws->d_scratch.reserve(sizeof(float) * (size_t)n_scratch)) return rc;
    std::memcpy(ws->h_grad.ptr, grad_accum, sizeof(int32_t) * n_grad_accum);
    MIST_HIP_CHECK(hipMemcpyAsync(ws->d_grad.ptr, ws->h_grad.ptr, sizeof(int32_t) * n_grad_accum,
                                  hipMemcpyHostToDevice, stream));
    const std::vector<float> zeros(n, 0.0f);
    if (int rc = run(rows, zeros, MIST_DP_BOTTLENECK, false, /*sync=*/false)) return rc;
    float *d_req = d_first;
    hipLaunchKernelGGL(window_request_kernel, dim3((n + 63) / 64), dim3(64), 0, stream,
                       ws->d_out.as<float>(), n_families, n,
                       reinterpret_cast<const int32_t *>(ws->d_in.as<float>() + n),
                       ws->d_grad.as<int32_t>(), n_grad_accum, kGap, d_req);
    MIST_HIP_CHECK(hipGetLastError());
    if (int rc = mist_dp_windows_first_batch(
            select_costs, n, reinterpret_cast<int32_t *>(d_req), d_req + n, d_req + 2 * n,
            d_req + 3 * n, kGap, window_capacity, first_chunk, kFirstLead,
            ws->d_win_values.as<float>(),
            ws->d_win_counts.as<int32_t>(), d_first + at_kept, kKeptCapacity,
            reinterpret_cast<int32_t *>(d_first + at_meta), ws->d_inst_t.as<float>(),
            ws->d_inst_row.as<int32_t>(), stream))
      return rc;
    for (int f = 0; f < n_families; ++f) {
      float *d_out = d_first + at_out + (size_t)f * 3 * n_inst;
      if (int rc = mist_dp_run(&shapes[f], &costs[f], ws->d_inst_t.as<float>(),
                               ws->d_inst_row.as<int32_t>(), n_inst, MIST_DP_THRESHOLD,
                               reinterpret_cast<int32_t *>(d_out), d_out + n_inst, d_out + 2 * n_inst,
                               nullptr, ws->d_scratch.as<float>(), stream))
        return rc;
    }
    MIST_HIP_CHECK(hipMemcpyAsync(h_first, d_first, sizeof(float) * (at_kept + kKeptHead),
                                  hipMemcpyDeviceToHost, stream));
    MIST_HIP_CHECK(hipStreamSynchronize(stream));
    ++round_trips;
    // kept thresholds beyond the part that travelled with the rest
    const int32_t *meta = first_meta;
    int64_t kept_end = 0;
    for (int r = 0; r < n; ++r)
      if (meta[8 * r + 2] == 0) kept_end = std::max<int64_t>(kept_end, (int64_t)meta[8 * r + 4] + meta[8 * r + 3]);
    if (kept_end > kKeptHead) {
      MIST_HIP_CHECK(hipMemcpyAsync(h_first + at_kept + kKeptHead, d_first + at_kept + kKeptHead,
                                    sizeof(float) * (size_t)(kept_end - kKeptHead),
                                    hipMemcpyDeviceToHost, stream));
      MIST_HIP_CHECK(hipStreamSynchronize(stream));
      ++round_trips;
    }
    return 0;
  }

  // runs the n requests that lie in ws->d_req and sorts what comes back by request
  int collect(int n, std::vector<Fetched> *out) {
    ++fetches;
    if (int rc = ws->d_counts.reserve(sizeof(int32_t) * (1 + n))) return rc;
    if (int rc = ws->h_counts.reserve(sizeof(int32_t) * (1 + n))) return rc;
    float *d_req = ws->d_req.as<float>();
    int total = 0, head = 0;
    for (;;) {
      const int capacity = ws->select_capacity;
      if (int rc = ws->d_values.reserve(sizeof(float) * capacity)) return rc;
      if (int rc = ws->d_request.reserve(sizeof(int32_t) * capacity)) return rc;
      MIST_HIP_CHECK(hipMemsetAsync(ws->d_counts.ptr, 0, sizeof(int32_t) * (1 + n), stream));
      if (int rc = mist_dp_select_candidates(
              select_costs, n, reinterpret_cast<int32_t *>(d_req), d_req + n, d_req + 2 * n,
              ws->d_values.as<float>(), ws->d_request.as<int32_t>(), capacity,
              ws->d_counts.as<int32_t>(), stream))
        return rc;
      MIST_HIP_CHECK(hipMemcpyAsync(ws->h_counts.ptr, ws->d_counts.ptr, sizeof(int32_t) * (1 + n),
                                    hipMemcpyDeviceToHost, stream));
      // the first kSelectHead values and requests travel with the counts: when they are all
      // there is (the usual case) the fetch is one round trip
      head = std::min(capacity, kSelectHead);
      if (int rc = ws->h_values.reserve(sizeof(float) * head)) return rc;
      if (int rc = ws->h_request.reserve(sizeof(int32_t) * head)) return rc;
      MIST_HIP_CHECK(hipMemcpyAsync(ws->h_values.ptr, ws->d_values.ptr, sizeof(float) * head,
                                    hipMemcpyDeviceToHost, stream));
      MIST_HIP_CHECK(hipMemcpyAsync(ws->h_request.ptr, ws->d_request.ptr, sizeof(int32_t) * head,
                                    hipMemcpyDeviceToHost, stream));
      MIST_HIP_CHECK(hipStreamSynchronize(stream));
      ++round_trips;
      total = ws->h_counts.as<int32_t>()[0];
      if (total <= capacity) break;
      ws->select_capacity = 2 * total;
    }
    selected += total;
    const int32_t *h_counts = ws->h_counts.as<int32_t>();
    for (int r = 0; r < n; ++r) (*out)[r].above = h_counts[1 + r];
    if (total == 0) return 0;
    if (total > head) {
      if (int rc = ws->h_values.reserve(sizeof(float) * total)) return rc;
      if (int rc = ws->h_request.reserve(sizeof(int32_t) * total)) return rc;
      MIST_HIP_CHECK(hipMemcpyAsync(ws->h_values.ptr, ws->d_values.ptr, sizeof(float) * total,
                                    hipMemcpyDeviceToHost, stream));
      MIST_HIP_CHECK(hipMemcpyAsync(ws->h_request.ptr, ws->d_request.ptr, sizeof(int32_t) * total,
                                    hipMemcpyDeviceToHost, stream));
      MIST_HIP_CHECK(hipStreamSynchronize(stream));
      ++round_trips;
    }
    const float *values = ws->h_values.as<float>();
    const int32_t *request = ws->h_request.as<int32_t>();
    std::vector<int> count(n, 0);
    for (int i = 0; i < total; ++i) ++count[request[i]];
    for (int r = 0; r < n; ++r) (*out)[r].values.reserve(count[r]);
    for (int i = 0; i < total; ++i) (*out)[request[i]].values.push_back(values[i]);
    for (int r = 0; r < n; ++r) sort_ascending(&(*out)[r].values);
    return 0;
  }

  // The values of a window are finite and lie in a narrow range: one pass into equal-width
  // buckets and an insertion sort of what lands in each beat a comparison sort several times.
  static void sort_ascending(std::vector<float> *v) {
    const size_t n = v->size();
    if (n < 64) {
      std::sort(v->begin(), v->end());
      return;
    }
    const auto [lo_it, hi_it] = std::minmax_element(v->begin(), v->end());
    const double lo = *lo_it, span = (double)*hi_it - lo;
    if (!(span > 0.0)) return;
    const size_t n_buckets = n / 4 + 1;
    const double scale = (double)(n_buckets - 1) / span;
    std::vector<uint32_t> start(n_buckets + 1, 0);
    std::vector<uint32_t> bucket(n);
    for (size_t i = 0; i < n; ++i) {
      bucket[i] = (uint32_t)(((double)(*v)[i] - lo) * scale);
      ++start[bucket[i] + 1];
    }
    for (size_t b = 0; b < n_buckets; ++b) start[b + 1] += start[b];
    std::vector<float> sorted(n);
    std::vector<uint32_t> cursor(start.begin(), start.end() - 1);
    for (size_t i = 0; i < n; ++i) sorted[cursor[bucket[i]]++] = (*v)[i];
    for (size_t i = 1; i < n; ++i) {  // buckets are ordered: elements move a few places at most
      const float x = sorted[i];
      size_t j = i;
      while (j > 0 && sorted[j - 1] > x) {
        sorted[j] = sorted[j - 1];
        --j;
      }
      sorted[j] = x;
    }
    v->swap(sorted);
  }

  int extend(Window *w, double best_cost) {
    const float want = w->extension_target(best_cost);
    std::vector<Fetched> got;
    if (int rc = fetch({w->row}, {w->hi}, {want}, &got)) return rc;
    return apply_extension(w, got[0], want);
  }

  // `got` = ascending candidates in (hi, want]: continue the gap walk from the last kept one
  int apply_extension(Window *w, const Fetched &got, float want) {
    std::vector<float> in, kept;
    const bool resume = !w->kept.empty();
    if (resume) in.push_back(w->kept.back());
    in.insert(in.end(), got.values.begin(), got.values.end());
    kept.resize(in.size());
    const int n = mist_dp_filter_tmax(in.data(), (int)in.size(), kGap, kept.data());
    if (n < 0) return n;
    w->hi = want;
    w->complete = got.above == 0;
    const int skip = resume && n > 0 ? 1 : 0;  // the walk keeps its first element
    w->append(kept.data() + skip, (size_t)(n - skip));
    return 0;
  }
};

// Replay state of inter_stage_tune_with_fixed_grad_accumu (inter_tuning.py:163-217) for one G.
//
// The reference runs the DP at every kept threshold below best / G.  Most of those runs change
// nothing, and for many that can be told from the outcome at a LATER threshold j: the DP at
// threshold i returns the partition the DP at i - 1 returned unless that one uses a stage cost
// above threshold i - 1 (same visiting order, strict "<": the first best candidate of a state
// among more candidates, if it is one of the fewer, is the first best among those too), and the
// same partition gives the same total, which is no improvement.  A partition that is new at i
// has a stage above threshold i - 1 and stage costs that sum to no less than the smallest sum at
// j >= i (the admissible costs only grow with the threshold; float32 adds are monotone), so its
// total is at least sum(j) + (G - 1) threshold(i - 1).  While that is no smaller than the running
// best, no threshold up to j improves it and the scan passes them without their outcomes.
struct Outcome {
  double cost = kInf;  // total of the DP's partition, inf = infeasible
  double sum = kInf;   // smallest stage-cost sum of a feasible family
  int stages = 0;
};
struct Scan {
  int G = 1;
  Window *w = nullptr;
  size_t pos = 0;    // next threshold the sequential scan looks at
  size_t first = 0;  // the first one at or above the smallest feasible threshold
  std::map<size_t, Outcome> known;  // DP outcomes by index of the kept threshold
  int limit = kFirstChunk;
  // thresholds t with t * G >= cap are not tried (kInf: the reference's stop rule alone): the
  // caller's tables hold their values only up to cap / G
  double cap = kInf;
  size_t n_kept() const { return w ? w->kept.size() : 0; }
  // lower bound of the total of any improvement at thresholds pos..j, from the sum at j
  double floor_total(size_t at, double sum_later) const {
    const double prev = at > first ? (double)w->kept[at - 1] : (double)w->start_value;
    return (sum_later + (double)(G - 1) * prev) * (1.0 - kFloorSlack);
  }
};

}  // namespace

extern "C" {

int mist_sizeof_strategy_index(void) { return (int)sizeof(MistStrategyIndex); }

static int search_families(int n_families, const MistDpShape *shapes,
                           const MistDpCosts *costs, const MistDpCosts *select_costs,
                           const MistStrategyIndex *strategy, int n_instances,
                           int n_grad_accum, const int32_t *rows,
                           const int32_t *grad_accum, int only_best_path, double *out_cost,
                           int32_t *out_g, float *out_tmax, int32_t *out_family,
                           int32_t *out_stages, int32_t *out_path, int32_t *out_rows,
                           int64_t *out_stats, void *stream_, const double *host_estimate,
                           double limit_factor, int32_t *out_unresolved) {
  if (out_unresolved) *out_unresolved = 0;
  if (!shapes || !costs || !select_costs || !rows || !grad_accum || !out_cost || !out_g ||
      !out_tmax || !out_family || !out_stages || !out_path)
    return fail(MIST_E_INVALID, "null pointer argument");
  if (n_families < 1) return fail(MIST_E_INVALID, "need at least one DP family, got %d", n_families);
  if (n_instances < 1 || n_grad_accum < 1)
    return fail(MIST_E_INVALID, "need at least one instance and one G, got %d x %d", n_instances,
                n_grad_accum);
  if ((int64_t)n_instances * n_grad_accum > 65535)
    return fail(MIST_E_INVALID, "%d x %d (instance, G) pairs; at most 65535", n_instances,
                n_grad_accum);
  if (strategy && !out_rows) return fail(MIST_E_INVALID, "strategy tables without out_rows");
  int S_max = 0;
  for (int f = 0; f < n_families; ++f) {
    if (mist_dp_scratch_floats(&shapes[f], 1) < 0) return MIST_E_INVALID;  // message set by the check
    if (shapes[f].num_layers != shapes[0].num_layers)
      return fail(MIST_E_INVALID, "family %d has %d layers, family 0 has %d", f,
                  shapes[f].num_layers, shapes[0].num_layers);
    S_max = std::max(S_max, shapes[f].max_stages);
  }
  if (strategy) {
    if (strategy->num_layers != shapes[0].num_layers || strategy->num_mesh < 1 ||
        strategy->num_mesh > MIST_MAX_MESH || strategy->p_dim < 1 || strategy->sample_size < 1 ||
        strategy->slot < 0 || strategy->slot >= strategy->sample_size)
      return fail(MIST_E_INVALID, "strategy tables do not fit the DP shape");
    for (int v = 0; v < 4; ++v)
      if (!strategy->index[v]) return fail(MIST_E_INVALID, "null strategy index table %d", v);
  }
  for (int i = 0; i < n_grad_accum; ++i)
    if (grad_accum[i] < 1) return fail(MIST_E_INVALID, "grad_accum[%d] = %d < 1", i, grad_accum[i]);

  std::lock_guard<std::mutex> guard(g_lock);
  int device = 0;
  MIST_HIP_CHECK(hipGetDevice(&device));
  Search S{n_families, shapes, costs, select_costs, strategy, (hipStream_t)stream_,
           &g_workspaces[device]};
  const int n_flat = n_instances * n_grad_accum;

  std::vector<int32_t> flat_rows(rows, rows + n_flat);
  std::vector<Window> windows(n_flat);
  // smallest feasible threshold (+inf if none) and the stage-cost sum there, from the outputs of
  // the bottleneck DP of every family (the first family with the smallest threshold)
  auto bottleneck_of = [&](int i, float *bott, float *sum) {
    const float *h = S.ws->h_out.as<float>();
    *bott = *sum = std::numeric_limits<float>::infinity();
    for (int f = 0; f < n_families; ++f) {
      const float b = h[(size_t)f * 3 * n_flat + n_flat + i];
      if (b < *bott) {
        *bott = b;
        *sum = h[(size_t)f * 3 * n_flat + 2 * n_flat + i];
      }
    }
  };

  // Decides windows on the host: `got[j]` = the ascending candidates of window todo[j] in
  // (lo[j], hi[j]] and how many lie above.  A window whose fetched part holds no certain start
  // of the walk is fetched again from further below; one whose first kept candidate lies higher
  // than assumed is extended upwards.
  auto decide_on_host = [&](const std::vector<int> &todo, std::vector<Fetched> got,
                            std::vector<float> lo, std::vector<float> hi) -> int {
    const std::vector<float> hi_first = hi;
    std::vector<int> pending(todo.size());
    for (size_t k = 0; k < pending.size(); ++k) pending[k] = (int)k;
    for (int widen = 0; !pending.empty(); ++widen) {
      if (widen > 0) {
        std::vector<int32_t> r;
        lo.clear();
        hi.clear();
        for (int k : pending) {
          const Window &w = windows[todo[k]];
          r.push_back(w.row);
          lo.push_back(widen >= 8 ? -std::numeric_limits<float>::infinity() : w.lower_margin(widen));
          hi.push_back(hi_first[k]);
        }
        if (int rc = S.fetch(r, lo, hi, &got)) return rc;
      }
      std::vector<int> again;
      std::vector<float> kept;
      for (size_t j = 0; j < pending.size(); ++j) {
        Window &w = windows[todo[pending[j]]];
        w.hi = hi[j];
        w.complete = got[j].above == 0;
        const std::vector<float> &v = got[j].values;
        if (v.empty()) continue;
        const bool below = std::isinf(lo[j]);
        kept.resize(v.size());
        const int n = mist_dp_window_begin(v.data(), (int)v.size(), below ? 0.0f : lo[j],
                                           below ? 1 : 0, w.start_value, kGap, kept.data());
        if (n == MIST_DP_NO_START) {
          again.push_back(pending[j]);
          continue;
        }
        if (n < 0) return n;
        w.append(kept.data(), (size_t)n);
      }
      pending.swap(again);
    }
    // one more pass for the windows whose first kept candidate lies higher than assumed
    std::vector<Window *> brief;
    for (int i : todo)
      if (!windows[i].covers(kInf)) brief.push_back(&windows[i]);
    if (!brief.empty()) {
      std::vector<int32_t> r;
      std::vector<float> from, want;
      for (Window *w : brief) {
        r.push_back(w->row);
        from.push_back(w->hi);
        want.push_back(w->extension_target(kInf));
      }
      std::vector<Fetched> more;
      if (int rc = S.fetch(r, from, want, &more)) return rc;
      for (size_t j = 0; j < brief.size(); ++j)
        if (int rc = S.apply_extension(brief[j], more[j], want[j])) return rc;
    }
    return 0;
  };
  auto new_window = [&](int i, float bott, float sum) -> Window & {
    Window &w = windows[i];
    w = Window();
    w.exists = true;
    w.row = flat_rows[i];
    w.G = grad_accum[i % n_grad_accum];
    w.start_value = bott;
    w.start_sum = (double)sum;
    return w;
  };

  std::vector<int> first_batch(n_flat, 0);  // instances of a window the first batch has run
  const char *capacity_env = getenv("MIST_INTER_WINDOW_CAPACITY");  // for tests
  const int window_capacity = capacity_env ? atoi(capacity_env) : kWindowCapacity;
  const bool on_device = !getenv("MIST_INTER_HOST_WINDOWS") && (int64_t)n_flat * kFirstChunk <= 65535;
  if (on_device) {
    // ---- smallest feasible threshold of every (instance, G), its window of kept thresholds
    // and the first scan batch, all decided on the device: one round trip.  A window the
    // device cannot decide (more candidates than it holds, no certain start, nothing kept at or
    // above the start inside the first fetch) is decided on the host afterwards and joins the
    // scan with the second batch. ----
    if (int rc = S.bottleneck_windows_first_batch(flat_rows, grad_accum, n_grad_accum,
                                                  window_capacity, kFirstChunk))
      return rc;
    const float *req = S.first_req;
    const int32_t *meta = S.first_meta;
    const float *kept = S.first_kept;
    std::vector<int> undecided;
    std::vector<int32_t> u_rows;
    std::vector<float> u_lo, u_hi;
    int64_t instances = 0;
    ++S.fetches;
    for (int i = 0; i < n_flat; ++i) {
      float bott, sum;
      bottleneck_of(i, &bott, &sum);
      if (!std::isfinite(bott)) continue;
      const int32_t *m = meta + 8 * i;
      Window &w = new_window(i, bott, sum);
      bool decided = m[2] == 0 && req[3 * n_flat + i] == bott;
      if (decided) {
        w.hi = req[2 * n_flat + i];
        w.complete = m[1] == 0;
        w.append(kept + m[4], (size_t)m[3]);
        const size_t pos = (size_t)(std::lower_bound(w.kept.begin(), w.kept.end(), w.start_value) -
                                    w.kept.begin());
        // (the host route extends a window that does not reach its bound before its first batch)
        decided = w.covers(kInf) && pos == (size_t)m[5];
      }
      if (decided) {
        first_batch[i] = m[6];
        S.selected += m[0];
        instances += m[6];
      } else {
        new_window(i, bott, sum);
        undecided.push_back(i);
        u_rows.push_back(flat_rows[i]);
        u_lo.push_back(req[n_flat + i]);
        u_hi.push_back(req[2 * n_flat + i]);
      }
    }
    if (instances > 0) S.launches += n_families;  // (an all-empty batch is no DP batch)
    S.thresholds_run += instances * n_families;
    S.left_to_host = (int64_t)undecided.size();
    if (!undecided.empty()) {
      std::vector<Fetched> got;
      if (int rc = S.fetch(u_rows, u_lo, u_hi, &got)) return rc;
      if (int rc = decide_on_host(undecided, std::move(got), u_lo, u_hi)) return rc;
    }
  } else {
    // ---- the host route: smallest feasible threshold of every (instance, G) and the first
    // fetch of its window in one round trip, the windows decided here ----
    std::vector<Fetched> first;
    if (int rc = S.bottleneck_and_fetch(flat_rows, grad_accum, n_grad_accum, &first)) return rc;
    const float *req = S.ws->h_req.as<float>();
    std::vector<int> feasible;
    std::vector<Fetched> got;
    std::vector<float> lo, hi;
    for (int i = 0; i < n_flat; ++i) {
      float bott, sum;
      bottleneck_of(i, &bott, &sum);
      if (!std::isfinite(bott)) continue;
      new_window(i, bott, sum);
      feasible.push_back(i);
      got.push_back(std::move(first[i]));
      lo.push_back(req[n_flat + i]);
      hi.push_back(req[2 * n_flat + i]);
    }
    if (int rc = decide_on_host(feasible, std::move(got), lo, hi)) return rc;
  }

  // ---- speculative batches + sequential replay ----
  struct Chain {
    std::vector<Scan> scans;
    size_t current = 0;
    double best_cost = kInf;
    int best_g = -1, best_stages = 0;
    float best_t = 0.0f;
  };
  // Exact part of the caller's tables (a search over tables that hold their values up to
  // limit(G) = estimate * limit_factor / G only): the estimate has arrived with the first round
  // trip (it was copied on this stream before the search was called).
  std::vector<float> limit_t(n_grad_accum, std::numeric_limits<float>::infinity());
  const bool bounded = host_estimate != nullptr && std::isfinite(*host_estimate);
  if (bounded)
    for (int i = 0; i < n_grad_accum; ++i)
      limit_t[i] = (float)(*host_estimate * limit_factor / (double)grad_accum[i]);
  // per (instance, G): the running best when the scan of G ended, and the cost of the best
  // partition whose stages all lie within limit(G)
  std::vector<double> best_after(bounded ? n_flat : 0, kInf), within_limit(bounded ? n_flat : 0, kInf);
  bool within_limit_known = !bounded;
  std::vector<Chain> chains(n_instances);
  for (int t = 0; t < n_instances; ++t) {
    chains[t].scans.resize(n_grad_accum);
    for (int i = 0; i < n_grad_accum; ++i) {
      Scan &sc = chains[t].scans[i];
      Window &w = windows[t * n_grad_accum + i];
      sc.G = grad_accum[i];
      if (bounded) sc.cap = (double)limit_t[i] * (double)grad_accum[i];
      sc.w = w.exists ? &w : nullptr;
      if (sc.w)
        sc.pos = (size_t)(std::lower_bound(w.kept.begin(), w.kept.end(), w.start_value) -
                          w.kept.begin());
      sc.first = sc.pos;  // everything below is infeasible: the scan passes it unchanged
      // the results of the first batch, when the device has run it: the thresholds the scan
      // below would have asked for first, the next request of this G grows as after any request
      const int idx = t * n_grad_accum + i, n_first = first_batch[idx];
      const int at = on_device ? S.first_meta[8 * idx + 7] : 0;
      const int n_avail = (int)(sc.n_kept() - sc.first);
      for (int k = 0; k < n_first; ++k) {
        Outcome o;
        o.cost = S.total(at + k, n_flat * kFirstChunk, sc.G, nullptr, S.first_out, &o.stages, &o.sum);
        sc.known[sc.first + (size_t)mist_dp_first_batch_index(k, n_avail, kFirstChunk, kFirstLead)] = o;
      }
      if (n_first > 0) sc.limit = std::min(kMaxChunk, sc.limit * 4);
    }
  }
  int rc_inner = 0;
  // makes sure threshold `pos` is materialised if the scan can get there
  auto reach = [&](Scan &sc, size_t pos, double best_cost) -> bool {
    Window *w = sc.w;
    best_cost = std::min(best_cost, sc.cap);
    while (w && pos >= w->kept.size() && !w->covers(best_cost)) {
      if (int rc = S.extend(w, best_cost)) {
        rc_inner = rc;
        return false;
      }
    }
    return pos < sc.n_kept();
  };
  // advances the sequential scan as far as the computed results allow; true = this G is done
  auto replay = [&](Scan &sc, double &best_cost, bool &improved, float &best_t,
                    int &best_stages) -> bool {
    for (;;) {
      if (!reach(sc, sc.pos, best_cost)) return true;
      if (sc.w->scaled[sc.pos] >= std::min(best_cost, sc.cap)) return true;  // inter_tuning.py:196-197
      const auto later = sc.known.lower_bound(sc.pos);
      if (later != sc.known.end() && sc.floor_total(sc.pos, later->second.sum) >= best_cost) {
        sc.pos = later->first + 1;  // nothing up to there improves the best
        continue;
      }
      if (later == sc.known.end() || later->first != sc.pos) return false;  // needs more DP results
      const Outcome &o = later->second;
      if (o.cost < best_cost) {
        best_cost = o.cost;
        best_t = sc.w->kept[sc.pos];
        best_stages = o.stages;
        improved = true;
      }
      ++sc.pos;
    }
  };
  // Dry run of replay under the bound `best_cost` (the running best when this G is reached is no
  // larger, so the true scan passes no fewer thresholds): the thresholds whose outcomes it would
  // miss, at most sc.limit of them (it goes on as if they improved nothing), and, if it stops at
  // that limit, kProbes more spread over what it did not get to.  A scan without any outcome
  // asks for its first batch (mist_dp_first_batch_index over everything below the bound).
  auto wanted = [&](Scan &sc, double best_cost, std::vector<size_t> *out) {
    out->clear();
    if (!sc.w) return;
    auto stop_of = [&](double bound) {
      return (size_t)(std::lower_bound(sc.w->scaled.begin(), sc.w->scaled.end(), bound) -
                      sc.w->scaled.begin());
    };
    if (sc.known.empty()) {
      reach(sc, sc.pos + (size_t)kFirstChunk, best_cost);
      if (rc_inner) return;
      const size_t stop = stop_of(std::min(best_cost, sc.cap));
      if (stop <= sc.pos) return;
      const int n_avail = (int)(stop - sc.pos), n = std::min(kFirstChunk, n_avail);
      for (int k = 0; k < n; ++k)
        out->push_back(sc.pos + (size_t)mist_dp_first_batch_index(k, n_avail, kFirstChunk, kFirstLead));
      return;
    }
    size_t pos = sc.pos;
    int budget = sc.limit;
    bool cut = false;
    while (reach(sc, pos, best_cost)) {
      if (sc.w->scaled[pos] >= std::min(best_cost, sc.cap)) break;
      const auto later = sc.known.lower_bound(pos);
      if (later != sc.known.end() && sc.floor_total(pos, later->second.sum) >= best_cost) {
        pos = later->first + 1;
        continue;
      }
      if (later != sc.known.end() && later->first == pos) {
        best_cost = std::min(best_cost, later->second.cost);
      } else {
        if (budget == 0) {
          cut = true;
          break;
        }
        out->push_back(pos);
        --budget;
      }
      ++pos;
    }
    if (rc_inner || !cut) return;
    const size_t stop = stop_of(std::min(best_cost, sc.cap));
    size_t last = 0;
    for (int k = 0; k < kProbes && stop > pos; ++k) {
      const size_t step = ((size_t)(k + 1) * (stop - pos)) / kProbes;
      if (step == 0) continue;
      const size_t at = pos + step - 1;
      if ((k > 0 && at <= last) || sc.known.count(at)) continue;
      out->push_back(at);
      last = at;
    }
  };
  struct Span {
    int t, i, first, n;  // the indices of the span: req_at[first .. first + n)
  };
  for (;;) {
    std::vector<int32_t> req_g;
    std::vector<float> req_t;
    std::vector<int> req_G;
    std::vector<size_t> req_at, ask;
    std::vector<Span> spans;
    bool all_done = true;
    for (int t = 0; t < n_instances; ++t) {
      Chain &ch = chains[t];
      while (ch.current < ch.scans.size()) {  // commit the sequential scan as far as possible
        Scan &sc = ch.scans[ch.current];
        bool improved = false;
        float best_t = ch.best_t;
        int best_stages = ch.best_stages;
        const bool finished = replay(sc, ch.best_cost, improved, best_t, best_stages);
        if (rc_inner) return rc_inner;
        if (improved) {
          ch.best_g = (int)ch.current;
          ch.best_t = best_t;
          ch.best_stages = best_stages;
        }
        if (!finished) break;
        if (bounded) best_after[t * n_grad_accum + (int)ch.current] = ch.best_cost;
        ++ch.current;
      }
      if (ch.current < ch.scans.size()) all_done = false;
      for (size_t i = ch.current; i < ch.scans.size(); ++i) {
        Scan &sc = ch.scans[i];
        wanted(sc, ch.best_cost, &ask);
        if (rc_inner) return rc_inner;
        if (ask.empty()) continue;
        // the range grows fourfold every time the same G asks again
        sc.limit = std::min(kMaxChunk, sc.limit * 4);
        spans.push_back(Span{t, (int)i, (int)req_at.size(), (int)ask.size()});
        for (size_t at : ask) {
          req_g.push_back(rows[t * n_grad_accum + (int)i]);
          req_t.push_back(sc.w->kept[at]);
          req_G.push_back(sc.G);
          req_at.push_back(at);
        }
      }
    }
    if (all_done && within_limit_known) break;
    if (spans.empty() && within_limit_known)
      return fail(MIST_E_INVALID, "inter-stage scan made no progress");
    // the DP at limit(G) of every (instance, G) with a window travels with the first batch
    const int n_scan_requests = (int)req_t.size();
    std::vector<int> limit_of;
    // (no partition of a pair costs less than G x its smallest feasible threshold: a pair for
    // which that is not below estimate * limit_factor has nothing to report)
    if (!within_limit_known)
      for (int i = 0; i < n_flat; ++i)
        if (windows[i].exists && (double)windows[i].start_value * (double)windows[i].G <
                                     *host_estimate * limit_factor) {
          limit_of.push_back(i);
          req_g.push_back(flat_rows[i]);
          req_t.push_back(limit_t[i % n_grad_accum]);
        }
    if (req_t.empty()) break;  // (nothing feasible anywhere)
    if (int rc = S.run(req_g, req_t, MIST_DP_THRESHOLD, false)) return rc;
    const int n = (int)req_t.size();
    for (size_t k = 0; k < limit_of.size(); ++k)
      within_limit[limit_of[k]] = S.total(n_scan_requests + (int)k, n,
                                          grad_accum[limit_of[k] % n_grad_accum], nullptr, nullptr,
                                          nullptr, nullptr);
    within_limit_known = true;
    for (const Span &sp : spans) {
      Scan &sc = chains[sp.t].scans[sp.i];
      for (int k = sp.first; k < sp.first + sp.n; ++k) {
        Outcome o;
        o.cost = S.total(k, n, req_G[k], nullptr, nullptr, &o.stages, &o.sum);
        sc.known[req_at[k]] = o;
      }
    }
  }

  // A partition inside the exact part of the tables that is cheaper than what the scan of its G
  // ended with was admissible at no threshold the scan tried: the reference may or may not find
  // it at a threshold above limit(G), which these tables cannot tell.  (One that costs
  // estimate * limit_factor or more changes nothing the scan does below the limits.)
  if (bounded && out_unresolved)
    for (int i = 0; i < n_flat; ++i)
      if (within_limit[i] < std::min(best_after[i], *host_estimate * limit_factor)) ++*out_unresolved;

  // ---- results and the partitions of the winners ----
  std::vector<int> winners;
  for (int t = 0; t < n_instances; ++t) {
    const Chain &ch = chains[t];
    out_cost[t] = ch.best_cost;
    out_g[t] = ch.best_g;
    out_tmax[t] = ch.best_g >= 0 ? ch.best_t : 0.0f;
    out_family[t] = -1;
    out_stages[t] = 0;
    for (int k = 0; k < S_max * 4; ++k) out_path[(size_t)t * S_max * 4 + k] = -1;
    if (out_rows)
      for (int k = 0; k < S_max; ++k) out_rows[(size_t)t * S_max + k] = -1;
    if (ch.best_g >= 0) winners.push_back(t);
  }
  if (only_best_path && !winners.empty()) {
    int best = winners[0];
    for (int t : winners)
      if (chains[t].best_cost < chains[best].best_cost) best = t;  // the first of equals stays
    winners.assign(1, best);
  }
  if (!winners.empty()) {
    std::vector<int32_t> g;
    std::vector<float> tm;
    int most_stages = 0;
    for (int t : winners) {
      g.push_back(rows[t * n_grad_accum + chains[t].best_g]);
      tm.push_back(chains[t].best_t);
      most_stages = std::max(most_stages, chains[t].best_stages);
    }
    S.stage_limit = most_stages;  // no winner has more stages than this
    if (int rc = S.run(g, tm, MIST_DP_THRESHOLD, true)) return rc;
    const int n = (int)winners.size();
    for (int k = 0; k < n; ++k) {
      const int t = winners[k];
      int family = -1;
      const double again = S.total(k, n, grad_accum[chains[t].best_g], &family);
      if (family < 0 || again != chains[t].best_cost)
        return fail(MIST_E_INVALID, "back-pointer run of instance %d gives %.17g, the scan %.17g", t,
                    again, chains[t].best_cost);
      int32_t best_s;
      std::memcpy(&best_s, S.ws->h_out.as<float>() + (size_t)family * 3 * n + k, sizeof(best_s));
      const size_t per = S.path_ints(family), at = S.path_offset(family, n) + (size_t)k * per;
      out_family[t] = family;
      out_stages[t] = best_s;
      std::memcpy(out_path + (size_t)t * S_max * 4, S.h_path + at,
                  sizeof(int32_t) * per);
      if (strategy)
        std::memcpy(out_rows + (size_t)t * S_max, S.h_rows + at / 4,
                    sizeof(int32_t) * per / 4);
    }
  }
  if (out_stats) {
    out_stats[0] = S.launches;
    out_stats[1] = S.fetches;
    out_stats[2] = S.selected;
    out_stats[3] = S.thresholds_run;
    out_stats[4] = S.round_trips;
    out_stats[5] = S.left_to_host;
  }
  return 0;
}

int mist_inter_stage_search_families(int n_families, const MistDpShape *shapes,
                                     const MistDpCosts *costs, const MistDpCosts *select_costs,
                                     const MistStrategyIndex *strategy, int n_instances,
                                     int n_grad_accum, const int32_t *rows,
                                     const int32_t *grad_accum, int only_best_path, double *out_cost,
                                     int32_t *out_g, float *out_tmax, int32_t *out_family,
                                     int32_t *out_stages, int32_t *out_path, int32_t *out_rows,
                                     int64_t *out_stats, void *stream) {
  return search_families(n_families, shapes, costs, select_costs, strategy, n_instances,
                         n_grad_accum, rows, grad_accum, only_best_path, out_cost, out_g, out_tmax,
                         out_family, out_stages, out_path, out_rows, out_stats, stream, nullptr, 0.0,
                         nullptr);
}

int mist_inter_stage_search_bounded(int n_families, const MistDpShape *shapes,
                                    const MistDpCosts *costs, const MistDpCosts *select_costs,
                                    const MistStrategyIndex *strategy, int n_instances,
                                    int n_grad_accum, const int32_t *rows,
                                    const int32_t *grad_accum, int only_best_path, double *out_cost,
                                    int32_t *out_g, float *out_tmax, int32_t *out_family,
                                    int32_t *out_stages, int32_t *out_path, int32_t *out_rows,
                                    int64_t *out_stats, void *stream, const double *host_estimate,
                                    double limit_factor, int32_t *out_unresolved) {
  if (!host_estimate || !out_unresolved) return fail(MIST_E_INVALID, "null pointer argument");
  if (!(limit_factor > 0.0)) return fail(MIST_E_INVALID, "limit_factor must be positive");
  return search_families(n_families, shapes, costs, select_costs, strategy, n_instances,
                         n_grad_accum, rows, grad_accum, only_best_path, out_cost, out_g, out_tmax,
                         out_family, out_stages, out_path, out_rows, out_stats, stream,
                         host_estimate, limit_factor, out_unresolved);
}

int mist_inter_stage_search(const MistDpShape *shape, const MistDpCosts *costs, int n_instances,
                            int n_grad_accum, const int32_t *rows, const int32_t *grad_accum,
                            int only_best_path, double *out_cost, int32_t *out_g, float *out_tmax,
                            int32_t *out_stages, int32_t *out_path, int64_t *out_stats,
                            void *stream) {
  if (!shape) return fail(MIST_E_INVALID, "null pointer argument");
  if (shape->free_devices != 0)
    return fail(MIST_E_INVALID, "a single family must be the per-mesh recurrence");
  if (n_instances < 1) return fail(MIST_E_INVALID, "need at least one instance, got %d", n_instances);
  std::vector<int32_t> family(n_instances);
  int64_t stats[6] = {0, 0, 0, 0, 0, 0};
  const int rc = mist_inter_stage_search_families(
      1, shape, costs, costs, nullptr, n_instances, n_grad_accum, rows, grad_accum, only_best_path,
      out_cost, out_g, out_tmax, family.data(), out_stages, out_path, nullptr, stats, stream);
  if (out_stats) std::memcpy(out_stats, stats, sizeof(int64_t) * 4);
  return rc;
}

}  // extern "C"
