// Host orchestration of the inter-stage search for the per-mesh DP (reference:
// inter_stage_tune / inter_stage_tune_with_fixed_grad_accumu, mist/analyzer/inter_tuning.py:
// 95-217): bottleneck DP, threshold windows, speculative scan batches with the sequential replay
// of the reference's rules, back-pointers of the winner.  Same steps as the Python driver
// (mist_amd/inter_tuning.py), which stays the implementation for the uniform-device recurrence;
// here they run without an interpreter between the batches: a search makes 5-6 dependent
// round trips to the GPU, and the glue between them was half of its time.
//
// Everything that decides a result is shared with the Python driver through the C ABI:
// mist_dp_run, mist_dp_select_candidates, mist_dp_window_begin, mist_dp_filter_tmax,
// mist_dp_backtrack.  How far a window is fetched or how many thresholds a batch speculates on
// only changes the work done, never the outcome: the replay consumes DP results in the
// reference's order with its stop rule and its strict "<".
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
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

constexpr int kFirstChunk = 48;   // thresholds per G in the first speculative batch
constexpr int kMaxChunk = 4096;   // most thresholds per G in one batch
constexpr double kGap = 1e-6;     // inter_tuning.py:177
constexpr int kSelectHead = 1 << 16;  // selected candidates that travel with the counts of a fetch
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
  Buffer d_in, d_out, d_scratch, d_req, d_counts, d_values, d_request, d_argmin, d_path;
  Buffer h_in, h_out, h_req, h_counts, h_values, h_request, h_path;
  int select_capacity = 1 << 18;
  Workspace() {
    h_in.pinned = h_out.pinned = h_req.pinned = h_counts.pinned = h_values.pinned =
        h_request.pinned = h_path.pinned = true;
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

struct Search {
  const MistDpShape *shape;
  const MistDpCosts *costs;
  hipStream_t stream;
  Workspace *ws;
  int64_t launches = 0, fetches = 0, selected = 0, thresholds_run = 0;

  // DP instances (g_index[i], tmax[i]) -> outputs in ws->h_out as [3][n] (best_s bits, best_sum,
  // stage_max); with `n_path` > 0 also the partitions of the first n (== n_path) instances.
  int run(const std::vector<int32_t> &g_index, const std::vector<float> &tmax, int mode,
          bool want_path) {
    const int n = (int)tmax.size();
    if (n == 0) return 0;
    if (int rc = ws->h_in.reserve(sizeof(float) * 2 * n)) return rc;
    if (int rc = ws->d_in.reserve(sizeof(float) * 2 * n)) return rc;
    if (int rc = ws->d_out.reserve(sizeof(float) * 3 * n)) return rc;
    if (int rc = ws->h_out.reserve(sizeof(float) * 3 * n)) return rc;
    const int64_t n_scratch = mist_dp_scratch_floats(shape, n);
    if (n_scratch < 0) return MIST_E_INVALID;
    if (int rc = ws->d_scratch.reserve(sizeof(float) * (size_t)std::max<int64_t>(n_scratch, 1)))
      return rc;
    float *h_in = ws->h_in.as<float>();
    std::memcpy(h_in, tmax.data(), sizeof(float) * n);
    std::memcpy(h_in + n, g_index.data(), sizeof(int32_t) * n);
    MIST_HIP_CHECK(hipMemcpyAsync(ws->d_in.ptr, h_in, sizeof(float) * 2 * n, hipMemcpyHostToDevice,
                                  stream));
    float *d_in = ws->d_in.as<float>(), *d_out = ws->d_out.as<float>();
    int32_t *d_argmin = nullptr;
    if (want_path) {
      const size_t slab = (size_t)(shape->max_stages + 1) * (shape->num_layers + 1) *
                          (shape->num_devices + 1) * 4;
      if (int rc = ws->d_argmin.reserve(sizeof(int32_t) * slab * n)) return rc;
      if (int rc = ws->d_path.reserve(sizeof(int32_t) * (size_t)n * shape->max_stages * 4)) return rc;
      if (int rc = ws->h_path.reserve(sizeof(int32_t) * (size_t)n * shape->max_stages * 4)) return rc;
      d_argmin = ws->d_argmin.as<int32_t>();  // no fill: the walk reads what the DP wrote
    }
    if (int rc = mist_dp_run(shape, costs, d_in, reinterpret_cast<int32_t *>(d_in + n), n, mode,
                             reinterpret_cast<int32_t *>(d_out), d_out + n, d_out + 2 * n, d_argmin,
                             ws->d_scratch.as<float>(), stream))
      return rc;
    if (want_path) {
      if (int rc = mist_dp_backtrack(shape, d_argmin, reinterpret_cast<int32_t *>(d_out), n,
                                     ws->d_path.as<int32_t>(), stream))
        return rc;
      MIST_HIP_CHECK(hipMemcpyAsync(ws->h_path.ptr, ws->d_path.ptr,
                                    sizeof(int32_t) * (size_t)n * shape->max_stages * 4,
                                    hipMemcpyDeviceToHost, stream));
    }
    MIST_HIP_CHECK(hipMemcpyAsync(ws->h_out.ptr, d_out, sizeof(float) * 3 * n,
                                  hipMemcpyDeviceToHost, stream));
    MIST_HIP_CHECK(hipStreamSynchronize(stream));
    ++launches;
    thresholds_run += n;
    return 0;
  }

  // best + (g - 1) * f_stage_max in float64 (inter_tuning.py:342), inf if infeasible
  double total(int i, int n, int G) const {
    const float *h = ws->h_out.as<float>();
    int32_t best_s;
    std::memcpy(&best_s, h + i, sizeof(best_s));
    if (best_s < 0) return kInf;
    return (double)h[n + i] + ((double)G - 1.0) * (double)h[2 * n + i];
  }

  // ascending candidates v of table row rows[r] with lo[r] < v <= hi[r], and how many lie above
  int fetch(const std::vector<int32_t> &rows, const std::vector<float> &lo,
            const std::vector<float> &hi, std::vector<Fetched> *out) {
    const int n = (int)rows.size();
    out->assign(n, Fetched());
    if (n == 0) return 0;
    ++fetches;
    if (int rc = ws->h_req.reserve(sizeof(float) * 3 * n)) return rc;
    if (int rc = ws->d_req.reserve(sizeof(float) * 3 * n)) return rc;
    if (int rc = ws->d_counts.reserve(sizeof(int32_t) * (1 + n))) return rc;
    if (int rc = ws->h_counts.reserve(sizeof(int32_t) * (1 + n))) return rc;
    float *h_req = ws->h_req.as<float>();
    std::memcpy(h_req, rows.data(), sizeof(int32_t) * n);
    std::memcpy(h_req + n, lo.data(), sizeof(float) * n);
    std::memcpy(h_req + 2 * n, hi.data(), sizeof(float) * n);
    MIST_HIP_CHECK(hipMemcpyAsync(ws->d_req.ptr, h_req, sizeof(float) * 3 * n,
                                  hipMemcpyHostToDevice, stream));
    float *d_req = ws->d_req.as<float>();
    int total = 0, head = 0;
    for (;;) {
      const int capacity = ws->select_capacity;
      if (int rc = ws->d_values.reserve(sizeof(float) * capacity)) return rc;
      if (int rc = ws->d_request.reserve(sizeof(int32_t) * capacity)) return rc;
      MIST_HIP_CHECK(hipMemsetAsync(ws->d_counts.ptr, 0, sizeof(int32_t) * (1 + n), stream));
      if (int rc = mist_dp_select_candidates(
              costs, n, reinterpret_cast<int32_t *>(d_req), d_req + n, d_req + 2 * n,
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
struct Scan {
  int G = 1;
  Window *w = nullptr;
  size_t pos = 0, have_lo = 0;
  std::vector<double> cost;  // DP outcome per computed threshold, inf = infeasible
  int limit = kFirstChunk;
  size_t n_kept() const { return w ? w->kept.size() : 0; }
};

}  // namespace

extern "C" {

int mist_inter_stage_search(const MistDpShape *shape, const MistDpCosts *costs, int n_instances,
                            int n_grad_accum, const int32_t *rows, const int32_t *grad_accum,
                            int only_best_path, double *out_cost, int32_t *out_g, float *out_tmax,
                            int32_t *out_stages, int32_t *out_path, int64_t *out_stats,
                            void *stream_) {
  if (!shape || !costs || !rows || !grad_accum || !out_cost || !out_g || !out_tmax || !out_stages ||
      !out_path)
    return fail(MIST_E_INVALID, "null pointer argument");
  if (n_instances < 1 || n_grad_accum < 1)
    return fail(MIST_E_INVALID, "need at least one instance and one G, got %d x %d", n_instances,
                n_grad_accum);
  if (shape->free_devices != 0)
    return fail(MIST_E_INVALID, "the search covers the per-mesh recurrence only");
  const int64_t n_scr = mist_dp_scratch_floats(shape, 1);
  if (n_scr < 0) return MIST_E_INVALID;  // bad shape: message set by the check
  for (int i = 0; i < n_grad_accum; ++i)
    if (grad_accum[i] < 1) return fail(MIST_E_INVALID, "grad_accum[%d] = %d < 1", i, grad_accum[i]);

  std::lock_guard<std::mutex> guard(g_lock);
  int device = 0;
  MIST_HIP_CHECK(hipGetDevice(&device));
  Search S{shape, costs, (hipStream_t)stream_, &g_workspaces[device]};
  const int n_flat = n_instances * n_grad_accum;
  const int S_max = shape->max_stages;

  // ---- smallest feasible threshold of every (instance, G) in one batch ----
  std::vector<int32_t> flat_rows(rows, rows + n_flat);
  std::vector<float> zeros(n_flat, 0.0f);
  if (int rc = S.run(flat_rows, zeros, MIST_DP_BOTTLENECK, false)) return rc;
  std::vector<Window> windows(n_flat);
  std::vector<int> feasible;
  std::vector<float> hi_first;
  {
    const float *h = S.ws->h_out.as<float>();
    for (int i = 0; i < n_flat; ++i) {
      const float bott = h[n_flat + i];
      if (!std::isfinite(bott)) continue;
      Window &w = windows[i];
      w.exists = true;
      w.row = flat_rows[i];
      w.G = grad_accum[i % n_grad_accum];
      w.start_value = bott;
      w.start_sum = (double)h[2 * n_flat + i];
      // the min-max partition is admissible at the bottleneck: its total bounds the scan's
      // best; the first KEPT candidate may lie a few gaps above, and when the bottleneck is a
      // single-stage cost (no candidate itself) a little further up
      const double cost0 = w.start_sum + (double)(w.G - 1) * (double)bott;
      const double room = (double)(w.G - 1) * (4 * kGap);
      float hi = std::nextafter((float)((cost0 + room) * (1.0 + 1e-5) / (double)w.G),
                                std::numeric_limits<float>::infinity());
      hi = std::max(hi, (float)((double)bott * (1.0 + 2e-3) + 2e-4));
      feasible.push_back(i);
      hi_first.push_back(hi);
    }
  }
  {
    std::vector<int> pending(feasible.size());
    for (size_t k = 0; k < pending.size(); ++k) pending[k] = (int)k;
    for (int widen = 0; !pending.empty(); ++widen) {
      std::vector<int32_t> r;
      std::vector<float> lo, hi;
      for (int k : pending) {
        const Window &w = windows[feasible[k]];
        r.push_back(w.row);
        lo.push_back(widen >= 8 ? -std::numeric_limits<float>::infinity() : w.lower_margin(widen));
        hi.push_back(hi_first[k]);
      }
      std::vector<Fetched> got;
      if (int rc = S.fetch(r, lo, hi, &got)) return rc;
      std::vector<int> again;
      std::vector<float> kept;
      for (size_t j = 0; j < pending.size(); ++j) {
        Window &w = windows[feasible[pending[j]]];
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
    for (int i : feasible)
      if (!windows[i].covers(kInf)) brief.push_back(&windows[i]);
    if (!brief.empty()) {
      std::vector<int32_t> r;
      std::vector<float> lo, want;
      for (Window *w : brief) {
        r.push_back(w->row);
        lo.push_back(w->hi);
        want.push_back(w->extension_target(kInf));
      }
      std::vector<Fetched> got;
      if (int rc = S.fetch(r, lo, want, &got)) return rc;
      for (size_t j = 0; j < brief.size(); ++j)
        if (int rc = S.apply_extension(brief[j], got[j], want[j])) return rc;
    }
  }

  // ---- speculative batches + sequential replay ----
  struct Chain {
    std::vector<Scan> scans;
    size_t current = 0;
    double best_cost = kInf;
    int best_g = -1;
    float best_t = 0.0f;
  };
  std::vector<Chain> chains(n_instances);
  for (int t = 0; t < n_instances; ++t) {
    chains[t].scans.resize(n_grad_accum);
    for (int i = 0; i < n_grad_accum; ++i) {
      Scan &sc = chains[t].scans[i];
      Window &w = windows[t * n_grad_accum + i];
      sc.G = grad_accum[i];
      sc.w = w.exists ? &w : nullptr;
      if (sc.w)
        sc.pos = (size_t)(std::lower_bound(w.kept.begin(), w.kept.end(), w.start_value) -
                          w.kept.begin());
      sc.have_lo = sc.pos;  // everything below is infeasible: the scan passes it unchanged
    }
  }
  int rc_inner = 0;
  // makes sure threshold `pos` is materialised if the scan can get there
  auto reach = [&](Scan &sc, size_t pos, double best_cost) -> bool {
    Window *w = sc.w;
    while (w && pos >= w->kept.size() && !w->covers(best_cost)) {
      if (int rc = S.extend(w, best_cost)) {
        rc_inner = rc;
        return false;
      }
    }
    return pos < sc.n_kept();
  };
  // advances the sequential scan as far as the computed results allow; true = this G is done
  auto replay = [&](Scan &sc, double &best_cost, bool &improved, float &best_t) -> bool {
    for (;;) {
      if (!reach(sc, sc.pos, best_cost)) return true;
      if (sc.w->scaled[sc.pos] >= best_cost) return true;  // inter_tuning.py:196-197
      if (sc.pos >= sc.have_lo + sc.cost.size()) return false;  // needs more DP results
      const double c = sc.cost[sc.pos - sc.have_lo];
      if (c < best_cost) {
        best_cost = c;
        best_t = sc.w->kept[sc.pos];
        improved = true;
      }
      ++sc.pos;
    }
  };
  // dry run of replay under the bound `best_cost`: true if the computed results do not suffice
  auto runs_out = [&](Scan &sc, double best_cost) -> bool {
    size_t pos = sc.pos;
    const size_t hi = sc.have_lo + sc.cost.size();
    while (reach(sc, pos, best_cost)) {
      if (sc.w->scaled[pos] >= best_cost) return false;
      if (pos >= hi) return true;
      best_cost = std::min(best_cost, sc.cost[pos - sc.have_lo]);
      ++pos;
    }
    return false;
  };
  struct Span {
    int t, i, n;
  };
  for (;;) {
    std::vector<int32_t> req_g;
    std::vector<float> req_t;
    std::vector<int> req_G;
    std::vector<Span> spans;
    bool all_done = true;
    for (int t = 0; t < n_instances; ++t) {
      Chain &ch = chains[t];
      while (ch.current < ch.scans.size()) {  // commit the sequential scan as far as possible
        Scan &sc = ch.scans[ch.current];
        bool improved = false;
        float best_t = ch.best_t;
        const bool finished = replay(sc, ch.best_cost, improved, best_t);
        if (rc_inner) return rc_inner;
        if (improved) {
          ch.best_g = (int)ch.current;
          ch.best_t = best_t;
        }
        if (!finished) break;
        ++ch.current;
      }
      if (ch.current < ch.scans.size()) all_done = false;
      for (size_t i = ch.current; i < ch.scans.size(); ++i) {
        Scan &sc = ch.scans[i];
        if (i > ch.current && !runs_out(sc, ch.best_cost)) {
          if (rc_inner) return rc_inner;
          continue;
        }
        if (rc_inner) return rc_inner;
        // the range grows fourfold every time the same G asks again
        const size_t a = sc.have_lo + sc.cost.size();
        reach(sc, a + sc.limit, ch.best_cost);
        if (rc_inner) return rc_inner;
        size_t stop = 0;
        if (sc.w)
          stop = (size_t)(std::lower_bound(sc.w->scaled.begin(), sc.w->scaled.end(), ch.best_cost) -
                          sc.w->scaled.begin());
        const size_t b = std::max(a, std::min(stop, a + sc.limit));
        if (b > a) {
          sc.limit = std::min(kMaxChunk, sc.limit * 4);
          for (size_t k = a; k < b; ++k) {
            req_g.push_back(rows[t * n_grad_accum + (int)i]);
            req_t.push_back(sc.w->kept[k]);
            req_G.push_back(sc.G);
          }
          spans.push_back(Span{t, (int)i, (int)(b - a)});
        }
      }
    }
    if (all_done) break;
    if (spans.empty()) return fail(MIST_E_INVALID, "inter-stage scan made no progress");
    if (int rc = S.run(req_g, req_t, MIST_DP_THRESHOLD, false)) return rc;
    const int n = (int)req_t.size();
    int off = 0;
    for (const Span &sp : spans) {
      Scan &sc = chains[sp.t].scans[sp.i];
      for (int k = 0; k < sp.n; ++k) sc.cost.push_back(S.total(off + k, n, req_G[off + k]));
      off += sp.n;
    }
  }

  // ---- results and the partitions of the winners ----
  std::vector<int> winners;
  for (int t = 0; t < n_instances; ++t) {
    const Chain &ch = chains[t];
    out_cost[t] = ch.best_cost;
    out_g[t] = ch.best_g;
    out_tmax[t] = ch.best_g >= 0 ? ch.best_t : 0.0f;
    out_stages[t] = 0;
    for (int k = 0; k < S_max * 4; ++k) out_path[(size_t)t * S_max * 4 + k] = -1;
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
    for (int t : winners) {
      g.push_back(rows[t * n_grad_accum + chains[t].best_g]);
      tm.push_back(chains[t].best_t);
    }
    if (int rc = S.run(g, tm, MIST_DP_THRESHOLD, true)) return rc;
    const int n = (int)winners.size();
    const float *h = S.ws->h_out.as<float>();
    const int32_t *path = S.ws->h_path.as<int32_t>();
    for (int k = 0; k < n; ++k) {
      const int t = winners[k];
      int32_t best_s;
      std::memcpy(&best_s, h + k, sizeof(best_s));
      const double again = S.total(k, n, grad_accum[chains[t].best_g]);
      if (best_s < 0 || again != chains[t].best_cost)
        return fail(MIST_E_INVALID, "back-pointer run of instance %d gives %.17g, the scan %.17g", t,
                    again, chains[t].best_cost);
      out_stages[t] = best_s;
      std::memcpy(out_path + (size_t)t * S_max * 4, path + (size_t)k * S_max * 4,
                  sizeof(int32_t) * S_max * 4);
    }
  }
  if (out_stats) {
    out_stats[0] = S.launches;
    out_stats[1] = S.fetches;
    out_stats[2] = S.selected;
    out_stats[3] = S.thresholds_run;
  }
  return 0;
}

}  // extern "C"
