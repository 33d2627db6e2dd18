// Inter-stage pipeline-partition DP on MI355X (gfx950).
//
// The stage index s is the sequential axis.  The (threshold, start layer k, devices d) states
// of one s are independent; each is scanned by one thread (or a team of lanes) that walks its
// (mesh, end layer, ckpt) candidates in the reference's order with float32 adds and strict "<",
// so ties resolve exactly as in the reference loop nest (mist/analyzer/inter_tuning.py:298-333).
// Two schedules: one launch per s with the states of all instances spread over the GPU
// (dp_step_kernel), or one workgroup per instance that keeps its state planes in LDS and loops
// over s itself (dp_fused_kernel).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <cstdlib>
#include <map>
#include <mutex>
#include <utility>

#include "mist_common.h"
#include "mist_dp.h"

namespace {

using mist::fail;

constexpr int kDpThreads = 64;  // one wavefront per workgroup
constexpr int kDpWideTeam = 8;  // lanes that share one DP state in small batches
constexpr size_t kDpLdsPerCu = 160 * 1024;  // LDS of a gfx950 compute unit
constexpr int kDpFusedThreads = 1024;  // largest workgroup of the one-launch kernel
constexpr int kDpFusedMinInstances = 64;  // threshold batches of at least this size use it
constexpr int kDpFusedSmallPlane = 2048;  // (L + 1)(D + 1) up to which every batch uses it
constexpr int kDpStageBatch = 8;   // row minima a lane copies together in the one-launch kernel
constexpr int kSelectBatch = 8;  // table values a lane of the candidate selection reads together
constexpr int kSelectBuffer = 4096;  // selected values a workgroup holds before it appends them
constexpr float kDpNoThreshold = 3.402823466e+38f;  // FLT_MAX: admits every finite stage cost
constexpr int kDpBatch = 4;  // end layers whose reads a lane of the one-lane-per-state kernel overlaps

// ------------------------------------------------------------------------------------------
// Adapter: float64 (stable, delta) tables -> float32 DP cost tables for every g.
// ------------------------------------------------------------------------------------------
// Table rows (fixed g, mesh, p, layers) hold the L+1 ckpt entries: cost = (float)stable +
// (float)delta / G, and alongside its running minimum pmin[j] = min(cost[0..j]).  A workgroup
// takes as many whole rows as fit its 256 lanes, one lane per entry, so that loads and stores
// are contiguous; the running minimum is a segmented scan (wavefront shuffles, LDS between the
// wavefronts a row spans).  Rows longer than the workgroup are walked in passes of 256 entries
// with the minimum of the earlier passes carried along.
// Most cells of a plan hold no strategy (no group for that (g, mesh), or nothing fits): their
// row index is -1 and their costs +inf, so with the index table (may be null) the 16 bytes of
// such a cell's costs are not read.
// The four tables of a call (base, with_pre, with_post, no_pp) go through one launch: table v
// owns the workgroups first_block[v] .. first_block[v + 1] - 1.
struct CostTableJob {
  const double *stable[4], *delta[4];
  const int32_t *index[4];
  float *out[4], *pmin[4];
  int64_t n_rows[4], rows_per_g[4];
  unsigned first_block[5];
};
__global__ __launch_bounds__(256) void cost_table_kernel(const CostTableJob job,
                                                         const int32_t *__restrict__ grad_accum,
                                                         int row_len, int sample_size, int slot) {
  __shared__ float lds[256];
  const int v = (blockIdx.x >= job.first_block[1]) + (blockIdx.x >= job.first_block[2]) +
                (blockIdx.x >= job.first_block[3]);
  const double *__restrict__ stable = job.stable[v], *__restrict__ delta = job.delta[v];
  const int32_t *__restrict__ index = job.index[v];
  float *__restrict__ out = job.out[v], *__restrict__ pmin = job.pmin[v];
  const int64_t n_rows = job.n_rows[v], rows_per_g = job.rows_per_g[v];
  const int seg = min(row_len, 256);  // entries of a row per pass
  const int rows_here = 256 / seg;
  const int local_row = threadIdx.x / seg, j0 = threadIdx.x % seg;
  const int64_t r = (int64_t)(blockIdx.x - job.first_block[v]) * rows_here + local_row;
  const bool live_row = local_row < rows_here && r < n_rows;
  const float G = live_row ? (float)grad_accum[r / rows_per_g] : 1.0f;
  float carry = INFINITY;
  for (int base = 0; base < row_len; base += seg) {
    const int j = base + j0;
    const bool live = live_row && j < row_len;
    const int64_t i = r * row_len + j;
    float c = INFINITY;
    if (live) {
      if (index == nullptr || index[i * sample_size + slot] >= 0) {
        const float s = (float)stable[i * sample_size + slot];
        const float d = (float)delta[i * sample_size + slot];
        c = s + d / G;
      }
      out[i] = c;
    }
    // running minimum over the row's lanes of this pass: inside a wavefront by shuffles that stop
    // at the row's first lane, then the part of the row that lies in earlier wavefronts (their
    // last lanes hold it)
    float run = c;
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int step = 1; step < 64; step <<= 1) {
      const float other = __shfl_up(run, step);
      if (lane >= step && j0 >= step) run = fminf(run, other);
    }
    lds[threadIdx.x] = run;
    __syncthreads();
    const int row_first = (int)threadIdx.x - j0;
    for (int at = (int)(threadIdx.x & ~63u) - 1; at >= row_first; at -= 64) run = fminf(run, lds[at]);
    if (live) pmin[i] = fminf(run, carry);
    if (base + seg < row_len)  // only rows longer than one pass: then the row is the workgroup
      carry = fminf(carry, fminf(fminf(lds[63], lds[127]), fminf(lds[191], lds[255])));
    __syncthreads();
  }
}

// ------------------------------------------------------------------------------------------
// t_max candidates of a value window: one pass over the three cost tables of a table row g
// (costs, with_pre, with_post; inter_tuning.py:180-186).  Request r selects the finite values v
// of row rows[r] with lo[r] < v <= hi[r]; they are appended, unordered, to one output list as
// (value, request) pairs; counts[0] = pairs wanted in total (may exceed the capacity, then the
// caller retries with a larger list), counts[1 + r] = finite values of request r above hi[r].
// ------------------------------------------------------------------------------------------
// With `per_request` every request appends to a list of its own instead, out_values[r][capacity],
// counted in counts[1 + n_requests + r] (then counts[0] and out_request are not touched).
__global__ __launch_bounds__(256) void select_candidates_kernel(
    const MistDpCosts tabs, const int32_t *__restrict__ rows, const float *__restrict__ lo,
    const float *__restrict__ hi, float *__restrict__ out_values, int32_t *__restrict__ out_request,
    int capacity, int32_t *__restrict__ counts, bool per_request) {
  // Selected values collect in LDS and leave in one piece: appends to the one output list go
  // through a single counter, and an atomic per wavefront round (thousands per launch) made
  // that counter the bottleneck of the kernel.
  __shared__ float kept[kSelectBuffer];
  __shared__ int n_kept, flush_at;
  __shared__ int above_of_wave[4];
  const int r = blockIdx.y;
  const int64_t g = rows[r];
  const int64_t n0 = tabs.g_stride[0], n1 = tabs.g_stride[1], n2 = tabs.g_stride[2];
  const int64_t n = n0 + n1 + n2;
  const float lo_r = lo[r], hi_r = hi[r];
  const int lane = threadIdx.x & 63;
  int above = 0;
  if (threadIdx.x == 0) n_kept = 0;
  __syncthreads();
  int32_t *list_count = per_request ? &counts[1 + gridDim.y + r] : &counts[0];
  float *list = per_request ? out_values + (int64_t)r * capacity : out_values;
  auto flush = [&]() {  // called by the whole workgroup
    if (threadIdx.x == 0) flush_at = n_kept > 0 ? atomicAdd(list_count, n_kept) : 0;
    __syncthreads();
    for (int i = threadIdx.x; i < n_kept; i += blockDim.x) {
      const int at = flush_at + i;
      if (at < capacity) {
        list[at] = kept[i];
        if (!per_request) out_request[at] = r;
      }
    }
    __syncthreads();
    if (threadIdx.x == 0) n_kept = 0;
    __syncthreads();
  };
  // every workgroup of a request runs the same number of rounds; kSelectBatch values per lane
  // are read together
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t base = (int64_t)blockIdx.x * blockDim.x; base < n; base += kSelectBatch * stride) {
    float value[kSelectBatch];
#pragma unroll
    for (int u = 0; u < kSelectBatch; ++u) {
      const int64_t e = base + u * stride + threadIdx.x;
      value[u] = INFINITY;
      if (e < n)
        value[u] = e < n0 ? tabs.costs[g * n0 + e]
                   : e < n0 + n1 ? tabs.costs_pre[g * n1 + (e - n0)]
                                 : tabs.costs_post[g * n2 + (e - n0 - n1)];
    }
#pragma unroll
    for (int u = 0; u < kSelectBatch; ++u) {
      const float v = value[u];
      const bool finite = v < INFINITY;  // +inf (nothing feasible) and NaN are not candidates
      above += finite && v > hi_r;
      const bool take = finite && v > lo_r && v <= hi_r;
      // one LDS atomic per wavefront reserves the slots of all its selected values
      const unsigned long long takers = __ballot(take);
      if (takers != 0) {
        const int leader = __ffsll(takers) - 1;
        int first = 0;
        if (lane == leader) first = atomicAdd(&n_kept, __popcll(takers));
        first = __shfl(first, leader);
        if (take) kept[first + __popcll(takers & ((1ull << lane) - 1))] = v;
      }
    }
    __syncthreads();
    // Room for another round of kSelectBatch values per thread?  Every wave reads the count
    // before any wave adds to it again (second barrier), so the whole workgroup takes the
    // same branch and flush()'s barriers are reached by all of its waves.
    const int kept_now = n_kept;
    __syncthreads();
    if (kept_now > kSelectBuffer - kSelectBatch * 256) flush();
  }
  flush();
  // one atomic per workgroup for the "above" count
  for (int step = 32; step >= 1; step >>= 1) above += __shfl_xor(above, step);
  if (lane == 0) above_of_wave[threadIdx.x >> 6] = above;
  __syncthreads();
  if (threadIdx.x == 0) {
    const int total = above_of_wave[0] + above_of_wave[1] + above_of_wave[2] + above_of_wave[3];
    if (total > 0) atomicAdd(&counts[1 + r], total);
  }
}

// ------------------------------------------------------------------------------------------
// The reference's gap rule (inter_tuning.py:198) and the start of a walk that does not begin at
// the bottom of the candidate list (see mist_dp_window_begin in mist_dp.h): the same code for
// the host entry points and for the kernel that walks the windows on the device.
// ------------------------------------------------------------------------------------------
// "t - last < 1e-6" as the reference evaluates it: float32 difference, float64 comparison
__host__ __device__ inline bool gap_below(float t, float last, double gap) {
  const float diff = t - last;
  return (double)diff < gap;
}
// Index the walk over `ascending` starts at, or -1 when the fetched part holds no certain start.
__host__ __device__ inline int window_walk_start(const float *ascending, int n, float lo,
                                                 bool open_below, float start_value, double gap) {
  // A candidate whose predecessor is at least the gap below it is kept whatever the walk did
  // before; the predecessor of the first fetched candidate is unknown unless the fetch was open
  // below.
  int first = -1;
  for (int i = 0; i < n && ascending[i] <= start_value; ++i) {
    const float prev = i == 0 ? (open_below ? 0.0f : lo) : ascending[i - 1];
    const bool certain = !gap_below(ascending[i], prev, gap) || (i == 0 && open_below);
    if (certain) first = i;
  }
  if (first < 0) {
    const bool certain0 = !gap_below(ascending[0], open_below ? 0.0f : lo, gap) || open_below;
    if (ascending[0] > start_value && certain0) first = 0;
  }
  return first;
}

// Which kept threshold (counted from the first one at or above the smallest feasible threshold)
// instance k of a window's first scan batch runs, when n_avail of them are there: all of them if
// they fit the batch; else the first `first_lead` ones, then the rest of the batch spread evenly
// up to the window's last one (probes: the stage-cost sum at a later threshold bounds the sums at
// every earlier one from below, which lets the scan pass thresholds that cannot improve its best).
__host__ __device__ __forceinline__ int dp_first_batch_index(int k, int n_avail, int first_chunk,
                                                             int first_lead) {
  if (n_avail <= first_chunk || k < first_lead || first_lead >= first_chunk) return k;
  const int spread = first_chunk - first_lead;
  return first_lead + (int)(((int64_t)(k - first_lead + 1) * (n_avail - first_lead)) / spread) - 1;
}

constexpr int kWindowThreads = 1024;
// status of a window walked on the device (meta[r][2])
constexpr int kWindowOk = 0, kWindowNone = 1, kWindowOverflow = 2, kWindowNoStart = 3,
              kWindowNoBound = 4, kWindowKeptOverflow = 5;

// One workgroup per request of a per-request candidate selection: sorts the request's values
// (bitonic, in LDS), walks them with the gap rule from the certain start below `start[r]` (the
// smallest feasible threshold; +inf = nothing feasible, the request is skipped), appends the kept
// thresholds to one list (kept_out, cursor in counts[0]) and lays out the first scan batch: up to
// `first_chunk` kept thresholds at or above start[r] (dp_first_batch_index) as DP instances,
// appended to inst_tmax / inst_row (cursor in counts[1 + 2 n_requests]; the caller pre-fills inst_row with
// -1, so that the live instances are the first workgroups of the DP launch and the empty slots
// its tail).
// meta[r][8] = (selected, above hi, status, kept, offset in kept_out, kept below start, instances,
// offset of the instances).
//
// The walk is the host's (mist_dp_window_begin), taken apart along its own argument: a candidate
// whose predecessor is at least the gap below it is kept whatever came before (the last kept
// value is at most the predecessor, and the float32 difference is monotone), so the candidates
// from such a one up to the next are a piece that is walked on its own, by the thread that owns
// its first element; the piece that starts at the walk's first element begins with "nothing kept
// yet" like the host's loop.
__global__ __launch_bounds__(kWindowThreads) void window_walk_kernel(
    const float *__restrict__ values, int capacity, int32_t *__restrict__ counts,
    const int32_t *__restrict__ rows, const float *__restrict__ lo,
    const float *__restrict__ start, double gap, int first_chunk, int first_lead,
    float *__restrict__ kept_out, int kept_capacity, int32_t *__restrict__ meta,
    float *__restrict__ inst_tmax, int32_t *__restrict__ inst_row) {
  extern __shared__ float win_lds[];
  float *v = win_lds;                                               // [capacity]
  uint8_t *keep = reinterpret_cast<uint8_t *>(win_lds + capacity);  // [capacity]
  __shared__ int32_t wave_kept[kWindowThreads / 64], wave_below[kWindowThreads / 64];
  __shared__ int32_t walk_first, kept_base, kept_overflow, inst_base;
  const int r = blockIdx.x, n_requests = gridDim.x, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6, n_waves = blockDim.x >> 6;
  const int n_sel = counts[1 + n_requests + r];
  const float start_r = start[r], lo_r = lo[r];
  int status = kWindowOk;
  if (!(start_r < INFINITY)) status = kWindowNone;
  else if (n_sel > capacity) status = kWindowOverflow;
  const int n = status == kWindowOk ? n_sel : 0;
  int m = 128;  // a wavefront's share of a sorting step is 128 consecutive values
  while (m < n) m <<= 1;  // capacity is a power of two >= 128
  for (int i = tid; i < m; i += blockDim.x) {
    v[i] = i < n ? values[(int64_t)r * capacity + i] : INFINITY;
    keep[i] = 0;
  }
  if (tid == 0) {
    walk_first = -1;
    kept_overflow = 0;
  }
  __syncthreads();
  // Bitonic sort, one compare-exchange per thread and step: thread x holds the pair
  // (i, i + j) with i = 2 j (x / j) + x % j.  For j <= 32 the 64 pairs of a wavefront lie in its
  // own 128 consecutive values, and so do those of the following smaller j: those steps need no
  // barrier between them (a wavefront's LDS accesses complete in order).
  for (int k = 2; k <= m; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int x = tid; x < m / 2; x += blockDim.x) {
        const int i = 2 * j * (x / j) + x % j, other = i + j;
        const float a = v[i], b = v[other];
        const bool ascending = (i & k) == 0;
        if ((a > b) == ascending) {
          v[i] = b;
          v[other] = a;
        }
      }
      if (j > 32) __syncthreads();
      else __builtin_amdgcn_wave_barrier();
    }
    if (k >= 64) __syncthreads();  // the next k starts with j = k: other wavefronts' values
  }
  __syncthreads();
  // start of the walk (window_walk_start with a fetch that is not open below): the last
  // candidate <= start_r whose predecessor is at least the gap below, else the first candidate
  // if it lies above start_r and is certain itself
  const int per = (m + blockDim.x - 1) / blockDim.x;
  const int i0 = tid * per, i1 = min(i0 + per, n);
  {
    int mine = -1;
    for (int i = i0; i < i1; ++i)
      if (v[i] <= start_r && !gap_below(v[i], i == 0 ? lo_r : v[i - 1], gap)) mine = i;
    if (mine >= 0) atomicMax(&walk_first, mine);
  }
  __syncthreads();
  int first = walk_first;
  if (status == kWindowOk && n > 0 && first < 0) {
    if (v[0] > start_r && !gap_below(v[0], lo_r, gap)) first = 0;
    else status = kWindowNoStart;
  }
  // the walk, piece by piece
  if (status == kWindowOk && n > 0) {
    for (int i = max(i0, first); i < i1; ++i) {
      const bool head = i == first;
      if (!head && gap_below(v[i], v[i - 1], gap)) continue;  // inside a piece: its owner walks it
      float last = 0.0f;  // the walk's first piece starts with nothing kept (mist_dp_filter_tmax)
      int j = i;
      if (!head) {
        keep[i] = 1;
        last = v[i];
        j = i + 1;
      }
      for (; j < n && (j == i || gap_below(v[j], v[j - 1], gap)); ++j) {
        if (gap_below(v[j], last, gap)) continue;
        keep[j] = 1;
        last = v[j];
      }
    }
  }
  __syncthreads();
  // kept values per thread (consecutive elements), those below the start among them
  int mine = 0, below = 0;
  if (status == kWindowOk)
    for (int i = i0; i < i1; ++i) {
      mine += keep[i];
      below += keep[i] && v[i] < start_r;
    }
  int scan_kept = mine, scan_below = below;  // inclusive scans over the wavefront
  for (int step = 1; step < 64; step <<= 1) {
    const int a = __shfl_up(scan_kept, step), b = __shfl_up(scan_below, step);
    if (lane >= step) {
      scan_kept += a;
      scan_below += b;
    }
  }
  if (lane == 63) {
    wave_kept[wave] = scan_kept;
    wave_below[wave] = scan_below;
  }
  __syncthreads();
  int before = 0, n_kept = 0, pos = 0;
  for (int w = 0; w < n_waves; ++w) {
    if (w < wave) before += wave_kept[w];
    n_kept += wave_kept[w];
    pos += wave_below[w];
  }
  if (status == kWindowOk && pos >= n_kept) status = kWindowNoBound;  // nothing kept at or above the start
  const int n_inst = status == kWindowOk ? min(first_chunk, n_kept - pos) : 0;
  if (tid == 0) {
    kept_base = inst_base = 0;
    if (status == kWindowOk) {
      kept_base = atomicAdd(&counts[0], n_kept);
      if (kept_base + n_kept > kept_capacity) kept_overflow = 1;
      else inst_base = atomicAdd(&counts[1 + 2 * n_requests], n_inst);  // <= n_requests * first_chunk
    }
  }
  __syncthreads();
  if (status == kWindowOk && kept_overflow) status = kWindowKeptOverflow;
  if (status == kWindowOk) {
    int at = before + scan_kept - mine;  // kept values in front of this thread's elements
    for (int i = i0; i < i1; ++i) {
      if (!keep[i]) continue;
      kept_out[kept_base + at] = v[i];
      ++at;
    }
  }
  __syncthreads();  // (the workgroup's own writes to kept_out are visible to it behind the barrier)
  if (status == kWindowOk) {
    for (int k = tid; k < n_inst; k += blockDim.x) {
      inst_tmax[inst_base + k] =
          kept_out[kept_base + pos + dp_first_batch_index(k, n_kept - pos, first_chunk, first_lead)];
      inst_row[inst_base + k] = rows[r];
    }
  }
  if (tid == 0) {
    int32_t *out = meta + 8 * r;
    out[0] = n_sel;
    out[1] = counts[1 + r];
    out[2] = status;
    out[3] = status == kWindowOk ? n_kept : 0;
    out[4] = kept_base;
    out[5] = pos;
    out[6] = status == kWindowOk ? n_inst : 0;
    out[7] = inst_base;
  }
}

// ------------------------------------------------------------------------------------------
// DP kernels.  The stage index s is the sequential axis: one launch per s.  Within a launch
// every (threshold, start layer k, devices d) state is one thread; workgroups are single
// wavefronts so that even a handful of thresholds spreads over many CUs.  F(s-1) / F(s) and
// the running stage maxima ping-pong between two planes per threshold in a global scratch slab
// (L2 resident: 4 * (L+1) * (D+1) floats per threshold).
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dp_init_kernel(const MistDpShape shape, int n_tmax,
                                                      float *__restrict__ scratch,
                                                      int32_t *__restrict__ ranges,
                                                      int32_t *__restrict__ best_s,
                                                      float *__restrict__ best_sum,
                                                      float *__restrict__ stage_max) {
  const int W = shape.num_devices + 1;
  const int plane = (shape.num_layers + 1) * W;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < (int64_t)n_tmax * W) {
    // Reachable start layers [first, last] per instance and device column, three buffers used
    // in rotation by the steps.  F(0) is reachable at (k = L, d = 0) only.
    const int64_t stride = (int64_t)n_tmax * W * 2;
    const bool origin = i % W == 0;
    ranges[2 * i] = origin ? shape.num_layers : shape.num_layers + 1;
    ranges[2 * i + 1] = origin ? shape.num_layers : -1;
    for (int b = 1; b < 3; ++b) {
      ranges[b * stride + 2 * i] = shape.num_layers + 1;
      ranges[b * stride + 2 * i + 1] = -1;
    }
  }
  if (i >= (int64_t)n_tmax * plane) return;
  const int t = (int)(i / plane), e = (int)(i % plane);
  float *state = scratch + (int64_t)t * 4 * plane;
  // plane 0 holds F(0, ., .): 0 at (k = L, d = 0), +inf elsewhere; maxima start at 0.
  state[e] = e == shape.num_layers * W ? 0.0f : INFINITY;
  state[2 * plane + e] = 0.0f;
  if (e == 0) {
    best_s[t] = -1;
    best_sum[t] = INFINITY;
    stage_max[t] = 0.0f;
  }
}

// Where the ckpt row of (variant, mesh q, pre-saved micro-batches p, layers k..i) starts and which
// table holds it.
struct DpRowRef {
  int v;
  int64_t at;
};
__device__ __forceinline__ DpRowRef dp_row_ref(const MistDpShape &shape, const int64_t (&off)[4],
                                               int p, int k, int q, int i) {
  const int L = shape.num_layers, P1 = shape.p_dim, C = L + 1;
  const int l = i - k + 1;
  DpRowRef r;
  if (k == 0 && i == L - 1) { r.v = 3; r.at = (int64_t)q * C; }
  else if (k == 0) { r.v = 1; r.at = (((int64_t)q * P1 + p) * L + (l - 1)) * C; }
  else if (i == L - 1) { r.v = 2; r.at = ((int64_t)q * L + (l - 1)) * C; }
  else { r.v = 0; r.at = (((int64_t)q * P1 + p) * L + (l - 1)) * C; }
  r.at += off[r.v];
  return r;
}
__device__ __forceinline__ const float *dp_table(const MistDpCosts &tabs, int v, bool running_min) {
  if (running_min)
    return v == 0 ? tabs.pmin : v == 1 ? tabs.pmin_pre : v == 2 ? tabs.pmin_post : tabs.pmin_nopp;
  return v == 0 ? tabs.costs : v == 1 ? tabs.costs_pre : v == 2 ? tabs.costs_post : tabs.costs_nopp;
}
// ckpt candidates j_begin..j_end of a stage k..i: 0..L-i (inter_tuning.py:315), or 0..l / only l
// (inter_tuning_uniform_device.py:400-404)
__device__ __forceinline__ int dp_j_last(const MistDpShape &shape, int k, int i) {
  return shape.ckpt_rule == MIST_DP_CKPT_TAIL ? shape.num_layers - i : i - k + 1;
}
// The reference walks j = j_begin..j_end with "cost <= t_max and cost + prev < best".  "+ prev" is
// monotone, so the smallest reachable sum is (smallest admissible cost) + prev, and the smallest
// admissible cost is the row's running minimum if that is <= t_max (else nothing is admissible).
__device__ __forceinline__ float dp_row_min(const MistDpShape &shape, const MistDpCosts &tabs,
                                            const int64_t (&off)[4], int p, int k, int q, int i) {
  const DpRowRef r = dp_row_ref(shape, off, p, k, q, i);
  return shape.ckpt_rule == MIST_DP_CKPT_ALL ? dp_table(tabs, r.v, false)[r.at + (i - k + 1)]
                                             : dp_table(tabs, r.v, true)[r.at + dp_j_last(shape, k, i)];
}

// Re-laid row minima (mist_dp_stage_minima): per (g, p, mesh) a triangle over (k, i >= k), row k
// at dp_triangle_row(L, k), entry i - k.
__device__ __host__ __forceinline__ int dp_triangle(int L) { return L * (L + 1) / 2; }
__device__ __host__ __forceinline__ int dp_triangle_row(int L, int k) {
  return k * L - k * (k - 1) / 2;
}

// Running winner of one state's scan.  The reference visits (q, i) in ascending order and
// replaces on a strict "<".  A state reachable only through an unreachable successor cannot
// improve (inf + c is never < best); skipping it changes nothing.
constexpr int kDpNoCandidate = 0x7fffffff;
struct DpBest {
  float best = INFINITY, best_m = 0.0f, best_rmin = 0.0f;
  int order = kDpNoCandidate;  // q * L + i of the candidate that set `best`: its place in the visit
  int arg_i = -1, arg_q = -1, arg_j = -1;
  // mesh and end layer of the winner, once the scan is over
  __device__ __forceinline__ void resolve(int L) {
    arg_q = order == kDpNoCandidate ? -1 : order / L;
    arg_i = order == kDpNoCandidate ? -1 : order % L;
  }
};
// One candidate, without a branch: an unreachable successor (+inf) gives a target of +inf, which
// is never below the winner's.
template <bool kBottleneck>
__device__ __forceinline__ void dp_consider(DpBest &w, float t_max, int order, float prev,
                                            float rmin) {
  const float target = kBottleneck ? fmaxf(rmin, prev) : rmin + prev;
  const bool better = rmin <= t_max && target < w.best;
  w.best = better ? target : w.best;
  w.best_rmin = better ? rmin : w.best_rmin;
  w.order = better ? order : w.order;
}

// The winner's ckpt count and stage maximum: the first j attaining the sum is the entry the
// reference's strict "<" keeps.  Only the final winner matters, so the row is walked once.
template <bool kBottleneck>
__device__ __forceinline__ void dp_finish_winner(DpBest &w, const MistDpShape &shape,
                                                 const MistDpCosts &tabs, const int64_t (&off)[4],
                                                 float t_max, int p, int k, int d,
                                                 const float *f_prev, const float *m_prev) {
  if (w.arg_i < 0) return;
  const int W = shape.num_devices + 1;
  const int nm = shape.free_devices != 0 ? 0 : shape.mesh_n[w.arg_q] * shape.mesh_m[w.arg_q];
  const int from = (w.arg_i + 1) * W + (d - nm);
  if (kBottleneck) {
    // the maxima plane carries the SUM of the stage costs along the min-max path: a partition
    // that is admissible at the returned threshold, with its float32 sum accumulated in the
    // threshold DP's order
    w.best_m = w.best_rmin + m_prev[from];
    return;
  }
  const DpRowRef r = dp_row_ref(shape, off, p, k, w.arg_q, w.arg_i);
  const float *__restrict__ row = dp_table(tabs, r.v, false) + r.at;
  const float prev = f_prev[from];
  const int j_begin = shape.ckpt_rule == MIST_DP_CKPT_ALL ? w.arg_i - k + 1 : 0;
  const int j_end = dp_j_last(shape, k, w.arg_i);
  // kDpBatch entries are read together and tested in order
  for (int j0 = j_begin; j0 <= j_end; j0 += kDpBatch) {
    float stage_cost[kDpBatch];
#pragma unroll
    for (int u = 0; u < kDpBatch; ++u) stage_cost[u] = j0 + u <= j_end ? row[j0 + u] : INFINITY;
#pragma unroll
    for (int u = 0; u < kDpBatch; ++u) {
      if (j0 + u <= j_end && stage_cost[u] <= t_max && stage_cost[u] + prev == w.best) {
        w.arg_j = j0 + u;
        w.best_m = fmaxf(m_prev[from], stage_cost[u]);
        return;
      }
    }
  }
}

// Upper bound of the smallest feasible threshold, for the bottleneck DP of one instance: the
// largest stage cost of any partition bounds the min-max optimum from above, and a stage that
// costs more than such a bound is on no min-max partition, so the bottleneck DP may treat it as
// inadmissible (same value, same first-wins path: every candidate it drops has a target above
// the optimum).  The bound is the min-max optimum over the partitions that put every stage on
// the same mesh q (n m s = D stages, or any s <= max_stages when stages do not consume devices)
// with the layers split freely: a recurrence over (stage count, start layer) alone,
//   B(s, k) = min over i >= k of max(cost(s, k, i, q), B(s - 1, i + 1)),
// one wavefront per mesh, its two rows of B in `rows` (LDS, 2 (L + 1) of its `n_rows` floats per
// wavefront).  Called by the whole workgroup; `slot` is one int of LDS.  +inf when no such
// partition is feasible (or L > 128: a lane holds two start layers; or `rows` is too small).
__device__ __forceinline__ float dp_uniform_mesh_bound(const MistDpShape &shape,
                                                       const float *__restrict__ relaid,
                                                       float *rows, int n_rows, int32_t *slot) {
  const int L = shape.num_layers, D = shape.num_devices, Q = shape.num_mesh;
  const int tri = dp_triangle(L);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n_waves = (blockDim.x + 63) >> 6;
  if (threadIdx.x == 0) *slot = __float_as_int(INFINITY);
  __syncthreads();
  if (L <= 128 && n_waves * 2 * (L + 1) <= n_rows) {
    float *prev = rows + wave * 2 * (L + 1), *cur = prev + (L + 1);
    for (int q = wave; q < Q; q += n_waves) {
      int s_last = shape.max_stages;
      if (shape.free_devices == 0) {
        const int nm = shape.mesh_n[q] * shape.mesh_m[q];
        if (nm <= 0 || D % nm != 0 || D / nm > shape.max_stages) continue;
        s_last = D / nm;
      }
      if (s_last > L) continue;
      for (int k = lane; k <= L; k += 64) prev[k] = k == L ? 0.0f : INFINITY;
      __builtin_amdgcn_wave_barrier();
      float bound = INFINITY;
      for (int s = 1; s <= s_last; ++s) {
        const float *__restrict__ block = relaid + ((int64_t)(s - 1) * Q + q) * tri;
        for (int k = lane; k <= L; k += 64) {
          float best = INFINITY;
          if (k <= L - s) {
            const float *__restrict__ row = block + dp_triangle_row(L, k) - k;  // row[i]
            // the s - 1 stages behind this one take a layer each at least
            for (int i = k; i <= L - s; ++i) best = fminf(best, fmaxf(row[i], prev[i + 1]));
          }
          cur[k] = best;
        }
        __builtin_amdgcn_wave_barrier();
        if (shape.free_devices != 0 || s == s_last) bound = fminf(bound, cur[0]);
        float *swap = prev;
        prev = cur;
        cur = swap;
        __builtin_amdgcn_wave_barrier();
      }
      // stage costs are not negative, and non-negative floats order like their bit patterns
      if (lane == 0 && bound >= 0.0f && bound < INFINITY) atomicMin(slot, __float_as_int(bound));
    }
  }
  __syncthreads();
  return __int_as_float(*slot);
}

// Scan of one state (start layer k, devices d) by one lane (member 0 of 1) or by its share of a
// team: meshes q and end layers i in the reachable range of the successor column.
// `row_min(q, i)` returns dp_row_min of the stage k..i on mesh q; `narrow(q, i_first, i_last)`
// may shrink the range of end layers to one that still holds every i with row_min <= t_max.
struct DpKeepRange {
  __device__ __forceinline__ void operator()(int, int &, int &) const {}
};
template <bool kBottleneck, int kDpTeam, typename RowMin, typename Narrow = DpKeepRange>
__device__ __forceinline__ void dp_scan_state(DpBest &w, const MistDpShape &shape, float t_max,
                                              int k, int d, int member, const float *f_prev,
                                              const int32_t *range_prev, RowMin row_min,
                                              Narrow narrow = Narrow()) {
  const int L = shape.num_layers, W = shape.num_devices + 1;
  const bool free_devices = shape.free_devices != 0;
  for (int q = 0; q < shape.num_mesh; ++q) {
    const int nm = free_devices ? 0 : shape.mesh_n[q] * shape.mesh_m[q];
    if (nm > d) continue;
    // reachable start layers i + 1 of the remaining stages on d - nm devices
    const int32_t *reach = range_prev + 2 * (d - nm);
    int i_first = max(k, reach[0] - 1), i_last = min(L - 1, reach[1] - 1);
    narrow(q, i_first, i_last);
    if constexpr (kDpTeam == 1) {
      // One lane per state: the scan is a chain of reads.  kDpBatch end layers at a time, first
      // all their successor values, then the row minima of the reachable ones, so that the reads
      // of a batch are in flight together; the comparisons keep the order.
      for (int i0 = i_first; i0 <= i_last; i0 += kDpBatch) {
        float prev[kDpBatch], rmin[kDpBatch];
#pragma unroll
        for (int u = 0; u < kDpBatch; ++u)
          prev[u] = i0 + u <= i_last ? f_prev[(i0 + u + 1) * W + (d - nm)] : INFINITY;
#pragma unroll
        for (int u = 0; u < kDpBatch; ++u)
          rmin[u] = prev[u] == INFINITY ? INFINITY : row_min(q, i0 + u);
#pragma unroll
        for (int u = 0; u < kDpBatch; ++u)
          dp_consider<kBottleneck>(w, t_max, q * L + i0 + u, prev[u], rmin[u]);
      }
    } else {
      for (int i = i_first + member; i <= i_last; i += kDpTeam) {
        const float prev = f_prev[(i + 1) * W + (d - nm)];
        if (prev == INFINITY) continue;
        dp_consider<kBottleneck>(w, t_max, q * L + i, prev, row_min(q, i));
      }
    }
  }
}

template <bool kBottleneck, int kDpTeam>
__global__ __launch_bounds__(kDpThreads) void dp_step_kernel(
    const MistDpShape shape, const MistDpCosts tabs, const float *__restrict__ tmax_list,
    const int32_t *__restrict__ g_list, int s, float *__restrict__ scratch,
    int32_t *__restrict__ ranges, int32_t *__restrict__ best_s_out,
    float *__restrict__ best_sum_out, float *__restrict__ stage_max_out,
    int32_t *__restrict__ argmin) {
  const int L = shape.num_layers, D = shape.num_devices;
  const int W = D + 1;            // row pitch of a state plane
  const int plane = (L + 1) * W;  // states per s
  // kDpTeam consecutive lanes share one state and split its end layers between them.  The scan
  // of a state is a chain of dependent L2 reads: in a small batch its latency, not the
  // arithmetic, sets the time of a launch (team of 8); a batch that fills the GPU anyway runs
  // one lane per state, which prunes better.
  const int member = threadIdx.x % kDpTeam;
  const int e_raw = (blockIdx.x * kDpThreads + threadIdx.x) / kDpTeam;
  const bool real = e_raw < plane;  // the last team of a plane may be a dummy (kept for shuffles)
  if constexpr (kDpTeam == 1) {
    if (!real) return;
  }
  const int e = real ? e_raw : plane - 1;
  const int t = blockIdx.y;
  float *state = scratch + (int64_t)t * 4 * plane;
  const int cur = s & 1, prv = cur ^ 1;
  const float *__restrict__ f_prev = state + prv * plane;
  const float *__restrict__ m_prev = state + (2 + prv) * plane;
  float *__restrict__ f_cur = state + cur * plane;
  float *__restrict__ m_cur = state + (2 + cur) * plane;
  // bottleneck mode has no threshold; the largest finite value skips the +inf entries, which
  // improve no state (inf is never < best)
  const float t_max = kBottleneck ? kDpNoThreshold : tmax_list[t];
  const int64_t g = g_list[t];
  if (g < 0) return;  // an empty slot of the batch (the whole workgroup: blockIdx.y is the instance)
  const int64_t off[4] = {g * tabs.g_stride[0], g * tabs.g_stride[1], g * tabs.g_stride[2],
                          g * tabs.g_stride[3]};
  const int k = e / W, d = e % W;
  const int p = s - 1;
  // Most states are unreachable.  Every step records, per instance and device column, the first
  // and last start layer it reached (buffer s % 3); the next step scans only that range.  The
  // buffer after that one is reset here: its last readers ran in the step before this one.
  const int64_t range_stride = (int64_t)gridDim.y * W * 2;
  const int32_t *range_prev = ranges + ((s + 2) % 3) * range_stride + (int64_t)t * W * 2;
  int32_t *range_cur = ranges + (s % 3) * range_stride + (int64_t)t * W * 2;
  int32_t *range_next = ranges + ((s + 1) % 3) * range_stride + (int64_t)t * W * 2;

  // the row minima of this stage count in (mesh, k, i) order, if the caller prepared them
  const int tri = dp_triangle(L);
  const float *__restrict__ relaid =
      tabs.stage_min == nullptr
          ? nullptr
          : tabs.stage_min + g * tabs.stage_min_g_stride + (int64_t)p * shape.num_mesh * tri +
                dp_triangle_row(L, k) - k;
  DpBest w;
  const bool live = k <= L - s && (d >= 1 || shape.free_devices != 0);
  if (live) {
    dp_scan_state<kBottleneck, kDpTeam>(
        w, shape, t_max, k, d, member, f_prev, range_prev,
        [&](int q, int i) {
          return relaid != nullptr ? relaid[q * tri + i] : dp_row_min(shape, tabs, off, p, k, q, i);
        });
    if constexpr (kDpTeam == 1) {
      w.resolve(L);
      dp_finish_winner<kBottleneck>(w, shape, tabs, off, t_max, p, k, d, f_prev, m_prev);
    }
  }
  // Team reduction: the winner is the first candidate that attains the minimum, i.e. the
  // lexicographic minimum of (target, q, i).  Each lane holds that minimum over its own
  // candidates.
  if constexpr (kDpTeam > 1) {
#pragma unroll
    for (int step = 1; step < kDpTeam; step <<= 1) {
      const float o_best = __shfl_xor(w.best, step);
      const float o_rmin = __shfl_xor(w.best_rmin, step);
      const int o_order = __shfl_xor(w.order, step);
      const bool take = o_best < w.best || (o_best == w.best && o_order < w.order);
      w.best = take ? o_best : w.best;
      w.best_rmin = take ? o_rmin : w.best_rmin;
      w.order = take ? o_order : w.order;
    }
    w.resolve(L);
    if (!real || member != 0) return;
    if (live) dp_finish_winner<kBottleneck>(w, shape, tabs, off, t_max, p, k, d, f_prev, m_prev);
  }
  f_cur[e] = w.best;
  m_cur[e] = w.best_m;
  if (w.best < INFINITY) {
    atomicMin(&range_cur[2 * d], k);
    atomicMax(&range_cur[2 * d + 1], k);
  }
  if (k == 0) {
    range_next[2 * d] = L + 1;
    range_next[2 * d + 1] = -1;
  }
  if (argmin != nullptr && w.arg_i >= 0) {
    int32_t *a = argmin + (((int64_t)t * (shape.max_stages + 1) + s) * plane + e) * 4;
    a[0] = w.arg_i;
    a[1] = shape.mesh_n[w.arg_q];
    a[2] = shape.mesh_m[w.arg_q];
    a[3] = w.arg_j;
  }
  // The state (k = 0, d = D) is the answer of this stage count; first s wins ties
  // (inter_tuning.py:335-340).  The same thread handles it in every launch.
  if (k == 0 && d == D && w.best < best_sum_out[t]) {
    best_sum_out[t] = w.best;
    best_s_out[t] = s;
    stage_max_out[t] = w.best_m;
  }
}

// ------------------------------------------------------------------------------------------
// The same recurrence with the whole instance in one workgroup: the four state planes and the
// reachable ranges live in LDS, the stage counts are a loop with a barrier between them, and one
// launch replaces init + max_stages step launches.  Used whenever the planes fit (16 bytes per
// state); the arithmetic per state is the code above.
// ------------------------------------------------------------------------------------------
template <bool kBottleneck>
__global__ __launch_bounds__(kDpFusedThreads) void dp_fused_kernel(
    const MistDpShape shape, const MistDpCosts tabs, const float *__restrict__ tmax_list,
    const int32_t *__restrict__ g_list, int32_t *__restrict__ best_s_out,
    float *__restrict__ best_sum_out, float *__restrict__ stage_max_out,
    int32_t *__restrict__ argmin) {
  extern __shared__ float dp_lds[];
  const int L = shape.num_layers, D = shape.num_devices;
  const int W = D + 1, plane = (L + 1) * W;
  float *f_plane = dp_lds;              // [2][plane]
  float *m_plane = dp_lds + 2 * plane;  // [2][plane]
  int32_t *range = reinterpret_cast<int32_t *>(dp_lds + 4 * plane);  // [3][W][2]
  // row minima of the current stage count: per mesh a triangle (k, i >= k)
  float *stage_min = dp_lds + 4 * plane + 6 * W;
  const int tri = dp_triangle(L), n_stage = shape.num_mesh * tri;
  // first and last end layer of a stage on mesh q from layer k whose row minimum is <= t_max
  int32_t *admissible = reinterpret_cast<int32_t *>(stage_min + n_stage);  // [Q][L][2]
  const int t = blockIdx.x;
  const int64_t g = g_list[t];
  if (g < 0) {  // an empty slot of the batch
    if (threadIdx.x == 0) {
      best_s_out[t] = -1;
      best_sum_out[t] = INFINITY;
      stage_max_out[t] = 0.0f;
    }
    return;
  }
  const int64_t off[4] = {g * tabs.g_stride[0], g * tabs.g_stride[1], g * tabs.g_stride[2],
                          g * tabs.g_stride[3]};
  const float *__restrict__ relaid = tabs.stage_min + g * tabs.stage_min_g_stride;
  // the bottleneck DP has no threshold of its own: an upper bound of its answer serves as one
  // (not with back-pointers: then every state gets the entry the unbounded recurrence gives it)
  const float t_max = !kBottleneck       ? tmax_list[t]
                      : argmin != nullptr
                          ? kDpNoThreshold
                          : fminf(kDpNoThreshold,
                                  dp_uniform_mesh_bound(shape, relaid, stage_min, n_stage, admissible));
  // F(0, ., .): 0 at (k = L, d = 0), +inf elsewhere; maxima start at 0; only that state is
  // reachable.
  for (int e = threadIdx.x; e < plane; e += blockDim.x) {
    f_plane[e] = e == L * W ? 0.0f : INFINITY;
    m_plane[e] = 0.0f;
  }
  for (int col = threadIdx.x; col < W; col += blockDim.x) {
    range[2 * col] = col == 0 ? L : L + 1;
    range[2 * col + 1] = col == 0 ? L : -1;
    for (int b = 1; b < 3; ++b) {
      range[(b * W + col) * 2] = L + 1;
      range[(b * W + col) * 2 + 1] = -1;
    }
  }
  // a thread's states are blockDim.x apart: (k, d) advance by fixed steps
  const int k_first = threadIdx.x / W, d_first = threadIdx.x % W;
  const int k_step = blockDim.x / W, d_step = blockDim.x % W;
  // the answer state (k = 0, d = D) belongs to the same thread in every step
  float answer_sum = INFINITY, answer_max = 0.0f;
  int answer_s = -1;
  __syncthreads();
  for (int s = 1; s <= shape.max_stages; ++s) {
    const int cur = s & 1, prv = cur ^ 1, p = s - 1;
    const float *f_prev = f_plane + prv * plane, *m_prev = m_plane + prv * plane;
    float *f_cur = f_plane + cur * plane, *m_cur = m_plane + cur * plane;
    const int32_t *range_prev = range + ((s + 2) % 3) * W * 2;
    int32_t *range_cur = range + (s % 3) * W * 2;
    int32_t *range_next = range + ((s + 1) % 3) * W * 2;
    // Every state with start layer k reads the same row minima: copy the block of this stage
    // count (contiguous in the re-laid table) once per workgroup, kDpStageBatch loads per lane
    // in flight, so that the scans below touch LDS only.  (The previous step's scans ended at
    // the barrier that closed it.)
    const float *__restrict__ block = relaid + (int64_t)p * n_stage;
    for (int x0 = threadIdx.x; x0 < n_stage; x0 += kDpStageBatch * blockDim.x) {
      float value[kDpStageBatch];
#pragma unroll
      for (int u = 0; u < kDpStageBatch; ++u) {
        const int x = x0 + u * blockDim.x;
        if (x < n_stage) value[u] = block[x];
      }
#pragma unroll
      for (int u = 0; u < kDpStageBatch; ++u) {
        const int x = x0 + u * blockDim.x;
        if (x < n_stage) stage_min[x] = value[u];
      }
    }
    __syncthreads();
    // Near the smallest feasible threshold only short stages are admissible: the end layers
    // outside [first, last] fail "cost <= t_max" for every device count, so the scans of all
    // states with this start layer skip them (what lies inside is still tested one by one).
    {
      for (int x = threadIdx.x; x < shape.num_mesh * L; x += blockDim.x) {
        const int q = x / L, k0 = x % L;
        const float *row = stage_min + q * tri + dp_triangle_row(L, k0) - k0;
        int first = L, last = -1;
        for (int i = k0; i < L; ++i) {
          if (row[i] <= t_max) {
            first = min(first, i);
            last = i;
          }
        }
        admissible[2 * x] = first;
        admissible[2 * x + 1] = last;
      }
      __syncthreads();
    }
    int k = k_first, d = d_first;
    for (int e = threadIdx.x; e < plane; e += blockDim.x) {
      DpBest w;
      if (k <= L - s && (d >= 1 || shape.free_devices != 0)) {
        const float *mine = stage_min + dp_triangle_row(L, k) - k;
        dp_scan_state<kBottleneck, 1>(w, shape, t_max, k, d, 0, f_prev, range_prev,
                                      [&](int q, int i) { return mine[q * tri + i]; },
                                      [&](int q, int &i_first, int &i_last) {
                                        const int32_t *a = admissible + 2 * (q * L + k);
                                        i_first = max(i_first, a[0]);
                                        i_last = min(i_last, a[1]);
                                      });
        w.resolve(L);
        dp_finish_winner<kBottleneck>(w, shape, tabs, off, t_max, p, k, d, f_prev, m_prev);
      }
      f_cur[e] = w.best;
      m_cur[e] = w.best_m;
      if (w.best < INFINITY) {
        atomicMin(&range_cur[2 * d], k);
        atomicMax(&range_cur[2 * d + 1], k);
      }
      if (k == 0) {
        range_next[2 * d] = L + 1;
        range_next[2 * d + 1] = -1;
      }
      if (argmin != nullptr && w.arg_i >= 0) {
        int32_t *a = argmin + (((int64_t)t * (shape.max_stages + 1) + s) * plane + e) * 4;
        a[0] = w.arg_i;
        a[1] = shape.mesh_n[w.arg_q];
        a[2] = shape.mesh_m[w.arg_q];
        a[3] = w.arg_j;
      }
      if (e == D && w.best < answer_sum) {  // first s wins ties (inter_tuning.py:335-340)
        answer_sum = w.best;
        answer_s = s;
        answer_max = w.best_m;
      }
      k += k_step;  // state e + blockDim.x
      d += d_step;
      if (d >= W) {
        d -= W;
        ++k;
      }
    }
    __syncthreads();
  }
  if ((int)threadIdx.x == D % (int)blockDim.x) {
    best_s_out[t] = answer_s;
    best_sum_out[t] = answer_sum;
    stage_max_out[t] = answer_max;
  }
}

// ------------------------------------------------------------------------------------------
// The recurrence for shapes whose four state planes do not fit the LDS of a compute unit (80
// layers x 256 devices: 333 KB).  One workgroup per instance keeps ONE plane in LDS, F(s - 1),
// the only one the scans read at random; F(s) and the maxima planes go through the instance's
// global scratch (one coalesced copy of F(s) into LDS per stage count), the row minima are read
// from the re-laid table.  A wavefront owns (start layer k, 64 consecutive device counts d): the
// loop over (mesh, end layer) is the same for all its lanes, so the row minimum is one uniform
// read, the test against t_max a scalar branch that skips the step for the whole wavefront, and
// the LDS reads of F(s - 1) are 64 consecutive floats.  Per state the candidates are still
// visited in the reference's (mesh, end layer) order with a strict "<": same winner, same ties.
// ------------------------------------------------------------------------------------------
constexpr int kDpPlaneThreads = 1024;
constexpr int kDpPlaneCols = 4;    // device counts per lane: d = 1 + lane + 64 j, so D <= 256
constexpr int kDpPlaneLoads = 20;  // row minima a lane fetches per start layer: Q * L <= 1280
#ifndef MIST_DP_PLANE_MIN_INSTANCES
#define MIST_DP_PLANE_MIN_INSTANCES 16
#endif
// smaller batches stay on the per-stage-count launches, which spread one instance over the GPU
constexpr int kDpPlaneMinInstances = MIST_DP_PLANE_MIN_INSTANCES;

template <bool kBottleneck>
__global__ __launch_bounds__(kDpPlaneThreads) void dp_plane_kernel(
    const MistDpShape shape, const MistDpCosts tabs, const float *__restrict__ tmax_list,
    const int32_t *__restrict__ g_list, float *__restrict__ scratch,
    int32_t *__restrict__ best_s_out, float *__restrict__ best_sum_out,
    float *__restrict__ stage_max_out, int32_t *__restrict__ argmin) {
  extern __shared__ float dp_lds[];
  const int L = shape.num_layers, D = shape.num_devices, Q = shape.num_mesh;
  const int W = D + 1, plane = (L + 1) * W;
  float *f_lds = dp_lds;                                        // F(s - 1)
  int32_t *range = reinterpret_cast<int32_t *>(dp_lds + plane);  // [3][W][2] reachable rows per column
  int32_t *reach_q = range + 6 * W;                              // [Q][2] the same per mesh, all columns
  float *wave_rows = reinterpret_cast<float *>(reach_q + 2 * Q);  // [n_waves][Q][L] row minima of a task
  const int t = blockIdx.x;
  const int64_t g = g_list[t];
  if (g < 0) {  // an empty slot of the batch
    if (threadIdx.x == 0) {
      best_s_out[t] = -1;
      best_sum_out[t] = INFINITY;
      stage_max_out[t] = 0.0f;
    }
    return;
  }
  const int64_t off[4] = {g * tabs.g_stride[0], g * tabs.g_stride[1], g * tabs.g_stride[2],
                          g * tabs.g_stride[3]};
  const int tri = dp_triangle(L);
  const float *__restrict__ relaid = tabs.stage_min + g * tabs.stage_min_g_stride;
  // the bottleneck DP has no threshold of its own: an upper bound of its answer serves as one
  // (reach_q is free until the first stage count)
  // (not with back-pointers: then every state gets the entry the unbounded recurrence gives it)
  const float t_max = !kBottleneck       ? tmax_list[t]
                      : argmin != nullptr
                          ? kDpNoThreshold
                          : fminf(kDpNoThreshold,
                                  dp_uniform_mesh_bound(shape, relaid, wave_rows,
                                                        (int)(blockDim.x >> 6) * Q * L, reach_q));
  float *state = scratch + (int64_t)t * 4 * plane;
  float *__restrict__ f_cur = state;  // F(s) on its way into LDS
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n_waves = blockDim.x >> 6;
  float *my_rows = wave_rows + wave * Q * L;
  int d_of[kDpPlaneCols];
  bool col_ok[kDpPlaneCols];
#pragma unroll
  for (int j = 0; j < kDpPlaneCols; ++j) {
    d_of[j] = 1 + lane + 64 * j;
    col_ok[j] = d_of[j] <= D;
  }

  for (int e = threadIdx.x; e < plane; e += blockDim.x) f_lds[e] = e == L * W ? 0.0f : INFINITY;
  for (int col = threadIdx.x; col < W; col += blockDim.x) {
    range[2 * col] = col == 0 ? L : L + 1;
    range[2 * col + 1] = col == 0 ? L : -1;
    for (int b = 1; b < 3; ++b) {
      range[(b * W + col) * 2] = L + 1;
      range[(b * W + col) * 2 + 1] = -1;
    }
  }
  if (threadIdx.x == 0) state[2 * plane + L * W] = 0.0f;  // maximum of the empty partition
  float answer_sum = INFINITY, answer_max = 0.0f;
  int answer_s = -1;
  __syncthreads();
  for (int s = 1; s <= shape.max_stages; ++s) {
    const int cur = s & 1, prv = cur ^ 1, p = s - 1;
    const float *m_prev = state + (2 + prv) * plane;
    float *__restrict__ m_cur = state + (2 + cur) * plane;
    const int32_t *range_prev = range + ((s + 2) % 3) * W * 2;
    int32_t *range_cur = range + (s % 3) * W * 2;
    int32_t *range_next = range + ((s + 1) % 3) * W * 2;
    // reachable successor rows per mesh (over all columns): bounds of the uniform loop
    if (wave < Q) {
      const int q = wave;
      const int nm = shape.mesh_n[q] * shape.mesh_m[q];
      int first = L + 1, last = -1;
      for (int c = lane; c + nm <= D; c += 64) {  // successor column c = d - nm of some d <= D
        first = min(first, range_prev[2 * c]);
        last = max(last, range_prev[2 * c + 1]);
      }
#pragma unroll
      for (int step = 32; step >= 1; step >>= 1) {
        first = min(first, __shfl_xor(first, step));
        last = max(last, __shfl_xor(last, step));
      }
      if (lane == 0) {
        reach_q[2 * q] = first;
        reach_q[2 * q + 1] = last;
      }
    }
    for (int q = n_waves + wave; q < Q; q += n_waves) {  // (more meshes than wavefronts)
      if (lane == 0) {
        reach_q[2 * q] = 0;
        reach_q[2 * q + 1] = L;
      }
    }
    if (threadIdx.x == 0) {  // column 0 holds the origin only: unreachable from here on
      range_next[0] = L + 1;
      range_next[1] = -1;
    }
    __syncthreads();
    const float *__restrict__ block = relaid + (int64_t)p * Q * tri;
    // One task = one start layer k with all its device counts.  Tasks go to the wavefronts in
    // snake order (their cost falls with k).  A task's row minima, [Q][L - k] floats, are fetched
    // one task ahead into registers and laid into this wavefront's LDS buffer, so the loops
    // below have no global read in their dependence chain.
    const int n_tasks = L - s + 1;  // start layers 0 .. L - s
    auto task_k = [&](int round) {
      const int at = round * n_waves + ((round & 1) ? n_waves - 1 - wave : wave);
      return at < n_tasks ? at : -1;
    };
    float fetched[kDpPlaneLoads];
    auto fetch = [&](int k) {
      const int width = L - k;
#pragma unroll
      for (int u = 0; u < kDpPlaneLoads; ++u) {
        const int x = lane + 64 * u;
        if (k >= 0 && x < Q * width) {
          const int q = x / width, di = x - q * width;
          fetched[u] = block[q * tri + dp_triangle_row(L, k) + di];
        }
      }
    };
    fetch(task_k(0));
    for (int round = 0; task_k(round) >= 0; ++round) {
      const int k = task_k(round);
      const int width = L - k;
#pragma unroll
      for (int u = 0; u < kDpPlaneLoads; ++u) {
        const int x = lane + 64 * u;
        if (x < Q * width) my_rows[x] = fetched[u];
      }
      fetch(task_k(round + 1));
      __builtin_amdgcn_wave_barrier();
      // Running winner per column, lean: the value and (mesh << 8 | end layer) of the candidate
      // that set it; an unreachable successor (+inf) never compares below the winner, and the
      // admissibility of the candidate is the same for every lane (tested once, below).
      float best[kDpPlaneCols];
      int best_at[kDpPlaneCols];
#pragma unroll
      for (int j = 0; j < kDpPlaneCols; ++j) {
        best[j] = INFINITY;
        best_at[j] = -1;
      }
      for (int q = 0; q < Q; ++q) {
        const int nm = shape.mesh_n[q] * shape.mesh_m[q];
        const int i_first = max(k, reach_q[2 * q] - 1);
        const int i_last = min(L - 1, reach_q[2 * q + 1] - 1);
        bool lane_ok[kDpPlaneCols];
        const float *col[kDpPlaneCols];
#pragma unroll
        for (int j = 0; j < kDpPlaneCols; ++j) {
          lane_ok[j] = col_ok[j] && nm <= d_of[j];
          col[j] = f_lds + (lane_ok[j] ? d_of[j] - nm : 0);
        }
        const float *rm = my_rows + q * width - k;  // rm[i]
        // 64 end layers at a time: which of them are admissible at all (the same for every
        // lane), then only those, in ascending order
        for (int i0 = i_first; i0 <= i_last; i0 += 64) {
          const int i_mine = i0 + lane;
          const float r_mine = i_mine <= i_last ? rm[i_mine] : INFINITY;
          unsigned long long todo = __ballot(i_mine <= i_last && r_mine <= t_max);
          while (todo != 0) {
            const int bit = __ffsll(todo) - 1;
            todo &= todo - 1;
            const int i = i0 + bit;
            const float rmin = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(r_mine), bit));
            float prev[kDpPlaneCols];
#pragma unroll
            for (int j = 0; j < kDpPlaneCols; ++j)
              prev[j] = lane_ok[j] ? col[j][(i + 1) * W] : INFINITY;
            const int at = (q << 8) | i;
#pragma unroll
            for (int j = 0; j < kDpPlaneCols; ++j) {
              const float target = kBottleneck ? fmaxf(rmin, prev[j]) : rmin + prev[j];
              const bool better = target < best[j];
              best[j] = better ? target : best[j];
              best_at[j] = better ? at : best_at[j];
            }
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
      DpBest w[kDpPlaneCols];
#pragma unroll
      for (int j = 0; j < kDpPlaneCols; ++j) {
        if (!col_ok[j]) continue;
        const int d = d_of[j];
        if (best_at[j] >= 0) {
          w[j].best = best[j];
          w[j].arg_q = best_at[j] >> 8;
          w[j].arg_i = best_at[j] & 255;
          w[j].best_rmin = my_rows[w[j].arg_q * width + (w[j].arg_i - k)];
        }
        dp_finish_winner<kBottleneck>(w[j], shape, tabs, off, t_max, p, k, d, f_lds, m_prev);
        const int e = k * W + d;
        f_cur[e] = w[j].best;
        m_cur[e] = w[j].best_m;
        if (w[j].best < INFINITY) {
          atomicMin(&range_cur[2 * d], k);
          atomicMax(&range_cur[2 * d + 1], k);
        }
        if (k == 0) {
          range_next[2 * d] = L + 1;
          range_next[2 * d + 1] = -1;
        }
        if (argmin != nullptr && w[j].arg_i >= 0) {
          int32_t *a = argmin + (((int64_t)t * (shape.max_stages + 1) + s) * plane + e) * 4;
          a[0] = w[j].arg_i;
          a[1] = shape.mesh_n[w[j].arg_q];
          a[2] = shape.mesh_m[w[j].arg_q];
          a[3] = w[j].arg_j;
        }
        // first s wins ties (inter_tuning.py:335-340); (k = 0, d = D) is wavefront 0's first
        // task in every step, the same lane's
        if (k == 0 && d == D && w[j].best < answer_sum) {
          answer_sum = w[j].best;
          answer_s = s;
          answer_max = w[j].best_m;
        }
      }
    }
    __syncthreads();  // every scan of F(s - 1) is done, F(s) is in the scratch plane
    for (int e = threadIdx.x; e < plane; e += blockDim.x) {
      const int k = e / W, d = e - k * W;
      f_lds[e] = (k <= L - s && d >= 1) ? f_cur[e] : INFINITY;
    }
    __syncthreads();
  }
  if (wave == 0 && lane == (D - 1) % 64) {
    best_s_out[t] = answer_s;
    best_sum_out[t] = answer_sum;
    stage_max_out[t] = answer_max;
  }
}

// Follows the back-pointers of each instance from (best_s, layer 0, all devices) and writes its
// stages in pipeline order (inter_tuning.py:341-355); one thread per instance.  Only entries the
// DP wrote are read: a state with a finite value has a winner, and so has every successor on
// its path.
__global__ __launch_bounds__(64) void backtrack_kernel(const MistDpShape shape,
                                                       const int32_t *__restrict__ argmin,
                                                       const int32_t *__restrict__ best_s, int n,
                                                       int32_t *__restrict__ path) {
  const int t = blockIdx.x * 64 + threadIdx.x;
  if (t >= n) return;
  const int L = shape.num_layers, W = shape.num_devices + 1;
  const int64_t plane = (int64_t)(L + 1) * W;
  int32_t *out = path + (int64_t)t * shape.max_stages * 4;
  for (int i = 0; i < shape.max_stages * 4; ++i) out[i] = -1;
  int s = best_s[t], k = 0, d = shape.num_devices, stage = 0;
  while (s > 0 && k < L && stage < shape.max_stages) {
    const int32_t *a = argmin + (((int64_t)t * (shape.max_stages + 1) + s) * plane + k * W + d) * 4;
    const int end = a[0], mesh_n = a[1], mesh_m = a[2];
    // an entry the DP did not write (caller's fill or stale memory) ends the walk: the host sees
    // a path that does not cover the layers
    if (end < k || end >= L || mesh_n < 1 || mesh_m < 1) break;
    if (shape.free_devices == 0 && mesh_n * mesh_m > d) break;
    out[stage * 4 + 0] = end;
    out[stage * 4 + 1] = mesh_n;
    out[stage * 4 + 2] = mesh_m;
    out[stage * 4 + 3] = a[3];
    ++stage;
    --s;
    k = end + 1;
    if (shape.free_devices == 0) d -= mesh_n * mesh_m;
  }
}

// Row minima in the order the recurrence reads them: out[g][p][q][triangle(k, i)] =
// dp_row_min(p, k, q, i).  A workgroup scanning stage count p + 1 of g finds all it needs in one
// contiguous block, and the end layers i of one (q, k) lie next to each other.
__global__ __launch_bounds__(256) void stage_minima_kernel(const MistDpShape shape,
                                                           const MistDpCosts tabs,
                                                           float *__restrict__ out) {
  const int L = shape.num_layers, tri = dp_triangle(L);
  const int x = blockIdx.x * 256 + threadIdx.x;
  if (x >= L * L) return;
  const int k = x / L, di = x % L;
  if (k + di >= L) return;
  const int p = blockIdx.y / shape.num_mesh, q = blockIdx.y % shape.num_mesh;
  const int64_t g = blockIdx.z;
  const int64_t off[4] = {g * tabs.g_stride[0], g * tabs.g_stride[1], g * tabs.g_stride[2],
                          g * tabs.g_stride[3]};
  // a stage count of p + 1 leaves start layers k <= L - 1 - p
  const float value = k <= L - 1 - p ? dp_row_min(shape, tabs, off, p, k, q, k + di) : INFINITY;
  out[((g * shape.max_stages + p) * shape.num_mesh + q) * tri + dp_triangle_row(L, k) + di] = value;
}

// Dynamic LDS the one-launch kernel may use on the current device: what the device reports per
// workgroup, once the kernel has been allowed more than the default 64 KB (0 if that failed).
size_t lds_limit_of(const void *kernel) {
  int device = 0, most = 0;
  if (hipGetDevice(&device) != hipSuccess ||
      hipDeviceGetAttribute(&most, hipDeviceAttributeMaxSharedMemoryPerBlock, device) != hipSuccess)
    return 0;
  if (most > 64 * 1024 &&
      hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, most) != hipSuccess) {
    (void)hipGetLastError();
    most = 64 * 1024;
  }
  return (size_t)most;
}
template <bool kBottleneck>
size_t fused_lds_limit_of() {
  return lds_limit_of(reinterpret_cast<const void *>(&dp_fused_kernel<kBottleneck>));
}
size_t plane_lds_limit(int mode) {
  // per device: the attribute belongs to the device's copy of the kernel
  static std::mutex lock;
  static std::map<std::pair<int, int>, size_t> known;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return 0;
  std::lock_guard<std::mutex> guard(lock);
  const auto key = std::make_pair(device, mode);
  auto it = known.find(key);
  if (it == known.end())
    it = known.emplace(key, lds_limit_of(mode == MIST_DP_BOTTLENECK
                                             ? reinterpret_cast<const void *>(&dp_plane_kernel<true>)
                                             : reinterpret_cast<const void *>(&dp_plane_kernel<false>))).first;
  return it->second;
}
size_t fused_lds_limit(int mode) {
  // per device: the attribute belongs to the device's copy of the kernel
  static std::mutex lock;
  static std::map<std::pair<int, int>, size_t> known;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return 0;
  std::lock_guard<std::mutex> guard(lock);
  const auto key = std::make_pair(device, mode);
  auto it = known.find(key);
  if (it == known.end())
    it = known.emplace(key, mode == MIST_DP_BOTTLENECK ? fused_lds_limit_of<true>()
                                                       : fused_lds_limit_of<false>()).first;
  return it->second;
}

// Scratch of mist_dp_run_static: callers that must not allocate (HIP graph capture, serving
// loops) get the state planes from this array instead of a workspace argument.  Every GPU the
// library runs on holds its own copy at its own address until the process ends.
constexpr int64_t kStaticScratchFloats = (int64_t)4 << 20;  // 16 MiB
static __device__ __align__(256) float scratch[kStaticScratchFloats];
constexpr int kMaxKnownDevices = 64;

// Device address of `scratch` on the current device.  In host code the array's name is only a
// handle for hipGetSymbolAddress, never a pointer a kernel can use; the address is looked up
// once per device (with that device current) and kept.
int static_scratch_of_current_device(float **out) {
  static std::mutex lock;
  static float *known[kMaxKnownDevices] = {};
  int device = 0;
  MIST_HIP_CHECK(hipGetDevice(&device));
  if (device < 0 || device >= kMaxKnownDevices)
    return fail(MIST_E_INVALID, "device ordinal %d outside [0, %d)", device, kMaxKnownDevices);
  std::lock_guard<std::mutex> guard(lock);
  if (known[device] == nullptr) {
    void *ptr = nullptr;
    MIST_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) return fail(MIST_E_HIP, "hipGetSymbolAddress returned a null address");
    known[device] = static_cast<float *>(ptr);
  }
  *out = known[device];
  return 0;
}

int check_shape(const MistDpShape *shape) {
  if (!shape) return fail(MIST_E_INVALID, "null DP shape");
  if (shape->free_devices != 0 && (shape->num_devices != 0 || shape->num_mesh != 1))
    return fail(MIST_E_INVALID, "free_devices needs num_devices = 0 and one mesh (got D=%d Q=%d)",
                shape->num_devices, shape->num_mesh);
  if (shape->ckpt_rule < MIST_DP_CKPT_TAIL || shape->ckpt_rule > MIST_DP_CKPT_ALL)
    return fail(MIST_E_INVALID, "unknown ckpt_rule %d", shape->ckpt_rule);
  if (shape->num_layers <= 0 || shape->p_dim <= 0 ||
      (shape->free_devices ? shape->num_devices != 0 : shape->num_devices <= 0))
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

int check_run_arguments(const MistDpShape *shape, const MistDpCosts *costs, const float *d_tmax,
                        const int32_t *d_g_index, int n_tmax, int mode, const int32_t *d_best_s,
                        const float *d_best_sum, const float *d_stage_max) {
  if (int rc = check_shape(shape)) return rc;
  if (!costs || !costs->costs || !costs->costs_pre || !costs->costs_post || !costs->costs_nopp ||
      !costs->pmin || !costs->pmin_pre || !costs->pmin_post || !costs->pmin_nopp)
    return fail(MIST_E_INVALID, "null cost table");
  if (!d_tmax || !d_g_index || !d_best_s || !d_best_sum || !d_stage_max)
    return fail(MIST_E_INVALID, "null threshold / output pointer");
  if (n_tmax <= 0 || n_tmax > 65535)
    return fail(MIST_E_INVALID, "n_tmax must be in [1, 65535], got %d", n_tmax);
  if (mode != MIST_DP_THRESHOLD && mode != MIST_DP_BOTTLENECK)
    return fail(MIST_E_INVALID, "unknown DP mode %d", mode);
  return 0;
}

// Small batches are latency-bound: spread every state over a team of lanes.
bool dp_wide_teams(int n_tmax, int plane) { return (int64_t)n_tmax * plane <= (1 << 19); }

// One launch per stage count; the state planes and reachable ranges of all instances live in
// d_scratch (mist_dp_scratch_floats() floats, no particular contents expected on entry: the
// first kernel writes everything a later one reads).
int run_step_schedule(const MistDpShape *shape, const MistDpCosts *costs, const float *d_tmax,
                      const int32_t *d_g_index, int n_tmax, int mode, int32_t *d_best_s,
                      float *d_best_sum, float *d_stage_max, int32_t *d_argmin, float *d_scratch,
                      void *stream) {
  const int plane = (shape->num_layers + 1) * (shape->num_devices + 1);
  const bool wide = dp_wide_teams(n_tmax, plane);
  const int64_t n_init = (int64_t)n_tmax * plane;
  int32_t *d_ranges = reinterpret_cast<int32_t *>(d_scratch + (int64_t)4 * n_tmax * plane);
  hipLaunchKernelGGL(dp_init_kernel, dim3((unsigned)((n_init + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, *shape, n_tmax, d_scratch, d_ranges, d_best_s,
                     d_best_sum, d_stage_max);
  MIST_HIP_CHECK(hipGetLastError());
  const int states_per_block = kDpThreads / (wide ? kDpWideTeam : 1);
  const dim3 grid((plane + states_per_block - 1) / states_per_block, n_tmax);
  for (int s = 1; s <= shape->max_stages; ++s) {
#define MIST_DP_STEP(BOTTLENECK, TEAM)                                                         \
  hipLaunchKernelGGL((dp_step_kernel<BOTTLENECK, TEAM>), grid, dim3(kDpThreads), 0,            \
                     (hipStream_t)stream, *shape, *costs, d_tmax, d_g_index, s, d_scratch,     \
                     d_ranges, d_best_s, d_best_sum, d_stage_max, d_argmin)
    if (mode == MIST_DP_BOTTLENECK) {
      if (wide) MIST_DP_STEP(true, kDpWideTeam); else MIST_DP_STEP(true, 1);
    } else {
      if (wide) MIST_DP_STEP(false, kDpWideTeam); else MIST_DP_STEP(false, 1);
    }
#undef MIST_DP_STEP
    MIST_HIP_CHECK(hipGetLastError());
  }
  return 0;
}

}  // namespace

extern "C" {

int mist_sizeof_dp_shape(void) { return (int)sizeof(MistDpShape); }

int mist_dp_cost_tables(const MistProblem *problem, const MistOutTables *tables,
                        const int32_t *d_grad_accum, int slot, float *const d_out[4],
                        float *const d_out_pmin[4], void *stream) {
  if (!problem || !tables || !d_grad_accum || !d_out || !d_out_pmin)
    return fail(MIST_E_INVALID, "null pointer argument");
  const int64_t L = problem->num_layers, P1 = problem->p_dim, S = problem->sample_size;
  const int64_t Gn = problem->num_grad_accum, Q = problem->num_mesh;
  if (L <= 0 || P1 <= 0 || S <= 0 || Gn <= 0 || Q <= 0)
    return fail(MIST_E_INVALID, "bad problem extents");
  if (slot < 0 || slot >= S) return fail(MIST_E_INVALID, "slot %d outside [0, %d)", slot, (int)S);
  const int64_t rows_per_g[4] = {Q * P1 * L, Q * P1 * L, Q * L, Q};
  const int64_t rows_per_block = 256 / std::min<int64_t>(L + 1, 256);
  CostTableJob job = {};
  int64_t blocks = 0;
  for (int v = 0; v < 4; ++v) {
    if (!tables->stable[v] || !tables->delta[v] || !d_out[v] || !d_out_pmin[v])
      return fail(MIST_E_INVALID, "table %d is null", v);
    job.stable[v] = tables->stable[v];
    job.delta[v] = tables->delta[v];
    job.index[v] = tables->index[v];
    job.out[v] = d_out[v];
    job.pmin[v] = d_out_pmin[v];
    job.n_rows[v] = Gn * rows_per_g[v];
    job.rows_per_g[v] = rows_per_g[v];
    job.first_block[v] = (unsigned)blocks;
    blocks += (job.n_rows[v] + rows_per_block - 1) / rows_per_block;
  }
  if (blocks >= (int64_t)1 << 31) return fail(MIST_E_INVALID, "cost tables too large for one launch");
  job.first_block[4] = (unsigned)blocks;
  hipLaunchKernelGGL(cost_table_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, job,
                     d_grad_accum, (int)(L + 1), (int)S, slot);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int mist_dp_backtrack(const MistDpShape *shape, const int32_t *d_argmin, const int32_t *d_best_s,
                      int n_tmax, int32_t *d_path, void *stream) {
  if (int rc = check_shape(shape)) return rc;
  if (!d_argmin || !d_best_s || !d_path) return fail(MIST_E_INVALID, "null pointer argument");
  if (n_tmax <= 0 || n_tmax > 65535)
    return fail(MIST_E_INVALID, "n_tmax must be in [1, 65535], got %d", n_tmax);
  hipLaunchKernelGGL(backtrack_kernel, dim3((unsigned)((n_tmax + 63) / 64)), dim3(64), 0,
                     (hipStream_t)stream, *shape, d_argmin, d_best_s, n_tmax, d_path);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int64_t mist_dp_stage_minima_floats(const MistDpShape *shape) {
  if (check_shape(shape) != 0) return -1;
  return (int64_t)shape->max_stages * shape->num_mesh * dp_triangle(shape->num_layers);
}

int mist_dp_stage_minima(const MistDpShape *shape, const MistDpCosts *costs, int num_grad_accum,
                         float *d_out, void *stream) {
  if (int rc = check_shape(shape)) return rc;
  if (!costs || !costs->costs || !costs->costs_pre || !costs->costs_post || !costs->costs_nopp ||
      !costs->pmin || !costs->pmin_pre || !costs->pmin_post || !costs->pmin_nopp)
    return fail(MIST_E_INVALID, "null cost table");
  if (!d_out) return fail(MIST_E_INVALID, "null output pointer");
  if (num_grad_accum < 1 || num_grad_accum > 65535)
    return fail(MIST_E_INVALID, "num_grad_accum must be in [1, 65535], got %d", num_grad_accum);
  const int L = shape->num_layers;
  hipLaunchKernelGGL(stage_minima_kernel,
                     dim3((unsigned)((L * L + 255) / 256),
                          (unsigned)(shape->max_stages * shape->num_mesh),
                          (unsigned)num_grad_accum),
                     dim3(256), 0, (hipStream_t)stream, *shape, *costs, d_out);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int mist_dp_filter_tmax(const float *sorted_unique, int n, double gap, float *out) {
  if (n < 0 || (n > 0 && (!sorted_unique || !out))) return fail(MIST_E_INVALID, "bad t_max list");
  int kept = 0;
  float last = 0.0f;
  for (int i = 0; i < n; ++i) {
    const float t = sorted_unique[i];
    if (gap_below(t, last, gap)) continue;
    out[kept++] = t;
    last = t;
  }
  return kept;
}

int mist_dp_window_begin(const float *ascending, int n, float lo, int open_below,
                         float start_value, double gap, float *out) {
  if (n < 0 || (n > 0 && (!ascending || !out))) return fail(MIST_E_INVALID, "bad candidate list");
  if (n == 0) return 0;
  const int first = window_walk_start(ascending, n, lo, open_below != 0, start_value, gap);
  if (first < 0) return MIST_DP_NO_START;
  return mist_dp_filter_tmax(ascending + first, n - first, gap, out);  // the walk from there
}

int mist_dp_window_begin_many(const float *ascending, const int64_t *offsets, int n_windows,
                              const float *lo, const uint8_t *open_below,
                              const float *start_value, double gap, float *out,
                              int32_t *out_count) {
  if (n_windows < 0) return fail(MIST_E_INVALID, "n_windows %d < 0", n_windows);
  if (n_windows == 0) return 0;
  if (!offsets || !lo || !open_below || !start_value || !out_count)
    return fail(MIST_E_INVALID, "null pointer argument");
  for (int w = 0; w < n_windows; ++w) {
    const int64_t first = offsets[w], count = offsets[w + 1] - first;
    if (first < 0 || count < 0 || count > INT32_MAX)
      return fail(MIST_E_INVALID, "offsets of window %d are not ascending", w);
    const int kept =
        mist_dp_window_begin(count ? ascending + first : nullptr, (int)count, lo[w], open_below[w],
                             start_value[w], gap, count ? out + first : nullptr);
    if (kept < 0 && kept != MIST_DP_NO_START) return kept;
    out_count[w] = kept;
  }
  return 0;
}

int mist_dp_select_candidates(const MistDpCosts *costs, int n_requests, const int32_t *d_rows,
                              const float *d_lo, const float *d_hi, float *d_out_values,
                              int32_t *d_out_request, int capacity, int32_t *d_counts,
                              void *stream) {
  if (!costs || !costs->costs || !costs->costs_pre || !costs->costs_post)
    return fail(MIST_E_INVALID, "null cost tables");
  if (n_requests <= 0 || n_requests > 65535)
    return fail(MIST_E_INVALID, "n_requests %d outside [1, 65535]", n_requests);
  if (!d_rows || !d_lo || !d_hi || !d_out_values || !d_out_request || !d_counts || capacity <= 0)
    return fail(MIST_E_INVALID, "null pointer / empty output list");
  const int64_t per_row = costs->g_stride[0] + costs->g_stride[1] + costs->g_stride[2];
  // few, long-running workgroups per request: each appends to the output list once per
  // kSelectBuffer values at most
  const unsigned blocks = (unsigned)std::min<int64_t>((per_row + 16383) / 16384, 64);
  hipLaunchKernelGGL(select_candidates_kernel, dim3(blocks, n_requests), dim3(256), 0,
                     (hipStream_t)stream, *costs, d_rows, d_lo, d_hi, d_out_values, d_out_request,
                     capacity, d_counts, false);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int mist_dp_first_batch_index(int k, int n_avail, int first_chunk, int first_lead) {
  if (k < 0 || first_chunk < 1 || first_lead < 1 || k >= std::min(first_chunk, n_avail)) return -1;
  return dp_first_batch_index(k, n_avail, first_chunk, first_lead);
}

int mist_dp_windows_first_batch(const MistDpCosts *costs, int n_requests, const int32_t *d_rows,
                                const float *d_lo, const float *d_hi, const float *d_start,
                                double gap, int window_capacity, int first_chunk, int first_lead,
                                float *d_values, int32_t *d_counts, float *d_kept,
                                int kept_capacity, int32_t *d_meta, float *d_inst_tmax,
                                int32_t *d_inst_row, void *stream) {
  if (!costs || !costs->costs || !costs->costs_pre || !costs->costs_post)
    return fail(MIST_E_INVALID, "null cost tables");
  if (n_requests <= 0 || n_requests > 65535)
    return fail(MIST_E_INVALID, "n_requests %d outside [1, 65535]", n_requests);
  if (!d_rows || !d_lo || !d_hi || !d_start || !d_values || !d_counts || !d_kept || !d_meta ||
      !d_inst_tmax || !d_inst_row)
    return fail(MIST_E_INVALID, "null pointer argument");
  if (window_capacity < 128 || window_capacity > 8192 || (window_capacity & (window_capacity - 1)))
    return fail(MIST_E_INVALID, "window_capacity %d is no power of two in [128, 8192]", window_capacity);
  if (first_chunk < 1 || kept_capacity < 1 || (int64_t)n_requests * first_chunk > 65535)
    return fail(MIST_E_INVALID, "first_chunk %d x %d requests outside [1, 65535] / empty kept list",
                first_chunk, n_requests);
  if (first_lead < 1) return fail(MIST_E_INVALID, "first_lead %d < 1", first_lead);
  hipStream_t st = (hipStream_t)stream;
  MIST_HIP_CHECK(hipMemsetAsync(d_counts, 0, sizeof(int32_t) * (2 + 2 * (size_t)n_requests), st));
  MIST_HIP_CHECK(hipMemsetAsync(d_inst_row, 0xFF, sizeof(int32_t) * (size_t)n_requests * first_chunk, st));
  const int64_t per_row = costs->g_stride[0] + costs->g_stride[1] + costs->g_stride[2];
  const unsigned blocks = (unsigned)std::min<int64_t>((per_row + 16383) / 16384, 64);
  hipLaunchKernelGGL(select_candidates_kernel, dim3(blocks, n_requests), dim3(256), 0, st, *costs,
                     d_rows, d_lo, d_hi, d_values, (int32_t *)nullptr, window_capacity, d_counts,
                     true);
  MIST_HIP_CHECK(hipGetLastError());
  const size_t lds = (size_t)window_capacity * (sizeof(float) + sizeof(uint8_t));
  hipLaunchKernelGGL(window_walk_kernel, dim3(n_requests), dim3(kWindowThreads), lds, st, d_values,
                     window_capacity, d_counts, d_rows, d_lo, d_start, gap, first_chunk, first_lead,
                     d_kept, kept_capacity, d_meta, d_inst_tmax, d_inst_row);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int64_t mist_dp_scratch_floats(const MistDpShape *shape, int n_tmax) {
  if (check_shape(shape) != 0 || n_tmax <= 0) return -1;
  // four state planes per instance, then three buffers of (first, last) reachable row per
  // instance and device column
  return (int64_t)4 * n_tmax * (shape->num_layers + 1) * (shape->num_devices + 1) +
         (int64_t)6 * n_tmax * (shape->num_devices + 1);
}

int mist_dp_run(const MistDpShape *shape, const MistDpCosts *costs, const float *d_tmax,
                const int32_t *d_g_index, int n_tmax, int mode, int32_t *d_best_s,
                float *d_best_sum, float *d_stage_max, int32_t *d_argmin, float *d_scratch,
                void *stream) {
  if (int rc = check_run_arguments(shape, costs, d_tmax, d_g_index, n_tmax, mode, d_best_s,
                                   d_best_sum, d_stage_max))
    return rc;
  if (!d_scratch) return fail(MIST_E_INVALID, "null scratch pointer");
  const int plane = (shape->num_layers + 1) * (shape->num_devices + 1);
  const bool wide = dp_wide_teams(n_tmax, plane);
  // Larger ones: one workgroup per instance with its planes in LDS when they fit and the caller
  // prepared the re-laid row minima.
  const size_t fused_lds =
      ((size_t)4 * plane + (size_t)6 * (shape->num_devices + 1) +
       (size_t)shape->num_mesh * dp_triangle(shape->num_layers) +
       (size_t)2 * shape->num_mesh * shape->num_layers) *
      sizeof(float);
  // (threshold batches from about 64 instances on: a workgroup's run through all stage counts
  // takes as long as the 1 + max_stages launches of a few dozen instances)
  bool fused_pays = mode == MIST_DP_THRESHOLD ? n_tmax >= kDpFusedMinInstances : !wide;
  // (small planes: a workgroup's run through all stage counts is shorter than the launches it
  // replaces whatever the batch size - GPT-7B's 33 x 33 plane: bottleneck batch of 40 instances
  // and the back-pointer run of one, 0.07 ms per search; 41 x 65 is already the other way round)
  fused_pays = fused_pays || plane <= kDpFusedSmallPlane;
  // For tests: MIST_DP_FORCE_SCHEDULE = step | fused | plane takes the choice of schedule away
  // from the batch size and the LDS need, so that each schedule can be run on any shape it
  // supports (a shape it does not support is an error, not a silent fallback).
  const char *forced = getenv("MIST_DP_FORCE_SCHEDULE");
  const bool force_step = forced && !strcmp(forced, "step");
  const bool force_fused = forced && !strcmp(forced, "fused");
  const bool force_plane = forced && !strcmp(forced, "plane");
  if (forced && *forced && !force_step && !force_fused && !force_plane)
    return fail(MIST_E_INVALID, "MIST_DP_FORCE_SCHEDULE=%s: expected step, fused or plane", forced);
  if (force_fused) {
    if (costs->stage_min == nullptr || fused_lds > fused_lds_limit(mode))
      return fail(MIST_E_INVALID, "forced fused schedule: needs stage_min and %zu B of LDS", fused_lds);
    fused_pays = true;
  }
  if (force_step || force_plane) fused_pays = false;
  if (fused_pays && costs->stage_min != nullptr && fused_lds <= fused_lds_limit(mode)) {
    // one workgroup per CU when the planes take more than half of the LDS: then a larger one
    const int most = 2 * fused_lds > kDpLdsPerCu ? kDpFusedThreads : kDpFusedThreads / 2;
    const int threads = std::min(most, (plane + 63) / 64 * 64);
    if (mode == MIST_DP_BOTTLENECK)
      hipLaunchKernelGGL(dp_fused_kernel<true>, dim3(n_tmax), dim3(threads), fused_lds,
                         (hipStream_t)stream, *shape, *costs, d_tmax, d_g_index, d_best_s,
                         d_best_sum, d_stage_max, d_argmin);
    else
      hipLaunchKernelGGL(dp_fused_kernel<false>, dim3(n_tmax), dim3(threads), fused_lds,
                         (hipStream_t)stream, *shape, *costs, d_tmax, d_g_index, d_best_s,
                         d_best_sum, d_stage_max, d_argmin);
    MIST_HIP_CHECK(hipGetLastError());
    return 0;
  }
  // Planes beyond the LDS of a compute unit (80 layers x 256 devices): one workgroup per instance
  // with F(s - 1) alone in LDS, one launch.
  const size_t plane_lds =
      ((size_t)plane + 6 * (size_t)(shape->num_devices + 1) + 2 * (size_t)shape->num_mesh +
       (size_t)(kDpPlaneThreads / 64) * shape->num_mesh * shape->num_layers) * sizeof(float);
  const bool plane_shape_ok = shape->num_devices <= 64 * kDpPlaneCols &&
                              shape->num_mesh * shape->num_layers <= 64 * kDpPlaneLoads &&
                              shape->num_layers <= 256;  // (mesh << 8 | end layer) of a winner
  const bool plane_possible = costs->stage_min != nullptr && shape->free_devices == 0 &&
                              plane_shape_ok && plane_lds <= plane_lds_limit(mode);
  if (force_plane && !plane_possible)
    return fail(MIST_E_INVALID, "forced plane schedule: needs stage_min, consumed devices, D <= %d, "
                "Q * L <= %d and %zu B of LDS", 64 * kDpPlaneCols, 64 * kDpPlaneLoads, plane_lds);
  if (plane_possible && !force_step &&
      (force_plane || (n_tmax >= kDpPlaneMinInstances && fused_lds > fused_lds_limit(mode)))) {
    if (mode == MIST_DP_BOTTLENECK)
      hipLaunchKernelGGL(dp_plane_kernel<true>, dim3(n_tmax), dim3(kDpPlaneThreads), plane_lds,
                         (hipStream_t)stream, *shape, *costs, d_tmax, d_g_index, d_scratch,
                         d_best_s, d_best_sum, d_stage_max, d_argmin);
    else
      hipLaunchKernelGGL(dp_plane_kernel<false>, dim3(n_tmax), dim3(kDpPlaneThreads), plane_lds,
                         (hipStream_t)stream, *shape, *costs, d_tmax, d_g_index, d_scratch,
                         d_best_s, d_best_sum, d_stage_max, d_argmin);
    MIST_HIP_CHECK(hipGetLastError());
    return 0;
  }
  return run_step_schedule(shape, costs, d_tmax, d_g_index, n_tmax, mode, d_best_s, d_best_sum,
                           d_stage_max, d_argmin, d_scratch, stream);
}

int64_t mist_dp_static_scratch_floats(void) { return kStaticScratchFloats; }

int mist_dp_run_static(const MistDpShape *shape, const MistDpCosts *costs, const float *d_tmax,
                       const int32_t *d_g_index, int n_tmax, int mode, int32_t *d_best_s,
                       float *d_best_sum, float *d_stage_max, int32_t *d_argmin, void *stream) {
  if (int rc = check_run_arguments(shape, costs, d_tmax, d_g_index, n_tmax, mode, d_best_s,
                                   d_best_sum, d_stage_max))
    return rc;
  const int64_t need = mist_dp_scratch_floats(shape, n_tmax);
  if (need < 0 || need > kStaticScratchFloats)
    return fail(MIST_E_INVALID,
                "mist_dp_run_static: %d instances of (L=%d, D=%d) need %lld scratch floats, the "
                "built-in scratch holds %lld; use mist_dp_run with a caller-owned scratch",
                n_tmax, shape->num_layers, shape->num_devices, (long long)need,
                (long long)kStaticScratchFloats);
  float *d_scratch = nullptr;
  if (int rc = static_scratch_of_current_device(&d_scratch)) return rc;
  return run_step_schedule(shape, costs, d_tmax, d_g_index, n_tmax, mode, d_best_s, d_best_sum,
                           d_stage_max, d_argmin, d_scratch, stream);
}

}  // extern "C"
