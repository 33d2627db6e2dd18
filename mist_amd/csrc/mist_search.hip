// Intra-stage configuration search on MI355X (gfx950): row terms, fused evaluate+mask+argmin,
// finalize.  Everything is float64 VALU work with float32 rounding points where the reference
// has them; there is no dense contraction here, so no MFMA.
//
// Bit-exactness rules for this file (results must equal the numpy formulation operation for
// operation): compile with -ffp-contract=off, keep the operand order of every sum exactly as
// written, use true divisions, and never reassociate.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <type_traits>

#include "mist_common.h"
#include "mist_search.h"
#define MIST_ARITH_FN __device__ __forceinline__
#include "exact_arith.h"

namespace {
thread_local char g_last_error[512] = "";
}  // namespace

namespace mist {
int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}
}  // namespace mist

namespace {

using mist::fail;

constexpr int kTermsBlock = 128;  // rows per workgroup of the row-term kernel
constexpr int kStageRows = 64;    // rows staged through LDS per step of the reduce kernel
constexpr int kSlots = 2 * MIST_P_TILE + 2;  // per-thread running minima: base, with_pre, post, no_pp
constexpr double kIncumbentSlack = 0.25;  // relative room above MistProblem.stage_cost_incumbent / G
// Stage summaries (written with the row terms, read by the reduce kernel): per stage of
// kStageRows workspace rows the term-wise minimum of the latency and memory columns and the
// maximum of MIST_T_OUT, kStageFloorPitch doubles per stage.
constexpr int kStageFloorPitch = 32;
constexpr int kStageMaxOut = MIST_T_GCB + 1;  // slot of max(MIST_T_OUT) behind the stage minima
// ... and behind it the minima of the post-layer terms that the last-stage / single-stage
// objectives add to every row: MIST_T_OPB, the smaller of MIST_T_NAG_CK / _NOCK, the smaller of
// MIST_T_NRS_CK / _NOCK.
constexpr int kStageMinOpb = kStageMaxOut + 1, kStageMinNag = kStageMaxOut + 2, kStageMinNrs = kStageMaxOut + 3;
static_assert(kStageMinNrs < kStageFloorPitch, "a stage summary is one 32-lane load");
static_assert(MIST_T_NAG_NOCK == MIST_T_NAG_CK + 1 && MIST_T_NRS_NOCK == MIST_T_NRS_CK + 1, "ck / nock pairs");
static_assert(kStageRows == 2 * kStageFloorPitch, "lane = (column, half of the rows)");

// ------------------------------------------------------------------------------------------
// Communication models (mist/tools/optimize.py:257-303, 459-470).
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ int size_index(double s) {
  return s == 1.0 ? 0 : (s == 2.0 ? 1 : (s == 4.0 ? 2 : 3));
}

__device__ __forceinline__ double gpu_gpu_latency(const double *gg, double mbytes, double inter,
                                                  double intra, double factor) {
  const double gbytes = mbytes / 1024.0;
  const double ngpu = intra * inter;
  double lat = 0.0;
  if (!(gbytes < 1e-5 || ngpu == 1.0)) {
    const double *cell = gg + (size_index(inter) * 4 + size_index(intra)) * 2;
    lat = gbytes / cell[0] * (ngpu - 1.0) / ngpu + cell[1];
  }
  return lat * factor;
}

__device__ __forceinline__ double host_link_latency(const double *kb, double mbytes) {
  const double gbytes = mbytes / 1024.0;
  const double lat = gbytes / kb[0] + kb[1];
  return gbytes == 0.0 ? 0.0 : lat;
}

// numpy's float64 floor_divide (npy_divmod), for a >= 0 and b > 0 as well as the general case.
__device__ __forceinline__ double np_floor_divide(double a, double b) {
  if (__builtin_expect(mist_arith::floor_divide_is_tame(a, b), 1))
    return mist_arith::floor_divide_tame(a, b);
  if (b == 0.0) return a / b;
  double mod = fmod(a, b);
  double div = (a - mod) / b;
  if (mod != 0.0) {
    if ((b < 0.0) != (mod < 0.0)) div -= 1.0;
  }
  double floordiv;
  if (div != 0.0) {
    floordiv = floor(div);
    if (div - floordiv > 0.5) floordiv += 1.0;
  } else {
    floordiv = copysign(0.0, a / b);
  }
  return floordiv;
}

// ------------------------------------------------------------------------------------------
// Four-resource interference model (mist/tools/optimize.py:1012-1122).  X = [C, G2G, C2G, G2C].
// Masks in evaluation order: 4-way, four 3-way, six 2-way; bit j set = resource j in the mask.
// ------------------------------------------------------------------------------------------
constexpr unsigned char kMaskBits[11] = {
    0xF,
    0x7, 0xB, 0xD, 0xE,
    0x3, 0x5, 0x9, 0x6, 0xA, 0xC,
};

// Index into kMaskBits of the mask equal to a pattern of two or more bits, as 16 nibbles of one
// constant (a table in memory would cost every peel a dependent load).
constexpr uint64_t pack_mask_of_pattern() {
  uint64_t packed = 0;
  for (int m = 0; m < 11; ++m) packed |= (uint64_t)m << (4 * kMaskBits[m]);
  return packed;
}
constexpr uint64_t kMaskOfPatternPacked = pack_mask_of_pattern();
__device__ __forceinline__ int mask_of_pattern(unsigned pattern) {
  return (int)((kMaskOfPatternPacked >> (4 * pattern)) & 0xF);
}
static_assert(((kMaskOfPatternPacked >> (4 * 0xF)) & 0xF) == 0 && ((kMaskOfPatternPacked >> (4 * 0x3)) & 0xF) == 5 &&
                  ((kMaskOfPatternPacked >> (4 * 0xC)) & 0xF) == 10 && ((kMaskOfPatternPacked >> (4 * 0xE)) & 0xF) == 4,
              "pattern -> mask index");

// The factor table lives in LDS and is read through a pointer of that address space: the model
// is out of line, and through a generic pointer every read would be a flat load.
typedef const __attribute__((address_space(3))) double LdsDouble;
constexpr int kFactorPitch = 8;  // per mask: the four factors, then their four reciprocals

// kInline: the model is expanded at every call site (for a kernel with few of them: its loads
// stay in flight across the evaluations, which a call would make it wait for) instead of called.
template <bool kInline>
struct InterferenceModel {
  LdsDouble *table;   // [11][kFactorPitch]: factor[m][0..3], 1 / factor[m][0..3] correctly rounded
  bool factors_tame;  // every factor lies in the divisor range of the reciprocal quotient

  // Operands (seconds) below this bound keep every scaled time and every quotient of a peel
  // inside the range where the reciprocal quotient is the IEEE quotient; a peel only divides
  // differences of scaled times of resources busier than 1e-8 s, which are zero or no smaller
  // than an ulp of 1e-8.
  static constexpr double kOperandBound = 0x1p500;

  // Arguments in the order of the reference's get_layer_critical_latency
  // (batched_module_analyzer.py:1413-1422): exec, gpu<->gpu, gpu->cpu, cpu->gpu.
  // kLive: bit i set when X[i] (exec, gpu<->gpu, cpu->gpu, gpu->cpu) can be non-zero at this call
  // site; the others are literal zeros there, never part of a mask, and their share of a round
  // (a multiplication and a division each) is left out at compile time.  The sums keep all four
  // operands, so the value is the one of the general form.
  // kByReciprocal: the quotients (s - overlap) / factor are taken with the stored reciprocals
  // (five multiply-adds, no branch, so that the four quotients of a peel interleave) instead of
  // the division sequence; eval() picks it when every operand of the wave is in range.
  template <unsigned kLive, bool kByReciprocal>
  __device__ __noinline__ double eval_called(double exec, double g2g, double g2c, double c2g) const {
    return eval_body<kLive, kByReciprocal>(exec, g2g, g2c, c2g);
  }
  template <unsigned kLive, bool kByReciprocal>
  __device__ __forceinline__ double eval_as(double exec, double g2g, double g2c, double c2g) const {
    if constexpr (kInline || __builtin_popcount(kLive) < 2)
      return eval_body<kLive, kByReciprocal>(exec, g2g, g2c, c2g);
    else
      return eval_called<kLive, kByReciprocal>(exec, g2g, g2c, c2g);
  }
  template <unsigned kLive, bool kByReciprocal>
  __device__ __forceinline__ double eval_body(double exec, double g2g, double g2c, double c2g) const {
    double x0 = (kLive & 1u) ? exec : 0.0, x1 = (kLive & 2u) ? g2g : 0.0;
    double x2 = (kLive & 4u) ? c2g : 0.0, x3 = (kLive & 8u) ? g2c : 0.0;
    double out = 0.0;
    // The reference tries the 11 masks in order and applies the one equal to the non-zero
    // pattern of X.  A pattern equals at most one mask, and after a peel the pattern has fewer
    // bits, i.e. it can only equal a mask further down the list (4-way, then 3-way, then
    // 2-way).  So the rounds are taken by the size of the pattern: a lane joins at the size of
    // its own pattern, and the wave runs each size once.
    // "not isclose(x, 0)" with numpy's default tolerances: |x| > 1e-8.
    auto pattern = [&]() {
      return (((kLive & 1u) && !(fabs(x0) <= 1e-8)) ? 1u : 0u) |
             (((kLive & 2u) && !(fabs(x1) <= 1e-8)) ? 2u : 0u) |
             (((kLive & 4u) && !(fabs(x2) <= 1e-8)) ? 4u : 0u) |
             (((kLive & 8u) && !(fabs(x3) <= 1e-8)) ? 8u : 0u);
    };
    // a / f for a = s - overlap >= +0 (never -0: a difference of equal numbers is +0).
    auto quotient = [&](double a, double f, double y) {
      if (!kByReciprocal) return a / f;
      return mist_arith::quotient_by_reciprocal<false>(a, f, y, a * y);
    };
    // One peel as the reference writes it: every busy resource gives up the smallest scaled
    // time.  (s - ov) / f * 1.0 there: the product with 1.0 changes nothing.
    auto peel = [&](unsigned mask) {
      LdsDouble *row = table + mask_of_pattern(mask) * kFactorPitch;
      const double f0 = row[0], f1 = row[1], f2 = row[2], f3 = row[3];
      const double y0 = row[4], y1 = row[5], y2 = row[6], y3 = row[7];
      const double s0 = x0 * f0, s1 = x1 * f1, s2 = x2 * f2, s3 = x3 * f3;
      double ov = INFINITY;
      if ((kLive & 1u) && (mask & 1u)) ov = fmin(ov, s0);
      if ((kLive & 2u) && (mask & 2u)) ov = fmin(ov, s1);
      if ((kLive & 4u) && (mask & 4u)) ov = fmin(ov, s2);
      if ((kLive & 8u) && (mask & 8u)) ov = fmin(ov, s3);
      if ((kLive & 1u) && (mask & 1u)) x0 = quotient(s0 - ov, f0, y0);
      if ((kLive & 2u) && (mask & 2u)) x1 = quotient(s1 - ov, f1, y1);
      if ((kLive & 4u) && (mask & 4u)) x2 = quotient(s2 - ov, f2, y2);
      if ((kLive & 8u) && (mask & 8u)) x3 = quotient(s3 - ov, f3, y3);
      out = out + ov;
    };
    // The same peel for two busy resources with one division: the one with the smaller scaled
    // time is left with (s - s) / f = +0 (factors are positive and finite), the other with
    // (larger - smaller) / its factor; with equal times both quotients are +0.
    auto peel_pair = [&](unsigned mask) {
      LdsDouble *row = table + mask_of_pattern(mask) * kFactorPitch;
      const double f0 = row[0], f1 = row[1], f2 = row[2], f3 = row[3];
      const double s0 = x0 * f0, s1 = x1 * f1, s2 = x2 * f2, s3 = x3 * f3;
      const bool b0 = (kLive & 1u) && (mask & 1u), b1 = (kLive & 2u) && (mask & 2u);
      const bool b2 = (kLive & 4u) && (mask & 4u), b3 = (kLive & 8u) && (mask & 8u);
      double lo = INFINITY, hi = -INFINITY;
      if (b0) { lo = fmin(lo, s0); hi = fmax(hi, s0); }
      if (b1) { lo = fmin(lo, s1); hi = fmax(hi, s1); }
      if (b2) { lo = fmin(lo, s2); hi = fmax(hi, s2); }
      if (b3) { lo = fmin(lo, s3); hi = fmax(hi, s3); }
      double den = 1.0, rden = 1.0;
      if (b0 && s0 == hi) { den = f0; rden = row[4]; }
      if (b1 && s1 == hi) { den = f1; rden = row[5]; }
      if (b2 && s2 == hi) { den = f2; rden = row[6]; }
      if (b3 && s3 == hi) { den = f3; rden = row[7]; }
      const double rest = quotient(hi - lo, den, rden);
      if (b0) x0 = s0 == hi ? rest : 0.0;
      if (b1) x1 = s1 == hi ? rest : 0.0;
      if (b2) x2 = s2 == hi ? rest : 0.0;
      if (b3) x3 = s3 == hi ? rest : 0.0;
      out = out + lo;
    };
    constexpr int kLiveCount = __builtin_popcount(kLive);
    if constexpr (kLiveCount == 4) {
      const unsigned nz = pattern();
      if (nz == 15u) peel(nz);
    }
    if constexpr (kLiveCount >= 3) {
      const unsigned nz = pattern();
      if (__popc(nz) == 3) peel(nz);
    }
    if constexpr (kLiveCount >= 2) {
      const unsigned nz = pattern();
      if (__popc(nz) == 2) peel_pair(nz);
    }
    return out + (((x0 + x1) + x2) + x3);
  }

  template <unsigned kLive>
  __device__ __forceinline__ double eval(double exec, double g2g, double g2c, double c2g) const {
    if constexpr (__builtin_popcount(kLive) < 2) {
      return eval_as<kLive, false>(exec, g2g, g2c, c2g);  // nothing to divide
    } else {
      // NaN and infinities fail the comparisons and take the division sequence, wave-wide.
      const bool tame = factors_tame &&
                        (!(kLive & 1u) || fabs(exec) < kOperandBound) &&
                        (!(kLive & 2u) || fabs(g2g) < kOperandBound) &&
                        (!(kLive & 4u) || fabs(c2g) < kOperandBound) &&
                        (!(kLive & 8u) || fabs(g2c) < kOperandBound);
      if (__builtin_expect(__all(tame), 1)) return eval_as<kLive, true>(exec, g2g, g2c, c2g);
      return eval_called<kLive, false>(exec, g2g, g2c, c2g);  // never expanded in place: cold
    }
  }

  __device__ __forceinline__ double operator()(double exec, double g2g, double g2c, double c2g) const {
    return eval<15u>(exec, g2g, g2c, c2g);
  }
  // Call sites whose literal zeros are known: operands named by what is live.
  __device__ __forceinline__ double exec_g2g_c2g(double exec, double g2g, double c2g) const {
    return eval<1u | 2u | 4u>(exec, g2g, 0.0, c2g);
  }
  __device__ __forceinline__ double exec_g2g_g2c(double exec, double g2g, double g2c) const {
    return eval<1u | 2u | 8u>(exec, g2g, g2c, 0.0);
  }
  __device__ __forceinline__ double g2g_c2g(double g2g, double c2g) const {
    return eval<2u | 4u>(0.0, g2g, 0.0, c2g);
  }
  __device__ __forceinline__ double g2g_g2c(double g2g, double g2c) const {
    return eval<2u | 8u>(0.0, g2g, g2c, 0.0);
  }
  __device__ __forceinline__ double exec_g2c(double exec, double g2c) const {
    return eval<1u | 8u>(exec, 0.0, g2c, 0.0);
  }
  __device__ __forceinline__ double g2c_only(double g2c) const {
    return eval<8u>(0.0, 0.0, g2c, 0.0);
  }
};

struct Family {
  double layer, first, last, extra_pre, extra_post;
};

__device__ __forceinline__ Family pick_family(bool second, const Family &a, const Family &b) {
  Family r;
  r.layer = second ? b.layer : a.layer;
  r.first = second ? b.first : a.first;
  r.last = second ? b.last : a.last;
  r.extra_pre = second ? b.extra_pre : a.extra_pre;
  r.extra_post = second ? b.extra_post : a.extra_post;
  return r;
}

// Slot of stage `stage` of group `group_index` in the stage-summary workspace.  Groups lie back
// to back in the row workspace and need not start at a multiple of kStageRows; adding the group
// index keeps the slots of consecutive groups apart (at most rows / kStageRows + groups + 1 slots).
__device__ __forceinline__ int64_t stage_floor_slot(const MistGroupDesc *g, int group_index,
                                                    int64_t stage) {
  return g->row_offset / kStageRows + group_index + stage;
}

__device__ __forceinline__ const MistGroupDesc *find_group(const MistGroupDesc *groups,
                                                           const int32_t *prefix, int n_groups,
                                                           int block, int *local) {
  int lo = 0, hi = n_groups;  // prefix[lo] <= block < prefix[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (prefix[mid] <= block) lo = mid; else hi = mid;
  }
  *local = block - prefix[lo];
  return groups + lo;
}

// Workspace order.  The reference numbers a group's rows parallelism-major with the activation
// offload ratio fastest (batched_module_analyzer.py:490-534); the workspace holds them per
// (parallelism row, activation ratio) in tiles of kOoTile optimizer ratios, and inside a tile
// pair by pair:
//   position = (par * n_ao + ao) * n_oo * n_pair + tile * kOoTile * n_pair + pair * width + oo % kOoTile
// with tile = oo / kOoTile and width = ratios in that tile (kOoTile, fewer in the last one).  A
// stage of the reduce kernel (64 consecutive positions) then covers 16 neighbouring (weight,
// gradient) pairs at 4 neighbouring optimizer ratios: rows of similar latency AND footprint, so
// the stage's term-wise minimum is close to a real row and its bounds prune.  (With all pairs of
// one optimizer ratio in a run, a stage spanned half of the pair list: its minimum was as fast as
// the rows without offloading and as small as those with all of it.)  Results carry row numbers.
constexpr int kOoTile = 4;

struct RowParts {
  int par, pair, oo, ao;
};

// Position inside the (par, ao) block of n_oo * n_pair rows.
__device__ __forceinline__ int tile_position(const MistGroupDesc *g, int oo, int pair) {
  const int tile = oo / kOoTile;
  const int width = min(kOoTile, g->n_oo - tile * kOoTile);
  return tile * kOoTile * g->n_pair + pair * width + (oo - tile * kOoTile);
}

__device__ __forceinline__ RowParts parts_of_position(const MistGroupDesc *g, int64_t pos) {
  RowParts r;
  r.par = (int)(pos / g->n_off);
  int rem = (int)(pos % g->n_off);
  const int per_ao = g->n_oo * g->n_pair;
  r.ao = rem / per_ao;
  rem -= r.ao * per_ao;
  const int tile = rem / (kOoTile * g->n_pair);
  rem -= tile * kOoTile * g->n_pair;
  const int width = min(kOoTile, g->n_oo - tile * kOoTile);
  r.pair = rem / width;
  r.oo = tile * kOoTile + (rem - r.pair * width);
  return r;
}

__device__ __forceinline__ int32_t row_of_position(const MistGroupDesc *g, int64_t pos) {
  const RowParts r = parts_of_position(g, pos);
  return (int32_t)((int64_t)r.par * g->n_off + (r.pair * g->n_oo + r.oo) * g->n_ao + r.ao);
}

__device__ __forceinline__ int64_t position_of_row(const MistGroupDesc *g, int64_t row) {
  const int par = (int)(row / g->n_off);
  const int off = (int)(row % g->n_off);
  const int n_tail = g->n_oo * g->n_ao;
  const int pair = off / n_tail;
  const int oo = (off / g->n_ao) % g->n_oo;
  const int ao = off % g->n_ao;
  return (int64_t)par * g->n_off + (int64_t)ao * g->n_oo * g->n_pair + tile_position(g, oo, pair);
}

// ------------------------------------------------------------------------------------------
// Kernel 1: row-invariant terms.  One thread per candidate row (workspace position).
// ------------------------------------------------------------------------------------------
// Of a row's 36 evaluations of the interference model only the eight of the forward phase of the
// first micro-batch see the optimizer ratio (through the optimizer-state swaps); the other 28
// are the same for the n_oo rows of one "key" = (parallelism, activation ratio, offload pair).
// key_terms_kernel evaluates those once per key into MIST_KEY_TERMS doubles, row_terms_kernel
// reads them: the same operations on the same operands as when every row evaluates everything
// (which it does when the caller passes no key-term workspace, and for the rows of the scout
// pass, which are computed ahead of all others).
constexpr int kKeyBwd = 0;        // [last?0:1 micro-batch][nock, ck] x (layer, first, last, extra_pre, extra_post)
constexpr int kKeyFwd = 20;       // forward, not the first micro-batch: [nock, ck] x (layer, last, extra_post)
constexpr int kKeyFwdFirst = 26;  //   its `first` and `extra_pre`, which do not depend on ckpt
constexpr int kKeyFwdExtraPre = 27;
static_assert(MIST_KEY_TERMS == 28 && MIST_KEY_TERMS % 2 == 0, "key terms are read as 16-byte pairs");

// Model tables of a workgroup in LDS (tables indexed at run time: indexing the by-value kernel
// argument would make every lane keep a private copy of the whole struct in scratch memory).
// Returns whether every interference factor is in the divisor range of the reciprocal quotient.
__device__ __forceinline__ bool load_model_tables(const MistProblem &prob,
                                                  double (*lds_factor)[kFactorPitch],
                                                  double *lds_gpu_gpu) {
  bool factors_tame = true;
  if (threadIdx.x < 44) {
    const double f = prob.interf_factor[threadIdx.x / 4][threadIdx.x % 4];
    lds_factor[threadIdx.x / 4][threadIdx.x % 4] = f;
    lds_factor[threadIdx.x / 4][4 + threadIdx.x % 4] = 1.0 / f;
    factors_tame = f >= mist_arith::kDivisorMin && f <= mist_arith::kDivisorMax;
  }
  if (threadIdx.x >= 64 && threadIdx.x < 96) lds_gpu_gpu[threadIdx.x - 64] = prob.gpu_gpu[threadIdx.x - 64];
  return __syncthreads_and(factors_tame) != 0;
}

// Operands of the interference evaluations that do not depend on the optimizer ratio: swap and
// collective latencies (:1362-1408) of one (parallelism row, offload pair, activation ratio).
struct KeyInputs {
  double exec_fwd, exec_bwd_nock, exec_bwd_ck, extra_fwd, extra_bwd, extra_fb;
  double wre, gre, ore;
  double so_W, si_W, so_G, si_G, so_A_ck, si_A_ck, so_A_nock, si_A_nock;
  double AG_w, RS_g, AR_g;
  double E_f, ag_wre, g2c_B, c2g_B, first_g2c, g2g_B[2];
};

__device__ __forceinline__ KeyInputs key_inputs(const MistProblem &prob, const double *lds_gpu_gpu,
                                                const MistGroupDesc *g, const double *par,
                                                double wo, double go, double ao) {
  KeyInputs in;
  const double dp = par[MIST_PAR_DP];
  in.wre = par[MIST_PAR_WRE];
  in.gre = par[MIST_PAR_GRE];
  in.ore = par[MIST_PAR_ORE];
  const double W = par[MIST_PAR_W], Gr = par[MIST_PAR_G];
  const double raw_ck = par[MIST_PAR_RAW_CK], raw_nock = par[MIST_PAR_RAW_NOCK];
  in.exec_fwd = par[MIST_PAR_EXEC_FWD];
  in.exec_bwd_nock = par[MIST_PAR_EXEC_BWD];
  in.extra_fwd = par[MIST_PAR_EXTRA_FWD];
  in.extra_bwd = par[MIST_PAR_EXTRA_BWD];
  const double wre_size = in.wre == 1.0 ? dp : 1.0;
  const double gre_size = in.gre == 1.0 ? dp : 1.0;
  in.so_W = host_link_latency(prob.gpu_cpu, W / wre_size * wo);
  in.si_W = host_link_latency(prob.cpu_gpu, W / wre_size * wo);
  in.so_G = host_link_latency(prob.gpu_cpu, Gr / gre_size * go);
  in.si_G = host_link_latency(prob.cpu_gpu, Gr / gre_size * go);
  in.so_A_ck = host_link_latency(prob.gpu_cpu, raw_ck * ao);
  in.si_A_ck = host_link_latency(prob.cpu_gpu, raw_ck * ao);
  in.so_A_nock = host_link_latency(prob.gpu_cpu, raw_nock * ao);
  in.si_A_nock = host_link_latency(prob.cpu_gpu, raw_nock * ao);
  const double n_nodes = (double)g->num_nodes;
  const double dp_inter = dp > n_nodes ? n_nodes : dp;
  const double dp_intra = dp > n_nodes ? floor(dp / n_nodes) : 1.0;
  in.AG_w = gpu_gpu_latency(lds_gpu_gpu, W, dp_inter, dp_intra, 1.0);
  in.RS_g = gpu_gpu_latency(lds_gpu_gpu, Gr, dp_inter, dp_intra, 1.1);
  in.AR_g = gpu_gpu_latency(lds_gpu_gpu, Gr, dp_inter, dp_intra, 2.1);
  const bool adv = prob.adv_first_block != 0;
  in.E_f = in.exec_fwd - in.extra_fwd;
  in.ag_wre = in.AG_w * in.wre;
  in.g2c_B = in.so_G;
  in.c2g_B = in.si_W + in.si_G;
  in.first_g2c = adv ? in.g2c_B : 0.0;
  in.g2g_B[0] = in.ag_wre + in.RS_g * in.ore + in.AR_g * (1.0 - in.ore);
  in.g2g_B[1] = in.ag_wre + in.RS_g * in.gre;
  in.extra_fb = in.extra_fwd + in.extra_bwd;
  in.exec_bwd_ck = in.exec_fwd + in.exec_bwd_nock;
  return in;
}

// Forward phases (:1432-1621): phase 0 = first micro-batch (the optimizer-state swaps so_O /
// si_O run beside it), phase 1 = the others.
struct FwdOperands {
  double g2c, c2g, g2g;
};
__device__ __forceinline__ FwdOperands fwd_operands(const KeyInputs &in, bool first_micro_batch,
                                                    double so_O, double si_O) {
  if (first_micro_batch) return FwdOperands{so_O + in.so_W, si_O + in.si_G, in.AG_w * in.ore};
  return FwdOperands{0.0, in.si_W, in.AG_w * in.wre};
}
// the members of a forward family that do not depend on ckpt ...
template <class Interference>
__device__ __forceinline__ void fwd_common(const Interference &I, const KeyInputs &in,
                                           const FwdOperands &op, bool first_micro_batch, bool adv,
                                           double &first, double &extra_pre) {
  const double pre_g2g = (first_micro_batch || adv) ? op.g2g : 0.0;
  const double pre_c2g = adv ? op.c2g : 0.0;
  first = I.exec_g2g_c2g(in.E_f, op.g2g, op.c2g) + in.extra_fwd;
  extra_pre = I.g2g_c2g(pre_g2g, pre_c2g);
}
// ... and those that do (with_ckpt: the saved activations of a checkpointed layer are swapped)
template <class Interference>
__device__ __forceinline__ void fwd_of_ckpt(const Interference &I, const KeyInputs &in,
                                            const FwdOperands &op, bool with_ckpt, double &layer,
                                            double &last, double &extra_post) {
  const double g2c = op.g2c + (with_ckpt ? in.so_A_ck : in.so_A_nock);
  layer = I(in.E_f, op.g2g, g2c, op.c2g) + in.extra_fwd;
  last = I.exec_g2c(in.E_f, g2c) + in.extra_fwd;
  extra_post = I.g2c_only(g2c);
}

// Backward phases (:1646-1902): not_last = false for the last micro-batch.
template <class Interference>
__device__ __forceinline__ Family bwd_family(const Interference &I, const KeyInputs &in,
                                             bool not_last, bool with_ckpt) {
  const bool k = with_ckpt;
  const double E = k ? in.exec_bwd_ck - in.extra_fb : in.exec_bwd_nock - in.extra_bwd;
  const double extra = k ? in.extra_fb : in.extra_bwd;
  const double c2g = in.c2g_B + (k ? in.si_A_ck : in.si_A_nock);
  const double red_last =
      k ? (in.ore == 1.0 ? in.RS_g : in.AR_g) : in.RS_g * in.ore + in.AR_g * (1.0 - in.ore);
  const double red = not_last ? in.RS_g * in.gre : red_last;
  // With checkpointing the reference adds the (always zero) all-gather of saved tensors.
  const double g2g_phase = not_last ? in.g2g_B[1] : in.g2g_B[0];
  const double g2g_layer = k ? g2g_phase + 0.0 : g2g_phase;
  Family f;
  f.layer = I(E, g2g_layer, in.g2c_B, c2g) + extra;
  f.last = I.exec_g2g_c2g(E, in.ag_wre, c2g) + extra;
  f.first = I.exec_g2g_g2c(E, red, in.first_g2c) + extra;
  f.extra_pre = I.g2g_c2g(in.ag_wre, c2g);
  f.extra_post = I.g2g_g2c(red, in.first_g2c);
  return f;
}

// Workgroup = (32 keys of one group) x (4 lanes per key); grid.y = group, grid.x covers the
// group with the most keys.  Lane j of a key evaluates backward family j (= 2 * not_last + ckpt)
// and the forward family of the later micro-batches with ckpt = j & 1.
__global__ __launch_bounds__(kTermsBlock) void key_terms_kernel(
    const MistProblem prob, const MistGroupDesc *__restrict__ groups, double *__restrict__ key_terms) {
  const MistGroupDesc *g = groups + blockIdx.y;
  const int n_keys = g->n_par * g->n_ao * g->n_pair;
  constexpr int kKeysPerBlock = kTermsBlock / 4;
  if ((int)blockIdx.x * kKeysPerBlock >= n_keys) return;
  __shared__ __align__(16) double lds_factor[11][kFactorPitch];
  __shared__ double lds_gpu_gpu[32];
  InterferenceModel<false> I;
  I.factors_tame = load_model_tables(prob, lds_factor, lds_gpu_gpu);
  I.table = (LdsDouble *)&lds_factor[0][0];
  const int key_here = (int)blockIdx.x * kKeysPerBlock + (int)threadIdx.x / 4;
  const int key = min(key_here, n_keys - 1);  // lanes past the end redo the last key, unwritten
  const int j = threadIdx.x & 3;
  const int pair = key % g->n_pair;
  const int ao_i = (key / g->n_pair) % g->n_ao;
  const int par_i = key / (g->n_pair * g->n_ao);
  const KeyInputs in = key_inputs(prob, lds_gpu_gpu, g, g->par[par_i], g->wo[g->pair_wo[pair]],
                                  g->go[g->pair_go[pair]], g->ao[ao_i]);
  const Family back = bwd_family(I, in, (j & 2) != 0, (j & 1) != 0);
  const FwdOperands op = fwd_operands(in, false, 0.0, 0.0);
  double first, extra_pre, layer, last, extra_post;
  fwd_common(I, in, op, false, prob.adv_first_block != 0, first, extra_pre);
  fwd_of_ckpt(I, in, op, (j & 1) != 0, layer, last, extra_post);
  if (key_here >= n_keys) return;
  double *out = key_terms + (g->key_offset + key) * MIST_KEY_TERMS;
  double *b = out + kKeyBwd + j * 5;
  b[0] = back.layer;
  b[1] = back.first;
  b[2] = back.last;
  b[3] = back.extra_pre;
  b[4] = back.extra_post;
  if (j < 2) {
    double *f = out + kKeyFwd + j * 3;
    f[0] = layer;
    f[1] = last;
    f[2] = extra_post;
  }
  if (j == 0) {
    out[kKeyFwdFirst] = first;
    out[kKeyFwdExtraPre] = extra_pre;
  }
}

// kMode 0: every row of every group.  kMode 1: only the rows the scout pass gathers (workgroup
// = (128 gathered rows, group); no stage summaries), so that the scout pass can start while
// kMode 2 computes everything: that one leaves the stores of the gathered rows out (the scout
// pass may be reading them) and is otherwise kMode 0.  kFromKeys: the key terms are read from
// `key_terms` (written by key_terms_kernel) instead of evaluated per row.
__device__ __forceinline__ int64_t gathered_position(const MistGroupDesc *g, int64_t q);
__device__ __forceinline__ bool is_scout_pair(const MistGroupDesc *g, int pair) {
  for (int k = 0; k < g->scout_stride; ++k)
    if (pair == g->scout_pair[k]) return true;
  return false;
}

template <int kMode, bool kFromKeys>
__global__ __launch_bounds__(kTermsBlock) void row_terms_kernel(
    const MistProblem prob, const MistGroupDesc *__restrict__ groups, int n_groups,
    const int32_t *__restrict__ block_prefix, double *__restrict__ row_terms,
    double *__restrict__ stage_floor, const double *__restrict__ key_terms) {
  int local_block;
  const MistGroupDesc *g;
  int64_t n_here_total;  // rows this launch computes for the group
  if (kMode == 1) {
    g = groups + blockIdx.y;
    local_block = blockIdx.x;
    n_here_total = g->scout_stride > 0 ? (int64_t)g->n_par * g->n_oo * g->n_ao * g->scout_stride : 0;
    if ((int64_t)local_block * kTermsBlock >= n_here_total) return;
  } else {
    g = find_group(groups, block_prefix, n_groups, blockIdx.x, &local_block);
    n_here_total = g->n_rows;
  }
  // The block's terms are written out as one contiguous, fully coalesced range (a lane writing
  // its own 272-byte row would touch 34 partial cache lines): wavefront by wavefront through one
  // LDS buffer of kStageRows rows (row pitch 35 doubles: conflict-free).  One buffer for the
  // block, not one per wavefront: LDS is what bounds the number of resident wavefronts here, and
  // the kernel is a chain of dependent loads and evaluations that needs them.
  __shared__ double lds_out[kStageRows * (MIST_ROW_TERMS + 1)];
  __shared__ __align__(16) double lds_factor[11][kFactorPitch];
  __shared__ double lds_gpu_gpu[32];
  __shared__ unsigned char lds_skip[kTermsBlock];
  __shared__ double lds_part[kTermsBlock / kStageRows - 1][2][kStageFloorPitch];  // stage summaries
  InterferenceModel<kFromKeys> I;  // with key terms only the first forward phase is evaluated here
  I.factors_tame = load_model_tables(prob, lds_factor, lds_gpu_gpu);
  I.table = (LdsDouble *)&lds_factor[0][0];
  const int64_t block_first = (int64_t)local_block * kTermsBlock;
  const int rows_here = (int)min((int64_t)kTermsBlock, n_here_total - block_first);
  // Lanes past the end recompute the last row (no divergent barrier); their result is dropped.
  const int64_t nth = block_first + min((int)threadIdx.x, rows_here - 1);
  const int64_t row = kMode == 1 ? gathered_position(g, nth) : nth;  // workspace position

  // ---- index decomposition (batched_module_analyzer.py:490-534) ----
  const RowParts parts = parts_of_position(g, row);
  const int par_i = parts.par, pair = parts.pair, oo_i = parts.oo, ao_i = parts.ao;
  const double wo = g->wo[g->pair_wo[pair]];
  const double go = g->go[g->pair_go[pair]];
  const double oo = g->oo[oo_i];
  const double ao = g->ao[ao_i];

  // the key terms are fetched first and used last: the loads are in flight across everything
  // computed here
  double v[kFromKeys ? MIST_KEY_TERMS : 2];
  if (kFromKeys) {
    const int64_t key = (int64_t)(par_i * g->n_ao + ao_i) * g->n_pair + pair;
    const double2 *__restrict__ kt =
        reinterpret_cast<const double2 *>(key_terms + (g->key_offset + key) * MIST_KEY_TERMS);
#pragma unroll
    for (int i = 0; i < MIST_KEY_TERMS / 2; ++i) {
      const double2 two = kt[i];
      v[2 * i] = two.x;
      v[2 * i + 1] = two.y;
    }
  }

  const double *par = g->par[par_i];
  const double b = par[MIST_PAR_B], dp = par[MIST_PAR_DP], tp = par[MIST_PAR_TP];
  const double wre = par[MIST_PAR_WRE], gre = par[MIST_PAR_GRE], ore = par[MIST_PAR_ORE];
  const double W = par[MIST_PAR_W], Gr = par[MIST_PAR_G], O = par[MIST_PAR_O];
  const double raw_ck = par[MIST_PAR_RAW_CK], raw_nock = par[MIST_PAR_RAW_NOCK];
  const double wre_size = wre == 1.0 ? dp : 1.0;
  const double gre_size = gre == 1.0 ? dp : 1.0;
  const double ore_size = ore == 1.0 ? dp : 1.0;

  // ---- memory factor (:1181-1199) ----
  double mf = 1.0;
  mf += prob.frag_factor;
  mf += wo > 0.0 ? 0.025 : 0.0;
  mf += go > 0.0 ? 0.025 : 0.0;
  mf += oo > 0.0 ? 0.03 : 0.0;
  mf += ao > 0.0 ? 0.04 : 0.0;
  mf += wre != 0.0 ? 0.025 : 0.0;
  mf += gre != 0.0 ? 0.025 : 0.0;
  mf += tp > 1.0 ? 0.04 : 0.0;
  mf += b >= 4.0 ? 0.01 : 0.0;
  const double mf_pp = mf + 0.025;

  // ---- memory pieces (:1216-1272, 2091-2162) ----
  const double pW = W / wre_size * (1.0 - wo);
  const double pG = Gr / gre_size * (1.0 - go);
  const double pO = O / ore_size * (1.0 - oo);
  const double S_ck = raw_ck * (1.0 - ao), D_ck = raw_ck * ao;
  const double S_nock = raw_nock * (1.0 - ao), D_nock = raw_nock * ao;
  const bool wbuf_on = wre_size > 1.0 || g->pp_wre == 1 || wo > 0.0;
  const bool gbuf_on = gre_size > 1.0 || g->pp_gre == 1 || go > 0.0;
  const double Wbuf = wbuf_on ? fmax(fmax(g->pre_full_w, g->post_full_w), W) : 0.0;
  const double Gbuf = gbuf_on ? fmax(fmax(g->pre_full_g, g->post_full_g), Gr) : 0.0;
  const double two_buf = 2.0 * (Wbuf + Gbuf);

  // ---- swap and collective latencies (:1362-1408) ----
  const KeyInputs in = key_inputs(prob, lds_gpu_gpu, g, par, wo, go, ao);
  const double so_O = host_link_latency(prob.gpu_cpu, O / ore_size * oo);
  const double si_O = host_link_latency(prob.cpu_gpu, O / ore_size * oo);
  const bool adv = prob.adv_first_block != 0;

  // ---- forward (:1432-1621) and backward (:1646-1902) families ----
  Family fwd[2][2];  // [0 = first micro-batch, 1 = not first][0 = nock, 1 = ck]
  Family bwd[2][2];  // [0 = last micro-batch, 1 = not last][0 = nock, 1 = ck]
  {
    const FwdOperands op = fwd_operands(in, true, so_O, si_O);
    double first, extra_pre;
    fwd_common(I, in, op, true, adv, first, extra_pre);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      fwd[0][k].first = first;
      fwd[0][k].extra_pre = extra_pre;
      fwd_of_ckpt(I, in, op, k != 0, fwd[0][k].layer, fwd[0][k].last, fwd[0][k].extra_post);
    }
  }
  if (kFromKeys) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const double *f = v + kKeyBwd + j * 5;
      bwd[j >> 1][j & 1] = Family{f[0], f[1], f[2], f[3], f[4]};
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const double *f = v + kKeyFwd + k * 3;
      fwd[1][k] = Family{f[0], v[kKeyFwdFirst], f[1], v[kKeyFwdExtraPre], f[2]};
    }
  } else {
    const FwdOperands op = fwd_operands(in, false, 0.0, 0.0);
    double first, extra_pre;
    fwd_common(I, in, op, false, adv, first, extra_pre);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      fwd[1][k].first = first;
      fwd[1][k].extra_pre = extra_pre;
      fwd_of_ckpt(I, in, op, k != 0, fwd[1][k].layer, fwd[1][k].last, fwd[1][k].extra_post);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) bwd[j >> 1][j & 1] = bwd_family(I, in, (j & 2) != 0, (j & 1) != 0);
  }

  // ---- stable / delta families (:1910-2028) ----
  double t[MIST_ROW_TERMS];  // compile-time indices only: registers
  const int st = g->grad_accum == 1 ? 0 : 1;  // phase index that forms the stable part
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    // selected field by field: indexing the arrays with a run-time phase would put them in
    // scratch memory
    const Family f = pick_family(st == 1, fwd[0][k], fwd[1][k]);
    const Family w = pick_family(st == 1, bwd[0][k], bwd[1][k]);
    const double s_layer = f.layer + w.layer;
    const double s_first = f.extra_pre + w.extra_post + f.first + w.first;
    const double s_last = f.extra_post + w.extra_pre + f.last + w.last;
    double d_layer = 0.0, d_first = 0.0, d_last = 0.0;
    if (st == 1) {
      const Family &f1 = fwd[0][k], &w1 = bwd[0][k];
      d_layer = f1.layer + w1.layer - s_layer;
      d_first = f1.extra_pre + w1.extra_post + f1.first + w1.first - s_first;
      d_last = f1.extra_post + w1.extra_pre + f1.last + w1.last - s_last;
    }
    // k == 1 is "with ckpt": the *_CK slot precedes the *_NOCK slot.
    t[MIST_T_S_LAYER_CK + (1 - k)] = s_layer;
    t[MIST_T_S_FIRST_CK + (1 - k)] = s_first;
    t[MIST_T_S_LAST_CK + (1 - k)] = s_last;
    t[MIST_T_D_LAYER_CK + (1 - k)] = d_layer;
    t[MIST_T_D_FIRST_CK + (1 - k)] = d_first;
    t[MIST_T_D_LAST_CK + (1 - k)] = d_last;
  }

  t[MIST_T_FWD_STATES0] = two_buf + np_floor_divide(O, ore_size);
  t[MIST_T_BWD_STATES0] = two_buf;
  t[MIST_T_PWG] = pW + pG;
  t[MIST_T_PO] = pO;
  t[MIST_T_PWGO] = pW + pG + pO;
  t[MIST_T_S_CK] = S_ck;
  t[MIST_T_S_NOCK] = S_nock;
  t[MIST_T_D_CK] = D_ck;
  t[MIST_T_D_NOCK] = D_nock;
  t[MIST_T_MF_BASE] = mf_pp + 0.01;
  t[MIST_T_MF_PP] = mf_pp;
  t[MIST_T_MF] = mf;
  t[MIST_T_FWD_PEAK] = par[MIST_PAR_FWD_PEAK];
  t[MIST_T_BWD_PEAK] = par[MIST_PAR_BWD_PEAK];
  t[MIST_T_OUT] = par[MIST_PAR_OUT];
  t[MIST_T_GCB] = par[MIST_PAR_GCB];

  // ---- post-layer overlap pieces (:2251-2292) ----
  const double ovw_ck = fmax(in.exec_fwd - 0.0 - in.so_A_ck, 0.0);
  const double ovw_nock = fmax(in.exec_fwd - 0.0 - in.so_A_nock, 0.0);
  t[MIST_T_NAG_CK] = fmax(g->post_ag - ovw_ck, 0.0);
  t[MIST_T_NAG_NOCK] = fmax(g->post_ag - ovw_nock, 0.0);
  const double ovg_ck = fmax(in.exec_bwd_ck - in.ag_wre - in.c2g_B - in.si_A_ck, 0.0);
  const double ovg_nock = fmax(in.exec_bwd_nock - in.ag_wre - in.c2g_B - in.si_A_nock, 0.0);
  t[MIST_T_NRS_CK] = fmax(g->post_rs - ovg_ck, 0.0);
  t[MIST_T_NRS_NOCK] = fmax(g->post_rs - ovg_nock, 0.0);
  t[MIST_T_OPB] = fmax(g->post_bwd - bwd[1][1].extra_pre, 0.0);
  t[MIST_T_RD] = raw_nock - S_nock;

  if (kMode == 1) {  // scattered rows: every lane writes its own
    if ((int)threadIdx.x < rows_here) {
      double2 *__restrict__ mine =
          reinterpret_cast<double2 *>(row_terms + (g->row_offset + row) * MIST_ROW_TERMS);
#pragma unroll
      for (int i = 0; i < MIST_ROW_TERMS / 2; ++i) mine[i] = make_double2(t[2 * i], t[2 * i + 1]);
    }
    return;
  }
  if (kMode == 2) lds_skip[threadIdx.x] = is_scout_pair(g, pair) ? 1 : 0;
  static_assert(kTermsBlock % kStageRows == 0 && kStageRows == 64, "a wavefront's rows are one stage");
  const int wave = threadIdx.x / kStageRows, lane = threadIdx.x % kStageRows;
  for (int stage_here = 0; stage_here < kTermsBlock / kStageRows; ++stage_here) {
    if (wave == stage_here) {
#pragma unroll
      for (int i = 0; i < MIST_ROW_TERMS; ++i) lds_out[lane * (MIST_ROW_TERMS + 1) + i] = t[i];
    }
    __syncthreads();
    const int stage_first = stage_here * kStageRows;
    const int stage_rows = min(kStageRows, rows_here - stage_first);  // <= 0: nothing left
    double2 *__restrict__ dst = reinterpret_cast<double2 *>(
        row_terms + (g->row_offset + block_first + stage_first) * MIST_ROW_TERMS);
    for (int i = threadIdx.x; i < stage_rows * (MIST_ROW_TERMS / 2); i += kTermsBlock) {
      const int r = i / (MIST_ROW_TERMS / 2);
      if (kMode == 2 && lds_skip[stage_first + r]) continue;  // written by the kMode 1 launch
      const int at = r * (MIST_ROW_TERMS + 1) + 2 * (i % (MIST_ROW_TERMS / 2));
      dst[i] = make_double2(lds_out[at], lds_out[at + 1]);
    }
    // Summary of the stage for the reduce kernel: thread = (column, one of kTermsBlock / 32
    // runs of the stage's rows); columns 0 .. MIST_T_GCB hold the minimum, column kStageMaxOut
    // the maximum of MIST_T_OUT, the three behind it minima of post-layer terms.  The runs of a wavefront meet by shuffle, the wavefronts in LDS.
    constexpr int kRuns = kTermsBlock / kStageFloorPitch, kRunRows = kStageRows / kRuns;
    const int col = threadIdx.x & (kStageFloorPitch - 1), run = threadIdx.x / kStageFloorPitch;
    const int src_col = col == kStageMaxOut ? MIST_T_OUT
                        : col == kStageMinOpb ? MIST_T_OPB
                        : col == kStageMinNag ? MIST_T_NAG_CK
                        : col == kStageMinNrs ? MIST_T_NRS_CK : col;
    const int second_col = (col == kStageMinNag || col == kStageMinNrs) ? src_col + 1 : src_col;
    double lo_v = INFINITY, hi_v = 0.0;
    {
#pragma unroll
      for (int i = 0; i < kRunRows; ++i) {
        const int r = run * kRunRows + i;
        const double *row_at = lds_out + min(r, kStageRows - 1) * (MIST_ROW_TERMS + 1);
        const double x = fmin(row_at[src_col], row_at[second_col]);
        lo_v = fmin(lo_v, r < stage_rows ? x : INFINITY);
        hi_v = fmax(hi_v, r < stage_rows ? x : 0.0);
      }
    }
    lo_v = fmin(lo_v, __shfl_xor(lo_v, kStageFloorPitch));
    hi_v = fmax(hi_v, __shfl_xor(hi_v, kStageFloorPitch));
    if (wave > 0 && lane < kStageFloorPitch) {
      lds_part[wave - 1][0][col] = lo_v;
      lds_part[wave - 1][1][col] = hi_v;
    }
    __syncthreads();  // every read of this stage is done; the other wavefronts' parts are in LDS
    if (wave == 0 && lane < kStageFloorPitch && stage_rows > 0) {
#pragma unroll
      for (int w = 0; w < kTermsBlock / kStageRows - 1; ++w) {
        lo_v = fmin(lo_v, lds_part[w][0][col]);
        hi_v = fmax(hi_v, lds_part[w][1][col]);
      }
      const int64_t slot = stage_floor_slot(g, (int)(g - groups), block_first / kStageRows + stage_here);
      stage_floor[slot * kStageFloorPitch + col] = col == kStageMaxOut ? hi_v : lo_v;
    }
  }
}

// ------------------------------------------------------------------------------------------
// Per-cell evaluation shared by the reduce and finalize kernels.
// ------------------------------------------------------------------------------------------
struct PairIndex {
  int l, c;  // layers in the stage (1..L), checkpointed layers (0..l)
};

// Valid (l, c <= l) pairs are numbered l-major: index(l, c) = l*(l+1)/2 - 1 + c.
__device__ __forceinline__ PairIndex decode_pair(int idx) {
  int l = (int)((sqrt(8.0 * (double)idx + 9.0) - 1.0) * 0.5);
  while (l * (l + 1) / 2 - 1 > idx) --l;
  while ((l + 1) * (l + 2) / 2 - 1 <= idx) ++l;
  return PairIndex{l, idx - (l * (l + 1) / 2 - 1)};
}

struct CellLatency {
  float x, d;           // stable, delta rounded to float32 (batched_module_analyzer.py:2212-2213)
  double sp, dpre;      // with_pre stable / delta (float64)
  double spost, dpost;  // with_post
  double spp, dpp;      // pre_and_post (no_pp)
};

struct GroupConsts {
  double pre_fwd, pre_bwd, post_fwd;
  double w1, w2, w1d, w2d;  // pre-layer all-gather / reduce-scatter split into stable / delta
  bool pp_wre, pp_gre;
};

__device__ __forceinline__ GroupConsts group_consts(const MistGroupDesc *g) {
  GroupConsts k;
  k.pre_fwd = g->pre_fwd;
  k.pre_bwd = g->pre_bwd;
  k.post_fwd = g->post_fwd;
  k.pp_wre = g->pp_wre == 1;
  k.pp_gre = g->pp_gre == 1;
  k.w1 = k.pp_wre ? g->pre_ag : 0.0;
  k.w2 = k.pp_gre ? g->pre_rs : 0.0;
  k.w1d = k.pp_wre ? 0.0 : g->pre_ag;
  k.w2d = k.pp_gre ? 0.0 : g->pre_rs;
  return k;
}

// get_latencies (:2165-2216) and the pre / post additions (:2233-2351) for one row and (l, c).
template <bool kWithPost>
__device__ __forceinline__ CellLatency cell_latency(const double *__restrict__ t, int l, int c,
                                                    const GroupConsts &k) {
  const int lm2 = max(l - 2, 0);
  const int n_ck = min(max(c - 1, 0), lm2);
  const int n_nock = lm2 - n_ck;
  const bool all_ck = c == l, no_ck = c == 0;
  const double stable = (double)n_ck * t[MIST_T_S_LAYER_CK] + (double)n_nock * t[MIST_T_S_LAYER_NOCK] +
                        (all_ck ? t[MIST_T_S_FIRST_CK] : t[MIST_T_S_FIRST_NOCK]) +
                        (no_ck ? t[MIST_T_S_LAST_NOCK] : t[MIST_T_S_LAST_CK]);
  const double delta = (double)n_ck * t[MIST_T_D_LAYER_CK] + (double)n_nock * t[MIST_T_D_LAYER_NOCK] +
                       (all_ck ? t[MIST_T_D_FIRST_CK] : t[MIST_T_D_FIRST_NOCK]) +
                       (no_ck ? t[MIST_T_D_LAST_NOCK] : t[MIST_T_D_LAST_CK]);
  CellLatency r;
  r.x = (float)stable;
  r.d = (float)delta;
  const double x = (double)r.x, d = (double)r.d;
  r.sp = x + k.pre_fwd + k.pre_bwd + k.w1 + k.w2;
  r.dpre = d + k.w1d + k.w2d;
  if (kWithPost) {
    const double nag = c > 0 ? t[MIST_T_NAG_CK] : t[MIST_T_NAG_NOCK];
    const double nrs = c > 0 ? t[MIST_T_NRS_CK] : t[MIST_T_NRS_NOCK];
    const double ps1 = k.pp_wre ? nag : 0.0, ps2 = k.pp_gre ? nrs : 0.0;
    const double pd1 = k.pp_wre ? 0.0 : nag, pd2 = k.pp_gre ? 0.0 : nrs;
    const double opb = t[MIST_T_OPB];
    r.spost = x + k.post_fwd + opb + ps1 + ps2;
    r.dpost = d + pd1 + pd2;
    r.spp = x + k.pre_fwd + k.pre_bwd + k.post_fwd + opb + k.w1 + k.w2 + ps1 + ps2;
    r.dpp = d + k.w1d + k.w2d + pd1 + pd2;
  } else {
    r.spost = r.dpost = r.spp = r.dpp = 0.0;
  }
  return r;
}

// Lexicographic (cost, row) minimum.  The reference scans rows in ascending order with a strict
// "<" (mist/utils/pareto.py:134-142), i.e. it keeps the lowest row among those with the
// smallest cost; comparing (cost, row) pairs gives the same winner in any processing order.
__device__ __forceinline__ bool lex_less(double cost, int32_t row, double best, int32_t best_row) {
  return cost < best || (cost == best && row < best_row);
}

__device__ __forceinline__ void take_min(double &best, int32_t &best_row, bool feasible,
                                         double cost, int32_t row) {
  const bool better = feasible && lex_less(cost, row, best, best_row);
  best = better ? cost : best;
  best_row = better ? row : best_row;
}

// ------------------------------------------------------------------------------------------
// Kernel 2: evaluate + mask + running argmin.
// Workgroup = one wavefront = one tile of 64 (l, c) pairs; it streams candidate rows through LDS
// and each lane keeps the minima of MIST_P_TILE pre-saved micro-batch values for its own
// (l, c).  No cross-lane reduction is needed: the reduction axis (rows) is the loop.
//
// Memory feasibility is monotone in p: the peaks are built from p * (non-negative) terms by
// additions only, every floating-point add / multiply is monotone in each operand, and the
// host rejects negative table values.  So per (row, l, c) the feasible p form a prefix
// [0, count) and `count` is found by bisection with the exact peak formula at the probed p
// (no closed-form shortcut: the comparison that decides is the reference's own expression).
// The minima of a thread are therefore non-decreasing in p, and a row changes a slot iff it is
// feasible at the lowest slot whose minimum it beats.
//
// Almost no row changes anything, so a stage of kStageRows rows goes through three sieves, each
// keeping a per-lane bit mask of surviving rows so that a lane only pays for its own survivors
// (a wave executes a sieve as often as its busiest lane, not once per row):
//   A  objective value against the minimum of the highest slot the stage can reach (a bound
//      from the term-wise minimum of the stage's memory terms); evaluated transposed, a lane
//      holding one ROW and the loop running over the tile's pairs;
//   B  lowest improvable slot and the exact memory test at that slot (minima as of stage start:
//      they only decrease afterwards, so nothing that could matter later is dropped);
//   C  survivors in row order against the live minima: bisection for `count`, update.
// A scout pass runs the same code over a few gathered rows of a whole group first (those of the
// group's scout offload pairs, see gathered_position); the
// main pass starts every chunk from the scout's minima (real rows of the same group, hence valid
// upper bounds), which removes the warm-up in which a fresh chunk lets most rows through.
// ------------------------------------------------------------------------------------------
// kPow2G: the group's G is a power of two, so x / G == x * (1 / G) bit for bit (float32 and
// float64) and the division leaves the inner loop; other G divide.  kFirstTile: this workgroup
// owns p = 0 and therefore also the last-stage and single-stage variants.
#ifndef MIST_REDUCE_MIN_WAVES
#define MIST_REDUCE_MIN_WAVES 2
#endif
#ifndef MIST_SCOUT_SPLIT
#define MIST_SCOUT_SPLIT 4
#endif
constexpr int kScoutSplit = MIST_SCOUT_SPLIT;  // scout workgroups per (group, (l, c) tile, p tile)
constexpr int32_t kSlabUnchanged = -2;  // first row index of a slab that was not written (rows are >= -1)
constexpr int kPairFields = 4;  // per-pair table of sieve A: thr_b, thr_o, n_ck, n_nock
constexpr int kLdsRowStride = MIST_ROW_TERMS + 1;  // odd number of doubles: lanes reading the
                                                   // same term of different rows hit different banks
static_assert(kStageRows == 64, "the sieve masks are 64-bit");
static_assert(MIST_ROW_TERMS % 2 == 0, "rows are staged as 16-byte pairs");
static_assert(MIST_LC_TILE == 64, "one wavefront per workgroup: the stage minima use wave shuffles");
static_assert(MIST_T_S_LAYER_CK == 0 && MIST_T_GCB < 32,
              "latency and memory terms must be the first columns: one lane per term in the stage minima");

struct LaneMemory {
  double fwd_states, bwd_states, cur_saved, mod_saved, ck_delta, fwd_pk, bwd_pk, out, gcb;
  double mf_base, mf_pp;

  // Peaks of the middle-stage variant for p pre-saved micro-batches (:2755-2786).
  __device__ __forceinline__ void peaks(int p, double &peak_f, double &peak_b) const {
    peaks_at((double)p, peak_f, peak_b);
  }
  __device__ __forceinline__ void peaks_at(double pf64, double &peak_f, double &peak_b) const {
    const double pipe_saved = pf64 * mod_saved + cur_saved;
    const double outp2 = out * pf64 * 2.0;
    const double out2 = out * 2.0;
    peak_f = fwd_states + pipe_saved + ck_delta + fwd_pk + outp2 + gcb;
    peak_b = bwd_states + pipe_saved + ck_delta + bwd_pk + outp2 + out2 + gcb;
  }
  // Left-hand sides of the reference's memory tests; a candidate is feasible iff <= capacity.
  __device__ __forceinline__ double scaled_base(int p) const {  // (:2805-2812)
    double pf, pb;
    peaks(p, pf, pb);
    return fmax(pf, pb) * mf_base;
  }
  __device__ __forceinline__ double scaled_pre(int p, double pre_saved,
                                               double pre_sas) const {  // (:2866-2875, 2893-2897)
    double pf, pb;
    peaks(p, pf, pb);
    const double pre_p = (double)p * pre_saved;
    return fmax(pre_p + pf + pre_sas, pre_p + pb + pre_sas) * mf_pp;
  }
  __device__ __forceinline__ bool feasible_base(int p, double cap) const {
    return scaled_base(p) <= cap;
  }
  __device__ __forceinline__ bool feasible_pre(int p, double cap, double pre_saved,
                                               double pre_sas) const {
    return scaled_pre(p, pre_saved, pre_sas) <= cap;
  }
};

// Distinct layer counts of one (l, c) tile up to which sieve A also drops rows by memory.
constexpr int kTileLayerCounts = 12;

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Logical workgroups
// that stream the same rows are consecutive, so runs of kXcdRun logical workgroups are given to
// one XCD (and the runs round-robin, which keeps the XCDs evenly loaded).  The grid is padded to
// a multiple of kNumXcd * kXcdRun; logical indices past the end do nothing.
constexpr int kNumXcd = 8;
constexpr int kXcdRun = 16;
__device__ __forceinline__ int xcd_run_block(int physical) {
  const int xcd = physical % kNumXcd, slot = physical / kNumXcd;
  return ((slot / kXcdRun) * kNumXcd + xcd) * kXcdRun + slot % kXcdRun;
}
__host__ __device__ constexpr int xcd_padded_grid(int n_blocks) {
  return (n_blocks + kNumXcd * kXcdRun - 1) / (kNumXcd * kXcdRun) * (kNumXcd * kXcdRun);
}

__device__ __forceinline__ LaneMemory cell_memory(const double *__restrict__ t, int l, int c);

struct ReduceRange {
  int64_t row_begin, row_end;  // rows of the group this workgroup covers (multiples of kStageRows)
  int stage_step;              // visit every stage_step-th stage of the range
  int skip_stride;             // > 0: skip stages whose index is a multiple (the scout did them)
  int gathered;                // != 0 (scout pass): "stage" t is not a run of consecutive rows but
                               // the rows number 64 t .. 64 t + 63 of the group's rows without
                               // weight / gradient offloading, see gathered_position()
};

// The search's winners sit almost exclusively on rows whose (weight, gradient) offload pair is
// the first one, (0, 0): 99.8 % of all cells of the GPT-7B plan, 95 % for LLaMA-13B.  In the
// workspace order those rows are scattered (one per (parallelism row, activation ratio, optimizer
// ratio)); the scout pass gathers them, n_par * n_oo * n_ao rows per group,
// and so seeds every chunk with minima that are final for most cells.
// With scout_stride = m > 1 the rows of the pairs scout_pair[1 .. m-1] follow.
__device__ __forceinline__ int64_t gathered_position(const MistGroupDesc *g, int64_t q) {
  const int n_tail = g->n_oo * g->n_ao;
  const int64_t per_pair = (int64_t)g->n_par * n_tail;
  const int64_t k = q / per_pair, rest = q - k * per_pair;
  const int64_t par = rest / n_tail, tail = rest - par * n_tail;
  const int64_t pair = g->scout_pair[k];
  const int ao = (int)(tail / g->n_oo), oo = (int)(tail - (int64_t)ao * g->n_oo);
  return par * g->n_off + (int64_t)ao * g->n_oo * g->n_pair + tile_position(g, oo, (int)pair);
}

// alpha / (1 - alpha) of the samples of one launch (by value in the kernel arguments)
struct RatioList {
  double r[MIST_MAX_SAMPLE_BATCH];
};
// sample position in the output tables of each sample of one finalize launch
struct SampleSlots {
  int32_t at[MIST_MAX_SAMPLE_BATCH];
};

template <bool kPow2G, bool kFirstTile>
__device__ __forceinline__ void reduce_block(
    const MistProblem &prob, const MistGroupDesc *__restrict__ g, const ReduceRange range,
    int p_tile, int lc_tile, const double *__restrict__ row_terms,
    const double *__restrict__ stage_floor /* of this group's stage 0 */, double ratio,
    double *lds_terms, double *lds_min, double *lds_pair, int32_t *lds_rowpos,
    const double *__restrict__ seed_cost,
    const int32_t *__restrict__ seed_index, double *__restrict__ out_cost,
    int32_t *__restrict__ out_index, bool skip_unchanged) {
  const int L = prob.num_layers;
  const int n_pairs = L * (L + 1) / 2 + L;  // sum over l = 1..L of (l + 1)
  const int pair_idx = lc_tile * MIST_LC_TILE + threadIdx.x;
  const bool active = pair_idx < n_pairs;
  const PairIndex pc = decode_pair(active ? pair_idx : 0);
  const int l = pc.l, c = pc.c;

  const int p0 = p_tile * MIST_P_TILE;
  const int n_tile_full = min(MIST_P_TILE, g->num_p - p0);  // p values of this tile
  // Cells with c == l - 1 are only kept for p == 0 of the base / with_pre variants
  // (batched_module_analyzer.py:3021-3023, 3103), so such a lane has at most one slot.
  // Lanes past the last pair of the tile keep no slots; they still hold rows in sieve A.
  const int n_tile =
      !active ? 0 : (c == l - 1 ? (kFirstTile ? min(n_tile_full, 1) : 0) : n_tile_full);
  int steps = 0;  // bisection steps that separate the n_tile + 1 possible counts
  while ((1 << steps) < n_tile + 1) ++steps;
  const bool do_post = kFirstTile && active && c != l - 1;
  const bool do_nopp = kFirstTile && active && l == L && c != l - 1;
  const GroupConsts k = group_consts(g);
  const double cap = prob.mem_cap_mb;
  const double G64 = (double)g->grad_accum;
  const float G32 = (float)g->grad_accum;
  const double inv_G64 = 1.0 / G64;
  const float inv_G32 = 1.0f / G32;
  // Stage costs the caller's search can use at all (MistProblem.stage_cost_incumbent): rows above
  // it are not looked for.  (The scout pass reads the first estimate, which a few rows gave
  // before it; the main launch reads the one the scout's seeds gave.)
  const double cutoff = prob.stage_cost_incumbent == nullptr || prob.sample_size != 1
                            ? (double)INFINITY
                            : *prob.stage_cost_incumbent * inv_G64 * (1.0 + kIncumbentSlack);
  const double pre_saved = g->pre_saved, pre_sas = g->pre_states_and_saved;
  const double pre_states = g->pre_states;
  const double post_states = g->post_states, post_fwd_peak = g->post_fwd_peak;
  const double post_bwd_peak = g->post_bwd_peak, post_output = g->post_output;

  double best_b[MIST_P_TILE], best_p[MIST_P_TILE];
  int32_t row_b[MIST_P_TILE], row_p[MIST_P_TILE];
  double best_post = INFINITY, best_pp = INFINITY;
  int32_t row_post = -1, row_pp = -1;
  // The minima of a tile are non-decreasing in p and finite on a prefix [0, fin); `top` is the
  // largest finite one.  A row that does not reach `top` can only fill the first empty slot.
  int fin_b = 0, fin_p = 0;
  double top_b = -INFINITY, top_p = -INFINITY;
  bool dirty = false;  // some slot of this lane differs from its seed
#pragma unroll
  for (int j = 0; j < MIST_P_TILE; ++j) {
    best_b[j] = best_p[j] = INFINITY;
    row_b[j] = row_p[j] = -1;
  }
  if (seed_cost != nullptr && active) {
    {  // the first slab of the tile's scout workgroups holds their combined minima
      const double *sc = seed_cost + threadIdx.x;
      const int32_t *si = seed_index + threadIdx.x;
#pragma unroll
      for (int j = 0; j < MIST_P_TILE; ++j) {
        const int32_t rb = si[j * MIST_LC_TILE], rp = si[(MIST_P_TILE + j) * MIST_LC_TILE];
        take_min(best_b[j], row_b[j], rb >= 0, sc[j * MIST_LC_TILE], rb);
        take_min(best_p[j], row_p[j], rp >= 0, sc[(MIST_P_TILE + j) * MIST_LC_TILE], rp);
      }
      const int32_t r2 = si[(2 * MIST_P_TILE) * MIST_LC_TILE];
      const int32_t r3 = si[(2 * MIST_P_TILE + 1) * MIST_LC_TILE];
      take_min(best_post, row_post, r2 >= 0, sc[(2 * MIST_P_TILE) * MIST_LC_TILE], r2);
      take_min(best_pp, row_pp, r3 >= 0, sc[(2 * MIST_P_TILE + 1) * MIST_LC_TILE], r3);
    }
#pragma unroll
    for (int j = 0; j < MIST_P_TILE; ++j) {
      if (row_b[j] >= 0) { fin_b = j + 1; top_b = best_b[j]; }
      if (row_p[j] >= 0) { fin_p = j + 1; top_p = best_p[j]; }
    }
  }

  const double *__restrict__ src = row_terms + g->row_offset * MIST_ROW_TERMS;

  // The tile's pairs are in (l, c) order, so its lanes hold a few consecutive l.  Per stage and
  // per such l, one wave-wide test tells which ROWS cannot fit any (c, p) of this tile with that
  // l (after sieve A's loops, below); it needs the group's pre / post terms to be non-negative.
  const int l_lo = __shfl(l, 0);
  const int n_active = __popcll((unsigned long long)__ballot(active));
  const int n_tile_l = __shfl(l, max(n_active - 1, 0)) - l_lo + 1;
  const bool rows_filtered = n_active > 0 && n_tile_l <= kTileLayerCounts && pre_saved >= 0.0 &&
                             pre_sas >= 0.0 && pre_states >= 0.0 && post_states >= 0.0 &&
                             post_output >= 0.0;

  // Sieve A visits pairs class by class (which first / last family member the latency uses is
  // fixed per class): 0 = 0 < c < l, 1 = c == 0, 2 = c == l.
  const int pair_class = !active ? 3 : (c == 0 ? 1 : (c == l ? 2 : 0));
  const uint64_t in_class0 = __ballot(pair_class == 0), in_class1 = __ballot(pair_class == 1);
  const uint64_t in_class2 = __ballot(pair_class == 2);

  const double lf = (double)l, lm1 = (double)max(l - 1, 0), cf = (double)c;
  const double l_minus_c = (double)(l - c), l_minus_c_1 = (double)(l - c - 1);
  const bool c_eq_l = c == l, c_ge_lm1 = c >= l - 1, c_eq_0 = c == 0;

  // get_latencies (:2165-2216): which family member a lane needs is fixed by its (l, c), so the
  // choice is made once as a column index instead of a per-row select.
  const int lm2 = max(l - 2, 0);
  const double n_ck = (double)min(max(c - 1, 0), lm2);
  const double n_nock = (double)(lm2 - min(max(c - 1, 0), lm2));
  const int first_col = c_eq_l ? 0 : 1, last_col = c_eq_0 ? 1 : 0;  // *_CK precedes *_NOCK
  const int post_col = c > 0 ? 0 : 1;
  lds_pair[threadIdx.x * kPairFields + 2] = n_ck;
  lds_pair[threadIdx.x * kPairFields + 3] = n_nock;
  auto div_G = [&](double v) { return kPow2G ? v * inv_G64 : v / G64; };
  // Group-wide terms the composite objectives add to the base latency (see `examine`): with x, d
  // the float32-rounded stable / delta latency,
  //   with_pre  = r (x + pre_fwd + pre_bwd + w1 + w2) + (d + w1d + w2d) / G
  //   with_post = r (x + post_fwd + [row terms >= 0]) + (d + [row terms >= 0]) / G
  //   no_pp     = r (x + pre_fwd + pre_bwd + post_fwd + [..] + w1 + w2 + [..]) + (d + w1d + w2d + [..]) / G
  // so each is at least r x + d / G plus the offset below, up to a few roundings of relative
  // size 1e-16 (all terms are non-negative).  A row can beat a minimum `t` of such an objective
  // only if r x + d / G <= t - offset; the offsets are taken 1e-9 short and `t` 1e-9 long, far
  // more than the roundings and far less than anything that matters for pruning.
  constexpr double kSlack = 1e-9;
  const double off_pre =
      (ratio * (k.pre_fwd + k.pre_bwd + k.w1 + k.w2) + div_G(k.w1d + k.w2d)) * (1.0 - kSlack);
  const double off_post = ratio * k.post_fwd * (1.0 - kSlack);
  const double off_pp = (ratio * (k.pre_fwd + k.pre_bwd + k.post_fwd + k.w1 + k.w2) +
                         div_G(k.w1d + k.w2d)) * (1.0 - kSlack);
  auto below = [&](double t, double offset) {
    return fabs(t) == INFINITY ? t : (t - offset) + kSlack * fabs(t);
  };

  // Memory model of one candidate row for this lane's (l, c) (:2150-2162, 2358-2385, 2755-2786).
  // `t` may also be the term-wise minimum of a stage: every operation below is monotone in
  // every term, so the peaks of that pseudo row bound the peaks of each row of the stage from
  // below.
  auto lane_memory = [&](const double *__restrict__ t) {
    LaneMemory mem;
    const double S_ck = t[MIST_T_S_CK], S_nock = t[MIST_T_S_NOCK];
    mem.fwd_states = t[MIST_T_FWD_STATES0] + lf * t[MIST_T_PWG] + lm1 * t[MIST_T_PO];
    mem.bwd_states = t[MIST_T_BWD_STATES0] + lf * t[MIST_T_PWGO];
    mem.cur_saved = c_eq_l ? (lf - 1.0) * S_ck : cf * S_ck + l_minus_c_1 * S_nock;
    mem.mod_saved = S_ck * cf + S_nock * l_minus_c;
    mem.ck_delta = c_ge_lm1 ? t[MIST_T_D_CK] : t[MIST_T_D_NOCK];
    mem.fwd_pk = t[MIST_T_FWD_PEAK];
    mem.bwd_pk = t[MIST_T_BWD_PEAK];
    mem.out = t[MIST_T_OUT];
    mem.gcb = t[MIST_T_GCB];
    mem.mf_base = t[MIST_T_MF_BASE];
    mem.mf_pp = t[MIST_T_MF_PP];
    return mem;
  };
  // Number of feasible p of this tile, in [lo, n_tile], by bisection with the exact test.
  auto feasible_count = [&](auto feasible, int lo) {
    int hi = n_tile;
    for (int it = 0; it < steps; ++it) {
      const int mid = (lo + hi) >> 1;
      const bool ok = feasible(p0 + mid);
      const bool open = lo < hi;
      lo = (open && ok) ? mid + 1 : lo;
      hi = (open && !ok) ? mid : hi;
    }
    return lo;
  };

  // Upper bound of that number for the pseudo row of a stage.  The peaks are linear in p up to
  // rounding, so the first infeasible slot is estimated from the values at the first two slots
  // and confirmed with the exact test: any slot at which the pseudo row is infeasible bounds the
  // count (monotonicity); an unconfirmed estimate falls back to the whole tile.
  auto count_bound = [&](auto scaled) {
    const double m0 = scaled(p0);
    if (!(m0 <= cap)) return 0;
    if (n_tile <= 1) return n_tile;
    const float slope = (float)(scaled(p0 + 1) - m0);
    if (!(slope > 0.0f)) return n_tile;
    const float est = fminf((float)(cap - m0) * __frcp_rn(slope), (float)n_tile);
    const int guess = (int)est + 1;  // slots 0 .. floor(est) are expected to be feasible
    if (guess >= n_tile) return n_tile;
    if (!(scaled(p0 + guess) <= cap)) return guess;
    if (guess + 1 < n_tile && !(scaled(p0 + guess + 1) <= cap)) return guess + 1;
    return n_tile;
  };

  // Stable / delta latency rounded to float32 (:2212-2213), the base objective r * x + y in
  // float64 (pareto.py:138; y = float32 array / python int, :2815) and a lower bound of the three
  // composite objectives: they add non-negative terms to x and d before the same monotone
  // operations, so none of them can be below it.
  auto objective = [&](const double *__restrict__ t, double &x, double &d, double &cost_base,
                       double &bound) {
    const double stable = n_ck * t[MIST_T_S_LAYER_CK] + n_nock * t[MIST_T_S_LAYER_NOCK] +
                          t[MIST_T_S_FIRST_CK + first_col] + t[MIST_T_S_LAST_CK + last_col];
    const double delta = n_ck * t[MIST_T_D_LAYER_CK] + n_nock * t[MIST_T_D_LAYER_NOCK] +
                         t[MIST_T_D_FIRST_CK + first_col] + t[MIST_T_D_LAST_CK + last_col];
    const float x32 = (float)stable, d32 = (float)delta;
    x = (double)x32;
    d = (double)d32;
    const float y32 = kPow2G ? d32 * inv_G32 : d32 / G32;
    const double rx = ratio * x;
    cost_base = rx + (double)y32;
    bound = rx + div_G(d);
  };

  // Sieves B (kCommit == false: would the row change anything, judged against the current
  // minima) and C (kCommit == true: apply it).  Returns whether the row survives / changed a slot.
  auto examine = [&](const double *__restrict__ t, int64_t pos, auto commit_tag) -> bool {
    constexpr bool kCommit = decltype(commit_tag)::value;
    double x, d, cost_base, bound;
    objective(t, x, d, cost_base, bound);
    const bool cand_b = (cost_base <= top_b || fin_b < n_tile) && cost_base <= cutoff;
    const bool want_pre = (bound <= top_p || fin_p < n_tile) && bound <= cutoff;
    const bool want_post = do_post && bound <= fmin(best_post, cutoff);
    const bool want_pp = do_nopp && bound <= fmin(best_pp, cutoff);
    if (!(cand_b || want_pre || want_post || want_pp)) return false;

    double cost_pre = INFINITY, cost_post = INFINITY, cost_pp = INFINITY;
    if (want_pre)
      cost_pre = ratio * (x + k.pre_fwd + k.pre_bwd + k.w1 + k.w2) + div_G(d + k.w1d + k.w2d);
    if (want_post || want_pp) {
      const double nag = t[MIST_T_NAG_CK + post_col], nrs = t[MIST_T_NRS_CK + post_col];
      const double ps1 = k.pp_wre ? nag : 0.0, ps2 = k.pp_gre ? nrs : 0.0;
      const double pd1 = k.pp_wre ? 0.0 : nag, pd2 = k.pp_gre ? 0.0 : nrs;
      const double opb = t[MIST_T_OPB];
      cost_post = ratio * (x + k.post_fwd + opb + ps1 + ps2) + div_G(d + pd1 + pd2);
      cost_pp = ratio * (x + k.pre_fwd + k.pre_bwd + k.post_fwd + opb + k.w1 + k.w2 + ps1 + ps2) +
                div_G(d + k.w1d + k.w2d + pd1 + pd2);
    }

    // Lowest slot the row could change: the minima are non-decreasing in p, so it is the number
    // of slots whose minimum is strictly below the row's value (empty slots hold +inf; a tie is
    // decided by the row index when the slot is updated).
    int lo_b = fin_b, lo_p = fin_p;
    if (cost_base <= top_b) {
      lo_b = 0;
#pragma unroll
      for (int j = 0; j < MIST_P_TILE; ++j) lo_b += best_b[j] < cost_base ? 1 : 0;
    }
    if (cost_pre <= top_p) {
      lo_p = 0;
#pragma unroll
      for (int j = 0; j < MIST_P_TILE; ++j) lo_p += best_p[j] < cost_pre ? 1 : 0;
    }
    bool need_b = cand_b && lo_b < n_tile, need_p = want_pre && lo_p < n_tile && cost_pre <= cutoff;
    bool need_post = want_post && cost_post <= fmin(best_post, cutoff);
    bool need_pp = want_pp && cost_pp <= fmin(best_pp, cutoff);
    if (!(need_b || need_p || need_post || need_pp)) return false;

    const LaneMemory mem = lane_memory(t);
    auto feasible_base = [&](int p) { return mem.feasible_base(p, cap); };
    auto feasible_pre = [&](int p) { return mem.feasible_pre(p, cap, pre_saved, pre_sas); };

    need_b = need_b && feasible_base(p0 + lo_b);
    need_p = need_p && feasible_pre(p0 + lo_p);
    bool ok_pp = false;
    if (need_post || need_pp) {
      // ---- last stage / single stage, p == 0 only (:2946-3106) ----
      double peak_f, peak_b;
      mem.peaks(0, peak_f, peak_b);
      const double f_in = mem.fwd_states + post_states + mem.mod_saved + post_fwd_peak + mem.gcb;
      const double b_in = mem.bwd_states + post_states + mem.mod_saved + post_bwd_peak +
                          (c_eq_0 ? t[MIST_T_RD] : 0.0) + mem.gcb;
      const double pf_post = fmax(f_in, peak_f + post_states);
      const double pb_post = fmax(b_in, peak_b - mem.out + post_states) + post_output;
      const bool ok_post = fmax(pf_post, pb_post) * mem.mf_pp <= cap;
      if (need_pp) {
        const double pf_pp = pf_post + pre_states + pre_saved;
        const double pb_pp = pb_post + pre_states + pre_saved;
        ok_pp = fmax(pf_pp, pb_pp) * t[MIST_T_MF] <= cap;
      }
      need_post = need_post && ok_post;
      need_pp = need_pp && ok_pp;
    }
    if (!kCommit) return need_b || need_p || need_post || need_pp;

    const int32_t row = row_of_position(g, pos);
    bool changed = false;
    if (need_b) {
      const double cost = cost_base;
      const int lo = feasible_count(feasible_base, lo_b + 1);  // slot lo_b is known feasible
#pragma unroll
      for (int j = 0; j < MIST_P_TILE; ++j) {
        const bool better = j >= lo_b && j < lo && lex_less(cost, row, best_b[j], row_b[j]);
        best_b[j] = better ? cost : best_b[j];
        row_b[j] = better ? row : row_b[j];
        changed |= better;
      }
      // Bookkeeping of (fin, top) without indexing the register array dynamically.
      if (lo > fin_b) { fin_b = lo; top_b = cost; }
      else if (lo == fin_b) top_b = fmin(top_b, cost);
    }
    if (need_p) {
      const double cost = cost_pre;
      const int lo = feasible_count(feasible_pre, lo_p + 1);
#pragma unroll
      for (int j = 0; j < MIST_P_TILE; ++j) {
        const bool better = j >= lo_p && j < lo && lex_less(cost, row, best_p[j], row_p[j]);
        best_p[j] = better ? cost : best_p[j];
        row_p[j] = better ? row : row_p[j];
        changed |= better;
      }
      if (lo > fin_p) { fin_p = lo; top_p = cost; }
      else if (lo == fin_p) top_p = fmin(top_p, cost);
    }
    if (need_post) {
      changed |= lex_less(cost_post, row, best_post, row_post);
      take_min(best_post, row_post, true, cost_post, row);
    }
    if (need_pp) {
      changed |= lex_less(cost_pp, row, best_pp, row_pp);
      take_min(best_pp, row_pp, true, cost_pp, row);
    }
    return changed;
  };

  // Stages this workgroup visits: every stage_step-th one of its range, without those the scout
  // pass has done.  (skip_stride > 1 goes with stage_step == 1: two skips are never adjacent.)
  const bool gathered = range.gathered != 0;
  const int64_t n_gather = (int64_t)g->n_par * g->n_oo * g->n_ao * max(g->scout_stride, 1);
  const int64_t end_stage =
      ((gathered ? n_gather : range.row_end) + kStageRows - 1) / kStageRows;
  auto skipped = [&](int64_t st) { return range.skip_stride > 0 && st % range.skip_stride == 0; };
  auto after = [&](int64_t st) {
    st += range.stage_step;
    return skipped(st) ? st + range.stage_step : st;
  };
  // The summary of a stage (term-wise minima of its rows, written with the row terms) is one
  // 32-lane load; the next stage's is in flight while the current stage is processed.
  // (Gathered rows have no summary: zero is a lower bound of every term, +inf an upper bound of
  // the output term.)
  auto load_floor = [&](int64_t st) {
    if (gathered) return (int)threadIdx.x == kStageMaxOut ? (double)INFINITY : 0.0;
    return threadIdx.x < kStageFloorPitch ? stage_floor[st * kStageFloorPitch + threadIdx.x] : 0.0;
  };
  int64_t stage = range.row_begin / kStageRows;
  if (skipped(stage)) stage += range.stage_step;
  double floor_v = stage < end_stage ? load_floor(stage) : 0.0;
  for (; stage < end_stage; stage = after(stage)) {
    const int64_t base = stage * kStageRows;
    const int n_stage =
        (int)min((int64_t)kStageRows, (gathered ? n_gather : range.row_end) - base);
    __syncthreads();
    // workspace position of row r of the stage
    lds_rowpos[threadIdx.x] =
        (int32_t)(gathered ? gathered_position(g, min(base + threadIdx.x, n_gather - 1))
                           : base + threadIdx.x);
    if (threadIdx.x < kStageFloorPitch) lds_min[threadIdx.x] = floor_v;
    if (after(stage) < end_stage) floor_v = load_floor(after(stage));
    __syncthreads();

    // ---- the pseudo row (term-wise minimum of the stage) against the loosest thresholds, the
    // largest minimum of each objective: the thresholds below are no larger, so a stage that
    // no lane passes here is closed, and its memory bounds need not be formed ----
    double floor_x, floor_d, floor_cost, floor_bound;
    objective(lds_min, floor_x, floor_d, floor_cost, floor_bound);
    // What the last-stage / single-stage objectives add to every row of this stage on top of
    // their group-wide offsets: at least the stage's smallest post-layer terms (same slack).
    const double nag_min = lds_min[kStageMinNag], nrs_min = lds_min[kStageMinNrs];
    const double stage_post =
        (ratio * (lds_min[kStageMinOpb] + (k.pp_wre ? nag_min : 0.0) + (k.pp_gre ? nrs_min : 0.0)) +
         div_G((k.pp_wre ? 0.0 : nag_min) + (k.pp_gre ? 0.0 : nrs_min))) * (1.0 - kSlack);
    {
      const double loose_b = fmin(fin_b < n_tile ? (double)INFINITY : top_b, cutoff);
      const double loose_p = fmin(fin_p < n_tile ? (double)INFINITY : top_p, cutoff);
      double loose_o = below(loose_p, off_pre);
      if (do_post) loose_o = fmax(loose_o, below(fmin(best_post, cutoff), off_post + stage_post));
      if (do_nopp) loose_o = fmax(loose_o, below(fmin(best_pp, cutoff), off_pp + stage_post));
      if (!__any(active && (floor_cost <= loose_b || floor_bound <= loose_o))) continue;
    }

    // ---- per-stage thresholds: no row of the stage is feasible beyond the pseudo row's count,
    // so only the minima of the slots below it can be beaten ----
    const LaneMemory floor_mem = lane_memory(lds_min);
    const int cnt_b = count_bound([&](int p) { return floor_mem.scaled_base(p); });
    const int cnt_p =
        count_bound([&](int p) { return floor_mem.scaled_pre(p, pre_saved, pre_sas); });
    double thr_b = -INFINITY, thr_p = -INFINITY;
#pragma unroll
    for (int j = 0; j < MIST_P_TILE; ++j) {  // minima are non-decreasing; empty slots hold +inf
      thr_b = j < cnt_b ? best_b[j] : thr_b;
      thr_p = j < cnt_p ? best_p[j] : thr_p;
    }
    thr_b = fmin(thr_b, cutoff);
    thr_p = fmin(thr_p, cutoff);
    // One threshold for the three composite objectives, expressed for `bound` (objective()):
    // each of them exceeds `bound` by at least its group-wide offset.
    double thr_o = below(thr_p, off_pre);
    if (do_post) {
      // Lower bounds of the last-stage / single-stage peaks (:2946-3106) from the pseudo row.
      double peak_f, peak_b;
      floor_mem.peaks(0, peak_f, peak_b);
      const double f_in =
          floor_mem.fwd_states + post_states + floor_mem.mod_saved + post_fwd_peak + floor_mem.gcb;
      const double b_in =
          floor_mem.bwd_states + post_states + floor_mem.mod_saved + post_bwd_peak + floor_mem.gcb;
      const double pf_post = fmax(f_in, peak_f + post_states);
      const double pb_post = fmax(b_in, peak_b - lds_min[kStageMaxOut] + post_states) + post_output;
      if (fmax(pf_post, pb_post) * floor_mem.mf_pp <= cap)
        thr_o = fmax(thr_o, below(fmin(best_post, cutoff), off_post + stage_post));
      if (do_nopp) {
        const double pf_pp = pf_post + pre_states + pre_saved;
        const double pb_pp = pb_post + pre_states + pre_saved;
        if (fmax(pf_pp, pb_pp) * lds_min[MIST_T_MF] <= cap)
          thr_o = fmax(thr_o, below(fmin(best_pp, cutoff), off_pp + stage_post));
      }
    }

    // ---- sieve A: the rows of the stage against those thresholds.  First the pseudo row of
    // term-wise minima: the objective is monotone in every term, so a pair the pseudo row does
    // not pass is passed by no row of the stage (two thirds of all stages end here).  For the
    // other pairs the test runs transposed: a lane holds the latency terms of ONE ROW in
    // registers and the loop runs over those pairs, whose constants and thresholds are
    // wave-uniform reads of the per-pair table.  The wave-wide comparison result is exactly the
    // 64-row survivor mask of that pair; it is handed to the pair's lane. ----
    uint64_t sieve = 0;
    uint64_t pairs_open;
    pairs_open = __ballot(active && (floor_cost <= thr_b || floor_bound <= thr_o));
    if (pairs_open != 0) {
      lds_pair[threadIdx.x * kPairFields + 0] = thr_b;
      lds_pair[threadIdx.x * kPairFields + 1] = thr_o;
      if (!gathered) {  // 16-byte loads: a row is 17 such pairs and starts 16-byte aligned
        const double2 *__restrict__ src2 =
            reinterpret_cast<const double2 *>(src + base * MIST_ROW_TERMS);
        for (int i = threadIdx.x; i < n_stage * (MIST_ROW_TERMS / 2); i += MIST_LC_TILE) {
          const double2 v = src2[i];
          const int at =
              (i / (MIST_ROW_TERMS / 2)) * kLdsRowStride + 2 * (i % (MIST_ROW_TERMS / 2));
          lds_terms[at] = v.x;
          lds_terms[at + 1] = v.y;
        }
      } else {  // the same, row by row from the gathered positions
        const double2 *__restrict__ src2 = reinterpret_cast<const double2 *>(src);
        for (int i = threadIdx.x; i < n_stage * (MIST_ROW_TERMS / 2); i += MIST_LC_TILE) {
          const int r = i / (MIST_ROW_TERMS / 2), c2 = i % (MIST_ROW_TERMS / 2);
          const double2 v = src2[(int64_t)lds_rowpos[r] * (MIST_ROW_TERMS / 2) + c2];
          lds_terms[r * kLdsRowStride + 2 * c2] = v.x;
          lds_terms[r * kLdsRowStride + 2 * c2 + 1] = v.y;
        }
      }
      __syncthreads();
      double rt[MIST_T_D_LAST_NOCK + 1];
#pragma unroll
      for (int i = 0; i <= MIST_T_D_LAST_NOCK; ++i)
        rt[i] = lds_terms[threadIdx.x * kLdsRowStride + i];  // stale beyond n_stage, masked below
      __syncthreads();
      const uint64_t valid_rows = n_stage < kStageRows ? (1ull << n_stage) - 1ull : ~0ull;
      auto sieve_class = [&](uint64_t todo, auto first_col_tag, auto last_col_tag) {
        constexpr int kFirstCol = decltype(first_col_tag)::value;
        constexpr int kLastCol = decltype(last_col_tag)::value;
        const double s_first = rt[MIST_T_S_FIRST_CK + kFirstCol];
        const double s_last = rt[MIST_T_S_LAST_CK + kLastCol];
        const double d_first = rt[MIST_T_D_FIRST_CK + kFirstCol];
        const double d_last = rt[MIST_T_D_LAST_CK + kLastCol];
        while (todo != 0) {
          const int pair_lane = __ffsll((unsigned long long)todo) - 1;
          todo &= todo - 1;
          const double pair_thr_b = lds_pair[pair_lane * kPairFields + 0];
          const double pair_thr_o = lds_pair[pair_lane * kPairFields + 1];
          const double pair_n_ck = lds_pair[pair_lane * kPairFields + 2];
          const double pair_n_nock = lds_pair[pair_lane * kPairFields + 3];
          const double stable = pair_n_ck * rt[MIST_T_S_LAYER_CK] +
                                pair_n_nock * rt[MIST_T_S_LAYER_NOCK] + s_first + s_last;
          const double delta = pair_n_ck * rt[MIST_T_D_LAYER_CK] +
                               pair_n_nock * rt[MIST_T_D_LAYER_NOCK] + d_first + d_last;
          const float x32 = (float)stable, d32 = (float)delta;
          const float y32 = kPow2G ? d32 * inv_G32 : d32 / G32;
          const double rx = ratio * (double)x32;
          const double cost_base = rx + (double)y32;
          const double bound = rx + div_G((double)d32);
          const uint64_t survivors =
              __ballot(cost_base <= pair_thr_b || bound <= pair_thr_o) & valid_rows;
          sieve = (int)threadIdx.x == pair_lane ? survivors : sieve;
        }
      };
      sieve_class(pairs_open & in_class0, std::integral_constant<int, 1>{},
                  std::integral_constant<int, 0>{});
      sieve_class(pairs_open & in_class1, std::integral_constant<int, 1>{},
                  std::integral_constant<int, 1>{});
      sieve_class(pairs_open & in_class2, std::integral_constant<int, 0>{},
                  std::integral_constant<int, 0>{});
      // Rows that exceed the capacity with tile_l layers whatever c, p and variant: every
      // variant's tested quantity is at least
      //   max(fwd, bwd) * (smallest of the row's three memory factors),
      //   fwd = fwd_states + (l - 1) min(S_ck, S_nock) + min(D_ck, D_nock) + fwd_peak + gcb
      //         + p0 (l min(S_ck, S_nock) + 2 out),   bwd likewise with out counted once
      // (cur_saved and mod_saved are sums of l - 1 and l saved terms; the last-stage variants
      // take one output off the backward peak; pre / post terms only add).  The bound is taken
      // 1e-9 short, far more than the roundings of the two evaluation orders.
      if (rows_filtered && __any(sieve != 0)) {
        uint64_t fits = ~0ull;
        const double *mine = lds_terms + threadIdx.x * kLdsRowStride;
        const double s_min = fmin(mine[MIST_T_S_CK], mine[MIST_T_S_NOCK]);
        const double d_min = fmin(mine[MIST_T_D_CK], mine[MIST_T_D_NOCK]);
        const double out = mine[MIST_T_OUT], gcb = mine[MIST_T_GCB];
        const double mf_min =
            fmin(fmin(mine[MIST_T_MF_BASE], mine[MIST_T_MF_PP]), mine[MIST_T_MF]);
        const double fwd0 = mine[MIST_T_FWD_STATES0] + d_min + mine[MIST_T_FWD_PEAK] + gcb;
        const double bwd0 = mine[MIST_T_BWD_STATES0] + d_min + mine[MIST_T_BWD_PEAK] + out + gcb;
        const double pwg = mine[MIST_T_PWG], po = mine[MIST_T_PO], pwgo = mine[MIST_T_PWGO];
#pragma unroll 1
        for (int i = 0; i < n_tile_l; ++i) {
          const double tl = (double)(l_lo + i), tl1 = (double)max(l_lo + i - 1, 0);
          const double per_p = tl * s_min + 2.0 * out;
          const double shared = tl1 * s_min + (double)p0 * per_p;
          const double low = fmax(fwd0 + tl * pwg + tl1 * po + shared, bwd0 + tl * pwgo + shared);
          const bool too_big = s_min >= 0.0 && out >= 0.0 && low >= 0.0 && mf_min >= 0.0 &&
                               low * mf_min * (1.0 - 1e-9) > cap;
          fits = l - l_lo == i ? ~__ballot(too_big) : fits;
        }
        sieve &= fits;
      }
    }

    // ---- sieve B: lowest improvable slot and the memory test there, per-lane survivors.  It
    // pays when it rejects most rows (the main pass: 96 %); the scout pass starts from empty
    // minima and most of what reaches it also changes a slot, so there C takes the rows as they
    // come (C repeats every test of B). ----
    uint64_t keep = 0;
    if (gathered) {
      keep = sieve;
      sieve = 0;
    }
    while (sieve != 0) {
      const int r = __ffsll((unsigned long long)sieve) - 1;
      sieve &= sieve - 1;
      const bool hit = examine(lds_terms + r * kLdsRowStride, lds_rowpos[r], std::false_type{});
      keep |= (uint64_t)(hit ? 1 : 0) << r;
    }

    // ---- sieve C: survivors in row order against the live minima ----
    while (keep != 0) {
      const int r = __ffsll((unsigned long long)keep) - 1;
      keep &= keep - 1;
      dirty |= examine(lds_terms + r * kLdsRowStride, lds_rowpos[r], std::true_type{});
    }
  }

  // A chunk that changed no slot holds exactly its seeds, which the first chunk of the tile
  // writes out anyway: it leaves a mark instead of its 26 KB slab, and the combining kernel
  // skips it.
  if (skip_unchanged && !__any(dirty)) {
    if (threadIdx.x == 0) out_index[0] = kSlabUnchanged;
    return;
  }

#pragma unroll
  for (int j = 0; j < MIST_P_TILE; ++j) {
    out_cost[j * MIST_LC_TILE + threadIdx.x] = best_b[j];
    out_index[j * MIST_LC_TILE + threadIdx.x] = row_b[j];
    out_cost[(MIST_P_TILE + j) * MIST_LC_TILE + threadIdx.x] = best_p[j];
    out_index[(MIST_P_TILE + j) * MIST_LC_TILE + threadIdx.x] = row_p[j];
  }
  out_cost[(2 * MIST_P_TILE) * MIST_LC_TILE + threadIdx.x] = best_post;
  out_index[(2 * MIST_P_TILE) * MIST_LC_TILE + threadIdx.x] = row_post;
  out_cost[(2 * MIST_P_TILE + 1) * MIST_LC_TILE + threadIdx.x] = best_pp;
  out_index[(2 * MIST_P_TILE + 1) * MIST_LC_TILE + threadIdx.x] = row_pp;
}

// scout != 0: kScoutSplit workgroups per (group, (l, c) tile, p tile) share the gathered rows
// of the whole group, results in slab n_blocks + logical workgroup.
// scout == 0: one workgroup per row chunk of such a tile, seeded from the scout's slabs when the
// group has them.
__global__ __launch_bounds__(MIST_LC_TILE, MIST_REDUCE_MIN_WAVES) void eval_reduce_kernel(
    const MistProblem prob, const MistGroupDesc *__restrict__ groups, int n_groups,
    const int32_t *__restrict__ block_prefix, int n_blocks,
    const int32_t *__restrict__ scout_prefix, int scout, const double *__restrict__ row_terms,
    const double *__restrict__ stage_floor, const RatioList ratios, int first_sample,
    int64_t scout_base, double *__restrict__ partial_cost, int32_t *__restrict__ partial_index) {
  __shared__ double lds_terms[kStageRows * kLdsRowStride];
  __shared__ double lds_min[kStageFloorPitch];
  __shared__ double lds_pair[MIST_LC_TILE * kPairFields];
  __shared__ int32_t lds_rowpos[kStageRows];
  // blockIdx.y = sample first_sample + y of the ratio list.  Slabs: the main launch of its y-th
  // sample writes slabs y * n_blocks + workgroup; the scout slabs of sample s (of the list) are
  // scout_base + s * n_scout_total + workgroup, and seed the main launch of the same sample.
  const int sample = first_sample + (int)blockIdx.y;
  const double ratio = ratios.r[sample];
  const int n_scout_total = scout_prefix != nullptr ? scout_prefix[n_groups] : 0;
  const int block = xcd_run_block(blockIdx.x);
  if (block >= (scout ? n_scout_total : n_blocks)) return;
  int local_block;
  const MistGroupDesc *g = find_group(groups, scout ? scout_prefix : block_prefix, n_groups,
                                      block, &local_block);
  const int gi = (int)(g - groups);
  const bool seeded = scout_prefix != nullptr && g->scout_stride > 0;
  int tile;
  ReduceRange range;
  int64_t out_slab;
  bool skip_unchanged = false;  // only the chunks after the first of a tile may leave a mark
  if (scout) {
    if (g->scout_stride <= 0) return;
    tile = local_block / kScoutSplit;
    const int part = local_block % kScoutSplit;  // gathered stages part, part + split, ...
    range = ReduceRange{(int64_t)part * kStageRows, g->n_rows, kScoutSplit, 0, 1};
    out_slab = scout_base + (int64_t)sample * n_scout_total + block;
  } else {
    const int n_tiles = g->n_lc_tiles * g->n_p_tiles;
    const int chunk = local_block / n_tiles;  // the tiles of one chunk are neighbours
    tile = local_block % n_tiles;
    const int64_t row_begin = (int64_t)chunk * g->rows_per_chunk;
    range = ReduceRange{row_begin, min(row_begin + (int64_t)g->rows_per_chunk, g->n_rows), 1, 0, 0};
    out_slab = (int64_t)blockIdx.y * n_blocks + block;
    skip_unchanged = chunk > 0;
  }
  const int p_tile = tile % g->n_p_tiles;
  const int lc_tile = g->lc_tile_begin + tile / g->n_p_tiles;  // position in the pair list
  const int64_t slab = (int64_t)kSlots * MIST_LC_TILE;
  const int64_t seed_slab = scout_base + (int64_t)sample * n_scout_total +
                            (seeded ? scout_prefix[gi] + tile * kScoutSplit : 0);
  const double *seed_cost = (!scout && seeded) ? partial_cost + seed_slab * slab : nullptr;
  const int32_t *seed_index = (!scout && seeded) ? partial_index + seed_slab * slab : nullptr;
  const bool pow2 = (g->grad_accum & (g->grad_accum - 1)) == 0;
#define MIST_REDUCE(P2, FT)                                                                   \
  reduce_block<P2, FT>(prob, g, range, p_tile, lc_tile, row_terms,                            \
                       stage_floor + stage_floor_slot(g, gi, 0) * kStageFloorPitch, ratio,    \
                       lds_terms, lds_min, lds_pair, lds_rowpos, seed_cost, seed_index,                   \
                       partial_cost + out_slab * slab, partial_index + out_slab * slab,       \
                       skip_unchanged)
  if (pow2) {
    if (p_tile == 0) MIST_REDUCE(true, true); else MIST_REDUCE(true, false);
  } else {
    if (p_tile == 0) MIST_REDUCE(false, true); else MIST_REDUCE(false, false);
  }
#undef MIST_REDUCE
}

// Rows offered in ascending order: the first of equal costs stays (pareto.py:134-142 as written).
__device__ __forceinline__ void take_first(double &best, int32_t &best_row, bool feasible,
                                           double cost, int32_t row) {
  const bool better = feasible && cost < best;
  best = better ? cost : best;
  best_row = better ? row : best_row;
}

// ------------------------------------------------------------------------------------------
// Kernel 2x: the same reduction with every cell evaluated.  No scout pass, no sieves, no bounds,
// no bisection: each (row, l, c) goes through the latency model and the memory model, and each
// of its p values through the reference's feasibility test and the (cost, row) comparison.  This
// is the work the reference's formulas describe cell by cell; the pruned kernel above must
// produce the same tables (tests) and is measured against it.  Same decomposition and slab
// layout as eval_reduce_kernel's main launch, so finalize_kernel reads either.
// ------------------------------------------------------------------------------------------
template <bool kFirstTile>
__device__ __forceinline__ void exhaustive_block(
    const MistProblem &prob, const MistGroupDesc *__restrict__ g, int64_t row_begin,
    int64_t row_end, int p_tile, int lc_tile, const double *__restrict__ row_terms, double ratio,
    double *lds_terms, int32_t *lds_row, double *__restrict__ out_cost,
    int32_t *__restrict__ out_index) {
  const int L = prob.num_layers;
  const int n_pairs = L * (L + 1) / 2 + L;
  const int pair_idx = lc_tile * MIST_LC_TILE + threadIdx.x;
  const bool active = pair_idx < n_pairs;
  const PairIndex pc = decode_pair(active ? pair_idx : 0);
  const int l = pc.l, c = pc.c;
  const int p0 = p_tile * MIST_P_TILE;
  const int n_tile = active ? min(MIST_P_TILE, g->num_p - p0) : 0;
  const GroupConsts k = group_consts(g);
  const double cap = prob.mem_cap_mb;
  const double G64 = (double)g->grad_accum;
  const float G32 = (float)g->grad_accum;
  const double pre_saved = g->pre_saved, pre_sas = g->pre_states_and_saved;

  double best_b[MIST_P_TILE], best_p[MIST_P_TILE];
  int32_t row_b[MIST_P_TILE], row_p[MIST_P_TILE];
  double best_post = INFINITY, best_pp = INFINITY;
  int32_t row_post = -1, row_pp = -1;
#pragma unroll
  for (int j = 0; j < MIST_P_TILE; ++j) {
    best_b[j] = best_p[j] = INFINITY;
    row_b[j] = row_p[j] = -1;
  }
  const double *__restrict__ src = row_terms + g->row_offset * MIST_ROW_TERMS;
  for (int64_t base = row_begin; base < row_end; base += kStageRows) {
    const int n_stage = (int)min((int64_t)kStageRows, row_end - base);
    __syncthreads();
    // Rows are visited in the REFERENCE's order (the chunk is a range of row numbers, gathered
    // from wherever the workspace order put them; lane = row for the index arithmetic), so that
    // within a chunk a strict "<" keeps the first of equal costs like the reference's scan does.
    lds_row[threadIdx.x] = (int32_t)position_of_row(g, min(base + threadIdx.x, row_end - 1));
    __syncthreads();
    const double2 *__restrict__ src2 = reinterpret_cast<const double2 *>(src);
    for (int i = threadIdx.x; i < n_stage * (MIST_ROW_TERMS / 2); i += MIST_LC_TILE) {
      const int r = i / (MIST_ROW_TERMS / 2), c2 = i % (MIST_ROW_TERMS / 2);
      const double2 v = src2[(int64_t)lds_row[r] * (MIST_ROW_TERMS / 2) + c2];
      lds_terms[r * kLdsRowStride + 2 * c2] = v.x;
      lds_terms[r * kLdsRowStride + 2 * c2 + 1] = v.y;
    }
    __syncthreads();
    if (!active) continue;
    for (int r = 0; r < n_stage; ++r) {
      const double *t = lds_terms + r * kLdsRowStride;
      const int32_t row = (int32_t)(base + r);
      const CellLatency lat = cell_latency<kFirstTile>(t, l, c, k);
      const LaneMemory mem = cell_memory(t, l, c);
      // objectives r * x + y (pareto.py:138): base with y = float32 delta / G in float32
      // (batched_module_analyzer.py:2815), the others in float64 (:2898-2903, 3002-3007, 3084-3089)
      const double cost_base = ratio * (double)lat.x + (double)(lat.d / G32);
      const double cost_pre = ratio * lat.sp + lat.dpre / G64;
      // Every slot through both feasibility tests (:2805-2812, 2893-2897), straight-line: the two
      // tests share the peaks of their p, and nothing is skipped by a branch (a lane whose tile
      // ends early only masks the update).
#pragma unroll
      for (int j = 0; j < MIST_P_TILE; ++j) {
        double peak_f, peak_b;
        mem.peaks(p0 + j, peak_f, peak_b);
        const bool fits_base = fmax(peak_f, peak_b) * mem.mf_base <= cap;
        const double pre_p = (double)(p0 + j) * pre_saved;
        const bool fits_pre = fmax(pre_p + peak_f + pre_sas, pre_p + peak_b + pre_sas) * mem.mf_pp <= cap;
        const bool live = j < n_tile;
        take_first(best_b[j], row_b[j], live & fits_base, cost_base, row);
        take_first(best_p[j], row_p[j], live & fits_pre, cost_pre, row);
      }
      if (kFirstTile) {  // last stage / single stage, p == 0 only (:2946-3106)
        double peak_f, peak_b;
        mem.peaks(0, peak_f, peak_b);
        const double f_in = mem.fwd_states + g->post_states + mem.mod_saved + g->post_fwd_peak + mem.gcb;
        const double b_in = mem.bwd_states + g->post_states + mem.mod_saved + g->post_bwd_peak +
                            (c == 0 ? t[MIST_T_RD] : 0.0) + mem.gcb;
        const double pf_post = fmax(f_in, peak_f + g->post_states);
        const double pb_post = fmax(b_in, peak_b - mem.out + g->post_states) + g->post_output;
        const bool ok_post = fmax(pf_post, pb_post) * mem.mf_pp <= cap;
        const double pf_pp = pf_post + g->pre_states + g->pre_saved;
        const double pb_pp = pb_post + g->pre_states + g->pre_saved;
        const bool ok_pp = fmax(pf_pp, pb_pp) * t[MIST_T_MF] <= cap;
        take_first(best_post, row_post, ok_post, ratio * lat.spost + lat.dpost / G64, row);
        take_first(best_pp, row_pp, ok_pp, ratio * lat.spp + lat.dpp / G64, row);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < MIST_P_TILE; ++j) {
    out_cost[j * MIST_LC_TILE + threadIdx.x] = best_b[j];
    out_index[j * MIST_LC_TILE + threadIdx.x] = row_b[j];
    out_cost[(MIST_P_TILE + j) * MIST_LC_TILE + threadIdx.x] = best_p[j];
    out_index[(MIST_P_TILE + j) * MIST_LC_TILE + threadIdx.x] = row_p[j];
  }
  out_cost[(2 * MIST_P_TILE) * MIST_LC_TILE + threadIdx.x] = best_post;
  out_index[(2 * MIST_P_TILE) * MIST_LC_TILE + threadIdx.x] = row_post;
  out_cost[(2 * MIST_P_TILE + 1) * MIST_LC_TILE + threadIdx.x] = best_pp;
  out_index[(2 * MIST_P_TILE + 1) * MIST_LC_TILE + threadIdx.x] = row_pp;
}

#ifndef MIST_EXHAUSTIVE_MIN_WAVES
#define MIST_EXHAUSTIVE_MIN_WAVES 2
#endif
__global__ __launch_bounds__(MIST_LC_TILE, MIST_EXHAUSTIVE_MIN_WAVES) void eval_reduce_exhaustive_kernel(
    const MistProblem prob, const MistGroupDesc *__restrict__ groups, int n_groups,
    const int32_t *__restrict__ block_prefix, int n_blocks, const double *__restrict__ row_terms,
    double ratio, double *__restrict__ partial_cost, int32_t *__restrict__ partial_index) {
  __shared__ double lds_terms[kStageRows * kLdsRowStride];
  __shared__ int32_t lds_row[kStageRows];
  const int block = xcd_run_block(blockIdx.x);
  if (block >= n_blocks) return;
  int local_block;
  const MistGroupDesc *g = find_group(groups, block_prefix, n_groups, block, &local_block);
  const int n_tiles = g->n_lc_tiles * g->n_p_tiles;
  const int chunk = local_block / n_tiles, tile = local_block % n_tiles;
  const int64_t row_begin = (int64_t)chunk * g->rows_per_chunk;
  const int64_t row_end = min(row_begin + (int64_t)g->rows_per_chunk, g->n_rows);
  const int p_tile = tile % g->n_p_tiles, lc_tile = g->lc_tile_begin + tile / g->n_p_tiles;
  const int64_t slab = (int64_t)kSlots * MIST_LC_TILE;
  if (p_tile == 0)
    exhaustive_block<true>(prob, g, row_begin, row_end, p_tile, lc_tile, row_terms, ratio,
                           lds_terms, lds_row, partial_cost + block * slab, partial_index + block * slab);
  else
    exhaustive_block<false>(prob, g, row_begin, row_end, p_tile, lc_tile, row_terms, ratio,
                            lds_terms, lds_row, partial_cost + block * slab, partial_index + block * slab);
}

// The equal-stage pipeline a group offers to the stage-cost estimates: S stages of L / S layers
// on the group's mesh, or 0 when the devices or the layers do not divide, the group has too few
// pre-saved micro-batch values, or the caller's search does not go that deep.
__device__ __forceinline__ int incumbent_stage_count(const MistProblem &prob,
                                                     const MistGroupDesc *__restrict__ g) {
  const int L = prob.num_layers, D = prob.incumbent_num_devices;
  const int nm = g->num_nodes * g->num_gpus_per_node;
  if (nm <= 0 || D % nm != 0) return 0;
  const int S = D / nm;
  if (S < 1 || S > L || L % S != 0 || S - 1 >= g->num_p) return 0;
  // (the per-mesh search goes up to min(devices, layers) / 2 stages, inter_tuning.py:279-281)
  if (prob.incumbent_ckpt_rule == 0 && S > (D < L ? D : L) / 2) return 0;
  return S;
}

// Cost of the best pipeline of equal stages on equal meshes that the scout pass's seeds allow
// (sample 0 of a call with one sample, whose objective is the stage cost): group (G, mesh (n, m))
// offers S = devices / (n m) stages of L / S layers each, the first one from the with_pre table
// at S - 1 pre-saved micro-batches, the last one from the with_post table, those between from
// the base table, a single one from the no_pp table, each at its cheapest admissible ckpt count
// (rule of the caller's search, MistProblem.incumbent_ckpt_rule); the cost is the sum of the
// stage costs + (G - 1) x the largest, as the search forms it (inter_tuning.py:342).  Seeds are
// minima over some rows, so the finished tables hold no larger values; the search that reads
// them returns no more than this unless its scan never tries the thresholds of that pipeline
// (a single-stage cost is no threshold candidate of the reference, and its gap rule drops
// some), which is why the caller checks its result against the bound that was used.
// Workgroup = group, its wavefronts take the stages in turn; lowers *incumbent.
constexpr int kIncumbentWaves = 4;
__global__ __launch_bounds__(64 * kIncumbentWaves) void incumbent_kernel(
    const MistProblem prob, const MistGroupDesc *__restrict__ groups,
    const int32_t *__restrict__ scout_prefix, int64_t scout_base,
    const double *__restrict__ partial_cost, const int32_t *__restrict__ partial_index) {
  const MistGroupDesc *g = groups + blockIdx.x;
  if (g->scout_stride <= 0) return;
  const int L = prob.num_layers;
  const int S = incumbent_stage_count(prob, g);
  if (S == 0) return;
  const int l = L / S;
  const int64_t slab = (int64_t)kSlots * MIST_LC_TILE;
  // cheapest seed of the stage's (l, c) cells, c = 0..c_last, in slot `slot` of p tile `p_tile`
  auto cheapest = [&](int slot, int p_tile, int c_last) {
    double best = INFINITY;
    for (int c = threadIdx.x & 63; c <= c_last; c += 64) {
      const int pair = l * (l + 1) / 2 - 1 + c;
      const int lc_tile = pair / MIST_LC_TILE - g->lc_tile_begin;
      if (lc_tile < 0 || lc_tile >= g->n_lc_tiles) continue;
      const int64_t at = (scout_base + scout_prefix[blockIdx.x] +
                          (int64_t)(lc_tile * g->n_p_tiles + p_tile) * kScoutSplit) * slab +
                         slot * MIST_LC_TILE + pair % MIST_LC_TILE;
      if (partial_index[at] >= 0) best = fmin(best, partial_cost[at]);
    }
    for (int step = 32; step > 0; step >>= 1) best = fmin(best, __shfl_xor(best, step));
    return best;
  };
  auto c_last_of = [&](int end_layer) {
    return prob.incumbent_ckpt_rule == 0 ? min(l, L - end_layer) : l;
  };
  __shared__ double wave_sum[kIncumbentWaves], wave_largest[kIncumbentWaves];
  const int wave = threadIdx.x >> 6;
  double sum = 0.0, largest = 0.0;
  for (int s = wave; s < S; s += kIncumbentWaves) {
    const int p = S - 1 - s, end_layer = (s + 1) * l - 1;
    int slot;
    if (S == 1) slot = 2 * MIST_P_TILE + 1;
    else if (s == 0) slot = MIST_P_TILE + p % MIST_P_TILE;
    else if (s == S - 1) slot = 2 * MIST_P_TILE;
    else slot = p % MIST_P_TILE;
    const int p_tile = (S == 1 || s == S - 1) ? 0 : p / MIST_P_TILE;
    double cost;
    if (prob.incumbent_ckpt_rule == 2) {  // every layer of the stage checkpointed
      cost = INFINITY;
      if ((threadIdx.x & 63) == 0) {
        const int pair = l * (l + 1) / 2 - 1 + l;
        const int lc_tile = pair / MIST_LC_TILE - g->lc_tile_begin;
        if (lc_tile >= 0 && lc_tile < g->n_lc_tiles) {
          const int64_t at = (scout_base + scout_prefix[blockIdx.x] +
                              (int64_t)(lc_tile * g->n_p_tiles + p_tile) * kScoutSplit) * slab +
                             slot * MIST_LC_TILE + pair % MIST_LC_TILE;
          if (partial_index[at] >= 0) cost = partial_cost[at];
        }
      }
      cost = __shfl(cost, 0);
    } else {
      cost = cheapest(slot, p_tile, c_last_of(end_layer));
    }
    sum += cost;
    largest = fmax(largest, cost);
  }
  if ((threadIdx.x & 63) == 0) {
    wave_sum[wave] = sum;
    wave_largest[wave] = largest;
  }
  __syncthreads();
  sum = 0.0;
  largest = 0.0;
  for (int w = 0; w < kIncumbentWaves; ++w) {
    sum += wave_sum[w];
    largest = fmax(largest, wave_largest[w]);
  }
  const double total = sum + (double)(g->grad_accum - 1) * largest;
  // costs are not negative, and non-negative doubles order like their bit patterns
  if (threadIdx.x == 0 && total >= 0.0 && total < INFINITY)
    atomicMin(reinterpret_cast<unsigned long long *>(prob.stage_cost_incumbent),
              (unsigned long long)__double_as_longlong(total));
}

// First estimate of the same pipeline cost, formed before the scout pass so that the scout pass
// can already leave out stage costs the caller's search cannot use.  Each group evaluates about
// kEstimateRows of its gathered rows - every parallelism row of every scout pair without
// activation / optimizer offloading first, then with the next ratios - for the layer count
// l = L / S and every ckpt count, exactly as the tables would (same latency and memory code as
// the evaluate-every-cell kernel, same cells kept: c == l - 1 only at p == 0 of the base /
// with_pre tables), and keeps per stage of the pipeline the cheapest feasible cost.  Minima over
// fewer rows than the scout pass sees, so the estimate is no smaller than the scout's.
// Grid (kEstimateSplit, group); workgroup k writes its S minima to doubles [k S, (k + 1) S) of
// the group's first scout slab (free until the scout pass writes it).
constexpr int kEstimateSplit = 16;
constexpr int kEstimateRows = 1024;
constexpr int kEstimateMaxStages = 256;
static_assert(kEstimateSplit * kEstimateMaxStages <= kScoutSplit * kSlots * MIST_LC_TILE,
              "the partial minima of a group fit the scout slabs of one tile");
__device__ __forceinline__ bool estimate_runs(const MistProblem &prob, const MistGroupDesc *g,
                                              const int32_t *__restrict__ scout_prefix, int gi,
                                              int *stages) {
  if (g->scout_stride <= 0 || scout_prefix[gi + 1] - scout_prefix[gi] < kScoutSplit) return false;
  *stages = incumbent_stage_count(prob, g);
  return *stages > 0 && *stages <= kEstimateMaxStages;
}

__global__ __launch_bounds__(256) void estimate_stage_minima_kernel(
    const MistProblem prob, const MistGroupDesc *__restrict__ groups,
    const int32_t *__restrict__ scout_prefix, int64_t scout_base,
    const double *__restrict__ row_terms, double ratio, double *__restrict__ partial_cost) {
  const int gi = (int)blockIdx.y;
  const MistGroupDesc *g = groups + gi;
  int S;
  if (!estimate_runs(prob, g, scout_prefix, gi, &S)) return;
  const int L = prob.num_layers, l = L / S, rule = prob.incumbent_ckpt_rule;
  __shared__ unsigned long long stage_min[kEstimateMaxStages];
  const unsigned long long kInf = (unsigned long long)__double_as_longlong((double)INFINITY);
  for (int st = threadIdx.x; st < S; st += blockDim.x) stage_min[st] = kInf;
  __syncthreads();
  const int n_tail = g->n_oo * g->n_ao;
  const int64_t per_pair = (int64_t)g->n_par * n_tail;
  const int64_t per_tail = (int64_t)g->n_par * max(g->scout_stride, 1);
  const int64_t n_tails = min((int64_t)n_tail, max((int64_t)1, (int64_t)kEstimateRows / per_tail));
  const int64_t n_items = per_tail * n_tails * (l + 1);
  const GroupConsts k = group_consts(g);
  const double cap = prob.mem_cap_mb;
  const double G64 = (double)g->grad_accum;
  const float G32 = (float)g->grad_accum;
  const double *__restrict__ src = row_terms + g->row_offset * MIST_ROW_TERMS;
  auto offer = [&](int st, bool ok, double cost) {
    // costs are not negative, and non-negative doubles order like their bit patterns
    if (ok && cost >= 0.0 && cost < INFINITY)
      atomicMin(&stage_min[st], (unsigned long long)__double_as_longlong(cost));
  };
  for (int64_t item = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; item < n_items;
       item += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(item % (l + 1));
    const int64_t q = item / (l + 1);
    const int64_t tail = q / per_tail, rest = q - tail * per_tail;
    const int64_t pair = rest / g->n_par, par = rest - pair * g->n_par;
    if (rule == 2 && c != l) continue;  // every layer of a stage checkpointed
    if (c == l - 1) continue;  // kept at p == 0 of base / with_pre only, which no stage below reads
    const double *__restrict__ t =
        src + gathered_position(g, pair * per_pair + par * n_tail + tail) * MIST_ROW_TERMS;
    const CellLatency lat = cell_latency<true>(t, l, c, k);
    const LaneMemory mem = cell_memory(t, l, c);
    // largest ckpt count of the stage that ends with layer end_layer (rule of the caller's search)
    auto c_last = [&](int st) { return rule == 0 ? min(l, L - ((st + 1) * l - 1)) : l; };
    double peak_f, peak_b;
    mem.peaks(0, peak_f, peak_b);
    const double f_in = mem.fwd_states + g->post_states + mem.mod_saved + g->post_fwd_peak + mem.gcb;
    const double b_in = mem.bwd_states + g->post_states + mem.mod_saved + g->post_bwd_peak +
                        (c == 0 ? t[MIST_T_RD] : 0.0) + mem.gcb;
    const double pf_post = fmax(f_in, peak_f + g->post_states);
    const double pb_post = fmax(b_in, peak_b - mem.out + g->post_states) + g->post_output;
    if (S == 1) {  // single stage: the no_pp table
      const double pf_pp = pf_post + g->pre_states + g->pre_saved;
      const double pb_pp = pb_post + g->pre_states + g->pre_saved;
      offer(0, c <= c_last(0) && fmax(pf_pp, pb_pp) * t[MIST_T_MF] <= cap,
            ratio * lat.spp + lat.dpp / G64);
      continue;
    }
    // first stage: with_pre table at S - 1 pre-saved micro-batches
    offer(0, c <= c_last(0) && mem.feasible_pre(S - 1, cap, g->pre_saved, g->pre_states_and_saved),
          ratio * lat.sp + lat.dpre / G64);
    // last stage: with_post table
    offer(S - 1, c <= c_last(S - 1) && fmax(pf_post, pb_post) * mem.mf_pp <= cap,
          ratio * lat.spost + lat.dpost / G64);
    // stages between: base table at S - 1 - st pre-saved micro-batches
    const double cost_base = ratio * (double)lat.x + (double)(lat.d / G32);
    for (int st = 1; st < S - 1; ++st)
      offer(st, c <= c_last(st) && mem.feasible_base(S - 1 - st, cap), cost_base);
  }
  __syncthreads();
  const int64_t slab = (int64_t)kSlots * MIST_LC_TILE;
  double *out = partial_cost + (scout_base + scout_prefix[gi]) * slab + (int64_t)blockIdx.x * S;
  for (int st = threadIdx.x; st < S; st += blockDim.x)
    out[st] = __longlong_as_double((long long)stage_min[st]);
}

// Sum of a group's stage minima + (G - 1) x the largest (inter_tuning.py:342) into *incumbent.
__global__ __launch_bounds__(64) void estimate_combine_kernel(
    const MistProblem prob, const MistGroupDesc *__restrict__ groups,
    const int32_t *__restrict__ scout_prefix, int64_t scout_base,
    const double *__restrict__ partial_cost) {
  const int gi = (int)blockIdx.x;
  const MistGroupDesc *g = groups + gi;
  int S;
  if (!estimate_runs(prob, g, scout_prefix, gi, &S)) return;
  const int64_t slab = (int64_t)kSlots * MIST_LC_TILE;
  const double *in = partial_cost + (scout_base + scout_prefix[gi]) * slab;
  double sum = 0.0, largest = 0.0;
  for (int st = threadIdx.x; st < S; st += 64) {
    double best = INFINITY;
    for (int k = 0; k < kEstimateSplit; ++k) best = fmin(best, in[(int64_t)k * S + st]);
    sum += best;
    largest = fmax(largest, best);
  }
  for (int step = 32; step > 0; step >>= 1) {
    sum += __shfl_xor(sum, step);
    largest = fmax(largest, __shfl_xor(largest, step));
  }
  const double total = sum + (double)(g->grad_accum - 1) * largest;
  if (threadIdx.x == 0 && total >= 0.0 && total < INFINITY)
    atomicMin(reinterpret_cast<unsigned long long *>(prob.stage_cost_incumbent),
              (unsigned long long)__double_as_longlong(total));
}

// Combines the slabs of the kScoutSplit scout workgroups of every tile into the first of them,
// so that each chunk of the main launch reads one slab of seeds instead of kScoutSplit.
// Workgroup = tile; the scout slabs of tile t are scout_base + t * kScoutSplit + k.
__global__ __launch_bounds__(256) void merge_scout_kernel(int64_t scout_base, int n_scout_total,
                                                          double *__restrict__ partial_cost,
                                                          int32_t *__restrict__ partial_index) {
  const int64_t slab = (int64_t)kSlots * MIST_LC_TILE;
  const int64_t first = (scout_base + (int64_t)blockIdx.y * n_scout_total +
                         (int64_t)blockIdx.x * kScoutSplit) * slab;
  for (int e = threadIdx.x; e < (int)slab; e += blockDim.x) {
    double best = INFINITY;
    int32_t best_row = -1;
    for (int k = 0; k < kScoutSplit; ++k) {
      const int32_t row = partial_index[first + k * slab + e];
      take_min(best, best_row, row >= 0, partial_cost[first + k * slab + e], row);
    }
    partial_cost[first + e] = best;
    partial_index[first + e] = best_row;
  }
}

// ------------------------------------------------------------------------------------------
// Kernel 3: combine the chunks' (cost, row) minima, recompute the winner's stable / delta, scatter.
// One thread per (group, (l, c) pair, slot); slots as in the reduce kernel but over all p.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void finalize_kernel(
    const MistProblem prob, const MistGroupDesc *__restrict__ groups, int n_groups,
    const int32_t *__restrict__ block_prefix, const double *__restrict__ row_terms,
    const double *__restrict__ partial_cost, const int32_t *__restrict__ partial_index,
    const SampleSlots samples, int n_blocks, MistOutTables tables) {
  const int L = prob.num_layers;
  const int n_pairs = L * (L + 1) / 2 + L;
  const int gi = blockIdx.z;
  const MistGroupDesc *g = groups + gi;
  // blockIdx.x = (sample of the launch, block of 256 pairs); the slabs of the launch's m-th
  // sample start at slab m * n_blocks
  const int pair_blocks = (n_pairs + (int)blockDim.x - 1) / (int)blockDim.x;
  const int m = blockIdx.x / pair_blocks;
  const int sample_index = samples.at[m];
  const int pair_idx = (blockIdx.x - m * pair_blocks) * blockDim.x + threadIdx.x;
  // blockIdx.y: 0..p_dim-1 base, p_dim..2*p_dim-1 with_pre, 2*p_dim with_post, 2*p_dim+1 no_pp
  const int P1 = prob.p_dim;
  const int slot = blockIdx.y;
  int variant, p;
  if (slot < P1) { variant = 0; p = slot; }
  else if (slot < 2 * P1) { variant = 1; p = slot - P1; }
  else { variant = 2 + (slot - 2 * P1); p = 0; }
  if (p >= g->num_p) return;
  // A wavefront = the 64 pairs of one tile (the workgroup starts at a multiple of 256 pairs):
  // what follows up to the chunk loop is the same for all its lanes.  The group's tiles are a
  // window of the pair list; cells outside were not evaluated.
  const int lc_tile = pair_idx / MIST_LC_TILE - g->lc_tile_begin, lane = pair_idx % MIST_LC_TILE;
  if (lc_tile < 0 || lc_tile >= g->n_lc_tiles) return;
  const PairIndex pc = decode_pair(min(pair_idx, n_pairs - 1));
  const int l = pc.l, c = pc.c;
  // Cells the reference never writes (batched_module_analyzer.py:3021-3023 rebinds the layer
  // mask inside the p == 0 branch, so it also governs base / with_pre for p >= 1; :3103).
  const bool written = pair_idx < n_pairs && !(variant <= 1 && p >= 1 && c == l - 1) &&
                       !(variant == 2 && c == l - 1) && !(variant == 3 && (l != L || c == L - 1));
  const int p_tile = p / MIST_P_TILE;
  int kslot;
  if (variant == 0) kslot = p % MIST_P_TILE;
  else if (variant == 1) kslot = MIST_P_TILE + p % MIST_P_TILE;
  else kslot = 2 * MIST_P_TILE + (variant - 2);
  const int n_tiles = g->n_lc_tiles * g->n_p_tiles;
  const int64_t first_block =
      (int64_t)m * n_blocks + (int64_t)block_prefix[gi] + (lc_tile * g->n_p_tiles + p_tile);
  double best = INFINITY;
  int32_t best_row = -1;
  // Most chunks leave their seeds as they are and write a mark instead of a slab: the marks of
  // 64 chunks are read at once, a lane each, and only the slabs that were written are visited
  // (in chunk order, as a walk over all chunks would).
  for (int ch0 = 0; ch0 < g->n_chunks; ch0 += 64) {
    const int ch_mine = ch0 + (int)(threadIdx.x & 63);
    bool has_slab = false;
    if (ch_mine < g->n_chunks)
      has_slab = ch_mine == 0 ||
                 partial_index[(first_block + (int64_t)ch_mine * n_tiles) * kSlots * MIST_LC_TILE] !=
                     kSlabUnchanged;
    unsigned long long todo = __ballot(has_slab);
    while (todo != 0) {
      const int ch = ch0 + __ffsll(todo) - 1;
      todo &= todo - 1;
      const int64_t at = (first_block + (int64_t)ch * n_tiles) * kSlots * MIST_LC_TILE +
                         (int64_t)kslot * MIST_LC_TILE + lane;
      const double cost = partial_cost[at];
      const int32_t row = partial_index[at];
      take_min(best, best_row, row >= 0, cost, row);
    }
  }
  if (!written) return;

  double stable = INFINITY, delta = INFINITY;
  if (best_row >= 0) {
    const double *t = row_terms + (g->row_offset + position_of_row(g, best_row)) * MIST_ROW_TERMS;
    const CellLatency lat = cell_latency<true>(t, l, c, group_consts(g));
    if (variant == 0) { stable = (double)lat.x; delta = (double)lat.d; }
    else if (variant == 1) { stable = lat.sp; delta = lat.dpre; }
    else if (variant == 2) { stable = lat.spost; delta = lat.dpost; }
    else { stable = lat.spp; delta = lat.dpp; }
  }

  const int S = prob.sample_size;
  const int64_t gq = (int64_t)g->g_index * prob.num_mesh + g->q_index;
  int64_t at;
  if (variant <= 1) at = (((gq * P1 + p) * L + (l - 1)) * (L + 1) + c) * S + sample_index;
  else if (variant == 2) at = ((gq * L + (l - 1)) * (L + 1) + c) * S + sample_index;
  else at = (gq * (L + 1) + c) * S + sample_index;
  tables.stable[variant][at] = stable;
  tables.delta[variant][at] = delta;
  tables.index[variant][at] = best_row;
}

// ------------------------------------------------------------------------------------------
// Analysis path: the quantities batched_stage_analyze(get_best_solution=False) reports for ONE
// given strategy row and one (layers, ckpt, pre-saved micro-batches) cell
// (batched_module_analyzer.py:2788-2803, 2876-2892, 2980-2996, 3063-3079), unmasked.
// One thread per request; per variant (middle, first, last, single stage): stable latency, delta
// latency, stable + delta / G, forward peak, backward peak.
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ LaneMemory cell_memory(const double *__restrict__ t, int l, int c) {
  const double lf = (double)l, lm1 = (double)max(l - 1, 0), cf = (double)c;
  const double S_ck = t[MIST_T_S_CK], S_nock = t[MIST_T_S_NOCK];
  LaneMemory mem;
  mem.fwd_states = t[MIST_T_FWD_STATES0] + lf * t[MIST_T_PWG] + lm1 * t[MIST_T_PO];  // :2150-2162
  mem.bwd_states = t[MIST_T_BWD_STATES0] + lf * t[MIST_T_PWGO];
  mem.cur_saved = c == l ? (lf - 1.0) * S_ck : cf * S_ck + (double)(l - c - 1) * S_nock;  // :2358-2385
  mem.mod_saved = S_ck * cf + S_nock * (double)(l - c);
  mem.ck_delta = c >= l - 1 ? t[MIST_T_D_CK] : t[MIST_T_D_NOCK];  // :2760-2769
  mem.fwd_pk = t[MIST_T_FWD_PEAK];
  mem.bwd_pk = t[MIST_T_BWD_PEAK];
  mem.out = t[MIST_T_OUT];
  mem.gcb = t[MIST_T_GCB];
  mem.mf_base = t[MIST_T_MF_BASE];
  mem.mf_pp = t[MIST_T_MF_PP];
  return mem;
}

__global__ __launch_bounds__(64) void analyze_kernel(
    const MistProblem prob, const MistGroupDesc *__restrict__ groups, int n_groups,
    const double *__restrict__ row_terms, const int32_t *__restrict__ requests, int n_requests,
    double *__restrict__ out) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_requests) return;
  const int32_t *req = requests + (int64_t)i * MIST_ANALYZE_REQUEST_FIELDS;
  double *o = out + (int64_t)i * MIST_ANALYZE_FIELDS;
  const int gi = req[0], l = req[2], c = req[3], p = req[4];
  const int64_t pos = req[1];
  const bool ok = gi >= 0 && gi < n_groups && l >= 1 && l <= prob.num_layers && c >= 0 && c <= l &&
                  p >= 0 && pos >= 0 && pos < groups[min(max(gi, 0), n_groups - 1)].n_rows;
  if (!ok) {
    for (int f = 0; f < MIST_ANALYZE_FIELDS; ++f) o[f] = NAN;
    return;
  }
  const MistGroupDesc *g = groups + gi;
  const double *t = row_terms + (g->row_offset + pos) * MIST_ROW_TERMS;
  const GroupConsts k = group_consts(g);
  const CellLatency lat = cell_latency<true>(t, l, c, k);
  const LaneMemory mem = cell_memory(t, l, c);
  const double G64 = (double)g->grad_accum;
  const float G32 = (float)g->grad_accum;
  double peak_f, peak_b;
  mem.peaks(p, peak_f, peak_b);
  // middle stage: float32 stable + float32 delta / G stays float32 (:2212-2216)
  o[0] = (double)lat.x;
  o[1] = (double)lat.d;
  o[2] = (double)(lat.x + lat.d / G32);
  o[3] = peak_f;
  o[4] = peak_b;
  // first stage (:2866-2875)
  const double pre_p = (double)p * g->pre_saved;
  o[5] = lat.sp;
  o[6] = lat.dpre;
  o[7] = lat.sp + lat.dpre / G64;
  o[8] = pre_p + peak_f + g->pre_states_and_saved;
  o[9] = pre_p + peak_b + g->pre_states_and_saved;
  // last stage (:2946-2979); the reference evaluates it for p == 0 only
  const double f_in =
      mem.fwd_states + g->post_states + mem.mod_saved + g->post_fwd_peak + mem.gcb;
  const double b_in = mem.bwd_states + g->post_states + mem.mod_saved + g->post_bwd_peak +
                      (c == 0 ? t[MIST_T_RD] : 0.0) + mem.gcb;
  const double pf_post = fmax(f_in, peak_f + g->post_states);
  const double pb_post = fmax(b_in, peak_b - mem.out + g->post_states) + g->post_output;
  o[10] = lat.spost;
  o[11] = lat.dpost;
  o[12] = lat.spost + lat.dpost / G64;
  o[13] = pf_post;
  o[14] = pb_post;
  // single stage (:3057-3062)
  o[15] = lat.spp;
  o[16] = lat.dpp;
  o[17] = lat.spp + lat.dpp / G64;
  o[18] = pf_post + g->pre_states + g->pre_saved;
  o[19] = pb_post + g->pre_states + g->pre_saved;
  // module-level memory of the cell (:2150-2162, 2378-2383), reported by get_extra_info
  o[20] = mem.fwd_states;
  o[21] = mem.bwd_states;
  o[22] = mem.mod_saved;
}

// The intermediate quantities of one candidate row that the row terms fold together: what the
// reference's get_extra_info (:2401-2749) reports besides them.  Thread = request = (group,
// workspace position); the same device functions as row_terms_kernel, every row on its own.
__global__ __launch_bounds__(kTermsBlock) void row_diagnostics_kernel(
    const MistProblem prob, const MistGroupDesc *__restrict__ groups, int n_groups,
    const int32_t *__restrict__ requests, int n_requests, double *__restrict__ out) {
  __shared__ __align__(16) double lds_factor[11][kFactorPitch];
  __shared__ double lds_gpu_gpu[32];
  InterferenceModel<false> I;
  I.factors_tame = load_model_tables(prob, lds_factor, lds_gpu_gpu);
  I.table = (LdsDouble *)&lds_factor[0][0];
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int i_safe = min(i, n_requests - 1);  // no early exit: the model's wave-wide test wants every lane
  const int32_t *req = requests + (int64_t)i_safe * 2;
  const int gi = req[0];
  const int64_t pos = req[1];
  const bool ok = gi >= 0 && gi < n_groups && pos >= 0 && pos < groups[min(max(gi, 0), n_groups - 1)].n_rows;
  const MistGroupDesc *g = groups + (ok ? gi : 0);
  const RowParts parts = parts_of_position(g, ok ? pos : 0);
  const double wo = g->wo[g->pair_wo[parts.pair]], go = g->go[g->pair_go[parts.pair]];
  const double oo = g->oo[parts.oo], ao = g->ao[parts.ao];
  const double *par = g->par[parts.par];
  const double dp = par[MIST_PAR_DP], wre = par[MIST_PAR_WRE], gre = par[MIST_PAR_GRE];
  const double ore = par[MIST_PAR_ORE], W = par[MIST_PAR_W], Gr = par[MIST_PAR_G], O = par[MIST_PAR_O];
  const double wre_size = wre == 1.0 ? dp : 1.0, gre_size = gre == 1.0 ? dp : 1.0;
  const double ore_size = ore == 1.0 ? dp : 1.0;
  const KeyInputs in = key_inputs(prob, lds_gpu_gpu, g, par, wo, go, ao);
  const double so_O = host_link_latency(prob.gpu_cpu, O / ore_size * oo);
  const double si_O = host_link_latency(prob.cpu_gpu, O / ore_size * oo);
  const bool adv = prob.adv_first_block != 0;
  Family fam[8];  // forward first / later micro-batch, backward last / not last; nock, ck each
#pragma unroll
  for (int ph = 0; ph < 2; ++ph) {
    const FwdOperands op = fwd_operands(in, ph == 0, so_O, si_O);
    double first, extra_pre;
    fwd_common(I, in, op, ph == 0, adv, first, extra_pre);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      Family &f = fam[ph * 2 + k];
      f.first = first;
      f.extra_pre = extra_pre;
      fwd_of_ckpt(I, in, op, k != 0, f.layer, f.last, f.extra_post);
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) fam[4 + j] = bwd_family(I, in, (j & 2) != 0, (j & 1) != 0);
  if (i >= n_requests) return;
  double *o = out + (int64_t)i * MIST_DIAG_FIELDS;
  if (!ok) {
    for (int f = 0; f < MIST_DIAG_FIELDS; ++f) o[f] = NAN;
    return;
  }
  const bool wbuf_on = wre_size > 1.0 || g->pp_wre == 1 || wo > 0.0;
  const bool gbuf_on = gre_size > 1.0 || g->pp_gre == 1 || go > 0.0;
  const FwdOperands f0 = fwd_operands(in, true, so_O, si_O), f1 = fwd_operands(in, false, 0.0, 0.0);
  o[MIST_DG_SO_W] = in.so_W;
  o[MIST_DG_SI_W] = in.si_W;
  o[MIST_DG_SO_G] = in.so_G;
  o[MIST_DG_SI_G] = in.si_G;
  o[MIST_DG_SO_O] = so_O;
  o[MIST_DG_SI_O] = si_O;
  o[MIST_DG_SO_A_CK] = in.so_A_ck;
  o[MIST_DG_SI_A_CK] = in.si_A_ck;
  o[MIST_DG_SO_A_NOCK] = in.so_A_nock;
  o[MIST_DG_SI_A_NOCK] = in.si_A_nock;
  o[MIST_DG_AG_W] = in.AG_w;
  o[MIST_DG_RS_G] = in.RS_g;
  o[MIST_DG_AR_G] = in.AR_g;
  o[MIST_DG_WBUF] = wbuf_on ? fmax(fmax(g->pre_full_w, g->post_full_w), W) : 0.0;
  o[MIST_DG_GBUF] = gbuf_on ? fmax(fmax(g->pre_full_g, g->post_full_g), Gr) : 0.0;
  o[MIST_DG_PW] = W / wre_size * (1.0 - wo);
  o[MIST_DG_PG] = Gr / gre_size * (1.0 - go);
  o[MIST_DG_G2C_F0] = f0.g2c;
  o[MIST_DG_C2G_F0] = f0.c2g;
  o[MIST_DG_G2G_F0] = f0.g2g;
  o[MIST_DG_G2C_F1] = f1.g2c;
  o[MIST_DG_C2G_F1] = f1.c2g;
  o[MIST_DG_G2G_F1] = f1.g2g;
  o[MIST_DG_G2C_B] = in.g2c_B;
  o[MIST_DG_C2G_B] = in.c2g_B;
  o[MIST_DG_G2G_B0] = in.g2g_B[0];
  o[MIST_DG_G2G_B1] = in.g2g_B[1];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    double *f = o + MIST_DG_FAMILIES + j * 5;
    f[0] = fam[j].layer;
    f[1] = fam[j].first;
    f[2] = fam[j].last;
    f[3] = fam[j].extra_pre;
    f[4] = fam[j].extra_post;
  }
}

int check_factors(const MistProblem *problem) {
  for (int m = 0; m < 11; ++m)
    for (int i = 0; i < 4; ++i) {
      const double f = problem->interf_factor[m][i];
      // the kernel takes 0 / f == +0 for granted
      if (!(f > 0.0) || std::isinf(f))
        return fail(MIST_E_INVALID, "interference factor [%d][%d] must be positive and finite", m, i);
    }
  return 0;
}

int check_common(const void *d_problem, const void *d_groups, int n_groups) {
  if (!d_problem || !d_groups) return fail(MIST_E_INVALID, "null problem / group pointer");
  if (n_groups <= 0) return fail(MIST_E_INVALID, "n_groups must be positive, got %d", n_groups);
  const MistProblem *problem = static_cast<const MistProblem *>(d_problem);
  if (problem->stage_cost_incumbent != nullptr) {
    if (problem->sample_size != 1)
      return fail(MIST_E_INVALID, "a stage-cost incumbent needs sample_size 1, got %d",
                  problem->sample_size);
    if (problem->incumbent_num_devices < 1 || problem->incumbent_ckpt_rule < 0 ||
        problem->incumbent_ckpt_rule > 2)
      return fail(MIST_E_INVALID, "stage-cost incumbent with %d devices, ckpt rule %d",
                  problem->incumbent_num_devices, problem->incumbent_ckpt_rule);
  }
  return 0;
}

}  // namespace

extern "C" {

const char *mist_version(void) { return "mist_search 0.1 (gfx950)"; }
const char *mist_last_error(void) { return g_last_error; }
int mist_sizeof_problem(void) { return (int)sizeof(MistProblem); }
int mist_sizeof_group(void) { return (int)sizeof(MistGroupDesc); }
int mist_reduce_p_tile(void) { return MIST_P_TILE; }
double mist_incumbent_slack(void) { return kIncumbentSlack; }

// key_terms_kernel over every group when the caller gave a key-term workspace and the bound the
// grid needs; *launched tells whether the row-term kernel can read key terms.
static int launch_key_terms(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                            double *d_key_terms, hipStream_t stream, bool *launched) {
  *launched = d_key_terms != nullptr && problem->max_group_keys > 0 && n_groups <= 65535;
  if (!*launched) return 0;
  constexpr int kKeysPerBlock = kTermsBlock / 4;
  const unsigned blocks = (unsigned)((problem->max_group_keys + kKeysPerBlock - 1) / kKeysPerBlock);
  hipLaunchKernelGGL(key_terms_kernel, dim3(blocks, n_groups), dim3(kTermsBlock), 0, stream, *problem,
                     d_groups, d_key_terms);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int mist_row_terms(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                   const int32_t *d_block_prefix, int n_blocks, double *d_row_terms,
                   double *d_stage_floor, double *d_key_terms, void *stream) {
  if (int rc = check_common(problem, d_groups, n_groups)) return rc;
  if (!d_block_prefix || !d_row_terms || !d_stage_floor)
    return fail(MIST_E_INVALID, "null workspace pointer");
  if (n_blocks <= 0) return fail(MIST_E_INVALID, "n_blocks must be positive, got %d", n_blocks);
  if (int rc = check_factors(problem)) return rc;
  bool from_keys = false;
  if (int rc = launch_key_terms(problem, d_groups, n_groups, d_key_terms, (hipStream_t)stream, &from_keys))
    return rc;
  if (from_keys)
    hipLaunchKernelGGL((row_terms_kernel<0, true>), dim3(n_blocks), dim3(kTermsBlock), 0,
                       (hipStream_t)stream, *problem, d_groups, n_groups, d_block_prefix, d_row_terms,
                       d_stage_floor, d_key_terms);
  else
    hipLaunchKernelGGL((row_terms_kernel<0, false>), dim3(n_blocks), dim3(kTermsBlock), 0,
                       (hipStream_t)stream, *problem, d_groups, n_groups, d_block_prefix, d_row_terms,
                       d_stage_floor, nullptr);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int64_t mist_key_terms_doubles(int64_t total_keys) {
  return total_keys < 0 ? -1 : total_keys * MIST_KEY_TERMS;
}

int mist_reduce_stage_rows(void) { return kStageRows; }
int mist_reduce_lc_tile(void) { return MIST_LC_TILE; }
int mist_terms_block_rows(void) { return kTermsBlock; }
int mist_reduce_scout_split(void) { return kScoutSplit; }
int mist_workspace_oo_tile(void) { return kOoTile; }
int mist_max_sample_batch(void) { return MIST_MAX_SAMPLE_BATCH; }
int mist_key_terms_per_key(void) { return MIST_KEY_TERMS; }
int mist_max_scout_pairs(void) { return MIST_MAX_SCOUT_PAIRS; }
int64_t mist_stage_floor_doubles(int64_t total_rows, int n_groups) {
  if (total_rows < 0 || n_groups < 0) return -1;
  return (total_rows / kStageRows + n_groups + 1) * kStageFloorPitch;
}

static int launch_first_estimate(const MistProblem *problem, const MistGroupDesc *d_groups,
                                 int n_groups, const int32_t *scout_prefix, int64_t scout_base,
                                 const double *d_row_terms, double ratio, double *d_partial_cost,
                                 void *stream) {
  hipLaunchKernelGGL(estimate_stage_minima_kernel, dim3(kEstimateSplit, n_groups), dim3(256), 0,
                     (hipStream_t)stream, *problem, d_groups, scout_prefix, scout_base, d_row_terms,
                     ratio, d_partial_cost);
  MIST_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL(estimate_combine_kernel, dim3(n_groups), dim3(64), 0, (hipStream_t)stream,
                     *problem, d_groups, scout_prefix, scout_base, d_partial_cost);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

// Scout launch + slab merge for n_samples ratios at once (grid.y = sample).
static int launch_scout(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                        const int32_t *d_block_prefix, int n_blocks, const int32_t *scout_prefix,
                        int n_scout_blocks, const double *d_row_terms, const double *d_stage_floor,
                        const RatioList &ratios, int n_samples, int64_t scout_base,
                        double *d_partial_cost, int32_t *d_partial_index, void *stream) {
  if (n_scout_blocks % kScoutSplit != 0)
    return fail(MIST_E_INVALID, "n_scout_blocks %d is not a multiple of the scout split %d",
                n_scout_blocks, kScoutSplit);
  if (problem->stage_cost_incumbent != nullptr && problem->incumbent_first_estimate != 0 &&
      n_samples == 1 && n_groups <= 65535)
    // a first estimate from a few rows, so that the scout pass itself runs under a bound
    if (int rc = launch_first_estimate(problem, d_groups, n_groups, scout_prefix, scout_base,
                                       d_row_terms, ratios.r[0], d_partial_cost, stream))
      return rc;
  hipLaunchKernelGGL(eval_reduce_kernel, dim3(xcd_padded_grid(n_scout_blocks), n_samples),
                     dim3(MIST_LC_TILE), 0, (hipStream_t)stream, *problem, d_groups, n_groups,
                     d_block_prefix, n_blocks, scout_prefix, 1, d_row_terms, d_stage_floor, ratios,
                     0, scout_base, d_partial_cost, d_partial_index);
  MIST_HIP_CHECK(hipGetLastError());
  if (kScoutSplit > 1) {
    hipLaunchKernelGGL(merge_scout_kernel, dim3(n_scout_blocks / kScoutSplit, n_samples), dim3(256),
                       0, (hipStream_t)stream, scout_base, n_scout_blocks, d_partial_cost,
                       d_partial_index);
    MIST_HIP_CHECK(hipGetLastError());
  }
  if (problem->stage_cost_incumbent != nullptr && n_samples == 1) {
    hipLaunchKernelGGL(incumbent_kernel, dim3(n_groups), dim3(64 * kIncumbentWaves), 0,
                       (hipStream_t)stream, *problem,
                       d_groups, scout_prefix, scout_base, d_partial_cost, d_partial_index);
    MIST_HIP_CHECK(hipGetLastError());
  }
  return 0;
}

static int check_reduce_arguments(const MistProblem *problem, const MistGroupDesc *d_groups,
                                  int n_groups, const int32_t *d_block_prefix, int n_blocks,
                                  const int32_t *d_scout_prefix, int n_scout_blocks,
                                  const double *d_row_terms, const double *d_stage_floor,
                                  const double *d_partial_cost, const int32_t *d_partial_index) {
  if (int rc = check_common(problem, d_groups, n_groups)) return rc;
  if (!d_block_prefix || !d_row_terms || !d_stage_floor || !d_partial_cost || !d_partial_index)
    return fail(MIST_E_INVALID, "null workspace pointer");
  if (n_blocks <= 0) return fail(MIST_E_INVALID, "n_blocks must be positive, got %d", n_blocks);
  if (n_scout_blocks < 0 || (n_scout_blocks > 0 && !d_scout_prefix))
    return fail(MIST_E_INVALID, "scout blocks need a scout prefix (n_scout_blocks=%d)",
                n_scout_blocks);
  return 0;
}

int mist_eval_reduce(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                     const int32_t *d_block_prefix, int n_blocks,
                     const int32_t *d_scout_prefix, int n_scout_blocks,
                     const double *d_row_terms, const double *d_stage_floor, double ratio,
                     double *d_partial_cost, int32_t *d_partial_index, void *stream) {
  if (int rc = check_reduce_arguments(problem, d_groups, n_groups, d_block_prefix, n_blocks,
                                      d_scout_prefix, n_scout_blocks, d_row_terms, d_stage_floor,
                                      d_partial_cost, d_partial_index))
    return rc;
  if (!(ratio >= 0.0)) return fail(MIST_E_INVALID, "ratio must be non-negative");
  const int32_t *scout_prefix = n_scout_blocks > 0 ? d_scout_prefix : nullptr;
  RatioList ratios = {};
  ratios.r[0] = ratio;
  if (scout_prefix)
    if (int rc = launch_scout(problem, d_groups, n_groups, d_block_prefix, n_blocks, scout_prefix,
                              n_scout_blocks, d_row_terms, d_stage_floor, ratios, 1, n_blocks,
                              d_partial_cost, d_partial_index, stream))
      return rc;
  hipLaunchKernelGGL(eval_reduce_kernel, dim3(xcd_padded_grid(n_blocks)), dim3(MIST_LC_TILE), 0,
                     (hipStream_t)stream, *problem, d_groups, n_groups, d_block_prefix, n_blocks,
                     scout_prefix, 0, d_row_terms, d_stage_floor, ratios, 0, (int64_t)n_blocks,
                     d_partial_cost, d_partial_index);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int mist_stage_cost_first_estimate(const MistProblem *problem, const MistGroupDesc *d_groups,
                                   int n_groups, const int32_t *d_scout_prefix, int n_blocks,
                                   const double *d_row_terms, double ratio, double *d_partial_cost,
                                   void *stream) {
  if (int rc = check_common(problem, d_groups, n_groups)) return rc;
  if (!d_scout_prefix || !d_row_terms || !d_partial_cost)
    return fail(MIST_E_INVALID, "null workspace pointer");
  if (n_blocks < 0) return fail(MIST_E_INVALID, "n_blocks must not be negative, got %d", n_blocks);
  if (problem->stage_cost_incumbent == nullptr)
    return fail(MIST_E_INVALID, "no stage-cost incumbent to lower");
  if (n_groups > 65535) return fail(MIST_E_INVALID, "at most 65535 groups per call, got %d", n_groups);
  if (!(ratio >= 0.0)) return fail(MIST_E_INVALID, "ratio must be non-negative");
  return launch_first_estimate(problem, d_groups, n_groups, d_scout_prefix, (int64_t)n_blocks,
                               d_row_terms, ratio, d_partial_cost, stream);
}

static int launch_finalize(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                           const int32_t *d_block_prefix, const double *d_row_terms,
                           const double *d_partial_cost, const int32_t *d_partial_index,
                           const int32_t *sample_index, int n_samples, int n_blocks,
                           const MistOutTables *tables, void *stream);

int mist_eval_reduce_samples(const MistProblem *problem, const MistGroupDesc *d_groups,
                             int n_groups, const int32_t *d_block_prefix, int n_blocks,
                             const int32_t *d_scout_prefix, int n_scout_blocks,
                             const double *d_row_terms, const double *d_stage_floor,
                             const double *ratios, const int32_t *sample_index, int n_samples,
                             int main_batch, double *d_partial_cost, int32_t *d_partial_index,
                             const MistOutTables *tables, void *stream) {
  if (int rc = check_reduce_arguments(problem, d_groups, n_groups, d_block_prefix, n_blocks,
                                      d_scout_prefix, n_scout_blocks, d_row_terms, d_stage_floor,
                                      d_partial_cost, d_partial_index))
    return rc;
  if (!ratios || !sample_index || n_samples < 1 || n_samples > MIST_MAX_SAMPLE_BATCH)
    return fail(MIST_E_INVALID, "n_samples %d outside [1, %d] or null sample lists", n_samples,
                MIST_MAX_SAMPLE_BATCH);
  if (main_batch < 1 || main_batch > n_samples)
    return fail(MIST_E_INVALID, "main_batch %d outside [1, n_samples = %d]", main_batch, n_samples);
  RatioList all = {};
  for (int i = 0; i < n_samples; ++i) {
    if (!(ratios[i] >= 0.0)) return fail(MIST_E_INVALID, "ratio %d must be non-negative", i);
    all.r[i] = ratios[i];
  }
  const int32_t *scout_prefix = n_scout_blocks > 0 ? d_scout_prefix : nullptr;
  const int64_t scout_base = (int64_t)main_batch * n_blocks;
  // the scout passes of all samples in one launch: a single one occupies a tenth of the GPU
  if (scout_prefix)
    if (int rc = launch_scout(problem, d_groups, n_groups, d_block_prefix, n_blocks, scout_prefix,
                              n_scout_blocks, d_row_terms, d_stage_floor, all, n_samples, scout_base,
                              d_partial_cost, d_partial_index, stream))
      return rc;
  // main launches and finalize launches of main_batch samples at a time (grid.y = sample): the
  // tail of one sample's wavefronts runs beside the next sample's
  for (int first = 0; first < n_samples; first += main_batch) {
    const int count = std::min(main_batch, n_samples - first);
    hipLaunchKernelGGL(eval_reduce_kernel, dim3(xcd_padded_grid(n_blocks), count), dim3(MIST_LC_TILE),
                       0, (hipStream_t)stream, *problem, d_groups, n_groups, d_block_prefix, n_blocks,
                       scout_prefix, 0, d_row_terms, d_stage_floor, all, first, scout_base,
                       d_partial_cost, d_partial_index);
    MIST_HIP_CHECK(hipGetLastError());
    if (int rc = launch_finalize(problem, d_groups, n_groups, d_block_prefix, d_row_terms,
                                 d_partial_cost, d_partial_index, sample_index + first, count,
                                 n_blocks, tables, stream))
      return rc;
  }
  return 0;
}

int mist_eval_reduce_exhaustive(const MistProblem *problem, const MistGroupDesc *d_groups,
                                int n_groups, const int32_t *d_block_prefix, int n_blocks,
                                const double *d_row_terms, double ratio, double *d_partial_cost,
                                int32_t *d_partial_index, void *stream) {
  if (int rc = check_common(problem, d_groups, n_groups)) return rc;
  if (!d_block_prefix || !d_row_terms || !d_partial_cost || !d_partial_index)
    return fail(MIST_E_INVALID, "null workspace pointer");
  if (n_blocks <= 0) return fail(MIST_E_INVALID, "n_blocks must be positive, got %d", n_blocks);
  if (!(ratio >= 0.0)) return fail(MIST_E_INVALID, "ratio must be non-negative");
  hipLaunchKernelGGL(eval_reduce_exhaustive_kernel, dim3(xcd_padded_grid(n_blocks)),
                     dim3(MIST_LC_TILE), 0, (hipStream_t)stream, *problem, d_groups, n_groups,
                     d_block_prefix, n_blocks, d_row_terms, ratio, d_partial_cost, d_partial_index);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

static int launch_finalize(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                           const int32_t *d_block_prefix, const double *d_row_terms,
                           const double *d_partial_cost, const int32_t *d_partial_index,
                           const int32_t *sample_index, int n_samples, int n_blocks,
                           const MistOutTables *tables, void *stream) {
  if (int rc = check_common(problem, d_groups, n_groups)) return rc;
  if (!d_block_prefix || !d_row_terms || !d_partial_cost || !d_partial_index || !tables)
    return fail(MIST_E_INVALID, "null pointer argument");
  for (int v = 0; v < 4; ++v)
    if (!tables->stable[v] || !tables->delta[v] || !tables->index[v])
      return fail(MIST_E_INVALID, "output table %d is null", v);
  const MistProblem &prob = *problem;
  const int L = prob.num_layers, P1 = prob.p_dim;
  if (L <= 0 || P1 <= 0 || prob.sample_size <= 0)
    return fail(MIST_E_INVALID, "bad problem extents L=%d P+1=%d S=%d", L, P1, prob.sample_size);
  SampleSlots slots = {};
  for (int i = 0; i < n_samples; ++i) {
    if (sample_index[i] < 0 || sample_index[i] >= prob.sample_size)
      return fail(MIST_E_INVALID, "sample_index %d outside [0, %d)", sample_index[i], prob.sample_size);
    slots.at[i] = sample_index[i];
  }
  if (n_groups > 65535) return fail(MIST_E_INVALID, "too many groups for one launch: %d", n_groups);
  const int n_pairs = L * (L + 1) / 2 + L;
  dim3 grid((n_pairs + 255) / 256 * n_samples, 2 * P1 + 2, n_groups);
  hipLaunchKernelGGL(finalize_kernel, grid, dim3(256), 0, (hipStream_t)stream, prob, d_groups,
                     n_groups, d_block_prefix, d_row_terms, d_partial_cost, d_partial_index, slots,
                     n_blocks, *tables);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int mist_finalize(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                  const int32_t *d_block_prefix, const double *d_row_terms,
                  const double *d_partial_cost, const int32_t *d_partial_index,
                  int sample_index, const MistOutTables *tables, void *stream) {
  return launch_finalize(problem, d_groups, n_groups, d_block_prefix, d_row_terms, d_partial_cost,
                         d_partial_index, &sample_index, 1, 0, tables, stream);
}

// Second stream and events of mist_intra_stage_eval, one set per device, kept for the life of
// the process.
namespace {
struct OverlapStreams {
  hipStream_t side = nullptr;
  hipEvent_t rows_ready = nullptr, scout_done = nullptr, main_done = nullptr;
};
std::mutex g_enqueue_lock;  // one call's records and waits on the shared events are a unit
int overlap_streams(OverlapStreams **out) {
  static std::mutex lock;
  static OverlapStreams known[64];
  int device = 0;
  MIST_HIP_CHECK(hipGetDevice(&device));
  if (device < 0 || device >= 64) return fail(MIST_E_INVALID, "device ordinal %d outside [0, 64)", device);
  std::lock_guard<std::mutex> guard(lock);
  OverlapStreams &s = known[device];
  if (s.side == nullptr) {
    MIST_HIP_CHECK(hipStreamCreateWithFlags(&s.side, hipStreamNonBlocking));  // default priority
    MIST_HIP_CHECK(hipEventCreateWithFlags(&s.rows_ready, hipEventDisableTiming));
    MIST_HIP_CHECK(hipEventCreateWithFlags(&s.scout_done, hipEventDisableTiming));
    MIST_HIP_CHECK(hipEventCreateWithFlags(&s.main_done, hipEventDisableTiming));
  }
  *out = &s;
  return 0;
}
}  // namespace

int mist_intra_stage_eval(const MistProblem *problem, const MistGroupDesc *d_groups,
                          int n_groups, const int32_t *d_terms_block_prefix, int n_terms_blocks,
                          const int32_t *d_reduce_block_prefix, int n_reduce_blocks,
                          const int32_t *d_scout_prefix, int n_scout_blocks, double *d_row_terms,
                          double *d_stage_floor, double *d_key_terms, double *d_partial_cost,
                          int32_t *d_partial_index, double ratio, int sample_index,
                          int compute_terms, const MistOutTables *tables, void *stream) {
  if (compute_terms && n_scout_blocks > 0 && problem != nullptr && problem->max_scout_rows > 0 &&
      n_groups > 0 && n_groups <= 65535) {
    // The scout pass reads a few hundred rows per group and leaves most of the GPU idle; the row
    // terms of everything else are computed beside it.  Stream order: [terms of the gathered
    // rows] -> side stream: scout pass + merge || this stream: all other row terms -> main
    // launch -> finalize.
    if (int rc = check_reduce_arguments(problem, d_groups, n_groups, d_reduce_block_prefix,
                                        n_reduce_blocks, d_scout_prefix, n_scout_blocks,
                                        d_row_terms, d_stage_floor, d_partial_cost, d_partial_index))
      return rc;
    if (!d_terms_block_prefix || n_terms_blocks <= 0)
      return fail(MIST_E_INVALID, "null / empty row-term decomposition");
    if (int rc = check_factors(problem)) return rc;
    if (!(ratio >= 0.0)) return fail(MIST_E_INVALID, "ratio must be non-negative");
    OverlapStreams *os = nullptr;
    if (int rc = overlap_streams(&os)) return rc;
    // the second stream and its events are shared by all callers: one call's records and waits
    // are enqueued as a unit
    std::lock_guard<std::mutex> enqueue_guard(g_enqueue_lock);
    hipStream_t main_stream = (hipStream_t)stream;
    const unsigned scout_term_blocks = (unsigned)((problem->max_scout_rows + kTermsBlock - 1) / kTermsBlock);
    hipLaunchKernelGGL((row_terms_kernel<1, false>), dim3(scout_term_blocks, n_groups),
                       dim3(kTermsBlock), 0, main_stream, *problem, d_groups, n_groups,
                       d_terms_block_prefix, d_row_terms, d_stage_floor, nullptr);
    MIST_HIP_CHECK(hipGetLastError());
    MIST_HIP_CHECK(hipEventRecord(os->rows_ready, main_stream));
    MIST_HIP_CHECK(hipStreamWaitEvent(os->side, os->rows_ready, 0));
    // (the other row terms are queued first: the scout pass is five launches, and this stream
    // would idle while they are made)
    bool from_keys = false;
    if (int rc = launch_key_terms(problem, d_groups, n_groups, d_key_terms, main_stream, &from_keys))
      return rc;
    if (from_keys)
      hipLaunchKernelGGL((row_terms_kernel<2, true>), dim3(n_terms_blocks), dim3(kTermsBlock), 0,
                         main_stream, *problem, d_groups, n_groups, d_terms_block_prefix, d_row_terms,
                         d_stage_floor, d_key_terms);
    else
      hipLaunchKernelGGL((row_terms_kernel<2, false>), dim3(n_terms_blocks), dim3(kTermsBlock), 0,
                         main_stream, *problem, d_groups, n_groups, d_terms_block_prefix, d_row_terms,
                         d_stage_floor, nullptr);
    MIST_HIP_CHECK(hipGetLastError());
    RatioList ratios = {};
    ratios.r[0] = ratio;
    if (int rc = launch_scout(problem, d_groups, n_groups, d_reduce_block_prefix, n_reduce_blocks,
                              d_scout_prefix, n_scout_blocks, d_row_terms, d_stage_floor, ratios, 1,
                              n_reduce_blocks, d_partial_cost, d_partial_index, os->side))
      return rc;
    MIST_HIP_CHECK(hipEventRecord(os->scout_done, os->side));
    MIST_HIP_CHECK(hipStreamWaitEvent(main_stream, os->scout_done, 0));
    hipLaunchKernelGGL(eval_reduce_kernel, dim3(xcd_padded_grid(n_reduce_blocks)), dim3(MIST_LC_TILE),
                       0, main_stream, *problem, d_groups, n_groups, d_reduce_block_prefix,
                       n_reduce_blocks, d_scout_prefix, 0, d_row_terms, d_stage_floor, ratios, 0,
                       (int64_t)n_reduce_blocks, d_partial_cost, d_partial_index);
    MIST_HIP_CHECK(hipGetLastError());
    return mist_finalize(problem, d_groups, n_groups, d_reduce_block_prefix, d_row_terms,
                         d_partial_cost, d_partial_index, sample_index, tables, stream);
  }
  if (compute_terms) {
    if (int rc = mist_row_terms(problem, d_groups, n_groups, d_terms_block_prefix,
                                n_terms_blocks, d_row_terms, d_stage_floor, d_key_terms, stream))
      return rc;
  }
  if (int rc = mist_eval_reduce(problem, d_groups, n_groups, d_reduce_block_prefix,
                                n_reduce_blocks, d_scout_prefix, n_scout_blocks, d_row_terms,
                                d_stage_floor, ratio, d_partial_cost, d_partial_index, stream))
    return rc;
  return mist_finalize(problem, d_groups, n_groups, d_reduce_block_prefix, d_row_terms,
                       d_partial_cost, d_partial_index, sample_index, tables, stream);
}

int mist_intra_stage_eval_samples(const MistProblem *problem, const MistGroupDesc *d_groups,
                                  int n_groups, const int32_t *d_terms_block_prefix,
                                  int n_terms_blocks, const int32_t *d_reduce_block_prefix,
                                  int n_reduce_blocks, const int32_t *d_scout_prefix,
                                  int n_scout_blocks, double *d_row_terms, double *d_stage_floor,
                                  double *d_key_terms, double *d_partial_cost,
                                  int32_t *d_partial_index, const double *ratios,
                                  const int32_t *sample_index, int n_samples, int sample_batch,
                                  int main_batch, const MistOutTables *tables, void *stream) {
  if (!ratios || !sample_index || n_samples < 1)
    return fail(MIST_E_INVALID, "n_samples %d < 1 or null sample lists", n_samples);
  if (sample_batch < 1 || sample_batch > MIST_MAX_SAMPLE_BATCH)
    return fail(MIST_E_INVALID, "sample_batch %d outside [1, %d]", sample_batch, MIST_MAX_SAMPLE_BATCH);
  if (main_batch < 1 || main_batch > sample_batch)
    return fail(MIST_E_INVALID, "main_batch %d outside [1, sample_batch = %d]", main_batch, sample_batch);
  const bool overlap = n_scout_blocks > 0 && problem != nullptr && problem->max_scout_rows > 0 &&
                       n_groups > 0 && n_groups <= 65535;
  if (!overlap) {
    if (int rc = mist_row_terms(problem, d_groups, n_groups, d_terms_block_prefix, n_terms_blocks,
                                d_row_terms, d_stage_floor, d_key_terms, stream))
      return rc;
    for (int first = 0; first < n_samples; first += sample_batch) {
      const int count = std::min(sample_batch, n_samples - first);
      if (int rc = mist_eval_reduce_samples(problem, d_groups, n_groups, d_reduce_block_prefix,
                                            n_reduce_blocks, d_scout_prefix, n_scout_blocks,
                                            d_row_terms, d_stage_floor, ratios + first,
                                            sample_index + first, count, std::min(main_batch, count),
                                            d_partial_cost, d_partial_index, tables, stream))
        return rc;
    }
    return 0;
  }
  // Stream order: [terms of the gathered rows] -> side stream: scout pass of the first batch of
  // samples || this stream: all other row terms -> per batch b: side stream: scout pass of batch
  // b + 1 (into the other scout region, once the main launches of batch b - 1, which read it,
  // are through) || this stream: main launches and finalize of batch b.
  if (int rc = check_reduce_arguments(problem, d_groups, n_groups, d_reduce_block_prefix,
                                      n_reduce_blocks, d_scout_prefix, n_scout_blocks, d_row_terms,
                                      d_stage_floor, d_partial_cost, d_partial_index))
    return rc;
  if (!d_terms_block_prefix || n_terms_blocks <= 0)
    return fail(MIST_E_INVALID, "null / empty row-term decomposition");
  if (int rc = check_factors(problem)) return rc;
  for (int i = 0; i < n_samples; ++i)
    if (!(ratios[i] >= 0.0)) return fail(MIST_E_INVALID, "ratio %d must be non-negative", i);
  OverlapStreams *os = nullptr;
  if (int rc = overlap_streams(&os)) return rc;
  std::lock_guard<std::mutex> enqueue_guard(g_enqueue_lock);
  hipStream_t main_stream = (hipStream_t)stream;
  const int n_batches = (n_samples + sample_batch - 1) / sample_batch;
  const int64_t main_slabs = (int64_t)main_batch * n_reduce_blocks;
  const int64_t scout_slabs = (int64_t)sample_batch * n_scout_blocks;
  auto batch_ratios = [&](int b, int *count) {
    RatioList list = {};
    const int first = b * sample_batch;
    *count = std::min(sample_batch, n_samples - first);
    for (int i = 0; i < *count; ++i) list.r[i] = ratios[first + i];
    return list;
  };
  auto scout_of = [&](int b) -> int {  // on the side stream
    int count = 0;
    const RatioList list = batch_ratios(b, &count);
    if (int rc = launch_scout(problem, d_groups, n_groups, d_reduce_block_prefix, n_reduce_blocks,
                              d_scout_prefix, n_scout_blocks, d_row_terms, d_stage_floor, list, count,
                              main_slabs + (b % 2) * scout_slabs, d_partial_cost, d_partial_index,
                              os->side))
      return rc;
    MIST_HIP_CHECK(hipEventRecord(os->scout_done, os->side));
    return 0;
  };
  const unsigned scout_term_blocks = (unsigned)((problem->max_scout_rows + kTermsBlock - 1) / kTermsBlock);
  hipLaunchKernelGGL((row_terms_kernel<1, false>), dim3(scout_term_blocks, n_groups),
                     dim3(kTermsBlock), 0, main_stream, *problem, d_groups, n_groups,
                     d_terms_block_prefix, d_row_terms, d_stage_floor, nullptr);
  MIST_HIP_CHECK(hipGetLastError());
  MIST_HIP_CHECK(hipEventRecord(os->rows_ready, main_stream));
  MIST_HIP_CHECK(hipStreamWaitEvent(os->side, os->rows_ready, 0));
  if (int rc = scout_of(0)) return rc;
  bool from_keys = false;
  if (int rc = launch_key_terms(problem, d_groups, n_groups, d_key_terms, main_stream, &from_keys))
    return rc;
  if (from_keys)
    hipLaunchKernelGGL((row_terms_kernel<2, true>), dim3(n_terms_blocks), dim3(kTermsBlock), 0,
                       main_stream, *problem, d_groups, n_groups, d_terms_block_prefix, d_row_terms,
                       d_stage_floor, d_key_terms);
  else
    hipLaunchKernelGGL((row_terms_kernel<2, false>), dim3(n_terms_blocks), dim3(kTermsBlock), 0,
                       main_stream, *problem, d_groups, n_groups, d_terms_block_prefix, d_row_terms,
                       d_stage_floor, nullptr);
  MIST_HIP_CHECK(hipGetLastError());
  for (int b = 0; b < n_batches; ++b) {
    // (a wait takes the event's latest record at the time of the call: the scout pass of batch b)
    MIST_HIP_CHECK(hipStreamWaitEvent(main_stream, os->scout_done, 0));
    if (b + 1 < n_batches) {
      if (b >= 1) MIST_HIP_CHECK(hipStreamWaitEvent(os->side, os->main_done, 0));  // batch b - 1
      if (int rc = scout_of(b + 1)) return rc;
    }
    int count = 0;
    const RatioList list = batch_ratios(b, &count);
    for (int first = 0; first < count; first += main_batch) {
      const int n = std::min(main_batch, count - first);
      hipLaunchKernelGGL(eval_reduce_kernel, dim3(xcd_padded_grid(n_reduce_blocks), n),
                         dim3(MIST_LC_TILE), 0, main_stream, *problem, d_groups, n_groups,
                         d_reduce_block_prefix, n_reduce_blocks, d_scout_prefix, 0, d_row_terms,
                         d_stage_floor, list, first, main_slabs + (b % 2) * scout_slabs, d_partial_cost,
                         d_partial_index);
      MIST_HIP_CHECK(hipGetLastError());
      if (int rc = launch_finalize(problem, d_groups, n_groups, d_reduce_block_prefix, d_row_terms,
                                   d_partial_cost, d_partial_index,
                                   sample_index + b * sample_batch + first, n, n_reduce_blocks, tables,
                                   stream))
        return rc;
    }
    MIST_HIP_CHECK(hipEventRecord(os->main_done, main_stream));
  }
  return 0;
}

int mist_row_diagnostics(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                         const int32_t *d_requests, int n_requests, double *d_out, void *stream) {
  if (int rc = check_common(problem, d_groups, n_groups)) return rc;
  if (!d_requests || !d_out) return fail(MIST_E_INVALID, "null pointer");
  if (n_requests <= 0) return fail(MIST_E_INVALID, "n_requests must be positive, got %d", n_requests);
  if (int rc = check_factors(problem)) return rc;
  hipLaunchKernelGGL(row_diagnostics_kernel, dim3((n_requests + kTermsBlock - 1) / kTermsBlock),
                     dim3(kTermsBlock), 0, (hipStream_t)stream, *problem, d_groups, n_groups,
                     d_requests, n_requests, d_out);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

int mist_stage_analyze(const MistProblem *problem, const MistGroupDesc *d_groups, int n_groups,
                       const double *d_row_terms, const int32_t *d_requests, int n_requests,
                       double *d_out, void *stream) {
  if (int rc = check_common(problem, d_groups, n_groups)) return rc;
  if (!d_row_terms || !d_requests || !d_out) return fail(MIST_E_INVALID, "null pointer");
  if (n_requests <= 0) return fail(MIST_E_INVALID, "n_requests must be positive, got %d", n_requests);
  hipLaunchKernelGGL(analyze_kernel, dim3((n_requests + 63) / 64), dim3(64), 0, (hipStream_t)stream,
                     *problem, d_groups, n_groups, d_row_terms, d_requests, n_requests, d_out);
  MIST_HIP_CHECK(hipGetLastError());
  return 0;
}

}  // extern "C"
