"""Known-answer cells of the stage model: three cells worked out BY HAND from the reference's
source (mist/analyzer/batched_module_analyzer.py, mist/tools/optimize.py; line numbers below),
typed here as literals, and held against the oracle (oracle/stage.py, numpy loops and C loops).

The numbers were derived on paper from the reference's statements, not from any code of this
repository; every step is written out so that it can be re-checked by hand.  A dropped term, a
swapped operand (gpu->cpu for cpu->gpu, first for last layer, with-ckpt for without), a wrong
factor slice of the interference model or a wrong memory factor changes at least one literal.
Tolerance 1e-12 relative: the hand arithmetic is exact in decimal, the oracle's is float64 (and
float32 where the reference rounds, which the expected values round too).

Toy inputs (chosen so that the arithmetic stays short):
  cluster 1 node x 2 GPUs, stage mesh (1, 2), global batch 8, G = 2, so b = 2, dp = 2, tp = 1
  hidden 2048, sequence 2048 -> fragmentation term 0 (:1170-1178)
  GPU<->GPU model (k GB/s, b s): (10, 0.001) for (inter 1, intra 2), (40, 0.005) elsewhere
  CPU->GPU (20, 0.002), GPU->CPU (25, 0.004)
  interference factors (optimize.py:951-964, slices :1036-1079):
     3-way (C,G2G,C2G) (1.25, 2, 4); (C,G2G,G2C) (1.25, 2, 2.5); (C,C2G,G2C) (1.6, 2, 2.5);
           (G2G,C2G,G2C) (2, 4, 5)
     2-way (C,G2G) (1.25, 2); (C,C2G) (1.5, 2.5); (C,G2C) (1.2, 1.5); (G2G,C2G) (1.1, 1.3);
           (G2G,G2C) (1.4, 1.7); (C2G,G2C) (2, 4)
  block layer: W = G = 1024 MB, O = 4096 MB, saved 64 MB with / 512 MB without ckpt, fwd peak 300,
     bwd peak 400, output 64 MB, exec fwd 0.04 s, bwd 0.08 s (so bwd with ckpt 0.12, :1355-1359)
  pre layer: W = G = 256, O = 1024, saved 32, exec 0.004 / 0.008
  post layer: W = G = 2048, O = 8192, fwd peak 700, bwd peak 900, output 8, exec 0.04 / 0.08
  (every backward time is below 2.3 x its forward time, so the clamp of :369-370 leaves it alone)

Shared pieces:
  all_gather of 1024 MB = 1 GB over (inter 1, intra 2): 1/10 * (2-1)/2 + 0.001 = 0.051
     (optimize.py:264-303); reduce_scatter = 1.1 x -> 0.0561; all_reduce = 2.1 x -> 0.1071 (:243-252)
  pre layer, dp = 2: all_gather(0.25 GB) = 0.25/10/2 + 0.001 = 0.0135, reduce_scatter 0.01485
  post layer: all_gather(2 GB) = 2/10/2 + 0.001 = 0.101, reduce_scatter 0.1111
  I(C, G2G) for two busy resources with factors (1.25, 2) (optimize.py:552-571, 1099-1113):
     scaled = (1.25 C, 2 G2G); overlap = min; remainder = (scaled - overlap) / factor; sum.
     I(0.04, 0.051): scaled (0.05, 0.102), overlap 0.05, rest 0.052/2 = 0.026 -> 0.076
     I(0.08, 0.0561): scaled (0.1, 0.1122), overlap 0.1, rest 0.0122/2 = 0.0061 -> 0.1061
     I(0.12, 0.0561): scaled (0.15, 0.1122), overlap 0.1122, rest 0.0378/1.25 = 0.03024 -> 0.14244
     I(0.08, 0.051): scaled (0.1, 0.102), overlap 0.1, rest 0.002/2 = 0.001 -> 0.101
"""
import copy

import numpy as np
import pytest

from mist_amd.config import MistConfig
from oracle.stage import batched_stage_analyze
from util import load_raw

REL = 1e-12

GPU_GPU = [40.0, 0.005] * 16
GPU_GPU[2:4] = [10.0, 0.001]  # [inter index 0][intra index 1]
INTERFERENCE = (
    [3.0, 3.0, 3.0, 3.0]
    + [1.25, 2.0, 4.0] + [1.25, 2.0, 2.5] + [1.6, 2.0, 2.5] + [2.0, 4.0, 5.0]
    + [1.25, 2.0] + [1.5, 2.5] + [1.2, 1.5] + [1.1, 1.3] + [1.4, 1.7] + [2.0, 4.0]
)


class ToyTables:
    """The layer quantities of the docstring, whatever (b, tp) - which must be (2, 1)."""

    FULL = {"block": (1024.0, 1024.0, 4096.0), "pre": (256.0, 256.0, 1024.0), "post": (2048.0, 2048.0, 8192.0)}
    SAVED = {("block", True): 64.0, ("block", False): 512.0, ("pre", False): 32.0, ("post", False): 16.0}
    PEAK = {("block", "fwd"): 300.0, ("block", "bwd"): 400.0, ("post", "fwd"): 700.0, ("post", "bwd"): 900.0}
    OUT = {"block": 64.0, "post": 8.0}
    EXEC = {"block": (0.04, 0.08), "pre": (0.004, 0.008), "post": (0.04, 0.08)}

    @staticmethod
    def _like(value, b, tp):
        assert np.all(np.asarray(b) == 2) and np.all(np.asarray(tp) == 1), (b, tp)
        return np.full(np.broadcast(b, tp).shape, value)[()]  # scalars in, scalar out

    def mem_full_states(self, kind, item, tp):
        assert np.all(np.asarray(tp) == 1)
        return np.full(np.shape(tp), self.FULL[kind][("weights", "grads", "opts").index(item)])[()]

    def mem_saved(self, kind, ckpt, b, tp):
        return self._like(self.SAVED[kind, bool(ckpt)], b, tp)

    def mem_peak(self, kind, phase, b, tp, ckpt=None):
        # (the analysis path's debugging entries also ask for the forward peak with ckpt, which no
        # quantity checked here uses)
        return self._like(self.PEAK[kind, phase] + (1000.0 if ckpt else 0.0), b, tp)

    def mem_output(self, kind, b, tp):
        return self._like(self.OUT[kind], b, tp)

    def op_profiles(self, kind, b, tp, inter_size, intra_size):
        assert (b, tp, inter_size, intra_size) == (2, 1, 1, 1)
        fwd, bwd = self.EXEC[kind]
        return [(fwd, bwd, 0.0, 0.0)]

    def grad_accum_profiles(self, kind, b, tp):
        return []

    def constraint(self, b, tp):
        return True


def _config(flash, pre_post, preset=None, capacity_mb=1e9):
    raw = copy.deepcopy(load_raw(1))
    raw["model"].update(hidden_size=2048, num_attention_heads=16, use_flash_attn=flash)
    raw["training"].update(global_batch_size=8, max_sequence_length=2048)
    raw["hardware"].update(
        num_nodes=1, num_gpus_per_node=2, gpu_gpu_comm_params=list(GPU_GPU),
        cpu_gpu_comm_params=[20.0, 0.002], gpu_cpu_comm_params=[25.0, 0.004],
        interference_model_params=list(INTERFERENCE),
        # capacity in MB as the path sees it: memory_capacity * 0.88 (config.py:294) * 1024
        memory_capacity=capacity_mb / 1024.0 / 0.88)
    raw["tuning"].update(pre_post_strategy=pre_post, pre_post_strategy_array=preset)
    raw["enable_advanced_opt_in_first_block"] = False
    raw["strategy"] = dict(enabled=True, pre_post_strategy=pre_post, pre_post_strategy_array=preset)
    return MistConfig(raw)


def _cell(cfg, row, L, p_count, variant, p, l, c, inner="numpy"):
    """(stable, delta, fwd peak, bwd peak) of one row at one cell: latencies from the tuning
    path's tables (a single candidate row is its own argmin), peaks from the analysis hook."""
    rows = np.array([row], dtype=np.float64)
    args = (ToyTables(), cfg, list(range(p_count)), list(range(1, L + 1)), list(range(L + 1)), 1, 2, 2, rows, 1)
    res = batched_stage_analyze(*args, inner=inner)
    at = {0: (p, l - 1, c, 0), 1: (p, l - 1, c, 0), 2: (l - 1, c, 0), 3: (c, 0)}[variant]
    stable, delta, index = res[variant][0][at], res[variant][1][at], res[variant][3][at]
    assert index == 0, "the single row must be feasible at a huge capacity"
    analysis = [{}, {}, {}, {}]
    batched_stage_analyze(*args, analysis=analysis)
    entry = analysis[variant][(p, l, c)]
    return float(stable), float(delta), float(entry["mem_fwd_peak"][0]), float(entry["mem_bwd_peak"][0])


def _feasible(cfg, row, L, p_count, variant, p, l, c, inner):
    rows = np.array([row], dtype=np.float64)
    res = batched_stage_analyze(ToyTables(), cfg, list(range(p_count)), list(range(1, L + 1)),
                                list(range(L + 1)), 1, 2, 2, rows, 1, inner=inner)
    at = {0: (p, l - 1, c, 0), 1: (p, l - 1, c, 0), 2: (l - 1, c, 0), 3: (c, 0)}[variant]
    return res[variant][3][at] == 0


def _f32(x):
    return float(np.float32(x))  # the reference's rounding point (:2212-2213)


@pytest.mark.parametrize("inner", ["numpy", "c"])
def test_middle_stage_cell_without_offloading(inner):
    """Base variant, row (b 2, dp 2, tp 1, ZeRO-1: wre 0, gre 0, ore 1, no offloading),
    l = 3 layers, c = 1 checkpointed, p = 1 pre-saved micro-batch.

    Swaps: every offloaded byte count is 0 -> all eight swap latencies 0 (optimize.py:469).
    Phases (:1432-1452, 1646-1672): forward first micro-batch g2g = AG ore = 0.051; forward later
    g2g = AG wre = 0; backward last g2g = AG wre + RS ore + AR (1 - ore) = 0.0561; backward not last
    g2g = AG wre + RS gre = 0; all cpu<->gpu operands 0.
    Members (:1455-1902), exec fwd 0.04, bwd 0.08 (no ckpt) / 0.12 (ckpt):
      fwd first mb : layer = first = I(0.04, 0.051) = 0.076, last = 0.04, extra_pre = 0.051 (g2g only),
                     extra_post = 0
      fwd later    : layer = first = last = 0.04, extras 0
      bwd last mb  : no ckpt layer = first = I(0.08, 0.0561) = 0.1061, last = 0.08, extra_pre 0,
                     extra_post = 0.0561; ckpt layer = first = I(0.12, 0.0561) = 0.14244, last = 0.12
      bwd not last : no ckpt 0.08 / 0.08 / 0.08, ckpt 0.12 / 0.12 / 0.12, extras 0
    G = 2 > 1 (:1952-2028): stable from (later, not last), delta = (first, last) - stable:
      no ckpt: s_layer = 0.12, s_first = 0 + 0 + 0.04 + 0.08 = 0.12, s_last = 0.12
               d_layer = 0.076 + 0.1061 - 0.12 = 0.0621
               d_first = 0.051 + 0.0561 + 0.076 + 0.1061 - 0.12 = 0.1692, d_last = 0.04 + 0.08 - 0.12 = 0
      ckpt   : s_layer = s_first = s_last = 0.16; d_last = 0.04 + 0.12 - 0.16 = 0
    get_latencies(l 3, c 1) (:2165-2216): inner layers l - 2 = 1, with ckpt clip(c - 1, 0, 1) = 0,
      without 1; c != l -> first family without ckpt; c != 0 -> last family with ckpt:
      stable = 0.12 + 0.12 + 0.16 = 0.40;  delta = 0.0621 + 0.1692 + 0 = 0.2313
    Memory (:1181-1199, 2091-2162, 2358-2385, 2755-2786): factor 1 (nothing applies);
      partial W = 1024, G = 1024, O = 4096 / 2 = 2048; no full buffers (no sharding of W / G, no
      offload); fwd states = 0 + 4096 // 2 + 3 (2048) + 2 (2048) = 12288; bwd states = 3 (4096) = 12288;
      saved: kept 64 (ckpt) / 512 (not); current = 1 x 64 + (3 - 1 - 1) x 512 = 576; module = 64 + 2 x 512
      = 1088; pipeline = 1 x 1088 + 576 = 1664; offloaded part 0;
      fwd peak = 12288 + 1664 + 0 + 300 + 64 x 1 x 2 = 14380
      bwd peak = 12288 + 1664 + 0 + 400 + 128 + 64 x 2 = 14608
    Mask (:2805-2812): max x (1 + 0.025 + 0.01) = 14608 x 1.035 = 15119.28 <= capacity."""
    row = (2, 2, 1, 0, 0, 1, 0.0, 0.0, 0.0, 0.0)
    cfg = _config(True, "dp")
    stable, delta, fwd, bwd = _cell(cfg, row, 3, 2, 0, p=1, l=3, c=1, inner=inner)
    assert stable == pytest.approx(_f32(0.40), rel=REL)
    assert delta == pytest.approx(_f32(0.2313), rel=REL)
    assert fwd == pytest.approx(14380.0, rel=REL) and bwd == pytest.approx(14608.0, rel=REL)
    assert _feasible(_config(True, "dp", capacity_mb=15119.5), row, 3, 2, 0, 1, 3, 1, inner)
    assert not _feasible(_config(True, "dp", capacity_mb=15119.0), row, 3, 2, 0, 1, 3, 1, inner)


@pytest.mark.parametrize("inner", ["numpy", "c"])
def test_first_stage_cell_with_activation_offloading(inner):
    """with_pre variant, row (b 2, dp 2, tp 1, wre 0, gre 1, ore 1, activation ratio 0.5), l = 2,
    c = 2 (all layers checkpointed), p = 2; pre / post strategy "dp" = (dp 2, tp 1, ore only).

    Swaps (:1362-1391): checkpointed activations 64 x 0.5 = 32 MB = 0.03125 GB: out 0.03125/25 +
    0.004 = 0.00525, in 0.03125/20 + 0.002 = 0.0035625; all state swaps 0.
    Phases: fwd first g2g = 0.051; fwd later g2g = 0; bwd last g2g = RS ore = 0.0561; bwd not last
    g2g = RS gre = 0.0561; cpu<->gpu operands only from the activations.
    Members, with ckpt (exec bwd 0.12):
      fwd later    : first = I(0.04) = 0.04; last = I(C 0.04, G2C 0.00525), factors (1.2, 1.5): scaled
                     (0.048, 0.007875), overlap 0.007875, rest 0.040125/1.2 = 0.0334375 -> 0.0413125;
                     extra_pre = 0 (advanced option off); extra_post = 0.00525
      bwd not last : first = I(0.12, 0.0561) = 0.14244; last = I(C 0.12, C2G 0.0035625), factors
                     (1.5, 2.5): scaled (0.18, 0.00890625), overlap 0.00890625, rest 0.17109375/1.5
                     = 0.1140625 -> 0.12296875; extra_pre = 0.0035625; extra_post = 0.0561
      fwd first    : first = I(0.04, 0.051) = 0.076; last = 0.0413125; extra_pre = 0.051; extra_post 0.00525
      bwd last     : first = 0.14244; last = 0.12296875; extra_pre = 0.0035625; extra_post = 0.0561
    Families: s_first = 0 + 0.0561 + 0.04 + 0.14244 = 0.23854
              s_last  = 0.00525 + 0.0035625 + 0.0413125 + 0.12296875 = 0.17309375
              d_first = 0.051 + 0.0561 + 0.076 + 0.14244 - 0.23854 = 0.087;  d_last = 0
    get_latencies(l 2, c 2): no inner layers; c == l -> first with ckpt; c > 0 -> last with ckpt:
      stable = 0.41163375, delta = 0.087, both rounded to float32 (:2212-2213)
    with_pre (:2233-2248): pre layer is neither weight- nor gradient-sharded, so its collectives go
      to delta: stable + 0.004 + 0.008; delta + 0.0135 + 0.01485
    Memory: factor 1 + 0.04 (activation offload) + 0.025 (gre) = 1.065; for pipelines + 0.025 = 1.09;
      partial W 1024, G 1024/2 = 512, O 2048; gradient buffer (gre) max(256, 2048, 1024) = 2048, no
      weight buffer; fwd states = 2 x 2048 + 2048 + 2 x 1536 + 1 x 2048 = 11264;
      bwd states = 4096 + 2 x 3584 = 11264; kept activations 32 (ckpt) / 256, offloaded 32 / 256;
      c == l: current = (2 - 1) x 32 = 32; module = 2 x 32 = 64; pipeline = 2 x 64 + 32 = 160;
      c >= l - 1 -> delta for peak 32;
      fwd peak = 11264 + 160 + 32 + 300 + 64 x 2 x 2 = 12012;  bwd = 11264 + 160 + 32 + 400 + 256 + 128 = 12240
      pre layer: states 256 + 256 + 1024/2 = 1024, saved 32 -> + 2 x 32 + 1056 (:2866-2875):
      fwd 13132, bwd 13360.  Mask (:2893-2897): 13360 x 1.09 = 14562.4."""
    row = (2, 2, 1, 0, 1, 1, 0.0, 0.0, 0.0, 0.5)
    cfg = _config(True, "dp")
    stable, delta, fwd, bwd = _cell(cfg, row, 2, 3, 1, p=2, l=2, c=2, inner=inner)
    assert stable == pytest.approx(_f32(0.41163375) + 0.004 + 0.008, rel=REL)
    assert delta == pytest.approx(_f32(0.087) + 0.0135 + 0.01485, rel=REL)
    assert fwd == pytest.approx(13132.0, rel=REL) and bwd == pytest.approx(13360.0, rel=REL)
    assert _feasible(_config(True, "dp", capacity_mb=14562.6), row, 2, 3, 1, 2, 2, 2, inner)
    assert not _feasible(_config(True, "dp", capacity_mb=14562.2), row, 2, 3, 1, 2, 2, 2, inner)


@pytest.mark.parametrize("inner", ["numpy", "c"])
def test_last_and_single_stage_cells_with_optimizer_offloading(inner):
    """with_post and no_pp variants, row (b 2, dp 2, tp 1, ZeRO-3: wre = gre = ore = 1, optimizer
    ratio 0.5), L = l = 2, c = 0, p = 0; flash attention off; pre / post strategy preset
    (dp 2, tp 1, gradients and optimizer states sharded).

    Swaps: optimizer states 4096 / 2 x 0.5 = 1024 MB = 1 GB: out 1/25 + 0.004 = 0.044, in 1/20 +
    0.002 = 0.052; nothing else.
    Phases: fwd first g2g = AG ore = 0.051, g2c = so_O + so_W = 0.044, c2g = si_O + si_G = 0.052;
    fwd later g2g = AG wre = 0.051; bwd last g2g = 0.051 + 0.0561 = 0.1071; bwd not last the same.
    Members, without ckpt:
      fwd later    : first = I(0.04, 0.051) = 0.076; last = 0.04; extras 0
      bwd not last : first = I(0.08, RS gre 0.0561) = 0.1061; last = I(0.08, AG wre 0.051) = 0.101;
                     extra_pre = 0.051; extra_post = 0.0561
      fwd first    : first = I(C 0.04, G2G 0.051, C2G 0.052), factors (1.25, 2, 4): scaled (0.05, 0.102,
                     0.208), overlap 0.05, rest (0, 0.026, 0.0395); then (G2G, C2G) with (1.1, 1.3): scaled
                     (0.0286, 0.05135), overlap 0.0286, rest 0.02275/1.3 = 0.0175 -> 0.05 + 0.0286 +
                     0.0175 = 0.0961;
                     last = I(C 0.04, G2C 0.044), factors (1.2, 1.5): scaled (0.048, 0.066), overlap
                     0.048, rest 0.018/1.5 = 0.012 -> 0.06; extra_pre = 0.051; extra_post = 0.044
      bwd last     : first = 0.1061; last = 0.101; extra_pre = 0.051; extra_post = 0.0561
    Families: s_first = 0 + 0.0561 + 0.076 + 0.1061 = 0.2382; s_last = 0 + 0.051 + 0.04 + 0.101 = 0.192
              d_first = 0.051 + 0.0561 + 0.0961 + 0.1061 - 0.2382 = 0.0711
              d_last  = 0.044 + 0.051 + 0.06 + 0.101 - 0.192 = 0.064
    get_latencies(l 2, c 0): stable = 0.4302, delta = 0.1351 (float32).
    Post layer (:2251-2321), last layer without ckpt (c == 0):
      weights all-gather 0.101 hides behind exec fwd 0.04 - 0 - 0 -> 0.061 left;
      gradient reduce-scatter 0.1111 hides behind 0.08 - AG wre 0.051 - 0 - 0 = 0.029 -> 0.0821 left;
      post backward 0.08 overlaps extra_pre (bwd not last, ckpt) = 0.051 -> 0.029 left.
      The preset shards gradients, not weights: the reduce-scatter remainder is paid every
      micro-batch (stable), the all-gather remainder once (delta):
      stable_post = stable + 0.04 + 0.029 + 0 + 0.0821;  delta_post = delta + 0.061
    no_pp (:2322-2355): pre layer 0.004 + 0.008, its reduce-scatter 0.01485 stable, its all-gather
      0.0135 delta: stable = stable + 0.004 + 0.008 + 0.04 + 0.029 + 0 + 0.01485 + 0 + 0.0821;
      delta = delta + 0.0135 + 0 + 0.061 + 0
    Memory: factor 1 + 0.03 (optimizer offload) + 0.025 + 0.025 = 1.08, pipelines 1.105;
      attention buffer 2 x 2 x 16 / 1 x 2048^2 / 1024^2 = 256 (:1203-1213);
      partial W = G = 512, O = 4096/2 x 0.5 = 1024; both full buffers max(256, 2048, 1024) = 2048;
      fwd states = 2 x 4096 + 4096 // 2 + 2 x 1024 + 1 x 1024 = 13312;  bwd = 8192 + 2 x 2048 = 12288;
      saved 64 / 512 kept, nothing offloaded; current = 0 + (2 - 0 - 1) x 512 = 512; module = 1024;
      fwd peak = 13312 + 512 + 0 + 300 + 0 + 256 = 14380; bwd = 12288 + 512 + 400 + 0 + 128 + 256 = 13584
      post states = 2048 + 2048 + 8192/2 = 8192 (:962-1003);
      inside the post layer (:2946-2960): fwd = 13312 + 8192 + 1024 + 700 + 256 = 23484,
      bwd = 12288 + 8192 + 1024 + 900 + 0 + 256 = 22660;
      fwd = max(23484, 14380 + 8192) = 23484;  bwd = max(22660, 13584 - 64 + 8192) + 8 = 22668
      mask (:2997-3001): 23484 x 1.105 = 25949.82
      no_pp: pre states 256 + 256/2 + 1024/2 = 896, saved 32: fwd 24412, bwd 23596;
      mask with the plain factor (:3080-3083): 24412 x 1.08 = 26364.96."""
    row = (2, 2, 1, 1, 1, 1, 0.0, 0.0, 0.5, 0.0)
    preset = [1, 2, 1, 0, 1, 1, 0.0, 0.0, 0.0, 0.0]
    cfg = _config(False, "preset", preset)
    stable, delta, fwd, bwd = _cell(cfg, row, 2, 1, 2, p=0, l=2, c=0, inner=inner)
    assert stable == pytest.approx(_f32(0.4302) + 0.04 + 0.029 + 0.0821, rel=REL)
    assert delta == pytest.approx(_f32(0.1351) + 0.061, rel=REL)
    assert fwd == pytest.approx(23484.0, rel=REL) and bwd == pytest.approx(22668.0, rel=REL)
    assert _feasible(_config(False, "preset", preset, 25950.0), row, 2, 1, 2, 0, 2, 0, inner)
    assert not _feasible(_config(False, "preset", preset, 25949.6), row, 2, 1, 2, 0, 2, 0, inner)
    stable, delta, fwd, bwd = _cell(cfg, row, 2, 1, 3, p=0, l=2, c=0, inner=inner)
    assert stable == pytest.approx(_f32(0.4302) + 0.004 + 0.008 + 0.04 + 0.029 + 0.01485 + 0.0821, rel=REL)
    assert delta == pytest.approx(_f32(0.1351) + 0.0135 + 0.061, rel=REL)
    assert fwd == pytest.approx(24412.0, rel=REL) and bwd == pytest.approx(23596.0, rel=REL)
    assert _feasible(_config(False, "preset", preset, 26365.2), row, 2, 1, 3, 0, 2, 0, inner)
    assert not _feasible(_config(False, "preset", preset, 26364.8), row, 2, 1, 3, 0, 2, 0, inner)


@pytest.mark.gpu
def test_known_answer_cells_on_the_gpu():
    """The same three hand-computed cells through the HIP kernels (row terms + the analysis
    kernel, which share their device functions with the search kernels): the literals above."""
    from mist_amd.analysis import batched_stage_analyze as gpu_analyze

    def cell(cfg, row, variant, p, l, c):
        res = gpu_analyze(ToyTables(), [p], [l], [c], 1, 2, 2, row, cfg)
        e = res[variant][(p, l, c)]
        suffix = ("", "_with_pre", "_with_post", "_with_pre_and_post")[variant]
        return (e["****latency_stable" + suffix], e["****latency_delta" + suffix],
                e["mem_fwd_peak"], e["mem_bwd_peak"])

    cfg = _config(True, "dp")
    got = cell(cfg, (2, 2, 1, 0, 0, 1, 0.0, 0.0, 0.0, 0.0), 0, 1, 3, 1)
    assert got == pytest.approx((_f32(0.40), _f32(0.2313), 14380.0, 14608.0), rel=REL)
    got = cell(cfg, (2, 2, 1, 0, 1, 1, 0.0, 0.0, 0.0, 0.5), 1, 2, 2, 2)
    assert got == pytest.approx((_f32(0.41163375) + 0.004 + 0.008, _f32(0.087) + 0.0135 + 0.01485,
                                 13132.0, 13360.0), rel=REL)
    cfg = _config(False, "preset", [1, 2, 1, 0, 1, 1, 0.0, 0.0, 0.0, 0.0])
    row = (2, 2, 1, 1, 1, 1, 0.0, 0.0, 0.5, 0.0)
    got = cell(cfg, row, 2, 0, 2, 0)
    assert got == pytest.approx((_f32(0.4302) + 0.04 + 0.029 + 0.0821, _f32(0.1351) + 0.061,
                                 23484.0, 22668.0), rel=REL)
    got = cell(cfg, row, 3, 0, 2, 0)
    assert got == pytest.approx((_f32(0.4302) + 0.004 + 0.008 + 0.04 + 0.029 + 0.01485 + 0.0821,
                                 _f32(0.1351) + 0.0135 + 0.061, 24412.0, 23596.0), rel=REL)
