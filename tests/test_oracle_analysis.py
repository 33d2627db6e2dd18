"""Pins the oracle of the analysis path: the totals against closed forms, and the whole path
against the assignment objective of the MIP search, which is the same function of the same
per-stage quantities (float32 tables there, float64 here)."""
import numpy as np
import pytest
import yaml

from mist_amd.config import MistConfig
from mist_amd.tune_one_case import best_solution_yaml
from oracle import analysis
from tests.util import tiny_plan


def _with_stage_results(monkeypatch, per_stage):
    def fake(tables, config, stage_idx):
        return per_stage[stage_idx]
    monkeypatch.setattr(analysis, "stage_results", fake)


def _cfg(S, G, **top):
    raw = tiny_plan(1, layers=6)[0].raw()
    raw["strategy"] = dict(
        enabled=True, gradient_accumulation_steps=G, layer_partitions=[1] * S,
        device_assignment=[[1, 1]] * S, gradient_checkpointing=[0] * S,
        stage_strategies=[[1, 1, 1, 0, 0, 1, 0.0, 0.0, 0.0, 0.0]] * S, pre_post_strategy="dp")
    raw.update(top)
    return MistConfig(raw)


def _entry(stable, delta, latency, fwd, bwd):
    return dict(latency_stable=stable, latency_delta=delta, latency=latency, mem_fwd_peak=fwd, mem_bwd_peak=bwd)


def test_totals_closed_forms(monkeypatch):
    e = [_entry(1.0, 5.0, 1.5, 10.0, 30.0), _entry(2.0, 0.25, 2.5, 40.0, 20.0), _entry(3.0, 0.0, 3.5, 5.0, 6.0)]
    _with_stage_results(monkeypatch, [[e[0]] * 4, [e[1]] * 4, [e[2]] * 4])
    total, stable, delta, peaks = analysis.analyze(_cfg(3, 4), None)
    # sum 6 + max 3 * (G - 1) 9 + max(5 - 0, 0.25 - 1, 0 - 3) 5
    assert (total, stable, delta, peaks) == (20.0, [1.0, 2.0, 3.0], [5.0, 0.25, 0.0], [30.0, 40.0, 6.0])
    total, stable, delta, _ = analysis.analyze(
        _cfg(3, 4, disable_non_uniform_pp_micro_batch_analysis=True), None)
    assert (total, stable, delta) == (7.5 + 3.5 * 3, [1.5, 2.5, 3.5], [0, 0, 0])
    _with_stage_results(monkeypatch, [[e[1]] * 4])
    assert analysis.analyze(_cfg(1, 8), None) == (2.5 * 8, [0], [], [40.0])


def test_stage_variant_and_presaved_micro_batches(monkeypatch):
    """First stage reads with_pre, last with_post, single stage pre_and_post (run.py:108-152)."""
    seen = []

    def fake(tables, config, stage_idx):
        seen.append(stage_idx)
        return [_entry(10.0 * v + stage_idx, 0.0, 0.0, 0.0, 0.0) for v in range(4)]
    monkeypatch.setattr(analysis, "stage_results", fake)
    _, stable, _, _ = analysis.analyze(_cfg(4, 2), None)
    assert stable == [10.0, 1.0, 2.0, 23.0] and seen == [0, 1, 2, 3]


@pytest.mark.parametrize(
    "overrides",
    [
        dict(hardware__num_nodes=1, hardware__num_gpus_per_node=4, training__global_batch_size=64,
             hardware__memory_capacity=4.0, tuning__pre_post_strategy="intra-node-tp-with-ore"),
        dict(hardware__num_nodes=2, hardware__num_gpus_per_node=2, training__global_batch_size=32,
             hardware__memory_capacity=3.0, tuning__pre_post_strategy="intra-node-tp-without-ore"),
    ],
)
def test_analysis_of_the_tuned_strategy_reproduces_its_cost(overrides):
    """``tune`` (MIP granularity) minimises exactly what ``analyze`` evaluates; with the same
    pre/post layer strategy on both sides the two numbers agree up to the float32 rounding of the
    tuner's tables."""
    from oracle.tune import tune

    cfg, tables = tiny_plan(1, layers=6, tuning__tuning_granularity="uniform-device-pp-mip",
                            tuning__sample_size=3, **overrides)
    cost, solution = tune(cfg, tables)
    assert solution is not None
    raw = yaml.safe_load(best_solution_yaml(cfg.raw(), solution))
    raw["strategy"]["pre_post_strategy"] = cfg.tuning.pre_post_strategy
    total, stable, delta, peaks = analysis.analyze(MistConfig(raw), tables)
    assert total == pytest.approx(cost, rel=2e-6)
    assert len(peaks) == len(solution[1])
    cap_mb = cfg.hardware.memory_capacity * 1024
    assert all(0 < peak <= cap_mb for peak in peaks)   # the tuner only keeps feasible strategies


def test_pre_post_batch_out_of_range_leaves_the_dictionaries_empty():
    """batched_module_analyzer.py:868-880: the analysis path returns before computing anything;
    the driver then fails on the missing key."""
    cfg, tables = tiny_plan(1, layers=6)
    raw = cfg.raw()
    raw["strategy"] = dict(
        enabled=True, gradient_accumulation_steps=8, layer_partitions=[6], device_assignment=[[1, 2]],
        gradient_checkpointing=[3], stage_strategies=[[1, 1, 2, 0, 0, 1, 0.0, 0.0, 0.75, 0.0]],
        pre_post_strategy="dp")           # 8 // 8 // 2 == 0
    with pytest.raises(KeyError):
        analysis.analyze(MistConfig(raw), tables)
    raw["strategy"]["pre_post_strategy"] = "tuned"   # the row's own dp = 1: batch size 1
    total, _, _, peaks = analysis.analyze(MistConfig(raw), tables)
    assert np.isfinite(total) and total > 0 and peaks[0] > 0


def test_extra_info_keys_and_structure():
    """The debugging entries of the analysis path: the oracle reports exactly the keys of the
    reference's get_extra_info (batched_module_analyzer.py:2401-2749; the names are held in
    tests/golden/extra_info_keys.json), and the entries are tied to each other by the
    reference's own combinations (:1910-2028 families -> stable / delta members, :2165-2216
    members -> stage latency, :2150-2162 module states), which a mislabelled entry breaks."""
    import json
    import os

    from oracle.stage import batched_stage_analyze

    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "golden", "extra_info_keys.json")) as f:
        names = json.load(f)
    assert len(names) == 135 and len(set(names)) == 135
    cfg, tables = tiny_plan(1, layers=6)
    raw = cfg.raw()
    raw["strategy"] = dict(
        enabled=True, gradient_accumulation_steps=4, layer_partitions=[6], device_assignment=[[1, 2]],
        gradient_checkpointing=[0], stage_strategies=[[1, 1, 1, 0, 0, 1, 0.0, 0.0, 0.0, 0.0]],
        pre_post_strategy="dp")
    cfg = MistConfig(raw)
    G, l = 4, 5
    row = [2, 2, 1, 1, 1, 1, 0.5, 0.5, 0.3, 0.2]  # dp 2 with ZeRO-3 flags, every offload ratio in use
    for c in (0, 2, 4, 5):
        found = [{}, {}, {}, {}]
        batched_stage_analyze(tables, cfg, [0], list(range(1, l + 1)), [c], 1, 2, G, [row], 1, analysis=found)
        e = found[0][(0, l, c)]["extra_info"]
        assert list(e) == names
        for ck in ("without_ckpt", "with_ckpt"):
            stars = "**" if ck == "without_ckpt" else "*"
            layer = (e[f"{stars}_latency_layer_critical_fwd_not_first_micro_batch_{ck}"]
                     + e[f"{stars}_latency_layer_critical_bwd_not_last_micro_batch_{ck}"])
            assert layer == e[f"****latency_layer_critical_stable_{ck}"]
            first = (e[f"****latency_extra_pre_fwd_not_first_micro_batch_{ck}"]
                     + e[f"****latency_extra_post_bwd_not_last_micro_batch_{ck}"]
                     + e[f"****latency_first_layer_critical_fwd_not_first_micro_batch_{ck}"]
                     + e[f"****latency_first_layer_critical_bwd_not_last_micro_batch_{ck}"])
            assert first == e[f"****latency_pre_fwd_and_post_bwd_and_first_layer_stable_{ck}"]
            last_first_mb = (e[f"****latency_extra_post_fwd_first_micro_batch_{ck}"]
                             + e[f"****latency_extra_pre_bwd_last_micro_batch_{ck}"]
                             + e[f"****latency_last_layer_critical_fwd_first_micro_batch_{ck}"]
                             + e[f"****latency_last_layer_critical_bwd_last_micro_batch_{ck}"])
            assert (last_first_mb - e[f"****latency_post_fwd_and_pre_bwd_and_last_layer_stable_{ck}"]
                    == e[f"****latency_post_fwd_and_pre_bwd_and_last_layer_delta_{ck}"])
        n_ck = min(max(c - 1, 0), l - 2)
        n_nock = l - 2 - n_ck
        first_ck, last_ck = ("with_ckpt" if c == l else "without_ckpt"), ("without_ckpt" if c == 0 else "with_ckpt")
        stable = (n_ck * e["****latency_layer_critical_stable_with_ckpt"]
                  + n_nock * e["****latency_layer_critical_stable_without_ckpt"]
                  + e[f"****latency_pre_fwd_and_post_bwd_and_first_layer_stable_{first_ck}"]
                  + e[f"****latency_post_fwd_and_pre_bwd_and_last_layer_stable_{last_ck}"])
        assert float(np.float32(stable)) == e["****latency_stable"]
        assert e["****latency_stable_with_pre"] == (
            e["****latency_stable"] + e["_latency_pre_fwd_latency"] + e["_latency_pre_bwd_latency"]
            + 0 + 0)  # "dp": neither ZeRO flag of the pre/post layers is set
        dp = row[1]
        assert e["_mem_layer_partial_opts"] == e["_mem_layer_full_opts"] / dp * (1 - row[8])
        assert e["_mem_layer_saved_with_ckpt"] == e["_mem_raw_layer_saved_with_ckpt"] * (1 - row[9])
        buffers = 2 * (e["*****mem_per_full_weight_buffer"] + e["*****mem_per_full_grad_buffer"])
        part = e["_mem_layer_partial_weights"] + e["_mem_layer_partial_grads"]
        assert e["_mem_module_fwd_states"] == (
            buffers + e["_mem_layer_full_opts"] // dp + l * part + (l - 1) * e["_mem_layer_partial_opts"])
        assert e["_mem_module_bwd_states"] == buffers + l * (part + e["_mem_layer_partial_opts"])
        assert e["_mem_module_fwd_saved"] == (
            e["_mem_layer_saved_with_ckpt"] * c + e["_mem_layer_saved_without_ckpt"] * (l - c))
        assert e["_latency_layer_exec_bwd_with_ckpt"] == (
            e["_latency_layer_exec_fwd"] + e["_latency_layer_exec_bwd_without_ckpt"])
        assert e["_latency_layer_gpu_to_cpu_bwd_last_micro_batch_exclude_act"] == e["_latency_layer_swap_out_grads"]
        assert e["_latency_layer_cpu_to_gpu_fwd_not_first_micro_batch_exclude_act"] == e["_latency_layer_swap_in_weights"]
