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
