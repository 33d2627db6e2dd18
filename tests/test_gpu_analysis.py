"""GPU parity of the analysis path (one given strategy -> latency and peak memory) against the
oracle, bit for bit, and its consistency with the search."""
import numpy as np
import pytest
import yaml

from mist_amd.config import MistConfig
from tests.util import load_plan, tiny_plan

pytestmark = pytest.mark.gpu

_KEYS = {"latency": "latency", "mem_fwd_peak": "mem_fwd_peak", "mem_bwd_peak": "mem_bwd_peak"}
_SUFFIX = ("", "_with_pre", "_with_post", "_with_pre_and_post")


def _strategy_cfg(cfg, pre_post="dp", array=None):
    raw = cfg.raw()
    raw["strategy"] = dict(enabled=True, gradient_accumulation_steps=1, layer_partitions=[1],
                           device_assignment=[[1, 1]], gradient_checkpointing=[0],
                           stage_strategies=[[1, 1, 1, 0, 0, 1, 0.0, 0.0, 0.0, 0.0]],
                           pre_post_strategy=pre_post, pre_post_strategy_array=array)
    return MistConfig(raw)


@pytest.mark.parametrize("pre_post", ["dp", "intra-node-tp-with-ore", "tuned", "preset"])
@pytest.mark.parametrize("plan,layers", [(1, 6), (1, None), (2, 8)])
def test_stage_dictionaries_match_oracle(plan, layers, pre_post):
    """Random rows of the search space, random cells: every returned entry equals the oracle's."""
    from mist_amd.analysis import batched_stage_analyze
    from mist_amd.search_space import (_get_device_mesh_candidates, _get_grad_accumu_steps_candidates,
                                       create_search_space_for_a_block_layer)
    from oracle.stage import batched_stage_analyze as oracle_analyze

    base, tables = load_plan(plan) if layers is None else tiny_plan(plan, layers=layers)
    L, hw = base.model.num_hidden_layers, base.hardware
    array = [2, 2, 1, 0, 1, 1, 0.0, 0.0, 0.5, 0.0] if pre_post == "preset" else None
    cfg = _strategy_cfg(base, pre_post, array)
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(base.training.global_batch_size)
    rng = np.random.default_rng(plan * 100 + (layers or 0) + len(pre_post))
    checked = empty = 0
    for trial in range(12):
        n, m = meshes[rng.integers(len(meshes))]
        G = int(Gs[rng.integers(len(Gs))])
        space = create_search_space_for_a_block_layer(
            n, m, base.training.global_batch_size, G, base, constraint_fn=tables.constraint,
            tp_size=None)
        if space.n_rows == 0:
            continue
        row = space.decode(np.array(rng.integers(space.n_rows)))
        l = int(rng.integers(1, L + 1))
        c = int(rng.integers(0, l + 1))
        p = int(rng.integers(0, 4))
        got = batched_stage_analyze(tables, [p], [l], [c], n, m, G, row, cfg)
        want = [{}, {}, {}, {}]
        oracle_analyze(tables, cfg, list(range(p + 1)), list(range(1, l + 1)), list(range(c + 1)),
                       n, m, G, row, sample_size=1, analysis=want)
        for v in range(4):
            w = want[v].get((p, l, c))
            g = got[v].get((p, l, c))
            if w is None:
                assert g is None
                empty += 1
                continue
            for key in ("latency", "mem_fwd_peak", "mem_bwd_peak"):
                assert g[key] == float(np.asarray(w[key]).reshape(-1)[0]), (trial, v, key)
            assert g["****latency_stable" + _SUFFIX[v]] == float(np.asarray(w["latency_stable"]).reshape(-1)[0])
            assert g["****latency_delta" + _SUFFIX[v]] == float(np.asarray(w["latency_delta"]).reshape(-1)[0])
            # the debugging entries (get_extra_info): the same keys, every value bit-equal
            extra = w["extra_info"]
            assert set(extra) | {"latency", "mem_fwd_peak", "mem_bwd_peak"} == set(g)
            differing = [k for k in extra if not (g[k] == extra[k] or (g[k] != g[k] and extra[k] != extra[k]))]
            assert not differing, (trial, v, differing[:5], [(g[k], extra[k]) for k in differing[:5]])
            checked += 1
    assert checked >= 4


@pytest.mark.parametrize(
    "granularity,overrides",
    [
        ("uniform-device-pp-mip", dict(hardware__num_nodes=1, hardware__num_gpus_per_node=4,
                                       training__global_batch_size=64, hardware__memory_capacity=4.0,
                                       tuning__sample_size=3, tuning__pre_post_strategy="intra-node-tp-with-ore")),
        ("uniform-device-pp-mip", dict(hardware__num_nodes=2, hardware__num_gpus_per_node=2,
                                       training__global_batch_size=32, hardware__memory_capacity=3.0,
                                       tuning__sample_size=3, tuning__pre_post_strategy="intra-node-tp-without-ore")),
        ("inter-stage", dict(hardware__num_nodes=2, hardware__num_gpus_per_node=4,
                             training__global_batch_size=32, hardware__memory_capacity=8.0)),
    ],
)
def test_analyze_tuned_strategy(granularity, overrides):
    """tune -> strategy YAML -> analyze: equal to the oracle's analysis of the same YAML; with the
    tuner's pre/post strategy on both sides the MIP cost is reproduced up to float32 rounding."""
    from mist_amd.analysis import analyze
    from mist_amd.tune_one_case import best_solution_yaml, tune
    from oracle.analysis import analyze as oracle_analyze

    cfg, tables = tiny_plan(1, layers=6, tuning__tuning_granularity=granularity, **overrides)
    cost, solution = tune(cfg)
    assert solution is not None
    raw = yaml.safe_load(best_solution_yaml(cfg.raw(), solution))
    as_written = MistConfig(raw)                       # preset from the last stage (:62-101)
    assert analyze(as_written, tables) == oracle_analyze(as_written, tables)
    raw["strategy"]["pre_post_strategy"] = cfg.tuning.pre_post_strategy
    same = MistConfig(raw)
    if granularity == "uniform-device-pp-mip":
        got = analyze(same, tables)
        assert got == oracle_analyze(same, tables)
        assert got[0] == pytest.approx(cost, rel=2e-6)


def test_analyze_gpt7b_tuned_strategy_invariants():
    """Full-size plan: the tuned strategy analysed stage by stage stays within the memory
    capacity and its total is the cost of the search's own model."""
    from mist_amd.analysis import analyze
    from mist_amd.tune_one_case import best_solution_yaml, tune

    cfg, tables = load_plan(2)
    cost, solution = tune(cfg)
    raw = yaml.safe_load(best_solution_yaml(cfg.raw(), solution))
    total, stable, delta, peaks = analyze(MistConfig(raw), tables)
    S = len(solution[1])
    assert len(stable) == len(delta) == len(peaks) == S
    assert np.isfinite(total) and total > 0
    assert total >= sum(stable) + max(stable) * (solution[0] - 1)
    assert all(0 < v for v in peaks)


def test_analysis_error_paths():
    from mist_amd.analysis import analyze, analyze_cells, batched_stage_analyze

    cfg, tables = tiny_plan(1, layers=6)
    with pytest.raises(ValueError, match="strategy block"):
        analyze(cfg, tables)
    scfg = _strategy_cfg(cfg)
    row = [1, 1, 2, 0, 0, 1, 0.0, 0.0, 0.75, 0.0]
    with pytest.raises(ValueError, match="outside"):
        analyze_cells(scfg, tables, [(1, 2, 2, row, [(0, 7, 0)])])
    with pytest.raises(ValueError, match="one strategy row"):
        batched_stage_analyze(tables, [0], [1], [0], 1, 2, 2, [row, row], scfg)
    # pre/post batch size 8 // 8 // 2 == 0: empty dictionaries, the driver fails on the key
    assert batched_stage_analyze(tables, [0], [6], [3], 1, 2, 8, row, scfg) == ({}, {}, {}, {})
    raw = scfg.raw()
    raw["strategy"].update(gradient_accumulation_steps=8, layer_partitions=[6], device_assignment=[[1, 2]],
                           gradient_checkpointing=[3], stage_strategies=[row])
    with pytest.raises(KeyError):
        analyze(MistConfig(raw), tables)
