"""The reference's own tuner outputs (tests/golden/tuned_configs) as fixtures: strategy-block
format, the preset rule, and the structural rules of the ``uniform-device-pp-mip`` granularity -
for the fixtures and for what this build's tuner writes for the same plans."""
import glob
import os

import numpy as np
import pytest
import yaml

from mist_amd.config import MistConfig
from mist_amd.inter_tuning_mip import layer_candidates
from mist_amd.inter_tuning_uniform import _uniform_device_mesh_partition
from mist_amd.tune_one_case import best_solution_yaml

FIXTURES = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "tuned_configs", "*.yaml")))


def _load(path):
    with open(path) as f:
        return yaml.safe_load(f)


def _check_structure(raw):
    """Rules every output of this granularity obeys (inter_tuning_mip.py:87-253, :282-290;
    tune_one_case.py:62-101)."""
    st, hw = raw["strategy"], raw["hardware"]
    L, B = raw["model"]["num_hidden_layers"], raw["training"]["global_batch_size"]
    S, G = len(st["layer_partitions"]), st["gradient_accumulation_steps"]
    assert st["enabled"] is True and st["pre_post_strategy"] == "preset"
    assert len(st["device_assignment"]) == len(st["gradient_checkpointing"]) == len(st["stage_strategies"]) == S
    assert sum(st["layer_partitions"]) == L
    lo, hi = layer_candidates(L, S, G, 2)
    assert all(lo <= l <= hi for l in st["layer_partitions"])
    mesh = _uniform_device_mesh_partition(S, hw["num_nodes"], hw["num_gpus_per_node"])
    assert all(tuple(a) == tuple(mesh) for a in st["device_assignment"])
    assert B % G == 0 and G & (G - 1) == 0
    for l, c, row in zip(st["layer_partitions"], st["gradient_checkpointing"], st["stage_strategies"]):
        assert 0 <= c <= l and len(row) == 10
        b, dp, tp = row[:3]
        assert b * dp * G == B and dp * tp == mesh[0] * mesh[1]
        assert all(v in (0, 1) for v in row[3:6]) and all(0.0 <= v <= 1.0 for v in row[6:])
    last = st["stage_strategies"][-1]
    assert st["pre_post_strategy_array"] == [last[0], last[1], last[2], 0, 0, 1, 0, 0, 0, 0]


@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p)[:28] for p in FIXTURES])
def test_reference_outputs_obey_the_structural_rules(path):
    assert len(FIXTURES) == 4
    raw = _load(path)
    assert raw["tuning"]["tuning_granularity"] == "uniform-device-pp-mip"
    _check_structure(raw)
    cfg = MistConfig(raw)
    assert cfg.strategy.num_stages == len(raw["strategy"]["layer_partitions"])
    assert cfg.strategy.stage_strategies[0][:3] == tuple(raw["strategy"]["stage_strategies"][0][:3])


@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p)[:28] for p in FIXTURES])
def test_strategy_block_round_trip(path):
    """The solution a tuner returns for the fixture's strategy, written with this build's
    ``best_solution_yaml``, gives back the fixture's strategy block key for key."""
    raw = _load(path)
    st = raw["strategy"]
    covered, stages = 0, []
    for l, mesh, c, row in zip(st["layer_partitions"], st["device_assignment"],
                               st["gradient_checkpointing"], st["stage_strategies"]):
        stages.append((((covered, covered + l - 1), tuple(mesh), c, 0), tuple(row)))
        covered += l
    plan = {k: v for k, v in raw.items() if k != "strategy"}
    out = yaml.safe_load(best_solution_yaml(plan, [st["gradient_accumulation_steps"], stages]))
    assert out["strategy"] == st
    assert {k: v for k, v in out.items() if k != "strategy"} == plan


@pytest.mark.gpu
@pytest.mark.parametrize("path", FIXTURES[:3], ids=[os.path.basename(p)[:28] for p in FIXTURES[:3]])
def test_own_tuner_output_obeys_the_same_rules_and_analyzes(path):
    """The same plan through this build (synthetic layer tables, so other numbers and possibly
    another strategy than the fixture's): the written YAML obeys the same rules, and both its
    strategy and the reference's go through the analysis path."""
    from mist_amd.analysis import analyze
    from mist_amd.layer_tables import LayerTables
    from mist_amd.tune_one_case import tune

    raw = _load(path)
    plan = {k: v for k, v in raw.items() if k != "strategy"}
    cfg = MistConfig(plan)
    cost, solution = tune(cfg)
    assert solution is not None and np.isfinite(cost)
    written = yaml.safe_load(best_solution_yaml(plan, solution))
    _check_structure(written)
    tables = LayerTables(cfg)
    for candidate in (written, raw):
        total, stable, delta, peaks = analyze(MistConfig(candidate), tables)
        assert np.isfinite(total) and total > 0 and all(p > 0 for p in peaks)
        assert len(peaks) == len(candidate["strategy"]["layer_partitions"])
