"""The pruned GPU search against the CPU oracle at full size, through committed fixtures.

tests/golden/search_tables_plan<N>.json (written by tests/golden/make_search_fixtures.py on the
CPU) holds, per (tp, G, mesh) group of a benchmark plan, a digest of each of the oracle's four
result tables (row indices + float32 stable / delta costs) and the oracle's end-to-end search
result: over the whole plan (``tune``) or, for the two largest plans, over the winning
tensor-parallel size and two gradient-accumulation candidates (``tune_scoped``).  Here the HIP kernels search the whole plan in
one batch (scout pass, row chunks, p tiles, sieves: everything the timed workload uses), the
same digests are taken from their tables and compared, and ``tune`` must return the oracle's
cost (bit-equal float64) and strategy.
"""
import glob
import json
import os
import re

import numpy as np
import pytest

from util import group_key, load_plan, table_digest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "search_tables_plan?.json")))
# the same for every alpha sample of a cell (the tables the uniform-device-pp-mip granularity reads)
SAMPLED_FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "search_tables_plan?_s*.json")))


def _plan_of(path):
    return int(re.search(r"plan(\d+)(_s\d+)?\.json$", path).group(1))


def _listify(x):
    """Tuples -> lists, numpy scalars -> python numbers (what a JSON round trip leaves)."""
    return json.loads(json.dumps(x, default=lambda o: o.item()))


def test_fixtures_cover_every_benchmark_plan():
    assert {_plan_of(p) for p in FIXTURES} == {1, 2, 3, 4, 5}
    assert {_plan_of(p) for p in SAMPLED_FIXTURES} >= {1, 2, 3}


@pytest.mark.parametrize("plan", [1, 2, 3, 4, 5])
def test_pruned_and_exhaustive_search_give_the_same_tables_on_whole_plans(plan):
    """Every table of every group of a benchmark plan (plan 2 is the timed workload), pruned
    search (scout pass, sieves, bounds) against the kernel that evaluates every cell: identical
    row indices and costs."""
    import torch

    from mist_amd.tune_one_case import PreparedSearch

    cfg, _ = load_plan(plan)
    tables = []
    for exhaustive in (False, True):
        search = PreparedSearch(cfg, exhaustive=exhaustive)
        results = search.tuner.run_prepared(search.plan, search.dev_plan)
        tables.append(results[0].batch)
    pruned, full = tables
    n_finite = 0
    for v in range(4):
        assert torch.equal(pruned.index[v], full.index[v]), f"row indices of variant {v}"
        assert torch.equal(pruned.stable[v], full.stable[v]), f"stable costs of variant {v}"
        assert torch.equal(pruned.delta[v], full.delta[v]), f"delta costs of variant {v}"
        n_finite += int((full.index[v] >= 0).sum())
    assert n_finite > (100000 if plan > 1 else 1000)


@pytest.mark.parametrize("exhaustive", [False, True], ids=["pruned", "exhaustive"])
@pytest.mark.parametrize("path", FIXTURES, ids=lambda p: f"plan{_plan_of(p)}")
def test_tables_and_tune_equal_the_oracle_fixture(path, exhaustive):
    from mist_amd.inter_tuning import inter_stage_tune_batch
    from mist_amd.tune_one_case import PreparedSearch

    with open(path) as f:
        fixture = json.load(f)
    plan = _plan_of(path)
    cfg, _ = load_plan(plan)
    assert cfg.tuning.tuning_granularity == "inter-stage" and cfg.tuning.sample_size == 1
    search = PreparedSearch(cfg, exhaustive=exhaustive)
    tuner = search.tuner
    results = tuner.run_prepared(search.plan, search.dev_plan)
    Gs, meshes = search.Gs, search.meshes
    present = {(int(r["g_index"]), int(r["q_index"])) for r in search.plan["groups"]}
    suffix = ("base", "with_pre", "with_post", "no_pp")
    bad, n_groups = [], 0
    for t, tp in enumerate(tuner.tp_sizes):
        res = results[t]
        host = [(res._fetch("index", v), res._fetch("stable", v), res._fetch("delta", v)) for v in range(4)]
        for g, G in enumerate(Gs):
            for q, mesh in enumerate(meshes):
                want = fixture["groups"].get(group_key(tp, G, mesh))
                if want is None:
                    # a plan covered in full lists every group that has candidate rows
                    assert fixture["select"] != "all" or (t * len(Gs) + g, q) not in present
                    continue
                n_groups += 1
                for v in range(4):
                    index, stable, delta = (a[g, q] for a in host[v])
                    if int((index >= 0).sum()) != want["finite"][v] or \
                            table_digest(index, stable, delta) != want["digest"][v]:
                        bad.append((group_key(tp, G, mesh), suffix[v], int((index >= 0).sum()), want["finite"][v]))
        del host
    assert n_groups == len(fixture["groups"])
    assert not bad, f"{len(bad)} of {4 * n_groups} tables differ from the oracle: {bad[:8]}"

    hw = cfg.hardware
    if "tune_scoped" in fixture:
        # the oracle's sequential threshold scan restricted to one tensor-parallel size and a
        # few G (the whole scan of a large plan takes the CPU hours): same restriction here
        scoped = fixture["tune_scoped"]
        tp, scope_Gs = scoped["scope"]["tp"], scoped["scope"]["Gs"]
        cost, solution = inter_stage_tune_batch(
            search.L, hw.num_nodes * hw.num_gpus_per_node, meshes, scope_Gs,
            [results[tuner.tp_sizes.index(tp)]], slot=0)[0]
        assert cost == float(scoped["cost"]), (cost, scoped["cost"])
        assert _listify(solution) == scoped["solution"]
        assert solution is not None
    if "tune" not in fixture:
        return
    outcomes = inter_stage_tune_batch(
        search.L, hw.num_nodes * hw.num_gpus_per_node, meshes, Gs, results, slot=0, only_best_solution=False)
    for tp, (cost, solution) in zip(tuner.tp_sizes, outcomes):
        want = fixture["tune"]["per_tp"][str(tp)]
        assert cost == float(want["cost"]), (tp, cost, want["cost"])
        assert _listify(solution) == want["solution"], tp
    cost, solution = search.run()
    assert cost == float(fixture["tune"]["cost"])
    assert _listify(solution) == fixture["tune"]["solution"]
    assert solution is not None


@pytest.mark.parametrize("exhaustive", [False, True], ids=["pruned", "exhaustive"])
@pytest.mark.parametrize("path", SAMPLED_FIXTURES, ids=lambda p: os.path.basename(p)[14:-5])
def test_sampled_tables_and_mip_tune_equal_the_oracle_fixture(path, exhaustive):
    """All alpha samples of every cell (mist/utils/pareto.py:124-144 with sample_size = 30, the
    reference's default) for every group the fixture holds, from the batched multi-sample launches
    (scout passes of 16 samples per launch, slabs behind one another) and from the kernel that
    evaluates every cell; then the ``uniform-device-pp-mip`` search on those tables: the oracle's
    cost and strategy per tensor-parallel size and overall."""
    from mist_amd.inter_tuning_mip import inter_stage_tune as inter_stage_tune_mip
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates
    from mist_amd.tune_one_case import tp_candidates, tune

    with open(path) as f:
        fixture = json.load(f)
    plan, S = _plan_of(path), fixture["sample_size"]
    assert S > 1
    cfg, tables = load_plan(plan, tuning__tuning_granularity="uniform-device-pp-mip", tuning__sample_size=S)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, contiguous_inter_node=False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    tps = tp_candidates(cfg)
    tuner = IntraStageTuner(tables, L, meshes, Gs, tps, cfg, sample_size=S, exhaustive=exhaustive)
    results = tuner.tune_all()
    suffix = ("base", "with_pre", "with_post", "no_pp")
    bad, n_groups = [], 0
    for t, tp in enumerate(tps):
        res = results[t]
        host = [(res._fetch("index", v), res._fetch("stable", v), res._fetch("delta", v)) for v in range(4)]
        for g, G in enumerate(Gs):
            for q, mesh in enumerate(meshes):
                want = fixture["groups"].get(group_key(tp, G, mesh))
                if want is None:
                    continue
                n_groups += 1
                for v in range(4):
                    index, stable, delta = (a[g, q] for a in host[v])
                    assert index.shape[-1] == S
                    if int((index >= 0).sum()) != want["finite"][v] or \
                            table_digest(index, stable, delta) != want["digest"][v]:
                        bad.append((group_key(tp, G, mesh), suffix[v], int((index >= 0).sum()), want["finite"][v]))
        res._host.clear()
        del host
    assert n_groups == len(fixture["groups"])
    assert not bad, f"{len(bad)} of {4 * n_groups} tables differ from the oracle: {bad[:8]}"
    if "tune" not in fixture:
        return
    assert fixture["tune"]["granularity"] == "uniform-device-pp-mip"
    for tp, res in zip(tps, results):
        cost, solution = inter_stage_tune_mip(L, hw.num_nodes, hw.num_gpus_per_node, meshes, Gs, res, cfg)
        want = fixture["tune"]["per_tp"][str(tp)]
        assert cost == float(want["cost"]), (tp, cost, want["cost"])
        assert _listify(solution) == want["solution"], tp
    del results, tuner
    if exhaustive:
        return
    cost, solution = tune(cfg)
    assert cost == float(fixture["tune"]["cost"])
    assert _listify(solution) == fixture["tune"]["solution"]
    assert solution is not None
