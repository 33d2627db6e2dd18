"""``tune_one_case``: resolved tuning YAML in, best strategy out.

Drop-in for the reference's ``benchmark/mist/tune/tune_one_case.py`` (``tune`` :104-415,
``best_solution_yaml`` :62-101, ``main`` :418-451) for the configuration-search path, with the
evaluation running on the GPU.  Differences, all forced by what the path needs here:

* the three traced ``LayerInfo`` objects are replaced by ``LayerTables`` (closed-form tables);
* hydra / omegaconf are not used: ``main`` takes ``--config <yaml>`` plus ``key=value``
  overrides, and the YAML written is produced with PyYAML;
* ``tuning_granularity``: every value of the reference is implemented: ``inter-stage`` (the
  per-mesh DP), ``uniform-device-pp`` (the DP with one uniform mesh per stage count),
  ``uniform-device-pp-mip`` (the stage assignment over sampled policies; an exact solver in the
  library stands in for the external MILP solver), ``uniform-pp``,
  ``uniform-pp-simple-heuristic-mem-opt`` and ``no-pp``.  The reference's ``inter-stage``,
  ``uniform-device-pp`` and ``no-pp`` branches call ``intra_stage_tune`` without the required
  ``tp_size`` and read cost fields that no longer exist; here they cover the tensor-parallel
  candidates like the working branches (:199-203), use the stable/delta adapter and take
  ``tuning.sample_size`` samples (slot 0).
"""
from __future__ import annotations

import argparse
import copy
import json
import os
import time
from pprint import pformat
from typing import Any, Dict, List, Optional

import numpy as np
import torch
import yaml

from . import _lib
from . import inter_tuning as _inter_tuning
from .config import OFFLOADING_RATIO_CANDIDATES, MistConfig, tp_candidates
from .inter_tuning import inter_stage_tune, inter_stage_tune_batch
from .inter_tuning_uniform import inter_stage_tune as inter_stage_tune_uniform
from .inter_tuning_uniform_device import inter_stage_tune_batch_uniform_device
from .inter_tuning_mip import cells_wanted as mip_cells_wanted
from .inter_tuning_mip import inter_stage_tune_batch as inter_stage_tune_batch_mip
from .intra_tuning import SAMPLE_SIZE, IntraStageTuner, intra_stage_tune
from .layer_tables import LayerTables
from .node_database import layer_tables_for
from .search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates


def best_solution_yaml(cfg: Dict[str, Any], best_solution: List[Any]) -> str:
    """tune_one_case.py:62-101 on a plain dict: fills the ``strategy`` block."""
    assert len(best_solution) == 2, f"len(best_solution)={len(best_solution)}. best_solution={best_solution}."
    gradient_accumulation_steps, stage_solutions = best_solution
    layer_partitions, device_assignment, gradient_checkpointing, stage_strategies = [], [], [], []
    for stage_solution in stage_solutions:
        (layer_partition, device_mesh, num_ckpt, _policy_index), stage_strategy = stage_solution
        layer_start, layer_end = layer_partition
        layer_partitions.append(int(layer_end - layer_start + 1))
        device_assignment.append([int(x) for x in device_mesh])
        gradient_checkpointing.append(int(num_ckpt))
        stage_strategies.append([int(x) for x in stage_strategy[:6]] + [float(x) for x in stage_strategy[6:]])
    pre_post_strategy_array = [None, None, None, 0, 0, 1, 0, 0, 0, 0]
    pre_post_strategy_array[:3] = stage_strategies[-1][:3]
    cfg = copy.deepcopy(cfg)
    strategy = cfg.setdefault("strategy", {})
    strategy["enabled"] = True
    strategy["gradient_accumulation_steps"] = int(gradient_accumulation_steps)
    strategy["layer_partitions"] = layer_partitions
    strategy["device_assignment"] = device_assignment
    strategy["gradient_checkpointing"] = gradient_checkpointing
    strategy["stage_strategies"] = stage_strategies
    strategy["pre_post_strategy"] = "preset"
    strategy["pre_post_strategy_array"] = pre_post_strategy_array
    return yaml.safe_dump(cfg, sort_keys=False)


def _no_pp(mist_config, tables, device, stats):
    """tune_one_case.py:123-184 with the tensor-parallel loop and the stable/delta adapter:
    cost per (G, ckpt) = (float32(stable) + float32(delta) / G) * G, first minimum wins."""
    hw, model, tuning = mist_config.hardware, mist_config.model, mist_config.tuning
    meshes = [(hw.num_nodes, hw.num_gpus_per_node)]
    Gs = _get_grad_accumu_steps_candidates(mist_config.training.global_batch_size)
    L = model.num_hidden_layers
    best_cost, best_solution = float("inf"), None
    for tp_size in tp_candidates(mist_config):
        r = intra_stage_tune(tables, L, meshes, Gs, tp_size, mist_config, sample_size=1, device=device)
        with np.errstate(invalid="ignore"):
            costs = r.costs_stable_no_pp[..., 0] + r.costs_delta_no_pp[..., 0] / np.array(
                Gs, dtype=np.float32
            ).reshape(-1, 1, 1)
        solutions = r.solutions_no_pp[..., 0, :]
        if not tuning.activation_checkpointing_tuning_enabled:
            costs, solutions = costs[..., -1:], solutions[..., -1:, :]
        costs = costs * np.array(Gs, dtype=np.float32).reshape(-1, 1, 1)
        if not np.isfinite(costs).any():
            continue
        idx = np.unravel_index(np.argmin(costs), costs.shape)
        if float(costs[idx]) < best_cost:
            row = solutions[idx].tolist()
            row[:6] = [int(x) for x in row[:6]]
            ckpt = int(idx[2]) if tuning.activation_checkpointing_tuning_enabled else L
            best_cost = float(costs[idx])
            best_solution = [Gs[idx[0]], [(((0, L - 1), meshes[idx[1]], ckpt, 0), tuple(row))]]
    return best_cost, best_solution


MIP_TABLE_BUDGET_BYTES = 48 << 30  # sampled tables of one batch of tensor-parallel candidates


# The stage assignment reads a few layer counts per (G, mesh) group (the stage count's average
# +- tuning.layers_offset): by default only the tiles of the intra-stage tables that hold them
# are evaluated.  True: the whole tables, as the reference's IntraStageTuner fills them (same
# result; what the fixtures of all 30 samples are compared with).
MIP_EVALUATE_ALL_CELLS = False


def _uniform_device_pp_mip(mist_config, device, stats):
    """tune_one_case.py:360-402: per tensor-parallel candidate the intra-stage tables with every
    one of ``tuning.sample_size`` samples, then the stage assignment; the first best tp wins.
    As many tp candidates as fit ``MIP_TABLE_BUDGET_BYTES`` of sampled tables go through one
    batch of launches per sample (for the GPT-7B plan with 30 samples all four: 9.7 GB)."""
    hw, tuning = mist_config.hardware, mist_config.tuning
    tables = layer_tables_for(mist_config)
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, contiguous_inter_node=False)
    Gs = _get_grad_accumu_steps_candidates(mist_config.training.global_batch_size)
    L = mist_config.model.num_hidden_layers
    tps = tp_candidates(mist_config)
    P1 = min(min(max(n * m for n, m in meshes), L), max(Gs))
    per_tp = len(Gs) * len(meshes) * (2 * P1 * L * (L + 1) + L * (L + 1) + (L + 1)) * tuning.sample_size * 20
    batch = max(1, min(len(tps), MIP_TABLE_BUDGET_BYTES // max(per_tp, 1)))
    best_cost, best_solution = float("inf"), None
    for first in range(0, len(tps), batch):
        t0 = time.perf_counter()
        tuner = IntraStageTuner(tables, L, meshes, Gs, tps[first:first + batch], mist_config,
                                sample_size=tuning.sample_size, device=device)
        if not MIP_EVALUATE_ALL_CELLS:
            tuner.cells_wanted = mip_cells_wanted(
                L, hw.num_nodes, hw.num_gpus_per_node, int(getattr(tuning, "layers_offset", 2)))
            tuner.prefill_wanted_cells_only = True  # nothing else of the tables is read below
        results = tuner.tune_all()
        t1 = time.perf_counter()
        stats["intra_s"] = stats.get("intra_s", 0.0) + (t1 - t0)
        # (the strategy rows are read back for the batch's first best candidate only)
        for cost, solution in inter_stage_tune_batch_mip(
                L, hw.num_nodes, hw.num_gpus_per_node, meshes, Gs, results, mist_config, stats=stats,
                only_best_solution=True):
            if cost < best_cost:
                best_cost, best_solution = cost, solution
        stats["inter_s"] = stats.get("inter_s", 0.0) + (time.perf_counter() - t1)
        del results, tuner
    return best_cost, best_solution


class PreparedSearch:
    """The host-side preparation of one ``tune`` call, separated from its execution: group
    descriptors are built and uploaded once (``__init__``), ``run`` then only launches kernels
    and the inter-stage search.  ``tune`` is ``PreparedSearch(config).run()``."""

    def __init__(self, mist_config: MistConfig, device: str = "cuda:0", exhaustive: bool = False):
        model, hw, tuning = mist_config.model, mist_config.hardware, mist_config.tuning
        self.config = mist_config
        self.granularity = tuning.tuning_granularity
        if self.granularity not in ("uniform-pp", "uniform-pp-simple-heuristic-mem-opt", "inter-stage",
                                    "uniform-device-pp"):
            raise ValueError(f"PreparedSearch does not cover '{self.granularity}'")
        self.tables = layer_tables_for(mist_config)
        self.meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, contiguous_inter_node=False)
        self.Gs = _get_grad_accumu_steps_candidates(mist_config.training.global_batch_size)
        self.L = model.num_hidden_layers
        # The reference forwards tuning.sample_size only on its MIP branch; the uniform
        # branch runs with the default of 30 and reads sample 0 (:206-217).
        sample_size = (tuning.sample_size if self.granularity in ("inter-stage", "uniform-device-pp")
                       else SAMPLE_SIZE)
        # All tensor-parallel candidates go through one batch of launches.
        self.tuner = IntraStageTuner(self.tables, self.L, self.meshes, self.Gs,
                                     tp_candidates(mist_config), mist_config,
                                     sample_size=sample_size, sample_slots=[0], device=device,
                                     exhaustive=exhaustive)
        self.plan = self.tuner.prepare()
        with torch.cuda.device(self.tuner.device):
            self.dev_plan = self.tuner.upload(self.plan)
        # The searches that scan thresholds below best / G (inter_tuning.py:196-197) never admit
        # a stage cost above that: the intra-stage kernels need not find the minima of such
        # cells (IntraStageTuner.run_prepared), given an estimate of the best cost.  ``run``
        # searches such tables below the limit up to which they are exact
        # (mist_inter_stage_search_bounded) and evaluates again without the estimate if that
        # search reports a partition it may have missed or its result is not below the limit
        # of the estimate that was used.  ckpt counts a stage may use, as those
        # searches restrict them: inter_tuning.py:315; inter_tuning_uniform_device.py:400-404.
        self.stage_cost_cutoff = None
        self._incumbent_host = self._incumbent_read = None
        if sample_size == 1 and not exhaustive and os.environ.get("MIST_NO_STAGE_COST_CUTOFF") is None:
            devices = hw.num_nodes * hw.num_gpus_per_node
            if self.granularity == "inter-stage":
                self.stage_cost_cutoff = dict(num_devices=devices, ckpt_rule=0)
            elif self.granularity == "uniform-device-pp":
                rule = 1 if tuning.activation_checkpointing_tuning_enabled else 2
                self.stage_cost_cutoff = dict(num_devices=devices, ckpt_rule=rule)

    def counts(self) -> Dict[str, int]:
        """Search-space sizes: strategy rows, candidates = rows * (L + 1), base-variant cells
        = rows * sum_l (l + 1) * (#pre-saved micro-batch values), groups."""
        L = self.L
        pairs = L * (L + 1) // 2 + L
        g = self.plan["groups"]
        rows = int(g["n_rows"].sum())
        cells = int((g["n_rows"] * g["num_p"]).sum()) * pairs
        groups = len(g)
        return dict(rows=rows, candidates=rows * (L + 1), cells=cells, groups=groups)

    def run(self, stats: Optional[dict] = None, split_timing: bool = False):
        """``split_timing`` waits for the intra-stage kernels before the inter-stage search
        starts, so that ``stats['intra_launch_s']`` and ``stats['inter_s']`` are the wall times
        of the two halves (otherwise the first is launch time only and the second includes the
        wait for the kernels)."""
        stats = {} if stats is None else stats
        hw = self.config.hardware
        t0 = time.perf_counter()
        # (tables with a limit are searched by the library's driver only)
        cutoff = self.stage_cost_cutoff if _inter_tuning.NATIVE_SEARCH else None
        results = self.tuner.run_prepared(self.plan, self.dev_plan, cutoff)
        if cutoff is not None:
            # the estimate the kernels ended with travels to the host behind them
            with torch.cuda.device(self.tuner.device):
                if self._incumbent_host is None:
                    self._incumbent_host = torch.empty(1, dtype=torch.float64, pin_memory=True)
                    self._incumbent_read = torch.cuda.Event()
                self._incumbent_host.copy_(self.dev_plan["incumbent"], non_blocking=True)
                self._incumbent_read.record()
        if split_timing:
            torch.cuda.synchronize(self.tuner.device)
        t1 = time.perf_counter()
        # The tables hold their values up to estimate * limit_factor / G: the search stays below
        # that and reports where this leaves its result uncertain.
        limit_factor = (1.0 + _lib.load().mist_incumbent_slack()) * (1.0 - 1e-5)
        table_limit = None if cutoff is None else (self._incumbent_host, limit_factor)
        unresolved_before = stats.get("dp_unresolved", 0)
        if self.granularity == "inter-stage":
            outcomes = inter_stage_tune_batch(
                self.L, hw.num_nodes * hw.num_gpus_per_node, self.meshes, self.Gs, results, slot=0, stats=stats,
                only_best_solution=True,  # the loop below keeps the first best entry only
                table_limit=table_limit,
            )
        elif self.granularity == "uniform-device-pp":
            outcomes = inter_stage_tune_batch_uniform_device(
                self.L, hw.num_nodes, hw.num_gpus_per_node, self.meshes, self.Gs, results,
                self.config, slot=0, stats=stats, only_best_solution=True, table_limit=table_limit,
            )
        else:
            outcomes = [
                inter_stage_tune_uniform(self.L, hw.num_nodes, hw.num_gpus_per_node, self.Gs, r, self.config)
                for r in results
            ]
        stats["intra_launch_s"] = stats.get("intra_launch_s", 0.0) + (t1 - t0)
        stats["inter_s"] = stats.get("inter_s", 0.0) + (time.perf_counter() - t1)
        best_cost, best_solution = float("inf"), None
        for cost, solution in outcomes:  # tune_one_case.py:228-231: the first best tp wins
            if cost < best_cost:
                best_cost, best_solution = cost, solution
        if cutoff is not None:
            self._incumbent_read.synchronize()
            estimate = float(self._incumbent_host[0])
            # Below this cost the search has read nothing but cells that hold their minima
            # (MistProblem.stage_cost_incumbent); an infinite estimate left every cell exact.
            safe_below = estimate * limit_factor
            unresolved = stats.get("dp_unresolved", 0) - unresolved_before
            if np.isfinite(estimate) and (unresolved > 0 or not best_cost < safe_below):
                stats["stage_cost_cutoff_retries"] = stats.get("stage_cost_cutoff_retries", 0) + 1
                self.stage_cost_cutoff = None
                try:
                    return self.run(stats, split_timing)
                finally:
                    self.stage_cost_cutoff = cutoff
        return best_cost, best_solution


def tune(mist_config: MistConfig, device: str = "cuda:0", stats: Optional[dict] = None):
    """tune_one_case.py:104-415.  Returns ``(best_cost, best_solution)`` with
    ``best_solution = [G, [(((l0, l1), (n, m), ckpt, policy), (b, dp, tp, wre, gre, ore, wo, go,
    oo, ao)), ...per stage]]``."""
    tuning = mist_config.tuning
    if tuning is None:
        raise ValueError("the tuning block is missing or disabled")
    granularity = tuning.tuning_granularity
    stats = {} if stats is None else stats
    t_start = time.perf_counter()

    if granularity == "no-pp":
        best_cost, best_solution = _no_pp(mist_config, layer_tables_for(mist_config), device, stats)
    elif granularity in ("uniform-pp", "inter-stage", "uniform-device-pp"):
        best_cost, best_solution = PreparedSearch(mist_config, device).run(stats)
    elif granularity == "uniform-pp-simple-heuristic-mem-opt":
        # tune_one_case.py:258-262: sweep a fixed optimizer-offload ratio, activation offload off.
        best_cost, best_solution = float("inf"), None
        for oo_ratio in OFFLOADING_RATIO_CANDIDATES:
            raw = mist_config.raw()
            raw["fixed_oo_ratio"] = oo_ratio
            raw["tuning"]["activation_offloading_enabled"] = False
            cost, solution = PreparedSearch(MistConfig(raw), device).run(stats)
            if cost < best_cost:
                best_cost, best_solution = cost, solution
    elif granularity == "uniform-device-pp-mip":
        best_cost, best_solution = _uniform_device_pp_mip(mist_config, device, stats)
    else:
        raise ValueError(f"Unknown tuning granularity: {granularity}")
    stats["tune_s"] = time.perf_counter() - t_start
    return best_cost, best_solution


def _apply_override(raw: Dict[str, Any], item: str) -> None:
    key, _, value = item.partition("=")
    node = raw
    parts = key.split(".")
    for p in parts[:-1]:
        node = node.setdefault(p, {})
    node[parts[-1]] = yaml.safe_load(value)


def main(argv: Optional[List[str]] = None) -> None:
    """tune_one_case.py:418-451: tunes, writes ``<output_path>.yaml`` and ``summary.json``."""
    parser = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    parser.add_argument("--config", required=True, help="resolved tuning YAML")
    parser.add_argument("--device", default="cuda:0")
    parser.add_argument("overrides", nargs="*", help="key.path=value overrides, e.g. output_path=out/x")
    args = parser.parse_args(argv)
    with open(args.config) as f:
        raw = yaml.safe_load(f)
    for item in args.overrides:
        _apply_override(raw, item)
    raw.setdefault("strategy", {})["enabled"] = False
    raw.setdefault("tuning", {})["enabled"] = True
    mist_config = MistConfig(raw)
    stats: Dict[str, Any] = {}
    best_cost, best_solution = tune(mist_config, device=args.device, stats=stats)
    print(f"Best cost: {best_cost}")
    print(f"Best solution: {pformat(best_solution)}")
    print(f"Tuning time: {stats.get('tune_s', 0.0):.3f} s")
    if best_solution is None:
        raise SystemExit("no feasible strategy found")
    text = best_solution_yaml(raw, best_solution)
    output_path = raw.get("output_path")
    if output_path is not None:
        folder = os.path.dirname(output_path) or "."
        os.makedirs(folder, exist_ok=True)
        if not output_path.endswith(".yaml"):
            output_path += ".yaml"
        name = os.path.basename(output_path).split(".")[0]
        with open(output_path, "w") as f:
            f.write(text)
        summary_path = os.path.join(folder, "summary.json")
        data = {}
        if os.path.exists(summary_path):
            with open(summary_path) as f:
                data = json.load(f)
        data.setdefault(name, {}).update(
            {"tuning_best_cost": f"{best_cost:.4f}", "tuning_best_solution": pformat(best_solution)}
        )
        with open(summary_path, "w") as f:
            json.dump(data, f, indent=2)
        print(f"Saved the best solution to {output_path}")


if __name__ == "__main__":
    main()
