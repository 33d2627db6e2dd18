"""Uniform inter-stage search: drop-in for the reference's
``mist/analyzer/inter_tuning_uniform.py`` (``inter_stage_tune`` :120-258,
``inter_stage_tune_with_fixed_inter_partition`` :261-397).

Layers and devices are split evenly over the stages, so the search is a few thousand table
look-ups; it runs on the host over the tables the GPU produced (sample slot 0 only, like the
reference).  Stage latency is ``stable + delta / G`` evaluated in float64: the reference adds
numpy float32 scalars to a python-int quotient, which numpy 1.24 promotes to float64.
"""
from __future__ import annotations

from typing import List, Optional

import numpy as np

from .config import MistConfig
from .inter_tuning import get_solution_from_intra_stage_tuner_output
from .intra_tuning import IntraStageTunerOutput


def _uniform_layer_partition(num_layers: int, num_stages: int) -> List[int]:
    """inter_tuning_uniform.py:95-102: remainder layers go to the last stages."""
    per_stage = num_layers // num_stages
    partition = [per_stage] * num_stages
    for i in range(num_layers % num_stages):
        partition[-i - 1] += 1
    return partition


def _uniform_device_mesh_partition(num_stages: int, num_nodes: int, num_gpus_per_node: int):
    """inter_tuning_uniform.py:105-120."""
    if num_nodes > num_stages:
        if num_nodes % num_stages != 0:
            return None
        return num_nodes // num_stages, num_gpus_per_node
    if num_stages % num_nodes != 0 or num_gpus_per_node % (num_stages // num_nodes) != 0:
        return None
    return 1, num_gpus_per_node // (num_stages // num_nodes)


def inter_stage_tune_with_fixed_inter_partition(
    num_layers: int,
    num_stages: int,
    layer_partition: List[int],
    device_mesh_index: int,
    gradient_accumulation_steps_candidates: List[int],
    gradient_accumulation_steps_index_candidates: List[int],
    tables,
    all_gradient_accumulation_steps: List[int],
    activation_checkpointing_tuning_enabled: bool,
    simple_activation_checkpointing_tuning_enabled: bool = False,
):
    """inter_tuning_uniform.py:261-397.  ``tables`` = (stable, delta) x 4 variants, float32;
    ``all_gradient_accumulation_steps[g]`` is the G of table index g."""
    (cs, cs_pre, cs_post, cs_nopp), (cd, cd_pre, cd_post, cd_nopp) = tables
    partition = np.array(layer_partition)
    starts = np.cumsum(partition) - partition
    ends = np.cumsum(partition) - 1
    q = device_mesh_index

    def t_intra(g, stage_index, l_start, l_end, c):
        l = l_end - l_start + 1
        p = num_stages - stage_index - 1
        if l_start == 0 and l_end == num_layers - 1:
            stable, delta = cs_nopp[g, q, c, 0], cd_nopp[g, q, c, 0]
        elif l_start == 0:
            stable, delta = cs_pre[g, q, p, l - 1, c, 0], cd_pre[g, q, p, l - 1, c, 0]
        elif l_end == num_layers - 1:
            stable, delta = cs_post[g, q, l - 1, c, 0], cd_post[g, q, l - 1, c, 0]
        else:
            stable, delta = cs[g, q, p, l - 1, c, 0], cd[g, q, p, l - 1, c, 0]
        return np.float64(stable) + np.float64(delta) / all_gradient_accumulation_steps[g]

    best_cost, best_g, best_g_index, best_ckpt = np.inf, None, None, None
    for G, g in zip(gradient_accumulation_steps_candidates, gradient_accumulation_steps_index_candidates):
        if simple_activation_checkpointing_tuning_enabled:
            for c in range(0, min(layer_partition) + 1):
                lat = [t_intra(g, s, starts[s], ends[s], c) for s in range(num_stages)]
                if np.inf in lat:
                    continue
                total = max(lat) * (G - 1) + sum(lat)
                if total < best_cost:
                    best_cost, best_g, best_g_index, best_ckpt = total, G, g, [c] * num_stages
        else:
            lat, ckpts = [], []
            for s in range(num_stages):
                if not activation_checkpointing_tuning_enabled:
                    c_best = ends[s] - starts[s] + 1
                    t_best = t_intra(g, s, starts[s], ends[s], c_best)
                else:
                    c_best, t_best = None, np.inf
                    for c in range(ends[s] - starts[s] + 2):
                        t = t_intra(g, s, starts[s], ends[s], c)
                        if t < t_best:
                            t_best, c_best = t, c
                lat.append(t_best)
                ckpts.append(c_best)
            if np.inf in lat:
                continue
            total = max(lat) * (G - 1) + sum(lat)
            if total < best_cost:
                best_cost, best_g, best_g_index, best_ckpt = total, G, g, ckpts
    return best_cost, best_g, best_g_index, best_ckpt


def inter_stage_tune(
    num_layers: int,
    num_nodes: int,
    num_gpus_per_node: int,
    gradient_accumulation_steps_candidates: List[int],
    intra_stage_results: IntraStageTunerOutput,
    config: MistConfig,
):
    """inter_tuning_uniform.py:120-258."""
    if not isinstance(intra_stage_results, IntraStageTunerOutput):
        raise TypeError(
            f"intra_stage_results must be an instance of IntraStageTunerOutput, got {type(intra_stage_results)}"
        )
    r = intra_stage_results
    ckpt_tuning = config.tuning.activation_checkpointing_tuning_enabled
    simple = config.tuning.tuning_granularity == "uniform-pp-simple-heuristic-mem-opt"
    tables = (
        (r.costs_stable, r.costs_stable_with_pre, r.costs_stable_with_post, r.costs_stable_no_pp),
        (r.costs_delta, r.costs_delta_with_pre, r.costs_delta_with_post, r.costs_delta_no_pp),
    )
    all_G = list(r.gradient_accumulation_steps_candidates)
    g_index = {G: i for i, G in enumerate(r.gradient_accumulation_steps_candidates)}
    q_index = {q: i for i, q in enumerate(r.device_mesh_candidates)}
    g_indices = [g_index[G] for G in gradient_accumulation_steps_candidates]

    best = (float("inf"), None, None, None, None)
    for num_stages in range(1, num_layers + 1):
        if num_nodes * num_gpus_per_node % num_stages != 0:
            continue
        partition = _uniform_layer_partition(num_layers, num_stages)
        n, m = _uniform_device_mesh_partition(num_stages, num_nodes, num_gpus_per_node)
        cost, G, g, ckpts = inter_stage_tune_with_fixed_inter_partition(
            num_layers, num_stages, partition, q_index[(n, m)],
            gradient_accumulation_steps_candidates, g_indices, tables, all_G, ckpt_tuning, simple,
        )
        if cost < best[0]:
            best = (cost, G, g, num_stages, ckpts)
    best_cost, best_g, best_g_index, best_num_stages, best_ckpts = best
    if best_g is None:
        return float("inf"), None

    partition = _uniform_layer_partition(num_layers, best_num_stages)
    n, m = _uniform_device_mesh_partition(best_num_stages, num_nodes, num_gpus_per_node)
    q = q_index[(n, m)]
    starts = np.cumsum(partition) - partition
    ends = np.cumsum(partition) - 1
    solutions = [best_g, []]
    for s in range(best_num_stages):
        row = get_solution_from_intra_stage_tuner_output(
            r, num_layers, best_g_index, best_num_stages - s - 1, int(starts[s]), int(ends[s]), q,
            int(best_ckpts[s]), slot=0,
        ).tolist()
        row[:6] = [int(x) for x in row[:6]]
        inter = ((int(starts[s]), int(ends[s])), (n, m), int(best_ckpts[s]), 0)
        solutions[1].append((inter, tuple(row)))
    return float(best_cost), solutions
