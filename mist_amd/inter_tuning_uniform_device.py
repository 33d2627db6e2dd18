"""Inter-stage search with one uniform device mesh per stage count: drop-in for the reference's
``mist/analyzer/inter_tuning_uniform_device.py`` (``inter_stage_tune`` :87-209,
``inter_stage_tune_with_fixed_grad_accumu`` :212-273, ``inter_stage_tune_dp_impl`` :276-441).

For every stage count S whose even split of the cluster is a mesh candidate the reference runs
a DP over (s <= S, start layer) with all stages on that mesh, ckpt candidates 0..l per stage (only
l when ckpt tuning is off), and keeps the best total over S; thresholds are enumerated as in the
per-mesh search.  Here every S is one *family* of the DP kernel (``free_devices`` shape, see
include/mist_dp.h) and the threshold scan, its exact shortcuts and the replay are shared with
``mist_amd.inter_tuning``.

As for the per-mesh DP, the cost tables come from the stable / delta tables
(``mist_dp_cost_tables``) because the fields the reference reads are no longer produced by its
intra tuner, and stage entries carry a trailing policy index 0.  A stage count whose
pre-saved-micro-batch index lies beyond the tables costs +inf (the reference's numba kernel reads
out of bounds there).
"""
from __future__ import annotations

from typing import List, Optional, Tuple

from .inter_tuning import inter_stage_tune_batch
from .intra_tuning import IntraStageTunerOutput


def inter_stage_tune_batch_uniform_device(
    num_layers: int,
    num_nodes: int,
    num_gpus_per_node: int,
    device_mesh_candidates: List[Tuple[int, int]],
    gradient_accumulation_steps_candidates: List[int],
    results_list: List[IntraStageTunerOutput],
    config,
    slot: int = 0,
    stats: Optional[dict] = None,
    only_best_solution: bool = False,
    table_limit=None,
):
    """All tensor-parallel candidates of one ``tune`` call in one batch of launches."""
    uniform = dict(
        num_nodes=num_nodes, num_gpus_per_node=num_gpus_per_node,
        ckpt_tuning=bool(config.tuning.activation_checkpointing_tuning_enabled),
    )
    return inter_stage_tune_batch(
        num_layers, num_nodes * num_gpus_per_node, device_mesh_candidates,
        gradient_accumulation_steps_candidates, results_list, slot, stats, uniform_device=uniform,
        only_best_solution=only_best_solution, table_limit=table_limit,
    )


def inter_stage_tune(
    num_layers: int,
    num_nodes: int,
    num_gpus_per_node: int,
    device_mesh_candidates: List[Tuple[int, int]],
    gradient_accumulation_steps_candidates: List[int],
    intra_stage_results: IntraStageTunerOutput,
    config,
    slot: int = 0,
    stats: Optional[dict] = None,
):
    """Reference signature (inter_tuning_uniform_device.py:87-95).  Returns ``(best_cost, [G,
    [(((l0, l1), (n, m), ckpt, 0), strategy_row), ...]])`` or ``(inf, None)``."""
    return inter_stage_tune_batch_uniform_device(
        num_layers, num_nodes, num_gpus_per_node, device_mesh_candidates,
        gradient_accumulation_steps_candidates, [intra_stage_results], config, slot, stats,
    )[0]
