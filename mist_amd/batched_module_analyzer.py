"""Operator boundary of the intra-stage search: the drop-in for the reference's
``batched_tune_best_latency_for_stage`` (mist/analyzer/batched_module_analyzer.py:581-684), the
function ``IntraStageTuner.tune`` calls once per (gradient-accumulation steps, device mesh)
(mist/analyzer/intra_tuning.py:213).

Same positional arguments, same return value: four tuples ``(costs_stable, costs_delta,
solutions)`` for a middle stage, the first stage (``with_pre``), the last stage (``with_post``)
and the single stage (``no_pp``), float64, ``inf`` where nothing is feasible or the reference
leaves the cell unwritten; shapes ``(P+1, L, C+1, S[, 10])``, ``(L, C+1, S[, 10])`` and
``(C+1, S[, 10])``.  The three ``LayerInfo`` arguments of the reference (traced symbolic
expressions) are replaced by one layer-table provider (``mist_amd.layer_tables.LayerTables`` or
``mist_amd.node_database.DatabaseLayerTables``) that answers for the block, pre and post layers;
it is passed as ``block_layer_info`` and ``pre_layer_info`` / ``post_layer_info`` must be the
same object or ``None``.  The work runs on the GPU (one group through the same three kernels as
a whole tuner call); there is no CPU path.
"""
from __future__ import annotations

from typing import Optional, Sequence

import numpy as np

from .intra_tuning import IntraStageTuner

N_FEATURES = 10  # (b, dp, tp, wre, gre, ore, wo, go, oo, ao), batched_module_analyzer.py:609-613


def _sequential(cands: Sequence[int], lo: int, name: str) -> int:
    """The reference's own precondition (:596-604)."""
    assert set(cands) == set(range(lo, max(cands) + 1)), f"{name}: {cands} is not sequential"
    return int(max(cands))


def batched_tune_best_latency_for_stage(
    block_layer_info,
    pre_layer_info,
    post_layer_info,
    pre_saved_micro_batches_candidates: Sequence[int],
    num_layers_candidates: Sequence[int],
    num_ckpt_layers_candidates: Sequence[int],
    num_nodes: int,
    num_gpus_per_node: int,
    gradient_accumulation_steps: int,
    config,
    tp_size: Optional[int] = None,
    sample_size: Optional[int] = None,
    device: str = "cuda:0",
):
    for other in (pre_layer_info, post_layer_info):
        if other is not None and other is not block_layer_info:
            raise ValueError(
                "pre_layer_info / post_layer_info must be the block layer's table provider (or "
                "None): one provider answers for all three layer kinds here"
            )
    P = _sequential(pre_saved_micro_batches_candidates, 0, "pre_saved_micro_batches_candidates")
    L = _sequential(num_layers_candidates, 1, "num_layers_candidates")
    C = _sequential(num_ckpt_layers_candidates, 0, "num_ckpt_layers_candidates")
    if C != L:
        # the reference's tuner always passes 0..L (intra_tuning.py:200-201); the kernels number
        # the (layers, ckpt) pairs of that triangle
        raise ValueError(f"num_ckpt_layers_candidates must be 0..{L} (got 0..{C})")
    if sample_size is None:
        sample_size = config.tuning.sample_size  # the reference reads config.sample_size (:608)
    tuner = IntraStageTuner(
        block_layer_info, L, [(int(num_nodes), int(num_gpus_per_node))],
        [int(gradient_accumulation_steps)], tp_size, config, sample_size=int(sample_size),
        device=device,
    )
    # every requested p is evaluated, whatever G is (the reference's tuner passes
    # range(min(G, L, P + 1)) itself, intra_tuning.py:185-193)
    tuner.max_possible_pre_saved_micro_batches = P
    tuner.evaluate_all_p = True
    res = tuner.tune()
    out = []
    for v in range(4):
        out.append((res.costs_f64("stable", v)[0, 0], res.costs_f64("delta", v)[0, 0],
                    res._solutions(v)[0, 0]))
    S = int(sample_size)
    assert out[0][0].shape == (P + 1, L, C + 1, S) and out[2][2].shape == (L, C + 1, S, N_FEATURES)
    assert out[3][0].shape == (C + 1, S)
    return tuple(out)
