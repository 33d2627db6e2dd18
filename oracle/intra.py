"""Oracle (test infrastructure): intra-stage driver.

Restates ``IntraStageTuner.tune`` (mist/analyzer/intra_tuning.py:84-282): loops the gradient
accumulation candidates and device meshes, calls the per-stage evaluation and pads the results
into ``(g, q, p+1, L, L+1, S[, 10])`` tables; cost tables are float32, solutions float64 with
``inf`` fill.  ``indices`` tables (int64, -1 fill) are an addition for comparisons.

Pinned by: shape / padding invariants and the per-group tables being sub-blocks of the packed
tables (tests/test_oracle_stage.py).
"""
from dataclasses import dataclass
from typing import List, Tuple

import numpy as np

from .stage import batched_tune_best_latency_for_stage


@dataclass(frozen=True)
class IntraStageTunerOutput:
    """intra_tuning.py:59-82 (+ ``indices*``)."""

    gradient_accumulation_steps_candidates: List[int]
    device_mesh_candidates: List[Tuple[int, int]]
    costs_stable: np.ndarray
    costs_stable_with_pre: np.ndarray
    costs_stable_with_post: np.ndarray
    costs_stable_no_pp: np.ndarray
    costs_delta: np.ndarray
    costs_delta_with_pre: np.ndarray
    costs_delta_with_post: np.ndarray
    costs_delta_no_pp: np.ndarray
    solutions: np.ndarray
    solutions_with_pre: np.ndarray
    solutions_with_post: np.ndarray
    solutions_no_pp: np.ndarray
    indices: np.ndarray = None
    indices_with_pre: np.ndarray = None
    indices_with_post: np.ndarray = None
    indices_no_pp: np.ndarray = None


def max_pre_saved_micro_batches(device_mesh_candidates, grad_accum_candidates, num_layers):
    """intra_tuning.py:117-126."""
    max_stages = min(max(n * m for n, m in device_mesh_candidates), num_layers)
    return min(max_stages, max(grad_accum_candidates)) - 1


def _set_corner(array, value):
    """``_np_set_item`` (intra_tuning.py:48-56)."""
    array[tuple(slice(0, v) for v in value.shape)] = value


def intra_stage_tune(
    tables,
    config,
    num_layers,
    device_mesh_candidates,
    gradient_accumulation_steps_candidates,
    tp_size,
    sample_size,
    groups=None,
):
    """intra_tuning.py:169-282.  ``groups`` optionally restricts the work to a list of (g, q)
    index pairs (used to time a bounded sample); all other cells stay ``inf``."""
    Gs, Q = list(gradient_accumulation_steps_candidates), list(device_mesh_candidates)
    g_n, q_n, L, S, F = len(Gs), len(Q), num_layers, sample_size, 10
    P = max_pre_saved_micro_batches(Q, Gs, L)
    inf = lambda *shape: np.full(shape, np.inf)
    neg = lambda *shape: np.full(shape, -1, dtype=np.int64)
    cs = [inf(g_n, q_n, P + 1, L, L + 1, S), inf(g_n, q_n, P + 1, L, L + 1, S),
          inf(g_n, q_n, L, L + 1, S), inf(g_n, q_n, L + 1, S)]
    cd = [a.copy() for a in cs]
    sol = [inf(*a.shape, F) for a in cs]
    idx = [neg(*a.shape) for a in cs]
    for g, G in enumerate(Gs):
        for q, (n, m) in enumerate(Q):
            if groups is not None and (g, q) not in groups:
                continue
            p_cands = list(range(min(G, L, P + 1)))
            res = batched_tune_best_latency_for_stage(
                tables,
                config,
                p_cands,
                list(range(1, L + 1)),
                list(range(0, L + 1)),
                n,
                m,
                G,
                tp_size=tp_size,
                sample_size=S,
            )
            for v in range(4):
                _set_corner(cs[v][g, q], res[v][0])
                _set_corner(cd[v][g, q], res[v][1])
                _set_corner(sol[v][g, q], res[v][2])
                _set_corner(idx[v][g, q], res[v][3])
    cs = [a.astype(np.float32) for a in cs]  # intra_tuning.py:244-259
    cd = [a.astype(np.float32) for a in cd]
    return IntraStageTunerOutput(
        Gs, Q, cs[0], cs[1], cs[2], cs[3], cd[0], cd[1], cd[2], cd[3],
        sol[0], sol[1], sol[2], sol[3], idx[0], idx[1], idx[2], idx[3],
    )
