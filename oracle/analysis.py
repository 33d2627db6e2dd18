"""Oracle (test infrastructure): the analysis path, i.e. the predicted iteration latency and peak
memory of ONE given strategy.

Restates benchmark/mist/analysis/run.py:37-185 (``analyze``) on top of the
``get_best_solution=False`` outputs of ``batched_stage_analyze``
(mist/analyzer/batched_module_analyzer.py:2788-2803, 2876-2892, 2980-2996, 3063-3079), which
``oracle.stage.batched_stage_analyze`` records when given ``analysis``.

Per stage i of S: pre-saved micro-batches ``min(S - i - 1, G - 1)``, the stage's layer count,
mesh, ckpt count and strategy row from the ``strategy`` block; the first stage uses the with_pre
variant, the last with_post, a single stage pre_and_post.  Total latency (:160-170)

    sum(stable) + max(stable) * (G - 1) + max_s (delta_s - sum_{i < s} stable_i)

or, with ``disable_non_uniform_pp_micro_batch_analysis``, ``sum(latency) + max(latency) * (G - 1)``
(:127-131), or ``latency * G`` for a single stage (:112).

Pinned by: the per-cell quantities are the tuner's own (same arrays, pinned in
tests/test_oracle_stage.py by the scalar re-derivation); the totals by closed-form cases and by
the identity with the assignment objective of ``oracle.inter_mip`` (tests/test_oracle_analysis.py).
"""
import numpy as np

from .stage import batched_stage_analyze


def stage_results(tables, config, stage_idx):
    """``get_stage_results`` (run.py:56-93): the four result dicts' entry for the stage."""
    st = config.strategy
    S, G = st.num_stages, st.gradient_accumulation_steps
    p = min(S - stage_idx - 1, G - 1)
    l = st.layer_partitions[stage_idx]
    n, m = st.device_assignment[stage_idx]
    c = st.gradient_checkpointing[stage_idx]
    analysis = [{}, {}, {}, {}]
    # The oracle's tables are indexed by whole candidate ranges; the wanted cell does not depend
    # on which other cells are computed with it (run.py passes the single values).
    batched_stage_analyze(
        tables, config, list(range(p + 1)), list(range(1, l + 1)), list(range(c + 1)), n, m, G,
        np.asarray(st.stage_strategies[stage_idx], dtype=np.float64), sample_size=1,
        analysis=analysis)
    missing = analysis[3 if S == 1 else (1 if stage_idx == 0 else (2 if stage_idx == S - 1 else 0))].get((p, l, c))
    if missing is None:
        raise KeyError((p, l, c))  # what run.py:84-93 raises on the empty dicts of :868-880
    return [d.get((p, l, c)) for d in analysis]


def _scalar(entry):
    return {k: float(np.asarray(v).reshape(-1)[0]) for k, v in entry.items() if k != "extra_info"}


def analyze(config, tables):
    """run.py:37-185.  Returns ``(total_latency, stage_stable_latencies, stage_delta_latencies,
    stage_peak_memories)``."""
    st = config.strategy
    S, G = st.num_stages, st.gradient_accumulation_steps
    if S == 1:
        r = _scalar(stage_results(tables, config, 0)[3])
        total = r["latency"] * G
        # run.py:113-114 overwrites the stable list with [0] and leaves the delta list empty
        return total, [0], [], [max(r["mem_fwd_peak"], r["mem_bwd_peak"])]
    uniform = bool(getattr(config, "disable_non_uniform_pp_micro_batch_analysis", False))
    stable, delta, peaks = [], [], []
    for i in range(S):
        variant = 1 if i == 0 else (2 if i == S - 1 else 0)
        r = _scalar(stage_results(tables, config, i)[variant])
        if uniform:
            stable.append(r["latency"])
            delta.append(0)
        else:
            stable.append(r["latency_stable"])
            delta.append(r["latency_delta"])
        peaks.append(max(r["mem_fwd_peak"], r["mem_bwd_peak"]))
    total = sum(stable) + max(stable) * (G - 1)
    if not uniform:
        total = total + max(d - sum(stable[i] for i in range(s)) for s, d in enumerate(delta))
    return total, stable, delta, peaks
