"""Oracle (test infrastructure): alpha-weighted argmin sampling over the candidate axis.

Restates ``sample_pareto_frontier`` (mist/utils/pareto.py:8-85, the path taken when
``alpha_based_sample_size == sample_size``) and ``compute_indices`` (:124-144).

Semantics: for ``alpha_k = linspace(0, 1, S + 2)[1:-1]``, ``r_k = alpha_k / (1 - alpha_k)``
(float64), every batch row picks ``argmin_k' r_k * x[k'] + y[k']`` over ``mask``-ed candidates
in float64, strict ``<`` from ``(inf, -1)`` so the first index wins ties and a row with no
feasible candidate returns -1.

Pinned by: S = 1 reduces to ``np.argmin(x + y)`` first-occurrence (numpy library routine); for
any S the reference's own numpy formulation (pareto.py:87-122) gives the same indices.
Parity unpinned: the reference's kernel is compiled with numba ``fastmath=True``, which allows
contracting ``r * x + y`` into one fused multiply-add or reassociating ``alpha/(1-alpha)*x``;
both are no-ops for S = 1 (r == 1.0 exactly) and undetermined for S > 1.  This restatement
uses the unfused float64 product and sum.
"""
import numpy as np


def alpha_ratios(sample_size):
    alpha = np.linspace(0, 1, sample_size + 2)[1:-1]
    return alpha / (1 - alpha)


def compute_indices(costs_x, costs_y, mask, ratios):
    """pareto.py:124-144 with ``ratios[k] = alpha_k / (1 - alpha_k)``; returns (batch, S) int64.

    Vectorised: ``inf`` where masked out, ``argmin`` picks the first minimum; an all-masked (or
    all-``inf``) row returns -1 like the strict-``<`` scan from ``min_cost = inf``."""
    x = np.asarray(costs_x).astype(np.float64)
    y = np.asarray(costs_y).astype(np.float64)
    mask = np.broadcast_to(np.asarray(mask, dtype=bool), x.shape)
    out = np.empty((x.shape[0], len(ratios)), dtype=np.int64)
    for k, r in enumerate(ratios):
        cost = np.float64(r) * x + y
        cost = np.where(mask, cost, np.inf)
        # NaN never satisfies ``cost < min_cost``; make it lose here as well.
        cost = np.where(np.isnan(cost), np.inf, cost)
        idx = np.argmin(cost, axis=-1)
        best = cost[np.arange(x.shape[0]), idx]
        out[:, k] = np.where(np.isinf(best), -1, idx)
    return out


def compute_indices_scan(costs_x, costs_y, mask, ratios):
    """Literal loop form of pareto.py:124-144 (small inputs only)."""
    batch, feat = costs_x.shape
    out = np.empty((batch, len(ratios)), dtype=np.int64)
    for i, r in enumerate(ratios):
        for j in range(batch):
            min_index, min_cost = -1, np.inf
            for k in range(feat):
                if mask[j, k]:
                    cost = np.float64(r) * np.float64(costs_x[j, k]) + np.float64(costs_y[j, k])
                    if cost < min_cost:
                        min_cost, min_index = cost, k
            out[j, i] = min_index
    return out


def sample_pareto_frontier(costs_x, costs_y, sample_size, mask=None):
    """pareto.py:8-85 for ``alpha_based_sample_size == sample_size``; returns indices only."""
    if mask is None:
        mask = np.ones_like(costs_x, dtype=bool)
    return compute_indices(costs_x, costs_y, mask, alpha_ratios(sample_size))
