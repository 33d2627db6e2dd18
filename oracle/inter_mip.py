"""Oracle (test infrastructure): inter-stage search of the ``uniform-device-pp-mip`` granularity.

Restates mist/analyzer/inter_tuning_mip.py:
  * ``inter_stage_tune`` (:87-253): for every gradient-accumulation count G and every stage count
    S that divides the device count and splits the cluster into one uniform mesh, solve one
    assignment problem; keep the first strictly better one, starting from ``MAX_VALUE``.
  * ``inter_stage_tune_with_fixed_grad_accumu_and_device_partition`` (:256-424): stage i takes
    ``j`` layers out of ``L_candidates`` (round(L / S) +- layers_offset, clipped; only the average
    when G == 1) and one of the sampled policies ``k`` of (i, j), with stable time ``T_i`` and
    delta time ``D_i``; minimise ``(G - 1) * max_i T_i + sum_i T_i + max(0, max_i (D_i - sum_{j<i}
    T_j))`` subject to ``sum_i j_i == L`` and ``(G - 1) * max_i T_i <= best_cost``.
  * ``preprocess_stable_and_delta_costs`` (:427-535) and ``fill_redundant_samples``
    (mist/utils/pareto.py:158-214): the per-(stage, layer count) policy samples.

The reference hands the problem to PuLP / CBC (absent from this image: ``pulp`` is a dependency
named in the reference's requirements, not vendored).  The problem is small and structured, so
this file solves it exactly instead (``solve``): with ``Z_0 = 0`` and ``Z_{i+1} = T_i + max(Z_i,
D_i)`` the last ``Z_S`` equals ``sum T + max(0, max_i (D_i - sum_{j<i} T_j))`` (induction over i
with ``Z_i = sum_{j<i} T_j + max(0, max_{j<i} (D_j - sum_{j'<j} T_j'))``), ``Z_{i+1}`` is
monotone in ``Z_i`` so the smallest ``Z`` per (stages done, layers used) suffices, and the
optimum's ``max T`` is one of the entry values, so enumerating it as a threshold ``tau`` and
minimising ``Z_S`` over entries with ``T <= tau`` gives the optimum of the MILP.

Tie rule of ``solve`` (a choice of this build, the same in the HIP library's host solver):
thresholds ascending, strict ``<`` on the total; within one threshold every state keeps the
first minimum in (layer count ascending, sample slot ascending) order.

Pinned by (tests/test_oracle_mip.py): ``solve`` against enumeration of every assignment with the
objective written as in the MILP, on random small instances incl. ties, ``inf`` entries and
G == 1; ``fill_redundant_samples`` against the definition (first occurrence of each pair);
``layer_candidates`` against hand-computed cases; the preprocessing against a per-cell scan.
Parity unpinned: which of several optimal assignments CBC returns (solver internals), and its
objective value beyond the solver's tolerances (CBC works to about 1e-7 relative).

Deviations, documented: (1) the reference returns ``best_inter_solution = None`` into
``len()`` when no problem yields a cost below ``MAX_VALUE`` (:214-221 can never see ``inf``);
here that case returns ``(inf, None)`` like the other granularities.  (2) ``with_pre[S - 1]`` and
``costs[S - i - 1]`` index past the pre-saved-micro-batch axis when S exceeds it (IndexError in
the reference); such stages cost ``inf`` here.  (3) a stage count whose uniform split is no mesh
(``_uniform_device_mesh_partition`` returns None, which the reference fails to unpack) is
skipped.
"""
import itertools

import numpy as np

from .inter_uniform_device import uniform_device_mesh_partition
from .pareto import alpha_ratios, compute_indices

MAX_VALUE = 1000000.0  # inter_tuning_mip.py:39


def layer_candidates(num_layers, num_stages, grad_accum, layers_offset=2):
    """inter_tuning_mip.py:282-290 (``round`` is Python's round-half-to-even)."""
    avg = round(num_layers / num_stages)
    if grad_accum == 1:
        return [avg]
    lo = max(avg - layers_offset, 1)
    hi = min(avg + layers_offset, num_layers - num_stages + 1)
    return list(range(lo, hi + 1))


def fill_redundant_samples(costs_x, costs_y, selected_indices, fill_value=np.inf):
    """mist/utils/pareto.py:158-214: per row keep the first occurrence of every distinct
    ``(x, y)`` pair; the kept slot indices come back in the order ``np.unique`` sorts the pairs."""
    batch, sample = selected_indices.shape
    x, y, idx = costs_x.copy(), costs_y.copy(), selected_indices.copy()
    unique = []
    for i in range(batch):
        pairs = np.stack([costs_x[i], costs_y[i]], axis=-1).reshape(-1, 2)
        _, keep = np.unique(pairs, axis=0, return_index=True)
        drop = np.setdiff1d(np.arange(sample), keep)
        x[i, drop] = fill_value
        y[i, drop] = fill_value
        idx[i, drop] = -1
        unique.append(keep.tolist())
    return unique, x, y, idx


def stage_tables(num_stages, stable, delta, stable_pre, delta_pre, stable_post, delta_post,
                 stable_nopp, delta_nopp):
    """inter_tuning_mip.py:448-468: ``t[i, l, c, k]`` of stage i with l layers.  Inputs are one
    (g, q) slice: ``stable`` / ``stable_pre`` (P1, L, L + 1, P), ``stable_post`` (L, L + 1, P),
    ``stable_nopp`` (L + 1, P), float32."""
    S = num_stages
    P1, L, C, P = stable.shape
    assert L == C - 1
    t_stable = np.full((S, L + 1, L + 1, P), np.inf, dtype=np.float32)
    t_delta = np.full((S, L + 1, L + 1, P), np.inf, dtype=np.float32)
    for i in range(1, S - 1):
        if S - i - 1 < P1:
            t_stable[i, 1:] = stable[S - i - 1]
            t_delta[i, 1:] = delta[S - i - 1]
    if S - 1 < P1:
        t_stable[0, 1:] = stable_pre[S - 1]
        t_delta[0, 1:] = delta_pre[S - 1]
    t_stable[S - 1, 1:] = stable_post
    t_delta[S - 1, 1:] = delta_post
    t_stable[0, -1] = stable_nopp
    t_delta[0, -1] = delta_nopp
    return t_stable, t_delta


def preprocess_stable_and_delta_costs(num_stages, ckpt_tuning, fixed_ckpt_value, stable, delta,
                                      stable_pre, delta_pre, stable_post, delta_post,
                                      stable_nopp, delta_nopp):
    """inter_tuning_mip.py:427-535 with ``output_sample_size = P``.  Returns ``(policy_choices,
    t_stable (S, L + 1, P), t_delta, (selected_ckpt, selected_policy))``."""
    S = num_stages
    _, L, _, P = stable.shape
    t_stable, t_delta = stage_tables(S, stable, delta, stable_pre, delta_pre, stable_post,
                                     delta_post, stable_nopp, delta_nopp)
    if ckpt_tuning:
        view_s = t_stable.reshape(S, L + 1, (L + 1) * P)
        view_d = t_delta.reshape(S, L + 1, (L + 1) * P)
    else:
        view_s = np.full((S, L + 1, P), np.inf, dtype=np.float32)
        view_d = np.full((S, L + 1, P), np.inf, dtype=np.float32)
        for l in range(1, L + 1):
            c = fixed_ckpt_value if fixed_ckpt_value is not None else l
            view_s[:, l] = t_stable[:, l, c]
            view_d[:, l] = t_delta[:, l, c]

    out_s = np.full((S, L + 1, P), np.inf, dtype=np.float32)
    out_d = np.full((S, L + 1, P), np.inf, dtype=np.float32)
    sel_ckpt = np.full((S, L + 1, P), -1, dtype=np.int32)
    sel_policy = np.full((S, L + 1, P), -1, dtype=np.int32)
    choices = []
    rows = np.arange(L + 1)[:, None]
    ratios = alpha_ratios(P)
    for i in range(S):
        mask = np.ones(view_s[i].shape, dtype=bool)
        indices = compute_indices(view_s[i], view_d[i], mask, ratios)
        # pareto.py:76-77: an index of -1 (no finite candidate) reads the last candidate.
        x, y = view_s[i][rows, indices], view_d[i][rows, indices]
        keep, x, y, _ = fill_redundant_samples(x, y, indices)
        out_s[i], out_d[i] = x, y
        choices.append(keep)
        if ckpt_tuning:
            sel_ckpt[i], sel_policy[i] = indices // P, indices % P
        else:
            fixed = (np.full(L + 1, fixed_ckpt_value) if fixed_ckpt_value is not None
                     else np.arange(L + 1))
            sel_ckpt[i] = np.broadcast_to(fixed.reshape(-1, 1), (L + 1, P))
            sel_policy[i] = indices
    out_s[out_s < 0] = 0
    out_d[out_d < 0] = 0
    out_s[out_s == np.inf] = MAX_VALUE
    out_d[out_d == np.inf] = MAX_VALUE
    return choices, out_s, out_d, (sel_ckpt, sel_policy)


# ----------------------------------------------------------------------------- the assignment
def objective(T, D, grad_accum):
    """inter_tuning_mip.py:352-361 for fixed stage times: the smallest ``Max_t``, ``Max_d`` the
    constraints allow, then the objective as written."""
    T = [float(v) for v in T]
    D = [float(v) for v in D]
    max_t = max(T)
    max_d = 0.0
    prefix = 0.0
    for t, d in zip(T, D):
        max_d = max(max_d, d - prefix)
        prefix += t
    return max_t * (grad_accum - 1) + sum(T) + max_d


def solve_bruteforce(num_layers, layers, choices, t_stable, t_delta, grad_accum,
                     best_cost=MAX_VALUE):
    """Every assignment of (layer count, slot) per stage; tiny instances only.  ``choices[i][j]``
    lists the slots of stage i with j layers, ``t_*[i, j, k]`` their times.  Returns the optimal
    objective (``inf`` when nothing satisfies the constraints)."""
    S = len(choices)
    per_stage = [[(j, k) for j in layers for k in choices[i][j]] for i in range(S)]
    best = np.inf
    for combo in itertools.product(*per_stage):
        if sum(j for j, _ in combo) != num_layers:
            continue
        T = [t_stable[i, j, k] for i, (j, k) in enumerate(combo)]
        D = [t_delta[i, j, k] for i, (j, k) in enumerate(combo)]
        if max(float(v) for v in T) * (grad_accum - 1) > best_cost:
            continue
        best = min(best, objective(T, D, grad_accum))
    return best


def _chain(num_layers, layers, allowed, T, D):
    """Smallest ``Z_S`` at ``num_layers`` over entries with ``allowed``; returns (Z, picks)."""
    S, nl, P = T.shape
    L = num_layers
    Z = np.full(L + 1, np.inf)
    Z[0] = 0.0
    back = np.full((S, L + 1), -1, dtype=np.int64)
    for i in range(S):
        cand = np.full((L + 1, nl, P), np.inf)
        for a, j in enumerate(layers):
            if j > L:
                continue
            prev = Z[: L + 1 - j]
            step = T[i, a][None, :] + np.maximum(prev[:, None], D[i, a][None, :])
            step = np.where(allowed[i, a][None, :] & np.isfinite(prev)[:, None], step, np.inf)
            cand[j:, a, :] = step
        flat = cand.reshape(L + 1, nl * P)
        arg = np.argmin(flat, axis=1)  # first minimum: layer count ascending, slot ascending
        Z = flat[np.arange(L + 1), arg]
        back[i] = np.where(np.isfinite(Z), arg, -1)
    if not np.isfinite(Z[L]):
        return np.inf, None
    picks, m = [], L
    for i in range(S - 1, -1, -1):
        a, k = divmod(int(back[i, m]), P)
        picks.append((layers[a], k))
        m -= layers[a]
    return float(Z[L]), picks[::-1]


def solve(num_layers, layers, choices, t_stable, t_delta, grad_accum, best_cost=MAX_VALUE):
    """Exact optimum of the assignment problem (module docstring).  Returns ``(cost, [(j, k)
    per stage])`` or ``(inf, None)``."""
    S, P = len(choices), t_stable.shape[-1]
    nl = len(layers)
    T = np.zeros((S, nl, P))
    D = np.zeros((S, nl, P))
    allowed = np.zeros((S, nl, P), dtype=bool)
    for i in range(S):
        for a, j in enumerate(layers):
            T[i, a] = t_stable[i, j].astype(np.float64)
            D[i, a] = t_delta[i, j].astype(np.float64)
            allowed[i, a, list(choices[i][j])] = True
    z_free, picks_free = _chain(num_layers, layers, allowed, T, D)
    if picks_free is None:
        return np.inf, None
    if grad_accum == 1:
        return z_free, picks_free
    best, best_picks = np.inf, None
    for tau in np.unique(T[allowed]):
        weight = (grad_accum - 1) * float(tau)
        if weight > best_cost or weight + z_free >= best:
            break
        z, picks = _chain(num_layers, layers, allowed & (T <= tau), T, D)
        if picks is not None and weight + z < best:
            best, best_picks = weight + z, picks
    return (best, best_picks) if best_picks is not None else (np.inf, None)


def tune_fixed(num_layers, num_stages, grad_accum, tables, device_mesh, best_cost=MAX_VALUE,
               ckpt_tuning=True, layers_offset=2, fixed_ckpt_value=None):
    """inter_tuning_mip.py:256-424 with ``solve`` in the solver's place.  ``tables`` = the eight
    (g, q) slices in the order of ``preprocess_stable_and_delta_costs``."""
    layers = layer_candidates(num_layers, num_stages, grad_accum, layers_offset)
    choices, t_s, t_d, (sel_ckpt, sel_policy) = preprocess_stable_and_delta_costs(
        num_stages, ckpt_tuning, fixed_ckpt_value, *tables)
    cost, picks = solve(num_layers, layers, choices, t_s, t_d, grad_accum, best_cost)
    if picks is None:
        return np.inf, None
    solution, covered = [], 0
    for i, (j, k) in enumerate(picks):
        solution.append(((covered, covered + j - 1), device_mesh,
                         int(sel_ckpt[i][j][k]), int(sel_policy[i][j][k])))
        covered += j
    return cost, solution


def get_intra_solution(results, num_layers, g, p, layer_start, layer_end, q, c, k):
    """inter_tuning_mip.py:62-84."""
    l = layer_end - layer_start + 1
    if layer_start == 0 and layer_end == num_layers - 1:
        return results.solutions_no_pp[g, q, c, k]
    if layer_start == 0:
        return results.solutions_with_pre[g, q, p, l - 1, c, k]
    if layer_end == num_layers - 1:
        return results.solutions_with_post[g, q, l - 1, c, k]
    return results.solutions[g, q, p, l - 1, c, k]


def inter_stage_tune(num_layers, num_nodes, num_gpus_per_node, meshes, grad_accum_candidates,
                     results, config):
    """inter_tuning_mip.py:87-253."""
    f32 = lambda a: np.asarray(a).astype(np.float32)
    tabs = [f32(results.costs_stable), f32(results.costs_delta),
            f32(results.costs_stable_with_pre), f32(results.costs_delta_with_pre),
            f32(results.costs_stable_with_post), f32(results.costs_delta_with_post),
            f32(results.costs_stable_no_pp), f32(results.costs_delta_no_pp)]
    g_index = {g: i for i, g in enumerate(results.gradient_accumulation_steps_candidates)}
    q_index = {q: i for i, q in enumerate(results.device_mesh_candidates)}
    tuning = config.tuning
    best_cost, best = MAX_VALUE, None
    for G in grad_accum_candidates:
        g = g_index[G]
        for S in range(1, num_layers + 1):
            if num_nodes * num_gpus_per_node % S != 0:
                continue
            mesh = uniform_device_mesh_partition(S, num_nodes, num_gpus_per_node)
            if mesh is None or mesh not in q_index:
                continue
            q = q_index[mesh]
            cost, sol = tune_fixed(
                num_layers, S, G, [t[g, q] for t in tabs], mesh, best_cost=best_cost,
                ckpt_tuning=tuning.activation_checkpointing_tuning_enabled,
                layers_offset=getattr(tuning, "layers_offset", 2),
                fixed_ckpt_value=getattr(config, "fixed_ckpt_value", None))
            if cost < best_cost:
                best_cost, best = cost, (G, g, sol)
    if best is None:
        return float("inf"), None
    G, g, inter = best
    S = len(inter)
    out = [G, []]
    for i, entry in enumerate(inter):
        (l0, l1), mesh, ckpt, policy = entry
        row = get_intra_solution(results, num_layers, g, S - i - 1, l0, l1, q_index[mesh],
                                 ckpt, policy).tolist()
        row[:6] = [int(v) for v in row[:6]]
        out[1].append((entry, tuple(row)))
    return best_cost, out
