"""Oracle (test infrastructure): inter-stage pipeline-partition DP with t_max enumeration.

Restates mist/analyzer/inter_tuning.py:63-355 (``inter_stage_tune``,
``inter_stage_tune_with_fixed_grad_accumu``, ``inter_stage_tune_dp_impl``).

The reference's DP reads ``intra_stage_results.costs / costs_with_pre / costs_with_post /
costs_no_pp`` (inter_tuning.py:75-92), fields that its own intra tuner no longer produces (it now
emits ``costs_stable*`` / ``costs_delta*`` with a trailing sample axis, intra_tuning.py:59-74).
``dp_cost_tables`` is the adapter both this restatement and the GPU path use:
``cost = costs_stable[..., slot] + costs_delta[..., slot] / G`` in float32 array arithmetic, the
combination the reference's uniform search applies to the same tables
(inter_tuning_uniform.py:300-316), and the DP emits 4-tuples ``(layers, mesh, ckpt, 0)`` so
that ``best_solution_yaml`` (tune_one_case.py:62-101) accepts them.

dtype notes: ``f`` / ``f_stage_max`` and ``stage_cost + f[...]`` are float32
(inter_tuning.py:281-295,326); the final ``best + (g - 1) * f_stage_max`` is float64.
Parity unpinned: the two scalar expressions of the scan, ``t_max * G >= best`` and
``t_max - last < 1e-6`` (inter_tuning.py:196-199), depend on numpy-1.24 legacy scalar promotion
in the reference (float32 scalar with python int -> float64; float32 difference compared with a
python float in float64); they are written here with explicit casts that reproduce 1.24.

Pinned by (tests/test_oracle_dp.py): brute-force enumeration of every partition on tiny
instances, ``total == sum(stage) + (G - 1) * max(stage)`` for the returned partition,
monotonicity of the sum part in t_max, and the single-mesh L = 1 special case
``min_c cost_no_pp[c]``.  The optional C build (oracle/dp.c) is checked against this module.
"""
import numpy as np


def dp_cost_tables(results, g_index, slot=0):
    """Adapter: float32 ``(costs, costs_with_pre, costs_with_post, costs_no_pp)`` for one
    gradient-accumulation candidate from the stable / delta tables."""
    G = results.gradient_accumulation_steps_candidates[g_index]
    out = []
    for suffix in ("", "_with_pre", "_with_post", "_no_pp"):
        stable = np.asarray(getattr(results, "costs_stable" + suffix), dtype=np.float32)
        delta = np.asarray(getattr(results, "costs_delta" + suffix), dtype=np.float32)
        with np.errstate(invalid="ignore"):
            out.append((stable[g_index, ..., slot] + delta[g_index, ..., slot] / G).astype(np.float32))
    return tuple(out)


def max_num_stages(device_mesh_candidates, num_layers):
    """inter_tuning.py:278-280."""
    return min(max(n * m for n, m in device_mesh_candidates), num_layers) // 2


def dp_impl(t_max, num_layers, num_devices, meshes, G, costs, costs_pre, costs_post, costs_nopp):
    """inter_tuning.py:220-355, literal loops (small instances only).  Returns
    ``(total_cost, [((l0, l1), (n, m), ckpt), ...])`` or ``(inf, None)``."""
    L, D = num_layers, num_devices
    t_max = np.float32(t_max)

    def t_intra(s, l_start, l_end, q, c):
        l, p = l_end - l_start + 1, s - 1
        if l_start == 0 and l_end == L - 1:
            return costs_nopp[q, c]
        if l_start == 0:
            return costs_pre[q, p, l - 1, c]
        if l_end == L - 1:
            return costs_post[q, l - 1, c]
        return costs[q, p, l - 1, c]

    S = max_num_stages(meshes, L)
    f = np.full((S + 1, L + 1, D + 1), np.inf, dtype=np.float32)
    f_max = np.zeros((S + 1, L + 1, D + 1), dtype=np.float32)
    arg = np.full((S + 1, L + 1, D + 1, 4), -1, dtype=np.int32)
    f[0, L, 0] = 0
    with np.errstate(invalid="ignore"):
        for s in range(1, S + 1):
            for k in range(L - s, -1, -1):
                for d in range(1, D + 1):
                    for q, (n, m) in enumerate(meshes):
                        if n * m > d:
                            continue
                        for i in range(k, L):
                            prev = f[s - 1, i + 1, d - n * m]
                            for j in range(L - i + 1):
                                stage_cost = t_intra(s, k, i, q, j)
                                new_cost = np.float32(stage_cost + prev)
                                if stage_cost <= t_max and new_cost < f[s, k, d]:
                                    f[s, k, d] = new_cost
                                    f_max[s, k, d] = max(f_max[s - 1, i + 1, d - n * m], stage_cost)
                                    arg[s, k, d] = (i, n, m, j)
    best_s, best_total = -1, np.inf
    for s in range(1, S + 1):
        if f[s, 0, D] < best_total:
            best_s, best_total = s, f[s, 0, D]
    if np.isinf(best_total):
        return np.inf, None
    total = float(np.float64(best_total) + np.float64(G - 1) * np.float64(f_max[best_s, 0, D]))
    res, cs, cl, cd = [], best_s, 0, D
    while cs > 0 and cl < L and cd > 0:
        end, n, m, ckpt = (int(v) for v in arg[cs, cl, cd])
        assert end != -1
        res.append(((cl, end), (n, m), ckpt))
        cs, cl, cd = cs - 1, end + 1, cd - n * m
    assert cs == 0 and cl == L and cd == 0
    return total, res


def tmax_candidates(costs, costs_pre, costs_post):
    """inter_tuning.py:180-186: ascending unique finite values of the three tables."""
    allv = np.concatenate((costs.flatten(), costs_pre.flatten(), costs_post.flatten()))
    allv = np.sort(np.unique(allv))
    return allv[allv != np.inf]


def tune_fixed_grad_accumu(
    num_layers, num_devices, meshes, G, costs, costs_pre, costs_post, costs_nopp,
    best_cost=float("inf"), dp=dp_impl, trace=None,
):
    """inter_tuning.py:163-217.  ``trace`` (a list) receives every t_max the DP was run for."""
    best_solution = None
    last = np.float32(0)
    gap = 1e-6
    for t in tmax_candidates(costs, costs_pre, costs_post):
        if float(np.float64(t) * G) >= best_cost:  # float32 scalar * python int -> float64 (numpy 1.24)
            break
        if float(np.float32(t - last)) < gap:  # float32 difference, compared in float64
            continue
        cost, solution = dp(t, num_layers, num_devices, meshes, G, costs, costs_pre, costs_post, costs_nopp)
        if trace is not None:
            trace.append(float(t))
        if cost < best_cost:
            best_cost, best_solution = cost, solution
        last = t
    return best_cost, best_solution


def get_intra_solution(results, num_layers, g, p, layer_start, layer_end, q, c, slot=0):
    """inter_tuning.py:38-60 with the sample slot made explicit."""
    l = layer_end - layer_start + 1
    if layer_start == 0 and layer_end == num_layers - 1:
        return results.solutions_no_pp[g, q, c, slot]
    if layer_start == 0:
        return results.solutions_with_pre[g, q, p, l - 1, c, slot]
    if layer_end == num_layers - 1:
        return results.solutions_with_post[g, q, l - 1, c, slot]
    return results.solutions[g, q, p, l - 1, c, slot]


def inter_stage_tune(num_layers, num_devices, meshes, grad_accum_candidates, results, slot=0, dp=dp_impl):
    """inter_tuning.py:63-160 on top of ``dp_cost_tables``; returns ``(best_cost,
    [G, [(((l0, l1), (n, m), ckpt, 0), strategy_row), ...]])`` or ``(inf, None)``."""
    best_cost, best_inter, best_G = float("inf"), None, None
    g_index = {g: i for i, g in enumerate(results.gradient_accumulation_steps_candidates)}
    q_index = {q: i for i, q in enumerate(results.device_mesh_candidates)}
    for G in grad_accum_candidates:
        tabs = dp_cost_tables(results, g_index[G], slot)
        cost, sol = tune_fixed_grad_accumu(
            num_layers, num_devices, meshes, G, *tabs, best_cost=best_cost, dp=dp
        )
        if cost < best_cost:
            best_cost, best_G, best_inter = cost, G, sol
    if best_inter is None:
        return float("inf"), None
    solution = [best_G, []]
    n_stages = len(best_inter)
    for i, ((l0, l1), (n, m), ckpt) in enumerate(best_inter):
        row = get_intra_solution(
            results, num_layers, g_index[best_G], n_stages - i - 1, l0, l1, q_index[(n, m)], ckpt, slot
        ).tolist()
        row[:6] = [int(x) for x in row[:6]]
        solution[1].append((((l0, l1), (n, m), ckpt, 0), tuple(row)))
    return best_cost, solution
