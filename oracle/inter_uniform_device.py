"""Oracle (test infrastructure): inter-stage search with one uniform device mesh per stage count.

Restates mist/analyzer/inter_tuning_uniform_device.py:87-441 (``inter_stage_tune``,
``inter_stage_tune_with_fixed_grad_accumu``, ``inter_stage_tune_dp_impl``,
``_uniform_device_mesh_partition``).  For every stage count S whose uniform split of the
cluster is a mesh candidate, a DP over (s <= S, start layer k) partitions the layers into s
stages that all run on that mesh; the ckpt candidates of a stage of l layers are 0..l, or only l
when ckpt tuning is off (:400-404).  The t_max enumeration, gap rule and stop rule are those of
the per-mesh search (oracle/inter_dp.py).

Like the per-mesh DP the reference reads ``costs / costs_with_pre / ...`` fields its intra tuner
no longer emits; ``oracle.inter_dp.dp_cost_tables`` is the adapter, and stage entries carry a
trailing policy index 0.  One more deviation, documented: the reference indexes the
pre-saved-micro-batch axis with ``p = s - 1`` without a bounds check (numba); a stage count whose
``p`` lies beyond the tables (more pipeline stages than the intra tuner considered) reads out of
bounds there, here such a stage costs +inf.

dtype notes as in oracle/inter_dp.py: ``f``, ``f_stage_max`` and ``stage_cost + f[...]`` float32,
``best + (g - 1) * f_stage_max`` float64; the two scalar expressions of the scan are parity
unpinned (numpy-1.24 legacy promotion written out with explicit casts).

Pinned by (tests/test_oracle_dp.py): brute-force enumeration of every partition and ckpt choice
on tiny instances for both ckpt rules, ``total == sum + (G - 1) * max`` of the returned
partition, and the mesh chosen for each S against the closed form of the uniform split.
"""
import numpy as np

from .inter_dp import dp_cost_tables, get_intra_solution, tmax_candidates


def uniform_device_mesh_partition(num_stages, num_nodes, num_gpus_per_node):
    """inter_tuning_uniform_device.py:68-84: the (n, m) every stage gets when ``num_stages``
    stages share the cluster evenly, or None."""
    if num_nodes > num_stages:
        if num_nodes % num_stages != 0:
            return None
        return num_nodes // num_stages, num_gpus_per_node
    if num_stages % num_nodes != 0 or num_gpus_per_node % (num_stages // num_nodes) != 0:
        return None
    return 1, num_gpus_per_node // (num_stages // num_nodes)


def dp_impl(t_max, num_layers, num_nodes, num_gpus_per_node, meshes, G, costs, costs_pre,
            costs_post, costs_nopp, ckpt_tuning=True):
    """inter_tuning_uniform_device.py:276-441, literal loops (small instances only)."""
    L = num_layers
    P1 = costs.shape[1]
    t_max = np.float32(t_max)

    def t_intra(s, l_start, l_end, q, c):
        l, p = l_end - l_start + 1, s - 1
        if l_start == 0 and l_end == L - 1:
            return costs_nopp[q, c]
        if p >= P1:
            return np.float32(np.inf)  # the reference reads out of bounds here (module docstring)
        if l_start == 0:
            return costs_pre[q, p, l - 1, c]
        if l_end == L - 1:
            return costs_post[q, l - 1, c]
        return costs[q, p, l - 1, c]

    best_total_all, best_res = np.inf, None
    for S in range(1, L + 1):
        mesh = uniform_device_mesh_partition(S, num_nodes, num_gpus_per_node)
        if mesh is None:
            continue
        assert mesh in meshes, f"uniform mesh {mesh} of {S} stages is not a candidate"
        q = max(i for i, nm in enumerate(meshes) if nm == mesh)  # the loop keeps the last match
        f = np.full((S + 1, L + 1), np.inf, dtype=np.float32)
        f_max = np.zeros((S + 1, L + 1), dtype=np.float32)
        arg = np.full((S + 1, L + 1, 2), -1, dtype=np.int32)
        f[0, L] = 0
        with np.errstate(invalid="ignore"):
            for s in range(1, S + 1):
                for k in range(L - s, -1, -1):
                    for i in range(k, L):
                        l = i - k + 1
                        for j in (range(l + 1) if ckpt_tuning else [l]):
                            stage_cost = t_intra(s, k, i, q, j)
                            new_cost = np.float32(stage_cost + f[s - 1, i + 1])
                            if stage_cost <= t_max and new_cost < f[s, k]:
                                f[s, k] = new_cost
                                f_max[s, k] = max(f_max[s - 1, i + 1], stage_cost)
                                arg[s, k] = (i, j)
        best_s, best_total = -1, np.inf
        for s in range(1, S + 1):
            if f[s, 0] < best_total:
                best_s, best_total = s, f[s, 0]
        if np.isinf(best_total):
            continue
        total = float(np.float64(best_total) + np.float64(G - 1) * np.float64(f_max[best_s, 0]))
        res, cs, cl = [], best_s, 0
        while cs > 0 and cl < L:
            end, ckpt = (int(v) for v in arg[cs, cl])
            assert end != -1
            res.append(((cl, end), mesh, ckpt))
            cs, cl = cs - 1, end + 1
        assert cs == 0 and cl == L
        if total < best_total_all:
            best_total_all, best_res = total, res
    return best_total_all, best_res


def tune_fixed_grad_accumu(num_layers, num_nodes, num_gpus_per_node, meshes, G, costs, costs_pre,
                           costs_post, costs_nopp, best_cost=float("inf"), ckpt_tuning=True,
                           dp=dp_impl, trace=None):
    """inter_tuning_uniform_device.py:212-273."""
    best_solution = None
    last = np.float32(0)
    gap = 1e-6
    for t in tmax_candidates(costs, costs_pre, costs_post):
        if float(np.float64(t) * G) >= best_cost:
            break
        if float(np.float32(t - last)) < gap:
            continue
        cost, solution = dp(t, num_layers, num_nodes, num_gpus_per_node, meshes, G, costs,
                            costs_pre, costs_post, costs_nopp, ckpt_tuning)
        if trace is not None:
            trace.append(float(t))
        if cost < best_cost:
            best_cost, best_solution = cost, solution
        last = t
    return best_cost, best_solution


def inter_stage_tune(num_layers, num_nodes, num_gpus_per_node, meshes, grad_accum_candidates,
                     results, config, slot=0, dp=dp_impl):
    """inter_tuning_uniform_device.py:87-209."""
    ckpt_tuning = bool(config.tuning.activation_checkpointing_tuning_enabled)
    best_cost, best_inter, best_G = float("inf"), None, None
    g_index = {g: i for i, g in enumerate(results.gradient_accumulation_steps_candidates)}
    q_index = {q: i for i, q in enumerate(results.device_mesh_candidates)}
    for G in grad_accum_candidates:
        tabs = dp_cost_tables(results, g_index[G], slot)
        cost, sol = tune_fixed_grad_accumu(
            num_layers, num_nodes, num_gpus_per_node, meshes, G, *tabs, best_cost=best_cost,
            ckpt_tuning=ckpt_tuning, dp=dp)
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
