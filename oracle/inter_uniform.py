"""Oracle (test infrastructure): uniform inter-stage search.

Restates mist/analyzer/inter_tuning_uniform.py:95-397 (``_uniform_layer_partition``,
``_uniform_device_mesh_partition``, ``inter_stage_tune``,
``inter_stage_tune_with_fixed_inter_partition``; sample 0 only).

Parity unpinned: ``stable + delta / G`` on numpy float32 scalars with a python int
(inter_tuning_uniform.py:316) evaluates in float64 under the reference's numpy 1.24 and in
float32 under numpy >= 2; written here with explicit float64 casts.
Pinned by (tests/test_oracle_dp.py): brute force over (stages, G, ckpt) on tiny tables and the
closed forms of the two partition helpers.
"""
import numpy as np

from .inter_dp import get_intra_solution


def uniform_layer_partition(num_layers, num_stages):
    part = [num_layers // num_stages] * num_stages
    for i in range(num_layers % num_stages):
        part[-i - 1] += 1
    return part


def uniform_device_mesh_partition(num_stages, num_nodes, num_gpus_per_node):
    if num_nodes > num_stages:
        if num_nodes % num_stages != 0:
            return None
        return num_nodes // num_stages, num_gpus_per_node
    if num_stages % num_nodes != 0 or num_gpus_per_node % (num_stages // num_nodes) != 0:
        return None
    return 1, num_gpus_per_node // (num_stages // num_nodes)


def stage_latency(results, num_layers, num_stages, g, q, stage_index, l_start, l_end, c):
    """``t_intra`` of inter_tuning_uniform.py:290-316."""
    l, p = l_end - l_start + 1, num_stages - stage_index - 1
    r = results
    if l_start == 0 and l_end == num_layers - 1:
        s, d = r.costs_stable_no_pp[g, q, c, 0], r.costs_delta_no_pp[g, q, c, 0]
    elif l_start == 0:
        s, d = r.costs_stable_with_pre[g, q, p, l - 1, c, 0], r.costs_delta_with_pre[g, q, p, l - 1, c, 0]
    elif l_end == num_layers - 1:
        s, d = r.costs_stable_with_post[g, q, l - 1, c, 0], r.costs_delta_with_post[g, q, l - 1, c, 0]
    else:
        s, d = r.costs_stable[g, q, p, l - 1, c, 0], r.costs_delta[g, q, p, l - 1, c, 0]
    return np.float64(s) + np.float64(d) / r.gradient_accumulation_steps_candidates[g]


def inter_stage_tune_uniform(num_layers, num_nodes, num_gpus_per_node, grad_accum_candidates,
                             results, ckpt_tuning=True, simple=False):
    """inter_tuning_uniform.py:120-258 + 261-397."""
    g_index = {G: i for i, G in enumerate(results.gradient_accumulation_steps_candidates)}
    q_index = {q: i for i, q in enumerate(results.device_mesh_candidates)}
    best = (float("inf"), None, None, None, None)
    for S in range(1, num_layers + 1):
        if num_nodes * num_gpus_per_node % S != 0:
            continue
        part = np.array(uniform_layer_partition(num_layers, S))
        n, m = uniform_device_mesh_partition(S, num_nodes, num_gpus_per_node)
        q = q_index[(n, m)]
        starts, ends = np.cumsum(part) - part, np.cumsum(part) - 1
        cur = (np.inf, None, None, None)
        for G in grad_accum_candidates:
            g = g_index[G]
            lat = lambda s, c: stage_latency(results, num_layers, S, g, q, s, starts[s], ends[s], c)
            if simple:
                for c in range(0, min(part) + 1):
                    lats = [lat(s, c) for s in range(S)]
                    if np.inf in lats:
                        continue
                    total = max(lats) * (G - 1) + sum(lats)
                    if total < cur[0]:
                        cur = (total, G, g, [c] * S)
                continue
            lats, ckpts = [], []
            for s in range(S):
                if not ckpt_tuning:
                    cb = ends[s] - starts[s] + 1
                    tb = lat(s, cb)
                else:
                    cb, tb = None, np.inf
                    for c in range(ends[s] - starts[s] + 2):
                        t = lat(s, c)
                        if t < tb:
                            tb, cb = t, c
                lats.append(tb)
                ckpts.append(cb)
            if np.inf in lats:
                continue
            total = max(lats) * (G - 1) + sum(lats)
            if total < cur[0]:
                cur = (total, G, g, ckpts)
        if cur[0] < best[0]:
            best = (cur[0], cur[1], cur[2], S, cur[3])
    cost, G, g, S, ckpts = best
    if G is None:
        return float("inf"), None
    part = np.array(uniform_layer_partition(num_layers, S))
    n, m = uniform_device_mesh_partition(S, num_nodes, num_gpus_per_node)
    starts, ends = np.cumsum(part) - part, np.cumsum(part) - 1
    sol = [G, []]
    for s in range(S):
        row = get_intra_solution(results, num_layers, g, S - s - 1, int(starts[s]), int(ends[s]),
                                 q_index[(n, m)], int(ckpts[s]), 0).tolist()
        row[:6] = [int(x) for x in row[:6]]
        sol[1].append((((int(starts[s]), int(ends[s])), (n, m), int(ckpts[s]), 0), tuple(row)))
    return float(cost), sol
