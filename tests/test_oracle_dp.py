"""Pins the oracle's inter-stage searches by brute force on tiny instances and invariants."""
import itertools

import numpy as np
import pytest

from oracle.dp_c import dp_impl_c
from oracle.inter_dp import dp_impl, max_num_stages, tmax_candidates, tune_fixed_grad_accumu
from oracle.inter_uniform import uniform_device_mesh_partition, uniform_layer_partition


def _tables(rng, Q, P1, L, inf_frac=0.15, quantum=None):
    def rand(shape):
        a = rng.uniform(0.1, 1.0, size=shape).astype(np.float32)
        if quantum:
            a = (np.round(a / quantum) * quantum).astype(np.float32)
        a[rng.random(shape) < inf_frac] = np.inf
        return a
    return rand((Q, P1, L, L + 1)), rand((Q, P1, L, L + 1)), rand((Q, L, L + 1)), rand((Q, L + 1))


def _stage_cost(tabs, L, s_from_last, k, i, q, j):
    costs, pre, post, nopp = tabs
    l, p = i - k + 1, s_from_last - 1
    if k == 0 and i == L - 1:
        return nopp[q, j]
    if k == 0:
        return pre[q, p, l - 1, j]
    if i == L - 1:
        return post[q, l - 1, j]
    return costs[q, p, l - 1, j]


def _brute_force(t_max, L, D, meshes, tabs):
    """min over every (stage count, layer split, mesh assignment, ckpt choice) of the float32
    suffix-accumulated stage-cost sum, subject to cost <= t_max and devices summing to D."""
    S = max_num_stages(meshes, L)
    best = np.float32(np.inf)
    for n_stages in range(1, S + 1):
        for cuts in itertools.combinations(range(1, L), n_stages - 1):
            bounds = [0, *cuts, L]
            spans = [(bounds[a], bounds[a + 1] - 1) for a in range(n_stages)]
            for qs in itertools.product(range(len(meshes)), repeat=n_stages):
                if sum(meshes[q][0] * meshes[q][1] for q in qs) != D:
                    continue
                # independent minimum per stage is valid for the SUM in exact arithmetic only;
                # enumerate ckpt choices explicitly to stay faithful to float32 accumulation.
                options = []
                for a, ((k, i), q) in enumerate(zip(spans, qs)):
                    s_from_last = n_stages - a
                    options.append([
                        _stage_cost(tabs, L, s_from_last, k, i, q, j) for j in range(L - i + 1)
                        if _stage_cost(tabs, L, s_from_last, k, i, q, j) <= t_max
                    ])
                if any(len(o) == 0 for o in options):
                    continue
                for combo in itertools.product(*options):
                    acc = np.float32(0)
                    for cst in reversed(combo):  # the DP accumulates from the last stage
                        acc = np.float32(cst + acc)
                    best = min(best, acc)
    return best


@pytest.mark.parametrize("L,D,meshes,seed", [
    (4, 4, [(1, 1), (1, 2), (1, 4)], 0),
    (5, 4, [(1, 1), (1, 2), (1, 4)], 1),
    (5, 6, [(1, 2), (1, 4), (2, 4)], 2),
    (4, 8, [(1, 1), (1, 2), (1, 4), (1, 8)], 3),
])
def test_dp_sum_equals_brute_force(L, D, meshes, seed):
    rng = np.random.default_rng(seed)
    P1 = max_num_stages(meshes, L) + 1
    tabs = _tables(rng, len(meshes), P1, L, quantum=0.125 if seed % 2 else None)
    hits = 0
    for t in (0.3, 0.55, 0.8, 1.1):
        cost, sol = dp_impl(t, L, D, meshes, 3, *tabs)
        want = _brute_force(np.float32(t), L, D, meshes, tabs)
        if sol is None:
            assert np.isinf(want)
            continue
        hits += 1
        # the returned partition is consistent: total = sum + (G - 1) * max over its stages
        stage = [
            _stage_cost(tabs, L, len(sol) - a, l0, l1, meshes.index(mesh), ckpt)
            for a, ((l0, l1), mesh, ckpt) in enumerate(sol)
        ]
        assert all(c <= np.float32(t) for c in stage)
        assert sum(n * m for _, (n, m), _ in sol) == D
        assert sol[0][0][0] == 0 and sol[-1][0][1] == L - 1
        acc = np.float32(0)
        for c in reversed(stage):
            acc = np.float32(c + acc)
        assert acc == want  # optimal sum
        assert cost == float(np.float64(acc) + 2 * np.float64(max(stage)))
        assert dp_impl_c(t, L, D, meshes, 3, *tabs) == (cost, sol)
    assert hits > 0


def test_dp_sum_is_monotone_in_tmax_and_c_matches_python():
    rng = np.random.default_rng(11)
    L, D, meshes = 6, 8, [(1, 1), (1, 2), (1, 4), (2, 4)]
    tabs = _tables(rng, len(meshes), 5, L, quantum=0.0625)
    prev = np.inf
    for t in np.linspace(0.2, 1.2, 15):
        a = dp_impl(t, L, D, meshes, 1, *tabs)  # G = 1: total == sum part
        b = dp_impl_c(t, L, D, meshes, 1, *tabs)
        assert a == b
        assert a[0] <= prev
        prev = a[0]
    assert np.isfinite(prev)


def test_single_stage_special_case():
    """One mesh, max_stages == 1 and the ckpt loop range(L - i + 1) = {0, 1}:
    the answer is min(cost_no_pp[0], cost_no_pp[1]) under the threshold."""
    rng = np.random.default_rng(5)
    L, meshes = 3, [(1, 2)]
    tabs = _tables(rng, 1, 2, L, inf_frac=0.0)
    nopp = tabs[3]
    cost, sol = dp_impl(2.0, L, 2, meshes, 4, *tabs)
    j = int(np.argmin(nopp[0, :2]))
    assert sol == [((0, L - 1), (1, 2), j)]
    assert cost == float(np.float64(nopp[0, j]) * 4)  # sum + 3 * max with a single stage


def test_threshold_scan_rules():
    rng = np.random.default_rng(2)
    L, D, meshes = 5, 4, [(1, 1), (1, 2), (1, 4)]
    tabs = _tables(rng, 3, 3, L)
    cands = tmax_candidates(*tabs[:3])
    assert np.all(np.diff(cands) > 0) and np.all(np.isfinite(cands))
    for G in (1, 4, 64):
        trace = []
        best, sol = tune_fixed_grad_accumu(L, D, meshes, G, *tabs, trace=trace)
        # every run threshold respected the gap rule and the stop rule that held when it ran
        assert all(b - a >= 1e-6 for a, b in zip(trace, trace[1:]))
        exhaustive = [(dp_impl(t, L, D, meshes, G, *tabs), t) for t in cands]
        feas = [(c, t) for (c, s), t in exhaustive if s is not None]
        assert best <= min(c for c, _ in feas) + 1e-6 or trace[-1] * G < best
        # an incoming best below every reachable total prunes everything
        pruned = []
        out = tune_fixed_grad_accumu(L, D, meshes, G, *tabs, best_cost=1e-9, trace=pruned)
        assert out == (1e-9, None) and pruned == []
    # the larger G, the earlier the stop rule fires
    t1, t64 = [], []
    tune_fixed_grad_accumu(L, D, meshes, 1, *tabs, trace=t1)
    tune_fixed_grad_accumu(L, D, meshes, 64, *tabs, trace=t64)
    assert len(t64) <= len(t1)


def test_uniform_partitions_closed_form():
    assert uniform_layer_partition(24, 4) == [6, 6, 6, 6]
    assert uniform_layer_partition(10, 4) == [2, 2, 3, 3]  # remainder goes to the last stages
    assert uniform_layer_partition(7, 3) == [2, 2, 3]
    assert uniform_device_mesh_partition(1, 4, 8) == (4, 8)
    assert uniform_device_mesh_partition(2, 4, 8) == (2, 8)
    assert uniform_device_mesh_partition(4, 4, 8) == (1, 8)
    assert uniform_device_mesh_partition(8, 4, 8) == (1, 4)
    assert uniform_device_mesh_partition(3, 4, 8) is None
    assert uniform_device_mesh_partition(32, 4, 8) == (1, 1)
    assert uniform_device_mesh_partition(64, 4, 8) is None


def test_uniform_search_equals_brute_force():
    from oracle.inter_uniform import inter_stage_tune_uniform, stage_latency
    from oracle.intra import intra_stage_tune
    from tests.util import tiny_plan

    L = 4
    cfg, tables = tiny_plan(1, layers=L, hardware__num_nodes=1, hardware__num_gpus_per_node=4,
                            training__global_batch_size=16, hardware__memory_capacity=6.0)
    meshes, Gs = [(1, 1), (1, 2), (1, 4)], [1, 2, 4, 8, 16]
    r = intra_stage_tune(tables, cfg, L, meshes, Gs, 1, 30)
    cost, sol = inter_stage_tune_uniform(L, 1, 4, Gs, r)
    assert sol is not None
    best = np.inf
    for S in (1, 2, 4):
        part = uniform_layer_partition(L, S)
        q = meshes.index(uniform_device_mesh_partition(S, 1, 4))
        starts = np.cumsum(part) - part
        for g, G in enumerate(Gs):
            for ckpts in itertools.product(*[range(part[s] + 1) for s in range(S)]):
                lat = [stage_latency(r, L, S, g, q, s, starts[s], starts[s] + part[s] - 1, ckpts[s]) for s in range(S)]
                if np.inf in lat:
                    continue
                best = min(best, max(lat) * (G - 1) + sum(lat))
    assert cost == pytest.approx(best, rel=1e-12)
    G = sol[0]
    assert sum(l1 - l0 + 1 for ((l0, l1), _, _, _), _ in sol[1]) == L
    for (_, mesh, _, policy), row in sol[1]:
        assert policy == 0 and row[0] * row[1] * G == 16 and row[1] * row[2] == mesh[0] * mesh[1]


def _brute_force_uniform_device(t_max, L, num_nodes, gpn, meshes, tabs, ckpt_tuning, S):
    """min float32 suffix-accumulated sum over every split into s <= S stages and every ckpt
    choice, all stages on the uniform mesh of S stages; also the best s (first on ties)."""
    from oracle.inter_uniform_device import uniform_device_mesh_partition as udmp

    q = meshes.index(udmp(S, num_nodes, gpn))
    best_per_s = []
    for n_stages in range(1, S + 1):
        best = np.float32(np.inf)
        for cuts in itertools.combinations(range(1, L), n_stages - 1):
            bounds = [0, *cuts, L]
            spans = [(bounds[a], bounds[a + 1] - 1) for a in range(n_stages)]
            options = []
            for a, (k, i) in enumerate(spans):
                l = i - k + 1
                js = range(l + 1) if ckpt_tuning else [l]
                cs = [_stage_cost(tabs, L, n_stages - a, k, i, q, j) for j in js]
                options.append([c for c in cs if c <= t_max])
            if any(len(o) == 0 for o in options):
                continue
            for combo in itertools.product(*options):
                acc = np.float32(0)
                for cst in reversed(combo):
                    acc = np.float32(cst + acc)
                best = min(best, acc)
        best_per_s.append(best)
    return best_per_s


@pytest.mark.parametrize("ckpt_tuning", [True, False])
@pytest.mark.parametrize("L,num_nodes,gpn,seed", [(4, 1, 4, 0), (5, 2, 2, 1), (4, 2, 4, 2)])
def test_uniform_device_dp_equals_brute_force(L, num_nodes, gpn, seed, ckpt_tuning):
    from oracle.inter_uniform_device import dp_impl as ud_dp, uniform_device_mesh_partition as udmp

    rng = np.random.default_rng(100 + seed)
    meshes = [(1, 2 ** i) for i in range(gpn.bit_length()) if 2 ** i <= gpn]
    meshes += [(2 ** j, gpn) for j in range(1, num_nodes.bit_length()) if 2 ** j <= num_nodes]
    tabs = _tables(rng, len(meshes), L + 1, L, quantum=0.125 if seed % 2 else None)
    G, hits = 4, 0
    for t in (0.3, 0.55, 0.8, 1.1):
        t32 = np.float32(t)
        cost, sol = ud_dp(t, L, num_nodes, gpn, meshes, G, *tabs, ckpt_tuning=ckpt_tuning)
        # candidates per S: the minimum sum over s <= S (first s on ties); the stage maximum that
        # goes with it is the DP's own, so the total is checked on the returned partition
        sums = {}
        for S in range(1, L + 1):
            if udmp(S, num_nodes, gpn) is None:
                continue
            per_s = _brute_force_uniform_device(t32, L, num_nodes, gpn, meshes, tabs, ckpt_tuning, S)
            if np.isfinite(min(per_s)):
                sums[S] = min(per_s)
        if sol is None:
            assert not sums
            continue
        hits += 1
        mesh = sol[0][1]
        assert all(m == mesh for _, m, _ in sol) and sol[0][0][0] == 0 and sol[-1][0][1] == L - 1
        q = meshes.index(mesh)
        stage = [_stage_cost(tabs, L, len(sol) - a, l0, l1, q, ck) for a, ((l0, l1), _, ck) in enumerate(sol)]
        assert all(c <= t32 for c in stage)
        if not ckpt_tuning:
            assert all(ck == l1 - l0 + 1 for (l0, l1), _, ck in sol)
        acc = np.float32(0)
        for c in reversed(stage):
            acc = np.float32(c + acc)
        assert cost == float(np.float64(acc) + (G - 1) * np.float64(max(stage)))
        # the partition's sum is the optimum (over s <= S) of a stage count S with that mesh
        S_of_mesh = [S for S in sums if udmp(S, num_nodes, gpn) == mesh]
        assert any(acc == sums[S] for S in S_of_mesh)
    assert hits > 0


def test_uniform_device_mesh_closed_form():
    from oracle.inter_uniform_device import uniform_device_mesh_partition as udmp

    assert udmp(1, 4, 8) == (4, 8) and udmp(2, 4, 8) == (2, 8) and udmp(4, 4, 8) == (1, 8)
    assert udmp(8, 4, 8) == (1, 4) and udmp(32, 4, 8) == (1, 1)
    assert udmp(3, 4, 8) is None and udmp(64, 4, 8) is None and udmp(6, 2, 4) is None
    for S in range(1, 40):
        got = udmp(S, 4, 8)
        if got is not None:
            assert got[0] * got[1] * S == 32  # the stages share all devices evenly
