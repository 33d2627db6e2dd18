"""GPU parity of the ``uniform-device-pp-mip`` path: the sampling kernel against the oracle's
preprocessing (bit for bit), the end-to-end tuner against the oracle, and at full size the
invariants the assignment must satisfy."""
import ctypes

import numpy as np
import pytest

from tests.util import load_plan, tiny_plan

pytestmark = pytest.mark.gpu


def _random_tables(rng, P1, L, P, inf_frac=0.2, quantum=None, neg_frac=0.0):
    shapes = [(P1, L, L + 1, P), (P1, L, L + 1, P), (L, L + 1, P), (L + 1, P)]
    stable, delta = [], []
    for shape in shapes:
        s = rng.uniform(0.05, 1.0, size=shape)
        d = rng.uniform(0.05, 1.0, size=shape)
        if quantum:
            s, d = np.round(s / quantum) * quantum, np.round(d / quantum) * quantum
        bad = rng.random(shape[:-1]) < inf_frac
        tail = rng.random(shape) < inf_frac / 2
        s[bad], d[bad] = np.inf, np.inf
        s[tail], d[tail] = np.inf, np.inf
        if neg_frac:
            d[(rng.random(shape) < neg_frac) & np.isfinite(d)] *= -1
        stable.append(s)
        delta.append(d)
    return stable, delta


def _gpu_samples(stable, delta, S, lo, hi, mode, fixed):
    import torch
    from mist_amd import _lib
    from mist_amd.intra_tuning import alpha_ratios

    lib = _lib.load()
    P1, L, _, P = stable[0].shape
    dev_s = [torch.from_numpy(np.ascontiguousarray(t)).cuda() for t in stable]
    dev_d = [torch.from_numpy(np.ascontiguousarray(t)).cuda() for t in delta]
    tabs = _lib.MipTables()
    for v in range(4):
        tabs.stable[v], tabs.delta[v] = dev_s[v].data_ptr(), dev_d[v].data_ptr()
    shape = _lib.MipShape(num_layers=L, p_dim=P1, sample_size=P, num_stages=S, layers_min=lo,
                          layers_max=hi, ckpt_mode=mode, fixed_ckpt=fixed)
    n = S * (hi - lo + 1) * P
    ratios = torch.from_numpy(alpha_ratios(P)).cuda()
    ts = torch.empty(n, dtype=torch.float32).cuda()
    td = torch.empty(n, dtype=torch.float32).cuda()
    ix = torch.empty(n, dtype=torch.int32).cuda()
    kp = torch.empty(n, dtype=torch.uint8).cuda()
    rc = lib.mist_mip_stage_samples(
        ctypes.byref(shape), ctypes.byref(tabs), ratios.data_ptr(), ts.data_ptr(), td.data_ptr(),
        ix.data_ptr(), kp.data_ptr(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    _lib.check(rc, "mist_mip_stage_samples")
    torch.cuda.synchronize()
    dims = (S, hi - lo + 1, P)
    return (ts.cpu().numpy().reshape(dims), td.cpu().numpy().reshape(dims),
            ix.cpu().numpy().reshape(dims), kp.cpu().numpy().reshape(dims))


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("L,P1,P,quantum", [(5, 3, 4, 0.125), (12, 6, 9, None), (32, 8, 30, 0.03125)])
def test_sampling_kernel_matches_oracle_preprocessing(mode, L, P1, P, quantum):
    from oracle import inter_mip

    rng = np.random.default_rng(L * 10 + mode)
    fixed = L // 2
    for S in sorted({1, 2, 3, min(P1 + 1, L), L}):
        stable, delta = _random_tables(rng, P1, L, P, quantum=quantum, neg_frac=0.03)
        f32 = lambda a: a.astype(np.float32)
        choices, want_s, want_d, (ck, pol) = inter_mip.preprocess_stable_and_delta_costs(
            S, mode == 0, fixed if mode == 1 else None,
            f32(stable[0]), f32(delta[0]), f32(stable[1]), f32(delta[1]),
            f32(stable[2]), f32(delta[2]), f32(stable[3]), f32(delta[3]))
        lo, hi = 1, L   # every layer count, more than the search itself asks for
        got_s, got_d, got_i, got_k = _gpu_samples(stable, delta, S, lo, hi, mode, fixed)
        assert np.array_equal(got_s, want_s[:, lo:hi + 1]), (S, "stable")
        assert np.array_equal(got_d, want_d[:, lo:hi + 1]), (S, "delta")
        want_k = np.zeros_like(got_k)
        for i in range(S):
            for j in range(lo, hi + 1):
                want_k[i, j - lo, choices[i][j]] = 1
        assert np.array_equal(got_k, want_k), (S, "keep")
        if mode == 0:
            assert np.array_equal(got_i // P, ck[:, lo:hi + 1]) and np.array_equal(got_i % P, pol[:, lo:hi + 1])
        else:
            assert np.array_equal(got_i, pol[:, lo:hi + 1])


def test_sampling_kernel_rejects_bad_arguments():
    import torch
    from mist_amd import _lib

    lib = _lib.load()
    buf = torch.zeros(4096, dtype=torch.float64).cuda()
    tabs = _lib.MipTables()
    for v in range(4):
        tabs.stable[v], tabs.delta[v] = buf.data_ptr(), buf.data_ptr()
    args = (buf.data_ptr(),) * 5 + (None,)
    big = _lib.MipShape(num_layers=400, p_dim=2, sample_size=64, num_stages=2, layers_min=1,
                        layers_max=3, ckpt_mode=0, fixed_ckpt=0)
    assert lib.mist_mip_stage_samples(ctypes.byref(big), ctypes.byref(tabs), *args) == -1
    assert b"LDS" in lib.mist_last_error()
    bad = _lib.MipShape(num_layers=8, p_dim=2, sample_size=4, num_stages=9, layers_min=1,
                        layers_max=3, ckpt_mode=0, fixed_ckpt=0)
    assert lib.mist_mip_stage_samples(ctypes.byref(bad), ctypes.byref(tabs), *args) == -1
    tabs.delta[2] = None
    ok = _lib.MipShape(num_layers=8, p_dim=2, sample_size=4, num_stages=2, layers_min=1,
                       layers_max=3, ckpt_mode=0, fixed_ckpt=0)
    assert lib.mist_mip_stage_samples(ctypes.byref(ok), ctypes.byref(tabs), *args) == -1


@pytest.mark.parametrize(
    "overrides",
    [
        dict(hardware__num_nodes=2, hardware__num_gpus_per_node=4, training__global_batch_size=32,
             hardware__memory_capacity=8.0, tuning__sample_size=4),
        dict(hardware__memory_capacity=5.0, tuning__sample_size=6),
        dict(hardware__num_nodes=1, hardware__num_gpus_per_node=4, training__global_batch_size=16,
             hardware__memory_capacity=6.0, tuning__sample_size=3,
             tuning__activation_checkpointing_tuning_enabled=False),
        dict(hardware__num_nodes=1, hardware__num_gpus_per_node=4, training__global_batch_size=16,
             hardware__memory_capacity=6.0, tuning__sample_size=3, fixed_ckpt_value=2,
             tuning__activation_checkpointing_tuning_enabled=False),
    ],
)
def test_mip_tune_end_to_end_matches_oracle(overrides):
    """YAML in, best strategy out.  The oracle solves the assignment with the same exact method
    and tie rule, on tables the kernels reproduce bit for bit: cost and solution are identical."""
    from mist_amd.tune_one_case import tune
    from oracle.tune import tune as oracle_tune

    cfg, tables = tiny_plan(1, layers=6, tuning__tuning_granularity="uniform-device-pp-mip", **overrides)
    got = tune(cfg)
    want = oracle_tune(cfg, tables)
    assert want[1] is not None, "degenerate case"
    assert got == want


def test_mip_infeasible_plan_returns_inf_none():
    from mist_amd.tune_one_case import tune
    from oracle.tune import tune as oracle_tune

    cfg, tables = tiny_plan(1, layers=4, hardware__memory_capacity=0.2, tuning__sample_size=3,
                            tuning__tuning_granularity="uniform-device-pp-mip")
    assert tune(cfg) == (float("inf"), None)
    assert oracle_tune(cfg, tables) == (float("inf"), None)


def test_mip_needs_every_sample():
    from mist_amd.inter_tuning_mip import inter_stage_tune
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates

    cfg, tables = tiny_plan(1, layers=4)
    hw = cfg.hardware
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    res = IntraStageTuner(tables, 4, meshes, Gs, 1, cfg, sample_size=3, sample_slots=[0]).tune()
    with pytest.raises(ValueError, match="every sample"):
        inter_stage_tune(4, hw.num_nodes, hw.num_gpus_per_node, meshes, Gs, res, cfg)
    with pytest.raises(TypeError):
        inter_stage_tune(4, hw.num_nodes, hw.num_gpus_per_node, meshes, Gs, object(), cfg)


def _check_solution_invariants(cfg, cost, solution):
    """Size-independent checks of a returned strategy: stages tile the layers, all stages use
    the uniform mesh of their count, and the cost equals the objective recomputed from the
    float32 stage times of the chosen table cells."""
    from mist_amd.inter_tuning_uniform import _uniform_device_mesh_partition

    L, hw = cfg.model.num_hidden_layers, cfg.hardware
    G, stages = solution
    S = len(stages)
    mesh = _uniform_device_mesh_partition(S, hw.num_nodes, hw.num_gpus_per_node)
    covered = 0
    for (span, stage_mesh, ckpt, policy), row in stages:
        assert span[0] == covered and span[1] >= span[0]
        covered = span[1] + 1
        assert tuple(stage_mesh) == tuple(mesh)
        assert 0 <= ckpt <= L and 0 <= policy < cfg.tuning.sample_size
        assert np.all(np.isfinite(row)) and len(row) == 10
    assert covered == L
    return G, S, mesh


@pytest.mark.parametrize("plan", [1, 2])
def test_mip_full_size_invariants(plan):
    """Plan 1 and the GPT-7B plan at their real sizes with 30 samples per cell."""
    from mist_amd.inter_tuning_mip import inter_stage_tune
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates
    from oracle.inter_mip import MAX_VALUE, objective

    cfg, tables = load_plan(plan, tuning__tuning_granularity="uniform-device-pp-mip",
                            tuning__sample_size=30)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    tp = 1 if plan == 1 else 2
    res = IntraStageTuner(tables, L, meshes, Gs, tp, cfg, sample_size=30).tune()
    cost, solution = inter_stage_tune(L, hw.num_nodes, hw.num_gpus_per_node, meshes, Gs, res, cfg)
    assert solution is not None and cost < MAX_VALUE
    G, S, mesh = _check_solution_invariants(cfg, cost, solution)
    g, q = Gs.index(G), meshes.index(mesh)
    T, D = [], []
    for i, ((span, _, ckpt, policy), row) in enumerate(solution[1]):
        l, p = span[1] - span[0] + 1, S - i - 1
        if S == 1:
            cell, v = (g, q, ckpt, policy), 3
        elif i == 0:
            cell, v = (g, q, p, l - 1, ckpt, policy), 1
        elif i == S - 1:
            cell, v = (g, q, l - 1, ckpt, policy), 2
        else:
            cell, v = (g, q, p, l - 1, ckpt, policy), 0
        T.append(np.float32(res.device.stable[v][cell].item()))
        D.append(max(np.float32(res.device.delta[v][cell].item()), np.float32(0)))
        assert np.array_equal(res.solution_at(v, cell), np.asarray(row, dtype=np.float64))
    assert objective(T, D, G) == pytest.approx(cost, rel=1e-12, abs=0)


@pytest.mark.parametrize("plan, samples, overrides", [
    (1, 30, {}),
    (2, 3, {}),
    (1, 4, dict(model__num_hidden_layers=9, hardware__num_nodes=2, hardware__num_gpus_per_node=4,
                training__global_batch_size=32, hardware__memory_capacity=10.0)),
])
def test_tables_restricted_to_the_cells_the_assignment_reads(monkeypatch, plan, samples, overrides):
    """``IntraStageTuner.cells_wanted`` with the assignment's own description of what it reads
    (inter_tuning_mip.py:267-290): every cell inside the evaluated tile windows equals the full
    tables, every other cell keeps inf / -1, the windows hold every cell the assignment reads,
    and ``tune`` returns the same cost and strategy either way."""
    import torch

    from mist_amd import _lib, tune_one_case
    from mist_amd.inter_tuning_mip import cells_wanted, layer_candidates
    from mist_amd.inter_tuning_uniform import _uniform_device_mesh_partition
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates
    from mist_amd.tune_one_case import tp_candidates

    cfg, tables = load_plan(plan, tuning__tuning_granularity="uniform-device-pp-mip",
                            tuning__sample_size=samples, **overrides)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    D = hw.num_nodes * hw.num_gpus_per_node
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    tps = tp_candidates(cfg)
    full = IntraStageTuner(tables, L, meshes, Gs, tps, cfg, sample_size=samples).tune_all()[0].batch
    tuner = IntraStageTuner(tables, L, meshes, Gs, tps, cfg, sample_size=samples)
    wanted = tuner.cells_wanted = cells_wanted(L, hw.num_nodes, hw.num_gpus_per_node)
    part = tuner.tune_all()[0].batch

    # which (table row, mesh, layers) were evaluated, from the plan's tile windows
    P1 = full.stable[0].shape[2]
    evaluated = np.zeros((len(tps) * len(Gs), len(meshes), L + 1), dtype=bool)  # [g][q][l]
    p_count = np.zeros((len(tps) * len(Gs), len(meshes)), dtype=np.int64)
    window = {}  # (table row, mesh) -> first and last pair of the evaluated tiles
    for rec in tuner._plan["groups"]:
        first = int(rec["lc_tile_begin"]) * _lib.LC_TILE
        last = first + int(rec["n_lc_tiles"]) * _lib.LC_TILE - 1
        window[int(rec["g_index"]), int(rec["q_index"])] = (first, last)
        for l in range(1, L + 1):
            lo, hi = l * (l + 1) // 2 - 1, l * (l + 1) // 2 - 1 + l
            # a layer count whose pairs straddle a window's edge is evaluated for some ckpt
            # counts only: compared where it lies inside as a whole
            evaluated[rec["g_index"], rec["q_index"], l] = first <= lo and hi <= last
        p_count[rec["g_index"], rec["q_index"]] = rec["num_p"]
    n_inside = n_outside = 0
    for t in range(len(tps)):
        for g, G in enumerate(Gs):
            for q, mesh in enumerate(meshes):
                row = t * len(Gs) + g
                w = wanted(G, mesh)
                if w is not None:  # everything the assignment reads lies inside
                    assert evaluated[row, q, w[0]:w[1] + 1].all() or p_count[row, q] == 0
                for l in range(1, L + 1):
                    inside = evaluated[row, q, l]
                    for v in range(4):
                        if v == 3 and l != L:
                            continue
                        for name in ("stable", "delta", "index"):
                            a, b = getattr(full, name)[v], getattr(part, name)[v]
                            if v <= 1:
                                a, b = a[row, q, :p_count[row, q], l - 1], b[row, q, :p_count[row, q], l - 1]
                            elif v == 2:
                                a, b = a[row, q, l - 1], b[row, q, l - 1]
                            else:
                                a, b = a[row, q], b[row, q]
                            if inside:
                                assert torch.equal(a, b), (tps[t], G, mesh, l, v, name)
                            elif w is None or not (w[0] <= l <= w[1]):
                                # straddling layer counts aside, nothing outside a window is written
                                lo, hi = l * (l + 1) // 2 - 1, l * (l + 1) // 2 - 1 + l
                                first, last = window.get((row, q), (0, -1))
                                if hi < first or lo > last:
                                    empty = torch.isinf(b).all() if name != "index" else (b == -1).all()
                                    assert bool(empty), (tps[t], G, mesh, l, v, name)
                    n_inside += inside
                    n_outside += not inside
    assert n_inside > 0 and n_outside > 0

    results = {}
    for all_cells in (False, True):
        monkeypatch.setattr(tune_one_case, "MIP_EVALUATE_ALL_CELLS", all_cells)
        results[all_cells] = tune_one_case.tune(cfg)
    assert results[False] == results[True]
    assert results[False][1] is not None


@pytest.mark.parametrize("plan, samples, overrides", [
    (2, 3, {}),
    (1, 30, {}),
    (1, 4, dict(model__num_hidden_layers=9, hardware__num_nodes=2, hardware__num_gpus_per_node=4,
                training__global_batch_size=32, hardware__memory_capacity=10.0)),
    (1, 3, dict(model__num_hidden_layers=6, hardware__memory_capacity=0.2)),  # nothing fits
])
def test_batched_search_equals_one_search_per_candidate(plan, samples, overrides):
    """``inter_stage_tune_batch`` (all tensor-parallel candidates of a plan: one sampling launch,
    one copy, ``mist_mip_solve_chains`` with a thread per candidate) against ``inter_stage_tune``
    on each candidate alone and against a python loop over ``mist_mip_solve`` with the
    reference's running bound; with ``only_best_solution`` the strategy of the first best
    candidate only."""
    from mist_amd import _lib
    from mist_amd.config import tp_candidates
    from mist_amd.inter_tuning_mip import inter_stage_tune, inter_stage_tune_batch
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates

    cfg, tables = load_plan(plan, tuning__tuning_granularity="uniform-device-pp-mip",
                            tuning__sample_size=samples, **overrides)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    results = IntraStageTuner(tables, L, meshes, Gs, tp_candidates(cfg), cfg, sample_size=samples).tune_all()
    args = (L, hw.num_nodes, hw.num_gpus_per_node, meshes, Gs)
    stats = {}
    together = inter_stage_tune_batch(*args, results, cfg, stats=stats)
    alone = [inter_stage_tune(*args, r, cfg) for r in results]
    assert together == alone
    assert stats["mip_problems"] % len(results) == 0
    best_only = inter_stage_tune_batch(*args, results, cfg, only_best_solution=True)
    found = [i for i, (_, sol) in enumerate(alone) if sol is not None]
    keep = min(found, key=lambda i: alone[i][0]) if found else None
    assert best_only == [(cost, sol if i == keep else None) for i, (cost, sol) in enumerate(alone)]
    assert (keep is None) == (overrides.get("hardware__memory_capacity") == 0.2)

    # the chains solver against the single-problem solver driven by the reference's loop
    rng = np.random.default_rng(5)
    P, n_chains = samples, 3
    shapes = [(S, lo, hi) for S, lo, hi in [(1, L, L), (2, max(L // 2 - 2, 1), L // 2 + 2), (3, 1, L - 2),
                                            (2, 1, L - 1)] if hi >= lo]
    items = np.zeros(n_chains * len(shapes), dtype=_lib.MIP_ITEM_DTYPE)
    items["num_layers"], items["p_dim"], items["sample_size"] = L, 4, P
    cursor = 0
    for k in range(len(items)):
        S, lo, hi = shapes[k % len(shapes)]
        items["num_stages"][k], items["layers_min"][k], items["layers_max"][k] = S, lo, hi
        items["out_offset"][k] = cursor
        cursor += S * (hi - lo + 1) * P
    t_stable = (np.round(rng.uniform(0.1, 2.0, cursor) * 16) / 16).astype(np.float32)  # ties
    t_delta = (np.round(rng.uniform(0.0, 3.0, cursor) * 8) / 8).astype(np.float32)
    keep_flags = (rng.random(cursor) < 0.8).astype(np.uint8)
    G_of = np.array([1, 4, 16, 64][:len(shapes)], dtype=np.int32)
    lib = _lib.load()
    ptr = lambda a: ctypes.c_void_p(a.ctypes.data)
    cost = np.empty(n_chains)
    winner = np.empty(n_chains, dtype=np.int32)
    layers = np.zeros((n_chains, L), dtype=np.int32)
    slots = np.zeros((n_chains, L), dtype=np.int32)
    _lib.check(lib.mist_mip_solve_chains(ptr(items), ptr(G_of), len(shapes), n_chains, ptr(t_stable),
                                         ptr(t_delta), ptr(keep_flags), ptr(cost), ptr(winner),
                                         ptr(layers), ptr(slots)), "mist_mip_solve_chains")
    for c in range(n_chains):
        best_cost, best = float(_lib.MIP_MAX_VALUE), None
        for i in range(len(shapes)):
            item = items[c * len(shapes) + i]
            S, at = int(item["num_stages"]), int(item["out_offset"])
            shape = _lib.MipShape(num_layers=L, p_dim=4, sample_size=P, num_stages=S,
                                  layers_min=int(item["layers_min"]), layers_max=int(item["layers_max"]))
            one_cost = ctypes.c_double()
            one_layers, one_slots = np.zeros(S, dtype=np.int32), np.zeros(S, dtype=np.int32)
            rc = lib.mist_mip_solve(ctypes.byref(shape), int(G_of[i]), best_cost, ptr(t_stable[at:]),
                                    ptr(t_delta[at:]), ptr(keep_flags[at:]), ctypes.byref(one_cost),
                                    ptr(one_layers), ptr(one_slots))
            assert rc >= 0
            if rc == 1 and one_cost.value < best_cost:
                best_cost, best = one_cost.value, (i, one_layers, one_slots)
        assert cost[c] == best_cost
        assert winner[c] == (best[0] if best else -1)
        if best:
            S = len(best[1])
            assert np.array_equal(layers[c, :S], best[1]) and np.array_equal(slots[c, :S], best[2])
    assert (winner >= 0).any()


@pytest.mark.parametrize("plan, samples, overrides", [
    (1, 30, {}),
    (2, 3, {}),
    (1, 4, dict(model__num_hidden_layers=9, hardware__num_nodes=2, hardware__num_gpus_per_node=4,
                training__global_batch_size=32, hardware__memory_capacity=1.5)),  # some cells fit nothing
])
def test_tables_prefilled_in_the_cells_the_assignment_reads_only(plan, samples, overrides):
    """``IntraStageTuner.prefill_wanted_cells_only`` (what ``tune`` sets for this granularity):
    the tables come from unfilled memory, holding a poison value here, and only the cells
    ``cells_wanted`` names are pre-filled; all of those - every ckpt count, sample and pre-saved
    micro-batch value the assignment can index, with or without a feasible strategy - equal the
    tables of a tuner that fills everything, and so does the search on them."""
    import torch

    from mist_amd.inter_tuning_mip import cells_wanted, inter_stage_tune_batch
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates
    from mist_amd.tune_one_case import tp_candidates

    cfg, tables = load_plan(plan, tuning__tuning_granularity="uniform-device-pp-mip",
                            tuning__sample_size=samples, **overrides)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    tps = tp_candidates(cfg)
    full_results = IntraStageTuner(tables, L, meshes, Gs, tps, cfg, sample_size=samples).tune_all()
    full = full_results[0].batch
    n_cost, n_index = 2 * sum(t.numel() for t in full.stable), sum(t.numel() for t in full.index)
    # the caching allocator hands the blocks of these two back to the next tables of that size
    poison = [torch.full((n_cost,), 0.125, dtype=torch.float64, device="cuda"),
              torch.full((n_index,), 7, dtype=torch.int32, device="cuda")]
    torch.cuda.synchronize()
    del poison
    tuner = IntraStageTuner(tables, L, meshes, Gs, tps, cfg, sample_size=samples)
    wanted = tuner.cells_wanted = cells_wanted(L, hw.num_nodes, hw.num_gpus_per_node)
    tuner.prefill_wanted_cells_only = True
    part_results = tuner.tune_all()
    part = part_results[0].batch
    P1 = full.stable[0].shape[2]
    n_read = n_infeasible = 0
    for t in range(len(tps)):
        for g, G in enumerate(Gs):
            for q, mesh in enumerate(meshes):
                w = wanted(G, mesh)
                if w is None:
                    continue
                row, (lo, hi, p_count) = t * len(Gs) + g, w
                lo, hi, p_count = max(lo, 1), min(hi, L), min(p_count, P1)
                for name in ("stable", "delta", "index"):
                    a, b = getattr(full, name), getattr(part, name)
                    for v in (0, 1):
                        assert torch.equal(a[v][row, q, :p_count, lo - 1:hi], b[v][row, q, :p_count, lo - 1:hi])
                    assert torch.equal(a[2][row, q, lo - 1:hi], b[2][row, q, lo - 1:hi])
                    if hi == L:
                        assert torch.equal(a[3][row, q], b[3][row, q])
                n_read += 1
                n_infeasible += int((full.index[0][row, q, :p_count, lo - 1:hi] == -1).any())
    assert n_read > 0 and n_infeasible > 0
    assert not torch.equal(full.index[0], part.index[0]), "the poison did not reach the tables: nothing tested"
    args = (L, hw.num_nodes, hw.num_gpus_per_node, meshes, Gs)
    assert inter_stage_tune_batch(*args, part_results, cfg) == inter_stage_tune_batch(*args, full_results, cfg)
