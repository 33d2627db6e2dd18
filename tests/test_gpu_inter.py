"""GPU parity of the inter-stage DP and of the end-to-end tuner against the oracle."""
import ctypes

import numpy as np
import pytest

from tests.util import tiny_plan, load_plan

pytestmark = pytest.mark.gpu


def _random_tables(rng, Q, P1, L, inf_frac=0.2, quantum=None):
    def rand(shape):
        a = rng.uniform(0.1, 1.0, size=shape).astype(np.float32)
        if quantum:
            a = (np.round(a / quantum) * quantum).astype(np.float32)  # many exact ties
        a[rng.random(shape) < inf_frac] = np.inf
        return a
    return rand((Q, P1, L, L + 1)), rand((Q, P1, L, L + 1)), rand((Q, L, L + 1)), rand((Q, L + 1))


def _gpu_dp(meshes, L, D, P1, tabs, tmax, want_argmin=False, mode=0, relaid=True):
    import torch
    from mist_amd import _lib

    lib = _lib.load()
    Q = len(meshes)
    shape = np.zeros(1, dtype=_lib.DP_SHAPE_DTYPE)
    shape["num_layers"], shape["num_devices"], shape["num_mesh"], shape["p_dim"] = L, D, Q, P1
    S = min(max(n * m for n, m in meshes), L) // 2
    shape["max_stages"] = S
    shape["mesh_n"][0, :Q] = [n for n, _ in meshes]
    shape["mesh_m"][0, :Q] = [m for _, m in meshes]
    dev = [torch.from_numpy(t).cuda() for t in tabs]
    dev += [torch.cummin(t, dim=-1).values.contiguous() for t in dev]  # running minima over ckpt
    costs = _lib.DpCosts(*[t.data_ptr() for t in dev])
    if relaid:
        # the row minima in stage-count order: large batches then run a workgroup per instance
        per_g = lib.mist_dp_stage_minima_floats(ctypes.c_void_p(shape.ctypes.data))
        stage_min = torch.empty(per_g, dtype=torch.float32).cuda()
        _lib.check(lib.mist_dp_stage_minima(
            ctypes.c_void_p(shape.ctypes.data), ctypes.byref(costs), 1, stage_min.data_ptr(),
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "mist_dp_stage_minima")
        costs.stage_min, costs.stage_min_g_stride = stage_min.data_ptr(), per_g
    n = len(tmax)
    d_t = torch.tensor(tmax, dtype=torch.float32).cuda()
    d_g = torch.zeros(n, dtype=torch.int32).cuda()
    d_s = torch.empty(n, dtype=torch.int32).cuda()
    d_sum = torch.empty(n, dtype=torch.float32).cuda()
    d_max = torch.empty(n, dtype=torch.float32).cuda()
    n_scr = lib.mist_dp_scratch_floats(ctypes.c_void_p(shape.ctypes.data), n)
    scr = torch.empty(max(n_scr, 1), dtype=torch.float32).cuda()
    arg = torch.full((n, S + 1, L + 1, D + 1, 4), -1, dtype=torch.int32).cuda() if want_argmin else None
    rc = lib.mist_dp_run(
        ctypes.c_void_p(shape.ctypes.data), ctypes.byref(costs), d_t.data_ptr(), d_g.data_ptr(), n,
        mode, d_s.data_ptr(), d_sum.data_ptr(), d_max.data_ptr(), arg.data_ptr() if want_argmin else None,
        scr.data_ptr(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream),
    )
    _lib.check(rc, "mist_dp_run")
    path = None
    if want_argmin:  # the partitions, walked on the GPU from the same back-pointers
        path = torch.full((n, S, 4), -7, dtype=torch.int32).cuda()
        _lib.check(lib.mist_dp_backtrack(
            ctypes.c_void_p(shape.ctypes.data), arg.data_ptr(), d_s.data_ptr(), n, path.data_ptr(),
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "mist_dp_backtrack")
    torch.cuda.synchronize()
    out = (d_s.cpu().numpy(), d_sum.cpu().numpy(), d_max.cpu().numpy())
    return out + ((arg.cpu().numpy(), path.cpu().numpy()) if want_argmin else ())


def _gpu_dp_many(meshes, L, D, P1, tabs_per_g, g_index, tmax, mode, schedule):
    """``mist_dp_run`` over instances of several gradient-accumulation rows (``tabs_per_g``: one
    table set per row) with the schedule forced through MIST_DP_FORCE_SCHEDULE ('' = the
    library's own choice); back-pointers included."""
    import os

    import torch
    from mist_amd import _lib

    lib = _lib.load()
    Q, n_g, n = len(meshes), len(tabs_per_g), len(tmax)
    shape = np.zeros(1, dtype=_lib.DP_SHAPE_DTYPE)
    shape["num_layers"], shape["num_devices"], shape["num_mesh"], shape["p_dim"] = L, D, Q, P1
    S = min(max(a * b for a, b in meshes), L) // 2
    shape["max_stages"] = S
    shape["mesh_n"][0, :Q] = [a for a, _ in meshes]
    shape["mesh_m"][0, :Q] = [b for _, b in meshes]
    sp = ctypes.c_void_p(shape.ctypes.data)
    dev = [torch.from_numpy(np.stack([t[v] for t in tabs_per_g])).cuda() for v in range(4)]
    dev += [torch.cummin(t, dim=-1).values.contiguous() for t in dev]
    costs = _lib.DpCosts(*[t.data_ptr() for t in dev])
    for v in range(4):
        costs.g_stride[v] = dev[v][0].numel()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    per_g = lib.mist_dp_stage_minima_floats(sp)
    stage_min = torch.empty(per_g * n_g, dtype=torch.float32).cuda()
    _lib.check(lib.mist_dp_stage_minima(sp, ctypes.byref(costs), n_g, stage_min.data_ptr(), stream),
               "mist_dp_stage_minima")
    costs.stage_min, costs.stage_min_g_stride = stage_min.data_ptr(), per_g
    d_t = torch.tensor(np.asarray(tmax, dtype=np.float32)).cuda()
    d_g = torch.tensor(np.asarray(g_index, dtype=np.int32)).cuda()
    d_s = torch.full((n,), -9, dtype=torch.int32).cuda()
    d_sum = torch.full((n,), -9.0, dtype=torch.float32).cuda()
    d_max = torch.full((n,), -9.0, dtype=torch.float32).cuda()
    scr = torch.empty(max(lib.mist_dp_scratch_floats(sp, n), 1), dtype=torch.float32).cuda()
    arg = torch.full((n, S + 1, L + 1, D + 1, 4), -1, dtype=torch.int32).cuda()
    old = os.environ.get("MIST_DP_FORCE_SCHEDULE")
    os.environ["MIST_DP_FORCE_SCHEDULE"] = schedule
    try:
        rc = lib.mist_dp_run(sp, ctypes.byref(costs), d_t.data_ptr(), d_g.data_ptr(), n, mode,
                             d_s.data_ptr(), d_sum.data_ptr(), d_max.data_ptr(), arg.data_ptr(),
                             scr.data_ptr(), stream)
    finally:
        if old is None:
            del os.environ["MIST_DP_FORCE_SCHEDULE"]
        else:
            os.environ["MIST_DP_FORCE_SCHEDULE"] = old
    _lib.check(rc, f"mist_dp_run ({schedule or 'auto'})")
    torch.cuda.synchronize()
    return d_s.cpu().numpy(), d_sum.cpu().numpy(), d_max.cpu().numpy(), arg.cpu().numpy()


@pytest.mark.parametrize(
    "L,D,meshes,P1,quantum",
    [
        (6, 4, [(1, 1), (1, 2), (1, 4)], 3, None),                      # D <= 64: three of a lane's four columns idle
        (9, 8, [(1, 1), (1, 2), (1, 4), (2, 4)], 5, 0.125),
        (12, 16, [(1, 1), (1, 2), (1, 4), (1, 8), (2, 8)], 7, 0.0625),
        (23, 70, [(1, 1), (1, 2), (1, 5), (2, 5), (7, 5), (7, 10)], 12, 0.0625),  # D no multiple of 64
        (40, 80, [(1, 1), (1, 2), (1, 4), (1, 8), (2, 8), (4, 8), (8, 8)], 21, 0.03125),
        (79, 33, [(1, k) for k in range(1, 17)], 9, 0.03125),           # Q L = 1264 of at most 1280 row minima per start layer
        (20, 256, [(1, 1), (1, 8), (4, 8), (32, 8)], 11, 0.125),         # the widest plane the schedule holds
    ],
)
@pytest.mark.parametrize("mode", [0, 1], ids=["threshold", "bottleneck"])
def test_every_dp_schedule_gives_the_same_states(L, D, meshes, P1, quantum, mode):
    """The three schedules of ``mist_dp_run`` (one launch per stage count; one workgroup per
    instance with all planes in LDS; one workgroup per instance with one plane in LDS, which the
    library itself only picks for the 80-layer, 256-device shape) forced on the same batch of
    DISTINCT instances - three gradient-accumulation rows with their own tables, a spread of
    thresholds - must agree on every output incl. all back-pointers; the per-stage-count launches
    are held against the C oracle in test_dp_kernel_matches_c_oracle."""
    from mist_amd import _lib

    rng = np.random.default_rng(L * 1000 + D + mode)
    tabs = [_random_tables(rng, len(meshes), P1, L, quantum=quantum) for _ in range(3)]
    n = 20
    tmax = rng.uniform(0.1, 1.1, size=n).astype(np.float32)
    g_index = rng.integers(0, 3, size=n).astype(np.int32)
    g_index[:3] = (0, 1, 2)
    want = _gpu_dp_many(meshes, L, D, P1, tabs, g_index, tmax, mode, "step")
    assert not np.any(want[0] == -9)
    assert (want[0] >= 0).any()
    lib = _lib.load()
    for schedule in ("fused", "plane", ""):
        try:
            got = _gpu_dp_many(meshes, L, D, P1, tabs, g_index, tmax, mode, schedule)
        except _lib.MistLibraryError as e:
            # the all-planes-in-LDS schedule does not hold the largest shapes
            assert schedule == "fused" and "forced fused schedule" in str(e), e
            continue
        for name, w, g in zip(("best_s", "best_sum", "stage_max", "argmin"), want, got):
            if name == "stage_max" and mode == 0:
                ok = np.array_equal(w[want[0] >= 0].view(np.int32), g[want[0] >= 0].view(np.int32))
            else:
                ok = np.array_equal(w.view(np.int32), g.view(np.int32))
            assert ok, (schedule or "auto", name)


def _walk(arg, best_s, D):
    """Partition from one instance's back-pointers, as the reference walks them
    (inter_tuning.py:341-355): [(end layer, n, m, ckpt), ...] in pipeline order."""
    out, cs, cl, cd = [], int(best_s), 0, D
    while cs > 0:
        end, n, m, ckpt = (int(v) for v in arg[cs, cl, cd])
        out.append([end, n, m, ckpt])
        cs, cl, cd = cs - 1, end + 1, cd - n * m
    return out


@pytest.mark.parametrize(
    "L,D,meshes,P1,quantum",
    [
        (6, 4, [(1, 1), (1, 2), (1, 4)], 3, None),
        (9, 8, [(1, 1), (1, 2), (1, 4), (2, 4)], 5, 0.125),
        (12, 16, [(1, 1), (1, 2), (1, 4), (1, 8), (2, 8)], 7, 0.0625),
        (40, 80, [(1, 1), (1, 2), (1, 4), (1, 8), (2, 8), (4, 8), (8, 8)], 21, 0.03125),  # large state planes
    ],
)
def test_dp_kernel_matches_c_oracle(L, D, meshes, P1, quantum):
    from oracle.dp_c import _load

    rng = np.random.default_rng(L * 100 + D)
    tabs = _random_tables(rng, len(meshes), P1, L, quantum=quantum)
    tmax = np.sort(rng.uniform(0.1, 1.1, size=24)).astype(np.float32)
    got_s, got_sum, got_max = _gpu_dp(meshes, L, D, P1, tabs, tmax)
    lib = _load()
    S = min(max(n * m for n, m in meshes), L) // 2
    mesh_n = np.array([n for n, _ in meshes], dtype=np.int32)
    mesh_m = np.array([m for _, m in meshes], dtype=np.int32)
    ptr = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    n_feasible = 0
    want = []
    for i, t in enumerate(tmax):
        bs, bsum, smax = ctypes.c_int(), ctypes.c_float(), ctypes.c_float()
        arg = np.empty((S + 1, L + 1, D + 1, 4), dtype=np.int32)
        assert lib.mist_oracle_dp(
            ctypes.c_float(float(t)), L, D, len(meshes), ptr(mesh_n), ptr(mesh_m), P1, ptr(tabs[0]),
            ptr(tabs[1]), ptr(tabs[2]), ptr(tabs[3]), ctypes.byref(bs), ctypes.byref(bsum),
            ctypes.byref(smax), ptr(arg)) == 0
        want.append((bs.value, np.float32(bsum.value), np.float32(smax.value), arg))
        assert got_s[i] == bs.value, (i, t)
        if bs.value >= 0:
            n_feasible += 1
            assert got_sum[i] == np.float32(bsum.value) and got_max[i] == np.float32(smax.value), (i, t)
            g = _gpu_dp(meshes, L, D, P1, tabs, [t], want_argmin=True)
            assert np.array_equal(g[3][0], arg), f"back-pointers differ at t={t}"
            stages = _walk(arg, bs.value, D)
            assert g[4][0][:len(stages)].tolist() == stages and np.all(g[4][0][len(stages):] == -1)
    assert n_feasible > 0
    # The library picks its kernels by batch size (teams of lanes per state for small batches; for
    # large ones a workgroup per instance with the planes in LDS, or a lane per state when they
    # do not fit): the same thresholds repeated until the batch passes 2^19 states.
    reps = (1 << 19) // ((L + 1) * (D + 1) * len(tmax)) + 1
    for relaid in (True, False):  # without the re-laid minima: always a launch per stage count
        big_s, big_sum, big_max, big_arg, big_path = _gpu_dp(
            meshes, L, D, P1, tabs, np.tile(tmax, reps), want_argmin=True, relaid=relaid)
        for r in range(reps):
            for i, (bs, bsum, smax, arg) in enumerate(want):
                at = r * len(tmax) + i
                assert big_s[at] == bs, (relaid, r, i)
                if bs >= 0:
                    assert big_sum[at] == bsum and big_max[at] == smax, (relaid, r, i)
                    assert np.array_equal(big_arg[at], arg), (relaid, r, i)
                    stages = _walk(arg, bs, D)
                    assert big_path[at][:len(stages)].tolist() == stages
                    assert np.all(big_path[at][len(stages):] == -1)
                else:
                    assert np.all(big_path[at] == -1)
    # the re-laid table itself: entry (p, q, k, i) is the smallest admissible-ckpt cost
    import torch
    from mist_amd import _lib as lib_mod
    shape = np.zeros(1, dtype=lib_mod.DP_SHAPE_DTYPE)
    shape["num_layers"], shape["num_devices"], shape["num_mesh"], shape["p_dim"] = L, D, len(meshes), P1
    shape["max_stages"] = S
    shape["mesh_n"][0, :len(meshes)], shape["mesh_m"][0, :len(meshes)] = mesh_n, mesh_m
    glib = lib_mod.load()
    per_g = glib.mist_dp_stage_minima_floats(ctypes.c_void_p(shape.ctypes.data))
    tri = L * (L + 1) // 2
    assert per_g == S * len(meshes) * tri
    dev = [torch.from_numpy(t).cuda() for t in tabs]
    dev += [torch.cummin(t, dim=-1).values.contiguous() for t in dev]
    costs = lib_mod.DpCosts(*[t.data_ptr() for t in dev])
    out = torch.empty(per_g, dtype=torch.float32).cuda()
    lib_mod.check(glib.mist_dp_stage_minima(
        ctypes.c_void_p(shape.ctypes.data), ctypes.byref(costs), 1, out.data_ptr(),
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "mist_dp_stage_minima")
    got = out.cpu().numpy().reshape(S, len(meshes), tri)
    for p_ in range(S):
        for q in range(len(meshes)):
            for k in range(L):
                for i in range(k, L):
                    l = i - k + 1
                    row = (tabs[3][q] if k == 0 and i == L - 1 else tabs[1][q, p_, l - 1] if k == 0
                           else tabs[2][q, l - 1] if i == L - 1 else tabs[0][q, p_, l - 1])
                    expect = row[: L - i + 1].min() if k <= L - 1 - p_ else np.inf
                    assert got[p_, q, k * L - k * (k - 1) // 2 + i - k] == expect, (p_, q, k, i)
    # bottleneck mode = the smallest threshold for which the threshold DP is feasible
    _, bott, path_sum = _gpu_dp(meshes, L, D, P1, tabs, [0.0], mode=1)
    # ... and the sum reported with it belongs to a partition admissible at that threshold
    at_bott = _gpu_dp(meshes, L, D, P1, tabs, [bott[0]])
    assert at_bott[0][0] >= 0 and at_bott[1][0] <= path_sum[0] and at_bott[2][0] == bott[0]
    big = _gpu_dp(meshes, L, D, P1, tabs, np.zeros(reps * len(tmax), dtype=np.float32), mode=1)
    assert np.all(big[1] == bott[0]) and np.all(big[2] == path_sum[0]) and np.all(big[0] == _[0])
    cand = np.unique(np.concatenate([t.ravel() for t in tabs[:3]]))
    cand = cand[np.isfinite(cand)]
    feas = _gpu_dp(meshes, L, D, P1, tabs, cand)[0] >= 0
    # (single-stage costs are not threshold candidates, so the bottleneck itself may be absent)
    assert feas.any() and cand[np.argmax(feas)] == cand[cand >= bott[0]].min()
    assert np.all(feas[np.argmax(feas):]) and not feas[: np.argmax(feas)].any()


@pytest.mark.parametrize(
    "overrides",
    [
        dict(hardware__num_nodes=2, hardware__num_gpus_per_node=4, training__global_batch_size=32,
             hardware__memory_capacity=8.0),
        dict(hardware__num_nodes=1, hardware__num_gpus_per_node=8, training__global_batch_size=16,
             hardware__memory_capacity=5.0, model__use_flash_attn=True),
        dict(hardware__num_nodes=2, hardware__num_gpus_per_node=4, training__global_batch_size=32,
             hardware__memory_capacity=8.0, tuning__tuning_granularity="uniform-pp"),
    ],
)
def test_tune_end_to_end_matches_oracle(overrides):
    """YAML in, best strategy out: identical cost (bit for bit) and identical solution."""
    from mist_amd.tune_one_case import tune
    from oracle.tune import tune as oracle_tune

    cfg, tables = tiny_plan(1, layers=8, **overrides)
    got_cost, got_sol = tune(cfg)
    want_cost, want_sol = oracle_tune(cfg, tables)
    assert want_sol is not None, "degenerate case"
    assert got_cost == want_cost
    assert got_sol == want_sol


@pytest.mark.parametrize("seed", range(6))
def test_randomized_tune_end_to_end_matches_oracle(seed):
    """Seeded random tiny plans through the whole tuner (intra-stage kernels, the search driver
    in the library, back-pointers, strategy read-back) against the oracle's tune: hardware
    coefficients, interference factors, memory capacity, cluster shape, batch size and layer count
    are drawn at random, so the scan meets different bottlenecks, window widths and stop points."""
    from mist_amd.tune_one_case import tune
    from oracle.tune import tune as oracle_tune

    rng = np.random.default_rng(4200 + seed)
    gg = []
    for _ in range(16):
        gg += [float(rng.uniform(8, 500)), float(rng.uniform(2e-6, 8e-5))]
    nodes, gpn = [(1, 2), (1, 4), (2, 2), (2, 4), (1, 8), (2, 4)][seed]
    overrides = dict(
        hardware__gpu_gpu_comm_params=gg,
        hardware__interference_model_params=[float(x) for x in rng.uniform(1.0, 3.0, size=28)],
        hardware__memory_capacity=float(rng.choice([3.0, 5.0, 8.0, 16.0])),
        hardware__num_nodes=nodes, hardware__num_gpus_per_node=gpn,
        training__global_batch_size=int(rng.choice([16, 32, 64])),
    )
    cfg, tables = tiny_plan(1, layers=int(rng.integers(5, 10)), **overrides)
    got = tune(cfg)
    want = oracle_tune(cfg, tables)
    assert got == want


RANDOM_PLAN_SEEDS = [0, 3, 5, 6, 27, 40, 42, 44, 48, 54, 57, 58, 63, 65, 77, 84, 97, 109, 119, 128, 180, 195, 216, 250]


def _random_plan(seed):
    """A seeded random plan over what a configuration file can vary: model shape (hidden size,
    heads, kv heads, gated MLP, norm, position embedding, tied embeddings, sequence length),
    cluster shape with slow or fast links between nodes, memory capacity, batch size, offload
    ratio lists, the tuning switches, the fixed / disabled offload ratios, the pre / post layer
    strategy, every tuning granularity and several sample sizes."""
    rng = np.random.default_rng(190000 + seed)
    slow = bool(rng.integers(0, 3) > 0)
    gg = []
    for entry in range(16):
        lo, hi = (8, 500) if (entry < 4 or not slow) else (0.3, 6)  # entries 4..15: several nodes
        if slow and entry < 4 and rng.integers(0, 2):
            lo, hi = 2, 20
        gg += [float(rng.uniform(lo, hi)), float(rng.uniform(2e-6, 8e-5))]
    nodes, gpn = [(1, 2), (1, 4), (2, 2), (2, 4), (1, 8), (4, 2), (2, 8)][int(rng.integers(0, 7))]
    granularity = str(rng.choice(["inter-stage", "inter-stage", "uniform-device-pp", "uniform-pp",
                                  "uniform-device-pp-mip", "uniform-device-pp-mip"]))
    samples = 1 if granularity != "uniform-device-pp-mip" else int(rng.choice([1, 2, 3, 5]))
    ratios = [float(x) for x in np.linspace(0, 1, int(rng.choice([2, 3, 5])))]
    hidden, heads = int(rng.choice([1024, 2048, 2048, 4096])), int(rng.choice([8, 16, 32]))
    overrides = dict(
        hardware__gpu_gpu_comm_params=gg,
        hardware__interference_model_params=[float(x) for x in rng.uniform(1.0, 3.0, size=28)],
        hardware__cpu_gpu_comm_params=[float(rng.uniform(20, 55)), float(rng.uniform(5e-6, 2e-5))],
        hardware__gpu_cpu_comm_params=[float(rng.uniform(20, 55)), float(rng.uniform(5e-6, 2e-5))],
        hardware__memory_capacity=float(rng.choice([2.5, 3.0, 5.0, 8.0, 12.0, 40.0])),
        hardware__num_nodes=nodes, hardware__num_gpus_per_node=gpn,
        training__global_batch_size=int(rng.choice([8, 16, 32, 64, 24, 48])),
        training__max_sequence_length=int(rng.choice([1024, 2048, 4096])),
        tuning__tuning_granularity=granularity, tuning__sample_size=samples,
        tuning__zero_2_and_3_enabled=bool(rng.integers(0, 2)),
        tuning__activation_checkpointing_tuning_enabled=bool(rng.integers(0, 4) > 0),
        tuning__state_offloading_enabled=bool(rng.integers(0, 4) > 0),
        tuning__activation_offloading_enabled=bool(rng.integers(0, 4) > 0),
        tuning__pre_post_strategy=str(rng.choice(["dp", "intra-node-tp-with-ore", "intra-node-tp-without-ore"])),
        tuning__search_space__offloading_ratio_candidates=ratios,
        tuning__search_space__sparse_offloading_ratio_candidates=ratios,
        tuning__search_space__batch_size_candidates=[1, 2, 3, 4, 6, 8],
        model__use_flash_attn=bool(rng.integers(0, 2)),
        model__hidden_size=hidden, model__num_attention_heads=heads,
        model__intermediate_size=int(hidden * rng.choice([2, 4])),
        model__mlp_type=str(rng.choice(["mlp", "gated_mlp"])),
        model__normalization=str(rng.choice(["layernorm", "rmsnorm"])),
        model__position_embedding_type=str(rng.choice(["absolute", "rope"])),
        model__tie_word_embeddings=bool(rng.integers(0, 2)),
        model__num_heads_kv=(None if rng.integers(0, 2) else int(heads // rng.choice([1, 2, 4]))),
        enable_advanced_opt_in_first_block=bool(rng.integers(0, 2)),
        disable_tp_tuning=bool(rng.integers(0, 5) == 0),
    )
    for key in ("disable_wo_tuning", "disable_go_tuning", "disable_oo_tuning"):
        if rng.integers(0, 4) == 0:
            overrides[key] = True
    if rng.integers(0, 5) == 0:
        overrides["fixed_ao_ratio"] = float(rng.choice(ratios))
    if rng.integers(0, 6) == 0:
        overrides["fixed_oo_ratio"] = float(rng.choice(ratios))
    return tiny_plan(1, layers=int(rng.integers(6, 14)), **overrides)


@pytest.mark.parametrize("seed", RANDOM_PLAN_SEEDS)
def test_randomized_plans_of_every_granularity_match_oracle(seed):
    """Cost and strategy of random plans equal the oracle's.  The seeds were picked by what the
    oracle answers: mostly pipelines of two to four stages, some single stages, some plans that
    fit nowhere."""
    from mist_amd.tune_one_case import tune
    from oracle.tune import tune as oracle_tune

    cfg, tables = _random_plan(seed)
    got = tune(cfg)
    want = oracle_tune(cfg, tables)
    assert got == want


def _realistic_plan(seed):
    """Seeded random plan at realistic sizes (8-64 layers, 2-128 devices, the GPT-7B or LLaMA-13B
    offload grid, random link / copy / interference parameters, capacities from "nothing fits"
    to "everything fits") for a search that scans thresholds: per-mesh or uniform-device."""
    rng = np.random.default_rng(333000 + seed)
    slow = bool(rng.integers(0, 2))
    gg = []
    for entry in range(16):
        lo, hi = (8, 500) if (entry < 4 or not slow) else (0.5, 20)
        gg += [float(rng.uniform(lo, hi)), float(rng.uniform(2e-6, 8e-5))]
    nodes, gpn = int(rng.choice([1, 2, 4, 8, 16])), int(rng.choice([2, 4, 8]))
    L = int(rng.integers(8, 65))
    granularity = str(rng.choice(["inter-stage", "inter-stage", "uniform-device-pp"]))
    overrides = dict(
        model__num_hidden_layers=L,
        hardware__gpu_gpu_comm_params=gg,
        hardware__cpu_gpu_comm_params=[float(rng.uniform(5, 60)), float(rng.uniform(2e-6, 3e-5))],
        hardware__gpu_cpu_comm_params=[float(rng.uniform(5, 60)), float(rng.uniform(2e-6, 3e-5))],
        hardware__interference_model_params=[float(x) for x in rng.uniform(1.0, 4.0, size=28)],
        hardware__memory_capacity=float(np.exp(rng.uniform(np.log(3.0), np.log(300.0)))),
        hardware__num_nodes=nodes, hardware__num_gpus_per_node=gpn,
        training__global_batch_size=int(rng.choice([64, 128, 256, 512, 96, 384])),
        model__use_flash_attn=bool(rng.integers(2)),
        enable_advanced_opt_in_first_block=bool(rng.integers(2)),
        tuning__pre_post_strategy=str(rng.choice(["dp", "intra-node-tp-with-ore", "intra-node-tp-without-ore"])),
        tuning__zero_2_and_3_enabled=bool(rng.integers(0, 4) > 0),
        tuning__activation_checkpointing_tuning_enabled=bool(rng.integers(0, 4) > 0),
        tuning__state_offloading_enabled=bool(rng.integers(0, 5) > 0),
        tuning__activation_offloading_enabled=bool(rng.integers(0, 5) > 0),
        tuning__tuning_granularity=granularity,
        synthetic__seed=int(rng.integers(1 << 20)),
    )
    return load_plan(int(rng.choice([2, 2, 3])), **overrides)[0]


def _tune_with_and_without_estimate(cfg):
    from mist_amd.tune_one_case import PreparedSearch

    search = PreparedSearch(cfg)
    assert search.stage_cost_cutoff is not None
    stats = {}
    got = search.run(stats)
    estimate = float(search.dev_plan["incumbent"].item())
    search.stage_cost_cutoff = None
    want = search.run()
    assert got == want
    return want, estimate, stats.get("stage_cost_cutoff_retries", 0)


@pytest.mark.parametrize("plan, overrides", [
    (1, {}), (2, {}), (3, {}), (4, {}), (5, {}),
    (2, dict(tuning__tuning_granularity="uniform-device-pp")),
    (3, dict(tuning__tuning_granularity="uniform-device-pp", tuning__activation_checkpointing_tuning_enabled=False)),
])
def test_tune_of_the_benchmark_plans_with_a_stage_cost_estimate(plan, overrides):
    """``tune`` lets the intra-stage kernels skip stage costs its search cannot use
    (``PreparedSearch.stage_cost_cutoff``): same cost, partition and strategies as the search on
    the full tables, for every benchmark plan, without a second evaluation; the scout pass of
    the large plans does produce an estimate."""
    (cost, solution), estimate, retries = _tune_with_and_without_estimate(load_plan(plan, **overrides)[0])
    assert solution is not None and retries == 0
    assert plan == 1 or (np.isfinite(estimate) and cost < estimate * 1.25)


_UNCERTAIN = (3, 252, 499, 785, 972, 2088, 3887, 823, 1000)


@pytest.mark.parametrize("seed", [1, 6, 7, 3, 31, 34, 47, 89, 149, 252, 315, 499, 144, 785, 972, 985, 2088, 3887, 823, 1000])
def test_tune_of_random_plans_with_a_stage_cost_estimate(seed):
    """The same on random plans.  The search over tables under the estimate stays below their
    limit and asks for a second evaluation on complete tables when a partition inside the limit
    is cheaper than what its scan found (a single-stage cost is no threshold candidate of the
    reference, so whether its scan finds such a partition hangs on the candidates above the
    limit) or its result is not below the limit: the seeds of ``_UNCERTAIN`` (785 ... 1000: the
    estimate lies below the result, the reference's scan never tries that pipeline)."""
    _, estimate, retries = _tune_with_and_without_estimate(_realistic_plan(seed))
    assert retries == (1 if seed in _UNCERTAIN else 0)
    assert seed == 144 or np.isfinite(estimate)  # (144: nothing fits)


def _sparse_candidate_plan():
    """64 devices, 33 layers, uniform-device-pp without ckpt tuning (few cells per group, so few
    threshold candidates): the best pipeline is a single stage at G = 2 whose cost no candidate
    of that G follows below the limit of the tables; on complete tables the reference's scan
    reaches it through a candidate above the limit."""
    rng = np.random.default_rng(333000 + 14190)
    gg = []
    slow = bool(rng.integers(0, 2))
    for e in range(16):
        lo, hi = (8, 500) if (e < 4 or not slow) else (0.5, 20)
        gg += [float(rng.uniform(lo, hi)), float(rng.uniform(2e-6, 8e-5))]
    nodes, gpn = int(rng.choice([1, 2, 4, 8, 16])), int(rng.choice([2, 4, 8]))
    layers = int(rng.integers(8, 65))
    granularity = str(rng.choice(["inter-stage", "inter-stage", "uniform-device-pp"]))
    overrides = dict(
        model__num_hidden_layers=layers,
        hardware__gpu_gpu_comm_params=gg,
        hardware__cpu_gpu_comm_params=[float(rng.uniform(5, 60)), float(rng.uniform(2e-6, 3e-5))],
        hardware__gpu_cpu_comm_params=[float(rng.uniform(5, 60)), float(rng.uniform(2e-6, 3e-5))],
        hardware__interference_model_params=[float(x) for x in rng.uniform(1.0, 4.0, size=28)],
        hardware__memory_capacity=float(np.exp(rng.uniform(np.log(3.0), np.log(300.0)))),
        hardware__num_nodes=nodes, hardware__num_gpus_per_node=gpn,
        training__global_batch_size=int(rng.choice([64, 128, 256, 512, 96, 384])),
        model__use_flash_attn=bool(rng.integers(2)),
        enable_advanced_opt_in_first_block=bool(rng.integers(2)),
        tuning__pre_post_strategy=str(rng.choice(["dp", "intra-node-tp-with-ore", "intra-node-tp-without-ore"])),
        tuning__zero_2_and_3_enabled=bool(rng.integers(0, 4) > 0),
        tuning__activation_checkpointing_tuning_enabled=bool(rng.integers(0, 4) > 0),
        tuning__state_offloading_enabled=bool(rng.integers(0, 5) > 0),
        tuning__activation_offloading_enabled=bool(rng.integers(0, 5) > 0),
        tuning__tuning_granularity=granularity,
        synthetic__seed=int(rng.integers(1 << 20)),
    )
    assert (layers, nodes, gpn, granularity) == (33, 8, 8, "uniform-device-pp")
    return load_plan(int(rng.choice([2, 2, 3])), **overrides)[0]


def test_partition_inside_the_limit_that_no_threshold_below_it_admits():
    """A plan on which the scan over tables under the estimate, left to run above their limit,
    returned 3.769 (G = 4) where the reference's scan on complete tables returns 3.665 (G = 2):
    the search now stops at the limit, sees that the partition within it beats its result, and
    ``tune`` evaluates again."""
    (cost, solution), estimate, retries = _tune_with_and_without_estimate(_sparse_candidate_plan())
    assert retries == 1 and solution[0] == 2 and len(solution[1]) == 1
    assert abs(cost - estimate) < 1e-6 * cost


def test_plan1_end_to_end():
    from mist_amd.tune_one_case import tune
    from oracle.tune import tune as oracle_tune

    cfg, tables = load_plan(1)
    got = tune(cfg)
    want = oracle_tune(cfg, tables)
    assert want[1] is not None
    assert got == want


@pytest.mark.parametrize("plan, tp, g_picks, n_below, n_above, n_min", [
    (2, 8, ("best", 32, "last"), 3, 9, 12),   # L = 32, D = 32, 6 meshes
    (4, 8, ("best", 16, "last"), 2, 4, 6),    # L = 48, D = 128, 8 meshes
    (5, 8, ("best",), 1, 3, 3),               # L = 80, D = 256, 9 meshes: ~10 s per oracle run
])
def test_full_size_dp_matches_c_oracle(plan, tp, g_picks, n_below, n_above, n_min):
    """The benchmark plans at full size (GPT-7B: L = 32, 32 devices, 6 meshes; GPT-22B: L = 48,
    128 devices, 8 meshes; LLaMA-70B: L = 80, 256 devices, 9 meshes, state planes beyond the LDS
    of a compute unit): the intra-stage tables come from the GPU search (checked against the
    oracle's fixtures elsewhere); the DP kernel is compared with the C oracle on those tables at
    the thresholds that matter - just below the smallest feasible one, at it, a run of kept
    candidates above it and the winning one, back-pointers included.  (The reference's full
    ascending scan needs ~10^5 DP runs per G on the CPU.)"""
    from mist_amd import _lib
    from mist_amd.inter_tuning import _DpRunner, _Window, inter_stage_tune
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates
    from oracle.dp_c import dp_impl_c
    from oracle.inter_dp import dp_cost_tables

    cfg, tables = load_plan(plan)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    D = hw.num_nodes * hw.num_gpus_per_node
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    res = IntraStageTuner(tables, L, meshes, Gs, tp, cfg, sample_size=1).tune()
    best_cost, best_solution = inter_stage_tune(L, D, meshes, Gs, res)
    assert best_solution is not None
    runner = _DpRunner(res, L, D, meshes, 0)
    n_checked = 0
    picks = [Gs.index(best_solution[0]) if g == "best" else len(Gs) - 1 if g == "last" else Gs.index(g)
             for g in g_picks]
    for g in picks:
        G = Gs[g]
        tabs = dp_cost_tables(res, g)
        _, bott, _ = runner.run(np.array([g], dtype=np.int32), np.zeros(1, dtype=np.float32),
                                _lib.DP_BOTTLENECK)
        assert np.isfinite(bott[0])
        lo = np.float32(bott[0] * 0.98)
        (vals, _), = runner.candidates_between(np.array([g]), np.array([lo]), np.array([bott[0] * 1.02], dtype=np.float32))
        vals = np.unique(vals)
        at = int(np.searchsorted(vals, bott[0]))
        tmax = np.concatenate([vals[max(at - n_below, 0):at], vals[at:at + n_above]])
        n_oracle = len(tmax)
        if plan == 5:
            # A batch of 16 or more instances of this shape runs one workgroup per instance with
            # one state plane in LDS; smaller ones take the per-stage-count launches.  Both
            # schedules are held against each other on the whole batch and against the oracle on
            # its first thresholds.
            tmax = np.concatenate([tmax, vals[at + n_above:at + n_above + 20]])
            assert len(tmax) >= 16
        bs, bsum, smax, arg = runner.run(np.full(len(tmax), g, dtype=np.int32), tmax, want_argmin=True)
        if plan == 5:
            for lo in range(0, len(tmax), 6):
                part = runner.run(np.full(len(tmax[lo:lo + 6]), g, dtype=np.int32), tmax[lo:lo + 6],
                                  want_argmin=True)
                for whole, piece in zip((bs, bsum, smax), part[:3]):
                    assert np.array_equal(whole[lo:lo + 6].view(np.int32), piece.view(np.int32))
                # back-pointers along the winning path (entries off the path may differ in
                # nothing either: both schedules write every finite state)
                assert np.array_equal(arg[lo:lo + 6], part[3])
            _, bott_many, _ = runner.run(np.full(16, g, dtype=np.int32), np.zeros(16, dtype=np.float32),
                                         _lib.DP_BOTTLENECK)
            assert np.all(bott_many == bott[0])
        tmax = tmax[:n_oracle]
        for i, t in enumerate(tmax):
            want_cost, want_sol = dp_impl_c(t, L, D, meshes, G, *tabs)
            assert (bs[i] >= 0) == (want_sol is not None), (G, t)
            assert (t >= bott[0]) == (bs[i] >= 0), "bottleneck DP disagrees with the threshold DP"
            if want_sol is None:
                continue
            got_cost = float(np.float64(bsum[i]) + np.float64(G - 1) * np.float64(smax[i]))
            assert got_cost == want_cost, (G, t)
            sol, cs, cl, cd = [], int(bs[i]), 0, D
            while cs > 0:
                end, n, m, ckpt = (int(v) for v in arg[i][cs, cl, cd])
                sol.append(((cl, end), (n, m), ckpt))
                cs, cl, cd = cs - 1, end + 1, cd - n * m
            assert sol == want_sol, (G, t)
            n_checked += 1
    assert n_checked >= n_min
    # the search's answer is one of the DP solutions: recompute it at its own bottleneck
    g = Gs.index(best_solution[0])
    tabs = dp_cost_tables(res, g)
    inter = [s[0][:3] for s in best_solution[1]]
    costs = []
    for i, ((l0, l1), mesh, ckpt) in enumerate(inter):
        q, l, p = meshes.index(mesh), l1 - l0 + 1, len(inter) - i - 1
        if len(inter) == 1:
            costs.append(tabs[3][q, ckpt])
        elif i == 0:
            costs.append(tabs[1][q, p, l - 1, ckpt])
        elif i == len(inter) - 1:
            costs.append(tabs[2][q, l - 1, ckpt])
        else:
            costs.append(tabs[0][q, p, l - 1, ckpt])
    want_cost, want_sol = dp_impl_c(np.float32(max(costs)), L, D, meshes, Gs[g], *tabs)
    assert want_cost == best_cost and want_sol == inter


@pytest.mark.parametrize("ckpt_tuning", [True, False])
@pytest.mark.parametrize("L,num_nodes,gpn,P1,quantum", [(6, 1, 4, 7, None), (7, 2, 4, 4, 0.125), (9, 2, 2, 10, 0.25)])
def test_uniform_device_dp_kernel_matches_oracle(L, num_nodes, gpn, P1, quantum, ckpt_tuning):
    """The free-device / per-stage ckpt-rule mode of the DP kernel, one launch family per
    admissible stage count, against the literal restatement of
    inter_tuning_uniform_device.py:276-441 (total over all S, partition, ties)."""
    import torch
    from mist_amd import _lib
    from oracle.inter_uniform_device import dp_impl as ud_dp, uniform_device_mesh_partition as udmp

    rng = np.random.default_rng(L * 10 + gpn)
    meshes = [(1, 2 ** i) for i in range(4) if 2 ** i <= gpn]
    meshes += [(2 ** j, gpn) for j in range(1, 4) if 2 ** j <= num_nodes]
    tabs = _random_tables(rng, len(meshes), P1, L, quantum=quantum)
    lib = _lib.load()
    dev = [torch.from_numpy(t).cuda() for t in tabs]
    dev += [torch.cummin(t, dim=-1).values.contiguous() for t in dev]
    G = 5
    tmax = np.sort(rng.uniform(0.1, 1.1, size=16)).astype(np.float32)
    n = len(tmax)
    best = [(np.inf, None)] * n
    for S in range(1, L + 1):
        mesh = udmp(S, num_nodes, gpn)
        if mesh is None:
            continue
        q = meshes.index(mesh)
        shape = np.zeros(1, dtype=_lib.DP_SHAPE_DTYPE)
        shape["num_layers"], shape["num_devices"], shape["num_mesh"], shape["p_dim"] = L, 0, 1, P1
        shape["max_stages"] = min(S, P1, L)
        shape["ckpt_rule"] = _lib.DP_CKPT_STAGE if ckpt_tuning else _lib.DP_CKPT_ALL
        shape["free_devices"] = 1
        shape["mesh_n"][0, 0], shape["mesh_m"][0, 0] = mesh
        per_q = [t[0].numel() for t in dev[:4]]
        costs = _lib.DpCosts(*[t.data_ptr() + 4 * q * per_q[v % 4] for v, t in enumerate(dev)])
        d_t = torch.from_numpy(tmax).cuda()
        d_g = torch.zeros(n, dtype=torch.int32).cuda()
        d_s = torch.empty(n, dtype=torch.int32).cuda()
        d_sum = torch.empty(n, dtype=torch.float32).cuda()
        d_max = torch.empty(n, dtype=torch.float32).cuda()
        Sm = int(shape["max_stages"][0])
        scr = torch.empty(lib.mist_dp_scratch_floats(ctypes.c_void_p(shape.ctypes.data), n), dtype=torch.float32).cuda()
        arg = torch.full((n, Sm + 1, L + 1, 1, 4), -1, dtype=torch.int32).cuda()
        _lib.check(lib.mist_dp_run(
            ctypes.c_void_p(shape.ctypes.data), ctypes.byref(costs), d_t.data_ptr(), d_g.data_ptr(), n, 0,
            d_s.data_ptr(), d_sum.data_ptr(), d_max.data_ptr(), arg.data_ptr(), scr.data_ptr(),
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "mist_dp_run")
        torch.cuda.synchronize()
        bs, bsum, smax, argmin = d_s.cpu().numpy(), d_sum.cpu().numpy(), d_max.cpu().numpy(), arg.cpu().numpy()
        # the same thresholds as a batch of more than 2^19 states (another kernel of the library)
        reps = (1 << 19) // ((L + 1) * n) + 1
        if reps * n <= 65535:
            N = reps * n
            b_t = d_t.repeat(reps)
            b_g = torch.zeros(N, dtype=torch.int32).cuda()
            b_s = torch.empty(N, dtype=torch.int32).cuda()
            b_sum = torch.empty(N, dtype=torch.float32).cuda()
            b_max = torch.empty(N, dtype=torch.float32).cuda()
            b_scr = torch.empty(lib.mist_dp_scratch_floats(ctypes.c_void_p(shape.ctypes.data), N), dtype=torch.float32).cuda()
            b_arg = torch.full((N, Sm + 1, L + 1, 1, 4), -1, dtype=torch.int32).cuda()
            per_g = lib.mist_dp_stage_minima_floats(ctypes.c_void_p(shape.ctypes.data))
            stage_min = torch.empty(per_g, dtype=torch.float32).cuda()
            _lib.check(lib.mist_dp_stage_minima(
                ctypes.c_void_p(shape.ctypes.data), ctypes.byref(costs), 1, stage_min.data_ptr(),
                ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "mist_dp_stage_minima")
            costs.stage_min, costs.stage_min_g_stride = stage_min.data_ptr(), per_g
            _lib.check(lib.mist_dp_run(
                ctypes.c_void_p(shape.ctypes.data), ctypes.byref(costs), b_t.data_ptr(), b_g.data_ptr(), N, 0,
                b_s.data_ptr(), b_sum.data_ptr(), b_max.data_ptr(), b_arg.data_ptr(), b_scr.data_ptr(),
                ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "mist_dp_run")
            torch.cuda.synchronize()
            assert np.array_equal(b_s.cpu().numpy(), np.tile(bs, reps))
            ok = np.tile(bs, reps) >= 0
            assert np.array_equal(b_sum.cpu().numpy()[ok], np.tile(bsum, reps)[ok])
            assert np.array_equal(b_max.cpu().numpy()[ok], np.tile(smax, reps)[ok])
            assert np.array_equal(b_arg.cpu().numpy()[ok], np.tile(argmin, (reps, 1, 1, 1, 1))[ok])
        for i in range(n):
            if bs[i] < 0:
                continue
            total = float(np.float64(bsum[i]) + np.float64(G - 1) * np.float64(smax[i]))
            if total < best[i][0]:
                sol, cs, cl = [], int(bs[i]), 0
                while cs > 0:
                    end, nn, mm, ck = (int(v) for v in argmin[i][cs, cl, 0])
                    sol.append(((cl, end), (nn, mm), ck))
                    cs, cl = cs - 1, end + 1
                best[i] = (total, sol)
    n_feasible = 0
    for i, t in enumerate(tmax):
        want = ud_dp(t, L, num_nodes, gpn, meshes, G, *tabs, ckpt_tuning=ckpt_tuning)
        assert best[i] == want, (i, t)
        n_feasible += want[1] is not None
    assert n_feasible > 0


@pytest.mark.parametrize(
    "overrides",
    [
        dict(hardware__num_nodes=2, hardware__num_gpus_per_node=4, training__global_batch_size=32,
             hardware__memory_capacity=8.0),
        dict(hardware__memory_capacity=5.0),
        dict(hardware__num_nodes=1, hardware__num_gpus_per_node=4, training__global_batch_size=16,
             hardware__memory_capacity=6.0, tuning__activation_checkpointing_tuning_enabled=False),
    ],
)
def test_uniform_device_tune_end_to_end_matches_oracle(overrides):
    from mist_amd.tune_one_case import tune
    from oracle.tune import tune as oracle_tune

    cfg, tables = tiny_plan(1, layers=6, tuning__tuning_granularity="uniform-device-pp", **overrides)
    got = tune(cfg)
    want = oracle_tune(cfg, tables)
    assert got == want
    assert want[1] is not None


def test_candidate_window_selection_matches_numpy():
    """mist_dp_select_candidates against a numpy filter of the same tables, including open
    ends, empty windows and the retry when the output list is too small."""
    from mist_amd.inter_tuning import _DpRunner
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates

    cfg, tables = load_plan(1)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    res = IntraStageTuner(tables, L, meshes, Gs, 1, cfg, sample_size=1).tune()
    runner = _DpRunner(res, L, hw.num_nodes * hw.num_gpus_per_node, meshes, 0)
    runner._select_capacity = 16  # force the retry path
    host = [np.concatenate([runner.cost[v][g].cpu().numpy().ravel() for v in range(3)]) for g in range(len(Gs))]
    finite = np.concatenate([h[np.isfinite(h)] for h in host])
    assert len(finite) > 100
    q = np.quantile(finite, [0.1, 0.4, 0.6, 0.9]).astype(np.float32)
    rows = np.array([0, 1, len(Gs) - 1, 1, 2, 0], dtype=np.int32)
    lo = np.array([-np.inf, q[0], q[1], q[3], q[2], 1e30], dtype=np.float32)
    hi = np.array([q[1], q[2], np.inf, q[3], q[3], np.inf], dtype=np.float32)
    got = runner.candidates_between(rows, lo, hi)
    for (values, above), g, a, b in zip(got, rows, lo, hi):
        h = host[g][np.isfinite(host[g])]
        want = np.sort(h[(h > a) & (h <= b)])
        assert np.array_equal(values, want)
        assert above == int((h > b).sum())
    assert len(got[3][0]) == 0 and len(got[5][0]) == 0 and len(got[0][0]) > 0


def test_candidate_selection_of_wide_windows_matches_numpy():
    """Windows that select (nearly) every finite stage cost of a table row of the GPT-7B plan:
    each workgroup of the selection kernel then buffers several times its 4096-value LDS list
    and appends it in pieces, a path the small tables never reach.  The selected multiset must
    equal numpy's filter of the same row."""
    from mist_amd.config import tp_candidates
    from mist_amd.inter_tuning import _DpRunner
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates

    cfg, tables = load_plan(2)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    res = IntraStageTuner(tables, L, meshes, Gs, 1, cfg, sample_size=1).tune()
    runner = _DpRunner(res, L, hw.num_nodes * hw.num_gpus_per_node, meshes, 0)
    host = [np.concatenate([runner.cost[v][g].cpu().numpy().ravel() for v in range(3)]) for g in range(len(Gs))]
    dense = int(np.argmax([np.isfinite(h).sum() for h in host]))
    h = host[dense][np.isfinite(host[dense])]
    assert len(h) > 20 * 4096, "the row must overflow the LDS list of its workgroups many times"
    med = np.float32(np.median(h))
    rows = np.array([dense, dense, dense, (dense + 1) % len(Gs)], dtype=np.int32)
    lo = np.array([-np.inf, med, -np.inf, -np.inf], dtype=np.float32)
    hi = np.array([np.inf, np.inf, med, np.inf], dtype=np.float32)
    for _ in range(3):  # the interleaving of the workgroups' waves differs from launch to launch
        got = runner.candidates_between(rows, lo, hi)
        for (values, above), g, a, b in zip(got, rows, lo, hi):
            hg = host[g][np.isfinite(host[g])]
            want = np.sort(hg[(hg > a) & (hg <= b)])
            assert np.array_equal(values, want)
            assert above == int((hg > b).sum())


@pytest.mark.parametrize("capacity, first_chunk, first_lead", [(8192, 48, 16), (256, 7, 7), (8192, 12, 3)])
def test_windows_walked_on_the_device_equal_the_host_walk(capacity, first_chunk, first_lead):
    """``mist_dp_windows_first_batch`` (per-request selection, sort, start of the walk, gap walk
    and first scan batch on the GPU) against the host route it replaces (numpy filter of the
    same tables, ``mist_dp_window_begin``): kept thresholds, their number below the smallest
    feasible threshold, the batch's instances (all of a short window; of a long one the first
    ``first_lead`` thresholds and the rest of the batch spread evenly up to its last one) and
    every status - windows of several widths
    around the real smallest feasible thresholds of the GPT-7B plan, a window whose start cannot
    be certain, an empty one, a skipped request, and (small capacity) windows that overflow."""
    import ctypes

    import torch

    from mist_amd import _lib
    from mist_amd.config import tp_candidates
    from mist_amd.inter_tuning import GAP, _DpRunner
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates

    cfg, tables = load_plan(2)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    res = IntraStageTuner(tables, L, meshes, Gs, tp_candidates(cfg), cfg, sample_size=1).tune_all()
    runner = _DpRunner(res[0], L, hw.num_nodes * hw.num_gpus_per_node, meshes, 0)
    lib = runner.lib
    all_rows = np.arange(len(Gs) * len(res), dtype=np.int32)
    bott, _ = runner.bottleneck(all_rows)
    feasible = all_rows[np.isfinite(bott)]
    assert len(feasible) >= 8
    rows, lo, hi, start = [], [], [], []
    widths = [1.0005, 1.002, 1.01, 1.03, 1.1]
    for k, g in enumerate(feasible):
        b = np.float32(bott[g])
        rows.append(g)
        start.append(b)
        lo.append(np.float32(b - np.float32(1e-4 + 1e-5 * abs(float(b)))))
        hi.append(np.float32(b * widths[k % len(widths)]))
    g0 = int(feasible[0])
    b0 = np.float32(bott[g0])
    # a skipped request, an empty window far above every cost, a window that begins one float
    # below a candidate above the start value (that candidate's predecessor is unknown and may be
    # within the gap: no certain start)
    above_start, _ = runner.candidates_between(
        np.array([g0], dtype=np.int32), np.array([b0 * 1.001], dtype=np.float32),
        np.array([b0 * 1.01], dtype=np.float32))[0]
    c = np.float32(above_start[0])
    rows += [g0, g0, g0]
    start += [np.float32(np.inf), b0, b0]
    lo += [np.float32(0.0), np.float32(1e30), np.nextafter(c, np.float32(0.0))]
    hi += [np.float32(1.0), np.float32(2e30), np.float32(b0 * 1.01)]
    rows = np.array(rows, dtype=np.int32)
    lo, hi, start = (np.array(x, dtype=np.float32) for x in (lo, hi, start))
    n = len(rows)

    dev = runner.device
    kept_capacity = 1 << 18
    d = lambda a: torch.from_numpy(a).to(dev)
    d_rows, d_lo, d_hi, d_start = d(rows), d(lo), d(hi), d(start)
    d_values = torch.empty(n * capacity, dtype=torch.float32, device=dev)
    d_counts = torch.empty(2 + 2 * n, dtype=torch.int32, device=dev)
    d_kept = torch.empty(kept_capacity, dtype=torch.float32, device=dev)
    d_meta = torch.empty(n * 8, dtype=torch.int32, device=dev)
    d_inst_t = torch.full((n * first_chunk,), -7.0, dtype=torch.float32, device=dev)
    d_inst_row = torch.full((n * first_chunk,), -7, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        rc = lib.mist_dp_windows_first_batch(
            ctypes.byref(runner._all_costs), n, d_rows.data_ptr(), d_lo.data_ptr(), d_hi.data_ptr(),
            d_start.data_ptr(), GAP, capacity, first_chunk, first_lead, d_values.data_ptr(), d_counts.data_ptr(),
            d_kept.data_ptr(), kept_capacity, d_meta.data_ptr(), d_inst_t.data_ptr(),
            d_inst_row.data_ptr(), None)
        _lib.check(rc, "mist_dp_windows_first_batch")
        torch.cuda.synchronize()
    meta = d_meta.cpu().numpy().reshape(n, 8)
    kept_all = d_kept.cpu().numpy()
    inst_t = d_inst_t.cpu().numpy()
    inst_row = d_inst_row.cpu().numpy()

    host = runner.candidates_between(rows, lo, hi)
    seen, used, spread = set(), [], 0
    for r in range(n):
        values, above = host[r]
        n_sel, n_above, status, n_kept, base, pos, n_inst, inst_at = (int(x) for x in meta[r])
        want_status = 0
        kept = np.empty(0, dtype=np.float32)
        if not np.isfinite(start[r]):
            want_status = 1
        elif len(values) > capacity:
            want_status = 2
        else:
            out = np.empty(max(len(values), 1), dtype=np.float32)
            k = lib.mist_dp_window_begin(
                ctypes.c_void_p(np.ascontiguousarray(values).ctypes.data), len(values), float(lo[r]), 0,
                float(start[r]), GAP, ctypes.c_void_p(out.ctypes.data))
            if k == _lib.DP_NO_START:
                want_status = 3
            else:
                assert k >= 0
                kept = out[:k]
                if not (kept >= start[r]).any():
                    want_status = 4
        seen.add(want_status)
        assert status == want_status, (r, status, want_status)
        assert n_sel == len(values) and n_above == above
        if status != 0:
            assert n_inst == 0
            continue
        assert n_kept == len(kept) and np.array_equal(kept_all[base:base + n_kept], kept)
        assert pos == int(np.searchsorted(kept, start[r], side="left"))
        assert n_inst == min(first_chunk, n_kept - pos) > 0
        n_avail = n_kept - pos
        picked = [lib.mist_dp_first_batch_index(k, n_avail, first_chunk, first_lead) for k in range(n_inst)]
        if n_avail <= first_chunk or first_lead >= first_chunk:
            assert picked == list(range(n_inst))
        else:
            spread += 1
            assert picked[:first_lead] == list(range(first_lead)) and picked[-1] == n_avail - 1
            assert all(a < b for a, b in zip(picked, picked[1:]))
            steps = np.diff(picked[first_lead - 1:])
            assert steps.max() - steps.min() <= 1
        assert lib.mist_dp_first_batch_index(n_inst, n_avail, first_chunk, first_lead) == -1
        assert np.array_equal(inst_t[inst_at:inst_at + n_inst], kept[pos:][picked])
        assert np.all(inst_row[inst_at:inst_at + n_inst] == rows[r])
        used.append((inst_at, n_inst))
    assert {0, 1, 3, 4} <= seen and (capacity > 1024 or 2 in seen)
    assert spread > 0 or first_lead >= first_chunk
    # the instances of all windows lie behind one another from slot 0 on, the rest is empty
    used.sort()
    assert used[0][0] == 0 and all(a + k == b for (a, k), (b, _) in zip(used, used[1:]))
    n_live = used[-1][0] + used[-1][1]
    assert np.all(inst_row[:n_live] >= 0) and np.all(inst_row[n_live:] == -1)

    # the instances as a DP batch: empty slots come back infeasible, the others as on their own
    fam = runner.families[0]
    flat_row, flat_t = inst_row, inst_t
    live = flat_row >= 0
    bs, bsum, smax = runner.run(np.where(live, flat_row, -1).astype(np.int32), np.where(live, flat_t, 0).astype(np.float32))
    bs1, bsum1, smax1 = runner.run(flat_row[live], flat_t[live])
    assert np.all(bs[~live] == -1)
    assert np.array_equal(bs[live], bs1) and np.array_equal(bsum[live], bsum1)
    assert np.array_equal(smax[live][bs1 >= 0], smax1[bs1 >= 0])


@pytest.mark.parametrize("granularity", ["inter-stage", "uniform-device-pp", "uniform-pp", "no-pp"])
def test_infeasible_plan_returns_inf_none(granularity):
    """Nothing fits into 0.2 GB: every table stays +inf / -1, the searches find no partition and
    the reference's contract is (inf, None) (inter_tuning.py:146-147), also through the oracle."""
    from mist_amd.tune_one_case import tune
    from oracle.tune import tune as oracle_tune

    cfg, tables = tiny_plan(1, layers=4, hardware__memory_capacity=0.2,
                            tuning__tuning_granularity=granularity)
    cost, solution = tune(cfg)
    assert cost == float("inf") and solution is None
    if granularity != "no-pp":
        assert oracle_tune(cfg, tables) == (float("inf"), None)


def test_groups_without_candidates_stay_empty():
    """A (G, mesh) pair without a valid (batch size, dp, tp) factorisation has no rows; the
    reference returns all-inf tables for it (batched_module_analyzer.py:648-666) and so must the
    batched launch, which simply has no group descriptor for it."""
    from mist_amd.intra_tuning import IntraStageTuner

    cfg, tables = tiny_plan(1, layers=4)
    meshes, Gs = [(1, 1), (1, 2)], [1, 8]
    tuner = IntraStageTuner(tables, 4, meshes, Gs, 2, cfg, sample_size=1)
    plan = tuner.prepare()
    present = {(int(r["g_index"]), int(r["q_index"])) for r in plan["groups"]}
    missing = {(g, q) for g in range(2) for q in range(2)} - present
    assert missing, "the case is meant to contain an empty group"
    got = tuner.tune()
    for g, q in missing:
        assert np.all(np.isinf(got.costs_stable[g, q])) and np.all(got.indices[g, q] == -1)
    from oracle.intra import intra_stage_tune
    want = intra_stage_tune(tables, cfg, 4, meshes, Gs, 2, 1)
    assert np.array_equal(got.indices, want.indices)


@pytest.mark.parametrize("plan, overrides", [
    (1, {}), (2, {}), (3, {}),
    (1, dict(model__num_hidden_layers=6, hardware__memory_capacity=6.0)),
    (1, dict(model__num_hidden_layers=7, hardware__num_gpus_per_node=4, training__global_batch_size=16)),
    (1, dict(model__num_hidden_layers=5, hardware__memory_capacity=1.0)),  # nothing fits
])
def test_native_search_equals_python_driver(monkeypatch, plan, overrides):
    """``mist_inter_stage_search`` (the search without the interpreter between the GPU batches)
    against the Python driver it mirrors: cost of every tensor-parallel entry, partitions and
    strategies, and the same number of DP instances and batches (the two make the same
    speculation decisions)."""
    from mist_amd import inter_tuning
    from mist_amd.config import tp_candidates
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates

    cfg, tables = load_plan(plan, **overrides)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    D = hw.num_nodes * hw.num_gpus_per_node
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    results = IntraStageTuner(tables, L, meshes, Gs, tp_candidates(cfg), cfg, sample_size=1).tune_all()
    out = {}
    for native in (True, False):
        monkeypatch.setattr(inter_tuning, "NATIVE_SEARCH", native)
        for only_best in (False, True):
            stats = {}
            got = inter_tuning.inter_stage_tune_batch(L, D, meshes, Gs, results, stats=stats,
                                                      only_best_solution=only_best)
            out[native, only_best] = (got, stats["dp_thresholds"], stats["dp_launches"],
                                      stats["dp_window_values"])
            if stats.get("dp_windows_left_to_host", 0):
                # a window the device left to the host joins the scan one batch later: other
                # batches, the same results
                out[native, only_best] = out[native, only_best][:1]
    for only_best in (False, True):
        n = len(out[True, only_best])
        assert out[True, only_best] == out[False, only_best][:n]
    assert any(sol is not None for _, sol in out[True, False][0]) == (plan != 1 or overrides.get("hardware__memory_capacity") != 1.0)


@pytest.mark.parametrize("plan", [1, 2, 3])
def test_search_decides_its_windows_on_the_device_or_on_the_host_alike(monkeypatch, plan):
    """The library's search driver with the windows and the first scan batch decided on the
    device (its default), on the host (``MIST_INTER_HOST_WINDOWS``), and on the host after the
    device left the windows larger than it holds to it (``MIST_INTER_WINDOW_CAPACITY`` = 128): same
    costs, partitions and strategies, the first two with the same counters; the device route saves
    a round trip."""
    from mist_amd import inter_tuning
    from mist_amd.config import tp_candidates
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates

    cfg, tables = load_plan(plan)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    D = hw.num_nodes * hw.num_gpus_per_node
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    results = IntraStageTuner(tables, L, meshes, Gs, tp_candidates(cfg), cfg, sample_size=1).tune_all()
    out = {}
    for route, env in (("device", {}), ("host", {"MIST_INTER_HOST_WINDOWS": "1"}),
                       ("gave up", {"MIST_INTER_WINDOW_CAPACITY": "128"})):
        for name in ("MIST_INTER_HOST_WINDOWS", "MIST_INTER_WINDOW_CAPACITY"):
            monkeypatch.delenv(name, raising=False)
        for name, value in env.items():
            monkeypatch.setenv(name, value)
        stats = {}
        got = inter_tuning.inter_stage_tune_batch(L, D, meshes, Gs, results, stats=stats)
        out[route] = (got, stats["dp_thresholds"], stats["dp_launches"], stats["dp_window_values"])
        trips = stats["dp_round_trips"]
        if route == "device":
            device_trips = trips
        elif route == "host":
            assert trips == device_trips + 1 or plan == 1
    assert out["device"] == out["host"]
    # windows the device left to the host join the scan one batch later: the same results from
    # other batches
    assert out["gave up"][0] == out["device"][0]
    assert any(sol is not None for _, sol in out["device"][0])


@pytest.mark.parametrize("plan, overrides, ckpt_tuning", [
    (1, {}, True), (2, {}, True), (2, {}, False),
    (1, dict(model__num_hidden_layers=6, hardware__num_nodes=2, hardware__num_gpus_per_node=4,
             training__global_batch_size=32, hardware__memory_capacity=8.0), True),
    (1, dict(model__num_hidden_layers=5, hardware__memory_capacity=1.0), True),  # nothing fits
])
def test_native_search_of_uniform_device_families_equals_python_driver(monkeypatch, plan, overrides,
                                                                        ckpt_tuning):
    """``mist_inter_stage_search_families`` with one DP family per admissible stage count (the
    uniform-device recurrence) against the Python driver: costs, partitions, strategies and the
    number of DP instances run."""
    from mist_amd import inter_tuning
    from mist_amd.config import tp_candidates
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates

    cfg, tables = load_plan(plan, **overrides)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    D = hw.num_nodes * hw.num_gpus_per_node
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    results = IntraStageTuner(tables, L, meshes, Gs, tp_candidates(cfg), cfg, sample_size=1).tune_all()
    uniform = dict(num_nodes=hw.num_nodes, num_gpus_per_node=hw.num_gpus_per_node, ckpt_tuning=ckpt_tuning)
    out = {}
    for native in (True, False):
        monkeypatch.setattr(inter_tuning, "NATIVE_SEARCH", native)
        for only_best in (False, True):
            stats = {}
            got = inter_tuning.inter_stage_tune_batch(L, D, meshes, Gs, results, stats=stats,
                                                      uniform_device=uniform,
                                                      only_best_solution=only_best)
            out[native, only_best] = (got, stats["dp_thresholds"], stats["dp_window_values"])
            if stats.get("dp_windows_left_to_host", 0):
                out[native, only_best] = out[native, only_best][:1]
    for only_best in (False, True):
        n = len(out[True, only_best])
        assert out[True, only_best] == out[False, only_best][:n]
    feasible = any(sol is not None for _, sol in out[True, False][0])
    assert feasible == (overrides.get("hardware__memory_capacity") != 1.0)



class _ToySpace:
    """Stand-in for a group's strategy rows: row index -> ten numbers (the first six whole)."""

    @staticmethod
    def decode(idx):
        idx = np.asarray(idx)
        out = np.full(idx.shape + (10,), np.inf, dtype=np.float64)
        ok = idx >= 0
        base = idx[ok].astype(np.float64)
        out[ok] = np.stack([base % 3 + 1, base % 5, base % 7, base % 2, base % 11, base % 13,
                            base / 4, base / 8, base / 16, base / 32], axis=-1)
        return out


def _synthetic_results(rng, n_entries, Gs, meshes, L, P1, S, quantum, inf_frac, structured,
                       structured_exponent=1.0, jitter=0.0):
    """Random intra-stage tables for ``n_entries`` tensor-parallel entries: in HBM in the layout
    the search kernels write (one leading axis over entry x G), and as the oracle's results
    objects.  Values are multiples of ``quantum`` (exact in float32, many ties after the division
    by G); ``structured`` makes a stage's cost grow with its layers and fall with its devices and
    its micro-batch count, as real tables do; otherwise it is uniform noise times
    ``(max G / G) ** structured_exponent``.  ``jitter`` adds 0..3 times itself to every stable
    cost."""
    import torch
    from mist_amd.intra_tuning import DeviceTables, IntraStageTunerOutput
    from oracle.intra import IntraStageTunerOutput as OracleOutput

    Gn, Q = n_entries * len(Gs), len(meshes)
    shapes = [(Gn, Q, P1, L, L + 1, S), (Gn, Q, P1, L, L + 1, S), (Gn, Q, L, L + 1, S), (Gn, Q, L + 1, S)]
    layers = np.arange(1, L + 1, dtype=np.float64)
    devices = np.array([n * m for n, m in meshes], dtype=np.float64)
    stable, delta, index = [], [], []
    for v, shape in enumerate(shapes):
        # the whole model on one mesh costs about as much as its layers in stages
        per_g = np.tile(max(Gs) / np.array(Gs, dtype=np.float64), n_entries).reshape((Gn,) + (1,) * (len(shape) - 1))
        if structured:
            per_q = (devices ** -0.7).reshape((Q,) + (1,) * (len(shape) - 2))
            per_l = layers.reshape((L, 1, 1)) if v < 3 else L
            scale = np.ones(shape) * per_l * per_q * per_g
        else:
            scale = np.ones(shape) * (1.0 if v < 3 else L / 2) * per_g ** structured_exponent
        s = np.maximum(np.round(rng.uniform(0.3, 1.0, size=shape) * scale / quantum), 1) * quantum
        d = np.round(rng.uniform(0.0, 0.5, size=shape) * scale / quantum) * quantum
        if jitter:  # neighbours closer than the scan's gap of 1e-6
            s = s + rng.integers(0, 4, size=shape) * jitter
        none = rng.random(shape) < (inf_frac if v < 3 else max(inf_frac, 0.6))  # one mesh rarely holds it
        s[none], d[none] = np.inf, np.inf
        idx = rng.integers(0, 1000, size=shape).astype(np.int32)
        idx[none] = -1
        stable.append(s), delta.append(d), index.append(idx)
    whole = DeviceTables(stable=[torch.from_numpy(a).cuda() for a in stable],
                         delta=[torch.from_numpy(a).cuda() for a in delta],
                         index=[torch.from_numpy(a).cuda() for a in index])
    n_g = len(Gs)
    spaces = {(g, q): _ToySpace for g in range(n_g) for q in range(Q)}
    ours, theirs = [], []
    for t in range(n_entries):
        cut = slice(t * n_g, (t + 1) * n_g)
        view = DeviceTables(stable=[x[cut] for x in whole.stable], delta=[x[cut] for x in whole.delta],
                            index=[x[cut] for x in whole.index])
        ours.append(IntraStageTunerOutput(Gs, meshes, view, spaces, range(S), batch=whole, batch_index=t))
        f32 = [a[cut].astype(np.float32) for a in stable] + [a[cut].astype(np.float32) for a in delta]
        theirs.append(OracleOutput(Gs, meshes, *f32, *[_ToySpace.decode(a[cut]) for a in index]))
    return ours, theirs


@pytest.mark.parametrize("seed, L, nodes, gpn, quantum, inf_frac", [
    (0, 8, 1, 8, 1 / 16, 0.15),
    (1, 10, 2, 4, 1 / 64, 0.3),
    (2, 7, 2, 2, 1 / 8, 0.05),
    (3, 11, 2, 4, 1 / 128, 0.2),
    (4, 9, 1, 4, 1 / 32, 0.6),
    (5, 6, 2, 4, 1 / 4, 0.0),
    # larger shapes, up to 11 stages deep: per-mesh only (its oracle DP is compiled C)
    (6, 16, 2, 8, 1 / 256, 0.25),
    (7, 20, 4, 4, 1 / 512, 0.1),
    (8, 24, 4, 8, 1 / 8, 0.4),
])
@pytest.mark.parametrize("recurrence", ["per-mesh", "uniform-device", "uniform-device, ckpt rule"])
def test_search_on_random_tables_equals_the_reference_scan(monkeypatch, seed, L, nodes, gpn, quantum,
                                                           inf_frac, recurrence):
    """The search driver (windows, speculative scan batches, replay, back-pointer run) against
    the reference's own procedure - every candidate threshold in ascending order through the DP,
    with the gap and stop rules of inter_tuning.py:163-217 /
    inter_tuning_uniform_device.py:212-273 - on random tables full of ties that no layer model
    made: up to three tensor-parallel entries searched in one call, each with its own running best, a
    sample slot other than the first, and the driver on each of its routes (windows decided on
    the device, on the host, on the host after the device gave up, the Python driver)."""
    from mist_amd import inter_tuning
    from oracle import inter_dp, inter_uniform_device
    from oracle.dp_c import dp_impl_c

    if seed >= 6 and recurrence != "per-mesh":
        pytest.skip("the uniform-device oracle is interpreted loops: small shapes only")
    rng = np.random.default_rng(9100 + seed)
    D = nodes * gpn
    n_entries = {7: 2, 8: 1}.get(seed, 3)
    meshes = [(1, 1 << k) for k in range(gpn.bit_length()) if (1 << k) <= gpn]
    meshes += [(n, gpn) for n in range(2, nodes + 1) if nodes % n == 0]
    Gs = [1, 2, 4, 8, 32][:3 + seed % 3]
    P1 = min(D, L)
    S, slot = 2, 1
    ours, theirs = _synthetic_results(rng, n_entries, Gs, meshes, L, P1, S, quantum, inf_frac,
                                      structured=seed % 2 == 0,
                                      structured_exponent=(1.1, 1.0, 0.9)[seed // 2 % 3],
                                      jitter=3e-7 if seed in (3, 4, 7) else 0.0)
    if recurrence == "per-mesh":
        uniform = None
        want = [inter_dp.inter_stage_tune(L, D, meshes, Gs, r, slot, dp=dp_impl_c) for r in theirs]
    else:
        ckpt_tuning = recurrence == "uniform-device"
        uniform = dict(num_nodes=nodes, num_gpus_per_node=gpn, ckpt_tuning=ckpt_tuning)

        class Config:
            class tuning:
                activation_checkpointing_tuning_enabled = ckpt_tuning

        want = [inter_uniform_device.inter_stage_tune(L, nodes, gpn, meshes, Gs, r, Config, slot)
                for r in theirs]
    if inf_frac < 0.5:
        assert any(sol is not None for _, sol in want), "degenerate case"
    routes = [(True, {}), (True, {"MIST_INTER_HOST_WINDOWS": "1"}),
              (True, {"MIST_INTER_WINDOW_CAPACITY": "128"}), (False, {})]
    for native, env in routes:
        for name in ("MIST_INTER_HOST_WINDOWS", "MIST_INTER_WINDOW_CAPACITY"):
            monkeypatch.delenv(name, raising=False)
        for name, value in env.items():
            monkeypatch.setenv(name, value)
        monkeypatch.setattr(inter_tuning, "NATIVE_SEARCH", native)
        got = inter_tuning.inter_stage_tune_batch(L, D, meshes, Gs, ours, slot=slot,
                                                  uniform_device=uniform)
        assert got == want, (native, env)
    got = inter_tuning.inter_stage_tune_batch(L, D, meshes, Gs, ours, slot=slot, uniform_device=uniform,
                                              only_best_solution=True)
    finite = [i for i, (_, sol) in enumerate(want) if sol is not None]
    keep = min(finite, key=lambda i: want[i][0]) if finite else None
    assert got == [(cost, sol if i == keep else None) for i, (cost, sol) in enumerate(want)]


@pytest.mark.parametrize("L, P1, quantum, inf_frac", [(8, 3, 1 / 16, 0.3), (40, 2, None, 0.1), (80, 2, 1 / 4, 0.5),
                                                      (130, 2, None, 0.0)])
def test_cost_tables_and_running_minima_equal_numpy(L, P1, quantum, inf_frac):
    """``mist_dp_cost_tables``: float32 cost = float32(stable) + float32(delta) / G of the sample
    slot, +inf where the cell holds no strategy, and beside it the running minimum over the ckpt
    counts of each table row - rows of 9 to 131 entries, i.e. several rows per wavefront up to a
    row across three wavefronts - against numpy on random tables with ties."""
    from mist_amd.inter_tuning import _DpRunner

    rng = np.random.default_rng(L)
    meshes, Gs, S, slot = [(1, 1), (1, 2), (1, 4)], [1, 2, 8], 2, 1
    ours, theirs = _synthetic_results(rng, 2, Gs, meshes, L, P1, S, quantum or 1 / 1024, inf_frac,
                                      structured=False)
    runner = _DpRunner(ours[0], L, 4, meshes, slot)
    G_of_row = np.tile(np.array(Gs, dtype=np.float32), 2)
    names = ("costs_stable", "costs_stable_with_pre", "costs_stable_with_post", "costs_stable_no_pp")
    for v, name in enumerate(names):
        stable = np.concatenate([getattr(t, name)[..., slot] for t in theirs])
        delta = np.concatenate([getattr(t, name.replace("stable", "delta"))[..., slot] for t in theirs])
        with np.errstate(invalid="ignore"):
            want = (stable + delta / G_of_row.reshape((-1,) + (1,) * (stable.ndim - 1))).astype(np.float32)
        got, got_min = runner.cost[v].cpu().numpy(), runner.pmin[v].cpu().numpy()
        assert np.array_equal(got.view(np.int32), want.view(np.int32)), name
        assert np.array_equal(got_min.view(np.int32), np.minimum.accumulate(want, axis=-1).view(np.int32)), name
        assert np.isfinite(want).any() and np.isinf(want).any() or inf_frac == 0.0
