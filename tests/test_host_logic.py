"""CPU tests of the package's host side: configuration, kernel-input preparation (bit-exact
against the oracle's own derivation), launch decomposition, output formatting, and the C ABI
(library loads and exports every symbol the headers declare; no compute calls)."""
import ctypes
import os
import re

import numpy as np
import pytest
import yaml

from mist_amd import _lib
from mist_amd.config import MistConfig, tp_candidates
from mist_amd.intra_tuning import IntraStageTuner, alpha_ratios
from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates
from mist_amd.stage_inputs import interference_factor_table, make_problem
from oracle.interference import mask_factor_table
from oracle.pareto import alpha_ratios as oracle_alpha_ratios
from oracle.stage import batched_tune_best_latency_for_stage
from tests.util import REPO, assert_same_f64, load_plan, load_raw, tiny_plan


def test_config_surface():
    cfg, _ = load_plan(2)
    assert cfg.hardware.memory_capacity == 80.0 * 0.88
    assert cfg.tuning.tuning_granularity == "inter-stage" and cfg.strategy is None
    assert cfg.enable_advanced_opt_in_first_block is True
    assert getattr(cfg, "fixed_wo_ratio", None) is None
    with pytest.raises(AttributeError):
        cfg.not_a_key
    assert tp_candidates(cfg) == [1, 2, 4, 8]
    cfg1, _ = load_plan(1, disable_tp_tuning=True)
    assert tp_candidates(cfg1) == [1]
    raw = load_raw(1)
    raw["tuning"]["tuning_granularity"] = "bogus"
    with pytest.raises(AssertionError):
        MistConfig(raw)
    raw = load_raw(1)
    raw["hardware"]["interference_model_params"] = [1.0] * 27
    with pytest.raises(AssertionError):
        MistConfig(raw)
    # defaults of the optional search-space block are the reference's module constants
    raw = load_raw(1)
    del raw["tuning"]["search_space"]
    t = MistConfig(raw).tuning
    assert t.batch_size_candidates == (1, 2, 4)
    assert t.offloading_ratio_candidates == (0.0, 0.25, 0.375, 0.5, 0.625, 0.75, 0.875, 1.0)
    assert t.sparse_offloading_ratio_candidates == (0.0, 0.25, 0.375, 0.5, 0.75, 1.0)
    assert t.zero_flag_choices == ((0, 0, 1), (0, 1, 1), (1, 1, 1))


def test_interference_table_and_ratios_match_oracle():
    p = np.random.default_rng(0).uniform(1, 3, 28)
    table = interference_factor_table(p)
    bits = [0xF, 0x7, 0xB, 0xD, 0xE, 0x3, 0x5, 0x9, 0x6, 0xA, 0xC]  # kMaskBits of the kernel
    for row, ((mask, factors), b) in enumerate(zip(mask_factor_table(p), bits)):
        assert np.array_equal(table[row], factors)
        assert sum(1 << j for j in range(4) if mask[j]) == b
    for S in (1, 4, 30):
        assert np.array_equal(alpha_ratios(S), oracle_alpha_ratios(S))
    with pytest.raises(ValueError):
        interference_factor_table(p[:20])


@pytest.mark.parametrize("overrides,tp", [
    (dict(), 1), (dict(), 2),
    (dict(tuning__pre_post_strategy="intra-node-tp-with-ore", model__use_flash_attn=True), 2),
    (dict(hardware__num_nodes=2, hardware__num_gpus_per_node=4, training__global_batch_size=64,
          tuning__pre_post_strategy="intra-node-tp-without-ore"), 4),
])
@pytest.mark.parametrize("builder", ["library", "python"])
def test_group_descriptors_bit_exact_against_oracle(monkeypatch, overrides, tp, builder):
    """Every per-group scalar and per-(b, tp) table value that is handed to the kernels equals
    what the oracle derives for the same group, bit for bit: from the plan builder in the
    library (``mist_plan_groups``, the default) and from the python builder."""
    if builder == "python":
        monkeypatch.setenv("MIST_PYTHON_PLAN_BUILDER", "1")
    else:
        monkeypatch.delenv("MIST_PYTHON_PLAN_BUILDER", raising=False)
    cfg, tables = tiny_plan(1, layers=4, **overrides)
    hw = cfg.hardware
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    tuner = IntraStageTuner(tables, 4, meshes, Gs, tp, cfg, sample_size=1, device="cpu")
    if builder == "library":
        assert tuner._build_groups_native() is not None, "the library's builder declined the plan"
    plan = tuner.prepare()
    assert len(plan["groups"]) > 0
    P = _lib.PAR
    for rec in plan["groups"]:
        n, m, G = int(rec["num_nodes"]), int(rec["num_gpus_per_node"]), int(rec["grad_accum"])
        dbg = {}
        batched_tune_best_latency_for_stage(tables, cfg, [0], [1, 2, 3, 4], [0, 1, 2, 3, 4], n, m, G,
                                            tp_size=tp, sample_size=1, debug=dbg)
        rows = dbg["rows"]
        assert rows.shape[0] == rec["n_rows"]
        space = plan["spaces"][(0, int(rec["g_index"]), int(rec["q_index"]))]
        assert np.array_equal(space.materialize(), rows)
        first = np.arange(0, rows.shape[0], int(rec["n_off"]))  # first row of every parallelism block
        par = rec["par"][: int(rec["n_par"])]
        assert np.array_equal(par[:, :6], rows[first, :6])
        bc = lambda a: np.broadcast_to(np.asarray(a, dtype=np.float64), (rows.shape[0],))[first]
        for name, key in [("exec_fwd", "exec_fwd"), ("exec_bwd", "exec_bwd_nock"), ("extra_fwd", "extra_fwd"),
                          ("extra_bwd", "extra_bwd"), ("fwd_peak", "fwd_peak_nock"), ("bwd_peak", "bwd_peak"),
                          ("out", "out"), ("gcb", "gcb")]:
            assert_same_f64(par[:, P[name]], bc(dbg[key]), name)
        # raw saved activations: S = raw * (1 - ao) with ao == 0 in the first row of each block
        assert_same_f64(par[:, P["raw_ck"]], bc(dbg["S_ck"]), "raw_ck")
        assert_same_f64(par[:, P["raw_nock"]], bc(dbg["S_nock"]), "raw_nock")
        pre, post = dbg["pre"], dbg["post"]
        for name, want in [
            ("pre_full_w", pre["W"]), ("pre_full_g", pre["G"]), ("post_full_w", post["W"]),
            ("post_full_g", post["G"]), ("pre_states", pre["states"]), ("pre_saved", pre["saved"]),
            ("pre_states_and_saved", pre["states"] + pre["saved"]), ("post_states", post["states"]),
            ("post_fwd_peak", post["fwd_peak"]), ("post_bwd_peak", post["bwd_peak"]),
            ("post_output", post["output"]), ("pre_fwd", pre["fwd"]), ("pre_bwd", pre["bwd"]),
            ("post_fwd", post["fwd"]), ("post_bwd", post["bwd"]), ("pre_ag", pre["AG"]),
            ("pre_rs", pre["RS"]), ("post_ag", post["AG"]), ("post_rs", post["RS"]),
        ]:
            assert_same_f64(np.array([rec[name]]), np.asarray(want, dtype=np.float64).reshape(1), name)
    prob = plan["problem"][0]
    assert prob["mem_cap_mb"] == cfg.hardware.memory_capacity * (1 << 30) / (1 << 20)
    assert prob["num_layers"] == 4 and prob["sample_size"] == 1


def _same_plans(a, b):
    """Two ``IntraStageTuner.prepare()`` results hold the same bytes (padding aside)."""
    def same_records(x, y):
        assert x.dtype == y.dtype and x.shape == y.shape
        for name in x.dtype.names:
            assert np.ascontiguousarray(x[name]).tobytes() == np.ascontiguousarray(y[name]).tobytes(), name

    same_records(a["groups"], b["groups"])
    same_records(a["problem"], b["problem"])
    for key in ("terms_prefix", "reduce_prefix", "scout_prefix"):
        assert a[key].dtype == b[key].dtype and np.array_equal(a[key], b[key]), key
    assert a["total_rows"] == b["total_rows"] and len(a["batches"]) == len(b["batches"])
    for x, y in zip(a["batches"], b["batches"]):
        assert x.keys() == y.keys()
        for key in x:
            if key == "groups":
                same_records(x[key], y[key])
            elif isinstance(x[key], np.ndarray):
                assert x[key].dtype == y[key].dtype and np.array_equal(x[key], y[key]), key
            else:
                assert x[key] == y[key], key
    assert list(a["spaces"]) == list(b["spaces"])
    for key in a["spaces"]:
        sa, sb = a["spaces"][key], b["spaces"][key]
        assert sa.par.shape == sb.par.shape and np.array_equal(sa.par, sb.par), key
        assert (sa.wo, sa.go, sa.oo, sa.ao) == (sb.wo, sb.go, sb.oo, sb.ao)
        assert np.array_equal(sa.pair_wo, sb.pair_wo) and np.array_equal(sa.pair_go, sb.pair_go)
        assert sa.n_rows == sb.n_rows


def _both_builders(cfg, tables, tp="all", **kw):
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    cells_wanted = kw.pop("cells_wanted", None)
    evaluate_all_p = kw.pop("evaluate_all_p", False)
    tuner = IntraStageTuner(tables, L, meshes, Gs, tp_candidates(cfg) if tp == "all" else tp, cfg,
                            sample_size=kw.pop("sample_size", 1), device="cpu", **kw)
    tuner.cells_wanted, tuner.evaluate_all_p = cells_wanted, evaluate_all_p
    native = tuner._build_groups_native()
    assert native is not None, "the library's builder declined the plan"
    return tuner._finish_plan(*native), tuner._finish_plan(*tuner._build_groups_python())


@pytest.mark.parametrize("plan", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("kw", [dict(), dict(exhaustive=True), dict(tp=None), dict(tp=2),
                                dict(evaluate_all_p=True, sample_size=30)],
                         ids=["all tp", "exhaustive", "tp latched", "tp 2", "every p"])
def test_plan_builder_of_the_library_equals_the_python_builder(plan, kw):
    """``mist_plan_groups`` against the python host side it replaces on the five benchmark plans
    (GPT with absolute positions and plain MLP, LLaMA with gated MLP, RMSNorm and grouped kv
    heads; 1 to 10 batches of groups): every field of every group descriptor, the problem
    record, the workgroup prefixes, the batches and every search space, byte for byte."""
    cfg, tables = load_plan(plan)
    got, want = _both_builders(cfg, tables, **dict(kw))
    assert len(got["groups"]) > 0
    _same_plans(got, want)


@pytest.mark.parametrize("overrides", [
    dict(model__use_flash_attn=False),
    dict(model__use_flash_attn=False, model__mlp_type="gated_mlp", model__normalization="rmsnorm",
         model__position_embedding_type="rotary", model__tie_word_embeddings=True),
    dict(tuning__pre_post_strategy="intra-node-tp-with-ore"),
    dict(tuning__pre_post_strategy="intra-node-tp-without-ore", hardware__num_nodes=2,
         hardware__num_gpus_per_node=4, training__global_batch_size=64),
    dict(hardware__num_nodes=4, hardware__num_gpus_per_node=8, training__global_batch_size=96),
    dict(tuning__zero_2_and_3_enabled=False, hardware__num_gpus_per_node=8, training__global_batch_size=48),
    dict(tuning__state_offloading_enabled=False),
    dict(tuning__activation_offloading_enabled=False, disable_wo_tuning=True, fixed_oo_ratio=0.5),
    dict(disable_tp_tuning=True, hardware__num_gpus_per_node=4),
    dict(hardware__memory_capacity=0.5),
    dict(training__params_dtype="float32"),
    dict(training__optimizer_name="sgd", hardware__num_gpus_per_node=8),
    dict(model__num_attention_heads=12, model__hidden_size=1536, hardware__num_gpus_per_node=8,
         training__global_batch_size=32),   # heads do not split over tp 8
], ids=lambda o: ",".join(f"{k.split('__')[-1]}={v}" for k, v in o.items())[:60])
def test_plan_builder_of_the_library_on_plan_variants(overrides):
    cfg, tables = tiny_plan(1, layers=10, **overrides)
    _same_plans(*_both_builders(cfg, tables))
    _same_plans(*_both_builders(cfg, tables, tp=None))


def test_plan_builder_of_the_library_with_cell_windows():
    """Callers that read a range of layer counts only (``cells_wanted``): same groups left out,
    same tile windows and pre-saved micro-batch counts."""
    from mist_amd.inter_tuning_mip import cells_wanted

    for plan in (2, 3):
        cfg, tables = load_plan(plan)
        hw = cfg.hardware
        wanted = cells_wanted(cfg.model.num_hidden_layers, hw.num_nodes, hw.num_gpus_per_node)
        got, want = _both_builders(cfg, tables, cells_wanted=wanted, sample_size=30)
        assert 0 < len(got["groups"])
        assert got["groups"]["lc_tile_begin"].max() > 0
        _same_plans(got, want)
    _same_plans(*_both_builders(cfg, tables, cells_wanted=lambda G, mesh: None))
    _same_plans(*_both_builders(cfg, tables, cells_wanted=lambda G, mesh: (3, 2, 1) if G > 4 else (0, 99, 2)))


@pytest.mark.parametrize("seed", range(12))
def test_plan_builder_of_the_library_on_random_configurations(seed):
    """Seeded random model shapes, cluster shapes, batch sizes, efficiencies and communication
    parameters: the builder in the library and the python builder write the same plan."""
    rng = np.random.default_rng(7700 + seed)
    heads = int(rng.choice([8, 16, 32, 40, 64]))
    gg = []
    for _ in range(16):
        gg += [float(rng.uniform(8, 500)), float(rng.uniform(2e-6, 8e-5))]
    nodes, gpus_per_node = int(rng.choice([1, 2, 4, 16])), int(rng.choice([1, 2, 4, 8]))
    overrides = dict(
        model__num_attention_heads=heads, model__hidden_size=heads * int(rng.choice([64, 96, 128])),
        model__num_heads_kv=int(rng.choice([heads, max(heads // 4, 1), 8])) if seed % 2 else None,
        model__mlp_type=str(rng.choice(["mlp", "gated_mlp"])),
        model__normalization=str(rng.choice(["layernorm", "rmsnorm"])),
        model__position_embedding_type=str(rng.choice(["absolute", "rotary"])),
        model__tie_word_embeddings=bool(rng.integers(0, 2)),
        model__use_flash_attn=bool(rng.integers(0, 2)),
        training__max_sequence_length=int(rng.choice([512, 2048, 4096, 3000])),
        training__global_batch_size=nodes * gpus_per_node * int(rng.choice([1, 2, 4, 16])) * int(rng.choice([1, 1, 1, 3])),
        hardware__num_nodes=nodes, hardware__num_gpus_per_node=gpus_per_node,
        hardware__memory_capacity=float(rng.uniform(2.0, 90.0)),
        hardware__gpu_gpu_comm_params=gg,
        tuning__pre_post_strategy=str(rng.choice(["dp", "intra-node-tp-with-ore", "intra-node-tp-without-ore"])),
        synthetic=dict(seed=int(rng.integers(0, 1000)), peak_tflops=float(rng.uniform(100, 2500)),
                       hbm_gbps=float(rng.uniform(900, 8000))),
    )
    cfg, tables = tiny_plan(1, layers=int(rng.integers(2, 40)), **overrides)
    got, want = _both_builders(cfg, tables)
    # (a factor of three in the batch size leaves no data-parallel size that divides the devices)
    assert len(got["groups"]) > 0 or cfg.training.global_batch_size % 3 == 0
    _same_plans(got, want)
    _same_plans(*_both_builders(cfg, tables, tp=None, exhaustive=True))


def test_plans_outside_the_library_builder_go_through_the_python_builder():
    """What ``mist_plan_groups`` declines (here: a collective over three devices, which the
    alpha-beta tables do not hold) is built, and its error worded, by the python host side."""
    cfg, tables = tiny_plan(1, layers=4, hardware__num_gpus_per_node=6, training__global_batch_size=24,
                            tuning__pre_post_strategy="dp")
    meshes = [(1, 1), (1, 2), (1, 6)]
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    tuner = IntraStageTuner(tables, 4, meshes, Gs, [1], cfg, sample_size=1, device="cpu")
    assert tuner._build_groups_native() is None
    assert b"communication group size" in _lib.load().mist_last_error()
    with pytest.raises(ValueError, match="communication group size"):
        tuner.prepare()


@pytest.mark.parametrize("plan", [2, 5])
def test_column_wise_fill_equals_record_by_record_fill(plan):
    """``GroupInputBuilder.fill_many`` (what a tuner call uses) writes the same bytes as ``fill``
    record by record, for every group of a benchmark plan with all its tp candidates."""
    from mist_amd.config import tp_candidates
    from mist_amd.stage_inputs import GroupInputBuilder
    from tests.util import load_plan

    cfg, tables = load_plan(plan)
    hw = cfg.hardware
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    tuner = IntraStageTuner(tables, cfg.model.num_hidden_layers, meshes, Gs, tp_candidates(cfg), cfg,
                            sample_size=1, device="cpu")
    groups = tuner.prepare()["groups"]
    assert len(groups) > 50
    builder = GroupInputBuilder(cfg, tables)
    one = np.zeros(len(groups), dtype=_lib.GROUP_DTYPE)
    spaces = tuner.prepare()["spaces"]
    for i, rec in enumerate(groups):
        row_g, q = int(rec["g_index"]), int(rec["q_index"])
        space = spaces[(row_g // len(Gs), row_g % len(Gs), q)]
        builder.fill(one[i], space, row_g, q, int(rec["num_nodes"]), int(rec["num_gpus_per_node"]),
                     int(rec["grad_accum"]), int(rec["num_p"]))
    decomposition = ("rows_per_chunk", "n_chunks", "n_lc_tiles", "n_p_tiles", "scout_stride", "scout_pair",
                     "row_offset", "key_offset")
    for name in _lib.GROUP_DTYPE.names:
        if name not in decomposition:
            assert np.ascontiguousarray(one[name]).tobytes() == np.ascontiguousarray(groups[name]).tobytes(), name


def test_tile_windows_hold_the_cells_the_stage_assignment_reads():
    """``cells_wanted`` of the uniform-device-pp-mip granularity (inter_tuning_mip.py:267-290) turned
    into tile windows by ``IntraStageTuner.prepare``: every (layers, ckpt) pair of the wanted layer
    counts lies in its group's window, the window is not larger than the tiles those pairs touch,
    groups whose mesh is no even split of the cluster are left out, and the pre-saved micro-batch
    values stop at the stage count."""
    from mist_amd.config import tp_candidates
    from mist_amd.inter_tuning_mip import cells_wanted
    from tests.util import load_plan

    for plan_no in (2, 3):
        cfg, tables = load_plan(plan_no)
        hw, L = cfg.hardware, cfg.model.num_hidden_layers
        D = hw.num_nodes * hw.num_gpus_per_node
        meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
        Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
        whole = IntraStageTuner(tables, L, meshes, Gs, tp_candidates(cfg), cfg, sample_size=1, device="cpu")
        part = IntraStageTuner(tables, L, meshes, Gs, tp_candidates(cfg), cfg, sample_size=1, device="cpu")
        wanted = part.cells_wanted = cells_wanted(L, hw.num_nodes, hw.num_gpus_per_node)
        g_all, g_part = whole.prepare()["groups"], part.prepare()["groups"]
        assert np.all(g_all["lc_tile_begin"] == 0)
        assert 0 < len(g_part) <= len(g_all)
        assert g_part["n_lc_tiles"].sum() * 2 < g_all["n_lc_tiles"][:len(g_part)].sum()
        kept = set()
        for rec in g_part:
            G, mesh = int(rec["grad_accum"]), (int(rec["num_nodes"]), int(rec["num_gpus_per_node"]))
            l_min, l_max, p_count = wanted(G, mesh)
            assert D % (mesh[0] * mesh[1]) == 0 and p_count == D // (mesh[0] * mesh[1])
            first_pair = l_min * (l_min + 1) // 2 - 1            # (l_min, ckpt 0)
            last_pair = l_max * (l_max + 1) // 2 - 1 + l_max     # (l_max, ckpt l_max)
            begin, count = int(rec["lc_tile_begin"]), int(rec["n_lc_tiles"])
            assert begin == first_pair // _lib.LC_TILE
            assert begin + count - 1 == last_pair // _lib.LC_TILE
            assert rec["num_p"] <= p_count
            kept.add((int(rec["g_index"]), int(rec["q_index"])))
        for rec in g_all:  # what was left out is not read
            if (int(rec["g_index"]), int(rec["q_index"])) not in kept:
                assert wanted(int(rec["grad_accum"]), (int(rec["num_nodes"]), int(rec["num_gpus_per_node"]))) is None


def test_launch_decomposition_covers_every_row_once():
    cfg, tables = load_plan(2)
    hw = cfg.hardware
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    tuner = IntraStageTuner(tables, 32, meshes, Gs, 2, cfg, sample_size=1, device="cpu")
    plan = tuner.prepare()
    g = plan["groups"]
    assert np.all(g["n_chunks"] * g["rows_per_chunk"] >= g["n_rows"])
    assert np.all((g["n_chunks"] - 1) * g["rows_per_chunk"] < g["n_rows"])
    assert np.all(g["rows_per_chunk"] % _lib.STAGE_ROWS == 0)
    assert np.array_equal(g["row_offset"], np.concatenate(([0], np.cumsum(g["n_rows"])[:-1])))
    assert np.all(g["n_p_tiles"] * _lib.P_TILE >= g["num_p"])
    pairs = 32 * 33 // 2 + 32
    assert np.all(g["n_lc_tiles"] * _lib.LC_TILE >= pairs)
    blocks = np.diff(plan["reduce_prefix"])
    assert np.array_equal(blocks, g["n_chunks"] * g["n_lc_tiles"] * g["n_p_tiles"])
    assert np.array_equal(np.diff(plan["terms_prefix"]), -(-g["n_rows"] // _lib.TERMS_BLOCK))
    assert tuner.max_possible_pre_saved_micro_batches == 31
    assert plan["total_rows"] == int(g["n_rows"].sum()) == 913308


def test_workspace_batches_partition_the_groups(monkeypatch):
    """Batches are runs of consecutive groups under the row-term workspace bound, each with row
    offsets and workgroup prefixes that start at zero."""
    from mist_amd import _lib, intra_tuning
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates

    cfg, tables = load_plan(1)
    hw = cfg.hardware
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    for budget_rows in (1, 700, 3000, 10**9):
        monkeypatch.setattr(intra_tuning, "ROW_TERMS_BUDGET_BYTES", budget_rows * 8 * _lib.ROW_TERMS)
        plan = IntraStageTuner(tables, cfg.model.num_hidden_layers, meshes, Gs, [1, 2], cfg, sample_size=1).prepare()
        groups, batches = plan["groups"], plan["batches"]
        assert [b["first"] for b in batches] == [0] + [b["last"] for b in batches[:-1]]
        assert batches[-1]["last"] == len(groups)
        for b in batches:
            sub, whole = b["groups"], groups[b["first"]:b["last"]]
            assert b["total_rows"] == int(whole["n_rows"].sum())
            assert len(sub) == 1 or b["total_rows"] <= budget_rows
            assert sub["row_offset"][0] == 0
            assert np.array_equal(np.diff(sub["row_offset"]), whole["n_rows"][:-1])
            # keys = (parallelism row, activation ratio, offload pair): n_rows / n_oo per group
            keys = whole["n_par"].astype(np.int64) * whole["n_ao"] * whole["n_pair"]
            assert np.array_equal(keys * whole["n_oo"], whole["n_rows"])
            assert sub["key_offset"][0] == 0 and np.array_equal(np.diff(sub["key_offset"]), keys[:-1])
            assert b["total_keys"] == int(keys.sum())
            assert int(plan["problem"]["max_group_keys"][0]) >= int(keys.max())
            for name in ("terms_prefix", "reduce_prefix", "scout_prefix"):
                assert b[name][0] == 0 and len(b[name]) == len(sub) + 1
                assert np.array_equal(np.diff(b[name]), np.diff(plan[name][b["first"]:b["last"] + 1]))
            for field in ("g_index", "q_index", "n_rows", "n_chunks", "scout_stride"):
                assert np.array_equal(sub[field], whole[field])
        if budget_rows == 10**9:
            assert len(batches) == 1


@pytest.mark.parametrize("plan, expected", [
    (2, {1: 72}),           # GPT-7B: the first offload pair only
    (3, {1: 110}),          # LLaMA-13B: likewise
    (5, {1: 24, 3: 96}),    # LLaMA-70B: tp 8 alone holds 30 % of the layers of a stage unsharded
])
def test_scout_pairs_follow_the_memory_pressure_of_a_group(plan, expected):
    """Which offload pairs the scout pass gathers (speed only, never results): the first one, and
    the middle and last one as well for groups none of whose parallelism rows holds 30 % of the
    model's layers within the capacity without sharding or offloading."""
    cfg, tables = load_plan(plan)
    hw = cfg.hardware
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    L = cfg.model.num_hidden_layers
    g = IntraStageTuner(tables, L, meshes, Gs, tp_candidates(cfg), cfg, sample_size=1,
                        device="cpu").prepare()["groups"]
    strides, counts = np.unique(g["scout_stride"], return_counts=True)
    assert dict(zip(strides.tolist(), counts.tolist())) == expected
    for d in g:
        par = d["par"][:d["n_par"]]
        states = (par[:, _lib.PAR["W"]] + par[:, _lib.PAR["G"]] + par[:, _lib.PAR["O"]]).min()
        tight = hw.memory_capacity * 1024.0 < 0.3 * L * states
        assert (d["scout_stride"] == 3) == tight
        picked = d["scout_pair"][:d["scout_stride"]].tolist()
        assert picked == ([0, (d["n_pair"] - 1) // 2, d["n_pair"] - 1] if tight else [0])


def test_best_solution_yaml_format():
    from mist_amd.tune_one_case import best_solution_yaml

    raw = load_raw(1)
    sol = [16, [(((0, 11), (1, 1), 5, 0), (2, 1, 1, 0, 0, 1, 0.0, 0.0, 0.0, 0.0)),
                (((12, 23), (1, 1), 0, 0), (2, 1, 1, 0, 0, 1, 0.0, 0.0, 0.0, 0.0))]]
    out = yaml.safe_load(best_solution_yaml(raw, sol))
    s = out["strategy"]
    assert s["enabled"] is True and s["gradient_accumulation_steps"] == 16
    assert s["layer_partitions"] == [12, 12] and s["device_assignment"] == [[1, 1], [1, 1]]
    assert s["gradient_checkpointing"] == [5, 0]
    assert s["stage_strategies"] == [[2, 1, 1, 0, 0, 1, 0.0, 0.0, 0.0, 0.0]] * 2
    assert s["pre_post_strategy"] == "preset"
    assert s["pre_post_strategy_array"] == [2, 1, 1, 0, 0, 1, 0, 0, 0, 0]
    assert out["model"] == raw["model"]


def test_mip_search_needs_the_gpu_library_path():
    """The MIP granularity has no CPU path either: without a GPU the intra-stage tuner refuses."""
    import torch

    from mist_amd._lib import MistLibraryError
    from mist_amd.tune_one_case import tune

    if torch.cuda.is_available():
        pytest.skip("covers the host without a GPU")
    cfg, _ = load_plan(1, tuning__tuning_granularity="uniform-device-pp-mip")
    with pytest.raises(MistLibraryError):
        tune(cfg)


def test_mip_layer_candidates_match_oracle():
    from mist_amd.inter_tuning_mip import layer_candidates
    from oracle.inter_mip import layer_candidates as want

    for L in (1, 2, 7, 10, 14, 32, 80):
        for S in range(1, L + 1):
            for G in (1, 2, 64):
                for off in (0, 1, 2, 3):
                    lo, hi = layer_candidates(L, S, G, off)
                    assert list(range(lo, hi + 1)) == want(L, S, G, off), (L, S, G, off)


def _declared_functions():
    names = []
    for header in ("mist_search.h", "mist_dp.h", "mist_mip.h", "mist_inter.h", "mist_plan.h"):
        text = open(os.path.join(REPO, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"\b(mist_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_library_loads_and_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_functions()
    assert len(declared) >= 12
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/ but not exported"
    assert set(_lib.exported_symbols()) == set(declared)
    assert lib.mist_sizeof_problem() == _lib.PROBLEM_DTYPE.itemsize
    assert lib.mist_sizeof_group() == _lib.GROUP_DTYPE.itemsize
    assert lib.mist_sizeof_dp_shape() == _lib.DP_SHAPE_DTYPE.itemsize
    assert b"gfx950" in lib.mist_version()


def test_argument_checks_reject_before_any_launch():
    """Host-side validation paths of the C ABI (no GPU needed: they return before launching)."""
    lib = _lib.load()
    hp = lambda a: ctypes.c_void_p(a.ctypes.data)
    assert lib.mist_row_terms(None, None, 1, None, 1, None, None, None, None) == -1
    assert b"null" in lib.mist_last_error()
    prob = make_problem(load_plan(1)[0], 4, 2, 1, 4, 2)
    pp = ctypes.c_void_p(prob.ctypes.data)
    fake = ctypes.c_void_p(4096)
    assert lib.mist_row_terms(pp, fake, 0, fake, 1, fake, fake, None, None) == -1
    assert lib.mist_row_terms(pp, fake, 1, fake, 1, fake, None, None, None) == -1
    for bad_factor in (0.0, -1.5, float("inf"), float("nan")):  # the kernel relies on 0 / f == +0
        bad = prob.copy()
        bad["interf_factor"][0][7, 2] = bad_factor
        assert lib.mist_row_terms(ctypes.c_void_p(bad.ctypes.data), fake, 1, fake, 1, fake, fake, None, None) == -1
        assert b"interference factor [7][2]" in lib.mist_last_error()
    assert lib.mist_stage_floor_doubles(640, 3) == (10 + 3 + 1) * 32 and lib.mist_stage_floor_doubles(-1, 3) == -1
    assert lib.mist_eval_reduce(pp, fake, 1, fake, 0, None, 0, fake, fake, 1.0, fake, fake, None) == -1
    assert lib.mist_eval_reduce(pp, fake, 1, fake, 1, None, 0, fake, fake, -1.0, fake, fake, None) == -1
    assert lib.mist_eval_reduce(pp, fake, 1, fake, 1, None, 3, fake, fake, 1.0, fake, fake, None) == -1
    assert b"scout" in lib.mist_last_error()
    # the evaluate-every-cell launch and the multi-sample call check the same things
    assert lib.mist_eval_reduce_exhaustive(pp, fake, 1, fake, 0, fake, 1.0, fake, fake, None) == -1
    assert lib.mist_eval_reduce_exhaustive(pp, fake, 1, fake, 1, fake, -1.0, fake, fake, None) == -1
    assert lib.mist_eval_reduce_exhaustive(pp, fake, 1, fake, 1, None, 1.0, fake, fake, None) == -1
    ratios = np.array([0.5, 1.0, -2.0])
    slots = np.arange(3, dtype=np.int32)
    rp, sp_ = ctypes.c_void_p(ratios.ctypes.data), ctypes.c_void_p(slots.ctypes.data)
    some_tables = _lib.OutTables()
    samples = lambda n, r=rp, batch=1: lib.mist_eval_reduce_samples(
        pp, fake, 1, fake, 1, None, 0, fake, fake, r, sp_, n, batch, fake, fake, ctypes.byref(some_tables), None)
    assert samples(0) == -1 and samples(_lib.MAX_SAMPLE_BATCH + 1) == -1 and samples(2, None) == -1
    assert samples(3) == -1 and b"ratio 2" in lib.mist_last_error()
    assert samples(2, batch=0) == -1 and samples(2, batch=3) == -1 and b"main_batch" in lib.mist_last_error()
    tabs = _lib.OutTables()
    assert lib.mist_finalize(pp, fake, 1, fake, fake, fake, fake, 0, ctypes.byref(tabs), None) == -1
    shape = np.zeros(1, dtype=_lib.DP_SHAPE_DTYPE)
    assert lib.mist_dp_scratch_floats(ctypes.c_void_p(shape.ctypes.data), 4) == -1
    shape["num_layers"], shape["num_devices"], shape["num_mesh"], shape["p_dim"] = 8, 8, 2, 4
    shape["max_stages"] = 4
    shape["mesh_n"][0, :2], shape["mesh_m"][0, :2] = [1, 1], [1, 2]
    assert lib.mist_dp_scratch_floats(ctypes.c_void_p(shape.ctypes.data), 4) == 4 * 4 * 9 * 9 + 6 * 4 * 9
    shape["num_layers"], shape["num_devices"] = 80, 256
    assert lib.mist_dp_scratch_floats(ctypes.c_void_p(shape.ctypes.data), 4) == 4 * 4 * 81 * 257 + 6 * 4 * 257
    costs = _lib.DpCosts(4096, 4096, 4096, 4096, 4096, 4096, 4096, 4096)
    sp = ctypes.c_void_p(shape.ctypes.data)
    assert lib.mist_dp_run(sp, ctypes.byref(costs), fake, fake, 1, 0, fake, fake, fake, None, None, None) == -1
    assert b"scratch" in lib.mist_last_error()
    assert lib.mist_dp_run(sp, ctypes.byref(costs), fake, fake, 70000, 0, fake, fake, fake, None, fake, None) == -1
    assert lib.mist_dp_run(sp, ctypes.byref(costs), fake, fake, 1, 7, fake, fake, fake, None, fake, None) == -1
    # the variant with the built-in scratch refuses batches beyond that scratch (80 x 256 planes:
    # 84 810 floats per instance) and the same bad arguments, all before any GPU call
    limit = lib.mist_dp_static_scratch_floats()
    assert limit == 4 << 20
    assert lib.mist_dp_scratch_floats(sp, 50) > limit >= lib.mist_dp_scratch_floats(sp, 49)
    assert lib.mist_dp_run_static(sp, ctypes.byref(costs), fake, fake, 50, 0, fake, fake, fake, None, None) == -1
    assert b"built-in scratch" in lib.mist_last_error()
    assert lib.mist_dp_run_static(sp, ctypes.byref(costs), fake, fake, 1, 7, fake, fake, fake, None, None) == -1
    assert lib.mist_dp_run_static(sp, ctypes.byref(costs), None, fake, 1, 0, fake, fake, fake, None, None) == -1
    assert lib.mist_dp_backtrack(sp, None, fake, 1, fake, None) == -1
    assert lib.mist_dp_backtrack(sp, fake, fake, 0, fake, None) == -1
    # the search driver checks its arguments before it touches the GPU
    shape_ok = np.zeros(1, dtype=_lib.DP_SHAPE_DTYPE)
    shape_ok["num_layers"], shape_ok["num_devices"], shape_ok["num_mesh"], shape_ok["p_dim"] = 8, 8, 2, 4
    shape_ok["max_stages"] = 4
    shape_ok["mesh_n"][0, :2], shape_ok["mesh_m"][0, :2] = [1, 1], [1, 2]
    so = ctypes.c_void_p(shape_ok.ctypes.data)
    one = np.ones(1, dtype=np.int32)
    op = ctypes.c_void_p(one.ctypes.data)
    search = lambda shape_ptr, n_inst, n_g, G: lib.mist_inter_stage_search(
        shape_ptr, ctypes.byref(costs), n_inst, n_g, op, G, 0, fake, fake, fake, fake, fake, None, None)
    assert search(so, 0, 1, op) == -1
    assert search(so, 1, 1, ctypes.c_void_p(np.zeros(1, dtype=np.int32).ctypes.data)) == -1
    assert b"grad_accum" in lib.mist_last_error()
    assert search(None, 1, 1, op) == -1
    free = shape_ok.copy()
    free["free_devices"], free["num_devices"], free["num_mesh"] = 1, 0, 1
    assert search(ctypes.c_void_p(free.ctypes.data), 1, 1, op) == -1
    assert b"per-mesh" in lib.mist_last_error()
    # the search over tables with a limit needs the estimate, a factor and the counter
    host_estimate, unresolved = np.full(1, np.inf), np.zeros(1, dtype=np.int32)
    bounded = lambda est, factor, out: lib.mist_inter_stage_search_bounded(
        1, so, ctypes.byref(costs), ctypes.byref(costs), None, 1, 1, op, op, 0, fake, fake, fake, fake,
        fake, fake, None, None, None, est, factor, out)
    assert bounded(None, 1.25, hp(unresolved)) == -1 and bounded(hp(host_estimate), 1.25, None) == -1
    assert bounded(hp(host_estimate), 0.0, hp(unresolved)) == -1 and b"limit_factor" in lib.mist_last_error()
    # the first stage-cost estimate: workspace pointers, an incumbent to lower, a ratio
    estimate = lambda problem, prefix=fake, ratio=1.0: lib.mist_stage_cost_first_estimate(
        problem, fake, 1, prefix, 4, fake, ratio, fake, None)
    assert estimate(pp) == -1 and b"incumbent" in lib.mist_last_error()
    with_incumbent = prob.copy()
    with_incumbent["stage_cost_incumbent"], with_incumbent["incumbent_num_devices"] = 4096, 8
    wp = ctypes.c_void_p(with_incumbent.ctypes.data)
    assert estimate(wp, None) == -1 and estimate(wp, fake, -1.0) == -1 and b"ratio" in lib.mist_last_error()
    assert estimate(None) == -1
    # re-laid row minima: max_stages * Q * L (L + 1) / 2 floats per g
    assert lib.mist_dp_stage_minima_floats(sp) == 4 * 2 * (80 * 81 // 2)
    assert lib.mist_dp_stage_minima_floats(ctypes.c_void_p(np.zeros(1, dtype=_lib.DP_SHAPE_DTYPE).ctypes.data)) == -1
    assert lib.mist_dp_stage_minima(sp, ctypes.byref(costs), 1, None, None) == -1
    assert lib.mist_dp_stage_minima(sp, ctypes.byref(costs), 0, fake, None) == -1
    assert lib.mist_dp_stage_minima(sp, ctypes.byref(_lib.DpCosts()), 1, fake, None) == -1
    # batched stage sampling: the problem list must be consistent before anything is launched
    items = (_lib.MipBatchItem * 2)()
    for it in items:
        it.shape = _lib.MipShape(num_layers=8, p_dim=4, sample_size=4, num_stages=2, layers_min=3,
                                 layers_max=5, ckpt_mode=_lib.MIP_CKPT_TUNED, fixed_ckpt=0)
        for v in range(4):
            it.tables.stable[v] = it.tables.delta[v] = 4096
    items[1].first_block, items[1].out_offset = 6, 24
    batch = lambda n: lib.mist_mip_stage_samples_batch(ctypes.byref(items), fake, n, fake, fake, fake, fake, fake, None)
    items[1].out_offset = 23
    assert batch(2) == -1 and b"continue the list" in lib.mist_last_error()
    items[1].out_offset = 24
    items[1].tables.delta[2] = None
    assert batch(2) == -1 and b"null table" in lib.mist_last_error()
    assert batch(0) == -1
    # the chains of assignment problems, the pre-fill of the cells an assignment reads, the
    # all-samples entry point and the plan builder check their arguments the same way
    items[1].tables.delta[2] = 4096
    G_of = np.array([4, 0], dtype=np.int32)
    out_f, out_i = np.zeros(16), np.zeros(16, dtype=np.int32)
    hp = lambda a: ctypes.c_void_p(a.ctypes.data)
    chains = lambda per_chain, n_chains, G=G_of: lib.mist_mip_solve_chains(
        ctypes.byref(items), hp(G), per_chain, n_chains, fake, fake, fake, hp(out_f), hp(out_i), hp(out_i), hp(out_i))
    assert chains(0, 1) == -1 and chains(2, 0) == -1
    assert chains(2, 1) == -1 and b"grad_accum" in lib.mist_last_error()
    assert lib.mist_mip_solve_chains(ctypes.byref(items), hp(G_of), 1, 1, None, fake, fake, hp(out_f),
                                     hp(out_i), hp(out_i), hp(out_i)) == -1
    regions = np.array([[0, 0, 2, 4, 3, 0], [1, 1, 1, 8, 2, 21]], dtype=np.int32)
    prefill = lambda r, n=2, L=8: lib.mist_mip_prefill_cells(L, 4, 3, 2, 2, hp(r), fake, n, ctypes.byref(some_tables), None)
    assert prefill(regions) == -1 and b"null table" in lib.mist_last_error()
    for v in range(4):
        some_tables.stable[v] = some_tables.delta[v] = some_tables.index[v] = 4096
    bad = regions.copy()
    bad[1, 5] = 20
    assert prefill(bad) == -1 and b"does not continue" in lib.mist_last_error()
    bad = regions.copy()
    bad[0, 1] = 2
    assert prefill(bad) == -1 and b"outside the tables" in lib.mist_last_error()
    bad = regions.copy()
    bad[1, 3] = 9
    assert prefill(bad) == -1 and b"layer counts" in lib.mist_last_error()
    assert prefill(regions, n=0) == -1
    all_samples = lambda n, sample_batch, main_batch, r=rp: lib.mist_intra_stage_eval_samples(
        pp, fake, 1, fake, 1, fake, 1, None, 0, fake, fake, fake, fake, fake, r, sp_, n, sample_batch,
        main_batch, ctypes.byref(some_tables), None)
    assert all_samples(0, 1, 1) == -1 and all_samples(2, 0, 1) == -1
    assert all_samples(2, _lib.MAX_SAMPLE_BATCH + 1, 1) == -1 and b"sample_batch" in lib.mist_last_error()
    assert all_samples(2, 2, 3) == -1 and b"main_batch" in lib.mist_last_error()
    assert all_samples(2, 2, 1, None) == -1
    request, result = _lib.PlanRequest(), _lib.PlanResult()
    groups = np.zeros(4, dtype=_lib.GROUP_DTYPE)
    words = np.zeros(64, dtype=np.int64)
    plan = lambda req, capacity: lib.mist_plan_groups(
        req, hp(groups), capacity, hp(words), hp(words), hp(words), hp(words), hp(words), hp(words),
        hp(words), ctypes.byref(result))
    assert plan(None, 4) == -1 and b"null" in lib.mist_last_error()
    assert plan(ctypes.byref(request), 4) == _lib.PLAN_UNSUPPORTED and b"list lengths" in lib.mist_last_error()


def test_window_begin_matches_numpy_formulation():
    """mist_dp_window_begin against the rule written with numpy: a candidate is certain to be
    kept if its predecessor is at least the gap below; start at the last certain candidate that
    is <= start_value, else at the first one if it is certain and above start_value."""
    lib = _lib.load()
    rng = np.random.default_rng(7)
    gap = 1e-6
    outcomes = set()
    for trial in range(400):
        n = int(rng.integers(0, 40))
        base = np.sort(rng.uniform(0.5, 0.5002, n)).astype(np.float32)
        if n and rng.random() < 0.5:   # clusters closer than the gap
            base = np.sort(np.concatenate([base, base[: n // 2] + np.float32(3e-7)])).astype(np.float32)
        values = np.unique(base)
        below = bool(rng.random() < 0.3)
        lo = np.float32(-np.inf) if below else np.float32(0.5 - rng.uniform(0, 2e-6))
        values = values[values > lo] if not below else values
        if len(values) and not below and rng.random() < 0.4:   # the fetch starts inside a cluster
            lo = np.float32(values[0] - np.float32(2e-7))
            values = values[: 1 + int(np.searchsorted(values, values[0] + np.float32(8e-7)))]
        start = np.float32(rng.uniform(0.4999, 0.5003))
        kept = np.empty(max(len(values), 1), dtype=np.float32)
        got = lib.mist_dp_window_begin(
            values.ctypes.data, len(values), 0.0 if below else float(lo), int(below), float(start), gap,
            kept.ctypes.data)
        if len(values) == 0:
            assert got == 0
            continue
        prev = np.concatenate(([np.float32(0) if below else lo], values[:-1])).astype(np.float32)
        certain = ~((values - prev).astype(np.float64) < gap)
        certain[0] = certain[0] or below
        cand = np.nonzero(certain & (values <= start))[0]
        if len(cand):
            first = int(cand[-1])
        elif values[0] > start and certain[0]:
            first = 0
        else:
            assert got == _lib.DP_NO_START
            outcomes.add("none")
            continue
        want = np.empty_like(values)
        n_want = lib.mist_dp_filter_tmax(values[first:].copy().ctypes.data, len(values) - first, gap, want.ctypes.data)
        assert got == n_want and np.array_equal(kept[:got], want[:n_want]), trial
        outcomes.add("mid" if first else "first")
    assert outcomes == {"none", "mid", "first"}


def test_gap_filter_matches_oracle_rule():
    lib = _lib.load()
    rng = np.random.default_rng(0)
    t = np.unique(np.concatenate([rng.uniform(0.01, 2, 500), 0.5 + np.arange(40) * 3e-7]).astype(np.float32))
    out = np.empty_like(t)
    n = lib.mist_dp_filter_tmax(ctypes.c_void_p(t.ctypes.data), len(t), 1e-6, ctypes.c_void_p(out.ctypes.data))
    want, last = [], np.float32(0)
    for v in t:
        if float(np.float32(v - last)) < 1e-6:
            continue
        want.append(v)
        last = v
    assert n == len(want) and np.array_equal(out[:n], np.array(want, dtype=np.float32))
    assert 0 < n < len(t)


class _FakeRunner:
    """Host stand-in of the DP runner's candidate store for one table row."""

    def __init__(self, values):
        from mist_amd import _lib

        self.values = np.sort(np.asarray(values, dtype=np.float32))
        self.lib = _lib.load()
        self.fetches = 0

    def candidates_between(self, rows, lo, hi):
        self.fetches += 1
        out = []
        for l, h in zip(lo, hi):
            v = self.values
            out.append((v[(v > l) & (v <= h)], int((v > h).sum())))
        return out

    def filter_gap(self, ascending):
        from mist_amd.inter_tuning import _DpRunner

        return _DpRunner.filter_gap(self, ascending)


@pytest.mark.parametrize("seed", range(12))
def test_threshold_window_equals_full_walk(seed):
    """The lazily materialised window of kept t_max candidates must equal the reference's walk
    over the complete sorted list (inter_tuning.py:180-198) from the smallest feasible
    threshold on, whatever the spacing of the candidates below it."""
    from mist_amd.inter_tuning import GAP, _Window

    rng = np.random.default_rng(seed)
    centres = rng.uniform(0.05, 40.0, size=300)
    dense = (centres[:, None] + rng.uniform(0, 3e-6, size=(300, 6)) * rng.integers(0, 2, size=(300, 1))).ravel()
    values = np.unique(np.concatenate([dense, rng.uniform(0.05, 40.0, size=500)]).astype(np.float32))
    runner = _FakeRunner(values)
    full = runner.filter_gap(values)
    # reference walk written out: keep t unless t - last < gap (float32 difference)
    last, want_full = None, []
    for t in values:
        if last is not None and np.float64(np.float32(t) - np.float32(last)) < GAP:
            continue
        want_full.append(t)
        last = t
    assert np.array_equal(full, np.array(want_full, dtype=np.float32))

    for trial in range(20):
        start = values[rng.integers(len(values))] if trial % 2 else np.float32(rng.uniform(0.0, 41.0))
        G = int(rng.choice([1, 2, 8, 64]))
        w = _Window(runner, 0, G, start, start_sum=float(start) * 2)
        widen = 0
        while True:
            lo = w.lower_margin(widen) if widen < 8 else np.float32(-np.inf)
            hi = np.float32(start + rng.uniform(0, 0.5))
            (vals, above), = runner.candidates_between([0], [lo], [hi])
            if w.begin(vals, above, lo, hi):
                break
            widen += 1
        while not w.complete:
            w.extend(float("inf"))
        want = full[full >= start]
        got = w.kept[np.searchsorted(w.kept, start, side="left"):]
        assert np.array_equal(got, want), (seed, trial)


def test_window_begin_many_equals_single_begins():
    """One library call for the first fetch of many windows gives what the per-window call gives
    (kept values, fetched range, completeness, and which windows must fetch from further below)."""
    from mist_amd.inter_tuning import _Window

    rng = np.random.default_rng(11)
    centres = rng.uniform(0.05, 40.0, size=200)
    dense = (centres[:, None] + rng.uniform(0, 3e-6, size=(200, 6)) * rng.integers(0, 2, size=(200, 1))).ravel()
    values = np.unique(np.concatenate([dense, rng.uniform(0.05, 40.0, size=300)]).astype(np.float32))
    runner = _FakeRunner(values)
    outcomes = set()
    for widen in (0, 3, 8):
        starts = [values[rng.integers(len(values))] if k % 2 else np.float32(rng.uniform(0.0, 41.0)) for k in range(24)]
        single = [_Window(runner, 0, 4, s, start_sum=float(s)) for s in starts]
        many = [_Window(runner, 0, 4, s, start_sum=float(s)) for s in starts]
        lo = np.array([w.lower_margin(widen) if widen < 8 else -np.inf for w in single], dtype=np.float32)
        hi = np.array([s + rng.uniform(0, 0.3) for s in starts], dtype=np.float32)
        hi[::5] = np.float32(41.0)   # nothing above
        lo[1::7] = hi[1::7]          # empty fetch
        for k in range(2, len(starts), 3):  # fetch that begins inside a run of near-equal values
            inside = np.float32(dense[rng.integers(len(dense))])
            single[k].start_value = many[k].start_value = inside
            lo[k], hi[k] = inside - np.float32(4e-7), inside + np.float32(0.1)
        got = runner.candidates_between(np.zeros(len(starts)), lo, hi)
        want_ok = [w.begin(v, a, l, h) for w, (v, a), l, h in zip(single, got, lo, hi)]
        flat = np.concatenate([v for v, _ in got]) if got else np.empty(0, dtype=np.float32)
        bounds = np.concatenate([[0], np.cumsum([len(v) for v, _ in got])]).astype(np.int64)
        above = np.array([a for _, a in got], dtype=np.int32)
        ok = _Window.begin_many(many, flat, bounds, above, lo, hi)
        assert ok == want_ok
        outcomes.update(ok)
        for a, b in zip(single, many):
            assert np.array_equal(a.kept, b.kept) and a.hi == b.hi and a.complete == b.complete
            assert a.bound == b.bound or (np.isinf(a.bound) and np.isinf(b.bound))
    assert outcomes == {True, False}
    assert _Window.begin_many([], np.empty(0, dtype=np.float32), np.zeros(1, dtype=np.int64),
                              np.empty(0, dtype=np.int32), np.empty(0), np.empty(0)) == []


def test_inputs_outside_the_kernels_preconditions_are_rejected():
    """Negative or non-finite table values / hardware parameters would break the monotonicity
    the reduce kernel's exact pruning relies on: the host refuses them before any launch."""
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.stage_inputs import make_problem

    cfg, tables = tiny_plan(1, layers=4)
    with pytest.raises(ValueError, match="interference factors"):
        make_problem(load_plan(1, hardware__interference_model_params=[0.0] * 28)[0], 4, 2, 1, 1, 1)
    bad = list(cfg.hardware.gpu_gpu_comm_params)
    bad[0] = -1.0
    with pytest.raises(ValueError, match="bandwidths"):
        make_problem(load_plan(1, hardware__gpu_gpu_comm_params=bad)[0], 4, 2, 1, 1, 1)

    class NegativeTables(type(tables)):
        def mem_output(self, kind, b, tp):
            return -super().mem_output(kind, b, tp)

    broken = NegativeTables(cfg)
    tuner = IntraStageTuner(broken, 4, [(1, 1), (1, 2)], [1, 2, 4, 8], 1, cfg, sample_size=1)
    with pytest.raises(ValueError, match="non-negative"):
        tuner.prepare()
