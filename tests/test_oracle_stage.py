"""Pins the oracle's per-stage model (oracle/stage.py, oracle/intra.py, oracle/pareto.py):
an independent scalar re-derivation per cell, algebraic invariants, the documented never-written
cells, and the library routine the reduction reduces to."""
import numpy as np
import pytest

from oracle.intra import intra_stage_tune, max_pre_saved_micro_batches
from oracle.pareto import alpha_ratios, compute_indices, compute_indices_scan
from oracle.stage import batched_tune_best_latency_for_stage
from tests.scalar_model import evaluate_cell
from tests.util import tiny_plan

GB_OVER_MB = 1024.0
VARIANTS = ("base", "with_pre", "with_post", "no_pp")


def _run(cfg, tables, n, m, G, tp, L, P, S=1):
    dbg = {}
    res = batched_tune_best_latency_for_stage(
        tables, cfg, list(range(P)), list(range(1, L + 1)), list(range(L + 1)), n, m, G,
        tp_size=tp, sample_size=S, debug=dbg)
    return res, dbg


CASES = [
    # (overrides, n, m, G, tp)
    (dict(hardware__memory_capacity=6.0), 1, 2, 2, 1),
    (dict(hardware__memory_capacity=4.0, model__use_flash_attn=True), 1, 2, 1, 1),
    (dict(hardware__memory_capacity=8.0, hardware__num_nodes=2, hardware__num_gpus_per_node=4,
          training__global_batch_size=32, tuning__pre_post_strategy="intra-node-tp-with-ore"), 2, 4, 4, 2),
    (dict(hardware__memory_capacity=5.0, hardware__num_nodes=2, hardware__num_gpus_per_node=4,
          training__global_batch_size=32, tuning__pre_post_strategy="intra-node-tp-without-ore",
          enable_advanced_opt_in_first_block=False), 1, 4, 8, 1),
]


@pytest.mark.parametrize("overrides,n,m,G,tp", CASES)
def test_cells_match_scalar_rederivation(overrides, n, m, G, tp):
    L, P = 5, 3
    # a reduced offload grid keeps the scalar model affordable: 3 values per ratio
    ov = dict(tuning__search_space=dict(
        batch_size_candidates=[1, 2, 4, 8], offloading_ratio_candidates=[0.0, 0.5, 1.0],
        sparse_offloading_ratio_candidates=[0.0, 0.5, 1.0],
        zero_flag_choices=[[0, 0, 0], [0, 0, 1], [0, 1, 1], [1, 1, 1]]))
    ov.update(overrides)
    cfg, tables = tiny_plan(1, layers=L, **ov)
    p_cands = min(G, L, P)
    res, dbg = _run(cfg, tables, n, m, G, tp, L, p_cands)
    rows = dbg["rows"]
    assert rows.shape[0] > 0
    cap = cfg.hardware.memory_capacity * GB_OVER_MB
    rng = np.random.default_rng(n * 100 + m * 10 + G)
    cells = [(l, c, p) for l in range(1, L + 1) for c in range(l + 1) for p in range(p_cands)]
    chosen = [cells[i] for i in rng.choice(len(cells), size=min(14, len(cells)), replace=False)]
    checked = 0
    for l, c, p in chosen:
        model = [evaluate_cell(cfg, tables, n, m, G, rows[r], l, c, p, L) for r in range(rows.shape[0])]
        for v, name in enumerate(VARIANTS):
            if name in ("with_post", "no_pp") and p != 0:
                continue
            if name == "no_pp" and l != L:
                continue
            stable_t, delta_t, _, idx_t = res[v]
            if name == "no_pp":
                got = stable_t[c, 0], delta_t[c, 0], idx_t[c, 0]
                written = c != L - 1
            elif name == "with_post":
                got = stable_t[l - 1, c, 0], delta_t[l - 1, c, 0], idx_t[l - 1, c, 0]
                written = c != l - 1
            else:
                got = stable_t[p, l - 1, c, 0], delta_t[p, l - 1, c, 0], idx_t[p, l - 1, c, 0]
                written = not (p >= 1 and c == l - 1)
            if not written:
                assert got[2] == -1 and np.isinf(got[0]) and np.isinf(got[1])
                continue
            obj = np.array([mm[name][0] + mm[name][1] / G for mm in model])
            peak = np.array([max(mm[name][2], mm[name][3]) * mm[name][4] for mm in model])
            inside = peak <= cap * (1 - 1e-9)
            outside = peak > cap * (1 + 1e-9)
            if got[2] == -1:
                assert not inside.any(), (name, l, c, p)
                continue
            r = int(got[2])
            assert not outside[r], f"{name} {(l, c, p)}: chosen row {r} is infeasible in the scalar model"
            # the chosen row's stored costs are the model's (float32 rounding of the middle-stage pair)
            assert got[0] == pytest.approx(model[r][name][0], rel=2e-7, abs=1e-12)
            assert got[1] == pytest.approx(model[r][name][1], rel=2e-7, abs=2e-9)
            # and no clearly feasible row is clearly better; earlier rows win exact ties
            if inside.any():
                best = obj[inside].min()
                assert obj[r] <= best * (1 + 5e-7) + 1e-12, (name, l, c, p)
            checked += 1
    assert checked >= 10


def test_latency_families_match_scalar_to_1e12():
    """float64 layer / first / last families of the oracle against the scalar model."""
    L = 4
    cfg, tables = tiny_plan(1, layers=L, hardware__memory_capacity=24.0)
    for G in (1, 4):
        res, dbg = _run(cfg, tables, 1, 2, G, 1, L, 1)
        rows, lat = dbg["rows"], dbg["lat"]
        for r in np.random.default_rng(G).choice(rows.shape[0], 40, replace=False):
            for l, c in [(1, 0), (1, 1), (2, 1), (4, 0), (4, 2), (4, 4), (3, 3)]:
                lm2 = max(l - 2, 0)
                n_ck = min(max(c - 1, 0), lm2)
                pick = lambda key, ck: np.broadcast_to(lat["ck" if ck else "nock"][key], (rows.shape[0],))[r]
                stable = (n_ck * pick("s_layer", True) + (lm2 - n_ck) * pick("s_layer", False)
                          + pick("s_first", c == l) + pick("s_last", c != 0))
                delta = (n_ck * pick("d_layer", True) + (lm2 - n_ck) * pick("d_layer", False)
                         + pick("d_first", c == l) + pick("d_last", c != 0))
                want = evaluate_cell(cfg, tables, 1, 2, G, rows[r], l, c, 0, L)["base"]
                assert stable == pytest.approx(want[0], rel=1e-12)
                assert delta == pytest.approx(want[1], rel=1e-9, abs=1e-15)
                if G == 1:
                    assert delta == 0


def test_unwritten_cells_and_shapes():
    L, P = 6, 3
    cfg, tables = tiny_plan(1, layers=L, hardware__memory_capacity=24.0)
    res, _ = _run(cfg, tables, 1, 2, 4, 1, L, P)
    base, pre, post, nopp = res
    assert base[0].shape == (P, L, L + 1, 1) and post[0].shape == (L, L + 1, 1) and nopp[0].shape == (L + 1, 1)
    for l in range(1, L + 1):
        for c in range(L + 1):
            for p in range(P):
                unwritten = c > l or (p >= 1 and c == l - 1)
                for t in (base, pre):
                    assert (t[3][p, l - 1, c, 0] == -1) == unwritten
                    if unwritten:
                        assert t[3][p, l - 1, c, 0] == -1 and np.isinf(t[0][p, l - 1, c, 0])
                    else:
                        assert t[3][p, l - 1, c, 0] >= 0  # 24 GB: always something feasible
            unwritten = c > l or c == l - 1
            assert (post[3][l - 1, c, 0] == -1) == unwritten
    for c in range(L + 1):
        assert (nopp[3][c, 0] == -1) == (c == L - 1)


def test_costs_nondecreasing_in_pre_saved_micro_batches_and_tighter_memory():
    """More resident micro-batches or less memory can only shrink the feasible set."""
    L, P = 5, 4
    out = {}
    for cap in (24.0, 5.0, 3.0):
        cfg, tables = tiny_plan(1, layers=L, hardware__memory_capacity=cap, training__global_batch_size=16)
        res, _ = _run(cfg, tables, 1, 2, 4, 1, L, P)
        out[cap] = res
        for v in (0, 1):
            stable, delta = res[v][0][..., 0], res[v][1][..., 0]
            obj = stable + delta / 4
            for p in range(1, P):
                a, b = obj[p - 1], obj[p]
                both = np.isfinite(a) | np.isfinite(b)
                written = np.isfinite(b)  # p >= 1 leaves c == l - 1 unwritten
                assert np.all(b[written] >= a[written])
    for v in range(4):
        o24 = out[24.0][v][0][..., 0] + out[24.0][v][1][..., 0] / 4
        o5 = out[5.0][v][0][..., 0] + out[5.0][v][1][..., 0] / 4
        o3 = out[3.0][v][0][..., 0] + out[3.0][v][1][..., 0] / 4
        assert np.all(o5 >= o24) and np.all(o3 >= o5)
    assert np.isinf(out[3.0][0][0]).sum() > np.isinf(out[24.0][0][0]).sum()


def test_reduction_is_numpy_argmin_for_one_sample():
    rng = np.random.default_rng(3)
    x = rng.integers(0, 6, size=(7, 300)).astype(np.float32)  # many exact ties
    y = rng.integers(0, 6, size=(7, 300)).astype(np.float32)
    mask = rng.random((7, 300)) < 0.6
    mask[2] = False
    got = compute_indices(x, y, mask, alpha_ratios(1))[:, 0]
    assert alpha_ratios(1)[0] == 1.0
    cost = np.where(mask, x.astype(np.float64) + y, np.inf)
    want = np.where(mask.any(axis=1), np.argmin(cost, axis=1), -1)
    assert np.array_equal(got, want)
    assert got[2] == -1
    for S in (1, 3, 30):
        r = alpha_ratios(S)
        assert np.array_equal(compute_indices(x, y, mask, r), compute_indices_scan(x, y, mask, r))
        # the reference's own vectorised numpy form (penalty on y, argmin per alpha)
        ref = np.stack([np.argmin(rk * x.astype(np.float64) + (y + np.where(mask, 0, np.inf)), axis=-1) for rk in r], axis=1)
        live = mask.any(axis=1)
        assert np.array_equal(compute_indices(x, y, mask, r)[live], ref[live])


def test_intra_driver_packs_group_tables():
    L = 4
    cfg, tables = tiny_plan(1, layers=L, hardware__memory_capacity=6.0)
    meshes, Gs = [(1, 1), (1, 2)], [1, 2, 4, 8]
    out = intra_stage_tune(tables, cfg, L, meshes, Gs, 1, 1)
    P = max_pre_saved_micro_batches(meshes, Gs, L)
    assert out.costs_stable.shape == (4, 2, P + 1, L, L + 1, 1) and out.costs_stable.dtype == np.float32
    assert out.solutions.shape == (4, 2, P + 1, L, L + 1, 1, 10) and out.solutions.dtype == np.float64
    for g, G in enumerate(Gs):
        for q, (n, m) in enumerate(meshes):
            p_n = min(G, L, P + 1)
            res, _ = _run(cfg, tables, n, m, G, 1, L, p_n)
            assert np.array_equal(out.costs_stable[g, q, :p_n], res[0][0].astype(np.float32))
            assert np.all(np.isinf(out.costs_stable[g, q, p_n:]))
            assert np.array_equal(out.indices_with_post[g, q], res[2][3])
            assert np.array_equal(out.costs_delta_no_pp[g, q], res[3][1].astype(np.float32))
            finite = np.isfinite(out.costs_stable[g, q])
            assert np.array_equal(finite, out.indices[g, q] >= 0)
            assert np.all(np.isinf(out.solutions[g, q][~finite]))
