"""Pins candidate enumeration (oracle and the package's factored form) by closed forms."""
from itertools import product

import numpy as np
import pytest

from mist_amd.search_space import (
    _get_device_mesh_candidates,
    _get_grad_accumu_steps_candidates,
    create_search_space_for_a_block_layer,
)
from oracle.search_space import create_search_space, device_mesh_candidates, grad_accumu_steps_candidates
from tests.util import load_plan, tiny_plan


def test_mesh_and_grad_accum_lists():
    assert device_mesh_candidates(1, 2, False) == [(1, 1), (1, 2)]
    assert device_mesh_candidates(4, 8, False) == [(1, 1), (1, 2), (1, 4), (1, 8), (2, 8), (4, 8)]
    assert device_mesh_candidates(3, 4, True) == [(1, 1), (1, 2), (1, 4), (2, 4), (3, 4)]
    assert device_mesh_candidates(3, 4, False) == [(1, 1), (1, 2), (1, 4), (2, 4)]
    assert grad_accumu_steps_candidates(512) == [2**i for i in range(10)]
    assert grad_accumu_steps_candidates(1536) == [2**i for i in range(10)]
    assert grad_accumu_steps_candidates(32) == [1, 2, 4, 8, 16, 32]
    for n, m, c in [(1, 2, False), (4, 8, False), (32, 8, False), (3, 4, True)]:
        assert _get_device_mesh_candidates(n, m, c) == device_mesh_candidates(n, m, c)
    assert _get_grad_accumu_steps_candidates(2048) == grad_accumu_steps_candidates(2048)


@pytest.mark.parametrize("plan,n,m,G,tp", [(1, 1, 2, 2, 1), (1, 1, 2, 4, 2), (2, 2, 8, 16, 2), (2, 4, 8, 64, 4), (3, 8, 8, 32, 4)])
def test_row_count_order_and_factored_form(plan, n, m, G, tp):
    cfg, tables = load_plan(plan)
    B = cfg.training.global_batch_size
    rows = create_search_space(n, m, B, G, cfg, constraint_fn=tables.constraint, tp_size=tp)
    k = len(cfg.tuning.offloading_ratio_candidates)
    par = np.unique(rows[:, :6], axis=0).shape[0]
    assert rows.shape == (par * (k**4 - (k - 1) * k**2), 10)
    # offload block = itertools.product order without (wo > 0 and go == 0), repeated per parallelism row
    r = cfg.tuning.offloading_ratio_candidates
    off = np.array([t for t in product(r, r, r, r) if not (t[0] > 0 and t[1] == 0)])
    assert np.array_equal(rows[: len(off), 6:], off)
    assert np.array_equal(rows[len(off): 2 * len(off), 6:], off) or par == 1
    # invariants of every row: b * dp * G == B, dp * tp == n * m, tp fixed
    assert np.all(rows[:, 0] * rows[:, 1] * G == B)
    assert np.all(rows[:, 1] * rows[:, 2] == n * m)
    assert np.all(rows[:, 2] == tp)
    space = create_search_space_for_a_block_layer(n, m, B, G, cfg, constraint_fn=tables.constraint, tp_size=tp)
    assert space.n_rows == rows.shape[0]
    assert np.array_equal(space.materialize(), rows)
    pick = np.array([[0, -1], [rows.shape[0] - 1, rows.shape[0] // 2]])
    dec = space.decode(pick)
    assert np.all(np.isinf(dec[0, 1])) and np.array_equal(dec[1, 0], rows[-1])


def test_zero_flags_and_dp1_rule():
    cfg, tables = load_plan(1)
    rows = create_search_space(1, 2, 8, 8, cfg, tables.constraint, tp_size=2)  # dp == 1
    assert {tuple(r) for r in rows[:, 3:6]} == {(0.0, 0.0, 1.0)}
    rows = create_search_space(1, 2, 8, 1, cfg, tables.constraint, tp_size=1)  # dp == 2
    assert {tuple(r) for r in rows[:, 3:6]} == {(0.0, 0.0, 0.0), (0.0, 0.0, 1.0), (0.0, 1.0, 1.0), (1.0, 1.0, 1.0)}
    cfg2, t2 = load_plan(1, tuning__zero_2_and_3_enabled=False)
    rows = create_search_space(1, 2, 8, 1, cfg2, t2.constraint, tp_size=1)
    assert {tuple(r) for r in rows[:, 3:6]} == {(0.0, 0.0, 1.0)}


def test_tp_latch_and_disable_flags():
    cfg, tables = load_plan(1)
    # tp_size=None latches to the tp of the first feasible micro-batch size
    rows = create_search_space(1, 2, 8, 2, cfg, tables.constraint, tp_size=None)
    assert len(np.unique(rows[:, 2])) == 1
    cfg2, t2 = load_plan(1, disable_tp_tuning=True)
    assert create_search_space(1, 2, 8, 8, cfg2, t2.constraint, tp_size=2).shape[0] == 0
    cfg3, t3 = load_plan(1, tuning__state_offloading_enabled=False, tuning__activation_offloading_enabled=False)
    rows = create_search_space(1, 2, 8, 2, cfg3, t3.constraint, tp_size=1)
    assert np.all(rows[:, 6:] == 0)
    cfg4, t4 = load_plan(1, fixed_oo_ratio=0.5, disable_wo_tuning=True)
    rows = create_search_space(1, 2, 8, 2, cfg4, t4.constraint, tp_size=1)
    assert np.all(rows[:, 8] == 0.5) and np.all(rows[:, 6] == 0)
    s = create_search_space_for_a_block_layer(1, 2, 8, 2, cfg4, t4.constraint, tp_size=1)
    assert np.array_equal(s.materialize(), rows)


def test_published_sizes_of_the_plans():
    """Row totals of the GPT-1.3B and GPT-7B plans: 1.05e4 rows / 1.06e8 candidates."""
    for plan, want_rows in [(1, 10500), (2, 3223440)]:
        cfg, tables = load_plan(plan)
        hw = cfg.hardware
        meshes = device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
        Gs = grad_accumu_steps_candidates(cfg.training.global_batch_size)
        total = 0
        for tp in [t for t in (1, 2, 4, 8) if t <= hw.num_gpus_per_node]:
            for G in Gs:
                for n, m in meshes:
                    total += create_search_space_for_a_block_layer(
                        n, m, cfg.training.global_batch_size, G, cfg, tables.constraint, tp).n_rows
        assert total == want_rows
    assert 3223440 * 33 == 106373520
