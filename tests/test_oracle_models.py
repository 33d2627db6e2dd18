"""Pins the oracle's communication and interference models without the reference: closed forms,
special cases, invariants and an independent scalar re-derivation."""
import numpy as np
import pytest

from oracle.comm import cpu_gpu_comm_latency, gpu_gpu_comm_latency
from oracle.interference import interference_one_group, mask_factor_table
from tests.scalar_model import alpha_beta, overlap_time
from tests.util import load_plan

RNG = np.random.default_rng(7)
GG = list(RNG.uniform(10, 400, 16).repeat(2))
for i in range(16):
    GG[2 * i + 1] = float(RNG.uniform(5e-6, 5e-5))


def test_alpha_beta_closed_form_and_special_cases():
    gb = np.array([0.0, 5e-6, 0.5, 2.0, 7.5])
    for inter, intra in [(1, 1), (1, 2), (2, 4), (4, 8), (8, 8), (16, 8)]:
        got = gpu_gpu_comm_latency("all_gather", gb, intra_size=intra, inter_size=inter, gpu_gpu_comm_params=GG)
        n = inter * intra
        oi, ii = min(int(np.log2(inter)), 3), min(int(np.log2(intra)), 3)
        k, b = GG[(oi * 4 + ii) * 2], GG[(oi * 4 + ii) * 2 + 1]
        want = np.where((gb < 1e-5) | (n == 1), 0.0, gb / k * (n - 1) / n + b)
        assert np.array_equal(got, want)
        for x, w in zip(gb, want):
            assert alpha_beta(x, inter, intra, GG, 1.0) == pytest.approx(w, rel=1e-15, abs=0)
        ar = gpu_gpu_comm_latency("all_reduce", gb, intra, inter, GG)
        rs = gpu_gpu_comm_latency("reduce_scatter", gb, intra, inter, GG)
        assert np.array_equal(ar, got * 2.1) and np.array_equal(rs, got * 1.1)
        assert np.all(gpu_gpu_comm_latency("none", gb, intra, inter, GG) == 0)
    # n == 1 and tiny messages cost nothing, whatever the table says
    assert np.all(gpu_gpu_comm_latency("all_reduce", gb, 1, 1, GG) == 0)


def test_alpha_beta_rejects_unknown_sizes_and_ops():
    with pytest.raises(ValueError):
        gpu_gpu_comm_latency("all_gather", np.array([1.0]), intra_size=3, inter_size=1, gpu_gpu_comm_params=GG)
    with pytest.raises(ValueError):
        gpu_gpu_comm_latency("broadcast", np.array([1.0]), 2, 1, GG)
    with pytest.raises(ValueError):
        gpu_gpu_comm_latency("all_gather", np.array([1.0]), 2, 1, GG[:30])


def test_p2p_uses_the_two_documented_cells():
    gb = np.array([1.0, 3.0])
    assert np.array_equal(gpu_gpu_comm_latency("p2p", gb, None, 1, GG), gb / GG[(1 * 4 + 0) * 2])
    assert np.array_equal(gpu_gpu_comm_latency("p2p", gb, 1, None, GG), gb / GG[(0 * 4 + 1) * 2])


def test_host_link_closed_form():
    gb = np.array([0.0, 1e-9, 0.25, 4.0])
    got = cpu_gpu_comm_latency(gb, (20.0, 1e-5))
    assert np.array_equal(got, np.where(gb == 0, 0.0, gb / 20.0 + 1e-5))


def _random_inputs(n, zero_frac=0.35):
    x = RNG.uniform(1e-4, 2.0, size=(n, 4))
    x[RNG.random((n, 4)) < zero_frac] = 0.0
    return x


def test_interference_single_resource_is_identity():
    p = RNG.uniform(1, 3, 28)
    for j in range(4):
        x = np.zeros((50, 4))
        x[:, j] = RNG.uniform(1e-3, 5, 50)
        assert np.array_equal(interference_one_group(*x.T, p), x[:, j])


def test_interference_unit_factors_give_max():
    x = _random_inputs(2000)
    # peeling re-adds what it subtracted: equal to max up to a few roundings
    np.testing.assert_allclose(interference_one_group(*x.T, np.ones(28)), x.max(axis=1), rtol=1e-15, atol=0)


def test_interference_at_least_max_when_factors_ge_one():
    x = _random_inputs(2000)
    out = interference_one_group(*x.T, RNG.uniform(1, 3, 28))
    assert np.all(out >= x.max(axis=1) * (1 - 1e-15))


def test_interference_worked_example():
    p = np.ones(28)
    p[16:18] = 50.0  # compute + gpu<->gpu pair
    assert interference_one_group(1.0, 100.0, 0.0, 0.0, p)[0] == 149.0


def test_interference_homogeneous():
    x = _random_inputs(500, zero_frac=0.3) + 0.0
    x[x != 0] += 1e-3  # stay clear of the 1e-8 threshold under scaling
    p = RNG.uniform(1, 3, 28)
    a = interference_one_group(*x.T, p)
    b = interference_one_group(*(x * 8.0).T, p)  # power of two: exact scaling
    assert np.array_equal(b, a * 8.0)


def test_interference_matches_scalar_drain_simulation():
    p = RNG.uniform(1, 3, 28)
    x = _random_inputs(3000)
    got = interference_one_group(*x.T, p)
    want = np.array([overlap_time(*row, p) for row in x])
    np.testing.assert_allclose(got, want, rtol=1e-13, atol=0)


def test_mask_table_order_and_slices():
    p = np.arange(1.0, 29.0)
    table = mask_factor_table(p)
    assert len(table) == 11
    assert [int(m.sum()) for m, _ in table] == [4, 3, 3, 3, 3, 2, 2, 2, 2, 2, 2]
    used = np.concatenate([f[m] for m, f in table])
    assert np.array_equal(used, p)  # every parameter is consumed once, in order
    for m, f in table:
        assert np.all(f[~m] == 1.0)


def test_real_plan_parameters_have_expected_shapes():
    cfg, _ = load_plan(2)
    assert len(cfg.hardware.gpu_gpu_comm_params) == 32
    assert len(cfg.hardware.interference_model_params) == 28
    assert cfg.hardware.memory_capacity == pytest.approx(80.0 * 0.88)
