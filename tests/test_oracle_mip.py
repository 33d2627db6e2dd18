"""Pins the oracle of the ``uniform-device-pp-mip`` inter-stage search: the exact assignment
solver against enumeration of every assignment with the objective written as in the reference's
MILP, the sample preprocessing against per-cell scans, and the library's host solver against the
oracle's (CPU only: the solver is host code inside the shared library)."""
import ctypes

import numpy as np
import pytest

from mist_amd import _lib
from oracle import inter_mip
from oracle.pareto import alpha_ratios, compute_indices_scan


def test_layer_candidates_hand_computed():
    lc = inter_mip.layer_candidates
    assert lc(32, 4, 2) == [6, 7, 8, 9, 10]
    assert lc(32, 4, 1) == [8]                 # G == 1: only the average
    assert lc(32, 32, 4) == [1]                # clipped by L - S + 1
    assert lc(32, 16, 4) == [1, 2, 3, 4]       # clipped below by 1
    assert lc(10, 4, 3) == [1, 2, 3, 4]        # round(2.5) == 2 (half to even)
    assert lc(14, 4, 3) == [2, 3, 4, 5, 6]     # round(3.5) == 4
    assert lc(32, 1, 8) == [30, 31, 32]
    assert lc(8, 2, 2, layers_offset=1) == [3, 4, 5]


def test_fill_redundant_samples_keeps_first_occurrence():
    rng = np.random.default_rng(0)
    x = rng.integers(0, 3, size=(20, 6)).astype(np.float32)
    y = rng.integers(0, 2, size=(20, 6)).astype(np.float32)
    x[3, :] = np.inf
    y[3, :] = np.inf
    idx = rng.integers(0, 100, size=(20, 6))
    keep, fx, fy, fidx = inter_mip.fill_redundant_samples(x, y, idx)
    for i in range(20):
        first = [a for a in range(6)
                 if not any(x[i, b] == x[i, a] and y[i, b] == y[i, a] for b in range(a))]
        assert sorted(keep[i]) == first
        # np.unique returns the kept slots in ascending (x, y) order
        pairs = [(float(x[i, a]), float(y[i, a])) for a in keep[i]]
        assert pairs == sorted(pairs)
        for a in range(6):
            if a in first:
                assert fx[i, a] == x[i, a] and fy[i, a] == y[i, a] and fidx[i, a] == idx[i, a]
            else:
                assert np.isinf(fx[i, a]) and np.isinf(fy[i, a]) and fidx[i, a] == -1


def _random_tables(rng, P1, L, P, inf_frac=0.2, quantum=None, neg_frac=0.0):
    def rand(shape):
        a = rng.uniform(0.05, 1.0, size=shape).astype(np.float32)
        if quantum:
            a = (np.round(a / quantum) * quantum).astype(np.float32)
        return a
    shapes = [(P1, L, L + 1, P), (P1, L, L + 1, P), (L, L + 1, P), (L + 1, P)]
    out = []
    for shape in shapes:
        s, d = rand(shape), rand(shape)
        bad = rng.random(shape[:-1]) < inf_frac   # a whole cell is infeasible at once ...
        s[bad] = np.inf
        d[bad] = np.inf
        tail = rng.random(shape) < inf_frac / 2     # ... or only its later samples
        s[tail] = np.inf
        d[tail] = np.inf
        if neg_frac:
            d[(rng.random(shape) < neg_frac) & np.isfinite(d)] *= -1
        out.append((s, d))
    (s0, d0), (s1, d1), (s2, d2), (s3, d3) = out
    return [s0, d0, s1, d1, s2, d2, s3, d3]


@pytest.mark.parametrize("mode", ["tuned", "fixed", "full"])
def test_preprocess_against_cell_scan(mode):
    rng = np.random.default_rng(5)
    L, P1, P = 5, 3, 4
    for S in (1, 2, 3, 4):
        tabs = _random_tables(rng, P1, L, P, quantum=0.125, neg_frac=0.05)
        fixed = 2 if mode == "fixed" else None
        choices, t_s, t_d, (ck, pol) = inter_mip.preprocess_stable_and_delta_costs(
            S, mode == "tuned", fixed, *tabs)
        stable, delta, stable_pre, delta_pre, stable_post, delta_post, stable_nopp, delta_nopp = tabs
        ratios = alpha_ratios(P)
        for i in range(S):
            for l in range(L + 1):
                # the table row the reference's assignments (:453-468) leave in t[i, l]
                if l == 0:
                    xs = ys = np.full((L + 1, P), np.inf, dtype=np.float32)
                elif i == 0 and l == L:
                    xs, ys = stable_nopp, delta_nopp
                elif i == S - 1:
                    xs, ys = stable_post[l - 1], delta_post[l - 1]
                elif i == 0:
                    xs, ys = ((stable_pre[S - 1, l - 1], delta_pre[S - 1, l - 1]) if S - 1 < P1
                              else (np.full((L + 1, P), np.inf),) * 2)
                else:
                    p = S - i - 1
                    xs, ys = ((stable[p, l - 1], delta[p, l - 1]) if p < P1
                              else (np.full((L + 1, P), np.inf),) * 2)
                if mode == "tuned":
                    cx, cy = xs.reshape(1, -1), ys.reshape(1, -1)
                else:
                    c = fixed if mode == "fixed" else l
                    cx, cy = (xs[c].reshape(1, -1), ys[c].reshape(1, -1)) if l > 0 else (
                        np.full((1, P), np.inf), np.full((1, P), np.inf))
                idx = compute_indices_scan(cx, cy, np.ones(cx.shape, dtype=bool), ratios)[0]
                seen = set()
                for a in range(P):
                    n = int(idx[a])
                    x, y = float(cx[0, n]), float(cy[0, n])   # n == -1 reads the last candidate
                    kept = (x, y) not in seen
                    seen.add((x, y))
                    assert (a in choices[i][l]) == kept
                    want_x = inter_mip.MAX_VALUE if (not kept or np.isinf(x)) else max(x, 0.0)
                    want_y = inter_mip.MAX_VALUE if (not kept or np.isinf(y)) else max(y, 0.0)
                    assert t_s[i, l, a] == np.float32(want_x), (S, i, l, a)
                    assert t_d[i, l, a] == np.float32(want_y), (S, i, l, a)
                    if mode == "tuned":
                        assert (ck[i, l, a], pol[i, l, a]) == (n // P, n % P)
                    else:
                        assert (ck[i, l, a], pol[i, l, a]) == (fixed if mode == "fixed" else l, n)


def _random_assignment_problem(rng, S, layers, P, quantum, max_frac):
    L_axis = max(layers) + 1
    t_s = np.full((S, L_axis, P), inter_mip.MAX_VALUE, dtype=np.float32)
    t_d = np.full((S, L_axis, P), inter_mip.MAX_VALUE, dtype=np.float32)
    choices = []
    for i in range(S):
        row = {}
        for j in layers:
            n = int(rng.integers(1, P + 1))
            slots = sorted(rng.choice(P, size=n, replace=False).tolist())
            row[j] = slots
            for k in slots:
                if rng.random() < max_frac:
                    continue
                t_s[i, j, k] = np.round(rng.uniform(0.1, 2.0) / quantum) * quantum
                t_d[i, j, k] = np.round(rng.uniform(0.0, 3.0) / quantum) * quantum
        choices.append(row)
    return choices, t_s, t_d


def test_solver_against_enumeration():
    rng = np.random.default_rng(11)
    checked = feasible = 0
    for trial in range(300):
        S = int(rng.integers(1, 5))
        lo = int(rng.integers(1, 3))
        layers = list(range(lo, lo + int(rng.integers(1, 4))))
        P = int(rng.integers(1, 4))
        L = int(rng.integers(S * layers[0], S * layers[-1] + 2))   # sometimes unreachable
        G = int(rng.choice([1, 2, 3, 8]))
        quantum = float(rng.choice([0.25, 0.001]))                 # coarse values tie often
        choices, t_s, t_d = _random_assignment_problem(rng, S, layers, P, quantum, 0.1)
        best_cost = float(rng.choice([inter_mip.MAX_VALUE, 4.0, 1.0]))
        want = inter_mip.solve_bruteforce(L, layers, choices, t_s, t_d, G, best_cost)
        cost, picks = inter_mip.solve(L, layers, choices, t_s, t_d, G, best_cost)
        checked += 1
        if np.isinf(want):
            assert picks is None and np.isinf(cost), trial
            continue
        feasible += 1
        assert cost == pytest.approx(want, rel=1e-12, abs=0), trial
        # the returned assignment is admissible and has the reported objective
        assert sum(j for j, _ in picks) == L
        assert all(k in choices[i][j] for i, (j, k) in enumerate(picks))
        T = [t_s[i, j, k] for i, (j, k) in enumerate(picks)]
        D = [t_d[i, j, k] for i, (j, k) in enumerate(picks)]
        assert inter_mip.objective(T, D, G) == pytest.approx(cost, rel=1e-12, abs=0)
        assert max(float(t) for t in T) * (G - 1) <= best_cost
    assert checked == 300 and feasible > 150


def test_objective_recurrence_identity():
    """Z_0 = 0, Z_{i+1} = T_i + max(Z_i, D_i) reproduces sum T + max(0, max_i(D_i - prefix_i))."""
    rng = np.random.default_rng(2)
    for _ in range(200):
        n = int(rng.integers(1, 9))
        T = rng.integers(0, 16, size=n) / 4.0      # dyadic: both sides exact
        D = rng.integers(0, 40, size=n) / 4.0
        z = 0.0
        for t, d in zip(T, D):
            z = t + max(z, d)
        assert z == inter_mip.objective(T, D, 1)
        assert inter_mip.objective(T, D, 5) == z + 4 * T.max()


def _solve_c(L, layers, choices, t_s, t_d, G, best_cost):
    lib = _lib.load()
    S, P = len(choices), t_s.shape[-1]
    nl = len(layers)
    shape = _lib.MipShape(num_layers=L, p_dim=1, sample_size=P, num_stages=S,
                          layers_min=layers[0], layers_max=layers[-1], ckpt_mode=0, fixed_ckpt=0)
    ts = np.ascontiguousarray(t_s[:, layers[0]:layers[-1] + 1], dtype=np.float32)
    td = np.ascontiguousarray(t_d[:, layers[0]:layers[-1] + 1], dtype=np.float32)
    keep = np.zeros((S, nl, P), dtype=np.uint8)
    for i in range(S):
        for a, j in enumerate(layers):
            keep[i, a, list(choices[i][j])] = 1
    cost = ctypes.c_double()
    out_layers = np.zeros(S, dtype=np.int32)
    out_slot = np.zeros(S, dtype=np.int32)
    rc = lib.mist_mip_solve(ctypes.byref(shape), G, best_cost, ts.ctypes.data, td.ctypes.data,
                            keep.ctypes.data, ctypes.byref(cost), out_layers.ctypes.data,
                            out_slot.ctypes.data)
    assert rc in (0, 1), lib.mist_last_error()
    if rc == 0:
        return np.inf, None
    return cost.value, list(zip(out_layers.tolist(), out_slot.tolist()))


def test_library_host_solver_equals_oracle():
    rng = np.random.default_rng(23)
    solved = 0
    for trial in range(120):
        S = int(rng.integers(1, 9))
        avg = int(rng.integers(1, 6))
        layers = list(range(max(avg - 2, 1), avg + 3))
        P = int(rng.integers(1, 9))
        L = S * avg + int(rng.integers(-1, 2))
        if L < S or layers[-1] > L:
            continue
        G = int(rng.choice([1, 2, 4, 16]))
        quantum = float(rng.choice([0.125, 1e-4]))
        choices, t_s, t_d = _random_assignment_problem(rng, S, layers, P, quantum, 0.15)
        best_cost = float(rng.choice([inter_mip.MAX_VALUE, 20.0, 6.0]))
        want_cost, want_picks = inter_mip.solve(L, layers, choices, t_s, t_d, G, best_cost)
        cost, picks = _solve_c(L, layers, choices, t_s, t_d, G, best_cost)
        if want_picks is None:
            assert picks is None
            continue
        solved += 1
        assert cost == want_cost and picks == want_picks, trial   # same arithmetic, same tie rule
    assert solved > 60


def test_library_host_solver_rejects_bad_shapes():
    lib = _lib.load()
    cost = ctypes.c_double()
    buf = np.zeros(64, dtype=np.int32)
    f = np.zeros(64, dtype=np.float32)
    k = np.ones(64, dtype=np.uint8)
    bad = _lib.MipShape(num_layers=4, p_dim=1, sample_size=65, num_stages=2, layers_min=1,
                        layers_max=3, ckpt_mode=0, fixed_ckpt=0)
    assert lib.mist_mip_solve(ctypes.byref(bad), 2, 1e6, f.ctypes.data, f.ctypes.data,
                              k.ctypes.data, ctypes.byref(cost), buf.ctypes.data, buf.ctypes.data) < 0
    assert b"sample_size" in lib.mist_last_error()
    empty = _lib.MipShape(num_layers=4, p_dim=1, sample_size=2, num_stages=4, layers_min=3,
                          layers_max=1, ckpt_mode=0, fixed_ckpt=0)
    assert lib.mist_mip_solve(ctypes.byref(empty), 2, 1e6, f.ctypes.data, f.ctypes.data,
                              k.ctypes.data, ctypes.byref(cost), buf.ctypes.data, buf.ctypes.data) == 0
    assert np.isinf(cost.value)
