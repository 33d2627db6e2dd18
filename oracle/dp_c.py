"""Oracle (test infrastructure): builds and wraps oracle/dp.c (the plain-C form of the
reference's numba DP kernel, mist/analyzer/inter_tuning.py:220-355) with the same call
signature as ``oracle.inter_dp.dp_impl``.  Output goes to oracle/_build/ (git-ignored)."""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "dp.c")
LIB = os.path.join(HERE, "_build", "libmist_oracle_dp.so")
_lib = None


def build(force=False):
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    if force or not os.path.exists(LIB) or os.path.getmtime(LIB) < os.path.getmtime(SRC):
        subprocess.run(
            ["gcc", "-O2", "-ffp-contract=off", "-shared", "-fPIC", SRC, "-o", LIB, "-lm"], check=True
        )
    return LIB


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = ctypes.CDLL(LIB)
        _lib.mist_oracle_dp.restype = ctypes.c_int
    return _lib


def dp_impl_c(t_max, num_layers, num_devices, meshes, G, costs, costs_pre, costs_post, costs_nopp,
              want_solution=True):
    lib = _load()
    L, D, Q = num_layers, num_devices, len(meshes)
    f32 = lambda a: np.ascontiguousarray(a, dtype=np.float32)
    costs, costs_pre, costs_post, costs_nopp = map(f32, (costs, costs_pre, costs_post, costs_nopp))
    P1 = costs.shape[1]
    assert costs.shape == (Q, P1, L, L + 1) and costs_pre.shape == costs.shape
    assert costs_post.shape == (Q, L, L + 1) and costs_nopp.shape == (Q, L + 1)
    S = min(max(n * m for n, m in meshes), L) // 2
    mesh_n = np.array([n for n, _ in meshes], dtype=np.int32)
    mesh_m = np.array([m for _, m in meshes], dtype=np.int32)
    arg = np.empty((S + 1, L + 1, D + 1, 4), dtype=np.int32) if want_solution else None
    best_s, best_sum, stage_max = ctypes.c_int(), ctypes.c_float(), ctypes.c_float()
    ptr = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    rc = lib.mist_oracle_dp(
        ctypes.c_float(float(t_max)), L, D, Q, ptr(mesh_n), ptr(mesh_m), P1, ptr(costs),
        ptr(costs_pre), ptr(costs_post), ptr(costs_nopp), ctypes.byref(best_s),
        ctypes.byref(best_sum), ctypes.byref(stage_max), ptr(arg) if want_solution else None,
    )
    assert rc == 0
    if best_s.value < 0:
        return np.inf, None
    total = float(np.float64(np.float32(best_sum.value)) + np.float64(G - 1) * np.float64(np.float32(stage_max.value)))
    if not want_solution:
        return total, None
    res, cs, cl, cd = [], best_s.value, 0, D
    while cs > 0 and cl < L and cd > 0:
        end, n, m, ckpt = (int(v) for v in arg[cs, cl, cd])
        assert end != -1
        res.append(((cl, end), (n, m), ckpt))
        cs, cl, cd = cs - 1, end + 1, cd - n * m
    assert cs == 0 and cl == L and cd == 0
    return total, res
