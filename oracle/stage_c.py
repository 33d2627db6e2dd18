"""Oracle (test infrastructure): builds and wraps oracle/stage_loop.c, the plain-C form of the
(ckpt layers, pre-saved micro-batches) loops of ``batched_stage_analyze``
(mist/analyzer/batched_module_analyzer.py:2165-3106) and of ``compute_indices``
(mist/utils/pareto.py:124-144).  ``oracle.stage.batched_stage_analyze(..., inner="c")`` hands the
row-invariant arrays it computed in numpy to ``run`` and gets the same four result tuples as from
its own numpy loops, bit for bit (tests/test_oracle_stage_c.py).  Output goes to oracle/_build/
(git-ignored)."""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "stage_loop.c")
LIB = os.path.join(HERE, "_build", "libmist_oracle_stage.so")
LIB_FUSED = os.path.join(HERE, "_build", "libmist_oracle_stage_fused.so")
_libs = {}

_P = ctypes.c_void_p
_D = ctypes.c_double


class StageLoopIn(ctypes.Structure):
    _fields_ = [
        ("n_rows", ctypes.c_int64), ("L", ctypes.c_int32), ("C", ctypes.c_int32),
        ("n_p", ctypes.c_int32), ("S", ctypes.c_int32), ("G", ctypes.c_int32),
        ("pp_wre", ctypes.c_int32), ("pp_gre", ctypes.c_int32), ("pad_", ctypes.c_int32),
        ("ratios", _P),
        ("s_layer", _P * 2), ("s_first", _P * 2), ("s_last", _P * 2),
        ("d_layer", _P * 2), ("d_first", _P * 2), ("d_last", _P * 2),
        ("T0", _P), ("T1", _P), ("pWG", _P), ("pO", _P), ("pWGO", _P),
        ("S_sav", _P * 2), ("D_sav", _P * 2),
        ("fwd_peak", _P), ("bwd_peak", _P), ("out", _P), ("gcb", _P), ("mf", _P), ("RD", _P),
        ("nAG", _P * 2), ("nRS", _P * 2), ("opb", _P),
        ("pre_fwd", _D), ("pre_bwd", _D), ("W1", _D), ("W2", _D), ("W1d", _D), ("W2d", _D),
        ("post_fwd", _D),
        ("pre_saved", _D), ("pre_states", _D), ("pre_states_and_saved", _D),
        ("post_states", _D), ("post_fwd_peak", _D), ("post_bwd_peak", _D), ("post_output", _D),
        ("cap", _D),
    ]


class StageLoopOut(ctypes.Structure):
    _fields_ = [("idx", _P * 4), ("stable", _P * 4), ("delta", _P * 4)]


def build(force=False, fused=False):
    """Compiles for plain AVX2 x86-64 (the library built here also runs on the GPU box's host).
    ``fused``: the variant whose argmin objective is one fused multiply-add (-DMIST_ORACLE_FUSED)."""
    lib = LIB_FUSED if fused else LIB
    os.makedirs(os.path.dirname(lib), exist_ok=True)
    if force or not os.path.exists(lib) or os.path.getmtime(lib) < os.path.getmtime(SRC):
        extra = ["-DMIST_ORACLE_FUSED", "-mfma"] if fused else []
        subprocess.run(
            ["gcc", "-O3", "-mavx2", "-ffp-contract=off", "-fno-fast-math", "-fopenmp", "-shared",
             "-fPIC", *extra, SRC, "-o", lib, "-lm"], check=True)
    return lib


def _load(fused=False):
    if fused not in _libs:
        path = LIB_FUSED if fused else LIB
        if not os.path.exists(path):
            build(fused=fused)
        lib = ctypes.CDLL(path)
        lib.mist_oracle_stage_loop.restype = ctypes.c_int
        lib.mist_oracle_stage_loop.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        assert lib.mist_oracle_stage_loop_struct_bytes() == ctypes.sizeof(StageLoopIn)
        _libs[fused] = lib
    return _libs[fused]


def _scalar(x):
    a = np.asarray(x, dtype=np.float64).reshape(-1)
    assert a.size == 1, "the pre / post layer strategy of the tuning path is a single row"
    return float(a[0])


def run(n_rows, L, C, n_p, S, G, ratios, lat, mem, post, scalars, pp_wre, pp_gre, cap, threads=0,
        fused=False):
    """``lat[k][name]``, ``mem[name]``, ``post[name]`` are per-row float64 arrays (or scalars that
    broadcast); ``scalars[name]`` python floats / one-element arrays.  Returns
    ``[(stable, delta, idx)] * 4`` with the numpy oracle's shapes and fills (inf / -1)."""
    lib = _load(fused)
    keep = []

    def rows(a):
        a = np.ascontiguousarray(np.broadcast_to(np.asarray(a, dtype=np.float64), (n_rows,)))
        keep.append(a)
        return a.ctypes.data

    s = StageLoopIn()
    s.n_rows, s.L, s.C, s.n_p, s.S, s.G = n_rows, L, C, n_p, S, G
    s.pp_wre, s.pp_gre = int(pp_wre), int(pp_gre)
    r = np.ascontiguousarray(ratios, dtype=np.float64)
    assert r.shape == (S,)
    s.ratios = r.ctypes.data
    for name in ("s_layer", "s_first", "s_last", "d_layer", "d_first", "d_last"):
        for k, key in enumerate(("nock", "ck")):
            getattr(s, name)[k] = rows(lat[key][name])
    for name in ("T0", "T1", "pWG", "pO", "pWGO", "fwd_peak", "bwd_peak", "out", "gcb", "mf", "RD"):
        setattr(s, name, rows(mem[name]))
    for k, key in enumerate(("nock", "ck")):
        s.S_sav[k] = rows(mem["S_" + key])
        s.D_sav[k] = rows(mem["D_" + key])
        s.nAG[k] = rows(post["nAG"][key])
        s.nRS[k] = rows(post["nRS"][key])
    s.opb = rows(post["opb"])
    for name in ("pre_fwd", "pre_bwd", "W1", "W2", "W1d", "W2d", "post_fwd", "pre_saved",
                 "pre_states", "pre_states_and_saved", "post_states", "post_fwd_peak",
                 "post_bwd_peak", "post_output"):
        setattr(s, name, _scalar(scalars[name]))
    s.cap = float(cap)
    shapes = [(n_p, L, C + 1, S), (n_p, L, C + 1, S), (L, C + 1, S), (C + 1, S)]
    o = StageLoopOut()
    res = []
    for v, shape in enumerate(shapes):
        idx = np.full(shape, -1, dtype=np.int64)
        stable = np.full(shape, np.inf)
        delta = np.full(shape, np.inf)
        o.idx[v], o.stable[v], o.delta[v] = idx.ctypes.data, stable.ctypes.data, delta.ctypes.data
        res.append((stable, delta, idx))
    rc = lib.mist_oracle_stage_loop(ctypes.byref(s), ctypes.byref(o), int(threads))
    assert rc == 0
    return res
