"""Shared helpers of the test-suite: plan loading, tiny plan variants, oracle <-> kernel maps."""
import copy
import hashlib
import os

import numpy as np
import yaml

from mist_amd.config import MistConfig
from mist_amd.layer_tables import LayerTables

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CONFIG_DIR = os.path.join(REPO, "mist_amd", "configs")
PLAN_FILES = [
    "gpt-1.3b-b8-1x2.yaml",
    "gpt-7b-b512-4x8.yaml",
    "llama-13b-b1024-8x8.yaml",
    "gpt-22b-b1536-16x8.yaml",
    "llama-70b-b2048-32x8.yaml",
]


def load_raw(index):
    with open(os.path.join(CONFIG_DIR, PLAN_FILES[index - 1])) as f:
        return yaml.safe_load(f)


def load_plan(index, **overrides):
    """Plan ``index`` (1..5) with optional overrides given as 'section.key' = value (top-level
    keys without a dot)."""
    raw = load_raw(index)
    for key, value in overrides.items():
        node = raw
        parts = key.split("__")
        for p in parts[:-1]:
            node = node[p]
        node[parts[-1]] = value
    cfg = MistConfig(raw)
    return cfg, LayerTables(cfg)


def tiny_plan(base=1, layers=6, **overrides):
    """A plan small enough for the numpy oracle to finish in well under a second per group."""
    ov = dict(model__num_hidden_layers=layers)
    ov.update(overrides)
    return load_plan(base, **ov)


def oracle_terms(dbg, n_rows):
    """Row-term matrix (N, ROW_TERMS) assembled from the oracle's debug arrays, in the column
    order of include/mist_search.h."""
    from mist_amd._lib import TERM_NAMES

    lat = dbg["lat"]
    bc = lambda a: np.broadcast_to(np.asarray(a, dtype=np.float64), (n_rows,))
    cols = dict(
        s_layer_ck=lat["ck"]["s_layer"], s_layer_nock=lat["nock"]["s_layer"],
        s_first_ck=lat["ck"]["s_first"], s_first_nock=lat["nock"]["s_first"],
        s_last_ck=lat["ck"]["s_last"], s_last_nock=lat["nock"]["s_last"],
        d_layer_ck=lat["ck"]["d_layer"], d_layer_nock=lat["nock"]["d_layer"],
        d_first_ck=lat["ck"]["d_first"], d_first_nock=lat["nock"]["d_first"],
        d_last_ck=lat["ck"]["d_last"], d_last_nock=lat["nock"]["d_last"],
        fwd_states0=dbg["T0"], bwd_states0=dbg["T1"], pWG=dbg["pWG"], pO=dbg["pO"],
        pWGO=dbg["pWGO"], S_ck=dbg["S_ck"], S_nock=dbg["S_nock"], D_ck=dbg["D_ck"],
        D_nock=dbg["D_nock"], mf_base=dbg["mf"] + 0.025 + 0.01, mf_pp=dbg["mf"] + 0.025,
        mf=dbg["mf"], fwd_peak=dbg["fwd_peak_nock"], bwd_peak=dbg["bwd_peak"], out=dbg["out"],
        gcb=dbg["gcb"], nAG_ck=dbg["nAG"]["ck"], nAG_nock=dbg["nAG"]["nock"],
        nRS_ck=dbg["nRS"]["ck"], nRS_nock=dbg["nRS"]["nock"], opb=dbg["opb"], RD=dbg["RD"],
    )
    return np.stack([bc(cols[name]) for name in TERM_NAMES], axis=1)


def bits(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float64)).view(np.uint64)


def assert_same_f64(got, want, what=""):
    """Bit-for-bit equality of float64 arrays (NaN-free inputs; +-0 are treated as equal)."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    same = (got == want) | (np.isinf(got) & np.isinf(want) & (np.sign(got) == np.sign(want)))
    if not same.all():
        bad = np.argwhere(~same)
        first = tuple(bad[0])
        raise AssertionError(
            f"{what}: {len(bad)} of {got.size} differ; first at {first}: got {got[first]!r} "
            f"want {want[first]!r} (rel {abs(got[first]-want[first])/max(abs(want[first]),1e-300):.3e})"
        )


def group_key(tp, G, mesh):
    """Name of a (tensor-parallel size, gradient-accumulation steps, stage mesh) group in the
    fixtures of tests/golden/search_tables_plan*.json."""
    return f"tp{tp}/G{G}/{mesh[0]}x{mesh[1]}"


def table_digest(index, stable, delta):
    """Digest of one result table of a group: row indices as little-endian int32, then the
    stable and delta costs as little-endian float32 (-0 folded into +0), all in C order."""
    h = hashlib.sha256()
    h.update(np.ascontiguousarray(index).astype("<i4").tobytes())
    for a in (stable, delta):
        a = np.ascontiguousarray(a).astype(np.float32) + np.float32(0)
        h.update(a.astype("<f4").tobytes())
    return h.hexdigest()[:32]
