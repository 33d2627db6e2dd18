"""Oracle (test infrastructure): four-resource interference model, vectorised numpy.

Restates ``interference_estimate_for_one_group`` / ``_update`` /
``calculate_overlap_and_remain`` (mist/tools/optimize.py:1012-1122, 552-571) with the mask
tables of :951-964.  Resources are ordered X = [C, G2G, C2G, G2C].

Pinned by (tests/test_oracle_models.py): one non-zero input -> identity; all 28 factors 1 ->
exactly ``max``; factors >= 1 -> ``out >= max``; brute-force scalar re-derivation of the
peeling on random inputs; the worked example X=(1,100,0,0), f=(50,50) -> 149.
"""
from copy import deepcopy

import numpy as np

THREE_CASE_MASKS = [
    [True, True, True, False],
    [True, True, False, True],
    [True, False, True, True],
    [False, True, True, True],
]
TWO_CASE_MASKS = [
    [True, True, False, False],
    [True, False, True, False],
    [True, False, False, True],
    [False, True, True, False],
    [False, True, False, True],
    [False, False, True, True],
]


def mask_factor_table(params):
    """The 11 (mask, factors) pairs in evaluation order: the 4-way case with params[0:4], the
    four 3-way cases with params[4:16] (three each, in position order), the six 2-way cases with
    params[16:28] (two each).  Positions outside the mask carry factor 1."""
    params = np.asarray(params, dtype=np.float64)
    if params.size != 28:
        raise ValueError(f"Length: {params.size}. It should be 28.")
    table = [(np.array([True] * 4), params[:4].copy())]
    for i, m in enumerate(THREE_CASE_MASKS):
        f = np.ones(4)
        f[np.array(m)] = params[4 + 3 * i : 4 + 3 * (i + 1)]
        table.append((np.array(m), f))
    for i, m in enumerate(TWO_CASE_MASKS):
        f = np.ones(4)
        f[np.array(m)] = params[16 + 2 * i : 16 + 2 * (i + 1)]
        table.append((np.array(m), f))
    return table


def _peel(X, out, mask, factors):
    """optimize.py:1082-1113 + 552-571: rows whose non-zero pattern (``not isclose(x, 0)``, i.e.
    ``|x| > 1e-8``) equals ``mask`` get ``ov = min(X*f over mask)`` added to ``out`` and
    ``X[mask] = ((X*f - ov) / f * 1.0)[mask]``."""
    nz = np.logical_not(np.isclose(X, 0))
    rows = np.where(np.all(nz == mask, axis=-1))[0]
    feat = np.where(mask)[0]
    vals = X[rows]
    scaled = vals * factors
    overlap = np.min(scaled[..., feat], axis=-1)
    updated = (scaled - overlap[:, None]) / factors * np.ones_like(factors)
    vals[..., feat] = updated[..., feat]
    out[rows] += overlap
    X[rows] = vals


def interference_one_group(C, G2G, C2G, G2C, params):
    """optimize.py:1012-1079."""
    arrs = np.broadcast_arrays(
        *[np.atleast_1d(np.asarray(a, dtype=np.float64)) for a in (C, G2G, C2G, G2C)]
    )
    # The reference deep-copies the transposed stack, which keeps its column-major layout.
    X = deepcopy(np.vstack(arrs).T)
    out = np.zeros(X.shape[0], dtype=np.float64)
    for mask, factors in mask_factor_table(params):
        _peel(X, out, mask, factors)
    out += np.sum(X, axis=-1)
    return out
