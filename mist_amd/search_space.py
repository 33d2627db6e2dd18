"""Candidate enumeration for one (mesh, gradient-accumulation) group, kept factored.

Mirrors ``create_search_space_for_a_block_layer`` (reference:
mist/analyzer/batched_module_analyzer.py:417-536) and the two live helpers of
mist/tuning/optimization.py:33-55, with one structural difference: the (N, 10) row matrix is
never built.  A group is described by its parallelism rows and its four offload-ratio lists; the
kernels and ``SearchSpace.decode`` recover row ``r`` by index decomposition
(parallelism-major, then ``itertools.product(wo, go, oo, ao)`` without ``wo > 0 and go == 0``).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, List, Optional, Sequence, Tuple

from functools import lru_cache

import numpy as np

from ._lib import MAX_PAIRS, MAX_PAR, MAX_RATIOS
from .config import MistConfig

POWER_OF_TWO = [2**i for i in range(0, 15)]


def _get_device_mesh_candidates(
    num_nodes: int, num_gpus_per_node: int, contiguous_inter_node: bool = True
) -> List[Tuple[int, int]]:
    """mist/tuning/optimization.py:33-51."""
    candidates = [(1, m) for m in range(1, num_gpus_per_node + 1) if m in POWER_OF_TWO]
    for n in range(2, num_nodes + 1):
        if contiguous_inter_node or n in POWER_OF_TWO:
            candidates.append((n, num_gpus_per_node))
    assert len(candidates) == len(set(candidates)), f"Duplicate device mesh candidates: {candidates}"
    return candidates


def _get_grad_accumu_steps_candidates(global_batch_size: int) -> List[int]:
    """mist/tuning/optimization.py:54-55."""
    return [i for i in POWER_OF_TWO if global_batch_size % i == 0]


@dataclass(frozen=True)
class SearchSpace:
    """Factored strategy rows ``(b, dp, tp, wre, gre, ore, wo, go, oo, ao)`` of one group."""

    par: np.ndarray  # (n_par, 6) float64
    wo: Tuple[float, ...]
    go: Tuple[float, ...]
    oo: Tuple[float, ...]
    ao: Tuple[float, ...]
    pair_wo: np.ndarray  # (n_pair,) uint8: index into ``wo`` of every valid (wo, go) pair
    pair_go: np.ndarray  # (n_pair,) uint8

    @property
    def n_par(self) -> int:
        return int(self.par.shape[0])

    @property
    def n_pair(self) -> int:
        return int(self.pair_wo.shape[0])

    @property
    def n_off(self) -> int:
        return self.n_pair * len(self.oo) * len(self.ao)

    @property
    def n_rows(self) -> int:
        return self.n_par * self.n_off

    def decode(self, index: np.ndarray) -> np.ndarray:
        """Rows for an integer index array of any shape -> ``index.shape + (10,)`` float64;
        ``-1`` decodes to an all-``inf`` row like the reference's unfilled solutions."""
        index = np.asarray(index, dtype=np.int64)
        out = np.full(index.shape + (10,), np.inf, dtype=np.float64)
        valid = index >= 0
        if self.n_rows == 0 or not valid.any():
            return out
        r = index[valid]
        assert int(r.max()) < self.n_rows, "row index outside the search space"
        n_oo, n_ao = len(self.oo), len(self.ao)
        par_i, off = np.divmod(r, self.n_off)
        pair, tail = np.divmod(off, n_oo * n_ao)
        oo_i, ao_i = np.divmod(tail, n_ao)
        rows = np.empty((r.shape[0], 10), dtype=np.float64)
        rows[:, :6] = self.par[par_i]
        rows[:, 6] = np.asarray(self.wo)[self.pair_wo[pair]]
        rows[:, 7] = np.asarray(self.go)[self.pair_go[pair]]
        rows[:, 8] = np.asarray(self.oo)[oo_i]
        rows[:, 9] = np.asarray(self.ao)[ao_i]
        out[valid] = rows
        return out

    def materialize(self) -> np.ndarray:
        """The full (N, 10) matrix (tests and small cases only)."""
        return self.decode(np.arange(self.n_rows))


@lru_cache(maxsize=None)
def _valid_pairs(wo: Tuple[float, ...], go: Tuple[float, ...]):
    """(wo index, go index) of ``itertools.product(wo, go)`` minus ``wo > 0 and go == 0``
    (batched_module_analyzer.py:522-530); the same lists recur for every (G, mesh, tp) group."""
    pair_wo, pair_go = [], []
    for i, w in enumerate(wo):
        for j, g in enumerate(go):
            if not (w > 0 and g == 0):
                pair_wo.append(i)
                pair_go.append(j)
    return tuple(pair_wo), tuple(pair_go)


class SearchSpaceFactory:
    """``create_search_space_for_a_block_layer`` for many groups of one configuration: what only
    depends on the configuration (ratio lists, valid pairs, flags) is read once."""

    def __init__(self, config: MistConfig, constraint_fn: Optional[Callable[[int, int], bool]] = None):
        tuning = config.tuning
        self.batch_sizes = tuple(tuning.batch_size_candidates)
        self.zero_2_and_3 = bool(tuning.zero_2_and_3_enabled)
        self.flag_choices = tuple(tuning.zero_flag_choices)
        self.disable_tp = bool(getattr(config, "disable_tp_tuning", False))
        self.constraint_fn = constraint_fn
        self.lists = _offload_lists(
            bool(tuning.state_offloading_enabled), bool(tuning.activation_offloading_enabled),
            tuple(tuning.offloading_ratio_candidates), tuple(tuning.sparse_offloading_ratio_candidates),
            bool(getattr(config, "disable_wo_tuning", False)), bool(getattr(config, "disable_go_tuning", False)),
            bool(getattr(config, "disable_oo_tuning", False)),
            *(getattr(config, f"fixed_{k}_ratio", None) for k in ("wo", "go", "oo", "ao")),
        )
        self._constraint = {}
        self._empty = np.zeros((0, 6), dtype=np.float64)

    def _allowed(self, batch_size: int, tp_size: int) -> bool:
        key = (batch_size, tp_size)
        if key not in self._constraint:
            self._constraint[key] = bool(self.constraint_fn(batch_size, tp_size))
        return self._constraint[key]

    def make(self, num_nodes: int, num_gpus_per_node: int, global_batch_size: int,
             gradient_accumulation_steps: int, tp_size: Optional[int] = None) -> SearchSpace:
        """Reference: batched_module_analyzer.py:417-536 (same filters, same order)."""
        num_gpus = num_nodes * num_gpus_per_node
        per_micro_batch = global_batch_size // gradient_accumulation_steps
        par = []
        for batch_size in self.batch_sizes:
            if batch_size > per_micro_batch or per_micro_batch % batch_size != 0:
                continue
            dp_size = per_micro_batch // batch_size
            if dp_size > num_gpus or num_gpus % dp_size != 0:
                continue
            curr_tp_size = num_gpus // dp_size
            if self.constraint_fn is not None and not self._allowed(batch_size, curr_tp_size):
                continue
            # The tp size latches to the first feasible batch size when the caller gave none.
            tp_size = curr_tp_size if tp_size is None else tp_size
            if tp_size != curr_tp_size:
                continue
            if tp_size > num_gpus_per_node:
                continue
            if self.disable_tp and tp_size > 1:
                continue
            if dp_size == 1 or not self.zero_2_and_3:
                flag_choices: Sequence[Tuple[int, int, int]] = ((0, 0, 1),)
            else:
                flag_choices = self.flag_choices
            for wre, gre, ore in flag_choices:
                par.append((batch_size, dp_size, tp_size, wre, gre, ore))
        par_np = np.array(par, dtype=np.float64).reshape(-1, 6) if par else self._empty
        if par_np.shape[0] > MAX_PAR:
            raise ValueError(f"{par_np.shape[0]} parallelism rows; at most {MAX_PAR} are supported")
        wo, go, oo, ao, pair_wo, pair_go = self.lists
        return SearchSpace(par=par_np, wo=wo, go=go, oo=oo, ao=ao, pair_wo=pair_wo, pair_go=pair_go)


def create_search_space_for_a_block_layer(
    num_nodes: int,
    num_gpus_per_node: int,
    global_batch_size: int,
    gradient_accumulation_steps: int,
    config: MistConfig,
    constraint_fn: Optional[Callable[[int, int], bool]] = None,
    tp_size: Optional[int] = None,
) -> SearchSpace:
    """Reference: batched_module_analyzer.py:417-536 (same filters, same order)."""
    return SearchSpaceFactory(config, constraint_fn).make(
        num_nodes, num_gpus_per_node, global_batch_size, gradient_accumulation_steps, tp_size)


@lru_cache(maxsize=64)
def _offload_lists(state_offloading, activation_offloading, dense, sparse, disable_wo, disable_go,
                   disable_oo, fixed_wo, fixed_go, fixed_oo, fixed_ao):
    """Ratio lists and valid (wo, go) pairs of a configuration (batched_module_analyzer.py:
    487-531); they do not depend on the group, so the 100+ groups of a plan share one result
    (the index arrays are read-only)."""
    if state_offloading:
        wo, go, oo = sparse, sparse, dense
        if disable_wo:
            wo = (0.0,)
        if disable_go:
            go = (0.0,)
        if disable_oo:
            oo = (0.0,)
    else:
        wo, go, oo = (0.0,), (0.0,), (0.0,)
    if fixed_wo is not None:
        wo = (float(fixed_wo),)
    if fixed_go is not None:
        go = (float(fixed_go),)
    if fixed_oo is not None:
        oo = (float(fixed_oo),)
    if activation_offloading:
        ao = dense
    elif fixed_ao is not None:
        ao = (float(fixed_ao),)
    else:
        ao = (0.0,)

    pair_wo, pair_go = _valid_pairs(tuple(wo), tuple(go))

    for name, values in (("wo", wo), ("go", go), ("oo", oo), ("ao", ao)):
        if len(values) > MAX_RATIOS:
            raise ValueError(f"{name} ratio list has {len(values)} values; at most {MAX_RATIOS}")
    assert len(pair_wo) <= MAX_PAIRS
    pair_wo_np, pair_go_np = np.array(pair_wo, dtype=np.uint8), np.array(pair_go, dtype=np.uint8)
    pair_wo_np.setflags(write=False)
    pair_go_np.setflags(write=False)
    return (tuple(float(x) for x in wo), tuple(float(x) for x in go), tuple(float(x) for x in oo),
            tuple(float(x) for x in ao), pair_wo_np, pair_go_np)
