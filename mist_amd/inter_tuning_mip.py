"""Inter-stage search of the ``uniform-device-pp-mip`` granularity: drop-in for the reference's
``mist/analyzer/inter_tuning_mip.py`` (``inter_stage_tune`` :87-253,
``inter_stage_tune_with_fixed_grad_accumu_and_device_partition`` :256-424,
``preprocess_stable_and_delta_costs`` :427-535).

For every gradient-accumulation count G and every stage count S that divides the device count and
splits the cluster into one uniform mesh, stage i takes ``j`` layers (around L / S) and one of the
sampled policies of its table cell; the reference minimises ``(G - 1) * max T + sum T + max(0,
max_i (D_i - sum_{i'<i} T_i'))`` with PuLP / CBC.  Here

* the policy samples of every (G, S) problem come from one kernel launch each on the float64
  tables resident in HBM (``mist_mip_stage_samples``); only the resulting (S, layer counts, P)
  arrays are copied to the host, once for all problems;
* the assignment is solved exactly by the library's host solver (``mist_mip_solve``): the
  objective's last two terms follow the recurrence ``Z' = T + max(Z, D)``, so a pass over the
  stages per candidate value of ``max T`` finds the optimum.  CBC returns *an* optimum within its
  tolerances; which one of several equal assignments it picks is not reproducible, the solver
  here takes the smallest ``max T`` first and then the first minimum in (layer count, sample)
  order.

The intra-stage tables must hold every sample (``sample_slots`` = all of ``sample_size``), as in
the reference's MIP branch (benchmark/mist/tune/tune_one_case.py:377-392).  Deviations: a search
in which no problem reaches a cost below ``MAX_VALUE`` returns ``(inf, None)`` (the reference
fails on ``len(None)`` there); stage counts beyond the pre-saved-micro-batch axis cost ``inf``
(IndexError in the reference); a stage count whose uniform split is no mesh candidate is skipped.
"""
from __future__ import annotations

import ctypes
import time
from typing import Any, List, Optional, Tuple

import numpy as np
import torch

from . import _lib
from .inter_tuning_uniform import _uniform_device_mesh_partition
from .intra_tuning import IntraStageTunerOutput, alpha_ratios

MAX_VALUE = _lib.MIP_MAX_VALUE  # inter_tuning_mip.py:39


def layer_candidates(num_layers: int, num_stages: int, grad_accum: int, layers_offset: int = 2):
    """inter_tuning_mip.py:282-290: the layer counts one stage may take, as (min, max)."""
    avg = round(num_layers / num_stages)
    if grad_accum == 1:
        return avg, avg
    return max(avg - layers_offset, 1), min(avg + layers_offset, num_layers - num_stages + 1)


def cells_wanted(num_layers: int, num_nodes: int, num_gpus_per_node: int, layers_offset: int = 2):
    """What the assignment reads of the intra-stage tables of a (G, mesh) group, for
    ``IntraStageTuner.cells_wanted``: a mesh is read for the one stage count S whose even split
    of the cluster it is (inter_tuning_mip.py:267-281), there for the layer counts of
    ``layer_candidates`` and the pre-saved micro-batch values 0..S-1 (stage i of S keeps S - i - 1);
    a mesh that is no such split is not read at all."""
    num_devices = num_nodes * num_gpus_per_node

    def wanted(G: int, mesh: Tuple[int, int]):
        n, m = mesh
        if n * m <= 0 or num_devices % (n * m) != 0:
            return None
        S = num_devices // (n * m)
        if S > num_layers or _uniform_device_mesh_partition(S, num_nodes, num_gpus_per_node) != mesh:
            return None
        lo, hi = layer_candidates(num_layers, S, G, layers_offset)
        return (lo, hi, S) if hi >= lo else None

    return wanted


class _Problem:
    """One (G, S) assignment problem: its shape and where its samples lie in the batch buffers."""

    __slots__ = ("G", "g", "S", "mesh", "q", "shape", "offset", "count")

    def __init__(self, G, g, S, mesh, q, shape, offset, count):
        self.G, self.g, self.S, self.mesh, self.q = G, g, S, mesh, q
        self.shape, self.offset, self.count = shape, offset, count


def _ckpt_mode(config) -> Tuple[int, int]:
    """inter_tuning_mip.py:471-489."""
    if config.tuning.activation_checkpointing_tuning_enabled:
        return _lib.MIP_CKPT_TUNED, 0
    fixed = getattr(config, "fixed_ckpt_value", None)
    if fixed is not None:
        return _lib.MIP_CKPT_FIXED, int(fixed)
    return _lib.MIP_CKPT_FULL, 0


def stage_samples(results: IntraStageTunerOutput, problems: List[_Problem]):
    """Launches ``mist_mip_stage_samples`` for every problem and returns the host copies
    ``(t_stable, t_delta, index, keep)`` of the concatenated outputs."""
    lib = _lib.load()
    tables = results.device
    dev = tables.stable[0].device
    total = sum(p.count for p in problems)
    P = tables.stable[0].shape[-1]
    with torch.cuda.device(dev):
        ratios = torch.from_numpy(alpha_ratios(P)).to(dev)
        t_stable = torch.empty(max(total, 1), dtype=torch.float32, device=dev)
        t_delta = torch.empty(max(total, 1), dtype=torch.float32, device=dev)
        index = torch.empty(max(total, 1), dtype=torch.int32, device=dev)
        keep = torch.empty(max(total, 1), dtype=torch.uint8, device=dev)
        stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        live = [p for p in problems if p.count > 0]
        if live:
            # every problem in one launch: the rows are a few hundred candidates each, and one
            # launch per problem (~220 for a 32-layer plan) left the GPU to one wavefront per row
            items = (_lib.MipBatchItem * len(live))()
            first_block = 0
            for item, p in zip(items, live):
                item.shape = p.shape
                for v in range(4):
                    item.tables.stable[v] = tables.stable[v][p.g, p.q].data_ptr()
                    item.tables.delta[v] = tables.delta[v][p.g, p.q].data_ptr()
                item.out_offset, item.first_block = p.offset, first_block
                first_block += p.count // P
            d_items = torch.frombuffer(bytearray(bytes(items)), dtype=torch.uint8).to(dev)
            rc = lib.mist_mip_stage_samples_batch(
                ctypes.byref(items), d_items.data_ptr(), len(live), ratios.data_ptr(),
                t_stable.data_ptr(), t_delta.data_ptr(), index.data_ptr(), keep.data_ptr(), stream)
            _lib.check(rc, "mist_mip_stage_samples_batch")
        return (t_stable.cpu().numpy(), t_delta.cpu().numpy(), index.cpu().numpy(),
                keep.cpu().numpy())


def solve(problem: _Problem, best_cost: float, t_stable, t_delta, keep):
    """``mist_mip_solve`` on one problem's slice of the host arrays.  Returns ``(cost, layers,
    slots)`` or ``(inf, None, None)``."""
    lib = _lib.load()
    S = problem.S
    lo, hi = problem.offset, problem.offset + problem.count
    ts = np.ascontiguousarray(t_stable[lo:hi])
    td = np.ascontiguousarray(t_delta[lo:hi])
    kp = np.ascontiguousarray(keep[lo:hi])
    cost = ctypes.c_double()
    layers = np.zeros(S, dtype=np.int32)
    slots = np.zeros(S, dtype=np.int32)
    rc = lib.mist_mip_solve(
        ctypes.byref(problem.shape), int(problem.G), float(best_cost), ts.ctypes.data,
        td.ctypes.data, kp.ctypes.data, ctypes.byref(cost), layers.ctypes.data, slots.ctypes.data)
    if rc < 0:
        _lib.check(rc, "mist_mip_solve")
    if rc == 0:
        return float("inf"), None, None
    return cost.value, layers, slots


def _variant_cell(num_layers, g, q, p, l0, l1, ckpt, slot):
    """Table variant and cell of a stage (inter_tuning_mip.py:62-84)."""
    l = l1 - l0 + 1
    if l0 == 0 and l1 == num_layers - 1:
        return 3, (g, q, ckpt, slot)
    if l0 == 0:
        return 1, (g, q, p, l - 1, ckpt, slot)
    if l1 == num_layers - 1:
        return 2, (g, q, l - 1, ckpt, slot)
    return 0, (g, q, p, l - 1, ckpt, slot)


def inter_stage_tune(
    num_layers: int,
    num_nodes: int,
    num_gpus_per_node: int,
    device_mesh_candidates: List[Tuple[int, int]],
    gradient_accumulation_steps_candidates: List[int],
    intra_stage_results: IntraStageTunerOutput,
    config,
    stats: Optional[dict] = None,
) -> Tuple[float, Optional[List[Any]]]:
    """Reference signature (inter_tuning_mip.py:87-95).  Returns ``(best_cost, [G, [(((l0, l1),
    (n, m), ckpt, policy), strategy_row), ...per stage]])`` or ``(inf, None)``."""
    res = intra_stage_results
    if not isinstance(res, IntraStageTunerOutput):
        raise TypeError(
            f"intra_stage_results must be an instance of IntraStageTunerOutput, got {type(res)}")
    tables = res.device
    _, _, P1, L, _, P = tables.stable[0].shape
    if L != num_layers:
        raise ValueError(f"tables hold {L} layers, the search asks for {num_layers}")
    if tuple(res.sample_slots) != tuple(range(P)):
        raise ValueError(
            f"the assignment needs every sample of the intra-stage tables; computed slots: "
            f"{tuple(res.sample_slots)} of {P}")
    if P > _lib.MIP_MAX_SAMPLES:
        raise ValueError(f"sample_size {P} exceeds {_lib.MIP_MAX_SAMPLES}")
    g_index = {g: i for i, g in enumerate(res.gradient_accumulation_steps_candidates)}
    q_index = {q: i for i, q in enumerate(res.device_mesh_candidates)}
    mode, fixed = _ckpt_mode(config)
    offset_layers = int(getattr(config.tuning, "layers_offset", 2))

    t0 = time.perf_counter()
    problems: List[_Problem] = []
    cursor = 0
    for G in gradient_accumulation_steps_candidates:
        for S in range(1, num_layers + 1):
            if num_nodes * num_gpus_per_node % S != 0:
                continue
            mesh = _uniform_device_mesh_partition(S, num_nodes, num_gpus_per_node)
            if mesh is None or mesh not in q_index:
                continue
            lo, hi = layer_candidates(num_layers, S, G, offset_layers)
            shape = _lib.MipShape(num_layers=L, p_dim=P1, sample_size=P, num_stages=S,
                                  layers_min=lo, layers_max=hi, ckpt_mode=mode, fixed_ckpt=fixed)
            count = S * max(hi - lo + 1, 0) * P
            problems.append(_Problem(G, g_index[G], S, mesh, q_index[mesh], shape, cursor, count))
            cursor += count
    t_stable, t_delta, index, keep = stage_samples(res, problems)
    t1 = time.perf_counter()

    best_cost, best = MAX_VALUE, None
    for prob in problems:  # in the reference's order: best_cost tightens as it goes
        if prob.count == 0:
            continue
        cost, layers, slots = solve(prob, best_cost, t_stable, t_delta, keep)
        if cost < best_cost:
            best_cost, best = cost, (prob, layers, slots)
    t2 = time.perf_counter()
    if stats is not None:
        stats["mip_problems"] = stats.get("mip_problems", 0) + len(problems)
        stats["mip_samples_s"] = stats.get("mip_samples_s", 0.0) + (t1 - t0)
        stats["mip_solve_s"] = stats.get("mip_solve_s", 0.0) + (t2 - t1)
    if best is None:
        return float("inf"), None

    prob, layers, slots = best
    nl = prob.shape.layers_max - prob.shape.layers_min + 1
    solution: List[Any] = [prob.G, []]
    requests = []
    covered = 0
    for i in range(prob.S):
        j, a = int(layers[i]), int(slots[i])
        n = int(index[prob.offset + (i * nl + (j - prob.shape.layers_min)) * P + a])
        if mode == _lib.MIP_CKPT_TUNED:
            ckpt, policy = n // P, n % P          # inter_tuning_mip.py:507-509
        else:
            ckpt, policy = (fixed if mode == _lib.MIP_CKPT_FIXED else j), n
        l0, l1 = covered, covered + j - 1
        covered += j
        variant, cell = _variant_cell(num_layers, prob.g, prob.q, prob.S - i - 1, l0, l1, ckpt, policy)
        requests.append((res, variant, cell))
        solution[1].append(((l0, l1), prob.mesh, ckpt, policy))
    for i, row in enumerate(IntraStageTunerOutput.solutions_at(requests)):  # one read-back
        row = row.tolist()
        row[:6] = [int(v) for v in row[:6]]
        solution[1][i] = (solution[1][i], tuple(row))
    return best_cost, solution
