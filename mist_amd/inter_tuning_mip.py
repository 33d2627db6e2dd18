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


def _ckpt_mode(config) -> Tuple[int, int]:
    """inter_tuning_mip.py:471-489."""
    if config.tuning.activation_checkpointing_tuning_enabled:
        return _lib.MIP_CKPT_TUNED, 0
    fixed = getattr(config, "fixed_ckpt_value", None)
    if fixed is not None:
        return _lib.MIP_CKPT_FIXED, int(fixed)
    return _lib.MIP_CKPT_FULL, 0


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


def _problems(num_layers, num_nodes, num_gpus_per_node, grad_accum_candidates, g_index, q_index,
              P1, P, mode, fixed, offset_layers):
    """The (G, S) assignment problems of one search in the reference's order
    (inter_tuning_mip.py:131-214) that have a layer count to sample, as ``MIP_ITEM_DTYPE``
    records without table pointers and offsets, with ``G``, table row ``g``, mesh index ``q``
    and mesh of each."""
    rows = []
    for G in grad_accum_candidates:
        for S in range(1, num_layers + 1):
            if num_nodes * num_gpus_per_node % S != 0:
                continue
            mesh = _uniform_device_mesh_partition(S, num_nodes, num_gpus_per_node)
            if mesh is None or mesh not in q_index:
                continue
            lo, hi = layer_candidates(num_layers, S, G, offset_layers)
            if hi >= lo:
                rows.append((G, g_index[G], S, mesh, q_index[mesh], lo, hi))
    items = np.zeros(len(rows), dtype=_lib.MIP_ITEM_DTYPE)
    items["num_layers"], items["p_dim"], items["sample_size"] = num_layers, P1, P
    items["ckpt_mode"], items["fixed_ckpt"] = mode, fixed
    if rows:
        items["num_stages"] = [r[2] for r in rows]
        items["layers_min"] = [r[5] for r in rows]
        items["layers_max"] = [r[6] for r in rows]
    return items, rows


def inter_stage_tune_batch(
    num_layers: int,
    num_nodes: int,
    num_gpus_per_node: int,
    device_mesh_candidates: List[Tuple[int, int]],
    gradient_accumulation_steps_candidates: List[int],
    results_list: List[IntraStageTunerOutput],
    config,
    stats: Optional[dict] = None,
    only_best_solution: bool = False,
) -> List[Tuple[float, Optional[List[Any]]]]:
    """``inter_stage_tune`` for several intra-stage results at once (the tensor-parallel
    candidates of one ``tune`` call, tables on one device): each is searched as if it were alone
    (its own bound, from ``MAX_VALUE`` down); the policy samples of all their problems come from
    one launch and one copy, the assignments are solved by one library call (a thread per
    search).  ``only_best_solution``: the strategy rows are read back for the first entry with
    the smallest cost only, the others come back as ``(cost, None)``."""
    lib = _lib.load()
    first = results_list[0]
    for res in results_list:
        if not isinstance(res, IntraStageTunerOutput):
            raise TypeError(
                f"intra_stage_results must be an instance of IntraStageTunerOutput, got {type(res)}")
        _, Q, P1, L, _, P = res.device.stable[0].shape
        if L != num_layers:
            raise ValueError(f"tables hold {L} layers, the search asks for {num_layers}")
        if tuple(res.sample_slots) != tuple(range(P)):
            raise ValueError(
                f"the assignment needs every sample of the intra-stage tables; computed slots: "
                f"{tuple(res.sample_slots)} of {P}")
        if P > _lib.MIP_MAX_SAMPLES:
            raise ValueError(f"sample_size {P} exceeds {_lib.MIP_MAX_SAMPLES}")
        if (res.device.stable[0].shape != first.device.stable[0].shape
                or res.gradient_accumulation_steps_candidates != first.gradient_accumulation_steps_candidates
                or res.device_mesh_candidates != first.device_mesh_candidates
                or res.device.stable[0].device != first.device.stable[0].device):
            raise ValueError("the results of one batch must share table shape, candidates and device")
    _, Q, P1, L, _, P = first.device.stable[0].shape
    g_index = {g: i for i, g in enumerate(first.gradient_accumulation_steps_candidates)}
    q_index = {q: i for i, q in enumerate(first.device_mesh_candidates)}
    mode, fixed = _ckpt_mode(config)
    offset_layers = int(getattr(config.tuning, "layers_offset", 2))
    n_res = len(results_list)

    t0 = time.perf_counter()
    one, rows = _problems(num_layers, num_nodes, num_gpus_per_node, gradient_accumulation_steps_candidates,
                          g_index, q_index, P1, P, mode, fixed, offset_layers)
    n_items = len(rows)
    if n_items == 0:
        return [(float("inf"), None)] * n_res
    # every search's problems one after the other: offsets continue through the whole list
    items = np.tile(one, n_res)
    blocks = (one["num_stages"] * (one["layers_max"] - one["layers_min"] + 1)).astype(np.int64)
    blocks = np.tile(blocks, n_res)
    first_block = np.concatenate(([0], np.cumsum(blocks)[:-1]))
    items["first_block"], items["out_offset"] = first_block, first_block * P
    total = int(blocks.sum()) * P
    cell = np.array([r[1] for r in rows], dtype=np.int64) * Q + np.array([r[4] for r in rows], dtype=np.int64)
    for t, res in enumerate(results_list):
        part = items[t * n_items:(t + 1) * n_items]
        for v in range(4):
            for name, tabs in (("stable", res.device.stable), ("delta", res.device.delta)):
                tab = tabs[v]
                assert tab.is_contiguous() and tab.dtype == torch.float64
                part[name][:, v] = tab.data_ptr() + cell * (tab.stride(1) * 8)
    dev = first.device.stable[0].device
    with torch.cuda.device(dev):
        ratios = torch.from_numpy(alpha_ratios(P)).to(dev)
        # t_stable, t_delta (float32), index (int32), keep (uint8) of every problem in one buffer
        out = torch.empty(13 * total, dtype=torch.uint8, device=dev)
        d_items = torch.from_numpy(items.view(np.uint8).reshape(-1)).to(dev)
        rc = lib.mist_mip_stage_samples_batch(
            ctypes.c_void_p(items.ctypes.data), d_items.data_ptr(), len(items), ratios.data_ptr(),
            out.data_ptr(), out.data_ptr() + 4 * total, out.data_ptr() + 8 * total,
            out.data_ptr() + 12 * total, ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
        _lib.check(rc, "mist_mip_stage_samples_batch")
        host = out.cpu().numpy()
    t_stable, t_delta = host[:4 * total].view(np.float32), host[4 * total:8 * total].view(np.float32)
    index, keep = host[8 * total:12 * total].view(np.int32), host[12 * total:]
    t1 = time.perf_counter()

    G_of = np.array([r[0] for r in rows], dtype=np.int32)
    cost = np.empty(n_res, dtype=np.float64)
    winner = np.empty(n_res, dtype=np.int32)
    layers = np.zeros((n_res, L), dtype=np.int32)
    slots = np.zeros((n_res, L), dtype=np.int32)
    ptr = lambda a: ctypes.c_void_p(a.ctypes.data)
    rc = lib.mist_mip_solve_chains(ptr(items), ptr(G_of), n_items, n_res, ptr(t_stable), ptr(t_delta),
                                   ptr(keep), ptr(cost), ptr(winner), ptr(layers), ptr(slots))
    _lib.check(rc, "mist_mip_solve_chains")
    t2 = time.perf_counter()
    if stats is not None:
        stats["mip_problems"] = stats.get("mip_problems", 0) + len(items)
        stats["mip_samples_s"] = stats.get("mip_samples_s", 0.0) + (t1 - t0)
        stats["mip_solve_s"] = stats.get("mip_solve_s", 0.0) + (t2 - t1)

    found = [t for t in range(n_res) if winner[t] >= 0]
    wanted = found
    if only_best_solution and found:
        wanted = [min(found, key=lambda t: cost[t])]  # the first of equals (tune_one_case.py:394-398)
    out_list: List[Tuple[float, Optional[List[Any]]]] = []
    requests, where = [], []
    for t, res in enumerate(results_list):
        if winner[t] < 0:
            out_list.append((float("inf"), None))
            continue
        if t not in wanted:
            out_list.append((float(cost[t]), None))
            continue
        G, g, S, mesh, q, lo, hi = rows[int(winner[t])]
        item = items[t * n_items + int(winner[t])]
        nl = hi - lo + 1
        solution: List[Any] = [G, []]
        covered = 0
        for i in range(S):
            j, a = int(layers[t, i]), int(slots[t, i])
            n = int(index[int(item["out_offset"]) + (i * nl + (j - lo)) * P + a])
            if mode == _lib.MIP_CKPT_TUNED:
                ckpt, policy = n // P, n % P          # inter_tuning_mip.py:507-509
            else:
                ckpt, policy = (fixed if mode == _lib.MIP_CKPT_FIXED else j), n
            l0, l1 = covered, covered + j - 1
            covered += j
            variant, cell_at = _variant_cell(num_layers, g, q, S - i - 1, l0, l1, ckpt, policy)
            requests.append((res, variant, cell_at))
            where.append((len(out_list), i))
            solution[1].append(((l0, l1), mesh, ckpt, policy))
        out_list.append((float(cost[t]), solution))
    for (at, i), row in zip(where, IntraStageTunerOutput.solutions_at(requests)):  # one read-back
        row = row.tolist()
        row[:6] = [int(v) for v in row[:6]]
        stages = out_list[at][1][1]
        stages[i] = (stages[i], tuple(row))
    return out_list


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
    if not isinstance(intra_stage_results, IntraStageTunerOutput):
        raise TypeError(
            f"intra_stage_results must be an instance of IntraStageTunerOutput, got "
            f"{type(intra_stage_results)}")
    return inter_stage_tune_batch(
        num_layers, num_nodes, num_gpus_per_node, device_mesh_candidates,
        gradient_accumulation_steps_candidates, [intra_stage_results], config, stats)[0]
