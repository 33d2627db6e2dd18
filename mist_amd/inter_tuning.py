"""Inter-stage pipeline-partition search on the GPU: drop-in for the reference's
``mist/analyzer/inter_tuning.py`` (``inter_stage_tune`` :63-160,
``inter_stage_tune_with_fixed_grad_accumu`` :163-217, ``inter_stage_tune_dp_impl`` :220-355).

The reference runs one numba DP per candidate ``t_max`` in an ascending host loop that stops
once ``t_max * G >= best``.  Here the DP for many thresholds runs in one launch (one workgroup
per threshold) and the host replays the reference's sequential rules on the returned
``(best_s, sum, stage_max)`` triples, so the accepted thresholds, the winner and all ties are
the reference's.  Two exact shortcuts: thresholds below the first feasible one are located by a
multi-way search instead of being run one by one (feasibility is monotone in ``t_max`` and an
infeasible run changes nothing), and thresholds past the stop condition are never used.

The reference's DP reads ``costs / costs_with_pre / ...`` fields that its intra tuner no longer
emits; the cost tables are built from the stable / delta tables as
``float32(stable) + float32(delta) / G`` (see ``mist_dp_cost_tables``), sample slot 0 by
default, and stage solutions carry a trailing policy index 0 so that ``best_solution_yaml``
accepts them.
"""
from __future__ import annotations

import ctypes
from typing import List, Optional, Tuple

import numpy as np
import torch

from . import _lib
from .intra_tuning import IntraStageTunerOutput

PROBES = 256      # thresholds per launch while searching for the first feasible one
CHUNK = 1024      # thresholds per launch while scanning
GAP = 1e-6        # inter_tuning.py:177


def _stream(device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class _DpRunner:
    """Owns the float32 cost tables of all g and runs batches of thresholds for one g."""

    def __init__(self, results: IntraStageTunerOutput, num_layers: int, num_devices: int,
                 meshes: List[Tuple[int, int]], slot: int):
        self.lib = _lib.load()
        dev_tabs = results.device
        self.device = dev_tabs.stable[0].device
        Gs = results.gradient_accumulation_steps_candidates
        Gn, Q, P1, L, C, S = dev_tabs.stable[0].shape
        assert L == num_layers and C == L + 1
        if list(meshes) != list(results.device_mesh_candidates):
            raise ValueError("the DP needs the mesh list the intra-stage tables were built for")
        self.L, self.D, self.Q, self.P1 = L, num_devices, Q, P1
        shape = np.zeros(1, dtype=_lib.DP_SHAPE_DTYPE)
        shape["num_layers"], shape["num_devices"], shape["num_mesh"], shape["p_dim"] = L, num_devices, Q, P1
        self.S_max = min(max(n * m for n, m in meshes), L) // 2  # inter_tuning.py:278-280
        shape["max_stages"] = self.S_max
        shape["mesh_n"][0, :Q] = [n for n, _ in meshes]
        shape["mesh_m"][0, :Q] = [m for _, m in meshes]
        self.shape = shape
        problem = np.zeros(1, dtype=_lib.PROBLEM_DTYPE)
        problem["num_layers"], problem["p_dim"], problem["sample_size"] = L, P1, S
        problem["num_grad_accum"], problem["num_mesh"] = Gn, Q
        with torch.cuda.device(self.device):
            self.cost = [
                torch.empty(tuple(t.shape[:-1]), dtype=torch.float32, device=self.device)
                for t in dev_tabs.stable
            ]
            d_G = torch.tensor(Gs, dtype=torch.int32, device=self.device)
            out_ptrs = (ctypes.c_void_p * 4)(*[t.data_ptr() for t in self.cost])
            tabs = dev_tabs.as_struct()
            rc = self.lib.mist_dp_cost_tables(
                ctypes.c_void_p(problem.ctypes.data), ctypes.byref(tabs), d_G.data_ptr(), slot,
                out_ptrs, _stream(self.device),
            )
            _lib.check(rc, "mist_dp_cost_tables")
        self.launches = 0
        self.thresholds_run = 0

    def thresholds(self, g: int) -> np.ndarray:
        """Ascending unique finite stage costs of g (inter_tuning.py:180-186) after the gap
        rule (:198), float32."""
        allv = torch.cat([self.cost[v][g].reshape(-1) for v in range(3)])
        allv = torch.unique(allv[torch.isfinite(allv)])  # sorted ascending
        host = allv.cpu().numpy()
        kept = np.empty_like(host)
        n = self.lib.mist_dp_filter_tmax(
            ctypes.c_void_p(host.ctypes.data), len(host), GAP, ctypes.c_void_p(kept.ctypes.data)
        )
        return kept[:n]

    def run(self, g: int, tmax: np.ndarray, want_argmin: bool = False):
        """DP for every threshold in ``tmax`` -> (best_s int32, best_sum f32, stage_max f32
        [, argmin])."""
        n = len(tmax)
        dev = self.device
        with torch.cuda.device(dev):
            d_t = torch.from_numpy(np.ascontiguousarray(tmax, dtype=np.float32)).to(dev)
            d_s = torch.empty(n, dtype=torch.int32, device=dev)
            d_sum = torch.empty(n, dtype=torch.float32, device=dev)
            d_max = torch.empty(n, dtype=torch.float32, device=dev)
            n_scratch = self.lib.mist_dp_scratch_floats(ctypes.c_void_p(self.shape.ctypes.data), n)
            if n_scratch < 0:
                _lib.check(-1, "mist_dp_scratch_floats")
            scratch = torch.empty(n_scratch, dtype=torch.float32, device=dev) if n_scratch else None
            argmin = None
            if want_argmin:
                argmin = torch.full((self.S_max + 1, self.L + 1, self.D + 1, 4), -1,
                                    dtype=torch.int32, device=dev)
            costs = _lib.DpCosts(*[self.cost[v][g].data_ptr() for v in range(4)])
            rc = self.lib.mist_dp_run(
                ctypes.c_void_p(self.shape.ctypes.data), ctypes.byref(costs), d_t.data_ptr(), n,
                d_s.data_ptr(), d_sum.data_ptr(), d_max.data_ptr(),
                argmin.data_ptr() if want_argmin else None,
                scratch.data_ptr() if scratch is not None else None, _stream(dev),
            )
            _lib.check(rc, "mist_dp_run")
            self.launches += 1
            self.thresholds_run += n
            out = (d_s.cpu().numpy(), d_sum.cpu().numpy(), d_max.cpu().numpy())
            if want_argmin:
                out = out + (argmin.cpu().numpy(),)
        return out

    def first_feasible(self, g: int, tmax: np.ndarray) -> int:
        """Index of the smallest feasible threshold (len(tmax) if none): multi-way search."""
        lo, hi = 0, len(tmax)  # invariant: everything below lo is infeasible
        if hi == 0:
            return 0
        best_s, _, _ = self.run(g, tmax[-1:])
        if best_s[0] < 0:
            return hi
        hi -= 1  # tmax[hi] is feasible
        while hi - lo > 0:
            probes = np.unique(np.linspace(lo, hi, min(PROBES, hi - lo + 1)).astype(np.int64))
            best_s, _, _ = self.run(g, tmax[probes])
            feas = np.nonzero(best_s >= 0)[0]
            first = int(feas[0])  # probes[-1] == hi is feasible, so this exists
            hi = int(probes[first])
            lo = int(probes[first - 1]) + 1 if first > 0 else lo
            if first == 0:
                break
        return hi


def inter_stage_tune_with_fixed_grad_accumu(
    runner: _DpRunner, g: int, gradient_accumulation_steps: int, best_cost: float = float("inf"),
):
    """inter_tuning.py:163-217 -> (best_cost, best_t_max or None)."""
    G = gradient_accumulation_steps
    tmax = runner.thresholds(g)
    best_t = None
    if len(tmax) == 0:
        return best_cost, best_t
    # float32 scalar * python int is float64 under the reference's numpy 1.24.
    scaled = tmax.astype(np.float64) * G
    start = runner.first_feasible(g, tmax[: int(np.searchsorted(scaled, best_cost, side="left"))])
    pos = start
    while pos < len(tmax):
        if scaled[pos] >= best_cost:
            break
        stop = int(np.searchsorted(scaled, best_cost, side="left"))
        chunk = tmax[pos: min(pos + CHUNK, stop)]
        best_s, best_sum, stage_max = runner.run(g, chunk)
        for i in range(len(chunk)):
            if scaled[pos + i] >= best_cost:
                return best_cost, best_t
            if best_s[i] < 0:
                continue
            cost = float(np.float64(best_sum[i]) + np.float64(G - 1) * np.float64(stage_max[i]))
            if cost < best_cost:
                best_cost, best_t = cost, chunk[i]
        pos += len(chunk)
    return best_cost, best_t


def get_solution_from_intra_stage_tuner_output(
    intra_stage_results, num_layers, gradient_accumulation_steps_index, pre_saved_micro_batches,
    layer_start, layer_end, device_mesh_idx, num_ckpt_layers, slot=0,
):
    """inter_tuning.py:38-60 with the sample slot made explicit."""
    g, q, p, c = gradient_accumulation_steps_index, device_mesh_idx, pre_saved_micro_batches, num_ckpt_layers
    l = layer_end - layer_start + 1
    r = intra_stage_results
    if layer_start == 0 and layer_end == num_layers - 1:
        return r.solutions_no_pp[g, q, c, slot]
    if layer_start == 0:
        return r.solutions_with_pre[g, q, p, l - 1, c, slot]
    if layer_end == num_layers - 1:
        return r.solutions_with_post[g, q, l - 1, c, slot]
    return r.solutions[g, q, p, l - 1, c, slot]


def inter_stage_tune(
    num_layers: int,
    num_devices: int,
    device_mesh_candidates: List[Tuple[int, int]],
    gradient_accumulation_steps_candidates: List[int],
    intra_stage_results: IntraStageTunerOutput,
    slot: int = 0,
    stats: Optional[dict] = None,
):
    """Reference signature (inter_tuning.py:63-69).  Returns ``(best_cost, [G, [(((l0, l1),
    (n, m), ckpt, 0), strategy_row), ...]])`` or ``(inf, None)`` when nothing is feasible."""
    if not isinstance(intra_stage_results, IntraStageTunerOutput):
        raise TypeError(
            f"intra_stage_results must be an instance of IntraStageTunerOutput, got {type(intra_stage_results)}"
        )
    runner = _DpRunner(intra_stage_results, num_layers, num_devices, device_mesh_candidates, slot)
    g_index = {G: i for i, G in enumerate(intra_stage_results.gradient_accumulation_steps_candidates)}
    q_index = {q: i for i, q in enumerate(intra_stage_results.device_mesh_candidates)}
    best_cost, best_G, best_t = float("inf"), None, None
    for G in gradient_accumulation_steps_candidates:
        cost, t = inter_stage_tune_with_fixed_grad_accumu(runner, g_index[G], G, best_cost)
        if cost < best_cost and t is not None:
            best_cost, best_G, best_t = cost, G, t
    if stats is not None:
        stats["dp_launches"] = stats.get("dp_launches", 0) + runner.launches
        stats["dp_thresholds"] = stats.get("dp_thresholds", 0) + runner.thresholds_run
    if best_G is None:
        return float("inf"), None

    # Back-pointers of the winning (G, t_max) run (inter_tuning.py:341-355).
    g = g_index[best_G]
    best_s, best_sum, stage_max, argmin = runner.run(g, np.array([best_t], dtype=np.float32), True)
    cs, cl, cd = int(best_s[0]), 0, num_devices
    inter = []
    while cs > 0 and cl < num_layers and cd > 0:
        end, n, m, ckpt = (int(v) for v in argmin[cs, cl, cd])
        assert end != -1
        inter.append(((cl, end), (n, m), ckpt))
        cs, cl, cd = cs - 1, end + 1, cd - n * m
    assert cs == 0 and cl == num_layers and cd == 0
    solution = [best_G, []]
    for i, ((l0, l1), (n, m), ckpt) in enumerate(inter):
        row = get_solution_from_intra_stage_tuner_output(
            intra_stage_results, num_layers, g, len(inter) - i - 1, l0, l1, q_index[(n, m)], ckpt, slot
        ).tolist()
        row[:6] = [int(x) for x in row[:6]]
        solution[1].append((((l0, l1), (n, m), ckpt, 0), tuple(row)))
    return best_cost, solution
