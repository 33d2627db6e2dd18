"""Inter-stage pipeline-partition search on the GPU: drop-in for the reference's
``mist/analyzer/inter_tuning.py`` (``inter_stage_tune`` :63-160,
``inter_stage_tune_with_fixed_grad_accumu`` :163-217, ``inter_stage_tune_dp_impl`` :220-355).

The reference runs one numba DP per candidate ``t_max`` in an ascending host loop that stops
once ``t_max * G >= best``, G after G.  Here many DP instances (any mix of G and thresholds)
run in one batch of launches and the host replays the reference's sequential rules on the
returned ``(best_s, sum, stage_max)`` triples, so the accepted thresholds, the winner and all
ties are the reference's.  Exact shortcuts: (1) thresholds below the smallest feasible one are
not run one by one; that point comes from one bottleneck (min-max) DP per G (an infeasible
run changes nothing in the reference's scan); (2) thresholds are computed ahead speculatively
under a bound on the running best that the sequential scan is certain to have reached, and the
replay asks for more wherever it runs out, so a wrong guess costs time, never correctness.

The reference's DP reads ``costs / costs_with_pre / ...`` fields that its intra tuner no longer
emits; the cost tables are built from the stable / delta tables as
``float32(stable) + float32(delta) / G`` (see ``mist_dp_cost_tables``), sample slot 0 by
default, and stage solutions carry a trailing policy index 0 so that ``best_solution_yaml``
accepts them.
"""
from __future__ import annotations

import ctypes
import time
from typing import List, Optional, Tuple

import numpy as np
import torch

from . import _lib
from .intra_tuning import IntraStageTunerOutput

FIRST_CHUNK = 48  # thresholds per G in the first speculative scan launch
MAX_CHUNK = 4096  # most thresholds per G in one launch
GAP = 1e-6        # inter_tuning.py:177


def _stream(device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class _DpRunner:
    """Owns the float32 cost tables of all g and runs batches of DP instances."""

    def __init__(self, results: IntraStageTunerOutput, num_layers: int, num_devices: int,
                 meshes: List[Tuple[int, int]], slot: int):
        self.lib = _lib.load()
        dev_tabs = results.batch  # tables of every tp candidate of the same launch
        self.device = dev_tabs.stable[0].device
        Gn, Q, P1, L, C, S = dev_tabs.stable[0].shape
        n_g = len(results.gradient_accumulation_steps_candidates)
        assert Gn % n_g == 0
        Gs = list(results.gradient_accumulation_steps_candidates) * (Gn // n_g)
        assert L == num_layers and C == L + 1
        if list(meshes) != list(results.device_mesh_candidates):
            raise ValueError("the DP needs the mesh list the intra-stage tables were built for")
        self.L, self.D, self.Q, self.P1, self.Gn = L, num_devices, Q, P1, Gn
        shape = np.zeros(1, dtype=_lib.DP_SHAPE_DTYPE)
        shape["num_layers"], shape["num_devices"], shape["num_mesh"], shape["p_dim"] = L, num_devices, Q, P1
        self.S_max = min(max(n * m for n, m in meshes), L) // 2  # inter_tuning.py:278-280
        shape["max_stages"] = self.S_max
        shape["mesh_n"][0, :Q] = [n for n, _ in meshes]
        shape["mesh_m"][0, :Q] = [m for _, m in meshes]
        self.shape = shape
        self.plane = (L + 1) * (num_devices + 1)
        problem = np.zeros(1, dtype=_lib.PROBLEM_DTYPE)
        problem["num_layers"], problem["p_dim"], problem["sample_size"] = L, P1, S
        problem["num_grad_accum"], problem["num_mesh"] = Gn, Q
        with torch.cuda.device(self.device):
            self.cost = [
                torch.empty(tuple(t.shape[:-1]), dtype=torch.float32, device=self.device)
                for t in dev_tabs.stable
            ]
            self.pmin = [torch.empty_like(t) for t in self.cost]
            d_G = torch.tensor(Gs, dtype=torch.int32, device=self.device)
            out_ptrs = (ctypes.c_void_p * 4)(*[t.data_ptr() for t in self.cost])
            pmin_ptrs = (ctypes.c_void_p * 4)(*[t.data_ptr() for t in self.pmin])
            tabs = dev_tabs.as_struct()
            rc = self.lib.mist_dp_cost_tables(
                ctypes.c_void_p(problem.ctypes.data), ctypes.byref(tabs), d_G.data_ptr(), slot,
                out_ptrs, pmin_ptrs, _stream(self.device),
            )
            _lib.check(rc, "mist_dp_cost_tables")
        self.costs_struct = _lib.DpCosts(*[t.data_ptr() for t in self.cost + self.pmin])
        for v in range(4):
            self.costs_struct.g_stride[v] = self.cost[v][0].numel()
        self.launches = 0
        self.thresholds_run = 0

    def thresholds(self) -> List[np.ndarray]:
        """Per g: ascending unique finite stage costs (inter_tuning.py:180-186) after the gap
        rule (:198), float32.  One device sort for all g, the sequential rule on the host."""
        allv = torch.cat([self.cost[v].reshape(self.Gn, -1) for v in range(3)], dim=1)
        n_fin = int(torch.isfinite(allv).sum(dim=1).max().item())
        # +inf sorts last: only the finite prefix is copied to the host
        host = torch.sort(allv, dim=1).values[:, :max(n_fin, 1)].contiguous().cpu().numpy()
        out = []
        kept = np.empty(host.shape[1], dtype=np.float32)
        for g in range(self.Gn):
            row = np.ascontiguousarray(host[g])
            n_finite = int(np.searchsorted(row, np.inf, side="left"))
            # duplicates have a zero difference to the last kept value and fall to the gap rule
            n = self.lib.mist_dp_filter_tmax(
                ctypes.c_void_p(row.ctypes.data), n_finite, GAP, ctypes.c_void_p(kept.ctypes.data)
            )
            out.append(kept[:n].copy())
        return out

    def run(self, g_index: np.ndarray, tmax: np.ndarray, mode: int = _lib.DP_THRESHOLD,
            want_argmin: bool = False):
        """DP instances (g_index[i], tmax[i]) -> (best_s int32, best_sum f32, stage_max f32
        [, argmin])."""
        n = len(tmax)
        dev = self.device
        with torch.cuda.device(dev):
            packed = np.empty((2, n), dtype=np.float32)
            packed[0] = tmax
            packed[1].view(np.int32)[:] = g_index
            d_in = torch.from_numpy(packed).to(dev)
            d_out = torch.empty((3, n), dtype=torch.float32, device=dev)
            scratch = torch.empty(4 * n * self.plane, dtype=torch.float32, device=dev)
            argmin = None
            if want_argmin:
                argmin = torch.full((n, self.S_max + 1, self.L + 1, self.D + 1, 4), -1,
                                    dtype=torch.int32, device=dev)
            rc = self.lib.mist_dp_run(
                ctypes.c_void_p(self.shape.ctypes.data), ctypes.byref(self.costs_struct),
                d_in[0].data_ptr(), d_in[1].data_ptr(), n, mode,
                d_out[0].data_ptr(), d_out[1].data_ptr(), d_out[2].data_ptr(),
                argmin.data_ptr() if want_argmin else None, scratch.data_ptr(), _stream(dev),
            )
            _lib.check(rc, "mist_dp_run")
            self.launches += 1
            self.thresholds_run += n
            host = d_out.cpu().numpy()
            out = (host[0].view(np.int32), host[1], host[2])
            if want_argmin:
                out = out + (argmin.cpu().numpy(),)
        return out


class _Scan:
    """Replay state of ``inter_stage_tune_with_fixed_grad_accumu`` (inter_tuning.py:163-217) for
    one G: ``pos`` = next threshold the sequential scan would look at, ``results`` = DP outcomes
    already computed for tmax[lo : lo + len]."""

    def __init__(self, G: int, tmax: np.ndarray, first: int):
        self.G, self.tmax = G, tmax
        # float32 scalar * python int is float64 under the reference's numpy 1.24.
        self.scaled = tmax.astype(np.float64) * G
        self.pos = first          # everything below is infeasible: the scan passes it unchanged
        self.have_lo = first
        self.best_s = np.empty(0, dtype=np.int32)
        self.best_sum = np.empty(0, dtype=np.float32)
        self.stage_max = np.empty(0, dtype=np.float32)
        self.limit = FIRST_CHUNK

    def wanted(self, best_cost: float) -> Tuple[int, int]:
        """Index range [a, b) of thresholds to compute next under the bound ``best_cost``; the
        range grows fourfold every time the same G asks again."""
        a = self.have_lo + len(self.best_s)
        stop = int(np.searchsorted(self.scaled, best_cost, side="left"))
        b = max(a, min(stop, a + self.limit))
        if b > a:
            self.limit = min(MAX_CHUNK, self.limit * 4)
        return a, b

    def runs_out(self, best_cost: float) -> bool:
        """Dry run of ``replay`` under the bound ``best_cost`` (the true running best when this G
        is reached is no larger, so the true scan stops no later): True if the computed results
        would not suffice."""
        pos, hi, G = self.pos, self.have_lo + len(self.best_s), self.G
        while pos < len(self.tmax):
            if self.scaled[pos] >= best_cost:
                return False
            if pos >= hi:
                return True
            i = pos - self.have_lo
            if self.best_s[i] >= 0:
                cost = float(np.float64(self.best_sum[i]) + np.float64(G - 1) * np.float64(self.stage_max[i]))
                best_cost = min(best_cost, cost)
            pos += 1
        return False

    def add(self, best_s, best_sum, stage_max):
        self.best_s = np.concatenate([self.best_s, best_s])
        self.best_sum = np.concatenate([self.best_sum, best_sum])
        self.stage_max = np.concatenate([self.stage_max, stage_max])

    def replay(self, best_cost: float, best_t):
        """Advances the sequential scan as far as the computed results allow.  Returns
        (best_cost, best_t, finished)."""
        G = self.G
        hi = self.have_lo + len(self.best_s)
        while self.pos < len(self.tmax):
            if self.scaled[self.pos] >= best_cost:  # inter_tuning.py:196-197
                return best_cost, best_t, True
            if self.pos >= hi:
                return best_cost, best_t, False     # needs more DP results
            i = self.pos - self.have_lo
            if self.best_s[i] >= 0:
                cost = float(np.float64(self.best_sum[i]) + np.float64(G - 1) * np.float64(self.stage_max[i]))
                if cost < best_cost:
                    best_cost, best_t = cost, self.tmax[self.pos]
            self.pos += 1
        return best_cost, best_t, True


def get_solution_from_intra_stage_tuner_output(
    intra_stage_results, num_layers, gradient_accumulation_steps_index, pre_saved_micro_batches,
    layer_start, layer_end, device_mesh_idx, num_ckpt_layers, slot=0,
):
    """inter_tuning.py:38-60 with the sample slot made explicit."""
    g, q, p, c = gradient_accumulation_steps_index, device_mesh_idx, pre_saved_micro_batches, num_ckpt_layers
    l = layer_end - layer_start + 1
    r = intra_stage_results
    if layer_start == 0 and layer_end == num_layers - 1:
        return r.solution_at(3, (g, q, c, slot))
    if layer_start == 0:
        return r.solution_at(1, (g, q, p, l - 1, c, slot))
    if layer_end == num_layers - 1:
        return r.solution_at(2, (g, q, l - 1, c, slot))
    return r.solution_at(0, (g, q, p, l - 1, c, slot))


def _same_batch(results_list) -> bool:
    first = results_list[0]
    return all(
        r.batch is first.batch and r.batch_index == i for i, r in enumerate(results_list)
    ) and first.batch.stable[0].shape[0] == len(results_list) * len(first.gradient_accumulation_steps_candidates)


def inter_stage_tune_batch(
    num_layers: int,
    num_devices: int,
    device_mesh_candidates: List[Tuple[int, int]],
    gradient_accumulation_steps_candidates: List[int],
    results_list: List[IntraStageTunerOutput],
    slot: int = 0,
    stats: Optional[dict] = None,
):
    """``inter_stage_tune`` for several intra-stage results at once (the tensor-parallel
    candidates of one ``tune`` call).  Each entry is searched exactly as if it were alone (its
    own running best, its own stop rule); only the launches are shared.  Returns a list of
    ``(best_cost, best_solution)``."""
    for r in results_list:
        if not isinstance(r, IntraStageTunerOutput):
            raise TypeError(
                f"intra_stage_results must be an instance of IntraStageTunerOutput, got {type(r)}"
            )
    if not _same_batch(results_list):
        out = []
        for r in results_list:
            one = r if r.batch is r.device else IntraStageTunerOutput(
                r.gradient_accumulation_steps_candidates, r.device_mesh_candidates, r.device,
                r.spaces, r.sample_slots)
            out += inter_stage_tune_batch(num_layers, num_devices, device_mesh_candidates,
                                          gradient_accumulation_steps_candidates, [one], slot, stats)
        return out
    t_start = time.perf_counter()
    first = results_list[0]
    runner = _DpRunner(first, num_layers, num_devices, device_mesh_candidates, slot)
    n_g = len(first.gradient_accumulation_steps_candidates)
    g_index = {G: i for i, G in enumerate(first.gradient_accumulation_steps_candidates)}
    q_index = {q: i for i, q in enumerate(first.device_mesh_candidates)}
    Gs = list(gradient_accumulation_steps_candidates)
    n_inst = len(results_list)
    # table row of (instance, G)
    rows = np.array([[t * n_g + g_index[G] for G in Gs] for t in range(n_inst)], dtype=np.int32)
    t_0 = time.perf_counter()
    tmax_all = runner.thresholds()
    t_1 = time.perf_counter()

    # Smallest feasible threshold of every (instance, G) in one launch (bottleneck DP).
    flat = rows.reshape(-1)
    _, bottleneck, _ = runner.run(flat, np.zeros(len(flat), dtype=np.float32), _lib.DP_BOTTLENECK)
    bottleneck = bottleneck.reshape(rows.shape)
    chains = []
    for t in range(n_inst):
        scans = []
        for i, G in enumerate(Gs):
            tmax = tmax_all[rows[t, i]]
            b = bottleneck[t, i]
            start = int(np.searchsorted(tmax, b, side="left")) if np.isfinite(b) else len(tmax)
            scans.append(_Scan(G, tmax, start))
        chains.append(dict(scans=scans, current=0, best=(float("inf"), None, None)))

    # Speculative batches + sequential replay (see the module docstring).
    while True:
        req_g, req_t, req_span = [], [], []
        for t, ch in enumerate(chains):
            scans = ch["scans"]
            best_cost, best_G, best_t = ch["best"]
            while ch["current"] < len(scans):  # commit the sequential scan as far as results allow
                sc = scans[ch["current"]]
                cost, tt, finished = sc.replay(best_cost, None)
                if tt is not None:
                    best_cost, best_G, best_t = cost, sc.G, tt
                if not finished:
                    break
                ch["current"] += 1
            ch["best"] = (best_cost, best_G, best_t)
            for i in range(ch["current"], len(scans)):
                sc = scans[i]
                if i > ch["current"] and not sc.runs_out(best_cost):
                    continue
                a, b = sc.wanted(best_cost)
                if b > a:
                    req_g.append(np.full(b - a, rows[t, i], dtype=np.int32))
                    req_t.append(sc.tmax[a:b])
                    req_span.append((t, i, b - a))
        if all(ch["current"] == len(ch["scans"]) for ch in chains):
            break
        if not req_span:
            raise RuntimeError("inter-stage scan made no progress")  # cannot happen: guards a hang
        bs, bsum, smax = runner.run(np.concatenate(req_g), np.concatenate(req_t))
        off = 0
        for t, i, n in req_span:
            chains[t]["scans"][i].add(bs[off:off + n], bsum[off:off + n], smax[off:off + n])
            off += n
    t_2 = time.perf_counter()

    # Back-pointers of each winning (G, t_max) run (inter_tuning.py:341-355), one launch.
    winners = [t for t, ch in enumerate(chains) if ch["best"][1] is not None]
    back = {}
    if winners:
        w_rows = np.array([t * n_g + g_index[chains[t]["best"][1]] for t in winners], dtype=np.int32)
        w_tmax = np.array([chains[t]["best"][2] for t in winners], dtype=np.float32)
        best_s, _, _, argmin = runner.run(w_rows, w_tmax, want_argmin=True)
        back = {t: (int(best_s[i]), argmin[i]) for i, t in enumerate(winners)}
    out = []
    for t, ch in enumerate(chains):
        best_cost, best_G, best_t = ch["best"]
        if best_G is None:
            out.append((float("inf"), None))
            continue
        r = results_list[t]
        g = g_index[best_G]
        cs, argmin = back[t]
        cl, cd = 0, num_devices
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
                r, num_layers, g, len(inter) - i - 1, l0, l1, q_index[(n, m)], ckpt, slot
            ).tolist()
            row[:6] = [int(x) for x in row[:6]]
            solution[1].append((((l0, l1), (n, m), ckpt, 0), tuple(row)))
        out.append((best_cost, solution))
    if stats is not None:
        stats["dp_setup_s"] = stats.get("dp_setup_s", 0.0) + (t_0 - t_start)
        stats["dp_thresholds_s"] = stats.get("dp_thresholds_s", 0.0) + (t_1 - t_0)
        stats["dp_scan_s"] = stats.get("dp_scan_s", 0.0) + (t_2 - t_1)
        stats["dp_backtrack_s"] = stats.get("dp_backtrack_s", 0.0) + (time.perf_counter() - t_2)
        stats["dp_launches"] = stats.get("dp_launches", 0) + runner.launches
        stats["dp_thresholds"] = stats.get("dp_thresholds", 0) + runner.thresholds_run
    return out


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
    return inter_stage_tune_batch(
        num_layers, num_devices, device_mesh_candidates, gradient_accumulation_steps_candidates,
        [intra_stage_results], slot, stats,
    )[0]
