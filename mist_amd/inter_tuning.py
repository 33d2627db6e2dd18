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
replay asks for more wherever it runs out, so a wrong guess costs time, never correctness;
(3) thresholds that cannot improve the running best are passed without their outcomes, by a
lower bound of their totals from the stage-cost sum at a later threshold (``_Scan``).

The reference's DP reads ``costs / costs_with_pre / ...`` fields that its intra tuner no longer
emits; the cost tables are built from the stable / delta tables as
``float32(stable) + float32(delta) / G`` (see ``mist_dp_cost_tables``), sample slot 0 by
default, and stage solutions carry a trailing policy index 0 so that ``best_solution_yaml``
accepts them.
"""
from __future__ import annotations

import bisect
import ctypes
import time
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from . import _lib
from .intra_tuning import IntraStageTunerOutput

FIRST_CHUNK = 48  # thresholds per G in the first speculative scan launch ...
FIRST_LEAD = 16   # ... of a window longer than that: the first ones, the rest spread up to its last
PROBES = 16       # thresholds spread over what a later request does not reach
FLOOR_SLACK = 1e-6  # relative slack of the bound that lets the scan pass thresholds
MAX_CHUNK = 4096  # most thresholds per G in one launch
GAP = 1e-6        # inter_tuning.py:177
_SELECT_HEAD = 1 << 16  # selected candidates read back together with their counts
NATIVE_SEARCH = True     # search through mist_inter_stage_search_families (False: the Python driver below)


def _stream(device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class _DpFamily:
    """One recurrence the DP kernel can run: a MistDpShape plus the cost tables it reads."""

    def __init__(self, shape: np.ndarray, costs_struct, consumes_devices: bool):
        self.shape, self.costs_struct, self.consumes_devices = shape, costs_struct, consumes_devices
        self.L, self.D = int(shape["num_layers"][0]), int(shape["num_devices"][0])
        self.S_max = int(shape["max_stages"][0])
        self.plane = (self.L + 1) * (self.D + 1)


class _DpRunner:
    """Owns the float32 cost tables of all g and runs batches of DP instances.  A search is made
    of one or more *families* (recurrences): the per-mesh DP has one, the uniform-device DP one
    per admissible stage count; an instance's cost is the smallest family cost, the first
    family winning ties."""

    def __init__(self, results: IntraStageTunerOutput, num_layers: int, num_devices: int,
                 meshes: List[Tuple[int, int]], slot: int, uniform_device: Optional[dict] = None):
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
        problem = np.zeros(1, dtype=_lib.PROBLEM_DTYPE)
        problem["num_layers"], problem["p_dim"], problem["sample_size"] = L, P1, S
        problem["num_grad_accum"], problem["num_mesh"] = Gn, Q
        with torch.cuda.device(self.device):
            # the four cost tables and their running minima: one allocation, eight views
            shapes = [tuple(t.shape[:-1]) for t in dev_tabs.stable]
            sizes = [int(np.prod(sh)) for sh in shapes]
            flat = torch.empty(2 * sum(sizes), dtype=torch.float32, device=self.device)
            starts = np.concatenate(([0], np.cumsum(sizes + sizes))).tolist()
            views = [flat[starts[i]:starts[i + 1]].view(shapes[i % 4]) for i in range(8)]
            self.cost, self.pmin = views[:4], views[4:]
            self._per_q = [sizes[v] // (Gn * Q) for v in range(4)]  # elements per (g, mesh)
            d_G = getattr(dev_tabs, "grad_accum", None)
            if d_G is None or d_G.numel() != Gn:
                d_G = torch.tensor(Gs, dtype=torch.int32, device=self.device)
            out_ptrs = (ctypes.c_void_p * 4)(*[t.data_ptr() for t in self.cost])
            pmin_ptrs = (ctypes.c_void_p * 4)(*[t.data_ptr() for t in self.pmin])
            tabs = dev_tabs.as_struct()
            rc = self.lib.mist_dp_cost_tables(
                ctypes.c_void_p(problem.ctypes.data), ctypes.byref(tabs), d_G.data_ptr(), slot,
                out_ptrs, pmin_ptrs, _stream(self.device),
            )
            _lib.check(rc, "mist_dp_cost_tables")
        if uniform_device is None:
            self.families = [self._per_mesh_family(meshes)]
            # large batches of this family run one workgroup per instance, which reads the row
            # minima in stage-count order (the uniform-device batches are far too small for that)
            self._prepare_stage_minima(self.families[0])
        else:
            self.families = self._uniform_device_families(meshes, **uniform_device)
        self.strategy_index = _lib.StrategyIndex(
            num_layers=L, p_dim=P1, num_mesh=Q, sample_size=S, slot=slot)
        for v in range(4):
            assert dev_tabs.index[v].dtype == torch.int32
            self.strategy_index.index[v] = dev_tabs.index[v].data_ptr()
        for i, (n, m) in enumerate(meshes):
            self.strategy_index.mesh_n[i], self.strategy_index.mesh_m[i] = n, m
        self._tables = dev_tabs  # the pointers above stay valid as long as the runner lives
        self.launches = 0
        self.thresholds_run = 0
        self._all_costs = self._costs_struct()
        self._select_capacity = 1 << 18
        self.fetches = 0
        self.selected = 0

    def _costs_struct(self, q: int = 0):
        """Table pointers starting at mesh ``q`` (strides between g unchanged)."""
        per_q = self._per_q
        ptrs = [t.data_ptr() + 4 * q * per_q[v] for v, t in enumerate(self.cost)]
        ptrs += [t.data_ptr() + 4 * q * per_q[v] for v, t in enumerate(self.pmin)]
        cs = _lib.DpCosts(*ptrs)
        for v in range(4):
            cs.g_stride[v] = per_q[v] * self.Q
        return cs

    def _prepare_stage_minima(self, fam: _DpFamily) -> None:
        """Fills ``MistDpCosts.stage_min`` of a family (``mist_dp_stage_minima``)."""
        shape_ptr = ctypes.c_void_p(fam.shape.ctypes.data)
        per_g = self.lib.mist_dp_stage_minima_floats(shape_ptr)
        if per_g < 0:
            _lib.check(-1, "mist_dp_stage_minima_floats")
        with torch.cuda.device(self.device):
            fam.stage_min = torch.empty((self.Gn, per_g), dtype=torch.float32, device=self.device)
            rc = self.lib.mist_dp_stage_minima(shape_ptr, ctypes.byref(fam.costs_struct), self.Gn,
                                               fam.stage_min.data_ptr(), _stream(self.device))
            _lib.check(rc, "mist_dp_stage_minima")
        fam.costs_struct.stage_min = fam.stage_min.data_ptr()
        fam.costs_struct.stage_min_g_stride = per_g

    def _per_mesh_family(self, meshes) -> _DpFamily:
        shape = np.zeros(1, dtype=_lib.DP_SHAPE_DTYPE)
        shape["num_layers"], shape["num_devices"] = self.L, self.D
        shape["num_mesh"], shape["p_dim"] = self.Q, self.P1
        shape["max_stages"] = min(max(n * m for n, m in meshes), self.L) // 2  # inter_tuning.py:278-280
        shape["ckpt_rule"] = _lib.DP_CKPT_TAIL
        shape["mesh_n"][0, :self.Q] = [n for n, _ in meshes]
        shape["mesh_m"][0, :self.Q] = [m for _, m in meshes]
        return _DpFamily(shape, self._costs_struct(), True)

    def _uniform_device_families(self, meshes, num_nodes, num_gpus_per_node, ckpt_tuning):
        """One family per stage count S whose even split of the cluster is a mesh candidate
        (inter_tuning_uniform_device.py:312-334, 360-367): s <= S stages, all on that mesh."""
        from .inter_tuning_uniform import _uniform_device_mesh_partition

        fams = []
        for S in range(1, self.L + 1):
            mesh = _uniform_device_mesh_partition(S, num_nodes, num_gpus_per_node)
            if mesh is None:
                continue
            if mesh not in meshes:
                raise ValueError(f"uniform mesh {mesh} of {S} stages is not a mesh candidate")
            q = max(i for i, nm in enumerate(meshes) if nm == mesh)
            shape = np.zeros(1, dtype=_lib.DP_SHAPE_DTYPE)
            shape["num_layers"], shape["num_devices"], shape["num_mesh"] = self.L, 0, 1
            shape["p_dim"] = self.P1
            # stage counts beyond the p axis of the tables cost +inf (the reference indexes out
            # of bounds there), so they need not be run
            shape["max_stages"] = min(S, self.P1, self.L)
            shape["ckpt_rule"] = _lib.DP_CKPT_STAGE if ckpt_tuning else _lib.DP_CKPT_ALL
            shape["free_devices"] = 1
            shape["mesh_n"][0, 0], shape["mesh_m"][0, 0] = mesh
            fams.append(_DpFamily(shape, self._costs_struct(q), False))
        return fams

    def candidates_between_flat(self, rows: np.ndarray, lo: np.ndarray, hi: np.ndarray):
        """Per requested table row g: the ascending t_max candidates v (finite stage costs of the
        costs / with_pre / with_post tables, inter_tuning.py:180-186) with lo < v <= hi (lo = -inf
        includes everything below), and how many finite candidates lie above hi.  One kernel
        pass over the requested rows; only the selected values come back: ``(values, bounds,
        above)`` with request i owning ``values[bounds[i]:bounds[i + 1]]``."""
        dev = self.device
        self.fetches += 1
        n = len(rows)
        with torch.cuda.device(dev):
            req = np.empty((3, n), dtype=np.float32)
            req[0].view(np.int32)[:] = rows
            req[1], req[2] = lo, hi
            d_req = torch.from_numpy(req).to(dev)
            capacity = self._select_capacity
            while True:
                counts = torch.zeros(1 + n, dtype=torch.int32, device=dev)
                values = torch.empty(capacity, dtype=torch.float32, device=dev)
                request = torch.empty(capacity, dtype=torch.int32, device=dev)
                # the first values and requests travel with the counts (one read-back when
                # they are all there is, which is the usual case)
                head = min(capacity, _SELECT_HEAD)
                rc = self.lib.mist_dp_select_candidates(
                    ctypes.byref(self._all_costs), n, d_req[0].data_ptr(), d_req[1].data_ptr(),
                    d_req[2].data_ptr(), values.data_ptr(), request.data_ptr(), capacity,
                    counts.data_ptr(), _stream(dev))
                _lib.check(rc, "mist_dp_select_candidates")
                packed = torch.cat([counts.view(torch.float32), values[:head],
                                    request[:head].view(torch.float32)]).cpu().numpy()
                h_counts = packed[:1 + n].view(np.int32)
                total = int(h_counts[0])
                if total <= capacity:
                    break
                capacity = self._select_capacity = 2 * total
            if total <= head:
                h_values = packed[1 + n:1 + n + total]
                h_request = packed[1 + n + head:1 + n + head + total].view(np.int32)
            else:
                h_values = values[:total].cpu().numpy()
                h_request = request[:total].cpu().numpy()
        self.selected += total
        # group by request: 16-bit keys (the entry point takes at most 65535 requests) make the
        # stable sort a radix sort
        order = np.argsort(h_request.astype(np.uint16), kind="stable")
        h_values, h_request = h_values[order], h_request[order]
        bounds = np.searchsorted(h_request, np.arange(n + 1)).astype(np.int64)
        for i in range(n):
            h_values[bounds[i]:bounds[i + 1]].sort()
        return h_values, bounds, h_counts[1:]

    def candidates_between(self, rows: np.ndarray, lo: np.ndarray, hi: np.ndarray):
        """``candidates_between_flat`` as one ``(ascending values, candidates above hi)`` pair
        per requested row."""
        values, bounds, above = self.candidates_between_flat(rows, lo, hi)
        return [(values[bounds[i]:bounds[i + 1]], int(above[i])) for i in range(len(above))]

    def filter_gap(self, ascending: np.ndarray) -> np.ndarray:
        """The reference's gap rule (inter_tuning.py:198) applied from the first element on
        (which is kept); duplicates have a zero difference to the last kept value."""
        ascending = np.ascontiguousarray(ascending, dtype=np.float32)
        kept = np.empty(len(ascending), dtype=np.float32)
        n = self.lib.mist_dp_filter_tmax(
            ctypes.c_void_p(ascending.ctypes.data), len(ascending), GAP,
            ctypes.c_void_p(kept.ctypes.data))
        return kept[:n]

    def run(self, g_index: np.ndarray, tmax: np.ndarray, mode: int = _lib.DP_THRESHOLD,
            want_argmin: bool = False, family: Optional[_DpFamily] = None,
            want_path: bool = False):
        """DP instances (g_index[i], tmax[i]) of one family -> (best_s int32, best_sum f32,
        stage_max f32 [, argmin] [, path]).  ``path`` [n, max_stages, 4]: the stages of each
        instance's partition as (end layer, n, m, ckpt), walked on the GPU."""
        fam = self.families[0] if family is None else family
        n = len(tmax)
        dev = self.device
        with torch.cuda.device(dev):
            packed = np.empty((2, n), dtype=np.float32)
            packed[0] = tmax
            packed[1].view(np.int32)[:] = g_index
            d_in = torch.from_numpy(packed).to(dev)
            # outputs and (if asked for) the walked partitions share a buffer: one read-back
            n_path = n * fam.S_max * 4 if want_path else 0
            d_all = torch.empty(3 * n + n_path, dtype=torch.float32, device=dev)
            d_out = d_all[:3 * n].view(3, n)
            n_scratch = self.lib.mist_dp_scratch_floats(ctypes.c_void_p(fam.shape.ctypes.data), n)
            scratch = torch.empty(n_scratch, dtype=torch.float32, device=dev)
            argmin = None
            arg_shape = (n, fam.S_max + 1, fam.L + 1, fam.D + 1, 4)
            if want_argmin:
                argmin = torch.full(arg_shape, -1, dtype=torch.int32, device=dev)
            elif want_path:  # the walk only reads entries the DP wrote: no fill
                argmin = torch.empty(arg_shape, dtype=torch.int32, device=dev)
            rc = self.lib.mist_dp_run(
                ctypes.c_void_p(fam.shape.ctypes.data), ctypes.byref(fam.costs_struct),
                d_in[0].data_ptr(), d_in[1].data_ptr(), n, mode,
                d_out[0].data_ptr(), d_out[1].data_ptr(), d_out[2].data_ptr(),
                argmin.data_ptr() if argmin is not None else None, scratch.data_ptr(), _stream(dev),
            )
            _lib.check(rc, "mist_dp_run")
            self.launches += 1
            self.thresholds_run += n
            if want_path:
                rc = self.lib.mist_dp_backtrack(
                    ctypes.c_void_p(fam.shape.ctypes.data), argmin.data_ptr(), d_out[0].data_ptr(),
                    n, d_all[3 * n:].data_ptr(), _stream(dev))
                _lib.check(rc, "mist_dp_backtrack")
            host_all = d_all.cpu().numpy()
            host = host_all[:3 * n].reshape(3, n)
            out = (host[0].view(np.int32), host[1], host[2])
            if want_argmin:
                out = out + (argmin.cpu().numpy(),)
            if want_path:
                out = out + (host_all[3 * n:].view(np.int32).reshape(n, fam.S_max, 4),)
        return out

    @staticmethod
    def _total(best_s, best_sum, stage_max, G) -> np.ndarray:
        """``best + (g - 1) * f_stage_max`` in float64 (inter_tuning.py:342), inf if infeasible."""
        total = best_sum.astype(np.float64) + (np.asarray(G, dtype=np.float64) - 1.0) * stage_max.astype(np.float64)
        return np.where(best_s >= 0, total, np.inf)

    def evaluate(self, g_index: np.ndarray, tmax: np.ndarray, G: np.ndarray):
        """Cost of every instance = smallest family total (first family on ties), the family
        that attains it (-1 if none) and the smallest feasible family sum."""
        cost = np.full(len(tmax), np.inf)
        winner = np.full(len(tmax), -1, dtype=np.int32)
        min_sum = np.full(len(tmax), np.inf)
        for f, fam in enumerate(self.families):
            bs, bsum, smax = self.run(g_index, tmax, family=fam)
            total = self._total(bs, bsum, smax, G)
            better = total < cost
            cost = np.where(better, total, cost)
            winner = np.where(better, f, winner)
            min_sum = np.minimum(min_sum, np.where(bs >= 0, bsum.astype(np.float64), np.inf))
        return cost, winner, min_sum

    def bottleneck(self, g_index: np.ndarray):
        """Smallest threshold for which any family is feasible (float32, +inf if none) and the
        stage-cost sum of a partition that is admissible there."""
        b = np.full(len(g_index), np.inf, dtype=np.float32)
        path_sum = np.full(len(g_index), np.inf)
        zeros = np.zeros(len(g_index), dtype=np.float32)
        for fam in self.families:
            _, bott, psum = self.run(g_index, zeros, _lib.DP_BOTTLENECK, family=fam)
            better = bott < b
            b = np.where(better, bott, b)
            path_sum = np.where(better, psum.astype(np.float64), path_sum)
        return b, path_sum

    def partitions(self, g_index: np.ndarray, tmax: np.ndarray, G: np.ndarray):
        """Per instance ``(total, [((l0, l1), (n, m), ckpt), ...])`` of its winning family, from
        the back-pointers (inter_tuning.py:341-355); one launch batch per family."""
        n = len(tmax)
        best = [(np.inf, None)] * n
        for fam in self.families:
            bs, bsum, smax, path = self.run(g_index, tmax, family=fam, want_path=True)
            total = self._total(bs, bsum, smax, G)
            for i in range(n):
                if total[i] < best[i][0]:
                    best[i] = (float(total[i]), (fam, int(bs[i]), path[i]))
        out = []
        for total, found in best:
            assert found is not None
            fam, n_stages, path = found
            out.append(self._partition_of(total, fam, n_stages, path))
        return out

    @staticmethod
    def _partition_of(total, fam, n_stages, path):
        """``(total, [((l0, l1), (n, m), ckpt), ...])`` from a walked path (mist_dp_backtrack)."""
        stages = path[:n_stages].tolist()
        cl, cd, inter = 0, fam.D, []
        for end, n_, m_, ckpt in stages:
            assert end >= cl, "back-pointer walk left the DP's states"
            inter.append(((cl, end), (n_, m_), ckpt))
            cl = end + 1
            if fam.consumes_devices:
                cd -= n_ * m_
        assert len(inter) == n_stages and cl == fam.L and (cd == 0 or not fam.consumes_devices)
        return total, inter


def _gap_reached(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """not (a - b < 1e-6) with the reference's arithmetic: float32 difference, float64 compare."""
    return ~((a.astype(np.float32) - b.astype(np.float32)).astype(np.float64) < GAP)


class _Window:
    """Kept t_max candidates of one table row, materialised lazily.

    The reference sorts every finite stage cost and walks the list with the gap rule from the
    bottom (inter_tuning.py:180-198).  Whether a candidate is kept only depends on the last kept
    one, and a candidate whose predecessor is at least the gap below is always kept, so the
    walk can start at such a candidate just below the smallest feasible threshold instead of
    at the bottom; everything below is infeasible and leaves the scan unchanged."""

    def __init__(self, runner: "_DpRunner", row: int, G: int, start_value: float, start_sum: float):
        self.runner, self.row, self.G, self.start_value = runner, row, G, np.float32(start_value)
        # Stage-cost sum of a partition that is admissible at the smallest feasible threshold.
        # At the first kept candidate t_s >= start_value it still is, so the scan's running best
        # is at most start_sum + (G - 1) * t_s once it has looked at t_s; candidates with t * G
        # beyond that are never reached.
        self.start_sum = float(start_sum)
        self.bound = float("inf")
        self.kept = np.empty(0, dtype=np.float32)
        self.scaled = np.empty(0, dtype=np.float64)
        self.hi = None          # every candidate <= hi has been walked
        self.complete = False   # no finite candidate above hi

    def lower_margin(self, widen: int) -> np.float32:
        return np.float32(self.start_value - (1e-4 + 1e-5 * abs(float(self.start_value))) * 4.0 ** widen)

    def begin(self, values: np.ndarray, n_above: int, lo: np.float32, hi: np.float32) -> bool:
        """First fetch: ``values`` = ascending candidates in (lo, hi].  Returns False if no
        certain start of the walk lies in the fetched part (the caller widens ``lo``).  The
        start is found and the walk done by ``mist_dp_window_begin``."""
        self.hi, self.complete = hi, n_above == 0
        if len(values) == 0:
            return True
        below = bool(np.isneginf(lo))
        values = np.ascontiguousarray(values, dtype=np.float32)
        kept = np.empty(len(values), dtype=np.float32)
        n = self.runner.lib.mist_dp_window_begin(
            ctypes.c_void_p(values.ctypes.data), len(values), 0.0 if below else float(lo),
            1 if below else 0, float(self.start_value), GAP, ctypes.c_void_p(kept.ctypes.data))
        if n == _lib.DP_NO_START:
            return False
        if n < 0:
            _lib.check(n, "mist_dp_window_begin")
        self._append(kept[:n])
        return True

    @staticmethod
    def begin_many(windows, values: np.ndarray, bounds: np.ndarray, above: np.ndarray,
                   lo: np.ndarray, hi: np.ndarray) -> List[bool]:
        """``begin`` of several windows on the flat result of one fetch (one library call)."""
        if not windows:
            return []
        n = len(windows)
        lib = windows[0].runner.lib
        values = np.ascontiguousarray(values, dtype=np.float32)
        bounds = np.ascontiguousarray(bounds, dtype=np.int64)
        below = np.isneginf(lo)
        lo_arg = np.where(below, np.float32(0.0), lo).astype(np.float32)
        open_below = below.astype(np.uint8)
        start = np.array([w.start_value for w in windows], dtype=np.float32)
        kept = np.empty(len(values), dtype=np.float32)
        count = np.empty(n, dtype=np.int32)
        rc = lib.mist_dp_window_begin_many(
            ctypes.c_void_p(values.ctypes.data), ctypes.c_void_p(bounds.ctypes.data), n,
            ctypes.c_void_p(lo_arg.ctypes.data), ctypes.c_void_p(open_below.ctypes.data),
            ctypes.c_void_p(start.ctypes.data), GAP, ctypes.c_void_p(kept.ctypes.data),
            ctypes.c_void_p(count.ctypes.data))
        _lib.check(rc, "mist_dp_window_begin_many")
        done = []
        for j, w in enumerate(windows):
            w.hi, w.complete = hi[j], above[j] == 0
            if count[j] == _lib.DP_NO_START:
                done.append(False)
                continue
            if count[j] > 0:
                w._append(kept[bounds[j]:bounds[j] + count[j]])
            done.append(True)
        return done

    def _append(self, kept: np.ndarray) -> None:
        self.kept = np.concatenate([self.kept, kept])
        # float32 scalar * python int is float64 under the reference's numpy 1.24.
        self.scaled = self.kept.astype(np.float64) * self.G
        if not np.isfinite(self.bound):
            i = int(np.searchsorted(self.kept, self.start_value, side="left"))
            if i < len(self.kept):
                self.bound = self.start_sum + (self.G - 1) * float(self.kept[i])

    def covers(self, best_cost: float) -> bool:
        """True if every kept candidate the scan can reach under the running best ``best_cost``
        is materialised."""
        need = min(best_cost, self.bound)
        return self.complete or float(np.float64(self.hi) * self.G) >= need

    def extension_target(self, best_cost: float) -> np.float32:
        # at least a geometric step, so that repeated calls end (an unbounded best_cost, i.e. no
        # solution yet, asks for "more" rather than for everything)
        want = np.float32(self.hi + max(16 * (abs(self.hi) * 1e-4 + 1e-4),
                                        2.0 * abs(float(self.hi) - float(self.start_value))))
        need = min(best_cost, self.bound)
        if np.isfinite(need):
            want = max(want, np.nextafter(np.float32(need / self.G), np.float32(np.inf)))
        return want

    def apply_extension(self, values: np.ndarray, n_above: int, want: np.float32) -> None:
        """``values`` = ascending candidates in (hi, want]."""
        if len(self.kept):
            # continue the walk from the last kept candidate: put it in front and drop it again
            values = self.runner.filter_gap(np.concatenate((self.kept[-1:], values)))[1:]
        else:
            values = self.runner.filter_gap(values)
        self.hi, self.complete = want, n_above == 0
        self._append(values)

    def extend(self, best_cost: float) -> None:
        want = self.extension_target(best_cost)
        (values, n_above), = self.runner.candidates_between(
            np.array([self.row]), np.array([self.hi], dtype=np.float32),
            np.array([want], dtype=np.float32))
        self.apply_extension(values, n_above, want)


class _Scan:
    """Replay state of ``inter_stage_tune_with_fixed_grad_accumu`` (inter_tuning.py:163-217) for
    one G: ``pos`` = next threshold the sequential scan would look at, ``known`` = DP outcomes
    (total, smallest family sum) by index of the kept threshold.

    The reference runs the DP at every kept threshold below ``best / G``.  Most of those runs
    change nothing, and for many that can be told from the outcome at a LATER threshold j: the
    DP at threshold i returns the partition the DP at i - 1 returned unless that one uses a
    stage cost above threshold i - 1 (same visiting order, strict "<"), and the same partition
    gives the same total, which is no improvement.  A partition that is new at i has a stage
    above threshold i - 1 and stage costs that sum to no less than the smallest sum at j >= i
    (the admissible costs only grow with the threshold; float32 adds are monotone), so its total
    is at least ``sum(j) + (G - 1) * threshold(i - 1)``.  While that is no smaller than the
    running best, no threshold up to j improves it and the scan passes them."""

    def __init__(self, G: int, window: Optional[_Window], first: int, first_index=None):
        self.G, self.window = G, window
        self.pos = first          # everything below is infeasible: the scan passes it unchanged
        self.first = first
        self.known: Dict[int, Tuple[float, float]] = {}
        self.keys: List[int] = []  # sorted indices of ``known``
        self.limit = FIRST_CHUNK
        self.first_index = first_index  # mist_dp_first_batch_index

    @property
    def tmax(self) -> np.ndarray:
        return self.window.kept if self.window is not None else np.empty(0, dtype=np.float32)

    @property
    def scaled(self) -> np.ndarray:
        return self.window.scaled if self.window is not None else np.empty(0, dtype=np.float64)

    def _reach(self, pos: int, best_cost: float) -> bool:
        """Makes sure threshold ``pos`` is materialised if the scan can get there; False if the
        scan ends before it."""
        w = self.window
        while w is not None and pos >= len(w.kept) and not w.covers(best_cost):
            w.extend(best_cost)
        return pos < len(self.tmax)

    def _floor_total(self, at: int, sum_later: float) -> float:
        """Lower bound of the total of any improvement at thresholds ``at``..j, from the sum at j."""
        prev = float(self.tmax[at - 1]) if at > self.first else float(self.window.start_value)
        return (sum_later + (self.G - 1) * prev) * (1.0 - FLOOR_SLACK)

    def _later(self, pos: int) -> Optional[int]:
        k = bisect.bisect_left(self.keys, pos)
        return self.keys[k] if k < len(self.keys) else None

    def wanted(self, best_cost: float) -> List[int]:
        """Dry run of ``replay`` under the bound ``best_cost`` (the true running best when this G
        is reached is no larger, so the true scan passes no fewer thresholds): the thresholds
        whose outcomes it would miss, at most ``limit`` of them (it goes on as if they improved
        nothing), and, if it stops at that limit, ``PROBES`` more spread over what it did not get
        to.  A scan without any outcome asks for its first batch."""
        if self.window is None:
            return []
        if not self.known:
            self._reach(self.pos + FIRST_CHUNK, best_cost)
            stop = int(np.searchsorted(self.scaled, best_cost, side="left"))
            if stop <= self.pos:
                return []
            n_avail = stop - self.pos
            return [self.pos + self.first_index(k, n_avail, FIRST_CHUNK, FIRST_LEAD)
                    for k in range(min(FIRST_CHUNK, n_avail))]
        out, pos, budget, cut = [], self.pos, self.limit, False
        while self._reach(pos, best_cost):
            if self.scaled[pos] >= best_cost:
                break
            later = self._later(pos)
            if later is not None and self._floor_total(pos, self.known[later][1]) >= best_cost:
                pos = later + 1
                continue
            if later == pos:
                best_cost = min(best_cost, self.known[pos][0])
            else:
                if budget == 0:
                    cut = True
                    break
                out.append(pos)
                budget -= 1
            pos += 1
        if cut:
            stop = int(np.searchsorted(self.scaled, best_cost, side="left"))
            last = 0
            for k in range(PROBES):
                if stop <= pos:
                    break
                at = pos + ((k + 1) * (stop - pos)) // PROBES - 1
                if at < pos or (k > 0 and at <= last) or at in self.known:
                    continue
                out.append(at)
                last = at
        return out

    def add(self, at: List[int], cost: np.ndarray, sums: np.ndarray):
        for i, c, s in zip(at, cost.tolist(), sums.tolist()):
            if i not in self.known:
                bisect.insort(self.keys, i)
            self.known[i] = (c, s)

    def replay(self, best_cost: float, best_t):
        """Advances the sequential scan as far as the computed results allow.  Returns
        (best_cost, best_t, finished)."""
        while self._reach(self.pos, best_cost):
            if self.scaled[self.pos] >= best_cost:  # inter_tuning.py:196-197
                return best_cost, best_t, True
            later = self._later(self.pos)
            if later is not None and self._floor_total(self.pos, self.known[later][1]) >= best_cost:
                self.pos = later + 1  # nothing up to there improves the best
                continue
            if later != self.pos:
                return best_cost, best_t, False     # needs more DP results
            cost = self.known[self.pos][0]
            if cost < best_cost:
                best_cost, best_t = cost, self.tmax[self.pos]
            self.pos += 1
        return best_cost, best_t, True


def _solution_cell(num_layers, g, p, layer_start, layer_end, q, c, slot=0):
    """Table variant and cell of a stage's strategy (inter_tuning.py:38-60 with the sample slot
    made explicit)."""
    l = layer_end - layer_start + 1
    if layer_start == 0 and layer_end == num_layers - 1:
        return 3, (g, q, c, slot)
    if layer_start == 0:
        return 1, (g, q, p, l - 1, c, slot)
    if layer_end == num_layers - 1:
        return 2, (g, q, l - 1, c, slot)
    return 0, (g, q, p, l - 1, c, slot)


def get_solution_from_intra_stage_tuner_output(
    intra_stage_results, num_layers, gradient_accumulation_steps_index, pre_saved_micro_batches,
    layer_start, layer_end, device_mesh_idx, num_ckpt_layers, slot=0,
):
    """inter_tuning.py:38-60."""
    variant, cell = _solution_cell(
        num_layers, gradient_accumulation_steps_index, pre_saved_micro_batches, layer_start,
        layer_end, device_mesh_idx, num_ckpt_layers, slot)
    return intra_stage_results.solution_at(variant, cell)


def _same_batch(results_list) -> bool:
    first = results_list[0]
    return all(
        r.batch is first.batch and r.batch_index == i for i, r in enumerate(results_list)
    ) and first.batch.stable[0].shape[0] == len(results_list) * len(first.gradient_accumulation_steps_candidates)


def _search(runner: _DpRunner, rows: np.ndarray, Gs: List[int], stats: Optional[dict]):
    """The reference's scan (G after G, ascending kept thresholds, stop rule, strict "<";
    inter_tuning.py:163-217 and :119-143) for ``rows.shape[0]`` independent instances whose
    table row for G index i is ``rows[t, i]``.  Returns per instance ``(best_cost, G, t_max)``
    (``G`` None if nothing is feasible)."""
    n_inst = rows.shape[0]
    t_0 = time.perf_counter()

    # Smallest feasible threshold of every (instance, G) in one batch (bottleneck DP), then one
    # threshold DP there: its cost bounds how far up the scan of that G can get.
    flat = rows.reshape(-1)
    flat_G = np.tile(np.array(Gs, dtype=np.int64), n_inst)
    bottleneck, path_sum = runner.bottleneck(flat)
    feasible = np.isfinite(bottleneck)
    windows: List[Optional[_Window]] = [None] * len(flat)
    if feasible.any():
        idx = np.nonzero(feasible)[0]
        # the min-max partition is admissible at the bottleneck: its total bounds the scan's best
        sum0 = path_sum[idx]
        cost0 = sum0 + (flat_G[idx] - 1).astype(np.float64) * bottleneck[idx].astype(np.float64)
        # The scan's bound uses the first KEPT candidate at or above the bottleneck, which the gap
        # rule can push up by a few gaps: leave room for that, or the window needs a second fetch.
        room = (flat_G[idx] - 1).astype(np.float64) * (4 * GAP)
        hi = np.nextafter(((cost0 + room) * (1.0 + 1e-5) / flat_G[idx]).astype(np.float32), np.float32(np.inf))
        # ... and when the smallest feasible threshold is no candidate itself (a single-stage
        # cost is none), the first candidate above it lies a little further up
        hi = np.maximum(hi, (bottleneck[idx].astype(np.float64) * (1.0 + 2e-3) + 2e-4).astype(np.float32))
        for k, i in enumerate(idx):
            windows[i] = _Window(runner, int(flat[i]), int(flat_G[i]), bottleneck[i], float(sum0[k]))
        pending, widen = list(range(len(idx))), 0
        while pending:
            lo = np.array([windows[idx[k]].lower_margin(widen) for k in pending], dtype=np.float32)
            if widen >= 8:
                lo[:] = -np.inf
            values, bounds, above = runner.candidates_between_flat(flat[idx[pending]], lo, hi[pending])
            done = _Window.begin_many([windows[idx[k]] for k in pending], values, bounds, above,
                                      lo, hi[pending])
            pending = [k for k, ok in zip(pending, done) if not ok]
            widen += 1
        # one more pass for the windows whose first kept candidate turned out to lie higher
        # than assumed (the remaining cases extend one by one while the scan runs)
        short = [windows[i] for i in idx if not windows[i].covers(float("inf"))]
        if short:
            want = np.array([w.extension_target(float("inf")) for w in short], dtype=np.float32)
            got = runner.candidates_between(
                np.array([w.row for w in short]), np.array([w.hi for w in short], dtype=np.float32), want)
            for w, (values, n_above), hi_w in zip(short, got, want):
                w.apply_extension(values, n_above, hi_w)
    t_1 = time.perf_counter()
    chains = []
    for t in range(n_inst):
        scans = []
        for i, G in enumerate(Gs):
            w = windows[t * len(Gs) + i]
            start = int(np.searchsorted(w.kept, w.start_value, side="left")) if w is not None else 0
            scans.append(_Scan(G, w, start, runner.lib.mist_dp_first_batch_index))
        chains.append(dict(scans=scans, current=0, best=(float("inf"), None, None)))

    # Speculative batches + sequential replay (see the module docstring).
    while True:
        req_g, req_t, req_G, req_span = [], [], [], []  # (spans: instance, G index, threshold indices)
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
                at = sc.wanted(best_cost)
                if at:
                    # the range grows fourfold every time the same G asks again
                    sc.limit = min(MAX_CHUNK, sc.limit * 4)
                    req_g.append(np.full(len(at), rows[t, i], dtype=np.int32))
                    req_t.append(sc.tmax[at])
                    req_G.append(np.full(len(at), sc.G, dtype=np.int64))
                    req_span.append((t, i, at))
        if all(ch["current"] == len(ch["scans"]) for ch in chains):
            break
        if not req_span:
            raise RuntimeError("inter-stage scan made no progress")  # cannot happen: guards a hang
        cost, _, sums = runner.evaluate(np.concatenate(req_g), np.concatenate(req_t), np.concatenate(req_G))
        off = 0
        for t, i, at in req_span:
            chains[t]["scans"][i].add(at, cost[off:off + len(at)], sums[off:off + len(at)])
            off += len(at)
    t_2 = time.perf_counter()
    if stats is not None:
        stats["dp_thresholds_s"] = stats.get("dp_thresholds_s", 0.0) + (t_1 - t_0)
        stats["dp_scan_s"] = stats.get("dp_scan_s", 0.0) + (t_2 - t_1)
    return [ch["best"] for ch in chains]


def _solutions(runner: _DpRunner, results_list, bests, n_g, g_index, q_index, num_layers, slot,
               only_best=False):
    """Back-pointers of each winning (G, t_max) run (inter_tuning.py:341-355) and the stage
    strategies that go with them.  ``only_best``: only the instance with the smallest cost (the
    first of them) gets its solution; the others report their cost with ``None``."""
    winners = [t for t, (_, best_G, _) in enumerate(bests) if best_G is not None]
    if only_best and winners:
        winners = [min(winners, key=lambda t: bests[t][0])]  # min() keeps the first of equals
    found = {}
    if winners:
        parts = runner.partitions(
            np.array([t * n_g + g_index[bests[t][1]] for t in winners], dtype=np.int32),
            np.array([bests[t][2] for t in winners], dtype=np.float32),
            np.array([bests[t][1] for t in winners], dtype=np.int64))
        found = dict(zip(winners, parts))
    # strategy rows of all stages of all winners: one read-back
    requests = []
    for t in winners:
        g = g_index[bests[t][1]]
        inter = found[t][1]
        for i, ((l0, l1), (n, m), ckpt) in enumerate(inter):
            variant, cell = _solution_cell(num_layers, g, len(inter) - i - 1, l0, l1, q_index[(n, m)], ckpt, slot)
            requests.append((results_list[t], variant, cell))
    rows = iter(IntraStageTunerOutput.solutions_at(requests)) if requests else iter(())
    out = []
    for t, (best_cost, best_G, best_t) in enumerate(bests):
        if best_G is None:
            out.append((float("inf"), None))
            continue
        if t not in found:
            out.append((best_cost, None))
            continue
        total, inter = found[t]
        assert total == best_cost
        solution = [best_G, []]
        for (l0, l1), (n, m), ckpt in inter:
            row = next(rows).tolist()
            row[:6] = [int(x) for x in row[:6]]
            solution[1].append((((l0, l1), (n, m), ckpt, 0), tuple(row)))
        out.append((best_cost, solution))
    return out


def _native_search(runner: _DpRunner, results_list, rows, Gs, n_g, g_index, q_index, num_layers,
                   slot, only_best, stats, table_limit=None):
    """The search of ``_search`` + the partitions and strategy rows of ``_solutions`` in one
    library call (``mist_inter_stage_search_families``: the same steps without the interpreter
    between the dependent GPU batches, for the per-mesh family or the uniform-device families
    of ``runner``); only the decoding of the strategy rows happens here."""
    fams = runner.families
    n_inst = len(results_list)
    rows = np.ascontiguousarray(rows, dtype=np.int32)
    G_arr = np.array(Gs, dtype=np.int32)
    shapes = np.concatenate([f.shape for f in fams])
    costs = (_lib.DpCosts * len(fams))()
    for i, f in enumerate(fams):
        ctypes.memmove(ctypes.byref(costs[i]), ctypes.byref(f.costs_struct), ctypes.sizeof(_lib.DpCosts))
    select = fams[0].costs_struct if len(fams) == 1 and fams[0].consumes_devices else runner._all_costs
    s_max = max(f.S_max for f in fams)
    cost = np.empty(n_inst, dtype=np.float64)
    best_g = np.empty(n_inst, dtype=np.int32)
    best_t = np.empty(n_inst, dtype=np.float32)
    family = np.empty(n_inst, dtype=np.int32)
    n_stages = np.empty(n_inst, dtype=np.int32)
    path = np.empty((n_inst, s_max, 4), dtype=np.int32)
    strategy_row = np.empty((n_inst, s_max), dtype=np.int32)
    counters = np.zeros(6, dtype=np.int64)
    t_0 = time.perf_counter()
    arguments = [
        len(fams), ctypes.c_void_p(shapes.ctypes.data), ctypes.cast(costs, ctypes.c_void_p),
        ctypes.byref(select), ctypes.byref(runner.strategy_index), n_inst, len(Gs),
        ctypes.c_void_p(rows.ctypes.data), ctypes.c_void_p(G_arr.ctypes.data),
        1 if only_best else 0, ctypes.c_void_p(cost.ctypes.data),
        ctypes.c_void_p(best_g.ctypes.data), ctypes.c_void_p(best_t.ctypes.data),
        ctypes.c_void_p(family.ctypes.data), ctypes.c_void_p(n_stages.ctypes.data),
        ctypes.c_void_p(path.ctypes.data), ctypes.c_void_p(strategy_row.ctypes.data),
        ctypes.c_void_p(counters.ctypes.data), _stream(runner.device)]
    unresolved = np.zeros(1, dtype=np.int32)
    with torch.cuda.device(runner.device):
        if table_limit is None:
            rc = runner.lib.mist_inter_stage_search_families(*arguments)
        else:
            # the tables hold their values up to estimate * factor / G only (``table_limit`` =
            # the estimate as a pinned host tensor that the stream fills, and the factor)
            rc = runner.lib.mist_inter_stage_search_bounded(
                *arguments, ctypes.c_void_p(table_limit[0].data_ptr()), float(table_limit[1]),
                ctypes.c_void_p(unresolved.ctypes.data))
    _lib.check(rc, "mist_inter_stage_search_families")
    if stats is not None:
        stats["dp_unresolved"] = stats.get("dp_unresolved", 0) + int(unresolved[0])
    t_1 = time.perf_counter()
    out = []
    for t in range(n_inst):
        if best_g[t] < 0:
            out.append((float("inf"), None))
            continue
        if n_stages[t] <= 0:
            out.append((float(cost[t]), None))
            continue
        fam = fams[int(family[t])]
        _, inter = _DpRunner._partition_of(float(cost[t]), fam, int(n_stages[t]), path[t, :fam.S_max])
        G = Gs[int(best_g[t])]
        spaces = results_list[t].spaces
        solution = [G, [None] * len(inter)]
        # the stages of a partition mostly share a mesh: one decode per search space
        by_space: Dict[Tuple[int, int], List[int]] = {}
        for i, (_, mesh, _) in enumerate(inter):
            by_space.setdefault((g_index[G], q_index[mesh]), []).append(i)
        for key, stages in by_space.items():
            rows = spaces[key].decode(strategy_row[t, stages].astype(np.int64)).tolist()
            for i, row in zip(stages, rows):
                row[:6] = [int(x) for x in row[:6]]
                (l0, l1), mesh, ckpt = inter[i]
                solution[1][i] = (((l0, l1), mesh, ckpt, 0), tuple(row))
        out.append((float(cost[t]), solution))
    if stats is not None:
        stats["dp_search_s"] = stats.get("dp_search_s", 0.0) + (t_1 - t_0)
        stats["dp_backtrack_s"] = stats.get("dp_backtrack_s", 0.0) + (time.perf_counter() - t_1)
        stats["dp_launches"] = stats.get("dp_launches", 0) + int(counters[0])
        stats["dp_window_fetches"] = stats.get("dp_window_fetches", 0) + int(counters[1])
        stats["dp_window_values"] = stats.get("dp_window_values", 0) + int(counters[2])
        stats["dp_thresholds"] = stats.get("dp_thresholds", 0) + int(counters[3])
        stats["dp_round_trips"] = stats.get("dp_round_trips", 0) + int(counters[4])
        stats["dp_windows_left_to_host"] = stats.get("dp_windows_left_to_host", 0) + int(counters[5])
    return out


def inter_stage_tune_batch(
    num_layers: int,
    num_devices: int,
    device_mesh_candidates: List[Tuple[int, int]],
    gradient_accumulation_steps_candidates: List[int],
    results_list: List[IntraStageTunerOutput],
    slot: int = 0,
    stats: Optional[dict] = None,
    uniform_device: Optional[dict] = None,
    only_best_solution: bool = False,
    table_limit=None,
):
    """``inter_stage_tune`` for several intra-stage results at once (the tensor-parallel
    candidates of one ``tune`` call).  Each entry is searched exactly as if it were alone (its
    own running best, its own stop rule); only the launches are shared.  Returns a list of
    ``(best_cost, best_solution)``.  ``uniform_device`` (``num_nodes``, ``num_gpus_per_node``,
    ``ckpt_tuning``) selects the recurrence of inter_tuning_uniform_device.py instead.
    ``only_best_solution``: a caller that keeps the best entry only (``tune``) gets the partition
    and strategies of that entry; the other entries come back as ``(cost, None)``.
    ``table_limit`` (pinned host tensor with an estimate, factor): the tables hold their values
    up to ``estimate * factor / G`` only (``IntraStageTuner.run_prepared`` with a stage-cost
    cutoff); the search then stays below that limit and ``stats['dp_unresolved']`` counts the
    (entry, G) pairs whose result is not certain to be the reference's (library search only)."""
    if table_limit is not None and not (NATIVE_SEARCH and _same_batch(results_list)):
        raise ValueError("tables with a limit need the library's search over one batch of tables")
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
                                          gradient_accumulation_steps_candidates, [one], slot, stats,
                                          uniform_device)
        if only_best_solution:
            finite = [i for i, (cost, sol) in enumerate(out) if sol is not None]
            keep = min(finite, key=lambda i: out[i][0]) if finite else None
            out = [(cost, sol if i == keep else None) for i, (cost, sol) in enumerate(out)]
        return out
    t_start = time.perf_counter()
    first = results_list[0]
    runner = _DpRunner(first, num_layers, num_devices, device_mesh_candidates, slot, uniform_device)
    n_g = len(first.gradient_accumulation_steps_candidates)
    g_index = {G: i for i, G in enumerate(first.gradient_accumulation_steps_candidates)}
    q_index = {q: i for i, q in enumerate(first.device_mesh_candidates)}
    Gs = list(gradient_accumulation_steps_candidates)
    # table row of (instance, G)
    rows = np.array([[t * n_g + g_index[G] for G in Gs] for t in range(len(results_list))], dtype=np.int32)
    t_0 = time.perf_counter()
    if NATIVE_SEARCH:
        out = _native_search(runner, results_list, rows, Gs, n_g, g_index, q_index, num_layers, slot,
                             only_best_solution, stats, table_limit)
        if stats is not None:
            stats["dp_setup_s"] = stats.get("dp_setup_s", 0.0) + (t_0 - t_start)
        return out
    bests = _search(runner, rows, Gs, stats)
    t_2 = time.perf_counter()
    out = _solutions(runner, results_list, bests, n_g, g_index, q_index, num_layers, slot,
                     only_best_solution)
    if stats is not None:
        stats["dp_setup_s"] = stats.get("dp_setup_s", 0.0) + (t_0 - t_start)
        stats["dp_backtrack_s"] = stats.get("dp_backtrack_s", 0.0) + (time.perf_counter() - t_2)
        stats["dp_launches"] = stats.get("dp_launches", 0) + runner.launches
        stats["dp_window_fetches"] = stats.get("dp_window_fetches", 0) + runner.fetches
        stats["dp_window_values"] = stats.get("dp_window_values", 0) + runner.selected
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
