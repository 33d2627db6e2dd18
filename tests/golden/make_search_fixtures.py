"""Writes tests/golden/search_tables_plan<N>[_s<S>].json: what the CPU oracle (``oracle/``, the
restatement of the reference's search) finds for whole (tp, G, mesh) groups of the five benchmark
plans at their full size, as one digest per group and table variant, plus the oracle's end-to-end
``(best_cost, best_solution)``.

    python tests/golden/make_search_fixtures.py --plan 2 --workers 4 --threads 2
    python tests/golden/make_search_fixtures.py --plan 2 --sample-size 30      # ..._plan2_s30.json
    python tests/golden/make_search_fixtures.py --plan 5 --tune-scope "8:64,128"
        # end-to-end search for tensor-parallel size 8 over G in {64, 128} only (the inter-stage
        # scan of the whole plan would take the C DP days)

Runs on the CPU only (the oracle never touches the GPU library).  A group is one call of the
oracle's ``batched_tune_best_latency_for_stage``; its four result tables (middle / first / last /
single stage), padded to the tuner's table shape like ``IntraStageTuner.tune`` pads them
(mist/analyzer/intra_tuning.py:228-259), are reduced to ``tests.util.table_digest``.  With
``--inner c`` (default) the loops over (ckpt layers, pre-saved micro-batches) of a group run in
oracle/stage_loop.c, with ``--inner numpy`` in the numpy statements of oracle/stage.py; both give
the same tables bit for bit, and a run over a plan whose committed fixture was written the other
way checks that (every digest the fixture holds must come out again, or the run stops).
Per-group results are kept in ``--cache`` so that an interrupted run resumes and the end-to-end
search can read the cost tables back.

End-to-end block: for one sample (``inter-stage`` granularity) the reference's threshold scan
with the C DP (inter_tuning.py:163-217); for several samples the ``uniform-device-pp-mip``
granularity (inter_tuning_mip.py, oracle/inter_mip.py).

The GPU tests (tests/test_gpu_golden_tables.py) compute the same digests from the tables the
HIP kernels produce and compare.
"""
import argparse
import json
import os
import sys
import time
from multiprocessing import get_context

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
for p in (REPO, os.path.join(REPO, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

from util import PLAN_FILES, group_key, load_plan, table_digest  # noqa: E402

# Groups for --select subset: a cross-section of a plan's shapes (one and four parallelism rows,
# single device to all nodes, one to many pre-saved micro-batch values, every tp).
SUBSETS = {
    2: [
        (1, 512, (1, 1)), (1, 16, (4, 8)), (2, 64, (1, 2)), (2, 32, (2, 8)), (4, 256, (1, 4)),
        (4, 16, (4, 8)), (8, 128, (1, 8)), (8, 16, (4, 8)), (8, 32, (2, 8)), (1, 2, (4, 8)),
    ],
    4: [
        (1, 512, (1, 1)), (2, 64, (1, 2)), (4, 256, (1, 4)), (8, 128, (1, 8)),
        (1, 1, (16, 8)), (2, 2, (8, 8)), (4, 4, (16, 8)), (1, 4, (2, 8)),
        (8, 8, (8, 8)), (1, 8, (1, 8)), (2, 8, (4, 8)), (4, 8, (4, 8)),
    ],
}


def plan_axes(cfg):
    from oracle.search_space import device_mesh_candidates, grad_accumu_steps_candidates
    from oracle.tune import tp_candidates

    hw = cfg.hardware
    meshes = device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, contiguous_inter_node=False)
    Gs = grad_accumu_steps_candidates(cfg.training.global_batch_size)
    return meshes, Gs, tp_candidates(cfg)


def group_rows(cfg, tables, tp, G, mesh):
    from oracle.search_space import create_search_space

    return create_search_space(mesh[0], mesh[1], cfg.training.global_batch_size, G, cfg,
                               constraint_fn=tables.constraint, tp_size=tp).shape[0]


# How a group goes through the oracle (set from the command line before the workers fork):
# the loops over (ckpt layers, pre-saved micro-batches) in C (oracle/stage_loop.c, bit-equal to
# the numpy statements and ~100 times faster on the large plans) or in numpy, the OpenMP threads
# of one C call, and the number of alpha samples per cell.
INNER, THREADS, SAMPLES = "c", 0, 1


def cache_path(cache, plan, tp, G, mesh):
    name = f"plan{plan}" if SAMPLES == 1 else f"plan{plan}_s{SAMPLES}"
    if INNER == "c-fused":
        name += "_fused"
    return os.path.join(cache, name, f"tp{tp}_G{G}_{mesh[0]}x{mesh[1]}.npz")


def fixture_name(plan):
    return f"search_tables_plan{plan}.json" if SAMPLES == 1 else f"search_tables_plan{plan}_s{SAMPLES}.json"


def p_values(cfg, G):
    """The pre-saved micro-batch values of a group (intra_tuning.py:185-193) and the plan's P."""
    from oracle.intra import max_pre_saved_micro_batches

    meshes, Gs, _ = plan_axes(cfg)
    L = cfg.model.num_hidden_layers
    P = max_pre_saved_micro_batches(meshes, Gs, L)
    return list(range(min(G, L, P + 1))), P


def finish_group(res, cfg, tables, plan, tp, G, mesh, cache, seconds):
    """Pads the oracle's four result tables to the tuner's shapes, digests them and stores them
    in the cache; returns the fixture record."""
    L = cfg.model.num_hidden_layers
    _, P = p_values(cfg, G)
    S = SAMPLES
    shapes = [(P + 1, L, L + 1, S), (P + 1, L, L + 1, S), (L, L + 1, S), (L + 1, S)]
    record = dict(rows=int(group_rows(cfg, tables, tp, G, mesh)), digest=[], finite=[])
    keep = {}
    for v in range(4):
        stable = np.full(shapes[v], np.inf)
        delta = np.full(shapes[v], np.inf)
        index = np.full(shapes[v], -1, dtype=np.int64)
        corner = tuple(slice(0, n) for n in res[v][0].shape)
        stable[corner], delta[corner], index[corner] = res[v][0], res[v][1], res[v][3]
        stable, delta = stable.astype(np.float32), delta.astype(np.float32)  # intra_tuning.py:244-259
        record["digest"].append(table_digest(index, stable, delta))
        record["finite"].append(int((index >= 0).sum()))
        keep[f"stable{v}"], keep[f"delta{v}"] = stable, delta
        keep[f"index{v}"] = index.astype(np.int32)
    record["oracle_seconds"] = round(seconds, 1)
    path = cache_path(cache, plan, tp, G, mesh)
    os.makedirs(os.path.dirname(path), exist_ok=True)
    tmp = path + f".tmp{os.getpid()}.npz"
    np.savez_compressed(tmp, record=json.dumps(record), **keep)
    os.replace(tmp, path)
    return record


def run_group(args):
    """One (tp, G, mesh) group through the oracle; returns its fixture record."""
    plan, tp, G, mesh, cache = args
    path = cache_path(cache, plan, tp, G, mesh)
    if os.path.exists(path):
        with np.load(path) as z:
            return group_key(tp, G, mesh), json.loads(str(z["record"]))
    from oracle.stage import batched_tune_best_latency_for_stage

    cfg, tables = load_plan(plan)
    L = cfg.model.num_hidden_layers
    ps, _ = p_values(cfg, G)
    t0 = time.time()
    res = batched_tune_best_latency_for_stage(
        tables, cfg, ps, list(range(1, L + 1)), list(range(0, L + 1)),
        mesh[0], mesh[1], G, tp_size=tp, sample_size=SAMPLES, inner=INNER, threads=THREADS)
    return group_key(tp, G, mesh), finish_group(res, cfg, tables, plan, tp, G, mesh, cache,
                                                time.time() - t0)


class CachedResults:
    """The oracle's ``IntraStageTunerOutput`` for one tp candidate, read back from the cache:
    float32 cost tables in full, strategy rows decoded on demand from the row indices."""

    def __init__(self, plan, cfg, tables, tp, cache):
        self.cfg, self.tables, self.tp = cfg, tables, tp
        meshes, Gs, _ = plan_axes(cfg)
        self.gradient_accumulation_steps_candidates = Gs
        self.device_mesh_candidates = meshes
        from oracle.intra import max_pre_saved_micro_batches

        L = cfg.model.num_hidden_layers
        P = max_pre_saved_micro_batches(meshes, Gs, L)
        S = SAMPLES
        shapes = [(P + 1, L, L + 1, S), (P + 1, L, L + 1, S), (L, L + 1, S), (L + 1, S)]
        lead = (len(Gs), len(meshes))
        self._stable = [np.full(lead + s, np.inf, dtype=np.float32) for s in shapes]
        self._delta = [np.full(lead + s, np.inf, dtype=np.float32) for s in shapes]
        self._index = [np.full(lead + s, -1, dtype=np.int32) for s in shapes]
        for g, G in enumerate(Gs):
            for q, mesh in enumerate(meshes):
                path = cache_path(cache, plan, tp, G, mesh)
                if not os.path.exists(path):
                    if group_rows(cfg, tables, tp, G, mesh) == 0:
                        continue  # empty search space: all-inf tables
                    raise FileNotFoundError(path)
                with np.load(path) as z:
                    for v in range(4):
                        self._stable[v][g, q] = z[f"stable{v}"]
                        self._delta[v][g, q] = z[f"delta{v}"]
                        self._index[v][g, q] = z[f"index{v}"]
        suffixes = ("", "_with_pre", "_with_post", "_no_pp")
        for v, s in enumerate(suffixes):
            setattr(self, "costs_stable" + s, self._stable[v])
            setattr(self, "costs_delta" + s, self._delta[v])
            setattr(self, "solutions" + s, _LazyRows(self, v))


class _LazyRows:
    """``solutions*[g, q, ..., slot]`` -> the strategy row of that cell's index."""

    def __init__(self, owner, v):
        self.owner, self.v = owner, v

    def __getitem__(self, cell):
        from oracle.search_space import create_search_space

        o = self.owner
        row = int(o._index[self.v][cell])
        if row < 0:
            return np.full(10, np.inf)
        G = o.gradient_accumulation_steps_candidates[cell[0]]
        n, m = o.device_mesh_candidates[cell[1]]
        rows = create_search_space(n, m, o.cfg.training.global_batch_size, G, o.cfg,
                                   constraint_fn=o.tables.constraint, tp_size=o.tp)
        return rows[row]


def scan_one(args):
    """The t_max scan of one (tp, G) without a bound from earlier candidates
    (``best_cost = inf``): every threshold the reference's scan would run under ANY tighter
    bound is among the ones run here, see ``end_to_end``."""
    plan, tp, G, cache = args
    from oracle.dp_c import dp_impl_c
    from oracle.inter_dp import dp_cost_tables, tmax_candidates

    cfg, tables = load_plan(plan)
    res = CachedResults(plan, cfg, tables, tp, cache)
    meshes, Gs, _ = plan_axes(cfg)
    L, D = cfg.model.num_hidden_layers, cfg.hardware.num_nodes * cfg.hardware.num_gpus_per_node
    costs, costs_pre, costs_post, costs_nopp = dp_cost_tables(res, Gs.index(G), 0)
    cands = tmax_candidates(costs, costs_pre, costs_post)
    run = lambda t, want: dp_impl_c(t, L, D, meshes, G, costs, costs_pre, costs_post, costs_nopp,
                                    want_solution=want)
    if len(cands) == 0 or not np.isfinite(run(cands[-1], False)[0]):
        return tp, G, []
    # Feasibility is monotone in t_max (a larger threshold admits a superset of stages): find the
    # first feasible candidate by bisection instead of running the DP for every smaller one.
    lo, hi = 0, len(cands) - 1  # cands[hi] feasible
    while lo < hi:
        mid = (lo + hi) // 2
        if np.isfinite(run(cands[mid], False)[0]):
            hi = mid
        else:
            lo = mid + 1
    first = lo
    # The reference's gap rule (inter_tuning.py:196-199) from the very first candidate: which
    # thresholds are "kept" does not depend on the DP results, only on the last kept value.
    out, best = [], np.inf
    last = np.float32(0)
    for n, t in enumerate(cands):
        if n >= first and float(np.float64(t) * G) >= best:
            break
        if float(np.float32(t - last)) < 1e-6:
            continue
        last = t
        if n < first:
            continue  # infeasible: the DP returns inf and changes nothing
        cost, sol = run(t, True)
        out.append((float(t), cost, sol))
        best = min(best, cost)
    return tp, G, out


def end_to_end(plan, cache, workers, scope=None):
    """``tune`` of the reference for the inter-stage granularity (tune_one_case.py:186-232,
    inter_tuning.py:63-217) on the cached oracle tables.  The scans of all (tp, G) run in
    parallel without a bound; replaying them in the reference's order (tp after tp with strict
    ``<``; within a tp G after G with the running best as the bound, ``t G >= best -> stop``)
    gives exactly the sequential result, because a bounded scan runs a prefix of the thresholds
    of the unbounded one.  ``scope = (tp, [G, ...])`` restricts the search to one tensor-parallel
    size and those gradient-accumulation counts (``inter_stage_tune`` called with that list)."""
    from oracle.inter_dp import get_intra_solution

    cfg, tables = load_plan(plan)
    meshes, Gs_all, tps = plan_axes(cfg)
    Gs = Gs_all
    if scope is not None:
        tps, Gs = [scope[0]], [G for G in Gs_all if G in scope[1]]
    L = cfg.model.num_hidden_layers
    jobs = [(plan, tp, G, cache) for tp in tps for G in Gs]
    with get_context("fork").Pool(workers, maxtasksperchild=1) as pool:
        scans = {(tp, G): out for tp, G, out in pool.imap_unordered(scan_one, jobs)}
    best_cost, best_solution, per_tp = float("inf"), None, {}
    for tp in tps:
        tp_best, tp_inter, tp_G = float("inf"), None, None
        n_dp = 0
        for G in Gs:
            bound = tp_best
            cur_best, cur_sol = bound, None
            for t, cost, sol in scans[(tp, G)]:
                if float(np.float64(np.float32(t)) * G) >= cur_best:
                    break
                n_dp += 1
                if cost < cur_best:
                    cur_best, cur_sol = cost, sol
            if cur_best < tp_best:
                tp_best, tp_inter, tp_G = cur_best, cur_sol, G
        solution = None
        if tp_inter is not None:
            res = CachedResults(plan, cfg, tables, tp, cache)
            solution = [tp_G, []]
            for i, ((l0, l1), (n, m), ckpt) in enumerate(tp_inter):
                row = get_intra_solution(res, L, Gs_all.index(tp_G), len(tp_inter) - i - 1, l0, l1,
                                         meshes.index((n, m)), ckpt, 0).tolist()
                row[:6] = [int(x) for x in row[:6]]
                solution[1].append([[[l0, l1], [n, m], ckpt, 0], row])
        per_tp[str(tp)] = dict(cost=repr(float(tp_best)), solution=solution, dp_runs_at_or_above_bottleneck=n_dp)
        if tp_best < best_cost:
            best_cost, best_solution = tp_best, solution
    out = dict(granularity="inter-stage", cost=repr(float(best_cost)), solution=best_solution, per_tp=per_tp)
    if scope is not None:
        out["scope"] = dict(tp=scope[0], Gs=Gs)
    return out


def end_to_end_mip(plan, cache):
    """``tune`` of the reference for the ``uniform-device-pp-mip`` granularity
    (tune_one_case.py:360-402) on the cached oracle tables with all their samples: per
    tensor-parallel size the stage assignment of oracle/inter_mip.py, first best wins."""
    from oracle.inter_mip import inter_stage_tune

    cfg, tables = load_plan(plan, tuning__tuning_granularity="uniform-device-pp-mip",
                            tuning__sample_size=SAMPLES)
    meshes, Gs, tps = plan_axes(cfg)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    best_cost, best_solution, per_tp = float("inf"), None, {}
    for tp in tps:
        res = CachedResults(plan, cfg, tables, tp, cache)
        cost, sol = inter_stage_tune(L, hw.num_nodes, hw.num_gpus_per_node, meshes, Gs, res, cfg)
        sol = json.loads(json.dumps(sol, default=lambda o: o.item()))
        per_tp[str(tp)] = dict(cost=repr(float(cost)), solution=sol)
        if cost < best_cost:
            best_cost, best_solution = cost, sol
    return dict(granularity="uniform-device-pp-mip", sample_size=SAMPLES, cost=repr(float(best_cost)),
                solution=best_solution, per_tp=per_tp)


def main():
    global INNER, THREADS, SAMPLES
    ap = argparse.ArgumentParser()
    ap.add_argument("--plan", type=int, required=True)
    ap.add_argument("--select", default="all", choices=["all", "subset"])
    ap.add_argument("--sample-size", type=int, default=1, help="alpha samples per cell (1: the slot the DP reads)")
    ap.add_argument("--inner", default="c", choices=["c", "numpy", "c-fused"],
                    help="c-fused: the argmin objective r x + y as one fused multiply-add (what numba's "
                    "fastmath permits); compares with the committed fixture and writes nothing")
    ap.add_argument("--workers", type=int, default=4, help="groups in flight (processes)")
    ap.add_argument("--threads", type=int, default=2, help="OpenMP threads of one group's C loops")
    ap.add_argument("--cache", default="/tmp/mist_oracle_cache")
    ap.add_argument("--no-tune", action="store_true", help="skip the end-to-end search")
    ap.add_argument("--tune-scope", default=None,
                    help="'tp:G,G,...': end-to-end search over this tensor-parallel size and these "
                    "gradient-accumulation counts only")
    a = ap.parse_args()
    INNER, THREADS, SAMPLES = a.inner, a.threads, a.sample_size
    cfg, tables = load_plan(a.plan)
    meshes, Gs, tps = plan_axes(cfg)
    if a.select == "all":
        wanted = [(tp, G, mesh) for tp in tps for G in Gs for mesh in meshes]
    else:
        wanted = SUBSETS[a.plan]
    jobs = []
    from mist_amd.search_space import create_search_space_for_a_block_layer

    for tp, G, mesh in wanted:
        # sizing only: the factored search space counts the rows without listing them (the
        # oracle's own count goes into the record, run_group)
        n = create_search_space_for_a_block_layer(
            mesh[0], mesh[1], cfg.training.global_batch_size, G, cfg, constraint_fn=tables.constraint,
            tp_size=tp).n_rows
        if n > 0:
            jobs.append((n * min(G, cfg.model.num_hidden_layers), (a.plan, tp, G, tuple(mesh), a.cache)))
    jobs.sort(key=lambda j: -j[0])  # long groups first
    path = os.path.join(HERE, fixture_name(a.plan))
    old = {}
    if os.path.exists(path):
        with open(path) as f:
            old = json.load(f)
    groups = {}
    t0 = time.time()
    import threading

    def heartbeat():  # long groups finish minutes apart: show that the run is alive
        while True:
            time.sleep(60)
            print(f"[{time.time() - t0:7.0f}s] ... {len(groups)}/{len(jobs)} groups done", flush=True)

    threading.Thread(target=heartbeat, daemon=True).start()
    reproduced, differing = 0, []
    with get_context("fork").Pool(a.workers, maxtasksperchild=1) as pool:
        for key, rec in pool.imap_unordered(run_group, [j[1] for j in jobs]):
            groups[key] = rec
            was = old.get("groups", {}).get(key)
            if was is not None:  # written earlier, possibly by the other form of the loops
                same = was["digest"] == rec["digest"] and was["finite"] == rec["finite"]
                if INNER == "c-fused" and not same:
                    differing.append(key)
                else:
                    assert same, f"{key}: the committed fixture holds other tables: {was} vs {rec}"
                    reproduced += 1
            print(f"[{time.time() - t0:7.0f}s] {len(groups)}/{len(jobs)} {key} rows={rec['rows']} "
                  f"finite={rec['finite']} ({rec['oracle_seconds']} s)", flush=True)
    print(f"{reproduced} groups of the committed fixture reproduced", flush=True)
    if INNER == "c-fused":
        print(f"fused objective: {len(differing)} of {len(groups)} groups pick other winners: {differing}")
        return
    out = dict(
        plan=PLAN_FILES[a.plan - 1], sample_size=SAMPLES, select=a.select,
        made_by=f"tests/golden/make_search_fixtures.py (CPU oracle, --inner {INNER})",
        groups={k: dict(rows=groups[k]["rows"], finite=groups[k]["finite"], digest=groups[k]["digest"])
                for k in sorted(groups)},
    )
    for k in ("tune", "tune_scoped"):  # kept unless this run writes them again
        if k in old and old.get("groups") == out["groups"]:
            out[k] = old[k]
    if a.tune_scope:
        tp, gs = a.tune_scope.split(":")
        out["tune_scoped"] = end_to_end(a.plan, a.cache, a.workers * max(a.threads, 1),
                                        scope=(int(tp), [int(g) for g in gs.split(",")]))
        print("tune (scoped):", out["tune_scoped"]["cost"], out["tune_scoped"]["solution"], flush=True)
    elif a.select == "all" and not a.no_tune:
        if SAMPLES == 1:
            out["tune"] = end_to_end(a.plan, a.cache, a.workers * max(a.threads, 1))
        else:
            out["tune"] = end_to_end_mip(a.plan, a.cache)
        print("tune:", out["tune"]["cost"], out["tune"]["solution"], flush=True)
    with open(path + ".tmp", "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    os.replace(path + ".tmp", path)
    print("wrote", path, flush=True)


if __name__ == "__main__":
    main()
