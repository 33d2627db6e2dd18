"""Writes tests/golden/search_tables_plan<N>.json: what the CPU oracle (``oracle/``, the numpy
restatement of the reference's search) finds for whole (tp, G, mesh) groups of the five
benchmark plans at their full size, as one digest per group and table variant, plus the
oracle's end-to-end ``(best_cost, best_solution)`` where every group of the plan is covered.

    python tests/golden/make_search_fixtures.py --plan 2 --workers 7            # all groups
    python tests/golden/make_search_fixtures.py --plan 4 --select subset        # listed groups
    python tests/golden/make_search_fixtures.py --plan 5 --shard 0/4 --out parts  # a quarter of the
        groups; --merge parts then joins the part files into the fixture
    python tests/golden/make_search_fixtures.py --plan 4 --skip-covered --split-p 3 --deadline 1100
        # the groups the fixture lacks, each as three jobs over a share of its p values

Runs on the CPU only (the oracle never touches the GPU library).  A group is one call of the
oracle's ``batched_tune_best_latency_for_stage`` with ``sample_size = 1`` (the slot the
inter-stage DP reads); its four result tables (middle / first / last / single stage), padded to
the tuner's table shape like ``IntraStageTuner.tune`` pads them
(mist/analyzer/intra_tuning.py:228-259), are reduced to ``tests.util.table_digest``.  Per-group
results are kept in ``--cache`` so that an interrupted run resumes and the end-to-end search can
read the cost tables back.

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

# Plan 4 (GPT-22B, 185 661 offload combinations per parallelism row) costs the oracle ~40
# core-hours as a whole; these groups (8 to 12 core-minutes each) cover its shapes: one and four
# parallelism rows, single device to 16 nodes, 1 to 48 pre-saved micro-batch values (1 to 3
# p tiles of the reduce kernel), every tp.
SUBSETS = {
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


def cache_path(cache, plan, tp, G, mesh):
    return os.path.join(cache, f"plan{plan}", f"tp{tp}_G{G}_{mesh[0]}x{mesh[1]}.npz")


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
    shapes = [(P + 1, L, L + 1, 1), (P + 1, L, L + 1, 1), (L, L + 1, 1), (L + 1, 1)]
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
        mesh[0], mesh[1], G, tp_size=tp, sample_size=1)
    return group_key(tp, G, mesh), finish_group(res, cfg, tables, plan, tp, G, mesh, cache,
                                                time.time() - t0)


def part_values(ps, part, n_parts):
    """The contiguous share ``part`` of the pre-saved micro-batch values ``ps``."""
    lo, hi = round(part * len(ps) / n_parts), round((part + 1) * len(ps) / n_parts)
    return ps[lo:hi]


def part_path(cache, plan, tp, G, mesh, part, n_parts):
    return cache_path(cache, plan, tp, G, mesh)[:-4] + f".part{part}of{n_parts}.npz"


def run_part(args):
    """A share of one group's pre-saved micro-batch values through the oracle (--split-p): a
    group too long for one core within the time there is.  The oracle's loop over p carries one
    thing from p = 0 to the later values of the same (l, c), the layer mask narrowed by the
    last-stage variant (batched_module_analyzer.py:3021-3023), so every share starts with
    p = 0; the other values are independent of each other."""
    plan, tp, G, mesh, cache, part, n_parts = args
    key = group_key(tp, G, mesh)
    path = part_path(cache, plan, tp, G, mesh, part, n_parts)
    if os.path.exists(cache_path(cache, plan, tp, G, mesh)) or os.path.exists(path):
        return key, part
    from oracle.search_space import create_search_space
    from oracle.stage import batched_stage_analyze

    cfg, tables = load_plan(plan)
    L = cfg.model.num_hidden_layers
    ps, _ = p_values(cfg, G)
    mine = part_values(ps, part, n_parts)
    t0 = time.time()
    rows = create_search_space(mesh[0], mesh[1], cfg.training.global_batch_size, G, cfg,
                               constraint_fn=tables.constraint, tp_size=tp)
    res = batched_stage_analyze(
        tables, cfg, mine if mine[0] == 0 else [0] + mine, list(range(1, L + 1)),
        list(range(0, L + 1)), mesh[0], mesh[1], G, rows, 1)
    keep = dict(seconds=time.time() - t0)
    for v in range(4 if part == 0 else 2):  # the p == 0 variants come from the first share
        keep[f"stable{v}"], keep[f"delta{v}"], keep[f"index{v}"] = res[v][0], res[v][1], res[v][3]
    os.makedirs(os.path.dirname(path), exist_ok=True)
    tmp = path + f".tmp{os.getpid()}.npz"
    np.savez_compressed(tmp, **keep)
    os.replace(tmp, path)
    return key, part


def merge_parts(plan, tp, G, mesh, cache, n_parts):
    """Joins the shares of a group written by run_part into the result of one oracle call."""
    cfg, tables = load_plan(plan)
    ps, _ = p_values(cfg, G)
    parts = [np.load(part_path(cache, plan, tp, G, mesh, i, n_parts)) for i in range(n_parts)]
    res = []
    for v in range(4):
        if v >= 2:
            res.append((parts[0][f"stable{v}"], parts[0][f"delta{v}"], None, parts[0][f"index{v}"]))
            continue
        whole = [np.array(parts[-1][f"{name}{v}"]) for name in ("stable", "delta", "index")]
        assert whole[0].shape[0] == len(ps)
        for i in range(n_parts - 1):
            mine = part_values(ps, i, n_parts)
            for k, name in enumerate(("stable", "delta", "index")):
                whole[k][mine] = parts[i][f"{name}{v}"][mine]
        res.append((whole[0], whole[1], None, whole[2]))
    seconds = sum(float(z["seconds"]) for z in parts)
    record = finish_group(res, cfg, tables, plan, tp, G, mesh, cache, seconds)
    for i in range(n_parts):
        os.remove(part_path(cache, plan, tp, G, mesh, i, n_parts))
    return record


def run_job(args):
    return run_part(args) if len(args) == 7 else run_group(args)


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
        shapes = [(P + 1, L, L + 1, 1), (P + 1, L, L + 1, 1), (L, L + 1, 1), (L + 1, 1)]
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


def end_to_end(plan, cache, workers):
    """``tune`` of the reference for the inter-stage granularity (tune_one_case.py:186-232,
    inter_tuning.py:63-217) on the cached oracle tables.  The scans of all (tp, G) run in
    parallel without a bound; replaying them in the reference's order (tp after tp with strict
    ``<``; within a tp G after G with the running best as the bound, ``t G >= best -> stop``)
    gives exactly the sequential result, because a bounded scan runs a prefix of the thresholds
    of the unbounded one."""
    from oracle.inter_dp import get_intra_solution

    cfg, tables = load_plan(plan)
    meshes, Gs, tps = plan_axes(cfg)
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
                row = get_intra_solution(res, L, Gs.index(tp_G), len(tp_inter) - i - 1, l0, l1,
                                         meshes.index((n, m)), ckpt, 0).tolist()
                row[:6] = [int(x) for x in row[:6]]
                solution[1].append([[[l0, l1], [n, m], ckpt, 0], row])
        per_tp[str(tp)] = dict(cost=repr(float(tp_best)), solution=solution, dp_runs_at_or_above_bottleneck=n_dp)
        if tp_best < best_cost:
            best_cost, best_solution = tp_best, solution
    return dict(granularity="inter-stage", cost=repr(float(best_cost)), solution=best_solution, per_tp=per_tp)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--plan", type=int, required=True)
    ap.add_argument("--select", default="all", choices=["all", "subset"])
    ap.add_argument("--workers", type=int, default=4)
    ap.add_argument("--cache", default="/tmp/mist_oracle_cache")
    ap.add_argument("--no-tune", action="store_true", help="skip the end-to-end search")
    ap.add_argument("--shard", default="0/1", help="i/n: only every n-th group, starting at the i-th")
    ap.add_argument("--out", default=HERE, help="directory the fixture is written to")
    ap.add_argument("--merge", default=None, help="join the part files of this directory (and the groups "
                    "of the committed fixture of a partly covered plan) and exit")
    ap.add_argument("--max-work", type=int, default=0,
                    help="leave out groups with more than this many rows x pre-saved micro-batch values "
                    "(one group runs on one core; 0 = no bound)")
    ap.add_argument("--skip-covered", action="store_true", help="leave out the groups the committed fixture holds")
    ap.add_argument("--split-p", type=int, default=1,
                    help="run every group as this many jobs, each with a share of the pre-saved "
                    "micro-batch values (for groups too long for one core within --deadline)")
    ap.add_argument("--deadline", type=float, default=0.0,
                    help="seconds after which the run stops and keeps what it has (0 = none)")
    a = ap.parse_args()
    if a.merge:
        import glob

        parts = sorted(glob.glob(os.path.join(a.merge, f"search_tables_plan{a.plan}.part*.json")))
        whole = os.path.join(a.merge, f"search_tables_plan{a.plan}.json")  # a run without --shard
        if os.path.exists(whole) and os.path.abspath(a.merge) != os.path.abspath(HERE):
            parts.append(whole)
        out, have = None, []
        for p in parts:
            with open(p) as f:
                d = json.load(f)
            have.append(d["select"])
            if out is None:
                out = d
            else:
                out["groups"].update(d["groups"])
        path = os.path.join(HERE, f"search_tables_plan{a.plan}.json")
        if os.path.exists(path):  # a partly covered plan grows: keep what the fixture already holds
            with open(path) as f:
                old = json.load(f)
            if old["select"] != "all" and "tune" not in old:
                have.insert(0, old["select"])
                for k, v in old["groups"].items():
                    out["groups"].setdefault(k, v)
        n = int(parts[0].rsplit("of", 1)[1].split(".")[0]) if "of" in os.path.basename(parts[0]) else 1
        bounded = any("at most" in h for h in have)
        out["select"] = "all" if len(parts) == n and not bounded and len(have) == len(parts) else "; ".join(have)
        with open(path, "w") as f:
            json.dump(out, f, indent=1, sort_keys=True)
            f.write("\n")
        print("wrote", path, len(out["groups"]), "groups,", out["select"])
        return
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
    if a.max_work > 0:
        jobs = [j for j in jobs if j[0] <= a.max_work]
    if a.skip_covered:
        with open(os.path.join(HERE, f"search_tables_plan{a.plan}.json")) as f:
            covered = set(json.load(f)["groups"])
        jobs = [j for j in jobs if group_key(j[1][1], j[1][2], j[1][3]) not in covered]
    shard, n_shards = (int(x) for x in a.shard.split("/"))
    jobs = jobs[shard::n_shards]
    groups = {}
    t0 = time.time()
    import threading

    def heartbeat():  # long groups finish minutes apart: show that the run is alive
        while True:
            time.sleep(60)
            print(f"[{time.time() - t0:7.0f}s] ... {len(groups)}/{len(jobs)} groups done", flush=True)

    threading.Thread(target=heartbeat, daemon=True).start()
    select = a.select if n_shards == 1 else f"shard {shard} of {n_shards} (groups by size, every {n_shards}th)"
    if a.max_work > 0:
        select += f", groups of at most {a.max_work} rows x pre-saved micro-batch values"
    if a.skip_covered:
        select += ", without those already covered"
    part = "" if n_shards == 1 else f".part{shard}of{n_shards}"
    os.makedirs(a.out, exist_ok=True)
    path = os.path.join(a.out, f"search_tables_plan{a.plan}{part}.json")

    def write(out):
        with open(path + ".tmp", "w") as f:
            json.dump(out, f, indent=1, sort_keys=True)
            f.write("\n")
        os.replace(path + ".tmp", path)

    def fixture():
        return dict(
            plan=PLAN_FILES[a.plan - 1], sample_size=1, select=select,
            made_by="tests/golden/make_search_fixtures.py (CPU oracle)",
            groups={k: dict(rows=groups[k]["rows"], finite=groups[k]["finite"], digest=groups[k]["digest"])
                    for k in sorted(groups)},
        )

    tasks = [j[1] for j in jobs]
    n_shares = {}
    if a.split_p > 1:  # never more shares than a group has values of p
        tasks = []
        for j in jobs:
            k = min(a.split_p, len(p_values(cfg, j[1][2])[0]))
            n_shares[group_key(j[1][1], j[1][2], j[1][3])] = k
            tasks += [j[1] + (part, k) for part in range(k)]
        select += f", up to {a.split_p} jobs per group"
    parts_done = {}
    with get_context("fork").Pool(a.workers, maxtasksperchild=1) as pool:
        results = pool.imap_unordered(run_job, tasks)
        for n in range(len(tasks)):
            try:
                key, rec = results.next(timeout=max(a.deadline - (time.time() - t0), 1.0) if a.deadline else None)
            except Exception as e:  # multiprocessing.TimeoutError: the deadline has passed
                if type(e).__name__ != "TimeoutError":
                    raise
                print(f"[{time.time() - t0:7.0f}s] deadline: {len(groups)} of {len(jobs)} groups kept", flush=True)
                select += f" (stopped after {len(groups)} of {len(jobs)})"
                write(fixture())
                pool.terminate()  # the unfinished groups are given up
                print("wrote", path, flush=True)
                return
            if a.split_p > 1:  # rec = the share that is done; the last one completes the group
                parts_done.setdefault(key, set()).add(rec)
                print(f"[{time.time() - t0:7.0f}s] {key} share {rec + 1} of {n_shares[key]}", flush=True)
                if len(parts_done[key]) < n_shares[key]:
                    continue
                job = next(j[1] for j in jobs if group_key(j[1][1], j[1][2], j[1][3]) == key)
                final = cache_path(job[4], job[0], job[1], job[2], job[3])
                if os.path.exists(final):
                    with np.load(final) as z:
                        rec = json.loads(str(z["record"]))
                else:
                    rec = merge_parts(job[0], job[1], job[2], job[3], job[4], n_shares[key])
            groups[key] = rec
            print(f"[{time.time() - t0:7.0f}s] {len(groups)}/{len(jobs)} {key} rows={rec['rows']} "
                  f"finite={rec['finite']} ({rec['oracle_seconds']} s)", flush=True)
            write(fixture())
    out = fixture()
    if a.select == "all" and not a.no_tune and n_shards == 1:
        out["tune"] = end_to_end(a.plan, a.cache, a.workers)
        print("tune:", out["tune"]["cost"], out["tune"]["solution"], flush=True)
    write(out)
    print("wrote", path, flush=True)


if __name__ == "__main__":
    main()
