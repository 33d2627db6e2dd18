"""Benchmark of the configuration-search hot path on one MI355X.

``python bench.py --gpus 1 --steps K --warmup W`` prints ONE JSON line.

Workload: the GPT-7B plan (mist_amd/configs/gpt-7b-b512-4x8.yaml: 32 layers, hidden 4096,
global batch 512, planned 4x8 devices, offload ratios in steps of 0.1; 1.06e8 candidates).
A step is one complete pass of the hot path over that search space with the group descriptors
already resident in HBM: for every tensor-parallel candidate the intra-stage kernels (row terms,
evaluate + mask + argmin, finalize) over all (gradient-accumulation, mesh) groups, then the
inter-stage pipeline-partition DP; the chosen strategy comes back to the host.

``value`` = candidates per second, candidate = (strategy row, checkpointed-layer count) summed
over all (G, mesh, tp) groups.  Extra keys: ``cells_per_s`` (cell = row x stage-layers x
ckpt-count x pre-saved micro-batches, the arithmetic unit), ``tune_end_to_end_s`` (YAML object
to strategy including descriptor building and upload), ``roofline`` of the dominant kernel and a
``cpu_baseline`` (the numpy oracle on a bounded sample of the same workload).
"""
import argparse
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

PLAN = os.path.join(REPO, "mist_amd", "configs", "gpt-7b-b512-4x8.yaml")
FP64_VECTOR_PEAK = 78.6e12  # MI355X published fp64 vector peak, FLOP/s
PROFILE = os.path.join(REPO, "profiles", "eval_reduce_gpt7b_counters.md")


def profile_counters():
    """Per-call counter sums of the reduce kernels on this workload, read from the committed
    rocprofv3 --pmc summary (rows ``| COUNTER | pruned | exhaustive |`` of PROFILE).  They are
    properties of the workload (the search is deterministic), so a separate profiler run supplies
    them and this run supplies the durations."""
    import re

    out = {}
    if not os.path.exists(PROFILE):
        return out
    for line in open(PROFILE):
        m = re.match(r"^\|\s*([A-Z][A-Z0-9_]+)\s*\|\s*([0-9.eE+-]+)\s*\|\s*([0-9.eE+-]+)\s*\|", line)
        if m:
            out[m.group(1)] = dict(pruned=float(m.group(2)), exhaustive=float(m.group(3)))
        m = re.match(r"^kernel source sha256: ([0-9a-f]+)", line)
        if m:
            out["_source_sha256"] = m.group(1)
    return out


def kernel_source_sha256():
    """Digest of the kernel sources the counters belong to (the profile records it)."""
    import hashlib

    h = hashlib.sha256()
    for name in ("mist_search.hip", "exact_arith.h", "mist_common.h"):
        with open(os.path.join(REPO, "mist_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    with open(os.path.join(REPO, "include", "mist_search.h"), "rb") as f:
        h.update(f.read())
    return h.hexdigest()[:16]


def executed_fp64_flops(counters, which):
    """float64 operations a launch executed, from the SQ instruction counters: ADD, MUL and
    TRANS (reciprocal seeds of the divisions) count one operation per active lane, FMA two
    (with contraction off the compiler emits FMAs only inside division sequences).  The
    counters count wave instructions; the average number of active lanes per VALU instruction
    (SQ_THREAD_CYCLES_VALU / SQ_ACTIVE_INST_VALU, both in quad-cycles) converts them to lanes."""
    c = {k: v[which] for k, v in counters.items()}
    need = ("SQ_INSTS_VALU_ADD_F64", "SQ_INSTS_VALU_MUL_F64", "SQ_INSTS_VALU_FMA_F64",
            "SQ_INSTS_VALU_TRANS_F64", "SQ_THREAD_CYCLES_VALU", "SQ_ACTIVE_INST_VALU")
    if any(k not in c for k in need) or c["SQ_ACTIVE_INST_VALU"] <= 0:
        return None, None
    lanes = min(64.0, c["SQ_THREAD_CYCLES_VALU"] / c["SQ_ACTIVE_INST_VALU"])
    wave_ops = (c["SQ_INSTS_VALU_ADD_F64"] + c["SQ_INSTS_VALU_MUL_F64"] + c["SQ_INSTS_VALU_TRANS_F64"]
                + 2.0 * c["SQ_INSTS_VALU_FMA_F64"])
    return wave_ops * lanes, lanes


def reduce_kernel_flops(plan, L):
    """Algorithmic float64 operations of one evaluate+mask+argmin launch (add / sub / mul / div /
    max / compare = 1 each, counted from the reference's formulas for the cells the reference
    evaluates and keeps, c <= l): per (row, l) 15, per (row, l, c) 22, per cell 30 for the middle-
    stage variant + 12 for the first-stage variant, and at p == 0 per (row, l, c) 25 for the
    last-stage variant + 10 for the single-stage variant."""
    g = plan["groups"]
    rows = int(g["n_rows"].sum())
    pairs = L * (L + 1) // 2 + L
    cells = int((g["n_rows"] * g["num_p"]).sum()) * pairs
    return 15 * rows * L + 22 * rows * pairs + (30 + 12) * cells + (25 + 10) * rows * pairs


def cpu_baseline(cfg, tables, results=None, budget_s=14.0, dp_budget_s=6.0):
    """Times the CPU oracle on whole (G, mesh, tp) groups of the same plan until ``budget_s`` is
    used, twice: (1) its numpy form (a port of the reference's own formulation, one thread) and
    (2) its C form (oracle/stage_loop.c: the same loops cell by cell, OpenMP over the (layers,
    ckpt) pairs like the reference's numba ``prange``) on every core of the host.  The sample
    starts with a multi-node group with four parallelism rows (53 724 candidate rows), then
    single-device groups.  With ``results`` (the GPU search's tables of tp = 1) the C restatement
    of the reference's DP kernel is timed on the same cost tables."""
    import numpy as np

    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates
    from oracle.intra import max_pre_saved_micro_batches
    from oracle.stage import batched_tune_best_latency_for_stage

    hw = cfg.hardware
    L = cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    P = max_pre_saved_micro_batches(meshes, Gs, L)
    sample = [(2, (4, 8), 1), (512, (1, 1), 1), (256, (1, 1), 1), (128, (1, 1), 1)]

    def run(inner, groups, budget, threads=0):
        done, cand, cells, elapsed = [], 0, 0, 0.0
        for G, (n, m), tp in groups:
            dbg = {}
            t0 = time.perf_counter()
            batched_tune_best_latency_for_stage(
                tables, cfg, list(range(min(G, L, P + 1))), list(range(1, L + 1)), list(range(L + 1)),
                n, m, G, tp_size=tp, sample_size=1, debug=dbg, inner=inner, threads=threads,
            )
            elapsed += time.perf_counter() - t0
            rows = dbg["rows"].shape[0]
            cand += rows * (L + 1)
            cells += rows * (L * (L + 1) // 2 + L) * min(G, L, P + 1)
            done.append(f"G={G} mesh={n}x{m} tp={tp} rows={rows}")
            if elapsed > budget:
                break
        return done, cand, cells, elapsed

    done, cand, cells, elapsed = run("numpy", sample, budget_s * 0.6)
    out = dict(
        value=cand / elapsed, unit="candidates/s", cores=1, kind="port",
        sample="; ".join(done) + f"; {elapsed:.1f} s of numpy, intra-stage evaluation only",
        cells_per_s=cells / elapsed,
    )
    # the C loops on all cores: every group of tp = 1 in table order, as far as the budget goes
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
    many = sample + [(G, mesh, 1) for G in reversed(Gs) for mesh in meshes if (G, mesh, 1) not in sample]
    from oracle.search_space import create_search_space

    many = [(G, (n, m), tp) for G, (n, m), tp in many
            if create_search_space(n, m, cfg.training.global_batch_size, G, cfg,
                                   constraint_fn=tables.constraint, tp_size=tp).shape[0] > 0]
    run("c", many[:1], 0.0, cores)  # loads the library, spins the thread pool up
    done, cand, cells, elapsed = run("c", many, budget_s * 0.4, cores)
    out["multicore"] = dict(
        value=cand / elapsed, unit="candidates/s", cores=cores, kind="port",
        sample=f"{len(done)} groups of tp=1 ({done[0]} ... {done[-1]}); {elapsed:.1f} s; row terms in numpy "
               f"(one thread), the (ckpt, pre-saved micro-batch) loops and the argmin scan in C on {cores} threads",
        cells_per_s=cells / elapsed,
    )
    if results is not None:
        from oracle.dp_c import dp_impl_c
        from oracle.inter_dp import dp_cost_tables, tmax_candidates

        g = len(Gs) // 2
        tabs = dp_cost_tables(results, g)
        cands = tmax_candidates(*tabs[:3])
        picks = cands[len(cands) // 2::max(len(cands) // 200, 1)]
        D = hw.num_nodes * hw.num_gpus_per_node
        n_dp, t0 = 0, time.perf_counter()
        for t in picks:
            dp_impl_c(t, L, D, meshes, Gs[g], *tabs, want_solution=False)
            n_dp += 1
            if time.perf_counter() - t0 > dp_budget_s:
                break
        dp_s = time.perf_counter() - t0
        out["dp"] = dict(
            value=n_dp / dp_s, unit="DP instances/s", cores=1, kind="port",
            sample=f"{n_dp} thresholds of G={Gs[g]}, tp=1 on the GPU search's cost tables "
                   f"(L={L}, D={D}, {len(meshes)} meshes), C restatement of the numba kernel, {dp_s:.1f} s",
        )
    return out


OTHER_PLANS = ("gpt-1.3b-b8-1x2.yaml", "llama-13b-b1024-8x8.yaml", "gpt-22b-b1536-16x8.yaml",
               "llama-70b-b2048-32x8.yaml")


def other_plans():
    """The other benchmark plans (parity cases, not the bench line): whole ``tune()`` from the
    configuration object, and one search step with the descriptors resident like the timed
    workload; cost and a digest of the chosen strategy."""
    import hashlib

    import torch

    from mist_amd.config import MistConfig
    from mist_amd.tune_one_case import PreparedSearch, tune

    out = {}
    for name in OTHER_PLANS:
        path = os.path.join(REPO, "mist_amd", "configs", name)
        tune(MistConfig.from_yaml(path))  # warm-up: buffers of this size
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        cost, solution = tune(MistConfig.from_yaml(path))
        torch.cuda.synchronize()
        tune_s = time.perf_counter() - t0
        search = PreparedSearch(MistConfig.from_yaml(path), "cuda:0")
        search.run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        step = search.run()
        torch.cuda.synchronize()
        step_s = time.perf_counter() - t0
        assert step == (cost, solution)
        counts = search.counts()
        out[name] = dict(
            tune_s=tune_s, step_s=step_s, cost=cost, candidates=counts["candidates"],
            cells=counts["cells"], candidates_per_s=counts["candidates"] / step_s,
            solution_sha256=hashlib.sha256(repr(solution).encode()).hexdigest()[:16],
            grad_accum=solution[0] if solution else None,
            stages=len(solution[1]) if solution else 0,
        )
        del search
        torch.cuda.empty_cache()
    return out


def mip_searches(plans=("gpt-7b-b512-4x8.yaml", "llama-13b-b1024-8x8.yaml"), sample_size=30):
    """``tune()`` with the reference's default granularity at HEAD, ``uniform-device-pp-mip``
    with 30 alpha samples per cell (mist/utils/pareto.py:124-144, inter_tuning_mip.py), then the
    stage assignment.  Whole call from the configuration object (descriptor building included),
    median of 3.  ``tune_s``: as ``tune`` runs it, with the intra-stage tables evaluated where
    the assignment reads them (the layer counts within ``layers_offset`` of a stage count's
    average, on that stage count's mesh); ``tune_all_cells_s``: with every sample of every cell
    of every tensor-parallel candidate, as the reference's IntraStageTuner fills its tables.
    Same cost and strategy either way (asserted)."""
    import hashlib

    import torch
    import yaml

    from mist_amd import tune_one_case
    from mist_amd.config import MistConfig
    from mist_amd.tune_one_case import tune

    out = {}
    for name in plans:
        with open(os.path.join(REPO, "mist_amd", "configs", name)) as f:
            raw = yaml.safe_load(f)
        raw["tuning"].update(tuning_granularity="uniform-device-pp-mip", sample_size=sample_size)
        timing, answers = {}, []
        for key, all_cells in (("tune_all_cells_s", True), ("tune_s", False)):
            tune_one_case.MIP_EVALUATE_ALL_CELLS = all_cells
            try:
                tune(MistConfig(raw))  # warm-up: buffers of this size
                torch.cuda.synchronize()
                times = []
                for _ in range(3):
                    t0 = time.perf_counter()
                    cost, solution = tune(MistConfig(raw))
                    torch.cuda.synchronize()
                    times.append(time.perf_counter() - t0)
            finally:
                tune_one_case.MIP_EVALUATE_ALL_CELLS = False
            timing[key] = sorted(times)[1]
            answers.append((cost, solution))
            torch.cuda.empty_cache()
        assert answers[0] == answers[1], "restricted and full tables give different strategies"
        out[name] = dict(tune_s=timing["tune_s"], tune_all_cells_s=timing["tune_all_cells_s"],
                         sample_size=sample_size, cost=cost,
                         grad_accum=solution[0] if solution else None,
                         stages=len(solution[1]) if solution else 0,
                         solution_sha256=hashlib.sha256(repr(solution).encode()).hexdigest()[:16])
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--sustain-s", type=float, default=2.0,
                    help="seconds the sustained leg repeats the step for (median step time)")
    ap.add_argument("--no-mip", action="store_true",
                    help="skip the 30-sample uniform-device-pp-mip searches")
    ap.add_argument("--no-other-plans", action="store_true",
                    help="skip the tune of the four other benchmark plans")
    ap.add_argument("--no-exhaustive", action="store_true",
                    help="skip the evaluate-every-cell kernel (the unpruned reference point)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy (known HBM traffic to scale the "
                         "FETCH_SIZE / WRITE_SIZE counters of a profiler run against)")
    ap.add_argument("--only-plan", default=None, metavar="YAML",
                    help="profiling aid: run --steps search steps of this plan of mist_amd/configs "
                         "with resident descriptors, print their time and exit (no bench line)")
    ap.add_argument("--only-mip", default=None, metavar="YAML",
                    help="profiling aid: --steps calls of tune() on this plan of mist_amd/configs with "
                         "the uniform-device-pp-mip granularity and 30 samples per cell, print their "
                         "time and exit (no bench line)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}): the search runs on a "
              "single MI355X and nothing here uses a second device", file=sys.stderr)
        sys.exit(2)

    import torch

    from mist_amd import _lib
    from mist_amd.config import MistConfig
    from mist_amd.tune_one_case import PreparedSearch, tune

    if not os.path.exists(_lib.LIB_PATH):
        from mist_amd.build import build_library

        build_library()
    _lib.load()
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU: the search kernels have no CPU path")
    torch.cuda.set_device(0)

    if args.only_plan:
        search = PreparedSearch(MistConfig.from_yaml(os.path.join(REPO, "mist_amd", "configs", args.only_plan)), "cuda:0")
        for _ in range(max(args.warmup, 1)):
            search.run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            cost, solution = search.run()
        torch.cuda.synchronize()
        print(json.dumps(dict(plan=args.only_plan, steps=args.steps, cost=cost,
                              ms_per_step=1e3 * (time.perf_counter() - t0) / args.steps, **search.counts())))
        return

    if args.only_mip:
        import yaml

        with open(os.path.join(REPO, "mist_amd", "configs", args.only_mip)) as f:
            raw = yaml.safe_load(f)
        raw["tuning"].update(tuning_granularity="uniform-device-pp-mip", sample_size=30)
        for _ in range(max(args.warmup, 1)):
            tune(MistConfig(raw))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            cost, solution = tune(MistConfig(raw))
        torch.cuda.synchronize()
        print(json.dumps(dict(plan=args.only_mip, steps=args.steps, cost=cost, sample_size=30,
                              ms_per_tune=1e3 * (time.perf_counter() - t0) / args.steps)))
        return

    cfg = MistConfig.from_yaml(PLAN)
    search = PreparedSearch(cfg, "cuda:0")
    counts = search.counts()

    for _ in range(args.warmup):
        search.run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    stats = {}
    for _ in range(args.steps):
        cost, solution = search.run(stats)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = 1e3 * elapsed / args.steps

    # Sustained: the same step for at least two seconds, the median of the per-step wall times
    # (each step ends with the strategy on the host, i.e. with a device synchronisation).
    sustained = []
    t_end = time.perf_counter() + args.sustain_s
    while time.perf_counter() < t_end or len(sustained) < 3:
        t1 = time.perf_counter()
        search.run()
        sustained.append(time.perf_counter() - t1)
    sustained_ms = 1e3 * sorted(sustained)[len(sustained) // 2]

    # The two halves of a step timed apart (a device synchronisation between them, so their sum
    # is slightly above the step time).
    split = {}
    for _ in range(5):
        search.run(split, split_timing=True)
    torch.cuda.synchronize()

    # End-to-end: configuration object -> strategy, including descriptor building and upload
    # (median of 7 calls).
    e2e = []
    for _ in range(7):
        t0 = time.perf_counter()
        e2e_cost, e2e_solution = tune(MistConfig.from_yaml(PLAN))
        torch.cuda.synchronize()
        e2e.append(time.perf_counter() - t0)
        assert (e2e_cost, e2e_solution) == (cost, solution)
    tune_end_to_end_s = sorted(e2e)[len(e2e) // 2]

    # Roofline of the dominant kernel, measured with events on the launch stream.  (The plan's
    # problem record is as the steps above left it: with the stage-cost estimate of tune().)
    def time_kernels(tuner, plan, dev_plan, reps):
        ms = {}
        for rep in range(reps + 1):
            events = []
            tables = tuner.allocate_tables()
            tuner.launch(plan, dev_plan, tables, events=events)
            torch.cuda.synchronize()
            if rep == 0:
                continue  # warm-up of the separately launched entry points
            for name, start, end in events:
                ms[name] = ms.get(name, 0.0) + start.elapsed_time(end) / reps
        return ms

    kernel_ms = time_kernels(search.tuner, search.plan, search.dev_plan, 2)
    counters = profile_counters()
    # the counters belong to the kernel sources and the launch decomposition they were taken
    # with: a profile of other sources or another grid gives no executed-work figures
    # (the launch pads its grid to whole runs of 16 workgroups on each of the 8 XCDs)
    main_waves = -(-int(search.plan["reduce_prefix"][-1]) // 128) * 128
    counters_stale = bool(counters) and (
        counters.pop("_source_sha256", None) != kernel_source_sha256()
        or int(counters.get("SQ_WAVES", {}).get("exhaustive", -1)) != main_waves)
    if counters_stale:
        counters = {}
    algorithmic = float(reduce_kernel_flops(search.plan, search.L))
    peak = FP64_VECTOR_PEAK / 1e12

    def hbm_bytes(which):
        if "FETCH_SIZE" not in counters or "WRITE_SIZE" not in counters:
            return None
        scale_f = counters.get("FETCH_SCALE", {}).get(which, 1.0)
        scale_w = counters.get("WRITE_SCALE", {}).get(which, 1.0)
        return int((counters["FETCH_SIZE"][which] * scale_f + counters["WRITE_SIZE"][which] * scale_w) * 1024)

    def roofline_of(kernel, which, ms):
        executed, lanes = executed_fp64_flops(counters, which) if counters else (None, None)
        traffic = hbm_bytes(which)
        sec = ms * 1e-3
        r = dict(
            bound="fp64-valu", kernel=kernel, avg_launch_ms=ms, peak=peak, unit="TFLOP/s",
            algorithmic_flop_per_launch=algorithmic, algorithmic_tflops=algorithmic / sec / 1e12,
            traffic=traffic,
        )
        if executed is not None:
            r.update(executed_fp64_flop_per_launch=executed, active_lanes_per_valu_inst=lanes)
        if traffic is not None:
            r["hbm"] = dict(achieved=traffic / sec / 1e9, peak=8000.0, unit="GB/s",
                            frac=traffic / sec / 8e12)
        if "SQ_ACTIVE_INST_VALU" in counters:
            # share of the VALU cycles of the chip (1024 SIMDs at 2.4 GHz; the counter is in
            # units of 4 cycles) in which a VALU instruction of this launch was executing
            r["valu_wave_insts"] = counters["SQ_INSTS_VALU"][which]
            r["valu_busy_frac"] = counters["SQ_ACTIVE_INST_VALU"][which] * 4 / (1024 * 2.4e9 * sec)
        return r, executed

    roofline, executed = roofline_of("eval_reduce_kernel (first estimate, scout and main launch of one call)", "pruned",
                                     kernel_ms["eval_reduce"])
    # achieved = what the pruned kernel EXECUTES (it skips most cells exactly); the reference's
    # per-cell formulas over the same time are reported as pruning_gain (> 1 by design)
    roofline["achieved"] = (executed if executed is not None else 0.0) / (kernel_ms["eval_reduce"] * 1e-3) / 1e12
    roofline["frac"] = roofline["achieved"] / peak if executed is not None else None
    roofline["pruning_gain"] = roofline["algorithmic_tflops"] / peak
    roofline["counters_from"] = os.path.relpath(PROFILE, REPO) if counters else None
    roofline["counters_stale"] = counters_stale
    exhaustive = None
    if not args.no_exhaustive:
        full = PreparedSearch(cfg, "cuda:0", exhaustive=True)
        full_ms = time_kernels(full.tuner, full.plan, full.dev_plan, 2)
        exhaustive, ex_exec = roofline_of("eval_reduce_exhaustive_kernel", "exhaustive", full_ms["eval_reduce"])
        # every cell is evaluated: the algorithmic operations are what is done
        exhaustive["achieved"] = exhaustive["algorithmic_tflops"]
        exhaustive["frac"] = exhaustive["achieved"] / peak
        if ex_exec is not None:
            exhaustive["executed_frac"] = ex_exec / (full_ms["eval_reduce"] * 1e-3) / FP64_VECTOR_PEAK
        exhaustive["cells_per_s"] = counts["cells"] / (full_ms["eval_reduce"] * 1e-3)
        exhaustive["candidates_per_s"] = counts["candidates"] / (full_ms["eval_reduce"] * 1e-3)
        del full
    kernel_ms = {k: 2 * v for k, v in kernel_ms.items()}  # (the report below halves two repetitions)
    intra_ms_per_step = sum(kernel_ms.values()) / 2
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    result = {
        "metric": "candidate configs evaluated/sec (fp64), GPT-7B space",
        "value": counts["candidates"] * args.steps / elapsed,
        "unit": "candidates/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": {
            "workload": "GPT-7B plan: 32 layers, hidden 4096, global batch 512, 4x8 devices, "
                        "offload step 0.1, micro-batch {1,2,4,8}, ZeRO 0-3, inter-stage DP",
            "plan": os.path.basename(PLAN),
            "groups": counts["groups"], "rows": counts["rows"],
            "candidates": counts["candidates"], "cells": counts["cells"],
        },
        "cells_per_s": counts["cells"] * args.steps / elapsed,
        "tune_time_s": ms_per_step / 1e3,
        "tune_end_to_end_s": tune_end_to_end_s,
        "intra_kernels_ms_per_step": intra_ms_per_step,
        "intra_kernel_ms": {k: v / 2 for k, v in kernel_ms.items()},
        # wall time of the two halves of a step, measured on 5 extra steps with a device
        # synchronisation between them: the intra-stage launches until the tables are complete,
        # then the inter-stage search (bottleneck DP, threshold windows, scan batches,
        # back-pointers) until the strategy is on the host
        "intra_stage_ms_per_step": 1e3 * split["intra_launch_s"] / 5,
        "inter_stage_ms_per_step": 1e3 * split["inter_s"] / 5,
        "sustained": {"seconds": args.sustain_s, "steps": len(sustained), "median_ms_per_step": sustained_ms,
                      "candidates_per_s": counts["candidates"] / (sustained_ms * 1e-3)},
        "dp_thresholds_per_step": stats.get("dp_thresholds", 0) / args.steps,
        # tune() lets the intra-stage kernels skip stage costs its search cannot use, from an
        # estimate of the best cost that the scout pass leaves; a step whose result the estimate
        # does not cover is evaluated again without it (none expected here)
        "stage_cost_estimate": (float(search.dev_plan["incumbent"].item())
                                if "incumbent" in search.dev_plan else None),
        "stage_cost_cutoff_retries": stats.get("stage_cost_cutoff_retries", 0),
        # (tp, G) pairs of the timed steps whose partition inside the limit of the tables under
        # the estimate the search could not rule out (each makes a step evaluate twice)
        "dp_unresolved": stats.get("dp_unresolved", 0),
        "best_cost": cost,
        "best_solution": repr(solution),
        "roofline": roofline,
        "exhaustive": exhaustive,
    }
    if not args.no_mip:
        result["mip_30_samples"] = mip_searches()
    if not args.no_other_plans:
        result["other_plans"] = other_plans()
    if not args.no_cpu_baseline:
        from mist_amd.layer_tables import LayerTables

        tp1 = search.tuner.run_prepared(search.plan, search.dev_plan)[0]
        result["cpu_baseline"] = cpu_baseline(cfg, LayerTables(cfg), results=tp1)
        result["cpu_baseline"]["host_cpu_count"] = os.cpu_count()
        if "dp" in result["cpu_baseline"]:
            # the GPU side of the same unit: DP instances of a step over the wall time of the
            # inter-stage half of a step
            result["cpu_baseline"]["dp"]["gpu_value"] = (
                result["dp_thresholds_per_step"] / (result["inter_stage_ms_per_step"] * 1e-3))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
