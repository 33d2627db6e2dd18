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
# HBM bytes of one mist_eval_reduce call (scout, seed merge and main launch) on this workload, from two
# rocprofv3 --pmc runs (FETCH_SIZE 4.572e5 KiB scaled x2.0, WRITE_SIZE 1.526e5 KiB scaled x1.0
# by what a 1 GiB device copy reads on the same counters; profiles/bench_gpt7b_kernel_stats.md).
EVAL_REDUCE_HBM_BYTES = int((4.572e5 * 2.0 + 1.526e5) * 1024)


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


def cpu_baseline(cfg, tables, budget_s=15.0):
    """Times the numpy oracle (a port of the reference's formulation, single thread) on whole
    (G, mesh, tp) groups of the same plan (single-device mesh, about 9 s each) until ``budget_s``
    is used."""
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates
    from oracle.intra import max_pre_saved_micro_batches
    from oracle.stage import batched_tune_best_latency_for_stage

    hw = cfg.hardware
    L = cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    P = max_pre_saved_micro_batches(meshes, Gs, L)
    sample = [(512, (1, 1), 1), (256, (1, 1), 1), (128, (1, 1), 1), (64, (1, 1), 1)]
    done, cand, cells, elapsed = [], 0, 0, 0.0
    for G, (n, m), tp in sample:
        dbg = {}
        t0 = time.perf_counter()
        batched_tune_best_latency_for_stage(
            tables, cfg, list(range(min(G, L, P + 1))), list(range(1, L + 1)), list(range(L + 1)),
            n, m, G, tp_size=tp, sample_size=1, debug=dbg,
        )
        elapsed += time.perf_counter() - t0
        rows = dbg["rows"].shape[0]
        cand += rows * (L + 1)
        cells += rows * (L * (L + 1) // 2 + L) * min(G, L, P + 1)
        done.append(f"G={G} mesh={n}x{m} tp={tp} rows={rows}")
        if elapsed > budget_s:
            break
    return dict(
        value=cand / elapsed, unit="candidates/s", cores=1, kind="port",
        sample="; ".join(done) + f"; {elapsed:.1f} s of numpy, intra-stage evaluation only",
        cells_per_s=cells / elapsed,
    )


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy (known HBM traffic to scale the "
                         "FETCH_SIZE / WRITE_SIZE counters of a profiler run against)")
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

    # The two halves of a step timed apart (a device synchronisation between them, so their sum
    # is slightly above the step time).
    split = {}
    for _ in range(5):
        search.run(split, split_timing=True)
    torch.cuda.synchronize()

    # End-to-end: configuration object -> strategy, including descriptor building and upload.
    t0 = time.perf_counter()
    e2e_cost, e2e_solution = tune(MistConfig.from_yaml(PLAN))
    torch.cuda.synchronize()
    tune_end_to_end_s = time.perf_counter() - t0
    assert (e2e_cost, e2e_solution) == (cost, solution)

    # Roofline of the dominant kernel, measured with events on the launch stream.
    flops = dur_ms = 0.0
    n_launches = 0
    kernel_ms = {}
    for rep in range(3):
        events = []
        tables = search.tuner.allocate_tables()
        search.tuner.launch(search.plan, search.dev_plan, tables, events=events)
        torch.cuda.synchronize()
        if rep == 0:
            continue  # warm-up of the separately launched entry points
        for name, start, end in events:
            kernel_ms[name] = kernel_ms.get(name, 0.0) + start.elapsed_time(end)
        flops += reduce_kernel_flops(search.plan, search.L)
        n_launches += 1
    dur_ms = kernel_ms["eval_reduce"]
    achieved = flops / (dur_ms * 1e-3) / 1e12
    roofline = dict(
        bound="fp64-valu", kernel="eval_reduce_kernel", achieved=achieved,
        peak=FP64_VECTOR_PEAK / 1e12, unit="TFLOP/s", frac=achieved / (FP64_VECTOR_PEAK / 1e12),
        traffic=EVAL_REDUCE_HBM_BYTES, avg_launch_ms=dur_ms / n_launches,
        flop_per_launch=flops / n_launches, launches_per_step=1,
        # the HBM side alongside: measured traffic of the launch pair over its duration
        hbm=dict(achieved=EVAL_REDUCE_HBM_BYTES / (dur_ms / n_launches * 1e-3) / 1e9, peak=8000.0,
                 unit="GB/s", frac=EVAL_REDUCE_HBM_BYTES / (dur_ms / n_launches * 1e-3) / 8e12),
        note="achieved = ALGORITHMIC flops (the reference's formulas for every cell) / time; the "
             "kernel prunes exactly and executes a fraction of them, so frac can exceed 1 "
             "(executed: 8.7e8 VALU wave-instructions per call, 39 % of the issue slots, in the "
             "rocprofv3 --pmc run under profiles/)",
    )
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
        "dp_thresholds_per_step": stats.get("dp_thresholds", 0) / args.steps,
        "best_cost": cost,
        "best_solution": repr(solution),
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        from mist_amd.layer_tables import LayerTables

        result["cpu_baseline"] = cpu_baseline(cfg, LayerTables(cfg))
        result["cpu_baseline"]["host_cpu_count"] = os.cpu_count()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
