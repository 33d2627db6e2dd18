"""Analysis path: predicted iteration latency and peak memory of ONE given strategy.

Drop-in for the reference's ``benchmark/mist/analysis/run.py`` (``analyze`` :37-185) and for the
``get_best_solution=False`` mode of ``batched_stage_analyze``
(mist/analyzer/batched_module_analyzer.py:687-3144, result entries :2788-2803, 2876-2892,
2980-2996, 3063-3079).  The strategy comes from the ``strategy`` block of the configuration, in
the form ``tune_one_case`` writes it.

A stage is one group descriptor whose search space is the single given row; the row-terms kernel
and ``mist_stage_analyze`` evaluate it on the GPU with the code the search uses (there is no CPU
path).  The per-cell dictionaries hold what the reference's hold: ``latency``, ``mem_fwd_peak``,
``mem_bwd_peak`` and the 135 debugging entries of ``get_extra_info`` (:2401-2749), among them
the stable / delta latency of each variant (``****latency_stable`` ..., :2550-2567) that the
driver reads; ``analyze`` itself asks for those few only.  The reference indexes the per-row
arrays of ``get_extra_info`` with the layer index, which only works for a single candidate
number of layers; here every cell reports its row's values.  As in the reference the pre/post layer strategy is ``strategy.pre_post_strategy``
(``preset``, ``dp``, ``intra-node-tp-*`` or ``tuned``), nothing is masked by the memory capacity,
and a pre/post batch size outside 1..4 yields empty dictionaries (:868-880).
"""
from __future__ import annotations

import argparse
import ctypes
from typing import Any, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib
from .comm_model import gpu_gpu_comm_latency
from .config import BATCH_SIZE_CANDIDATES, MistConfig
from .layer_tables import LayerTables
from .node_database import layer_tables_for
from .search_space import SearchSpace
from .stage_inputs import GroupInputBuilder, make_problem, pre_post_strategy_fields

_VARIANT_KEYS = ("", "_with_pre", "_with_post", "_with_pre_and_post")


def _single_row_space(row: Sequence[float]) -> SearchSpace:
    return SearchSpace(
        par=np.array([list(row[:6])], dtype=np.float64),
        wo=(float(row[6]),), go=(float(row[7]),), oo=(float(row[8]),), ao=(float(row[9]),),
        pair_wo=np.zeros(1, dtype=np.uint8), pair_go=np.zeros(1, dtype=np.uint8),
    )


def _pre_post_batch_ok(config: MistConfig, n: int, m: int, G: int, row) -> bool:
    """batched_module_analyzer.py:862-880."""
    pp_dp = pre_post_strategy_fields(config, n, m, row)[0]
    b = config.training.global_batch_size // G // pp_dp
    return 1 <= b <= max(BATCH_SIZE_CANDIDATES)


class StageDiagnostics:
    """Everything ``get_extra_info`` reports for one stage's strategy row: the row terms and the
    intermediate quantities behind them (device), the descriptor's table look-ups and a few more
    of the same kind that only the debugging entries show (host)."""

    def __init__(self, config: MistConfig, tables: LayerTables, builder: GroupInputBuilder, rec,
                 terms: np.ndarray, diag: np.ndarray, n: int, m: int, G: int, row):
        self.rec, self.terms, self.diag, self.G = rec, terms, diag, G
        self.p2p = _p2p_output_latency(config, tables, m, row)
        fb, ftp = np.float64(row[0]), np.float64(row[2])
        self.fwd_peak_ck = float(tables.mem_peak("block", "fwd", fb, ftp, True))
        pp_dp, pp_tp, pp_wre, pp_gre, pp_ore, _wo, _go, _oo, _ac = pre_post_strategy_fields(config, n, m, row)
        pp_b = config.training.global_batch_size // G // pp_dp
        pb, ptp = np.float64(pp_b), np.float64(pp_tp)
        self.pre_O = float(tables.mem_full_states("pre", "opts", ptp))
        self.post_O = float(tables.mem_full_states("post", "opts", ptp))
        self.post_saved = float(tables.mem_saved("post", False, pb, ptp))
        # amortized pre / post collectives (:1077-1138)
        pre_AR = builder._gpu_gpu("all_reduce", float(rec["pre_full_g"]), pp_dp, n)
        post_AR = builder._gpu_gpu("all_reduce", float(rec["post_full_g"]), pp_dp, n)
        G64 = G
        amortized = lambda flag, v: v if flag else v / G64
        sync = lambda rs, ar: ar / G64 if not pp_ore else amortized(pp_gre, rs)
        self.pre_AG_amortized = amortized(pp_wre, float(rec["pre_ag"]))
        self.post_AG_amortized = amortized(pp_wre, float(rec["post_ag"]))
        self.pre_sync_amortized = sync(float(rec["pre_rs"]), pre_AR)
        self.post_sync_amortized = sync(float(rec["post_rs"]), post_AR)

    def extra_info(self, c: int, values: np.ndarray, module_memory: np.ndarray) -> Dict[str, float]:
        """``values``: float64[4][5] of the cell (variant x (stable, delta, ...)); ``module_memory``:
        (forward states, backward states, saved activations of one micro-batch)."""
        T, D = _lib.TERM, _lib.DIAG
        t, d, rec = self.terms, self.diag, self.rec
        par = rec["par"][0]
        P = _lib.PAR
        fam = {name: d[_lib.DIAG_FAMILIES + 5 * j: _lib.DIAG_FAMILIES + 5 * j + 5]
               for j, name in enumerate(_lib.DIAG_FAMILY_NAMES)}
        M = {m: i for i, m in enumerate(_lib.DIAG_MEMBERS)}
        last = "ck" if c > 0 else "nock"
        e = {
            "*****memory_factor": t[T["mf"]],
            "*****mem_per_full_weight_buffer": d[D["Wbuf"]],
            "*****mem_per_full_grad_buffer": d[D["Gbuf"]],
            "****non_overlapped_post_weights_all_gather_latency": t[T["nAG_" + last]],
            "****non_overlapped_post_grad_sync_latency": t[T["nRS_" + last]],
            "****overlapped_post_bwd_latency": t[T["opb"]],
        }
        for k, ck_name in (("nock", "without_ckpt"), ("ck", "with_ckpt")):
            stars = "**" if k == "nock" else "*"
            for ph, mb in (("first", "first"), ("later", "not_first")):
                f = fam[f"fwd_{ph}_{k}"]
                e[f"****latency_first_layer_critical_fwd_{mb}_micro_batch_{ck_name}"] = f[M["first"]]
                e[f"****latency_last_layer_critical_fwd_{mb}_micro_batch_{ck_name}"] = f[M["last"]]
                e[f"****latency_extra_pre_fwd_{mb}_micro_batch_{ck_name}"] = f[M["extra_pre"]]
                e[f"****latency_extra_post_fwd_{mb}_micro_batch_{ck_name}"] = f[M["extra_post"]]
                e[f"{stars}_latency_layer_critical_fwd_{mb}_micro_batch_{ck_name}"] = f[M["layer"]]
            for ph, mb in (("last", "last"), ("not_last", "not_last")):
                f = fam[f"bwd_{ph}_{k}"]
                e[f"****latency_last_layer_critical_bwd_{mb}_micro_batch_{ck_name}"] = f[M["last"]]
                e[f"****latency_first_layer_critical_bwd_{mb}_micro_batch_{ck_name}"] = f[M["first"]]
                e[f"****latency_extra_pre_bwd_{mb}_micro_batch_{ck_name}"] = f[M["extra_pre"]]
                e[f"****latency_extra_post_bwd_{mb}_micro_batch_{ck_name}"] = f[M["extra_post"]]
                e[f"{stars}_latency_layer_critical_bwd_{mb}_micro_batch_{ck_name}"] = f[M["layer"]]
            e[f"****latency_layer_critical_stable_{ck_name}"] = t[T["s_layer_" + k]]
            e[f"****latency_layer_critical_delta_{ck_name}"] = t[T["d_layer_" + k]]
            e[f"****latency_pre_fwd_and_post_bwd_and_first_layer_stable_{ck_name}"] = t[T["s_first_" + k]]
            e[f"****latency_post_fwd_and_pre_bwd_and_last_layer_stable_{ck_name}"] = t[T["s_last_" + k]]
            e[f"****latency_pre_fwd_and_post_bwd_and_first_layer_delta_{ck_name}"] = t[T["d_first_" + k]]
            e[f"****latency_post_fwd_and_pre_bwd_and_last_layer_delta_{ck_name}"] = t[T["d_last_" + k]]
        for w, key in enumerate(_VARIANT_KEYS):
            e["****latency_stable" + key] = values[w][0]
            e["****latency_delta" + key] = values[w][1]
        exec_fwd, exec_bwd = par[P["exec_fwd"]], par[P["exec_bwd"]]
        e.update({
            "_latency_pre_fwd_latency": rec["pre_fwd"],
            "_latency_pre_bwd_latency": rec["pre_bwd"],
            "_latency_pre_weights_all_gather_latency": rec["pre_ag"],
            "_latency_pre_weights_all_gather_latency_amortized": self.pre_AG_amortized,
            "_latency_pre_grad_sync_latency": rec["pre_rs"],
            "_latency_pre_grad_sync_amortized": self.pre_sync_amortized,
            "_latency_post_fwd_latency": rec["post_fwd"],
            "_latency_post_bwd_latency": rec["post_bwd"],
            "_latentcy_post_weights_all_gather_latency_amortized": self.post_AG_amortized,
            "_latency_post_grad_sync_amortized": self.post_sync_amortized,
            "_latency_post_grad_sync_latency": rec["post_rs"],
            "_latency_post_weights_all_gather_latency": rec["post_ag"],
            "_latency_layer_exec_fwd": exec_fwd,
            "_latency_layer_exec_bwd_without_ckpt": exec_bwd,
            "_latency_layer_exec_bwd_with_ckpt": exec_fwd + exec_bwd,
            "_latency_layer_gpu_to_cpu_fwd_first_micro_batch_exclude_act": d[D["g2c_F0"]],
            "_latency_layer_cpu_to_gpu_fwd_first_micro_batch_exclude_act": d[D["c2g_F0"]],
            "_latency_layer_gpu_gpu_fwd_first_micro_batch_exclude_act": d[D["g2g_F0"]],
            "_latency_layer_gpu_to_cpu_fwd_not_first_micro_batch_exclude_act": d[D["g2c_F1"]],
            "_latency_layer_cpu_to_gpu_fwd_not_first_micro_batch_exclude_act": d[D["c2g_F1"]],
            "_latency_layer_gpu_gpu_fwd_not_first_micro_batch_exclude_act": d[D["g2g_F1"]],
            "_latency_layer_gpu_to_cpu_bwd_last_micro_batch_exclude_act": d[D["g2c_B"]],
            "_latency_layer_cpu_to_gpu_bwd_last_micro_batch_exclude_act": d[D["c2g_B"]],
            "_latency_layer_gpu_gpu_bwd_last_micro_batch_exclude_act": d[D["g2g_B0"]],
            "_latency_layer_gpu_to_cpu_bwd_not_last_micro_batch_exclude_act": d[D["g2c_B"]],
            "_latency_layer_cpu_to_gpu_bwd_not_last_micro_batch_exclude_act": d[D["c2g_B"]],
            "_latency_layer_gpu_gpu_bwd_not_last_micro_batch_exclude_act": d[D["g2g_B1"]],
            "_latency_layer_swap_out_weights": d[D["so_W"]],
            "_latency_layer_swap_in_weights": d[D["si_W"]],
            "_latency_layer_all_gather_weights": d[D["AG_w"]],
            "_latency_layer_swap_in_grads": d[D["si_G"]],
            "_latency_layer_swap_in_activations_with_ckpt": d[D["si_A_ck"]],
            "_latency_layer_swap_in_activations_without_ckpt": d[D["si_A_nock"]],
            "_latency_layer_swap_out_grads": d[D["so_G"]],
            "_latency_layer_swap_out_activations_with_ckpt": d[D["so_A_ck"]],
            "_latency_layer_swap_out_activations_without_ckpt": d[D["so_A_nock"]],
            "_latency_layer_reduce_scatter_grads": d[D["RS_g"]],
            "_latency_layer_bwd_all_gather_saved_with_ckpt": 0.0,  # saved tensors are not partitioned (:1355-1356)
            "_latency_p2p_output": self.p2p,
            "_mem_layer_full_weights": par[P["W"]],
            "_mem_layer_full_grads": par[P["G"]],
            "_mem_layer_full_opts": par[P["O"]],
            "_mem_layer_partial_weights": d[D["pW"]],
            "_mem_layer_partial_grads": d[D["pG"]],
            "_mem_layer_partial_opts": t[T["pO"]],
            "_mem_layer_saved_with_ckpt": t[T["S_ck"]],
            "_mem_layer_saved_without_ckpt": t[T["S_nock"]],
            "_mem_raw_layer_saved_with_ckpt": par[P["raw_ck"]],
            "_mem_raw_layer_saved_without_ckpt": par[P["raw_nock"]],
            "_mem_layer_fwd_peak_with_ckpt": self.fwd_peak_ck,
            "_mem_layer_fwd_peak_without_ckpt": par[P["fwd_peak"]],
            "_mem_layer_bwd_peak": par[P["bwd_peak"]],
            "_mem_layer_output": par[P["out"]],
            "_mem_module_fwd_saved": module_memory[2],
            "_mem_pre_layer_full_weights": rec["pre_full_w"],
            "_mem_pre_layer_full_grads": rec["pre_full_g"],
            "_mem_pre_layer_full_opts": self.pre_O,
            "_mem_pre_layer_saved_without_ckpt": rec["pre_saved"],
            "_mem_pre_layer_states": rec["pre_states"],
            "_mem_post_layer_full_weights": rec["post_full_w"],
            "_mem_post_layer_full_grads": rec["post_full_g"],
            "_mem_post_layer_full_opts": self.post_O,
            "_mem_post_layer_saved_without_ckpt": self.post_saved,
            "_mem_post_layer_states": rec["post_states"],
            "_mem_post_layer_fwd_peak": rec["post_fwd_peak"],
            "_mem_post_layer_bwd_peak": rec["post_bwd_peak"],
            "_mem_post_layer_output": rec["post_output"],
            "_mem_module_fwd_states": module_memory[0],
            "_mem_module_bwd_states": module_memory[1],
        })
        return {k: float(v) for k, v in e.items()}


def analyze_cells(config: MistConfig, tables: LayerTables, stages, device: str = "cuda:0",
                  diagnostics: bool = False):
    """``stages``: list of ``(num_nodes, num_gpus_per_node, G, strategy_row, [(p, l, c), ...])``.
    Returns per stage a dict ``(p, l, c) -> float64[4][5]`` (variant x (stable, delta, stable +
    delta / G, forward peak, backward peak)), or None for a stage whose pre/post batch size is
    out of range.  One launch of each kernel for all stages.  With ``diagnostics`` the result
    is a pair: that list and, per stage, a function ``(p, l, c) -> dict`` with the entries of
    the reference's ``get_extra_info`` (None where the stage has no result)."""
    dev = torch.device(device)
    if dev.type != "cuda" or not torch.cuda.is_available():
        raise _lib.MistLibraryError("the analysis path needs a GPU: the kernels have no CPU path")
    lib = _lib.load()
    L = int(config.model.num_hidden_layers)
    live = [i for i, (n, m, G, row, _) in enumerate(stages) if _pre_post_batch_ok(config, n, m, G, row)]
    out: List[Optional[Dict[Tuple[int, int, int], np.ndarray]]] = [None] * len(stages)
    if not live:
        return (out, [None] * len(stages)) if diagnostics else out
    builder = GroupInputBuilder(config, tables)
    groups = np.zeros(len(live), dtype=_lib.GROUP_DTYPE)
    requests = []
    for gi, i in enumerate(live):
        n, m, G, row, cells = stages[i]
        builder.fill(groups[gi], _single_row_space(row), 0, gi, n, m, G, 1, analysis_row=row)
        groups[gi]["row_offset"] = gi
        for p, l, c in cells:
            if not (1 <= l <= L and 0 <= c <= l and p >= 0):
                raise ValueError(f"cell (p={p}, l={l}, c={c}) outside 1 <= l <= {L}, 0 <= c <= l, p >= 0")
            requests.append((gi, 0, l, c, p))
    builder.validate(groups)
    if not requests:
        empty = [({} if i in live else None) for i in range(len(stages))]
        return (empty, [None] * len(stages)) if diagnostics else empty
    problem = make_problem(config, L, 1, 1, 1, len(live))
    n_groups = len(live)
    terms_prefix = np.arange(n_groups + 1, dtype=np.int32)  # one workgroup per single-row group
    req = np.asarray(requests, dtype=np.int32)
    with torch.cuda.device(dev):
        to_dev = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1)).to(dev)
        d_groups, d_prefix, d_req = to_dev(groups), to_dev(terms_prefix), to_dev(req)
        row_terms = torch.empty(n_groups * _lib.ROW_TERMS, dtype=torch.float64, device=dev)
        stage_floor = torch.empty(lib.mist_stage_floor_doubles(n_groups, n_groups), dtype=torch.float64, device=dev)
        result = torch.empty((len(requests), _lib.ANALYZE_FIELDS), dtype=torch.float64, device=dev)
        stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        prob_ptr = ctypes.c_void_p(problem.ctypes.data)
        _lib.check(lib.mist_row_terms(prob_ptr, d_groups.data_ptr(), n_groups, d_prefix.data_ptr(),
                                      n_groups, row_terms.data_ptr(), stage_floor.data_ptr(), None, stream),
                   "mist_row_terms")
        _lib.check(lib.mist_stage_analyze(prob_ptr, d_groups.data_ptr(), n_groups, row_terms.data_ptr(),
                                          d_req.data_ptr(), len(requests), result.data_ptr(), stream),
                   "mist_stage_analyze")
        if diagnostics:
            diag_req = to_dev(np.array([(gi, 0) for gi in range(n_groups)], dtype=np.int32))
            diag = torch.empty((n_groups, _lib.DIAG_FIELDS), dtype=torch.float64, device=dev)
            _lib.check(lib.mist_row_diagnostics(prob_ptr, d_groups.data_ptr(), n_groups, diag_req.data_ptr(),
                                                n_groups, diag.data_ptr(), stream), "mist_row_diagnostics")
            h_diag = diag.cpu().numpy()
            h_terms = row_terms.cpu().numpy().reshape(n_groups, _lib.ROW_TERMS)
        everything = result.cpu().numpy()
    host = everything[:, :20].reshape(len(requests), 4, 5)
    for i in live:
        out[i] = {}
    for (gi, _, l, c, p), values in zip(requests, host):
        out[live[gi]][(p, l, c)] = values
    if not diagnostics:
        return out
    extra: List[Any] = [None] * len(stages)
    module_memory = {(gi, p, l, c): everything[j, 20:23] for j, (gi, _, l, c, p) in enumerate(requests)}
    for gi, i in enumerate(live):
        n, m, G, row, _cells = stages[i]
        info = StageDiagnostics(config, tables, builder, groups[gi], h_terms[gi], h_diag[gi], n, m, G, row)
        def of_cell(key, info=info, gi=gi, cells=out[i]):
            p, l, c = key
            return info.extra_info(c, cells[key], module_memory[(gi, p, l, c)])
        extra[i] = of_cell
    return out, extra


def _p2p_output_latency(config: MistConfig, tables: LayerTables, m: int, row) -> float:
    """Twice the p2p latency of the layer output (batched_module_analyzer.py:1298-1308)."""
    out_mb = float(tables.mem_output("block", np.float64(row[0]), np.float64(row[2])))
    across_nodes = m == config.hardware.num_gpus_per_node
    return float(gpu_gpu_comm_latency(
        "p2p", np.float64(out_mb) / 1024, inter_size=1 if across_nodes else None,
        intra_size=None if across_nodes else 1,
        gpu_gpu_comm_params=config.hardware.gpu_gpu_comm_params)) * 2


def _entries(values: np.ndarray, p: int, p2p: float, extra: Optional[Dict[str, float]] = None):
    """The four per-variant dictionaries of one cell; the last two only exist for p == 0.
    ``extra``: the entries of ``get_extra_info``, merged into each of them as the reference
    does; without it only the stable / delta latencies of the variants are added."""
    dicts = []
    for v, suffix in enumerate(_VARIANT_KEYS):
        if v >= 2 and p != 0:
            dicts.append(None)
            continue
        stable, delta, latency, fwd, bwd = (float(x) for x in values[v])
        entry = {
            # the pre-and-post variant carries no p2p term (:3071)
            "latency": latency if v == 3 else latency + p2p,
            "mem_fwd_peak": fwd,
            "mem_bwd_peak": bwd,
        }
        if extra is not None:
            entry.update(extra)
        else:
            for w, key in enumerate(_VARIANT_KEYS):
                if w >= 2 and p != 0:
                    continue
                entry["****latency_stable" + key] = float(values[w][0])
                entry["****latency_delta" + key] = float(values[w][1])
        dicts.append(entry)
    return dicts


def batched_stage_analyze(
    layer_tables: LayerTables,
    pre_saved_micro_batches_candidates: List[int],
    num_layers_candidates: List[int],
    num_ckpt_layers_candidates: List[int],
    num_nodes: int,
    num_gpus_per_node: int,
    gradient_accumulation_steps: int,
    stage_strategies,
    config: MistConfig,
    device: str = "cuda:0",
):
    """``batched_stage_analyze(..., get_best_solution=False)`` of the reference for one strategy
    row (the three ``LayerInfo`` arguments are replaced by ``layer_tables``).  Returns the four
    dictionaries ``results, results_with_pre, results_with_post, results_with_pre_and_post`` keyed
    ``(pre_saved_micro_batches, num_layers, num_ckpt_layers)``."""
    row = np.asarray(stage_strategies, dtype=np.float64).reshape(-1)
    if row.shape[0] != 10:
        raise ValueError("the analysis path takes exactly one strategy row of 10 values")
    cells = [(p, l, c) for c in num_ckpt_layers_candidates for p in pre_saved_micro_batches_candidates
             for l in num_layers_candidates if c <= l]
    (found,), (extra_of,) = analyze_cells(
        config, layer_tables, [(num_nodes, num_gpus_per_node, gradient_accumulation_steps, row, cells)],
        device, diagnostics=True)
    results: Tuple[Dict, Dict, Dict, Dict] = ({}, {}, {}, {})
    if found is None:
        return results
    p2p = _p2p_output_latency(config, layer_tables, num_gpus_per_node, row)
    for (p, l, c), values in found.items():
        for v, entry in enumerate(_entries(values, p, p2p, extra_of((p, l, c)))):
            if entry is not None:
                results[v][(p, l, c)] = entry
    return results


def analyze(mist_config: MistConfig, layer_tables: Optional[LayerTables] = None, device: str = "cuda:0"):
    """run.py:37-185.  Returns ``(total_latency, stage_stable_latencies, stage_delta_latencies,
    stage_peak_memories)``."""
    st = mist_config.strategy
    if st is None or "layer_partitions" not in st:
        raise ValueError("the strategy block is missing or disabled")
    tables = layer_tables_for(mist_config) if layer_tables is None else layer_tables
    S, G = st.num_stages, st.gradient_accumulation_steps
    stages, keys = [], []
    for i in range(S):
        p = min(S - i - 1, G - 1)                                            # run.py:57-59
        l, c = st.layer_partitions[i], st.gradient_checkpointing[i]
        n, m = st.device_assignment[i]
        stages.append((n, m, G, st.stage_strategies[i], [(p, l, c)]))
        keys.append((p, l, c))
    found = analyze_cells(mist_config, tables, stages, device)
    results = []
    for i, (cells, key) in enumerate(zip(found, keys)):
        variant = 3 if S == 1 else (1 if i == 0 else (2 if i == S - 1 else 0))
        entry = None
        if cells is not None:
            p2p = _p2p_output_latency(mist_config, tables, stages[i][1], stages[i][3])
            entry = _entries(cells[key], key[0], p2p)[variant]
        if entry is None:
            raise KeyError(key)  # the reference indexes its empty result dictionary (run.py:84-93)
        results.append((entry, _VARIANT_KEYS[variant]))
    if S == 1:
        entry, _ = results[0]
        total = entry["latency"] * G
        # run.py:113-114 overwrites the stable list with [0] and leaves the delta list empty
        return total, [0], [], [max(entry["mem_fwd_peak"], entry["mem_bwd_peak"])]
    uniform = bool(getattr(mist_config, "disable_non_uniform_pp_micro_batch_analysis", False))
    stable, delta, peaks = [], [], []
    for entry, suffix in results:
        if uniform:
            stable.append(entry["latency"])
            delta.append(0)
        else:
            stable.append(entry["****latency_stable" + suffix])
            delta.append(entry["****latency_delta" + suffix])
        peaks.append(max(entry["mem_fwd_peak"], entry["mem_bwd_peak"]))
    total = sum(stable) + max(stable) * (G - 1)
    if not uniform:
        total = total + max(d - sum(stable[i] for i in range(s)) for s, d in enumerate(delta))
    return total, stable, delta, peaks


def main(argv: Optional[List[str]] = None) -> None:
    parser = argparse.ArgumentParser(description="Predicted latency and peak memory of the strategy block of a plan")
    parser.add_argument("--config", required=True, help="resolved YAML with an enabled strategy block")
    parser.add_argument("--device", default="cuda:0")
    args = parser.parse_args(argv)
    total, stable, delta, peaks = analyze(MistConfig.from_yaml(args.config), device=args.device)
    print(f"Stage Stable Latencies: {stable}")
    print(f"Stage Delta Latencies: {delta}")
    print(f"Total latency: {total}")
    print(f"Peak memory (MB): {peaks}")


if __name__ == "__main__":
    main()
