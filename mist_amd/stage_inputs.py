"""Host-side preparation of the kernel inputs for one (G, mesh) group.

Everything here is O(1) per group or O(#parallelism rows): the pre / post layer scalars
(reference: mist/analyzer/batched_module_analyzer.py:777-1138), the per-(b, tp) table look-ups
(:1216-1297), the op-latency aggregation (:259-414) and the 11 x 4 interference factor table
(mist/tools/optimize.py:951-964,1027-1074).  The per-candidate work is done by the HIP kernels.

All arithmetic is float64 in the reference's operation order so that the kernel inputs are
bit-identical to what the numpy formulation derives for the same group.
"""
from __future__ import annotations

from functools import lru_cache
from typing import Tuple

import numpy as np

from . import _lib
from .comm_model import gpu_gpu_comm_latency
from .config import MistConfig, frag_factor
from .layer_tables import LayerTables
from .search_space import SearchSpace

GB = 1 << 30
MB = 1 << 20

THREE_CASE_MASKS = (
    (True, True, True, False),
    (True, True, False, True),
    (True, False, True, True),
    (False, True, True, True),
)
TWO_CASE_MASKS = (
    (True, True, False, False),
    (True, False, True, False),
    (True, False, False, True),
    (False, True, True, False),
    (False, True, False, True),
    (False, False, True, True),
)


def interference_factor_table(params) -> np.ndarray:
    """(11, 4) factors in evaluation order: 4-way (params[0:4]), 3-way (params[4:16], three per
    mask in position order), 2-way (params[16:28]); 1 outside the mask."""
    params = [float(x) for x in params]
    if len(params) != 28:
        raise ValueError(f"Length: {len(params)}. It should be 28.")
    table = np.ones((11, 4), dtype=np.float64)
    table[0] = params[:4]
    cursor = 4
    for row, mask in enumerate(THREE_CASE_MASKS + TWO_CASE_MASKS, start=1):
        for pos in range(4):
            if mask[pos]:
                table[row, pos] = params[cursor]
                cursor += 1
    assert cursor == 28
    return table


def latency_exec(
    tables: LayerTables, kind: str, b: int, tp: int, inter_size, intra_size, grad_accum_steps: int
) -> Tuple[float, float, float, float]:
    """Op-latency aggregation of one layer, reference ``_single_get_concrete_latency_exec``
    (batched_module_analyzer.py:324-414): backward clamp ``bwd > 2.3*fwd -> 2*fwd``, drop of ops
    with ``fwd < 5e-5 or bwd < 1e-4`` and the gradient-accumulation term."""
    fwd_latencies = 0
    bwd_latencies = 0
    extra_fwd_latencies = 0
    extra_bwd_latencies = 0
    for fwd, bwd, extra_fwd, extra_bwd in tables.op_profiles(kind, b, tp, inter_size, intra_size):
        if bwd != 0 and bwd > 2.3 * fwd:
            bwd = fwd * 2
        fwd += extra_fwd
        bwd += extra_bwd
        if fwd < 5e-5 or bwd < 1e-4:
            continue
        fwd_latencies += fwd
        bwd_latencies += bwd
        extra_fwd_latencies += extra_fwd
        extra_bwd_latencies += extra_bwd
    for grad_accumu in tables.grad_accum_profiles(kind, b, tp):
        bwd_latencies += grad_accumu * (grad_accum_steps - 1) / grad_accum_steps
    return (
        float(fwd_latencies),
        float(bwd_latencies),
        float(extra_fwd_latencies),
        float(extra_bwd_latencies),
    )


def pre_post_strategy_fields(config: MistConfig, num_nodes: int, num_gpus_per_node: int,
                             analysis_row=None):
    """(dp, tp, wre, gre, ore, wo, go, oo, ac) of the pre / post layers
    (batched_module_analyzer.py:777-845).  The tuning path reads ``tuning.pre_post_strategy``; the
    analysis path (``analysis_row`` = the strategy row) reads ``strategy.pre_post_strategy`` and
    also knows ``tuned`` (the row's own parallelism, :789-799)."""
    if analysis_row is None:
        strategy = config.tuning.pre_post_strategy
    else:
        if config.strategy is None:
            raise ValueError("the analysis path needs an enabled strategy block")
        strategy = config.strategy.pre_post_strategy
        if strategy == "tuned":
            r = analysis_row
            return int(r[1]), int(r[2]), bool(r[3]), bool(r[4]), bool(r[5]), 0.0, 0.0, 0.0, 0.0
    if strategy == "preset":
        if config.strategy is None:
            raise ValueError(
                "pre_post_strategy 'preset' reads strategy.pre_post_strategy_array, "
                "but the strategy block is disabled"
            )
        a = config.strategy.pre_post_strategy_array
        return int(a[1]), int(a[2]), bool(a[3]), bool(a[4]), bool(a[5]), float(a[6]), float(a[7]), float(a[8]), float(a[9])
    if strategy == "dp":
        return num_nodes * num_gpus_per_node, 1, False, False, True, 0.0, 0.0, 0.0, 0.0
    if strategy in ("intra-node-tp-with-ore", "intra-node-tp-without-ore"):
        ore = strategy == "intra-node-tp-with-ore"
        return num_nodes, num_gpus_per_node, False, True, ore, 0.0, 0.0, 0.0, 0.0
    raise NotImplementedError(f"config.tuning.pre_post_strategy: {strategy}")


def make_problem(
    config: MistConfig, num_layers: int, p_dim: int, sample_size: int, num_grad_accum: int,
    num_mesh: int,
) -> np.ndarray:
    """One ``MistProblem`` record (numpy structured scalar array of shape (1,))."""
    hw = config.hardware
    prob = np.zeros(1, dtype=_lib.PROBLEM_DTYPE)
    prob["gpu_gpu"][0] = hw.gpu_gpu_comm_params
    prob["cpu_gpu"][0] = hw.cpu_gpu_comm_params
    prob["gpu_cpu"][0] = hw.gpu_cpu_comm_params
    prob["interf_factor"][0] = interference_factor_table(hw.interference_model_params)
    prob["mem_cap_mb"] = hw.memory_capacity * GB / MB
    prob["frag_factor"] = frag_factor(config)
    prob["num_layers"] = num_layers
    prob["p_dim"] = p_dim
    prob["sample_size"] = sample_size
    prob["num_grad_accum"] = num_grad_accum
    prob["num_mesh"] = num_mesh
    prob["adv_first_block"] = 1 if config.enable_advanced_opt_in_first_block else 0
    bandwidths = np.concatenate([prob["gpu_gpu"][0][0::2], prob["cpu_gpu"][0][:1], prob["gpu_cpu"][0][:1]])
    offsets = np.concatenate([prob["gpu_gpu"][0][1::2], prob["cpu_gpu"][0][1:], prob["gpu_cpu"][0][1:]])
    if not (np.all(np.isfinite(bandwidths)) and np.all(bandwidths > 0)):
        raise ValueError("communication bandwidths (k of every (k, b) pair) must be positive and finite")
    if not (np.all(np.isfinite(offsets)) and np.all(offsets >= 0)):
        raise ValueError("communication latencies (b of every (k, b) pair) must be non-negative and finite")
    factors = prob["interf_factor"][0]
    if not (np.all(np.isfinite(factors)) and np.all(factors > 0)):
        raise ValueError("interference factors must be positive and finite")
    if not (np.isfinite(prob["mem_cap_mb"][0]) and prob["mem_cap_mb"][0] > 0):
        raise ValueError("memory capacity must be positive and finite")
    return prob


def _partial(full, shard, ratio):
    # get_concrete_mem_partial_states (batched_module_analyzer.py:143-153)
    return np.float64(full) / np.float64(shard) * (np.float64(1) - np.float64(ratio))


class GroupInputBuilder:
    """Builds ``MistGroupDesc`` records; caches table look-ups across groups."""

    def __init__(self, config: MistConfig, tables: LayerTables):
        self.config = config
        self.tables = tables
        self.hw = config.hardware
        self._exec = lru_cache(maxsize=None)(self._exec_uncached)
        self._block = lru_cache(maxsize=None)(self._block_uncached)
        self._par_fields = lru_cache(maxsize=None)(self._par_fields_uncached)
        self._pre_post = lru_cache(maxsize=None)(self._pre_post_uncached)

    def _exec_uncached(self, kind, b, tp, inter, intra, G):
        return latency_exec(self.tables, kind, b, tp, inter, intra, G)

    def _block_uncached(self, b: int, tp: int):
        t = self.tables
        fb, ftp = np.float64(b), np.float64(tp)
        gcb = 0.0
        if not self.config.model.use_flash_attn:
            # batched_module_analyzer.py:1203-1213
            gcb = float(
                2
                * fb
                * self.config.model.num_attention_heads
                / ftp
                * (self.config.training.max_sequence_length**2)
                / (1024**2)
            )
        return dict(
            W=float(t.mem_full_states("block", "weights", ftp)),
            G=float(t.mem_full_states("block", "grads", ftp)),
            O=float(t.mem_full_states("block", "opts", ftp)),
            raw_ck=float(t.mem_saved("block", True, fb, ftp)),
            raw_nock=float(t.mem_saved("block", False, fb, ftp)),
            fwd_peak=float(t.mem_peak("block", "fwd", fb, ftp, False)),
            bwd_peak=float(t.mem_peak("block", "bwd", fb, ftp)),
            out=float(t.mem_output("block", fb, ftp)),
            gcb=gcb,
        )

    def _par_fields_uncached(self, b: int, tp: int, gpus_per_node: int, grad_accum: int) -> np.ndarray:
        """The table look-ups of a parallelism row (``MIST_PAR_*`` fields from W on; the six
        strategy fields in front stay zero) - the same (b, tp) recurs in most groups of a plan."""
        P, m = _lib.PAR, gpus_per_node
        v = np.zeros(_lib.PAR_FIELDS, dtype=np.float64)
        for name, value in self._block(b, tp).items():
            v[P[name]] = value
        inter = tp // m if tp > m else 1
        intra = m if tp > m else tp
        fwd, bwd, efwd, ebwd = self._exec("block", b, tp, inter, intra, grad_accum)
        v[P["exec_fwd"]], v[P["exec_bwd"]] = fwd, bwd
        v[P["extra_fwd"]], v[P["extra_bwd"]] = efwd, ebwd
        return v

    def _gpu_gpu(self, op_name: str, mbytes: float, dp: int, num_nodes: int) -> float:
        inter = num_nodes if dp > num_nodes else dp
        intra = dp // num_nodes if dp > num_nodes else 1
        return float(
            gpu_gpu_comm_latency(
                op_name, np.float64(mbytes) / 1024, inter_size=inter, intra_size=intra,
                gpu_gpu_comm_params=self.hw.gpu_gpu_comm_params,
            )
        )

    def fill(
        self, rec: np.void, space: SearchSpace, g_index: int, q_index: int, num_nodes: int,
        num_gpus_per_node: int, grad_accum: int, num_p: int, analysis_row=None,
    ) -> None:
        """Fills one record of a ``GROUP_DTYPE`` array (decomposition fields are set later; the
        caller runs ``validate`` over the filled records)."""
        cfg, t = self.config, self.tables
        n, m, G = num_nodes, num_gpus_per_node, grad_accum
        rec["g_index"], rec["q_index"] = g_index, q_index
        rec["num_nodes"], rec["num_gpus_per_node"] = n, m
        rec["grad_accum"], rec["num_p"] = G, num_p
        rec["n_par"], rec["n_pair"] = space.n_par, space.n_pair
        rec["n_oo"], rec["n_ao"], rec["n_off"] = len(space.oo), len(space.ao), space.n_off
        rec["n_rows"] = space.n_rows
        rec["wo"][: len(space.wo)] = space.wo
        rec["go"][: len(space.go)] = space.go
        rec["oo"][: len(space.oo)] = space.oo
        rec["ao"][: len(space.ao)] = space.ao
        rec["pair_wo"][: space.n_pair] = space.pair_wo
        rec["pair_go"][: space.n_pair] = space.pair_go

        # ---- parallelism rows: table look-ups at (b, tp) ----
        if space.n_par:
            rows = np.stack([self._par_fields(int(r[0]), int(r[2]), m, G) for r in space.par])
            rows[:, :6] = space.par
            rec["par"][: space.n_par] = rows

        # ---- pre / post layers: the same for every tp candidate of a (mesh, G) ----
        if analysis_row is None:
            fields = self._pre_post(n, m, G)
        else:
            fields = self._pre_post_uncached(n, m, G, analysis_row)
        for name, value in fields.items():
            rec[name] = value

    def fill_many(self, recs: np.ndarray, pending) -> None:
        """``fill`` for all groups of a tuner call at once: ``pending[i] = (g_index, q_index,
        num_nodes, num_gpus_per_node, grad_accum, num_p, space)`` describes ``recs[i]``.  Same
        values as ``fill`` record by record, written column by column (a record is 13.5 KB and
        has 40 fields: per-record assignment is most of the host time of a search)."""
        if not len(pending):
            return
        cols = list(zip(*[(g, q, n, m, G, num_p, sp.n_par, sp.n_pair, len(sp.oo), len(sp.ao), sp.n_off,
                           sp.n_rows) for g, q, n, m, G, num_p, sp in pending]))
        for name, values in zip(("g_index", "q_index", "num_nodes", "num_gpus_per_node", "grad_accum",
                                 "num_p", "n_par", "n_pair", "n_oo", "n_ao", "n_off", "n_rows"), cols):
            recs[name] = values
        first = pending[0][6]
        shared = all(sp.wo is first.wo and sp.go is first.go and sp.oo is first.oo and sp.ao is first.ao
                     and sp.pair_wo is first.pair_wo and sp.pair_go is first.pair_go
                     for *_, sp in pending)
        for i, (*_, sp) in enumerate(pending if not shared else pending[:1]):
            at = slice(None) if shared else i
            recs["wo"][at, : len(sp.wo)] = sp.wo
            recs["go"][at, : len(sp.go)] = sp.go
            recs["oo"][at, : len(sp.oo)] = sp.oo
            recs["ao"][at, : len(sp.ao)] = sp.ao
            recs["pair_wo"][at, : sp.n_pair] = sp.pair_wo
            recs["pair_go"][at, : sp.n_pair] = sp.pair_go
        # parallelism rows: the table look-ups at (b, tp), one block assignment
        group_of, slot_of, rows = [], [], []
        for i, (_, _, _, m, G, _, sp) in enumerate(pending):
            for k, r in enumerate(sp.par):
                v = self._par_fields(int(r[0]), int(r[2]), m, G).copy()
                v[:6] = r
                group_of.append(i)
                slot_of.append(k)
                rows.append(v)
        if rows:
            recs["par"][group_of, slot_of] = np.stack(rows)
        # pre / post layers: the same for every tp candidate of a (mesh, G)
        fields = [self._pre_post(n, m, G) for _, _, n, m, G, _, _ in pending]
        for name in fields[0]:
            recs[name] = [f[name] for f in fields]

    def _pre_post_uncached(self, n: int, m: int, G: int, analysis_row=None) -> dict:
        """``MistGroupDesc`` fields of the pre and post layers of a (mesh, G) group."""
        cfg, t = self.config, self.tables
        rec = {}
        pp_dp, pp_tp, pp_wre, pp_gre, pp_ore, pp_wo, pp_go, pp_oo, _pp_ac = pre_post_strategy_fields(
            cfg, n, m, analysis_row
        )
        pp_b = cfg.training.global_batch_size // G // pp_dp
        fb, ftp = np.float64(pp_b), np.float64(pp_tp)
        pre_W = t.mem_full_states("pre", "weights", ftp)
        pre_G = t.mem_full_states("pre", "grads", ftp)
        pre_O = t.mem_full_states("pre", "opts", ftp)
        pre_states = (
            _partial(pre_W, pp_dp if pp_wre else 1, pp_wo)
            + _partial(pre_G, pp_dp if pp_gre else 1, pp_go)
            + _partial(pre_O, pp_dp if pp_ore else 1, pp_oo)
        )
        pre_saved = t.mem_saved("pre", False, fb, ftp)
        post_W = t.mem_full_states("post", "weights", ftp)
        post_G = t.mem_full_states("post", "grads", ftp)
        post_O = t.mem_full_states("post", "opts", ftp)
        post_pO = _partial(post_O, pp_dp if pp_ore else 1, pp_oo)
        rec["pp_wre"], rec["pp_gre"] = int(bool(pp_wre)), int(bool(pp_gre))
        rec["pre_full_w"], rec["pre_full_g"] = float(pre_W), float(pre_G)
        rec["post_full_w"], rec["post_full_g"] = float(post_W), float(post_G)
        rec["pre_states"] = float(pre_states)
        rec["pre_saved"] = float(pre_saved)
        rec["pre_states_and_saved"] = float(pre_states + pre_saved)
        rec["post_states"] = float(post_W + post_G + post_pO)
        rec["post_fwd_peak"] = float(t.mem_peak("post", "fwd", fb, ftp, None))
        rec["post_bwd_peak"] = float(t.mem_peak("post", "bwd", fb, ftp))
        rec["post_output"] = float(t.mem_output("post", fb, ftp))
        inter = pp_tp // m if pp_tp > m else 1
        intra = m if pp_tp > m else pp_tp
        rec["pre_fwd"], rec["pre_bwd"], _, _ = self._exec("pre", pp_b, pp_tp, inter, intra, G)
        rec["post_fwd"], rec["post_bwd"], _, _ = self._exec("post", pp_b, pp_tp, inter, intra, G)
        if pp_dp == 1:
            rec["pre_ag"] = rec["post_ag"] = rec["pre_rs"] = rec["post_rs"] = 0.0
        else:
            rec["pre_ag"] = self._gpu_gpu("all_gather", pre_W, pp_dp, n)
            rec["post_ag"] = self._gpu_gpu("all_gather", post_W, pp_dp, n)
            rec["pre_rs"] = self._gpu_gpu("reduce_scatter", pre_G, pp_dp, n)
            rec["post_rs"] = self._gpu_gpu("reduce_scatter", post_G, pp_dp, n)
        return rec

    @staticmethod
    def validate(recs: np.ndarray) -> None:
        """The reduce kernel prunes with bounds that rely on every memory and latency input being
        finite and non-negative and on ratios in [0, 1] (then peaks are monotone in the number of
        pre-saved micro-batches and in every row term).  Real tables always are; a violation is
        rejected here instead of silently changing which rows get evaluated.  ``recs``: filled
        ``GROUP_DTYPE`` records (unused array slots hold zero)."""
        par = recs["par"]
        if not np.all(np.isfinite(par)) or np.any(par < 0):
            raise ValueError("layer table values must be finite and non-negative")
        for name in ("wo", "go", "oo", "ao"):
            v = recs[name]
            if not np.all((v >= 0) & (v <= 1)):
                raise ValueError(f"offload ratios '{name}' must lie in [0, 1], got {v[~((v >= 0) & (v <= 1))]}")
        names = recs.dtype.names
        for name in names[names.index("pre_full_w"):]:
            v = recs[name]
            if not np.all(np.isfinite(v) & (v >= 0)):
                raise ValueError(f"pre/post layer input '{name}' must be finite and non-negative, got {v}")
