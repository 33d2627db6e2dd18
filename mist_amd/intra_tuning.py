"""Intra-stage tuner: the drop-in for the reference's ``mist/analyzer/intra_tuning.py``.

``IntraStageTuner.tune()`` (reference :169-282) loops the gradient-accumulation candidates and
device meshes and calls the numpy evaluation once per (G, mesh).  Here the host only prepares
one small descriptor per (G, mesh) group; all groups of a tuner call are then evaluated by three
kernel launches on the GPU (row terms, evaluate+mask+argmin, finalize) and the result tables
stay resident in HBM for the inter-stage search.  ``IntraStageTunerOutput`` exposes the same
fields and layouts as the reference (:59-82); numpy copies are made lazily on first access.
"""
from __future__ import annotations

import ctypes
import os
from collections.abc import Mapping
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib
from .config import MistConfig
from .layer_tables import LayerTables
from .search_space import SearchSpace, SearchSpaceFactory, create_search_space_for_a_block_layer
from .stage_inputs import GroupInputBuilder, make_problem

SAMPLE_SIZE = 30  # reference default (batched_module_analyzer.py:67)
VARIANTS = ("", "_with_pre", "_with_post", "_no_pp")
# wavefronts of the reduce kernel the row chunks are sized for: 64 per SIMD, so that the tail of
# the launch is short; a chunk that changes no slot writes no slab, which keeps small chunks cheap
TARGET_REDUCE_WAVES = 65536
SCOUT_MIN_STAGES = 128  # groups with fewer stages get no scout pass (0 = never scout)
SCOUT_MIN_PAIRS = 4     # ... and so do groups with fewer (weight, gradient) offload pairs
SCOUT_PAIRS = 1         # offload pairs whose rows the scout pass gathers: the first, (0, 0), then evenly spread ones
SCOUT_PAIR_SPAN = 200   # ... one more for every so many pairs of the group (GPT-22B: 421 pairs, 3 gathered)
# ... and three for a group none of whose parallelism rows can hold this fraction of the model's
# layers (weights, gradients and optimizer states of a layer at the group's tensor parallelism,
# unsharded, nothing offloaded) within the memory capacity: such stages need sharding or
# offloading, and the winners spread over the weight / gradient offload pairs.  (Speed only,
# set from four plans: LLaMA-70B has 0.07 - 0.28 there for tp 1 - 4 and 0.55 for tp 8 and runs
# 140 -> 98 ms with the two further pairs; GPT-7B has 0.73 - 5.9 and LLaMA-13B 0.37 - 3.0, and
# they run 17 - 20 % slower with further pairs for every group, 2 % with them for tp 1.)
SCOUT_TIGHT_FRACTION = 0.3
SCOUT_TIGHT_PAIRS = 3
# Upper bound of the row-term workspace (272 bytes per candidate row): the groups of a tuner call
# go through the kernels in batches of consecutive groups whose rows fit it (a group larger than
# the bound is a batch of its own).  GPT-7B (0.88 GB) and LLaMA-13B (1.4 GB) are one batch,
# GPT-22B (18.4 GB of row terms) ten; with more than one batch two such workspaces alternate.
ROW_TERMS_BUDGET_BYTES = 2 << 30
# Partial-minima slabs the main launches of a multi-sample call may hold at once: samples in
# flight = this / (workgroups of the launch x 26 KB); GPT-7B (63 232 workgroups): 4.
MAIN_BATCH_SLAB_BYTES = 8 << 30


_SIDE_STREAMS: Dict[str, "torch.cuda.Stream"] = {}


def _side_stream(device) -> "torch.cuda.Stream":
    """The second stream that plans of several batches alternate with, one per device for the
    life of the process.  A stream per tuner would take another hardware queue each time (there
    are four): sooner or later one shared with the caller's stream or with the library's own
    scout stream, whose kernels then no longer overlap (GPT-22B: 150 ms became 164 to 187 ms,
    depending on how many tuners the process had created before)."""
    key = str(torch.device(device))
    if key not in _SIDE_STREAMS:
        _SIDE_STREAMS[key] = torch.cuda.Stream(device=device)
    return _SIDE_STREAMS[key]


def _scout_pairs(group, count: int) -> List[int]:
    """The (weight, gradient) offload pairs whose rows the scout pass of a group gathers: the
    first one, (0, 0), then evenly spread ones up to the last.  Any set of distinct pairs gives
    the same tables (scout rows only seed the search); the choice is about speed."""
    n_pair = int(group["n_pair"])
    if count <= 1:
        return [0] * count
    return sorted({k * (n_pair - 1) // (count - 1) for k in range(count)})


def alpha_ratios(sample_size: int) -> np.ndarray:
    """``alpha_k / (1 - alpha_k)`` for ``alpha = linspace(0, 1, S + 2)[1:-1]``
    (mist/utils/pareto.py:53-55,138)."""
    alpha = np.linspace(0, 1, sample_size + 2)[1:-1]
    return alpha / (1 - alpha)


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


@dataclass
class DeviceTables:
    """float64 cost tables and int32 row-index tables in HBM, reference layout."""

    stable: List[torch.Tensor]
    delta: List[torch.Tensor]
    index: List[torch.Tensor]
    # gradient-accumulation count of every table row g (int32, on the device), uploaded with the
    # plan so that the inter-stage search need not wait for the kernels to copy it
    grad_accum: Optional[torch.Tensor] = None

    def as_struct(self) -> _lib.OutTables:
        s = _lib.OutTables()
        for v in range(4):
            s.stable[v] = self.stable[v].data_ptr()
            s.delta[v] = self.delta[v].data_ptr()
            s.index[v] = self.index[v].data_ptr()
        return s


class IntraStageTunerOutput:
    """Same attributes as the reference's ``IntraStageTunerOutput`` (intra_tuning.py:59-82):
    ``costs_stable*`` / ``costs_delta*`` float32, ``solutions*`` float64 with ``inf`` fill.
    Additionally ``indices*`` (row index per cell, -1 = none) and ``device`` (the HBM tables)."""

    def __init__(
        self,
        gradient_accumulation_steps_candidates: List[int],
        device_mesh_candidates: List[Tuple[int, int]],
        device: DeviceTables,
        spaces: Dict[Tuple[int, int], SearchSpace],
        sample_slots: Sequence[int],
        batch: Optional[DeviceTables] = None,
        batch_index: int = 0,
    ):
        self.gradient_accumulation_steps_candidates = list(gradient_accumulation_steps_candidates)
        self.device_mesh_candidates = list(device_mesh_candidates)
        self.device = device
        self.spaces = spaces
        self.sample_slots = tuple(sample_slots)
        # Tables of every tensor-parallel candidate evaluated in the same launch (leading axis
        # = batch_index * len(G candidates) + g); ``device`` is this candidate's slice of them.
        self.batch = device if batch is None else batch
        self.batch_index = batch_index
        self._host: Dict[str, np.ndarray] = {}

    def _fetch(self, kind: str, v: int) -> np.ndarray:
        key = f"{kind}{v}"
        if key not in self._host:
            self._host[key] = getattr(self.device, kind)[v].cpu().numpy()
        return self._host[key]

    def costs_f64(self, kind: str, variant: int) -> np.ndarray:
        """float64 ``stable`` / ``delta`` table of variant 0..3 as computed on the GPU."""
        return self._fetch(kind, variant)

    def _solutions(self, v: int) -> np.ndarray:
        key = f"solutions{v}"
        if key not in self._host:
            idx = self._fetch("index", v)
            out = np.full(idx.shape + (10,), np.inf, dtype=np.float64)
            for (g, q), space in self.spaces.items():
                out[g, q] = space.decode(idx[g, q])
            self._host[key] = out
        return self._host[key]

    def solution_at(self, variant: int, cell: Tuple[int, ...]) -> np.ndarray:
        """One strategy row ``solutions<variant>[cell]`` (cell = full index incl. g, q and the
        sample slot) without building the whole solutions table: a single index is read back."""
        key = f"solutions{variant}"
        if key in self._host:
            return self._host[key][cell]
        idx = self._host.get(f"index{variant}")
        row = int(idx[cell]) if idx is not None else int(self.device.index[variant][cell].item())
        return self.spaces[(cell[0], cell[1])].decode(np.array(row))

    @staticmethod
    def solutions_at(requests) -> List[np.ndarray]:
        """``solution_at`` for many ``(results, variant, cell)`` requests (results objects on one
        device) with a single read-back of the row indices that are not on the host yet."""
        rows: List[Optional[int]] = []
        pending = []
        for i, (res, variant, cell) in enumerate(requests):
            idx = res._host.get(f"index{variant}")
            rows.append(int(idx[cell]) if idx is not None else None)
            if idx is None:
                pending.append(i)
        if pending:
            fetched = torch.stack(
                [requests[i][0].device.index[requests[i][1]][requests[i][2]] for i in pending]
            ).cpu().numpy()
            for i, row in zip(pending, fetched):
                rows[i] = int(row)
        return [res.spaces[(cell[0], cell[1])].decode(np.array(row))
                for (res, _, cell), row in zip(requests, rows)]

    def __getattr__(self, name: str):
        for v, suffix in enumerate(VARIANTS):
            if name == "costs_stable" + suffix:
                return self._fetch("stable", v).astype(np.float32)
            if name == "costs_delta" + suffix:
                return self._fetch("delta", v).astype(np.float32)
            if name == "solutions" + suffix:
                return self._solutions(v)
            if name == "indices" + suffix:
                return self._fetch("index", v).astype(np.int64)
        raise AttributeError(name)

    def __repr__(self) -> str:
        return (
            f"IntraStageTunerOutput("
            f"gradient_accumulation_steps_candidates={self.gradient_accumulation_steps_candidates}, "
            f"device_mesh_candidates={self.device_mesh_candidates}."
        )


class _PlanSpaces(Mapping):
    """``(t, g, q) -> SearchSpace`` over the parallelism rows ``mist_plan_groups`` returns; a
    space is made when it is asked for (a search decodes a handful of its 240)."""

    def __init__(self, shape, offsets, rows, lists):
        self._shape, self._offsets, self._rows, self._lists = shape, offsets, rows, lists
        self._made: Dict[Tuple[int, int, int], SearchSpace] = {}

    def __getitem__(self, key):
        space = self._made.get(key)
        if space is None:
            t, g, q = key
            T, Gn, Qn = self._shape
            if not (0 <= t < T and 0 <= g < Gn and 0 <= q < Qn):
                raise KeyError(key)
            entry = (t * Gn + g) * Qn + q
            wo, go, oo, ao, pair_wo, pair_go = self._lists
            par = self._rows[self._offsets[entry]:self._offsets[entry + 1]]
            space = self._made[key] = SearchSpace(par=par, wo=wo, go=go, oo=oo, ao=ao,
                                                  pair_wo=pair_wo, pair_go=pair_go)
        return space

    def __iter__(self):
        T, Gn, Qn = self._shape
        return ((t, g, q) for t in range(T) for g in range(Gn) for q in range(Qn))

    def __len__(self):
        T, Gn, Qn = self._shape
        return T * Gn * Qn


class _SpacesOfEntry(Mapping):
    """The ``(g, q) -> SearchSpace`` view of one tensor-parallel entry ``t`` of a plan's spaces."""

    def __init__(self, spaces, t: int):
        self._spaces, self._t = spaces, t

    def __getitem__(self, key):
        return self._spaces[(self._t, key[0], key[1])]

    def __iter__(self):
        return ((g, q) for (t, g, q) in self._spaces if t == self._t)

    def __len__(self):
        return sum(1 for _ in iter(self))


class IntraStageTuner:
    """Reference: ``IntraStageTuner`` (mist/analyzer/intra_tuning.py:84-282).  ``layer_tables``
    replaces the three ``LayerInfo`` arguments."""

    def __init__(
        self,
        layer_tables: LayerTables,
        num_layers: int,
        device_mesh_candidates: List[Tuple[int, int]],
        gradient_accumulation_steps_candidates: List[int],
        tp_size: Optional[int],
        config: MistConfig,
        disable_tqdm: bool = True,
        sample_size: int = SAMPLE_SIZE,
        sample_slots: Optional[Sequence[int]] = None,
        device: str = "cuda:0",
        exhaustive: bool = False,
    ):
        # exhaustive: evaluate every cell (no scout pass, no sieves) with
        # mist_eval_reduce_exhaustive; same tables, the reference point for tests and bench
        self.exhaustive = bool(exhaustive)
        self.layer_tables = layer_tables
        self.num_layers = int(num_layers)
        self.device_mesh_candidates = list(device_mesh_candidates)
        self.gradient_accumulation_steps_candidates = list(gradient_accumulation_steps_candidates)
        self.tp_size = tp_size
        # A list of tp sizes evaluates all of them in one batch of launches (``tune_all``).
        self.tp_sizes = list(tp_size) if isinstance(tp_size, (list, tuple)) else [tp_size]
        self.config = config
        self.sample_size = int(sample_size)
        # Which of the S alpha samples to evaluate (default: all); unevaluated slots stay inf / -1.
        self.sample_slots = tuple(range(self.sample_size)) if sample_slots is None else tuple(sample_slots)
        if not self.sample_slots or not all(0 <= s < self.sample_size for s in self.sample_slots):
            raise ValueError(f"sample_slots must be a non-empty subset of 0..{self.sample_size - 1}")
        self.device = torch.device(device)
        # intra_tuning.py:117-126
        self.max_possible_num_stages = min(
            max(n * m for n, m in self.device_mesh_candidates), self.num_layers
        )
        self.max_possible_pre_saved_micro_batches = (
            min(self.max_possible_num_stages, max(self.gradient_accumulation_steps_candidates)) - 1
        )
        # True: every p of 0..P is evaluated for every G (the operator boundary
        # batched_tune_best_latency_for_stage takes the p candidates from its caller)
        self.evaluate_all_p = False
        # Optional ``cells_wanted(G, (n, m)) -> None | (l_min, l_max, p_count)``: a caller that
        # reads only a range of layer counts and the first ``p_count`` pre-saved micro-batch
        # values of a (G, mesh) group - or nothing of it (None) - has only the tiles of (layers,
        # ckpt) pairs that hold them evaluated; every other cell keeps its pre-filled inf / -1.
        # The evaluated cells are the same as without it.
        self.cells_wanted = None
        # True (with ``cells_wanted``): the output tables are pre-filled (+inf / -1) in the cells
        # ``cells_wanted`` names only, whatever else they hold is undefined - for a caller that
        # reads nothing else (the stage assignment; with 30 samples the fill of the whole tables
        # is a tenth of its search)
        self.prefill_wanted_cells_only = False
        self.results: Optional[IntraStageTunerOutput] = None
        self.stats: Dict[str, float] = {}

    # ------------------------------------------------------------------ host side
    def prepare(self):
        """Builds the group descriptors and the launch decomposition (host only, no GPU): in the
        library (``mist_plan_groups``) for plans on the closed-form layer tables, in python
        otherwise and when ``MIST_PYTHON_PLAN_BUILDER`` is set; the two give the same bytes."""
        _lib.load()  # the tile sizes of the decomposition are the library's
        wanted = self._wanted_cells()
        built = None
        if not os.environ.get("MIST_PYTHON_PLAN_BUILDER"):
            built = self._build_groups_native(wanted)
        if built is None:
            built = self._build_groups_python(wanted)
        plan = self._finish_plan(*built)
        plan["wanted"] = wanted
        return plan

    def _wanted_cells(self) -> Optional[np.ndarray]:
        """``cells_wanted`` of every (G, mesh) as int32 ``[G][mesh][3]`` = (smallest layer count,
        largest, number of pre-saved micro-batch values), -1s where nothing is read; None without
        ``cells_wanted``."""
        if self.cells_wanted is None:
            return None
        Gs, Q = self.gradient_accumulation_steps_candidates, self.device_mesh_candidates
        wanted = np.full((len(Gs), len(Q), 3), -1, dtype=np.int32)
        for g, G in enumerate(Gs):
            for q, mesh in enumerate(Q):
                cells = self._cells_wanted_of(G, mesh)
                if cells is not None:
                    wanted[g, q] = cells
        return wanted

    def _cells_wanted_of(self, G, mesh):
        """``cells_wanted`` of a (G, mesh) as ``(smallest layer count, largest, number of
        pre-saved micro-batch values)`` or None when the caller reads nothing of it."""
        wanted = self.cells_wanted(G, mesh)
        if wanted is None:
            return None
        l_min, l_max, p_count = wanted
        l_min, l_max = max(int(l_min), 1), min(int(l_max), self.num_layers)
        if l_min > l_max or p_count < 1:
            return None
        return l_min, l_max, int(p_count)

    def _build_groups_native(self, wanted: Optional[np.ndarray] = None):
        """The groups of this call from ``mist_plan_groups``, or None when the plan is outside
        what it covers or fails one of its checks (the python builder then words the error)."""
        cfg, tables, L = self.config, self.layer_tables, self.num_layers
        if type(tables) is not LayerTables:
            return None  # latencies from an operator database: python look-ups
        Gs, Q = self.gradient_accumulation_steps_candidates, self.device_mesh_candidates
        factory = SearchSpaceFactory(cfg, tables.constraint)
        wo, go, oo, ao, pair_wo, pair_go = factory.lists
        pp_mode = _lib.PLAN_PP_MODES.get(cfg.tuning.pre_post_strategy)
        ints = [*Gs, *(n for n, _ in Q), *(m for _, m in Q), *factory.batch_sizes, L,
                cfg.training.global_batch_size, cfg.model.num_attention_heads,
                cfg.training.max_sequence_length, *(t for t in self.tp_sizes if t is not None)]
        if (pp_mode is None or (pp_mode == _lib.PLAN_PP_MODES["preset"] and cfg.strategy is None)
                or len(self.tp_sizes) > _lib.PLAN_MAX_LIST or len(Gs) > _lib.PLAN_MAX_LIST
                or len(Q) > _lib.MAX_MESH or len(factory.batch_sizes) > _lib.PLAN_MAX_BATCH_SIZES
                or len(factory.flag_choices) > _lib.PLAN_MAX_LIST
                or not all(isinstance(v, (int, np.integer)) and 0 < v < 2**31 for v in ints)):
            return None
        req = _lib.PlanRequest()
        lay = req.layers
        lay.hidden, lay.heads, lay.kv_heads, lay.ffn = tables.h, tables.heads, tables.kv_heads, tables.ffn
        lay.vocab, lay.seq_len, lay.norm_params = tables.vocab, tables.s, tables.norm_params
        lay.opt_mult, lay.bytes_per_param = tables.opt_mult, tables.bytes_per_param
        lay.peak_flops, lay.hbm_bw = tables.peak_flops, tables.hbm_bw
        for i, name in enumerate(_lib.PLAN_OP_CLASSES):
            lay.efficiency[i][0], lay.efficiency[i][1] = tables.eff[name]
        lay.flash, lay.gated, lay.abs_pos, lay.tied = tables.flash, tables.gated, tables.abs_pos, tables.tied
        if len(tables.gpu_gpu_comm_params) != 32 or len(cfg.hardware.gpu_gpu_comm_params) != 32:
            return None
        if tuple(tables.gpu_gpu_comm_params) != tuple(cfg.hardware.gpu_gpu_comm_params):
            return None
        req.gpu_gpu[:] = [float(x) for x in cfg.hardware.gpu_gpu_comm_params]
        req.memory_capacity_gb = cfg.hardware.memory_capacity
        req.wo[:len(wo)], req.go[:len(go)], req.oo[:len(oo)], req.ao[:len(ao)] = wo, go, oo, ao
        req.n_wo, req.n_go, req.n_oo, req.n_ao, req.n_pair = len(wo), len(go), len(oo), len(ao), len(pair_wo)
        ctypes.memmove(req.pair_wo, pair_wo.ctypes.data, len(pair_wo))
        ctypes.memmove(req.pair_go, pair_go.ctypes.data, len(pair_go))
        if pp_mode == _lib.PLAN_PP_MODES["preset"]:
            preset = [float(x) for x in cfg.strategy.pre_post_strategy_array]
            if len(preset) != 10 or any(x != int(x) for x in preset[1:3]):
                return None
            req.pp_preset[:] = preset
        req.pp_mode = pp_mode
        req.scout_tight_fraction = SCOUT_TIGHT_FRACTION
        req.global_batch_size = cfg.training.global_batch_size
        req.workspace_rows = max(ROW_TERMS_BUDGET_BYTES // (8 * _lib.ROW_TERMS), 1)
        req.model_heads, req.model_seq_len = cfg.model.num_attention_heads, cfg.training.max_sequence_length
        req.model_flash = bool(cfg.model.use_flash_attn)
        req.num_layers, req.max_pre_saved = L, self.max_possible_pre_saved_micro_batches
        req.evaluate_all_p, req.exhaustive = bool(self.evaluate_all_p), bool(self.exhaustive)
        req.n_tp, req.n_grad_accum, req.n_mesh = len(self.tp_sizes), len(Gs), len(Q)
        req.tp_size[:req.n_tp] = [0 if t is None else t for t in self.tp_sizes]
        req.grad_accum[:req.n_grad_accum] = Gs
        req.mesh_n[:req.n_mesh] = [n for n, _ in Q]
        req.mesh_m[:req.n_mesh] = [m for _, m in Q]
        req.n_batch_sizes = len(factory.batch_sizes)
        req.batch_size[:req.n_batch_sizes] = factory.batch_sizes
        req.zero_2_and_3, req.disable_tp, req.check_shapes = factory.zero_2_and_3, factory.disable_tp, 1
        req.n_flag_choices = len(factory.flag_choices)
        for i, flags in enumerate(factory.flag_choices):
            req.flag_choice[i][:] = flags
        req.target_reduce_waves, req.scout_min_stages = TARGET_REDUCE_WAVES, SCOUT_MIN_STAGES
        req.scout_min_pairs, req.scout_pairs = SCOUT_MIN_PAIRS, SCOUT_PAIRS
        req.scout_pair_span, req.scout_tight_pairs = SCOUT_PAIR_SPAN, SCOUT_TIGHT_PAIRS
        if wanted is None:
            wanted = self._wanted_cells()
        if wanted is not None:
            req.cells_wanted = wanted.ctypes.data
        entries = req.n_tp * req.n_grad_accum * req.n_mesh
        groups = np.zeros(entries, dtype=_lib.GROUP_DTYPE)
        space_offset = np.empty(entries + 1, dtype=np.int64)
        space_rows = np.empty((entries * _lib.MAX_PAR, 6), dtype=np.float64)
        group_of_entry = np.empty(entries, dtype=np.int32)
        prefixes = np.empty((4, entries + 1), dtype=np.int32)
        result = _lib.PlanResult()
        ptr = lambda a: ctypes.c_void_p(a.ctypes.data)
        rc = _lib.load().mist_plan_groups(
            ctypes.byref(req), ptr(groups), entries, ptr(space_offset), ptr(space_rows),
            ptr(group_of_entry), ptr(prefixes[0]), ptr(prefixes[1]), ptr(prefixes[2]), ptr(prefixes[3]),
            ctypes.byref(result))
        if rc == _lib.PLAN_UNSUPPORTED:
            return None
        _lib.check(rc, "mist_plan_groups")
        n = result.n_groups
        spaces = _PlanSpaces((req.n_tp, req.n_grad_accum, req.n_mesh), space_offset,
                             space_rows[:result.n_space_rows], factory.lists)
        bounds = [(int(prefixes[3, i]), int(prefixes[3, i + 1])) for i in range(result.n_batches)]
        return (groups[:n], spaces, prefixes[0, :n + 1], prefixes[1, :n + 1], prefixes[2, :n + 1], bounds,
                result.max_scout_rows, result.max_group_keys)

    def _build_groups_python(self, wanted: Optional[np.ndarray] = None):
        cfg, L = self.config, self.num_layers
        Gs, Q = self.gradient_accumulation_steps_candidates, self.device_mesh_candidates
        P = self.max_possible_pre_saved_micro_batches
        builder = GroupInputBuilder(cfg, self.layer_tables)
        spaces: Dict[Tuple[int, int, int], SearchSpace] = {}
        pending = []
        factory = SearchSpaceFactory(cfg, self.layer_tables.constraint)
        B = cfg.training.global_batch_size
        n_pairs = L * (L + 1) // 2 + L
        tile_window = []  # per group: first tile of its (layers, ckpt) pairs and how many
        if wanted is None:
            wanted = self._wanted_cells()
        for t, tp_size in enumerate(self.tp_sizes):
            for g, G in enumerate(Gs):
                for q, (n, m) in enumerate(Q):
                    space = factory.make(n, m, B, G, tp_size)
                    spaces[(t, g, q)] = space
                    if space.n_rows == 0:
                        continue  # the reference returns all-inf tables for an empty space (:648-666)
                    if space.n_rows >= 2**31:
                        raise ValueError(f"group (G={G}, mesh={(n, m)}) has {space.n_rows} rows (>= 2**31)")
                    num_p = min(G, L, P + 1)  # intra_tuning.py:185-193
                    if self.evaluate_all_p:
                        num_p = P + 1
                    window = (0, -(-n_pairs // _lib.LC_TILE))
                    if wanted is not None:
                        l_min, l_max, p_count = (int(x) for x in wanted[g, q])
                        if l_min < 0:
                            continue
                        num_p = min(num_p, p_count)
                        # pairs are numbered l-major: index(l, c) = l (l + 1) / 2 - 1 + c
                        first = (l_min * (l_min + 1) // 2 - 1) // _lib.LC_TILE
                        last = (l_max * (l_max + 1) // 2 - 1 + l_max) // _lib.LC_TILE
                        window = (first, last - first + 1)
                    tile_window.append(window)
                    pending.append((t * len(Gs) + g, q, n, m, G, num_p, space))
        groups = np.zeros(len(pending), dtype=_lib.GROUP_DTYPE)
        builder.fill_many(groups, pending)
        builder.validate(groups)

        bounds = self._batch_bounds(groups["n_rows"]) if len(pending) else []
        max_scout_rows = max_group_keys = 0
        if len(pending):
            groups["lc_tile_begin"] = [w[0] for w in tile_window]
            n_lc_tiles = np.array([w[1] for w in tile_window], dtype=np.int64)
            n_p_tiles = -(-groups["num_p"] // _lib.P_TILE)
            # the row chunks are sized per batch of groups (one reduce launch each, see below)
            for first, last in bounds:
                sel = slice(first, last)
                tile_rows = int(np.sum(groups["n_rows"][sel] * n_lc_tiles[sel] * n_p_tiles[sel]))
                rows_per_chunk = -(-tile_rows // max(TARGET_REDUCE_WAVES * 64 // _lib.LC_TILE, 1))
                rows_per_chunk = max(256, min(16384, -(-rows_per_chunk // _lib.STAGE_ROWS) * _lib.STAGE_ROWS))
                groups["rows_per_chunk"][sel] = rows_per_chunk
            groups["n_chunks"] = -(-groups["n_rows"] // groups["rows_per_chunk"])
            groups["n_lc_tiles"] = n_lc_tiles
            groups["n_p_tiles"] = n_p_tiles
            groups["row_offset"] = np.concatenate(([0], np.cumsum(groups["n_rows"])[:-1]))
            # keys = (parallelism row, activation ratio, offload pair): what 28 of a row's 36
            # interference evaluations depend on; evaluated once per key, not once per row
            n_keys = groups["n_par"].astype(np.int64) * groups["n_ao"] * groups["n_pair"]
            groups["key_offset"] = np.concatenate(([0], np.cumsum(n_keys)[:-1]))
            terms_blocks = -(-groups["n_rows"] // _lib.TERMS_BLOCK)
            reduce_blocks = groups["n_chunks"].astype(np.int64) * n_lc_tiles * n_p_tiles
            # Scout pass: the rows of a group without weight / gradient offloading (one in n_pair)
            # seed its chunks; groups that are small or have few offload pairs go without.
            n_stages = -(-groups["n_rows"] // _lib.STAGE_ROWS)
            scout = (n_stages >= SCOUT_MIN_STAGES) & (groups["n_pair"] >= SCOUT_MIN_PAIRS) & (SCOUT_MIN_STAGES > 0)
            scout &= not self.exhaustive
            pairs = SCOUT_PAIRS + groups["n_pair"] // SCOUT_PAIR_SPAN
            par = groups["par"]
            layer_states = par[..., _lib.PAR["W"]] + par[..., _lib.PAR["G"]] + par[..., _lib.PAR["O"]]
            layer_states = np.where(np.arange(_lib.MAX_PAR)[None, :] < groups["n_par"][:, None],
                                    layer_states, np.inf).min(axis=1)
            capacity_mb = cfg.hardware.memory_capacity * 1024.0
            tight = capacity_mb < SCOUT_TIGHT_FRACTION * L * layer_states
            pairs = np.where(tight, np.maximum(pairs, SCOUT_TIGHT_PAIRS), pairs)
            pairs = np.minimum(np.minimum(pairs, groups["n_pair"]), _lib.MAX_SCOUT_PAIRS)
            groups["scout_stride"] = np.where(scout, pairs, 0)
            for i in range(len(groups)):
                picked = _scout_pairs(groups[i], int(groups["scout_stride"][i]))
                groups["scout_stride"][i] = len(picked)
                groups["scout_pair"][i, :len(picked)] = picked
            scout_blocks = n_lc_tiles * _lib.SCOUT_SPLIT * n_p_tiles
            if not np.any(groups["scout_stride"] > 0):
                scout_blocks[:] = 0
            scouted = groups["scout_stride"] > 0
            gathered = groups["n_par"] * groups["n_oo"] * groups["n_ao"] * groups["scout_stride"]
            max_scout_rows = int(gathered[scouted].max()) if scouted.any() else 0
            max_group_keys = int(n_keys.max())
        else:
            terms_blocks = reduce_blocks = scout_blocks = np.zeros(0, dtype=np.int64)
        terms_prefix = np.concatenate(([0], np.cumsum(terms_blocks))).astype(np.int64)
        reduce_prefix = np.concatenate(([0], np.cumsum(reduce_blocks))).astype(np.int64)
        scout_prefix = np.concatenate(([0], np.cumsum(scout_blocks))).astype(np.int64)
        if terms_prefix[-1] >= 2**31 or reduce_prefix[-1] + scout_prefix[-1] >= 2**31:
            raise ValueError("launch decomposition exceeds 2**31 workgroups")
        return (groups, spaces, terms_prefix, reduce_prefix, scout_prefix, bounds, max_scout_rows,
                max_group_keys)

    def _finish_plan(self, groups, spaces, terms_prefix, reduce_prefix, scout_prefix, bounds,
                     max_scout_rows, max_group_keys):
        cfg, L = self.config, self.num_layers
        Gs, Q = self.gradient_accumulation_steps_candidates, self.device_mesh_candidates
        P = self.max_possible_pre_saved_micro_batches
        problem = make_problem(cfg, L, P + 1, self.sample_size, len(self.tp_sizes) * len(Gs), len(Q))
        if len(groups):
            problem["max_scout_rows"] = max_scout_rows
            problem["max_group_keys"] = max_group_keys
        n_keys = groups["n_par"].astype(np.int64) * groups["n_ao"] * groups["n_pair"]
        # Batches of consecutive groups under the workspace bound: each holds its own copy of the
        # descriptors with row offsets that start at 0 and its own workgroup prefixes.
        batches = []
        for first, last in bounds:
            rows = int(groups["n_rows"][first:last].sum())
            if first == 0:
                sub = groups[:last]  # offsets start at 0 already
            else:
                sub = groups[first:last].copy()
                sub["row_offset"] -= groups["row_offset"][first]
                sub["key_offset"] -= groups["key_offset"][first]
            rebase = lambda prefix: (prefix[first:last + 1] - prefix[first]).astype(np.int32)
            batches.append(dict(
                first=first, last=last, groups=sub, total_rows=rows,
                total_keys=int(n_keys[first:last].sum()),
                terms_prefix=rebase(terms_prefix), reduce_prefix=rebase(reduce_prefix),
                scout_prefix=rebase(scout_prefix),
            ))
        return dict(
            problem=problem, groups=groups, spaces=spaces, batches=batches,
            terms_prefix=terms_prefix.astype(np.int32), reduce_prefix=reduce_prefix.astype(np.int32),
            scout_prefix=scout_prefix.astype(np.int32),
            total_rows=int(groups["n_rows"].sum()) if len(groups) else 0,
        )

    @staticmethod
    def _batch_bounds(n_rows) -> List[Tuple[int, int]]:
        """Runs of consecutive groups whose rows fit the row-term workspace bound (a larger
        group is a run of its own)."""
        budget_rows = max(ROW_TERMS_BUDGET_BYTES // (8 * _lib.ROW_TERMS), 1)
        bounds, first = [], 0
        while first < len(n_rows):
            last, rows = first, 0
            while last < len(n_rows) and (last == first or rows + int(n_rows[last]) <= budget_rows):
                rows += int(n_rows[last])
                last += 1
            bounds.append((first, last))
            first = last
        return bounds

    def _table_layout(self):
        """Shapes of the four variants' tables and where each starts in the flat allocations."""
        Gn = len(self.tp_sizes) * len(self.gradient_accumulation_steps_candidates)
        Qn = len(self.device_mesh_candidates)
        P1, L, S = self.max_possible_pre_saved_micro_batches + 1, self.num_layers, self.sample_size
        shapes = [(Gn, Qn, P1, L, L + 1, S), (Gn, Qn, P1, L, L + 1, S), (Gn, Qn, L, L + 1, S), (Gn, Qn, L + 1, S)]
        starts = [0]
        for shape in shapes:
            starts.append(starts[-1] + int(np.prod(shape)))
        return shapes, starts

    def _allocate_flat(self, plan: Optional[dict] = None):
        """The output tables as two flat allocations (float64 costs: stable then delta; int32
        row indices) with their pre-fill queued on the current stream, and the ``MistOutTables``
        of pointers into them.  Pre-filled with +inf / -1: everywhere, or (``plan`` of a tuner
        with ``prefill_wanted_cells_only``) in the cells ``cells_wanted`` names."""
        shapes, starts = self._table_layout()
        total, dev = starts[-1], self.device
        wanted = plan.get("wanted") if plan is not None and self.prefill_wanted_cells_only else None
        if wanted is None:
            # one allocation and one fill per element type
            costs = torch.full((2 * total,), float("inf"), dtype=torch.float64, device=dev)
            index = torch.full((total,), -1, dtype=torch.int32, device=dev)
        else:
            costs = torch.empty((2 * total,), dtype=torch.float64, device=dev)
            index = torch.empty((total,), dtype=torch.int32, device=dev)
        struct = _lib.OutTables()
        cost_ptr, index_ptr = costs.data_ptr(), index.data_ptr()
        for v in range(4):
            struct.stable[v] = cost_ptr + 8 * starts[v]
            struct.delta[v] = cost_ptr + 8 * (total + starts[v])
            struct.index[v] = index_ptr + 4 * starts[v]
        if wanted is not None:
            Gn, Qn, P1, L, _, S = shapes[0]
            g, q = np.nonzero(wanted[:, :, 0] >= 0)
            if len(g):
                n_g = wanted.shape[0]
                one = np.zeros((len(g), 6), dtype=np.int32)
                one[:, 0], one[:, 1], one[:, 2:5] = g, q, wanted[g, q]
                regions = np.tile(one, (len(self.tp_sizes), 1))
                regions[:, 0] += np.repeat(np.arange(len(self.tp_sizes), dtype=np.int32) * n_g, len(g))
                nl = (regions[:, 3] - regions[:, 2] + 1).astype(np.int64)
                rows = 2 * np.minimum(regions[:, 4], P1) * nl + nl + (regions[:, 3] == L)
                first = np.concatenate(([0], np.cumsum(rows)[:-1]))
                if int(rows.sum()) >= 2**31:
                    raise ValueError("the cells to pre-fill exceed one launch")
                regions[:, 5] = first
                d_regions = torch.from_numpy(regions.reshape(-1)).to(dev)
                rc = _lib.load().mist_mip_prefill_cells(
                    L, P1, S, Qn, Gn, ctypes.c_void_p(regions.ctypes.data), d_regions.data_ptr(),
                    len(regions), ctypes.byref(struct),
                    ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
                _lib.check(rc, "mist_mip_prefill_cells")
        return costs, index, struct

    def _table_views(self, costs: torch.Tensor, index: torch.Tensor) -> DeviceTables:
        shapes, starts = self._table_layout()
        total = starts[-1]
        def views(flat, base):
            return [flat[base + starts[v]:base + starts[v + 1]].view(shapes[v]) for v in range(4)]
        return DeviceTables(stable=views(costs, 0), delta=views(costs, total), index=views(index, 0))

    def allocate_tables(self, plan: Optional[dict] = None) -> DeviceTables:
        """Output tables, pre-filled with +inf / -1: all of them, or (``plan`` of a tuner with
        ``prefill_wanted_cells_only``) the cells ``cells_wanted`` names."""
        costs, index, _ = self._allocate_flat(plan)
        return self._table_views(costs, index)

    # ------------------------------------------------------------------ device side
    def upload(self, plan) -> dict:
        """Descriptors and workgroup prefixes of every batch to the device; one workspace (row
        terms, stage summaries, partial minima) sized for the largest batch and shared by all.
        The top-level entries are those of the first batch (all there is for most plans)."""
        dev = self.device
        def to_dev(a: np.ndarray) -> torch.Tensor:
            return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1)).to(dev)
        lib = _lib.load()
        batches = []
        for b in plan["batches"]:
            batches.append(dict(
                n_groups=len(b["groups"]), groups=to_dev(b["groups"]),
                terms_prefix=to_dev(b["terms_prefix"]), reduce_prefix=to_dev(b["reduce_prefix"]),
                scout_prefix=to_dev(b["scout_prefix"]),
                n_terms_blocks=int(b["terms_prefix"][-1]), n_reduce_blocks=int(b["reduce_prefix"][-1]),
                n_scout_blocks=int(b["scout_prefix"][-1]), total_rows=b["total_rows"],
                total_keys=b["total_keys"],
            ))
        max_rows = max([b["total_rows"] for b in batches], default=0)
        max_groups = max([b["n_groups"] for b in batches], default=0)
        max_keys = max([b["total_keys"] for b in batches], default=0)
        # several samples share one scout launch: their scout slabs lie behind one another; the
        # main launches take as many samples at a time as their slabs (26 KB per workgroup and
        # sample, written only where a chunk changes a minimum) fit MAIN_BATCH_SLAB_BYTES
        self._sample_batch = min(len(self.sample_slots), _lib.MAX_SAMPLE_BATCH)
        slab_bytes = _lib.SLOTS * _lib.LC_TILE * 12
        most = max([b["n_reduce_blocks"] for b in batches] + [1])
        self._main_batch = int(max(1, min(self._sample_batch, MAIN_BATCH_SLAB_BYTES // (most * slab_bytes))))
        # (two scout regions: the scout pass of the next batch of samples runs beside the main
        # launches of the current one)
        n_slabs = max([self._main_batch * b["n_reduce_blocks"] + 2 * self._sample_batch * b["n_scout_blocks"]
                       for b in batches] + [1])
        def workspace():
            return dict(
                row_terms=torch.empty(max(max_rows, 1) * _lib.ROW_TERMS, dtype=torch.float64, device=dev),
                stage_floor=torch.empty(lib.mist_stage_floor_doubles(max_rows, max_groups),
                                        dtype=torch.float64, device=dev),
                key_terms=torch.empty(max(lib.mist_key_terms_doubles(max_keys), 1),
                                      dtype=torch.float64, device=dev),
                partial_cost=torch.empty(n_slabs * _lib.SLOTS * _lib.LC_TILE, dtype=torch.float64, device=dev),
                partial_index=torch.empty(n_slabs * _lib.SLOTS * _lib.LC_TILE, dtype=torch.int32, device=dev),
            )
        # several batches alternate between two workspaces on two streams, so that the tail of
        # one batch's launches overlaps the start of the next
        workspaces = [workspace() for _ in range(2 if len(batches) > 1 else 1)]
        out = dict(
            batches=batches, workspaces=workspaces, **workspaces[0],
            n_groups=0, groups=None, terms_prefix=None, reduce_prefix=None, scout_prefix=None,
            n_terms_blocks=0, n_reduce_blocks=0, n_scout_blocks=0,
            grad_accum=torch.tensor(
                list(self.gradient_accumulation_steps_candidates) * len(self.tp_sizes),
                dtype=torch.int32, device=dev),
        )
        if batches:
            out.update({k: batches[0][k] for k in (
                "n_groups", "groups", "terms_prefix", "reduce_prefix", "scout_prefix",
                "n_terms_blocks", "n_reduce_blocks", "n_scout_blocks")})
        return out

    def launch(self, plan, dev_plan, tables, events: Optional[list] = None) -> None:
        """Enqueues the kernels for every requested sample on the current stream; ``tables`` are
        the output tables (``DeviceTables``) or the ``MistOutTables`` of their pointers.  With
        ``events`` (a list) the three kernels are launched through their own entry points and
        ``(name, start_event, end_event)`` triples recorded on that stream are appended."""
        if not dev_plan["batches"]:
            return
        lib = _lib.load()
        current = torch.cuda.current_stream(self.device)
        streams = [current]
        if len(dev_plan["workspaces"]) > 1 and events is None:
            side = _side_stream(self.device)
            streams.append(side)
            side.wait_stream(current)  # the tables are filled on the current stream
        ratios = alpha_ratios(self.sample_size)
        out = tables.as_struct() if isinstance(tables, DeviceTables) else tables
        prob_ptr = ctypes.c_void_p(plan["problem"].ctypes.data)

        def timed(name, call):
            if events is None:
                _lib.check(call(), name)
                return
            start = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            start.record()
            _lib.check(call(), name)
            end.record()
            events.append((name, start, end))

        for bi, d in enumerate(dev_plan["batches"]):
            # batch bi: stream bi % 2 and workspace bi % 2 (the same pairing every time, so a
            # workspace is reused in stream order)
            stream = ctypes.c_void_p(streams[bi % len(streams)].cuda_stream)
            w = dev_plan["workspaces"][bi % len(dev_plan["workspaces"])]
            # (the structure is read when a call is made: only the first batch of a search forms
            # a first estimate, the others find the estimates of the batches before them)
            plan["problem"]["incumbent_first_estimate"] = (
                1 if bi == 0 and os.environ.get("MIST_NO_FIRST_ESTIMATE") is None else 0)

            def reduce_call(slot):
                if self.exhaustive:
                    return lib.mist_eval_reduce_exhaustive(
                        prob_ptr, _ptr(d["groups"]), d["n_groups"], _ptr(d["reduce_prefix"]),
                        d["n_reduce_blocks"], _ptr(w["row_terms"]), float(ratios[slot]),
                        _ptr(w["partial_cost"]), _ptr(w["partial_index"]), stream)
                return lib.mist_eval_reduce(
                    prob_ptr, _ptr(d["groups"]), d["n_groups"], _ptr(d["reduce_prefix"]),
                    d["n_reduce_blocks"], _ptr(d["scout_prefix"]), d["n_scout_blocks"],
                    _ptr(w["row_terms"]), _ptr(w["stage_floor"]), float(ratios[slot]),
                    _ptr(w["partial_cost"]), _ptr(w["partial_index"]), stream)

            if events is None and not self.exhaustive and len(self.sample_slots) > 1:
                slots = np.array(self.sample_slots, dtype=np.int32)
                all_ratios = np.ascontiguousarray(ratios[slots], dtype=np.float64)
                rc = lib.mist_intra_stage_eval_samples(
                    prob_ptr, _ptr(d["groups"]), d["n_groups"], _ptr(d["terms_prefix"]),
                    d["n_terms_blocks"], _ptr(d["reduce_prefix"]), d["n_reduce_blocks"],
                    _ptr(d["scout_prefix"]), d["n_scout_blocks"], _ptr(w["row_terms"]),
                    _ptr(w["stage_floor"]), _ptr(w["key_terms"]), _ptr(w["partial_cost"]),
                    _ptr(w["partial_index"]), ctypes.c_void_p(all_ratios.ctypes.data),
                    ctypes.c_void_p(slots.ctypes.data), len(slots), self._sample_batch,
                    min(self._main_batch, self._sample_batch), ctypes.byref(out), stream)
                _lib.check(rc, "mist_intra_stage_eval_samples")
                continue
            for i, slot in enumerate(self.sample_slots):
                if events is None and not self.exhaustive:
                    rc = lib.mist_intra_stage_eval(
                        prob_ptr, _ptr(d["groups"]), d["n_groups"],
                        _ptr(d["terms_prefix"]), d["n_terms_blocks"],
                        _ptr(d["reduce_prefix"]), d["n_reduce_blocks"],
                        _ptr(d["scout_prefix"]), d["n_scout_blocks"],
                        _ptr(w["row_terms"]), _ptr(w["stage_floor"]), _ptr(w["key_terms"]),
                        _ptr(w["partial_cost"]), _ptr(w["partial_index"]), float(ratios[slot]), int(slot),
                        1 if i == 0 else 0, ctypes.byref(out), stream,
                    )
                    _lib.check(rc, "mist_intra_stage_eval")
                    continue
                if i == 0:
                    timed("row_terms", lambda: lib.mist_row_terms(
                        prob_ptr, _ptr(d["groups"]), d["n_groups"], _ptr(d["terms_prefix"]),
                        d["n_terms_blocks"], _ptr(w["row_terms"]), _ptr(w["stage_floor"]),
                        _ptr(w["key_terms"]), stream))
                timed("eval_reduce", lambda: reduce_call(slot))
                timed("finalize", lambda: lib.mist_finalize(
                    prob_ptr, _ptr(d["groups"]), d["n_groups"], _ptr(d["reduce_prefix"]),
                    _ptr(w["row_terms"]), _ptr(w["partial_cost"]), _ptr(w["partial_index"]), int(slot),
                    ctypes.byref(out), stream))
        if len(streams) > 1:
            current.wait_stream(streams[1])

    def _outputs(self, plan, tables: DeviceTables) -> List[IntraStageTunerOutput]:
        Gn = len(self.gradient_accumulation_steps_candidates)
        outs = []
        for t in range(len(self.tp_sizes)):
            view = DeviceTables(
                stable=[x[t * Gn:(t + 1) * Gn] for x in tables.stable],
                delta=[x[t * Gn:(t + 1) * Gn] for x in tables.delta],
                index=[x[t * Gn:(t + 1) * Gn] for x in tables.index],
            )
            spaces = _SpacesOfEntry(plan["spaces"], t)
            outs.append(IntraStageTunerOutput(
                self.gradient_accumulation_steps_candidates, self.device_mesh_candidates, view,
                spaces, self.sample_slots, batch=tables, batch_index=t,
            ))
        return outs

    def run_prepared(self, plan, dev_plan,
                     stage_cost_cutoff: Optional[dict] = None) -> List[IntraStageTunerOutput]:
        """Device part only: fresh output tables + kernel launches for an uploaded plan; one
        output per tp size, all resident in the same tables.

        ``stage_cost_cutoff`` (``num_devices``, ``ckpt_rule``; one sample only) is for a caller
        whose inter-stage search is all that reads the tables: the scout pass turns its seeds
        into an upper bound of the best pipeline cost (``MistProblem.stage_cost_incumbent``),
        and the main launch does not look for stage costs that no threshold of that search can
        admit.  Cells above that bound then hold some value above it, not their minimum."""
        problem = plan["problem"]
        problem["stage_cost_incumbent"] = 0
        if stage_cost_cutoff is not None and self.sample_size == 1 and not self.exhaustive:
            with torch.cuda.device(self.device):
                if "incumbent" not in dev_plan:
                    dev_plan["incumbent"] = torch.empty(1, dtype=torch.float64, device=self.device)
                dev_plan["incumbent"].fill_(float("inf"))
            problem["stage_cost_incumbent"] = dev_plan["incumbent"].data_ptr()
            problem["incumbent_num_devices"] = int(stage_cost_cutoff["num_devices"])
            problem["incumbent_ckpt_rule"] = int(stage_cost_cutoff["ckpt_rule"])
        with torch.cuda.device(self.device):
            costs, index, struct = self._allocate_flat(plan)
            self.launch(plan, dev_plan, struct)
            # (the tensor views of the tables are made while the kernels run)
            tables = self._table_views(costs, index)
            tables.grad_accum = dev_plan.get("grad_accum")
        return self._outputs(plan, tables)

    def tune_all(self) -> List[IntraStageTunerOutput]:
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise _lib.MistLibraryError("IntraStageTuner needs a GPU: the search kernels have no CPU path")
        _lib.load()
        plan = self.prepare()
        with torch.cuda.device(self.device):
            dev_plan = self.upload(plan)
        self._plan, self._dev_plan = plan, dev_plan
        return self.run_prepared(plan, dev_plan)

    def tune(self) -> IntraStageTunerOutput:
        if len(self.tp_sizes) != 1:
            raise ValueError("tune() returns one table set; use tune_all() for several tp sizes")
        self.results = self.tune_all()[0]
        return self.results


def intra_stage_tune(
    layer_tables: LayerTables,
    num_layers: int,
    device_mesh_candidates: List[Tuple[int, int]],
    gradient_accumulation_steps_candidates: List[int],
    tp_size: Optional[int],
    mist_config: MistConfig,
    disable_tqdm: bool = True,
    sample_size: int = SAMPLE_SIZE,
    sample_slots: Optional[Sequence[int]] = None,
    device: str = "cuda:0",
) -> IntraStageTunerOutput:
    """Reference: ``intra_stage_tune`` (mist/analyzer/intra_tuning.py:285-370) without the
    pickle cache (results are recomputed; a tuner call takes milliseconds here)."""
    return IntraStageTuner(
        layer_tables, num_layers, device_mesh_candidates, gradient_accumulation_steps_candidates,
        tp_size, mist_config, disable_tqdm=disable_tqdm, sample_size=sample_size,
        sample_slots=sample_slots, device=device,
    ).tune()
