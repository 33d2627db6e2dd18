"""ctypes binding of libmist_search.so (declarations in include/mist_search.h).

There is no CPU fallback: if the shared library is missing or a call fails, this raises.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmist_search.so")

MAX_PAR = 64
MAX_RATIOS = 32
MAX_PAIRS = MAX_RATIOS * MAX_RATIOS
PAR_FIELDS = 20
ROW_TERMS = 34
LC_TILE = 64  # replaced by the library's own value in load()
P_TILE = 32  # replaced by the library's own value in load()
SLOTS = 2 * P_TILE + 2
SCOUT_SPLIT = 4  # replaced by the library's own value in load()
STAGE_ROWS = 64  # replaced by the library's own value in load()
TERMS_BLOCK = 128  # replaced by the library's own value in load()
MAX_MESH = 16
MAX_SAMPLE_BATCH = 16  # MIST_MAX_SAMPLE_BATCH; replaced by the library's own value in load()
MAX_SCOUT_PAIRS = 8  # MIST_MAX_SCOUT_PAIRS (sizes a field of GROUP_DTYPE; checked in load())
KEY_TERMS = 28  # MIST_KEY_TERMS; replaced by the library's own value in load()
DP_NO_START = -3
DP_CKPT_TAIL, DP_CKPT_STAGE, DP_CKPT_ALL = 0, 1, 2
DP_THRESHOLD, DP_BOTTLENECK = 0, 1

PAR_NAMES = (
    "b", "dp", "tp", "wre", "gre", "ore", "W", "G", "O", "raw_ck", "raw_nock", "fwd_peak",
    "bwd_peak", "out", "gcb", "exec_fwd", "exec_bwd", "extra_fwd", "extra_bwd", "reserved",
)
PAR = {name: i for i, name in enumerate(PAR_NAMES)}
TERM_NAMES = (
    "s_layer_ck", "s_layer_nock", "s_first_ck", "s_first_nock", "s_last_ck", "s_last_nock",
    "d_layer_ck", "d_layer_nock", "d_first_ck", "d_first_nock", "d_last_ck", "d_last_nock",
    "fwd_states0", "bwd_states0", "pWG", "pO", "pWGO", "S_ck", "S_nock", "D_ck", "D_nock",
    "mf_base", "mf_pp", "mf", "fwd_peak", "bwd_peak", "out", "gcb",
    "nAG_ck", "nAG_nock", "nRS_ck", "nRS_nock", "opb", "RD",
)
TERM = {name: i for i, name in enumerate(TERM_NAMES)}
assert len(TERM_NAMES) == ROW_TERMS and len(PAR_NAMES) == PAR_FIELDS

PROBLEM_DTYPE = np.dtype(
    [
        ("gpu_gpu", "<f8", (32,)),
        ("cpu_gpu", "<f8", (2,)),
        ("gpu_cpu", "<f8", (2,)),
        ("interf_factor", "<f8", (11, 4)),
        ("mem_cap_mb", "<f8"),
        ("frag_factor", "<f8"),
        ("num_layers", "<i4"),
        ("p_dim", "<i4"),
        ("sample_size", "<i4"),
        ("num_grad_accum", "<i4"),
        ("num_mesh", "<i4"),
        ("adv_first_block", "<i4"),
        ("max_scout_rows", "<i4"),
        ("max_group_keys", "<i4"),
        ("stage_cost_incumbent", "<u8"),
        ("incumbent_num_devices", "<i4"),
        ("incumbent_ckpt_rule", "<i4"),
        ("incumbent_first_estimate", "<i4"),
        ("reserved0", "<i4"),
    ],
    align=True,
)

GROUP_DTYPE = np.dtype(
    [
        ("g_index", "<i4"), ("q_index", "<i4"),
        ("num_nodes", "<i4"), ("num_gpus_per_node", "<i4"),
        ("grad_accum", "<i4"), ("num_p", "<i4"),
        ("n_par", "<i4"), ("n_pair", "<i4"), ("n_oo", "<i4"), ("n_ao", "<i4"), ("n_off", "<i4"),
        ("pp_wre", "<i4"), ("pp_gre", "<i4"),
        ("rows_per_chunk", "<i4"), ("n_chunks", "<i4"), ("n_lc_tiles", "<i4"),
        ("n_p_tiles", "<i4"), ("lc_tile_begin", "<i4"), ("scout_stride", "<i4"),
        ("scout_pair", "<i2", (MAX_SCOUT_PAIRS,)),
        ("n_rows", "<i8"), ("row_offset", "<i8"), ("key_offset", "<i8"),
        ("par", "<f8", (MAX_PAR, PAR_FIELDS)),
        ("wo", "<f8", (MAX_RATIOS,)), ("go", "<f8", (MAX_RATIOS,)),
        ("oo", "<f8", (MAX_RATIOS,)), ("ao", "<f8", (MAX_RATIOS,)),
        ("pair_wo", "u1", (MAX_PAIRS,)), ("pair_go", "u1", (MAX_PAIRS,)),
        ("pre_full_w", "<f8"), ("pre_full_g", "<f8"), ("post_full_w", "<f8"), ("post_full_g", "<f8"),
        ("pre_states", "<f8"), ("pre_saved", "<f8"), ("pre_states_and_saved", "<f8"),
        ("post_states", "<f8"), ("post_fwd_peak", "<f8"), ("post_bwd_peak", "<f8"),
        ("post_output", "<f8"),
        ("pre_fwd", "<f8"), ("pre_bwd", "<f8"), ("post_fwd", "<f8"), ("post_bwd", "<f8"),
        ("pre_ag", "<f8"), ("pre_rs", "<f8"), ("post_ag", "<f8"), ("post_rs", "<f8"),
    ],
    align=True,
)


class OutTables(ctypes.Structure):
    _fields_ = [
        ("stable", ctypes.c_void_p * 4),
        ("delta", ctypes.c_void_p * 4),
        ("index", ctypes.c_void_p * 4),
    ]


class MistLibraryError(RuntimeError):
    pass


_LIB = None

_VP = ctypes.c_void_p
_SIGNATURES = {
    "mist_version": (ctypes.c_char_p, []),
    "mist_last_error": (ctypes.c_char_p, []),
    "mist_sizeof_problem": (ctypes.c_int, []),
    "mist_incumbent_slack": (ctypes.c_double, []),
    "mist_sizeof_group": (ctypes.c_int, []),
    "mist_reduce_p_tile": (ctypes.c_int, []),
    "mist_reduce_stage_rows": (ctypes.c_int, []),
    "mist_workspace_oo_tile": (ctypes.c_int, []),
    "mist_reduce_lc_tile": (ctypes.c_int, []),
    "mist_terms_block_rows": (ctypes.c_int, []),
    "mist_reduce_scout_split": (ctypes.c_int, []),
    "mist_max_sample_batch": (ctypes.c_int, []),
    "mist_key_terms_per_key": (ctypes.c_int, []),
    "mist_max_scout_pairs": (ctypes.c_int, []),
    "mist_stage_floor_doubles": (ctypes.c_int64, [ctypes.c_int64, ctypes.c_int]),
    "mist_key_terms_doubles": (ctypes.c_int64, [ctypes.c_int64]),
    "mist_row_terms": (ctypes.c_int, [_VP, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, _VP, _VP, _VP]),
    "mist_eval_reduce": (
        ctypes.c_int,
        [_VP, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, _VP, ctypes.c_double,
         _VP, _VP, _VP],
    ),
    "mist_stage_cost_first_estimate": (
        ctypes.c_int,
        [_VP, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, ctypes.c_double, _VP, _VP],
    ),
    "mist_eval_reduce_samples": (
        ctypes.c_int,
        [_VP, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, _VP, _VP, _VP,
         ctypes.c_int, ctypes.c_int, _VP, _VP, ctypes.POINTER(OutTables), _VP],
    ),
    "mist_intra_stage_eval_samples": (
        ctypes.c_int,
        [_VP, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, ctypes.c_int,
         _VP, _VP, _VP, _VP, _VP, _VP, _VP, ctypes.c_int, ctypes.c_int, ctypes.c_int,
         ctypes.POINTER(OutTables), _VP],
    ),
    "mist_eval_reduce_exhaustive": (
        ctypes.c_int,
        [_VP, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, ctypes.c_double, _VP, _VP, _VP],
    ),
    "mist_finalize": (
        ctypes.c_int,
        [_VP, _VP, ctypes.c_int, _VP, _VP, _VP, _VP, ctypes.c_int, ctypes.POINTER(OutTables), _VP],
    ),
    "mist_stage_analyze": (
        ctypes.c_int, [_VP, _VP, ctypes.c_int, _VP, _VP, ctypes.c_int, _VP, _VP]),
    "mist_row_diagnostics": (
        ctypes.c_int, [_VP, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, _VP]),
    "mist_intra_stage_eval": (
        ctypes.c_int,
        [_VP, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, ctypes.c_int, _VP, ctypes.c_int,
         _VP, _VP, _VP, _VP, _VP, ctypes.c_double, ctypes.c_int, ctypes.c_int, ctypes.POINTER(OutTables), _VP],
    ),
}


def workspace_positions(n_par: int, n_pair: int, n_oo: int, n_ao: int) -> np.ndarray:
    """Position in the row-term workspace of every reference row of a group (see
    include/mist_search.h: per (par, ao) the workspace holds the optimizer ratios in tiles of
    ``mist_workspace_oo_tile()`` and the pairs inside a tile one after the other; the reference
    numbers rows (par, pair, oo, ao))."""
    T = load().mist_workspace_oo_tile()
    n_off = n_pair * n_oo * n_ao
    row = np.arange(n_par * n_off, dtype=np.int64)
    par, off = row // n_off, row % n_off
    pair, oo, ao = off // (n_oo * n_ao), (off // n_ao) % n_oo, off % n_ao
    tile = oo // T
    width = np.minimum(T, n_oo - tile * T)
    return par * n_off + ao * (n_oo * n_pair) + tile * T * n_pair + pair * width + oo % T


def exported_symbols():
    """Names every entry point declared in include/mist_search.h, mist_dp.h, mist_mip.h,
    mist_inter.h and mist_plan.h."""
    return (tuple(_SIGNATURES) + tuple(_DP_SIGNATURES) + tuple(_MIP_SIGNATURES) + tuple(_INTER_SIGNATURES)
            + tuple(_PLAN_SIGNATURES))


DP_SHAPE_DTYPE = np.dtype(
    [
        ("num_layers", "<i4"), ("num_devices", "<i4"), ("num_mesh", "<i4"), ("p_dim", "<i4"),
        ("max_stages", "<i4"), ("ckpt_rule", "<i4"), ("free_devices", "<i4"), ("reserved", "<i4"),
        ("mesh_n", "<i4", (MAX_MESH,)), ("mesh_m", "<i4", (MAX_MESH,)),
    ],
    align=True,
)


class DpCosts(ctypes.Structure):
    _fields_ = [
        ("costs", ctypes.c_void_p),
        ("costs_pre", ctypes.c_void_p),
        ("costs_post", ctypes.c_void_p),
        ("costs_nopp", ctypes.c_void_p),
        ("pmin", ctypes.c_void_p),
        ("pmin_pre", ctypes.c_void_p),
        ("pmin_post", ctypes.c_void_p),
        ("pmin_nopp", ctypes.c_void_p),
        ("g_stride", ctypes.c_int64 * 4),
        ("stage_min", ctypes.c_void_p),
        ("stage_min_g_stride", ctypes.c_int64),
    ]


_DP_SIGNATURES = {
    "mist_sizeof_dp_shape": (ctypes.c_int, []),
    "mist_dp_cost_tables": (
        ctypes.c_int,
        [_VP, ctypes.POINTER(OutTables), _VP, ctypes.c_int, ctypes.c_void_p * 4, ctypes.c_void_p * 4, _VP],
    ),
    "mist_dp_filter_tmax": (ctypes.c_int, [_VP, ctypes.c_int, ctypes.c_double, _VP]),
    "mist_dp_windows_first_batch": (
        ctypes.c_int,
        [ctypes.POINTER(DpCosts), ctypes.c_int, _VP, _VP, _VP, _VP, ctypes.c_double, ctypes.c_int,
         ctypes.c_int, ctypes.c_int, _VP, _VP, _VP, ctypes.c_int, _VP, _VP, _VP, _VP]),
    "mist_dp_first_batch_index": (
        ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "mist_dp_window_begin": (
        ctypes.c_int,
        [_VP, ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_double, _VP]),
    "mist_dp_window_begin_many": (
        ctypes.c_int, [_VP, _VP, ctypes.c_int, _VP, _VP, _VP, ctypes.c_double, _VP, _VP]),
    "mist_dp_select_candidates": (
        ctypes.c_int,
        [ctypes.POINTER(DpCosts), ctypes.c_int, _VP, _VP, _VP, _VP, _VP, ctypes.c_int, _VP, _VP],
    ),
    "mist_dp_scratch_floats": (ctypes.c_int64, [_VP, ctypes.c_int]),
    "mist_dp_backtrack": (ctypes.c_int, [_VP, _VP, _VP, ctypes.c_int, _VP, _VP]),
    "mist_dp_stage_minima_floats": (ctypes.c_int64, [_VP]),
    "mist_dp_stage_minima": (ctypes.c_int, [_VP, ctypes.POINTER(DpCosts), ctypes.c_int, _VP, _VP]),
    "mist_dp_run": (
        ctypes.c_int,
        [_VP, ctypes.POINTER(DpCosts), _VP, _VP, ctypes.c_int, ctypes.c_int, _VP, _VP, _VP, _VP, _VP, _VP],
    ),
    "mist_dp_static_scratch_floats": (ctypes.c_int64, []),
    "mist_dp_run_static": (
        ctypes.c_int,
        [_VP, ctypes.POINTER(DpCosts), _VP, _VP, ctypes.c_int, ctypes.c_int, _VP, _VP, _VP, _VP, _VP],
    ),
}


ANALYZE_REQUEST_FIELDS, ANALYZE_FIELDS = 5, 23
# MistDiagField: scalars, then 8 families x 5 members
DIAG_NAMES = (
    "so_W", "si_W", "so_G", "si_G", "so_O", "si_O", "so_A_ck", "si_A_ck", "so_A_nock", "si_A_nock",
    "AG_w", "RS_g", "AR_g", "Wbuf", "Gbuf", "pW", "pG",
    "g2c_F0", "c2g_F0", "g2g_F0", "g2c_F1", "c2g_F1", "g2g_F1", "g2c_B", "c2g_B", "g2g_B0", "g2g_B1",
)
DIAG = {name: i for i, name in enumerate(DIAG_NAMES)}
DIAG_FAMILIES = len(DIAG_NAMES)
DIAG_FAMILY_NAMES = ("fwd_first_nock", "fwd_first_ck", "fwd_later_nock", "fwd_later_ck",
                     "bwd_last_nock", "bwd_last_ck", "bwd_not_last_nock", "bwd_not_last_ck")
DIAG_MEMBERS = ("layer", "first", "last", "extra_pre", "extra_post")
DIAG_FIELDS = DIAG_FAMILIES + len(DIAG_FAMILY_NAMES) * len(DIAG_MEMBERS)
MIP_CKPT_TUNED, MIP_CKPT_FIXED, MIP_CKPT_FULL = 0, 1, 2
MIP_MAX_SAMPLES = 64
MIP_MAX_VALUE = 1000000.0


class MipShape(ctypes.Structure):
    """``MistMipShape`` of include/mist_mip.h."""

    _fields_ = [
        ("num_layers", ctypes.c_int32),
        ("p_dim", ctypes.c_int32),
        ("sample_size", ctypes.c_int32),
        ("num_stages", ctypes.c_int32),
        ("layers_min", ctypes.c_int32),
        ("layers_max", ctypes.c_int32),
        ("ckpt_mode", ctypes.c_int32),
        ("fixed_ckpt", ctypes.c_int32),
    ]


class MipTables(ctypes.Structure):
    """``MistMipTables``: device pointers of one (gradient accumulation, mesh) slice."""

    _fields_ = [("stable", ctypes.c_void_p * 4), ("delta", ctypes.c_void_p * 4)]


class MipBatchItem(ctypes.Structure):
    """``MistMipBatchItem``: one problem of a batched ``mist_mip_stage_samples_batch`` call."""

    _fields_ = [("shape", MipShape), ("tables", MipTables), ("out_offset", ctypes.c_int64),
                ("first_block", ctypes.c_int32), ("reserved", ctypes.c_int32)]


# MistMipBatchItem as a numpy record: a search fills the items of all its problems column-wise
MIP_ITEM_DTYPE = np.dtype(
    [
        ("num_layers", "<i4"), ("p_dim", "<i4"), ("sample_size", "<i4"), ("num_stages", "<i4"),
        ("layers_min", "<i4"), ("layers_max", "<i4"), ("ckpt_mode", "<i4"), ("fixed_ckpt", "<i4"),
        ("stable", "<u8", (4,)), ("delta", "<u8", (4,)),
        ("out_offset", "<i8"), ("first_block", "<i4"), ("reserved", "<i4"),
    ],
    align=True,
)
assert MIP_ITEM_DTYPE.itemsize == ctypes.sizeof(MipBatchItem)


class StrategyIndex(ctypes.Structure):
    """``MistStrategyIndex`` of include/mist_inter.h."""

    _fields_ = [
        ("index", ctypes.c_void_p * 4),
        ("num_layers", ctypes.c_int32),
        ("p_dim", ctypes.c_int32),
        ("num_mesh", ctypes.c_int32),
        ("sample_size", ctypes.c_int32),
        ("slot", ctypes.c_int32),
        ("mesh_n", ctypes.c_int32 * MAX_MESH),
        ("mesh_m", ctypes.c_int32 * MAX_MESH),
    ]


_INTER_SIGNATURES = {
    "mist_sizeof_strategy_index": (ctypes.c_int, []),
    "mist_inter_stage_search": (
        ctypes.c_int,
        [_VP, ctypes.POINTER(DpCosts), ctypes.c_int, ctypes.c_int, _VP, _VP, ctypes.c_int,
         _VP, _VP, _VP, _VP, _VP, _VP, _VP]),
    "mist_inter_stage_search_families": (
        ctypes.c_int,
        [ctypes.c_int, _VP, _VP, ctypes.POINTER(DpCosts), ctypes.POINTER(StrategyIndex),
         ctypes.c_int, ctypes.c_int, _VP, _VP, ctypes.c_int,
         _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP]),
    "mist_inter_stage_search_bounded": (
        ctypes.c_int,
        [ctypes.c_int, _VP, _VP, ctypes.POINTER(DpCosts), ctypes.POINTER(StrategyIndex),
         ctypes.c_int, ctypes.c_int, _VP, _VP, ctypes.c_int,
         _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, ctypes.c_double, _VP]),
}

PLAN_MAX_LIST = 32
PLAN_MAX_BATCH_SIZES = 64
PLAN_UNSUPPORTED = -3  # MIST_E_PLAN_UNSUPPORTED
# efficiency classes in the order of MistLayerShapes.efficiency (include/mist_plan.h)
PLAN_OP_CLASSES = (
    "qkv_gemm", "attn_core", "attn_softmax", "out_gemm", "fc1_gemm", "fc2_gemm", "activation",
    "norm", "embedding", "lm_head_gemm", "xentropy", "grad_accum",
)
PLAN_PP_MODES = {"dp": 0, "intra-node-tp-with-ore": 1, "intra-node-tp-without-ore": 2, "preset": 3}


class LayerShapes(ctypes.Structure):
    """MistLayerShapes (include/mist_plan.h)."""
    _fields_ = [
        ("hidden", ctypes.c_double), ("heads", ctypes.c_double), ("kv_heads", ctypes.c_double),
        ("ffn", ctypes.c_double), ("vocab", ctypes.c_double), ("seq_len", ctypes.c_double),
        ("norm_params", ctypes.c_double), ("opt_mult", ctypes.c_double),
        ("bytes_per_param", ctypes.c_double), ("peak_flops", ctypes.c_double),
        ("hbm_bw", ctypes.c_double),
        ("efficiency", (ctypes.c_double * 2) * len(PLAN_OP_CLASSES)),
        ("flash", ctypes.c_int32), ("gated", ctypes.c_int32), ("abs_pos", ctypes.c_int32),
        ("tied", ctypes.c_int32),
    ]


class PlanRequest(ctypes.Structure):
    """MistPlanRequest (include/mist_plan.h)."""
    _fields_ = [
        ("layers", LayerShapes),
        ("gpu_gpu", ctypes.c_double * 32),
        ("memory_capacity_gb", ctypes.c_double),
        ("wo", ctypes.c_double * MAX_RATIOS), ("go", ctypes.c_double * MAX_RATIOS),
        ("oo", ctypes.c_double * MAX_RATIOS), ("ao", ctypes.c_double * MAX_RATIOS),
        ("pp_preset", ctypes.c_double * 10),
        ("scout_tight_fraction", ctypes.c_double),
        ("global_batch_size", ctypes.c_int64),
        ("workspace_rows", ctypes.c_int64),
        ("model_heads", ctypes.c_int32), ("model_seq_len", ctypes.c_int32), ("model_flash", ctypes.c_int32),
        ("num_layers", ctypes.c_int32), ("max_pre_saved", ctypes.c_int32),
        ("evaluate_all_p", ctypes.c_int32), ("exhaustive", ctypes.c_int32),
        ("n_tp", ctypes.c_int32), ("tp_size", ctypes.c_int32 * PLAN_MAX_LIST),
        ("n_grad_accum", ctypes.c_int32), ("grad_accum", ctypes.c_int32 * PLAN_MAX_LIST),
        ("n_mesh", ctypes.c_int32), ("mesh_n", ctypes.c_int32 * MAX_MESH), ("mesh_m", ctypes.c_int32 * MAX_MESH),
        ("n_batch_sizes", ctypes.c_int32), ("batch_size", ctypes.c_int32 * PLAN_MAX_BATCH_SIZES),
        ("zero_2_and_3", ctypes.c_int32), ("n_flag_choices", ctypes.c_int32),
        ("flag_choice", (ctypes.c_int32 * 3) * PLAN_MAX_LIST),
        ("disable_tp", ctypes.c_int32), ("check_shapes", ctypes.c_int32),
        ("n_wo", ctypes.c_int32), ("n_go", ctypes.c_int32), ("n_oo", ctypes.c_int32),
        ("n_ao", ctypes.c_int32), ("n_pair", ctypes.c_int32),
        ("pair_wo", ctypes.c_uint8 * MAX_PAIRS), ("pair_go", ctypes.c_uint8 * MAX_PAIRS),
        ("pp_mode", ctypes.c_int32),
        ("target_reduce_waves", ctypes.c_int32), ("scout_min_stages", ctypes.c_int32),
        ("scout_min_pairs", ctypes.c_int32), ("scout_pairs", ctypes.c_int32),
        ("scout_pair_span", ctypes.c_int32), ("scout_tight_pairs", ctypes.c_int32),
        ("cells_wanted", ctypes.c_void_p),
    ]


class PlanResult(ctypes.Structure):
    """MistPlanResult (include/mist_plan.h)."""
    _fields_ = [
        ("n_groups", ctypes.c_int32), ("n_batches", ctypes.c_int32),
        ("max_scout_rows", ctypes.c_int32), ("max_group_keys", ctypes.c_int32),
        ("total_rows", ctypes.c_int64), ("n_space_rows", ctypes.c_int64),
    ]


_PLAN_SIGNATURES = {
    "mist_sizeof_plan_request": (ctypes.c_int, []),
    "mist_plan_groups": (
        ctypes.c_int,
        [ctypes.POINTER(PlanRequest), _VP, ctypes.c_int32, _VP, _VP, _VP, _VP, _VP, _VP, _VP,
         ctypes.POINTER(PlanResult)]),
}

_MIP_SIGNATURES = {
    "mist_sizeof_mip_shape": (ctypes.c_int, []),
    "mist_mip_stage_samples": (
        ctypes.c_int,
        [ctypes.POINTER(MipShape), ctypes.POINTER(MipTables), _VP, _VP, _VP, _VP, _VP, _VP],
    ),
    "mist_sizeof_mip_batch_item": (ctypes.c_int, []),
    "mist_mip_stage_samples_batch": (
        ctypes.c_int, [_VP, _VP, ctypes.c_int, _VP, _VP, _VP, _VP, _VP, _VP]),
    "mist_mip_prefill_cells": (
        ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, _VP, _VP,
                       ctypes.c_int, ctypes.POINTER(OutTables), _VP]),
    "mist_mip_solve_chains": (
        ctypes.c_int, [_VP, _VP, ctypes.c_int, ctypes.c_int, _VP, _VP, _VP, _VP, _VP, _VP, _VP]),
    "mist_mip_solve": (
        ctypes.c_int,
        [ctypes.POINTER(MipShape), ctypes.c_int, ctypes.c_double, _VP, _VP, _VP,
         ctypes.POINTER(ctypes.c_double), _VP, _VP],
    ),
}


def load():
    """Loads the shared library once; raises if it has not been built."""
    global _LIB
    if _LIB is not None:
        return _LIB
    if not os.path.exists(LIB_PATH):
        raise MistLibraryError(
            f"{LIB_PATH} is missing: build it with `python -m mist_amd.build` "
            "(there is no CPU fallback for the search kernels)"
        )
    # PyTorch brings its own HIP runtime; loaded first, the library binds to that one, and the
    # streams and device pointers torch hands over belong to the runtime the kernels run on
    # (loaded the other way round, the library's runtime sees no device).
    import torch  # noqa: F401

    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in {**_SIGNATURES, **_DP_SIGNATURES, **_MIP_SIGNATURES,
                                      **_INTER_SIGNATURES, **_PLAN_SIGNATURES}.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.mist_sizeof_problem() != PROBLEM_DTYPE.itemsize:
        raise MistLibraryError(
            f"MistProblem layout mismatch: C {lib.mist_sizeof_problem()} vs numpy {PROBLEM_DTYPE.itemsize}"
        )
    if lib.mist_sizeof_dp_shape() != DP_SHAPE_DTYPE.itemsize:
        raise MistLibraryError(
            f"MistDpShape layout mismatch: C {lib.mist_sizeof_dp_shape()} vs numpy {DP_SHAPE_DTYPE.itemsize}"
        )
    if lib.mist_sizeof_strategy_index() != ctypes.sizeof(StrategyIndex):
        raise MistLibraryError(
            f"MistStrategyIndex layout mismatch: C {lib.mist_sizeof_strategy_index()} vs ctypes "
            f"{ctypes.sizeof(StrategyIndex)}")
    if lib.mist_sizeof_mip_shape() != ctypes.sizeof(MipShape):
        raise MistLibraryError(
            f"MistMipShape layout mismatch: C {lib.mist_sizeof_mip_shape()} vs ctypes {ctypes.sizeof(MipShape)}"
        )
    if lib.mist_sizeof_mip_batch_item() != ctypes.sizeof(MipBatchItem):
        raise MistLibraryError(
            f"MistMipBatchItem layout mismatch: C {lib.mist_sizeof_mip_batch_item()} vs ctypes "
            f"{ctypes.sizeof(MipBatchItem)}")
    if lib.mist_sizeof_plan_request() != ctypes.sizeof(PlanRequest):
        raise MistLibraryError(
            f"MistPlanRequest layout mismatch: C {lib.mist_sizeof_plan_request()} vs ctypes "
            f"{ctypes.sizeof(PlanRequest)}")
    if lib.mist_sizeof_group() != GROUP_DTYPE.itemsize:
        raise MistLibraryError(
            f"MistGroupDesc layout mismatch: C {lib.mist_sizeof_group()} vs numpy {GROUP_DTYPE.itemsize}"
        )
    if lib.mist_max_scout_pairs() != MAX_SCOUT_PAIRS:
        raise MistLibraryError(
            f"MIST_MAX_SCOUT_PAIRS mismatch: C {lib.mist_max_scout_pairs()} vs python {MAX_SCOUT_PAIRS}")
    global P_TILE, SLOTS, STAGE_ROWS, LC_TILE, SCOUT_SPLIT, TERMS_BLOCK, MAX_SAMPLE_BATCH, KEY_TERMS
    MAX_SAMPLE_BATCH = lib.mist_max_sample_batch()
    KEY_TERMS = lib.mist_key_terms_per_key()
    TERMS_BLOCK = lib.mist_terms_block_rows()
    SCOUT_SPLIT = lib.mist_reduce_scout_split()
    LC_TILE = lib.mist_reduce_lc_tile()
    STAGE_ROWS = lib.mist_reduce_stage_rows()
    P_TILE = lib.mist_reduce_p_tile()
    SLOTS = 2 * P_TILE + 2
    _LIB = lib
    return lib


def check(rc: int, what: str):
    if rc != 0:
        msg = load().mist_last_error().decode(errors="replace")
        raise MistLibraryError(f"{what} failed with code {rc}: {msg}")
