"""Oracle (test infrastructure): candidate enumeration.

Restates ``create_search_space_for_a_block_layer`` (mist/analyzer/batched_module_analyzer.py:
417-536, ``np_product`` :78-97) and the two live helpers of mist/tuning/optimization.py:30-55.

Pinned by: closed-form row count ``|par| * (k_wo*k_go*k_oo*k_ao - (#wo>0)*(#go==0)*k_oo*k_ao)``,
``itertools.product`` ordering, powers-of-two closed form for the mesh / G lists
(tests/test_oracle_search_space.py).
"""
from itertools import product

import numpy as np

POWER_OF_TWO = [2**i for i in range(0, 15)]


def device_mesh_candidates(num_nodes, num_gpus_per_node, contiguous_inter_node=True):
    """optimization.py:33-51."""
    out = []
    for m in range(1, num_gpus_per_node + 1):
        if m in POWER_OF_TWO:
            out.append((1, m))
    for n in range(2, num_nodes + 1):
        if contiguous_inter_node or n in POWER_OF_TWO:
            out.append((n, num_gpus_per_node))
    assert len(out) == len(set(out))
    return out


def grad_accumu_steps_candidates(global_batch_size):
    """optimization.py:54-55."""
    return [i for i in POWER_OF_TWO if global_batch_size % i == 0]


def create_search_space(
    num_nodes,
    num_gpus_per_node,
    global_batch_size,
    gradient_accumulation_steps,
    config,
    constraint_fn=None,
    tp_size=None,
):
    """batched_module_analyzer.py:417-536.  Candidate lists come from ``config.tuning``
    (defaults = the reference's module constants).  Returns an (N, 10) float64 array of rows
    ``(b, dp, tp, wre, gre, ore, wo, go, oo, ao)``, parallelism-major, offload-minor."""
    tuning = config.tuning
    num_gpus = num_nodes * num_gpus_per_node
    per_micro_batch = global_batch_size // gradient_accumulation_steps

    par = []
    for b in tuning.batch_size_candidates:
        if b > per_micro_batch or per_micro_batch % b != 0:
            continue
        dp = per_micro_batch // b
        if dp > num_gpus or num_gpus % dp != 0:
            continue
        cur_tp = num_gpus // dp
        if constraint_fn is not None and not constraint_fn(b, cur_tp):
            continue
        tp_size = cur_tp if tp_size is None else tp_size  # latches to the first feasible b
        if tp_size != cur_tp:
            continue
        if tp_size > num_gpus_per_node:
            continue
        if getattr(config, "disable_tp_tuning", False) and tp_size > 1:
            continue
        if dp == 1 or not tuning.zero_2_and_3_enabled:
            flag_choices = [(0, 0, 1)]
        else:
            flag_choices = tuning.zero_flag_choices
        for wre, gre, ore in flag_choices:
            par.append((b, dp, tp_size, wre, gre, ore))
    par = np.array(par).reshape(-1, 6)

    dense = tuning.offloading_ratio_candidates
    sparse = tuning.sparse_offloading_ratio_candidates
    if tuning.state_offloading_enabled:
        wo, go, oo = sparse, sparse, dense
        if getattr(config, "disable_wo_tuning", False):
            wo = [0.0]
        if getattr(config, "disable_go_tuning", False):
            go = [0.0]
        if getattr(config, "disable_oo_tuning", False):
            oo = [0.0]
    else:
        wo, go, oo = [0.0], [0.0], [0.0]
    fixed = {k: getattr(config, f"fixed_{k}_ratio", None) for k in ("wo", "go", "oo", "ao")}
    if fixed["wo"] is not None:
        wo = [fixed["wo"]]
    if fixed["go"] is not None:
        go = [fixed["go"]]
    if fixed["oo"] is not None:
        oo = [fixed["oo"]]
    if tuning.activation_offloading_enabled:
        ao = dense
    elif fixed["ao"] is not None:
        ao = [fixed["ao"]]
    else:
        ao = [0.0]
    off = [r for r in product(wo, go, oo, ao) if not (r[0] > 0 and r[1] == 0)]
    off = np.array(off, dtype=np.float64).reshape(-1, 4)

    # np_product(par, off, combine_dims=True): repeat par rows, tile off rows.
    rows = np.concatenate(
        [np.repeat(par, off.shape[0], axis=0), np.tile(off, (par.shape[0], 1))], axis=-1
    )
    return rows.astype(np.float64).reshape(-1, 10)
