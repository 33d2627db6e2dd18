"""Oracle (test infrastructure): end-to-end composition, the CPU counterpart of
``mist_amd.tune_one_case.tune`` for the granularities that module implements.

Follows the working branches of benchmark/mist/tune/tune_one_case.py (:186-232 loop over the
tensor-parallel candidates, strict ``<`` keeps the first best) with the inter-stage DP
(:326-360) on top of the stable/delta adapter of ``oracle.inter_dp``.
"""
from .dp_c import dp_impl_c
from .inter_dp import dp_impl, inter_stage_tune
from .inter_uniform import inter_stage_tune_uniform
from .inter_mip import inter_stage_tune as inter_stage_tune_mip
from .inter_uniform_device import inter_stage_tune as inter_stage_tune_uniform_device
from .intra import intra_stage_tune
from .search_space import device_mesh_candidates, grad_accumu_steps_candidates


def tp_candidates(config):
    if getattr(config, "disable_tp_tuning", False):
        return [1]
    return [tp for tp in (1, 2, 4, 8) if tp <= config.hardware.num_gpus_per_node]


def tune(config, tables, use_c_dp=True):
    hw = config.hardware
    L = config.model.num_hidden_layers
    meshes = device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, contiguous_inter_node=False)
    Gs = grad_accumu_steps_candidates(config.training.global_batch_size)
    gran = config.tuning.tuning_granularity
    best_cost, best_solution = float("inf"), None
    for tp in tp_candidates(config):
        if gran == "inter-stage":
            r = intra_stage_tune(tables, config, L, meshes, Gs, tp, config.tuning.sample_size)
            cost, sol = inter_stage_tune(
                L, hw.num_nodes * hw.num_gpus_per_node, meshes, Gs, r, slot=0,
                dp=dp_impl_c if use_c_dp else dp_impl,
            )
        elif gran == "uniform-device-pp":
            r = intra_stage_tune(tables, config, L, meshes, Gs, tp, config.tuning.sample_size)
            cost, sol = inter_stage_tune_uniform_device(
                L, hw.num_nodes, hw.num_gpus_per_node, meshes, Gs, r, config, slot=0)
        elif gran == "uniform-device-pp-mip":
            r = intra_stage_tune(tables, config, L, meshes, Gs, tp, config.tuning.sample_size)
            cost, sol = inter_stage_tune_mip(L, hw.num_nodes, hw.num_gpus_per_node, meshes, Gs, r, config)
        elif gran in ("uniform-pp", "uniform-pp-simple-heuristic-mem-opt"):
            r = intra_stage_tune(tables, config, L, meshes, Gs, tp, 30)
            cost, sol = inter_stage_tune_uniform(
                L, hw.num_nodes, hw.num_gpus_per_node, Gs, r,
                ckpt_tuning=config.tuning.activation_checkpointing_tuning_enabled,
                simple=gran == "uniform-pp-simple-heuristic-mem-opt",
            )
        else:
            raise NotImplementedError(gran)
        if cost < best_cost:
            best_cost, best_solution = cost, sol
    return best_cost, best_solution
