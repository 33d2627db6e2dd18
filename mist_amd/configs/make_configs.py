"""Writes the five seeded synthetic tuning plans next to this file (``python make_configs.py``).

Each YAML is a fully resolved tuning input in the reference's format
(benchmark/mist/configs/test-small-base.yaml is the model) plus the ``tuning.search_space`` and
``synthetic`` extension blocks.  Hardware coefficients are drawn from
``numpy.random.default_rng(1000 + index)`` in this fixed order:

1. the 16 GPU<->GPU cells, inter size (1,2,4,8) outer, intra size (1,2,4,8) inner, each
   ``k ~ U(100, 450)`` GB/s when inter == 1 (intra-node) else ``U(10, 50)``, then
   ``alpha ~ U(5e-6, 50e-6)`` s;
2. CPU->GPU ``(k ~ U(20, 55), alpha ~ U(5e-6, 20e-6))``, then GPU->CPU likewise;
3. the 28 interference factors ``~ U(1, 3)``.

Op efficiencies come from ``layer_tables.draw_op_efficiency(seed)``.  All drawn values are
stored in the YAML, so the files, not the generator, are the source of truth.
"""
import os
import sys

import numpy as np
import yaml

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from mist_amd.layer_tables import draw_op_efficiency  # noqa: E402


def ratios(step):
    n = int(round(1.0 / step))
    return [round(i * step, 10) for i in range(n + 1)]


PLANS = [
    dict(
        file="gpt-1.3b-b8-1x2",
        model=dict(name="gpt2-1.3b", hidden_size=2048, num_attention_heads=16,
                   num_hidden_layers=24, vocab_size=50257, use_flash_attn=False),
        seq=2048, dtype="float16", batch=8, nodes=1, gpus=2, mem=24.0, peak=121.0, hbm=300.0,
        b_cands=[1, 2, 4, 8], off=ratios(0.25),
    ),
    dict(
        file="gpt-7b-b512-4x8",
        model=dict(name="gpt2-7b", hidden_size=4096, num_attention_heads=32,
                   num_hidden_layers=32, vocab_size=50257, use_flash_attn=True),
        seq=2048, dtype="float16", batch=512, nodes=4, gpus=8, mem=80.0, peak=312.0, hbm=2039.0,
        b_cands=[1, 2, 4, 8], off=ratios(0.1),
    ),
    dict(
        file="llama-13b-b1024-8x8",
        model=dict(name="llama-13b", hidden_size=5120, num_attention_heads=40,
                   num_hidden_layers=40, vocab_size=32000, use_flash_attn=True,
                   intermediate_size=13824, mlp_type="gated_mlp", normalization="rmsnorm",
                   position_embedding_type="rotary"),
        seq=4096, dtype="bfloat16", batch=1024, nodes=8, gpus=8, mem=80.0, peak=312.0, hbm=2039.0,
        b_cands=list(range(1, 17)), off=ratios(0.1),
    ),
    dict(
        file="gpt-22b-b1536-16x8",
        model=dict(name="gpt2-22b", hidden_size=6144, num_attention_heads=48,
                   num_hidden_layers=48, vocab_size=50257, use_flash_attn=True),
        seq=2048, dtype="float16", batch=1536, nodes=16, gpus=8, mem=80.0, peak=312.0, hbm=2039.0,
        # 1536 = 3 * 2**9: power-of-two data-parallel sizes need micro-batches that carry the 3.
        b_cands=[3, 6, 12, 24], off=ratios(0.05),
    ),
    dict(
        file="llama-70b-b2048-32x8",
        model=dict(name="llama-70b", hidden_size=8192, num_attention_heads=64, num_heads_kv=8,
                   num_hidden_layers=80, vocab_size=32000, use_flash_attn=True,
                   intermediate_size=28672, mlp_type="gated_mlp", normalization="rmsnorm",
                   position_embedding_type="rotary"),
        seq=4096, dtype="bfloat16", batch=2048, nodes=32, gpus=8, mem=80.0, peak=312.0, hbm=2039.0,
        b_cands=[1, 2, 4, 8], off=ratios(0.1),
    ),
]


def draw_hardware(seed):
    rng = np.random.default_rng(seed)
    gg = []
    for inter in (1, 2, 4, 8):
        for _intra in (1, 2, 4, 8):
            k = rng.uniform(100, 450) if inter == 1 else rng.uniform(10, 50)
            alpha = rng.uniform(5e-6, 50e-6)
            gg += [float(k), float(alpha)]
    cg = [float(rng.uniform(20, 55)), float(rng.uniform(5e-6, 20e-6))]
    gc = [float(rng.uniform(20, 55)), float(rng.uniform(5e-6, 20e-6))]
    interf = [float(x) for x in rng.uniform(1, 3, size=28)]
    return gg, cg, gc, interf


def build(index, plan):
    seed = 1000 + index
    gg, cg, gc, interf = draw_hardware(seed)
    model = dict(
        intermediate_size=4 * plan["model"]["hidden_size"], num_heads_kv=None, mlp_type="mlp",
        normalization="layernorm", position_embedding_type="absolute",
        tie_word_embeddings=False,
    )
    model.update(plan["model"])
    return dict(
        name=plan["file"],
        training=dict(
            max_sequence_length=plan["seq"], vocab_size=plan["model"]["vocab_size"],
            global_batch_size=plan["batch"], params_dtype=plan["dtype"],
            exec_dtype=plan["dtype"], optimizer_dtype="float32", autocast_enabled=False,
            optimizer_name="adamw",
        ),
        hardware=dict(
            gpu_type=None, num_nodes=plan["nodes"], num_gpus_per_node=plan["gpus"],
            gpu_gpu_comm_params=gg, cpu_gpu_comm_params=cg, gpu_cpu_comm_params=gc,
            interference_model_params=interf, nvlink=True, memory_capacity=plan["mem"],
        ),
        strategy=dict(enabled=False),
        tuning=dict(
            enabled=True, zero_2_and_3_enabled=True,
            activation_checkpointing_tuning_enabled=True, state_offloading_enabled=True,
            activation_offloading_enabled=True, tuning_granularity="inter-stage", sample_size=1,
            pre_post_strategy="dp", pre_post_strategy_array=None,
            search_space=dict(
                batch_size_candidates=plan["b_cands"],
                offloading_ratio_candidates=plan["off"],
                sparse_offloading_ratio_candidates=plan["off"],
                zero_flag_choices=[[0, 0, 0], [0, 0, 1], [0, 1, 1], [1, 1, 1]],
            ),
        ),
        enable_advanced_opt_in_first_block=True,
        disable_tp_tuning=False,
        model=model,
        synthetic=dict(
            seed=seed, peak_tflops=plan["peak"], hbm_gbps=plan["hbm"],
            op_efficiency=draw_op_efficiency(seed),
        ),
    )


def main():
    for index, plan in enumerate(PLANS, start=1):
        path = os.path.join(HERE, plan["file"] + ".yaml")
        with open(path, "w") as f:
            f.write(f"# plan {index}; generated by make_configs.py, seed {1000 + index}\n")
            yaml.safe_dump(build(index, plan), f, sort_keys=False)
        print("wrote", path)


if __name__ == "__main__":
    main()
