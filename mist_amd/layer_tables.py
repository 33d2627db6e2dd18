"""Synthetic layer tables: the stand-in for the reference's three traced ``LayerInfo`` objects.

In the reference, ``LayerInfo`` (mist/analyzer/info.py:120-222) carries sympy memory expressions
in the two symbols (per-device batch ``b``, tensor-parallel size ``tp``) and a list of op specs
whose latencies come from a per-GPU profiling database.  Producing it needs a CUDA GPU and the
reference's tracer, so this module supplies the same *quantities* from Megatron-style closed
forms of the model shape, and op latencies from ``flops / (efficiency * peak)`` with seeded
efficiencies.  Everything downstream (the search itself) only ever sees these values through
the accessor methods below, which correspond one-to-one to the reference's evaluation helpers:

=====================  ======================================================================
method                  reference helper (mist/analyzer/batched_module_analyzer.py)
=====================  ======================================================================
``mem_full_states``     ``get_concrete_mem_full_states``            :100-140
``mem_saved``           ``get_concrete_mem_saved``                  :156-183
``mem_peak``            ``get_concrete_mem_peak``                   :186-226
``mem_output``          ``get_concrete_mem_output``                 :229-256
``op_profiles``         ``concrete_node_spec.profile`` per fwd op   :353-366
``grad_accum_profiles`` ``_grad_accumulation_node_specs`` profile   :403-412
``constraint``          ``get_func_constraints_semantic``           :539-578
=====================  ======================================================================

All memory values are MB (bytes / 2**20), all latencies seconds.  Every accessor evaluates in
float64 with a fixed operation order and works on python scalars and numpy arrays alike, so a
table built entry-by-entry and a vectorised evaluation give bit-identical values.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import numpy as np

from .comm_model import gpu_gpu_comm_latency
from .config import MistConfig

MB = float(1 << 20)
KINDS = ("pre", "block", "post")

# Op classes whose efficiencies are drawn from the seed (fwd and bwd separately).
OP_CLASSES = (
    "qkv_gemm",
    "attn_core",
    "attn_softmax",
    "out_gemm",
    "fc1_gemm",
    "fc2_gemm",
    "activation",
    "norm",
    "embedding",
    "lm_head_gemm",
    "xentropy",
    "grad_accum",
)


def draw_op_efficiency(seed: int) -> Dict[str, List[float]]:
    """Efficiencies ~ U(0.5, 0.8) for (fwd, bwd) of every op class, in OP_CLASSES order, from
    ``numpy.random.default_rng(seed + 7)`` (offset so they are independent of the hardware
    draws made from ``seed`` itself)."""
    rng = np.random.default_rng(seed + 7)
    out = {}
    for name in OP_CLASSES:
        f, b = rng.uniform(0.5, 0.8, size=2)
        out[name] = [float(f), float(b)]
    return out


def _f64(x):
    return np.asarray(x, dtype=np.float64)


class LayerTables:
    """Closed-form provider of the per-layer memory / latency quantities for one model plan."""

    def __init__(self, config: MistConfig):
        model, training = config.model, config.training
        syn = dict(getattr(config, "synthetic", None) or {})
        self.h = float(model.hidden_size)
        self.heads = float(model.num_attention_heads)
        kv = getattr(model, "num_heads_kv", None)
        self.kv_heads = float(kv if kv else model.num_attention_heads)
        inter = getattr(model, "intermediate_size", None)
        self.ffn = float(inter if inter else 4 * model.hidden_size)
        self.vocab = float(getattr(model, "vocab_size", None) or training.vocab_size)
        self.s = float(training.max_sequence_length)
        self.flash = bool(model.use_flash_attn)
        mlp_type = str(getattr(model, "mlp_type", "mlp")).lower()
        self.gated = mlp_type in ("gated_mlp", "swiglu", "glu")
        norm = str(getattr(model, "normalization", "layernorm")).lower()
        self.norm_params = self.h if norm == "rmsnorm" else 2.0 * self.h
        pos = str(getattr(model, "position_embedding_type", "absolute")).lower()
        self.abs_pos = pos == "absolute"
        self.tied = bool(getattr(model, "tie_word_embeddings", False))
        # Optimizer-state multiplier, mist/analyzer/info.py:199-212.
        half = str(training.params_dtype) in ("float16", "bfloat16", "half", "fp16", "bf16")
        opt32 = str(training.optimizer_dtype) in ("float32", "fp32", "float")
        opt_name = str(training.optimizer_name).lower()
        if half and opt32:
            if opt_name in ("adam", "adamw"):
                self.opt_mult = 6.0
            elif opt_name == "sgd":
                self.opt_mult = 4.0
            else:
                raise ValueError(f"Unsupported optimizer name: {opt_name}")
        else:
            self.opt_mult = 2.0
        self.bytes_per_param = 2.0 if half else 4.0
        self.peak_flops = float(syn.get("peak_tflops", 312.0)) * 1e12
        self.hbm_bw = float(syn.get("hbm_gbps", 1555.0)) * 1e9
        eff = syn.get("op_efficiency")
        if eff is None:
            eff = draw_op_efficiency(int(syn.get("seed", 0)))
        self.eff = {k: (float(v[0]), float(v[1])) for k, v in eff.items()}
        for name in OP_CLASSES:
            assert name in self.eff, f"synthetic.op_efficiency lacks '{name}'"
        self.gpu_gpu_comm_params = tuple(config.hardware.gpu_gpu_comm_params)
        # scalar look-ups recur for every (G, mesh) group of a plan
        self._params_cache: Dict[tuple, np.ndarray] = {}
        self._act_cache: Dict[tuple, tuple] = {}

    # ------------------------------------------------------------------ parameters
    def _params(self, kind: str, tp):
        """Parameter count of one layer of ``kind`` on one tensor-parallel rank."""
        if np.ndim(tp) == 0:
            key = (kind, float(tp))
            hit = self._params_cache.get(key)
            if hit is None:
                hit = self._params_cache[key] = self._params_uncached(kind, tp)
            return hit
        return self._params_uncached(kind, tp)

    def _params_uncached(self, kind: str, tp):
        tp = _f64(tp)
        h = self.h
        if kind == "block":
            kvh = h * self.kv_heads / self.heads
            attn = h * (h + 2.0 * kvh) + h * h
            mlp = (3.0 if self.gated else 2.0) * h * self.ffn
            return (attn + mlp) / tp + 2.0 * self.norm_params
        if kind == "pre":
            p = self.vocab * h / tp
            if self.abs_pos:
                p = p + self.s * h
            return p
        if kind == "post":
            p = self.norm_params + 0.0 * tp
            if not self.tied:
                p = p + self.vocab * h / tp
            return p
        raise ValueError(kind)

    # ------------------------------------------------------------------ memory (MB)
    def mem_full_states(self, kind: str, item: str, tp):
        assert item in ("weights", "grads", "opts")
        w = self._params(kind, tp) * self.bytes_per_param / MB
        if item == "opts":
            return w * self.opt_mult
        return w

    def _act_bytes(self, kind: str, b, tp):
        """(saved without checkpointing, extra transient fwd, extra transient bwd) in bytes."""
        if np.ndim(b) == 0 and np.ndim(tp) == 0:
            key = (kind, float(b), float(tp))
            hit = self._act_cache.get(key)
            if hit is None:
                hit = self._act_cache[key] = self._act_bytes_uncached(kind, b, tp)
            return hit
        return self._act_bytes_uncached(kind, b, tp)

    def _act_bytes_uncached(self, kind: str, b, tp):
        b, tp = _f64(b), _f64(tp)
        s, h = self.s, self.h
        bsh = b * s * h
        if kind == "block":
            kvh = h * self.kv_heads / self.heads
            attn = 2.0 * bsh + 2.0 * b * s * (h + 2.0 * kvh) / tp + 2.0 * bsh / tp
            if self.flash:
                attn = attn + 4.0 * b * self.heads / tp * s
                attn_tmp = 0.0 * b
            else:
                attn = attn + 5.0 * b * self.heads / tp * s * s
                attn_tmp = 4.0 * b * self.heads / tp * s * s
            n_fc1 = 3.0 if self.gated else 2.0
            mlp = 2.0 * bsh + 2.0 * n_fc1 * b * s * self.ffn / tp
            saved = attn + mlp + 2.0 * bsh
            tmp_f = attn_tmp + 2.0 * b * s * self.ffn / tp
            tmp_b = attn_tmp + 4.0 * b * s * self.ffn / tp + 4.0 * bsh
            return saved, tmp_f, tmp_b
        if kind == "pre":
            saved = 8.0 * b * s + 0.0 * tp
            return saved, 2.0 * bsh, 2.0 * bsh
        if kind == "post":
            logits = b * s * self.vocab / tp
            saved = 2.0 * bsh + 6.0 * logits
            return saved, 4.0 * logits, 6.0 * logits
        raise ValueError(kind)

    def mem_saved(self, kind: str, ckpt: bool, b, tp):
        if ckpt:
            return 2.0 * _f64(b) * self.s * self.h / MB + 0.0 * _f64(tp)
        return self._act_bytes(kind, b, tp)[0] / MB

    def mem_peak(self, kind: str, phase: str, b, tp, ckpt=None):
        assert phase in ("fwd", "bwd")
        saved, tmp_f, tmp_b = self._act_bytes(kind, b, tp)
        if phase == "fwd":
            if ckpt:
                return (saved + 2.0 * tmp_f) / MB
            return (saved + tmp_f) / MB
        return (saved + tmp_b) / MB

    def mem_output(self, kind: str, b, tp):
        b = _f64(b)
        if kind == "post":
            return 4.0 * b * self.s / MB + 0.0 * _f64(tp)
        return 2.0 * b * self.s * self.h / MB + 0.0 * _f64(tp)

    # ------------------------------------------------------------------ constraints
    def constraint(self, b, tp) -> bool:
        """Integer-shape check of the block layer (attention heads, kv heads, ffn and vocab
        must split evenly over tp), batched_module_analyzer.py:563-578."""
        tp = int(tp)
        for v in (self.heads, self.kv_heads, self.ffn, self.h):
            if int(v) % tp != 0:
                return False
        return True

    # ------------------------------------------------------------------ op latencies
    def _gemm(self, name: str, flops: float) -> Tuple[float, float]:
        ef, eb = self.eff[name]
        return flops / (ef * self.peak_flops), 2.0 * flops / (eb * self.peak_flops)

    def _membound(self, name: str, nbytes: float) -> Tuple[float, float]:
        ef, eb = self.eff[name]
        return nbytes / (ef * self.hbm_bw), 2.0 * nbytes / (eb * self.hbm_bw)

    def _tp_all_reduce(self, nbytes: float, inter_size, intra_size) -> float:
        return gpu_gpu_comm_latency(
            "all_reduce",
            nbytes / float(1 << 30),
            inter_size=inter_size,
            intra_size=intra_size,
            gpu_gpu_comm_params=self.gpu_gpu_comm_params,
        )

    def op_profiles(self, kind: str, b, tp, inter_size, intra_size):
        """List of ``(fwd, bwd, extra_fwd, extra_bwd)`` per forward op of one layer, the raw
        values the reference obtains from ``concrete_node_spec.profile`` before its clamps."""
        b, tp = float(int(b)), float(int(tp))
        s, h = self.s, self.h
        act = 2.0 * b * s * h  # bytes of one (b, s, h) half-precision activation
        ar = self._tp_all_reduce(act, inter_size, intra_size) if tp > 1 else 0.0
        ops = []
        if kind == "block":
            kvh = h * self.kv_heads / self.heads
            ops.append(self._membound("norm", 2.0 * act) + (0.0, 0.0))
            ops.append(self._gemm("qkv_gemm", 2.0 * b * s * h * (h + 2.0 * kvh) / tp) + (0.0, ar))
            if self.flash:
                ops.append(self._gemm("attn_core", 4.0 * b * s * s * h / tp) + (0.0, 0.0))
            else:
                ops.append(self._gemm("attn_core", 2.0 * b * s * s * h / tp) + (0.0, 0.0))
                ops.append(
                    self._membound("attn_softmax", 6.0 * b * self.heads / tp * s * s) + (0.0, 0.0)
                )
                ops.append(self._gemm("attn_core", 2.0 * b * s * s * h / tp) + (0.0, 0.0))
            ops.append(self._gemm("out_gemm", 2.0 * b * s * h * h / tp) + (ar, 0.0))
            ops.append(self._membound("norm", 2.0 * act) + (0.0, 0.0))
            n_fc1 = 2.0 if self.gated else 1.0
            ops.append(self._gemm("fc1_gemm", 2.0 * n_fc1 * b * s * h * self.ffn / tp) + (0.0, ar))
            ops.append(
                self._membound("activation", (2.0 + n_fc1) * 2.0 * b * s * self.ffn / tp)
                + (0.0, 0.0)
            )
            ops.append(self._gemm("fc2_gemm", 2.0 * b * s * self.ffn * h / tp) + (ar, 0.0))
        elif kind == "pre":
            ops.append(self._membound("embedding", 3.0 * act) + (ar, 0.0))
        elif kind == "post":
            ops.append(self._membound("norm", 2.0 * act) + (0.0, 0.0))
            ops.append(self._gemm("lm_head_gemm", 2.0 * b * s * h * self.vocab / tp) + (0.0, ar))
            xe = self._tp_all_reduce(3.0 * 4.0 * b * s, inter_size, intra_size) if tp > 1 else 0.0
            ops.append(self._membound("xentropy", 10.0 * b * s * self.vocab / tp) + (xe, 0.0))
        else:
            raise ValueError(kind)
        return ops

    def grad_accum_profiles(self, kind: str, b, tp) -> List[float]:
        """Latency of accumulating one micro-batch's gradients into the main gradients."""
        nbytes = 3.0 * float(self._params(kind, float(int(tp)))) * self.bytes_per_param
        return [nbytes / (self.eff["grad_accum"][0] * self.hbm_bw)]
