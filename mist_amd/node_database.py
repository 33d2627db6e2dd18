"""Reader of the reference's per-GPU operator latency database and the layer latencies built
from it (reference: ``NodeSpec.profile``, mist/node_database/node_spec.py:234-372, and the files
under ``mist/node_database/cache_<device name>/``).

A database folder holds one JSON file per operator, ``<identifier>.json``.  Each file maps
``repr(NodeSpec)`` - the operator with the shapes, dtypes and constants of one concrete call -
to ``{"fwd": [mean, median, std], "bwd": [mean, median, std]}`` in seconds.  The reference
fills a missing entry by benchmarking the operator on the spot; this reader has no operator
implementations to run, so a missing entry is an error that names the key.

``NodeKey`` parses and prints the key grammar (``parse(text).format() == text`` for every key
of the reference's shipped files), ``NodeLatencyDB.profile`` restates the lookup including the
tensor-parallel collective extras, and ``GptNodeTemplate`` / ``DatabaseLayerTables`` turn a
model shape into the keys of its three layer kinds so that a search can run on measured
latencies instead of the synthetic efficiencies of ``LayerTables``.
"""
from __future__ import annotations

import json
import os
from collections import OrderedDict
from typing import Any, Dict, List, Optional, Sequence, Tuple

from .comm_model import gpu_gpu_comm_latency
from .layer_tables import LayerTables

GB = float(1 << 30)  # node_spec.py:44

_DTYPE_BYTES = {
    "torch.float16": 2, "torch.bfloat16": 2, "torch.float32": 4, "torch.float64": 8,
    "torch.int64": 8, "torch.int32": 4, "torch.int16": 2, "torch.int8": 1, "torch.uint8": 1,
    "torch.bool": 1,
}


class TensorSpec:
    """Shape, dtype and requires_grad of a tensor argument (mist/node_database/tensor_spec.py)."""

    __slots__ = ("shape", "dtype", "requires_grad")

    def __init__(self, shape: Sequence[int], dtype: str = "torch.float16", requires_grad: bool = True):
        self.shape, self.dtype, self.requires_grad = tuple(int(d) for d in shape), dtype, bool(requires_grad)

    def nbytes(self) -> int:
        n = _DTYPE_BYTES[self.dtype]
        for d in self.shape:
            n *= d
        return n

    def __eq__(self, other):
        return (isinstance(other, TensorSpec) and self.shape == other.shape
                and self.dtype == other.dtype and self.requires_grad == other.requires_grad)

    def __repr__(self):
        return f"TensorSpec(shape={_fmt(self.shape)}, dtype={self.dtype}, requires_grad={self.requires_grad})"


class ProcessGroup:
    """``MistProcessGroup(world_size=.., rank=..)`` as it appears in a key."""

    __slots__ = ("world_size", "rank")

    def __init__(self, world_size: int, rank: int = 0):
        self.world_size, self.rank = int(world_size), int(rank)

    def size(self) -> int:
        return self.world_size

    def __eq__(self, other):
        return isinstance(other, ProcessGroup) and (self.world_size, self.rank) == (other.world_size, other.rank)

    def __repr__(self):
        return f"MistProcessGroup(world_size={self.world_size}, rank={self.rank})"


class Name:
    """A dotted name printed without quotes (``torch.float16``, ``torch.preserve_format``)."""

    __slots__ = ("text",)

    def __init__(self, text: str):
        self.text = text

    def __eq__(self, other):
        return isinstance(other, Name) and self.text == other.text

    def __repr__(self):
        return self.text


def _fmt(value: Any) -> str:
    """Python's repr for the value kinds a key holds."""
    if isinstance(value, tuple):
        inner = ", ".join(_fmt(v) for v in value)
        return f"({inner},)" if len(value) == 1 else f"({inner})"
    if isinstance(value, list):
        return "[" + ", ".join(_fmt(v) for v in value) + "]"
    if isinstance(value, dict):
        return "{" + ", ".join(f"{_fmt(k)}: {_fmt(v)}" for k, v in value.items()) + "}"
    return repr(value)


class _Parser:
    """Recursive descent over the repr grammar of a key."""

    def __init__(self, text: str):
        self.text, self.at = text, 0

    def fail(self, what: str):
        raise ValueError(f"{what} at offset {self.at}: ...{self.text[self.at:self.at + 40]!r}")

    def peek(self, token: str) -> bool:
        return self.text.startswith(token, self.at)

    def take(self, token: str) -> None:
        if not self.peek(token):
            self.fail(f"expected {token!r}")
        self.at += len(token)

    def space(self) -> None:
        while self.at < len(self.text) and self.text[self.at] == " ":
            self.at += 1

    def word(self) -> str:
        start = self.at
        while self.at < len(self.text) and (self.text[self.at].isalnum() or self.text[self.at] in "._+-"):
            self.at += 1
        if start == self.at:
            self.fail("expected a name or number")
        return self.text[start:self.at]

    def value(self) -> Any:
        self.space()
        if self.peek("TensorSpec("):
            self.take("TensorSpec(shape=")
            shape = self.value()
            self.take(", dtype=")
            dtype = self.word()
            self.take(", requires_grad=")
            grad = self.word()
            self.take(")")
            return TensorSpec(shape, dtype, grad == "True")
        if self.peek("MistProcessGroup("):
            self.take("MistProcessGroup(world_size=")
            world = int(self.word())
            self.take(", rank=")
            rank = int(self.word())
            self.take(")")
            return ProcessGroup(world, rank)
        if self.peek("'") or self.peek('"'):
            quote = self.text[self.at]
            end = self.text.index(quote, self.at + 1)
            out = self.text[self.at + 1:end]
            self.at = end + 1
            return out
        if self.peek("("):
            return tuple(self.sequence("(", ")"))
        if self.peek("["):
            return list(self.sequence("[", "]"))
        if self.peek("{"):
            return self.mapping()
        token = self.word()
        if token in ("None", "True", "False"):
            return {"None": None, "True": True, "False": False}[token]
        try:
            return int(token)
        except ValueError:
            pass
        try:
            return float(token)
        except ValueError:
            return Name(token)

    def sequence(self, opening: str, closing: str) -> List[Any]:
        self.take(opening)
        out = []
        while True:
            self.space()
            if self.peek(closing):
                self.take(closing)
                return out
            out.append(self.value())
            self.space()
            if self.peek(","):
                self.take(",")

    def mapping(self) -> "OrderedDict[Any, Any]":
        self.take("{")
        out: "OrderedDict[Any, Any]" = OrderedDict()
        while True:
            self.space()
            if self.peek("}"):
                self.take("}")
                return out
            key = self.value()
            self.take(": ")
            out[key] = self.value()
            self.space()
            if self.peek(","):
                self.take(",")


class NodeKey:
    """One database key: the operator (``kind`` = FunctionSpec / MethodDescriptorSpec /
    NNModuleSpec, ``identifier`` = its dotted name, for modules also ``constants``,
    ``param_requires_grad`` and ``param_dtype``, node_spec.py:537-620) and the arguments of the
    call in signature order (``repr(NodeSpec)``, node_spec.py:475-476)."""

    def __init__(self, kind: str, identifier: str, arguments: "OrderedDict[str, Any]",
                 constants: Optional[dict] = None, param_requires_grad: Optional[dict] = None,
                 param_dtype: Optional[dict] = None):
        self.kind, self.identifier, self.arguments = kind, identifier, OrderedDict(arguments)
        self.constants, self.param_requires_grad, self.param_dtype = constants, param_requires_grad, param_dtype

    @classmethod
    def function(cls, identifier: str, **arguments) -> "NodeKey":
        return cls("FunctionSpec", identifier, OrderedDict(arguments))

    @classmethod
    def method(cls, identifier: str, **arguments) -> "NodeKey":
        return cls("MethodDescriptorSpec", identifier, OrderedDict(arguments))

    @classmethod
    def module(cls, identifier: str, constants: dict, param_requires_grad: dict, param_dtype: dict,
               **arguments) -> "NodeKey":
        return cls("NNModuleSpec", identifier, OrderedDict(arguments), OrderedDict(constants),
                   OrderedDict(param_requires_grad), OrderedDict(param_dtype))

    @classmethod
    def parse(cls, text: str) -> "NodeKey":
        p = _Parser(text)
        p.take("NodeSpec(target_spec=")
        kind = p.word()
        p.take("(")
        identifier = p.word()
        constants = grads = dtypes = None
        if p.peek(" [constants] "):
            p.take(" [constants] ")
            constants = p.mapping()
            p.take(", [requires_grad] ")
            grads = p.mapping()
            p.take(", [dtype] ")
            dtypes = p.mapping()
        p.take("), bounded_signature=")
        arguments = p.mapping()
        p.take(")")
        if p.at != len(text):
            p.fail("trailing text")
        return cls(kind, identifier, arguments, constants, grads, dtypes)

    def target(self) -> str:
        if self.constants is None:
            return f"{self.kind}({self.identifier})"
        return (f"{self.kind}({self.identifier} [constants] {_fmt(self.constants)}, "
                f"[requires_grad] {_fmt(self.param_requires_grad)}, [dtype] {_fmt(self.param_dtype)})")

    def format(self) -> str:
        return f"NodeSpec(target_spec={self.target()}, bounded_signature={_fmt(self.arguments)})"

    __repr__ = format

    def file_name(self) -> str:
        return self.identifier + ".json"  # node_spec.py:240-244

    def process_group(self) -> Optional[ProcessGroup]:
        found = [v for v in self.arguments.values() if isinstance(v, ProcessGroup)]
        if self.constants:
            found += [v for v in self.constants.values() if isinstance(v, ProcessGroup)]
        if len(found) > 1:
            raise ValueError(f"more than one process group in {self.format()}")
        return found[0] if found else None


Latency = Tuple[float, float, float]  # mean, median, std


class NodeLatencyDB:
    """The files of one ``cache_<device name>`` folder."""

    def __init__(self, folder: str):
        if not os.path.isdir(folder):
            raise FileNotFoundError(f"operator latency database folder not found: {folder}")
        self.folder = folder
        self._files: Dict[str, Dict[str, dict]] = {}

    def identifiers(self) -> List[str]:
        return sorted(f[:-5] for f in os.listdir(self.folder) if f.endswith(".json"))

    def entries(self, identifier: str) -> Dict[str, dict]:
        """All entries of one operator file (``{}`` if the file does not exist)."""
        if identifier not in self._files:
            path = os.path.join(self.folder, identifier + ".json")
            data = {}
            if os.path.exists(path):
                with open(path) as f:
                    data = json.load(f)
            self._files[identifier] = data
        return self._files[identifier]

    def lookup(self, key: NodeKey) -> Tuple[Latency, Latency]:
        """``(fwd, bwd)`` triples of a key (node_spec.py:322-335)."""
        entry = self.entries(key.identifier).get(key.format())
        if entry is None:
            raise KeyError(
                f"no entry in {os.path.join(self.folder, key.file_name())} for {key.format()} "
                f"(the reference would benchmark the operator here)")
        return tuple(entry["fwd"]), tuple(entry["bwd"])

    def profile(self, key: NodeKey, inter_size=None, intra_size=None,
                gpu_gpu_comm_params: Sequence[float] = ()):
        """``NodeSpec.profile`` (node_spec.py:234-372): ``(fwd, bwd, extra_fwd, extra_bwd)`` with
        fwd / bwd the (mean, median, std) triples of the database and the extras the modelled
        latency of the collectives a tensor-parallel operator issues."""
        zeros = (0.0, 0.0, 0.0)
        extra_fwd = extra_bwd = 0.0
        group = key.process_group()
        if group is not None:
            first = next(iter(key.arguments.values()))
            direct = False
            if key.identifier.startswith("mist.distributed.op"):
                direct = True
                fwd_op = key.identifier.split(".")[-1]
                bwd_op = _COUNTERPART[fwd_op]
                gbytes = first.nbytes() / GB
            elif key.identifier == "mist.modules.fused_dense.fused_dense_func":
                fwd_op = "all_gather" if key.arguments["sequence_parallel"] else "none"
                bwd_op = "all_reduce"
                gbytes = first.nbytes() / GB
            elif key.identifier == "mist.modules.losses._vocab_parallel_cross_entropy":
                fwd_op, bwd_op = "all_reduce", "none"
                if len(first.shape) != 2:
                    raise ValueError(f"logits of {key.format()} are not 2-d")
                gbytes = 3 * first.shape[0] * _DTYPE_BYTES[first.dtype] / GB
            else:
                raise NotImplementedError(f"no communication model registered for {key.format()}")
            if group.size() != 1:
                if inter_size is None or intra_size is None or group.size() != inter_size * intra_size:
                    raise ValueError(
                        f"group of {group.size()} ranks needs inter_size * intra_size of that size, "
                        f"got {inter_size} x {intra_size}")
                extra_fwd = gpu_gpu_comm_latency(fwd_op, gbytes, inter_size, intra_size, gpu_gpu_comm_params)
                extra_bwd = gpu_gpu_comm_latency(bwd_op, gbytes, inter_size, intra_size, gpu_gpu_comm_params)
            if direct:  # a collective has no kernel of its own to time
                return zeros, zeros, extra_fwd, extra_bwd
        fwd, bwd = self.lookup(key)
        return fwd, bwd, extra_fwd, extra_bwd


_COUNTERPART = {"reduce_scatter": "all_gather", "all_gather": "reduce_scatter",
                "all_reduce": "none", "none": "all_reduce"}  # node_spec.py:188-200


class GptNodeTemplate:
    """Operator calls of the three layer kinds of the reference's decoder models
    (mist/models/gpt.py, llama.py with mist/modules/mha.py, mlp.py, fused_dense.py, embedding.py,
    losses.py) for per-device batch ``b`` and tensor-parallel size ``tp``.

    ``flash``: the attention core is one ``flash_attn_qkvpacked_func`` call, or - flash attention
    off, as in the reference's kick-the-tires plan - the calls of ``SelfAttention.forward_fused_softmax``
    (mist/modules/mha.py:316-391): unbind, the transposes of q / k / v and of the context,
    ``torch.baddbmm`` into the score buffer, the fused causal softmax, the (identity) attention
    dropout and ``torch.bmm``.  ``gated``: the MLP is ``ParallelGatedMlp`` with SiLU
    (mist/modules/mlp.py:67-128: one projection to 2 x ffn, chunk, swiglu, projection back) instead
    of ``ParallelMLP`` with GELU; ``norm`` "rmsnorm" swaps the norm function (mist/modules/rms_norm.py).

    The reference obtains these lists by tracing the model; this template is written from the
    module code and checked against the reference's shipped database, which holds an entry for
    every call of the GELU / LayerNorm model listed here at tp = 1, with and without flash
    attention (the calls the tracer recorded): how often a call occurs in a layer is this
    module's reading of the code, not something the database can confirm.  The shipped database
    has no gated or RMS-norm model: the operator names of that path (chunk, swiglu, rms_norm)
    are read from the module code alone.
    """

    def __init__(self, hidden: int, heads: int, seq_len: int, vocab: int, ffn: Optional[int] = None,
                 dtype: str = "torch.float16", layer_norm_epsilon: float = 1e-06, flash: bool = True,
                 gated: bool = False, norm: str = "layernorm"):
        self.h, self.heads, self.s, self.v = int(hidden), int(heads), int(seq_len), int(vocab)
        self.ffn = int(ffn) if ffn else 4 * self.h
        self.dtype, self.eps = dtype, layer_norm_epsilon
        self.flash, self.gated = bool(flash), bool(gated)
        if norm not in ("layernorm", "rmsnorm"):
            raise ValueError(f"norm: {norm}")
        self.norm = norm

    def _t(self, *shape, grad=True, dtype=None) -> TensorSpec:
        return TensorSpec(shape, dtype or self.dtype, grad)

    def _dense(self, b, in_features, out_features, group) -> NodeKey:
        return NodeKey.function(
            "mist.modules.fused_dense.fused_dense_func",
            x=self._t(b, self.s, in_features), weight=self._t(out_features, in_features), bias=None,
            return_residual=False, process_group=group, sequence_parallel=False)

    def _norm(self, b) -> NodeKey:
        if self.norm == "rmsnorm":
            return NodeKey.function(
                "mist.modules.rms_norm.rms_norm", x=self._t(b, self.s, self.h),
                weight=self._t(self.h), epsilon=self.eps)
        return NodeKey.function(
            "mist.modules.layer_norm.layer_norm", x=self._t(b, self.s, self.h),
            weight=self._t(self.h), bias=self._t(self.h), epsilon=self.eps)

    def _attention_core(self, b, tp) -> List[NodeKey]:
        """The calls between the qkv projection and the output projection."""
        s, heads, d = self.s, self.heads // tp, self.h // self.heads
        if self.flash:
            return [NodeKey.function(
                "mist.modules.flash_attn.flash_attn_qkvpacked_func",
                qkv=self._t(b, s, 3, heads, d), dropout_p=0.0, softmax_scale=d ** -0.5, causal=True,
                window_size=(-1, -1), return_attn_probs=False)]
        transpose = lambda shape, d0, d1: NodeKey.method(
            "torch._C._TensorBase.transpose", input=self._t(*shape), dim0=d0, dim1=d1)
        bh = b * heads
        return [
            NodeKey.method("torch._C._TensorBase.unbind", input=self._t(b, s, 3, heads, d), dim=2),
            transpose((b, s, heads, d), 1, 2),   # q -> (b, heads, t, d)
            transpose((b, s, heads, d), 1, 2),   # k -> (b, heads, s, d)
            transpose((b, heads, s, d), 2, 3),   # k -> (b, heads, d, s)
            NodeKey.function(
                "torch.baddbmm", input=self._t(bh, s, s, grad=False), batch1=self._t(bh, s, d),
                batch2=self._t(bh, d, s), alpha=1, beta=0.0, out=None),
            NodeKey.function(
                "mist.modules.fused_softmax.scaled_upper_triang_masked_softmax_fn",
                inputs=self._t(bh, s, s), scale=d ** -0.5),
            NodeKey.module("torch.nn.modules.linear.Identity", {}, {}, {}, input=self._t(b, heads, s, s)),
            transpose((b, s, heads, d), 1, 2),   # v -> (b, heads, s, d)
            NodeKey.function("torch.bmm", input=self._t(bh, s, s), mat2=self._t(bh, s, d), out=None),
            transpose((b, heads, s, d), 1, 2),   # context -> (b, t, heads, d)
        ]

    def _mlp(self, b, tp, group) -> List[NodeKey]:
        s, f = self.s, self.ffn // tp
        if not self.gated:
            return [self._dense(b, self.h, f, group),
                    NodeKey.function("torch._C._nn.gelu", input=self._t(b, s, f), approximate="tanh"),
                    self._dense(b, f, self.h, None)]
        return [self._dense(b, self.h, 2 * f, group),
                NodeKey.method("torch._C._TensorBase.chunk", input=self._t(b, s, 2 * f), chunks=2, dim=-1),
                NodeKey.function("mist.modules.activations.swiglu", x=self._t(b, s, f), y=self._t(b, s, f)),
                self._dense(b, f, self.h, None)]

    def _dropout(self, b) -> NodeKey:
        return NodeKey.module("torch.nn.modules.dropout.Dropout", {"p": 0.0, "inplace": False}, {}, {},
                              input=self._t(b, self.s, self.h))

    def _residual_add(self, b) -> NodeKey:
        return NodeKey.function("_operator.add", a=self._t(b, self.s, self.h), b=self._t(b, self.s, self.h))

    def _all_reduce(self, b, group) -> NodeKey:
        return NodeKey.function("mist.distributed.op.all_reduce", input_=self._t(b, self.s, self.h),
                                process_group=group)

    def nodes(self, kind: str, b: int, tp: int) -> List[NodeKey]:
        b, tp = int(b), int(tp)
        h, s = self.h, self.s
        if h % tp or self.heads % tp or self.ffn % tp or self.v % tp:
            raise ValueError(f"tensor-parallel size {tp} does not divide the model shape")
        group = ProcessGroup(tp, 0)
        head_dim = h // self.heads
        if kind == "pre":
            return [NodeKey.module(
                "mist.modules.embedding.VocabParallelEmbedding",
                OrderedDict(num_embeddings=self.v // tp, embedding_dim=h, padding_idx=None, max_norm=None,
                            norm_type=2.0, scale_grad_by_freq=False, sparse=False,
                            process_group=None if tp == 1 else group),
                {"weight": True}, {"weight": Name(self.dtype)},
                input=self._t(b, s, grad=False, dtype="torch.int64"))]
        if kind == "block":
            out = [self._dropout(b), self._residual_add(b), self._norm(b),
                   self._dense(b, h, 3 * h // tp, group)]
            out += self._attention_core(b, tp)
            out.append(self._dense(b, h // tp, h, None))
            if tp > 1:
                out.append(self._all_reduce(b, group))
            out += [self._dropout(b), self._residual_add(b), self._norm(b)]
            out += self._mlp(b, tp, group)
            if tp > 1:
                out.append(self._all_reduce(b, group))
            return out
        if kind == "post":
            tokens = b * s
            return [self._dropout(b), self._residual_add(b), self._norm(b),
                    self._dense(b, h, self.v // tp, group),
                    NodeKey.method("torch._C._TensorBase.half", self=self._t(b, s, self.v // tp),
                                   memory_format=Name("torch.preserve_format")),
                    NodeKey.function(
                        "mist.modules.losses._vocab_parallel_cross_entropy",
                        vocab_parallel_logits=self._t(tokens, self.v // tp),
                        target=self._t(tokens, grad=False, dtype="torch.int64"), process_group=group,
                        label_smoothing=0.0),
                    NodeKey.method("torch._C._TensorBase.mean", input=self._t(tokens), dim=None)]
        raise ValueError(kind)

    def params(self, kind: str, tp: int) -> int:
        """Elements of the layer's flat parameter (the operand of the gradient-accumulation add)."""
        h, tp = self.h, int(tp)
        if kind == "pre":
            return self.v // tp * h
        if kind == "block":
            n_fc1 = 2 if self.gated else 1
            norm_params = 2 * h if self.norm == "rmsnorm" else 4 * h
            return (3 * h * h + h * h + (n_fc1 + 1) * h * self.ffn) // tp + norm_params
        if kind == "post":
            # the shipped database holds the add of vocab * hidden elements only: the output
            # projection, without the final norm's 2 * hidden parameters
            return self.v // tp * h
        raise ValueError(kind)

    def grad_accum_nodes(self, kind: str, tp: int) -> List[NodeKey]:
        n = self.params(kind, tp)
        return [NodeKey.function("torch.add", input=self._t(n), other=self._t(n), out=None)]


class DatabaseLayerTables(LayerTables):
    """``LayerTables`` whose operator latencies come from a database folder
    (``synthetic.node_database`` of the plan) instead of seeded efficiencies; the memory
    quantities stay the closed forms of the base class."""

    def __init__(self, config, folder: Optional[str] = None):
        super().__init__(config)
        syn = dict(getattr(config, "synthetic", None) or {})
        folder = folder or syn.get("node_database")
        if not folder:
            raise ValueError("DatabaseLayerTables needs a database folder (synthetic.node_database)")
        if self.kv_heads != self.heads:
            raise NotImplementedError(
                "the operator template covers blocks whose key / value heads equal the query heads "
                "(the packed qkv projection of mist/modules/mha.py:863-891)")
        self.db = NodeLatencyDB(folder)
        dtype = {"float16": "torch.float16", "half": "torch.float16", "fp16": "torch.float16",
                 "bfloat16": "torch.bfloat16", "bf16": "torch.bfloat16"}.get(
                     str(config.training.params_dtype), "torch.float32")
        model = config.model
        norm = "rmsnorm" if str(getattr(model, "normalization", "layernorm")).lower().startswith("rms") else "layernorm"
        self.template = GptNodeTemplate(int(self.h), int(self.heads), int(self.s), int(self.vocab),
                                        int(self.ffn), dtype, flash=bool(self.flash), gated=bool(self.gated),
                                        norm=norm)

    def op_profiles(self, kind: str, b, tp, inter_size, intra_size):
        out = []
        for key in self.template.nodes(kind, int(b), int(tp)):
            fwd, bwd, extra_fwd, extra_bwd = self.db.profile(
                key, inter_size, intra_size, self.gpu_gpu_comm_params)
            out.append((fwd[0], bwd[0], extra_fwd, extra_bwd))
        return out

    def grad_accum_profiles(self, kind: str, b, tp) -> List[float]:
        return [self.db.profile(key)[0][0] for key in self.template.grad_accum_nodes(kind, int(tp))]


def layer_tables_for(config) -> LayerTables:
    """The layer-table provider a plan asks for: database-driven latencies when its
    ``synthetic.node_database`` names a folder, the seeded closed forms otherwise."""
    syn = dict(getattr(config, "synthetic", None) or {})
    if syn.get("node_database"):
        return DatabaseLayerTables(config)
    return LayerTables(config)

