"""Resolved tuning-YAML reader: the fields of the reference configuration that the
configuration-search path consumes, with PyYAML only (hydra / omegaconf are not used).

Mirrors the attribute surface of the reference's ``MistConfig`` (mist/config.py:582-641):
``config.model / .training / .hardware / .tuning / .strategy`` plus fall-through of unknown
attributes to the top level of the raw YAML (mist/config.py:615-619), which is how
``disable_tp_tuning``, ``enable_advanced_opt_in_first_block``, ``fixed_*_ratio`` and
``disable_*_tuning`` reach the search (batched_module_analyzer.py:472,498-503,619-627,749).

Extension over the reference (all optional, defaults reproduce the reference's module
constants, batched_module_analyzer.py:53-55,477-485): ``tuning.search_space`` may carry
``batch_size_candidates``, ``offloading_ratio_candidates``,
``sparse_offloading_ratio_candidates`` and ``zero_flag_choices``; the top-level ``synthetic``
block parameterises the synthetic layer-table provider.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, List, Optional

import yaml

# batched_module_analyzer.py:53-55
BATCH_SIZE_CANDIDATES = (1, 2, 4)
OFFLOADING_RATIO_CANDIDATES = (0.0, 0.25, 0.375, 0.5, 0.625, 0.75, 0.875, 1.0)
SPARSE_OFFLOADING_RATIO_CANDIDATES = (0.0, 0.25, 0.375, 0.5, 0.75, 1.0)
# batched_module_analyzer.py:480-485 (the (0,0,0) entry is commented out at HEAD)
ZERO_FLAG_CHOICES = ((0, 0, 1), (0, 1, 1), (1, 1, 1))

TUNING_GRANULARITIES = (
    "no-pp",
    "uniform-pp",
    "uniform-device-pp",
    "uniform-device-pp-mip",
    "inter-stage",
    "uniform-pp-simple-heuristic-mem-opt",
)
PRE_POST_STRATEGIES = (
    "preset",
    "dp",
    "intra-node-tp-with-ore",
    "intra-node-tp-without-ore",
)


class _Section:
    """Attribute view over one YAML mapping; missing keys raise AttributeError."""

    def __init__(self, data: Optional[Dict[str, Any]]):
        object.__setattr__(self, "_data", dict(data or {}))

    def __getattr__(self, name: str):
        data = object.__getattribute__(self, "_data")
        if name in data:
            return data[name]
        raise AttributeError(name)

    def __setattr__(self, name: str, value: Any):
        object.__getattribute__(self, "_data")[name] = value

    def __contains__(self, name: str) -> bool:
        return name in object.__getattribute__(self, "_data")

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(object.__getattribute__(self, "_data"))


class HardwareConfig(_Section):
    """mist/config.py:273-316. ``memory_capacity`` is scaled by 0.88 on construction."""

    def __init__(self, data: Dict[str, Any]):
        super().__init__(data)
        d = object.__getattribute__(self, "_data")
        for key, size in (
            ("gpu_gpu_comm_params", 32),
            ("cpu_gpu_comm_params", 2),
            ("gpu_cpu_comm_params", 2),
            ("interference_model_params", 28),
        ):
            d[key] = tuple(float(x) for x in d[key])
            assert len(d[key]) == size, f"hardware.{key} must have {size} entries, got {len(d[key])}"
        d["num_nodes"] = int(d["num_nodes"])
        d["num_gpus_per_node"] = int(d["num_gpus_per_node"])
        d["raw_memory_capacity"] = float(d["memory_capacity"])
        d["memory_capacity"] = float(d["memory_capacity"]) * 0.88  # config.py:294


class TuningConfig(_Section):
    """mist/config.py:358-422 (+ the optional ``search_space`` extension)."""

    def __init__(self, data: Dict[str, Any]):
        super().__init__(data)
        d = object.__getattribute__(self, "_data")
        assert d["tuning_granularity"] in TUNING_GRANULARITIES, d["tuning_granularity"]
        d["sample_size"] = int(d.get("sample_size", 1))
        assert d["pre_post_strategy"] in PRE_POST_STRATEGIES, d["pre_post_strategy"]
        arr = d.get("pre_post_strategy_array") or []
        if d["pre_post_strategy"] == "preset":
            assert len(arr) == 10, "pre_post_strategy_array needs 10 entries for 'preset'"
            arr = (
                [int(x) for x in arr[:3]]
                + [bool(x) for x in arr[3:6]]
                + [float(x) for x in arr[6:]]
            )
        d["pre_post_strategy_array"] = list(arr)
        ss = dict(d.get("search_space") or {})
        d["batch_size_candidates"] = tuple(
            int(x) for x in ss.get("batch_size_candidates", BATCH_SIZE_CANDIDATES)
        )
        d["offloading_ratio_candidates"] = tuple(
            float(x) for x in ss.get("offloading_ratio_candidates", OFFLOADING_RATIO_CANDIDATES)
        )
        d["sparse_offloading_ratio_candidates"] = tuple(
            float(x)
            for x in ss.get(
                "sparse_offloading_ratio_candidates", SPARSE_OFFLOADING_RATIO_CANDIDATES
            )
        )
        d["zero_flag_choices"] = tuple(
            tuple(int(v) for v in flags) for flags in ss.get("zero_flag_choices", ZERO_FLAG_CHOICES)
        )
        for flags in d["zero_flag_choices"]:
            assert len(flags) == 3 and all(v in (0, 1) for v in flags), flags
        for key in (
            "zero_2_and_3_enabled",
            "activation_checkpointing_tuning_enabled",
            "state_offloading_enabled",
            "activation_offloading_enabled",
        ):
            d[key] = bool(d.get(key, False))


class StrategyConfig(_Section):
    """mist/config.py:425-492: one strategy (the tuner's output, the analysis path's input)."""

    def __init__(self, data: Dict[str, Any]):
        super().__init__(data)
        d = object.__getattribute__(self, "_data")
        n = len(d["layer_partitions"])
        assert n == len(d["device_assignment"]) == len(d["stage_strategies"]) == len(d["gradient_checkpointing"]), (
            "The length of layer_partitions, device_assignment, stage_strategies, and "
            "gradient_checkpointing should be the same."
        )
        d["num_stages"] = n
        d["layer_partitions"] = [int(x) for x in d["layer_partitions"]]
        d["gradient_checkpointing"] = [int(x) for x in d["gradient_checkpointing"]]
        d["gradient_accumulation_steps"] = int(d["gradient_accumulation_steps"])
        for a in d["device_assignment"]:
            assert len(a) == 2, f"Device assignment should be [num_nodes, num_gpus_per_node], got {a}"
        d["device_assignment"] = [tuple(int(x) for x in a) for a in d["device_assignment"]]

        def row(r):
            assert len(r) == 10, f"a strategy row has 10 entries, got {r}"
            return tuple([int(x) for x in r[:3]] + [bool(x) for x in r[3:6]] + [float(x) for x in r[6:]])

        d["stage_strategies"] = [row(r) for r in d["stage_strategies"]]
        d.setdefault("pre_post_strategy", "heuristic")
        if d["pre_post_strategy"] == "preset":
            assert d.get("pre_post_strategy_array") is not None, "preset needs pre_post_strategy_array"
            d["pre_post_strategy_array"] = list(row(d["pre_post_strategy_array"]))


class MistConfig:
    """Attribute-compatible stand-in for the reference's ``MistConfig``."""

    def __init__(self, raw: Dict[str, Any]):
        raw = copy.deepcopy(raw)
        self._original_config = raw
        self.model = _Section(raw.get("model"))
        training = dict(raw.get("training") or {})
        self.training = _Section(training)
        self.hardware = HardwareConfig(raw["hardware"])
        tuning = raw.get("tuning")
        self.tuning = TuningConfig(tuning) if tuning and tuning.get("enabled", True) else None
        strategy = raw.get("strategy")
        if strategy and strategy.get("enabled", False):
            # a block without partitions only carries the preset pre/post strategy of a tuning run
            self.strategy = StrategyConfig(strategy) if "layer_partitions" in strategy else _Section(strategy)
        else:
            self.strategy = None

    def __getattr__(self, name: str):
        # Only reached when normal lookup fails: fall through to the raw YAML top level
        # (mist/config.py:615-619).
        raw = self.__dict__.get("_original_config", {})
        if name in raw:
            return raw[name]
        raise AttributeError(name)

    @classmethod
    def from_yaml(cls, path: str) -> "MistConfig":
        # the C parser of PyYAML when the installation has it (same documents, ~10x faster)
        loader = getattr(yaml, "CSafeLoader", yaml.SafeLoader)
        with open(path) as f:
            return cls(yaml.load(f, Loader=loader))

    def raw(self) -> Dict[str, Any]:
        return copy.deepcopy(self._original_config)


def frag_factor(config: MistConfig) -> float:
    """batched_module_analyzer.py:1171-1178."""
    frag = 0.0
    if "hidden_size" in config.model and "max_sequence_length" in config.training:
        frag += max(0, config.model.hidden_size / 2048 - 1) * 0.005
        frag += max(0, config.training.max_sequence_length / 2048 - 1) * 0.045
    return frag


def tp_candidates(config: MistConfig) -> List[int]:
    """tune_one_case.py:199-203,370-374."""
    if getattr(config, "disable_tp_tuning", False):
        return [1]
    return [tp for tp in (1, 2, 4, 8) if tp <= config.hardware.num_gpus_per_node]
