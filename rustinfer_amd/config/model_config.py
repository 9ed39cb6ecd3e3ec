"""Typed model configuration read from a model folder's ``config.json``.

Every size and constant of the model comes from here; no part of the engine
carries a size of its own.  Keys, defaults and meanings follow the reference's
``HfConfig`` / ``build_load_config`` (crates/infer-worker/src/bin/worker_main.rs:55-181,
:389-449) with the differences listed in ``LlamaConfig``.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, asdict
from typing import Any, Dict, List, Optional


class ConfigError(ValueError):
    """A config.json (or launch file) that cannot be used."""


def _require(d: Dict[str, Any], key: str, typ, where: str):
    if key not in d or d[key] is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return _typed(d[key], key, typ, where)


def _typed(value, key: str, typ, where: str):
    if typ is int:
        if isinstance(value, bool) or not isinstance(value, int):
            raise ConfigError(f"{where}: '{key}' must be an integer, got {value!r}")
        return int(value)
    if typ is float:
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"{where}: '{key}' must be a number, got {value!r}")
        return float(value)
    if typ is bool:
        if not isinstance(value, bool):
            raise ConfigError(f"{where}: '{key}' must be true or false, got {value!r}")
        return value
    if typ is str:
        if not isinstance(value, str):
            raise ConfigError(f"{where}: '{key}' must be a string, got {value!r}")
        return value
    raise TypeError(typ)


@dataclass(frozen=True)
class RopeScaling:
    """``rope_scaling`` of config.json.  Only ``rope_type == "llama3"`` rescales
    (crates/infer-worker/src/bin/worker_main.rs:393-404); the reference silently
    ignores other types, this engine refuses them."""

    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str) -> Optional["RopeScaling"]:
        rope_type = d.get("rope_type", d.get("type"))
        if rope_type is None:
            raise ConfigError(f"{where}: rope_scaling has no 'rope_type'")
        if rope_type == "default":
            return None
        if rope_type != "llama3":
            raise ConfigError(
                f"{where}: rope_scaling.rope_type {rope_type!r} is not supported "
                f"(supported: 'default', 'llama3')")
        w = where + ".rope_scaling"
        rs = RopeScaling(
            rope_type="llama3",
            factor=_require(d, "factor", float, w),
            low_freq_factor=_require(d, "low_freq_factor", float, w),
            high_freq_factor=_require(d, "high_freq_factor", float, w),
            original_max_position_embeddings=_require(
                d, "original_max_position_embeddings", int, w),
        )
        if rs.factor <= 0:
            raise ConfigError(f"{w}: factor must be > 0")
        if rs.high_freq_factor <= rs.low_freq_factor:
            raise ConfigError(f"{w}: high_freq_factor must exceed low_freq_factor")
        if rs.low_freq_factor <= 0 or rs.original_max_position_embeddings <= 0:
            raise ConfigError(f"{w}: low_freq_factor and original_max_position_embeddings must be > 0")
        return rs


class ModelConfig:
    """Base of every architecture's typed configuration.

    A subclass is a dataclass with ``from_dict`` (parse + validate config.json)
    and ``to_dict`` (what the random-weights mode writes back as config.json).
    """

    architecture: str = ""

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError


DEFAULT_EOS_IDS = (128001, 128008, 128009)  # worker_main.rs:327-373 fallback
MAX_HEAD_DIM = 256      # the attention kernel that takes any head size keeps one head's features in a block of this many lanes


@dataclass(frozen=True)
class LlamaConfig(ModelConfig):
    """Dense Llama-3 decoder (``LlamaForCausalLM``).

    Differences from the reference's reader: ``tie_word_embeddings`` is read (the
    reference decides by the presence of ``lm_head.weight``,
    crates/infer-worker/src/models/decoder.rs:245-262) and cross-checked by the
    loader; ``hidden_act`` must be ``silu`` and ``attention_bias``/``mlp_bias``
    must be false if present, because this architecture's parts have neither.
    """

    hidden_size: int = 0
    intermediate_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    vocab_size: int = 0
    max_position_embeddings: int = 4096     # worker_main.rs:173-175
    rms_norm_eps: float = 1e-5              # worker_main.rs:176-178
    rope_theta: float = 10000.0             # worker_main.rs:179-181
    rope_scaling: Optional[RopeScaling] = None
    tie_word_embeddings: bool = False
    eos_token_ids: tuple = DEFAULT_EOS_IDS
    architecture: str = "LlamaForCausalLM"

    # derived sizes (reference: ModelDims, crates/infer-worker/src/domain/model.rs:12-54)
    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def qkv_dim(self) -> int:
        return self.q_dim + 2 * self.kv_dim

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "LlamaConfig":
        d = dict(d)
        hidden = _require(d, "hidden_size", int, where)
        heads = _require(d, "num_attention_heads", int, where)
        if heads <= 0:
            raise ConfigError(f"{where}: num_attention_heads must be > 0")
        head_dim = d.get("head_dim")
        if head_dim is None:
            if hidden % heads != 0:
                raise ConfigError(
                    f"{where}: hidden_size {hidden} is not divisible by "
                    f"num_attention_heads {heads} and no head_dim is given")
            head_dim = hidden // heads          # worker_main.rs:390-392
        head_dim = _typed(head_dim, "head_dim", int, where)
        rs = d.get("rope_scaling")
        if rs is not None and not isinstance(rs, dict):
            raise ConfigError(f"{where}: rope_scaling must be an object")
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids = DEFAULT_EOS_IDS
        elif isinstance(eos, list):
            eos_ids = tuple(_typed(e, "eos_token_id", int, where) for e in eos)
        else:
            eos_ids = (_typed(eos, "eos_token_id", int, where),)
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"{where}: hidden_act {act!r} is not supported (only 'silu')")
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key):
                raise ConfigError(f"{where}: {key}=true is not supported by this architecture")
        cfg = cls(
            hidden_size=hidden,
            intermediate_size=_require(d, "intermediate_size", int, where),
            num_hidden_layers=_require(d, "num_hidden_layers", int, where),
            num_attention_heads=heads,
            num_key_value_heads=_require(d, "num_key_value_heads", int, where),
            head_dim=head_dim,
            vocab_size=_require(d, "vocab_size", int, where),
            max_position_embeddings=_typed(d.get("max_position_embeddings", 4096),
                                           "max_position_embeddings", int, where),
            rms_norm_eps=_typed(d.get("rms_norm_eps", 1e-5), "rms_norm_eps", float, where),
            rope_theta=_typed(d.get("rope_theta", 10000.0), "rope_theta", float, where),
            rope_scaling=RopeScaling.from_dict(rs, where) if rs is not None else None,
            tie_word_embeddings=_typed(d.get("tie_word_embeddings", False),
                                       "tie_word_embeddings", bool, where),
            eos_token_ids=eos_ids,
        )
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config") -> None:
        for key in ("hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim",
                    "vocab_size", "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"{where}: {key} must be > 0, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"{where}: num_attention_heads {self.num_attention_heads} is not a multiple "
                f"of num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"{where}: head_dim {self.head_dim} must be even for rotary pairs")
        if self.head_dim > MAX_HEAD_DIM:
            raise ConfigError(f"{where}: head_dim {self.head_dim} exceeds {MAX_HEAD_DIM}, the largest head "
                              f"the attention kernels take")
        if not (self.rms_norm_eps > 0):
            raise ConfigError(f"{where}: rms_norm_eps must be > 0")
        if not (self.rope_theta > 0):
            raise ConfigError(f"{where}: rope_theta must be > 0")

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "eos_token_id": list(self.eos_token_ids),
        }
        if self.rope_scaling is not None:
            d["rope_scaling"] = asdict(self.rope_scaling)
        return d


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path}: no such file")
    with open(path, "r", encoding="utf-8") as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON: {e}") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    # generation_config.json's eos ids win over config.json's (worker_main.rs:327-373)
    gen = os.path.join(model_dir, "generation_config.json")
    if os.path.isfile(gen):
        try:
            with open(gen, "r", encoding="utf-8") as f:
                g = json.load(f)
            if isinstance(g, dict) and g.get("eos_token_id") is not None:
                d["eos_token_id"] = g["eos_token_id"]
        except (OSError, json.JSONDecodeError):
            pass
    return d
