"""Typed model configuration read from a model folder's ``config.json``.

The reference engine hard-codes every model dimension as a compile-time constant
(``base/src/config.h:41-65``, with a TODO at ``:42`` to read ``config.json``).  Here nothing about
the model is fixed in code: every size and constant is a field of :class:`LlamaConfig`, filled
from the keys a Llama ``config.json`` carries.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, asdict
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A ``config.json`` that cannot describe a model this engine can run."""


def _require(d: Mapping[str, Any], key: str, kind):
    if key not in d or d[key] is None:
        raise ConfigError(f"config.json: required key '{key}' is missing")
    v = d[key]
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"config.json: '{key}' must be an integer, got {v!r}")
        return v
    if kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"config.json: '{key}' must be a number, got {v!r}")
        return float(v)
    return v


@dataclass(frozen=True)
class RopeScaling:
    """``rope_scaling`` section; the reference's constants are ``base/src/config.h:60-65``."""

    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    @staticmethod
    def from_dict(d: Mapping[str, Any]) -> "RopeScaling":
        rope_type = d.get("rope_type", d.get("type"))
        if rope_type != "llama3":
            raise ConfigError(
                f"config.json: rope_scaling.rope_type {rope_type!r} is not supported "
                f"(supported: 'llama3', or no rope_scaling at all)")
        rs = RopeScaling(
            rope_type="llama3",
            factor=_require(d, "factor", float),
            low_freq_factor=_require(d, "low_freq_factor", float),
            high_freq_factor=_require(d, "high_freq_factor", float),
            original_max_position_embeddings=_require(d, "original_max_position_embeddings", int),
        )
        if rs.factor <= 0 or rs.original_max_position_embeddings <= 0:
            raise ConfigError("config.json: rope_scaling.factor and "
                              "original_max_position_embeddings must be positive")
        if rs.high_freq_factor == rs.low_freq_factor:
            raise ConfigError("config.json: rope_scaling.high_freq_factor must differ from "
                              "low_freq_factor")
        return rs


@dataclass(frozen=True)
class LlamaConfig:
    """The keys of a Llama ``config.json`` (dense GQA decoder, RMSNorm, RoPE, SwiGLU)."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    rope_scaling: Optional[RopeScaling] = None
    tie_word_embeddings: bool = False
    hidden_act: str = "silu"
    attention_bias: bool = False
    mlp_bias: bool = False
    torch_dtype: str = "bfloat16"
    eos_token_id: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    architectures: Tuple[str, ...] = ("LlamaForCausalLM",)
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False)

    # ------------------------------------------------------------------ construction
    @staticmethod
    def from_dict(d: Mapping[str, Any]) -> "LlamaConfig":
        hidden = _require(d, "hidden_size", int)
        heads = _require(d, "num_attention_heads", int)
        if heads <= 0 or hidden <= 0:
            raise ConfigError("config.json: hidden_size and num_attention_heads must be positive")
        kv_heads = d.get("num_key_value_heads")
        if kv_heads is None:
            kv_heads = heads
        head_dim = d.get("head_dim")
        if head_dim is None:
            if hidden % heads != 0:
                raise ConfigError(
                    f"config.json: hidden_size {hidden} is not a multiple of num_attention_heads "
                    f"{heads} and no head_dim is given")
            head_dim = hidden // heads
        if not isinstance(kv_heads, int) or kv_heads <= 0 or heads % kv_heads != 0:
            raise ConfigError(
                f"config.json: num_attention_heads {heads} is not a multiple of "
                f"num_key_value_heads {kv_heads}")
        if not isinstance(head_dim, int) or head_dim <= 0 or head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim {head_dim} must be a positive even integer")
        if head_dim % 4 != 0:
            raise ConfigError(f"config.json: head_dim {head_dim} is not supported: the attention kernels "
                              f"take head sizes that are multiples of 4 (multiples of 16 run on the matrix cores)")
        if head_dim > 256:
            raise ConfigError(f"config.json: head_dim {head_dim} is not supported: no attention kernel here "
                              f"takes a head size above 256")
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act {act!r} is not supported (only 'silu')")
        if d.get("attention_bias", False):
            raise ConfigError("config.json: attention_bias=true is not supported")
        if d.get("mlp_bias", False):
            raise ConfigError("config.json: mlp_bias=true is not supported")
        scaling = d.get("rope_scaling")
        rope_scaling = None
        if scaling is not None:
            rtype = scaling.get("rope_type", scaling.get("type"))
            if rtype not in (None, "default"):
                rope_scaling = RopeScaling.from_dict(scaling)
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, (list, tuple)):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)
        archs = d.get("architectures") or ()
        dtype = d.get("torch_dtype", d.get("dtype", "bfloat16"))
        if dtype not in ("bfloat16", "float32"):
            raise ConfigError(f"config.json: torch_dtype {dtype!r} is not supported "
                              f"(supported: 'bfloat16', 'float32')")
        known = {f for f in LlamaConfig.__dataclass_fields__}  # type: ignore[attr-defined]
        cfg = LlamaConfig(
            vocab_size=_require(d, "vocab_size", int),
            hidden_size=hidden,
            intermediate_size=_require(d, "intermediate_size", int),
            num_hidden_layers=_require(d, "num_hidden_layers", int),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            rms_norm_eps=_require(d, "rms_norm_eps", float),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            max_position_embeddings=_require(d, "max_position_embeddings", int),
            rope_scaling=rope_scaling,
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            hidden_act=act,
            attention_bias=False,
            mlp_bias=False,
            torch_dtype=dtype,
            eos_token_id=eos_ids,
            bos_token_id=d.get("bos_token_id"),
            architectures=tuple(archs),
            extra={k: v for k, v in d.items() if k not in known and k != "dtype"},
        )
        for key in ("vocab_size", "intermediate_size", "num_hidden_layers",
                    "max_position_embeddings"):
            if getattr(cfg, key) <= 0:
                raise ConfigError(f"config.json: '{key}' must be positive")
        if not cfg.rms_norm_eps >= 0:
            raise ConfigError("config.json: rms_norm_eps must be non-negative")
        if not cfg.rope_theta > 0:
            raise ConfigError("config.json: rope_theta must be positive")
        return cfg

    def to_dict(self) -> dict:
        d = asdict(self)
        d.pop("extra")
        d["architectures"] = list(self.architectures)
        eos = list(self.eos_token_id)
        d["eos_token_id"] = eos[0] if len(eos) == 1 else (eos or None)
        if self.rope_scaling is None:
            d["rope_scaling"] = None
        d["model_type"] = "llama"
        return d

    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in model folder {model_dir!r}")
    with open(path, "r", encoding="utf-8") as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return d


def write_config_json(model_dir: str, config_dict: Mapping[str, Any]) -> None:
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(dict(config_dict), f, indent=2)
        f.write("\n")
