"""Typed model configurations read from an architecture's own ``config.json`` keys.

Every size and constant a model needs comes from here; no part of the engine
holds a literal width, head count, eps or theta.  The Llama reader follows the
key names and defaults of the reference (inference_engine/config.py:23-42).
"""
from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass, fields
from typing import Any, Mapping


class ConfigError(ValueError):
    """A config.json is missing a key, has a value of the wrong kind, or asks
    for something this engine does not compute."""


def _take_int(d: Mapping[str, Any], key: str, *, default=None, minimum: int = 1) -> int:
    if key not in d or d[key] is None:
        if default is None:
            raise ConfigError(f"config.json: required key '{key}' is missing")
        return default
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"config.json: '{key}' must be an integer, found {v!r}")
    if v < minimum:
        raise ConfigError(f"config.json: '{key}' must be >= {minimum}, found {v}")
    return v


def _take_float(d: Mapping[str, Any], key: str, *, default=None) -> float:
    if key not in d or d[key] is None:
        if default is None:
            raise ConfigError(f"config.json: required key '{key}' is missing")
        return float(default)
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: '{key}' must be a number, found {v!r}")
    return float(v)


def _take_bool(d: Mapping[str, Any], key: str, default: bool) -> bool:
    v = d.get(key, default)
    if v is None:
        return default
    if not isinstance(v, bool):
        raise ConfigError(f"config.json: '{key}' must be true or false, found {v!r}")
    return v


@dataclass(frozen=True)
class ModelConfig:
    """Base of every architecture's configuration."""

    architecture = "?"

    def to_dict(self) -> dict:
        raise NotImplementedError

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "ModelConfig":
        raise NotImplementedError


@dataclass(frozen=True)
class LlamaConfig(ModelConfig):
    """Llama dense decoder.  Fields carry config.json's own key names.

    Keys and defaults as the reference reads them (inference_engine/config.py:26-42):
    required are vocab_size, hidden_size, intermediate_size, num_hidden_layers,
    num_attention_heads, rms_norm_eps, max_position_embeddings; num_key_value_heads
    defaults to the head count, head_dim to hidden_size // heads, rope_theta to
    10000, tie_word_embeddings to false, eos_token_id to 2.  The reference keeps the first entry of a list of
    stop ids; here every entry stops a request (``eos_token_id`` is the tuple of them).
    """

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
    tie_word_embeddings: bool = False
    eos_token_id: tuple = (2,)

    architecture = "LlamaForCausalLM"

    def __post_init__(self):
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) must be a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"head_dim ({self.head_dim}) must be even for rotary pairs")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"rms_norm_eps must be positive, found {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, found {self.rope_theta}")

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "LlamaConfig":
        heads = _take_int(d, "num_attention_heads")
        hidden = _take_int(d, "hidden_size")
        # What the reference never reads (hidden_act, rope_scaling, biases) must
        # hold the value its formulas assume, or the logits would silently differ.
        act = d.get("hidden_act")
        if act not in (None, "silu"):
            raise ConfigError(f"config.json: hidden_act '{act}' is not computed here (only 'silu')")
        if d.get("rope_scaling") not in (None, {}):
            raise ConfigError("config.json: rope_scaling is not computed here (plain rotary only)")
        for key in ("attention_bias", "mlp_bias"):
            if _take_bool(d, key, False):
                raise ConfigError(f"config.json: {key}=true is not computed here")
        head_dim = d.get("head_dim") or hidden // heads
        eos = d.get("eos_token_id", 2)
        if not isinstance(eos, (list, tuple)):
            eos = [eos]
        if not eos:
            raise ConfigError("config.json: eos_token_id is an empty list")
        eos = tuple(_take_int({"eos_token_id": e}, "eos_token_id", minimum=0) for e in eos)
        return cls(
            vocab_size=_take_int(d, "vocab_size"),
            hidden_size=hidden,
            intermediate_size=_take_int(d, "intermediate_size"),
            num_hidden_layers=_take_int(d, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=_take_int(d, "num_key_value_heads", default=heads),
            head_dim=_take_int({"head_dim": head_dim}, "head_dim"),
            rms_norm_eps=_take_float(d, "rms_norm_eps"),
            rope_theta=_take_float(d, "rope_theta", default=10000.0),
            max_position_embeddings=_take_int(d, "max_position_embeddings"),
            tie_word_embeddings=_take_bool(d, "tie_word_embeddings", False),
            eos_token_id=eos,
        )

    def to_dict(self) -> dict:
        d = asdict(self)
        d["eos_token_id"] = self.eos_token_id[0] if len(self.eos_token_id) == 1 else list(self.eos_token_id)
        d["architectures"] = [self.architecture]
        d["model_type"] = "llama"
        d["hidden_act"] = "silu"
        return d

    @property
    def num_parameters(self) -> int:
        h, i, v = self.hidden_size, self.intermediate_size, self.vocab_size
        qkv = (self.num_attention_heads + 2 * self.num_key_value_heads) * self.head_dim * h
        o = h * self.num_attention_heads * self.head_dim
        per_layer = qkv + o + 3 * i * h + 2 * h
        head = 0 if self.tie_word_embeddings else v * h
        return v * h + self.num_hidden_layers * per_layer + h + head


def read_config_json(path: str) -> dict:
    """``path`` is a model folder or the config.json itself."""
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json at {path}")
    with open(path) as f:
        d = json.load(f)
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return d


def config_field_names(cls) -> list[str]:
    return [f.name for f in fields(cls)]
