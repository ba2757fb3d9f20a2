"""Typed model configuration read from an architecture's own config.json keys."""

import dataclasses
import json
import os
from dataclasses import dataclass


class ConfigError(ValueError):
    """config.json lacks a key, holds a value of the wrong kind, or asks for
    something this engine does not compute."""


def _require(data, key, kind):
    if key not in data:
        raise ConfigError("config.json: required key %r is missing" % key)
    value = data[key]
    if kind is float and isinstance(value, int) and not isinstance(value, bool):
        value = float(value)
    if kind is int and isinstance(value, bool):
        raise ConfigError("config.json: %r must be an integer, found %r" % (key, value))
    if not isinstance(value, kind):
        raise ConfigError(
            "config.json: %r must be %s, found %r" % (key, kind.__name__, value)
        )
    return value


@dataclass(frozen=True)
class ModelConfig:
    """The Qwen3 dense decoder's sizes and constants.

    Field names are config.json's. The set of required and optional keys is that
    of the reference's reader (src/qwen3_from_scratch/factory/config.py:107-130):
    every size, `rms_norm_eps`, `rope_theta` and `hidden_act` are required,
    `tie_word_embeddings` defaults to false. There are no defaults for sizes:
    a config that omits one is refused.
    """

    architecture: str
    vocab_size: int
    hidden_size: int
    hidden_act: str
    num_hidden_layers: int
    max_position_embeddings: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool = False
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, data, architecture=None):
        if architecture is None:
            names = data.get("architectures")
            if not names or not isinstance(names, list):
                raise ConfigError(
                    "config.json: 'architectures' must name the model class, "
                    "e.g. [\"Qwen3ForCausalLM\"]"
                )
            architecture = names[0]
        rope_theta = data.get("rope_theta")
        if rope_theta is None and isinstance(data.get("rope_parameters"), dict):
            rope_theta = data["rope_parameters"].get("rope_theta")
        if rope_theta is None:
            raise ConfigError("config.json: required key 'rope_theta' is missing")
        eos = data.get("eos_token_id", ())
        if isinstance(eos, int):
            eos = (eos,)
        elif eos is None:
            eos = ()
        config = cls(
            architecture=architecture,
            vocab_size=_require(data, "vocab_size", int),
            hidden_size=_require(data, "hidden_size", int),
            hidden_act=_require(data, "hidden_act", str),
            num_hidden_layers=_require(data, "num_hidden_layers", int),
            max_position_embeddings=_require(data, "max_position_embeddings", int),
            num_attention_heads=_require(data, "num_attention_heads", int),
            num_key_value_heads=_require(data, "num_key_value_heads", int),
            head_dim=_require(data, "head_dim", int),
            intermediate_size=_require(data, "intermediate_size", int),
            rms_norm_eps=_require(data, "rms_norm_eps", float),
            rope_theta=float(rope_theta),
            tie_word_embeddings=bool(data.get("tie_word_embeddings", False)),
            eos_token_ids=tuple(int(t) for t in eos),
        )
        config.validate(data)
        return config

    @classmethod
    def from_json(cls, path):
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as fh:
            return cls.from_dict(json.load(fh))

    def validate(self, raw=None):
        """Refuse what the engine would compute wrongly or not at all."""
        for name in (
            "vocab_size", "hidden_size", "num_hidden_layers", "max_position_embeddings",
            "num_attention_heads", "num_key_value_heads", "head_dim", "intermediate_size",
        ):
            if getattr(self, name) <= 0:
                raise ConfigError("config.json: %r must be positive" % name)
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                "config.json: num_attention_heads (%d) is not a multiple of "
                "num_key_value_heads (%d)" % (self.num_attention_heads, self.num_key_value_heads)
            )
        if self.head_dim % 2:
            raise ConfigError("config.json: head_dim (%d) must be even for rotation" % self.head_dim)
        if self.hidden_act != "silu":
            raise ConfigError(
                "config.json: hidden_act %r is not supported (only 'silu')" % self.hidden_act
            )
        if not (self.rms_norm_eps >= 0.0):
            raise ConfigError("config.json: rms_norm_eps must not be negative")
        if not (self.rope_theta > 0.0):
            raise ConfigError("config.json: rope_theta must be positive")
        raw = raw or {}
        if raw.get("attention_bias"):
            raise ConfigError("config.json: attention_bias=true is not supported")
        if raw.get("use_sliding_window"):
            raise ConfigError("config.json: use_sliding_window=true is not supported")
        scaling = raw.get("rope_scaling")
        if scaling and scaling.get("rope_type", scaling.get("type", "default")) != "default":
            raise ConfigError("config.json: rope_scaling %r is not supported" % (scaling,))

    def to_dict(self):
        """The config.json form of this configuration."""
        data = dataclasses.asdict(self)
        data["architectures"] = [data.pop("architecture")]
        eos = data.pop("eos_token_ids")
        if eos:
            data["eos_token_id"] = list(eos) if len(eos) > 1 else eos[0]
        data["torch_dtype"] = "bfloat16"
        return data
