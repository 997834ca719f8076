"""Typed model configurations read from an architecture's own config.json keys.

The Qwen3 fields, their defaults and their types follow the reference's
``ModelConfig`` (src/models/model_config.hpp:7-47).  Unlike the reference,
which never consults ``model_type``/``hidden_act`` and wires the model class in
code (src/engine/model_runner.hpp:21), every value is validated here and the
model class is looked up by ``architectures[0]``.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, ClassVar, Dict, List, Optional


class ConfigError(ValueError):
    """A config.json that this engine cannot run, with the reason."""


@dataclasses.dataclass
class ModelConfig:
    """Base of all architecture configurations.

    A subclass lists its config.json keys as dataclass fields (the field name is
    the key), gives defaults where the architecture defines them, and checks
    consistency in ``validate``.
    """

    architectures: List[str] = dataclasses.field(default_factory=list)

    #: keys that must be present in config.json
    required: ClassVar[tuple] = ()

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "ModelConfig":
        missing = [k for k in cls.required if k not in raw]
        if missing:
            raise ConfigError("config.json lacks required key(s): " + ", ".join(missing))
        known = {f.name: f for f in dataclasses.fields(cls)}
        kwargs = {}
        for name, field in known.items():
            if name not in raw or raw[name] is None:
                continue
            kwargs[name] = _coerce(name, raw[name], field.type)
        cfg = cls(**kwargs)
        cfg._raw = dict(raw)
        cfg.fill_defaults()
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str) -> "ModelConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> Dict[str, Any]:
        return {f.name: getattr(self, f.name) for f in dataclasses.fields(self)}

    def fill_defaults(self) -> None:
        pass

    def validate(self) -> None:
        pass

    # What the engine itself asks of any architecture's configuration, whatever its config.json keys are called.
    @property
    def position_limit(self) -> Optional[int]:
        """Most tokens a request may reach (the architecture's positions end there); None = no limit."""
        return None

    @property
    def end_token_id(self) -> Optional[int]:
        """The token at which generation ends; None = the architecture names none."""
        return None


def _coerce(name, value, type_name):
    t = str(type_name)
    try:
        if t in ("int", "<class 'int'>"):
            if isinstance(value, bool) or (isinstance(value, float) and value != int(value)):
                raise TypeError
            if isinstance(value, (list, dict, str)):
                raise TypeError
            return int(value)
        if t in ("float", "<class 'float'>"):
            if isinstance(value, (bool, list, dict, str)):
                raise TypeError
            return float(value)
        if t in ("bool", "<class 'bool'>"):
            if not isinstance(value, bool):
                raise TypeError
            return value
        if t in ("str", "<class 'str'>"):
            if not isinstance(value, str):
                raise TypeError
            return value
    except (TypeError, ValueError):
        raise ConfigError("config.json key %r has value %r, expected %s" % (name, value, t)) from None
    return value


@dataclasses.dataclass
class Qwen3Config(ModelConfig):
    """Qwen3 dense decoder.  Keys and defaults: src/models/model_config.hpp:32-46."""

    model_type: str = ""
    hidden_act: str = ""
    hidden_size: int = -1
    intermediate_size: int = -1
    num_key_value_heads: int = -1
    num_hidden_layers: int = -1
    num_attention_heads: int = -1
    tie_word_embeddings: bool = False
    rope_theta: float = 1000000.0
    rms_norm_eps: float = 1e-6
    head_dim: int = -1  # falls back to hidden_size / num_attention_heads (model_config.hpp:42)
    bos_token_id: int = -1
    eos_token_id: int = -1
    max_position_embeddings: int = 16384
    vocab_size: int = -1

    required: ClassVar[tuple] = ("model_type", "hidden_act")

    @property
    def position_limit(self):
        return self.max_position_embeddings

    @property
    def end_token_id(self):
        return self.eos_token_id if self.eos_token_id >= 0 else None

    def fill_defaults(self) -> None:
        if self.head_dim == -1 and self.num_attention_heads > 0:
            self.head_dim = self.hidden_size // self.num_attention_heads

    def validate(self) -> None:
        raw = getattr(self, "_raw", {})
        for name in ("hidden_size", "intermediate_size", "num_key_value_heads", "num_hidden_layers",
                     "num_attention_heads", "head_dim", "max_position_embeddings", "vocab_size"):
            if getattr(self, name) <= 0:
                raise ConfigError("config.json: %s must be a positive integer, got %r" % (name, getattr(self, name)))
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError("config.json: num_attention_heads (%d) is not a multiple of num_key_value_heads (%d)"
                              % (self.num_attention_heads, self.num_key_value_heads))
        if self.head_dim % 2 != 0:
            raise ConfigError("config.json: head_dim (%d) must be even for rotary pairs" % self.head_dim)
        # The reference fixes SiLU in code (src/backends/cpu/x64/kernels.cpp:224-247) and never reads hidden_act.
        if self.hidden_act != "silu":
            raise ConfigError("config.json: hidden_act %r is not supported (the architecture uses 'silu')" % self.hidden_act)
        if not (self.rms_norm_eps > 0.0):
            raise ConfigError("config.json: rms_norm_eps must be positive")
        if not (self.rope_theta > 0.0):
            raise ConfigError("config.json: rope_theta must be positive")
        # Options that the reference does not implement are refused rather than silently ignored.
        if raw.get("attention_bias"):
            raise ConfigError("config.json: attention_bias is set, but this architecture has no projection biases "
                              "(src/models/qwen3.hpp:39)")
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError("config.json: rope_scaling is not supported (src/utils/constant_table.hpp:28-41 has no scaling)")
        if raw.get("use_sliding_window"):
            raise ConfigError("config.json: use_sliding_window is set, but this architecture attends to all keys "
                              "(src/backends/cpu/cpu_attention.cpp:98-111)")
