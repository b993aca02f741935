"""Typed configuration of the Qwen3 dense decoder, read from config.json's own keys.

Keys, defaults and checks follow crates/synaptix-models/llm/qwen3/src/config.rs:6-87 of
the reference.  Two deliberate differences: the reference parses `attention_bias`,
`use_sliding_window` and `sliding_window` and then ignores them (config.rs:117-118);
here a value that the model would not honour is an error instead of being dropped
silently.  Sizes that the reference leaves unchecked (layers, vocabulary,
intermediate size, an odd head size, eps, theta) are checked as well.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, fields, asdict
from typing import Optional

import numpy as np

from .errors import ConfigError


@dataclass(frozen=True)
class Qwen3Config:
    # defaults are those of the reference (the 1.7B model): config.rs:28-50
    vocab_size: int = 151936
    hidden_size: int = 2048
    intermediate_size: int = 6144
    num_hidden_layers: int = 28
    num_attention_heads: int = 16
    num_key_value_heads: int = 8
    head_dim: int = 128
    max_position_embeddings: int = 40960
    rms_norm_eps: float = 1.0e-6
    rope_theta: float = 1_000_000.0
    hidden_act: str = "silu"
    attention_bias: bool = False
    bos_token_id: Optional[int] = 151643
    eos_token_id: Optional[int] = 151645
    tie_word_embeddings: bool = True
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None

    architecture = "Qwen3ForCausalLM"
    model_type = "qwen3"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: dict) -> "Qwen3Config":
        """Known keys are typed; unknown keys (model_type, torch_dtype, ...) are ignored,
        as serde's `default` on the whole struct does in the reference (config.rs:7-8)."""
        kw = {}
        for f in fields(cls):
            if f.name not in d:
                continue
            v = d[f.name]
            try:
                kw[f.name] = _coerce(f.name, f.type, v)
            except (TypeError, ValueError) as e:
                raise ConfigError(f"config key {f.name!r}: {e}") from None
        cfg = cls(**kw)
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str) -> "Qwen3Config":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        try:
            with open(path) as f:
                d = json.load(f)
        except OSError as e:
            raise ConfigError(f"read {path}: {e}") from None
        except json.JSONDecodeError as e:
            raise ConfigError(f"parse {path}: {e}") from None
        if not isinstance(d, dict):
            raise ConfigError(f"parse {path}: top level is not an object")
        return cls.from_dict(d)

    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = [self.architecture]
        d["model_type"] = self.model_type
        return d

    # ------------------------------------------------------------------ checks
    def validate(self) -> None:
        def bad(msg):
            raise ConfigError(msg)

        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                     "num_attention_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                bad(f"{name} == {getattr(self, name)} (must be positive)")
        if self.num_key_value_heads <= 0 or self.num_attention_heads % self.num_key_value_heads != 0:
            bad(f"GQA constraint: heads={self.num_attention_heads} must be divisible by "
                f"kv_heads={self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            bad(f"head_dim {self.head_dim} must be even for the rotation")
        if self.hidden_act not in ("silu", "swish"):
            bad(f"hidden_act unsupported: {self.hidden_act} (only silu/swish)")
        if not (self.rms_norm_eps > 0.0):
            bad(f"rms_norm_eps {self.rms_norm_eps} must be positive")
        if not (self.rope_theta > 0.0):
            bad(f"rope_theta {self.rope_theta} must be positive")
        if self.attention_bias:
            bad("attention_bias = true: this decoder has no projection biases")
        if self.use_sliding_window:
            bad("use_sliding_window = true: every layer of this decoder attends to all keys")

    # ------------------------------------------------------------------ derived
    @property
    def group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @property
    def q_total_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_total_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def eps_f32(self) -> float:
        """eps as the reference holds it: a 32-bit float (config.rs:17)."""
        return float(np.float32(self.rms_norm_eps))

    @property
    def theta_f32(self) -> float:
        """theta as the reference holds it: a 32-bit float (config.rs:18)."""
        return float(np.float32(self.rope_theta))

    @property
    def stop_token_ids(self) -> tuple:
        return () if self.eos_token_id is None else (self.eos_token_id,)


def _coerce(name, typ, v):
    typ = str(typ)
    if "Optional" in typ and v is None:
        return None
    if "bool" in typ:
        if not isinstance(v, bool):
            raise TypeError(f"expected true/false, got {v!r}")
        return v
    if "int" in typ:
        if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
            raise TypeError(f"expected an integer, got {v!r}")
        return int(v)
    if "float" in typ:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise TypeError(f"expected a number, got {v!r}")
        return float(v)
    if "str" in typ:
        if not isinstance(v, str):
            raise TypeError(f"expected a string, got {v!r}")
        return v
    return v
