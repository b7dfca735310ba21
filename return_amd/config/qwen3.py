"""Configuration of the Qwen3 dense decoder, read from its config.json keys.

The reference reads these through HF objects: head_dim with the fallback
hidden // heads (rollout/monkey_patch/qwen3.py:117), num_key_value_heads
(qwen3.py:116), vocab_size (qwen3.py:115), the norms' variance_epsilon
(qwen3.py:17), rope inv_freq and attention_scaling (qwen3.py:121-127); it asserts
that no layer has a sliding window (qwen3.py:130-132) and fuses gate and up only
when there is no bias (qwen3.py:99-105).

The rotation's base comes in one of two layouts: the key rope_theta at the top level (with
rope_scaling beside it), or a dictionary rope_parameters {rope_theta, rope_type, ...}
that newer config.json files carry instead. Both are read; one of them must give the base;
any rope_type other than "default" is refused in either.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

from .base import ConfigError, ModelConfig


@dataclasses.dataclass(frozen=True)
class Qwen3Config(ModelConfig):
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    intermediate_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float                              # top-level key, or rope_parameters.rope_theta
    num_key_value_heads: Optional[int] = None      # absent: one per query head
    head_dim: Optional[int] = None                 # absent: hidden_size // num_attention_heads
    tie_word_embeddings: bool = False
    attention_bias: bool = False
    hidden_act: str = "silu"
    use_sliding_window: bool = False
    model_type: str = "qwen3"

    @classmethod
    def from_dict(cls, raw):
        raw = dict(raw)
        arch = (raw.get("architectures") or ["?"])[0]
        params = raw.get("rope_parameters")
        if params is not None:
            if not isinstance(params, dict):
                raise ConfigError(f"{arch}: rope_parameters must be a dictionary, got {params!r}")
            kind = params.get("rope_type", params.get("type"))
            if kind not in (None, "default"):
                raise ConfigError(f"{arch}: rope_parameters {params!r} is not supported (only rope_type 'default')")
            inner = params.get("rope_theta")
            if inner is not None:
                outer = raw.get("rope_theta")
                if outer is not None and float(outer) != float(inner):
                    raise ConfigError(f"{arch}: rope_theta is {outer!r} at the top level and {inner!r} in rope_parameters")
                raw["rope_theta"] = inner
        return super().from_dict(raw)

    def _coerce(self):
        super()._coerce()
        for name in ("num_key_value_heads", "head_dim"):
            v = getattr(self, name)
            if v is not None:
                if isinstance(v, bool) or float(v) != int(v):
                    raise ConfigError(f"{self.architecture}: {name} must be an integer, got {v!r}")
                object.__setattr__(self, name, int(v))
        if self.num_key_value_heads is None:
            object.__setattr__(self, "num_key_value_heads", self.num_attention_heads)
        if self.head_dim is None:
            if self.hidden_size % self.num_attention_heads:
                raise ConfigError(
                    f"{self.architecture}: no head_dim given and hidden_size {self.hidden_size} "
                    f"is not a multiple of num_attention_heads {self.num_attention_heads}")
            object.__setattr__(self, "head_dim", self.hidden_size // self.num_attention_heads)

    def validate(self, raw):
        a = self.architecture
        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "intermediate_size",
                     "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{a}: {name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"{a}: num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"{a}: head_dim {self.head_dim} must be even for rotary positions")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"{a}: rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"{a}: rope_theta must be positive, got {self.rope_theta}")
        if self.attention_bias:
            raise ConfigError(f"{a}: attention_bias=true is not supported (projections have no bias)")
        if self.hidden_act != "silu":
            raise ConfigError(f"{a}: hidden_act {self.hidden_act!r} is not supported (only 'silu')")
        if self.use_sliding_window:
            raise ConfigError(f"{a}: use_sliding_window=true is not supported (full causal attention only)")
        scaling = raw.get("rope_scaling")
        if scaling is not None:
            kind = scaling.get("rope_type", scaling.get("type")) if isinstance(scaling, dict) else scaling
            if kind not in (None, "default"):
                raise ConfigError(f"{a}: rope_scaling {scaling!r} is not supported (only null/default)")
        if self.model_type != "qwen3":
            raise ConfigError(f"{a}: model_type {self.model_type!r} does not belong to this architecture")

    @property
    def q_width(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.num_key_value_heads * self.head_dim
