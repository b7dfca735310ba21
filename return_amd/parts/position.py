"""Rotary position encoding, half-split pairing.

x1 = x[:R/2], x2 = x[R/2:R]; o1 = x1*cos - x2*sin, o2 = x2*cos + x1*sin in 32-bit;
dimensions from R on pass through: rollout/attention.py:10-25, rollout/fused.py:59-83.
Angles are position * inv_freq with inv_freq[j] = theta^(-2j/R), and the tables are
cos and sin of them times attention_scaling: rollout/monkey_patch/qwen3.py:121-127
(the reference stores the tables in bf16; here they stay 32-bit).
"""
from __future__ import annotations

import torch

from .registry import register_part


class RotaryPosition:
    @staticmethod
    def tensor_shapes(params):
        return {}

    def __init__(self, params, tensors, rt, shared=None):
        self.head_dim = int(params["head_dim"])
        self.rotary_dim = int(params.get("rotary_dim", self.head_dim))
        self.theta = float(params["theta"])
        self.max_position = int(params["max_position"])
        self.scaling = float(params.get("attention_scaling", 1.0))
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        self.rt = rt
        half = self.rotary_dim // 2
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, half, dtype=torch.float32) / half))
        angle = torch.outer(torch.arange(self.max_position, dtype=torch.float32), inv_freq)
        self.cos = (angle.cos() * self.scaling).to(rt.device).contiguous()
        self.sin = (angle.sin() * self.scaling).to(rt.device).contiguous()

    def tables(self):
        """(cos, sin, rotary_dim): fp32 [max_position, rotary_dim/2] each."""
        return self.cos, self.sin, self.rotary_dim

    def apply(self, q, k, positions):
        """Rotate q and k ([T, heads, D], compute dtype) in place by their tokens' positions."""
        self.rt.ops.rope(q, positions, self.cos, self.sin, self.rotary_dim)
        if k is not None:
            self.rt.ops.rope(k, positions, self.cos, self.sin, self.rotary_dim)


register_part("position", "rotary", RotaryPosition)
