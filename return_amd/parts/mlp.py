"""SwiGLU feed-forward: down(silu(gate(x)) * up(x)).

rollout/monkey_patch/qwen3.py:20-22 with gate and up fused into one weight, gate
rows first (qwen3.py:99-105); silu(g) * u in 32-bit: rollout/fused.py:103-114.
"""
from __future__ import annotations

import torch

from .registry import register_part


class SwiGLU:
    @staticmethod
    def tensor_shapes(params):
        H, I = params["hidden_size"], params["intermediate_size"]
        return {"gate_proj": (I, H), "up_proj": (I, H), "down_proj": (H, I)}

    @staticmethod
    def random_init(params, role):
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.inter = int(params["intermediate_size"])
        self.w_gate_up = rt.product(torch.cat([rt.matrix(tensors["gate_proj"]), rt.matrix(tensors["up_proj"])],
                                              dim=0).contiguous(), gated=True)
        self.w_down = rt.product(rt.matrix(tensors["down_proj"]), residual=True)
        self.first_product = (self.w_gate_up, True)        # (see PagedAttention)
        self.last_product = self.w_down

    def forward(self, x, step=None, sink=None):
        ops = self.rt.ops
        a = ops.linear_silu_mul(x, self.w_gate_up)         # [T, I] = silu(gate) * up, gate rows first
        return sink.project(a, self.w_down) if sink is not None else ops.linear(a, self.w_down)


register_part("feed_forward", "swiglu", SwiGLU)
