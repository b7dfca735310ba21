"""RMSNorm over the last axis, with the residual addition folded in.

y = x * rsqrt(mean(x^2) + eps) * (offset + w), all in 32-bit, rounded to the
compute dtype after the weight multiply: rollout/fused.py:6-17. Qwen3 uses
offset 0.0 (rollout/monkey_patch/qwen3.py:15-17).
"""
from __future__ import annotations

from .registry import register_part
from .runtime import ScaledRows


class RMSNorm:
    takes_slabs = True          # forward's delta may be Slabs (the kernel set's add_rmsnorm adds them up)

    @staticmethod
    def tensor_shapes(params):
        return {"weight": (params["size"],)}

    @staticmethod
    def random_init(params, role):
        return "norm"

    def __init__(self, params, tensors, rt, shared=None):
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.offset = float(params.get("offset", 0.0))
        self.rt = rt
        w = rt.vector32(tensors["weight"])
        self.weight = w + self.offset if self.offset != 0.0 else w

    def forward(self, h, delta=None, out_rows=None):
        """h (fp32 [T, size]) += delta in place; returns norm(h) (only rows out_rows, if given)."""
        if isinstance(delta, ScaledRows):
            # the product before has added its result into h and left this norm's rows unfinished:
            # the next product applies 1/rms itself
            if delta.norm is not self or out_rows is not None:
                raise ValueError("rows prepared for another norm, or for all rows where some are wanted")
            return delta
        rows = h.shape[0] if out_rows is None else out_rows.shape[0]
        out = self.rt.empty(rows, self.size)
        self.rt.ops.add_rmsnorm(h, delta, self.weight, self.eps, out, out_rows)
        return out


register_part("norm", "rms_norm", RMSNorm)
