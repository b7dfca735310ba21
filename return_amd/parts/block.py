"""How a mixer, a feed-forward and their norms are arranged in one layer.

"pre_norm" is rollout/monkey_patch/qwen3.py:59-68: h = h + attn(norm(h));
h = h + mlp(norm(h)). The addition of a part's output into the residual stream is
left to the next norm, which does it in 32-bit in the same kernel.
"""
from __future__ import annotations

from .registry import part_class, register_part


class PreNormBlock:
    def __init__(self, spec, tensors_of, rt, shared):
        """tensors_of(part_spec) -> dict role -> tensor, for the part's own tensors."""
        build = lambda cat, ps: part_class(cat, ps.kind)(ps.params, tensors_of(ps), rt, shared)
        self.mixer_norm = build("norm", spec.mixer_norm)
        self.mixer = build("mixer", spec.mixer)
        self.feed_forward_norm = build("norm", spec.feed_forward_norm)
        self.feed_forward = build("feed_forward", spec.feed_forward)

    def forward(self, h, pending, step, cache, write_cache=True):
        """h: fp32 residual; pending: output of the last part, not yet added. Returns (h, pending)."""
        x = self.mixer_norm.forward(h, pending)
        a = self.mixer.forward(x, step, cache, write_cache)
        x = self.feed_forward_norm.forward(h, a)
        f = self.feed_forward.forward(x, step)
        return h, f


BLOCKS = {"pre_norm": PreNormBlock}


def register_arrangement(name, cls):
    BLOCKS[name] = cls
