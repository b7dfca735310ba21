"""How the parts of one layer are arranged.

"pre_norm" is rollout/monkey_patch/qwen3.py:59-68: h = h + attn(norm(h));
h = h + mlp(norm(h)). The addition of a part's output into the residual stream is
left to the next norm, which does it in 32-bit in the same kernel.

An arrangement is a class with
    __init__(self, spec: BlockSpec, build)      build(name) -> the built part spec.parts[name]
    cache_spec(self)                            what the layer keeps between steps (its mixer's
                                                PagedKVSpec or StateSpec), or None
    step_needs(self) -> dict                    what its parts ask of the step's tables (may be {})
    forward(self, h, pending, step, cache, write_cache) -> (h, pending)
        h: fp32 residual stream [T, H]; pending: the last part's output, not yet added to h
        (or None); cache: the cache manager's view for this call's cache layer (or None).
It is registered with register_arrangement(name, cls) and named in BlockSpec.arrangement.
"""
from __future__ import annotations


class PreNormBlock:
    def __init__(self, spec, build):
        self.mixer_norm = build("mixer_norm")
        self.mixer = build("mixer")
        self.feed_forward_norm = build("feed_forward_norm")
        self.feed_forward = build("feed_forward")

    def cache_spec(self):
        return self.mixer.cache_spec()

    def step_needs(self):
        return self.mixer.step_needs() if hasattr(self.mixer, "step_needs") else {}

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
