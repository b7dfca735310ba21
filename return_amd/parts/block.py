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
    Optional: first_norm / first_product attributes and an after= argument of forward (see PreNormBlock),
    with which the norm between two blocks can be finished inside their products.
It is registered with register_arrangement(name, cls) and named in BlockSpec.arrangement.
"""
from __future__ import annotations

import inspect

from .runtime import NormSink, ResidualSink


_TAKES_SINK = {}


def takes_sink(part):
    """Whether the part's forward has a ``sink`` parameter (a part may note its last product for the
    kernel set's measurement and still form it itself: then it is never handed a sink)."""
    cls = type(part)
    hit = _TAKES_SINK.get(cls)
    if hit is None:
        try:
            hit = "sink" in inspect.signature(cls.forward).parameters
        except (AttributeError, TypeError, ValueError):
            hit = False
        _TAKES_SINK[cls] = hit
    return hit


def norm_sink(h, producer, norm, consumer_first_product):
    """The sink for the last product of ``producer``, whose result goes through ``norm`` into the next
    part, or None. A NormSink when the producer ends in one product and the consumer begins with one
    (their last_product / first_product attributes), the norm is a plain RMSNorm part, and the kernel
    set says that it can finish the norm inside these two products for this many rows
    (can_defer_norm); else a ResidualSink when the norm takes a product's result in every form
    (takes_slabs); else None: the part forms its product as it does for anyone."""
    ops = getattr(getattr(norm, "rt", None), "ops", None)
    last = getattr(producer, "last_product", None)
    if last is None or ops is None or norm is None or not takes_sink(producer):
        return None
    if consumer_first_product is not None and hasattr(ops, "can_defer_norm") and \
            hasattr(norm, "weight") and hasattr(norm, "eps"):
        first, gated = consumer_first_product
        if ops.can_defer_norm(h.shape[0], last, first, gated):
            return NormSink(ops, h, norm)
    return ResidualSink(ops) if getattr(norm, "takes_slabs", False) else None


class PreNormBlock:
    def __init__(self, spec, build):
        self.mixer_norm = build("mixer_norm")
        self.mixer = build("mixer")
        self.feed_forward_norm = build("feed_forward_norm")
        self.feed_forward = build("feed_forward")
        # what the block before may fuse into: this block's first norm and the product behind it
        self.first_norm = self.mixer_norm
        self.first_product = getattr(self.mixer, "first_product", None)
        self.last_product = getattr(self.feed_forward, "last_product", None)

    def norm_pairs(self):
        """(product before, norm weight, eps, product after, gated) of the norm inside the block, if it sits
        between two products."""
        last, first = getattr(self.mixer, "last_product", None), getattr(self.feed_forward, "first_product", None)
        if last is None or first is None or not hasattr(self.feed_forward_norm, "weight"):
            return []
        return [(last, self.feed_forward_norm.weight, self.feed_forward_norm.eps, *first)]

    def cache_spec(self):
        return self.mixer.cache_spec()

    def step_needs(self):
        return self.mixer.step_needs() if hasattr(self.mixer, "step_needs") else {}

    def forward(self, h, pending, step, cache, write_cache=True, after=None):
        """h: fp32 residual; pending: output of the last part, not yet added. Returns (h, pending).
        after: (norm, first product) of what takes this block's pending output, the next block's
        first_norm and first_product or the model's last norm and None; None: unknown. The norm may be
        finished inside this block's last product and that first one, or take the product in shares."""
        x = self.mixer_norm.forward(h, pending)
        sink = norm_sink(h, self.mixer, self.feed_forward_norm, getattr(self.feed_forward, "first_product", None))
        a = self.mixer.forward(x, step, cache, write_cache, sink) if sink is not None else \
            self.mixer.forward(x, step, cache, write_cache)
        x = self.feed_forward_norm.forward(h, a)
        sink = norm_sink(h, self.feed_forward, after[0], after[1]) if after is not None else None
        f = self.feed_forward.forward(x, step, sink) if sink is not None else self.feed_forward.forward(x, step)
        return h, f


BLOCKS = {"pre_norm": PreNormBlock}


def register_arrangement(name, cls):
    BLOCKS[name] = cls
