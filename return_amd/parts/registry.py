"""Registry of part kinds. A part class is registered under a category and a name;
a PartSpec names it by ``kind``. Tests register toy parts the same way.

Interfaces (``rt`` is the return_amd.parts.runtime.Runtime of the engine):

  every part    __init__(self, params: dict, tensors: dict[str, Tensor], rt, shared)
                    (shared: the model's named position encodings)
                @staticmethod tensor_shapes(params) -> dict role -> shape tuple
                    (roles the checkpoint must hold; used to check shapes before loading)
                @staticmethod random_init(params, role) -> "matrix" | "embedding" | "norm"
                    (which distribution the random-weights mode draws for the role), or a callable
                    (shape, generator) -> tensor for a law of the part's own, drawn from that
                    torch.Generator (set its attribute keep_dtype = True to keep the tensor's dtype
                    whatever precision the model is written in)
  norm          forward(h, delta, out_rows=None) -> x
                    h: fp32 residual [T, H]; delta: last part's output or None.
                    Adds delta into h in place, returns norm(h) in the compute dtype;
                    with out_rows (int32 indices) only those rows are returned.
  mixer         cache_spec() -> PagedKVSpec | StateSpec | None, or a tuple of them for a mixer that keeps
                    more than one thing (paged keys and a state of fixed size, say): the run order then
                    gives the call a tuple of cache layers (LayerCall.cache) and forward's ``cache`` is
                    the tuple of their views, in that order
                step_needs() -> dict (optional): what it asks of the step's tables, e.g.
                    {"prefill_tile_rows": {128}} for the q-tile list its attention kernel reads
                forward(x, step, cache) -> y      x, y: [T, H] compute dtype
                    step: return_amd.engine.batch.StepBatch; cache: the view the cache
                    manager gives for this call's cache layer (None without cache_spec)
  feed_forward  forward(x, step) -> y

  Optional, for a mixer or feed-forward whose input goes into ONE product and whose output comes out
  of ONE (then the kernel set may finish the norms around the part inside those products, or form the
  last product as shares that the next norm adds up). All or none of it:
                first_product = (w, gated)   attribute: the weight [N, K] (gated: [2N, K], gate rows
                    first) of the product that x goes into and nowhere else; x may then arrive as
                    return_amd.parts.runtime.ScaledRows, which ops.linear / ops.linear_silu_mul take
                last_product = w             attribute: the weight of the product whose result is y
                forward(..., sink=None)      one more parameter, last: when a sink is given, y is
                    sink.project(a, w) instead of ops.linear(a, w) (it may be ScaledRows or Slabs and
                    goes to the next norm as it is). A part without that parameter is never given one.
  and for a norm: weight, eps attributes (a plain RMS norm whose 1/rms a product can apply) and
                takes_slabs = True if forward's delta may be Slabs.
  position      an object the mixer uses; rotary ones offer tables() -> (cos, sin, rotary_dim)
                and every one offers apply(q, k, positions) in place on [T, heads, D].
                One with more than one axis per token declares step_needs() ->
                {"token_columns": ("name", ...)}: the step then carries step.token_columns[name],
                int32 [T] (what a request brings with its tokens, StepEntry.columns / Engine.submit's
                token_columns; the position where it brings nothing), and apply is called as
                apply(q, k, positions, step). Mixers and embeddings may declare columns the same way.
  embedding     forward(token_ids, step) -> h  fp32 [T, H]   (step.positions for absolute positions)
  head          forward(x) -> logits fp32 [rows, V]
"""
from __future__ import annotations

from typing import Dict

CATEGORIES = ("norm", "mixer", "feed_forward", "position", "embedding", "head")
_PARTS: Dict[str, Dict[str, type]] = {c: {} for c in CATEGORIES}


def register_part(category: str, kind: str, cls: type) -> None:
    if category not in _PARTS:
        raise KeyError(f"unknown part category {category!r}; one of {CATEGORIES}")
    _PARTS[category][kind] = cls


def part_class(category: str, kind: str) -> type:
    try:
        return _PARTS[category][kind]
    except KeyError:
        known = ", ".join(sorted(_PARTS.get(category, {}))) or "(none)"
        raise KeyError(f"no {category} part named {kind!r}; registered: {known}") from None
