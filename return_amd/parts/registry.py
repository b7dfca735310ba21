"""Registry of part kinds. A part class is registered under a category and a name;
a PartSpec names it by ``kind``. Tests register toy parts the same way.

Interfaces (``rt`` is the return_amd.parts.runtime.Runtime of the engine):

  every part    __init__(self, params: dict, tensors: dict[str, Tensor], rt, shared)
                    (shared: the model's named position encodings)
                @staticmethod tensor_shapes(params) -> dict role -> shape tuple
                    (roles the checkpoint must hold; used to check shapes before loading)
                @staticmethod random_init(params, role) -> "matrix" | "embedding" | "norm"
                    (which distribution the random-weights mode draws for the role)
  norm          forward(h, delta, out_rows=None) -> x
                    h: fp32 residual [T, H]; delta: last part's output or None.
                    Adds delta into h in place, returns norm(h) in the compute dtype;
                    with out_rows (int32 indices) only those rows are returned.
  mixer         cache_spec() -> PagedKVSpec | StateSpec | None
                step_needs() -> dict (optional): what it asks of the step's tables, e.g.
                    {"prefill_tile_rows": {128}} for the q-tile list its attention kernel reads
                forward(x, step, cache) -> y      x, y: [T, H] compute dtype
                    step: return_amd.engine.batch.StepBatch; cache: the view the cache
                    manager gives for this call's cache layer (None without cache_spec)
  feed_forward  forward(x, step) -> y
  position      an object the mixer uses; rotary ones offer tables() -> (cos, sin, rotary_dim)
                and every one offers apply(q, k, positions) in place on [T, heads, D]
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
