"""The generic decoder: parts built from a ModelSpec, run in the order the spec gives.

The reference's counterpart is the patched HF module: embed, layers in a loop,
final norm (rollout/monkey_patch/qwen3.py:71-81), then the head on selected rows
only (qwen3.py:145-156, rollout/model.py:286-290).
"""
from __future__ import annotations

from typing import Dict

import torch

from ..parts.block import BLOCKS
from ..parts.registry import part_class
from ..parts.spec import ModelSpec


class Decoder:
    def __init__(self, spec: ModelSpec, weights: Dict[str, torch.Tensor], rt):
        self.spec = spec
        self.rt = rt

        def tensors_of(ps):
            return {role: weights[name] for role, name in ps.tensors.items()}

        build = lambda cat, ps, shared=None: part_class(cat, ps.kind)(ps.params, tensors_of(ps), rt, shared)
        self.positions = {name: build("position", ps) for name, ps in spec.positions.items()}
        self.embedding = build("embedding", spec.embedding, self.positions)
        self.blocks = []
        for b in spec.blocks:
            if b.arrangement not in BLOCKS:
                raise KeyError(f"no block arrangement {b.arrangement!r}; registered: {sorted(BLOCKS)}")

            def build_named(name, b=b):
                b.part(name)                              # (a clear error for a name the block lacks)
                category, ps = b.parts[name]
                return build(category, ps, self.positions)
            self.blocks.append(BLOCKS[b.arrangement](b, build_named))
        self.final_norm = build("norm", spec.final_norm)
        self.head = build("head", spec.head)
        self.schedule = list(spec.schedule)
        for call in self.schedule:
            if not 0 <= call.block < len(self.blocks):
                raise ValueError(f"run order names block {call.block}, the model has {len(self.blocks)}")
        # the norms that sit between two products (inside a block, and between one block and the next in
        # the run order), for the kernel set to measure whether it finishes them inside those products
        for i, call in enumerate(self.schedule):
            block = self.blocks[call.block]
            rt.norm_pairs.extend(block.norm_pairs() if hasattr(block, "norm_pairs") else [])
            nxt = self.blocks[self.schedule[i + 1].block] if i + 1 < len(self.schedule) else None
            last = getattr(block, "last_product", None)
            if nxt is not None and last is not None and getattr(nxt, "first_product", None) is not None and \
                    hasattr(getattr(nxt, "first_norm", None), "weight"):
                rt.norm_pairs.append((last, nxt.first_norm.weight, nxt.first_norm.eps, *nxt.first_product))
        rt.forget_casts()

    def cache_layers(self):
        """cache layer number -> what the mixer that writes it needs (for the cache manager)."""
        need, writers = {}, set()
        for call in self.schedule:
            if call.cache is None:
                continue
            spec = self.blocks[call.block].cache_spec()
            if spec is None:
                raise ValueError(f"block {call.block} keeps nothing but the run order gives it cache layer {call.cache}")
            # a block that keeps several things names them as a tuple, and the call a cache layer for each
            specs = tuple(spec) if isinstance(spec, (tuple, list)) else (spec,)
            layers = tuple(call.cache) if isinstance(call.cache, (tuple, list)) else (call.cache,)
            if len(specs) != len(layers):
                raise ValueError(f"block {call.block} keeps {len(specs)} things but the run order gives it "
                                 f"cache layers {call.cache}")
            for layer, one in zip(layers, specs):
                if layer in need and need[layer] != one:
                    raise ValueError(f"cache layer {layer} is used by mixers with different needs")
                need[layer] = one
                if call.writes_cache:
                    if layer in writers:
                        raise ValueError(f"cache layer {layer} has two writers in the run order")
                    writers.add(layer)
        missing = set(need) - writers
        if missing:
            raise ValueError(f"cache layers {sorted(missing)} are read but never written")
        return need

    def step_needs(self):
        """What the parts ask of a step's tables beyond what every step has, merged over the model:
        {"prefill_tile_rows": set of q-tile heights whose tile lists the attention kernels read,
         "token_columns": set of names of further integers per token (StepBatch.token_columns) that a
         block, a position encoding or the embedding reads beside the position}."""
        tile_rows, columns = set(), set()
        for part in list(self.blocks) + list(self.positions.values()) + [self.embedding]:
            needs = part.step_needs() if hasattr(part, "step_needs") else {}
            tile_rows.update(needs.get("prefill_tile_rows", ()))
            columns.update(needs.get("token_columns", ()))
        return {"prefill_tile_rows": tile_rows, "token_columns": columns}

    def forward(self, step, cache):
        """Run the step's tokens through every call of the run order; logits [m, V] fp32 at step.logit_rows."""
        h = self.embedding.forward(step.token_ids, step)
        pending = None
        for i, call in enumerate(self.schedule):
            view = None
            if call.cache is not None:
                view = tuple(cache.view(c) for c in call.cache) if isinstance(call.cache, (tuple, list)) \
                    else cache.view(call.cache)
            block = self.blocks[call.block]
            if getattr(block, "first_norm", None) is not None:
                # an arrangement that says what it begins with is also told what takes its output: the
                # next block's first norm and first product (which may finish that norm between them),
                # or the last norm (which runs on the wanted rows only, as a kernel of its own)
                if i + 1 < len(self.schedule):
                    nxt = self.blocks[self.schedule[i + 1].block]
                    after = (nxt.first_norm, getattr(nxt, "first_product", None)) \
                        if getattr(nxt, "first_norm", None) is not None else None
                else:
                    after = (self.final_norm, None)
                h, pending = block.forward(h, pending, step, view, call.writes_cache, after=after)
            else:
                h, pending = block.forward(h, pending, step, view, call.writes_cache)
        if step.n_logit_rows == 0:
            return None
        x = self.final_norm.forward(h, pending, out_rows=step.logit_rows)
        return self.head.forward(x)
