"""What a model is made of, as data: parts with their constants and tensor names,
blocks put together from parts, and the order in which the blocks run.

An architecture turns its configuration into a ModelSpec; the generic decoder
(return_amd/models/decoder.py) builds the parts from the registry and runs the
schedule. No part knows which model it is in.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional, Tuple


@dataclasses.dataclass
class PartSpec:
    """One part: its registry key, its sizes and constants, its checkpoint tensors."""
    kind: str
    params: Dict[str, Any] = dataclasses.field(default_factory=dict)
    tensors: Dict[str, str] = dataclasses.field(default_factory=dict)   # role -> tensor name


@dataclasses.dataclass
class BlockSpec:
    """One layer: its parts by name, and the arrangement (a class registered with
    return_amd.parts.block.register_arrangement) that builds and runs them.

    parts: name -> (category, PartSpec). Which names there are is the arrangement's business:
    "pre_norm" has mixer_norm, mixer, feed_forward_norm and feed_forward
    (h += mixer(mixer_norm(h)); h += feed_forward(feed_forward_norm(h))); another arrangement
    may have post-norms, no feed-forward or two mixers. Tensor names, shapes and random
    weights follow from the parts, whatever their names.
    """
    parts: Dict[str, Tuple[str, PartSpec]]
    arrangement: str = "pre_norm"

    @classmethod
    def pre_norm(cls, mixer: PartSpec, feed_forward: PartSpec, mixer_norm: PartSpec,
                 feed_forward_norm: PartSpec) -> "BlockSpec":
        return cls({"mixer_norm": ("norm", mixer_norm), "mixer": ("mixer", mixer),
                    "feed_forward_norm": ("norm", feed_forward_norm),
                    "feed_forward": ("feed_forward", feed_forward)}, "pre_norm")

    def part(self, name: str) -> PartSpec:
        if name not in self.parts:
            raise KeyError(f"arrangement {self.arrangement!r} wants a part named {name!r}; the block has "
                           f"{sorted(self.parts)}")
        return self.parts[name][1]


@dataclasses.dataclass
class LayerCall:
    """One entry of the run order.

    block:  index into ModelSpec.blocks; the same block may be called more than once.
    cache:  number of the cache layer this call uses (None if the mixer keeps nothing), or a
            tuple of numbers, one for each spec of a block whose cache_spec() is a tuple.
            Two calls may name the same cache layer; only calls with writes_cache=True
            append to it, the others read what an earlier call wrote in the same step.
    """
    block: int
    cache: Optional[object] = None
    writes_cache: bool = True


@dataclasses.dataclass
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_position: int
    embedding: PartSpec
    positions: Dict[str, PartSpec]      # named position encodings that mixers refer to
    blocks: List[BlockSpec]
    schedule: List[LayerCall]
    final_norm: PartSpec
    head: PartSpec
    ignorable: List[str] = dataclasses.field(default_factory=list)  # tensors a checkpoint may hold unused

    def all_parts(self):
        """(category, where it sits, PartSpec) of every part of the model."""
        yield "embedding", "embedding", self.embedding
        for name, p in self.positions.items():
            yield "position", f"positions[{name}]", p
        for i, b in enumerate(self.blocks):
            for name, (category, p) in b.parts.items():
                yield category, f"blocks[{i}].{name}", p
        yield "norm", "final_norm", self.final_norm
        yield "head", "head", self.head

    def expected_tensors(self):
        """tensor name -> (shape, how the random-weights mode draws it)."""
        from .registry import part_class
        out = {}
        for category, where, ps in self.all_parts():
            cls = part_class(category, ps.kind)
            shapes = cls.tensor_shapes(ps.params)
            for role, shape in shapes.items():
                if role not in ps.tensors:
                    raise KeyError(f"{where} ({ps.kind}): no tensor name given for role {role!r}")
                name = ps.tensors[role]
                draw = cls.random_init(ps.params, role) if hasattr(cls, "random_init") else "matrix"
                if name in out:
                    if tuple(out[name][0]) != tuple(shape):
                        raise ValueError(f"tensor {name} is used with shapes {out[name][0]} and {tuple(shape)}")
                    continue            # a shared tensor keeps the draw of its first use
                out[name] = (tuple(shape), draw)
        return out
