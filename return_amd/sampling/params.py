"""Sampling options of a request and its stream of uniform numbers.

Names, defaults and meanings are the reference's (rollout/engine.py:13-21,
rollout/server.py:25-35): temperature <= 0 is greedy; top_k 0 and top_p 1.0 are
off; generation stops at max_new_tokens or when the output ends with one of the
stop_ids sequences (rollout/engine.py:49-57). The reference draws from the global
torch generator; here every request has its own stream, seeded from the engine's
seed and the request's, so that a request's tokens do not depend on what else is
in the batch.
"""
from __future__ import annotations

import dataclasses
import hashlib
import struct
from typing import List, Optional, Sequence


@dataclasses.dataclass
class SamplingParams:
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int = 0
    max_new_tokens: int = 32
    stop_ids: List[List[int]] = dataclasses.field(default_factory=list)
    seed: Optional[int] = None          # None: derived from the request's number in the engine

    def __post_init__(self):
        if self.max_new_tokens < 1:
            raise ValueError(f"max_new_tokens must be at least 1, got {self.max_new_tokens}")
        if not 0.0 <= self.top_p <= 1.0:
            raise ValueError(f"top_p must lie in [0, 1], got {self.top_p}")
        if self.top_k < 0:
            raise ValueError(f"top_k must be 0 (off) or positive, got {self.top_k}")
        self.stop_ids = [list(map(int, s)) for s in self.stop_ids]

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0


class UniformStream:
    """u_0, u_1, ... in [0, 1): a pure function of (engine seed, request seed, index)."""

    def __init__(self, engine_seed: int, request_seed: int):
        self._key = struct.pack("<qq", int(engine_seed), int(request_seed))
        self._i = 0

    def at(self, i: int) -> float:
        h = hashlib.blake2b(self._key + struct.pack("<q", i), digest_size=8).digest()
        return (int.from_bytes(h, "little") >> 40) / float(1 << 24)      # 24 bits: exact in fp32

    def next(self) -> float:
        u = self.at(self._i)
        self._i += 1
        return u


def ends_with_stop(output: Sequence[int], stop_ids: Sequence[Sequence[int]]) -> bool:
    """True if the output ends with one of the stop sequences (rollout/engine.py:52-56)."""
    for seq in stop_ids:
        n = len(seq)
        if n and len(output) >= n and list(output[-n:]) == list(seq):
            return True
    return False
