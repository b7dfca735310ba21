"""What a mixer tells the cache manager it needs to keep between steps."""
from __future__ import annotations

import dataclasses
from typing import Optional, Tuple


@dataclasses.dataclass(frozen=True)
class PagedKVSpec:
    """Keys and values that grow by one row per token, kept in pages.

    window None: every key stays until the request ends. window w: a query at
    position p reads keys at positions p-w+1..p, and pages that lie wholly before
    that are given back while the request still runs.
    """
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class StateSpec:
    """State of fixed size per request: named tensors (name, shape, dtype name), zero at the start.

    The reference's LinearStateCache is of this kind: conv tail [C, K] bf16 and a
    recurrent matrix [Hv, dk, dv] fp32 per session (rollout/cache.py:340-356).
    """
    tensors: Tuple[Tuple[str, Tuple[int, ...], str], ...]
