"""Options of the engine itself, as distinct from the model's config.json.

The reference keeps these as module constants (rollout/constant.py:1-5: PAGE_SIZE,
PREFILL_CHUNK, USE_CUDA_GRAPH) and two command-line options, --max-token (tokens in
the KV pool) and --max-reside (most live sessions) (rollout/server.py:90-91). The
names max_token and max_reside keep the reference's meaning.
"""
from __future__ import annotations

import dataclasses


@dataclasses.dataclass
class EngineConfig:
    dtype: str = "bfloat16"            # "bfloat16" | "float32": storage and matrix precision
    page_size: int = 16                # tokens per cache page
    max_token: int = 65536             # tokens the cache pool of every layer group can hold
    max_reside: int = 64               # most requests that are live at a time
    max_step_tokens: int = 8192        # token budget of one step (decoded tokens + prompt portions)
    prefill_chunk: int = 8192          # longest portion of one prompt in one step
    use_graphs: bool = True            # replay decode-only steps from captured HIP graphs (USE_CUDA_GRAPH of the reference)
    lookahead: bool = True             # launch every step before the sampled tokens of the one before it are read
    tune_products: bool = True         # measure at load which kernel forms each projection fastest at few rows
    defer_norms: bool = True           # steps of few rows: finish every RMSNorm inside the products around it (two kernels less per layer)
    check_invariants: bool = False     # debugging: after every step and every freed request the cache manager checks that no page
                                       # or slot is lost, held twice, or both free and held (the reference's audit wraps its cache's
                                       # methods the same way, rollout/utils/check_search_swap_timing.py:107-138)
    seed: int = 0                      # base seed of the sampling streams
    device: str = "cuda:0"

    def __post_init__(self):
        if self.dtype in ("bf16",):
            self.dtype = "bfloat16"
        if self.dtype in ("fp32", "float"):
            self.dtype = "float32"
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be bfloat16 or float32, got {self.dtype!r}")
        for name in ("page_size", "max_token", "max_reside", "max_step_tokens", "prefill_chunk"):
            if int(getattr(self, name)) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")
        if self.max_token < self.page_size:
            raise ValueError(f"max_token {self.max_token} holds less than one page of {self.page_size}")

    @property
    def num_pages(self) -> int:
        return self.max_token // self.page_size
