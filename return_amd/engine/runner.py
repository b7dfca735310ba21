"""The model runner: a model, its cache and the ONE step function.

The reference has two entry points, prefill(reqs) for packed prompt pieces and
decode(reqs) for one token per request (rollout/model.py:184-294, 318-343); they
build the same tables and call the same forward. Here both are one step(): every
entry brings a request's next tokens, one or many, cut anywhere, and the logits
come back at the places asked for. Keys and values of the new tokens are written
first and attention then reads everything from the cache, as the reference does
(rollout/monkey_patch/qwen3.py:40-45), so whole prompts, portions and single
tokens take the same path.
"""
from __future__ import annotations

import os
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..cache.manager import CacheManager
from ..config.base import ModelConfig, load_config, lookup_architecture
from ..config.engine import EngineConfig
from ..models.decoder import Decoder
from ..parts.runtime import Runtime
from ..weights.loader import load_weights
from .batch import StepBatch, StepBuilder


class StepEntry:
    """One request's share of a step: its next tokens and the places (among them) whose logits are wanted."""
    __slots__ = ("request_id", "tokens", "want")

    def __init__(self, request_id, tokens: Sequence[int], want: Sequence[int] = ()):
        self.request_id = request_id
        self.tokens = list(tokens)
        self.want = list(want)


class ModelRunner:
    def __init__(self, model_dir: Optional[str] = None, *, config: Optional[ModelConfig] = None,
                 weights: Optional[Dict[str, torch.Tensor]] = None,
                 engine_config: Optional[EngineConfig] = None, ops=None):
        """Either model_dir (config.json + safetensors) or config + weights (name -> tensor)."""
        self.engine_config = ec = engine_config or EngineConfig()
        import return_amd.models  # noqa: F401  (fills the architecture registry)
        if model_dir is not None:
            config = load_config(model_dir)
        if config is None:
            raise ValueError("ModelRunner needs a model folder or a configuration")
        self.config = config
        _, build_spec = lookup_architecture(config.architecture)
        self.spec = build_spec(config)
        self.rt = Runtime(ec.device, ec.dtype, ops=ops)
        if weights is None:
            if model_dir is None:
                raise ValueError("ModelRunner got a configuration but no weights")
            weights = load_weights(model_dir, self.spec, device=self.rt.device)
        self.model = Decoder(self.spec, weights, self.rt)
        del weights
        self.cache = CacheManager(self.model.cache_layers(), ec.page_size, ec.max_token,
                                  ec.max_reside, self.rt.dtype, self.rt.device)
        self.builder = StepBuilder(self.cache, ec.max_step_tokens, ec.max_reside, self.rt.device)
        self.vocab_size = self.spec.vocab_size
        self.max_position = self.spec.max_position

    # ------------------------------------------------------------------ requests
    def add_request(self, request_id) -> None:
        self.cache.add_request(request_id)

    def free_request(self, request_id) -> None:
        self.cache.free_request(request_id)

    def is_live(self, request_id) -> bool:
        return request_id in self.cache.live

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run exactly the tokens the entries bring, as one batch, on top of the cache.

        Returns fp32 logits [number of wanted places, vocab] on the device, in the order
        of the entries and of each entry's ``want``; None if nothing is wanted.
        """
        if not entries:
            return None
        rows: List[int] = []
        at = 0
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"request {e.request_id!r} brings no tokens")
            for t in e.tokens:
                if not 0 <= int(t) < self.vocab_size:
                    raise ValueError(f"request {e.request_id!r}: token {t} outside the vocabulary of {self.vocab_size}")
            if e.request_id in self.cache.live and self.cache.seq_len(e.request_id) + n > self.max_position:
                raise ValueError(
                    f"request {e.request_id!r} would reach {self.cache.seq_len(e.request_id) + n} tokens, "
                    f"the model's max_position_embeddings is {self.max_position}")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise ValueError(f"request {e.request_id!r}: wanted place {w} is not among its {n} tokens")
                rows.append(at + int(w))
            at += n
        tables = self.cache.begin_step([(e.request_id, len(e.tokens)) for e in entries])
        try:
            batch = self.builder.build(tables, [e.tokens for e in entries], rows)
            with torch.no_grad():
                logits = self.model.forward(batch, self.cache)
        finally:
            self.cache.end_step()
        return logits

    def sample(self, logits: torch.Tensor, temperature, top_k, top_p, uniforms):
        """Choose a token per logits row on the device; returns (tokens, logprobs) as Python lists."""
        dev = self.rt.device
        m = logits.shape[0]
        packed = torch.tensor([list(map(float, temperature)), list(map(float, top_p)),
                               list(map(float, uniforms))], dtype=torch.float32).to(dev, non_blocking=True)
        ks = torch.tensor(list(map(int, top_k)), dtype=torch.int32).to(dev, non_blocking=True)
        out = self.rt.ops.sample(logits, packed[0].contiguous(), ks, packed[1].contiguous(),
                                 packed[2].contiguous())
        host = out.cpu()
        return host[:, 0].tolist(), host[:, 1].contiguous().view(torch.float32).tolist()
