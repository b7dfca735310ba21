"""Token embedding (row gather, no scaling: rollout/monkey_patch/qwen3.py:73-75) and the
output head (rollout/monkey_patch/qwen3.py:151-156; tied to the embedding through
tie_weights(), rollout/engine_actor.py:46)."""
from __future__ import annotations

import torch

from .registry import register_part


class TokenEmbedding:
    @staticmethod
    def tensor_shapes(params):
        return {"weight": (params["vocab_size"], params["hidden_size"])}

    @staticmethod
    def random_init(params, role):
        return "embedding"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.vocab = int(params["vocab_size"])
        self.hidden = int(params["hidden_size"])
        self.table = rt.matrix(tensors["weight"])

    def forward(self, token_ids, step=None):
        """int32 ids [T] -> fp32 residual stream [T, H]. (step: the whole step, for an embedding that
        adds something of the positions; this one does not look at it.)"""
        h = self.rt.empty(token_ids.shape[0], self.hidden, dtype=torch.float32)
        self.rt.ops.embed(self.table, token_ids, h)
        return h


class LinearHead:
    """logits = x @ W^T in fp32. When tied, ``weight`` names the embedding table."""

    @staticmethod
    def tensor_shapes(params):
        return {"weight": (params["vocab_size"], params["hidden_size"])}

    @staticmethod
    def random_init(params, role):
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.weight = rt.product(rt.matrix(tensors["weight"]), out_dtype=torch.float32)

    def forward(self, x):
        return self.rt.ops.linear(x, self.weight, out_dtype=torch.float32)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
