"""Grouped-query attention over the paged cache, with optional per-head RMSNorm on
queries and keys and a position encoding that is handed in.

Order of operations as in rollout/monkey_patch/qwen3.py:25-56: q/k/v projections
(three GEMMs there, one fused GEMM here), view as heads, q_norm and k_norm over the
head dimension with one weight [D] for all heads, K and V of the new tokens written
to the cache (qwen3.py:40-42), attention of the new queries over everything the
cache then holds (qwen3.py:43-45), output projection. The reference rotates inside
the attention kernel when it reads (rollout/attention.py:89-96, 116-125) and keeps K
un-rotated in the pool; here K is rotated once when it is written, which gives the
same scores because a request's positions never change.
Scale is D^-0.5 unless given (rollout/attention.py:195). Query head h reads kv head
h // (Hq/Hkv) (rollout/attention.py:65).
"""
from __future__ import annotations

import torch

from ..cache.spec import PagedKVSpec
from .registry import register_part


class PagedAttention:
    @staticmethod
    def tensor_shapes(params):
        H, Hq, Hkv, D = (params["hidden_size"], params["num_heads"], params["num_kv_heads"],
                         params["head_dim"])
        shapes = {"q_proj": (Hq * D, H), "k_proj": (Hkv * D, H), "v_proj": (Hkv * D, H),
                  "o_proj": (H, Hq * D)}
        if params.get("qk_norm_eps") is not None:
            shapes["q_norm"] = (D,)
            shapes["k_norm"] = (D,)
        return shapes

    @staticmethod
    def random_init(params, role):
        return "norm" if role in ("q_norm", "k_norm") else "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.hidden = int(params["hidden_size"])
        self.n_q = int(params["num_heads"])
        self.n_kv = int(params["num_kv_heads"])
        self.d = int(params["head_dim"])
        if self.n_q % self.n_kv:
            raise ValueError(f"{self.n_q} query heads are not a multiple of {self.n_kv} kv heads")
        if hasattr(rt.ops, "check_attention_sizes"):      # sizes the kernels do not take are refused now, not at the first step
            rt.ops.check_attention_sizes(self.n_q, self.n_kv, self.d, rt.dtype)
        self.scale = float(params["scale"]) if params.get("scale") is not None else self.d ** -0.5
        self.window = params.get("window")
        self.eps = params.get("qk_norm_eps")
        self.position = (shared or {}).get(params["position"]) if params.get("position") else None
        if params.get("position") and self.position is None:
            raise KeyError(f"attention names position encoding {params['position']!r}, which the model lacks")
        self.w_qkv = rt.product(torch.cat([rt.matrix(tensors["q_proj"]), rt.matrix(tensors["k_proj"]),
                                           rt.matrix(tensors["v_proj"])], dim=0).contiguous())
        self.w_o = rt.product(rt.matrix(tensors["o_proj"]), residual=True)
        self.w_qn = rt.vector32(tensors["q_norm"]) if self.eps is not None else None
        self.w_kn = rt.vector32(tensors["k_norm"]) if self.eps is not None else None
        self._fusable = self.position is None or hasattr(self.position, "tables")
        # x goes into one product only and the output comes out of one: a norm before may be left to
        # the first (ScaledRows as x), a norm after may be finished inside the second (sink)
        self.first_product = (self.w_qkv, False)
        self.last_product = self.w_o

    def cache_spec(self):
        return PagedKVSpec(self.n_kv, self.d, self.window)

    def step_needs(self):
        """The q-tile list that the kernel set's attention reads for requests with more than one token."""
        ops = self.rt.ops
        rows = ops.prefill_tile_rows(self.d, self.rt.dtype) if hasattr(ops, "prefill_tile_rows") else None
        return {"prefill_tile_rows": set(rows)} if rows else {}

    def forward(self, x, step, cache, write_cache=True, sink=None):
        rt, ops = self.rt, self.rt.ops
        project = sink.project if sink is not None else ops.linear
        T, Hq, Hkv, D = x.shape[0], self.n_q, self.n_kv, self.d
        tables = step.groups[cache.group]
        qkv = ops.linear(x, self.w_qkv)                              # [T, (Hq+2Hkv)*D]
        if self._fusable and write_cache and hasattr(ops, "attention_qkv"):
            # every request brings one token: the kernel set may prepare q, k and v inside its attention
            cos, sin, rot = self.position.tables() if self.position is not None else (None, None, 0)
            o = rt.empty(T, Hq, D)
            if ops.attention_qkv(qkv, o, cache.k_pool, cache.v_pool, step, cache.group, self.scale,
                                 int(self.window) if self.window else 0, Hq, Hkv, D, self.w_qn, self.w_kn,
                                 float(self.eps) if self.eps is not None else 0.0, cos, sin, rot):
                return project(o.view(T, Hq * D), self.w_o)
        q = rt.empty(T, Hq, D)
        if self._fusable:
            cos, sin, rot = self.position.tables() if self.position is not None else (None, None, 0)
            ops.qkv_prepare(qkv, Hq, Hkv, D, self.w_qn, self.w_kn,
                            float(self.eps) if self.eps is not None else 0.0,
                            step.positions, cos, sin, rot, q,
                            cache.k_pool if write_cache else None,
                            cache.v_pool if write_cache else None, tables.slot_mapping)
        else:
            # a position encoding without rotary tables: norm, its own apply(), then the write
            k = rt.empty(T, Hkv, D)
            v = rt.empty(T, Hkv, D)
            ops.split_heads(qkv, Hq, Hkv, D, q, k, v)
            if self.eps is not None:
                ops.head_rmsnorm(q, self.w_qn, float(self.eps))
                ops.head_rmsnorm(k, self.w_kn, float(self.eps))
            # (a position encoding that asks for more of the step than positions, step_needs(), is given the step)
            if hasattr(self.position, "step_needs"):
                self.position.apply(q, k, step.positions, step)
            else:
                self.position.apply(q, k, step.positions)
            if write_cache:
                ops.kv_write(k, v, cache.k_pool, cache.v_pool, tables.slot_mapping)
        o = rt.empty(T, Hq, D)
        ops.attention(q, o, cache.k_pool, cache.v_pool, step, cache.group, self.scale,
                      int(self.window) if self.window else 0)
        return project(o.view(T, Hq * D), self.w_o)


register_part("mixer", "attention", PagedAttention)
