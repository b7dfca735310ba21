"""Qwen3 dense decoder as a ModelSpec: which parts, which constants, which tensor names.

Architecture as the reference runs it (rollout/monkey_patch/qwen3.py): pre-RMSNorm
blocks (59-68) of GQA attention with per-head RMSNorm on q and k (25-31), rotary
positions over the whole head (121-127), full causal attention (130-132), SwiGLU
feed-forward without bias (20-22, 99-105), final RMSNorm (80), head tied to the
embedding when the config says so (rollout/engine_actor.py:46). Tensor names are
the attribute paths the reference touches plus ".weight".
"""
from __future__ import annotations

from ..config.base import register_architecture
from ..config.qwen3 import Qwen3Config
from ..parts.spec import BlockSpec, LayerCall, ModelSpec, PartSpec


def build_spec(cfg: Qwen3Config) -> ModelSpec:
    H, eps = cfg.hidden_size, cfg.rms_norm_eps
    norm = lambda name: PartSpec("rms_norm", {"size": H, "eps": eps, "offset": 0.0}, {"weight": name})
    blocks = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        attn = PartSpec(
            "attention",
            {"hidden_size": H, "num_heads": cfg.num_attention_heads,
             "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
             "scale": None, "window": None, "qk_norm_eps": eps, "position": "rotary"},
            {"q_proj": p + "self_attn.q_proj.weight", "k_proj": p + "self_attn.k_proj.weight",
             "v_proj": p + "self_attn.v_proj.weight", "o_proj": p + "self_attn.o_proj.weight",
             "q_norm": p + "self_attn.q_norm.weight", "k_norm": p + "self_attn.k_norm.weight"})
        mlp = PartSpec(
            "swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size},
            {"gate_proj": p + "mlp.gate_proj.weight", "up_proj": p + "mlp.up_proj.weight",
             "down_proj": p + "mlp.down_proj.weight"})
        blocks.append(BlockSpec.pre_norm(attn, mlp, norm(p + "input_layernorm.weight"),
                                         norm(p + "post_attention_layernorm.weight")))
    tied = cfg.tie_word_embeddings
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=H, vocab_size=cfg.vocab_size,
        max_position=cfg.max_position_embeddings,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size, "hidden_size": H},
                           {"weight": "model.embed_tokens.weight"}),
        positions={"rotary": PartSpec("rotary", {"head_dim": cfg.head_dim, "rotary_dim": cfg.head_dim,
                                                 "theta": cfg.rope_theta,
                                                 "max_position": cfg.max_position_embeddings})},
        blocks=blocks,
        schedule=[LayerCall(block=i, cache=i, writes_cache=True) for i in range(cfg.num_hidden_layers)],
        final_norm=norm("model.norm.weight"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "hidden_size": H, "tied": tied},
                      {"weight": "model.embed_tokens.weight" if tied else "lm_head.weight"}),
        ignorable=["lm_head.weight"] if tied else [])


register_architecture("Qwen3ForCausalLM", Qwen3Config, build_spec)
