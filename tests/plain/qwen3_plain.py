"""Plain, slow implementation of the Qwen3 dense decoder, written from the
formulas of the reference (wenhaoli-xmu/ReTurn). Whole sequences, no cache,
one function per part, dense matrices everywhere.

It shares no code with ``return_amd``: it reads ``config.json`` as a raw dict
and ``model.safetensors`` with safetensors directly. Every function cites the
reference lines it restates. The reference runs these formulas in bf16 with
fp32 inside the kernels; here everything runs in one dtype (fp32 by default,
fp64 on request), which is what the engine's results are compared with.
"""
from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


# --------------------------------------------------------------------------
# folder reading (no product code)
# --------------------------------------------------------------------------

def read_folder(folder, dtype=torch.float32):
    """config.json as a dict, every tensor of model.safetensors upcast to dtype."""
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).to(dtype)
    return cfg, w


def head_dim_of(cfg):
    # rollout/monkey_patch/qwen3.py:117  getattr(cfg, "head_dim", hidden // heads)
    return cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------

def rms_norm(x, weight, eps, offset=0.0):
    """y = x * rsqrt(mean(x^2) + eps) * (offset + w) over the last axis.

    rollout/fused.py:6-17 (sum of squares / N + eps, 1/sqrt, times (OFFSET + w));
    Qwen3 calls it with offset 0.0: rollout/monkey_patch/qwen3.py:15-17.
    """
    ms = (x * x).sum(-1, keepdim=True) / x.shape[-1]
    return x * (1.0 / torch.sqrt(ms + eps)) * (offset + weight)


def rope_angles(positions, head_dim, theta, dtype=torch.float32):
    """cos and sin of position * inv_freq, [len(positions), head_dim/2].

    rollout/monkey_patch/qwen3.py:121-127: freqs = outer(pos, inv_freq), cos and
    sin of it times attention_scaling (1 for the default rope). inv_freq is read
    off the HF rotary module there; rollout/utils/test_decode.py:14-18 states it
    as 1 / base^(arange(0, HALF) / HALF), the same as base^(-2j/D).
    The angle is formed in fp32 as the reference does (fp32 pos times fp32
    inv_freq), then cos/sin are taken in the asked dtype.
    """
    half = head_dim // 2
    inv_freq = 1.0 / (float(theta) ** (torch.arange(0, half, dtype=torch.float32) / half))
    ang = torch.outer(positions.to(torch.float32), inv_freq)
    ang = ang.to(dtype)
    return ang.cos(), ang.sin()


def rope_rotate(x, cos, sin):
    """Half-split (neox) rotation of x [T, heads, D] by cos/sin [T, D/2].

    rollout/attention.py:10-25: o1 = x1*cos - x2*sin, o2 = x2*cos + x1*sin with
    x1 = x[..., :HALF], x2 = x[..., HALF:2*HALF]; the same rotate is written out
    in opd/test_parallel.py:16-22 and rollout/utils/test_decode.py:23-30.
    Qwen3 rotates the whole head (HALF = D/2): rollout/attention.py:147-153.
    """
    half = cos.shape[-1]
    c, s = cos[:, None, :], sin[:, None, :]
    x1, x2 = x[..., :half], x[..., half:2 * half]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s, x[..., 2 * half:]], dim=-1)


def causal_attention(q, k, v, q_pos, k_pos, scale, window=None):
    """Dense GQA attention. q [Tq, Hq, D] and k, v [Tk, Hkv, D] are already rotated.

    Scores, mask and softmax: rollout/attention.py:126-137 (keep where
    pos_q >= pos_k, scale, softmax over keys); query head h reads kv head
    h // G: rollout/attention.py:65; dense statement of the same thing:
    opd/test_parallel.py:38-43. ``window`` is not in the reference (it asserts
    there is none, rollout/monkey_patch/qwen3.py:130-132); with a window w a
    query at p sees keys in (p - w, p].
    """
    group = q.shape[1] // k.shape[1]
    kk = k.repeat_interleave(group, dim=1)
    vv = v.repeat_interleave(group, dim=1)
    score = torch.einsum("qhd,khd->hqk", q, kk) * scale
    hide = k_pos[None, :] > q_pos[:, None]
    if window is not None:
        hide = hide | (k_pos[None, :] <= q_pos[:, None] - window)
    score = score.masked_fill(hide[None], float("-inf"))
    return torch.einsum("hqk,khd->qhd", score.softmax(-1), vv)


def attention_part(x, w, prefix, cfg, positions, window=None):
    """Projections, per-head q/k norm, rotation, attention, output projection.

    rollout/monkey_patch/qwen3.py:25-56: q = q_norm(q_proj(x).view(.., -1, D)),
    k = k_norm(k_proj(x).view(..)), v = v_proj(x).view(..); the norm is over D
    with one weight [D] for all heads (rollout/fused.py:36-56); rotation happens
    after the norm, inside the attention kernel (rollout/attention.py:89-96,
    116-125); scale is D^-0.5 (rollout/attention.py:195).
    """
    d = head_dim_of(cfg)
    eps = cfg.get("rms_norm_eps", 1e-6)
    t = x.shape[0]
    q = (x @ w[prefix + "q_proj.weight"].T).view(t, -1, d)
    k = (x @ w[prefix + "k_proj.weight"].T).view(t, -1, d)
    v = (x @ w[prefix + "v_proj.weight"].T).view(t, -1, d)
    q = rms_norm(q, w[prefix + "q_norm.weight"], eps)
    k = rms_norm(k, w[prefix + "k_norm.weight"], eps)
    cos, sin = rope_angles(positions, d, cfg.get("rope_theta", 10000.0), dtype=x.dtype)
    q = rope_rotate(q, cos, sin)
    k = rope_rotate(k, cos, sin)
    o = causal_attention(q, k, v, positions, positions, d ** -0.5, window)
    return o.reshape(t, -1) @ w[prefix + "o_proj.weight"].T


def swiglu(x, w, prefix):
    """down(silu(gate(x)) * up(x)); silu(g) = g * sigmoid(g).

    rollout/monkey_patch/qwen3.py:20-22 with the fused weight cat([gate, up])
    (qwen3.py:103), rollout/fused.py:103-114 (first half is the gate).
    """
    g = x @ w[prefix + "gate_proj.weight"].T
    u = x @ w[prefix + "up_proj.weight"].T
    return ((g * torch.sigmoid(g)) * u) @ w[prefix + "down_proj.weight"].T


def block(h, w, i, cfg, positions, window=None):
    """Pre-norm block: h += attn(norm(h)); h += mlp(norm(h)).

    rollout/monkey_patch/qwen3.py:59-68.
    """
    eps = cfg.get("rms_norm_eps", 1e-6)
    p = f"model.layers.{i}."
    x = rms_norm(h, w[p + "input_layernorm.weight"], eps)
    h = h + attention_part(x, w, p + "self_attn.", cfg, positions, window)
    x = rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
    return h + swiglu(x, w, p + "mlp.")


def hidden_states(cfg, w, tokens, start_pos=0):
    """Embedding, all blocks, final norm. rollout/monkey_patch/qwen3.py:71-81."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(start_pos, start_pos + tokens.numel())
    h = w["model.embed_tokens.weight"][tokens]
    for i in range(cfg["num_hidden_layers"]):
        h = block(h, w, i, cfg, positions)
    return rms_norm(h, w["model.norm.weight"], cfg.get("rms_norm_eps", 1e-6))


def logits(cfg, w, tokens, start_pos=0):
    """Logits at every position of one whole sequence, [T, V].

    Head: rollout/monkey_patch/qwen3.py:151-156; tied embeddings through
    hf_model.tie_weights(): rollout/engine_actor.py:46.
    """
    h = hidden_states(cfg, w, tokens, start_pos)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) \
        else w["lm_head.weight"]
    return h @ head.T


# --------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------

def sample_distribution(row, temperature=1.0, top_k=0, top_p=1.0):
    """The distribution the reference draws from, as probabilities over the vocabulary.

    rollout/model.py:15-61: temperature <= 0 is argmax (23-26, 58); otherwise
    logits / temperature (32-34); keep the top_k largest (45-50); on the sorted
    kept values cum = softmax.cumsum, remove where cum > top_p shifted right by
    one so that the crossing token stays and the first always stays (51-55);
    softmax over what is left (56).
    """
    row = row.to(torch.float64)
    v = row.numel()
    if temperature <= 0:
        p = torch.zeros(v, dtype=torch.float64)
        p[int(row.argmax())] = 1.0
        return p
    x = row / temperature
    vals, idx = torch.sort(x, descending=True, stable=True)
    k = top_k if top_k > 0 else v
    vals = vals.masked_fill(torch.arange(v) >= k, float("-inf"))
    cum = vals.softmax(-1).cumsum(-1)
    remove = cum > top_p
    remove[1:] = remove[:-1].clone()
    remove[0] = False
    vals = vals.masked_fill(remove, float("-inf"))
    p = torch.zeros(v, dtype=torch.float64)
    p[idx] = vals.softmax(-1)
    return p


def chosen_logprob(row, token):
    """log_softmax of the raw (un-tempered) logits at the token. rollout/model.py:64-67."""
    return float(row.to(torch.float64).log_softmax(-1)[token])


def greedy_generate(cfg, w, prompt, n_new, stop_ids=()):
    """Greedy decoding by recomputing the whole sequence for every token.

    Stop rule: rollout/engine.py:49-57 (length, or the output ends with a stop sequence).
    """
    seq = list(prompt)
    out = []
    for _ in range(n_new):
        out.append(int(logits(cfg, w, seq)[-1].argmax()))
        seq.append(out[-1])
        if any(len(s) and out[-len(s):] == list(s) for s in stop_ids):
            break
    return out
