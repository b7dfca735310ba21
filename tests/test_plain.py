"""The plain implementation pinned by what fixes it beside the reference's text: library
routines it must reduce to, vectors of the reference's own tests, and invariants. Each check is
chosen so that a plausible mistake (sign, pairing, norm in the wrong place) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

from tests.plain import qwen3_plain as plain

torch.manual_seed(0)


def test_rms_norm_is_the_library_routine():
    x, w = torch.randn(5, 37), torch.rand(37) + 0.5
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (37,), w, 1e-5), atol=1e-6, rtol=1e-5)
    # eps sits inside the square root, with the mean (not the sum) of squares
    tiny = torch.full((1, 4), 1e-4)
    assert abs(float(plain.rms_norm(tiny, torch.ones(4), 1e-6)[0, 0]) - 1e-4 / math.sqrt(1e-8 + 1e-6)) < 1e-6
    # scale invariance for large inputs
    torch.testing.assert_close(plain.rms_norm(x * 1e3, w, 1e-6), plain.rms_norm(x * 1e4, w, 1e-6), atol=1e-4, rtol=1e-4)


def test_rope_pairs_halves_and_rotates_forward():
    """Half-split pairing (j, j + D/2) with o1 = x1 cos - x2 sin: the vector of the reference's own
    rotate (opd/test_parallel.py:16-22) for D = 4, one position."""
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0]]])
    ang = torch.tensor([[0.3, 1.1]])
    got = plain.rope_rotate(x, ang.cos(), ang.sin())[0, 0]
    want = torch.tensor([1 * math.cos(0.3) - 3 * math.sin(0.3), 2 * math.cos(1.1) - 4 * math.sin(1.1),
                         3 * math.cos(0.3) + 1 * math.sin(0.3), 4 * math.cos(1.1) + 2 * math.sin(1.1)])
    torch.testing.assert_close(got, want)
    # an interleaved pairing or a flipped sign gives a different vector
    inter = torch.tensor([1 * math.cos(0.3) - 2 * math.sin(0.3), 2 * math.cos(0.3) + 1 * math.sin(0.3)])
    assert not torch.allclose(got[:2], inter)


def test_rope_angles_and_invariants():
    cos, sin = plain.rope_angles(torch.arange(50), 16, 10000.0)
    assert cos.shape == (50, 8)
    # inv_freq[j] = theta^(-2j/D): position 1, pair j
    for j in (0, 3, 7):
        assert abs(float(cos[1, j]) - math.cos(10000.0 ** (-2 * j / 16))) < 1e-6
    x = torch.randn(50, 3, 16)
    r = plain.rope_rotate(x, cos, sin)
    torch.testing.assert_close(r[0], x[0])                                   # position 0 is the identity
    torch.testing.assert_close((r[..., :8] ** 2 + r[..., 8:] ** 2), (x[..., :8] ** 2 + x[..., 8:] ** 2),
                               atol=1e-5, rtol=1e-5)                         # each pair keeps its length
    # scores depend on distances only: shift all positions by 17
    q, k = torch.randn(6, 2, 16), torch.randn(6, 2, 16)
    def scores(shift):
        c, s = plain.rope_angles(torch.arange(shift, shift + 6), 16, 10000.0)
        return torch.einsum("qhd,khd->hqk", plain.rope_rotate(q, c, s), plain.rope_rotate(k, c, s))
    torch.testing.assert_close(scores(0), scores(17), atol=1e-4, rtol=1e-4)
    # partial rotary: the rest passes through (rollout/fused.py:69-70)
    c4, s4 = plain.rope_angles(torch.arange(50), 8, 10000.0)
    rp = plain.rope_rotate(x, c4, s4)
    torch.testing.assert_close(rp[..., 8:], x[..., 8:])


def test_attention_reduces_to_the_library_routine():
    T, Hq, Hkv, D = 11, 6, 2, 8
    q, k, v = torch.randn(T, Hq, D), torch.randn(T, Hkv, D), torch.randn(T, Hkv, D)
    pos = torch.arange(T)
    got = plain.causal_attention(q, k, v, pos, pos, D ** -0.5)
    kk, vv = k.repeat_interleave(3, 1), v.repeat_interleave(3, 1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kk.transpose(0, 1)[None],
                                          vv.transpose(0, 1)[None], is_causal=True, scale=D ** -0.5)
    torch.testing.assert_close(got, want[0].transpose(0, 1), atol=1e-5, rtol=1e-5)
    # one key: the output is its value; the first token sees only itself
    torch.testing.assert_close(got[0], vv[0], atol=1e-6, rtol=1e-6)


def test_gqa_maps_head_h_to_kv_head_h_div_g():
    """Distinct values per kv head (rollout/attention.py:65: off_kv_h = off_h // GROUP_SIZE)."""
    T, Hq, Hkv, D = 3, 6, 2, 4
    q, k = torch.randn(T, Hq, D), torch.randn(T, Hkv, D)
    v = torch.zeros(T, Hkv, D)
    v[:, 0], v[:, 1] = 1.0, 2.0
    out = plain.causal_attention(q, k, v, torch.arange(T), torch.arange(T), 0.5)
    assert torch.allclose(out[:, :3], torch.ones(T, 3, D)) and torch.allclose(out[:, 3:], 2 * torch.ones(T, 3, D))


def test_chunk_with_context_equals_whole():
    """Queries at positions 5.. over all keys give the rows of the whole computation (qpos semantics)."""
    T, D = 9, 8
    q, k, v = torch.randn(T, 2, D), torch.randn(T, 1, D), torch.randn(T, 1, D)
    pos = torch.arange(T)
    whole = plain.causal_attention(q, k, v, pos, pos, 0.3)
    part = plain.causal_attention(q[5:], k, v, pos[5:], pos, 0.3)
    torch.testing.assert_close(part, whole[5:])
    win = plain.causal_attention(q, k, v, pos, pos, 0.3, window=3)
    torch.testing.assert_close(win[:3], whole[:3])
    torch.testing.assert_close(win[8], plain.causal_attention(q[8:], k[6:], v[6:], pos[8:], pos[6:], 0.3)[0])


def test_swiglu_gate_first():
    x = torch.randn(4, 6)
    w = {"p.gate_proj.weight": torch.randn(10, 6), "p.up_proj.weight": torch.randn(10, 6),
         "p.down_proj.weight": torch.randn(6, 10)}
    want = (F.silu(x @ w["p.gate_proj.weight"].T) * (x @ w["p.up_proj.weight"].T)) @ w["p.down_proj.weight"].T
    torch.testing.assert_close(plain.swiglu(x, w, "p."), want, atol=1e-5, rtol=1e-5)


def test_values_are_not_normed_and_the_norm_removes_the_scale_of_q(folder_b):
    """V is untouched (rollout/monkey_patch/qwen3.py:31): scaling v_proj scales the attention output
    linearly; q passes a per-head norm (qwen3.py:29): scaling q_proj changes nothing."""
    cfg, w = plain.read_folder(folder_b)
    x = torch.randn(7, cfg["hidden_size"])
    pos = torch.arange(7)
    base = plain.attention_part(x, w, "model.layers.0.self_attn.", cfg, pos)
    w2 = dict(w)
    w2["model.layers.0.self_attn.v_proj.weight"] = 2 * w["model.layers.0.self_attn.v_proj.weight"]
    torch.testing.assert_close(plain.attention_part(x, w2, "model.layers.0.self_attn.", cfg, pos), 2 * base,
                               atol=1e-5, rtol=1e-4)
    w3 = dict(w)
    w3["model.layers.0.self_attn.q_proj.weight"] = 5 * w["model.layers.0.self_attn.q_proj.weight"]
    torch.testing.assert_close(plain.attention_part(x, w3, "model.layers.0.self_attn.", cfg, pos), base,
                               atol=1e-4, rtol=1e-3)      # the per-head norm removes the scale of q


def test_norm_sits_before_rotation(folder_b):
    """QK-norm first, rotation after it (rollout/monkey_patch/qwen3.py:29-30 norm q and k; the
    rotation happens later, inside the attention kernel, rollout/attention.py:89-96, 116-125). With a
    constant norm weight the two orders give the same vectors (a rotation keeps a head's mean square),
    so the weights here differ strongly along the head: then w * rotate(x) and rotate(w * x) differ,
    because the rotation mixes element j with element j + D/2, which carry different weights.
    The scores are written out here for one head from the norm, the angles and the rotation alone."""
    cfg, w = plain.read_folder(folder_b)
    pre = "model.layers.0.self_attn."
    D, eps, theta = cfg["head_dim"], cfg["rms_norm_eps"], cfg["rope_theta"]
    w = dict(w)
    w[pre + "q_norm.weight"] = torch.linspace(0.2, 3.0, D)
    w[pre + "k_norm.weight"] = torch.linspace(2.5, 0.3, D) ** 2
    T = 9
    x = torch.randn(T, cfg["hidden_size"])
    pos = torch.arange(40, 40 + T)                        # far from 0, so that the angles are large
    got = plain.attention_part(x, w, pre, cfg, pos)

    def by_hand(norm_first):
        q = (x @ w[pre + "q_proj.weight"].T).view(T, -1, D)
        k = (x @ w[pre + "k_proj.weight"].T).view(T, -1, D)
        v = (x @ w[pre + "v_proj.weight"].T).view(T, -1, D)
        inv = 1.0 / theta ** (torch.arange(0, D // 2).float() / (D // 2))
        ang = pos.float()[:, None] * inv[None, :]
        cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]

        def norm(t, weight):
            return t * torch.rsqrt((t * t).mean(-1, keepdim=True) + eps) * weight

        def rotate(t):
            a, b = t[..., :D // 2], t[..., D // 2:]
            return torch.cat([a * cos - b * sin, b * cos + a * sin], -1)
        if norm_first:
            q, k = rotate(norm(q, w[pre + "q_norm.weight"])), rotate(norm(k, w[pre + "k_norm.weight"]))
        else:
            q, k = norm(rotate(q), w[pre + "q_norm.weight"]), norm(rotate(k), w[pre + "k_norm.weight"])
        out = torch.zeros(T, q.shape[1], D)
        G = q.shape[1] // k.shape[1]
        for h in range(q.shape[1]):
            s = (q[:, h] @ k[:, h // G].T) * D ** -0.5
            s = s.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), float("-inf"))
            out[:, h] = s.softmax(-1) @ v[:, h // G]
        return out.reshape(T, -1) @ w[pre + "o_proj.weight"].T

    torch.testing.assert_close(got, by_hand(True), atol=1e-5, rtol=1e-4)
    wrong = by_hand(False)
    assert (got - wrong).abs().max() > 50 * (got - by_hand(True)).abs().max() + 1e-3   # the other order is another function


def test_whole_model_shapes_and_tying(folder_a, folder_b):
    for folder in (folder_a, folder_b):
        cfg, w = plain.read_folder(folder)
        toks = list(range(3, 20))
        lg = plain.logits(cfg, w, toks)
        assert lg.shape == (17, cfg["vocab_size"]) and torch.isfinite(lg).all()
        # causal: a prefix gives the same logits
        torch.testing.assert_close(plain.logits(cfg, w, toks[:9]), lg[:9], atol=1e-5, rtol=1e-4)
        # fp64 agrees with fp32
        cfg64, w64 = plain.read_folder(folder, torch.float64)
        torch.testing.assert_close(plain.logits(cfg64, w64, toks).float(), lg, atol=1e-5, rtol=1e-4)
    cfg, w = plain.read_folder(folder_a)
    assert "lm_head.weight" not in w and cfg["tie_word_embeddings"]


def test_sampling_rules():
    row = torch.tensor([2.0, 0.5, 1.0, -1.0, 0.0])
    p = plain.sample_distribution(row, 0.0)
    assert p.tolist() == [1, 0, 0, 0, 0]                                        # greedy is argmax
    assert plain.sample_distribution(row, 1.0, top_k=1).tolist() == [1, 0, 0, 0, 0]
    assert plain.sample_distribution(row, 1.0, top_p=0.0).tolist() == [1, 0, 0, 0, 0]   # first always stays
    torch.testing.assert_close(plain.sample_distribution(row, 0.5).float(), (row / 0.5).softmax(-1))
    p2 = plain.sample_distribution(row, 1.0, top_k=2)
    assert p2[1] == 0 and p2[3] == 0 and abs(float(p2[0] + p2[2]) - 1) < 1e-9
    # top_p keeps the token that crosses the threshold (rollout/model.py:52-54)
    full = row.double().softmax(-1)
    p3 = plain.sample_distribution(row, 1.0, top_p=float(full[0]) + 1e-3)
    assert (p3 > 0).sum() == 2 and p3[2] > 0
    assert abs(plain.chosen_logprob(row, 2) - float(row.log_softmax(-1)[2])) < 1e-6
