"""Each part of the model alone on the GPU, built through the registry with its own sizes and
constants, against the plain implementation's function for that part (32-bit and bfloat16)."""
import types

import pytest
import torch

import return_amd.models  # noqa: F401
from return_amd.cache import CacheManager
from return_amd.engine.batch import StepBuilder
from return_amd.parts import PartSpec, Runtime, part_class
from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"float32": dict(atol=3e-5, rtol=3e-5), "bfloat16": dict(atol=3e-2, rtol=3e-2)}


def close(got, want, dtype_name):
    """32-bit: element-wise. bfloat16: the norm-wise bound the reference's own kernel tests use
    (relative L2 error below 2e-2, rollout/utils/test_prefill_fwd_bwd.py:117), here 1e-2, and no
    element off by more than 3 % of the largest value."""
    if dtype_name == "float32":
        torch.testing.assert_close(got, want, **TOL["float32"])
        return
    rel = float((got - want).norm() / want.norm())
    assert rel < 1e-2, f"relative L2 error {rel}"
    assert float((got - want).abs().max()) < 3e-2 * float(want.abs().max()) + 1e-3


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def rt(request):
    return Runtime(DEV, request.param)


def test_rms_norm_part(rt):
    H = 200
    w = 1 + 0.1 * rnd(H, seed=1)
    part = part_class("norm", "rms_norm")({"size": H, "eps": 3e-5}, {"weight": w}, rt)
    h = rnd(9, H, seed=2, scale=4.0)
    delta = rnd(9, H, seed=3).to(rt.dtype)
    hd = h.to(DEV)
    out = part.forward(hd, delta.to(DEV))
    want_h = h + delta.float()
    torch.testing.assert_close(hd.cpu(), want_h)                         # the residual stream stays 32-bit
    torch.testing.assert_close(out.float().cpu(), plain.rms_norm(want_h, w, 3e-5), **TOL[rt.dtype_name])
    rows = torch.tensor([8, 0, 3], dtype=torch.int32, device=DEV)
    out2 = part.forward(hd, None, out_rows=rows)
    torch.testing.assert_close(out2.float().cpu(), plain.rms_norm(want_h[[8, 0, 3]], w, 3e-5), **TOL[rt.dtype_name])


def test_rotary_part(rt):
    part = part_class("position", "rotary")({"head_dim": 48, "rotary_dim": 32, "theta": 5e4, "max_position": 300},
                                            {}, rt)
    pos = torch.tensor([0, 1, 7, 299, 150], dtype=torch.int32)
    q, k = rnd(5, 3, 48, seed=4), rnd(5, 1, 48, seed=5)
    qd, kd = q.to(rt.dtype).to(DEV), k.to(rt.dtype).to(DEV)
    part.apply(qd, kd, pos.to(DEV))
    cos, sin = plain.rope_angles(pos, 32, 5e4)
    torch.testing.assert_close(qd.float().cpu(), plain.rope_rotate(q.to(rt.dtype).float(), cos, sin), **TOL[rt.dtype_name])
    torch.testing.assert_close(kd.float().cpu(), plain.rope_rotate(k.to(rt.dtype).float(), cos, sin), **TOL[rt.dtype_name])


def test_swiglu_part(rt):
    H, I = 72, 136
    w = {"gate_proj": rnd(I, H, seed=6, scale=0.2), "up_proj": rnd(I, H, seed=7, scale=0.2),
         "down_proj": rnd(H, I, seed=8, scale=0.2)}
    w = {k: v.to(rt.dtype) for k, v in w.items()}
    part = part_class("feed_forward", "swiglu")({"hidden_size": H, "intermediate_size": I}, w, rt)
    for T in (1, 5, 40):
        x = rnd(T, H, seed=9 + T).to(rt.dtype)
        y = part.forward(x.to(DEV))
        ref = plain.swiglu(x.float(), {"p." + k + ".weight": v.float() for k, v in w.items()}, "p.")
        close(y.float().cpu(), ref, rt.dtype_name)


def test_embedding_and_head_parts(rt):
    V, H = 131, 40
    table = rnd(V, H, seed=10).to(rt.dtype)
    emb = part_class("embedding", "token_embedding")({"vocab_size": V, "hidden_size": H}, {"weight": table}, rt)
    head = part_class("head", "linear_head")({"vocab_size": V, "hidden_size": H}, {"weight": table}, rt)
    ids = torch.tensor([0, 130, 5, 5], dtype=torch.int32, device=DEV)
    h = emb.forward(ids)
    assert h.dtype == torch.float32 and torch.equal(h.cpu(), table.float()[[0, 130, 5, 5]])
    x = rnd(3, H, seed=11).to(rt.dtype)
    lg = head.forward(x.to(DEV))
    assert lg.dtype == torch.float32
    torch.testing.assert_close(lg.cpu(), x.float() @ table.float().T, atol=1e-3, rtol=1e-3)


@pytest.mark.parametrize("window,qk_eps,scale", [(None, 1e-6, None), (11, None, 0.2)])
def test_attention_part(rt, window, qk_eps, scale):
    """The attention part over a real cache, in two portions and a decoded token, against the plain
    attention over the whole sequence (with and without QK-norm, window and an explicit scale)."""
    H, Hq, Hkv, D, T = 80, 6, 2, 32, 45
    names = {"q_proj": (Hq * D, H), "k_proj": (Hkv * D, H), "v_proj": (Hkv * D, H), "o_proj": (H, Hq * D)}
    w = {k: rnd(*s, seed=20 + i, scale=0.15).to(rt.dtype) for i, (k, s) in enumerate(names.items())}
    if qk_eps is not None:
        w["q_norm"], w["k_norm"] = (1 + 0.1 * rnd(D, seed=30)).to(rt.dtype), (1 + 0.1 * rnd(D, seed=31)).to(rt.dtype)
    pos = part_class("position", "rotary")({"head_dim": D, "theta": 1e4, "max_position": 128}, {}, rt)
    params = {"hidden_size": H, "num_heads": Hq, "num_kv_heads": Hkv, "head_dim": D, "scale": scale,
              "window": window, "qk_norm_eps": qk_eps, "position": "rotary"}
    part = part_class("mixer", "attention")(params, w, rt, {"rotary": pos})
    cache = CacheManager({0: part.cache_spec()}, 8, 64, 2, rt.dtype, DEV)
    builder = StepBuilder(cache, 64, 2, DEV)
    cache.add_request("r")
    x = rnd(T, H, seed=40).to(rt.dtype)
    outs = []
    for a, b in ((0, 30), (30, 44), (44, 45)):
        tables = cache.begin_step([("r", b - a)])
        step = builder.build(tables, [[0] * (b - a)], [])
        outs.append(part.forward(x[a:b].to(DEV).contiguous(), step, cache.view(0)))
        cache.end_step()
    got = torch.cat(outs).float().cpu()
    # plain: the same formulas on the whole sequence
    xf = x.float()
    p = torch.arange(T)
    q = (xf @ w["q_proj"].float().T).view(T, Hq, D)
    k = (xf @ w["k_proj"].float().T).view(T, Hkv, D)
    v = (xf @ w["v_proj"].float().T).view(T, Hkv, D)
    if qk_eps is not None:
        q, k = plain.rms_norm(q, w["q_norm"].float(), qk_eps), plain.rms_norm(k, w["k_norm"].float(), qk_eps)
    cos, sin = plain.rope_angles(p, D, 1e4)
    o = plain.causal_attention(plain.rope_rotate(q, cos, sin), plain.rope_rotate(k, cos, sin), v, p, p,
                               scale if scale is not None else D ** -0.5, window)
    want = o.reshape(T, -1) @ w["o_proj"].float().T
    close(got, want, rt.dtype_name)
    if window:
        assert len(cache.live["r"].pages[0]) <= -(-(window + 8) // 8) + 1     # the window gave pages back
