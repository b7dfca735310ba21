"""Generality of the parts: a toy architecture, defined here and registered through the public
registries only, with
  - a mixer that keeps state of its own (an exponential moving average per request),
  - a feed-forward with routing (top-1 of two experts, router logits in 32-bit),
  - a position encoding that is no rotation (keys scaled by their position),
  - an embedding that adds a learned vector per absolute position (it sees the step's positions),
  - a windowed attention layer (pages of its own, given back as the window passes),
  - a block arrangement with other parts than the framework's own (no feed-forward, a norm after
    the mixer as well as before it),
  - a run order that calls one block twice and lets one layer read another layer's cache.
It is built and stepped without a change to the framework's files and compared, in 32-bit,
with a dense whole-sequence evaluation written below. This toy is no model of anyone's."""
import dataclasses

import pytest
import torch

from return_amd.cache.spec import StateSpec
from return_amd.config import EngineConfig, ModelConfig, register_architecture
from return_amd.engine import ModelRunner
from return_amd.parts import BlockSpec, LayerCall, ModelSpec, PartSpec, register_part
from return_amd.parts.block import register_arrangement
from return_amd.weights import random_weights
from tests import trace_tools as tt
from tests.plain import qwen3_plain as plain


# ------------------------------------------------------------------ toy parts (torch on whatever device)
class EmaMixer:
    """s_t = decay * s_{t-1} + W x_t ; y_t = s_t. The state lives in the cache manager's slots."""

    @staticmethod
    def tensor_shapes(params):
        return {"w": (params["hidden_size"], params["hidden_size"])}

    @staticmethod
    def random_init(params, role):
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt, self.decay, self.h = rt, float(params["decay"]), int(params["hidden_size"])
        self.w = rt.matrix(tensors["w"])

    def cache_spec(self):
        return StateSpec((("s", (self.h,), "float32"),))

    def forward(self, x, step, cache, write_cache=True):
        u = self.rt.ops.linear(x, self.w).float()
        if step.all_decode:
            # one token each: everything on the device from the step's tables, no number of the host's
            # is baked in, so the step can be captured in a graph and replayed on other requests
            state = cache.tensors["s"]
            s = self.decay * state.index_select(0, step.slot_ids) + u
            state.index_copy_(0, step.slot_ids.long(), s)
            return s.to(x.dtype)
        y = torch.empty_like(u)
        for i in range(step.n_seqs):
            a, b = step.cu_q_host[i], step.cu_q_host[i + 1]
            s = cache.tensors["s"][step.slot_ids_host[i]].clone()
            for t in range(a, b):
                s = self.decay * s + u[t]
                y[t] = s
            cache.tensors["s"][step.slot_ids_host[i]] = s
        return y.to(x.dtype)


class RoutedFeedForward:
    """y = expert_e(x) for e = argmax(router(x)); expert = relu(x W1_e^T) W2_e^T."""

    @staticmethod
    def tensor_shapes(params):
        H, I, E = params["hidden_size"], params["intermediate_size"], params["experts"]
        shapes = {"router": (E, H)}
        for e in range(E):
            shapes[f"w1_{e}"] = (I, H)
            shapes[f"w2_{e}"] = (H, I)
        return shapes

    @staticmethod
    def random_init(params, role):
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt, self.E = rt, int(params["experts"])
        self.router = tensors["router"].to(rt.device).float()
        self.w1 = [rt.matrix(tensors[f"w1_{e}"]) for e in range(self.E)]
        self.w2 = [rt.matrix(tensors[f"w2_{e}"]) for e in range(self.E)]

    def forward(self, x, step=None):
        choice = (x.float() @ self.router.t()).argmax(-1)
        if step is not None and step.all_decode:
            # few rows: every expert on every row and a choice on the device (nothing waits for the
            # device, so the step can be captured in a graph)
            y = torch.zeros_like(x)
            for e in range(self.E):
                out = self.rt.ops.linear(self.rt.ops.linear(x, self.w1[e]).relu().contiguous(), self.w2[e])
                y = torch.where((choice == e)[:, None], out, y)
            return y
        y = torch.zeros_like(x)
        for e in range(self.E):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                hid = self.rt.ops.linear(x[rows].contiguous(), self.w1[e]).relu()
                y[rows] = self.rt.ops.linear(hid.contiguous(), self.w2[e])
        return y


class KeyFade:
    """Not a rotation: keys are scaled by 1 / (1 + position / horizon). No tables(), so the
    attention part takes its general path (norm, apply(), cache write)."""

    @staticmethod
    def tensor_shapes(params):
        return {}

    def __init__(self, params, tensors, rt, shared=None):
        self.horizon = float(params["horizon"])

    def apply(self, q, k, positions):
        if k is not None:
            k.mul_((1.0 / (1.0 + positions.float() / self.horizon)).to(k.dtype)[:, None, None])


class PositionedEmbedding:
    """table[token] + place[position]: an absolute position encoding, added where the tokens come in."""

    @staticmethod
    def tensor_shapes(params):
        return {"table": (params["vocab_size"], params["hidden_size"]),
                "place": (params["max_position"], params["hidden_size"])}

    @staticmethod
    def random_init(params, role):
        return "embedding"

    def __init__(self, params, tensors, rt, shared=None):
        self.table = tensors["table"].to(rt.device).float()
        self.place = tensors["place"].to(rt.device).float()

    def forward(self, token_ids, step):
        return (self.table.index_select(0, token_ids) + self.place.index_select(0, step.positions)).contiguous()


class MixerBetweenNorms:
    """h += after(mixer(before(h))): three parts, none of them a feed-forward."""

    def __init__(self, spec, build):
        self.before, self.mixer, self.after = build("before"), build("mixer"), build("after")

    def cache_spec(self):
        return self.mixer.cache_spec()

    def forward(self, h, pending, step, cache, write_cache=True):
        x = self.before.forward(h, pending)
        a = self.mixer.forward(x, step, cache, write_cache)
        return h, self.after.forward(a.float().contiguous())


register_part("mixer", "toy_ema", EmaMixer)
register_part("embedding", "toy_positioned", PositionedEmbedding)
register_arrangement("toy_mixer_between_norms", MixerBetweenNorms)
register_part("feed_forward", "toy_routed", RoutedFeedForward)
register_part("position", "toy_key_fade", KeyFade)


@dataclasses.dataclass(frozen=True)
class ToyConfig(ModelConfig):
    vocab_size: int
    hidden_size: int
    heads: int
    kv_heads: int
    head_dim: int
    intermediate_size: int
    window: int
    decay: float
    max_position_embeddings: int
    eps: float = 1e-5


def toy_spec(c: ToyConfig) -> ModelSpec:
    H = c.hidden_size
    norm = lambda name: PartSpec("rms_norm", {"size": H, "eps": c.eps}, {"weight": name})

    def attn(i, window, position, qk_eps):
        p = f"blocks.{i}.attn."
        t = {"q_proj": p + "q", "k_proj": p + "k", "v_proj": p + "v", "o_proj": p + "o"}
        if qk_eps is not None:
            t.update(q_norm=p + "qn", k_norm=p + "kn")
        return PartSpec("attention", {"hidden_size": H, "num_heads": c.heads, "num_kv_heads": c.kv_heads,
                                      "head_dim": c.head_dim, "scale": None, "window": window,
                                      "qk_norm_eps": qk_eps, "position": position}, t)

    def mlp(i):
        p = f"blocks.{i}.mlp."
        return PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c.intermediate_size},
                        {"gate_proj": p + "g", "up_proj": p + "u", "down_proj": p + "d"})

    routed = PartSpec("toy_routed", {"hidden_size": H, "intermediate_size": c.intermediate_size, "experts": 2},
                      dict([("router", "blocks.1.ffn.router")] +
                           [(f"w{k}_{e}", f"blocks.1.ffn.w{k}_{e}") for k in (1, 2) for e in (0, 1)]))
    blocks = [
        BlockSpec.pre_norm(attn(0, None, "rotary", c.eps), mlp(0), norm("blocks.0.n1"), norm("blocks.0.n2")),
        BlockSpec.pre_norm(PartSpec("toy_ema", {"hidden_size": H, "decay": c.decay}, {"w": "blocks.1.ema.w"}), routed,
                           norm("blocks.1.n1"), norm("blocks.1.n2")),
        BlockSpec.pre_norm(attn(2, c.window, "fade", None), mlp(2), norm("blocks.2.n1"), norm("blocks.2.n2")),
        BlockSpec.pre_norm(attn(3, None, "rotary", c.eps), mlp(3), norm("blocks.3.n1"), norm("blocks.3.n2")),
        BlockSpec({"before": ("norm", norm("blocks.4.before")),
                   "mixer": ("mixer", PartSpec("toy_ema", {"hidden_size": H, "decay": 0.5}, {"w": "blocks.4.ema.w"})),
                   "after": ("norm", norm("blocks.4.after"))}, "toy_mixer_between_norms"),
    ]
    schedule = [LayerCall(0, cache=0), LayerCall(1, cache=1), LayerCall(2, cache=2),
                LayerCall(0, cache=3),                           # block 0 a second time, a cache of its own
                LayerCall(3, cache=0, writes_cache=False),       # block 3 reads what the first call wrote
                LayerCall(4, cache=4)]
    return ModelSpec(
        architecture=c.architecture, hidden_size=H, vocab_size=c.vocab_size, max_position=c.max_position_embeddings,
        embedding=PartSpec("toy_positioned", {"vocab_size": c.vocab_size, "hidden_size": H,
                                              "max_position": c.max_position_embeddings},
                           {"table": "embed", "place": "embed_place"}),
        positions={"rotary": PartSpec("rotary", {"head_dim": c.head_dim, "rotary_dim": c.head_dim // 2,
                                                 "theta": 500.0, "max_position": c.max_position_embeddings}),
                   "fade": PartSpec("toy_key_fade", {"horizon": 40.0})},
        blocks=blocks, schedule=schedule, final_norm=norm("final_norm"),
        head=PartSpec("linear_head", {"vocab_size": c.vocab_size, "hidden_size": H}, {"weight": "head"}))


register_architecture("ToyForTests", ToyConfig, toy_spec)

TOY = dict(architectures=["ToyForTests"], vocab_size=97, hidden_size=48, heads=4, kv_heads=2, head_dim=16,
           intermediate_size=40, window=9, decay=0.8, max_position_embeddings=128, eps=1e-5)


# ------------------------------------------------------------------ dense whole-sequence evaluation
def toy_plain_logits(c, w, tokens):
    T, D = len(tokens), c.head_dim
    pos = torch.arange(T)
    h = w["embed"][torch.tensor(tokens)] + w["embed_place"][:T]
    kv0 = {}

    def attention(x, i, window, kind, qk_eps, keep=None, reuse=None):
        p = f"blocks.{i}.attn."
        q = (x @ w[p + "q"].T).view(T, -1, D)
        k = (x @ w[p + "k"].T).view(T, -1, D)
        v = (x @ w[p + "v"].T).view(T, -1, D)
        if qk_eps is not None:
            q, k = plain.rms_norm(q, w[p + "qn"], qk_eps), plain.rms_norm(k, w[p + "kn"], qk_eps)
        if kind == "rotary":
            cos, sin = plain.rope_angles(pos, D // 2, 500.0)
            q, k = plain.rope_rotate(q, cos, sin), plain.rope_rotate(k, cos, sin)
        else:
            k = k * (1.0 / (1.0 + pos.float() / 40.0))[:, None, None]
        if keep is not None:
            kv0[keep] = (k, v)
        if reuse is not None:
            k, v = kv0[reuse]
        o = plain.causal_attention(q, k, v, pos, pos, D ** -0.5, window)
        return o.reshape(T, -1) @ w[p + "o"].T

    def swiglu(x, i):
        p = f"blocks.{i}.mlp."
        g = x @ w[p + "g"].T
        return (g * torch.sigmoid(g) * (x @ w[p + "u"].T)) @ w[p + "d"].T

    def block0(h, keep):
        h = h + attention(plain.rms_norm(h, w["blocks.0.n1"], c.eps), 0, None, "rotary", c.eps, keep=keep)
        return h + swiglu(plain.rms_norm(h, w["blocks.0.n2"], c.eps), 0)

    h = block0(h, "first")
    x = plain.rms_norm(h, w["blocks.1.n1"], c.eps)
    u, s, ys = x @ w["blocks.1.ema.w"].T, torch.zeros(c.hidden_size), []
    for t in range(T):
        s = c.decay * s + u[t]
        ys.append(s)
    h = h + torch.stack(ys)
    x = plain.rms_norm(h, w["blocks.1.n2"], c.eps)
    choice = (x @ w["blocks.1.ffn.router"].T).argmax(-1)
    y = torch.zeros_like(x)
    for e in (0, 1):
        m = choice == e
        y[m] = (x[m] @ w[f"blocks.1.ffn.w1_{e}"].T).relu() @ w[f"blocks.1.ffn.w2_{e}"].T
    h = h + y
    h = h + attention(plain.rms_norm(h, w["blocks.2.n1"], c.eps), 2, c.window, "fade", None)
    h = h + swiglu(plain.rms_norm(h, w["blocks.2.n2"], c.eps), 2)
    h = block0(h, None)
    h = h + attention(plain.rms_norm(h, w["blocks.3.n1"], c.eps), 3, None, "rotary", c.eps, reuse="first")
    h = h + swiglu(plain.rms_norm(h, w["blocks.3.n2"], c.eps), 3)
    u, s, ys = plain.rms_norm(h, w["blocks.4.before"], c.eps) @ w["blocks.4.ema.w"].T, torch.zeros(c.hidden_size), []
    for t in range(T):
        s = 0.5 * s + u[t]
        ys.append(s)
    h = h + plain.rms_norm(torch.stack(ys), w["blocks.4.after"], c.eps)
    return plain.rms_norm(h, w["final_norm"], c.eps) @ w["head"].T


def run_toy(device, ops):
    cfg = ToyConfig.from_dict(TOY)
    spec = toy_spec(cfg)
    weights = random_weights(spec, seed=4, std=0.08, norm_jitter=0.05, dtype="float32")
    reqs = {rid: tt.random_tokens(cfg.vocab_size, n, seed=ord(rid)) for rid, n in
            {"a": 40, "b": 7, "c": 23, "d": 61, "e": 1}.items()}
    want = {rid: toy_plain_logits(cfg, weights, toks) for rid, toks in reqs.items()}
    for cut in (tt.whole, tt.portions, tt.mixed):
        steps = cut(reqs)
        ec = EngineConfig(dtype="float32", page_size=4, max_token=tt.peak_tokens(steps), max_reside=4,
                          max_step_tokens=256, prefill_chunk=256, device=device)
        runner = ModelRunner(config=cfg, weights={k: v.clone() for k, v in weights.items()},
                             engine_config=ec, ops=ops)
        cache = runner.cache
        assert len(cache.groups) == 2 and len(cache.state_layers) == 2      # full, windowed; two state layers
        got = tt.run_in_process(runner, steps)
        for rid, toks in reqs.items():
            for p in range(len(toks)):
                torch.testing.assert_close(got[(rid, p)], want[rid][p], atol=3e-4, rtol=3e-4,
                                           msg=lambda m: f"{cut.__name__} request {rid} position {p}: {m}")
        windowed = [g for g in cache.groups if g.spec.window][0]
        assert all(g.pages.in_use() == 0 for g in cache.groups) and windowed.spec.window == 9


def test_toy_architecture_on_cpu_stand_in():
    from tests.torch_ops import TorchOps
    run_toy("cpu", TorchOps())


@pytest.mark.gpu
def test_toy_architecture_on_gpu():
    run_toy("cuda:0", None)


def generate_toy(device, ops, **options):
    """Greedy generation of the toy through Engine.generate against the dense evaluation: the state
    of the toy's mixers advances once per token, whichever way the engine runs its decode steps."""
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    cfg = ToyConfig.from_dict(TOY)
    weights = random_weights(toy_spec(cfg), seed=4, std=0.08, norm_jitter=0.05, dtype="float32")
    prompts = [tt.random_tokens(cfg.vocab_size, n, seed=70 + n) for n in (9, 1, 30, 17, 4)]
    new = 24
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(new):
            toks.append(int(toy_plain_logits(cfg, weights, toks)[-1].argmax()))
        want.append(toks[len(p):])
    ec = EngineConfig(dtype="float32", page_size=4, max_token=512, max_reside=3, max_step_tokens=32,
                      prefill_chunk=16, device=device, check_invariants=True, **options)
    runner = ModelRunner(config=cfg, weights={k: v.clone() for k, v in weights.items()}, engine_config=ec, ops=ops)
    got = Engine(runner=runner).generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=new))
    assert [r.output_ids for r in got] == want
    return runner


def test_toy_generation_on_cpu_stand_in():
    from tests.torch_ops import TorchOps
    generate_toy("cpu", TorchOps(), lookahead=True)


@pytest.mark.gpu
@pytest.mark.parametrize("use_graphs", [True, False])
@pytest.mark.parametrize("lookahead", [True, False])
def test_toy_generation_on_gpu(use_graphs, lookahead):
    """With graphs, the warm-up and the capture of every new (batch size, context bucket) must leave the
    requests' state alone: a step that ran twice would advance the moving averages twice."""
    runner = generate_toy("cuda:0", None, use_graphs=use_graphs, lookahead=lookahead)
    assert bool(runner._graphs) == use_graphs


# ------------------------------------------------------------------ a model whose mixers keep state only
def state_only_spec(c: ToyConfig) -> ModelSpec:
    """Two layers of the moving-average mixer and nothing else that keeps anything: no attention, so
    the cache manager has no paged group at all, only state slots."""
    H = c.hidden_size
    norm = lambda name: PartSpec("rms_norm", {"size": H, "eps": c.eps}, {"weight": name})
    mlp = lambda i: PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c.intermediate_size},
                             {"gate_proj": f"blocks.{i}.g", "up_proj": f"blocks.{i}.u", "down_proj": f"blocks.{i}.d"})
    ema = lambda i, decay: PartSpec("toy_ema", {"hidden_size": H, "decay": decay}, {"w": f"blocks.{i}.w"})
    blocks = [BlockSpec.pre_norm(ema(i, d), mlp(i), norm(f"blocks.{i}.n1"), norm(f"blocks.{i}.n2"))
              for i, d in enumerate((c.decay, 0.4))]
    return ModelSpec(
        architecture=c.architecture, hidden_size=H, vocab_size=c.vocab_size, max_position=c.max_position_embeddings,
        embedding=PartSpec("token_embedding", {"vocab_size": c.vocab_size, "hidden_size": H}, {"weight": "embed"}),
        positions={}, blocks=blocks, schedule=[LayerCall(0, cache=0), LayerCall(1, cache=1)],
        final_norm=norm("final_norm"),
        head=PartSpec("linear_head", {"vocab_size": c.vocab_size, "hidden_size": H}, {"weight": "head"}))


@dataclasses.dataclass(frozen=True)
class StateOnlyConfig(ToyConfig):
    pass


register_architecture("ToyStateOnlyForTests", StateOnlyConfig, state_only_spec)


def state_only_logits(c, w, tokens):
    T = len(tokens)
    h = w["embed"][torch.tensor(tokens)]
    for i, decay in enumerate((c.decay, 0.4)):
        u = plain.rms_norm(h, w[f"blocks.{i}.n1"], c.eps) @ w[f"blocks.{i}.w"].T
        s, ys = torch.zeros(c.hidden_size), []
        for t in range(T):
            s = decay * s + u[t]
            ys.append(s)
        h = h + torch.stack(ys)
        x = plain.rms_norm(h, w[f"blocks.{i}.n2"], c.eps)
        g = x @ w[f"blocks.{i}.g"].T
        h = h + (g * torch.sigmoid(g) * (x @ w[f"blocks.{i}.u"].T)) @ w[f"blocks.{i}.d"].T
    return plain.rms_norm(h, w["final_norm"], c.eps) @ w["head"].T


def run_state_only(device, ops, **options):
    """Replay under every cut, then greedy generation through the entry point: a model without a single
    page of cache goes through admission, the step's tables, the step function and the scheduler."""
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    cfg = StateOnlyConfig.from_dict(dict(TOY, architectures=["ToyStateOnlyForTests"]))
    weights = random_weights(state_only_spec(cfg), seed=6, std=0.08, norm_jitter=0.05, dtype="float32")
    reqs = {rid: tt.random_tokens(cfg.vocab_size, n, seed=ord(rid)) for rid, n in
            {"a": 40, "b": 7, "c": 23, "d": 61, "e": 1}.items()}
    want = {rid: state_only_logits(cfg, weights, toks) for rid, toks in reqs.items()}
    for cut in (tt.whole, tt.portions, tt.mixed):
        steps = cut(reqs)
        ec = EngineConfig(dtype="float32", page_size=4, max_token=64, max_reside=4, max_step_tokens=256,
                          prefill_chunk=256, device=device, check_invariants=True)
        runner = ModelRunner(config=cfg, weights={k: v.clone() for k, v in weights.items()}, engine_config=ec, ops=ops)
        assert len(runner.cache.groups) == 0 and len(runner.cache.state_layers) == 2
        got = tt.run_in_process(runner, steps)
        for rid, toks in reqs.items():
            for p in range(len(toks)):
                torch.testing.assert_close(got[(rid, p)], want[rid][p], atol=3e-4, rtol=3e-4,
                                           msg=lambda m: f"{cut.__name__} request {rid} position {p}: {m}")
        assert runner.cache.free_slots() == 4
    prompts = [tt.random_tokens(cfg.vocab_size, n, seed=90 + n) for n in (9, 1, 30, 17, 4)]
    new = 20
    expect = []
    for p in prompts:
        toks = list(p)
        for _ in range(new):
            toks.append(int(state_only_logits(cfg, weights, toks)[-1].argmax()))
        expect.append(toks[len(p):])
    # max_token is as small as it may be: nothing here is held in pages, so requests of any length are let in
    ec = EngineConfig(dtype="float32", page_size=4, max_token=4, max_reside=3, max_step_tokens=32, prefill_chunk=16,
                      device=device, check_invariants=True, **options)
    runner = ModelRunner(config=cfg, weights={k: v.clone() for k, v in weights.items()}, engine_config=ec, ops=ops)
    out = Engine(runner=runner).generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=new))
    assert [r.output_ids for r in out] == expect
    assert not runner.cache.live and runner.cache.free_slots() == 3
    return runner


def test_state_only_model_on_cpu_stand_in():
    from tests.torch_ops import TorchOps
    run_state_only("cpu", TorchOps(), lookahead=True)


@pytest.mark.gpu
@pytest.mark.parametrize("use_graphs", [True, False])
def test_state_only_model_on_gpu(use_graphs):
    runner = run_state_only("cuda:0", None, use_graphs=use_graphs)
    assert bool(runner._graphs) == use_graphs


# ------------------------------------------------------------------ a mixer that keeps two things, a weight with a law
# of its own, and a position encoding with a second axis
class ConvThenAttention:
    """A short causal convolution over the tokens (taps that are positive and sum to one), then attention over
    the paged cache: the layer keeps paged keys and values AND a state of fixed size, the last K - 1 inputs."""

    @staticmethod
    def tensor_shapes(params):
        from return_amd.parts.attention import PagedAttention
        return dict(PagedAttention.tensor_shapes(params), taps=(params["taps"],))

    @staticmethod
    def random_init(params, role):
        from return_amd.parts.attention import PagedAttention
        if role == "taps":
            # a law of its own: no normal draw gives positive numbers that sum to one
            draw = lambda shape, gen: torch.randn(*shape, generator=gen).softmax(-1)
            draw.keep_dtype = True                         # and they stay 32-bit in a bfloat16 model folder
            return draw
        return PagedAttention.random_init(params, role)

    def __init__(self, params, tensors, rt, shared=None):
        from return_amd.parts.attention import PagedAttention
        self.rt, self.h, self.k = rt, int(params["hidden_size"]), int(params["taps"])
        self.attention = PagedAttention(params, {r: t for r, t in tensors.items() if r != "taps"}, rt, shared)
        assert tensors["taps"].dtype == torch.float32
        self.taps = tensors["taps"].to(rt.device).float()             # taps[j] weighs the input j tokens back

    def cache_spec(self):
        return (self.attention.cache_spec(), StateSpec((("tail", (self.k - 1, self.h), "float32"),)))

    def step_needs(self):
        return self.attention.step_needs()

    def forward(self, x, step, cache, write_cache=True):
        paged, state = cache
        tail_of = state.tensors["tail"]
        back = self.taps.flip(0)[None, :, None]                       # oldest input first
        if step.all_decode:
            window = torch.cat([tail_of.index_select(0, step.slot_ids), x.float()[:, None, :]], dim=1)
            y = (window * back).sum(1)
            if write_cache:
                tail_of.index_copy_(0, step.slot_ids.long(), window[:, 1:].contiguous())
        else:
            y = torch.empty(x.shape, dtype=torch.float32, device=x.device)
            for i in range(step.n_seqs):
                a, b = step.cu_q_host[i], step.cu_q_host[i + 1]
                slot = step.slot_ids_host[i]
                seq = torch.cat([tail_of[slot], x[a:b].float()], dim=0)
                y[a:b] = (seq.unfold(0, self.k, 1) * self.taps.flip(0)[None, None, :]).sum(-1)
                if write_cache:
                    tail_of[slot] = seq[-(self.k - 1):]
        return self.attention.forward(y.to(x.dtype).contiguous(), step, paged, write_cache)


class GridFade:
    """A position encoding of two axes: keys fade with the token's position AND with its row on a grid, an
    integer that the request brings with every token (the step's token column "row")."""

    @staticmethod
    def tensor_shapes(params):
        return {}

    def __init__(self, params, tensors, rt, shared=None):
        self.along, self.down = float(params["along"]), float(params["down"])

    def step_needs(self):
        return {"token_columns": ("row",)}

    def apply(self, q, k, positions, step):
        if k is not None:
            row = step.token_columns["row"]
            fade = 1.0 / ((1.0 + positions.float() / self.along) * (1.0 + row.float() / self.down))
            k.mul_(fade.to(k.dtype)[:, None, None])


register_part("mixer", "toy_conv_then_attention", ConvThenAttention)
register_part("position", "toy_grid_fade", GridFade)


@dataclasses.dataclass(frozen=True)
class HybridConfig(ToyConfig):
    taps: int = 3


def hybrid_spec(c: HybridConfig) -> ModelSpec:
    H = c.hidden_size
    norm = lambda name: PartSpec("rms_norm", {"size": H, "eps": c.eps}, {"weight": name})
    mlp = lambda i: PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c.intermediate_size},
                             {"gate_proj": f"blocks.{i}.g", "up_proj": f"blocks.{i}.u", "down_proj": f"blocks.{i}.d"})

    def attn(i, kind, position, **more):
        names = {r: f"blocks.{i}.{r}" for r in ("q_proj", "k_proj", "v_proj", "o_proj") + tuple(more.pop("roles", ()))}
        return PartSpec(kind, dict({"hidden_size": H, "num_heads": c.heads, "num_kv_heads": c.kv_heads,
                                    "head_dim": c.head_dim, "scale": None, "window": None, "qk_norm_eps": None,
                                    "position": position}, **more), names)
    blocks = [BlockSpec.pre_norm(attn(0, "toy_conv_then_attention", "grid", taps=c.taps, roles=("taps",)), mlp(0),
                                 norm("blocks.0.n1"), norm("blocks.0.n2")),
              BlockSpec.pre_norm(attn(1, "attention", "grid"), mlp(1), norm("blocks.1.n1"), norm("blocks.1.n2"))]
    return ModelSpec(
        architecture=c.architecture, hidden_size=H, vocab_size=c.vocab_size, max_position=c.max_position_embeddings,
        embedding=PartSpec("token_embedding", {"vocab_size": c.vocab_size, "hidden_size": H}, {"weight": "embed"}),
        positions={"grid": PartSpec("toy_grid_fade", {"along": 40.0, "down": 3.0})}, blocks=blocks,
        # the first call names two cache layers, one for each thing its mixer keeps
        schedule=[LayerCall(0, cache=(0, 1)), LayerCall(1, cache=2)], final_norm=norm("final_norm"),
        head=PartSpec("linear_head", {"vocab_size": c.vocab_size, "hidden_size": H}, {"weight": "head"}))


register_architecture("ToyHybridForTests", HybridConfig, hybrid_spec)


def grid_rows(n, width=4, start=0):
    """The rows of n tokens laid out on a grid of the given width, then counting on."""
    return [start + i // width for i in range(n)]


def hybrid_logits(c, w, tokens, rows):
    T, D = len(tokens), c.head_dim
    pos, row = torch.arange(T), torch.tensor(rows)
    h = w["embed"][torch.tensor(tokens)]
    fade = 1.0 / ((1.0 + pos.float() / 40.0) * (1.0 + row.float() / 3.0))

    def attention(x, i):
        p = f"blocks.{i}."
        q = (x @ w[p + "q_proj"].T).view(T, -1, D)
        k = (x @ w[p + "k_proj"].T).view(T, -1, D) * fade[:, None, None]
        v = (x @ w[p + "v_proj"].T).view(T, -1, D)
        return plain.causal_attention(q, k, v, pos, pos, D ** -0.5, None).reshape(T, -1) @ w[p + "o_proj"].T

    def swiglu(x, i):
        g = x @ w[f"blocks.{i}.g"].T
        return (g * torch.sigmoid(g) * (x @ w[f"blocks.{i}.u"].T)) @ w[f"blocks.{i}.d"].T

    x = plain.rms_norm(h, w["blocks.0.n1"], c.eps)
    taps = w["blocks.0.taps"]
    padded = torch.cat([torch.zeros(c.taps - 1, c.hidden_size), x])
    y = sum(taps[j] * padded[c.taps - 1 - j: c.taps - 1 - j + T] for j in range(c.taps))
    h = h + attention(y, 0)
    h = h + swiglu(plain.rms_norm(h, w["blocks.0.n2"], c.eps), 0)
    h = h + attention(plain.rms_norm(h, w["blocks.1.n1"], c.eps), 1)
    h = h + swiglu(plain.rms_norm(h, w["blocks.1.n2"], c.eps), 1)
    return plain.rms_norm(h, w["final_norm"], c.eps) @ w["head"].T


def run_hybrid(device, ops, **options):
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    cfg = HybridConfig.from_dict(dict(TOY, architectures=["ToyHybridForTests"], taps=3))
    weights = random_weights(hybrid_spec(cfg), seed=8, std=0.08, norm_jitter=0.05, dtype="float32")
    taps = weights["blocks.0.taps"]
    assert taps.dtype == torch.float32 and bool((taps > 0).all()) and abs(float(taps.sum()) - 1.0) < 1e-6
    # in a bfloat16 model the taps stay as their law drew them
    assert random_weights(hybrid_spec(cfg), seed=8, dtype="bfloat16")["blocks.0.taps"].dtype == torch.float32
    reqs = {rid: tt.random_tokens(cfg.vocab_size, n, seed=ord(rid)) for rid, n in
            {"a": 40, "b": 7, "c": 23, "d": 61, "e": 1}.items()}
    rows = {rid: grid_rows(len(toks), start=ord(rid) % 3) for rid, toks in reqs.items()}
    want = {rid: hybrid_logits(cfg, weights, toks, rows[rid]) for rid, toks in reqs.items()}
    for cut in (tt.whole, tt.portions, tt.mixed):
        steps = cut(reqs)
        at = {rid: 0 for rid in reqs}
        for s in steps:                                   # every entry brings its tokens' rows
            for e in s["entries"]:
                n = len(e["tokens"])
                e["columns"] = {"row": rows[e["id"]][at[e["id"]]:at[e["id"]] + n]}
                at[e["id"]] += n
        ec = EngineConfig(dtype="float32", page_size=4, max_token=tt.peak_tokens(steps), max_reside=4,
                          max_step_tokens=256, prefill_chunk=256, device=device, check_invariants=True)
        runner = ModelRunner(config=cfg, weights={k: v.clone() for k, v in weights.items()}, engine_config=ec, ops=ops)
        assert runner.builder.token_columns == ("row",)
        assert len(runner.cache.groups) == 1 and sorted(runner.cache.state_layers) == [1]
        assert runner.cache.groups[0].layers == [0, 2]
        got = tt.run_in_process(runner, steps)
        for rid, toks in reqs.items():
            for p in range(len(toks)):
                torch.testing.assert_close(got[(rid, p)], want[rid][p], atol=3e-4, rtol=3e-4,
                                           msg=lambda m: f"{cut.__name__} request {rid} position {p}: {m}")
    # generation: the prompt's rows come with the request, the generated tokens' rows count on from the last
    prompts = [tt.random_tokens(cfg.vocab_size, n, seed=40 + n) for n in (9, 1, 30, 17, 4)]
    new = 16
    columns, expect = [], []
    for p in prompts:
        r = grid_rows(len(p))
        columns.append({"row": r})
        toks, r = list(p), list(r)
        for _ in range(new):
            toks.append(int(hybrid_logits(cfg, weights, toks, r)[-1].argmax()))
            r.append(r[-1] + 1)
        expect.append(toks[len(p):])
    ec = EngineConfig(dtype="float32", page_size=4, max_token=512, max_reside=3, max_step_tokens=32, prefill_chunk=16,
                      device=device, check_invariants=True, **options)
    runner = ModelRunner(config=cfg, weights={k: v.clone() for k, v in weights.items()}, engine_config=ec, ops=ops)
    eng = Engine(runner=runner)
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=new), token_columns=columns)
    assert [r.output_ids for r in out] == expect
    # without its rows a request is computed as if every token's row were its position: other logits
    from return_amd.engine import StepEntry
    p = prompts[2]
    rows_of = {"with": {"row": grid_rows(len(p))}, "without": None, "as_positions": {"row": list(range(len(p)))}}
    for rid in rows_of:
        runner.add_request(rid)
    got = {rid: runner.step([StepEntry(rid, p, [len(p) - 1], cols)])[0].cpu() for rid, cols in rows_of.items()}
    for rid in rows_of:
        runner.free_request(rid)
    torch.testing.assert_close(got["with"], hybrid_logits(cfg, weights, p, grid_rows(len(p)))[-1], atol=3e-4, rtol=3e-4)
    assert torch.equal(got["without"], got["as_positions"])
    assert float((got["with"] - got["without"]).abs().max()) > 1e-2
    with pytest.raises(ValueError, match="column"):
        eng.submit(prompts[0], token_columns={"depth": [0] * len(prompts[0])})
    return runner


def test_layer_with_pages_and_state_and_a_second_position_axis_on_cpu_stand_in():
    from tests.torch_ops import TorchOps
    run_hybrid("cpu", TorchOps(), lookahead=True)


@pytest.mark.gpu
@pytest.mark.parametrize("use_graphs", [True, False])
def test_layer_with_pages_and_state_and_a_second_position_axis_on_gpu(use_graphs):
    runner = run_hybrid("cuda:0", None, use_graphs=use_graphs)
    assert bool(runner._graphs) == use_graphs


# ------------------------------------------------------------------ a part that notes its products and forms them itself
class PlainFeedForward:
    """down(relu(up(x))). It names its first and last product (so that a kernel set may measure them) but its
    forward has no ``sink`` parameter: it forms its last product itself, and no norm is finished inside it."""

    @staticmethod
    def tensor_shapes(params):
        return {"up": (params["intermediate_size"], params["hidden_size"]),
                "down": (params["hidden_size"], params["intermediate_size"])}

    @staticmethod
    def random_init(params, role):
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.up = rt.product(rt.matrix(tensors["up"]))
        self.down = rt.product(rt.matrix(tensors["down"]), residual=True)
        self.first_product = (self.up, False)
        self.last_product = self.down

    def forward(self, x, step=None):
        from return_amd.parts.runtime import ScaledRows
        assert not isinstance(x, ScaledRows) or hasattr(self.rt.ops, "linear_add_norm")
        return self.rt.ops.linear(self.rt.ops.linear(x, self.up).relu().contiguous(), self.down)


register_part("feed_forward", "toy_plain_ff", PlainFeedForward)


def test_a_part_without_a_sink_parameter_is_never_handed_one():
    """PreNormBlock gives a part a sink for its last product only if the part's forward takes one: a part
    that sets last_product and keeps the plain signature runs as it is, on a kernel set that would finish
    norms inside products (the stand-in says it can, for up to 16 rows), in steps of one and of many rows."""
    from return_amd.parts.block import takes_sink
    from tests.torch_ops import TorchOps
    cfg = ToyConfig.from_dict(dict(TOY, architectures=["ToyPlainFFForTests"]))
    H = cfg.hidden_size
    norm = lambda name: PartSpec("rms_norm", {"size": H, "eps": cfg.eps}, {"weight": name})
    attn = PartSpec("attention", {"hidden_size": H, "num_heads": cfg.heads, "num_kv_heads": cfg.kv_heads,
                                  "head_dim": cfg.head_dim, "scale": None, "window": None, "qk_norm_eps": None,
                                  "position": None},
                    {r: f"b.{r}" for r in ("q_proj", "k_proj", "v_proj", "o_proj")})
    ff = PartSpec("toy_plain_ff", {"hidden_size": H, "intermediate_size": cfg.intermediate_size}, {"up": "b.up", "down": "b.down"})
    spec = ModelSpec(
        architecture=cfg.architecture, hidden_size=H, vocab_size=cfg.vocab_size, max_position=cfg.max_position_embeddings,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size, "hidden_size": H}, {"weight": "embed"}),
        positions={}, blocks=[BlockSpec.pre_norm(attn, ff, norm("b.n1"), norm("b.n2"))],
        schedule=[LayerCall(0, cache=0), LayerCall(0, cache=1)], final_norm=norm("final_norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "hidden_size": H}, {"weight": "head"}))
    register_architecture("ToyPlainFFForTests", ToyConfig, lambda c: spec)
    weights = random_weights(spec, seed=3, std=0.08, norm_jitter=0.05, dtype="float32")
    ec = EngineConfig(dtype="float32", page_size=4, max_token=256, max_reside=4, max_step_tokens=64, prefill_chunk=64,
                      device="cpu", check_invariants=True)
    runner = ModelRunner(config=cfg, weights=weights, engine_config=ec, ops=TorchOps())
    block = runner.model.blocks[0]
    assert takes_sink(block.mixer) and not takes_sink(block.feed_forward)
    toks = tt.random_tokens(cfg.vocab_size, 30, seed=2)
    from return_amd.engine import StepEntry
    runner.add_request("whole")
    whole = runner.step([StepEntry("whole", toks, list(range(30)))])
    runner.add_request("cut")
    rows = [runner.step([StepEntry("cut", toks[:9], list(range(9)))])]
    rows += [runner.step([StepEntry("cut", [t], [0])]) for t in toks[9:]]          # single rows: norms inside products where they may be
    torch.testing.assert_close(torch.cat(rows), whole, atol=2e-5, rtol=1e-4)


def test_a_request_brings_a_column_value_for_its_prompt_tokens_at_most():
    from return_amd.engine.scheduler import Request
    r = Request("r", [1, 2, 3, 4], token_columns={"row": [0, 0, 1]})
    assert r.columns_at(0, 4) == {"row": [0, 0, 1, 2]} and r.columns_at(3, 3) == {"row": [2, 3, 4]}
    assert Request("s", [1, 2]).columns_at(0, 2) is None
    for bad in ([], [0, 0, 0, 0, 0]):
        with pytest.raises(ValueError, match="column"):
            Request("t", [1, 2, 3, 4], token_columns={"row": bad})
