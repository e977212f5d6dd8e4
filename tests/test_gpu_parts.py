"""Each part alone against the plain formulas, and the framework's openness: toy parts and toy
architectures defined here are registered, built from a model folder and stepped without any
change to the framework's files (a mixer with state of its own, windowed attention in a group
of its own, a layer that runs twice, a layer that reads another layer's cache; a second toy with
an embedding and an output head of its own, a block with one norm, and a mixer with state whose
decode steps replay as HIP graphs)."""

import json
from dataclasses import dataclass

import pytest
import torch

from clockwork_amd.config.spec import LayerSpec, ModelSpec, PagedRowsSpec, ParamSpec, RunEntry, StateSpec, WeightTarget
from clockwork_amd.parts.specs import AttentionSpec, RMSNormSpec, RopeNeoxSpec, SwiGLUSpec
from clockwork_amd.registry import (Architecture, build_part, register_architecture, register_part,
                                    unregister_architecture, unregister_arrangement, unregister_part)
from tests import replay
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _bind(part, dtype, scale=0.1, seed=0):
    gen = torch.Generator().manual_seed(seed)
    params = {}
    for name, spec in part.param_specs().items():
        t = torch.randn(spec.shape, generator=gen) * scale
        if spec.init[0] == "one_plus_uniform":
            t = 1 + t
        params[name] = t.to(dtype).to(DEV)
    part.bind(params, torch.device(DEV), dtype)
    return {k: v.float().cpu() for k, v in params.items()}


TOL = {torch.float32: dict(rtol=1e-5, atol=1e-5), torch.bfloat16: dict(rtol=3e-2, atol=3e-2)}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    part = build_part(RMSNormSpec(size=100, eps=2e-6))
    w = _bind(part, dtype)
    resid = torch.randn(6, 100, device=DEV)
    delta = torch.randn(6, 100, device=DEV).to(dtype)
    before = resid.clone()
    out = part.forward(resid, delta)
    torch.testing.assert_close(resid, before + delta.float())
    torch.testing.assert_close(out.float().cpu(), plain.rmsnorm(resid.cpu(), w["weight"], 2e-6), **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    part = build_part(SwiGLUSpec(hidden_size=80, intermediate_size=100))
    w = _bind(part, dtype)
    x = torch.randn(5, 80, device=DEV).to(dtype)
    got = part.forward(x, None)
    gu = w["gate_up_weight"]
    want = plain.swiglu(x.float().cpu(), gu[:100], gu[100:], w["down_weight"])
    torch.testing.assert_close(got.float().cpu(), want, **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 7])
def test_attention_part_whole_and_in_portions(dtype, window):
    """The mixer alone, through the real cache manager and pools: a sequence run whole, then the
    same sequence in portions and single tokens, against the plain formulas."""
    from clockwork_amd.cache import CacheManager, plan_groups
    from clockwork_amd.cache.pools import CachePools
    from clockwork_amd.engine.batch import StepEntry, build_context

    spec = AttentionSpec(hidden_size=72, num_heads=6, num_kv_heads=2, head_dim=48, qkv_bias=True, out_bias=True,
                         scale=0.2, window=window, position=RopeNeoxSpec(rotary_dim=48, theta=5000.0))
    part = build_part(spec)
    # the expected values are computed in float64, so all of the allowed error is the engine's
    w = {k: v.double() for k, v in _bind(part, dtype, scale=0.12).items()}
    T = 41
    x = torch.randn(T, 72).to(dtype)
    xf = x.double()
    qkv = plain.linear(xf, w["qkv_weight"], w["qkv_bias"])
    q, k, v = qkv[:, :288].view(T, 6, 48), qkv[:, 288:384].view(T, 2, 48), qkv[:, 384:].view(T, 2, 48)
    cos, sin = plain.rope_tables(torch.arange(T), 48, 5000.0, torch.float64)
    a = plain.attention_dense(plain.apply_rope(q, cos, sin), plain.apply_rope(k, cos, sin), v, 0.2, window=window)
    want = plain.linear(a.reshape(T, 288), w["out_weight"], w["out_bias"]).float()

    for cuts in ([T], [5, 1, 1, 17, 2, 1, 14]):
        groups = plan_groups([part.cache_need()])
        manager = CacheManager(groups, 8, 12)
        pools = CachePools(groups, 8, 12, 4, dtype, torch.device(DEV), fill=float("nan"))
        cache = pools.entry_cache(0)
        got, at = [], 0
        for n in cuts:
            if at == 0:
                manager.admit("s", n)
            manager.extend("s", at, at + n)
            ctx = build_context([StepEntry("s", at, [0] * n)], manager, torch.device(DEV), 10)
            got.append(part.forward(x[at : at + n].to(DEV), ctx, cache))
            at += n
            manager.release_behind_window("s", at)
        torch.testing.assert_close(torch.cat(got).float().cpu(), want, **TOL[dtype])


# ---------------------------------------------------------------------------------- toy parts
@dataclass(frozen=True)
class EmaMixerSpec:
    """y_t = s_t with s_t = decay * s_{t-1} + (1 - decay) * (x_t W): a recurrence whose only cache
    is a fixed-size state per request."""

    hidden_size: int
    decay: float


class EmaMixer:
    def __init__(self, spec):
        self.spec = spec

    def param_specs(self):
        return {"weight": ParamSpec((self.spec.hidden_size, self.spec.hidden_size))}

    def cache_need(self):
        return StateSpec((self.spec.hidden_size,), "float32")

    def bind(self, params, device, dtype):
        self.weight = params["weight"]

    def forward(self, x, ctx, cache):
        u = (x.float() @ self.weight.float().t())
        out = torch.empty_like(u)
        at = 0
        for r, n in enumerate(ctx.h_q_lens):
            slot = ctx.h_state_slots[r]
            s = cache.state[slot]
            for t in range(at, at + n):
                s = self.spec.decay * s + (1 - self.spec.decay) * u[t]
                out[t] = s
            cache.state[slot] = s
            at += n
        return out.to(x.dtype)


@dataclass(frozen=True)
class RoutedFFNSpec:
    """A feed-forward with routing: a float32 softmax over ``experts`` router logits, the best
    ``top_k`` renormalised, each expert a two-layer ReLU network."""

    hidden_size: int
    inner_size: int
    experts: int
    top_k: int


class RoutedFFN:
    def __init__(self, spec):
        self.spec = spec

    def param_specs(self):
        s = self.spec
        return {
            "router": ParamSpec((s.experts, s.hidden_size), init=("normal", 0.5)),
            "w_in": ParamSpec((s.experts, s.inner_size, s.hidden_size), init=("normal", 0.1)),
            "w_out": ParamSpec((s.experts, s.hidden_size, s.inner_size), init=("normal", 0.1)),
        }

    def bind(self, params, device, dtype):
        self.router, self.w_in, self.w_out = params["router"], params["w_in"], params["w_out"]

    def forward(self, x, ctx):
        gates = torch.softmax(x.float() @ self.router.float().t(), dim=-1)
        top, idx = gates.topk(self.spec.top_k, dim=-1)
        top = top / top.sum(-1, keepdim=True)
        out = torch.zeros(x.shape[0], self.spec.hidden_size, dtype=torch.float32, device=x.device)
        for e in range(self.spec.experts):
            weight = (top * (idx == e)).sum(-1, keepdim=True)  # zero for tokens that did not choose e
            out += weight * (torch.relu(x.float() @ self.w_in[e].float().t()) @ self.w_out[e].float().t())
        return out.to(x.dtype)


@dataclass(frozen=True)
class SinePositionSpec:
    """A position encoding that is no rotation: scale * sin(pos / (i + 1)) is added to element i of
    every query and key head."""

    scale: float


class SinePosition:
    # no ``graph_safe``: the cache write below picks rows with a mask, so steps run eagerly

    def __init__(self, spec):
        self.spec = spec

    def param_specs(self):
        return {}

    def bind(self, params, device, dtype):
        pass

    def rotate_and_store(self, qkv, bias, positions, slots, nh, nkv, hd, k_cache, v_cache):
        T = qkv.shape[0]
        if bias is not None:
            qkv += bias.to(qkv.dtype)
        i = torch.arange(hd, device=qkv.device, dtype=torch.float32)
        enc = self.spec.scale * torch.sin(positions.float()[:, None, None] / (i + 1.0))
        q = qkv[:, : nh * hd].view(T, nh, hd)
        q.copy_((q.float() + enc).to(qkv.dtype))
        if nkv:
            k = qkv[:, nh * hd : (nh + nkv) * hd].view(T, nkv, hd)
            v = qkv[:, (nh + nkv) * hd :].view(T, nkv, hd)
            k.copy_((k.float() + enc).to(qkv.dtype))
            keep = slots >= 0
            rows = slots[keep].long()
            k_cache.reshape(-1, nkv, hd)[rows] = k[keep]
            v_cache.reshape(-1, nkv, hd)[rows] = v[keep]


@dataclass(frozen=True)
class ToyConfig:
    vocab: int
    hidden: int
    kinds: tuple
    window: int
    eps: float


def _toy_spec(cfg: ToyConfig) -> ModelSpec:
    norm = RMSNormSpec(cfg.hidden, cfg.eps)
    ffn = SwiGLUSpec(cfg.hidden, 2 * cfg.hidden)
    rope = RopeNeoxSpec(rotary_dim=16, theta=1000.0)

    def attn(window, position=rope):
        return AttentionSpec(cfg.hidden, 4, 2, 16, True, False, 0.25, window=window, position=position)

    layers, run = [], []
    for kind in cfg.kinds:
        if kind == "again":       # the previous layer's weights once more, with a cache of its own
            run.append(RunEntry(layer=len(layers) - 1))
            continue
        if kind == "borrow":      # a layer that makes queries only and reads the first entry's keys
            layers.append(LayerSpec("prenorm", attn(None), ffn, norm, norm))
            run.append(RunEntry(layer=len(layers) - 1, cache_from=0))
            continue
        if kind == "routed":      # full attention with the sine encoding, then a routed feed-forward
            layers.append(LayerSpec("prenorm", attn(None, SinePositionSpec(0.5)), RoutedFFNSpec(cfg.hidden, 40, 3, 2), norm, norm))
            run.append(RunEntry(layer=len(layers) - 1))
            continue
        mixer = {"full": attn(None), "window": attn(cfg.window), "ema": EmaMixerSpec(cfg.hidden, 0.75)}[kind]
        layers.append(LayerSpec("prenorm", mixer, ffn, norm, norm))
        run.append(RunEntry(layer=len(layers) - 1))
    return ModelSpec("ToyForCausalLM", cfg.vocab, cfg.hidden, layers, run, norm, tie_embeddings=True)


def _toy_plan(cfg: ToyConfig, spec: ModelSpec):
    """The toy's checkpoint simply uses the model's own parameter names."""
    from clockwork_amd.parts.model import model_param_specs

    plan = []
    for name, p in model_param_specs(spec).items():
        plan.append(WeightTarget(name, (name,), (tuple(p.shape),), optional=(name == "lm_head.weight")))
    return plan


@pytest.fixture(scope="module")
def toy_dir(tmp_path_factory):
    from clockwork_amd.weights.random_init import write_random_model

    register_part(EmaMixerSpec, EmaMixer)
    register_part(RoutedFFNSpec, RoutedFFN)
    register_part(SinePositionSpec, SinePosition)
    register_architecture(
        ["ToyForCausalLM"],
        Architecture(
            "ToyForCausalLM",
            parse_config=lambda d: ToyConfig(d["vocab"], d["hidden"], tuple(d["kinds"]), d["window"], d["eps"]),
            build_spec=_toy_spec,
            weight_plan=_toy_plan,
        ),
    )
    config = {"architectures": ["ToyForCausalLM"], "vocab": 300, "hidden": 64, "window": 6, "eps": 1e-5,
              "kinds": ["full", "window", "again", "ema", "borrow", "routed"]}
    yield write_random_model(tmp_path_factory.mktemp("toy") / "toy", config, seed=3)
    # what this file brought into the registries leaves with it
    unregister_architecture(["ToyForCausalLM"])
    for spec_type in (EmaMixerSpec, RoutedFFNSpec, SinePositionSpec):
        unregister_part(spec_type)


def _toy_plain_logits(model_dir, tokens, close_calls=None):
    """The toy model from the plain formulas, whole sequence, no cache. ``close_calls`` (a list)
    receives the positions whose second and third router logits lie within 0.1 of each other: a
    rounding of the router's input can send such a token to another expert."""
    from safetensors.torch import load_file

    cfg = json.loads((model_dir / "config.json").read_text())
    w = {k: v.float() for k, v in load_file(str(model_dir / "model.safetensors")).items()}
    T, H = len(tokens), cfg["hidden"]
    h = plain.embedding(w["embed.weight"], torch.tensor(tokens))
    cos, sin = plain.rope_tables(torch.arange(T), 16, 1000.0)
    layer_of, kv_of, run = [], {}, []
    n_layers = 0
    for kind in cfg["kinds"]:
        if kind == "again":
            run.append((n_layers - 1, run[-1][1], None))
            continue
        run.append((n_layers, kind, 0 if kind == "borrow" else None))
        n_layers += 1
    for i, (layer, kind, borrow) in enumerate(run):
        p = f"layers.{layer}."
        x = plain.rmsnorm(h, w[p + "mixer_norm.weight"], cfg["eps"])
        if kind == "ema":
            u = x @ w[p + "mixer.weight"].t()
            s = torch.zeros(H)
            rows = []
            for t in range(T):
                s = 0.75 * s + 0.25 * u[t]
                rows.append(s)
            a = torch.stack(rows)
        else:
            qkv = plain.linear(x, w[p + "mixer.qkv_weight"], w[p + "mixer.qkv_bias"])
            if kind == "routed":
                enc = 0.5 * torch.sin(torch.arange(T).float()[:, None, None] / (torch.arange(16).float() + 1.0))
                encode = lambda t: t + enc
            else:
                encode = lambda t: plain.apply_rope(t, cos, sin)
            q = encode(qkv[:, :64].view(T, 4, 16))
            if borrow is None:
                k = encode(qkv[:, 64:96].view(T, 2, 16))
                v = qkv[:, 96:].view(T, 2, 16)
                kv_of[i] = (k, v)
            else:
                k, v = kv_of[borrow]
            window = cfg["window"] if kind == "window" else None
            a = plain.linear(plain.attention_dense(q, k, v, 0.25, window=window).reshape(T, 64), w[p + "mixer.out_weight"])
        h = h + a
        x = plain.rmsnorm(h, w[p + "ffn_norm.weight"], cfg["eps"])
        if kind == "routed":
            gates = torch.softmax(x @ w[p + "feed_forward.router"].t(), dim=-1)
            y = torch.zeros(T, H)
            for t in range(T):  # token by token, expert by expert
                best = sorted(range(3), key=lambda e: -float(gates[t, e]))[:2]
                ranked = sorted(float(g) for g in gates[t].log())  # logits up to a common shift
                if close_calls is not None and ranked[1] - ranked[0] < 0.1:
                    close_calls.append(t)
                total = sum(float(gates[t, e]) for e in best)
                for e in best:
                    hidden = torch.relu(w[p + "feed_forward.w_in"][e] @ x[t])
                    y[t] += float(gates[t, e]) / total * (w[p + "feed_forward.w_out"][e] @ hidden)
            h = h + y
            continue
        gu = w[p + "feed_forward.gate_up_weight"]
        h = h + plain.swiglu(x, gu[: 2 * H], gu[2 * H :], w[p + "feed_forward.down_weight"])
    return plain.linear(plain.rmsnorm(h, w["final_norm.weight"], cfg["eps"]), w["embed.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "prefill_then_decode", "portions", "mixed"])
def test_a_toy_architecture_registers_builds_and_steps(toy_dir, dtype, mode):
    gen = torch.Generator().manual_seed(5)
    requests = {f"t{i}": torch.randint(0, 300, (n,), generator=gen).tolist() for i, n in enumerate([50, 9, 77, 30, 64])}
    runner = replay.make_runner(toy_dir, dtype, 8, 64)
    # three groups: all keys (the first and the last entry; a borrower reads the first's), a window
    # (two entries: the layer and its rerun), a state
    assert [(g.is_kv, g.window, g.entries) for g in runner.manager.groups] == [(True, None, (0, 5)), (True, 6, (1, 2)), (False, None, (3,))]
    assert not runner.manager.supports_prefix_sharing
    got = replay.run_trace(runner, getattr(replay, mode)(requests))
    close = {rid: [] for rid in requests}
    ref = {rid: _toy_plain_logits(toy_dir, toks, close[rid]) for rid, toks in requests.items()}
    if dtype == "float32":
        replay.compare(got, ref, rtol=1e-5, atol=1e-5)
    else:
        # Routing is a discrete choice: where two experts' gates nearly tie, the rounding of
        # bfloat16 may choose the other one, which is no fault. Those positions are left out (the
        # routed layer is the last, so a choice touches its own position only); float32 checks them.
        sure = {key: row for key, row in got.items() if key[1] not in close[key[0]]}
        assert len(sure) > 0.9 * len(got)
        # The largest error allowed is 20% of the logits' scale here, not the 10% of the Qwen2
        # models (the root mean square keeps its 2%): this toy's experts have weights five times
        # as large as its other layers, so the last feed-forward decides the logits and passes on
        # whatever rounding its input carries; at a sequence's first positions attention averages
        # one to four values, its rounded output weighs most beside the exact embedding, and
        # errors reach 15% of the scale there (2% elsewhere). float32 holds 1e-5 at every position.
        replay.compare_to_scale(sure, ref, worst_bound=2e-1)
    assert not runner.manager.live_requests()
    assert [p.num_free for p in runner.manager.pools] == [64, 64]


def test_random_traces_of_the_toy_architecture(toy_dir):
    """Fifteen random traces (replay.random_trace with forks only: this model's cache cannot share
    prefixes) in float32: state copied at a fork, pages behind the window given back while the
    request runs, a borrowed cache, on pools that hold little more than four requests."""
    for seed in range(15):
        steps, seqs = replay.random_trace(seed, 300, kinds=("fork",))
        block_size = (4, 8, 16)[seed % 3]
        longest = sorted((-(-len(t) // block_size) for t in seqs.values()), reverse=True)[:4]
        runner = replay.make_runner(toy_dir, "float32", block_size, sum(longest) + len(seqs) + 2, max_model_len=1024)
        got = replay.run_trace(runner, steps)
        ref = {rid: _toy_plain_logits(toy_dir, toks) for rid, toks in seqs.items()}
        replay.compare(got, ref, rtol=1e-5, atol=1e-5)
        assert not runner.manager.live_requests()
        assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


# ---------------------------------------------------------------------------------- a second toy
@dataclass(frozen=True)
class ScaledEmbeddingSpec:
    """The stream starts as multiplier * table[id]."""

    vocab_size: int
    hidden_size: int
    multiplier: float


class ScaledEmbedding:
    graph_safe = True

    def __init__(self, spec):
        self.spec = spec

    def param_specs(self):
        return {"weight": ParamSpec((self.spec.vocab_size, self.spec.hidden_size))}

    def bind(self, params, device, dtype):
        self.weight = params["weight"]

    def table(self):
        return self.weight

    def forward(self, ctx):
        return self.weight[ctx.token_ids.long()].float() * self.spec.multiplier


@dataclass(frozen=True)
class CappedHeadSpec:
    """logits = cap * tanh(rows @ table^T / cap), the table being the embedding's."""

    cap: float
    tied: bool = True


class CappedHead:
    graph_safe = True

    def __init__(self, spec):
        self.spec = spec

    def param_specs(self):
        return {}

    def use_embedding(self, embedding):
        self.embedding = embedding

    def bind(self, params, device, dtype):
        pass

    def forward(self, rows, ctx):
        from clockwork_amd import ops

        logits = ops.linear(rows, self.embedding.table(), out_dtype=torch.float32)
        return self.spec.cap * torch.tanh(logits / self.spec.cap)


class OneNormBlock:
    """h = h + mixer(norm(h)) + ffn(norm(h)): one norm feeds both branches."""

    def __init__(self, mixer, feed_forward, mixer_norm):
        self.mixer, self.feed_forward, self.mixer_norm = mixer, feed_forward, mixer_norm

    def parts(self):
        return {"mixer": self.mixer, "feed_forward": self.feed_forward, "mixer_norm": self.mixer_norm}

    def forward(self, resid, delta, ctx, cache):
        from clockwork_amd import ops

        x = self.mixer_norm.forward(resid, delta)
        a = self.mixer.forward(x, ctx, cache)
        f = self.feed_forward.forward(x, ctx)
        a = a.sum(x.dtype) if isinstance(a, ops.PartialSums) else a
        f = f.sum(x.dtype) if isinstance(f, ops.PartialSums) else f
        return (a.float() + f.float()).to(x.dtype)


@dataclass(frozen=True)
class DecayMixerSpec:
    """s_t = decay * s_{t-1} + x_t, y_t = s_t W: a state per request, kept in float32."""

    hidden_size: int
    decay: float


class DecayMixer:
    """Steps of single tokens run on the device alone (a gather and a scatter by the step's state
    slots), so they can be captured as graphs; portions walk their tokens from the host."""

    graph_safe = True

    def __init__(self, spec):
        self.spec = spec

    def param_specs(self):
        return {"weight": ParamSpec((self.spec.hidden_size, self.spec.hidden_size), init=("normal", 0.05))}

    def cache_need(self):
        return StateSpec((self.spec.hidden_size,), "float32")

    def bind(self, params, device, dtype):
        self.weight = params["weight"]

    def forward(self, x, ctx, cache):
        xf = x.float()
        if all(n == 1 for n in ctx.h_q_lens):
            slots = ctx.state_slots.long()       # rows that hold no request carry the spare slot
            s = self.spec.decay * cache.state[slots] + xf
            cache.state[slots] = s
        else:
            s = torch.empty_like(xf)
            at = 0
            for r, n in enumerate(ctx.h_q_lens):
                state = cache.state[ctx.h_state_slots[r]].clone()
                for t in range(at, at + n):
                    state = self.spec.decay * state + xf[t]
                    s[t] = state
                cache.state[ctx.h_state_slots[r]] = state
                at += n
        return (s @ self.weight.float().t()).to(x.dtype)


@dataclass(frozen=True)
class Toy2Config:
    vocab: int
    hidden: int
    multiplier: float
    cap: float
    decay: float
    eps: float


def _toy2_spec(cfg: Toy2Config) -> ModelSpec:
    norm = RMSNormSpec(cfg.hidden, cfg.eps)
    ffn = SwiGLUSpec(cfg.hidden, 3 * cfg.hidden)
    attn = AttentionSpec(cfg.hidden, 4, 1, 16, True, False, 0.25, position=RopeNeoxSpec(rotary_dim=16, theta=500.0))
    layers = [
        LayerSpec("one_norm", mixer=attn, feed_forward=ffn, mixer_norm=norm),      # no second norm
        LayerSpec("prenorm", DecayMixerSpec(cfg.hidden, cfg.decay), ffn, norm, norm),
    ]
    return ModelSpec("Toy2ForCausalLM", cfg.vocab, cfg.hidden, layers, [RunEntry(0), RunEntry(1)], norm,
                     embedding=ScaledEmbeddingSpec(cfg.vocab, cfg.hidden, cfg.multiplier), head=CappedHeadSpec(cfg.cap))


@pytest.fixture(scope="module")
def toy2_dir(tmp_path_factory):
    from clockwork_amd.registry import register_arrangement
    from clockwork_amd.weights.random_init import write_random_model

    register_part(ScaledEmbeddingSpec, ScaledEmbedding)
    register_part(CappedHeadSpec, CappedHead)
    register_part(DecayMixerSpec, DecayMixer)
    register_arrangement("one_norm", OneNormBlock)
    register_architecture(
        ["Toy2ForCausalLM"],
        Architecture(
            "Toy2ForCausalLM",
            parse_config=lambda d: Toy2Config(d["vocab"], d["hidden"], d["multiplier"], d["cap"], d["decay"], d["eps"]),
            build_spec=_toy2_spec,
            weight_plan=_toy_plan,
        ),
    )
    config = {"architectures": ["Toy2ForCausalLM"], "vocab": 211, "hidden": 64, "multiplier": 3.0, "cap": 0.4,
              "decay": 0.8, "eps": 1e-5}
    yield write_random_model(tmp_path_factory.mktemp("toy2") / "toy2", config, seed=8)
    unregister_architecture(["Toy2ForCausalLM"])
    unregister_arrangement("one_norm")
    for spec_type in (ScaledEmbeddingSpec, CappedHeadSpec, DecayMixerSpec):
        unregister_part(spec_type)


def _toy2_plain_logits(model_dir, tokens):
    from safetensors.torch import load_file

    cfg = json.loads((model_dir / "config.json").read_text())
    w = {k: v.float() for k, v in load_file(str(model_dir / "model.safetensors")).items()}
    assert not any(k.startswith("lm_head.") for k in w)
    T, H = len(tokens), cfg["hidden"]
    h = cfg["multiplier"] * plain.embedding(w["embed.weight"], torch.tensor(tokens))
    # block 0: one norm, attention and feed-forward side by side
    x = plain.rmsnorm(h, w["layers.0.mixer_norm.weight"], cfg["eps"])
    qkv = plain.linear(x, w["layers.0.mixer.qkv_weight"], w["layers.0.mixer.qkv_bias"])
    cos, sin = plain.rope_tables(torch.arange(T), 16, 500.0)
    q = plain.apply_rope(qkv[:, :64].view(T, 4, 16), cos, sin)
    k = plain.apply_rope(qkv[:, 64:80].view(T, 1, 16), cos, sin)
    v = qkv[:, 80:].view(T, 1, 16)
    a = plain.linear(plain.attention_dense(q, k, v, 0.25).reshape(T, 64), w["layers.0.mixer.out_weight"])
    gu = w["layers.0.feed_forward.gate_up_weight"]
    h = h + a + plain.swiglu(x, gu[: 3 * H], gu[3 * H :], w["layers.0.feed_forward.down_weight"])
    # block 1: the recurrence, then a feed-forward behind a norm of its own
    x = plain.rmsnorm(h, w["layers.1.mixer_norm.weight"], cfg["eps"])
    s, rows = torch.zeros(H), []
    for t in range(T):
        s = cfg["decay"] * s + x[t]
        rows.append(s)
    h = h + torch.stack(rows) @ w["layers.1.mixer.weight"].t()
    x = plain.rmsnorm(h, w["layers.1.ffn_norm.weight"], cfg["eps"])
    gu = w["layers.1.feed_forward.gate_up_weight"]
    h = h + plain.swiglu(x, gu[: 3 * H], gu[3 * H :], w["layers.1.feed_forward.down_weight"])
    logits = plain.linear(plain.rmsnorm(h, w["final_norm.weight"], cfg["eps"]), w["embed.weight"])
    return cfg["cap"] * torch.tanh(logits / cfg["cap"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "prefill_then_decode", "portions", "mixed"])
def test_a_second_toy_with_its_own_embedding_head_and_block(toy2_dir, dtype, mode):
    """An embedding with a multiplier, a capped head tied to it, a block with one norm and a mixer
    with state, all registered from this file. Its single-token steps replay as HIP graphs although
    it keeps state: a fresh request's state is cleared by a kernel inside the step."""
    gen = torch.Generator().manual_seed(6)
    requests = {f"u{i}": torch.randint(0, 211, (n,), generator=gen).tolist() for i, n in enumerate([50, 9, 77, 1, 64])}
    runner = replay.make_runner(toy2_dir, dtype, 8, 40)
    assert [(g.is_kv, g.entries) for g in runner.manager.groups] == [(True, (0,)), (False, (1,))]
    assert runner.use_graphs and runner.manager.idle_state_slot == runner.manager.max_num_seqs
    got = replay.run_trace(runner, getattr(replay, mode)(requests))
    ref = {rid: _toy2_plain_logits(toy2_dir, toks) for rid, toks in requests.items()}
    if dtype == "float32":
        replay.compare(got, ref, rtol=1e-5, atol=1e-5)
    else:
        replay.compare_to_scale(got, ref)
    captured = [k for k, v in runner._graphs.items() if isinstance(v, tuple)]
    if mode in ("prefill_then_decode", "mixed"):
        assert captured, "no single-token step was replayed as a graph"
        assert all(set(runner.graph_nodes[k]) == {"kernel"} for k in captured)
    assert not runner.manager.live_requests()
    # slots come back, and a slot that another request used is cleared for the next one
    assert len(runner.manager._free_slots) == runner.manager.max_num_seqs


# ---------------------------------------------------------------------------------- a third toy
# What the first two leave to the framework's defaults: a mixer that pages rows of its own (one
# 24-wide latent a token, no values), checkpoint tensors that are stored transposed and fused,
# positions that the embedding part decides, a block whose parts have other names, a state that
# does not begin at zero.
@dataclass(frozen=True)
class OffsetEmbeddingSpec:
    """A table lookup whose tokens count their positions from ``offset``, not from 0."""

    vocab_size: int
    hidden_size: int
    offset: int


class OffsetEmbedding:
    def __init__(self, spec):
        self.spec = spec

    def param_specs(self):
        return {"weight": ParamSpec((self.spec.vocab_size, self.spec.hidden_size))}

    def bind(self, params, device, dtype):
        self.weight = params["weight"]

    def table(self):
        return self.weight

    def positions(self, ctx):
        return ctx.sequence_positions + self.spec.offset

    def forward(self, ctx):
        return self.weight[ctx.token_ids.long()].float()


@dataclass(frozen=True)
class LatentMixerSpec:
    """c_t = x_t Wc^T + 0.3 sin(pos_t / (j + 1)) is cached, 24 wide, one row a token; a token
    attends over the latents up to its own: y_t = softmax_s(scale (x_t Wq^T) . c_s) c_s Wo^T."""

    hidden_size: int
    latent: int
    scale: float


class LatentMixer:
    def __init__(self, spec):
        self.spec = spec

    def param_specs(self):
        s = self.spec
        return {"w_c": ParamSpec((s.latent, s.hidden_size), init=("normal", 0.2)),
                "w_q": ParamSpec((s.latent, s.hidden_size), init=("normal", 0.2)),
                "w_o": ParamSpec((s.hidden_size, s.latent), init=("normal", 0.1))}

    def cache_need(self):
        return PagedRowsSpec((("latent", (self.spec.latent,)),))

    def bind(self, params, device, dtype):
        self.w_c, self.w_q, self.w_o = (params[k].float() for k in ("w_c", "w_q", "w_o"))

    def forward(self, x, ctx, cache):
        xf = x.float()
        j = torch.arange(self.spec.latent, device=x.device, dtype=torch.float32)
        c = xf @ self.w_c.t() + 0.3 * torch.sin(ctx.positions.float()[:, None] / (j + 1.0))
        pages = cache.planes["latent"]                     # [pages * page size, latent]
        slots = ctx.slots[cache.group]
        keep = slots >= 0
        pages[slots[keep].long()] = c[keep].to(pages.dtype)
        q = xf @ self.w_q.t()
        out = torch.empty_like(q)
        at = 0
        for r, n in enumerate(ctx.h_q_lens):
            have, start = ctx.h_ctx_lens[r], ctx.h_starts[r]
            at_token = torch.arange(have, device=x.device)
            table = ctx.block_tables[cache.group][r].long()
            rows = table[at_token // cache.block_size] * cache.block_size + at_token % cache.block_size
            latents = pages[rows].float()                  # what the request has cached, through its block table
            scores = self.spec.scale * q[at : at + n] @ latents.t()
            seen = at_token[None, :] <= (start + torch.arange(n, device=x.device))[:, None]
            out[at : at + n] = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1) @ latents
            at += n
        return (out @ self.w_o.t()).to(x.dtype)


@dataclass(frozen=True)
class WarmDecayMixerSpec:
    """DecayMixer's recurrence, begun at s = ``begin`` in every element instead of at zero."""

    hidden_size: int
    decay: float
    begin: float


class WarmDecayMixer(DecayMixer):
    graph_safe = False

    def cache_need(self):
        return StateSpec((self.spec.hidden_size,), "float32", init=("fill", self.spec.begin))


class RenamedBlock:
    """The pre-norm wiring under names of its own: nothing in it is called ``mixer_norm``."""

    def __init__(self, mixer, feed_forward, norm_a, norm_b):
        self.mixer, self.feed_forward, self.norm_a, self.norm_b = mixer, feed_forward, norm_a, norm_b

    def parts(self):
        return {"mixer": self.mixer, "feed_forward": self.feed_forward, "norm_a": self.norm_a, "norm_b": self.norm_b}

    def first_norm(self):
        return self.norm_a

    def forward(self, resid, delta, ctx, cache):
        a = self.mixer.forward(self.norm_a.forward(resid, delta), ctx, cache)
        return self.feed_forward.forward(self.norm_b.forward(resid, a), ctx)


@dataclass(frozen=True)
class Toy3Config:
    vocab: int
    hidden: int
    latent: int
    offset: int
    begin: float
    eps: float


def _toy3_spec(cfg: Toy3Config) -> ModelSpec:
    norm = RMSNormSpec(cfg.hidden, cfg.eps)
    ffn = SwiGLUSpec(cfg.hidden, 2 * cfg.hidden)
    norms = (("norm_a", norm), ("norm_b", norm))
    layers = [
        LayerSpec("renamed", mixer=LatentMixerSpec(cfg.hidden, cfg.latent, 0.1), feed_forward=ffn, extra=norms),
        LayerSpec("renamed", mixer=WarmDecayMixerSpec(cfg.hidden, 0.7, cfg.begin), feed_forward=ffn, extra=norms),
    ]
    return ModelSpec("Toy3ForCausalLM", cfg.vocab, cfg.hidden, layers, [RunEntry(0), RunEntry(1), RunEntry(0)], norm,
                     tie_embeddings=True, embedding=OffsetEmbeddingSpec(cfg.vocab, cfg.hidden, cfg.offset))


def _toy3_plan(cfg: Toy3Config, spec: ModelSpec):
    """The latent mixer's checkpoint holds Wc and Wq as one tensor [2 latent, hidden] and Wo the
    other way round, [latent, hidden]; everything else under the model's own names."""
    plan = []
    for target in _toy_plan(cfg, spec):
        if target.param.endswith(".mixer.w_c"):
            fused = target.param[:-3] + "cq"
            plan.append(WeightTarget(target.param, (fused,), ((2 * cfg.latent, cfg.hidden),), transform=("split_rows", 0, 2)))
        elif target.param.endswith(".mixer.w_q"):
            fused = target.param[:-3] + "cq"
            plan.append(WeightTarget(target.param, (fused,), ((2 * cfg.latent, cfg.hidden),), transform=("split_rows", 1, 2)))
        elif target.param.endswith(".mixer.w_o"):
            plan.append(WeightTarget(target.param, (target.param + "_t",), ((cfg.latent, cfg.hidden),), transform=("transpose",)))
        else:
            plan.append(target)
    return plan


@pytest.fixture(scope="module")
def toy3_dir(tmp_path_factory):
    from clockwork_amd.registry import register_arrangement
    from clockwork_amd.weights.random_init import write_random_model

    register_part(OffsetEmbeddingSpec, OffsetEmbedding)
    register_part(LatentMixerSpec, LatentMixer)
    register_part(WarmDecayMixerSpec, WarmDecayMixer)
    register_arrangement("renamed", RenamedBlock)
    register_architecture(
        ["Toy3ForCausalLM"],
        Architecture(
            "Toy3ForCausalLM",
            parse_config=lambda d: Toy3Config(d["vocab"], d["hidden"], d["latent"], d["offset"], d["begin"], d["eps"]),
            build_spec=_toy3_spec,
            weight_plan=_toy3_plan,
        ),
    )
    config = {"architectures": ["Toy3ForCausalLM"], "vocab": 190, "hidden": 48, "latent": 24, "offset": 11, "begin": 0.5,
              "eps": 1e-5}
    yield write_random_model(tmp_path_factory.mktemp("toy3") / "toy3", config, seed=21)
    unregister_architecture(["Toy3ForCausalLM"])
    unregister_arrangement("renamed")
    for spec_type in (OffsetEmbeddingSpec, LatentMixerSpec, WarmDecayMixerSpec):
        unregister_part(spec_type)


def _toy3_plain_logits(model_dir, tokens, offset=None):
    from safetensors.torch import load_file

    cfg = json.loads((model_dir / "config.json").read_text())
    w = {k: v.float() for k, v in load_file(str(model_dir / "model.safetensors")).items()}
    # the checkpoint's own layout: the fused and the transposed tensors, no model-side names
    assert tuple(w["layers.0.mixer.cq"].shape) == (48, 48) and tuple(w["layers.0.mixer.w_o_t"].shape) == (24, 48)
    assert not any(k.endswith(("mixer.w_c", "mixer.w_q", "mixer.w_o")) for k in w)
    T, H, L = len(tokens), cfg["hidden"], cfg["latent"]
    pos = torch.arange(T).float() + (cfg["offset"] if offset is None else offset)
    h = plain.embedding(w["embed.weight"], torch.tensor(tokens))
    for layer in (0, 1, 0):
        p = f"layers.{layer}."
        x = plain.rmsnorm(h, w[p + "norm_a.weight"], cfg["eps"])
        if layer == 0:
            wc, wq = w[p + "mixer.cq"][:L], w[p + "mixer.cq"][L:]
            c = x @ wc.t() + 0.3 * torch.sin(pos[:, None] / (torch.arange(L).float() + 1.0))
            scores = 0.1 * (x @ wq.t()) @ c.t()
            scores = scores.masked_fill(torch.ones(T, T).triu(1).bool(), float("-inf"))
            a = torch.softmax(scores, dim=-1) @ c @ w[p + "mixer.w_o_t"]   # Wo^T as stored
        else:
            s, rows = torch.full((H,), cfg["begin"]), []
            for t in range(T):
                s = 0.7 * s + x[t]
                rows.append(s)
            a = torch.stack(rows) @ w[p + "mixer.weight"].t()
        h = h + a
        x = plain.rmsnorm(h, w[p + "norm_b.weight"], cfg["eps"])
        gu = w[p + "feed_forward.gate_up_weight"]
        h = h + plain.swiglu(x, gu[: 2 * H], gu[2 * H :], w[p + "feed_forward.down_weight"])
    return plain.linear(plain.rmsnorm(h, w["final_norm.weight"], cfg["eps"]), w["embed.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "prefill_then_decode", "portions", "mixed"])
def test_a_third_toy_pages_latents_and_loads_transposed_and_fused_tensors(toy3_dir, dtype, mode):
    """One latent row a token in pages (no value plane), a layer run twice with a page pool entry
    each, weights that the checkpoint holds fused and transposed, positions that begin at 11
    because the embedding part says so, a state that begins at 0.5, a block without a
    ``mixer_norm``: registered from this file, no framework file knows of any of it."""
    gen = torch.Generator().manual_seed(9)
    requests = {f"v{i}": torch.randint(0, 190, (n,), generator=gen).tolist() for i, n in enumerate([50, 9, 77, 1, 64])}
    runner = replay.make_runner(toy3_dir, dtype, 8, 40)
    assert [(g.is_kv, g.entries) for g in runner.manager.groups] == [(True, (0, 2)), (False, (1,))]
    assert tuple(runner.pools.kv[0].shape) == (2, 1, 40, 8, 24)
    # the loader has split the fused tensor and turned the transposed one round
    assert tuple(runner.model.params["layers.0.mixer.w_o"].shape) == (48, 24)
    got = replay.run_trace(runner, getattr(replay, mode)(requests))
    ref = {rid: _toy3_plain_logits(toy3_dir, toks) for rid, toks in requests.items()}
    if dtype == "float32":
        replay.compare(got, ref, rtol=1e-5, atol=1e-5)
        # the offset and the warm state are not idle: without either the logits are others
        first = next(iter(requests))
        for other in (_toy3_plain_logits(toy3_dir, requests[first], offset=0),):
            assert not torch.allclose(other, ref[first], rtol=1e-3, atol=1e-3)
    else:
        replay.compare_to_scale(got, ref)
    assert not runner.manager.live_requests()
    assert [p.num_free for p in runner.manager.pools] == [40]


def test_random_traces_of_the_third_toy_fork_and_copy_latent_pages(toy3_dir):
    """Random traces with forks (shared pages of latents copied on the first write, the warm state
    copied at the fork) on pools that hold little more than four requests."""
    for seed in range(8):
        steps, seqs = replay.random_trace(seed, 190, kinds=("fork",))
        block_size = (4, 8, 16)[seed % 3]
        longest = sorted((-(-len(t) // block_size) for t in seqs.values()), reverse=True)[:4]
        runner = replay.make_runner(toy3_dir, "float32", block_size, sum(longest) + len(seqs) + 2, max_model_len=1024)
        got = replay.run_trace(runner, steps)
        ref = {rid: _toy3_plain_logits(toy3_dir, toks) for rid, toks in seqs.items()}
        replay.compare(got, ref, rtol=1e-5, atol=1e-5)
        assert not runner.manager.live_requests()
        assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


def test_pages_of_planes_with_different_widths_are_copied_plane_by_plane():
    from clockwork_amd.cache import plan_groups
    from clockwork_amd.cache.pools import CachePools

    groups = plan_groups([PagedRowsSpec((("k", (2, 16)), ("v", (2, 8)))), PagedRowsSpec((("k", (2, 16)), ("v", (2, 8))))])
    pools = CachePools(groups, 4, 6, 2, torch.bfloat16, torch.device(DEV))
    for t in pools.planes[0].values():
        t.copy_(torch.randn(t.shape))
    before = {n: t.clone() for n, t in pools.planes[0].items()}
    pools.copy_pages(0, [(1, 4), (2, 0)])
    torch.cuda.synchronize()
    for name, t in pools.planes[0].items():
        want = before[name].clone()
        want[:, 4], want[:, 0] = before[name][:, 1], before[name][:, 2]
        assert torch.equal(t, want), name


def test_windowed_group_uses_few_pages_for_a_long_request(toy_dir):
    runner = replay.make_runner(toy_dir, "float32", 8, 64)
    toks = torch.randint(0, 300, (200,), generator=torch.Generator().manual_seed(6)).tolist()
    runner.reserve("x", 0, 100)
    from clockwork_amd.engine.batch import StepEntry

    runner.step([StepEntry("x", 0, toks[:100], [])])
    for p in range(100, 200):
        runner.reserve("x", p, 1)
        runner.step([StepEntry("x", p, toks[p : p + 1], [])])
        assert 64 - runner.manager.pools[1].num_free <= 2  # a window of 6 tokens spans at most two pages of 8
    assert 64 - runner.manager.pools[0].num_free == 25
    runner.release("x")


def test_unknown_parts_and_architectures_are_refused():
    @dataclass(frozen=True)
    class Unknown:
        x: int = 0

    with pytest.raises(KeyError, match="no part is registered"):
        build_part(Unknown())
    from clockwork_amd.registry import resolve_architecture

    with pytest.raises(ValueError, match="no architecture is registered"):
        resolve_architecture({"architectures": ["NopeForCausalLM"], "model_type": "nope"})
