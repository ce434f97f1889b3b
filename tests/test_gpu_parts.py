"""Each part of a layer alone against the plain implementation, a run order that names a
layer twice and lets a site read another site's cache, and a toy architecture with a mixer
that keeps state of its own: registered, built and stepped from this file alone."""

import pytest
import torch

import configs
import plain_qwen3 as plain
import traces
from helpers import compare, prompts_for, random_weights, replay
from lucciola_amd import parts  # noqa: F401  (registers the built-in parts)
from lucciola_amd.cache.manager import CacheManager
from lucciola_amd.cache.specs import FixedState, PagedKV
from lucciola_amd.config.engine_config import EngineConfig
from lucciola_amd.config.registry import ARCHITECTURES, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Architecture
from lucciola_amd.config.specs import LayerSpec, ModelSpec, PartSpec, RunEntry, prenorm_layer
from lucciola_amd.engine.batch import SiteView, StepEntry, build_batch
from lucciola_amd.engine.loading import _build
from lucciola_amd.engine.runner import ModelRunner
from lucciola_amd.kernels import ops
from lucciola_amd.models.causal_lm import declared_tensors
from lucciola_amd.models.qwen3 import qwen3_model_spec
from lucciola_amd.parts.base import BuildContext, Part, ResidualStream, build_part
from lucciola_amd.weights.loader import DictSource, ParamDecl
from lucciola_amd.weights.random_init import random_tensors

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def rel(got, want):
    return float((got.double().cpu() - want.double().cpu()).abs().max() / want.double().abs().max())


TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(dtype):
    ctx = BuildContext(dtype, DEV)
    norm = build_part(NORMS, PartSpec("rms", {"size": 200, "eps": 1e-5}))
    assert norm.declare()["weight"].shape == (200,) and norm.declare()["weight"].init == "ones_plus_normal"
    w = 1 + rnd(200, seed=1, scale=0.1)
    norm.bind({"weight": w}, ctx)
    h, delta = rnd(9, 200, seed=2), rnd(9, 200, seed=3, dtype=dtype)
    stream = ResidualStream(h.clone())
    stream.pending = delta
    want_h = h.double() + delta.double()
    x = norm.add_norm(stream)
    assert stream.pending is None and x.dtype == dtype
    torch.testing.assert_close(stream.h.double(), want_h, rtol=1e-6, atol=1e-6)
    assert rel(x, plain.rmsnorm(want_h.cpu(), w.cpu(), 1e-5)) < TOL[dtype]
    rows = torch.tensor([8, 2], dtype=torch.int32, device=DEV)
    stream.pending = delta
    picked = norm.add_norm_rows(stream, rows)
    want = plain.rmsnorm((want_h + delta.double())[rows.long()].cpu(), w.cpu(), 1e-5)
    assert rel(picked, want) < TOL[dtype]


def test_rotary_part():
    rot = build_part(POSITION_ENCODINGS, PartSpec("rotary", {"rotary_dim": 48, "theta": 50000.0,
                                                              "max_positions": 300}))
    rot.bind({}, BuildContext(torch.float32, DEV))
    table = rot.rotary_table(100)
    assert table.shape[1] == 48 and table.shape[0] > 100
    x = rnd(5, 3, 48, seed=4).cpu().double()
    positions = [0, 1, 17, 99, 100]
    want = plain.rope(x, positions, 50000.0)
    cs = table[torch.tensor(positions)].cpu().double()
    cos, sin = cs[:, None, :24], cs[:, None, 24:]
    got = torch.cat([x[..., :24] * cos - x[..., 24:] * sin, x[..., :24] * sin + x[..., 24:] * cos], -1)
    torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)
    epoch = rot.tables_epoch()
    bigger = rot.rotary_table(5000)           # grows on demand
    assert bigger.shape[0] > 5000 and rot.tables_epoch() == epoch + 1 and rot.ready(5000)
    torch.testing.assert_close(bigger[:table.shape[0]], table)


@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_part(dtype):
    ff = build_part(FEED_FORWARDS, PartSpec("gated_mlp", {"hidden_size": 72, "intermediate_size": 200}))
    assert {k: v.shape for k, v in ff.declare().items()} == {
        "gate_proj": (200, 72), "up_proj": (200, 72), "down_proj": (72, 200)}
    w = {"gate_proj": rnd(200, 72, seed=5, scale=0.1, dtype=torch.bfloat16),
         "up_proj": rnd(200, 72, seed=6, scale=0.1, dtype=torch.bfloat16),
         "down_proj": rnd(72, 200, seed=7, scale=0.1, dtype=torch.bfloat16)}
    ff.bind(w, BuildContext(dtype, DEV))
    x = rnd(11, 72, seed=8, dtype=dtype)
    named = {"m.gate_proj.weight": w["gate_proj"].cpu(), "m.up_proj.weight": w["up_proj"].cpu(),
             "m.down_proj.weight": w["down_proj"].cpu()}
    assert rel(ff.forward(x), plain.mlp_block(x.cpu(), named, "m.")) < TOL[dtype]
    with pytest.raises(ValueError, match="activation"):
        build_part(FEED_FORWARDS, PartSpec("gated_mlp", {"hidden_size": 8, "intermediate_size": 8,
                                                         "activation": "gelu"}))


def attention_site(part, T, page, dtype, first=0):
    """A one-request batch and a cache for one attention part."""
    cache = CacheManager([part.cache_need()], page, 64, 2)
    cache.allocate_tensors(dtype, DEV)
    cache.admit("r")
    if first:
        cache.reserve("r", first)
        cache.commit("r")
    cache.reserve("r", T)
    batch = build_batch([StepEntry("r", list(range(T)), [])], cache, DEV,
                        planners=dict([part.batch_planner()]))
    return SiteView(batch=batch, index=0, writes_cache=True, caches=cache.storage[0],
                    page_views=(batch.groups[0],)), cache


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page,window", [(4, 2, 16, 4, None), (6, 2, 48, 16, 9), (8, 1, 32, 16, None),
                                                  (4, 4, 64, 16, None)])
def test_attention_part(dtype, nh, nkv, d, page, window):
    H, T, eps, theta = 40, 37, 1e-5, 1e4
    spec = PartSpec("attention", {
        "hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d, "window": window,
        "qk_norm": PartSpec("rms", {"size": d, "eps": eps}),
        "position": PartSpec("rotary", {"rotary_dim": d, "theta": theta, "max_positions": 64})})
    part = build_part(MIXERS, spec)
    assert part.cache_need() == PagedKV(nkv, d, window, granule=16)
    names = {"q_proj": (nh * d, H), "k_proj": (nkv * d, H), "v_proj": (nkv * d, H), "o_proj": (H, nh * d),
             "q_norm.weight": (d,), "k_norm.weight": (d,)}
    assert {k: v.shape for k, v in part.declare().items()} == names
    w = {}
    for i, (name, shape) in enumerate(names.items()):
        if name.endswith("norm.weight"):
            w[name] = 1 + rnd(*shape, seed=20 + i, scale=0.2)
        else:
            w[name] = rnd(*shape, seed=20 + i, scale=0.3, dtype=torch.bfloat16)
    part.bind(dict(w), BuildContext(dtype, DEV))
    x = rnd(T, H, seed=30, dtype=dtype)
    site, _ = attention_site(part, T, page, dtype)
    got = part.forward(x, site)
    cfg = {"num_attention_heads": nh, "num_key_value_heads": nkv, "head_dim": d,
           "rms_norm_eps": eps, "rope_theta": theta}
    named = {"a." + k + ("" if k.endswith(".weight") else ".weight"): v.cpu() for k, v in w.items()}
    want, _ = plain.attention_block(x.cpu(), named, "a.", cfg, list(range(T)), window)
    assert rel(got, want) < TOL[dtype] * (2 if dtype == torch.bfloat16 else 1)


# ------------------------------------------------------------------ the run order is data
def looped_spec(cfg_dict):
    """Qwen3 parts in another order: layer 0 runs twice (two sites, two caches), and the last
    site runs layer 1 on the cache that layer 1's first site wrote."""
    from lucciola_amd.config.model_config import Qwen3Config
    from dataclasses import replace
    spec = qwen3_model_spec(Qwen3Config.from_dict(cfg_dict))
    return replace(spec, run_order=[RunEntry(0), RunEntry(1), RunEntry(0), RunEntry(1, cache_of=1)])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_run_order_names_a_layer_twice_and_shares_a_cache(dtype):
    cfg, page, seed = configs.ALL["A"]
    ARCHITECTURES.register("LoopedQwen3", Architecture("LoopedQwen3", read_config=lambda d: d,
                                                       model_spec=looped_spec), replace=True)
    try:
        cfg = dict(cfg, architectures=["LoopedQwen3"])
        weights = random_weights(cfg, seed, std=0.05)
        model = _build(looped_spec(cfg), DictSource(weights), dtype, DEV)
        assert model.site_needs()[3] is None and model.site_needs()[0] == model.site_needs()[2]
        prompts = prompts_for(cfg, [30, 9, 21], seed)
        refs = {n: plain.forward(cfg, weights, ids, run_order=[(0, None), (1, None), (0, None), (1, 1)])
                for n, ids in prompts.items()}
        for family in (traces.whole, traces.chunked, traces.mixed):
            steps = family(prompts)
            runner = ModelRunner(model, EngineConfig(dtype=dtype, block_size=page, max_seqs=4, device="cuda:0",
                                                     max_blocks=traces.max_live_tokens(steps, page) // page))
            assert len(runner.cache.storage) == 3     # three sites own a cache, one borrows
            got = replay(runner, steps)
            compare(got, cfg, weights, prompts, 2e-5 if dtype == "float32" else 3e-2, refs)
    finally:
        ARCHITECTURES.unregister("LoopedQwen3")


# ------------------------------------------------------------------ a toy architecture
class ToyDecay(Part):
    """s_t = decay * s_{t-1} + W_in x_t;  y_t = W_out s_t.  The state s lives in the request's
    slot; tokens of a portion are taken in order."""

    def __init__(self, hidden_size, state_size, decay):
        super().__init__(hidden_size=hidden_size, state_size=state_size, decay=decay)
        self.H, self.S, self.decay = hidden_size, state_size, decay

    def declare(self):
        return {"in_proj": ParamDecl((self.S, self.H)), "out_proj": ParamDecl((self.H, self.S))}

    def bind(self, tensors, ctx):
        self.w_in, self.w_out, self.dtype = tensors["in_proj"], tensors["out_proj"], ctx.dtype

    def cache_need(self):
        return FixedState((self.S,), torch.float32)

    def forward(self, x, site):
        u = ops.gemm(x, self.w_in, torch.float32)                 # [T, S]
        states = torch.empty_like(u)
        batch = site.batch
        for r, slot in enumerate(batch.slot_list):
            s = site.cache[slot]
            for t in range(batch.q_start[r], batch.q_start[r + 1]):
                s = self.decay * s + u[t]
                states[t] = s
            site.cache[slot] = s
        return ops.gemm(states.to(self.dtype), self.w_out, self.dtype)


class ToyScale(Part):
    """A feed-forward of one matrix."""

    def __init__(self, hidden_size):
        super().__init__(hidden_size=hidden_size)
        self.H = hidden_size

    def declare(self):
        return {"proj": ParamDecl((self.H, self.H))}

    def bind(self, tensors, ctx):
        self.w, self.dtype = tensors["proj"], ctx.dtype

    def forward(self, x):
        return ops.gemm(x, self.w, self.dtype)


TOY = {"architectures": ["ToyForCausalLM"], "hidden_size": 24, "vocab_size": 50, "state_size": 10,
       "decay": 0.8, "eps": 1e-5, "heads": 2, "head_dim": 16}


def toy_spec(c):
    norm = PartSpec("rms", {"size": c["hidden_size"], "eps": c["eps"]})
    attn = PartSpec("attention", {"hidden_size": c["hidden_size"], "num_heads": c["heads"],
                                  "num_kv_heads": 1, "head_dim": c["head_dim"],
                                  "position": PartSpec("rotary", {"rotary_dim": c["head_dim"], "theta": 100.0})})
    decay = PartSpec("toy_decay", {"hidden_size": c["hidden_size"], "state_size": c["state_size"],
                                   "decay": c["decay"]})
    ff = PartSpec("toy_scale", {"hidden_size": c["hidden_size"]})
    layers = []
    for i, mixer in enumerate([decay, attn, decay]):
        names = {"mixer_norm.weight": f"l{i}.n1", "feed_forward_norm.weight": f"l{i}.n2",
                 "feed_forward.proj": f"l{i}.ff"}
        if mixer is attn:
            names.update({f"mixer.{k}_proj": f"l{i}.{k}" for k in "qkvo"})
        else:
            names.update({"mixer.in_proj": f"l{i}.in", "mixer.out_proj": f"l{i}.out"})
        layers.append(prenorm_layer(mixer, ff, norm, norm, names))
    return ModelSpec(hidden_size=c["hidden_size"], vocab_size=c["vocab_size"], embedding_name="emb",
                     layers=layers, run_order=[RunEntry(0), RunEntry(1), RunEntry(2), RunEntry(0)],
                     final_norm=norm, final_norm_names={"weight": "final"}, head_name="head", init_std=0.2)


def toy_plain(c, w, ids):
    """Whole sequence, float64, no cache."""
    w = {k: v.double() for k, v in w.items()}
    T = len(ids)
    h = w["emb"][torch.tensor(ids)]
    for layer in (0, 1, 2, 0):
        x = plain.rmsnorm(h, w[f"l{layer}.n1"], c["eps"])
        if layer == 1:
            q = plain.rope((x @ w["l1.q"].T).view(T, c["heads"], c["head_dim"]), range(T), 100.0)
            k = plain.rope((x @ w["l1.k"].T).view(T, 1, c["head_dim"]), range(T), 100.0)
            v = (x @ w["l1.v"].T).view(T, 1, c["head_dim"])
            a = plain.attention(q, k, v, list(range(T))).reshape(T, -1) @ w["l1.o"].T
        else:
            u = x @ w[f"l{layer}.in"].T
            s = torch.zeros(c["state_size"], dtype=F64)
            states = []
            for t in range(T):
                s = c["decay"] * s + u[t]
                states.append(s)
            a = torch.stack(states) @ w[f"l{layer}.out"].T
        h = h + a
        h = h + plain.rmsnorm(h, w[f"l{layer}.n2"], c["eps"]) @ w[f"l{layer}.ff"].T
    return plain.rmsnorm(h, w["final"], c["eps"]) @ w["head"].T


def test_toy_architecture_with_a_stateful_mixer():
    MIXERS.register("toy_decay", ToyDecay, replace=True)
    FEED_FORWARDS.register("toy_scale", ToyScale, replace=True)
    ARCHITECTURES.register("ToyForCausalLM", Architecture("ToyForCausalLM", read_config=dict,
                                                          model_spec=toy_spec), replace=True)
    try:
        spec = toy_spec(TOY)
        weights = dict(random_tensors(declared_tensors(spec), 5, spec.init_std, torch.float32))
        model = _build(spec, DictSource(weights), "float32", "cuda:0")
        needs = model.site_needs()
        assert isinstance(needs[0], FixedState) and isinstance(needs[1], PagedKV) and needs[3] == needs[0]
        assert not model.graph_safe()
        prompts = prompts_for({"vocab_size": 50}, [25, 7, 40, 13, 31], 3)
        refs = {n: toy_plain(TOY, weights, ids) for n, ids in prompts.items()}
        for family in (traces.whole, traces.tail_decode, traces.chunked, traces.mixed):
            steps = family(prompts)
            runner = ModelRunner(model, EngineConfig(dtype="float32", block_size=4, max_seqs=4, device="cuda:0",
                                                     max_blocks=traces.max_live_tokens(steps, 4) // 4))
            assert sorted(runner.cache.storage) == [0, 1, 2, 3] and runner.cache.has_fixed_state
            assert [site for g in runner.cache.groups for site in g.sites] == [1]
            for site in (0, 2, 3):
                runner.cache.storage[site][0].fill_(7.0)   # a new request must not see an old state
            got = replay(runner, steps)
            compare(got, TOY, weights, prompts, 2e-5, refs)
    finally:
        MIXERS.unregister("toy_decay")
        FEED_FORWARDS.unregister("toy_scale")
        ARCHITECTURES.unregister("ToyForCausalLM")


def test_toy_architecture_through_the_engine_with_preemption():
    """The toy model (state slots beside pages) through LLMEngine and the scheduler, with so few
    pages that running requests are preempted and fed again: a preempted request's state
    starts from zero again, and every request's tokens are the plain implementation's."""
    from lucciola_amd.engine.llm_engine import LLMEngine
    from lucciola_amd.sampling.sampler import SamplingParams
    MIXERS.register("toy_decay", ToyDecay, replace=True)
    FEED_FORWARDS.register("toy_scale", ToyScale, replace=True)
    ARCHITECTURES.register("ToyForCausalLM", Architecture("ToyForCausalLM", read_config=dict,
                                                          model_spec=toy_spec), replace=True)
    try:
        spec = toy_spec(TOY)
        weights = dict(random_tensors(declared_tensors(spec), 5, 0.6, torch.float32))
        model = _build(spec, DictSource(weights), "float32", "cuda:0")
        prompts = list(prompts_for({"vocab_size": 50}, [9, 14, 6, 11], 8).values())
        for ahead in (False, True):
            engine = LLMEngine(model, TOY, EngineConfig(dtype="float32", block_size=4, max_blocks=18,
                                                        max_seqs=4, max_tokens_per_step=12,
                                                        device="cuda:0", run_ahead=ahead))
            for site, stored in engine.runner.cache.storage.items():
                if isinstance(engine.runner.cache.site_needs[site][0], FixedState):
                    stored[0].fill_(3.0)
            got = engine.generate(prompts, SamplingParams(max_new_tokens=20))
            assert engine.scheduler.num_preemptions > 0
            for prompt, tokens in zip(prompts, got):
                ids = list(prompt)
                for tok in tokens:
                    assert tok == int(torch.argmax(toy_plain(TOY, weights, ids)[-1]))
                    ids.append(tok)
            engine.runner.cache.check()
            assert not engine.runner.cache.requests
    finally:
        MIXERS.unregister("toy_decay")
        FEED_FORWARDS.unregister("toy_scale")
        ARCHITECTURES.unregister("ToyForCausalLM")


# ------------------------------------------------------------------ routing and another position encoding
class ToyRouted(Part):
    """A feed-forward with routing: a float32 router picks the top 2 of E one-matrix experts per
    token; their outputs are mixed with the softmax of the two router logits."""

    def __init__(self, hidden_size, experts):
        super().__init__(hidden_size=hidden_size, experts=experts)
        self.H, self.E = hidden_size, experts

    def declare(self):
        out = {"router": ParamDecl((self.E, self.H))}
        for e in range(self.E):
            out[f"expert{e}"] = ParamDecl((self.H, self.H))
        return out

    def bind(self, tensors, ctx):
        self.router = tensors["router"]
        self.experts = [tensors[f"expert{e}"] for e in range(self.E)]
        self.dtype = ctx.dtype

    def forward(self, x):
        logits = ops.gemm(x, self.router, torch.float32)           # routing in float32
        top, idx = logits.topk(2, dim=1)
        mix = torch.softmax(top, dim=1)
        out = torch.zeros(x.shape[0], self.H, dtype=torch.float32, device=x.device)
        for e, w in enumerate(self.experts):
            rows = (idx == e).any(dim=1).nonzero().flatten()
            if rows.numel() == 0:
                continue
            y = ops.gemm(x[rows].contiguous(), w, torch.float32)
            weight = (mix[rows] * (idx[rows] == e)).sum(dim=1, keepdim=True)
            out[rows] += weight * y
        return out.to(self.dtype)


class ToyOffset(Part):
    """A position encoding that is no rotation: q and k get sin(position * rate_j) added to
    entry j of every head (in place, before the cache write)."""

    def __init__(self, rate):
        super().__init__(rate=rate)
        self.rate = rate

    def bind(self, tensors, ctx):
        pass

    def rotary_table(self, max_position):
        return None                                    # not a table the fused kernel can use

    def apply(self, qkv, nh, nkv, d, positions):
        j = torch.arange(d, device=qkv.device, dtype=torch.float32)
        add = torch.sin(positions.float()[:, None] * self.rate * (j + 1))     # [T, d]
        heads = qkv.view(qkv.shape[0], nh + 2 * nkv, d)
        heads[:, :nh + nkv] += add[:, None, :].to(qkv.dtype)


TOY2 = {"architectures": ["Toy2ForCausalLM"], "hidden_size": 40, "vocab_size": 61, "experts": 5,
        "eps": 1e-6, "heads": 3, "head_dim": 16, "rate": 0.37}


def toy2_spec(c):
    norm = PartSpec("rms", {"size": c["hidden_size"], "eps": c["eps"]})
    attn = PartSpec("attention", {"hidden_size": c["hidden_size"], "num_heads": c["heads"],
                                  "num_kv_heads": 1, "head_dim": c["head_dim"],
                                  "position": PartSpec("toy_offset", {"rate": c["rate"]})})
    ff = PartSpec("toy_routed", {"hidden_size": c["hidden_size"], "experts": c["experts"]})
    layers = []
    for i in range(2):
        names = {"mixer_norm.weight": f"l{i}.n1", "feed_forward_norm.weight": f"l{i}.n2",
                 "feed_forward.router": f"l{i}.router"}
        names.update({f"feed_forward.expert{e}": f"l{i}.e{e}" for e in range(c["experts"])})
        names.update({f"mixer.{k}_proj": f"l{i}.{k}" for k in "qkvo"})
        layers.append(prenorm_layer(attn, ff, norm, norm, names))
    return ModelSpec(hidden_size=c["hidden_size"], vocab_size=c["vocab_size"], embedding_name="emb",
                     layers=layers, run_order=[RunEntry(0), RunEntry(1)],
                     final_norm=norm, final_norm_names={"weight": "final"}, head_name="head", init_std=0.3)


def toy2_plain(c, w, ids):
    w = {k: v.double() for k, v in w.items()}
    T, d = len(ids), c["head_dim"]
    h = w["emb"][torch.tensor(ids)]
    add = torch.sin(torch.arange(T, dtype=F64)[:, None] * c["rate"] * (torch.arange(d, dtype=F64) + 1))
    for i in range(2):
        x = plain.rmsnorm(h, w[f"l{i}.n1"], c["eps"])
        q = (x @ w[f"l{i}.q"].T).view(T, c["heads"], d) + add[:, None, :]
        k = (x @ w[f"l{i}.k"].T).view(T, 1, d) + add[:, None, :]
        v = (x @ w[f"l{i}.v"].T).view(T, 1, d)
        h = h + plain.attention(q, k, v, list(range(T))).reshape(T, -1) @ w[f"l{i}.o"].T
        x = plain.rmsnorm(h, w[f"l{i}.n2"], c["eps"])
        logits = x @ w[f"l{i}.router"].T
        top, idx = logits.topk(2, dim=1)
        mix = torch.softmax(top, dim=1)
        y = torch.zeros_like(h)
        for t in range(T):
            for slot in range(2):
                y[t] += mix[t, slot] * (w[f"l{i}.e{int(idx[t, slot])}"] @ x[t])
        h = h + y
    return plain.rmsnorm(h, w["final"], c["eps"]) @ w["head"].T


def test_toy_routed_feed_forward_and_another_position_encoding():
    """A feed-forward with routing and a position encoding that is no rotation, both defined
    here, registered, built and stepped without a change to the package: the cache, the step
    function and the scheduler know nothing of either."""
    from lucciola_amd.config.registry import POSITION_ENCODINGS
    FEED_FORWARDS.register("toy_routed", ToyRouted, replace=True)
    POSITION_ENCODINGS.register("toy_offset", ToyOffset, replace=True)
    ARCHITECTURES.register("Toy2ForCausalLM", Architecture("Toy2ForCausalLM", read_config=dict,
                                                           model_spec=toy2_spec), replace=True)
    try:
        spec = toy2_spec(TOY2)
        weights = dict(random_tensors(declared_tensors(spec), 9, spec.init_std, torch.float32))
        model = _build(spec, DictSource(weights), "float32", "cuda:0")
        prompts = prompts_for({"vocab_size": TOY2["vocab_size"]}, [19, 5, 44, 30], 4)
        refs = {n: toy2_plain(TOY2, weights, ids) for n, ids in prompts.items()}
        for family in (traces.whole, traces.tail_decode, traces.mixed):
            steps = family(prompts)
            runner = ModelRunner(model, EngineConfig(dtype="float32", block_size=8, max_seqs=4, device="cuda:0",
                                                     max_blocks=traces.max_live_tokens(steps, 8) // 8))
            got = replay(runner, steps)
            compare(got, TOY2, weights, prompts, 2e-5, refs)
    finally:
        FEED_FORWARDS.unregister("toy_routed")
        POSITION_ENCODINGS.unregister("toy_offset")
        ARCHITECTURES.unregister("Toy2ForCausalLM")


# ------------------------------------------------------------------ another arrangement, head norm and ends
class ParallelBlock:
    """One shared norm, mixer and feed-forward side by side: h += mixer(norm(h)) + ff(norm(h))."""

    slots = {"norm": "norm", "mixer": "mixer", "feed_forward": "feed_forward"}

    def __init__(self, norm, mixer, feed_forward):
        self.norm, self.mixer, self.feed_forward = norm, mixer, feed_forward

    def forward(self, stream, site):
        x = self.norm.add_norm(stream)
        stream.pending = ops.value(self.mixer.forward(x, site)) + ops.value(self.feed_forward.forward(x))


class UnitLength(Part):
    """A head norm that the fused kernel does not know: x / sqrt(sum x^2 + eps) * w."""

    def __init__(self, size, eps):
        super().__init__(size=size, eps=eps)
        self.size, self.eps = size, eps

    def declare(self):
        return {"weight": ParamDecl((self.size,), role="vector", init="ones_plus_normal")}

    def bind(self, tensors, ctx):
        self.weight = tensors["weight"]

    def apply(self, x):
        v = x.float()
        return (v * torch.rsqrt((v * v).sum(-1, keepdim=True) + self.eps) * self.weight).to(x.dtype)


class BiasHead(Part):
    """An output head with a bias."""

    def __init__(self, vocab_size, hidden_size, tied=False):
        super().__init__(vocab_size=vocab_size, hidden_size=hidden_size, tied=tied)
        self.V, self.H = vocab_size, hidden_size

    def declare(self):
        return {"weight": ParamDecl((self.V, self.H)), "bias": ParamDecl((self.V,), role="vector")}

    def bind(self, tensors, ctx, shared=None):
        self.weight, self.bias = tensors["weight"], tensors["bias"]

    def forward(self, x):
        return ops.gemm(x, self.weight, torch.float32) + self.bias


TOY3 = {"architectures": ["Toy3ForCausalLM"], "hidden_size": 40, "vocab_size": 53, "eps": 1e-6,
        "heads": 4, "kv_heads": 2, "head_dim": 16, "inner": 56, "scale": 3.0}


def toy3_spec(c):
    H = c["hidden_size"]
    norm = PartSpec("rms", {"size": H, "eps": c["eps"]})
    attn = PartSpec("attention", {"hidden_size": H, "num_heads": c["heads"], "num_kv_heads": c["kv_heads"],
                                  "head_dim": c["head_dim"],
                                  "qk_norm": PartSpec("unit_length", {"size": c["head_dim"], "eps": c["eps"]}),
                                  "position": PartSpec("rotary", {"rotary_dim": c["head_dim"], "theta": 500.0})})
    ff = PartSpec("gated_mlp", {"hidden_size": H, "intermediate_size": c["inner"]})
    layers = []
    for i in range(2):
        names = {"norm.weight": f"l{i}.n", "mixer.q_norm.weight": f"l{i}.qn", "mixer.k_norm.weight": f"l{i}.kn"}
        names.update({f"mixer.{k}_proj": f"l{i}.{k}" for k in "qkvo"})
        names.update({f"feed_forward.{k}_proj": f"l{i}.{k}" for k in ("gate", "up", "down")})
        layers.append(LayerSpec("toy_parallel", {"norm": norm, "mixer": attn, "feed_forward": ff}, names))
    sizes = {"vocab_size": c["vocab_size"], "hidden_size": H}
    return ModelSpec(hidden_size=H, vocab_size=c["vocab_size"], embedding_name="emb", layers=layers,
                     run_order=[RunEntry(0), RunEntry(1)], final_norm=norm,
                     final_norm_names={"weight": "final"}, head_name="head", init_std=0.3,
                     embedding=PartSpec("token_embedding", dict(sizes, scale=c["scale"])),
                     head=PartSpec("bias_head", sizes), head_names={"bias": "head_b"})


def toy3_plain(c, w, ids):
    w = {k: v.double() for k, v in w.items()}
    T, d, nh, nkv = len(ids), c["head_dim"], c["heads"], c["kv_heads"]
    unit = lambda x, wt: x / torch.sqrt((x * x).sum(-1, keepdim=True) + c["eps"]) * wt
    h = w["emb"][torch.tensor(ids)] * c["scale"]
    for i in range(2):
        x = plain.rmsnorm(h, w[f"l{i}.n"], c["eps"])
        q = plain.rope(unit((x @ w[f"l{i}.q"].T).view(T, nh, d), w[f"l{i}.qn"]), range(T), 500.0)
        k = plain.rope(unit((x @ w[f"l{i}.k"].T).view(T, nkv, d), w[f"l{i}.kn"]), range(T), 500.0)
        v = (x @ w[f"l{i}.v"].T).view(T, nkv, d)
        a = plain.attention(q, k, v, list(range(T))).reshape(T, -1) @ w[f"l{i}.o"].T
        m = plain.swiglu(x @ w[f"l{i}.gate"].T, x @ w[f"l{i}.up"].T) @ w[f"l{i}.down"].T
        h = h + a + m
    return plain.rmsnorm(h, w["final"], c["eps"]) @ w["head"].T + w["head_b"]


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_block_with_one_norm_and_parallel_branches(dtype):
    """Registered from this file alone: a block arrangement with other slots than the built-in
    one (one shared norm, two branches side by side), a q/k norm the fused kernel does not know
    (applied through its own ``apply``), a scaled embedding and a head with a bias."""
    from lucciola_amd.config.registry import BLOCKS, HEADS
    BLOCKS.register("toy_parallel", ParallelBlock, replace=True)
    NORMS.register("unit_length", UnitLength, replace=True)
    HEADS.register("bias_head", BiasHead, replace=True)
    ARCHITECTURES.register("Toy3ForCausalLM", Architecture("Toy3ForCausalLM", read_config=dict,
                                                           model_spec=toy3_spec), replace=True)
    try:
        spec = toy3_spec(TOY3)
        declared = declared_tensors(spec)
        assert "head_b" in declared and "l1.qn" in declared and "l0.n" in declared
        weights = dict(random_tensors(declared, 13, spec.init_std, torch.float32))
        model = _build(spec, DictSource(weights), dtype, "cuda:0")
        prompts = prompts_for({"vocab_size": TOY3["vocab_size"]}, [19, 5, 44, 30], 6)
        refs = {n: toy3_plain(TOY3, weights, ids) for n, ids in prompts.items()}
        for family in (traces.whole, traces.tail_decode, traces.mixed):
            steps = family(prompts)
            runner = ModelRunner(model, EngineConfig(dtype=dtype, block_size=16, max_seqs=4, device="cuda:0",
                                                     max_blocks=traces.max_live_tokens(steps, 16) // 16))
            got = replay(runner, steps)
            compare(got, TOY3, weights, prompts, {torch.float32: 2e-5, torch.bfloat16: 3e-2}[dtype], refs)
        with pytest.raises(ValueError, match="has the slots"):
            _build(replace_block(spec, "prenorm_residual"), DictSource(weights), dtype, "cuda:0")
    finally:
        BLOCKS.unregister("toy_parallel")
        NORMS.unregister("unit_length")
        HEADS.unregister("bias_head")
        ARCHITECTURES.unregister("Toy3ForCausalLM")


def replace_block(spec, block):
    from dataclasses import replace
    return replace(spec, layers=[replace(layer, block=block) for layer in spec.layers])


def test_block_arrangement_alone():
    """The pre-norm residual arrangement with stand-in parts: h1 = h + mixer(norm1(h)),
    h2 = h1 + ff(norm2(h1)); the second branch's output is still pending when the block ends."""
    from lucciola_amd.config.registry import BLOCKS

    class Scale:
        def __init__(self, factor):
            self.factor = factor

        def forward(self, x, site=None):
            return (x.float() * self.factor).to(x.dtype)

    ctx = BuildContext(torch.float32, DEV)
    n1 = build_part(NORMS, PartSpec("rms", {"size": 40, "eps": 1e-6}))
    n2 = build_part(NORMS, PartSpec("rms", {"size": 40, "eps": 1e-6}))
    w1, w2 = 1 + rnd(40, seed=1, scale=0.1), 1 + rnd(40, seed=2, scale=0.1)
    n1.bind({"weight": w1}, ctx)
    n2.bind({"weight": w2}, ctx)
    block = BLOCKS.get("prenorm_residual")(Scale(2.0), Scale(-0.5), n1, n2)
    h = rnd(6, 40, seed=3)
    stream = ResidualStream(h.clone())
    stream.pending = rnd(6, 40, seed=4)               # the previous block's last branch
    h0 = h.double().cpu() + stream.pending.double().cpu()
    block.forward(stream, None)
    h1 = h0 + 2.0 * plain.rmsnorm(h0, w1.cpu(), 1e-6)
    pending = -0.5 * plain.rmsnorm(h1, w2.cpu(), 1e-6)
    torch.testing.assert_close(stream.h.double().cpu(), h1, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(stream.pending.double().cpu(), pending, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("rows", [6, 16, 40])
def test_block_mixes_parts_that_take_scaled_rows_with_parts_that_do_not(rows):
    """Widths that the fused decode kernels take (bfloat16, 128 wide): a stand-in mixer that
    knows nothing of scaled rows or pending products beside the real feed-forward that uses
    both, and two blocks in a row so that a pending product meets the next block's norm.  Few
    rows (fused norms), 16 (their limit) and 40 (more: products cut along K hand their shares to
    the norm) must all give what the plain formulas give."""
    from lucciola_amd.config.registry import BLOCKS

    class Scale:                                  # takes and returns tensors only
        def __init__(self, factor):
            self.factor = factor

        def forward(self, x, site=None):
            assert isinstance(x, torch.Tensor)
            return (x.float() * self.factor).to(x.dtype)

    H, I, eps = 128, 2048, 1e-6
    ctx = BuildContext(torch.bfloat16, DEV)
    norm_w = [1 + rnd(H, seed=40 + i, scale=0.1) for i in range(4)]
    norms = []
    for w in norm_w:
        n = build_part(NORMS, PartSpec("rms", {"size": H, "eps": eps}))
        n.bind({"weight": w}, ctx)
        norms.append(n)
    ffs, ff_w = [], []
    for i in range(2):
        ff = build_part(FEED_FORWARDS, PartSpec("gated_mlp", {"hidden_size": H, "intermediate_size": I}))
        w = {"gate_proj": rnd(I, H, seed=50 + i, scale=H ** -0.5, dtype=torch.bfloat16),
             "up_proj": rnd(I, H, seed=52 + i, scale=H ** -0.5, dtype=torch.bfloat16),
             "down_proj": rnd(H, I, seed=54 + i, scale=I ** -0.5, dtype=torch.bfloat16)}
        ff.bind(dict(w), ctx)
        ffs.append(ff)
        ff_w.append({"m." + k + ".weight": v.cpu() for k, v in w.items()})
    make = BLOCKS.get("prenorm_residual")
    blocks = [make(Scale(0.5), ffs[0], norms[0], norms[1]), make(Scale(-0.25), ffs[1], norms[2], norms[3])]
    h = rnd(rows, H, seed=60)
    stream = ResidualStream(h.clone())
    for block in blocks:
        block.forward(stream, None)
    # plain formulas, float64
    want = h.double().cpu()
    pending = torch.zeros_like(want)
    for i, factor in enumerate((0.5, -0.25)):
        want = want + pending
        want = want + factor * plain.rmsnorm(want, norm_w[2 * i].cpu(), eps)
        pending = plain.mlp_block(plain.rmsnorm(want, norm_w[2 * i + 1].cpu(), eps), ff_w[i], "m.")
    if rows <= 16:
        assert isinstance(stream.pending, ops.PendingProduct)
    assert rel(stream.h, want) < 2e-2
    assert rel(ops.value(stream.pending), pending) < 3e-2


# ------------------------------------------------------------------ a paged cache of another layout
from dataclasses import dataclass  # noqa: E402

from lucciola_amd.cache.specs import CacheNeed  # noqa: E402


@dataclass(frozen=True)
class LatentPages(CacheNeed):
    """One latent vector of ``rank`` numbers per token, in pages: a single float32 tensor
    [pages, page, rank] per site instead of a key/value pair; ``window`` as for keys."""

    rank: int
    window: int = None

    paged = True

    def bytes_per_page(self, page_size, dtype):
        return page_size * self.rank * 4

    def allocate(self, layout, dtype, device):
        return torch.full((layout.kernel_pages, layout.kernel_page, self.rank), 77.0,
                          dtype=torch.float32, device=device)


class ToyLatentMean(Part):
    """c_t = W_c x_t is written to the token's place in the pages; y_t = W_o mean(c_s, s <= t),
    read back through the block table.  Plain torch on the device: a toy, not a kernel."""

    def __init__(self, hidden_size, rank):
        super().__init__(hidden_size=hidden_size, rank=rank)
        self.H, self.rank = hidden_size, rank

    def declare(self):
        return {"c_proj": ParamDecl((self.rank, self.H)), "o_proj": ParamDecl((self.H, self.rank))}

    def bind(self, tensors, ctx):
        self.w_c, self.w_o, self.dtype = tensors["c_proj"], tensors["o_proj"], ctx.dtype

    def cache_need(self):
        return LatentPages(self.rank)

    def forward(self, x, site):
        latents = site.cache.view(-1, self.rank)                   # every place of every page
        pages, batch = site.pages, site.batch
        c = ops.gemm(x, self.w_c, torch.float32)
        latents[pages.slots.long()] = c                            # this step's tokens, at their places
        means = torch.empty_like(c)
        for r in range(batch.num_requests):
            first, lo, hi = batch.first_position[r], batch.q_start[r], batch.q_start[r + 1]
            upto = first + hi - lo
            position = torch.arange(upto, device=x.device)
            place = pages.block_table[r].long()[position // pages.page_size] * pages.page_size \
                + position % pages.page_size
            running = latents[place].cumsum(0) / (position + 1)[:, None]
            means[lo:hi] = running[first:upto]
        return ops.gemm(means.to(self.dtype), self.w_o, self.dtype)


class TwoMixerBlock:
    """h += latent_mean(norm(h)) + attention(norm(h)); h += feed_forward(norm(h)): two parts of
    one layer keep a cache, each of its own kind."""

    slots = {"latent": "mixer", "attention": "mixer", "feed_forward": "feed_forward",
             "mixer_norm": "norm", "feed_forward_norm": "norm"}

    def __init__(self, latent, attention, feed_forward, mixer_norm, feed_forward_norm):
        self.latent, self.attention, self.feed_forward = latent, attention, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm

    def forward(self, stream, site):
        x = self.mixer_norm.add_norm(stream)
        a = self.latent.forward(x, site.part(0))
        b = ops.value(self.attention.forward(x, site.part(1)))
        stream.pending = (a.float() + b.float()).to(a.dtype)
        x = self.feed_forward_norm.add_norm(stream)
        stream.pending = self.feed_forward.forward(x)


TOY4 = {"architectures": ["Toy4ForCausalLM"], "hidden_size": 24, "vocab_size": 61, "rank": 6,
        "eps": 1e-5, "heads": 2, "head_dim": 16}


def toy4_spec(c):
    norm = PartSpec("rms", {"size": c["hidden_size"], "eps": c["eps"]})
    latent = PartSpec("toy_latent_mean", {"hidden_size": c["hidden_size"], "rank": c["rank"]})
    attn = PartSpec("attention", {"hidden_size": c["hidden_size"], "num_heads": c["heads"],
                                  "num_kv_heads": 1, "head_dim": c["head_dim"],
                                  "position": PartSpec("rotary", {"rotary_dim": c["head_dim"], "theta": 100.0})})
    ff = PartSpec("toy_scale", {"hidden_size": c["hidden_size"]})
    plain_names = {"mixer_norm.weight": "l0.n1", "feed_forward_norm.weight": "l0.n2", "feed_forward.proj": "l0.ff",
                   "mixer.c_proj": "l0.c", "mixer.o_proj": "l0.o"}
    both_names = {"mixer_norm.weight": "l1.n1", "feed_forward_norm.weight": "l1.n2", "feed_forward.proj": "l1.ff",
                  "latent.c_proj": "l1.c", "latent.o_proj": "l1.lo"}
    both_names.update({f"attention.{k}_proj": f"l1.{k}" for k in "qkvo"})
    layers = [prenorm_layer(latent, ff, norm, norm, plain_names),
              LayerSpec("toy_two_mixers", {"latent": latent, "attention": attn, "feed_forward": ff,
                                           "mixer_norm": norm, "feed_forward_norm": norm}, both_names)]
    return ModelSpec(hidden_size=c["hidden_size"], vocab_size=c["vocab_size"], embedding_name="emb",
                     layers=layers, run_order=[RunEntry(0), RunEntry(1), RunEntry(0)],
                     final_norm=norm, final_norm_names={"weight": "final"}, head_name="head", init_std=0.3)


def toy4_plain(c, w, ids):
    w = {k: v.double() for k, v in w.items()}
    T = len(ids)
    h = w["emb"][torch.tensor(ids)]
    steps = torch.arange(1, T + 1, dtype=F64)[:, None]
    for layer in (0, 1, 0):
        x = plain.rmsnorm(h, w[f"l{layer}.n1"], c["eps"])
        if layer == 0:
            a = ((x @ w["l0.c"].T).cumsum(0) / steps) @ w["l0.o"].T
        else:
            a = ((x @ w["l1.c"].T).cumsum(0) / steps) @ w["l1.lo"].T
            q = plain.rope((x @ w["l1.q"].T).view(T, c["heads"], c["head_dim"]), range(T), 100.0)
            k = plain.rope((x @ w["l1.k"].T).view(T, 1, c["head_dim"]), range(T), 100.0)
            v = (x @ w["l1.v"].T).view(T, 1, c["head_dim"])
            a = a + plain.attention(q, k, v, list(range(T))).reshape(T, -1) @ w["l1.o"].T
        h = h + a
        h = h + plain.rmsnorm(h, w[f"l{layer}.n2"], c["eps"]) @ w[f"l{layer}.ff"].T
    return plain.rmsnorm(h, w["final"], c["eps"]) @ w["head"].T


def test_toy_mixer_with_a_paged_cache_of_its_own_layout():
    """A mixer whose cache is pages of ONE tensor per site (a latent vector per token), defined
    here with its need, beside attention's key/value pages: in a layer of its own and as one of
    two caching parts of one layer.  Registered, built, replayed in every family with so few
    pages that they are used again (they start out holding 77), and driven through LLMEngine
    with preemption, with no change to the package."""
    from lucciola_amd.config.registry import BLOCKS
    from lucciola_amd.engine.llm_engine import LLMEngine
    from lucciola_amd.sampling.sampler import SamplingParams
    MIXERS.register("toy_latent_mean", ToyLatentMean, replace=True)
    FEED_FORWARDS.register("toy_scale", ToyScale, replace=True)
    BLOCKS.register("toy_two_mixers", TwoMixerBlock, replace=True)
    ARCHITECTURES.register("Toy4ForCausalLM", Architecture("Toy4ForCausalLM", read_config=dict,
                                                           model_spec=toy4_spec), replace=True)
    try:
        spec = toy4_spec(TOY4)
        weights = dict(random_tensors(declared_tensors(spec), 9, spec.init_std, torch.float32))
        model = _build(spec, DictSource(weights), "float32", "cuda:0")
        needs = model.site_needs()
        assert needs[0] == LatentPages(6) == needs[2] and isinstance(needs[1], tuple)
        assert needs[1][0] == LatentPages(6) and isinstance(needs[1][1], PagedKV)
        prompts = prompts_for({"vocab_size": 61}, [25, 7, 40, 13, 31], 4)
        refs = {n: toy4_plain(TOY4, weights, ids) for n, ids in prompts.items()}
        for family in (traces.whole, traces.tail_decode, traces.chunked, traces.mixed):
            steps = family(prompts)
            blocks = traces.max_live_tokens(steps, 4) // 4
            runner = ModelRunner(model, EngineConfig(dtype="float32", block_size=4, max_seqs=4, device="cuda:0",
                                                     max_blocks=blocks))
            cache = runner.cache
            # two groups of pages: the three latent caches share one, attention has its own
            assert [g.sites for g in cache.groups] == [[0, 1, 2], [1]]
            assert cache.storage[0][0].shape == (blocks, 4, 6) and len(cache.storage[1]) == 2
            assert cache.bytes_per_block(torch.float32) == 3 * 4 * 6 * 4 + 2 * 1 * 4 * 16 * 4
            got = replay(runner, steps)
            compare(got, TOY4, weights, prompts, 2e-5, refs)
            assert all(g.pool.num_free() == blocks for g in cache.groups)
        weights = dict(random_tensors(declared_tensors(spec), 9, 0.6, torch.float32))
        model = _build(spec, DictSource(weights), "float32", "cuda:0")
        asked = list(prompts_for({"vocab_size": 61}, [9, 14, 6, 11], 8).values())
        for ahead in (False, True):
            engine = LLMEngine(model, TOY4, EngineConfig(dtype="float32", block_size=4, max_blocks=18,
                                                         max_seqs=4, max_tokens_per_step=12,
                                                         device="cuda:0", run_ahead=ahead))
            got = engine.generate(asked, SamplingParams(max_new_tokens=20))
            assert engine.scheduler.num_preemptions > 0
            for prompt, tokens in zip(asked, got):
                ids = list(prompt)
                for tok in tokens:
                    assert tok == int(torch.argmax(toy4_plain(TOY4, weights, ids)[-1]))
                    ids.append(tok)
            engine.runner.cache.check()
    finally:
        MIXERS.unregister("toy_latent_mean")
        FEED_FORWARDS.unregister("toy_scale")
        BLOCKS.unregister("toy_two_mixers")
        ARCHITECTURES.unregister("Toy4ForCausalLM")


class ToyHinted(Part):
    """A mixer of one matrix whose launch depends on more of the batch than its make-up: its
    planner counts the cached tokens of the step's requests, and where that number is odd the
    mixer doubles its output, a choice made on the host when the step is launched.  The planner
    says so through ``graph_hint``, so a captured step is replayed only for its own kind."""

    graph_safe = True

    def __init__(self, hidden_size):
        super().__init__(hidden_size=hidden_size)
        self.H = hidden_size

    def declare(self):
        return {"proj": ParamDecl((self.H, self.H))}

    def bind(self, tensors, ctx):
        self.w, self.dtype = tensors["proj"], ctx.dtype

    def batch_planner(self):
        def plan(layout):
            odd = sum(layout.first_position) % 2
            return {"toy_odd": [odd]}, {"odd": odd, "graph_hint": odd}
        return "toy_hinted", plan

    def forward(self, x, site):
        y = ops.gemm(x, self.w, self.dtype)
        return y * 2 if site.batch.plans["toy_hinted"].info["odd"] else y


class ToyScaleInGraphs(ToyScale):
    graph_safe = True       # one product of the library, whose arguments stay put between steps


def test_toy_mixer_whose_launch_follows_a_hint_of_its_planner():
    """Three requests decode side by side, so the number of cached tokens is odd in every other
    step: with captured steps the runner keeps one step per hint, and every replay gives what
    an engine without graphs gives (a step replayed for a batch of the other kind would double,
    or not, at the wrong time)."""
    import numpy as np  # noqa: F401
    MIXERS.register("toy_hinted", ToyHinted, replace=True)
    FEED_FORWARDS.register("toy_scale", ToyScaleInGraphs, replace=True)
    try:
        H = 64
        norm = PartSpec("rms", {"size": H, "eps": 1e-5})
        layers = []
        for i in range(2):
            names = {"mixer_norm.weight": f"l{i}.n1", "feed_forward_norm.weight": f"l{i}.n2",
                     "feed_forward.proj": f"l{i}.ff", "mixer.proj": f"l{i}.mix"}
            layers.append(prenorm_layer(PartSpec("toy_hinted", {"hidden_size": H}),
                                        PartSpec("toy_scale", {"hidden_size": H}), norm, norm, names))
        spec = ModelSpec(hidden_size=H, vocab_size=40, embedding_name="emb", layers=layers,
                         run_order=[RunEntry(0), RunEntry(1)], final_norm=norm,
                         final_norm_names={"weight": "final"}, head_name="head", init_std=0.2)
        weights = dict(random_tensors(declared_tensors(spec), 9, spec.init_std, torch.bfloat16))
        prompts = prompts_for({"vocab_size": 40}, [30, 30, 30], 4)
        results = {}
        for use_graphs in (False, True):
            model = _build(spec, DictSource(weights), "bfloat16", "cuda:0")
            assert model.graph_safe()
            runner = ModelRunner(model, EngineConfig(dtype="bfloat16", block_size=16, max_blocks=16, max_seqs=4,
                                                     device="cuda:0", use_graphs=use_graphs))
            for name, ids in prompts.items():
                runner.step([StepEntry(name, ids[:10], [])])
            rows = []
            for step in range(10, 22):
                rows.append(runner.step([StepEntry(n, [prompts[n][step]], [0]) for n in prompts]).float().cpu())
            results[use_graphs] = torch.stack(rows)
            if use_graphs:
                assert sorted(k[2] for k in runner._graphs) == [(0,), (1,)]
                assert runner.graph_captures == 2 and runner.graph_replays == 10
        assert torch.equal(results[True], results[False])
        assert not torch.equal(results[True][0], results[True][1])
    finally:
        MIXERS.unregister("toy_hinted")
        FEED_FORWARDS.unregister("toy_scale")


def test_kernel_signatures_can_be_registered_from_outside():
    """A part that brings kernels of its own declares their entry points itself: here one that
    the library already has is declared under the public door and launched through it."""
    ops.register_signatures({"lc_attn_page_granule": ""})            # the same again: fine
    with pytest.raises(ops.KernelError, match="already declared"):
        ops.register_signatures({"lc_attn_page_granule": "i"})
    with pytest.raises(ops.KernelError, match="unknown argument kinds"):
        ops.register_signatures({"lc_new_kernel": "pz"})
    with pytest.raises(ops.KernelError, match="lacks the entry point"):
        ops.register_signatures({"lc_no_such_entry_point": "pi"})
    assert "lc_no_such_entry_point" not in ops._SIGNATURES
    ids = torch.zeros(3, dtype=torch.int32, device=DEV)
    source = torch.tensor([2, -1, 0], dtype=torch.int32, device=DEV)
    sampled = torch.tensor([5, 6, 7], dtype=torch.int32, device=DEV)
    ops.call("lc_feed_tokens", ops.ptr(ids), ops.ptr(source), ops.ptr(sampled), 3, 3, ops.stream())
    assert ids.tolist() == [7, 0, 5]
