"""Each part alone against the plain implementation, and the generality of the assembly:
a toy mixer with state of its own, defined here, is registered, built into a model beside
attention layers and stepped; a run order that names a layer twice and lets a layer read
another layer's cache; two more toy architectures bring a position encoding and a routed
feed-forward, and a norm and an arrangement of their own. No file of the package changes for this.

Runs on the CPU test double, and on the HIP kernels when a GPU is there."""

import pytest
import torch

import plain_qwen2 as plain
from distie_amd.cache import CacheManager
from distie_amd.config import LayerCall, LayerSpec, ModelSpec, PartSpec, register_architecture
from distie_amd.engine.batch import BatchBuilder, StepEntry
from distie_amd.engine.model import Model
from distie_amd.engine.runner import ModelRunner
from distie_amd.parts import (FeedForward, FixedState, Mixer, PagedKV, PagedTensors, ParamSpec, PositionEncoding, ResidualStream,
                              StepContext, build_part, register_part)
from torch_ops import TorchOps


@pytest.fixture(scope="module", params=["cpu", pytest.param("hip", marks=pytest.mark.gpu)])
def ops(request):
    if request.param == "cpu":
        return TorchOps()
    from distie_amd.kernels.hip_ops import HipOps

    return HipOps("cuda:0")


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def dense(ops, x):
    return ops.dense(x) if hasattr(ops, "dense") else x


def context(ops, requirements, lengths, block=4, dtype=torch.float32):
    """A cache and the batch of whole sequences of the given lengths."""
    cache = CacheManager(requirements, block, 64, 8, device=ops.device, dtype=dtype)
    builder = BatchBuilder(cache, 512, ops.device, 1000)
    entries = []
    for i, n in enumerate(lengths):
        cache.add(i)
        cache.reserve(i, n)
        entries.append(StepEntry(i, [0] * n, []))
    ids, meta, _ = builder.build(entries)
    return cache, meta


def test_rmsnorm_part(ops):
    part = build_part("norm", PartSpec("rmsnorm", "n.", {"size": 50, "eps": 1e-3}))
    assert {k: v.shape for k, v in part.param_specs().items()} == {"weight": (50,)}
    w = 1 + rnd(50, seed=1, scale=0.3)
    part.load({"weight": w.to(ops.device)})
    x = rnd(6, 50, seed=2, scale=2.0)
    got = part.apply(ops, x.to(ops.device), torch.float32)
    assert (got.cpu() - plain.rms_norm(x, w, 1e-3)).abs().max() < 1e-5
    stream = ResidualStream(x.clone().to(ops.device))
    stream.pending = rnd(6, 50, seed=3).to(ops.device)
    got = part.of_stream(ops, stream, torch.float32)
    want = x + rnd(6, 50, seed=3)
    assert stream.pending is None and (stream.hidden.cpu() - want).abs().max() < 1e-6
    assert (got.cpu() - plain.rms_norm(want, w, 1e-3)).abs().max() < 1e-5


def test_rotary_part(ops):
    part = build_part("position", PartSpec("rope", "", {"dim": 24, "theta": 500.0}))
    assert torch.allclose(part.rotary(), plain.rope_inv_freq(24, 500.0))
    with pytest.raises(ValueError):
        build_part("position", PartSpec("rope", "", {"dim": 7, "theta": 500.0}))
    assert build_part("position", PartSpec("none")).rotary() is None


def test_swiglu_part(ops):
    part = build_part("feed_forward", PartSpec("swiglu", "mlp.", {"hidden_size": 40, "intermediate_size": 72}))
    w = {"gate_proj.weight": rnd(72, 40, seed=1, scale=0.2), "up_proj.weight": rnd(72, 40, seed=2, scale=0.2),
         "down_proj.weight": rnd(40, 72, seed=3, scale=0.2)}
    assert {k: v.shape for k, v in part.param_specs().items()} == {k: tuple(v.shape) for k, v in w.items()}
    part.load({k: v.to(ops.device) for k, v in w.items()})
    x = rnd(5, 40, seed=4)
    got = dense(ops, part.forward(ops, x.to(ops.device), None))
    want = plain.swiglu(x.double(), *(w[k].double() for k in ("gate_proj.weight", "up_proj.weight", "down_proj.weight")))
    assert (got.cpu().double() - want).abs().max() < 1e-5


@pytest.mark.parametrize("heads,kv_heads,dim,window,bias", [(4, 2, 16, None, True), (3, 1, 32, 5, True), (2, 2, 48, None, False)])
def test_attention_part(ops, heads, kv_heads, dim, window, bias):
    hidden = 40
    spec = PartSpec("attention", "a.", {"hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads,
                                        "head_dim": dim, "qkv_bias": bias, "window": window,
                                        "position": PartSpec("rope", "", {"dim": dim, "theta": 1e4})})
    part = build_part("mixer", spec)
    assert part.cache_requirement() == PagedKV(kv_heads, dim, window)
    w = {}
    for i, (name, pspec) in enumerate(part.param_specs().items()):
        w[name] = rnd(*pspec.shape, seed=10 + i, scale=0.2)
    part.load({k: v.to(ops.device) for k, v in w.items()})
    lengths = [9, 1, 14]
    cache, meta = context(ops, [part.cache_requirement()], lengths)
    x = rnd(sum(lengths), hidden, seed=5)
    got = dense(ops, part.forward(ops, x.to(ops.device), StepContext(meta, torch.float32), cache.layer(0)["mixer"], True)).cpu()
    cfg = {"num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": dim, "hidden_size": hidden,
           "rope_theta": 1e4}
    named = {"a." + k: v.double() for k, v in w.items()}
    if not bias:
        for n, rows in (("q", heads * dim), ("k", kv_heads * dim), ("v", kv_heads * dim)):
            named[f"a.{n}_proj.bias"] = torch.zeros(rows, dtype=torch.float64)
    at = 0
    for n in lengths:
        want = plain.self_attention(x[at:at + n].double(), named, "a.", torch.arange(n), cfg, window)
        assert (got[at:at + n].double() - want).abs().max() < 1e-5
        at += n


def test_prenorm_block(ops):
    """h += mixer(norm(h)); h += ffn(norm(h)), with the additions left to the next norm."""
    calls = []

    class Twice(Mixer):
        def forward(self, ops, x, ctx, cache, writes_cache):
            calls.append("mixer")
            return x * 2

    register_part("mixer", "test_twice", Twice)

    class Half(FeedForward):
        def forward(self, ops, x, ctx):
            calls.append("ffn")
            return x * 0.5

    register_part("feed_forward", "test_half", Half)
    norm = PartSpec("rmsnorm", "", {"size": 8, "eps": 1e-6})
    block = build_part("block", PartSpec("prenorm_residual"), {
        "mixer": PartSpec("test_twice"), "feed_forward": PartSpec("test_half"), "mixer_norm": norm, "feed_forward_norm": norm})
    assert [type(p).__name__ for p in block.parts()] == ["RMSNorm", "Twice", "RMSNorm", "Half", "PreNormResidual"]
    for n in (block.mixer_norm, block.feed_forward_norm):
        n.load({"weight": torch.ones(8, device=ops.device)})
    with pytest.raises(ValueError, match="missing \\['feed_forward_norm'\\], not known to it \\['third_norm'\\]"):
        build_part("block", PartSpec("prenorm_residual"), {
            "mixer": PartSpec("test_twice"), "feed_forward": PartSpec("test_half"), "mixer_norm": norm, "third_norm": norm})
    x = rnd(3, 8, seed=1)
    stream = ResidualStream(x.clone().to(ops.device))
    block.forward(ops, stream, StepContext(None, torch.float32), {"mixer": None}, True)
    rms = lambda t: plain.rms_norm(t, torch.ones(8), 1e-6)
    h1 = x + 2 * rms(x)
    assert calls == ["mixer", "ffn"]
    assert (stream.hidden.cpu() - h1).abs().max() < 1e-5
    assert (stream.pending.cpu() - 0.5 * rms(h1)).abs().max() < 1e-5


# ---------------------------------------------------------------------------------------------
# a toy mixer with state of its own: y_t = s_t, s_t = decay * s_{t-1} + x_t W, one state row a request
# ---------------------------------------------------------------------------------------------
class DecayMixer(Mixer):
    def __init__(self, spec):
        super().__init__(spec)
        self.size = int(spec.params["hidden_size"])
        self.decay = float(spec.params["decay"])
        self.weight = None

    def cache_requirement(self):
        return FixedState.of((self.size,))

    def param_specs(self):
        return {"mix.weight": ParamSpec((self.size, self.size))}

    def load(self, tensors):
        self.weight = tensors["mix.weight"].float()

    def forward(self, ops, x, ctx, cache, writes_cache):
        meta = ctx.meta
        u = ops.dense(x).float() @ self.weight.T        # computes on the values itself: the finished tensor first
        out = torch.empty_like(u)
        slots = meta.state_slots.tolist()
        cu = meta.cu_q.tolist()
        for b in range(meta.num_requests):          # tokens of a request in order; the state carries over
            s = cache["state"][slots[b]]
            for t in range(cu[b], cu[b + 1]):
                s = self.decay * s + u[t]
                out[t] = s
            if writes_cache:
                cache["state"][slots[b]] = s
        return out.to(x.dtype)


class ToyConfig:
    """An architecture of the test: attention and decay layers in turn, layer 0 run twice, and
    the last call reads layer 0's cache."""

    def __init__(self, hidden, vocab, decay):
        self.hidden, self.vocab, self.decay = hidden, vocab, decay

    @classmethod
    def from_dict(cls, data):
        return cls(data["hidden"], data["vocab"], data["decay"])

    def model_spec(self):
        norm = lambda p: PartSpec("rmsnorm", p, {"size": self.hidden, "eps": 1e-5})
        ffn = lambda p: PartSpec("swiglu", p, {"hidden_size": self.hidden, "intermediate_size": 2 * self.hidden})

        def attention(p):
            return PartSpec("attention", p, {"hidden_size": self.hidden, "num_heads": 2, "num_kv_heads": 1,
                                             "head_dim": self.hidden // 2, "qkv_bias": False,
                                             "position": PartSpec("rope", "", {"dim": self.hidden // 2, "theta": 100.0})})

        layers = []
        for l, mixer in enumerate([attention("l0.attn."), PartSpec("test_decay", "l1.", {"hidden_size": self.hidden, "decay": self.decay}),
                                   attention("l2.attn.")]):
            layers.append(LayerSpec(PartSpec("prenorm_residual"), {
                "mixer": mixer, "feed_forward": ffn(f"l{l}.ffn."), "mixer_norm": norm(f"l{l}.n1."),
                "feed_forward_norm": norm(f"l{l}.n2.")}))
        order = (LayerCall(0), LayerCall(1), LayerCall(2), LayerCall(2, cache_of=0))
        sizes = {"vocab_size": self.vocab, "hidden_size": self.hidden}
        return ModelSpec("ToyForCausalLM", self.vocab, self.hidden, 256, PartSpec("token_embedding", "emb.", sizes), layers,
                         order, norm("final."), PartSpec("lm_head", "head.", dict(sizes, tied_to="emb.weight")))


def toy_plain(weights, cfg, ids):
    """The toy model in plain torch (float64), whole sequence, no cache."""
    w = {k: v.double() for k, v in weights.items()}
    x = w["emb.weight"][torch.tensor(ids)]
    n = len(ids)
    att_cfg = {"num_attention_heads": 2, "num_key_value_heads": 1, "head_dim": cfg.hidden // 2, "rope_theta": 100.0}
    zero = lambda rows: torch.zeros(rows, dtype=torch.float64)

    def attention(x, p, kv_from=None):
        named = dict(w)
        for name, rows in (("q", cfg.hidden), ("k", cfg.hidden // 2), ("v", cfg.hidden // 2)):
            named[p + f"{name}_proj.bias"] = zero(rows)
        if kv_from is not None:      # keys and values of another layer's cache: its k/v of its own input
            return kv_from
        return plain.self_attention(x, named, p, torch.arange(n), att_cfg, None)

    def ffn(x, p):
        return plain.swiglu(x, w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"])

    rms = lambda t, p: plain.rms_norm(t, w[p + "weight"], 1e-5)
    # layer 0 (its keys and values are kept for the last call)
    n0 = rms(x, "l0.n1.")
    x = x + attention(n0, "l0.attn.")
    x = x + ffn(rms(x, "l0.n2."), "l0.ffn.")
    # layer 1: decay mixer
    u = rms(x, "l1.n1.") @ w["l1.mix.weight"].T
    s = torch.zeros(cfg.hidden, dtype=torch.float64)
    y = []
    for t in range(n):
        s = cfg.decay * s + u[t]
        y.append(s)
    x = x + torch.stack(y)
    x = x + ffn(rms(x, "l1.n2."), "l1.ffn.")
    # layer 2 with its own cache
    x = x + attention(rms(x, "l2.n1."), "l2.attn.")
    x = x + ffn(rms(x, "l2.n2."), "l2.ffn.")
    # layer 2 again, reading layer 0's keys and values: q from layer 2's weights, k/v as layer 0 made them
    n2 = rms(x, "l2.n1.")
    d = cfg.hidden // 2
    q = (n2 @ w["l2.attn.q_proj.weight"].T).view(n, 2, d)
    k = (n0 @ w["l0.attn.k_proj.weight"].T).view(n, 1, d)
    v = (n0 @ w["l0.attn.v_proj.weight"].T).view(n, 1, d)
    cos, sin = plain.rope_cos_sin(torch.arange(n), d, 100.0, torch.float64)
    mixed = plain.attention(plain.apply_rope(q, cos, sin), plain.apply_rope(k, cos, sin), v)
    x = x + mixed.reshape(n, cfg.hidden) @ w["l2.attn.o_proj.weight"].T
    x = x + ffn(rms(x, "l2.n2."), "l2.ffn.")
    return plain.rms_norm(x, w["final.weight"], 1e-5) @ w["emb.weight"].T


def test_toy_architecture_with_a_state_mixer_is_registered_built_and_stepped(ops):
    register_part("mixer", "test_decay", DecayMixer)
    register_architecture("ToyForCausalLM", ToyConfig)
    from distie_amd.config import config_from_dict

    cfg = config_from_dict({"architectures": ["ToyForCausalLM"], "hidden": 32, "vocab": 70, "decay": 0.8})
    model = Model(cfg.model_spec())
    specs = model.param_specs()
    assert "l1.mix.weight" in specs and "l0.attn.q_proj.weight" in specs and "head.weight" not in specs
    gen = torch.Generator().manual_seed(3)
    weights = {n: (torch.ones(s.shape) if s.init == "ones" else torch.randn(s.shape, generator=gen) * 0.2)
               for n, s in specs.items()}
    model.load_tensors(lambda name: weights[name].to(ops.device))
    needs = model.cache_requirements()
    assert isinstance(needs[1]["mixer"], FixedState) and needs[0] == {"mixer": PagedKV(1, 16)} and \
        isinstance(needs[0]["mixer"], PagedTensors)
    cache = CacheManager(needs, 4, 32, 4, device=ops.device, dtype=torch.float32)
    runner = ModelRunner(model, cache, ops, torch.float32, 256)
    a = torch.randint(0, 70, (23,), generator=gen).tolist()
    b = torch.randint(0, 70, (9,), generator=gen).tolist()
    want_a, want_b = toy_plain(weights, cfg, a).float(), toy_plain(weights, cfg, b).float()
    # whole
    got = runner.step([StepEntry("a", a, list(range(23)))]).cpu()
    assert (got - want_a).abs().max() < 1e-4
    runner.finish("a")
    # in portions, mixed with another request, the state slot taken again after a request ended
    rows = {"a": [], "b": []}
    plan = [[("a", 0, 5)], [("a", 5, 7), ("b", 0, 3)], [("a", 7, 20), ("b", 3, 4)], [("b", 4, 9), ("a", 20, 21)],
            [("a", 21, 23)]]
    seqs = {"a": a, "b": b}
    for step in plan:
        entries = [StepEntry(r, seqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in step]
        logits = runner.step(entries).cpu()
        at = 0
        for r, lo, hi in step:
            rows[r].append(logits[at:at + hi - lo])
            at += hi - lo
    assert (torch.cat(rows["a"]) - want_a).abs().max() < 1e-4
    assert (torch.cat(rows["b"]) - want_b).abs().max() < 1e-4
    runner.finish("a")
    runner.finish("b")
    cache.check()
    assert cache.slots.num_free == 4
    # a new request in a used slot starts from a zero state
    got = runner.step([StepEntry("c", b, list(range(9)))]).cpu()
    assert (got - want_b).abs().max() < 1e-4


@pytest.mark.gpu
def test_toy_state_mixer_in_bfloat16_on_the_hip_kernels():
    """The same toy in the serving precision, where a step of few rows hands a mixer values that are not
    tensors yet (the norm is left to the product that reads it): the toy asks for the finished tensor with
    `ops.dense`, as the interface says, and one that does not is told so."""
    from distie_amd.config import config_from_dict
    from distie_amd.kernels.hip_ops import HipOps, KernelError

    ops = HipOps("cuda:0")
    register_part("mixer", "test_decay", DecayMixer)
    register_architecture("ToyForCausalLM", ToyConfig)
    cfg = config_from_dict({"architectures": ["ToyForCausalLM"], "hidden": 32, "vocab": 70, "decay": 0.8})
    model = Model(cfg.model_spec())
    gen = torch.Generator().manual_seed(3)
    weights = {n: (torch.ones(s.shape) if s.init == "ones" else torch.randn(s.shape, generator=gen) * 0.2).bfloat16().float()
               for n, s in model.param_specs().items()}
    model.load_tensors(lambda name: weights[name].to(ops.device).bfloat16())
    cache = CacheManager(model.cache_requirements(), 16, 16, 4, device=ops.device, dtype=torch.bfloat16)
    runner = ModelRunner(model, cache, ops, torch.bfloat16, 256)
    a = torch.randint(0, 70, (40,), generator=gen).tolist()
    want = toy_plain(weights, cfg, a).float()
    rows = [runner.step([StepEntry("a", a[:20], list(range(20)))])]            # 20 rows: tensors all the way
    rows += [runner.step([StepEntry("a", a[i:i + 1], [0])]) for i in range(20, 40)]      # 1 row: pending values
    got = torch.cat(rows).float().cpu()
    scale = want.abs().max().item()
    assert (got - want).abs().max().item() < scale / 16 and (got - want).pow(2).mean().sqrt().item() < scale / 64
    runner.finish("a")

    class Careless(DecayMixer):
        def forward(self, ops, x, ctx, cache, writes_cache):
            return x.float().to(torch.bfloat16)

    register_part("mixer", "test_decay", Careless)
    try:
        careless = Model(cfg.model_spec())
        careless.load_tensors(lambda name: weights[name].to(ops.device).bfloat16())
        runner = ModelRunner(careless, cache, ops, torch.bfloat16, 256)
        with pytest.raises(KernelError, match="ops.dense"):
            runner.step([StepEntry("b", a[:1], [0])])
    finally:
        register_part("mixer", "test_decay", DecayMixer)


# ---------------------------------------------------------------------------------------------
# a position encoding that lives inside attention: a bias on every score by the distance to the key, with a
# slope per head, and scores bent by a cap; both reach the kernels as `ScoreExtras`
# ---------------------------------------------------------------------------------------------
class DistanceBias(PositionEncoding):
    def head_slopes(self, num_heads):
        return torch.tensor([2.0 ** (-8.0 * (h + 1) / num_heads) for h in range(num_heads)])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,window,cap", [(4, 2, 16, None, 3.0), (3, 1, 32, 6, None), (8, 2, 128, None, 5.0)])
def test_attention_with_a_bias_by_distance_and_capped_scores(ops, heads, kv_heads, dim, window, cap, dtype):
    if dtype == torch.bfloat16 and ops.device.type != "cuda":
        pytest.skip("the test double is run in float32")
    register_part("position", "test_distance_bias", DistanceBias)
    hidden = 48
    spec = PartSpec("attention", "a.", {"hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": dim,
                                        "qkv_bias": True, "window": window, "score_cap": cap,
                                        "position": PartSpec("test_distance_bias")})
    part = build_part("mixer", spec)
    w = {name: rnd(*pspec.shape, seed=40 + i, scale=0.5 if "q_proj" in name or "k_proj" in name else 0.2)
         for i, (name, pspec) in enumerate(part.param_specs().items())}
    w = {k: v.to(dtype).float() for k, v in w.items()}
    part.load({k: v.to(ops.device).to(dtype if v.dim() == 2 else torch.float32) for k, v in w.items()})
    part.prepare(ops)
    assert part.extras is not None and part.extras.score_cap == cap and part.extras.head_slopes.shape == (heads,)
    lengths = [70, 1, 20]          # 70: beyond one chunk of 64 keys
    cache, meta = context(ops, [part.cache_requirement()], lengths, block=16, dtype=dtype)
    x = rnd(sum(lengths), hidden, seed=6).to(dtype)
    got = dense(ops, part.forward(ops, x.to(ops.device), StepContext(meta, dtype), cache.layer(0)["mixer"], True)).float().cpu()
    slopes = DistanceBias(PartSpec("test_distance_bias")).head_slopes(heads).double()
    at = 0
    for n in lengths:
        xs = x[at:at + n].double()
        q = (xs @ w["q_proj.weight"].double().T + w["q_proj.bias"].double()).view(n, heads, dim)
        k = (xs @ w["k_proj.weight"].double().T + w["k_proj.bias"].double()).view(n, kv_heads, dim)
        v = (xs @ w["v_proj.weight"].double().T + w["v_proj.bias"].double()).view(n, kv_heads, dim)
        if dtype == torch.bfloat16:                 # what the cache holds
            q, k, v = (t.to(dtype).double() for t in (q, k, v))
        k, v = plain.repeat_kv(k, heads // kv_heads), plain.repeat_kv(v, heads // kv_heads)
        s = torch.einsum("ihd,jhd->hij", q, k) * dim ** -0.5
        if cap is not None:
            s = cap * torch.tanh(s / cap)
        i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
        s = s + slopes[:, None, None] * (j - i).double()
        seen = (j <= i) if window is None else (j <= i) & (i - j < window)
        s = s.masked_fill(~seen, float("-inf"))
        mixed = torch.einsum("hij,jhd->ihd", torch.softmax(s, -1), v).reshape(n, heads * dim)
        if dtype == torch.bfloat16:
            mixed = mixed.to(dtype).double()
        want = mixed @ w["o_proj.weight"].double().T
        err = (got[at:at + n].double() - want).abs().max().item()
        size = want.abs().max().item()               # float32: 1e-5 of the largest value, which is well above 1 here
        assert err < (1e-5 * max(size, 1.0) if dtype == torch.float32 else 0.02 * size + 1e-3), (n, err, size)
        at += n
    # the slopes matter: without them the result is another
    part.extras = None
    plain_scores = dense(ops, part.forward(ops, x.to(ops.device), StepContext(meta, dtype), cache.layer(0)["mixer"], True)).float().cpu()
    assert (plain_scores - got).abs().max().item() > 1e-2


# ---------------------------------------------------------------------------------------------
# a second toy architecture: positions learned and added to the embeddings (attention without rotation),
# and in one layer a routed feed-forward (the best of three experts of different widths, scaled by its
# router weight) beside a dense one in the other: chosen layer by layer by the configuration
# ---------------------------------------------------------------------------------------------

class LearnedPositions(PositionEncoding):
    def __init__(self, spec):
        super().__init__(spec)
        self.shape = (int(spec.params["max_positions"]), int(spec.params["hidden_size"]))
        self.table = None

    def param_specs(self):
        return {"weight": ParamSpec(self.shape)}

    def load(self, tensors):
        self.table = tensors["weight"].float()

    def on_embedding(self, ops, hidden, meta):
        hidden += self.table[meta.positions.long()]


class BestOfExperts(FeedForward):
    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec.params["hidden_size"])
        self.widths = [int(w) for w in spec.params["expert_sizes"]]
        self.router = None
        self.gate_up, self.down = [], []

    def param_specs(self):
        specs = {"router.weight": ParamSpec((len(self.widths), self.hidden))}
        for e, width in enumerate(self.widths):
            specs[f"experts.{e}.gate_proj.weight"] = ParamSpec((width, self.hidden))
            specs[f"experts.{e}.up_proj.weight"] = ParamSpec((width, self.hidden))
            specs[f"experts.{e}.down_proj.weight"] = ParamSpec((self.hidden, width))
        return specs

    def load(self, tensors):
        self.router = tensors["router.weight"].contiguous()
        for e in range(len(self.widths)):
            self.gate_up.append(torch.cat([tensors[f"experts.{e}.gate_proj.weight"],
                                           tensors[f"experts.{e}.up_proj.weight"]]).contiguous())
            self.down.append(tensors[f"experts.{e}.down_proj.weight"].contiguous())

    def prepare(self, ops):
        for gate_up, down in zip(self.gate_up, self.down):
            ops.prepare_linear(gate_up, gated=True)
            ops.prepare_linear(down)

    def forward(self, ops, x, ctx):
        weights = torch.softmax(ops.dense(ops.linear(x, self.router)).float(), dim=-1)      # router in float32
        best = weights.argmax(-1)
        out = torch.zeros(x.shape[0], self.hidden, dtype=torch.float32, device=x.device)
        for e in range(len(self.widths)):
            rows = (best == e).nonzero().view(-1).to(torch.int32)
            if rows.numel() == 0:
                continue
            mine = ops.gather_rows(x, rows)
            y = ops.dense(ops.linear(ops.linear_silu_mul(mine, self.gate_up[e]), self.down[e])).float()
            out[rows.long()] = y * weights[rows.long(), e][:, None]
        return out.to(x.dtype)


class RoutedToyConfig:
    def __init__(self, data):
        self.hidden, self.vocab, self.heads = data["hidden"], data["vocab"], data["heads"]
        self.expert_sizes, self.max_positions = data["expert_sizes"], data["max_positions"]

    @classmethod
    def from_dict(cls, data):
        return cls(data)

    def model_spec(self):
        h = self.hidden
        norm = lambda p: PartSpec("rmsnorm", p, {"size": h, "eps": 1e-6})
        attention = lambda p: PartSpec("attention", p, {"hidden_size": h, "num_heads": self.heads, "num_kv_heads": self.heads,
                                                        "head_dim": h // self.heads, "qkv_bias": False})     # no position inside
        feed_forward = [PartSpec("swiglu", "l0.ffn.", {"hidden_size": h, "intermediate_size": 3 * h}),
                        PartSpec("test_best_of_experts", "l1.moe.", {"hidden_size": h, "expert_sizes": self.expert_sizes})]
        layers = [LayerSpec(PartSpec("prenorm_residual"), {
            "mixer": attention(f"l{l}.attn."), "feed_forward": feed_forward[l], "mixer_norm": norm(f"l{l}.n1."),
            "feed_forward_norm": norm(f"l{l}.n2.")}) for l in range(2)]
        sizes = {"vocab_size": self.vocab, "hidden_size": h}
        return ModelSpec("RoutedToyForCausalLM", self.vocab, h, self.max_positions, PartSpec("token_embedding", "emb.", sizes),
                         layers, (LayerCall(0), LayerCall(1)), norm("final."), PartSpec("lm_head", "head.", sizes),
                         position=PartSpec("test_learned_positions", "pos.", {"max_positions": self.max_positions,
                                                                              "hidden_size": h}))


def routed_toy_plain(weights, cfg, ids, first_position=0):
    """-> (logits, smallest gap between the two best router weights): float64, whole sequence, no cache."""
    w = {k: v.double() for k, v in weights.items()}
    n, h, heads = len(ids), cfg.hidden, cfg.heads
    x = w["emb.weight"][torch.tensor(ids)] + w["pos.weight"][first_position:first_position + n]
    rms = lambda t, p: plain.rms_norm(t, w[p + "weight"], 1e-6)

    def attention(t, p):
        q, k, v = ((t @ w[p + f"{name}_proj.weight"].T).view(n, heads, h // heads) for name in "qkv")
        return plain.attention(q, k, v).reshape(n, h) @ w[p + "o_proj.weight"].T

    swiglu = lambda t, p: plain.swiglu(t, w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"])
    x = x + attention(rms(x, "l0.n1."), "l0.attn.")
    x = x + swiglu(rms(x, "l0.n2."), "l0.ffn.")
    x = x + attention(rms(x, "l1.n1."), "l1.attn.")
    t = rms(x, "l1.n2.")
    route = torch.softmax(t @ w["l1.moe.router.weight"].T, -1)
    top = route.topk(2, dim=-1).values
    y = torch.stack([swiglu(t[i:i + 1], f"l1.moe.experts.{int(route[i].argmax())}.")[0] * route[i].max() for i in range(n)])
    x = x + y
    return rms(x, "final.") @ w["head.weight"].T, float((top[:, 0] - top[:, 1]).min())


def test_toy_architecture_with_learned_positions_and_a_routed_feed_forward(ops):
    register_part("position", "test_learned_positions", LearnedPositions)
    register_part("feed_forward", "test_best_of_experts", BestOfExperts)
    register_architecture("RoutedToyForCausalLM", RoutedToyConfig)
    from distie_amd.config import config_from_dict

    cfg = config_from_dict({"architectures": ["RoutedToyForCausalLM"], "hidden": 48, "vocab": 90, "heads": 3,
                            "expert_sizes": [40, 72, 24], "max_positions": 64})
    model = Model(cfg.model_spec())
    specs = model.param_specs()
    assert {"pos.weight", "l1.moe.router.weight", "l1.moe.experts.2.down_proj.weight", "l0.ffn.up_proj.weight",
            "head.weight"} <= set(specs)
    gen = torch.Generator().manual_seed(8)
    weights = {n: (torch.ones(s.shape) if s.init == "ones" else torch.randn(s.shape, generator=gen) * 0.25)
               for n, s in specs.items()}
    weights["l1.moe.router.weight"] *= 6.0          # decided choices: rounding must not flip an expert
    model.load_tensors(lambda name: weights[name].to(ops.device))
    cache = CacheManager(model.cache_requirements(), 4, 32, 4, device=ops.device, dtype=torch.float32)
    runner = ModelRunner(model, cache, ops, torch.float32, 64)
    a = torch.randint(0, 90, (29,), generator=gen).tolist()
    b = torch.randint(0, 90, (11,), generator=gen).tolist()
    (want_a, gap_a), (want_b, gap_b) = routed_toy_plain(weights, cfg, a), routed_toy_plain(weights, cfg, b)
    assert min(gap_a, gap_b) > 1e-3
    # the pin of the plain side: positions are absolute here, so a shift of all positions does change the result
    assert (routed_toy_plain(weights, cfg, a[:5], first_position=3)[0] - want_a[:5]).abs().max() > 1e-3
    got = runner.step([StepEntry("a", a, list(range(29)))]).cpu()
    assert (got - want_a.float()).abs().max() < 1e-4
    runner.finish("a")
    rows = {"a": [], "b": []}
    seqs = {"a": a, "b": b}
    for step in [[("a", 0, 6)], [("a", 6, 8), ("b", 0, 4)], [("a", 8, 27), ("b", 4, 5)], [("b", 5, 11), ("a", 27, 28)],
                 [("a", 28, 29)]]:
        logits = runner.step([StepEntry(r, seqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in step]).cpu()
        at = 0
        for r, lo, hi in step:
            rows[r].append(logits[at:at + hi - lo])
            at += hi - lo
    assert (torch.cat(rows["a"]) - want_a.float()).abs().max() < 1e-4
    assert (torch.cat(rows["b"]) - want_b.float()).abs().max() < 1e-4
    runner.finish("a")
    runner.finish("b")
    cache.check()


# ---------------------------------------------------------------------------------------------
# a third toy architecture: a norm of its own (centred, with a bias) and an arrangement of its own
# (post-norm: h = norm(h + sublayer(h))) in layer 0, beside the pre-norm RMS layer of the package in
# layer 1: norm and arrangement are chosen layer by layer like every other part
# ---------------------------------------------------------------------------------------------
from distie_amd.parts import Block, Norm   # noqa: E402


class CentredNorm(Norm):
    def __init__(self, spec):
        super().__init__(spec)
        self.size, self.eps = int(spec.params["size"]), float(spec.params["eps"])
        self.weight = self.bias = None

    def param_specs(self):
        return {"weight": ParamSpec((self.size,), "ones"), "bias": ParamSpec((self.size,))}

    def load(self, tensors):
        self.weight, self.bias = tensors["weight"].float(), tensors["bias"].float()

    def apply(self, ops, x, out_dtype):
        x = x.float()
        x = x - x.mean(-1, keepdim=True)
        return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight + self.bias).to(out_dtype)

    def add_apply(self, ops, residual, delta, out_dtype):
        residual += dense(ops, delta).float()
        return self.apply(ops, residual, out_dtype)


class PostNormResidual(Block):
    CHILDREN = {"mixer": "mixer", "mixer_norm": "norm", "feed_forward": "feed_forward", "feed_forward_norm": "norm"}

    def forward(self, ops, stream, ctx, cache, writes_cache):
        if stream.pending is not None:                   # what the layer before left to be added
            stream.hidden += dense(ops, stream.pending).float()
            stream.pending = None
        y = self.mixer.forward(ops, stream.hidden.to(ctx.act_dtype), ctx, cache["mixer"], writes_cache)
        stream.hidden = self.mixer_norm.apply(ops, stream.hidden + dense(ops, y).float(), torch.float32)
        y = self.feed_forward.forward(ops, stream.hidden.to(ctx.act_dtype), ctx)
        stream.hidden = self.feed_forward_norm.apply(ops, stream.hidden + dense(ops, y).float(), torch.float32)


class PostNormToyConfig:
    def __init__(self, data):
        self.hidden, self.vocab, self.heads, self.eps = data["hidden"], data["vocab"], data["heads"], data["eps"]

    @classmethod
    def from_dict(cls, data):
        return cls(data)

    def model_spec(self):
        h, d = self.hidden, self.hidden // self.heads
        centred = lambda p: PartSpec("test_centred_norm", p, {"size": h, "eps": self.eps})
        rms = lambda p: PartSpec("rmsnorm", p, {"size": h, "eps": self.eps})
        attention = lambda p: PartSpec("attention", p, {
            "hidden_size": h, "num_heads": self.heads, "num_kv_heads": 1, "head_dim": d, "qkv_bias": False,
            "position": PartSpec("rope", "", {"dim": d, "theta": 300.0})})
        ffn = lambda p: PartSpec("swiglu", p, {"hidden_size": h, "intermediate_size": 2 * h + 8})
        named = lambda mixer, feed_forward, n1, n2: {"mixer": mixer, "feed_forward": feed_forward, "mixer_norm": n1,
                                                    "feed_forward_norm": n2}
        layers = [LayerSpec(PartSpec("test_postnorm_residual"),
                            named(attention("l0.attn."), ffn("l0.ffn."), centred("l0.n1."), centred("l0.n2."))),
                  LayerSpec(PartSpec("prenorm_residual"),
                            named(attention("l1.attn."), ffn("l1.ffn."), rms("l1.n1."), rms("l1.n2.")))]
        sizes = {"vocab_size": self.vocab, "hidden_size": h}
        return ModelSpec("PostNormToyForCausalLM", self.vocab, h, 128, PartSpec("token_embedding", "emb.", sizes), layers,
                         (LayerCall(0), LayerCall(1)), centred("final."), PartSpec("lm_head", "head.", sizes))


def postnorm_toy_plain(weights, cfg, ids, norm_first=False):
    """float64, whole sequence, no cache. `norm_first`: layer 0 arranged pre-norm instead (the mistake the
    test must tell from the right arrangement)."""
    w = {k: v.double() for k, v in weights.items()}
    n, h = len(ids), cfg.hidden
    att_cfg = {"num_attention_heads": cfg.heads, "num_key_value_heads": 1, "head_dim": h // cfg.heads, "rope_theta": 300.0}

    def centred(t, p):
        t = t - t.mean(-1, keepdim=True)
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + cfg.eps) * w[p + "weight"] + w[p + "bias"]

    def attention(t, p):
        named = dict(w)
        for name, rows in (("q", h), ("k", h // cfg.heads), ("v", h // cfg.heads)):
            named[p + f"{name}_proj.bias"] = torch.zeros(rows, dtype=torch.float64)
        return plain.self_attention(t, named, p, torch.arange(n), att_cfg, None)

    ffn = lambda t, p: plain.swiglu(t, w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"])
    rms = lambda t, p: plain.rms_norm(t, w[p + "weight"], cfg.eps)
    x = w["emb.weight"][torch.tensor(ids)]
    if norm_first:
        x = x + attention(centred(x, "l0.n1."), "l0.attn.")
        x = x + ffn(centred(x, "l0.n2."), "l0.ffn.")
    else:
        x = centred(x + attention(x, "l0.attn."), "l0.n1.")
        x = centred(x + ffn(x, "l0.ffn."), "l0.n2.")
    x = x + attention(rms(x, "l1.n1."), "l1.attn.")
    x = x + ffn(rms(x, "l1.n2."), "l1.ffn.")
    return centred(x, "final.") @ w["head.weight"].T


def test_toy_architecture_with_a_norm_and_an_arrangement_of_its_own(ops):
    register_part("norm", "test_centred_norm", CentredNorm)
    register_part("block", "test_postnorm_residual", PostNormResidual)
    register_architecture("PostNormToyForCausalLM", PostNormToyConfig)
    from distie_amd.config import config_from_dict

    cfg = config_from_dict({"architectures": ["PostNormToyForCausalLM"], "hidden": 48, "vocab": 77, "heads": 3, "eps": 1e-4})
    model = Model(cfg.model_spec())
    specs = model.param_specs()
    assert {"l0.n1.bias", "l0.n2.weight", "final.bias", "l1.n1.weight"} <= set(specs) and "l1.n1.bias" not in specs
    gen = torch.Generator().manual_seed(21)
    weights = {n: (torch.ones(s.shape) + 0.2 * torch.randn(s.shape, generator=gen) if s.init == "ones"
                   else torch.randn(s.shape, generator=gen) * 0.25) for n, s in specs.items()}
    model.load_tensors(lambda name: weights[name].to(ops.device))
    cache = CacheManager(model.cache_requirements(), 4, 32, 4, device=ops.device, dtype=torch.float32)
    runner = ModelRunner(model, cache, ops, torch.float32, 64)
    a = torch.randint(0, 77, (23,), generator=gen).tolist()
    b = torch.randint(0, 77, (9,), generator=gen).tolist()
    want_a, want_b = postnorm_toy_plain(weights, cfg, a), postnorm_toy_plain(weights, cfg, b)
    # the pin of the plain side: the other arrangement of the same parts gives other logits
    assert (postnorm_toy_plain(weights, cfg, a, norm_first=True) - want_a).abs().max() > 1e-2
    got = runner.step([StepEntry("a", a, list(range(23)))]).cpu()
    assert (got - want_a.float()).abs().max() < 1e-4
    runner.finish("a")
    rows = {"a": [], "b": []}
    seqs = {"a": a, "b": b}
    for step in [[("a", 0, 5)], [("a", 5, 7), ("b", 0, 3)], [("a", 7, 22), ("b", 3, 4)], [("b", 4, 9), ("a", 22, 23)]]:
        logits = runner.step([StepEntry(r, seqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in step]).cpu()
        at = 0
        for r, lo, hi in step:
            rows[r].append(logits[at:at + hi - lo])
            at += hi - lo
    assert (torch.cat(rows["a"]) - want_a.float()).abs().max() < 1e-4
    assert (torch.cat(rows["b"]) - want_b.float()).abs().max() < 1e-4
    runner.finish("a")
    runner.finish("b")
    cache.check()


# ---------------------------------------------------------------------------------------------
# a fourth toy architecture: embeddings scaled by a constant and a head with a bias and capped logits;
# layer 0 arranged as a sandwich (a norm before and after each sub-layer: four norms) around a mixer that
# keeps one latent vector per token, and the token's position beside it as an integer, instead of keys and
# values; layer 1 is the package's pre-norm attention layer, so two kinds of pages live side by side. The
# latent mixer reads numbers back to the host and therefore says that it cannot be captured.
# ---------------------------------------------------------------------------------------------
from distie_amd.parts import PAGE, Embedding, Head, TensorDecl   # noqa: E402


class ScaledEmbedding(Embedding):
    def __init__(self, spec):
        super().__init__(spec)
        self.shape = (int(spec.params["vocab_size"]), int(spec.params["hidden_size"]))
        self.scale = float(spec.params["scale"])
        self.weight = None

    def param_specs(self):
        return {"weight": ParamSpec(self.shape)}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, ops, ids, meta):
        return ops.embed(ids, self.weight) * self.scale


class CappedBiasedHead(Head):
    def __init__(self, spec):
        super().__init__(spec)
        self.shape = (int(spec.params["vocab_size"]), int(spec.params["hidden_size"]))
        self.cap = float(spec.params["cap"])
        self.weight = self.bias = None

    def param_specs(self):
        return {"weight": ParamSpec(self.shape), "bias": ParamSpec(self.shape[:1])}

    def load(self, tensors):
        self.weight, self.bias = tensors["weight"], tensors["bias"].float()

    def forward(self, ops, normed):
        return self.cap * torch.tanh((ops.linear_f32out(normed, self.weight) + self.bias) / self.cap)


class SandwichBlock(Block):
    CHILDREN = {"before_mixer": "norm", "mixer": "mixer", "after_mixer": "norm",
                "before_feed_forward": "norm", "feed_forward": "feed_forward", "after_feed_forward": "norm"}

    def forward(self, ops, stream, ctx, cache, writes_cache):
        y = self.mixer.forward(ops, self.before_mixer.of_stream(ops, stream, ctx.act_dtype), ctx, cache["mixer"], writes_cache)
        stream.hidden += self.after_mixer.apply(ops, dense(ops, y).float(), torch.float32)
        y = self.feed_forward.forward(ops, self.before_feed_forward.apply(ops, stream.hidden, ctx.act_dtype), ctx)
        stream.hidden += self.after_feed_forward.apply(ops, dense(ops, y).float(), torch.float32)


class LatentMixer(Mixer):
    """c_t = x_t D is all that is kept of token t; y_t = softmax_j<=t(q_t . c_j / sqrt(R) - slope (t - j)) c_j U."""

    capturable = False

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden, self.rank, self.slope = int(spec.params["hidden_size"]), int(spec.params["rank"]), float(spec.params["slope"])
        self.down = self.query = self.up = None

    def cache_requirement(self):
        return PagedTensors((TensorDecl("latent", (PAGE, self.rank), torch.float32),
                             TensorDecl("stamp", (PAGE,), torch.int32)))

    def param_specs(self):
        return {"down.weight": ParamSpec((self.rank, self.hidden)), "query.weight": ParamSpec((self.rank, self.hidden)),
                "up.weight": ParamSpec((self.hidden, self.rank))}

    def load(self, tensors):
        self.down, self.query, self.up = (tensors[f"{n}.weight"].float() for n in ("down", "query", "up"))

    def forward(self, ops, x, ctx, cache, writes_cache):
        meta = ctx.meta
        latent, stamp = cache["latent"], cache["stamp"]
        assert latent.dtype == torch.float32 and stamp.dtype == torch.int32
        P = latent.shape[1]
        c = x.float() @ self.down.T
        q = x.float() @ self.query.T
        slots = meta.groups[cache.group].slots.long()
        if writes_cache:
            latent[slots // P, slots % P] = c
            stamp[slots // P, slots % P] = meta.positions
        table = meta.groups[cache.group].block_table.long()[meta.table_rows.long()]       # each request's own row
        out = torch.empty(x.shape[0], self.hidden, dtype=torch.float32, device=x.device)
        cu, positions = meta.cu_q.tolist(), meta.positions.tolist()          # the host waits here: not capturable
        for b in range(meta.num_requests):
            for t in range(cu[b], cu[b + 1]):
                keys = torch.arange(positions[t] + 1, device=x.device)
                pages = table[b, keys // P]
                assert bool((pages >= 0).all()) and torch.equal(stamp[pages, keys % P].long(), keys), "a wrong page was read"
                kept = latent[pages, keys % P]
                scores = kept @ q[t] / self.rank ** 0.5 - self.slope * (positions[t] - keys).float()
                out[t] = (torch.softmax(scores, 0) @ kept) @ self.up.T
        return out.to(x.dtype)


class SandwichToyConfig:
    def __init__(self, data):
        self.hidden, self.vocab, self.rank, self.cap, self.slope = (data[k] for k in ("hidden", "vocab", "rank", "cap", "slope"))

    @classmethod
    def from_dict(cls, data):
        return cls(data)

    def model_spec(self):
        h = self.hidden
        norm = lambda p: PartSpec("rmsnorm", p, {"size": h, "eps": 1e-5})
        ffn = lambda p: PartSpec("swiglu", p, {"hidden_size": h, "intermediate_size": 3 * h})
        sandwich = LayerSpec(PartSpec("test_sandwich"), {
            "before_mixer": norm("l0.n1."), "after_mixer": norm("l0.n2."), "before_feed_forward": norm("l0.n3."),
            "after_feed_forward": norm("l0.n4."), "feed_forward": ffn("l0.ffn."),
            "mixer": PartSpec("test_latent", "l0.mix.", {"hidden_size": h, "rank": self.rank, "slope": self.slope})})
        usual = LayerSpec(PartSpec("prenorm_residual"), {
            "mixer_norm": norm("l1.n1."), "feed_forward_norm": norm("l1.n2."), "feed_forward": ffn("l1.ffn."),
            "mixer": PartSpec("attention", "l1.attn.", {"hidden_size": h, "num_heads": 2, "num_kv_heads": 2, "head_dim": h // 2,
                                                        "qkv_bias": False,
                                                        "position": PartSpec("rope", "", {"dim": h // 2, "theta": 50.0})})})
        sizes = {"vocab_size": self.vocab, "hidden_size": h}
        return ModelSpec("SandwichToyForCausalLM", self.vocab, h, 128,
                         PartSpec("test_scaled_embedding", "emb.", dict(sizes, scale=h ** 0.5)), (sandwich, usual),
                         (LayerCall(0), LayerCall(1)), norm("final."),
                         PartSpec("test_capped_head", "head.", dict(sizes, cap=self.cap)))


def sandwich_toy_plain(weights, cfg, ids, scaled=True):
    """float64, whole sequence, no cache. `scaled=False` leaves the embeddings unscaled (the mistake that the
    test must tell from the right model)."""
    w = {k: v.double() for k, v in weights.items()}
    n, h = len(ids), cfg.hidden
    rms = lambda t, p: plain.rms_norm(t, w[p + "weight"], 1e-5)
    ffn = lambda t, p: plain.swiglu(t, w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"])
    x = w["emb.weight"][torch.tensor(ids)] * (h ** 0.5 if scaled else 1.0)
    t = rms(x, "l0.n1.")
    c, q = t @ w["l0.mix.down.weight"].T, t @ w["l0.mix.query.weight"].T
    place = torch.arange(n, dtype=torch.float64)
    scores = q @ c.T / cfg.rank ** 0.5 - cfg.slope * (place[:, None] - place[None, :])
    scores = scores.masked_fill(place[None, :] > place[:, None], float("-inf"))
    x = x + rms((torch.softmax(scores, -1) @ c) @ w["l0.mix.up.weight"].T, "l0.n2.")
    x = x + rms(ffn(rms(x, "l0.n3."), "l0.ffn."), "l0.n4.")
    named = dict(w)
    for name in "qkv":
        named[f"l1.attn.{name}_proj.bias"] = torch.zeros(h, dtype=torch.float64)
    att_cfg = {"num_attention_heads": 2, "num_key_value_heads": 2, "head_dim": h // 2, "rope_theta": 50.0}
    x = x + plain.self_attention(rms(x, "l1.n1."), named, "l1.attn.", torch.arange(n), att_cfg, None)
    x = x + ffn(rms(x, "l1.n2."), "l1.ffn.")
    return cfg.cap * torch.tanh((rms(x, "final.") @ w["head.weight"].T + w["head.bias"]) / cfg.cap)


def test_toy_architecture_with_four_norms_a_latent_cache_and_ends_of_its_own(ops):
    register_part("embedding", "test_scaled_embedding", ScaledEmbedding)
    register_part("head", "test_capped_head", CappedBiasedHead)
    register_part("block", "test_sandwich", SandwichBlock)
    register_part("mixer", "test_latent", LatentMixer)
    register_architecture("SandwichToyForCausalLM", SandwichToyConfig)
    from distie_amd.config import config_from_dict

    data = {"architectures": ["SandwichToyForCausalLM"], "hidden": 32, "vocab": 61, "rank": 12, "cap": 5.0, "slope": 0.3}
    cfg = config_from_dict(data)
    model = Model(cfg.model_spec())
    specs = model.param_specs()
    assert {"l0.n1.weight", "l0.n2.weight", "l0.n3.weight", "l0.n4.weight", "l0.mix.down.weight", "head.bias",
            "emb.weight", "l1.attn.o_proj.weight"} <= set(specs)
    assert not model.capturable and Model(config_from_dict(plain.TINY_A).model_spec()).capturable
    gen = torch.Generator().manual_seed(31)
    weights = {n: (torch.ones(s.shape) + 0.2 * torch.randn(s.shape, generator=gen) if s.init == "ones"
                   else torch.randn(s.shape, generator=gen) * 0.2) for n, s in specs.items()}
    model.load_tensors(lambda name: weights[name].to(ops.device))
    needs = model.cache_requirements()
    assert [t.name for t in needs[0]["mixer"].tensors] == ["latent", "stamp"] and needs[1] == {"mixer": PagedKV(2, 16)}
    cache = CacheManager(needs, 4, 24, 4, device=ops.device, dtype=torch.float32)
    assert len(cache.groups) == 2 and cache.groups[0].tensors["latent"].shape == (1, 25, 4, 12) and \
        cache.groups[0].tensors["stamp"].dtype == torch.int32 and cache.groups[1].tensors["v"].shape == (1, 25, 2, 16, 4)
    for group in cache.groups:                   # stale pages must not be read: poison what can be poisoned
        for slab in group.tensors.values():
            slab.fill_(float("nan") if slab.dtype.is_floating_point else -5)
    runner = ModelRunner(model, cache, ops, torch.float32, 128)
    a = torch.randint(0, 61, (23,), generator=gen).tolist()
    b = torch.randint(0, 61, (9,), generator=gen).tolist()
    want_a, want_b = sandwich_toy_plain(weights, cfg, a).float(), sandwich_toy_plain(weights, cfg, b).float()
    assert (sandwich_toy_plain(weights, cfg, a, scaled=False).float() - want_a).abs().max() > 1e-2
    assert want_a.abs().max() < 5.0 and want_a.abs().max() > 2.0          # the cap bends the logits
    got = runner.step([StepEntry("a", a, list(range(23)))]).cpu()
    assert (got - want_a).abs().max() < 1e-4
    runner.finish("a")
    rows = {"a": [], "b": []}
    seqs = {"a": a, "b": b}
    for step in [[("a", 0, 5)], [("a", 5, 7), ("b", 0, 3)], [("a", 7, 22), ("b", 3, 4)], [("b", 4, 9), ("a", 22, 23)]]:
        logits = runner.step([StepEntry(r, seqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in step]).cpu()
        at = 0
        for r, lo, hi in step:
            rows[r].append(logits[at:at + hi - lo])
            at += hi - lo
    assert (torch.cat(rows["a"]) - want_a).abs().max() < 1e-4
    assert (torch.cat(rows["b"]) - want_b).abs().max() < 1e-4
    runner.finish("a")
    runner.finish("b")
    cache.check()
    assert cache.free_pages() == [24, 24]
    # through the entry point: the registry finds the architecture, and a model with a part that cannot be
    # captured runs its decode steps uncaptured, whatever the options ask for
    from distie_amd import LLM, SamplingParams

    llm = LLM(config=data, random_weights=True, seed=5, ops=ops, dtype="fp32", block_size=4, num_blocks=24, max_seqs=4,
              use_graphs=True)
    assert llm.runner.graphs is None
    outs = llm.generate([a[:6], b[:3]], SamplingParams(max_new_tokens=5))
    assert [len(o.token_ids) for o in outs] == [5, 5] and all(o.finish_reason == "length" for o in outs)
    again = llm.generate([a[:6]], SamplingParams(max_new_tokens=5))
    assert again[0].token_ids == outs[0].token_ids
