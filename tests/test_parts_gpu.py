"""Each part alone against its plain twin; the run order and the cache groups as
data (a layer run twice, a layer reading another's cache, a windowed layer); and a
toy mixer with state of its own, defined here, registered, built and stepped
without touching the framework's files."""
import math
from dataclasses import dataclass, replace

import numpy as np
import pytest
import torch

import trace_util as tu
from conftest import TINY_A

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def kslot(keys, ps, hd, s):
    """Where the cache keeps the key of slot s of one (page, head): `keys` is that head's
    ps * hd elements; chunks of 16 dims lie together ([hd / 16][slot][16]) where hd is a
    multiple of 16, else a key's dims in a row.  A view of shape [hd / chunk, chunk]: assign
    `k.view(-1, chunk)` to it, or read it with `.reshape(hd)`."""
    kc = 16 if hd % 16 == 0 else hd
    return keys.view(hd // kc, ps, kc)[:, s, :]


def vslot(s):
    """Where the cache keeps slot s of a value column: bits 2 and 3 exchanged."""
    return (s & ~12) | ((s & 4) << 1) | ((s & 8) >> 1)


def rel(a, b):
    a = a.double().cpu() if isinstance(a, torch.Tensor) else torch.as_tensor(np.asarray(a)).double()
    b = b.double().cpu() if isinstance(b, torch.Tensor) else torch.as_tensor(np.asarray(b)).double()
    return float((a - b).abs().max() / b.abs().max())


# ---------------------------------------------------------------- parts alone ---

def _one_layer_engine(cfg_json, dtype, seed=3):
    """An engine over a model of the given configuration; its parts are then called
    one by one with a real step context."""
    import hfee_amd  # noqa: F401
    from hfee_amd.config import config_from_dict
    from hfee_amd.engine import Engine, random_model
    cfg = config_from_dict(cfg_json)
    model = random_model(cfg, seed=seed, dtype=dtype, device=DEV, std=0.1)
    return cfg, model, Engine(model, num_pages=32, page_size=16, max_requests=2, max_batch_tokens=128, use_graphs=False)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_part_alone(dtype):
    """Sizes unlike any tiny configuration: 10 heads on 5 KV heads of 80, width 112."""
    from plain_llama import plain_attention, plain_matmul, plain_rope, plain_rope_frequencies
    from hfee_amd.engine import StepEntry
    cj = dict(TINY_A, hidden_size=112, num_attention_heads=10, num_key_value_heads=5, head_dim=80,
              num_hidden_layers=1, rope_theta=777.0)
    cfg, model, eng = _one_layer_engine(cj, dtype)
    att = model.blocks[0].mixer
    T = 45
    g = torch.Generator().manual_seed(1)
    h = (torch.randn(T, 112, generator=g)).to(model.dtype)
    x0 = torch.randn(T, 112, generator=g)
    eng.admit("r")
    entries = [StepEntry("r", [1] * T, [])]
    ctx, _, _ = eng.begin(entries)
    x = x0.clone().to(DEV)
    att.forward_add(ctx, x, h.to(DEV), cache_layer=0, writes_cache=True)
    eng.commit(entries)
    H, K, hd = 10, 5, 80
    wq, wk, wv = att.w_qkv.double().cpu().split([H * hd, K * hd, K * hd])
    inv = plain_rope_frequencies(hd, 777.0)
    # the part keeps q and k rows with rotation pairs side by side (2i, 2i+1)
    q = plain_rope(plain_matmul(h, wq).reshape(T, H, hd), range(T), inv, "interleaved")
    k = plain_rope(plain_matmul(h, wk).reshape(T, K, hd), range(T), inv, "interleaved")
    v = plain_matmul(h, wv).reshape(T, K, hd)
    want = x0.double() + plain_matmul(plain_attention(q, k, v).reshape(T, H * hd), att.w_o.double().cpu())
    assert rel(x, want) < (2e-5 if dtype == "float32" else 3e-2)
    # the same tokens one at a time on a second request give the same rows
    eng.admit("s")
    xs = []
    for t in range(T):
        entries = [StepEntry("s", [1], [])]
        ctx, _, _ = eng.begin(entries)
        xt = x0[t:t + 1].clone().to(DEV)
        att.forward_add(ctx, xt, h[t:t + 1].to(DEV), 0, True)
        eng.commit(entries)
        xs.append(xt.cpu())
    assert rel(torch.cat(xs), want) < (2e-5 if dtype == "float32" else 3e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_feed_forward_norm_embedding_and_head_alone(dtype):
    from plain_llama import plain_matmul, plain_rmsnorm, plain_swiglu
    from hfee_amd.engine import StepEntry
    cj = dict(TINY_A, hidden_size=72, intermediate_size=100, vocab_size=301, num_attention_heads=3,
              num_key_value_heads=3, head_dim=16, num_hidden_layers=1, rms_norm_eps=3e-4, tie_word_embeddings=False)
    cfg, model, eng = _one_layer_engine(cj, dtype)
    tol = 2e-5 if dtype == "float32" else 3e-2
    T = 19
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, 301, (T,), generator=g).tolist()
    eng.admit("r")
    entries = [StepEntry("r", ids, [0, T - 1])]
    ctx, w, _ = eng.begin(entries)
    # embedding
    x = torch.empty(T, 72, dtype=torch.float32, device=DEV)
    model.embedding.forward(ctx, x)
    assert torch.equal(x.cpu(), model.embedding.table.float().cpu()[ids])
    # norm
    blk = model.blocks[0]
    xin = torch.randn(T, 72, generator=g) * 2
    h = torch.empty(T, 72, dtype=model.dtype, device=DEV)
    blk.mixer_norm.forward(ctx, h, xin.to(DEV))
    assert rel(h, plain_rmsnorm(xin, blk.mixer_norm.weight.cpu(), 3e-4)) < tol
    # feed-forward
    ff = blk.feed_forward
    hin = torch.randn(T, 72, generator=g).to(model.dtype)
    xr = xin.clone().to(DEV)
    ff.forward_add(ctx, xr, hin.to(DEV))
    wg, wu = ff.w_gate_up.double().cpu()[0::2], ff.w_gate_up.double().cpu()[1::2]     # rows alternate gate, up
    want = xin.double() + plain_matmul(plain_swiglu(plain_matmul(hin, wg), plain_matmul(hin, wu)), ff.w_down.double().cpu())
    assert rel(xr, want) < tol
    # head: final norm and vocabulary product on the wanted rows only
    logits = torch.empty(2, 301, dtype=torch.float32, device=DEV)
    model.head.forward(ctx, logits, xin.to(DEV), ctx.extra["logit_rows"])
    want = plain_matmul(plain_rmsnorm(xin[[0, T - 1]], model.head.norm.weight.cpu(), 3e-4), model.head.weight.double().cpu())
    assert rel(logits, want) < tol
    eng.commit(entries)


def test_rotary_part_tables():
    from plain_llama import plain_rope_frequencies
    from hfee_amd.config.specs import PositionSpec, params
    from hfee_amd.parts import Rotary
    rot = Rotary(PositionSpec("rope", params(head_dim=64, rotary_dim=64, theta=500000.0,
                                             scaling=("llama3", 8.0, 1.0, 4.0, 8192), pairing="half")))
    rot.prepare(9000, DEV)
    inv = plain_rope_frequencies(64, 500000.0, dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                                    original_max_position_embeddings=8192))
    p = 8191
    assert torch.allclose(rot.cos[p].double().cpu(), torch.cos(p * inv), atol=1e-7)
    assert torch.allclose(rot.sin[p].double().cpu(), torch.sin(p * inv), atol=1e-7)
    with pytest.raises(ValueError, match="pairing"):
        Rotary(PositionSpec("rope", params(head_dim=8, theta=1.0, pairing="odd")))


# ------------------------------------------------ run order and cache groups ---

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layer_twice_shared_cache_and_window(model_folders, dtype):
    """Schedule: layer 0, layer 1 (window 24, own group), layer 0 again with a cache of
    its own, layer 1 again reading the cache its first run wrote."""
    from plain_llama import PlainLlama
    import hfee_amd  # noqa: F401
    from hfee_amd.config import config_from_folder, model_spec_of
    from hfee_amd.config.specs import MixerSpec, ScheduleEntry
    from hfee_amd.engine import Engine, Model, StepEntry
    from hfee_amd.weights import load_tensors
    folder = model_folders[("A", dtype)]
    cfg = config_from_folder(folder)
    spec = model_spec_of(cfg)
    m1 = spec.layers[1].mixer
    windowed = MixerSpec(m1.kind, tuple(sorted(dict(m1.params, window=24).items())), m1.position)
    spec = replace(spec, layers=(spec.layers[0], replace(spec.layers[1], mixer=windowed)),
                   schedule=(ScheduleEntry(0, 0), ScheduleEntry(1, 1), ScheduleEntry(0, 2), ScheduleEntry(1, 1, False)))
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    model = Model(spec, dt)
    model.bind(load_tensors(folder, model.tensor_specs(), dt, DEV))
    eng = Engine(model, num_pages=[16, 6], page_size=16, max_requests=2, max_batch_tokens=64)
    assert sorted(g.kind for g in eng.groups) == ["full", "window"]
    toks = tu.make_requests(256, [120], seed=8)["r0"]
    want = PlainLlama(folder).forward(toks, schedule=[(0, 0, True), (1, 1, True), (0, 2, True), (1, 1, False)],
                                      windows={1: 24})
    tol = 3e-5 if dtype == "float32" else 5e-2
    eng.admit("r")
    got, i = [], 0
    for n in [7, 16, 2, 33, 1, 1, 1, 20, 5, 34]:          # portions, some decode steps
        got.append(eng.step([StepEntry("r", toks[i:i + n], list(range(n)))]).cpu().clone())
        i += n
        eng.cache.check()
    assert i == 120
    assert rel(torch.cat(got), want) < tol
    # the window group never held more than its window needs: 6 pages were enough for 120 tokens
    win = [g for g, s in enumerate(eng.groups) if s.kind == "window"][0]
    assert sum(p >= 0 for p in eng.cache.block_table("r", win)) <= 3
    eng.release("r")
    eng.cache.check()


# ----------------------------------------------------------- a toy mixer ---

def test_toy_mixer_with_state_registers_builds_and_steps(tmp_path):
    """A mixer with per-request state of fixed size (an exponential moving average of
    its input, then a projection), in a toy architecture that alternates it with
    attention.  Everything toy is defined here."""
    import hfee_amd  # noqa: F401
    from hfee_amd.config import (ConfigError, FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                                 ScheduleEntry, config_from_folder, params, register_architecture)
    from hfee_amd.config.base import KeyReader
    from hfee_amd.engine import Engine, StepEntry, load_model
    from hfee_amd.parts import Mixer, register_mixer
    from hfee_amd.weights import TensorSpec, write_model_folder

    @register_mixer("toy_ema")
    class ToyEma(Mixer):
        def __init__(self, spec, prefix, dtype):
            self.hidden, self.decay, self.prefix, self.dtype = spec.get("hidden"), spec.get("decay"), prefix, dtype
            self.state_name = prefix + "state"

        def tensor_specs(self):
            return [TensorSpec(self.prefix + "proj.weight", (self.hidden, self.hidden))]

        def bind(self, tensors):
            self.w = tensors.pop(self.prefix + "proj.weight")

        def state_specs(self):
            return [(self.state_name, (self.hidden,), torch.float32)]

        def prepare(self, info):
            self.state = info.storage.states[self.state_name]

        def forward_add(self, ctx, x, h, cache_layer, writes_cache):
            for seg in ctx.segments:                      # tokens of a request in order: state feeds on
                s = self.state[seg.slot]
                for r in range(seg.row0, seg.row0 + seg.length):
                    s.mul_(self.decay).add_(h[r].float(), alpha=1 - self.decay)
                    x[r] += (self.w.float() @ s)

    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str
        hidden: int
        layers: int
        vocab: int
        decay: float

        @staticmethod
        def from_dict(d, where="config.json"):
            r = KeyReader(d, where)
            c = ToyConfig("ToyForCausalLM", r.int("toy_hidden"), r.int("toy_layers"), r.int("toy_vocab"), r.float("toy_decay"))
            r.finish()
            return c

        def to_dict(self):
            return {"architectures": ["ToyForCausalLM"], "toy_hidden": self.hidden, "toy_layers": self.layers,
                    "toy_vocab": self.vocab, "toy_decay": self.decay}

    def toy_spec(c):
        norm = NormSpec("rmsnorm", c.hidden, 1e-5)
        ffn = FeedForwardSpec("gated_mlp", params(hidden=c.hidden, intermediate=2 * c.hidden, activation="silu"))
        ema = MixerSpec("toy_ema", params(hidden=c.hidden, decay=c.decay))
        att = MixerSpec("attention", params(hidden=c.hidden, num_heads=2, num_kv_heads=1, head_dim=16, scale=0.25, window=0),
                        position=PositionSpec("rope", params(head_dim=16, rotary_dim=16, theta=100.0, scaling=None, pairing="half")))
        layers = tuple(LayerSpec("prenorm", c.hidden, ema if i % 2 == 0 else att, ffn, norm, norm, f"toy.{i}.")
                       for i in range(c.layers))
        return ModelSpec("ToyForCausalLM", c.hidden, c.vocab, layers, tuple(ScheduleEntry(i, i) for i in range(c.layers)),
                         norm, "toy.embed.weight", "toy.norm.weight", None, max_positions=512)

    register_architecture("ToyForCausalLM", ToyConfig, toy_spec)
    cfg = ToyConfig("ToyForCausalLM", 48, 3, 90, 0.75)
    folder = write_model_folder(str(tmp_path / "toy"), cfg, seed=1, std=0.1)
    assert config_from_folder(folder) == cfg
    model, _ = load_model(folder, "float32")
    eng = Engine(model, num_pages=16, page_size=16, max_requests=2, max_batch_tokens=64)
    assert not eng.use_graphs, "a part that reads host data keeps the model eager"
    assert len(eng.groups) == 1 and eng.groups[0].cache_layers == (1,)
    assert set(eng.storage.states) == {"toy.0.mixer.state", "toy.2.mixer.state"}

    toks = tu.make_requests(90, [40, 23], seed=3)
    eng.admit("a")
    whole = eng.step([StepEntry("a", toks["r0"], list(range(40)))]).cpu().clone()
    eng.release("a")
    # in portions, beside another request, on the slot that "a" used: the state starts from zero again
    eng.admit("b")
    eng.admit("c")
    got, i, ci = [], 0, 0
    for n in [5, 1, 1, 13, 2, 18]:
        entries = [StepEntry("b", toks["r0"][i:i + n], list(range(n)))]
        if ci < len(toks["r1"]):
            entries.insert(0, StepEntry("c", toks["r1"][ci:ci + 3], []))
            ci += 3
        got.append(eng.step(entries).cpu().clone())
        i += n
    assert torch.allclose(torch.cat(got), whole, atol=1e-5, rtol=1e-5)

    # the plain twin of the toy model's first layer, to show that the state is what it should be
    w = model.blocks[0].mixer.w.double().cpu()
    from plain_llama import plain_rmsnorm
    emb = model.embedding.table.double().cpu()[toks["r0"]]
    h = plain_rmsnorm(emb, model.blocks[0].mixer_norm.weight.cpu(), 1e-5)
    s = torch.zeros(48, dtype=torch.float64)
    for t in range(40):
        s = 0.75 * s + 0.25 * h[t]
    assert torch.allclose(eng.storage.states["toy.0.mixer.state"][eng.cache.get("b").slot].double().cpu(), s, atol=1e-5)
    with pytest.raises(ConfigError, match="toy_hidden"):
        ToyConfig.from_dict({"architectures": ["ToyForCausalLM"]})


def test_toy_routed_feed_forward_and_toy_position_encoding(tmp_path):
    """A feed-forward that routes every token to one of three experts, and a position
    encoding that is not the architecture's (rotation by sqrt(position) * frequency), in
    a toy architecture; both registered here, built by the registries, stepped in
    portions and compared with a plain computation.  Nothing of the framework changes."""
    import numpy as np
    import hfee_amd  # noqa: F401
    from hfee_amd.config import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                                 ScheduleEntry, params, register_architecture)
    from hfee_amd.config.base import KeyReader
    from hfee_amd.engine import Engine, StepEntry, load_model
    from hfee_amd.parts import FeedForward, Part, register_feed_forward, register_position
    from hfee_amd.weights import TensorSpec, write_model_folder
    from plain_llama import plain_attention, plain_rmsnorm, plain_rope

    @register_position("toy_sqrt_rope")
    class SqrtRope(Part):
        def __init__(self, spec):
            self.head_dim = self.rotary_dim = spec.get("head_dim")
            self.base = float(spec.get("base"))
            self.pairing = 0               # pairs (i, i + head_dim / 2)
            self.cos = self.sin = None

        def signature(self):
            return ("toy_sqrt_rope", self.head_dim, self.base)

        def frequencies(self):
            return np.array([self.base ** (-2 * i / self.head_dim) for i in range(self.head_dim // 2)])

        def prepare(self, num_positions, device):
            angles = np.sqrt(np.arange(num_positions, dtype=np.float64))[:, None] * self.frequencies()[None, :]
            self.cos = torch.from_numpy(np.cos(angles).astype(np.float32)).to(device)
            self.sin = torch.from_numpy(np.sin(angles).astype(np.float32)).to(device)

    @register_feed_forward("toy_top1_experts")
    class Top1Experts(FeedForward):
        def __init__(self, spec, prefix, dtype):
            self.hidden, self.experts, self.prefix = spec.get("hidden"), spec.get("experts"), prefix

        def tensor_specs(self):
            return [TensorSpec(self.prefix + "router.weight", (self.experts, self.hidden)),
                    TensorSpec(self.prefix + "experts.weight", (self.experts * self.hidden, self.hidden))]

        def bind(self, tensors):
            self.router = tensors.pop(self.prefix + "router.weight")
            self.w = tensors.pop(self.prefix + "experts.weight").view(self.experts, self.hidden, self.hidden)

        def forward_add(self, ctx, x, h):
            choice = (h.float() @ self.router.float().t()).argmax(-1)          # router logits in 32-bit
            for e in range(self.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    x[rows] += h[rows].float() @ self.w[e].float().t()

    @dataclass(frozen=True)
    class RoutedConfig:
        architecture: str
        hidden: int
        layers: int
        vocab: int
        experts: int

        @staticmethod
        def from_dict(d, where="config.json"):
            r = KeyReader(d, where)
            c = RoutedConfig("ToyRoutedForCausalLM", r.int("r_hidden"), r.int("r_layers"), r.int("r_vocab"), r.int("r_experts"))
            r.finish()
            return c

        def to_dict(self):
            return {"architectures": ["ToyRoutedForCausalLM"], "r_hidden": self.hidden, "r_layers": self.layers,
                    "r_vocab": self.vocab, "r_experts": self.experts}

    H, KV, HD = 3, 1, 16

    def routed_spec(c):
        norm = NormSpec("rmsnorm", c.hidden, 1e-6)
        ffn = FeedForwardSpec("toy_top1_experts", params(hidden=c.hidden, experts=c.experts))
        att = MixerSpec("attention", params(hidden=c.hidden, num_heads=H, num_kv_heads=KV, head_dim=HD, scale=0.2, window=0),
                        position=PositionSpec("toy_sqrt_rope", params(head_dim=HD, base=50.0)))
        layers = tuple(LayerSpec("prenorm", c.hidden, att, ffn, norm, norm, f"r.{i}.") for i in range(c.layers))
        return ModelSpec("ToyRoutedForCausalLM", c.hidden, c.vocab, layers, tuple(ScheduleEntry(i, i) for i in range(c.layers)),
                         norm, "r.embed.weight", "r.norm.weight", None, max_positions=256)

    register_architecture("ToyRoutedForCausalLM", RoutedConfig, routed_spec)
    cfg = RoutedConfig("ToyRoutedForCausalLM", 40, 2, 70, 3)
    folder = write_model_folder(str(tmp_path / "routed"), cfg, seed=5, std=0.2)
    model, _ = load_model(folder, "float32")
    eng = Engine(model, num_pages=8, page_size=16, max_requests=2, max_batch_tokens=64)
    toks = tu.make_requests(70, [45], seed=8)["r0"]
    eng.admit("a")
    got, i = [], 0
    for n in [7, 1, 20, 2, 15]:
        got.append(eng.step([StepEntry("a", toks[i:i + n], list(range(n)))]).double().cpu())
        i += n
    got = torch.cat(got)

    # the plain computation, whole sequence, float64
    from hfee_amd.weights import Checkpoint
    ck = Checkpoint(folder)
    t = {n: ck.tensor(n).double() for n in ck.names()}
    x = t["r.embed.weight"][toks]
    pos = list(range(len(toks)))
    inv_freq = torch.tensor([50.0 ** (-2 * j / HD) for j in range(HD // 2)], dtype=torch.float64)
    used = set()
    for l in range(cfg.layers):
        p = f"r.{l}."
        h = plain_rmsnorm(x, t[p + "mixer_norm.weight"], 1e-6)
        q = (h @ t[p + "mixer.q_proj.weight"].t()).view(-1, H, HD)
        k = (h @ t[p + "mixer.k_proj.weight"].t()).view(-1, KV, HD)
        v = (h @ t[p + "mixer.v_proj.weight"].t()).view(-1, KV, HD)
        sqrt_pos = [math.sqrt(i) for i in pos]
        q, k = plain_rope(q, sqrt_pos, inv_freq, "half"), plain_rope(k, sqrt_pos, inv_freq, "half")
        x = x + plain_attention(q, k, v, 0.2).reshape(len(toks), H * HD) @ t[p + "mixer.o_proj.weight"].t()
        h = plain_rmsnorm(x, t[p + "feed_forward_norm.weight"], 1e-6)
        choice = (h @ t[p + "feed_forward.router.weight"].t()).argmax(-1)
        used |= set(choice.tolist())
        w = t[p + "feed_forward.experts.weight"].view(cfg.experts, cfg.hidden, cfg.hidden)
        x = x + torch.stack([h[r] @ w[int(choice[r])].t() for r in range(len(toks))])
    want = plain_rmsnorm(x, t["r.norm.weight"], 1e-6) @ t["r.embed.weight"].t()
    assert len(used) > 1, "the test is meant to route to more than one expert"
    assert torch.allclose(got, want, atol=2e-4, rtol=2e-4), float((got - want).abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_step_between_the_projections_and_the_rotation(tmp_path, dtype):
    """A bias on q, k and v and a norm over each head of q and k with a weight per dimension,
    between the projections and the rotation: defined and registered here as a
    `projection_step`, named by the attention mixer's `after_projection` parameter in a toy
    architecture, stepped in portions and token by token (the mixer then runs projections,
    this step and the rotation as launches of their own) and compared with a plain computation.
    The rows of a q or k head lie in the mixer's own order; the step's tensors follow it."""
    import hfee_amd  # noqa: F401
    from hfee_amd.config import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                                 ScheduleEntry, params, register_architecture)
    from hfee_amd.config.base import KeyReader
    from hfee_amd.engine import Engine, StepEntry, load_model
    from hfee_amd.parts import ProjectionStep, register_projection_step
    from hfee_amd.weights import Checkpoint, TensorSpec, write_model_folder
    from plain_llama import plain_attention, plain_rmsnorm, plain_rope, plain_rope_frequencies, plain_swiglu

    @register_projection_step("toy_bias_and_head_norm")
    class BiasAndHeadNorm(ProjectionStep):
        def __init__(self, options, prefix, num_heads, kv_heads, head_dim, dtype):
            self.prefix, self.H, self.K, self.hd, self.eps = prefix, num_heads, kv_heads, head_dim, options["eps"]

        def tensor_specs(self):
            p = self.prefix
            return [TensorSpec(p + "q_proj.bias", (self.H * self.hd,), role="vector", init=("normal",)),
                    TensorSpec(p + "k_proj.bias", (self.K * self.hd,), role="vector", init=("normal",)),
                    TensorSpec(p + "v_proj.bias", (self.K * self.hd,), role="vector", init=("normal",)),
                    TensorSpec(p + "q_norm.weight", (self.hd,), role="vector", init=("one_plus_normal",)),
                    TensorSpec(p + "k_norm.weight", (self.hd,), role="vector", init=("one_plus_normal",))]

        def bind(self, tensors, order=None):
            p = self.prefix
            self.bq = tensors.pop(p + "q_proj.bias").float().view(self.H, self.hd)[:, order].reshape(-1)
            self.bk = tensors.pop(p + "k_proj.bias").float().view(self.K, self.hd)[:, order].reshape(-1)
            self.bv = tensors.pop(p + "v_proj.bias").float()
            self.wq = tensors.pop(p + "q_norm.weight").float()[order]
            self.wk = tensors.pop(p + "k_norm.weight").float()[order]

        def forward(self, ctx, q, k, v):
            def head_norm(t, bias, w, heads):
                y = (t.float() + bias).view(t.shape[0], heads, self.hd)
                y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + self.eps) * w
                t.copy_(y.view(t.shape[0], -1))
            head_norm(q, self.bq, self.wq, self.H)
            if k is not None:
                head_norm(k, self.bk, self.wk, self.K)
                v.copy_(v.float() + self.bv)

    @dataclass(frozen=True)
    class StepConfig:
        architecture: str
        hidden: int
        vocab: int

        @staticmethod
        def from_dict(d, where="config.json"):
            r = KeyReader(d, where)
            c = StepConfig("ToyStepForCausalLM", r.int("s_hidden"), r.int("s_vocab"))
            r.finish()
            return c

        def to_dict(self):
            return {"architectures": ["ToyStepForCausalLM"], "s_hidden": self.hidden, "s_vocab": self.vocab}

    H, KV, HD, F, EPS = 4, 2, 32, 56, 1e-5

    def spec_of(c):
        norm = NormSpec("rmsnorm", c.hidden, EPS)
        ffn = FeedForwardSpec("gated_mlp", params(hidden=c.hidden, intermediate=F))
        att = MixerSpec("attention", params(hidden=c.hidden, num_heads=H, num_kv_heads=KV, head_dim=HD, window=0,
                                            after_projection=("toy_bias_and_head_norm", params(eps=1e-3))),
                        position=PositionSpec("rope", params(head_dim=HD, theta=10000.0, rotary_dim=HD, pairing="half", scaling=None)))
        layers = tuple(LayerSpec("prenorm", c.hidden, att, ffn, norm, norm, f"s.{i}.") for i in range(2))
        return ModelSpec("ToyStepForCausalLM", c.hidden, c.vocab, layers, tuple(ScheduleEntry(i, i) for i in range(2)),
                         norm, "s.embed.weight", "s.norm.weight", None, max_positions=128)

    register_architecture("ToyStepForCausalLM", StepConfig, spec_of)
    cfg = StepConfig("ToyStepForCausalLM", 48, 90)
    folder = write_model_folder(str(tmp_path / "m"), cfg, seed=6, std=0.15,
                                dtype={"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype])
    model, _ = load_model(folder, dtype)
    assert model.blocks[0].mixer.after_projection is not None and model.blocks[0].mixer.second_half_rows == 0
    eng = Engine(model, num_pages=8, page_size=16, max_requests=2, max_batch_tokens=64)
    assert not eng.use_graphs, "a part inside a mixer that does not say it is graph-safe keeps the model eager"
    toks = tu.make_requests(90, [50], seed=4)["r0"]
    eng.admit("a")
    got, i = [], 0
    for n in [33, 1, 1, 9, 2, 1, 1, 1, 1]:
        got.append(eng.step([StepEntry("a", toks[i:i + n], list(range(n)))]).double().cpu())
        i += n
    got = torch.cat(got)

    ck = Checkpoint(folder)
    t = {n: ck.tensor(n).double() for n in ck.names()}
    x = t["s.embed.weight"][toks]
    T, pos, inv = len(toks), list(range(len(toks))), plain_rope_frequencies(HD, 10000.0)
    for l in range(2):
        p = f"s.{l}."
        h = plain_rmsnorm(x, t[p + "mixer_norm.weight"], EPS)
        q = (h @ t[p + "mixer.q_proj.weight"].t() + t[p + "mixer.q_proj.bias"]).view(T, H, HD)
        k = (h @ t[p + "mixer.k_proj.weight"].t() + t[p + "mixer.k_proj.bias"]).view(T, KV, HD)
        v = (h @ t[p + "mixer.v_proj.weight"].t() + t[p + "mixer.v_proj.bias"]).view(T, KV, HD)
        q = plain_rope(plain_rmsnorm(q, t[p + "mixer.q_norm.weight"], 1e-3), pos, inv)
        k = plain_rope(plain_rmsnorm(k, t[p + "mixer.k_norm.weight"], 1e-3), pos, inv)
        x = x + plain_attention(q, k, v).reshape(T, H * HD) @ t[p + "mixer.o_proj.weight"].t()
        h = plain_rmsnorm(x, t[p + "feed_forward_norm.weight"], EPS)
        x = x + plain_swiglu(h @ t[p + "feed_forward.gate_proj.weight"].t(), h @ t[p + "feed_forward.up_proj.weight"].t()) \
            @ t[p + "feed_forward.down_proj.weight"].t()
    want = plain_rmsnorm(x, t["s.norm.weight"], EPS) @ t["s.embed.weight"].t()
    assert rel(got, want) < (3e-5 if dtype == "float32" else 5e-2), rel(got, want)
    assert float(t["s.0.mixer.q_proj.bias"].abs().max()) > 0.1          # (the step has something to add)


# -------------------------------------------------------------- the sampler ---

@pytest.mark.parametrize("V", [1000, 1001, 8201])      # (from 8,192 ids on a row is cut into slices first)
def test_sampler_kernel_follows_the_plain_rules(V):
    from plain_llama import plain_repeat_penalty, plain_sampling_distribution
    from hfee_amd.sampling import SampleRow, Sampler, SamplingParams, uniform
    g = torch.Generator().manual_seed(0)
    base = torch.randn(V, generator=g) * 2
    base[17] = base[400] = base.max() + 0.5          # tied maxima
    sampler = Sampler(V, DEV, max_rows=64)
    cases = [SamplingParams(temperature=0.8, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.0),
             SamplingParams(temperature=1.3, top_k=40, top_p=1.0, min_p=0.0, repeat_penalty=1.0),
             SamplingParams(temperature=1.0, top_k=0, top_p=0.7, min_p=0.0, repeat_penalty=1.0),
             SamplingParams(temperature=1.0, top_k=0, top_p=1.0, min_p=0.2, repeat_penalty=1.0),
             SamplingParams(temperature=0.8, top_k=40, top_p=0.9, min_p=0.05, repeat_penalty=1.1, repeat_last_n=64),
             SamplingParams()]
    history = torch.randint(0, V, (100,), generator=g).tolist() + [17]
    for p in cases:
        pen = plain_repeat_penalty(base, history, p.repeat_penalty, p.repeat_last_n)
        dist = plain_sampling_distribution(pen, p.temperature, p.top_k, p.top_p, p.min_p)
        support = set(dist.nonzero().flatten().tolist())
        counts = torch.zeros(V)
        exact = 0
        draws = 64 * 30
        for c in range(30):
            logits = base.repeat(64, 1).to(DEV)
            rows = [SampleRow(p, seed=99, draw=c * 64 + r, history=history, logits_row=r) for r in range(64)]
            ids = sampler.sample(logits, rows)
            for r, i in enumerate(ids):
                counts[i] += 1
                # the kernel walks the kept set in ascending id with r = u * total
                cum = torch.cumsum(dist, 0)
                exact += int(i == int((cum >= uniform(99, c * 64 + r)).nonzero()[0]))
        assert set(counts.nonzero().flatten().tolist()) <= support, f"{p}: sampled outside the kept set"
        assert exact >= 0.99 * draws, f"{p}: only {exact} of {draws} draws match the inverse CDF"
        if V <= 1001:      # (over thousands of ids 1,920 draws say too little about the shape; the check above is the exact one)
            tv = 0.5 * float((counts / draws - dist.float()).abs().sum())
            assert tv < 0.12, f"{p}: total variation {tv}"
    # greedy with and without penalty; one stream per request, whatever shares the call
    greedy = SamplingParams(temperature=0.0, repeat_penalty=1.0)
    logits = base.repeat(3, 1).to(DEV)
    assert sampler.sample(logits, [SampleRow(greedy, 1, 0, [], r) for r in range(3)]) == [17, 17, 17]
    pen = SamplingParams(temperature=0.0, repeat_penalty=5.0, repeat_last_n=-1)
    assert sampler.sample(base.repeat(1, 1).to(DEV), [SampleRow(pen, 1, 0, [17], 0)]) == [400]
    p = SamplingParams(temperature=1.0, top_k=50, top_p=1.0, repeat_penalty=1.0)
    alone = sampler.sample(base.repeat(1, 1).to(DEV), [SampleRow(p, 7, 5, [], 0)])
    mixed = sampler.sample(base.repeat(4, 1).to(DEV), [SampleRow(p, 3, 1, [], 0), SampleRow(greedy, 0, 0, [], 1),
                                                       SampleRow(p, 7, 5, [], 2), SampleRow(p, 8, 5, [], 3)])
    assert mixed[2] == alone[0] and mixed[1] == 17


@pytest.mark.parametrize("top_k,V", [(40, 9001), (700, 9001), (1500, 9001), (40, 7001), (64, 9004), (65, 9004), (12, 200000)])
def test_sampler_takes_the_first_ties_at_the_top_k_threshold(top_k, V):
    """Thousands of equal logits at the top_k threshold, spread over the whole vocabulary (so
    over all the waves that gather the kept set, and over all the slices of a large
    vocabulary with a small top_k): the ones with the smallest ids belong, as
    many as top_k leaves room for after the larger logits (sampler.go:132-151)."""
    from plain_llama import plain_sampling_distribution
    from hfee_amd.sampling import SampleRow, Sampler, SamplingParams
    g = torch.Generator().manual_seed(top_k)
    base = torch.full((V,), -2.0)
    tied = torch.randperm(V, generator=g)[:4000]
    base[tied] = 1.0
    larger = torch.randperm(V, generator=g)[:10]
    base[larger] = 1.5
    p = SamplingParams(temperature=1.0, top_k=top_k, top_p=1.0, min_p=0.0, repeat_penalty=1.0)
    support = set(plain_sampling_distribution(base, p.temperature, p.top_k, p.top_p, p.min_p).nonzero().flatten().tolist())
    assert len(support) == top_k
    sampler = Sampler(V, DEV, max_rows=64)
    seen = set()
    for c in range(12):
        rows = [SampleRow(p, seed=3, draw=64 * c + r, history=[], logits_row=r) for r in range(64)]
        seen |= set(sampler.sample(base.repeat(64, 1).to(DEV), rows))
    assert seen <= support, sorted(seen - support)[:5]
    assert len(seen) >= min(top_k, 300) // 2            # and the draws do spread over it


def test_sampler_with_a_top_k_too_large_to_gather():
    """A top_k above 1,024 is not gathered into LDS: the radix select's threshold then
    serves the rules that run over the whole vocabulary.  Draws match the inverse CDF of
    the plain distribution."""
    from plain_llama import plain_sampling_distribution
    from hfee_amd.sampling import SampleRow, Sampler, SamplingParams, uniform
    V = 3001
    g = torch.Generator().manual_seed(9)
    base = torch.randn(V, generator=g) * 3
    p = SamplingParams(temperature=1.1, top_k=1500, top_p=0.95, min_p=0.0, repeat_penalty=1.0)
    dist = plain_sampling_distribution(base, p.temperature, p.top_k, p.top_p, p.min_p)
    cum = torch.cumsum(dist, 0)
    sampler = Sampler(V, DEV, max_rows=64)
    rows = [SampleRow(p, seed=5, draw=r, history=[], logits_row=r) for r in range(64)]
    ids = sampler.sample(base.repeat(64, 1).to(DEV), rows)
    exact = sum(int(i == int((cum >= uniform(5, r)).nonzero()[0])) for r, i in enumerate(ids))
    assert all(dist[i] > 0 for i in ids) and exact >= 62, exact


@pytest.mark.parametrize("top_k", [40, 0, 1024, 1025, 5000])
def test_sampler_at_the_vocabulary_of_the_real_models(top_k):
    """128,256 logits a row (32 sets of radix counters, the gather of up to 1,024 ids and the
    path beyond it, a penalty bit set of 16 KB), with the reference's default options
    (/root/reference/internal/llm/sampler.go:23-34: temperature 0.8, top_p 0.9, a penalty of 1.1
    on the last 64 ids) and top_k as given: at least 99 in 100 draws are exactly the inverse
    CDF of the plain distribution at the request's own random number, none is outside the kept set."""
    from plain_llama import plain_repeat_penalty, plain_sampling_distribution
    from hfee_amd.sampling import SampleRow, Sampler, SamplingParams, uniform
    V = 128256
    g = torch.Generator().manual_seed(top_k + 1)
    base = torch.randn(V, generator=g) * 2.5
    base[100000] = base[77] = base.max() + 0.25                  # tied maxima far apart
    p = SamplingParams(top_k=top_k)
    assert (p.temperature, p.top_p, p.repeat_penalty, p.repeat_last_n, p.min_p) == (0.8, 0.9, 1.1, 64, 0.0)
    history = torch.randint(0, V, (90,), generator=g).tolist() + [77]
    pen = plain_repeat_penalty(base, history, p.repeat_penalty, p.repeat_last_n)
    dist = plain_sampling_distribution(pen, p.temperature, p.top_k, p.top_p, p.min_p)
    cum = torch.cumsum(dist, 0)
    kept = int((dist > 0).sum())
    assert kept >= 2 and (top_k == 0 or kept <= top_k)
    sampler = Sampler(V, DEV, max_rows=64)
    exact = draws = 0
    for c in range(3):
        logits = base.repeat(64, 1).to(DEV)
        rows = [SampleRow(p, seed=1234, draw=c * 64 + r, history=history, logits_row=r) for r in range(64)]
        for r, i in enumerate(sampler.sample(logits, rows)):
            assert dist[i] > 0, f"id {i} is outside the kept set of {kept}"
            want = int(torch.searchsorted(cum, torch.tensor(uniform(1234, c * 64 + r), dtype=cum.dtype)))
            exact += int(i == want)
            draws += 1
    assert exact >= 0.99 * draws, f"top_k {top_k}: only {exact} of {draws} draws match the inverse CDF ({kept} ids kept)"


@pytest.mark.parametrize("V", [700, 1003, 4099, 8209, 8212])
def test_sampler_takes_the_newest_id_of_a_history_from_the_device(V):
    """The newest id of each row's history may lie on the device only (`latest`: the ids of
    the sampling before, not yet collected), even in the tensor that takes this sampling's
    ids: the repeat penalty then sees the same window of ids, and the same ids come out, as
    with the whole history on the host.  A window of one id is that id alone; a window
    switched off stays off."""
    from hfee_amd.sampling import SampleRow, Sampler, SamplingParams
    g = torch.Generator().manual_seed(5)             # (a vocabulary that is no multiple of 4: rows that are not 16-byte aligned)
    base = torch.randn(6, V, generator=g) * 2
    sampler = Sampler(V, DEV, max_rows=8)
    histories = [torch.randint(0, V, (n,), generator=g).tolist() for n in (90, 3, 64, 65, 10, 30)]
    for h, row in zip(histories, base):
        row[h[-1]] = row.max() + 1.0          # the newest id would win if it were not penalised
    cases = [SamplingParams(temperature=0.0, repeat_penalty=3.0, repeat_last_n=64),
             SamplingParams(temperature=0.9, top_k=30, top_p=0.9, repeat_penalty=1.5, repeat_last_n=-1),
             SamplingParams(temperature=0.0, repeat_penalty=4.0, repeat_last_n=1),
             SamplingParams(temperature=0.7, top_k=0, top_p=1.0, repeat_penalty=2.0, repeat_last_n=64),
             SamplingParams(temperature=0.0, repeat_penalty=9.0, repeat_last_n=0),
             SamplingParams(temperature=0.0, repeat_penalty=1.0)]
    whole = sampler.sample(base.clone().to(DEV), [SampleRow(p, 11 + i, 4, h, i) for i, (p, h) in enumerate(zip(cases, histories))])
    place = torch.tensor([h[-1] for h in histories] + [0, 0], dtype=torch.int32, device=DEV)
    rows = [SampleRow(p, 11 + i, 4, h[:-1], i) for i, (p, h) in enumerate(zip(cases, histories))]
    ahead = sampler.collect(sampler.launch(base.clone().to(DEV), rows, out=place, latest=place))
    assert ahead == whole
    assert place[:6].tolist() == whole
    assert whole[0] != histories[0][-1] and whole[2] != histories[2][-1]      # the penalty did bite
    assert whole[4] == histories[4][-1] and whole[5] == histories[5][-1]      # and where it is off, it did not


def test_kernels_refuse_what_they_cannot_do():
    from hfee_amd.kernels import KernelError, ops
    with pytest.raises(KernelError, match="GPU tensors"):
        ops.rmsnorm(torch.empty(1, 4), torch.empty(1, 4), torch.empty(4), 1e-5)
    with pytest.raises(KernelError, match="shapes"):
        ops.linear(torch.empty(2, 3, device=DEV), torch.empty(2, 4, device=DEV), torch.empty(3, 5, device=DEV))
    with pytest.raises(KernelError, match="head sizes"):
        from hfee_amd.kernels import lib
        lib.attention_bf16(40)
    with pytest.raises(ValueError, match="head sizes"):
        import hfee_amd  # noqa: F401
        from hfee_amd.config import config_from_dict
        from hfee_amd.engine import random_model
        random_model(config_from_dict(dict(TINY_A, head_dim=40)), dtype="bfloat16", device=DEV)


def test_attention_finds_a_far_key_among_hundreds():
    """One key far back is made to stand out (its query and key are scaled); the
    output must be that key's value, in both kernels of the bfloat16 path and in the
    32-bit path, also across a page's edge and for the first key of all."""
    from hfee_amd.kernels import ops
    H, K, hd, T, ps = 4, 2, 64, 600, 16
    for dtype in (torch.float32, torch.bfloat16):
        for far in (0, 15, 16, 333, 599):
            g = torch.Generator().manual_seed(far)
            q = torch.randn(T, H, hd, generator=g) * 0.1
            k = torch.randn(T, K, hd, generator=g) * 0.1
            v = torch.randn(T, K, hd, generator=g)
            direction = torch.randn(hd, generator=g)
            direction /= direction.norm()
            k[far] = 40 * direction
            q[T - 1] = 40 * direction
            nblocks = (T + ps - 1) // ps
            order = torch.randperm(nblocks + 3, generator=g)[:nblocks].tolist()
            layer = torch.zeros(nblocks + 3, 2, K, ps * hd)
            for t in range(T):
                p, s = order[t // ps], t % ps
                for kh in range(K):
                    kslot(layer[p, 0, kh], ps, hd, s)[:] = k[t].view(K, -1, 16 if hd % 16 == 0 else hd)[kh]
                layer[p, 1].view(K, hd, ps)[:, :, vslot(s)] = v[t]
            layer = layer.to(dtype).to(DEV)
            table = torch.tensor([order], dtype=torch.int32, device=DEV)
            qd = q.reshape(T, H * hd).to(dtype).to(DEV)
            positions = torch.arange(T, dtype=torch.int32, device=DEV)
            seg = torch.zeros(T, dtype=torch.int32, device=DEV)
            want = v[far].to(dtype).float().repeat_interleave(H // K, 0).reshape(-1)
            outs = {}
            out = torch.zeros(T, H * hd, dtype=dtype, device=DEV)
            ops.attention_plain(out, qd, layer, positions, seg, table, H, K, hd, ps, 1.0, 0)
            outs["plain"] = out[T - 1]
            if dtype == torch.bfloat16:
                tiles = torch.tensor([(o, min(32, T - o), o, 0) for o in range(0, T, 32)], dtype=torch.int32, device=DEV)
                out = torch.zeros(T, H * hd, dtype=dtype, device=DEV)
                ops.attention_bf16_prefill(out, qd, layer, tiles, table, H, K, hd, ps, 1.0, 0)
                outs["prefill"] = out[T - 1]
                rows = torch.tensor([T - 1], dtype=torch.int32, device=DEV)
                for splits in (1, 5):
                    out = torch.zeros(T, H * hd, dtype=dtype, device=DEV)
                    partial = torch.zeros(H * splits * (hd + 2), dtype=torch.float32, device=DEV)
                    ops.attention_bf16_decode(out, qd, layer, rows, rows.clone(), torch.zeros(1, dtype=torch.int32, device=DEV),
                                              table, H, K, hd, ps, 1.0, 0, partial, splits)
                    outs[f"decode{splits}"] = out[T - 1]
            for name, o in outs.items():
                assert torch.allclose(o.float().cpu(), want, atol=2e-2), (dtype, far, name)


def test_attention_window_edge():
    """A window of W keys: the key at distance W-1 is the last one seen, the key at
    distance W is not.  Both are made to stand out in turn; the result must be that
    key's value in the first case and must not feel it in the second (all kernels,
    window edges inside a page, on a page's edge and across a 32-key tile)."""
    from plain_llama import plain_attention
    from hfee_amd.kernels import ops
    H, K, hd, ps = 2, 1, 32, 16
    for dtype in (torch.float32, torch.bfloat16):
        for T, W in ((100, 20), (97, 33), (130, 64), (64, 16), (50, 49)):
            for inside in (True, False):
                g = torch.Generator().manual_seed(T + W)
                q = torch.randn(T, H, hd, generator=g) * 0.1
                k = torch.randn(T, K, hd, generator=g) * 0.1
                v = torch.randn(T, K, hd, generator=g)
                direction = torch.randn(hd, generator=g)
                direction /= direction.norm()
                edge = T - W if inside else T - W - 1
                k[edge] = 40 * direction
                q[T - 1] = 40 * direction
                want = plain_attention(q.to(dtype), k.to(dtype), v.to(dtype), 1.0, window=W)[T - 1].reshape(-1).float()
                if inside:
                    assert torch.allclose(want, v[edge].to(dtype).float().repeat(H, 1).reshape(-1), atol=2e-2)
                nblocks = (T + ps - 1) // ps
                order = torch.randperm(nblocks + 2, generator=g)[:nblocks].tolist()
                layer = torch.full((nblocks + 2, 2, K, ps * hd), 9.0)
                for t in range(T):
                    p, sl = order[t // ps], t % ps
                    for kh in range(K):
                        kslot(layer[p, 0, kh], ps, hd, sl)[:] = k[t].view(K, -1, 16 if hd % 16 == 0 else hd)[kh]
                    layer[p, 1].view(K, hd, ps)[:, :, vslot(sl)] = v[t]
                layer = layer.to(dtype).to(DEV)
                table = torch.tensor([order], dtype=torch.int32, device=DEV)
                qd = q.reshape(T, H * hd).to(dtype).to(DEV)
                positions = torch.arange(T, dtype=torch.int32, device=DEV)
                seg = torch.zeros(T, dtype=torch.int32, device=DEV)
                outs = {}
                out = torch.zeros(T, H * hd, dtype=dtype, device=DEV)
                ops.attention_plain(out, qd, layer, positions, seg, table, H, K, hd, ps, 1.0, W)
                outs["plain"] = out[T - 1]
                if dtype == torch.bfloat16:
                    tiles = torch.tensor([(o, min(32, T - o), o, 0) for o in range(0, T, 32)], dtype=torch.int32, device=DEV)
                    out = torch.zeros(T, H * hd, dtype=dtype, device=DEV)
                    ops.attention_bf16_prefill(out, qd, layer, tiles, table, H, K, hd, ps, 1.0, W)
                    outs["prefill"] = out[T - 1]
                    rows = torch.tensor([T - 1], dtype=torch.int32, device=DEV)
                    for splits in (1, 2):
                        out = torch.zeros(T, H * hd, dtype=dtype, device=DEV)
                        partial = torch.zeros(H * splits * (hd + 2), dtype=torch.float32, device=DEV)
                        ops.attention_bf16_decode(out, qd, layer, rows, rows.clone(), torch.zeros(1, dtype=torch.int32, device=DEV),
                                                  table, H, K, hd, ps, 1.0, W, partial, splits)
                        outs[f"decode{splits}"] = out[T - 1]
                for name, o in outs.items():
                    assert torch.allclose(o.float().cpu(), want, atol=3e-2), (dtype, T, W, inside, name)


def test_toy_parts_of_every_kind_without_a_change_to_the_framework(tmp_path):
    """A toy architecture in which nothing is the built-in kind: an embedding with a scale,
    a mixer whose growing memory is one latent vector a token (not keys and values), a
    feed-forward that keeps per-request state and plans per-step metadata, a block
    arrangement without a mixer, and a head that scales its logits.  All are defined and
    registered here; the engine collects their cache needs, state, preparation and step
    metadata like anybody's, runs them in portions beside another request, and the result is
    the plain computation's."""
    import numpy as np
    import hfee_amd  # noqa: F401
    from hfee_amd.config import (CacheNeed, EmbeddingSpec, FeedForwardSpec, HeadSpec, LayerSpec, MixerSpec, ModelSpec,
                                 NormSpec, ScheduleEntry, params, register_architecture)
    from hfee_amd.config.base import KeyReader
    from hfee_amd.engine import Engine, StepEntry, load_model
    from hfee_amd.parts import (FeedForward, Mixer, Part, lookup, register_block, register_embedding,
                                register_feed_forward, register_head, register_mixer)
    from hfee_amd.weights import Checkpoint, TensorSpec, write_model_folder
    from plain_llama import plain_rmsnorm

    @register_embedding("toy_scaled_lookup")
    class ScaledLookup(Part):
        def __init__(self, spec, name, vocab, hidden, dtype):
            self.name, self.vocab, self.hidden, self.scale = name, vocab, hidden, float(spec.get("scale"))

        def tensor_specs(self):
            return [TensorSpec(self.name, (self.vocab, self.hidden))]

        def bind(self, tensors):
            self.table = tensors[self.name]

        def forward(self, ctx, x):
            x.copy_(self.table[ctx.token_ids.long()].float() * self.scale)

    @register_mixer("toy_latent_mean")
    class LatentMean(Mixer):
        """x += W mean(h of the sequence so far); the h are kept in the paged cache, one vector a token."""

        def __init__(self, spec, prefix, dtype):
            self.width, self.prefix = spec.get("hidden"), prefix

        def tensor_specs(self):
            return [TensorSpec(self.prefix + "w.weight", (self.width, self.width))]

        def bind(self, tensors):
            self.w = tensors.pop(self.prefix + "w.weight")

        def cache_spec(self):
            return CacheNeed("full", (self.width,), layout="a latent vector a slot")

        def forward_add(self, ctx, x, h, cache_layer, writes_cache):
            ps = ctx.page_size
            pages = ctx.storage.layer(cache_layer, (ps, self.width))
            tables = ctx.block_tables[ctx.storage.group_of(cache_layer)].cpu()
            for i, seg in enumerate(ctx.segments):
                for j in range(seg.length):
                    p = seg.start + j
                    pages[int(tables[i, p // ps]), p % ps] = h[seg.row0 + j].to(pages.dtype)
                held = torch.stack([pages[int(tables[i, p // ps]), p % ps] for p in range(seg.start + seg.length)]).float()
                sums = held.cumsum(0)
                for j in range(seg.length):
                    p = seg.start + j
                    x[seg.row0 + j] += self.w.float() @ (sums[p] / (p + 1))

    @register_feed_forward("toy_counting")
    class Counting(FeedForward):
        """x[t] += (W h[t]) * (1 + t % 2) + t / 100: the parity comes with the step's metadata, the
        count of tokens that the request has run before lives in its state slot."""

        def __init__(self, spec, prefix, dtype):
            self.width, self.prefix = spec.get("hidden"), prefix

        def tensor_specs(self):
            return [TensorSpec(self.prefix + "w.weight", (self.width, self.width))]

        def bind(self, tensors):
            self.w = tensors.pop(self.prefix + "w.weight")

        def state_specs(self):
            return [(self.prefix + "seen", (1,), torch.float32)]

        def prepare(self, info):
            self.seen = info.storage.states[self.prefix + "seen"]

        def plan(self, plan):
            if "toy.parity" not in plan.arrays:          # (the layers' feed-forwards share it)
                plan.add("toy.parity", np.concatenate([np.arange(s.start, s.start + s.length) % 2 for s in plan.segments]))

        def forward_add(self, ctx, x, h):
            x += (h.float() @ self.w.float().t()) * (1 + ctx.extra["toy.parity"].float())[:, None]
            for seg in ctx.segments:
                rows = slice(seg.row0, seg.row0 + seg.length)
                x[rows] += 0.01 * (self.seen[seg.slot] + torch.arange(seg.length, device=x.device))[:, None]
                self.seen[seg.slot] += seg.length

    @register_block("toy_feed_forward_only")
    class FeedForwardOnly(Part):
        def __init__(self, spec, dtype):
            self.norm = lookup("norm", spec.feed_forward_norm.kind)(spec.feed_forward_norm, spec.prefix + "norm.weight")
            self.ffn = lookup("feed_forward", spec.feed_forward.kind)(spec.feed_forward, spec.prefix + "ffn.", dtype)
            self.hidden = spec.hidden

        def parts(self):
            return [self.norm, self.ffn]

        def tensor_specs(self):
            return self.norm.tensor_specs() + self.ffn.tensor_specs()

        def bind(self, tensors):
            self.norm.bind(tensors)
            self.ffn.bind(tensors)

        def forward(self, ctx, x, entry):
            h = ctx.rows("toy.normed", self.hidden)
            self.norm.forward(ctx, h, x)
            self.ffn.forward_add(ctx, x, h)

    @register_head("toy_scaled_head")
    class ScaledHead(Part):
        def __init__(self, spec, norm, name, vocab, hidden, embedding, dtype):
            self.norm, self.embedding, self.hidden, self.scale = norm, embedding, hidden, float(spec.get("logit_scale"))

        def parts(self):
            return [self.norm, self]

        def tensor_specs(self):
            return self.norm.tensor_specs()

        def bind(self, tensors):
            self.norm.bind(tensors)

        def forward(self, ctx, logits, x, rows):
            h = ctx.rows("toy.head", self.hidden, n=logits.shape[0])
            self.norm.forward(ctx, h, x, rows)
            logits.copy_((h.float() @ self.embedding.table.float().t()) * self.scale)

    @dataclass(frozen=True)
    class EveryConfig:
        architecture: str
        hidden: int
        vocab: int

        @staticmethod
        def from_dict(d, where="config.json"):
            r = KeyReader(d, where)
            c = EveryConfig("ToyEveryKindForCausalLM", r.int("e_hidden"), r.int("e_vocab"))
            r.finish()
            return c

        def to_dict(self):
            return {"architectures": ["ToyEveryKindForCausalLM"], "e_hidden": self.hidden, "e_vocab": self.vocab}

    def every_spec(c):
        norm = NormSpec("rmsnorm", c.hidden, 1e-5)
        ffn = FeedForwardSpec("toy_counting", params(hidden=c.hidden))
        latent = MixerSpec("toy_latent_mean", params(hidden=c.hidden))
        layers = (LayerSpec("prenorm", c.hidden, latent, ffn, norm, norm, "e.0."),
                  LayerSpec("toy_feed_forward_only", c.hidden, MixerSpec("none"), ffn, norm, norm, "e.1."))
        return ModelSpec("ToyEveryKindForCausalLM", c.hidden, c.vocab, layers, (ScheduleEntry(0, 0), ScheduleEntry(1, 1)),
                         norm, "e.embed.weight", "e.norm.weight", None, max_positions=256,
                         embedding=EmbeddingSpec("toy_scaled_lookup", params(scale=3.0)),
                         head=HeadSpec("toy_scaled_head", params(logit_scale=0.5)))

    register_architecture("ToyEveryKindForCausalLM", EveryConfig, every_spec)
    cfg = EveryConfig("ToyEveryKindForCausalLM", 24, 60)
    folder = write_model_folder(str(tmp_path / "every"), cfg, seed=2, std=0.2)
    model, _ = load_model(folder, "float32")
    eng = Engine(model, num_pages=8, page_size=16, max_requests=2, max_batch_tokens=64)
    assert not eng.use_graphs
    assert [(g.kind, g.token_shape, g.cache_layers) for g in eng.groups] == [("full", (24,), (0,))]
    assert eng.storage.pages[0].shape == (1, 8, 16 * 24)
    assert set(eng.storage.states) == {"e.0.feed_forward.seen", "e.1.ffn.seen"}

    toks = tu.make_requests(60, [50, 30], seed=4)
    eng.admit("other")
    eng.admit("a")
    got, i, oi = [], 0, 0
    for n in [9, 1, 22, 2, 16]:
        entries = [StepEntry("a", toks["r0"][i:i + n], list(range(n)))]
        if oi < 30:
            entries.insert(0, StepEntry("other", toks["r1"][oi:oi + 7], []))
            oi += 7
        got.append(eng.step(entries).double().cpu())
        i += n
    got = torch.cat(got)
    assert float(eng.storage.states["e.1.ffn.seen"][eng.cache.get("a").slot]) == 50
    eng.cache.check()

    ck = Checkpoint(folder)
    t = {n: ck.tensor(n).double() for n in ck.names()}
    T = 50
    x = t["e.embed.weight"][toks["r0"]] * 3.0
    at = torch.arange(T, dtype=torch.float64)
    h = plain_rmsnorm(x, t["e.0.mixer_norm.weight"], 1e-5)
    x = x + (h.cumsum(0) / (at + 1)[:, None]) @ t["e.0.mixer.w.weight"].t()
    for norm_name, w_name in (("e.0.feed_forward_norm.weight", "e.0.feed_forward.w.weight"), ("e.1.norm.weight", "e.1.ffn.w.weight")):
        h = plain_rmsnorm(x, t[norm_name], 1e-5)
        x = x + (h @ t[w_name].t()) * (1 + at % 2)[:, None] + 0.01 * at[:, None]
    want = plain_rmsnorm(x, t["e.norm.weight"], 1e-5) @ t["e.embed.weight"].t() * 0.5
    assert torch.allclose(got, want, atol=2e-4, rtol=2e-4), float((got - want).abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_model_with_no_norm_at_two_places(tmp_path, dtype):
    """The norm kind "none" where an arrangement expects a norm: a toy architecture, registered
    here, that is the dense decoder without its final norm and without the norm in front of the
    second layer's feed-forward.  A prompt of 70 tokens in one step (the kernels for many rows),
    then tokens one by one (the streaming kernels, whose fused norms must stand back), against
    the plain model with the same two norms left out."""
    import hfee_amd  # noqa: F401
    from conftest import make_model_folder
    from hfee_amd.config import NormSpec, register_architecture
    from hfee_amd.config.llama import LlamaConfig
    from hfee_amd.engine import Engine, StepEntry, load_model
    from hfee_amd.models.llama import llama_model_spec
    from plain_llama import PlainLlama, plain_matmul, plain_swiglu

    def spec_without(cfg):
        spec = llama_model_spec(cfg)
        none = NormSpec("none", cfg.hidden_size, 0.0)
        layers = list(spec.layers)
        layers[1] = replace(layers[1], feed_forward_norm=none)
        return replace(spec, layers=tuple(layers), final_norm=none)

    register_architecture("ToyFewerNormsForCausalLM", LlamaConfig, spec_without)
    cj = dict(TINY_A, architectures=["ToyFewerNormsForCausalLM"], num_hidden_layers=2, hidden_size=72, intermediate_size=104,
              num_attention_heads=3, num_key_value_heads=1, head_dim=16, vocab_size=211, tie_word_embeddings=False)
    folder = make_model_folder(tmp_path / "m", cj, seed=8, dtype=dtype, std=0.1, norm_init="one_plus_normal")
    model, _ = load_model(folder, dtype)
    names = {s.name for s in model.tensor_specs()}
    assert "model.norm.weight" not in names and "model.layers.1.post_attention_layernorm.weight" not in names
    assert "model.layers.0.post_attention_layernorm.weight" in names

    class Plain(PlainLlama):
        def feed_forward_sublayer(self, x, l):
            if l != 1:
                return super().feed_forward_sublayer(x, l)
            w, p, xb = self.w, f"model.layers.{l}.", self.r(x)
            h = plain_swiglu(plain_matmul(xb, w[p + "mlp.gate_proj.weight"]), plain_matmul(xb, w[p + "mlp.up_proj.weight"]), self.act)
            return plain_matmul(self.r(h), w[p + "mlp.down_proj.weight"])

        def head(self, x):
            return plain_matmul(self.r(x), self.w["lm_head.weight"])

    toks = tu.make_requests(211, [76], seed=5)["r0"]
    eng = Engine(model, num_pages=8, page_size=16, max_requests=2, max_batch_tokens=128)
    eng.admit("a")
    got = [eng.step([StepEntry("a", toks[:70], list(range(70)))]).double().cpu()]
    for t in range(70, 76):
        got.append(eng.step([StepEntry("a", toks[t:t + 1], [0])]).double().cpu())
    got = torch.cat(got)
    eng.cache.check()
    want = Plain(folder).forward(toks).double().cpu()
    worst = float(((got - want).abs().amax(1) / want.abs().amax(1)).max())
    assert worst < (3e-5 if dtype == "float32" else 5e-2), worst
