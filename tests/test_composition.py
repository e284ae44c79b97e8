"""What pins the order in which the parts are put together: the embedding as it is stored,
the norm before each half of a layer, the two additions to the stream, the final norm and
the head (/root/reference/internal/llm/forward.go:75-141).  Each vector is an identity
that the reference's composition satisfies and a plausible other one does not; the other
ones are written down below and every vector is shown to fail on at least one of them.
The same vectors run through the engine in 32-bit on the GPU (logits are all it shows, so
there the identities are stated on logits)."""
import json
import math
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from conftest import make_model_folder
from plain_llama import (PlainLlama, plain_attention, plain_matmul, plain_rmsnorm, plain_rope,
                         plain_rope_frequencies, plain_swiglu)

F64 = torch.float64

# eps is large beside the mean square of an embedding row (0.05^2), so that a scaled
# embedding shows through the final norm; sizes are no powers of two
CONFIG = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 1, "hidden_size": 40, "num_attention_heads": 6, "num_key_value_heads": 3,
    "head_dim": 16, "intermediate_size": 52, "vocab_size": 90, "max_position_embeddings": 64,
    "rope_theta": 10000.0, "rope_scaling": None, "rms_norm_eps": 1e-3, "tie_word_embeddings": False,
    "hidden_act": "silu",
}
TOKENS = [5, 80, 17, 3, 3, 61, 42, 0, 89]


def folder_with(path, config=None, seed=4, **edits):
    """A model folder with random weights (norm weights 1 + N(0, 0.1), so that no two norms
    are alike); edits: tensor-name suffix -> factor that the matching tensors are scaled by."""
    folder = make_model_folder(path, dict(CONFIG, **(config or {})), seed=seed, std=0.1, norm_init="one_plus_normal")
    if edits:
        file = os.path.join(folder, "model.safetensors")
        tensors = load_file(file)
        for suffix, factor in edits.items():
            hit = [n for n in tensors if n.endswith(suffix)]
            assert hit, suffix
            for n in hit:
                tensors[n] = tensors[n] * factor
        save_file(tensors, file)
    return folder


# ---- the identities, stated through the part functions alone -----------------------------

def parts_of(folder):
    with open(os.path.join(folder, "config.json")) as f:
        c = json.load(f)
    w = {k: v.to(F64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return c, w


def head_of(c, w, x):
    return plain_matmul(plain_rmsnorm(x, w["model.norm.weight"], c["rms_norm_eps"]), w["lm_head.weight"])


def attention_delta(c, w, x):
    """Wo . attention(rotated q, rotated k, v) of the normed stream, layer 0, positions 0.."""
    T, H, K, hd = x.shape[0], c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"]
    p = "model.layers.0."
    xb = plain_rmsnorm(x, w[p + "input_layernorm.weight"], c["rms_norm_eps"])
    inv = plain_rope_frequencies(hd, c["rope_theta"])
    pos = list(range(T))
    q = plain_rope(plain_matmul(xb, w[p + "self_attn.q_proj.weight"]).reshape(T, H, hd), pos, inv)
    k = plain_rope(plain_matmul(xb, w[p + "self_attn.k_proj.weight"]).reshape(T, K, hd), pos, inv)
    v = plain_matmul(xb, w[p + "self_attn.v_proj.weight"]).reshape(T, K, hd)
    return plain_matmul(plain_attention(q, k, v).reshape(T, H * hd), w[p + "self_attn.o_proj.weight"])


def feed_forward_delta(c, w, x):
    p = "model.layers.0."
    xb = plain_rmsnorm(x, w[p + "post_attention_layernorm.weight"], c["rms_norm_eps"])
    return plain_matmul(plain_swiglu(plain_matmul(xb, w[p + "mlp.gate_proj.weight"]),
                                     plain_matmul(xb, w[p + "mlp.up_proj.weight"])), w[p + "mlp.down_proj.weight"])


def expected_logits(folder, what):
    """The logits of TOKENS that the identity `what` says the folder must give."""
    c, w = parts_of(folder)
    x = w["model.embed_tokens.weight"][torch.tensor(TOKENS)]
    if what == "embedding, final norm and head alone":          # o_proj = down_proj = 0
        return head_of(c, w, x)
    if what == "the first addition alone":                      # down_proj = 0
        return head_of(c, w, x + attention_delta(c, w, x))
    if what == "the second addition alone":                     # o_proj = 0
        return head_of(c, w, x + feed_forward_delta(c, w, x))
    if what == "both":
        x = x + attention_delta(c, w, x)
        return head_of(c, w, x + feed_forward_delta(c, w, x))
    raise ValueError(what)


VECTORS = [("embedding, final norm and head alone", {"o_proj.weight": 0.0, "down_proj.weight": 0.0}),
           ("the first addition alone", {"down_proj.weight": 0.0}),
           ("the second addition alone", {"o_proj.weight": 0.0}),
           ("both", {})]


def rel(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max())


# ---- other compositions, each a plausible mistake ---------------------------------------

class ScaledEmbedding(PlainLlama):
    def embed(self, tokens):
        return super().embed(tokens) * math.sqrt(self.d)


class NoFinalNorm(PlainLlama):
    def head(self, x):
        return plain_matmul(x, self.w["lm_head.weight"])


class PostNorm(PlainLlama):
    """x <- norm(x + f(x)): the norm behind each half instead of before it."""
    def block(self, x, l, pos, kv=None, window=0):
        w, p, T = self.w, f"model.layers.{l}.", x.shape[0]
        q = plain_rope(plain_matmul(x, w[p + "self_attn.q_proj.weight"]).reshape(T, self.H, self.hd), pos, self.inv_freq)
        k = plain_rope(plain_matmul(x, w[p + "self_attn.k_proj.weight"]).reshape(T, self.K, self.hd), pos, self.inv_freq)
        v = plain_matmul(x, w[p + "self_attn.v_proj.weight"]).reshape(T, self.K, self.hd)
        att = plain_matmul(plain_attention(q, k, v).reshape(T, -1), w[p + "self_attn.o_proj.weight"])
        x = plain_rmsnorm(x + att, w[p + "input_layernorm.weight"], self.eps)
        h = plain_swiglu(plain_matmul(x, w[p + "mlp.gate_proj.weight"]), plain_matmul(x, w[p + "mlp.up_proj.weight"]))
        x = plain_rmsnorm(x + plain_matmul(h, w[p + "mlp.down_proj.weight"]), w[p + "post_attention_layernorm.weight"], self.eps)
        return x, (k, v)


class NormedStream(PlainLlama):
    """x <- norm(x) + f(norm(x)): the addition goes to the normed stream."""
    def block(self, x, l, pos, kv=None, window=0):
        p = f"model.layers.{l}."
        delta, kv = self.attention_sublayer(x, l, pos, kv, window)
        x = plain_rmsnorm(x, self.w[p + "input_layernorm.weight"], self.eps) + delta
        x = plain_rmsnorm(x, self.w[p + "post_attention_layernorm.weight"], self.eps) + self.feed_forward_sublayer(x, l)
        return x, kv


class ParallelHalves(PlainLlama):
    """x <- x + attention(norm1(x)) + feed_forward(norm2(x)): both halves read the same stream."""
    def block(self, x, l, pos, kv=None, window=0):
        delta, kv = self.attention_sublayer(x, l, pos, kv, window)
        return x + delta + self.feed_forward_sublayer(x, l), kv


class NormsSwapped(PlainLlama):
    """The two norm weights of a layer exchanged."""
    def __init__(self, folder):
        super().__init__(folder)
        for l in range(self.L):
            a, b = f"model.layers.{l}.input_layernorm.weight", f"model.layers.{l}.post_attention_layernorm.weight"
            self.w[a], self.w[b] = self.w[b], self.w[a]


OTHERS = [ScaledEmbedding, NoFinalNorm, PostNorm, NormedStream, ParallelHalves, NormsSwapped]


def test_the_plain_model_satisfies_every_identity_and_the_other_compositions_do_not(tmp_path):
    caught = {cls.__name__: [] for cls in OTHERS}
    for i, (what, edits) in enumerate(VECTORS):
        folder = folder_with(tmp_path / str(i), **edits)
        want = expected_logits(folder, what)
        assert rel(PlainLlama(folder).forward(TOKENS), want) < 1e-12, what
        for cls in OTHERS:
            if rel(cls(folder).forward(TOKENS), want) > 1e-2:
                caught[cls.__name__].append(what)
    # which vector is there for which mistake
    assert "embedding, final norm and head alone" in caught["ScaledEmbedding"]
    assert "embedding, final norm and head alone" in caught["NoFinalNorm"]
    assert "the first addition alone" in caught["PostNorm"] and "the first addition alone" in caught["NormedStream"]
    assert "the second addition alone" in caught["PostNorm"] and "the second addition alone" in caught["NormedStream"]
    assert "the second addition alone" in caught["NormsSwapped"]
    assert caught["ParallelHalves"] == ["both"]          # only the whole layer tells the halves' order


def test_a_half_of_a_layer_sees_only_the_direction_of_the_stream(tmp_path):
    """With eps -> 0 a half reads norm(x), which a scaling of x does not change: what it adds
    is the same for x and 3x.  A half without its norm, or with the norm behind it, fails this."""
    folder = folder_with(tmp_path / "m", config={"rms_norm_eps": 1e-30})
    x = PlainLlama(folder).embed(TOKENS)
    pos = list(range(len(TOKENS)))
    for cls, holds in ((PlainLlama, True), (PostNorm, False)):
        m = cls(folder)
        d1 = m.block(x, 0, pos)[0] - x
        d3 = m.block(3 * x, 0, pos)[0] - 3 * x
        # (the feed-forward half of 3x reads norm(3x + a), not norm(x + a): take the halves one by one)
        if cls is PlainLlama:
            a1, a3 = m.attention_sublayer(x, 0, pos)[0], m.attention_sublayer(3 * x, 0, pos)[0]
            f1, f3 = m.feed_forward_sublayer(x, 0), m.feed_forward_sublayer(3 * x, 0)
            assert rel(a3, a1) < 1e-12 and rel(f3, f1) < 1e-12
            assert rel(m.block(x, 0, pos)[0], x + a1 + m.feed_forward_sublayer(x + a1, 0)) < 1e-12
        else:
            assert (rel(d3, d1) < 1e-6) == holds
    # and with the norm's eps at work the same scaling does show
    m = PlainLlama(folder_with(tmp_path / "e", config={"rms_norm_eps": 1e-1}))
    assert rel(m.feed_forward_sublayer(3 * x, 0), m.feed_forward_sublayer(x, 0)) > 1e-2


def test_the_final_norm_weight_scales_the_logits_and_the_embedding_is_taken_as_stored(tmp_path):
    a = PlainLlama(folder_with(tmp_path / "a")).forward(TOKENS)
    b = PlainLlama(folder_with(tmp_path / "b", **{"model.norm.weight": 2.0})).forward(TOKENS)
    assert rel(b, 2 * a) < 1e-12
    assert rel(NoFinalNorm(folder_with(tmp_path / "c", **{"model.norm.weight": 2.0})).forward(TOKENS), 2 * a) > 1e-2
    # row t of the stream is row tokens[t] of the table: equal tokens at 3 and 4, no others alike
    m = PlainLlama(folder_with(tmp_path / "d"))
    x = m.embed(TOKENS)
    assert torch.equal(x[3], x[4]) and torch.equal(x[1], m.w["model.embed_tokens.weight"][80])
    # tied: the head is the table itself
    t = PlainLlama(folder_with(tmp_path / "t", config={"tie_word_embeddings": True},
                               **{"o_proj.weight": 0.0, "down_proj.weight": 0.0}))
    E = t.w["model.embed_tokens.weight"]
    assert "lm_head.weight" not in t.w
    assert rel(t.forward(TOKENS), plain_matmul(plain_rmsnorm(E[torch.tensor(TOKENS)], t.w["model.norm.weight"], 1e-3), E)) < 1e-12


@pytest.mark.gpu
@pytest.mark.parametrize("cut", ["whole", "one by one"])
def test_the_engine_satisfies_every_identity(tmp_path, cut):
    """The same four vectors through the engine's own block, embedding and head, in 32-bit, whole
    and token by token; then the scaling of the stream (the embedding table times 3 with a
    negligible eps changes the logits exactly as the identity says: 3x + a, not 3(x + a))."""
    from hfee_amd.trace_replay import Replayer

    def engine_logits(folder):
        rep = Replayer(folder, "float32", max_tokens=64)
        if cut == "whole":
            return torch.from_numpy(rep.step([("r", TOKENS, list(range(len(TOKENS))))], ["r"]).copy())
        rows = [torch.from_numpy(rep.step([("r", [t], [0])]).copy()) for t in TOKENS]
        return torch.cat(rows)

    for i, (what, edits) in enumerate(VECTORS):
        folder = folder_with(tmp_path / str(i), **edits)
        want = expected_logits(folder, what)
        assert rel(engine_logits(folder), want) < 3e-5, what
    folder = folder_with(tmp_path / "s", config={"rms_norm_eps": 1e-12},
                         **{"model.embed_tokens.weight": 3.0, "down_proj.weight": 0.0})
    c, w = parts_of(folder)
    x3 = w["model.embed_tokens.weight"][torch.tensor(TOKENS)]
    want = head_of(c, w, x3 + attention_delta(c, w, x3 / 3))
    assert rel(want, head_of(c, w, x3 + attention_delta(c, w, x3))) < 1e-9      # (the identity itself)
    assert rel(engine_logits(folder), want) < 3e-5
    assert rel(head_of(c, w, x3 / 3 + attention_delta(c, w, x3)), want) > 1e-2     # what it is told from
    # doubling the final norm's weight doubles the logits
    a = engine_logits(folder_with(tmp_path / "a"))
    b = engine_logits(folder_with(tmp_path / "b", **{"model.norm.weight": 2.0}))
    assert rel(b, 2 * a) < 3e-5
