"""What fixes the plain implementation beside the reference's text: special cases
that reduce to a library routine, invariants, and the vectors that the reference's
own tests hold.  Each is chosen so that a plausible mistake fails it."""
import math

import pytest

import torch
import torch.nn.functional as F

from plain_llama import (PlainLlama, plain_argmax, plain_attention, plain_matmul, plain_repeat_penalty,
                         plain_rmsnorm, plain_rope, plain_rope_frequencies, plain_sampling_distribution,
                         plain_softmax, plain_swiglu)

F64 = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


def test_rmsnorm():
    x, w = rnd(5, 33) * 3, rnd(33, seed=1)
    assert torch.allclose(plain_rmsnorm(x, w, 1e-5), F.rms_norm(x, (33,), w, 1e-5), atol=1e-12)
    y = plain_rmsnorm(x, torch.ones(33, dtype=F64), 0.0)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=F64), atol=1e-12)        # RMS exactly 1
    assert torch.allclose(plain_rmsnorm(7.5 * x, w, 0.0), plain_rmsnorm(x, w, 0.0), atol=1e-12)
    # eps sits inside the root, added to the mean: a tiny input shows where it is
    tiny = torch.full((1, 4), 1e-4, dtype=F64)
    want = 1e-4 / math.sqrt(1e-8 + 1e-2)
    assert torch.allclose(plain_rmsnorm(tiny, torch.ones(4, dtype=F64), 1e-2), torch.full((1, 4), want, dtype=F64), rtol=1e-12)


def test_matmul_and_head():
    x, w = rnd(4, 6), rnd(9, 6, seed=1)
    y = plain_matmul(x, w)
    assert y.shape == (4, 9) and torch.allclose(y[2, 5], (w[5] * x[2]).sum())
    assert torch.allclose(plain_matmul(x, torch.eye(6, dtype=F64)), x)


def test_rope_is_a_complex_rotation():
    T, H, hd = 6, 2, 8
    x = rnd(T, H, hd)
    inv = plain_rope_frequencies(hd, 10000.0)
    pos = [3, 0, 7, 100, 1, 2]
    y = plain_rope(x, pos, inv, "half")
    z = torch.complex(x[..., :hd // 2], x[..., hd // 2:])
    rot = torch.polar(torch.ones(T, hd // 2, dtype=F64), torch.tensor(pos, dtype=F64)[:, None] * inv[None, :])
    zz = z * rot[:, None, :]
    assert torch.allclose(y, torch.cat([zz.real, zz.imag], dim=-1), atol=1e-12)
    assert torch.equal(plain_rope(x, [0] * T, inv), x)                                     # position 0: identity
    assert torch.allclose((y[..., :4] ** 2 + y[..., 4:] ** 2), (x[..., :4] ** 2 + x[..., 4:] ** 2), atol=1e-12)
    # interleaved pairing is the same rotation under a permutation of each head's rows
    perm = torch.tensor([0, 4, 1, 5, 2, 6, 3, 7])        # new[2i] = old[i], new[2i+1] = old[i+half]
    yi = plain_rope(x[..., perm], pos, inv, "interleaved")
    assert torch.allclose(yi, y[..., perm], atol=1e-12)
    # a wrong sign would rotate backwards: check one angle by hand
    one = torch.zeros(1, 1, 2, dtype=F64)
    one[0, 0, 0] = 1.0
    r = plain_rope(one, [1], torch.tensor([math.pi / 2], dtype=F64))
    assert torch.allclose(r[0, 0], torch.tensor([0.0, 1.0], dtype=F64), atol=1e-12)      # (1,0) -> (cos, sin)


def test_rope_scores_depend_on_distance_only():
    hd = 16
    q, k = rnd(1, 1, hd), rnd(1, 1, hd, seed=1)
    inv = plain_rope_frequencies(hd, 500000.0)

    def score(m, n):
        return float((plain_rope(q, [m], inv) * plain_rope(k, [n], inv)).sum())
    assert abs(score(5, 2) - score(105, 102)) < 1e-9 and abs(score(9, 9) - score(0, 0)) < 1e-9
    assert abs(score(5, 2) - score(2, 5)) > 1e-6


def test_llama3_frequency_scaling():
    base = plain_rope_frequencies(32, 500000.0)
    same = plain_rope_frequencies(32, 500000.0, dict(factor=1.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                                     original_max_position_embeddings=64))
    assert torch.allclose(base, same, rtol=1e-12)
    sc = plain_rope_frequencies(32, 500000.0, dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                                   original_max_position_embeddings=64))
    ratio = (base / sc).tolist()
    # Tiny B: frequencies 0 and 1 are kept, 2 is blended, 3..15 are divided by exactly 8
    assert ratio[0] == 1.0 and ratio[1] == 1.0 and 1.0 < ratio[2] < 8.0
    assert all(abs(r - 8.0) < 1e-12 for r in ratio[3:])
    # The blended one, worked by hand: inv_freq[2] = 500000^(-4/32) = 0.193923, wavelength
    # 2 pi / 0.193923 = 32.4005; s = (64 / 32.4005 - 1) / (4 - 1) = 0.325094; the frequency becomes
    # (1 - s) f / 8 + s f = 0.409457 f, so base / scaled = 2.44226.  A blend that is linear in the
    # wavelength instead of in N0 / wavelength ((32.40 - 16) / (64 - 16) of the way to f / 8) would
    # give 1.4265, and s put on the divided frequency instead of the kept one 1.3975.
    assert abs(float(base[2]) - 0.193923) < 1e-6
    assert abs(ratio[2] - 2.44226) < 1e-4
    assert all(a >= b for a, b in zip(sc.tolist(), sc.tolist()[1:])), "monotone"
    # continuous at both edges of the band: a wavelength just inside matches just outside
    n0, lo, hi, f = 64.0, 1.0, 4.0, 8.0

    def scaled(freq):
        wl = 2 * math.pi / freq
        if wl < n0 / hi:
            return freq
        if wl > n0 / lo:
            return freq / f
        s = (n0 / wl - lo) / (hi - lo)
        return (1 - s) * freq / f + s * freq
    for edge in (n0 / hi, n0 / lo):
        a, b = 2 * math.pi / (edge * (1 - 1e-9)), 2 * math.pi / (edge * (1 + 1e-9))
        assert abs(scaled(a) / a - scaled(b) / b) < 1e-6
    # 8B shape: 29 kept, 6 blended, 29 divided of 64
    big = plain_rope_frequencies(128, 500000.0, dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                                     original_max_position_embeddings=8192))
    r = (plain_rope_frequencies(128, 500000.0) / big)
    assert int((r == 1).sum()) == 29 and int(((r - 8).abs() < 1e-9).sum()) == 29


def test_attention_reduces_to_the_library_routine():
    T, H, K, hd = 9, 6, 2, 8
    q, k, v = rnd(T, H, hd), rnd(T, K, hd, seed=1), rnd(T, K, hd, seed=2)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.repeat_interleave(H // K, 1).transpose(0, 1)[None],
                                         v.repeat_interleave(H // K, 1).transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    assert torch.allclose(plain_attention(q, k, v), ref, atol=1e-12)
    # grouping: head h reads kv head h // group (contiguous groups, not h % K)
    v2 = v.clone()
    v2[:, 1] += 100
    out = plain_attention(q, k, v2)
    assert torch.allclose(out[:, :3], plain_attention(q, k, v)[:, :3], atol=1e-12) and (out[:, 3:] > 50).all()
    # one key: the output is its value; equal keys: the mean of the values
    assert torch.allclose(plain_attention(q[:1], k[:1], v[:1])[0, 0], v[0, 0])
    keq = k[:1].expand(T, K, hd)
    assert torch.allclose(plain_attention(q, keq, v)[4, 0], v[:5, 0].mean(0), atol=1e-12)
    # causality: later tokens do not change earlier outputs
    k3, v3 = k.clone(), v.clone()
    k3[6:] = 5.0
    v3[6:] = -3.0
    assert torch.allclose(plain_attention(q, k3, v3)[:6], plain_attention(q, k, v)[:6], atol=1e-12)
    # no rotation, no mask, one head: plain softmax(q k^T / sqrt(d)) v for the last row
    p = torch.softmax((k[:, 0] @ q[-1, 0]) / math.sqrt(hd), 0)
    assert torch.allclose(plain_attention(q, k, v)[-1, 0], p @ v[:, 0], atol=1e-12)
    # a window of w keeps the last w keys
    w = plain_attention(q, k, v, window=3)
    p = torch.softmax((k[4:7, 1] @ q[6, 5]) / math.sqrt(hd), 0)
    assert torch.allclose(w[6, 5], p @ v[4:7, 1], atol=1e-12)
    assert torch.allclose(plain_attention(q, k, v, window=100), plain_attention(q, k, v), atol=1e-12)


def test_softmax_and_swiglu():
    s = rnd(11)
    assert torch.allclose(plain_softmax(s), torch.softmax(s, 0), atol=1e-14) and abs(float(plain_softmax(s).sum()) - 1) < 1e-12
    g, u = rnd(7, 5) * 4, rnd(7, 5, seed=1)
    assert torch.allclose(plain_swiglu(g, u), F.silu(g) * u, atol=1e-12)
    assert float(plain_swiglu(torch.zeros(1, dtype=F64), torch.ones(1, dtype=F64))) == 0
    assert abs(float(plain_swiglu(torch.tensor([40.0], dtype=F64), torch.tensor([2.0], dtype=F64))) - 80) < 1e-9
    assert abs(float(plain_swiglu(torch.tensor([-40.0], dtype=F64), torch.tensor([2.0], dtype=F64)))) < 1e-12
    # the other names of config.json's hidden_act, which the reference does not have: the library's functions
    assert torch.allclose(plain_swiglu(g, u, "gelu"), F.gelu(g) * u, atol=1e-12)
    assert torch.allclose(plain_swiglu(g, u, "gelu_pytorch_tanh"), F.gelu(g, approximate="tanh") * u, atol=1e-12)
    assert torch.allclose(plain_swiglu(g, u, "relu"), F.relu(g) * u, atol=0)
    assert not torch.allclose(plain_swiglu(g, u, "gelu"), plain_swiglu(g, u, "gelu_pytorch_tanh"), atol=1e-6)
    with pytest.raises(ValueError):
        plain_swiglu(g, u, "swoosh")


def test_sampler_rules():
    logits = torch.tensor([1.0, 3.0, 3.0, -2.0, 0.5, 2.5])
    assert plain_argmax(logits) == 1                                   # the first maximum
    d = plain_sampling_distribution(logits, 0.7)
    assert torch.allclose(d, torch.softmax(logits.double() / torch.tensor(0.7, dtype=torch.float32).double(), 0), atol=1e-9)
    d = plain_sampling_distribution(logits, 1.0, top_k=3)
    assert sorted(d.nonzero().flatten().tolist()) == [1, 2, 5] and abs(float(d.sum()) - 1) < 1e-12
    d = plain_sampling_distribution(logits, 1.0, top_p=0.5)            # 0.31 + 0.31 >= 0.5: two kept
    assert sorted(d.nonzero().flatten().tolist()) == [1, 2]
    # an exact hit: four equal logits are 0.25 each, the sum reaches 0.5 at the second, and ">=" stops there
    # (sampler.go:101-106; with ">" three would be kept); just above 0.5 it takes the third
    d = plain_sampling_distribution(torch.zeros(4), 1.0, top_p=0.5)
    assert d.tolist() == [0.5, 0.5, 0.0, 0.0]
    assert plain_sampling_distribution(torch.zeros(4), 1.0, top_p=0.5000001).tolist()[2] > 0
    # an exact hit of min_p: a candidate at exactly min_p x the best stays ("<" cuts, sampler.go:110-113)
    d = plain_sampling_distribution(torch.tensor([0.0, 0.0, -50.0]), 1.0, min_p=1.0)
    assert d.tolist() == [0.5, 0.5, 0.0]
    d = plain_sampling_distribution(logits, 1.0, min_p=0.5)            # exp(-0.5) = 0.61 stays, exp(-2) goes
    assert sorted(d.nonzero().flatten().tolist()) == [1, 2, 5]
    cold = plain_sampling_distribution(torch.tensor([1.0, 2.0, 1.5]), 1e-3)
    assert float(cold[1]) > 1 - 1e-9
    pen = plain_repeat_penalty(torch.tensor([2.0, -2.0, 1.0, 4.0]), [0, 1, 1, 9, 3, 2], 2.0, 4)
    assert pen.tolist() == [2.0, -4.0, 0.5, 2.0]                       # last 4 ids: 1, 9, 3, 2; id 1 once
    assert plain_repeat_penalty(torch.tensor([2.0]), [0], 2.0, 0).tolist() == [2.0]
    assert plain_repeat_penalty(torch.tensor([2.0, 2.0]), [0, 1, 1], 2.0, -1).tolist() == [1.0, 1.0]


def test_tied_and_untied_head_and_causality_of_the_model(tmp_path):
    import json, os
    from safetensors.torch import load_file, save_file
    from conftest import TINY_A, make_model_folder
    folder = make_model_folder(tmp_path / "a", TINY_A, seed=2, std=0.1)
    plain = PlainLlama(folder)
    toks = [5, 200, 17, 3, 99, 100, 42]
    lg = plain.forward(toks)
    # tied: logits are x . E^T; untying with lm_head = E gives the same numbers
    w = load_file(os.path.join(folder, "model.safetensors"))
    w["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    os.makedirs(tmp_path / "b")
    save_file(w, str(tmp_path / "b" / "model.safetensors"))
    json.dump(dict(TINY_A, tie_word_embeddings=False), open(tmp_path / "b" / "config.json", "w"))
    assert torch.equal(PlainLlama(str(tmp_path / "b")).forward(toks), lg)
    # logits at position i do not change when later tokens do
    other = toks[:4] + [1, 2, 3]
    assert torch.allclose(plain.forward(other)[:4], lg[:4], atol=1e-12)
    assert not torch.allclose(plain.forward(other)[4:], lg[4:], atol=1e-3)
    # (the order of the parts inside the model is pinned in test_composition.py)
    assert plain.greedy(toks, 3) == [plain_argmax(plain.forward(toks)[-1])] + plain.greedy(toks + plain.greedy(toks, 1), 2)


def test_reference_text_vectors():
    """/root/reference/internal/llm/text_test.go:5-40"""
    from hfee_amd.text import Stopper, Utf8Buffer
    s, out = Stopper(["</end>"]), ""
    for piece in ["Hello", " wor", "ld</", "en", "d> ignored"]:
        text, hit = s.push(piece)
        out += text
        if hit:
            break
    assert out == "Hello world" and hit
    s = Stopper(["STOP"])
    assert s.push("go ST") == ("go ", False) and s.flush() == "ST"
    u, euro = Utf8Buffer(), "€".encode()
    assert u.add(euro[:2]) == "" and u.add(euro[2:]) == "€"


def test_product_frequencies_and_random_stream_match_their_plain_twins():
    from hfee_amd.parts.rotary import rope_frequencies
    from hfee_amd.sampling import uniform
    sc = ("llama3", 8.0, 1.0, 4.0, 64)
    a = rope_frequencies(32, 500000.0, sc)
    b = plain_rope_frequencies(32, 500000.0, dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                                  original_max_position_embeddings=64))
    assert torch.allclose(torch.from_numpy(a), b, rtol=1e-15)
    us = [uniform(12345, i) for i in range(2000)]
    assert all(0 <= u < 1 for u in us) and abs(sum(us) / 2000 - 0.5) < 0.03 and len(set(us)) == 2000
    assert uniform(1, 0) != uniform(2, 0)
