"""Replay: the same requests whole, with the last 32 tokens one by one, in portions
of changing size and mixed with other requests on a small page pool, in 32-bit and
in bfloat16, all compared with the plain implementation."""
import json
import os
import shutil
import subprocess
import sys

import numpy as np
import pytest
import torch

import trace_util as tu
from conftest import ROOT, TINY

pytestmark = pytest.mark.gpu

TOL = {"float32": 3e-5, "bfloat16": 5e-2}
LENGTHS = {"A": [5, 17, 64, 1, 100, 33, 128, 49], "B": [40, 3, 100, 130, 2, 77, 256], "C": [150, 70, 300, 41, 97]}


def rel(a, b):
    a = torch.as_tensor(np.asarray(a)).double()
    b = torch.as_tensor(np.asarray(b)).double()
    return float((a - b).abs().max() / b.abs().max())


@pytest.fixture(scope="module")
def plain_logits(model_folders):
    """(config, dtype) -> (requests, {(request, position): row} from the plain implementation,
    the same from its rounding twin in bfloat16)."""
    cache = {}

    def get(name, dtype):
        if (name, dtype) not in cache:
            reqs = tu.make_requests(TINY[name]["vocab_size"], LENGTHS[name], seed=ord(name))
            folder = model_folders[(name, dtype)]
            cache[(name, dtype)] = (reqs, plain_rows(folder, reqs),
                                    plain_rows(folder, reqs, rounded=True) if dtype == "bfloat16" else None)
        return cache[(name, dtype)]
    return get


def check(got, want, tol, what, twin=None):
    """Every row of `got` within tol of `want` (relative to the row's largest logit).  With the
    rounding twin's rows given (bfloat16 only) the bound follows the format's own noise as well:
    the twin rounds to bfloat16 where the engine does and sums in float64, so its distance to
    the plain model is what the format alone costs on these weights and tokens, and the
    engine may be at most FORMAT_FACTOR_WORST times as far in its worst row and
    FORMAT_FACTOR_MEDIAN times in the median row (a fault of a kernel that touches many
    rows moves the median, which is the steadier of the two).  On most models here these
    bounds are 2 to 10 times tighter than `tol`.  The twin's own rows are no closer to the
    engine's than the plain model's are: the roundings of the two fall differently, so the
    twin gives the size of the format's noise, not its sign."""
    assert set(got) == set(want), f"{what}: positions differ"
    worst, where = 0.0, None
    errors, noise = [], []
    for key in sorted(want, key=str):
        e = rel(got[key], want[key])
        errors.append(e)
        if twin is not None:
            noise.append(rel(twin[key], want[key]))
        if e > worst:
            worst, where = e, key
    if twin is not None:
        print(f"{what}: engine to plain worst {worst:.3e} median {np.median(errors):.3e}; "
              f"twin to plain worst {max(noise):.3e} median {np.median(noise):.3e}")
        assert worst < FORMAT_FACTOR_WORST * max(noise), \
            f"{what}: worst error {worst:.3e} at {where}, the format alone gives {max(noise):.3e}"
        assert np.median(errors) < FORMAT_FACTOR_MEDIAN * np.median(noise), \
            f"{what}: median error {np.median(errors):.3e}, the format alone gives {np.median(noise):.3e}"
    if tol is not None:
        assert worst < tol, f"{what}: worst relative error {worst:.3e} at {where}"


# Seen over all bfloat16 tests: the worst row up to 1.84 x the twin's worst row (two layers of
# the 8B sizes), the median up to 1.20 x the twin's median (width 296, head size 64).
FORMAT_FACTOR_WORST = 2.5
FORMAT_FACTOR_MEDIAN = 1.5


def plain_rows(folder, reqs, positions=None, rounded=False, device="cpu", both=False):
    """{(request, position): logits row} of the plain model (of its rounding twin), at all
    positions of every request or at the given {request: positions}.  both: the pair
    (plain model's rows, twin's rows), from one reading of the weights."""
    from plain_llama import PlainLlama
    plain = PlainLlama(folder, round_like_engine=rounded and not both, device=device)
    models = [plain] + ([PlainLlama(folder, round_like_engine=True, device=device, weights=plain.w)] if both else [])
    outs = []
    for model in models:
        out = {}
        for rid, toks in reqs.items():
            rows = sorted(range(len(toks)) if positions is None else positions.get(rid, []))
            if not rows:
                continue
            lg = model.forward(toks, rows=rows)
            for i, p in enumerate(rows):
                out[(rid, p)] = lg[i].numpy()
        outs.append(out)
    return tuple(outs) if both else outs[0]


def positions_of(got):
    out = {}
    for rid, p in got:
        out.setdefault(rid, []).append(p)
    return out


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cut_matches_the_plain_implementation(model_folders, plain_logits, name, dtype):
    from hfee_amd.trace_replay import Replayer
    reqs, want, twin = plain_logits(name, dtype)
    mixed_steps, peak = tu.mixed(reqs, seed=7)
    rep = Replayer(model_folders[(name, dtype)], dtype, max_tokens=max(peak, 512))
    results = {}
    for what, steps in (("whole", tu.whole(reqs)), ("bulk+tail", tu.bulk_then_tail(reqs)),
                        ("portions", tu.portions(reqs)), ("mixed", mixed_steps)):
        results[what] = tu.run(rep, steps)
        check(results[what], want, TOL[dtype], f"{name} {dtype} {what}", twin)
        rep.engine.cache.check()
        assert not rep.engine.cache.requests
    if dtype == "float32":
        # the 32-bit path gives the same bits however the work is cut
        for what in ("bulk+tail", "portions", "mixed"):
            for key, row in results["whole"].items():
                assert np.array_equal(row, results[what][key]), f"{name} {what}: bits differ at {key}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_trace_reuses_pages(model_folders, plain_logits, dtype):
    """The pool is just large enough for the live requests, so pages of finished
    requests are handed to later ones within the trace."""
    from hfee_amd.trace_replay import Replayer
    reqs, want, twin = plain_logits("B", dtype)
    steps, peak = tu.mixed(reqs, seed=3, live_max=3)
    rep = Replayer(model_folders[("B", dtype)], dtype, max_tokens=peak)
    total_pages = rep.engine.cache.pools[0].num_pages
    assert sum((len(t) + 15) // 16 for t in reqs.values()) > total_pages, "the trace must need page reuse"
    check(tu.run(rep, steps), want, TOL[dtype], f"B {dtype} mixed on {total_pages} pages", twin)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(model_folders, dtype):
    """One token per step for many hundreds of steps."""
    from plain_llama import PlainLlama
    from hfee_amd.trace_replay import Replayer
    toks = tu.make_requests(TINY["C"]["vocab_size"], [700], seed=5)["r0"]
    want = PlainLlama(model_folders[("C", dtype)]).forward(toks)
    rep = Replayer(model_folders[("C", dtype)], dtype, max_tokens=704)
    worst = 0.0
    for i, t in enumerate(toks):
        row = rep.step([("x", [t], [0])])
        worst = max(worst, rel(row[0], want[i]))
    assert worst < TOL[dtype], worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_folders, tmp_path, dtype):
    """bin/trace_run as a user calls it: JSON lines in, <step>.f32 files and `done` lines out."""
    from plain_llama import PlainLlama
    folder = model_folders[("A", dtype)]
    toks = tu.make_requests(256, [21, 9], seed=9)
    lines = [
        {"step": 0, "entries": [{"id": "a", "tokens": toks["r0"][:10], "want": [0, 9]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": toks["r0"][10:12], "want": []},
                                {"id": "b", "tokens": toks["r1"], "want": [8]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": toks["r0"][12:19], "want": []}], "end": []},
        {"step": 3, "entries": [{"id": "a", "tokens": toks["r0"][19:], "want": [1, 0]}], "end": ["a"]},
        {"step": 4, "entries": [{"id": "b", "tokens": toks["r1"][:4], "want": "last"}], "end": []},
        {"step": 5, "entries": [{"id": "b", "tokens": toks["r1"][4:], "want": "all"}], "end": ["b"]},
    ]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                        "--out", str(out), "--max-tokens", "128"],
                       input="\n".join(json.dumps(l) for l in lines) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(6)]
    assert not (out / "2.f32").exists(), "a step in which nothing is wanted writes no file"
    assert sorted(f.name for f in out.iterdir()) == ["0.f32", "1.f32", "3.f32", "4.f32", "5.f32"]
    plain = PlainLlama(folder)
    la, lb = plain.forward(toks["r0"]), plain.forward(toks["r1"])
    V = 256
    s0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V)
    s1 = np.fromfile(out / "1.f32", dtype="<f4").reshape(-1, V)
    s3 = np.fromfile(out / "3.f32", dtype="<f4").reshape(-1, V)
    s4 = np.fromfile(out / "4.f32", dtype="<f4").reshape(-1, V)
    s5 = np.fromfile(out / "5.f32", dtype="<f4").reshape(-1, V)
    assert s0.shape[0] == 2 and s1.shape[0] == 1 and s3.shape[0] == 2 and s4.shape[0] == 1 and s5.shape[0] == 5
    tol = TOL[dtype]
    assert rel(s0[0], la[0]) < tol and rel(s0[1], la[9]) < tol
    assert rel(s1[0], lb[8]) < tol
    assert rel(s3[0], la[20]) < tol and rel(s3[1], la[19]) < tol          # in the order of `want`
    assert rel(s4[0], lb[3]) < tol and all(rel(s5[i], lb[4 + i]) < tol for i in range(5))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_short_requests_just_fit_the_pool(model_folders, dtype):
    """Ten live requests of 3 to 64 tokens under max_tokens = 10 x 64: every page of the pool is
    taken at the end (a request's count rounds up to 64), more requests are live than the
    four of the other traces, and all of them decode in one step."""
    from plain_llama import PlainLlama
    from hfee_amd.trace_replay import Replayer
    folder = model_folders[("A", dtype)]
    lengths = [64, 3, 17, 64, 33, 50, 64, 16, 48, 61]
    reqs = tu.make_requests(256, lengths, seed=21)
    rep = Replayer(folder, dtype, max_tokens=64 * len(lengths))
    assert rep.engine.cache.pools[0].num_pages == 4 * len(lengths)
    steps = [{"entries": [(r, t[:-2], [len(t) - 3]) for r, t in reqs.items()], "end": []},
             {"entries": [(r, t[-2:-1], [0]) for r, t in reqs.items()], "end": []},
             {"entries": [(r, t[-1:], [0]) for r, t in reversed(list(reqs.items()))], "end": list(reqs)}]
    got = tu.run(rep, steps)
    plain = PlainLlama(folder)
    want = {}
    for rid, t in reqs.items():
        lg = plain.forward(t)
        for (r, p) in got:
            if r == rid:
                want[(r, p)] = lg[p].numpy()
    check(got, want, TOL[dtype], f"ten live requests, {dtype}")
    rep.engine.cache.check()
    assert not rep.engine.cache.requests
    with pytest.raises(Exception, match="pages"):        # one token more than the pool holds is refused, loudly
        rep.step([(f"x{i}", [1] * 64, []) for i in range(len(lengths))] + [("y", [1], [])])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_step_larger_than_the_engine_takes_is_cut(model_folders, plain_logits, dtype):
    """A replayer whose engine takes 40 tokens a step runs steps of up to 300: they are cut into
    consecutive engine steps (an entry may be cut in the middle), the wanted rows come back in
    the order of the entries and of `want`.  Same numbers as the uncut steps (in 32-bit the same bits)."""
    from hfee_amd.trace_replay import Replayer
    reqs, want, twin = plain_logits("C", dtype)
    folder = model_folders[("C", dtype)]
    ids = list(reqs)
    steps = [{"entries": [(ids[0], reqs[ids[0]][:100], [99, 0, 50]), (ids[1], reqs[ids[1]], [69, 3]),
                          (ids[3], reqs[ids[3]], list(range(41)))], "end": [ids[1], ids[3]]},
             {"entries": [(ids[0], reqs[ids[0]][100:], [49, 7]), (ids[2], reqs[ids[2]], [299, 39, 40, 0])],
              "end": [ids[0], ids[2]]}]
    results = {}
    for limit in (40, None):
        rep = Replayer(folder, dtype, max_tokens=1024, batch_limit=limit)
        results[limit] = tu.run(rep, steps)
        assert not rep.engine.cache.requests
        assert set(results[limit]) == {(ids[0], p) for p in (99, 0, 50, 149, 107)} | {(ids[1], 69), (ids[1], 3)} | \
            {(ids[3], p) for p in range(41)} | {(ids[2], p) for p in (299, 39, 40, 0)}
        check(results[limit], {k: want[k] for k in results[limit]}, TOL[dtype], f"C {dtype} steps cut at {limit}",
              twin and {k: twin[k] for k in results[limit]})
    if dtype == "float32":
        for k, row in results[None].items():
            assert np.array_equal(row, results[40][k]), f"bits differ at {k}"


def random_configuration(rng):
    """A small configuration of the architecture with every size drawn: head sizes in steps of
    16 up to 256, any number of heads and groups, widths that are multiples of 8, 4 or 2,
    any feed-forward width and vocabulary."""
    kv_heads = rng.randint(1, 4)
    scaling = None
    if rng.random() < 0.4:
        scaling = {"rope_type": "llama3", "factor": rng.choice([2.0, 8.0, 32.0]), "low_freq_factor": 1.0,
                   "high_freq_factor": rng.choice([2.0, 4.0]),
                   "original_max_position_embeddings": rng.choice([32, 64, 128])}
    return {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": rng.randint(1, 4),
            "hidden_size": rng.choice([8, 8, 8, 4, 2]) * rng.randint(5, 40),
            "num_attention_heads": kv_heads * rng.choice([1, 1, 2, 3, 4, 5, 7, 8]), "num_key_value_heads": kv_heads,
            "head_dim": 16 * rng.randint(1, 16), "intermediate_size": rng.choice([8, 8, 4, 2, 1]) * rng.randint(9, 70),
            "vocab_size": rng.randint(50, 3000), "max_position_embeddings": 512,
            "rope_theta": rng.choice([10000.0, 500000.0, 1e6]), "rope_scaling": scaling,
            "rms_norm_eps": rng.choice([1e-5, 1e-6, 3e-4]), "tie_word_embeddings": rng.random() < 0.5,
            "hidden_act": "silu"}


@pytest.mark.parametrize("seed", [7, 10, 18, 22, 30, 37])
def test_drawn_configurations_match_the_plain_implementation(tmp_path, seed):
    """Six configurations with sizes drawn at random, whole and mixed, in both types.  These seeds
    draw widths of 36, 58 and 68, head sizes from 80 to 224, 15 heads in 3 groups, 32 in 4,
    feed-forward widths of 9, 11 and 37, a vocabulary of 66, and the scaled rotation thrice.  The
    gate's activation goes round the four that config.json can name."""
    import random

    from conftest import make_model_folder
    from plain_llama import PlainLlama
    from hfee_amd.trace_replay import Replayer
    rng = random.Random(4000 + seed)
    cj = random_configuration(rng)
    cj["hidden_act"] = {7: "silu", 10: "gelu_pytorch_tanh", 18: "gelu", 22: "relu", 30: "silu", 37: "gelu_pytorch_tanh"}[seed]
    lengths = [rng.randint(1, 200) for _ in range(4)]
    reqs = tu.make_requests(cj["vocab_size"], lengths, seed=seed)
    mixed_steps, peak = tu.mixed(reqs, seed=seed)
    for dtype in ("float32", "bfloat16"):
        folder = make_model_folder(tmp_path / dtype, cj, seed=seed, dtype=dtype, std=0.05, norm_init="one_plus_normal")
        want = plain_rows(folder, reqs)
        twin = plain_rows(folder, reqs, rounded=True) if dtype == "bfloat16" else None
        rep = Replayer(folder, dtype, max_tokens=max(peak, 256))
        for what, steps in (("whole", tu.whole(reqs)), ("mixed", mixed_steps)):
            sizes = {k: cj[k] for k in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim",
                                        "intermediate_size", "vocab_size", "num_hidden_layers")}
            check(tu.run(rep, steps), want, TOL[dtype], f"{sizes} {dtype} {what}", twin)
            rep.engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_requests_decoding_together(tmp_path, dtype):
    """72, then 40, 20, 10 and 3 requests decode in one step each, in a changing order: products
    and decode attention of more than 64, of 17 to 64 and of fewer rows inside the whole model
    (the other replays hold four requests at most); the prompts come seven requests a step."""
    import random

    from conftest import make_model_folder
    from plain_llama import PlainLlama
    from hfee_amd.trace_replay import Replayer
    cj = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 2, "hidden_size": 512,
          "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 64, "intermediate_size": 1000,
          "vocab_size": 777, "max_position_embeddings": 256, "rope_theta": 10000.0, "rope_scaling": None,
          "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "hidden_act": "silu"}
    rng = random.Random(5)
    count, tail = 72, 12
    lengths = [rng.randint(tail + 2, 90) for _ in range(count)]
    folder = make_model_folder(tmp_path / "m", cj, seed=5, dtype=dtype, std=0.03, norm_init="one_plus_normal")
    reqs = tu.make_requests(cj["vocab_size"], lengths, seed=5)
    ids = list(reqs)
    rep = Replayer(folder, dtype, max_tokens=sum((n + 63) // 64 * 64 for n in lengths), max_requests=count)
    steps = []
    for i in range(0, count, 7):
        steps.append({"entries": [(r, reqs[r][:-tail], [len(reqs[r]) - tail - 1]) for r in ids[i:i + 7]], "end": []})
    live, fed = list(ids), {r: len(reqs[r]) - tail for r in ids}
    for t in range(tail):
        live = live[:{3: 40, 6: 20, 8: 10, 10: 3}.get(t, len(live))]
        order = list(live)
        rng.shuffle(order)
        steps.append({"entries": [(r, [reqs[r][fed[r]]], [0]) for r in order], "end": []})
        for r in order:
            fed[r] += 1
    steps[-1]["end"] = ids
    got = tu.run(rep, steps)
    want = plain_rows(folder, reqs, positions_of(got))
    twin = plain_rows(folder, reqs, positions_of(got), rounded=True) if dtype == "bfloat16" else None
    assert len(got) == count + 3 * 72 + 3 * 40 + 2 * 20 + 2 * 10 + 2 * 3
    check(got, want, TOL[dtype], f"many live requests, {dtype}", twin)
    rep.engine.cache.check()
    assert not rep.engine.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_context_of_thousands_of_tokens_inside_the_whole_model(tmp_path, dtype):
    """One request read in portions of 2,048 tokens up to position 4,600 and then decoded for
    eight steps, beside a short request that decodes in the same steps, with the head shape of
    the large models (heads of 128 in groups of four, scaled rotation): block tables of hundreds
    of pages (the attention kernels hold 64 entries at a time), portions that start deep in the
    context, decode steps that split thousands of keys.  The query and key projections are
    scaled up so that attention is sharp (a few far keys carry most of the weight): a page that
    is skipped, read twice or taken from the wrong request would show.  Logits at the edges of
    every portion, at the places where the kernels' window of the block table moves, and at
    every decoded token, against the plain implementation."""
    import safetensors.torch
    from conftest import make_model_folder
    from plain_llama import PlainLlama
    from hfee_amd.trace_replay import Replayer
    cj = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 2, "hidden_size": 1024,
          "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 128, "intermediate_size": 2048,
          "vocab_size": 3000, "max_position_embeddings": 8192, "rope_theta": 500000.0,
          "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                           "original_max_position_embeddings": 2048},
          "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "hidden_act": "silu"}
    folder = make_model_folder(tmp_path / "m", cj, seed=3, dtype=dtype, std=0.03, norm_init="one_plus_normal")
    path = os.path.join(folder, "model.safetensors")
    tensors = safetensors.torch.load_file(path)
    for name in tensors:
        if name.endswith("q_proj.weight") or name.endswith("k_proj.weight"):
            tensors[name] = (tensors[name].float() * 1.6).to(tensors[name].dtype)
    safetensors.torch.save_file(tensors, path)
    long_len, tail = 4600, 8
    reqs = tu.make_requests(cj["vocab_size"], [long_len + tail, 40 + 2 + tail], seed=17)
    big, small = reqs["r0"], reqs["r1"]
    rep = Replayer(folder, dtype, max_tokens=4672 + 64)
    edges = [0, 1, 1023, 1024, 2046, 2047]
    steps = [{"entries": [("big", big[:2048], edges), ("small", small[:40], [39])], "end": []},
             {"entries": [("small", small[40:41], [0]), ("big", big[2048:4096], [0, 1, 1023, 1024, 2047])], "end": []},
             {"entries": [("big", big[4096:long_len], [0, 1, 503]), ("small", small[41:42], [0])], "end": []}]
    for i in range(tail):
        steps.append({"entries": [("big", [big[long_len + i]], [0]), ("small", [small[42 + i]], [0])], "end": []})
    steps[-1]["end"] = ["big", "small"]
    got = tu.run(rep, steps)
    rep.engine.cache.check()
    assert not rep.engine.cache.requests
    del rep
    want = plain_rows(folder, {"big": big, "small": small}, positions_of(got))
    assert len(got) == 6 + 1 + 1 + 5 + 3 + 1 + 2 * tail
    check(got, want, TOL[dtype], f"a context of {long_len + tail} tokens, {dtype}")


PRODUCTION_SIZES = {
    # Llama-3.1-8B
    "8B": dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=14336,
               vocab_size=128256, max_position_embeddings=8192, rope_theta=500000.0, tie_word_embeddings=False,
               rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                             "original_max_position_embeddings": 8192}),
    # Llama-2-13B: as many KV heads as heads, widths of 5,120 and 13,824 (an odd multiple of 512), no scaling
    "13B": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=40, head_dim=128, intermediate_size=13824,
                vocab_size=32000, max_position_embeddings=4096, rope_theta=10000.0, tie_word_embeddings=False,
                rope_scaling=None),
    # Llama-3.2-1B: heads of 64, a tied head of 128,256 rows, factor 32
    "1B": dict(hidden_size=2048, num_attention_heads=32, num_key_value_heads=8, head_dim=64, intermediate_size=8192,
               vocab_size=128256, max_position_embeddings=8192, rope_theta=500000.0, tie_word_embeddings=True,
               rope_scaling={"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                             "original_max_position_embeddings": 8192}),
}


@pytest.mark.parametrize("size", ["8B", "13B", "1B"])
def test_layers_of_a_production_size_match_the_plain_implementation(tmp_path, size):
    """Two layers with the sizes of Llama-3.1-8B, Llama-2-13B and Llama-3.2-1B (vocabulary
    included) in bfloat16: the kernels and branches that only such sizes choose, inside the whole
    model.  Prompts of 2,048 (one step), 1,024, 300, 130 and 70 rows, 40 short ones eight a step,
    then 44, 30, 17, 8 and 2 requests decoding together.
    8B: tiles of 256 rows, K cut over workgroups, the pair of kernels for 17 to 64 rows, the
    streaming kernels with their fused norms, the prefill attention with four heads a KV head.
    13B (the only whole-model cover of these): the last half slice of the 17-to-64-row pair at
    K = 13,824, the streaming kernel with half blocks for 320 workgroups, the kernel for many weight
    rows at K = 5,120, the rotation whose 40 KV heads are dealt over several workgroups, the
    prefill attention by runs of row tiles (as many KV heads as heads) at head size 128.
    1B (likewise): head size 64 in both attention kernels, the tied head of 128,256 rows, the down
    product of 2,048 rows cut along K by the kernel of 256 x 128 tiles, K = 2,048 and 8,192 in the
    decode products, the rotation scaled by 32."""
    import random

    from conftest import make_model_folder
    from hfee_amd.trace_replay import Replayer
    cj = dict({"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 2,
               "rms_norm_eps": 1e-5, "hidden_act": "silu"}, **PRODUCTION_SIZES[size])
    if shutil.disk_usage(tmp_path).free < 8 << 30:
        pytest.skip("the model folder of this test takes up to 3 GB of the temporary folder")
    rng = random.Random(0)
    tail = 10
    lengths = [2048 + tail, 1024 + tail, 300 + tail, 130 + tail, 70 + tail] + [rng.randint(tail + 2, 40) for _ in range(39)]
    # (the weights are made on the device: the same numbers as on the CPU, in a fraction of the time)
    folder = make_model_folder(tmp_path / "m", cj, seed=1, dtype="bfloat16", std=0.02, norm_init="one_plus_normal",
                               device="cuda:0")
    reqs = tu.make_requests(cj["vocab_size"], lengths, seed=1)
    ids = list(reqs)
    rep = Replayer(folder, "bfloat16", max_tokens=sum((n + 63) // 64 * 64 for n in lengths), max_requests=64)
    steps = [{"entries": [(r, reqs[r][:-tail], [0, len(reqs[r]) - tail - 1])], "end": []} for r in ids[:5]]
    for i in range(5, len(ids), 8):
        steps.append({"entries": [(r, reqs[r][:-tail], [len(reqs[r]) - tail - 1]) for r in ids[i:i + 8]], "end": []})
    live, fed = list(ids), {r: len(reqs[r]) - tail for r in ids}
    for t in range(tail):
        live = live[:{3: 30, 5: 17, 7: 8, 9: 2}.get(t, len(live))]
        order = list(live)
        rng.shuffle(order)
        steps.append({"entries": [(r, [reqs[r][fed[r]]], [0]) for r in order], "end": []})
        for r in order:
            fed[r] += 1
    steps[-1]["end"] = ids
    got = {k: v.copy() for k, v in tu.run(rep, steps).items()}
    rep.engine.cache.check()
    del rep
    torch.cuda.empty_cache()
    # (the plain model's float64 products of this size run through the library on the GPU)
    want, twin = plain_rows(folder, reqs, positions_of(got), device="cuda:0", both=True)
    shutil.rmtree(folder, ignore_errors=True)          # (up to 3 GB of weights)
    check(got, want, TOL["bfloat16"], f"two layers of the {size} sizes", twin)


@pytest.mark.parametrize("head_dim", [64, 128, 224])
def test_weights_of_a_large_spread_stay_within_the_noise_of_the_format(tmp_path, head_dim):
    """Weights of standard deviation 0.1 at a width of 296 make attention scores sharp and logits
    large; in bfloat16 the engine then is 5 to 8 % of the largest logit away from the plain model,
    more than the bound of the other tests.  The rounding twin (bfloat16 between the parts, float64
    sums, no kernels) is 4.5 to 5.6 % away itself: what is left for the kernels is tested here as
    everywhere, engine to plain at most FORMAT_FACTOR_WORST x twin to plain (medians: FORMAT_FACTOR_MEDIAN); in 32-bit the same model is
    within 3e-5."""
    from conftest import make_model_folder
    from hfee_amd.trace_replay import Replayer
    cj = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 3,
          "hidden_size": 296, "num_attention_heads": 4, "num_key_value_heads": 4, "head_dim": head_dim,
          "intermediate_size": 68, "vocab_size": 1292, "max_position_embeddings": 512,
          "rope_theta": 10000.0, "rope_scaling": None, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
          "hidden_act": "silu"}
    reqs = tu.make_requests(1292, [145, 72], seed=0)
    mixed_steps, peak = tu.mixed(reqs, seed=0)
    for dtype in ("bfloat16", "float32"):
        folder = make_model_folder(tmp_path / dtype, cj, seed=0, dtype=dtype, std=0.1, norm_init="one_plus_normal")
        want = plain_rows(folder, reqs)
        rep = Replayer(folder, dtype, max_tokens=max(peak, 320))
        for what, steps in (("whole", tu.whole(reqs)), ("mixed", mixed_steps)):
            if dtype == "float32":
                check(tu.run(rep, steps), want, TOL[dtype], f"width 296, head size {head_dim}, 32-bit, {what}")
            else:
                check(tu.run(rep, steps), want, None, f"width 296, head size {head_dim}, bfloat16, {what}",
                      plain_rows(folder, reqs, rounded=True))
