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
    """{(config, dtype): {(request, position): row}} from the plain implementation."""
    from plain_llama import PlainLlama
    cache = {}

    def get(name, dtype):
        if (name, dtype) not in cache:
            plain = PlainLlama(model_folders[(name, dtype)])
            reqs = tu.make_requests(TINY[name]["vocab_size"], LENGTHS[name], seed=ord(name))
            out = {}
            for rid, toks in reqs.items():
                lg = plain.forward(toks)
                for p in range(len(toks)):
                    out[(rid, p)] = lg[p].numpy()
            cache[(name, dtype)] = (reqs, out)
        return cache[(name, dtype)]
    return get


def check(got, want, tol, what):
    assert set(got) == set(want), f"{what}: positions differ"
    worst, where = 0.0, None
    for key in sorted(want, key=str):
        e = rel(got[key], want[key])
        if e > worst:
            worst, where = e, key
    assert worst < tol, f"{what}: worst relative error {worst:.3e} at {where}"


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cut_matches_the_plain_implementation(model_folders, plain_logits, name, dtype):
    from hfee_amd.replay import Replayer
    reqs, want = plain_logits(name, dtype)
    mixed_steps, peak = tu.mixed(reqs, seed=7)
    rep = Replayer(model_folders[(name, dtype)], dtype, max_tokens=max(peak, 512))
    results = {}
    for what, steps in (("whole", tu.whole(reqs)), ("bulk+tail", tu.bulk_then_tail(reqs)),
                        ("portions", tu.portions(reqs)), ("mixed", mixed_steps)):
        results[what] = tu.run(rep, steps)
        check(results[what], want, TOL[dtype], f"{name} {dtype} {what}")
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
    from hfee_amd.replay import Replayer
    reqs, want = plain_logits("B", dtype)
    steps, peak = tu.mixed(reqs, seed=3, live_max=3)
    rep = Replayer(model_folders[("B", dtype)], dtype, max_tokens=peak)
    total_pages = rep.engine.cache.pools[0].num_pages
    assert sum((len(t) + 15) // 16 for t in reqs.values()) > total_pages, "the trace must need page reuse"
    check(tu.run(rep, steps), want, TOL[dtype], f"B {dtype} mixed on {total_pages} pages")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(model_folders, dtype):
    """One token per step for many hundreds of steps."""
    from plain_llama import PlainLlama
    from hfee_amd.replay import Replayer
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
        {"step": 2, "entries": [{"id": "a", "tokens": toks["r0"][12:], "want": [8, 0]}], "end": ["a"]},
    ]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                        "--out", str(out), "--max-tokens", "128"],
                       input="\n".join(json.dumps(l) for l in lines) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert not (out / "1.f32").exists() or True
    plain = PlainLlama(folder)
    la, lb = plain.forward(toks["r0"]), plain.forward(toks["r1"])
    V = 256
    s0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V)
    s1 = np.fromfile(out / "1.f32", dtype="<f4").reshape(-1, V)
    s2 = np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V)
    assert s0.shape[0] == 2 and s1.shape[0] == 1 and s2.shape[0] == 2
    tol = TOL[dtype]
    assert rel(s0[0], la[0]) < tol and rel(s0[1], la[9]) < tol
    assert rel(s1[0], lb[8]) < tol
    assert rel(s2[0], la[20]) < tol and rel(s2[1], la[12]) < tol


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
    feed-forward widths of 9, 11 and 37, a vocabulary of 66, and the scaled rotation thrice."""
    import random

    from conftest import make_model_folder
    from plain_llama import PlainLlama
    from hfee_amd.replay import Replayer
    rng = random.Random(4000 + seed)
    cj = random_configuration(rng)
    lengths = [rng.randint(1, 200) for _ in range(4)]
    reqs = tu.make_requests(cj["vocab_size"], lengths, seed=seed)
    mixed_steps, peak = tu.mixed(reqs, seed=seed)
    for dtype in ("float32", "bfloat16"):
        folder = make_model_folder(tmp_path / dtype, cj, seed=seed, dtype=dtype, std=0.05, norm_init="one_plus_normal")
        plain = PlainLlama(folder)
        want = {}
        for rid, toks in reqs.items():
            lg = plain.forward(toks)
            for p in range(len(toks)):
                want[(rid, p)] = lg[p].numpy()
        rep = Replayer(folder, dtype, max_tokens=max(peak, 256))
        for what, steps in (("whole", tu.whole(reqs)), ("mixed", mixed_steps)):
            sizes = {k: cj[k] for k in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim",
                                        "intermediate_size", "vocab_size", "num_hidden_layers")}
            check(tu.run(rep, steps), want, TOL[dtype], f"{sizes} {dtype} {what}")
            rep.engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_requests_decoding_together(tmp_path, dtype):
    """72, then 40, 20, 10 and 3 requests decode in one step each, in a changing order: products
    and decode attention of more than 64, of 17 to 64 and of fewer rows inside the whole model
    (the other replays hold four requests at most); the prompts come seven requests a step."""
    import random

    from conftest import make_model_folder
    from plain_llama import PlainLlama
    from hfee_amd.replay import Replayer
    cj = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 2, "hidden_size": 512,
          "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 64, "intermediate_size": 1000,
          "vocab_size": 777, "max_position_embeddings": 256, "rope_theta": 10000.0, "rope_scaling": None,
          "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "hidden_act": "silu"}
    rng = random.Random(5)
    count, tail = 72, 12
    lengths = [rng.randint(tail + 2, 90) for _ in range(count)]
    folder = make_model_folder(tmp_path / "m", cj, seed=5, dtype=dtype, std=0.03, norm_init="one_plus_normal")
    plain = PlainLlama(folder)
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
    want = {}
    for rid, toks in reqs.items():
        lg = plain.forward(toks)
        for (r, p) in got:
            if r == rid:
                want[(r, p)] = lg[p].numpy()
    assert len(got) == count + 3 * 72 + 3 * 40 + 2 * 20 + 2 * 10 + 2 * 3
    check(got, want, TOL[dtype], f"many live requests, {dtype}")
    rep.engine.cache.check()
    assert not rep.engine.cache.requests


def test_layers_of_a_production_size_match_the_plain_implementation(tmp_path):
    """Two layers with the sizes of Llama-3.1-8B (width 4,096, 32 heads in 8 groups, feed-forward
    14,336, vocabulary 128,256, scaled rotation) in bfloat16: the kernels that only such sizes
    choose (tiles of 256 rows, K cut over workgroups, the pair of kernels for 17 to 64 rows, the
    streaming kernels with their fused norms) inside the whole model.  Prompts of 1,024, 300, 130
    and 70 rows, 40 short ones eight a step, then 44, 30, 17, 8 and 2 requests decoding together."""
    import random

    from conftest import make_model_folder
    from plain_llama import PlainLlama
    from hfee_amd.replay import Replayer
    cj = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 2, "hidden_size": 4096,
          "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 14336,
          "vocab_size": 128256, "max_position_embeddings": 8192, "rope_theta": 500000.0,
          "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                           "original_max_position_embeddings": 8192},
          "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "hidden_act": "silu"}
    if shutil.disk_usage(tmp_path).free < 8 << 30:
        pytest.skip("the model folder of this test takes 3 GB of the temporary folder")
    rng = random.Random(0)
    tail = 10
    lengths = [1024 + tail, 300 + tail, 130 + tail, 70 + tail] + [rng.randint(tail + 2, 40) for _ in range(40)]
    folder = make_model_folder(tmp_path / "m", cj, seed=1, dtype="bfloat16", std=0.02, norm_init="one_plus_normal")
    reqs = tu.make_requests(cj["vocab_size"], lengths, seed=1)
    ids = list(reqs)
    rep = Replayer(folder, "bfloat16", max_tokens=sum((n + 63) // 64 * 64 for n in lengths), max_requests=64)
    steps = [{"entries": [(r, reqs[r][:-tail], [0, len(reqs[r]) - tail - 1])], "end": []} for r in ids[:4]]
    for i in range(4, len(ids), 8):
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
    got = tu.run(rep, steps)
    rep.engine.cache.check()
    del rep
    plain = PlainLlama(folder)
    want = {}
    for rid, toks in reqs.items():
        lg = plain.forward(toks)
        for (r, p) in got:
            if r == rid:
                want[(r, p)] = lg[p].numpy()
    del plain
    shutil.rmtree(folder, ignore_errors=True)          # (3 GB of weights)
    check(got, want, TOL["bfloat16"], "two layers of the 8B sizes")
