"""The random-weights stream: the same bits from the numpy code, from the header that the
kernel is built from (compiled here for the host) and, on the GPU, from the kernel; the
numbers are standard normal; a model made on the device equals the folder written on the
CPU, and `trace_run --random-weights` gives the folder's logits."""
import ctypes
import json
import math
import os
import shutil
import subprocess
import sys

import numpy as np
import pytest
import torch

from conftest import ROOT, TINY_A, TINY_B, make_model_folder
from hfee_amd.weights import random_stream as rs

HARNESS = r"""
#include "random_stream.h"
extern "C" void fill_normal(float* out, long count, unsigned long long key, int plus_one, double std) {
  for (long j = 0; 2 * j < count; ++j) {
    float a, b;
    hfee_random::normal_pair(key, (unsigned long long)j, plus_one != 0, std, a, b);
    out[2 * j] = a;
    if (2 * j + 1 < count) out[2 * j + 1] = b;
  }
}
extern "C" void fill_integers(int* out, long count, unsigned long long key, unsigned bound) {
  for (long i = 0; i < count; ++i) out[i] = hfee_random::integer(key, (unsigned long long)i, bound);
}
"""


def test_the_stream_is_standard_normal_and_its_functions_are_accurate():
    key = rs.tensor_key(5, "model.embed_tokens.weight")
    z = rs.normal(key, 1_000_001, 1.0).astype(np.float64)
    assert abs(z.mean()) < 4e-3 and abs(z.std() - 1) < 3e-3
    assert abs((z ** 3).mean()) < 2e-2 and abs((z ** 4).mean() - 3) < 5e-2
    assert abs(np.mean(np.abs(z) < 1) - math.erf(1 / math.sqrt(2))) < 2e-3      # 68.27 % within one sigma
    assert 4.5 < np.abs(z).max() < 6.7                                          # tails are there, bounded by 32 bits
    assert abs(np.corrcoef(z[0:-1:2], z[1::2])[0, 1]) < 4e-3 and abs(np.corrcoef(z[:-2], z[2:])[0, 1]) < 4e-3
    # any stretch of the stream is the stream: element i does not depend on the count or the chunking
    assert np.array_equal(rs.normal(key, 40_001, 1.0), rs.normal(key, 1_000_001, 1.0)[:40_001])
    assert np.allclose(rs.normal(key, 7, 0.5, plus_one=True), 1.0 + 0.5 * rs.normal(key, 7, 1.0), rtol=0, atol=2e-7)
    assert not np.array_equal(rs.normal(key, 8, 1.0), rs.normal(rs.tensor_key(6, "model.embed_tokens.weight"), 8, 1.0))
    assert not np.array_equal(rs.normal(key, 8, 1.0), rs.normal(rs.tensor_key(5, "model.norm.weight"), 8, 1.0))
    # the home-made logarithm, cosine and sine against the library's
    k = np.random.default_rng(0).integers(0, 2 ** 32, size=100_000, dtype=np.uint64)
    k[:6] = [0, 1, 2 ** 29, 2 ** 29 - 1, 2 ** 32 - 1, 2 ** 31]
    c, s = rs._cos_sin_turn(k)
    angle = 2 * np.pi * k.astype(np.float64) / 2 ** 32
    assert np.abs(c - np.cos(angle)).max() < 2e-15 and np.abs(s - np.sin(angle)).max() < 2e-15
    n = np.uint64(2) * k + np.uint64(1)
    want = -2 * np.log(n.astype(np.float64) / 2 ** 33)
    assert (np.abs(rs._minus_two_log(n) - want) < 1e-14 * np.maximum(want, 1)).all() and (rs._minus_two_log(n) > 0).all()
    i = rs.integers(key, 100_000, 777)
    assert i.dtype == np.int32 and i.min() == 0 and i.max() == 776 and abs(i.mean() - 388) < 3


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs a host compiler")
def test_the_kernels_arithmetic_built_for_the_host_gives_the_numpy_bits(tmp_path):
    """csrc/random_stream.h is what the kernel computes with; compiled by the host compiler
    (no contraction of products and sums, as in the kernel) it must give the numpy twin's bits."""
    src = tmp_path / "harness.cpp"
    src.write_text(HARNESS)
    lib_path = tmp_path / "harness.so"
    subprocess.run(["g++", "-O2", "-ffp-contract=off", "-shared", "-fPIC", "-D__host__=", "-D__device__=",
                    "-Wno-unknown-pragmas", "-I", os.path.join(ROOT, "hfee_amd", "csrc"), str(src), "-o", str(lib_path)],
                   check=True, capture_output=True, timeout=120)
    lib = ctypes.CDLL(str(lib_path))
    for seed, name, count, std, plus_one in ((5, "a", 300_001, 0.02, False), (0, "b", 1000, 0.1, True), (9, "c", 1, 1.0, False)):
        key = rs.tensor_key(seed, name)
        out = np.empty(count, dtype=np.float32)
        lib.fill_normal(out.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(count), ctypes.c_ulonglong(key),
                        int(plus_one), ctypes.c_double(std))
        assert np.array_equal(out.view(np.uint32), rs.normal(key, count, std, plus_one).view(np.uint32))
    ints = np.empty(50_000, dtype=np.int32)
    lib.fill_integers(ints.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(50_000), ctypes.c_ulonglong(key), 31)
    assert np.array_equal(ints, rs.integers(key, 50_000, 31))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_model_made_on_the_device_equals_the_folder_written_on_the_cpu(tmp_path, dtype):
    """Bit for bit: every tensor of `random_model` against the tensor of the same name that
    `write_model_folder` wrote with the same seed (through the library's reader), for both tiny
    configurations and a vocabulary matrix of three million numbers; and a folder written from
    the device equals the one written on the CPU byte for byte."""
    from safetensors import safe_open
    from hfee_amd.config import config_from_dict
    from hfee_amd.engine import declared_tensors
    from hfee_amd.weights import random_tensors, write_model_folder
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    big = dict(TINY_B, vocab_size=31_999, hidden_size=104, num_attention_heads=13, num_key_value_heads=13, head_dim=8)
    for i, (cj, seed, std, norm_init) in enumerate(((TINY_A, 3, 0.02, None), (TINY_B, 11, 0.1, "one_plus_normal"),
                                                     (big, 0, 0.02, "normal"))):
        cfg = config_from_dict(cj)
        folder = write_model_folder(str(tmp_path / f"cpu{i}"), cfg, seed=seed, std=std, dtype=dt, norm_init=norm_init)
        device = random_tensors(declared_tensors(cfg), seed, std, dt, "cuda:0", norm_init)
        with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
            assert set(f.keys()) == set(device)
            for name in f.keys():
                a, b = f.get_tensor(name), device[name].cpu()
                assert a.dtype == b.dtype and a.shape == b.shape
                assert torch.equal(a.view(torch.int16 if dt == torch.bfloat16 else torch.int32),
                                   b.view(torch.int16 if dt == torch.bfloat16 else torch.int32)), name
        other = write_model_folder(str(tmp_path / f"gpu{i}"), cfg, seed=seed, std=std, dtype=dt, norm_init=norm_init,
                                   device="cuda:0")
        with open(os.path.join(folder, "model.safetensors"), "rb") as fa, open(os.path.join(other, "model.safetensors"), "rb") as fb:
            assert fa.read() == fb.read()
    # integers
    from hfee_amd.kernels import ops
    out = torch.empty(70_001, dtype=torch.int32, device="cuda:0")
    ops.random_fill(out, rs.tensor_key(1, "table"), "integers", bound=12345)
    assert np.array_equal(out.cpu().numpy(), rs.integers(rs.tensor_key(1, "table"), 70_001, 12345))


@pytest.mark.gpu
def test_trace_run_with_random_weights_gives_the_folders_logits(tmp_path):
    """`trace_run --random-weights --seed S` reads config.json alone and makes the weights on the
    device; a folder written with the same seed holds the same model, so the 32-bit logits are the
    same bits, and the plain implementation, which reads the folder, is its reference too."""
    from plain_llama import PlainLlama
    folder = make_model_folder(tmp_path / "m", TINY_B, seed=4, dtype="float32", std=0.02)
    only_config = tmp_path / "c"
    only_config.mkdir()
    shutil.copy(os.path.join(folder, "config.json"), only_config / "config.json")
    toks = np.random.default_rng(2).integers(0, TINY_B["vocab_size"], size=37).tolist()
    lines = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:30], "want": "all"}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[30:], "want": "all"}], "end": ["a"]}]
    rows = {}
    for what, model, extra in (("folder", folder, []), ("seed", str(only_config), ["--random-weights", "--seed", "4"])):
        out = tmp_path / f"out_{what}"
        p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model, "--dtype", "float32",
                            "--out", str(out), "--max-tokens", "64"] + extra,
                           input="\n".join(json.dumps(l) for l in lines) + "\n", capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-2000:]
        rows[what] = np.concatenate([np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, TINY_B["vocab_size"]) for i in (0, 1)])
    assert np.array_equal(rows["folder"], rows["seed"])
    want = PlainLlama(folder).forward(toks).numpy()
    assert np.abs(rows["seed"] - want).max() / np.abs(want).max() < 3e-5


@pytest.mark.gpu
def test_a_whole_trace_that_names_its_model_by_configuration_and_seed(tmp_path):
    """`hfee_amd.replay(trace)` and `trace_run --trace FILE`: the trace carries config.json's keys and
    a seed instead of a folder; two cuts of the same requests agree bit for bit in 32-bit, key by
    key, on a pool so small that the second request gets the first one's pages, and agree with the
    plain model reading a folder of that seed."""
    import hfee_amd
    from plain_llama import PlainLlama
    rng = np.random.default_rng(3)
    a, b = (rng.integers(0, TINY_A["vocab_size"], size=n).tolist() for n in (45, 50))
    model = {"config": TINY_A, "random_weights": {"seed": 8, "std": 0.1}}
    whole = {"model": model, "dtype": "float32", "page_size": 16, "num_pages": 4,
             "steps": [{"segments": [{"req": "a", "tokens": a, "want": "all"}], "release": ["a"]},
                       {"segments": [{"req": "b", "tokens": b, "want": "all"}], "release": ["b"]}]}
    cut = dict(whole, steps=[{"segments": [{"req": "a", "tokens": a[:20], "want": "all"}]},
                             {"segments": [{"req": "a", "tokens": a[20:], "want": "all"}], "release": ["a"]},
                             {"segments": [{"req": "b", "tokens": b[:33], "want": [0, 32]}]},
                             {"segments": [{"req": "b", "tokens": b[33:], "want": "last"}], "release": ["b"]}])
    r_whole, r_cut = hfee_amd.replay(whole), hfee_amd.replay(cut)
    assert set(r_whole) == {("a", i) for i in range(45)} | {("b", i) for i in range(50)}
    assert set(r_cut) == {("a", i) for i in range(45)} | {("b", 0), ("b", 32), ("b", 49)}
    assert all(np.array_equal(r_cut[k], r_whole[k]) for k in r_cut)
    folder = make_model_folder(tmp_path / "m", TINY_A, seed=8, dtype="float32", std=0.1)
    want = PlainLlama(folder).forward(b).numpy()
    assert max(np.abs(r_whole[("b", i)] - want[i]).max() for i in range(50)) / np.abs(want).max() < 3e-5
    # the program, from a file
    (tmp_path / "trace.json").write_text(json.dumps(cut))
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--trace", str(tmp_path / "trace.json"),
                        "--out", str(tmp_path / "out")], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    last = np.fromfile(tmp_path / "out" / "3.f32", dtype="<f4")
    assert np.array_equal(last, r_whole[("b", 49)])
    with pytest.raises(Exception, match="pages"):          # the pool is what the trace says: five pages' worth is refused
        hfee_amd.replay(dict(whole, steps=[{"segments": [{"req": "a", "tokens": a, "want": "last"},
                                                         {"req": "b", "tokens": b[:30], "want": "last"}]}]))
