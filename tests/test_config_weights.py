"""Configuration, registry, safetensors and weight-binding errors (CPU)."""
import json
import os

import pytest
import torch

import hfee_amd  # noqa: F401
from conftest import TINY_A, TINY_B, make_model_folder
from hfee_amd.config import ConfigError, config_from_dict, config_from_folder, model_spec_of
from hfee_amd.engine.model import Model, declared_tensors
from hfee_amd.weights import (Checkpoint, SafetensorsError, WeightsError, convert_for_engine,
                              load_tensors, random_tensors, write_safetensors)


def test_llama_config_reads_every_key_and_defaults():
    c = config_from_dict(TINY_B)
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (3, 96, 3, 1, 32)
    assert (c.intermediate_size, c.vocab_size, c.max_position_embeddings) == (256, 320, 256)
    assert c.rope_theta == 500000.0 and c.rms_norm_eps == 1e-6 and not c.tie_word_embeddings
    s = c.rope_scaling
    assert (s.rope_type, s.factor, s.low_freq_factor, s.high_freq_factor, s.original_max_position_embeddings) == \
        ("llama3", 8.0, 1.0, 4.0, 64)
    # the reference's defaults (/root/reference/internal/llm/model.go:90-100)
    d = config_from_dict({"architectures": ["LlamaForCausalLM"], "hidden_size": 64, "intermediate_size": 100,
                          "num_hidden_layers": 1, "num_attention_heads": 4, "vocab_size": 10})
    assert d.num_key_value_heads == 4 and d.head_dim == 16 and d.max_position_embeddings == 2048
    assert d.rms_norm_eps == 1e-5 and d.rope_theta == 10000.0 and d.rope_scaling is None
    # round trip through config.json
    assert config_from_dict(c.to_dict()) == c


def test_config_errors_name_everything_that_is_wrong():
    with pytest.raises(ConfigError, match='unsupported model architecture "MambaForCausalLM"'):
        config_from_dict({"architectures": ["MambaForCausalLM"]})
    with pytest.raises(ConfigError) as e:
        config_from_dict({"architectures": ["LlamaForCausalLM"], "hidden_size": "x"})
    msg = str(e.value)
    for key in ("hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads", "vocab_size"):
        assert key in msg
    bad = dict(TINY_A, num_key_value_heads=3)
    with pytest.raises(ConfigError, match="multiple of num_key_value_heads"):
        config_from_dict(bad)
    with pytest.raises(ConfigError, match="rope_type 'yarn' is not supported"):
        config_from_dict(dict(TINY_A, rope_scaling={"rope_type": "yarn", "factor": 2.0}))
    with pytest.raises(ConfigError, match="high_freq_factor must be greater"):
        config_from_dict(dict(TINY_B, rope_scaling=dict(TINY_B["rope_scaling"], high_freq_factor=1.0)))
    with pytest.raises(ConfigError, match="metadata is incomplete"):
        config_from_dict(dict(TINY_A, num_hidden_layers=0))
    with pytest.raises(ConfigError, match="hidden_act.*'silu'.*got 'swoosh'"):
        config_from_dict(dict(TINY_A, hidden_act="swoosh"))


def test_model_spec_carries_no_constant_of_its_own():
    spec = model_spec_of(config_from_dict(TINY_B))
    assert len(spec.layers) == 3 and [e.layer for e in spec.schedule] == [0, 1, 2]
    m = spec.layers[1].mixer
    assert m.kind == "attention" and m.get("num_heads") == 3 and m.get("num_kv_heads") == 1 and m.get("head_dim") == 32
    assert abs(m.get("scale") - 32 ** -0.5) < 1e-12 and m.position.get("theta") == 500000.0
    assert spec.layers[0].mixer_norm.eps == 1e-6 and spec.head_name == "lm_head.weight"
    assert model_spec_of(config_from_dict(TINY_A)).head_name is None        # tied
    # the gate's activation is config.json's to say, under the part's own name for it
    assert spec.layers[0].feed_forward.get("activation") == "silu"
    other = config_from_dict(dict(TINY_B, hidden_act="gelu_pytorch_tanh"))
    assert model_spec_of(other).layers[2].feed_forward.get("activation") == "gelu_tanh"
    assert config_from_dict(other.to_dict()) == other


def test_random_weights_folder_round_trip(tmp_path):
    folder = make_model_folder(tmp_path / "m", TINY_A, seed=5, dtype="bfloat16")
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    cfg = config_from_folder(folder)
    assert cfg == config_from_dict(dict(TINY_A, torch_dtype="bfloat16"))
    ck = Checkpoint(folder)
    names = {s.name for s in declared_tensors(cfg)}
    assert set(ck.names()) == names and "lm_head.weight" not in names
    # same seed, same numbers, whatever the order of making; another seed differs
    a = random_tensors(declared_tensors(cfg), 5, dtype=torch.bfloat16)
    for n in names:
        assert torch.equal(ck.tensor(n), a[n])
    b = random_tensors(reversed(declared_tensors(cfg)), 5, dtype=torch.bfloat16)
    assert all(torch.equal(a[n], b[n]) for n in names)
    c = random_tensors(declared_tensors(cfg), 6, dtype=torch.bfloat16)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    # the safetensors library reads the same file
    from safetensors import safe_open
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        assert set(f.keys()) == names
        assert torch.equal(f.get_tensor("model.norm.weight"), a["model.norm.weight"])
    # norm weights are near one, matrices near zero
    assert abs(float(a["model.norm.weight"].float().mean()) - 1) < 0.05
    assert abs(float(a["model.layers.0.mlp.up_proj.weight"].float().mean())) < 0.01


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = config_from_dict(TINY_A)
    specs = declared_tensors(cfg)
    t = random_tensors(specs, 1)
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)      # known non-weight: ignored
    t["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(64)
    t["model.layers.0.mlp.down_proj.weight"] = torch.zeros(172, 64)
    os.makedirs(tmp_path / "bad")
    json.dump(cfg.to_dict(), open(tmp_path / "bad" / "config.json", "w"))
    write_safetensors(str(tmp_path / "bad" / "model.safetensors"), t)
    spec = model_spec_of(cfg)
    with pytest.raises(WeightsError) as e:
        load_tensors(str(tmp_path / "bad"), specs, torch.float32, "cpu", spec.ignored_tensor_suffixes)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.q_proj.bias"]
    assert err.wrong_shapes == [("model.layers.0.mlp.down_proj.weight", (64, 172), (172, 64))]
    text = str(err)
    assert "missing tensors (2)" in text and "unexpected tensors (1)" in text and "expected [64, 172], got [172, 64]" in text


def test_storage_rule():
    bf, f32 = torch.bfloat16, torch.float32
    m = torch.randn(4, 4)
    assert convert_for_engine(m, "matrix", bf).dtype == bf
    assert convert_for_engine(m.to(bf), "matrix", f32).dtype == f32
    assert convert_for_engine(torch.ones(4), "vector", bf).dtype == f32          # stored in 32-bit: stays
    assert convert_for_engine(torch.ones(4, dtype=bf), "vector", bf).dtype == bf
    assert convert_for_engine(torch.ones(4, dtype=torch.float16), "vector", bf).dtype == bf
    assert convert_for_engine(torch.arange(4), "table", bf).dtype == torch.int32
    with pytest.raises(ValueError):
        convert_for_engine(torch.arange(4), "matrix", bf)


def test_safetensors_reader_refuses_broken_files(tmp_path):
    good = tmp_path / "g.safetensors"
    write_safetensors(str(good), {"a": torch.arange(6, dtype=torch.float32).reshape(2, 3), "b": torch.ones(2, dtype=torch.bfloat16)})
    raw = good.read_bytes()
    (tmp_path / "model.safetensors").write_bytes(raw[:-4])
    with pytest.raises(SafetensorsError, match="out of range"):
        Checkpoint(str(tmp_path))
    (tmp_path / "model.safetensors").write_bytes(b"\x05\x00")
    with pytest.raises(SafetensorsError, match="not a safetensors file"):
        Checkpoint(str(tmp_path))
    (tmp_path / "model.safetensors").write_bytes((10 ** 12).to_bytes(8, "little") + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        Checkpoint(str(tmp_path))
    os.remove(tmp_path / "model.safetensors")
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        Checkpoint(str(tmp_path))
    # shards through the index
    write_safetensors(str(tmp_path / "s1.safetensors"), {"a": torch.zeros(2)})
    json.dump({"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}, open(tmp_path / "model.safetensors.index.json", "w"))
    with pytest.raises(SafetensorsError, match="s2.safetensors is listed but absent"):
        Checkpoint(str(tmp_path))
    write_safetensors(str(tmp_path / "s2.safetensors"), {"b": torch.ones(3)})
    ck = Checkpoint(str(tmp_path))
    assert sorted(ck.names()) == ["a", "b"] and torch.equal(ck.tensor("b"), torch.ones(3))


def test_a_checkpoint_in_two_shards_loads_like_the_single_file(tmp_path):
    """A folder whose tensors lie in two safetensors files behind model.safetensors.index.json
    is read end to end: the same tensors, in both engine types, come out of `load_tensors` as
    from the single file."""
    from safetensors.torch import load_file
    folder = make_model_folder(tmp_path / "one", TINY_B, seed=3, dtype="bfloat16", std=0.1)
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    names = sorted(tensors)
    first = {n: tensors[n] for n in names[::2]}
    second = {n: tensors[n] for n in names[1::2]}
    two = tmp_path / "two"
    os.makedirs(two)
    write_safetensors(str(two / "model-00001-of-00002.safetensors"), first)
    write_safetensors(str(two / "model-00002-of-00002.safetensors"), second)
    weight_map = {n: "model-00001-of-00002.safetensors" for n in first}
    weight_map.update({n: "model-00002-of-00002.safetensors" for n in second})
    json.dump({"metadata": {"total_size": 0}, "weight_map": weight_map}, open(two / "model.safetensors.index.json", "w"))
    json.dump(json.load(open(os.path.join(folder, "config.json"))), open(two / "config.json", "w"))
    cfg = config_from_folder(str(two))
    specs = declared_tensors(cfg)
    for dtype in (torch.bfloat16, torch.float32):
        a = load_tensors(folder, specs, dtype, "cpu")
        b = load_tensors(str(two), specs, dtype, "cpu")
        assert set(a) == set(b) == set(names)
        assert all(torch.equal(a[n], b[n]) and a[n].dtype == b[n].dtype for n in names)
    # a tensor missing from one shard is reported by name, with everything else that is wrong
    write_safetensors(str(two / "model-00002-of-00002.safetensors"), {n: t for n, t in second.items() if n != "model.norm.weight"})
    with pytest.raises(Exception, match="model.norm.weight"):
        load_tensors(str(two), specs, torch.bfloat16, "cpu")


def test_schedule_and_cache_groups_are_data():
    """A layer may run twice, or read another layer's cache; layers with different
    needs land in different cache groups."""
    from dataclasses import replace
    from hfee_amd.config.specs import MixerSpec, ScheduleEntry
    spec = model_spec_of(config_from_dict(TINY_A))
    # layer 1 gets a window of 32: its own group
    m1 = spec.layers[1].mixer
    windowed = MixerSpec(m1.kind, tuple(sorted(dict(m1.params, window=32).items())), m1.position)
    spec2 = replace(spec, layers=(spec.layers[0], replace(spec.layers[1], mixer=windowed)),
                    schedule=(ScheduleEntry(0, 0), ScheduleEntry(1, 1), ScheduleEntry(0, 2), ScheduleEntry(1, 1, False)))
    groups = Model(spec2, torch.float32).cache_groups()
    kinds = {g.kind: g for g in groups}
    assert kinds["full"].cache_layers == (0, 2) and kinds["window"].cache_layers == (1,) and kinds["window"].window == 32
    with pytest.raises(ValueError, match="which no layer writes"):
        Model(replace(spec, schedule=(ScheduleEntry(0, 0), ScheduleEntry(1, 5, False))), torch.float32).cache_groups()


def test_the_benchmark_refuses_more_than_one_gpu():
    """`bench.py --gpus N` for N > 1 prints one line that says so and exits with 2, before
    anything touches a GPU."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    done = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "4", "--steps", "2", "--warmup", "1"],
                          capture_output=True, text=True, timeout=120)
    assert done.returncode == 2
    lines = [l for l in (done.stdout + done.stderr).splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_second_copies_of_the_weights_only_while_they_leave_room():
    """The weights' second copies in tiles are made while a fifth of the device's memory stays
    free; on tensors that are not on a GPU nothing is asked and the tiles are made (all of a
    part's weights or none), in the layout the kernels read: 16 rows x 32 columns a kilobyte."""
    import torch
    from hfee_amd.kernels import ops
    gib = 1 << 30
    assert ops.room_for_tiles(2 * gib, free=100 * gib, total=288 * gib)
    assert ops.room_for_tiles(42 * gib, free=100 * gib, total=288 * gib)
    assert not ops.room_for_tiles(43 * gib, free=100 * gib, total=288 * gib)
    assert not ops.room_for_tiles(1, free=57 * gib, total=288 * gib)
    w = torch.arange(40 * 72, dtype=torch.float32).reshape(40, 72).to(torch.bfloat16)
    tiles = ops.tile_weights_if_room(w, w[:16])
    assert len(tiles) == 2 and (tiles[0].n, tiles[0].k) == (40, 72)
    t = tiles[0].tiles
    assert t.shape == (3, 3, 512)                        # rows and columns padded to whole tiles
    # element (row r, column c) lies in tile (r // 16, c // 32) at ((c % 32) // 8) * 128 + (r % 16) * 8 + c % 8
    for r, c in ((0, 0), (5, 9), (17, 40), (39, 71)):
        assert t[r // 16, c // 32, ((c % 32) // 8) * 128 + (r % 16) * 8 + c % 8] == w[r, c]
    assert t[2, 2, 511] == 0                             # padding


def test_where_a_product_of_a_prompt_is_cut_along_k():
    """The host's rule for the products of 65 and more rows (asked of the library, which needs no
    GPU for it): with too few tiles of 128 x 128 for the chip K is cut over more workgroups and the
    caller brings scratch for the cuts; one round of such tiles runs whole where K is short and the
    tiles are many for it; nothing is cut up to 16 rows, up to 64 rows of a small weight (they go to the
    kernel that streams the weight's rows), nor once the tiles fill the chip."""
    from hfee_amd.kernels import ops

    def cuts(M, N, K):
        words = ops.linear_scratch(M, N, K)
        assert words % (M * N) == 0
        return words // (M * N)
    # the 8B shape's narrow products at a prompt of 128 tokens: 48 and 32 tiles
    assert cuts(128, 6144, 4096) == 5 and cuts(128, 4096, 4096) == 8 and cuts(128, 4096, 14336) == 8
    # two cuts by the tiles of 256 x 128 from K = 4,096 on
    assert cuts(512, 6144, 4096) == 2 and cuts(1024, 4096, 4096) == 2 and cuts(1024, 4096, 7680) == 2
    # one round of tiles, a short K: whole (the 1B shape's q/k/v and output products)
    assert cuts(512, 3072, 2048) == 0 and cuts(1024, 3072, 2048) == 0 and cuts(2048, 2048, 2048) == 0
    assert cuts(1024, 3072, 3072) == 0
    # ... but few tiles for the length of K are cut, and a long K always
    assert cuts(128, 3072, 2048) == 4 and cuts(256, 2048, 2048) == 4 and cuts(1024, 2048, 8192) >= 2
    # the rows of a decode step over a weight that lies as rows only: cut from 17 rows on where the weight is large
    assert cuts(16, 4096, 14336) == 0 and cuts(8, 4096, 14336) == 0 and cuts(64, 3072, 2048) == 0 and cuts(40, 768, 2048) == 0
    assert cuts(17, 4096, 14336) == 8 and cuts(64, 4096, 4096) == 8 and cuts(64, 6144, 4096) == 5
    # products that fill the chip
    assert cuts(2048, 4096, 4096) == 0 and cuts(2048, 28672, 4096) == 0 and cuts(512, 28672, 4096) == 0
