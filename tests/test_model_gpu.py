"""The engine against the plain implementation: whole prompts first."""
import pytest
import torch


pytestmark = pytest.mark.gpu

TOL = {"float32": 2e-5, "bfloat16": 4e-2}


def rel_err(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).abs().max() / b.abs().max())


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt(model_folders, name, dtype):
    from plain_llama import PlainLlama
    from hfee_amd.engine import Engine, StepEntry, load_model
    folder = model_folders[(name, dtype)]
    plain = PlainLlama(folder)
    model, cfg = load_model(folder, dtype)
    eng = Engine(model, num_pages=64, page_size=16, max_requests=4, max_batch_tokens=256)
    g = torch.Generator().manual_seed(1)
    for T in (1, 5, 17, 100):
        toks = torch.randint(0, cfg.vocab_size, (T,), generator=g).tolist()
        eng.admit("r")
        logits = eng.step([StepEntry("r", toks, list(range(T)))])
        ref = plain.forward(toks)
        eng.release("r")
        assert rel_err(logits, ref) < TOL[dtype], (T, rel_err(logits, ref))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_step_planned_ahead_is_the_same_step(model_folders, dtype):
    """prepare() plans a step before its tokens are known: the logits are those of the
    step planned at once, whether the announced shape comes true, comes true in part
    (another request, another count) or not at all; decoding across a page's edge."""
    from hfee_amd.engine import Engine, StepEntry, load_model
    folder = model_folders[("B", dtype)]
    model, cfg = load_model(folder, dtype)
    g = torch.Generator().manual_seed(5)
    prompts = {r: torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for r, n in (("x", 14), ("y", 30), ("z", 3))}
    follow = {r: torch.randint(0, cfg.vocab_size, (40,), generator=g).tolist() for r in prompts}

    def run(announce):
        eng = Engine(model, num_pages=24, page_size=16, max_requests=4, max_batch_tokens=64)
        for r, p in prompts.items():
            eng.admit(r)
        out = [eng.step([StepEntry(r, p, [len(p) - 1]) for r, p in prompts.items()]).clone()]
        live = list(prompts)
        for i in range(40):
            if i == 20:
                eng.release("y")
                live.remove("y")
            if announce == "right":
                assert eng.prepare([(r, 1, [0]) for r in live])
            elif announce == "wrong":       # another order, other counts, a request that will be gone
                eng.prepare([(r, 2 if i % 3 == 0 else 1, [0]) for r in reversed(list(prompts)) if eng.is_live(r)])
            out.append(eng.step([StepEntry(r, [follow[r][i]], [0]) for r in live]).clone())
        eng.cache.check()
        return out

    plain, right, wrong = run(None), run("right"), run("wrong")
    for a, b, c in zip(plain, right, wrong):
        assert torch.equal(a, b) and torch.equal(a, c)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prefix_kept_from_an_earlier_request(model_folders, dtype):
    """A request whose prompt begins with 50 tokens of an earlier one takes over the three full
    pages that hold 48 of them and runs the rest: the logits are those of the plain model over
    the whole prompt, in 32-bit bit for bit those of an engine that keeps nothing; the pages
    are the same ones; and when other requests have needed the memory in between, the prefix
    is gone and everything is run again, with the same result."""
    from plain_llama import PlainLlama
    from hfee_amd.engine import Engine, StepEntry, load_model
    folder = model_folders[("B", dtype)]
    plain = PlainLlama(folder)
    model, cfg = load_model(folder, dtype)
    g = torch.Generator().manual_seed(9)
    stem = torch.randint(0, cfg.vocab_size, (50,), generator=g).tolist()
    first = stem + torch.randint(0, cfg.vocab_size, (9,), generator=g).tolist()
    second = stem + torch.randint(0, cfg.vocab_size, (21,), generator=g).tolist()
    other = torch.randint(0, cfg.vocab_size, (100,), generator=g).tolist()

    def run(eng, rid, tokens):
        rc = eng.admit(rid, tokens)
        have, pages = rc.length, list(rc.tables[0])
        rest = tokens[have:]
        logits = eng.step([StepEntry(rid, rest, list(range(len(rest))))]).clone()
        return have, pages, logits

    keeping = Engine(model, num_pages=8, page_size=16, max_requests=2, max_batch_tokens=128, keep_prefixes=True)
    fresh = Engine(model, num_pages=8, page_size=16, max_requests=2, max_batch_tokens=128)
    have, pages_first, _ = run(keeping, "first", first)
    assert have == 0
    pages_first = list(keeping.cache.get("first").tables[0])
    keeping.release("first", first)
    have, pages, got = run(keeping, "second", second)
    assert have == 48 and pages == pages_first[:3]
    _, _, want = run(fresh, "second", second)
    ref = plain.forward(second)[48:]
    assert rel_err(got, ref) < TOL[dtype]
    if dtype == "float32":
        assert torch.equal(got, want[48:])
    else:
        assert rel_err(got, want[48:]) < 2e-2
    keeping.release("second", second)
    keeping.cache.check()
    # 100 tokens of something else take seven of the eight pages: what was kept has to go
    keeping.admit("other", other)
    keeping.step([StepEntry("other", other, [])])
    keeping.release("other")
    have, _, again = run(keeping, "third", second)
    assert have < 48
    assert rel_err(again[48 - have:], ref) < TOL[dtype]
    if dtype == "float32":
        assert torch.equal(again[48 - have:], got)
    keeping.release("third")
    keeping.cache.check()
    assert keeping.cache.free_pages() == [8]


@pytest.mark.parametrize("tiled_calls", [0, 2])
def test_a_model_too_large_for_second_copies_of_its_weights(model_folders, monkeypatch, tiled_calls):
    """Where the weights' second copies in tiles would not leave room, the parts bound last do
    without them (none of them, or all but the first layer's attention and feed-forward; the head, bound last, in neither case): steps
    of few rows then go through the kernels that read the weights' rows as they lie, beside
    layers that have their tiles, and give the plain model's logits, whole and decoding."""
    from plain_llama import PlainLlama
    from hfee_amd.engine import Engine, StepEntry, load_model
    from hfee_amd.kernels import ops
    made = ops.tile_weights_if_room
    calls = {"n": 0}

    def no_room(*weights):
        calls["n"] += 1
        return made(*weights) if calls["n"] <= tiled_calls else None

    monkeypatch.setattr(ops, "tile_weights_if_room", no_room)
    folder = model_folders[("B", "bfloat16")]
    plain = PlainLlama(folder)
    model, cfg = load_model(folder, "bfloat16")
    with_tiles = [b.mixer.streams for b in model.blocks] + [b.feed_forward.streams for b in model.blocks] + [model.head.streams]
    assert sum(with_tiles) == tiled_calls and calls["n"] == len(with_tiles)
    assert not model.head.streams            # the head is bound last: it is the first to do without
    eng = Engine(model, num_pages=64, page_size=16, max_requests=4, max_batch_tokens=256)
    g = torch.Generator().manual_seed(2)
    toks = torch.randint(0, cfg.vocab_size, (90,), generator=g).tolist()
    ref = plain.forward(toks)
    eng.admit("r")
    got = [eng.step([StepEntry("r", toks[:70], list(range(70)))]).clone()]
    for t in toks[70:]:
        got.append(eng.step([StepEntry("r", [t], [0])]).clone())
    assert rel_err(torch.cat(got), ref) < TOL["bfloat16"]
    # another request beside it: 17 to 64 rows in a step, then both decoding
    other = torch.randint(0, cfg.vocab_size, (40,), generator=g).tolist()
    eng.admit("s")
    both = eng.step([StepEntry("r", [toks[0]], []), StepEntry("s", other, list(range(40)))])
    assert rel_err(both, plain.forward(other)) < TOL["bfloat16"]


def test_the_cache_pool_follows_the_free_memory(model_folders):
    """Without a number the pool is what every slot at its full context takes (there is room for
    that here); a number that the free memory does not hold is refused with the bytes it needs
    and the bytes there are, and nothing has been allocated by then."""
    from hfee_amd.cache import CacheError, bytes_per_token
    from hfee_amd.engine import Engine, load_model
    model, cfg = load_model(model_folders[("A", "bfloat16")], "bfloat16")
    eng = Engine(model, page_size=16, max_requests=4, max_batch_tokens=64)
    assert eng.num_pages == 4 * (cfg.max_position_embeddings // 16) == eng.cache.pools[0].num_pages
    assert Engine(model, page_size=16, max_requests=4, max_batch_tokens=64, cache_tokens=100).num_pages == 7
    free, total = torch.cuda.mem_get_info()
    page = 16 * bytes_per_token(eng.groups, torch.bfloat16)
    before = torch.cuda.memory_allocated()
    with pytest.raises(CacheError, match="pages would fit") as e:
        Engine(model, num_pages=free // page + 10, page_size=16, max_requests=4, max_batch_tokens=64)
    assert f"{total:,}" in str(e.value) and torch.cuda.memory_allocated() == before


def test_a_pool_whose_layers_are_larger_than_four_gigabytes(tmp_path):
    """One layer with 8 KV heads of 128 and a pool of 70,000 pages: 4.6 GB a cache layer, as
    the free memory of this GPU makes them at production sizes.  A request that holds the
    first 66,000 pages pushes the others' pages beyond the 4 GiB mark.  A prompt of 150 tokens
    from its start (the step's plan asks for the prefill kernel that walks a row tile's keys in
    two halves, which does not take such a layer: the mixer falls back at the launch), another
    in portions beside decoded tokens, then both decode; against the plain model."""
    from conftest import make_model_folder
    from plain_llama import PlainLlama
    from hfee_amd.engine import Engine, StepEntry, load_model
    from hfee_amd.kernels import ops
    if torch.cuda.mem_get_info()[0] < 12 << 30:
        pytest.skip("needs 12 GB of free device memory")
    cj = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 1, "hidden_size": 64,
          "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 96, "vocab_size": 256,
          "max_position_embeddings": 512, "rope_theta": 10000.0, "rope_scaling": None, "rms_norm_eps": 1e-5,
          "tie_word_embeddings": True, "hidden_act": "silu"}
    folder = make_model_folder(tmp_path / "m", cj, seed=5, dtype="bfloat16", std=0.1, norm_init="one_plus_normal")
    plain = PlainLlama(folder)
    model, cfg = load_model(folder, "bfloat16")
    eng = Engine(model, num_pages=70_000, page_size=16, max_requests=4, max_batch_tokens=256)
    layer = eng.storage.layer(0, (2, 8, 16 * 128))
    assert layer.numel() * 2 > 1 << 32 and not ops.attention_halves_fit(128, 4, layer) and ops.attention_halves_fit(128, 4)
    eng.admit("holder")
    eng.cache.reserve("holder", 66_000 * 16)
    g = torch.Generator().manual_seed(3)
    a = torch.randint(0, 256, (170,), generator=g).tolist()
    b = torch.randint(0, 256, (120,), generator=g).tolist()
    eng.admit("a")
    eng.admit("b")
    got = {}
    out = eng.step([StepEntry("a", a[:150], [0, 149])])
    got["a", 0], got["a", 149] = out[0].clone(), out[1].clone()
    assert min(eng.cache.block_table("a", 0)) >= 66_000
    out = eng.step([StepEntry("b", b[:70], [69]), StepEntry("a", a[150:151], [0])])
    got["b", 69], got["a", 150] = out[0].clone(), out[1].clone()
    out = eng.step([StepEntry("a", a[151:152], [0]), StepEntry("b", b[70:100], [29])])
    got["a", 151], got["b", 99] = out[0].clone(), out[1].clone()
    for i in range(18):
        out = eng.step([StepEntry("a", [a[152 + i]], [0]), StepEntry("b", [b[100 + i]], [0])])
        got["a", 152 + i], got["b", 100 + i] = out[0].clone(), out[1].clone()
    eng.cache.check()
    ref = {"a": plain.forward(a), "b": plain.forward(b[:118])}
    for (r, p), row in got.items():
        assert rel_err(row, ref[r][p]) < TOL["bfloat16"], (r, p, rel_err(row, ref[r][p]))
    del eng, layer
    torch.cuda.empty_cache()
