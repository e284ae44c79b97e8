"""Generation through the entry point: greedy and seeded sampling, scheduler on the GPU."""
import pytest

import trace_util as tu

pytestmark = pytest.mark.gpu


def test_greedy_generation_matches_the_plain_implementation(model_folders):
    """Tiny A's workload: prompts of 5, 17, 32 and 1 tokens, 16 greedy tokens each."""
    from plain_llama import PlainLlama
    from hfee_amd import LLM, SamplingParams
    folder = model_folders[("A", "float32")]
    plain = PlainLlama(folder)
    prompts = list(tu.make_requests(256, [5, 17, 32, 1], seed=1).values())
    llm = LLM(folder, dtype="float32", num_ctx=128, num_parallel=4, max_batch_tokens=24)
    outs = llm.generate(prompts, SamplingParams.greedy(num_predict=16))
    for p, o in zip(prompts, outs):
        assert o.token_ids == plain.greedy(p, 16)
        assert o.done_reason == "length" and o.stats.eval_tokens == 16 and o.stats.prompt_tokens == len(p)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_seeded_sampling_does_not_depend_on_the_batch(model_folders, dtype):
    """Tiny B's workload: prompts of 40, 3 and 100 tokens, portions of 16, 24 tokens at
    temperature 0.8 with a fixed seed.  In 32-bit, together, alone and in another order give
    the same tokens (the bits of a row do not depend on the batch).  In bfloat16 the kernels
    differ with the number of rows, and a draw from a flat distribution turns on the last
    bits: there the requests run together in the opposite order with a budget that takes all
    prompts in one step, which changes which row of the batch and of the sampler each one is
    and nothing else, and the tokens must be the same."""
    from hfee_amd import LLM, SamplingParams
    folder = model_folders[("B", dtype)]
    prompts = list(tu.make_requests(320, [40, 3, 100], seed=2).values())
    params = [SamplingParams(temperature=0.8, seed=100 + i, num_predict=24) for i in range(3)]
    if dtype == "float32":
        llm = LLM(folder, dtype=dtype, num_ctx=256, num_parallel=3, max_batch_tokens=16)
        together = llm.generate(prompts, params)
        assert len({tuple(o.token_ids) for o in together}) == 3, "three requests, three streams"
        for p, sp, o in zip(prompts, params, together):
            assert len(o.token_ids) == 24 and llm.generate([p], sp)[0].token_ids == o.token_ids
        order = [2, 0, 1]
        again = llm.generate([prompts[i] for i in order], [params[i] for i in order])
        assert [o.token_ids for o in again] == [together[i].token_ids for i in order]
    # (nothing kept between the calls: a prompt of which whole pages are found in the cache runs
    # its rest as a smaller step, through other kernels, and bfloat16 rounds differently there)
    wide = LLM(folder, dtype=dtype, num_ctx=256, num_parallel=3, max_batch_tokens=256, keep_prefixes=False)
    a = wide.generate(prompts, params)
    b = wide.generate(list(reversed(prompts)), list(reversed(params)))
    assert all(len(o.token_ids) == 24 for o in a) and len({tuple(o.token_ids) for o in a}) == 3
    assert [o.token_ids for o in a] == [o.token_ids for o in reversed(b)]


def test_greedy_bfloat16_does_not_depend_on_the_batch(model_folders):
    """bfloat16, greedy: each request alone, all together, and the plain implementation
    agree on every token up to the first choice that is a near tie in the plain
    implementation's logits (there a last bit may decide, and what follows is another
    sequence)."""
    from plain_llama import PlainLlama
    from hfee_amd import LLM, SamplingParams
    checked = 0
    for name, vocab, lengths in (("A", 256, [5, 17, 32, 1]), ("B", 320, [40, 3, 100])):
        folder = model_folders[(name, "bfloat16")]
        plain = PlainLlama(folder)
        prompts = list(tu.make_requests(vocab, lengths, seed=12).values())
        sp = SamplingParams.greedy(num_predict=20)
        llm = LLM(folder, dtype="bfloat16", num_ctx=128, num_parallel=4, max_batch_tokens=24)
        together = llm.generate(prompts, sp)
        for p, o in zip(prompts, together):
            want = plain.greedy(p, 20)
            margins = tu.greedy_margins(plain, p, want)
            alone = llm.generate([p], sp)[0]
            checked += tu.agree_until_a_near_tie(o.token_ids, want, margins, f"{name} together")
            tu.agree_until_a_near_tie(alone.token_ids, want, margins, f"{name} alone")
    assert checked >= 40, f"only {checked} tokens could be compared: the test has lost its teeth"


def test_scarce_pages_preempt_and_still_give_the_same_tokens(model_folders):
    from hfee_amd import LLM, SamplingParams
    folder = model_folders[("A", "float32")]
    prompts = list(tu.make_requests(256, [30, 28, 26, 31], seed=4).values())
    sp = SamplingParams.greedy(num_predict=40)
    roomy = LLM(folder, dtype="float32", num_ctx=128, num_parallel=4)
    want = [o.token_ids for o in roomy.generate(prompts, sp)]
    tight = LLM(folder, dtype="float32", num_ctx=128, num_parallel=4, num_pages=10)   # 160 tokens for 4 x 70
    outs = tight.generate(prompts, sp)
    assert [o.token_ids for o in outs] == want
    assert sum(o.stats.preemptions for o in outs) > 0
    assert outs[0].stats.preemptions == 0, "the request admitted first is never preempted"
    tight.engine.cache.check()
    assert not tight.engine.cache.requests


def test_scarce_pages_preempt_in_bfloat16(model_folders):
    """The same on the bfloat16 kernels: a preempted request reads its own tokens again as a
    prompt (other kernels than the single steps that made them), so its tokens are compared
    with the plain implementation's up to the first near tie."""
    from plain_llama import PlainLlama
    from hfee_amd import LLM, SamplingParams
    folder = model_folders[("A", "bfloat16")]
    plain = PlainLlama(folder)
    prompts = list(tu.make_requests(256, [30, 28, 26, 31], seed=4).values())
    sp = SamplingParams.greedy(num_predict=40)
    tight = LLM(folder, dtype="bfloat16", num_ctx=128, num_parallel=4, num_pages=10)
    outs = tight.generate(prompts, sp)
    assert sum(o.stats.preemptions for o in outs) > 0 and outs[0].stats.preemptions == 0
    assert all(len(o.token_ids) == 40 and o.done_reason == "length" for o in outs)
    checked = 0
    for p, o in zip(prompts, outs):
        want = plain.greedy(p, 40)
        checked += tu.agree_until_a_near_tie(o.token_ids, want, tu.greedy_margins(plain, p, want), "preempted")
    assert checked >= 30, f"only {checked} tokens could be compared"
    tight.engine.cache.check()
    assert not tight.engine.cache.requests


def test_stop_on_eos_and_context_limit(model_folders, tmp_path):
    import json, os, shutil
    from plain_llama import PlainLlama
    from hfee_amd import LLM, SamplingParams
    src = model_folders[("A", "float32")]
    plain = PlainLlama(src)
    prompt = tu.make_requests(256, [12], seed=6)["r0"]
    cont = plain.greedy(prompt, 8)
    # make the 4th generated token the end-of-sequence id
    dst = tmp_path / "eos"
    shutil.copytree(src, dst)
    cj = json.load(open(dst / "config.json"))
    eos = cont[3]
    cj["eos_token_id"] = eos
    json.dump(cj, open(dst / "config.json", "w"))
    llm = LLM(str(dst), dtype="float32", num_ctx=128, num_parallel=2)
    o = llm.generate([prompt], SamplingParams.greedy(num_predict=8))[0]
    first = cont.index(eos)
    assert o.token_ids == cont[:first] and o.done_reason == "stop"
    o = llm.generate([prompt], SamplingParams.greedy(num_predict=8, ignore_eos=True))[0]
    assert o.token_ids == cont and o.done_reason == "length"
    # the context window ends a request with "length"
    small = LLM(src, dtype="float32", num_ctx=20, num_parallel=1)
    o = small.generate([prompt], SamplingParams.greedy())[0]
    assert o.done_reason == "length" and len(prompt) + len(o.token_ids) == 21
    with pytest.raises(ValueError, match="context window"):
        small.generate([list(range(20))], SamplingParams.greedy())


def test_a_prompt_given_as_text(model_folders, tmp_path):
    """A folder with a tokenizer.json takes text: the prompt's ids (after the begin-of-sequence
    id the configuration names) are the tokenizer's, the tokens are the plain implementation's,
    the text is their bytes joined (leading spaces of the answer dropped), and a stop string
    ends the answer in front of it."""
    import json, shutil
    from plain_llama import PlainLlama
    from test_text import MERGES, byte_level_folder
    from hfee_amd import LLM, SamplingParams
    from hfee_amd.text import FolderTokenizer
    dst = tmp_path / "with_text"
    shutil.copytree(model_folders[("B", "float32")], dst)
    path, vocab = byte_level_folder(dst, MERGES, added=[("<|eot|>", True)])
    cj = json.load(open(dst / "config.json"))
    cj["bos_token_id"] = len(vocab)
    json.dump(cj, open(dst / "config.json", "w"))
    tok = FolderTokenizer(path)
    prompt = "hello world 123<|eot|>hello"
    ids = [len(vocab)] + tok.encode(prompt)
    assert ids[1] == vocab["hello"] and ids.count(len(vocab)) == 2 and len(ids) < len(prompt)
    want = PlainLlama(str(dst)).greedy(ids, 24)
    text = b"".join(tok.piece(t) for t in want).decode("utf-8", errors="replace").lstrip(" ")
    assert len(text) >= 8            # tokens beyond the tokenizer's vocabulary print nothing
    llm = LLM(str(dst), dtype="float32", num_ctx=128, num_parallel=2)
    assert llm.encode(prompt) == ids
    seen = []
    o = llm.generate([prompt], SamplingParams.greedy(num_predict=24), on_token=lambda i, t, piece: seen.append(piece))[0]
    assert o.token_ids == want and o.text == text and "".join(seen) + o.text[len("".join(seen)):] == text
    stop = text[5:7]
    o = llm.generate([prompt], SamplingParams.greedy(num_predict=24, stop=(stop,)))[0]
    assert o.text == text[:text.index(stop)] and o.done_reason == "stop"
    assert len(o.token_ids) < len(want) and o.token_ids == want[:len(o.token_ids)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_conversation_that_goes_on_runs_only_what_is_new(model_folders, dtype):
    """Through the entry point: the second call's prompt is the first prompt, its answer and a
    few more tokens.  Whole pages of it are found in the cache (the statistics say how many
    tokens were run, as the reference counts them), and the tokens are those of the plain
    model over the whole prompt.  With keep_prefixes=False everything is run."""
    from plain_llama import PlainLlama
    from hfee_amd import LLM, SamplingParams
    folder = model_folders[("A", dtype)]
    plain = PlainLlama(folder)
    prompt = tu.make_requests(256, [40], seed=12)["r0"]
    llm = LLM(folder, dtype=dtype, num_ctx=128, num_parallel=2)
    first = llm.generate([prompt], SamplingParams.greedy(num_predict=12))[0]
    assert first.stats.prompt_tokens == 40 and first.stats.reused_tokens == 0
    follow = prompt + first.token_ids + [3, 1, 4]
    out = llm.generate([follow], SamplingParams.greedy(num_predict=10))[0]
    assert out.stats.reused_tokens == 48 and out.stats.prompt_tokens == len(follow) - 48      # 51 tokens lie in the cache
    want = plain.greedy(follow, 10)
    if dtype == "float32":
        assert out.token_ids == want
    else:
        assert tu.agree_until_a_near_tie(out.token_ids, want, tu.greedy_margins(plain, follow, want), "after a kept prefix") >= 3
    plain_llm = LLM(folder, dtype=dtype, num_ctx=128, num_parallel=2, keep_prefixes=False)
    plain_llm.generate([prompt], SamplingParams.greedy(num_predict=12))
    again = plain_llm.generate([follow], SamplingParams.greedy(num_predict=10))[0]
    assert again.stats.reused_tokens == 0 and again.stats.prompt_tokens == len(follow)
    if dtype == "float32":
        assert again.token_ids == out.token_ids
    llm.engine.cache.check()


def test_an_interrupted_call_leaves_nothing_behind(model_folders):
    """An error from the caller's on_token ends the call; its requests are cancelled and
    their pages freed, and the next call gives the usual tokens."""
    from hfee_amd import LLM, SamplingParams
    folder = model_folders[("A", "float32")]
    prompts = list(tu.make_requests(256, [9, 20], seed=4).values())
    llm = LLM(folder, dtype="float32", num_ctx=128, num_parallel=2)
    want = [o.token_ids for o in llm.generate(prompts, SamplingParams.greedy(num_predict=10))]

    class Stop(Exception):
        pass

    seen = []

    def on_token(index, token, text):
        seen.append(token)
        if len(seen) == 5:
            raise Stop()

    with pytest.raises(Stop):
        llm.generate(prompts, SamplingParams.greedy(num_predict=10), on_token=on_token)
    assert not llm.scheduler.has_work() and not llm.engine.cache.requests
    llm.engine.cache.check()
    assert [o.token_ids for o in llm.generate(prompts, SamplingParams.greedy(num_predict=10))] == want


def test_the_command_line_generates_from_token_ids(model_folders):
    """`hfee run <model> --tokens ...` as a user calls it: the ids of the greedy
    continuation, and with --verbose the counts that the reference prints."""
    import os, subprocess, sys
    from plain_llama import PlainLlama
    folder = model_folders[("A", "float32")]
    prompt = tu.make_requests(256, [11], seed=8)["r0"]
    want = PlainLlama(folder).greedy(prompt, 7)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "hfee"), "run", folder, "--tokens",
                        ",".join(map(str, prompt)), "--dtype", "float32", "--temperature", "0", "--repeat-penalty", "1",
                        "--num-predict", "7", "--num-ctx", "128", "--verbose"],
                       capture_output=True, text=True, timeout=300, stdin=subprocess.DEVNULL)
    assert p.returncode == 0, p.stderr[-2000:]
    first = p.stdout.strip().splitlines()[0]
    assert [int(t) for t in first.split()] == want
    assert "prompt eval count:    11 token(s)" in p.stdout and "eval count:           7 token(s)" in p.stdout
    assert "done reason:          length" in p.stdout
    # without a prompt and without a terminal there is nothing to do
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "hfee"), "run", folder, "--dtype", "float32"],
                       capture_output=True, text=True, timeout=300, stdin=subprocess.DEVNULL)
    assert p.returncode == 1 and "usage" in p.stderr


@pytest.mark.parametrize("dtype,temperature,penalty", [("float32", 0.0, 1.0), ("bfloat16", 0.0, 1.0), ("float32", 0.7, 1.0),
                                                       ("float32", 0.7, 1.3), ("float32", 0.0, 1.5)])
def test_steps_launched_ahead_give_the_tokens_of_steps_that_wait(model_folders, dtype, temperature, penalty):
    """The scheduler launches a decode step before it has read the ids of the step before
    (they go from the sampler to the embedding on the device).  With that switched off the
    same requests give the same tokens and reasons: greedy and seeded sampling, with and
    without a penalty on the requests' own earlier tokens (the newest of which the sampler
    then takes from the device), requests of different lengths of which some end early on an end-of-sequence id, so that steps that
    were launched ahead for them run for nobody."""
    from hfee_amd import LLM, SamplingParams
    folder = model_folders[("A", dtype)]
    prompts = list(tu.make_requests(256, [5, 17, 32, 1], seed=7).values())

    def run(look_ahead, eos=None):
        llm = LLM(folder, dtype=dtype, num_ctx=128, num_parallel=4, max_batch_tokens=24)
        assert llm.scheduler.look_ahead
        llm.scheduler.look_ahead = look_ahead
        if eos is not None:
            llm.scheduler.eos = {eos}
        params = [SamplingParams(temperature=temperature, top_k=0, top_p=1.0, repeat_penalty=penalty,
                                 repeat_last_n=[64, 5, -1, 1][i], seed=50 + i, num_predict=n)
                  for i, n in enumerate([40, 12, 33, 25])]
        outs = llm.generate(prompts, params)
        llm.engine.cache.check()
        assert not llm.engine.cache.requests
        return [(o.token_ids, o.done_reason) for o in outs], llm.scheduler.steps_ahead

    waited, none_ahead = run(False)
    assert none_ahead == 0
    # an id that the longest request samples in its middle: with it as end-of-sequence id that request stops early
    eos = waited[0][0][20]
    waited, _ = run(False, eos)
    assert any(reason == "stop" for _, reason in waited)
    ahead, launched_ahead = run(True, eos)
    assert launched_ahead > 10
    assert ahead == waited
