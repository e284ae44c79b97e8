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
