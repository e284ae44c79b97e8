"""The engine against the plain implementation: whole prompts first."""
import pytest
import torch

from conftest import TINY

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
