"""Helpers for the replay tests: ways of cutting the same requests into steps."""
import random

import numpy as np


def whole(requests):
    """Each request alone, all its tokens in one step, logits everywhere."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"entries": [(rid, toks, list(range(len(toks))))], "end": [rid]})
    return steps


def bulk_then_tail(requests, tail=32):
    """All but the last `tail` tokens in one step, then one token per step."""
    steps = []
    for rid, toks in requests.items():
        cut = max(1, len(toks) - tail)
        steps.append({"entries": [(rid, toks[:cut], list(range(cut)))], "end": []})
        for i in range(cut, len(toks)):
            steps.append({"entries": [(rid, toks[i:i + 1], [0])], "end": [rid] if i == len(toks) - 1 else []})
        if cut == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests, sizes=(7, 16, 2, 5, 3, 2, 11, 17, 2, 31, 4, 2, 9)):
    """Portions of changing size, down to two tokens."""
    steps = []
    for rid, toks in requests.items():
        i, k = 0, 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            steps.append({"entries": [(rid, toks[i:i + n], list(range(n)))], "end": [rid] if i + n == len(toks) else []})
            i += n
    return steps


def mixed(requests, seed=0, live_max=4, tail=32, max_portion=19):
    """Up to live_max requests at a time: portions of some beside single decoded tokens
    of others; a request may sit a step out; finished requests end so that their pages
    are used again.  Returns (steps, peak tokens held, each rounded up to 64)."""
    rng = random.Random(seed)
    pending = list(requests.items())
    live = {}      # rid -> (tokens, fed)
    steps, peak = [], 0
    while pending or live:
        while pending and len(live) < live_max and (not live or rng.random() < 0.6):
            rid, toks = pending.pop(0)
            live[rid] = [toks, 0]
        entries, end = [], []
        for rid in list(live):
            toks, fed = live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue
            left = len(toks) - fed
            n = 1 if left <= tail else min(rng.randint(2, max_portion), left - tail)
            entries.append((rid, toks[fed:fed + n], list(range(n))))
            live[rid][1] = fed + n
            if fed + n == len(toks):
                end.append(rid)
        if not entries:
            continue
        rng.shuffle(entries)
        held = sum((v[1] + 63) // 64 * 64 for v in live.values())
        peak = max(peak, held)
        steps.append({"entries": entries, "end": end})
        for rid in end:
            del live[rid]
    return steps, peak


def run(replayer, steps):
    """Runs the steps; returns {(request, position): logits row}."""
    out, fed = {}, {}
    for st in steps:
        logits = replayer.step(st["entries"], st["end"])
        i = 0
        for rid, toks, want in st["entries"]:
            base = fed.get(rid, 0)
            for w in want:
                out[(rid, base + w)] = logits[i]
                i += 1
            fed[rid] = base + len(toks)
        for rid in st["end"]:
            fed.pop(rid, None)
        assert logits is None or i == logits.shape[0]
    return out


def make_requests(vocab, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, vocab, size=n).tolist() for i, n in enumerate(lengths)}


# A greedy token can only be compared across precisions where the choice is clear.  The
# margin of a choice is (largest logit - second largest) / max |logit| in the plain
# implementation; bfloat16 logits are within a few thousandths of max |logit| of it, so a
# choice with a margin above NEAR_TIE is the same in every precision and every batch.
NEAR_TIE = 3e-2


def greedy_margins(plain, prompt, tokens):
    """The margin of every greedy choice along prompt + tokens (teacher-forced)."""
    import torch
    seq = list(prompt) + list(tokens)
    logits = plain.forward(seq[:-1]) if len(seq) > 1 else None
    out = []
    for i in range(len(tokens)):
        row = logits[len(prompt) - 1 + i]
        top = torch.topk(row, 2).values
        out.append(float((top[0] - top[1]) / row.abs().max()))
    return out


def agree_until_a_near_tie(got, want, margins, what=""):
    """Asserts that `got` equals `want` token by token; they may part only at a choice whose
    margin is below NEAR_TIE (after that the two are different sequences and nothing more
    can be compared).  Returns how many tokens agreed."""
    n = 0
    for g, w, m in zip(got, want, margins):
        if g != w:
            assert m < NEAR_TIE, f"{what}: token {n} is {g}, expected {w} (margin {m:.3f}); got {got}, want {want}"
            break
        n += 1
    return n
