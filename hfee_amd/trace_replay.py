"""Trace replay: feeds given token ids through the engine step by step and writes
the logits that are asked for.  Nothing is sampled.  It drives the same model,
step function, cache and kernels that generation uses.

The closest thing in the reference is State.Forward, which appends tokens and
returns the last logits (/root/reference/internal/llm/forward.go:36-39).

Input: one JSON object per line,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
`want` may also be "all" (every token of the entry) or "last".
Output: for a step in which something is wanted, <out>/<step>.f32 holds the logits
at the wanted places as little-endian float32 [wanted, vocab], in the order of the
entries and of `want`.  After every step a line `done <step>` is printed.

Or a whole trace in one file (`--trace FILE`, `replay(trace)` in Python), which names its
model itself:
    {"model": DIR | {"config": {config.json's keys}, "random_weights": {"seed": S}},
     "dtype": "float32", "page_size": 16, "num_pages": N | "max_tokens": T,
     "steps": [{"segments": [{"req": "a", "tokens": [...], "want": "all" | "last" | [k...]}],
                "release": ["a"]}]}
(`entries` / `id` / `end` are read as well).  Step i writes <out>/<i>.f32 as above.
"""
from __future__ import annotations

import json
import os
import sys

import numpy as np


def _split(entries, limit):
    """Cuts a step that is larger than the workspace into consecutive steps."""
    from .engine import StepEntry
    steps, current, room = [], [], limit
    for e in entries:
        tokens, want, offset = list(e.tokens), sorted(set(e.want)), 0
        while offset < len(tokens):
            take = min(room, len(tokens) - offset)
            current.append(StepEntry(e.request_id, tokens[offset:offset + take],
                                     [w - offset for w in want if offset <= w < offset + take]))
            offset += take
            room -= take
            if room == 0:
                steps.append(current)
                current, room = [], limit
    if current:
        steps.append(current)
    return steps


def wanted_places(want, count: int) -> list:
    """`want` of a trace entry as a list of places among the entry's tokens: a list is
    taken as it is, "all" is every token, "last" the last one."""
    if want is None:
        return []
    if isinstance(want, str):
        if want == "all":
            return list(range(count))
        if want == "last":
            return [count - 1]
        raise ValueError(f'want must be a list of places, "all" or "last", not {want!r}')
    return [int(w) for w in want]


class Replayer:
    """max_tokens: the most tokens that live requests hold at any time, each request's count
    rounded up to a multiple of 64 (to a whole page where pages are larger: then every live
    request may leave one more page partly empty, and the pool has one for each).  The page
    pool is made for exactly that, so that pages are given back and used again.
    batch_limit: the most tokens one engine step takes (larger steps of a trace are cut).
    model_dir may be config.json's keys as a dict: the weights are then seeded random ones
    (seed; random_options: std, norm_init).  num_pages, if given, is the pool as it is."""

    def __init__(self, model_dir: str, dtype: str, max_tokens: int, page_size: int = 16,
                 max_requests: int = 64, device: str = "cuda:0", batch_limit: int | None = None,
                 random_weights: bool = False, seed: int = 0, num_pages: int | None = None,
                 random_options: dict | None = None):
        from .engine import Engine, load_model, random_model
        from .config.registry import config_from_dict, config_from_folder
        if isinstance(model_dir, dict):            # config.json's keys instead of a folder: random weights
            model = random_model(config_from_dict(model_dir), seed, dtype, device, **(random_options or {}))
        elif random_weights:
            model = random_model(config_from_folder(model_dir), seed, dtype, device, **(random_options or {}))
        else:
            model, _ = load_model(model_dir, dtype, device)
        page = page_size
        if num_pages is not None:
            max_tokens = num_pages * page
        tokens = max(max_tokens, 64)
        pages = (tokens + page - 1) // page + (max_requests if page > 64 else 0)
        if num_pages is not None:
            pages = num_pages
        self.batch_limit = max(1, min(tokens, 8192) if batch_limit is None else batch_limit)
        self.engine = Engine(model, num_pages=pages, page_size=page,
                             max_requests=max_requests, max_batch_tokens=self.batch_limit,
                             num_positions=min(tokens, model.spec.max_positions), device=device)

    def step(self, entries, end=()):
        """entries: [(id, tokens, want)]; returns float32 numpy [wanted, vocab] or None.
        `want` order within an entry is kept."""
        from .engine import StepEntry
        ents = []
        for rid, tokens, want in entries:
            if not self.engine.is_live(rid):
                self.engine.admit(rid)
            ents.append(StepEntry(rid, list(tokens), wanted_places(want, len(tokens))))
        total = sum(len(e.tokens) for e in ents)
        if total <= self.batch_limit:
            logits = self.engine.step(ents)
            out = None if logits is None else logits.cpu().numpy()
        else:
            # rows come back entry by entry, ascending within an entry; put them in `want` order
            parts = {}
            for sub in _split(ents, self.batch_limit):
                logits = self.engine.step(sub)
                if logits is None:
                    continue
                rows = logits.cpu().numpy()
                i = 0
                for e in sub:
                    for _ in e.want:
                        parts.setdefault(e.request_id, []).append(rows[i].copy())
                        i += 1
            out_rows = []
            for e in ents:
                order = sorted(set(e.want))
                got = dict(zip(order, parts.get(e.request_id, [])))
                out_rows += [got[w] for w in e.want]
            out = np.stack(out_rows) if out_rows else None
        for rid in end:
            if self.engine.is_live(rid):
                self.engine.release(rid)
        return out


def replayer_of(trace: dict, device: str = "cuda:0", dtype: str | None = None) -> "Replayer":
    """The replayer that a whole trace describes (its model, dtype, page size and pool)."""
    model = trace.get("model")
    if model is None:
        raise ValueError('the trace names no "model" (a folder, or {"config": {...}, "random_weights": {"seed": S}})')
    options = {}
    seed, random_weights = 0, False
    if isinstance(model, dict):
        if "config" not in model:
            raise ValueError('a trace\'s "model" object needs "config" (the keys of a config.json)')
        rw = dict(model.get("random_weights") or {})
        seed = int(rw.pop("seed", 0))
        options = rw
        model = model["config"]
    if "num_pages" not in trace and "max_tokens" not in trace:
        raise ValueError('the trace must give "num_pages" or "max_tokens"')
    return Replayer(model, dtype or trace.get("dtype", "float32"), int(trace.get("max_tokens", 0)),
                    page_size=int(trace.get("page_size", 16)), max_requests=int(trace.get("max_requests", 64)),
                    device=device, random_weights=random_weights, seed=seed,
                    num_pages=trace.get("num_pages"), random_options=options)


def trace_steps(trace: dict):
    """The steps of a whole trace as (entries, end) with entries [(id, tokens, want)]."""
    for st in trace.get("steps", []):
        entries = [(e.get("req", e.get("id")), e["tokens"], e.get("want", [])) for e in st.get("segments", st.get("entries", []))]
        yield entries, list(st.get("release", st.get("end", [])))


def replay(trace: dict, device: str = "cuda:0", dtype: str | None = None) -> dict:
    """Runs a whole trace; returns {(request, position): float32 logits row} for every wanted
    place, so that runs which cut the same requests differently can be compared key by key."""
    rep = replayer_of(trace, device, dtype)
    out, fed = {}, {}
    for entries, end in trace_steps(trace):
        rows = rep.step(entries, end) if entries else None
        i = 0
        for rid, tokens, want in entries:
            base = fed.get(rid, 0)
            for w in wanted_places(want, len(tokens)):
                out[(rid, base + w)] = rows[i]
                i += 1
            fed[rid] = base + len(tokens)
        for rid in end:
            fed.pop(rid, None)
            if rep.engine.is_live(rid):
                rep.engine.release(rid)
    return out


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int,
                    help="most tokens that live requests hold at any time (the cache pool is made for it)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-requests", type=int, default=64, help="most requests that are live at a time")
    ap.add_argument("--random-weights", action="store_true",
                    help="read config.json only; the weights are seeded random ones")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--trace", help="a whole trace in one JSON file that names its model, dtype and pool itself "
                    "(then nothing is read from standard input)")
    args = ap.parse_args(argv)
    os.makedirs(args.out, exist_ok=True)

    def write(step, out):
        if out is not None:
            tmp = os.path.join(args.out, f".{step}.f32.tmp")
            out.astype("<f4").tofile(tmp)
            os.replace(tmp, os.path.join(args.out, f"{step}.f32"))
        print(f"done {step}", flush=True)

    if args.trace:
        with open(args.trace, "r", encoding="utf-8") as f:
            trace = json.load(f)
        rep = replayer_of(trace, dtype=args.dtype)
        for i, (entries, end) in enumerate(trace_steps(trace)):
            out = rep.step(entries, end) if entries else None
            for rid in end:
                if rep.engine.is_live(rid):
                    rep.engine.release(rid)
            write(i, out)
        return 0
    if not (args.model and args.dtype and args.max_tokens):
        ap.error("--model, --dtype and --max-tokens are required (or --trace FILE)")
    rep = Replayer(args.model, args.dtype, args.max_tokens, page_size=args.page_size,
                   max_requests=args.max_requests, random_weights=args.random_weights, seed=args.seed)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want", [])) for e in rec.get("entries", [])]
        step = rec["step"]
        out = rep.step(entries, rec.get("end", [])) if entries else None
        if not entries:
            for rid in rec.get("end", []):
                if rep.engine.is_live(rid):
                    rep.engine.release(rid)
        write(step, out)
    return 0
