"""The Python entry point: LLM(model_folder).generate(prompts, SamplingParams).

It stands where the reference has Runner.Generate(ctx, prompt, opts, emit)
(/root/reference/internal/llm/runner.go:93-141), called in-process: the prompt (text
or token ids) is queued, the scheduler runs steps until every request has finished,
and each request returns its tokens, text (when the folder has a tokenizer), stats
and the reason it ended.
"""
from __future__ import annotations

import os
from dataclasses import dataclass

from .engine import Engine, load_model, random_model
from .engine.scheduler import Request, Scheduler, Stats
from .sampling import Sampler, SamplingParams
from .text import Stopper, Utf8Buffer, load_tokenizer


@dataclass
class Output:
    token_ids: list
    text: str | None
    stats: Stats
    done_reason: str
    error: str | None = None


class LLM:
    def __init__(self, model=None, *, config=None, random_weights: bool = False, seed: int = 0,
                 dtype: str = "bfloat16", num_ctx: int = 4096, num_parallel: int = 4,
                 max_batch_tokens: int = 2048, page_size: int = 16, num_pages: int | None = None,
                 device: str = "cuda:0", weight_std: float = 0.02, keep_prefixes: bool = True):
        """model: a folder with config.json and model.safetensors.  With
        random_weights=True (or config=... and no folder) the weights are seeded
        random numbers made on the device.  num_ctx is the context window of one
        request, num_parallel the number of requests served at once (the
        reference's HFEE_NUM_CTX and HFEE_NUM_PARALLEL,
        /root/reference/internal/server/server.go:46-57), max_batch_tokens the token
        budget of a step (256 in the reference, /root/reference/internal/llm/runner.go:11).
        keep_prefixes: a finished request's full pages stay in the cache, and a prompt that
        begins with the same tokens does not run them again (the reference reuses the longest
        common prefix of a free slot's tokens, runner.go:198-229).  num_pages: the cache pool in
        pages of page_size tokens; by default every request slot can hold its whole context, as
        far as the device's free memory allows after the weights."""
        from .config import config_from_folder
        if model is not None and not random_weights:
            self.model, self.config = load_model(model, dtype, device)
        else:
            self.config = config if config is not None else config_from_folder(model)
            self.model = random_model(self.config, seed, dtype, device, std=weight_std)
        spec = self.model.spec
        self.num_ctx = max(1, min(num_ctx, spec.max_positions))
        max_batch_tokens = max(1, min(max_batch_tokens, 65536))
        # (num_pages None: what num_parallel requests of num_ctx tokens take, or what the free memory
        # holds if that is less; a number that does not fit is refused before anything is allocated)
        self.engine = Engine(self.model, num_pages=num_pages, page_size=page_size, max_requests=num_parallel,
                             keep_prefixes=keep_prefixes,
                             max_batch_tokens=max_batch_tokens, num_positions=self.num_ctx, device=device)
        self.sampler = Sampler(spec.vocab, self.engine.device, max_rows=num_parallel)
        self.scheduler = Scheduler(self.engine, self.sampler, max_num_seqs=num_parallel,
                                   max_batch_tokens=max_batch_tokens, num_ctx=self.num_ctx,
                                   eos_token_ids=spec.eos_token_ids)
        self.tokenizer = load_tokenizer(model) if isinstance(model, str) and os.path.isdir(model) else None
        self._next_id = 0

    def encode(self, text: str) -> list:
        if self.tokenizer is None:
            raise ValueError("this model folder has no tokenizer.json: give prompts as lists of token ids")
        ids = self.tokenizer.encode(text)
        bos = self.model.spec.bos_token_id
        if bos is not None and (not ids or ids[0] != bos):
            ids = [bos] + ids
        return ids

    def generate(self, prompts, params=None, on_token=None) -> list:
        """prompts: list of token-id lists (or strings, with a tokenizer).  params:
        one SamplingParams for all, or one per prompt.  on_token(index, token_id, text)
        is called as tokens arrive."""
        if params is None:
            params = SamplingParams()
        plist = list(params) if isinstance(params, (list, tuple)) else [params] * len(prompts)
        if len(plist) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        requests, helpers = [], {}
        for i, (prompt, p) in enumerate(zip(prompts, plist)):
            ids = self.encode(prompt) if isinstance(prompt, str) else [int(t) for t in prompt]
            rid = self._next_id
            self._next_id += 1
            req = Request(rid, ids, p, seed=p.resolved_seed())
            helpers[rid] = {"index": i, "utf8": Utf8Buffer(), "stop": Stopper(list(p.stop)), "text": [],
                            "first": True, "hit": False}
            req.on_token = self._make_emit(helpers[rid], on_token)
            requests.append(req)
        outputs: dict = {}
        for req in requests:
            self.scheduler.add(req)
        try:
            while self.scheduler.has_work():
                for fin in self.scheduler.step():
                    h = helpers[fin.request.request_id]
                    text = None
                    if self.tokenizer is not None:
                        tail = h["stop"].flush() + h["utf8"].flush()
                        if tail and not h["hit"]:
                            h["text"].append(tail)
                        text = "".join(h["text"])
                    outputs[fin.request.request_id] = Output(list(fin.request.generated), text, fin.request.stats,
                                                             fin.reason, fin.error)
        except BaseException:
            # interrupted (Ctrl-C, an error in on_token): what is unfinished is cancelled, as the
            # reference ends a request whose caller has gone (/root/reference/internal/llm/runner.go:244-247),
            # so that its pages are free for the next call
            for req in requests:
                if req.request_id not in outputs:
                    self.scheduler.cancel(req.request_id)
            while self.scheduler.has_work():
                self.scheduler.step()
            raise
        return [outputs[r.request_id] for r in requests]

    def _make_emit(self, h, on_token):
        def emit(req, token):
            text = None
            hit = False
            if self.tokenizer is not None:
                piece = h["utf8"].add(self.tokenizer.piece(token))
                if h["first"]:
                    piece = piece.lstrip(" ")      # runner.go:296-299
                    h["first"] = piece == ""
                text, hit = h["stop"].push(piece)
                h["hit"] = hit
                if text:
                    h["text"].append(text)
            if on_token is not None:
                on_token(h["index"], token, text)
            return hit
        return emit
