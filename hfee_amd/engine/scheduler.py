"""The scheduler: continuous batching over the step function.

Every step feeds one token from each request that is decoding, then portions of
the prompts still being read, under a token budget, through one step()
(/root/reference/internal/llm/runner.go:231-280).  What the reference decides, it
decides the same way here:

  * a prompt that does not leave room for one new token in the context is refused
    before it queues (runner.go:95-97);
  * decoding requests come first, then prompt portions, in admission order; a
    portion is min(what is left of the prompt, what is left of the budget), and
    logits are asked for only when the portion ends the prompt (runner.go:238-259);
  * after the logits: sample; an end-of-sequence id finishes the request with
    "stop" and is neither kept nor emitted; num_predict is checked after the token
    is emitted, so 0 still yields one token; a full context finishes with "length"
    at the top of a step (runner.go:248-251, 283-314).

The reference reserves a whole context per slot up front, so pages never run out
there.  Here they can, and this is what happens:

  1. requests that run come before requests that wait: decoding requests first, then the
     prompts that are still being read, oldest first, and only then is a waiting request
     admitted, if a state slot is free and a page is free for the beginning of its first
     portion (so the pages that a preemption frees go to those who needed them, not back to
     the request that gave them up); a request that was preempted comes back, while others
     run, not in the step that preempted it and only when the free pages hold all it has to
     run again, its next token, and a page for every running request's next page edge (let
     in on less it would run its tokens again only to give way again);
  2. a prompt portion is shortened to what the free pages hold (or waits a step);
  3. if a decoding request cannot get the page its next token needs, requests younger than
     it are preempted, youngest first: their pages go back, and they return to the front
     of the waiting line with prompt + generated tokens as their new prompt (the sampler
     stream goes on where it was, so the tokens they produce are the same); if it is the
     youngest itself, it is the one that is preempted.  Nobody is ever preempted for the
     sake of a younger request;
  4. a request that is alone and still cannot get a page finishes with "length".
The request admitted first is never preempted, so every step makes progress.

One step ahead.  While every running request only decodes, the next step is known but
for its tokens, and those lie on the device as soon as the sampler has run.  The
scheduler then launches step t+1 (its tokens taken from the sampler's output on the
device) before it reads the tokens of step t: the GPU goes from one step to the next
without waiting for the host.  If a request turns out to have ended at step t (an
end-of-sequence token, a stop from its callback), the token that step t+1 made for it
is dropped; its pages were still its own when that step was queued, and whoever gets
them next runs after it on the same stream.  Nothing is launched ahead when a request
waits, a prompt is unfinished, a request is at its limit of tokens or of context or is
cancelled, or when pages are short: then the step is an ordinary one.  (A penalty on a
request's own earlier tokens needs the latest one, which the host has not seen yet: the
sampler takes it from the device.)
"""
from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field

from ..sampling import SampleRow, SamplingParams
from .step import StepEntry


@dataclass
class Stats:
    """/root/reference/internal/llm/runner.go:15-21"""
    prompt_tokens: int = 0          # tokens of the prompt that were run (runner.go:222: what is fed)
    reused_tokens: int = 0          # tokens of the prompt found in the cache from an earlier request
    prompt_duration: float = 0.0
    eval_tokens: int = 0
    eval_duration: float = 0.0
    done_reason: str = ""
    preemptions: int = 0


@dataclass(eq=False)      # a request is itself, not its contents: membership tests must not compare prompts
class Request:
    request_id: object
    prompt: list
    params: SamplingParams
    seed: int = 0
    feed: list = field(default_factory=list)        # tokens to run next
    generated: list = field(default_factory=list)
    history: list = field(default_factory=list)     # prompt + generated (repeat penalty)
    draws: int = 0
    decoding: bool = False                          # the prompt has been read
    stats: Stats = field(default_factory=Stats)
    started: float = 0.0
    eval_started: float = 0.0
    admitted_order: int = -1
    cancelled: bool = False
    on_token: object = None


@dataclass
class Finished:
    request: Request
    reason: str
    error: str | None = None


class PromptTooLong(ValueError):
    pass


class Scheduler:
    def __init__(self, engine, sampler, *, max_num_seqs: int, max_batch_tokens: int, num_ctx: int,
                 eos_token_ids=(), clock=time.perf_counter):
        self.engine, self.sampler = engine, sampler
        self.cache = engine.cache
        self.max_num_seqs = max_num_seqs
        self.max_batch_tokens = max_batch_tokens
        self.num_ctx = num_ctx
        self.eos = set(eos_token_ids)
        self.clock = clock
        self.waiting: deque = deque()
        self._preempted_now: set = set()      # requests preempted by the step being put together
        self.running: list = []          # in admission order
        self._order = 0
        self.last_batch: list = []       # (request_id, tokens in the step) of the latest step, for tests
        self._ahead = None               # a step that runs already: (owners of its rows, handle of its ids)
        self.steps_ahead = 0             # how many steps were launched before their tokens were known
        self.look_ahead = bool(getattr(engine, "takes_device_tokens", False)) and hasattr(sampler, "device_ids")

    # ----------------------------------------------------------------- intake
    def add(self, request: Request) -> None:
        if len(request.prompt) < 1:
            raise ValueError("an empty prompt")
        if len(request.prompt) >= self.num_ctx:
            raise PromptTooLong(f"prompt is {len(request.prompt)} tokens but the context window is {self.num_ctx}")
        request.feed = list(request.prompt)
        request.history = list(request.prompt)
        request.stats.prompt_tokens = len(request.prompt)
        if request.seed is None or request.seed < 0:
            request.seed = request.params.resolved_seed()
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)       # (a step launched ahead for nobody is just dropped)

    def cancel(self, request_id) -> None:
        for r in list(self.waiting) + self.running:
            if r.request_id == request_id:
                r.cancelled = True

    # ------------------------------------------------------------------ pages
    def _room(self, request: Request) -> int:
        """How many more tokens of `request` the free pages can hold."""
        rc = self.cache.get(request.request_id)
        ps = self.cache.page_size
        room = None
        for table, pool in zip(rc.tables, self.cache.pools):
            r = len(table) * ps - rc.length + pool.num_free * ps
            room = r if room is None else min(room, r)
        return max(room or 0, 0)

    def _comes_back_with(self, request: Request) -> int:
        """Free tokens that a preempted request waits for while others run: room for all it has
        to run again and its next token, and a page for every running request's next page edge.
        Let in on a single free page it would run its prompt and its tokens again only to be
        preempted at the next edge of an older request, step after step."""
        ps = self.cache.page_size
        return (len(request.feed) + 1 + ps - 1) // ps * ps + len(self.running) * ps

    def _preempt(self, victim: Request) -> None:
        self.engine.release(victim.request_id, victim.history)
        self.running.remove(victim)
        self._preempted_now.add(victim.request_id)
        victim.feed = list(victim.prompt) + list(victim.generated)
        victim.decoding = False
        victim.stats.preemptions += 1
        self.waiting.appendleft(victim)

    def _finish(self, request: Request, reason: str, finished: list, error: str | None = None) -> None:
        now = self.clock()
        request.stats.done_reason = reason
        if request.eval_started:
            request.stats.eval_duration = now - request.eval_started
        if self.engine.is_live(request.request_id):
            # (position p of its cache holds history[p]; a last token that was drawn but never
            # run, or run ahead and dropped, is beyond what the two have in common)
            self.engine.release(request.request_id, request.history)
        if request in self.running:
            self.running.remove(request)
        finished.append(Finished(request, reason, error))

    def _decode_shape(self, owners):
        """The shape of the next step if it can only be "each of these requests, which are all
        that run, decodes one more token" (nobody waits for a place, no prompt is unfinished,
        nobody reaches its limit of tokens, nobody is at the end of the context or cancelled),
        else None."""
        if self.waiting or len(owners) != len(self.running):
            return None
        shape = []
        for r, q in zip(owners, self.running):
            if r is not q or len(r.feed) != 0 or r.cancelled:
                return None
            limit = r.params.num_predict
            if limit >= 0 and len(r.generated) + 1 >= limit:
                return None
            if self.cache.get(r.request_id).length + 1 > self.num_ctx:
                return None
            shape.append((r.request_id, 1, [0]))
        return shape

    def _plan_ahead(self, owners) -> None:
        """If the next step is certain but for its tokens, the engine plans it now, while the
        GPU is busy with this one.  A guess that fails (an end-of-sequence token, a
        cancellation) costs nothing but the planning."""
        shape = self._decode_shape(owners)
        if shape:
            self.engine.prepare(shape)

    def _launch_ahead(self, owners):
        """Launches the step after the one whose ids are still on their way, if it is certain
        but for its tokens: they are taken from the sampler's output on the device.
        Returns (owners, handle of the ids) or None."""
        shape = self._decode_shape(owners) if self.look_ahead else None
        if not shape or not self.engine.prepare(shape):
            return None                                  # (pages are short: an ordinary step decides what gives)
        entries = [StepEntry(rid, [0], [0]) for rid, _, _ in shape]
        self.last_batch = [(rid, 1) for rid, _, _ in shape]
        logits = self.engine.step(entries, tokens_from=self.sampler.device_ids)
        # (a request's draw counter and history move when its token is read: this step's draw is
        # the one after, and the newest id of every history is the one that the sampler still
        # holds on the device)
        rows = [SampleRow(r.params, r.seed, r.draws + 1, r.history, i) for i, r in enumerate(owners)]
        self.steps_ahead += 1
        return owners, self.sampler.launch(logits, rows, out=getattr(self.engine, "token_place", None),
                                           latest=self.sampler.device_ids)

    # ------------------------------------------------------------------- step
    def step(self) -> list:
        """One pass: admit, batch, run, sample.  Returns the requests that finished."""
        finished: list = []
        if self._ahead is not None:              # this pass's step runs already
            launched, self._ahead = self._ahead, None
            return self._collect(*launched, finished)
        launched = self._launch(finished)
        return self._collect(*launched, finished) if launched else finished

    def _launch(self, finished: list):
        """Admits, batches, runs a step and starts its sampling: (owners of the sampled rows,
        handle of their ids), or None if no step ran."""
        # cancelled or out of context (runner.go:244-251)
        for r in list(self.running):
            if r.cancelled:
                self._finish(r, "cancelled", finished)
            elif self.cache.get(r.request_id).length >= self.num_ctx:
                self._finish(r, "length", finished)
        for r in [w for w in self.waiting if w.cancelled]:
            self.waiting.remove(r)
            self._finish(r, "cancelled", finished)

        budget = self.max_batch_tokens
        batch: list = []     # (request, tokens, wants_logits)
        self._preempted_now.clear()

        # decoding requests first, oldest first; preempt from the young end if pages run out
        ps = self.cache.page_size
        for r in [x for x in self.running if x.decoding]:
            if r not in self.running:
                continue          # preempted while an older request was served
            if budget == 0:
                break
            rc = self.cache.requests[r.request_id]
            if any(len(t) * ps <= rc.length for t in rc.tables):      # its next token starts a new page
                while self._room(r) < 1 and self.running[-1] is not r:
                    victim = self.running[-1]          # always younger than r
                    batch = [b for b in batch if b[0] is not victim]
                    self._preempt(victim)
                if self._room(r) < 1 and len(self.running) > 1:
                    self._preempt(r)                   # r is the youngest itself: nobody older gives way to it
                    continue
                if self._room(r) < 1:
                    self._finish(r, "length", finished, "the cache cannot hold this request even alone")
                    continue
                self.cache.reserve(r.request_id, 1)
            batch.append((r, r.feed[:1], True))
            budget -= 1
        budget = self.max_batch_tokens - sum(len(t) for _, t, _ in batch)

        # prompt portions of requests admitted earlier, oldest first: they come before anybody
        # new is let in, so that pages which a preemption has freed go to those who waited
        # for them and not back to the request that gave them up
        for r in self.running:
            if r.decoding or budget == 0:
                continue
            n = min(len(r.feed), budget, self._room(r))
            if n < 1:
                continue
            self.cache.reserve(r.request_id, n)
            batch.append((r, r.feed[:n], n == len(r.feed)))
            budget -= n

        # admit waiting requests while there is a slot, a place and pages for a first portion
        while self.waiting and len(self.running) < self.max_num_seqs and self.cache.num_free_slots > 0 and budget > 0:
            r = self.waiting[0]
            first = min(len(r.feed), budget)
            free_tokens = min(p.num_free for p in self.cache.pools) * self.cache.page_size if self.cache.pools else first
            if free_tokens < min(first, self.cache.page_size) and self.running:
                break                      # wait until pages come back
            if r.request_id in self._preempted_now:
                break                      # it has just given its pages up: not back in the same step
            if r.stats.preemptions and self.running and free_tokens < self._comes_back_with(r):
                break                      # it would run its tokens again only to give way again
            if free_tokens < 1:
                self.waiting.popleft()
                self._finish(r, "length", finished, "the cache has no free page for this request")
                continue
            self.waiting.popleft()
            # the beginning of the prompt may lie in the cache from an earlier request
            # (runner.go:198-223): whole pages, and never the whole prompt
            reused = self.engine.admit(r.request_id, r.feed).length
            if reused:
                r.feed = r.feed[reused:]
                if not r.stats.preemptions:
                    r.stats.reused_tokens = reused
                    r.stats.prompt_tokens = len(r.prompt) - reused
            r.admitted_order = self._order
            self._order += 1
            if not r.started:
                r.started = self.clock()
            self.running.append(r)
            # its portion is taken below with the other prompts
            n = min(len(r.feed), budget, self._room(r))
            if n >= 1:
                self.cache.reserve(r.request_id, n)
                batch.append((r, r.feed[:n], n == len(r.feed)))
                budget -= n

        if not batch:
            if self.running and not finished:
                # nothing fits: give the oldest request room by preempting the youngest
                if len(self.running) > 1:
                    self._preempt(self.running[-1])
                else:
                    self._finish(self.running[0], "length", finished,
                                 "the cache cannot hold this request even alone")
            self.last_batch = []
            return None

        entries = [StepEntry(r.request_id, toks, [len(toks) - 1] if want else []) for r, toks, want in batch]
        self.last_batch = [(r.request_id, len(toks)) for r, toks, _ in batch]
        logits = self.engine.step(entries)

        rows, owners = [], []
        for r, toks, want in batch:
            r.feed = r.feed[len(toks):]
            if want:
                owners.append(r)
                rows.append(SampleRow(r.params, r.seed, r.draws, r.history, len(rows)))
        place = getattr(self.engine, "token_place", None) if self.look_ahead else None
        return owners, (self.sampler.launch(logits, rows, out=place) if place is not None
                        else self.sampler.launch(logits, rows))

    def _collect(self, owners, pending, finished: list) -> list:
        """Reads the ids of a step that runs (after launching the step behind it, if that one
        is certain) and gives each request its token."""
        self._ahead = self._launch_ahead(owners)
        if self._ahead is None:
            self._plan_ahead(owners)     # while the GPU runs this step
        fed_ahead = set(id(r) for r in self._ahead[0]) if self._ahead else ()
        ids = self.sampler.collect(pending)
        now = self.clock()
        for r, token in zip(owners, ids):
            if r not in self.running:
                continue                 # it ended at the step before; this token was made for nobody
            if not r.decoding:
                r.decoding = True
                if not r.eval_started:
                    r.stats.prompt_duration = now - r.started
                    r.eval_started = now
            r.draws += 1
            if token in self.eos and not r.params.ignore_eos:
                self._finish(r, "stop", finished)
                continue
            r.generated.append(token)
            r.history.append(token)
            r.stats.eval_tokens = len(r.generated)
            stop_now = False
            if r.on_token is not None:
                stop_now = bool(r.on_token(r, token))
            if stop_now:
                self._finish(r, "stop", finished)
            elif r.params.num_predict >= 0 and len(r.generated) >= r.params.num_predict:
                self._finish(r, "length", finished)
            elif id(r) not in fed_ahead:
                r.feed = [token]         # (else the step that runs already took it on the device)
        if self._ahead and not any(r in self.running for r in self._ahead[0]):
            self._ahead = None           # everybody ended: what the step ahead makes is for nobody
        return finished
