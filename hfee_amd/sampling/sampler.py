"""The sampler: packs each row's options for the device kernel and reads the
chosen ids back.

One random stream per request (/root/reference/internal/llm/sampler.go:41-47,
/root/reference/internal/llm/runner.go:223): the uniform number of a request's k-th
draw is splitmix64(seed, k), so a request's tokens do not depend on what else is
sampled in the same call.  `uniform()` is the host twin of the kernel's generator.
"""
from __future__ import annotations

import struct
from dataclasses import dataclass

import numpy as np
import torch

from ..kernels import ops
from .params import SamplingParams

_MASK = (1 << 64) - 1


def uniform(seed: int, draw: int) -> float:
    """The number in [0, 1) that the kernel uses for draw number `draw` of stream `seed`."""
    z = (seed + (draw + 1) * 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z ^= z >> 31
    return (z >> 11) * (1.0 / 9007199254740992.0)


@dataclass
class SampleRow:
    params: SamplingParams
    seed: int             # resolved (non-negative) seed of the request
    draw: int             # how many tokens the request has sampled so far
    history: list         # prompt + generated ids (for the repeat penalty)
    logits_row: int       # row of the logits tensor


def _f2i(x: float) -> int:
    return struct.unpack("<i", struct.pack("<f", float(x)))[0]


def pack_rows(rows, one_more: bool = False) -> tuple:
    """rows -> ([n, 12] int32 parameter array, flat int32 history).  one_more: every row's
    history has one newer id that is not in `history` (the kernel gets it on the device):
    the window of the repeat penalty then takes one id fewer from here."""
    params = np.zeros((len(rows), 12), dtype=np.int32)
    hist = []
    for i, r in enumerate(rows):
        p = r.params
        recent = []
        if p.repeat_penalty != 1 and p.repeat_last_n != 0:
            recent = list(r.history)
            if p.repeat_last_n > 0:
                keep = p.repeat_last_n - (1 if one_more else 0)
                recent = recent[-keep:] if keep > 0 else []
        seed, draw = r.seed & _MASK, r.draw & _MASK
        # (a window of 0 ids switches the penalty off: the kernel sees a penalty of 1)
        words = [_f2i(p.temperature), int(p.top_k), _f2i(p.top_p), _f2i(p.min_p),
                 _f2i(p.repeat_penalty if p.repeat_last_n != 0 else 1.0),
                 len(hist), len(recent)]
        params[i, :7] = words
        params[i, 7:11] = np.array([seed & 0xffffffff, seed >> 32, draw & 0xffffffff, draw >> 32],
                                   dtype=np.uint32).view(np.int32)
        params[i, 11] = r.logits_row
        hist += recent
    return params, np.asarray(hist if hist else [0], dtype=np.int32)


class Sampler:
    def __init__(self, vocab: int, device, max_rows: int):
        self.vocab, self.device, self.max_rows = vocab, device, max_rows
        self._out = torch.empty(max_rows, dtype=torch.int32, device=device)
        self._latest = self._out
        # two places for the ids on the host, taken in turn: a caller may launch the next
        # sampling before it has collected this one
        self._slots = [(torch.empty(max_rows, dtype=torch.int32, pin_memory=True), torch.cuda.Event())
                       for _ in range(2)]
        self._turn = 0
        self._scratch = None
        self._stage = [None, None]          # pinned buffers for the rows' options, taken in turn with _slots
        self._options = None                # the same on the device
        # for the argmax over several workgroups a row
        self._partial = torch.empty(max_rows * ops.ARGMAX_PARTS * 2, dtype=torch.float32, device=device)
        self._counters = torch.zeros(max_rows, dtype=torch.int32, device=device)

    @property
    def device_ids(self) -> torch.Tensor:
        """The ids of the latest launch(), on the device, in the order of its rows: a step that
        is launched before they are collected can take its tokens from here."""
        return self._latest

    @staticmethod
    def needs_history(params: SamplingParams) -> bool:
        """Whether sampling with these options reads the request's earlier tokens."""
        return params.repeat_penalty != 1 and params.repeat_last_n != 0

    def sample(self, logits: torch.Tensor, rows) -> list:
        """logits: float32 [*, vocab] on the device (changed in place by the repeat
        penalty, as the reference changes them).  Returns one id per row."""
        return self.collect(self.launch(logits, rows))

    def launch(self, logits: torch.Tensor, rows, out=None, latest=None):
        """Starts the sampling of `rows` and returns what collect() takes: the caller may
        do other work on the host between the two while the GPU runs.  out: an int32
        tensor on the device that takes the ids in place of the sampler's own (the place
        where the engine's next step looks for its tokens, say).  latest: an int32 tensor
        on the device with one id a row that is newer than the rows' histories (the ids of
        the sampling before, when this one is launched before they were collected): the
        repeat penalty counts it in.  It may be the tensor that `out` names."""
        n = len(rows)
        if n == 0:
            return (0, 0)
        dst = self._out if out is None or out.numel() < n else out
        self._latest = dst
        if n > self.max_rows:
            raise ValueError(f"{n} rows to sample, the sampler was made for {self.max_rows}")
        plain_greedy = all(r.params.temperature <= 0 and not self.needs_history(r.params) for r in rows)
        if plain_greedy and [r.logits_row for r in rows] == list(range(logits.shape[0])):
            ops.argmax(dst, logits, self._partial, self._counters)
        else:
            params, hist = pack_rows(rows, one_more=latest is not None)
            if self._scratch is None:
                self._scratch = torch.empty((self.max_rows, self.vocab), dtype=torch.float32, device=self.device)
            dparams, dhist = self._send(params, hist)
            ops.sample(dst, logits, dparams, dhist, self._scratch,
                       latest if any(self.needs_history(r.params) for r in rows) else None)
        slot = self._turn
        self._turn ^= 1
        host, done = self._slots[slot]
        host[:n].copy_(dst[:n], non_blocking=True)
        done.record()
        return (n, slot)

    def _send(self, params: np.ndarray, hist: np.ndarray):
        """The rows' options and recent ids to the device through pinned memory, without
        making the host wait for the stream (a copy from pageable memory would wait for
        everything queued before it: the whole step)."""
        need = params.size + hist.size
        stage = self._stage[self._turn]
        if stage is None or stage[0].numel() < need:
            cap = max(2 * need, 12 * self.max_rows + 4096)
            stage = self._stage[self._turn] = (torch.empty(cap, dtype=torch.int32, pin_memory=True), torch.cuda.Event())
        pinned, sent = stage
        sent.synchronize()                  # the copy that used this buffer two launches ago
        if self._options is None or self._options.numel() < need:
            self._options = torch.empty(max(2 * need, 12 * self.max_rows + 4096), dtype=torch.int32, device=self.device)
        host = pinned.numpy()
        host[:params.size] = params.reshape(-1)
        host[params.size:need] = hist
        self._options[:need].copy_(pinned[:need], non_blocking=True)
        sent.record()
        return self._options[:params.size].view(params.shape), self._options[params.size:need]

    def collect(self, pending) -> list:
        """Waits for the ids of a launch() (the latest one or the one before it)."""
        n, slot = pending
        if n == 0:
            return []
        host, done = self._slots[slot]
        done.synchronize()
        return host[:n].tolist()
