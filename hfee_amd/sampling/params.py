"""Sampling options, with the reference's names, meanings and defaults
(/root/reference/internal/llm/sampler.go:10-34)."""
from __future__ import annotations

import os
from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 0.8      # <= 0: greedy
    top_k: int = 40               # <= 0: off
    top_p: float = 0.9            # outside (0, 1): off
    min_p: float = 0.0            # 0: off
    repeat_penalty: float = 1.1   # 1: off
    repeat_last_n: int = 64       # 0: off, < 0: the whole history
    seed: int = -1                # < 0: a random seed
    num_predict: int = -1         # most new tokens, < 0: no limit but the context
    stop: tuple = ()              # stop strings (need a tokenizer)
    ignore_eos: bool = False      # keep generating past end-of-sequence ids (benchmarks)

    def resolved_seed(self) -> int:
        if self.seed is not None and self.seed >= 0:
            return int(self.seed) & ((1 << 64) - 1)
        return int.from_bytes(os.urandom(8), "little")

    @staticmethod
    def greedy(num_predict: int = -1, **kw) -> "SamplingParams":
        return SamplingParams(temperature=0.0, top_k=0, top_p=1.0, repeat_penalty=1.0,
                              num_predict=num_predict, **kw)
