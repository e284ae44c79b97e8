"""What a part says about each of its tensors."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class TensorSpec:
    name: str            # full name in the checkpoint
    shape: tuple
    role: str = "matrix"  # "matrix": cast to the engine's dtype;
                          # "vector": cast likewise unless stored in 32-bit (then kept);
                          # "table": integers, kept as int32
    init: tuple = ("normal",)   # random-weights mode: ("normal",) | ("one_plus_normal",) |
                                # ("zeros",) | ("randint", high)
    optional: bool = False
