"""Binding a checkpoint's tensors to the names a model's parts declare.

The reference binds tensors by name, remembers the first missing one and fails
after all binds (/root/reference/internal/llm/model.go:162-174, 143-145), and
checks the rank of matrices (/root/reference/internal/llm/model.go:188-191).
Here every problem is gathered first: one error lists missing tensors, unexpected
tensors and wrong shapes together.
"""
from __future__ import annotations

from typing import Iterable

import torch

from .safetensors_io import Checkpoint
from .spec import TensorSpec


class WeightsError(ValueError):
    def __init__(self, where: str, missing, unexpected, wrong_shapes, other=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shapes = list(wrong_shapes)
        self.other = list(other)
        lines = [f"{where}: the tensors do not match the model"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shapes:
            lines.append(f"  wrong shapes ({len(self.wrong_shapes)}): " + "; ".join(
                f"{n}: expected {list(e)}, got {list(g)}" for n, e, g in self.wrong_shapes))
        for o in self.other:
            lines.append("  " + o)
        super().__init__("\n".join(lines))


def engine_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name in (torch.float32, torch.bfloat16):
            return name
    table = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
             "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32}
    if name in table:
        return table[name]
    raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {name!r}")


def convert_for_engine(t: torch.Tensor, role: str, dtype: torch.dtype) -> torch.Tensor:
    """Storage rule: weights are kept in the engine's dtype; integer tables become
    int32; a vector stored in 32-bit stays in 32-bit."""
    if role == "table":
        return t.to(torch.int32)
    if not t.is_floating_point():
        raise ValueError(f"expected floating-point data, got {t.dtype}")
    if role == "vector" and t.dtype == torch.float32:
        return t
    return t.to(dtype)


def check_tensors(where: str, available: dict, specs: Iterable[TensorSpec], ignored_suffixes=()):
    """available: name -> shape.  Raises WeightsError listing every mismatch."""
    specs = list(specs)
    wanted = {s.name: s for s in specs}
    missing = [s.name for s in specs if not s.optional and s.name not in available]
    unexpected = [n for n in available if n not in wanted
                  and not any(n.endswith(suf) for suf in ignored_suffixes)]
    wrong = [(s.name, s.shape, tuple(available[s.name])) for s in specs
             if s.name in available and tuple(available[s.name]) != tuple(s.shape)]
    if missing or unexpected or wrong:
        raise WeightsError(where, missing, unexpected, wrong)


def load_tensors(model_dir: str, specs: Iterable[TensorSpec], dtype: torch.dtype,
                 device, ignored_suffixes=()) -> dict:
    """Reads every declared tensor from the folder's safetensors onto the device."""
    specs = list(specs)
    ckpt = Checkpoint(model_dir)
    available = {n: ckpt.entry(n).shape for n in ckpt.names()}
    check_tensors(model_dir, available, specs, ignored_suffixes)
    bad_types = []
    out = {}
    for s in specs:
        if s.name not in available:
            continue
        t = ckpt.tensor(s.name)
        try:
            out[s.name] = convert_for_engine(t, s.role, dtype).to(device, copy=True)
        except ValueError as e:
            bad_types.append(f"tensor {s.name}: {e}")
    if bad_types:
        raise WeightsError(model_dir, (), (), (), bad_types)
    return out


def bind_tensors(tensors: dict, specs: Iterable[TensorSpec], dtype: torch.dtype, device,
                 where: str = "given tensors", ignored_suffixes=()) -> dict:
    """The same binding for tensors that are already in memory (random weights made
    on the device, tests)."""
    specs = list(specs)
    check_tensors(where, {n: tuple(t.shape) for n, t in tensors.items()}, specs, ignored_suffixes)
    return {s.name: convert_for_engine(tensors[s.name], s.role, dtype).to(device)
            for s in specs if s.name in tensors}
