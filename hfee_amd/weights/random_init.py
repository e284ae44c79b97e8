"""Random-weights mode: a model folder, or a model on the device, from a configuration
and a seed.

The reference cannot run without a model file; this stands in for one.  A tensor's values
depend only on (seed, tensor name, element index) and not on where or in which order they
are made: a folder written here on the CPU, the tensors an engine makes on the GPU
(`random_model`, `--random-weights`) and a plain implementation that reads the folder all
hold the same bits (`random_stream.py` on the host, `csrc/random_fill.hip` on the device).
"""
from __future__ import annotations

import json
import os
from typing import Iterable

import torch

from . import random_stream
from .safetensors_io import write_safetensors
from .spec import TensorSpec


def random_tensor(spec: TensorSpec, seed: int, std: float, dtype: torch.dtype,
                  device="cpu") -> torch.Tensor:
    """The tensor that `spec` declares: init ("normal",) is N(0, std), ("one_plus_normal",)
    1 + N(0, std), ("zeros",), ("randint", bound) int32 in [0, bound).  Float64 rounded once to
    float32, then to `dtype`; the same numbers on the CPU and on the GPU."""
    kind = spec.init[0]
    key = random_stream.tensor_key(seed, spec.name)
    shape = tuple(spec.shape)
    count = 1
    for n in shape:
        count *= n
    if kind == "zeros":
        return torch.zeros(shape, dtype=dtype, device=device)
    if kind not in ("normal", "one_plus_normal", "randint"):
        raise ValueError(f"tensor {spec.name}: unknown init {spec.init!r}")
    if torch.device(device).type == "cpu":
        if kind == "randint":
            return torch.from_numpy(random_stream.integers(key, count, spec.init[1])).reshape(shape)
        v = torch.from_numpy(random_stream.normal(key, count, std, plus_one=kind == "one_plus_normal"))
        return v.reshape(shape).to(dtype)
    from ..kernels import ops
    if kind == "randint":
        out = torch.empty(shape, dtype=torch.int32, device=device)
        ops.random_fill(out, key, "integers", bound=spec.init[1])
        return out
    out = torch.empty(shape, dtype=dtype, device=device)
    ops.random_fill(out, key, kind, std=std)
    return out


def random_tensors(specs: Iterable[TensorSpec], seed: int, std: float = 0.02,
                   dtype: torch.dtype = torch.float32, device="cpu", norm_init: str | None = None) -> dict:
    """norm_init overrides the init of 'vector' tensors ("normal" or "one_plus_normal")."""
    out = {}
    for s in specs:
        if s.optional:
            continue
        if norm_init is not None and s.role == "vector":
            s = TensorSpec(s.name, s.shape, s.role, (norm_init,), s.optional)
        out[s.name] = random_tensor(s, seed, std, dtype, device)
    return out


def write_model_folder(path: str, config, seed: int, std: float = 0.02,
                       dtype: torch.dtype = torch.float32, norm_init: str | None = None,
                       device="cpu") -> str:
    """Writes config.json and model.safetensors for `config` with seeded random weights.
    device: where the numbers are made (the same ones either way; a GPU makes the tensors of
    a large model in a fraction of the time)."""
    from ..engine.model import declared_tensors   # the parts say which tensors exist
    os.makedirs(path, exist_ok=True)
    cfg = config.to_dict()
    cfg["torch_dtype"] = {torch.float32: "float32", torch.bfloat16: "bfloat16"}[dtype]
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=1)
    tensors = random_tensors(declared_tensors(config), seed, std, dtype, device, norm_init)
    if torch.device(device).type != "cpu":
        tensors = {name: t.cpu() for name, t in tensors.items()}
    write_safetensors(os.path.join(path, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": seed})
    return path
