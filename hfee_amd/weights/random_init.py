"""Random-weights mode: a model folder from a configuration and a seed.

The reference cannot run without a model file; this stands in for one.  Each
tensor's values depend only on (seed, tensor name), not on the order in which
tensors are made, so a folder written here, the engine and a plain
implementation that all start from the same seed hold the same numbers.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Iterable

import numpy as np
import torch

from .safetensors_io import write_safetensors
from .spec import TensorSpec


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    return int.from_bytes(digest[:8], "little")


def random_tensor(spec: TensorSpec, seed: int, std: float, dtype: torch.dtype,
                  device="cpu") -> torch.Tensor:
    kind = spec.init[0]
    if torch.device(device).type == "cpu":
        rng = np.random.Generator(np.random.Philox(key=_tensor_seed(seed, spec.name)))
        if kind == "randint":
            return torch.from_numpy(rng.integers(0, spec.init[1], size=spec.shape, dtype=np.int32))
        if kind == "zeros":
            return torch.zeros(spec.shape, dtype=dtype)
        v = torch.from_numpy(rng.standard_normal(size=spec.shape, dtype=np.float32)) * std
    else:
        g = torch.Generator(device=device)
        g.manual_seed(_tensor_seed(seed, spec.name) & ((1 << 63) - 1))
        if kind == "randint":
            return torch.randint(0, spec.init[1], spec.shape, generator=g, device=device, dtype=torch.int32)
        if kind == "zeros":
            return torch.zeros(spec.shape, dtype=dtype, device=device)
        v = torch.empty(spec.shape, dtype=dtype, device=device).normal_(0.0, std, generator=g)
        if kind == "one_plus_normal":
            v += 1
        return v
    if kind == "one_plus_normal":
        v = v + 1
    elif kind != "normal":
        raise ValueError(f"tensor {spec.name}: unknown init {spec.init!r}")
    return v.to(dtype)


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
                       dtype: torch.dtype = torch.float32, norm_init: str | None = None) -> str:
    """Writes config.json and model.safetensors for `config` with seeded random weights."""
    from ..engine.model import declared_tensors   # the parts say which tensors exist
    os.makedirs(path, exist_ok=True)
    cfg = config.to_dict()
    cfg["torch_dtype"] = {torch.float32: "float32", torch.bfloat16: "bfloat16"}[dtype]
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=1)
    tensors = random_tensors(declared_tensors(config), seed, std, dtype, "cpu", norm_init)
    write_safetensors(os.path.join(path, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": seed})
    return path
