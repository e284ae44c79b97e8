"""Rotary position encoding.

Frequencies as the reference builds them in float64
(/root/reference/internal/llm/model.go:150-158): inv_freq[i] = 1 / theta^(2i/dim),
then a per-dimension divisor.  The reference reads the divisors of llama 3.1 models
from a tensor; here they come from the configuration's llama3 rule (wavelengths
shorter than N0/high keep their frequency, longer than N0/low are divided by
`factor`, in between the two are blended linearly in N0/wavelength).

The reference takes sin and cos of the float64 angle position * inv_freq at every
use (/root/reference/internal/llm/forward.go:186).  Here a table [positions, dim/2]
of cos and sin is made once from those float64 angles and rounded to float32, so
large positions lose nothing to a float32 angle.
"""
from __future__ import annotations

import math

import numpy as np
import torch

from ..config.specs import PositionSpec
from .base import Part, register_position

PAIRINGS = {"half": 0, "interleaved": 1}


def rope_frequencies(rotary_dim: int, theta: float, scaling=None) -> np.ndarray:
    half = rotary_dim // 2
    inv = np.array([1.0 / math.pow(theta, (2 * i) / rotary_dim) for i in range(half)], dtype=np.float64)
    if scaling is None:
        return inv
    kind, factor, low, high, original = scaling
    if kind != "llama3":
        raise ValueError(f"unknown rope scaling {kind!r}")
    out = inv.copy()
    for i, f in enumerate(inv):
        wavelength = 2 * math.pi / f
        if wavelength < original / high:
            continue
        if wavelength > original / low:
            out[i] = f / factor
        else:
            smooth = (original / wavelength - low) / (high - low)
            out[i] = (1 - smooth) * f / factor + smooth * f
    return out


@register_position("rope")
class Rotary(Part):
    def __init__(self, spec: PositionSpec):
        self.head_dim = spec.get("head_dim")
        self.rotary_dim = spec.get("rotary_dim", self.head_dim)
        self.theta = float(spec.get("theta"))
        self.scaling = spec.get("scaling")
        pairing = spec.get("pairing", "half")
        if pairing not in PAIRINGS:
            raise ValueError(f"rotary pairing must be 'half' or 'interleaved', got {pairing!r}")
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        self.pairing = PAIRINGS[pairing]
        self.inv_freq = rope_frequencies(self.rotary_dim, self.theta, self.scaling)
        self.cos = self.sin = None

    def signature(self):
        """What two mixers must share to read one another's rotated keys."""
        return ("rope", self.rotary_dim, self.theta, self.scaling)

    def prepare(self, num_positions: int, device) -> None:
        if self.cos is not None and self.cos.shape[0] >= num_positions and self.cos.device == torch.device(device):
            return
        angles = np.arange(num_positions, dtype=np.float64)[:, None] * self.inv_freq[None, :]
        self.cos = torch.from_numpy(np.cos(angles).astype(np.float32)).to(device)
        self.sin = torch.from_numpy(np.sin(angles).astype(np.float32)).to(device)
