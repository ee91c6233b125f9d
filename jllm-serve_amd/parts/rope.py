"""Rotary position encoding: the cos/sin table of one RopeSpec.

model/Rope.java:24-38: inverse frequencies in double, ``cos[p, i] = (float)(cos(p * inv[i]) * amp)``;
:122-167 the frequencies (plain ``theta^(-2i/rotary_dim)``, ``linear`` divides by the factor, ``llama3``
blends by wavelength); :190-208 YaRN's ramp between extrapolation and interpolation; :75-85 the amplitude.
The mixers rotate the pair (i, i + rotary_dim/2) by entry i ("half" pairing, model/RopeTable.java:9-18).
"""
from __future__ import annotations

import math

import numpy as np
import torch

from ..config.schema import RopeScaling, RopeSpec
from .base import BuildContext, Part, register_part


def inverse_frequencies(spec: RopeSpec) -> np.ndarray:
    dim = spec.rotary_dim
    half = dim // 2
    i = np.arange(half, dtype=np.float64)
    f = 1.0 / np.power(float(spec.theta), (2.0 * i) / dim)
    s = spec.scaling
    if s.kind == "none":
        return f
    if s.kind == "linear":
        return f / s.factor
    if s.kind == "llama3":
        low_wavelen = s.original_max_positions / s.low_freq_factor
        high_wavelen = s.original_max_positions / s.high_freq_factor
        out = f.copy()
        for k in range(half):
            wavelen = 2 * math.pi / f[k]
            if wavelen < high_wavelen:
                continue
            if wavelen > low_wavelen:
                out[k] = f[k] / s.factor
            else:
                span = s.high_freq_factor - s.low_freq_factor
                smooth = (s.original_max_positions / wavelen - s.low_freq_factor) / span if span > 0 else 0.0
                out[k] = (1 - smooth) * f[k] / s.factor + smooth * f[k]
        return out
    if s.kind == "yarn":
        def correction_dim(rotations):
            return dim * math.log(s.original_max_positions / (rotations * 2 * math.pi)) / (2 * math.log(spec.theta))
        low_dim, high_dim = correction_dim(s.beta_fast), correction_dim(s.beta_slow)
        low = max(math.floor(low_dim) if s.truncate else low_dim, 0)
        high = min(math.ceil(high_dim) if s.truncate else high_dim, dim - 1)
        if low == high:
            high += 0.001
        extra = f
        inter = 1.0 / (s.factor * np.power(float(spec.theta), (2.0 * i) / dim))
        ramp = np.clip((i - low) / (high - low), 0.0, 1.0)
        return inter * ramp + extra * (1 - ramp)
    raise ValueError(f"unknown rope scaling '{s.kind}'")


def amplitude(s: RopeScaling) -> float:
    if s.kind != "yarn":
        return 1.0
    if s.attention_factor > 0:
        return s.attention_factor

    def mscale(scale, m):
        return 1.0 if scale <= 1 else 0.1 * m * math.log(scale) + 1.0
    return mscale(s.factor, s.mscale) / mscale(s.factor, s.mscale_all_dim)


def rope_table(spec: RopeSpec, positions: int):
    """(cos, sin) as float32 arrays [positions, rotary_dim/2], computed in double."""
    inv = inverse_frequencies(spec)
    amp = amplitude(spec.scaling)
    ang = np.arange(positions, dtype=np.float64)[:, None] * inv[None, :]
    return (np.cos(ang) * amp).astype(np.float32), (np.sin(ang) * amp).astype(np.float32)


class RotaryPosition(Part):
    def __init__(self, spec: RopeSpec, build: BuildContext):
        if spec.pairing != "half":
            raise ValueError(f"rotary pairing '{spec.pairing}' is not built (only 'half')")
        self.spec = spec
        cos, sin = rope_table(spec, build.max_positions)
        self.cos = torch.from_numpy(cos).to(build.device)
        self.sin = torch.from_numpy(sin).to(build.device)

    def rotary(self):
        return self.cos, self.sin, self.spec.rotary_dim


register_part("position", "rope", RotaryPosition, replace=True)
