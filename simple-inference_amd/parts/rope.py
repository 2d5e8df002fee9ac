"""Rotary position encoding with llama3 frequency scaling.

Frequencies (reference: ``ops/rope.py:95-118``): ``inv_freq_i = 1 / theta^(2i/d)``
for ``i = 0 .. d/2-1`` in float32.  With ``rope_type == "llama3"`` each frequency
is rescaled by its wavelength (reference: ``ops/rope.py:120-155``): unchanged below
``original/high_freq_factor``, divided by ``factor`` above
``original/low_freq_factor``, interpolated in between; that loop runs in Python
floats on the float32 values, as the reference's does.  Angles are
``float32(position) * inv_freq`` and the cos/sin tables stay float32.  The
rotation itself pairs element ``i`` with ``i + d/2`` (reference:
``ops/rope.py:167-182``) and is applied by the kernel that also writes the cache.

Two further forms, each a parameter: ``scaling["rope_type"] == "yarn"`` stretches the frequencies by a ramp over the
pair index and raises the amplitude of both tables (see ``yarn_inv_freq``); ``pairing == "interleaved"`` says that a
consumer pairs element ``2i`` with ``2i + 1`` (the tables are the same; the kernel that rotates reads the flag).
"""

from __future__ import annotations

import math

import torch

from .registry import register_position_encoding


def rotary_inv_freq(rotary_dim: int, theta: float, scaling=None) -> torch.Tensor:
    idx = torch.arange(0, rotary_dim, 2, dtype=torch.float32)
    inv_freq = 1.0 / (theta ** (idx / rotary_dim))
    if scaling is None or scaling.get("rope_type", "default") != "llama3":
        return inv_freq
    factor = float(scaling["factor"])
    low = float(scaling["low_freq_factor"])
    high = float(scaling["high_freq_factor"])
    original = float(scaling["original_max_position_embeddings"])
    low_wavelen = original / low
    high_wavelen = original / high
    scaled = []
    for f in inv_freq.tolist():
        wavelen = 2 * math.pi / f
        if wavelen < high_wavelen:
            scaled.append(f)
        elif wavelen > low_wavelen:
            scaled.append(f / factor)
        else:
            smooth = (original / wavelen - low) / (high - low)
            scaled.append((1 - smooth) * f / factor + smooth * f)
    return torch.tensor(scaled, dtype=torch.float32)


def yarn_inv_freq(rotary_dim: int, theta: float, scaling) -> tuple:
    """Frequencies and table amplitude of the ramp form.  With ``turn(t) = d * ln(original / (2 pi t)) / (2 ln theta)``
    (the pair index whose wave makes ``t`` turns over ``original`` positions), ``lo = max(floor(turn(fast)), 0)``,
    ``hi = min(ceil(turn(slow)), d - 1)`` and ``ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``, pair ``i``
    turns at ``f_i / factor * ramp_i + f_i * (1 - ramp_i)``; cos and sin are multiplied by ``0.1 ln(factor) + 1``."""
    idx = torch.arange(0, rotary_dim, 2, dtype=torch.float64)
    f = theta ** (-idx / rotary_dim)
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turn(t):
        return rotary_dim * math.log(original / (2 * math.pi * t)) / (2 * math.log(theta))

    lo = max(math.floor(turn(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn(float(scaling["slow"]))), rotary_dim - 1)
    ramp = ((torch.arange(rotary_dim // 2, dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


@register_position_encoding("rope")
class RotaryEncoding:
    """params: rotary_dim, theta, scaling (dict or None), and optionally pairing ("half", the default, or
    "interleaved") and angles ("float32", the default: positions times frequencies as float32 products, or "float64":
    frequencies and angles in float64 on the host, the tables rounded once)."""

    def __init__(self, params, env):
        self.rotary_dim = int(params["rotary_dim"])
        if self.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even, got {self.rotary_dim}")
        self.theta = float(params["theta"])
        self.scaling = params.get("scaling")
        self.pairing = str(params.get("pairing", "half"))
        if self.pairing not in ("half", "interleaved"):
            raise ValueError(f"pairing must be 'half' or 'interleaved', got {self.pairing!r}")
        self.angles = str(params.get("angles", "float32"))
        if self.angles not in ("float32", "float64"):
            raise ValueError(f"angles must be 'float32' or 'float64', got {self.angles!r}")
        self.max_positions = int(env.max_positions)
        self.device = env.device
        self._tables = None

    def weight_specs(self):
        return {}

    def bind(self, tensors):
        pass

    def tables(self):
        """(cos, sin), each float32 ``[max_positions, rotary_dim/2]``, on the device."""
        if self._tables is None:
            amplitude = 1.0
            if self.scaling is not None and self.scaling.get("rope_type") == "yarn":
                inv_freq, amplitude = yarn_inv_freq(self.rotary_dim, self.theta, self.scaling)
            elif self.angles == "float64" and self.scaling is None:
                inv_freq = self.theta ** (-torch.arange(0, self.rotary_dim, 2, dtype=torch.float64) / self.rotary_dim)
            else:
                inv_freq = rotary_inv_freq(self.rotary_dim, self.theta, self.scaling)
            # the ramp form's angles are taken in float64 on the host and the tables rounded once
            pos = torch.arange(self.max_positions, dtype=inv_freq.dtype)
            angles = torch.outer(pos, inv_freq)
            cos, sin = angles.cos(), angles.sin()
            if amplitude != 1.0:
                cos, sin = cos * amplitude, sin * amplitude
            cos, sin = cos.float(), sin.float()
            self._tables = (cos.to(self.device).contiguous(), sin.to(self.device).contiguous())
        return self._tables


@register_position_encoding("none")
class NoPositionEncoding:
    rotary_dim = 0

    def __init__(self, params, env):
        pass

    def weight_specs(self):
        return {}

    def bind(self, tensors):
        pass

    def tables(self):
        return None, None
