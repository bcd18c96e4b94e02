"""Position encodings used inside a mixer."""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, Optional

import torch

from .base import POSITIONS, PositionEncoding

PAIRING = {"interleaved": 0, "half": 1}


@dataclass
class RotaryArgs:
    """What the rotate-and-store kernel needs: angle of pair i at position p is ``p * inv_freq[i]``."""

    inv_freq: torch.Tensor  # float32 [rotary_dim / 2], on the device
    rotary_dim: int
    pairing: int  # 0: pairs (2i, 2i+1); 1: pairs (i, i + rotary_dim/2)
    magnitude: float = 1.0  # a factor on cosines and sines alike (rescaled long contexts)


def step_table(rot: "RotaryArgs", ctx) -> torch.Tensor:
    """Cosines and sines of this step's positions, float32 [n, rotary_dim / 2, 2]: made once per step and shared by
    every layer whose position encoding has the same frequencies and magnitude (``ctx.scratch`` keeps it)."""
    from ..kernels import ops

    key = ("rope_table", rot.inv_freq.data_ptr(), rot.magnitude)
    table = ctx.scratch.get(key)
    if table is None:
        table = ctx.scratch[key] = ops.rope_table(ctx.positions, rot.inv_freq, rot.magnitude)
    return table


def rotary_inverse_frequencies(rotary_dim: int, theta: float, scaling: Optional[Dict[str, Any]]) -> torch.Tensor:
    """Inverse frequencies in 32-bit, with the "llama3" rescaling of long wavelengths when asked for.

    Plain: ``1 / theta^(2i / rotary_dim)``.  llama3: wavelengths beyond ``original / low_freq_factor``
    are stretched by ``factor``, those below ``original / high_freq_factor`` stay, and the band
    between is blended linearly in ``original / wavelength``
    (reference: torchllms/models/networks.py:252-279).
    """
    exponents = torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim
    inv_freq = 1.0 / (theta ** exponents)
    if not scaling or scaling.get("rope_type", "default") == "default":
        return inv_freq
    if scaling["rope_type"] == "yarn":
        return yarn_inverse_frequencies(rotary_dim, theta, scaling)
    if scaling["rope_type"] != "llama3":
        raise ValueError(f"Unknown RoPE type: {scaling['rope_type']}")
    factor = scaling["factor"]
    low = scaling["low_freq_factor"]
    high = scaling["high_freq_factor"]
    original = scaling["original_max_position_embeddings"]
    wavelength = 2 * math.pi / inv_freq
    long_edge = original / low
    short_edge = original / high
    stretched = torch.where(wavelength > long_edge, inv_freq / factor, inv_freq)
    blend = (original / wavelength - low) / (high - low)
    blended = (1 - blend) * stretched / factor + blend * stretched
    in_band = (wavelength >= short_edge) & (wavelength <= long_edge)
    return torch.where(in_band, blended, stretched)


def yarn_inverse_frequencies(rotary_dim: int, theta: float, scaling: Dict[str, Any]) -> torch.Tensor:
    """YaRN: pair i turns ``dims ln(original / (2 pi t)) / (2 ln theta)`` = i times within ``original`` positions when
    that expression is taken at t; between the pairs that turn ``fast`` and ``slow`` times (floor and ceiling, kept
    inside 0 .. dims - 1) a ramp rises from 0 to 1, and the frequency is ``f / factor * ramp + f * (1 - ramp)``.
    Worked out in 64-bit, rounded once to 32-bit."""
    factor, original = float(scaling["factor"]), float(scaling["original"])
    i = torch.arange(rotary_dim // 2, dtype=torch.float64)
    f = float(theta) ** (-2.0 * i / rotary_dim)

    def pair_that_turns(t: float) -> float:
        return rotary_dim * math.log(original / (2 * math.pi * t)) / (2 * math.log(float(theta)))

    lo = max(math.floor(pair_that_turns(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_that_turns(float(scaling["slow"]))), rotary_dim - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return (f / factor * ramp + f * (1.0 - ramp)).to(torch.float32)


def yarn_magnitude(scaling: Optional[Dict[str, Any]]) -> float:
    """The factor ``0.1 ln(factor) + 1`` on cosines and sines of a YaRN-scaled rotation (1 without one)."""
    if not scaling or scaling.get("rope_type") != "yarn":
        return 1.0
    return 0.1 * math.log(float(scaling["factor"])) + 1.0


#: inverse frequencies on a device, by (device, values)
_DEVICE_FREQUENCIES: Dict[Any, torch.Tensor] = {}


@POSITIONS.register("rope")
class RotaryEmbedding(PositionEncoding):
    """Rotation of (query, key) channel pairs by ``position * inv_freq`` in 32-bit
    (reference: torchllms/models/networks.py:284-352 builds a cos/sin table and rotates
    interleaved pairs over all positions; here the cosines and sines of a step's positions are
    formed from the same 32-bit product, once per step).  Instances with equal frequencies share
    one device tensor, so that the layers of a model also share the step's table.  ``scaling`` with ``rope_type``
    "yarn" (``factor``, ``original``, ``fast``, ``slow``) rescales the slow pairs and multiplies cosines and sines by
    ``0.1 ln(factor) + 1``; ``precise``: the unscaled frequencies are worked out in 64-bit and rounded once."""

    def __init__(self, head_dim: int, rotary_dim: int, theta: float, scaling: Optional[Dict[str, Any]], pairing: str = "interleaved",
                 precise: bool = False):
        if rotary_dim % 2 or rotary_dim > head_dim:
            raise ValueError(f"rotary_dim={rotary_dim} must be even and at most head_dim={head_dim}")
        if pairing not in PAIRING:
            raise ValueError(f"pairing must be one of {sorted(PAIRING)}")
        self.head_dim = head_dim
        self.rotary_dim = rotary_dim
        self.theta = float(theta)
        self.scaling = scaling
        self.pairing = pairing
        self.inv_freq = rotary_inverse_frequencies(rotary_dim, self.theta, scaling)
        if precise and not scaling:
            self.inv_freq = (self.theta ** (-torch.arange(0, rotary_dim, 2, dtype=torch.float64) / rotary_dim)).to(torch.float32)
        self.magnitude = yarn_magnitude(scaling)
        self._device_args: Optional[RotaryArgs] = None

    def to(self, device) -> None:
        key = (str(torch.device(device)), self.inv_freq.numpy().tobytes())
        freqs = _DEVICE_FREQUENCIES.get(key)
        if freqs is None:
            freqs = _DEVICE_FREQUENCIES[key] = self.inv_freq.to(device).contiguous()
        self._device_args = RotaryArgs(freqs, self.rotary_dim, PAIRING[self.pairing], self.magnitude)

    def rotary_args(self) -> Optional[RotaryArgs]:
        return self._device_args


@POSITIONS.register("none")
class NoPosition(PositionEncoding):
    """Queries and keys pass unrotated."""

    def __init__(self, **_ignored):
        pass

    def to(self, device) -> None:
        pass
