"""Position encodings.  Reference: somi_inference/models/qwen2.py:65-113."""

from __future__ import annotations

import math

import torch

from .base import Fetch, PositionEncoding, Runtime


def scaled_frequencies(inv_freq: torch.Tensor, factor: float, low: float, high: float, original: int) -> torch.Tensor:
    """Frequencies rescaled by wavelength l = 2 pi / f against a context of ``original`` positions: f stays where
    l < original / high, becomes f / factor where l > original / low, and in between is the blend
    (1 - s) f / factor + s f with s = (original / l - low) / (high - low).  Computed in double precision, rounded once."""
    f = inv_freq.to(torch.float64)
    wavelength = 2.0 * math.pi / f
    s = ((original / wavelength - low) / (high - low)).clamp(0.0, 1.0)
    blended = (1.0 - s) * f / factor + s * f
    out = torch.where(wavelength < original / high, f, torch.where(wavelength > original / low, f / factor, blended))
    return out.to(torch.float32)


def ramped_frequencies(inv_freq: torch.Tensor, theta: float, rotary_dim: int, factor: float, original: int, fast: float,
                       slow: float) -> torch.Tensor:
    """Frequencies rescaled by a ramp over the channel index: with ``at(turns) = rotary_dim * ln(original / (2 pi
    turns)) / (2 ln theta)``, the index of the channel that makes ``turns`` turns over ``original`` positions, ``lo =
    max(floor(at(fast)), 0)``, ``hi = min(ceil(at(slow)), rotary_dim - 1)`` and ``r_i = clamp((i - lo) / max(hi - lo,
    0.001), 0, 1)``, channel i gets ``f_i / factor * r_i + f_i * (1 - r_i)``: fast channels stay, slow ones are
    stretched by ``factor``.  Computed in double precision, rounded once."""
    f = inv_freq.to(torch.float64)

    def at(turns: float) -> float:
        return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    lo = max(math.floor(at(fast)), 0)
    hi = min(math.ceil(at(slow)), rotary_dim - 1)
    index = torch.arange(f.numel(), dtype=torch.float64)
    ramp = ((index - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return (f / factor * ramp + f * (1.0 - ramp)).to(torch.float32)


class RotaryPosition(PositionEncoding):
    """Rotary embedding: channel pairs of a head are turned by the angle p * theta^(-2j/rotary_dim)
    (qwen2.py:76-79).  ``pairing`` "half" pairs element i with i + rotary_dim/2 (rotate-half, qwen2.py:95-99);
    "neighbours" pairs element 2i with 2i + 1.  ``scaling`` (factor, low, high, original) rescales the frequencies by
    their wavelength, see :func:`scaled_frequencies`; ``scaling`` (factor, original, fast, slow) by a ramp over the channel
    index, see :func:`ramped_frequencies`, and then cosines and sines are also multiplied by ``amplitude`` = 0.1 ln(factor)
    + 1 (kernels that take an amplitude read it from the part).  Only the first ``rotary_dim`` channels of a head turn.  No
    table over positions is kept (the reference bounds the sequence length by its table, qwen2.py:72-81): the angle is
    computed from the position in float32 by the kernel that also writes k into its cache page."""
    graph_safe = True

    PAIRINGS = ("half", "neighbours")

    def __init__(self, prefix: str, head_dim: int, theta: float, rotary_dim: int | None = None,
                 pairing: str = "half", scaling: dict | None = None) -> None:
        super().__init__(prefix)
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        if pairing not in self.PAIRINGS:
            raise ValueError(f"pairing must be one of {self.PAIRINGS}, got {pairing!r}")
        self.pairing = pairing
        self.scaling = self.ramp = None
        self.amplitude = 1.0
        if scaling and "fast" in scaling:
            self.ramp = {"factor": float(scaling["factor"]), "original": int(scaling["original"]),
                         "fast": float(scaling["fast"]), "slow": float(scaling["slow"])}
            if min(self.ramp["factor"], self.ramp["fast"], self.ramp["slow"]) <= 0.0 or self.ramp["original"] < 1 or self.theta <= 1.0:
                raise ValueError(f"a frequency ramp needs factor, fast, slow > 0, original >= 1 and theta > 1, got {scaling}")
            self.amplitude = 0.1 * math.log(self.ramp["factor"]) + 1.0
        elif scaling:
            self.scaling = {"factor": float(scaling["factor"]), "low": float(scaling["low"]),
                            "high": float(scaling["high"]), "original": int(scaling["original"])}
            if self.scaling["high"] == self.scaling["low"] or self.scaling["factor"] <= 0.0:
                raise ValueError(f"frequency scaling needs high != low and factor > 0, got {scaling}")
        self.inv_freq: torch.Tensor | None = None

    def frequencies(self) -> torch.Tensor:
        """[rotary_dim / 2] float32 on the host."""
        exponents = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64) / self.rotary_dim
        inv_freq = 1.0 / (self.theta ** exponents)
        if self.ramp:
            return ramped_frequencies(inv_freq, self.theta, self.rotary_dim, **self.ramp)
        inv_freq = inv_freq.to(torch.float32)
        return scaled_frequencies(inv_freq, **self.scaling) if self.scaling else inv_freq

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        if self.scaling is None and self.ramp is None and self.pairing == "half":
            # the reference's own arithmetic (float32 powers), bit for bit
            exponents = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
            self.inv_freq = (1.0 / (self.theta ** exponents)).to(runtime.device)
        else:
            self.inv_freq = self.frequencies().to(runtime.device)

    def rotation_table(self) -> tuple[torch.Tensor, int]:
        return self.inv_freq, self.rotary_dim


class NoPosition(PositionEncoding):
    """No position information (attention is then invariant to a shift of all positions)."""
    graph_safe = True

    def __init__(self, prefix: str = "") -> None:
        super().__init__(prefix)
