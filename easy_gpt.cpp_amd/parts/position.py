"""Position encodings.

Rotary, half-split pairing as in the reference (/root/reference/src/ops.cpp:154-179
for the frequency table, :392-458 for the rotation): for i in [0, d/2):
inv_freq_i = 1 / theta^(2i/d) (float32), angle = float(position) * inv_freq_i,
(x_i, x_{i+d/2}) <- (x_i cos - x_{i+d/2} sin, x_i sin + x_{i+d/2} cos); applied to
queries and keys, never to values.
"""
from __future__ import annotations

import math

import torch

from .. import kernels
from .base import PositionEncoding, register_part


class RotaryHalfSplit(PositionEncoding):
    """Rotation of the first `rotary_dim` features of each head (all of them by default)."""

    graph_safe = True
    pairing = "half"        # which places turn together: (i, i + rotary_dim / 2)

    def __init__(self, prefix: str, head_dim: int, theta: float, rotary_dim: int | None = None, scaling=None,
                 exact_frequencies: bool = False, **_):
        """scaling {rule: 'wavelength', factor, low, high, original} stretches the slow frequencies
        (`stretch_by_wavelength`).  exact_frequencies: f_i = theta^(-2i / rotary_dim) is computed in float64 and
        rounded once (implied by a scaling); otherwise in float32 steps, as the reference does."""
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and in (0, head_dim={self.head_dim}]")
        if not self.theta > 0:
            raise ValueError("rope theta must be positive")
        self.scaling = dict(scaling) if scaling else None
        if self.scaling is not None and self.scaling.get("rule") != "wavelength":
            raise ValueError(f"this rotation stretches frequencies by the rule 'wavelength', not {self.scaling.get('rule')!r}")
        self.exact = bool(exact_frequencies) or self.scaling is not None
        self._inv_freq: dict = {}

    def inv_freq_host(self) -> torch.Tensor:
        d = self.rotary_dim
        if self.exact:
            i = torch.arange(0, d // 2, dtype=torch.float64)
            f = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * i / float(d))
            if self.scaling is not None:
                f = stretch_by_wavelength(f, **{k: v for k, v in self.scaling.items() if k != "rule"})
            return f.to(torch.float32)
        i = torch.arange(0, d // 2, dtype=torch.float32)
        # float32 pow of a float32 base, then a float32 reciprocal, as in ops.cpp:172-175
        freq = torch.pow(torch.tensor(self.theta, dtype=torch.float32), (2.0 * i) / float(d))
        return (1.0 / freq).to(torch.float32)

    def rotary(self, device):
        key = str(device)
        if key not in self._inv_freq:
            self._inv_freq[key] = self.inv_freq_host().to(device)
        return self._inv_freq[key], self.rotary_dim

    def table(self, ctx):
        """The step's cosines and sines [T, rotary_dim / 2, 2], computed by the first layer that asks and
        shared by the others (the angles depend on the positions only); None if the backend has no such kernel."""
        sc = tuple(sorted(self.scaling.items())) if self.scaling else None
        key = ("rope_table", self.theta, self.rotary_dim, sc, self.exact)
        if key not in ctx.shared:
            inv_freq, _ = self.rotary(ctx.positions.device)
            ctx.shared[key] = kernels.backend().rope_table(ctx.positions, inv_freq)
        return ctx.shared[key]


def stretch_by_wavelength(f: torch.Tensor, factor: float, low: float, high: float, original: float) -> torch.Tensor:
    """Frequencies f (float64) with the slow ones stretched for contexts beyond `original` tokens: with the wavelength
    l = 2 pi / f, f stays where l < original / high, becomes f / factor where l > original / low, and in between is
    (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""
    factor, low, high, original = float(factor), float(low), float(high), float(original)
    if not (factor > 0 and original > 0 and high > low > 0):
        raise ValueError("stretching by wavelength needs positive factor and original and high > low > 0")
    wavelength = 2.0 * math.pi / f
    s = (original / wavelength - low) / (high - low)
    mixed = (1.0 - s) * f / factor + s * f
    return torch.where(wavelength < original / high, f, torch.where(wavelength > original / low, f / factor, mixed))


class RotaryInterleaved(RotaryHalfSplit):
    """Rotation of neighbouring places: the pair (2i, 2i + 1) of the first `rotary_dim` places turns by
    position * f_i, f_i = theta^(-2i / rotary_dim).  The kernels of the mixers that use it rotate from the step's
    table of cosines and sines (`table`) and multiply both by `magnitude`.

    scaling = {factor, original, fast, slow} stretches the slow frequencies for contexts beyond the `original`
    length (YaRN): with dim(t) = rotary_dim * ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(dim(fast)), 0),
    hi = min(ceil(dim(slow)), rotary_dim - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), the
    frequency is f_i / factor * ramp_i + f_i * (1 - ramp_i), and magnitude = 0.1 * ln(factor) + 1."""

    pairing = "interleaved"

    def __init__(self, prefix: str, head_dim: int, theta: float, rotary_dim: int | None = None, scaling=None, **_):
        by_wavelength = bool(scaling) and dict(scaling).get("rule") == "wavelength"
        super().__init__(prefix, head_dim, theta, rotary_dim, scaling=scaling if by_wavelength else None)
        self.scaling = dict(scaling) if scaling else None
        self.magnitude = 1.0
        if self.scaling and not by_wavelength:
            for key in ("factor", "original", "fast", "slow"):
                if not float(self.scaling.get(key, 0)) > 0:
                    raise ValueError(f"rotation scaling needs a positive '{key}'")
            self.magnitude = 0.1 * math.log(float(self.scaling["factor"])) + 1.0

    def inv_freq_host(self) -> torch.Tensor:
        d = self.rotary_dim
        i = torch.arange(0, d // 2, dtype=torch.float64)
        f = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * i / float(d))
        if self.scaling and self.scaling.get("rule") == "wavelength":
            f = stretch_by_wavelength(f, **{k: v for k, v in self.scaling.items() if k != "rule"})
        elif self.scaling:
            sc = self.scaling
            factor, original = float(sc["factor"]), float(sc["original"])

            def place_of(turns: float) -> float:
                return d * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

            lo = max(math.floor(place_of(float(sc["fast"]))), 0)
            hi = min(math.ceil(place_of(float(sc["slow"]))), d - 1)
            ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
            f = f / factor * ramp + f * (1.0 - ramp)
        return f.to(torch.float32)

    def table(self, ctx):
        sc = tuple(sorted(self.scaling.items())) if self.scaling else None
        key = ("rope_table_interleaved", self.theta, self.rotary_dim, sc)
        if key not in ctx.shared:
            inv_freq, _ = self.rotary(ctx.positions.device)
            ctx.shared[key] = kernels.backend().rope_table(ctx.positions, inv_freq)
        return ctx.shared[key]


class NoPosition(PositionEncoding):
    """No position information enters the mixer."""

    graph_safe = True

    def __init__(self, prefix: str = "", **_):
        pass

    def rotary(self, device):
        return None

    def apply(self, q, k, positions):
        return None


register_part("position_encoding", "rope_half_split", RotaryHalfSplit)
register_part("position_encoding", "rope_interleaved", RotaryInterleaved)
register_part("position_encoding", "none", NoPosition)
