"""Rotary position encoding over the first ``dim`` elements of each head, in pairs (j, j + dim/2)
(``pairing="halves"``, the default) or (2j, 2j + 1) (``pairing="adjacent"``). Frequencies ``inv_freq[j] = 1 / theta**(2j/dim)`` are computed on the host in float32
exactly as the reference does (miniserve/model/qwen3.py:97-100) and moved once; the angles
``float32(position) * inv_freq[j]`` and their cosines and sines are formed in float32 on the device
once per step, as a table that every layer with the same frequencies shares (the reference builds
float32 tables per pass, :105-108).

``scaling`` (optional) slows the long wavelengths down, ``{"kind": "wavelength_bands", "factor", "low", "high",
"original"}``: with wavelength ``l = 2 pi / f``, a frequency stays where ``l < original / high``, becomes ``f / factor``
where ``l > original / low``, and in between is the blend ``(1 - s) f / factor + s f`` with
``s = (original / l - low) / (high - low)``. A second kind, ``{"kind": "turn_ramp", "factor", "original", "fast", "slow"}``,
blends by the pair's index instead: with ``index(n) = dim ln(original / (2 pi n)) / (2 ln theta)`` (the index whose wave makes
``n`` turns within ``original`` positions), ``lo = max(floor(index(fast)), 0)``, ``hi = min(ceil(index(slow)), dim - 1)`` and
``r_j = clamp((j - lo) / max(hi - lo, 0.001), 0, 1)``, pair ``j`` turns by ``r_j f_j / factor + (1 - r_j) f_j``, and every
cosine and sine is multiplied by the magnitude ``0.1 ln(factor) + 1`` (``Rotary.magnitude``; 1 for the other kind). No
counterpart in the reference, which refuses ``rope_scaling``."""

from __future__ import annotations

import math

import torch

from ..config.spec import PartSpec
from .base import PositionEncoding, Rotation
from .registry import register


@register("position", "rotary")
class Rotary(PositionEncoding):
    def __init__(self, spec: PartSpec, rt):
        super().__init__(spec, rt)
        self.dim = int(spec["dim"])
        self.theta = float(spec["theta"])
        if self.dim < 2 or self.dim % 2:
            raise ValueError(f"rotary dim {self.dim} must be even")
        self.pairing = spec.get("pairing", "halves")
        self.scaling = dict(spec["scaling"]) if spec.get("scaling") else None
        expo = torch.arange(0, self.dim, 2, dtype=torch.int64).to(torch.float32) / self.dim
        self.inv_freq_host = 1.0 / (self.theta**expo)
        self.magnitude = 1.0
        if self.scaling is not None:
            self.inv_freq_host = scale_frequencies(self.inv_freq_host, self.scaling, self.theta)
            self.magnitude = scaling_magnitude(self.scaling)
        self.inv_freq = self.inv_freq_host.to(rt.device) if rt is not None else None
        self._key = ("rotary", self.dim, self.theta, tuple(sorted(self.scaling.items())) if self.scaling else None)

    def rotation(self, batch) -> Rotation:
        table = batch.memo.get(self._key)
        if table is None:
            table = batch.memo[self._key] = self.rt.ops.rope_table(batch.positions, self.inv_freq, self.magnitude)
        return Rotation(self.dim, table, self.pairing)


SCALING_KINDS = ("wavelength_bands", "turn_ramp")


def scaling_magnitude(scaling: dict) -> float:
    """What cosines and sines are multiplied by under ``scaling``."""
    if scaling.get("kind", "wavelength_bands") == "turn_ramp":
        return 0.1 * math.log(float(scaling["factor"])) + 1.0
    return 1.0


def _turn_ramp(inv_freq: torch.Tensor, scaling: dict, theta: float) -> torch.Tensor:
    factor, original, fast, slow = (float(scaling[k]) for k in ("factor", "original", "fast", "slow"))
    if not (factor > 0 and original > 0 and fast > 0 and slow > 0 and theta > 1):
        raise ValueError(f"frequency scaling needs positive factor, original, fast and slow and theta > 1, got {scaling}")
    dim = 2 * inv_freq.shape[0]

    def index_of(turns: float) -> float:
        return dim * math.log(original / (2 * math.pi * turns)) / (2 * math.log(theta))

    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), dim - 1)
    out = []
    for j in range(dim // 2):
        f = theta ** (-2.0 * j / dim)  # in double precision: the blend is rounded to float32 once
        r = min(max((j - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(r * f / factor + (1 - r) * f)
    return torch.tensor(out, dtype=torch.float64).to(torch.float32)


def scale_frequencies(inv_freq: torch.Tensor, scaling: dict, theta: float | None = None) -> torch.Tensor:
    """The frequencies after ``scaling`` (see the module's text), evaluated in float64 and rounded to float32 once."""
    kind = scaling.get("kind", "wavelength_bands")
    if kind not in SCALING_KINDS:
        raise NotImplementedError(f"frequency scaling {kind!r} is not supported, expected one of {SCALING_KINDS}")
    if kind == "turn_ramp":
        if theta is None:
            raise ValueError("the turn ramp needs the rotation's base")
        return _turn_ramp(inv_freq, scaling, float(theta))
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    if not (factor > 0 and high > low >= 0 and original > 0):
        raise ValueError(f"frequency scaling needs factor > 0, high > low >= 0 and original > 0, got {scaling}")
    out = []
    shortest, longest = original / high, (original / low if low > 0 else math.inf)
    for f in inv_freq.to(torch.float64).tolist():
        wavelength = 2 * math.pi / f
        if wavelength < shortest:
            out.append(f)
        elif wavelength > longest:
            out.append(f / factor)
        else:
            s = (original / wavelength - low) / (high - low)
            out.append((1 - s) * f / factor + s * f)
    return torch.tensor(out, dtype=torch.float64).to(torch.float32)


@register("position", "none")
class NoPosition(PositionEncoding):
    """No position signal inside the mixer."""
