"""Rotary position encodings as tables for the rotation kernel.

The kernel rotates the pair ``(f, f + rot/2)`` of every head by the angle
``float32(position[freq_row[f]]) * inv_freq[f]``.  A position encoding is therefore a choice
of ``inv_freq`` and ``freq_row``:

* MRoPE (reference src/qwen25vl_lite/rope.py:26-33, 48-96): ``inv_freq[f] = theta^(-2f/hd)``;
  the three section counts, repeated as a list over both halves of the head, give frequency
  ``f`` the row 0, 1 or 2 (t, h, w) according to the section it falls in.
* Plain 1-D RoPE: every frequency reads row 0; ``rotary_dim`` below the head size leaves the
  remaining channels unrotated.
"""

from __future__ import annotations

import math
from typing import Tuple

import torch

from .base import PositionEncoding, register_part

__all__ = ["MRoPE", "RoPE1D", "inverse_frequencies", "rescale_frequencies", "ramp_frequencies"]


def inverse_frequencies(rotary_dim: int, theta: float) -> torch.Tensor:
    """``1 / theta^(2f / rotary_dim)`` in float32, as the reference builds it (rope.py:32-33)."""
    idx = torch.arange(0, rotary_dim, 2, dtype=torch.float32)
    return 1.0 / (float(theta) ** (idx / rotary_dim))


class MRoPE(PositionEncoding):
    """params: ``theta``, ``sections`` (three counts adding up to half the head size)."""

    num_rows = 3

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.theta = float(params["theta"])
        self.sections = tuple(int(s) for s in params["sections"])
        if len(self.sections) != 3:
            raise ValueError("MRoPE takes three section counts (t, h, w)")
        self._tables = {}

    def table_key(self, head_dim: int):
        return ("mrope", self.theta, self.sections, head_dim)

    def rotary_tables(self, head_dim: int) -> Tuple[torch.Tensor, torch.Tensor]:
        if head_dim not in self._tables:
            half = head_dim // 2
            if sum(self.sections) != half:
                # reference rope.py:89-93
                raise ValueError(f"mrope sections {self.sections} do not cover half the head size {half}")
            rows = []
            for row, count in enumerate(self.sections):
                rows += [row] * count
            self._tables[head_dim] = (
                inverse_frequencies(head_dim, self.theta).to(self.device),
                torch.tensor(rows, dtype=torch.int32, device=self.device),
            )
        return self._tables[head_dim]


def rescale_frequencies(freqs: torch.Tensor, factor: float, low: float, high: float, original: int) -> torch.Tensor:
    """Frequencies stretched for contexts beyond the ``original`` length, by wavelength
    ``l = 2 pi / f``: ``l < original / high`` keeps ``f``; ``l > original / low`` gives ``f / factor``;
    between the two, with ``s = (original / l - low) / (high - low)``, the blend
    ``(1 - s) f / factor + s f``.  Computed in float64."""
    f = freqs.to(torch.float64)
    wavelength = 2.0 * math.pi / f
    s = ((original / wavelength - low) / (high - low)).clamp(0.0, 1.0)
    blended = (1.0 - s) * f / factor + s * f
    return torch.where(wavelength < original / high, f, torch.where(wavelength > original / low, f / factor, blended))


def ramp_frequencies(freqs: torch.Tensor, theta: float, factor: float, original: int, fast: float, slow: float):
    """Frequencies stretched by a ramp over the channel index, and the factor that goes on every
    cosine and sine.  With ``d = 2 len(freqs)`` rotated channels, a frequency that makes ``t`` turns
    over the ``original`` length sits at index ``i(t) = d ln(original / (2 pi t)) / (2 ln theta)``;
    ``lo = max(floor(i(fast)), 0)``, ``hi = min(ceil(i(slow)), d - 1)``, ``r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``;
    frequency ``i`` becomes ``f_i / factor * r_i + f_i (1 - r_i)`` and the amplitude is
    ``0.1 ln(factor) + 1``.  Computed in float64."""
    f = freqs.to(torch.float64)
    d = 2 * f.shape[0]

    def index_of(turns: float) -> float:
        return d * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), d - 1)
    ramp = ((torch.arange(f.shape[0], dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


class RoPE1D(PositionEncoding):
    """params: ``theta``, optional ``rotary_dim`` (default: the whole head), optional ``scaling``
    (``factor``, ``low``, ``high``, ``original``: see :func:`rescale_frequencies`; or ``kind: "ramp"``
    with ``factor``, ``original``, ``fast``, ``slow``: see :func:`ramp_frequencies`, which also scales
    the cosines and sines: ``amplitude``; or ``kind: "linear"`` with ``factor``: every frequency divided by it), optional
    ``interleaved`` (True: channel 2f is rotated with channel 2f+1; default: f with f + rot/2.  The
    kernel that rotates reads it from the encoding)."""

    num_rows = 1

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.theta = float(params["theta"])
        self.rotary_dim = params.get("rotary_dim")
        self.interleaved = bool(params.get("interleaved", False))
        sc = params.get("scaling")
        self.scaling = None
        self.ramp = None
        self.divide = None
        self.amplitude = 1.0
        if sc and sc.get("kind") == "linear":
            self.divide = float(sc["factor"])
            if not self.divide > 0:
                raise ValueError("frequencies are divided by a positive factor")
        elif sc and sc.get("kind") == "ramp":
            self.ramp = (float(sc["factor"]), int(sc["original"]), float(sc["fast"]), float(sc["slow"]))
            if not (self.ramp[0] > 0 and self.ramp[2] > 0 and self.ramp[3] > 0 and self.theta > 1):
                raise ValueError("a frequency ramp needs a positive factor and turn counts, and a base above 1")
            self.amplitude = 0.1 * math.log(self.ramp[0]) + 1.0
        elif sc:
            self.scaling = (float(sc["factor"]), float(sc["low"]), float(sc["high"]), int(sc["original"]))
            if not (self.scaling[0] > 0 and self.scaling[2] > self.scaling[1]):
                raise ValueError("frequency scaling needs a positive factor and high > low")
        self._tables = {}

    def table_key(self, head_dim: int):
        return ("rope", self.theta, self.rotary_dim, self.scaling, self.ramp, self.divide, head_dim)

    def rotary_tables(self, head_dim: int) -> Tuple[torch.Tensor, torch.Tensor]:
        if head_dim not in self._tables:
            rot = int(self.rotary_dim) if self.rotary_dim is not None else head_dim
            if rot % 2 or rot > head_dim:
                raise ValueError(f"rotary_dim {rot} must be even and at most the head size {head_dim}")
            if self.ramp is not None:
                idx = torch.arange(0, rot, 2, dtype=torch.float64)
                freqs = ramp_frequencies(float(self.theta) ** (-idx / rot), self.theta, *self.ramp)[0].to(torch.float32)
            elif self.divide is not None:
                idx = torch.arange(0, rot, 2, dtype=torch.float64)
                freqs = (float(self.theta) ** (-idx / rot) / self.divide).to(torch.float32)
            elif self.scaling is None:
                freqs = inverse_frequencies(rot, self.theta)
            else:
                idx = torch.arange(0, rot, 2, dtype=torch.float64)
                freqs = rescale_frequencies(float(self.theta) ** (-idx / rot), *self.scaling).to(torch.float32)
            self._tables[head_dim] = (
                freqs.to(self.device),
                torch.zeros(rot // 2, dtype=torch.int32, device=self.device),
            )
        return self._tables[head_dim]


register_part("position", "mrope", MRoPE)
register_part("position", "rope", RoPE1D)
