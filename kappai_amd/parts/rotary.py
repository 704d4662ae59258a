"""Rotary position encoding.

Angles are ``p * theta^(-2j/d)``; the cosine and sine tables are built once in double
precision and stored as float32, as kappai does (src/compute.c:22-56).  ``pairing`` is
"half" for rotate-half pairs (j, j + rot/2) (src/backend/cpu/quants.h:395-409) or
"interleaved" for (2j, 2j+1) (src/backend/cpu/quants.h:411-438); ``rot_dim`` may be less
than the head size (partial rotation).

``stretch`` (factor, original, fast, slow) changes the frequencies for contexts longer than the
``original`` one: with ``place(turns) = rot_dim * ln(original / (2 pi turns)) / (2 ln theta)``,
``lo = max(floor(place(fast)), 0)``, ``hi = min(ceil(place(slow)), rot_dim - 1)`` and
``ramp_j = clamp((j - lo) / max(hi - lo, 0.001), 0, 1)`` pair j turns with
``f_j / factor * ramp_j + f_j * (1 - ramp_j)``: pairs that turn often within the original context
keep their frequency, slow ones are slowed by ``factor``, and those between are blended.  Cosine
and sine are then multiplied by ``0.1 * ln(factor) + 1``.

``wavelength_scaling`` (factor, low, high, original) is another rule for the same end, by the
pair's wavelength ``l = 2 pi / f``: ``f`` stays where ``l < original / high``, becomes
``f / factor`` where ``l > original / low``, and between the two is
``(1 - s) f / factor + s f`` with ``s = (original / l - low) / (high - low)``.  Cosine and sine
keep their size.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import math

import numpy as np
import torch

from ..kernels import ops
from .base import PositionEncoding, register_part


@dataclass
class Rotation:
    cos: torch.Tensor      # [positions, rot_dim/2] float32
    sin: torch.Tensor
    rot_dim: int
    mode: int              # ops.ROT_HALF | ops.ROT_INTERLEAVED


class RotaryEncoding(PositionEncoding):
    def __init__(self, head_dim: int, theta: float, rot_dim: Optional[int] = None,
                 pairing: str = "half", stretch: Optional[dict] = None,
                 wavelength_scaling: Optional[dict] = None):
        if pairing not in ("half", "interleaved"):
            raise ValueError(f"pairing must be 'half' or 'interleaved', got {pairing!r}")
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rot_dim = head_dim if rot_dim is None else rot_dim
        if self.rot_dim % 2 or not 0 < self.rot_dim <= head_dim:
            raise ValueError(f"rot_dim {self.rot_dim} must be even and at most head_dim {head_dim}")
        self.mode = ops.ROT_HALF if pairing == "half" else ops.ROT_INTERLEAVED
        self.stretch = None
        if stretch:
            self.stretch = {k: float(stretch[k]) for k in ("factor", "original", "fast", "slow")}
            if (self.stretch["factor"] <= 0.0 or self.stretch["original"] <= 0.0
                    or self.stretch["fast"] <= 0.0 or self.stretch["slow"] <= 0.0
                    or self.theta <= 1.0):
                raise ValueError(f"stretched rotation needs positive numbers and a base above 1, "
                                 f"got {self.stretch} with base {self.theta}")
        self.wavelength_scaling = None
        if wavelength_scaling:
            ws = {k: float(wavelength_scaling[k]) for k in ("factor", "low", "high", "original")}
            if stretch:
                raise ValueError("one rule for the frequencies of long contexts, not two")
            if ws["factor"] <= 0.0 or ws["original"] <= 0.0 or not ws["high"] > ws["low"] > 0.0:
                raise ValueError(f"scaling by wavelength needs a positive factor and original "
                                 f"length and high > low > 0, got {ws}")
            self.wavelength_scaling = ws
        self._rotation: Optional[Rotation] = None
        self._retired = []      # earlier, shorter tables: captured graphs may still read them

    def frequencies(self):
        """(float64 frequencies of the pairs, factor on cosine and sine)."""
        half = self.rot_dim // 2
        freq = np.power(self.theta, -2.0 * np.arange(half, dtype=np.float64) / self.rot_dim)
        ws = self.wavelength_scaling
        if ws is not None:
            wave = 2.0 * math.pi / freq
            blend = (ws["original"] / wave - ws["low"]) / (ws["high"] - ws["low"])
            between = (1.0 - blend) * freq / ws["factor"] + blend * freq
            freq = np.where(wave < ws["original"] / ws["high"], freq,
                            np.where(wave > ws["original"] / ws["low"], freq / ws["factor"],
                                     between))
            return freq, 1.0
        st = self.stretch
        if st is None:
            return freq, 1.0

        def place(turns: float) -> float:
            return (self.rot_dim * math.log(st["original"] / (2.0 * math.pi * turns))
                    / (2.0 * math.log(self.theta)))

        lo = max(math.floor(place(st["fast"])), 0)
        hi = min(math.ceil(place(st["slow"])), self.rot_dim - 1)
        ramp = np.clip((np.arange(half, dtype=np.float64) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return (freq / st["factor"] * ramp + freq * (1.0 - ramp),
                0.1 * math.log(st["factor"]) + 1.0)

    def tables(self, n_positions: int):
        freq, factor = self.frequencies()
        ang = np.arange(n_positions, dtype=np.float64)[:, None] * freq[None, :]
        return ((np.cos(ang) * factor).astype(np.float32),
                (np.sin(ang) * factor).astype(np.float32))

    def rotation(self, device, max_position: int) -> Rotation:
        """Tables that cover positions 0..max_position; grown in powers of two."""
        r = self._rotation
        if r is None or r.cos.shape[0] <= max_position or r.cos.device != torch.device(device):
            n = 256
            while n <= max_position:
                n *= 2
            c, s = self.tables(n)
            if r is not None:
                self._retired.append(r)
            self._rotation = Rotation(torch.from_numpy(c).to(device), torch.from_numpy(s).to(device),
                                      self.rot_dim, self.mode)
        return self._rotation


register_part("position_encoding", "rotary", RotaryEncoding)
