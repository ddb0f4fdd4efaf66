"""Rotary position encoding as a table of inverse frequencies.

inv_freq[d] = theta^(-2d / rotary_dim) for d in [0, rotary_dim / 2), computed once in
fp32 as 1 / theta^(arange(0, dim, 2) / dim) (model/export_gemma.py:53).  The rotation
itself (pairs (d, d + rotary_dim/2), angle = position * inv_freq[d], fp32 cos/sin:
runtime/cuda/codebook_gemv.cu:219-230) is applied by the mixer's kernel just before
the cache write; a variant with other frequencies only needs another table, which is
how the reference carries its scaled variants too (runtime/src/lib.rs:1071-1076).
`pairing` says which elements turn together: "halves", the reference's (d, d + rotary_dim/2),
or "neighbours" (2d, 2d + 1); the kernel that fuses a decode step's rotation with its
attention knows the halves only, so another pairing takes the separate launches.
"""
import math

import torch

from ..registry import register_part
from .base import Position


class RotaryPosition(Position):
    def __init__(self, rotary_dim, theta, pairing="halves", scaling=None):
        """scaling: None, or {"factor", "low", "high", "original"}: a frequency f whose wavelength 2 pi / f is longer than
        original / low is divided by factor, one shorter than original / high is kept, and in between the two are mixed,
        (1 - s) f / factor + s f with s = (original / wavelength - low) / (high - low)."""
        if rotary_dim % 2:
            raise ValueError(f"rotary_dim {rotary_dim} must be even")
        if pairing not in ("halves", "neighbours"):
            raise ValueError(f"pairing '{pairing}' is neither halves nor neighbours")
        self.rotary_dim = rotary_dim
        self.theta = float(theta)
        self.pairing = pairing
        self.scaling = None
        if scaling is not None:
            self.scaling = {k: float(scaling[k]) for k in ("factor", "low", "high", "original")}
            if self.scaling["high"] <= self.scaling["low"] or self.scaling["factor"] <= 0:
                raise ValueError(f"frequency scaling {scaling!r}: high must exceed low and factor be positive")
        self._tables = {}

    def inv_freq(self, device):
        key = str(device)
        if key not in self._tables:
            e = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
            f = 1.0 / (self.theta ** e)
            if self.scaling is not None:
                sc = self.scaling
                wave = 2.0 * math.pi / f
                s = ((sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])).clamp(0.0, 1.0)
                mixed = (1.0 - s) * f / sc["factor"] + s * f
                f = torch.where(wave > sc["original"] / sc["low"], f / sc["factor"],
                                torch.where(wave < sc["original"] / sc["high"], f, mixed))
            self._tables[key] = f.to(torch.float32).to(device)
        return self._tables[key]


class NoPosition(Position):
    """Keys and queries are used as projected."""
    rotary_dim = 0

    def inv_freq(self, device):
        return None


register_part("position", "rope", RotaryPosition)
register_part("position", "none", NoPosition)
