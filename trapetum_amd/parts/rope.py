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
import torch

from ..registry import register_part
from .base import Position


class RotaryPosition(Position):
    def __init__(self, rotary_dim, theta, pairing="halves"):
        if rotary_dim % 2:
            raise ValueError(f"rotary_dim {rotary_dim} must be even")
        if pairing not in ("halves", "neighbours"):
            raise ValueError(f"pairing '{pairing}' is neither halves nor neighbours")
        self.rotary_dim = rotary_dim
        self.theta = float(theta)
        self.pairing = pairing
        self._tables = {}

    def inv_freq(self, device):
        key = str(device)
        if key not in self._tables:
            e = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
            self._tables[key] = (1.0 / (self.theta ** e)).to(device)
        return self._tables[key]


class NoPosition(Position):
    """Keys and queries are used as projected."""
    rotary_dim = 0

    def inv_freq(self, device):
        return None


register_part("position", "rope", RotaryPosition)
register_part("position", "none", NoPosition)
