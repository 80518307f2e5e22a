"""Rotary position encoding.

Angles are ``p * theta^(-2j/d)``; the cosine and sine tables are built once in double
precision and stored as float32, as kappai does (src/compute.c:22-56).  ``pairing`` is
"half" for rotate-half pairs (j, j + rot/2) (src/backend/cpu/quants.h:395-409) or
"interleaved" for (2j, 2j+1) (src/backend/cpu/quants.h:411-438); ``rot_dim`` may be less
than the head size (partial rotation).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

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
                 pairing: str = "half"):
        if pairing not in ("half", "interleaved"):
            raise ValueError(f"pairing must be 'half' or 'interleaved', got {pairing!r}")
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rot_dim = head_dim if rot_dim is None else rot_dim
        if self.rot_dim % 2 or not 0 < self.rot_dim <= head_dim:
            raise ValueError(f"rot_dim {self.rot_dim} must be even and at most head_dim {head_dim}")
        self.mode = ops.ROT_HALF if pairing == "half" else ops.ROT_INTERLEAVED
        self._rotation: Optional[Rotation] = None
        self._retired = []      # earlier, shorter tables: captured graphs may still read them

    def tables(self, n_positions: int):
        half = self.rot_dim // 2
        freq = np.power(self.theta, -2.0 * np.arange(half, dtype=np.float64) / self.rot_dim)
        ang = np.arange(n_positions, dtype=np.float64)[:, None] * freq[None, :]
        return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)

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
