"""Rotary position encoding.  theta_j = base^(-2j / rotary_dim); the pair of channels that
shares theta_j is (j, j + rotary_dim/2) in the half-split form the reference uses
(src/lfm25_gpu.cu:459-474) or (2j, 2j + 1) in the interleaved form.  theta is computed in
float64 once and rounded to float32; angle, cosine and sine are float32 in the kernel.

Frequency scaling by wavelength (`scaling` = {factor, low, high, original}, the scheme of Llama 3.1's long-context
rotary): with wavelength l = 2 pi / theta, a theta with l < original / high stays, one with l > original / low is
divided by factor, and between the two s = (original / l - low) / (high - low) blends them,
(1 - s) theta / factor + s theta.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from .base import POSITION_ENCODINGS, PositionEncoding, Runtime


_TABLES: dict = {}          # (device, base, rotary_dim, positions) -> table, shared between layers


@POSITION_ENCODINGS.register("rotary")
class Rotary(PositionEncoding):
    graph_safe = True
    records_portions = True

    def __init__(self, head_dim: int, base: float, rotary_dim: Optional[int] = None,
                 interleaved: bool = False, table_positions: Optional[int] = None, scaling: Optional[dict] = None):
        """table_positions: keep the cosines and sines of this many positions in a table on the device
        (shared by all encodings of the same base and size) for kernels that would otherwise spend
        more time on computing them than on the rest of their work."""
        self.head_dim, self.base = int(head_dim), float(base)
        self.table_positions = int(table_positions) if table_positions else 0
        self.angles: Optional[torch.Tensor] = None
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        self.interleaved = bool(interleaved)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within the head size "
                             f"{self.head_dim}")
        self.inv_freq: Optional[torch.Tensor] = None
        self.scaling = None
        if scaling is not None:
            self.scaling = {k: float(scaling[k]) for k in ("factor", "low", "high", "original")}
            if not self.scaling["high"] > self.scaling["low"] or min(self.scaling.values()) <= 0:
                raise ValueError(f"frequency scaling needs positive numbers with high above low, got {scaling}")

    def frequencies(self) -> torch.Tensor:
        """theta_j in float64, scaled where the encoding has a scaling."""
        j = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
        inv = torch.tensor(self.base, dtype=torch.float64) ** (-2.0 * j / self.rotary_dim)
        if self.scaling is None:
            return inv
        sc = self.scaling
        wave = 2.0 * math.pi / inv
        share = ((sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])).clamp(0.0, 1.0)
        # share 1: the wavelength is below original / high and theta stays; share 0: above original / low
        return (1.0 - share) * inv / sc["factor"] + share * inv

    def kernel_modules(self):
        return ["rope_kv"]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        self.inv_freq = self.frequencies().to(torch.float32).to(rt.device)
        if self.table_positions and rt.device.type == "cuda":
            from ..csrc import ops
            key = (str(rt.device), self.base, self.rotary_dim, self.table_positions,
                   None if self.scaling is None else tuple(sorted(self.scaling.items())))
            if key not in _TABLES:
                while len(_TABLES) >= 4:             # tables of models long gone
                    _TABLES.pop(next(iter(_TABLES)))
                _TABLES[key] = ops.rope_table(self.inv_freq, self.table_positions)
            self.angles = _TABLES[key]

    def angle_table(self) -> Optional[torch.Tensor]:
        """float32 [positions, 2, rotary_dim / 2] (cosines, sines) or None."""
        return self.angles

    def rotary_tables(self):
        return self.inv_freq, self.rotary_dim, self.interleaved
