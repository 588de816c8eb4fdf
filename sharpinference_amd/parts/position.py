"""Position encodings."""
from __future__ import annotations

import math
from typing import Optional

import torch

from .base import Part


class RotaryInterleaved(Part):
    """Rotary encoding on interleaved pairs (2i, 2i+1): angle = pos * freq_i,
    freq_i = theta^(-2i/head_dim) (reference: src/SharpInference.Cpu/SimdKernels.cs:4591-4629,
    4789-4811).  ``scaling`` (llama3 rule) stretches the long wavelengths: with wavelength
    L = 2*pi/freq and o the original context, L < o/high keeps freq, L > o/low divides it by
    factor, and between the two it is blended linearly in o/L.  The reference only consumes a
    precomputed divisor table (src/SharpInference.Engine/ForwardPass.cs:259-276); here the table
    comes from the configuration.  Frequencies are computed in double and rounded once."""

    def __init__(self, head_dim: int, theta: float, scaling=None):
        if head_dim % 2:
            raise ValueError("rotary encoding needs an even head_dim")
        self.head_dim, self.theta, self.scaling = int(head_dim), float(theta), scaling
        self._table: Optional[torch.Tensor] = None

    def frequencies(self) -> torch.Tensor:
        hd = self.head_dim
        freqs = []
        for i in range(hd // 2):
            f = math.pow(self.theta, -2.0 * i / hd)
            s = self.scaling
            if s is not None:
                wavelength = 2.0 * math.pi / f
                lo_edge = s.original_max_position_embeddings / s.low_freq_factor
                hi_edge = s.original_max_position_embeddings / s.high_freq_factor
                if wavelength > lo_edge:
                    f = f / s.factor
                elif wavelength >= hi_edge:
                    t = (s.original_max_position_embeddings / wavelength - s.low_freq_factor) / (
                        s.high_freq_factor - s.low_freq_factor)
                    f = (1.0 - t) * f / s.factor + t * f
            freqs.append(f)
        return torch.tensor(freqs, dtype=torch.float64).to(torch.float32)

    def table(self, device) -> torch.Tensor:
        if self._table is None or self._table.device != torch.device(device):
            self._table = self.frequencies().to(device)
        return self._table
