"""Position encodings.

What a mixer needs of a rotary encoding is small: ``table(device)`` (float32 frequencies, one per
rotated pair), ``pair_layout`` ("interleaved": pairs (2i, 2i+1); "half": pairs (i, i + r/2)) and
``rotary_dim`` (r: how many leading elements of a head rotate).  Any object with these three can
be handed to the attention mixer; each layer may hold its own (another base, another width).
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from .base import Part

PAIR_LAYOUTS = ("interleaved", "half")


class Rotary(Part):
    """Rotary encoding: angle = pos * freq_i, freq_i = theta^(-2i/rotary_dim), i < rotary_dim/2,
    on the first ``rotary_dim`` elements of a head (all of it by default)
    (reference: src/SharpInference.Cpu/SimdKernels.cs:4591-4629, 4789-4811 for the interleaved
    pairing; the reference's other pairing and its partial width are IsNeoxRope and RopeDim,
    src/SharpInference.Core/ModelGraph.cs:129-141).  ``scaling`` (llama3 rule) stretches the long
    wavelengths: with wavelength L = 2*pi/freq and o the original context, L < o/high keeps freq,
    L > o/low divides it by factor, and between the two it is blended linearly in o/L.  The
    reference only consumes a precomputed divisor table
    (src/SharpInference.Engine/ForwardPass.cs:259-276); here the table comes from the
    configuration.  Frequencies are computed in double and rounded once."""

    def __init__(self, head_dim: int, theta: float, scaling=None, pair_layout: str = "interleaved",
                 rotary_dim: Optional[int] = None):
        rotary_dim = int(head_dim if rotary_dim is None else rotary_dim)
        if rotary_dim % 2 or not 2 <= rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {rotary_dim} must be even and lie in 2..head_dim {head_dim}")
        if pair_layout not in PAIR_LAYOUTS:
            raise ValueError(f"pair_layout {pair_layout!r} is not known ({', '.join(PAIR_LAYOUTS)})")
        self.head_dim, self.theta, self.scaling = int(head_dim), float(theta), scaling
        self.pair_layout, self.rotary_dim = pair_layout, rotary_dim
        self._table: Optional[torch.Tensor] = None

    def frequencies(self) -> torch.Tensor:
        rd = self.rotary_dim
        freqs = []
        for i in range(rd // 2):
            f = math.pow(self.theta, -2.0 * i / rd)
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


class RotaryInterleaved(Rotary):
    """The whole head rotated on pairs (2i, 2i+1): what Llama 4 uses."""

    def __init__(self, head_dim: int, theta: float, scaling=None):
        super().__init__(head_dim, theta, scaling, "interleaved", None)
