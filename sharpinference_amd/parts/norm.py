"""Normalisation parts."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..ops.profile import section
from .base import INIT_NORM_WEIGHT, ParamSpec, Part, ResidualStream, TensorSource


class RMSNorm(Part):
    """x * rsqrt(mean(x^2) + eps) * w, statistics in float
    (reference: src/SharpInference.Cpu/SimdKernels.cs:4209-4246; CUDA twin
    src/SharpInference.Cuda/CudaTextKernels.cs:199-224).  ``has_weight=False`` is the
    weightless form (SimdKernels.cs:4252-4283)."""

    def __init__(self, dim: int, eps: float, has_weight: bool = True):
        self.dim, self.eps, self.has_weight = int(dim), float(eps), bool(has_weight)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        return {prefix + "weight": ParamSpec((self.dim,), INIT_NORM_WEIGHT)} if self.has_weight else {}

    def load(self, prefix: str, source: TensorSource) -> None:
        if self.has_weight:
            self.weight = source.get(prefix + "weight")

    def forward(self, stream: ResidualStream, out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Fold the pending branch output into the residual sum and normalise.  With ``rows``
        only those rows are produced and the stream is left as it is."""
        n = stream.h.shape[0] if rows is None else rows.shape[0]
        with section("norm", nbytes=n * self.dim * 12):
            out = ops.add_rmsnorm(stream.h, stream.pending, self.weight, self.eps, out_dtype, rows=rows,
                                  write_back=rows is None)
        if rows is None:
            stream.pending = None
        return out
