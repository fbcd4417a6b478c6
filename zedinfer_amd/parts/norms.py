"""Normalisation parts."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import Norm, Runtime, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """y = w * x * rsqrt(mean(x^2) + eps); with ``add_one`` the weight is (1 + w)
    (reference: src/backend/ops/rms_norm/cpu/rms_norm_cpu.cpp:14-29).
    params: dim, eps, add_one (default False)."""

    graph_safe = True
    tape_safe = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        # a gain: 1 in random-weights mode (0 when the norm multiplies by 1 + w)
        return {"weight": WeightSpec((int(spec.params["dim"]),),
                                     init="zeros" if spec.params.get("add_one", False) else "ones")}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.dim = int(spec.params["dim"])
        self.eps = float(spec.params["eps"])
        self.add_one = bool(spec.params.get("add_one", False))
        self.weight = weights["weight"]

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        out = self.rt.buffer("norm_out", (x.shape[0], self.dim), out_dtype or self.rt.dtype)
        return ops.rms_norm(x, self.weight, self.eps, out=out, add_one=self.add_one)

    def add_forward(self, resid: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        out = self.rt.buffer("norm_out", (resid.shape[0], self.dim), self.rt.dtype)
        return ops.add_rms_norm(resid, delta, self.weight, self.eps, out=out, add_one=self.add_one)
