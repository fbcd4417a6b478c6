"""Feed-forward parts."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import FeedForward, Runtime, register_feed_forward


def stack_rows(tensors):
    """Concatenate [n_i, k] matrices along rows when they share a storage type; else None."""
    if len({t.dtype for t in tensors}) != 1:
        return None
    return torch.cat(list(tensors), dim=0).contiguous()


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """down(up(x) * silu(gate(x))), no biases (reference:
    src/frontend/models/transformer_forward.cpp:128-137; src/backend/ops/swiglu/cpu/swiglu_cpu.cpp:9-23).
    gate and up are stacked into one [2I, H] matrix at load: one product instead of two, the same
    sums per output element.  params: hidden_size, intermediate_size."""

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        H, I = int(spec.params["hidden_size"]), int(spec.params["intermediate_size"])
        return {"gate": WeightSpec((I, H)), "up": WeightSpec((I, H)), "down": WeightSpec((H, I))}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        self.gate_up = stack_rows([weights["gate"], weights["up"]])
        self.gate, self.up = (None, None) if self.gate_up is not None else (weights["gate"], weights["up"])
        self.down = weights["down"]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        n, I = x.shape[0], self.inter
        gu = self.rt.buffer("ffn_gate_up", (n, 2 * I))
        if self.gate_up is not None:
            ops.linear(x, self.gate_up, out=gu)
        else:
            ops.linear(x, self.gate, out=gu[:, :I])
            ops.linear(x, self.up, out=gu[:, I:])
        act = self.rt.buffer("ffn_act", (n, I))
        ops.swiglu(gu[:, :I], gu[:, I:], out=act)
        out = self.rt.buffer("ffn_out", (n, self.hidden))
        return ops.linear(act, self.down, out=out)
