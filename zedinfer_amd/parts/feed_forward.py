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


def interleave_rows(a: torch.Tensor, b: torch.Tensor, block: int) -> torch.Tensor:
    """[a rows 0..block-1, b rows 0..block-1, a rows block..2*block-1, ...] for two [n, k] matrices."""
    n, k = a.shape
    return torch.stack([a.view(n // block, block, k), b.view(n // block, block, k)], dim=1).reshape(2 * n, k).contiguous()


GATE_UP_BLOCK = 8    # gate and up rows alternate in blocks of 8: one matrix-core tile holds both for 8 columns


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """down(up(x) * silu(gate(x))), no biases (reference:
    src/frontend/models/transformer_forward.cpp:128-137; src/backend/ops/swiglu/cpu/swiglu_cpu.cpp:9-23).
    gate and up are stacked into one [2I, H] matrix at load: one product instead of two, the same
    sums per output element.  In bfloat16 (and with I a multiple of 8) their rows alternate in
    blocks of 8, so that the few-rows product can apply the activation in its epilogue.
    params: hidden_size, intermediate_size."""

    graph_safe = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        H, I = int(spec.params["hidden_size"]), int(spec.params["intermediate_size"])
        return {"gate": WeightSpec((I, H)), "up": WeightSpec((I, H)), "down": WeightSpec((H, I))}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        g, u = weights["gate"], weights["up"]
        self.interleave = 0
        self.gate = self.up = None
        if g.dtype == u.dtype == torch.bfloat16 and self.inter % GATE_UP_BLOCK == 0:
            self.gate_up = interleave_rows(g, u, GATE_UP_BLOCK)
            self.interleave = GATE_UP_BLOCK
        else:
            self.gate_up = stack_rows([g, u])
            if self.gate_up is None:
                self.gate, self.up = g, u
        self.down = weights["down"]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        n, I = x.shape[0], self.inter
        act = self.rt.buffer("ffn_act", (n, I))
        if self.interleave and ops.linear_swiglu_supported(x, self.gate_up):
            ops.linear_swiglu(x, self.gate_up, out=act)
        elif self.interleave and ops.linear_sums_supported(x, self.gate_up):
            S = ops.linear_splits(n, 2 * I, self.hidden)
            sums = ops.linear_sums(x, self.gate_up, out=self.rt.buffer("ffn_gate_up_sums", (S, n, 2 * I), torch.float32))
            ops.swiglu(sums, out=act, interleave=self.interleave)
        else:
            gu = self.rt.buffer("ffn_gate_up", (n, 2 * I))
            if self.gate_up is not None:
                ops.linear(x, self.gate_up, out=gu)
            else:
                ops.linear(x, self.gate, out=gu[:, :I])
                ops.linear(x, self.up, out=gu[:, I:])
            if self.interleave:
                ops.swiglu(gu, out=act, interleave=self.interleave)
            else:
                ops.swiglu(gu[:, :I], gu[:, I:], out=act)
        if ops.linear_sums_supported(act, self.down):
            S = ops.linear_splits(n, self.hidden, I)
            return ops.linear_sums(act, self.down, out=self.rt.buffer("ffn_out_sums", (S, n, self.hidden), torch.float32))
        out = self.rt.buffer("ffn_out", (n, self.hidden))
        return ops.linear(act, self.down, out=out)
