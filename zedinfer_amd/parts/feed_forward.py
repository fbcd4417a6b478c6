"""Feed-forward parts."""
from __future__ import annotations

import os
from typing import Dict

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import FeedForward, Runtime, register_feed_forward
from .rows import ProductRows


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
    tape_safe = True
    # For many rows the gate/up product is the library's, and at some sizes it makes the transposed
    # result, W . x^T, faster than x . W^T (measured at the 1.5B sizes: 100 against 119 us at 2,048 rows,
    # 31 against 37 at 512, 73 against 67 at 1,024).  The transposed result goes through the activation
    # kernel that turns it back; the two ways differ by rounding.  Which one a step of n rows takes is
    # read from ``rt.choices[("gate_up_transposed", n, 2I, H)]``: absent, the straight product (or what
    # ZEDINFER_GATE_UP_TRANSPOSED=0/1 says).  ``tune(n)`` measures both outside of any step and records
    # the winner there; nothing is measured while a step runs.
    TRANSPOSED_MIN_ROWS = 128

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        H, I = int(spec.params["hidden_size"]), int(spec.params["intermediate_size"])
        return {"gate": WeightSpec((I, H)), "up": WeightSpec((I, H)), "down": WeightSpec((H, I))}

    def _choice_key(self, n: int) -> tuple:
        return ("gate_up_transposed", int(n), 2 * self.inter, self.hidden)

    def _can_transpose(self, n: int) -> bool:
        return (self.interleave == GATE_UP_BLOCK and self.rt.dtype == torch.bfloat16
                and n >= self.TRANSPOSED_MIN_ROWS and n % 8 == 0)

    def _gate_up_straight(self, x: torch.Tensor, act: torch.Tensor) -> None:
        gu = self.rt.buffer("ffn_gate_up", (x.shape[0], 2 * self.inter))
        ops.linear(x, self.gate_up, out=gu)
        ops.swiglu(gu, out=act, interleave=self.interleave)

    def _gate_up_transposed(self, x: torch.Tensor, act: torch.Tensor) -> None:
        n, I = x.shape[0], self.inter
        gut = self.rt.buffer("ffn_gate_up", (n, 2 * I)).view(-1)[:2 * I * n].view(2 * I, n)      # the same memory
        ops.linear_transposed(x, self.gate_up, out=gut)
        ops.swiglu_t(gut, out=act)

    def _gate_up_many_rows(self, x: torch.Tensor, act: torch.Tensor) -> None:
        """act = swiglu of the gate/up product of x, bfloat16, interleaved weights, more rows than the
        few-rows kernels take."""
        n = x.shape[0]
        if self._can_transpose(n) and x.is_contiguous():
            wins = self.rt.choices.get(self._choice_key(n))
            if wins is None:
                wins = os.environ.get("ZEDINFER_GATE_UP_TRANSPOSED", "") == "1"
            if wins:
                return self._gate_up_transposed(x, act)
        return self._gate_up_straight(x, act)

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def tune(self, num_tokens: int) -> None:
        """For steps of ``num_tokens`` rows: the library's algorithms for the gate/up and down products, then the
        orientation of the gate/up product: three runs each of product plus activation; the transposed one must
        win by 5 %."""
        n, key = int(num_tokens), self._choice_key(num_tokens)
        x = self.rt.buffer("norm_out", (n, self.hidden))
        act = self.rt.buffer("ffn_act", (n, self.inter))
        # first the library's algorithm for each product, then the way round with those
        if self.gate_up is not None:
            self.rt.tune_linear(x, self.gate_up)
            if self._can_transpose(n):
                self.rt.tune_linear(x, self.gate_up, transposed=True)
        self.rt.tune_linear(act, self.down)
        forced = os.environ.get("ZEDINFER_GATE_UP_TRANSPOSED", "")
        if key in self.rt.choices or not self._can_transpose(n) or forced in ("0", "1"):
            return

        def clock(fn):
            fn(x, act)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(3):
                fn(x, act)
            b.record()
            b.synchronize()
            return a.elapsed_time(b)
        self.rt.choices[key] = bool(clock(self._gate_up_transposed) < 0.95 * clock(self._gate_up_straight))

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
        elif self.interleave and ops.linear_sums_supported(x, self.gate_up, ops.FEW_ROWS):
            S = ops.linear_splits(n, 2 * I, self.hidden)
            sums = ops.linear_sums(x, self.gate_up, out=self.rt.buffer("ffn_gate_up_sums", (S, n, 2 * I), torch.float32))
            ops.swiglu(sums, out=act, interleave=self.interleave)
        elif self.interleave == GATE_UP_BLOCK and x.dtype == torch.bfloat16:
            self._gate_up_many_rows(x, act)
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
