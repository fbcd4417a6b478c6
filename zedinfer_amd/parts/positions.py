"""Position encodings.  They act where queries and keys leave the projection; the mixer stores what they made."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.forward_config import PartSpec
from .base import PositionEncoding, Runtime, register_position_encoding


@register_position_encoding("rope_neox")
class RopeNeox(PositionEncoding):
    """Split-half rotary encoding: pairs (k, k + R/2) of the first R = ``rotary_dim`` dims of
    each head turn by pos * theta^(-2k/R) (reference: src/backend/ops/rope/cpu/rope_cpu.cpp:12-66;
    the reference rotates the whole head, no scaling: rope_nvidia.cu:50).
    params: head_dim, theta, rotary_dim (default head_dim)."""

    graph_safe = True
    tape_safe = True

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.head_dim = int(spec.params["head_dim"])
        self.rotary_dim = int(spec.params.get("rotary_dim", self.head_dim))
        self.theta = float(spec.params["theta"])
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= self.head_dim):
            raise ValueError(f"rope_neox: rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        self.inv_freq = ops.rope_inv_freq(self.rotary_dim, self.theta, rt.device)

    def step_table(self, batch):
        key = ("rope_neox", self.rotary_dim, self.theta)
        table = batch.shared.get(key)
        if table is None:
            out = self.rt.buffer(f"rope_table_{self.rotary_dim}_{self.theta!r}",
                                 (batch.num_tokens, self.rotary_dim // 2, 2), torch.float32)
            table = batch.shared[key] = ops.rope_table(batch.positions, self.inv_freq, out=out)
        return table

    def encode(self, q, k, positions, nh: int, nkv: int, d: int) -> None:
        """(A mixer that takes ``step_table`` does not come here.)"""
        table = ops.rope_table(positions, self.inv_freq)
        ops.rope_kv_store(q, None, None, table, None, None, None, nh, nkv, d)
        ops.rope_kv_store(k, None, None, table, None, None, None, nkv, nkv, d)


@register_position_encoding("none")
class NoPosition(PositionEncoding):
    """No encoding: keys and values are stored as they are."""

    graph_safe = True
    tape_safe = True

    def step_table(self, batch):
        return "none"

    def encode(self, q, k, positions, nh: int, nkv: int, d: int) -> None:
        pass
