"""Token embedding and the output head."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import Part, Runtime, register_embedding, register_head


@register_embedding("token")
class TokenEmbedding(Part):
    """h[i,:] = table[ids[i],:], unscaled, widened into the float32 residual stream
    (reference: src/frontend/models/transformer_forward.cpp:54-60).  params: vocab_size, hidden_size."""

    graph_safe = True
    tape_safe = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((int(spec.params["vocab_size"]), int(spec.params["hidden_size"])))}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.weight = weights["weight"]
        self.vocab, self.hidden = self.weight.shape

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        out = self.rt.buffer("resid", (ids.numel(), self.hidden), torch.float32)
        return ops.embedding(ids, self.weight, out=out)


@register_head("linear")
class LinearHead(Part):
    """logits = x . W^T in float32, no bias (reference: transformer_forward.cpp:155-156).  With
    ``tied_to`` in the spec's weights the checkpoint may leave the tensor out and the embedding
    table stands in (reference: src/frontend/models/base.cpp:410-416).
    params: vocab_size, hidden_size, tied_to (tensor name or None)."""

    graph_safe = True
    tape_safe = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((int(spec.params["vocab_size"]), int(spec.params["hidden_size"])),
                                     fallback=spec.params.get("tied_to"))}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        self.weight = weights["weight"]
        self.vocab = self.weight.shape[0]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out = self.rt.buffer("logits", (x.shape[0], self.vocab), torch.float32)
        return ops.linear(x, self.weight, out=out)
