"""Block arrangements."""
from __future__ import annotations

from typing import Optional

import torch

from .base import Block, LayerMemory, Runtime, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """h += mixer(norm_in(h)); h += feed_forward(norm_post(h))
    (reference: src/frontend/models/transformer_forward.cpp:63-149).  The residual stream is
    float32 and every add into it happens inside the norm that follows it."""

    graph_safe = True
    tape_safe = True

    norm_names = ("input", "post_mixer")

    def __init__(self, norms, mixer, feed_forward, rt: Runtime):
        self.norm_in = norms["input"]
        self.norm_post = norms["post_mixer"]
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.rt = rt

    def forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor], batch, memory: LayerMemory):
        x = self.norm_in.add_forward(resid, delta) if delta is not None else self.norm_in.forward(resid)
        a = self.mixer.forward(x, batch, memory)
        y = self.norm_post.add_forward(resid, a)
        return self.feed_forward.forward(y)
