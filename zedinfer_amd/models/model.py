"""Building a decoder from its description and running one step through it.

``DecoderModel`` knows parts and the schedule, nothing about architectures: it
collects the tensors every part asks for, binds them by name, builds the parts
through the registries and runs ``schedule`` in order (reference: the dense loop
of src/frontend/models/transformer_forward.cpp:63-156).
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from .. import ops
from ..config.forward_config import ModelForwardConfig, PartSpec
from ..parts import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, KVCacheRequest, LayerMemory, Part,
                     Runtime, StateRequest)
from ..weights.loader import WeightSpec


def _part_weights(registry, spec: PartSpec) -> Dict[str, WeightSpec]:
    """tensor name -> spec, for one part."""
    cls = registry.get(spec.kind)
    out: Dict[str, WeightSpec] = {}
    for param, ws in cls.weight_specs(spec).items():
        if param not in spec.weights:
            raise ValueError(f"part '{spec.kind}' needs parameter '{param}' but its spec names no tensor for it")
        out[spec.weights[param]] = ws
    return out


def expected_weights(fc: ModelForwardConfig) -> Dict[str, WeightSpec]:
    """Every checkpoint tensor the model needs, with its shape."""
    exp: Dict[str, WeightSpec] = {}

    def merge(d: Dict[str, WeightSpec]):
        for name, ws in d.items():
            if name in exp and exp[name].shape != ws.shape:
                raise ValueError(f"tensor '{name}' is asked for with shapes {exp[name].shape} and {ws.shape}")
            # a part that can live without the tensor does not make it optional for another
            if name not in exp or exp[name].fallback is not None:
                exp[name] = ws
    merge(_part_weights(EMBEDDINGS, fc.embedding))
    for layer in fc.layers:
        merge(_part_weights(MIXERS, layer.mixer))
        merge(_part_weights(FEED_FORWARDS, layer.feed_forward))
        for n in layer.norms.values():
            merge(_part_weights(NORMS, n))
    merge(_part_weights(NORMS, fc.final_norm))
    merge(_part_weights(HEADS, fc.lm_head))
    return exp


def _build(registry, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
    cls = registry.get(spec.kind)
    local = {param: weights[name] for param, name in spec.weights.items() if param in cls.weight_specs(spec)}
    return cls(spec, local, rt)


class DecoderModel:
    def __init__(self, fc: ModelForwardConfig, weights: Dict[str, torch.Tensor], rt: Runtime):
        fc.validate()
        self.fc = fc
        self.rt = rt
        self.embedding = _build(EMBEDDINGS, fc.embedding, weights, rt)
        self.blocks = []
        self.parts = []         # every part that was built, blocks included
        for layer in fc.layers:
            block_cls = BLOCKS.get(layer.block)
            missing = [n for n in block_cls.norm_names if n not in layer.norms]
            if missing:
                raise ValueError(f"block '{layer.block}' needs norms {missing}")
            norms = {n: _build(NORMS, layer.norms[n], weights, rt) for n in block_cls.norm_names}
            mixer = _build(MIXERS, layer.mixer, weights, rt)
            ffn = _build(FEED_FORWARDS, layer.feed_forward, weights, rt)
            self.blocks.append(block_cls(norms, mixer, ffn, rt))
            # a mixer's position encoding is a part of its own
            self.parts += [self.blocks[-1], mixer, ffn, *norms.values()]
            self.parts += [p for p in vars(mixer).values() if isinstance(p, Part)]
        self.final_norm = _build(NORMS, fc.final_norm, weights, rt)
        self.lm_head = _build(HEADS, fc.lm_head, weights, rt)
        self.parts += [self.embedding, self.final_norm, self.lm_head]
        self.vocab_size = fc.vocab_size
        self.hidden_size = fc.hidden_size
        # the parts that have a say in the numbers of rows steps are padded to
        self._row_parts = [p for p in self.parts if getattr(type(p), "step_rows", Part.step_rows) is not Part.step_rows]
        self._step_rows: Dict[tuple, int] = {}

    # ---- what the cache manager has to provide ------------------------------
    def cache_requests(self) -> Dict[int, KVCacheRequest]:
        """cache id -> what the step that writes it needs."""
        out: Dict[int, KVCacheRequest] = {}
        for st in self.fc.schedule:
            req = self.blocks[st.layer].mixer.cache_request()
            if req is None:
                continue
            if st.cache in out and out[st.cache].tensors != req.tensors:
                raise ValueError(f"cache {st.cache} is shared by layers that keep different tensors in a page")
            if st.writes_cache or st.cache not in out:
                out[st.cache] = req
        return out

    def state_requests(self) -> Dict[int, StateRequest]:
        out: Dict[int, StateRequest] = {}
        for st in self.fc.schedule:
            req = self.blocks[st.layer].mixer.state_request()
            if req is not None:
                out[st.cache] = req
        return out

    def planners(self) -> tuple:
        """The planners of the mixers' launches, one per key, in the order of the layers."""
        out = {}
        for b in self.blocks:
            pl = b.mixer.planner()
            if pl is not None and pl.key not in out:
                out[pl.key] = pl
        return tuple(out.values())

    def step_rows(self, rows: int, kind: str) -> int:
        """The number of rows (``Part.step_rows`` says of what, by ``kind``) a step of ``rows`` is run with when it
        is padded: the least number from ``rows`` on that every part accepts."""
        key = (int(rows), kind)
        found = self._step_rows.get(key)
        if found is None:
            r = max(int(rows), 1)
            for _ in range(64):
                nxt = max(int(p.step_rows(r, kind)) for p in self._row_parts) if self._row_parts else r
                if nxt < r:
                    raise ValueError(f"a part wants a step of {r} rows run with fewer ({nxt})")
                if nxt == r:
                    break
                r = nxt
            else:
                raise ValueError(f"the parts do not agree on a number of rows for a step of {rows} ({kind})")
            found = self._step_rows[key] = r
        return found

    def position_axes(self) -> int:
        """The axes the step's positions need: the most any position encoding of the model reads."""
        return max([int(getattr(p, "position_axes", 1)) for p in self.parts] + [1])

    def padding_safe(self) -> bool:
        """Whether steps may be padded to recurring shapes: every mixer says that padding is harmless to it."""
        return all(getattr(b.mixer, "padding_safe", False) for b in self.blocks)

    def graph_safe(self) -> bool:
        """Whether a step's launches can be captured and replayed: every part says so."""
        return all(getattr(p, "graph_safe", False) for p in self.parts)

    def tape_safe(self) -> bool:
        """Whether a step's device work is calls into the kernel library alone: every part says so."""
        return all(getattr(p, "graph_safe", False) and getattr(p, "tape_safe", False) for p in self.parts)

    # ---- one step -------------------------------------------------------------
    def run(self, batch, memories: Sequence[LayerMemory]) -> Optional[torch.Tensor]:
        """Run the tokens of ``batch`` through the schedule; float32 logits [wanted, vocab]
        at ``batch.logit_rows``, or None when no row is wanted."""
        shared = getattr(batch, "shared", None)
        if shared is not None:
            shared.clear()      # what parts share holds for one run: a batch object may serve several steps
        resid = self.embedding.forward(batch.token_ids)
        delta = None
        for st, mem in zip(self.fc.schedule, memories):
            delta = self.blocks[st.layer].forward(resid, delta, batch, mem)
        if batch.num_logit_rows == 0:
            if delta is not None:
                pass  # the last feed-forward's output is not needed when no logits are
            return None
        rows = batch.logit_rows
        if delta is not None and delta.dim() == 3:
            # float32 partial sums (few tokens): norm every row, then pick the wanted ones
            x_all = self.final_norm.add_forward(resid, delta)
            if getattr(batch, "all_rows_wanted", False):
                return self.lm_head.forward(x_all)
            x = ops.gather_rows(x_all, rows, out=self.rt.buffer("norm_rows", (batch.num_logit_rows, self.hidden_size),
                                                               x_all.dtype))
            return self.lm_head.forward(x)
        if getattr(batch, "all_rows_wanted", False):      # every row, in order: nothing to pick
            x = self.final_norm.add_forward(resid, delta) if delta is not None else self.final_norm.forward(resid)
            return self.lm_head.forward(x)
        r = self.rt.buffer("resid_rows", (batch.num_logit_rows, self.hidden_size), torch.float32)
        ops.gather_rows(resid, rows, out=r)
        if delta is not None:
            dsel = self.rt.buffer("delta_rows", (batch.num_logit_rows, self.hidden_size), delta.dtype)
            ops.gather_rows(delta, rows, out=dsel)
            x = self.final_norm.add_forward(r, dsel)
        else:
            x = self.final_norm.forward(r)
        return self.lm_head.forward(x)
