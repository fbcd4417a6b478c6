"""The description a model is built from: parts chosen layer by layer, and the
order in which layers run.

An architecture turns its typed config into one ``ModelForwardConfig``.  The
engine never looks at the architecture again: it builds every part from its
``PartSpec`` through the part registries, binds weights by the tensor names the
specs carry, and runs ``schedule`` in order.  The reference keeps the same
facts as flags on one struct (reference: include/frontend/models/forward_config.hpp:27-64,
qwen2.hpp:29-34); here they are data per layer, so that one model can mix
mixers and feed-forwards.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part: which registered kind, its sizes and constants, and the
    checkpoint tensor name behind each of its parameters."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    weights: Dict[str, str] = field(default_factory=dict)  # parameter -> tensor name

    def with_params(self, **kw) -> "PartSpec":
        p = dict(self.params)
        p.update(kw)
        return PartSpec(self.kind, p, dict(self.weights))


@dataclass(frozen=True)
class LayerSpec:
    """One block: an arrangement kind and the parts it arranges."""

    block: str                      # registered block arrangement, e.g. "prenorm"
    mixer: PartSpec
    feed_forward: PartSpec
    norms: Dict[str, PartSpec]      # arrangement-specific names, e.g. "input", "post_mixer"


@dataclass(frozen=True)
class ScheduleStep:
    """One entry of the run order.

    ``layer`` indexes ``ModelForwardConfig.layers`` (a layer may appear more
    than once).  ``cache`` names the cache/state buffer this run uses; two
    steps with the same ``cache`` share it.  Only a step with ``writes_cache``
    stores keys and values; a step that reads another step's cache sets it to
    False and names that step's ``cache``.
    """

    layer: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelForwardConfig:
    """Everything the engine needs to build and run a decoder."""

    architecture: str
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleStep, ...]
    final_norm: PartSpec
    lm_head: PartSpec
    tie_word_embeddings: bool = False
    eos_token_ids: Tuple[int, ...] = ()
    max_position_embeddings: int = 0
    # What the architecture wants to say about itself, for whoever inspects a model (the reference keeps family
    # flags on its forward config: forward_config.hpp:36-37).  Nothing in the engine reads it: what a part needs
    # is in its PartSpec.
    family: Dict[str, Any] = field(default_factory=dict)

    def validate(self) -> None:
        n = len(self.layers)
        writers: Dict[int, int] = {}
        for i, st in enumerate(self.schedule):
            if not (0 <= st.layer < n):
                raise ValueError(f"schedule step {i} names layer {st.layer}; the model has {n} layers")
            if st.writes_cache:
                if st.cache in writers:
                    raise ValueError(
                        f"schedule steps {writers[st.cache]} and {i} both write cache {st.cache}")
                writers[st.cache] = i
        for i, st in enumerate(self.schedule):
            if not st.writes_cache:
                w = writers.get(st.cache)
                if w is None or w > i:
                    raise ValueError(
                        f"schedule step {i} reads cache {st.cache}, which no earlier step writes")


def default_schedule(num_layers: int) -> Tuple[ScheduleStep, ...]:
    """Each layer once, in order, each with a cache of its own."""
    return tuple(ScheduleStep(layer=i, cache=i) for i in range(num_layers))
