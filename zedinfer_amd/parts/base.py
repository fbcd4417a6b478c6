"""What every part shares: the registries by kind, the runtime a part is built
with, and the interfaces a new part has to meet.

A part is a class registered under a kind.  It states the checkpoint tensors it
needs from its spec alone (``weight_specs``), is built from (spec, weights,
runtime) and never learns which model it sits in.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Callable, Dict, Optional, Sequence, Tuple

import torch

from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec


class Runtime:
    """Device, activation type and reusable workspaces.

    ``buffer(name, shape)`` hands out a view into a named allocation that only
    ever grows, so that steady-state steps allocate nothing and buffers keep
    their addresses (what a captured graph needs).  When a larger step outgrows
    an allocation, the old one is kept, not freed: graphs captured earlier go on
    reading and writing it, and freed memory would by then belong to someone
    else.  Allocations grow by at least half, so what is kept stays below twice
    the largest.
    """

    def __init__(self, device: torch.device | str, dtype: torch.dtype):
        self.device = torch.device(device)
        self.dtype = dtype
        self._buffers: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
        self._views: Dict[tuple, torch.Tensor] = {}     # (name, dtype, shape) -> the view handed out last time
        self._outgrown: list = []                       # allocations that captured graphs may still use
        # Decisions between equivalent ways of computing something (which differ by rounding), by a key
        # the deciding part chooses.  They are made outside of steps (``Part.tune``, ``Engine.warm_up``)
        # or given by the caller, never while a step runs: a run with the same choices gives the same bits.
        self.choices: Dict[tuple, object] = {}

    def tune_linear(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                    transposed: bool = False, out_dtype: Optional[torch.dtype] = None) -> None:
        """Outside of any step: let the library choose, by timing its proposals, the algorithm of the product
        ``ops.linear`` (``ops.linear_transposed``) makes of operands of these shapes, and record the choice in
        ``choices``; a choice already recorded there (an earlier run's) is put in force instead.  Nothing happens
        for products that are not the library's (few rows, float32) or with ZEDINFER_TUNE_LIBRARY=0."""
        if os.environ.get("ZEDINFER_TUNE_LIBRARY", "1") == "0" or x.device.type != "cuda":
            return
        from .. import ops
        key = ("library_product", int(x.shape[0]), int(weight.shape[0]), int(x.shape[1]), bias is not None,
               bool(transposed), "float32" if out_dtype == torch.float32 else "bfloat16")
        known = self.choices.get(key)
        if known is not None:
            ops.linear_choose(x, weight, int(known), bias, transposed, out_dtype)
            return
        found = ops.linear_tune(x, weight, bias, transposed, out_dtype)
        if found is not None:
            self.choices[key] = found[0]

    def buffer(self, name: str, shape: Tuple[int, ...], dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        dtype = dtype or self.dtype
        vkey = (name, dtype, tuple(shape))
        view = self._views.get(vkey)
        if view is not None:
            return view                 # steps of a shape seen before ask for the same views again
        n = 1
        for s in shape:
            n *= int(s)
        key = (name, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < n:
            if buf is not None:
                self._outgrown.append(buf)
                n_alloc = max(n, buf.numel() + buf.numel() // 2)
            else:
                n_alloc = max(n, 1)
            buf = torch.empty((n_alloc,), dtype=dtype, device=self.device)
            self._buffers[key] = buf
            self._views = {k: v for k, v in self._views.items() if k[:2] != key}    # they point into the old one
        if len(self._views) >= 4096:
            self._views.clear()
        view = self._views[vkey] = buf[:n].view(tuple(shape))
        return view

    def poison(self) -> None:
        """Make every floating-point workspace NaN (a check that a replay writes all it reads; integer workspaces
        may hold indices and are left alone)."""
        for buf in self._buffers.values():
            if buf.dtype.is_floating_point:
                buf.fill_(float("nan"))

    def outgrown_bytes(self) -> int:
        """Bytes of allocations that were outgrown and are kept for graphs captured before."""
        return sum(b.numel() * b.element_size() for b in self._outgrown)

    def reserve(self, name: str, numel: int, dtype: Optional[torch.dtype] = None) -> None:
        self.buffer(name, (numel,), dtype)


class Registry:
    def __init__(self, what: str):
        self.what = what
        self._kinds: Dict[str, type] = {}

    def register(self, kind: str) -> Callable[[type], type]:
        def deco(cls: type) -> type:
            self._kinds[kind] = cls
            cls.kind = kind
            return cls
        return deco

    def get(self, kind: str) -> type:
        if kind not in self._kinds:
            raise KeyError(f"no {self.what} registered as '{kind}'; registered: {', '.join(sorted(self._kinds))}")
        return self._kinds[kind]

    def kinds(self) -> Tuple[str, ...]:
        return tuple(sorted(self._kinds))


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block arrangement")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("output head")

register_mixer = MIXERS.register
register_feed_forward = FEED_FORWARDS.register
register_norm = NORMS.register
register_position_encoding = POSITION_ENCODINGS.register
register_block = BLOCKS.register
register_embedding = EMBEDDINGS.register
register_head = HEADS.register


PAGE = -1      # in the shape of a page tensor: where the number of tokens a page holds goes


@dataclass(frozen=True)
class PageTensor:
    """One tensor a mixer keeps per page of the cache: ``shape`` is that of one page, with PAGE where the page
    size goes (the cache manager knows it, the mixer need not); ``dtype`` None is the engine's activation type."""

    shape: Tuple[int, ...]
    dtype: Optional[torch.dtype] = None

    def page_shape(self, page_size: int) -> Tuple[int, ...]:
        return tuple(int(page_size) if s == PAGE else int(s) for s in self.shape)


@dataclass(frozen=True)
class KVCacheRequest:
    """What a mixer needs from the paged cache: pages for all positions ("full") or for the last ``window``
    positions ("window"), and in every page the named ``tensors`` (name, PageTensor).  The cache manager
    allocates [pages, *page shape] for each and hands them to the mixer's runs by name
    (``LayerMemory.tensors``); what they hold and how they are laid out is the mixer's business."""

    kind: str
    window: int = 0
    tensors: Tuple[Tuple[str, PageTensor], ...] = ()


@dataclass(frozen=True)
class StateRequest:
    """Fixed-size state a mixer keeps per request: one tensor of ``shape`` per slot."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerMemory:
    """What the cache manager binds to one run of a layer."""

    group: int = -1                       # cache group whose slots and block tables apply
    tensors: Dict[str, torch.Tensor] = field(default_factory=dict)   # name -> [pages, *page shape], as requested
    writes: bool = True
    state: Optional[torch.Tensor] = None  # [slots, *StateRequest.shape]


class Part:
    """Base of all parts."""

    kind: str = ""
    # A part whose forward only launches kernels that read device arrays (no copies to the host, no
    # launches whose number or size depends on the arrays' contents, no allocations after its first
    # calls) may set this.  When every part of a model does, steps of decoded tokens are captured as
    # graphs and replayed; a part that leaves the default keeps the whole model on eager launches.
    graph_safe: bool = False
    # A graph-safe part all of whose device work is calls into the kernel library (``ops``) with outputs in
    # buffers of the runtime, none through torch operators, may set this too.  When every part of a model
    # does, the library calls of a step are recorded the first time a shape comes and made again from native
    # code when it recurs, before (or without) a graph.
    tape_safe: bool = False

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        """parameter name -> what the checkpoint must hold for it."""
        return {}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        self.spec = spec
        self.rt = rt

    def tune(self, num_tokens: int) -> None:
        """Measure, outside of any step, which of several equivalent ways is faster for steps of
        ``num_tokens`` tokens and record the decision in ``rt.choices`` (``Engine.warm_up`` calls this).
        ``forward`` only reads ``rt.choices``; without an entry it takes a fixed default."""

    def step_rows(self, rows: int, kind: str) -> int:
        """The number of rows, at least ``rows``, that this part wants a step to be run with when the engine may
        pad it (so that the kinds of steps are few and recur, and so that the part's kernels meet numbers of
        rows they are built or were measured for).  ``kind`` says what is counted:
        "decode"  the entries of a step in which every entry brings one token;
        "portion" the tokens of one portion of a prompt;
        "beside"  the entries of one token beside portions of prompts;
        "mixed"   all rows of a step with portions.
        The engine takes the least number every part of the model accepts (``DecoderModel.step_rows``).  The
        default accepts every number."""
        return int(rows)


@dataclass
class HostBatch:
    """A step as a planner sees it, on the host: entry e brings ``entry_len[e]`` tokens (those added as
    padding included), the flat tokens ``entry_start[e]...``, after ``entry_past[e]`` tokens already in
    the cache.

    ``bound_single`` / ``bound_multi``: when a step is to be replayed as a graph, launch sizes must recur
    from step to step, so the engine gives upper bounds that do: no entry of one token (of several
    tokens) holds more than this many tokens once the step has run.  0: no bound is given, exact sizes
    are fine."""

    num_tokens: int
    num_entries: int
    entry_start: "np.ndarray"
    entry_len: "np.ndarray"
    entry_past: "np.ndarray"
    single_tokens: bool
    bound_single: int = 0
    bound_multi: int = 0


@dataclass
class StepPlan:
    """What a planner makes of a step: int32 index arrays, which travel to the device with the step's
    other arrays in the same copy (``dev`` then holds them under the same names), and launch sizes the
    host needs."""

    arrays: Dict[str, "np.ndarray"] = field(default_factory=dict)
    sizes: Dict[str, int] = field(default_factory=dict)
    dev: Dict[str, torch.Tensor] = field(default_factory=dict)


class StepPlanner:
    """Plans a mixer's launches for one step on the host.  A mixer whose kernels need index arrays or
    launch sizes derived from the step's entries returns one from ``Mixer.planner()``; planners with
    equal ``key`` are run once per step and share the plan (``batch.plans[key]``).  The names, the order
    and, for steps of equal (tokens, entries), the sizes of ``arrays`` must not depend on the step's
    contents beyond what ``sizes`` reports: a captured graph reads them at fixed places."""

    key: tuple = ()
    # In steps in which every entry brings one token the arrays depend on the number of entries only:
    # they need not be made again while the same requests go on decoding.
    fixed_for_single_tokens: bool = False

    def plan(self, hb: HostBatch) -> StepPlan:
        raise NotImplementedError

    def shape(self, entry_lens: Sequence[int], bound_single: int, bound_multi: int) -> tuple:
        """Everything of the entries' token counts (as the step runs them, padding included) that the sizes of
        this planner's arrays and launches depend on, beyond their number and their sum: steps that agree in it
        (and in the bounds, the number of entries and of tokens) can share a recorded graph or tape.  The default
        is the counts themselves; a planner whose plan depends on less says so."""
        return tuple(sorted(int(n) for n in entry_lens))


class Mixer(Part):
    """Mixes information across the tokens of a sequence.

    ``forward(x, batch, memory)`` takes the normed hidden states [n, hidden] of all tokens
    of the step and returns the addition to the residual stream: [n, hidden], or a stack
    [S, n, hidden] of float32 partial sums that the next norm adds in rising order (what
    the few-rows matrix product leaves when it is cut along k).  ``batch`` is the step's
    device-side description (``engine.batch.DeviceBatch``); ``memory`` is this run's
    ``LayerMemory``."""

    # To make the shapes of steps recur (so that they can be replayed as graphs) the engine may run an
    # entry of several tokens as if it brought more: tokens of id 0 at the positions that follow, with no
    # place in the cache (slot -1), whose results nobody reads; and it may add entries of one such token
    # that belong to no request (state slot 0, an empty block table).  A mixer for which that changes
    # nothing any real token sees sets this; one that keeps state per request must leave it False, or
    # the padding would advance its state.  One mixer that leaves it False keeps the whole model's steps
    # unpadded.
    padding_safe: bool = False

    def planner(self) -> Optional[StepPlanner]:
        """The planner of this mixer's launches, or None when its kernels need no more than the batch."""
        return None

    def cache_request(self) -> Optional[KVCacheRequest]:
        return None

    def state_request(self) -> Optional[StateRequest]:
        return None

    def forward(self, x: torch.Tensor, batch, memory: LayerMemory) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """``forward(x)``: [n, hidden] -> [n, hidden] (or a stack [S, n, hidden] of float32 partial
    sums, as for a mixer), token by token."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    """``forward(x)`` normalises rows; ``add_forward(resid, delta)`` first adds ``delta`` ([n, hidden],
    or a stack [S, n, hidden] of float32 partial sums, added in rising order) into the float32
    residual stream in place and returns the normalised sum."""

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        raise NotImplementedError

    def add_forward(self, resid: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """Encodes positions into queries and keys.  It transforms; what is stored where is the mixer's business.

    ``encode(q, k, positions, nh, nkv, d)`` encodes q [n, nh*d] and k [n, nkv*d] in place (either may be a
    column slice of a wider tensor).

    ``step_table(batch)`` lets a mixer fold the encoding into kernels of its own: an encoding that
    is a rotation of pairs (k, k + R/2) of the first R dims of every head returns the step's angles
    as a float32 tensor [n, R/2, 2] of (cos, sin), computed once per step and kept in
    ``batch.shared``; an encoding that does nothing returns the string "none"; every other encoding
    returns None (the default), and the mixer calls ``encode``.

    ``positions`` is what the step gives for each token: int32 [n], the token's index in its sequence,
    when ``position_axes`` is 1; with more axes int32 [n, position_axes], every axis the index in the
    sequence unless the caller of the step gave the entry positions of its own (``StepEntry.positions``)."""

    position_axes: int = 1

    def step_table(self, batch):
        return None

    def encode(self, q, k, positions, nh: int, nkv: int, d: int) -> None:
        raise NotImplementedError


class Block:
    """Arranges norms, a mixer and a feed-forward around the residual stream.  Built from
    (norms by name, mixer, feed_forward, runtime); ``norm_names`` lists the norms it needs.

    ``forward(resid, delta, batch, memory)``: ``resid`` is the float32 residual stream
    [n, hidden], ``delta`` a pending addition to it (or None; [n, hidden] or a stack
    [S, n, hidden] of float32 partial sums); returns the next pending addition.  The add is
    folded into the following norm."""

    norm_names: Tuple[str, ...] = ()

    def forward(self, resid, delta, batch, memory: LayerMemory):
        raise NotImplementedError
