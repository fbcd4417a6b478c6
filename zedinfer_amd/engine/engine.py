"""The engine: a model, its cache and the one step function.

``Engine.step(entries)`` runs exactly the tokens it is given, as one batch, from
the cache that earlier steps left, and returns float32 logits at the wanted
places (the reference returns logits for all rows and lets the caller slice,
reference: src/zedinfer/serving_loop.cpp:182-422,
src/frontend/models/transformer_forward.cpp:155-159).  It grows each request's
block tables before the run and commits the new lengths after it.
"""
from __future__ import annotations

import os
from typing import Dict, Optional, Sequence

import torch

from .. import ops
from ..cache.manager import NO_GROWTH, CacheManager, SequenceCache
from ..config import ModelConfig, ModelForwardConfig, SchedulerConfig, load_config
from ..models import DecoderModel, expected_weights
from ..parts import Runtime
from ..sampling.sampler import default_sampling
from ..weights import load_weights, random_weights
from ..ops.tape import Recording
from .batch import DecodeImage, StagingRing, StepEntry, build_device_batch

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           "f32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.float32, torch.bfloat16):
            raise ValueError(f"engine dtype must be float32 or bfloat16, got {name}")
        return name
    if str(name) not in _DTYPES:
        raise ValueError(f"unknown dtype {name!r}; choose bfloat16 or float32")
    return _DTYPES[str(name)]


def require_gpu() -> torch.device:
    """The engine runs on the GPU only; there is no CPU path."""
    if not torch.cuda.is_available():
        raise RuntimeError("zedinfer_amd needs a GPU (torch.cuda.is_available() is False); "
                           "there is no CPU fallback")
    ops.load()
    return torch.device("cuda", torch.cuda.current_device())


class Engine:
    def __init__(self, fc: ModelForwardConfig, weights: Dict[str, torch.Tensor], dtype: torch.dtype,
                 sched: Optional[SchedulerConfig] = None, device: Optional[torch.device] = None):
        self.device = device or require_gpu()
        self.dtype = parse_dtype(dtype)
        self.sched = sched or SchedulerConfig()
        self.sched.validate()
        self.fc = fc
        self.rt = Runtime(self.device, self.dtype)
        self.model = DecoderModel(fc, weights, self.rt)
        kv = self.model.cache_requests()
        num_pages = self.sched.num_kv_blocks or self._pages_from_free_memory(kv)
        self.cache = CacheManager(kv, self.model.state_requests(), num_pages, self.sched.kv_block_size,
                                  self.sched.max_batch_requests, self.dtype, self.device,
                                  max_step_tokens=self.sched.max_batch_tokens)
        self.memories = self.cache.memories(fc.schedule)
        self.vocab_size = fc.vocab_size
        self.steps_run = 0
        self.default_sampling = None      # what requests without sampling options use (None: greedy)
        self.staging = StagingRing(self.device)
        # Steps of single decoded tokens are captured as HIP graphs and replayed, one graph per
        # (entries, wanted rows, block-table widths, attention launch size).
        self.use_graphs = (self.device.type == "cuda" and self.model.graph_safe()
                           and os.environ.get("ZEDINFER_DISABLE_GRAPHS", "0") in ("", "0"))
        # Before a shape has a graph (or when graphs are off, or for prompt portions too long to be worth one) its
        # second and later steps run from a tape of the first's library calls: the host then spends what the
        # launches cost, not the interpreter's time for every part (about 5 ms for 28 layers).
        self.use_tapes = (self.device.type == "cuda" and self.model.tape_safe()
                          and os.environ.get("ZEDINFER_DISABLE_TAPES", "0") in ("", "0"))
        self.tape_runs = 0
        self.graph_max_entries = 256     # measured: 128 requests decode 77% faster as a graph, 256 37%
        self.graph_limit = 48
        self.graph_after = int(os.environ.get("ZEDINFER_GRAPH_AFTER", "6"))   # steps of a kind before it is captured
        self._graphs: Dict[tuple, "_DecodeGraph"] = {}
        self.graph_replays = 0
        # A step that is one portion of one prompt, alone or beside single decoded tokens, has the portion
        # padded to a number of tokens that the model's parts choose (``step_rows``) and is captured too (launching a step
        # kernel by kernel costs the host about 5 ms, more than the GPU needs for a short prompt), one graph
        # per (entries, padded tokens, wanted rows, table widths, attention launch sizes).  Portions of
        # more tokens are bound by the GPU and run as they are.
        self.prompt_graph_max_tokens = int(os.environ.get("ZEDINFER_PROMPT_GRAPH_MAX_TOKENS", "1024"))
        self.prompt_graph_limit = 128    # shapes held; the one used longest ago goes first
        self._prompt_graphs: Dict[tuple, "_DecodeGraph"] = {}
        self.prompt_graph_replays = 0
        # what the batch is built with: the planners of the mixers' launches, the axes of the position
        # encodings, and whether steps may be padded (every mixer must say that padding is harmless to it)
        self.planners = self.model.planners()
        self.position_axes = self.model.position_axes()
        self.padding_safe = self.model.padding_safe()
        # The parts' choices (``Part.tune``) for a number of rows are measured the first time a step of that many
        # rows is about to run, between steps, when this is set (``InferenceEngine`` sets it): an engine is then
        # made at once, and a size costs its measurement when it first comes instead of every possible size
        # costing it before the first request.
        self.tune_when_scheduled = False
        self._tuned_rows: set = set()
        self._tapes_checked: Dict[tuple, bool] = {}     # kinds of steps whose first tape has been held against its own step: did it repeat it

    # ---- construction ------------------------------------------------------------
    @classmethod
    def from_folder(cls, folder: str, dtype="bfloat16", sched: Optional[SchedulerConfig] = None) -> "Engine":
        """Load config.json and the safetensors of ``folder``; the model class comes from config.json."""
        device = require_gpu()
        arch, cfg = load_config(folder)
        fc = arch.forward_config(cfg)
        dt = parse_dtype(dtype)
        weights = load_weights(folder, expected_weights(fc), dt, device)
        engine = cls(fc, weights, dt, sched, device)
        engine.default_sampling = default_sampling(folder)
        return engine

    @classmethod
    def from_config(cls, cfg: ModelConfig, arch_name: Optional[str] = None, dtype="bfloat16", seed: int = 0,
                    sched: Optional[SchedulerConfig] = None, noisy_norms: bool = False) -> "Engine":
        """A model with seeded random weights made on the device (no files)."""
        from ..config.registry import find_architecture
        device = require_gpu()
        arch = find_architecture({"architectures": [arch_name] if arch_name else list(cfg.architectures),
                                  "model_type": cfg.model_type})
        fc = arch.forward_config(cfg)
        dt = parse_dtype(dtype)
        weights = random_weights(expected_weights(fc), seed, dt, device, noisy_norms=noisy_norms)
        return cls(fc, weights, dt, sched, device)

    def _pages_from_free_memory(self, kv) -> int:
        """Pool size from free device memory (reference: src/zedinfer/engine.cpp:949-995), capped by
        what max_batch_requests sequences of max_seq_len tokens could ever use."""
        per_page = max(1, CacheManager.bytes_per_page(kv, self.sched.kv_block_size, self.dtype))
        free, total = torch.cuda.mem_get_info(self.device)
        budget = int(free - (1.0 - self.sched.gpu_memory_utilization) * total)
        pages = max(16, budget // per_page)
        cap = self.sched.max_batch_requests * (-(-self.sched.max_seq_len // self.sched.kv_block_size))
        return int(min(pages, cap))

    def with_cache(self, sched: SchedulerConfig) -> "Engine":
        """Another engine over the same model and weights with a cache pool of its own (``sched``
        sizes it); the two must not run steps at the same time, they share workspaces."""
        sched.validate()
        other = Engine.__new__(Engine)
        other.__dict__.update(self.__dict__)
        other.sched = sched
        kv = self.model.cache_requests()
        other.cache = CacheManager(kv, self.model.state_requests(), sched.num_kv_blocks or self._pages_from_free_memory(kv),
                                   sched.kv_block_size, sched.max_batch_requests, self.dtype, self.device,
                                   max_step_tokens=sched.max_batch_tokens)
        other.memories = other.cache.memories(self.fc.schedule)
        other.staging = StagingRing(self.device)
        other._graphs = {}
        other._prompt_graphs = {}
        other.steps_run = other.graph_replays = 0
        return other

    # ---- decisions made outside of steps ---------------------------------------------
    def warm_up(self, step_sizes: Sequence[int] = (), choices: Optional[Dict[tuple, object]] = None
                ) -> Dict[tuple, object]:
        """Let every part decide, for steps of the given numbers of tokens, between ways of computing the
        same thing that differ in speed and by rounding (``Part.tune``); nothing of the kind is decided
        while a step runs.  ``choices`` (what an earlier call returned) are taken as they are, which makes
        a run repeat another's bits.  Returns all decisions in force."""
        if choices:
            self.rt.choices.update(choices)
        for n in step_sizes:
            for part in self.model.parts:
                part_tune = getattr(part, "tune", None)
                if part_tune is not None:
                    part_tune(int(n))
        self._tuned_rows.update(int(n) for n in step_sizes)
        if step_sizes:
            torch.cuda.synchronize(self.device)
        return dict(self.rt.choices)

    def _tune_if_new(self, rows: int) -> None:
        """Before a step of ``rows`` rows runs (never inside one): the parts' choices for that many rows, once."""
        if self.tune_when_scheduled and rows not in self._tuned_rows:
            self.warm_up([rows])

    # ---- requests ------------------------------------------------------------------
    def open(self, request_id, expected_tokens: int = 0) -> SequenceCache:
        return self.cache.open(request_id, expected_tokens)

    def close(self, seq: SequenceCache) -> None:
        self.cache.close(seq)

    # ---- the step ------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], copy: bool = True,
             token_source: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run one batch.  Returns float32 logits [wanted, vocab] in the order of the entries and
        of each entry's ``want`` (None when nothing is wanted).  With ``copy`` False the result is
        a view of a workspace that the next step overwrites.  Raises OutOfPages, with no
        request's length changed, when the pool cannot hold the new tokens.

        ``token_source``: an int32 device tensor [k], k <= entries.  The first k entries then bring one token
        each whose value is read from there on the device (``tokens`` holds a placeholder), so that a step can
        be queued before the host has seen what the step before it sampled."""
        single = all(len(e.tokens) == 1 for e in entries)
        if token_source is not None:
            k = token_source.shape[0] if token_source.dim() == 1 else -1
            if token_source.dtype != torch.int32 or token_source.device != self.device or not (0 < k <= len(entries)):
                raise ValueError(f"token_source must be an int32 tensor of at most {len(entries)} entries on {self.device}")
            if any(len(e.tokens) != 1 for e in entries[:k]):
                raise ValueError("tokens can come from the device only for entries that bring one token")
        grown = []
        try:
            for e in entries:
                growth = self.cache.ensure(e.seq, e.seq.length + len(e.tokens))
                if growth is not NO_GROWTH:
                    grown.append((e.seq, growth))
            if (self.use_graphs or self.use_tapes) and 0 < len(entries) <= self.graph_max_entries and single:
                logits = self._graph_step(entries, token_source)
            elif (self.use_graphs or self.use_tapes) and self._one_portion(entries):
                logits = self._prompt_graph_step(entries, token_source)
            else:
                self._tune_if_new(sum(len(e.tokens) for e in entries))
                batch = build_device_batch(entries, self.cache, self.vocab_size, self.device, self.staging,
                                           planners=self.planners, position_axes=self.position_axes)
                if token_source is not None:        # the entries' tokens lie in their order: the first k are the first k tokens
                    batch.token_ids[:token_source.shape[0]].copy_(token_source, non_blocking=True)
                logits = self.model.run(batch, self.memories)
        except BaseException:
            # nothing of a step that did not run to its end stays: the pages and promises it took go back, no
            # length has changed (what a step that failed half-way wrote lies beyond every length)
            for seq, growth in reversed(grown):
                self.cache.undo(seq, growth)
            for dg in self._graphs.values():       # a host image may have been rewritten half-way: made again next time
                dg.image = None
            raise
        for e in entries:
            self.cache.commit(e.seq, e.seq.length + len(e.tokens))
        self.steps_run += 1
        return logits.clone() if (copy and logits is not None) else logits

    # ---- decode steps as graphs ------------------------------------------------------
    def _graph_step(self, entries: Sequence[StepEntry], token_source: Optional[torch.Tensor] = None
                    ) -> Optional[torch.Tensor]:
        """A step in which every entry brings one token.  Its launches depend on the number of entries
        and wanted rows, on the width of the block tables and on the size of the attention launch
        only: the first step of a kind runs eagerly and is captured, later ones replay the graph
        after the step's index arrays have been copied into the graph's buffer."""
        E = len(entries)
        wanted = R = sum(len(e.want) for e in entries)
        more_entries = 0
        if self.padding_safe and (self.use_graphs or self.use_tapes):
            # the number of requests moves (they end one by one): entries that belong to no request bring it to
            # one of few numbers, a row wanted of each, so that the kinds of steps are few
            more_entries = self.model.step_rows(E, "decode") - E
            E += more_entries
            # (an entry may name its one token several times: more rows than entries are left as they are)
            R = E if 0 < wanted <= E else wanted
        self._tune_if_new(E)
        widths = tuple(_pow2_at_least(max(len(e.seq.pages[g]) for e in entries), 8)
                       for g in range(len(self.cache.groups)))
        # a bound, the same for many steps, of the tokens any sequence holds after this step: the
        # mixers' planners size their launches by it
        bound = _bucket_at_least(max(e.seq.length for e in entries) + 1, 256)
        # (whether every token's row is wanted, in order, decides if the model picks rows at all: such steps and
        # steps that want some rows only, or rows of padding entries, are different kinds)
        every_row = more_entries == 0 and all(len(e.want) == 1 for e in entries)
        key = (E, R, widths, bound, every_row)
        dg = self._graphs.pop(key, None)
        if dg is not None:
            self._graphs[key] = dg              # used last: the last to go
        else:
            if len(self._graphs) >= self.graph_limit:
                self._drop_oldest(self._graphs)
            dg = self._graphs[key] = _DecodeGraph()
        if dg.image is not None and dg.image.matches(entries):
            batch = dg.image.refresh(entries)      # the same sequences go on: only what changed is rewritten
        else:
            dg.image = DecodeImage(entries, self.cache, self.vocab_size, self.device, self.staging, widths, dg.buffer,
                                   planners=self.planners, position_axes=self.position_axes, bound_single=bound,
                                   pad_entries=more_entries, pad_rows=R - wanted)
            dg.buffer = dg.image.static         # the first step's buffer serves all later ones of the shape
            batch = dg.image.batch
        if token_source is not None:
            batch.token_ids[:token_source.shape[0]].copy_(token_source, non_blocking=True)
        logits = self._decode_step(dg, batch)
        return logits[:wanted] if (logits is not None and R != wanted) else logits      # the requests' rows come first

    def _decode_step(self, dg: "_DecodeGraph", batch) -> Optional[torch.Tensor]:
        if dg.graph is not None:
            dg.graph.replay()
            self.graph_replays += 1
            return dg.logits
        # the first step of a kind runs part by part (it allocates every workspace), the second is recorded as a
        # tape, and a kind that keeps coming is captured as a graph (capturing costs about ten steps: kinds that
        # come a few times only, as while a batch of requests ends one by one, stay with their tape)
        logits = self._run_or_replay(dg, batch)
        dg.seen += 1
        if self.use_graphs and dg.seen >= (self.graph_after if self.use_tapes and not dg.no_tape else 2):
            torch.cuda.synchronize(self.device)
            first = logits.clone() if logits is not None else None
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                dg.logits = self.model.run(batch, self.memories)
            dg.graph = g
            return first
        return logits

    def _run_or_replay(self, dg: "_DecodeGraph", batch) -> Optional[torch.Tensor]:
        """A step of a shape that has no graph: from the shape's tape when it has one, else part by part, recorded
        as its tape on the way.  A recording during which device memory was taken is dropped (the memory would be
        another's at the next run): that is the rule at a shape's first step when workspaces still grow, and the
        step is then recorded again the next time; a second such recording marks the shape as one that cannot be
        taped.  The batch lives in the shape's own buffer, as for a graph."""
        self._same_plans(dg, batch)
        if dg.tape is not None:
            dg.tape.run()
            self.tape_runs += 1
            return dg.logits
        if not self.use_tapes or dg.no_tape:
            dg.ran = True
            return self.model.run(batch, self.memories)
        with Recording(self.device) as rec:
            logits = self.model.run(batch, self.memories)
        if rec.allocations:
            dg.no_tape = dg.ran       # at the first step workspaces may still get their sizes
        else:
            tape = rec.tape()
            if tape is None:
                dg.no_tape = True
            elif self._tape_repeats_the_step(tape, logits, batch):
                dg.tape, dg.logits = tape, logits
            else:
                dg.no_tape = True
                logits = self.model.run(batch, self.memories)     # what the failed replay left in cache and workspaces is made again
        dg.ran = True
        return logits

    def _tape_repeats_the_step(self, tape, logits: Optional[torch.Tensor], batch) -> bool:
        """A new tape is run once, right after the step it was recorded from and on the same inputs, with every
        floating-point workspace of the runtime (the logits among them) made NaN before, and must leave the same
        logits bit for bit: device work that is no call into the kernel library (a torch operator in a part that
        says ``tape_safe``) is not on the tape, its result would be stale at every replay, and here it is NaN.  A
        model with state per request is not run twice (the second run would advance the state): its tapes are
        trusted as before.  The check costs a step; it is made for the first tape of every kind of step (single
        tokens or portions; up to 16, 64, 128 or more rows: where the parts take different ways), not for every
        shape."""
        if logits is None or self.model.state_requests():
            return True
        n = batch.num_tokens
        kind = (bool(batch.single_tokens), 0 if n <= 16 else 1 if n <= 64 else 2 if n <= 128 else 3)
        if kind in self._tapes_checked:
            return self._tapes_checked[kind]         # what the kind's first tape showed holds for the others
        self._tapes_checked[kind] = True
        first = logits.clone()
        self.rt.poison()
        logits.fill_(float("nan"))
        tape.run()
        same = bool(torch.equal(first, logits))
        if not same:
            self._tapes_checked[kind] = False
            import logging
            logging.getLogger("zedinfer_amd").warning(
                "a recorded step does not repeat its logits: some device work of the model is not a call into the "
                "kernel library; steps of this shape run part by part")
        return same


    @staticmethod
    def _same_plans(dg: "_DecodeGraph", batch) -> None:
        """A recorded step fixes its launches: the sizes that the mixers' planners gave its first step must be what
        they give every later step of the shape (``StepPlanner.shape`` has to name all that they depend on)."""
        planned = {key: (tuple(sorted(plan.sizes.items())), tuple((name, int(a.size)) for name, a in plan.arrays.items()))
                   for key, plan in batch.plans.items()}
        if dg.planned is None:
            dg.planned = planned
        elif planned != dg.planned:
            raise RuntimeError(f"a step of a recorded shape plans its launches differently: {planned} against {dg.planned}")

    def _drop_oldest(self, graphs: Dict[tuple, "_DecodeGraph"]) -> None:
        """Forget the first graph of the dictionary.  One that was recorded may still be running, and with
        it goes the memory it was recorded with: the device is waited for first (this is rare)."""
        dg = graphs.pop(next(iter(graphs)))
        if dg.graph is not None:
            torch.cuda.synchronize(self.device)

    # ---- portions of prompts as graphs and tapes -------------------------------------------
    def portion_rows(self, tokens: int) -> int:
        """The tokens a portion of ``tokens`` tokens is run with when the step is padded (the parts' choice)."""
        return self.model.step_rows(tokens, "portion")

    # padded tokens of the portions of a step that is still padded and run from a tape (a step of many tokens does
    # not need the tape, the GPU takes far longer than the host, but its padded rows are a size whose library
    # products can have been measured)
    TAPE_MAX_TOKENS = 32768

    def _one_portion(self, entries: Sequence[StepEntry]) -> bool:
        """Portions of prompts (entries of several tokens) of a size worth a graph together, beside any
        number of single decoded tokens; at most one row wanted of each.  Such steps are padded, so every
        mixer must have said that padding is harmless to it."""
        if not self.padding_safe:
            return False
        total = real = 0
        for e in entries:
            n = len(e.tokens)
            if len(e.want) > 1 or e.positions is not None:
                return False
            if n > 1:
                total += self.portion_rows(n)
                real += n
        most = max(self.prompt_graph_max_tokens if self.use_graphs else 0, self.TAPE_MAX_TOKENS if self.use_tapes else 0)
        # many very short portions would be padded to many times their tokens: such a step runs as it is
        return 0 < total <= most and total <= 4 * real + self.portion_rows(2) and len(entries) <= self.graph_max_entries

    def _prompt_graph_step(self, entries: Sequence[StepEntry], token_source: Optional[torch.Tensor] = None
                           ) -> Optional[torch.Tensor]:
        """A step of portions of prompts (entries of several tokens) beside single decoded tokens,
        with every portion run as if it brought the number of tokens the model's parts round it up to (see
        ``build_device_batch``): the first step of a kind runs eagerly, the second is captured, later
        ones replay."""
        portions = [e for e in entries if len(e.tokens) > 1]
        sizes = tuple(sorted(self.portion_rows(len(e.tokens)) for e in portions))     # tokens of the portions, padded
        padded = sum(sizes)
        wanted = sum(len(e.want) for e in entries)
        E, R, more_entries = len(entries), wanted, 0
        if E > 1:
            # the numbers of portions and of decoding requests move from step to step: the decoding entries are
            # brought to a number the parts choose with entries that belong to no request, and a row is wanted of
            # every entry: fewer shapes, and the step's rows are among the numbers that a warm-up has measured
            # the parts' choices for (``InferenceEngine.default_warm_up_sizes``).
            decoding = E - len(portions)
            more_entries = self.model.step_rows(decoding, "beside") - decoding if decoding else 0
            E += more_entries
            R = E
        # the parts may want the whole step's rows rounded up further (measured sizes lie further apart for large
        # steps): more padding behind the longest portion
        rows = padded + (E - len(portions))
        more_tokens = self.model.step_rows(rows, "mixed") - rows
        if more_tokens:
            sizes = tuple(sorted(sizes[:-1] + (sizes[-1] + more_tokens,)))
            padded += more_tokens
        self._tune_if_new(rows + more_tokens)
        widths = tuple(_pow2_at_least(max(len(e.seq.pages[g]) for e in entries), 8)
                       for g in range(len(self.cache.groups)))
        long_bucket = _pow2_at_least(max(e.seq.length + self.portion_rows(len(e.tokens)) for e in portions) + more_tokens, 2048)
        # (a power of two here: beside portions of prompts the decoding requests' attention is a small part of the
        # step, and every further value of the bound is a further kind of step)
        short_bucket = _pow2_at_least(max([e.seq.length + 1 for e in entries if len(e.tokens) == 1], default=0), 256)
        singles = len(entries) - len(portions) + more_entries
        # everything the launches' sizes depend on: the tokens of the step, and what of the portions' sizes one by
        # one the planners say their plans depend on (tiles are cut portion by portion, by rules of their own)
        entry_lens = sizes + (1,) * singles
        shapes = tuple(pl.shape(entry_lens, short_bucket if singles else 0, long_bucket) for pl in self.planners)
        key = (E, singles, padded, shapes, R, widths, long_bucket, short_bucket)
        dg = self._prompt_graphs.pop(key, None)
        if dg is not None:
            self._prompt_graphs[key] = dg       # used last: the last to go
        else:
            if len(self._prompt_graphs) >= self.prompt_graph_limit:
                self._drop_oldest(self._prompt_graphs)
            dg = self._prompt_graphs[key] = _DecodeGraph()
        batch = build_device_batch(entries, self.cache, self.vocab_size, self.device, self.staging, widths, dg.buffer,
                                   pad_to=self.portion_rows, pad_more=more_tokens, pad_entries=more_entries, pad_rows=R - wanted,
                                   planners=self.planners, position_axes=self.position_axes,
                                   bound_single=short_bucket if singles else 0, bound_multi=long_bucket)
        dg.buffer = batch.device_image          # the first step's buffer serves all later ones of the shape
        if token_source is not None:
            batch.token_ids[:token_source.shape[0]].copy_(token_source, non_blocking=True)
        if dg.graph is not None:
            self._same_plans(dg, batch)
            dg.graph.replay()
            self.prompt_graph_replays += 1
            return dg.logits[:wanted] if wanted else None
        logits = self._run_or_replay(dg, batch)
        dg.seen += 1
        # Capturing a graph costs about as much as ten steps: a portion alone is captured the second time its
        # shape comes, a shape with decoded tokens beside the portion only the third time; portions too long
        # to be worth a graph (the GPU needs longer for them than the host) stay with their tape.
        if self.use_graphs and padded <= self.prompt_graph_max_tokens and dg.seen >= (2 if len(entries) == 1 else 3):
            torch.cuda.synchronize(self.device)
            first = logits.clone() if logits is not None else None
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                dg.logits = self.model.run(batch, self.memories)
            dg.graph = g
            logits = first
        return logits[:wanted] if (wanted and logits is not None) else None


class _DecodeGraph:
    def __init__(self):
        self.buffer: Optional[torch.Tensor] = None      # the device buffer of the step's index arrays
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None
        self.seen = 0
        self.ran = False                                # a step of the shape has run part by part
        self.tape = None                                # the library calls of one step of the shape
        self.no_tape = False                            # a step of the shape cannot be recorded
        self.planned = None                             # the sizes the planners gave the shape's first step
        self.image: Optional[DecodeImage] = None


def _bucket_at_least(n: int, floor: int = 1) -> int:
    """A bound of the tokens a decoding sequence holds that many steps share: a power of two up to 1,024, then
    the next multiple of 512 (of 2,048 beyond 8,192).  The attention launch is sized by it, and workgroups
    for keys that no sequence has yet cost time: with powers of two alone a batch just past 2,048 tokens
    launched twice the workgroups it needed."""
    if n <= 1024:
        return _pow2_at_least(n, floor)
    step = 512 if n <= 8192 else 2048
    return max(-(-n // step) * step, floor)


def _pow2_at_least(n: int, floor: int = 1) -> int:
    v = max(int(floor), 1)
    while v < n:
        v *= 2
    return v
