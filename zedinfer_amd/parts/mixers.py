"""Token mixers."""
from __future__ import annotations

import math
from typing import Dict, Optional

import numpy as np
import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import (PAGE, HostBatch, KVCacheRequest, LayerMemory, Mixer, PageTensor, POSITION_ENCODINGS, Runtime, StepPlan,
                   StepPlanner, register_mixer)
from .rows import ProductRows
from .feed_forward import stack_rows

SHORT_ENTRY = 4     # entries of up to this many tokens are attended token by token, split over the keys
LONG_TILE = 64      # longer entries are cut into tiles of this many queries for the prompt kernel (or 128: see below)


class AttentionPlanner(StepPlanner):
    """How the attention kernels divide a step: tokens of entries that bring at most SHORT_ENTRY tokens
    ("decoded" tokens) go, one by one, to the kernel that splits a query's keys over many wavefronts;
    longer entries are cut into tiles of queries for the prompt kernel, the tile that sees most keys first.

    Tiles hold LONG_TILE queries, or ``wide_tile`` (twice as many, where the mixer's prompt kernel takes them:
    a block of keys staged on the chip then serves twice the queries) when the step is large enough to fill
    the chip with those: measured with 28 layers of the 1.5B sizes (12 heads), 16,384 tokens of one prompt run
    88 against 99 ms with the wide tiles, 8,192 tokens 33.7 against 37.0, 3,072 tokens 12.8 against 13.3, and
    2,048 tokens 9.2 against 9.1 ms; with 28 heads 2,048 tokens gain 2%.  Larger steps still take the wide tiles
    in workgroups of four wavefronts, two to a compute unit (``alone``: 16,384 tokens 83 against 86.4 ms, 4,096
    tokens 16.0 against 16.4; the result differs by rounding).  The choice is a function of the entries' (padded) lengths
    and of the bound of their keys, so that a recorded step meets the same one again.

    arrays: ``short_idx`` / ``long_idx``, the flat indices of the tokens of either kind; ``tile_entry`` /
    ``tile_off``: tile i covers tokens [tile_off[i], tile_off[i] + tile) of entry tile_entry[i].
    sizes: ``num_short``, ``num_long``, ``num_tiles``, ``tile``, ``alone``; ``max_short_keys`` / ``max_long_keys``: an upper
    bound of the keys a token of either kind sees (its position + 1), which sizes the launches."""

    fixed_for_single_tokens = True
    # Workgroups of wide tiles from which they pay: one and a half a compute unit (384 on the 256 of an MI355X);
    # and from which workgroups of four wavefronts, two to a compute unit, pay (``alone``): three a compute unit.
    # FILL / FILL_ALONE, when set, stand for the products (tests set them).
    FILL_PER_UNIT, FILL_ALONE_PER_UNIT = 1.5, 3.0
    FILL = FILL_ALONE = None
    CUT_KEYS = 2048     # a tile's keys are cut over several workgroups every so many

    def __init__(self, wide_tile: int = LONG_TILE, heads: int = 1):
        self.wide_tile, self.heads = int(wide_tile), int(heads)
        self.key = ("attention", SHORT_ENTRY, self.wide_tile, self.heads)
        self.units = compute_units()

    def plan(self, hb: HostBatch) -> StepPlan:
        lens, past = hb.entry_len, hb.entry_past
        short = lens <= SHORT_ENTRY
        short_tok = np.repeat(short, lens)
        flat = np.arange(hb.num_tokens, dtype=np.int32)
        short_idx, long_idx = flat[short_tok], flat[~short_tok]
        ends = past + lens
        max_short = int(ends[short].max()) if short_idx.size else 0
        max_long = int(ends[~short].max()) if long_idx.size else 0
        if short_idx.size and (hb.bound_single or hb.bound_multi):
            # bounds that recur from step to step (the step is replayed as a graph)
            several = bool((lens[short] > 1).any())
            max_short = max(hb.bound_single if bool((lens[short] == 1).any()) else 0,
                            hb.bound_multi if several else 0, 1)
        if long_idx.size and hb.bound_multi:
            max_long = hb.bound_multi
        tile, alone = self._tile([int(n) for n in lens[~short]], max_long)
        tiles = [(int(past[i]) + off + min(tile, int(lens[i]) - off), i, off)
                 for i in range(hb.num_entries) if not short[i] for off in range(0, int(lens[i]), tile)]
        tiles.sort(key=lambda t: -t[0])
        return StepPlan(
            arrays={"short_idx": short_idx, "long_idx": long_idx,
                    "tile_entry": np.array([t[1] for t in tiles], dtype=np.int32),
                    "tile_off": np.array([t[2] for t in tiles], dtype=np.int32)},
            sizes={"num_short": int(short_idx.size), "num_long": int(long_idx.size), "num_tiles": len(tiles),
                   "tile": tile, "alone": alone, "max_short_keys": max_short, "max_long_keys": max_long})


    def _tile(self, long_lens, max_long: int):
        """(queries a tile, workgroups of four wavefronts) for portions of these many tokens whose keys are bounded
        by ``max_long``: the wide tile when that many workgroups still fill the chip."""
        tile, alone = LONG_TILE, False
        if self.wide_tile > LONG_TILE and long_lens:
            wide = int(sum(-(-int(n) // self.wide_tile) for n in long_lens))
            groups = wide * -(-max_long // self.CUT_KEYS) * self.heads
            if groups >= (self.FILL if self.FILL is not None else self.FILL_PER_UNIT * self.units):
                tile = self.wide_tile
                alone = groups >= (self.FILL_ALONE if self.FILL_ALONE is not None else self.FILL_ALONE_PER_UNIT * self.units)
        return tile, alone

    def shape(self, entry_lens, bound_single: int, bound_multi: int) -> tuple:
        """The tile, and how many tiles and short tokens there are: how the tokens are dealt out over the portions
        matters no further (tiles of 64 queries: not at all, for portions that are multiples of 64)."""
        long_lens = [int(n) for n in entry_lens if n > SHORT_ENTRY]
        tile, alone = self._tile(long_lens, int(bound_multi))
        return (tile, alone, sum(-(-n // tile) for n in long_lens), sum(int(n) for n in entry_lens if n <= SHORT_ENTRY))


_PLANNERS: Dict[tuple, AttentionPlanner] = {}


def compute_units() -> int:
    """The device's compute units (an MI355X's 256 where no device can be asked: planning on the host alone)."""
    return ops.compute_units() if torch.cuda.is_available() else 256


def attention_cache_request(kind: str, num_kv_heads: int, head_dim: int, window: int = 0) -> KVCacheRequest:
    """What the attention kernels keep in a page: keys as [kv_head][slot][head_dim], values transposed as
    [kv_head][head_dim][slot] (a run of positions of one value dim is contiguous, which is the order the matrix
    cores read P.V in)."""
    return KVCacheRequest(kind, int(window), (("k", PageTensor((int(num_kv_heads), PAGE, int(head_dim)))),
                                              ("v", PageTensor((int(num_kv_heads), int(head_dim), PAGE)))))


def attention_planner(wide_tile: int, heads: int) -> AttentionPlanner:
    """One planner per (widest tile, heads): mixers that agree in both share a plan."""
    if (wide_tile, heads) not in _PLANNERS:
        _PLANNERS[(wide_tile, heads)] = AttentionPlanner(wide_tile, heads)
    return _PLANNERS[(wide_tile, heads)]


@register_mixer("attention")
class Attention(Mixer):
    """Causal grouped-query attention over the paged cache.

    q/k/v projections (with biases when ``qkv_bias``), position encoding of q and k, keys
    and values stored to the cache, attention of every token over the cached positions it
    may see, output projection without bias (reference:
    src/frontend/models/transformer_forward.cpp:71-112; the scale 1/sqrt(head_dim) at :31).
    The three projections are stacked into one [Qd + 2 KVd, H] matrix at load.

    params: hidden_size, num_heads, num_kv_heads, head_dim, qkv_bias, window (0: all keys),
    scale (default 1/sqrt(head_dim)), position (a PartSpec of a position encoding), qk_norm (an RMS norm
    over head_dim of every query and key head before the position encoding, gains ``q_norm`` and ``k_norm``
    [head_dim], eps ``qk_norm_eps``; reference: transformer_forward.cpp:80-96.  The architecture built here
    has none; the three projections then run one by one and the one-kernel decode path is not taken)."""

    graph_safe = True
    tape_safe = True
    padding_safe = True      # padding has no place in the cache, and causal attention lets no real token see it
    # Every workgroup of the fused kernel adds and rotates its token's query again (one per chunk of
    # 256 keys), which costs more than the separate rotary kernel once many tokens decode together:
    # measured faster at 1 and 8 tokens, slower at 64.
    FUSED_DECODE_MAX_TOKENS = 16
    # ... and once the launch (tokens x key/value heads x chunks of the keys) is more workgroups than the chip
    # holds at a time (two a compute unit, FUSED_DECODE_WORKGROUPS_PER_UNIT; FUSED_DECODE_MAX_WORKGROUPS, when set,
    # stands for the product): the workgroups of a second round pay the three dependent trips to
    # memory that come before their keys once more.  Measured at the 1.5B sizes, fused against separate kernels:
    # 8 tokens at 2,048 keys (176 workgroups) 1.47 against 1.54 ms a step, 12 at 4,096 (456) 1.72 against 1.76;
    # 8 at 8,192 (656) 1.98 against 1.87, 16 at 8,192 (1,312) 2.43 against 2.21; the 7B and 32B sizes turn over
    # between 352 and 704 workgroups as well.
    FUSED_DECODE_WORKGROUPS_PER_UNIT = 2
    FUSED_DECODE_MAX_WORKGROUPS = None
    # The one-kernel decode path leaves its chunks unmerged and the output projection merges them as it
    # loads its operand: one launch less a layer.  That kernel does not stream a large weight as well as
    # the plain product does (measured: 6.9 against 4.4 + 3.7 us with 4.7 MB of weight, 31.7 against
    # about 16 us with 52 MB), so it is taken for small output weights only.
    PROJECT_FROM_CHUNKS_MAX_BYTES = 8 << 20

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        p = spec.params
        H, nh, nkv, d = int(p["hidden_size"]), int(p["num_heads"]), int(p["num_kv_heads"]), int(p["head_dim"])
        w = {"q": WeightSpec((nh * d, H)), "k": WeightSpec((nkv * d, H)), "v": WeightSpec((nkv * d, H)),
             "o": WeightSpec((H, nh * d))}
        if p.get("qkv_bias", False):
            w.update({"q_bias": WeightSpec((nh * d,)), "k_bias": WeightSpec((nkv * d,)),
                      "v_bias": WeightSpec((nkv * d,))})
        if p.get("qk_norm", False):
            w.update({"q_norm": WeightSpec((d,), init="ones"), "k_norm": WeightSpec((d,), init="ones")})
        return w

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nh, self.nkv, self.d = int(p["num_heads"]), int(p["num_kv_heads"]), int(p["head_dim"])
        if self.nh % self.nkv:
            raise ValueError(f"attention: {self.nh} heads are not a multiple of {self.nkv} key/value heads")
        # any head size: the matrix-core kernels take multiples of 16 up to 128, the plain ones the rest
        self.window = int(p.get("window", 0) or 0)
        self.scale = float(p.get("scale") or 1.0 / math.sqrt(self.d))
        self.qd, self.kvd = self.nh * self.d, self.nkv * self.d
        pos_spec: PartSpec = p["position"]
        self.position = POSITION_ENCODINGS.get(pos_spec.kind)(pos_spec, {}, rt)
        mats = [weights["q"], weights["k"], weights["v"]]
        self.qkv = stack_rows(mats)
        self.mats = None if self.qkv is not None else mats
        self.bias = self.biases = None
        if p.get("qkv_bias", False):
            bs = [weights["q_bias"], weights["k_bias"], weights["v_bias"]]
            if self.qkv is not None and all(b.dtype == self.qkv.dtype for b in bs):
                self.bias = torch.cat(bs).contiguous()
            elif self.qkv is not None:
                self.bias = torch.cat([b.float() for b in bs]).contiguous()
            else:
                self.biases = bs
        self.o = weights["o"]
        self.qk_norm = bool(p.get("qk_norm", False))
        if self.qk_norm:
            self.q_norm, self.k_norm = weights["q_norm"], weights["k_norm"]
            self.qk_norm_eps = float(p.get("qk_norm_eps", 1e-6))
            if self.qkv is not None:        # the projections run one by one, each into a buffer of its own
                self.mats = [self.qkv[:self.qd], self.qkv[self.qd:self.qd + self.kvd], self.qkv[self.qd + self.kvd:]]
                if self.bias is not None:
                    self.biases = [self.bias[:self.qd], self.bias[self.qd:self.qd + self.kvd], self.bias[self.qd + self.kvd:]]
        # the widest prompt tile the prompt kernel of this head size takes (the planner chooses step by step)
        self.wide_tile = ops.attention_prefill_tile(rt.dtype, self.d) if rt.device.type == "cuda" else LONG_TILE
        self.plan_key = attention_planner(self.wide_tile, self.nh).key

    def attend(self, q, att, batch, view, memory: LayerMemory) -> None:
        """Tokens of short entries (decoded tokens) go to the kernel that splits one query's keys over
        many wavefronts, longer portions to the matrix-core prompt kernel; every shape those kernels do
        not take goes to the plain one."""
        kc, vc = memory.tensors["k"], memory.tensors["v"]
        args = (kc, vc, batch.tok_seq, batch.positions, view.block_tables, self.nh, self.nkv, self.d, self.scale)
        plan = batch.plans[self.plan_key]
        n_short, n_long, N = plan.sizes["num_short"], plan.sizes["num_long"], batch.num_tokens
        if n_short:
            if ops.attention_decode_supported(q.dtype, self.nh, self.nkv, self.d, kc.shape[2]):
                ws = self.rt.buffer("attn_split", (ops.attention_decode_workspace(n_short, self.nh, self.d),),
                                    torch.float32)
                ops.attention_decode(q, *args, plan.sizes["max_short_keys"], self.window, out=att,
                                     tok_index=plan.dev["short_idx"] if n_short < N else None, workspace=ws)
            else:
                n_long = -1      # everything through the plain kernel
        if n_long < 0:
            ops.attention(q, *args, self.window, out=att)
        elif n_long > 0:
            if ops.attention_prefill_supported(q.dtype, self.nh, self.nkv, self.d, kc.shape[2]):
                max_keys = plan.sizes["max_long_keys"]
                need = ops.attention_prefill_workspace(q.shape[0], self.nh, self.d, max_keys, self.window,
                                                       plan.sizes["num_tiles"])
                ws = self.rt.buffer("attn_prompt_split", (need,), torch.float32) if need else None
                ops.attention_prefill(q, kc, vc, plan.dev["tile_entry"], plan.dev["tile_off"],
                                      batch.entry_start, batch.entry_len, batch.entry_past, view.block_tables, self.nh,
                                      self.nkv, self.d, self.scale, self.window, out=att, max_keys=max_keys,
                                      workspace=ws, tile=plan.sizes["tile"], alone=plan.sizes["alone"])
            else:
                ops.attention(q, *args, self.window, out=att, tok_index=plan.dev["long_idx"] if n_long < N else None)

    def planner(self) -> StepPlanner:
        return attention_planner(self.wide_tile, self.nh)

    def positions_of(self, batch) -> torch.Tensor:
        """What the position encoding is given: every token's index in its sequence, or the step's
        positions on several axes when the encoding has more than one."""
        return batch.position_ids if self.position.position_axes > 1 else batch.positions

    def cache_request(self) -> Optional[KVCacheRequest]:
        return attention_cache_request("window" if self.window > 0 else "full", self.nkv, self.d, self.window)

    def step_rows(self, rows: int, kind: str) -> int:
        """The projections are few-rows products up to a number of rows and the library's beyond; portions are cut
        into tiles of LONG_TILE queries (PORTION_ROWS is a multiple)."""
        return ProductRows.step_rows(rows, kind)

    def encode_and_store(self, q, k, v, batch, view, memory: LayerMemory) -> None:
        """Queries and keys get their positions, keys and values go into the cache (when this run writes it).  An
        encoding that hands over the step's table of angles (or says that it does nothing) is folded into the
        kernel that stores; any other transforms q and k itself first."""
        table = self.position.step_table(batch)
        if table is None:
            self.position.encode(q, k, self.positions_of(batch), self.nh, self.nkv, self.d)
            if memory.writes:
                ops.kv_store(k, v, view.slots, memory.tensors["k"], memory.tensors["v"], self.nkv, self.d)
            return
        angles = None if isinstance(table, str) else table
        if memory.writes:
            ops.rope_kv_store(q, k, v, angles, view.slots, memory.tensors["k"], memory.tensors["v"], self.nh, self.nkv,
                              self.d)
        elif angles is not None:
            ops.rope_kv_store(q, None, None, angles, None, None, None, self.nh, self.nkv, self.d)

    def encode_and_store_sums(self, sums, q_out, batch, view, memory: LayerMemory) -> None:
        """The same from the float32 partial sums [S, n, Qd + 2 KVd] of the fused projection (the bias is added
        here); the encoded queries go to ``q_out``."""
        table = self.position.step_table(batch)
        if table is None:
            qkv = ops.reduce_sums(sums, self.bias, out_dtype=q_out.dtype,
                                  out=self.rt.buffer("attn_qkv", (sums.shape[1], self.qd + 2 * self.kvd)))
            q, k, v = qkv[:, :self.qd], qkv[:, self.qd:self.qd + self.kvd], qkv[:, self.qd + self.kvd:]
            self.encode_and_store(q, k, v, batch, view, memory)
            q_out.copy_(q)
            return
        angles = None if isinstance(table, str) else table
        if memory.writes:
            ops.rope_kv_store_sums(sums, self.bias, q_out, angles, view.slots, memory.tensors["k"], memory.tensors["v"],
                                   self.nh, self.nkv, self.d)
        else:
            ops.rope_kv_store_sums(sums, self.bias, q_out, angles, None, None, None, self.nh, self.nkv, self.d)

    def forward(self, x: torch.Tensor, batch, memory: LayerMemory) -> torch.Tensor:
        n = x.shape[0]
        view = batch.groups[memory.group]
        if self.qk_norm:
            q, k, v = (self.rt.buffer(name, (n, width)) for name, width in
                       (("attn_q", self.qd), ("attn_k", self.kvd), ("attn_v", self.kvd)))
            for dst, m, b in zip((q, k, v), self.mats, self.biases or (None, None, None)):
                ops.linear(x, m, b, out=dst)
            # every head is a row of head_dim values: normed in place
            ops.rms_norm(q.view(n * self.nh, self.d), self.q_norm, self.qk_norm_eps, out=q.view(n * self.nh, self.d))
            ops.rms_norm(k.view(n * self.nkv, self.d), self.k_norm, self.qk_norm_eps, out=k.view(n * self.nkv, self.d))
            self.encode_and_store(q, k, v, batch, view, memory)
        elif self.qkv is not None and ops.linear_sums_supported(x, self.qkv):
            # few rows: the projection leaves float32 partial sums; the rotary kernel adds them and the bias
            S = ops.linear_splits(n, self.qkv.shape[0], self.hidden)
            sums = self.rt.buffer("attn_qkv_sums", (S, n, self.qd + 2 * self.kvd), torch.float32)
            ops.linear_sums(x, self.qkv, out=sums)
            out = self.decode_from_sums(sums, batch, view, memory)
            if out is not None:
                return out
            q = self.rt.buffer("attn_q", (n, self.qd))
            self.encode_and_store_sums(sums, q, batch, view, memory)
        else:
            qkv = self.rt.buffer("attn_qkv", (n, self.qd + 2 * self.kvd))
            q, k, v = qkv[:, :self.qd], qkv[:, self.qd:self.qd + self.kvd], qkv[:, self.qd + self.kvd:]
            if self.qkv is not None:
                ops.linear(x, self.qkv, self.bias, out=qkv)
            else:
                for dst, m, b in zip((q, k, v), self.mats, self.biases or (None, None, None)):
                    ops.linear(x, m, b, out=dst)
            self.encode_and_store(q, k, v, batch, view, memory)
        att = self.rt.buffer("attn_out", (n, self.qd))
        self.attend(q, att, batch, view, memory)
        return self.project(att, n)

    def tune(self, num_tokens: int) -> None:
        """The library's algorithms for the projections of a step of ``num_tokens`` rows."""
        n = int(num_tokens)
        x = self.rt.buffer("norm_out", (n, self.hidden))
        if self.qkv is not None and not self.qk_norm:
            self.rt.tune_linear(x, self.qkv, self.bias)
        else:
            for m, b in zip(self.mats, self.biases or (None, None, None)):
                self.rt.tune_linear(x, m, b)
        self.rt.tune_linear(self.rt.buffer("attn_out", (n, self.qd)), self.o)

    def project(self, att: torch.Tensor, n: int) -> torch.Tensor:
        if ops.linear_sums_supported(att, self.o):
            S = ops.linear_splits(n, self.hidden, self.qd)
            return ops.linear_sums(att, self.o, out=self.rt.buffer("attn_proj_sums", (S, n, self.hidden), torch.float32))
        out = self.rt.buffer("attn_proj", (n, self.hidden))
        return ops.linear(att, self.o, out=out)

    def decode_from_sums(self, sums, batch, view, memory: LayerMemory) -> Optional[torch.Tensor]:
        """A pure decode step (one token a sequence): rotation, cache store and attention in one kernel,
        when the position encoding is a rotation it can hand over as a table of angles (or nothing) and
        the kernel takes the shape; then the output projection, read straight from the attention's
        chunks over the keys where that kernel takes the shape.  None: nothing was done."""
        if not batch.single_tokens or batch.num_tokens > self.FUSED_DECODE_MAX_TOKENS:
            return None
        table = self.position.step_table(batch)
        if table is None:
            return None
        rot = 0 if isinstance(table, str) else 2 * table.shape[1]
        S, n, width = sums.shape
        kc, vc = memory.tensors["k"], memory.tensors["v"]
        ps = kc.shape[2]
        max_keys = batch.plans[self.plan_key].sizes["max_short_keys"]
        if not ops.attention_decode_fused_supported(kc.dtype, self.nh, self.nkv, self.d, ps, rot, S, width, n):
            return None
        most = self.FUSED_DECODE_MAX_WORKGROUPS
        if most is None:
            most = self.FUSED_DECODE_WORKGROUPS_PER_UNIT * compute_units()
        if n * self.nkv * ops.attention_decode_chunks(max_keys) > most:
            return None
        ws = self.rt.buffer("attn_split", (ops.attention_decode_workspace(n, self.nh, self.d),), torch.float32)
        # every entry brings one token: token t is of entry t
        args = (sums, self.bias, None if rot == 0 else table, view.slots if memory.writes else None, kc, vc, None, batch.positions, view.block_tables, self.nh, self.nkv, self.d, self.scale,
                max_keys, self.window)
        if (self.o.numel() * self.o.element_size() <= self.PROJECT_FROM_CHUNKS_MAX_BYTES
                and ops.attention_decode_project_supported(self.o, n, self.nh, self.d)):
            ops.attention_decode_fused(*args, workspace=ws, write_kv=memory.writes, leave_chunks=True)
            out = self.rt.buffer("attn_proj_heads", (ops.attention_decode_project_splits(self.nh), n, self.hidden),
                                 torch.float32)
            return ops.attention_decode_project(ws, self.o, batch.positions, self.nh, self.d, max_keys, self.window,
                                                out=out)
        att = self.rt.buffer("attn_out", (n, self.qd))
        ops.attention_decode_fused(*args, out=att, workspace=ws, write_kv=memory.writes)
        return self.project(att, n)
