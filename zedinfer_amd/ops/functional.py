"""Checked launches of the HIP kernels on torch tensors."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_float, c_int, c_void_p
from typing import Optional, Tuple

import numpy as np
import torch

from . import _lib

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def has_gpu() -> bool:
    return torch.cuda.is_available()


has_cuda = has_gpu      # the reference module's name for it (python/zedinfer_ops.cpp:316-355)


def device_synchronize() -> None:
    torch.cuda.synchronize()


def _code(t: torch.Tensor, what: str) -> int:
    if t.dtype not in _CODES:
        raise TypeError(f"{what}: dtype {t.dtype} is not supported (float32 and bfloat16 are)")
    return _CODES[t.dtype]


def _gpu(what: str, *tensors: Optional[torch.Tensor]) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError(f"{what}: every tensor must live on the GPU; got one on {t.device}")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError(f"{what}: tensors on different devices ({dev} and {t.device})")


def _rows(t: torch.Tensor, what: str) -> Tuple[int, int]:
    """(row stride, width) of a 2-D tensor whose rows are dense."""
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise ValueError(f"{what}: expected a 2-D tensor with dense rows, got shape {tuple(t.shape)} "
                         f"strides {t.stride()}")
    ld = t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])
    if ld < t.shape[1]:
        raise ValueError(f"{what}: rows overlap (stride {ld} < width {t.shape[1]})")
    return ld, t.shape[1]


def _p(t: Optional[torch.Tensor]) -> c_void_p:
    return c_void_p(t.data_ptr() if t is not None else 0)


def _stream() -> c_void_p:
    # the raw handle of torch's current stream on the current device; torch.cuda.current_stream() builds
    # a Python object and resolves the device each time, which costs more than a whole launch
    return c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _i32(t: torch.Tensor, what: str, n: Optional[int] = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise TypeError(f"{what}: expected a contiguous int32 tensor, got {t.dtype}")
    if n is not None and t.numel() < n:
        raise ValueError(f"{what}: {t.numel()} entries, {n} needed")


# ---------------------------------------------------------------------------
def embedding(ids: torch.Tensor, table: torch.Tensor, out: Optional[torch.Tensor] = None,
              out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """out[i,:] = table[ids[i],:] for int32 ids."""
    _gpu("embedding", ids, table, out)
    n = ids.numel()
    _i32(ids, "embedding ids")
    if table.dim() != 2 or not table.is_contiguous():
        raise ValueError("embedding: table must be a contiguous [vocab, hidden] tensor")
    V, H = table.shape
    if out is None:
        out = torch.empty((n, H), dtype=out_dtype or table.dtype, device=table.device)
    if tuple(out.shape) != (n, H) or not out.is_contiguous():
        raise ValueError(f"embedding: out must be contiguous [{n}, {H}], got {tuple(out.shape)}")
    _lib.call("zi_embedding", _p(out), _code(out, "embedding out"), _p(table), _code(table, "embedding table"),
              _p(ids), n, H, V, _stream())
    return out


def gather_rows(x: torch.Tensor, idx: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _gpu("gather_rows", x, idx, out)
    _i32(idx, "gather_rows idx")
    if x.dim() != 2 or not x.is_contiguous():
        raise ValueError("gather_rows: x must be contiguous 2-D")
    n = idx.numel()
    if out is None:
        out = torch.empty((n, x.shape[1]), dtype=x.dtype, device=x.device)
    if tuple(out.shape) != (n, x.shape[1]) or out.dtype != x.dtype or not out.is_contiguous():
        raise ValueError("gather_rows: out has the wrong shape or dtype")
    _lib.call("zi_gather_rows", _p(out), _p(x), _code(x, "gather_rows"), _p(idx), n, x.shape[0], x.shape[1],
              _stream())
    return out


def add(a: torch.Tensor, b: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """c = a + b, added in float32."""
    _gpu("add", a, b, out)
    if a.shape != b.shape or not a.is_contiguous() or not b.is_contiguous():
        raise ValueError(f"add: shapes {tuple(a.shape)} and {tuple(b.shape)} must match and be contiguous")
    if out is None:
        out = torch.empty_like(a)
    if out.shape != a.shape or not out.is_contiguous():
        raise ValueError("add: out has the wrong shape")
    _lib.call("zi_add", _p(out), _code(out, "add out"), _p(a), _code(a, "add a"), _p(b), _code(b, "add b"),
              a.numel(), _stream())
    return out


def swiglu(gate: torch.Tensor, up: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
           interleave: int = 0, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """out = up * gate / (1 + exp(-gate)).

    ``gate`` and ``up`` [n, I] may be column slices of one tensor.  With ``interleave`` = B, ``gate``
    is one [n, 2I] matrix that holds B gate columns, then the B up columns of the same places, and so
    on (``up`` is not given).  A 3-D ``gate`` [S, n, 2I] (interleaved only) is a stack of float32
    partial sums that are added in rising order first."""
    _gpu("swiglu", gate, up, out)
    splits, split_stride = 1, 0
    if gate.dim() == 3:
        if interleave <= 0 or not gate.is_contiguous():
            raise ValueError("swiglu: partial sums must be one contiguous interleaved [S, n, 2I] tensor")
        splits, split_stride = gate.shape[0], gate.shape[1] * gate.shape[2]
        gate = gate[0]
    ldg, wg = _rows(gate, "swiglu gate")
    n = gate.shape[0]
    if interleave > 0:
        if up is not None or wg % (2 * interleave):
            raise ValueError(f"swiglu: an interleaved input of width {wg} must hold whole blocks of 2*{interleave}")
        I, ldu = wg // 2, 0
    else:
        ldu, I2 = _rows(up, "swiglu up")
        if gate.shape != up.shape or gate.dtype != up.dtype:
            raise ValueError(f"swiglu: gate {tuple(gate.shape)} {gate.dtype} and up {tuple(up.shape)} {up.dtype} differ")
        I = wg
    if out is None:
        out = torch.empty((n, I), dtype=out_dtype or gate.dtype, device=gate.device)
    if tuple(out.shape) != (n, I) or not out.is_contiguous():
        raise ValueError("swiglu: out has the wrong shape")
    _lib.call("zi_swiglu", _p(out), _code(out, "swiglu out"), _p(gate), _p(up), _code(gate, "swiglu"), n, I, ldg, ldu,
              int(interleave), splits, split_stride, _stream())
    return out


def swiglu_t(gate_up_t: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The same from the transposed product: ``gate_up_t`` [2I, n] bfloat16 holds, block of 8 channels by
    block, 8 rows of gate values and the 8 rows of their up values; returns [n, I].  n and I must be
    multiples of 8."""
    _gpu("swiglu_t", gate_up_t, out)
    ldt, n = _rows(gate_up_t, "swiglu_t input")
    if gate_up_t.dtype != torch.bfloat16 or gate_up_t.shape[0] % 16 or n % 8:
        raise ValueError(f"swiglu_t: a bfloat16 [2I, n] tensor with I and n multiples of 8 is needed, got "
                         f"{tuple(gate_up_t.shape)} {gate_up_t.dtype}")
    I = gate_up_t.shape[0] // 2
    if out is None:
        out = torch.empty((n, I), dtype=torch.bfloat16, device=gate_up_t.device)
    if tuple(out.shape) != (n, I) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise ValueError("swiglu_t: out has the wrong shape or dtype")
    _lib.call("zi_swiglu_t", _p(out), _p(gate_up_t), BF16, n, I, ldt, _stream())
    return out


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None,
             out_dtype: Optional[torch.dtype] = None, add_one: bool = False) -> torch.Tensor:
    """y = (w [+1]) * x * rsqrt(mean(x^2) + eps) over the last dimension of a 2-D x."""
    _gpu("rms_norm", x, weight, out)
    ldx, H = _rows(x, "rms_norm x")
    if weight.dim() != 1 or weight.numel() != H or not weight.is_contiguous():
        raise ValueError(f"rms_norm: weight must be [{H}], got {tuple(weight.shape)}")
    n = x.shape[0]
    if out is None:
        out = torch.empty((n, H), dtype=out_dtype or x.dtype, device=x.device)
    ldo, Ho = _rows(out, "rms_norm out")
    if tuple(out.shape) != (n, H):
        raise ValueError("rms_norm: out has the wrong shape")
    if not eps > 0:
        raise ValueError("rms_norm: eps must be positive")
    _lib.call("zi_rmsnorm", _p(out), _code(out, "rms_norm out"), _p(x), _code(x, "rms_norm x"), _p(weight),
              _code(weight, "rms_norm weight"), n, H, ldx, ldo, float(eps), int(add_one), _stream())
    return out


def add_rms_norm(resid: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor, eps: float,
                 out: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None,
                 add_one: bool = False) -> torch.Tensor:
    """resid (float32, changed in place) += delta; returns norm(resid) * w.  ``delta`` is [n, H], or a
    stack [S, n, H] of float32 partial sums that are added in rising order."""
    _gpu("add_rms_norm", resid, delta, weight, out)
    if resid.dtype != torch.float32 or resid.dim() != 2 or not resid.is_contiguous():
        raise ValueError("add_rms_norm: the residual stream must be a contiguous float32 [n, hidden] tensor")
    n, H = resid.shape
    splits, split_stride = 1, 0
    if delta.dim() == 3:
        if delta.dtype != torch.float32:
            raise ValueError("add_rms_norm: partial sums must be float32")
        splits, split_stride = delta.shape[0], n * H
    if tuple(delta.shape[-2:]) != (n, H) or not delta.is_contiguous():
        raise ValueError("add_rms_norm: delta must match the residual's shape and be contiguous")
    if weight.dim() != 1 or weight.numel() != H or not weight.is_contiguous():
        raise ValueError(f"add_rms_norm: weight must be [{H}]")
    if out is None:
        out = torch.empty((n, H), dtype=out_dtype or (delta.dtype if delta.dim() == 2 else torch.bfloat16),
                          device=resid.device)
    if tuple(out.shape) != (n, H) or not out.is_contiguous():
        raise ValueError("add_rms_norm: out has the wrong shape")
    _lib.call("zi_add_rmsnorm", _p(out), _code(out, "add_rms_norm out"), _p(resid), _p(delta),
              _code(delta, "add_rms_norm delta"), splits, split_stride, _p(weight),
              _code(weight, "add_rms_norm weight"), n, H, float(eps), int(add_one), _stream())
    return out


def rope_inv_freq(rotary_dim: int, theta: float, device) -> torch.Tensor:
    """inv_freq[k] = 1 / theta^(2k / rotary_dim) in float32
    (reference: src/backend/ops/rope/cpu/rope_cpu.cpp:62-65)."""
    k = np.arange(rotary_dim // 2, dtype=np.float32)
    expo = (2.0 * k / np.float32(rotary_dim)).astype(np.float32)
    inv = (np.float32(1.0) / np.power(np.float32(theta), expo)).astype(np.float32)
    return torch.from_numpy(inv).to(device)


def rope(x: torch.Tensor, pos: torch.Tensor, inv_freq: torch.Tensor, out: Optional[torch.Tensor] = None
         ) -> torch.Tensor:
    """Split-half rotation of x [n, heads, head_dim] by int32 positions [n]."""
    _gpu("rope", x, pos, inv_freq, out)
    if x.dim() != 3 or not x.is_contiguous():
        raise ValueError("rope: x must be a contiguous [n, heads, head_dim] tensor")
    n, nh, d = x.shape
    _i32(pos, "rope positions", n)
    rot = 2 * inv_freq.numel()
    if inv_freq.dtype != torch.float32 or not inv_freq.is_contiguous() or rot > d:
        raise ValueError("rope: inv_freq must be float32 with at most head_dim/2 entries")
    if out is None:
        out = torch.empty_like(x)
    if out.shape != x.shape or out.dtype != x.dtype or not out.is_contiguous():
        raise ValueError("rope: out has the wrong shape or dtype")
    _lib.call("zi_rope", _p(out), _p(x), _code(x, "rope"), n, nh * d, nh * d, _p(pos), _p(inv_freq), nh, d, rot,
              _stream())
    return out


def _check_cache(kcache: torch.Tensor, vcache: torch.Tensor, nkv: int, d: int, dtype, what: str) -> Tuple[int, int]:
    """A layer's key cache is [pages, kv_heads, page_size, head_dim], its value cache is stored
    transposed, [pages, kv_heads, head_dim, page_size]; returns (pages, page_size)."""
    if (kcache.dim() != 4 or not kcache.is_contiguous() or kcache.shape[1] != nkv or kcache.shape[3] != d
            or kcache.dtype != dtype):
        raise ValueError(f"{what}: key cache must be contiguous [pages, {nkv}, page_size, {d}] of {dtype}, "
                         f"got {tuple(kcache.shape)} {kcache.dtype}")
    pages, ps = kcache.shape[0], kcache.shape[2]
    if tuple(vcache.shape) != (pages, nkv, d, ps) or not vcache.is_contiguous() or vcache.dtype != dtype:
        raise ValueError(f"{what}: value cache must be contiguous [{pages}, {nkv}, {d}, {ps}] of {dtype}, "
                         f"got {tuple(vcache.shape)} {vcache.dtype}")
    return pages, ps


def _angle_table(table: Optional[torch.Tensor], n: int, d: int, what: str) -> int:
    """Checks a step's table of (cos, sin) [n, R/2, 2] and returns R, the rotated dims (0 without a table)."""
    if table is None:
        return 0
    if (table.dim() != 3 or table.shape[0] != n or table.shape[2] != 2 or table.dtype != torch.float32
            or not table.is_contiguous() or 2 * table.shape[1] > d):
        raise ValueError(f"{what}: the table of angles must be a contiguous float32 [{n}, R/2, 2] tensor with R <= {d}")
    return 2 * int(table.shape[1])


def rope_kv_store(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor], table: Optional[torch.Tensor],
                  slots: Optional[torch.Tensor], kcache: Optional[torch.Tensor], vcache: Optional[torch.Tensor],
                  nh: int, nkv: int, d: int) -> None:
    """Rotate q [n, nh*d] in place by the step's ``table`` of (cos, sin) [n, R/2, 2] (``rope_table``); rotate k
    and copy v [n, nkv*d] into the cache at ``slots``.  q, k and v may be column slices of one tensor.  With
    ``k`` None nothing is stored; with ``table`` None nothing is rotated."""
    _gpu("rope_kv_store", q, k, v, table, slots, kcache, vcache)
    ldq, wq = _rows(q, "rope_kv_store q")
    n = q.shape[0]
    if wq != nh * d:
        raise ValueError(f"rope_kv_store: q has width {wq}, expected {nh}*{d}")
    write = k is not None
    ldk = ldv = 0
    pages = ps = 0
    if write:
        ldk, wk = _rows(k, "rope_kv_store k")
        ldv, wv = _rows(v, "rope_kv_store v")
        if wk != nkv * d or wv != nkv * d or k.shape[0] != n or v.shape[0] != n or k.dtype != q.dtype or v.dtype != q.dtype:
            raise ValueError("rope_kv_store: k and v must be [n, kv_heads*head_dim] of q's dtype")
        pages, ps = _check_cache(kcache, vcache, nkv, d, q.dtype, "rope_kv_store")
        _i32(slots, "rope_kv_store slots", n)
    rot = _angle_table(table, n, d, "rope_kv_store")
    _lib.call("zi_rope_kv_store", _p(q), _p(k), _p(v), _code(q, "rope_kv_store"), n, ldq, ldk, ldv, _p(slots), _p(table),
              _p(kcache), _p(vcache), pages * ps, nh, nkv, d, rot, max(ps, 1), int(write), _stream())


def kv_store(k: torch.Tensor, v: torch.Tensor, slots: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
             nkv: int, d: int) -> None:
    """Copy keys and values [n, nkv*d] (already encoded) into the cache at ``slots``."""
    rope_kv_store(k, k, v, None, slots, kcache, vcache, nkv, nkv, d)


def rope_kv_store_sums(sums: torch.Tensor, bias: Optional[torch.Tensor], q_out: torch.Tensor,
                       table: Optional[torch.Tensor], slots: Optional[torch.Tensor], kcache: Optional[torch.Tensor],
                       vcache: Optional[torch.Tensor], nh: int, nkv: int, d: int) -> None:
    """The same from the float32 partial sums [S, n, nh*d + 2*nkv*d] of one fused q/k/v projection:
    adds the splits in rising order and the bias, rotates, writes q to ``q_out`` [n, nh*d] and k, v
    into the cache.  With ``kcache`` None only q is made (the sums may then be [S, n, nh*d])."""
    _gpu("rope_kv_store_sums", sums, bias, q_out, table, slots, kcache, vcache)
    if sums.dim() != 3 or sums.dtype != torch.float32 or not sums.is_contiguous():
        raise ValueError("rope_kv_store_sums: sums must be a contiguous float32 [S, n, width] tensor")
    S, n, width = sums.shape
    write = kcache is not None
    need = nh * d + (2 * nkv * d if write else 0)
    if width < need:
        raise ValueError(f"rope_kv_store_sums: rows of {width} values, {need} needed")
    if bias is not None and (bias.dim() != 1 or bias.numel() < need or not bias.is_contiguous()):
        raise ValueError(f"rope_kv_store_sums: bias must hold {need} values")
    ldq, wq = _rows(q_out, "rope_kv_store_sums q_out")
    if q_out.shape[0] != n or wq != nh * d:
        raise ValueError(f"rope_kv_store_sums: q_out must be [{n}, {nh * d}]")
    pages = ps = 0
    if write:
        pages, ps = _check_cache(kcache, vcache, nkv, d, q_out.dtype, "rope_kv_store_sums")
        _i32(slots, "rope_kv_store_sums slots", n)
    rot = _angle_table(table, n, d, "rope_kv_store_sums")
    _lib.call("zi_rope_kv_store_split", _p(q_out), _code(q_out, "rope_kv_store_sums"), ldq, _p(sums), S, n * width,
              width, _p(bias), _code(bias, "rope_kv_store_sums bias") if bias is not None else F32, n, _p(slots),
              _p(table), _p(kcache), _p(vcache), pages * ps, nh, nkv, d, rot, max(ps, 1), int(write), _stream())


def _attention_args(what, q, kcache, vcache, tok_seq, tok_pos, block_tables, nh, nkv, d, tok_index, out):
    _gpu(what, q, kcache, vcache, tok_seq, tok_pos, block_tables, tok_index, out)
    ldq, wq = _rows(q, f"{what} q")
    n = q.shape[0]
    if wq != nh * d:
        raise ValueError(f"{what}: q has width {wq}, expected {nh}*{d}")
    if nkv <= 0 or nh % nkv:
        raise ValueError(f"{what}: {nh} query heads are not a multiple of {nkv} key/value heads")
    pages, ps = _check_cache(kcache, vcache, nkv, d, q.dtype, what)
    _i32(tok_seq, f"{what} tok_seq", n)
    _i32(tok_pos, f"{what} tok_pos", n)
    if tok_index is not None:
        _i32(tok_index, f"{what} tok_index")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise ValueError(f"{what}: block_tables must be a contiguous int32 [seqs, max_pages] tensor")
    if out is None:
        out = torch.empty((n, nh * d), dtype=q.dtype, device=q.device)
    ldo, wo = _rows(out, f"{what} out")
    if tuple(out.shape) != (n, nh * d) or out.dtype != q.dtype:
        raise ValueError(f"{what}: out has the wrong shape or dtype")
    count = tok_index.numel() if tok_index is not None else n
    return out, n, count, ldq, ldo, pages, ps


def attention(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, tok_seq: torch.Tensor,
              tok_pos: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int, d: int, scale: float,
              window: int = 0, out: Optional[torch.Tensor] = None, tok_index: Optional[torch.Tensor] = None
              ) -> torch.Tensor:
    """Causal grouped-query attention of q [n, nh*d] over the paged cache: the plain kernel, for
    every shape and both storage types.

    Token i belongs to row ``tok_seq[i]`` of ``block_tables`` [seqs, max_pages] and sits at
    absolute position ``tok_pos[i]``; it sees the cached keys at positions
    [max(0, pos - window + 1), pos] (window 0: all of them).  With ``tok_index`` only the listed
    tokens are computed (the other rows of ``out`` are left alone).  Returns [n, nh*d]."""
    out, n, count, ldq, ldo, pages, ps = _attention_args("attention", q, kcache, vcache, tok_seq, tok_pos,
                                                         block_tables, nh, nkv, d, tok_index, out)
    _lib.call("zi_attention_generic", _p(out), _p(q), _code(q, "attention"), count, ldq, ldo, _p(kcache), _p(vcache),
              _p(tok_index), _p(tok_seq), _p(tok_pos), _p(block_tables), block_tables.shape[1], pages, nh, nkv, d,
              ps, int(window), float(scale), _stream())
    return out




def attention_decode_supported(dtype: torch.dtype, nh: int, nkv: int, d: int, page_size: int) -> bool:
    if dtype not in _CODES:
        return False
    return bool(_lib.load().zi_attention_decode_supported(_CODES[dtype], nh, nkv, d, page_size))


def attention_decode_chunks(max_keys: int) -> int:
    """Chunks of the keys that the decode attention launches for every token and key/value head when no token
    sees more than ``max_keys`` keys."""
    return int(_lib.load().zi_attention_decode_chunks(int(max_keys)))


def attention_decode_workspace(tokens: int, nh: int, d: int) -> int:
    """Floats of workspace for the chunk partials of ``tokens`` tokens."""
    return int(_lib.load().zi_attention_decode_workspace(int(tokens), int(nh), int(d)))


def attention_decode(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, tok_seq: torch.Tensor,
                     tok_pos: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int, d: int, scale: float,
                     max_keys: int, window: int = 0, out: Optional[torch.Tensor] = None,
                     tok_index: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None
                     ) -> torch.Tensor:
    """The same attention for single query tokens, split over the keys, on the matrix cores
    (bfloat16, head_dim a multiple of 16 up to 128, group size <= 16, page size a multiple of 8).
    ``max_keys`` is an upper bound of the keys any listed token sees (its position + 1), known on
    the host; it only sizes the launch."""
    out, n, count, ldq, ldo, pages, ps = _attention_args("attention_decode", q, kcache, vcache, tok_seq, tok_pos,
                                                         block_tables, nh, nkv, d, tok_index, out)
    if window > 0:
        max_keys = min(max_keys, window)
    max_chunks = int(_lib.load().zi_attention_decode_chunks(int(max_keys)))
    need = attention_decode_workspace(count, nh, d)
    if max_chunks > 1:
        if workspace is None:
            workspace = torch.empty((need,), dtype=torch.float32, device=q.device)
        if workspace.dtype != torch.float32 or workspace.numel() < need or not workspace.is_contiguous():
            raise ValueError(f"attention_decode: workspace must be a contiguous float32 buffer of {need} entries")
    _lib.call("zi_attention_decode", _p(out), _p(q), _code(q, "attention_decode"), count, ldq, ldo, _p(kcache),
              _p(vcache), _p(tok_index), _p(tok_seq), _p(tok_pos), _p(block_tables), block_tables.shape[1], pages,
              nh, nkv, d, ps, int(window), float(scale), max_chunks, _p(workspace),
              workspace.numel() if workspace is not None else 0, _stream())
    return out


def rope_table(pos: torch.Tensor, inv_freq: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """cos and sin of pos[t] * inv_freq[k] as float32 [n, rotary_dim/2, 2]: the angles of one step, which
    every layer with the same frequencies shares."""
    _gpu("rope_table", pos, inv_freq, out)
    n, half = pos.numel(), inv_freq.numel()
    _i32(pos, "rope_table positions", n)
    if inv_freq.dtype != torch.float32 or not inv_freq.is_contiguous():
        raise ValueError("rope_table: inv_freq must be contiguous float32")
    if out is None:
        out = torch.empty((n, half, 2), dtype=torch.float32, device=pos.device)
    if tuple(out.shape) != (n, half, 2) or out.dtype != torch.float32 or not out.is_contiguous():
        raise ValueError(f"rope_table: out must be a contiguous float32 [{n}, {half}, 2] tensor")
    _lib.call("zi_rope_table", _p(out), _p(pos), _p(inv_freq), n, half, _stream())
    return out


def attention_decode_fused_supported(dtype: torch.dtype, nh: int, nkv: int, d: int, page_size: int, rotary_dim: int,
                                     splits: int, width: int, rows: int) -> bool:
    """Whether ``attention_decode_fused`` takes partial sums [splits, rows, width] with this rotation."""
    if dtype not in _CODES:
        return False
    return bool(_lib.load().zi_attention_decode_fused_supported(_CODES[dtype], nh, nkv, d, page_size, rotary_dim,
                                                                splits, rows * width, width))


def attention_decode_fused(sums: torch.Tensor, bias: Optional[torch.Tensor], table: Optional[torch.Tensor],
                           slots: Optional[torch.Tensor], kcache: torch.Tensor, vcache: torch.Tensor,
                           tok_seq: Optional[torch.Tensor], tok_pos: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int,
                           d: int, scale: float, max_keys: int, window: int = 0, out: Optional[torch.Tensor] = None,
                           workspace: Optional[torch.Tensor] = None, write_kv: bool = True,
                           leave_chunks: bool = False) -> torch.Tensor:
    """Rotation, cache store and attention of single decoded tokens in one kernel.

    ``sums`` [S, n, nh*d + 2*nkv*d] float32 are the partial sums of the fused q/k/v projection of the
    step's n tokens; splits are added in rising order, then ``bias``.  The first ``2 * table.shape[1]``
    dims of every query and key head turn by the angles of ``table`` ([n, pairs, 2] from ``rope_table``;
    None: no rotation).  With ``write_kv`` each token's new key and value go to slot ``slots[t]`` of the
    cache.  Every token must be the only one of its sequence in the call; ``tok_seq`` None means that
    token t is of sequence t (row t of ``block_tables``), which saves the kernel a dependent load.  Same shapes
    as ``attention_decode``; the result is what rope_kv_store_sums followed by attention_decode gives.
    With ``leave_chunks`` the chunks of the keys are not merged: they stay in ``workspace`` (which is
    returned) for ``attention_decode_project``, and ``out`` is not written."""
    _gpu("attention_decode_fused", sums, bias, table, slots, kcache, vcache, tok_seq, tok_pos, block_tables, out,
         workspace)
    if sums.dim() != 3 or sums.dtype != torch.float32 or not sums.is_contiguous():
        raise ValueError("attention_decode_fused: sums must be a contiguous float32 [S, n, width] tensor")
    S, n, width = sums.shape
    need_w = (nh + 2 * nkv) * d
    if width < need_w:
        raise ValueError(f"attention_decode_fused: rows of {width} values, {need_w} needed")
    if nkv <= 0 or nh % nkv:
        raise ValueError(f"attention_decode_fused: {nh} query heads are not a multiple of {nkv} key/value heads")
    if bias is not None and (bias.dim() != 1 or bias.numel() < need_w or not bias.is_contiguous()):
        raise ValueError(f"attention_decode_fused: bias must hold {need_w} values")
    pages, ps = _check_cache(kcache, vcache, nkv, d, kcache.dtype, "attention_decode_fused")
    if tok_seq is not None:
        _i32(tok_seq, "attention_decode_fused tok_seq", n)
    _i32(tok_pos, "attention_decode_fused tok_pos", n)
    if write_kv:
        _i32(slots, "attention_decode_fused slots", n)
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise ValueError("attention_decode_fused: block_tables must be a contiguous int32 [seqs, max_pages] tensor")
    if tok_seq is None and block_tables.shape[0] < n:
        raise ValueError(f"attention_decode_fused: {n} tokens without tok_seq need {n} rows of block_tables")
    rot = 0
    if table is not None:
        if table.dim() != 3 or table.shape[0] != n or table.shape[2] != 2 or table.dtype != torch.float32 \
                or not table.is_contiguous():
            raise ValueError(f"attention_decode_fused: table must be a contiguous float32 [{n}, pairs, 2] tensor")
        rot = 2 * table.shape[1]
    ldo = 0
    if leave_chunks:
        out = None
    else:
        if out is None:
            out = torch.empty((n, nh * d), dtype=kcache.dtype, device=sums.device)
        ldo, wo = _rows(out, "attention_decode_fused out")
        if tuple(out.shape) != (n, nh * d) or out.dtype != kcache.dtype:
            raise ValueError("attention_decode_fused: out has the wrong shape or dtype")
    if window > 0:
        max_keys = min(max_keys, window)
    max_chunks = int(_lib.load().zi_attention_decode_chunks(int(max_keys)))
    need = attention_decode_workspace(n, nh, d)
    if max_chunks > 1 or leave_chunks:
        if workspace is None:
            workspace = torch.empty((need,), dtype=torch.float32, device=sums.device)
        if workspace.dtype != torch.float32 or workspace.numel() < need or not workspace.is_contiguous():
            raise ValueError(f"attention_decode_fused: workspace must be a contiguous float32 buffer of {need} entries")
    _lib.call("zi_attention_decode_fused", _p(out), _code(kcache, "attention_decode_fused"), n, ldo, _p(sums), S,
              n * width, width, _p(bias), _code(bias, "attention_decode_fused bias") if bias is not None else F32,
              _p(table), rot, _p(slots), pages * ps, int(write_kv), _p(kcache), _p(vcache), _p(None), _p(tok_seq),
              _p(tok_pos), _p(block_tables), block_tables.shape[1], pages, nh, nkv, d, ps, int(window), float(scale),
              max_chunks, _p(workspace), workspace.numel() if workspace is not None else 0, _stream())
    return workspace if leave_chunks else out


def attention_decode_project_supported(weight: torch.Tensor, n: int, nh: int, d: int) -> bool:
    """Whether ``attention_decode_project`` multiplies ``weight`` [N, nh*d] with n tokens' chunks."""
    if weight.dtype not in _CODES or weight.dim() != 2 or weight.stride(1) != 1 or weight.shape[1] != nh * d:
        return False
    return bool(_lib.load().zi_attention_decode_project_supported(_CODES[weight.dtype], n, nh, d, weight.stride(0)))


def attention_decode_project_splits(nh: int) -> int:
    """Partial sums ``attention_decode_project`` leaves: one for each group of heads."""
    hg = int(_lib.load().zi_attention_decode_project_heads(nh))
    return -(-nh // hg)


def attention_decode_project(workspace: torch.Tensor, weight: torch.Tensor, tok_pos: torch.Tensor, nh: int, d: int,
                             max_keys: int, window: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The output projection of decoded tokens straight from the chunks that ``attention_decode_fused(...,
    leave_chunks=True)`` left in ``workspace`` (same tokens, heads, ``max_keys`` and ``window``): float32
    partial sums [splits, n, N] over groups of heads, to be added in rising order.  ``weight`` is [N, nh*d]."""
    _gpu("attention_decode_project", workspace, weight, tok_pos, out)
    n = tok_pos.numel()
    _i32(tok_pos, "attention_decode_project tok_pos", n)
    if not attention_decode_project_supported(weight, n, nh, d):
        raise ValueError(f"attention_decode_project: unsupported shape: {n} tokens, {nh} heads of {d}, weight "
                         f"{tuple(weight.shape)} {weight.dtype}")
    N = weight.shape[0]
    S = attention_decode_project_splits(nh)
    if out is None:
        out = torch.empty((S, n, N), dtype=torch.float32, device=weight.device)
    if tuple(out.shape) != (S, n, N) or out.dtype != torch.float32 or not out.is_contiguous():
        raise ValueError(f"attention_decode_project: out must be a contiguous float32 [{S}, {n}, {N}] tensor")
    need = attention_decode_workspace(n, nh, d)
    if workspace.dtype != torch.float32 or workspace.numel() < need or not workspace.is_contiguous():
        raise ValueError(f"attention_decode_project: workspace must be a contiguous float32 buffer of {need} entries")
    if window > 0:
        max_keys = min(max_keys, window)
    max_chunks = int(_lib.load().zi_attention_decode_chunks(int(max_keys)))
    _lib.call("zi_attention_decode_project", _p(out), _p(workspace), workspace.numel(), n, _p(tok_pos), int(window),
              max_chunks, _p(weight), _code(weight, "attention_decode_project"), weight.stride(0), N, nh, d, _stream())
    return out


DECODE_LAYER_SPIN_LIMIT = 400000      # polls of a barrier inside the resident layer kernel before it gives up (about 0.2 s)


def decode_layer_sync_words() -> int:
    """int32 words of synchronisation state the resident layer kernel needs (zeroed once, shared by every call)."""
    return int(_lib.load().zi_decode_layer_sync_words())


def decode_layer_stamps() -> int:
    """Clock stamps a workgroup of the resident layer kernel leaves per launch behind the synchronisation words:
    32 in a library built with -DDL_TIMING (a probe for tuning), 0 in the product's."""
    return int(_lib.load().zi_decode_layer_stamps())


def decode_layer_supported(dtype: torch.dtype, n: int, hidden: int, inter: int, nh: int, nkv: int, d: int, rot: int,
                           page_size: int, max_keys: int, window: int = 0) -> bool:
    """Whether ``decode_layer`` takes a step of ``n`` single tokens of these sizes on the current device."""
    if dtype not in _CODES:
        return False
    return bool(_lib.load().zi_decode_layer_supported(_CODES[dtype], int(n), int(hidden), int(inter), int(nh), int(nkv),
                                                       int(d), int(rot), int(page_size), int(max_keys), int(window)))


def decode_layer_workspace(n: int, hidden: int, inter: int, nh: int, nkv: int, d: int, max_keys: int,
                           window: int = 0) -> int:
    """Bytes of workspace ``decode_layer`` needs for these sizes."""
    need = int(_lib.load().zi_decode_layer_workspace(int(n), int(hidden), int(inter), int(nh), int(nkv), int(d),
                                                     int(max_keys), int(window)))
    if need < 0:
        raise _lib.KernelLibraryError(_lib.load().zi_last_error().decode("utf-8", "replace"))
    return need


def decode_layer(resid: torch.Tensor, norm1: torch.Tensor, norm2: torch.Tensor, eps1: float, eps2: float, add_one: bool,
                 wqkv: torch.Tensor, bias: Optional[torch.Tensor], wo: torch.Tensor, wgu: torch.Tensor, wd: torch.Tensor,
                 table: Optional[torch.Tensor], slots: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                 tok_pos: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int, d: int, scale: float,
                 max_keys: int, window: int, workspace: torch.Tensor, sync: torch.Tensor, err: torch.Tensor,
                 spin_limit: int = DECODE_LAYER_SPIN_LIMIT) -> torch.Tensor:
    """One pre-norm decoder layer (attention with a split-half rotation, SwiGLU feed-forward, RMS norms) for
    n <= 16 tokens that are each the only one of their sequence in the step, in one launch of resident
    workgroups: ``resid`` [n, hidden] float32 is replaced by the layer's output and the tokens' new keys and
    values are stored at ``slots``.  ``wgu`` [2I, hidden] holds gate and up rows alternating in blocks of 8;
    ``table`` [n, pairs, 2] are the step's (cos, sin) from ``rope_table`` (None: no rotation).  ``sync``
    (``decode_layer_sync_words()`` zeroed int32 words on the device) is shared by every call; ``err`` is one
    int32 word of pinned host memory which the kernel sets when one of its waits ran out: the step's result is
    then garbage (NaN), and ``sync`` must be zeroed before the next call."""
    _gpu("decode_layer", resid, norm1, norm2, wqkv, bias, wo, wgu, wd, table, slots, kcache, vcache, tok_pos,
         block_tables, workspace, sync)
    if resid.dim() != 2 or resid.dtype != torch.float32 or not resid.is_contiguous():
        raise ValueError("decode_layer: resid must be a contiguous float32 [n, hidden] tensor")
    n, H = resid.shape
    for name, w in (("wqkv", wqkv), ("wo", wo), ("wgu", wgu), ("wd", wd)):
        if w.dim() != 2 or w.dtype != torch.bfloat16 or w.stride(1) != 1:
            raise ValueError(f"decode_layer: {name} must be a bfloat16 matrix with dense rows")
    Qd, KVd = nh * d, nkv * d
    inter = wd.shape[1]
    if (tuple(wqkv.shape) != (Qd + 2 * KVd, H) or tuple(wo.shape) != (H, Qd) or tuple(wgu.shape) != (2 * inter, H)
            or wd.shape[0] != H):
        raise ValueError(f"decode_layer: weight shapes {tuple(wqkv.shape)}, {tuple(wo.shape)}, {tuple(wgu.shape)}, "
                         f"{tuple(wd.shape)} do not fit hidden {H}, heads {nh}/{nkv} of {d}")
    for name, g in (("norm1", norm1), ("norm2", norm2)):
        if g.dim() != 1 or g.numel() != H or not g.is_contiguous() or g.dtype != norm1.dtype:
            raise ValueError(f"decode_layer: {name} must hold {H} gains of one type")
    if bias is not None and (bias.dim() != 1 or bias.numel() != Qd + 2 * KVd or not bias.is_contiguous()):
        raise ValueError(f"decode_layer: bias must hold {Qd + 2 * KVd} values")
    pages, ps = _check_cache(kcache, vcache, nkv, d, torch.bfloat16, "decode_layer")
    _i32(tok_pos, "decode_layer tok_pos", n)
    _i32(slots, "decode_layer slots", n)
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous() \
            or block_tables.shape[0] < n:
        raise ValueError(f"decode_layer: block_tables must be a contiguous int32 [>= {n}, max_pages] tensor")
    rot = 0
    if table is not None:
        if table.dim() != 3 or table.shape[0] != n or table.shape[2] != 2 or table.dtype != torch.float32 \
                or not table.is_contiguous():
            raise ValueError(f"decode_layer: table must be a contiguous float32 [{n}, pairs, 2] tensor")
        rot = 2 * table.shape[1]
    if sync.dtype != torch.int32 or sync.numel() < decode_layer_sync_words() or not sync.is_contiguous():
        raise ValueError("decode_layer: sync must hold decode_layer_sync_words() int32 words")
    if err.dtype != torch.int32 or err.numel() < 1 or err.is_cuda or not err.is_pinned():
        raise ValueError("decode_layer: err must be an int32 word of pinned host memory")
    if workspace.dtype != torch.uint8 or not workspace.is_contiguous():
        raise ValueError("decode_layer: workspace must be a contiguous uint8 tensor")
    _lib.call("zi_decode_layer", _p(resid), n, H, inter, _p(norm1), _p(norm2), _code(norm1, "decode_layer gains"),
              c_float(eps1), c_float(eps2), int(bool(add_one)), _p(wqkv), wqkv.stride(0), _p(bias),
              _code(bias, "decode_layer bias") if bias is not None else 0, _p(wo), wo.stride(0), _p(wgu), wgu.stride(0),
              _p(wd), wd.stride(0), BF16, _p(table), rot, _p(slots), pages * ps, _p(kcache), _p(vcache), _p(tok_pos),
              _p(block_tables), block_tables.shape[1], pages, nh, nkv, d, ps, int(window), c_float(scale), int(max_keys),
              _p(workspace), workspace.numel(), _p(sync), c_void_p(err.data_ptr()), int(spin_limit), _stream())
    return resid


def attention_prefill_variant(variant: int = -1) -> int:
    """Which prompt-attention kernel head sizes 64 and 128 take: 1 (the default) loads keys and values
    straight into LDS, 0 stages them through registers like the other head sizes; both give the same
    bits.  Returns the variant in force before; -1 only asks."""
    return int(_lib.load().zi_attention_prefill_variant(int(variant)))


def compute_units() -> int:
    """Compute units of the current device: what the kernels' cuts and the parts' tile choices are balanced over
    (256 when there is no device to ask)."""
    return int(_lib.load().zi_compute_units())


def attention_prefill_tile_min() -> int:
    """Queries of the smallest tile of ``attention_prefill`` (every head size takes it)."""
    return int(_lib.load().zi_attention_prefill_tile_min())


def attention_prefill_tile(dtype: torch.dtype, d: int) -> int:
    """Queries of the widest tile of ``attention_prefill`` for this head size: the smallest, or twice that where
    the kernel that loads keys and values straight into LDS serves (a staged block then serves twice the
    queries).  The caller cuts its entries into tiles of this many queries."""
    if dtype not in _CODES:
        return attention_prefill_tile_min()
    return int(_lib.load().zi_attention_prefill_tile(_CODES[dtype], int(d)))



def attention_prefill_supported(dtype: torch.dtype, nh: int, nkv: int, d: int, page_size: int) -> bool:
    if dtype not in _CODES:
        return False
    return bool(_lib.load().zi_attention_prefill_supported(_CODES[dtype], nh, nkv, d, page_size))


def attention_prefill_workspace(rows: int, nh: int, d: int, max_keys: int, window: int = 0, num_tiles: int = 0) -> int:
    """float32 entries of workspace ``attention_prefill`` needs for ``rows`` query rows in ``num_tiles`` tiles of
    which none sees more than ``max_keys`` keys (0: none)."""
    lib = _lib.load()
    return int(lib.zi_attention_prefill_workspace(int(rows), nh, d, _prefill_cut(max_keys, window, int(num_tiles) * nh)[1]))


def _prefill_cut(max_keys: int, window: int, groups: int) -> Tuple[int, int]:
    """(keys between cuts, most cuts of a tile) of a prompt attention launch of ``groups`` tiles x heads none of
    whose queries sees more than ``max_keys`` keys: the cut is the library's choice (longer when there are tiles
    enough to fill the chip without cuts: every cut costs a merge)."""
    chunk = c_int(0)
    cuts = int(_lib.load().zi_attention_prefill_cuts(max(int(max_keys), 1), int(window), int(groups), ctypes.byref(chunk)))
    return chunk.value, cuts


def attention_prefill(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, tile_entry: torch.Tensor,
                      tile_off: torch.Tensor, entry_start: torch.Tensor, entry_len: torch.Tensor,
                      entry_past: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int, d: int, scale: float,
                      window: int = 0, out: Optional[torch.Tensor] = None, max_keys: int = 0,
                      workspace: Optional[torch.Tensor] = None, tile: int = 0, alone: bool = False) -> torch.Tensor:
    """The same attention for portions of prompts, on the matrix cores (bfloat16, head_dim a multiple
    of 16 up to 128, page size a power of two from 8).

    Entry e brings ``entry_len[e]`` tokens, rows ``entry_start[e]...`` of q, that continue a sequence
    holding ``entry_past[e]`` tokens whose block table is row e of ``block_tables``.  Tile i covers the
    queries [tile_off[i], tile_off[i] + tile) of entry ``tile_entry[i]`` (``tile``: 0 for the smallest,
    ``attention_prefill_tile_min()``, or what ``attention_prefill_tile`` says for the head size); rows of ``out`` that no tile covers are left alone.  ``max_keys`` is an upper bound, known on the host, of the keys any query
    sees (its position + 1; 0: what the block tables could hold): tiles that see more than 2,048 keys are
    cut over several workgroups and merged, which needs ``workspace`` (``attention_prefill_workspace``
    entries of float32; allocated here when not given).  A bound that is too low leaves NaN in the rows
    concerned.  ``alone`` (where the head size has tiles of 128): workgroups of four wavefronts, two to a compute
    unit, which pays for launches of many tiles; the result differs by rounding."""
    _gpu("attention_prefill", q, kcache, vcache, tile_entry, tile_off, entry_start, entry_len, entry_past,
         block_tables, out)
    ldq, wq = _rows(q, "attention_prefill q")
    n = q.shape[0]
    if wq != nh * d:
        raise ValueError(f"attention_prefill: q has width {wq}, expected {nh}*{d}")
    if nkv <= 0 or nh % nkv:
        raise ValueError(f"attention_prefill: {nh} query heads are not a multiple of {nkv} key/value heads")
    pages, ps = _check_cache(kcache, vcache, nkv, d, q.dtype, "attention_prefill")
    num_tiles = tile_entry.numel()
    _i32(tile_entry, "attention_prefill tile_entry")
    _i32(tile_off, "attention_prefill tile_off", num_tiles)
    E = entry_start.numel()
    for name, t in (("entry_start", entry_start), ("entry_len", entry_len), ("entry_past", entry_past)):
        _i32(t, f"attention_prefill {name}", E)
    if (block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous()
            or block_tables.shape[0] < E):
        raise ValueError("attention_prefill: block_tables must be a contiguous int32 [entries, max_pages] tensor")
    tile = int(tile) or attention_prefill_tile_min()
    if tile not in (attention_prefill_tile_min(), attention_prefill_tile(q.dtype, d)):
        raise ValueError(f"attention_prefill: tiles of {tile} queries are not taken for head size {d}")
    if alone and attention_prefill_tile(q.dtype, d) == attention_prefill_tile_min():
        raise ValueError(f"attention_prefill: workgroups of four wavefronts are not made for head size {d}")
    if out is None:
        out = torch.empty((n, nh * d), dtype=q.dtype, device=q.device)
    ldo, wo = _rows(out, "attention_prefill out")
    if tuple(out.shape) != (n, nh * d) or out.dtype != q.dtype:
        raise ValueError("attention_prefill: out has the wrong shape or dtype")
    if max_keys <= 0:
        max_keys = block_tables.shape[1] * ps      # no bound given: what the block tables could hold
    chunk_keys, max_chunks = _prefill_cut(int(max_keys), int(window), num_tiles * nh)
    need = int(_lib.load().zi_attention_prefill_workspace(n, nh, d, max_chunks))
    if need:
        if workspace is None:
            workspace = torch.empty((need,), dtype=torch.float32, device=q.device)
        if workspace.dtype != torch.float32 or workspace.numel() < need or not workspace.is_contiguous():
            raise ValueError(f"attention_prefill: workspace must be a contiguous float32 buffer of {need} entries")
    _lib.call("zi_attention_prefill", _p(out), _p(q), _code(q, "attention_prefill"), num_tiles, ldq, ldo, _p(kcache),
              _p(vcache), _p(tile_entry), _p(tile_off), _p(entry_start), _p(entry_len), _p(entry_past),
              _p(block_tables), block_tables.shape[1], pages, nh, nkv, d, ps, int(window), float(scale), n,
              max_chunks, _p(workspace) if need else _p(None), workspace.numel() if need else 0, int(tile), int(bool(alone)),
              chunk_keys, _stream())
    return out


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """out[M,N] = x[M,K] . weight[N,K]^T + bias[N], accumulated in float32
    (reference: src/backend/ops/linear/op.cpp:57-58).

    bfloat16 inputs with bfloat16 weights and output (or float32 output and more than 64 rows) go
    to the library matrix product, as the reference sends them to its vendor library (reference:
    src/backend/ops/linear/nvidia/linear_cublas.cu:134-231); every other pairing, and all of
    the float32 path, runs the plain FMA kernel, which has no reduced-precision mode."""
    _gpu("linear", x, weight, bias, out)
    ldx, K = _rows(x, "linear x")
    ldw, Kw = _rows(weight, "linear weight")
    M, N = x.shape[0], weight.shape[0]
    if K != Kw:
        raise ValueError(f"linear: x has {K} columns, weight has {Kw}")
    if bias is not None and (bias.dim() != 1 or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError(f"linear: bias must be [{N}]")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or x.dtype, device=x.device)
    ldo, No = _rows(out, "linear out")
    if tuple(out.shape) != (M, N):
        raise ValueError(f"linear: out must be [{M}, {N}], got {tuple(out.shape)}")
    if M == 0:
        return out
    bf = torch.bfloat16
    all_bf = x.dtype == bf and weight.dtype == bf and (bias is None or bias.dtype == bf)
    if all_bf and out.dtype == torch.float32 and M > SKINNY_MAX_ROWS and bias is None and _library_ok(x, weight, out):
        # float32 output for many rows (logits of a large decode batch or of every place of a prompt): the
        # library's product with float32 results, one pass over the weights instead of one per 64 rows
        _library_product(out, x, weight, None, False)
        return out
    if all_bf and (M <= FEW_ROWS or out.dtype == torch.float32) and _skinny_ok(x, weight, K, ldx, ldw):
        # few rows (decoding), or float32 output (logits): the hand-written matrix-core kernel
        lib = _lib.load()
        for m0 in range(0, M, SKINNY_MAX_ROWS):
            m = min(SKINNY_MAX_ROWS, M - m0)
            need = lib.zi_gemm_skinny_workspace(m, N, K)
            ws = _workspace(x.device, need) if need else None
            _lib.call("zi_gemm_skinny", _p(out[m0:m0 + m]), _code(out, "linear out"), 0, _p(x[m0:m0 + m]), _p(weight),
                      _p(bias), m, N, K, ldx, ldw, ldo, _p(ws), need, _stream())
        return out
    if all_bf and out.dtype == bf and _library_ok(x, weight, out):
        _library_product(out, x, weight, bias, False)
        return out
    _lib.call("zi_gemm_generic", _p(out), _code(out, "linear out"), _p(x), _code(x, "linear x"), _p(weight),
              _code(weight, "linear weight"), _p(bias), _code(bias, "linear bias") if bias is not None else F32,
              M, N, K, ldx, ldw, ldo, _stream())
    return out


def linear_transposed(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out [N, M] = weight [N, K] . x[M, K]^T: the transposed result of ``linear`` by the library's product
    with the operands' roles swapped, which it makes faster than ``linear`` at some sizes (bfloat16, many
    rows, no bias)."""
    _gpu("linear_transposed", x, weight, out)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or x.dim() != 2 or weight.dim() != 2 \
            or x.shape[1] != weight.shape[1] or not x.is_contiguous() or not weight.is_contiguous():
        raise ValueError("linear_transposed: contiguous bfloat16 x [M, K] and weight [N, K] are needed")
    M, N = x.shape[0], weight.shape[0]
    if out is None:
        out = torch.empty((N, M), dtype=torch.bfloat16, device=x.device)
    if tuple(out.shape) != (N, M) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise ValueError(f"linear_transposed: out must be a contiguous bfloat16 [{N}, {M}] tensor")
    _library_product(out, x, weight, None, True)
    return out


LIBRARY_WORKSPACE_BYTES = 64 << 20     # what an algorithm of the library's product may use beside its operands
_LIBRARY_WORKSPACES = {}


def _library_ok(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor) -> bool:
    """Rows one element apart in memory and 16-byte aligned: what the library's product is given."""
    return all(t.stride(1) == 1 and t.data_ptr() % 16 == 0 and t.stride(0) % 8 == 0 for t in (x, weight)) \
        and out.stride(1) == 1 and out.data_ptr() % 16 == 0


def _library_args(out, x, weight, bias, transposed):
    ws = _LIBRARY_WORKSPACES.get(x.device)
    if ws is None:
        ws = _LIBRARY_WORKSPACES[x.device] = torch.empty((LIBRARY_WORKSPACE_BYTES,), dtype=torch.uint8, device=x.device)
    return (_p(out), _code(out, "linear out"), _p(x), _p(weight), _p(bias), int(transposed), x.shape[0], weight.shape[0],
            x.shape[1], x.stride(0), weight.stride(0), out.stride(0), _p(ws), LIBRARY_WORKSPACE_BYTES)


def _library_product(out, x, weight, bias, transposed) -> None:
    _lib.call("zi_gemm_lt", *_library_args(out, x, weight, bias, transposed), _stream())


def linear_tune(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, transposed: bool = False,
                out_dtype: Optional[torch.dtype] = None, candidates: Optional[int] = None, rounds: Optional[int] = None):
    """Let the library time its proposals for the product ``linear`` (``linear_transposed``) makes of these operands
    and keep the fastest for every later call of the shape; returns (chosen, proposed, microseconds), or None when
    the product is not the library's (few rows, float32 operands).  Waits for the device.  ``candidates``: how
    many of the proposals are timed (None: the first 16, the first 8 of a product of about 250 us and more);
    ``rounds``: timed runs of each (None: five of a short product, fewer of one that takes long enough for the
    clock: three beyond about 50 us, two beyond 250)."""
    bf = torch.bfloat16
    M, N = x.shape[0], weight.shape[0]
    about_us = 2.0 * M * N * x.shape[1] / 1e9        # at a petaflop a second
    if rounds is None:
        rounds = 5 if about_us < 50 else (3 if about_us < 250 else 2)
    if candidates is None:
        candidates = 16 if about_us < 250 else 8
    out_dtype = out_dtype or bf
    if x.dtype != bf or weight.dtype != bf or (bias is not None and bias.dtype != bf):
        return None
    if M <= (SKINNY_MAX_ROWS if out_dtype == torch.float32 else FEW_ROWS) or (out_dtype == torch.float32 and bias is not None):
        return None
    out = torch.empty((N, M) if transposed else (M, N), dtype=out_dtype, device=x.device)
    if not _library_ok(x, weight, out):
        return None
    chosen, proposed, us = c_int(0), c_int(0), c_float(0.0)
    _lib.call("zi_gemm_lt_tune", *_library_args(out, x, weight, bias, transposed), int(candidates), int(rounds),
              ctypes.byref(chosen), ctypes.byref(proposed), ctypes.byref(us), _stream())
    return chosen.value, proposed.value, us.value


def linear_choose(x: torch.Tensor, weight: torch.Tensor, which: int, bias: Optional[torch.Tensor] = None,
                  transposed: bool = False, out_dtype: Optional[torch.dtype] = None,
                  out_stride: Optional[int] = None) -> None:
    """Fix the library's algorithm for the product of these operands to proposal ``which`` (what ``linear_tune``
    returned in an earlier run) without timing anything.  ``out_stride``: the row stride of the result the
    product will be given when that is a slice of a wider tensor (None: a contiguous result); the stride is part
    of what the library's plan for a shape is kept by."""
    _gpu("linear_choose", x, weight, bias)
    M, N, K = x.shape[0], weight.shape[0], x.shape[1]
    code = F32 if out_dtype == torch.float32 else BF16
    ldo = int(out_stride) if out_stride is not None else (M if transposed else N)
    _lib.call("zi_gemm_lt_choose", code, int(bias is not None), int(transposed), M, N, K, x.stride(0), weight.stride(0),
              ldo, LIBRARY_WORKSPACE_BYTES, int(which))


def _few_rows_operands(x: torch.Tensor, weight: torch.Tensor, most: int) -> bool:
    """Operands the few-rows kernels take: bfloat16 matrices, at most ``most`` rows of x, rows they can load."""
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or x.dim() != 2 or weight.dim() != 2:
        return False
    if not (0 < x.shape[0] <= most) or x.shape[1] != weight.shape[1]:
        return False
    if (x.shape[1] > 1 and x.stride(1) != 1) or (weight.shape[1] > 1 and weight.stride(1) != 1):
        return False
    return _skinny_ok(x, weight, x.shape[1], x.stride(0), weight.stride(0))


def linear_sums_supported(x: torch.Tensor, weight: torch.Tensor, most_rows: Optional[int] = None) -> bool:
    """Whether ``linear_sums`` takes this product: bfloat16, at most SUMS_MAX_ROWS rows (or ``most_rows``,
    if that is fewer), and a shape at which the library's own product is not the faster one (the kernel
    library says: measured)."""
    most = SUMS_MAX_ROWS if most_rows is None else min(int(most_rows), SUMS_MAX_ROWS)
    if not _few_rows_operands(x, weight, most):
        return False
    return bool(_lib.load().zi_gemm_skinny_pays(int(x.shape[0]), int(weight.shape[0]), int(weight.shape[1])))


def linear_splits(M: int, N: int, K: int) -> int:
    """Partial sums the few-rows product with a weight matrix [N, K] leaves: a function of N and K alone."""
    return int(_lib.load().zi_gemm_skinny_splits(int(M), int(N), int(K)))


def linear_sums(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x[M,K] . weight[N,K]^T for M <= SUMS_MAX_ROWS as float32 partial sums [S, M, N], S =
    ``linear_splits(M, N, K)``, without bias: the consumer adds them in rising order."""
    _gpu("linear_sums", x, weight, out)
    if not linear_sums_supported(x, weight):
        raise ValueError(f"linear_sums: needs bfloat16 x and weight, at most {SUMS_MAX_ROWS} rows, 16-byte aligned rows")
    M, K = x.shape
    N = weight.shape[0]
    S = linear_splits(M, N, K)
    if out is None:
        out = torch.empty((S, M, N), dtype=torch.float32, device=x.device)
    if tuple(out.shape) != (S, M, N) or out.dtype != torch.float32 or not out.is_contiguous():
        raise ValueError(f"linear_sums: out must be a contiguous float32 [{S}, {M}, {N}] tensor")
    _lib.call("zi_gemm_skinny", _p(out), F32, 1, _p(x), _p(weight), c_void_p(0), M, N, K, x.stride(0), weight.stride(0),
              N, c_void_p(0), 0, _stream())
    return out


def linear_swiglu_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    # (beyond 64 rows the kernel for many rows never cuts k under this epilogue)
    return (_few_rows_operands(x, weight, SWIGLU_MAX_ROWS) and weight.shape[0] % 16 == 0
            and (x.shape[0] > FEW_ROWS or linear_splits(x.shape[0], weight.shape[0], weight.shape[1]) == 1))


def linear_swiglu(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """up * silu(gate) of x . weight^T in one kernel, for a weight [2I, K] whose rows are 8 gate rows,
    then the 8 up rows of the same columns, and so on; out [M, I] bfloat16."""
    _gpu("linear_swiglu", x, weight, out)
    if not linear_swiglu_supported(x, weight):
        raise ValueError("linear_swiglu: needs an unsplit bfloat16 few-rows product with 2I a multiple of 16")
    M, K = x.shape
    N = weight.shape[0]
    if out is None:
        out = torch.empty((M, N // 2), dtype=torch.bfloat16, device=x.device)
    ldo, wo = _rows(out, "linear_swiglu out")
    if tuple(out.shape) != (M, N // 2) or out.dtype != torch.bfloat16:
        raise ValueError(f"linear_swiglu: out must be bfloat16 [{M}, {N // 2}]")
    _lib.call("zi_gemm_skinny", _p(out), BF16, 2, _p(x), _p(weight), c_void_p(0), M, N, K, x.stride(0), weight.stride(0),
              ldo, c_void_p(0), 0, _stream())
    return out


def reduce_sums(sums: torch.Tensor, bias: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """out[m,n] = sum_s sums[s,m,n] + bias[n], added in rising order."""
    _gpu("reduce_sums", sums, bias, out)
    if sums.dim() != 3 or sums.dtype != torch.float32 or not sums.is_contiguous():
        raise ValueError("reduce_sums: sums must be a contiguous float32 [S, M, N] tensor")
    S, M, N = sums.shape
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError(f"reduce_sums: bias must be bfloat16 [{N}]")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or torch.bfloat16, device=sums.device)
    ldo, wo = _rows(out, "reduce_sums out")
    if tuple(out.shape) != (M, N):
        raise ValueError("reduce_sums: out has the wrong shape")
    _lib.call("zi_reduce_splits", _p(out), _code(out, "reduce_sums out"), _p(sums), _p(bias), M, N, ldo, S, _stream())
    return out


SKINNY_MAX_ROWS = 64   # rows ``linear`` gives the few-rows kernels in one launch
FEW_ROWS = 64          # up to here they beat the library product: the weights stream once, x stays on the chip
# Products that leave partial sums (q/k/v, output, down: few weight rows, k cut over workgroups) go to the
# few-rows kernel up to this many rows: measured at 128 rows with the weights coming from memory, 1.5B sizes,
# 6.2 / 5.6 / 17.5 us against the library's 9.7 / 8.1 / 24.5; 7B sizes 20 / 16 / 55 against 20 / 16 / 92.  The
# gate/up product with its activation does not (37 against 24 + 5 us at the 1.5B sizes: every wavefront reads
# all of x from LDS for its 16 weight rows, and with 128 rows those reads bound it): FEW_ROWS stays its limit.
# Beyond 128 rows and up to 256 a kernel with 32 weight rows a wavefront (gemm_rows32.hip) takes the products whose
# weights have at least twice as many columns as rows (the down projection; the library decides,
# ``zi_gemm_skinny_pays``).  With the SwiGLU epilogue it loses to the library from 65 rows on (1.5B sizes at 128
# rows 32.5 against 26.7 us with the activation's own launch: 560 wavefronts of 32 rows are too few for the
# chip, and the epilogue forbids a cut of k): SWIGLU_MAX_ROWS stays at FEW_ROWS.
# (ZEDINFER_SUMS_MAX_ROWS=64 gives such products of more than 64 rows back to the library.)
SUMS_MAX_ROWS = max(FEW_ROWS, min(256, int(os.environ.get("ZEDINFER_SUMS_MAX_ROWS", "256") or 256)))
SWIGLU_MAX_ROWS = max(FEW_ROWS, min(256, int(os.environ.get("ZEDINFER_SWIGLU_MAX_ROWS", "64") or 64)))
_WORKSPACES = {}
_OUTGROWN_WORKSPACES: list = []


def _workspace(device: torch.device, floats: int) -> torch.Tensor:
    """A float32 scratch buffer per device that only grows (split partial sums live in it).  One that is
    outgrown is kept: a captured graph may still use it."""
    ws = _WORKSPACES.get(device)
    if ws is None or ws.numel() < floats:
        if ws is not None:
            _OUTGROWN_WORKSPACES.append(ws)
            floats = max(floats, 2 * ws.numel())
        ws = torch.empty((max(floats, 1 << 20),), dtype=torch.float32, device=device)
        _WORKSPACES[device] = ws
    return ws


def _skinny_ok(x: torch.Tensor, w: torch.Tensor, K: int, ldx: int, ldw: int) -> bool:
    return (K >= 8 and K % 8 == 0 and ldx % 8 == 0 and ldw % 8 == 0 and x.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None, return_values: bool = False):
    """Index of the highest value of each row (lowest index among equals) as int32."""
    _gpu("argmax", logits, out)
    if logits.dim() == 1:
        logits = logits.unsqueeze(0)
    ld, V = _rows(logits, "argmax logits")
    R = logits.shape[0]
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _i32(out, "argmax out", R)
    vals = torch.empty((R,), dtype=torch.float32, device=logits.device) if return_values else None
    need = _lib.load().zi_argmax_workspace(R, V)      # long rows are cut over several workgroups
    ws = _workspace(logits.device, need) if need else None
    _lib.call("zi_argmax", _p(out), _p(vals), _p(logits), _code(logits, "argmax"), R, V, ld, _p(ws), need, _stream())
    return (out, vals) if return_values else out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           penalty: torch.Tensor, uniform: torch.Tensor, recent: Optional[torch.Tensor] = None,
           recent_len: Optional[torch.Tensor] = None, work: Optional[torch.Tensor] = None,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row of float32 logits [R, V]; per-row parameters are device tensors [R].
    A row with temperature <= 0 takes the argmax."""
    _gpu("sample", logits, temperature, top_k, top_p, penalty, uniform, recent, recent_len, work, out)
    if logits.dtype != torch.float32:
        raise TypeError("sample: logits must be float32")
    ld, V = _rows(logits, "sample logits")
    R = logits.shape[0]
    for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                        ("top_p", top_p, torch.float32), ("penalty", penalty, torch.float32),
                        ("uniform", uniform, torch.float32)):
        if t.dtype != dt or t.numel() < R or not t.is_contiguous():
            raise ValueError(f"sample: {name} must be a contiguous {dt} tensor with {R} entries")
    max_recent = 0
    if recent is not None:
        if recent.dim() != 2 or recent.shape[0] < R or recent.dtype != torch.int32 or not recent.is_contiguous():
            raise ValueError("sample: recent must be a contiguous int32 [R, max_recent] tensor")
        _i32(recent_len, "sample recent_len", R)
        max_recent = recent.shape[1]
    if work is None:
        work = torch.empty((R, V), dtype=torch.float32, device=logits.device)
    if work.dtype != torch.float32 or work.numel() < R * V or not work.is_contiguous():
        raise ValueError("sample: work must be a contiguous float32 buffer of R*V entries")
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _i32(out, "sample out", R)
    _lib.call("zi_sample", _p(out), _p(logits), ld, _p(work), R, V, _p(temperature), _p(top_k), _p(top_p),
              _p(penalty), _p(uniform), _p(recent), _p(recent_len) if recent is not None else c_void_p(0),
              max_recent, _stream())
    return out
