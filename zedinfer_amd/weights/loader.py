"""Binding checkpoint tensors to the names a model expects.

The reference looks weights up lazily, so a missing tensor only shows during
the first forward as "Tensor not found: <name>" (reference:
include/frontend/models/base.hpp:139-163; loading at src/frontend/models/base.cpp:1099-1382).
Here the whole expected set is checked right after the files are opened and
ONE error lists every missing tensor, every unexpected tensor and every wrong
shape.

Storage types.  Floating tensors stay in bfloat16 in the bfloat16 engine; a
tensor the file stores in 32-bit floating point stays 32-bit; float16 becomes
bfloat16.  In the float32 engine everything floating is widened to float32
(reference: base.cpp:1233-1239, :406-408).  Integer tables become int32.
"""
from __future__ import annotations

import sys
from dataclasses import dataclass
from typing import Dict, List, Mapping, Optional, Tuple

import torch

from .safetensors_io import SafetensorsFolder


class WeightError(ValueError):
    """The checkpoint does not hold what the model needs."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


@dataclass(frozen=True)
class WeightSpec:
    """What a part needs from the checkpoint for one parameter."""

    shape: Tuple[int, ...]
    kind: str = "float"              # "float" or "int"
    fallback: Optional[str] = None   # tensor to alias when this one is absent (tied head)
    # what the random-weights mode fills it with: "normal" (N(0, std)), "ones" (a gain: 1, or 1 + N(0, std)
    # with noisy gains) or "zeros"
    init: str = "normal"


def canonical_name(name: str) -> str:
    """Strip the wrappers checkpoints put before the decoder's own names
    (reference: map_weight_name, base.cpp:1386-1410)."""
    for prefix in ("model.", "language_model."):
        if name.startswith(prefix):
            name = name[len(prefix):]
    return name


def storage_dtype(file_dtype: torch.dtype, kind: str, engine_dtype: torch.dtype) -> torch.dtype:
    if kind == "int":
        return torch.int32
    if engine_dtype == torch.float32:
        return torch.float32
    if file_dtype in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def check_names(expected: Mapping[str, WeightSpec],
                found: Mapping[str, Tuple[int, ...]]) -> None:
    """Compare expected tensors with (canonical name -> shape) found; raise one WeightError."""
    exp = {canonical_name(n): (n, s) for n, s in expected.items()}
    missing: List[str] = []
    wrong: List[str] = []
    for cn, (n, spec) in exp.items():
        if cn not in found:
            fb = canonical_name(spec.fallback) if spec.fallback else None
            if fb is None or fb not in found:
                missing.append(n)
            continue
        if tuple(found[cn]) != tuple(spec.shape):
            wrong.append(f"{n}: expected {list(spec.shape)}, file has {list(found[cn])}")
    unexpected = sorted(n for n in found if n not in exp)
    if missing or wrong or unexpected:
        parts = []
        if missing:
            parts.append(f"missing tensors ({len(missing)}): " + ", ".join(sorted(missing)))
        if unexpected:
            parts.append(f"unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            parts.append(f"wrong shapes ({len(wrong)}): " + "; ".join(sorted(wrong)))
        raise WeightError("checkpoint does not match the model: " + " | ".join(parts),
                          missing=sorted(missing), unexpected=unexpected, wrong_shape=sorted(wrong))


def load_weights(folder: str, expected: Mapping[str, WeightSpec], engine_dtype: torch.dtype,
                 device: torch.device | str) -> Dict[str, torch.Tensor]:
    """Open every ``*.safetensors`` in ``folder``, check it against ``expected`` and
    return ``{expected name: tensor on device}``."""
    st = SafetensorsFolder(folder)
    try:
        by_canon: Dict[str, str] = {}
        for n in st.names():
            by_canon[canonical_name(n)] = n
        check_names(expected, {cn: st.entry(n).shape for cn, n in by_canon.items()})
        out: Dict[str, torch.Tensor] = {}
        for name, spec in expected.items():
            cn = canonical_name(name)
            if cn not in by_canon:
                continue  # tied: aliased below
            t = st.tensor(by_canon[cn])
            dt = storage_dtype(t.dtype, spec.kind, engine_dtype)
            out[name] = t.to(device=device, dtype=dt).contiguous()
        for name, spec in expected.items():
            if name not in out:
                out[name] = out[_expected_name(expected, spec.fallback)]
        if engine_dtype == torch.bfloat16:
            wide = [n for n, t in out.items() if t.dtype == torch.float32 and t.dim() >= 2]
            if wide:
                # said once per load: such a model runs, but far from the speed of a bfloat16 checkpoint
                print(f"[zedinfer_amd] {len(wide)} of {len(out)} tensors in {folder} are stored in 32 bits and stay so "
                      f"(first: {wide[0]}); their matrix products take the plain 32-bit kernel, not the matrix cores. "
                      "Store the checkpoint in bfloat16 for serving speed.", file=sys.stderr, flush=True)
        return out
    finally:
        st.close()


def _expected_name(expected: Mapping[str, WeightSpec], name: str) -> str:
    cn = canonical_name(name)
    for n in expected:
        if canonical_name(n) == cn:
            return n
    raise KeyError(name)
