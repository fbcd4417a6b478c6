"""Seeded random weights for a model description.

The reference has no such mode; benchmarks and tests here need models without
a checkpoint.  A tensor's values depend only on (seed, tensor name), so the
order in which tensors are made does not matter.  What a tensor is filled with
is the part's word (``WeightSpec.init``), not guessed from its name: "normal"
tensors (matrices, biases) are N(0, std); "ones" (the gains of norms) are 1, or
1 + N(0, std) when ``noisy_norms`` is set so that a forgotten weight multiply
shows; "zeros" (gains that are added to 1) are 0, or N(0, std) with
``noisy_norms``.
"""
from __future__ import annotations

import hashlib
import os
from typing import Dict, Mapping

import torch

from .loader import WeightSpec, canonical_name
from .safetensors_io import write_safetensors


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{canonical_name(name)}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFF_FFFF_FFFF_FFFF


def random_weights(expected: Mapping[str, WeightSpec], seed: int, dtype: torch.dtype,
                   device: torch.device | str = "cpu", std: float = 0.02,
                   noisy_norms: bool = False, tied: bool = True) -> Dict[str, torch.Tensor]:
    """Make every expected tensor.  A tensor with a ``fallback`` (a tied head) aliases
    it when ``tied`` is set and is drawn on its own otherwise."""
    device = torch.device(device)
    out: Dict[str, torch.Tensor] = {}
    for name, spec in expected.items():
        if spec.fallback is not None and tied:
            continue
        g = torch.Generator(device=device)
        g.manual_seed(_tensor_seed(seed, name))
        if spec.kind == "int":
            out[name] = torch.zeros(spec.shape, dtype=torch.int32, device=device)
            continue
        if spec.init == "ones":
            t = torch.ones(spec.shape, dtype=torch.float32, device=device)
            if noisy_norms:
                t += torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * std
        elif spec.init == "zeros":
            t = torch.zeros(spec.shape, dtype=torch.float32, device=device)
            if noisy_norms:
                t += torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * std
        elif spec.init == "normal":
            t = torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * std
        else:
            raise ValueError(f"tensor '{name}': unknown init '{spec.init}' (normal, ones, zeros)")
        out[name] = t.to(dtype)
    for name, spec in expected.items():
        if name not in out:
            out[name] = out[spec.fallback]
    return out


def write_model_folder(folder: str, config, expected: Mapping[str, WeightSpec], seed: int,
                       dtype: torch.dtype = torch.bfloat16, std: float = 0.02,
                       noisy_norms: bool = False) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` (a typed config
    with ``save``) with seeded random weights.  A tied head is not written."""
    os.makedirs(folder, exist_ok=True)
    config.save(folder)
    tensors = random_weights(expected, seed, dtype, "cpu", std, noisy_norms, tied=True)
    to_write = {n: t for n, t in tensors.items() if expected[n].fallback is None}
    write_safetensors(os.path.join(folder, "model.safetensors"), to_write,
                      metadata={"format": "pt", "seed": str(seed)})
    return folder
