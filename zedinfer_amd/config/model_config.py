"""Typed views of a model folder's ``config.json``.

Every size and constant of a model comes from here; no layer size is written
in code.  The keys, their defaults and which of them are required follow the
reference's parser (reference: src/frontend/models/base.cpp:683-720 for the
shared keys, :807-813 for the Qwen2 extras).
"""
from __future__ import annotations

import json
import os
import sys
from dataclasses import dataclass, asdict
from typing import Any, Dict, Mapping, Tuple


class ConfigError(ValueError):
    """A config.json that cannot describe a runnable model."""


_REQUIRED = (
    "hidden_size",
    "intermediate_size",
    "vocab_size",
    "max_position_embeddings",
    "num_hidden_layers",
    "num_attention_heads",
)


def _as_int(d: Mapping[str, Any], key: str) -> int:
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
        raise ConfigError(f"config.json: '{key}' must be an integer, got {v!r}")
    return int(v)


@dataclass(frozen=True)
class ModelConfig:
    """Keys shared by every decoder family the reference parses
    (reference: include/frontend/models/base.hpp:91-137)."""

    architectures: Tuple[str, ...] = ()
    model_type: str = "unknown"
    hidden_act: str = "silu"
    torch_dtype: str = "bfloat16"
    bos_token_id: int = 151643
    eos_token_ids: Tuple[int, ...] = (151643,)
    hidden_size: int = 0
    intermediate_size: int = 0
    vocab_size: int = 0
    max_position_embeddings: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False

    @property
    def eos_token_id(self) -> int:
        return self.eos_token_ids[0] if self.eos_token_ids else 151643

    # ---- parsing -------------------------------------------------------
    @classmethod
    def _base_kwargs(cls, d: Mapping[str, Any]) -> Dict[str, Any]:
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError("config.json lacks required key(s): " + ", ".join(missing))
        eos = d.get("eos_token_id", 151643)
        eos_ids = tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        nh = _as_int(d, "num_attention_heads")
        hidden = _as_int(d, "hidden_size")
        # The reference reads hidden_act (base.cpp:686) and computes SiLU whatever it says
        # (transformer_forward.cpp:128-137); a checkpoint trained with another activation would run and be
        # silently something else, so it is refused here.
        act = str(d.get("hidden_act") or "silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act '{act}' is not supported: the feed-forward computes 'silu'")
        # rope_scaling is not among the keys the reference parses (base.cpp:683-720): positions rotate by
        # rope_theta alone.  Said once, so that a long-context variant is not taken for what its config says.
        if d.get("rope_scaling") is not None:
            print("zedinfer_amd: config.json has 'rope_scaling'; it is ignored, as the reference ignores it "
                  "(src/frontend/models/base.cpp:683-720 does not parse it): angles come from rope_theta alone",
                  file=sys.stderr, flush=True)
        head_dim = int(d.get("head_dim") or 0)
        if head_dim == 0:
            if nh <= 0 or hidden % nh:
                raise ConfigError(
                    f"config.json: hidden_size {hidden} is not divisible by num_attention_heads {nh} "
                    "and no head_dim is given")
            head_dim = hidden // nh
        return dict(
            architectures=tuple(d.get("architectures") or ()),
            model_type=str(d.get("model_type") or "unknown"),
            hidden_act=act,
            torch_dtype=str(d.get("torch_dtype") or "bfloat16"),
            bos_token_id=int(d.get("bos_token_id", 151643)),
            eos_token_ids=eos_ids,
            hidden_size=hidden,
            intermediate_size=_as_int(d, "intermediate_size"),
            vocab_size=_as_int(d, "vocab_size"),
            max_position_embeddings=_as_int(d, "max_position_embeddings"),
            num_hidden_layers=_as_int(d, "num_hidden_layers"),
            num_attention_heads=nh,
            num_key_value_heads=int(d.get("num_key_value_heads", nh)),
            head_dim=head_dim,
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-6)),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
        )

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "ModelConfig":
        cfg = cls(**cls._base_kwargs(d))
        cfg.validate()
        return cfg

    @classmethod
    def from_json_file(cls, path: str) -> "ModelConfig":
        return cls.from_dict(read_config_json(path))

    # ---- checks --------------------------------------------------------
    def validate(self) -> None:
        pos = ("hidden_size", "intermediate_size", "vocab_size", "num_hidden_layers",
               "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings")
        for k in pos:
            if getattr(self, k) <= 0:
                raise ConfigError(f"config.json: '{k}' must be positive, got {getattr(self, k)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even for rotary encoding")
        if not (self.rms_norm_eps > 0):
            raise ConfigError(f"config.json: rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not (self.rope_theta > 0):
            raise ConfigError(f"config.json: rope_theta must be positive, got {self.rope_theta}")

    # ---- writing -------------------------------------------------------
    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        d["architectures"] = list(self.architectures)
        eos = list(d.pop("eos_token_ids"))
        d["eos_token_id"] = eos[0] if len(eos) == 1 else eos
        return d

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=2)


@dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    """Qwen2 adds the three sliding-window keys
    (reference: include/frontend/models/qwen2.hpp:10-15, base.cpp:807-813)."""

    sliding_window: int = 4096
    max_window_layers: int = 21
    use_sliding_window: bool = False

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Qwen2Config":
        kw = cls._base_kwargs(d)
        sw = d.get("sliding_window")
        kw["sliding_window"] = int(sw) if isinstance(sw, (int, float)) and not isinstance(sw, bool) else 4096
        kw["max_window_layers"] = int(d.get("max_window_layers", 21))
        kw["use_sliding_window"] = bool(d.get("use_sliding_window", False))
        cfg = cls(**kw)
        cfg.validate()
        return cfg

    def validate(self) -> None:
        super().validate()
        if self.use_sliding_window:
            if self.sliding_window <= 0:
                raise ConfigError(f"config.json: sliding_window must be positive, got {self.sliding_window}")
            if self.max_window_layers < 0:
                raise ConfigError(
                    f"config.json: max_window_layers must be non-negative, got {self.max_window_layers}")


def read_config_json(path: str) -> Dict[str, Any]:
    """Read ``config.json`` from a model folder or a file path."""
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json at {path}")
    with open(path) as f:
        try:
            return json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path} is not valid JSON: {e}") from e
