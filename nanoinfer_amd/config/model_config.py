"""Typed configuration of the Llama family, read from the keys of ``config.json``.

The reference keeps seven integers of a file header plus constants chosen by an enum
(include/nanoinfer/model/config.h:13-57, src/model/model.cpp:134-195): theta, eps and the
rope-scaling numbers are fixed in code there.  Here every one of them is a key of
``config.json``; a key that the file must give and does not is an error that names it.
"""
from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple


class ConfigError(ValueError):
    """A ``config.json`` that cannot describe a model of this framework."""


@dataclass(frozen=True)
class RopeScaling:
    """The four numbers of llama3 frequency scaling (src/model/model.cpp:157-161 fixes them)."""

    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    @staticmethod
    def from_dict(d: Optional[Dict[str, Any]]) -> Optional["RopeScaling"]:
        if d is None:
            return None
        kind = d.get("rope_type", d.get("type"))
        if kind in (None, "default"):
            return None
        if kind != "llama3":
            raise ConfigError(f"rope_scaling.rope_type {kind!r} is not supported (known: 'default', 'llama3')")
        missing = [k for k in ("factor", "low_freq_factor", "high_freq_factor",
                               "original_max_position_embeddings") if k not in d]
        if missing:
            raise ConfigError(f"rope_scaling lacks {missing}")
        rs = RopeScaling(kind, float(d["factor"]), float(d["low_freq_factor"]),
                         float(d["high_freq_factor"]), int(d["original_max_position_embeddings"]))
        if rs.factor <= 0 or rs.high_freq_factor == rs.low_freq_factor or rs.low_freq_factor <= 0 \
                or rs.high_freq_factor <= 0 or rs.original_max_position_embeddings <= 0:
            raise ConfigError(f"rope_scaling has an impossible value: {d}")
        return rs

    def to_dict(self) -> Dict[str, Any]:
        return dataclasses.asdict(self)


_REQUIRED = ("hidden_size", "num_hidden_layers", "num_attention_heads", "vocab_size",
             "intermediate_size", "rms_norm_eps", "max_position_embeddings")


@dataclass(frozen=True)
class LlamaConfig:
    """What ``LlamaForCausalLM`` needs of ``config.json`` (keys read by tools/export_llama3.py:544-554
    plus those the reference fixes in code: rope_theta, rope_scaling, tie_word_embeddings, head_dim)."""

    architecture: str
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Optional[RopeScaling]
    max_position_embeddings: int
    tie_word_embeddings: bool
    hidden_act: str
    bos_token_id: Optional[int]
    eos_token_ids: Tuple[int, ...]
    torch_dtype: str

    @staticmethod
    def from_dict(d: Dict[str, Any]) -> "LlamaConfig":
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks the keys {missing}")
        archs = d.get("architectures") or []
        if not archs:
            raise ConfigError("config.json lacks 'architectures'")
        heads = int(d["num_attention_heads"])
        hidden = int(d["hidden_size"])
        kv_heads = int(d.get("num_key_value_heads") or heads)
        head_dim = d.get("head_dim")
        if head_dim is None:
            if hidden % heads:
                raise ConfigError(f"hidden_size {hidden} is not a multiple of num_attention_heads {heads} "
                                  "and head_dim is not given")
            head_dim = hidden // heads
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, (list, tuple)):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)
        for flag in ("attention_bias", "mlp_bias"):
            if d.get(flag, False):
                raise ConfigError(f"{flag}=true is not supported: the projections of this family carry no bias")
        cfg = LlamaConfig(
            architecture=str(archs[0]),
            hidden_size=hidden,
            num_hidden_layers=int(d["num_hidden_layers"]),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=int(head_dim),
            intermediate_size=int(d["intermediate_size"]),
            vocab_size=int(d["vocab_size"]),
            rms_norm_eps=float(d["rms_norm_eps"]),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            rope_scaling=RopeScaling.from_dict(d.get("rope_scaling")),
            max_position_embeddings=int(d["max_position_embeddings"]),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            hidden_act=str(d.get("hidden_act", "silu")),
            bos_token_id=None if d.get("bos_token_id") is None else int(d["bos_token_id"]),
            eos_token_ids=eos_ids,
            torch_dtype=str(d.get("torch_dtype", "float32")),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        positive = ("hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                    "head_dim", "intermediate_size", "vocab_size", "max_position_embeddings")
        for name in positive:
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} is odd: rotation works on pairs")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta}")
        if self.hidden_act != "silu":
            raise ConfigError(f"hidden_act {self.hidden_act!r} is not supported (known: 'silu')")

    def to_dict(self) -> Dict[str, Any]:
        """The ``config.json`` of this configuration."""
        d: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None if self.rope_scaling is None else self.rope_scaling.to_dict(),
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": self.hidden_act,
            "attention_bias": False,
            "mlp_bias": False,
            "torch_dtype": self.torch_dtype,
        }
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        return d


def read_config_json(folder: str) -> Dict[str, Any]:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {folder!r}")
    with open(path) as fh:
        try:
            d = json.load(fh)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path} is not valid JSON: {e}") from e
    if not isinstance(d, dict):
        raise ConfigError(f"{path} does not hold an object")
    return d
