"""Typed configuration of the Llama 3 dense decoder (`LlamaForCausalLM`).

Keys and defaults follow the metadata block of the reference's loader
(internal/engine/engine.go:450-699: layer count :452-456, width :459-461, head
count required :465-469, feed-forward width :473-478, kv heads default to heads
:482-506, head size = width / heads :509-511, context :515-519, rope base 10000
:523-530, eps 1e-5 :536-542) and its checks (internal/config/config.go:57-105;
heads % kv_heads in internal/engine/validation.go:52-54), with config.json's key
names in place of the GGUF ones.  `rope_scaling` (types `llama3` and `linear`; `default` means none) has no
counterpart in the reference.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, coerce, optional, require


@dataclass(frozen=True)
class RopeScaling:
    """`rope_scaling` of type `llama3` (low frequencies divided by `factor`, high ones kept, a
    linear blend between the two thresholds) or `linear` (every frequency divided by `factor`;
    the other fields are None)."""

    rope_type: str
    factor: float
    low_freq_factor: Optional[float] = None
    high_freq_factor: Optional[float] = None
    original_max_position_embeddings: Optional[int] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> Optional["RopeScaling"]:
        """None for the type `default` (frequencies as they are)."""
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: 'rope_scaling' must be an object, found {d!r}")
        kind = d.get("rope_type", d.get("type"))
        if kind is None:
            raise ConfigError("config.json: 'rope_scaling' has neither 'rope_type' nor 'type'")
        if kind == "default":
            return None
        if kind not in ("llama3", "linear"):
            raise ConfigError(
                f"config.json: rope_scaling type {kind!r} is not supported (supported: 'default', 'linear', 'llama3')"
            )
        keys = [("factor", float)]
        if kind == "llama3":
            keys += [("low_freq_factor", float), ("high_freq_factor", float), ("original_max_position_embeddings", int)]
        vals = {}
        for key, typ in keys:
            if key not in d or d[key] is None:
                raise ConfigError(f"config.json: rope_scaling.{key} is missing")
            vals[key] = coerce(d[key], "rope_scaling." + key, typ)
        if vals["factor"] < 1.0:
            raise ConfigError(f"config.json: rope_scaling.factor must be >= 1, found {vals['factor']}")
        if kind == "llama3":
            if not vals["high_freq_factor"] > vals["low_freq_factor"]:
                raise ConfigError(
                    "config.json: rope_scaling.high_freq_factor must exceed low_freq_factor "
                    f"(found {vals['high_freq_factor']} and {vals['low_freq_factor']})"
                )
            if vals["low_freq_factor"] <= 0:
                raise ConfigError("config.json: rope_scaling.low_freq_factor must be positive")
            if vals["original_max_position_embeddings"] <= 0:
                raise ConfigError("config.json: rope_scaling.original_max_position_embeddings must be positive")
        return cls(rope_type=kind, **vals)

    def to_dict(self) -> Dict[str, Any]:
        return {k: v for k, v in dataclasses.asdict(self).items() if v is not None}


@dataclass(frozen=True)
class LlamaConfig(ModelConfig):
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Optional[RopeScaling]
    tie_word_embeddings: bool
    bos_token_id: Optional[int]
    eos_token_ids: Tuple[int, ...]
    torch_dtype: str

    architecture = "LlamaForCausalLM"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LlamaConfig":
        hidden = require(d, "hidden_size")
        heads = require(d, "num_attention_heads")
        inter = require(d, "intermediate_size")
        layers = require(d, "num_hidden_layers")
        vocab = require(d, "vocab_size")
        kv_heads = optional(d, "num_key_value_heads", heads)
        if heads <= 0:
            raise ConfigError(f"config.json: 'num_attention_heads' must be positive, found {heads}")
        if "head_dim" in d and d["head_dim"] is not None:
            head_dim = coerce(d["head_dim"], "head_dim", int)
        else:
            if hidden % heads != 0:
                raise ConfigError(
                    f"config.json: 'hidden_size' {hidden} is not a multiple of "
                    f"'num_attention_heads' {heads} and no 'head_dim' is given"
                )
            head_dim = hidden // heads
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, (list, tuple)):
            eos_ids = tuple(coerce(e, "eos_token_id", int) for e in eos)
        else:
            eos_ids = (coerce(eos, "eos_token_id", int),)
        bos = d.get("bos_token_id")
        # newer config files keep the base and the scaling together under `rope_parameters`
        rope = d.get("rope_parameters") if isinstance(d.get("rope_parameters"), dict) else {}
        scaling = d.get("rope_scaling")
        if scaling is None and rope.get("rope_type", rope.get("type")) is not None:
            scaling = rope
        theta = d["rope_theta"] if d.get("rope_theta") is not None else rope.get("rope_theta", 10000.0)
        act = d.get("hidden_act", "silu")
        if act not in ("silu", "swish"):
            # the feed-forward is silu(gate) * up: internal/device/cpu_ref.go:132-149
            raise ConfigError(f"config.json: 'hidden_act' {act!r} is not supported (supported: 'silu')")
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key):
                # the reference accepts no bias tensor: internal/engine/engine.go:416-425
                raise ConfigError(f"config.json: {key!r} = true is not supported (projections have no bias)")
        cfg = cls(
            hidden_size=hidden,
            intermediate_size=inter,
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            vocab_size=vocab,
            max_position_embeddings=optional(d, "max_position_embeddings", 2048),
            rms_norm_eps=optional(d, "rms_norm_eps", 1e-5, float),
            rope_theta=coerce(theta, "rope_theta", float),
            rope_scaling=RopeScaling.from_dict(scaling) if scaling is not None else None,
            tie_word_embeddings=optional(d, "tie_word_embeddings", False, bool),
            bos_token_id=None if bos is None else coerce(bos, "bos_token_id", int),
            eos_token_ids=eos_ids,
            torch_dtype=str(d.get("torch_dtype") or d.get("dtype") or "bfloat16"),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for key in (
            "hidden_size",
            "intermediate_size",
            "num_hidden_layers",
            "num_attention_heads",
            "num_key_value_heads",
            "head_dim",
            "vocab_size",
            "max_position_embeddings",
        ):
            v = getattr(self, key)
            if key == "num_hidden_layers":
                if v < 0:
                    raise ConfigError(f"config.json: {key!r} must not be negative, found {v}")
            elif v <= 0:
                raise ConfigError(f"config.json: {key!r} must be positive, found {v}")
        if self.num_key_value_heads > self.num_attention_heads:
            raise ConfigError(
                f"config.json: 'num_key_value_heads' {self.num_key_value_heads} exceeds "
                f"'num_attention_heads' {self.num_attention_heads}"
            )
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"config.json: 'num_attention_heads' {self.num_attention_heads} is not a multiple of "
                f"'num_key_value_heads' {self.num_key_value_heads}"
            )
        if self.head_dim % 2 != 0:
            raise ConfigError(f"config.json: 'head_dim' must be even for the rotation, found {self.head_dim}")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"config.json: 'rms_norm_eps' must be positive, found {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"config.json: 'rope_theta' must be positive, found {self.rope_theta}")
        if self.torch_dtype not in ("bfloat16", "float32", "float16"):
            raise ConfigError(f"config.json: 'torch_dtype' {self.torch_dtype!r} is not supported")

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling.to_dict() if self.rope_scaling else None,
            "tie_word_embeddings": self.tie_word_embeddings,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": list(self.eos_token_ids) if len(self.eos_token_ids) != 1 else self.eos_token_ids[0],
            "torch_dtype": self.torch_dtype,
            "hidden_act": "silu",
            "attention_bias": False,
            "mlp_bias": False,
        }
        if not self.eos_token_ids:
            d["eos_token_id"] = None
        return d
