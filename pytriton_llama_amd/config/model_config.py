"""Typed model configuration read from an architecture's own config.json keys.

The reference keeps one dataclass per architecture and renames the HF keys
(lite_llama/models/model_config.py:6-106); unknown options are dropped and
unsupported ones ignored. Here the HF key names are the field names, every
size comes from the file, and an option the engine cannot honour is an error.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, fields
from typing import Any, Dict, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that this engine cannot run, with the reason."""


@dataclass(frozen=True)
class RopeScaling:
    """rope_scaling of config.json (lite_llama/models/RotaryEmbedding.py:80-83,
    133-136). ``rope_type`` "default" means plain frequencies."""
    rope_type: str = "default"
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 1.0
    original_max_position_embeddings: int = 0

    @classmethod
    def from_dict(cls, d: Optional[Dict[str, Any]]) -> "RopeScaling":
        if d is None:
            return cls()
        kind = d.get("rope_type", d.get("type"))
        if kind is None:
            raise ConfigError("rope_scaling has neither 'rope_type' nor 'type'")
        if kind == "default":
            return cls()
        if kind != "llama3":
            raise ConfigError(
                f"rope_scaling type {kind!r} is not supported (supported: 'default', 'llama3')")
        need = ("factor", "low_freq_factor", "high_freq_factor",
                "original_max_position_embeddings")
        missing = [k for k in need if k not in d]
        if missing:
            raise ConfigError(f"rope_scaling of type 'llama3' lacks {missing}")
        rs = cls("llama3", float(d["factor"]), float(d["low_freq_factor"]),
                 float(d["high_freq_factor"]), int(d["original_max_position_embeddings"]))
        if rs.factor <= 0 or rs.original_max_position_embeddings <= 0:
            raise ConfigError("rope_scaling factor and original_max_position_embeddings must be > 0")
        if rs.high_freq_factor == rs.low_freq_factor:
            raise ConfigError("rope_scaling high_freq_factor must differ from low_freq_factor")
        return rs


@dataclass(frozen=True)
class LlamaConfig:
    """config.json of ``LlamaForCausalLM``. Sizes have no defaults: a file that
    leaves one out is rejected rather than run with a guess (the reference
    fills 2048/8192/32... in, lite_llama/models/model_config.py:71-104)."""
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: RopeScaling
    tie_word_embeddings: bool
    tie_word_embeddings_given: bool = True    # False: config.json has no such key (tied by default)
    max_position_embeddings: Optional[int] = None
    bos_token_id: Optional[int] = None
    eos_token_id: Any = None
    initializer_range: float = 0.02
    torch_dtype: str = "bfloat16"
    architectures: Tuple[str, ...] = ("LlamaForCausalLM",)
    model_type: str = "llama"

    # ---- derived -----------------------------------------------------------
    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @property
    def eos_token_ids(self) -> Tuple[int, ...]:
        e = self.eos_token_id
        if e is None:
            return ()
        if isinstance(e, (list, tuple)):
            return tuple(int(x) for x in e)
        return (int(e),)

    # ---- construction --------------------------------------------------------
    REQUIRED = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                "num_attention_heads")

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LlamaConfig":
        missing = [k for k in cls.REQUIRED if d.get(k) is None]
        if missing:
            raise ConfigError(f"config.json lacks required keys: {missing}")
        if d.get("attention_bias", False):
            raise ConfigError("attention_bias=true is not supported (Llama projections have no bias)")
        if d.get("mlp_bias", False):
            raise ConfigError("mlp_bias=true is not supported (Llama projections have no bias)")
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act {act!r} is not supported (only 'silu')")
        heads = int(d["num_attention_heads"])
        kv_heads = d.get("num_key_value_heads")
        kv_heads = heads if kv_heads is None else int(kv_heads)
        hidden = int(d["hidden_size"])
        head_dim = d.get("head_dim")
        if head_dim is None:
            if heads <= 0 or hidden % heads:
                raise ConfigError(
                    f"hidden_size {hidden} is not a multiple of num_attention_heads {heads} "
                    "and head_dim is not given")
            head_dim = hidden // heads
        head_dim = int(head_dim)
        cfg = cls(
            vocab_size=int(d["vocab_size"]),
            hidden_size=hidden,
            intermediate_size=int(d["intermediate_size"]),
            num_hidden_layers=int(d["num_hidden_layers"]),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-5)),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            rope_scaling=RopeScaling.from_dict(d.get("rope_scaling")),
            # absent: tied, as the reference's LlamaConfig has it
            # (lite_llama/models/model_config.py:37-104), unless the checkpoint brings a head of
            # its own: then the file decides (tie_word_embeddings_given tells the model builder
            # that config.json was silent)
            tie_word_embeddings=bool(d.get("tie_word_embeddings", True)),
            tie_word_embeddings_given=d.get("tie_word_embeddings") is not None,
            max_position_embeddings=d.get("max_position_embeddings"),
            bos_token_id=d.get("bos_token_id"),
            eos_token_id=d.get("eos_token_id"),
            initializer_range=float(d.get("initializer_range", 0.02)),
            torch_dtype=str(d.get("torch_dtype", "bfloat16")),
            architectures=tuple(d.get("architectures") or ("LlamaForCausalLM",)),
            model_type=str(d.get("model_type", "llama")),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size",
                     "num_attention_heads", "num_key_value_heads", "head_dim"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_hidden_layers < 0:
            raise ConfigError("num_hidden_layers must be >= 0")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even for rotary pairs")
        if self.rms_norm_eps < 0:
            raise ConfigError("rms_norm_eps must be >= 0")
        if self.rope_theta <= 0:
            raise ConfigError("rope_theta must be > 0")

    def to_dict(self) -> Dict[str, Any]:
        """The config.json that reads back as this configuration."""
        d: Dict[str, Any] = {}
        for f in fields(self):
            v = getattr(self, f.name)
            if f.name == "rope_scaling":
                v = None if v.rope_type == "default" else {
                    "rope_type": v.rope_type, "factor": v.factor,
                    "low_freq_factor": v.low_freq_factor,
                    "high_freq_factor": v.high_freq_factor,
                    "original_max_position_embeddings": v.original_max_position_embeddings}
            elif isinstance(v, tuple):
                v = list(v)
            if f.name == "tie_word_embeddings_given":
                continue
            d[f.name] = v
        d["hidden_act"] = "silu"
        d["attention_bias"] = False
        d["mlp_bias"] = False
        return d


def read_config_json(folder: str) -> Dict[str, Any]:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {folder!r}")
    with open(path) as f:
        return json.load(f)
