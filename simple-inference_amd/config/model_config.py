"""Typed model configuration, read from the architecture's own config.json keys.

Every size and constant the model uses comes from here; no part of the engine
holds a number that config.json gives.  The reference reads the same keys in
``config.py:84-109`` (``ModelConfig.from_hf_config``) and derives ``head_dim``
and ``num_kv_groups`` in ``config.py:72-82``.  Unlike the reference this
configuration

* honours an explicit ``head_dim`` key (the reference always derives it),
* accepts ``rope_scaling: null`` as "no scaling" (the reference's model
  constructor dereferences it unconditionally, ``model/llama.py:77-86``),
* checks the keys the reference silently ignores (``hidden_act``,
  ``attention_bias``, ``mlp_bias``) and refuses values the engine does not
  implement instead of computing something else.
"""

from __future__ import annotations

import json
from dataclasses import dataclass, field, asdict
from pathlib import Path
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that is missing a key or holds a value the engine refuses."""


@dataclass(frozen=True)
class RopeScaling:
    """The ``rope_scaling`` object of config.json (reference: ``config.py:19-36``)."""

    rope_type: str = "default"
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "RopeScaling":
        # HF checkpoints older than the ``rope_type`` key spell it ``type``.
        rope_type = d.get("rope_type", d.get("type", "default"))
        out = cls(
            rope_type=str(rope_type),
            factor=float(d.get("factor", 1.0)),
            low_freq_factor=float(d.get("low_freq_factor", 1.0)),
            high_freq_factor=float(d.get("high_freq_factor", 4.0)),
            original_max_position_embeddings=int(d.get("original_max_position_embeddings", 8192)),
        )
        if out.rope_type not in ("default", "llama3"):
            raise ConfigError(
                f"rope_scaling.rope_type {out.rope_type!r} is not implemented "
                "(known: 'default', 'llama3')"
            )
        if out.rope_type == "llama3":
            if out.factor <= 0:
                raise ConfigError(f"rope_scaling.factor must be positive, got {out.factor}")
            if out.high_freq_factor == out.low_freq_factor:
                raise ConfigError("rope_scaling.high_freq_factor must differ from low_freq_factor")
        return out

    def to_dict(self) -> dict:
        return asdict(self)


_REQUIRED = (
    "hidden_size",
    "intermediate_size",
    "num_hidden_layers",
    "vocab_size",
    "num_attention_heads",
    "num_key_value_heads",
    "rms_norm_eps",
    "rope_theta",
    "max_position_embeddings",
)


@dataclass(frozen=True)
class LlamaConfig:
    """Hyperparameters of the dense pre-norm GQA decoder (``LlamaForCausalLM``)."""

    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    vocab_size: int
    num_attention_heads: int
    num_key_value_heads: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    head_dim: int = 0  # 0 → hidden_size // num_attention_heads
    rope_scaling: Optional[RopeScaling] = None
    bos_token_id: int = 128000
    eos_token_ids: Tuple[int, ...] = (128001,)
    tie_word_embeddings: bool = True
    torch_dtype: str = "bfloat16"
    architecture: str = "LlamaForCausalLM"
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False, repr=False)

    def __post_init__(self):
        pos = lambda name: getattr(self, name) > 0
        for name in ("hidden_size", "intermediate_size", "num_hidden_layers", "vocab_size",
                     "num_attention_heads", "num_key_value_heads", "max_position_embeddings"):
            if not isinstance(getattr(self, name), int) or not pos(name):
                raise ConfigError(f"{name} must be a positive integer, got {getattr(self, name)!r}")
        if self.head_dim == 0:
            if self.hidden_size % self.num_attention_heads:
                raise ConfigError(
                    f"hidden_size {self.hidden_size} is not divisible by num_attention_heads "
                    f"{self.num_attention_heads} and config.json gives no head_dim"
                )
            object.__setattr__(self, "head_dim", self.hidden_size // self.num_attention_heads)
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_attention_heads} is not divisible by "
                f"num_key_value_heads {self.num_key_value_heads}"
            )
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even for rotary pairs")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta}")
        if self.torch_dtype not in ("bfloat16", "float16", "float32"):
            raise ConfigError(f"torch_dtype {self.torch_dtype!r} is not one of bfloat16/float16/float32")

    # -- derived ---------------------------------------------------------
    @property
    def num_kv_groups(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @property
    def eos_token_id(self) -> int:
        return self.eos_token_ids[0]

    def kv_bytes_per_token(self, bytes_per_element: int = 2) -> int:
        """K and V of one token over all layers (reference: ``config.py:144-149``)."""
        return 2 * self.num_hidden_layers * self.num_key_value_heads * self.head_dim * bytes_per_element

    def num_parameters(self) -> int:
        h, i, v = self.hidden_size, self.intermediate_size, self.vocab_size
        q = self.num_attention_heads * self.head_dim
        kv = self.num_key_value_heads * self.head_dim
        per_layer = h * q + 2 * h * kv + q * h + 3 * h * i + 2 * h
        head = 0 if self.tie_word_embeddings else v * h
        return v * h + self.num_hidden_layers * per_layer + h + head

    # -- json --------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "LlamaConfig":
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required key(s): {', '.join(missing)}")
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act {act!r} is not implemented (the feed-forward is SwiGLU: 'silu')")
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key, False):
                raise ConfigError(f"{key}=true is not implemented (linear layers carry no bias)")
        scaling = d.get("rope_scaling")
        eos = d.get("eos_token_id", 128001)
        eos_ids = tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        archs = d.get("architectures") or ["LlamaForCausalLM"]
        known = set(cls.__dataclass_fields__) | {
            "architectures", "eos_token_id", "hidden_act", "attention_bias", "mlp_bias", "rope_scaling"}
        return cls(
            hidden_size=int(d["hidden_size"]),
            intermediate_size=int(d["intermediate_size"]),
            num_hidden_layers=int(d["num_hidden_layers"]),
            vocab_size=int(d["vocab_size"]),
            num_attention_heads=int(d["num_attention_heads"]),
            num_key_value_heads=int(d["num_key_value_heads"]),
            rms_norm_eps=float(d["rms_norm_eps"]),
            rope_theta=float(d["rope_theta"]),
            max_position_embeddings=int(d["max_position_embeddings"]),
            head_dim=int(d.get("head_dim") or 0),
            rope_scaling=RopeScaling.from_dict(scaling) if scaling is not None else None,
            bos_token_id=int(d.get("bos_token_id", 128000)),
            eos_token_ids=eos_ids,
            tie_word_embeddings=bool(d.get("tie_word_embeddings", True)),
            torch_dtype=str(d.get("torch_dtype", "bfloat16")),
            architecture=str(archs[0]),
            extra={k: v for k, v in d.items() if k not in known},
        )

    def to_dict(self) -> dict:
        """The config.json that reads back to this configuration."""
        d = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "vocab_size": self.vocab_size,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "hidden_act": "silu",
            "attention_bias": False,
            "mlp_bias": False,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling.to_dict() if self.rope_scaling else None,
            "max_position_embeddings": self.max_position_embeddings,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0],
            "tie_word_embeddings": self.tie_word_embeddings,
            "torch_dtype": self.torch_dtype,
        }
        return d


def read_config_json(folder_or_file) -> dict:
    """The dictionary of ``config.json`` in a model folder (or of the file itself)."""
    path = Path(folder_or_file)
    if path.is_dir():
        path = path / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json at {path}")
    with open(path) as f:
        return json.load(f)
