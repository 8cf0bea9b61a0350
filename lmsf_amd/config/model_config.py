"""Typed architecture configurations, read from the architecture's own config.json keys.

The reference parses config.json into a serde struct per architecture
(core/src/model_executor/models/llama/config.rs:6-27) behind an accessor trait
(core/src/model_executor/models/model.rs:8-37). Here a configuration is a frozen
dataclass with explicit defaults and validation; every size and constant that the model
code uses comes from one of its fields.
"""
import dataclasses
import json
import os
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that cannot be used; the message names the key."""


_MISSING = object()


def _take(d: Dict[str, Any], key: str, kind, default=_MISSING):
    """d[key] converted to ``kind``; a missing key without default is an error."""
    if key not in d or d[key] is None:
        if default is _MISSING:
            raise ConfigError("config.json: required key '%s' is missing" % key)
        return default
    v = d[key]
    try:
        if kind is bool:
            if not isinstance(v, bool):
                raise TypeError
            return v
        if kind is int:
            if isinstance(v, bool) or (isinstance(v, float) and v != int(v)):
                raise TypeError
            return int(v)
        if kind is float:
            if isinstance(v, bool):
                raise TypeError
            return float(v)
        if kind is str:
            if not isinstance(v, str):
                raise TypeError
            return v
    except (TypeError, ValueError):
        raise ConfigError("config.json: key '%s' has value %r, expected %s" % (key, v, kind.__name__))
    raise AssertionError(kind)


@dataclass(frozen=True)
class RopeScaling:
    """config.json's ``rope_scaling`` object. rope_type "llama3" rescales each frequency by its
    wavelength relative to the original context length; "default" changes nothing."""

    rope_type: str = "default"
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192

    KNOWN_TYPES = ("default", "llama3")

    @classmethod
    def from_dict(cls, d: Optional[Dict[str, Any]]) -> Optional["RopeScaling"]:
        if d is None:
            return None
        if not isinstance(d, dict):
            raise ConfigError("config.json: 'rope_scaling' must be an object or null, got %r" % (d,))
        kind = d.get("rope_type", d.get("type", "default"))
        if kind not in cls.KNOWN_TYPES:
            raise ConfigError("config.json: rope_scaling.rope_type %r is not supported (known: %s)"
                              % (kind, ", ".join(cls.KNOWN_TYPES)))
        if kind == "default":
            return cls()
        rs = cls(
            rope_type=kind,
            factor=_take(d, "factor", float),
            low_freq_factor=_take(d, "low_freq_factor", float),
            high_freq_factor=_take(d, "high_freq_factor", float),
            original_max_position_embeddings=_take(d, "original_max_position_embeddings", int),
        )
        if rs.factor <= 0 or rs.original_max_position_embeddings <= 0:
            raise ConfigError("config.json: rope_scaling factor and original_max_position_embeddings must be > 0")
        if rs.high_freq_factor <= rs.low_freq_factor:
            raise ConfigError("config.json: rope_scaling.high_freq_factor must exceed low_freq_factor")
        return rs

    def to_dict(self) -> Dict[str, Any]:
        if self.rope_type == "default":
            return {"rope_type": "default"}
        return {
            "rope_type": self.rope_type,
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }


_TORCH_DTYPES = ("float32", "bfloat16", "float16", "half", "float")


@dataclass(frozen=True)
class ArchConfig:
    """What every architecture's configuration gives the engine
    (the accessor trait of core/src/model_executor/models/model.rs:8-37)."""

    architecture: str
    vocab_size: int
    max_position_embeddings: int
    torch_dtype: str
    eos_token_ids: Tuple[int, ...]
    bos_token_id: Optional[int]

    def to_dict(self) -> Dict[str, Any]:  # pragma: no cover - interface
        raise NotImplementedError

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ArchConfig":  # pragma: no cover - interface
        raise NotImplementedError


@dataclass(frozen=True)
class LlamaConfig(ArchConfig):
    """config.json of LlamaForCausalLM.

    Keys of the reference's struct (core/src/model_executor/models/llama/config.rs:6-27) plus
    the ones it lacks and a correct engine needs: head_dim, attention_bias, mlp_bias,
    rope_scaling, and a tie_word_embeddings that is honoured.
    """

    hidden_size: int = 0
    intermediate_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    rope_scaling: Optional[RopeScaling] = None
    tie_word_embeddings: bool = False
    attention_bias: bool = False
    mlp_bias: bool = False
    hidden_act: str = "silu"

    ARCHITECTURE = "LlamaForCausalLM"
    MODEL_TYPE = "llama"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LlamaConfig":
        hidden = _take(d, "hidden_size", int)
        heads = _take(d, "num_attention_heads", int)
        if heads <= 0:
            raise ConfigError("config.json: num_attention_heads must be > 0")
        head_dim = _take(d, "head_dim", int, None)
        if head_dim is None:
            if hidden % heads != 0:
                raise ConfigError("config.json: hidden_size %d is not a multiple of num_attention_heads %d "
                                  "and no head_dim is given" % (hidden, heads))
            head_dim = hidden // heads
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, list):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)
        dtype = _take(d, "torch_dtype", str, _take(d, "dtype", str, "bfloat16"))
        cfg = cls(
            architecture=cls.ARCHITECTURE,
            vocab_size=_take(d, "vocab_size", int),
            max_position_embeddings=_take(d, "max_position_embeddings", int),
            torch_dtype=dtype,
            eos_token_ids=eos_ids,
            bos_token_id=_take(d, "bos_token_id", int, None),
            hidden_size=hidden,
            intermediate_size=_take(d, "intermediate_size", int),
            num_hidden_layers=_take(d, "num_hidden_layers", int),
            num_attention_heads=heads,
            num_key_value_heads=_take(d, "num_key_value_heads", int, heads),
            head_dim=head_dim,
            rms_norm_eps=_take(d, "rms_norm_eps", float),
            rope_theta=_take(d, "rope_theta", float, 10000.0),
            rope_scaling=RopeScaling.from_dict(d.get("rope_scaling")),
            tie_word_embeddings=_take(d, "tie_word_embeddings", bool, False),
            attention_bias=_take(d, "attention_bias", bool, False),
            mlp_bias=_take(d, "mlp_bias", bool, False),
            hidden_act=_take(d, "hidden_act", str, "silu"),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                     "num_attention_heads", "num_key_value_heads", "head_dim",
                     "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError("config.json: %s must be > 0, got %r" % (name, getattr(self, name)))
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError("config.json: num_attention_heads %d is not a multiple of num_key_value_heads %d"
                              % (self.num_attention_heads, self.num_key_value_heads))
        if self.head_dim % 2 != 0:
            raise ConfigError("config.json: head_dim %d must be even for rotary embedding" % self.head_dim)
        if not (self.rms_norm_eps > 0):
            raise ConfigError("config.json: rms_norm_eps must be > 0")
        if not (self.rope_theta > 0):
            raise ConfigError("config.json: rope_theta must be > 0")
        if self.hidden_act != "silu":
            raise ConfigError("config.json: hidden_act %r is not supported by LlamaForCausalLM (silu)"
                              % self.hidden_act)
        if self.torch_dtype not in _TORCH_DTYPES:
            raise ConfigError("config.json: torch_dtype %r is not one of %s"
                              % (self.torch_dtype, ", ".join(_TORCH_DTYPES)))
        for e in self.eos_token_ids:
            if not (0 <= e < self.vocab_size):
                raise ConfigError("config.json: eos_token_id %d outside vocabulary of %d" % (e, self.vocab_size))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architectures": [self.ARCHITECTURE],
            "model_type": self.MODEL_TYPE,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None if self.rope_scaling is None else self.rope_scaling.to_dict(),
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": self.attention_bias,
            "mlp_bias": self.mlp_bias,
            "hidden_act": self.hidden_act,
            "torch_dtype": self.torch_dtype,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": (None if not self.eos_token_ids else
                             self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)),
            "initializer_range": 0.02,
            "use_cache": True,
        }
        return d


def read_config_json(folder: str) -> Dict[str, Any]:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError("no config.json in model folder %r" % folder)
    with open(path) as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError("%s is not valid JSON: %s" % (path, e))
    if not isinstance(d, dict):
        raise ConfigError("%s does not hold a JSON object" % path)
    return d


def replace(cfg, **changes):
    """A copy of a configuration with fields changed, validated again."""
    new = dataclasses.replace(cfg, **changes)
    if hasattr(new, "validate"):
        new.validate()
    return new
