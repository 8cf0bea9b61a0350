"""Typed architecture configurations, read from the architecture's own config.json keys.

The reference parses config.json into a serde struct per architecture
(core/src/model_executor/models/llama/config.rs:6-27) behind an accessor trait
(core/src/model_executor/models/model.rs:8-37). Here the struct, its defaults and its validation are
C++ (csrc/host/llama_config.{h,cc}: one message per fault, naming the key); ``LlamaConfig`` and
``RopeScaling`` below are its face, frozen dataclasses whose fields are what the C++ side read. Every
size and constant that the model code uses comes from one of these fields.
"""
import ctypes
import dataclasses
import json
import os
from ctypes import Structure, c_char, c_double, c_int, c_int64
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

MAX_EOS_IDS = 16


class _NativeRopeScaling(Structure):
    _fields_ = [("present", c_int), ("rope_type", c_char * 16), ("factor", c_double), ("low_freq_factor", c_double),
                ("high_freq_factor", c_double), ("original_max_position_embeddings", c_int64)]


class _NativeLlamaConfig(Structure):
    _fields_ = ([(n, c_int64) for n in ("vocab_size", "max_position_embeddings", "hidden_size", "intermediate_size",
                                        "num_hidden_layers", "num_attention_heads", "num_key_value_heads", "head_dim")]
                + [("rms_norm_eps", c_double), ("rope_theta", c_double), ("rope_scaling", _NativeRopeScaling)]
                + [(n, c_int) for n in ("tie_word_embeddings", "attention_bias", "mlp_bias")]
                + [("hidden_act", c_char * 32), ("torch_dtype", c_char * 16), ("has_bos_token_id", c_int),
                   ("bos_token_id", c_int64), ("n_eos_token_ids", c_int), ("eos_token_ids", c_int64 * MAX_EOS_IDS)])


def _native(call: str, *args) -> None:
    """Calls the host library's ``call``; a refusal becomes a ConfigError with the library's message."""
    from ..host.library import last_error, load_host_library
    lib = load_host_library()
    if getattr(lib, call)(*args) != 0:
        raise ConfigError(last_error(lib))


def _as_json(d: Any, what: str) -> bytes:
    try:
        return json.dumps(d, allow_nan=False).encode()
    except (TypeError, ValueError) as e:
        raise ConfigError("%s cannot be written as JSON: %s" % (what, e))


class ConfigError(ValueError):
    """A config.json that cannot be used; the message names the key."""


@dataclass(frozen=True)
class RopeScaling:
    """config.json's ``rope_scaling`` object. rope_type "llama3" rescales each frequency by its
    wavelength relative to the original context length; "default" changes nothing."""

    rope_type: str = "default"
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192

    @classmethod
    def from_dict(cls, d: Optional[Dict[str, Any]]) -> Optional["RopeScaling"]:
        if d is None:
            return None
        native = _NativeRopeScaling()
        _native("lmsf_rope_scaling_parse", _as_json(d, "rope_scaling"), ctypes.byref(native))
        return cls._from_native(native) or cls()

    @classmethod
    def _from_native(cls, n: _NativeRopeScaling) -> Optional["RopeScaling"]:
        if not n.present:
            return None
        return cls(n.rope_type.decode(), n.factor, n.low_freq_factor, n.high_freq_factor,
                   int(n.original_max_position_embeddings))

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
        """Parsed, completed with defaults and validated by the host library."""
        n = _NativeLlamaConfig()
        _native("lmsf_llama_config_parse", _as_json(d, "the configuration"), ctypes.byref(n))
        return cls(
            architecture=cls.ARCHITECTURE,
            vocab_size=int(n.vocab_size),
            max_position_embeddings=int(n.max_position_embeddings),
            torch_dtype=n.torch_dtype.decode(),
            eos_token_ids=tuple(int(n.eos_token_ids[i]) for i in range(n.n_eos_token_ids)),
            bos_token_id=int(n.bos_token_id) if n.has_bos_token_id else None,
            hidden_size=int(n.hidden_size),
            intermediate_size=int(n.intermediate_size),
            num_hidden_layers=int(n.num_hidden_layers),
            num_attention_heads=int(n.num_attention_heads),
            num_key_value_heads=int(n.num_key_value_heads),
            head_dim=int(n.head_dim),
            rms_norm_eps=n.rms_norm_eps,
            rope_theta=n.rope_theta,
            rope_scaling=RopeScaling._from_native(n.rope_scaling),
            tie_word_embeddings=bool(n.tie_word_embeddings),
            attention_bias=bool(n.attention_bias),
            mlp_bias=bool(n.mlp_bias),
            hidden_act=n.hidden_act.decode(),
        )

    def _to_native(self) -> _NativeLlamaConfig:
        n = _NativeLlamaConfig()
        for name in ("vocab_size", "max_position_embeddings", "hidden_size", "intermediate_size", "num_hidden_layers",
                     "num_attention_heads", "num_key_value_heads", "head_dim", "rms_norm_eps", "rope_theta"):
            setattr(n, name, getattr(self, name))
        for name in ("tie_word_embeddings", "attention_bias", "mlp_bias"):
            setattr(n, name, 1 if getattr(self, name) else 0)
        for name, cap in (("hidden_act", 32), ("torch_dtype", 16)):
            text = str(getattr(self, name)).encode()
            if len(text) >= cap:
                raise ConfigError("config.json: %s %r is too long" % (name, getattr(self, name)))
            setattr(n, name, text)
        if self.bos_token_id is not None:
            n.has_bos_token_id, n.bos_token_id = 1, self.bos_token_id
        if len(self.eos_token_ids) > MAX_EOS_IDS:
            raise ConfigError("config.json: eos_token_id lists %d ids, at most %d are taken"
                              % (len(self.eos_token_ids), MAX_EOS_IDS))
        n.n_eos_token_ids = len(self.eos_token_ids)
        for i, e in enumerate(self.eos_token_ids):
            n.eos_token_ids[i] = e
        rs = self.rope_scaling
        if rs is not None and rs.rope_type != "default":
            n.rope_scaling.present = 1
            n.rope_scaling.rope_type = rs.rope_type.encode()
            n.rope_scaling.factor, n.rope_scaling.low_freq_factor = rs.factor, rs.low_freq_factor
            n.rope_scaling.high_freq_factor = rs.high_freq_factor
            n.rope_scaling.original_max_position_embeddings = rs.original_max_position_embeddings
        return n

    def validate(self) -> None:
        """The host library's checks on the fields as they are (after ``replace``)."""
        _native("lmsf_llama_config_validate", ctypes.byref(self._to_native()))

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
