"""Rotary position embedding.

Frequencies f_i = theta^(-2i/rot), angle = position * f_i, cos and sin kept as a float32 table
[max_positions, rot] = [cos | sin] (core/src/model_executor/layers/rotary_embedding.rs:46-66 builds
the same table, but with the base fixed to 10000 (:105), 4096 rows
(core/src/model_executor/models/llama/llama.rs:18) and cast to the model's dtype). The rotation
itself is done by the kernel that also writes the cache.

rope_scaling "llama3" changes each frequency by its wavelength L = 2 pi / f relative to the
original context length o: L < o / high_freq_factor keeps f, L > o / low_freq_factor gives
f / factor, in between (1 - s) f / factor + s f with s = (o / L - low) / (high - low).
"""
import math
from typing import Any, Callable, Mapping, Optional

import torch

from .base import PositionEncoding, Runtime, register_part


def inverse_frequencies(rotary_dim: int, theta: float, scaling: Optional[Mapping[str, Any]]) -> torch.Tensor:
    """float32 [rotary_dim / 2]."""
    exponent = torch.arange(0, rotary_dim, 2, dtype=torch.float32) / float(rotary_dim)
    inv = torch.reciprocal(torch.pow(torch.tensor(theta, dtype=torch.float32), exponent))
    kind = "default" if not scaling else scaling.get("rope_type", "default")
    if kind == "default":
        return inv
    if kind != "llama3":
        raise ValueError("rotary scaling %r is not supported (default, llama3)" % kind)
    factor = float(scaling["factor"])
    low, high = float(scaling["low_freq_factor"]), float(scaling["high_freq_factor"])
    orig = float(scaling["original_max_position_embeddings"])
    f = inv.to(torch.float64)
    wavelength = 2.0 * math.pi / f
    smooth = (orig / wavelength - low) / (high - low)
    blended = (1.0 - smooth) * f / factor + smooth * f
    scaled = torch.where(wavelength < orig / high, f, torch.where(wavelength > orig / low, f / factor, blended))
    return scaled.to(torch.float32)


@register_part("position", "rotary")
class RotaryEncoding(PositionEncoding):
    """style "neox" pairs (i, i + rot/2), "gptj" pairs (2i, 2i+1)
    (vllm/kernels/pos_encoding_kernels.cu:12-36)."""

    graph_safe = True

    def __init__(self, prefix: str, rt: Runtime, head_dim: int, theta: float, rotary_dim: Optional[int] = None,
                 scaling: Optional[Mapping[str, Any]] = None, style: str = "neox"):
        super().__init__(prefix, rt)
        self.head_dim = int(head_dim)
        self.rotary_dim = int(rotary_dim) if rotary_dim else self.head_dim
        if self.rotary_dim % 2 or self.rotary_dim > self.head_dim or self.rotary_dim <= 0:
            raise ValueError("rotary_dim %d must be even and within head_dim %d" % (self.rotary_dim, self.head_dim))
        if style not in ("neox", "gptj"):
            raise ValueError("rotary style %r unknown (neox, gptj)" % style)
        self.theta = float(theta)
        self.scaling = None if not scaling else dict(scaling)
        self.neox = style == "neox"
        self.table: Optional[torch.Tensor] = None

    def _key(self):
        sc = None if self.scaling is None else tuple(sorted(self.scaling.items()))
        return ("rotary_table", self.rotary_dim, self.theta, sc, self.rt.max_positions)

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        key = self._key()
        if key not in self.rt.shared:
            inv = inverse_frequencies(self.rotary_dim, self.theta, self.scaling)
            pos = torch.arange(self.rt.max_positions, dtype=torch.float32)
            angles = pos[:, None] * inv[None, :]
            table = torch.cat([torch.cos(angles), torch.sin(angles)], dim=1).contiguous()
            self.rt.shared[key] = table.to(self.rt.device)
        self.table = self.rt.shared[key]

    def rotary_table(self):
        """(table float32 [max_positions, rot], rotary_dim, neox) for the fused rotate-and-store kernel."""
        return self.table, self.rotary_dim, self.neox

    def apply(self, qkv: torch.Tensor, nh: int, nkv: int, d: int, positions: torch.Tensor) -> None:
        self.rt.ops.rope_cache_write(qkv, nh, nkv, d, positions, self.table, self.rotary_dim, self.neox,
                                     None, None, None)
