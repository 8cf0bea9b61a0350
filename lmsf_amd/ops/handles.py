"""What an operation may hand to the next one instead of a tensor."""
from typing import Optional, Tuple

import torch


class PendingProduct:
    """A bfloat16 product [M, N] whose sum over K is not finished: float32 partial sums ``partials``
    [n_split, M, N] and the bias that is still to be added. The kernel that consumes the product adds
    them up while it loads its operand, which saves the reduction kernel and one pass over the result;
    the value it sees is the one the reduction would have stored, to the bit.

    Only ``HipOps.linear(..., pending_ok=True)`` makes one, and only operations that say so take one
    (``HipOps.add_rms_norm`` as the branch); ``HipOps.materialize`` turns it into the tensor.
    """

    __slots__ = ("partials", "bias", "dtype")

    def __init__(self, partials: torch.Tensor, bias: Optional[torch.Tensor], dtype: torch.dtype):
        self.partials = partials
        self.bias = bias
        self.dtype = dtype

    @property
    def shape(self) -> Tuple[int, int]:
        return (self.partials.shape[1], self.partials.shape[2])

    @property
    def device(self) -> torch.device:
        return self.partials.device


class DeferredLinear:
    """A bfloat16 product x weight^T + bias [M, N] of one or two rows that has not been started: the norm
    that takes it as its branch runs it as a product that adds its result, rounded to bfloat16, straight
    into the float32 residual stream, so that the addition is no kernel of its own. Made and taken by the
    same operations as ``PendingProduct``."""

    __slots__ = ("x", "weight", "bias", "dtype")

    def __init__(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], dtype: torch.dtype):
        self.x = x
        self.weight = weight
        self.bias = bias
        self.dtype = dtype

    @property
    def shape(self) -> Tuple[int, int]:
        return (self.x.shape[0], self.weight.shape[0])

    @property
    def device(self) -> torch.device:
        return self.x.device


class ScaledRows:
    """The RMSNorm of the float32 residual stream [M, H], M up to 16, with its row factor still to come
    (RMSNorm is r * inv(r) * w with one inv per row, and (r * w * inv) W^T = inv * ((r * w) W^T)):
    ``xw`` is bf16(stream * (w + offset)) and ``sumsq`` [tiles][rows_per_tile] holds sums of stream^2 over a
    part of the columns each (16 columns, or what a workgroup produced), both written by the product before
    the norm
    (``HipOps.add_rms_norm(DeferredLinear, ..., defer_ok=True)``). The product that takes it
    (``HipOps.qkv_rope_cache``, ``HipOps.linear_gated``) multiplies its rows by rsqrt(sum / H + eps), which
    is the same product as with the normalised rows up to where the rounding falls. ``HipOps.materialize``
    runs the norm kernel on the stream instead."""

    __slots__ = ("xw", "sumsq", "tiles", "rows_per_tile", "stream", "weight", "eps", "weight_offset", "dtype")

    def __init__(self, xw: torch.Tensor, sumsq: torch.Tensor, tiles: int, rows_per_tile: int, stream: torch.Tensor,
                 weight: torch.Tensor, eps: float, weight_offset: float, dtype: torch.dtype):
        self.xw = xw
        self.sumsq = sumsq
        self.tiles = tiles
        self.rows_per_tile = rows_per_tile   # 16: written by the few-rows product; M: by the one-or-two-rows product
        self.stream = stream
        self.weight = weight
        self.eps = eps
        self.weight_offset = weight_offset
        self.dtype = dtype

    @property
    def shape(self) -> Tuple[int, int]:
        return tuple(self.xw.shape)

    @property
    def device(self) -> torch.device:
        return self.xw.device
