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
