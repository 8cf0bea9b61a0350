"""Linear layers, with the fusion of several checkpoint matrices into one product.

y = x W^T (+ b), W stored [out, in]. The reference fuses q, k, v into one weight of
(nh + 2 nkv) d rows (core/src/model_executor/layers/linear.rs:499-728, row offsets :573-583) and
gate, up into one of 2 I rows (:325-497, offsets :364-366) by copying the checkpoint tensors into
row slices of a zeroed buffer at load time; the same is done here, for weights and biases alike.
"""
from typing import Callable, Dict, Optional, Sequence, Tuple

import torch

from .base import Part, Runtime, TensorDecl


class FusedLinear(Part):
    """One matrix product whose weight rows are the concatenation of several checkpoint tensors.

    ``sources`` is a list of (checkpoint sub-name, rows): the tensor ``prefix.sub-name.weight`` has
    shape [rows, in_features] and, with ``bias``, ``prefix.sub-name.bias`` has [rows]."""

    graph_safe = True

    def __init__(self, prefix: str, rt: Runtime, in_features: int, sources: Sequence[Tuple[str, int]],
                 bias: bool = False):
        super().__init__(prefix, rt)
        if not sources:
            raise ValueError("FusedLinear needs at least one source")
        self.in_features = int(in_features)
        self.sources = [(str(n), int(r)) for n, r in sources]
        self.out_features = sum(r for _, r in self.sources)
        self.has_bias = bool(bias)
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def _name(self, sub: str, what: str) -> str:
        return "%s.%s.%s" % (self.prefix, sub, what) if self.prefix else "%s.%s" % (sub, what)

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        out = {}
        for sub, rows in self.sources:
            out[self._name(sub, "weight")] = TensorDecl((rows, self.in_features))
            if self.has_bias:
                out[self._name(sub, "bias")] = TensorDecl((rows,))
        return out

    def _buffer(self, what: str, dtype: torch.dtype, device) -> torch.Tensor:
        """The fused tensor's memory. A weight's rows are laid out with the distance between two rows that the
        kernels ask for (``ops.weight_row_pad``: a few elements more than a row holds, so that rows do not all
        begin on the same memory channel); what is returned is the [out, in] view of it."""
        if what != "weight":
            return torch.empty((self.out_features,), dtype=dtype, device=device)
        pad_of = getattr(self.rt.ops, "weight_row_pad", None)
        pad = int(pad_of(self.in_features, dtype)) if pad_of is not None else 0
        buf = torch.empty((self.out_features, self.in_features + pad), dtype=dtype, device=device)
        return buf[:, :self.in_features]

    def _gather(self, fetch: Callable[[str], torch.Tensor], what: str) -> torch.Tensor:
        """The sources' tensors as the row slices of one buffer, allocated once; every source is copied in
        as it is read and dropped at once, so that beside the fused tensor only one source is alive at a time
        (core/src/model_executor/layers/linear.rs:573-583, :603-622 copy into a zeroed buffer likewise). If
        sources differ in element type the buffer takes the widest."""
        # the buffer is made before the first source is read: made after it, torch would cut it out of the block
        # that the source's conversion has just freed and leave a hole of the difference for good
        out = self._buffer(what, self.rt.dtype, self.rt.device)
        row = 0
        for sub, rows in self.sources:
            t = fetch(self._name(sub, what))
            if (t.dtype != out.dtype and t.dtype == torch.float32) or t.device != out.device:
                # a source stored in 32 bits: the buffer takes the widest type (and lies where the sources lie)
                wider = self._buffer(what, torch.float32 if t.dtype == torch.float32 else out.dtype, t.device)
                wider[:row].copy_(out[:row])
                out = wider
            out[row:row + rows].copy_(t)
            row += rows
            del t
        return out

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        self.weight = self._gather(fetch, "weight")
        if self.has_bias:
            self.bias = self._gather(fetch, "bias").to(self.weight.dtype)

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None, pending_ok: bool = False):
        if pending_ok:
            return self.rt.ops.linear(x, self.weight, self.bias, out_dtype=out_dtype, pending_ok=True)
        return self.rt.ops.linear(x, self.weight, self.bias, out_dtype=out_dtype)


class Linear(FusedLinear):
    """A single checkpoint matrix ``prefix.name.weight`` [out_features, in_features]."""

    def __init__(self, prefix: str, rt: Runtime, name: str, in_features: int, out_features: int, bias: bool = False):
        super().__init__(prefix, rt, in_features, [(name, out_features)], bias)
