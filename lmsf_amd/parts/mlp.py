"""Gated feed-forward: y = (act(x Wg^T) * (x Wu^T)) Wd^T.

core/src/model_executor/models/llama/llama.rs:223-274: gate and up are one fused product of 2 I
rows (gate first), then silu_and_mul (vllm/kernels/activation_kernels.cu:26-42), then down.
"""
import torch

from .base import FeedForward, Runtime, register_part
from .linear import FusedLinear, Linear


@register_part("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    graph_safe = True

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, intermediate_size: int, activation: str = "silu",
                 bias: bool = False, gate_name: str = "gate_proj", up_name: str = "up_proj",
                 down_name: str = "down_proj"):
        super().__init__(prefix, rt)
        if activation not in ("silu", "gelu"):
            raise ValueError("gated_mlp activation %r unknown (silu, gelu)" % activation)
        self.activation = activation
        self.gate_up = FusedLinear(prefix, rt, hidden_size,
                                   [(gate_name, intermediate_size), (up_name, intermediate_size)], bias=bias)
        self.down = Linear(prefix, rt, down_name, intermediate_size, hidden_size, bias=bias)

    def children(self):
        return [self.gate_up, self.down]

    may_return_pending = True
    accepts_normed = True

    def forward(self, h: torch.Tensor, pending_ok: bool = False):
        a = self.rt.ops.linear_gated(h, self.gate_up.weight, self.gate_up.bias, self.activation)
        return self.down.forward(a, pending_ok=pending_ok)
