"""RMSNorm.

y = x * rsqrt(mean(x^2) + eps) * (w + weight_offset), in float32
(vllm/kernels/layernorm_kernels.cu:13-38; used as input_layernorm, post_attention_layernorm and
model.norm, core/src/model_executor/models/llama/llama.rs:362-374, :494-495). weight_offset is 0
for Llama and 1 for Gemma's "w + 1" (vllm/src/rms_norm.rs:54-56).
"""
from typing import Callable, Dict, Optional

import torch

from .base import Norm, Runtime, TensorDecl, register_part


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    graph_safe = True
    accepts_pending = True
    may_defer = True

    def __init__(self, prefix: str, rt: Runtime, size: int, eps: float, weight_offset: float = 0.0,
                 weight_name: str = "weight"):
        super().__init__(prefix, rt)
        self.size = int(size)
        self.eps = float(eps)
        self.weight_offset = float(weight_offset)
        self.weight_name = "%s.%s" % (prefix, weight_name)
        self.weight: Optional[torch.Tensor] = None

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        init = "ones" if self.weight_offset == 0.0 else "zeros"
        return {self.weight_name: TensorDecl((self.size,), init=init, keeps_float32=True)}

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        self.weight = fetch(self.weight_name).contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.rt.ops.add_rms_norm(x, None, self.weight, self.eps, self.rt.dtype,
                                        weight_offset=self.weight_offset)

    def forward_add(self, branch: Optional[torch.Tensor], residual: torch.Tensor,
                    rows: Optional[torch.Tensor] = None, defer_ok: bool = False):
        if defer_ok:
            return self.rt.ops.add_rms_norm(branch, residual, self.weight, self.eps, self.rt.dtype, rows=rows,
                                            weight_offset=self.weight_offset, defer_ok=True)
        return self.rt.ops.add_rms_norm(branch, residual, self.weight, self.eps, self.rt.dtype, rows=rows,
                                        weight_offset=self.weight_offset)
