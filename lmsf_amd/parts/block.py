"""Arrangements of a layer's parts around the residual stream."""
from typing import Optional

import torch

from .base import Block, CacheBinding, register_part


@register_part("block", "prenorm_residual")
class PreNormResidualBlock(Block):
    """stream += mixer(norm_in(stream)); stream += ffn(norm_post(stream)).

    core/src/model_executor/models/llama/llama.rs:286-340. As there, an addition is carried out by
    the norm that follows it (vllm/kernels/layernorm_kernels.cu:41-68): the block receives the
    previous block's output not yet added, and returns its feed-forward output not yet added.
    """

    graph_safe = True

    ROLES = ("input", "post_mixer")

    def forward(self, branch: Optional[torch.Tensor], residual: torch.Tensor, ctx,
                binding: CacheBinding) -> torch.Tensor:
        h = self.norms["input"].forward_add(branch, residual)
        a = self.mixer.forward(h, ctx, binding)
        h = self.norms["post_mixer"].forward_add(a, residual)
        return self.feed_forward.forward(h)
