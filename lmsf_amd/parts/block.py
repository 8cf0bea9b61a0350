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
    Where the norm that follows accepts it, the o and down products may stay unfinished
    (``PendingProduct``) and the norm's kernel adds up their partial sums; where a norm may defer
    its work and the part after it takes that, the norm runs inside that part's first product.
    """

    graph_safe = True

    ROLES = ("input", "post_mixer")

    @property
    def accepts_pending_branch(self) -> bool:
        return self.norms["input"].accepts_pending

    def forward(self, branch: Optional[torch.Tensor], residual: torch.Tensor, ctx,
                binding: CacheBinding) -> torch.Tensor:
        first, post = self.norms["input"], self.norms["post_mixer"]
        if first.may_defer and self.mixer.accepts_normed:
            h = first.forward_add(branch, residual, defer_ok=True)
        else:
            h = first.forward_add(branch, residual)
        if self.mixer.may_return_pending and post.accepts_pending:
            a = self.mixer.forward(h, ctx, binding, pending_ok=True)
        else:
            a = self.mixer.forward(h, ctx, binding)
        if post.may_defer and self.feed_forward.accepts_normed:
            h = post.forward_add(a, residual, defer_ok=True)
        else:
            h = post.forward_add(a, residual)
        if self.feed_forward.may_return_pending and self.pending_output_ok:
            return self.feed_forward.forward(h, pending_ok=True)
        return self.feed_forward.forward(h)
