"""Token embedding and the LM head.

Embedding: a row gather of the [V, H] table (core/src/model_executor/layers/vocab_parallel_embedding.rs:28-38),
written as the float32 residual stream, optionally scaled (Gemma multiplies by sqrt(H),
core/src/model_executor/models/gemma/gemma.rs:244). Head: logits = h W^T in float32
(core/src/model_executor/models/llama/llama.rs:471); with tied embeddings the head's matrix is the
embedding table (the reference parses tie_word_embeddings and ignores it, llama.rs:487-492).
"""
from typing import Callable, Dict, Optional

import torch

from .base import Part, Runtime, TensorDecl, register_part


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, prefix: str, rt: Runtime, vocab_size: int, hidden_size: int, scale: float = 1.0,
                 weight_name: str = "weight"):
        super().__init__(prefix, rt)
        self.vocab_size, self.hidden_size, self.scale = int(vocab_size), int(hidden_size), float(scale)
        self.weight_name = "%s.%s" % (prefix, weight_name)
        self.weight: Optional[torch.Tensor] = None

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        return {self.weight_name: TensorDecl((self.vocab_size, self.hidden_size))}

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        self.weight = fetch(self.weight_name).contiguous()

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        """int32 [N] -> float32 [N, H]."""
        return self.rt.ops.embedding(token_ids, self.weight, self.scale)


@register_part("head", "lm_head")
class LMHead(Part):
    """``weight_name`` is the full checkpoint name of the [V, H] matrix: the head's own, or the
    embedding table's when the two are tied (the loader then shares one device tensor)."""

    graph_safe = True

    def __init__(self, prefix: str, rt: Runtime, vocab_size: int, hidden_size: int, weight_name: Optional[str] = None,
                 bias: bool = False):
        super().__init__(prefix, rt)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight_name = weight_name or "%s.weight" % prefix
        self.bias_name = "%s.bias" % prefix if bias else None
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        out = {self.weight_name: TensorDecl((self.vocab_size, self.hidden_size))}
        if self.bias_name:
            out[self.bias_name] = TensorDecl((self.vocab_size,))
        return out

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        self.weight = fetch(self.weight_name).contiguous()
        if self.bias_name:
            self.bias = fetch(self.bias_name).to(self.weight.dtype).contiguous()

    def forward(self, h: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """[R, H] -> float32 logits [R, V], written into ``out`` if one is given."""
        if out is not None:
            return self.rt.ops.linear(h, self.weight, self.bias, out_dtype=torch.float32, out=out)
        return self.rt.ops.linear(h, self.weight, self.bias, out_dtype=torch.float32)
