"""Self-attention over a paged key/value cache.

Per token: qkv = h Wqkv^T (+ b); rotate q and k by the position; store k and v in the request's
pages; every query attends to the keys of its request at positions <= its own (within the
window, if there is one), read from the pages; out = attn Wo^T (+ b).

The reference's CausalSelfAttention (core/src/model_executor/models/llama/llama.rs:45-221) does
the same steps, but attends to the step's own k and v for prompts
(core/src/model_executor/layers/attention.rs:209-211) and to the pages only when decoding
(:213-231); here the pages are the only source, which is what lets one step hold portions of
prompts beside single decoded tokens. Query head h uses kv head h / (nh / nkv) (attention.rs:91-103).
"""
import math
from typing import Optional

import torch

from .base import (CacheBinding, CacheSpec, Mixer, PartSpec, PositionEncoding, Runtime, build_part,
                   register_part)
from .linear import FusedLinear, Linear


@register_part("mixer", "paged_attention")
class PagedAttention(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, num_heads: int, num_kv_heads: int,
                 head_dim: int, position: Optional[PartSpec] = None, qkv_bias: bool = False,
                 out_bias: bool = False, scale: Optional[float] = None, window: Optional[int] = None,
                 q_name: str = "q_proj", k_name: str = "k_proj", v_name: str = "v_proj", o_name: str = "o_proj"):
        super().__init__(prefix, rt)
        if num_heads % num_kv_heads != 0:
            raise ValueError("num_heads %d is not a multiple of num_kv_heads %d" % (num_heads, num_kv_heads))
        self.nh, self.nkv, self.d = int(num_heads), int(num_kv_heads), int(head_dim)
        check = getattr(rt.ops, "check_head_dim", None)
        if check is not None:
            check(self.d)          # a size no kernel takes is refused here, not at the first step
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.d)
        self.window = int(window) if window else None
        self.qkv = FusedLinear(prefix, rt, hidden_size,
                               [(q_name, self.nh * self.d), (k_name, self.nkv * self.d), (v_name, self.nkv * self.d)],
                               bias=qkv_bias)
        self.o = Linear(prefix, rt, o_name, self.nh * self.d, hidden_size, bias=out_bias)
        self.position: Optional[PositionEncoding] = None
        if position is not None:
            self.position = build_part("position", position, prefix, rt)

    def children(self):
        return [self.qkv, self.o] + ([self.position] if self.position is not None else [])

    def cache_spec(self) -> Optional[CacheSpec]:
        return CacheSpec(num_kv_heads=self.nkv, head_dim=self.d, window=self.window)

    may_return_pending = True

    @property
    def accepts_normed(self) -> bool:
        # the fused projection takes the norm into itself; an encoding that acts on the projections needs h
        return self.position is None or self.position.rotary_table() is not None

    def forward(self, h: torch.Tensor, ctx, binding: CacheBinding, pending_ok: bool = False):
        ops = self.rt.ops
        group = ctx.groups[binding.group]
        slots = group.slots if binding.writes_cache else None
        rotary = self.position.rotary_table() if self.position is not None else None
        if self.position is not None and rotary is None:
            # an encoding that acts on the projections itself
            qkv = self.qkv.forward(h)
            self.position.apply(qkv, self.nh, self.nkv, self.d, ctx.positions)
            if slots is not None:
                ops.rope_cache_write(qkv, self.nh, self.nkv, self.d, ctx.positions, None, 0, True, slots,
                                     binding.k_pages, binding.v_pages)
        else:
            table, rot, neox = rotary if rotary is not None else (None, 0, True)
            qkv = ops.qkv_rope_cache(h, self.qkv.weight, self.qkv.bias, self.nh, self.nkv, self.d, ctx.positions,
                                     table, rot, neox, slots, binding.k_pages, binding.v_pages)
        a = ops.paged_attention(qkv, binding.k_pages, binding.v_pages, group.block_tables, ctx.seg_of_token,
                                ctx.positions, self.nh, self.nkv, self.d, self.scale, self.window or 0, batch=ctx)
        return self.o.forward(a, pending_ok=pending_ok)
