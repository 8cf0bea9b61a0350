"""A decoder-only model assembled from a ModelSpec.

Embedding, the layers in the order of the schedule, final norm on the wanted rows, LM head
(core/src/model_executor/models/llama/llama.rs:397-476 is the reference's fixed version of this
loop). The model holds no sizes of its own: everything comes from the spec.
"""
import inspect
from typing import List, Optional, Sequence, Tuple

import torch

from ..parts.base import (Block, CacheBinding, CacheSpec, ModelSpec, Part, Runtime, ScheduleEntry, StateSpec,
                          build_part)


class DecoderModel:
    def __init__(self, spec: ModelSpec, rt: Runtime):
        self.spec = spec
        self.rt = rt
        self.embedding = build_part("embedding", spec.embedding, _prefix_of(spec.embedding), rt)
        self.blocks: List[Block] = []
        for ls in spec.layers:
            mixer = build_part("mixer", ls.mixer, _sub(ls.prefix, ls.mixer), rt)
            ffn = build_part("feed_forward", ls.feed_forward, _sub(ls.prefix, ls.feed_forward), rt)
            norms = {role: build_part("norm", ns, _sub(ls.prefix, ns), rt) for role, ns in ls.norms.items()}
            self.blocks.append(build_part("block", ls.block, ls.prefix, rt, mixer=mixer, feed_forward=ffn,
                                          norms=norms))
        self.final_norm = build_part("norm", spec.final_norm, _prefix_of(spec.final_norm), rt)
        self.head = build_part("head", spec.head, _prefix_of(spec.head), rt)
        self._head_takes_out = "out" in inspect.signature(self.head.forward).parameters
        self.schedule: Tuple[ScheduleEntry, ...] = tuple(spec.schedule)
        for i, e in enumerate(self.schedule):
            if not (0 <= e.layer < len(self.blocks)):
                raise ValueError("schedule entry %d names layer %d of %d" % (i, e.layer, len(self.blocks)))
            if e.cache_from is not None:
                if not (0 <= e.cache_from < i):
                    raise ValueError("schedule entry %d reads the cache of entry %r, which does not run before it"
                                     % (i, e.cache_from))
                if self.schedule[e.cache_from].cache_from is not None:
                    raise ValueError("schedule entry %d reads entry %d, which has no cache of its own"
                                     % (i, e.cache_from))
                a = self.blocks[e.layer].mixer.cache_spec()
                b = self.blocks[self.schedule[e.cache_from].layer].mixer.cache_spec()
                if a is None or b is None or (a.num_kv_heads, a.head_dim, a.value_dim) != (b.num_kv_heads, b.head_dim,
                                                                                          b.value_dim):
                    raise ValueError("schedule entry %d cannot read the cache of entry %d: cache shapes differ"
                                     % (i, e.cache_from))
        self.bindings: List[CacheBinding] = [CacheBinding() for _ in self.schedule]
        # a block may return an unfinished product where everything that ever receives it can take one
        takes = [self.blocks[e.layer].accepts_pending_branch for e in self.schedule[1:]] + [self.final_norm.accepts_pending]
        for li, b in enumerate(self.blocks):
            after = [t for e, t in zip(self.schedule, takes) if e.layer == li]
            b.pending_output_ok = bool(after) and all(after)

    # ------------------------------------------------------------------ structure

    def parts(self) -> List[Part]:
        """Every part once (a layer named twice in the schedule has one set of weights)."""
        out: List[Part] = []
        for top in [self.embedding] + list(self.blocks) + [self.final_norm, self.head]:
            out.extend(top.walk())
        return out

    def cache_requirements(self) -> List[Tuple[Optional[CacheSpec], Optional[StateSpec], Optional[int]]]:
        """Per schedule entry: (paged cache spec, state spec, entry whose cache is read instead)."""
        out = []
        for e in self.schedule:
            m = self.blocks[e.layer].mixer
            out.append((m.cache_spec(), m.state_spec(), e.cache_from))
        return out

    def bind_cache(self, bindings: Sequence[CacheBinding]) -> None:
        if len(bindings) != len(self.schedule):
            raise ValueError("need one cache binding per schedule entry")
        self.bindings = list(bindings)

    # ------------------------------------------------------------------ forward

    def forward(self, ctx, logits_out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Run the step's tokens; float32 logits [R, V] at ctx.logit_rows, in ``logits_out`` if one is given
        (a head that does not take ``out`` gets its result copied there)."""
        residual = self.embedding.forward(ctx.token_ids)
        branch = None
        for e, binding in zip(self.schedule, self.bindings):
            branch = self.blocks[e.layer].forward(branch, residual, ctx, binding)
        if ctx.n_logit_rows == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=residual.device)
        h = self.final_norm.forward_add(branch, residual, rows=ctx.logit_rows)
        if logits_out is None:
            return self.head.forward(h)
        if self._head_takes_out:
            return self.head.forward(h, out=logits_out)
        return logits_out.copy_(self.head.forward(h))


def _prefix_of(spec) -> str:
    p = spec.params.get("prefix")
    if p is None:
        raise ValueError("spec of kind %r needs a 'prefix' parameter" % spec.kind)
    return p


def _sub(layer_prefix: str, spec) -> str:
    """Prefix of a layer's part: the layer's prefix plus the spec's optional 'prefix' parameter."""
    sub = spec.params.get("prefix")
    return "%s.%s" % (layer_prefix, sub) if sub else layer_prefix
