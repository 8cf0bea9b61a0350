"""From a step's logits to one token per request.

Order of the reference's Sampler::forward (core/src/model_executor/layers/sampler.rs:839-971):
penalties, temperature, top-k/top-p, min-p, then argmax for greedy rows and the exponential race
for random rows. The reference applies the first two in the model's dtype (:872-888) and needs a
sort of the vocabulary; here the logits are float32 from the start and two kernels do the whole
pipeline: one for the penalties (only when a request has any), one for everything else.
"""
from typing import List, Optional, Sequence

import torch

from .params import SamplingParams


class SamplingRow:
    """What the sampler needs to know about the request behind one row of logits."""

    __slots__ = ("params", "seed", "draw", "prompt_ids", "output_ids")

    def __init__(self, params: SamplingParams, seed: int, draw: int, prompt_ids: Sequence[int] = (),
                 output_ids: Sequence[int] = ()):
        self.params = params
        self.seed = int(seed)
        self.draw = int(draw)
        self.prompt_ids = prompt_ids
        self.output_ids = output_ids


class Sampler:
    def __init__(self, ops, device: torch.device):
        self.ops = ops
        self.device = device

    def sample(self, logits: torch.Tensor, rows: Sequence[SamplingRow]) -> List[int]:
        """One token id per row of float32 ``logits`` [R, V]."""
        R = len(rows)
        if logits.shape[0] != R:
            raise ValueError("%d rows of logits for %d requests" % (logits.shape[0], R))
        if R == 0:
            return []
        dev = self.device
        if any(r.params.has_penalties for r in rows):
            logits = logits.clone()
            tokens: List[int] = []
            offsets = [0]
            plens = []
            for r in rows:
                if r.params.has_penalties:
                    tokens.extend(r.prompt_ids)
                    tokens.extend(r.output_ids)
                    plens.append(len(r.prompt_ids))
                else:
                    plens.append(0)
                offsets.append(len(tokens))
            self.ops.apply_penalties(
                logits,
                torch.tensor(tokens or [0], dtype=torch.int32, device=dev),
                torch.tensor(offsets, dtype=torch.int32, device=dev),
                torch.tensor(plens, dtype=torch.int32, device=dev),
                torch.tensor([r.params.presence_penalty for r in rows], dtype=torch.float32, device=dev),
                torch.tensor([r.params.frequency_penalty for r in rows], dtype=torch.float32, device=dev),
                torch.tensor([r.params.repetition_penalty for r in rows], dtype=torch.float32, device=dev))
        if all(r.params.greedy for r in rows):
            out = self.ops.sample(logits)
        else:
            out = self.ops.sample(
                logits,
                torch.tensor([0.0 if r.params.greedy else r.params.temperature for r in rows], dtype=torch.float32,
                             device=dev),
                torch.tensor([r.params.top_k for r in rows], dtype=torch.int32, device=dev),
                torch.tensor([r.params.top_p for r in rows], dtype=torch.float32, device=dev),
                torch.tensor([r.params.min_p for r in rows], dtype=torch.float32, device=dev),
                torch.tensor([_to_i64(r.seed) for r in rows], dtype=torch.int64, device=dev),
                torch.tensor([r.draw & 0x7FFFFFFF for r in rows], dtype=torch.int32, device=dev))
        return [int(t) for t in out.tolist()]


def _to_i64(seed: int) -> int:
    seed &= 0xFFFFFFFFFFFFFFFF
    return seed - (1 << 64) if seed >= (1 << 63) else seed
