"""From a step's logits to one token per request.

Order of the reference's Sampler::forward (core/src/model_executor/layers/sampler.rs:839-971):
penalties, temperature, top-k/top-p, min-p, then argmax for greedy rows and the exponential race
for random rows. The reference applies the first two in the model's dtype (:872-888) and needs a
sort of the vocabulary; here the logits are float32 from the start and two kernels do the whole
pipeline: one for the penalties (only when a request has any), one for everything else.
"""
from typing import List, Optional, Sequence

import numpy as np
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

    def _upload(self, words: "np.ndarray") -> torch.Tensor:
        """One copy to the device for everything a call needs: int32 words, float32 values as their bits. Through
        the kernels' pinned buffers where there are any (they take turns behind events), so that the host does not
        wait for the step that is computing."""
        upload = getattr(self.ops, "upload_ints", None)
        if upload is not None and self.device.type == "cuda":
            return upload(words, self.device)
        return torch.from_numpy(words).to(self.device, non_blocking=False)

    def sample(self, logits: torch.Tensor, rows: Sequence[SamplingRow]) -> List[int]:
        """One token id per row of float32 ``logits`` [R, V]."""
        out = self.sample_on_device(logits, rows)
        return [] if out is None else [int(t) for t in out.tolist()]

    def sample_on_device(self, logits: torch.Tensor, rows: Sequence[SamplingRow]) -> Optional[torch.Tensor]:
        """The same, left on the device (int32 [R]; None for no rows): nothing here waits for the GPU."""
        R = len(rows)
        if logits.shape[0] != R:
            raise ValueError("%d rows of logits for %d requests" % (logits.shape[0], R))
        if R == 0:
            return None
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
            T = max(len(tokens), 1)
            # tokens | offsets | prompt lengths | presence | frequency | repetition, in one upload
            words = np.zeros(T + (R + 1) + 4 * R, dtype=np.int32)
            words[:len(tokens)] = tokens
            words[T:T + R + 1] = offsets
            at = T + R + 1
            words[at:at + R] = plens
            fl = words[at + R:].view(np.float32)
            fl[0:R] = [r.params.presence_penalty for r in rows]
            fl[R:2 * R] = [r.params.frequency_penalty for r in rows]
            fl[2 * R:3 * R] = [r.params.repetition_penalty for r in rows]
            d = self._upload(words)
            f = d[at + R:].view(torch.float32)
            self.ops.apply_penalties(logits, d[:T], d[T:T + R + 1], d[at:at + R], f[0:R], f[R:2 * R], f[2 * R:3 * R])
        if all(r.params.greedy for r in rows):
            out = self.ops.sample(logits)
        else:
            # seeds (two words each) | temperature | top_p | min_p | top_k | draws, in one upload
            words = np.zeros(7 * R, dtype=np.int32)
            words[:2 * R].view(np.int64)[:] = [_to_i64(r.seed) for r in rows]
            fl = words[2 * R:5 * R].view(np.float32)
            fl[0:R] = [0.0 if r.params.greedy else r.params.temperature for r in rows]
            fl[R:2 * R] = [r.params.top_p for r in rows]
            fl[2 * R:3 * R] = [r.params.min_p for r in rows]
            words[5 * R:6 * R] = [r.params.top_k for r in rows]
            words[6 * R:7 * R] = [r.draw & 0x7FFFFFFF for r in rows]
            d = self._upload(words)
            seeds = d[:2 * R].view(torch.int64)
            fd = d[2 * R:5 * R].view(torch.float32)
            temperature, draws = fd[0:R], d[6 * R:7 * R]
            if all(r.params.top_k <= 0 and r.params.top_p >= 1.0 and r.params.min_p <= 0.0 for r in rows):
                # no row cuts anything: the kernel can split a row over several workgroups
                out = self.ops.sample(logits, temperature, None, None, None, seeds, draws)
            else:
                out = self.ops.sample(logits, temperature, d[5 * R:6 * R], fd[R:2 * R], fd[2 * R:3 * R], seeds, draws)
        return out


def _to_i64(seed: int) -> int:
    seed &= 0xFFFFFFFFFFFFFFFF
    return seed - (1 << 64) if seed >= (1 << 63) else seed
