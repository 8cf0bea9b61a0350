"""SamplingParams with the reference's names, defaults and checks
(core/src/common/sampling_params.rs:29-80 fields and defaults, :166-298 verify).

Options that need several sequences per request (n, best_of, beam search) or log-probabilities are
accepted only at their defaults: this engine keeps one sequence per request. Stop strings need the
model folder's tokenizer; the engine refuses them at ``add_request`` if it has none. ``seed`` is an
addition: a request with a seed draws the same
tokens whatever else is in the batch; without one the engine derives a seed from its own --seed and
the request's arrival number.
"""
from dataclasses import dataclass, field
from typing import List, Optional

SAMPLING_EPS = 1e-5   # core/src/common/sampling_params.rs:8


@dataclass
class SamplingParams:
    n: int = 1
    best_of: Optional[int] = 1
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    repetition_penalty: float = 1.0
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int = -1
    min_p: float = 0.0
    use_beam_search: bool = False
    length_penalty: float = 1.0
    early_stopping: bool = False
    stop: List[str] = field(default_factory=list)
    stop_token_ids: Optional[List[int]] = None
    include_stop_str_in_output: bool = False
    ignore_eos: bool = False
    max_tokens: int = 128
    logprobs: Optional[int] = None
    prompt_logprobs: Optional[int] = None
    skip_special_tokens: bool = True
    spaces_between_special_tokens: bool = True
    seed: Optional[int] = None

    def __post_init__(self):
        self.verify()

    @property
    def greedy(self) -> bool:
        return self.temperature < SAMPLING_EPS

    @property
    def has_penalties(self) -> bool:
        return (abs(self.presence_penalty) >= SAMPLING_EPS or abs(self.frequency_penalty) >= SAMPLING_EPS
                or abs(self.repetition_penalty - 1.0) >= SAMPLING_EPS)

    def verify(self) -> None:
        if self.n < 1:
            raise ValueError("n must be at least 1, got %r." % self.n)
        if self.best_of is not None and self.best_of < self.n:
            raise ValueError("best_of must be greater than or equal to n, got n=%r and best_of=%r."
                             % (self.n, self.best_of))
        if not (-2.0 <= self.presence_penalty <= 2.0):
            raise ValueError("presence_penalty must be in [-2, 2], got %r." % self.presence_penalty)
        if not (-2.0 <= self.frequency_penalty <= 2.0):
            raise ValueError("frequency_penalty must be in [-2, 2], got %r." % self.frequency_penalty)
        if not (0.0 < self.repetition_penalty <= 2.0):
            raise ValueError("repetition_penalty must be in (0, 2], got %r." % self.repetition_penalty)
        if self.temperature < 0.0:
            raise ValueError("temperature must be non-negative, got %r." % self.temperature)
        if not (0.0 < self.top_p <= 1.0):
            raise ValueError("top_p must be in (0, 1], got %r." % self.top_p)
        if self.top_k < -1 or self.top_k == 0:
            raise ValueError("top_k must be -1 (disable), or at least 1, got %r." % self.top_k)
        if not (0.0 <= self.min_p <= 1.0):
            raise ValueError("min_p must be in [0, 1], got %r." % self.min_p)
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be at least 1, got %r." % self.max_tokens)
        if self.use_beam_search:
            raise ValueError("use_beam_search is not supported: this engine keeps one sequence per request.")
        if self.n != 1 or (self.best_of is not None and self.best_of != 1):
            raise ValueError("n and best_of must be 1: this engine keeps one sequence per request.")
        if self.early_stopping:
            raise ValueError("early_stopping is not effective and must be False when not using beam search")
        if abs(self.length_penalty - 1.0) > SAMPLING_EPS:
            raise ValueError("length_penalty is not effective and must be the default value of 1.0 when not "
                             "using beam search.")
        if isinstance(self.stop, str):
            self.stop = [self.stop]
        if any(not isinstance(x, str) or not x for x in self.stop):
            raise ValueError("stop must be a list of non-empty strings.")
        if self.logprobs is not None or self.prompt_logprobs is not None:
            raise ValueError("logprobs and prompt_logprobs are not supported; trace replay gives the logits.")
        if self.stop_token_ids is not None and any(int(t) < 0 for t in self.stop_token_ids):
            raise ValueError("stop_token_ids must be non-negative.")
        if self.greedy:
            # core/src/common/sampling_params.rs:231-236: greedy ignores the cuts
            self.top_p, self.top_k, self.min_p = 1.0, -1, 0.0
