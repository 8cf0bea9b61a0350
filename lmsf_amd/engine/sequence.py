"""A request's state between the engine, the scheduler and the sampler.

The reference keeps Sequence / SequenceGroup / SequenceData with logical token blocks
(core/src/common/sequence.rs:68-531). With one sequence per request and the pages owned by the
cache manager, one class is left: the token ids, how many of them are in the cache, and the state.
States and finish reasons follow core/src/common/sequence.rs:36-64.
"""
import enum
import time
from dataclasses import dataclass, field
from typing import Any, Hashable, List, Optional

from ..sampling.params import SamplingParams


class SequenceState(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED_STOPPED = "finished_stopped"
    FINISHED_LENGTH_CAPPED = "finished_length_capped"
    FINISHED_ABORTED = "finished_aborted"
    FINISHED_IGNORED = "finished_ignored"

    @property
    def finished(self) -> bool:
        return self.value in _FINISH_REASONS

    @property
    def finish_reason(self) -> Optional[str]:
        return _FINISH_REASONS.get(self.value)


# core/src/common/sequence.rs:56-64
_FINISH_REASONS = {"finished_stopped": "stop", "finished_length_capped": "length", "finished_aborted": "abort",
                   "finished_ignored": "length"}


@dataclass
class RequestMetrics:
    """core/src/common/sequence.rs:13-33."""
    arrival_time: float
    first_scheduled_time: Optional[float] = None
    first_token_time: Optional[float] = None
    finished_time: Optional[float] = None


@dataclass
class Sequence:
    request_id: Hashable
    prompt_token_ids: List[int]
    params: SamplingParams
    arrival: int                           # arrival number: the FCFS order, no clocks
    seed: int
    output_token_ids: List[int] = field(default_factory=list)
    state: SequenceState = SequenceState.WAITING
    num_computed: int = 0                  # tokens whose keys and values are in the cache
    num_preemptions: int = 0
    metrics: RequestMetrics = field(default_factory=lambda: RequestMetrics(time.monotonic()))
    prompt: Optional[str] = None           # the prompt's text, if the request came as text
    output_text: str = ""                  # text of the generated tokens (engines with a tokenizer)
    detokenizer: Any = None                # engine.detokenizer.IncrementalDetokenizer
    pending: int = 0                       # 1 while a sampled token is still on the device, unread by the host

    @property
    def length(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids) + self.pending

    @property
    def remaining(self) -> int:
        """Tokens that still have to go through the model before the next token can be sampled."""
        return self.length - self.num_computed

    def tokens(self, start: int, n: int) -> List[int]:
        """Token ids of positions start .. start + n - 1 (a pending token's place holds 0)."""
        if self.pending and start + n == self.length:
            return self.tokens_known(start, n - 1) + [0]
        return self.tokens_known(start, n)

    def tokens_known(self, start: int, n: int) -> List[int]:
        p = len(self.prompt_token_ids)
        if start + n <= p:
            return self.prompt_token_ids[start:start + n]
        if start >= p:
            return self.output_token_ids[start - p:start - p + n]
        return self.prompt_token_ids[start:] + self.output_token_ids[:start + n - p]

    @property
    def last_token_id(self) -> int:
        return self.output_token_ids[-1] if self.output_token_ids else self.prompt_token_ids[-1]
