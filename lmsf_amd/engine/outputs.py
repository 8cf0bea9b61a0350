"""What the engine hands back per request and step
(core/src/common/output.rs:5-132: RequestOutput with its CompletionOutputs). The text fields are
filled by engines that have the model's tokenizer and are empty otherwise."""
from dataclasses import dataclass
from typing import Hashable, List, Optional

from .sequence import RequestMetrics, Sequence


@dataclass
class CompletionOutput:
    index: int
    token_ids: List[int]
    latest_token: Optional[int]          # the token this step produced (None if the step produced none)
    finish_reason: Optional[str] = None  # "stop", "length", "abort"
    text: str = ""                       # the generated text so far
    latest_text: str = ""                # what this step added to it

    def finished(self) -> bool:
        return self.finish_reason is not None


@dataclass
class RequestOutput:
    request_id: Hashable
    prompt_token_ids: List[int]
    outputs: List[CompletionOutput]
    finished: bool
    metrics: Optional[RequestMetrics] = None
    prompt: Optional[str] = None

    @classmethod
    def from_sequence(cls, seq: Sequence, latest: Optional[int], latest_text: str = "") -> "RequestOutput":
        # a finished request gets lists of its own; while it runs, the output shows the request's live lists
        # (copying a long prompt for every request at every step costs more than the step's host work)
        done = seq.state.finished
        return cls(seq.request_id, list(seq.prompt_token_ids) if done else seq.prompt_token_ids,
                   [CompletionOutput(0, list(seq.output_token_ids) if done else seq.output_token_ids, latest,
                                     seq.state.finish_reason, seq.output_text, latest_text)],
                   done, seq.metrics, seq.prompt)
