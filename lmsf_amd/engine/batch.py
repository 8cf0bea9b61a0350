"""The description of one step's batch, as the parts see it.

A step holds *segments*: for each request its next tokens (a portion of a prompt, or one decoded
token), laid out flat one after the other. The reference builds a padded rectangle of whole
prompts or a column of single decode tokens, never both
(core/src/worker/model_worker.rs:266-353 and :427-505); here there is one flat form for all.
"""
from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import torch


@dataclass
class StepEntry:
    """One request's part of a step: its next tokens and the places among them whose logits are wanted."""

    request_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()
    # >= 0: the entry is one token that the host does not know yet, row ``prev_row`` of the tokens that the step
    # before this one sampled (``ModelExecutor.step(..., prev_tokens=...)``); ``tokens`` then holds a placeholder
    prev_row: int = -1


@dataclass
class GroupView:
    """What the runs of one cache group need: where this step's keys go and where each request's pages are."""

    slots: torch.Tensor            # int32 [N]: page * page_size + offset of every token of the step
    block_tables: torch.Tensor     # int32 [S, W]: page of logical block b of segment s (0 where none)
    page_size: int


@dataclass
class StepContext:
    n_tokens: int
    n_segments: int
    token_ids: torch.Tensor        # int32 [N]
    positions: torch.Tensor        # int32 [N]: position of every token in its request
    seg_of_token: torch.Tensor     # int32 [N]: segment every token belongs to
    seg_starts: torch.Tensor       # int32 [S + 1]: first flat index of every segment, then N
    seg_first_pos: torch.Tensor    # int32 [S]: position of every segment's first token (0 = request begins)
    state_slots: torch.Tensor      # int32 [S]: state slot of every segment's request
    logit_rows: torch.Tensor       # int32 [R]: flat indices whose logits are wanted
    n_logit_rows: int
    groups: List[GroupView]
    # a step of single tokens: its tokens, the longest context first (int32 [N]); a kernel whose work grows with
    # the context starts its workgroups in this order
    longest_first: Optional[torch.Tensor] = None
    # host-side facts, for choosing kernels and for parts that loop over segments
    host_seg_starts: List[int] = field(default_factory=list)
    host_seg_lens: List[int] = field(default_factory=list)
    host_seg_first_pos: List[int] = field(default_factory=list)
    host_state_slots: List[int] = field(default_factory=list)
    request_ids: List[Hashable] = field(default_factory=list)
    max_seg_len: int = 0
    max_context: int = 0           # longest context (tokens in cache after this step) among the segments
    all_single: bool = False       # every segment has exactly one token (a pure decode step)
    aux: dict = field(default_factory=dict)   # what a part derived from this batch and keeps for the next layers
    replayed: bool = False         # the step is captured as a graph: parts must decide nothing from host facts
                                   # that change from step to step (max_context is the model's limit then)
