"""The engine: requests in, tokens out, one step at a time.

LLMEngine mirrors the reference's (core/src/engine/llm_engine.rs:74-582): ``add_request``,
``abort_request``, ``has_unfinished_requests`` and ``step``, which schedules, runs the model once,
samples and applies the stop rules. ``LLM.generate`` is the convenience loop around it.
"""
import hashlib
import sys
import time
from typing import Any, Dict, Hashable, List, Optional, Sequence as Seq, Set, Union

import torch

from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler, SamplingRow
from .args import EngineArgs
from .batch import StepEntry
from .core import EngineCore, load_engine_core
from .detokenizer import IncrementalDetokenizer, load_tokenizer
from .metrics import Metrics, init_logging
from .outputs import RequestOutput
from .scheduler import Scheduler, SchedulerConfig, StepPlan
from .sequence import Sequence, SequenceState


class _InFlight:
    """A step that has been launched: its plan, the requests it samples for and where their tokens will be."""

    __slots__ = ("plan", "sampled", "tokens_dev", "t_start", "host_tokens", "event")

    def __init__(self, plan, sampled, tokens_dev, t_start):
        self.plan, self.sampled, self.tokens_dev, self.t_start = plan, sampled, tokens_dev, t_start
        self.host_tokens = None
        self.event = None


class LLMEngine:
    def __init__(self, args: EngineArgs, ops: Any = None):
        args.verify()
        self.args = args
        self.core: EngineCore = load_engine_core(
            args.model or None, dtype=args.dtype, block_size=args.block_size, max_model_len=args.max_model_len,
            num_pages=args.num_gpu_blocks_override, gpu_memory_utilization=args.gpu_memory_utilization,
            max_num_seqs=args.max_num_seqs, max_num_batched_tokens=args.max_num_batched_tokens, device=args.device,
            ops=ops, load_format=args.load_format, seed=args.seed, enforce_eager=args.enforce_eager,
            keep_float32_weights=args.keep_float32_weights)
        max_len = self.core.max_model_len
        budget = args.max_num_batched_tokens or max(max_len, 2048)      # core/src/common/config.rs:301-307
        self.scheduler = Scheduler(SchedulerConfig(budget, args.max_num_seqs, max_len, args.prefill_chunk_size),
                                   self.core.storage.manager)
        self.sampler = Sampler(self.core.rt.ops, self.core.rt.device)
        self.eos_token_ids = set(self.core.config.eos_token_ids)
        if args.tune_products and self.core.rt.device.type == "cuda":
            # the shapes of a full step's products, as the reference profiles cuBLASLt's tactics per weight shape
            # and bucket of rows (tops/src/cublas.rs:121-223)
            self.tuned_products = self.core.executor.tune_products(
                sorted({budget, min(budget, args.prefill_chunk_size or budget)}))
        self.tokenizer = None if args.skip_tokenizer_init else load_tokenizer(args.model)
        self._arrivals = 0
        self._requests: Dict[Hashable, Sequence] = {}
        self.stats = {"steps": 0, "tokens": 0, "generated_tokens": 0, "preemptions": 0}
        # --log-dir / --alsologtostderr as in the reference (common/src/tracing.rs:1-22): without either the
        # engine does not log; the metrics are kept either way and reported once a minute where there is a log
        self.logger = init_logging(args.log_dir, args.alsologtostderr) if (args.log_dir or args.alsologtostderr) else None
        self.metrics = Metrics(logger=self.logger)
        self.last_step: Dict[str, Any] = {}
        # one step may be in flight on the GPU while the host prepares the next (see ``step``)
        self.run_ahead = bool(getattr(args, "run_ahead", True))
        self._inflight: Optional[_InFlight] = None
        self._undelivered: List[RequestOutput] = []          # outputs finished by a step() that then raised
        self._token_slots = [[None, None], [None, None]]     # pinned buffer and event, two steps in turn
        self._token_turn = 0

    @classmethod
    def from_engine_args(cls, args: EngineArgs) -> "LLMEngine":
        return cls(args)

    # ------------------------------------------------------------------ requests

    def add_request(self, request_id: Hashable, prompt: Union[str, Seq[int], None],
                    sampling_params: Optional[SamplingParams] = None,
                    prompt_token_ids: Optional[Seq[int]] = None) -> None:
        """core/src/engine/llm_engine.rs:136-169: ``prompt`` is text, encoded with the model folder's
        tokenizer unless ``prompt_token_ids`` brings the ids; a list of token ids in its place is
        taken as the ids."""
        if request_id in self._requests:
            raise ValueError("request id %r is already in use" % (request_id,))
        params = sampling_params or SamplingParams()
        params.verify()
        text: Optional[str] = None
        if isinstance(prompt, str):
            text = prompt
            if prompt_token_ids is None:
                if self.tokenizer is None:
                    raise ValueError("request %r: a text prompt needs %s/tokenizer.json; give token ids instead"
                                     % (request_id, self.args.model or "<model>"))
                prompt_token_ids = self.tokenizer.encode(prompt, add_special_tokens=True)
        elif prompt_token_ids is None:
            prompt_token_ids = prompt
        if prompt_token_ids is None:
            raise ValueError("request %r has no prompt" % (request_id,))
        if params.stop and self.tokenizer is None:
            raise ValueError("request %r: stop strings need %s/tokenizer.json; use stop_token_ids"
                             % (request_id, self.args.model or "<model>"))
        ids = [int(t) for t in prompt_token_ids]
        V = self.core.config.vocab_size
        if not ids:
            raise ValueError("request %r has an empty prompt" % (request_id,))
        bad = [t for t in ids if not (0 <= t < V)]
        if bad:
            raise ValueError("request %r: token id %d outside the vocabulary of %d" % (request_id, bad[0], V))
        seed = params.seed
        if seed is None:
            h = hashlib.sha256(("%d:%d" % (self.args.seed, self._arrivals)).encode()).digest()
            seed = int.from_bytes(h[:8], "little")
        seq = Sequence(request_id, ids, params, self._arrivals, seed, prompt=text)
        if self.tokenizer is not None:
            seq.detokenizer = IncrementalDetokenizer(self.tokenizer, len(ids), params.skip_special_tokens)
        self._arrivals += 1
        self._requests[request_id] = seq
        self.scheduler.add(seq)
        self.metrics.counter("llm.prompt_recv")                   # core/src/engine/llm_engine.rs:794-795
        self.metrics.gauge("llm.alive_prompt", len(self._requests))

    def abort_request(self, request_id: Hashable) -> None:
        """core/src/engine/llm_engine.rs:171-178."""
        seq = self.scheduler.abort(request_id)
        if seq is not None:
            seq.metrics.finished_time = time.monotonic()
        self._requests.pop(request_id, None)

    def has_unfinished_requests(self) -> bool:
        return self.scheduler.has_unfinished() or bool(self._undelivered)

    def get_num_unfinished_requests(self) -> int:
        return self.scheduler.num_unfinished()

    # ------------------------------------------------------------------ the step

    def step(self) -> List[RequestOutput]:
        """Schedule, run the model once, sample, apply the stop rules
        (core/src/engine/llm_engine.rs:536-582); returns the outputs of the step that has finished.

        The host runs one step ahead of the GPU where it can: once a step and its sampler are launched, the
        next step is scheduled and launched before the first one's tokens are read. Its single tokens come from
        where the sampler left them on the device (``StepEntry.prev_row``), everything else a step needs
        (positions, pages, block tables) does not depend on their values. The host's work between two steps
        then passes while the GPU computes. What cannot be known without the values: a request that ends with
        an end-of-sequence token or a stop string has one more token computed for nothing, which is dropped.
        A step is not launched ahead when a request of the step before reaches its length limit with the token
        being sampled, or uses penalties (which count the tokens on the host)."""
        # (what a step that failed half-way had already finished comes first)
        outputs: List[RequestOutput] = self._undelivered
        self._undelivered = []
        if self._inflight is None:
            self._inflight = self._launch(outputs, None)
            if self._inflight is None:
                return outputs
        cur = self._inflight
        ahead = None
        if self.run_ahead and self._may_run_ahead(cur):
            for seq in cur.sampled:
                seq.pending = 1           # counts as a token from here on; its value comes when ``cur`` is finished
            try:
                ahead = self._launch(outputs, cur)
            except BaseException:
                # the step ahead failed; the one in flight is sound: its tokens are read and its outputs kept for
                # the caller's next step(), with whatever the failed launch had already finished (ignored prompts)
                for seq in cur.sampled:
                    seq.pending = 0
                self._inflight = None
                self._finish(cur, outputs)
                self._undelivered = outputs
                raise
        self._finish(cur, outputs)
        self._inflight = ahead if self.scheduler.has_unfinished() else None
        return outputs

    def _may_run_ahead(self, cur: "_InFlight") -> bool:
        limit = self.core.max_model_len
        for seq in cur.sampled:
            if seq.params.has_penalties or len(seq.output_token_ids) + 1 >= seq.params.max_tokens \
                    or seq.length + 1 >= limit:
                return False
        return True

    def _launch(self, outputs: List[RequestOutput], prev: Optional["_InFlight"]) -> Optional["_InFlight"]:
        """Schedule a step, launch it and its sampler; nothing here waits for the GPU. ``prev``: the step in
        flight, whose sampled tokens this one may take from the device."""
        t_start = time.monotonic()
        plan: StepPlan = self.scheduler.schedule()
        now = time.monotonic()
        for seq in plan.ignored:
            # as the reference's scheduler warns (core/src/sched/scheduler.rs:368-388)
            msg = ("Input prompt of request %r (%d tokens) is too long: it exceeds the limit of the engine or the capacity "
                   "of the cache; ignored" % (seq.request_id, len(seq.prompt_token_ids)))
            if self.logger is not None:
                self.logger.warning(msg)
            else:
                print("warning: " + msg, file=sys.stderr)
        for seq in plan.ignored + plan.capped:
            seq.metrics.finished_time = now
            self._requests.pop(seq.request_id, None)
            outputs.append(RequestOutput.from_sequence(seq, None))
        self.stats["preemptions"] += len(plan.preempted)
        if plan.empty:
            return None
        prev_row = {}
        if prev is not None:
            prev_row = {id(seq): i for i, seq in enumerate(prev.sampled) if seq.pending}
        entries = []
        pending_of = set()
        for s in plan.scheduled:
            row = prev_row.get(id(s.seq), -1)
            if row >= 0 and s.start + s.n_tokens == s.seq.length:
                pending_of.add(id(s.seq))
            else:
                row = -1
            entries.append(StepEntry(s.seq.request_id, s.seq.tokens(s.start, s.n_tokens),
                                     [s.n_tokens - 1] if s.samples else [], prev_row=row))
        logits = self.core.executor.step(entries, prev_tokens=prev.tokens_dev if pending_of else None)
        self.stats["steps"] += 1
        sampled = []
        for s in plan.scheduled:
            s.seq.num_computed += s.n_tokens
            if s.samples:
                sampled.append(s.seq)
        rows = [SamplingRow(seq.params, seq.seed, len(seq.output_token_ids) + seq.pending, seq.prompt_token_ids,
                            seq.output_token_ids) for seq in sampled]
        tokens_dev = self.sampler.sample_on_device(logits, rows)
        rec = _InFlight(plan, sampled, tokens_dev, t_start)
        if tokens_dev is not None and tokens_dev.is_cuda:
            # the tokens travel to pinned memory behind the sampler, ahead of whatever is launched next; the
            # event says when they are there
            n = tokens_dev.numel()
            slot = self._token_slots[self._token_turn]
            self._token_turn ^= 1
            if slot[0] is None or slot[0].numel() < n:
                slot[0] = torch.empty(max(n, 256), dtype=torch.int32, pin_memory=True)
                slot[1] = torch.cuda.Event()
            slot[0][:n].copy_(tokens_dev, non_blocking=True)
            slot[1].record()
            rec.host_tokens, rec.event = slot[0], slot[1]
        return rec

    def _finish(self, rec: "_InFlight", outputs: List[RequestOutput]) -> None:
        """Read the step's tokens, append them, apply the stop rules."""
        n = len(rec.sampled)
        if n == 0:
            tokens: List[int] = []
        elif rec.event is not None:
            rec.event.synchronize()
            tokens = rec.host_tokens[:n].tolist()
        else:
            tokens = [int(t) for t in rec.tokens_dev.tolist()]
        now = time.monotonic()
        n_sampled = 0
        for seq, tok in zip(rec.sampled, tokens):
            seq.pending = 0
            if seq.state.finished or self._requests.get(seq.request_id) is not seq:
                continue          # it ended with the step before (or was aborted): this token was one too many
            n_sampled += 1
            seq.output_token_ids.append(tok)
            if seq.metrics.first_token_time is None:
                seq.metrics.first_token_time = now
            piece = ""
            if seq.detokenizer is not None:
                piece = seq.detokenizer.step(seq.prompt_token_ids + seq.output_token_ids)
                seq.output_text += piece
            before = len(seq.output_text)
            check_stop(seq, self.core.max_model_len, self.eos_token_ids)
            if len(seq.output_text) < before:       # a stop string was cut off the end
                piece = piece[:max(0, len(piece) - (before - len(seq.output_text)))]
            if seq.state.finished:
                seq.metrics.finished_time = now
                self.scheduler.finish(seq)
                self._requests.pop(seq.request_id, None)
            outputs.append(RequestOutput.from_sequence(seq, tok, piece))
        n_tokens = rec.plan.num_tokens
        self.stats["generated_tokens"] += n_sampled
        self.stats["tokens"] += n_tokens
        self._record_step(rec.plan, n_tokens, n_sampled, outputs, rec.t_start)

    def _record_step(self, plan: StepPlan, n_tokens: int, n_sampled: int, outputs: List[RequestOutput],
                     t_start: float) -> None:
        """What the step did, for ``last_step`` and the metrics."""
        now = time.monotonic()
        decode = sum(1 for s in plan.scheduled if s.n_tokens == 1 and s.samples and s.start > 0)
        m = self.metrics
        self.last_step = {"tokens": n_tokens, "decode_tokens": decode, "prefill_tokens": n_tokens - decode,
                          "sequences": len(plan.scheduled), "sampled": n_sampled, "preempted": len(plan.preempted),
                          "free_pages": self.core.storage.manager.num_free_pages(0) if self.core.storage.manager.groups else 0,
                          "ms": (now - t_start) * 1e3}
        m.counter("llm.steps")
        m.counter("llm.tokens", n_tokens)
        m.counter("llm.generated_tokens", n_sampled)
        m.counter("llm.preemptions", len(plan.preempted))
        m.gauge("llm.alive_prompt", len(self._requests))
        m.gauge("llm.free_pages", self.last_step["free_pages"])
        m.histogram("llm.step_ms", self.last_step["ms"])
        m.histogram("llm.step_tokens", n_tokens)
        for out in outputs:
            if out.finished and out.metrics is not None and out.metrics.finished_time is not None:
                t = out.metrics
                m.histogram("llm.request_s", t.finished_time - t.arrival_time)
                if t.first_token_time is not None:
                    m.histogram("llm.first_token_s", t.first_token_time - t.arrival_time)
        m.maybe_report(now)


def check_stop(seq: Sequence, max_model_len: int, eos_token_ids: Set[int]) -> None:
    """The reference's rules in its order (core/src/engine/llm_engine.rs:221-258): the text ends with a
    stop string (which is cut off unless ``include_stop_str_in_output``), stop_token_ids, longer than
    max_model_len, max_tokens reached, EOS unless ignore_eos."""
    p = seq.params
    last = seq.last_token_id
    for stop in p.stop:
        if seq.output_text.endswith(stop):
            if not p.include_stop_str_in_output:
                seq.output_text = seq.output_text[:len(seq.output_text) - len(stop)]
            seq.state = SequenceState.FINISHED_STOPPED
            return
    if p.stop_token_ids and last in p.stop_token_ids:
        seq.state = SequenceState.FINISHED_STOPPED
    elif seq.length > max_model_len:
        seq.state = SequenceState.FINISHED_LENGTH_CAPPED
    elif len(seq.output_token_ids) >= p.max_tokens:
        seq.state = SequenceState.FINISHED_LENGTH_CAPPED
    elif not p.ignore_eos and last in eos_token_ids:
        seq.state = SequenceState.FINISHED_STOPPED
    elif seq.length >= max_model_len:
        # the next token would have no position left
        seq.state = SequenceState.FINISHED_LENGTH_CAPPED


class LLM:
    """``LLM(model=..., **engine options).generate(prompts, sampling_params)``: every prompt a list of
    token ids, or text if the model folder has a tokenizer.json; returns one finished RequestOutput per
    prompt, in the order given."""

    def __init__(self, model: str, **kwargs):
        self.engine = LLMEngine(EngineArgs(model=model, **kwargs))
        self._next_id = 0

    def generate(self, prompts: Seq[Union[str, Seq[int]]], sampling_params=None) -> List[RequestOutput]:
        if sampling_params is None or isinstance(sampling_params, SamplingParams):
            params_list = [sampling_params] * len(prompts)
        else:
            params_list = list(sampling_params)
            if len(params_list) != len(prompts):
                raise ValueError("one SamplingParams per prompt, or one for all")
        ids = []
        for prompt, params in zip(prompts, params_list):
            rid = self._next_id
            self._next_id += 1
            # every request gets its own copy: verify() may normalise fields
            p = None if params is None else SamplingParams(**vars(params))
            self.engine.add_request(rid, prompt, p)
            ids.append(rid)
        done: Dict[Hashable, RequestOutput] = {}
        while self.engine.has_unfinished_requests():
            for out in self.engine.step():
                if out.finished:
                    done[out.request_id] = out
        return [done[r] for r in ids]
