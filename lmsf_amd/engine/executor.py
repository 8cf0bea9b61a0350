"""The step function: runs a batch of (request, its next tokens) from the cache and returns the
logits at the wanted places.

The reference's Worker::execute_model (core/src/worker/model_worker.rs:213-264) prepares either a
prompt batch or a decode batch, runs the model and samples inside the worker. Here the step only
produces logits: it takes pages for the new tokens, builds the flat batch, runs the model once over
exactly the tokens it was given, and commits them to the cache. Sampling is a separate call, so that
trace replay can take the logits.
"""
from collections import OrderedDict
from typing import Hashable, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import CacheError, CacheManager
from ..cache.storage import CacheStorage
from ..parts.base import Runtime
from .batch import GroupView, StepContext, StepEntry


class StepError(ValueError):
    """A step that cannot be run as given (unknown token id, too long a request, bad ``want``)."""


class ModelExecutor:
    def __init__(self, model, storage: CacheStorage, rt: Runtime, max_model_len: int, use_graphs: bool = True,
                 max_graph_batch: int = 256, max_graphs: int = 48, use_program: bool = True,
                 max_step_tokens: Optional[int] = None, max_step_seqs: Optional[int] = None):
        self.model = model
        self.storage = storage
        self.manager: CacheManager = storage.manager
        self.rt = rt
        self.max_model_len = int(max_model_len)
        if self.max_model_len > rt.max_positions:
            raise ValueError("max_model_len %d exceeds the positions the parts were built for (%d)"
                             % (self.max_model_len, rt.max_positions))
        self.vocab_size = model.spec.vocab_size
        self._pinned: Optional[torch.Tensor] = None
        self._pinned_np: Optional[np.ndarray] = None
        self._prev_tokens: Optional[torch.Tensor] = None   # the step before's sampled tokens, while a step is built
        # steps of single tokens run at a padded batch size and are captured as HIP graphs, one per padded
        # size and context bucket, the least recently used dropped beyond max_graphs
        self.pad_decode = all(getattr(p, "graph_safe", False) for p in model.parts())
        self.use_graphs = bool(use_graphs) and rt.device.type == "cuda" and self.pad_decode
        self.max_graph_batch = int(max_graph_batch)
        self.max_graphs = int(max_graphs)
        self._static: "OrderedDict[Tuple[int, int], _StaticBatch]" = OrderedDict()
        self._graph_pool = None
        self._decode_logits: Optional[torch.Tensor] = None     # [rows, V]: every captured step writes here
        # the model's kernel calls recorded once and run from C++, a step a call; None where the model's parts
        # do more with their activations than hand them to the kernels (then the parts run one by one)
        self.program = None
        self.use_program = bool(use_program) and rt.device.type == "cuda"
        self.max_step_tokens = int(max_step_tokens) if max_step_tokens else None
        self.max_step_seqs = int(max_step_seqs) if max_step_seqs else None
        self.program_steps = 0          # steps that the program ran
        self.python_parts = None        # (part, method name) -> True: that call runs in Python inside the program (tests, debugging)
        self.program_workspace_bytes = 32 << 20    # the workspace's size; it doubles if a step finds no room all the same
        if self.use_program:
            self._record_program()

    def _record_program(self) -> None:
        """Records the model's kernel calls and gives the program its workspace: once, at the size that the largest
        step the engine will build needs (found by walking such steps without launching), so that no step in
        the middle of serving has to allocate."""
        from ..ops.program import record_program
        self.program = record_program(self.model, self.rt.ops, self.python_parts)
        self._static.clear()            # captured steps belong to the program that launched them
        if self.program is None:
            return
        if self.max_step_tokens:
            self.program_workspace_bytes = max(self.program_workspace_bytes, self.workspace_for(
                self.max_step_tokens, self.max_step_seqs or self.max_graph_batch))
        self.program.ensure_workspace(self.program_workspace_bytes)

    def workspace_for(self, max_tokens: int, max_seqs: int) -> int:
        """Bytes of program workspace that steps of up to ``max_tokens`` tokens of up to ``max_seqs`` requests need:
        the most over a ladder of step sizes, each as one portion of a prompt, as a portion beside single tokens
        and (where it fits) as single tokens only, plus a tenth."""
        prog = self.program
        G = len(self.manager.groups)
        sizes = sorted({n for n in (1, 2, 8, 16, 17, 64, 65, 128, 129, 256, 257, 512, 1024, 2048, 4096, max_tokens // 2,
                                    max_tokens) if 1 <= n <= max_tokens})
        need = 0
        for n in sizes:
            shapes = {(1, 1), (min(max_seqs, max(1, n // 2)), min(max_seqs, max(1, n // 2)))}
            if n <= max_seqs:
                shapes.add((n, n))
            for segs, rows in shapes:
                if segs <= n:
                    need = max(need, prog.workspace_need(n, segs, rows, self.max_model_len, G))
        return int(need * 1.1) + (1 << 20)

    # ------------------------------------------------------------------ the step

    def step(self, entries: Sequence[StepEntry], prev_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Run one batch. Returns float32 logits [R, V] on the device, rows in the order of the entries
        and of each entry's ``want``. Raises OutOfPages (and takes nothing) if the cache cannot hold
        the new tokens. ``prev_tokens`` (int32, on the device): the tokens that the step before sampled, for
        entries that name one of them (``StepEntry.prev_row``) instead of a token the host knows."""
        entries = [e for e in entries if len(e.tokens) > 0]
        self._validate(entries)
        if self.program is not None and self.program.stale():
            # somebody moved the kernels' switch points (tests, tuning): record again before anything of this step
            # is built for the old program, and forget what was captured
            self._record_program()
        from_prev = any(e.prev_row >= 0 for e in entries)
        if from_prev and prev_tokens is None:
            raise StepError("an entry names a token of the step before, which was not given")
        self._prev_tokens = prev_tokens if from_prev else None
        if not entries:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.rt.device)
        mgr = self.manager
        rids = [e.request_id for e in entries]
        lens = [len(e.tokens) for e in entries]
        handles, starts, added = mgr.begin_step(rids, lens)      # OutOfPages: nothing was taken
        try:
            if self.storage.has_state and added.any():
                # a request that has just taken a state slot finds it cleared
                self.storage.clear_state_slots([mgr.state_slot(rids[i]) for i in np.nonzero(added)[0]])
            if self.pad_decode and all(n == 1 for n in lens) and len(entries) <= self.max_graph_batch:
                logits = self._decode_step(entries, handles, starts)
            else:
                logits = self._forward(self._build_context(entries, handles, starts))
        except Exception:
            mgr.abort_step(rids, handles, added)
            raise
        mgr.commit_step(handles)
        return logits

    def _forward(self, ctx: StepContext, logits_out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The model over the step: through the recorded program where there is one, else part by part."""
        prog = self.program
        plan = ctx.aux.get("program_plan")
        if prog is not None and (ctx.all_single or plan is not None):
            from ..ops.hip_ops import _current_device, _raw_stream
            R = ctx.n_logit_rows
            out = logits_out
            if out is None and R:
                out = torch.empty((R, self.vocab_size), dtype=torch.float32, device=self.rt.device)
            stream = _raw_stream(_current_device())
            capturing = torch.cuda.is_current_stream_capturing()
            while True:
                if prog.run(ctx, out, plan, stream):
                    self.program_steps += 1
                    if out is None:
                        return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.rt.device)
                    return out
                # a step larger than the workspace was sized for: a larger one (never while a step is captured, and
                # what has been captured points into the one that goes)
                if capturing or self.program_workspace_bytes >= (64 << 30):
                    break
                self.program_workspace_bytes *= 2
                kept = [k for k, sb in self._static.items() if sb.graph is None]
                for k in [k for k in self._static if k not in kept]:
                    del self._static[k]
                prog.ensure_workspace(self.program_workspace_bytes)
        if logits_out is not None:
            return self.model.forward(ctx, logits_out=logits_out)
        return self.model.forward(ctx)

    def tune_products(self, rows: Sequence[int], candidates: int = 16, reps: int = 5) -> dict:
        """For steps of these numbers of tokens, lets the BLAS library's candidates race for every shape of matrix
        product the model has and keeps the winners (``HipOps.tune_products``; tops/src/cublas.rs:121-223 profiles
        cuBLASLt's tactics per weight shape and bucket of rows likewise). Only products that go to the library at
        that many rows are looked at. Returns {(rows, N, K): (first choice's us, fastest's us)}."""
        from ..ops import dispatch as D
        from ..parts.linear import FusedLinear
        import ctypes
        ops = self.rt.ops
        shapes = {}
        for p in self.model.parts():
            w = getattr(p, "weight", None)
            if isinstance(p, FusedLinear) and w is not None and w.dtype == torch.bfloat16 and w.is_cuda:
                shapes.setdefault((w.shape[0], w.shape[1], w.stride(0), p.bias is not None), []).append(p)
        found = {}
        for M in sorted(set(int(m) for m in rows)):
            for (N, K, ld, has_bias), parts in shapes.items():
                x = torch.randn((M, K), device=self.rt.device, dtype=torch.float32).to(torch.bfloat16)
                rt = D.Route()
                ops.lib.lmsf_route_linear(ctypes.byref(ops._tun), ctypes.byref(ops._shape(x, parts[0].weight, x.dtype)),
                                          0, ctypes.byref(rt))
                if rt.route == D.BLAS:
                    found[(M, N, K)] = ops.tune_products(x, [p.weight for p in parts], parts[0].bias, candidates, reps)
        return found

    def release(self, request_id: Hashable) -> None:
        """The request is finished: its pages and state slot go back."""
        if self.manager.has_request(request_id):
            self.manager.free_request(request_id)

    # ------------------------------------------------------------------ helpers

    def _validate(self, entries: Sequence[StepEntry]) -> None:
        seen = set()
        V = self.vocab_size
        for e in entries:
            if e.request_id in seen:
                raise StepError("request %r appears twice in one step" % (e.request_id,))
            seen.add(e.request_id)
            n = len(e.tokens)
            if e.prev_row >= 0 and n != 1:
                raise StepError("request %r: a token of the step before stands for exactly one token" % (e.request_id,))
            if n == 1:
                bad = not (0 <= int(e.tokens[0]) < V)
            else:
                ids = np.asarray(e.tokens, dtype=np.int64)
                bad = bool(((ids < 0) | (ids >= V)).any())
            if bad:
                t = next(t for t in e.tokens if not (0 <= int(t) < V))
                raise StepError("request %r: token id %r outside the vocabulary of %d" % (e.request_id, t, V))
            for w in e.want:
                if not (0 <= int(w) < n):
                    raise StepError("request %r: wanted place %r outside its %d tokens" % (e.request_id, w, n))
        held = self.manager.tokens_held([e.request_id for e in entries])
        for e, h in zip(entries, held.tolist()):
            if h + len(e.tokens) > self.max_model_len:
                raise StepError("request %r would hold %d tokens, more than max_model_len %d"
                                % (e.request_id, h + len(e.tokens), self.max_model_len))

    def _build_context(self, entries: Sequence[StepEntry], handles: np.ndarray, starts_a: np.ndarray,
                       static: Optional["_StaticBatch"] = None) -> StepContext:
        """Flatten the entries into the step's device tensors. Everything goes through one pinned staging
        buffer, which the host library fills, and one copy. With ``static`` (a step of single tokens) the
        batch is padded to that kind's size with tokens that store nothing (slot -1, position 0, a segment of
        their own whose block table is all zeros, the spare state slot), the copy goes into its fixed device
        buffer, block tables padded to their full width, and every token's logits are asked for."""
        mgr = self.manager
        S = len(entries)
        lens = [len(e.tokens) for e in entries]
        N = sum(lens)
        starts = starts_a.tolist()
        Np = Sp = None
        if static is not None:
            Np = Sp = static.batch                      # N == S: single tokens
            logit_rows = np.arange(Np, dtype=np.int32)
        else:
            seg_start, rows = 0, []
            for e, n in zip(entries, lens):
                rows.extend(seg_start + int(w) for w in e.want)
                seg_start += n
            logit_rows = np.asarray(rows, dtype=np.int32)
        R = int(logit_rows.shape[0])
        G = len(mgr.groups)
        widths = static.widths if static is not None else mgr.step_widths(handles)
        if static is not None:
            if static.layout is None:
                static.layout = mgr.step_layout(Np, Sp, R, widths)
            offsets, raw_offsets, total = static.layout
        else:
            offsets, raw_offsets, total = mgr.step_layout(N, S, R, widths)
        # a step of single tokens also carries its tokens ordered by context, the longest first, behind the
        # sections the host library lays out
        single = N == S
        n_all = Np if static is not None else N
        order_at, total = total, total + (_pad4(n_all) if single else 0)
        # where tokens come from the step before: per token the row of that step's sampled tokens, or -1
        src_at = 0
        if self._prev_tokens is not None or static is not None:
            src_at, total = total, total + _pad4(n_all)
        # a step that the recorded program may run carries its attention plan behind that
        plan_at = plan_cap = 0
        if self.program is not None and static is None and N != S:
            plan_at, plan_cap = total, self.program.plan_capacity(N)
            total += plan_cap
        if self._pinned is None or self._pinned.numel() < total:
            self._pinned = torch.empty(max(total, 4096), dtype=torch.int32,
                                       pin_memory=self.rt.device.type == "cuda")
            self._pinned_np = self._pinned.numpy()
        host = self._pinned[:total]
        host_np = self._pinned_np
        if single:
            host_np[order_at:order_at + N] = np.argsort(-starts_a, kind="stable")
            if n_all > N:
                host_np[order_at + N:order_at + n_all] = np.arange(N, n_all, dtype=np.int32)

        def section(name: str) -> np.ndarray:
            o, n = offsets[name]
            return host_np[o:o + n]

        if N == S:
            section("token_ids")[:N] = [e.tokens[0] for e in entries]
        else:
            section("token_ids")[:] = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries])
        if R:
            section("logit_rows")[:] = logit_rows
        if src_at:
            src = host_np[src_at:src_at + n_all]
            src[:] = -1
            if self._prev_tokens is not None:
                at = 0
                for e, n in zip(entries, lens):
                    if e.prev_row >= 0:
                        src[at] = e.prev_row
                    at += n
        try:
            mgr.fill_step(handles, starts_a, lens, widths, raw_offsets, host_np)
        except CacheError as e:
            raise CacheError("%s (requests %s)" % (e, ", ".join(repr(x.request_id) for x in entries)))
        if static is not None and Np > N:
            pad = np.arange(N, Np, dtype=np.int32)
            section("token_ids")[N:] = 0
            section("positions")[N:] = 0
            section("seg_of")[N:] = pad
            section("seg_starts")[N:Np + 1] = np.arange(N, Np + 1, dtype=np.int32)
            section("seg_first")[N:] = 0
            section("state_slots")[N:] = self.storage.spare_state_slot
            for gi in range(G):
                section("slots%d" % gi)[N:] = -1
                section("tables%d" % gi)[N * widths[gi]:] = 0
        plan_info = None
        if plan_cap:
            used, plan_info = self.program.write_plan(lens, starts, host_np[plan_at:plan_at + plan_cap], plan_cap)
            total = plan_at + _pad4(max(used, 1))
            host = self._pinned[:total]
        # the copy is synchronous: the staging buffer is free again when the next step fills it
        if static is not None:
            static.device_buffer.copy_(host, non_blocking=False)
            if self._prev_tokens is not None:
                self.rt.ops.patch_tokens(static.device_buffer[offsets["token_ids"][0]:offsets["token_ids"][0] + n_all],
                                         static.device_buffer[src_at:src_at + n_all], self._prev_tokens)
            if static.context is not None:
                return static.context
            dev = static.device_buffer
        elif self.rt.device.type == "cuda":
            dev = torch.empty(total, dtype=torch.int32, device=self.rt.device)
            dev.copy_(host, non_blocking=False)
        else:
            dev = host.clone()

        def view(name: str) -> torch.Tensor:
            o, n = offsets[name]
            return dev[o:o + n]

        if static is None and self._prev_tokens is not None:
            self.rt.ops.patch_tokens(view("token_ids"), dev[src_at:src_at + n_all], self._prev_tokens)
        S_all = Sp if static is not None else S
        if static is None:
            seg_starts = section("seg_starts").tolist()
            state_slots = section("state_slots").tolist()
        else:
            # a captured step is told nothing that changes from step to step
            seg_starts, state_slots, lens, starts = list(range(S_all + 1)), [], [1] * S_all, []
        groups = [GroupView(slots=view("slots%d" % gi),
                            block_tables=view("tables%d" % gi).view(S_all, widths[gi]),
                            page_size=mgr.groups[gi].page_size) for gi in range(G)]
        # (where the plan lies on the device and how it is laid out travel with the step, not with the program)
        aux = {"program_plan": (dev.data_ptr() + 4 * plan_at, plan_info)} if plan_cap else {}
        return StepContext(
            aux=aux, n_tokens=n_all, n_segments=S_all, token_ids=view("token_ids"), positions=view("positions"),
            seg_of_token=view("seg_of"), seg_starts=view("seg_starts"), seg_first_pos=view("seg_first"),
            state_slots=view("state_slots"), logit_rows=view("logit_rows"), n_logit_rows=R, groups=groups,
            longest_first=dev[order_at:order_at + n_all] if single else None,
            host_seg_starts=seg_starts, host_seg_lens=lens, host_seg_first_pos=list(starts),
            host_state_slots=list(state_slots),
            request_ids=[e.request_id for e in entries] if static is None else [],
            max_seg_len=max(lens),
            max_context=(static.max_context if static is not None else
                         max(st + n for st, n in zip(starts, lens))),
            all_single=all(n == 1 for n in lens), replayed=static is not None)

    def _context_bucket(self, longest: int) -> int:
        """The longest context of a step of single tokens, rounded up to a power of two (at least 256, at
        most the model's limit). The parts are told this number instead of the true one, so that every step
        of a kind splits the work alike, captured or not."""
        bucket = 256
        while bucket < longest:
            bucket *= 2
        return min(bucket, self.max_model_len)

    # ------------------------------------------------------------------ steps of single tokens

    def _decode_step(self, entries: Sequence[StepEntry], handles: np.ndarray, starts: np.ndarray) -> torch.Tensor:
        """A step of single tokens. Its batch is padded to one of a few sizes (``padded_batch``) and its
        longest context rounded up to a power of two; what is left is a *kind* of step, whose metadata has a
        fixed layout in a fixed device buffer. The first step of a kind runs kernel by kernel and is then
        captured as a HIP graph; later steps of that kind copy their metadata into the buffer and replay the
        graph: one launch instead of hundreds. Inside a graph nothing may depend on the step's actual
        context lengths but through the device tensors, so the parts are told the bucket as the longest
        context. Every kind writes the logits of all its tokens into one buffer shared by all kinds; the wanted
        rows are picked from it afterwards. At most ``max_graphs`` kinds are kept, the least recently used is
        dropped. Without graphs the same padded steps run kernel by kernel, to the same bits."""
        B = len(entries)
        Bp = padded_batch(B, self.max_graph_batch)
        bucket = self._context_bucket(int(starts.max()) + 1)
        sb = self._static.get((Bp, bucket))
        if sb is None:
            widths = [-(-bucket // g.page_size) for g in self.manager.groups]
            _, _, total = self.manager.step_layout(Bp, Bp, Bp, widths)
            sb = _StaticBatch(Bp, widths, torch.zeros(total + 2 * _pad4(Bp), dtype=torch.int32, device=self.rt.device),
                              bucket)
            self._static[(Bp, bucket)] = sb
            while len(self._static) > self.max_graphs:
                self._static.popitem(last=False)
        else:
            self._static.move_to_end((Bp, bucket))
        if self._decode_logits is None:
            rows = padded_batch(min(self.max_graph_batch, max(1, self.storage.num_state_slots)), self.max_graph_batch)
            self._decode_logits = torch.empty((max(rows, Bp), self.vocab_size), dtype=torch.float32,
                                              device=self.rt.device)
        elif self._decode_logits.shape[0] < Bp:
            # more live requests than state slots cannot be; a caller that builds such a step all the same gets
            # a larger buffer, and the kinds captured so far, which write into the old one, are dropped
            self._static = OrderedDict({(Bp, bucket): sb})
            self._decode_logits = torch.empty((Bp, self.vocab_size), dtype=torch.float32, device=self.rt.device)
        out = self._decode_logits[:Bp]
        ctx = self._build_context(entries, handles, starts, static=sb)
        if sb.graph is None:
            sb.context = ctx
            self._forward(ctx, logits_out=out)               # launched one by one: this step's result, and the warm-up
            if self.use_graphs:
                torch.cuda.current_stream().synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, pool=self._graph_pool):   # records, runs nothing: ``out`` stays
                    self._forward(ctx, logits_out=out)
                sb.graph = graph
                if self._graph_pool is None:
                    self._graph_pool = graph.pool()
        else:
            sb.graph.replay()
        # the rows go to the caller as a copy: the buffer is written again by the next step of single tokens
        wanted = [i for i, e in enumerate(entries) if len(e.want)]
        if len(wanted) == B:
            return out[:B].clone()
        if not wanted:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.rt.device)
        return out[torch.tensor(wanted, device=self.rt.device)]

    def graph_memory_bytes(self) -> int:
        """Device memory the captured steps hold beside the weights and the cache: the shared logits buffer and
        the metadata buffers (the kernels' temporaries live in one pool that the graphs share)."""
        total = 0 if self._decode_logits is None else self._decode_logits.numel() * 4
        return total + sum(sb.device_buffer.numel() * 4 for sb in self._static.values())


def padded_batch(batch: int, limit: int = 256) -> int:
    """The size at which a step of ``batch`` single tokens runs: 1, 2, 4, 8, then multiples of 8."""
    if batch <= 8:
        size = 1
        while size < batch:
            size *= 2
    else:
        size = (batch + 7) // 8 * 8
    return max(batch, min(size, limit))


def _pad4(n: int) -> int:
    return (n + 3) // 4 * 4


class _StaticBatch:
    """What a kind of decode step (padded batch size, context bucket) keeps: the fixed metadata buffer, the
    context whose tensors are views into it, and the graph."""

    def __init__(self, batch: int, widths: Sequence[int], device_buffer: torch.Tensor, max_context: int):
        self.batch = int(batch)
        self.widths = list(widths)
        self.max_context = int(max_context)
        self.device_buffer = device_buffer
        self.context: Optional[StepContext] = None
        self.layout = None                 # the metadata buffer's sections: the same at every step of this kind
        self.graph = None
