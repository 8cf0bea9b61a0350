"""Records a model's kernel calls once and runs them from C++ for every step.

The parts of a model call the kernels through ``rt.ops`` (ops.HipOps), one Python call per kernel.
``record_program`` runs the model's forward once over a ``Recorder`` that stands in for ``rt.ops``: the
activations it hands out are placeholders (``Sym``), the weights it is given are the real tensors. What
comes out is a list of operations over value registers, which ``csrc/program.hip`` keeps and runs: it
asks the same functions as ``HipOps`` which kernel an operation runs in (csrc/dispatch.h), takes
temporaries from one workspace, and launches; a step of any number of tokens is then one call from Python
instead of hundreds (the BLAS library's products included, through csrc/blas.hip).

A part that does nothing to activations but pass them to ``rt.ops`` is recorded kernel by kernel. A part that
computes on a tensor itself (a toy mixer written with torch, a position encoding that acts in place, a kernel
the program has no operation for) meets a placeholder and fails; the recorder then takes back what that part
had recorded and notes one *callback* operation instead: at run time the program stops there, calls back into
Python with the places of the part's operands in the workspace, the part runs as it is on real tensors, and the
program goes on. So one foreign part costs one trip to Python, not the whole model's. If even that cannot be
done (a part with more than two activations among its arguments, say), ``record_program`` returns None with the
reason in ``last_failure`` and the engine runs the model part by part. No part knows of any of this.

The reference's step is native from the worker down (core/src/worker/model_worker.rs:213-264,
core/src/model_executor/models/llama/llama.rs:397-476).
"""
import ctypes
from ctypes import CFUNCTYPE, POINTER, Structure, c_float, c_int, c_long, c_void_p
from typing import Any, Callable, List, Optional

import numpy as np
import torch

from . import library
from .dispatch import Tunables

MAX_GROUPS = 8
MAX_PLANS = 4
NO_ROOM = 4

(OP_EMBEDDING, OP_ADD_RMS_NORM, OP_QKV_ROPE_CACHE, OP_ATTENTION, OP_LINEAR, OP_LINEAR_GATED, OP_MATERIALIZE,
 OP_ROPE_CACHE_WRITE, OP_GATED_ACT, OP_CALLBACK) = range(1, 11)
CTX_NONE, CTX_TOKEN_IDS, CTX_POSITIONS, CTX_SEG_OF, CTX_LOGIT_ROWS, CTX_SLOTS, CTX_TABLES = 0, 1, 2, 3, 4, 16, 32


class OpDesc(Structure):
    _fields_ = ([(n, c_int) for n in ("kind", "in0", "in1", "out", "ctx0", "ctx1", "rows_ctx")]
                + [(n, c_void_p) for n in ("w", "bias", "table", "k_pages", "v_pages")]
                + [(n, c_int) for n in ("wdtype", "out_dtype", "cache_dtype", "N", "K")]
                + [("ldw", c_long)]
                + [(n, c_int) for n in ("nh", "nkv", "d", "rot", "neox", "ps", "window", "max_pos", "act", "defer_ok",
                                        "pending_ok", "is_head", "vocab")]
                + [("num_pages", c_long)]
                + [(n, c_float) for n in ("eps", "weight_offset", "scale")]
                + [("callback_id", c_int)])


class PlanInfo(Structure):
    _fields_ = ([("n_plans", c_int)]
                + [(n, c_int * MAX_PLANS) for n in ("tq", "n_tiles", "n_single")]
                + [(n, c_long * MAX_PLANS) for n in ("tiles_at", "single_at")])


class StepDesc(Structure):
    _fields_ = ([(n, c_int) for n in ("n_tokens", "n_segments", "n_logit_rows", "max_context", "all_single", "n_groups")]
                + [(n, c_void_p) for n in ("token_ids", "positions", "seg_of", "logit_rows", "longest_first")]
                + [("slots", c_void_p * MAX_GROUPS), ("tables", c_void_p * MAX_GROUPS), ("widths", c_int * MAX_GROUPS)]
                + [("plan", c_void_p), ("plan_info", PlanInfo), ("workspace", c_void_p), ("workspace_bytes", c_long),
                   ("logits", c_void_p), ("bad_flag", c_void_p)])


class TensorRef(Structure):
    _fields_ = [("offset", c_long), ("rows", c_int), ("cols", c_int), ("dtype", c_int)]


class CallbackArgs(Structure):
    _fields_ = [("callback_id", c_int), ("in0", TensorRef), ("in1", TensorRef), ("out", TensorRef)]


CallbackFn = CFUNCTYPE(c_int, POINTER(CallbackArgs))

_SIGNATURES = {
    "lmsf_program_create": (c_void_p, [POINTER(Tunables)]),
    "lmsf_program_destroy": (None, [c_void_p]),
    "lmsf_program_add": (c_int, [c_void_p, POINTER(OpDesc)]),
    "lmsf_program_seal": (c_int, [c_void_p]),
    "lmsf_program_set_callback": (None, [c_void_p, CallbackFn]),
    "lmsf_program_plan": (c_long, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_long, POINTER(PlanInfo)]),
    "lmsf_program_plan_capacity": (c_long, [c_void_p, c_int]),
    "lmsf_program_run": (c_int, [c_void_p, POINTER(StepDesc), c_int, c_void_p]),
    "lmsf_program_stats": (c_int, [c_void_p, POINTER(c_long), c_int]),
}


def _declare(lib) -> None:
    if getattr(lib, "_lmsf_program_declared", False):
        return
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    lib._lmsf_program_declared = True


_TORCH_OF_CODE = {0: torch.float32, 1: torch.bfloat16}


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return 0
    if dtype == torch.bfloat16:
        return 1
    raise NotRecordable("a tensor of %s" % dtype)


class NotRecordable(Exception):
    """The model does something that the step program has no operation for."""


class Sym:
    """An activation that does not exist yet: the value of a register. ``cols`` and ``dtype`` are what the
    recorder knows of it (None where it does not)."""

    __slots__ = ("reg", "cols", "dtype")

    def __init__(self, reg: int, cols: Optional[int] = None, dtype: Optional[torch.dtype] = None):
        self.reg = reg
        self.cols = cols
        self.dtype = dtype

    def __getattr__(self, name):
        raise NotRecordable("a part reads .%s of an activation itself" % name)


class CtxRef:
    """One of the step's device arrays, by its code."""

    __slots__ = ("code",)

    def __init__(self, code: int):
        self.code = code

    def __getattr__(self, name):
        raise NotRecordable("a part reads .%s of one of the step's arrays itself" % name)


def _w(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


class _Callback:
    """A part's method that runs in Python in the middle of a program, and how to build its arguments."""

    __slots__ = ("fn", "args", "kwargs", "in_place", "what")

    def __init__(self, fn, args, kwargs, in_place: bool, what: str):
        self.fn, self.args, self.kwargs, self.in_place, self.what = fn, args, kwargs, in_place, what


class Recorder:
    """Stands in for ``HipOps`` while the model's forward is recorded: the same methods, which note what they
    were asked instead of launching it."""

    name = "recorder"

    def __init__(self, run_dtype: torch.dtype, hidden_size: int = 0, vocab_size: int = 0):
        self.ops: List[OpDesc] = []
        self.keep: List[torch.Tensor] = []      # every tensor an operation points to stays alive with the program
        self.n_regs = 0
        self.run_dtype = run_dtype
        self.hidden_size, self.vocab_size = int(hidden_size), int(vocab_size)
        self.callbacks: List[_Callback] = []
        self.step_ctx = None                    # the placeholder StepContext of the recording
        self.roles = {}                         # id(part) -> "embedding" / "head"
        self.in_python = None                   # (part, method name) -> True: record this call as a callback anyway

    # -- helpers
    def _new(self, cols: Optional[int] = None, dtype: Optional[torch.dtype] = None) -> Sym:
        self.n_regs += 1
        return Sym(self.n_regs - 1, cols, dtype)

    @staticmethod
    def _reg(v: Any, what: str, optional: bool = False) -> int:
        if v is None and optional:
            return -1
        if not isinstance(v, Sym):
            raise NotRecordable("%s is not an activation made by a kernel" % what)
        return v.reg

    @staticmethod
    def _ctx(v: Any, what: str, optional: bool = False) -> int:
        if v is None and optional:
            return CTX_NONE
        if not isinstance(v, CtxRef):
            raise NotRecordable("%s is not one of the step's arrays" % what)
        return v.code

    def _weight(self, t: Optional[torch.Tensor], what: str, dims: int) -> Optional[torch.Tensor]:
        if t is None:
            return None
        if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dim() != dims or t.stride(-1) != 1:
            raise NotRecordable("%s is not a device tensor of %d dimensions with unit stride" % (what, dims))
        self.keep.append(t)
        return t

    def _add(self, **fields) -> None:
        op = OpDesc()
        for k in ("in0", "in1", "out"):
            setattr(op, k, -1)
        for k, v in fields.items():
            setattr(op, k, v)
        self.ops.append(op)

    def check_head_dim(self, d: int) -> None:      # parts are already built; nothing to ask
        pass

    # -- the kernels' methods
    def embedding(self, ids, table, scale: float = 1.0):
        table = self._weight(table, "the embedding table", 2)
        if not table.is_contiguous():
            raise NotRecordable("the embedding table is not contiguous")
        out = self._new(table.shape[1], torch.float32)
        self._add(kind=OP_EMBEDDING, out=out.reg, ctx0=self._ctx(ids, "the embedding's ids"), w=_w(table),
                  wdtype=_code(table.dtype), N=table.shape[1], vocab=table.shape[0], scale=float(scale))
        return out

    def add_rms_norm(self, branch, residual, weight, eps, out_dtype, rows=None, weight_offset: float = 0.0,
                     defer_ok: bool = False):
        weight = self._weight(weight, "a norm's weight", 1)
        out = self._new(weight.shape[0], out_dtype)
        self._add(kind=OP_ADD_RMS_NORM, in0=self._reg(branch, "a norm's branch", optional=True),
                  in1=self._reg(residual, "a norm's residual", optional=True), out=out.reg,
                  rows_ctx=self._ctx(rows, "a norm's rows", optional=True), w=_w(weight), wdtype=_code(weight.dtype),
                  N=weight.shape[0], eps=float(eps), weight_offset=float(weight_offset), out_dtype=_code(out_dtype),
                  defer_ok=1 if defer_ok else 0)
        return out

    def _rotary_fields(self, table, rot_dim, neox) -> dict:
        if table is not None:
            table = self._weight(table, "the rotary table", 2)
            if table.dtype != torch.float32 or table.shape[1] != rot_dim or not table.is_contiguous():
                raise NotRecordable("the rotary table is not contiguous float32 [max_pos, %d]" % rot_dim)
        return dict(table=_w(table), rot=int(rot_dim) if table is not None else 0, neox=1 if neox else 0,
                    max_pos=table.shape[0] if table is not None else 0)

    def qkv_rope_cache(self, x, weight, bias, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages, v_pages):
        weight = self._weight(weight, "the QKV weight", 2)
        bias = self._weight(bias, "the QKV bias", 1)
        if bias is not None and (bias.dtype != weight.dtype or bias.shape[0] != weight.shape[0] or not bias.is_contiguous()):
            raise NotRecordable("the QKV bias does not fit its weight")
        fields = self._rotary_fields(table, rot_dim, neox)
        if slots is not None:
            fields.update(self._pages(k_pages, v_pages, nkv, d))
        out = self._new(weight.shape[0], getattr(x, "dtype", None) if isinstance(x, Sym) else None)
        self._add(kind=OP_QKV_ROPE_CACHE, in0=self._reg(x, "the QKV projection's input"), out=out.reg,
                  ctx0=self._ctx(positions, "positions"), ctx1=self._ctx(slots, "slots", optional=True), w=_w(weight),
                  bias=_w(bias), wdtype=_code(weight.dtype), N=weight.shape[0], K=weight.shape[1],
                  ldw=weight.stride(0), nh=int(nh), nkv=int(nkv), d=int(d), **fields)
        return out

    def rope_cache_write(self, qkv, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages, v_pages) -> None:
        fields = self._rotary_fields(table, rot_dim, neox)
        if slots is not None:
            fields.update(self._pages(k_pages, v_pages, nkv, d))
        self._add(kind=OP_ROPE_CACHE_WRITE, in0=self._reg(qkv, "the projections to rotate and store"),
                  ctx0=self._ctx(positions, "positions", optional=table is None),
                  ctx1=self._ctx(slots, "slots", optional=True), nh=int(nh), nkv=int(nkv), d=int(d), **fields)

    def _pages(self, k_pages, v_pages, nkv, d) -> dict:
        k_pages = self._weight(k_pages, "the key pages", 4)
        v_pages = self._weight(v_pages, "the value pages", 4)
        pages, ps = k_pages.shape[0], k_pages.shape[2]
        if tuple(k_pages.shape) != (pages, nkv, ps, d) or tuple(v_pages.shape) != (pages, nkv, d, ps) \
                or not k_pages.is_contiguous() or not v_pages.is_contiguous() or k_pages.dtype != v_pages.dtype:
            raise NotRecordable("the cache pages do not have the layout the kernels read")
        return dict(k_pages=_w(k_pages), v_pages=_w(v_pages), num_pages=pages, ps=ps, cache_dtype=_code(k_pages.dtype))

    def paged_attention(self, q, k_pages, v_pages, block_tables, seg, pos, nh, nkv, d, scale, window=0, batch=None,
                        kernel=None):
        if kernel is not None:
            raise NotRecordable("a part forces an attention kernel")
        if self._ctx(seg, "seg") != CTX_SEG_OF or self._ctx(pos, "pos") != CTX_POSITIONS:
            raise NotRecordable("attention over other segments or positions than the step's")
        out = self._new(int(nh) * int(d), getattr(q, "dtype", None) if isinstance(q, Sym) else None)
        self._add(kind=OP_ATTENTION, in0=self._reg(q, "the queries"), out=out.reg,
                  ctx0=self._ctx(block_tables, "block tables"), nh=int(nh), nkv=int(nkv), d=int(d), scale=float(scale),
                  window=int(window or 0), **self._pages(k_pages, v_pages, nkv, d))
        return out

    def _linear_fields(self, weight, bias, what: str) -> dict:
        weight = self._weight(weight, what + " weight", 2)
        bias = self._weight(bias, what + " bias", 1)
        if bias is not None and (bias.dtype != weight.dtype or bias.shape[0] != weight.shape[0] or not bias.is_contiguous()):
            raise NotRecordable("%s bias does not fit its weight" % what)
        return dict(w=_w(weight), bias=_w(bias), wdtype=_code(weight.dtype), N=weight.shape[0], K=weight.shape[1],
                    ldw=weight.stride(0))

    def linear(self, x, weight, bias=None, out_dtype=None, pending_ok: bool = False, out=None):
        is_head = out is not None
        if is_head and not isinstance(out, LogitsOut):
            raise NotRecordable("a product writes into a tensor of the part's own")
        dtype = out_dtype or (x.dtype if isinstance(x, Sym) and x.dtype is not None else self.run_dtype)
        res = self._new(weight.shape[0], dtype)
        self._add(kind=OP_LINEAR, in0=self._reg(x, "a product's input"), out=res.reg, out_dtype=_code(dtype),
                  pending_ok=1 if pending_ok else 0, is_head=1 if is_head else 0,
                  **self._linear_fields(weight, bias, "a product's"))
        return res

    def linear_gated(self, x, weight, bias=None, kind: str = "silu"):
        kinds = {"silu": 1, "gelu": 2}
        if kind not in kinds or weight.shape[0] % 2 != 0:
            raise NotRecordable("a gated product of kind %r" % (kind,))
        res = self._new(weight.shape[0] // 2, getattr(x, "dtype", None) if isinstance(x, Sym) else None)
        self._add(kind=OP_LINEAR_GATED, in0=self._reg(x, "a gated product's input"), out=res.reg, act=kinds[kind],
                  **self._linear_fields(weight, bias, "a gated product's"))
        return res

    def gated_act(self, gu, kind: str = "silu"):
        kinds = {"silu": 1, "gelu": 2}
        if kind not in kinds or not isinstance(gu, Sym) or gu.cols is None or gu.cols % 2 != 0:
            raise NotRecordable("a gated activation of kind %r over an activation of unknown width" % (kind,))
        res = self._new(gu.cols // 2, gu.dtype)
        self._add(kind=OP_GATED_ACT, in0=gu.reg, out=res.reg, act=kinds[kind], N=gu.cols)
        return res

    def materialize(self, y):
        if not isinstance(y, Sym):
            return y
        res = self._new(y.cols, y.dtype)
        self._add(kind=OP_MATERIALIZE, in0=y.reg, out=res.reg)
        return res

    def __getattr__(self, name):
        raise NotRecordable("a part calls the kernel %r, which the step program does not have" % name)

    # -- parts that cannot be followed: one callback each
    def mark(self):
        return len(self.ops), self.n_regs, len(self.keep), len(self.callbacks)

    def rollback(self, mark) -> None:
        n_ops, self.n_regs, n_keep, n_cb = mark
        del self.ops[n_ops:], self.keep[n_keep:], self.callbacks[n_cb:]

    def guarded(self, part, name: str, fn: Callable) -> Callable:
        """``fn`` (the bound method ``part.name``) for the time of the recording: it runs as it is; if it fails on a
        placeholder, what it recorded is taken back and the whole call becomes one callback operation."""

        def call(*args, **kwargs):
            if self.in_python is not None and self.in_python(part, name):
                return self._callback(part, name, fn, args, kwargs, "asked for")
            mark = self.mark()
            try:
                return fn(*args, **kwargs)
            except Exception as e:  # noqa: BLE001 - a part that computes on a placeholder fails in its own way
                self.rollback(mark)
                return self._callback(part, name, fn, args, kwargs, "%s: %s" % (type(e).__name__, e))

        return call

    def _callback(self, part, name: str, fn: Callable, args, kwargs, why: str):
        from ..parts.base import Block, FeedForward, Mixer, Norm, PositionEncoding
        what = "%s.%s of %s at %r (%s)" % (type(part).__name__, name, type(part).__mro__[1].__name__, part.prefix, why)
        syms = [a for a in list(args) + list(kwargs.values()) if isinstance(a, Sym)]
        if len(syms) > 2:
            raise NotRecordable("%s takes more than two activations" % what)
        role = self.roles.get(id(part))
        in_place = isinstance(part, PositionEncoding) and name == "apply"
        # what comes out: the part's interface says (parts/base.py), the recorder cannot look
        rows_ctx, is_head = CTX_NONE, False
        if in_place:
            out_cols = out_dtype = None
        elif role == "embedding":
            out_cols, out_dtype = self.hidden_size, torch.float32
        elif role == "head":
            out_cols, out_dtype = self.vocab_size, torch.float32
            is_head = any(isinstance(a, LogitsOut) for a in list(args) + list(kwargs.values()))
        elif isinstance(part, (Norm, Mixer, FeedForward, Block)) and syms:
            out_cols, out_dtype = syms[-1].cols, self.run_dtype
            rows = kwargs.get("rows", args[2] if isinstance(part, Norm) and name == "forward_add" and len(args) > 2 else None)
            if isinstance(rows, CtxRef):
                rows_ctx = rows.code
        else:
            raise NotRecordable("%s: what it returns is not known" % what)
        if not in_place and not out_cols:
            raise NotRecordable("%s: the width of what it returns is not known" % what)
        # its activations become finished tensors (the one it works on in place must be one already)
        regs = {}
        for s in syms:
            regs[id(s)] = s.reg if in_place else self.materialize(s).reg
        order = [regs[id(s)] for s in syms]

        def spec(a):
            if isinstance(a, Sym):
                return ("reg", order.index(regs[id(a)]))
            if isinstance(a, CtxRef):
                return ("ctx", a.code)
            if isinstance(a, LogitsOut):
                return ("logits",)
            if a is self.step_ctx and a is not None:
                return ("step",)
            return ("const", a)

        cb = _Callback(fn, [spec(a) for a in args], {k: spec(v) for k, v in kwargs.items()}, in_place, what)
        self.callbacks.append(cb)
        out = None if in_place else self._new(out_cols, out_dtype)
        self._add(kind=OP_CALLBACK, in0=order[0] if order else -1, in1=order[1] if len(order) > 1 else -1,
                  out=-1 if out is None else out.reg, rows_ctx=rows_ctx, N=out_cols or 0,
                  out_dtype=_code(out_dtype) if out_dtype is not None else 0, is_head=1 if is_head else 0,
                  callback_id=len(self.callbacks) - 1)
        return out


class LogitsOut:
    """Stands for the step's logits buffer while recording."""


class StepProgram:
    """A recorded model on the C++ side. ``run`` executes one step; it returns False if the workspace is too
    small for the step, with nothing launched."""

    def __init__(self, hip_ops, recorder: Recorder, device: torch.device):
        self.hip_ops = hip_ops
        self.lib = hip_ops.lib
        _declare(self.lib)
        self.device = device
        self._keep = recorder.keep
        self.tunables = hip_ops.tunables()
        self.handle = c_void_p(self.lib.lmsf_program_create(ctypes.byref(hip_ops._tun)))
        for op in recorder.ops:
            if self.lib.lmsf_program_add(self.handle, ctypes.byref(op)) != 0:
                raise RuntimeError("step program: " + library.last_error(self.lib))
        if self.lib.lmsf_program_seal(self.handle) != 0:
            raise RuntimeError("step program: " + library.last_error(self.lib))
        self.n_ops = len(recorder.ops)
        self.callbacks = recorder.callbacks
        self._callback_fn = CallbackFn(self._on_callback)      # kept: the C side holds its address
        self.lib.lmsf_program_set_callback(self.handle, self._callback_fn)
        self._callback_error: Optional[BaseException] = None
        self._step = None                   # (context, logits) of the step that is running
        self.workspace: Optional[torch.Tensor] = None
        self.last_refusal = ""
        if hip_ops._bad_flag is None or hip_ops._bad_flag.device != device:
            hip_ops._bad_flag = torch.zeros(1, dtype=torch.int32, device=device)

    def __del__(self):
        try:
            self.lib.lmsf_program_destroy(self.handle)
        except Exception:  # noqa: BLE001 - interpreter shutdown
            pass

    def stale(self) -> bool:
        """True once somebody has changed the kernels' switch points since the recording (tests, tuning)."""
        return self.tunables != self.hip_ops.tunables()

    STAT_NAMES = ("plain", "mid", "large", "deferred", "gemv", "chunks", "skinny", "blas", "materialize", "mid_scaled",
                  "gemv_scaled", "skinny_scaled", "separate", "gemv_add_norm", "skinny_add_norm", "gemv_add",
                  "norm_over_partials", "rope_over_partials", "reduce_partials", "prefill_attention",
                  "decode_attention", "generic_attention", "callback")

    def last_step_stats(self) -> dict:
        """What the last step that ran launched, by kind: the products by their routes (csrc/dispatch.h), the
        kernels that took an unfinished product, the attention kernels, the callbacks."""
        out = (c_long * len(self.STAT_NAMES))()
        n = self.lib.lmsf_program_stats(self.handle, out, len(self.STAT_NAMES))
        return {name: int(out[i]) for i, name in enumerate(self.STAT_NAMES[:n]) if out[i]}

    def plan_capacity(self, n_tokens: int) -> int:
        return int(self.lib.lmsf_program_plan_capacity(self.handle, n_tokens))

    def write_plan(self, seg_lens, seg_first_pos, out_host, capacity: int):
        """The step's attention plan into ``out_host`` (int32 numpy view of pinned memory). Returns (ints written,
        where the plan's parts lie): the second travels with the step to ``run``."""
        lens = np.ascontiguousarray(seg_lens, dtype=np.int32)
        first = np.ascontiguousarray(seg_first_pos, dtype=np.int32)
        info = PlanInfo()
        n = self.lib.lmsf_program_plan(self.handle, len(lens), lens.ctypes.data, first.ctypes.data,
                                       out_host.ctypes.data, capacity, ctypes.byref(info))
        if n < 0:
            raise RuntimeError("step program: " + library.last_error(self.lib))
        return int(n), info

    def ensure_workspace(self, nbytes: int) -> None:
        if self.workspace is None or self.workspace.numel() < nbytes:
            self.workspace = None
            self.workspace = torch.empty((int(nbytes) + 255) // 256 * 256, dtype=torch.uint8, device=self.device)

    # -- sizing
    def workspace_need(self, n_tokens: int, n_segments: int, n_logit_rows: int, max_context: int,
                       n_groups: int, limit: int = 1 << 40) -> int:
        """Bytes of workspace with which a step of these sizes runs: the step is walked without launching at
        workspaces of growing size until one holds it. A step of ``n_tokens`` in ``n_segments`` requests; single
        tokens if the two are equal, else the first request holds the rest."""
        st = StepDesc()
        st.n_tokens, st.n_segments, st.n_logit_rows = n_tokens, n_segments, n_logit_rows
        st.max_context, st.all_single, st.n_groups = int(max_context), 1 if n_tokens == n_segments else 0, n_groups
        fake = 256                  # an address that a walk without launches never follows
        st.token_ids = st.positions = st.seg_of = st.logit_rows = st.longest_first = fake
        for g in range(n_groups):
            st.slots[g], st.tables[g], st.widths[g] = fake, fake, 1
        if not st.all_single:
            lens = [n_tokens - (n_segments - 1)] + [1] * (n_segments - 1)
            buf = np.empty(self.plan_capacity(n_tokens), dtype=np.int32)
            _, st.plan_info = self.write_plan(lens, [0] * n_segments, buf, buf.shape[0])
            st.plan = fake
        st.workspace, st.logits, st.bad_flag = fake, fake, fake

        def fits(nbytes: int) -> bool:
            st.workspace_bytes = nbytes
            rc = self.lib.lmsf_program_run(self.handle, ctypes.byref(st), 1, None)
            if rc not in (0, NO_ROOM):
                raise RuntimeError("step program: " + library.last_error(self.lib))
            return rc == 0

        hi = 1 << 20
        while not fits(hi):
            hi *= 2
            if hi > limit:
                raise RuntimeError("step program: a step of %d tokens needs more than %d bytes of workspace"
                                   % (n_tokens, limit))
        lo = hi // 2
        while hi - lo > max(1 << 20, hi // 64):
            mid = (lo + hi) // 2
            lo, hi = (lo, mid) if fits(mid) else (mid, hi)
        return hi

    # -- a step
    def run(self, ctx, logits: Optional[torch.Tensor], plan, stream: int) -> bool:
        st = StepDesc()
        st.n_tokens, st.n_segments, st.n_logit_rows = ctx.n_tokens, ctx.n_segments, ctx.n_logit_rows
        st.max_context, st.all_single, st.n_groups = int(ctx.max_context), 1 if ctx.all_single else 0, len(ctx.groups)
        st.token_ids, st.positions, st.seg_of = ctx.token_ids.data_ptr(), ctx.positions.data_ptr(), ctx.seg_of_token.data_ptr()
        st.logit_rows = ctx.logit_rows.data_ptr() if ctx.n_logit_rows else None
        st.longest_first = ctx.longest_first.data_ptr() if ctx.longest_first is not None else None
        for gi, g in enumerate(ctx.groups):
            st.slots[gi], st.tables[gi], st.widths[gi] = g.slots.data_ptr(), g.block_tables.data_ptr(), g.block_tables.shape[1]
        if plan is not None:
            st.plan, st.plan_info = plan
        st.workspace, st.workspace_bytes = self.workspace.data_ptr(), self.workspace.numel()
        st.logits = logits.data_ptr() if logits is not None else None
        st.bad_flag = self.hip_ops._bad_flag.data_ptr()
        self._step, self._callback_error = (ctx, logits), None
        try:
            rc = self.lib.lmsf_program_run(self.handle, ctypes.byref(st), 0, c_void_p(stream))
        finally:
            self._step = None
        if rc == 0:
            return True
        if self._callback_error is not None:
            err, self._callback_error = self._callback_error, None
            raise err
        if rc == NO_ROOM:
            self.last_refusal = library.last_error(self.lib)
            return False
        raise RuntimeError("lmsf_amd kernel error: " + library.last_error(self.lib))

    # -- a part that runs in Python in the middle of the program
    def _view(self, ref: TensorRef, logits: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        if ref.offset == -1:
            return None
        if ref.offset == -2:
            return logits
        dtype = _TORCH_OF_CODE[ref.dtype]
        nbytes = ref.rows * ref.cols * (4 if ref.dtype == 0 else 2)
        return self.workspace[ref.offset:ref.offset + nbytes].view(dtype).view(ref.rows, ref.cols)

    def _on_callback(self, args_p) -> int:
        try:
            a = args_p.contents
            cb = self.callbacks[a.callback_id]
            ctx, logits = self._step
            tensors = [self._view(a.in0, logits), self._view(a.in1, logits)]

            def real(spec):
                kind = spec[0]
                if kind == "reg":
                    return tensors[spec[1]]
                if kind == "ctx":
                    return _step_array(ctx, spec[1])
                if kind == "logits":
                    return logits
                if kind == "step":
                    return ctx
                return spec[1]

            result = cb.fn(*[real(s) for s in cb.args], **{k: real(s) for k, s in cb.kwargs.items()})
            if cb.in_place:
                return 0
            out = self._view(a.out, logits)
            if not isinstance(result, torch.Tensor):
                result = self.hip_ops.materialize(result)
            if result.data_ptr() != out.data_ptr():
                if tuple(result.shape) != tuple(out.shape) or result.dtype != out.dtype:
                    raise RuntimeError("%s returned %s of %s, its place in the program holds %s of %s"
                                       % (cb.what, tuple(result.shape), result.dtype, tuple(out.shape), out.dtype))
                out.copy_(result)
            return 0
        except BaseException as e:  # noqa: BLE001 - carried over the C frames and raised again by run()
            self._callback_error = e
            return 1


def _step_array(ctx, code: int):
    if code == CTX_TOKEN_IDS:
        return ctx.token_ids
    if code == CTX_POSITIONS:
        return ctx.positions
    if code == CTX_SEG_OF:
        return ctx.seg_of_token
    if code == CTX_LOGIT_ROWS:
        return ctx.logit_rows
    if CTX_SLOTS <= code < CTX_SLOTS + MAX_GROUPS:
        return ctx.groups[code - CTX_SLOTS].slots
    if CTX_TABLES <= code < CTX_TABLES + MAX_GROUPS:
        return ctx.groups[code - CTX_TABLES].block_tables
    raise KeyError(code)


last_failure: Optional[str] = None


def record_program(model, hip_ops, in_python: Optional[Callable[[Any, str], bool]] = None) -> Optional[StepProgram]:
    """The model's forward as a step program, or None if the model cannot be recorded (``last_failure`` says why).
    ``in_python(part, method name)``: True for calls that are to run in Python as callbacks although the recorder
    could follow them (to watch a part's operands in the middle of a step, say)."""
    global last_failure
    from ..engine.batch import GroupView, StepContext
    rt = model.rt
    if rt.device.type != "cuda" or type(hip_ops).__name__ != "HipOps":
        last_failure = "the kernels are not the HIP library's"
        return None
    n_groups = 1 + max((b.group for b in model.bindings if b.group is not None), default=-1)
    if n_groups > MAX_GROUPS:
        last_failure = "%d cache groups, the step program takes %d" % (n_groups, MAX_GROUPS)
        return None
    rec = Recorder(rt.dtype, model.spec.hidden_size, model.spec.vocab_size)
    rec.roles = {id(model.embedding): "embedding", id(model.head): "head"}
    rec.in_python = in_python
    groups = [GroupView(slots=CtxRef(CTX_SLOTS + g), block_tables=CtxRef(CTX_TABLES + g), page_size=0)
              for g in range(n_groups)]
    ctx = StepContext(
        n_tokens=1, n_segments=1, token_ids=CtxRef(CTX_TOKEN_IDS), positions=CtxRef(CTX_POSITIONS),
        seg_of_token=CtxRef(CTX_SEG_OF), seg_starts=None, seg_first_pos=None, state_slots=None,
        logit_rows=CtxRef(CTX_LOGIT_ROWS), n_logit_rows=1, groups=groups, replayed=True)
    rec.step_ctx = ctx
    real = rt.ops
    rt.ops = rec
    shadowed = []
    try:
        # every part's entry methods are guarded for the time of the recording (an attribute of the object that
        # shadows the class's method), so that a part the recorder cannot follow becomes a callback
        for part in model.parts():
            for name in ("forward", "forward_add", "apply"):
                if name in part.__dict__ or not callable(getattr(type(part), name, None)):
                    continue
                setattr(part, name, rec.guarded(part, name, getattr(part, name)))
                shadowed.append((part, name))
        out = model.forward(ctx, logits_out=LogitsOut())
        if not isinstance(out, Sym) or not rec.ops or rec.ops[-1].is_head != 1 or rec.ops[-1].out != out.reg:
            raise NotRecordable("the model's result is not its head's product into the logits buffer")
    except NotRecordable as e:
        last_failure = str(e)
        return None
    except Exception as e:  # noqa: BLE001 - a part that computes on a placeholder fails in its own way
        last_failure = "%s: %s" % (type(e).__name__, e)
        return None
    finally:
        rt.ops = real
        for part, name in shadowed:
            delattr(part, name)
    last_failure = None
    return StepProgram(hip_ops, rec, rt.device)
