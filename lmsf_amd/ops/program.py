"""Records a model's kernel calls once and runs them from C++ for every step.

The parts of a model call the kernels through ``rt.ops`` (ops.HipOps), one Python call per kernel.
``record_program`` runs the model's forward once over a ``Recorder`` that stands in for ``rt.ops``: the
activations it hands out are placeholders (``Sym``), the weights it is given are the real tensors. What
comes out is a list of operations over value registers, which ``csrc/program.hip`` keeps and runs: it
chooses the kernel of every operation from the step's number of rows exactly as ``HipOps`` does, takes
temporaries from one workspace, and launches; a step is then one call from Python instead of hundreds.

A model is recordable if its parts do nothing to activations but pass them to ``rt.ops``. A part that
computes on a tensor itself (a toy mixer written with torch, a position encoding that acts in place)
meets a placeholder, the recording fails, ``record_program`` returns None with the reason in
``last_failure``, and the engine runs that model part by part as before. No part knows of any of this.

The reference's step is native from the worker down (core/src/worker/model_worker.rs:213-264,
core/src/model_executor/models/llama/llama.rs:397-476).
"""
import ctypes
from ctypes import POINTER, Structure, c_float, c_int, c_long, c_void_p
from typing import Any, List, Optional

import torch

from . import library
from .handles import DeferredLinear, PendingProduct, ScaledRows  # noqa: F401  (what the placeholders stand for)

MAX_GROUPS = 8
NOT_NATIVE, NO_ROOM = 3, 4

OP_EMBEDDING, OP_ADD_RMS_NORM, OP_QKV_ROPE_CACHE, OP_ATTENTION, OP_LINEAR, OP_LINEAR_GATED, OP_MATERIALIZE = range(1, 8)
CTX_NONE, CTX_TOKEN_IDS, CTX_POSITIONS, CTX_SEG_OF, CTX_LOGIT_ROWS, CTX_SLOTS, CTX_TABLES = 0, 1, 2, 3, 4, 16, 32


class Tunables(Structure):
    _fields_ = [(n, c_int) for n in (
        "fuse_norm_rows", "fuse_stream_rows", "gemv_max_rows", "skinny_variant", "mid_wide_max_cols", "mid_max_rows",
        "skinny_max_rows", "prefill_attention_variant", "decode_attention_order", "decode_attention_splits",
        "use_library_gemm", "large_max_rows", "large_deep_min_rows", "mid_scaled_rows")]


class OpDesc(Structure):
    _fields_ = ([(n, c_int) for n in ("kind", "in0", "in1", "out", "ctx0", "ctx1", "rows_ctx")]
                + [(n, c_void_p) for n in ("w", "bias", "table", "k_pages", "v_pages")]
                + [(n, c_int) for n in ("wdtype", "out_dtype", "cache_dtype", "N", "K")]
                + [("ldw", c_long)]
                + [(n, c_int) for n in ("nh", "nkv", "d", "rot", "neox", "ps", "window", "max_pos", "act", "defer_ok",
                                        "pending_ok", "is_head", "vocab")]
                + [("num_pages", c_long)]
                + [(n, c_float) for n in ("eps", "weight_offset", "scale")])


class StepDesc(Structure):
    _fields_ = ([(n, c_int) for n in ("n_tokens", "n_segments", "n_logit_rows", "max_context", "all_single", "n_groups")]
                + [(n, c_void_p) for n in ("token_ids", "positions", "seg_of", "logit_rows", "longest_first")]
                + [("slots", c_void_p * MAX_GROUPS), ("tables", c_void_p * MAX_GROUPS), ("widths", c_int * MAX_GROUPS)]
                + [("plan", c_void_p), ("workspace", c_void_p), ("workspace_bytes", c_long), ("logits", c_void_p),
                   ("bad_flag", c_void_p)])


_SIGNATURES = {
    "lmsf_program_create": (c_void_p, [POINTER(Tunables)]),
    "lmsf_program_destroy": (None, [c_void_p]),
    "lmsf_program_add": (c_int, [c_void_p, POINTER(OpDesc)]),
    "lmsf_program_seal": (c_int, [c_void_p]),
    "lmsf_program_plan": (c_long, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_long]),
    "lmsf_program_plan_capacity": (c_long, [c_void_p, c_int]),
    "lmsf_program_run": (c_int, [c_void_p, POINTER(StepDesc), c_int, c_void_p]),
}


def _declare(lib) -> None:
    if getattr(lib, "_lmsf_program_declared", False):
        return
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    lib._lmsf_program_declared = True


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return 0
    if dtype == torch.bfloat16:
        return 1
    raise NotRecordable("a tensor of %s" % dtype)


class NotRecordable(Exception):
    """The model does something that the step program has no operation for."""


class Sym:
    """An activation that does not exist yet: the value of a register."""

    __slots__ = ("reg",)

    def __init__(self, reg: int):
        self.reg = reg

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


class Recorder:
    """Stands in for ``HipOps`` while the model's forward is recorded: the same methods, which note what they
    were asked instead of launching it."""

    name = "recorder"

    def __init__(self, run_dtype: torch.dtype):
        self.ops: List[OpDesc] = []
        self.keep: List[torch.Tensor] = []      # every tensor an operation points to stays alive with the program
        self.n_regs = 0
        self.run_dtype = run_dtype

    # -- helpers
    def _new(self) -> Sym:
        self.n_regs += 1
        return Sym(self.n_regs - 1)

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
        out = self._new()
        self._add(kind=OP_EMBEDDING, out=out.reg, ctx0=self._ctx(ids, "the embedding's ids"), w=_w(table),
                  wdtype=_code(table.dtype), N=table.shape[1], vocab=table.shape[0], scale=float(scale))
        return out

    def add_rms_norm(self, branch, residual, weight, eps, out_dtype, rows=None, weight_offset: float = 0.0,
                     defer_ok: bool = False):
        weight = self._weight(weight, "a norm's weight", 1)
        out = self._new()
        self._add(kind=OP_ADD_RMS_NORM, in0=self._reg(branch, "a norm's branch", optional=True),
                  in1=self._reg(residual, "a norm's residual", optional=True), out=out.reg,
                  rows_ctx=self._ctx(rows, "a norm's rows", optional=True), w=_w(weight), wdtype=_code(weight.dtype),
                  N=weight.shape[0], eps=float(eps), weight_offset=float(weight_offset), out_dtype=_code(out_dtype),
                  defer_ok=1 if defer_ok else 0)
        return out

    def qkv_rope_cache(self, x, weight, bias, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages, v_pages):
        weight = self._weight(weight, "the QKV weight", 2)
        bias = self._weight(bias, "the QKV bias", 1)
        if bias is not None and (bias.dtype != weight.dtype or bias.shape[0] != weight.shape[0] or not bias.is_contiguous()):
            raise NotRecordable("the QKV bias does not fit its weight")
        if table is not None:
            table = self._weight(table, "the rotary table", 2)
            if table.dtype != torch.float32 or table.shape[1] != rot_dim or not table.is_contiguous():
                raise NotRecordable("the rotary table is not contiguous float32 [max_pos, %d]" % rot_dim)
        fields = {}
        if slots is not None:
            fields = self._pages(k_pages, v_pages, nkv, d)
        out = self._new()
        self._add(kind=OP_QKV_ROPE_CACHE, in0=self._reg(x, "the QKV projection's input"), out=out.reg,
                  ctx0=self._ctx(positions, "positions"), ctx1=self._ctx(slots, "slots", optional=True), w=_w(weight),
                  bias=_w(bias), table=_w(table), wdtype=_code(weight.dtype), N=weight.shape[0], K=weight.shape[1],
                  ldw=weight.stride(0), nh=int(nh), nkv=int(nkv), d=int(d), rot=int(rot_dim) if table is not None else 0,
                  neox=1 if neox else 0, max_pos=table.shape[0] if table is not None else 0, **fields)
        return out

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
        out = self._new()
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
        res = self._new()
        self._add(kind=OP_LINEAR, in0=self._reg(x, "a product's input"), out=res.reg,
                  out_dtype=_code(out_dtype or self.run_dtype), pending_ok=1 if pending_ok else 0,
                  is_head=1 if is_head else 0, **self._linear_fields(weight, bias, "a product's"))
        return res

    def linear_gated(self, x, weight, bias=None, kind: str = "silu"):
        kinds = {"silu": 1, "gelu": 2}
        if kind not in kinds or weight.shape[0] % 2 != 0:
            raise NotRecordable("a gated product of kind %r" % (kind,))
        res = self._new()
        self._add(kind=OP_LINEAR_GATED, in0=self._reg(x, "a gated product's input"), out=res.reg, act=kinds[kind],
                  **self._linear_fields(weight, bias, "a gated product's"))
        return res

    def materialize(self, y):
        if not isinstance(y, Sym):
            return y
        res = self._new()
        self._add(kind=OP_MATERIALIZE, in0=y.reg, out=res.reg)
        return res

    def __getattr__(self, name):
        raise NotRecordable("a part calls the kernel %r, which the step program does not have" % name)


class LogitsOut:
    """Stands for the step's logits buffer while recording."""


class StepProgram:
    """A recorded model on the C++ side. ``run`` executes one step; it returns False if the step has to go the
    long way (it needs a product of the BLAS library, or more workspace than there is), with nothing launched."""

    def __init__(self, hip_ops, recorder: Recorder, device: torch.device):
        self.hip_ops = hip_ops
        self.lib = hip_ops.lib
        _declare(self.lib)
        self.device = device
        self._keep = recorder.keep
        t = Tunables(*(int(getattr(hip_ops, n)) for n, _ in Tunables._fields_))
        self.handle = c_void_p(self.lib.lmsf_program_create(ctypes.byref(t)))
        self.tunables = tuple(int(getattr(hip_ops, n)) for n, _ in Tunables._fields_)
        for op in recorder.ops:
            if self.lib.lmsf_program_add(self.handle, ctypes.byref(op)) != 0:
                raise RuntimeError("step program: " + library.last_error(self.lib))
        if self.lib.lmsf_program_seal(self.handle) != 0:
            raise RuntimeError("step program: " + library.last_error(self.lib))
        self.n_ops = len(recorder.ops)
        self.workspace: Optional[torch.Tensor] = None
        self._refused = set()          # (tokens, wanted rows) of steps that were refused once: not asked again
        if hip_ops._bad_flag is None or hip_ops._bad_flag.device != device:
            hip_ops._bad_flag = torch.zeros(1, dtype=torch.int32, device=device)

    def __del__(self):
        try:
            self.lib.lmsf_program_destroy(self.handle)
        except Exception:  # noqa: BLE001 - interpreter shutdown
            pass

    def stale(self) -> bool:
        """True once somebody has changed the kernels' switch points since the recording (tests, tuning)."""
        return self.tunables != tuple(int(getattr(self.hip_ops, n)) for n, _ in Tunables._fields_)

    def plan_capacity(self, n_tokens: int) -> int:
        return int(self.lib.lmsf_program_plan_capacity(self.handle, n_tokens))

    def write_plan(self, seg_lens, seg_first_pos, out_host, capacity: int) -> int:
        """The step's attention plan into ``out_host`` (int32 numpy view of pinned memory); ints written."""
        import numpy as np
        lens = np.ascontiguousarray(seg_lens, dtype=np.int32)
        first = np.ascontiguousarray(seg_first_pos, dtype=np.int32)
        n = self.lib.lmsf_program_plan(self.handle, len(lens), lens.ctypes.data, first.ctypes.data,
                                       out_host.ctypes.data, capacity)
        if n < 0:
            raise RuntimeError("step program: " + library.last_error(self.lib))
        return int(n)

    def ensure_workspace(self, nbytes: int) -> None:
        if self.workspace is None or self.workspace.numel() < nbytes:
            self.workspace = None
            self.workspace = torch.empty(int(nbytes), dtype=torch.uint8, device=self.device)

    def run(self, ctx, logits: Optional[torch.Tensor], plan_ptr: Optional[int], stream: int,
            check_only: bool = False) -> bool:
        key = (ctx.n_tokens, ctx.n_logit_rows)
        if key in self._refused:
            return False
        st = StepDesc()
        st.n_tokens, st.n_segments, st.n_logit_rows = ctx.n_tokens, ctx.n_segments, ctx.n_logit_rows
        st.max_context, st.all_single, st.n_groups = int(ctx.max_context), 1 if ctx.all_single else 0, len(ctx.groups)
        st.token_ids, st.positions, st.seg_of = ctx.token_ids.data_ptr(), ctx.positions.data_ptr(), ctx.seg_of_token.data_ptr()
        st.logit_rows = ctx.logit_rows.data_ptr() if ctx.n_logit_rows else None
        st.longest_first = ctx.longest_first.data_ptr() if ctx.longest_first is not None else None
        for gi, g in enumerate(ctx.groups):
            st.slots[gi], st.tables[gi], st.widths[gi] = g.slots.data_ptr(), g.block_tables.data_ptr(), g.block_tables.shape[1]
        st.plan = plan_ptr
        st.workspace, st.workspace_bytes = self.workspace.data_ptr(), self.workspace.numel()
        st.logits = logits.data_ptr() if logits is not None else None
        st.bad_flag = self.hip_ops._bad_flag.data_ptr()
        rc = self.lib.lmsf_program_run(self.handle, ctypes.byref(st), 1 if check_only else 0, c_void_p(stream))
        if rc == 0:
            return True
        if rc in (NOT_NATIVE, NO_ROOM):
            if rc == NOT_NATIVE:
                self._refused.add(key)
            self.last_refusal = library.last_error(self.lib)
            return False
        raise RuntimeError("lmsf_amd kernel error: " + library.last_error(self.lib))


last_failure: Optional[str] = None


def record_program(model, hip_ops) -> Optional[StepProgram]:
    """The model's forward as a step program, or None if the model cannot be recorded (``last_failure`` says why)."""
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
    rec = Recorder(rt.dtype)
    groups = [GroupView(slots=CtxRef(CTX_SLOTS + g), block_tables=CtxRef(CTX_TABLES + g), page_size=0)
              for g in range(n_groups)]
    ctx = StepContext(
        n_tokens=1, n_segments=1, token_ids=CtxRef(CTX_TOKEN_IDS), positions=CtxRef(CTX_POSITIONS),
        seg_of_token=CtxRef(CTX_SEG_OF), seg_starts=None, seg_first_pos=None, state_slots=None,
        logit_rows=CtxRef(CTX_LOGIT_ROWS), n_logit_rows=1, groups=groups, replayed=True)
    real = rt.ops
    rt.ops = rec
    try:
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
    last_failure = None
    return StepProgram(hip_ops, rec, rt.device)
