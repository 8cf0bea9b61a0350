"""The kernels as Python calls on torch tensors.

Every method checks on the host that shapes, dtypes, devices and contiguity match what the
kernel and its grid assume, then passes raw device pointers and the current HIP stream to
the library. Nothing here computes on the CPU and nothing falls back to a library routine
except where the matrix products say so (``linear``).
"""
import ctypes
from typing import Optional

import torch

from . import dispatch as D
from . import library
from .handles import DeferredLinear, PendingProduct, ScaledRows

F32 = 0
BF16 = 1


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise TypeError("kernels take float32 or bfloat16 tensors, got %s" % dtype)


try:
    _raw_stream, _current_device = torch._C._cuda_getCurrentRawStream, torch._C._cuda_getDevice
except AttributeError:      # a torch without these: the documented way

    def _raw_stream(device_index: int) -> int:
        return torch.cuda.current_stream(device_index).cuda_stream

    _current_device = torch.cuda.current_device


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


class HipOps:
    """Kernel calls of the product path. One instance per process is enough."""

    name = "hip"

    def __init__(self):
        if not torch.cuda.is_available():
            raise library.KernelLibraryError(
                "lmsf_amd needs a GPU: torch.cuda.is_available() is False and there is no CPU path")
        self.lib = library.load_library()
        buf = ctypes.create_string_buffer(256)
        if self.lib.lmsf_device_arch(buf, 256) != 0:
            raise library.KernelLibraryError(library.last_error(self.lib))
        self.device_arch = buf.value.decode()
        if not self.device_arch.startswith("gfx950"):
            raise library.KernelLibraryError(
                "the kernels are built for gfx950 only; this device reports %r" % self.device_arch)
        self._bad_flag = None
        # The switch points between the kernels live in one structure that the C++ side reads (csrc/dispatch.h says
        # what each means); they are attributes of this object all the same (see __setattr__).
        self.use_library_gemm = True   # bfloat16 matrix products of many rows go to the BLAS library
        self.prefill_attention_variant = 0
        self.decode_attention_order = 0
        self.decode_attention_splits = 0
        self.fuse_norm_rows = 16
        self.fuse_stream_rows = 1
        self.gemv_max_rows = 2
        self.skinny_variant = 0
        self.mid_wide_max_cols = 8192  # beyond 64 rows only products of up to this many columns: the library is good at the wide ones (measured)
        self.mid_max_rows = 128        # rows up to which the 17-and-more-rows kernel beats the library (64 with the gated activation)
        self.skinny_max_rows = 16      # rows up to which the few-rows kernel beats the library (measured)
        self.large_max_rows = 256      # rows up to which the many-rows kernel beats the library (measured; 0: never)
        self.large_deep_min_rows = 64    # products whose K is at least three times N go to the many-rows kernel from beyond this many rows already (down at 128 rows: 42.8 -> 38.0 us; decode at batch 128: 6.63 -> 6.53 ms a step, at 96: 5.83 -> 5.74)
        self.mid_scaled_rows = 16        # rows up to which the gated product after a norm runs in the 17-and-more-rows kernel where that kernel's workgroups fit on the chip at once (0: never)
        self.large_deep_max_rows = 1024  # the same for products whose K is at least three times N (down: 57 against 76 us at 320 rows, 74 against 94 at 512, 102 against 108 at 768, level at 1,024)
        self.qkv_fused_max_rows = 32     # rows up to which the QKV product with rotation and cache write runs in the few-rows kernel, beyond skinny_max_rows (one kernel against the 17-and-more-rows product and the rotary kernel over its partial sums: decode at batch 24 3.99 -> 3.92 ms a step, at 32 4.11 -> 3.99; level at 48, behind at 64: 4.80 -> 4.87)
        self.weight_row_pad_bytes = 512  # bytes left between two rows of a linear layer's weight (see weight_row_pad)
        # the BLAS library's products are called from C++ (csrc/blas.hip); its handle and workspace are made here
        if self.lib.lmsf_blas_init(self.blas_workspace_bytes) != 0:
            raise library.KernelLibraryError("the BLAS library cannot be used: " + library.last_error(self.lib))

    blas_workspace_bytes = 128 << 20

    def __setattr__(self, name, value):
        if name in D.TUNABLE_NAMES:
            setattr(self.__dict__.setdefault("_tun", D.Tunables()), name, int(value))
        else:
            object.__setattr__(self, name, value)

    def __getattr__(self, name):
        # (called only for names that are no ordinary attributes: the switch points)
        if name in D.TUNABLE_NAMES and "_tun" in self.__dict__:
            return int(getattr(self.__dict__["_tun"], name))
        raise AttributeError(name)

    def tunables(self) -> tuple:
        """The switch points as they are now, in the order of ``dispatch.TUNABLE_NAMES``."""
        return self._tun.as_tuple()

    def _shape(self, x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype) -> D.ProductShape:
        """What the C++ side wants to know of a product x weight^T before it names the kernel."""
        return D.ProductShape(x.shape[0], weight.shape[0], x.shape[1], _code(x.dtype), _code(weight.dtype),
                              _code(out_dtype), x.stride(0), weight.stride(0), 1 if x.data_ptr() % 16 == 0 else 0,
                              1 if weight.data_ptr() % 16 == 0 else 0)

    # ------------------------------------------------------------------ helpers

    def _stream(self):
        # (the raw handle of the current device's current stream; torch.cuda.current_stream() gives the same
        # handle wrapped in an object and costs 8 us a call, a third of the host's time in a step of few tokens)
        return ctypes.c_void_p(_raw_stream(_current_device()))

    def _check(self, rc: int):
        if rc != 0:
            raise RuntimeError("lmsf_amd kernel error: " + library.last_error(self.lib))

    @staticmethod
    def _dev(*tensors):
        for t in tensors:
            if t is not None and not t.is_cuda:
                raise ValueError("kernel operand is not on the GPU")

    @staticmethod
    def _i32(t: Optional[torch.Tensor], name: str, numel: Optional[int] = None):
        if t is None:
            return
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise ValueError("%s must be a contiguous int32 tensor" % name)
        if numel is not None and t.numel() < numel:
            raise ValueError("%s holds %d elements, %d needed" % (name, t.numel(), numel))

    # ------------------------------------------------------------------ embedding

    def embedding(self, ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        """float32 [N, H] rows of ``table`` [V, H] selected by int32 ``ids`` [N], times ``scale``."""
        self._dev(ids, table)
        self._i32(ids, "ids")
        if table.dim() != 2 or not table.is_contiguous():
            raise ValueError("embedding table must be contiguous [V, H]")
        n, (V, H) = ids.numel(), table.shape
        out = torch.empty((n, H), dtype=torch.float32, device=table.device)
        if self._bad_flag is None or self._bad_flag.device != table.device:
            self._bad_flag = torch.zeros(1, dtype=torch.int32, device=table.device)
        self._check(self.lib.lmsf_embedding(_ptr(ids), _ptr(table), _code(table.dtype), _ptr(out), n, H, V,
                                            float(scale), _ptr(self._bad_flag), self._stream()))
        return out

    def patch_tokens(self, ids: torch.Tensor, src: torch.Tensor, prev: torch.Tensor) -> None:
        """ids[i] = prev[src[i]] where src[i] >= 0 (all int32, on the device): a step launched ahead takes the
        tokens that the step before it sampled from where the sampler left them."""
        self._dev(ids, src, prev)
        self._i32(ids, "ids")
        self._i32(src, "src", ids.numel())
        self._i32(prev, "prev")
        self._check(self.lib.lmsf_patch_tokens(_ptr(ids), _ptr(src), _ptr(prev), ids.numel(), prev.numel(),
                                               self._stream()))

    def bad_token_seen(self) -> bool:
        """True if an embedding call since the last query met an id outside the vocabulary."""
        if self._bad_flag is None:
            return False
        bad = bool(self._bad_flag.item())
        if bad:
            self._bad_flag.zero_()
        return bad

    # ------------------------------------------------------------------ norm

    def add_rms_norm(self, branch: Optional[torch.Tensor], residual: Optional[torch.Tensor], weight: torch.Tensor,
                     eps: float, out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                     weight_offset: float = 0.0, defer_ok: bool = False):
        """out = rms_norm(branch + residual) * (weight + weight_offset).

        ``residual`` (float32 [N, H]) is updated to the sum in place when both operands are given
        and ``rows`` is None. ``rows`` (int32 [R]) selects input rows; the output then has R rows.
        ``branch`` may be a ``PendingProduct``: its partial sums are added up on the way in; or a
        ``DeferredLinear``, which then runs as a product that adds into ``residual``. With ``defer_ok``
        the caller takes a ``ScaledRows`` as well (up to 16 rows, after a ``DeferredLinear``).
        """
        if isinstance(branch, PendingProduct):
            return self._add_rms_norm_pending(branch, residual, weight, eps, out_dtype, rows, weight_offset)
        if isinstance(branch, DeferredLinear):
            handle, branch = self._run_deferred(branch, residual, weight, eps, out_dtype, rows, weight_offset, defer_ok)
            if handle is not None:
                return handle
        self._dev(branch, residual, weight, rows)
        ref = branch if branch is not None else residual
        if ref is None:
            raise ValueError("add_rms_norm needs a branch or a residual")
        if ref.dim() != 2 or not ref.is_contiguous():
            raise ValueError("add_rms_norm operands must be contiguous [N, H]")
        N, H = ref.shape
        if branch is not None and residual is not None and branch.shape != residual.shape:
            raise ValueError("branch %s and residual %s differ in shape" % (tuple(branch.shape), tuple(residual.shape)))
        if residual is not None and (residual.dtype != torch.float32 or not residual.is_contiguous()):
            raise ValueError("the residual stream must be contiguous float32")
        if weight.shape != (H,) or not weight.is_contiguous():
            raise ValueError("norm weight must be [%d], got %s" % (H, tuple(weight.shape)))
        self._i32(rows, "rows")
        n_out = N if rows is None else rows.numel()
        out = torch.empty((n_out, H), dtype=out_dtype, device=ref.device)
        self._check(self.lib.lmsf_add_rms_norm(
            _ptr(branch), _code(branch.dtype) if branch is not None else F32, _ptr(residual), _ptr(weight),
            _code(weight.dtype), _ptr(out), _code(out_dtype), _ptr(rows), n_out, H, float(eps),
            float(weight_offset), self._stream()))
        return out

    def _run_deferred(self, branch: DeferredLinear, residual: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                      out_dtype: torch.dtype, rows: Optional[torch.Tensor], weight_offset: float, defer_ok: bool):
        """Runs the product that ``branch`` stands for, in the form that leaves the norm the least to do.
        Returns (handle, branch): a ``ScaledRows`` if the product did the norm's preparation as well (then the
        norm is done), else None and what is left to add: nothing if the product added into the stream itself,
        the product's tensor otherwise."""
        M, N = branch.shape
        K = branch.x.shape[1]
        fits = (rows is None and residual is not None and residual.dtype == torch.float32
                and residual.is_contiguous() and tuple(residual.shape) == branch.shape)
        prepares = (fits and defer_ok and out_dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
                    and weight.is_contiguous() and weight.shape == (N,))
        rt = D.Route()
        self.lib.lmsf_route_deferred_norm(ctypes.byref(self._tun), M, N, K, 1 if fits else 0, 1 if prepares else 0,
                                          ctypes.byref(rt))
        operands = (_ptr(branch.x), branch.x.stride(0), _ptr(branch.weight), branch.weight.stride(0), _ptr(branch.bias))
        if rt.route == D.GEMV_ADD_NORM:
            # adds into the stream, leaves stream * w and its workgroups' sums of squares
            self._dev(branch.x, branch.weight, branch.bias, residual, weight)
            parts = self.lib.lmsf_gemv_partials(N)
            xw = torch.empty((M, N), dtype=torch.bfloat16, device=residual.device)
            sumsq = torch.empty(parts * M, dtype=torch.float32, device=residual.device)
            self._check(self.lib.lmsf_gemv_add_norm(*operands, _ptr(residual), residual.stride(0), _ptr(weight),
                                                    float(weight_offset), _ptr(xw), xw.stride(0), _ptr(sumsq), M, N, K,
                                                    self._stream()))
            return ScaledRows(xw, sumsq, parts, M, residual, weight, float(eps), float(weight_offset), out_dtype), None
        if rt.route == D.SKINNY_ADD_NORM:
            # the same from the few-rows kernel: sums of squares per 16 columns
            self._dev(branch.x, branch.weight, branch.bias, residual, weight)
            tiles = -(-N // 16)
            xw = torch.empty((M, N), dtype=torch.bfloat16, device=residual.device)
            sumsq = torch.empty(tiles * 16, dtype=torch.float32, device=residual.device)
            self._check(self.lib.lmsf_gemm_skinny_add_norm(*operands, _ptr(residual), residual.stride(0), _ptr(weight),
                                                           float(weight_offset), _ptr(xw), xw.stride(0), _ptr(sumsq), M,
                                                           N, K, self.skinny_variant, self._stream()))
            return ScaledRows(xw, sumsq, tiles, 16, residual, weight, float(eps), float(weight_offset), out_dtype), None
        if rt.route == D.GEMV_ADD:
            # adds into the stream; the norm kernel follows
            self._dev(branch.x, branch.weight, branch.bias, residual)
            self._check(self.lib.lmsf_gemv_add(*operands, _ptr(residual), residual.stride(0), M, N, K, self._stream()))
            return None, None
        return None, self.materialize(branch)

    def _add_rms_norm_pending(self, branch: PendingProduct, residual: Optional[torch.Tensor], weight: torch.Tensor,
                              eps: float, out_dtype: torch.dtype, rows: Optional[torch.Tensor],
                              weight_offset: float) -> torch.Tensor:
        M, H = branch.shape
        fits = (H % 4 == 0 and H <= 16384 and weight.shape == (H,) and weight.is_contiguous()
                and weight.data_ptr() % 16 == 0
                and (residual is None or (residual.dtype == torch.float32 and residual.is_contiguous()
                                          and tuple(residual.shape) == (M, H) and residual.data_ptr() % 16 == 0)))
        if not fits:
            return self.add_rms_norm(self.materialize(branch), residual, weight, eps, out_dtype, rows, weight_offset)
        self._dev(residual, weight, rows)
        self._i32(rows, "rows")
        n_out = M if rows is None else rows.numel()
        out = torch.empty((n_out, H), dtype=out_dtype, device=branch.device)
        self._check(self.lib.lmsf_add_rms_norm_partial(
            _ptr(branch.partials), _ptr(branch.bias), branch.partials.shape[0], M, _ptr(residual), _ptr(weight),
            _code(weight.dtype), _ptr(out), _code(out_dtype), _ptr(rows), n_out, H, float(eps), float(weight_offset),
            self._stream()))
        return out

    def materialize(self, y):
        """The tensor behind ``y``: ``y`` itself, the finished sum of a ``PendingProduct``, the product of a
        ``DeferredLinear`` or the norm of a ``ScaledRows``."""
        if isinstance(y, DeferredLinear):
            return self.linear(y.x, y.weight, y.bias, out_dtype=y.dtype)
        if isinstance(y, ScaledRows):
            return self.add_rms_norm(None, y.stream, y.weight, y.eps, y.dtype, weight_offset=y.weight_offset)
        if not isinstance(y, PendingProduct):
            return y
        M, N = y.shape
        out = torch.empty((M, N), dtype=y.dtype, device=y.device)
        self._check(self.lib.lmsf_gemm_mid_reduce(_ptr(y.partials), _ptr(y.bias), _ptr(out), _code(y.dtype),
                                                  out.stride(0), M, N, y.partials.shape[0], self._stream()))
        return out

    # ------------------------------------------------------------------ rotary + cache write

    def rope_cache_write(self, qkv: torch.Tensor, nh: int, nkv: int, d: int, positions: Optional[torch.Tensor],
                         table: Optional[torch.Tensor], rot_dim: int, neox: bool, slots: Optional[torch.Tensor],
                         k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor]) -> None:
        """Rotate the q and k heads of the fused ``qkv`` [N, (nh + 2 nkv) d] in place and store k, v in
        the pages at ``slots``. ``table`` None: no rotation. ``slots`` None: no cache write."""
        self._dev(qkv, positions, table, slots, k_pages, v_pages)
        if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] != (nh + 2 * nkv) * d:
            raise ValueError("qkv must be [N, %d] with unit column stride, got %s" % ((nh + 2 * nkv) * d,
                                                                                      tuple(qkv.shape)))
        N = qkv.shape[0]
        es = qkv.element_size()
        max_pos = 0
        if table is not None:
            if table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] != rot_dim or not table.is_contiguous():
                raise ValueError("rotary table must be contiguous float32 [max_pos, %d]" % rot_dim)
            self._i32(positions, "positions", N)
            if positions is None:
                raise ValueError("rotation needs positions")
            max_pos = table.shape[0]
        num_pages, ps = 0, 1
        if slots is not None:
            self._i32(slots, "slots", N)
            if k_pages is None or k_pages.dim() != 4 or k_pages.shape[1] != nkv or k_pages.shape[3] != d \
                    or not k_pages.is_contiguous() or k_pages.dtype != qkv.dtype:
                raise ValueError("k_pages must be contiguous [pages, %d, page_size, %d] of %s" % (nkv, d, qkv.dtype))
            num_pages, ps = k_pages.shape[0], k_pages.shape[2]
            if v_pages is None or tuple(v_pages.shape) != (num_pages, nkv, d, ps) or not v_pages.is_contiguous() \
                    or v_pages.dtype != qkv.dtype:
                raise ValueError("v_pages must be contiguous [%d, %d, %d, %d] of %s" % (num_pages, nkv, d, ps, qkv.dtype))
        base = qkv.data_ptr()
        q = ctypes.c_void_p(base)
        k = ctypes.c_void_p(base + nh * d * es)
        v = ctypes.c_void_p(base + (nh + nkv) * d * es)
        self._check(self.lib.lmsf_rope_cache_write(
            q, k, v, _code(qkv.dtype), N, qkv.stride(0), _ptr(positions), _ptr(table), rot_dim, 1 if neox else 0,
            max_pos, _ptr(slots), _ptr(k_pages), _ptr(v_pages), num_pages, nh, nkv, d, ps, self._stream()))

    def _check_qkv_fused(self, bias, weight, N, table, d, positions, slots, M, k_pages, v_pages, nkv):
        """Operand checks of the fused QKV forms; returns (pages, page size)."""
        if bias is not None and (bias.shape != (N,) or bias.dtype != weight.dtype or not bias.is_contiguous()):
            raise ValueError("qkv_rope_cache: bias must be [%d] of the weight's dtype" % N)
        if table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] != d or not table.is_contiguous():
            raise ValueError("rotary table must be contiguous float32 [max_pos, %d]" % d)
        self._i32(positions, "positions", M)
        self._i32(slots, "slots", M)
        if k_pages.dim() != 4 or k_pages.shape[1] != nkv or k_pages.shape[3] != d or not k_pages.is_contiguous():
            raise ValueError("k_pages must be contiguous [pages, %d, page_size, %d]" % (nkv, d))
        num_pages, ps = k_pages.shape[0], k_pages.shape[2]
        if v_pages is None or tuple(v_pages.shape) != (num_pages, nkv, d, ps) or not v_pages.is_contiguous() \
                or v_pages.dtype != torch.bfloat16:
            raise ValueError("v_pages must be contiguous bfloat16 [%d, %d, %d, %d]" % (num_pages, nkv, d, ps))
        return num_pages, ps

    def qkv_rope_cache(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], nh: int, nkv: int,
                       d: int, positions: torch.Tensor, table: Optional[torch.Tensor], rot_dim: int, neox: bool,
                       slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                       v_pages: Optional[torch.Tensor]) -> torch.Tensor:
        """The fused QKV projection, the rotation of its q and k heads and the write of k and v into the
        pages: ``linear`` followed by ``rope_cache_write``, with the same results. With few bfloat16 rows and
        a NeoX rotation over the whole head, the rotation and the write are the product's epilogue. ``x`` may
        be a ``ScaledRows``."""
        M, K = x.shape
        N = (nh + 2 * nkv) * d
        scaled = isinstance(x, ScaledRows)
        xt = x.xw if scaled else x
        fused_shape = (table is not None and slots is not None and neox and rot_dim == d and d % 32 == 0
                       and weight.dtype == torch.bfloat16 and tuple(weight.shape) == (N, K) and xt.stride(1) == 1
                       and weight.stride(1) == 1 and k_pages is not None and k_pages.dtype == torch.bfloat16)
        rt = D.Route()
        self.lib.lmsf_route_qkv(ctypes.byref(self._tun), ctypes.byref(self._shape(xt, weight, xt.dtype)),
                                1 if fused_shape else 0, x.rows_per_tile if scaled else 0, ctypes.byref(rt))
        if rt.route == D.MATERIALIZE:
            return self.qkv_rope_cache(self.materialize(x), weight, bias, nh, nkv, d, positions, table, rot_dim,
                                       neox, slots, k_pages, v_pages)
        if rt.route != D.SEPARATE:
            self._dev(xt, weight, bias, positions, table, slots, k_pages, v_pages)
            num_pages, ps = self._check_qkv_fused(bias, weight, N, table, d, positions, slots, M, k_pages, v_pages, nkv)
            y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
            head = (_ptr(xt), xt.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(y), y.stride(0), M, K,
                    _ptr(positions), _ptr(table), table.shape[0], _ptr(slots), _ptr(k_pages), _ptr(v_pages), num_pages,
                    nh, nkv, d, ps)
            if rt.route == D.GEMV_SCALED:
                self._dev(x.sumsq)
                self._check(self.lib.lmsf_gemv_scaled_qkv_rope_cache(*head, _ptr(x.sumsq), x.tiles, x.eps, self._stream()))
            elif rt.route == D.SKINNY_SCALED:
                self._dev(x.sumsq)
                self._check(self.lib.lmsf_gemm_qkv_rope_cache_scaled(*head, _ptr(x.sumsq), x.tiles, x.eps, self._stream()))
            elif rt.route == D.GEMV:
                self._check(self.lib.lmsf_gemv_qkv_rope_cache(*head, self._stream()))
            else:
                self._check(self.lib.lmsf_gemm_qkv_rope_cache(*head, self.skinny_variant, self._stream()))
            return y
        y = self.linear(x, weight, bias, pending_ok=bool(rt.pending))
        if isinstance(y, PendingProduct):
            # 17 and more rows with K split: the rotation and the cache write add up the partial sums themselves
            if (table is None and slots is None) or tuple(weight.shape) != (N, K):
                return self.materialize(y)
            return self._rope_cache_write_pending(y, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages,
                                                  v_pages)
        if table is not None or slots is not None:
            self.rope_cache_write(y, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages, v_pages)
        return y

    def _rope_cache_write_pending(self, p: PendingProduct, nh: int, nkv: int, d: int,
                                  positions: Optional[torch.Tensor], table: Optional[torch.Tensor], rot_dim: int,
                                  neox: bool, slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                                  v_pages: Optional[torch.Tensor]) -> torch.Tensor:
        M, N = p.shape
        y = torch.empty((M, N), dtype=torch.bfloat16, device=p.device)
        self._dev(positions, table, slots, k_pages, v_pages)
        max_pos = 0
        if table is not None:
            if table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] != rot_dim or not table.is_contiguous():
                raise ValueError("rotary table must be contiguous float32 [max_pos, %d]" % rot_dim)
            if positions is None:
                raise ValueError("rotation needs positions")
            self._i32(positions, "positions", M)
            max_pos = table.shape[0]
        num_pages, ps = 0, 1
        if slots is not None:
            self._i32(slots, "slots", M)
            if k_pages is None or k_pages.dim() != 4 or k_pages.shape[1] != nkv or k_pages.shape[3] != d \
                    or not k_pages.is_contiguous() or k_pages.dtype != torch.bfloat16:
                raise ValueError("k_pages must be contiguous bfloat16 [pages, %d, page_size, %d]" % (nkv, d))
            num_pages, ps = k_pages.shape[0], k_pages.shape[2]
            if v_pages is None or tuple(v_pages.shape) != (num_pages, nkv, d, ps) or not v_pages.is_contiguous() \
                    or v_pages.dtype != torch.bfloat16:
                raise ValueError("v_pages must be contiguous bfloat16 [%d, %d, %d, %d]" % (num_pages, nkv, d, ps))
        self._check(self.lib.lmsf_rope_cache_write_partial(
            _ptr(p.partials), _ptr(p.bias), p.partials.shape[0], _ptr(y), y.stride(0), M, _ptr(positions), _ptr(table),
            rot_dim, 1 if neox else 0, max_pos, _ptr(slots), _ptr(k_pages), _ptr(v_pages), num_pages, nh, nkv, d, ps,
            self._stream()))
        return y

    # ------------------------------------------------------------------ attention

    @staticmethod
    def check_head_dim(d: int) -> None:
        """Raises if no attention kernel takes head size ``d``: the matrix-core kernels take multiples of 16
        up to 256 (bfloat16), the general kernel multiples of 4 up to 256 (either dtype). Parts ask this when
        they are built, before any weight is loaded."""
        if d <= 0 or d % 4 != 0 or d > 256:
            raise ValueError("head size %d is not supported by the attention kernels: they take multiples of 4 "
                             "up to 256 (multiples of 16 on the matrix cores)" % d)

    def paged_attention(self, q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                        block_tables: torch.Tensor, seg: torch.Tensor, pos: torch.Tensor, nh: int, nkv: int, d: int,
                        scale: float, window: int = 0, batch=None, kernel: Optional[str] = None) -> torch.Tensor:
        """Attention of every query token over the cached keys of its request.

        ``q`` is [N, >= nh*d] with unit column stride (it may be the fused QKV buffer, of which the
        first nh*d columns are read). ``k_pages`` [pages, nkv, page_size, d], ``v_pages``
        [pages, nkv, d, page_size]. ``block_tables`` int32 [S, W]; ``seg``, ``pos`` int32 [N].
        ``batch`` (engine.batch.StepContext) carries host-side facts about the step for the choice of
        kernel; without it they are read back from ``seg`` and ``pos``. ``kernel`` forces "generic" or
        "mfma" (tests). Returns [N, nh*d] in q's dtype.
        """
        self._dev(q, k_pages, v_pages, block_tables, seg, pos)
        if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < nh * d:
            raise ValueError("q must be [N, >= %d] with unit column stride" % (nh * d))
        N = q.shape[0]
        if k_pages.dim() != 4 or k_pages.shape[1] != nkv or k_pages.shape[3] != d or not k_pages.is_contiguous() \
                or k_pages.dtype != q.dtype:
            raise ValueError("k_pages must be contiguous [pages, %d, page_size, %d] of %s" % (nkv, d, q.dtype))
        num_pages, ps = k_pages.shape[0], k_pages.shape[2]
        if tuple(v_pages.shape) != (num_pages, nkv, d, ps) or not v_pages.is_contiguous() or v_pages.dtype != q.dtype:
            raise ValueError("v_pages must be contiguous [%d, %d, %d, %d] of %s" % (num_pages, nkv, d, ps, q.dtype))
        if block_tables.dim() != 2:
            raise ValueError("block_tables must be [segments, width]")
        self._i32(block_tables, "block_tables")
        self._i32(seg, "seg", N)
        self._i32(pos, "pos", N)
        out = torch.empty((N, nh * d), dtype=q.dtype, device=q.device)
        if N == 0:
            return out
        fast_ok = (q.dtype == torch.bfloat16 and d % 16 == 0 and 16 <= d <= 256 and ps % 4 == 0
                   and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0 and scale > 0)
        if kernel == "mfma" and not fast_ok:
            raise ValueError("the matrix-core attention kernels need bfloat16, a head size that is a multiple of 16 "
                             "up to 256, a page size that is a multiple of 4, 16-byte aligned query rows and a positive scale")
        if kernel == "generic" or not fast_ok:
            self._check(self.lib.lmsf_paged_attention_generic(
                _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages), num_pages,
                _ptr(block_tables), block_tables.shape[1], _ptr(seg), _ptr(pos), N, nh, nkv, d, ps, float(scale),
                int(window or 0), _code(q.dtype), self._stream()))
            return out
        plan = self._attention_plan(batch, seg, pos, nh, nkv)
        common = (_ptr(k_pages), _ptr(v_pages), num_pages, _ptr(block_tables), block_tables.shape[1])
        if plan.tiles is not None:
            self._check(self.lib.lmsf_paged_attention_prefill_mfma(
                _ptr(q), q.stride(0), _ptr(out), out.stride(0), *common, _ptr(plan.tiles), plan.n_tiles,
                _ptr(seg), _ptr(pos), nh, nkv, d, ps, float(scale), int(window or 0), self.prefill_attention_variant,
                self._stream()))
        if plan.n_single:
            c_chunk, c_splits = ctypes.c_int(0), ctypes.c_int(0)
            self.lib.lmsf_route_decode_attention(ctypes.byref(self._tun), plan.n_single, nh, nkv, plan.max_context,
                                                 ctypes.byref(c_chunk), ctypes.byref(c_splits))
            chunk, n_splits = c_chunk.value, c_splits.value
            floats = self.lib.lmsf_attention_decode_scratch_floats(plan.n_single, nh, d, n_splits)
            scratch = torch.empty(floats if n_splits > 1 else 1, dtype=torch.float32, device=q.device)
            self._check(self.lib.lmsf_paged_attention_decode_mfma(
                _ptr(q), q.stride(0), _ptr(out), out.stride(0), *common, _ptr(plan.single_tokens), plan.n_single,
                None if plan.token_is_request else _ptr(seg), _ptr(pos), nh, nkv, d, ps, float(scale),
                int(window or 0), chunk, n_splits, _ptr(scratch), self.decode_attention_order, self._stream()))
        return out

    def _attention_plan(self, batch, seg: torch.Tensor, pos: torch.Tensor, nh: int, nkv: int) -> "_AttentionPlan":
        """How a step's tokens are split between the two matrix-core kernels: requests with one token go
        to the decode kernel, the others are cut into tiles for the prefill kernel. Computed once per step
        and tile size, and kept on the batch for the other layers."""
        tq = self.lib.lmsf_attention_tile_tokens(nh, nkv)
        if batch is not None:
            aux = batch.aux
            key = ("attention_plan", tq)
            if key in aux:
                return aux[key]
            lens, starts, max_context = batch.host_seg_lens, batch.host_seg_starts, batch.max_context
            first_pos = batch.host_seg_first_pos
            if batch.replayed or batch.all_single:
                # the order matters from 16 tokens on (the kernel starts the longest contexts first); below that
                # the tokens are taken as they come, which saves the kernel the trip to the list
                order = getattr(batch, "longest_first", None) if batch.n_tokens >= 16 else None
                plan = _AttentionPlan(None, 0, order, batch.n_tokens, max_context, token_is_request=True)
                aux[key] = plan
                return plan
        else:
            seg_h = seg.tolist()
            lens, starts = [], []
            for i, sg in enumerate(seg_h):
                if i == 0 or sg != seg_h[i - 1]:
                    starts.append(i)
                    lens.append(0)
                lens[-1] += 1
            pos_h = pos.tolist()
            max_context = max(pos_h) + 1
            first_pos = [pos_h[st] for st in starts]
            aux, key = None, None
        by_keys, single = [], []
        for st, n, p0 in zip(starts, lens, first_pos):
            if n == 1:
                single.append((p0, st))
            else:
                for t in range(0, n, tq):
                    by_keys.append((p0 + t + min(tq, n - t), st + t, min(tq, n - t)))
        # the tiles with the most keys first: the prefill kernel starts its workgroups in this order
        by_keys.sort(key=lambda e: -e[0])
        tiles = [x for e in by_keys for x in e[1:]]
        # likewise the single tokens with the longest contexts first
        single = [st for _, st in sorted(single, key=lambda e: -e[0])]
        dev = seg.device
        if len(single) == len(lens):
            plan = _AttentionPlan(None, 0, None, len(single), max_context)
        else:
            both = self.upload_ints(tiles + single, dev)
            plan = _AttentionPlan(both[:len(tiles)], len(tiles) // 2,
                                  both[len(tiles):] if single else None, len(single), max_context)
        if aux is not None:
            aux[key] = plan
        return plan

    def upload_ints(self, values, dev: torch.device) -> torch.Tensor:
        """int32 values to the device through pinned memory, without waiting for the copy. Four buffers take
        turns; before a buffer is written again its last copy's event is waited for (long past, as a rule)."""
        n = len(values)
        turn = self._pinned_turn = (getattr(self, "_pinned_turn", -1) + 1) % 4
        bufs = self.__dict__.setdefault("_pinned_ints", [None] * 4)
        events = self.__dict__.setdefault("_pinned_events", [None] * 4)
        if events[turn] is not None:
            events[turn].synchronize()
        if bufs[turn] is None or bufs[turn].numel() < n:
            bufs[turn] = torch.empty(max(n, 4096), dtype=torch.int32, pin_memory=True)
        host = bufs[turn][:n]
        host.numpy()[:] = values
        out = host.to(dev, non_blocking=True)
        if events[turn] is None:
            events[turn] = torch.cuda.Event()
        events[turn].record()
        return out

    # ------------------------------------------------------------------ feed-forward

    def gated_act(self, gu: torch.Tensor, kind: str = "silu") -> torch.Tensor:
        """act(gu[:, :I]) * gu[:, I:] for gu [N, 2I]; kind "silu" or "gelu"."""
        self._dev(gu)
        if gu.dim() != 2 or gu.stride(1) != 1 or gu.shape[1] % 2 != 0:
            raise ValueError("gated_act input must be [N, 2I] with unit column stride")
        kinds = {"silu": 0, "gelu": 1}
        if kind not in kinds:
            raise ValueError("unknown activation %r (known: %s)" % (kind, ", ".join(kinds)))
        N, I = gu.shape[0], gu.shape[1] // 2
        out = torch.empty((N, I), dtype=gu.dtype, device=gu.device)
        self._check(self.lib.lmsf_gated_act(_ptr(gu), _ptr(out), _code(gu.dtype), N, I, gu.stride(0), kinds[kind],
                                            self._stream()))
        return out

    # ------------------------------------------------------------------ matrix products

    def weight_row_pad(self, in_features: int, dtype: torch.dtype) -> int:
        """Elements to leave between the end of one row of a linear layer's weight and the start of the next.
        With rows of 8 KB (or any multiple of 4 KB) lying back to back, the rows that a workgroup reads side by
        side begin on the same memory channels: a kernel that only reads a 28,672 x 4,096 matrix 64 rows at a
        time, 128 bytes of each, gets 4.8 TB/s, and 5.6 to 5.75 with 128 to 2,048 bytes between the rows; 16 rows
        at a time, 1 KB of each: 5.0 and 5.9 to 6.0. Which distances help depends on the row's length (rows of
        16 KB: 128 bytes hurt, 256 and more help; rows of 28 KB: 256 hurts); 512 bytes help or do no harm at 4,096,
        8,192, 14,336 and 28,672 columns, for the few-rows, the many-rows and the library's products alike (gate_up
        of 57,344 x 8,192 at 64 rows: 207 -> 181 us). Every product takes the distance between rows as an
        argument."""
        return self.weight_row_pad_bytes // torch.empty((), dtype=dtype).element_size()

    def linear(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
               out_dtype: Optional[torch.dtype] = None, pending_ok: bool = False,
               out: Optional[torch.Tensor] = None):
        """y = x weight^T (+ bias); x [M, K], weight [N, K]; y [M, N] in ``out_dtype`` (default x's).
        With ``pending_ok`` the caller takes a ``PendingProduct`` as well, which comes back where the
        product splits K over workgroups, or a ``DeferredLinear`` (few rows). ``out``: a contiguous [M, N]
        tensor of ``out_dtype`` that takes the result instead of a new one (not together with ``pending_ok``).

        Which kernel runs is decided by ``lmsf_route_linear`` (csrc/dispatch.hip), as for the step program:
        float32 operands always run the float32 multiply-add kernel; bfloat16 products with bfloat16 output
        and many rows go to the BLAS library, as the reference's do (core/src/model_executor/layers/linear.rs:44-106
        calls cuBLASLt), through csrc/blas.hip; the rest run in this package's kernels.
        """
        self._dev(x, weight, bias)
        if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
            raise ValueError("linear: x %s and weight %s do not match" % (tuple(x.shape), tuple(weight.shape)))
        if x.stride(1) != 1 or weight.stride(1) != 1:
            raise ValueError("linear: operands need unit column stride")
        M, K = x.shape
        N = weight.shape[0]
        if bias is not None and (bias.shape != (N,) or bias.dtype != weight.dtype or not bias.is_contiguous()):
            raise ValueError("linear: bias must be [%d] of the weight's dtype" % N)
        out_dtype = out_dtype or x.dtype
        if out is not None:
            if pending_ok or tuple(out.shape) != (M, N) or out.dtype != out_dtype or not out.is_contiguous() \
                    or out.device != x.device:
                raise ValueError("linear: out must be a contiguous [%d, %d] %s tensor on x's device" % (M, N, out_dtype))
        rt = D.Route()
        self.lib.lmsf_route_linear(ctypes.byref(self._tun), ctypes.byref(self._shape(x, weight, out_dtype)),
                                   1 if pending_ok else 0, ctypes.byref(rt))
        if rt.route == D.MID:
            return self._linear_mid(x, weight, bias, 0, out_dtype, rt, out=out)
        if rt.route == D.LARGE:
            return self._linear_large(x, weight, bias, 0, bool(rt.pending), out=out, plan=rt.plan)
        if rt.route == D.DEFERRED:
            return DeferredLinear(x, weight, bias, out_dtype)
        y = out if out is not None else torch.empty((M, N), dtype=out_dtype, device=x.device)
        if rt.route == D.GEMV:
            self._check(self.lib.lmsf_gemv(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(y),
                                           _code(out_dtype), y.stride(0), M, N, K, 0, self._stream()))
        elif rt.route == D.CHUNKS:
            for r0 in range(0, M, rt.chunk_rows):
                rows = min(rt.chunk_rows, M - r0)
                self.linear(x[r0:r0 + rows], weight, bias, out_dtype=out_dtype, out=y[r0:r0 + rows])
        elif rt.route == D.SKINNY:
            for r0 in range(0, M, 64):
                rows = min(64, M - r0)
                xs, ys = x[r0:r0 + rows], y[r0:r0 + rows]
                self._check(self.lib.lmsf_gemm_skinny(
                    _ptr(xs), xs.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(ys),
                    _code(out_dtype), ys.stride(0), rows, N, K, self.skinny_variant, 0, self._stream()))
        elif rt.route == D.BLAS:
            self._check(self.lib.lmsf_blas_linear(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias),
                                                  _ptr(y), y.stride(0), M, N, K, self._stream()))
        else:
            self._check(self.lib.lmsf_gemm_plain(_ptr(x), _code(x.dtype), x.stride(0), _ptr(weight),
                                                 _code(weight.dtype), weight.stride(0), _ptr(bias), _ptr(y),
                                                 _code(out_dtype), y.stride(0), M, N, K, self._stream()))
        return y

    def linear_gated(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                     kind: str = "silu") -> torch.Tensor:
        """act(x Wg^T + bg) * (x Wu^T + bu) for the fused weight [2 I, K] = [Wg; Wu] (bias [2 I] likewise);
        [M, I] in x's dtype. Where ``lmsf_route_linear_gated`` says so the activation is the epilogue of the
        product; otherwise the product and the activation kernel run one after the other. Both ways round
        the two products to the storage type before the activation, so they give the same bits wherever
        they add up K in the same order (the default tilings of the fused and the plain product do not: they
        split K over 8 and over 16 waves). ``x`` may be a ``ScaledRows``."""
        if weight.dim() != 2 or weight.shape[0] % 2 != 0:
            raise ValueError("linear_gated: weight must be [2 I, K]")
        kinds = {"silu": 1, "gelu": 2}
        if kind not in kinds:
            raise ValueError("unknown activation %r (known: %s)" % (kind, ", ".join(kinds)))
        M, I = x.shape[0], weight.shape[0] // 2
        scaled = isinstance(x, ScaledRows)
        xt = x.xw if scaled else x
        if xt.dim() != 2 or xt.shape[1] != weight.shape[1] or xt.stride(1) != 1 or weight.stride(1) != 1:
            raise ValueError("linear_gated: x %s and weight %s do not match" % (tuple(xt.shape), tuple(weight.shape)))
        K = xt.shape[1]
        rt = D.Route()
        self.lib.lmsf_route_linear_gated(ctypes.byref(self._tun), ctypes.byref(self._shape(xt, weight, xt.dtype)),
                                         x.rows_per_tile if scaled else 0, x.tiles if scaled else 0, ctypes.byref(rt))
        if rt.route == D.MATERIALIZE:
            return self.linear_gated(self.materialize(x), weight, bias, kind)
        if rt.route == D.SEPARATE:
            return self.gated_act(self.linear(x, weight, bias), kind)
        self._dev(xt, weight, bias)
        if bias is not None and (bias.shape != (2 * I,) or bias.dtype != weight.dtype or not bias.is_contiguous()):
            raise ValueError("linear_gated: bias must be [%d] of the weight's dtype" % (2 * I))
        if rt.route == D.MID:
            return self._linear_mid(x, weight, bias, kinds[kind], torch.bfloat16, rt)
        if rt.route == D.LARGE:
            return self._linear_large(x, weight, bias, kinds[kind], plan=rt.plan)
        y = torch.empty((M, I), dtype=torch.bfloat16, device=x.device)
        head = (_ptr(xt), xt.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(y))
        if rt.route == D.MID_SCALED:
            self._check(self.lib.lmsf_gemm_mid_scaled(*head, y.stride(0), M, I, K, kinds[kind], _ptr(x.sumsq), x.tiles,
                                                      x.eps, self._stream()))
        elif rt.route == D.GEMV_SCALED:
            self._check(self.lib.lmsf_gemv_scaled(*head, y.stride(0), M, I, K, kinds[kind], _ptr(x.sumsq), x.tiles,
                                                  x.eps, self._stream()))
        elif rt.route == D.SKINNY_SCALED:
            self._check(self.lib.lmsf_gemm_skinny_scaled(*head, y.stride(0), M, I, K, kinds[kind], _ptr(x.sumsq),
                                                         x.tiles, x.eps, self.skinny_variant, self._stream()))
        elif rt.route == D.GEMV:
            self._check(self.lib.lmsf_gemv(*head, BF16, y.stride(0), M, I, K, kinds[kind], self._stream()))
        else:
            self._check(self.lib.lmsf_gemm_skinny(*head, BF16, y.stride(0), M, I, K, self.skinny_variant, kinds[kind],
                                                  self._stream()))
        return y

    def _linear_mid(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], act: int,
                    out_dtype: torch.dtype, rt: D.Route, out: Optional[torch.Tensor] = None):
        """The 17-and-more-rows product (csrc/gemm_mid.hip) as ``rt`` says."""
        self._dev(x, weight, bias)
        M, K = x.shape
        N = weight.shape[0] // 2 if act else weight.shape[0]
        if bias is not None and (bias.shape != (weight.shape[0],) or bias.dtype != weight.dtype
                                 or not bias.is_contiguous()):
            raise ValueError("linear: bias must be [%d] of the weight's dtype" % weight.shape[0])
        splits = rt.splits
        if rt.pending:
            partials = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
            self._check(self.lib.lmsf_gemm_mid_partial(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), M, N, K,
                                                       splits, _ptr(partials), self._stream()))
            return PendingProduct(partials, bias, out_dtype)
        floats = self.lib.lmsf_gemm_mid_scratch_floats(M, N, splits, act)
        scratch = torch.empty(floats, dtype=torch.float32, device=x.device) if floats else None
        y = out if out is not None else torch.empty((M, N), dtype=out_dtype, device=x.device)
        self._check(self.lib.lmsf_gemm_mid(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(y),
                                           _code(out_dtype), y.stride(0), M, N, K, act, splits, _ptr(scratch),
                                           self._stream()))
        return y

    def _linear_large(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], act: int,
                      pending_ok: bool = False, out: Optional[torch.Tensor] = None, plan: Optional[int] = None):
        """The many-rows product (csrc/gemm_large.hip); K a multiple of 64, W's rows of 8, row strides of 8,
        16-byte aligned bases. ``plan``: tiling and split (``lmsf_gemm_large_plan`` proposes one)."""
        self._dev(x, weight, bias)
        M, K = x.shape
        N = weight.shape[0] // 2 if act else weight.shape[0]
        if bias is not None and (bias.shape != (weight.shape[0],) or bias.dtype != weight.dtype
                                 or not bias.is_contiguous()):
            raise ValueError("linear: bias must be [%d] of the weight's dtype" % weight.shape[0])
        if plan is None:
            plan = self.lib.lmsf_gemm_large_plan(M, N, K, act)
        splits = plan % 16
        scratch = None
        if splits > 1:
            scratch = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
            if pending_ok:
                self._check(self.lib.lmsf_gemm_large(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), None, None, 0,
                                                     M, N, K, 0, plan, _ptr(scratch), 0, self._stream()))
                return PendingProduct(scratch, bias, torch.bfloat16)
        y = out if out is not None else torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
        self._check(self.lib.lmsf_gemm_large(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(y),
                                             y.stride(0), M, N, K, act, plan, _ptr(scratch), 1, self._stream()))
        return y

    def tune_products(self, x: torch.Tensor, weights, bias: Optional[torch.Tensor] = None, candidates: int = 16,
                      reps: int = 5):
        """Lets the BLAS library's candidates for the product of ``x`` [M, K] with matrices like ``weights`` (a list of
        [N, K] tensors of one shape and row distance: the same product of several layers, so that no run finds its
        weights in cache) race, and keeps the fastest for later products of that shape
        (tops/src/cublas.rs:121-223 profiles cuBLASLt's tactics likewise). Returns (first choice's us, fastest's us)."""
        w0 = weights[0]
        self._dev(x, bias, *weights)
        if any(w.shape != w0.shape or w.stride(0) != w0.stride(0) or w.dtype != torch.bfloat16 or w.stride(1) != 1
               for w in weights) or x.dtype != torch.bfloat16 or x.shape[1] != w0.shape[1] or x.stride(1) != 1:
            raise ValueError("tune_products: bfloat16 operands of one shape are needed")
        M, K = x.shape
        N = w0.shape[0]
        y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
        ptrs = (ctypes.c_void_p * len(weights))(*[w.data_ptr() for w in weights])
        times = (ctypes.c_float * 2)()
        self._check(self.lib.lmsf_blas_tune(_ptr(x), x.stride(0), ptrs, len(weights), w0.stride(0), _ptr(bias), _ptr(y),
                                            y.stride(0), M, N, K, int(candidates), int(reps), times, self._stream()))
        return float(times[0]), float(times[1])

    # ------------------------------------------------------------------ sampling

    def sample(self, logits: torch.Tensor, temperature: Optional[torch.Tensor] = None,
               top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
               min_p: Optional[torch.Tensor] = None, seeds: Optional[torch.Tensor] = None,
               draws: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One token per row of float32 ``logits`` [R, V]; int32 [R]. All parameters are per-row device
        tensors: temperature/top_p/min_p float32, top_k int32, seeds int64, draws int32."""
        self._dev(logits, temperature, top_k, top_p, min_p, seeds, draws)
        if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
            raise ValueError("sample: logits must be float32 [R, V] with unit column stride")
        R, V = logits.shape
        for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                            ("top_p", top_p, torch.float32), ("min_p", min_p, torch.float32),
                            ("seeds", seeds, torch.int64), ("draws", draws, torch.int32)):
            if t is not None and (t.dtype != dt or t.numel() != R or not t.is_contiguous()):
                raise ValueError("sample: %s must be a contiguous %s tensor of %d elements" % (name, dt, R))
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
        scratch = None
        if temperature is None or (top_k is None and top_p is None and min_p is None):
            elems = self.lib.lmsf_sample_scratch_elems(R, V)
            if elems:
                scratch = torch.empty(2 * elems, dtype=torch.float32, device=logits.device)
        self._check(self.lib.lmsf_sample(_ptr(logits), logits.stride(0), R, V, _ptr(temperature), _ptr(top_k),
                                         _ptr(top_p), _ptr(min_p), _ptr(seeds), _ptr(draws), _ptr(out),
                                         _ptr(scratch), self._stream()))
        return out

    def apply_penalties(self, logits: torch.Tensor, tokens: torch.Tensor, offsets: torch.Tensor,
                        prompt_lens: torch.Tensor, presence: torch.Tensor, frequency: torch.Tensor,
                        repetition: torch.Tensor) -> None:
        """Presence, frequency and repetition penalties on float32 ``logits`` [R, V], in place.
        ``tokens`` int32: each row's prompt then output tokens, concatenated; ``offsets`` int32 [R+1];
        ``prompt_lens`` int32 [R]; the penalties float32 [R]."""
        self._dev(logits, tokens, offsets, prompt_lens, presence, frequency, repetition)
        if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
            raise ValueError("apply_penalties: logits must be float32 [R, V] with unit column stride")
        R, V = logits.shape
        self._i32(tokens, "tokens")
        self._i32(offsets, "offsets", R + 1)
        self._i32(prompt_lens, "prompt_lens", R)
        for name, t in (("presence", presence), ("frequency", frequency), ("repetition", repetition)):
            if t.dtype != torch.float32 or t.numel() != R or not t.is_contiguous():
                raise ValueError("apply_penalties: %s must be contiguous float32 [%d]" % (name, R))
        counts = torch.zeros((R, V), dtype=torch.int32, device=logits.device)
        self._check(self.lib.lmsf_apply_penalties(_ptr(logits), logits.stride(0), R, V, _ptr(tokens), _ptr(offsets),
                                                  _ptr(prompt_lens), _ptr(counts), _ptr(presence), _ptr(frequency),
                                                  _ptr(repetition), self._stream()))


    # ------------------------------------------------------------------ what the machine gives

    def measure(self, nbytes: int = 4 << 30, reps: int = 5) -> dict:
        """Measured rates of this GPU: reading and copying ``nbytes`` of device memory with plain kernels (GB/s,
        a copy counted as bytes read plus bytes written) and the bfloat16 matrix-core instruction in a loop
        without memory traffic (TFLOP/s). The best of ``reps`` runs each, timed with events."""
        dev = torch.device("cuda", _current_device())
        src = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        src.random_(0, 255)
        dst = torch.empty_like(src)
        sink = torch.zeros(64, dtype=torch.float32, device=dev)

        def timed(launch):
            best = None
            for _ in range(reps + 1):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                launch()
                b.record()
                b.synchronize()
                ms = a.elapsed_time(b)
                best = ms if best is None else min(best, ms)
            return best * 1e-3

        t_read = timed(lambda: self._check(self.lib.lmsf_measure_read(_ptr(src), nbytes, _ptr(sink), self._stream())))
        t_copy = timed(lambda: self._check(self.lib.lmsf_measure_copy(_ptr(src), _ptr(dst), nbytes, self._stream())))
        flops = [0.0]

        def mfma():
            flops[0] = self.lib.lmsf_measure_mfma(_ptr(sink), 4096, 256 * 8, self._stream())
            if flops[0] == 0.0:
                self._check(1)
        t_mfma = timed(mfma)
        return {"read_GBps": nbytes / t_read / 1e9, "copy_GBps": 2 * nbytes / t_copy / 1e9,
                "mfma_bf16_TFLOPs": flops[0] / t_mfma / 1e12}


class _AttentionPlan:
    __slots__ = ("tiles", "n_tiles", "single_tokens", "n_single", "max_context", "token_is_request")

    def __init__(self, tiles, n_tiles, single_tokens, n_single, max_context, token_is_request=False):
        self.tiles = tiles                    # int32 [n_tiles, 2] on the device, or None
        self.n_tiles = n_tiles
        self.single_tokens = single_tokens    # int32 flat indices of the one-token requests; None: every token
        self.n_single = n_single
        self.max_context = max_context
        self.token_is_request = token_is_request   # a step of single tokens: token i is request i of the tables


_default_ops: Optional[HipOps] = None


def get_ops() -> HipOps:
    """The process-wide kernel object; raises if the GPU or the library is missing."""
    global _default_ops
    if _default_ops is None:
        _default_ops = HipOps()
    return _default_ops
