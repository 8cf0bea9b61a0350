"""The one table of switch points between the kernels (csrc/dispatch.hip), asked as the step program and the
Python face of the kernels ask it: which kernel a product of Llama-3-8B's shapes runs in at which number of rows,
what the forms around a norm take, and how decode attention splits its keys. Host code only: no GPU needed."""
import ctypes

import pytest

from lmsf_amd.ops import dispatch as D
from lmsf_amd.ops import library

F32, BF16 = 0, 1
H, I, QKV, V = 4096, 14336, 6144, 128256


@pytest.fixture(scope="module")
def lib():
    return library.load_library()


def defaults():
    """The switch points as ``HipOps`` sets them."""
    return D.Tunables(fuse_norm_rows=16, fuse_stream_rows=1, gemv_max_rows=2, skinny_variant=0, mid_wide_max_cols=8192,
                      mid_max_rows=128, skinny_max_rows=16, prefill_attention_variant=0, decode_attention_order=0,
                      decode_attention_splits=0, use_library_gemm=1, large_max_rows=256, large_deep_min_rows=64,
                      mid_scaled_rows=16, large_deep_max_rows=1024, qkv_fused_max_rows=32)


def shape(M, N, K, x=BF16, w=BF16, out=BF16, ld_pad=256, ok16=1):
    return D.ProductShape(M, N, K, x, w, out, K, K + ld_pad, ok16, ok16)


def linear(lib, t, M, N, K, pending_ok=False, **kw):
    r = D.Route()
    lib.lmsf_route_linear(ctypes.byref(t), ctypes.byref(shape(M, N, K, **kw)), 1 if pending_ok else 0, ctypes.byref(r))
    return r


def test_plain_products_change_kernels_with_the_number_of_rows(lib):
    t = defaults()
    o = lambda M, **kw: linear(lib, t, M, H, H, **kw).route          # noqa: E731
    assert [o(M) for M in (1, 2, 16, 17, 64, 128, 129, 256, 257, 4096)] == \
        [D.GEMV, D.SKINNY, D.SKINNY, D.MID, D.MID, D.MID, D.LARGE, D.LARGE, D.BLAS, D.BLAS]
    # a product whose K is at least three times N (down) leaves the 17-and-more-rows kernel at 65 rows and stays
    # with the many-rows kernel up to 1,024
    down = lambda M: linear(lib, t, M, H, I).route                   # noqa: E731
    assert [down(M) for M in (64, 65, 128, 512, 1024, 1025)] == [D.MID, D.LARGE, D.LARGE, D.LARGE, D.LARGE, D.BLAS]
    # beyond 64 rows the wide products (gate_up's 28,672 columns) are the library's
    assert linear(lib, t, 64, 2 * I, H).route == D.MID and linear(lib, t, 65, 2 * I, H).route == D.BLAS
    assert linear(lib, t, 100, 2 * I, H).route == D.BLAS and linear(lib, t, 100, 8192, H).route == D.MID
    # float32 operands, a K that is no multiple of 8, or no library: the float32 multiply-add kernel
    assert linear(lib, t, 8, H, H, x=F32, w=F32, out=F32).route == D.PLAIN
    assert linear(lib, t, 300, H, 4100).route == D.BLAS and linear(lib, t, 8, H, 4100).route == D.PLAIN
    t.use_library_gemm = 0
    assert linear(lib, t, 300, H, H).route == D.PLAIN and linear(lib, t, 300, H, I).route == D.LARGE


def test_logits_in_float32_for_any_number_of_rows(lib):
    t = defaults()
    head = lambda M: linear(lib, t, M, V, H, out=F32)                # noqa: E731
    # (one row of this matrix stays with the few-rows kernel: it is large enough to stream at the same rate there)
    assert head(1).route == D.SKINNY and linear(lib, t, 1, H, H, out=F32).route == D.GEMV
    assert head(8).route == D.SKINNY and head(64).route == D.MID
    r = head(300)
    assert r.route == D.CHUNKS and r.chunk_rows == 128


def test_unfinished_forms_only_where_the_caller_takes_them(lib):
    t = defaults()
    assert linear(lib, t, 8, H, H, pending_ok=True).route == D.DEFERRED       # the norm that follows runs it
    assert linear(lib, t, 8, H, H).route == D.SKINNY
    r = linear(lib, t, 40, H, H, pending_ok=True)
    assert r.route == D.MID and r.splits > 1 and r.pending == 1               # partial sums for the norm to add up
    r = linear(lib, t, 40, H, H)
    assert r.route == D.MID and r.splits > 1 and r.pending == 0               # the product's own reduction kernel
    r = linear(lib, t, 200, H, I, pending_ok=True)
    assert r.route == D.LARGE and r.splits == r.plan % 16 and r.pending == (1 if r.splits > 1 else 0)
    t.fuse_norm_rows = 0
    t.fuse_stream_rows = 0
    assert linear(lib, t, 8, H, H, pending_ok=True).route == D.SKINNY


def test_gated_and_qkv_products(lib):
    t = defaults()

    def gated(M, scaled=0, tiles=0):
        r = D.Route()
        lib.lmsf_route_linear_gated(ctypes.byref(t), ctypes.byref(shape(M, 2 * I, H)), scaled, tiles, ctypes.byref(r))
        return r.route

    assert [gated(M) for M in (1, 2, 3, 16, 17, 64, 65, 256, 257)] == \
        [D.GEMV, D.GEMV, D.SKINNY, D.SKINNY, D.MID, D.MID, D.LARGE, D.LARGE, D.SEPARATE]
    assert gated(1, scaled=1, tiles=8) == D.GEMV_SCALED                       # rows whose norm factor is still to come
    assert gated(8, scaled=16, tiles=H // 16) in (D.SKINNY_SCALED, D.MID_SCALED)

    def qkv(M, fused=1, scaled=0):
        r = D.Route()
        lib.lmsf_route_qkv(ctypes.byref(t), ctypes.byref(shape(M, QKV, H)), fused, scaled, ctypes.byref(r))
        return r

    # (with its rotation and cache write as epilogue the few-rows kernel keeps the QKV product up to 32 rows)
    assert [qkv(M).route for M in (1, 2, 3, 16, 17, 32, 33, 2048)] == [D.GEMV, D.GEMV, D.SKINNY, D.SKINNY, D.SKINNY,
                                                                     D.SKINNY, D.SEPARATE, D.SEPARATE]
    assert qkv(33).pending == 1 and qkv(8, fused=0).route == D.SEPARATE and qkv(8, fused=0).pending == 0
    assert qkv(17, fused=0).route == D.SEPARATE and qkv(17, fused=0).pending == 1
    assert qkv(8, scaled=16).route == D.SKINNY_SCALED and qkv(2, scaled=2).route == D.GEMV_SCALED
    assert qkv(8, fused=0, scaled=16).route == D.MATERIALIZE


def test_a_norm_that_finds_its_branch_unstarted(lib):
    t = defaults()

    def norm(M, fits=1, prepares=1):
        r = D.Route()
        lib.lmsf_route_deferred_norm(ctypes.byref(t), M, H, H, fits, prepares, ctypes.byref(r))
        return r.route

    assert [norm(M) for M in (1, 2, 8, 16)] == [D.GEMV_ADD_NORM, D.SKINNY_ADD_NORM, D.SKINNY_ADD_NORM, D.SKINNY_ADD_NORM]
    assert norm(1, prepares=0) == D.GEMV_ADD and norm(8, prepares=0) == D.MATERIALIZE
    assert norm(1, fits=0, prepares=0) == D.MATERIALIZE               # rows are selected: the product runs first


def test_decode_attention_splits(lib):
    t = defaults()

    def split(n, ctx, nh=32, nkv=8):
        c, s = ctypes.c_int(), ctypes.c_int()
        lib.lmsf_route_decode_attention(ctypes.byref(t), n, nh, nkv, ctx, ctypes.byref(c), ctypes.byref(s))
        assert c.value % 128 == 0 and c.value * s.value >= ctx > c.value * (s.value - 1)
        return s.value

    assert split(64, 585) == 1                       # 512 workgroups without a split
    assert split(8, 585) == 5 and split(1, 585) == 5    # one step of 128 keys a workgroup
    assert split(1, 8000) == 63 and split(8, 8000) == 8
    assert split(8, 100000) > split(8, 30000)         # long contexts: more workgroups than the chip holds at once
    t.decode_attention_splits = 2
    assert split(8, 8000) == 2
