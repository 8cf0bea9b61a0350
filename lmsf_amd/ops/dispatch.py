"""ctypes mirrors of csrc/dispatch.h: the kernels' switch points and the routes they lead to.

Which kernel runs a product is decided in C++ (``lmsf_route_*``), for the step program and for
``HipOps`` alike; this module only carries the questions and the answers.
"""
from ctypes import Structure, c_int, c_long

TUNABLE_NAMES = (
    "fuse_norm_rows", "fuse_stream_rows", "gemv_max_rows", "skinny_variant", "mid_wide_max_cols", "mid_max_rows",
    "skinny_max_rows", "prefill_attention_variant", "decode_attention_order", "decode_attention_splits",
    "use_library_gemm", "large_max_rows", "large_deep_min_rows", "mid_scaled_rows", "large_deep_max_rows",
    "qkv_fused_max_rows")


class Tunables(Structure):
    _fields_ = [(n, c_int) for n in TUNABLE_NAMES]

    def as_tuple(self):
        return tuple(int(getattr(self, n)) for n in TUNABLE_NAMES)


class Route(Structure):
    _fields_ = [(n, c_int) for n in ("route", "splits", "plan", "pending", "chunk_rows")]


class ProductShape(Structure):
    _fields_ = ([(n, c_int) for n in ("M", "N", "K", "x_dtype", "w_dtype", "out_dtype")]
                + [("ldx", c_long), ("ldw", c_long), ("x_ok16", c_int), ("w_ok16", c_int)])


(PLAIN, MID, LARGE, DEFERRED, GEMV, CHUNKS, SKINNY, BLAS, MATERIALIZE, MID_SCALED, GEMV_SCALED, SKINNY_SCALED, SEPARATE,
 GEMV_ADD_NORM, SKINNY_ADD_NORM, GEMV_ADD) = range(16)
