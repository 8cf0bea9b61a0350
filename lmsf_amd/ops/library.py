"""Loads the HIP kernel library and declares its entry points.

There is no fallback: if the library cannot be built or loaded, or reports another ABI
version, importing the kernels fails with the reason.
"""
import ctypes
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_long, c_void_p
from typing import Optional

from ..csrc import build as _build
from .dispatch import ProductShape, Route, Tunables

ABI_VERSION = 23

_lib: Optional[ctypes.CDLL] = None
_lib_path: Optional[str] = None


class KernelLibraryError(RuntimeError):
    pass


_P = c_void_p
_SIGNATURES = {
    "lmsf_last_error": (c_char_p, []),
    "lmsf_abi_version": (c_int, []),
    "lmsf_device_arch": (c_int, [c_char_p, c_int]),
    "lmsf_embedding": (c_int, [_P, _P, c_int, _P, c_int, c_int, c_int, c_float, _P, _P]),
    "lmsf_patch_tokens": (c_int, [_P, _P, _P, c_int, c_int, _P]),
    "lmsf_add_rms_norm": (c_int, [_P, c_int, _P, _P, c_int, _P, c_int, _P, c_int, c_int, c_float, c_float, _P]),
    "lmsf_rope_cache_write": (c_int, [_P, _P, _P, c_int, c_int, c_long, _P, _P, c_int, c_int, c_int, _P, _P, _P,
                                      c_long, c_int, c_int, c_int, c_int, _P]),
    "lmsf_paged_attention_generic": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, _P, c_int, _P, _P, c_int,
                                             c_int, c_int, c_int, c_int, c_float, c_int, c_int, _P]),
    "lmsf_attention_tile_tokens": (c_int, [c_int, c_int]),
    "lmsf_paged_attention_prefill_mfma": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, _P, c_int, _P, c_int, _P, _P,
                                                  c_int, c_int, c_int, c_int, c_float, c_int, c_int, _P]),
    "lmsf_attention_decode_scratch_floats": (c_long, [c_int, c_int, c_int, c_int]),
    "lmsf_paged_attention_decode_mfma": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, _P, c_int, _P, c_int, _P, _P,
                                                 c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, _P, c_int,
                                                 _P]),
    "lmsf_gated_act": (c_int, [_P, _P, c_int, c_int, c_int, c_long, c_int, _P]),
    "lmsf_gemm_plain": (c_int, [_P, c_int, c_long, _P, c_int, c_long, _P, _P, c_int, c_long, c_int, c_int, c_int, _P]),
    "lmsf_gemm_skinny": (c_int, [_P, c_long, _P, c_long, _P, _P, c_int, c_long, c_int, c_int, c_int, c_int, c_int, _P]),
    "lmsf_gemm_qkv_rope_cache": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, c_int, c_int, _P, _P, c_int, _P, _P, _P,
                                         c_long, c_int, c_int, c_int, c_int, c_int, _P]),
    "lmsf_gemm_skinny_add_norm": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, _P, c_float, _P, c_long, _P, c_int,
                                          c_int, c_int, c_int, _P]),
    "lmsf_gemm_skinny_scaled": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, c_int, c_int, c_int, c_int, _P, c_int,
                                        c_float, c_int, _P]),
    "lmsf_gemm_qkv_rope_cache_scaled": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, c_int, c_int, _P, _P, c_int, _P,
                                                _P, _P, c_long, c_int, c_int, c_int, c_int, _P, c_int, c_float, _P]),
    "lmsf_gemv": (c_int, [_P, c_long, _P, c_long, _P, _P, c_int, c_long, c_int, c_int, c_int, c_int, _P]),
    "lmsf_gemv_qkv_rope_cache": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, c_int, c_int, _P, _P, c_int, _P, _P, _P,
                                         c_long, c_int, c_int, c_int, c_int, _P]),
    "lmsf_gemv_add": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, c_int, c_int, c_int, _P]),
    "lmsf_gemv_partials": (c_int, [c_int]),
    "lmsf_gemv_add_norm": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, _P, c_float, _P, c_long, _P, c_int, c_int,
                                   c_int, _P]),
    "lmsf_gemv_scaled": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, c_int, c_int, c_int, c_int, _P, c_int, c_float,
                                 _P]),
    "lmsf_gemv_scaled_qkv_rope_cache": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, c_int, c_int, _P, _P, c_int, _P,
                                                _P, _P, c_long, c_int, c_int, c_int, c_int, _P, c_int, c_float, _P]),
    "lmsf_gemm_mid_splits": (c_int, [c_int, c_int, c_int, c_int]),
    "lmsf_gemm_mid_scratch_floats": (c_long, [c_int, c_int, c_int, c_int]),
    "lmsf_gemm_mid": (c_int, [_P, c_long, _P, c_long, _P, _P, c_int, c_long, c_int, c_int, c_int, c_int, c_int, _P, _P]),
    "lmsf_gemm_mid_scaled_fits": (c_int, [c_int, c_int, c_int, c_int]),
    "lmsf_gemm_mid_scaled": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, c_int, c_int, c_int, c_int, _P, c_int, c_float, _P]),
    "lmsf_gemm_mid_partial": (c_int, [_P, c_long, _P, c_long, c_int, c_int, c_int, c_int, _P, _P]),
    "lmsf_gemm_mid_reduce": (c_int, [_P, _P, _P, c_int, c_long, c_int, c_int, c_int, _P]),
    "lmsf_gemm_large_plan": (c_int, [c_int, c_int, c_int, c_int]),
    "lmsf_gemm_large_scratch_floats": (c_long, [c_int, c_int, c_int]),
    "lmsf_gemm_large": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, c_int, c_int, c_int, c_int, c_int, _P, c_int, _P]),
    "lmsf_add_rms_norm_partial": (c_int, [_P, _P, c_int, c_int, _P, _P, c_int, _P, c_int, _P, c_int, c_int, c_float,
                                          c_float, _P]),
    "lmsf_rope_cache_write_partial": (c_int, [_P, _P, c_int, _P, c_long, c_int, _P, _P, c_int, c_int, c_int, _P, _P, _P,
                                              c_long, c_int, c_int, c_int, c_int, _P]),
    "lmsf_sample": (c_int, [_P, c_long, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P, _P]),
    "lmsf_sample_scratch_elems": (c_long, [c_int, c_int]),
    "lmsf_greedy_tokens_static": (c_int, [_P, c_long, c_int, c_int, _P, _P]),
    "lmsf_measure_read": (c_int, [_P, c_long, _P, _P]),
    "lmsf_measure_copy": (c_int, [_P, _P, c_long, _P]),
    "lmsf_measure_mfma": (c_double, [_P, c_int, c_int, _P]),
    "lmsf_apply_penalties": (c_int, [_P, c_long, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P]),
    "lmsf_blas_init": (c_int, [c_long]),
    "lmsf_blas_ready": (c_int, []),
    "lmsf_blas_linear": (c_int, [_P, c_long, _P, c_long, _P, _P, c_long, c_int, c_int, c_int, _P]),
    "lmsf_blas_tune": (c_int, [_P, c_long, _P, c_int, c_long, _P, _P, c_long, c_int, c_int, c_int, c_int, c_int, _P, _P]),
    "lmsf_blas_plans": (c_long, []),
    "lmsf_route_linear": (None, [POINTER(Tunables), POINTER(ProductShape), c_int, POINTER(Route)]),
    "lmsf_route_linear_gated": (None, [POINTER(Tunables), POINTER(ProductShape), c_int, c_int, POINTER(Route)]),
    "lmsf_route_qkv": (None, [POINTER(Tunables), POINTER(ProductShape), c_int, c_int, POINTER(Route)]),
    "lmsf_route_deferred_norm": (None, [POINTER(Tunables), c_int, c_int, c_int, c_int, c_int, POINTER(Route)]),
    "lmsf_route_decode_attention": (None, [POINTER(Tunables), c_int, c_int, c_int, c_int, POINTER(c_int),
                                           POINTER(c_int)]),
}


def load_library() -> ctypes.CDLL:
    """The kernel library, built first if no current build exists."""
    global _lib, _lib_path
    if _lib is not None:
        return _lib
    try:
        path = _build.ensure_built()
    except Exception as e:  # noqa: BLE001 - reported with its cause
        raise KernelLibraryError("the HIP kernel library of lmsf_amd could not be built: %s" % e) from e
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise KernelLibraryError("the HIP kernel library %s could not be loaded: %s" % (path, e)) from e
    for name, (res, args) in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            raise KernelLibraryError("%s lacks the entry point %s; rebuild it (python -m lmsf_amd.csrc.build)"
                                     % (path, name))
        fn.restype = res
        fn.argtypes = args
    got = lib.lmsf_abi_version()
    if got != ABI_VERSION:
        raise KernelLibraryError("%s has ABI version %d, this package needs %d; rebuild it" % (path, got, ABI_VERSION))
    _lib, _lib_path = lib, path
    return lib


def library_path() -> Optional[str]:
    return _lib_path


def last_error(lib: ctypes.CDLL) -> str:
    msg = lib.lmsf_last_error()
    return msg.decode("utf-8", "replace") if msg else "unknown error"
