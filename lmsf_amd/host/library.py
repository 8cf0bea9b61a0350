"""Loads ``liblmsf_host.so``: the cache manager, the scheduler and the step's metadata, written in C++
(``lmsf_amd/csrc/host``). It has no GPU code and is built with the system's C++ compiler at its first
use, so the host side of the engine runs wherever the package does."""
import ctypes
from ctypes import POINTER, c_char_p, c_double, c_int, c_int64, c_void_p
from typing import Optional

from ..csrc import build as _build

HOST_ABI_VERSION = 4

OK, CACHE_ERROR, OUT_OF_PAGES, VALUE_ERROR = 0, 1, 2, 3


class HostLibraryError(RuntimeError):
    """The host library cannot be built or loaded, or is not the one this package was written for."""


_lib: Optional[ctypes.CDLL] = None
_P = c_void_p
_PP = POINTER(c_void_p)

_SIGNATURES = {
    "lmsf_host_abi_version": (c_int, []),
    "lmsf_host_last_error": (c_char_p, []),
    "lmsf_pool_create": (c_int, [c_int, _PP]),
    "lmsf_pool_destroy": (None, [_P]),
    "lmsf_pool_num_free": (c_int, [_P]),
    "lmsf_pool_allocate": (c_int, [_P, POINTER(c_int)]),
    "lmsf_pool_release": (c_int, [_P, c_int]),
    "lmsf_cm_create": (c_int, [c_int, _P, _P, _P, c_int, _PP]),
    "lmsf_cm_destroy": (None, [_P]),
    "lmsf_cm_has_request": (c_int, [_P, c_int64]),
    "lmsf_cm_num_free_state_slots": (c_int, [_P]),
    "lmsf_cm_num_free_pages": (c_int, [_P, c_int, POINTER(c_int)]),
    "lmsf_cm_request_info": (c_int, [_P, c_int64, _P]),
    "lmsf_cm_tokens_held": (c_int, [_P, c_int, _P, _P, _P]),
    "lmsf_cm_block_table": (c_int, [_P, c_int64, c_int, _P, c_int, POINTER(c_int), POINTER(c_int)]),
    "lmsf_cm_live_requests": (c_int, [_P, _P, c_int, POINTER(c_int)]),
    "lmsf_cm_pages_needed": (c_int, [_P, c_int, c_int64, c_int64, _P]),
    "lmsf_cm_can_append": (c_int, [_P, c_int, c_int64, c_int64, c_int]),
    "lmsf_cm_add_request": (c_int, [_P, c_int64, POINTER(c_int)]),
    "lmsf_cm_append": (c_int, [_P, c_int64, c_int64, POINTER(c_int64)]),
    "lmsf_cm_commit": (c_int, [_P, c_int64]),
    "lmsf_cm_rollback": (c_int, [_P, c_int64]),
    "lmsf_cm_free_request": (c_int, [_P, c_int64]),
    "lmsf_cm_reset": (c_int, [_P]),
    "lmsf_cm_slot_mapping": (c_int, [_P, c_int64, c_int, c_int64, c_int64, _P]),
    "lmsf_cm_check_invariants": (c_int, [_P]),
    "lmsf_cm_begin_step": (c_int, [_P, c_int, _P, _P, _P, _P]),
    "lmsf_cm_abort_step": (c_int, [_P, c_int, _P, _P]),
    "lmsf_cm_commit_step": (c_int, [_P, c_int, _P]),
    "lmsf_cm_step_widths": (c_int, [_P, c_int, _P, _P]),
    "lmsf_step_layout": (c_int, [c_int64, c_int64, c_int64, c_int, _P, _P, POINTER(c_int64)]),
    "lmsf_cm_fill_step": (c_int, [_P, c_int, _P, _P, _P, _P, _P, _P]),
    "lmsf_sched_create": (c_int, [_P, c_int64, c_int, c_int64, c_int64, c_double, _PP]),
    "lmsf_sched_destroy": (None, [_P]),
    "lmsf_sched_add": (c_int, [_P, c_int64, c_int64, c_int64]),
    "lmsf_sched_set_progress": (c_int, [_P, c_int, _P, _P, _P]),
    "lmsf_sched_abort": (c_int, [_P, c_int64, POINTER(c_int)]),
    "lmsf_sched_finish": (c_int, [_P, c_int64]),
    "lmsf_sched_schedule": (c_int, [_P, _P]),
    "lmsf_sched_plan": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P]),
    "lmsf_sched_queue": (c_int, [_P, c_int, _P, c_int, POINTER(c_int)]),
    "lmsf_sched_num_preemptions": (c_int64, [_P]),
    "lmsf_llama_config_parse": (c_int, [c_char_p, _P]),
    "lmsf_llama_config_validate": (c_int, [_P]),
    "lmsf_rope_scaling_parse": (c_int, [c_char_p, _P]),
    "lmsf_safetensors_open": (c_int, [c_char_p, _PP]),
    "lmsf_safetensors_close": (None, [_P]),
    "lmsf_safetensors_count": (c_int64, [_P]),
    "lmsf_safetensors_record": (c_int, [_P, c_int64, _P]),
    "lmsf_safetensors_data": (c_void_p, [_P, POINTER(c_int64)]),
}


def load_host_library() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    try:
        path = _build.ensure_host_built()
    except Exception as e:  # noqa: BLE001 - reported with its cause
        raise HostLibraryError("the host library of lmsf_amd could not be built: %s" % e) from e
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise HostLibraryError("the host library %s could not be loaded: %s" % (path, e)) from e
    for name, (res, args) in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            raise HostLibraryError("%s lacks the entry point %s; rebuild it (python -m lmsf_amd.csrc.build)"
                                   % (path, name))
        fn.restype = res
        fn.argtypes = args
    got = lib.lmsf_host_abi_version()
    if got != HOST_ABI_VERSION:
        raise HostLibraryError("%s has ABI version %d, this package needs %d; rebuild it" % (path, got, HOST_ABI_VERSION))
    _lib = lib
    return lib


def last_error(lib: ctypes.CDLL) -> str:
    msg = lib.lmsf_host_last_error()
    return msg.decode("utf-8", "replace") if msg else "unknown error"
