"""Loads the native libraries through ctypes and declares their entry points.

There is no fallback: if a library cannot be built or loaded the import of
whatever needs it fails with the reason.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import c_char_p, c_float, c_int, c_long, c_longlong, c_void_p, POINTER

from . import build

_lock = threading.Lock()
_kernels = None
_host = None

P = c_void_p
I = c_int
F = c_float
IP = POINTER(c_int)
LLP = POINTER(c_longlong)


class NativeError(RuntimeError):
    pass


def _declare(lib, name, restype, argtypes):
    fn = getattr(lib, name)
    fn.restype = restype
    fn.argtypes = argtypes
    return fn


_KERNEL_API = {
    "pa_last_error": (c_char_p, []),
    "pa_device_arch": (I, [c_char_p, I]),
    "pa_num_compute_units": (I, []),
    "pa_stream_read": (I, [P, P, c_long, P, I]),
    "pa_embed_gather": (I, [P, I, P, P, P, I, I, I]),
    "pa_carry_tokens": (I, [P, P, P, P, P, I, I, I]),
    "pa_zero_fresh_rows": (I, [P, P, c_long, P, P, I, I]),
    "pa_rmsnorm": (I, [P, I, P, P, P, P, P, I, I, F]),
    "pa_silu_mul": (I, [P, I, P, P, I, I, I]),
    "pa_gather_rows": (I, [P, I, P, P, P, I, I]),
    "pa_add_bias": (I, [P, I, P, P, I, I]),
    "pa_to_f32": (I, [P, I, P, P, c_long]),
    "pa_qknorm_rope_kv": (I, [P, I, P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, F]),
    "pa_gemm_plain": (I, [P, I, I, P, P, P, P, I, I, I, c_long, c_long, c_long]),
    "pa_gemm_library": (I, [P, P, P, P, I, I, I, c_long, c_long, P, c_long]),
    "pa_gemm_skinny": (I, [P, I, I, P, P, P, P, I, I, I, c_long, c_long, I]),
    "pa_pack_tiles": (I, [P, P, P, I, I]),
    "pa_gemm_mid_slices": (I, [I, I]),
    "pa_gemm_mid_parts": (c_long, [I, I, I]),
    "pa_gemm_mid": (I, [P, I, I, P, P, P, P, P, I, I, I, c_long, c_long, I, I]),
    "pa_gemm_skinny_slices": (I, [I, I]),
    "pa_gemm_skinny_sliced": (I, [P, P, P, P, P, I, I, I, c_long, I, I]),
    "pa_gemm_mid_normed": (I, [P, I, P, P, P, F, P, P, P, I, I, I, c_long, c_long, I]),
    "pa_sum_slices": (I, [P, I, P, P, I, c_long]),
    "pa_gemm_tall_shape": (None, [I, I, I, I, IP]),
    "pa_gemm_tall": (I, [P, I, P, P, P, P, P, I, I, I, c_long, c_long, I, I, I]),
    "pa_rmsnorm_slices": (I, [P, I, P, I, c_long, P, P, P, P, I, I, F]),
    "pa_attn_generic": (I, [P, I, P, P, P, P, I, P, P, P, I, I, I, I, I, I, F, F]),
    "pa_attn_mfma_supports": (I, [I, I]),
    "pa_attn_decode_workspace": (c_long, [I, I, I, I]),
    "pa_attn_decode": (I, [P, P, P, P, P, I, P, P, P, P, P, I, I, I, I, I, I, F, F, I, I]),
    "pa_attn_decode_fused": (I, [P, P, P, P, P, P, P, F, P, P, P, I, P, P, P, P, P, I, I, I, I, I, I, F, F, I, I]),
    "pa_attn_decode_fused_supports": (I, [I, I, I, I, I]),
    "pa_attn_prefill": (I, [P, P, P, P, P, I, P, P, P, P, I, I, I, I, I, I, I, I, F, F]),
    "pa_attn_prefill_cut": (I, [P, P, P, P, P, I, P, P, P, P, I, I, I, I, I, I, I, I, F, F, I, I, I, I]),
    "pa_argmax_scratch": (I, [I, I]),
    "pa_argmax": (I, [P, P, P, P, I, I]),
    "pa_argmax_static_capacity": (I, []),
    "pa_argmax_static": (I, [P, P, P, I, I]),
    "pa_sample": (I, [P, P, P, P, P, P, P, I, I]),
    "pa_sample_wide_workspace": (c_long, [I, I]),
    "pa_logprobs": (I, [P, P, P, P, P, P, P, I, I, I, I]),
    "pa_sample_wide": (I, [P, P, P, P, P, P, P, P, I, I, I]),
}

_HOST_API = {
    "pa_cache_create": (P, [I, I, IP, IP, I]),
    "pa_cache_destroy": (None, [P]),
    "pa_cache_open": (I, [P, c_longlong, I]),
    "pa_cache_reserve": (I, [P, c_longlong, I]),
    "pa_cache_commit": (I, [P, c_longlong, I]),
    "pa_cache_rollback": (I, [P, c_longlong]),
    "pa_cache_close": (I, [P, c_longlong]),
    "pa_cache_has": (I, [P, c_longlong]),
    "pa_cache_len": (I, [P, c_longlong]),
    "pa_cache_state_slot": (I, [P, c_longlong]),
    "pa_cache_page_size": (I, [P]),
    "pa_cache_num_groups": (I, [P]),
    "pa_cache_free_pages": (I, [P, I]),
    "pa_cache_capacity_pages": (I, [P, I]),
    "pa_cache_free_state_slots": (I, [P]),
    "pa_cache_num_requests": (I, [P]),
    "pa_cache_live_pages": (I, [P, c_longlong, I]),
    "pa_cache_reservable_len": (I, [P, c_longlong]),
    "pa_cache_peak_pages": (I, [P, I, I, I]),
    "pa_cache_table": (I, [P, c_longlong, I, P, I]),
    "pa_cache_fill_step": (I, [P, I, P, P, P, I, P, P, P, P, P, P, P, P]),
    "pa_cache_audit": (c_char_p, [P]),
    "pa_cache_error": (c_char_p, [P]),
    "pa_sched_create": (P, [P, I, I, I, I, I, I, I]),
    "pa_sched_destroy": (None, [P]),
    "pa_sched_add": (I, [P, c_longlong, I, I, I, I]),
    "pa_sched_schedule": (I, [P, P, P, P, P, I]),
    "pa_sched_step_done": (I, [P]),
    "pa_sched_step_cancelled": (None, [P]),
    "pa_sched_on_token": (I, [P, c_longlong]),
    "pa_sched_finish": (I, [P, c_longlong]),
    "pa_sched_num_waiting": (I, [P]),
    "pa_sched_num_running": (I, [P]),
    "pa_sched_tokens_in_use": (I, [P]),
    "pa_sched_preemptions": (c_long, [P]),
    "pa_sched_last_preempted": (I, [P, P, I]),
    "pa_sched_info": (I, [P, c_longlong, P]),
    "pa_sched_error": (c_char_p, [P]),
}


def _load(path: str, api: dict, what: str):
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise NativeError(f"cannot load the {what} library {path}: {e}") from None
    for name, (res, args) in api.items():
        try:
            _declare(lib, name, res, args)
        except AttributeError:
            raise NativeError(f"the {what} library {path} lacks `{name}`; rebuild it "
                              f"(python -c 'import __graft_entry__ as g; g.build()')") from None
    return lib


def host():
    """The host runtime (cache manager, scheduler); needs no GPU."""
    global _host
    if _host is None:
        with _lock:
            if _host is None:
                _host = _load(build.build_host(), _HOST_API, "host runtime")
    return _host


def kernels():
    """The HIP kernel library.  Loading it needs the ROCm runtime; running it needs a gfx950 GPU."""
    global _kernels
    if _kernels is None:
        with _lock:
            if _kernels is None:
                _kernels = _load(build.build_kernels(), _KERNEL_API, "kernel")
    return _kernels


def check(rc: int) -> None:
    """Raises with the library's message when an entry point refused or failed."""
    if rc != 0:
        msg = kernels().pa_last_error()
        raise NativeError(msg.decode() if msg else f"kernel entry point failed with code {rc}")
