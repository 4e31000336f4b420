"""Loads the two native libraries with ctypes and declares their signatures.

The kernel library is needed for any model step; there is no fallback.  If it is
missing it is compiled once (csrc/build.py); if it cannot be loaded the error
says so loudly.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_long, c_ulonglong, c_void_p, POINTER

from ..csrc import build as _build

_kernels = None
_host = None
_recording = None      # a list that collects (launcher name, arguments) of every launch, or None


class NativeLibraryError(RuntimeError):
    pass


def _load(path: str) -> ctypes.CDLL:
    try:
        return ctypes.CDLL(path)
    except OSError as exc:
        raise NativeLibraryError(f"cannot load native library {path}: {exc}") from exc


def kernels() -> ctypes.CDLL:
    """The gfx950 kernel library.  torch is imported first so that both share one HIP runtime."""
    global _kernels
    if _kernels is None:
        import torch  # noqa: F401  (loads libamdhip64 before our library resolves it)
        lib = _load(_build.ensure_kernels())
        P, I, L, F = c_void_p, c_int, c_long, c_float
        lib.mgpt_embed.argtypes = [P, P, P, P, P, I, I, I, P]
        lib.mgpt_layernorm.argtypes = [P, P, P, P, P, I, I, F, I, P]
        lib.mgpt_linear_generic.argtypes = [P, I, L, P, I, P, P, I, L, I, I, I, I, P]
        lib.mgpt_kv_write.argtypes = [P, I, L, I, I, P, P, P, I, I, I, I, P]
        lib.mgpt_paged_attention_generic.argtypes = [P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, F, I, I, I, P]
        lib.mgpt_sample.argtypes = [P, L, I, I, I, P, P, P, P, P, c_ulonglong, P, P, P, I, P]
        lib.mgpt_sample_advance.argtypes = [P, L, I, I, I, P, P, P, P, P, c_ulonglong, P,
                                            P, P, P, P, P, P, P, I, I, I, I, P, P, I, I, P, P, I, P]
        for name in ("mgpt_embed", "mgpt_layernorm", "mgpt_linear_generic", "mgpt_kv_write",
                     "mgpt_paged_attention_generic", "mgpt_sample", "mgpt_sample_advance"):
            getattr(lib, name).restype = I
        _declare_optional(lib)
        lib.mgpt_plan_create.restype = c_void_p
        lib.mgpt_plan_create.argtypes = []
        lib.mgpt_plan_destroy.restype = None
        lib.mgpt_plan_destroy.argtypes = [c_void_p]
        lib.mgpt_plan_size.argtypes = [c_void_p]
        lib.mgpt_plan_add.argtypes = [c_void_p, c_char_p, POINTER(c_ulonglong), c_int]
        lib.mgpt_plan_run.argtypes = [c_void_p, c_void_p, POINTER(c_int)]
        for name in ("mgpt_plan_size", "mgpt_plan_add", "mgpt_plan_run"):
            getattr(lib, name).restype = c_int
        _kernels = _Recording(lib)
    return _kernels


class _Recording:
    """The kernel library with its launchers wrapped: while a recording is on (record()), every
    launch that was made (return code 0) is noted with its arguments, for ops.plan.LaunchPlan."""

    def __init__(self, lib: ctypes.CDLL) -> None:
        self._lib = lib

    def __getattr__(self, name: str):
        fn = getattr(self._lib, name)
        argtypes = getattr(fn, "argtypes", None)
        # launchers take the stream last; everything else (queries, the plan's own calls) passes through
        if not name.startswith("mgpt_") or name.startswith("mgpt_plan_") or not argtypes or argtypes[-1] is not c_void_p \
                or fn.restype is not c_int:
            setattr(self, name, fn)
            return fn

        def launch(*args):
            rc = fn(*args)
            if _recording is not None and rc == 0:
                _recording.append((name, argtypes, args))
            return rc

        setattr(self, name, launch)
        return launch


class unrecorded:
    """Launches inside the block are not noted: work done once (a matrix packed or folded at its
    first use) is no part of a step's plan."""

    def __enter__(self):
        global _recording
        self._outer = _recording
        _recording = None

    def __exit__(self, *exc):
        global _recording
        _recording = self._outer
        return False


class record:
    """with record() as launches: ... collects (launcher, argtypes, arguments) of every launch made
    inside the block."""

    def __enter__(self):
        global _recording
        self._outer = _recording
        _recording = []
        return _recording

    def __exit__(self, *exc):
        global _recording
        _recording = self._outer
        return False


def _declare_optional(lib: ctypes.CDLL) -> None:
    """Signatures of the bfloat16 fast kernels."""
    P, I, L, F = c_void_p, c_int, c_long, c_float
    table = {
        "mgpt_linear_skinny": [P, L, P, P, P, F, P, P, P, P, I, L, I, I, I, I, P, P, P, I, I, I, I, I, I, P, L, P],
        "mgpt_linear_head_best": [P, L, P, P, P, F, P, P, P, P, L, I, I, I, P, P, I, P],
        "mgpt_pack_weight": [P, P, I, I, P],
        "mgpt_linear_skinny_partials": [I, I, I, I, I],
        "mgpt_linear_skinny_row_groups": [I, I, I],
        "mgpt_fold_layernorm": [P, P, P, P, P, P, P, I, I, P],
        "mgpt_paged_attention_split_bf16": [P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, F, I, P],
        "mgpt_paged_attention_split_fast_bf16": [P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, F, I, P],
        "mgpt_paged_attention_decode_bf16": [P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, I, F, I, I, P],
        "mgpt_linear_mfma": [P, L, P, P, P, I, L, I, I, I, I, P, L, P],
        "mgpt_linear_mfma_shape": [I, I, P, L, P, P, P, I, L, I, I, I, I, P, L, P],
        "mgpt_linear_mfma_partials": [I, I, I, I],
        "mgpt_linear_mfma_parts": [P, L, P, P, P, L, I, I, I, P],
        "mgpt_linear_mfma_qkv": [P, L, P, P, P, L, I, I, I, P, P, P, I, I, I, I, I, I, P],
        "mgpt_prefill_attention_bf16": [P, L, P, L, P, P, P, I, P, P, I, I, I, I, I, I, F, I, I, P],
        # a residual that is still a sum: base, partials, n_parts, part_stride, token table, position table, ids, positions
        "mgpt_fused_attention_decode": [P, P, I, L, P, P, P, P, P, P, P, P, F, P, P, P, P, P, L, P, P, P, P, I, P, P,
                                        I, I, I, I, I, I, F, P],
        "mgpt_fused_attention_tokens": [I, I, I],
        "mgpt_fused_mlp_decode": [P, P, I, L, P, P, P, P, P, P, P, F, P, P, P, P, P, L, I, I, I, P],
        "mgpt_residual_layernorm": [P, P, I, L, P, P, P, P, P, P, F, P, P, I, I, I, P, P],
        "mgpt_residual_parts_limit": [I],
        "mgpt_linear_decode_parts": [P, L, P, P, P, P, I, I, I, P],
        "mgpt_linear_decode_parts_count": [],
        "mgpt_residual_settle": [P, P, I, L, P, P, P, P, P, I, I, P],
        "mgpt_fused_parts_limit": [I],
    }
    for name, argtypes in table.items():
        fn = getattr(lib, name, None)
        if fn is not None:
            fn.argtypes = argtypes
            fn.restype = L if name in ("mgpt_linear_skinny_partials", "mgpt_linear_mfma_partials") else I


def host() -> ctypes.CDLL:
    """The host runtime: cache manager and scheduler."""
    global _host
    if _host is None:
        lib = _load(_build.ensure_host())
        P, I = c_void_p, c_int
        IP = POINTER(c_int)
        lib.mgpt_host_last_error.restype = c_char_p
        lib.mgpt_cache_create.restype = P
        lib.mgpt_cache_create.argtypes = [I, IP, IP, IP, I]
        lib.mgpt_cache_destroy.argtypes = [P]
        lib.mgpt_cache_destroy.restype = None
        for name, args in {
            "mgpt_cache_num_groups": [P], "mgpt_cache_acquire_slot": [P], "mgpt_cache_slot_live": [P, I],
            "mgpt_cache_num_free_slots": [P], "mgpt_cache_pages_needed": [P, I, I],
            "mgpt_cache_can_allocate": [P, I], "mgpt_cache_reserve": [P, I, I],
            "mgpt_cache_release_passed": [P, I, I], "mgpt_cache_free_slot": [P, I],
            "mgpt_cache_num_free_pages": [P, I], "mgpt_cache_held_pages": [P, I, I],
            "mgpt_cache_table_len": [P, I, I], "mgpt_cache_copy_table": [P, I, I, P, I],
            "mgpt_cache_check": [P],
            "mgpt_cache_build_step": [P, I, P, P, P, I, I, I, P, P, P, P, P, P],
            "mgpt_sched_add": [P, P, I, I, I, c_float, I, c_float, c_ulonglong, I],
            "mgpt_sched_has_work": [P], "mgpt_sched_cancel": [P, I], "mgpt_sched_schedule": [P, P],
            "mgpt_sched_entries": [P, P, P, P, P, I],
            "mgpt_sched_fill": [P, P, I, I, I, I, I] + [P] * 14,
            "mgpt_sched_plan_burst": [P, I], "mgpt_sched_commit_burst": [P, P, I, I, P, P, P, P, I],
            "mgpt_sched_commit": [P, P, I, P, P, P, P, I],
            "mgpt_sched_queue": [P, I, P, I], "mgpt_sched_request_info": [P, I, P],
            "mgpt_sched_copy_output": [P, I, P, I],
        }.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = I
        lib.mgpt_sched_create.restype = P
        lib.mgpt_sched_create.argtypes = [P, I, I, I, I, I, I]
        lib.mgpt_sched_destroy.argtypes = [P]
        lib.mgpt_sched_destroy.restype = None
        lib.mgpt_sched_counter.argtypes = [P, I]
        lib.mgpt_sched_counter.restype = c_long
        lib.mgpt_sched_forget_finished.argtypes = [P]
        lib.mgpt_sched_forget_finished.restype = None
        lib.mgpt_sched_num_records.argtypes = [P]
        lib.mgpt_sched_num_records.restype = I
        _host = lib
    return _host


def host_error() -> str:
    return host().mgpt_host_last_error().decode("utf-8", "replace")
