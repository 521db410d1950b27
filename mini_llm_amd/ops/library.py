"""Loads the HIP kernel library with ctypes and declares its entry points.

There is no fallback: without the library (or without a GPU) every op raises. The reference
loads its engine the same way (pytorch/src/mini_llm/native.py:203-214); the path may be given
with MINI_LLM_LIBRARY, as there."""

from __future__ import annotations

import ctypes
import os
from ctypes import c_float, c_int, c_longlong, c_void_p
from pathlib import Path

_library: ctypes.CDLL | None = None

P = c_void_p
_SIGNATURES = {
    "mllm_embed": [P, P, P, P, P, P, P, c_int, c_int, c_int, P],
    "mllm_layernorm": [P, P, P, P, P, c_int, c_int, c_float, c_int, c_int, P],
    "mllm_add": [P, P, P, c_longlong, c_int, P],
    "mllm_gemm": [P, P, c_int, P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, P],
    "mllm_gemm_takes_packed_rows": [c_int, c_int, c_int, c_int],
    "mllm_gemm_split": [P, P, c_int, P, c_int, c_int, c_int, c_int, c_int, c_int, P],
    "mllm_gemm_split_blocks": [c_int, c_int, c_int, c_int],
    "mllm_gemm_qkv_cache": [P, P, c_int, P, P, P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, P],
    "mllm_convert": [P, P, c_int, c_int, c_int, c_int, c_int, P],
    "mllm_pack_matrix": [P, P, c_int, c_int, c_int, c_int, c_int, P],
    "mllm_packed_elements": [c_int, c_int, c_int],
    "mllm_probe_read": [P, c_longlong, P, c_int, P],
    "mllm_probe_mfma": [P, c_int, c_int, c_int, P],
    "mllm_cache_write": [P, P, c_int, P, P, P, c_int, c_int, c_int, c_int, c_int, P],
    "mllm_attention": [P, c_int, P, P, P, c_int, P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, P],
    "mllm_attention_decode": [P, c_int, P, P, P, c_int, P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_int, P, P, P],
    "mllm_attention_decode_supported": [c_int, c_int, c_int],
    "mllm_attention_prefill": [P, c_int, P, P, P, c_int, P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, P],
    "mllm_attention_prefill_supported": [c_int, c_int],
    "mllm_sample": [P, c_int, c_int, P, P, P, P, P, P, P, P],
    "mllm_gemm_best_per_row": [c_int, c_int, c_int, c_int],
    "mllm_gemm_best": [P, P, c_int, P, P, P, c_int, c_int, c_int, c_int, c_int, P],
    "mllm_choose": [P, P, c_int, c_int, P, P, P, P, c_int, c_int, P, c_int, P, P, P, P, P, P, c_int, c_int, c_int, P],
    "mllm_decode_layer_supported": [c_int, c_int, c_int, c_int],
    "mllm_decode_layer_rows": [c_int],
    "mllm_decode_attention_half": [P, P, P, c_int, P, P, P, c_float, P, P, P, P, P, P, P, P, P, c_int, P,
                                   c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, P],
    "mllm_decode_mlp_half": [P, P, P, c_int, P, P, P, c_float, P, P, P, P, c_int, c_int, c_int, c_int, c_int, P],
    "mllm_pending_sum": [P, P, P, c_int, P, c_int, c_int, P],
    "mllm_linear_split_static": [P, P, c_int, P, P, P, c_int, c_int, c_int, c_int, c_int, P],
    "mllm_static_scratch_prepare": [],
    "mllm_pending_layernorm": [P, P, P, c_int, c_int, P, P, P, P, P, c_int, c_int, c_float, c_int, c_int, P],
}


class KernelLibraryError(RuntimeError):
    pass


def library() -> ctypes.CDLL:
    global _library
    if _standing_in is not None:
        return _standing_in
    if _library is None:
        path = os.environ.get("MINI_LLM_LIBRARY")
        if path:
            if not Path(path).is_file():
                raise KernelLibraryError(f"MINI_LLM_LIBRARY={path} does not exist")
        else:
            from ..csrc import build

            try:
                path = str(build.ensure_built())
            except build.BuildError as error:
                raise KernelLibraryError(f"the HIP kernel library is missing and cannot be built: {error}") from None
        lib = ctypes.CDLL(path)
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = c_int
        lib.mllm_packed_elements.restype = c_longlong
        lib.mllm_static_scratch_bytes.restype = c_longlong
        lib.mllm_static_scratch_bytes.argtypes = []
        lib.mllm_last_error.restype = ctypes.c_char_p
        lib.mllm_last_error.argtypes = []
        lib.mllm_kernel_kinds.restype, lib.mllm_kernel_kinds.argtypes = c_int, []
        lib.mllm_kernel_name.restype, lib.mllm_kernel_name.argtypes = ctypes.c_char_p, [c_int]
        lib.mllm_launch_count.restype, lib.mllm_launch_count.argtypes = ctypes.c_ulonglong, [c_int]
        lib.path = path
        _library = lib
    return _library


class _FirstLaunches:
    """Stands in for the library while ``first_launches`` is active: lets the first so many kernel launches through,
    answers every later one with "launched" without launching, and keeps the names of all that were asked for."""

    def __init__(self, lib, limit, period):
        self._lib, self._limit, self._period = lib, limit, period
        self.asked = []

    def __getattr__(self, name):
        fn = getattr(self._lib, name)
        argtypes = _SIGNATURES.get(name)
        if not argtypes or argtypes[-1] is not P or name.startswith("mllm_probe"):
            return fn   # a question about sizes, not a launch (every launching entry point ends with its stream)

        def launch(*args):
            at = len(self.asked)
            self.asked.append(name[len("mllm_"):])
            if self._limit is not None and (at % self._period if self._period else at) >= self._limit:
                return 0
            return fn(*args)

        return launch


_standing_in: _FirstLaunches | None = None


class first_launches:
    """``with first_launches(n) as seen:`` - inside, only the first ``n`` kernel launches of this process's calls into the
    library really happen (``n`` None: all of them; with ``period`` p: the first n of every p, for work that is run
    several times over, as a step is before and during its capture); ``seen.asked`` lists the entry points of all
    launches that were asked for, in order. For measuring: a step captured under it is the first n kernels of that step, so the time of kernel n
    inside the step is the difference between two such graphs' replays (the reference times the stages of its steps with
    event pairs instead, engine/src/gpu_timer.cu:13-120; a replayed graph has no place for those). Whatever the skipped
    kernels would have written is left as it was: nothing computed inside may be used."""

    def __init__(self, limit: int | None, period: int | None = None):
        self._limit, self._period = limit, period

    def __enter__(self):
        global _standing_in
        if _standing_in is not None:
            raise RuntimeError("first_launches is already active")
        _standing_in = _FirstLaunches(library(), self._limit, self._period)
        return _standing_in

    def __exit__(self, *_):
        global _standing_in
        _standing_in = None


def check(status: int) -> None:
    if status != 0:
        raise KernelLibraryError(library().mllm_last_error().decode())
