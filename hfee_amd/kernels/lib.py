"""Loading the compiled kernel libraries and declaring their entry points.

There is no fallback: if a library cannot be built or loaded, KernelLibraryError
is raised and nothing runs.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import c_void_p, c_int, c_int64, c_float, c_double, c_uint64, c_char_p

from . import build


class KernelLibraryError(RuntimeError):
    pass


class KernelError(RuntimeError):
    """An entry point refused its arguments or its launch failed."""


P, I, L, F, D, U64 = c_void_p, c_int, c_int64, c_float, c_double, c_uint64

_CORE_SIGNATURES = {
    "hfee_embed": [P, P, I, P, I, I, P],
    "hfee_embed_emit": [P, P, P, I, I, P, I, P, L, P, L, P],
    "hfee_rmsnorm": [P, I, P, P, I, P, F, I, I, P],
    "hfee_cast_rows": [P, I, P, P, I, I, P],
    "hfee_swiglu": [P, L, P, P, L, I, I, I, I, I, P],
    "hfee_residual_add": [P, P, I, L, P],
    "hfee_rope_cache_write": [P, L, P, L, P, L, I, P, P, P, I, P, P, I, I, I, I, P, I, I, I, I, I, I, P],
    "hfee_gemm_f32": [P, L, P, L, P, L, I, I, I, I, P],
    "hfee_attention_ref": [P, L, P, L, P, I, P, P, P, I, I, I, I, I, F, I, I, P],
    "hfee_gemm_bf16": [P, I, L, P, L, P, L, I, I, I, I, P, L, I, P],
    "hfee_gemm_bf16_add_norm": [P, P, L, P, L, I, I, I, P, L, P, P, I, F, P],
    "hfee_gemm_bf16_cuts": [P, L, P, L, I, I, I, P, L, P, P],
    "hfee_rope_cache_write_cuts": [P, L, P, I, P, P, P, I, P, P, I, I, I, P, I, I, I, I, I, I, P],
    "hfee_gemm_bf16_scratch": [I, I, I],
    "hfee_gemm_bf16_plan": [I, I, I, P, P, P],
    "hfee_gemm_skinny": [P, L, P, I, L, P, L, I, I, I, I, P, I, F, P, P, P, P, I, P, P, I, I, P, I, I, I, I,
                         P, I, P, L, P, P, I, F, P, L, I, P],
    "hfee_gemm_qkv_rows": [P, L, P, L, P, L, I, I, I, P, P, P, I, P, P, I, I, P, I, I, I, I, P],
    "hfee_argmax": [P, P, L, I, I, P, L, P, I, P],
    "hfee_sample": [P, P, L, I, I, P, P, P, P, L, P],
    "hfee_argmax_static": [P, P, L, I, I, P],
    "hfee_random_fill": [P, I, L, U64, I, D, L, P],
    "hfee_read_stream": [P, L, P, I, I, P],
    "hfee_mfma_loop": [P, I, I, P],
}

_ATTENTION_SIGNATURES = {
    "hfee_attention_bf16_head_dim": [],
    "hfee_attention_bf16_run_tiles": [],
    "hfee_attention_bf16_halves": [],
    "hfee_attention_bf16_layer_limit_log2": [],
    "hfee_attention_bf16_prefill": [P, L, P, L, P, I, P, I, P, I, P, I, I, I, I, F, I, I, P],
    "hfee_attention_bf16_decode": [P, L, P, L, P, P, P, P, I, P, I, I, I, I, F, I, P, L, I, I, P, I, P],
}

_lock = threading.Lock()
_loaded: dict[str, "Library"] = {}


class Library:
    def __init__(self, name: str, path: str, signatures: dict):
        self.name, self.path = name, path
        try:
            self._dll = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryError(f"cannot load kernel library {path}: {e}") from None
        self._dll.hfee_last_error.restype = c_char_p
        self._dll.hfee_last_error.argtypes = []
        for fn, argtypes in signatures.items():
            try:
                f = getattr(self._dll, fn)
            except AttributeError:
                raise KernelLibraryError(f"kernel library {path} has no entry point {fn}") from None
            f.argtypes = argtypes
            f.restype = c_int

    def call(self, fn: str, *args):
        rc = getattr(self._dll, fn)(*args)
        if rc != 0:
            msg = self._dll.hfee_last_error()
            raise KernelError((msg or b"unknown error").decode("utf-8", "replace"))

    def raw(self, fn: str):
        return getattr(self._dll, fn)


def load(name: str) -> Library:
    """The named library, built first if no up-to-date build exists."""
    with _lock:
        lib = _loaded.get(name)
        if lib is None:
            try:
                path = build.build_library(name)
            except build.BuildError as e:
                raise KernelLibraryError(f"the HIP kernel library '{name}' is not available: {e}") from None
            sigs = _CORE_SIGNATURES if name == "core" else _ATTENTION_SIGNATURES
            lib = _loaded[name] = Library(name, path, sigs)
        return lib


def core() -> Library:
    return load("core")


def attention_bf16(head_dim: int) -> Library:
    if head_dim % 16 != 0 or not 16 <= head_dim <= 256:
        raise KernelError(f"the bfloat16 attention kernels take head sizes 16..256 in steps of 16, "
                          f"not {head_dim}")
    return load(f"attention_bf16_hd{head_dim}")
