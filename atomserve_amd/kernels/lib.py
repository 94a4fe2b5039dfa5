"""Loads the compiled kernel libraries through ctypes and declares their entry points.

The libraries use the HIP runtime that PyTorch has already loaded into the process,
so that device pointers and streams of torch tensors are valid in them; torch is
therefore imported before the first library.  There is no fallback: a kernel whose
library cannot be built or loaded raises.
"""

import ctypes
from ctypes import c_double, c_float, c_int, c_longlong, c_size_t, c_void_p

import torch  # noqa: F401  (loads libamdhip64 first)

from atomserve_amd.kernels import build

P, I, F = c_void_p, c_int, c_float

# name -> (library, argument types); every entry point returns an int status.
SIGNATURES = {
    "as_embed_gather": ("elementwise", [P, I, P, P, I, I, I, F, P]),
    "as_logits_finish": ("elementwise", [P, c_longlong, F, F, P]),
    "as_rmsnorm": ("elementwise", [P, P, P, P, I, F, P, I, I, I, I, P]),
    "as_rmsnorm_split": ("elementwise", [P, P, I, I, P, P, I, F, P, I, I, I, I, P]),
    "as_rope_table": ("elementwise", [P, P, P, I, I, P]),
    "as_qk_norm_rope_store": ("elementwise", [P, I, P, P, I, P, P, P, P, P, I, I, I, I, I, F, I, I, P]),
    "as_silu_mul": ("elementwise", [P, P, I, I, I, P]),
    "as_attn_single_query": ("attention", [P, P, P, I, P, I, P, P, P, I, P, P, P, P, I, I, I, I, F, I, I, I, P]),
    "as_attn_decode_mfma": ("attention", [P, P, P, P, I, P, P, P, I, P, P, P, P, I, I, I, I, F, I, I, I, P]),
    "as_attn_decode_fresh": ("attention", [P, P, P, I, P, P, F, I, P, P, P, I, P, P, I, P, P, P, P, I, I, I, I, F, I, I, I, P]),
    "as_attn_prefill_mfma": ("attention", [P, P, P, P, I, P, I, P, I, I, I, I, F, I, I, I, I, P, P, P, P]),
    "as_gemm_f32": ("gemm", [P, P, P, I, I, I, P]),
    "as_gemm_bf16_skinny": ("gemm", [P, P, P, P, I, I, I, I, I, P]),
    "as_gemm_bf16_gated": ("gemm", [P, P, P, P, I, I, I, P]),
    "as_gemm_bf16_link": ("gemm", [P, P, P, P, P, P, P, I, I, I, P]),
    "as_gemm_bf16_scaled": ("gemm", [P, P, I, F, P, P, P, I, I, I, I, P]),
    "as_wave_order": ("gemm", [P, P, I, I, P]),
    "as_gemm_bf16_tile": ("gemm", [P, P, P, P, P, I, I, I, I, I, I, I, P]),
    "as_blas_plan": ("blas", [I, I, I, I, c_size_t]),
    "as_blas_candidate_index": ("blas", [I, I, I, I, c_size_t, I]),
    "as_blas_adopt": ("blas", [I, I, I, I, c_size_t, I]),
    "as_blas_prepare_adoption": ("blas", []),
    "as_blas_gemm": ("blas", [P, P, P, I, I, I, I, I, P, c_size_t, P]),
    "as_argmax": ("sampling", [P, P, I, I, P]),
    "as_sample": ("sampling", [P, I, I, P, P, P, P, P, P, P]),
    "as_sample_split": ("sampling", [P, I, I, P, P, P, P, P, P, P, P, P]),
    "as_apply_penalty": ("sampling", [P, P, P, P, I, I, P]),
    "as_topk": ("sampling", [P, I, I, I, P, P, P]),
}

STATUS = {-1: "unsupported dtype", -2: "unsupported shape or size", -3: "kernel launch failed",
          -4: "partial results exceed the library's static scratch array"}

_libs: dict = {}
_funcs: dict = {}


class KernelError(RuntimeError):
    pass


def _library(name: str):
    if name not in _libs:
        path = build.library_path(name)
        try:
            _libs[name] = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load {path}: {e}") from e
    return _libs[name]


def entry(name: str):
    """The ctypes function `name`, loading (and if needed compiling) its library."""
    fn = _funcs.get(name)
    if fn is None:
        lib_name, argtypes = SIGNATURES[name]
        try:
            fn = getattr(_library(lib_name), name)
        except AttributeError as e:
            raise KernelError(f"lib_{lib_name}.so has no entry point {name}") from e
        fn.argtypes = argtypes
        fn.restype = c_int
        _funcs[name] = fn
    return fn


def call(name: str, *args) -> None:
    status = entry(name)(*args)
    if status != 0:
        raise KernelError(f"{name}: {STATUS.get(status, status)}")


def loaded_libraries() -> list:
    return sorted(_libs)


__all__ = ["KernelError", "call", "entry", "loaded_libraries", "c_double"]
