"""Loads the kernel library and declares its C entry points for ctypes."""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

from .build import ensure_built

ABI_VERSION = 21


class KernelLibraryError(RuntimeError):
    """The compiled kernels are missing, stale or failed to load."""


class KernelError(RuntimeError):
    """An entry point refused its arguments or a launch failed."""


_P, _I, _F, _Z = c_void_p, c_int, c_float, c_size_t

_SIGNATURES = {
    "tff_embed": [_P, _P, _P, _I, _I, _I, _I, _P],
    "tff_add_rmsnorm": [_P, _P, _I, _Z, _P, _F, _P, _P, _I, _I, _I, _P],
    "tff_rmsnorm": [_P, _P, _F, _P, _I, _I, _I, _P],
    "tff_gemm": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _Z, _I, _P],
    "tff_gemm_workspace_bytes": [_I, _I, _I, _I, _I, _I],
    "tff_gemm_plan": [_I, _I, _I, _I, _I, _P, _P, _P],
    "tff_gemm_residual_prenorm": [_P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _I, _P],
    "tff_gemm_row_scaled": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I, _I, _I, _F, _P],
    "tff_pack_weight": [_P, _P, _I, _I, _P],
    "tff_embed_packed": [_P, _P, _P, _I, _I, _I, _P],
    "tff_qk_norm_rope_kv": [_P, _I, _I, _I, _I, _P, _P, _F, _P, _I, _I, _I, _P, _P, _P, _P,
                            _I, _I, _I, _I, _P],
    "tff_attention_generic": [_P, _I, _P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I,
                              _F, _I, _I, _P],
    "tff_attention_mfma_supported": [_I, _I],
    "tff_attention_mfma": [_P, _I, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I,
                           _I, _I, _I, _I, _I, _I, _F, _P],
    "tff_attention_decode_fused": [_P, _I, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _F, _P, _I, _I,
                                   _I, _I, _I, _I, _I, _I, _I, _I, _F, _P],
    "tff_attention_decode_runs": [_P, _I, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _F, _P, _I, _I,
                                  _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _F, _P],
    "tff_attention_mfma_runs": [_P, _I, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I,
                                _I, _F, _P],
    "tff_attention_decode_fused_static": [_P, _I, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _F, _P, _I, _I,
                                          _I, _I, _I, _I, _I, _I, _I, _I, _F, _P],
    "tff_attention_split_reduce": [_P, _P, _P, _I, _I, _I, _I, _P, _I, _P],
    "tff_swiglu": [_P, _P, _I, _I, _I, _P],
    "tff_cast": [_P, _I, _P, _I, c_int64, _P],
    "tff_argmax_workspace_bytes": [_I, _I],
    "tff_argmax": [_P, _P, _I, _I, _P, _P],
    "tff_repetition_penalty": [_P, _I, _I, _P, _P, _P, _P],
    "tff_sample": [_P, _P, _I, _I, _P, _P, _P, _P, _P, _P, _P],
    "tff_probe_stream_read": [_P, _Z, _P, _I, _P],
    "tff_probe_mfma": [_P, _I, _I, _I, _P],
}

_lib = None


def load() -> ctypes.CDLL:
    """The library, built on first use if the tree holds none for these sources."""
    global _lib
    if _lib is not None:
        return _lib
    try:
        path = ensure_built()
        lib = ctypes.CDLL(path)
    except Exception as e:  # build errors, missing hipcc, dlopen errors
        raise KernelLibraryError(
            f"the HIP kernel library could not be built or loaded: {e}\n"
            "There is no fallback path; build it with `python -c 'import __graft_entry__ as g; g.build()'`."
        ) from e
    lib.tff_last_error.restype = c_char_p
    lib.tff_last_error.argtypes = []
    lib.tff_abi_version.restype = c_int
    if lib.tff_abi_version() != ABI_VERSION:
        raise KernelLibraryError(
            f"{path} has ABI {lib.tff_abi_version()}, the package expects {ABI_VERSION}; rebuild it")
    for name, args in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_size_t if name.endswith("_bytes") else c_int
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != 0:
        raise KernelError(load().tff_last_error().decode())
