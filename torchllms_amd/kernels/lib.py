"""Loads the compiled HIP libraries with ``ctypes`` and declares their C interface.

There is no fallback: if a library cannot be built or loaded, or a kernel refuses its arguments,
an exception is raised.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_uint64, c_void_p
from typing import Dict, Optional

from . import build as _build


class KernelError(RuntimeError):
    """A kernel launcher refused its arguments or HIP reported an error."""


_P = c_void_p
_I = c_int
_F = c_float
_U64 = c_uint64
_I64 = c_int64

# name -> argument types (every function returns int status)
_CORE_SIGNATURES = {
    "tl_embed": [_P, _P, _P, _I, _I, _I, _P],
    "tl_rmsnorm": [_P, _P, _P, _P, _I, _P, _P, _I, _I, _F, _I, _P],
    "tl_rmsnorm_split": [_P, _P, _I, _I64, _P, _P, _I, _P, _P, _I, _I, _F, _P],
    "tl_rope_table": [_P, _P, _I, _I, _P, _P],
    "tl_rope_kv_write": [_P, _I, _I, _I, _I, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I, _P],
    "tl_silu_mul": [_P, _P, _I, _I, _I, _P],
    "tl_add_bias": [_P, _P, _I, _I, _I, _I, _P],
    "tl_attention_generic": [_P, _I, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _P],
    "tl_attention_generic_split": [_P, _I, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P, _P],
    "tl_gemm_f32": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _P],
    "tl_gemm_stream": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _P],
    "tl_gemm_stream_glu": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _P, _I, _F, _P],
    "tl_gemm_stream_residual": [_P, _I, _P, _I, _P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _P],
    "tl_gemm_stream_qkv": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _I, _I, _P, _I, _F, _P],
    "tl_gemm_wide": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P],
    "tl_gemm_wide_splits": [_I, _I],
    "tl_gemm_wide_reduce": [_P, _P, _I, _I, _I, _I, _I, _P],
    "tl_gemm_wide_glu": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _P],
    "tl_gemm_wide_qkv": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _I, _I, _I, _I, _P, _P],
    "tl_sample": [_P, _I, _I, _I, _P, _P, _P, _P, _P, _P],
    "tl_sample_chunks": [_P, _I, _I, _I, _P, _P, _P, _I, _P, _P, _P],
    "tl_sample_chunks_static": [_P, _I, _I, _I, _P, _P, _P, _I, _P, _P],
    "tl_philox_uniform": [_U64, _U64, _P, _I, _P],
}

_core: Optional[ctypes.CDLL] = None
_variants: Dict[str, ctypes.CDLL] = {}


def _declare(lib: ctypes.CDLL, signatures) -> None:
    for name, argtypes in signatures.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = c_int


def core() -> ctypes.CDLL:
    """The core kernel library, built on first use if no current build exists."""
    global _core
    if _core is None:
        path = _build.build_core()
        lib = ctypes.CDLL(str(path))
        lib.tl_last_error.restype = c_char_p
        lib.tl_last_error.argtypes = []
        _declare(lib, _CORE_SIGNATURES)
        _core = lib
    return _core


#: the GPU this package is written for (MI355X): what launch plans assume where no GPU is to be asked
TARGET_COMPUTE_UNITS, TARGET_LDS_BYTES = 256, 160 * 1024
_facts: Optional[tuple] = None


def device_facts() -> tuple:
    """``(compute units, bytes of LDS a block may use)`` of the GPU, as the device itself gives them
    (read once, by the core library); the target's own figures where there is no GPU, so that launch
    plans can be made and tested on a host without one."""
    global _facts
    if _facts is None:
        import torch

        if torch.cuda.is_available():
            lib = core()
            lib.tl_device_compute_units.restype = lib.tl_device_lds_bytes.restype = c_int
            lib.tl_device_compute_units.argtypes = lib.tl_device_lds_bytes.argtypes = []
            _facts = (int(lib.tl_device_compute_units()), int(lib.tl_device_lds_bytes()))
        else:
            _facts = (TARGET_COMPUTE_UNITS, TARGET_LDS_BYTES)
    return _facts


def variant(kind: str, value: int, signatures) -> ctypes.CDLL:
    """A size-specific library (see ``build.VARIANTS``), built on first use."""
    key = _build.variant_name(kind, value)
    lib = _variants.get(key)
    if lib is None:
        path = _build.build_variant(kind, value)
        lib = ctypes.CDLL(str(path))
        lib.tl_variant_last_error.restype = c_char_p
        lib.tl_variant_last_error.argtypes = []
        _declare(lib, signatures)
        _variants[key] = lib
    return lib


def check(status: int, lib: Optional[ctypes.CDLL] = None, getter: str = "tl_last_error") -> None:
    if status != 0:
        lib = lib or core()
        msg = getattr(lib, getter)()
        raise KernelError(msg.decode() if msg else f"kernel status {status}")
