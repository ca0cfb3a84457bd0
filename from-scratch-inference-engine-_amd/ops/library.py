"""Loads the kernel library through ctypes and declares its functions.

There is no fallback: without the library every op raises ``KernelLibraryMissing``."""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_double, c_float, c_int, c_int32, c_int64, c_void_p
from typing import Optional

from ..csrc import build as _build


class KernelLibraryMissing(RuntimeError):
    pass


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or failed to launch."""


_LIB: Optional[ctypes.CDLL] = None

_P = c_void_p
_SIGNATURES = {
    "fsie_version": ([], c_int),
    "fsie_device_info": ([c_char_p, c_int, ctypes.POINTER(c_int)], c_int),
    "fsie_device_compute_units": ([], c_int),
    "fsie_embedding": ([_P, c_int, _P, _P, c_int, c_int, c_int, _P], c_int),
    "fsie_rmsnorm": ([_P, _P, _P, _P, _P, c_int, c_int, c_float, c_int, c_int, c_int, c_int, _P], c_int),
    "fsie_rmsnorm_plain": ([_P, c_int64, _P, _P, c_int64, c_int, c_int, c_int, c_float, c_int, _P], c_int),
    "fsie_zero_rows": ([_P, _P, c_int, c_int64, c_int, _P], c_int),
    "fsie_zero_pages": ([_P, _P, _P, c_int, c_int, c_int, c_int64, _P], c_int),
    "fsie_random_fill": ([_P, c_int64, ctypes.c_uint64, c_int, c_float, _P], c_int),
    "fsie_swiglu": ([_P, _P, c_int, c_int, c_int, _P], c_int),
    "fsie_residual_add": ([_P, _P, c_int64, c_int, _P], c_int),
    "fsie_bias_add": ([_P, _P, c_int, c_int, c_int, _P], c_int),
    "fsie_rope_kv_write": ([_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_int64,
                            c_int, _P], c_int),
    "fsie_rope_kv_write_table": ([_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int64, c_int, _P, c_int, _P],
                                 c_int),
    "fsie_gemm": ([_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, _P], c_int),
    "fsie_gemm_mfma_fp32": ([_P, _P, _P, _P, c_int, c_int, c_int, c_int, _P], c_int),
    "fsie_gemm_mfma_skinny": ([_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, _P], c_int),
    "fsie_gemm_mfma_skinny_rope": ([_P, _P, _P, _P, c_int, c_int, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int,
                                    c_int64, _P], c_int),
    "fsie_rope_table": ([_P, _P, c_int, c_int, _P, _P], c_int),
    "fsie_gemm_mfma_wide_slice": ([c_int, c_int], c_int),
    "fsie_gemm_mfma_wide_best_splits": ([c_int, c_int, c_int], c_int),
    "fsie_gemm_mfma_wide": ([_P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, _P], c_int),
    "fsie_gemm_mfma_wide_swiglu": ([_P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, _P], c_int),
    "fsie_gemm_mfma_wide_takes": ([c_int, c_int, c_int, c_int, c_int, c_int], c_int),
    "fsie_fragment_order_size": ([c_int, c_int], c_int64),
    "fsie_fragment_order": ([_P, _P, c_int, c_int, _P], c_int),
    "fsie_attention_scalar": ([_P, c_int64, _P, _P, _P, c_int, _P, c_int, _P, _P, c_int, c_int, c_int,
                               c_int, c_int, c_float, c_int, _P], c_int),
    "fsie_attention_mfma": ([_P, c_int64, _P, _P, _P, c_int, _P, c_int, _P, _P, c_int, c_int, c_int,
                             c_int, c_int, c_float, c_int, c_int, _P], c_int),
    "fsie_attention_mfma_qkv_ok": ([c_int, c_int], c_int),
    "fsie_attention_mfma_qkv": ([_P, c_int, c_int, _P, _P, _P, _P, _P, c_int64, _P, c_int, _P, c_int, _P, _P, c_int,
                                 c_int, c_int, c_int, c_int, c_float, c_int, _P], c_int),
    "fsie_attention_mfma_max_waves": ([c_int], c_int),
    "fsie_attention_mfma_lds_ok": ([c_int, c_int], c_int),
    "fsie_attention_mfma_lds": ([_P, c_int64, _P, _P, _P, c_int, _P, _P, c_int, _P, c_int, c_int, c_int, c_int, c_int,
                                 c_float, _P], c_int),
    "fsie_attention_mfma_tiles": ([c_int, c_int], c_int),
    "fsie_attention_merge": ([_P, _P, c_int, _P, c_int, c_int, c_int, _P], c_int),
    "fsie_attention_scalar_tile_tokens": ([c_int, c_int], c_int),
    "fsie_static_scratch_bytes": ([], c_int64),
    "fsie_attention_split_static": ([_P, c_int64, _P, _P, _P, c_int, _P, c_int, _P, c_int, c_int, _P, c_int, c_int,
                                     c_int, c_int, c_int, c_float, c_int, c_int, c_int, _P], c_int),
    "fsie_sample": ([_P, c_int, c_int, _P, _P, _P, _P, _P, _P], c_int),
}


def load(build_if_missing: bool = True) -> ctypes.CDLL:
    """The loaded library.  Builds it first when nothing is built for the present sources."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = _build.find_built()
    if path is None:
        if not build_if_missing:
            raise KernelLibraryMissing(
                "the HIP kernel library is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
        try:
            path = _build.ensure_built()
        except Exception as e:  # noqa: BLE001 - reported with its cause
            raise KernelLibraryMissing(f"the HIP kernel library could not be built: {e}") from e
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as e:
        raise KernelLibraryMissing(f"cannot load {path}: {e}") from e
    lib.fsie_last_error.argtypes = []
    lib.fsie_last_error.restype = c_char_p
    for name, (args, res) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = res
    _LIB = lib
    return lib


def loaded_path() -> Optional[str]:
    return None if _LIB is None else _LIB._name


def check(status: int) -> None:
    if status != 0:
        raise KernelError(load().fsie_last_error().decode("utf-8", "replace"))
