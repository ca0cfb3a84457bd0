"""The hand-written kernels as functions over torch tensors.

Each function checks on the host that the operands have the shapes, types and contiguity that the
kernel and its grid assume, then queues the kernel on torch's current stream.  Nothing here
computes with torch; a missing kernel library is an error, not a reason to fall back.
"""

from .functions import (FragmentOrdered, attention_merge, attention_mfma, attention_mfma_lds, attention_mfma_lds_ok,
                        attention_mfma_max_waves, attention_mfma_qkv, attention_mfma_qkv_ok, attention_mfma_rows, attention_scalar,
                        attention_tile_tokens, bias_add, compute_units, dtype_code, embedding, fragment_order, gemm, gemm_mfma_fp32, gemm_mfma_skinny,
                        gemm_mfma_skinny_rope, gemm_mfma_wide, gemm_mfma_wide_best_splits, gemm_mfma_wide_splits_ok,
                        gemm_mfma_wide_swiglu, gemm_mfma_wide_takes, random_fill,
                        residual_add,
                        rmsnorm, rmsnorm_plain, rope_kv_write, rope_table, sample, swiglu, zero_pages, zero_rows)
from .library import KernelError, KernelLibraryMissing, load
from .tuning import disable_library_tuning, enable_library_tuning, library_mm, library_tuning_enabled

__all__ = ["FragmentOrdered", "KernelError", "KernelLibraryMissing", "attention_merge", "attention_mfma", "attention_mfma_lds",
           "attention_mfma_lds_ok", "attention_mfma_max_waves", "attention_mfma_qkv", "attention_mfma_qkv_ok", "attention_mfma_rows", "attention_scalar",
           "attention_tile_tokens", "bias_add", "compute_units", "disable_library_tuning", "dtype_code", "embedding",
           "enable_library_tuning", "fragment_order", "gemm", "gemm_mfma_fp32", "gemm_mfma_skinny", "gemm_mfma_skinny_rope", "gemm_mfma_wide",
           "gemm_mfma_wide_best_splits", "gemm_mfma_wide_splits_ok", "gemm_mfma_wide_swiglu", "gemm_mfma_wide_takes", "library_mm", "library_tuning_enabled", "load", "random_fill", "residual_add",
           "rmsnorm", "rmsnorm_plain", "rope_kv_write", "rope_table", "sample", "swiglu", "zero_pages", "zero_rows"]
