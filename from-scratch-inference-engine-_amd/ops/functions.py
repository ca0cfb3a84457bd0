"""Host-side checks and launches of the kernels."""

from __future__ import annotations

from typing import Optional

import torch

from .library import KernelError, check, load

F32, BF16 = 0, 1
ATTN_ITEM_INTS = 8
ATTN_MERGE_INTS = 4
GEMM_SKINNY_MAX_M = 8
GEMM_MFMA_SKINNY_MAX_M = 64
GEMM_MFMA_WIDE_MAX_M = 128  # the product that shares x through LDS, on a fragment-ordered weight
GEMM_MFMA_SKINNY_BEST_M = 16
GEMM_SPLITS = (2, 4, 8)  # slices of K that the few-rows product may leave as partial sums
GEMM_MAX_SPLITS = 16     # most slices of the product that shares x through LDS, and most that a norm adds up
GEMM_AUTO, GEMM_TILED, GEMM_SKINNY = 0, 1, 2


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16, not {dtype}")


# the current stream's handle straight from the runtime where torch offers it: the Stream object that
# torch.cuda.current_stream() builds costs some 10 us, and every kernel launch asks for it
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _need(t: torch.Tensor, name: str, dtype=None, shape=None, ndim=None) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: must be a tensor on the GPU")
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, found {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        raise KernelError(f"{name}: expected {ndim} dimensions, found shape {tuple(t.shape)}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name}: expected shape {tuple(shape)}, found {tuple(t.shape)}")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def embedding(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 rows of ``table`` [V, H] at ``ids`` (int32 [T]).  The caller has checked the ids."""
    _need(table, "embedding table", ndim=2)
    _need(ids, "embedding ids", dtype=torch.int32, ndim=1)
    v, h = table.shape
    t = ids.shape[0]
    if out is None:
        out = torch.empty((t, h), dtype=torch.float32, device=table.device)
    _need(out, "embedding out", dtype=torch.float32, shape=(t, h))
    check(load().fsie_embedding(table.data_ptr(), dtype_code(table.dtype), ids.data_ptr(), out.data_ptr(),
                                t, h, v, _stream()))
    return out


def rmsnorm(residual: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
            write_back: bool = False, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm of ``residual (+ delta)`` (float32 stream) times ``weight`` (float32).  ``delta``
    is [T, H] in ``out_dtype``, or float32 [S, T, H] with S in (2, 4, 8): partial sums that are
    added in order.  ``write_back`` stores the sum into ``residual``; ``rows`` (int32) selects rows."""
    _need(residual, "rmsnorm residual", dtype=torch.float32, ndim=2)
    t, h = residual.shape
    _need(weight, "rmsnorm weight", dtype=torch.float32, shape=(h,))
    n_parts = 0
    if delta is not None and delta.ndim == 3:
        n_parts = delta.shape[0]
        _need(delta, "rmsnorm delta parts", dtype=torch.float32, shape=(n_parts, t, h))
        if not 2 <= n_parts <= GEMM_MAX_SPLITS:
            raise KernelError(f"rmsnorm: {n_parts} partial sums; 2 to {GEMM_MAX_SPLITS} are taken")
    elif delta is not None:
        _need(delta, "rmsnorm delta", dtype=out_dtype, shape=(t, h))
    n_rows = t
    if rows is not None:
        _need(rows, "rmsnorm rows", dtype=torch.int32, ndim=1)
        n_rows = rows.shape[0]
    if out is None:
        out = torch.empty((n_rows, h), dtype=out_dtype, device=residual.device)
    _need(out, "rmsnorm out", dtype=out_dtype, shape=(n_rows, h))
    check(load().fsie_rmsnorm(residual.data_ptr(), _ptr(delta), weight.data_ptr(), out.data_ptr(), _ptr(rows),
                              n_rows, h, float(eps), dtype_code(out_dtype), int(write_back), n_parts, t, _stream()))
    return out


def rmsnorm_plain(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm of a plain tensor ``x`` [T, W] (no residual stream), float32 sums: every run of
    ``weight.shape[0]`` values of a row is normalised by itself and multiplied by ``weight``
    (float32), so a weight as long as a head normalises every head of a row.  ``x`` may be a view
    whose rows are a stride apart (the q columns of a q/k/v row); ``out`` may be ``x``."""
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dim() != 2 or x.stride(1) != 1:
        raise KernelError("rmsnorm_plain x: must be a 2-d tensor on the GPU whose rows are contiguous")
    _need(weight, "rmsnorm_plain weight", dtype=torch.float32, ndim=1)
    t, w = x.shape
    width = weight.shape[0]
    if width == 0 or w % width:
        raise KernelError(f"rmsnorm_plain: rows of {w} values are not whole runs of {width}")
    if out is None:
        out = torch.empty((t, w), dtype=x.dtype, device=x.device)
    if out.shape != x.shape or out.dtype != x.dtype or out.stride(1) != 1 or not out.is_cuda:
        raise KernelError("rmsnorm_plain out: must have the shape and type of x and contiguous rows")
    check(load().fsie_rmsnorm_plain(x.data_ptr(), x.stride(0), weight.data_ptr(), out.data_ptr(), out.stride(0), t,
                                    w // width, width, float(eps), dtype_code(x.dtype), _stream()))
    return out


def zero_rows(table: torch.Tensor, slots: torch.Tensor) -> torch.Tensor:
    """``table[slots[i]] = 0`` for every non-negative entry of ``slots`` (int32); rows are whole
    multiples of four bytes."""
    _need(table, "zero_rows table")
    _need(slots, "zero_rows slots", dtype=torch.int32, ndim=1)
    if table.dim() < 1:
        raise KernelError("zero_rows: the table needs a first dimension of slots")
    row_bytes = (table.numel() // max(table.shape[0], 1)) * table.element_size()
    if row_bytes % 4:
        raise KernelError(f"zero_rows: rows of {row_bytes} bytes are not whole 4-byte words")
    check(load().fsie_zero_rows(table.data_ptr(), slots.data_ptr(), slots.shape[0], row_bytes, table.shape[0], _stream()))
    return table


def zero_pages(pool_a: torch.Tensor, pool_b: torch.Tensor, pages: torch.Tensor) -> None:
    """Pages ``pages`` (int32, negative = none) of two pools [planes, n_pages, ...] of equal page
    size set to zero in every plane."""
    _need(pool_a, "zero_pages pool")
    _need(pool_b, "zero_pages pool", dtype=pool_a.dtype)
    _need(pages, "zero_pages pages", dtype=torch.int32, ndim=1)
    if pool_a.dim() < 3 or pool_b.dim() < 3 or pool_a.shape[:2] != pool_b.shape[:2] or pool_a[0, 0].numel() != pool_b[0, 0].numel():
        raise KernelError(f"zero_pages: pools of shapes {tuple(pool_a.shape)} and {tuple(pool_b.shape)} do not go together")
    page_bytes = pool_a[0, 0].numel() * pool_a.element_size()
    check(load().fsie_zero_pages(pool_a.data_ptr(), pool_b.data_ptr(), pages.data_ptr(), pages.shape[0], pool_a.shape[0],
                                 pool_a.shape[1], page_bytes, _stream()))


def random_fill(out: torch.Tensor, key: int, init: str, std: float = 0.0) -> torch.Tensor:
    """Fill ``out`` (float32, or int32 for ``init == 'int'``) with the counter-based random values
    of the sequence ``key``: ``std * z`` ('weight', 'bias'), ``1 + std * z`` ('norm'), 15 random
    bits ('int'); element i is a function of (key, i) alone."""
    kind = {"weight": 0, "bias": 0, "norm": 1, "int": 2}.get(init)
    if kind is None:
        raise KernelError(f"random_fill: unknown init '{init}'")
    _need(out, "random_fill out", dtype=torch.int32 if kind == 2 else torch.float32)
    check(load().fsie_random_fill(out.data_ptr(), out.numel(), int(key) & ((1 << 64) - 1), kind, float(std), _stream()))
    return out


def swiglu(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(x[:, 0::2]) * x[:, 1::2] for x [T, 2I] (gate and up interleaved)."""
    _need(x, "swiglu input", ndim=2)
    t, two_i = x.shape
    if two_i % 2:
        raise KernelError(f"swiglu: the input width {two_i} must be even")
    inter = two_i // 2
    if out is None:
        out = torch.empty((t, inter), dtype=x.dtype, device=x.device)
    _need(out, "swiglu out", dtype=x.dtype, shape=(t, inter))
    check(load().fsie_swiglu(x.data_ptr(), out.data_ptr(), t, inter, dtype_code(x.dtype), _stream()))
    return out


def residual_add(residual: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _need(residual, "residual", dtype=torch.float32)
    _need(delta, "delta", shape=residual.shape)
    check(load().fsie_residual_add(residual.data_ptr(), delta.data_ptr(), residual.numel(),
                                   dtype_code(delta.dtype), _stream()))
    return residual


def bias_add(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """y[r, :] += bias (float32) in place."""
    _need(y, "bias_add y", ndim=2)
    _need(bias, "bias", dtype=torch.float32, shape=(y.shape[1],))
    check(load().fsie_bias_add(y.data_ptr(), bias.data_ptr(), y.shape[0], y.shape[1], dtype_code(y.dtype), _stream()))
    return y


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                  inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor] = None,
                  k_pool: Optional[torch.Tensor] = None, v_pool: Optional[torch.Tensor] = None,
                  page_size: int = 0, bias: Optional[torch.Tensor] = None,
                  cos_sin: Optional[torch.Tensor] = None, parts: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotate the q and k heads of ``qkv`` [T, (n_heads + 2 n_kv) head_dim] in place by the angles
    ``positions * inv_freq`` (float64 table of rotary_dim/2 entries; ``None`` = no rotation) and
    copy k and v to the cache slots ``slots`` (int32 [T], negative = not stored) of the pools: keys
    [pages, n_kv, page_size, head_dim], values [pages, n_kv, head_dim, page_size].  ``cos_sin``
    (``rope_table`` of these positions and frequencies): where the whole head is rotated and
    head_dim is a multiple of 8, the kernel reads the angles' cosines and sines there; the table
    alone, without ``inv_freq``, says that the whole head is rotated by it.
    ``parts`` (float32 [S, T, width], only with ``cos_sin``): the projection as the partial sums of a
    product cut along its inner dimension; they are added in order, ``qkv`` is then only written: its
    q columns get the rotated q heads, k and v go to the pools alone."""
    _need(qkv, "qkv", ndim=2)
    t = qkv.shape[0]
    if qkv.shape[1] != (n_heads + 2 * n_kv) * head_dim:
        raise KernelError(f"qkv: width {qkv.shape[1]} != (heads {n_heads} + 2 * kv heads {n_kv}) * {head_dim}")
    _need(positions, "positions", dtype=torch.int32, shape=(t,))
    rotary_dim = 0
    if inv_freq is not None:
        _need(inv_freq, "inv_freq", dtype=torch.float64, ndim=1)
        rotary_dim = 2 * inv_freq.shape[0]
    elif cos_sin is not None:
        if head_dim % 8:
            raise KernelError("rope_kv_write: a table of cosines and sines alone needs a head of a multiple of 8 dimensions")
        rotary_dim = head_dim
    if bias is not None:
        _need(bias, "qkv bias", dtype=torch.float32, shape=(qkv.shape[1],))
    pool_slots = 0
    if k_pool is not None:
        if v_pool is None or slots is None:
            raise KernelError("rope_kv_write: k_pool needs v_pool and slots")
        _need(slots, "slots", dtype=torch.int32, shape=(t,))
        _need(k_pool, "k_pool", dtype=qkv.dtype, ndim=4)
        _need(v_pool, "v_pool", dtype=qkv.dtype, shape=(k_pool.shape[0], n_kv, head_dim, page_size))
        if tuple(k_pool.shape[1:]) != (n_kv, page_size, head_dim):
            raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} is not [pages, {n_kv}, {page_size}, {head_dim}]")
        pool_slots = k_pool.shape[0] * page_size
    n_parts = 0
    if parts is not None:
        if cos_sin is None or rotary_dim != head_dim or head_dim % 8:
            raise KernelError("rope_kv_write: partial sums need the table of cosines and sines and a whole head "
                              "of a multiple of 8 dimensions rotated")
        n_parts = parts.shape[0] if parts.dim() == 3 else 0
        _need(parts, "qkv partial sums", dtype=torch.float32, shape=(n_parts, t, qkv.shape[1]))
        if not 1 <= n_parts <= GEMM_MAX_SPLITS:
            raise KernelError(f"rope_kv_write: {n_parts} partial sums; 1 to {GEMM_MAX_SPLITS} are taken")
    if cos_sin is not None and rotary_dim == head_dim and head_dim % 8 == 0:
        _need(cos_sin, "cos_sin", dtype=torch.float32, shape=(t, head_dim // 2, 2))
        check(load().fsie_rope_kv_write_table(qkv.data_ptr(), cos_sin.data_ptr(), _ptr(slots), _ptr(bias),
                                              _ptr(k_pool), _ptr(v_pool), t, n_heads, n_kv, head_dim, page_size,
                                              pool_slots, dtype_code(qkv.dtype), _ptr(parts), n_parts, _stream()))
        return qkv
    check(load().fsie_rope_kv_write(qkv.data_ptr(), positions.data_ptr(), _ptr(slots), _ptr(inv_freq),
                                    _ptr(bias), _ptr(k_pool), _ptr(v_pool), t, n_heads, n_kv, head_dim, rotary_dim,
                                    page_size, pool_slots, dtype_code(qkv.dtype), _stream()))
    return qkv


def gemm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
         out_dtype: Optional[torch.dtype] = None, kind: int = GEMM_AUTO,
         out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [M, K] . weight [N, K]^T + bias [N] (float32) with float32 accumulation."""
    _need(x, "gemm x", ndim=2)
    _need(weight, "gemm weight", dtype=x.dtype, ndim=2)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"gemm: weight inner size {weight.shape[1]} does not match x's {k}")
    if bias is not None:
        _need(bias, "gemm bias", dtype=torch.float32, shape=(n,))
    out_dtype = out_dtype or x.dtype
    if out_dtype not in (x.dtype, torch.float32):
        raise KernelError(f"gemm: output {out_dtype} from {x.dtype} operands is not offered")
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    _need(out, "gemm out", dtype=out_dtype, shape=(m, n))
    check(load().fsie_gemm(x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(), m, n, k,
                           dtype_code(x.dtype), int(out_dtype == torch.float32), kind, _stream()))
    return out


def gemm_mfma_fp32(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, waves: int = 0,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [M, K] . weight [N, K]^T + bias in true float32 on the matrix cores, for up to 64 rows and K a
    multiple of 4 (the 32-bit path's decoding).  A row's sums do not depend on the other rows."""
    _need(x, "gemm x", dtype=torch.float32, ndim=2)
    _need(weight, "gemm weight", dtype=torch.float32, ndim=2)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"gemm: weight inner size {weight.shape[1]} does not match x's {k}")
    if bias is not None:
        _need(bias, "gemm bias", dtype=torch.float32, shape=(n,))
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    _need(out, "gemm out", dtype=torch.float32, shape=(m, n))
    check(load().fsie_gemm_mfma_fp32(x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(), m, n, k, waves, _stream()))
    return out


def gemm_mfma_skinny(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                     out_dtype: Optional[torch.dtype] = None, waves: int = 0, blocks: int = 0,
                     out: Optional[torch.Tensor] = None, epilogue: str = "plain", splits: int = 1) -> torch.Tensor:
    """The same product on the matrix cores for bfloat16 operands (K a multiple of 8): at most 16
    rows for a bfloat16 result, at most 64 for a float32 one.
    ``epilogue="swiglu"``: the rows of ``weight`` are gate and up interleaved and the result is
    silu(gate) * up, [M, N/2].  ``splits`` in (2, 4, 8): K is cut into that many slices and the
    result is their float32 partial sums [splits, M, N] (no bias), for ``rmsnorm`` to add up."""
    _need(x, "gemm x", dtype=torch.bfloat16, ndim=2)
    _need(weight, "gemm weight", dtype=torch.bfloat16, ndim=2)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"gemm: weight inner size {weight.shape[1]} does not match x's {k}")
    if bias is not None:
        _need(bias, "gemm bias", dtype=torch.float32, shape=(n,))
    out_dtype = out_dtype or x.dtype
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise KernelError(f"gemm: output {out_dtype} is not offered")
    if epilogue not in ("plain", "swiglu"):
        raise KernelError(f"gemm: unknown epilogue '{epilogue}'")
    if epilogue == "swiglu" and n % 2:
        raise KernelError(f"gemm: the swiglu epilogue needs an even number of weight rows, found {n}")
    n_out = n // 2 if epilogue == "swiglu" else n
    shape = (m, n_out)
    if splits != 1:
        if splits not in GEMM_SPLITS or epilogue != "plain" or bias is not None:
            raise KernelError(f"gemm: partial sums come in {GEMM_SPLITS} slices, without bias or epilogue")
        out_dtype, shape = torch.float32, (splits, m, n)
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=x.device)
    _need(out, "gemm out", dtype=out_dtype, shape=shape)
    check(load().fsie_gemm_mfma_skinny(x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(), m, n, k,
                                       int(out_dtype == torch.float32), waves, blocks, int(epilogue == "swiglu"),
                                       splits, _stream()))
    return out


class FragmentOrdered:
    """The copy of a bfloat16 matrix [rows, cols] in the order of the matrix instruction's A
    fragments (``fragment_order``): the 64 16-byte units of a block of 16 rows and 32 columns lie
    together in the order of the lanes that hold them, so that a wave's load of the weight is one
    piece of 1 KB and can be a streaming load.  ``gemm_mfma_wide`` and ``gemm_mfma_wide_swiglu``
    take it in place of the matrix."""

    __slots__ = ("data", "rows", "cols")

    def __init__(self, data: torch.Tensor, rows: int, cols: int):
        self.data, self.rows, self.cols = data, rows, cols

    @property
    def shape(self):
        return (self.rows, self.cols)


def fragment_order(weight: torch.Tensor) -> FragmentOrdered:
    """The copy of ``weight`` [N, K] (bfloat16, K a multiple of 32) in fragment order; the rows that
    fill N up to a multiple of 16 are zeros."""
    _need(weight, "fragment_order weight", dtype=torch.bfloat16, ndim=2)
    n, k = weight.shape
    size = int(load().fsie_fragment_order_size(n, k))
    if size <= 0:
        raise KernelError(f"fragment_order: the inner size {k} must be a multiple of 32")
    data = torch.empty(size, dtype=torch.bfloat16, device=weight.device)
    check(load().fsie_fragment_order(weight.data_ptr(), data.data_ptr(), n, k, _stream()))
    return FragmentOrdered(data, n, k)


def _wide_weight(weight, k: int):
    """(pointer, N, whether it is in fragment order) of a weight given to the wide products."""
    if isinstance(weight, FragmentOrdered):
        _need(weight.data, "gemm weight", dtype=torch.bfloat16, ndim=1)
        n, kw, ptr, frags = weight.rows, weight.cols, weight.data.data_ptr(), 1
    else:
        _need(weight, "gemm weight", dtype=torch.bfloat16, ndim=2)
        n, kw, ptr, frags = weight.shape[0], weight.shape[1], weight.data_ptr(), 0
    if kw != k:
        raise KernelError(f"gemm: weight inner size {kw} does not match x's {k}")
    return ptr, n, frags


def gemm_mfma_wide_takes(m: int, weight, splits: int = 1, gate_up: bool = False) -> bool:
    """Whether ``gemm_mfma_wide`` (``gate_up``: ``gemm_mfma_wide_swiglu``) takes ``m`` rows against this
    weight in ``splits`` slices: up to 64 rows wherever it takes the inner size; 65 to 128 rows only on a
    ``FragmentOrdered`` copy, for the launch shapes that have kernels of five to eight tiles of rows."""
    n, k = weight.shape
    return bool(load().fsie_gemm_mfma_wide_takes(int(m), int(n), int(k), int(splits), int(gate_up),
                                                 int(isinstance(weight, FragmentOrdered))))


def gemm_mfma_wide_splits_ok(k: int, splits: int) -> bool:
    """Whether ``gemm_mfma_wide`` can cut an inner size ``k`` into ``splits`` slices (whole stages
    of 128 values each)."""
    return load().fsie_gemm_mfma_wide_slice(int(k), int(splits)) > 0


def gemm_mfma_wide_swiglu(x: torch.Tensor, weight: torch.Tensor, waves: int = 0, blocks: int = 0,
                          out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(gate) * up [M, N/2] (bfloat16) of x [M, K] and a weight [N, K] whose rows are gate and up
    in turn (or its ``FragmentOrdered`` copy), by the kernel that shares x through LDS; up to 64
    rows, N a multiple of 4, K of 128."""
    _need(x, "gemm x", dtype=torch.bfloat16, ndim=2)
    m, k = x.shape
    wptr, n, frags = _wide_weight(weight, k)
    if n % 4:
        raise KernelError(f"gemm_mfma_wide_swiglu: the number of weight rows {n} must be a multiple of 4")
    if out is None:
        out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    _need(out, "gemm out", dtype=torch.bfloat16, shape=(m, n // 2))
    check(load().fsie_gemm_mfma_wide_swiglu(x.data_ptr(), wptr, out.data_ptr(), m, n, k, waves, blocks, frags,
                                            _stream()))
    return out


def gemm_mfma_wide_best_splits(m: int, n: int, k: int) -> int:
    """Into how many slices of K ``gemm_mfma_wide`` best cuts a product of ``m`` rows that leaves
    partial sums (1: it does not cut, or does not take this K)."""
    return int(load().fsie_gemm_mfma_wide_best_splits(int(m), int(n), int(k)))


def gemm_mfma_wide(x: torch.Tensor, weight: torch.Tensor, splits: int = 1, waves: int = 0,
                   out: Optional[torch.Tensor] = None, blocks: int = 0) -> torch.Tensor:
    """x [M, K] . weight [N, K]^T for bfloat16 operands and up to 64 rows, the rows of x shared by
    a workgroup's waves through LDS (made for 17 rows and more); ``weight`` may be the matrix's
    ``FragmentOrdered`` copy.  The result is float32: [M, N],
    or with ``splits`` of 2 to 16 the partial sums [splits, M, N] of the slices of K, for
    ``rmsnorm`` to add up.  K must be a multiple of 128 that the slices cover in whole stages
    (``gemm_mfma_wide_splits_ok``)."""
    _need(x, "gemm x", dtype=torch.bfloat16, ndim=2)
    m, k = x.shape
    wptr, n, frags = _wide_weight(weight, k)
    if not 1 <= splits <= GEMM_MAX_SPLITS:
        raise KernelError(f"gemm_mfma_wide: splits must be 1 to {GEMM_MAX_SPLITS}, got {splits}")
    shape = (m, n) if splits == 1 else (splits, m, n)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32, device=x.device)
    _need(out, "gemm out", dtype=torch.float32, shape=shape)
    check(load().fsie_gemm_mfma_wide(x.data_ptr(), wptr, out.data_ptr(), m, n, k, splits, waves, blocks, frags,
                                     _stream()))
    return out


def gemm_mfma_skinny_rope(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                          positions: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                          inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor] = None,
                          k_pool: Optional[torch.Tensor] = None, v_pool: Optional[torch.Tensor] = None,
                          page_size: int = 0, cos_sin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The fused q/k/v projection x [M, K] . weight [(n_heads + 2 n_kv) head_dim, K]^T of at most 64
    rows (bfloat16) with the position encoding in its epilogue: bias, rotation of the q and k
    heads over the whole head (``inv_freq``: float64 [head_dim / 2], ``None`` = none) and the
    write of k and v into the cache pools at ``slots``.  ``cos_sin``: what ``rope_table`` made of
    these positions and frequencies (the kernel then reads the cosines and sines instead of
    computing them; the table may come without ``inv_freq``).  Returns [M, N] whose q columns are filled; the k and v columns are not
    written."""
    _need(x, "gemm x", dtype=torch.bfloat16, ndim=2)
    _need(weight, "gemm weight", dtype=torch.bfloat16, ndim=2)
    m, k = x.shape
    n = (n_heads + 2 * n_kv) * head_dim
    if tuple(weight.shape) != (n, k):
        raise KernelError(f"gemm: weight shape {tuple(weight.shape)} is not [{n}, {k}]")
    if bias is not None:
        _need(bias, "qkv bias", dtype=torch.float32, shape=(n,))
    _need(positions, "positions", dtype=torch.int32, shape=(m,))
    if inv_freq is not None:
        _need(inv_freq, "inv_freq", dtype=torch.float64, shape=(head_dim // 2,))
    if cos_sin is not None:
        _need(cos_sin, "cos_sin", dtype=torch.float32, shape=(m, head_dim // 2, 2))
    pool_slots = 0
    if k_pool is not None:
        if v_pool is None or slots is None:
            raise KernelError("gemm_mfma_skinny_rope: k_pool needs v_pool and slots")
        _need(slots, "slots", dtype=torch.int32, shape=(m,))
        _need(k_pool, "k_pool", dtype=torch.bfloat16, ndim=4)
        _need(v_pool, "v_pool", dtype=torch.bfloat16, shape=(k_pool.shape[0], n_kv, head_dim, page_size))
        if tuple(k_pool.shape[1:]) != (n_kv, page_size, head_dim):
            raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} is not [pages, {n_kv}, {page_size}, {head_dim}]")
        pool_slots = k_pool.shape[0] * page_size
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    check(load().fsie_gemm_mfma_skinny_rope(x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(), m, k,
                                            positions.data_ptr(), _ptr(slots), _ptr(inv_freq), _ptr(cos_sin),
                                            _ptr(k_pool), _ptr(v_pool), n_heads, n_kv, head_dim, page_size, pool_slots,
                                            _stream()))
    return out


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """float32 [T, half, 2]: cos and sin of positions[t] * inv_freq[i] (the angle in float64, as in
    the kernels that rotate).  The angles of a step are the same in every layer: a step makes the
    table once."""
    _need(positions, "positions", dtype=torch.int32, ndim=1)
    _need(inv_freq, "inv_freq", dtype=torch.float64, ndim=1)
    t, half = positions.shape[0], inv_freq.shape[0]
    table = torch.empty((t, half, 2), dtype=torch.float32, device=positions.device)
    check(load().fsie_rope_table(positions.data_ptr(), inv_freq.data_ptr(), t, half, table.data_ptr(), _stream()))
    return table


def attention_tile_tokens(n_heads: int, n_kv: int) -> int:
    n = load().fsie_attention_scalar_tile_tokens(n_heads, n_kv)
    if n <= 0:
        raise KernelError(f"attention: heads {n_heads} must be a positive multiple of kv heads {n_kv}")
    return n


def attention_scalar(q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                     block_tables: torch.Tensor, items: torch.Tensor, n_items: int, out: torch.Tensor,
                     partials: Optional[torch.Tensor], n_heads: int, n_kv: int, head_dim: int,
                     window: Optional[int], scale: float, n_query_rows: int) -> torch.Tensor:
    """Attention of the work items over the paged cache (float32 arithmetic).

    ``q`` is a view into rows of stride ``q_stride`` elements whose first n_heads*head_dim columns
    are the queries; ``out`` is [n_query_rows, n_heads*head_dim]."""
    if not q.is_cuda:
        raise KernelError("attention q: must be on the GPU")
    _need(k_pool, "k_pool", dtype=q.dtype, ndim=4)
    _need(v_pool, "v_pool", dtype=q.dtype, shape=(k_pool.shape[0], k_pool.shape[1], k_pool.shape[3], k_pool.shape[2]))
    _need(block_tables, "block_tables", dtype=torch.int32, ndim=2)
    _need(items, "attention items", dtype=torch.int32, ndim=2)
    if items.shape[1] != ATTN_ITEM_INTS or items.shape[0] < n_items:
        raise KernelError(f"attention items: shape {tuple(items.shape)} does not hold {n_items} items")
    _need(out, "attention out", dtype=q.dtype, shape=(n_query_rows, n_heads * head_dim))
    pages, kvh, page_size, hd = k_pool.shape
    if kvh != n_kv or hd != head_dim:
        raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} does not match kv heads {n_kv}, head_dim {head_dim}")
    if q_stride < n_heads * head_dim:
        raise KernelError("attention: q_stride is smaller than the query width")
    if partials is not None:
        _need(partials, "attention partials", dtype=torch.float32, ndim=1)
    check(load().fsie_attention_scalar(q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                                       block_tables.data_ptr(), block_tables.shape[1], items.data_ptr(),
                                       n_items, out.data_ptr(), _ptr(partials), n_heads, n_kv, head_dim,
                                       page_size, int(window or 0), float(scale), dtype_code(q.dtype), _stream()))
    return out


def attention_mfma_rows(head_dim: int, large: bool) -> int:
    """Query rows (tokens x heads of a kv head's group) that one work item of the matrix-core
    attention holds; 0 if the head size is not offered."""
    return 16 * load().fsie_attention_mfma_tiles(head_dim, int(large))


def compute_units() -> int:
    """Compute units of the current device; 0 where there is none to ask."""
    return load().fsie_device_compute_units()


def attention_mfma_max_waves(head_dim: int) -> int:
    return load().fsie_attention_mfma_max_waves(head_dim)


def attention_mfma(q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                   block_tables: torch.Tensor, items: torch.Tensor, n_items: int, out: torch.Tensor,
                   partials: Optional[torch.Tensor], n_heads: int, n_kv: int, head_dim: int,
                   window: Optional[int], scale: float, n_query_rows: int, large: bool, waves: int = 1) -> torch.Tensor:
    """Attention of the work items over the paged cache on the matrix cores (bfloat16; head_dim a
    multiple of 16; page size a multiple of 4).  ``items`` may be a view into a longer table.
    ``waves`` waves of a workgroup split each item's keys and combine inside the workgroup."""
    if not q.is_cuda or q.dtype != torch.bfloat16:
        raise KernelError("attention_mfma q: must be bfloat16 on the GPU")
    _need(k_pool, "k_pool", dtype=q.dtype, ndim=4)
    _need(v_pool, "v_pool", dtype=q.dtype, shape=(k_pool.shape[0], k_pool.shape[1], k_pool.shape[3], k_pool.shape[2]))
    _need(block_tables, "block_tables", dtype=torch.int32, ndim=2)
    _need(items, "attention items", dtype=torch.int32, ndim=2)
    if items.shape[1] != ATTN_ITEM_INTS or items.shape[0] < n_items:
        raise KernelError(f"attention items: shape {tuple(items.shape)} does not hold {n_items} items")
    _need(out, "attention out", dtype=q.dtype, shape=(n_query_rows, n_heads * head_dim))
    pages, kvh, page_size, hd = k_pool.shape
    if kvh != n_kv or hd != head_dim:
        raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} does not match kv heads {n_kv}, head_dim {head_dim}")
    if q_stride < n_heads * head_dim:
        raise KernelError("attention: q_stride is smaller than the query width")
    if partials is not None:
        _need(partials, "attention partials", dtype=torch.float32, ndim=1)
    check(load().fsie_attention_mfma(q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                                     block_tables.data_ptr(), block_tables.shape[1], items.data_ptr(), n_items,
                                     out.data_ptr(), _ptr(partials), n_heads, n_kv, head_dim, page_size,
                                     int(window or 0), float(scale), int(large), int(waves), _stream()))
    return out


def attention_mfma_qkv_ok(head_dim: int, page_size: int) -> bool:
    """Whether the attention kernel that finishes the q/k/v product itself takes this geometry."""
    return bool(load().fsie_attention_mfma_qkv_ok(head_dim, page_size))


def attention_mfma_qkv(sums: torch.Tensor, bias: Optional[torch.Tensor], cos_sin: torch.Tensor, slots: torch.Tensor,
                       k_pool: torch.Tensor, v_pool: torch.Tensor, block_tables: torch.Tensor, items: torch.Tensor,
                       n_items: int, out: torch.Tensor, partials: Optional[torch.Tensor], n_heads: int, n_kv: int,
                       head_dim: int, window: Optional[int], scale: float, waves: int = 1) -> torch.Tensor:
    """Attention of a step of one token a request (every item: one query row a head) from the q/k/v
    product's float32 partial sums [S, T, (heads + 2 kv heads) head_dim]: the kernel adds them up, adds
    ``bias``, rotates queries and keys by ``cos_sin`` [T, head_dim / 2, 2], scores each request's new key
    from registers and writes it and the value to ``slots[t]`` of the pools (negative: nowhere)."""
    width = (n_heads + 2 * n_kv) * head_dim
    _need(sums, "q/k/v sums", dtype=torch.float32, ndim=3)
    n_parts, t = sums.shape[0], sums.shape[1]
    if sums.shape[2] != width or t < 1:
        raise KernelError(f"q/k/v sums: shape {tuple(sums.shape)} does not hold rows of {width}")
    if bias is not None:
        _need(bias, "q/k/v bias", dtype=torch.float32, shape=(width,))
    _need(cos_sin, "cos_sin", dtype=torch.float32)
    if cos_sin.numel() != t * head_dim:
        raise KernelError(f"cos_sin: {cos_sin.numel()} values for {t} tokens of head_dim {head_dim}")
    _need(slots, "slots", dtype=torch.int32, shape=(t,))
    _need(k_pool, "k_pool", dtype=torch.bfloat16, ndim=4)
    _need(v_pool, "v_pool", dtype=torch.bfloat16,
          shape=(k_pool.shape[0], k_pool.shape[1], k_pool.shape[3], k_pool.shape[2]))
    _need(block_tables, "block_tables", dtype=torch.int32, ndim=2)
    _need(items, "attention items", dtype=torch.int32, ndim=2)
    if items.shape[1] != ATTN_ITEM_INTS or items.shape[0] < n_items:
        raise KernelError(f"attention items: shape {tuple(items.shape)} does not hold {n_items} items")
    _need(out, "attention out", dtype=torch.bfloat16, shape=(t, n_heads * head_dim))
    pages, kvh, page_size, hd = k_pool.shape
    if kvh != n_kv or hd != head_dim:
        raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} does not match kv heads {n_kv}, head_dim {head_dim}")
    if partials is not None:
        _need(partials, "attention partials", dtype=torch.float32, ndim=1)
    check(load().fsie_attention_mfma_qkv(sums.data_ptr(), n_parts, t, _ptr(bias), cos_sin.data_ptr(), slots.data_ptr(),
                                         k_pool.data_ptr(), v_pool.data_ptr(), pages * page_size,
                                         block_tables.data_ptr(), block_tables.shape[1], items.data_ptr(), n_items,
                                         out.data_ptr(), _ptr(partials), n_heads, n_kv, head_dim, page_size,
                                         int(window or 0), float(scale), int(waves), _stream()))
    return out


def attention_mfma_lds_ok(head_dim: int, page_size: int) -> bool:
    """Whether the kernel that shares a block of keys among four waves takes this geometry."""
    return bool(load().fsie_attention_mfma_lds_ok(head_dim, page_size))


def attention_mfma_lds(q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                       block_tables: torch.Tensor, items: torch.Tensor, groups: torch.Tensor, n_groups: int,
                       out: torch.Tensor, n_heads: int, n_kv: int, head_dim: int, window: Optional[int], scale: float,
                       n_query_rows: int) -> torch.Tensor:
    """Attention of large work items (long portions) with the keys and values of a block staged in
    LDS for four tiles at once.  ``groups`` int32 [n, 2]: index in ``items`` of a group's first
    tile and its number of tiles (1..4, consecutive tiles of one request)."""
    if not q.is_cuda or q.dtype != torch.bfloat16:
        raise KernelError("attention_mfma_lds q: must be bfloat16 on the GPU")
    _need(k_pool, "k_pool", dtype=q.dtype, ndim=4)
    _need(v_pool, "v_pool", dtype=q.dtype, shape=(k_pool.shape[0], k_pool.shape[1], k_pool.shape[3], k_pool.shape[2]))
    _need(block_tables, "block_tables", dtype=torch.int32, ndim=2)
    _need(items, "attention items", dtype=torch.int32, ndim=2)
    _need(groups, "attention groups", dtype=torch.int32, ndim=2)
    if items.shape[1] != ATTN_ITEM_INTS or groups.shape[1] != 2 or groups.shape[0] < n_groups:
        raise KernelError(f"attention: items {tuple(items.shape)} / groups {tuple(groups.shape)} do not hold {n_groups} groups")
    _need(out, "attention out", dtype=q.dtype, shape=(n_query_rows, n_heads * head_dim))
    pages, kvh, page_size, hd = k_pool.shape
    if kvh != n_kv or hd != head_dim:
        raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} does not match kv heads {n_kv}, head_dim {head_dim}")
    if q_stride < n_heads * head_dim:
        raise KernelError("attention: q_stride is smaller than the query width")
    check(load().fsie_attention_mfma_lds(q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                                         block_tables.data_ptr(), block_tables.shape[1], items.data_ptr(),
                                         groups.data_ptr(), n_groups, out.data_ptr(), n_heads, n_kv, head_dim,
                                         page_size, int(window or 0), float(scale), _stream()))
    return out


def attention_merge(partials: torch.Tensor, merges: torch.Tensor, n_merges: int, out: torch.Tensor,
                    n_heads: int, head_dim: int) -> torch.Tensor:
    _need(partials, "attention partials", dtype=torch.float32, ndim=1)
    _need(merges, "attention merges", dtype=torch.int32, ndim=2)
    if merges.shape[1] != ATTN_MERGE_INTS or merges.shape[0] < n_merges:
        raise KernelError(f"attention merges: shape {tuple(merges.shape)} does not hold {n_merges} items")
    _need(out, "attention out", ndim=2)
    check(load().fsie_attention_merge(partials.data_ptr(), merges.data_ptr(), n_merges, out.data_ptr(),
                                      n_heads, head_dim, dtype_code(out.dtype), _stream()))
    return out


def sample(logits: torch.Tensor, temperature: Optional[torch.Tensor] = None,
           top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
           uniform: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token id per row of float32 ``logits`` [n, V]: argmax where temperature <= 0 (or no
    temperatures are given), else temperature/top-k/top-p sampling against ``uniform`` (float64)."""
    _need(logits, "logits", dtype=torch.float32, ndim=2)
    n, v = logits.shape
    if temperature is not None:
        _need(temperature, "temperature", dtype=torch.float32, shape=(n,))
        if uniform is None:
            raise KernelError("sample: temperatures need uniform numbers")
        _need(uniform, "uniform", dtype=torch.float64, shape=(n,))
    if top_k is not None:
        _need(top_k, "top_k", dtype=torch.int32, shape=(n,))
    if top_p is not None:
        _need(top_p, "top_p", dtype=torch.float32, shape=(n,))
    if out is None:
        out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _need(out, "sample out", dtype=torch.int32, shape=(n,))
    check(load().fsie_sample(logits.data_ptr(), n, v, _ptr(temperature), _ptr(top_k), _ptr(top_p),
                             _ptr(uniform), out.data_ptr(), _stream()))
    return out
