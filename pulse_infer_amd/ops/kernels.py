"""Python faces of the HIP entry points.

Each function checks on the host that devices, storage types, shapes and
strides are what its kernel assumes, then launches on torch's current stream.
Tensors are passed as raw device pointers; nothing here allocates unless a
result tensor is asked for, and nothing falls back to another implementation.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .library import KernelError, call

_TAG = {torch.float32: 0, torch.bfloat16: 1}


def _tag(t: torch.Tensor, what: str) -> int:
    try:
        return _TAG[t.dtype]
    except KeyError:
        raise KernelError(f"{what}: storage type {t.dtype} is not supported (float32 or bfloat16)") from None


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _i32(v: int) -> ctypes.c_int:
    return ctypes.c_int(int(v))


def _i64(v: int) -> ctypes.c_int64:
    return ctypes.c_int64(int(v))


def _f32(v: float) -> ctypes.c_float:
    return ctypes.c_float(float(v))


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> ctypes.c_void_p:
    """torch's current stream of the current device, as the raw handle the entry points take."""
    if _raw_stream is not None and _raw_device is not None:   # one C call each; a Stream object costs ten times that
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _gpu(what: str, *tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError(f"{what}: every tensor must live on the GPU, got one on {t.device}")


def _int_vec(what: str, t: torch.Tensor, n: Optional[int] = None) -> None:
    _need(t.dtype == torch.int32 and t.is_contiguous(), f"{what} must be a contiguous int32 tensor")
    if n is not None:
        _need(t.numel() >= n, f"{what} holds {t.numel()} entries, {n} are needed")


# ---------------------------------------------------------------------------
def embed_gather(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, bad_id: torch.Tensor) -> None:
    """out[t] = float32(table[ids[t]]); ``bad_id`` (int32[1]) is raised for an id outside the table."""
    _gpu("embed_gather", ids, table, out, bad_id)
    tokens = ids.numel()
    vocab, hidden = table.shape
    _int_vec("embed_gather: ids", ids)
    _need(table.is_contiguous() and out.is_contiguous(), "embed_gather: table and out must be contiguous")
    _need(out.dtype == torch.float32 and tuple(out.shape) == (tokens, hidden),
          f"embed_gather: out must be float32 [{tokens}, {hidden}], got {out.dtype} {tuple(out.shape)}")
    _need(bad_id.dtype == torch.int32 and bad_id.numel() >= 1, "embed_gather: bad_id must be int32[1]")
    call("pulse_embed_gather", _ptr(ids), _ptr(table), _i32(_tag(table, "embed_gather")), _ptr(out),
         _i32(tokens), _i32(hidden), _i32(vocab), _ptr(bad_id), _stream())


def add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None, write_back: bool = True) -> None:
    """out[r] = rmsnorm(h[s] + delta[s]) * weight, s = rows[r] or r; with write_back h[s] keeps the sum.
    ``delta`` may be float32 [parts, T, H]: the shares of a product whose inner dimension was split, added in order."""
    _gpu("add_rmsnorm", h, delta, weight, out, rows)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous(), "add_rmsnorm: h must be contiguous float32 [T, H]")
    hidden = h.shape[1]
    n_out = rows.numel() if rows is not None else h.shape[0]
    if rows is not None:
        _int_vec("add_rmsnorm: rows", rows)
        write_back = False
    parts = 1
    if delta is not None:
        if delta.dim() == 3:
            parts = delta.shape[0]
            _need(parts >= 1 and delta.shape[1:] == h.shape and delta.is_contiguous() and delta.dtype == torch.float32
                  and hidden % 4 == 0, "add_rmsnorm: an update in parts must be contiguous float32 [parts, T, H], H % 4 == 0")
        else:
            _need(delta.shape == h.shape and delta.is_contiguous(), "add_rmsnorm: delta must match h")
    _need(weight.numel() == hidden and weight.is_contiguous(), f"add_rmsnorm: weight must hold {hidden} values")
    _need(out.is_contiguous() and tuple(out.shape) == (n_out, hidden),
          f"add_rmsnorm: out must be [{n_out}, {hidden}], got {tuple(out.shape)}")
    call("pulse_add_rmsnorm", _ptr(h), _ptr(delta), _i32(_tag(delta, "add_rmsnorm") if delta is not None else 0),
         _i32(parts), _i64(h.numel()), _ptr(rows), _ptr(weight), _i32(_tag(weight, "add_rmsnorm")), _ptr(out), _i32(_tag(out, "add_rmsnorm")),
         _i32(n_out), _i32(hidden), _f32(eps), _i32(1 if (write_back and delta is not None) else 0), _stream())


def residual_add(h: torch.Tensor, delta: torch.Tensor) -> None:
    """h += delta; ``delta`` of the shape of h, or [parts, *h.shape] (added in order)."""
    _gpu("residual_add", h, delta)
    parts = delta.shape[0] if delta.dim() == h.dim() + 1 else 1
    _need(h.dtype == torch.float32 and h.is_contiguous() and delta.is_contiguous()
          and (delta.shape == h.shape or delta.shape[1:] == h.shape),
          "residual_add: h must be contiguous float32 and delta of the same shape (or several of them)")
    call("pulse_residual_add", _ptr(h), _ptr(delta), _i32(_tag(delta, "residual_add")), _i32(parts), _i64(h.numel()),
         _stream())


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, slab: int = 0) -> None:
    """out[t, i] = silu(gate) * up; gate_up holds [gate | up] halves (slab 0) or alternating slabs of ``slab`` columns."""
    _gpu("swiglu", gate_up, out)
    tokens, two_i = gate_up.shape
    _need(two_i % 2 == 0 and tuple(out.shape) == (tokens, two_i // 2), "swiglu: out must be [T, I] for gate_up [T, 2I]")
    _need(gate_up.is_contiguous() and out.is_contiguous() and gate_up.dtype == out.dtype,
          "swiglu: contiguous tensors of one storage type are needed")
    call("pulse_swiglu", _ptr(gate_up), _ptr(out), _i32(_tag(out, "swiglu")), _i32(tokens), _i32(two_i // 2),
         _i32(slab), _stream())


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, cos_out: torch.Tensor, sin_out: torch.Tensor) -> None:
    """cos/sin of position * inv_freq, computed in float64 and stored as float32 [T, half]."""
    _gpu("rope_table", positions, inv_freq, cos_out, sin_out)
    tokens, half = positions.numel(), inv_freq.numel()
    _int_vec("rope_table: positions", positions)
    _need(inv_freq.dtype == torch.float64 and inv_freq.is_contiguous(), "rope_table: inv_freq must be float64")
    for t in (cos_out, sin_out):
        _need(t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == (tokens, half),
              f"rope_table: tables must be float32 [{tokens}, {half}]")
    call("pulse_rope_table", _ptr(positions), _ptr(inv_freq), _ptr(cos_out), _ptr(sin_out), _i32(tokens), _i32(half),
         _stream())


def gather_rows(src: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> None:
    _gpu("gather_rows", src, rows, out)
    _int_vec("gather_rows: rows", rows)
    _need(src.dtype == torch.float32 and out.dtype == torch.float32 and src.is_contiguous() and out.is_contiguous()
          and out.shape[0] == rows.numel() and out.shape[1] == src.shape[1], "gather_rows: bad tensors")
    call("pulse_gather_rows", _ptr(src), _ptr(rows), _ptr(out), _i32(rows.numel()), _i32(src.shape[1]), _stream())


def gemm_f32(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """out[M, N] = a[M, K] @ w[N, K]^T with float32 fused multiply-adds in a fixed order."""
    _gpu("gemm_f32", a, w, out)
    _need(a.dim() == 2 and w.dim() == 2 and out.dim() == 2, "gemm_f32: matrices are needed")
    m, k = a.shape
    n, k2 = w.shape
    _need(k == k2, f"gemm_f32: inner sizes differ: a is [{m}, {k}], w is [{n}, {k2}]")
    _need(tuple(out.shape) == (m, n), f"gemm_f32: out must be [{m}, {n}], got {tuple(out.shape)}")
    _need(a.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1, "gemm_f32: rows must be contiguous")
    call("pulse_gemm_f32", _ptr(a), _i32(_tag(a, "gemm_f32")), _ptr(w), _i32(_tag(w, "gemm_f32")), _ptr(out),
         _i32(_tag(out, "gemm_f32")), _i32(m), _i32(n), _i32(k), _i64(a.stride(0) if m > 1 else k),
         _i64(w.stride(0) if n > 1 else k), _i64(out.stride(0) if m > 1 else n), _stream())


SKINNY_MAX_ROWS = 64           # what the kernel takes
SKINNY_FAST_ROWS = 16          # up to here it beats the vendor library on every layer shape
SKINNY_SWIGLU_MAX_ROWS = 32
_OUT_MODES = {"store": None, "add": 2}


def gemm_skinny_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the few-rows matrix-core product takes these operands."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and w.dim() == 2
            and a.shape[0] <= SKINNY_MAX_ROWS and a.shape[1] % 8 == 0 and a.stride(1) == 1 and w.stride(1) == 1
            and (a.shape[0] <= 1 or a.stride(0) % 8 == 0) and (w.shape[0] <= 1 or w.stride(0) % 8 == 0)
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_skinny_fusable(m: int, n: int, k: int) -> bool:
    """Whether the few-rows product can take its input as (residual, row sums of squares, norm weight) and leave
    row sums of squares of what it adds into (the streaming kernel's shapes)."""
    return 1 <= m <= SKINNY_FAST_ROWS and n > 0 and k > 0 and k % 1024 == 0   # as pulse_gemm_skinny_fusable


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, add: bool = False, swiglu: bool = False,
                tune: int = 0, sumsq_out: Optional[torch.Tensor] = None, row_scale: Optional[tuple] = None,
                copy_out: Optional[torch.Tensor] = None, copy_scale: Optional[torch.Tensor] = None) -> None:
    """out = a @ w^T for at most 64 rows of bfloat16, float32 accumulation on the matrix cores.

    ``out`` bfloat16 or float32 is stored; with ``add`` (float32 only) the product is added to it.  With
    ``swiglu`` the weight holds gate and up rows in alternating slabs of 16 and out is silu(gate) * up.
    ``tune`` picks a kernel variant by hand (tests and measurements); 0 lets the library choose.

    Fusions for shapes that ``gemm_skinny_fusable`` accepts.  ``row_scale = (sumsq, eps)``: row m of the product is
    multiplied by 1 / sqrt(sum(sumsq[m]) / K + eps) before it is stored or goes through SwiGLU: the division of an
    RMSNorm moved behind the product, ``sumsq`` [M, parts] being the sums of squares, in parts, of the rows that were
    normed (the norm's weight has to be in ``a`` already).  ``sumsq_out`` [M, ceil(N / 16)] with ``add``: the kernel
    also leaves the sums of squares of the rows of the updated ``out``, 16 columns a part; ``copy_out`` [M, N] bfloat16
    with ``add``: the updated ``out`` once more, every column multiplied by its ``copy_scale`` (bfloat16 [N], the weight
    of the norm that reads ``out`` next; None: as it is) and rounded: what ``row_scale`` of the next product takes.
    """
    scale_sumsq, scale_eps = row_scale if row_scale is not None else (None, 0.0)
    _gpu("gemm_skinny", a, w, out, sumsq_out, copy_out, scale_sumsq, copy_scale)
    _need(gemm_skinny_ok(a, w), "gemm_skinny: needs bfloat16 operands with at most 64 rows, K a multiple of 8, "
          "contiguous 16-byte aligned rows")
    m, k = a.shape
    ldx = a.stride(0) if m > 1 else k
    n, k2 = w.shape
    _need(k == k2, f"gemm_skinny: inner sizes differ: a is [{m}, {k}], w is [{n}, {k2}]")
    cols = n // 2 if swiglu else n
    _need(tuple(out.shape) == (m, cols) and out.stride(1) == 1, f"gemm_skinny: out must be [{m}, {cols}]")
    if add:
        _need(out.dtype == torch.float32 and not swiglu, "gemm_skinny: adding needs a float32 target")
        mode = 2
    else:
        mode = 0 if out.dtype == torch.bfloat16 else 1
        _need(out.dtype in (torch.bfloat16, torch.float32), "gemm_skinny: out must be bfloat16 or float32")
    if swiglu:
        _need(m <= SKINNY_SWIGLU_MAX_ROWS and n % 32 == 0 and out.dtype == torch.bfloat16,
              "gemm_skinny: the SwiGLU epilogue needs at most 32 rows, N a multiple of 32 and bfloat16 output")
    if sumsq_out is not None or row_scale is not None or copy_out is not None:
        _need(gemm_skinny_fusable(m, n, k), f"gemm_skinny: M={m} N={n} K={k} cannot take the fused kernel")
    if sumsq_out is not None:
        _need(add and sumsq_out.dtype == torch.float32 and sumsq_out.is_contiguous() and sumsq_out.dim() == 2
              and sumsq_out.shape[0] >= m and sumsq_out.shape[1] == (n + 15) // 16,
              "gemm_skinny: sumsq_out must be a contiguous float32 [M, ceil(N / 16)] and comes with add")
    if copy_out is not None:
        _need(add and copy_out.dtype == torch.bfloat16 and tuple(copy_out.shape) == (m, n) and copy_out.stride(1) == 1,
              f"gemm_skinny: copy_out must be bfloat16 [{m}, {n}] and comes with add")
    ldcopy = 0 if copy_out is None else (copy_out.stride(0) if m > 1 else n)
    _need(copy_scale is None or (copy_out is not None and copy_scale.dtype == torch.bfloat16 and copy_scale.numel() == n
                                 and copy_scale.is_contiguous()),
          f"gemm_skinny: copy_scale must hold {n} bfloat16 values and comes with copy_out")
    scale_parts = 0
    if scale_sumsq is not None:
        _need(scale_sumsq.dtype == torch.float32 and scale_sumsq.dim() == 2 and scale_sumsq.shape[0] >= m
              and scale_sumsq.is_contiguous() and scale_sumsq.shape[1] > 0 and scale_sumsq.data_ptr() % 16 == 0,
              "gemm_skinny: the row sums of squares must be a contiguous, 16-byte aligned float32 [M, parts]")
        scale_parts = scale_sumsq.shape[1]
    call("pulse_gemm_skinny_fused", _ptr(a), _i64(ldx), _ptr(w), _i64(w.stride(0) if n > 1 else k), _ptr(out),
         _i64(out.stride(0) if m > 1 else cols), _i32(m), _i32(n), _i32(k), _i32(mode), _i32(1 if swiglu else 0),
         _i32(tune), _ptr(scale_sumsq), _i32(scale_parts), _f32(scale_eps), _ptr(sumsq_out), _ptr(copy_out),
         _i64(ldcopy), _ptr(copy_scale), _stream(), label=f"N={n} K={k}")


ROWS_MAX_ROWS = 64
ROWS_CHUNK = 256


def gemm_rows_takes(m: int, n: int, k: int) -> bool:
    """Whether ``gemm_rows`` takes a shape (as pulse_gemm_rows_takes)."""
    return 1 <= m <= ROWS_MAX_ROWS and n > 0 and n % 16 == 0 and k > 0 and k % ROWS_CHUNK == 0


def gemm_rows(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, add: bool = False,
              sumsq_out: Optional[torch.Tensor] = None, row_scale: Optional[tuple] = None,
              copy_out: Optional[torch.Tensor] = None, copy_scale: Optional[torch.Tensor] = None, slabs: int = 0) -> None:
    """out = a @ w^T for up to 64 rows of bfloat16 and a weight of few rows: a workgroup owns 16 weight rows and all
    of K, its four wavefronts share K out among themselves (the regime of 17 to 64 rows for the projections around
    attention and the feed-forward's way back).

    ``out`` bfloat16 [M, N] is stored; with ``add`` the product is added to ``out`` float32 [M, N].  The fusions are
    those of ``gemm_skinny``: ``row_scale = (sumsq, eps)`` multiplies row m of the product by
    1 / sqrt(sum(sumsq[m]) / K + eps) first; with ``add``, ``sumsq_out`` [M, N / 16] takes the sums of squares of the
    updated rows, 16 columns a part, and ``copy_out`` [M, N] bfloat16 the updated rows once more, every column
    multiplied by its ``copy_scale`` (bfloat16 [N]; None: as it is)."""
    scale_sumsq, scale_eps = row_scale if row_scale is not None else (None, 0.0)
    _gpu("gemm_rows", a, w, out, sumsq_out, copy_out, scale_sumsq, copy_scale)
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and w.dim() == 2
          and a.stride(1) == 1 and w.stride(1) == 1, "gemm_rows: a and w must be bfloat16 matrices with contiguous rows")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k, f"gemm_rows: inner sizes differ ({k} and {w.shape[1]})")
    _need(gemm_rows_takes(m, n, k), f"gemm_rows: M={m} N={n} K={k} is not a shape it takes")
    _need(tuple(out.shape) == (m, n) and out.stride(1) == 1, f"gemm_rows: out must be [{m}, {n}]")
    if add:
        _need(out.dtype == torch.float32, "gemm_rows: adding needs a float32 target")
        mode = 2
    else:
        _need(out.dtype == torch.bfloat16 and sumsq_out is None and copy_out is None,
              "gemm_rows: a stored result is bfloat16; sums of squares and the copy come with add")
        mode = 0
    if sumsq_out is not None:
        _need(sumsq_out.dtype == torch.float32 and sumsq_out.is_contiguous() and sumsq_out.dim() == 2
              and sumsq_out.shape[0] >= m and sumsq_out.shape[1] == n // 16,
              "gemm_rows: sumsq_out must be a contiguous float32 [M, N / 16]")
    if copy_out is not None:
        _need(copy_out.dtype == torch.bfloat16 and tuple(copy_out.shape) == (m, n) and copy_out.stride(1) == 1,
              f"gemm_rows: copy_out must be bfloat16 [{m}, {n}]")
    ldcopy = 0 if copy_out is None else (copy_out.stride(0) if m > 1 else n)
    _need(copy_scale is None or (copy_out is not None and copy_scale.dtype == torch.bfloat16 and copy_scale.numel() == n
                                 and copy_scale.is_contiguous()),
          f"gemm_rows: copy_scale must hold {n} bfloat16 values and comes with copy_out")
    scale_parts = 0
    if scale_sumsq is not None:
        _need(scale_sumsq.dtype == torch.float32 and scale_sumsq.dim() == 2 and scale_sumsq.shape[0] >= m
              and scale_sumsq.is_contiguous() and scale_sumsq.shape[1] > 0 and scale_sumsq.data_ptr() % 16 == 0,
              "gemm_rows: the row sums of squares must be a contiguous, 16-byte aligned float32 [M, parts]")
        scale_parts = scale_sumsq.shape[1]
    call("pulse_gemm_rows", _ptr(a), _i64(a.stride(0) if m > 1 else k), _ptr(w), _i64(w.stride(0) if n > 1 else k),
         _ptr(out), _i64(out.stride(0) if m > 1 else n), _i32(m), _i32(n), _i32(k), _i32(mode), _ptr(scale_sumsq),
         _i32(scale_parts), _f32(scale_eps), _ptr(sumsq_out), _ptr(copy_out), _i64(ldcopy), _ptr(copy_scale),
         _i32(slabs), _stream(), label=f"N={n} K={k}")


TILE_K = 64      # k a stage of the many-rows product
TILE_ROWS = 256  # rows of X and of W an output tile


def gemm_tile_takes(m: int, n: int, k: int, swiglu: bool = False, splits: int = 1, float32: bool = False) -> bool:
    """Whether ``gemm_tile`` takes a shape (as pulse_gemm_tile_takes)."""
    if m <= 0 or n <= 0 or k <= 0 or splits < 1 or (splits > 1 and not float32) or (swiglu and float32):
        return False
    step = 32 if swiglu else (4 if float32 else 8)
    return k % (TILE_K * splits) == 0 and n % step == 0


def gemm_tile(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, swiglu: bool = False) -> None:
    """a @ w^T for many rows of bfloat16 (prompt portions): output tiles of 256 x 256 on the matrix cores, float32
    accumulation, one rounding.

    ``out`` bfloat16 [M, N]: the product; with ``swiglu`` the weight holds gate and up rows in alternating slabs of 16
    and out [M, N / 2] is silu(gate) * up.  ``out`` float32 [splits, M, N] (or [M, N]): the partial products of equal
    shares of K, which the consumer adds up in order."""
    _gpu("gemm_tile", a, w, out)
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and w.dim() == 2
          and a.stride(1) == 1 and w.stride(1) == 1, "gemm_tile: a and w must be bfloat16 matrices with contiguous rows")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k, f"gemm_tile: inner sizes differ ({k} and {w.shape[1]})")
    if out.dtype == torch.float32:
        parts = out if out.dim() == 3 else out.view(1, *out.shape)
        splits = parts.shape[0]
        _need(not swiglu and tuple(parts.shape[1:]) == (m, n) and parts.stride(2) == 1,
              f"gemm_tile: float32 results go to [shares, {m}, {n}] with contiguous rows")
        _need(gemm_tile_takes(m, n, k, splits=splits, float32=True),
              f"gemm_tile: M={m} N={n} K={k} in {splits} shares is not a shape it takes")
        mode, ldc, part_stride = 2, (parts.stride(1) if m > 1 else n), (parts.stride(0) if splits > 1 else 0)
    else:
        cols = n // 2 if swiglu else n
        _need(gemm_tile_takes(m, n, k, swiglu=swiglu), f"gemm_tile: M={m} N={n} K={k} is not a shape it takes")
        _need(out.dtype == torch.bfloat16 and out.dim() == 2 and tuple(out.shape) == (m, cols) and out.stride(1) == 1,
              f"gemm_tile: out must be bfloat16 [{m}, {cols}]")
        mode, ldc, part_stride, splits = (1 if swiglu else 0), (out.stride(0) if m > 1 else cols), 0, 1
    call("pulse_gemm_tile", _ptr(a), _i64(a.stride(0) if m > 1 else k), _ptr(w), _i64(w.stride(0) if n > 1 else k),
         _ptr(out), _i64(ldc), _i32(m), _i32(n), _i32(k), _i32(mode), _i32(splits), _i64(part_stride), _stream(),
         label=f"N={n} K={k}")


MID_MAX_ROWS = 192


def gemm_mid_takes(m: int, n: int, k: int, splits: int = 1) -> bool:
    """Whether ``gemm_mid`` takes a shape (as pulse_gemm_mid_takes)."""
    return 1 <= m <= MID_MAX_ROWS and n > 0 and k > 0 and 1 <= splits <= 64 and k % splits == 0 and (k // splits) % 128 == 0


def gemm_mid(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, swiglu: bool = False, splits: int = 1,
             waves: int = 0) -> None:
    """a @ w^T for up to 192 rows of bfloat16 with X shared through LDS (the regime of 17 to 192 rows).

    ``out`` bfloat16 [M, N]: the product (``splits`` must be 1); with ``swiglu`` the weight holds gate and up rows in
    alternating slabs of 16 and out [M, N / 2] is silu(gate) * up.  ``out`` float32 [splits, M, N]: the partial
    products of ``splits`` equal shares of K, which the consumer adds up in order."""
    _gpu("gemm_mid", a, w, out)
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and w.dim() == 2
          and a.stride(1) == 1 and w.stride(1) == 1, "gemm_mid: a and w must be bfloat16 matrices with contiguous rows")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k, f"gemm_mid: inner sizes differ ({k} and {w.shape[1]})")
    _need(gemm_mid_takes(m, n, k, splits), f"gemm_mid: M={m} N={n} K={k} in {splits} shares is not a shape it takes")
    if out.dtype == torch.float32:
        _need(not swiglu and out.is_contiguous() and tuple(out.shape) == (splits, m, n),
              f"gemm_mid: partial sums go to a contiguous float32 [{splits}, {m}, {n}]")
        mode, ldc = 1, n
    else:
        cols = n // 2 if swiglu else n
        _need(out.dtype == torch.bfloat16 and splits == 1 and out.dim() == 2 and out.shape[0] == m
              and out.shape[1] == cols and out.stride(1) == 1, f"gemm_mid: out must be bfloat16 [{m}, {cols}]")
        mode, ldc = 0, (out.stride(0) if m > 1 else cols)
    call("pulse_gemm_mid", _ptr(a), _i64(a.stride(0) if m > 1 else k), _ptr(w), _i64(w.stride(0) if n > 1 else k),
         _ptr(out), _i64(ldc), _i32(m), _i32(n), _i32(k), _i32(mode), _i32(1 if swiglu else 0), _i32(splits), _i32(waves),
         _stream(), label=f"N={n} K={k}")


def _check_cache(what: str, kcache: torch.Tensor, vcache: torch.Tensor, nkv: int, d: int):
    _need(kcache.dim() == 4 and vcache.dim() == 4, f"{what}: caches must be [pages, kv_heads, ., .]")
    pages, h, page_size, dd = kcache.shape
    _need(h == nkv and dd == d, f"{what}: key cache is {tuple(kcache.shape)}, expected [P, {nkv}, page, {d}]")
    _need(tuple(vcache.shape) == (pages, nkv, d, page_size),
          f"{what}: value cache is {tuple(vcache.shape)}, expected {(pages, nkv, d, page_size)}")
    _need(kcache.is_contiguous() and vcache.is_contiguous() and kcache.dtype == vcache.dtype,
          f"{what}: caches must be contiguous and of one storage type")
    return pages, page_size


def qk_rope_kv(qkv: torch.Tensor, nq: int, nkv: int, d: int, q_weight: Optional[torch.Tensor],
               k_weight: Optional[torch.Tensor], eps: float, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
               rotary_dim: int, pairing: int, kcache: Optional[torch.Tensor], vcache: Optional[torch.Tensor],
               positions: torch.Tensor, token_entry: torch.Tensor, block_table: Optional[torch.Tensor],
               write_kv: bool = True) -> None:
    """Per-head norm and rotation of q (in place) and k, and the page write of k and v."""
    _gpu("qk_rope_kv", qkv, q_weight, k_weight, cos, sin, kcache, vcache, positions, token_entry, block_table)
    tokens = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.stride(1) == 1, "qk_rope_kv: qkv must be [T, columns] with contiguous rows")
    cols = (nq + 2 * nkv) * d if write_kv else nq * d
    _need(qkv.shape[1] >= cols, f"qk_rope_kv: qkv has {qkv.shape[1]} columns, {cols} are needed")
    _int_vec("qk_rope_kv: positions", positions, tokens)
    _int_vec("qk_rope_kv: token_entry", token_entry, tokens)
    w_tag = 0
    if q_weight is not None:
        _need(k_weight is not None and q_weight.numel() == d and k_weight.numel() == d
              and q_weight.dtype == k_weight.dtype and q_weight.is_contiguous() and k_weight.is_contiguous(),
              f"qk_rope_kv: the two norm weights must hold {d} values of one storage type")
        w_tag = _tag(q_weight, "qk_rope_kv")
    if cos is not None:
        half = rotary_dim // 2
        for t in (cos, sin):
            _need(t is not None and t.dtype == torch.float32 and t.is_contiguous() and t.shape[0] >= tokens
                  and t.shape[1] == half, f"qk_rope_kv: cos/sin must be float32 [T, {half}]")
    pages = page_size = width = 0
    c_tag = 0
    if write_kv:
        _need(kcache is not None and vcache is not None and block_table is not None, "qk_rope_kv: the cache is missing")
        pages, page_size = _check_cache("qk_rope_kv", kcache, vcache, nkv, d)
        _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
              "qk_rope_kv: block_table must be contiguous int32 [entries, width]")
        width = block_table.shape[1]
        c_tag = _tag(kcache, "qk_rope_kv")
    call("pulse_qk_rope_kv", _ptr(qkv), _i32(_tag(qkv, "qk_rope_kv")), _i64(qkv.stride(0)), _ptr(q_weight),
         _ptr(k_weight), _i32(w_tag), _f32(eps), _ptr(cos), _ptr(sin), _i32(rotary_dim if cos is not None else 0),
         _i32(pairing), _ptr(kcache if write_kv else None), _ptr(vcache if write_kv else None), _i32(c_tag),
         _ptr(positions), _ptr(token_entry), _ptr(block_table if write_kv else None), _i32(width), _i32(tokens),
         _i32(nq), _i32(nkv), _i32(d), _i32(page_size), _i32(pages), _i32(1 if write_kv else 0), _stream())


def attn_generic(q: torch.Tensor, out: torch.Tensor, nq: int, nkv: int, d: int, kcache: torch.Tensor,
                 vcache: torch.Tensor, positions: torch.Tensor, token_entry: torch.Tensor, block_table: torch.Tensor,
                 scale: float, window: int = 0) -> None:
    """Paged causal attention, one wavefront per (token, head), float32 arithmetic.

    ``q`` is [T, >= nq*d] (rows may be strided, e.g. the front of a fused qkv buffer); ``out`` is [T, nq*d].
    """
    _gpu("attn_generic", q, out, kcache, vcache, positions, token_entry, block_table)
    tokens = q.shape[0]
    _need(q.dim() == 2 and out.dim() == 2 and q.stride(1) == 1 and out.stride(1) == 1 and q.dtype == out.dtype,
          "attn_generic: q and out must be matrices of one storage type with contiguous rows")
    _need(q.shape[1] >= nq * d and out.shape[1] >= nq * d and out.shape[0] == tokens, "attn_generic: q/out too narrow")
    pages, page_size = _check_cache("attn_generic", kcache, vcache, nkv, d)
    _int_vec("attn_generic: positions", positions, tokens)
    _int_vec("attn_generic: token_entry", token_entry, tokens)
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
          "attn_generic: block_table must be contiguous int32 [entries, width]")
    call("pulse_attn_generic", _ptr(q), _i64(q.stride(0)), _ptr(out), _i64(out.stride(0)), _i32(_tag(q, "attn_generic")),
         _ptr(kcache), _ptr(vcache), _i32(_tag(kcache, "attn_generic")), _ptr(positions), _ptr(token_entry),
         _ptr(block_table), _i32(block_table.shape[1]), _i32(tokens), _i32(nq), _i32(nkv), _i32(d), _i32(page_size),
         _i32(pages), _f32(scale), _i32(window), _stream())


def sample(logits: torch.Tensor, out: torch.Tensor, temperature: Optional[torch.Tensor] = None,
           top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
           uniform: Optional[torch.Tensor] = None, penalty: Optional[torch.Tensor] = None,
           seen_row: Optional[torch.Tensor] = None, seen_masks: Optional[torch.Tensor] = None,
           banned: Optional[torch.Tensor] = None) -> None:
    """out[r] = next token of row r (largest logit when temperature is absent or <= 0)."""
    _gpu("sample", logits, out, temperature, top_k, top_p, uniform, penalty, seen_row, seen_masks, banned)
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1, "sample: logits must be float32 [R, V]")
    rows, vocab = logits.shape
    _int_vec("sample: out", out, rows)
    for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                        ("top_p", top_p, torch.float32), ("uniform", uniform, torch.float32),
                        ("penalty", penalty, torch.float32), ("seen_row", seen_row, torch.int32)):
        if t is not None:
            _need(t.dtype == dt and t.is_contiguous() and t.numel() >= rows, f"sample: {name} must be {dt}[{rows}]")
    words = 0
    for name, t in (("seen_masks", seen_masks), ("banned", banned)):
        if t is not None:
            _need(t.dtype == torch.int32 and t.is_contiguous(), f"sample: {name} must be contiguous int32 words")
            w = t.shape[-1]
            _need(words in (0, w), "sample: masks differ in width")
            words = w
    call("pulse_sample", _ptr(logits), _i32(rows), _i32(vocab), _i64(logits.stride(0) if rows > 1 else vocab),
         _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform), _ptr(penalty), _ptr(seen_row), _ptr(seen_masks),
         _ptr(banned), _i32(words), _ptr(out), _stream())


SAMPLE_CHUNK = 2048      # as SIMPLE_CHUNK of sampling.hip
SAMPLE_SEGMENT = 32      # as TOPK_SEGMENT of sampling.hip


def sample_chunks(vocab: int) -> int:
    """Chunks of the vocabulary that ``sample_chunked`` cuts a row into."""
    return (vocab + SAMPLE_CHUNK - 1) // SAMPLE_CHUNK


def sample_chunked_scratch(rows: int, vocab: int, device) -> dict:
    """Scratch tensors of the sizes ``sample_chunked`` asks for."""
    per_row = sample_chunks(vocab)
    f32 = lambda n: torch.empty(n, dtype=torch.float32, device=device)
    i32 = lambda n: torch.empty(n, dtype=torch.int32, device=device)
    return {"part_max": f32(rows * per_row), "part_idx": i32(rows * per_row), "part_mass": f32(rows * per_row),
            "seg_n": i32(rows * per_row), "done": i32(rows), "seg_i": i32(rows * per_row * SAMPLE_SEGMENT),
            "seg_x": f32(rows * per_row * SAMPLE_SEGMENT)}


def sample_chunked(logits: torch.Tensor, out: torch.Tensor, scratch: dict, temperature: Optional[torch.Tensor] = None,
                   top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
                   uniform: Optional[torch.Tensor] = None, penalty: Optional[torch.Tensor] = None,
                   seen_row: Optional[torch.Tensor] = None, seen_masks: Optional[torch.Tensor] = None,
                   banned: Optional[torch.Tensor] = None) -> None:
    """``sample`` in chunks of the vocabulary with a workgroup each instead of a workgroup a row: greedy rows, rows
    that draw from the whole vocabulary and rows with top-k (k at most the number of chunks) are chosen from what the
    chunks leave; rows with top-p alone, and what does not fit, go through the kernel of ``sample`` behind them.
    Which way a row goes depends on the row alone.  ``scratch`` as ``sample_chunked_scratch`` makes it."""
    names = ("part_max", "part_idx", "part_mass", "seg_i", "seg_x", "seg_n", "done")
    _gpu("sample_chunked", logits, out, temperature, top_k, top_p, uniform, penalty, seen_row, seen_masks, banned,
         *(scratch[n] for n in names))
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1,
          "sample_chunked: logits must be float32 [R, V]")
    rows, vocab = logits.shape
    _int_vec("sample_chunked: out", out, rows)
    for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                        ("top_p", top_p, torch.float32), ("uniform", uniform, torch.float32),
                        ("penalty", penalty, torch.float32), ("seen_row", seen_row, torch.int32)):
        if t is not None:
            _need(t.dtype == dt and t.is_contiguous() and t.numel() >= rows, f"sample_chunked: {name} must be {dt}[{rows}]")
    per_row = sample_chunks(vocab)
    for name, dt, need in (("part_max", torch.float32, rows * per_row), ("part_idx", torch.int32, rows * per_row),
                           ("part_mass", torch.float32, rows * per_row), ("seg_n", torch.int32, rows * per_row),
                           ("done", torch.int32, rows), ("seg_i", torch.int32, rows * per_row * SAMPLE_SEGMENT),
                           ("seg_x", torch.float32, rows * per_row * SAMPLE_SEGMENT)):
        t = scratch[name]
        _need(t.dtype == dt and t.is_contiguous() and t.numel() >= need, f"sample_chunked: {name} must hold {need} {dt}")
    words = 0
    for name, t in (("seen_masks", seen_masks), ("banned", banned)):
        if t is not None:
            _need(t.dtype == torch.int32 and t.is_contiguous(), f"sample_chunked: {name} must be contiguous int32 words")
            w = t.shape[-1]
            _need(words in (0, w), "sample_chunked: masks differ in width")
            words = w
    call("pulse_sample_chunked", _ptr(logits), _i32(rows), _i32(vocab), _i64(logits.stride(0) if rows > 1 else vocab),
         _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform), _ptr(penalty), _ptr(seen_row), _ptr(seen_masks),
         _ptr(banned), _i32(words), _ptr(scratch["part_max"]), _ptr(scratch["part_idx"]), _ptr(scratch["part_mass"]),
         _ptr(scratch["seg_i"]), _ptr(scratch["seg_x"]), _ptr(scratch["seg_n"]), _ptr(scratch["done"]), _ptr(out),
         _stream())


def argmax(logits: torch.Tensor, out: torch.Tensor, part_val: torch.Tensor, part_idx: torch.Tensor) -> None:
    """out[r] = index of the largest logit of row r, lowest index among equals (two-stage, for few rows of a wide vocabulary)."""
    _gpu("argmax", logits, out, part_val, part_idx)
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1, "argmax: logits must be float32 [R, V]")
    rows, vocab = logits.shape
    chunks = argmax_chunks(vocab)
    _int_vec("argmax: out", out, rows)
    _need(part_val.dtype == torch.float32 and part_val.numel() >= rows * chunks and part_val.is_contiguous()
          and part_idx.dtype == torch.int32 and part_idx.numel() >= rows * chunks and part_idx.is_contiguous(),
          f"argmax: scratch must hold {rows * chunks} entries")
    call("pulse_argmax", _ptr(logits), _i32(rows), _i32(vocab), _i64(logits.stride(0) if rows > 1 else vocab),
         _ptr(part_val), _ptr(part_idx), _ptr(out), _stream())


def argmax_chunks(vocab: int) -> int:
    return (vocab + 2047) // 2048


def mark_seen(masks: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor, vocab: int) -> None:
    _gpu("mark_seen", masks, rows, tokens)
    _need(masks.dtype == torch.int32 and masks.dim() == 2 and masks.is_contiguous(), "mark_seen: masks must be int32 [slots, words]")
    _int_vec("mark_seen: rows", rows)
    _int_vec("mark_seen: tokens", tokens, rows.numel())
    call("pulse_mark_seen", _ptr(masks), _i32(masks.shape[1]), _ptr(rows), _ptr(tokens), _i32(rows.numel()),
         _i32(vocab), _stream())
