"""Python faces of the HIP entry points.

Each function checks on the host that devices, storage types, shapes and
strides are what its kernel assumes, then launches on torch's current stream.
Tensors are passed as raw device pointers; nothing here allocates unless a
result tensor is asked for, and nothing falls back to another implementation.
"""
from __future__ import annotations

import ctypes
from typing import Any, Optional

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
def embed_gather(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, bad_id: torch.Tensor,
                 scale: float = 1.0) -> None:
    """out[t] = float32(table[ids[t]]) * scale; ``bad_id`` (int32[1]) is raised for an id outside the table."""
    _gpu("embed_gather", ids, table, out, bad_id)
    tokens = ids.numel()
    vocab, hidden = table.shape
    _int_vec("embed_gather: ids", ids)
    _need(table.is_contiguous() and out.is_contiguous(), "embed_gather: table and out must be contiguous")
    _need(out.dtype == torch.float32 and tuple(out.shape) == (tokens, hidden),
          f"embed_gather: out must be float32 [{tokens}, {hidden}], got {out.dtype} {tuple(out.shape)}")
    _need(bad_id.dtype == torch.int32 and bad_id.numel() >= 1, "embed_gather: bad_id must be int32[1]")
    call("pulse_embed_gather", _ptr(ids), _ptr(table), _i32(_tag(table, "embed_gather")), _ptr(out),
         _i32(tokens), _i32(hidden), _i32(vocab), _ptr(bad_id), _f32(scale), _stream())


def add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None, write_back: bool = True,
                weight_offset: float = 0.0, delta_scale: float = 1.0) -> None:
    """out[r] = rmsnorm(h[s] + delta_scale * delta[s]) * (weight_offset + weight), s = rows[r] or r; with write_back
    h[s] keeps the sum.  ``weight_offset`` is 1 for a weight stored as its distance from one (added in float32), else 0.
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
         _i32(n_out), _i32(hidden), _f32(eps), _i32(1 if (write_back and delta is not None) else 0), _f32(weight_offset),
         _f32(delta_scale), _stream())


def residual_add(h: torch.Tensor, delta: torch.Tensor, scale: float = 1.0) -> None:
    """h += scale * delta; ``delta`` of the shape of h, or [parts, *h.shape] (added in order)."""
    _gpu("residual_add", h, delta)
    parts = delta.shape[0] if delta.dim() == h.dim() + 1 else 1
    _need(h.dtype == torch.float32 and h.is_contiguous() and delta.is_contiguous()
          and (delta.shape == h.shape or delta.shape[1:] == h.shape),
          "residual_add: h must be contiguous float32 and delta of the same shape (or several of them)")
    call("pulse_residual_add", _ptr(h), _ptr(delta), _i32(_tag(delta, "residual_add")), _i32(parts), _i64(h.numel()),
         _f32(scale), _stream())


def residual_add_row(h: torch.Tensor, row: torch.Tensor) -> None:
    """h[t] += row for every row t of h [T, H]; ``row`` holds H values."""
    _gpu("residual_add_row", h, row)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous() and row.is_contiguous()
          and row.numel() == h.shape[1], "residual_add_row: h must be contiguous float32 [T, H] and row hold H values")
    call("pulse_residual_add_row", _ptr(h), _ptr(row), _i32(_tag(row, "residual_add_row")), _i64(h.numel()),
         _i32(h.shape[1]), _stream())


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def gate_code(swiglu) -> int:
    """What the products that multiply gate and up on their way out are told: 0 none, 1 silu (True), 2 the tanh form
    of gelu."""
    if not swiglu:
        return 0
    if swiglu is True or swiglu == "silu":
        return 1
    if swiglu == "gelu_tanh":
        return 2
    raise KernelError(f"a gated product knows the activations {sorted(GATE_ACTIVATIONS)}, not {swiglu!r}")


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, slab: int = 0, activation: str = "silu") -> None:
    """out[t, i] = act(gate) * up, act silu or the tanh form of gelu; gate_up holds [gate | up] halves (slab 0) or
    alternating slabs of ``slab`` columns."""
    _need(activation in GATE_ACTIVATIONS, f"swiglu: unknown activation '{activation}'")
    _gpu("swiglu", gate_up, out)
    tokens, two_i = gate_up.shape
    _need(two_i % 2 == 0 and tuple(out.shape) == (tokens, two_i // 2), "swiglu: out must be [T, I] for gate_up [T, 2I]")
    _need(gate_up.is_contiguous() and out.is_contiguous() and gate_up.dtype == out.dtype,
          "swiglu: contiguous tensors of one storage type are needed")
    call("pulse_swiglu", _ptr(gate_up), _ptr(out), _i32(_tag(out, "swiglu")), _i32(tokens), _i32(two_i // 2),
         _i32(slab), _i32(GATE_ACTIVATIONS[activation]), _stream())


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
                copy_out: Optional[torch.Tensor] = None, copy_scale: Optional[torch.Tensor] = None,
                copy_offset: float = 0.0) -> None:
    """out = a @ w^T for at most 64 rows of bfloat16, float32 accumulation on the matrix cores.

    ``out`` bfloat16 or float32 is stored; with ``add`` (float32 only) the product is added to it.  With
    ``swiglu`` the weight holds gate and up rows in alternating slabs of 16 and out is silu(gate) * up.
    ``tune`` picks a kernel variant by hand (tests and measurements); 0 lets the library choose.

    Fusions for shapes that ``gemm_skinny_fusable`` accepts.  ``row_scale = (sumsq, eps)``: row m of the product is
    multiplied by 1 / sqrt(sum(sumsq[m]) / K + eps) before it is stored or goes through SwiGLU: the division of an
    RMSNorm moved behind the product, ``sumsq`` [M, parts] being the sums of squares, in parts, of the rows that were
    normed (the norm's weight has to be in ``a`` already).  ``sumsq_out`` [M, ceil(N / 16)] with ``add``: the kernel
    also leaves the sums of squares of the rows of the updated ``out``, 16 columns a part; ``copy_out`` [M, N] bfloat16
    with ``add``: the updated ``out`` once more, every column multiplied by ``copy_offset`` + its ``copy_scale``
    (bfloat16 [N], the weight of the norm that reads ``out`` next, and what that norm adds to its weight; None: as it
    is) and rounded: what ``row_scale`` of the next product takes.
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
         _i64(out.stride(0) if m > 1 else cols), _i32(m), _i32(n), _i32(k), _i32(mode), _i32(gate_code(swiglu)),
         _i32(tune), _ptr(scale_sumsq), _i32(scale_parts), _f32(scale_eps), _ptr(sumsq_out), _ptr(copy_out),
         _i64(ldcopy), _ptr(copy_scale), _f32(copy_offset), _stream(), label=f"N={n} K={k}")


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
         _ptr(out), _i64(ldc), _i32(m), _i32(n), _i32(k), _i32(mode), _i32(gate_code(swiglu)), _i32(splits), _i32(waves),
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
               write_kv: bool = True, plain_norm: bool = False, v_head0: Optional[int] = None,
               q_temperature: Optional[tuple] = None) -> None:
    """Per-head norm and rotation of q (in place) and k, and the page write of k and v.  ``plain_norm``: q and k are
    divided by their root mean square without weights; ``v_head0``: the head number at which the values start in a
    row (default nq + nkv: behind the keys; nq: the values are the raw keys); ``q_temperature`` = (coef, every):
    q *= 1 + coef * ln(floor((position + 1) / every) + 1) after the norm."""
    _gpu("qk_rope_kv", qkv, q_weight, k_weight, cos, sin, kcache, vcache, positions, token_entry, block_table)
    tokens = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.stride(1) == 1, "qk_rope_kv: qkv must be [T, columns] with contiguous rows")
    v_head0 = nq + nkv if v_head0 is None else int(v_head0)
    cols = max(nq + nkv, v_head0 + nkv) * d if write_kv else nq * d
    _need(v_head0 >= 0 and not (plain_norm and q_weight is not None), "qk_rope_kv: bad value columns or norm options")
    temp_coef, temp_every = (float(q_temperature[0]), int(q_temperature[1])) if q_temperature is not None else (0.0, 0)
    _need(q_temperature is None or temp_every > 0, "qk_rope_kv: the query temperature's interval must be positive")
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
         _i32(nq), _i32(nkv), _i32(d), _i32(page_size), _i32(pages), _i32(1 if write_kv else 0),
         _i32(1 if plain_norm else 0), _i32(v_head0), _f32(temp_coef), _i32(temp_every), _stream())


def attn_generic(q: torch.Tensor, out: torch.Tensor, nq: int, nkv: int, d: int, kcache: torch.Tensor,
                 vcache: torch.Tensor, positions: torch.Tensor, token_entry: torch.Tensor, block_table: torch.Tensor,
                 scale: float, window: int = 0, gate: Optional[torch.Tensor] = None, gate_width: int = 0,
                 sink: Optional[torch.Tensor] = None, softcap: float = 0.0, keep_first: int = 0,
                 all_values: bool = False) -> None:
    """Paged causal attention, one wavefront per (token, head), float32 arithmetic.

    ``keep_first`` > 0 (with a window): the request's first ``keep_first`` keys stay visible below the window.
    ``all_values``: every query head's weights are applied to the values of all kv heads; ``out`` is then float32
    [T, nq * nkv * d] (head h, value head c at (h * nkv + c) * d).  ``out`` may be float32 in any case.

    ``gate_width`` > 0: the gate holds a logit for each of the first ``gate_width`` channels of every head
    ([T, nq * gate_width]) instead of one a head.  ``sink`` float32 [nq]: exp(sink[h]) is one more term of head h's
    softmax denominator.  ``softcap`` > 0: scaled scores become cap * tanh(score / cap).

    ``q`` is [T, >= nq*d] (rows may be strided, e.g. the front of a fused qkv buffer); ``out`` is [T, nq*d].
    ``gate`` [T, nq] of q's storage type (rows may be strided): head h of token t is multiplied by sigmoid(gate[t, h]).
    """
    _gpu("attn_generic", q, out, kcache, vcache, positions, token_entry, block_table)
    tokens = q.shape[0]
    out_f32 = out.dtype == torch.float32 and q.dtype != torch.float32
    _need(q.dim() == 2 and out.dim() == 2 and q.stride(1) == 1 and out.stride(1) == 1
          and (q.dtype == out.dtype or out_f32),
          "attn_generic: q and out must be matrices with contiguous rows, out of q's storage type or float32")
    _need(not all_values or (out.dtype == torch.float32 and gate is None),
          "attn_generic: all values side by side come out in float32 and ungated")
    out_width = nq * d * (nkv if all_values else 1)
    _need(q.shape[1] >= nq * d and out.shape[1] >= out_width and out.shape[0] == tokens, "attn_generic: q/out too narrow")
    _need(keep_first >= 0, "attn_generic: negative number of kept keys")
    pages, page_size = _check_cache("attn_generic", kcache, vcache, nkv, d)
    _int_vec("attn_generic: positions", positions, tokens)
    _int_vec("attn_generic: token_entry", token_entry, tokens)
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
          "attn_generic: block_table must be contiguous int32 [entries, width]")
    if gate is not None:
        _gpu("attn_generic", gate)
        _need(0 <= gate_width <= d, f"attn_generic: {gate_width} gated channels of a head of {d}")
        _need(gate.dtype == q.dtype and gate.dim() == 2 and gate.shape[0] == tokens
              and gate.shape[1] >= nq * max(1, gate_width) and gate.stride(1) == 1,
              f"attn_generic: the gate must be [{tokens}, {nq * max(1, gate_width)}] of q's storage type")
    if sink is not None:
        _gpu("attn_generic", sink)
        _need(sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == nq,
              f"attn_generic: the sinks must be float32 [{nq}]")
    gate_stride = 0 if gate is None else (gate.stride(0) if tokens > 1 else max(nq * max(1, gate_width), gate.shape[1]))
    o_stride = out.stride(0) if tokens > 1 else max(out_width, out.shape[1])
    call("pulse_attn_generic_ex", _ptr(q), _i64(q.stride(0)), _ptr(out), _i64(o_stride), _i32(_tag(q, "attn_generic")),
         _ptr(kcache), _ptr(vcache), _i32(_tag(kcache, "attn_generic")), _ptr(positions), _ptr(token_entry),
         _ptr(block_table), _i32(block_table.shape[1]), _i32(tokens), _i32(nq), _i32(nkv), _i32(d), _i32(page_size),
         _i32(pages), _f32(scale), _i32(window), _ptr(gate), _i64(gate_stride),
         _i32(gate_width if gate is not None else 0), _ptr(sink), _f32(softcap), _i32(keep_first),
         _i32(1 if all_values else 0), _i32(1 if out.dtype == torch.float32 else 0), _stream())


def attn_wide_takes(q: torch.Tensor, kcache: torch.Tensor, d: int) -> bool:
    """Whether ``attn_wide`` takes these operands: bfloat16 queries and pages, pages of a multiple of 16 keys, heads
    stored a multiple of 16 channels wide."""
    return (q.dtype == torch.bfloat16 and kcache.dtype == torch.bfloat16 and kcache.dim() == 4
            and kcache.shape[2] % 16 == 0 and d % 16 == 0)


WIDE_ROW_TILES = (1, 4)     # row tiles of 16 an item of ``attn_wide`` may have


def attn_wide_row_tiles(tokens: int) -> int:
    """Row tiles an item gets in a step of ``tokens`` tokens.  Always 1: items of 4 row tiles (every key and value
    fetched serves four times the rows, 128 value channels a workgroup) need all the registers a wavefront can have, so
    a compute unit holds a wavefront a SIMD, and a prompt of 2,048 tokens took 1.5 times as long with them (window
    attention over 8 kv heads' values 6.7 ms against 4.5 for three layers, a latent row of 576 channels 3.2 against
    2.2): what bounds this kernel is the trips to memory that a wavefront waits for, not the bytes."""
    return WIDE_ROW_TILES[0]


def attn_wide_items(entries, nq: int, nkv: int, row_tiles: int = 1):
    """The work list of ``attn_wide`` for a step's entries (anything with ``first_row`` and ``count``): items of
    16 row_tiles rows, ``hp`` heads of one kv head for 16 row_tiles // hp consecutive tokens of one entry.  Returns (flat
    list of quadruples first token, tokens, first head, heads; hp)."""
    group = nq // nkv
    hp = min(group, 16)
    tp = 16 * row_tiles // hp
    flat = []
    for e in entries:
        for t in range(0, e.count, tp):
            nt = min(tp, e.count - t)
            for a in range(nkv):
                for hb in range(0, group, hp):
                    flat.extend((e.first_row + t, nt, a * group + hb, min(hp, group - hb)))
    return flat, hp


def attn_wide(q: torch.Tensor, out: torch.Tensor, nq: int, nkv: int, d: int, wv: int, all_values: bool,
              kcache: torch.Tensor, vcache: torch.Tensor, positions: torch.Tensor, token_entry: torch.Tensor,
              block_table: torch.Tensor, items: torch.Tensor, hp: int, scale: float, window: int = 0,
              keep_first: int = 0, sink: Optional[torch.Tensor] = None, softcap: float = 0.0, row_tiles: int = 1,
              n_splits: int = 1, part: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None) -> None:
    """Paged attention on the matrix cores for heads that gather wide values: with ``all_values`` every query head's
    weights on the values of all kv heads (out float32 [T, nq * nkv * d], as ``attn_generic`` leaves it), else on its
    own kv head's (out float32 [T, nq * d]); of a head's channels the first ``wv`` (a multiple of 16) are written.
    Window, kept first keys, sinks and score cap as for ``attn_generic``."""
    _gpu("attn_wide", q, out, kcache, vcache, positions, token_entry, block_table, items, sink)
    tokens = q.shape[0]
    _need(attn_wide_takes(q, kcache, d), "attn_wide: bfloat16 operands, pages of a multiple of 16 keys, d % 16 == 0")
    _need(row_tiles in WIDE_ROW_TILES, f"attn_wide: items of {WIDE_ROW_TILES} row tiles, not {row_tiles}")
    if n_splits > 1:
        _gpu("attn_wide", part, part_ml)
        head_width = d * (nkv if all_values else 1)
        _need(part is not None and part.dtype == torch.float32 and part.is_contiguous()
              and part.numel() >= tokens * nq * n_splits * head_width, "attn_wide: the splits' scratch is too small")
        _need(part_ml is not None and part_ml.dtype == torch.float32 and part_ml.is_contiguous()
              and part_ml.numel() >= tokens * nq * n_splits * 2, "attn_wide: the splits' scratch is too small")
    width = nq * d * (nkv if all_values else 1)
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nq * d, "attn_wide: q too narrow")
    _need(out.dtype == torch.float32 and out.dim() == 2 and out.stride(1) == 1 and out.shape[0] == tokens
          and out.shape[1] >= width, f"attn_wide: out must be float32 [{tokens}, {width}]")
    pages, page_size = _check_cache("attn_wide", kcache, vcache, nkv, d)
    _int_vec("attn_wide: positions", positions, tokens)
    _int_vec("attn_wide: token_entry", token_entry, tokens)
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
          "attn_wide: block_table must be contiguous int32 [entries, width]")
    _need(items.dtype == torch.int32 and items.is_contiguous() and items.numel() % 4 == 0, "attn_wide: items are int32 quadruples")
    if sink is not None:
        _need(sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == nq, f"attn_wide: the sinks must be float32 [{nq}]")
    call("pulse_attn_wide", _ptr(q), _i64(q.stride(0) if tokens > 1 else q.shape[1]), _ptr(out),
         _i64(out.stride(0) if tokens > 1 else out.shape[1]), _ptr(kcache), _ptr(vcache), _ptr(positions), _ptr(token_entry),
         _ptr(block_table), _i32(block_table.shape[1]), _ptr(items), _i32(items.numel() // 4), _i32(hp), _i32(row_tiles),
         _i32(nq), _i32(nkv), _i32(d), _i32(wv), _i32(1 if all_values else 0), _i32(page_size), _i32(pages), _f32(scale), _i32(window),
         _i32(keep_first), _ptr(sink), _f32(softcap), _i32(n_splits), _ptr(part if n_splits > 1 else None),
         _ptr(part_ml if n_splits > 1 else None), _i32(tokens), _stream(),
         label=f"d={d} values={wv} tiles={row_tiles} splits={n_splits}")


def attn_wide_splits(n_items: int, chunks: int, keys: int) -> int:
    """Over how many workgroups ``attn_wide`` shares an item's keys out: enough that the launch has about two
    workgroups a compute unit, every one with at least four steps of 32 keys."""
    from .device import compute_units
    base = max(1, n_items * chunks)
    want = (2 * compute_units() + base - 1) // base
    return max(1, min(want, 16, keys // 128))


def head_mix(x: torch.Tensor, mix: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int, d: int, dv: int,
             out_d: int, scale: float = 1.0) -> None:
    """out[t, h, e] = scale * sum_g mix[h, g] * x[t, g, h // (heads // kv_heads), e] for e < dv, zero for dv <= e <
    out_d: the heads' attention weights mixed behind the attention kernel (x float32 [T, heads * kv_heads * d], as
    ``attn_generic`` leaves it with ``all_values``); out [T, heads * out_d], rows may be strided."""
    _gpu("head_mix", x, mix, out)
    tokens = x.shape[0]
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] == heads * kv_heads * d,
          f"head_mix: x must be contiguous float32 [{tokens}, {heads * kv_heads * d}]")
    _need(mix.is_contiguous() and tuple(mix.shape) == (heads, heads), f"head_mix: mix must be [{heads}, {heads}]")
    _need(out.dim() == 2 and out.shape[0] == tokens and out.shape[1] == heads * out_d and out.stride(1) == 1,
          f"head_mix: out must be [{tokens}, {heads * out_d}] with contiguous rows")
    stride = out.stride(0) if tokens > 1 else max(heads * out_d, out.shape[1])
    call("pulse_head_mix", _ptr(x), _ptr(mix), _i32(_tag(mix, "head_mix")), _ptr(out), _i64(stride),
         _i32(_tag(out, "head_mix")), _i32(tokens), _i32(heads), _i32(kv_heads), _i32(d), _i32(dv), _i32(out_d),
         _f32(scale), _stream())


def rotate_qk_rows(x: torch.Tensor, q0: int, k0: int, v0: int, out: torch.Tensor, heads: int, d: int, dv: int,
                   cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rotary_dim: int, pairing: int,
                   key_scale: float = 1.0) -> None:
    """out [T, 2 heads d + heads dv] float32 = q, k, v of the projection output ``x`` (columns q0, k0, v0), the first
    ``rotary_dim`` channels of every head of q and k turned by the tokens' tables, k times ``key_scale``."""
    _gpu("rotate_qk_rows", x, out, cos, sin)
    tokens = x.shape[0]
    rot = rotary_dim if cos is not None else 0
    _need(x.dim() == 2 and x.stride(1) == 1, "rotate_qk_rows: x must have contiguous rows")
    _need(out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (tokens, 2 * heads * d + heads * dv),
          f"rotate_qk_rows: out must be contiguous float32 [{tokens}, {2 * heads * d + heads * dv}]")
    if rot:
        for t in (cos, sin):
            _need(t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == (tokens, rot // 2),
                  f"rotate_qk_rows: the tables must be contiguous float32 [{tokens}, {rot // 2}]")
    stride = x.stride(0) if tokens > 1 else x.shape[1]
    call("pulse_rotate_qk_rows", _ptr(x), _i64(stride), _i32(_tag(x, "rotate_qk_rows")), _i32(q0), _i32(k0), _i32(v0),
         _ptr(out), _i32(tokens), _i32(heads), _i32(d), _i32(dv), _ptr(cos if rot else None), _ptr(sin if rot else None),
         _i32(rot), _i32(pairing), _f32(key_scale), _stream())


GATE_FORMS = {"sigmoid": 0, "silu": 1}


def group_norm_gate(o: torch.Tensor, weight: Optional[torch.Tensor], gate: Optional[torch.Tensor], out: torch.Tensor,
                    groups: int, eps: float, scale: float = 1.0, gate_form: str = "sigmoid") -> None:
    """Every one of the ``groups`` equal parts of a row of ``o`` (float32) divided by its own root mean square, times
    ``weight`` (optional, one a column), times sigmoid(gate) or silu(gate) (optional), times ``scale``; one rounding."""
    _gpu("group_norm_gate", o, weight, gate, out)
    tokens, width = o.shape
    _need(groups > 0 and width % groups == 0, f"group_norm_gate: {width} columns in {groups} groups")
    _need(gate_form in GATE_FORMS, f"group_norm_gate: a gate is one of {sorted(GATE_FORMS)}, not '{gate_form}'")
    _need(o.dtype == torch.float32 and o.stride(1) == 1, "group_norm_gate: o must be float32 with contiguous rows")
    _need(out.dim() == 2 and out.shape[0] == tokens and out.shape[1] == width and out.stride(1) == 1,
          f"group_norm_gate: out must be [{tokens}, {width}] with contiguous rows")
    _need(gate is None or (gate.shape == out.shape and gate.stride(1) == 1 and gate.dtype == out.dtype),
          "group_norm_gate: the gate must have out's shape and storage type")
    _need(weight is None or (weight.numel() == width and weight.is_contiguous()),
          f"group_norm_gate: weight must hold {width} values")
    row = lambda t: t.stride(0) if tokens > 1 else max(width, t.shape[1])
    call("pulse_group_norm_gate", _ptr(o), _i64(row(o)), _ptr(weight),
         _i32(_tag(weight, "group_norm_gate") if weight is not None else 0), _ptr(gate),
         _i64(row(gate) if gate is not None else 0), _ptr(out), _i64(row(out)), _i32(_tag(out, "group_norm_gate")),
         _i32(tokens), _i32(groups), _i32(width // groups), _f32(eps), _f32(scale), _i32(GATE_FORMS[gate_form]), _stream())


def latent_rows(x: torch.Tensor, q0: int, c0: int, q: torch.Tensor, norm_weight: torch.Tensor, cos: torch.Tensor,
                sin: torch.Tensor, pairing: int, kcache: torch.Tensor, vcache: torch.Tensor, positions: torch.Tensor,
                token_entry: torch.Tensor, block_table: torch.Tensor, heads: int, d: int, rot: int, rank: int,
                stored: int, eps: float, write: bool = True) -> None:
    """Latent attention's preparation: the normed latent row and the turned key part of every token into the pages
    (keys [pages, 1, page, stored] = [c | turned | 0], values [pages, 1, stored, page] = [c | 0]) and the queries'
    turned parts into ``q`` [T, heads * stored] at rank .. rank + rot of every head (zeros behind)."""
    _gpu("latent_rows", x, q, norm_weight, cos, sin, kcache, vcache, positions, token_entry, block_table)
    tokens = x.shape[0]
    _need(x.dim() == 2 and x.stride(1) == 1 and q.dim() == 2 and q.stride(1) == 1 and q.dtype == x.dtype
          and q.shape[0] == tokens and q.shape[1] >= heads * stored, "latent_rows: x and q must be matrices of one type")
    pages, page_size = _check_cache("latent_rows", kcache, vcache, 1, stored)
    _int_vec("latent_rows: positions", positions, tokens)
    _int_vec("latent_rows: token_entry", token_entry, tokens)
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
          "latent_rows: block_table must be contiguous int32 [entries, width]")
    _need(norm_weight.numel() == rank and norm_weight.is_contiguous(), f"latent_rows: the norm's weight must hold {rank} values")
    for t in (cos, sin):
        _need(t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == (tokens, rot // 2),
              f"latent_rows: the tables must be contiguous float32 [{tokens}, {rot // 2}]")
    call("pulse_latent_rows", _ptr(x), _i64(x.stride(0) if tokens > 1 else x.shape[1]), _i32(_tag(x, "latent_rows")),
         _i32(q0), _i32(c0), _ptr(q), _i64(q.stride(0) if tokens > 1 else q.shape[1]), _ptr(norm_weight),
         _i32(_tag(norm_weight, "latent_rows")), _ptr(cos), _ptr(sin), _i32(pairing), _ptr(kcache), _ptr(vcache),
         _i32(_tag(kcache, "latent_rows")), _ptr(positions), _ptr(token_entry), _ptr(block_table),
         _i32(block_table.shape[1]), _i32(tokens), _i32(heads), _i32(d), _i32(rot), _i32(rank), _i32(stored),
         _i32(page_size), _i32(pages), _f32(eps), _i32(1 if write else 0), _stream())


def latent_absorb(x: torch.Tensor, q0: int, q_head: int, w_uk: torch.Tensor, q: torch.Tensor, stored: int, heads: int,
                  d: int, rank: int) -> None:
    """q[t, h * stored + r] = sum_e x[t, q0 + h * q_head + e] * w_uk[h * d + e, r]: a head's plain query part taken
    into the latent space (float32 sums, one rounding)."""
    _gpu("latent_absorb", x, w_uk, q)
    tokens = x.shape[0]
    _need(x.dim() == 2 and x.stride(1) == 1 and q.dim() == 2 and q.stride(1) == 1 and q.dtype == x.dtype
          and q.shape[0] == tokens and q.shape[1] >= heads * stored, "latent_absorb: x and q must be matrices of one type")
    _need(w_uk.is_contiguous() and tuple(w_uk.shape) == (heads * d, rank), f"latent_absorb: w_uk must be [{heads * d}, {rank}]")
    call("pulse_latent_absorb", _ptr(x), _i64(x.stride(0) if tokens > 1 else x.shape[1]), _i32(_tag(x, "latent_absorb")),
         _i32(q0), _i32(q_head), _ptr(w_uk), _i32(_tag(w_uk, "latent_absorb")), _ptr(q),
         _i64(q.stride(0) if tokens > 1 else q.shape[1]), _i32(stored), _i32(tokens), _i32(heads), _i32(d), _i32(rank),
         _stream())


def latent_expand(o: torch.Tensor, stored: int, w_uv: torch.Tensor, gate: Optional[torch.Tensor], out: torch.Tensor,
                  heads: int, dv: int, rank: int, scale: float = 1.0) -> None:
    """out[t, h * dv + e] = scale * (sum_r w_uv[h * dv + e, r] * o[t, h * stored + r]) * sigmoid(gate[t, h * dv + e]):
    the heads' weighted latent rows expanded to their values, gated channel by channel; one rounding."""
    _gpu("latent_expand", o, w_uv, gate, out)
    tokens = o.shape[0]
    _need(o.dim() == 2 and o.stride(1) == 1 and o.shape[1] >= heads * stored, "latent_expand: o too narrow")
    _need(w_uv.is_contiguous() and tuple(w_uv.shape) == (heads * dv, rank), f"latent_expand: w_uv must be [{heads * dv}, {rank}]")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[0] == tokens and out.shape[1] >= heads * dv,
          "latent_expand: out too narrow")
    _need(gate is None or (gate.dtype == out.dtype and gate.dim() == 2 and gate.stride(1) == 1 and gate.shape[0] == tokens
                           and gate.shape[1] >= heads * dv), "latent_expand: the gate must be of out's type and width")
    row = lambda t: t.stride(0) if tokens > 1 else t.shape[1]
    call("pulse_latent_expand", _ptr(o), _i64(row(o)), _i32(_tag(o, "latent_expand")), _i32(stored), _ptr(w_uv),
         _i32(_tag(w_uv, "latent_expand")), _ptr(gate), _i64(row(gate) if gate is not None else 0), _ptr(out),
         _i64(row(out)), _i32(_tag(out, "latent_expand")), _i32(tokens), _i32(heads), _i32(dv), _i32(rank), _f32(scale),
         _stream())


def heads_product_takes(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, x_head: int) -> bool:
    """Whether ``heads_product`` takes these operands (bfloat16 weights and results, aligned rows)."""
    size = x.element_size()
    return (w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and x.dtype in (torch.bfloat16, torch.float32)
            and w.shape[2] % 8 == 0 and (x.stride(0) * size) % 16 == 0 and (x_head * size) % 16 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def heads_product(x: torch.Tensor, x_head: int, w: torch.Tensor, gate: Optional[torch.Tensor], out: torch.Tensor,
                  out_head: int, scale: float = 1.0) -> None:
    """out[t, h * out_head + m] = scale * (sum_k w[h, m, k] * x[t, h * x_head + k]) * sigmoid(gate[t, h * M + m]) on
    the matrix cores: a product a head (w bfloat16 [heads, M, K]; x bfloat16 or float32; gate optional, of out's type)."""
    _gpu("heads_product", x, w, gate, out)
    tokens = x.shape[0]
    heads, m_out, k_in = w.shape
    _need(heads_product_takes(x, w, out, x_head) and w.is_contiguous(), "heads_product: bfloat16 weights [heads, M, K], aligned rows")
    _need(x.dim() == 2 and x.stride(1) == 1 and x.shape[1] >= (heads - 1) * x_head + k_in, "heads_product: x too narrow")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[0] == tokens and out.shape[1] >= (heads - 1) * out_head + m_out,
          "heads_product: out too narrow")
    _need(gate is None or (gate.dtype == out.dtype and gate.dim() == 2 and gate.stride(1) == 1 and gate.shape[0] == tokens
                           and gate.shape[1] >= heads * m_out), "heads_product: the gate must be of out's type and width")
    row = lambda t: t.stride(0) if tokens > 1 else t.shape[1]
    call("pulse_heads_product", _ptr(x), _i64(row(x)), _i32(x_head), _i32(_tag(x, "heads_product")), _ptr(w), _ptr(gate),
         _i64(row(gate) if gate is not None else 0), _ptr(out), _i64(row(out)), _i32(out_head), _i32(tokens), _i32(heads),
         _i32(m_out), _i32(k_in), _f32(scale), _stream(), label=f"M={m_out} K={k_in}")


def xielu(x: torch.Tensor, out: torch.Tensor, pq: torch.Tensor) -> None:
    """out = a z^2 + z / 2 for z > 0, else b (exp(z) - 1 - z) + z / 2, a = softplus(pq[0]), b = 1/2 + softplus(pq[1])."""
    _gpu("xielu", x, out, pq)
    _need(x.shape == out.shape and x.dtype == out.dtype and x.is_contiguous() and out.is_contiguous(),
          "xielu: x and out must be contiguous and alike")
    _need(pq.numel() == 2 and pq.is_contiguous(), "xielu: the activation has two numbers")
    call("pulse_xielu", _ptr(x), _ptr(out), _i32(_tag(x, "xielu")), _i64(x.numel()), _ptr(pq), _i32(_tag(pq, "xielu")),
         _stream())


def token_gate_add(x: torch.Tensor, w: torch.Tensor, y: torch.Tensor, acc: torch.Tensor) -> None:
    """acc[t] += sigmoid(w . x[t]) * y[t]; acc float32 [T, H], x and y [T, H] of one storage type, w holds H values."""
    _gpu("token_gate_add", x, w, y, acc)
    tokens, hidden = x.shape
    _need(x.is_contiguous() and y.is_contiguous() and acc.is_contiguous() and y.shape == x.shape and y.dtype == x.dtype
          and acc.shape == x.shape and acc.dtype == torch.float32, "token_gate_add: x, y [T, H] alike, acc float32 [T, H]")
    _need(w.numel() == hidden and w.is_contiguous(), f"token_gate_add: w must hold {hidden} values")
    call("pulse_token_gate_add", _ptr(x), _ptr(w), _i32(_tag(w, "token_gate_add")), _ptr(y), _i32(_tag(x, "token_gate_add")),
         _ptr(acc), _i32(tokens), _i32(hidden), _stream())


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


# ---------------------------------------------------------------------------
# A layer whose norm comes after the sum; small element-wise kernels
ACTIVATIONS = {"relu2": 1, "gelu_tanh": 2, "silu": 3}


def scale_add_rmsnorm(h: torch.Tensor, weight: torch.Tensor, eps: float, alpha: float = 1.0,
                      delta: Optional[torch.Tensor] = None, delta2: Optional[torch.Tensor] = None,
                      column_scale: Optional[torch.Tensor] = None, copy: Optional[torch.Tensor] = None) -> None:
    """h <- rmsnorm(alpha * h + column_scale * (delta + delta2)) * weight, float32 in place; ``copy`` receives the new
    rows once more, rounded to its storage type.  The updates may be of any of the two storage types."""
    _gpu("scale_add_rmsnorm", h, weight, delta, delta2, column_scale, copy)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous(), "scale_add_rmsnorm: h must be contiguous float32 [T, H]")
    rows, hidden = h.shape
    for d in (delta, delta2, copy):
        _need(d is None or (tuple(d.shape) == (rows, hidden) and d.is_contiguous()),
              f"scale_add_rmsnorm: updates and the copy must be contiguous [{rows}, {hidden}]")
    _need(delta is not None or delta2 is None, "scale_add_rmsnorm: a second update without a first")
    _need(weight.numel() == hidden and weight.is_contiguous(), f"scale_add_rmsnorm: weight must hold {hidden} values")
    _need(column_scale is None or (column_scale.numel() == hidden and column_scale.is_contiguous()
                                   and column_scale.dtype == weight.dtype),
          f"scale_add_rmsnorm: the column factors must hold {hidden} values of the weight's storage type")
    tag = lambda t: _tag(t, "scale_add_rmsnorm") if t is not None else 0
    call("pulse_scale_add_rmsnorm", _ptr(h), _ptr(delta), _i32(tag(delta)), _ptr(delta2), _i32(tag(delta2)),
         _ptr(column_scale), _ptr(weight), _i32(tag(weight)), _ptr(copy), _i32(tag(copy)), _i32(rows), _i32(hidden),
         _f32(alpha), _f32(eps), _stream())


def activation(x: torch.Tensor, out: torch.Tensor, kind: str) -> None:
    """out = act(x) element by element: ``relu2`` (the square of relu), ``gelu_tanh``, ``silu``."""
    _gpu("activation", x, out)
    _need(kind in ACTIVATIONS, f"activation: unknown activation '{kind}' (known: {sorted(ACTIVATIONS)})")
    _need(x.shape == out.shape and x.dtype == out.dtype and x.is_contiguous() and out.is_contiguous(),
          "activation: contiguous tensors of one shape and storage type are needed")
    call("pulse_activation", _ptr(x), _ptr(out), _i32(_tag(x, "activation")), _i64(x.numel()), _i32(ACTIVATIONS[kind]),
         _stream())


def softcap(x: torch.Tensor, cap: float) -> None:
    """x <- cap * tanh(x / cap), in place on float32."""
    _gpu("softcap", x)
    _need(x.dtype == torch.float32 and x.is_contiguous() and cap > 0, "softcap: a contiguous float32 tensor and a positive cap")
    call("pulse_softcap", _ptr(x), _i64(x.numel()), _f32(cap), _stream())


def round_rows(x: torch.Tensor, out: torch.Tensor) -> None:
    """out = x (float32) in out's storage type."""
    _gpu("round_rows", x, out)
    _need(x.dtype == torch.float32 and x.shape == out.shape and x.is_contiguous() and out.is_contiguous(),
          "round_rows: a contiguous float32 tensor and a contiguous result of its shape")
    call("pulse_round_rows", _ptr(x), _ptr(out), _i32(_tag(out, "round_rows")), _i64(x.numel()), _stream())


# ---------------------------------------------------------------------------
# Attention inputs with a norm over the whole projection, biases, and keys and values of different widths
def qkv_rows(qkv: torch.Tensor, q_out: torch.Tensor, nq: int, nkv: int, d: int, dv: int, stored: int,
             biases: Optional[tuple], norm_weights: Optional[tuple], eps: float, cos: Optional[torch.Tensor],
             sin: Optional[torch.Tensor], rotary_dim: int, pairing: int, kcache: Optional[torch.Tensor],
             vcache: Optional[torch.Tensor], positions: torch.Tensor, token_entry: torch.Tensor,
             block_table: Optional[torch.Tensor], write_kv: bool = True, value_scale: float = 1.0,
             norm: Any = True) -> None:
    """q, k, v of ``qkv`` [T, nq*d + nkv*d + nkv*dv] -> biased, q and k normed over the whole row (``norm`` True, with
    ``norm_weights`` = (wq [nq*d], wk [nkv*d]) or None) or head by head without weights (``norm`` "head"), rotated; q to ``q_out`` [T, nq*stored], k and v (times
    ``value_scale``) to their pages, every head filled with zeros up to ``stored`` channels."""
    _gpu("qkv_rows", qkv, q_out, cos, sin, kcache, vcache, positions, token_entry, block_table)
    tokens = qkv.shape[0]
    cols = nq * d + (nkv * (d + dv) if write_kv else 0)
    _need(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= cols, f"qkv_rows: qkv needs {cols} contiguous columns")
    _need(q_out.dim() == 2 and q_out.stride(1) == 1 and q_out.shape[0] == tokens and q_out.shape[1] >= nq * stored
          and q_out.dtype == qkv.dtype, f"qkv_rows: q_out must be [{tokens}, {nq * stored}] of qkv's storage type")
    _int_vec("qkv_rows: positions", positions, tokens)
    _int_vec("qkv_rows: token_entry", token_entry, tokens)
    w_tag = None
    ptrs = [None] * 5
    sizes = (nq * d, nkv * d, nkv * dv, nq * d, nkv * d)
    given = list(biases or (None, None, None)) + list(norm_weights or (None, None))
    for i, (t, n) in enumerate(zip(given, sizes)):
        if t is None:
            continue
        _gpu("qkv_rows", t)
        _need(t.numel() == n and t.is_contiguous(), f"qkv_rows: a bias or norm weight must hold {n} values")
        tag = _tag(t, "qkv_rows")
        _need(w_tag is None or w_tag == tag, "qkv_rows: biases and norm weights must be of one storage type")
        w_tag = tag
        ptrs[i] = t
    if cos is not None:
        half = rotary_dim // 2
        for t in (cos, sin):
            _need(t is not None and t.dtype == torch.float32 and t.is_contiguous() and t.shape[0] >= tokens
                  and t.shape[1] == half, f"qkv_rows: cos/sin must be float32 [T, {half}]")
    pages = page_size = width = 0
    c_tag = 0
    if write_kv:
        _need(kcache is not None and vcache is not None and block_table is not None, "qkv_rows: the cache is missing")
        pages, page_size = _check_cache("qkv_rows", kcache, vcache, nkv, stored)
        _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
              "qkv_rows: block_table must be contiguous int32 [entries, width]")
        width = block_table.shape[1]
        c_tag = _tag(kcache, "qkv_rows")
    call("pulse_qkv_rows", _ptr(qkv), _i32(_tag(qkv, "qkv_rows")), _i64(qkv.stride(0)), _ptr(ptrs[0]), _ptr(ptrs[1]),
         _ptr(ptrs[2]), _ptr(ptrs[3]), _ptr(ptrs[4]), _i32(w_tag or 0), _i32(2 if norm == "head" else (1 if norm else 0)), _f32(eps), _ptr(cos),
         _ptr(sin), _i32(rotary_dim if cos is not None else 0), _i32(pairing), _ptr(q_out), _i64(q_out.stride(0)),
         _ptr(kcache if write_kv else None), _ptr(vcache if write_kv else None), _i32(c_tag), _ptr(positions),
         _ptr(token_entry), _ptr(block_table if write_kv else None), _i32(width), _i32(tokens), _i32(nq), _i32(nkv),
         _i32(d), _i32(dv), _i32(stored), _i32(page_size), _i32(pages), _i32(1 if write_kv else 0), _f32(value_scale),
         _stream())


# ---------------------------------------------------------------------------
# Linear attention with a decay per head
def lightning_row_groups(entries: int, heads: int, d: int, dv: int) -> int:
    """Over how many lanes ``lightning_scan`` shares a column's rows out: the fewest (1, 4, 16) that give the launch
    about as many wavefronts as the chip has places for."""
    from .device import compute_units
    want = 8 * compute_units()
    # (a workgroup's four wavefronts own 256 columns when a lane holds a whole column: narrower heads would leave
    # wavefronts idle, so they start at 4 lanes a column)
    choices = (1, 4, 16) if dv >= 256 else (4, 16)
    for r in choices:
        if r == 16 and d <= 32:
            break
        if entries * heads * ((dv * r + 255) // 256) * 4 >= want:
            return r
    return 16 if d > 32 else 4


def lightning_scan(x: torch.Tensor, q0: int, k0: int, v0: int, out: torch.Tensor, state: torch.Tensor,
                   decay: torch.Tensor, entry_first_row: torch.Tensor, entry_start: torch.Tensor,
                   entry_slot: torch.Tensor, heads: int, d: int, dv: int, activation: str = "silu",
                   row_groups: int = 1, pieces: Optional[torch.Tensor] = None,
                   scratch: Optional[torch.Tensor] = None, turn: Optional[tuple] = None, key_scale: float = 1.0) -> None:
    """For every entry of the step, token by token: S <- decay_h S + k v^T, out = S^T q, per head, in float32;
    S [slots, heads, d, dv] is the state of the entry's slot, zero when the entry starts at position 0.

    ``pieces`` (int32 [n, 4]: first row, tokens, entry, 1 for an entry's first piece | 2 for its last; an entry's
    pieces in order and next to each other) with ``scratch`` (float32 [n, heads, d, dv]): the entries are walked in
    these pieces, all at the same time: every piece from a zero state, then the states between the pieces from what
    each left, then every piece again with its outputs.

    ``turn`` = (cos, sin, rotary_dim, pairing): q and k are turned by the tokens' tables (float32 [T, rotary_dim / 2])
    as they are fetched, in float32 (activation "none" only); ``key_scale``: k is multiplied by it after the turn."""
    _gpu("lightning_scan", x, out, state, decay, entry_first_row, entry_start, entry_slot)
    cos = sin = None
    rot = pairing = 0
    if turn is not None and turn[0] is not None and turn[2]:
        cos, sin, rot, pairing = turn
        _gpu("lightning_scan", cos, sin)
        _need(activation == "none", "lightning_scan: q and k are turned as they are projected (activation 'none')")
        for t in (cos, sin):
            _need(t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == (x.shape[0], rot // 2),
                  f"lightning_scan: the tables must be contiguous float32 [{x.shape[0]}, {rot // 2}]")
    entries = entry_start.numel()
    _need(x.dim() == 2 and x.stride(1) == 1, "lightning_scan: x must be a matrix with contiguous rows")
    _need(out.dtype == torch.float32 and out.dim() == 2 and out.stride(1) == 1 and out.shape[0] == x.shape[0]
          and out.shape[1] >= heads * dv, f"lightning_scan: out must be float32 [{x.shape[0]}, {heads * dv}]")
    _need(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 4
          and tuple(state.shape[1:]) == (heads, d, dv), f"lightning_scan: state must be float32 [slots, {heads}, {d}, {dv}]")
    _need(decay.dtype == torch.float32 and decay.is_contiguous() and decay.numel() == heads,
          f"lightning_scan: decay must hold {heads} float32 values")
    _int_vec("lightning_scan: entry_first_row", entry_first_row, entries + 1)
    _int_vec("lightning_scan: entry_start", entry_start, entries)
    _int_vec("lightning_scan: entry_slot", entry_slot, entries)
    _need(activation in ("none", "silu"), "lightning_scan: the activation is 'none' or 'silu'")
    width = x.shape[1]
    _need(min(q0, k0, v0) >= 0 and max(q0, k0) + heads * d <= width and v0 + heads * dv <= width,
          "lightning_scan: q, k or v columns lie outside x")
    def walk(mode: int, n_pieces: int) -> None:
        call("pulse_lightning_scan_turned", _ptr(x), _i32(_tag(x, "lightning_scan")), _i64(x.stride(0)), _i32(q0), _i32(k0),
             _i32(v0), _ptr(out), _i64(out.stride(0)), _ptr(state), _i32(state.shape[0]), _ptr(decay),
             _ptr(entry_first_row), _ptr(entry_start), _ptr(entry_slot), _i32(entries), _i32(heads), _i32(d), _i32(dv),
             _i32(1 if activation == "silu" else 0), _i32(row_groups), _i32(mode), _ptr(pieces), _i32(n_pieces),
             _ptr(scratch), _ptr(cos), _ptr(sin), _i32(rot), _i32(pairing), _f32(key_scale), _stream())

    if pieces is None:
        walk(0, 0)
        return
    _gpu("lightning_scan", pieces, scratch)
    n_pieces = pieces.numel() // 4
    _need(pieces.dtype == torch.int32 and pieces.is_contiguous() and pieces.numel() == 4 * n_pieces and n_pieces > 0,
          "lightning_scan: pieces must be int32 quadruples")
    _need(scratch is not None and scratch.dtype == torch.float32 and scratch.is_contiguous()
          and scratch.numel() >= n_pieces * heads * d * dv, "lightning_scan: the scratch for the pieces' states is too small")
    walk(1, n_pieces)
    call("pulse_lightning_combine", _ptr(scratch), _ptr(state), _ptr(decay), _ptr(pieces), _i32(n_pieces), _ptr(entry_start),
         _ptr(entry_slot), _i32(heads), _i32(d), _i32(dv), _stream())
    walk(2, n_pieces)


def lightning_pieces(entries, piece_tokens: int):
    """The step's entries cut into pieces of ``piece_tokens`` tokens for ``lightning_scan`` (flat quadruples), or None
    when no entry is long enough for the walk in pieces to pay (twice ``piece_tokens``)."""
    if not any(e.count >= 2 * piece_tokens for e in entries):
        return None
    flat = []
    for index, e in enumerate(entries):
        cuts = list(range(0, e.count, piece_tokens)) if e.count >= 2 * piece_tokens else [0]
        for j, at in enumerate(cuts):
            end = cuts[j + 1] if j + 1 < len(cuts) else e.count
            flat.extend((e.first_row + at, end - at, index, (1 if j == 0 else 0) | (2 if j + 1 == len(cuts) else 0)))
    return flat


def gated_rmsnorm(o: torch.Tensor, weight: torch.Tensor, gate: Optional[torch.Tensor], out: torch.Tensor, eps: float,
                  scale: float = 1.0) -> None:
    """out = scale * o / sqrt(mean(o^2) + eps) * weight * sigmoid(gate) row by row; o float32, gate and out (rows may
    be strided) of one storage type."""
    _gpu("gated_rmsnorm", o, weight, gate, out)
    tokens, n = o.shape
    _need(o.dtype == torch.float32 and o.stride(1) == 1, "gated_rmsnorm: o must be float32 with contiguous rows")
    _need(out.dim() == 2 and out.shape[0] == tokens and out.shape[1] == n and out.stride(1) == 1,
          f"gated_rmsnorm: out must be [{tokens}, {n}] with contiguous rows")
    _need(gate is None or (gate.shape == out.shape and gate.stride(1) == 1 and gate.dtype == out.dtype),
          "gated_rmsnorm: the gate must have out's shape and storage type")
    _need(weight.numel() == n and weight.is_contiguous(), f"gated_rmsnorm: weight must hold {n} values")
    row = lambda t: t.stride(0) if tokens > 1 else max(n, t.shape[1])
    call("pulse_gated_rmsnorm", _ptr(o), _i64(row(o)), _ptr(weight), _i32(_tag(weight, "gated_rmsnorm")), _ptr(gate),
         _i64(row(gate) if gate is not None else 0), _ptr(out), _i64(row(out)), _i32(_tag(out, "gated_rmsnorm")),
         _i32(tokens), _i32(n), _f32(eps), _f32(scale), _stream())


# ---------------------------------------------------------------------------
# Routed feed-forward
ROUTER_SCORES = {"softmax": 0, "sigmoid": 1}
EXPERT_ACTIVATIONS = {"silu": 0, "clamped_swish": 1}


def moe_route(logits: torch.Tensor, correction: Optional[torch.Tensor], top: int, idx: torch.Tensor,
              weight: torch.Tensor, score: str = "softmax", renormalize: bool = True) -> None:
    """Softmax over a row of router logits, the ``top`` outputs with the largest score + correction, and their scores
    divided by their sum: idx int32 [T, top], weight float32 [T, top]."""
    _gpu("moe_route", logits, correction, idx, weight)
    tokens, n = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "moe_route: logits must be contiguous float32")
    _need(correction is None or (correction.numel() == n and correction.is_contiguous()),
          f"moe_route: the correction must hold {n} values")
    _need(idx.dtype == torch.int32 and idx.is_contiguous() and tuple(idx.shape) == (tokens, top)
          and weight.dtype == torch.float32 and weight.is_contiguous() and tuple(weight.shape) == (tokens, top),
          f"moe_route: idx int32 and weight float32 must be [{tokens}, {top}]")
    call("pulse_moe_route", _ptr(logits), _ptr(correction), _i32(_tag(correction, "moe_route") if correction is not None else 0),
         _ptr(idx), _ptr(weight), _i32(tokens), _i32(n), _i32(top), _i32(ROUTER_SCORES[score]),
         _i32(1 if renormalize else 0), _stream())


def moe_router(x: torch.Tensor, w_router: torch.Tensor, correction: Optional[torch.Tensor], top: int, idx: torch.Tensor,
               weight: torch.Tensor, score: str = "softmax", renormalize: bool = True) -> None:
    """``moe_route`` of the logits x w_router^T, which are formed in float32 inside the kernel.  ``score``: softmax
    over all outputs or a sigmoid of each; ``renormalize`` False leaves the chosen scores as the weights."""
    _need(score in ROUTER_SCORES, f"moe_router: unknown score function '{score}'")
    _gpu("moe_router", x, w_router, correction, idx, weight)
    tokens, hidden = x.shape
    n = w_router.shape[0]
    _need(x.is_contiguous() and w_router.is_contiguous() and w_router.shape[1] == hidden,
          f"moe_router: x [T, {hidden}] and the router's weight [outputs, {hidden}] must be contiguous")
    _need(correction is None or (correction.numel() == n and correction.is_contiguous()
                                 and correction.dtype == w_router.dtype),
          f"moe_router: the correction must hold {n} values of the weight's storage type")
    _need(idx.dtype == torch.int32 and idx.is_contiguous() and tuple(idx.shape) == (tokens, top)
          and weight.dtype == torch.float32 and weight.is_contiguous() and tuple(weight.shape) == (tokens, top),
          f"moe_router: idx int32 and weight float32 must be [{tokens}, {top}]")
    call("pulse_moe_router", _ptr(x), _i32(_tag(x, "moe_router")), _ptr(w_router), _ptr(correction),
         _i32(_tag(w_router, "moe_router")), _ptr(idx), _ptr(weight), _i32(tokens), _i32(hidden), _i32(n), _i32(top),
         _i32(ROUTER_SCORES[score]), _i32(1 if renormalize else 0), _stream())


def _in_weight(what: str, in_weight: Optional[torch.Tensor], tokens: int, top: int) -> None:
    if in_weight is not None:
        _gpu(what, in_weight)
        _need(in_weight.dtype == torch.float32 and in_weight.is_contiguous() and tuple(in_weight.shape) == (tokens, top),
              f"{what}: the weights on the experts' inputs must be float32 [{tokens}, {top}]")


def moe_gate_up(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, idx: torch.Tensor, act: torch.Tensor,
                in_weight: Optional[torch.Tensor] = None, activation: str = "silu", limit: float = 0.0) -> None:
    """act[(t, k)] = silu(gate_e x_t) * (up_e x_t) for e = idx[t, k] < experts; rows of identity experts are left alone.
    ``in_weight`` [T, top]: the expert is fed in_weight[t, k] * x_t.  ``activation`` "clamped_swish": with
    g = min(gate, limit) and u = clamp(up, -limit, limit), act = g * sigmoid(1.702 g) * (u + 1)."""
    _need(activation in EXPERT_ACTIVATIONS, f"moe_gate_up: unknown activation '{activation}'")
    _in_weight("moe_gate_up", in_weight, x.shape[0], idx.shape[1])
    _gpu("moe_gate_up", x, w_gate, w_up, idx, act)
    tokens, hidden = x.shape
    experts, ff, h2 = w_gate.shape
    top = idx.shape[1]
    _need(h2 == hidden and w_up.shape == w_gate.shape and w_gate.is_contiguous() and w_up.is_contiguous()
          and w_gate.dtype == w_up.dtype, "moe_gate_up: stacked weights [experts, ff, hidden] of one storage type")
    _need(x.is_contiguous() and act.is_contiguous() and act.dtype == x.dtype and tuple(act.shape) == (tokens * top, ff),
          f"moe_gate_up: act must be [{tokens * top}, {ff}] of x's storage type")
    _need(idx.dtype == torch.int32 and idx.is_contiguous() and idx.shape[0] == tokens, "moe_gate_up: idx must be int32 [T, top]")
    call("pulse_moe_gate_up", _ptr(x), _i32(_tag(x, "moe_gate_up")), _ptr(w_gate), _ptr(w_up),
         _i32(_tag(w_gate, "moe_gate_up")), _ptr(idx), _ptr(act), _i32(tokens), _i32(hidden), _i32(ff), _i32(experts),
         _i32(top), _ptr(in_weight), _i32(EXPERT_ACTIVATIONS[activation]), _f32(limit), _stream())


def moe_down(x: torch.Tensor, act: torch.Tensor, w_down: torch.Tensor, idx: torch.Tensor,
             weight: Optional[torch.Tensor], out: torch.Tensor) -> None:
    """out[t] = sum_k weight[t, k] * (down_e act[(t, k)] if e = idx[t, k] < experts else x[t]), float32; ``weight``
    None: every weight is one."""
    _gpu("moe_down", x, act, w_down, idx, weight, out)
    tokens, hidden = x.shape
    experts, h2, ff = w_down.shape
    top = idx.shape[1]
    _need(h2 == hidden and w_down.is_contiguous(), "moe_down: the stacked weight must be [experts, hidden, ff]")
    _need(x.is_contiguous() and act.is_contiguous() and act.dtype == x.dtype and tuple(act.shape) == (tokens * top, ff),
          f"moe_down: act must be [{tokens * top}, {ff}] of x's storage type")
    _need(idx.dtype == torch.int32 and idx.is_contiguous() and tuple(idx.shape) == (tokens, top)
          and (weight is None or (weight.dtype == torch.float32 and weight.is_contiguous()
                                  and tuple(weight.shape) == (tokens, top))),
          "moe_down: idx int32 and weight float32 must be [T, top]")
    _need(out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (tokens, hidden),
          f"moe_down: out must be float32 [{tokens}, {hidden}]")
    call("pulse_moe_down", _ptr(x), _ptr(act), _i32(_tag(x, "moe_down")), _ptr(w_down), _i32(_tag(w_down, "moe_down")),
         _ptr(idx), _ptr(weight), _ptr(out), _i32(tokens), _i32(hidden), _i32(ff), _i32(experts), _i32(top), _stream())


MOE_TILE_ROWS = (32, 128)   # rows of an expert's tile in the grouped products


def moe_grouped_takes(x: torch.Tensor, w_gate: torch.Tensor, w_down: torch.Tensor) -> bool:
    """Whether the experts' products run grouped on the matrix cores: bfloat16 everywhere, rows of multiples of 8."""
    experts, ff, hidden = w_gate.shape
    return (x.dtype == torch.bfloat16 and w_gate.dtype == torch.bfloat16 and w_down.dtype == torch.bfloat16
            and hidden % 8 == 0 and ff % 8 == 0 and experts <= 1024 and x.data_ptr() % 16 == 0)


def moe_max_tiles(pairs: int, experts: int, tile_rows: int) -> int:
    """The most tiles a step of ``pairs`` (token, choice) pairs can have, however they choose."""
    return (pairs + tile_rows - 1) // tile_rows + experts


def moe_grouped(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, idx: torch.Tensor,
                weight: torch.Tensor, act: torch.Tensor, y: torch.Tensor, out: torch.Tensor, scratch: torch.Tensor,
                tile_rows: int, weight_on_input: bool = False, activation: str = "silu", limit: float = 0.0) -> None:
    """out[t] = sum_k weight[t, k] * (expert idx[t, k] of x[t], or x[t] itself for an identity expert), the experts'
    products grouped by expert on the matrix cores.  ``act`` bfloat16 [T * top, ff] and ``y`` float32 [T * top, hidden]
    are scratch; ``scratch`` int32 holds 2 * T * top + 3 * moe_max_tiles + 1 entries.  ``weight_on_input``: an expert is
    fed weight * x and the results are added as they are; ``activation`` / ``limit`` as for ``moe_gate_up``."""
    _need(activation in EXPERT_ACTIVATIONS, f"moe_grouped: unknown activation '{activation}'")
    _gpu("moe_grouped", x, w_gate, w_up, w_down, idx, weight, act, y, out, scratch)
    tokens, hidden = x.shape
    experts, ff, h2 = w_gate.shape
    top = idx.shape[1]
    pairs = tokens * top
    _need(moe_grouped_takes(x, w_gate, w_down) and w_up.dtype == torch.bfloat16, "moe_grouped: bfloat16 operands with rows of multiples of 8")
    _need(tile_rows in MOE_TILE_ROWS, f"moe_grouped: tiles of {MOE_TILE_ROWS} rows")
    _need(h2 == hidden and w_up.shape == w_gate.shape and tuple(w_down.shape) == (experts, hidden, ff)
          and w_gate.is_contiguous() and w_up.is_contiguous() and w_down.is_contiguous() and x.is_contiguous(),
          "moe_grouped: stacked contiguous weights [experts, ff, hidden] and [experts, hidden, ff]")
    _need(idx.dtype == torch.int32 and idx.is_contiguous() and tuple(idx.shape) == (tokens, top)
          and weight.dtype == torch.float32 and weight.is_contiguous() and tuple(weight.shape) == (tokens, top),
          "moe_grouped: idx int32 and weight float32 must be [T, top]")
    _need(act.dtype == torch.bfloat16 and act.is_contiguous() and tuple(act.shape) == (pairs, ff)
          and y.dtype == torch.float32 and y.is_contiguous() and tuple(y.shape) == (pairs, hidden)
          and out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (tokens, hidden),
          "moe_grouped: act, y or out of the wrong shape or storage type")
    tiles = moe_max_tiles(pairs, experts, tile_rows)
    _need(scratch.dtype == torch.int32 and scratch.is_contiguous() and scratch.numel() >= 2 * pairs + 3 * tiles + 1,
          "moe_grouped: the integer scratch is too small")
    base = scratch.data_ptr()
    at = lambda n: ctypes.c_void_p(base + 4 * n)
    rank, order = at(0), at(pairs)
    t_expert, t_row0, t_rows, count = at(2 * pairs), at(2 * pairs + tiles), at(2 * pairs + 2 * tiles), at(2 * pairs + 3 * tiles)
    call("pulse_moe_group", _ptr(idx), _i32(pairs), _i32(experts), _i32(tile_rows), _i32(tiles), rank, order, t_expert,
         t_row0, t_rows, count, _stream())
    call("pulse_moe_gate_up_grouped", _ptr(x), _ptr(w_gate), _ptr(w_up), order, t_expert, t_row0, t_rows, count, _i32(tiles),
         _i32(tile_rows), _ptr(act), _i32(hidden), _i32(ff), _i32(top), _ptr(weight if weight_on_input else None),
         _i32(EXPERT_ACTIVATIONS[activation]), _f32(limit), _stream())
    call("pulse_moe_down_grouped", _ptr(act), _ptr(w_down), order, t_expert, t_row0, t_rows, count, _i32(tiles),
         _i32(tile_rows), _ptr(y), _i32(hidden), _i32(ff), _stream())
    call("pulse_moe_combine", _ptr(x), _i32(_tag(x, "moe_grouped")), _ptr(y), _ptr(idx),
         _ptr(None if weight_on_input else weight), _ptr(out),
         _i32(tokens), _i32(hidden), _i32(experts), _i32(top), _stream())


# ---------------------------------------------------------------------------
# A residual in several streams, and the layer norm that reads it
NORM_KINDS = {"layernorm": 0, "rmsnorm": 1}


def embed_streams(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, bad_id: torch.Tensor, streams: int,
                  scale: float = 1.0) -> None:
    """out[t, s] = float32(table[ids[t]]) * scale for every stream s; out float32 [T, streams * hidden]."""
    _gpu("embed_streams", ids, table, out, bad_id)
    tokens = ids.numel()
    vocab, hidden = table.shape
    _int_vec("embed_streams: ids", ids)
    _need(streams >= 1 and table.is_contiguous() and out.is_contiguous() and out.dtype == torch.float32
          and tuple(out.shape) == (tokens, streams * hidden),
          f"embed_streams: out must be contiguous float32 [{tokens}, {streams * hidden}]")
    _need(bad_id.dtype == torch.int32 and bad_id.numel() >= 1, "embed_streams: bad_id must be int32[1]")
    call("pulse_embed_streams", _ptr(ids), _ptr(table), _i32(_tag(table, "embed_streams")), _ptr(out), _i32(tokens),
         _i32(hidden), _i32(vocab), _i32(streams), _ptr(bad_id), _f32(scale), _stream())


MAX_STREAMS = 16


def streams_step(x: torch.Tensor, streams: int, update: Optional[tuple] = None, in_weight: Optional[torch.Tensor] = None,
                 norm: Optional[tuple] = None, out: Optional[torch.Tensor] = None,
                 rows: Optional[torch.Tensor] = None) -> None:
    """One pass over a residual of ``streams`` rows a token, x float32 [T, streams * H].

    ``update`` = (y [T, H], mix float32 [streams, streams] indexed [from, to], out_factors float32 [streams]):
    x_t <- sum_s mix[s, t] x_s + out_factors[t] * y, all streams at once, written back.  ``norm`` = (kind, weight,
    bias or None, eps) with ``out`` [rows, H]: u = sum_s in_weight[s] x_s (None: the plain sum) over the new streams,
    normed (kind "layernorm" or "rmsnorm") and rounded once; ``rows`` gathers, and an update of gathered rows is
    formed but not written back (the residual is then read for the last time)."""
    _gpu("streams_step", x, in_weight, out, rows)
    _need(1 <= streams <= MAX_STREAMS, f"streams_step: 1 to {MAX_STREAMS} streams, got {streams}")
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous() and x.shape[1] % streams == 0,
          "streams_step: x must be contiguous float32 [T, streams * H]")
    tokens, hidden = x.shape[0], x.shape[1] // streams
    y = mix = out_w = None
    if update is not None:
        y, mix, out_w = update
        _gpu("streams_step", y, mix, out_w)
        _need(rows is None or norm is not None, "streams_step: an update of gathered rows comes with a norm")
        _need(y.is_contiguous() and tuple(y.shape) == (tokens, hidden), f"streams_step: y must be [{tokens}, {hidden}]")
        _need(mix.dtype == torch.float32 and mix.is_contiguous() and tuple(mix.shape) == (streams, streams)
              and out_w.dtype == torch.float32 and out_w.is_contiguous() and out_w.numel() == streams,
              "streams_step: mix float32 [streams, streams] and out_factors float32 [streams]")
    if in_weight is not None:
        _need(in_weight.dtype == torch.float32 and in_weight.is_contiguous() and in_weight.numel() == streams,
              "streams_step: in_weight must be float32 [streams]")
    n_rows = tokens
    w = b = None
    kind, eps = 0, 0.0
    if norm is not None:
        name, w, b, eps = norm
        _gpu("streams_step", w, b)
        _need(name in NORM_KINDS, f"streams_step: unknown norm '{name}'")
        kind = NORM_KINDS[name]
        _need(out is not None, "streams_step: a norm needs its output")
        if rows is not None:
            _int_vec("streams_step: rows", rows)
            n_rows = rows.numel()
        _need(w.numel() == hidden and w.is_contiguous() and (b is None or (b.numel() == hidden and b.is_contiguous()
                                                                           and b.dtype == w.dtype)),
              f"streams_step: weight and bias must hold {hidden} values of one storage type")
        _need(out.is_contiguous() and tuple(out.shape) == (n_rows, hidden),
              f"streams_step: out must be [{n_rows}, {hidden}], got {tuple(out.shape)}")
        _need(hidden * 4 <= 60 * 1024, f"streams_step: rows of {hidden} values are too long")
    else:
        _need(update is not None and out is None, "streams_step: nothing to do")
    call("pulse_streams_step", _ptr(x), _i32(tokens), _i32(streams), _i32(hidden), _ptr(y),
         _i32(_tag(y, "streams_step") if y is not None else 0), _ptr(mix), _ptr(out_w), _ptr(in_weight), _ptr(rows),
         _i32(n_rows), _ptr(w), _ptr(b), _i32(_tag(w, "streams_step") if w is not None else 0), _i32(kind), _f32(eps),
         _ptr(out if norm is not None else None), _i32(_tag(out, "streams_step") if norm is not None else 0), _stream())


# ---------------------------------------------------------------------------
# Selective state-space mixer
def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                state: torch.Tensor, n_state: int, positions: torch.Tensor, token_entry: torch.Tensor,
                entry_start: torch.Tensor, entry_first_row: torch.Tensor, entry_slot: torch.Tensor, entries: int) -> None:
    """out[t, c] = silu(bias[c] + sum_j taps[c, j] * input at position p - (K - 1) + j), a convolution along each
    request's tokens; ``x`` [T, >= C] (rows may be strided), ``taps`` [C, K], ``state`` float32 [slots, C, n_state +
    K - 1], whose last K - 1 values a channel hold the inputs that came last and are moved on to this step's end."""
    _gpu("causal_conv", x, taps, bias, out, state, positions, token_entry, entry_start, entry_first_row, entry_slot)
    tokens = x.shape[0]
    channels, k = taps.shape
    _need(x.dim() == 2 and x.stride(1) == 1 and x.shape[1] >= channels and out.dim() == 2 and out.stride(1) == 1
          and tuple(out.shape) == (tokens, channels) and out.dtype == x.dtype,
          f"causal_conv: x [T, >= {channels}] and out [T, {channels}] of one storage type with contiguous rows")
    _need(taps.is_contiguous() and (bias is None or (bias.is_contiguous() and bias.numel() == channels
                                                     and bias.dtype == taps.dtype)),
          "causal_conv: taps [C, K] and bias [C] contiguous and of one storage type")
    _need(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 3 and state.shape[1] == channels
          and state.shape[2] == n_state + k - 1, f"causal_conv: state must be float32 [slots, {channels}, {n_state + k - 1}]")
    _int_vec("causal_conv: positions", positions, tokens)
    _int_vec("causal_conv: token_entry", token_entry, tokens)
    _int_vec("causal_conv: entry_start", entry_start, entries)
    _int_vec("causal_conv: entry_first_row", entry_first_row, entries + 1)
    _int_vec("causal_conv: entry_slot", entry_slot, entries)
    call("pulse_causal_conv", _ptr(x), _i64(x.stride(0) if tokens > 1 else x.shape[1]), _i32(_tag(x, "causal_conv")),
         _ptr(taps), _ptr(bias), _i32(_tag(taps, "causal_conv")), _ptr(out), _i64(out.stride(0) if tokens > 1 else channels),
         _ptr(state), _i32(state.shape[0]), _i32(n_state), _ptr(positions), _ptr(token_entry), _ptr(entry_start),
         _ptr(entry_first_row), _ptr(entry_slot), _i32(tokens), _i32(entries), _i32(channels), _i32(k), _stream())


def selective_scan(x: torch.Tensor, dt_raw: torch.Tensor, bc: torch.Tensor, b0: int, c0: int, z: Optional[torch.Tensor],
                   y: torch.Tensor, dt_bias: Optional[torch.Tensor], a_log: torch.Tensor, d_skip: Optional[torch.Tensor],
                   state: torch.Tensor, entry_start: torch.Tensor, entry_first_row: torch.Tensor,
                   entry_slot: torch.Tensor, entries: int) -> None:
    """The recurrence of a selective state-space mixer over every entry's tokens in order:
    dt = softplus(dt_raw + dt_bias); S[c, n] <- exp(dt A[c, n]) S[c, n] + dt x_c B_n with A = -exp(a_log);
    y_c = (sum_n S[c, n] C_n + d_skip_c x_c) * silu(z_c).  ``bc`` holds B at columns b0.. and C at c0.. of a row;
    ``state`` float32 [slots, C, >= N]: its first N values a channel are S (zeros for an entry that starts at 0)."""
    _gpu("selective_scan", x, dt_raw, bc, z, y, dt_bias, a_log, d_skip, state, entry_start, entry_first_row, entry_slot)
    tokens = x.shape[0]
    channels, n_state = a_log.shape
    rows2 = lambda t: t.dim() == 2 and t.stride(1) == 1 and t.shape[0] == tokens and t.dtype == x.dtype
    _need(rows2(x) and rows2(dt_raw) and rows2(bc) and rows2(y) and (z is None or rows2(z)),
          "selective_scan: x, dt_raw, bc, z and y must be matrices of one storage type with contiguous rows")
    _need(x.shape[1] >= channels and dt_raw.shape[1] >= channels and y.shape[1] >= channels
          and (z is None or z.shape[1] >= channels), f"selective_scan: rows of at least {channels} channels")
    _need(b0 >= 0 and c0 >= 0 and bc.shape[1] >= max(b0, c0) + n_state, "selective_scan: B and C lie outside their rows")
    small = [t for t in (dt_bias, d_skip) if t is not None]
    _need(a_log.is_contiguous() and all(t.is_contiguous() and t.numel() == channels and t.dtype == a_log.dtype for t in small),
          "selective_scan: a_log [C, N], dt_bias [C] and d_skip [C] contiguous and of one storage type")
    _need(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 3 and state.shape[1] == channels
          and state.shape[2] >= n_state, f"selective_scan: state must be float32 [slots, {channels}, >= {n_state}]")
    _int_vec("selective_scan: entry_start", entry_start, entries)
    _int_vec("selective_scan: entry_first_row", entry_first_row, entries + 1)
    _int_vec("selective_scan: entry_slot", entry_slot, entries)
    stride = lambda t, cols: t.stride(0) if tokens > 1 else max(cols, t.shape[1])
    call("pulse_selective_scan", _ptr(x), _i64(stride(x, channels)), _ptr(dt_raw), _i64(stride(dt_raw, channels)),
         _ptr(bc), _i64(stride(bc, bc.shape[1])), _i32(b0), _i32(c0), _ptr(z), _i64(stride(z, channels) if z is not None else 0),
         _ptr(y), _i64(stride(y, channels)), _i32(_tag(x, "selective_scan")), _ptr(dt_bias), _ptr(a_log), _ptr(d_skip),
         _i32(_tag(a_log, "selective_scan")), _ptr(state), _i32(state.shape[0]), _i32(state.shape[2]), _ptr(entry_start),
         _ptr(entry_first_row), _ptr(entry_slot), _i32(entries), _i32(channels), _i32(n_state), _stream())
