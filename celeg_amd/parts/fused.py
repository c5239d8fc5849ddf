"""Helpers of the fused path for steps of few rows (decode and small portions).

A step of up to 64 rows is bound by the number of dependent kernels, so the parts
fold their neighbours into their matrix products (``HipOps.fused_linear``): the norm in
front of a product is applied to the rows of the 32-bit residual stream as they are
read, and a product that ends a sub-block adds its result into the stream itself.
Whoever writes the stream this way also leaves partial sums of squares of its rows
("stream statistics"), which the next norm reads instead of walking the rows again.

``rt.stream_stat_blocks`` says how many partial sums are valid (0: none; the prologue
then recomputes the sums).  Anything else that writes the stream resets it to 0.
"""
from __future__ import annotations

import torch

STAT_COLUMNS = 64   # most rows of a fused step (rows of the partial-sum table)
# Most rows of the fused path: 64 where every inner size is a multiple of 32 (the kernel
# for 9 to 64 rows); else 32, above which the library's product (with separate norm and
# activation kernels) is the faster one on MI355X.
FUSED_MAX_ROWS = 64
FUSED_MAX_ROWS_OLD_KERNEL = 32


TILED_MAX_STAT_BLOCKS = 128   # partial sums of squares a row of a step of many rows may come with


def tiled_step(rt, rows: int) -> bool:
    """Whether a step of ``rows`` rows is one of many rows that takes the fused path through
    the tiled products (``rt.use_tiled_products``; otherwise steps of many rows run the
    library's products with separate norm and activation kernels)."""
    return rows > FUSED_MAX_ROWS and getattr(rt, "use_tiled_products", False) \
        and rt.dtype == torch.bfloat16 and getattr(rt, "use_fused", True) \
        and hasattr(rt.ops, "tiled_linear_ok")


def fused_rows_ok(rt, batch, *inner_sizes) -> bool:
    """Whether this step's rows can take the fused path through products with these
    inner sizes."""
    ops = rt.ops
    rows = batch.n_tokens
    if rows > FUSED_MAX_ROWS:
        # every inner size is also the width of some product's output
        return tiled_step(rt, rows) and ops.tiled_linear_ok(rows, 4, *inner_sizes) \
            and max(inner_sizes) <= 64 * TILED_MAX_STAT_BLOCKS
    if not (rt.dtype == torch.bfloat16 and getattr(ops, "has_fused_linear", False)
            and getattr(rt, "use_fused", True) and ops.fused_linear_ok(rows, *inner_sizes)):
        return False
    limit = getattr(rt, "fused_max_rows", None)
    if limit is None:
        streamed = hasattr(ops, "rows_kernel_ok") and ops.rows_kernel_ok(rows, *inner_sizes)
        limit = FUSED_MAX_ROWS if streamed else FUSED_MAX_ROWS_OLD_KERNEL
    return rows <= limit


SLICED_MAX_ROWS = 16      # rows of the k-sliced kernels
SLICED_MAX_STAT_BLOCKS = 512   # partial sums of squares a row may come with
SLICED_MAX_COLUMNS = 16384   # wider products (the output head) keep their rows in LDS instead


def stream_stats(rt, width: int, rows: int = 0) -> torch.Tensor:
    if rows > STAT_COLUMNS:       # a step of many rows: one partial sum per tile of columns
        return rt.ws.buf("stream_stats_many", (rows, TILED_MAX_STAT_BLOCKS), torch.float32)
    # up to one partial sum per 4 columns (the products for few rows use narrow workgroups)
    return rt.ws.buf("stream_stats", (STAT_COLUMNS, (width + 3) // 4), torch.float32)


def _side_by_side(rt, rows: int, width: int, *producer_inner: int) -> bool:
    """Whether a bfloat16 operand of ``width`` values a row, of a step of ``rows`` rows, lies
    with the rows side by side inside every group of 8 values (the layout that the kernel for
    9 to 64 rows reads whole runs of memory from) rather than one row after the other: where
    that kernel both reads it and, if a product writes it (inner size ``producer_inner``),
    writes it."""
    return hasattr(rt.ops, "rows_kernel_ok") and rt.ops.rows_kernel_ok(rows, width, *producer_inner)


def operand_rows(rt, name: str, rows: int, width: int, *producer_inner: int) -> torch.Tensor:
    """Room for a bfloat16 operand of the fused products, [rows, width] (up to 16 rows, or
    sizes the kernel for 9 to 64 rows does not take) or the view [rows, width/8, 8] of
    [width/8, 64, 8]."""
    if rows > STAT_COLUMNS:
        return rt.ws.buf(name + "_many", (rows, width), torch.bfloat16)
    if _side_by_side(rt, rows, width, *producer_inner):
        return rt.ws.buf(name + "_side_by_side", (width // 8, STAT_COLUMNS, 8), torch.bfloat16).permute(1, 0, 2)[:rows]
    return rt.ws.buf(name, (STAT_COLUMNS, width), torch.bfloat16)[:rows]


def stream_bf16(rt, rows: int, width: int) -> torch.Tensor:
    """The bfloat16 copy of the residual stream that products behind a norm read."""
    return operand_rows(rt, "stream_bf16", rows, width)


def _sliced(rt, rows: int, inner: int) -> bool:
    """Whether a product of ``rows`` bfloat16 rows with this inner size takes the form with
    the norm folded into the weights (the kernels for up to 16 and for 9 to 64 rows)."""
    if hasattr(rt.ops, "rows_kernel_ok") and rt.ops.rows_kernel_ok(rows, inner):
        return True
    return rows <= SLICED_MAX_ROWS and getattr(rt.ops, "use_sliced", False)


def _pack(rt, w: torch.Tensor) -> torch.Tensor:
    return rt.ops.pack_weight(w) if w.shape[1] % 32 == 0 and hasattr(rt.ops, "pack_weight") else w


def folded_weight(rt, w: torch.Tensor, norm_weight: torch.Tensor) -> torch.Tensor:
    """``w`` with the norm's weight multiplied into its columns: (x * nw) w^T = x (w * nw)^T,
    in the layout the products for few rows read best.  Made once per (weight, norm) pair
    and kept."""
    cache = rt.__dict__.setdefault("folded_weights", {})
    key = (w.data_ptr(), norm_weight.data_ptr())
    hit = cache.get(key)
    if hit is None:
        # (the entry holds on to both tensors: their addresses cannot pass to other weights
        # while it exists)
        hit = cache[key] = (_pack(rt, (w.float() * norm_weight.float().reshape(1, -1)).to(w.dtype)),
                            w, norm_weight)
    return hit[0]


def folded_plain_weight(rt, w: torch.Tensor, norm_weight: torch.Tensor) -> torch.Tensor:
    """``w`` with the norm's weight multiplied into its columns, rows one after the other (what
    the tiled products read).  Made once per (weight, norm) pair and kept."""
    cache = rt.__dict__.setdefault("folded_plain_weights", {})
    key = (w.data_ptr(), norm_weight.data_ptr())
    hit = cache.get(key)
    if hit is None:
        hit = cache[key] = ((w.float() * norm_weight.float().reshape(1, -1)).to(w.dtype).contiguous(),
                            w, norm_weight)
    return hit[0]


def packed_weight(rt, w: torch.Tensor) -> torch.Tensor:
    """A copy of ``w`` in the layout the products for few rows read best; made once."""
    cache = rt.__dict__.setdefault("packed_weights", {})
    hit = cache.get(w.data_ptr())
    if hit is None:
        hit = cache[w.data_ptr()] = (_pack(rt, w), w)
    return hit[0]


def norm_linear(rt, h, norm, w, out, *, epilogue="store", rows=None, n_rows=None, **kw):
    """out = epilogue(norm(h) w^T), the norm applied while the rows of ``h`` are read."""
    blocks = getattr(rt, "stream_stat_blocks", 0)
    M = n_rows if n_rows is not None else (rows.numel() if rows is not None else h.shape[0])
    if tiled_step(rt, h.shape[0]):
        if rows is not None or epilogue not in ("store", "swiglu") or w.dtype != torch.bfloat16:
            raise RuntimeError("norm_linear: not a product of the path for many rows")
        stats = stream_stats(rt, h.shape[1], h.shape[0])
        xb = stream_bf16(rt, h.shape[0], h.shape[1])
        if not (0 < blocks <= TILED_MAX_STAT_BLOCKS and getattr(rt, "stream_has_bf16", False)):
            rt.ops.stream_prepare(h, xb, stats)
            rt.stream_stat_blocks = blocks = 1
            rt.stream_has_bf16 = True
        return rt.ops.tiled_linear(xb, folded_plain_weight(rt, w, norm.weight), out, epilogue=epilogue,
                                   eps=norm.eps, stats=stats, stat_blocks=blocks, bias=kw.get("bias"))
    streams = {"swiglu": 2, "conv": 3}.get(epilogue, 1)
    streamed = hasattr(rt.ops, "rows_kernel_ok") and rt.ops.rows_kernel_ok(M, h.shape[1])
    if _sliced(rt, M, h.shape[1]) and w.dtype == torch.bfloat16 \
            and (streamed or w.shape[0] // streams <= SLICED_MAX_COLUMNS):
        # the stream's bfloat16 copy times the weight with the norm's weight folded in,
        # scaled by the rows' 1/rms at the end
        stats = stream_stats(rt, h.shape[1])
        xb = stream_bf16(rt, h.shape[0], h.shape[1])
        if xb.dim() == 3 and not streamed:
            # few wanted rows of a step of many: the kernel for few rows reads rows that lie one
            # after the other, so the stream gets such a copy too
            xb = rt.ws.buf("stream_bf16", (STAT_COLUMNS, h.shape[1]), torch.bfloat16)[:h.shape[0]]
            rt.ops.stream_prepare(h, xb, stats)
            rt.stream_stat_blocks = blocks = 1
        elif not (0 < blocks <= SLICED_MAX_STAT_BLOCKS and getattr(rt, "stream_has_bf16", False)):
            rt.ops.stream_prepare(h, xb, stats)
            rt.stream_stat_blocks = blocks = 1
            rt.stream_has_bf16 = True
        return rt.ops.fused_linear(xb, folded_weight(rt, w, norm.weight), out, epilogue=epilogue,
                                   eps=norm.eps, stats=stats, stat_blocks=blocks, rows=rows,
                                   n_rows=n_rows, **kw)
    return rt.ops.fused_linear(h, w, out, epilogue=epilogue, norm_weight=norm.weight,
                               eps=norm.eps, stats=stream_stats(rt, h.shape[1]) if blocks else None,
                               stat_blocks=blocks, rows=rows, n_rows=n_rows, **kw)


def linear_into_stream(rt, a, w, h, bias=None):
    """h += a w^T, leaving the partial sums of squares of the new rows (and, for few rows,
    the stream's bfloat16 copy)."""
    if tiled_step(rt, h.shape[0]):
        stats = stream_stats(rt, h.shape[1], h.shape[0])
        rt.ops.tiled_linear(a, w, h, epilogue="residual", bias=bias, stats_out=stats,
                            out_bf16=stream_bf16(rt, h.shape[0], h.shape[1]))
        rt.stream_stat_blocks = rt.ops.last_stat_blocks
        rt.stream_has_bf16 = True
        return h
    stats = stream_stats(rt, h.shape[1])
    inner = a.shape[1] * (8 if a.dim() == 3 else 1)
    sliced = _sliced(rt, h.shape[0], inner)
    xb = stream_bf16(rt, h.shape[0], h.shape[1]) if sliced else None
    if xb is not None and xb.dim() == 3 and not rt.ops.rows_kernel_ok(h.shape[0], inner):
        xb = None      # this product's kernel writes rows one after the other only: the next norm prepares the copy
    rt.ops.fused_linear(a, packed_weight(rt, w) if sliced else w, h, epilogue="residual", bias=bias,
                        stats_out=stats, out_bf16=xb)
    rt.stream_stat_blocks = rt.ops.last_stat_blocks
    rt.stream_has_bf16 = xb is not None
    return h
