"""Matrix products of the step, ``y = x W^T`` with ``W`` stored ``[out, in]`` as in the
reference's linears (model.py:110, 174-175, 222-224), with the epilogues the blocks need.

float32 engine: the library's own float32 kernel, for every shape (a true 32-bit
product; one fused-multiply-add chain per output).

bfloat16 engine, by the rows of x: up to 16, hand-written kernels that stream the weights
once (csrc/gemm_bf16.hip; up to 24 rows inside a layer's chain where a matrix has no
tiled copy); 17..64, hand-written kernels over a second copy of the weights in the matrix
cores' operand order (csrc/gemm_tiled_bf16.hip), and without that copy the sliced kernel of
csrc/gemm_wide_bf16.hip or the vendor library, whichever measures faster for the shape;
more rows, the vendor matrix library through ``torch.matmul`` - the reference uses the
vendor library for these as well - cut into slices of the inner size (``torch.bmm``) where
the result has too few tiles to fill the chip.  A sliced product leaves float32 partial
sums that the kernel behind it adds in slice order (:class:`SlicedRows`).  Accumulation is
float32 everywhere.
"""
from typing import Optional

import torch

from . import kernels as K
from .library import KernelError

# products with at most this many rows go to the hand-written streaming kernels (one 16-row
# matrix-core tile of x); beyond that x no longer fits a wave's registers and the vendor
# library's tiled kernels are faster (measured at 32 and 64 rows)
SKINNY_MAX_ROWS = 16


_units = {}


def _compute_units(device) -> int:
    n = _units.get(device)
    if n is None:
        n = _units[device] = torch.cuda.get_device_properties(device).multi_processor_count
    return n


def _own_gate_is_faster(M: int, inner: int, K_: int, device) -> bool:
    """17..64 rows through the gate: the hand-written kernel (the gate in its epilogue) against
    the vendor library's product followed by the gate kernel.  A workgroup of the own kernel
    takes 64 gate columns, so what decides is how the ``inner / 64`` workgroups fill the chip
    (measured at 17..64 rows): with fewer than four fifths of the compute units (inner 11008:
    172 on 256) the library wins by 1-8 us at every row count; from there on the own kernel
    wins by 5-7 us up to 48 rows (inner 14336: 46-52 us against 52-59), and at more rows only
    where every compute unit has a workgroup and a half or more (inner 28672: 173 against 192
    us at 64 rows, while inner 14336 loses 55 to 51)."""
    if K_ % 8 or not 16 < M <= _wide().MAX_ROWS:
        return False
    wgs, cus = (inner + 63) // 64, _compute_units(device)
    if wgs * 5 < cus * 4:
        return False
    return M <= 48 or wgs * 2 >= cus * 3


def _fast():
    from . import gemm_bf16
    return gemm_bf16


# From this many rows on (up to 64), a product reads its weights from a second copy kept in the
# matrix cores' operand order (gemm_tiled_bf16), if the device has room for that copy: measured
# on the 8B shapes at 17..64 rows, 41-44 us against 55-65 for the gate product with the vendor
# library and the gate kernel behind it, 22-24 against 29-39 for the second feed-forward product,
# 11-13 against 13-18 for the projections; per step 3.60-3.65 ms at 17..24 rows against
# 4.01-4.07 for the chain of few-row kernels, which is what runs there without the copy.
TILED_FROM_ROWS = 17


def _tiled_for(rows: int, w: torch.Tensor, gate: bool = False):
    """The tiled form of ``w`` if a product of this many rows should use it, else None."""
    from . import gemm_tiled_bf16 as T
    if rows < TILED_FROM_ROWS or not T.takes(rows, w.shape[1]) or w.dtype != torch.bfloat16:
        return None
    return T.tiled_of(w, gate)


def _library_slices(M: int, N: int, K_: int, device) -> int:
    """Slices of the inner size for a product of more than 64 rows through the vendor library.
    Its kernels give every 128 x 128 tile (or so) of the result to one workgroup that walks the
    whole inner size: a few hundred rows make fewer tiles than the chip has compute units, and
    a long inner size makes each of them slow (512 rows times the feed-forward's second matrix
    of the 8B shape: 128 tiles, 88 us = 0.68 PFLOP/s).  Cut into S slices, run as one batched
    product with float32 results, the tiles are S times as many (60 us with four slices); the
    kernels that add the slices are the ones that follow the product anyway (residual sum and
    norm, rotation and cache write).  Measured on 256 compute units at 128..2048 rows: the
    slices pay while they bring the tiles up to about 2.5 per compute unit, more for a longer
    inner size (the float32 partial sums, S * M * N * 4 bytes written and read, are then the
    smaller part), and never for the gate product, whose result is seven times its x."""
    if K_ % 8 or M <= 0:
        return 1
    tiles = ((M + 127) // 128) * ((N + 127) // 128)
    want = 2.5 * _compute_units(device) * (K_ / 4096.0) ** 0.5 / tiles
    # more than four slices only for few rows: from 512 rows on eight are no faster than four
    # (60.1 against 59.6 us in the example above) and cost twice the partial sums
    most = 8 if M <= 256 else 4
    S = 1
    while 2 * S <= want and 2 * S <= most and K_ % (16 * S) == 0 and K_ // (2 * S) >= 1024:
        S *= 2
    return S


def _library_partial_sums(x: torch.Tensor, w: torch.Tensor, S: int) -> torch.Tensor:
    """float32 [S, M, N]: x W^T over each of S equal slices of the inner size, as one batched
    product of the vendor library over views of x and w (nothing is copied)."""
    M, K_ = x.shape
    N = w.shape[0]
    xs = x.view(M, S, K_ // S).permute(1, 0, 2)
    ws = w.view(N, S, K_ // S).permute(1, 2, 0)
    return torch.bmm(xs, ws, out_dtype=torch.float32)


class HalfNormed:
    """Rows of an RMS norm in two halves, as the few-row product that completed the residual
    stream left them: ``xg`` = bfloat16(residual * norm weight) (``gemm_bf16.ChunkedRows``
    of [M, D]) and ``ssq`` [shares, 4, 8 or 16],
    whose column sums are the rows' sums of squares (float32, from the float32 residual).
    The products of this module take it in place of x and apply the missing factor
    rsqrt(sum / D + eps) to their float32 result; a factor per row commutes with the product,
    so this is the norm of model.py:236-241 with the rounding to bfloat16 before the row
    factor instead of after it.  No kernel runs between the two products."""

    __slots__ = ("xg", "ssq", "eps")

    def __init__(self, xg, ssq, eps):
        self.xg, self.ssq, self.eps = xg, ssq, eps

    @property
    def shape(self):
        return self.xg.shape

    @property
    def dtype(self):
        return self.xg.dtype


class SlicedRows:
    """Rows of a product whose inner size was cut into slices, before the slices are added:
    ``part`` float32 [S, M, N].  A reader that adds them on its way (the rotation and cache
    write of ``ops.kernels.rope_cache_write_sliced``) saves the pass that :meth:`rows` is."""

    __slots__ = ("part", "dtype")

    def __init__(self, part, dtype):
        self.part, self.dtype = part, dtype

    @property
    def shape(self):
        return tuple(self.part.shape[1:])

    def rows(self) -> torch.Tensor:
        """[M, N] in the product's type: the slices added in order."""
        return _wide().sum_store(self.part, self.dtype)


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           may_stay_sliced: bool = False):
    """[M, N] = x [M, K] times w [N, K] transposed, in ``out_dtype`` (default: x's).
    ``may_stay_sliced``: the caller also takes a :class:`SlicedRows`."""
    out_dtype = out_dtype or x.dtype
    if isinstance(x, HalfNormed):
        return _fast().skinny_after_chain(x.xg, x.ssq, x.eps, w, out_dtype=out_dtype)
    if x.dtype == torch.float32:
        if out_dtype != torch.float32:
            raise KernelError("a float32 product has a float32 result")
        return K.gemm_f32(x, w)
    M = x.shape[0]
    if M <= SKINNY_MAX_ROWS:
        return _fast().skinny(x, w, out_dtype=out_dtype)
    t = _tiled_for(M, w)
    if t is not None:
        from . import gemm_tiled_bf16 as T
        if out_dtype == torch.float32:
            return T.product_f32(x, t)
        rows = SlicedRows(T.partial_sums(x, t), out_dtype)
        return rows if may_stay_sliced else rows.rows()
    if out_dtype == torch.float32:
        return _fast().wide_f32_out(x, w)
    if M > _wide().MAX_ROWS and w.shape[0] % 4 == 0 and x.is_contiguous() and w.is_contiguous():
        S = _library_slices(M, w.shape[0], x.shape[1], x.device)
        if S > 1:
            rows = SlicedRows(_library_partial_sums(x, w, S), out_dtype)
            return rows if may_stay_sliced else rows.rows()
    return torch.matmul(x, w.t())


def linear_into(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, then_norm=None,
                takes_halves: bool = False):
    """residual (float32 [M, N]) += x W^T.  ``then_norm``: the norm that reads the residual
    stream next.  Where the sum is a kernel of its own (many bfloat16 rows) and the norm is a
    factor per row times a weight per column, sum and norm run as one pass and the normed
    rows are returned; with few rows and ``takes_halves`` (the reader of the norm is a product
    of this module) they are returned as a :class:`HalfNormed`; else None, and the caller runs
    the norm."""
    form = getattr(then_norm, "row_and_column_form", None)
    if _chains(x.shape[0], x.dtype, w, then_norm, takes_halves):
        weight, eps = form()
        xg, ssq = _fast().skinny_into_chain(x, w, residual, weight)
        return HalfNormed(xg, ssq, eps)
    if x.dtype == torch.bfloat16 and x.shape[0] > SKINNY_MAX_ROWS:
        weight, eps = form() if form is not None else (None, 0.0)
        t = _tiled_for(x.shape[0], w) if w.shape[0] % 4 == 0 and w.shape[0] <= 16384 else None
        if t is not None:
            from . import gemm_tiled_bf16 as T
            return _wide().sum_add_norm(residual, T.partial_sums(x, t), weight, eps)
        if _sliced_is_faster(x.shape[0], w.shape[0], x.shape[1]):
            return _wide().product_into(x, w, residual, weight, eps)
        if x.shape[0] > _wide().MAX_ROWS and w.shape[0] % 4 == 0 and w.shape[0] <= 16384 \
                and x.is_contiguous() and w.is_contiguous():
            S = _library_slices(x.shape[0], w.shape[0], x.shape[1], x.device)
            if S > 1:
                return _wide().sum_add_norm(residual, _library_partial_sums(x, w, S), weight, eps)
        if form is not None:
            return K.add_rmsnorm(residual, torch.matmul(x, w.t()), weight, eps)
    _linear_into(x, w, residual)
    return None


def takes_chunked_rows(rows: int, dtype, w, then_norm, takes_halves: bool) -> bool:
    """:func:`linear_into` with these arguments runs the few-row kernel that also reads its x
    as ``gemm_bf16.ChunkedRows``."""
    return _chains(rows, dtype, w, then_norm, takes_halves)


def _chains(rows: int, dtype, w, then_norm, takes_halves: bool) -> bool:
    """The few-row product with ``w`` that completes the residual stream also prepares
    ``then_norm`` for a reader that takes it in halves."""
    return (takes_halves and dtype == torch.bfloat16
            and getattr(then_norm, "row_and_column_form", None) is not None
            and _fast().can_chain_norm(rows, w.shape[0], w.shape[1])
            and _tiled_for(rows, w) is None)        # with the second copy, 17..24 rows go there


def _wide():
    from . import gemm_wide_bf16
    return gemm_wide_bf16


def _sliced_is_faster(M: int, N: int, K_: int) -> bool:
    """17..64 rows times a matrix with few rows and a long inner size (the feed-forward's
    second product): the hand-written kernel cuts K into slices over many workgroups where
    the vendor library runs few; measured faster from an inner size of twice the width."""
    return M <= _wide().MAX_ROWS and K_ % 8 == 0 and N % 4 == 0 and N <= 16384 and K_ >= 2 * N


def _linear_into(x, w, residual):
    if x.dtype == torch.float32:
        return K.gemm_f32(x, w, out=residual, accumulate=True)
    if x.shape[0] <= SKINNY_MAX_ROWS:
        return _fast().skinny(x, w, residual=residual)
    return K.add_into(residual, torch.matmul(x, w.t()))


def gated_linear(x: torch.Tensor, w13: torch.Tensor):
    """[M, I] = silu(x W1^T) * (x W3^T), with w13 = rows of W1 then rows of W3
    (model.py:227)."""
    if isinstance(x, HalfNormed):
        return _fast().skinny_after_chain_gated(x.xg, x.ssq, x.eps, w13)
    if x.dtype == torch.float32:
        return K.silu_mul(K.gemm_f32(x, w13))
    if x.shape[0] <= SKINNY_MAX_ROWS:
        return _fast().skinny_gated(x, w13)
    t = _tiled_for(x.shape[0], w13, gate=True) if w13.shape[0] % 2 == 0 else None
    if t is not None:
        from . import gemm_tiled_bf16 as T
        return T.product_gated(x, t)
    if w13.shape[0] % 2 == 0 and _own_gate_is_faster(x.shape[0], w13.shape[0] // 2, x.shape[1], x.device):
        return _wide().product_gated(x, w13)
    return K.silu_mul(torch.matmul(x, w13.t()))


def gated_into(x, w13: torch.Tensor, w2: torch.Tensor, residual: torch.Tensor, then_norm=None,
               takes_halves: bool = False):
    """residual += (silu(x W1^T) * (x W3^T)) W2^T: :func:`gated_linear`, then
    :func:`linear_into` with its arguments and result.  Between two few-row kernels that take
    and leave a norm in halves, the gate's result stays in the order the second one loads it
    in (``gemm_bf16.ChunkedRows``)."""
    if isinstance(x, HalfNormed) and _chains(x.shape[0], x.dtype, w2, then_norm, takes_halves):
        h = _fast().skinny_after_chain_gated(x.xg, x.ssq, x.eps, w13, chunked=True)
    else:
        h = gated_linear(x, w13)
    return linear_into(h, w2, residual, then_norm, takes_halves)


# ----------------------------------------------------------------------------- fused projection
def can_project_rotate_store(x: torch.Tensor, wqkv: torch.Tensor, head_dim: int) -> bool:
    """True if the fused projection / rotation / cache-write kernel takes these rows."""
    if isinstance(x, HalfNormed):
        return head_dim % 16 == 0
    return (x.dtype == torch.bfloat16 and 0 < x.shape[0] <= SKINNY_MAX_ROWS
            and wqkv.shape[1] % 8 == 0 and head_dim % 16 == 0)


def qkv_rope_store(x, wqkv, freqs, tok_seq, tok_pos, table, k_pages, v_pages, n_heads, n_kv_heads,
                   head_dim, rotary_dim):
    """q [M, H, hd] of normed rows ``x`` (a tensor or a :class:`HalfNormed`) through the fused
    projection / rotation / cache-write kernel."""
    if isinstance(x, HalfNormed):
        return _fast().qkv_rope_store(x.xg, wqkv, freqs, tok_seq, tok_pos, table, k_pages, v_pages,
                                      n_heads, n_kv_heads, head_dim, rotary_dim, ssq=x.ssq, eps=x.eps)
    return _fast().qkv_rope_store(x, wqkv, freqs, tok_seq, tok_pos, table, k_pages, v_pages,
                                  n_heads, n_kv_heads, head_dim, rotary_dim)
