"""Python faces of the bfloat16 matrix-product kernels (csrc/gemm_bf16.hip)."""
import ctypes
from typing import Optional

import torch

from .library import KernelError, check, library, ptr, require_contiguous, require_device, stream_handle

_i = ctypes.c_int
MAX_ROWS = 64
# rows of x up to which the dot-product kernel is used; above, the matrix-core kernel
DOT_MAX_ROWS = 1


class ChunkedRows:
    """Up to 64 rows of bfloat16 as one few-row product leaves them for the next:
    ``data`` holds [cols / 8][pad][8] (pad = 4, 8, 16, 32 or 64, the least that holds the rows), so
    that the lanes which load one 16-byte chunk each of different rows read consecutive
    bytes.  Only the kernels of this module look inside; :meth:`to_rows` is for tests."""

    __slots__ = ("data", "rows", "cols", "pad")

    def __init__(self, rows: int, cols: int, device):
        if not 0 < rows <= MAX_ROWS or cols % 8:
            raise KernelError(f"chunked rows: {rows} x {cols} (1..{MAX_ROWS} rows, columns in eights)")
        self.rows, self.cols, self.pad = rows, cols, share_rows(rows)
        self.data = torch.empty(cols * self.pad, dtype=torch.bfloat16, device=device)

    @property
    def shape(self):
        return (self.rows, self.cols)

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device

    def to_rows(self) -> torch.Tensor:
        t = self.data.view(self.cols // 8, self.pad, 8).permute(1, 0, 2).reshape(self.pad, self.cols)
        return t[:self.rows].contiguous()


def share_rows(n_rows: int) -> int:
    """Rows per record of the sums-of-squares shares, and per chunk of chunked rows, for this
    many rows of x."""
    return 4 if n_rows <= 4 else 8 if n_rows <= 8 else 16 if n_rows <= 16 else 32 if n_rows <= 32 else 64


def _entry(M: int, K: int):
    lib = library("gemm_bf16")
    if M > DOT_MAX_ROWS and K % 8 == 0:
        return lib.gfa_skinny_mfma_bf16
    return lib.gfa_skinny_bf16


def _check_operands(x, w, what):
    require_device(x, w)
    require_contiguous(x=x, w=w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"{what}: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"{what}: x {tuple(x.shape)} and w {tuple(w.shape)} do not fit")
    if not 0 < x.shape[0] <= MAX_ROWS:
        raise KernelError(f"{what}: {x.shape[0]} rows; this kernel takes 1..{MAX_ROWS}")


def skinny(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None):
    """x [M<=64, K] times w [N, K] transposed.  With ``residual`` (float32 [M, N]) the
    product is added into it; else a new [M, N] tensor of ``out_dtype`` (bfloat16 or
    float32) is returned."""
    _check_operands(x, w, "skinny")
    M, K = x.shape
    N = w.shape[0]
    if residual is not None:
        require_device(residual)
        if (residual.shape != (M, N) or residual.dtype != torch.float32
                or not residual.is_contiguous()):
            raise KernelError("skinny: residual must be contiguous float32 [M, N]")
        out, mode = residual, 2
    else:
        out_dtype = out_dtype or torch.bfloat16
        if out_dtype not in (torch.bfloat16, torch.float32):
            raise KernelError(f"skinny: output type {out_dtype}")
        if out is None:
            out = torch.empty((M, N), dtype=out_dtype, device=x.device)
        elif out.shape != (M, N) or out.dtype != out_dtype or not out.is_contiguous():
            raise KernelError("skinny: out has the wrong shape or dtype")
        mode = 0 if out_dtype == torch.bfloat16 else 1
    check(_entry(M, K)(ptr(x), ptr(w), ptr(out), _i(M), _i(N), _i(K), _i(N), _i(mode), _i(0),
                       stream_handle()), "skinny")
    return out


def skinny_gated(x: torch.Tensor, w13: torch.Tensor, out: Optional[torch.Tensor] = None):
    """[M, I] = silu(x W1^T) * (x W3^T), w13 = [2I, K]: rows of W1, then rows of W3."""
    _check_operands(x, w13, "skinny_gated")
    M, K = x.shape
    if w13.shape[0] % 2:
        raise KernelError("skinny_gated: w13 needs an even number of rows")
    I = w13.shape[0] // 2
    if out is None:
        out = torch.empty((M, I), dtype=torch.bfloat16, device=x.device)
    elif out.shape != (M, I) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise KernelError("skinny_gated: out has the wrong shape or dtype")
    check(_entry(M, K)(ptr(x), ptr(w13), ptr(out), _i(M), _i(I), _i(K), _i(I), _i(3), _i(I),
                       stream_handle()), "skinny_gated")
    return out


# Rows up to which the products of a layer hand their rows to one another (the norms in two
# halves, the rows chunked); the kernels take up to MAX_ROWS.  Measured against the vendor
# library's products with the passes between them, per step: 8B shape 4.14 -> 3.95 ms at
# 17..24 rows, 4.30 -> 4.22 at 32, 4.60 -> 5.9 at 40 (every workgroup of a consumer reads all
# shares of the norm, 64 rows wide from 33 rows on); 70B shape 26.6 -> 26.5 ms at 24 rows,
# 27.1 -> 27.8 at 32.
CHAIN_MAX_ROWS = 24


def can_chain_norm(n_rows: int, n_out: int, inner: int) -> bool:
    """The residual-completing product of this shape prepares the norm that follows (where
    that is the faster way; the kernel itself takes up to MAX_ROWS rows)."""
    return 0 < n_rows <= CHAIN_MAX_ROWS and n_out % 8 == 0 and inner % 8 == 0


def skinny_into_chain(x, w: torch.Tensor, residual: torch.Tensor, next_g: torch.Tensor):
    """residual += x w^T, and the first half of the RMS norm that follows: returns
    ``xg`` = bfloat16(new residual * next_g) as :class:`ChunkedRows` and ``ssq`` float32
    [workgroups, R]: per workgroup (one or two tiles of 12 to 16 columns) its share of each row's sum of
    squares, R = 4, 8, 16, 32 or 64 rows per record (the least that holds M).  Up to 64 rows; x a
    tensor [M, K] or :class:`ChunkedRows` (the gate's result, left so on request)."""
    chunked = isinstance(x, ChunkedRows)
    _check_operands(x.data.view(x.pad, x.cols)[:x.rows] if chunked else x, w, "skinny_into_chain")
    M, K = x.shape
    N = w.shape[0]
    require_device(residual, next_g)
    if residual.shape != (M, N) or residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("skinny_into_chain: residual must be contiguous float32 [M, N]")
    if next_g.dtype != torch.float32 or next_g.numel() != N or not next_g.is_contiguous():
        raise KernelError("skinny_into_chain: one float32 norm weight per column")
    if N % 8 or K % 8:                                   # up to MAX_ROWS rows: checked above
        raise KernelError(f"skinny_into_chain: [{M}, {K}] x [{N}, {K}] is outside this kernel")
    xg = ChunkedRows(M, N, w.device)
    records = library("gemm_bf16").gfa_skinny_workgroups(_i(2), _i(M), _i(N))   # one per workgroup
    ssq = torch.empty((records, share_rows(M)), dtype=torch.float32, device=w.device)
    check(library("gemm_bf16").gfa_skinny_into_chain_bf16(
        ptr(x.data if chunked else x), _i(int(chunked)), ptr(w), ptr(residual), _i(M), _i(N), _i(K),
        ptr(next_g), ptr(xg.data), ptr(ssq), stream_handle()), "skinny_into_chain")
    return xg, ssq


def _check_chain(xg, ssq, w, what):
    if not isinstance(xg, ChunkedRows):
        raise KernelError(f"{what}: the first half of the norm comes as ChunkedRows")
    require_device(xg.data, w, ssq)
    require_contiguous(w=w)
    if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != xg.cols or w.shape[1] % 8:
        raise KernelError(f"{what}: xg {xg.shape} and w {tuple(w.shape)} do not fit")
    if ssq.dtype != torch.float32 or ssq.dim() != 2 or ssq.shape[1] != xg.pad \
            or not ssq.is_contiguous():
        raise KernelError(f"{what}: ssq must be contiguous float32 [shares, {xg.pad}]")


def skinny_after_chain(xg, ssq, eps: float, w, out_dtype=torch.bfloat16):
    """The second half: (xg w^T) scaled per row m by rsqrt(sum(ssq[:, m]) / K + eps)."""
    _check_chain(xg, ssq, w, "skinny_after_chain")
    M, K = xg.shape
    N = w.shape[0]
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise KernelError(f"skinny_after_chain: output type {out_dtype}")
    out = torch.empty((M, N), dtype=out_dtype, device=w.device)
    check(library("gemm_bf16").gfa_skinny_after_chain_bf16(
        ptr(xg.data), ptr(ssq), _i(ssq.shape[0]), ctypes.c_float(eps), ptr(w), ptr(out), _i(M), _i(N),
        _i(K), _i(N), _i(0 if out_dtype == torch.bfloat16 else 1), _i(0), _i(0), stream_handle()),
        "skinny_after_chain")
    return out


def skinny_after_chain_gated(xg, ssq, eps: float, w13, chunked: bool = False):
    """silu(n W1^T) * (n W3^T) with n the normed rows given by their two halves; ``chunked``:
    as :class:`ChunkedRows`, for :func:`skinny_into_chain` to read."""
    _check_chain(xg, ssq, w13, "skinny_after_chain_gated")
    M, K = xg.shape
    if w13.shape[0] % 2:
        raise KernelError("skinny_after_chain_gated: w13 needs an even number of rows")
    I = w13.shape[0] // 2
    if chunked:
        res = ChunkedRows(M, I, w13.device)
        out = res.data
    else:
        res = out = torch.empty((M, I), dtype=torch.bfloat16, device=w13.device)
    check(library("gemm_bf16").gfa_skinny_after_chain_bf16(
        ptr(xg.data), ptr(ssq), _i(ssq.shape[0]), ctypes.c_float(eps), ptr(w13), ptr(out), _i(M), _i(I),
        _i(K), _i(I), _i(3), _i(I), _i(int(chunked)), stream_handle()), "skinny_after_chain_gated")
    return res


def wide_f32_out(x: torch.Tensor, w: torch.Tensor):
    """Many rows, float32 result (logits of every position of a prompt): the vendor
    library with a float32 output; products of bfloat16 values are exact in float32 and
    the accumulation is float32."""
    require_device(x, w)
    return torch.mm(x, w.t(), out_dtype=torch.float32)


def qkv_rope_store(x, wqkv, freqs, tok_seq, tok_pos, table, k_pages, v_pages, n_heads: int,
                   n_kv_heads: int, head_dim: int, rotary_dim: int,
                   ssq: Optional[torch.Tensor] = None, eps: float = 0.0):
    """Fused q/k/v projection, rotation of interleaved pairs and the cache write in one
    kernel; returns q [M, H, hd].  ``x`` [M, K] bfloat16 holds normed rows (up to 64), or,
    with ``ssq`` and ``eps``, the two halves of a norm as :func:`skinny_into_chain` leaves
    them (:class:`ChunkedRows`, up to 16 rows).  k_pages None: nothing is stored."""
    if ssq is not None:
        _check_chain(x, ssq, wqkv, "qkv_rope_store")
        xdata = x.data
    else:
        xdata = x
        _check_operands(x, wqkv, "qkv_rope_store")
        if wqkv.shape[1] % 8:
            raise KernelError("qkv_rope_store: the inner size must be a multiple of 8")
    M, K = x.shape
    if wqkv.shape[0] != (n_heads + 2 * n_kv_heads) * head_dim:
        raise KernelError("qkv_rope_store: wqkv does not have (H + 2 Hkv) * hd rows")
    if head_dim % 16 or rotary_dim % 2 or not 0 <= rotary_dim <= head_dim:
        raise KernelError("qkv_rope_store: head_dim must be a multiple of 16, rotary_dim even")
    require_device(freqs, tok_seq, tok_pos, table, k_pages, v_pages)
    if rotary_dim and (freqs is None or freqs.numel() != rotary_dim // 2
                       or freqs.dtype != torch.float32):
        raise KernelError("qkv_rope_store: one float32 frequency per rotary pair")
    for name, t in (("tok_seq", tok_seq), ("tok_pos", tok_pos), ("table", table)):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise KernelError(f"qkv_rope_store: {name} must be contiguous int32")
    if tok_seq.numel() < M or tok_pos.numel() < M:
        raise KernelError("qkv_rope_store: token maps are shorter than the batch")
    if (k_pages is None) != (v_pages is None):
        raise KernelError("qkv_rope_store: give both k_pages and v_pages, or neither")
    if k_pages is not None:
        if tuple(k_pages.shape[1:]) != (n_kv_heads, 64, head_dim) \
                or tuple(v_pages.shape[1:]) != (n_kv_heads, head_dim, 64) \
                or k_pages.dtype != torch.bfloat16 or v_pages.dtype != torch.bfloat16 \
                or not k_pages.is_contiguous() or not v_pages.is_contiguous():
            raise KernelError("qkv_rope_store: pages have the wrong shape or dtype")
    q = torch.empty((M, n_heads, head_dim), dtype=torch.bfloat16, device=wqkv.device)
    check(library("gemm_bf16").gfa_qkv_rope_store_bf16(
        ptr(xdata), ptr(ssq), _i(0 if ssq is None else ssq.shape[0]), ctypes.c_float(eps), ptr(wqkv),
        ptr(q), ptr(k_pages), ptr(v_pages), ptr(freqs), ptr(tok_seq), ptr(tok_pos), ptr(table),
        _i(table.shape[1]), _i(M), _i(K), _i(n_heads), _i(n_kv_heads), _i(head_dim),
        _i(rotary_dim), stream_handle()), "qkv_rope_store")
    return q
