"""Python faces of the matrix-product kernels for 17..64 rows (csrc/gemm_wide_bf16.hip)."""
import ctypes
from typing import Optional

import torch

from .library import KernelError, check, library, ptr, require_contiguous, require_device, stream_handle

_i = ctypes.c_int
MAX_ROWS = 64


def _check(x, w, what):
    require_device(x, w)
    require_contiguous(x=x, w=w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"{what}: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"{what}: x {tuple(x.shape)} and w {tuple(w.shape)} do not fit")
    if not 0 < x.shape[0] <= MAX_ROWS or x.shape[1] % 8:
        raise KernelError(f"{what}: takes 1..{MAX_ROWS} rows and an inner size that is a multiple "
                          f"of 8, not {tuple(x.shape)}")


def takes(n_rows: int, inner: int) -> bool:
    return 0 < n_rows <= MAX_ROWS and inner % 8 == 0


def slices(M: int, N: int, K: int) -> int:
    """Slices of K the product is cut into (1 where N is no multiple of 4)."""
    if N % 4:
        return 1
    return int(library("gemm_wide_bf16").gfa_wide_slices(_i(M), _i(N), _i(K), _i(5)))


def _launch(x, w, out, N, ldo, mode, gate_rows, what):
    M, K = x.shape
    check(library("gemm_wide_bf16").gfa_wide_bf16(ptr(x), ptr(w), ptr(out), _i(M), _i(N), _i(K),
                                                  _i(ldo), _i(mode), _i(gate_rows), stream_handle()),
          what)


def partial_sums(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """float32 [S, M, N]: the product's sums over each of S slices of K."""
    _check(x, w, "partial_sums")
    M, K = x.shape
    N = w.shape[0]
    S = slices(M, N, K)
    part = torch.empty((S, M, N), dtype=torch.float32, device=x.device)
    _launch(x, w, part, N, N, 5, 0, "partial_sums")
    return part


def sum_store(part: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """The slices added in order, as bfloat16 or float32 [M, N]."""
    S, M, N = part.shape
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise KernelError(f"sum_store: output type {out_dtype}")
    out = torch.empty((M, N), dtype=out_dtype, device=part.device)
    check(library("gemm_wide_bf16").gfa_wide_sum_store(
        ptr(part), _i(S), _i(M), _i(N), ptr(out), _i(out_dtype == torch.bfloat16), stream_handle()),
        "sum_store")
    return out


def sum_add_norm(residual: torch.Tensor, part: torch.Tensor, norm_w: Optional[torch.Tensor] = None,
                 eps: float = 0.0) -> Optional[torch.Tensor]:
    """residual += the slices added in order; with ``norm_w`` also returns the RMS norm of
    the new rows in bfloat16."""
    S, M, N = part.shape
    require_device(residual, part, norm_w)
    if residual.shape != (M, N) or residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("sum_add_norm: residual must be contiguous float32 [M, N]")
    if N % 4 or N > 16384:
        raise KernelError("sum_add_norm: the width must be a multiple of 4, at most 16384")
    xn = None
    if norm_w is not None:
        if norm_w.dtype != torch.float32 or norm_w.numel() != N or not norm_w.is_contiguous():
            raise KernelError("sum_add_norm: one float32 norm weight per column")
        xn = torch.empty((M, N), dtype=torch.bfloat16, device=residual.device)
    check(library("gemm_wide_bf16").gfa_wide_sum_add_norm(
        ptr(residual), ptr(part), _i(S), _i(M), _i(N), ptr(norm_w), ptr(xn), ctypes.c_float(eps),
        stream_handle()), "sum_add_norm")
    return xn


def product(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16):
    """x [M <= 64, K] times w [N, K] transposed, bfloat16 or float32 [M, N]."""
    _check(x, w, "product")
    M, K = x.shape
    N = w.shape[0]
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise KernelError(f"product: output type {out_dtype}")
    if slices(M, N, K) > 1:
        return sum_store(partial_sums(x, w), out_dtype)
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _launch(x, w, out, N, N, 0 if out_dtype == torch.bfloat16 else 1, 0, "product")
    return out


def product_into(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor,
                 norm_w: Optional[torch.Tensor] = None, eps: float = 0.0):
    """residual (float32 [M, N]) += x w^T; with ``norm_w`` returns the RMS norm of the new
    rows in bfloat16 if the product was sliced (the norm then rides on the second kernel),
    else None."""
    _check(x, w, "product_into")
    M, K = x.shape
    N = w.shape[0]
    if residual.shape != (M, N) or residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("product_into: residual must be contiguous float32 [M, N]")
    if slices(M, N, K) > 1 and N <= 16384:
        return sum_add_norm(residual, partial_sums(x, w), norm_w, eps)
    _launch(x, w, residual, N, N, 2, 0, "product_into")
    return None


def product_gated(x: torch.Tensor, w13: torch.Tensor):
    """[M, I] = silu(x W1^T) * (x W3^T), w13 = [2I, K]: rows of W1, then rows of W3."""
    _check(x, w13, "product_gated")
    M, K = x.shape
    if w13.shape[0] % 2:
        raise KernelError("product_gated: w13 needs an even number of rows")
    I = w13.shape[0] // 2
    out = torch.empty((M, I), dtype=torch.bfloat16, device=x.device)
    _launch(x, w13, out, I, I, 3, I, "product_gated")
    return out
