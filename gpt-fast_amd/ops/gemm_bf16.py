"""Python faces of the bfloat16 matrix-product kernels (csrc/gemm_bf16.hip)."""
import ctypes
from typing import Optional

import torch

from .library import KernelError, check, library, ptr, require_contiguous, require_device, stream_handle

_i = ctypes.c_int
MAX_ROWS = 64
# rows of x up to which the dot-product kernel is used; above, the matrix-core kernel
DOT_MAX_ROWS = 1


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


def wide_f32_out(x: torch.Tensor, w: torch.Tensor):
    """Many rows, float32 result (logits of every position of a prompt): the vendor
    library with a float32 output; products of bfloat16 values are exact in float32 and
    the accumulation is float32."""
    require_device(x, w)
    try:
        return torch.mm(x, w.t(), out_dtype=torch.float32)
    except (TypeError, RuntimeError):
        out = torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32, device=x.device)
        step = 8192
        xf = x.float()
        for n0 in range(0, w.shape[0], step):
            out[:, n0:n0 + step] = xf @ w[n0:n0 + step].float().t()
        return out
