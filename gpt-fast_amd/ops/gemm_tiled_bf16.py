"""Python faces of the 17..64-row products over weights kept in matrix-core operand order
(csrc/gemm_tiled_bf16.hip).

A weight matrix gets its tiled form the first time a step of that many rows uses it, if the
device has room for it (the row-major matrix stays: the prompt's products and the few-row
kernels read that one); the tiled form hangs on the weight tensor and lives as long as it.
"""
import ctypes
from typing import Optional

import torch

from .library import KernelError, check, library, ptr, require_contiguous, require_device, stream_handle

_i = ctypes.c_int
MIN_ROWS, MAX_ROWS = 17, 64
# a tiled copy is only made while this fraction of the device's memory stays free afterwards
KEEP_FREE_FRACTION = 0.2


class Tiled:
    """The tiled form of a weight matrix [rows, K] (``gate``: of [2 I, K], rows of W1 then rows
    of W3, tiles of eight and eight)."""

    __slots__ = ("data", "rows", "cols", "gate")

    def __init__(self, data, rows, cols, gate):
        self.data, self.rows, self.cols, self.gate = data, rows, cols, gate


def _lib():
    lib = library("gemm_tiled_bf16")
    lib.gfa_tiled_elements.restype = ctypes.c_size_t
    return lib


def tile(w: torch.Tensor, gate: bool = False) -> Tiled:
    """A new tiled copy of ``w`` [rows, K] (bfloat16, K a multiple of 8)."""
    require_device(w)
    require_contiguous(w=w)
    if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] % 8 or (gate and w.shape[0] % 2):
        raise KernelError(f"tile: a bfloat16 matrix [rows, K], K a multiple of 8 (gate: an even "
                          f"number of rows), not {tuple(w.shape)} {w.dtype}")
    rows, K = w.shape
    gate_rows = rows // 2 if gate else 0
    n = _lib().gfa_tiled_elements(_i(rows), _i(K), _i(gate_rows))
    data = torch.empty(n, dtype=torch.bfloat16, device=w.device)
    check(_lib().gfa_tile_weights(ptr(w), ptr(data), _i(rows), _i(K), _i(gate_rows), stream_handle()),
          "tile_weights")
    return Tiled(data, rows, K, gate)


def tiled_of(w: torch.Tensor, gate: bool = False) -> Optional[Tiled]:
    """The tiled form that hangs on ``w``, made now if there is none and the device has room
    (never while a step is being recorded: a recording's first run makes it); else None."""
    name = "_gfa_tiled_gate" if gate else "_gfa_tiled"
    t = getattr(w, name, None)
    if t is not None or getattr(w, name + "_refused", False):
        return t
    if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] % 8 or not w.is_contiguous() \
            or (gate and w.shape[0] % 2) or torch.cuda.is_current_stream_capturing():
        return None
    free, total = torch.cuda.mem_get_info(w.device)
    need = _lib().gfa_tiled_elements(_i(w.shape[0]), _i(w.shape[1]), _i(w.shape[0] // 2 if gate else 0)) * 2
    if free - need < KEEP_FREE_FRACTION * total:
        setattr(w, name + "_refused", True)          # asked once, not at every step
        return None
    t = tile(w, gate)
    setattr(w, name, t)
    return t


def takes(n_rows: int, inner: int) -> bool:
    return MIN_ROWS <= n_rows <= MAX_ROWS and inner % 8 == 0


def _check_x(x, t: Tiled, what):
    require_device(x, t.data)
    require_contiguous(x=x)
    if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != t.cols:
        raise KernelError(f"{what}: x {tuple(x.shape)} {x.dtype} does not fit a matrix of {t.cols} columns")
    if not 0 < x.shape[0] <= MAX_ROWS:
        raise KernelError(f"{what}: {x.shape[0]} rows; this kernel takes 1..{MAX_ROWS}")


def slices(N: int, K: int) -> int:
    return int(_lib().gfa_tiled_slices(_i(N), _i(K), _i(5)))


def partial_sums(x: torch.Tensor, t: Tiled) -> torch.Tensor:
    """float32 [S, M, N]: the product's sums over each of S slices of K (S may be 1)."""
    _check_x(x, t, "tiled partial_sums")
    if t.gate:
        raise KernelError("tiled partial_sums: a gate matrix has its own product")
    M, K = x.shape
    N = t.rows
    part = torch.empty((slices(N, K), M, N), dtype=torch.float32, device=x.device)
    check(_lib().gfa_tiled_bf16(ptr(x), ptr(t.data), ptr(part), _i(M), _i(N), _i(K), _i(N), _i(5),
                                stream_handle()), "tiled partial_sums")
    return part


def product_f32(x: torch.Tensor, t: Tiled) -> torch.Tensor:
    """float32 [M, N] = x W^T in one kernel (for matrices of many rows: the output head)."""
    _check_x(x, t, "tiled product_f32")
    if t.gate:
        raise KernelError("tiled product_f32: a gate matrix has its own product")
    M, K = x.shape
    out = torch.empty((M, t.rows), dtype=torch.float32, device=x.device)
    check(_lib().gfa_tiled_bf16(ptr(x), ptr(t.data), ptr(out), _i(M), _i(t.rows), _i(K), _i(t.rows),
                                _i(1), stream_handle()), "tiled product_f32")
    return out


def product_gated(x: torch.Tensor, t: Tiled) -> torch.Tensor:
    """bfloat16 [M, I] = silu(x W1^T) * (x W3^T) for the tiled form of [W1; W3]."""
    _check_x(x, t, "tiled product_gated")
    if not t.gate:
        raise KernelError("tiled product_gated: the matrix was not tiled for the gate")
    M, K = x.shape
    I = t.rows // 2
    out = torch.empty((M, I), dtype=torch.bfloat16, device=x.device)
    check(_lib().gfa_tiled_bf16(ptr(x), ptr(t.data), ptr(out), _i(M), _i(I), _i(K), _i(I), _i(3),
                                stream_handle()), "tiled product_gated")
    return out
