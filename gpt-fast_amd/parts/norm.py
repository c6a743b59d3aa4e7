"""RMS norm (reference model.py:230-241)."""
import torch

from ..config.spec import NormSpec
from ..ops import kernels as K
from .base import Param, Part, Runtime, check_bound, register_norm


class RMSNorm(Part):
    """``x * rsqrt(mean(x^2) + eps) * weight`` over the last dimension; statistics and
    scaling in float32 from the float32 residual stream, one rounding to the compute type
    at the store.  ``eps`` and the width are the spec's."""

    replayable = True

    def __init__(self, spec: NormSpec, runtime: Runtime):
        self.spec = spec
        self.rt = runtime
        self.weight = None

    def parameters(self):
        return {"weight": Param((self.spec.dim,), role="vector", init="norm")}

    def bind(self, tensors):
        check_bound("RMSNorm", self.parameters(), tensors)
        self.weight = tensors["weight"].to(torch.float32).contiguous()

    def forward(self, residual: torch.Tensor, rows=None) -> torch.Tensor:
        return K.rmsnorm(residual, self.weight, self.spec.eps, self.rt.dtype, rows=rows)

    def row_and_column_form(self):
        """This norm is a factor per row, rsqrt(mean(x^2) + eps), times a weight per column:
        (column weights, eps).  A kernel that completes the residual stream can apply it in
        the same pass."""
        return self.weight, self.spec.eps


register_norm("rms", RMSNorm)
