"""Gated feed-forward (reference model.py:219-227)."""
from ..config.spec import GatedFeedForwardSpec
from ..ops import linear as L
from .base import Param, Part, Runtime, add_late, check_bound, register_feed_forward


class GatedFeedForward(Part):
    """``w2( silu(w1 x) * (w3 x) )`` without biases.  w1 and w3 are one matrix ``w13``
    (rows of w1, then rows of w3) so that the gate is applied where the products end."""

    def __init__(self, spec: GatedFeedForwardSpec, runtime: Runtime):
        if spec.activation != "silu":
            raise ValueError(f"activation '{spec.activation}': only silu has a kernel")
        self.spec = spec
        self.rt = runtime
        self.w13 = self.w2 = None

    def parameters(self):
        s = self.spec
        return {"w13": Param((2 * s.hidden, s.dim)), "w2": Param((s.dim, s.hidden))}

    def bind(self, tensors):
        check_bound("GatedFeedForward", self.parameters(), tensors)
        self.w13, self.w2 = tensors["w13"], tensors["w2"]

    replayable = True
    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream
    # x may be an ops.linear.HalfNormed, from one row on (the least number of rows; with the
    # weights streamed past the caches the matrix-core kernel that takes the halves is as fast
    # at one row as the dot-product kernel that does not, and the norm kernel is saved)
    takes_prepared = 1

    def step_flops(self, q_lens, starts) -> float:
        return 2.0 * sum(q_lens) * 3 * self.spec.hidden * self.spec.dim

    def forward(self, x, batch, residual):
        # both products wait until the stream is read next: whether the gate's result stays in
        # the order the second product loads it in depends on the norm that follows
        add_late(residual, lambda rows, then_norm, takes_halves: L.gated_into(
            x, self.w13, self.w2, rows, then_norm, takes_halves))


register_feed_forward("gated", GatedFeedForward)
