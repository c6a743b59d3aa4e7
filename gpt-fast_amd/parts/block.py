"""How norms, mixer, feed-forward and the residual stream are wired in one layer."""
from ..config.spec import LayerSpec
from .base import FEED_FORWARDS, MIXERS, NORMS, Part, Runtime, register_block


class PreNormBlock(Part):
    """``h = x + mixer(norm1(x)); out = h + ffn(norm2(h))`` (reference model.py:161-164).
    The residual stream is float32 and updated in place; the sums happen in the
    parts' epilogues."""

    def __init__(self, spec: LayerSpec, runtime: Runtime):
        self.spec = spec
        self.mixer_norm = NORMS.build(spec.mixer_norm, runtime)
        self.mixer = MIXERS.build(spec.mixer, runtime)
        self.feed_forward_norm = NORMS.build(spec.feed_forward_norm, runtime)
        self.feed_forward = FEED_FORWARDS.build(spec.feed_forward, runtime)

    def children(self):
        s = self.spec
        return {s.mixer_norm_name: self.mixer_norm, s.mixer_name: self.mixer,
                s.feed_forward_norm_name: self.feed_forward_norm,
                s.feed_forward_name: self.feed_forward}

    def parameters(self):
        out = {}
        for child_name, child in self.children().items():
            for name, p in child.parameters().items():
                out[f"{child_name}.{name}"] = p
        return out

    def bind(self, tensors):
        for child_name, child in self.children().items():
            prefix = child_name + "."
            child.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})

    def cache_need(self):
        return self.mixer.cache_need()

    def step_flops(self, q_lens, starts) -> float:
        """Matrix-product work of one run of this block (parts that do not say count as 0)."""
        return sum(getattr(c, "step_flops", lambda q, s: 0.0)(q_lens, starts)
                   for c in self.children().values())

    def step_fields(self):
        out = []
        for child in self.children().values():
            out += list(getattr(child, "step_fields", lambda: ())())
        return out

    # Norm hand-over, optional for every part: a mixer or feed-forward that sets
    # ``prepares_norm`` takes ``then_norm=`` (the norm that reads the residual stream after
    # it) and ``takes_halves=`` (whether that norm's reader accepts an ops.linear.HalfNormed
    # in place of x; a part says so with ``takes_prepared``: True, or the least number of
    # rows from which it wants them), and returns that norm's rows if
    # it produced them on the way, else None.  A block that sets ``prepares_norm`` takes
    # ``x=`` (the rows of its first norm, if the caller has them), ``then_norm=`` and
    # ``takes_halves=`` in the same sense, and names its first norm ``mixer_norm``.
    prepares_norm = True

    @property
    def replayable(self):
        return all(getattr(c, "replayable", False) for c in self.children().values())

    @property
    def takes_prepared(self):
        return getattr(self.mixer, "takes_prepared", False)

    @staticmethod
    def _wants_halves(part, n_rows: int) -> bool:
        least = getattr(part, "takes_prepared", False)
        return bool(least) and n_rows >= int(least)

    def forward(self, residual, batch, entry, x=None, then_norm=None, takes_halves=False):
        if x is None:
            x = self.mixer_norm.forward(residual)
        h = None
        if getattr(self.mixer, "prepares_norm", False):
            h = self.mixer.forward(x, batch, entry, residual, then_norm=self.feed_forward_norm,
                                   takes_halves=self._wants_halves(self.feed_forward,
                                                                   residual.shape[0]))
        else:
            self.mixer.forward(x, batch, entry, residual)
        if h is None:
            h = self.feed_forward_norm.forward(residual)
        if then_norm is not None and getattr(self.feed_forward, "prepares_norm", False):
            return self.feed_forward.forward(h, batch, residual, then_norm=then_norm,
                                             takes_halves=takes_halves)
        self.feed_forward.forward(h, batch, residual)
        return None


register_block("pre_norm", PreNormBlock)
