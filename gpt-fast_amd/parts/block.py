"""How norms, mixer, feed-forward and the residual stream are wired in one layer."""
from ..config.spec import LayerSpec
from .base import FEED_FORWARDS, MIXERS, NORMS, Part, ResidualStream, Runtime, register_block


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

    # Reads the stream through ``stream.normed`` so that the kernel which completed it can
    # hand over the norm's rows (parts.base.ResidualStream); parts that do not put off their
    # sum get the plain tensor.
    takes_stream = True

    @property
    def replayable(self):
        return all(getattr(c, "replayable", False) for c in self.children().values())

    @property
    def takes_prepared(self):
        return getattr(self.mixer, "takes_prepared", False)

    @staticmethod
    def _residual_for(part, stream):
        return stream if getattr(part, "defers_sum", False) else stream.tensor

    def forward(self, residual, batch, entry):
        stream = residual if isinstance(residual, ResidualStream) else ResidualStream(residual)
        x = stream.normed(self.mixer_norm, reader=self.mixer)
        self.mixer.forward(x, batch, entry, self._residual_for(self.mixer, stream))
        h = stream.normed(self.feed_forward_norm, reader=self.feed_forward)
        self.feed_forward.forward(h, batch, self._residual_for(self.feed_forward, stream))
        if stream is not residual:
            stream.tensor                    # a caller with a plain tensor gets the sums now


register_block("pre_norm", PreNormBlock)
