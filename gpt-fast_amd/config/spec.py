"""Descriptions of a model as data: what each layer is made of and in which order
layers run.

An architecture's configuration (read from its ``config.json``) is turned into a
:class:`ModelPlan` by that architecture's ``plan`` function.  Everything below the
plan (parts, cache, step function, generation) reads only the plan, never the
architecture's name.  Every size and constant a part needs is a field of its spec.

A spec's ``kind`` selects the part class in the registries of ``parts``; a test or an
application can define a new spec class with a new ``kind`` and register a part for it.
"""
from dataclasses import dataclass
from typing import List, Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    """Root-mean-square norm over the last dimension (reference model.py:230-241)."""
    dim: int
    eps: float
    kind: str = "rms"


@dataclass(frozen=True)
class PositionSpec:
    """How positions enter a mixer.

    kind "rope": rotate pairs of the first ``rotary_dim`` elements of each query and
    key head by ``position * frequency[i]`` (reference model.py:266-293).  ``layout``
    is "interleaved" (pairs (2i, 2i+1), the reference's) or "half" (pairs
    (i, i + rotary_dim/2)).  ``scaling`` is None or a dict with ``rope_type`` and that
    rule's constants (reference model.py:244-263 for "llama3").
    kind "none": no position information is added.
    """
    kind: str = "rope"
    rotary_dim: int = 0
    base: float = 10000.0
    layout: str = "interleaved"
    scaling: Optional[Tuple[Tuple[str, object], ...]] = None   # dict items, hashable

    def scaling_dict(self) -> Optional[dict]:
        return None if self.scaling is None else dict(self.scaling)


@dataclass(frozen=True)
class AttentionSpec:
    """Causal attention with grouped key/value heads over the cache
    (reference model.py:167-216).  ``window`` None means every earlier key is read;
    an integer W means keys at distance < W only."""
    dim: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    position: PositionSpec
    scale: Optional[float] = None          # None: 1/sqrt(head_dim)
    window: Optional[int] = None
    kind: str = "attention"


@dataclass(frozen=True)
class GatedFeedForwardSpec:
    """w2( act(w1 x) * (w3 x) ) without biases (reference model.py:219-227)."""
    dim: int
    hidden: int
    activation: str = "silu"
    kind: str = "gated"


@dataclass(frozen=True)
class LayerSpec:
    """One block.  ``arrangement`` names how norms, mixer, feed-forward and the residual
    stream are wired ("pre_norm": reference model.py:161-164).  ``name`` is the prefix of
    the layer's tensors.  Parameter sub-names are those of the arrangement."""
    name: str
    mixer: object
    mixer_norm: NormSpec
    feed_forward: object
    feed_forward_norm: NormSpec
    arrangement: str = "pre_norm"
    mixer_name: str = "mixer"
    mixer_norm_name: str = "mixer_norm"
    feed_forward_name: str = "feed_forward"
    feed_forward_norm_name: str = "feed_forward_norm"


@dataclass(frozen=True)
class Run:
    """One entry of the order in which layers run.  ``layer`` indexes
    ``ModelPlan.layers``; a layer may be named by several entries (its weights are then
    used more than once).  ``cache`` names the cache entry the mixer reads and writes;
    it defaults to an entry of this run's own.  A run with ``cache_from`` = index of an
    earlier run reads that run's cache and writes nothing."""
    layer: int
    cache_from: Optional[int] = None


@dataclass
class ModelPlan:
    """A whole decoder: embedding, layers in run order, final norm, output head.
    ``max_positions`` bounds prompt + new tokens of a generated request."""
    dim: int
    vocab_size: int
    layers: List[LayerSpec]
    order: List[Run]
    final_norm: NormSpec
    tie_embeddings: bool = False
    max_positions: int = 2048
    embedding_name: str = "tok_embeddings.weight"
    final_norm_name: str = "norm"               # prefix of the final norm's tensors ("norm.weight")
    head_name: str = "output.weight"
    stop_tokens: Tuple[int, ...] = ()
    # Optional steps around the layers; None leaves the step out (the reference has none
    # of them, model.py:136-146).
    embedding_scale: Optional[float] = None     # embedded rows are multiplied by this
    input_position: object = None               # a position spec whose part adds to the embedded
    input_position_name: str = "input_position"  # rows (``add_to_stream``); prefix of its tensors
    logit_scale: Optional[float] = None         # logits are multiplied by this,
    logit_softcap: Optional[float] = None       # then capped: cap * tanh(logits / cap)

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("a model plan needs at least one layer")
        for n, run in enumerate(self.order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"order[{n}] names layer {run.layer}, "
                                 f"but there are {len(self.layers)} layers")
            if run.cache_from is not None:
                if not 0 <= run.cache_from < n:
                    raise ValueError(f"order[{n}].cache_from={run.cache_from} must name "
                                     f"an earlier entry of the order")
                if self.order[run.cache_from].cache_from is not None:
                    raise ValueError(f"order[{n}].cache_from={run.cache_from} names an "
                                     f"entry that itself borrows a cache")
