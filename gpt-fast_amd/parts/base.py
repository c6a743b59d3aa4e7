"""Interfaces of the parts a layer is made of, and the registries that map a spec's
``kind`` to the part that runs it.

A part is built from its spec and a :class:`Runtime`, states the parameters it owns
(:meth:`Part.parameters`), receives them (:meth:`Part.bind`) and then runs.  No part knows
which model it is in; it sees its own spec, the step's batch and its own cache entry.

Interfaces (N = tokens of the step, D = model width):

* norm:          ``forward(residual float32 [N, D], rows=None) -> [n, D]`` in the compute type
* mixer:         ``cache_need() -> KVNeed | StateNeed | None``;
                 ``forward(x [N, D], batch, entry, residual)`` adds its output into
                 ``residual`` (float32 [N, D], in place)
* feed-forward:  ``forward(x [N, D], batch, residual)`` adds its output into ``residual``
* position:      ``rotate_and_store(qkv, batch, entry, n_heads, n_kv_heads, head_dim) -> q``
* block:         ``forward(residual, batch, entry)`` updates ``residual`` in place

A new part is a class with these methods, registered under a new ``kind``; its spec is
any object with that ``kind`` attribute.

``replayable = True`` on a part says that its ``forward`` issues the same kernels, with
the same arguments, whatever the batch holds - it reads the batch's device fields only,
never ``host_field`` or a host copy - so that a step recorded once can be replayed for
later steps of the same shape.  A part without it (the default) makes generation step the
model without a recording.

Optional, for speed only: a mixer or feed-forward that sets ``prepares_norm = True`` also
takes ``then_norm=`` (the norm that reads the residual stream after it) and
``takes_halves=`` and returns that norm's rows if its last kernel produced them on the way,
else None; with ``takes_halves`` they may be an ``ops.linear.HalfNormed``, which the products
of ``ops.linear`` accept in place of x, and a part that passes its x only to those sets
``takes_prepared = True``.  A norm offers this by ``row_and_column_form() -> (column
weights, eps)``.  A block with ``prepares_norm`` takes ``x=`` (the rows of its first norm,
``mixer_norm``, if the caller has them), ``then_norm=`` and ``takes_halves=`` and returns
likewise.  Parts without the flags are called as above and get plain tensors.
"""
from dataclasses import dataclass
from typing import Callable, Dict, Tuple

import torch


@dataclass(frozen=True)
class Param:
    """A parameter a part owns: shape, role ("matrix" | "vector" | "index", as in
    weights.bindings) and how random weights draw it."""
    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "linear"


class Runtime:
    """What parts need to know about the engine they run in."""

    def __init__(self, dtype: torch.dtype, device):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"compute type {dtype}: float32 or bfloat16")
        self.dtype = dtype
        self.device = torch.device(device)

    @property
    def is_float32(self) -> bool:
        return self.dtype == torch.float32


class Part:
    replayable = False

    def parameters(self) -> Dict[str, Param]:
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        pass

    def step_fields(self):
        """Further int32 fields of a step's description that this part reads
        (``engine.batch.StepField``); none by default."""
        return ()


class _Registry:
    def __init__(self, what: str):
        self.what = what
        self._kinds: Dict[str, Callable] = {}

    def register(self, kind: str, factory: Callable) -> Callable:
        self._kinds[kind] = factory
        return factory

    def build(self, spec, runtime: Runtime):
        kind = getattr(spec, "kind", None)
        if kind not in self._kinds:
            raise KeyError(f"no {self.what} is registered for kind '{kind}'; "
                           f"known: {sorted(self._kinds)}")
        return self._kinds[kind](spec, runtime)

    def kinds(self):
        return sorted(self._kinds)


NORMS = _Registry("norm")
POSITIONS = _Registry("position encoding")
MIXERS = _Registry("mixer")
FEED_FORWARDS = _Registry("feed-forward")
BLOCKS = _Registry("block arrangement")      # keyed by LayerSpec.arrangement


def register_norm(kind, factory):
    return NORMS.register(kind, factory)


def register_position(kind, factory):
    return POSITIONS.register(kind, factory)


def register_mixer(kind, factory):
    return MIXERS.register(kind, factory)


def register_feed_forward(kind, factory):
    return FEED_FORWARDS.register(kind, factory)


def register_block(arrangement, factory):
    return BLOCKS.register(arrangement, factory)


def check_bound(owner: str, declared: Dict[str, Param], tensors: Dict[str, torch.Tensor]) -> None:
    """Every declared parameter is there with its shape."""
    for name, p in declared.items():
        if name not in tensors:
            raise KeyError(f"{owner}: parameter '{name}' was not given")
        if tuple(tensors[name].shape) != tuple(p.shape):
            raise ValueError(f"{owner}: parameter '{name}' is {list(tensors[name].shape)}, "
                             f"expected {list(p.shape)}")
