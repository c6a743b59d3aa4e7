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

Optional, for speed only: the kernel that completes the residual stream can apply the norm
that reads it next on its way, if it knows that norm.  It is known when the stream is read
next, so a part may put off its last kernels until then: a mixer or feed-forward that sets
``defers_sum = True`` is given the step's :class:`ResidualStream` as ``residual`` and hands it
a function ``finish(rows, then_norm, takes_halves) -> normed rows | None`` (:func:`add_late`)
instead of adding into a tensor; the stream calls it when the next reader asks for
``stream.normed(norm, reader)`` - or for the plain tensor - and nothing else has touched the
stream in between.  ``takes_halves`` says that the reader accepts the norm in two halves
(``ops.linear.HalfNormed``, which the products of ``ops.linear`` take in place of x); a part
that passes its x only to those sets ``takes_prepared = True`` (or the least number of rows
from which it wants them).  A norm offers the fused form by ``row_and_column_form() ->
(column weights, eps)``.  A block that sets ``takes_stream = True`` is given the stream
instead of the tensor and reads it with ``stream.normed``.  Parts and blocks without these
flags get plain tensors, as the interfaces above say, and lose nothing but the fusion.
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


class ResidualStream:
    """The float32 residual stream of a step, ``[N, D]``, with at most one part's last
    kernels put off until the stream is read next (see the module's text).  Whoever reads it
    says how: ``normed(norm, reader)`` for the rows of a norm over it, ``tensor`` for the
    stream itself; both run what was put off first, so the order of the arithmetic is that
    of the plain wiring."""

    def __init__(self, rows: torch.Tensor):
        self._rows = rows
        self._finish = None

    @property
    def shape(self):
        return self._rows.shape

    def defer(self, finish: Callable) -> None:
        """``finish(rows, then_norm, takes_halves)`` adds a part's result into ``rows`` and
        returns the rows of ``then_norm`` over the sum if its kernel made them, else None."""
        self._settle(None, False)
        self._finish = finish

    def _settle(self, norm, takes_halves: bool):
        finish, self._finish = self._finish, None
        return None if finish is None else finish(self._rows, norm, takes_halves)

    @property
    def tensor(self) -> torch.Tensor:
        self._settle(None, False)
        return self._rows

    def normed(self, norm, reader=None, rows=None):
        """The rows of ``norm`` over the stream (``rows``: only these, by index), for
        ``reader``: from the kernel that completes the stream where it can make them, else by
        the norm's own kernel."""
        least = getattr(reader, "takes_prepared", False)
        halves = bool(least) and self._rows.shape[0] >= int(least)
        out = self._settle(norm if rows is None else None, halves)
        if out is not None and rows is None:
            return out
        return norm.forward(self._rows, rows=rows)


def add_late(residual, finish: Callable) -> None:
    """For a part with ``defers_sum``: put ``finish`` off on a :class:`ResidualStream`, or run
    it now on a plain tensor."""
    if isinstance(residual, ResidualStream):
        residual.defer(finish)
    else:
        finish(residual, None, False)


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
