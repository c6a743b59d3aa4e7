"""Loading a model's parameters from safetensors files by tensor name.

An architecture states, as data, which checkpoint tensors make up each parameter of
its plan (:class:`Binding`); this module finds the tensors, checks all names and shapes
in one pass and reports every problem in a single :class:`WeightsError`, then builds
the parameters on the device.

Dtype rule.  ``role`` says how a parameter is used (the table ``ROLES``, open to further
roles through :func:`register_role`): a "matrix" (operand of a matrix
product, also the embedding table) is kept in the engine's compute type (bfloat16 or
float32); a "vector" (norm weights and the like) is kept in float32, which holds a
bfloat16 value exactly; an "index" table is int32.  A tensor stored in 32-bit is never
narrowed unless it is a matrix operand of a bfloat16 engine.
"""
import re
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch

from .safetensors_io import open_model_files


@dataclass(frozen=True)
class Source:
    """One tensor of the checkpoint: its name, shape, and how random weights draw it
    ("linear": N(0, std); "norm": 1 + N(0, norm_std))."""
    name: str
    shape: Tuple[int, ...]
    init: str = "linear"


@dataclass(frozen=True)
class Binding:
    """Parameter ``target`` = ``combine(list of source tensors)`` (identity for one
    source).  If ``alias_of`` is set and none of the sources is in the files, the
    parameter shares the tensor of that other target (tied embeddings)."""
    target: str
    sources: Tuple[Source, ...]
    role: str = "matrix"
    combine: Optional[Callable[[List[torch.Tensor]], torch.Tensor]] = None
    alias_of: Optional[str] = None


@dataclass(frozen=True)
class CheckpointLayout:
    bindings: Tuple[Binding, ...]
    ignored: Tuple[str, ...] = ()        # regular expressions of tensor names to skip


class WeightsError(ValueError):
    """Names every missing tensor, unexpected tensor and wrong shape at once."""

    def __init__(self, where, missing, unexpected, wrong_shape, other=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.other = list(other)
        lines = [f"{where}: the checkpoint does not fit the configuration"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): "
                         + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): "
                         + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n} is {list(got)}, expected {list(exp)}"
                for n, got, exp in self.wrong_shape))
        for o in self.other:
            lines.append("  " + o)
        super().__init__("\n".join(lines))


def compute_dtype(name) -> torch.dtype:
    if name in ("bfloat16", "bf16", torch.bfloat16):
        return torch.bfloat16
    if name in ("float32", "fp32", "f32", torch.float32):
        return torch.float32
    raise ValueError(f"dtype '{name}': bfloat16 or float32")


# role -> (storage type given the engine's compute type, whether the stored tensor must be
# of a floating type)
ROLES: Dict[str, Tuple[Callable[[torch.dtype], torch.dtype], bool]] = {
    "matrix": (lambda dtype: dtype, True),
    "vector": (lambda dtype: torch.float32, True),
    "index": (lambda dtype: torch.int32, False),
}


def register_role(role: str, storage: Callable[[torch.dtype], torch.dtype],
                  floating: bool = True) -> None:
    """A further way a parameter is used (a state-space model's float32 recurrence
    matrices, say): ``storage(compute type)`` is the type it is kept in."""
    ROLES[role] = (storage, floating)


def dtype_for_role(role: str, dtype: torch.dtype) -> torch.dtype:
    if role not in ROLES:
        raise ValueError(f"unknown parameter role '{role}'; known: {sorted(ROLES)}")
    return ROLES[role][0](dtype)


def check_layout(layout: CheckpointLayout, entries: Dict[str, Tuple[str, tuple]], where: str):
    """Compare the files' tensors with the layout; raise one error for all problems.
    Returns the set of targets that are aliases."""
    missing, wrong, other = [], [], []
    used = set()
    aliased = set()
    for b in layout.bindings:
        present = [s for s in b.sources if s.name in entries]
        if b.alias_of is not None and not present:
            aliased.add(b.target)
            continue
        for s in b.sources:
            if s.name not in entries:
                missing.append(s.name)
                continue
            used.add(s.name)
            dt, shape = entries[s.name]
            if tuple(shape) != tuple(s.shape):
                wrong.append((s.name, tuple(shape), tuple(s.shape)))
            if ROLES.get(b.role, (None, True))[1] and dt not in ("F64", "F32", "F16", "BF16"):
                other.append(f"{s.name} is stored as {dt}, expected a floating type")
    ignored = [re.compile(p) for p in layout.ignored]
    unexpected = [n for n in entries
                  if n not in used and not any(p.search(n) for p in ignored)]
    if missing or unexpected or wrong or other:
        raise WeightsError(where, sorted(missing), sorted(unexpected), wrong, other)
    return aliased


def choose_layout(layouts: Sequence[CheckpointLayout], names) -> CheckpointLayout:
    """The layout most of whose tensor names are among ``names`` (the first on a tie): a
    checkpoint is told by the names it uses, and its errors are reported against those."""
    names = set(names)

    def found(layout):
        return sum(s.name in names for b in layout.bindings for s in b.sources)

    return max(layouts, key=found)


def load_parameters(folder: str, layout, dtype, device) -> Dict[str, torch.Tensor]:
    """Read every parameter from the safetensors files of ``folder``.  ``layout`` is one
    :class:`CheckpointLayout` or several, of which the files' tensor names choose."""
    dtype = compute_dtype(dtype)
    files = open_model_files(folder)
    entries, owner = {}, {}
    for f in files:
        for name, meta in f.entries.items():
            entries[name] = meta
            owner[name] = f
    if not isinstance(layout, CheckpointLayout):
        layout = choose_layout(tuple(layout), entries)
    aliased = check_layout(layout, entries, folder)
    params: Dict[str, torch.Tensor] = {}
    for b in layout.bindings:
        if b.target in aliased:
            continue
        want = dtype_for_role(b.role, dtype)
        parts = []
        for s in b.sources:
            t = owner[s.name].tensor(s.name)
            # bytes go to the device as stored; the cast happens there
            t = t.to(device) if device is not None else t.clone()
            if t.dtype != want:
                t = t.to(want)
            parts.append(t)
        params[b.target] = (b.combine(parts) if b.combine is not None else parts[0]).contiguous()
    for b in layout.bindings:
        if b.target in aliased:
            if b.alias_of not in params:
                raise WeightsError(folder, [s.name for s in b.sources], [], [],
                                   [f"{b.target} is tied to {b.alias_of}, which is absent"])
            params[b.target] = params[b.alias_of]
    return params
