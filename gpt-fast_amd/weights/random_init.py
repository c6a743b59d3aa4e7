"""Seeded random weights: as a model folder on disk, or directly on the device.

The reference has no such mode (its model is built on the meta device and always
filled from a checkpoint, generate.py:221-241).  Tensors are drawn one by one under
their checkpoint names, each from a generator seeded by (seed, name), so a tensor's
values depend neither on the order of drawing nor on the other tensors.
"""
import json
import os
import zlib
from typing import Dict

import torch

from .bindings import CheckpointLayout, compute_dtype, dtype_for_role
from .safetensors_io import write_safetensors


def _tensor_seed(seed: int, name: str) -> int:
    return (int(seed) * 1000003 + zlib.crc32(name.encode("utf-8"))) % (2 ** 63 - 1)


# init name -> function(standard normal float32 tensor, std, norm_std) -> tensor
INITS = {
    "linear": lambda t, std, norm_std: t.mul_(std),                    # N(0, std)
    "norm": lambda t, std, norm_std: t.mul_(norm_std).add_(1.0),       # 1 + N(0, norm_std)
}


def register_init(name: str, fn) -> None:
    """A further law for random weights: ``fn(t, std, norm_std)`` maps a tensor of standard
    normal draws of the parameter's shape to the parameter (a decay rate kept in (0, 1), a
    table of integers, ...)."""
    INITS[name] = fn


def draw(source, seed: int, device, std: float, norm_std: float) -> torch.Tensor:
    """One checkpoint tensor in float32, by the law its ``init`` names in ``INITS``."""
    if source.init not in INITS:
        raise ValueError(f"unknown init '{source.init}' for {source.name}; known: {sorted(INITS)}")
    g = torch.Generator(device=device)
    g.manual_seed(_tensor_seed(seed, source.name))
    t = torch.randn(source.shape, generator=g, device=device, dtype=torch.float32)
    return INITS[source.init](t, std, norm_std)


def random_checkpoint(layout: CheckpointLayout, seed: int, dtype="bfloat16", *,
                      std=0.02, norm_std=0.1, tie=False) -> Dict[str, torch.Tensor]:
    """CPU tensors under checkpoint names, stored in ``dtype``."""
    dtype = compute_dtype(dtype)
    out = {}
    for b in layout.bindings:
        if b.alias_of is not None and tie:
            continue
        for s in b.sources:
            out[s.name] = draw(s, seed, "cpu", std, norm_std).to(dtype)
    return out


def write_random_model(folder: str, arch, config, seed: int, dtype="bfloat16", *,
                       std=0.02, norm_std=0.1) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` of ``arch``."""
    os.makedirs(folder, exist_ok=True)
    cfg = arch.config_dict(config)
    cfg["torch_dtype"] = "float32" if compute_dtype(dtype) == torch.float32 else "bfloat16"
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    layout = arch.bindings(config)
    # whether the head shares the embedding table is the plan's to say, under whatever key
    # the architecture's config.json holds it
    tensors = random_checkpoint(layout, seed, dtype, std=std, norm_std=norm_std,
                                tie=bool(arch.plan(config).tie_embeddings))
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder


def random_parameters(layout: CheckpointLayout, seed: int, dtype, device, *,
                      std=0.02, norm_std=0.1, tie=False) -> Dict[str, torch.Tensor]:
    """The plan's parameters drawn directly on ``device`` (no file): for shapes too
    large to be worth a trip over the disk.  Values differ from those of
    :func:`random_checkpoint` (another generator), the distribution does not."""
    dtype = compute_dtype(dtype)
    params = {}
    for b in layout.bindings:
        if b.alias_of is not None and tie:
            continue
        want = dtype_for_role(b.role, dtype)
        parts = [draw(s, seed, device, std, norm_std).to(want) for s in b.sources]
        params[b.target] = (b.combine(parts) if b.combine else parts[0]).contiguous()
    for b in layout.bindings:
        if b.alias_of is not None and tie:
            params[b.target] = params[b.alias_of]
    return params
