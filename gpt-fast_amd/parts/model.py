"""A whole decoder assembled from a plan (reference model.py:102-146)."""
from typing import Dict, List

import torch

from ..config.spec import ModelPlan
from ..ops import kernels as K
from ..ops import linear as L
from .base import BLOCKS, NORMS, POSITIONS, Param, ResidualStream, Runtime, check_bound


class DecoderModel:
    """Embedding, the plan's layers in the plan's order, final norm, output head; around
    them the optional steps a plan may state (a factor on the embedded rows, a position
    encoding added to them, a factor and a soft cap on the logits).

    ``forward`` runs the tokens of one step: embeds them, passes the float32 residual
    stream through every run of the order with that run's cache entry, then norms and
    projects only the rows whose logits are wanted (the reference projects every
    position, model.py:144-146)."""

    def __init__(self, plan: ModelPlan, runtime: Runtime):
        plan.validate()
        self.plan = plan
        self.rt = runtime
        self.blocks = [BLOCKS.build(_Arranged(layer), runtime) for layer in plan.layers]
        self.final_norm = NORMS.build(plan.final_norm, runtime)
        self.input_position = None
        if plan.input_position is not None:
            self.input_position = POSITIONS.build(plan.input_position, runtime)
            if not hasattr(self.input_position, "add_to_stream"):
                raise TypeError(f"position kind '{plan.input_position.kind}' cannot be a plan's "
                                f"input_position: its part has no add_to_stream(residual, batch)")
        self.embedding = self.head = None

    # ------------------------------------------------------------------ parameters
    def parameters(self) -> Dict[str, Param]:
        p = {self.plan.embedding_name: Param((self.plan.vocab_size, self.plan.dim)),
             self.plan.head_name: Param((self.plan.vocab_size, self.plan.dim))}
        for name, param in self.final_norm.parameters().items():
            p[f"{self.plan.final_norm_name}.{name}"] = param
        if self.input_position is not None:
            for name, param in self.input_position.parameters().items():
                p[f"{self.plan.input_position_name}.{name}"] = param
        for layer, block in zip(self.plan.layers, self.blocks):
            for name, param in block.parameters().items():
                p[f"{layer.name}.{name}"] = param
        return p

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        declared = self.parameters()
        check_bound("model", declared, tensors)
        extra = sorted(set(tensors) - set(declared))
        if extra:
            raise KeyError(f"model: parameters {extra} belong to no part")
        self._tensors = dict(tensors)
        self.embedding = tensors[self.plan.embedding_name]
        self.head = tensors[self.plan.head_name]
        prefix = self.plan.final_norm_name + "."
        self.final_norm.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})
        if self.input_position is not None:
            prefix = self.plan.input_position_name + "."
            self.input_position.bind({k[len(prefix):]: v for k, v in tensors.items()
                                      if k.startswith(prefix)})
        for layer, block in zip(self.plan.layers, self.blocks):
            prefix = layer.name + "."
            block.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})

    def parameter_bytes(self, exclude_embedding: bool = True) -> int:
        """Bytes of the parameters one decode step reads (the embedding table is a
        gather of a few rows, as in the reference's accounting, generate.py:251-268)."""
        seen, total = set(), 0
        for name, t in self._tensors.items():
            if exclude_embedding and name == self.plan.embedding_name \
                    and t.data_ptr() != self.head.data_ptr():
                continue
            if t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        return total

    @property
    def replayable(self) -> bool:
        """Every part issues the same kernels whatever a batch holds: a recorded step can be
        replayed."""
        return (all(getattr(b, "replayable", False) for b in self.blocks)
                and getattr(self.final_norm, "replayable", False)
                and (self.input_position is None
                     or getattr(self.input_position, "replayable", False)))

    def parameter_count(self, exclude_embedding: bool = True) -> int:
        """Elements of the same parameters (the reference's ``params`` of
        generate.py:251-268, which feeds its FLOPS line)."""
        seen, total = set(), 0
        for name, t in self._tensors.items():
            if exclude_embedding and name == self.plan.embedding_name \
                    and t.data_ptr() != self.head.data_ptr():
                continue
            if t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel()
        return total

    # ------------------------------------------------------------------ cache
    def cache_needs(self) -> List[object]:
        return [self.blocks[run.layer].cache_need() for run in self.plan.order]

    def cache_borrow(self) -> List[object]:
        return [run.cache_from for run in self.plan.order]

    def step_flops(self, q_lens, starts, n_want: int) -> float:
        """Matrix-product work (multiply-adds times two) of one step that brings
        ``q_lens[b]`` tokens to sequences holding ``starts[b]`` and wants ``n_want`` rows of
        logits: every run of the order, as its parts count themselves, and the head."""
        flops = 2.0 * n_want * self.plan.dim * self.plan.vocab_size
        for run in self.plan.order:
            block = self.blocks[run.layer]
            flops += getattr(block, "step_flops", lambda q, s: 0.0)(q_lens, starts)
        return flops

    def step_fields(self):
        """The further fields of a step's description that the parts ask for, each once (by
        name: layers of one kind ask for the same field)."""
        seen = {}
        parts = list(self.blocks) + [self.final_norm, self.input_position]
        for part in parts:
            for f in (getattr(part, "step_fields", lambda: ())() if part is not None else ()):
                seen.setdefault(f.name, f)
        return list(seen.values())

    # ------------------------------------------------------------------ step
    def forward(self, batch, cache) -> torch.Tensor:
        """float32 logits [n_wanted, vocab] of the step described by ``batch``."""
        plan = self.plan
        residual = K.embed(self.embedding, batch.tokens)                  # model.py:140
        if plan.embedding_scale is not None:
            K.scale_cap(residual, plan.embedding_scale)
        if self.input_position is not None:
            self.input_position.add_to_stream(residual, batch)
        stream = ResidualStream(residual)
        for n, run in enumerate(plan.order):                              # model.py:142-143
            block = self.blocks[run.layer]
            block.forward(stream if getattr(block, "takes_stream", False) else stream.tensor,
                          batch, cache.entries[n])
        if batch.n_want == 0:
            stream.tensor
            return torch.empty((0, self.plan.vocab_size), dtype=torch.float32,
                               device=residual.device)
        # the head takes plain rows (no reader named): with its many columns the halves of a
        # norm cost more than the norm kernel they save
        every = getattr(batch, "every_row_wanted", False)
        x = stream.normed(self.final_norm, rows=None if every else batch.want_rows)   # model.py:144
        logits = L.linear(x, self.head, out_dtype=torch.float32)          # model.py:145
        if plan.logit_scale is not None or plan.logit_softcap is not None:
            K.scale_cap(logits, 1.0 if plan.logit_scale is None else plan.logit_scale,
                        plan.logit_softcap or 0.0)
        return logits


class _Arranged:
    """Gives a LayerSpec the ``kind`` its arrangement is registered under."""

    def __init__(self, layer):
        self._layer = layer
        self.kind = layer.arrangement

    def __getattr__(self, name):
        return getattr(self._layer, name)
