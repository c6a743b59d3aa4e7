"""The engine: a model, its cache, and the one step function everything else calls.

``Engine.step(entries)`` runs exactly the tokens it is given, as one batch, from the
cache that earlier steps left, and returns float32 logits at the wanted places.  Prompts
of unequal length go in one step; later steps bring one token per live sequence (or any
run of tokens: a step at a non-zero position is what the reference does when it verifies
a draft, generate.py:104-108).  The reference's step is ``model(idx[B, S], input_pos[S])``
over a batch of equal rows (model.py:136-146, generate.py:59-68).
"""
from typing import List, Optional, Sequence

import torch

from ..cache.store import Cache
from ..config.registry import architecture, read_model_folder
from ..ops.kernels import PAGE
from ..parts.base import Runtime
from ..parts.model import DecoderModel
from ..weights.bindings import compute_dtype, load_parameters
from ..weights.random_init import random_parameters
from .batch import BatchUploader, Entry, StepBatch
from .decode import RecordedSteps


def _device(device):
    dev = torch.device(device)
    if dev.type != "cuda":
        raise RuntimeError("this engine runs on a GPU only (device 'cuda:N'); there is no CPU path")
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible to torch; this engine has no CPU path")
    return dev


class Engine:
    def __init__(self, model: DecoderModel, *, max_tokens: int, max_sequences: Optional[int] = None):
        self.model = model
        self.rt = model.rt
        pages = (max_tokens + PAGE - 1) // PAGE
        if max_sequences is None:
            max_sequences = pages                 # a live sequence holds at least one page
        self.cache = Cache(model.cache_needs(), model.cache_borrow(), max_tokens=max_tokens,
                           max_sequences=max_sequences, dtype=self.rt.dtype, device=self.rt.device)
        self.step_fields = tuple(model.step_fields())  # further fields of a step's description
        self.uploader = BatchUploader(self.rt.device, self.step_fields)
        self.vocab_size = model.plan.vocab_size
        self.recorded_steps = RecordedSteps(self)      # HIP graphs of the one-token step

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_plan(cls, plan, parameters, dtype, device="cuda:0", **cache_args) -> "Engine":
        rt = Runtime(compute_dtype(dtype), _device(device))
        model = DecoderModel(plan, rt)
        model.bind(parameters)
        return cls(model, **cache_args)

    @classmethod
    def from_folder(cls, folder: str, dtype="bfloat16", device="cuda:0", **cache_args) -> "Engine":
        """Model class by ``config.json``; weights from the folder's safetensors files."""
        arch, config = read_model_folder(folder)
        dev = _device(device)
        params = load_parameters(folder, arch.layouts(config), dtype, dev)
        return cls.from_plan(arch.plan(config), params, dtype, dev, **cache_args)

    @classmethod
    def from_random(cls, arch_name: str, config, seed: int, dtype="bfloat16", device="cuda:0",
                    std=0.02, norm_std=0.1, **cache_args) -> "Engine":
        """Seeded random weights drawn on the device (no file)."""
        arch = architecture(arch_name)
        dev = _device(device)
        plan = arch.plan(config)
        params = random_parameters(arch.bindings(config), seed, dtype, dev, std=std,
                                   norm_std=norm_std, tie=plan.tie_embeddings)
        return cls.from_plan(plan, params, dtype, dev, **cache_args)

    # ------------------------------------------------------------------ sequences
    def start_sequence(self) -> int:
        return self.cache.acquire()

    def end_sequence(self, slot: int) -> None:
        self.cache.release(slot)

    # ------------------------------------------------------------------ the step
    def prepare(self, entries: Sequence[Entry]) -> StepBatch:
        """Check the entries, reserve cache room, and put the step's description on the
        device."""
        if not entries:
            raise ValueError("a step needs at least one sequence")
        V = self.vocab_size
        for e in entries:
            if e.slot is None:
                raise ValueError("an entry without a slot is a filler row of a decode session; "
                                 "a step takes sequences that hold a slot")
            if len(e.tokens) == 0:
                raise ValueError(f"slot {e.slot}: a step brings at least one token per sequence")
            lo, hi = min(e.tokens), max(e.tokens)
            if lo < 0 or hi >= V:
                raise ValueError(f"slot {e.slot}: token ids must lie in [0, {V}), got {lo}..{hi}")
        starts = self.cache.extend_many([(e.slot, len(e.tokens)) for e in entries])
        return self.uploader.build(entries, starts, self.cache)

    @torch.no_grad()
    def step(self, entries: Sequence[Entry]) -> torch.Tensor:
        """float32 logits [sum of len(want), vocab], in the order of entries and want."""
        batch = self.prepare(entries)
        return self.model.forward(batch, self.cache)
