"""One-token steps without a trip to the host: the hot loop of generation.

A :class:`DecodeSession` holds the live sequences of a batch after their prefill.  Every
:meth:`advance` runs one step of the engine for all of them: the tokens drawn by the
previous step are already on the device and feed the embedding directly, positions
advance by one, and the sampler writes the next tokens back into the same buffer
(the reference keeps its position tensor on the device and samples without a
synchronisation for the same reason, generate.py:40-42, 70-83).  The host only appends a
page to a sequence's table every 64 tokens.

With ``use_graph`` the step's kernels are captured once per batch shape into a HIP graph
and replayed; the step's description lives in a buffer at a fixed address that the host
refreshes before each replay.
"""
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..sampling import SamplingParams, sample
from .batch import BatchLayout, Entry, StepBatch, fill_host


class DecodeSession:
    def __init__(self, engine, slots: Sequence[int], keys: Sequence[int],
                 last_tokens: torch.Tensor, params: SamplingParams, *, use_graph: bool = True,
                 max_new_tokens: Optional[int] = None):
        """``last_tokens``: int32 device tensor [B], the token each sequence feeds next."""
        self.engine = engine
        self.cache = engine.cache
        self.params = params
        self.slots = list(slots)
        self.keys = list(keys)
        self.use_graph = use_graph
        B = len(self.slots)
        if last_tokens.numel() != B or last_tokens.dtype != torch.int32:
            raise ValueError("last_tokens must be int32 [number of sequences]")
        dev = engine.rt.device
        # table width: room for the pages the sequences will hold at the end of the run
        widths = {}
        for gid, _ in self.cache.kv_groups:
            most = 0
            for s in self.slots:
                final = self.cache.length(s) + (max_new_tokens or 0) + 1
                most = max(most, (final + 63) // 64, len(self.cache.page_list(gid, s)) + 1)
            widths[gid] = most
        self.layout = BatchLayout(B, B, B, widths)
        self.host = torch.empty(self.layout.size, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.staged = [torch.empty(self.layout.size, dtype=torch.int32, pin_memory=True)
                       for _ in range(4)]
        self.staged_events = [None] * 4
        self.turn = 0
        self.device_buffer = torch.zeros(self.layout.size, dtype=torch.int32, device=dev)
        self.batch = None
        self.tokens = torch.empty(B, dtype=torch.int32, device=dev)      # fed next
        self.tokens.copy_(last_tokens)
        self.graph = None
        self.logits = None
        self.steps = 0

    # ------------------------------------------------------------------
    def _refresh(self) -> None:
        """Reserve room for one more token per sequence and put the step's description
        (positions, page tables) into the device buffer; the token field is left alone."""
        starts = self.cache.extend_many([(s, 1) for s in self.slots])
        entries = [Entry(s, [0], want=[0], key=k) for s, k in zip(self.slots, self.keys)]
        for gid, _ in self.cache.kv_groups:
            for s in self.slots:
                if len(self.cache.page_list(gid, s)) > self.layout.table_widths[gid]:
                    raise RuntimeError("the decode session was sized for fewer tokens")
        i = self.turn % len(self.staged)
        self.turn += 1
        if self.staged_events[i] is not None:
            self.staged_events[i].synchronize()
        stage = self.staged[i]
        host = stage.numpy()
        fill_host(self.layout, host, entries, starts, self.cache)
        tok_off, tok_n = self.layout.fields["tokens"]
        # everything but the tokens (first field) is copied
        self.device_buffer[tok_off + tok_n:].copy_(stage[tok_off + tok_n:], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.staged_events[i] = ev
        if self.batch is None:
            self.batch = StepBatch(self.layout, self.device_buffer, host.copy())
            self.batch.tokens = self.tokens

    def _run(self) -> None:
        logits = self.engine.model.forward(self.batch, self.cache)
        sample(logits, self.params, self.batch.row_keys, self.batch.tok_pos, position_offset=1,
               out=self.tokens)
        self.logits = logits

    @torch.no_grad()
    def advance(self) -> torch.Tensor:
        """Run one step; returns the device buffer that now holds the new tokens (it is
        overwritten by the next step: copy what must be kept)."""
        self._refresh()
        if not self.use_graph:
            self._run()
        elif self.graph is None:
            # warm up once outside capture (library handles, first-use allocations)
            keep = self.tokens.clone()
            self._run()
            torch.cuda.synchronize()
            self.tokens.copy_(keep)
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self._run()
            self.graph.replay()
        else:
            self.graph.replay()
        self.steps += 1
        return self.tokens

    def drop(self, rows: Sequence[int]) -> None:
        """Take the sequences at these batch rows out of the session (they ended).  The
        session's shape changes, so it is rebuilt on the next step."""
        raise NotImplementedError("build a new session for the remaining sequences")
