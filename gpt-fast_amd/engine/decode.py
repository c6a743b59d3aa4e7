"""One-token steps without a trip to the host: the hot loop of generation.

A :class:`DecodeSession` holds the sequences of a batch after their prefill.  Every
:meth:`launch` runs one step of the engine for all of them: the tokens drawn by the
previous step are already on the device and feed the embedding directly, positions
advance by one, and the sampler writes the next tokens back into the same buffer (the
reference keeps its position tensor on the device and samples without a synchronisation
for the same reason, generate.py:40-42, 70-83).  The host only refreshes the step's
description (positions, page tables) and, one step late, reads the drawn tokens.

The step's kernels are captured once per session into a HIP graph and replayed; the
description lives in a buffer at a fixed address.  A session has a fixed number of
rows; a row whose sequence has ended stays in the batch as a filler that touches only
the cache's spare page and whose token is ignored, so the graph keeps its shape while
the sequence's slot and pages are given back at once.
"""
from typing import List, Optional, Sequence

import torch

from ..sampling import SamplingParams, sample
from .batch import BatchLayout, Entry, StepBatch, fill_host


class DecodeSession:
    RING = 4

    def __init__(self, engine, slots: Sequence[int], keys: Sequence[int],
                 last_tokens: torch.Tensor, params: SamplingParams, *, use_graph: bool = True,
                 max_new_tokens: Optional[int] = None):
        """``last_tokens``: int32 device tensor [B], the token each sequence feeds next.
        ``max_new_tokens`` bounds how far any sequence will grow during the session (it
        sizes the page tables)."""
        self.engine = engine
        self.cache = engine.cache
        self.params = params
        self.slots: List[Optional[int]] = list(slots)
        self.keys = list(keys)
        self.use_graph = use_graph
        B = len(self.slots)
        if last_tokens.numel() != B or last_tokens.dtype != torch.int32:
            raise ValueError("last_tokens must be int32 [number of sequences]")
        dev = engine.rt.device
        widths = {}
        for gid, _ in self.cache.kv_groups:
            most = 1
            for s in self.slots:
                final = self.cache.length(s) + (max_new_tokens or 0) + 1
                most = max(most, (final + 63) // 64, len(self.cache.page_list(gid, s)) + 1)
            widths[gid] = most
        self.layout = BatchLayout(B, B, B, widths)
        self.staged = [torch.empty(self.layout.size, dtype=torch.int32, pin_memory=True)
                       for _ in range(self.RING)]
        self.staged_events = [None] * self.RING
        self.turn = 0
        self.device_buffer = torch.zeros(self.layout.size, dtype=torch.int32, device=dev)
        self.batch = None
        self.tokens = torch.empty(B, dtype=torch.int32, device=dev)      # fed next
        self.tokens.copy_(last_tokens)
        self.host_tokens = [torch.empty(B, dtype=torch.int32, pin_memory=True)
                            for _ in range(self.RING)]
        self.graph = None
        self.steps = 0

    @property
    def n_rows(self) -> int:
        return len(self.slots)

    def retire(self, row: int) -> None:
        """The sequence of this row has ended; the row stays as a filler."""
        self.slots[row] = None

    # ------------------------------------------------------------------
    def _refresh(self) -> None:
        """Reserve room for one more token per live sequence and put the step's
        description (positions, page tables) into the device buffer; the token field is
        left alone."""
        live = [(s, 1) for s in self.slots if s is not None]
        starts_live = iter(self.cache.extend_many(live)) if live else iter(())
        starts = [next(starts_live) if s is not None else 0 for s in self.slots]
        entries = [Entry(s, [0], want=[0], key=k) for s, k in zip(self.slots, self.keys)]
        for gid, _ in self.cache.kv_groups:
            for s in self.slots:
                if s is not None and len(self.cache.page_list(gid, s)) > self.layout.table_widths[gid]:
                    raise RuntimeError("the decode session was sized for fewer tokens")
        i = self.turn % self.RING
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

    @torch.no_grad()
    def launch(self):
        """Start one step.  Returns a handle for :meth:`collect`; the device buffer
        ``self.tokens`` holds the new tokens once the step has run."""
        self._refresh()
        if not self.use_graph:
            self._run()
        elif self.graph is None:
            # once outside capture (first-use allocations), then capture and replay; the
            # step is a pure function of the cache and the tokens, so running it twice
            # for the same position changes nothing
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
        i = self.turn % self.RING
        self.turn += 1
        self.steps += 1
        out = self.host_tokens[i]
        out.copy_(self.tokens, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        return (out, ev)

    def collect(self, handle) -> List[int]:
        """The tokens a launched step drew, one per row (fillers' tokens are junk)."""
        out, ev = handle
        ev.synchronize()
        return out.tolist()

    def advance(self) -> torch.Tensor:
        """Launch one step and return the device buffer of its tokens (no read-back)."""
        self.launch()
        return self.tokens
