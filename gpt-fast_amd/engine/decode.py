"""One-token steps without a trip to the host: the hot loop of generation.

A :class:`DecodeSession` holds the sequences of a batch after their prefill.  Every
:meth:`launch` runs one step of the engine for all of them: the tokens drawn by the
previous step are already on the device and feed the embedding directly, positions
advance by one, and the sampler writes the next tokens back into the same buffer (the
reference keeps its position tensor on the device and samples without a synchronisation
for the same reason, generate.py:40-42, 70-83).  The host only refreshes the step's
description (positions, page tables, seed) and, one step late, reads the drawn tokens.

The step's kernels are recorded once into a HIP graph and replayed; the description
lives in a buffer at a fixed address.  The recording belongs to the engine, not to the
session: a :class:`RecordedStep` is kept per shape (rows, page-table widths, sampling
law) and the next session of that shape replays it, as the reference compiles its decode
step once and reuses it for every sample (generate.py:338-345, 352-354).  A session has a
fixed number of rows; a row whose sequence has ended stays in the batch as a filler that
touches only the cache's spare page and spare state slot and whose token is ignored, so
the graph keeps its shape while the sequence's slot and pages are given back at once.

A step can only be recorded if every part issues the same kernels whatever the batch
holds; a part says so with ``replayable = True``.  A model with a part that does not
(one that loops over the batch on the host, say) is stepped without a recording.
"""
from collections import OrderedDict
from typing import List, Optional, Sequence

import torch

from ..sampling import SamplingParams, sample
from ..cache.store import pages_for
from .batch import BatchLayout, Entry, StepBatch, fill_host


class RecordedStep:
    """Buffers of the one-token step for one shape, and its HIP graph once recorded."""

    RING = 4

    def __init__(self, engine, n_rows: int, widths, params: SamplingParams):
        dev = engine.rt.device
        self.key = step_key(n_rows, widths, params)
        self.params = params
        self.layout = BatchLayout(n_rows, n_rows, n_rows, widths, engine.step_fields)
        self.staged = [torch.empty(self.layout.size, dtype=torch.int32, pin_memory=True)
                       for _ in range(self.RING)]
        self.staged_events = [None] * self.RING
        self.host_tokens = [torch.empty(n_rows, dtype=torch.int32, pin_memory=True)
                            for _ in range(self.RING)]
        self.turn = 0
        self.device_buffer = torch.zeros(self.layout.size, dtype=torch.int32, device=dev)
        self.tokens = torch.zeros(n_rows, dtype=torch.int32, device=dev)      # fed next
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.busy = False


def table_width(pages: int, most: int) -> int:
    """Entries per row of a session's page table for sequences that grow to ``pages`` pages:
    the next power of two (at most ``most``, the pool's pages, and never below ``pages``), so
    that sessions of similar lengths share one recording instead of recording one for every
    64 tokens of difference."""
    width = 1 << max(pages - 1, 0).bit_length()
    return max(pages, min(width, most))


def step_key(n_rows: int, widths, params: SamplingParams):
    """What a recording depends on; the seed is read from the step's buffer, not recorded."""
    return (n_rows, tuple(sorted(widths.items())), float(params.temperature), params.top_k)


class RecordedSteps:
    """The engine's recordings, most recently used last; the oldest idle one goes when
    there are more than ``limit`` (each holds the memory of its step's intermediates)."""

    def __init__(self, engine, limit: int = 8):
        self.engine = engine
        self.limit = limit
        self._steps: "OrderedDict[tuple, RecordedStep]" = OrderedDict()

    def take(self, n_rows: int, widths, params: SamplingParams) -> RecordedStep:
        key = step_key(n_rows, widths, params)
        step = self._steps.get(key)
        if step is not None and not step.busy:
            self._steps.move_to_end(key)
        else:
            # none of this shape, or it is in use by another open session
            step = RecordedStep(self.engine, n_rows, widths, params)
            if key not in self._steps:
                self._steps[key] = step
                for old in [k for k, s in self._steps.items() if not s.busy and k != key]:
                    if len(self._steps) <= self.limit:
                        break
                    del self._steps[old]
        step.busy = True
        return step

    def give_back(self, step: RecordedStep) -> None:
        step.busy = False

    def __len__(self):
        return len(self._steps)

    def clear(self) -> None:
        self._steps.clear()


class DecodeSession:
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
        self.use_graph = bool(use_graph) and engine.model.replayable
        B = len(self.slots)
        if B == 0:
            raise ValueError("a decode session needs at least one sequence")
        if any(s is None for s in self.slots):
            raise ValueError("a decode session starts with live sequences only")
        if last_tokens.numel() != B or last_tokens.dtype != torch.int32:
            raise ValueError("last_tokens must be int32 [number of sequences]")
        lo, hi = int(last_tokens.min()), int(last_tokens.max())
        if lo < 0 or hi >= engine.vocab_size:
            raise ValueError(f"token ids must lie in [0, {engine.vocab_size}), got {lo}..{hi}")
        widths = {}
        for gid, group in self.cache.paged_groups:
            most = 1
            for s in self.slots:
                final = self.cache.length(s) + (max_new_tokens or 0) + 1
                most = max(most, pages_for(final), group.table_entries(s) + 1)
            widths[gid] = table_width(most, self.cache.n_pages)
        self.rec = engine.recorded_steps.take(B, widths, params)
        self.layout = self.rec.layout
        self.tokens = self.rec.tokens
        self.tokens.copy_(last_tokens)
        self.batch: Optional[StepBatch] = None
        self.steps = 0
        self.closed = False

    @property
    def n_rows(self) -> int:
        return len(self.slots)

    def retire(self, row: int) -> None:
        """The sequence of this row has ended; the row stays as a filler."""
        self.slots[row] = None

    def close(self) -> None:
        """The session is over; its recording may serve the next session of this shape."""
        if not self.closed:
            self.closed = True
            self.engine.recorded_steps.give_back(self.rec)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ------------------------------------------------------------------
    def _refresh(self) -> None:
        """Reserve room for one more token per live sequence and put the step's
        description (positions, page tables, seed) into the device buffer; the token field
        is left alone."""
        rec = self.rec
        live = [(s, 1) for s in self.slots if s is not None]
        starts_live = iter(self.cache.extend_many(live)) if live else iter(())
        starts = [next(starts_live) if s is not None else 0 for s in self.slots]
        entries = [Entry(s, [0], want=[0], key=k) for s, k in zip(self.slots, self.keys)]
        for gid, group in self.cache.paged_groups:
            for s in self.slots:
                if s is not None and group.table_entries(s) > self.layout.table_widths[gid]:
                    raise RuntimeError("the decode session was sized for fewer tokens")
        i = rec.turn % rec.RING
        if rec.staged_events[i] is not None:
            rec.staged_events[i].synchronize()
        stage = rec.staged[i]
        host = stage.numpy()
        fill_host(self.layout, host, entries, starts, self.cache, seed=self.params.seed)
        tok_off, tok_n = self.layout.fields["tokens"]
        # everything but the tokens (first field) is copied
        rec.device_buffer[tok_off + tok_n:].copy_(stage[tok_off + tok_n:], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        rec.staged_events[i] = ev
        # the host copies that parts may read (host_field) are those of this step
        self.batch = StepBatch(self.layout, rec.device_buffer, host.copy())
        self.batch.tokens = self.tokens

    def _run(self) -> None:
        logits = self.engine.model.forward(self.batch, self.cache)
        sample(logits, self.params, self.batch.row_keys, self.batch.tok_pos, position_offset=1,
               out=self.tokens, seed_words=self.batch.seed)

    def _record(self) -> None:
        """Run the step once outside the recording (first-use allocations, library
        set-up), undo what that run changed, then record.  Keys and values written twice
        for one position are the same bytes; fixed-size state is not, so it is put back,
        and so are the tokens the run drew."""
        keep_tokens = self.tokens.clone()
        put_back = self.cache.snapshots()
        self._run()
        torch.cuda.synchronize()
        self.tokens.copy_(keep_tokens)
        for restore in put_back:
            restore()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self._run()
        self.rec.graph = graph

    @torch.no_grad()
    def launch(self):
        """Start one step.  Returns a handle for :meth:`collect`; the device buffer
        ``self.tokens`` holds the new tokens once the step has run."""
        if self.closed:
            raise RuntimeError("the decode session is closed")
        rec = self.rec
        self._refresh()
        if not self.use_graph:
            self._run()
        else:
            if rec.graph is None:
                self._record()
            rec.graph.replay()
        i = rec.turn % rec.RING
        rec.turn += 1
        self.steps += 1
        out = rec.host_tokens[i]
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
