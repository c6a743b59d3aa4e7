"""The description of one step's batch, as the kernels read it.

A step brings, for each of its sequences, a run of new tokens; tokens of all sequences
are packed back to back.  Everything the kernels need to place a token (its sequence,
its position, where that sequence's cache pages are) is laid out in one int32 buffer
that goes to the device in a single copy:

    tokens[N] tok_seq[N] tok_pos[N] q_start[B+1] start_pos[B] slots[B] row_keys[B]
    want_rows[W] want_pos[W] seed[2] <fields that parts ask for> table_g[B, P_g] for every
    paged cache group g

``tok_seq[n]`` is the index of token n's sequence in this batch, ``tok_pos[n]`` its
position in that sequence (tokens cached before the step + offset in the run);
``table_g[b, i]`` is the cache page that holds positions ``64 i .. 64 i + 63`` of
sequence b in group g; ``want_rows`` are the indices of the tokens whose logits are wanted and
``want_pos`` their positions; ``slots[b]`` is the sequence's slot, which indexes the fixed-size
state of mixers that keep some; ``seed`` holds the two words of the sampler's seed for
steps whose sampling is recorded and replayed.  A part that needs something else of the step
on the device (cumulative lengths, a ring index, ...) declares a :class:`StepField`; the
model collects them and every step fills and uploads them with the rest.

The reference's step takes ``idx[B, S]`` and one shared ``input_pos[S]`` (model.py:136)
and a dense ``[Smax, Smax]`` mask (model.py:134); here lengths differ per sequence and
the mask is implied by ``tok_pos``.
"""
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache.store import Cache, pages_for


@dataclass
class Entry:
    """One sequence's share of a step: its slot, its new tokens, and the indices among
    these tokens whose logits are wanted.  ``slot`` None marks a row that belongs to no
    sequence and only keeps a recorded batch's shape: it reads and writes the cache's
    spare page and spare state slot and its results are ignored.  Only a decode session
    makes such rows; :meth:`Engine.step` refuses them."""
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()
    key: int = 0             # identifies the request to the sampler's noise


@dataclass(frozen=True)
class StepField:
    """A further int32 field of the step's description, asked for by a part (its
    ``step_fields()``): ``count(n_tokens, n_seqs)`` numbers, written on the host by
    ``fill(view, entries, starts, cache)`` (``starts[b]`` = tokens cached before the step;
    an entry whose ``slot`` is None is a filler row).  The part reads it as
    ``batch.<name>`` (device) or ``batch.host_field(name)``."""
    name: str
    count: Callable[[int, int], int]
    fill: Callable


def _round_up(n: int, k: int) -> int:
    return (n + k - 1) // k * k


class BatchLayout:
    """Offsets of the fields in the int32 buffer for given counts."""

    def __init__(self, n_tokens: int, n_seqs: int, n_want: int, table_widths: Dict[int, int],
                 extra: Sequence[StepField] = ()):
        self.n_tokens, self.n_seqs, self.n_want = n_tokens, n_seqs, n_want
        self.table_widths = dict(table_widths)
        self.extra = tuple(extra)
        off = 0
        self.fields = {}
        own = [("tokens", n_tokens), ("tok_seq", n_tokens), ("tok_pos", n_tokens),
               ("q_start", n_seqs + 1), ("start_pos", n_seqs), ("slots", n_seqs),
               ("row_keys", n_seqs), ("want_rows", n_want), ("want_pos", n_want), ("seed", 2)]
        for f in self.extra:
            if f.name in dict(own) or f.name in ("buffer", "host", "layout", "table"):
                raise ValueError(f"a part's step field cannot be named '{f.name}'")
            own.append((f.name, int(f.count(n_tokens, n_seqs))))
        for name, count in own:
            if name in self.fields:
                raise ValueError(f"two parts ask for a step field named '{name}'")
            self.fields[name] = (off, count)
            off = _round_up(off + count, 4)          # 16-byte aligned fields
        self.tables = {}
        for gid, width in self.table_widths.items():
            self.tables[gid] = (off, n_seqs * width)
            off = _round_up(off + n_seqs * width, 4)
        self.size = max(off, 4)

    def key(self):
        return (self.n_tokens, self.n_seqs, self.n_want, tuple(sorted(self.table_widths.items())),
                tuple(f.name for f in self.extra))


class StepBatch:
    """Device views of one step's description plus the host copies decisions need."""

    def __init__(self, layout: BatchLayout, device_buffer: torch.Tensor, host: np.ndarray):
        self.layout = layout
        self.buffer = device_buffer
        self.host = host
        self.n_tokens, self.n_seqs, self.n_want = layout.n_tokens, layout.n_seqs, layout.n_want
        for name, (off, count) in layout.fields.items():
            setattr(self, name, device_buffer[off:off + count])
        self._tables = {gid: device_buffer[off:off + count].view(self.n_seqs, layout.table_widths[gid])
                        for gid, (off, count) in layout.tables.items()}
        q_off, _ = layout.fields["q_start"]
        s_off, _ = layout.fields["start_pos"]
        q_start = host[q_off:q_off + self.n_seqs + 1]
        start = host[s_off:s_off + self.n_seqs]
        q_lens = q_start[1:] - q_start[:-1]
        self.max_q_len = int(q_lens.max()) if self.n_seqs else 0
        self.max_kv_len = int((start + q_lens).max()) if self.n_seqs else 0
        self.is_decode = self.max_q_len == 1
        w_off, _ = layout.fields["want_rows"]
        # every row's logits are wanted, in order: the final norm needs no gather
        self.every_row_wanted = self.n_want == self.n_tokens and bool(
            (host[w_off:w_off + self.n_want] == np.arange(self.n_want)).all())

    def table(self, group_id: int) -> torch.Tensor:
        return self._tables[group_id]

    def host_field(self, name: str) -> np.ndarray:
        off, count = self.layout.fields[name]
        return self.host[off:off + count]


def fill_host(layout: BatchLayout, host: np.ndarray, entries: Sequence[Entry],
              starts: Sequence[int], cache: Optional[Cache], seed: int = 0) -> None:
    """Write the step's description into ``host`` (int32 of ``layout.size``)."""
    from ..sampling import seed_words
    f = layout.fields
    host[f["seed"][0]:f["seed"][0] + 2] = seed_words(seed)
    spare_slot = cache.spare_slot if cache is not None else -1
    n = 0
    w = 0
    for b, (e, start) in enumerate(zip(entries, starts)):
        q = len(e.tokens)
        t0 = f["tokens"][0] + n
        host[t0:t0 + q] = e.tokens
        s0 = f["tok_seq"][0] + n
        host[s0:s0 + q] = b
        p0 = f["tok_pos"][0] + n
        host[p0:p0 + q] = np.arange(start, start + q, dtype=np.int32)
        host[f["q_start"][0] + b] = n
        host[f["start_pos"][0] + b] = start
        host[f["slots"][0] + b] = spare_slot if e.slot is None else e.slot
        host[f["row_keys"][0] + b] = e.key
        for i in e.want:
            if not 0 <= i < q:
                raise ValueError(f"want index {i} is outside the {q} tokens of the entry")
            host[f["want_rows"][0] + w] = n + i
            host[f["want_pos"][0] + w] = start + i
            w += 1
        n += q
    host[f["q_start"][0] + len(entries)] = n
    for field in layout.extra:
        off, count = f[field.name]
        field.fill(host[off:off + count], entries, starts, cache)
    if cache is not None:
        for gid, (off, _) in layout.tables.items():
            width = layout.table_widths[gid]
            group = cache.groups[gid]
            for b, e in enumerate(entries):           # slot None: a row that only fills the shape
                group.fill_table_row(host[off + b * width: off + (b + 1) * width], e.slot)


class BatchUploader:
    """Builds StepBatches: a small ring of pinned host buffers, one copy per step."""

    RING = 4

    def __init__(self, device, extra: Sequence[StepField] = ()):
        self.device = torch.device(device)
        self.extra = tuple(extra)
        self._ring: List[Optional[tuple]] = [None] * self.RING
        self._next = 0

    def _staging(self, size: int):
        i = self._next
        self._next = (self._next + 1) % self.RING
        item = self._ring[i]
        if item is not None:
            item[1].synchronize()                 # the copy that last used this buffer
        if item is None or item[0].numel() < size:
            cap = max(1024, 1 << (size - 1).bit_length())
            pinned = torch.empty(cap, dtype=torch.int32, pin_memory=self.device.type == "cuda")
            event = torch.cuda.Event() if self.device.type == "cuda" else _NoEvent()
            item = (pinned, event)
            self._ring[i] = item
        return item

    def build(self, entries: Sequence[Entry], starts: Sequence[int], cache: Cache,
              table_multiple: int = 1) -> StepBatch:
        n_tokens = sum(len(e.tokens) for e in entries)
        n_want = sum(len(e.want) for e in entries)
        widths = {}
        for gid, group in cache.paged_groups:
            most = max(group.table_entries(e.slot) for e in entries)
            widths[gid] = _round_up(max(most, 1), table_multiple)
        layout = BatchLayout(n_tokens, len(entries), n_want, widths, self.extra)
        pinned, event = self._staging(layout.size)
        host = pinned.numpy()[:layout.size]
        fill_host(layout, host, entries, starts, cache)
        dev = torch.empty(layout.size, dtype=torch.int32, device=self.device)
        dev.copy_(pinned[:layout.size], non_blocking=True)
        event.record()
        return StepBatch(layout, dev, host.copy())


class _NoEvent:
    def record(self):
        pass

    def synchronize(self):
        pass
